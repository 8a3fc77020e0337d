/*
 * The thnets high level calls for networks that live on the MI355X engine:
 * THCreateHipNetwork / THCreateHipLowpNetwork beside the reference's
 * THCreateCudaNetwork / THCreateLowpNetwork (thapi.c:730-742, 784-796), and the
 * ENGINE_HIP branches of THProcessFloat / THProcessImages (cf. the ENGINE_CUDA
 * and ENGINE_LOWP branches, thapi.c:405-439, 452-563).
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "th_engine.h"

static int lasterror;

/* thapi.c:637-640: the code of the last recoverable failure (loaders, and the
 * calls this engine does not implement) */
int THLastError(void)
{
	return lasterror ? lasterror : thhip_load_error();
}

void THInit(void)
{
	/* nothing to prepare on the host; fail here, not at the first kernel, when
	 * no GPU is visible */
	if (thhip_device_count() < 1)
		THError("thnets HIP engine: no AMD GPU visible; this library has no CPU fallback");
	/* whether the GPU hands the workgroups of a launch to the XCDs in order (the convolutions add the K
	 * parts of cut tiles inside the kernel only where it does), and the flag kernels raise: probed and
	 * allocated now, not in the first forward */
	thhip_xcd_map();
	thhip_fault_flag();
	/* the fixed partial-sum array of thhip_linear_batched_noalloc: look its address up now */
	if (thhip_linear_batched_noalloc_init())	/* only that entry point is affected: it then returns -3 */
		fprintf(stderr, "thnets HIP engine: the fixed device array of thhip_linear_batched_noalloc could not be "
			"resolved; that call is unavailable\n");
}

static THNETWORK *create_engine_network(THNETWORK *net, int lowp, float range)
{
	if (!net || !net->net)
		THError("THCreateHipNetwork: network without modules (only Torch-style module lists are supported)");
	THNETWORK *nn = malloc(sizeof(*nn));
	memcpy(nn, net, sizeof(*nn));
	nn->netobj = 0;
	nn->statobj = 0;
	nn->pynet = 0;
	nn->allpynodes = 0;
	nn->out = 0;
	nn->net = THHip_ToHip(net->net, lowp, range);
	return nn;
}

THNETWORK *THCreateHipNetwork(THNETWORK *net)
{
	return create_engine_network(net, 0, 0);
}

THNETWORK *THCreateHipLowpNetwork(THNETWORK *net, float range)
{
	return create_engine_network(net, 1, range);
}

static int engine_of(THNETWORK *network)
{
	if (!network || !network->net)
		THError("network without modules");
	int e = network->net->engine;
	if (e != ENGINE_HIP && e != ENGINE_HIPLOWP)
		THError("This library only runs networks made by THCreateHipNetwork / THCreateHipLowpNetwork "
			"(engine %d given); it carries no CPU path", e);
	return e;
}

void THFreeNetwork(THNETWORK *network)
{
	if (network && network->net && network->net->engine == ENGINE_CPU && network->netobj) {
		thhip_free_loaded_network(network);	/* made by THLoadNetwork */
		return;
	}
	engine_of(network);
	thhip_sync();
	thhip_free_network(network->net);
	if (network->out)
		THFloatTensor_free(network->out);
	free(network);
}

THFloatTensor *THForward(THNETWORK *net, THFloatTensor *in)
{
	engine_of(net);
	return thhip_forward(net->net, in);
}

static int finish(THFloatTensor *out, float **result, int *outwidth, int *outheight)
{
	*result = out->storage->data;
	if (out->nDimension >= 3) {
		*outwidth = (int)out->size[out->nDimension - 1];
		*outheight = (int)out->size[out->nDimension - 2];
	} else
		*outwidth = *outheight = 1;
	return (int)THFloatTensor_nElement(out);
}

/* thapi.c:363-450 with the engine's branch (th_io.c) as the only one. */
int THProcessFloat(THNETWORK *network, float *data, int batchsize, int width, int height, int nplanes,
	float **result, int *outwidth, int *outheight)
{
	engine_of(network);
	return finish(thhip_process_float(network, data, batchsize, width, height, nplanes), result, outwidth, outheight);
}

/* thapi.c:452-563 likewise. */
int THProcessImages(THNETWORK *network, unsigned char **images, int batchsize, int width, int height, int stride,
	float **results, int *outwidth, int *outheight, int bgr)
{
	engine_of(network);
	return finish(thhip_process_images(network, images, batchsize, width, height, stride, bgr), results, outwidth,
		outheight);
}

/* thapi.c:642-690: Views dropped, Linear -> size x size convolution on the host
 * description; the weight memory is reinterpreted, not moved. */
void THMakeSpatial(THNETWORK *network, int size)
{
	int nInputPlane = 3;
	struct network *net = network->net;
	if (net->engine != ENGINE_CPU)
		THError("THMakeSpatial works on the host network, before THCreateHipNetwork");
	for (int i = 0; i < net->nelem; i++) {
		struct module *m = &net->modules[i];
		if (m->type == MT_View || m->type == MT_Reshape) {
			if (network->netobj)		/* loaded network: the library owns the module */
				THFloatTensor_free(m->output);
			memmove(m, m + 1, sizeof(*m) * (net->nelem - i - 1));
			net->nelem--;
			i--;
		} else if (m->type == MT_Linear) {
			THFloatTensor *w = m->Linear.weight, *b = m->Linear.bias;
			struct SpatialConvolution *c = &m->SpatialConvolution;
			if (network->netobj)
				THFloatTensor_free(m->Linear.addBuffer);	/* thapi.c:656; its slot becomes finput */
			m->type = MT_SpatialConvolutionVirtMM;
			memset(c, 0, sizeof(*c));
			c->weight = w;
			c->bias = b;
			c->dW = c->dH = 1;
			c->kW = c->kH = size;
			c->nInputPlane = nInputPlane;
			nInputPlane = c->nOutputPlane = (int)w->size[0];
			size = (size + 2 * c->padW - c->kW) / c->dW + 1;
		} else if (m->type == MT_SpatialConvolution || m->type == MT_SpatialConvolutionMM ||
			m->type == MT_SpatialConvolutionVirtMM) {
			struct SpatialConvolution *c = &m->SpatialConvolution;
			size = (size + 2 * c->padW - c->kW) / c->dW + 1;
			nInputPlane = c->nOutputPlane;
		} else if (m->type == MT_SpatialMaxPooling) {
			struct SpatialMaxPooling *c = &m->SpatialMaxPooling;
			if (c->ceil_mode)
				size = (ceil((float)(size - c->kH + 2 * c->padH) / c->dH)) + 1;
			else
				size = (floor((float)(size - c->kH + 2 * c->padH) / c->dH)) + 1;
		}
	}
}

/* thapi.c:692-728.  The engine has a single convolution algorithm, so this
 * only keeps the type tag coherent; the direct (mm_type 0) path does not
 * exist here. */
int THUseSpatialConvolutionMM(THNETWORK *network, int mm_type)
{
	if (!network->net || mm_type == 0)
		return lasterror = ERR_NOTIMPLEMENTED;
	for (int i = 0; i < network->net->nelem; i++) {
		struct module *m = &network->net->modules[i];
		if (m->type == MT_SpatialConvolution || m->type == MT_SpatialConvolutionMM ||
			m->type == MT_SpatialConvolutionVirtMM)
			m->type = mm_type == 2 ? MT_SpatialConvolutionVirtMM : MT_SpatialConvolutionMM;
	}
	return 0;
}

long THHipNetwork_copyModuleOutput(THNETWORK *net, int idx, float **dst, long size[4], int *ndim)
{
	engine_of(net);
	struct hipnet *hn = (struct hipnet *)net->net;
	if (idx < 0 || idx >= net->net->nelem)
		THError("THHipNetwork_copyModuleOutput: module %d out of range", idx);
	THFloatTensor *o = net->net->modules[idx].output;
	if (net->net->modules[idx].type == MT_ConcatTable || !o || !o->storage)
		THError("THHipNetwork_copyModuleOutput: module %d has no tensor output", idx);
	thhip_materialize_output(net->net, idx);	/* (a module that left its work to its consumer) */
	thhip_sync();
	THFloatTensor *h;
	const int nd = o->nDimension;
	if (hn->hm[idx].out_cl && nd >= 3 && o->size[nd - 1] * o->size[nd - 2] > 1) {
		/* kept channels-last inside the engine: hand out the reference's order */
		THFloatTensor *pm = thhip_device_tensor_like(o, hn->dtype);
		thhip_relayout(thhip_tensor_ptr(o, hn->dtype), pm->storage->data, nd == 4 ? (int)o->size[0] : 1,
			(int)o->size[nd - 3], (int)(o->size[nd - 1] * o->size[nd - 2]), 0, hn->dtype);
		h = thhip_download_as_float(pm, hn->dtype);
		THFloatTensor_free(pm);
	} else
		h = thhip_download_as_float(o, hn->dtype);
	const long n = THFloatTensor_nElement(h);
	*ndim = h->nDimension;
	for (int i = 0; i < 4; i++)
		size[i] = i < h->nDimension ? h->size[i] : 1;
	*dst = h->storage->data;
	h->storage->mustfree = 0;	/* ownership moves to the caller */
	THFloatTensor_free(h);
	return n;
}

int THHipNetwork_getModuleQuant(THNETWORK *net, int idx, float *mult, float *sub)
{
	if (engine_of(net) != ENGINE_HIPLOWP || idx < 0 || idx >= net->net->nelem)
		return ERR_NOTIMPLEMENTED;
	struct hipnet *hn = (struct hipnet *)net->net;
	*mult = hn->hm[idx].q_mult;
	*sub = hn->hm[idx].q_sub;
	return 0;
}

int THHipNetwork_setInputQuant(THNETWORK *net, float mult, float sub)
{
	if (engine_of(net) != ENGINE_HIPLOWP)
		return ERR_NOTIMPLEMENTED;
	struct hipnet *hn = (struct hipnet *)net->net;
	hn->cur_mult = mult;
	hn->cur_sub = sub;
	return 0;
}

/* Device counterpart of THLowpTensor_newFromFloatTensor (lowp_basic.c:5-38):
 * uploads a host float tensor, quantises it on the device with one min/max
 * over the whole tensor and records (mult, sub) as the quantisation of the
 * network's next input. */
THFloatTensor *THHipLowpTensor_newFromFloatTensor(THNETWORK *net, THFloatTensor *t)
{
	if (engine_of(net) != ENGINE_HIPLOWP)
		THError("THHipLowpTensor_newFromFloatTensor needs a network made by THCreateHipLowpNetwork");
	struct hipnet *hn = (struct hipnet *)net->net;
	THFloatTensor *f = thhip_upload_as(t, THHIP_F32);
	THFloatTensor *q = thhip_device_tensor_like(f, THHIP_U8);
	thhip_quantize((const float *)f->storage->data, (unsigned char *)q->storage->data, THFloatTensor_nElement(f),
		&hn->cur_mult, &hn->cur_sub);
	thhip_sync();
	THFloatTensor_free(f);
	return q;
}
