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
	/* the fixed partial-sum array of thhip_linear_batched_noalloc: look its address up now */
	if (thhip_linear_batched_noalloc_init())
		THError("thnets HIP engine: the fixed device array of thhip_linear_batched_noalloc could not be resolved");
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

/* cudnn_basic.c:64-80 is the CUDA analogue: same shape, contiguous device
 * copy in the engine's activation type. */
static THFloatTensor *device_tensor_like(THFloatTensor *t, int dtype)
{
	THFloatTensor *n = malloc(sizeof(*n));
	memcpy(n, t, sizeof(*n));
	n->storage = 0;
	n->storageOffset = 0;
	if (t->storage) {
		long stride = 1;
		for (int i = t->nDimension - 1; i >= 0; i--) {
			n->stride[i] = stride;
			stride *= t->size[i];
		}
		n->storage = malloc(sizeof(*n->storage));
		n->storage->nref = 1;
		n->storage->mustfree = TH_MUSTFREE_HIP_OF(dtype);
		n->storage->data = thhip_malloc((size_t)THFloatTensor_nElement(t) * (dtype == THHIP_F32 ? 4 : dtype == THHIP_U8 ? 1 : 2));
	}
	return n;
}

static void require_contiguous(THFloatTensor *t)
{
	long stride = 1;
	for (int i = t->nDimension - 1; i >= 0; i--) {
		if (t->size[i] != 1 && t->stride[i] != stride)
			THError("tensor is not contiguous");
		stride *= t->size[i];
	}
}

static THFloatTensor *upload_as(THFloatTensor *t, int dtype)
{
	THFloatTensor *n = device_tensor_like(t, dtype);
	if (!t->storage)
		return n;
	require_contiguous(t);
	const long cnt = THFloatTensor_nElement(t);
	if (dtype == THHIP_F32)
		thhip_memcpy_h2d(n->storage->data, THFloatTensor_data(t), sizeof(float) * cnt);
	else {
		float *tmp = thhip_malloc(sizeof(float) * cnt);
		thhip_memcpy_h2d(tmp, THFloatTensor_data(t), sizeof(float) * cnt);
		thhip_convert(tmp, THHIP_F32, n->storage->data, dtype, cnt);
		thhip_sync();
		thhip_free(tmp);
	}
	return n;
}

THFloatTensor *THHipTensor_newFromFloatTensor(THFloatTensor *t)
{
	return upload_as(t, thhip_engine_dtype());
}

static THFloatTensor *download_as_float(THFloatTensor *t, int dtype)
{
	THFloatTensor *n = malloc(sizeof(*n));
	memcpy(n, t, sizeof(*n));
	n->storage = 0;
	n->storageOffset = 0;
	if (!t->storage)
		return n;
	const long cnt = THFloatTensor_nElement(t);
	n->storage = THFloatStorage_new(cnt);
	const void *src = thhip_tensor_ptr(t, dtype);
	if (dtype == THHIP_F32)
		thhip_memcpy_d2h(n->storage->data, src, sizeof(float) * cnt);
	else {
		float *tmp = thhip_malloc(sizeof(float) * cnt);
		thhip_convert(src, dtype, tmp, THHIP_F32, cnt);
		thhip_memcpy_d2h(n->storage->data, tmp, sizeof(float) * cnt);
		thhip_free(tmp);
	}
	return n;
}

THFloatTensor *THFloatTensor_newFromHipTensor(THFloatTensor *t)
{
	return download_as_float(t, thhip_engine_dtype());
}

THFloatTensor *THForward(THNETWORK *net, THFloatTensor *in)
{
	engine_of(net);
	return thhip_forward(net->net, in);
}

static int finish(THNETWORK *network, THFloatTensor *out, float **result, int *outwidth, int *outheight)
{
	*result = out->storage->data;
	if (out->nDimension >= 3) {
		*outwidth = (int)out->size[out->nDimension - 1];
		*outheight = (int)out->size[out->nDimension - 2];
	} else
		*outwidth = *outheight = 1;
	(void)network;
	return (int)THFloatTensor_nElement(out);
}

/* uint8 engine: runs a device tensor of codes whose quantisation is in
 * hn->cur_mult / cur_sub, de-quantises the result (lowp_basic.c:40-58) and
 * leaves it in network->out. */
static THFloatTensor *run_codes(THNETWORK *network, THFloatTensor *q)
{
	struct hipnet *hn = (struct hipnet *)network->net;
	THFloatTensor *out = thhip_forward(network->net, q);
	THFloatTensor *f = device_tensor_like(out, THHIP_F32);
	thhip_dequantize(thhip_tensor_ptr(out, THHIP_U8), f->storage->data, THFloatTensor_nElement(out),
		hn->cur_mult, hn->cur_sub);
	if (network->out)
		THFloatTensor_free(network->out);
	network->out = download_as_float(f, THHIP_F32);
	THFloatTensor_free(f);
	return network->out;
}

/* Runs a device tensor of floats (engine dtype for ENGINE_HIP, fp32 for the
 * uint8 engine, which quantises it first) and leaves the float result in
 * network->out. */
/* The caller's buffer as THProcessFloat leaves it: planes 0..2 normalised in
 * place (thapi.c:389-403).  mean/std hold three planes: further planes are left
 * untouched here (the reference reads past the arrays for them). */
struct host_input {
	float *data;
	int batchsize, nplanes;
	long hw;
	const float *mean, *std;
};

static void normalize_on_host(const struct host_input *h)
{
	for (int b = 0; b < h->batchsize; b++)
		for (int c = 0; c < h->nplanes && c < 3; c++) {
			float *p = h->data + ((long)b * h->nplanes + c) * h->hw;
			const float mean = h->mean[c], std = h->std[c];
			for (long i = 0; i < h->hw; i++)
				p[i] = (p[i] - mean) / std;
		}
}

/* Runs a device tensor in the engine's float dtype (fp32 for the
 * uint8 engine, which quantises it first) and leaves the float result in
 * network->out.  The kernels of the forward pass are queued without waiting;
 * `host` (if any) is normalised while they run. */
static THFloatTensor *run_float_input(THNETWORK *network, THFloatTensor *dev_in, const struct host_input *host)
{
	struct hipnet *hn = (struct hipnet *)network->net;
	if (network->net->engine == ENGINE_HIPLOWP) {
		/* THLowpTensor_newFromFloatTensor on the whole batch (one min/max),
		 * lowp_basic.c:15-35 */
		const long cnt = THFloatTensor_nElement(dev_in);
		THFloatTensor *q = device_tensor_like(dev_in, THHIP_U8);
		thhip_quantize((const float *)thhip_tensor_ptr(dev_in, THHIP_F32), (unsigned char *)q->storage->data, cnt,
			&hn->cur_mult, &hn->cur_sub);
		THFloatTensor *out = thhip_forward(network->net, q);
		THFloatTensor *f = device_tensor_like(out, THHIP_F32);
		thhip_dequantize(thhip_tensor_ptr(out, THHIP_U8), f->storage->data, THFloatTensor_nElement(out),
			hn->cur_mult, hn->cur_sub);
		if (host)
			normalize_on_host(host);
		if (network->out)
			THFloatTensor_free(network->out);
		network->out = download_as_float(f, THHIP_F32);
		THFloatTensor_free(f);
		THFloatTensor_free(q);
	} else {
		THFloatTensor *out = thhip_forward(network->net, dev_in);
		if (host)
			normalize_on_host(host);
		if (network->out)
			THFloatTensor_free(network->out);
		network->out = download_as_float(out, hn->dtype);
	}
	return network->out;
}

int THProcessFloat(THNETWORK *network, float *data, int batchsize, int width, int height, int nplanes,
	float **result, int *outwidth, int *outheight)
{
	const int engine = engine_of(network);
	struct hipnet *hn = (struct hipnet *)network->net;
	const long hw = (long)width * height;
	/* The reference normalises the caller's buffer in place before any engine
	 * sees it (thapi.c:389-403), and callers observe that.  Here the raw data
	 * goes to the device first (the copy has finished when the call returns),
	 * a kernel applies the same arithmetic there, and the host loop over the
	 * caller's buffer runs while the GPU works on the forward pass: same bits
	 * on both sides, the host pass off the critical path. */
	THFloatTensor t;
	memset(&t, 0, sizeof(t));
	THFloatStorage st = { data, 1, 0 };
	t.nDimension = 4;
	t.size[0] = batchsize; t.size[1] = nplanes; t.size[2] = height; t.size[3] = width;
	t.stride[3] = 1; t.stride[2] = width; t.stride[1] = hw; t.stride[0] = hw * nplanes;
	t.storage = &st;
	const int dt = engine == ENGINE_HIPLOWP ? THHIP_F32 : hn->dtype;
	THFloatTensor *raw = upload_as(&t, THHIP_F32);
	THFloatTensor *dev = dt == THHIP_F32 ? raw : device_tensor_like(&t, dt);
	thhip_normalize(raw->storage->data, dev->storage->data, batchsize, nplanes, hw, network->mean, network->std, dt);
	const struct host_input host = { data, batchsize, nplanes, hw, network->mean, network->std };
	THFloatTensor *out = run_float_input(network, dev, &host);
	if (dev != raw)
		THFloatTensor_free(raw);
	THFloatTensor_free(dev);
	return finish(network, out, result, outwidth, outheight);
}

int THProcessImages(THNETWORK *network, unsigned char **images, int batchsize, int width, int height, int stride,
	float **results, int *outwidth, int *outheight, int bgr)
{
	const int engine = engine_of(network);
	struct hipnet *hn = (struct hipnet *)network->net;
	int cp = 3;
	if (stride < width * 3)
		cp = 1;	/* thapi.c:458-459 */
	if (engine == ENGINE_HIPLOWP) {
		/* thapi.c:485-487, 551-558: Lowp_LoadImages (always three planes, always
		 * 4-D), forward, de-quantise.  It reads three bytes per pixel whatever the
		 * stride: with stride < 3 * width (what the float engines take as one
		 * plane, thapi.c:458-459) the reference reads past the image; here that
		 * would be a device read past the staging copy, so it is refused. */
		if (cp != 3)
			THError("THProcessImages: the uint8 engine takes three-plane images only (stride %d < 3 * width %d)",
				stride, width);
		THFloatTensor *q = THFloatTensor_new();
		q->storage = malloc(sizeof(*q->storage));
		q->storage->nref = 1;
		q->storage->mustfree = TH_MUSTFREE_HIP_OF(THHIP_U8);
		q->storage->data = thhip_malloc((size_t)batchsize * 3 * width * height);
		unsigned char *staging = thhip_malloc((size_t)stride * height);
		for (int i = 0; i < batchsize; i++) {
			thhip_memcpy_h2d(staging, images[i], (size_t)stride * height);
			thhip_rgb2code((unsigned char *)q->storage->data + (size_t)i * 3 * width * height, staging, width, height,
				stride, network->mean, network->std, bgr, &hn->cur_mult, &hn->cur_sub);
		}
		thhip_sync();
		thhip_free(staging);
		long s4[4] = { batchsize, 3, height, width };
		q->nDimension = 4;
		long st = 1;
		for (int i = 3; i >= 0; st *= s4[i], i--) {
			q->size[i] = s4[i];
			q->stride[i] = st;
		}
		THFloatTensor *out = run_codes(network, q);
		THFloatTensor_free(q);
		return finish(network, out, results, outwidth, outheight);
	}
	const int dt = hn->dtype;
	const size_t esz = dt == THHIP_F32 ? 4 : 2;
	THFloatTensor *t = THFloatTensor_new();
	t->storage = malloc(sizeof(*t->storage));
	t->storage->nref = 1;
	t->storage->mustfree = TH_MUSTFREE_HIP_OF(dt);
	t->storage->data = thhip_malloc((size_t)batchsize * cp * width * height * esz);
	unsigned char *staging = thhip_malloc((size_t)stride * height);
	for (int i = 0; i < batchsize; i++) {
		thhip_memcpy_h2d(staging, images[i], (size_t)stride * height);
		thhip_rgb2float((char *)t->storage->data + (size_t)i * cp * width * height * esz, staging, width, height,
			stride, cp, network->mean, network->std, bgr, dt);
	}
	thhip_sync();
	thhip_free(staging);
	if (batchsize == 1) {	/* thapi.c:497-516 */
		long s[3] = { cp, height, width };
		t->nDimension = 3;
		for (int i = 2, st = 1; i >= 0; st *= s[i], i--) {
			t->size[i] = s[i];
			t->stride[i] = st;
		}
	} else {
		long s[4] = { batchsize, cp, height, width };
		t->nDimension = 4;
		long st = 1;
		for (int i = 3; i >= 0; st *= s[i], i--) {
			t->size[i] = s[i];
			t->stride[i] = st;
		}
	}
	THFloatTensor *out = run_float_input(network, t, 0);
	THFloatTensor_free(t);
	return finish(network, out, results, outwidth, outheight);
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
	thhip_sync();
	THFloatTensor *h;
	const int nd = o->nDimension;
	if (hn->hm[idx].out_cl && nd >= 3 && o->size[nd - 1] * o->size[nd - 2] > 1) {
		/* kept channels-last inside the engine: hand out the reference's order */
		THFloatTensor *pm = device_tensor_like(o, hn->dtype);
		thhip_relayout(thhip_tensor_ptr(o, hn->dtype), pm->storage->data, nd == 4 ? (int)o->size[0] : 1,
			(int)o->size[nd - 3], (int)(o->size[nd - 1] * o->size[nd - 2]), 0, hn->dtype);
		h = download_as_float(pm, hn->dtype);
		THFloatTensor_free(pm);
	} else
		h = download_as_float(o, hn->dtype);
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
	THFloatTensor *f = upload_as(t, THHIP_F32);
	THFloatTensor *q = device_tensor_like(f, THHIP_U8);
	thhip_quantize((const float *)f->storage->data, (unsigned char *)q->storage->data, THFloatTensor_nElement(f),
		&hn->cur_mult, &hn->cur_sub);
	thhip_sync();
	THFloatTensor_free(f);
	return q;
}
