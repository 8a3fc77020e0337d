/*
 * The MI355X engine: turns a host `struct network` into one whose modules
 * run on the GPU, the way THcudnn_ToCUDNN (cudnn/cudnn_basic.c:189-303) and
 * THLowp_ToLowp (lowp/lowp_basic.c:133-212) re-target a network, and provides
 * the updateOutput of every module type the convolution / Linear / LOWP path
 * traverses.  Host code only: every number is produced by a kernel behind the
 * thhip_* C ABI.
 *
 * Differences from the reference engines that a caller can observe:
 *   - activations stay on the device between modules and module outputs are
 *     kept (not freed per layer as thapi.c:205-209 does), so repeated forwards
 *     allocate nothing once shapes are known;
 *   - a Threshold that follows a convolution / Linear is folded into that
 *     module's epilogue and becomes a pass-through;
 *   - nested containers (Sequential, ConcatTable + CAddTable) are converted
 *     recursively; the reference's GPU engines refuse them;
 *   - the uint8 engine keeps each module's (mult, sub) with the module, works
 *     at any batch size and for any number of forwards.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include "th_engine.h"

static int g_halfmode;	/* 0 fp32, 1 fp16, 2 bf16: THHipHalfFloat */

int THHipHalfFloat(int enable)
{
	if (enable < 0 || enable > 2)
		return ERR_NOTIMPLEMENTED;
	g_halfmode = enable;
	return 0;
}

static int g_fold_bn = 1;

/* 1 (default): a SpatialBatchNormalization that directly follows a convolution
 * is folded into that convolution's epilogue when the engine is created;
 * 0: it runs as its own kernel, as in the reference's CPU path.  Returns the
 * previous setting. */
int THHipImageLayerInFront(int mode)
{
	extern int thhip_image_layer_in_front;
	const int old = thhip_image_layer_in_front;
	if (mode >= 0 && mode <= 2)
		thhip_image_layer_in_front = mode;
	return old;
}

int THHipFoldBatchNorm(int enable)
{
	const int old = g_fold_bn;
	g_fold_bn = enable != 0;
	return old;
}

static int g_table_math;

/* 0 (default): CAddTable / CSubTable compute what the reference's shipped modules compute
 * (two inputs: a - b for CAddTable and a + b for CSubTable; more: 2a + b + c + ..., 0 - b - c - ...
 * CAddTable.c:59-84).  1: what the modules' names say (the sum of all inputs; the first minus the
 * others), for networks trained against Torch's modules.  Read at engine creation; returns the
 * previous setting. */
int THHipTableArithmetic(int as_named)
{
	const int old = g_table_math;
	g_table_math = as_named != 0;
	return old;
}

int thhip_engine_dtype(void)
{
	return g_halfmode == 1 ? THHIP_F16 : g_halfmode == 2 ? THHIP_BF16 : THHIP_F32;
}

static int esize_of(int dtype)
{
	return dtype == THHIP_F32 ? 4 : dtype == THHIP_U8 ? 1 : 2;
}

struct hipnet *hipnet_of(struct module *m)
{
	return (struct hipnet *)m->net;
}

struct hipmod *hipmod_of(struct module *m)
{
	struct hipnet *hn = hipnet_of(m);
	return &hn->hm[m - hn->pub.modules];
}

static const char *thhip_dtype_name(int dtype)
{
	return dtype == THHIP_F32 ? "fp32" : dtype == THHIP_F16 ? "fp16" : dtype == THHIP_BF16 ? "bf16" : "uint8";
}

void *thhip_tensor_ptr(THFloatTensor *t, int dtype)
{
	if (!t || !t->storage || !t->storage->data)
		THError("HIP engine: tensor without storage");
	if (!TH_IS_HIP_STORAGE(t->storage->mustfree))
		THError("HIP engine: module input is not a device tensor (create it with THHipTensor_newFromFloatTensor)");
	if (TH_HIP_STORAGE_DTYPE(t->storage->mustfree) != dtype)
		THError("HIP engine: device tensor holds %s elements, %s expected (it was made under another THHipHalfFloat "
			"setting or for another network type)", thhip_dtype_name(TH_HIP_STORAGE_DTYPE(t->storage->mustfree)),
			thhip_dtype_name(dtype));
	return (char *)t->storage->data + t->storageOffset * esize_of(dtype);
}

/* Gives module m a contiguous device output of the given shape, reusing its
 * allocation whenever it is large enough. */
static void *out_resize(struct module *m, int dtype, int nd, const long *size)
{
	struct hipmod *hm = hipmod_of(m);
	THFloatTensor *o = m->output;
	long n = 1, stride = 1;
	for (int i = 0; i < nd; i++)
		n *= size[i];
	size_t bytes = (size_t)n * esize_of(dtype);
	/* uint8 tensors are followed by a few codes of 0.0 as a convolution output
	 * has it (range / 2 * 255 / range rounds to 128): the convolution kernel that
	 * loads straight into LDS fetches its padding from there */
	const size_t tail = dtype == THHIP_U8 ? TH_U8_TAIL : 0;
	if (!o->storage || !TH_IS_HIP_STORAGE(o->storage->mustfree) || hm->cap < bytes + tail || !hm->owns_output) {
		THFloatStorage *s = malloc(sizeof(*s));
		s->data = thhip_malloc(bytes + tail);
		s->nref = 1;
		s->mustfree = TH_MUSTFREE_HIP_OF(dtype);
		if (o->storage)
			thhip_storage_release(o->storage);
		o->storage = s;
		hm->cap = bytes + tail;
		hm->owns_output = 1;
		hm->tail_at = (size_t)-1;
	}
	if (tail && hm->tail_at != bytes) {
		thhip_memset((char *)o->storage->data + bytes, TH_U8_TAIL_CODE, tail);
		hm->tail_at = bytes;
	}
	o->storage->mustfree = TH_MUSTFREE_HIP_OF(dtype);
	o->storageOffset = 0;
	o->nDimension = nd;
	for (int i = nd - 1; i >= 0; i--) {
		o->size[i] = size[i];
		o->stride[i] = stride;
		stride *= size[i];
	}
	return o->storage->data;
}

/* Output becomes another view of the input (in-place modules, View, Dropout). */
static void out_alias(struct module *m, THFloatTensor *in)
{
	hipmod_of(m)->owns_output = 0;
	THFloatTensor_set(m->output, in);
}

/* ------------------------------------------------------------------ */
/* fp32 / fp16 / bf16 modules                                          */
/* ------------------------------------------------------------------ */

/* Whether the image layer of a half network is left to the convolution after it (Hip_SpatialConvolution_updateOutput):
 * 0 never, 2 always, 1 (default) for batches of up to 2048 of that convolution's 32 x 8 tiles -- measured on
 * VGG-16 fp16 at 224 x 224, one kernel against two: batch 1 -1.6 %, 2 -4 %, 4 -3.3 %, 8 -1 % of the forward,
 * batch 16 and 64 +0.8 % (there the patch computation of a tile costs more than the image layer's own kernel,
 * which runs at the rate its stores allow). */
int thhip_image_layer_in_front = 1;	/* (THHipImageLayerInFront) */

struct convshape { int B, H, W, outnd; };

/* Input shapes a convolution accepts: 3-D (one image) and 4-D as
 * SpatialConvolutionMM.c:146-152; vectors and matrices are taken as 1x1
 * images the way the GPU engines run Linear (cudnn_SpatialConvolution.c:41-47,
 * lowp_SpatialConvolution.c:138-147). */
static struct convshape conv_input_shape(struct module *m, THFloatTensor *in)
{
	struct convshape s;
	long planes;
	switch (in->nDimension) {
	case 1: s.B = 1; planes = in->size[0]; s.H = s.W = 1; break;
	case 2: s.B = (int)in->size[0]; planes = in->size[1]; s.H = s.W = 1; break;
	case 3: s.B = 1; planes = in->size[0]; s.H = (int)in->size[1]; s.W = (int)in->size[2]; break;
	case 4: s.B = (int)in->size[0]; planes = in->size[1]; s.H = (int)in->size[2]; s.W = (int)in->size[3]; break;
	default: THError("convolution input must have 1 to 4 dimensions"); planes = 0;
	}
	s.outnd = in->nDimension;
	if (planes != m->SpatialConvolution.nInputPlane)
		THError("nInputPlane %ld does not match input planes %ld", (long)m->SpatialConvolution.nInputPlane, planes);
	return s;
}

static void *conv_out(struct module *m, int dtype, const struct convshape *s, int Co, int oH, int oW)
{
	long sz[4];
	switch (s->outnd) {
	case 1: sz[0] = Co; return out_resize(m, dtype, 1, sz);
	case 2: sz[0] = s->B; sz[1] = Co; return out_resize(m, dtype, 2, sz);
	case 3: sz[0] = Co; sz[1] = oH; sz[2] = oW; return out_resize(m, dtype, 3, sz);
	default: sz[0] = s->B; sz[1] = Co; sz[2] = oH; sz[3] = oW; return out_resize(m, dtype, 4, sz);
	}
}

static THFloatTensor *Hip_SpatialConvolution_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct SpatialConvolution *c = &m->SpatialConvolution;
	const int dt = hn->dtype;
	struct convshape s = conv_input_shape(m, in);
	const int oW = (s.W + 2 * c->padW - c->kW) / c->dW + 1;
	const int oH = (s.H + 2 * c->padH - c->kH) / c->dH + 1;
	if (oW < 1 || oH < 1)
		THError("Given input size: (%dx%dx%d). Calculated output size: (%dx%dx%d). Output size is too small",
			c->nInputPlane, s.H, s.W, c->nOutputPlane, oH, oW);
	const void *x = thhip_tensor_ptr(in, dt);
	const int K = c->nInputPlane * c->kH * c->kW;
	/* the weights were packed for the planned memory order of the input; with
	 * one pixel per plane both orders coincide */
	if (s.H * s.W > 1 && hn->cur_cl != hm->in_cl)
		THError("HIP engine: a convolution planned for %s input got the other memory order",
			hm->in_cl ? "channels-last" : "plane-major");
	/* conv -> (Threshold) -> 2x2 max pooling in one kernel, where the kernel that
	 * would run this layer can do it */
	const struct SpatialMaxPooling *pq = hm->pool_next ? &hn->pub.modules[hm->pool_next].SpatialMaxPooling : 0;
	const int pool22 = pq && pq->kW == 2 && pq->kH == 2 && pq->dW == 2 && pq->dH == 2 && pq->padW == 0 && pq->padH == 0 && !pq->ceil_mode;
	/* the image layer of a half network: left to the convolution after it, which computes this layer's
	 * output patch by patch in LDS; nothing is written here (the output tensor keeps its shape and memory, and
	 * is filled on demand: thhip_materialize_output).  Not while th_minmax wants every tensor's range. */
	hm->deferred = 0;
	if (hm->front_of && !th_minmax && s.outnd == 4 &&
	    (thhip_image_layer_in_front == 2 ||
	     (thhip_image_layer_in_front == 1 && (long)s.B * ((oH + 7) / 8) * ((oW + 31) / 32) *
			((hn->pub.modules[hm->front_of].SpatialConvolution.nOutputPlane + 63) / 64) <= 2048)) &&
	    thhip_conv2d_image_pair_supported(s.B, s.H, s.W, c->nOutputPlane,
			hn->pub.modules[hm->front_of].SpatialConvolution.nOutputPlane, dt, 1)) {
		conv_out(m, dt, &s, c->nOutputPlane, oH, oW);
		hn->cur_cl = hm->out_cl;
		hm->deferred = 1;
		hm->front_img = x;
		hm->front_B = s.B; hm->front_H = s.H; hm->front_W = s.W;
		return m->output;
	}
	if (hm->front && hn->hm[hm->front - 1].deferred) {
		struct hipmod *fm = &hn->hm[hm->front - 1];
		const int pool = pool22 && oH >= 2 && oW >= 2;
		if (fm->front_B == s.B && fm->front_H == s.H && fm->front_W == s.W) {
			void *yp = conv_out(m, dt, &s, c->nOutputPlane, pool ? oH / 2 : oH, pool ? oW / 2 : oW);
			hn->cur_cl = hm->out_cl && (pool ? (oH / 2) * (oW / 2) : oH * oW) > 1;
			thhip_conv2d_image_pair(fm->front_img, fm->wfront, fm->scale, fm->bias, fm->fused_act, fm->thr, fm->val,
				hm->wpacked, hm->scale, hm->bias, yp, s.B, s.H, s.W, c->nOutputPlane, hm->fused_act, hm->thr, hm->val,
				pool, dt);
			if (pool)
				hn->hm[hm->pool_next].pooled_by_producer = 1;
			return m->output;
		}
		thhip_materialize_output(&hn->pub, hm->front - 1);	/* (another shape than the image layer saw: never in a list of modules) */
	}
	if (pool22 && thhip_conv2d_pool2_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW,
			c->dH, c->dW, c->padH, c->padW, dt, hm->x_layout, hm->out_cl)) {
		void *yp = conv_out(m, dt, &s, c->nOutputPlane, oH / 2, oW / 2);
		hn->cur_cl = hm->out_cl && (oH / 2) * (oW / 2) > 1;
		thhip_conv2d_layout_pool2(x, hm->wpacked, hm->scale, hm->bias, yp, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, hm->fused_act, hm->thr, hm->val, dt, hm->x_layout,
			hm->out_cl);
		hn->hm[hm->pool_next].pooled_by_producer = 1;
		return m->output;
	}
	/* an fp32 image layer followed by a 3x3 / stride 2 pooling (ResNet's stem): one kernel, no convolution output */
	if (pq && dt == THHIP_F32 && !hm->x_layout && !hm->out_cl && s.outnd >= 3 &&
	    thhip_conv2d_image_pool_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW,
			c->padH, c->padW, pq->kH, pq->kW, pq->dH, pq->dW, pq->padH, pq->padW, pq->ceil_mode, dt, hm->x_layout)) {
		int pH, pW;
		thhip_pool_outsize(oH, oW, pq->kH, pq->kW, pq->dH, pq->dW, pq->padH, pq->padW, pq->ceil_mode, &pH, &pW);
		void *yp = conv_out(m, dt, &s, c->nOutputPlane, pH, pW);
		hn->cur_cl = 0;
		thhip_conv2d_image_pool(x, hm->wpacked, hm->scale, hm->bias, yp, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, pq->padH, hm->fused_act, hm->thr, hm->val, dt);
		hn->hm[hm->pool_next].pooled_by_producer = 1;
		return m->output;
	}
	/* fp32, a layer of a few tiles (its K is split and a second kernel adds the parts): that kernel takes
	 * a max pooling of any window as well */
	if (pq && dt == THHIP_F32 && !hm->x_layout && !hm->out_cl && s.outnd >= 3 &&
	    thhip_conv2d_poolk_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW, c->padH, c->padW,
			pq->kH, pq->kW, pq->dH, pq->dW, pq->padH, pq->padW, pq->ceil_mode, dt)) {
		int pH, pW;
		thhip_pool_outsize(oH, oW, pq->kH, pq->kW, pq->dH, pq->dW, pq->padH, pq->padW, pq->ceil_mode, &pH, &pW);
		void *yp = conv_out(m, dt, &s, c->nOutputPlane, pH, pW);
		hn->cur_cl = 0;
		thhip_conv2d_poolk(x, hm->wpacked, hm->scale, hm->bias, yp, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, pq->kH, pq->kW, pq->dH, pq->dW, pq->padH, pq->padW, pq->ceil_mode,
			hm->fused_act, hm->thr, hm->val, dt);
		hn->hm[hm->pool_next].pooled_by_producer = 1;
		return m->output;
	}
	void *y = conv_out(m, dt, &s, c->nOutputPlane, oH, oW);
	hn->cur_cl = hm->out_cl && oH * oW > 1;
	/* the last convolution of a residual block: the table add and its Threshold in the epilogue */
	if (hm->res_mode && hm->res_ptr) {
		const void *res = hm->res_ptr;
		const long res_n = hm->res_n;
		hm->res_ptr = 0;
		if (res != y && res_n == (long)s.B * c->nOutputPlane * oH * oW && s.outnd >= 3 &&
		    thhip_conv2d_residual_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW,
				c->padH, c->padW, dt)) {
			thhip_conv2d_residual(x, hm->wpacked, hm->scale, hm->bias, res, hm->res_mode, hm->res_c, hm->res_act, y,
				s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW, c->padH, c->padW,
				hm->fused_act, hm->thr, hm->val, dt);
			hm->res_add->added_by_producer = hm->res_mode;	/* mode 1: branch 0 holds the sum, mode 2: branch 1 */
			return m->output;
		}
	}
	/* the row-major copy is made from plane-major packing; for a 1x1 kernel the
	 * channels-last packing is the same (k is the plane in both) */
	const int one_position = oH == 1 && oW == 1 && c->padH == 0 && c->padW == 0 && c->kH == s.H && c->kW == s.W &&
		(!hm->x_layout || (hm->x_layout == 1 && c->kH == 1 && c->kW == 1));
	if (one_position && !hm->scale && (s.B == 1 || thhip_linear_batched_supported(s.B, K, c->nOutputPlane, dt))) {
		/* one output position per image: a matrix-vector (or skinny matrix)
		 * product over the flattened input, bound by reading the weights once */
		if (!hm->wrow)
			hm->wrow = thhip_conv_unpack_rows(hm->wpacked, c->nOutputPlane, c->nInputPlane, c->kH * c->kW, dt);
		if (s.B == 1)
			thhip_gemv(x, hm->wrow, hm->bias, y, K, c->nOutputPlane, hm->fused_act, hm->thr, hm->val, dt);
		else
			thhip_linear_batched(x, hm->wrow, hm->bias, y, s.B, K, c->nOutputPlane, hm->fused_act, hm->thr,
				hm->val, dt);
	} else
		thhip_conv2d_layout(x, hm->wpacked, hm->scale, hm->bias, y, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, hm->fused_act, hm->thr, hm->val, dt, hm->x_layout,
			hm->out_cl);
	return m->output;
}

static THFloatTensor *Hip_Threshold_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct Threshold *t = &m->Threshold;
	const int dt = hn->dtype;
	if (hm->passthrough) {	/* already applied by the producer's epilogue */
		out_alias(m, in);
		return m->output;
	}
	const long n = THFloatTensor_nElement(in);
	void *x = thhip_tensor_ptr(in, dt);
	if (t->inplace == 1) {
		thhip_threshold(x, x, n, t->threshold, t->val, t->alpha, 1, dt);
		out_alias(m, in);
	} else {
		void *y = out_resize(m, dt, in->nDimension, in->size);
		thhip_threshold(x, y, n, t->threshold, t->val, t->alpha, 0, dt);
	}
	return m->output;
}

struct planes { int B, C, H, W, nd; };

static struct planes planes_of(THFloatTensor *in, const char *who)
{
	struct planes p;
	if (in->nDimension == 3) {
		p.B = 1; p.C = (int)in->size[0]; p.H = (int)in->size[1]; p.W = (int)in->size[2];
	} else if (in->nDimension == 4) {
		p.B = (int)in->size[0]; p.C = (int)in->size[1]; p.H = (int)in->size[2]; p.W = (int)in->size[3];
	} else
		THError("%s: 3D or 4D (batch mode) tensor expected", who);
	p.nd = in->nDimension;
	return p;
}

static void *planes_out(struct module *m, int dtype, const struct planes *p, int oH, int oW)
{
	long sz[4];
	if (p->nd == 3) {
		sz[0] = p->C; sz[1] = oH; sz[2] = oW;
		return out_resize(m, dtype, 3, sz);
	}
	sz[0] = p->B; sz[1] = p->C; sz[2] = oH; sz[3] = oW;
	return out_resize(m, dtype, 4, sz);
}

static THFloatTensor *Hip_SpatialMaxPooling_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct SpatialMaxPooling *q = &m->SpatialMaxPooling;
	if (hipmod_of(m)->pooled_by_producer) {	/* done in the convolution's epilogue */
		hipmod_of(m)->pooled_by_producer = 0;
		out_alias(m, in);
		return m->output;
	}
	struct planes p = planes_of(in, "SpatialMaxPooling");
	int oH, oW;
	q->iwidth = p.W;
	q->iheight = p.H;
	thhip_pool_outsize(p.H, p.W, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, q->ceil_mode, &oH, &oW);
	if (oH < 1 || oW < 1)
		THError("SpatialMaxPooling: input %dx%d smaller than the window", p.H, p.W);
	const void *x = thhip_tensor_ptr(in, hn->dtype);
	void *y = planes_out(m, hn->dtype, &p, oH, oW);
	struct hipmod *hm = hipmod_of(m);
	if (hm->want_indices) {
		/* a SpatialMaxUnpooling later in this network scatters by these
		 * (SpatialMaxPooling.c:213-217 keeps them in every forward) */
		const size_t need = sizeof(int) * (size_t)p.B * p.C * oH * oW;
		if (hn->cur_cl)
			THError("HIP engine: a pooling that keeps indices got channels-last input");
		if (hm->pool_ind_cap < need) {
			thhip_free(hm->pool_ind);
			hm->pool_ind = thhip_malloc(need);
			hm->pool_ind_cap = need;
		}
		thhip_maxpool_indices(x, y, hm->pool_ind, p.B, p.C, p.H, p.W, oH, oW, q->kH, q->kW, q->dH, q->dW, q->padH,
			q->padW, hn->dtype);
	} else if (hn->cur_cl)
		thhip_maxpool_cl(x, y, p.B, p.C, p.H, p.W, oH, oW, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, hn->dtype);
	else
		thhip_maxpool(x, y, p.B, p.C, p.H, p.W, oH, oW, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, hn->dtype);
	if (oH * oW == 1)
		hn->cur_cl = 0;		/* one pixel per plane: both orders coincide */
	return m->output;
}

/* SpatialMaxUnpooling.c:43-120: the output has the extent the paired pooling
 * saw at its last forward; its indices say where each value goes. */
static THFloatTensor *Hip_SpatialMaxUnpooling_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct module *pm = &hn->pub.modules[hm->pool_index];
	struct hipmod *ph = &hn->hm[hm->pool_index];
	const struct SpatialMaxPooling *q = &pm->SpatialMaxPooling;
	struct planes p = planes_of(in, "SpatialMaxUnpooling");
	THFloatTensor *po = pm->output;
	if (!ph->pool_ind || !po || po->nDimension != in->nDimension)
		THError("Invalid input size w.r.t current indices size");	/* :73-74 */
	for (int i = 0; i < in->nDimension; i++)
		if (po->size[i] != in->size[i])
			THError("Invalid input size w.r.t current indices size");
	if (hn->cur_cl)
		THError("HIP engine: SpatialMaxUnpooling got channels-last input");
	void *y = planes_out(m, hn->dtype, &p, q->iheight, q->iwidth);
	thhip_maxunpool(thhip_tensor_ptr(in, hn->dtype), ph->pool_ind, y, p.B, p.C, q->iheight, q->iwidth, p.H, p.W,
		q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, hn->dtype);
	return m->output;
}

/* SpatialFullConvolution.c:136-250.  With a bias the reference's bias GEMM
 * scales the transposed convolution by its beta argument, 11 (:231-237). */
#define FULLCONV_BIAS_BETA 11.0f

static THFloatTensor *Hip_SpatialFullConvolution_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	const struct SpatialFullConvolution *c = &m->SpatialFullConvolution;
	const int dt = hn->dtype;
	struct planes p = planes_of(in, "SpatialFullConvolution");
	if (p.C != c->nInputPlane)
		THError("input channels and nInputPlane dont match");	/* :160-166 */
	if (hn->cur_cl)
		THError("HIP engine: SpatialFullConvolution got channels-last input");
	const int oW = (p.W - 1) * c->dW - 2 * c->padW + c->kW + c->adjW;
	const int oH = (p.H - 1) * c->dH - 2 * c->padH + c->kH + c->adjH;
	if (oW < 1 || oH < 1)
		THError("SpatialFullConvolution: output size %dx%d is too small", oH, oW);
	const size_t need = (size_t)p.B * c->nOutputPlane * c->kH * c->kW * p.H * p.W * esize_of(dt);
	if (hm->col_cap < need) {
		thhip_free(hm->col);
		hm->col = thhip_malloc(need);
		hm->col_cap = need;
	}
	struct planes po = p;
	po.C = c->nOutputPlane;
	void *y = planes_out(m, dt, &po, oH, oW);
	thhip_fullconv2d(thhip_tensor_ptr(in, dt), hm->wpacked, hm->bias, FULLCONV_BIAS_BETA, hm->col, y, p.B, p.C, p.H, p.W,
		c->nOutputPlane, c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, c->adjH, c->adjW, hm->fused_act, hm->thr,
		hm->val, dt);
	return m->output;
}

static THFloatTensor *Hip_SpatialAveragePooling_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct SpatialAveragePooling *q = &m->SpatialAveragePooling;
	struct planes p = planes_of(in, "SpatialAveragePooling");
	int kW = q->kW, kH = q->kH, oH, oW;
	if (!(kW / 2 >= q->padW && kH / 2 >= q->padH))	/* SpatialAveragePooling.c:100-101 */
		THError("pad should be smaller than half of kernel size");
	if (kW == 0)
		kW = p.W;	/* :116-119, global pooling */
	if (kH == 0)
		kH = p.H;
	thhip_pool_outsize(p.H, p.W, kH, kW, q->dH, q->dW, q->padH, q->padW, q->ceil_mode, &oH, &oW);
	if (!(p.W >= kW - 2 * q->padW && p.H >= kH - 2 * q->padH))
		THError("input image smaller than kernel size");
	const void *x = thhip_tensor_ptr(in, hn->dtype);
	void *y = planes_out(m, hn->dtype, &p, oH, oW);
	thhip_avgpool(x, y, p.B, p.C, p.H, p.W, oH, oW, kH, kW, q->dH, q->dW, q->padH, q->padW,
		q->count_include_pad, hn->dtype);
	return m->output;
}

/* frame / dim / stride rule of SoftMax.c:31-57 */
static void softmax_shape(THFloatTensor *in, long *nframe, long *dim, long *stride)
{
	switch (in->nDimension) {
	case 1: *nframe = 1; *dim = in->size[0]; *stride = 1; break;
	case 2: *nframe = in->size[0]; *dim = in->size[1]; *stride = 1; break;
	case 3: *nframe = 1; *dim = in->size[0]; *stride = in->size[1] * in->size[2]; break;
	case 4: *nframe = in->size[0]; *dim = in->size[1]; *stride = in->size[2] * in->size[3]; break;
	default: THError("1D, 2D, 3D or 4D tensor expected");
	}
}

static THFloatTensor *Hip_SoftMax_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	long nframe, dim, stride;
	softmax_shape(in, &nframe, &dim, &stride);
	const void *x = thhip_tensor_ptr(in, hn->dtype);
	void *y = out_resize(m, hn->dtype, in->nDimension, in->size);
	thhip_softmax(x, y, nframe, dim, stride, hn->dtype);
	return m->output;
}

static THFloatTensor *Hip_SpatialBatchNormalization_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	if (hm->passthrough) {	/* folded into the convolution before it */
		out_alias(m, in);
		return m->output;
	}
	if (in->nDimension != 3 && in->nDimension != 4)
		THError("SpatialBatchNormalization: 3D or 4D tensor expected");
	const long B = in->nDimension == 4 ? in->size[0] : 1;
	const long C = in->nDimension == 4 ? in->size[1] : in->size[0];
	const long HW = THFloatTensor_nElement(in) / (B * C);
	if (C != hm->bn_planes)
		THError("SpatialBatchNormalization: %ld planes, module has %ld", C, hm->bn_planes);
	const void *x = thhip_tensor_ptr(in, hn->dtype);
	void *y = out_resize(m, hn->dtype, in->nDimension, in->size);
	thhip_batchnorm(x, y, B, C, HW, hm->bn[0], hm->bn[1], hm->bn[2], hm->bn[3], hn->dtype);
	return m->output;
}

/* View.c:48-100: pointer-only reshape. */
static THFloatTensor *Hip_View_updateOutput(struct module *m, THFloatTensor *in)
{
	struct View *p = &m->View;
	const long nElements = THFloatTensor_nElement(in);
	out_alias(m, in);
	THFloatTensor *o = m->output;
	if (p->nDimension) {
		long size[4], total = 1;
		int ndim, i, j;
		if (in->nDimension == 4) {
			ndim = p->nDimension;
			memcpy(size, p->size, sizeof(size));
		} else {
			ndim = p->nDimension - 1;
			memcpy(size, p->size + 1, sizeof(size[0]) * 3);
		}
		for (i = 0; i < ndim; i++) {
			if (size[i] == 0)
				size[i] = in->size[i];
			else if (size[i] < 0) {
				size[i] = 1;
				for (j = i; j < ndim; j++)
					size[i] *= in->size[j];
			}
			total *= size[i];
		}
		if (total != nElements)
			THError("Wrong number of elements in Reshape: %ld (input) vs %ld (reshaped)\n", nElements, total);
		long stride = 1;
		o->nDimension = ndim;
		for (i = ndim - 1; i >= 0; i--) {
			o->size[i] = size[i];
			o->stride[i] = stride;
			stride *= size[i];
		}
	} else {
		long numElements = p->numElements;
		long batch = in->nDimension == 4 ? in->size[0] : 1;
		if (numElements == -1)
			numElements = nElements / batch;
		else
			batch = nElements / numElements;
		if (batch > 1) {
			o->nDimension = 2;
			o->size[0] = batch;
			o->size[1] = numElements;
			o->stride[0] = numElements;
			o->stride[1] = 1;
		} else {
			o->nDimension = 1;
			o->size[0] = numElements;
			o->stride[0] = 1;
		}
	}
	return o;
}

/* Dropout.c:37-53 at inference with v2 semantics is the identity. */
static THFloatTensor *Hip_Identity_updateOutput(struct module *m, THFloatTensor *in)
{
	out_alias(m, in);
	return m->output;
}

static THFloatTensor *run_network(struct network *net, THFloatTensor *in);

/* Sequential.c:20-51 */
static THFloatTensor *Hip_Sequential_updateOutput(struct module *m, THFloatTensor *in)
{
	in = run_network(m->Sequential.net, in);
	out_alias(m, in);
	return m->output;
}

/* ConcatTable.c:20-50: every branch sees the same input; the "table" handed
 * on is the module itself. */
static THFloatTensor *Hip_ConcatTable_updateOutput(struct module *m, THFloatTensor *in)
{
	struct network *net = m->ConcatTable.net;
	struct hipmod *hm = hipmod_of(m);
	struct hipmod *target = hm->res_target;
	if (hm->shortcut_first) {
		/* the shortcut's convolution is held back and goes out with the main branch's first one */
		thhip_conv_pair_begin();
		net->modules[1].updateOutput(&net->modules[1], in);
		THFloatTensor *other = net->modules[1].output;
		target->res_ptr = thhip_tensor_ptr(other, hipnet_of(m)->dtype);
		target->res_n = THFloatTensor_nElement(other);
		net->modules[0].updateOutput(&net->modules[0], in);
		thhip_conv_pair_end();
		target->res_ptr = 0;
		return (THFloatTensor *)m;
	}
	for (int i = 0; i < net->nelem; i++) {
		if (target && i == (hm->res_from_input ? 0 : 1)) {
			/* what the planned convolution combines its result with: the table's input (identity
			 * branch), or what branch 0 has just made */
			THFloatTensor *other = hm->res_from_input ? in : net->modules[0].output;
			target->res_ptr = thhip_tensor_ptr(other, hipnet_of(m)->dtype);
			target->res_n = THFloatTensor_nElement(other);
		}
		net->modules[i].updateOutput(&net->modules[i], in);
	}
	if (target)
		target->res_ptr = 0;	/* (a convolution that did not run, or refused, leaves the add to the table add) */
	return (THFloatTensor *)m;
}

/* CAddTable.c:32-86, arithmetic as shipped (see thhip_axpby2). */
static THFloatTensor *Hip_CAddTable_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct module *table = (struct module *)in;
	struct network *tn = table->ConcatTable.net;
	const int nelem = tn->nelem, dt = hn->dtype;
	struct module *mods = tn->modules;
	const int sub = m->type == MT_CSubTable;
	if (nelem < 1)
		THError("CAddTable: empty table");
	for (int i = 1; i < nelem; i++) {
		if (mods[i].output->nDimension != mods[0].output->nDimension)
			THError("Sum of tensors of different dimensionality");
		for (int j = 0; j < mods[0].output->nDimension; j++)
			if (mods[0].output->size[j] < mods[i].output->size[j])
				THError("Sum of tensors of different sizes");
	}
	THFloatTensor *a = mods[0].output;
	const long na = THFloatTensor_nElement(a);
	if (hm->added_by_producer) {	/* done, with the Threshold folded into this module, by a convolution's epilogue */
		out_alias(m, mods[hm->added_by_producer - 1].output);
		hm->added_by_producer = 0;
		return m->output;
	}
	void *y = out_resize(m, dt, a->nDimension, a->size);
	if (hm->table_named) {	/* THHipTableArithmetic(1): the first input plus (minus) every other one */
		if (nelem == 1)
			thhip_memcpy_d2d(y, thhip_tensor_ptr(a, dt), (size_t)na * esize_of(dt));
		for (int i = 1; i < nelem; i++)
			thhip_axpby2(i == 1 ? thhip_tensor_ptr(a, dt) : y, thhip_tensor_ptr(mods[i].output, dt), y, na,
				THFloatTensor_nElement(mods[i].output), sub ? -1.0f : 1.0f, (i == nelem - 1) ? hm->fused_act : 0, dt);
	} else if (nelem == 2) {
		THFloatTensor *b = mods[1].output;
		thhip_axpby2(thhip_tensor_ptr(a, dt), thhip_tensor_ptr(b, dt), y, na, THFloatTensor_nElement(b),
			sub ? 1.0f : -1.0f, hm->fused_act, dt);
	} else {
		/* out = a, then every input including the first is added (subtracted) */
		thhip_memcpy_d2d(y, thhip_tensor_ptr(a, dt), (size_t)na * esize_of(dt));
		for (int i = 0; i < nelem; i++)
			thhip_axpby2(y, thhip_tensor_ptr(mods[i].output, dt), y, na, THFloatTensor_nElement(mods[i].output),
				sub ? -1.0f : 1.0f, (i == nelem - 1) ? hm->fused_act : 0, dt);
	}
	return m->output;
}

/* ------------------------------------------------------------------ */
/* uint8 modules                                                       */
/* ------------------------------------------------------------------ */

/* THLowp_ScaleFloat, lowp_basic.c:214-222 */
static int lowp_scale_float(float mult, float sub, float value)
{
	float scaled = (value - sub) * mult;
	if (scaled < 0)
		return 0;
	if (scaled > 255)
		return 255;
	return (unsigned char)scaled;
}

static THFloatTensor *HipLowp_SpatialConvolution_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct SpatialConvolution *c = &m->SpatialConvolution;
	struct convshape s = conv_input_shape(m, in);
	const int oW = (s.W + 2 * c->padW - c->kW) / c->dW + 1;
	const int oH = (s.H + 2 * c->padH - c->kH) / c->dH + 1;
	if (oW < 1 || oH < 1)
		THError("Given input size: (%dx%dx%d). Calculated output size: (%dx%dx%d). Output size is too small",
			c->nInputPlane, s.H, s.W, c->nOutputPlane, oH, oW);
	/* THLowpTensor_mm, lowp_basic.c:309-320: the five integers gemmlowp gets */
	const float im = hn->cur_mult, isub = hn->cur_sub;
	const float om = hm->q_mult, osub = hm->q_sub;
	float scaling = hm->wm * im / om;
	int shift = roundf((log(scaling) / log(2))) + 10;
	int mult = roundf((1 << shift) / scaling);
	int offset = roundf(-osub * hm->wm * im);
	int a_off = roundf(hm->wsub * hm->wm);
	int b_off = roundf(isub * im);
	int zero = roundf(-isub * im);	/* lowp_SpatialConvolution.c:101 */
	int thr = 0, val = 0;
	if (hm->fused_act) {	/* Lowp_Threshold on this module's output codes */
		thr = lowp_scale_float(om, osub, hm->thr);
		val = lowp_scale_float(om, osub, hm->val);
	}
	const void *x = thhip_tensor_ptr(in, THHIP_U8);
	const int K = c->nInputPlane * c->kH * c->kW;
	/* the weights were packed for the planned memory order of the input; with
	 * one pixel per plane both orders coincide */
	if (s.H * s.W > 1 && hn->cur_cl != hm->in_cl)
		THError("uint8 engine: a convolution planned for %s input got the other memory order",
			hm->in_cl ? "channels-last" : "plane-major");
	const int x_cl = hm->x_layout;
	/* image layer -> (Threshold) -> 3x3 / stride 2 max pooling in one kernel, where that kernel takes the shape */
	if (hm->pool_next && x_cl == 2 && hm->out_cl && s.outnd >= 3) {
		const struct SpatialMaxPooling *q = &hn->pub.modules[hm->pool_next].SpatialMaxPooling;
		if (thhip_conv2d_u8_image_pool_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW,
				c->padH, c->padW, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, q->ceil_mode)) {
			const int pH = (oH - 3) / 2 + 1, pW = (oW - 3) / 2 + 1;
			void *yp = conv_out(m, THHIP_U8, &s, c->nOutputPlane, pH, pW);
			thhip_conv2d_u8_image_pool(x, hm->wpacked, hm->addend, yp, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
				c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, zero, a_off, b_off, offset, mult, shift,
				hm->fused_act, thr, val);
			hn->hm[hm->pool_next].pooled_by_producer = 1;
			hn->cur_cl = pH * pW > 1;
			hn->cur_mult = om;
			hn->cur_sub = osub;
			return m->output;
		}
	}
	/* small channels-last images followed by a 3x3 / stride 2 pooling: the kernel that keeps the
	 * input patch in LDS and pools its own codes */
	if (hm->wpatch_u8 && hm->pool_next && x_cl == 1 && hm->out_cl && s.outnd >= 3 &&
	    thhip_conv2d_u8_patch_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW,
			c->padH, c->padW, 1)) {
		const int pH = (oH - 3) / 2 + 1, pW = (oW - 3) / 2 + 1;
		void *yp = conv_out(m, THHIP_U8, &s, c->nOutputPlane, pH, pW);
		thhip_conv2d_u8_patch(x, hm->wpatch_u8, hm->addend, yp, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, zero, a_off, b_off, offset, mult, shift,
			hm->fused_act, thr, val, 1);
		hn->hm[hm->pool_next].pooled_by_producer = 1;
		hn->cur_cl = pH * pW > 1;
		hn->cur_mult = om;
		hn->cur_sub = osub;
		return m->output;
	}
	void *y = conv_out(m, THHIP_U8, &s, c->nOutputPlane, oH, oW);
	/* the same kernel without a pooling, for images one workgroup holds whole (AlexNet's conv3 and conv4) */
	if (hm->wpatch_u8 && x_cl == 1 && hm->out_cl && s.outnd >= 3 && oH * oW <= 192 && oH * oW > 1 &&
	    thhip_conv2d_u8_patch_supported(s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW,
			c->padH, c->padW, 0)) {
		thhip_conv2d_u8_patch(x, hm->wpatch_u8, hm->addend, y, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, zero, a_off, b_off, offset, mult, shift,
			hm->fused_act, thr, val, 0);
		hn->cur_cl = 1;
		hn->cur_mult = om;
		hn->cur_sub = osub;
		return m->output;
	}
	if (hm->wrow_u8 && oH == 1 && oW == 1 && c->padH == 0 && c->padW == 0 && c->kH == s.H && c->kW == s.W &&
	    thhip_linear_batched_u8_supported(s.B, K, c->nOutputPlane))
		thhip_linear_batched_u8(x, hm->wrow_u8, hm->rowsum_u8, hm->addend, y, s.B, K, c->nOutputPlane,
			a_off, b_off, offset, mult, shift, hm->fused_act, thr, val);
	else
		/* a planned channels-last input is an output of this engine: it has the tail */
		thhip_conv2d_u8_layout_tail(x, hm->wpacked, hm->addend, y, s.B, c->nInputPlane, s.H, s.W, c->nOutputPlane,
			c->kH, c->kW, c->dH, c->dW, c->padH, c->padW, zero, a_off, b_off, offset, mult, shift,
			hm->fused_act, thr, val, x_cl, hm->out_cl,
			x_cl == 1 && zero == TH_U8_TAIL_CODE && in->storage && TH_IS_HIP_STORAGE(in->storage->mustfree) &&
			in->storageOffset == 0 ? TH_U8_TAIL : 0);
	hn->cur_cl = hm->out_cl;
	hn->cur_mult = om;
	hn->cur_sub = osub;
	return m->output;
}

static THFloatTensor *HipLowp_Threshold_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct Threshold *t = &m->Threshold;
	if (hm->passthrough) {
		out_alias(m, in);
		return m->output;
	}
	const int thr = lowp_scale_float(hn->cur_mult, hn->cur_sub, t->threshold);
	const int val = lowp_scale_float(hn->cur_mult, hn->cur_sub, t->val);
	const long n = THFloatTensor_nElement(in);
	void *x = thhip_tensor_ptr(in, THHIP_U8);
	if (t->inplace == 1) {
		thhip_threshold_u8(x, x, n, thr, val, 1);
		out_alias(m, in);
	} else {
		void *y = out_resize(m, THHIP_U8, in->nDimension, in->size);
		thhip_threshold_u8(x, y, n, thr, val, 0);
	}
	hm->q_mult = hn->cur_mult;
	hm->q_sub = hn->cur_sub;
	return m->output;
}

static THFloatTensor *HipLowp_SpatialMaxPooling_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	struct SpatialMaxPooling *q = &m->SpatialMaxPooling;
	if (hm->pooled_by_producer) {	/* done by the convolution before it */
		hm->pooled_by_producer = 0;
		out_alias(m, in);
		hm->q_mult = hn->cur_mult;
		hm->q_sub = hn->cur_sub;
		return m->output;
	}
	struct planes p = planes_of(in, "SpatialMaxPooling");
	int oH, oW;
	thhip_pool_outsize(p.H, p.W, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, q->ceil_mode, &oH, &oW);
	if (oH < 1 || oW < 1)
		THError("SpatialMaxPooling: input %dx%d smaller than the window", p.H, p.W);
	const void *x = thhip_tensor_ptr(in, THHIP_U8);
	void *y = planes_out(m, THHIP_U8, &p, oH, oW);
	if (hn->cur_cl)
		thhip_maxpool_u8_cl(x, y, p.B, p.C, p.H, p.W, oH, oW, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW);
	else
		thhip_maxpool(x, y, p.B, p.C, p.H, p.W, oH, oW, q->kH, q->kW, q->dH, q->dW, q->padH, q->padW, THHIP_U8);
	hm->q_mult = hn->cur_mult;	/* lowp_SpatialMaxPooling.c:104-105 */
	hm->q_sub = hn->cur_sub;
	return m->output;
}

static THFloatTensor *HipLowp_SoftMax_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	long nframe, dim, stride;
	softmax_shape(in, &nframe, &dim, &stride);
	if (hn->cur_cl && stride > 1)
		THError("uint8 engine: channels-last codes reached SoftMax");
	hn->cur_cl = 0;
	const void *x = thhip_tensor_ptr(in, THHIP_U8);
	void *y = out_resize(m, THHIP_U8, in->nDimension, in->size);
	hn->cur_mult = thhip_softmax_u8(x, y, nframe, dim, stride, hn->cur_mult, hn->cur_sub);
	hn->cur_sub = 0;
	hm->q_mult = hn->cur_mult;
	hm->q_sub = 0;
	return m->output;
}

static THFloatTensor *HipLowp_View_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	if (hn->cur_cl && THFloatTensor_nElement(in) != in->size[0] * (in->nDimension > 1 ? in->size[1] : 1) &&
	    !(in->nDimension == 3 && in->size[1] * in->size[2] == 1))
		THError("uint8 engine: channels-last codes reached View");
	hn->cur_cl = 0;
	Hip_View_updateOutput(m, in);
	hm->q_mult = hn->cur_mult;
	hm->q_sub = hn->cur_sub;
	return m->output;
}

static THFloatTensor *HipLowp_Identity_updateOutput(struct module *m, THFloatTensor *in)
{
	struct hipnet *hn = hipnet_of(m);
	struct hipmod *hm = hipmod_of(m);
	out_alias(m, in);
	hm->q_mult = hn->cur_mult;
	hm->q_sub = hn->cur_sub;
	return m->output;
}

/* ------------------------------------------------------------------ */
/* executor                                                            */
/* ------------------------------------------------------------------ */

int th_debug, th_profile, th_minmax;
double th_convtot, th_convflops;

static double seconds_now(void)
{
	struct timespec ts;
	clock_gettime(CLOCK_MONOTONIC, &ts);
	return ts.tv_sec + ts.tv_nsec * 1e-9;
}

static int is_conv_type(int type)
{
	return type == MT_SpatialConvolutionMM || type == MT_SpatialConvolutionVirtMM || type == MT_SpatialConvolution;
}

/* The output of a module that left its work to its consumer in the last forward (the image layer of a half
 * network, above), computed now by the module's own kernel: for callers that read module outputs. */
void thhip_materialize_output(struct network *net, int idx)
{
	struct hipnet *hn = (struct hipnet *)net;
	struct hipmod *hm = &hn->hm[idx];
	if (!hm->deferred)
		return;
	struct module *m = &net->modules[idx];
	struct SpatialConvolution *c = &m->SpatialConvolution;
	thhip_conv2d_layout(hm->front_img, hm->wpacked, hm->scale, hm->bias, thhip_tensor_ptr(m->output, hn->dtype), hm->front_B,
		c->nInputPlane, hm->front_H, hm->front_W, c->nOutputPlane, c->kH, c->kW, c->dH, c->dW, c->padH, c->padW,
		hm->fused_act, hm->thr, hm->val, hn->dtype, hm->x_layout, hm->out_cl);
	hm->deferred = 0;
}

/* forward(), thapi.c:158-235, without the per-layer frees; with th_profile
 * the stream is drained around each module the way the OpenCL engine calls
 * clFinish (thapi.c:213-216), so the printed seconds are kernel time. */
static int g_run_depth;	/* 1 while the top-level module list runs, more inside containers */

static THFloatTensor *run_modules(struct network *net, THFloatTensor *in, int first, int last);

static THFloatTensor *run_network(struct network *net, THFloatTensor *in)
{
	((struct hipnet *)net)->cur_cl = 0;	/* inputs arrive in the reference's plane-major order */
	return run_modules(net, in, 0, net->nelem);
}

/* modules [first, last) of the list, the first of them on `in` */
static THFloatTensor *run_modules(struct network *net, THFloatTensor *in, int first, int last)
{
	double t = 0;
	g_run_depth++;
	for (int i = first; i < last; i++) {
		struct module *m = &net->modules[i];
		if (th_profile) {
			thhip_sync();
			t = seconds_now();
		}
		/* A module that names its inputs (the loaders of graph formats fill
		 * ninputs / inputs[]: thapi.c:173-193) takes them from the modules it
		 * names, which come earlier in the list; several inputs are handed over
		 * as a table, the way ConcatTable does it.  Without named inputs the
		 * network is sequential. */
		if (m->ninputs == 1 && m->type != MT_JoinTable) {
			if (m->inputs[0] < 0 || m->inputs[0] >= i)
				THError("module %d names input %d, which has not run yet", i + 1, m->inputs[0] + 1);
			in = m->updateOutput(m, net->modules[m->inputs[0]].output);
		} else if (m->ninputs >= 1) {
			struct module srcs[MAXMODULEINPUTS], table;
			struct network subnet;
			if (m->ninputs > MAXMODULEINPUTS)
				THError("module %d: too many inputs", i + 1);
			for (int j = 0; j < m->ninputs; j++) {
				if (m->inputs[j] < 0 || m->inputs[j] >= i)
					THError("module %d names input %d, which has not run yet", i + 1, m->inputs[j] + 1);
				srcs[j].output = net->modules[m->inputs[j]].output;
			}
			subnet.nelem = m->ninputs;
			subnet.modules = srcs;
			subnet.engine = net->engine;
			table.ConcatTable.net = &subnet;
			in = m->updateOutput(m, (THFloatTensor *)&table);
		} else
			in = m->updateOutput(m, in);
		/* thapi.c:197-202: the executor (not the containers) prints every module
		 * output's range.  The uint8 engine prints the range of the values its
		 * codes stand for (the reference reads the code bytes as floats there). */
		if (th_minmax && g_run_depth == 1 && m->type != MT_ConcatTable && in && in->storage) {
			struct hipnet *hn = (struct hipnet *)net;
			float mn, mx;
			thhip_minmax(thhip_tensor_ptr(in, hn->dtype), THFloatTensor_nElement(in), hn->dtype, &mn, &mx);
			if (hn->dtype == THHIP_U8 && hn->cur_mult != 0) {
				mn = mn * (1 / hn->cur_mult) + hn->cur_sub;	/* lowp_basic.c:52-55 */
				mx = mx * (1 / hn->cur_mult) + hn->cur_sub;
			}
			printf("Layer %d output: min=%f, max=%f\n", i + 1, mn, mx);
		}
		if (th_profile) {
			thhip_sync();
			t = seconds_now() - t;
			if (is_conv_type(m->type) && m->type != MT_ConcatTable) {
				double flops = 2.0 * THFloatTensor_nElement(in) * m->SpatialConvolution.nInputPlane *
					m->SpatialConvolution.kW * m->SpatialConvolution.kH;
				printf("%f seconds for module %d, %f Gflops/s\n", t, i + 1, flops * 1e-9 / t);
				th_convtot += t;
				th_convflops += flops;
			} else
				printf("%f seconds for module %d\n", t, i + 1);
		}
		if (th_debug > 1 && m->type != MT_ConcatTable)
			printf("%d) %d %d %ld %ld %ld %ld\n", i + 1, m->type, in->nDimension, in->size[0], in->size[1],
				in->size[2], in->size[3]);
	}
	g_run_depth--;
	return in;
}

/* How many leading modules of the list work image by image on kernels that honour a window of the batch
 * (thhip_batch_window): the first two convolutions with what follows each of them up to the third.  0:
 * none (a graph, a list that does not start that way, or nothing after them). */
static int window_prefix(struct network *net)
{
	int convs = 0, i;
	if (((struct hipnet *)net)->dag || net->engine != ENGINE_HIP)
		return 0;
	for (i = 0; i < net->nelem; i++) {
		const int type = net->modules[i].type;
		if (net->modules[i].ninputs)
			return 0;
		if (is_conv_type(type)) {
			if (convs == 2)
				break;
			convs++;
		} else if (type != MT_Threshold && type != MT_SpatialMaxPooling && type != MT_SpatialBatchNormalization &&
			   type != MT_Dropout)
			break;
	}
	return convs && i < net->nelem ? i : 0;
}

/* forward passes so far whose first modules ran window by window (for the tests) */
static long g_windowed_forwards;
long thhip_windowed_forwards(void)
{
	return g_windowed_forwards;
}

/* thhip_forward, the first modules window by window: before(ctx, w) makes the images of window w ready
 * (their upload may still be on its way while the window before is worked on).  Where the list does not
 * allow it, or a module of the prefix turns out to launch something that works on the whole batch (noted
 * by hip_rt.hip; remembered for the network), every window is made ready first and the list runs on the
 * whole batch as thhip_forward runs it: what the first window's launches wrote is written again. */
THFloatTensor *thhip_forward_windows(struct network *net, THFloatTensor *in, int nwin, const int *b0, const int *bn,
	void (*before)(void *ctx, int w), void *ctx)
{
	struct hipnet *hn = (struct hipnet *)net;
	const int prefix = nwin > 1 && !hn->no_windows && !th_profile && !th_minmax && !th_debug ? window_prefix(net) : 0;
	int w = 0;
	if (prefix) {
		THFloatTensor *x = in;
		thhip_batch_window_violated();
		for (; w < nwin; w++) {
			before(ctx, w);
			thhip_batch_window(b0[w], bn[w]);
			hn->cur_cl = 0;
			x = run_modules(net, in, 0, prefix);
			thhip_batch_window(0, 0);
			if (thhip_batch_window_violated()) {
				hn->no_windows = 1;
				w++;
				break;
			}
		}
		if (!hn->no_windows) {
			g_windowed_forwards++;
			return run_modules(net, x, prefix, net->nelem);
		}
	}
	for (; w < nwin; w++)
		before(ctx, w);
	return thhip_forward(net, in);
}

THFloatTensor *thhip_forward(struct network *net, THFloatTensor *in)
{
	if (net->engine != ENGINE_HIP && net->engine != ENGINE_HIPLOWP)
		THError("This library only runs networks made by THCreateHipNetwork / THCreateHipLowpNetwork "
			"(engine %d given); it carries no CPU path", net->engine);
	th_convtot = 0;
	th_convflops = 0;
	THFloatTensor *out = run_network(net, in);
	if (th_profile)
		printf("%f seconds for convolutions %f Gflops/s\n", th_convtot, th_convflops * 1e-9 / th_convtot);
	return out;
}

/* ------------------------------------------------------------------ */
/* engine construction                                                 */
/* ------------------------------------------------------------------ */

static THFloatTensor *contiguous_host_floats(THFloatTensor *t, const char *what, long expect)
{
	if (!t || !t->storage || !t->storage->data)
		return 0;
	if (TH_IS_HIP_STORAGE(t->storage->mustfree))
		THError("%s already lives on the device: pass the host network to THCreateHipNetwork", what);
	long stride = 1;
	for (int i = t->nDimension - 1; i >= 0; i--) {
		if (t->size[i] != 1 && t->stride[i] != stride)
			THError("%s is not contiguous", what);
		stride *= t->size[i];
	}
	if (expect >= 0 && THFloatTensor_nElement(t) != expect)
		THError("%s has %ld elements, %ld expected", what, THFloatTensor_nElement(t), expect);
	return t;
}

static float *upload_floats(THFloatTensor *t, const char *what, long expect)
{
	if (!contiguous_host_floats(t, what, expect))
		return 0;
	const long n = THFloatTensor_nElement(t);
	float *d = thhip_malloc(sizeof(float) * n);
	thhip_memcpy_h2d(d, THFloatTensor_data(t), sizeof(float) * n);
	return d;
}

/* THLowpTensor_newFromFloatTensor's arithmetic on the host for the (small,
 * one-off) weight and bias tensors: lowp_basic.c:15-35. */
static unsigned char *quantize_host(const float *buf, long len, float *mult_out, float *sub_out)
{
	unsigned char *dst = malloc(len ? len : 1);
	float min = 0, max = 0, mult;
	long i;
	for (i = 0; i < len; i++) {
		if (buf[i] < min)
			min = buf[i];
		if (buf[i] > max)
			max = buf[i];
	}
	if (max - min > 0)
		mult = 255.0 / (max - min);
	else
		mult = 0;
	const float zero = roundf(min * mult);
	for (i = 0; i < len; i++)
		dst[i] = (unsigned char)(int)(roundf(buf[i] * mult) - zero);
	*mult_out = mult;
	*sub_out = min;
	return dst;
}

static struct network *to_hip(struct network *net, int engine, int dtype, float range);

static void convert_module(struct hipnet *hn, struct network *src, int i, int engine, int dtype, float range)
{
	struct module *m = &hn->pub.modules[i];
	struct module *sm = &src->modules[i];
	struct hipmod *hm = &hn->hm[i];
	const int lowp = engine == ENGINE_HIPLOWP;
	m->output = THFloatTensor_new();
	m->net = &hn->pub;
	m->nnfree = 0;
	hm->q_mult = 255 / range;	/* lowp_basic.c:135-136 */
	hm->q_sub = -range / 2;
	switch (sm->type) {
	case MT_SpatialConvolution:
	case MT_SpatialConvolutionMM:
	case MT_SpatialConvolutionVirtMM:
	case MT_Linear: {
		THFloatTensor *w, *b;
		int Co, K, Ci, kHW;
		if (sm->type == MT_Linear) {
			/* Linear runs as a 1x1 convolution (cudnn_basic.c:244-265) */
			w = sm->Linear.weight;
			b = sm->Linear.bias;
			if (sm->Linear.commute)
				THError("Linear with commute is not supported by the HIP engine");
			if (!w || w->nDimension != 2)
				THError("Linear weight must be a matrix");
			Co = (int)w->size[0];
			K = (int)w->size[1];
			Ci = K;
			kHW = 1;
			memset(&m->SpatialConvolution, 0, sizeof(m->SpatialConvolution));
			m->type = MT_SpatialConvolutionMM;
			m->SpatialConvolution.dW = m->SpatialConvolution.dH = 1;
			m->SpatialConvolution.kW = m->SpatialConvolution.kH = 1;
			m->SpatialConvolution.nOutputPlane = Co;
			m->SpatialConvolution.nInputPlane = K;
			hm->is_linear = 1;
		} else {
			struct SpatialConvolution *c = &sm->SpatialConvolution;
			w = c->weight;
			b = c->bias;
			Co = c->nOutputPlane;
			Ci = c->nInputPlane;
			kHW = c->kH * c->kW;
			K = Ci * kHW;
		}
		contiguous_host_floats(w, "convolution weight", (long)Co * K);
		m->SpatialConvolution.weight = m->SpatialConvolution.bias = m->SpatialConvolution.finput = 0;
		if (lowp) {
			float bm = 0, bsub = 0;
			unsigned char *wq = quantize_host(THFloatTensor_data(w), (long)Co * K, &hm->wm, &hm->wsub);
			hm->wq_host = wq;	/* plan_channels_last() packs them once the input's order is known */
			if (!contiguous_host_floats(b, "convolution bias", Co))
				THError("the uint8 engine needs a bias on every convolution (lowp_SpatialConvolution.c:111-120)");
			unsigned char *bq = quantize_host(THFloatTensor_data(b), Co, &bm, &bsub);
			int *addend = malloc(sizeof(int) * Co);
			/* lowp_SpatialConvolution.c:112-119 */
			float mult = hm->q_mult / bm;
			int add = roundf(bsub * hm->q_mult);
			for (int o = 0; o < Co; o++) {
				int a = bq[o];
				a = roundf(a * mult) + add;
				addend[o] = a;
			}
			hm->addend = thhip_malloc(sizeof(int) * Co);
			thhip_memcpy_h2d(hm->addend, addend, sizeof(int) * Co);
			free(addend);
			free(bq);
			m->updateOutput = HipLowp_SpatialConvolution_updateOutput;
		} else {
			hm->wpacked = thhip_conv_pack_weight(THFloatTensor_data(w), Co, Ci, kHW, dtype);
			hm->bias = upload_floats(b, "convolution bias", Co);
			m->updateOutput = Hip_SpatialConvolution_updateOutput;
		}
		break;
	}
	case MT_SpatialFullConvolution: {
		if (lowp)
			THError("MT_SpatialFullConvolution not supported in Lowp");
		struct SpatialFullConvolution *c = &sm->SpatialFullConvolution;
		THFloatTensor *w = c->weight;
		if (!w || w->nDimension != 4 || c->dW < 1 || c->dH < 1)
			THError("SpatialFullConvolution needs a 4-D weight [nInputPlane][nOutputPlane][kH][kW] and positive strides");
		/* the weight's own extents rule (SpatialFullConvolution.c:153-154) */
		m->SpatialFullConvolution.nInputPlane = (int)w->size[0];
		m->SpatialFullConvolution.nOutputPlane = (int)w->size[1];
		m->SpatialFullConvolution.kH = (int)w->size[2];
		m->SpatialFullConvolution.kW = (int)w->size[3];
		if (!contiguous_host_floats(w, "full convolution weight", -1))
			THError("SpatialFullConvolution without weights");
		hm->wpacked = thhip_fullconv_pack_weight(THFloatTensor_data(w), (int)w->size[0], (int)w->size[1], (int)w->size[2],
			(int)w->size[3], dtype);
		hm->bias = upload_floats(c->bias, "full convolution bias", w->size[1]);
		m->SpatialFullConvolution.weight = m->SpatialFullConvolution.bias = 0;
		m->SpatialFullConvolution.ones = m->SpatialFullConvolution.columns = 0;
		m->updateOutput = Hip_SpatialFullConvolution_updateOutput;
		break;
	}
	case MT_SpatialMaxUnpooling: {
		if (lowp)
			THError("MT_SpatialMaxUnpooling not supported in Lowp");
		/* SpatialMaxUnpooling.c:63-72: the pooling is looked up among the
		 * modules of the same network by its loader object */
		hm->pool_index = -1;
		for (int j = 0; j < src->nelem; j++)
			if (src->modules[j].type == MT_SpatialMaxPooling && sm->SpatialMaxUnpooling.pooling &&
			    src->modules[j].nnmodule == sm->SpatialMaxUnpooling.pooling) {
				hm->pool_index = j;
				break;
			}
		if (hm->pool_index < 0)
			THError("SpatialMaxUnpooling: its SpatialMaxPooling is not a module of the same network");
		hn->hm[hm->pool_index].want_indices = 1;
		m->updateOutput = Hip_SpatialMaxUnpooling_updateOutput;
		break;
	}
	case MT_Threshold:
		m->updateOutput = lowp ? HipLowp_Threshold_updateOutput : Hip_Threshold_updateOutput;
		break;
	case MT_SpatialMaxPooling:
		m->SpatialMaxPooling.indices = 0;	/* only SpatialMaxUnpooling reads them */
		m->updateOutput = lowp ? HipLowp_SpatialMaxPooling_updateOutput : Hip_SpatialMaxPooling_updateOutput;
		break;
	case MT_SoftMax:
		m->updateOutput = lowp ? HipLowp_SoftMax_updateOutput : Hip_SoftMax_updateOutput;
		break;
	case MT_Dropout:
		if (!sm->Dropout.v2)
			THError("Non v2 dropout not supported in the HIP engine");
		m->Dropout.inplace = 1;
		m->updateOutput = lowp ? HipLowp_Identity_updateOutput : Hip_Identity_updateOutput;
		break;
	case MT_Identity:
		m->updateOutput = lowp ? HipLowp_Identity_updateOutput : Hip_Identity_updateOutput;
		break;
	case MT_View:
		m->updateOutput = lowp ? HipLowp_View_updateOutput : Hip_View_updateOutput;
		break;
	case MT_SpatialAveragePooling:
		if (lowp)
			THError("MT_SpatialAveragePooling not supported in lowp");
		m->updateOutput = Hip_SpatialAveragePooling_updateOutput;
		break;
	case MT_SpatialBatchNormalization: {
		if (lowp)
			THError("MT_SpatialBatchNormalization not supported in Lowp");
		struct SpatialBatchNormalization *bn = &sm->SpatialBatchNormalization;
		if (!contiguous_host_floats(bn->running_mean, "running_mean", -1) ||
		    !contiguous_host_floats(bn->running_var, "running_var", -1))
			THError("SpatialBatchNormalization needs running_mean and running_var");
		const long C = THFloatTensor_nElement(bn->running_mean);
		contiguous_host_floats(bn->running_var, "running_var", C);	/* one variance per mean */
		float *invstd = malloc(sizeof(float) * C);
		const float *var = THFloatTensor_data(bn->running_var);
		for (long f = 0; f < C; f++)
			invstd[f] = 1 / sqrt(var[f] + bn->eps);	/* SpatialBatchNormalization.c:85 */
		hm->bn_planes = C;
		hm->bn[0] = upload_floats(bn->running_mean, "running_mean", C);
		hm->bn[1] = thhip_malloc(sizeof(float) * C);
		thhip_memcpy_h2d(hm->bn[1], invstd, sizeof(float) * C);
		free(invstd);
		hm->bn[2] = upload_floats(bn->weight, "batchnorm weight", C);
		hm->bn[3] = upload_floats(bn->bias, "batchnorm bias", C);
		memset(&m->SpatialBatchNormalization, 0, sizeof(m->SpatialBatchNormalization));
		m->SpatialBatchNormalization.eps = bn->eps;
		m->updateOutput = Hip_SpatialBatchNormalization_updateOutput;
		break;
	}
	case MT_Sequential:
		if (lowp)
			THError("MT_Sequential not supported in lowp");
		m->Sequential.net = to_hip(sm->Sequential.net, engine, dtype, range);
		m->updateOutput = Hip_Sequential_updateOutput;
		break;
	case MT_ConcatTable:
		if (lowp)
			THError("MT_ConcatTable not supported in lowp");
		m->ConcatTable.net = to_hip(sm->ConcatTable.net, engine, dtype, range);
		m->updateOutput = Hip_ConcatTable_updateOutput;
		break;
	case MT_CAddTable:
	case MT_CSubTable:
		if (lowp)
			THError("MT_CAddTable not supported in lowp");
		m->updateOutput = Hip_CAddTable_updateOutput;
		hm->table_named = g_table_math;
		break;
	default:
		THError("module type %d is not supported by the HIP engine", sm->type);
	}
}

/* uint8 and half engines: decides which tensors live channels-last
 * ([B][H][W][C]) in memory.  A convolution reads 16 bytes of adjacent planes of
 * one pixel per operand vector (16 codes, 8 halfs), so it takes channels-last
 * input whenever its planes come in whole vectors and the producer is another
 * convolution reached only through modules that work in either order
 * (Threshold, max pooling, Dropout, Identity, a batch norm folded away).
 * Network inputs and every tensor another module sees stay plane-major.
 * Weights are (re-)packed here, because their K order follows how the input
 * is read; so are the row-major copies of the uint8 one-position (matrix) path. */
static void plan_channels_last(struct hipnet *hn, struct network *src)
{
	const int lowp = hn->pub.engine == ENGINE_HIPLOWP;
	const int vec = lowp ? 16 : 8;
	int prev = -1;
	if (!lowp && hn->dtype == THHIP_F32)
		return;		/* fp32 gathers element-wise at full speed; it stays plane-major */
	/* (a graph keeps every tensor plane-major: the chains below assume that a
	 * module reads what the module before it wrote) */
	for (int i = 0; i < hn->pub.nelem && !hn->dag; i++) {
		struct module *m = &hn->pub.modules[i];
		struct hipmod *hm = &hn->hm[i];
		if (is_conv_type(m->type)) {
			if (prev >= 0 && m->SpatialConvolution.nInputPlane % vec == 0) {
				for (int j = prev; j < i; j++)
					hn->hm[j].out_cl = 1;
				hm->in_cl = 1;
			}
			prev = i;
		} else if (m->type != MT_Threshold && !(m->type == MT_SpatialMaxPooling && !hm->want_indices) && m->type != MT_Dropout &&
			m->type != MT_Identity && !(m->type == MT_SpatialBatchNormalization && hm->passthrough))
			prev = -1;
	}
	for (int i = 0; i < hn->pub.nelem && !lowp; i++) {
		struct module *m = &hn->pub.modules[i];
		struct hipmod *hm = &hn->hm[i];
		if (!is_conv_type(m->type) || !hm->in_cl)
			continue;
		/* packed plane-major by convert_module: pack again for channels-last input */
		const struct SpatialConvolution *c = &m->SpatialConvolution;
		THFloatTensor *w = src->modules[i].type == MT_Linear ? src->modules[i].Linear.weight :
			src->modules[i].SpatialConvolution.weight;
		thhip_free(hm->wpacked);
		hm->x_layout = 1;
		hm->wpacked = thhip_conv_pack_weight_layout(THFloatTensor_data(w), c->nOutputPlane, c->nInputPlane, c->kH, c->kW,
			hn->dtype, 1);
	}
	for (int i = 0; i < hn->pub.nelem; i++) {
		struct module *m = &hn->pub.modules[i];
		struct hipmod *hm = &hn->hm[i];
		if (!hm->wq_host)
			continue;
		const struct SpatialConvolution *c = &m->SpatialConvolution;
		const int Co = c->nOutputPlane, Ci = c->nInputPlane, kHW = c->kH * c->kW;
		const long K = (long)Ci * kHW;
		/* the image layer (<= 4 planes, plane-major) goes through the four-plane pixel copy */
		hm->x_layout = hm->in_cl ? 1 : Ci <= 4 ? 2 : 0;
		hm->wpacked = thhip_conv_pack_weight_u8_layout(hm->wq_host, Co, Ci, c->kH, c->kW, hm->x_layout);
		/* stride-1 layers between channels-last tensors with planes in blocks of 64 may run on the
		 * kernel that keeps its input patch in LDS (decided per forward by the image size) */
		if (hm->in_cl && hm->out_cl && Ci % 64 == 0 && Co % 64 == 0 && c->dH == 1 && c->dW == 1 && kHW >= 4)
			hm->wpatch_u8 = thhip_conv_pack_weight_u8_patch(hm->wq_host, Co, Ci, c->kH, c->kW);
		if (K % 16 == 0 && K >= 512) {
			unsigned char *rows = hm->wq_host;
			if (hm->in_cl && kHW > 1) {
				/* k = (tap, plane) instead of (plane, tap) */
				rows = malloc((size_t)Co * K);
				for (int o = 0; o < Co; o++)
					for (int ci = 0; ci < Ci; ci++)
						for (int t = 0; t < kHW; t++)
							rows[(size_t)o * K + (size_t)t * Ci + ci] =
								hm->wq_host[(size_t)o * K + (size_t)ci * kHW + t];
			}
			hm->wrow_u8 = thhip_linear_pack_weight_u8(rows, Co, (int)K);
			hm->rowsum_u8 = thhip_u8_rowsums(rows, Co, (int)K);
			if (rows != hm->wq_host)
				free(rows);
		}
		free(hm->wq_host);
		hm->wq_host = 0;
	}
}

/* The convolution whose result is a ConcatTable branch's output: the branch itself, or the last
 * module of a Sequential before its folded batch norms, if that is a convolution with no
 * Threshold and no pooling of its own in its epilogue.  NULL otherwise. */
static struct module *branch_last_conv(struct module *b)
{
	if (b->type == MT_Sequential && b->Sequential.net) {
		struct network *sn = b->Sequential.net;
		struct hipnet *shn = (struct hipnet *)sn;
		int i = sn->nelem - 1;
		if (shn->dag)
			return 0;
		while (i >= 0 && shn->hm[i].passthrough && sn->modules[i].type == MT_SpatialBatchNormalization)
			i--;
		if (i < 0)
			return 0;
		b = &sn->modules[i];
	}
	if (!is_conv_type(b->type))
		return 0;
	struct hipmod *hm = hipmod_of(b);
	if (hm->is_linear || hm->fused_act || hm->pool_next || hm->passthrough)
		return 0;
	return b;
}

static int foldable_threshold(struct module *t)
{
	return t->type == MT_Threshold && t->Threshold.alpha == 0;
}

static struct network *to_hip(struct network *net, int engine, int dtype, float range)
{
	struct hipnet *hn = calloc(1, sizeof(*hn));
	hn->pub.nelem = net->nelem;
	hn->pub.engine = engine;
	hn->pub.modules = malloc(sizeof(struct module) * (net->nelem ? net->nelem : 1));
	memcpy(hn->pub.modules, net->modules, sizeof(struct module) * net->nelem);
	hn->hm = calloc(net->nelem ? net->nelem : 1, sizeof(struct hipmod));
	hn->dtype = dtype;
	hn->range = range;
	for (int i = 0; i < net->nelem; i++)
		convert_module(hn, net, i, engine, dtype, range);
	/* Modules that name their inputs make the list a graph: a module may then be
	 * folded into its producer only if it is that producer's sole consumer. */
	int dag = 0;
	int *consumers = calloc(net->nelem ? net->nelem : 1, sizeof(int));
	for (int i = 0; i < net->nelem; i++) {
		if (net->modules[i].ninputs > 0)
			dag = 1;
		for (int j = 0; j < net->modules[i].ninputs && j < MAXMODULEINPUTS; j++)
			if (net->modules[i].inputs[j] >= 0 && net->modules[i].inputs[j] < net->nelem)
				consumers[net->modules[i].inputs[j]]++;
	}
	hn->dag = dag;
#define FEEDS_ONLY(a, b) (!dag ? (b) == (a) + 1 : (net->modules[b].ninputs == 1 && net->modules[b].inputs[0] == (a) && consumers[a] == 1))
	if (dag && engine == ENGINE_HIPLOWP)
		for (int i = 1; i < net->nelem; i++)
			if (net->modules[i].ninputs > 1 || (net->modules[i].ninputs == 1 && net->modules[i].inputs[0] != i - 1))
				THError("the uint8 engine runs sequential networks only (module %d names other inputs)", i + 1);
	/* fold a SpatialBatchNormalization into the convolution that feeds it:
	 * ((sum + cb - mean) * invstd) * w + b  =  sum * s + ((cb - mean) * s + b),  s = invstd * w
	 * (SpatialBatchNormalization.c:57-116; the reference's loader-side folding is absorb_bn, onnx.cc:529-557) */
	for (int i = 0; i + 1 < net->nelem && engine == ENGINE_HIP && g_fold_bn; i++) {
		struct module *m = &hn->pub.modules[i], *sb = &net->modules[i + 1];
		if (!is_conv_type(m->type) || hn->hm[i].is_linear || sb->type != MT_SpatialBatchNormalization || !FEEDS_ONLY(i, i + 1))
			continue;
		struct SpatialBatchNormalization *bn = &sb->SpatialBatchNormalization;
		const int Co = m->SpatialConvolution.nOutputPlane;
		if (THFloatTensor_nElement(bn->running_mean) != Co || THFloatTensor_nElement(bn->running_var) != Co)
			continue;	/* the mismatch is reported by the module's own conversion or when the network runs */
		const float *mean = THFloatTensor_data(bn->running_mean), *var = THFloatTensor_data(bn->running_var);
		const float *w = contiguous_host_floats(bn->weight, "batchnorm weight", Co) ? THFloatTensor_data(bn->weight) : 0;
		const float *b = contiguous_host_floats(bn->bias, "batchnorm bias", Co) ? THFloatTensor_data(bn->bias) : 0;
		THFloatTensor *cbt = net->modules[i].SpatialConvolution.bias;
		const float *cb = contiguous_host_floats(cbt, "convolution bias", Co) ? THFloatTensor_data(cbt) : 0;
		float *scale = malloc(sizeof(float) * Co), *shift = malloc(sizeof(float) * Co);
		for (int o = 0; o < Co; o++) {
			const float invstd = 1 / sqrt(var[o] + bn->eps);
			scale[o] = w ? invstd * w[o] : invstd;
			shift[o] = ((cb ? cb[o] : 0) - mean[o]) * scale[o] + (b ? b[o] : 0);
		}
		thhip_free(hn->hm[i].bias);
		hn->hm[i].scale = thhip_malloc(sizeof(float) * Co);
		hn->hm[i].bias = thhip_malloc(sizeof(float) * Co);
		thhip_memcpy_h2d(hn->hm[i].scale, scale, sizeof(float) * Co);
		thhip_memcpy_h2d(hn->hm[i].bias, shift, sizeof(float) * Co);
		free(scale);
		free(shift);
		hn->hm[i + 1].passthrough = 1;
	}
	/* fold a Threshold into the epilogue of the module that feeds it */
	for (int i = 0; i + 1 < net->nelem; i++) {
		struct module *m = &hn->pub.modules[i];
		int ti = i + 1;
		if (!FEEDS_ONLY(i, i + 1))
			continue;
		if (hn->hm[ti].passthrough && hn->pub.modules[ti].type == MT_SpatialBatchNormalization && ti + 1 < net->nelem) {
			ti++;	/* conv -> (folded BN) -> Threshold */
			if (!FEEDS_ONLY(i + 1, i + 2))
				continue;
		}
		struct module *t = &hn->pub.modules[ti];
		if (!foldable_threshold(t))
			continue;
		if (is_conv_type(m->type) || (m->type == MT_SpatialFullConvolution && ti == i + 1)) {
			hn->hm[i].fused_act = 1;
			hn->hm[i].thr = t->Threshold.threshold;
			hn->hm[i].val = t->Threshold.val;
			hn->hm[ti].passthrough = 1;
		} else if (ti != i + 1) {
			continue;
		} else if ((m->type == MT_CAddTable || m->type == MT_CSubTable) &&
			t->Threshold.threshold == 0 && t->Threshold.val == 0) {
			hn->hm[i].fused_act = 1;
			hn->hm[i + 1].passthrough = 1;
		}
	}
	plan_channels_last(hn, net);
	/* a 2x2 / stride 2 max pooling right after a convolution (and its folded
	 * Threshold; half engines: between channels-last tensors) may be done by the
	 * convolution's epilogue; whether it is, is decided per forward by the layer's shape */
	for (int i = 0; i + 1 < net->nelem && engine == ENGINE_HIP; i++) {
		/* (fp32: plane-major tensors, the kernel that loads its tiles straight into LDS) */
		if (!is_conv_type(hn->pub.modules[i].type) || hn->hm[i].is_linear || (dtype != THHIP_F32 && !hn->hm[i].in_cl))
			continue;
		int j = i + 1, chain = FEEDS_ONLY(i, i + 1);
		while (j < net->nelem && hn->hm[j].passthrough) {
			j++;
			chain = chain && j < net->nelem && FEEDS_ONLY(j - 1, j);
		}
		/* (in a graph: the pooling, through the folded modules between, is the convolution's only consumer) */
		if (j >= net->nelem || !chain || hn->pub.modules[j].type != MT_SpatialMaxPooling || hn->hm[j].want_indices)
			continue;
		const struct SpatialMaxPooling *q = &hn->pub.modules[j].SpatialMaxPooling;
		if (q->kW == 2 && q->kH == 2 && q->dW == 2 && q->dH == 2 && q->padW == 0 && q->padH == 0 && !q->ceil_mode)
			hn->hm[i].pool_next = j;
		else if (dtype == THHIP_F32)	/* any window: by the kernel that adds the parts of a K split (layers of a few tiles) */
			hn->hm[i].pool_next = j;
	}
	/* half engines, a list of modules: the image layer (3 -> 64 planes, 3x3 / stride 1 / padding 1, plane-major
	 * in, channels-last out) followed, through its folded Threshold, by a 3x3 / stride 1 / padding 1 layer of at
	 * most 256 planes between channels-last tensors: that layer may compute the image layer's output itself */
	for (int i = 0; i + 1 < net->nelem && engine == ENGINE_HIP && dtype != THHIP_F32 && !dag; i++) {
		if (!is_conv_type(hn->pub.modules[i].type) || hn->hm[i].is_linear || hn->hm[i].in_cl || !hn->hm[i].out_cl || hn->hm[i].pool_next)
			continue;
		const struct SpatialConvolution *a = &hn->pub.modules[i].SpatialConvolution;
		if (a->nInputPlane != 3 || a->nOutputPlane != 64 || a->kW != 3 || a->kH != 3 || a->dW != 1 || a->dH != 1 || a->padW != 1 || a->padH != 1)
			continue;
		int j = i + 1;
		while (j < net->nelem && hn->hm[j].passthrough)
			j++;
		if (j >= net->nelem || !is_conv_type(hn->pub.modules[j].type) || hn->hm[j].is_linear || !hn->hm[j].in_cl || !hn->hm[j].out_cl)
			continue;
		const struct SpatialConvolution *b = &hn->pub.modules[j].SpatialConvolution;
		if (b->nInputPlane != 64 || b->nOutputPlane > 256 || b->nOutputPlane % 8 || b->kW != 3 || b->kH != 3 || b->dW != 1 || b->dH != 1 ||
		    b->padW != 1 || b->padH != 1)
			continue;
		const THFloatTensor *w = net->modules[i].SpatialConvolution.weight;
		if (!w || !w->storage || THFloatTensor_nElement((THFloatTensor *)w) != 64 * 27)
			continue;
		hn->hm[i].wfront = thhip_conv_pack_weight_image_front(w->storage->data + w->storageOffset, dtype);
		hn->hm[i].front_of = j;
		hn->hm[j].front = i + 1;
	}
#undef FEEDS_ONLY
	free(consumers);
	/* uint8 engine: the image layer (at most four planes, plane-major), or a convolution between
	 * channels-last tensors, followed by its folded Threshold and a 3x3 / stride 2 max pooling
	 * may run as one kernel; whether it does is decided per forward by the layer's shape */
	for (int i = 0; i + 1 < net->nelem && engine == ENGINE_HIPLOWP; i++) {
		if (!is_conv_type(hn->pub.modules[i].type) || hn->hm[i].is_linear || !hn->hm[i].out_cl ||
		    (!hn->hm[i].in_cl && hn->pub.modules[i].SpatialConvolution.nInputPlane > 4))
			continue;
		int j = i + 1;
		while (j < net->nelem && hn->hm[j].passthrough)
			j++;
		if (j >= net->nelem || hn->pub.modules[j].type != MT_SpatialMaxPooling)
			continue;
		const struct SpatialMaxPooling *q = &hn->pub.modules[j].SpatialMaxPooling;
		if (q->kW == 3 && q->kH == 3 && q->dW == 2 && q->dH == 2 && q->padW == 0 && q->padH == 0 && !q->ceil_mode)
			hn->hm[i].pool_next = j;
	}
	/* fp32 residual blocks in table form, ConcatTable{main, shortcut} -> CAddTable (-> Threshold(0, 0)):
	 * the add (and the Threshold folded into it) may be done by the epilogue of the convolution that
	 * runs last in the table: the main branch's last one when the shortcut is the identity, else the
	 * shortcut's (branch 0 has run by then).  Whether it is, is decided per forward by the layer's
	 * shape; the table add then passes that convolution's tensor on. */
	for (int i = 0; i + 1 < net->nelem && engine == ENGINE_HIP && dtype == THHIP_F32 && !hn->dag; i++) {
		struct module *ct = &hn->pub.modules[i], *add = &hn->pub.modules[i + 1];
		if (ct->type != MT_ConcatTable || !ct->ConcatTable.net || ct->ConcatTable.net->nelem != 2 ||
		    (add->type != MT_CAddTable && add->type != MT_CSubTable))
			continue;
		struct module *b0 = &ct->ConcatTable.net->modules[0], *b1 = &ct->ConcatTable.net->modules[1];
		const int identity = b1->type == MT_Dropout || b1->type == MT_Identity;
		/* A shortcut that is one convolution (with its folded batch norm) beside a main branch of several
		 * modules that starts with a convolution: both read the table's input, so the shortcut runs first
		 * and shares a launch with that convolution (thhip_conv_pair_begin: ResNet-18 batch 32, the three
		 * blocks with a projection: 65 -> 57, 60 -> 56, 64 -> 61 us for the pair), and the main branch's last
		 * convolution does the add. */
		int shortcut_first = 0;
		if (!identity && b0->type == MT_Sequential && b0->Sequential.net && b0->Sequential.net->nelem > 1 &&
		    is_conv_type(b0->Sequential.net->modules[0].type) && !((struct hipnet *)b0->Sequential.net)->dag) {
			struct module *c0 = branch_last_conv(b0), *c1 = branch_last_conv(b1);
			struct module *f1 = b1->type == MT_Sequential && b1->Sequential.net && b1->Sequential.net->nelem > 0 ?
				&b1->Sequential.net->modules[0] : b1;
			shortcut_first = c0 && c1 && c1 == f1 && c0 != &b0->Sequential.net->modules[0];
		}
		struct module *conv = branch_last_conv(identity || shortcut_first ? b0 : b1);
		if (!conv)
			continue;
		struct hipmod *chm = hipmod_of(conv);
		chm->res_mode = identity || shortcut_first ? 1 : 2;
		/* the arithmetic as shipped (CAddTable.c:59-70: the two-input CAddTable subtracts), or as named */
		chm->res_c = (add->type == MT_CSubTable) != (hn->hm[i + 1].table_named != 0) ? 1.0f : -1.0f;
		chm->res_act = hn->hm[i + 1].fused_act;
		chm->res_add = &hn->hm[i + 1];
		hn->hm[i].res_target = chm;
		hn->hm[i].res_from_input = identity;
		hn->hm[i].shortcut_first = shortcut_first;
	}
	return &hn->pub;
}

struct network *THHip_ToHip(struct network *net, int lowp, float range)
{
	if (thhip_device_count() < 1)
		THError("thnets HIP engine: no AMD GPU visible; this library has no CPU fallback");
	if (lowp && !(range > 0))
		THError("THCreateHipLowpNetwork: range must be positive");
	return to_hip(net, lowp ? ENGINE_HIPLOWP : ENGINE_HIP, lowp ? THHIP_U8 : thhip_engine_dtype(), lowp ? range : 1);
}

void thhip_free_network(struct network *net)
{
	struct hipnet *hn = (struct hipnet *)net;
	for (int i = 0; i < net->nelem; i++) {
		struct module *m = &net->modules[i];
		struct hipmod *hm = &hn->hm[i];
		if (m->type == MT_Sequential && m->Sequential.net)
			thhip_free_network(m->Sequential.net);
		else if (m->type == MT_ConcatTable && m->ConcatTable.net)
			thhip_free_network(m->ConcatTable.net);
		THFloatTensor_free(m->output);
		thhip_free(hm->wpacked);
		thhip_free(hm->wrow);
		thhip_free(hm->wfront);
		thhip_free(hm->bias);
		thhip_free(hm->scale);
		thhip_free(hm->addend);
		thhip_free(hm->wrow_u8);
		thhip_free(hm->wpatch_u8);
		thhip_free(hm->rowsum_u8);
		thhip_free(hm->col);
		thhip_free(hm->pool_ind);
		for (int j = 0; j < 4; j++)
			thhip_free(hm->bn[j]);
	}
	thhip_io_free(hn);
	free(hn->hm);
	free(net->modules);
	free(hn);
}
