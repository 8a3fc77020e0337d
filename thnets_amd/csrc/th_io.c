/*
 * Data in and out of the engine: device <-> host tensors (the CUDA analogues are
 * cudnn_basic.c:64-97) and the ENGINE_HIP / ENGINE_HIPLOWP bodies of THProcessFloat
 * and THProcessImages (thapi.c:363-450, 452-563).  This file and th_engine.c are the
 * host objects a thnets tree links when it takes the engine in (the rest of the host
 * side there is thnets' own thbasic.c / thapi.c); the stand-alone library adds
 * th_tensor.c, th_api.c and th_load.c.
 *
 * A network keeps its staging memory between calls (struct hipio): the device copy of
 * the input, the page-locked host buffers the input and the result pass through, the
 * float copy of a half or uint8 result.  A call of the same shape allocates nothing.
 */
#include <stdlib.h>
#include <string.h>
#include "th_engine.h"

void thhip_storage_release(THFloatStorage *s)
{
	if (__sync_sub_and_fetch(&s->nref, 1) > 0)
		return;
	if (TH_IS_HIP_STORAGE(s->mustfree))
		thhip_free(s->data);
	else if (s->mustfree)
		free(s->data);
	free(s);
}

static size_t esize_of(int dtype)
{
	return dtype == THHIP_F32 ? 4 : dtype == THHIP_U8 ? 1 : 2;
}

static void set_contiguous(THFloatTensor *t, int nd, const long *size)
{
	long stride = 1;
	t->nDimension = nd;
	for (int i = nd - 1; i >= 0; i--) {
		t->size[i] = size[i];
		t->stride[i] = stride;
		stride *= size[i];
	}
}

/* cudnn_basic.c:64-80 is the CUDA analogue: same shape, contiguous device
 * tensor in the given element type. */
THFloatTensor *thhip_device_tensor_like(THFloatTensor *t, int dtype)
{
	THFloatTensor *n = malloc(sizeof(*n));
	memcpy(n, t, sizeof(*n));
	n->storage = 0;
	n->storageOffset = 0;
	if (t->storage) {
		set_contiguous(n, t->nDimension, t->size);
		n->storage = malloc(sizeof(*n->storage));
		n->storage->nref = 1;
		n->storage->mustfree = TH_MUSTFREE_HIP_OF(dtype);
		n->storage->data = thhip_malloc((size_t)THFloatTensor_nElement(t) * esize_of(dtype));
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

THFloatTensor *thhip_upload_as(THFloatTensor *t, int dtype)
{
	THFloatTensor *n = thhip_device_tensor_like(t, dtype);
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
	return thhip_upload_as(t, thhip_engine_dtype());
}

THFloatTensor *thhip_download_as_float(THFloatTensor *t, int dtype)
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
	return thhip_download_as_float(t, thhip_engine_dtype());
}

/* ------------------------------------------------------------------ */
/* staging memory kept with the network                                */
/* ------------------------------------------------------------------ */

/* A device tensor of the staging area with room for `bytes`.  The storage is
 * replaced, not resized, when it has to grow: a module of the last forward may
 * still hold a view of the old one (in-place modules alias their input). */
static THFloatTensor *io_device_tensor(struct hipio_buf *b, size_t bytes, int dtype)
{
	if (!b->t)
		b->t = THFloatTensor_new();
	THFloatTensor *t = b->t;
	if (!t->storage || b->cap < bytes) {
		THFloatStorage *s = malloc(sizeof(*s));
		s->data = thhip_malloc(bytes);
		s->nref = 1;
		if (t->storage)
			thhip_storage_release(t->storage);
		t->storage = s;
		b->cap = bytes;
	}
	t->storage->mustfree = TH_MUSTFREE_HIP_OF(dtype);
	t->storageOffset = 0;
	return t;
}

static void *io_pinned(struct hipio_pin *p, size_t bytes)
{
	if (p->cap < bytes) {
		thhip_host_free(p->ptr);
		p->ptr = thhip_host_malloc(bytes);
		p->cap = bytes;
	}
	return p->ptr;
}

void thhip_io_free(struct hipnet *hn)
{
	struct hipio *io = &hn->io;
	struct hipio_buf *bufs[] = { &io->in_raw, &io->in_dev, &io->in_q, &io->out_f, &io->img };
	for (unsigned i = 0; i < sizeof(bufs) / sizeof(bufs[0]); i++)
		if (bufs[i]->t)
			THFloatTensor_free(bufs[i]->t);
	thhip_host_free(io->pin_in.ptr);
	thhip_host_free(io->pin_out.ptr);
	memset(io, 0, sizeof(*io));
}

/* Host memory -> device through the page-locked buffer, in pieces: the host copy
 * of piece i + 1 runs while piece i crosses the link.  When the call returns the
 * caller's memory has been read (the device copy is still on its way). */
/* (the host copy is memory-bound: one thread moves a fresh 9.6 MB batch in 0.3 ms, the
 * link takes 0.18 ms) */
static void copy_to_pinned(char *dst, const char *src, size_t bytes)
{
	const size_t blk = (size_t)128 << 10;
	const long nblk = (long)((bytes + blk - 1) / blk);
#pragma omp parallel for schedule(static) if (bytes >= ((size_t)1 << 19))
	for (long i = 0; i < nblk; i++) {
		const size_t at = (size_t)i * blk;
		memcpy(dst + at, src + at, bytes - at < blk ? bytes - at : blk);
	}
}

#define IO_MIN_PIECE ((size_t)1 << 20)
#define IO_MAX_PIECES 4
static void io_upload(struct hipnet *hn, void *dst, const void *src, size_t bytes, size_t pin_offset)
{
	char *pin = (char *)hn->io.pin_in.ptr + pin_offset;
	size_t piece = (bytes + IO_MAX_PIECES - 1) / IO_MAX_PIECES;
	if (piece < IO_MIN_PIECE)
		piece = IO_MIN_PIECE;
	piece = (piece + 255) & ~(size_t)255;
	for (size_t at = 0; at < bytes; at += piece) {
		const size_t n = bytes - at < piece ? bytes - at : piece;
		copy_to_pinned(pin + at, (const char *)src + at, n);
		thhip_memcpy_h2d_async((char *)dst + at, pin + at, n);
	}
}

/* The result of the forward pass as floats in network->out, whose storage is the
 * network's page-locked result buffer (library-owned, like the `out` tensor of
 * the reference's GPU engines, thapi.c:411-414; valid until the next call). */
static THFloatTensor *io_download_result(THNETWORK *network, THFloatTensor *out, int dtype, int dequantize)
{
	struct hipnet *hn = (struct hipnet *)network->net;
	const long cnt = THFloatTensor_nElement(out);
	const void *src = thhip_tensor_ptr(out, dtype);
	if (dtype != THHIP_F32) {
		THFloatTensor *f = io_device_tensor(&hn->io.out_f, sizeof(float) * (size_t)cnt, THHIP_F32);
		if (dequantize)		/* THFloatTensor_newFromLowpTensor, lowp_basic.c:40-58 */
			thhip_dequantize(src, f->storage->data, cnt, hn->cur_mult, hn->cur_sub);
		else
			thhip_convert(src, dtype, f->storage->data, THHIP_F32, cnt);
		src = f->storage->data;
	}
	float *host = io_pinned(&hn->io.pin_out, sizeof(float) * (size_t)cnt);
	thhip_memcpy_d2h_async(host, src, sizeof(float) * (size_t)cnt);
	THFloatTensor *o = network->out;
	if (!o || !o->storage || o->storage->mustfree != 0 || o->storage->nref != 1) {
		if (o)
			THFloatTensor_free(o);
		o = network->out = THFloatTensor_new();
		o->storage = malloc(sizeof(*o->storage));
		o->storage->nref = 1;
		o->storage->mustfree = 0;	/* the buffer belongs to the network's staging area */
	}
	o->storage->data = host;
	o->storageOffset = 0;
	set_contiguous(o, out->nDimension, out->size);
	thhip_sync();
	return o;
}

/* The caller's buffer as THProcessFloat leaves it: planes 0..2 normalised in
 * place (thapi.c:389-403).  mean / std hold three planes: further planes are left
 * untouched here (the reference reads past the arrays for them). */
static void normalize_on_host(float *data, int batchsize, int nplanes, long hw, const float *mean3, const float *std3)
{
	const int np3 = nplanes < 3 ? nplanes : 3;
	/* IEEE subtraction and division element by element: the compiler's vector forms and
	 * any split over threads give the bits of the reference's scalar loop */
#pragma omp parallel for collapse(2) if ((long)batchsize * np3 * hw >= (1L << 20))
	for (int b = 0; b < batchsize; b++)
		for (int c = 0; c < np3; c++) {
			float *restrict p = data + ((long)b * nplanes + c) * hw;
			const float mean = mean3[c], std = std3[c];
#pragma omp simd
			for (long i = 0; i < hw; i++)
				p[i] = (p[i] - mean) / std;
		}
}

/* Runs a device tensor (codes with hn->cur_mult / cur_sub for the uint8 engine,
 * the engine's float type otherwise) and leaves the float result in network->out. */
static THFloatTensor *run_and_download(THNETWORK *network, THFloatTensor *dev_in)
{
	struct hipnet *hn = (struct hipnet *)network->net;
	const int lowp = network->net->engine == ENGINE_HIPLOWP;
	/* A kernel may report that it ran where its results cannot be trusted (hip_rt.hip: thhip_fault_flag;
	 * the path that depends on it is switched off by the report): the input is still on the device, so the
	 * forward pass is simply run once more. */
	thhip_fault_hold(1);
	THFloatTensor *out = thhip_forward(network->net, dev_in);
	THFloatTensor *res = io_download_result(network, out, lowp ? THHIP_U8 : hn->dtype, lowp);
	thhip_fault_hold(0);
	if (thhip_fault_take()) {
		out = thhip_forward(network->net, dev_in);
		res = io_download_result(network, out, lowp ? THHIP_U8 : hn->dtype, lowp);
	}
	return res;
}

/* A batch uploaded in pieces, the first modules of the network at work on one piece while the next
 * crosses the link (thhip_forward_windows): what thhip_process_float hands to the engine per window. */
struct io_windows {
	struct hipnet *hn;
	THNETWORK *network;
	const float *data;	/* the caller's batch */
	float *raw;		/* its copy on the device, un-normalised */
	void *dev;		/* normalised, in the engine's type (raw itself for fp32) */
	int dt, nplanes;
	long hw;
	int b0[8], bn[8];
};

static void io_window_ready(void *ctx, int w)
{
	struct io_windows *iw = ctx;
	const size_t img = (size_t)iw->nplanes * iw->hw, at = img * iw->b0[w], bytes = sizeof(float) * img * iw->bn[w];
	char *pin = (char *)iw->hn->io.pin_in.ptr + sizeof(float) * at;
	copy_to_pinned(pin, (const char *)(iw->data + at), bytes);
	thhip_memcpy_h2d_piece(iw->raw + at, pin, bytes, w);
	thhip_wait_h2d_piece(w);
	thhip_normalize(iw->raw + at, (char *)iw->dev + esize_of(iw->dt) * at, iw->bn[w], iw->nplanes, iw->hw,
		iw->network->mean, iw->network->std, iw->dt);
}

/* The engine's body of THProcessFloat (thapi.c:363-450): `data` is [batchsize][nplanes]
 * [height][width] floats, not yet normalised.  The reference normalises the caller's
 * buffer in place before any engine sees it (thapi.c:389-403), and callers observe
 * that.  Here the raw data goes to the device first, a kernel applies the same
 * arithmetic there (same bits: fp32 subtraction, correctly rounded division), the
 * forward pass is queued, and the host loop over the caller's buffer runs while the
 * GPU works.  Returns network->out. */
THFloatTensor *thhip_process_float(THNETWORK *network, float *data, int batchsize, int width, int height, int nplanes)
{
	struct hipnet *hn = (struct hipnet *)network->net;
	const int lowp = network->net->engine == ENGINE_HIPLOWP;
	const long hw = (long)width * height, cnt = hw * nplanes * batchsize;
	const long size[4] = { batchsize, nplanes, height, width };
	const int dt = lowp ? THHIP_F32 : hn->dtype;
	THFloatTensor *raw = io_device_tensor(&hn->io.in_raw, sizeof(float) * (size_t)cnt, THHIP_F32);
	io_pinned(&hn->io.pin_in, sizeof(float) * (size_t)cnt);
	THFloatTensor *dev = dt == THHIP_F32 ? raw : io_device_tensor(&hn->io.in_dev, esize_of(dt) * (size_t)cnt, dt);
	set_contiguous(dev, 4, size);
	/* a batch of eight images and 4 MiB or more on a float engine: in pieces, the network's first
	 * modules at work on one while the next is uploaded */
	if (!lowp && batchsize >= 8 && sizeof(float) * (size_t)cnt >= ((size_t)4 << 20) && !hn->no_windows) {
		struct io_windows iw = { hn, network, data, (float *)raw->storage->data, dev->storage->data, dt, nplanes, hw };
		/* three windows, a quarter and twice three eighths of the batch: the first upload, which nothing
		 * hides, is the short one (VGG-16 at batch 16, per-call overhead over the bare forward pass:
		 * one piece 0.30-0.32 ms, two halves 0.23-0.26, these three 0.18-0.20, four 0.19-0.24) */
		const int nw = 3;
		static const int sixteenths[4] = { 0, 4, 10, 16 };
		for (int w = 0; w < nw; w++) {
			iw.b0[w] = (int)((long)batchsize * sixteenths[w] / 16);
			iw.bn[w] = (int)((long)batchsize * sixteenths[w + 1] / 16) - iw.b0[w];
		}
		thhip_fault_hold(1);	/* (as in run_and_download) */
		THFloatTensor *out = thhip_forward_windows(network->net, dev, nw, iw.b0, iw.bn, io_window_ready, &iw);
		normalize_on_host(data, batchsize, nplanes, hw, network->mean, network->std);
		THFloatTensor *res = io_download_result(network, out, hn->dtype, 0);
		thhip_fault_hold(0);
		if (thhip_fault_take()) {
			out = thhip_forward(network->net, dev);
			res = io_download_result(network, out, hn->dtype, 0);
		}
		return res;
	}
	io_upload(hn, raw->storage->data, data, sizeof(float) * (size_t)cnt, 0);
	thhip_normalize(raw->storage->data, dev->storage->data, batchsize, nplanes, hw, network->mean, network->std, dt);
	THFloatTensor *in = dev;
	if (lowp) {
		/* THLowpTensor_newFromFloatTensor on the whole batch (one min / max),
		 * lowp_basic.c:15-35; waits for the device: (mult, sub) come back */
		in = io_device_tensor(&hn->io.in_q, (size_t)cnt, THHIP_U8);
		set_contiguous(in, 4, size);
		thhip_quantize((const float *)dev->storage->data, (unsigned char *)in->storage->data, cnt,
			&hn->cur_mult, &hn->cur_sub);
	}
	thhip_fault_hold(1);	/* (as in run_and_download) */
	THFloatTensor *out = thhip_forward(network->net, in);
	normalize_on_host(data, batchsize, nplanes, hw, network->mean, network->std);
	THFloatTensor *res = io_download_result(network, out, lowp ? THHIP_U8 : hn->dtype, lowp);
	thhip_fault_hold(0);
	if (thhip_fault_take()) {
		out = thhip_forward(network->net, in);
		res = io_download_result(network, out, lowp ? THHIP_U8 : hn->dtype, lowp);
	}
	return res;
}

/* The engine's body of THProcessImages (thapi.c:452-563): interleaved 8-bit images
 * -> normalised planes (rgb2float / bgr2float, thapi.c:20-46) or, for the uint8
 * engine, codes in the fixed range Lowp_LoadImages derives from mean / std
 * (lowp_basic.c:60-131), on the device: every image crosses the link as the bytes
 * the caller holds, nothing waits until the result is fetched.  Returns network->out. */
THFloatTensor *thhip_process_images(THNETWORK *network, unsigned char **images, int batchsize, int width, int height,
	int stride, int bgr)
{
	struct hipnet *hn = (struct hipnet *)network->net;
	const int lowp = network->net->engine == ENGINE_HIPLOWP;
	int cp = 3;
	if (stride < width * 3)
		cp = 1;	/* thapi.c:458-459 */
	/* Lowp_LoadImages reads three bytes per pixel whatever the stride: with stride <
	 * 3 * width (one plane for the float engines) the reference reads past the image;
	 * here that would be a device read past the staging copy, so it is refused. */
	if (lowp && cp != 3)
		THError("THProcessImages: the uint8 engine takes three-plane images only (stride %d < 3 * width %d)",
			stride, width);
	const int dt = lowp ? THHIP_U8 : hn->dtype;
	const size_t ibytes = (size_t)stride * height, obytes = (size_t)cp * width * height * esize_of(dt);
	const size_t islot = (ibytes + 255) & ~(size_t)255;
	THFloatTensor *img = io_device_tensor(&hn->io.img, islot * batchsize, THHIP_U8);
	THFloatTensor *t = io_device_tensor(lowp ? &hn->io.in_q : &hn->io.in_dev, obytes * batchsize, dt);
	/* the images side by side in the page-locked buffer, over the link in a few large
	 * pieces, then one launch for all of them */
	unsigned char *pin = io_pinned(&hn->io.pin_in, islot * batchsize);
	unsigned char *dimg = (unsigned char *)img->storage->data;
	const int group = batchsize < 8 ? 1 : (batchsize + 7) / 8;
	for (int i = 0; i < batchsize; i += group) {
		const int n = batchsize - i < group ? batchsize - i : group;
#pragma omp parallel for schedule(static) if (ibytes * n >= ((size_t)1 << 19))
		for (int j = i; j < i + n; j++)
			memcpy(pin + islot * j, images[j], ibytes);
		thhip_memcpy_h2d_async(dimg + islot * i, pin + islot * i, islot * n);
	}
	if (lowp)
		thhip_rgb2code_batch((unsigned char *)t->storage->data, dimg, batchsize, (long)islot, width, height, stride,
			network->mean, network->std, bgr, &hn->cur_mult, &hn->cur_sub);
	else
		thhip_rgb2float_batch(t->storage->data, dimg, batchsize, (long)islot, width, height, stride, cp,
			network->mean, network->std, bgr, dt);
	if (batchsize == 1 && !lowp) {	/* thapi.c:497-516; the uint8 loader is always 4-D (thapi.c:485-487) */
		const long s[3] = { cp, height, width };
		set_contiguous(t, 3, s);
	} else {
		const long s[4] = { batchsize, cp, height, width };
		set_contiguous(t, 4, s);
	}
	return run_and_download(network, t);
}
