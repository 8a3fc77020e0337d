/*
 * The small HBM-bound kernels that keep activations on the device between
 * the GEMM-shaped modules: Threshold, max / average pooling, SoftMax, batch
 * normalisation, the two-input table add, dtype conversion, 8-bit image
 * loading, and the uint8 (LOWP) counterparts.  Each one reads its input once
 * and writes its output once; lanes run along the innermost (W) dimension.
 */
#include <float.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include "thhip_internal.h"

#define EW_THREADS 256

/* Several of these kernels are held to bit-exact parity with a CPU evaluation
 * that rounds after every operation, so nothing in this file may be fused
 * into a multiply-add. */
#pragma clang fp contract(off)

static inline dim3 ew_grid(long n, int per_thread = 1)
{
	long blocks = (n + (long)EW_THREADS * per_thread - 1) / ((long)EW_THREADS * per_thread);
	if (blocks < 1)
		blocks = 1;
	if (blocks > 65536 * 16)
		blocks = 65536 * 16;
	return dim3((unsigned)blocks);
}

/* ---------------- Threshold (modules/Threshold.c:38-63) ---------------- */

template <int DT>
__global__ void threshold_kernel(const void *x, void *y, long n, float thr, float val, float alpha, int mode)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < n; i += step) {
		const float v = ThhipElem<DT>::ld(x, i);
		float r;
		if (mode == 0)		/* in place: x <= thr -> val */
			r = v <= thr ? val : v;
		else if (mode == 1)	/* out of place, alpha != 0 */
			r = v >= 0 ? v : v * alpha;
		else			/* out of place */
			r = v > thr ? v : val;
		ThhipElem<DT>::st(y, i, r);
	}
}

extern "C" void thhip_threshold(const void *x, void *y, long n, float thr, float val, float alpha, int inplace, int dtype)
{
	if (n <= 0)
		return;
	const int mode = inplace ? 0 : (alpha != 0 ? 1 : 2);
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * n * thhip_esize(dtype));
	THHIP_DISPATCH_FLOAT(dtype, (threshold_kernel<DT><<<ew_grid(n, 4), dim3(EW_THREADS), 0, thhip_stream()>>>(
		x, y, n, thr, val, alpha, mode)));
}

__global__ void threshold_u8_kernel(const unsigned char *x, unsigned char *y, long n, int thr, int val, int inplace)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < n; i += step) {
		const int v = x[i];
		/* lowp_Threshold.c:14-24: the two branches differ only in how they are
		 * written; both give v > thr ? v : val */
		y[i] = (unsigned char)((inplace ? !(v <= thr) : (v > thr)) ? v : val);
	}
}

extern "C" void thhip_threshold_u8(const unsigned char *x, unsigned char *y, long n, int thr, int val, int inplace)
{
	if (n <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * n);
	threshold_u8_kernel<<<ew_grid(n, 8), dim3(EW_THREADS), 0, thhip_stream()>>>(x, y, n, thr, val, inplace);
}

/* ---------------- pooling ---------------- */

/* Output extent: modules/SpatialMaxPooling.c:187-203 (float division, floor
 * or ceil, drop a last window starting beyond the padded input). */
extern "C" void thhip_pool_outsize(int H, int W, int kH, int kW, int dH, int dW, int padH, int padW, int ceil_mode,
	int *oH, int *oW)
{
	long oh, ow;
	if (ceil_mode) {
		oh = (long)(ceilf((float)(H - kH + 2 * padH) / dH)) + 1;
		ow = (long)(ceilf((float)(W - kW + 2 * padW) / dW)) + 1;
	} else {
		oh = (long)(floorf((float)(H - kH + 2 * padH) / dH)) + 1;
		ow = (long)(floorf((float)(W - kW + 2 * padW) / dW)) + 1;
	}
	if (padW || padH) {
		if ((oh - 1) * dH >= H + padH)
			--oh;
		if ((ow - 1) * dW >= W + padW)
			--ow;
	}
	*oH = (int)oh;
	*oW = (int)ow;
}

struct PoolParams {
	int C, H, W, oH, oW, kH, kW, dH, dW, padH, padW;
	long total;
};

template <int DT>
__global__ void maxpool_kernel(const void *x, void *y, PoolParams p)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int ox = (int)(i % p.oW);
		const long t = i / p.oW;
		const int oy = (int)(t % p.oH);
		const long plane = t / p.oH;
		int hs = oy * p.dH - p.padH, ws = ox * p.dW - p.padW;
		const int he = min(hs + p.kH, p.H), we = min(ws + p.kW, p.W);
		hs = max(hs, 0);
		ws = max(ws, 0);
		const long base = plane * p.H * p.W;
		if constexpr (DT == THHIP_U8) {
			int m = 0;	/* lowp_SpatialMaxPooling.c:28 */
			for (int yy = hs; yy < he; yy++)
				for (int xx = ws; xx < we; xx++)
					m = max(m, (int)((const unsigned char *)x)[base + (long)yy * p.W + xx]);
			((unsigned char *)y)[i] = (unsigned char)m;
		} else {
			float m = -FLT_MAX;	/* SpatialMaxPooling.c:96 */
			for (int yy = hs; yy < he; yy++)
				for (int xx = ws; xx < we; xx++) {
					const float v = ThhipElem<DT>::ld(x, base + (long)yy * p.W + xx);
					if (v > m)
						m = v;
				}
			ThhipElem<DT>::st(y, i, m);
		}
	}
}

/* The common 2x2 / stride 2 / no padding pooling of fp32 planes whose width is a
 * multiple of four: a thread reads four columns of two rows as two 16-byte
 * vectors and writes two outputs.  Same comparisons in the same order as the
 * general kernel. */
__global__ void maxpool_f32_2x2_kernel(const floatx4 *x, float2 *y, int H4, int oH, int oW2, long total2)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total2; i += step) {
		const int xq = (int)(i % oW2);
		const long t = i / oW2;
		const int oy = (int)(t % oH);
		const long plane = t / oH;
		const floatx4 *row = x + (plane * H4 * 2 + (long)oy * 2) * oW2 + xq;	/* W/4 == oW/2 vectors per row */
		const floatx4 a = row[0], b = row[oW2];
		float2 o;
		float m = -FLT_MAX;
		m = a[0] > m ? a[0] : m;
		m = a[1] > m ? a[1] : m;
		m = b[0] > m ? b[0] : m;
		m = b[1] > m ? b[1] : m;
		o.x = m;
		m = -FLT_MAX;
		m = a[2] > m ? a[2] : m;
		m = a[3] > m ? a[3] : m;
		m = b[2] > m ? b[2] : m;
		m = b[3] > m ? b[3] : m;
		o.y = m;
		y[i] = o;
	}
}

/* The 3x3 / stride 2 / padding 1 pooling of fp32 planes whose width is a
 * multiple of eight (ResNet's stem): a thread makes four neighbouring outputs
 * of a row from the nine columns they read, fetched per input row as one
 * scalar and two 16-byte vectors.  Same comparisons in the same order as the
 * general kernel (what lies outside the plane is never the maximum). */
__global__ void maxpool_f32_3x3s2p1_kernel(const float *x, floatx4 *y, int H, int W, int oH, int oW4, long total4)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total4; i += step) {
		const int xq = (int)(i % oW4);
		const long t = i / oW4;
		const int oy = (int)(t % oH);
		const long plane = t / oH;
		const float *px = x + plane * H * W + 8 * xq;
		floatx4 m = { -FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX };
#pragma unroll
		for (int r = 0; r < 3; r++) {
			const int yy = 2 * oy - 1 + r;
			if (yy < 0 || yy >= H)
				continue;
			const float *row = px + (long)yy * W;
			float v[9];
			v[0] = xq ? row[-1] : -FLT_MAX;
			const floatx4 a = *(const floatx4 *)row, b = *(const floatx4 *)(row + 4);
#pragma unroll
			for (int e = 0; e < 4; e++) {
				v[1 + e] = a[e];
				v[5 + e] = b[e];
			}
#pragma unroll
			for (int o = 0; o < 4; o++)
#pragma unroll
				for (int c = 0; c < 3; c++)
					m[o] = v[2 * o + c] > m[o] ? v[2 * o + c] : m[o];
		}
		y[i] = m;
	}
}

extern "C" void thhip_maxpool(const void *x, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype)
{
	PoolParams p = { C, H, W, oH, oW, kH, kW, dH, dW, padH, padW, (long)B * C * oH * oW };
	if (p.total <= 0)
		return;
	const double esz = thhip_esize(dtype);
	ThhipLaunchScope scope(THHIP_FAM_OTHER, esz * ((double)B * C * H * W + (double)p.total));
	if (dtype == THHIP_F32 && kH == 2 && kW == 2 && dH == 2 && dW == 2 && padH == 0 && padW == 0 && W % 4 == 0 &&
	    H % 2 == 0 && oH == H / 2 && oW == W / 2 && ((size_t)x & 15) == 0 && ((size_t)y & 7) == 0) {
		const long total2 = p.total / 2;
		maxpool_f32_2x2_kernel<<<ew_grid(total2), dim3(EW_THREADS), 0, thhip_stream()>>>((const floatx4 *)x, (float2 *)y,
			H / 2, oH, oW / 2, total2);
		return;
	}
	if (dtype == THHIP_F32 && kH == 3 && kW == 3 && dH == 2 && dW == 2 && padH == 1 && padW == 1 && W % 8 == 0 &&
	    oW == W / 2 && oH == (H - 1) / 2 + 1 && ((size_t)x & 15) == 0 && ((size_t)y & 15) == 0) {
		const long total4 = p.total / 4;
		maxpool_f32_3x3s2p1_kernel<<<ew_grid(total4), dim3(EW_THREADS), 0, thhip_stream()>>>((const float *)x, (floatx4 *)y,
			H, W, oH, oW / 4, total4);
		return;
	}
	const dim3 grid = ew_grid(p.total);
	switch (dtype) {
	case THHIP_F32: maxpool_kernel<THHIP_F32><<<grid, dim3(EW_THREADS), 0, thhip_stream()>>>(x, y, p); break;
	case THHIP_F16: maxpool_kernel<THHIP_F16><<<grid, dim3(EW_THREADS), 0, thhip_stream()>>>(x, y, p); break;
	case THHIP_BF16: maxpool_kernel<THHIP_BF16><<<grid, dim3(EW_THREADS), 0, thhip_stream()>>>(x, y, p); break;
	case THHIP_U8: maxpool_kernel<THHIP_U8><<<grid, dim3(EW_THREADS), 0, thhip_stream()>>>(x, y, p); break;
	default: THError("thhip_maxpool: unsupported dtype %d", dtype);
	}
}

/* Max pooling that also records where each maximum was found, for
 * SpatialMaxUnpooling: the reference keeps float `indices` (position in the
 * input plane + 1, SpatialMaxPooling.c:100-114); here an int per output
 * element, the position itself, -1 for an empty window.  First maximum wins. */
template <int DT>
__global__ void maxpool_indices_kernel(const void *x, void *y, int *ind, PoolParams p)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int ox = (int)(i % p.oW);
		const long t = i / p.oW;
		const int oy = (int)(t % p.oH);
		const long plane = t / p.oH;
		int hs = oy * p.dH - p.padH, ws = ox * p.dW - p.padW;
		const int he = min(hs + p.kH, p.H), we = min(ws + p.kW, p.W);
		hs = max(hs, 0);
		ws = max(ws, 0);
		const long base = plane * p.H * p.W;
		float m = -INFINITY;	/* SpatialMaxPooling.c:100 */
		int at = -1;
		for (int yy = hs; yy < he; yy++)
			for (int xx = ws; xx < we; xx++) {
				const float v = ThhipElem<DT>::ld(x, base + (long)yy * p.W + xx);
				if (v > m) {
					m = v;
					at = yy * p.W + xx;
				}
			}
		ThhipElem<DT>::st(y, i, m);
		ind[i] = at;
	}
}

extern "C" void thhip_maxpool_indices(const void *x, void *y, int *ind, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype)
{
	PoolParams p = { C, H, W, oH, oW, kH, kW, dH, dW, padH, padW, (long)B * C * oH * oW };
	if (p.total <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, thhip_esize(dtype) * ((double)B * C * H * W + (double)p.total) + 4.0 * p.total);
	THHIP_DISPATCH_FLOAT(dtype, (maxpool_indices_kernel<DT><<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>(x, y, ind, p)));
}

/* nn_SpatialMaxUnpooling_updateOutput (SpatialMaxUnpooling.c:14-41, 92-119)
 * as a gather, so that no two threads write one element: the reference zeroes
 * the output plane and then writes every input element at its index in
 * row-major order, the last writer staying.  An output element therefore holds
 * the input of the last pooling window (row-major) whose maximum sat there;
 * only the windows that contain the element can name it.  p describes the
 * pooling: H x W its input (this output), oH x oW its output (this input). */
template <int DT>
__global__ void maxunpool_kernel(const void *x, const int *ind, void *y, PoolParams p)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int px = (int)(i % p.W);
		const long t = i / p.W;
		const int py = (int)(t % p.H);
		const long plane = t / p.H;
		const int at = py * p.W + px;
		/* windows row r covers rows r*dH - padH .. r*dH - padH + kH - 1 */
		const int r1 = min((py + p.padH) / p.dH, p.oH - 1), c1 = min((px + p.padW) / p.dW, p.oW - 1);
		const int r0 = max(0, (py + p.padH - p.kH + p.dH) / p.dH), c0 = max(0, (px + p.padW - p.kW + p.dW) / p.dW);
		const long base = plane * p.oH * p.oW;
		float v = 0;
		bool found = false;
		for (int r = r1; r >= r0 && !found; r--)
			for (int c = c1; c >= c0; c--)
				if (ind[base + (long)r * p.oW + c] == at) {
					v = ThhipElem<DT>::ld(x, base + (long)r * p.oW + c);
					found = true;
					break;
				}
		ThhipElem<DT>::st(y, i, v);
	}
}

extern "C" void thhip_maxunpool(const void *x, const int *ind, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype)
{
	PoolParams p = { C, H, W, oH, oW, kH, kW, dH, dW, padH, padW, (long)B * C * H * W };
	if (p.total <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, thhip_esize(dtype) * ((double)B * C * oH * oW + (double)p.total) + 4.0 * B * C * oH * oW);
	THHIP_DISPATCH_FLOAT(dtype, (maxunpool_kernel<DT><<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>(x, ind, y, p)));
}

/* col2im of nn_SpatialFullConvolution_updateOutput (SpatialFullConvolution.c:104-134)
 * as a gather, with the bias step (:225-237) and an optional threshold fused:
 * columns [B][Co*kH*kW][H*W] (the product of the transposed weights with the
 * input planes) -> y [B][Co][oH][oW],
 *   y = beta * sum_{kh,kw} columns[(o*kH+kh)*kW+kw][iy*W+ix] + bias[o],  oy = iy*dH - padH + kh, ox = ix*dW - padW + kw
 * (no bias: the plain sum).  The taps are added in the reference's order. */
struct Col2imParams {
	int Co, H, W, oH, oW, kH, kW, dH, dW, padH, padW;
	long total;
	float beta;
	int act;
	float thr, val;
};

/* A thread makes the dW neighbouring outputs ox = xb*dW .. xb*dW + dW - 1 of
 * one row: which taps (kh, kw) reach an output depends only on (oy + padH) mod
 * dH and (ox + padW) mod dW, so all lanes of a wave (consecutive xb, one oy)
 * walk the same taps, read consecutive column elements and together write one
 * contiguous stretch of the output row. */
template <int DT>
__global__ void col2im_kernel(const void *col, const float *bias, void *y, Col2imParams p)
{
	const int kHW = p.kH * p.kW;
	const long HW = (long)p.H * p.W;
	const unsigned nxb = (p.oW + p.dW - 1) / p.dW;
	const unsigned groups = (unsigned)p.total;	/* (b, o, oy, xb), fewer than 2^31 */
	const unsigned step = gridDim.x * blockDim.x;
	for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < groups; i += step) {
		const unsigned xb = i % nxb;
		unsigned t = i / nxb;
		const int oy = (int)(t % (unsigned)p.oH);
		t /= (unsigned)p.oH;		/* b * Co + o */
		const int o = (int)(t % (unsigned)p.Co);
		const long cbase = (long)t * kHW * HW;
		const float bo = bias ? bias[o] : 0.0f;
		/* tap kh = ry + n*dH reads row qy - n; the same along x */
		const int qy = (oy + p.padH) / p.dH, ry = oy + p.padH - qy * p.dH;
		for (int rx = 0; rx < p.dW; rx++) {
			const int ox = (int)xb * p.dW + rx;
			if (ox >= p.oW)
				break;
			const int cx = rx + p.padW;	/* the same for every lane */
			const int qx = (int)xb + cx / p.dW, rxx = cx % p.dW;
			float acc = 0;
			for (int n = 0, kh = ry; kh < p.kH && n <= qy; n++, kh += p.dH) {
				const int iy = qy - n;
				if (iy >= p.H)
					continue;
				const long rbase = cbase + (long)kh * p.kW * HW + (long)iy * p.W;
				for (int m = 0, kw = rxx; kw < p.kW && m <= qx; m++, kw += p.dW) {
					const int ix = qx - m;
					if (ix >= p.W)
						continue;
					acc += ThhipElem<DT>::ld(col, rbase + (long)kw * HW + ix);
				}
			}
			float v = bias ? p.beta * acc + bo : acc;
			if (p.act)
				v = v > p.thr ? v : p.val;
			ThhipElem<DT>::st(y, ((long)t * p.oH + oy) * p.oW + ox, v);
		}
	}
}

extern "C" void thhip_col2im(const void *col, const float *bias, float beta, void *y, int B, int Co, int H, int W,
	int kH, int kW, int dH, int dW, int padH, int padW, int adjH, int adjW, int act, float thr, float val, int dtype)
{
	const int oH = (H - 1) * dH - 2 * padH + kH + adjH, oW = (W - 1) * dW - 2 * padW + kW + adjW;
	if (oH < 1 || oW < 1 || dH < 1 || dW < 1)
		THError("thhip_col2im: output %dx%d", oH, oW);
	const long groups = (long)B * Co * oH * ((oW + dW - 1) / dW);
	if (groups >= (1L << 31))
		THError("thhip_col2im: %ld output groups (at most 2^31 - 1)", groups);
	Col2imParams p = { Co, H, W, oH, oW, kH, kW, dH, dW, padH, padW, groups, beta, act, thr, val };
	ThhipLaunchScope scope(THHIP_FAM_OTHER, thhip_esize(dtype) * ((double)B * Co * kH * kW * H * W + (double)B * Co * oH * oW));
	THHIP_DISPATCH_FLOAT(dtype, (col2im_kernel<DT><<<ew_grid(groups), dim3(EW_THREADS), 0, thhip_stream()>>>(col, bias, y, p)));
}

/* Weights of a full convolution, [Ci][Co][kH][kW] host floats, as the packed
 * operand of the 1x1 convolution that makes the columns: row (o*kH+kh)*kW+kw
 * holds the Ci factors of that output tap (the reference multiplies with the
 * transposed weight matrix, SpatialFullConvolution.c:204-212). */
extern "C" void *thhip_fullconv_pack_weight(const float *w, int Ci, int Co, int kH, int kW, int dtype)
{
	const long M = (long)Co * kH * kW;
	float *wt = (float *)malloc(sizeof(float) * M * Ci);
	if (!wt)
		THError("thhip_fullconv_pack_weight: out of memory");
	for (int c = 0; c < Ci; c++)
		for (long m = 0; m < M; m++)
			wt[m * Ci + c] = w[(long)c * M + m];
	void *wp = thhip_conv_pack_weight(wt, (int)M, Ci, 1, dtype);
	free(wt);
	return wp;
}

/* nn_SpatialFullConvolution_updateOutput (SpatialFullConvolution.c:136-250):
 * columns = 1x1 convolution with the packed transposed weights (the MFMA
 * kernel; col is scratch for B*Co*kH*kW*H*W elements), then thhip_col2im. */
extern "C" void thhip_fullconv2d(const void *x, const void *wp, const float *bias, float beta, void *col, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int adjH, int adjW,
	int act, float thr, float val, int dtype)
{
	thhip_conv2d(x, wp, 0, col, B, Ci, H, W, Co * kH * kW, 1, 1, 1, 1, 0, 0, 0, 0, 0, dtype);
	thhip_col2im(col, bias, beta, y, B, Co, H, W, kH, kW, dH, dW, padH, padW, adjH, adjW, act, thr, val, dtype);
}

/* The same pooling on channels-last codes [B][H][W][C], C % 4 == 0: a thread
 * owns four adjacent planes of one output position and reads them as one word
 * per window element (lowp_SpatialMaxPooling.c:20-50 per plane). */
__global__ void maxpool_u8_cl_kernel(const unsigned *x, unsigned *y, PoolParams p)
{
	const int C4 = p.C / 4;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int c4 = (int)(i % C4);
		long t = i / C4;
		const int ox = (int)(t % p.oW);
		t /= p.oW;
		const int oy = (int)(t % p.oH);
		const long b = t / p.oH;
		int hs = oy * p.dH - p.padH, ws = ox * p.dW - p.padW;
		const int he = min(hs + p.kH, p.H), we = min(ws + p.kW, p.W);
		hs = max(hs, 0);
		ws = max(ws, 0);
		unsigned m0 = 0, m1 = 0, m2 = 0, m3 = 0;
		for (int yy = hs; yy < he; yy++)
			for (int xx = ws; xx < we; xx++) {
				const unsigned v = x[((b * p.H + yy) * p.W + xx) * C4 + c4];
				m0 = max(m0, v & 255u);
				m1 = max(m1, (v >> 8) & 255u);
				m2 = max(m2, (v >> 16) & 255u);
				m3 = max(m3, v >> 24);
			}
		y[i] = m0 | (m1 << 8) | (m2 << 16) | (m3 << 24);
	}
}

/* Sixteen planes per thread (C % 16 == 0): 16-byte loads and stores. */
__global__ void maxpool_u8_cl16_kernel(const uintx4 *x, uintx4 *y, PoolParams p)
{
	const int C16 = p.C / 16;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int c16 = (int)(i % C16);
		long t = i / C16;
		const int ox = (int)(t % p.oW);
		t /= p.oW;
		const int oy = (int)(t % p.oH);
		const long b = t / p.oH;
		int hs = oy * p.dH - p.padH, ws = ox * p.dW - p.padW;
		const int he = min(hs + p.kH, p.H), we = min(ws + p.kW, p.W);
		hs = max(hs, 0);
		ws = max(ws, 0);
		unsigned m[16];
#pragma unroll
		for (int k = 0; k < 16; k++)
			m[k] = 0;
		for (int yy = hs; yy < he; yy++)
			for (int xx = ws; xx < we; xx++) {
				const uintx4 v = x[((b * p.H + yy) * p.W + xx) * C16 + c16];
#pragma unroll
				for (int d = 0; d < 4; d++) {
					m[4 * d] = max(m[4 * d], v[d] & 255u);
					m[4 * d + 1] = max(m[4 * d + 1], (v[d] >> 8) & 255u);
					m[4 * d + 2] = max(m[4 * d + 2], (v[d] >> 16) & 255u);
					m[4 * d + 3] = max(m[4 * d + 3], v[d] >> 24);
				}
			}
		uintx4 o;
#pragma unroll
		for (int d = 0; d < 4; d++)
			o[d] = m[4 * d] | (m[4 * d + 1] << 8) | (m[4 * d + 2] << 16) | (m[4 * d + 3] << 24);
		y[i] = o;
	}
}

extern "C" void thhip_maxpool_u8_cl(const unsigned char *x, unsigned char *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW)
{
	if (C % 4)
		THError("thhip_maxpool_u8_cl: C = %d is not a multiple of 4", C);
	const int per = C % 16 == 0 && ((size_t)x & 15) == 0 && ((size_t)y & 15) == 0 ? 16 : 4;
	PoolParams p = { C, H, W, oH, oW, kH, kW, dH, dW, padH, padW, (long)B * oH * oW * (C / per) };
	if (p.total <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, (double)B * C * H * W + (double)per * p.total);
	if (per == 16)
		maxpool_u8_cl16_kernel<<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>((const uintx4 *)x, (uintx4 *)y, p);
	else
		maxpool_u8_cl_kernel<<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>((const unsigned *)x, (unsigned *)y, p);
}

/* SpatialMaxPooling (SpatialMaxPooling.c:168-247) on channels-last half tensors
 * [B][H][W][C], C % 8 == 0: a thread owns eight adjacent planes of one output
 * position and reads them as one 16-byte vector per window element. */
template <int DT>
__global__ void maxpool_half_cl_kernel(const uintx4 *x, uintx4 *y, PoolParams p)
{
	typedef typename ThhipElem<DT>::T elem;
	const int C8 = p.C / 8;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int c8 = (int)(i % C8);
		long t = i / C8;
		const int ox = (int)(t % p.oW);
		t /= p.oW;
		const int oy = (int)(t % p.oH);
		const long b = t / p.oH;
		int hs = oy * p.dH - p.padH, ws = ox * p.dW - p.padW;
		const int he = min(hs + p.kH, p.H), we = min(ws + p.kW, p.W);
		hs = max(hs, 0);
		ws = max(ws, 0);
		float m[8];
#pragma unroll
		for (int k = 0; k < 8; k++)
			m[k] = -FLT_MAX;
		for (int yy = hs; yy < he; yy++)
			for (int xx = ws; xx < we; xx++) {
				const uintx4 raw = x[((b * p.H + yy) * p.W + xx) * C8 + c8];
				elem v[8];
				__builtin_memcpy(v, &raw, 16);
#pragma unroll
				for (int k = 0; k < 8; k++) {
					const float f = (float)v[k];
					if (f > m[k])
						m[k] = f;
				}
			}
		elem o[8];
#pragma unroll
		for (int k = 0; k < 8; k++)
			o[k] = (elem)m[k];
		uintx4 raw;
		__builtin_memcpy(&raw, o, 16);
		y[i] = raw;
	}
}

extern "C" void thhip_maxpool_cl(const void *x, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype)
{
	if (dtype == THHIP_U8) {
		thhip_maxpool_u8_cl((const unsigned char *)x, (unsigned char *)y, B, C, H, W, oH, oW, kH, kW, dH, dW, padH, padW);
		return;
	}
	if (dtype != THHIP_F16 && dtype != THHIP_BF16)
		THError("thhip_maxpool_cl: dtype %d has no channels-last form", dtype);
	if (C % 8)
		THError("thhip_maxpool_cl: C = %d is not a multiple of 8", C);
	PoolParams p = { C, H, W, oH, oW, kH, kW, dH, dW, padH, padW, (long)B * oH * oW * (C / 8) };
	if (p.total <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * B * C * H * W + 16.0 * p.total);
	if (dtype == THHIP_F16)
		maxpool_half_cl_kernel<THHIP_F16><<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>((const uintx4 *)x, (uintx4 *)y, p);
	else
		maxpool_half_cl_kernel<THHIP_BF16><<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>((const uintx4 *)x, (uintx4 *)y, p);
}

/* Codes between plane-major [B][C][HW] and channels-last [B][HW][C] memory
 * order (to_cl = 1: the former to the latter), through a 32 x 32 LDS tile. */
template <typename E>
__global__ void relayout_kernel(const E *x, E *y, int C, int HW, int to_cl)
{
	__shared__ E t[32][33];
	/* source [R][S] -> destination [S][R] per image */
	const int R = to_cl ? C : HW, S = to_cl ? HW : C;
	const size_t img = (size_t)blockIdx.z * C * HW;
	const int r0 = blockIdx.y * 32, s0 = blockIdx.x * 32;
	const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
	for (int k = ty; k < 32; k += 8)
		if (r0 + k < R && s0 + tx < S)
			t[k][tx] = x[img + (size_t)(r0 + k) * S + s0 + tx];
	__syncthreads();
	for (int k = ty; k < 32; k += 8)
		if (s0 + k < S && r0 + tx < R)
			y[img + (size_t)(s0 + k) * R + r0 + tx] = t[tx][k];
}

extern "C" void thhip_relayout(const void *x, void *y, int B, int C, int HW, int to_channels_last, int dtype)
{
	if (B < 1 || C < 1 || HW < 1)
		return;
	if (B > 65535)
		THError("thhip_relayout: batch %d too large", B);
	const int R = to_channels_last ? C : HW, S = to_channels_last ? HW : C;
	const int esz = thhip_esize(dtype);
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * esz * B * C * HW);
	const dim3 grid((S + 31) / 32, (R + 31) / 32, B);
	if (esz == 1)
		relayout_kernel<unsigned char><<<grid, dim3(256), 0, thhip_stream()>>>((const unsigned char *)x,
			(unsigned char *)y, C, HW, to_channels_last != 0);
	else if (esz == 2)
		relayout_kernel<unsigned short><<<grid, dim3(256), 0, thhip_stream()>>>((const unsigned short *)x,
			(unsigned short *)y, C, HW, to_channels_last != 0);
	else
		relayout_kernel<float><<<grid, dim3(256), 0, thhip_stream()>>>((const float *)x, (float *)y, C, HW,
			to_channels_last != 0);
}

extern "C" void thhip_relayout_u8(const unsigned char *x, unsigned char *y, int B, int C, int HW, int to_channels_last)
{
	thhip_relayout(x, y, B, C, HW, to_channels_last, THHIP_U8);
}

/* modules/SpatialAveragePooling.c:156-203 */
template <int DT>
__global__ void avgpool_kernel(const void *x, void *y, PoolParams p, int count_include_pad)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < p.total; i += step) {
		const int ox = (int)(i % p.oW);
		const long t = i / p.oW;
		const int oy = (int)(t % p.oH);
		const long plane = t / p.oH;
		int hs = oy * p.dH - p.padH, ws = ox * p.dW - p.padW;
		int he = min(hs + p.kH, p.H + p.padH), we = min(ws + p.kW, p.W + p.padW);
		const int pool = (he - hs) * (we - ws);
		hs = max(hs, 0);
		ws = max(ws, 0);
		he = min(he, p.H);
		we = min(we, p.W);
		const int div = count_include_pad ? pool : (he - hs) * (we - ws);
		const long base = plane * p.H * p.W;
		float sum = 0;
		for (int yy = hs; yy < he; yy++)
			for (int xx = ws; xx < we; xx++)
				sum += ThhipElem<DT>::ld(x, base + (long)yy * p.W + xx);
		ThhipElem<DT>::st(y, i, sum / (float)div);
	}
}

/* The same for a window that is the whole plane (the pooling before a classifier): sixteen lanes per
 * plane, neighbouring lanes on neighbouring values (one thread per plane reads 4 HW bytes apart from its
 * neighbours and leaves most CUs idle: 32 x 512 planes of 7 x 7, 12 -> 4 us). */
template <int DT>
__global__ __launch_bounds__(256) void avgpool_plane_kernel(const void *x, void *y, long planes, int HW)
{
	const long plane = ((long)blockIdx.x * 256 + threadIdx.x) >> 4;
	const int l = threadIdx.x & 15;
	float sum = 0;
	if (plane < planes)
		for (int i = l; i < HW; i += 16)
			sum += ThhipElem<DT>::ld(x, plane * HW + i);
	for (int off = 8; off > 0; off >>= 1)
		sum += __shfl_xor(sum, off, 64);
	if (plane < planes && l == 0)
		ThhipElem<DT>::st(y, plane, sum / (float)HW);
}

extern "C" void thhip_avgpool(const void *x, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int count_include_pad, int dtype)
{
	PoolParams p = { C, H, W, oH, oW, kH, kW, dH, dW, padH, padW, (long)B * C * oH * oW };
	if (p.total <= 0)
		return;
	const double esz = thhip_esize(dtype);
	ThhipLaunchScope scope(THHIP_FAM_OTHER, esz * ((double)B * C * H * W + (double)p.total));
	if (oH == 1 && oW == 1 && kH == H && kW == W && !padH && !padW && H * W >= 16 && p.total <= (0x7fffffffL >> 4)) {
		THHIP_DISPATCH_FLOAT(dtype, (avgpool_plane_kernel<DT><<<dim3((unsigned)((p.total * 16 + 255) / 256)), dim3(256), 0, thhip_stream()>>>(
			x, y, p.total, H * W)));
		return;
	}
	THHIP_DISPATCH_FLOAT(dtype, (avgpool_kernel<DT><<<ew_grid(p.total), dim3(EW_THREADS), 0, thhip_stream()>>>(
		x, y, p, count_include_pad)));
}

/* ---------------- SoftMax ---------------- */

/* THExpMinusApprox, thbasic.c:462-491 */
__device__ __forceinline__ double exp_minus_approx(double x)
{
	if (x < 13.0) {
		double y = 1.0 + x * (0.125 + x * (0.0078125 + x * (0.00032552083 + x * 1.0172526e-5)));
		y *= y;
		y *= y;
		y *= y;
		return 1 / y;
	}
	return 0;
}

/* modules/SoftMax.c:24-90: one workgroup of T threads per (frame, position): a wavefront where there
 * are many positions, sixteen for a few long vectors (a classifier's 1000 values at batch 1 took 11 us
 * with one wavefront, the double-precision exponential twice per value; a thread's first four values are
 * kept). */
template <int DT, int T>
__global__ __launch_bounds__(T) void softmax_kernel(const void *x, void *y, long dim, long stride)
{
	constexpr int KEEP = 4, WAVES = T / 64;
	__shared__ float red[2][WAVES > 1 ? WAVES : 1];
	const long t = blockIdx.x;
	const long base = (t / stride) * dim * stride + t % stride;
	const int tid = threadIdx.x;
	float m = -FLT_MAX;
	for (long d = tid; d < dim; d += T)
		m = fmaxf(m, ThhipElem<DT>::ld(x, base + d * stride));
	for (int off = 32; off > 0; off >>= 1)
		m = fmaxf(m, __shfl_xor(m, off, 64));
	if constexpr (WAVES > 1) {
		if ((tid & 63) == 0)
			red[0][tid >> 6] = m;
		__syncthreads();
#pragma unroll
		for (int w = 0; w < WAVES; w++)
			m = fmaxf(m, red[0][w]);
	}
	float sum = 0, zk[KEEP];
#pragma unroll
	for (int i = 0; i < KEEP; i++) {
		const long d = tid + (long)i * T;
		zk[i] = d < dim ? (float)exp_minus_approx((double)(m - ThhipElem<DT>::ld(x, base + d * stride))) : 0.0f;
		sum += zk[i];
	}
	for (long d = tid + (long)KEEP * T; d < dim; d += T)
		sum += (float)exp_minus_approx((double)(m - ThhipElem<DT>::ld(x, base + d * stride)));
	for (int off = 32; off > 0; off >>= 1)
		sum += __shfl_xor(sum, off, 64);
	if constexpr (WAVES > 1) {
		if ((tid & 63) == 0)
			red[1][tid >> 6] = sum;
		__syncthreads();
		sum = 0;
#pragma unroll
		for (int w = 0; w < WAVES; w++)
			sum += red[1][w];
	}
	const float inv = 1 / sum;
#pragma unroll
	for (int i = 0; i < KEEP; i++) {
		const long d = tid + (long)i * T;
		if (d < dim)
			ThhipElem<DT>::st(y, base + d * stride, zk[i] * inv);
	}
	for (long d = tid + (long)KEEP * T; d < dim; d += T) {
		const float z = (float)exp_minus_approx((double)(m - ThhipElem<DT>::ld(x, base + d * stride)));
		ThhipElem<DT>::st(y, base + d * stride, z * inv);
	}
}

extern "C" void thhip_softmax(const void *x, void *y, long nframe, long dim, long stride, int dtype)
{
	const long npos = nframe * stride;
	if (npos <= 0 || dim <= 0)
		return;
	if (npos > 0x7fffffffL)
		THError("thhip_softmax: too many positions");
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * npos * dim * thhip_esize(dtype));
	if (dim >= 512 && npos <= 2048)
		THHIP_DISPATCH_FLOAT(dtype, (softmax_kernel<DT, 1024><<<dim3((unsigned)npos), dim3(1024), 0, thhip_stream()>>>(
			x, y, dim, stride)));
	else
		THHIP_DISPATCH_FLOAT(dtype, (softmax_kernel<DT, 64><<<dim3((unsigned)npos), dim3(64), 0, thhip_stream()>>>(
			x, y, dim, stride)));
}

/* lowp/lowp_SoftMax.c:3-89.  The exponent argument keeps the tensor offset,
 * and the float running sum is taken in index order by one lane so that the
 * codes match a sequential evaluation bit for bit. */
#define SOFTMAX_U8_MAXDIM 8192
__global__ __launch_bounds__(64) void softmax_u8_kernel(const unsigned char *x, unsigned char *y, long dim, long stride,
	float invmult, float sub, int single, float *max_out)
{
	__shared__ float tmp[SOFTMAX_U8_MAXDIM];
	__shared__ float s_scale, s_max;
	const long t = blockIdx.x;
	const long base = (t / stride) * dim * stride + t % stride;
	const int lane = threadIdx.x;
	int qmax = 0;
	for (long d = lane; d < dim; d += 64)
		qmax = max(qmax, (int)x[base + d * stride]);
	for (int off = 32; off > 0; off >>= 1)
		qmax = max(qmax, __shfl_xor(qmax, off, 64));
	for (long d = lane; d < dim; d += 64) {
		const float arg = (float)(qmax - (int)x[base + d * stride]) * invmult + sub;
		tmp[d] = (float)exp_minus_approx((double)arg);
	}
	__syncthreads();
	if (lane == 0) {
		float sum = 0;
		for (long d = 0; d < dim; d++)
			sum = sum + tmp[d];
		s_scale = 1 / sum;
	}
	__syncthreads();
	const float scale = s_scale;
	if (!single) {
		for (long d = lane; d < dim; d += 64)
			y[base + d * stride] = (unsigned char)(int)(255.0f * (tmp[d] * scale));
		return;
	}
	float mx = 0;
	for (long d = lane; d < dim; d += 64) {
		tmp[d] = tmp[d] * scale;
		mx = fmaxf(mx, tmp[d]);
	}
	for (int off = 32; off > 0; off >>= 1)
		mx = fmaxf(mx, __shfl_xor(mx, off, 64));
	if (lane == 0) {
		s_max = mx;
		*max_out = mx;
	}
	__syncthreads();
	const float rmax = 1 / s_max;
	for (long d = lane; d < dim; d += 64)
		y[base + d * stride] = (unsigned char)(int)((255.0f * tmp[d]) * rmax);
}

extern "C" float thhip_softmax_u8(const unsigned char *x, unsigned char *y, long nframe, long dim, long stride,
	float in_mult, float in_sub)
{
	const long npos = nframe * stride;
	if (npos <= 0 || dim <= 0)
		return 0;
	if (dim > SOFTMAX_U8_MAXDIM)
		THError("thhip_softmax_u8: dim %ld exceeds %d", dim, SOFTMAX_U8_MAXDIM);
	const float invmult = in_mult ? 1 / in_mult : 0;
	const int single = npos == 1;
	float *dmax = single ? (float *)thhip_malloc(4) : 0;
	{
		ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * npos * dim);
		softmax_u8_kernel<<<dim3((unsigned)npos), dim3(64), 0, thhip_stream()>>>(x, y, dim, stride, invmult, in_sub,
			single, dmax);
	}
	if (!single)
		return 255;
	float mx = 0;
	thhip_memcpy_d2h(&mx, dmax, 4);
	thhip_free(dmax);
	return 255 / mx;
}

/* ---------------- batch normalisation ---------------- */

/* modules/SpatialBatchNormalization.c:78-109: y = ((x - mean) * invstd) * w + b */
template <int DT>
__global__ void batchnorm_kernel(const void *x, void *y, long total, long C, long HW,
	const float *mean, const float *invstd, const float *weight, const float *bias)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const long f = (i / HW) % C;
		const float w = weight ? weight[f] : 1.0f, b = bias ? bias[f] : 0.0f;
		const float v = ThhipElem<DT>::ld(x, i);
		ThhipElem<DT>::st(y, i, ((v - mean[f]) * invstd[f]) * w + b);
	}
}

extern "C" void thhip_batchnorm(const void *x, void *y, long B, long C, long HW,
	const float *mean, const float *invstd, const float *weight, const float *bias, int dtype)
{
	const long total = B * C * HW;
	if (total <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * total * thhip_esize(dtype));
	THHIP_DISPATCH_FLOAT(dtype, (batchnorm_kernel<DT><<<ew_grid(total, 4), dim3(EW_THREADS), 0, thhip_stream()>>>(
		x, y, total, C, HW, mean, invstd, weight, bias)));
}

/* ---------------- two-input table add (modules/CAddTable.c:59-70) ---------------- */

template <int DT>
__global__ void axpby2_kernel(const void *a, const void *b, void *y, long na, long nb, float sign, int act)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < na; i += step) {
		float v = ThhipElem<DT>::ld(a, i);
		if (i < nb)
			v = v + sign * ThhipElem<DT>::ld(b, i);
		if (act)
			v = v > 0.0f ? v : 0.0f;
		ThhipElem<DT>::st(y, i, v);
	}
}

extern "C" void thhip_axpby2(const void *a, const void *b, void *y, long na, long nb, float sign, int act, int dtype)
{
	if (na <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, (2.0 * na + nb) * thhip_esize(dtype));
	THHIP_DISPATCH_FLOAT(dtype, (axpby2_kernel<DT><<<ew_grid(na, 4), dim3(EW_THREADS), 0, thhip_stream()>>>(
		a, b, y, na, nb, sign, act)));
}

/* ---------------- dtype conversion ---------------- */

template <int SD, int DD>
__global__ void convert_kernel(const void *src, void *dst, long n)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < n; i += step) {
		float v;
		if constexpr (SD == THHIP_U8)
			v = (float)((const unsigned char *)src)[i];
		else
			v = ThhipElem<SD>::ld(src, i);
		ThhipElem<DD>::st(dst, i, v);
	}
}

extern "C" void thhip_convert(const void *src, int sd, void *dst, int dd, long n)
{
	if (n <= 0)
		return;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, (double)n * (thhip_esize(sd) + thhip_esize(dd)));
	const dim3 grid = ew_grid(n, 4), blk(EW_THREADS);
	hipStream_t s = thhip_stream();
#define CV(S, D) if (sd == S && dd == D) { convert_kernel<S, D><<<grid, blk, 0, s>>>(src, dst, n); return; }
	CV(THHIP_F32, THHIP_F32) CV(THHIP_F32, THHIP_F16) CV(THHIP_F32, THHIP_BF16)
	CV(THHIP_F16, THHIP_F32) CV(THHIP_BF16, THHIP_F32) CV(THHIP_U8, THHIP_F32)
#undef CV
	THError("thhip_convert: unsupported conversion %d -> %d", sd, dd);
}

/* ---------------- (x - mean) / std on the first three planes (thapi.c:389-403) ---------------- */

/* THProcessFloat's normalisation of a [B][C][HW] fp32 tensor, on the device
 * copy: the same subtraction and correctly rounded division as the host loop,
 * so both give the same bits.  src is fp32; dst may be any float dtype. */
template <int DT>
__global__ void normalize_kernel(const float *src, void *dst, int C, long HW, long total, floatx4 mean, floatx4 std)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const int c = (int)((i / HW) % C);
		float v = src[i];
		if (c < 3)
			v = (v - mean[c]) / std[c];
		ThhipElem<DT>::st(dst, i, v);
	}
}

extern "C" void thhip_normalize(const float *src, void *dst, int B, int C, long HW, const float *mean3, const float *std3,
	int dtype)
{
	const long total = (long)B * C * HW;
	if (total <= 0)
		return;
	const floatx4 mean = { mean3[0], mean3[1], mean3[2], 0 }, std = { std3[0], std3[1], std3[2], 1 };
	ThhipLaunchScope scope(THHIP_FAM_OTHER, (4.0 + thhip_esize(dtype)) * total);
	THHIP_DISPATCH_FLOAT(dtype, (normalize_kernel<DT><<<ew_grid(total, 4), dim3(EW_THREADS), 0, thhip_stream()>>>(src, dst, C, HW,
		total, mean, std)));
}

/* ---------------- 8-bit image -> normalised planar float (thapi.c:20-46) ---------------- */

template <int DT>
__global__ void rgb2float_kernel(void *dst, const unsigned char *src, long src_pitch, int width, int height, int stride, int cp,
	floatx4 mean, floatx4 std1, int bgr)
{
	const long total = (long)cp * width * height;
	src += src_pitch * blockIdx.y;		/* one image per blockIdx.y */
	dst = (char *)dst + (long)blockIdx.y * total * (DT == THHIP_F32 ? 4 : 2);
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const int j = (int)(i % width);
		const long t = i / width;
		const int r = (int)(t % height);
		const int c = (int)(t / height);
		const int sc = bgr ? cp - 1 - c : c;
		const float byte = (float)src[sc + cp * j + (long)stride * r];
		/* (byte * (1/255) - mean) * (1/std), three separately rounded steps */
		const float v = (byte * 0.003921568f - mean[c]) * std1[c];
		ThhipElem<DT>::st(dst, i, v);
	}
}

/* n images, `src_pitch` bytes apart in src, become n consecutive [cp][height][width] tensors in dst */
extern "C" void thhip_rgb2float_batch(void *dst, const unsigned char *src, int n, long src_pitch, int width, int height,
	int stride, int cp, const float *mean, const float *std, int bgr, int dtype)
{
	if (cp < 1 || cp > 3)
		THError("thhip_rgb2float: %d colour planes", cp);
	if (n < 1 || n > 65535)
		THError("thhip_rgb2float: %d images", n);
	floatx4 m = { 0, 0, 0, 0 }, s = { 1, 1, 1, 1 };
	for (int i = 0; i < cp; i++) {
		m[i] = mean[i];
		s[i] = 1 / std[i];
	}
	const long total = (long)cp * width * height;
	ThhipLaunchScope scope(THHIP_FAM_OTHER, (double)n * total * (1 + thhip_esize(dtype)));
	dim3 grid = ew_grid(total, 4);
	grid.y = n;
	THHIP_DISPATCH_FLOAT(dtype, (rgb2float_kernel<DT><<<grid, dim3(EW_THREADS), 0, thhip_stream()>>>(
		dst, src, src_pitch, width, height, stride, cp, m, s, bgr)));
}

extern "C" void thhip_rgb2float(void *dst, const unsigned char *src, int width, int height, int stride, int cp,
	const float *mean, const float *std, int bgr, int dtype)
{
	thhip_rgb2float_batch(dst, src, 1, 0, width, height, stride, cp, mean, std, bgr, dtype);
}

/* ---------------- 8-bit image -> planar uint8 codes (lowp/lowp_basic.c:60-131) ---------------- */

__global__ void rgb2code_kernel(unsigned char *dst, const unsigned char *src, long src_pitch, int width, int height, int stride,
	int sub0, int sub1, int sub2, float mult0, float mult1, float mult2, int bgr)
{
	const long total = 3L * width * height;
	src += src_pitch * blockIdx.y;		/* one image per blockIdx.y */
	dst += total * blockIdx.y;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const int j = (int)(i % width);
		const long t = i / width;
		const int r = (int)(t % height);
		const int c = (int)(t / height);
		const int sc = bgr ? 2 - c : c;
		const int sub = c == 0 ? sub0 : c == 1 ? sub1 : sub2;
		const float mult = c == 0 ? mult0 : c == 1 ? mult1 : mult2;
		/* rgb2tensord, lowp_basic.c:68: integer difference, one float product,
		 * roundf, then the conversion to a byte of the reference's x86 build
		 * (through int, so values outside 0..255 wrap) */
		const float v = roundf((float)((int)src[sc + 3 * j + (long)stride * r] - sub) * mult);
		dst[i] = (unsigned char)(int)v;
	}
}

/* One image of Lowp_LoadImages (lowp_basic.c:82-131): the fixed input range
 * derived from mean / std gives the tensor's (mult, sub), returned through the
 * pointers, and per-plane integer offsets and factors.  src is a device copy
 * of the interleaved 8-bit image. */
extern "C" void thhip_rgb2code_batch(unsigned char *dst, const unsigned char *src, int n, long src_pitch, int width,
	int height, int stride, const float *mean, const float *std, int bgr, float *mult_out, float *sub_out)
{
	if (n < 1 || n > 65535)
		THError("thhip_rgb2code: %d images", n);
	int sub[3];
	float mult[3], mn = 1e30, mx = -1e30, tmult;
	/* the kernel reads three bytes of every pixel: the source must hold
	 * stride * (height - 1) + 3 * width bytes, which a copy of `height` rows of
	 * `stride` bytes only does for stride >= 3 * width.  (The reference's loader
	 * reads past its host image for narrower rows; a device read out of bounds
	 * can fault.) */
	if (stride < 3 * width)
		THError("thhip_rgb2code: row stride %d is less than 3 * width %d: the uint8 image loader takes three-plane "
			"images only (lowp_basic.c:82-131)", stride, width);
	for (int i = 0; i < 3; i++) {
		if (-mean[i] / std[i] < mn)
			mn = -mean[i] / std[i];
		if ((1 - mean[i]) / std[i] > mx)
			mx = (1 - mean[i]) / std[i];
	}
	tmult = (mx - mn) ? 255 / (mx - mn) : 0;
	for (int i = 0; i < 3; i++) {
		sub[i] = roundf(255 * (mean[i] + std[i] * mn));
		mult[i] = tmult / (255 * std[i]);
	}
	const long total = 3L * width * height;
	if (total > 0) {
		ThhipLaunchScope scope(THHIP_FAM_OTHER, 2.0 * n * total);
		dim3 grid = ew_grid(total, 4);
		grid.y = n;
		rgb2code_kernel<<<grid, dim3(EW_THREADS), 0, thhip_stream()>>>(dst, src, src_pitch, width, height, stride,
			sub[0], sub[1], sub[2], mult[0], mult[1], mult[2], bgr);
	}
	*mult_out = tmult;
	*sub_out = mn;
}

extern "C" void thhip_rgb2code(unsigned char *dst, const unsigned char *src, int width, int height, int stride,
	const float *mean, const float *std, int bgr, float *mult_out, float *sub_out)
{
	thhip_rgb2code_batch(dst, src, 1, 0, width, height, stride, mean, std, bgr, mult_out, sub_out);
}

/* ---------------- smallest and largest element (FindMinMax, thapi.c:141-154) ---------------- */

template <int DT>
__global__ void minmax_any_kernel(const void *x, long n, float *part)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	float mn = FLT_MAX, mx = -FLT_MAX;	/* THInf / -THInf (thnets.h:463: FLT_MAX); comparisons skip NaN like the reference's */
	for (; i < n; i += step) {
		float v;
		if constexpr (DT == THHIP_U8)
			v = (float)((const unsigned char *)x)[i];
		else
			v = ThhipElem<DT>::ld(x, i);
		mn = v < mn ? v : mn;
		mx = v > mx ? v : mx;
	}
	for (int off = 32; off > 0; off >>= 1) {
		const float a = __shfl_xor(mn, off, 64), b = __shfl_xor(mx, off, 64);
		mn = a < mn ? a : mn;
		mx = b > mx ? b : mx;
	}
	__shared__ float smn[4], smx[4];
	if ((threadIdx.x & 63) == 0) {
		smn[threadIdx.x >> 6] = mn;
		smx[threadIdx.x >> 6] = mx;
	}
	__syncthreads();
	if (threadIdx.x == 0) {
		for (int w = 1; w < 4; w++) {
			mn = smn[w] < mn ? smn[w] : mn;
			mx = smx[w] > mx ? smx[w] : mx;
		}
		part[2 * blockIdx.x] = mn;
		part[2 * blockIdx.x + 1] = mx;
	}
}

extern "C" void thhip_minmax(const void *x, long n, int dtype, float *min_out, float *max_out)
{
	float mn = FLT_MAX, mx = -FLT_MAX;	/* THInf, thnets.h:463; an empty tensor returns them as they are */
	if (n > 0) {
		long blocks = (n + 1023) / 1024;
		if (blocks > 1024)
			blocks = 1024;
		float *d = (float *)thhip_malloc(sizeof(float) * 2 * blocks);
		float *h = (float *)malloc(sizeof(float) * 2 * blocks);
		{
			ThhipLaunchScope scope(THHIP_FAM_OTHER, (double)thhip_esize(dtype) * n);
			if (dtype == THHIP_U8)
				minmax_any_kernel<THHIP_U8><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(x, n, d);
			else
				THHIP_DISPATCH_FLOAT(dtype, (minmax_any_kernel<DT><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(x, n, d)));
		}
		thhip_memcpy_d2h(h, d, sizeof(float) * 2 * blocks);
		for (long b = 0; b < blocks; b++) {
			mn = h[2 * b] < mn ? h[2 * b] : mn;
			mx = h[2 * b + 1] > mx ? h[2 * b + 1] : mx;
		}
		free(h);
		thhip_free(d);
	}
	*min_out = mn;
	*max_out = mx;
}

/* ---------------- uint8 quantise / de-quantise (lowp/lowp_basic.c:5-58) ---------------- */

__global__ void minmax_kernel(const float *x, long n, unsigned *out)
{
	/* out[0]: bits of the most negative value, out[1]: bits of the largest
	 * positive value; both start at +0.0f, so zero is always in range
	 * (lowp_basic.c:17).  Among same-sign floats the bit patterns order like
	 * the magnitudes. */
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	float mn = 0, mx = 0;
	for (; i < n; i += step) {
		const float v = x[i];
		if (v < mn)
			mn = v;
		if (v > mx)
			mx = v;
	}
	for (int off = 32; off > 0; off >>= 1) {
		mn = fminf(mn, __shfl_xor(mn, off, 64));
		mx = fmaxf(mx, __shfl_xor(mx, off, 64));
	}
	/* one pair of atomics per workgroup: they all hit the same two words */
	__shared__ float smn[4], smx[4];
	if ((threadIdx.x & 63) == 0) {
		smn[threadIdx.x >> 6] = mn;
		smx[threadIdx.x >> 6] = mx;
	}
	__syncthreads();
	if (threadIdx.x == 0) {
		mn = fminf(fminf(smn[0], smn[1]), fminf(smn[2], smn[3]));
		mx = fmaxf(fmaxf(smx[0], smx[1]), fmaxf(smx[2], smx[3]));
		if (mn < 0)
			atomicMax(&out[0], __float_as_uint(mn));
		if (mx > 0)
			atomicMax(&out[1], __float_as_uint(mx));
	}
}

__global__ void quantize_kernel(const float *x, unsigned char *q, long n, float mult, float zero)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < n; i += step)
		q[i] = (unsigned char)(int)(roundf(x[i] * mult) - zero);
}

extern "C" void thhip_quantize(const float *x, unsigned char *q, long n, float *mult_out, float *sub_out)
{
	unsigned bits[2] = { 0, 0 };
	unsigned *d = (unsigned *)thhip_malloc(8);
	thhip_memcpy_h2d(d, bits, 8);
	if (n > 0) {
		long blocks = (n + 255) / 256;
		if (blocks > 1024)
			blocks = 1024;
		ThhipLaunchScope scope(THHIP_FAM_OTHER, 4.0 * n);
		minmax_kernel<<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(x, n, d);
	}
	thhip_memcpy_d2h(bits, d, 8);
	thhip_free(d);
	float mn, mx, mult;
	memcpy(&mn, &bits[0], 4);
	memcpy(&mx, &bits[1], 4);
	if (mx - mn > 0)
		mult = (float)(255.0 / (mx - mn));	/* lowp_basic.c:25-27 */
	else
		mult = 0;
	const float zero = roundf(mn * mult);
	if (n > 0) {
		ThhipLaunchScope scope(THHIP_FAM_OTHER, 5.0 * n);
		quantize_kernel<<<ew_grid(n, 4), dim3(EW_THREADS), 0, thhip_stream()>>>(x, q, n, mult, zero);
	}
	*mult_out = mult;
	*sub_out = mn;
}

__global__ void dequantize_kernel(const unsigned char *q, float *x, long n, float invmult, float sub)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < n; i += step)
		x[i] = (float)q[i] * invmult + sub;
}

extern "C" void thhip_dequantize(const unsigned char *q, float *x, long n, float mult, float sub)
{
	if (n <= 0)
		return;
	const float invmult = mult ? (float)(1.0 / mult) : 0;	/* lowp_basic.c:54 */
	ThhipLaunchScope scope(THHIP_FAM_OTHER, 5.0 * n);
	dequantize_kernel<<<ew_grid(n, 4), dim3(EW_THREADS), 0, thhip_stream()>>>(q, x, n, invmult, sub);
}
