/*
 * thnets_oracle.c -- CPU restatement of the thnets conv / Linear / LOWP path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing under thnets_amd/ links, loads or calls
 * this file; it is the checker that tests/, the smoke run and the benchmark's
 * cpu_baseline leg compare the HIP engine against.  Every function cites the
 * reference source it restates (paths relative to the thnets tree).
 *
 * Pinning status (what each restatement has been checked against):
 *   fp32 conv / linear / threshold / maxpool / avgpool / softmax / batchnorm /
 *   caddtable: the reference's own compiled CPU library (oracle/_ref, built
 *   from the reference sources) on seeded inputs, committed golden vectors
 *   made with it, and closed forms (double precision direct convolution,
 *   delta kernels, 1x1 conv == Linear, brute force on tiny shapes).
 *   full (transposed) convolution, max pooling indices, max unpooling: the
 *   reference's compiled CPU library on seeded inputs, and closed forms
 *   (double precision scatter form of the transposed convolution; it is the
 *   adjoint of the convolution: <conv(x), y> == <x, fullconv(y)>; unpooling
 *   of a pooling's own output restores the maxima in place).
 *   lowp quantize / dequantize / threshold / maxpool / softmax: the
 *   reference's lowp_*.c compiled -DLOWP (oracle/_ref, without gemm8.cc).
 *   lowp gemm (orc_lowp_gemm): PARITY UNPINNED against the reference -- the
 *   arithmetic lives in gemmlowp (github.com/google/gemmlowp, no version
 *   pinned by the reference, not vendored, absent here).  It restates
 *   gemmlowp's published legacy contract (EightBitIntGemm ->
 *   OutputStageQuantizeDownInt32ToUint8Scale + SaturatingCastToUint8) and is
 *   pinned only by mathematics: int64 brute force, the expanded-offset
 *   identity, and agreement with the fp32 path within one code step.
 *   lowp conv parameter derivation, uint8 im2col and lowpadd
 *   (orc_lowp_mm_params, orc_lowp_unfold, orc_lowp_add): static functions of
 *   the reference reachable only through the gemmlowp call, so PARITY
 *   UNPINNED against running code; pinned by hand-computed cases.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_MIN(a, b) ((a) < (b) ? (a) : (b))
#define ORC_MAX(a, b) ((a) > (b) ? (a) : (b))

int orc_num_threads(void)
{
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

void orc_set_num_threads(int n)
{
#ifdef _OPENMP
	omp_set_num_threads(n);
#else
	(void)n;
#endif
}

/* ------------------------------------------------------------------ */
/* fp32 convolution                                                    */
/* ------------------------------------------------------------------ */

/* Output extent of a convolution: C integer division,
 * modules/SpatialConvolutionMM.c:159-160. */
int orc_conv_outsize(int in, int k, int d, int pad)
{
	return (in + 2 * pad - k) / d + 1;
}

/* im2col of one image, modules/SpatialConvolutionMM.c:11-73:
 * col[k][y*oW+x] = x[c][y*dH-padH+kh][x*dW-padW+kw] or 0 outside,
 * k = (c*kH+kh)*kW+kw. */
void orc_unfold_f32(const float *x, float *col, int Ci, int H, int W, int kH, int kW,
	int dH, int dW, int padH, int padW, int oH, int oW)
{
	long K = (long)Ci * kH * kW;
	long k;
#pragma omp parallel for
	for (k = 0; k < K; k++) {
		int c = (int)(k / (kH * kW));
		int rest = (int)(k % (kH * kW));
		int kh = rest / kW, kw = rest % kW;
		float *dst = col + k * (long)oH * oW;
		const float *src = x + (long)c * H * W;
		for (int y = 0; y < oH; y++) {
			long iy = (long)y * dH - padH + kh;
			for (int xx = 0; xx < oW; xx++) {
				long ix = (long)xx * dW - padW + kw;
				dst[(long)y * oW + xx] =
					(iy < 0 || iy >= H || ix < 0 || ix >= W) ? 0.0f : src[iy * W + ix];
			}
		}
	}
}

/* C[M][N] += A[M][K] * B[K][N], all row-major, fp32 accumulation.  This is
 * the product thbasic.c:601-711 hands to sgemm with beta = 1
 * (SpatialConvolutionMM.c:103).  The blocking is this file's own; the
 * reference's 384-wide K blocking (OpenBLAS-stripped/sgemm.c:66-70) is not
 * mirrored, which the fp32 tolerance covers. */
typedef float orc_v8 __attribute__((vector_size(32), aligned(4)));

#define ORC_KC 256
#define ORC_NC 512
#define ORC_MR 4
#define ORC_NR 16

static void orc_micro_4x16(int kc, const float *a0, const float *a1, const float *a2, const float *a3,
	const float *bp, float *c, long ldc, int mr, int nr)
{
	orc_v8 acc[ORC_MR][2];
	const float *ar[ORC_MR] = { a0, a1, a2, a3 };
	for (int i = 0; i < ORC_MR; i++)
		acc[i][0] = acc[i][1] = (orc_v8){ 0, 0, 0, 0, 0, 0, 0, 0 };
	for (int k = 0; k < kc; k++) {
		orc_v8 b0 = *(const orc_v8 *)(bp + (long)k * ORC_NR);
		orc_v8 b1 = *(const orc_v8 *)(bp + (long)k * ORC_NR + 8);
		for (int i = 0; i < ORC_MR; i++) {
			float av = ar[i][k];
			orc_v8 a = { av, av, av, av, av, av, av, av };
			acc[i][0] += a * b0;
			acc[i][1] += a * b1;
		}
	}
	for (int i = 0; i < mr; i++)
		for (int j = 0; j < nr; j++)
			c[i * ldc + j] += j < 8 ? acc[i][0][j] : acc[i][1][j - 8];
}

/* Source of B rows: either a dense row-major matrix or a virtual im2col
 * of an image (the reference's VirtMM idea, thbasic.c:1073-1103). */
struct orc_bsrc {
	const float *dense;	/* [K][N] or NULL */
	long N;
	const float *img;	/* [Ci][H][W] */
	int H, W, kH, kW, dH, dW, padH, padW, oW;
};

static inline float orc_b_at(const struct orc_bsrc *s, long k, long n)
{
	if (s->dense)
		return s->dense[k * s->N + n];
	int c = (int)(k / (s->kH * s->kW));
	int rest = (int)(k % (s->kH * s->kW));
	int kh = rest / s->kW, kw = rest % s->kW;
	long oy = n / s->oW, ox = n % s->oW;
	long iy = oy * s->dH - s->padH + kh, ix = ox * s->dW - s->padW + kw;
	if (iy < 0 || iy >= s->H || ix < 0 || ix >= s->W)
		return 0.0f;
	return s->img[((long)c * s->H + iy) * s->W + ix];
}

static void orc_gemm_acc(int M, long N, int K, const float *A, const struct orc_bsrc *bs, float *C, int parallel)
{
	long npanels = (N + ORC_NC - 1) / ORC_NC;
	long jp;
#pragma omp parallel for if(parallel) schedule(dynamic)
	for (jp = 0; jp < npanels; jp++) {
		long j0 = jp * ORC_NC;
		int nc = (int)ORC_MIN((long)ORC_NC, N - j0);
		int nblk = (nc + ORC_NR - 1) / ORC_NR;
		float *bp = (float *)aligned_alloc(64, sizeof(float) * ORC_KC * nblk * ORC_NR);
		for (int k0 = 0; k0 < K; k0 += ORC_KC) {
			int kc = ORC_MIN(ORC_KC, K - k0);
			/* pack: bp[blk][k][16] */
			for (int jb = 0; jb < nblk; jb++)
				for (int k = 0; k < kc; k++)
					for (int j = 0; j < ORC_NR; j++) {
						long n = j0 + (long)jb * ORC_NR + j;
						bp[((long)jb * kc + k) * ORC_NR + j] = n < j0 + nc ? orc_b_at(bs, k0 + k, n) : 0.0f;
					}
			for (int i = 0; i < M; i += ORC_MR) {
				int mr = ORC_MIN(ORC_MR, M - i);
				const float *a0 = A + (long)i * K + k0;
				const float *a1 = mr > 1 ? a0 + K : a0;
				const float *a2 = mr > 2 ? a0 + 2L * K : a0;
				const float *a3 = mr > 3 ? a0 + 3L * K : a0;
				for (int jb = 0; jb < nblk; jb++) {
					int nr = ORC_MIN(ORC_NR, nc - jb * ORC_NR);
					orc_micro_4x16(kc, a0, a1, a2, a3, bp + (long)jb * kc * ORC_NR,
						C + (long)i * N + j0 + (long)jb * ORC_NR, N, mr, nr);
				}
			}
		}
		free(bp);
	}
}

void orc_sgemm_acc(int M, int N, int K, const float *A, const float *B, float *C)
{
	struct orc_bsrc bs;
	memset(&bs, 0, sizeof(bs));
	bs.dense = B;
	bs.N = N;
	orc_gemm_acc(M, N, K, A, &bs, C, 1);
}

/* nn_SpatialConvolutionMM_updateOutput, modules/SpatialConvolutionMM.c:126-225
 * with _frame :75-109: per image, every output plane is filled with its bias
 * (:93-99) and the GEMM accumulates on top (beta = 1).  x [B][Ci][H][W],
 * w [Co][Ci*kH*kW], bias [Co] or NULL, y [B][Co][oH][oW].
 * use_unfold = 1 materialises the im2col matrix first (MT_SpatialConvolutionMM),
 * 0 packs straight from the image (MT_SpatialConvolutionVirtMM). */
int orc_conv2d_f32(const float *x, const float *w, const float *bias, float *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int use_unfold)
{
	int oW = orc_conv_outsize(W, kW, dW, padW);
	int oH = orc_conv_outsize(H, kH, dH, padH);
	if (oW < 1 || oH < 1)
		return -1;	/* the reference calls THError here (:162-164) */
	int K = Ci * kH * kW;
	long N = (long)oH * oW;
	int par_images = B >= 4;	/* :201 */
	int t;
#pragma omp parallel for if(par_images)
	for (t = 0; t < B; t++) {
		const float *xi = x + (long)t * Ci * H * W;
		float *yi = y + (long)t * Co * N;
		for (int o = 0; o < Co; o++) {
			float b = bias ? bias[o] : 0.0f;
			for (long j = 0; j < N; j++)
				yi[o * N + j] = b;
		}
		struct orc_bsrc bs;
		memset(&bs, 0, sizeof(bs));
		float *col = 0;
		if (use_unfold) {
			col = (float *)malloc(sizeof(float) * K * N);
			orc_unfold_f32(xi, col, Ci, H, W, kH, kW, dH, dW, padH, padW, oH, oW);
			bs.dense = col;
			bs.N = N;
		} else {
			bs.img = xi;
			bs.H = H; bs.W = W; bs.kH = kH; bs.kW = kW;
			bs.dH = dH; bs.dW = dW; bs.padH = padH; bs.padW = padW; bs.oW = oW;
			bs.N = N;
		}
		orc_gemm_acc(Co, N, K, w, &bs, yi, !par_images);
		free(col);
	}
	return 0;
}

/* Closed form used to pin the above: direct convolution with double
 * accumulation. */
void orc_conv2d_f64(const float *x, const float *w, const float *bias, double *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW)
{
	int oW = orc_conv_outsize(W, kW, dW, padW);
	int oH = orc_conv_outsize(H, kH, dH, padH);
	long bo;
#pragma omp parallel for
	for (bo = 0; bo < (long)B * Co; bo++) {
		int b = (int)(bo / Co), o = (int)(bo % Co);
		for (int oy = 0; oy < oH; oy++)
			for (int ox = 0; ox < oW; ox++) {
				double acc = bias ? bias[o] : 0.0;
				for (int c = 0; c < Ci; c++)
					for (int kh = 0; kh < kH; kh++) {
						int iy = oy * dH - padH + kh;
						if (iy < 0 || iy >= H)
							continue;
						for (int kw = 0; kw < kW; kw++) {
							int ix = ox * dW - padW + kw;
							if (ix < 0 || ix >= W)
								continue;
							acc += (double)w[((long)(o * Ci + c) * kH + kh) * kW + kw] *
								x[(((long)b * Ci + c) * H + iy) * W + ix];
						}
					}
				y[((bo * oH) + oy) * oW + ox] = acc;
			}
	}
}

/* ------------------------------------------------------------------ */
/* fp32 Linear                                                         */
/* ------------------------------------------------------------------ */

/* 1-D branch of nn_Linear_updateOutput, modules/Linear.c:86-90: output = bias,
 * then addmv -> sgemv('t') -> sgemv_t (OpenBLAS-stripped/gemv_t.c:51-63):
 * a strictly sequential fp32 dot per row, y[j] += 1 * temp. */
void orc_linear1d_f32(const float *x, const float *w, const float *bias, float *y, int nIn, int nOut)
{
	int j;
#pragma omp parallel for
	for (j = 0; j < nOut; j++) {
		const float *a = w + (long)j * nIn;
		float temp = 0.0f;
		for (int i = 0; i < nIn; i++)
			temp += a[i] * x[i];
		float yj = bias ? bias[j] : 0.0f;
		yj += 1.0f * temp;
		y[j] = yj;
	}
}

/* 2-D branch, modules/Linear.c:92-108: Y = X * W^T with beta = 0, then the
 * rank-1 update Y += ones * bias^T (thbasic.c:757-789 -> sger.c:55-61). */
void orc_linear2d_f32(const float *x, const float *w, const float *bias, float *y, int B, int nIn, int nOut)
{
	int j;
#pragma omp parallel for
	for (j = 0; j < nOut; j++) {
		const float *a = w + (long)j * nIn;
		for (int b = 0; b < B; b++) {
			const float *xb = x + (long)b * nIn;
			float acc[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
			int i = 0;
			for (; i + 8 <= nIn; i += 8)
				for (int l = 0; l < 8; l++)
					acc[l] += a[i + l] * xb[i + l];
			float s = ((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]));
			for (; i < nIn; i++)
				s += a[i] * xb[i];
			y[(long)b * nOut + j] = s + (bias ? 1.0f * bias[j] : 0.0f);
		}
	}
}

/* ------------------------------------------------------------------ */
/* fp32 element-wise and pooling modules                               */
/* ------------------------------------------------------------------ */

/* nn_Threshold_updateOutput, modules/Threshold.c:38-63.  In place: x <= thr
 * becomes val.  Out of place: alpha != 0 selects x >= 0 ? x : x*alpha, else
 * x > thr ? x : val. */
void orc_threshold_f32(const float *x, float *y, long n, float thr, float val, float alpha, int inplace)
{
	long i;
	if (inplace) {
		for (i = 0; i < n; i++)
			y[i] = x[i] <= thr ? val : x[i];
	} else if (alpha) {
		for (i = 0; i < n; i++)
			y[i] = x[i] >= 0 ? x[i] : x[i] * alpha;
	} else {
		for (i = 0; i < n; i++)
			y[i] = x[i] > thr ? x[i] : val;
	}
}

/* Output extent of max / average pooling, modules/SpatialMaxPooling.c:187-203
 * (same rule in SpatialAveragePooling.c:121-140): float division, floor or
 * ceil, then drop a last window that would start past the padded input. */
void orc_pool_outsize(int H, int W, int kH, int kW, int dH, int dW, int padH, int padW, int ceil_mode,
	int *oH, int *oW)
{
	long oh, ow;
	if (ceil_mode) {
		oh = (long)(ceil((float)(H - kH + 2 * padH) / dH)) + 1;
		ow = (long)(ceil((float)(W - kW + 2 * padW) / dW)) + 1;
	} else {
		oh = (long)(floor((float)(H - kH + 2 * padH) / dH)) + 1;
		ow = (long)(floor((float)(W - kW + 2 * padW) / dW)) + 1;
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

/* nn_SpatialMaxPooling_updateOutput_frame, modules/SpatialMaxPooling.c:73-120:
 * window clipped to the image, start value -FLT_MAX, strict '>' (first
 * maximum wins). */
void orc_maxpool_f32(const float *x, float *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW)
{
	long p;
#pragma omp parallel for
	for (p = 0; p < (long)B * C; p++) {
		const float *ip = x + p * H * W;
		float *op = y + p * oH * oW;
		for (int i = 0; i < oH; i++)
			for (int j = 0; j < oW; j++) {
				long hs = (long)i * dH - padH, ws = (long)j * dW - padW;
				long he = ORC_MIN(hs + kH, (long)H), we = ORC_MIN(ws + kW, (long)W);
				hs = ORC_MAX(hs, 0L);
				ws = ORC_MAX(ws, 0L);
				float m = -3.402823466e+38F;
				for (long yy = hs; yy < he; yy++)
					for (long xx = ws; xx < we; xx++) {
						float v = ip[yy * W + xx];
						if (v > m)
							m = v;
					}
				op[(long)i * oW + j] = m;
			}
	}
}

/* The same with the float `indices` the reference keeps for unpooling
 * (modules/SpatialMaxPooling.c:100-114): position of the first maximum inside
 * the input plane, plus one; 0 when the window is empty. */
void orc_maxpool_indices_f32(const float *x, float *y, float *ind, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW)
{
	long p;
#pragma omp parallel for
	for (p = 0; p < (long)B * C; p++) {
		const float *ip = x + p * H * W;
		float *op = y + p * oH * oW, *np = ind + p * oH * oW;
		for (int i = 0; i < oH; i++)
			for (int j = 0; j < oW; j++) {
				long hs = (long)i * dH - padH, ws = (long)j * dW - padW;
				long he = ORC_MIN(hs + kH, (long)H), we = ORC_MIN(ws + kW, (long)W);
				hs = ORC_MAX(hs, 0L);
				ws = ORC_MAX(ws, 0L);
				float m = -INFINITY;
				long at = -1;
				for (long yy = hs; yy < he; yy++)
					for (long xx = ws; xx < we; xx++) {
						float v = ip[yy * W + xx];
						if (v > m) {
							m = v;
							at = yy * W + xx;
						}
					}
				op[(long)i * oW + j] = m;
				np[(long)i * oW + j] = (float)(at + 1);
			}
	}
}

/* nn_SpatialMaxUnpooling_updateOutput, modules/SpatialMaxUnpooling.c:14-41,
 * 92-119: the output plane (the pooling's input extent) is zeroed, then every
 * input element is written at the position its index names, in row-major
 * order, so of several elements with one index the last one stays.  Returns -1
 * for an index outside the plane (the reference calls THError). */
int orc_maxunpool_f32(const float *x, const float *ind, float *y, int B, int C, int iH, int iW, int oH, int oW)
{
	int bad = 0;
	memset(y, 0, sizeof(float) * (size_t)B * C * oH * oW);
	long p;
#pragma omp parallel for
	for (p = 0; p < (long)B * C; p++) {
		const float *ip = x + p * iH * iW, *np = ind + p * iH * iW;
		float *op = y + p * oH * oW;
		for (long e = 0; e < (long)iH * iW; e++) {
			long at = (long)np[e] - 1;
			if (at < 0 || at >= (long)oH * oW)
				bad = 1;
			else
				op[at] = ip[e];
		}
	}
	return bad ? -1 : 0;
}

/* nn_SpatialFullConvolution_updateOutput, modules/SpatialFullConvolution.c:136-250:
 * per image columns = W^T x (W is [Ci][Co*kH*kW]), col2im (:104-134) adds
 * columns[(o*kH+kh)*kW+kw][iy*W+ix] into out[o][iy*dH-padH+kh][ix*dW-padW+kw],
 * then the bias GEMM.  That GEMM is called with beta = 11 (:231-237), so with a
 * bias the result is 11 * (transposed convolution) + bias; without one the
 * transposed convolution itself.  oH = (H-1)*dH - 2*padH + kH + adjH. */
void orc_fullconv2d_f32(const float *x, const float *w, const float *bias, float *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int adjH, int adjW)
{
	const int oH = (H - 1) * dH - 2 * padH + kH + adjH, oW = (W - 1) * dW - 2 * padW + kW + adjW;
	const long M = (long)Co * kH * kW, N = (long)H * W;
	float *col = malloc(sizeof(float) * M * N);
	for (int b = 0; b < B; b++) {
		const float *xb = x + (long)b * Ci * N;
		float *yb = y + (long)b * Co * oH * oW;
		long m;
#pragma omp parallel for
		for (m = 0; m < M; m++)
			for (long n = 0; n < N; n++) {
				float acc = 0;
				for (int c = 0; c < Ci; c++)
					acc += w[(long)c * M + m] * xb[(long)c * N + n];
				col[m * N + n] = acc;
			}
		memset(yb, 0, sizeof(float) * (size_t)Co * oH * oW);
		for (m = 0; m < M; m++) {
			const int kw = (int)(m % kW), kh = (int)(m / kW % kH), o = (int)(m / kW / kH);
			for (int iy = 0; iy < H; iy++)
				for (int ix = 0; ix < W; ix++) {
					const int oy = iy * dH - padH + kh, ox = ix * dW - padW + kw;
					if (oy >= 0 && oy < oH && ox >= 0 && ox < oW)
						yb[((long)o * oH + oy) * oW + ox] += col[m * N + (long)iy * W + ix];
				}
		}
		if (bias)
			for (int o = 0; o < Co; o++)
				for (long e = 0; e < (long)oH * oW; e++)
					yb[(long)o * oH * oW + e] = 11.0f * yb[(long)o * oH * oW + e] + bias[o];
	}
	free(col);
}

/* The transposed convolution in double precision, scatter form straight from
 * the definition (no columns, no bias rule): for checks against the above. */
void orc_fullconv2d_f64(const float *x, const float *w, double *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int adjH, int adjW)
{
	const int oH = (H - 1) * dH - 2 * padH + kH + adjH, oW = (W - 1) * dW - 2 * padW + kW + adjW;
	memset(y, 0, sizeof(double) * (size_t)B * Co * oH * oW);
	for (int b = 0; b < B; b++)
		for (int c = 0; c < Ci; c++)
			for (int iy = 0; iy < H; iy++)
				for (int ix = 0; ix < W; ix++) {
					const double v = x[(((long)b * Ci + c) * H + iy) * W + ix];
					for (int o = 0; o < Co; o++)
						for (int kh = 0; kh < kH; kh++)
							for (int kw = 0; kw < kW; kw++) {
								const int oy = iy * dH - padH + kh, ox = ix * dW - padW + kw;
								if (oy >= 0 && oy < oH && ox >= 0 && ox < oW)
									y[(((long)b * Co + o) * oH + oy) * oW + ox] +=
										v * w[(((long)c * Co + o) * kH + kh) * kW + kw];
							}
				}
}

/* nn_SpatialAveragePooling_updateOutput, modules/SpatialAveragePooling.c:156-203:
 * pool_size is measured on the padded extent, the sum on the clipped one;
 * divide by pool_size when count_include_pad, else by the clipped count.
 * kW == 0 / kH == 0 mean "whole input" (:116-119) and are resolved by the
 * caller. */
void orc_avgpool_f32(const float *x, float *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int count_include_pad)
{
	long p;
#pragma omp parallel for
	for (p = 0; p < (long)B * C; p++) {
		const float *ip = x + p * H * W;
		float *op = y + p * oH * oW;
		for (int yy = 0; yy < oH; yy++)
			for (int xx = 0; xx < oW; xx++) {
				long hs = (long)yy * dH - padH, ws = (long)xx * dW - padW;
				long he = ORC_MIN(hs + kH, (long)H + padH), we = ORC_MIN(ws + kW, (long)W + padW);
				long pool = (he - hs) * (we - ws);
				hs = ORC_MAX(hs, 0L);
				ws = ORC_MAX(ws, 0L);
				he = ORC_MIN(he, (long)H);
				we = ORC_MIN(we, (long)W);
				float sum = 0;
				long div = count_include_pad ? pool : (he - hs) * (we - ws);
				for (long ky = hs; ky < he; ky++)
					for (long kx = ws; kx < we; kx++)
						sum += ip[ky * W + kx];
				op[(long)yy * oW + xx] = 0.0f + sum / div;
			}
	}
}

/* THExpMinusApprox, thbasic.c:462-491: 1/(1+x/8+x^2/128+...)^8 for x < 13,
 * else 0.  The coefficients are the published constants of that routine. */
double orc_exp_minus_approx(double x)
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

/* nn_SoftMax_updateOutput, modules/SoftMax.c:24-90: per (frame, position):
 * max with '>=' from -FLT_MAX, z = approx(max - x) stored as float, float
 * running sum, then every z multiplied by the float 1/sum. */
void orc_softmax_f32(const float *x, float *y, long nframe, long dim, long stride)
{
	long t;
#pragma omp parallel for
	for (t = 0; t < stride * nframe; t++) {
		const float *ip = x + (t / stride) * dim * stride + t % stride;
		float *op = y + (t / stride) * dim * stride + t % stride;
		float m = -3.402823466e+38F, sum = 0;
		for (long d = 0; d < dim; d++)
			if (ip[d * stride] >= m)
				m = ip[d * stride];
		for (long d = 0; d < dim; d++) {
			float z = (float)orc_exp_minus_approx(m - ip[d * stride]);
			op[d * stride] = z;
			sum += z;
		}
		for (long d = 0; d < dim; d++)
			op[d * stride] *= 1 / sum;
	}
}

/* nn_SpatialBatchNormalization_updateOutput,
 * modules/SpatialBatchNormalization.c:57-116: invstd = 1/sqrt(var+eps) in
 * double narrowed to float; y = ((x - mean) * invstd) * w + b. */
void orc_batchnorm_f32(const float *x, float *y, long B, long C, long HW,
	const float *mean, const float *var, const float *weight, const float *bias, double eps)
{
	long bc;
#pragma omp parallel for
	for (bc = 0; bc < B * C; bc++) {
		long f = bc % C;
		float mu = mean[f];
		float invstd = (float)(1 / sqrt(var[f] + eps));
		float w = weight ? weight[f] : 1, b = bias ? bias[f] : 0;
		for (long i = 0; i < HW; i++)
			y[bc * HW + i] = ((x[bc * HW + i] - mu) * invstd) * w + b;
	}
}

/* nn_CAddTable_updateOutput, modules/CAddTable.c:32-86, arithmetic exactly as
 * shipped.  Two inputs: MT_CAddTable computes a - b and MT_CSubTable a + b
 * over n[1] elements, the remaining n[0]-n[1] are copied from a (:59-70).
 * More inputs: out = a, then every input INCLUDING the first is added
 * (subtracted for CSubTable) again (:71-84). */
void orc_caddtable_f32(int is_csubtable, int nelem, const float **ins, const long *n, float *out)
{
	long j;
	if (nelem == 2) {
		if (is_csubtable)
			for (j = 0; j < n[1]; j++)
				out[j] = ins[0][j] + ins[1][j];
		else
			for (j = 0; j < n[1]; j++)
				out[j] = ins[0][j] - ins[1][j];
		for (; j < n[0]; j++)
			out[j] = ins[0][j];
	} else {
		for (j = 0; j < n[0]; j++)
			out[j] = ins[0][j];
		for (int i = 0; i < nelem; i++)
			for (j = 0; j < n[i]; j++) {
				if (is_csubtable)
					out[j] -= ins[i][j];
				else
					out[j] += ins[i][j];
			}
	}
}

/* Input normalisation of THProcessFloat, thapi.c:397-402 (plane-major
 * branch): data = (data - mean[c]) / std[c], in place. */
void orc_normalize_f32(float *data, int B, int C, long HW, const float *mean, const float *std)
{
	for (int b = 0; b < B; b++)
		for (int c = 0; c < C; c++)
			for (long i = 0; i < HW; i++) {
				float *p = data + ((long)b * C + c) * HW + i;
				*p = (*p - mean[c]) / std[c];
			}
}

/* rgb2float / bgr2float, thapi.c:20-46: dst planar, src interleaved with
 * `stride` bytes per row; (byte * (1/255 as the float 0.003921568) - mean) *
 * (1/std). */
void orc_rgb2float(float *dst, const unsigned char *src, int width, int height, int stride, int cp,
	const float *mean, const float *std, int bgr)
{
	for (int c = 0; c < cp; c++) {
		float std1 = 1 / std[c];
		int sc = bgr ? cp - 1 - c : c;
		for (int i = 0; i < height; i++)
			for (int j = 0; j < width; j++)
				dst[j + ((long)i + (long)c * height) * width] =
					(src[sc + cp * j + (long)stride * i] * 0.003921568f - mean[c]) * std1;
	}
}

/* ------------------------------------------------------------------ */
/* LOWP (uint8) path                                                   */
/* ------------------------------------------------------------------ */

/* THLowpTensor_newFromFloatTensor, lowp/lowp_basic.c:15-35: min and max start
 * at 0; mult = 255.0/(max-min) evaluated in double and narrowed; each value is
 * roundf(v*mult) - roundf(min*mult) in float, narrowed to a byte.  The
 * narrowing of an out-of-range float (256 can occur) is undefined in C; x86-64
 * gcc converts through a 32-bit integer and keeps the low byte, which is what
 * is restated here. */
void orc_lowp_quantize(const float *x, long n, unsigned char *q, float *mult_out, float *sub_out)
{
	float mn = 0, mx = 0, mult;
	long i;
	for (i = 0; i < n; i++) {
		if (x[i] < mn)
			mn = x[i];
		if (x[i] > mx)
			mx = x[i];
	}
	if (mx - mn > 0)
		mult = (float)(255.0 / (mx - mn));
	else
		mult = 0;
	float zero = roundf(mn * mult);
	for (i = 0; i < n; i++)
		q[i] = (unsigned char)(int)(roundf(x[i] * mult) - zero);
	*sub_out = mn;
	*mult_out = mult;
}

/* THFloatTensor_newFromLowpTensor, lowp/lowp_basic.c:40-58: invmult is
 * 1.0/mult narrowed to float; v = q*invmult + sub as separate float ops. */
void orc_lowp_dequantize(const unsigned char *q, long n, float mult, float sub, float *x)
{
	float invmult = mult ? (float)(1.0 / mult) : 0;
	for (long i = 0; i < n; i++) {
		float prod = q[i] * invmult;
		x[i] = prod + sub;
	}
}

/* THLowp_ScaleFloat, lowp/lowp_basic.c:214-222: clamp then truncate. */
unsigned char orc_lowp_scale_float(float mult, float sub, float value)
{
	float scaled = (value - sub) * mult;
	if (scaled < 0)
		return 0;
	if (scaled > 255)
		return 255;
	return (unsigned char)scaled;
}

/* Parameter derivation of THLowpTensor_mm, lowp/lowp_basic.c:309-320.
 * (wm, wsub) weight, (im, isub) im2col input, (om, osub) output.
 * out[0..4] = a_off, b_off, c_off, c_mult, c_shift as the ints the callee
 * receives. */
void orc_lowp_mm_params(float wm, float wsub, float im, float isub, float om, float osub, int *out)
{
	float scaling = wm * im / om;
	int shift = roundf((log(scaling) / log(2))) + 10;
	int mult = roundf((1 << shift) / scaling);
	int offset = roundf(-osub * wm * im);
	out[0] = roundf(wsub * wm);
	out[1] = roundf(isub * im);
	out[2] = offset;
	out[3] = mult;
	out[4] = shift;
}

/* Bias addend of the lowp convolution, lowp/lowp_SpatialConvolution.c:112-119:
 * roundf(code * (om/bm)) + roundf(bsub*om), both in float then summed as int. */
int orc_lowp_bias_addend(unsigned char bq, float bm, float bsub, float om)
{
	float mult = om / bm;
	int add = roundf(bsub * om);
	int addend = bq;
	addend = roundf(addend * mult) + add;
	return addend;
}

/* gemmlowp EightBitIntGemm(A8B8) with all three matrices "transposed", i.e.
 * row-major A[m][k], B[k][n], C[m][n], as called from lowp/gemm8.cc:13-16.
 * Published legacy contract (gemmlowp public/output_stages.h,
 * OutputStageQuantizeDownInt32ToUint8Scale then SaturatingCastToUint8):
 *   acc = sum_l (A[i][l]+a_off) * (B[l][j]+b_off)           (int32)
 *   t   = (acc + c_off) * c_mult + (c_shift < 1 ? 0 : 1 << (c_shift-1))
 *         in wrapping 32-bit arithmetic
 *   C   = clamp(t >> c_shift, 0, 255)                       (arithmetic shift)
 * PARITY UNPINNED against the reference (see file header). */
static inline unsigned char orc_requant(int32_t acc, int c_off, int c_mult, int c_shift)
{
	uint32_t u = ((uint32_t)acc + (uint32_t)c_off) * (uint32_t)c_mult;
	u += c_shift < 1 ? 0u : (uint32_t)1 << (c_shift - 1);
	int32_t t = (int32_t)u;
	t >>= c_shift;
	return (unsigned char)(t < 0 ? 0 : t > 255 ? 255 : t);
}

unsigned char orc_lowp_requant(int acc, int c_off, int c_mult, int c_shift)
{
	return orc_requant(acc, c_off, c_mult, c_shift);
}

void orc_lowp_gemm(int m, int n, int k, const unsigned char *a, const unsigned char *b, unsigned char *c,
	int lda, int ldb, int ldc, int a_off, int b_off, int c_off, int c_mult, int c_shift)
{
	int i;
#pragma omp parallel for if(!omp_in_parallel())
	for (i = 0; i < m; i++) {
		int32_t *acc = (int32_t *)calloc(n, sizeof(int32_t));
		for (int l = 0; l < k; l++) {
			int32_t av = (int32_t)a[(long)i * lda + l] + a_off;
			const unsigned char *br = b + (long)l * ldb;
			for (int j = 0; j < n; j++)
				acc[j] += av * ((int32_t)br[j] + b_off);
		}
		for (int j = 0; j < n; j++)
			c[(long)i * ldc + j] = orc_requant(acc[j], c_off, c_mult, c_shift);
		free(acc);
	}
}

/* uint8 im2col, lowp/lowp_SpatialConvolution.c:5-69: as the float one but
 * padding is the byte `zero`. */
void orc_lowp_unfold(const unsigned char *x, unsigned char *col, int Ci, int H, int W, int kH, int kW,
	int dH, int dW, int padH, int padW, int oH, int oW, unsigned char zero)
{
	long K = (long)Ci * kH * kW;
	for (long k = 0; k < K; k++) {
		int c = (int)(k / (kH * kW));
		int rest = (int)(k % (kH * kW));
		int kh = rest / kW, kw = rest % kW;
		unsigned char *dst = col + k * (long)oH * oW;
		const unsigned char *src = x + (long)c * H * W;
		for (int y = 0; y < oH; y++) {
			long iy = (long)y * dH - padH + kh;
			for (int xx = 0; xx < oW; xx++) {
				long ix = (long)xx * dW - padW + kw;
				dst[(long)y * oW + xx] =
					(iy < 0 || iy >= H || ix < 0 || ix >= W) ? zero : src[iy * W + ix];
			}
		}
	}
}

/* lowpadd, lowp/lowp_SpatialConvolution.c:71-88: blocks of eight saturate at
 * both ends; the remaining len%8 elements saturate only above, so a negative
 * sum keeps its low byte. */
void orc_lowp_add(unsigned char *dst, int add, int len)
{
	int i;
	for (i = 0; i < len - 7; i += 8)
		for (int l = 0; l < 8; l++) {
			int s = dst[i + l] + add;
			dst[i + l] = (unsigned char)(s > 255 ? 255 : s < 0 ? 0 : s);
		}
	for (; i < len; i++) {
		int s = dst[i] + add;
		dst[i] = (unsigned char)(s > 255 ? 255 : s);
	}
}

/* Lowp_SpatialConvolution_updateOutput, lowp/lowp_SpatialConvolution.c:90-187,
 * for a batch addressed correctly image by image (the shipped code is only
 * correct at batch 1; each image here goes through exactly the batch-1
 * arithmetic).  wq [Co][K] codes with (wm, wsub); bq [Co] codes with
 * (bm, bsub); x codes with (im, isub); output codes in (om, osub).
 * zero = roundf(-isub*im) (:101). */
int orc_lowp_conv2d(const unsigned char *x, float im, float isub,
	const unsigned char *wq, float wm, float wsub,
	const unsigned char *bq, float bm, float bsub,
	unsigned char *y, float om, float osub,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW)
{
	int oW = orc_conv_outsize(W, kW, dW, padW);
	int oH = orc_conv_outsize(H, kH, dH, padH);
	if (oW < 1 || oH < 1)
		return -1;
	int K = Ci * kH * kW;
	long N = (long)oH * oW;
	int prm[5];
	orc_lowp_mm_params(wm, wsub, im, isub, om, osub, prm);
	int zero = roundf(-isub * im);
	int t;
#pragma omp parallel for
	for (t = 0; t < B; t++) {
		unsigned char *col = (unsigned char *)malloc((size_t)K * N);
		unsigned char *yi = y + (long)t * Co * N;
		orc_lowp_unfold(x + (long)t * Ci * H * W, col, Ci, H, W, kH, kW, dH, dW, padH, padW, oH, oW,
			(unsigned char)zero);
		orc_lowp_gemm(Co, (int)N, K, wq, col, yi, K, (int)N, (int)N, prm[0], prm[1], prm[2], prm[3], prm[4]);
		for (int o = 0; o < Co; o++)
			orc_lowp_add(yi + (long)o * N, orc_lowp_bias_addend(bq[o], bm, bsub, om), (int)N);
		free(col);
	}
	return 0;
}

/* Lowp_Threshold_updateOutput, lowp/lowp_Threshold.c:3-28 on codes. */
void orc_lowp_threshold(const unsigned char *x, unsigned char *y, long n, unsigned char thr, unsigned char val,
	int inplace)
{
	long i;
	if (inplace)
		for (i = 0; i < n; i++)
			y[i] = x[i] <= thr ? val : x[i];
	else
		for (i = 0; i < n; i++)
			y[i] = x[i] > thr ? x[i] : val;
}

/* Lowp_SpatialMaxPooling_updateOutput_frame, lowp/lowp_SpatialMaxPooling.c:4-43:
 * start value 0. */
void orc_lowp_maxpool(const unsigned char *x, unsigned char *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW)
{
	long p;
#pragma omp parallel for
	for (p = 0; p < (long)B * C; p++) {
		const unsigned char *ip = x + p * H * W;
		unsigned char *op = y + p * oH * oW;
		for (int i = 0; i < oH; i++)
			for (int j = 0; j < oW; j++) {
				long hs = (long)i * dH - padH, ws = (long)j * dW - padW;
				long he = ORC_MIN(hs + kH, (long)H), we = ORC_MIN(ws + kW, (long)W);
				hs = ORC_MAX(hs, 0L);
				ws = ORC_MAX(ws, 0L);
				unsigned char m = 0;
				for (long yy = hs; yy < he; yy++)
					for (long xx = ws; xx < we; xx++)
						if (ip[yy * W + xx] > m)
							m = ip[yy * W + xx];
				op[(long)i * oW + j] = m;
			}
	}
}

/* Lowp_SoftMax_updateOutput, lowp/lowp_SoftMax.c:3-89, run sequentially (the
 * shipped loop shares one scratch row between OpenMP threads).  Note the
 * argument of the exponential keeps the tensor offset:
 * approx((max-q)*invmult + sub).  Returns the output mult; output sub is 0. */
float orc_lowp_softmax(const unsigned char *x, unsigned char *y, long nframe, long dim, long stride,
	float in_mult, float in_sub)
{
	float invmult = in_mult ? 1 / in_mult : 0;
	float *tmp = (float *)malloc(dim * sizeof(*tmp));
	float out_mult = 0;
	for (long t = 0; t < stride * nframe; t++) {
		const unsigned char *ip = x + (t / stride) * dim * stride + t % stride;
		unsigned char *op = y + (t / stride) * dim * stride + t % stride;
		unsigned char qmax = 0;
		float sum = 0, max;
		long d;
		for (d = 0; d < dim; d++)
			if (ip[d * stride] >= qmax)
				qmax = ip[d * stride];
		for (d = 0; d < dim; d++) {
			float arg = (qmax - ip[d * stride]) * invmult;
			arg = arg + in_sub;
			tmp[d] = (float)orc_exp_minus_approx(arg);
			sum += tmp[d];
		}
		if (stride * nframe > 1) {
			for (d = 0; d < dim; d++)
				tmp[d] *= 1 / sum;
			for (d = 0; d < dim; d++)
				op[d * stride] = (unsigned char)(int)(255 * tmp[d]);
		} else {
			max = 0;
			for (d = 0; d < dim; d++) {
				tmp[d] *= 1 / sum;
				if (tmp[d] > max)
					max = tmp[d];
			}
			for (d = 0; d < dim; d++) {
				float v = 255 * tmp[d];
				v = v * (1 / max);
				op[d * stride] = (unsigned char)(int)v;
			}
			out_mult = 255 / max;
		}
	}
	free(tmp);
	if (stride * nframe > 1)
		out_mult = 255;
	return out_mult;
}

/* Lowp_LoadImages, lowp/lowp_basic.c:82-131 with rgb2tensord/bgr2tensord
 * :60-80: a fixed input range from mean/std, then
 * byte = roundf((src - sub[c]) * mult[c]).  Returns mult/sub of the tensor. */
void orc_lowp_load_images(unsigned char *dst, const unsigned char *const *src, int nimages, int width, int height,
	int stride, const float *mean, const float *std, int bgr, float *mult_out, float *sub_out)
{
	int sub[3];
	float mult[3], mn = 1e30, mx = -1e30, tsub, tmult;
	for (int i = 0; i < 3; i++) {
		if (-mean[i] / std[i] < mn)
			mn = -mean[i] / std[i];
		if ((1 - mean[i]) / std[i] > mx)
			mx = (1 - mean[i]) / std[i];
	}
	tsub = mn;
	tmult = (mx - mn) ? 255 / (mx - mn) : 0;
	for (int i = 0; i < 3; i++) {
		sub[i] = roundf(255 * (mean[i] + std[i] * tsub));
		mult[i] = tmult / (255 * std[i]);
	}
	for (int n = 0; n < nimages; n++)
		for (int c = 0; c < 3; c++)
			for (int i = 0; i < height; i++)
				for (int j = 0; j < width; j++) {
					int sc = bgr ? 2 - c : c;
					float v = roundf((src[n][sc + 3 * j + (long)stride * i] - sub[c]) * mult[c]);
					dst[(long)n * 3 * width * height + j + ((long)i + (long)c * height) * width] =
						(unsigned char)(int)v;
				}
	*mult_out = tmult;
	*sub_out = tsub;
}
