/*
 * The image layer of a ResNet-style fp32 network with what follows it, in one kernel:
 *
 *   SpatialConvolution(<= 4 planes -> 64 n planes, e.g. 7x7, stride 2, padding 3) on plane-major input
 *   (modules/SpatialConvolutionMM.c:126-225: im2col + sgemm + bias), the batch norm folded into its
 *   epilogue (modules/SpatialBatchNormalization.c:57-116 as a factor and a shift per plane), the
 *   Threshold (modules/Threshold.c:38-63) and SpatialMaxPooling 3x3 / stride 2 with padding 0 or 1
 *   in floor mode (modules/SpatialMaxPooling.c:168-247).
 *
 * As an implicit GEMM the layer gathers every operand element by element with a tap decode per
 * element (3 planes are no whole block of anything), writes 64 planes per pixel (103 MB at
 * batch 32) and the pooling reads them back.  Here a workgroup owns 8 x 14 pooled positions of
 * one image and 64 output planes, i.e. up to 17 x 29 = 493 convolution positions (16 MFMA tiles
 * of 32):
 *  1. The input patch those positions read goes into LDS once (three planes of 39 rows x 63
 *     columns for a 7x7 / stride 2 kernel; elements outside the image arrive as zeros), the
 *     weights of the 64 planes beside it in the order the matrix core reads them, and a table
 *     with the patch offset of every k = (plane, kernel row, kernel column).
 *  2. Eight wavefronts take two position tiles each; two workgroups share a CU, so that one
 *     multiplies while the other loads its patch or pools (measured at batch 32: 116 us; four
 *     wavefronts of four tiles, two workgroups a CU: 126 us; eight wavefronts, one workgroup a
 *     CU: 137 us; the generic kernel followed by the pooling kernel: 132 us).  A step of the K
 *     loop is two values of k (the two lane halves of v_mfma_f32_32x32x2_f32): per lane one
 *     8-byte read for the A values of both row blocks, one table entry, two B values at
 *     (position base) + (table entry), four MFMAs.
 *  3. Epilogue, one block of 32 planes at a time: factor, shift and Threshold, the values into LDS
 *     (over patch and weights, which are done with) as [plane][position] - convolution
 *     positions outside the output (the pooling's padding) as -FLT_MAX - and every thread takes
 *     the maximum of 3x3 windows and writes the pooled plane-major result.
 *
 * The convolution's output is never written.  Sums run over k in the reference's order
 * (plane, kernel row, kernel column), two partial sums of alternate k per output.
 */
#include <float.h>
#include "thhip_internal.h"

#define FI_THREADS 512
#define FI_WAVES 8
#define FI_TPW 2		/* position tiles per wavefront */
#define FI_PR 8		/* pooled rows per workgroup */
#define FI_PC 14	/* pooled columns per workgroup: (2 * 8 + 1) * (2 * 14 + 1) = 493 <= 512 positions */
#define FI_MAXPOS 512
#define FI_LDS_MAX (150 * 1024)

struct ConvImgF32Params {
	const float *x;		/* [B][Ci][H][W] */
	const float *wp;	/* packed for plane-major input: [32-row block][KC chunks of 8][k half][32 rows][4] */
	const float *bias, *scale;
	float *y;		/* [B][Co][pH][pW] */
	int B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, oH, oW, pH, pW, ppad;
	int KC, K, nsteps;
	int prows, pw;		/* rows of a plane's patch, elements per patch row */
	int front;		/* bytes of LDS shared by patch + weights and, later, the values to pool */
	unsigned m_cwl, m_pw, m_pca;	/* x / d == __umulhi(x, m_d) for the small x used here */
	int act;
	float thr, val;
};

__device__ __forceinline__ int fi_div(int x, unsigned magic)
{
	return magic ? (int)__umulhi((unsigned)x, magic) : x;
}

/* two workgroups per CU (their LDS allows no more): 128 registers per lane */
__global__ __launch_bounds__(FI_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void conv_f32_image_pool_kernel(ConvImgF32Params p)
{
	extern __shared__ __align__(16) unsigned char lds[];
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int n = lane & 31, h = lane >> 5;
	const int pc0 = blockIdx.x * FI_PC, pr0 = blockIdx.y * FI_PR;
	const int zgroups = p.Co / 64;
	const int b = blockIdx.z / zgroups, mz = blockIdx.z - b * zgroups;
	const int pra = min(FI_PR, p.pH - pr0), pca = min(FI_PC, p.pW - pc0);	/* pooled rows / columns of this workgroup */
	const int chl = 2 * pra + 1, cwl = 2 * pca + 1;				/* its convolution rows / columns */
	const int npos = chl * cwl;
	const int cy0 = 2 * pr0 - p.ppad, cx0 = 2 * pc0 - p.ppad;		/* convolution position of local (0, 0) */
	/* LDS: patch | weights [step][k half][row][2 blocks]   (later: values [32 planes][npos])
	 *      | k table [2 nsteps] | shift[64], factor[64] */
	const int patch_elems = p.Ci * p.prows * p.pw;
	float *const patch = (float *)lds;
	float *const wl = patch + patch_elems;
	int *const ktab = (int *)(lds + p.front);
	float *const rowc = (float *)(ktab + 2 * p.nsteps);

	/* ---- 1. the patch: row r of plane c is input row iy0 + r, element e of a row input column ix0 + e;
	 * eight loads in flight per thread ---- */
	{
		const int iy0 = cy0 * p.dH - p.padH, ix0 = cx0 * p.dW - p.padW;
		const int rows = (chl - 1) * p.dH + p.kH;
		/* this image's planes as a buffer: an offset past them reads as zero (the padding) */
		const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
			(void *)(p.x + (size_t)b * p.Ci * p.H * p.W), 0, p.Ci * p.H * p.W * 4, 0x00020000);
		/* the weights, four consecutive k of a row at a time: element (k, row nn, block mb) of the LDS copy is
		 * weight (row 32 mb + nn of this workgroup's 64, k); k >= K (the padding of the last chunk) is zero in
		 * the packed array.  They are requested first and stored last: patch and weights make one trip to
		 * memory together (every trip a thread waits for is a microsecond the matrix core idles). */
		constexpr int WV = 5, PV = 15;
		const int wquads = ((2 * p.nsteps + 3) / 4) * 64;	/* (k quad, block, row) */
		floatx4 wv[WV];
#pragma unroll
		for (int u = 0; u < WV; u++) {
			const int e = min(u * FI_THREADS + tid, wquads - 1);
			const int nn = e & 31, mb = (e >> 5) & 1, kq = e >> 6;
			wv[u] = *(const floatx4 *)(p.wp + ((((size_t)(mz * 2 + mb) * p.KC + (kq >> 1)) * 2 + (kq & 1)) * 32 + nn) * 4);
		}
		for (int e0 = 0; e0 < patch_elems; e0 += PV * FI_THREADS) {
			float v[PV];
#pragma unroll
			for (int u = 0; u < PV; u++) {
				const int e = e0 + u * FI_THREADS + tid;
				const int r = fi_div(e, p.m_pw), pc = e - r * p.pw;	/* row of the whole patch, column */
				int c = 0, pr = r;
				while (pr >= p.prows) {	/* (at most Ci - 1 <= 3 turns) */
					pr -= p.prows;
					c++;
				}
				const int iy = iy0 + pr, ix = ix0 + pc;
				const bool in = e < patch_elems && pr < rows && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W;
				v[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xrsrc,
					in ? ((c * p.H + iy) * p.W + ix) * 4 : (int)0x80000000, 0, 0));
			}
#pragma unroll
			for (int u = 0; u < PV; u++) {
				const int e = e0 + u * FI_THREADS + tid;
				if (e < patch_elems)
					patch[e] = v[u];
			}
		}
#pragma unroll
		for (int u = 0; u < WV; u++) {
			const int e = u * FI_THREADS + tid;
			const int nn = e & 31, mb = (e >> 5) & 1, kq = e >> 6;
			if (e < wquads) {
#pragma unroll
				for (int i = 0; i < 4; i++)
					if (4 * kq + i < 2 * p.nsteps)
						wl[((4 * kq + i) * 32 + nn) * 2 + mb] = wv[u][i];
			}
		}
		/* where k = (plane, kernel row, kernel column) lies in the patch, relative to a position's base;
		 * k >= K: anywhere (its weight is zero and every patch value is finite or zero) */
		for (int k = tid; k < 2 * p.nsteps; k += FI_THREADS) {
			const int kk = min(k, p.K - 1);
			const int c = kk / (p.kH * p.kW), t = kk - c * p.kH * p.kW, kh = t / p.kW, kw = t - kh * p.kW;
			ktab[k] = ((c * p.prows + kh) * p.pw + kw) * 4;
		}
		if (tid < 64) {
			rowc[tid] = p.bias ? p.bias[mz * 64 + tid] : 0.0f;
			rowc[64 + tid] = p.scale ? p.scale[mz * 64 + tid] : 1.0f;
		}
	}
	__syncthreads();

	/* ---- 2. the K loop.  This lane's positions: tile FI_TPW wave + j, position n of it ---- */
	int pbase[FI_TPW];
#pragma unroll
	for (int j = 0; j < FI_TPW; j++) {
		const int pos = min((FI_TPW * wave + j) * 32 + n, npos - 1);
		const int ly = fi_div(pos, p.m_cwl), lx = pos - ly * cwl;
		pbase[j] = (ly * p.dH * p.pw + lx * p.dW) * 4;
	}
	floatx16 acc[FI_TPW][2];	/* [tile][row block] */
#pragma unroll
	for (int j = 0; j < FI_TPW; j++)
#pragma unroll
		for (int mb = 0; mb < 2; mb++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[j][mb][r] = 0.0f;
	{
		typedef float floatx2 __attribute__((ext_vector_type(2)));
		const unsigned char *pb = (const unsigned char *)patch;
		const floatx2 *wa = (const floatx2 *)wl + h * 32 + n;	/* + 64 per step */
		const int *kt = ktab + h;				/* + 2 per step */
		/* an odd K: k = K of the last step does not exist (its weight is zero, but the patch value read for
		 * it need not be finite) */
		const bool nok = (p.K & 1) && h;
		/* the table entry two steps ahead, the operands one step ahead */
		int ko2 = kt[2 * min(1, p.nsteps - 1)];
		floatx2 a = wa[0];
		float bv[FI_TPW];
		{
			const int ko1 = kt[0];
#pragma unroll
			for (int j = 0; j < FI_TPW; j++)
				bv[j] = nok && p.nsteps == 1 ? 0.0f : *(const float *)(pb + pbase[j] + ko1);
		}
		for (int s = 0; s < p.nsteps; s++) {
			const int sn = min(s + 1, p.nsteps - 1), sn2 = min(s + 2, p.nsteps - 1);
			const floatx2 an = wa[sn * 64];
			float bn[FI_TPW];
#pragma unroll
			for (int j = 0; j < FI_TPW; j++)
				bn[j] = *(const float *)(pb + pbase[j] + ko2);
			if (nok && sn == p.nsteps - 1) {
#pragma unroll
				for (int j = 0; j < FI_TPW; j++)
					bn[j] = 0.0f;
			}
			const int ko3 = kt[2 * sn2];
#pragma unroll
			for (int j = 0; j < FI_TPW; j++) {
				acc[j][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], bv[j], acc[j][0], 0, 0, 0);
				acc[j][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], bv[j], acc[j][1], 0, 0, 0);
			}
			a = an;
#pragma unroll
			for (int j = 0; j < FI_TPW; j++)
				bv[j] = bn[j];
			ko2 = ko3;
		}
	}
	__syncthreads();	/* patch and weights are done with */

	/* ---- 3. factor, shift, Threshold; the values of a block of 32 planes to LDS; pooling ---- */
	float *const cbuf = (float *)lds;	/* [32][npos] */
	const bool has_scale = p.scale != 0;
	const size_t plane_out = (size_t)p.pH * p.pW;
	for (int mb = 0; mb < 2; mb++) {
#pragma unroll
		for (int j = 0; j < FI_TPW; j++) {
			const int pos = (FI_TPW * wave + j) * 32 + n;
			const int posc = min(pos, npos - 1);
			const int ly = fi_div(posc, p.m_cwl), lx = posc - ly * cwl;
			const int cy = cy0 + ly, cx = cx0 + lx;
			const bool real = cy >= 0 && cy < p.oH && cx >= 0 && cx < p.oW;	/* else: the pooling's padding */
#pragma unroll
			for (int g = 0; g < 4; g++) {
				const int ml = 8 * g + 4 * h;	/* register 4 g + e is plane 8 g + 4 h + e of the block */
				const floatx4 rb = *(const floatx4 *)(rowc + mb * 32 + ml), rs = *(const floatx4 *)(rowc + 64 + mb * 32 + ml);
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const float a = mb ? acc[j][1][4 * g + e] : acc[j][0][4 * g + e];
					float v = has_scale ? a * rs[e] + rb[e] : a + rb[e];
					if (p.act)
						v = v > p.thr ? v : p.val;
					if (pos < npos)
						cbuf[(ml + e) * npos + posc] = real ? v : -FLT_MAX;
				}
			}
		}
		__syncthreads();
		/* eight threads a plane, neighbouring threads along a pooled row */
		const int per_plane = pra * pca, pl = tid >> 4;
		for (int t = tid & 15; t < per_plane; t += 16) {
			const int prl = fi_div(t, p.m_pca), pcl = t - prl * pca;
			const float *q = cbuf + pl * npos + (2 * prl) * cwl + 2 * pcl;
			float m = -FLT_MAX;	/* SpatialMaxPooling.c:96; first-max-wins does not show in the values */
#pragma unroll
			for (int dy = 0; dy < 3; dy++)
#pragma unroll
				for (int dx = 0; dx < 3; dx++) {
					const float v = q[dy * cwl + dx];
					m = v > m ? v : m;
				}
			p.y[((size_t)b * p.Co + mz * 64 + mb * 32 + pl) * plane_out + (size_t)(pr0 + prl) * p.pW + pc0 + pcl] = m;
		}
		__syncthreads();
	}
}

static unsigned fi_magic(int d)
{
	return d <= 1 ? 0u : (unsigned)((((unsigned long long)1 << 32) + d - 1) / d);
}

/* Geometry; returns the bytes of LDS, or 0 when the kernel does not take the layer. */
static size_t fi_plan(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode, int dtype, ConvImgF32Params *p)
{
	if (dtype != THHIP_F32 || B < 1 || Ci < 1 || Ci > 4 || Co < 64 || Co % 64 || kH < 1 || kW < 1 || dH < 1 || dW < 1 ||
	    dH > 4 || dW > 4 || padH < 0 || padW < 0)
		return 0;
	if (pkH != 3 || pkW != 3 || pdH != 2 || pdW != 2 || ppadH != ppadW || ppadH < 0 || ppadH > 1 || ceil_mode)
		return 0;
	const int oH = (H + 2 * padH - kH) / dH + 1, oW = (W + 2 * padW - kW) / dW + 1;
	if (oH < 3 || oW < 3)
		return 0;
	int pH, pW;
	thhip_pool_outsize(oH, oW, 3, 3, 2, 2, ppadH, ppadW, 0, &pH, &pW);
	if (pH < 1 || pW < 1 || pW % FI_PC)	/* (whole groups of pooled columns: the divisions by a group's width are by constants) */
		return 0;
	const int K = Ci * kH * kW, nsteps = (K + 1) / 2;
	const int prows = 2 * FI_PR * dH + kH, pw = (2 * FI_PC * dW + kW + 1) / 2 * 2;
	const size_t patch = (size_t)Ci * prows * pw * 4, weights = (size_t)nsteps * 512;
	size_t front = patch + weights;
	if (front < (size_t)32 * FI_MAXPOS * 4)
		front = (size_t)32 * FI_MAXPOS * 4;
	front = (front + 15) / 16 * 16;
	size_t total = front + (size_t)2 * nsteps * 4 + 128 * 4;
	if (total > FI_LDS_MAX || (double)Ci * H * W * 4 >= 2147483000.0 || (long)B * (Co / 64) > 65535)
		return 0;
	if ((2 * nsteps + 3) / 4 * 64 > 5 * FI_THREADS)	/* the weights of 64 planes: at most ten 16-byte loads a thread (K <= 160) */
		return 0;
	if (total < 56 * 1024)
		total = 56 * 1024;	/* (never three workgroups on a CU: the kernel is built for four wavefronts per SIMD) */
	if (p) {
		p->B = B; p->Ci = Ci; p->H = H; p->W = W; p->Co = Co; p->kH = kH; p->kW = kW; p->dH = dH; p->dW = dW;
		p->padH = padH; p->padW = padW; p->oH = oH; p->oW = oW; p->pH = pH; p->pW = pW; p->ppad = ppadH;
		p->K = K; p->nsteps = nsteps; p->prows = prows; p->pw = pw; p->front = (int)front;
		p->m_pw = fi_magic(pw);
	}
	return total;
}

bool thhip_conv_image_pool_f32_ok(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode, int dtype)
{
	return fi_plan(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pkH, pkW, pdH, pdW, ppadH, ppadW, ceil_mode, dtype, 0) != 0;
}

/* wpacked: the weights as thhip_conv_pack_weight_layout packs them for plane-major fp32 input of a plane
 * count that is no multiple of 32 (K order plane, kernel row, kernel column; KC chunks of 8 per 32-row
 * block).  y: [B][Co][pH][pW].  The caller brackets the launch. */
void thhip_conv_image_pool_f32(const float *x, const float *wpacked, int KC, const float *scale, const float *bias, float *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int ppad,
	int act, float thr, float val)
{
	ConvImgF32Params p;
	const size_t ldsbytes = fi_plan(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, 3, 3, 2, 2, ppad, ppad, 0, THHIP_F32, &p);
	if (!ldsbytes)
		THError("thhip_conv_image_pool_f32: unsupported layer");
	if (KC * 8 < 2 * p.nsteps)
		THError("thhip_conv_image_pool_f32: %d chunks of weights for K = %d", KC, p.K);
	p.x = x; p.wp = wpacked; p.bias = bias; p.scale = scale; p.y = y; p.KC = KC;
	p.act = act; p.thr = thr; p.val = val;
	static bool attr_set;
	if (!attr_set) {	/* more than 64 KiB of dynamic LDS has to be asked for */
		hipcheck(hipFuncSetAttribute((const void *)conv_f32_image_pool_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, FI_LDS_MAX));
		attr_set = true;
	}
	p.m_cwl = fi_magic(2 * FI_PC + 1);
	p.m_pca = fi_magic(FI_PC);
	const dim3 grid(p.pW / FI_PC, (p.pH + FI_PR - 1) / FI_PR, B * (Co / 64));
	conv_f32_image_pool_kernel<<<grid, dim3(FI_THREADS), ldsbytes, thhip_stream()>>>(p);
}
