/*
 * Linear on a small batch (2..32 rows): Y[b][o] = bias[o] + sum_k W[o][k] X[b][k].
 *
 * Replaces the matrix branch of nn_Linear_updateOutput (modules/Linear.c:92-108:
 * addmm with beta = 0, then the rank-1 bias update through addr / sger,
 * thbasic.c:757-789, OpenBLAS-stripped/sger.c:55-61).
 *
 * With so few columns the product is bound by reading W once from HBM, like
 * the batch-1 matrix-vector kernel, but every weight is used B times, which is
 * exactly one 16x16x4 fp32 MFMA per 16 rows x 16 batch columns x 4 k.  A
 * wavefront owns 16 output rows and a slice of K: per step lane (m = lane%16,
 * q = lane/16) holds four 16-byte vectors of row m (k = k0 + 16j + 4q + s),
 * the matching lane of the B operand the same k of batch row n = lane%16 (X
 * is small and stays in L2), and 16 MFMAs contract them; the order of k
 * inside a dot product is free as long as both operands use the same one.
 * The vectors are loaded by other lanes than the ones that use them, so that
 * neighbouring lanes read neighbouring addresses (64 or 128 adjacent bytes of
 * a row instead of 16), and moved with lane permutes: 25088 -> 4096 at batch
 * 16, fp32, 107 -> 83 us.  K is split over the four wavefronts of a workgroup (summed
 * through LDS) and over gridDim.y workgroups (partials in a scratch buffer,
 * summed by a second tiny kernel that also applies bias and Threshold).
 * For wide layers a wavefront owns RB = 4 such blocks of 16 rows: the batch
 * operand, which every wavefront has to fetch from L2 for its K slice and
 * which is as large per step as a block's weights, is then read once for 64
 * rows instead of once for 16.
 */
#include <stdio.h>
#include <stdlib.h>
#include "thhip_internal.h"

#define SK_THREADS 256
#define SK_KBYTES 256	/* bytes of a weight row one K-step covers: 64 per lane quarter */

/* One 16-byte vector of both operands -> MFMAs.  fp32: four 16x16x4 steps;
 * half types: one 16x16x32, whose lane quarter q holds 8 consecutive k. */
template <int DT> __device__ __forceinline__ void skinny_mma(floatx4 &acc, const floatx4 &a, const floatx4 &b);
template <> __device__ __forceinline__ void skinny_mma<THHIP_F32>(floatx4 &acc, const floatx4 &a, const floatx4 &b)
{
#pragma unroll
	for (int s = 0; s < 4; s++)
		acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], b[s], acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void skinny_mma<THHIP_F16>(floatx4 &acc, const floatx4 &a, const floatx4 &b)
{
	acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void skinny_mma<THHIP_BF16>(floatx4 &acc, const floatx4 &a, const floatx4 &b)
{
	acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}

/* The vector held by the lane whose byte index (lane * 4) is given. */
__device__ __forceinline__ floatx4 skinny_permute(const floatx4 &v, int src_lane4)
{
	floatx4 r;
#pragma unroll
	for (int e = 0; e < 4; e++)
		r[e] = __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane4, __float_as_int(v[e])));
	return r;
}

template <int DT, int NB, int RB>	/* NB 16-column groups: batch <= 16 * NB; RB 16-row blocks per wavefront */
__global__ __launch_bounds__(SK_THREADS) void skinny_kernel(const void *xv, const void *wv, float *part,
	int B, int nIn, int nOut, int ksplit)
{
	typedef typename ThhipElem<DT>::T elem;
	constexpr int VEC = 16 / (int)sizeof(elem);		/* elements per 16-byte vector */
	constexpr int KSTEP = SK_KBYTES / (int)sizeof(elem);	/* k per step */
	const elem *x = (const elem *)xv, *w = (const elem *)wv;
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int m = lane & 15, q = lane >> 4;
	/* The MFMA wants row m = lane % 16 in lane q * 16 + m, so neighbouring lanes
	 * would load from rows a whole row length apart, 64 separate 16-byte requests
	 * per instruction.  Instead neighbouring lanes load neighbouring vectors and a
	 * lane permute brings every vector to the lane that feeds it to the matrix
	 * core.  Batch operand: lane 4 m' + q' loads for (row m', quarter q'), 64
	 * adjacent bytes per four lanes.  Weights (four row blocks per wavefront): load i of a step takes rows
	 * 8 (i % 2) + lane / 8 and vector 8 (i / 2) + lane % 8 of the step's sixteen,
	 * whole 128-byte lines per eight lanes; the vector for (m, q) of MFMA group j
	 * then sits in load 2 (j / 2) + m / 8, lane 8 (m % 8) + 4 (j % 2) + q. */
	constexpr bool WIDE_W = RB == 4;
	const int lm = lane >> 2, lq = lane & 3;
	const int src_lane4 = (m * 4 + q) * 4;	/* byte index of the lane that loaded for (m, q) */
	const int wsrc4[2] = { ((m & 7) * 8 + q) * 4, ((m & 7) * 8 + 4 + q) * 4 };
	const bool upper = m >= 8;
	const int row0 = blockIdx.x * (16 * RB);
	/* K-steps are dealt round-robin to (workgroup slice, wave) */
	const int nsteps = (nIn + KSTEP - 1) / KSTEP;
	const int stride = ksplit * 4;
	const elem *wr[RB][2];
#pragma unroll
	for (int rb = 0; rb < RB; rb++)
#pragma unroll
		for (int h = 0; h < 2; h++)
			wr[rb][h] = w + (size_t)min(row0 + rb * 16 + (WIDE_W ? h * 8 + (lane >> 3) : lm), nOut - 1) * nIn;
	const elem *xr[NB];
#pragma unroll
	for (int g = 0; g < NB; g++)
		xr[g] = x + (size_t)min(g * 16 + lm, B - 1) * nIn;

	floatx4 acc[RB][NB];
#pragma unroll
	for (int rb = 0; rb < RB; rb++)
#pragma unroll
		for (int g = 0; g < NB; g++)
			acc[rb][g] = floatx4{ 0, 0, 0, 0 };

	for (int st = blockIdx.y * 4 + wave; st < nsteps; st += stride) {
		/* load j of the four lane quarters covers 64 adjacent bytes of a row */
		const int kb = st * KSTEP + lq * VEC;
		constexpr int NJ = SK_KBYTES / 64;
		static_assert(NJ == 4, "the weight loads pair up: two rows halves x two vector halves");
		floatx4 a[RB][NJ], raw[RB][NJ], b[NB][NJ];
#pragma unroll
		for (int j = 0; j < NJ; j++) {
			const int k = kb + j * (4 * VEC);
			const bool ok = k < nIn;	/* nIn % VEC == 0: a vector is all in or all out */
			/* whole lines per eight lanes with four row blocks per wavefront; with one
			 * the second permute costs more than it saves (9216 -> 4096 at batch 4:
			 * 27 against 31 us) and the weights are loaded like the batch operand */
			const int kw = WIDE_W ? st * KSTEP + ((j >> 1) * 8 + (lane & 7)) * VEC : k;
			const bool okw = kw < nIn;
#pragma unroll
			for (int rb = 0; rb < RB; rb++)
				raw[rb][j] = okw ? *(const floatx4 *)(wr[rb][WIDE_W ? j & 1 : 0] + kw) : floatx4{ 0, 0, 0, 0 };
#pragma unroll
			for (int g = 0; g < NB; g++)
				b[g][j] = ok ? *(const floatx4 *)(xr[g] + k) : floatx4{ 0, 0, 0, 0 };
		}
#pragma unroll
		for (int j = 0; j < NJ; j++) {
#pragma unroll
			for (int rb = 0; rb < RB; rb++) {
				if constexpr (WIDE_W) {
					const floatx4 lo = skinny_permute(raw[rb][2 * (j >> 1)], wsrc4[j & 1]);
					const floatx4 hi = skinny_permute(raw[rb][2 * (j >> 1) + 1], wsrc4[j & 1]);
#pragma unroll
					for (int e = 0; e < 4; e++)
						a[rb][j][e] = upper ? hi[e] : lo[e];
				} else
					a[rb][j] = skinny_permute(raw[rb][j], src_lane4);
			}
#pragma unroll
			for (int g = 0; g < NB; g++)
				b[g][j] = skinny_permute(b[g][j], src_lane4);
		}
#pragma unroll
		for (int j = 0; j < NJ; j++)
#pragma unroll
			for (int rb = 0; rb < RB; rb++)
#pragma unroll
				for (int g = 0; g < NB; g++)
					skinny_mma<DT>(acc[rb][g], a[rb][j], b[g][j]);
	}

	/* D layout: lane holds column n = lane%16, rows 4*(lane/16) + r */
	__shared__ float red[4][RB * NB][16][17];
#pragma unroll
	for (int rb = 0; rb < RB; rb++)
#pragma unroll
		for (int g = 0; g < NB; g++)
#pragma unroll
			for (int r = 0; r < 4; r++)
				red[wave][rb * NB + g][q * 4 + r][m] = acc[rb][g][r];
	__syncthreads();
	for (int i = tid; i < RB * NB * 256; i += SK_THREADS) {
		const int t = i >> 8, rr = (i >> 4) & 15, n = i & 15;
		const int rb = t / NB, g = t - rb * NB;
		const int o = row0 + rb * 16 + rr, bcol = g * 16 + n;
		if (o < nOut && bcol < B) {
			const float s = (red[0][t][rr][n] + red[1][t][rr][n]) + (red[2][t][rr][n] + red[3][t][rr][n]);
			part[((size_t)blockIdx.y * B + bcol) * nOut + o] = s;
		}
	}
}

template <int DT>
__global__ void skinny_finish_kernel(const float *part, const float *bias, void *y, int B, int nOut, int ksplit,
	int act, float thr, float val)
{
	const long total = (long)B * nOut;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	for (; i < total; i += (long)gridDim.x * blockDim.x) {
		float s = 0;
		for (int p = 0; p < ksplit; p++)
			s += part[(size_t)p * total + i];
		s += bias ? bias[i % nOut] : 0.0f;
		if (act)
			s = s > thr ? s : val;
		ThhipElem<DT>::st(y, i, s);
	}
}

static float *g_scratch;
static size_t g_scratch_bytes;

static float *skinny_scratch(size_t bytes)
{
	if (bytes > g_scratch_bytes) {
		if (g_scratch) {
			hipcheck(hipStreamSynchronize(thhip_stream()));
			thhip_free(g_scratch);
		}
		g_scratch = (float *)thhip_malloc(bytes);
		g_scratch_bytes = bytes;
	}
	return g_scratch;
}

/* A launch takes 32 batch columns; larger batches run in slices of 32, each
 * reading the weights again: up to four slices that still beats the tiled
 * GEMM on the layers this is for (25088 -> 4096 fp16 at batch 64: 283 us as a
 * convolution of one position, two slices of 60 us here). */
#define SK_MAX_BATCH 128

extern "C" int thhip_linear_batched_supported(int B, int nIn, int nOut, int dtype)
{
	if (dtype != THHIP_F32 && dtype != THHIP_F16 && dtype != THHIP_BF16)
		return 0;
	const int vec = dtype == THHIP_F32 ? 4 : 8;
	return B >= 1 && B <= SK_MAX_BATCH && nIn % vec == 0 && nIn >= vec && nOut >= 1;
}

template <int DT, bool SCOPED>
static void skinny_launch(const void *x, const void *wrow, const float *bias, void *y, float *part,
	int B, int nIn, int nOut, int rb, int groups, int ksplit, int act, float thr, float val)
{
	{
		/* algorithmic bytes: W once, X once, Y once */
		ThhipLaunchScope scope(SCOPED ? THHIP_FAM_GEMV : -1, (double)thhip_esize(DT) * ((double)nOut * nIn + (double)B * nIn + (double)B * nOut));
		dim3 grid(groups, ksplit);
		if (B <= 16 && rb == 4)
			skinny_kernel<DT, 1, 4><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, ksplit);
		else if (B <= 16)
			skinny_kernel<DT, 1, 1><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, ksplit);
		else if (rb == 4)
			skinny_kernel<DT, 2, 4><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, ksplit);
		else
			skinny_kernel<DT, 2, 1><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, ksplit);
	}
	{
		ThhipLaunchScope scope(SCOPED ? THHIP_FAM_OTHER : -1, 4.0 * (ksplit + 1.0) * B * nOut);
		long total = (long)B * nOut;
		long blocks = (total + 255) / 256;
		skinny_finish_kernel<DT><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(part, bias, y, B, nOut,
			ksplit, act, thr, val);
	}
}

/* Tests and tuning: force the 16-row blocks per wavefront (1 or 4); 0 = choose by the layer's width. */
static int g_skinny_rb;
extern "C" void thhip_linear_batched_set_tuning(int row_blocks)
{
	if (row_blocks != 0 && row_blocks != 1 && row_blocks != 4)
		THError("thhip_linear_batched_set_tuning(%d): 0, 1 or 4", row_blocks);
	g_skinny_rb = row_blocks;
}

/* Row blocks per wavefront, row groups and K split of one launch (B <= 32). */
struct skinny_plan { int rb, groups, ksplit; };
static struct skinny_plan skinny_choose(int B, int nIn, int nOut, int dtype)
{
	struct skinny_plan p;
	/* four row blocks per wavefront for wide layers and batches that fill most of
	 * the 16 MFMA columns (measured: 12 % on 25088 -> 4096 at batch 16; at batch 4
	 * the unused columns re-read their rows from L1 and one block is faster) */
	p.rb = nOut >= 1024 && B > 8 ? 4 : 1;
	if (g_skinny_rb)
		p.rb = g_skinny_rb;
	p.groups = (nOut + 16 * p.rb - 1) / (16 * p.rb);
	const int kstep = SK_KBYTES / thhip_esize(dtype);
	const int nsteps = (nIn + kstep - 1) / kstep;
	/* aim at ~4096 wavefronts, ~2048 with four row blocks each (two per SIMD:
	 * 25088 -> 4096 at batch 16 runs 4 % (fp32) and 8 % (fp16) faster than with
	 * four, and 16-27 % faster than with eight or sixteen), at least two K-steps
	 * per wavefront */
	p.ksplit = ((p.rb == 4 ? 512 : 1024) + p.groups - 1) / p.groups;
	if (p.ksplit > nsteps / 8)
		p.ksplit = nsteps / 8;
	if (p.ksplit < 1)
		p.ksplit = 1;
	if (p.ksplit > 64)
		p.ksplit = 64;
	return p;
}

extern "C" void thhip_linear_batched(const void *x, const void *wrow, const float *bias, void *y,
	int B, int nIn, int nOut, int act, float thr, float val, int dtype)
{
	if (!thhip_linear_batched_supported(B, nIn, nOut, dtype))
		THError("thhip_linear_batched: unsupported shape B=%d nIn=%d nOut=%d dtype=%d", B, nIn, nOut, dtype);
	if (B > 32) {
		const size_t esize = thhip_esize(dtype);
		for (int b0 = 0; b0 < B; b0 += 32)
			thhip_linear_batched((const char *)x + (size_t)b0 * nIn * esize, wrow, bias, (char *)y + (size_t)b0 * nOut * esize,
				B - b0 < 32 ? B - b0 : 32, nIn, nOut, act, thr, val, dtype);
		return;
	}
	const struct skinny_plan p = skinny_choose(B, nIn, nOut, dtype);
	float *part = skinny_scratch((size_t)p.ksplit * B * nOut * sizeof(float));
	THHIP_DISPATCH_FLOAT(dtype, (skinny_launch<DT, true>(x, wrow, bias, y, part, B, nIn, nOut, p.rb, p.groups, p.ksplit, act, thr, val)));
}

/*
 * The same product for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid it): the partial sums
 * of the K slices go to a fixed array in device memory instead of a buffer that
 * grows on demand.  Every GPU the library runs on holds its own copy of the
 * array at its own address until the process ends; the address is looked up
 * once per device (at THInit for the current device, else at the first call)
 * and only that pointer is ever handed to a kernel.  The kernels write every
 * partial sum they later read, so nothing has to be cleared between calls, but
 * two calls that overlap on one GPU (other streams, other threads) race on the
 * array.
 */
#define SK_STATIC_BYTES (8u << 20)
#define SK_STATIC_MAXDEV 16
static __device__ __align__(256) float scratch[SK_STATIC_BYTES / sizeof(float)];
static float *g_static_part[SK_STATIC_MAXDEV];

static float *skinny_static_part(void)
{
	int dev = -1;
	thhip_stream();		/* first use: selects the device and makes the stream */
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SK_STATIC_MAXDEV)
		return 0;
	if (!g_static_part[dev]) {
		float *p = 0;
		const hipError_t rc = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
		if (rc != hipSuccess || !p) {
			fprintf(stderr, "thhip_linear_batched_noalloc: hipGetSymbolAddress failed on device %d: %s\n", dev,
				hipGetErrorString(rc));
			return 0;
		}
		g_static_part[dev] = p;
	}
	return g_static_part[dev];
}

extern "C" int thhip_linear_batched_noalloc_init(void)
{
	return skinny_static_part() ? 0 : -1;
}

extern "C" size_t thhip_linear_batched_noalloc_limit(void)
{
	return SK_STATIC_BYTES;
}

extern "C" int thhip_linear_batched_noalloc(const void *x, const void *wrow, const float *bias, void *y,
	int B, int nIn, int nOut, int act, float thr, float val, int dtype)
{
	if (!thhip_linear_batched_supported(B, nIn, nOut, dtype)) {
		fprintf(stderr, "thhip_linear_batched_noalloc: unsupported shape B=%d nIn=%d nOut=%d dtype=%d\n", B, nIn, nOut, dtype);
		return -1;
	}
	/* every slice of 32 batch rows must fit: check before anything is launched */
	for (int b0 = 0; b0 < B; b0 += 32) {
		const int bs = B - b0 < 32 ? B - b0 : 32;
		const struct skinny_plan p = skinny_choose(bs, nIn, nOut, dtype);
		const size_t need = (size_t)p.ksplit * bs * nOut * sizeof(float);
		if (need > SK_STATIC_BYTES) {
			fprintf(stderr, "thhip_linear_batched_noalloc: B=%d nIn=%d nOut=%d needs %zu bytes of partial sums "
				"(%d K slices x %d rows x %d outputs), the fixed array holds %u; use thhip_linear_batched\n",
				B, nIn, nOut, need, p.ksplit, bs, nOut, (unsigned)SK_STATIC_BYTES);
			return -2;
		}
	}
	float *part = skinny_static_part();
	if (!part)
		return -3;
	const size_t esize = thhip_esize(dtype);
	for (int b0 = 0; b0 < B; b0 += 32) {
		const int bs = B - b0 < 32 ? B - b0 : 32;
		const struct skinny_plan p = skinny_choose(bs, nIn, nOut, dtype);
		const void *xs = (const char *)x + (size_t)b0 * nIn * esize;
		void *ys = (char *)y + (size_t)b0 * nOut * esize;
		THHIP_DISPATCH_FLOAT(dtype, (skinny_launch<DT, false>(xs, wrow, bias, ys, part, bs, nIn, nOut, p.rb, p.groups, p.ksplit, act, thr, val)));
	}
	return 0;
}

/* ------------------------------------------------------------------ */
/* uint8 (LOWP) variant                                                */
/* ------------------------------------------------------------------ */

/*
 * One output position per image in the uint8 engine (Linear layers, or a
 * convolution whose window covers its whole input): C[b][o] over K codes.
 * Both operands are K-contiguous in memory -- weights row-major [nOut][K],
 * activations [B][K] -- and v_mfma_i32_32x32x32_i8 wants 16 consecutive k per
 * lane (lane = row or column lane%32, k half lane/32), so operands go from
 * global memory to the matrix core through registers only.  A K-step is 128
 * codes, four MFMAs of 32: for MFMA j lane (m, h) reads the 16 bytes
 * k0 + 32j + 16h .. +15 of its row, so the two halves of a load are adjacent
 * in memory.  Weights are stored re-centred (code - 128, done
 * once at pack time), activations are re-centred on the fly (x ^ 0x80).
 *
 * The four wavefronts of a workgroup own the same RG*32 rows and every fourth
 * K-step of the workgroup's slice; their int32 tiles are summed through LDS
 * and written as one partial per (K slice, row, batch column).  A finishing
 * kernel sums the slices, applies the expanded offset terms, gemmlowp's output
 * stage, the saturating bias add (a plane of one element is all "tail": no
 * lower clamp, lowp_SpatialConvolution.c:86-87) and the threshold.  Integer
 * sums are exact, so the split changes nothing in the result.
 */
#define SKU_KSTEP 128
#define SKU_BPAD 64	/* batch columns per partial row */

template <int RG, int NB>	/* RG 32-row groups per wavefront; NB 32-column groups: batch <= 32 * NB */
__global__ __launch_bounds__(SK_THREADS) void skinny_u8_kernel(const unsigned char *x, const unsigned char *w,
	int *part, int *cspart, int B, int K, int nOut, int ksplit)
{
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int m = lane & 31, h = lane >> 5;
	const int row0 = blockIdx.x * (32 * RG);
	const int nsteps = (K + SKU_KSTEP - 1) / SKU_KSTEP;
	const int stride = ksplit * 4;
	const bool want_cs = blockIdx.x == 0;
	const unsigned char *wr[RG], *xr[NB];
#pragma unroll
	for (int rg = 0; rg < RG; rg++)
		wr[rg] = w + (size_t)min(row0 + rg * 32 + m, nOut - 1) * K + h * 16;
#pragma unroll
	for (int g = 0; g < NB; g++)
		xr[g] = x + (size_t)min(g * 32 + m, B - 1) * K + h * 16;
	intx16 acc[RG][NB];
	int cs[NB];
#pragma unroll
	for (int g = 0; g < NB; g++) {
		cs[g] = 0;
#pragma unroll
		for (int rg = 0; rg < RG; rg++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[rg][g][r] = 0;
	}
	const intx4 zero_a = { 0, 0, 0, 0 };
	const intx4 zero_b = { (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };
	intx4 a[RG][4], b[NB][4], an[RG][4], bn[NB][4];

	/* K % 16 == 0: a 16-byte piece is all inside the row or all outside */
#define SKU_LOAD(A_, B_, ST_)                                                                  \
	do {                                                                                   \
		const int kk_ = (ST_) * SKU_KSTEP;                                             \
		_Pragma("unroll") for (int j = 0; j < 4; j++) {                                \
			const bool ok_ = kk_ + j * 32 + h * 16 < K;                            \
			_Pragma("unroll") for (int rg = 0; rg < RG; rg++)                      \
				A_[rg][j] = ok_ ? *(const intx4 *)(wr[rg] + kk_ + j * 32) : zero_a; \
			_Pragma("unroll") for (int g = 0; g < NB; g++)                         \
				B_[g][j] = ok_ ? *(const intx4 *)(xr[g] + kk_ + j * 32) : zero_b;  \
		}                                                                              \
	} while (0)

	int st = blockIdx.y * 4 + wave;
	if (st < nsteps)
		SKU_LOAD(a, b, st);
	for (; st < nsteps; st += stride) {
		const int sn = st + stride;
		if (sn < nsteps)
			SKU_LOAD(an, bn, sn);
#pragma unroll
		for (int j = 0; j < 4; j++) {
#pragma unroll
			for (int g = 0; g < NB; g++) {
#pragma unroll
				for (int d = 0; d < 4; d++)
					b[g][j][d] ^= (int)0x80808080;
				if (want_cs) {
#pragma unroll
					for (int d = 0; d < 4; d++)
						cs[g] = __builtin_amdgcn_sdot4(b[g][j][d], 0x01010101, cs[g], false);
				}
#pragma unroll
				for (int rg = 0; rg < RG; rg++)
					acc[rg][g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[rg][j], b[g][j], acc[rg][g], 0, 0, 0);
			}
		}
		if (sn < nsteps) {
#pragma unroll
			for (int j = 0; j < 4; j++) {
#pragma unroll
				for (int rg = 0; rg < RG; rg++)
					a[rg][j] = an[rg][j];
#pragma unroll
				for (int g = 0; g < NB; g++)
					b[g][j] = bn[g][j];
			}
		}
	}
#undef SKU_LOAD

	/* D layout: lane holds column n = lane%32, rows 8*(r/4) + 4*(lane/32) + r%4 */
	__shared__ int red[4][16][65];
	__shared__ int csred[4][NB][64];
#pragma unroll
	for (int rg = 0; rg < RG; rg++)
#pragma unroll
		for (int g = 0; g < NB; g++) {
			if (rg + g)
				__syncthreads();
#pragma unroll
			for (int r = 0; r < 16; r++)
				red[wave][r][lane] = acc[rg][g][r];
			__syncthreads();
#pragma unroll
			for (int i = 0; i < 4; i++) {
				const int idx = tid + i * SK_THREADS;
				const int n = idx & 31, o = idx >> 5;
				const int r = 4 * (o >> 3) + (o & 3), ln = n + 32 * ((o >> 2) & 1);
				const int s = (red[0][r][ln] + red[1][r][ln]) + (red[2][r][ln] + red[3][r][ln]);
				const int bcol = g * 32 + n, orow = row0 + rg * 32 + o;
				if (orow < nOut && bcol < B)
					part[((size_t)blockIdx.y * nOut + orow) * SKU_BPAD + bcol] = s;
			}
		}
	if (want_cs) {
#pragma unroll
		for (int g = 0; g < NB; g++)
			csred[wave][g][lane] = cs[g];
		__syncthreads();
		if (tid < 32 * NB) {
			const int g = tid >> 5, n = tid & 31;
			int s = 0;
#pragma unroll
			for (int wv = 0; wv < 4; wv++)
				s += csred[wv][g][n] + csred[wv][g][n + 32];
			cspart[blockIdx.y * SKU_BPAD + tid] = s;
		}
	}
}

/* One workgroup per 32 output rows x 16 batch columns: sums the K slices,
 * requantises and transposes [row][batch] partials into y [B][nOut] through LDS. */
__global__ __launch_bounds__(256) void skinny_u8_finish_kernel(const int *part, const int *cspart, const int *rowsum,
	const int *addend, unsigned char *y, int B, int K, int nOut, int ksplit, int offA, int offB,
	int c_off, int c_mult, int c_shift, int act, int thr, int val)
{
	__shared__ int t[32][17];
	__shared__ int csum[16];
	const int tid = threadIdx.x, o0 = blockIdx.x * 32, b0 = blockIdx.y * 16;
	if (tid < 16) {
		int s = 0;
		for (int p = 0; p < ksplit; p++)
			s += cspart[p * SKU_BPAD + b0 + tid];
		csum[tid] = s;
	}
	{
		const int bl = tid & 15, oo = tid >> 4;
#pragma unroll
		for (int i = 0; i < 2; i++) {
			const int ol = oo + 16 * i, o = o0 + ol;
			int s = 0;
			if (o < nOut && b0 + bl < B)
				for (int p = 0; p < ksplit; p++)
					s += part[((size_t)p * nOut + o) * SKU_BPAD + b0 + bl];
			t[ol][bl] = s;
		}
	}
	__syncthreads();
	const int ol = tid & 31, o = o0 + ol, bb = tid >> 5;
	if (o >= nOut)
		return;
	const int rs = offB * rowsum[o] + K * offA * offB;
	const int add = addend ? addend[o] : 0;
#pragma unroll
	for (int i = 0; i < 2; i++) {
		const int bl = bb + 8 * i, b = b0 + bl;
		if (b >= B)
			break;
		const int a = t[ol][bl] + rs + offA * csum[bl];
		unsigned u = ((unsigned)a + (unsigned)c_off) * (unsigned)c_mult;
		u += c_shift < 1 ? 0u : 1u << (c_shift - 1);
		int q = (int)u >> c_shift;
		q = q < 0 ? 0 : q > 255 ? 255 : q;
		if (addend) {
			const int sum = q + add;
			q = sum > 255 ? 255 : (sum & 255);
		}
		if (act)
			q = q > thr ? q : val;
		y[(size_t)b * nOut + o] = (unsigned char)q;
	}
}

static int *g_u8_scratch;
static size_t g_u8_scratch_words;
static int g_u8_ksplit, g_u8_rg;

extern "C" int thhip_linear_batched_u8_supported(int B, int K, int nOut)
{
	return B >= 1 && B <= 64 && K % 16 == 0 && K >= 16 && nOut >= 1;
}

/* Test and tuning hook: force the K split (1..64) and the row groups per
 * wavefront (1 or 2) of thhip_linear_batched_u8; 0 restores the heuristic. */
extern "C" void thhip_linear_batched_u8_set_tuning(int ksplit, int rg)
{
	if (ksplit < 0 || ksplit > 64 || rg < 0 || rg > 2)
		THError("thhip_linear_batched_u8_set_tuning(%d, %d): out of range", ksplit, rg);
	g_u8_ksplit = ksplit;
	g_u8_rg = rg;
}

/* Device copy of row-major weight codes [nOut][K], re-centred to signed bytes. */
extern "C" unsigned char *thhip_linear_pack_weight_u8(const unsigned char *w_host, int nOut, int K)
{
	const size_t n = (size_t)nOut * K;
	unsigned char *h = (unsigned char *)malloc(n);
	for (size_t i = 0; i < n; i++)
		h[i] = w_host[i] ^ 0x80;
	unsigned char *d = (unsigned char *)thhip_malloc(n);
	thhip_memcpy_h2d(d, h, n);
	free(h);
	return d;
}

/* Row sums of the re-centred weight codes, as a device array (made once per layer). */
extern "C" int *thhip_u8_rowsums(const unsigned char *w_host, int nOut, int K)
{
	int *h = (int *)malloc(sizeof(int) * (size_t)nOut);
	for (int o = 0; o < nOut; o++) {
		int s = 0;
		for (int k = 0; k < K; k++)
			s += (int)w_host[(size_t)o * K + k] - 128;
		h[o] = s;
	}
	int *d = (int *)thhip_malloc(sizeof(int) * (size_t)nOut);
	thhip_memcpy_h2d(d, h, sizeof(int) * (size_t)nOut);
	free(h);
	return d;
}

template <int RG, int NB>
static void skinny_u8_launch(dim3 grid, const unsigned char *x, const unsigned char *wrow, int *part, int *cspart,
	int B, int K, int nOut, int ksplit)
{
	skinny_u8_kernel<RG, NB><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, cspart, B, K, nOut, ksplit);
}

extern "C" void thhip_linear_batched_u8(const unsigned char *x, const unsigned char *wrow, const int *rowsum,
	const int *addend, unsigned char *y, int B, int K, int nOut,
	int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val)
{
	if (!thhip_linear_batched_u8_supported(B, K, nOut))
		THError("thhip_linear_batched_u8: unsupported shape B=%d K=%d nOut=%d", B, K, nOut);
	if (c_shift < 0 || c_shift > 31)
		THError("thhip_linear_batched_u8: shift %d out of range", c_shift);
	const int rg = g_u8_rg ? g_u8_rg : nOut >= 2048 ? 2 : 1;
	const int groups = (nOut + 32 * rg - 1) / (32 * rg);
	const int nsteps = (K + SKU_KSTEP - 1) / SKU_KSTEP;
	/* aim at ~1024 wavefronts with at least two K-steps each */
	int ksplit = (256 + groups - 1) / groups;
	if (ksplit > nsteps / 8)
		ksplit = nsteps / 8;
	if (g_u8_ksplit)
		ksplit = g_u8_ksplit;
	if (ksplit < 1)
		ksplit = 1;
	if (ksplit > 64)
		ksplit = 64;
	const size_t words = (size_t)ksplit * SKU_BPAD * ((size_t)nOut + 1);
	if (words > g_u8_scratch_words) {
		if (g_u8_scratch) {
			hipcheck(hipStreamSynchronize(thhip_stream()));
			thhip_free(g_u8_scratch);
		}
		g_u8_scratch_words = words < (1u << 20) ? (1u << 20) : words;
		g_u8_scratch = (int *)thhip_malloc(g_u8_scratch_words * sizeof(int));
	}
	int *cspart = g_u8_scratch, *part = g_u8_scratch + (size_t)ksplit * SKU_BPAD;
	{
		ThhipLaunchScope scope(THHIP_FAM_CONV_I8, 2.0 * nOut * (double)K * B);
		dim3 grid(groups, ksplit);
		if (rg == 1 && B <= 32)
			skinny_u8_launch<1, 1>(grid, x, wrow, part, cspart, B, K, nOut, ksplit);
		else if (rg == 1)
			skinny_u8_launch<1, 2>(grid, x, wrow, part, cspart, B, K, nOut, ksplit);
		else if (B <= 32)
			skinny_u8_launch<2, 1>(grid, x, wrow, part, cspart, B, K, nOut, ksplit);
		else
			skinny_u8_launch<2, 2>(grid, x, wrow, part, cspart, B, K, nOut, ksplit);
	}
	{
		ThhipLaunchScope scope(THHIP_FAM_OTHER, (4.0 * ksplit + 1.0) * B * nOut);
		skinny_u8_finish_kernel<<<dim3((nOut + 31) / 32, (B + 15) / 16), dim3(256), 0, thhip_stream()>>>(part, cspart, rowsum, addend, y,
			B, K, nOut, ksplit, 128 + a_off, 128 + b_off, c_off, c_mult, c_shift, act, thr, val);
	}
}
