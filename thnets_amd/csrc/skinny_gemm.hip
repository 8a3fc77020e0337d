/*
 * Linear on a small batch (2..64 rows a launch): Y[b][o] = bias[o] + sum_k W[o][k] X[b][k].
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
 * rows instead of once for 16.  A launch takes up to 64 batch rows: four groups of
 * sixteen columns, beside which two row blocks per wavefront are what the registers
 * hold.
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

/* FINAL: K is not split over workgroups (gridDim.y == 1), and the workgroup adds the bias, applies the
 * Threshold and stores the outputs itself: no partial sums in memory and no second launch. */
template <int DT, int NB, int RB, bool FINAL = false>	/* NB 16-column groups: batch <= 16 * NB; RB 16-row blocks per wavefront */
__global__ __launch_bounds__(SK_THREADS) void skinny_kernel(const void *xv, const void *wv, float *part,
	int B, int nIn, int nOut, int ksplit, const float *bias = 0, void *y = 0, int act = 0, float thr = 0, float val = 0)
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
			float s = (red[0][t][rr][n] + red[1][t][rr][n]) + (red[2][t][rr][n] + red[3][t][rr][n]);
			if constexpr (FINAL) {	/* as skinny_finish_kernel with one part */
				s = 0.0f + s;
				s += bias ? bias[o] : 0.0f;
				if (act)
					s = s > thr ? s : val;
				ThhipElem<DT>::st(y, (size_t)bcol * nOut + o, s);
			} else
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

/* A launch takes 64 batch columns (four groups of sixteen beside two row blocks per wavefront:
 * what the registers hold); larger batches run in slices of 64, each reading the weights again,
 * which still beats the tiled GEMM on the layers this is for (25088 -> 4096 fp16 at batch 64:
 * 283 us as a convolution of one position, two slices of 32 of 50 + 39 us, one launch here). */
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
	if (ksplit == 1 && rb == 1 && B <= 32) {
		/* a short K (fewer than sixteen K-steps), one row block per workgroup: the workgroup finishes its outputs itself */
		ThhipLaunchScope scope(SCOPED ? THHIP_FAM_GEMV : -1, (double)thhip_esize(DT) * ((double)nOut * nIn + (double)B * nIn + (double)B * nOut));
		if (B <= 16)
			skinny_kernel<DT, 1, 1, true><<<dim3(groups, 1), dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, 1,
				bias, y, act, thr, val);
		else
			skinny_kernel<DT, 2, 1, true><<<dim3(groups, 1), dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, 1,
				bias, y, act, thr, val);
		return;
	}
	{
		/* algorithmic bytes: W once, X once, Y once */
		ThhipLaunchScope scope(SCOPED ? THHIP_FAM_GEMV : -1, (double)thhip_esize(DT) * ((double)nOut * nIn + (double)B * nIn + (double)B * nOut));
		dim3 grid(groups, ksplit);
		if (B > 32 && rb == 2)
			skinny_kernel<DT, 4, 2><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, ksplit);
		else if (B > 32)
			skinny_kernel<DT, 4, 1><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>(x, wrow, part, B, nIn, nOut, ksplit);
		else if (B <= 16 && rb == 4)
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

/* Batch rows one launch takes: 64, or 32 when the row blocks per wavefront are forced. */
static inline int skinny_slice(void);

/* Row blocks per wavefront, row groups and K split of one launch (B <= 64). */
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
	else if (B > 32 && p.rb == 4)
		p.rb = 2;	/* 33..64 batch rows: four column groups, and the registers of two row blocks beside them */
	p.groups = (nOut + 16 * p.rb - 1) / (16 * p.rb);
	const int kstep = SK_KBYTES / thhip_esize(dtype);
	const int nsteps = (nIn + kstep - 1) / kstep;
	/* aim at ~4096 wavefronts, ~2048 with four row blocks each (two per SIMD:
	 * 25088 -> 4096 at batch 16 runs 4 % (fp32) and 8 % (fp16) faster than with
	 * four, and 16-27 % faster than with eight or sixteen), at least two K-steps
	 * per wavefront */
	p.ksplit = ((p.rb == 4 ? 512 : p.rb == 2 ? 768 : 1024) + p.groups - 1) / p.groups;
	if (p.ksplit > nsteps / 8)
		p.ksplit = nsteps / 8;
	if (p.ksplit < 1)
		p.ksplit = 1;
	if (p.ksplit > 64)
		p.ksplit = 64;
	/* (4096 -> 4096 at batch 16 as 256 workgroups over all of K, which then finish their outputs without the
	 * second launch, took as long as the two launches: VGG-16 fp16 0.706 against 0.705 ms) */
	return p;
}

static inline int skinny_slice(void) { return g_skinny_rb ? 32 : 64; }

extern "C" void thhip_linear_batched(const void *x, const void *wrow, const float *bias, void *y,
	int B, int nIn, int nOut, int act, float thr, float val, int dtype)
{
	if (!thhip_linear_batched_supported(B, nIn, nOut, dtype))
		THError("thhip_linear_batched: unsupported shape B=%d nIn=%d nOut=%d dtype=%d", B, nIn, nOut, dtype);
	const int slice = skinny_slice();
	if (B > slice) {
		const size_t esize = thhip_esize(dtype);
		for (int b0 = 0; b0 < B; b0 += slice)
			thhip_linear_batched((const char *)x + (size_t)b0 * nIn * esize, wrow, bias, (char *)y + (size_t)b0 * nOut * esize,
				B - b0 < slice ? B - b0 : slice, nIn, nOut, act, thr, val, dtype);
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
	/* every slice of batch rows must fit: check before anything is launched */
	const int slice = skinny_slice();
	for (int b0 = 0; b0 < B; b0 += slice) {
		const int bs = B - b0 < slice ? B - b0 : slice;
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
	for (int b0 = 0; b0 < B; b0 += slice) {
		const int bs = B - b0 < slice ? B - b0 : slice;
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
 * convolution whose window covers its whole input): C[b][o] over K codes,
 * batch <= 64.  The layer is bound by reading its weights once from HBM, so
 * the weights are stored in the order the matrix core wants them and the whole
 * layer is one kernel:
 *
 * - v_mfma_i32_16x16x64_i8 takes, of a 16-row block, 16 consecutive k per lane
 *   (lane = row lane % 16, k quarter lane / 16).  The pack step stores every
 *   (16-row block, 64-code K-step) as the 1 KiB a wavefront loads for it, lane
 *   by lane, re-centred to signed bytes (code - 128), K-steps of a block one
 *   after the other: a load instruction reads 1 KiB contiguous, no permutes.
 *   Rows and K are padded with re-centred zeros, which add nothing.
 * - A workgroup of sixteen wavefronts owns one 16-row block (or two, see below) and all of K, which
 *   it walks in chunks of sixteen K-steps (1024 codes), wavefront w taking step
 *   w of every chunk: the workgroup reads 16 KiB of contiguous weights per
 *   chunk, each wavefront keeps the weights of the next three chunks on their
 *   way.
 * - The activations [B][K] of a chunk are needed by every wavefront's fragment
 *   in a layout that is bad to fetch (16 rows x 64 bytes per load), so the
 *   workgroup fetches them together, whole 1 KiB runs of a row per load, four
 *   chunks ahead into registers, and passes them on through LDS (two buffers,
 *   one barrier per chunk).  A 16-byte piece (row b, k piece p) goes to slot
 *   b % 16 ^ p % 16 of its 256-byte line [step p / 4][group b / 16][quarter
 *   p % 4], which keeps both the writes (one row, 64 pieces per wavefront) and
 *   the fragment reads (16 rows of one piece per quarter) free of bank
 *   conflicts.  Rows past B repeat the last one, pieces past K hold code 128
 *   (0 once re-centred: x ^ 0x80); the column sums are taken with v_dot4.
 * - The sixteen partial tiles are summed through LDS (integer sums: exact in
 *   any order) and the same workgroup applies the expanded offset terms,
 *   gemmlowp's output stage in wrapping int32, the saturating bias add (a plane
 *   of one element is all "tail": no lower clamp,
 *   lowp_SpatialConvolution.c:86-87) and the threshold, and writes y [B][nOut].
 *   No partial sums in global memory, no second launch.
 * - What a wide layer at batch 64 waits for is the path from L2 to the CUs: every workgroup fetches the
 *   activations of all its batch columns, four times the bytes of a row block's weights.  So a workgroup
 *   takes RB row blocks and NCG groups of sixteen columns, gridDim.y slices of the batch: two row blocks x
 *   32 columns for layers of 256 row blocks and more (a fifth fewer bytes than 16 rows x 64 columns for
 *   as many outputs; two row blocks x 64 columns do not fit the 128 registers a thread of 1024 has), and
 *   one row block x 16 columns for layers of fewer row blocks than CUs, which then spread over four
 *   times the CUs.  AlexNet-OWT batch 64: 9216 -> 4096 18.1 -> 14.4 us, 4096 -> 4096 12.2 -> 9.4 us,
 *   4096 -> 1000 10.5 -> 5.8 us.  (Walking the chunks from a different one on in every workgroup, so that
 *   they do not ask for the same activations at the same time, was slower.)
 */
#define LU_THREADS 1024
#define LU_WAVES 16
#define LU_KSTEP 64
#define LU_ROWS 16
#define LU_CHUNK (LU_WAVES * LU_KSTEP)	/* codes per chunk */
#define LU_AHEAD 4			/* chunks of activations in flight (in registers); weights: one fewer */

template <int NCG, int RB>	/* groups of 16 batch columns: batch <= 16 * NCG; 16-row blocks per workgroup */
__global__ __launch_bounds__(LU_THREADS) void linear_u8_kernel(const unsigned char *x, const unsigned char *wfrag,
	const int *rowsum, const int *addend, unsigned char *y, int B, int K, int nOut, int nsteps, int offA, int offB,
	int c_off, int c_mult, int c_shift, int act, int thr, int val)
{
	extern __shared__ __align__(16) unsigned char lds[];	/* two buffers of NCG * 16 KiB */
	/* (gridDim.y slices of 16 NCG batch columns.)  With several slices the workgroups of one row group
	 * are made neighbours on one XCD (workgroup b of the grid's x-fastest order runs on XCD b % 8: the
	 * launch rounds gridDim.x up to a multiple of eight), so that the row group's weights come from memory
	 * once and from that XCD's L2 for the other slices: 4096 -> 1000 at batch 64 fetched 18.7 MB for 4.4 MB
	 * of weights and activations before. */
	int bx = blockIdx.x, by = blockIdx.y;
	if (gridDim.y > 1) {
		const int id = (int)(blockIdx.x + gridDim.x * blockIdx.y), slot = id >> 3;
		by = slot % (int)gridDim.y;
		bx = slot / (int)gridDim.y * 8 + (id & 7);
	}
	if (bx * RB * LU_ROWS >= nOut)
		return;		/* (the padding of gridDim.x) */
	x += (size_t)by * (16 * NCG) * K;
	y += (size_t)by * (16 * NCG) * nOut;
	B = min(B - by * (16 * NCG), 16 * NCG);
	constexpr int XBUF = NCG * 16 * LU_CHUNK;
	const int tid = threadIdx.x, lane = tid & 63;
	/* what this thread needs to finish its outputs (row rr of every row block, batch column bcol), asked
	 * for now: at the end a trip to memory would be all the kernel waits for */
	const int rr = tid & 15, bcol = tid >> 4;
	constexpr bool EARLY = NCG < 4;	/* (four column groups leave no registers for it) */
	int rsum[RB], radd[RB];
	if constexpr (EARLY) {
#pragma unroll
		for (int rb = 0; rb < RB; rb++) {
			const int o = min((bx * RB + rb) * LU_ROWS + rr, nOut - 1);
			rsum[rb] = rowsum[o];
			radd[rb] = addend ? addend[o] : 0;
		}
	}
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int m = lane & 15, q = lane >> 4;
	const int nchunks = (nsteps + LU_WAVES - 1) / LU_WAVES;
	/* uniform bases plus 32-bit lane offsets: the addresses stay on the scalar unit */
	const int nblocks = (nOut + LU_ROWS - 1) / LU_ROWS;
	const unsigned char *wp[RB];	/* (a block past the last one reads the last one again: never stored) */
#pragma unroll
	for (int rb = 0; rb < RB; rb++)
		wp[rb] = wfrag + ((size_t)min(bx * RB + rb, nblocks - 1) * nsteps) * 1024;
	const unsigned woff = lane * 16;
	/* staging: this thread moves piece `lane` of rows wave, wave + 16, ... of a chunk */
	unsigned xsrc[NCG], xdst[NCG];
#pragma unroll
	for (int g = 0; g < NCG; g++) {
		xsrc[g] = (unsigned)min(g * 16 + wave, B - 1) * (unsigned)K + lane * 16;
		xdst[g] = (((lane >> 2) * NCG + g) * 4 + (lane & 3)) * 256 + ((wave ^ lane) & 15) * 16;
	}
	/* fragments: step `wave` of the chunk, group g, quarter q, row m */
	const unsigned fsrc = ((wave * NCG) * 4 + q) * 256 + ((m ^ (wave * 4 + q)) & 15) * 16;
	intx4 acc[RB][NCG];
	int cs[NCG];
#pragma unroll
	for (int g = 0; g < NCG; g++) {
#pragma unroll
		for (int rb = 0; rb < RB; rb++)
			acc[rb][g] = intx4{ 0, 0, 0, 0 };
		cs[g] = 0;
	}
	intx4 a[LU_AHEAD][RB], xr[LU_AHEAD][NCG];
	const intx4 zero_b = { (int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080 };

	/* Requests past the end repeat the last valid address (a hit, and never used), so
	 * the loop body has no divergent branches. */
#define LU_LOAD_A(SLOT_, C_)                                                                       \
	do {                                                                                       \
		const size_t o_ = (size_t)min((C_) * LU_WAVES + wave, nsteps - 1) * 1024 + woff;   \
		_Pragma("unroll") for (int rb = 0; rb < RB; rb++)                                  \
			a[SLOT_][rb] = *(const intx4 *)(wp[rb] + o_);                              \
	} while (0)
#define LU_LOAD_X(SLOT_, C_)                                                                       \
	do {                                                                                       \
		const int k_ = min((C_), nchunks - 1) * LU_CHUNK;                                  \
		const bool ok_ = k_ + lane * 16 < K;	/* K % 16 == 0: a piece is all in or all out */ \
		_Pragma("unroll") for (int g = 0; g < NCG; g++)                                    \
			xr[SLOT_][g] = *(const intx4 *)(x + (ok_ ? k_ + xsrc[g] : 0u));            \
	} while (0)
	/* Staging re-centres the codes (x ^ 0x80) and takes their column sums, so that a
	 * fragment read is followed by its MFMA and nothing else.  Pieces past K are
	 * replaced here, not when they are requested (touching a register that a load is
	 * still filling would wait for the load), and only the last chunk has any. */
#define LU_STAGE(SLOT_, BUF_, C_)                                                                  \
	do {                                                                                       \
		if ((C_) < nchunks) {                                                              \
			const bool tail_ = (C_) == nchunks - 1;                                    \
			const bool ok_ = (C_) * LU_CHUNK + lane * 16 < K;                          \
			_Pragma("unroll") for (int g = 0; g < NCG; g++) {                          \
				intx4 v_ = xr[SLOT_][g];                                           \
				if (tail_)                                                         \
					v_ = ok_ ? v_ : zero_b;                                    \
				_Pragma("unroll") for (int d = 0; d < 4; d++) {                    \
					v_[d] ^= (int)0x80808080;                                  \
					cs[g] = __builtin_amdgcn_sdot4(v_[d], 0x01010101, cs[g], false); \
				}                                                                  \
				*(intx4 *)(lds + (BUF_) * XBUF + xdst[g]) = v_;                    \
			}                                                                          \
		}                                                                                  \
	} while (0)
#define LU_MMA(SLOT_, C_)                                                                          \
	do {                                                                                       \
		if ((C_) * LU_WAVES + wave < nsteps) {                                             \
			intx4 bb_[NCG];                                                            \
			_Pragma("unroll") for (int g = 0; g < NCG; g++)                            \
				bb_[g] = *(const intx4 *)(lds + ((C_) & 1) * XBUF + fsrc + g * 1024); \
			_Pragma("unroll") for (int rb = 0; rb < RB; rb++)                          \
			_Pragma("unroll") for (int g = 0; g < NCG; g++)                            \
				acc[rb][g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[SLOT_][rb], bb_[g], acc[rb][g], 0, 0, 0); \
		}                                                                                  \
	} while (0)

	/* Loads complete in the order they were issued, so waiting for one waits for all
	 * older ones: the activations of a chunk are requested four chunks before they
	 * are staged, the weights three chunks before they are used, and each request
	 * is issued after everything that is needed before it. */
#pragma unroll
	for (int i = 0; i < LU_AHEAD; i++)
		LU_LOAD_X(i, i);
#pragma unroll
	for (int i = 0; i < LU_AHEAD - 1; i++)
		LU_LOAD_A(i, i);
	LU_STAGE(0, 0, 0);
	LU_LOAD_X(0, LU_AHEAD);
	__syncthreads();
	for (int c = 0; c < nchunks; c += LU_AHEAD) {
#pragma unroll
		for (int i = 0; i < LU_AHEAD; i++) {
			/* chunk c + i: its activations are in LDS buffer (c + i) % 2, those of the
			 * following chunks in registers */
			LU_LOAD_A((i + LU_AHEAD - 1) % LU_AHEAD, c + i + LU_AHEAD - 1);
			LU_MMA(i, c + i);
			LU_STAGE((i + 1) % LU_AHEAD, (c + i + 1) & 1, c + i + 1);
			LU_LOAD_X((i + 1) % LU_AHEAD, c + i + 1 + LU_AHEAD);
			__syncthreads();
		}
	}
#undef LU_LOAD_A
#undef LU_LOAD_X
#undef LU_STAGE
#undef LU_MMA

	/* D layout: lane holds column n = lane % 16 of its group, rows 4 * (lane / 16) + r.
	 * Waves 8..15 hand their tiles to waves 0..7, those put the pair sums into LDS,
	 * and every thread finishes one (row, column).  (The loop's last barrier has
	 * passed: the activation buffers are free.) */
	int (*red)[RB][NCG * 4][64] = (int (*)[RB][NCG * 4][64])lds;			/* [8] */
	int *colsum = (int *)(lds + 8 * RB * NCG * 4 * 64 * sizeof(int));		/* [16 * NCG] */
	/* a staging thread summed its pieces of rows wave, wave + 16, ...: the lanes of a
	 * wavefront hold the 64 parts of one column sum */
#pragma unroll
	for (int g = 0; g < NCG; g++) {
		int v = cs[g];
#pragma unroll
		for (int off = 32; off > 0; off >>= 1)
			v += __shfl_xor(v, off, 64);
		if (lane == 0)
			colsum[g * 16 + wave] = v;
	}
	if constexpr (!EARLY) {
#pragma unroll
		for (int rb = 0; rb < RB; rb++) {
			const int o = min((bx * RB + rb) * LU_ROWS + rr, nOut - 1);
			rsum[rb] = rowsum[o];
			radd[rb] = addend ? addend[o] : 0;
		}
	}
	/* (every row block at once: three barriers whatever RB) */
	if (wave >= 8) {
#pragma unroll
		for (int rb = 0; rb < RB; rb++)
#pragma unroll
			for (int gg = 0; gg < NCG; gg++)
#pragma unroll
				for (int r = 0; r < 4; r++)
					red[wave - 8][rb][gg * 4 + r][lane] = acc[rb][gg][r];
	}
	__syncthreads();
	if (wave < 8) {
#pragma unroll
		for (int rb = 0; rb < RB; rb++)
#pragma unroll
			for (int gg = 0; gg < NCG; gg++)
#pragma unroll
				for (int r = 0; r < 4; r++)
					acc[rb][gg][r] += red[wave][rb][gg * 4 + r][lane];
	}
	__syncthreads();
	if (wave < 8) {
#pragma unroll
		for (int rb = 0; rb < RB; rb++)
#pragma unroll
			for (int gg = 0; gg < NCG; gg++)
#pragma unroll
				for (int r = 0; r < 4; r++)
					red[wave][rb][gg * 4 + r][lane] = acc[rb][gg][r];
	}
	__syncthreads();
	/* thread -> (row rr, batch column bcol): neighbouring threads write neighbouring bytes of y */
	const int g = (bcol >> 4) % NCG, n = bcol & 15;	/* (bcol < 16 NCG is checked before use) */
	const int src = (rr >> 2) * 16 + n, reg = g * 4 + (rr & 3);
#pragma unroll
	for (int rb = 0; rb < RB; rb++) {
		const int o = (bx * RB + rb) * LU_ROWS + rr;
		if (bcol >= 16 * NCG || bcol >= B || o >= nOut)
			continue;
		int sum = 0;
#pragma unroll
		for (int wv = 0; wv < 8; wv++)
			sum += red[wv][rb][reg][src];
		const int csum = colsum[bcol];
		const int t = sum + offB * rsum[rb] + K * offA * offB + offA * csum;
		unsigned u = ((unsigned)t + (unsigned)c_off) * (unsigned)c_mult;
		u += c_shift < 1 ? 0u : 1u << (c_shift - 1);
		int code = (int)u >> c_shift;
		code = code < 0 ? 0 : code > 255 ? 255 : code;
		if (addend) {
			const int sa = code + radd[rb];
			code = sa > 255 ? 255 : (sa & 255);
		}
		if (act)
			code = code > thr ? code : val;
		y[(size_t)bcol * nOut + o] = (unsigned char)code;
	}
}

extern "C" int thhip_linear_batched_u8_supported(int B, int K, int nOut)
{
	return B >= 1 && B <= 64 && K % 16 == 0 && K >= 16 && nOut >= 1;
}

/* Device copy of row-major weight codes [nOut][K] in the order linear_u8_kernel
 * streams them: [16-row block][K-step of 64][lane][16 bytes], lane = row % 16 +
 * 16 * (k quarter), re-centred to signed bytes; rows and K padded with zeros. */
extern "C" unsigned char *thhip_linear_pack_weight_u8(const unsigned char *w_host, int nOut, int K)
{
	const int nblocks = (nOut + LU_ROWS - 1) / LU_ROWS, nsteps = (K + LU_KSTEP - 1) / LU_KSTEP;
	const size_t n = (size_t)nblocks * nsteps * 1024;
	unsigned char *h = (unsigned char *)calloc(n, 1);
	for (int o = 0; o < nOut; o++) {
		const unsigned char *src = w_host + (size_t)o * K;
		unsigned char *blk = h + ((size_t)(o / LU_ROWS) * nsteps) * 1024 + (o % LU_ROWS) * 16;
		for (int k = 0; k < K; k++)
			blk[(size_t)(k / LU_KSTEP) * 1024 + ((k % LU_KSTEP) / 16) * 256 + (k % 16)] = src[k] ^ 0x80;
	}
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

extern "C" void thhip_linear_batched_u8(const unsigned char *x, const unsigned char *wfrag, const int *rowsum,
	const int *addend, unsigned char *y, int B, int K, int nOut,
	int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val)
{
	if (!thhip_linear_batched_u8_supported(B, K, nOut))
		THError("thhip_linear_batched_u8: unsupported shape B=%d K=%d nOut=%d", B, K, nOut);
	if (c_shift < 0 || c_shift > 31)
		THError("thhip_linear_batched_u8: shift %d out of range", c_shift);
	const int nblocks = (nOut + LU_ROWS - 1) / LU_ROWS, nsteps = (K + LU_KSTEP - 1) / LU_KSTEP;
	/* algorithmic work for the profiler: 2 nOut K B operations */
	ThhipLaunchScope scope(THHIP_FAM_CONV_I8, 2.0 * nOut * (double)K * B);
	/* Every workgroup fetches the activations of all its batch columns, at batch 64 four times the bytes
	 * of a row block's weights, and the path from L2 to the CUs is what a wide layer waits for: there a
	 * workgroup takes two row blocks and 32 columns (a fifth fewer bytes for as many outputs; two row
	 * blocks and all 64 columns would not fit the 128 registers a thread of 1024 has). */
	const bool square = nblocks >= 256 && B > 32;
	const int rb = square ? 2 : 1;
	/* a narrow layer (fewer row blocks than CUs): slices of 16 or 32 batch columns to more workgroups,
	 * each of which then waits for a quarter or half of the activations only */
	int ncg = square ? 2 : B <= 16 ? 1 : B <= 32 ? 2 : 4;
	if (!square && ncg > 1 && nblocks * ((B + 15) / 16) <= 256)
		ncg = 1;
	else if (!square && ncg > 2 && nblocks * ((B + 31) / 32) <= 256)
		ncg = 2;
	dim3 grid((nblocks + rb - 1) / rb, (B + 16 * ncg - 1) / (16 * ncg)), block(LU_THREADS);
	if (grid.y > 1)
		grid.x = (grid.x + 7) / 8 * 8;	/* (the kernel places the batch slices of a row group on one XCD) */
	/* two activation buffers of NCG * 16 KiB: more than the 64 KiB a kernel gets without asking */
	static bool lds_ok[4];
#define LU_GO(NCG_, RB_, I_) do { \
		const int bytes_ = 2 * NCG_ * 16 * LU_CHUNK; \
		if (!lds_ok[I_]) { \
			hipcheck(hipFuncSetAttribute((const void *)linear_u8_kernel<NCG_, RB_>, hipFuncAttributeMaxDynamicSharedMemorySize, bytes_)); \
			lds_ok[I_] = true; \
		} \
		linear_u8_kernel<NCG_, RB_><<<grid, block, bytes_, thhip_stream()>>>(x, wfrag, rowsum, addend, y, B, K, nOut, \
			nsteps, 128 + a_off, 128 + b_off, c_off, c_mult, c_shift, act, thr, val); \
	} while (0)
	if (square)
		LU_GO(2, 2, 3);
	else if (ncg == 1)
		LU_GO(1, 1, 0);
	else if (ncg == 2)
		LU_GO(2, 1, 1);
	else
		LU_GO(4, 1, 2);
#undef LU_GO
}
