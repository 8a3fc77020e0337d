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
 * wavefront owns 16 output rows and a slice of K: lane (m = lane%16,
 * q = lane/16) streams 64 contiguous bytes of row m per step (four 16-byte
 * loads, k = k0 + 16q + 4j + s), the matching lane of the B operand reads the
 * same k of batch row n = lane%16 (X is small and stays in L2), and 16 MFMAs
 * contract them.  K is split over the four wavefronts of a workgroup (summed
 * through LDS) and over gridDim.y workgroups (partials in a scratch buffer,
 * summed by a second tiny kernel that also applies bias and Threshold).
 */
#include "thhip_internal.h"

#define SK_THREADS 256
#define SK_KSTEP 64

template <int NB>	/* NB 16-column groups: batch <= 16 * NB */
__global__ __launch_bounds__(SK_THREADS) void skinny_kernel(const float *x, const float *w, float *part,
	int B, int nIn, int nOut, int ksplit)
{
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int m = lane & 15, q = lane >> 4;
	const int row0 = blockIdx.x * 16;
	const int row = min(row0 + m, nOut - 1);
	/* K-steps of 64 are dealt round-robin to (workgroup slice, wave) */
	const int nsteps = (nIn + SK_KSTEP - 1) / SK_KSTEP;
	const int stride = ksplit * 4;
	const float *wr = w + (size_t)row * nIn;
	const float *xr[NB];
#pragma unroll
	for (int g = 0; g < NB; g++)
		xr[g] = x + (size_t)min(g * 16 + m, B - 1) * nIn;

	floatx4 acc[NB];
#pragma unroll
	for (int g = 0; g < NB; g++)
		acc[g] = floatx4{ 0, 0, 0, 0 };

	for (int st = blockIdx.y * 4 + wave; st < nsteps; st += stride) {
		const int kb = st * SK_KSTEP + q * 16;
		floatx4 a[4], b[NB][4];
#pragma unroll
		for (int j = 0; j < 4; j++) {
			const int k = kb + j * 4;
			const bool ok = k < nIn;	/* nIn % 4 == 0: a vector is all in or all out */
			a[j] = ok ? *(const floatx4 *)(wr + k) : floatx4{ 0, 0, 0, 0 };
#pragma unroll
			for (int g = 0; g < NB; g++)
				b[g][j] = ok ? *(const floatx4 *)(xr[g] + k) : floatx4{ 0, 0, 0, 0 };
		}
#pragma unroll
		for (int j = 0; j < 4; j++)
#pragma unroll
			for (int s = 0; s < 4; s++)
#pragma unroll
				for (int g = 0; g < NB; g++)
					acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j][s], b[g][j][s], acc[g], 0, 0, 0);
	}

	/* D layout: lane holds column n = lane%16, rows 4*(lane/16) + r */
	__shared__ float red[4][NB][16][17];
#pragma unroll
	for (int g = 0; g < NB; g++)
#pragma unroll
		for (int r = 0; r < 4; r++)
			red[wave][g][q * 4 + r][m] = acc[g][r];
	__syncthreads();
	for (int i = tid; i < NB * 256; i += SK_THREADS) {
		const int g = i >> 8, rr = (i >> 4) & 15, n = i & 15;
		const int o = row0 + rr, bcol = g * 16 + n;
		if (o < nOut && bcol < B) {
			const float s = (red[0][g][rr][n] + red[1][g][rr][n]) + (red[2][g][rr][n] + red[3][g][rr][n]);
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

extern "C" int thhip_linear_batched_supported(int B, int nIn, int nOut, int dtype)
{
	return dtype == THHIP_F32 && B >= 1 && B <= 32 && nIn % 4 == 0 && nIn >= 4 && nOut >= 1;
}

extern "C" void thhip_linear_batched(const void *x, const void *wrow, const float *bias, void *y,
	int B, int nIn, int nOut, int act, float thr, float val, int dtype)
{
	if (!thhip_linear_batched_supported(B, nIn, nOut, dtype))
		THError("thhip_linear_batched: unsupported shape B=%d nIn=%d nOut=%d dtype=%d", B, nIn, nOut, dtype);
	const int groups = (nOut + 15) / 16;
	const int nsteps = (nIn + SK_KSTEP - 1) / SK_KSTEP;
	/* aim at ~4096 wavefronts, at least two K-steps per wavefront */
	int ksplit = (1024 + groups - 1) / groups;
	if (ksplit > nsteps / 8)
		ksplit = nsteps / 8;
	if (ksplit < 1)
		ksplit = 1;
	if (ksplit > 64)
		ksplit = 64;
	float *part = skinny_scratch((size_t)ksplit * B * nOut * sizeof(float));
	{
		/* algorithmic bytes: W once, X once, Y once */
		ThhipLaunchScope scope(THHIP_FAM_GEMV, 4.0 * ((double)nOut * nIn + (double)B * nIn + (double)B * nOut));
		dim3 grid(groups, ksplit);
		if (B <= 16)
			skinny_kernel<1><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>((const float *)x, (const float *)wrow, part,
				B, nIn, nOut, ksplit);
		else
			skinny_kernel<2><<<grid, dim3(SK_THREADS), 0, thhip_stream()>>>((const float *)x, (const float *)wrow, part,
				B, nIn, nOut, ksplit);
	}
	{
		ThhipLaunchScope scope(THHIP_FAM_OTHER, 4.0 * (ksplit + 1.0) * B * nOut);
		long total = (long)B * nOut;
		long blocks = (total + 255) / 256;
		skinny_finish_kernel<THHIP_F32><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(part, bias, y, B, nOut,
			ksplit, act, thr, val);
	}
}
