/*
 * Batch-1 Linear as an HBM-bandwidth kernel.
 *
 * Replaces nn_Linear_updateOutput's vector branch (modules/Linear.c:86-90),
 * i.e. output = bias, then addmv -> sgemv('t') -> sgemv_t
 * (thbasic.c:713-741, OpenBLAS-stripped/sgemv.c:48-105, gemv_t.c:51-63):
 * y[j] = bias[j] + sum_i W[j][i] * x[i].
 *
 * The weight matrix is read exactly once (nOut*nIn elements, the whole
 * cost); x is tiny and stays in cache.  A workgroup owns ROWS consecutive
 * rows; its 256 lanes stride through K with 16-byte loads, several in flight
 * per lane, then reduce across the wavefront with cross-lane shuffles and
 * across the four wavefronts through LDS.  The optional Threshold of the next
 * module is applied to the finished sum.
 */
#include "thhip_internal.h"

#define GEMV_THREADS 256

template <int DT> struct GemvVec;
template <> struct GemvVec<THHIP_F32> {
	static constexpr int N = 4;
	static __device__ __forceinline__ void load(const void *p, long vec_index, float *out)
	{
		floatx4 v = ((const floatx4 *)p)[vec_index];
		out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3];
	}
};
template <> struct GemvVec<THHIP_F16> {
	static constexpr int N = 8;
	static __device__ __forceinline__ void load(const void *p, long vec_index, float *out)
	{
		halfx8 v = ((const halfx8 *)p)[vec_index];
#pragma unroll
		for (int i = 0; i < 8; i++)
			out[i] = (float)v[i];
	}
};
template <> struct GemvVec<THHIP_BF16> {
	static constexpr int N = 8;
	static __device__ __forceinline__ void load(const void *p, long vec_index, float *out)
	{
		bf16x8 v = ((const bf16x8 *)p)[vec_index];
#pragma unroll
		for (int i = 0; i < 8; i++)
			out[i] = (float)v[i];
	}
};

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		v += __shfl_xor(v, off, 64);
	return v;
}

template <int DT, int ROWS>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(const void *x, const void *w, const float *bias, void *y,
	int nIn, int nOut, int act, float thr, float val)
{
	typedef GemvVec<DT> V;
	constexpr int VN = V::N;
	const int tid = threadIdx.x;
	const int row0 = blockIdx.x * ROWS;
	const long nvec = nIn / VN;		/* whole vectors per row (rows are 16-byte aligned when nIn % VN == 0) */
	const bool aligned = (nIn % VN) == 0;
	float acc[ROWS];
#pragma unroll
	for (int r = 0; r < ROWS; r++)
		acc[r] = 0.0f;

	if (aligned) {
		for (long v = tid; v < nvec; v += GEMV_THREADS) {
			float xv[VN];
			V::load(x, v, xv);
#pragma unroll
			for (int r = 0; r < ROWS; r++) {
				const int row = row0 + r < nOut ? row0 + r : nOut - 1;
				float wv[VN];
				V::load(w, (long)row * nvec + v, wv);
#pragma unroll
				for (int i = 0; i < VN; i++)
					acc[r] += wv[i] * xv[i];
			}
		}
	} else {
		for (long i = tid; i < nIn; i += GEMV_THREADS) {
			const float xi = ThhipElem<DT>::ld(x, i);
#pragma unroll
			for (int r = 0; r < ROWS; r++) {
				const int row = row0 + r < nOut ? row0 + r : nOut - 1;
				acc[r] += ThhipElem<DT>::ld(w, (long)row * nIn + i) * xi;
			}
		}
	}

	__shared__ float part[ROWS][GEMV_THREADS / 64];
#pragma unroll
	for (int r = 0; r < ROWS; r++) {
		float s = wave_sum(acc[r]);
		if ((tid & 63) == 0)
			part[r][tid >> 6] = s;
	}
	__syncthreads();
	if (tid < ROWS && row0 + tid < nOut) {
		float s = (part[tid][0] + part[tid][1]) + (part[tid][2] + part[tid][3]);
		s += bias ? bias[row0 + tid] : 0.0f;
		if (act)
			s = s > thr ? s : val;
		ThhipElem<DT>::st(y, row0 + tid, s);
	}
}

template <int DT>
static void gemv_dispatch(const void *x, const void *w, const float *bias, void *y, int nIn, int nOut, int act,
	float thr, float val)
{
	/* enough workgroups to cover 256 CUs several times; fewer rows per group
	 * for short matrices */
	if (nOut >= 8192) {
		dim3 grid((nOut + 3) / 4);
		gemv_kernel<DT, 4><<<grid, dim3(GEMV_THREADS), 0, thhip_stream()>>>(x, w, bias, y, nIn, nOut, act, thr, val);
	} else if (nOut >= 2048) {
		dim3 grid((nOut + 1) / 2);
		gemv_kernel<DT, 2><<<grid, dim3(GEMV_THREADS), 0, thhip_stream()>>>(x, w, bias, y, nIn, nOut, act, thr, val);
	} else {
		dim3 grid(nOut);
		gemv_kernel<DT, 1><<<grid, dim3(GEMV_THREADS), 0, thhip_stream()>>>(x, w, bias, y, nIn, nOut, act, thr, val);
	}
}

extern "C" void thhip_gemv(const void *x, const void *w, const float *bias, void *y,
	int nIn, int nOut, int act, float thr, float val, int dtype)
{
	if (nIn < 1 || nOut < 1)
		THError("thhip_gemv: bad sizes %d x %d", nOut, nIn);
	/* algorithmic bytes: the matrix, the vector, bias and result */
	const double esz = thhip_esize(dtype);
	ThhipLaunchScope scope(THHIP_FAM_GEMV, esz * ((double)nOut * nIn + nIn + nOut) + 4.0 * nOut);
	THHIP_DISPATCH_FLOAT(dtype, gemv_dispatch<DT>(x, w, bias, y, nIn, nOut, act, thr, val));
}
