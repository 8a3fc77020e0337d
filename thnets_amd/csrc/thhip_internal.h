/* Internal helpers shared by the .hip translation units (not installed). */
#ifndef THHIP_INTERNAL_H
#define THHIP_INTERNAL_H

#include <hip/hip_runtime.h>
#include "../../include/thnets_hip.h"

/* The HIP counterpart of the reference's errcheck (cudnn/cudnn_th.h:3):
 * a failed runtime call is fatal and names file:line. */
#define hipcheck(f) do { hipError_t rc_ = (f); if (rc_ != hipSuccess) \
	THError("HIP error %d (%s) in %s:%d", (int)rc_, hipGetErrorString(rc_), __FILE__, __LINE__); } while (0)

hipStream_t thhip_stream(void);

/* Profiling hooks: bracket one kernel launch.  `work` is the algorithmic
 * work of the launch (flops for GEMM-like kernels, bytes otherwise). */
int thhip_prof_begin(int family);
void thhip_prof_end(int token, double work);

/* conv_mfma.hip: layout of the weights thhip_conv_pack_weight_u8_layout makes */
int thhip_conv_u8_packed_chunks(int Ci, int kH, int kW, int x_layout);
size_t thhip_conv_u8_packed_code_bytes(int Co, int Ci, int kH, int kW, int x_layout);

/* conv_stem.hip: 3 -> 64 n planes, 3x3, stride 1, padding 1 on plane-major input, read from
 * weights packed by thhip_conv_pack_weight_layout (KC chunks per 32-row block) */
bool thhip_conv_stem_ok(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int dtype, int y_cl);
void thhip_conv_stem(const void *x, const void *wpacked, int KC, const float *scale, const float *bias, void *y,
	int B, int H, int W, int Co, int act, float thr, float val, int dtype, int y_cl);

struct ThhipLaunchScope {
	int token;
	double work;
	ThhipLaunchScope(int family, double w) : token(thhip_prof_begin(family)), work(w) {}
	~ThhipLaunchScope()
	{
		hipcheck(hipGetLastError());
		thhip_prof_end(token, work);
	}
};

static inline int thhip_esize(int dtype)
{
	return dtype == THHIP_F32 ? 4 : dtype == THHIP_U8 ? 1 : 2;
}

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short ushortx8 __attribute__((ext_vector_type(8)));

/* Element load / store in the activation dtype, computing in fp32. */
template <int DT> struct ThhipElem;
template <> struct ThhipElem<THHIP_F32> {
	typedef float T;
	static __device__ __forceinline__ float ld(const void *p, long i) { return ((const float *)p)[i]; }
	static __device__ __forceinline__ void st(void *p, long i, float v) { ((float *)p)[i] = v; }
};
template <> struct ThhipElem<THHIP_F16> {
	typedef _Float16 T;
	static __device__ __forceinline__ float ld(const void *p, long i) { return (float)((const _Float16 *)p)[i]; }
	static __device__ __forceinline__ void st(void *p, long i, float v) { ((_Float16 *)p)[i] = (_Float16)v; }
};
template <> struct ThhipElem<THHIP_BF16> {
	typedef __bf16 T;
	static __device__ __forceinline__ float ld(const void *p, long i) { return (float)((const __bf16 *)p)[i]; }
	static __device__ __forceinline__ void st(void *p, long i, float v) { ((__bf16 *)p)[i] = (__bf16)v; }
};

#define THHIP_DISPATCH_FLOAT(dtype, CALL) do { \
	switch (dtype) { \
	case THHIP_F32: { constexpr int DT = THHIP_F32; CALL; } break; \
	case THHIP_F16: { constexpr int DT = THHIP_F16; CALL; } break; \
	case THHIP_BF16: { constexpr int DT = THHIP_BF16; CALL; } break; \
	default: THError("unsupported dtype %d in %s", (int)(dtype), __func__); \
	} } while (0)

#endif
