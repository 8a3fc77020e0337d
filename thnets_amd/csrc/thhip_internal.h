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

/* s_getreg operand of the XCC id (hardware register 20, bits 0 .. 3): the XCD this wave runs on */
#define THHIP_GETREG_XCC_ID ((3 << 11) | 20)
extern "C" unsigned thhip_xcd_map(void);	/* hip_rt.hip: 0x80000000 | r where workgroup b of a probe launch ran on XCD (b + r) % 8 for every b; 0 otherwise */
extern "C" int *thhip_fault_flag(void);		/* hip_rt.hip: set by a kernel, turned into an error at the next synchronisation */
extern "C" void thhip_fault_hold(int on);	/* hip_rt.hip: 1: the error is held back for thhip_fault_take() */
extern "C" int thhip_fault_take(void);		/* hip_rt.hip: the fault reported while errors were held back (0: none); clears it */
extern "C" void thhip_conv_parts_fault(void);	/* conv_mfma.hip: what a report of fault 1 switches off */
extern "C" int thhip_batch_window_get(int *b0);	/* hip_rt.hip: the images [b0, b0 + n) the convolutions are to work on (n = 0: all) */
extern "C" void thhip_batch_window_scope(int on);	/* hip_rt.hip: 1 while code that honours the window launches */
extern "C" void thhip_batch_window_violate(void);	/* hip_rt.hip: this call works on the whole batch in spite of a window */

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

/* ---- test and tuning hooks: process-wide switches of the kernel choice, exported from the library
 * for the tests and the tuning scripts but not part of the installed interface ---- */
extern "C" {
/* Tuning override for tests and experiments: force the convolution's workgroup
 * tile (bm x bn in {64,128}), its split-K factor and the number of workgroups
 * allowed to share a CU; 0 leaves a choice automatic.  A forced tile runs on
 * the kernel that stages its operands through registers, except:
 *   splitk == 9 asks for the kernels that load their operands straight into
 *     LDS (no K split of the whole layer there): half types and uint8 with channels-last input,
 *     tiles 64x64, 128x64, 64x128, 128x128; fp32 plane-major with Ci % 32 == 0,
 *     tiles 64x64 and 128x64, wgs_per_cu == 2 selecting K-tiles of 16 values;
 *   bn == 256 (half types): the 256x256 and 128x256 tiles of the same kernel
 *     (splitk == 4 with bm == 256: K-tiles of 64 values in two stages);
 *   (64, 1): the half-type kernel for 3x3 stride-1 layers of 64, 128, 256 or 512 planes
 *     that keeps an input patch in LDS.
 * A layer the forced kernel cannot take ends in THError. */
void thhip_conv_set_tuning(int bm, int bn, int splitk, int wgs_per_cu);
/* fp32 only: force K-tiles of 16 values (chunks = 2) or 32 (4); 0 restores the
 * per-layer choice.  Tests and tuning, like thhip_conv_set_tuning. */
void thhip_conv_set_ktile(int chunks);
/* fp32 and half-type tiles loaded straight into LDS, layers without a K split
 * of their own: the tiles an XCD cannot spread evenly over its CUs (its tile
 * count modulo the workgroups it holds at once; half types: only after at
 * least one whole round) are dispatched last and cut along K into up to
 * `parts` parts of at least eight K-tiles, summed in their order by a small
 * kernel (results do not depend on timing).  Default 8, which is also the most
 * that is used; 1 = never cut.  Tests and tuning. */
void thhip_conv_set_tail_parts(int parts);
/* th_engine.c: forward passes so far whose first modules ran window by window under THProcessFloat */
long thhip_windowed_forwards(void);
/* launches so far whose cut tiles were added in the kernel (0) / by a second launch (1) */
long thhip_conv_cut_launches(int second_launch);
/* Force how the tile grid is cut over the eight XCDs: the M tiles into
 * mparts (1, 2, 4, 8) groups, the N tiles into 8 / mparts ranges; 0 restores
 * the choice by weight size.  Tests and tuning. */
void thhip_conv_set_xcd_parts(int mparts);
/* Channels-last inputs whose plane count is a multiple of the K-tile are
 * gathered with the filter tap tracked on the scalar unit; on = 1 forces the
 * per-thread tap decode that serves every plane count.  Tests and tuning. */
void thhip_conv_set_generic_cl(int on);
/* Tests and tuning: 16-row blocks a wavefront of thhip_linear_batched owns
 * (1 or 4); 0 restores the choice by the layer's width. */
void thhip_linear_batched_set_tuning(int row_blocks);
}

/* conv_f32_image.hip: an fp32 image layer (<= 4 planes, plane-major) with factor, shift, Threshold and a
 * 3x3 / stride 2 max pooling in one kernel; weights packed by thhip_conv_pack_weight_layout for plane-major input */
bool thhip_conv_image_pool_f32_ok(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode, int dtype);
void thhip_conv_image_pool_f32(const float *x, const float *wpacked, int KC, const float *scale, const float *bias, float *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int ppad,
	int act, float thr, float val);

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
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
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
