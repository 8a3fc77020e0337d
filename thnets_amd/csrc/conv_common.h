/*
 * Shared by the convolution kernels of this library (conv_mfma.hip, conv_half_patch.hip):
 * the launch parameters, the per-type traits and MFMA wrappers, and the explicit
 * waits of the kernels that load their operands straight into LDS.
 */
#ifndef THNETS_AMD_CONV_COMMON_H
#define THNETS_AMD_CONV_COMMON_H
#include <type_traits>
#include "thhip_internal.h"

#define CONV_THREADS 256
#define CONV_C4_SLACK 16	/* bytes before and after the four-plane pixel copy of an input */

struct ConvParams {
	const void *x;
	const void *wp;
	const float *bias;
	const float *scale;	/* float types: per-plane factor applied before the bias (folded batch norm), or NULL */
	void *y;
	int B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, oH, oW;
	int K, KC, N, oHW, HW, kHW;
	unsigned magic_khw, magic_kw, magic_ci;	/* low words of floor(2^32/d)+1 */
	unsigned mhi_khw, mhi_kw, mhi_ci;	/* their bit 32 (set only for d == 1) */
	int act;
	float thr, val;
	int tiles_m, tiles_n;
	int mparts;		/* the tile grid is cut mparts x (8 / mparts) over the XCDs */
	unsigned x_bytes;
	unsigned w_bytes;	/* packed weights (the wide kernel's buffer descriptor) */
	int pool;		/* the 2x2 / stride 2 max pooling that follows is done in the epilogue (conv_patch_kernel, conv_f32_direct_kernel) */
	/* conv_f32_direct_kernel: a second tensor of the output's shape combined with the result after the
	 * (factor,) bias and Threshold: res_mode 1: v + res_c * res, 2: res + res_c * v; then ReLU if res_act
	 * (the table add of a residual block and the Threshold after it, modules/CAddTable.c:59-70) */
	const float *res;
	int res_mode, res_act;
	float res_c;
	int cl_shift;		/* channels-last input in whole K-tiles of planes: log2 of the K-tile (K runs block, tap, plane); else 0 */
	int pW, pHW, npool;	/* pooled width, plane size and positions in all; conv_f32_direct_kernel then walks the
				 * positions in blocks of 64 = sixteen windows (conv_pool_member), N = 64 ceil(npool / 16) */
	unsigned x_tail;	/* uint8: bytes of the padding code that follow x (0: none) */
	/* split-K: S workgroups share an output tile, each over a K range */
	int splitk;
	int *ws;		/* [tile][S][BM*BN] partial accumulators (float or int bits) */
	unsigned *cnt;		/* [tile] arrival counters, zero between launches */
	/* conv_f32_direct_kernel: K split of the last tiles of every XCD only (0 slots: none) */
	int tail_slots;		/* workgroups an XCD holds at once */
	int tail_max;		/* most parts per tile */
	int tail_cap;		/* scratch blocks (parts of BM*BN sums) reserved per XCD: [xcd][tile][part] */
	int tail_tiles;		/* most cut tiles of an XCD */
	int tail_round;		/* 1: an XCD with less than one whole round of tiles is left uncut */
	int tail_inline;	/* 1: the part of a cut tile that arrives last adds the parts and finishes the tile (cnt) */
	unsigned *rot;		/* [64] device words, one per launch in flight: the set of (XCC id - blockIdx.x) % 8 its part workgroups saw */
	int rot_slot, rot_clear;	/* this launch's word, and the word a later launch will use (cleared by this one) */
	int *fault;		/* thhip_fault_flag() */
	/* conv_f32_direct_kernel with a K split of the whole layer: a max pooling that follows, taken by the kernel
	 * that adds the parts (pk_kH 0: none); pk_oH x pk_oW is the pooled plane */
	int pk_kH, pk_kW, pk_dH, pk_dW, pk_padH, pk_padW, pk_oH, pk_oW;
	/* uint8 path only */
	const int *rowsum;	/* sum_k (w[m][k] - 128), per packed row */
	const int *addend;	/* per-plane bias addend, or NULL */
	int zero, offA, offB, c_off, c_mult, c_shift, ithr, ival;
	int kwv;		/* GM_PIXELS4: vectors (four pixels) per kernel row; magic_kw divides by it */
	unsigned c4_fill;	/* GM_PIXELS4: one pixel outside the image */
	/* conv_patch_kernel with the network's image layer in front (img != 0): the three-plane image, plane-major,
	 * that layer's weights as thhip_conv_pack_weight_image_front packs them, its shift, factor and Threshold */
	const void *img, *wstem;
	const float *sbias, *sscale;
	int sact;
	float sthr, sval;
	unsigned img_bytes;
	/* host side only: memory order of x and y, 0 = [B][C][H][W], 1 = [B][H][W][C] */
	int x_cl, y_cl;
};

/* floor(n / d) = (n * m) >> 32 for n*d < 2^32 with the 33-bit m = floor(2^32/d) + 1,
 * evaluated as n*m_hi + umulhi(n, m_lo); m_hi is 1 only for d == 1. */
static inline unsigned long long conv_magic(unsigned d)
{
	return (1ull << 32) / d + 1;
}

/* Chunks per K-tile (one LDS stage).  An int8 MFMA retires 32 k in the time
 * an fp32 one retires 1, so where the gather is cheap (channels-last codes)
 * deeper K-tiles keep the work per barrier up. */
#define CONV_KCH_U8_CL 2
#define CONV_KCH_F32 4
#define CONV_KCH_HALF_CL 2
__host__ __device__ constexpr int conv_kch(int dtype, bool x_cl)
{
	return dtype == THHIP_U8 ? (x_cl ? CONV_KCH_U8_CL : 2) : dtype == THHIP_F32 ? CONV_KCH_F32 : (x_cl ? CONV_KCH_HALF_CL : 2);
}

/* Waves per SIMD to ask the register allocator for (what each tile reaches
 * without spilling): more for the small tiles, whose residency matters most. */
__host__ __device__ constexpr int conv_min_waves(int dtype, int tile_elems, bool generic_gather, int kch)
{
	const bool deep = dtype == THHIP_F32 && kch > 2;	/* fp32 K-tiles of 32: LDS limits first */
	return generic_gather ? 1
		: tile_elems <= 64 * 64 ? (deep ? 3 : 4)
		: tile_elems <= 128 * 64 ? (deep ? 2 : 4)
		: (deep ? 1 : 2);
}

template <int DT> struct ConvTraits;
template <> struct ConvTraits<THHIP_F32> {
	static constexpr int CHUNK = 8;		/* k values per chunk */
	static constexpr int VEC = 4;		/* elements per 16-byte lane vector */
	typedef float elem;
};
template <> struct ConvTraits<THHIP_F16> {
	static constexpr int CHUNK = 16;
	static constexpr int VEC = 8;
	typedef _Float16 elem;
};
template <> struct ConvTraits<THHIP_BF16> {
	static constexpr int CHUNK = 16;
	static constexpr int VEC = 8;
	typedef __bf16 elem;
};

template <> struct ConvTraits<THHIP_U8> {
	static constexpr int CHUNK = 32;
	static constexpr int VEC = 16;
	typedef unsigned char elem;
};

template <int DT> struct ConvAcc { typedef floatx16 T; };
template <> struct ConvAcc<THHIP_U8> { typedef intx16 T; };

template <int DT>
__device__ __forceinline__ void conv_mma(typename ConvAcc<DT>::T &acc, const floatx4 &a, const floatx4 &b);

template <>
__device__ __forceinline__ void conv_mma<THHIP_F32>(floatx16 &acc, const floatx4 &a, const floatx4 &b)
{
	acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], acc, 0, 0, 0);
	acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], acc, 0, 0, 0);
	acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], acc, 0, 0, 0);
	acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], acc, 0, 0, 0);
}

template <>
__device__ __forceinline__ void conv_mma<THHIP_F16>(floatx16 &acc, const floatx4 &a, const floatx4 &b)
{
	acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), acc, 0, 0, 0);
}

template <>
__device__ __forceinline__ void conv_mma<THHIP_BF16>(floatx16 &acc, const floatx4 &a, const floatx4 &b)
{
	acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}

template <>
__device__ __forceinline__ void conv_mma<THHIP_U8>(intx16 &acc, const floatx4 &a, const floatx4 &b)
{
	acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), acc, 0, 0, 0);
}

#define WIDE_LDS(p) ((__attribute__((address_space(3))) void *)(p))
/* s_waitcnt immediate that waits for all but n vector-memory operations only */
#define WIDE_VMCNT(n) (0x0f70 | ((n) & 15) | (((n) >> 4) << 14))

/* Waits until at most N vector-memory operations of the wave are outstanding
 * (LGKM0: and no LDS / scalar ones).  The builtin wants a literal: a value that
 * depends on a template parameter makes the host pass drop the kernel. */
template <int N, bool LGKM0>
__device__ __forceinline__ void wide_wait()
{
	static_assert(N >= 0 && N <= 48, "add the count below");
#define WIDE_WAIT_CASE(n)                                                          \
	if constexpr (N == n) {                                                    \
		if constexpr (LGKM0)                                               \
			__builtin_amdgcn_s_waitcnt(WIDE_VMCNT(n) & 0xf0ff);        \
		else                                                               \
			__builtin_amdgcn_s_waitcnt(WIDE_VMCNT(n));                 \
	}
	WIDE_WAIT_CASE(0)
	WIDE_WAIT_CASE(1)
	WIDE_WAIT_CASE(2)
	WIDE_WAIT_CASE(3)
	WIDE_WAIT_CASE(4)
	WIDE_WAIT_CASE(5)
	WIDE_WAIT_CASE(6)
	WIDE_WAIT_CASE(7)
	WIDE_WAIT_CASE(8)
	WIDE_WAIT_CASE(9)
	WIDE_WAIT_CASE(10)
	WIDE_WAIT_CASE(11)
	WIDE_WAIT_CASE(12)
	WIDE_WAIT_CASE(13)
	WIDE_WAIT_CASE(14)
	WIDE_WAIT_CASE(15)
	WIDE_WAIT_CASE(16)
	WIDE_WAIT_CASE(17)
	WIDE_WAIT_CASE(18)
	WIDE_WAIT_CASE(19)
	WIDE_WAIT_CASE(20)
	WIDE_WAIT_CASE(21)
	WIDE_WAIT_CASE(22)
	WIDE_WAIT_CASE(23)
	WIDE_WAIT_CASE(24)
	WIDE_WAIT_CASE(25)
	WIDE_WAIT_CASE(26)
	WIDE_WAIT_CASE(27)
	WIDE_WAIT_CASE(28)
	WIDE_WAIT_CASE(29)
	WIDE_WAIT_CASE(30)
	WIDE_WAIT_CASE(31)
	WIDE_WAIT_CASE(32)
	WIDE_WAIT_CASE(33)
	WIDE_WAIT_CASE(34)
	WIDE_WAIT_CASE(35)
	WIDE_WAIT_CASE(36)
	WIDE_WAIT_CASE(37)
	WIDE_WAIT_CASE(38)
	WIDE_WAIT_CASE(39)
	WIDE_WAIT_CASE(40)
	WIDE_WAIT_CASE(41)
	WIDE_WAIT_CASE(42)
	WIDE_WAIT_CASE(43)
	WIDE_WAIT_CASE(44)
	WIDE_WAIT_CASE(45)
	WIDE_WAIT_CASE(46)
	WIDE_WAIT_CASE(47)
	WIDE_WAIT_CASE(48)
#undef WIDE_WAIT_CASE
}

/* Channels-last stores of a 32x32 accumulator.  Lane l holds, for position
 * l % 32, the four planes 4 (l / 32) + 8 g + e of group g = 0..3: stored as it
 * lies, an instruction writes 64 separate pieces of four values.
 * v_permlane32_swap(x, y) exchanges x of lanes 32..63 with y of lanes 0..31, so
 * after it the low lane owns both halves of x's group and the high lane both
 * halves of y's: every lane then writes 16 bytes, in half (uint8: a quarter)
 * as many instructions, and lanes l and l + 32 write neighbouring pieces.
 * Every lane of the wave must take part (no divergence around the calls). */
__device__ __forceinline__ void conv_swap32(unsigned &x, unsigned &y)
{
	const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
	x = r[0];
	y = r[1];
}

/* Half types: lo[g], hi[g] = planes 0..1 and 2..3 of group g as packed pairs.
 * yn points at the position's plane 0 of this accumulator's 32 planes; planes
 * from `left` on do not exist (left % 8 == 0, rows 16-byte aligned). */
__device__ __forceinline__ void conv_store_cl_half(unsigned short *yn, int left, bool valid, unsigned (&lo)[4], unsigned (&hi)[4], int lane)
{
#pragma unroll
	for (int h = 0; h < 2; h++) {
		conv_swap32(lo[2 * h], lo[2 * h + 1]);
		conv_swap32(hi[2 * h], hi[2 * h + 1]);
		const int m = 16 * h + 8 * (lane >> 5);
		if (valid && m < left) {
			uintx4 v = { lo[2 * h], hi[2 * h], lo[2 * h + 1], hi[2 * h + 1] };
			*(uintx4 *)(yn + m) = v;
		}
	}
}

/* conv_patch_kernel's output tile (positions of one image) */
#define PATCH_TW 32
#define PATCH_TH 8

/* conv_half_patch.hip: the half types' 3x3 / stride 1 layers with their taps read from an input patch in LDS */
bool thhip_conv_half_patch_ok(const ConvParams &p, int dtype);
bool thhip_conv_half_patch_flat_ok(const ConvParams &p, int dtype);
void thhip_conv_half_patch_launch(ConvParams &p, int dtype, int bm, int flat);

#endif
