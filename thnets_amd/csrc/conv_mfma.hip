/*
 * Implicit-GEMM convolution for gfx950 on the matrix cores.
 *
 * Replaces the reference's per-image im2col + SGEMM + bias fill
 * (modules/SpatialConvolutionMM.c:11-109, thbasic.c:601-711, 1073-1103,
 * OpenBLAS-stripped/sgemm.c) and the Threshold module that usually follows
 * (modules/Threshold.c:38-63) with one kernel:
 *
 *     C[M = Co][N = B*oH*oW] = Wp[M][K = Ci*kH*kW] * im2col(x)[K][N]
 *
 * The im2col matrix is never materialised: each workgroup gathers its
 * K-tile x N-tile slab straight from the NCHW input (lanes run along the
 * output row, so loads coalesce along W), zero-filling the padding, and
 * stages it through LDS.  Weights are pre-packed once at engine creation
 * into the exact order the LDS tile wants, so their loads are 16-byte,
 * fully coalesced and written to LDS unchanged.
 *
 * Fragment layout.  K is cut into chunks (8 values for fp32, 16 for
 * fp16/bf16); within a chunk, lane half h = lane/32 owns the contiguous
 * sub-range [h*C/2, (h+1)*C/2) as ONE 16-byte vector, for row (A) or column
 * (B) lane%32.  A 32x32x2 fp32 MFMA contracts the two lane halves, so step s
 * of a chunk uses element s of every lane's vector; a 32x32x16 half MFMA
 * consumes the whole vector.  The contraction order inside a chunk is thus
 * permuted relative to k, which a sum does not care about.  Both LDS tiles
 * are stored [chunk][32-row block][h][32][16 B]: every ds_read_b128 /
 * ds_write_b128 of a wave touches 1 KiB contiguous, i.e. no bank conflicts.
 */
#include <float.h>
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include <vector>
#include "thhip_internal.h"

#include "conv_common.h"

/* gemmlowp's legacy output stage as the reference calls it (lowp/gemm8.cc:13-16):
 * ((acc + c_off) * c_mult + rounding) >> c_shift in wrapping 32-bit arithmetic,
 * arithmetic shift, saturated to a byte. */
__device__ __forceinline__ int conv_requant(int acc, int c_off, int c_mult, int c_shift)
{
	unsigned u = ((unsigned)acc + (unsigned)c_off) * (unsigned)c_mult;
	u += c_shift < 1 ? 0u : 1u << (c_shift - 1);
	int t = (int)u >> c_shift;
	return t < 0 ? 0 : t > 255 ? 255 : t;
}

/* uint8: w[g] = the four codes of group g; left % 16 == 0. */
__device__ __forceinline__ void conv_store_cl_u8(unsigned char *yn, int left, bool valid, unsigned (&w)[4], int lane)
{
	conv_swap32(w[0], w[1]);
	conv_swap32(w[2], w[3]);
	conv_swap32(w[0], w[2]);
	conv_swap32(w[1], w[3]);
	const int m = 16 * (lane >> 5);
	if (valid && m < left) {
		uintx4 v = { w[0], w[1], w[2], w[3] };
		*(uintx4 *)(yn + m) = v;
	}
}

/* Scalar (wave-uniform) decode of k -> offset of tap (c,kh,kw) in the image. */
struct KTap { int koff, kh, kw; };

__device__ __forceinline__ KTap conv_ktap(const ConvParams &p, int k)
{
	KTap t;
	const unsigned c = (unsigned)k * p.mhi_khw + __umulhi((unsigned)k, p.magic_khw);
	const unsigned rem = k - c * p.kHW;
	const unsigned kh = rem * p.mhi_kw + __umulhi(rem, p.magic_kw);
	t.kh = kh;
	t.kw = rem - kh * p.kW;
	t.koff = c * p.HW + t.kh * p.W + t.kw;
	t.kh = k < p.K ? t.kh : 0x40000000;	/* K padding: forces the bounds test to fail */
	return t;
}

/* GM, how the B operand is gathered: */
enum { GM_PLANE_TAP, GM_TAP_MAJOR, GM_CHANNELS_LAST, GM_PIXELS4, GM_CL_UNIFORM };
/* GM_CL_UNIFORM is GM_CHANNELS_LAST for Ci a multiple of the K-tile depth: a
 * K-tile then lies inside one filter tap, the tap is the same for every thread
 * and is tracked on the scalar unit, and K has no padding. */

template <int DT, int BM, int BN, int WGM, int WGN, int GM, bool CLO, int KCH>
__global__ __launch_bounds__(CONV_THREADS)
/* ask for four waves per SIMD where the tile allows it: without the hint the
 * compiler spreads the accumulators over AGPRs plus a generous VGPR budget and
 * halves the number of workgroups a CU can hold */
__attribute__((amdgpu_waves_per_eu(conv_min_waves(DT, BM * BN, GM == 0, KCH), 8))) void conv_mfma_kernel(ConvParams p)
{
	constexpr bool TAP = GM == GM_TAP_MAJOR;
	constexpr bool C4 = GM == GM_PIXELS4;		/* uint8, <= 4 planes, re-laid out as [B][H][W][4] */
	constexpr bool CLU = GM == GM_CL_UNIFORM;
	constexpr bool CLI = GM == GM_CHANNELS_LAST || C4 || CLU;
	static_assert(!C4 || DT == THHIP_U8, "the four-plane pixel layout is a uint8 path");
	typedef ConvTraits<DT> TR;
	typedef typename TR::elem elem;
	constexpr int CHUNK = TR::CHUNK, VEC = TR::VEC;
	/* KCH chunks per K-tile (one LDS stage).  Weights are packed in blocks of
	 * PKCH chunks; a shallower K-tile walks a block in SUB steps (more, smaller
	 * stages: more workgroups per CU, which the widest layers prefer). */
	constexpr int PKCH = conv_kch(DT, CLI), SUB = PKCH / KCH;
	static_assert(PKCH % KCH == 0 && KCH % 2 == 0, "K-tile depth");
	constexpr int MB = BM / 32, NB = BN / 32;		/* 32-row blocks per tile */
	constexpr int TM = BM / WGM / 32, TN = BN / WGN / 32;	/* MFMA tiles per wave */
	constexpr int A_VECS = MB * KCH * 64;			/* 16-byte vectors per K-tile (KCH chunks) */
	constexpr int B_VECS = NB * KCH * 64;
	constexpr int A_PER_WAVE = MB * KCH / 4;		/* 1 KiB blocks loaded per wave */
	constexpr int B_PER_THREAD = BN * KCH / 128;		/* (chunk,h) vectors gathered per thread */
	static_assert(WGM * WGN == 4, "four waves per workgroup");
	static_assert(MB * KCH % 4 == 0 && BN % 64 == 0, "tile shape");

	constexpr int STAGE_VECS = A_VECS + B_VECS;
	__shared__ floatx4 lds[3 * STAGE_VECS];		/* three K-tile stages */

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave % WGM, wn = wave / WGM;

	/* XCD-aware tile order.  Workgroups are dealt round-robin to the 8 XCDs,
	 * each with its own L2, so every XCD gets one rectangle of the tile grid:
	 * the M tiles are cut into p.mparts groups and the N tiles into 8 / mparts
	 * ranges.  One part along M (every XCD: all weight rows, an eighth of the
	 * positions) reads the least in total, but an XCD's workgroups all run at
	 * once and sweep every weight row they own, so the launcher raises mparts
	 * until an XCD's share of the weights fits its L2.  Inside the rectangle
	 * M runs fastest: neighbours share an input slab. */
	int tile_m, tile_n, split = 0;
	{
		const int bid = blockIdx.x;
		const int xcd = bid & 7;
		int local = bid >> 3;
		if (p.splitk > 1) {	/* the S parts of a tile are neighbours in the order */
			split = local % p.splitk;
			local /= p.splitk;
		}
		const int mp = xcd % p.mparts, np = xcd / p.mparts, nparts = 8 / p.mparts;
		const int m0 = p.tiles_m * mp / p.mparts, m1 = p.tiles_m * (mp + 1) / p.mparts;
		const int n0 = p.tiles_n * np / nparts, n1 = p.tiles_n * (np + 1) / nparts;
		const int mw = m1 - m0;
		if (local >= mw * (n1 - n0))
			return;		/* the rectangles differ by a row or column: this slot is empty */
		tile_m = m0 + local % mw;
		tile_n = n0 + local / mw;
	}
	const int tile = tile_n * p.tiles_m + tile_m;	/* names the tile's split-K scratch */

	/* ---- B gather role ----
	 * Plane-major input: one output position per thread (lanes run along the
	 * output row, so element loads coalesce along W); the 256/BN threads of a
	 * position take different (chunk, half) vectors.
	 * Channels-last input: the 2*KCH vectors of a position's K-tile slice are
	 * adjacent in memory (whole runs of Ci bytes per tap), so eight
	 * neighbouring lanes take the eight vectors of one position and a wave's
	 * load touches few cache lines; a thread then serves B_PER_THREAD positions. */
	constexpr int VPP = 2 * KCH;			/* vectors per position per K-tile */
	constexpr int PPI = CONV_THREADS / VPP;		/* positions per pass (CLI) */
	constexpr int NPOS = CLI ? B_PER_THREAD : 1;
	static_assert(!CLI || BN % PPI == 0, "tile shape");
	const int n_local = CLI ? tid / VPP : tid % BN;
	const int slot = __builtin_amdgcn_readfirstlane(tid / BN);
	const int pv = tid % VPP;			/* (CLI) this thread's vector */
	bool n_ok_[NPOS];
	int iy0_[NPOS], ix0_[NPOS], xoff_[NPOS];
	int xmask_[NPOS];	/* (CLU, uint8) what a vector outside the image is XORed with */
#pragma unroll
	for (int q = 0; q < NPOS; q++) {
		const int n_glob = tile_n * BN + n_local + q * PPI;
		n_ok_[q] = n_glob < p.N;
		int nn = n_ok_[q] ? n_glob : 0;
		int b = nn / p.oHW, r = nn - b * p.oHW;
		int oy = r / p.oW, ox = r - oy * p.oW;
		iy0_[q] = oy * p.dH - p.padH;
		ix0_[q] = ox * p.dW - p.padW;
		if constexpr (C4)
			xoff_[q] = ((b * p.H + iy0_[q]) * p.W + ix0_[q]) * 4 + CONV_C4_SLACK;
		else if constexpr (CLU)	/* byte offset of this thread's vector at tap (0,0), plane block 0 */
			xoff_[q] = (((b * p.H + iy0_[q]) * p.W + ix0_[q]) * p.Ci + (tid % (2 * KCH)) * VEC) * (int)sizeof(elem);
		else if constexpr (CLI)
			xoff_[q] = ((b * p.H + iy0_[q]) * p.W + ix0_[q]) * p.Ci;
		else
			xoff_[q] = b * p.Ci * p.HW + iy0_[q] * p.W + ix0_[q];
		/* a load outside the image returns 0; XORed with this it becomes the
		 * re-centred padding code (0 for columns past N) */
		xmask_[q] = ((n_ok_[q] ? p.zero : 128) * 0x01010101) ^ (int)0x80808080;
	}
	const bool n_ok = n_ok_[0];
	const int iy0 = iy0_[0], ix0 = ix0_[0], xoff = xoff_[0];
	const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes, 0x00020000);

	const floatx4 *wp = (const floatx4 *)p.wp;
	/* K-tiles on their way from global memory to LDS: PFD register sets, the
	 * oldest in set 0.  The scalar tap walk leaves registers free and the half /
	 * int8 K-tiles are short, so that path holds a tile one step longer before
	 * it goes to LDS (measured: 10 % on the int8 layers, nothing on fp16). */
	constexpr int PFD = CLU ? 2 : 1;
	floatx4 areg[PFD][A_PER_WAVE];
	floatx4 breg[PFD][B_PER_THREAD];
	int bmask[PFD][B_PER_THREAD];	/* (CLU, uint8) re-centring mask of each vector, applied on the way to LDS */
	int colsum[NPOS];	/* uint8 path: sums of this thread's gathered (code - 128) */
#pragma unroll
	for (int q = 0; q < NPOS; q++)
		colsum[q] = 0;

	/* Tap-major K order (TAP, plane-major input): K-tile t covers one filter tap
	 * (kh, kw) and KCH*CHUNK consecutive input planes, tiles ordered plane
	 * block outer, tap inner.  Bounds test and in-plane offset are then one
	 * computation per thread per K-tile and every element differs only by a
	 * wave-uniform plane offset, which rides in the load's scalar offset.
	 *
	 * Channels-last input (CLI): k = tap * Ci + plane, so the VEC planes of a
	 * lane vector are 16 adjacent bytes of one pixel.  Which tap a vector
	 * belongs to is wave-uniform and decoded on the scalar unit. */
	int t_cb = 0, t_kh = 0, t_kw = 0, t_sub = 0;
	const int plane_bytes = p.HW * (int)sizeof(elem);

	auto load_tile = [&](int kt, auto set_) {
		constexpr int set = decltype(set_)::value;
#pragma unroll
		for (int i = 0; i < A_PER_WAVE; i++) {
			const int idx = wave + 4 * i;
			const int mbi = idx % MB, kci = idx / MB;
			areg[set][i] = wp[((size_t)(tile_m * MB + mbi) * p.KC + kt * KCH + kci) * 64 + lane];
		}
		unsigned tap_voff = 0;
		bool tap_ok = false;
		if constexpr (TAP) {
			const int iy = iy0 + t_kh, ix = ix0 + t_kw;
			tap_ok = n_ok && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
			tap_voff = tap_ok ? (unsigned)(xoff + t_kh * p.W + t_kw) * (unsigned)sizeof(elem) : 0xfffffff0u;
		}
		/* (CLI) decode of this thread's vector: the same for all its positions */
		int cl_kh = 0, cl_kw = 0, cl_off = 0;
		bool k_ok = true;		/* (CLI) the vector lies inside K */
		if constexpr (C4) {
			/* vector = four pixels of one kernel row: K runs (kh, kw4, pixel, plane) */
			const unsigned vi = kt * VPP + pv;
			const unsigned kh = vi * p.mhi_kw + __umulhi(vi, p.magic_kw);	/* / vectors per kernel row */
			cl_kh = (int)kh;
			cl_kw = (int)(vi - kh * p.kwv) * 4;
			cl_off = (cl_kh * p.W + cl_kw) * 4;
			k_ok = cl_kh < p.kH;
		} else if constexpr (CLU) {
			cl_kh = t_kh;
			cl_kw = t_kw;
			cl_off = ((t_kh * p.W + t_kw) * p.Ci + t_cb) * (int)sizeof(elem);	/* scalar; t_cb counts planes */
		} else if constexpr (CLI) {
			const int kv = (kt * VPP + pv) * VEC;
			unsigned tap;
			int c;
			if (p.cl_shift) {	/* K runs (block of planes, tap, plane of the block) */
				const unsigned kb = (unsigned)kv >> p.cl_shift;
				const unsigned blk = kb * p.mhi_khw + __umulhi(kb, p.magic_khw);
				tap = kb - blk * p.kHW;
				c = (int)(blk << p.cl_shift) + (kv & ((1 << p.cl_shift) - 1));
			} else {
				tap = (unsigned)kv * p.mhi_ci + __umulhi((unsigned)kv, p.magic_ci);
				c = kv - tap * p.Ci;
			}
			const unsigned kh = tap * p.mhi_kw + __umulhi(tap, p.magic_kw);
			cl_kh = (int)kh;
			cl_kw = (int)(tap - kh * p.kW);
			cl_off = (cl_kh * p.W + cl_kw) * p.Ci + c;
			k_ok = kv < p.K;
		}
#pragma unroll
		for (int j = 0; j < B_PER_THREAD; j++) {
			const int pidx = CLI ? pv : slot * B_PER_THREAD + j;
			const int q = CLI ? j : 0;	/* which of the thread's positions */
			elem v[VEC];
			bool vec_ok = tap_ok;		/* (TAP, CLI) the vector lies inside the image */
			if constexpr (C4) {
				const int iy = iy0_[q] + cl_kh, ix = ix0_[q] + cl_kw;
				const bool row_ok = n_ok_[q] && k_ok && (unsigned)iy < (unsigned)p.H;
				/* the copy has slack on both sides, so a vector that sticks
				 * out of its row still lies inside the buffer */
				const unsigned voff = row_ok ? (unsigned)(xoff_[q] + cl_off) : 0x80000000u;
				uintx4 ld = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, voff, 0, 0);
				/* per pixel: a tap past the kernel row or a column past N is
				 * code 128 (0 once re-centred, and its weight is 0 too); a
				 * pixel outside the image is the code of 0.0 in the real
				 * planes and 128 in the padding planes */
				const unsigned fillpix = p.c4_fill;
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const bool live = n_ok_[q] && k_ok && cl_kw + e < p.kW;
					const bool inside = row_ok && (unsigned)(ix + e) < (unsigned)p.W;
					ld[e] = !live ? 0x80808080u : inside ? ld[e] : fillpix;
				}
				__builtin_memcpy(v, &ld, 16);
			} else if constexpr (CLU) {
				const int iy = iy0_[q] + cl_kh, ix = ix0_[q] + cl_kw;
				vec_ok = n_ok_[q] && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
				const unsigned voff = vec_ok ? (unsigned)(xoff_[q] + cl_off) : 0x80000000u;
				const uintx4 ld = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, voff, 0, 0);
				__builtin_memcpy(v, &ld, 16);
			} else if constexpr (CLI) {
				const int iy = iy0_[q] + cl_kh, ix = ix0_[q] + cl_kw;
				vec_ok = n_ok_[q] && k_ok && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
				/* the buffer is shorter than 2^31 bytes: the second offset is
				 * out of range, reads as zero, and adding 16 cannot wrap */
				const unsigned voff = vec_ok ? (unsigned)(xoff_[q] + cl_off) * (unsigned)sizeof(elem) : 0x80000000u;
				const uintx4 ld = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, voff, 0, 0);
				__builtin_memcpy(v, &ld, 16);
			} else if constexpr (TAP) {
				const int cbase = (t_cb * SUB + t_sub) * (KCH * CHUNK) + (pidx >> 1) * CHUNK + (pidx & 1) * VEC;
#pragma unroll
				for (int e = 0; e < VEC; e++) {
					/* the scalar offset is not range checked: planes exist
					 * because Ci is a multiple of the block */
					const int soff = (cbase + e) * plane_bytes;
					if constexpr (DT == THHIP_U8)
						v[e] = __builtin_amdgcn_raw_buffer_load_b8(xrsrc, tap_voff, soff, 0);
					else if constexpr (sizeof(elem) == 4)
						v[e] = __builtin_bit_cast(elem, __builtin_amdgcn_raw_buffer_load_b32(xrsrc, tap_voff, soff, 0));
					else
						v[e] = __builtin_bit_cast(elem, __builtin_amdgcn_raw_buffer_load_b16(xrsrc, tap_voff, soff, 0));
				}
			} else {
				const int kbase = (kt * KCH + (pidx >> 1)) * CHUNK + (pidx & 1) * VEC;
#pragma unroll
				for (int e = 0; e < VEC; e++) {
					const KTap t = conv_ktap(p, kbase + e);
					const int iy = iy0 + t.kh, ix = ix0 + t.kw;
					const bool ok = n_ok && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
					/* an offset past the buffer's extent reads as zero */
					const unsigned voff = ok ? (unsigned)(xoff + t.koff) * (unsigned)sizeof(elem) : 0xfffffff0u;
					if constexpr (DT == THHIP_U8) {
						/* padding is the code of 0.0 (lowp_SpatialConvolution.c:101);
						 * columns past N and the K padding hold 128, which the
						 * re-centring below turns into 0 */
						const unsigned char ld = __builtin_amdgcn_raw_buffer_load_b8(xrsrc, voff, 0, 0);
						v[e] = ok ? ld : (unsigned char)((n_ok && kbase + e < p.K) ? p.zero : 128);
					} else if constexpr (sizeof(elem) == 4) {
						v[e] = __builtin_bit_cast(elem, __builtin_amdgcn_raw_buffer_load_b32(xrsrc, voff, 0, 0));
					} else {
						v[e] = __builtin_bit_cast(elem, __builtin_amdgcn_raw_buffer_load_b16(xrsrc, voff, 0, 0));
					}
				}
			}
			floatx4 packed;
			__builtin_memcpy(&packed, v, 16);
			if constexpr (DT == THHIP_U8 && CLU) {
				/* the loaded codes are touched when they move on to LDS */
				bmask[set][j] = vec_ok ? (int)0x80808080 : xmask_[q];
			} else if constexpr (DT == THHIP_U8) {
				/* code - 128 as a signed byte, and this thread's share of the
				 * column sum of the re-centred codes */
				intx4 cw = __builtin_bit_cast(intx4, packed);
				if constexpr (TAP || (CLI && !C4)) {
					/* the whole vector shares one tap: fill it at once */
					const int fill = ((n_ok_[q] && k_ok) ? p.zero : 128) * 0x01010101;
#pragma unroll
					for (int d = 0; d < 4; d++)
						cw[d] = vec_ok ? cw[d] : fill;
				}
#pragma unroll
				for (int d = 0; d < 4; d++) {
					cw[d] ^= (int)0x80808080;
					colsum[q] = __builtin_amdgcn_sdot4(cw[d], 0x01010101, colsum[q], false);
				}
				packed = __builtin_bit_cast(floatx4, cw);
			}
			breg[set][j] = packed;
		}
		if constexpr (CLU) {
			/* next tap of the block of planes, then the next block */
			if (++t_kw == p.kW) {
				t_kw = 0;
				if (++t_kh == p.kH) {
					t_kh = 0;
					t_cb += KCH * CHUNK;
				}
			}
		}
		if constexpr (TAP) {
			if (++t_sub < SUB) {
				/* same tap, next planes of the block */
			} else if (t_sub = 0, ++t_kw == p.kW) {
				t_kw = 0;
				if (++t_kh == p.kH) {
					t_kh = 0;
					++t_cb;
				}
			}
		}
	};

	auto store_tile = [&](int stage) {
		floatx4 *la = lds + stage * STAGE_VECS;
		floatx4 *lb = la + A_VECS;
#pragma unroll
		for (int i = 0; i < A_PER_WAVE; i++) {
			const int idx = wave + 4 * i;
			const int mbi = idx % MB, kci = idx / MB;
			la[(kci * MB + mbi) * 64 + lane] = areg[0][i];
		}
#pragma unroll
		for (int j = 0; j < B_PER_THREAD; j++) {
			if constexpr (DT == THHIP_U8 && CLU) {
				/* code - 128 as a signed byte (padding: its own code), and this
				 * thread's share of the column sum of the re-centred codes */
				intx4 cw = __builtin_bit_cast(intx4, breg[0][j]);
#pragma unroll
				for (int d = 0; d < 4; d++) {
					cw[d] ^= bmask[0][j];
					colsum[j] = __builtin_amdgcn_sdot4(cw[d], 0x01010101, colsum[j], false);
				}
				breg[0][j] = __builtin_bit_cast(floatx4, cw);
			}
			if constexpr (CLI) {
				/* neighbouring lanes write the VPP vectors of one position,
				 * 512 bytes apart: move the position inside its group of
				 * eight by the vector index to spread them over the banks
				 * (the fragment reads undo it) */
				const int nl = n_local + j * PPI;
				const int kci = pv >> 1, h = pv & 1;
				lb[((kci * NB + (nl >> 5)) * 2 + h) * 32 + ((nl & 31) ^ ((pv * (8 / VPP)) & 7))] = breg[0][j];
			} else {
				const int pidx = slot * B_PER_THREAD + j;
				const int kci = pidx >> 1, h = pidx & 1;
				lb[((kci * NB + (n_local >> 5)) * 2 + h) * 32 + (n_local & 31)] = breg[0][j];
			}
		}
	};

	typename ConvAcc<DT>::T acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; i++)
#pragma unroll
		for (int j = 0; j < TN; j++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[i][j][r] = 0;

	const int nkt_all = p.KC / KCH;
	const int kt0 = p.splitk > 1 ? (int)((long)nkt_all * split / p.splitk) : 0;
	const int nkt = p.splitk > 1 ? (int)((long)nkt_all * (split + 1) / p.splitk) : nkt_all;
	if constexpr (CLU) {
		const int blk = kt0 / p.kHW, tap = kt0 - blk * p.kHW;
		t_cb = blk * (KCH * CHUNK);
		t_kh = tap / p.kW;
		t_kw = tap - t_kh * p.kW;
	}
	if constexpr (TAP) {
		const int blk = kt0 / SUB;
		t_sub = kt0 - blk * SUB;
		t_cb = blk / p.kHW;
		const int tap = blk - t_cb * p.kHW;
		t_kh = tap / p.kW;
		t_kw = tap - t_kh * p.kW;
	}
	/* Software pipeline over three LDS stages.  While tile kt is multiplied,
	 * tile kt+1 is already complete in LDS, tile kt+2 moves from registers to
	 * LDS and tile kt+3 is on its way from global memory to registers, so a
	 * load has a whole K-tile of MFMAs to arrive and fragments are read one
	 * chunk ahead of their
	 * MFMAs, across the tile boundary too, and a wave's matrix core never
	 * waits on LDS latency; one barrier per K-tile. */
	floatx4 af[2][TM], bf[2][TN];
	auto read_frags = [&](int stage, int kci, floatx4 (&a)[TM], floatx4 (&b)[TN]) {
		const floatx4 *la = lds + stage * STAGE_VECS;
		const floatx4 *lb = la + A_VECS;
		const int bl = CLI ? lane ^ ((((kci << 1) | (lane >> 5)) * (8 / VPP)) & 7) : lane;
#pragma unroll
		for (int i = 0; i < TM; i++)
			a[i] = la[(kci * MB + wm * TM + i) * 64 + lane];
#pragma unroll
		for (int j = 0; j < TN; j++)
			b[j] = lb[(kci * NB + wn * TN + j) * 64 + bl];
	};
	typedef std::integral_constant<int, 0> R0;
	typedef std::integral_constant<int, PFD - 1> RL;
	load_tile(kt0, R0{});
	store_tile(0);
	if (kt0 + 1 < nkt) {
		load_tile(kt0 + 1, R0{});
		store_tile(1);
	}
	if (kt0 + 2 < nkt)
		load_tile(kt0 + 2, R0{});
	if constexpr (PFD > 1) {
		if (kt0 + 3 < nkt)
			load_tile(kt0 + 3, RL{});
	}
	__syncthreads();
	read_frags(0, 0, af[0], bf[0]);
	static_assert(KCH % 2 == 0, "fragment sets alternate by chunk parity");
	/* tile kt is in stage st, tile kt+1 in st1, and tile kt+2 goes to st2 */
	auto step = [&](int kt, auto st, auto st1, auto st2, auto steady_) {
		/* steady: tiles kt+2 and kt+2+PFD exist, no tests (and no branches for
		 * the instruction scheduler to stop at) */
		constexpr bool steady = decltype(steady_)::value;
		/* tile kt+2 was requested a whole step ago: it has had the time to
		 * arrive, so parking it in LDS does not stall the MFMAs */
		if (steady || kt + 2 < nkt)
			store_tile(st2);
#pragma unroll
		for (int r = 0; r + 1 < PFD; r++) {	/* the tiles in flight move up */
#pragma unroll
			for (int i = 0; i < A_PER_WAVE; i++)
				areg[r][i] = areg[r + 1][i];
#pragma unroll
			for (int j = 0; j < B_PER_THREAD; j++) {
				breg[r][j] = breg[r + 1][j];
				bmask[r][j] = bmask[r + 1][j];
			}
		}
		if (steady || kt + 2 + PFD < nkt)
			load_tile(kt + 2 + PFD, RL{});
#pragma unroll
		for (int c = 0; c < KCH; c++) {
			if (c + 1 < KCH)
				read_frags(st, c + 1, af[(c + 1) & 1], bf[(c + 1) & 1]);
			else if (steady || kt + 1 < nkt)
				read_frags(st1, 0, af[0], bf[0]);
#pragma unroll
			for (int i = 0; i < TM; i++)
#pragma unroll
				for (int j = 0; j < TN; j++)
					conv_mma<DT>(acc[i][j], af[c & 1][i], bf[c & 1][j]);
		}
		if constexpr (DT == THHIP_F32 && GM != GM_PLANE_TAP) {
			/* Ask the scheduler to spread the K-tile's loads, LDS traffic and
			 * address arithmetic between the MFMAs instead of bunching them
			 * before and after: the matrix core then works while they issue
			 * (measured: +2.5 % on fp32, nothing on the shorter half and
			 * int8 MFMAs). */
			constexpr int NM = KCH * TM * TN * 4;
#pragma unroll
			for (int m = 0; m < NM; m++) {
				__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
				__builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
				__builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
				__builtin_amdgcn_sched_group_barrier(0x006, 6, 0);
				__builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
			}
		}
		__syncthreads();
	};
	if constexpr (TAP || CLI) {
		/* small gather code: unroll three times so every stage is a constant */
		typedef std::integral_constant<int, 0> S0;
		typedef std::integral_constant<int, 1> S1;
		typedef std::integral_constant<int, 2> S2;
		int kt = kt0;
		for (; kt + 4 + PFD < nkt; kt += 3) {	/* steady state */
			step(kt, S0{}, S1{}, S2{}, std::true_type{});
			step(kt + 1, S1{}, S2{}, S0{}, std::true_type{});
			step(kt + 2, S2{}, S0{}, S1{}, std::true_type{});
		}
		for (; kt + 2 < nkt; kt += 3) {		/* the last tiles drain */
			step(kt, S0{}, S1{}, S2{}, std::false_type{});
			step(kt + 1, S1{}, S2{}, S0{}, std::false_type{});
			step(kt + 2, S2{}, S0{}, S1{}, std::false_type{});
		}
		if (kt < nkt) {
			step(kt, S0{}, S1{}, S2{}, std::false_type{});
			if (kt + 1 < nkt)
				step(kt + 1, S1{}, S2{}, S0{}, std::false_type{});
		}
	} else {
		/* the element-wise gather is long: one copy, stages rotate at run time */
		int st = 0;
		for (int kt = kt0; kt < nkt; kt++) {
			const int st1 = st == 2 ? 0 : st + 1, st2 = st1 == 2 ? 0 : st1 + 1;
			step(kt, st, st1, st2, std::false_type{});
			st = st1;
		}
	}

	/* ---- epilogue ---- */
	elem *y = (elem *)p.y;
	__shared__ int cs[DT == THHIP_U8 ? BN : 1];
	/* Per-row constants go through LDS (the tiles are done with it): loads from
	 * global memory inside the store loops would each wait out a round trip,
	 * and registers are what limits how many workgroups share a CU. */
	int *lrow = (int *)lds;		/* [BM] bias bits, or uint8 row term; [BM..2BM) uint8 addend */
	if (tid < BM) {
		const int mc = min(tile_m * BM + tid, p.Co - 1);
		if constexpr (DT == THHIP_U8) {
			/* (128+b_off) rowsum + K (128+a_off)(128+b_off) */
			lrow[tid] = p.offB * p.rowsum[mc] + p.K * p.offA * p.offB;
			lrow[BM + tid] = p.addend ? p.addend[mc] : 0;
		} else {
			lrow[tid] = __float_as_int(p.bias ? p.bias[mc] : 0.0f);
			if (p.scale)
				lrow[BM + tid] = __float_as_int(p.scale[mc]);
		}
	}
	if constexpr (DT != THHIP_U8)
		__syncthreads();
	if constexpr (DT == THHIP_U8) {
		/* Every (chunk, half) share of a column was gathered by one of the
		 * 256/BN threads that own it: add the shares up in LDS. */
		if (tid < BN)
			cs[tid] = 0;
		__syncthreads();
#pragma unroll
		for (int q = 0; q < NPOS; q++)
			atomicAdd(&cs[n_local + q * PPI], colsum[q]);
		__syncthreads();
	}
	if (p.splitk > 1) {
		/* Each part stores its accumulators (for uint8 with its share of the
		 * column-sum term folded in) in its own slice; the part that arrives
		 * last adds the slices in a fixed order and finishes the tile, so the
		 * result does not depend on timing. */
		constexpr int TILE_WORDS = BM * BN;
		int *mine = p.ws + ((size_t)tile * p.splitk + split) * TILE_WORDS;
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++) {
				int colterm = 0;
				if constexpr (DT == THHIP_U8)
					colterm = p.offA * cs[(wn * TN + j) * 32 + (lane & 31)];
#pragma unroll
				for (int r = 0; r < 16; r++) {
					int word;
					if constexpr (DT == THHIP_U8)
						word = acc[i][j][r] + colterm;
					else
						word = __float_as_int(acc[i][j][r]);
					mine[((i * TN + j) * 16 + r) * CONV_THREADS + tid] = word;
				}
			}
		__threadfence();
		__shared__ unsigned ticket;
		__syncthreads();
		if (tid == 0)
			ticket = atomicAdd(&p.cnt[tile], 1u);
		__syncthreads();
		if (ticket != (unsigned)p.splitk - 1)
			return;
		__threadfence();
		if (tid == 0)
			p.cnt[tile] = 0;	/* ready for the next launch */
		const int *all = p.ws + (size_t)tile * p.splitk * TILE_WORDS + tid;
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] = 0;
		/* one slice at a time, sixteen of its words in flight together */
		for (int q = 0; q < p.splitk; q++) {
			const int *src = all + (size_t)q * TILE_WORDS;
#pragma unroll
			for (int i = 0; i < TM; i++)
#pragma unroll
				for (int j = 0; j < TN; j++) {
					int part[16];
#pragma unroll
					for (int r = 0; r < 16; r++)
						part[r] = __hip_atomic_load(src + ((i * TN + j) * 16 + r) * CONV_THREADS,
							__ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
					for (int r = 0; r < 16; r++) {
						if constexpr (DT == THHIP_U8)
							acc[i][j][r] += part[r];
						else
							acc[i][j][r] += __int_as_float(part[r]);
					}
				}
		}
	}
	if constexpr (DT == THHIP_U8) {
		/* sum (w+a_off)(x+b_off) with w = w'+128, x = x'+128:
		 *   sum w'x' + (128+b_off) rowsum + (128+a_off) colsum + K (128+a_off)(128+b_off) */
		const int tail0 = (p.oHW / 8) * 8;	/* lowpadd's unclamped tail starts here */
		const bool has_add = p.addend != 0;
		const bool cl16 = CLO && p.Co % 16 == 0 && ((size_t)p.y & 15) == 0;	/* whole 16-byte stores (conv_store_cl_u8) */
#pragma unroll
		for (int j = 0; j < TN; j++) {
			const int nl = (wn * TN + j) * 32 + (lane & 31);
			const int n = tile_n * BN + nl;
			const bool valid = n < p.N;
			if (!cl16 && !valid)
				continue;
			const int b = n / p.oHW, rem = n - b * p.oHW;
			const size_t ybase = (size_t)b * p.Co * p.oHW + rem;
			const int colterm = p.splitk > 1 ? 0 : p.offA * cs[nl];
			const bool tail = rem >= tail0;
#pragma unroll
			for (int i = 0; i < TM; i++) {
				const int m0 = tile_m * BM + (wm * TM + i) * 32 + 4 * (lane >> 5);
				unsigned word[4];
#pragma unroll
				for (int g = 0; g < 4; g++) {
					unsigned packed = 0;
					const int ml = (wm * TM + i) * 32 + 4 * (lane >> 5) + 8 * g;
					const intx4 rowterm = *(const intx4 *)(lrow + ml);
					const intx4 rowadd = *(const intx4 *)(lrow + BM + ml);
#pragma unroll
					for (int e = 0; e < 4; e++) {
						const int r = 4 * g + e, m = m0 + 8 * g + e;
						const int a = acc[i][j][r] + rowterm[e] + colterm;
						int q = conv_requant(a, p.c_off, p.c_mult, p.c_shift);
						if (has_add) {
							/* lowpadd, lowp_SpatialConvolution.c:71-88 */
							const int sum = q + rowadd[e];
							q = sum > 255 ? 255 : (tail ? (sum & 255) : (sum < 0 ? 0 : sum));
						}
						if (p.act)
							q = q > p.ithr ? q : p.ival;
						if constexpr (CLO)
							packed |= (unsigned)q << (8 * e);
						else if (m < p.Co)
							y[ybase + (size_t)m * p.oHW] = (unsigned char)q;
					}
					if constexpr (CLO) {
						word[g] = packed;
						/* Co % 4 == 0: the four planes are one aligned word */
						if (!cl16 && m0 + 8 * g < p.Co)
							*(unsigned *)(y + (size_t)n * p.Co + m0 + 8 * g) = packed;
					}
				}
				if constexpr (CLO) {
					if (cl16) {
						const int mt = tile_m * BM + (wm * TM + i) * 32;
						conv_store_cl_u8(y + (size_t)n * p.Co + mt, p.Co - mt, valid, word, lane);
					}
				}
			}
		}
	} else {
		/* (folded batch norm factor,) bias, optional threshold, store */
		const bool has_scale = p.scale != 0;
		/* half types, channels-last: whole 16-byte stores (conv_store_cl_half) */
		const bool cl16 = CLO && sizeof(elem) == 2 && p.Co % 8 == 0 && ((size_t)p.y & 15) == 0;
#pragma unroll
		for (int j = 0; j < TN; j++) {
			const int n = tile_n * BN + (wn * TN + j) * 32 + (lane & 31);
			const bool valid = n < p.N;
			if (!cl16 && !valid)
				continue;
			const int b = n / p.oHW, rem = n - b * p.oHW;
			const size_t ybase = (size_t)b * p.Co * p.oHW + rem;
#pragma unroll
			for (int i = 0; i < TM; i++) {
				const int m0 = tile_m * BM + (wm * TM + i) * 32 + 4 * (lane >> 5);
				unsigned lo[4], hi[4];
#pragma unroll
				for (int g = 0; g < 4; g++) {
					struct alignas(4 * sizeof(elem)) Quad { elem v[4]; } quad;
					const int ml = (wm * TM + i) * 32 + 4 * (lane >> 5) + 8 * g;
					const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
					floatx4 rowscale = { 1, 1, 1, 1 };
					if (has_scale)
						rowscale = *(const floatx4 *)(lrow + BM + ml);
#pragma unroll
					for (int e = 0; e < 4; e++) {
						const int r = 4 * g + e, m = m0 + 8 * g + e;
						float v = has_scale ? acc[i][j][r] * rowscale[e] + rowbias[e] : acc[i][j][r] + rowbias[e];
						if (p.act)
							v = v > p.thr ? v : p.val;
						if constexpr (!CLO) {
							if (m < p.Co)
								y[ybase + (size_t)m * p.oHW] = (elem)v;
						}
						quad.v[e] = (elem)v;
					}
					if constexpr (CLO) {
						if constexpr (sizeof(elem) == 2) {
							unsigned pair[2];
							__builtin_memcpy(pair, &quad, 8);
							lo[g] = pair[0];
							hi[g] = pair[1];
						}
						if (!cl16 && m0 + 8 * g < p.Co)
							*(Quad *)(y + (size_t)n * p.Co + m0 + 8 * g) = quad;
					}
				}
				if constexpr (CLO && sizeof(elem) == 2) {
					if (cl16) {
						const int mt = tile_m * BM + (wm * TM + i) * 32;
						conv_store_cl_half((unsigned short *)y + (size_t)n * p.Co + mt, p.Co - mt, valid, lo, hi, lane);
					}
				}
			}
		}
	}
}

/* ------------------------------------------------------------------ */
/* wide tile for the half types                                        */
/* ------------------------------------------------------------------ */

/* A 32x32x16 half MFMA retires in 32 cycles what the fp32 one needs 512 for,
 * so a 128x128 tile asks the LDS and the path from L2 for about as many bytes
 * per cycle as they can deliver.  This kernel halves both appetites: a 256x256
 * tile, eight waves of 128x64 each, K-tiles of 32 values, and the operands go
 * from global memory straight into LDS (buffer loads with the LDS bit: no
 * staging registers, no ds_write), four stages deep.
 *
 * For channels-last input whose plane count is a multiple of the K-tile (the
 * GM_CL_UNIFORM case).  A wave-wide 16-byte load puts lane l's data at
 * base + 16 l, so what a lane fetches decides the LDS layout:
 *   A: the packed weights already are [32-row block][chunk][h][32][16 B]; a
 *      wave copies 1 KiB blocks unchanged.
 *   B: a position's K-tile slice is 64 contiguous bytes (four vectors), so four
 *      neighbouring lanes fetch one position and a wave sixteen positions.  Slot
 *      4 pl + s of a sixteen-position group holds vector s ^ (pl / 4) of
 *      position pl: the fragment reads (32 positions x 2 vectors) then hit every
 *      bank equally (measured at the full ds_read_b128 rate; 4x slower unswizzled).
 * Loads outside the image are sent out of the buffer's range and write zeros.
 *
 * The compiler does not track these LDS writes: the waits are explicit
 * (s_waitcnt vmcnt counts whole tiles, four loads per wave each), and the
 * barrier sits in the middle of a step, between the two chunks of a K-tile:
 * before it a wave has seen its share of tile kt+1 land and has read the last
 * fragments of tile kt, after it that stage is free for tile kt+4 and tile
 * kt+1 is complete, so its first fragments are fetched under the second
 * chunk's MFMAs. */

/* XCD x's rectangle of the tile grid (mparts x 8/mparts rectangles): first tile
 * row, rows, first tile column, and the number of tiles. */
__device__ inline void conv_xcd_rect(const ConvParams &p, int xcd, int &m0, int &mw, int &n0, int &cnt)
{
	const int mp = xcd % p.mparts, np = xcd / p.mparts, nparts = 8 / p.mparts;
	m0 = p.tiles_m * mp / p.mparts;
	const int m1 = p.tiles_m * (mp + 1) / p.mparts;
	n0 = p.tiles_n * np / nparts;
	const int n1 = p.tiles_n * (np + 1) / nparts;
	mw = m1 - m0;
	cnt = mw * (n1 - n0);
}

/* The parts of a cut tile are computed by workgroups whose blockIdx.x agree modulo 8, and the hardware
 * hands workgroup b of a launch to XCD (b + r) % 8 -- r is the same for every workgroup of a launch, but
 * changes from launch to launch when queues are created or mapped anew (another stream, another process)
 * -- so they run on one XCD and share its L2: a part's sums need only reach L2 (the vector caches write
 * through; the wait for the stores' acknowledgement is the release) before the ticket is drawn there (an
 * atomic without the device-scope bit executes in the XCD's L2), and the workgroup that draws the last
 * ticket reads them from L2.  No L2 write-back or invalidate as a device-scope fence would do (measured with
 * those, and with device-scope loads and stores of the parts: slower than a second launch; this way
 * ResNet-18 batch 32 1.269 -> 1.239 ms and VGG-16 batch 16 3.825 -> 3.803 ms against the second launch.
 * The parts of a layer whose whole K is split stay with their second launch: every tile's last workgroup
 * adding parts cost 8 us a layer more than it).
 *
 * That every part workgroup of the launch saw the same r is checked, not assumed: each of them ORs
 * 1 << r into the launch's word of p.rot when it starts (conv_xcd_report: a device-scope atomic nobody waits
 * for; it is complete before the workgroup draws its ticket, whose release waits for everything the
 * wavefront has outstanding), and the workgroup that draws a tile's last ticket reads the word: more than
 * one bit, and the host hears of it (p.fault; hip_rt.hip turns that into a repeat or an error). */
__device__ __forceinline__ void conv_xcd_report(const ConvParams &p, bool part)
{
	if (threadIdx.x != 0)
		return;
	if (part) {
		const unsigned r = ((unsigned)__builtin_amdgcn_s_getreg(THHIP_GETREG_XCC_ID) - blockIdx.x) & 7u;
		__hip_atomic_fetch_or(p.rot + p.rot_slot, 1u << r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
	if (blockIdx.x == 0)	/* the word of a launch to come (this launch's was cleared as long ago) */
		__hip_atomic_store(p.rot + p.rot_clear, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* Returns whether this workgroup drew the last of `parts` tickets (and has reset the counter for the next
 * launch); `slot` is one int of LDS nobody else uses until the next barrier after the call. */
__device__ __forceinline__ bool conv_xcd_last_arriver(const ConvParams &p, unsigned *counter, int parts, int *slot)
{
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
	__syncthreads();
	if (threadIdx.x == 0)
		*slot = (int)__hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
	__syncthreads();
	const bool last = *slot == parts - 1;
	if (last && threadIdx.x == 0) {
		*counter = 0;
		const unsigned seen = __hip_atomic_load(p.rot + p.rot_slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		if (seen & (seen - 1))
			__hip_atomic_store(p.fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
	}
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
	return last;
}

/* One fp32 sum of another workgroup's part, from L2 (sc0: not from this CU's vector cache). */
__device__ __forceinline__ float conv_load_part(const float *p)
{
	return __builtin_bit_cast(float, __hip_atomic_load((const int *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
}

/* The tiles an XCD cannot spread evenly: of its cnt tiles the last cnt % slots
 * would run a few to a CU (or alone) while the other CUs idle.  Those are cut
 * along K into as many parts as fill the slots once, at most smax; *full is
 * the number of tiles that stay whole.  need_round: cut only where at least
 * one whole round precedes.  Returns the parts (1: no cut). */
__host__ __device__ inline int conv_tail_parts(int cnt, int slots, int smax, int need_round, int *full)
{
	*full = cnt;
	if (slots <= 0)
		return 1;
	const int f = cnt / slots * slots, rem = cnt - f;
	/* after more than four rounds the workgroups of an XCD have drifted apart
	 * and its CUs run dry at different times anyway (64->64 @224^2 batch 16,
	 * eight rounds: 473 us uncut, 479 + 6 us cut) */
	if (!rem || f > 4 * slots || (need_round && !f))
		return 1;
	int s = slots / rem;
	if (s > smax)
		s = smax;
	if (s < 2)
		return 1;
	*full = f;
	return s;
}

/* conv_f32_direct_kernel and conv_wide_kernel with the 2x2 / stride 2 pooling in their epilogue: member t of a
 * block of 64 positions.  The block is sixteen neighbouring pooling windows; t = 32 half + 16 dy + 2 w + dx
 * is column dx of row dy of window 8 half + w.  Sixteen neighbouring lanes thus gather sixteen
 * neighbouring pixels of a row (whole 64-byte runs, as without the pooling), a 32-position MFMA
 * tile holds eight whole windows, the other column of a window is the next lane and the other
 * row is lane ^ 16. */
__device__ __forceinline__ void conv_pool_member(int n, int &pp, int &dy, int &dx)
{
	pp = (n >> 6) * 16 + ((n >> 5) & 1) * 8 + ((n >> 1) & 7);
	dy = (n >> 4) & 1;
	dx = n & 1;
}

/* v of lane + 1 (for even lanes), v of lane ^ 16 */
__device__ __forceinline__ float conv_lane_next(float v)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xF5, 0xf, 0xf, true));
}

__device__ __forceinline__ float conv_lane_xor16(float v)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}

/* Epilogue of the half-type tiles of conv_wide_kernel (WGM x WGN waves, each
 * TMF x TNF accumulators of 32x32, of which acc holds the TM x TN from
 * (i0, j0) on): (folded batch norm factor,) bias, optional threshold, store in
 * either memory order.  lrow: 2 * BM ints of LDS no wave still reads. */
template <int DT, bool CLO, int BM, int BN, int WGM, int WGN, int TMF, int TNF, int TM, int TN>
__device__ __forceinline__ void conv_wide_store_half(const ConvParams &p, floatx16 (&acc)[TM][TN], int tile_m, int tile_n, int *lrow,
	int i0 = 0, int j0 = 0)
{
	typedef typename ConvTraits<DT>::elem elem;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave % WGM, wn = wave / WGM;
	elem *y = (elem *)p.y;
	if (tid < BM) {
		const int mc = min(tile_m * BM + tid, p.Co - 1);
		lrow[tid] = __float_as_int(p.bias ? p.bias[mc] : 0.0f);
		if (p.scale)
			lrow[BM + tid] = __float_as_int(p.scale[mc]);
	}
	__syncthreads();
	const bool has_scale = p.scale != 0;
	/* channels-last: whole 16-byte stores (conv_store_cl_half) */
	const bool cl16 = CLO && p.Co % 8 == 0 && ((size_t)p.y & 15) == 0;
	/* With the pooling (p.pool: positions counted in blocks of sixteen windows, conv_pool_member) the first
	 * lane of a window takes the maximum of the four stored (rounded) values, with SpatialMaxPooling.c:51-66's
	 * comparisons in their order, and stores it; every lane runs the loop (the lanes of a window exchange). */
	const int oHW = p.pool ? p.pHW : p.oHW;
#pragma unroll
	for (int j = 0; j < TN; j++) {
		int n = tile_n * BN + (wn * TNF + j0 + j) * 32 + (lane & 31);
		bool valid = n < p.N;
		if (p.pool) {
			int pp, dy, dx;
			conv_pool_member(n, pp, dy, dx);
			valid = pp < p.npool && !dy && !dx;
			n = pp;
		} else if (!cl16 && !valid)
			continue;
		const int b = n / oHW, rem = n - b * oHW;
		const size_t ybase = (size_t)b * p.Co * oHW + rem;
#pragma unroll
		for (int i = 0; i < TM; i++) {
			const int m0 = tile_m * BM + (wm * TMF + i0 + i) * 32 + 4 * (lane >> 5);
			unsigned lo[4], hi[4];
#pragma unroll
			for (int g = 0; g < 4; g++) {
				struct alignas(4 * sizeof(elem)) Quad { elem v[4]; } quad;
				const int ml = (wm * TMF + i0 + i) * 32 + 4 * (lane >> 5) + 8 * g;
				const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
				floatx4 rowscale = { 1, 1, 1, 1 };
				if (has_scale)
					rowscale = *(const floatx4 *)(lrow + BM + ml);
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const int r = 4 * g + e, m = m0 + 8 * g + e;
					float v = has_scale ? acc[i][j][r] * rowscale[e] + rowbias[e] : acc[i][j][r] + rowbias[e];
					if (p.act)
						v = v > p.thr ? v : p.val;
					if (p.pool) {
						const float v00 = (float)(elem)v, v01 = conv_lane_next(v00);
						const float v10 = conv_lane_xor16(v00), v11 = conv_lane_xor16(v01);
						float mx = -FLT_MAX;
						mx = v00 > mx ? v00 : mx;
						mx = v01 > mx ? v01 : mx;
						mx = v10 > mx ? v10 : mx;
						mx = v11 > mx ? v11 : mx;
						v = mx;
					}
					if constexpr (!CLO) {
						if (valid && m < p.Co)
							y[ybase + (size_t)m * oHW] = (elem)v;
					}
					quad.v[e] = (elem)v;
				}
				if constexpr (CLO) {
					unsigned pair[2];
					__builtin_memcpy(pair, &quad, 8);
					lo[g] = pair[0];
					hi[g] = pair[1];
					if (!cl16 && valid && m0 + 8 * g < p.Co)
						*(Quad *)(y + (size_t)n * p.Co + m0 + 8 * g) = quad;
				}
			}
			if constexpr (CLO) {
				if (cl16) {
					const int mt = tile_m * BM + (wm * TMF + i0 + i) * 32;
					conv_store_cl_half((unsigned short *)y + (size_t)n * p.Co + mt, p.Co - mt, valid, lo, hi, lane);
				}
			}
		}
	}
}

template <int DT, bool CLO, int BM, int BN, int WGM, int WGN, int KCH, int NST, int KG = 1>
__global__ __launch_bounds__(64 * WGM * WGN * KG) void conv_wide_kernel(ConvParams p)
{
	/* The host pass only needs the launch stub; it gets no body, because it
	 * silently drops the whole kernel when it meets the LDS-load builtin in a
	 * generic lambda of this template (the launch then fails to link). */
#if defined(__HIP_DEVICE_COMPILE__)
	typedef ConvTraits<DT> TR;
	typedef typename TR::elem elem;
	constexpr int CHUNK = TR::CHUNK, VEC = TR::VEC;
	static_assert(CHUNK * sizeof(elem) == 32 && DT != THHIP_F32, "a half type or uint8 codes");
	constexpr int WAVES = WGM * WGN;
	constexpr int MB = BM / 32, TM = BM / WGM / 32, TN = BN / WGN / 32;
	constexpr int VPP = 2 * KCH;			/* 16-byte vectors of a position's K-tile slice */
	constexpr int PPG = 64 / VPP;			/* positions one wave-wide load covers (a group) */
	constexpr int FSH = KCH == 2 ? 2 : 1;		/* swizzle: vector index ^ (position >> FSH) */
	constexpr int A_VECS = MB * KCH * 64, B_VECS = BN * VPP, STAGE_VECS = A_VECS + B_VECS;
	constexpr int A_PW = MB * KCH / WAVES;		/* 1 KiB weight blocks per wave and K-tile */
	constexpr int NPOS = BN / PPG / WAVES;		/* position groups per wave */
	constexpr int LOADS = A_PW + NPOS;		/* per wave and K-tile */
	static_assert(KCH == 2 || KCH == 4, "K-tiles of 32 or 64 values");
	static_assert(MB * KCH % WAVES == 0 && BN / PPG % WAVES == 0 && NST >= 2 && NST <= 4, "tile shape");
	static_assert((2 * BM + BN) * sizeof(int) <= NST * STAGE_VECS * sizeof(floatx4), "the epilogue's row and column constants fit");
	/* KG = 2: two groups of WGM x WGN waves share the tile, each with its own LDS stages and its own half of
	 * the K-tiles; their sums are added through LDS at the end (a K split inside the workgroup: no partial
	 * sums in global memory, no second launch, the same order of additions every time).  For layers of few
	 * tiles and a long K, where a CU holds one or two workgroups and little overlaps a K step's latency. */
	static_assert(KG == 1 || KG == 2, "one or two K groups");
	static_assert(KG == 1 || TM * TN * 16 * 64 * WAVES * sizeof(int) + TN * 64 * WAVES * sizeof(int) <= NST * STAGE_VECS * sizeof(floatx4),
		"the exchange of the groups' sums fits one group's stages");
	__shared__ floatx4 lds_all[KG * NST * STAGE_VECS];

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int kg = KG > 1 ? wave_all / WAVES : 0;
	const int wave = KG > 1 ? wave_all - kg * WAVES : wave_all;	/* within the group */
	const int wm = wave % WGM, wn = wave / WGM;
	floatx4 *const lds = lds_all + kg * (NST * STAGE_VECS);

	int tile_m, tile_n, split = 0, nsplit = 1;
	long tail_blk = -1;
	{	/* every XCD gets a rectangle of the tile grid, as in conv_mfma_kernel */
		const int bid = blockIdx.x;
		const int xcd = bid & 7;
		int local = bid >> 3;
		int m0, mw, n0, cnt;
		conv_xcd_rect(p, xcd, m0, mw, n0, cnt);
		if (DT != THHIP_U8 && p.tail_slots) {	/* the XCD's last tiles, dispatched last, in parts along K */
			int full;
			const int s = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
			if (s > 1 && local >= full) {
				const int t = (local - full) / s;
				split = (local - full) - t * s;
				nsplit = s;
				local = full + t;
				tail_blk = (long)xcd * p.tail_cap + t * s + split;
			}
		}
		if (local >= cnt)
			return;
		tile_m = m0 + local % mw;
		tile_n = n0 + local / mw;
	}

	/* ---- what this lane fetches: slot lane % VPP of position lane / VPP of a group ---- */
	bool n_ok_[NPOS];
	int iy0_[NPOS], ix0_[NPOS], xoff_[NPOS];
#pragma unroll
	for (int q = 0; q < NPOS; q++) {
		const int n_tile = (wave + WAVES * q) * PPG + lane / VPP;
		const int myvec = (lane % VPP) ^ ((n_tile >> FSH) & (VPP - 1));
		const int n_glob = tile_n * BN + n_tile;
		n_ok_[q] = n_glob < p.N;
		const int nn = n_ok_[q] ? n_glob : 0;
		int b, oy, ox;
		if (p.pool) {	/* positions in blocks of sixteen pooling windows */
			int pp, dy, dx;
			conv_pool_member(n_glob, pp, dy, dx);
			n_ok_[q] = pp < p.npool;
			pp = n_ok_[q] ? pp : 0;
			b = pp / p.pHW;
			const int r = pp - b * p.pHW, py = r / p.pW;
			oy = 2 * py + dy;
			ox = 2 * (r - py * p.pW) + dx;
		} else {
			b = nn / p.oHW;
			const int r = nn - b * p.oHW;
			oy = r / p.oW;
			ox = r - oy * p.oW;
		}
		iy0_[q] = oy * p.dH - p.padH;
		ix0_[q] = ox * p.dW - p.padW;
		xoff_[q] = (((b * p.H + iy0_[q]) * p.W + ix0_[q]) * p.Ci + myvec * VEC) * (int)sizeof(elem);
	}
	/* uint8: the tensor is followed by x_tail >= 64 bytes of the padding code, and
	 * what lies outside the image is fetched from there (a load out of range would
	 * give code 0, which is not the code of 0.0) */
	const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes + p.x_tail, 0x00020000);
	const unsigned outside = DT == THHIP_U8 ? p.x_bytes + (unsigned)(lane & 3) * 16u : 0x80000000u;
	const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.wp, 0, p.w_bytes, 0x00020000);
	/* this wave's weight blocks: wave + WAVES i counts (chunk, 32-row block), 1 KiB each */
	unsigned a_off_[A_PW];
	int a_lds_[A_PW];
#pragma unroll
	for (int i = 0; i < A_PW; i++) {
		const int idx = wave + WAVES * i, mbi = idx % MB, kci = idx / MB;
		a_off_[i] = ((unsigned)(tile_m * MB + mbi) * (unsigned)p.KC + kci) * 1024u;
		a_lds_[i] = (kci * MB + mbi) * 64;
	}
	/* K-tiles: block of planes outer, tap inner; a part of a cut tile walks [kt0, kt0 + nkt) */
	const int nkt_all = p.KC / KCH;
	int kt0 = nsplit > 1 ? (int)((long)nkt_all * split / nsplit) : 0;
	int nkt = (nsplit > 1 ? (int)((long)nkt_all * (split + 1) / nsplit) : nkt_all) - kt0;
	int nkt_live = nkt;	/* K-tiles that exist; the groups walk the same number of steps (the barriers are the workgroup's) */
	if constexpr (KG > 1) {
		const int per = (nkt + KG - 1) / KG;
		nkt_live = min(per, nkt - kg * per);
		kt0 += kg * per;
		nkt = per;
	}
	int issued = 0;
	int t_cb, t_kh, t_kw, t_kc = kt0 * KCH;
	{
		const int blk = kt0 / p.kHW, tap = kt0 - blk * p.kHW;
		t_cb = blk * (KCH * CHUNK);
		t_kh = tap / p.kW;
		t_kw = tap - t_kh * p.kW;
	}

	auto issue = [&](auto st_) {
		constexpr int st = decltype(st_)::value;
		floatx4 *la = lds + st * STAGE_VECS, *lb = la + A_VECS;
		/* (KG > 1) a step past this group's last K-tile loads zeros: weights out of the buffer's range,
		 * positions as outside the image */
		const bool live = KG == 1 || issued < nkt_live;
		++issued;
#pragma unroll
		for (int i = 0; i < A_PW; i++)
			__builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, WIDE_LDS(la + a_lds_[i]), 16, live ? lane * 16 : 0x80000000u,
				a_off_[i] + (unsigned)t_kc * 1024u, 0, 0);
		const int cl_off = ((t_kh * p.W + t_kw) * p.Ci + t_cb) * (int)sizeof(elem);
#pragma unroll
		for (int q = 0; q < NPOS; q++) {
			const int iy = iy0_[q] + t_kh, ix = ix0_[q] + t_kw;
			/* (no branches in a K step: the compiler may then spread its loads between the MFMAs) */
			const bool ok = (int)live & (int)n_ok_[q] & (int)((unsigned)iy < (unsigned)p.H) & (int)((unsigned)ix < (unsigned)p.W);
			const unsigned voff = ok ? (unsigned)(xoff_[q] + cl_off) : outside;
			__builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, WIDE_LDS(lb + (wave + WAVES * q) * 64), 16, voff, 0, 0, 0);
		}
		t_kc += KCH;
		const int kw1 = t_kw + 1, wrap_w = kw1 == p.kW;
		t_kw = __builtin_amdgcn_readfirstlane(wrap_w ? 0 : kw1);
		const int kh1 = t_kh + wrap_w, wrap_h = kh1 == p.kH;
		t_kh = __builtin_amdgcn_readfirstlane(wrap_h ? 0 : kh1);
		t_cb = __builtin_amdgcn_readfirstlane(t_cb + (wrap_h ? KCH * CHUNK : 0));
	};

	/* fragment addresses: A rows lane % 32 of a block, half lane / 32; B position
	 * lane % 32 of a block, vector 2 chunk + lane / 32, through the swizzle */
	const int b_pos = ((lane & 31) / PPG) * 64 + ((lane & 31) % PPG) * VPP;
	const int b_f = ((lane & 31) >> FSH) & (VPP - 1);
	floatx4 af[2][TM], bf[2][TN];
	auto read_frags = [&](auto st_, int kci, floatx4 (&a)[TM], floatx4 (&b)[TN]) {
		constexpr int st = decltype(st_)::value;
		const floatx4 *la = lds + st * STAGE_VECS, *lb = la + A_VECS;
#pragma unroll
		for (int i = 0; i < TM; i++)
			a[i] = la[(kci * MB + wm * TM + i) * 64 + lane];
#pragma unroll
		for (int j = 0; j < TN; j++)
			b[j] = lb[(wn * TN + j) * 32 * VPP + b_pos + ((kci * 2 + (lane >> 5)) ^ b_f)];
	};

	typename ConvAcc<DT>::T acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; i++)
#pragma unroll
		for (int j = 0; j < TN; j++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[i][j][r] = 0;
	int colsum[TN];		/* uint8, waves with wm == 0: this lane's share of the column sums of the re-centred codes */
#pragma unroll
	for (int j = 0; j < TN; j++)
		colsum[j] = 0;
	auto mma = [&](int set, int kt) {
		/* (KG > 1) a step past the group's last K-tile has read padding codes, which are not zero once
		 * re-centred unless the padding code is 128: they meet zero weights, but stay out of the column sums */
		const bool sums = wm == 0 && (KG == 1 || kt < nkt_live);
		if constexpr (DT == THHIP_U8) {
			/* code - 128 as a signed byte, done on the fragments (they never
			 * pass through registers on their way to LDS) */
#pragma unroll
			for (int j = 0; j < TN; j++) {
				intx4 cw = __builtin_bit_cast(intx4, bf[set][j]);
#pragma unroll
				for (int d = 0; d < 4; d++) {
					cw[d] ^= (int)0x80808080;
					if (sums)
						colsum[j] = __builtin_amdgcn_sdot4(cw[d], 0x01010101, colsum[j], false);
				}
				bf[set][j] = __builtin_bit_cast(floatx4, cw);
			}
		}
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
				conv_mma<DT>(acc[i][j], af[set][i], bf[set][j]);
	};

	typedef std::integral_constant<int, 0> S0;
	typedef std::integral_constant<int, 1> S1;
	typedef std::integral_constant<int, NST >= 3 ? 2 : 0> S2;
	typedef std::integral_constant<int, NST >= 4 ? 3 : 0> S3;
	issue(S0{});
	if (1 < nkt)
		issue(S1{});
	if constexpr (NST >= 3) {
		if (2 < nkt)
			issue(S2{});
	}
	if constexpr (NST >= 4) {
		if (3 < nkt)
			issue(S3{});
	}
	if (NST - 1 < nkt)
		wide_wait<(NST - 1) * LOADS, false>();
	else
		wide_wait<0, false>();
	__builtin_amdgcn_s_barrier();
	read_frags(S0{}, 0, af[0], bf[0]);

	/* tile kt is in stage st (its first fragments in set 0), tile kt+1 in st1 */
	auto step = [&](int kt, auto st, auto st1, auto steady_) {
		constexpr bool steady = decltype(steady_)::value;	/* tiles up to kt+NST exist */
#pragma unroll
		for (int c = 0; c + 1 < KCH; c++) {
			read_frags(st, c + 1, af[(c + 1) & 1], bf[(c + 1) & 1]);
			/* the next chunk's fragments are asked for before this chunk's MFMAs (left alone, the
			 * compiler puts the reads right before their first use) */
			__builtin_amdgcn_sched_barrier(0);
			mma(c & 1, kt);
		}
		/* this wave's loads of tile kt+1 are in LDS (younger tiles may still be
		 * on their way) and the fragments just requested have arrived */
		if (steady)
			wide_wait<(NST - 2) * LOADS, true>();
		else
			wide_wait<0, true>();
		__builtin_amdgcn_s_barrier();
		if (steady || kt + 1 < nkt)
			read_frags(st1, 0, af[0], bf[0]);
		__builtin_amdgcn_sched_barrier(0);	/* (as above; the loads below mix with the MFMAs) */
		if (steady || kt + NST < nkt)
			issue(st);
		mma((KCH - 1) & 1, kt);
	};
	/* NST steps: every stage index a constant */
	auto round = [&](int kt, auto steady_) {
		if constexpr (NST == 2) {
			step(kt, S0{}, S1{}, steady_);
			step(kt + 1, S1{}, S0{}, steady_);
		} else if constexpr (NST == 3) {
			step(kt, S0{}, S1{}, steady_);
			step(kt + 1, S1{}, S2{}, steady_);
			step(kt + 2, S2{}, S0{}, steady_);
		} else {
			step(kt, S0{}, S1{}, steady_);
			step(kt + 1, S1{}, S2{}, steady_);
			step(kt + 2, S2{}, S3{}, steady_);
			step(kt + 3, S3{}, S0{}, steady_);
		}
	};
	int kt = 0;
	for (; kt + 2 * NST - 1 < nkt; kt += NST)
		round(kt, std::true_type{});
	for (; kt + NST - 1 < nkt; kt += NST)
		round(kt, std::false_type{});
	if (kt < nkt) {
		step(kt, S0{}, S1{}, std::false_type{});
		if constexpr (NST >= 3) {
			if (kt + 1 < nkt)
				step(kt + 1, S1{}, S2{}, std::false_type{});
		}
		if constexpr (NST >= 4) {
			if (kt + 2 < nkt)
				step(kt + 2, S2{}, S3{}, std::false_type{});
		}
	}

	/* ---- the second K group hands its sums (and its share of the column sums) to the first and is done ---- */
	if constexpr (KG > 1) {
		typedef typename std::conditional<DT == THHIP_U8, int, float>::type accel;
		accel *xch = (accel *)lds_all;			/* [wave][accumulator register][lane] */
		int *xcs = (int *)(xch + TM * TN * 16 * 64 * WAVES);	/* [wave][tile column][lane] */
		__syncthreads();		/* every wave is done with the tiles */
		if (kg == 1) {
#pragma unroll
			for (int i = 0; i < TM; i++)
#pragma unroll
				for (int j = 0; j < TN; j++)
#pragma unroll
					for (int r = 0; r < 16; r++)
						xch[((wave * TM * TN + i * TN + j) * 16 + r) * 64 + lane] = acc[i][j][r];
			if constexpr (DT == THHIP_U8) {
#pragma unroll
				for (int j = 0; j < TN; j++)
					xcs[(wave * TN + j) * 64 + lane] = colsum[j];
			}
		}
		__syncthreads();
		if (kg == 1)
			return;		/* (a wavefront that has ended no longer counts at the workgroup's barriers) */
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] += xch[((wave * TM * TN + i * TN + j) * 16 + r) * 64 + lane];
		if constexpr (DT == THHIP_U8) {
#pragma unroll
			for (int j = 0; j < TN; j++)
				colsum[j] += xcs[(wave * TN + j) * 64 + lane];
		}
	}
	int *const lds_epi = (int *)lds_all;
	/* ---- epilogue ---- */
	if constexpr (DT != THHIP_U8) {
		if (tail_blk >= 0) {
			/* a part of one of the XCD's last tiles: the accumulators as they lie in
			 * the registers, [register][thread]; conv_wide_tail_finish_kernel adds
			 * the parts in their order */
			float *part = (float *)p.ws + tail_blk * (BM * BN);
#pragma unroll
			for (int i = 0; i < TM; i++)
#pragma unroll
				for (int j = 0; j < TN; j++)
#pragma unroll
					for (int r = 0; r < 16; r++)
						part[((i * TN + j) * 16 + r) * (64 * WAVES) + tid] = acc[i][j][r];
			return;
		}
		__syncthreads();		/* every wave is done with the tiles */
		conv_wide_store_half<DT, CLO, BM, BN, WGM, WGN, TM, TN, TM, TN>(p, acc, tile_m, tile_n, lds_epi);
	} else {
	elem *y = (elem *)p.y;
	int *lrow = lds_epi;		/* [BM] bias bits or uint8 row term, [BM..2BM) factor bits or uint8 addend */
	int *cs = lrow + 2 * BM;	/* uint8: [BN] column sums */
	__syncthreads();		/* every wave is done with the tiles */
	if (tid < BM) {
		const int mc = min(tile_m * BM + tid, p.Co - 1);
		lrow[tid] = p.offB * p.rowsum[mc] + p.K * p.offA * p.offB;
		lrow[BM + tid] = p.addend ? p.addend[mc] : 0;
	}
	if constexpr (DT == THHIP_U8) {
		for (int i = tid; i < BN; i += 64 * WAVES)	/* (the first K group's threads: the second has left) */
			cs[i] = 0;
		__syncthreads();
		if (wm == 0) {	/* the two halves of a column's K values sit in lanes l and l + 32 */
#pragma unroll
			for (int j = 0; j < TN; j++)
				atomicAdd(&cs[(wn * TN + j) * 32 + (lane & 31)], colsum[j]);
		}
	}
	__syncthreads();
	if constexpr (DT == THHIP_U8) {
		/* as in conv_mfma_kernel: sum (w+a_off)(x+b_off) expanded, gemmlowp's
		 * output stage, lowpadd with its unclamped tail, threshold */
		const int tail0 = (p.oHW / 8) * 8;
		const bool has_add = p.addend != 0;
		const bool cl16 = CLO && p.Co % 16 == 0 && ((size_t)p.y & 15) == 0;	/* whole 16-byte stores (conv_store_cl_u8) */
#pragma unroll
		for (int j = 0; j < TN; j++) {
			const int nl = (wn * TN + j) * 32 + (lane & 31);
			const int n = tile_n * BN + nl;
			const bool valid = n < p.N;
			if (!cl16 && !valid)
				continue;
			const int b = n / p.oHW, rem = n - b * p.oHW;
			const size_t ybase = (size_t)b * p.Co * p.oHW + rem;
			const int colterm = p.offA * cs[nl];
			const bool tail = rem >= tail0;
#pragma unroll
			for (int i = 0; i < TM; i++) {
				const int m0 = tile_m * BM + (wm * TM + i) * 32 + 4 * (lane >> 5);
				unsigned word[4];
#pragma unroll
				for (int g = 0; g < 4; g++) {
					unsigned packed = 0;
					const int ml = (wm * TM + i) * 32 + 4 * (lane >> 5) + 8 * g;
					const intx4 rowterm = *(const intx4 *)(lrow + ml);
					const intx4 rowadd = *(const intx4 *)(lrow + BM + ml);
#pragma unroll
					for (int e = 0; e < 4; e++) {
						const int r = 4 * g + e, m = m0 + 8 * g + e;
						const int a = acc[i][j][r] + rowterm[e] + colterm;
						int q = conv_requant(a, p.c_off, p.c_mult, p.c_shift);
						if (has_add) {
							const int sum = q + rowadd[e];
							q = sum > 255 ? 255 : (tail ? (sum & 255) : (sum < 0 ? 0 : sum));
						}
						if (p.act)
							q = q > p.ithr ? q : p.ival;
						if constexpr (CLO)
							packed |= (unsigned)q << (8 * e);
						else if (m < p.Co)
							y[ybase + (size_t)m * p.oHW] = (unsigned char)q;
					}
					if constexpr (CLO) {
						word[g] = packed;
						if (!cl16 && m0 + 8 * g < p.Co)
							*(unsigned *)(y + (size_t)n * p.Co + m0 + 8 * g) = packed;
					}
				}
				if constexpr (CLO) {
					if (cl16) {
						const int mt = tile_m * BM + (wm * TM + i) * 32;
						conv_store_cl_u8(y + (size_t)n * p.Co + mt, p.Co - mt, valid, word, lane);
					}
				}
			}
		}
	}
	}
#endif
}

/* Adds the K parts of the tiles conv_wide_kernel cut
 * ([xcd][tile][part][register][thread] in scratch) in their order and finishes
 * them as that kernel's epilogue does.  One workgroup per cut tile and
 * accumulator (i, j) of a wave, so that a thread waits for as many loads in
 * turn as there are parts, not TM * TN times that. */
template <int DT, bool CLO, int BM, int BN, int WGM, int WGN>
__global__ __launch_bounds__(64 * WGM * WGN) void conv_wide_tail_finish_kernel(ConvParams p)
{
	constexpr int TM = BM / WGM / 32, TN = BN / WGN / 32, THREADS = 64 * WGM * WGN;
	__shared__ int lrow[2 * BM];
	const int tid = threadIdx.x, xcd = blockIdx.x & 7;
	const int t = (blockIdx.x >> 3) / (TM * TN), ij = (blockIdx.x >> 3) % (TM * TN);
	int m0, mw, n0, cnt, full;
	conv_xcd_rect(p, xcd, m0, mw, n0, cnt);
	const int s = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
	if (s < 2 || t >= cnt - full)
		return;
	const int local = full + t;
	const float *part = (const float *)p.ws + ((long)xcd * p.tail_cap + t * s) * (BM * BN) + (ij * 16) * THREADS + tid;
	/* all parts requested at once (at most eight: conv_tail_plan), added in their order */
	floatx16 acc[1][1], in[8];
#pragma unroll
	for (int q = 0; q < 8; q++)
		if (q < s) {
#pragma unroll
			for (int r = 0; r < 16; r++)
				in[q][r] = part[(long)q * (BM * BN) + r * THREADS];
		}
	acc[0][0] = in[0];
#pragma unroll
	for (int q = 1; q < 8; q++)
		if (q < s) {
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[0][0][r] += in[q][r];
		}
	conv_wide_store_half<DT, CLO, BM, BN, WGM, WGN, TM, TN, 1, 1>(p, acc, m0 + local % mw, n0 + local / mw, lrow, ij / TN, ij % TN);
}

/* ------------------------------------------------------------------ */
/* 3x3, stride 1, 64 to 512 planes in: taps from an input patch in LDS */
/* ------------------------------------------------------------------ */


/* ------------------------------------------------------------------ */
/* fp32, plane-major: operands straight into LDS                       */
/* ------------------------------------------------------------------ */

/* Epilogue of the fp32 tiles whose accumulators are laid out as in
 * conv_f32_direct_kernel (2 x 2 waves): (folded batch norm factor,) bias,
 * optional threshold, plane-major store.  lrow: 2 * BM ints of LDS no wave
 * still reads. */
template <int BM, int BN, int TM, int TN>
__device__ __forceinline__ void conv_f32_direct_store(const ConvParams &p, floatx16 (&acc)[TM][TN], int tile_m, int tile_n, int *lrow)
{
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave % 2, wn = wave / 2;
	float *y = (float *)p.y;
	if (tid < BM) {
		const int mc = min(tile_m * BM + tid, p.Co - 1);
		lrow[tid] = __float_as_int(p.bias ? p.bias[mc] : 0.0f);
		if (p.scale)
			lrow[BM + tid] = __float_as_int(p.scale[mc]);
	}
	__syncthreads();
	const bool has_scale = p.scale != 0;
	/* With the pooling the first lane of a window (conv_pool_member) takes the maximum, with
	 * SpatialMaxPooling.c:51-66's comparisons in their order, and stores it. */
	const int oHW = p.pool ? p.pHW : p.oHW;
#pragma unroll
	for (int j = 0; j < TN; j++) {
		const int n = tile_n * BN + (wn * TN + j) * 32 + (lane & 31);
		int pos = n;
		bool valid = n < p.N;
		if (p.pool) {
			int dy, dx;
			conv_pool_member(n, pos, dy, dx);
			valid = pos < p.npool && !dy && !dx;
		} else if (!valid)
			continue;
		const int b = pos / oHW, rem = pos - b * oHW;
		const size_t ybase = (size_t)b * p.Co * oHW + rem;
#pragma unroll
		for (int i = 0; i < TM; i++) {
			const int m0 = tile_m * BM + (wm * TM + i) * 32 + 4 * (lane >> 5);
			/* the other tensor's sixteen values of this accumulator, all requested before the first is used */
			float other[16];
			if (p.res_mode) {
#pragma unroll
				for (int r = 0; r < 16; r++) {
					const int m = m0 + 8 * (r >> 2) + (r & 3);
					other[r] = valid && m < p.Co ? p.res[ybase + (size_t)m * oHW] : 0.0f;
				}
			}
#pragma unroll
			for (int g = 0; g < 4; g++) {
				const int ml = (wm * TM + i) * 32 + 4 * (lane >> 5) + 8 * g;
				const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
				floatx4 rowscale = { 1, 1, 1, 1 };
				if (has_scale)
					rowscale = *(const floatx4 *)(lrow + BM + ml);
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const int r = 4 * g + e, m = m0 + 8 * g + e;
					float v = has_scale ? acc[i][j][r] * rowscale[e] + rowbias[e] : acc[i][j][r] + rowbias[e];
					if (p.act)
						v = v > p.thr ? v : p.val;
					if (p.pool) {
						const float v01 = conv_lane_next(v);
						const float v10 = conv_lane_xor16(v), v11 = conv_lane_xor16(v01);
						float mx = -FLT_MAX;
						mx = v > mx ? v : mx;
						mx = v01 > mx ? v01 : mx;
						mx = v10 > mx ? v10 : mx;
						mx = v11 > mx ? v11 : mx;
						v = mx;
					}
					if (valid && m < p.Co) {
						if (p.res_mode) {
							v = p.res_mode == 1 ? v + p.res_c * other[r] : other[r] + p.res_c * v;
							if (p.res_act)
								v = v > 0.0f ? v : 0.0f;
						}
						y[ybase + (size_t)m * oHW] = v;
					}
				}
			}
		}
	}
}

/* The pipeline of conv_wide_kernel for the fp32 path (plane-major tensors as
 * the reference has them, tap-major K order: a K-tile is one filter tap x 32
 * planes).  The packed weights are copied in 1 KiB blocks as there.  Of the
 * input a wave-wide 4-byte load fetches one K value for 64 neighbouring
 * positions (coalesced along the output row; what lies outside the image is
 * pointed past the buffer's range and arrives as 0.0) and lands as one row of
 * the stage's B tile, [k][position].  A 32x32x2 MFMA takes B[k][n] from lane
 * (n, k): step s of a chunk reads rows 8 c + s (lanes 0..31) and 8 c + 4 + s
 * (lanes 32..63); rows are BN + 8 floats apart, so the two halves use different
 * banks.  Needs Ci % 32 == 0. */
#if defined(__HIP_DEVICE_COMPILE__)
template <int BM, int BN, int KCH, int NST, bool ROWS>
__device__ __forceinline__ void conv_f32_direct_body(const ConvParams &p, const int bid)
{
	constexpr int CHUNK = 8, KT = KCH * CHUNK, SUB = 4 / KCH, WAVES = 4, WGM = 2, WGN = 2;
	static_assert(KCH == 2 || KCH == 4, "the packed blocks of 32 planes are walked in one or two K-tiles");
	constexpr int MB = BM / 32, TM = BM / WGM / 32, TN = BN / WGN / 32;
	constexpr int BROW = BN + 8;				/* floats between B rows */
	constexpr int A_VECS = MB * KCH * 64, B_VECS = KT * BROW / 4, STAGE_VECS = A_VECS + B_VECS;
	constexpr int A_PW = MB * KCH / WAVES;			/* 1 KiB weight blocks per wave and K-tile */
	constexpr int NPOS = BN / 64;				/* positions per lane */
	constexpr int B_PW = KT / WAVES * NPOS;			/* 256-byte input rows per wave and K-tile */
	constexpr int LOADS = A_PW + B_PW;
	static_assert(MB * KCH % WAVES == 0 && BN % 64 == 0 && NST >= 3 && NST <= 4 && (NST - 1) * LOADS <= 48, "tile shape");
	static_assert(2 * BM * sizeof(int) <= NST * STAGE_VECS * sizeof(floatx4), "the epilogue's row constants fit");
	__shared__ floatx4 lds[NST * STAGE_VECS];

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave % WGM, wn = wave / WGM;

	int tile_m, tile_n, split = 0, nsplit = p.splitk > 1 ? p.splitk : 1;
	long tail_blk = -1;
	{	/* every XCD gets a rectangle of the tile grid, as in conv_mfma_kernel */
		
		const int xcd = bid & 7;
		int local = bid >> 3;
		if (p.splitk > 1) {	/* the parts of a tile are neighbours in the order */
			split = local % p.splitk;
			local /= p.splitk;
		}
		int m0, mw, n0, cnt;
		conv_xcd_rect(p, xcd, m0, mw, n0, cnt);
		if (p.tail_slots) {	/* the XCD's last tiles, dispatched last, in parts along K */
			int full;
			const int s = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
			if (s > 1 && local >= full) {
				const int t = (local - full) / s;
				split = (local - full) - t * s;
				nsplit = s;
				local = full + t;
				tail_blk = (long)xcd * p.tail_cap + t * s + split;
			}
		}
		if (p.tail_inline)
			conv_xcd_report(p, tail_blk >= 0);
		if (local >= cnt)
			return;
		tile_m = m0 + local % mw;
		tile_n = n0 + local / mw;
	}

	/* ---- this lane's positions: lane + 64 q of the tile ---- */
	bool n_ok_[NPOS];
	int iy0_[NPOS], ix0_[NPOS], xoff_[NPOS];
#pragma unroll
	for (int q = 0; q < NPOS; q++) {
		const int n_glob = tile_n * BN + q * 64 + lane;
		n_ok_[q] = n_glob < p.N;
		const int nn = n_ok_[q] ? n_glob : 0;
		int b, oy, ox;
		if (p.pool) {
			int pp, dy, dx;
			conv_pool_member(n_glob, pp, dy, dx);
			n_ok_[q] = pp < p.npool;
			pp = n_ok_[q] ? pp : 0;
			b = pp / p.pHW;
			const int r = pp - b * p.pHW, py = r / p.pW;
			oy = 2 * py + dy;
			ox = 2 * (r - py * p.pW) + dx;
		} else {
			b = nn / p.oHW;
			const int r = nn - b * p.oHW;
			oy = r / p.oW;
			ox = r - oy * p.oW;
		}
		iy0_[q] = oy * p.dH - p.padH;
		ix0_[q] = ox * p.dW - p.padW;
		xoff_[q] = b * p.Ci * p.HW + iy0_[q] * p.W + ix0_[q];
	}
	const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes, 0x00020000);
	const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.wp, 0, p.w_bytes, 0x00020000);
	unsigned a_off_[A_PW];
	int a_lds_[A_PW];
#pragma unroll
	for (int i = 0; i < A_PW; i++) {
		const int idx = wave + WAVES * i, mbi = idx % MB, kci = idx / MB;
		a_off_[i] = ((unsigned)(tile_m * MB + mbi) * (unsigned)p.KC + kci) * 1024u;
		a_lds_[i] = (kci * MB + mbi) * 64;
	}
	/* K-tiles: plane block outer, tap inner; with a K split this workgroup walks
	 * the K-tiles [kt0, kt0 + nkt) */
	const int nkt_all = p.KC / KCH;
	const int kt0 = nsplit > 1 ? (int)((long)nkt_all * split / nsplit) : 0;
	const int nkt = (nsplit > 1 ? (int)((long)nkt_all * (split + 1) / nsplit) : nkt_all) - kt0;
	int t_cb, t_kh, t_kw, t_kc = kt0 * KCH, t_sub;
	{
		const int blk = kt0 / SUB;
		t_sub = kt0 - blk * SUB;
		t_cb = blk / p.kHW;
		const int tap = blk - t_cb * p.kHW;
		t_kh = tap / p.kW;
		t_kw = tap - t_kh * p.kW;
	}
	const int plane_bytes = p.HW * (int)sizeof(float);
	/* ROWS (any number of planes, K order (plane, tap)): every row of a K-tile is a (plane, tap) of its own.
	 * This wave's rows wave + 4 r of the K-tile: plane, kernel row and column, walked on the scalar unit
	 * KT values at a time (KT = d_c kH kW + d_kh kW + d_kw). */
	constexpr int RPW = KT / WAVES;
	int r_c[RPW], r_kh[RPW], r_kw[RPW];
	int d_c = 0, d_kh = 0, d_kw = 0;
	if constexpr (ROWS) {
#pragma unroll
		for (int r = 0; r < RPW; r++) {
			const int k = kt0 * KT + wave + WAVES * r;
			r_c[r] = k / p.kHW;
			const int tap = k - r_c[r] * p.kHW;
			r_kh[r] = tap / p.kW;
			r_kw[r] = tap - r_kh[r] * p.kW;
		}
		d_c = KT / p.kHW;
		const int tap = KT - d_c * p.kHW;
		d_kh = tap / p.kW;
		d_kw = tap - d_kh * p.kW;
	}

	auto issue = [&](auto st_) {
		constexpr int st = decltype(st_)::value;
		floatx4 *la = lds + st * STAGE_VECS;
		float *lb = (float *)(la + A_VECS);
#pragma unroll
		for (int i = 0; i < A_PW; i++)
			__builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, WIDE_LDS(la + a_lds_[i]), 16, lane * 16,
				a_off_[i] + (unsigned)t_kc * 1024u, 0, 0);
		if constexpr (ROWS) {
#pragma unroll
			for (int r = 0; r < RPW; r++) {
				const int k = wave + WAVES * r;	/* row of the K-tile */
				const int tap_off = r_kh[r] * p.W + r_kw[r];
				const bool row_ok = r_c[r] < p.Ci;	/* (rows past K: zero weights, no plane) */
#pragma unroll
				for (int q = 0; q < NPOS; q++) {
					const int iy = iy0_[q] + r_kh[r], ix = ix0_[q] + r_kw[r];
					const bool ok = (int)n_ok_[q] & (int)row_ok & (int)((unsigned)iy < (unsigned)p.H) & (int)((unsigned)ix < (unsigned)p.W);
					const unsigned voff = ok ? (unsigned)(xoff_[q] + tap_off) * (unsigned)sizeof(float) : 0x80000000u;
					__builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, WIDE_LDS(lb + k * BROW + q * 64), 4, voff,
						row_ok ? r_c[r] * plane_bytes : 0, 0, 0);
				}
				/* KT values on: column, row and plane with their carries */
				const int kw1 = r_kw[r] + d_kw, cw = kw1 >= p.kW;
				r_kw[r] = __builtin_amdgcn_readfirstlane(cw ? kw1 - p.kW : kw1);
				const int kh1 = r_kh[r] + d_kh + cw, ch = kh1 >= p.kH;
				r_kh[r] = __builtin_amdgcn_readfirstlane(ch ? kh1 - p.kH : kh1);
				r_c[r] = __builtin_amdgcn_readfirstlane(r_c[r] + d_c + ch);
			}
			t_kc += KCH;
			return;
		}
		const int tap_off = t_kh * p.W + t_kw;
		const int plane0 = (t_cb * SUB + t_sub) * KT;
#pragma unroll
		for (int q = 0; q < NPOS; q++) {
			const int iy = iy0_[q] + t_kh, ix = ix0_[q] + t_kw;
			/* (no branches in a K step: the compiler may then spread its loads between the MFMAs) */
			const bool ok = (int)n_ok_[q] & (int)((unsigned)iy < (unsigned)p.H) & (int)((unsigned)ix < (unsigned)p.W);
			const unsigned voff = ok ? (unsigned)(xoff_[q] + tap_off) * (unsigned)sizeof(float) : 0x80000000u;
#pragma unroll
			for (int r = 0; r < KT / WAVES; r++) {
				const int k = wave + WAVES * r;	/* row of the K-tile */
				/* the scalar offset is not range checked: the planes exist */
				__builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, WIDE_LDS(lb + k * BROW + q * 64), 4, voff,
					(plane0 + k) * plane_bytes, 0, 0);
			}
		}
		t_kc += KCH;
		/* the next planes of the block first, then the next tap */
		const int sub1 = t_sub + 1, wrap_s = sub1 == SUB;
		t_sub = __builtin_amdgcn_readfirstlane(wrap_s ? 0 : sub1);
		const int kw1 = t_kw + wrap_s, wrap_w = kw1 == p.kW;
		t_kw = __builtin_amdgcn_readfirstlane(wrap_w ? 0 : kw1);
		const int kh1 = t_kh + wrap_w, wrap_h = kh1 == p.kH;
		t_kh = __builtin_amdgcn_readfirstlane(wrap_h ? 0 : kh1);
		t_cb = __builtin_amdgcn_readfirstlane(t_cb + wrap_h);
	};

	floatx4 af[2][TM], bf[2][TN];
	auto read_frags = [&](auto st_, int kci, floatx4 (&a)[TM], floatx4 (&b)[TN]) {
		constexpr int st = decltype(st_)::value;
		const floatx4 *la = lds + st * STAGE_VECS;
		const float *lb = (const float *)(la + A_VECS);
#pragma unroll
		for (int i = 0; i < TM; i++)
			a[i] = la[(kci * MB + wm * TM + i) * 64 + lane];
		const float *row = lb + (kci * CHUNK + (lane >> 5) * 4) * BROW + (lane & 31);
#pragma unroll
		for (int j = 0; j < TN; j++)
#pragma unroll
			for (int e = 0; e < 4; e++)
				b[j][e] = row[e * BROW + (wn * TN + j) * 32];
	};

	floatx16 acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; i++)
#pragma unroll
		for (int j = 0; j < TN; j++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[i][j][r] = 0;
	auto mma = [&](int set) {
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
				conv_mma<THHIP_F32>(acc[i][j], af[set][i], bf[set][j]);
	};

	typedef std::integral_constant<int, 0> S0;
	typedef std::integral_constant<int, 1> S1;
	typedef std::integral_constant<int, 2> S2;
	typedef std::integral_constant<int, NST >= 4 ? 3 : 0> S3;
	issue(S0{});
	if (1 < nkt)
		issue(S1{});
	if (2 < nkt)
		issue(S2{});
	if constexpr (NST >= 4) {
		if (3 < nkt)
			issue(S3{});
	}
	if (NST - 1 < nkt)
		wide_wait<(NST - 1) * LOADS, false>();
	else
		wide_wait<0, false>();
	__builtin_amdgcn_s_barrier();
	read_frags(S0{}, 0, af[0], bf[0]);
	/* as in conv_wide_kernel: one barrier per K-tile, before its last chunk */
	auto step = [&](int kt, auto st, auto st1, auto steady_) {
		constexpr bool steady = decltype(steady_)::value;
#pragma unroll
		for (int c = 0; c + 1 < KCH; c++) {
			read_frags(st, c + 1, af[(c + 1) & 1], bf[(c + 1) & 1]);
			/* the next chunk's fragments are asked for before this chunk's MFMAs (left alone, the
			 * compiler puts the reads right before their first use) */
			__builtin_amdgcn_sched_barrier(0);
			mma(c & 1);
		}
		if (steady)
			wide_wait<(NST - 2) * LOADS, true>();
		else
			wide_wait<0, true>();
		__builtin_amdgcn_s_barrier();
		if (steady || kt + 1 < nkt)
			read_frags(st1, 0, af[0], bf[0]);
		__builtin_amdgcn_sched_barrier(0);	/* (as above; the loads below mix with the MFMAs) */
		if (steady || kt + NST < nkt)
			issue(st);
		mma((KCH - 1) & 1);
	};
	auto round = [&](int kt, auto steady_) {
		if constexpr (NST == 3) {
			step(kt, S0{}, S1{}, steady_);
			step(kt + 1, S1{}, S2{}, steady_);
			step(kt + 2, S2{}, S0{}, steady_);
		} else {
			step(kt, S0{}, S1{}, steady_);
			step(kt + 1, S1{}, S2{}, steady_);
			step(kt + 2, S2{}, S3{}, steady_);
			step(kt + 3, S3{}, S0{}, steady_);
		}
	};
	int kt = 0;
	for (; kt + 2 * NST - 1 < nkt; kt += NST)
		round(kt, std::true_type{});
	for (; kt + NST - 1 < nkt; kt += NST)
		round(kt, std::false_type{});
	if (kt < nkt) {
		step(kt, S0{}, S1{}, std::false_type{});
		if (kt + 1 < nkt)
			step(kt + 1, S1{}, S2{}, std::false_type{});
		if constexpr (NST >= 4) {
			if (kt + 2 < nkt)
				step(kt + 2, S2{}, S3{}, std::false_type{});
		}
	}

	if (tail_blk >= 0) {
		/* a part of one of the XCD's last tiles: the accumulators as they lie in the registers,
		 * [register][thread], in block tail_blk of scratch */
		const long blk0 = tail_blk - split;
		float *part = (float *)p.ws + (blk0 + split) * (BM * BN);
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					part[((i * TN + j) * 16 + r) * 256 + tid] = acc[i][j][r];
		if (!p.tail_inline)
			return;		/* conv_f32_tail_finish_kernel adds the parts */
		/* the part that arrives last adds them all in their order (four on their way at a time) */
		if (!conv_xcd_last_arriver(p, p.cnt + blk0, nsplit, (int *)lds))
			return;
		const float *all = (const float *)p.ws + blk0 * (BM * BN) + tid;
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
				for (int q0 = 0; q0 < nsplit; q0 += 4) {
					float in[4][16];
#pragma unroll
					for (int q = 0; q < 4; q++)
						if (q0 + q < nsplit) {
#pragma unroll
							for (int r = 0; r < 16; r++)
								in[q][r] = conv_load_part(all + (long)(q0 + q) * (BM * BN) + ((i * TN + j) * 16 + r) * 256);
						}
#pragma unroll
					for (int q = 0; q < 4; q++)
						if (q0 + q < nsplit) {
#pragma unroll
							for (int r = 0; r < 16; r++)
								acc[i][j][r] = q0 + q == 0 ? in[q][r] : acc[i][j][r] + in[q][r];
						}
				}
		__syncthreads();
		conv_f32_direct_store<BM, BN, TM, TN>(p, acc, tile_m, tile_n, (int *)lds);
		return;
	}
	if (p.splitk > 1) {
		/* this part's sums as they are, [part][plane][position]; a finishing kernel
		 * adds the parts in a fixed order (the result does not depend on timing) */
		float *part = (float *)p.ws + (size_t)split * p.Co * p.N;
#pragma unroll
		for (int j = 0; j < TN; j++) {
			const int n = tile_n * BN + (wn * TN + j) * 32 + (lane & 31);
			if (n >= p.N)
				continue;
#pragma unroll
			for (int i = 0; i < TM; i++) {
				const int m0 = tile_m * BM + (wm * TM + i) * 32 + 4 * (lane >> 5);
#pragma unroll
				for (int r = 0; r < 16; r++) {
					const int m = m0 + 8 * (r >> 2) + (r & 3);
					if (m < p.Co)
						part[(size_t)m * p.N + n] = acc[i][j][r];
				}
			}
		}
		return;
	}
	__syncthreads();
	conv_f32_direct_store<BM, BN, TM, TN>(p, acc, tile_m, tile_n, (int *)lds);
}
#endif

template <int BM, int BN, int KCH, int NST, bool ROWS = false>
__global__ __launch_bounds__(256) void conv_f32_direct_kernel(ConvParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)	/* as for conv_wide_kernel: the host pass gets the stub only */
	conv_f32_direct_body<BM, BN, KCH, NST, ROWS>(p, (int)blockIdx.x);
#endif
}

/* Two layers that do not depend on each other in one launch (workgroups 0 .. na - 1 run a, the others b): a
 * short layer beside a longer one fills the CUs the longer one leaves idle at its end, and costs no launch
 * of its own (the 1x1 shortcut projection of a residual block beside the block's first convolution). */
template <int BM, int BN, int KCH, int NST, bool ROWS = false>
__global__ __launch_bounds__(256) void conv_f32_direct_pair_kernel(ConvParams a, ConvParams b, int na)
{
#if defined(__HIP_DEVICE_COMPILE__)
	const bool first = (int)blockIdx.x < na;
	conv_f32_direct_body<BM, BN, KCH, NST, ROWS>(first ? a : b, first ? (int)blockIdx.x : (int)blockIdx.x - na);
#endif
}

/* ------------------------------------------------------------------ */
/* fp32, plane-major, 3x3 / stride 1 / padding 1: taps from a patch in LDS */
/* ------------------------------------------------------------------ */

/* A tile of conv_f32_patch_kernel: 64 output pixels as NP patches of SW x SH (16x4, 8x8: one patch;
 * 4x4: four neighbouring patches in the order image, patch row, patch column). */
template <int SW, int SH>
struct ConvPatchGeo {
	static_assert((SW == 16 && SH == 4) || (SW == 8 && SH == 8) || (SW == 4 && SH == 4), "16x4, 8x8 or four 4x4 patches");
	static constexpr int NPOS = SW * SH, NP = 64 / NPOS;
	static constexpr int PWD = SW + 2, PEL_S = (SH + 2) * PWD;	/* the input under one patch: row length, elements */
	static constexpr int PEL = NP * PEL_S, NL = (PEL + 63) / 64;	/* elements and wave-wide loads per plane */
	static constexpr int PSTRIDE = 64 * NL + 4;	/* floats between the planes of a buffer (four planes = 16 banks) */
};

/* patch sp of the layer: image and first output pixel; false past the last patch */
template <int SW, int SH>
__device__ __forceinline__ bool conv_patch_origin(const ConvParams &p, int sp, int &b, int &y0, int &x0)
{
	const int SX = p.oW / SW, SXY = SX * (p.oH / SH);
	b = sp / SXY;
	const int rem = sp - b * SXY, sy = rem / SX;
	y0 = sy * SH;
	x0 = (rem - sy * SX) * SW;
	return b < p.B;
}

/* v of lane ^ 8, v of lane ^ 4 */
__device__ __forceinline__ float conv_lane_xor8(float v)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x201F));
}

__device__ __forceinline__ float conv_lane_xor4(float v)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x101F));
}

/* Epilogue of conv_f32_patch_kernel: position n = wn 32 + lane % 32 of tile tile_n is pixel
 * ((n % NPOS) / SW, n % SW) of patch tile_n NP + n / NPOS.  (Folded batch norm factor,) bias, threshold,
 * the 2x2 / stride 2 max pooling that follows (a window's other column is the next lane, its other row
 * lane ^ SW; SpatialMaxPooling.c:51-66's comparisons in their order), the second tensor of a table
 * add, plane-major store.  lrow: 128 ints of LDS no wave still reads. */
template <int SW, int SH>
__device__ __forceinline__ void conv_f32_patch_store(const ConvParams &p, floatx16 &acc, int tile_m, int tile_n, int *lrow)
{
	typedef ConvPatchGeo<SW, SH> GEO;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave % 2, wn = wave / 2;
	float *y = (float *)p.y;
	if (tid < 64) {
		const int mc = min(tile_m * 64 + tid, p.Co - 1);
		lrow[tid] = __float_as_int(p.bias ? p.bias[mc] : 0.0f);
		if (p.scale)
			lrow[64 + tid] = __float_as_int(p.scale[mc]);
	}
	__syncthreads();
	const bool has_scale = p.scale != 0;
	const int n = wn * 32 + (lane & 31), ln = n % GEO::NPOS, py = ln / SW, px = ln % SW;
	int b, y0, x0;
	bool valid = conv_patch_origin<SW, SH>(p, tile_n * GEO::NP + n / GEO::NPOS, b, y0, x0);
	b = valid ? b : 0;
	const int oHW = p.pool ? p.pHW : p.oHW;
	if (p.pool)
		valid = valid && !(py & 1) && !(px & 1);
	const size_t ybase = (size_t)b * p.Co * oHW +
		(p.pool ? ((y0 + py) >> 1) * p.pW + ((x0 + px) >> 1) : (y0 + py) * p.oW + x0 + px);
	const int m0 = tile_m * 64 + wm * 32 + 4 * (lane >> 5);
	/* the other tensor's sixteen values, all requested before the first is used */
	float other[16];
	if (p.res_mode) {
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int m = m0 + 8 * (r >> 2) + (r & 3);
			other[r] = valid && m < p.Co ? p.res[ybase + (size_t)m * oHW] : 0.0f;
		}
	}
#pragma unroll
	for (int g = 0; g < 4; g++) {
		const int ml = wm * 32 + 4 * (lane >> 5) + 8 * g;
		const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
		floatx4 rowscale = { 1, 1, 1, 1 };
		if (has_scale)
			rowscale = *(const floatx4 *)(lrow + 64 + ml);
#pragma unroll
		for (int e = 0; e < 4; e++) {
			const int r = 4 * g + e, m = m0 + 8 * g + e;
			float v = has_scale ? acc[r] * rowscale[e] + rowbias[e] : acc[r] + rowbias[e];
			if (p.act)
				v = v > p.thr ? v : p.val;
			if (p.pool) {
				const float v01 = conv_lane_next(v);
				const float v10 = SW == 16 ? conv_lane_xor16(v) : SW == 8 ? conv_lane_xor8(v) : conv_lane_xor4(v);
				const float v11 = SW == 16 ? conv_lane_xor16(v01) : SW == 8 ? conv_lane_xor8(v01) : conv_lane_xor4(v01);
				float mx = -FLT_MAX;
				mx = v > mx ? v : mx;
				mx = v01 > mx ? v01 : mx;
				mx = v10 > mx ? v10 : mx;
				mx = v11 > mx ? v11 : mx;
				v = mx;
			}
			if (valid && m < p.Co) {
				if (p.res_mode) {
					v = p.res_mode == 1 ? v + p.res_c * other[r] : other[r] + p.res_c * v;
					if (p.res_act)
						v = v > 0.0f ? v : 0.0f;
				}
				y[ybase + (size_t)m * oHW] = v;
			}
		}
	}
}

/* 3x3 / stride 1 / padding 1 layers whose output splits into whole 16x4, 8x8 or 4x4 patches: a
 * workgroup computes 64 planes of 64 pixels (one patch, or four of 4x4).  Where
 * conv_f32_direct_kernel fetches every tap's 64 pixels of a plane with a load of its own (nine loads
 * a plane, 0.5 wave-wide loads per MFMA: measured, they cost 5-8 % of that kernel's time even when
 * they all hit the cache), this kernel loads the (SH + 2) x (SW + 2) input pixels under each patch
 * once per plane (two or three loads, what lies outside the image pointed past the buffer's range
 * and so 0.0) and every tap reads them from LDS at its own offset; no tap arithmetic and no bounds
 * tests remain in the K loop.  The packed weights' K order (block of 32 planes, tap, plane) is
 * walked as (half block of 16 planes, tap): sixteen planes' patches are one buffer (two buffers, the
 * next half block's loads spread over this one's taps), the weights' 1 KiB blocks go through a ring
 * of three K-tiles as in conv_f32_direct_kernel.  The nine taps of a half block are straight-line
 * code: every LDS offset and wait count a constant.  The last tiles of an XCD are cut along K as
 * there (conv_tail_parts; a part is whole half blocks of 16 planes) and added by the workgroup whose part
 * is ready last (conv_xcd_last_arriver), or, with THHipSumPartsInKernel(0), by
 * conv_f32_patch_tail_finish_kernel. */
template <int SW, int SH>
__global__ __launch_bounds__(256) void conv_f32_patch_kernel(ConvParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)	/* as for conv_wide_kernel: the host pass gets the stub only */
	typedef ConvPatchGeo<SW, SH> GEO;
	constexpr int MB = 2, KCH = 2, NST = 3, BLK = 16;
	constexpr int PWD = GEO::PWD, PSTRIDE = GEO::PSTRIDE, NL = GEO::NL;
	constexpr int BL = 4 * NL;	/* patch loads per wave and half block: planes wave + 4 i, NL loads each */
	static_assert(BL <= 8 || BL == 12, "the patch loads are spread over the first taps of a half block");
	constexpr int A_VECS = MB * KCH * 64, B_FLOATS = BLK * PSTRIDE;
	/* (one array, every stage and buffer at a constant offset, as in the kernels above: with separate
	 * arrays, or a buffer index computed at run time, the compiler waits for all outstanding loads
	 * before every LDS read) */
	__shared__ floatx4 lds[NST * A_VECS + 2 * B_FLOATS / 4];
	floatx4 *const lds_a = lds;
	float *const lds_b0 = (float *)(lds + NST * A_VECS), *const lds_b1 = lds_b0 + B_FLOATS;

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave % 2, wn = wave / 2;
	int tile_m, tile_n, split = 0, nsplit = 1;
	long tail_blk = -1;
	{	/* every XCD gets a rectangle of the tile grid, its last tiles in parts along K, as in conv_f32_direct_kernel */
		const int bid = blockIdx.x, xcd = bid & 7;
		int local = bid >> 3;
		int m0, mw, n0, cnt;
		conv_xcd_rect(p, xcd, m0, mw, n0, cnt);
		if (p.tail_slots) {
			int full;
			const int s = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
			if (s > 1 && local >= full) {
				const int t = (local - full) / s;
				split = (local - full) - t * s;
				nsplit = s;
				local = full + t;
				tail_blk = (long)xcd * p.tail_cap + t * s + split;
			}
		}
		if (p.tail_inline)
			conv_xcd_report(p, tail_blk >= 0);
		if (local >= cnt)
			return;
		tile_m = m0 + local % mw;
		tile_n = n0 + local / mw;
	}
	/* this workgroup's half blocks of 16 planes [hb0, hb1) */
	const int blocks16 = p.Ci / 16;
	const int hb0 = (int)((long)blocks16 * split / nsplit), hb1 = (int)((long)blocks16 * (split + 1) / nsplit);

	/* ---- what this lane fetches of every plane: elements lane + 64 j of the tile's patches ---- */
	unsigned voff_[NL];
#pragma unroll
	for (int j = 0; j < NL; j++) {
		const int e = 64 * j + lane, q = e / GEO::PEL_S, le = e - q * GEO::PEL_S, r = le / PWD, c = le - r * PWD;
		int b, y0, x0;
		bool ok = conv_patch_origin<SW, SH>(p, tile_n * GEO::NP + q, b, y0, x0) && e < GEO::PEL;
		const int iy = y0 - 1 + r, ix = x0 - 1 + c;
		ok = ok && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
		voff_[j] = ok ? (unsigned)(((b * p.Ci * p.H + iy) * p.W + ix) * (int)sizeof(float)) : 0x80000000u;
	}
	const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes, 0x00020000);
	const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.wp, 0, p.w_bytes, 0x00020000);
	const int plane_bytes = p.HW * (int)sizeof(float);
	/* this wave's weight block of a K-tile: 32-row block wave % 2, chunk wave / 2 */
	const unsigned a_base = (unsigned)(tile_m * MB + wave % MB) * (unsigned)p.KC * 1024u;
	const int a_kci = wave / MB, a_lds = (a_kci * MB + wave % MB) * 64;

	/* the weights of K-tile (half block hb, tap): chunks ((hb / 2) 9 + tap) 4 + (hb % 2) 2 + {0, 1};
	 * past the last half block nothing is fetched (zeros arrive, nobody reads them) */
	auto issue_a = [&](auto st_, int hb, int tap) {
		constexpr int st = decltype(st_)::value;
		const unsigned kc = (unsigned)(((hb >> 1) * 9 + tap) * 4 + (hb & 1) * 2 + a_kci);
		__builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, WIDE_LDS(lds_a + st * A_VECS + a_lds), 16,
			hb < hb1 ? lane * 16 : 0x80000000u, a_base + kc * 1024u, 0, 0);
	};
	/* load t (0 .. BL-1) of this wave's share of half block hb's patches into buffer buf: plane
	 * wave + 4 (t / NL), elements 64 (t % NL).. */
	auto issue_b = [&](auto t_, int hb, auto buf_) {
		constexpr int buf = decltype(buf_)::value, t = decltype(t_)::value;
		const int plane = wave + 4 * (t / NL);
		constexpr int j = t % NL;
		float *dst = (buf ? lds_b1 : lds_b0) + plane * PSTRIDE + 64 * j;
		/* the scalar offset is not range checked: the planes exist (hb < hb1) */
		__builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, WIDE_LDS(dst), 4,
			hb < hb1 ? voff_[j] : 0x80000000u, hb < hb1 ? (hb * BLK + plane) * plane_bytes : 0, 0, 0);
	};

	/* fragments: A rows lane % 32 of block wm, half lane / 32; B pixel n of the tile, planes
	 * 8 chunk + 4 (lane / 32) + step of the half block, at the tap's offset */
	const int n = wn * 32 + (lane & 31), ln = n % GEO::NPOS;
	const int bfrag = (lane >> 5) * 4 * PSTRIDE + (n / GEO::NPOS) * GEO::PEL_S + (ln / SW) * PWD + ln % SW;
	auto read_frags = [&](auto st_, auto buf_, auto tap_, int c, floatx4 &a, floatx4 &bq) {
		constexpr int st = decltype(st_)::value, tap = decltype(tap_)::value, buf = decltype(buf_)::value;
		a = lds_a[st * A_VECS + (c * MB + wm) * 64 + lane];
		const float *src = (buf ? lds_b1 : lds_b0) + bfrag + (tap / 3) * PWD + tap % 3 + c * 8 * PSTRIDE;
#pragma unroll
		for (int e = 0; e < 4; e++)
			bq[e] = src[e * PSTRIDE];
	};

	floatx16 acc;
#pragma unroll
	for (int r = 0; r < 16; r++)
		acc[r] = 0;
	floatx4 af[2], bf[2];

	typedef std::integral_constant<int, 0> C0;
	typedef std::integral_constant<int, 1> C1;
	typedef std::integral_constant<int, 2> C2;
	/* Patch loads of the next half block: BL of them over the nine steps of this one, step `tap` issues
	 * numbers [PB(tap), PB(tap + 1)): one a step (BL = 8: none in the last) or two in each of the
	 * first four steps and one after (BL = 12: none in the last). */
#define CONV_PATCH_PB(tap) (BL == 8 ? ((tap) < 8 ? (tap) : 8) : ((tap) < 4 ? 2 * (tap) : (tap) < 8 ? 4 + (tap) : 12))
	{
		auto all_b = [&](auto self, auto t_) {
			constexpr int t = decltype(t_)::value;
			if constexpr (t < BL) {
				issue_b(t_, hb0, C0{});
				self(self, std::integral_constant<int, t + 1>{});
			}
		};
		all_b(all_b, C0{});
	}
	issue_a(C0{}, hb0, 0);
	issue_a(C1{}, hb0, 1);
	issue_a(C2{}, hb0, 2);
	wide_wait<2, false>();	/* the patches and the first K-tile's weights */
	__builtin_amdgcn_s_barrier();
	read_frags(C0{}, C0{}, C0{}, 0, af[0], bf[0]);

	/* K-tile (hb, tap): its weights in stage tap % 3, the next K-tile's in the next stage.  A step issues its
	 * patch loads first, its weights last; the weights of the next K-tile were issued two steps ago, so what
	 * may still be on its way is the last step's loads.  A half block's last step waits for the patch loads
	 * of the next as well (none are issued in that step, the last before it are older than that step's
	 * weights). */
	auto step = [&](int hb, auto buf_, auto tap_) {
		constexpr int tap = decltype(tap_)::value, buf = decltype(buf_)::value;
		typedef std::integral_constant<int, tap % 3> ST;
		typedef std::integral_constant<int, (tap + 1) % 3> ST1;
		typedef std::integral_constant<int, (tap + 1) % 9> TAP1;
		typedef std::integral_constant<int, buf ^ 1> OTHER;
		typedef std::integral_constant<int, tap == 8 ? buf ^ 1 : buf> BUF1;
		constexpr int prev = (tap + 8) % 9;	/* the step before */
		constexpr int last_loads = 1 + CONV_PATCH_PB(prev + 1) - CONV_PATCH_PB(prev);
		read_frags(ST{}, buf_, tap_, 1, af[1], bf[1]);
		/* (the fragments are asked for before the MFMAs that follow in the source; left alone, the
		 * compiler puts the reads right before their first use) */
		__builtin_amdgcn_sched_barrier(0);
		conv_mma<THHIP_F32>(acc, af[0], bf[0]);
		wide_wait<tap == 8 ? 1 : last_loads, true>();
		__builtin_amdgcn_s_barrier();
		read_frags(ST1{}, BUF1{}, TAP1{}, 0, af[0], bf[0]);
		__builtin_amdgcn_sched_barrier(0);
		if constexpr (CONV_PATCH_PB(tap + 1) - CONV_PATCH_PB(tap) >= 1)
			issue_b(std::integral_constant<int, CONV_PATCH_PB(tap)>{}, hb + 1, OTHER{});
		if constexpr (CONV_PATCH_PB(tap + 1) - CONV_PATCH_PB(tap) >= 2)
			issue_b(std::integral_constant<int, CONV_PATCH_PB(tap) + 1>{}, hb + 1, OTHER{});
		if constexpr (tap + 3 < 9)
			issue_a(ST{}, hb, tap + 3);
		else
			issue_a(ST{}, hb + 1, tap + 3 - 9);
		conv_mma<THHIP_F32>(acc, af[1], bf[1]);
	};
#undef CONV_PATCH_PB
	auto half_block = [&](int hb, auto buf_) {
		step(hb, buf_, std::integral_constant<int, 0>{});
		step(hb, buf_, std::integral_constant<int, 1>{});
		step(hb, buf_, std::integral_constant<int, 2>{});
		step(hb, buf_, std::integral_constant<int, 3>{});
		step(hb, buf_, std::integral_constant<int, 4>{});
		step(hb, buf_, std::integral_constant<int, 5>{});
		step(hb, buf_, std::integral_constant<int, 6>{});
		step(hb, buf_, std::integral_constant<int, 7>{});
		step(hb, buf_, std::integral_constant<int, 8>{});
	};
	for (int hb = hb0; hb < hb1; hb += 2) {	/* (a part may be an odd number of half blocks; the first goes to buffer 0) */
		half_block(hb, C0{});
		if (hb + 1 < hb1)
			half_block(hb + 1, C1{});
	}
	wide_wait<0, false>();	/* (the loads past the end bring zeros into LDS: done before the workgroup ends or the epilogue reuses it) */
	if (tail_blk >= 0) {
		/* a part of one of the XCD's last tiles: the accumulator as it lies in the registers,
		 * [register][thread] */
		float *part = (float *)p.ws + tail_blk * (64 * 64);
#pragma unroll
		for (int r = 0; r < 16; r++)
			part[r * 256 + tid] = acc[r];
		if (!p.tail_inline)
			return;		/* conv_f32_patch_tail_finish_kernel adds the parts */
		/* the part that arrives last adds them all in their order (four on their way at a time) */
		if (!conv_xcd_last_arriver(p, p.cnt + (tail_blk - split), nsplit, (int *)lds_a))
			return;
		const float *all = (const float *)p.ws + (tail_blk - split) * (64 * 64) + tid;
		for (int q0 = 0; q0 < nsplit; q0 += 4) {
			float in[4][16];
#pragma unroll
			for (int q = 0; q < 4; q++)
				if (q0 + q < nsplit) {
#pragma unroll
					for (int r = 0; r < 16; r++)
						in[q][r] = conv_load_part(all + (long)(q0 + q) * (64 * 64) + r * 256);
				}
#pragma unroll
			for (int q = 0; q < 4; q++)
				if (q0 + q < nsplit) {
#pragma unroll
					for (int r = 0; r < 16; r++)
						acc[r] = q0 + q == 0 ? in[q][r] : acc[r] + in[q][r];
				}
		}
	}
	__syncthreads();
	conv_f32_patch_store<SW, SH>(p, acc, tile_m, tile_n, (int *)lds_a);
#endif
}

/* Adds the K parts of the tiles conv_f32_patch_kernel cut (one workgroup per such tile,
 * [xcd][tile][part][register][thread] in scratch) in their order and finishes them as that kernel's
 * epilogue does. */
template <int SW, int SH>
__global__ __launch_bounds__(256) void conv_f32_patch_tail_finish_kernel(ConvParams p)
{
	__shared__ int lrow[128];
	const int tid = threadIdx.x, xcd = blockIdx.x & 7, t = blockIdx.x >> 3;
	int m0, mw, n0, cnt, full;
	conv_xcd_rect(p, xcd, m0, mw, n0, cnt);
	const int s = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
	if (s < 2 || t >= cnt - full)
		return;
	const int local = full + t;
	const float *part = (const float *)p.ws + ((long)xcd * p.tail_cap + t * s) * (64 * 64);
	floatx16 in[8];		/* all parts requested at once (at most eight: conv_tail_plan), added in their order */
#pragma unroll
	for (int q = 0; q < 8; q++)
		if (q < s) {
#pragma unroll
			for (int r = 0; r < 16; r++)
				in[q][r] = part[(long)q * (64 * 64) + r * 256 + tid];
		}
	floatx16 acc = in[0];
#pragma unroll
	for (int q = 1; q < 8; q++)
		if (q < s) {
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[r] += in[q][r];
		}
	conv_f32_patch_store<SW, SH>(p, acc, m0 + local % mw, n0 + local / mw, lrow);
}

/* Adds the K parts of the tiles conv_f32_direct_kernel cut (one workgroup per
 * such tile, [xcd][tile][part][register][thread] in scratch) in their order
 * and finishes them as that kernel's epilogue does. */
template <int BM, int BN>
__global__ __launch_bounds__(256) void conv_f32_tail_finish_kernel(ConvParams p)
{
	constexpr int TM = BM / 64, TN = BN / 64;
	__shared__ int lrow[2 * BM];
	const int tid = threadIdx.x, xcd = blockIdx.x & 7, t = blockIdx.x >> 3;
	int m0, mw, n0, cnt, full;
	conv_xcd_rect(p, xcd, m0, mw, n0, cnt);
	const int s = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
	if (s < 2 || t >= cnt - full)
		return;
	const int local = full + t;
	const float *part = (const float *)p.ws + ((long)xcd * p.tail_cap + t * s) * (BM * BN);
	floatx16 acc[TM][TN];
	/* accumulator by accumulator: all parts requested at once (at most eight:
	 * conv_tail_plan), added in their order */
#pragma unroll
	for (int i = 0; i < TM; i++)
#pragma unroll
		for (int j = 0; j < TN; j++) {
			floatx16 in[8];
#pragma unroll
			for (int q = 0; q < 8; q++)
				if (q < s) {
#pragma unroll
					for (int r = 0; r < 16; r++)
						in[q][r] = part[(long)q * (BM * BN) + ((i * TN + j) * 16 + r) * 256 + tid];
				}
			acc[i][j] = in[0];
#pragma unroll
			for (int q = 1; q < 8; q++)
				if (q < s) {
#pragma unroll
					for (int r = 0; r < 16; r++)
						acc[i][j][r] += in[q][r];
				}
		}
	conv_f32_direct_store<BM, BN, TM, TN>(p, acc, m0 + local % mw, n0 + local / mw, lrow);
}

/* Sums the parts of a K split, [part][plane][position] fp32, in their order and
 * finishes as the convolution epilogue does; plane-major output. */
__global__ void conv_f32_splitk_finish_kernel(const float *ws, const float *bias, const float *scale, float *y,
	int parts, int Co, int N, int oHW, int act, float thr, float val, const float *res, int res_mode, float res_c, int res_act)
{
	const long total = (long)Co * N;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const int m = (int)(i / N), n = (int)(i - (long)m * N);
		float v = 0;
		for (int s = 0; s < parts; s++)
			v += ws[(size_t)s * total + i];
		/* (the factor and the bias in one rounding, said here so that it does not hang on how the compiler contracts) */
		v = scale ? __builtin_fmaf(v, scale[m], bias ? bias[m] : 0.0f) : v + (bias ? bias[m] : 0.0f);
		if (act)
			v = v > thr ? v : val;
		const int b = n / oHW, rem = n - b * oHW;
		const size_t at = ((size_t)b * Co + m) * oHW + rem;
		if (res_mode) {
			const float r = res[at];
			v = res_mode == 1 ? v + res_c * r : r + res_c * v;
			if (res_act)
				v = v > 0.0f ? v : 0.0f;
		}
		y[at] = v;
	}
}

/* The same for layers whose positions (batch x plane size) are a multiple of four: a thread adds and
 * finishes four neighbouring positions (16-byte reads of the parts, a quarter of the index arithmetic);
 * the same values. */
__global__ void conv_f32_splitk_finish4_kernel(const float *ws, const float *bias, const float *scale, float *y,
	int parts, int Co, int N, int oHW, int act, float thr, float val, const float *res, int res_mode, float res_c, int res_act)
{
	const int N4 = N >> 2;
	const long total4 = (long)Co * N4, total = (long)Co * N;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total4; i += step) {
		const int m = (int)(i / N4), n = (int)(i - (long)m * N4) * 4;
		floatx4 v = { 0, 0, 0, 0 };
		for (int s = 0; s < parts; s++) {
			const floatx4 w = *(const floatx4 *)(ws + (size_t)s * total + (size_t)m * N + n);
#pragma unroll
			for (int e = 0; e < 4; e++)
				v[e] += w[e];
		}
		const float bi = bias ? bias[m] : 0.0f, sc = scale ? scale[m] : 1.0f;
		const int b = n / oHW, rem = n - b * oHW;
		const size_t at = ((size_t)b * Co + m) * oHW + rem;
		/* the four lie in one image at an aligned address (always, for plane sizes that are multiples of four):
		 * 16-byte accesses to the output (and the second tensor) too */
		const bool together = rem + 3 < oHW && (at & 3) == 0;
		floatx4 r = { 0, 0, 0, 0 };
		if (res_mode) {
			if (together)
				r = *(const floatx4 *)(res + at);
			else {
#pragma unroll
				for (int e = 0; e < 4; e++) {
					const int ne = n + e, be = ne / oHW;
					r[e] = res[((size_t)be * Co + m) * oHW + (ne - be * oHW)];
				}
			}
		}
#pragma unroll
		for (int e = 0; e < 4; e++) {
			float u = scale ? __builtin_fmaf(v[e], sc, bi) : v[e] + bi;
			if (act)
				u = u > thr ? u : val;
			if (res_mode) {
				u = res_mode == 1 ? u + res_c * r[e] : r[e] + res_c * u;
				if (res_act)
					u = u > 0.0f ? u : 0.0f;
			}
			v[e] = u;
		}
		if (together)
			*(floatx4 *)(y + at) = v;
		else {
#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int ne = n + e, be = ne / oHW;
				y[((size_t)be * Co + m) * oHW + (ne - be * oHW)] = v[e];
			}
		}
	}
}

/* The same followed by a max pooling (any window, SpatialMaxPooling.c:6-98): LPO (four or sixteen) lanes per
 * pooled value, a lane per value of the window (lane, lane + LPO, ... for larger windows).  A lane adds the
 * parts of its values and finishes them as above; the maximum is then taken over those lanes as
 * the reference's scan would: the first of equal values wins (+0 and -0), values that are not greater
 * than -FLT_MAX (NaNs) never do.  y is the pooled tensor, plane-major.  For the layers of a few tiles
 * that split K (a batch of one or a few images), where the pooling's own launch costs as much as its
 * work. */
template <int LPO>
__global__ __launch_bounds__(256) void conv_f32_splitk_finish_pool_kernel(const float *ws, const float *bias, const float *scale, float *y,
	int parts, int B, int Co, int N, int oH, int oW, int act, float thr, float val,
	int kH, int kW, int dH, int dW, int padH, int padW, int pH, int pW)
{
	const long total = (long)B * Co * pH * pW, part = (long)Co * N;
	const long i = ((long)blockIdx.x * 256 + threadIdx.x) / LPO;
	const int l = threadIdx.x % LPO;
	float mx = -FLT_MAX;
	int me = 0x7fffffff;	/* the window element mx came from */
	if (i < total) {
		const int px = (int)(i % pW);
		long t = i / pW;
		const int py = (int)(t % pH);
		t /= pH;
		const int m = (int)(t % Co), b = (int)(t / Co);
		const int hs = py * dH - padH, wst = px * dW - padW;
		const float sc = scale ? scale[m] : 1.0f, bi = bias ? bias[m] : 0.0f;
		const float *src = ws + (long)m * N + (long)b * oH * oW;
		for (int e = l; e < kH * kW; e += LPO) {
			const int yy = hs + e / kW, xx = wst + e % kW;
			if (yy < 0 || yy >= oH || xx < 0 || xx >= oW)
				continue;
			const float *at = src + yy * oW + xx;
			float v = 0;
#pragma unroll 4
			for (int q = 0; q < parts; q++)
				v += at[q * part];
			v = scale ? __builtin_fmaf(v, sc, bi) : v + bi;	/* (one rounding, as in conv_f32_splitk_finish_kernel) */
			if (act)
				v = v > thr ? v : val;
			if (v > mx) {
				mx = v;
				me = e;
			}
		}
	}
#pragma unroll
	for (int off = LPO / 2; off > 0; off >>= 1) {
		const float ov = __shfl_xor(mx, off, 64);
		const int oe = __shfl_xor(me, off, 64);
		if (ov > mx || (ov == mx && oe < me)) {
			mx = ov;
			me = oe;
		}
	}
	if (i < total && l == 0)
		y[i] = mx;
}

/* ------------------------------------------------------------------ */
/* host side                                                           */
/* ------------------------------------------------------------------ */

#define CONV_MPAD 256	/* packed rows are padded to the largest M tile */

static inline int conv_chunk(int dtype) { return dtype == THHIP_F32 ? 8 : dtype == THHIP_U8 ? 32 : 16; }

/* Order of (plane c, tap) along the packed K axis; follows how the input is
 * read (xl: 0 plane-major, 1 channels-last, 2 plane-major read through a
 * four-plane pixel copy), so weights are packed for one of them. */
enum { KORD_PLANE_TAP, KORD_TAP_MAJOR, KORD_CHANNELS_LAST, KORD_PIXELS4, KORD_CL_BLOCKED };

/* Tap-major K order needs whole blocks of KCH*chunk input planes. */
static inline bool conv_tap_major(int Ci, int dtype) { return Ci % (conv_kch(dtype, false) * conv_chunk(dtype)) == 0; }

static inline int conv_korder(int Ci, int dtype, int xl)
{
	if (xl == 1) {
		if (Ci % (conv_chunk(dtype) / 2))
			THError("thhip_conv2d: channels-last input needs Ci %% %d == 0 (Ci = %d)", conv_chunk(dtype) / 2, Ci);
		/* whole K-tiles of planes: K runs (block of planes, tap, plane of the block), so that the taps
		 * of a block, which read the same pixels shifted, follow one another while those pixels are
		 * still in the caches; other plane counts: (tap, plane) */
		return Ci % (conv_kch(dtype, true) * conv_chunk(dtype)) == 0 ? KORD_CL_BLOCKED : KORD_CHANNELS_LAST;
	}
	if (xl == 2) {
		if (dtype != THHIP_U8 || Ci > 4)
			THError("thhip_conv2d: the four-plane pixel path is for uint8 inputs of at most 4 planes (Ci = %d)", Ci);
		return KORD_PIXELS4;
	}
	if (xl)
		THError("thhip_conv2d: unknown input layout %d", xl);
	return conv_tap_major(Ci, dtype) ? KORD_TAP_MAJOR : KORD_PLANE_TAP;
}

/* Number of K chunks (always whole K-tiles). */
static inline int conv_kc(int Ci, int kH, int kW, int dtype, int xl)
{
	const int c = conv_chunk(dtype), kch = conv_kch(dtype, xl != 0);
	const int ord = conv_korder(Ci, dtype, xl);
	if (ord == KORD_TAP_MAJOR)
		return Ci / c * kH * kW;
	/* four-plane pixels: a kernel row is (kW+3)/4 vectors of 4 pixels x 4 planes */
	const long K = ord == KORD_PIXELS4 ? (long)kH * ((kW + 3) / 4) * 16 : (long)Ci * kH * kW;
	const int kc = (int)((K + c - 1) / c);
	return (kc + kch - 1) / kch * kch;
}

/* Position of weight (plane c, tap (kh, kw)) along the packed K axis. */
static inline long conv_kpos(int c, int kh, int kw, int Ci, int kH, int kW, int dtype, int xl)
{
	const int tap = kh * kW + kw, kHW = kH * kW;
	switch (conv_korder(Ci, dtype, xl)) {
	case KORD_CHANNELS_LAST:
		return (long)tap * Ci + c;
	case KORD_CL_BLOCKED: {
		const int cb = conv_kch(dtype, true) * conv_chunk(dtype);
		return ((long)(c / cb) * kHW + tap) * cb + c % cb;
	}
	case KORD_PIXELS4:
		return (((long)kh * ((kW + 3) / 4) + kw / 4) * 4 + kw % 4) * 4 + c;
	case KORD_TAP_MAJOR: {
		const int cb = conv_kch(dtype, false) * conv_chunk(dtype);
		return ((long)(c / cb) * kHW + tap) * cb + c % cb;
	}
	default:
		return (long)c * kHW + tap;
	}
}

/* Element index of (row m, packed K position kp) in the packed buffer. */
static inline size_t conv_pack_index(int m, long kp, int KC, int chunk)
{
	const int vec = chunk / 2;
	const long kc = kp / chunk;
	const int h = (int)(kp % chunk) / vec, e = (int)(kp % vec);
	return ((((size_t)(m >> 5) * KC + kc) * 2 + h) * 32 + (m & 31)) * vec + e;
}

static size_t conv_packed_bytes(int Co, int Ci, int kH, int kW, int dtype, int xl)
{
	size_t mpad = (size_t)(Co + CONV_MPAD - 1) / CONV_MPAD * CONV_MPAD;
	return mpad / 32 * conv_kc(Ci, kH, kW, dtype, xl) * 1024;
}

/* For the kernels in other files that read weights packed by thhip_conv_pack_weight_u8_layout:
 * K chunks of 32 codes per row block, and the bytes of packed codes (the per-row sums follow). */
int thhip_conv_u8_packed_chunks(int Ci, int kH, int kW, int x_layout)
{
	return conv_kc(Ci, kH, kW, THHIP_U8, x_layout);
}

size_t thhip_conv_u8_packed_code_bytes(int Co, int Ci, int kH, int kW, int x_layout)
{
	return conv_packed_bytes(Co, Ci, kH, kW, THHIP_U8, x_layout);
}

/* (for plane-major input the packed size depends on kH * kW only) */
extern "C" size_t thhip_conv_packed_bytes(int Co, int Ci, int kHW, int dtype)
{
	return conv_packed_bytes(Co, Ci, 1, kHW, dtype, 0);
}

static inline unsigned short f32_to_f16_bits(float f)
{
	_Float16 h = (_Float16)f;
	unsigned short u;
	memcpy(&u, &h, 2);
	return u;
}

static inline unsigned short f32_to_bf16_bits(float f)
{
	unsigned u;
	memcpy(&u, &f, 4);
	if ((u & 0x7fffffffu) > 0x7f800000u)
		return (unsigned short)((u >> 16) | 0x40);
	u += 0x7fffu + ((u >> 16) & 1);	/* round to nearest even */
	return (unsigned short)(u >> 16);
}

extern "C" void *thhip_conv_pack_weight_layout(const float *w, int Co, int Ci, int kH, int kW, int dtype, int x_layout)
{
	if (dtype != THHIP_F32 && dtype != THHIP_F16 && dtype != THHIP_BF16)
		THError("thhip_conv_pack_weight: unsupported dtype %d", dtype);
	if (x_layout != 0 && !(x_layout == 1 && dtype != THHIP_F32))
		THError("thhip_conv_pack_weight: input layout %d with dtype %d", x_layout, dtype);
	const int kHW = kH * kW;
	const int chunk = conv_chunk(dtype), KC = conv_kc(Ci, kH, kW, dtype, x_layout);
	const size_t bytes = conv_packed_bytes(Co, Ci, kH, kW, dtype, x_layout);
	unsigned char *host = (unsigned char *)calloc(1, bytes);
	if (!host)
		THError("thhip_conv_pack_weight: out of host memory (%zu bytes)", bytes);
	for (int m = 0; m < Co; m++)
		for (int c = 0; c < Ci; c++)
			for (int tap = 0; tap < kHW; tap++) {
				const size_t idx = conv_pack_index(m, conv_kpos(c, tap / kW, tap % kW, Ci, kH, kW, dtype, x_layout), KC, chunk);
				const float v = w[((size_t)m * Ci + c) * kHW + tap];
				if (dtype == THHIP_F32)
					((float *)host)[idx] = v;
				else if (dtype == THHIP_F16)
					((unsigned short *)host)[idx] = f32_to_f16_bits(v);
				else
					((unsigned short *)host)[idx] = f32_to_bf16_bits(v);
			}
	void *dev = thhip_malloc(bytes);
	thhip_memcpy_h2d(dev, host, bytes);
	free(host);
	return dev;
}

extern "C" void *thhip_conv_pack_weight(const float *w, int Co, int Ci, int kHW, int dtype)
{
	return thhip_conv_pack_weight_layout(w, Co, Ci, 1, kHW, dtype, 0);
}

/* Experiment / tuning override: 0 = choose automatically. */
static int g_force_bm, g_force_bn, g_force_splitk, g_force_wgs, g_force_kch, g_force_mparts, g_force_generic_cl;

/* Channels-last inputs: 1 = always decode the tap per thread (the path for any Ci); 0 = choose automatically. */
extern "C" void thhip_conv_set_generic_cl(int on)
{
	g_force_generic_cl = on;
}

/* Force the number of parts the M tiles are cut into over the XCDs (1, 2, 4 or 8); 0 = choose automatically. */
extern "C" void thhip_conv_set_xcd_parts(int mparts)
{
	if (mparts != 0 && mparts != 1 && mparts != 2 && mparts != 4 && mparts != 8)
		THError("thhip_conv_set_xcd_parts(%d): 0, 1, 2, 4 or 8", mparts);
	g_force_mparts = mparts;
}

/* fp32 and half-type tiles loaded straight into LDS: the most K parts for the
 * tiles an XCD cannot spread evenly over its CUs (1: never cut them). */
static int g_tail_parts = 8;
/* Whether the parts of a cut tile are added by the part that arrives last (conv_xcd_last_arriver) or by a
 * second launch; the first only where the workgroups of a residue of blockIdx.x % 8 were seen on one XCD. */
static int g_tail_inline = 1;
/* launches so far whose cut tiles were added in the kernel / by a second launch (for the tests) */
static long g_tail_launches[2];
extern "C" long thhip_conv_cut_launches(int second_launch)
{
	return g_tail_launches[second_launch != 0];
}

extern "C" int THHipSumPartsInKernel(int on)
{
	const int was = g_tail_inline;
	g_tail_inline = on != 0;
	return was;
}
extern "C" void thhip_conv_set_tail_parts(int parts)
{
	if (parts < 1 || parts > 64)
		THError("thhip_conv_set_tail_parts(%d): 1 .. 64", parts);
	g_tail_parts = parts;
}

/* fp32 only: force K-tiles of 16 (chunks = 2) or 32 (4); 0 = choose automatically. */
extern "C" void thhip_conv_set_ktile(int chunks)
{
	if (chunks != 0 && chunks != 2 && chunks != CONV_KCH_F32)
		THError("thhip_conv_set_ktile(%d): 0, 2 or %d", chunks, CONV_KCH_F32);
	g_force_kch = chunks;
}

extern "C" void thhip_conv_set_tuning(int bm, int bn, int splitk, int wgs_per_cu)
{
	g_force_bm = bm;
	g_force_bn = bn;
	g_force_splitk = splitk;
	g_force_wgs = wgs_per_cu;
}

/* Split-K scratch: partial tiles and arrival counters (grow-only). */
static int *g_ws;
static size_t g_ws_bytes;
static unsigned *g_cnt, *g_cnt_rot;
static size_t g_cnt_n;

/* Points p.cnt at `tiles` arrival counters, zero between launches (the workgroup that draws a tile's last
 * ticket resets it). */
static void conv_counters(ConvParams &p, size_t tiles)
{
	if (tiles > g_cnt_n) {
		hipcheck(hipStreamSynchronize(thhip_stream()));
		thhip_free(g_cnt);
		g_cnt_n = tiles < 4096 ? 4096 : tiles;
		g_cnt = (unsigned *)thhip_malloc(g_cnt_n * sizeof(unsigned));
		thhip_memset(g_cnt, 0, g_cnt_n * sizeof(unsigned));
	}
	if (!g_cnt_rot) {	/* (conv_xcd_report's words, one per launch in flight) */
		g_cnt_rot = (unsigned *)thhip_malloc(64 * sizeof(unsigned));
		thhip_memset(g_cnt_rot, 0, 64 * sizeof(unsigned));
	}
	p.cnt = g_cnt;
}

/* The part workgroups of a launch did not all see the same offset between their place in the grid and the
 * XCD they ran on: from now on the parts are added by the second launch, and the arrival counters, which
 * such a launch may have left anywhere, start from zero again. */
extern "C" void thhip_conv_parts_fault(void)
{
	static int told;
	g_tail_inline = 0;
	if (g_cnt)
		thhip_memset(g_cnt, 0, g_cnt_n * sizeof(unsigned));
	if (g_cnt_rot)
		thhip_memset(g_cnt_rot, 0, 64 * sizeof(unsigned));
	if (!told)
		fprintf(stderr, "thnets HIP engine: the workgroups of a convolution were not handed to the XCDs in one "
			"order; the K parts of cut tiles are added by a second launch from now on\n");
	told = 1;
}

static void conv_scratch(ConvParams &p, size_t tiles, size_t tile_words)
{
	const size_t need = tiles * p.splitk * tile_words * sizeof(int);
	if (need > g_ws_bytes) {
		hipcheck(hipStreamSynchronize(thhip_stream()));
		thhip_free(g_ws);
		g_ws = (int *)thhip_malloc(need);
		g_ws_bytes = need;
	}
	p.ws = g_ws;
	conv_counters(p, tiles);
}

#define CONV_LDS_PER_CU (160 * 1024)

/* Launches kernel K with LDS padded so that at most `wgs` workgroups share a
 * CU (0 = whatever registers and LDS allow).  The hardware hands left-over
 * workgroups to as few CUs as it can fill, so fewer, faster residents per CU
 * shorten the last, partially filled round of a grid. */
template <void (*kernel)(ConvParams)>
static void conv_launch_kernel(ConvParams &p, dim3 grid, int wgs)
{
	static int static_lds = -1, max_wgs;	/* per kernel: one instance of this function each */
	if (static_lds < 0) {
		hipFuncAttributes attr;
		hipcheck(hipFuncGetAttributes(&attr, (const void *)kernel));
		static_lds = (int)attr.sharedSizeBytes;
		hipcheck(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
			CONV_LDS_PER_CU - static_lds));
		hipcheck(hipOccupancyMaxActiveBlocksPerMultiprocessor(&max_wgs, (const void *)kernel, CONV_THREADS, 0));
	}
	int dyn = 0;
	if (wgs > 0 && wgs < max_wgs) {
		dyn = CONV_LDS_PER_CU / (wgs + 1) + 512 - static_lds;
		if (dyn < 0)
			dyn = 0;
	}
	kernel<<<grid, dim3(CONV_THREADS), dyn, thhip_stream()>>>(p);
}

template <int DT, int BM, int BN, int WGM, int WGN, int KCH>
static void conv_launch(ConvParams &p, int splitk, int wgs)
{
	p.tiles_m = (p.Co + BM - 1) / BM;
	p.tiles_n = (p.N + BN - 1) / BN;
	const int nkt = p.KC / KCH;
	if (splitk > nkt)
		splitk = nkt;
	p.splitk = splitk < 1 ? 1 : splitk;
	const size_t tiles = (size_t)p.tiles_m * p.tiles_n;
	if (p.splitk > 1)
		conv_scratch(p, tiles, (size_t)BM * BN);
	/* XCD rectangles: as few parts along M as keep an XCD's weight rows within
	 * about half of its 4 MB L2 */
	const double wbytes = (double)p.Co * p.K * thhip_esize(DT);
	p.mparts = 1;
	while (p.mparts < 8 && p.mparts * 2 <= p.tiles_m && wbytes / p.mparts > 2.5e6)
		p.mparts *= 2;
	if (g_force_mparts)
		p.mparts = g_force_mparts <= p.tiles_m ? g_force_mparts : 1;
	size_t maxcnt = 0;
	for (int x = 0; x < 8; x++) {
		const int mp = x % p.mparts, np = x / p.mparts, nparts = 8 / p.mparts;
		const size_t cnt = (size_t)(p.tiles_m * (mp + 1) / p.mparts - p.tiles_m * mp / p.mparts) *
			(p.tiles_n * (np + 1) / nparts - p.tiles_n * np / nparts);
		if (cnt > maxcnt)
			maxcnt = cnt;
	}
	dim3 grid((unsigned)(8 * maxcnt * p.splitk));
	const bool tap = conv_tap_major(p.Ci, DT);
	/* channels-last: every K-tile inside one tap (and the byte offsets fit an int) */
	const bool uniform = p.x_cl == 1 && p.Ci % (KCH * conv_chunk(DT)) == 0 && p.x_bytes < 0x7fffffffu && !g_force_generic_cl;
	if (p.y_cl && p.Co % 4)
		THError("thhip_conv2d: channels-last output needs Co %% 4 == 0 (Co = %d)", p.Co);
	/* a K-tile depth exists only for the layouts whose packed blocks it divides */
#define CONV_GO(GM, CLO)                                                                                         \
	do {                                                                                                     \
		if constexpr (conv_kch(DT, GM == GM_CHANNELS_LAST || GM == GM_PIXELS4 || GM == GM_CL_UNIFORM) % KCH == 0) \
			return conv_launch_kernel<conv_mfma_kernel<DT, BM, BN, WGM, WGN, GM, CLO, KCH>>(p, grid, wgs); \
		else                                                                                             \
			THError("thhip_conv2d: no K-tile of %d chunks for this layout", KCH);                    \
	} while (0)
	if constexpr (DT == THHIP_U8) {
		/* the uint8 engine keeps its activations channels-last between convolutions */
		if (p.x_cl == 2) {
			if (p.y_cl)
				CONV_GO(GM_PIXELS4, true);
			CONV_GO(GM_PIXELS4, false);
		}
		if (p.x_cl) {
			if (uniform) {
				if (p.y_cl)
					CONV_GO(GM_CL_UNIFORM, true);
				CONV_GO(GM_CL_UNIFORM, false);
			}
			if (p.y_cl)
				CONV_GO(GM_CHANNELS_LAST, true);
			CONV_GO(GM_CHANNELS_LAST, false);
		}
		if (p.y_cl) {
			if (tap)
				CONV_GO(GM_TAP_MAJOR, true);
			CONV_GO(GM_PLANE_TAP, true);
		}
	} else if constexpr (DT == THHIP_F16 || DT == THHIP_BF16) {
		/* the half engines do the same: a 16-byte gather is eight planes of one pixel */
		if (p.x_cl == 1) {
			if (uniform) {
				if (p.y_cl)
					CONV_GO(GM_CL_UNIFORM, true);
				CONV_GO(GM_CL_UNIFORM, false);
			}
			if (p.y_cl)
				CONV_GO(GM_CHANNELS_LAST, true);
			CONV_GO(GM_CHANNELS_LAST, false);
		}
		if (p.x_cl)
			THError("thhip_conv2d: input layout %d is a uint8 feature", p.x_cl);
		if (p.y_cl) {
			if (tap)
				CONV_GO(GM_TAP_MAJOR, true);
			CONV_GO(GM_PLANE_TAP, true);
		}
	} else if (p.x_cl || p.y_cl)
		THError("thhip_conv2d: channels-last tensors are for the uint8 and half types");
	if (tap)
		CONV_GO(GM_TAP_MAJOR, false);
	CONV_GO(GM_PLANE_TAP, false);
#undef CONV_GO
}

/* Points p.ws at scratch of at least that many bytes. */
static void conv_f32_scratch(ConvParams &p, size_t need)
{
	if (need > g_ws_bytes) {
		hipcheck(hipStreamSynchronize(thhip_stream()));
		thhip_free(g_ws);
		g_ws = (int *)thhip_malloc(need);
		g_ws_bytes = need;
	}
	p.ws = g_ws;
}

/* Plans the cut of every XCD's last tiles (conv_tail_parts) for a kernel that
 * holds `resident` workgroups per CU and walks nkt K-tiles per tile: sets
 * p.tail_*, points p.ws at scratch for the parts and returns the largest
 * number of workgroups an XCD needs (its whole tiles plus the parts). */
static size_t conv_tail_plan(ConvParams &p, int resident, int nkt, size_t tile_floats, int need_round, bool inline_ok = false)
{
	static int cus;
	if (!cus) {
		int dev;
		hipcheck(hipGetDevice(&dev));
		hipcheck(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
	}
	p.tail_slots = p.tail_max = p.tail_cap = p.tail_tiles = p.tail_inline = 0;
	p.tail_round = need_round;
	if (p.splitk == 1 && g_tail_parts != 1) {
		p.tail_slots = cus / 8 * (resident < 1 ? 1 : resident);
		p.tail_max = nkt / 8 < g_tail_parts ? nkt / 8 : g_tail_parts;	/* at least eight K-tiles a part (four and two: slower) */
		if (p.tail_max > 8)
			p.tail_max = 8;	/* the finishing kernels hold eight parts in registers */
		if (p.tail_max < 2)
			p.tail_slots = 0;
	}
	size_t maxwgs = 0;
	for (int x = 0; x < 8; x++) {
		const int mp = x % p.mparts, np = x / p.mparts, nparts = 8 / p.mparts;
		const int cnt = (p.tiles_m * (mp + 1) / p.mparts - p.tiles_m * mp / p.mparts) *
			(p.tiles_n * (np + 1) / nparts - p.tiles_n * np / nparts);
		int full;
		const int sx = conv_tail_parts(cnt, p.tail_slots, p.tail_max, p.tail_round, &full);
		if (sx > 1) {
			if ((cnt - full) * sx > p.tail_cap)
				p.tail_cap = (cnt - full) * sx;
			if (cnt - full > p.tail_tiles)
				p.tail_tiles = cnt - full;
		}
		const size_t wgs = (size_t)full + (size_t)(cnt - full) * sx;
		if (wgs > maxwgs)
			maxwgs = wgs;
	}
	if (!p.tail_cap)
		p.tail_slots = 0;
	else {
		conv_f32_scratch(p, (size_t)8 * p.tail_cap * tile_floats * sizeof(float));
		p.tail_inline = inline_ok && g_tail_inline && (thhip_xcd_map() >> 31);
		if (p.tail_inline) {
			static unsigned seq;
			conv_counters(p, (size_t)8 * p.tail_cap);
			p.rot = g_cnt_rot;
			p.rot_slot = (int)(seq & 63);
			p.rot_clear = (int)((seq + 32) & 63);
			seq++;
			p.fault = thhip_fault_flag();
		}
	}
	return maxwgs;
}

/* Whether the kernel that loads straight into LDS can run this layer: a half
 * type or uint8, channels-last input with whole K-tiles (32 halfs, 64 codes)
 * inside a tap, 32-bit byte offsets; uint8 input followed by a K-tile slice of
 * the padding code. */
template <int DT>
static bool conv_wide_ok(const ConvParams &p)
{
	if constexpr (DT == THHIP_F16 || DT == THHIP_BF16)
		return p.x_cl == 1 && p.Ci % 32 == 0 && p.x_bytes < 0x7fffffffu && !g_force_generic_cl &&
			(!p.y_cl || p.Co % 4 == 0);
	if constexpr (DT == THHIP_U8)
		return p.x_cl == 1 && p.Ci % 64 == 0 && p.x_bytes < 0x7fffff00u && !g_force_generic_cl && p.x_tail >= 64 &&
			(!p.y_cl || p.Co % 4 == 0);
	return false;
}

template <int DT, int BM, int BN, int WGM, int WGN, int KCH, int NST, int KG = 1>
static void conv_launch_wide(ConvParams &p)
{
	if constexpr (DT == THHIP_F16 || DT == THHIP_BF16 || (DT == THHIP_U8 && BM <= 128 && BN <= 128 && KCH == 2)) {
		p.tiles_m = (p.Co + BM - 1) / BM;
		p.tiles_n = (p.N + BN - 1) / BN;
		p.splitk = 1;
		if ((size_t)p.tiles_m * BM / 32 * p.KC * 1024 > p.w_bytes)
			THError("thhip_conv2d: packed weights shorter than the tile grid");
		const double wbytes = (double)p.Co * p.K * thhip_esize(DT);
		p.mparts = 1;
		while (p.mparts < 8 && p.mparts * 2 <= p.tiles_m && wbytes / p.mparts > 2.5e6)
			p.mparts *= 2;
		if (g_force_mparts)
			p.mparts = g_force_mparts <= p.tiles_m ? g_force_mparts : 1;
		/* half types: the tiles an XCD cannot spread evenly over its CUs are cut
		 * along K, as in conv_launch_f32_direct (uint8 tiles stay whole: their
		 * column sums run over all of K) */
		int resident = 0;
		if constexpr (DT != THHIP_U8 && KG == 1) {
			static int res_cl, res_pm;
			int &res = p.y_cl ? res_cl : res_pm;
			if (!res) {
				if (p.y_cl)
					hipcheck(hipOccupancyMaxActiveBlocksPerMultiprocessor(&res, conv_wide_kernel<DT, true, BM, BN, WGM, WGN, KCH, NST>, 64 * WGM * WGN, 0));
				else
					hipcheck(hipOccupancyMaxActiveBlocksPerMultiprocessor(&res, conv_wide_kernel<DT, false, BM, BN, WGM, WGN, KCH, NST>, 64 * WGM * WGN, 0));
				if (res < 1)
					res = 1;
			}
			resident = res;
		}
		/* few tiles all cut measured slower here (512->512 @14^2 batch 16, fp16: 31 -> 36 us) */
		/* (tiles shared by two K groups stay whole, like the uint8 ones) */
		const size_t maxcnt = conv_tail_plan(p, resident, DT == THHIP_U8 || KG > 1 ? 0 : p.KC / KCH, (size_t)BM * BN, 1);
		dim3 grid((unsigned)(8 * maxcnt));
		if (p.y_cl)
			conv_wide_kernel<DT, true, BM, BN, WGM, WGN, KCH, NST, KG><<<grid, dim3(64 * WGM * WGN * KG), 0, thhip_stream()>>>(p);
		else
			conv_wide_kernel<DT, false, BM, BN, WGM, WGN, KCH, NST, KG><<<grid, dim3(64 * WGM * WGN * KG), 0, thhip_stream()>>>(p);
		if constexpr (DT != THHIP_U8) {
			if (p.tail_slots) {
				dim3 fgrid((unsigned)(8 * p.tail_tiles * (BM / WGM / 32) * (BN / WGN / 32)));
				if (p.y_cl)
					conv_wide_tail_finish_kernel<DT, true, BM, BN, WGM, WGN><<<fgrid, dim3(64 * WGM * WGN), 0, thhip_stream()>>>(p);
				else
					conv_wide_tail_finish_kernel<DT, false, BM, BN, WGM, WGN><<<fgrid, dim3(64 * WGM * WGN), 0, thhip_stream()>>>(p);
			}
		}
	} else
		THError("thhip_conv2d: no such tile loaded straight into LDS for this type");
}

/* Whether conv_f32_direct_kernel can run this layer: plane-major fp32 on both
 * sides, whole blocks of 32 planes, 32-bit byte offsets. */
static bool conv_f32_direct_ok(const ConvParams &p)
{
	return !p.x_cl && !p.y_cl && p.Ci % 32 == 0 && p.x_bytes < 0x7fffffffu;
}

/* The same kernel with a (plane, tap) of its own for every row of a K-tile: plane-major fp32 layers of any
 * other number of planes (K order (plane, tap)). */
static bool conv_f32_rows_ok(const ConvParams &p)
{
	return !p.x_cl && !p.y_cl && p.Ci % 32 != 0 && p.x_bytes < 0x7fffffffu && p.kHW <= 4096;
}

/* Pairing (thhip_conv_pair_begin / _end): the launch of a layer that conv_f32_direct_kernel<64, 64, 4, 3> runs whole
 * (no K split, no cut tiles, no pooling) is held back, and goes out together with the next launch of that kernel
 * as one grid (conv_f32_direct_pair_kernel); any other convolution call, or _end, sends it out alone. */
static int g_pair_mode;		/* 1: the launch of the next convolution call is held back if it can be */
static int g_pair_have;		/* a launch is held back */
static int g_pair_fresh;	/* ... by the convolution call that is running */
static ConvParams g_pair_p;
static unsigned g_pair_grid;

static void conv_pair_flush(void)
{
	if (!g_pair_have)
		return;
	g_pair_have = 0;
	conv_f32_direct_kernel<64, 64, 4, 3, false><<<dim3(g_pair_grid), dim3(256), 0, thhip_stream()>>>(g_pair_p);
}

extern "C" void thhip_conv_pair_begin(void)
{
	conv_pair_flush();
	g_pair_mode = 1;
}

extern "C" void thhip_conv_pair_end(void)
{
	g_pair_mode = 0;
	conv_pair_flush();
}

template <int BM, int BN, int KCH, int NST, bool ROWS = false>
static void conv_launch_f32_direct(ConvParams &p, int splitk)
{
	p.tiles_m = (p.Co + BM - 1) / BM;
	p.tiles_n = (p.N + BN - 1) / BN;
	const int nkt = p.KC / KCH;
	if (splitk > nkt)
		splitk = nkt;
	p.splitk = splitk < 1 ? 1 : splitk;
	if (p.pk_kH && p.splitk < 2)
		THError("thhip_conv2d: a pooling after the convolution is taken by the kernel that adds the parts of a K split only");
	if (p.splitk > 1)
		conv_f32_scratch(p, (size_t)p.splitk * p.Co * p.N * sizeof(float));
	if ((size_t)p.tiles_m * BM / 32 * p.KC * 1024 > p.w_bytes)
		THError("thhip_conv2d: packed weights shorter than the tile grid");
	const double wbytes = (double)p.Co * p.K * 4;
	p.mparts = 1;
	while (p.mparts < 8 && p.mparts * 2 <= p.tiles_m && wbytes / p.mparts > 2.5e6)
		p.mparts *= 2;
	if (g_force_mparts)
		p.mparts = g_force_mparts <= p.tiles_m ? g_force_mparts : 1;
	/* Without a K split of the whole layer: the tiles an XCD cannot spread evenly
	 * over its CUs are cut along K (conv_tail_parts). */
	static int resident;
	if (!resident) {
		hipcheck(hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, conv_f32_direct_kernel<BM, BN, KCH, NST, ROWS>, 256, 0));
		if (resident < 1)
			resident = 1;
	}
	const size_t maxcnt = conv_tail_plan(p, resident, nkt, (size_t)BM * BN, 0, true);
	const unsigned grid = (unsigned)(8 * maxcnt * p.splitk);
	bool launched = false;
	if constexpr (BM == 64 && BN == 64 && KCH == 4 && NST == 3 && !ROWS) {
		if (g_pair_mode && !g_pair_have && p.splitk == 1 && !p.tail_slots && !p.pk_kH) {
			g_pair_p = p;	/* held back: goes out with the next launch of this kernel */
			g_pair_grid = grid;
			g_pair_have = g_pair_fresh = 1;
			g_pair_mode = 0;
			return;
		}
		if (g_pair_have) {
			g_pair_have = 0;
			conv_f32_direct_pair_kernel<BM, BN, KCH, NST, ROWS><<<dim3(grid + g_pair_grid), dim3(256), 0, thhip_stream()>>>(p, g_pair_p, (int)grid);
			launched = true;
		}
	}
	if (!launched) {
		conv_pair_flush();
		conv_f32_direct_kernel<BM, BN, KCH, NST, ROWS><<<dim3(grid), dim3(256), 0, thhip_stream()>>>(p);
	}
	if (p.pk_kH) {
		/* four lanes per pooled value for windows of up to four values, else sixteen */
		const int lpo = p.pk_kH * p.pk_kW <= 4 ? 4 : 16;
		const long blocks = ((long)p.B * p.Co * p.pk_oH * p.pk_oW * lpo + 255) / 256;
		if (blocks > 0x7fffffffL)
			THError("thhip_conv2d: pooled output too large");
		if (lpo == 4)
			conv_f32_splitk_finish_pool_kernel<4><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>((const float *)p.ws, p.bias, p.scale,
				(float *)p.y, p.splitk, p.B, p.Co, p.N, p.oH, p.oW, p.act, p.thr, p.val,
				p.pk_kH, p.pk_kW, p.pk_dH, p.pk_dW, p.pk_padH, p.pk_padW, p.pk_oH, p.pk_oW);
		else
			conv_f32_splitk_finish_pool_kernel<16><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>((const float *)p.ws, p.bias, p.scale,
				(float *)p.y, p.splitk, p.B, p.Co, p.N, p.oH, p.oW, p.act, p.thr, p.val,
				p.pk_kH, p.pk_kW, p.pk_dH, p.pk_dW, p.pk_padH, p.pk_padW, p.pk_oH, p.pk_oW);
	} else if (p.splitk > 1 && p.N % 4 == 0 && ((size_t)p.y & 15) == 0 && ((size_t)p.res & 15) == 0) {
		long blocks = ((long)p.Co * (p.N / 4) + 255) / 256;
		if (blocks > 4096)
			blocks = 4096;
		conv_f32_splitk_finish4_kernel<<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>((const float *)p.ws, p.bias, p.scale,
			(float *)p.y, p.splitk, p.Co, p.N, p.oHW, p.act, p.thr, p.val, p.res, p.res_mode, p.res_c, p.res_act);
	} else if (p.splitk > 1) {
		long blocks = ((long)p.Co * p.N + 255) / 256;
		if (blocks > 4096)
			blocks = 4096;
		conv_f32_splitk_finish_kernel<<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>((const float *)p.ws, p.bias, p.scale,
			(float *)p.y, p.splitk, p.Co, p.N, p.oHW, p.act, p.thr, p.val, p.res, p.res_mode, p.res_c, p.res_act);
	}
	if (p.tail_slots)
		g_tail_launches[!p.tail_inline]++;
	if (p.tail_slots && !p.tail_inline)
		conv_f32_tail_finish_kernel<BM, BN><<<dim3((unsigned)(8 * p.tail_tiles)), dim3(256), 0, thhip_stream()>>>(p);
}

/* Whether conv_f32_patch_kernel can run this layer, and with which patches: plane-major fp32 on both
 * sides, 3x3 / stride 1 / padding 1, whole blocks of 32 input and 64 output planes, an output of whole
 * 16x4, 8x8 or 4x4 patches.  Returns the patch width (16, 8, 4) or 0. */
static int conv_f32_patch_width(const ConvParams &p)
{
	if (p.x_cl || p.y_cl || p.kH != 3 || p.kW != 3 || p.dH != 1 || p.dW != 1 || p.padH != 1 || p.padW != 1)
		return 0;
	if (p.Ci % 32 || p.Co % 64 || p.x_bytes >= 0x7fffffffu)
		return 0;
	if (p.oW % 16 == 0 && p.oH % 4 == 0)
		return 16;
	if (p.oW % 8 == 0 && p.oH % 8 == 0)
		return 8;
	if (p.oW % 4 == 0 && p.oH % 4 == 0)
		return 4;
	return 0;
}

template <int SW, int SH>
static void conv_launch_f32_patch(ConvParams &p)
{
	typedef ConvPatchGeo<SW, SH> GEO;
	p.tiles_m = p.Co / 64;
	p.tiles_n = (int)(((long)p.B * (p.oH / SH) * (p.oW / SW) + GEO::NP - 1) / GEO::NP);
	p.splitk = 1;
	if ((size_t)p.tiles_m * 2 * p.KC * 1024 > p.w_bytes || p.KC != p.Ci / 8 * 9)
		THError("thhip_conv2d: packed weights do not fit the patch kernel's tile grid");
	const double wbytes = (double)p.Co * p.K * 4;
	p.mparts = 1;
	while (p.mparts < 8 && p.mparts * 2 <= p.tiles_m && wbytes / p.mparts > 2.5e6)
		p.mparts *= 2;
	if (g_force_mparts)
		p.mparts = g_force_mparts <= p.tiles_m ? g_force_mparts : 1;
	/* the tiles an XCD cannot spread evenly over its CUs are cut along K into parts of whole half blocks of
	 * 16 planes (conv_tail_parts; `8 half blocks` K-tiles so that conv_tail_plan allows at most one part a half block) */
	static int resident, static_lds, cus;
	if (!resident) {
		hipcheck(hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, conv_f32_patch_kernel<SW, SH>, 256, 0));
		if (resident < 1)
			resident = 1;
		hipFuncAttributes attr;
		hipcheck(hipFuncGetAttributes(&attr, (const void *)conv_f32_patch_kernel<SW, SH>));
		static_lds = (int)attr.sharedSizeBytes;
		int dev;
		hipcheck(hipGetDevice(&dev));
		hipcheck(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
	}
	/* How many workgroups a CU should hold: with few rounds of tiles, the number that leaves the smallest
	 * part of a round empty after the cut (VGG-16's 28^2 layers at batch 16, 196 tiles an XCD: four a CU
	 * leave a second round half empty with nothing to cut, three make two rounds and four tiles cut in
	 * eight).  Rounds an XCD needs: whole rounds, plus 1 / parts for the cut tiles or 1 if they cannot be cut. */
	int use = resident;
	{
		const int smax = p.Ci / 16 < g_tail_parts ? p.Ci / 16 : g_tail_parts;
		double best = 0;
		for (int r = resident; r >= 3 && r >= resident - 2; r--) {
			double worst = 1.0;
			for (int x = 0; x < 8; x++) {
				const int mp = x % p.mparts, np = x / p.mparts, nparts = 8 / p.mparts;
				const int cnt = (p.tiles_m * (mp + 1) / p.mparts - p.tiles_m * mp / p.mparts) *
					(p.tiles_n * (np + 1) / nparts - p.tiles_n * np / nparts);
				if (!cnt)
					continue;
				int full;
				const int slots = cus / 8 * r;
				const int sx = g_tail_parts != 1 ? conv_tail_parts(cnt, slots, smax > 8 ? 8 : smax, 0, &full) : (full = cnt, 1);
				const double rounds = sx > 1 ? (double)full / slots + 1.0 / sx : (double)((cnt + slots - 1) / slots);
				const double eff = (double)cnt / slots / rounds;
				if (eff < worst)
					worst = eff;
			}
			if (worst > best + 0.02) {	/* (fewer residents only for a clear gain) */
				best = worst;
				use = r;
			}
		}
	}
	int dyn = 0;
	if (use < resident) {	/* LDS nobody uses, so that no more than `use` workgroups fit a CU */
		dyn = CONV_LDS_PER_CU / (use + 1) + 512 - static_lds;
		if (dyn < 0)
			dyn = 0;
	}
	const size_t maxcnt = conv_tail_plan(p, use, p.Ci / 16 * 8, 64 * 64, 0, true);
	conv_f32_patch_kernel<SW, SH><<<dim3((unsigned)(8 * maxcnt)), dim3(256), dyn, thhip_stream()>>>(p);
	if (p.tail_slots)
		g_tail_launches[!p.tail_inline]++;
	if (p.tail_slots && !p.tail_inline)
		conv_f32_patch_tail_finish_kernel<SW, SH><<<dim3((unsigned)(8 * p.tail_tiles)), dim3(256), 0, thhip_stream()>>>(p);
}

/* Whether conv_patch_kernel (conv_half_patch.hip) can run this layer. */
template <int DT>
static bool conv_patch_ok(const ConvParams &p)
{
	return thhip_conv_half_patch_ok(p, DT) && !g_force_generic_cl;
}

/* ... and in its whole-image form (outputs of at most 14 x 14) */
template <int DT>
static bool conv_patch_flat(const ConvParams &p)
{
	return thhip_conv_half_patch_flat_ok(p, DT) && !g_force_generic_cl;
}

/* Half types, convolution followed by a 2x2 pooling: whether the kernel that keeps an input patch in LDS is
 * the one that runs (and pools) the layer; the rule conv_dispatch applies to the layer without the pooling. */
template <int DT>
static bool conv_pool_uses_patch(const ConvParams &p)
{
	if constexpr (DT == THHIP_F16 || DT == THHIP_BF16) {
		const long tpatch = (long)((p.Co + 63) / 64) * p.B * ((p.oW + PATCH_TW - 1) / PATCH_TW) * ((p.oH + PATCH_TH - 1) / PATCH_TH);
		/* 256 and 512 planes: where the 32 x 8 tiles waste at most a third of their pixels (56^2: an eighth;
		 * 28^2: 31 %, and still faster than the tiles loaded straight into LDS: VGG-16 fp16 batch 16
		 * 0.712 -> 0.693 ms, batch 64 2.26 -> 2.22 ms; 14^2 would waste three fifths) */
		const bool fits = (long)((p.oW + PATCH_TW - 1) / PATCH_TW) * ((p.oH + PATCH_TH - 1) / PATCH_TH) * 256 * 100 <= (long)p.oH * p.oW * 132;
		return conv_patch_flat<DT>(p) || (conv_patch_ok<DT>(p) && tpatch >= 128 && (fits || p.Ci <= 128));
	}
	return false;
}

/* fp32 layers of at most 512 tiles of 64 x 64 (a long K, few positions): the K parts their whole K range is cut
 * into -- about 1024 workgroups' worth, at least eight K-tiles each, at most sixteen; 1: no split.  The one rule
 * both conv_dispatch and the entry points that must know the split beforehand (thhip_conv2d_poolk_supported) use. */
static int conv_f32_ksplit(long t64, int nkt)
{
	if (t64 > 512)
		return 1;
	int parts = (int)((1024 + t64 - 1) / t64);
	if (parts > nkt / 8)
		parts = nkt / 8;
	if (parts > 16)
		parts = 16;
	return parts > 1 ? parts : 1;
}

/* conv_f32_patch_kernel takes layers of at least this many 64 x 64 tiles (below, conv_dispatch splits K
 * of the whole layer) */
#define CONV_F32_PATCH_MIN 513
template <int DT>
static void conv_dispatch(ConvParams &p)
{
	/* Tile choice, from sweeps over the VGG / AlexNet / ResNet layer shapes on
	 * a 256-CU part.  With fragments prefetched across K-tiles a 64x64 tile
	 * keeps its four matrix cores nearly as busy as a bigger one, and small
	 * tiles quantise best: the hardware packs the workgroups of a grid's last,
	 * partially filled round onto as few CUs as they fit, so a round costs
	 * (residents per CU) x (tile time) even when nearly empty.
	 *   fp32: layers wide enough to keep every CU supplied (>= 300 tiles of
	 * 128x128) run K-tiles of 16 (small LDS stages, up to six workgroups per
	 * CU; 128x64 tiles from 700 such tiles up for the operand reuse); narrower
	 * layers run 64x64 tiles with K-tiles of 32, which halve the barriers per
	 * MFMA of the few workgroups each CU gets.
	 *   uint8: int8 MFMAs outrun everything else at the sizes of a batch of 64,
	 * so the tile with the most workgroups in flight, 64x64, wins; from 512
	 * tiles of 128x128 up (channels-last layers of larger batches) that tile
	 * is 10-25 % faster for its operand reuse.
	 *   half types: 128x128 (64x128 for <= 64 planes) from 200 such tiles up
	 * for the operand reuse, 64x64 below.
	 * Splitting K measured slower than unsplit 64x64 tiles on every layer that
	 * has tiles for all CUs, so only layers of a few tiles are split (below). */
	/* pooling in the epilogue: the half types' patch kernel where that kernel would run the layer, else the
	 * kernels that load their tiles straight into LDS, which then count positions in blocks of sixteen windows */
	bool pool_patch = false;
	if (p.pool && DT != THHIP_F32)
		pool_patch = conv_pool_uses_patch<DT>(p);
	if (p.pool && !pool_patch)
		p.N = 64 * ((p.npool + 15) / 16);	/* whole pooling windows only: a last odd row or column is not computed */
	const long t128 = (long)((p.Co + 127) / 128) * ((p.N + 127) / 128);
	const long t64 = (long)((p.Co + 63) / 64) * ((p.N + 63) / 64);
	int bm = 64, bn = 64, splitk = 1, wgs = 0, kch = conv_kch(DT, p.x_cl != 0);
	bool direct = false;	/* half types: operands loaded straight into LDS (conv_wide_kernel) */
	bool rows = false;	/* fp32: conv_f32_direct_kernel with a (plane, tap) per K row */
	if (DT == THHIP_F16 || DT == THHIP_BF16) {
		/* tiles of 256 positions (operands straight to LDS) where whole tiles of
		 * 256 planes fill most CUs for a turn: one such tile per CU multiplies
		 * 1.3-1.4x faster than two 128x128 ones (measured with random data:
		 * 256->256 @56^2 batch 16, 196 tiles, 97 -> 68 us; 512->512 @28^2 batch
		 * 32, 133 vs 187 us); with 80..128 of them the 128-plane tile (two
		 * workgroups per CU) wins by 6-15 %; with fewer, and for layers of 128
		 * planes or less, the smaller tiles below do. */
		const long t256 = (long)((p.Co + 255) / 256) * ((p.N + 255) / 256);
		/* 64 or 128 input planes, 3x3: the taps come from a patch in LDS (measured
		 * with random data, batch 16 / 64: 64->64 @224^2 129 -> 101 / 560 -> 414 us,
		 * 64->128 @112^2 55 -> 49 / 226 -> 209 us, 64->64 @56^2 12.9 -> 11.3 /
		 * 36 -> 29 us, 128->128 @112^2 90 -> 76 / 382 -> 361 us, 128->256 @56^2
		 * 54 -> 42 / 183 -> 157 us (the 256x256 tile: 41 / 171 us); 128 rows per
		 * workgroup measured slower than 64).  With its patches in two buffers the
		 * same kernel also takes 256 and 512 input planes where its 32 x 8 tiles fit
		 * the output (VGG-16's 56^2 layers; with them and 128->256 @56^2, which the
		 * 256x256 tile used to take: fp16 batch 16 0.691 -> 0.676 ms, batch 64
		 * 2.18 -> 2.14 ms in one session). */
		const bool wide256 = conv_wide_ok<DT>(p) && p.Co % 256 == 0 && t256 > 128;
		if (conv_pool_uses_patch<DT>(p))	/* (the rule is there: the fused pooling asks the same question) */
			bm = 64, bn = 1;
		else if (conv_wide_ok<DT>(p)) {
			/* operands straight into LDS, the tile by how many there are (random
			 * data; us for the register-staged kernel's best tile -> this one):
			 * 256x256 from 129 whole tiles (256->256 @56^2 batch 16 97 -> 68);
			 * below that 128x128 from 300 tiles of that size (512->512 @28^2 batch
			 * 16 96 -> 73, where 128x256 takes 86), 128x64 from 150 (256->256
			 * @14^2 batch 64 37 -> 25), else 64x64 (512->512 @14^2 batch 16 41 ->
			 * 31, @7^2 48 -> 24, 192->384 @13^2 17 -> 13; also at batch 1, where
			 * the other kernel splits K: 192->384 @13^2 22 -> 11, 512->512 @14^2
			 * 31 -> 24); 64-row tiles when 128 rows would leave a partly empty tile */
			direct = true;
			if (wide256)
				bm = bn = 256;
			else if (p.Co % 128 == 0 && t128 >= 300)
				bm = bn = 128;
			else if (p.Co % 128 == 0 && t128 >= 150)
				bm = 128;
			else if (t128 >= 150)
				bn = 128;
		} else if (p.Co <= 64)
			bn = 128;
		else if (t128 >= 200)
			bm = bn = 128;
	} else if (DT == THHIP_U8) {
		if (conv_wide_ok<DT>(p)) {	/* as for the half types */
			direct = true;
			if (p.Co % 128 == 0 && t128 >= 300)
				bm = bn = 128;
			else if (p.Co % 128 == 0 && t128 >= 150)
				bm = 128;
			else if (t128 >= 150)
				bn = 128;
		} else if (p.x_cl == 1 && t128 >= 512)
			bm = bn = 128;
	} else if (DT == THHIP_F32 && conv_f32_patch_width(p) && t64 >= CONV_F32_PATCH_MIN && !g_force_kch && !g_force_bm && !g_force_bn) {
		/* 3x3 layers of many whole patches: the taps from a patch in LDS (conv_f32_patch_kernel) */
		bn = 1;
	} else if (DT == THHIP_F32 && conv_f32_direct_ok(p) && !g_force_kch) {
		/* planes in blocks of 32: operands straight into LDS, 64x64 tiles
		 * (measured 2-7 % over the register-staged kernel on every VGG layer,
		 * random data; 64x128 and 128x128 tiles are slower).  Layers of many
		 * tiles take K-tiles of 16 (1-3 %), and 128x64 tiles when that is one
		 * tile of planes (128->128 @112^2 batch 16: 584 -> 569 us). */
		direct = true;
		if (t64 >= 2000) {
			kch = 2;
			if (p.Co == 128)
				bm = 128;
		} else if (t64 <= 512) {
			/* Few tiles of a long K (a 32x32 MFMA tile over K = 4608 is most of a
			 * SIMD's fair share of a 392-tile layer): split K, about 1024
			 * workgroups, at least eight K-tiles each; the parts go to scratch and
			 * a small kernel adds them in order.  Measured: 512->512 @14^2 batch 16
			 * 181 -> 161 us (3 parts), @7^2 batch 32 108 -> 96 us; AlexNet batch 1,
			 * against the other kernel's in-kernel split: conv2 32 -> 15, conv3
			 * 25 -> 14, conv4 27 -> 16, conv5 31 -> 15 us. */
			splitk = conv_f32_ksplit(t64, p.KC / kch);
		}
	} else if (DT == THHIP_F32 && conv_f32_rows_ok(p) && (p.dW == 1 || t64 <= 512) && !g_force_kch && !g_force_bm && !g_force_bn) {
		/* any other number of planes (image layers with larger kernels): the same kernel with a tap of
		 * its own per K row, K-tiles of 16.  Not for strided layers of many tiles: a wave-wide load
		 * then spans twice the cache lines, and ResNet-18's 7x7 / stride 2 image layer at batch 32 took
		 * 117 us against the register-staged kernel's 108 (AlexNet's 11x11 / stride 4 one at batch 1,
		 * a few tiles with a K split: 17 -> 11 us). */
		direct = rows = true;
		kch = 2;
		if (t64 <= 512)
			splitk = conv_f32_ksplit(t64, p.KC / kch);
	} else if (DT == THHIP_F32 && t128 >= 300) {
		kch = 2;
		if (p.Co > 64 && t128 >= 700)
			bm = 128;
		else if (p.Co > 64)
			wgs = 4;
	}
	/* A layer of a few tiles (batch 1) leaves most CUs idle and every workgroup
	 * alone with the whole K loop, which then sets the layer's time: there the
	 * deterministic K split pays, one part per sixteen K-tiles up to eight parts
	 * (AlexNet batch 1: conv3 42 -> 23 us, conv4 81 -> 27 us, conv5 55 -> 29 us;
	 * more parts lose again to the serial sum of the last arriver). */
	if (!direct && bm == 64 && bn == 64 && t64 <= 128) {	/* 65..128 tiles: two parts at most */
		const int nkt = p.KC / kch;
		int parts = (nkt + 8) / 16;
		if (parts > 256 / t64)
			parts = (int)(256 / t64);
		if (parts > 8)
			parts = 8;
		if (parts > 1)
			splitk = parts;
	}
	if (g_force_bm || g_force_bn)
		direct = g_force_splitk == 9;
	if (g_force_bm)
		bm = g_force_bm;
	if (g_force_bn)
		bn = g_force_bn;
	if (g_force_splitk && g_force_splitk != 9)
		splitk = g_force_splitk;
	if (g_force_wgs)
		wgs = g_force_wgs;
	if (DT == THHIP_F32 && g_force_kch)
		kch = g_force_kch;
	if (pool_patch)
		bm = 64, bn = 1;
	if (p.pk_kH && !(DT == THHIP_F32 && direct && bn != 1 && splitk > 1 && !g_force_bm))
		THError("thhip_conv2d: a pooling after the convolution is taken by the kernel that adds the parts of a K split only "
			"(see thhip_conv2d_poolk_supported)");
	if (p.pool && !pool_patch && DT != THHIP_F32 && (!direct || bn == 1))
		THError("thhip_conv2d: half-type pooling in the epilogue needs the patch kernel or the tiles loaded straight into LDS");
	if constexpr (DT == THHIP_F32) {
		if (bn == 1) {	/* (64, 1): the fp32 patch kernel */
			const int tw = conv_f32_patch_width(p);
			if (!tw)
				THError("thhip_conv2d: the fp32 patch kernel needs plane-major tensors, 3x3 / stride 1 / padding 1, "
					"Ci %% 32 == 0, Co %% 64 == 0 and an output of whole 16x4, 8x8 or 4x4 patches");
			if (tw == 16)
				return conv_launch_f32_patch<16, 4>(p);
			if (tw == 8)
				return conv_launch_f32_patch<8, 8>(p);
			return conv_launch_f32_patch<4, 4>(p);
		}
	}
	if (p.res_mode && (DT != THHIP_F32 || !direct || p.pool))
		THError("thhip_conv2d: a second tensor is combined only by the fp32 tiles loaded straight into LDS, without pooling");
	if (p.pool && DT == THHIP_F32 && (!direct || splitk != 1))
		THError("thhip_conv2d: fp32 pooling in the epilogue needs the tiles loaded straight into LDS, without a K split");
	if (bn == 1) {	/* (64, 1): the patch kernel */
		if (!conv_patch_ok<DT>(p))
			THError("thhip_conv2d: the patch kernel needs a half type, channels-last input of 64, 128, 256 or 512 planes, 3x3, stride 1");
		/* a whole image of at most 14 x 14 per workgroup: 64 planes where that makes 256 workgroups, else 32
		 * (the tuning hook's last argument: 3 forces 32, 4 forces 64, 5 the 32 x 8 tiles) */
		if (conv_patch_flat<DT>(p) && g_force_wgs != 5) {
			const bool small = g_force_wgs == 3 || (g_force_wgs != 4 && (long)p.B * (p.Co / 64) < 256);
			return thhip_conv_half_patch_launch(p, DT, small ? 32 : 64, 1);
		}
		return thhip_conv_half_patch_launch(p, DT, 64, 0);
	}
	if constexpr (DT == THHIP_F32) {
		if (direct && rows)
			return conv_launch_f32_direct<64, 64, 2, 3, true>(p, splitk);
		if (direct) {
			if (!conv_f32_direct_ok(p))
				THError("thhip_conv2d: fp32 tiles loaded straight into LDS need plane-major tensors and Ci %% 32 == 0");
			/* K-tiles of 16 or 32 values (the tuning hook's last argument, 2, asks for 16) */
			const bool k16 = g_force_bm ? g_force_wgs % 10 == 2 : kch == 2;
			/* (forced tuning: the last argument / 10 is the K split) */
			const int dsplit = g_force_bm ? g_force_wgs / 10 : splitk;
			if (bm == 64 && bn == 64 && k16)
				return conv_launch_f32_direct<64, 64, 2, 3>(p, dsplit);
			if (bm == 64 && bn == 64)
				return conv_launch_f32_direct<64, 64, 4, 3>(p, dsplit);
			if (bm == 128 && bn == 64 && k16)
				return conv_launch_f32_direct<128, 64, 2, 3>(p, dsplit);
			if (bm == 128 && bn == 64)
				return conv_launch_f32_direct<128, 64, 4, 3>(p, dsplit);
			THError("thhip_conv2d: no %dx%d tile", bm, bn);
		}
	}
	/* tiles whose operands are loaded straight into LDS (the tuning hook asks for
	 * them with 9 as its split-K argument, or with a 256-position tile) */
	if (direct || bn >= 256) {
		if (!conv_wide_ok<DT>(p))
			THError("thhip_conv2d: tiles loaded straight into LDS need channels-last input with whole K-tiles of planes (and, uint8, a tail of padding codes)");
		if (bm == 256 && bn == 256)
			return conv_launch_wide<DT, 256, 256, 2, 4, 2, 4>(p);
		if (bm == 128 && bn == 256)
			return conv_launch_wide<DT, 128, 256, 1, 4, 2, 3>(p);
		if (bm == 128 && bn == 128)
			return conv_launch_wide<DT, 128, 128, 2, 2, 2, 4>(p);
		if (bm == 128 && bn == 64)
			return conv_launch_wide<DT, 128, 64, 2, 2, 2, 4>(p);
		if (bm == 64 && bn == 128)
			return conv_launch_wide<DT, 64, 128, 2, 2, 2, 4>(p);
		if (bm == 64 && bn == 64) {
			/* Few tiles and a long K: one or two workgroups per CU with little to overlap a K step's
			 * latency with.  Two K groups per workgroup then walk half the K-tiles each: 512 -> 512 @14^2
			 * batch 16, fp16, 33 -> 31 us; ResNet-18 fp16 batch 32 0.679 -> 0.662 ms (the tuning hook's
			 * last argument forces one group, 1, or two, 2). */
			const bool two = g_force_wgs ? g_force_wgs == 2 : t64 <= 512 && p.KC / 2 >= 32;
			if (two)
				return conv_launch_wide<DT, 64, 64, 2, 2, 2, 4, 2>(p);
			return conv_launch_wide<DT, 64, 64, 2, 2, 2, 4>(p);
		}
		THError("thhip_conv2d: no %dx%d tile", bm, bn);
	}
#define CONV_TILES(KCH)                                                      \
	do {                                                                 \
		if (bm == 128 && bn == 128)                                  \
			conv_launch<DT, 128, 128, 2, 2, KCH>(p, splitk, wgs); \
		else if (bm == 128 && bn == 64)                              \
			conv_launch<DT, 128, 64, 2, 2, KCH>(p, splitk, wgs);  \
		else if (bm == 64 && bn == 128)                              \
			conv_launch<DT, 64, 128, 2, 2, KCH>(p, splitk, wgs);  \
		else if (bm == 64 && bn == 64)                               \
			conv_launch<DT, 64, 64, 2, 2, KCH>(p, splitk, wgs);   \
		else                                                         \
			THError("thhip_conv2d: no %dx%d tile", bm, bn);      \
	} while (0)
	if constexpr (DT == THHIP_F32) {
		if (kch == 2)
			CONV_TILES(2);
		else
			CONV_TILES(CONV_KCH_F32);
	} else {
		/* one depth per dtype and input layout */
		if (p.x_cl)
			CONV_TILES(conv_kch(DT, true));
		else
			CONV_TILES(conv_kch(DT, false));
	}
#undef CONV_TILES
}

struct ConvU8Args {
	const int *addend;
	int zero, a_off, b_off, c_off, c_mult, c_shift, ithr, ival;
	int x_cl;	/* 0 plane-major, 1 channels-last, 2 plane-major read through a four-plane pixel copy */
	int y_cl;
	int x_tail;	/* bytes of the padding code after x */
};

/* Codes [B][C][HW], C <= 4 -> [B][HW][4] with code 128 (0 once re-centred) in
 * the planes that do not exist: one word per pixel, so that four neighbouring
 * pixels of a kernel row are one 16-byte operand vector. */
__global__ void conv_pixels4_kernel(const unsigned char *x, unsigned *y, int C, long HW, long total)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const long b = i / HW, r = i - b * HW;
		const unsigned char *src = x + b * C * HW + r;
		unsigned w = 0x80808080u;
		for (int c = 0; c < C; c++)
			w = (w & ~(255u << (8 * c))) | ((unsigned)src[c * HW] << (8 * c));
		y[i] = w;
	}
}

/* The same, four pixels per thread (HW % 4 == 0): one word per plane in, 16 bytes out. */
__global__ void conv_pixels4x4_kernel(const unsigned *x, uintx4 *y, int C, long HW4, long total4)
{
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long step = (long)gridDim.x * blockDim.x;
	for (; i < total4; i += step) {
		const long b = i / HW4, r = i - b * HW4;
		const unsigned *src = x + b * C * HW4 + r;
		unsigned pl[4] = { 0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u };
		for (int c = 0; c < C; c++)
			pl[c] = src[c * HW4];
		uintx4 o;
#pragma unroll
		for (int e = 0; e < 4; e++)	/* pixel e: byte e of every plane word */
			o[e] = ((pl[0] >> (8 * e)) & 255u) | (((pl[1] >> (8 * e)) & 255u) << 8) |
				(((pl[2] >> (8 * e)) & 255u) << 16) | (((pl[3] >> (8 * e)) & 255u) << 24);
		y[i] = o;
	}
}

static unsigned char *g_c4;
static size_t g_c4_bytes;

static unsigned char *conv_pixels4_scratch(size_t bytes)
{
	if (bytes > g_c4_bytes) {
		hipcheck(hipStreamSynchronize(thhip_stream()));
		thhip_free(g_c4);
		g_c4 = (unsigned char *)thhip_malloc(bytes);
		g_c4_bytes = bytes;
	}
	return g_c4;
}

/* A max pooling that follows the convolution, for conv_run: window, stride, padding, pooled plane. */
struct ConvPoolK { int kH, kW, dH, dW, padH, padW, oH, oW; };

struct ConvResidual {
	const float *res;
	int mode, act;
	float c;
};

/* the network's image layer (3 planes -> 64, 3x3 / stride 1 / padding 1) in front of the convolution */
struct ConvImageFront {
	const void *img, *wfront;
	const float *scale, *shift;
	int act;
	float thr, val;
};

static void conv_run(const void *x, const void *wpacked, const float *scale, const float *bias, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype, const ConvU8Args *u8, int f_x_layout = 0, int f_y_cl = 0, int f_pool2 = 0,
	const ConvResidual *f_res = 0, const ConvPoolK *f_pk = 0, const ConvImageFront *f_front = 0)
{
	if (B < 1 || Ci < 1 || Co < 1 || kH < 1 || kW < 1 || dH < 1 || dW < 1 || padH < 0 || padW < 0)
		THError("thhip_conv2d: bad geometry");
	const int oW = (W + 2 * padW - kW) / dW + 1;	/* SpatialConvolutionMM.c:159-160 */
	const int oH = (H + 2 * padH - kH) / dH + 1;
	if (oW < 1 || oH < 1)
		THError("Given input size: (%dx%dx%d). Calculated output size: (%dx%dx%d). Output size is too small",
			Ci, H, W, Co, oH, oW);
	const int esize = thhip_esize(dtype);
	const long K = (long)Ci * kH * kW;
	if (K * kH * kW >= (1L << 32) || K > (1 << 30))
		THError("thhip_conv2d: K = %ld too large", K);
	/* 32-bit offsets inside the kernel: run the batch in slices whose input
	 * and output stay below 2^31 bytes. */
	const int xl = u8 ? u8->x_cl : f_x_layout;
	const long in_img = (long)Ci * H * W;
	const long out_img = f_pk ? (long)Co * f_pk->oH * f_pk->oW : f_pool2 ? (long)Co * (oH / 2) * (oW / 2) : (long)Co * oH * oW;
	const long in_eff = xl == 2 ? 4L * H * W : in_img;	/* bytes the kernel addresses per image */
	long bmax = ((1L << 31) - 64) / (esize * (in_eff > out_img ? in_eff : out_img));
	if (bmax < 1)
		THError("thhip_conv2d: one image exceeds 2 GiB");
	if ((long)oH * oW * bmax > (1L << 30))
		bmax = (1L << 30) / ((long)oH * oW);
	/* a window of the batch (hip_rt.hip: thhip_batch_window): the images of the window only */
	int win0 = 0;
	int winn = thhip_batch_window_get(&win0);
	if (winn && (f_pk || f_front || u8)) {	/* (these take the batch in one piece: the caller hears of it) */
		thhip_batch_window_violate();
		winn = 0;
	}
	const int bfirst = winn ? (win0 < B ? win0 : B) : 0, bend = winn ? (win0 + winn < B ? win0 + winn : B) : B;
	thhip_batch_window_scope(1);
	for (int b0 = bfirst; b0 < bend; b0 += (int)bmax) {
		const int bn = bend - b0 < bmax ? bend - b0 : (int)bmax;
		ConvParams p;
		memset(&p, 0, sizeof(p));
		p.x = (const char *)x + (size_t)b0 * in_img * esize;
		p.y = (char *)y + (size_t)b0 * out_img * esize;
		p.wp = wpacked;
		p.bias = bias;
		p.scale = scale;
		p.B = bn; p.Ci = Ci; p.H = H; p.W = W; p.Co = Co; p.kH = kH; p.kW = kW;
		p.dH = dH; p.dW = dW; p.padH = padH; p.padW = padW; p.oH = oH; p.oW = oW;
		p.K = (int)K;
		p.KC = conv_kc(Ci, kH, kW, dtype, xl);
		p.N = bn * oH * oW;
		p.oHW = oH * oW;
		if (xl == 1 && conv_korder(Ci, dtype, xl) == KORD_CL_BLOCKED)
			for (int cb = conv_kch(dtype, true) * conv_chunk(dtype); (1 << p.cl_shift) < cb; )
				p.cl_shift++;
		p.pW = oW / 2;
		p.pHW = (oH / 2) * (oW / 2);
		p.npool = bn * p.pHW;
		p.HW = H * W;
		p.kHW = kH * kW;
		p.magic_khw = (unsigned)conv_magic(kH * kW);
		p.mhi_khw = (unsigned)(conv_magic(kH * kW) >> 32);
		p.magic_kw = (unsigned)conv_magic(kW);
		p.mhi_kw = (unsigned)(conv_magic(kW) >> 32);
		p.magic_ci = (unsigned)conv_magic(Ci);
		p.mhi_ci = (unsigned)(conv_magic(Ci) >> 32);
		p.act = act; p.thr = thr; p.val = val;
		p.x_bytes = (unsigned)(bn * in_img * esize);
		p.w_bytes = (unsigned)conv_packed_bytes(Co, Ci, kH, kW, dtype, xl);
		if (u8) {
			p.rowsum = (const int *)((const char *)wpacked + conv_packed_bytes(Co, Ci, kH, kW, THHIP_U8, xl));
			p.addend = u8->addend;
			p.zero = u8->zero;
			p.offA = 128 + u8->a_off;
			p.offB = 128 + u8->b_off;
			p.c_off = u8->c_off; p.c_mult = u8->c_mult; p.c_shift = u8->c_shift;
			p.ithr = u8->ithr; p.ival = u8->ival;
			p.x_cl = xl; p.y_cl = u8->y_cl;
			p.x_tail = b0 + bn == B ? (unsigned)u8->x_tail : 0;	/* (a batch slice that ends inside x has no tail) */
			if (xl == 2) {
				/* the kernel reads a [B][H][W][4] copy with slack on both sides */
				const long pixels = (long)bn * H * W;
				const size_t bytes = (size_t)pixels * 4 + 2 * CONV_C4_SLACK;
				unsigned char *c4 = conv_pixels4_scratch(bytes);
				{
					ThhipLaunchScope scope(THHIP_FAM_OTHER, (double)bn * in_img + 4.0 * pixels);
					const bool quads = ((long)H * W) % 4 == 0 && ((size_t)p.x & 3) == 0;
					const long work = quads ? pixels / 4 : pixels;
					long blocks = (work + 255) / 256;
					if (blocks > 65536 * 16)
						blocks = 65536 * 16;
					if (quads)
						conv_pixels4x4_kernel<<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(
							(const unsigned *)p.x, (uintx4 *)(c4 + CONV_C4_SLACK), Ci, (long)H * W / 4, work);
					else
						conv_pixels4_kernel<<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(
							(const unsigned char *)p.x, (unsigned *)(c4 + CONV_C4_SLACK), Ci, (long)H * W, pixels);
				}
				p.x = c4;
				p.x_bytes = (unsigned)bytes;
				p.kwv = (kW + 3) / 4;
				p.magic_kw = (unsigned)conv_magic(p.kwv);
				p.mhi_kw = (unsigned)(conv_magic(p.kwv) >> 32);
				unsigned fill = 0x80808080u;
				for (int c = 0; c < Ci; c++)
					fill = (fill & ~(255u << (8 * c))) | ((unsigned)p.zero << (8 * c));
				p.c4_fill = fill;
			}
			ThhipLaunchScope scope(THHIP_FAM_CONV_I8, 2.0 * Co * (double)K * p.N);
			conv_dispatch<THHIP_U8>(p);
		} else {
			p.x_cl = xl;
			p.y_cl = f_y_cl;
			p.pool = f_pool2;
			if (f_pk) {
				if (bn != B)
					THError("thhip_conv2d: a pooling after the convolution needs the batch in one slice");
				p.pk_kH = f_pk->kH; p.pk_kW = f_pk->kW; p.pk_dH = f_pk->dH; p.pk_dW = f_pk->dW;
				p.pk_padH = f_pk->padH; p.pk_padW = f_pk->padW; p.pk_oH = f_pk->oH; p.pk_oW = f_pk->oW;
			}
			if (f_res) {
				p.res = f_res->res + (size_t)b0 * out_img;
				p.res_mode = f_res->mode;
				p.res_c = f_res->c;
				p.res_act = f_res->act;
			}
			if (f_front) {
				/* (x is not read: the kernel computes its input patches from the image) */
				if (bn != B)
					THError("thhip_conv2d_image_pair: the batch must fit one slice");
				p.x = 0;
				p.x_bytes = 0;
				p.img = f_front->img;
				p.img_bytes = (unsigned)((size_t)bn * 3 * H * W * esize);
				p.wstem = f_front->wfront;
				p.sscale = f_front->scale;
				p.sbias = f_front->shift;
				p.sact = f_front->act;
				p.sthr = f_front->thr;
				p.sval = f_front->val;
				ThhipLaunchScope scope(THHIP_FAM_CONV, 2.0 * Co * (double)K * p.N + 2.0 * 64 * 27 * p.N);
				thhip_conv_half_patch_launch(p, dtype, 64, 0);
				continue;
			}
			ThhipLaunchScope scope(THHIP_FAM_CONV, 2.0 * Co * (double)K * p.N);
			/* a 3x3 image layer: whole rows from a patch in LDS (conv_stem.hip), unless a test forces a tile */
			if (!f_pool2 && !f_res && !f_pk && xl == 0 && !g_force_bm &&
			    thhip_conv_stem_ok(bn, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, dtype, f_y_cl))
				thhip_conv_stem(p.x, wpacked, p.KC, scale, bias, p.y, bn, H, W, Co, act, thr, val, dtype, f_y_cl);
			else
				THHIP_DISPATCH_FLOAT(dtype, conv_dispatch<DT>(p));
		}
		/* a launch held back by an earlier call that this call did not take along goes out now */
		if (g_pair_have && !g_pair_fresh)
			conv_pair_flush();
		g_pair_fresh = 0;
		g_pair_mode = 0;	/* (only the call right after thhip_conv_pair_begin may be held back) */
	}
	thhip_batch_window_scope(0);
}

extern "C" void thhip_conv2d_affine(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype)
{
	if (dtype != THHIP_F32 && dtype != THHIP_F16 && dtype != THHIP_BF16)
		THError("thhip_conv2d: unsupported dtype %d", dtype);
	conv_run(x, wpacked, scale, shift, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, thr, val, dtype, 0);
}

extern "C" void thhip_conv2d_layout(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype, int x_layout, int y_channels_last)
{
	if (dtype != THHIP_F16 && dtype != THHIP_BF16 && (x_layout || y_channels_last))
		THError("thhip_conv2d_layout: channels-last tensors need a half dtype (got %d)", dtype);
	if (dtype != THHIP_F32 && dtype != THHIP_F16 && dtype != THHIP_BF16)
		THError("thhip_conv2d: unsupported dtype %d", dtype);
	conv_run(x, wpacked, scale, shift, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, thr, val, dtype, 0,
		x_layout, y_channels_last != 0);
}

/* Whether thhip_conv2d_layout_pool2 takes this layer (and is the kernel the
 * layer would run on anyway): half type, channels-last input in blocks of 32
 * planes; or fp32, plane-major, planes in blocks of 32 and enough tiles that K
 * is not split. */
extern "C" int thhip_conv2d_pool2_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int dtype, int x_layout, int y_channels_last)
{
	if (dtype == THHIP_F32) {
		/* conv_f32_direct_kernel without a K split (conv_dispatch's choice for more than 512 tiles of 64 x 64) */
		if (x_layout || y_channels_last || Ci % 32 || kH < 1 || kW < 1 || dH < 1 || dW < 1 || padH < 0 || padW < 0)
			return 0;
		const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
		if (oW < 2 || oH < 2)
			return 0;
		if ((double)B * Ci * H * W * 4 >= 2147483000.0 || (double)B * Co * oH * oW * 4 >= 2147483000.0)
			return 0;	/* (the batch would be cut into slices) */
		const long t64 = (long)((Co + 63) / 64) * (((long)B * (oH / 2) * (oW / 2) + 15) / 16);
		return t64 > 512 && !g_force_kch && !g_force_bm && !g_force_bn && !g_force_splitk;
	}
	if (dtype != THHIP_F16 && dtype != THHIP_BF16)
		return 0;
	/* half types: channels-last input in whole K-tiles of planes (the patch kernel for 3x3 layers of 64 or 128
	 * planes with enough tiles, else the tiles loaded straight into LDS: conv_dispatch decides) */
	if (x_layout != 1 || Ci % 32 || kH < 1 || kW < 1 || dH < 1 || dW < 1 || padH < 0 || padW < 0)
		return 0;
	if (y_channels_last && Co % 4)
		return 0;
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	if (oW < 2 || oH < 2)
		return 0;
	if ((double)B * Ci * H * W * 2 >= 2147483000.0 || (double)B * Co * oH * oW * 2 >= 2147483000.0)
		return 0;	/* (the batch would be cut into slices) */
	return !g_force_generic_cl && !g_force_bm && !g_force_bn;
}

/* thhip_conv2d_layout followed by a 2x2 / stride 2 max pooling without padding
 * (floor mode), in one kernel: y is [B][Co][oH/2][oW/2] (or channels-last).  For
 * layers thhip_conv2d_pool2_supported accepts.  Replaces the module sequence
 * SpatialConvolutionMM -> Threshold -> SpatialMaxPooling
 * (modules/SpatialMaxPooling.c:6-98) for those layers. */
extern "C" void thhip_conv2d_layout_pool2(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype, int x_layout, int y_channels_last)
{
	if (!thhip_conv2d_pool2_supported(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, dtype, x_layout, y_channels_last))
		THError("thhip_conv2d_layout_pool2: layer not supported (see thhip_conv2d_pool2_supported)");
	conv_run(x, wpacked, scale, shift, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, thr, val, dtype, 0,
		x_layout, y_channels_last != 0, 1);
}

/* Whether thhip_conv2d_image_pool takes the layer: fp32, plane-major, at most four input planes, whole
 * blocks of 64 output planes, strides up to 4, followed by a 3x3 / stride 2 max pooling (padding 0 or 1,
 * floor mode) whose output rows are whole groups of 14 positions (ResNet's 7x7 / stride 2 stem and its
 * pooling at 224 x 224). */
extern "C" int thhip_conv2d_image_pool_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode, int dtype, int x_layout)
{
	if (x_layout || g_force_bm || g_force_bn || g_force_splitk)
		return 0;
	return thhip_conv_image_pool_f32_ok(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pkH, pkW, pdH, pdW, ppadH, ppadW,
		ceil_mode, dtype);
}

/* SpatialConvolutionMM (-> folded batch norm: per-plane factor before the shift) -> Threshold ->
 * SpatialMaxPooling(3, 3, 2, 2, ppad, ppad) in one kernel for the layers
 * thhip_conv2d_image_pool_supported accepts (modules/SpatialConvolutionMM.c:126-225,
 * modules/SpatialMaxPooling.c:168-247): the convolution's output is never written.  y is
 * [B][Co][pH][pW]; wpacked as thhip_conv_pack_weight_layout(..., x_layout 0) packs it. */
extern "C" void thhip_conv2d_image_pool(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int ppad,
	int act, float thr, float val, int dtype)
{
	if (!thhip_conv2d_image_pool_supported(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, 3, 3, 2, 2, ppad, ppad, 0, dtype, 0))
		THError("thhip_conv2d_image_pool: layer not supported (see thhip_conv2d_image_pool_supported)");
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	ThhipLaunchScope scope(THHIP_FAM_CONV, 2.0 * Co * (double)Ci * kH * kW * B * oH * oW);
	thhip_conv_image_pool_f32((const float *)x, (const float *)wpacked, conv_kc(Ci, kH, kW, THHIP_F32, 0), scale, shift,
		(float *)y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, ppad, act, thr, val);
}

/* Whether thhip_conv2d_residual takes this layer: fp32, plane-major tensors, planes in blocks of 32 (the
 * kernel that loads its tiles straight into LDS), the batch in one slice. */
/* The image layer's weights [64][3][3][3] in the order the kernel of thhip_conv2d_image_pair multiplies them:
 * [32-row block][chunk of 16][lane half h][row][8 values], value e of chunk s being tap j = 8 s + e of the
 * eighteen of planes 2 h and 2 h + 1 (plane j / 9, kernel row j % 9 / 3, column j % 3; zero beyond and for the
 * fourth plane).  A device buffer of 6 KiB (thhip_free). */
extern "C" void *thhip_conv_pack_weight_image_front(const float *w, int dtype)
{
	if (dtype != THHIP_F16 && dtype != THHIP_BF16)
		THError("thhip_conv_pack_weight_image_front: a half dtype");
	std::vector<unsigned short> host(2 * 3 * 64 * 8, 0);
	for (int mb = 0; mb < 2; mb++)
		for (int s = 0; s < 3; s++)
			for (int lane = 0; lane < 64; lane++)
				for (int e = 0; e < 8; e++) {
					const int m = mb * 32 + (lane & 31), h = lane >> 5, j = 8 * s + e, c = 2 * h + j / 9;
					float v = 0.0f;
					if (j < 18 && c < 3)
						v = w[(m * 3 + c) * 9 + j % 9];
					host[(((size_t)mb * 3 + s) * 64 + lane) * 8 + e] = dtype == THHIP_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
				}
	void *d = thhip_malloc(host.size() * 2);
	thhip_memcpy_h2d(d, host.data(), host.size() * 2);
	return d;
}

/* Whether thhip_conv2d_image_pair takes the two layers: half type; the first 3 -> 64 planes, the second 64 ->
 * at most 256 planes, both 3x3 / stride 1 / padding 1; channels-last output; an even image width. */
extern "C" int thhip_conv2d_image_pair_supported(int B, int H, int W, int Co1, int Co2, int dtype, int y_channels_last)
{
	if (dtype != THHIP_F16 && dtype != THHIP_BF16)
		return 0;
	if (Co1 != 64 || Co2 < 1 || Co2 > 256 || Co2 % 8 || !y_channels_last || W % 2 || H < 1 || W < 2 || B < 1)
		return 0;
	if ((double)B * 64 * H * W * 2 >= 2147483000.0 || (double)B * Co2 * H * W * 2 >= 2147483000.0)
		return 0;
	return !g_force_generic_cl && !g_force_bm && !g_force_bn;
}

/* Two modules' worth in one kernel: the image layer SpatialConvolutionMM(3 -> 64, 3x3, 1, 1) with its factor /
 * shift and Threshold, and the 3x3 layer that follows it with its own (and optionally the 2x2 max pooling after
 * that): the first layer's output (64 planes a pixel) is computed patch by patch in LDS and never written
 * (modules/SpatialConvolutionMM.c:126-225 twice, Threshold.c:38-63, SpatialMaxPooling.c:6-98).  img: [B][3][H][W]
 * plane-major; wfront from thhip_conv_pack_weight_image_front; wpacked as for thhip_conv2d_layout with
 * channels-last input; y channels-last. */
extern "C" void thhip_conv2d_image_pair(const void *img, const void *wfront, const float *scale1, const float *shift1,
	int act1, float thr1, float val1, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int H, int W, int Co, int act, float thr, float val, int pool2, int dtype)
{
	if (!thhip_conv2d_image_pair_supported(B, H, W, 64, Co, dtype, 1))
		THError("thhip_conv2d_image_pair: layers not supported (see thhip_conv2d_image_pair_supported)");
	const ConvImageFront f = { img, wfront, scale1, shift1, act1, thr1, val1 };
	conv_run(img, wpacked, scale, shift, y, B, 64, H, W, Co, 3, 3, 1, 1, 1, 1, act, thr, val, dtype, 0, 1, 1, pool2 != 0, 0, 0, &f);
}

extern "C" int thhip_conv2d_residual_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int dtype)
{
	if (dtype != THHIP_F32 || Ci % 32 || B < 1 || Co < 1 || kH < 1 || kW < 1 || dH < 1 || dW < 1 || padH < 0 || padW < 0)
		return 0;
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	if (oW < 1 || oH < 1)
		return 0;
	if ((double)B * Ci * H * W * 4 >= 2147483000.0 || (double)B * Co * oH * oW * 4 >= 2147483000.0)
		return 0;
	return !g_force_kch && !g_force_bm && !g_force_bn && !g_force_splitk;
}

/* thhip_conv2d_affine followed by the two-input table add of a residual block and the Threshold(0, 0)
 * after it, in the convolution's epilogue: with v = the convolution's result (after factor, bias and its
 * own Threshold) and r = res (a tensor of y's shape), y = v + c r (mode 1) or r + c v (mode 2), then
 * max(y, 0) if res_act.  Replaces SpatialConvolutionMM -> CAddTable -> Threshold
 * (modules/CAddTable.c:59-70 with the coefficient its caller gives: -1 for the reference's two-input
 * CAddTable) for the layers thhip_conv2d_residual_supported accepts; the same values, bit for bit, as
 * thhip_conv2d_affine followed by thhip_axpby2. */
extern "C" void thhip_conv2d_residual(const void *x, const void *wpacked, const float *scale, const float *shift,
	const void *res, int mode, float c, int res_act, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype)
{
	if (!thhip_conv2d_residual_supported(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, dtype) || (mode != 1 && mode != 2) || !res)
		THError("thhip_conv2d_residual: layer not supported (see thhip_conv2d_residual_supported), or mode %d not 1 or 2", mode);
	const ConvResidual r = { (const float *)res, mode, res_act, c };
	conv_run(x, wpacked, scale, shift, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, thr, val, dtype, 0, 0, 0, 0, &r);
}

/* Parts of the K split conv_dispatch gives an fp32 plane-major layer that runs on conv_f32_direct_kernel
 * and has its parts added by a second kernel (its rule, restated: at most 512 tiles of 64 x 64, about
 * 1024 workgroups, at least eight K-tiles a part); 0: another kernel, or no split. */
static int conv_f32_split_parts(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW)
{
	if (B < 1 || Ci < 1 || Co < 1 || kH < 1 || kW < 1 || dH < 1 || dW < 1 || padH < 0 || padW < 0)
		return 0;
	if (g_force_kch || g_force_bm || g_force_bn || g_force_splitk)
		return 0;
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	if (oW < 1 || oH < 1)
		return 0;
	if ((double)B * Ci * H * W * 4 >= 2147483000.0 || (double)B * Co * oH * oW * 4 >= 2147483000.0)
		return 0;	/* (the batch would be cut into slices) */
	const long N = (long)B * oH * oW, t64 = (long)((Co + 63) / 64) * ((N + 63) / 64);
	if (t64 > 512)
		return 0;
	int kch;
	if (Ci % 32 == 0)
		kch = CONV_KCH_F32;
	else if (kH * kW <= 4096)
		kch = 2;	/* a (plane, tap) per K row */
	else
		return 0;
	const int parts = conv_f32_ksplit(t64, conv_kc(Ci, kH, kW, THHIP_F32, 0) / kch);
	return parts > 1 ? parts : 0;
}

extern "C" int thhip_conv2d_poolk_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppH, int ppW, int ceil_mode, int dtype)
{
	if (dtype != THHIP_F32 || pkH < 1 || pkW < 1 || pdH < 1 || pdW < 1 || ppH < 0 || ppW < 0 || 2 * ppH > pkH || 2 * ppW > pkW)
		return 0;
	if (conv_f32_split_parts(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW) < 2)
		return 0;
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	/* windows of more than four values: where the two launches cost more than their work only (sixteen lanes per
	 * pooled value and every value of the convolution fetched once per window it lies in; 512->512 @14^2 at
	 * batch 16 with a 3x3 / stride 2 window would take longer than the two kernels) */
	if (pkH * pkW > 4 && (long)B * Co * oH * oW > (1L << 18))
		return 0;
	int pH, pW;
	thhip_pool_outsize(oH, oW, pkH, pkW, pdH, pdW, ppH, ppW, ceil_mode, &pH, &pW);
	return pH >= 1 && pW >= 1;
}

/* thhip_conv2d_affine followed by a max pooling of any window (SpatialMaxPooling.c:6-98), for the layers
 * thhip_conv2d_poolk_supported accepts: fp32 layers of a few tiles, whose K is split and whose parts a
 * second kernel adds -- that kernel then takes the maximum of every window as well, and the pooling's
 * own launch is saved.  y is [B][Co][pH][pW].  Replaces SpatialConvolutionMM -> Threshold ->
 * SpatialMaxPooling; the same values, bit for bit, as the convolution followed by thhip_maxpool. */
extern "C" void thhip_conv2d_poolk(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppH, int ppW, int ceil_mode,
	int act, float thr, float val, int dtype)
{
	if (!thhip_conv2d_poolk_supported(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pkH, pkW, pdH, pdW, ppH, ppW, ceil_mode, dtype))
		THError("thhip_conv2d_poolk: layer not supported (see thhip_conv2d_poolk_supported)");
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	ConvPoolK pk = { pkH, pkW, pdH, pdW, ppH, ppW, 0, 0 };
	thhip_pool_outsize(oH, oW, pkH, pkW, pdH, pdW, ppH, ppW, ceil_mode, &pk.oH, &pk.oW);
	conv_run(x, wpacked, scale, shift, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, thr, val, dtype, 0, 0, 0, 0, 0, &pk);
}

extern "C" void thhip_conv2d(const void *x, const void *wpacked, const float *bias, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype)
{
	thhip_conv2d_affine(x, wpacked, 0, bias, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, thr, val, dtype);
}

/* uint8 codes [Co][Ci][kH][kW] -> (code - 128) as signed bytes in the packed
 * layout for input layout xl, followed by the per-row sums of the re-centred codes. */
extern "C" void *thhip_conv_pack_weight_u8_layout(const unsigned char *w, int Co, int Ci, int kH, int kW, int x_layout)
{
	const int xl = x_layout;
	const int chunk = 32, KC = conv_kc(Ci, kH, kW, THHIP_U8, xl);
	const size_t bytes = conv_packed_bytes(Co, Ci, kH, kW, THHIP_U8, xl);
	const size_t mpad = (size_t)(Co + CONV_MPAD - 1) / CONV_MPAD * CONV_MPAD;
	const size_t total = bytes + mpad * sizeof(int);
	unsigned char *host = (unsigned char *)calloc(1, total);
	if (!host)
		THError("thhip_conv_pack_weight_u8: out of host memory (%zu bytes)", total);
	int *rowsum = (int *)(host + bytes);
	for (int m = 0; m < Co; m++) {
		int sum = 0;
		for (int c = 0; c < Ci; c++)
			for (int kh = 0; kh < kH; kh++)
				for (int kw = 0; kw < kW; kw++) {
					const size_t idx = conv_pack_index(m, conv_kpos(c, kh, kw, Ci, kH, kW, THHIP_U8, xl), KC, chunk);
					const int v = (int)w[(((size_t)m * Ci + c) * kH + kh) * kW + kw] - 128;
					host[idx] = (unsigned char)(signed char)v;
					sum += v;
				}
		rowsum[m] = sum;
	}
	void *dev = thhip_malloc(total);
	thhip_memcpy_h2d(dev, host, total);
	free(host);
	return dev;
}

extern "C" void *thhip_conv_pack_weight_u8(const unsigned char *w, int Co, int Ci, int kHW)
{
	return thhip_conv_pack_weight_u8_layout(w, Co, Ci, 1, kHW, 0);
}

extern "C" void thhip_conv2d_u8_layout_tail(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift,
	int act, int thr, int val, int x_layout, int y_channels_last, int x_tail_bytes)
{
	if (c_shift < 0 || c_shift > 31)
		THError("thhip_conv2d_u8: shift %d out of range", c_shift);
	if (x_tail_bytes < 0)
		THError("thhip_conv2d_u8: negative tail");
	ConvU8Args u8 = { addend, zero & 255, a_off, b_off, c_off, c_mult, c_shift, thr, val,
		x_layout, y_channels_last != 0, x_tail_bytes };
	conv_run(x, wpacked, 0, 0, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, act, 0, 0, THHIP_U8, &u8);
}

extern "C" void thhip_conv2d_u8_layout(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift,
	int act, int thr, int val, int x_layout, int y_channels_last)
{
	thhip_conv2d_u8_layout_tail(x, wpacked, addend, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW,
		zero, a_off, b_off, c_off, c_mult, c_shift, act, thr, val, x_layout, y_channels_last, 0);
}

extern "C" void thhip_conv2d_u8(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift,
	int act, int thr, int val)
{
	thhip_conv2d_u8_layout(x, wpacked, addend, y, B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW,
		zero, a_off, b_off, c_off, c_mult, c_shift, act, thr, val, 0, 0);
}

/* The reference's only entry into gemmlowp (lowp/gemm8.cc:4-17): host
 * matrices, row-major A[m][k], B[k][n], C[m][n].  Run as a 1x1 "convolution"
 * over an image of n positions (oH = 1, oW = n), without bias add. */
extern "C" void lowpgemm(const int is_a_transposed, const int is_b_transposed, const int is_c_transposed,
	const int m, const int n, const int k,
	const unsigned char *a, const unsigned char *b, unsigned char *c,
	const int lda, const int ldb, const int ldc,
	const int a_offset, const int b_offset, const int c_offset,
	const int c_mult, const int c_shift)
{
	if (!is_a_transposed || !is_b_transposed || !is_c_transposed)
		THError("lowpgemm: only the all-transposed (row-major) form of lowp_basic.c:314-320 is implemented");
	if (m < 1 || n < 1 || k < 1 || lda < k || ldb < n || ldc < n)
		THError("lowpgemm: bad sizes");
	unsigned char *wtmp = 0, *btmp = 0, *ctmp = 0;
	const unsigned char *ap = a, *bp = b;
	if (lda != k) {
		wtmp = (unsigned char *)malloc((size_t)m * k);
		for (int i = 0; i < m; i++)
			memcpy(wtmp + (size_t)i * k, a + (size_t)i * lda, k);
		ap = wtmp;
	}
	if (ldb != n) {
		btmp = (unsigned char *)malloc((size_t)k * n);
		for (int i = 0; i < k; i++)
			memcpy(btmp + (size_t)i * n, b + (size_t)i * ldb, n);
		bp = btmp;
	}
	void *wp = thhip_conv_pack_weight_u8(ap, m, k, 1);
	unsigned char *dx = (unsigned char *)thhip_malloc((size_t)k * n);
	unsigned char *dy = (unsigned char *)thhip_malloc((size_t)m * n);
	thhip_memcpy_h2d(dx, bp, (size_t)k * n);
	thhip_conv2d_u8(dx, wp, 0, dy, 1, k, 1, n, m, 1, 1, 1, 1, 0, 0, 0, a_offset, b_offset, c_offset, c_mult, c_shift, 0, 0, 0);
	if (ldc != n) {
		ctmp = (unsigned char *)malloc((size_t)m * n);
		thhip_memcpy_d2h(ctmp, dy, (size_t)m * n);
		for (int i = 0; i < m; i++)
			memcpy(c + (size_t)i * ldc, ctmp + (size_t)i * n, n);
	} else
		thhip_memcpy_d2h(c, dy, (size_t)m * n);
	thhip_free(wp);
	thhip_free(dx);
	thhip_free(dy);
	free(wtmp);
	free(btmp);
	free(ctmp);
}

/* Packed weights -> row-major [Co][Ci*kHW] in the same dtype, on the device;
 * used when a layer turns out to be a matrix-vector product (one output
 * position). */
template <typename E>
__global__ void conv_unpack_rows_kernel(const E *wp, E *rows, int Co, int Ci, int kHW, int KC, int chunk, int kch, int tapmajor)
{
	const int K = Ci * kHW, vec = chunk / 2, cb = kch * chunk;
	long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
	const long total = (long)Co * K, step = (long)gridDim.x * blockDim.x;
	for (; i < total; i += step) {
		const int m = (int)(i / K), k = (int)(i % K);
		long kp = k;
		if (tapmajor) {
			const int c = k / kHW, tap = k % kHW;
			kp = ((long)(c / cb) * kHW + tap) * cb + c % cb;
		}
		const long kc = kp / chunk;
		const int h = (int)(kp % chunk) / vec, e = (int)(kp % vec);
		rows[i] = wp[((((size_t)(m >> 5) * KC + kc) * 2 + h) * 32 + (m & 31)) * vec + e];
	}
}

extern "C" void *thhip_conv_unpack_rows(const void *wpacked, int Co, int Ci, int kHW, int dtype)
{
	const int KC = conv_kc(Ci, 1, kHW, dtype, 0), chunk = conv_chunk(dtype), tm = conv_tap_major(Ci, dtype);
	const long total = (long)Co * Ci * kHW;
	void *rows = thhip_malloc((size_t)total * thhip_esize(dtype));
	long blocks = (total + 255) / 256;
	if (blocks > 65536)
		blocks = 65536;
	if (dtype == THHIP_F32)
		conv_unpack_rows_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(
			(const float *)wpacked, (float *)rows, Co, Ci, kHW, KC, chunk, conv_kch(dtype, false), tm);
	else if (dtype == THHIP_F16 || dtype == THHIP_BF16)
		conv_unpack_rows_kernel<unsigned short><<<dim3((unsigned)blocks), dim3(256), 0, thhip_stream()>>>(
			(const unsigned short *)wpacked, (unsigned short *)rows, Co, Ci, kHW, KC, chunk, conv_kch(dtype, false), tm);
	else
		THError("thhip_conv_unpack_rows: unsupported dtype %d", dtype);
	hipcheck(hipGetLastError());
	return rows;
}
