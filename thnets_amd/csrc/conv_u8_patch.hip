/*
 * uint8 convolution of small channels-last images that keeps the input patch in LDS:
 * Lowp_SpatialConvolution_updateOutput (lowp/lowp_SpatialConvolution.c:124-187: uint8
 * im2col with the padding code, gemmlowp GEMM, saturating bias add with its unclamped
 * tail), the Lowp_Threshold that follows (lowp_Threshold.c:3-28) and, optionally, a
 * 3x3 / stride 2 Lowp_SpatialMaxPooling (lowp_SpatialMaxPooling.c:45-108), for stride-1
 * layers whose input planes come in blocks of 64 and whose output rows are at most 64
 * positions wide (AlexNet's conv2-5 at 27 x 27 and 13 x 13).
 *
 * Why: as an implicit GEMM over flattened positions every tap of the kernel fetches
 * its own copy of the input from L2 (nine times for a 3x3 layer), and the path from L2
 * to LDS, not the matrix core, sets the time of these layers.  Here a workgroup owns a
 * band of output rows of one image (up to 192 positions, six MFMA tiles of 32) and 64
 * output planes.  The band's input patch (with its halo, ALL input planes) is in LDS
 * once - before the K loop, or (3x3 and 5x5 kernels on 128 planes and more) plane block by
 * plane block just ahead of the taps that read it, one barrier a block; the loop itself
 * has no barrier: the B fragments of every tap come from the patch, and the A
 * fragments - the weights, which thhip_conv_pack_weight_u8_patch stores in exactly the
 * order the matrix core wants them - go from global memory straight into the registers
 * the MFMA reads.
 *
 *  - K order: (block of 64 planes, tap, plane in the block); a K-tile is one tap of one
 *    block: 64 codes = two chunks of 32.  The pack step stores, per 64 output planes and
 *    K-tile, the four 1 KiB fragments (row half i, chunk c), re-centred to signed bytes.
 *  - Eight wavefronts: (row half i, half nh of the position tiles, chunk kp).  A wavefront
 *    multiplies its row half with three position tiles over its chunk of every K-tile:
 *    one 16-byte load from global memory (a few K-tiles ahead) and three fragment reads
 *    for three MFMAs.  Two wavefronts per SIMD keep the matrix core issuing (one alone
 *    gets an MFMA through every 55 cycles of the shader clock counter, two together one every 37).  The two chunks'
 *    partial sums are added through LDS at the end (integers: exact).
 *  - A patch pixel is Ci bytes = Ci / 16 vectors; the patch is kept plane block by plane
 *    block, vector plane by vector plane ([block][vector][pixel][16 bytes]), so the 32
 *    positions of a fragment read (neighbouring pixels, one vector each) are 512
 *    contiguous bytes and a tap is an offset.  Pixels outside the image hold the padding
 *    code.  The codes are re-centred (x ^ 0x80) when the patch is stored.  The sum of
 *    each pixel's codes (LDS atomics as the vectors are stored) and from those the column
 *    sums of the expanded offset term (one value per position: the sum over the taps, taken
 *    along the kernel rows and then down its columns) are made once, before the loop.
 *  - Epilogue as in the other uint8 kernels (expanded offset terms, gemmlowp's output stage
 *    in wrapping int32, bias add with its unclamped tail, threshold), every wavefront
 *    finishing half of what it and its partner summed; then either 8-byte channels-last
 *    stores, or the codes go to LDS and every thread takes the maximum of a 3x3 window for
 *    16 planes.
 */
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include "thhip_internal.h"

#define CP_THREADS 512
#define CP_MAXPOS 192		/* positions of a workgroup: six tiles of 32 */
#define CP_MAXPIX 1024		/* pixels of a patch */
#define CP_PLANES 64
#define CP_DEPTH 6		/* K-tiles of weights on their way to a wavefront's registers */
#define CP_NB 6			/* patch vectors a thread has on their way at once */
#define CP_XCH (8 * 24 * 64 * 4)	/* exchange of partial sums: 24 registers of eight wavefronts */
#define CP_CBUF (CP_MAXPOS * CP_PLANES)	/* codes of a band before the pooling */
/* column terms, row terms, bias addends, pixel sums, their sums along the kernel rows (reads of up to 3 + 4
 * sums past a patch's last stay inside) */
#define CP_TABLES ((CP_MAXPOS + 2 * CP_PLANES + 2 * (CP_MAXPIX + 8)) * 4)
#define CP_LDS_MAX (150 * 1024)

struct ConvPatchParams {
	const unsigned char *x;		/* [B][H][W][Ci] codes */
	const unsigned char *wp;	/* thhip_conv_pack_weight_u8_patch */
	const int *rowsum;
	const int *addend;		/* per output plane, or NULL */
	unsigned char *y;		/* [B][oH][oW][Co], or [B][pH][pW][Co] when pooling */
	int B, Ci, H, W, Co, kH, kW, padH, padW, oH, oW, pH, pW;
	int pool;			/* the 3x3 / stride 2 pooling is done here */
	int rb;				/* output rows (pooled rows when pooling) per workgroup */
	int cwl;			/* convolution columns a workgroup computes */
	int pw;				/* patch width in pixels: cwl + kW - 1 */
	int taps, nkt, K;
	int vp;				/* bytes between the vector planes of a patch */
	int front;			/* bytes of LDS before the tables */
	unsigned m_pw, m_cwl, m_pW;	/* x / d == __umulhi(x, m_d) for the small x used here (0: d == 1) */
	int zero, offA, offB, c_off, c_mult, c_shift, act, ithr, ival;
};

typedef unsigned short cp_us2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));

/* v_permlane32_swap(x, y) exchanges x of lanes 32..63 with y of lanes 0..31. */
__device__ __forceinline__ void cp_swap32(unsigned &x, unsigned &y)
{
	const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
	x = r[0];
	y = r[1];
}

__device__ __forceinline__ int cp_div(int x, unsigned magic)
{
	return magic ? (int)__umulhi((unsigned)x, magic) : x;
}

/* Sum of n values q[0], q[step], ...: four reads on their way at once, those past the end (which read the
 * last one again) count nothing. */
__device__ __forceinline__ int cp_sum_strided(const int *q, int n, int step)
{
	int s0 = 0, s1 = 0, s2 = 0, s3 = 0;
	for (int k = 0; k < n; k += 4) {
		const int v0 = q[k * step], v1 = q[min(k + 1, n - 1) * step], v2 = q[min(k + 2, n - 1) * step],
			v3 = q[min(k + 3, n - 1) * step];
		s0 += v0;
		s1 += k + 1 < n ? v1 : 0;
		s2 += k + 2 < n ? v2 : 0;
		s3 += k + 3 < n ? v3 : 0;
	}
	return s0 + s1 + s2 + s3;
}

/* f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>) */
template <int I, int N, typename F>
__device__ __forceinline__ void cp_static_for(F &&f)
{
	if constexpr (I < N) {
		f(std::integral_constant<int, I>{});
		cp_static_for<I + 1, N>(f);
	}
}

/* D = 0: the whole patch before the K loop.  D > 0 (3 or 5; the kernel's taps a multiple of it, taps / D odd,
 * at least two plane blocks, a patch of at most 256 pixels): the patch is streamed - block 0 before the loop,
 * block cb + 1 requested when block cb's taps begin and stored when they end (one barrier per block), the
 * weights through a ring of D K-tiles that starts anew with every block, so that every wait count is a
 * constant of straight-line code.
 * Two workgroups per CU where the patch allows: 128 registers per lane. */
template <bool POOL, int D>
__global__ __launch_bounds__(CP_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void conv_u8_patch_kernel(ConvPatchParams p)
{
	/* patch: blocks x 4 vector planes                    (the front: later the exchange of sums | the codes)
	 * column terms | row terms | bias addends | pixel sums | their row sums        (the tables, from p.front on) */
	extern __shared__ __align__(16) unsigned char lds[];
	int *const colterm = (int *)(lds + p.front);
	int *const rowterm = colterm + CP_MAXPOS;
	int *const rowadd = rowterm + CP_PLANES;
	int *const psum = rowadd + CP_PLANES;
	int *const hsum = psum + CP_MAXPIX + 8;

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int ri = wave & 1, nh = (wave >> 1) & 1, kp = wave >> 2;	/* row half, half of the position tiles, chunk of every K-tile */
	const int n = lane & 31, h = lane >> 5;
	const int band = blockIdx.x, mz = blockIdx.y, b = blockIdx.z;
	/* the band: output rows row0 .. row0 + rows - 1 */
	const int row0 = POOL ? 2 * band * p.rb : band * p.rb;
	const int pra = POOL ? min(p.rb, p.pH - band * p.rb) : 0;	/* pooled rows of this band */
	const int rows = POOL ? 2 * pra + 1 : min(p.rb, p.oH - row0);
	const int npos = rows * p.cwl;
	const int prows = rows + p.kH - 1;
	const int npix = prows * p.pw;
	const int nblocks = p.Ci >> 6;
	const int blk = 4 * p.vp;	/* bytes of a plane block of the patch */

	/* ---- weights: fragment (row half ri, chunk kp) of every K-tile, CP_DEPTH K-tiles ahead; a base that is
	 * uniform in the wavefront plus a 32-bit lane offset ---- */
	const unsigned char *wsrc = p.wp + ((size_t)mz * p.nkt) * 4096 + (ri * 2 + kp) * 1024;
	const unsigned woff = lane * 16;
	constexpr int RING = D ? D : CP_DEPTH;
	intx4 wr[RING];
#define CP_WFETCH(SLOT_, KT_) (wr[SLOT_] = *(const intx4 *)(wsrc + (size_t)min((KT_), p.nkt - 1) * 4096 + woff))
#pragma unroll
	for (int d = 0; d < RING; d++)
		CP_WFETCH(d, d);

	for (int pp = tid; pp < npix + 8; pp += CP_THREADS)
		psum[pp] = 0;
	/* (asked for now, put into LDS once the patch is: nothing waits for memory before the patch's own loads are out) */
	int rs = 0, ra = 0;
	if (tid < CP_PLANES) {
		rs = p.rowsum[mz * CP_PLANES + tid];
		ra = p.addend ? p.addend[mz * CP_PLANES + tid] : 0;
	}
	__syncthreads();

	/* ---- the patch, plane block by plane block: of a block, vector s = vector s % 4 of pixel s / 4 (a
	 * wavefront's load covers 16 whole pixels: 64 contiguous bytes each), re-centred (code - 128 as signed
	 * bytes: x ^ 0x80); with a vector goes its share of the sum of its pixel's codes.  CP_NB loads of a
	 * thread are on their way before the first is stored. ---- */
	const int zero4 = p.zero * 0x01010101;
	if constexpr (D == 0) {
		const int nvec = npix * 4 * nblocks;	/* vector s: vector s % 4 of pixel (s / 4) % npix of block s / (4 npix) */
		const float inv_npix = 1.0f / (float)npix;	/* ((q + 0.5) / npix is at least 0.5 / npix away from an integer: rounding cannot cross it) */
		for (int s0 = tid; s0 < nvec; s0 += CP_NB * CP_THREADS) {
			intx4 pv[CP_NB];
			int dst[CP_NB], pix[CP_NB];
#pragma unroll
			for (int u = 0; u < CP_NB; u++) {
				const int s = s0 + u * CP_THREADS, q = s >> 2;
				const int cb = (int)(((float)q + 0.5f) * inv_npix), pp = q - cb * npix;
				const int pr = cp_div(pp, p.m_pw), pc = pp - pr * p.pw;
				const int iy = row0 - p.padH + pr, ix = pc - p.padW;
				const bool in = s < nvec && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W;
				dst[u] = s < nvec ? cb * blk + (s & 3) * p.vp + pp * 16 : -1;
				pix[u] = pp;
				if (in)
					pv[u] = *(const intx4 *)(p.x + ((size_t)((b * p.H + iy) * p.W + ix) * p.Ci + cb * 64 + (s & 3) * 16));
				else
					pv[u] = intx4{ zero4, zero4, zero4, zero4 };
			}
#pragma unroll
			for (int u = 0; u < CP_NB; u++) {
				intx4 v = pv[u];
				int part = 0;
#pragma unroll
				for (int d = 0; d < 4; d++) {
					v[d] ^= (int)0x80808080;
					part = __builtin_amdgcn_sdot4(v[d], 0x01010101, part, false);
				}
				part += __shfl_xor(part, 1, 64);	/* the four vectors of a pixel sit in four neighbouring lanes */
				part += __shfl_xor(part, 2, 64);
				if (dst[u] >= 0) {
					*(intx4 *)(lds + dst[u]) = v;
					if ((lane & 3) == 0)
						atomicAdd(&psum[pix[u]], part);
				}
			}
		}
	}
	/* streamed: of every block this thread moves vectors tid and tid + 512 (vector s % 4 of pixel s / 4) */
	int psrc[2];	/* byte offset in x of the vector (without the plane block), or -1: outside the image or the patch */
#pragma unroll
	for (int u = 0; u < 2; u++) {
		const int s = tid + u * CP_THREADS, pp = s >> 2;
		const int pr = cp_div(pp, p.m_pw), pc = pp - pr * p.pw;
		const int iy = row0 - p.padH + pr, ix = pc - p.padW;
		const bool in = pp < npix && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W;
		psrc[u] = in ? ((b * p.H + iy) * p.W + ix) * p.Ci + (s & 3) * 16 : -1;
	}
	intx4 pvn[2];
	auto patch_fetch = [&](int cb) {	/* (always two loads: what lies outside fetches the tensor's first bytes) */
#pragma unroll
		for (int u = 0; u < 2; u++)
			pvn[u] = *(const intx4 *)(p.x + (psrc[u] >= 0 ? psrc[u] + cb * 64 : 0));
	};
	auto patch_store = [&](int cb) {
#pragma unroll
		for (int u = 0; u < 2; u++) {
			const int s = tid + u * CP_THREADS, pp = s >> 2;
			intx4 v = psrc[u] >= 0 ? pvn[u] : intx4{ zero4, zero4, zero4, zero4 };
			int part = 0;
#pragma unroll
			for (int d = 0; d < 4; d++) {
				v[d] ^= (int)0x80808080;
				part = __builtin_amdgcn_sdot4(v[d], 0x01010101, part, false);
			}
			part += __shfl_xor(part, 1, 64);
			part += __shfl_xor(part, 2, 64);
			if (pp < npix) {
				*(intx4 *)(lds + cb * blk + (s & 3) * p.vp + pp * 16) = v;
				if ((lane & 3) == 0)
					atomicAdd(&psum[pp], part);
			}
		}
	};
	if constexpr (D != 0) {
		patch_fetch(0);
		patch_store(0);
	}
	if (tid < CP_PLANES) {
		/* (wrapping, like the sum they join; multiplier and rounding term of the output stage folded in:
		 * (acc + rowterm + colterm) mult + round = acc mult + (rowterm mult + round) + colterm mult) */
		rowterm[tid] = (p.offB * rs + p.K * p.offA * p.offB + p.c_off) * p.c_mult + (p.c_shift < 1 ? 0 : 1 << (p.c_shift - 1));
		rowadd[tid] = ra;
	}
	__syncthreads();
	/* the column sums of the expanded offset term: a position's pixel sums under all the taps, in two passes:
	 * along the kernel rows for every pixel (the sums of pixels whose kernel row leaves the patch are not
	 * used), then down the kernel columns for every position.  (Once the whole patch is in LDS.) */
	auto column_terms = [&]() {
		for (int pp = tid; pp < npix; pp += CP_THREADS)
			hsum[pp] = cp_sum_strided(psum + pp, p.kW, 1);
		__syncthreads();
		if (tid < CP_MAXPOS) {
			const int posc = min(tid, npos - 1);
			const int ly = cp_div(posc, p.m_cwl), lx = posc - ly * p.cwl;
			colterm[tid] = cp_sum_strided(hsum + ly * p.pw + lx, p.kH, p.pw) * p.offA * p.c_mult;	/* (multiplier folded in) */
		}
	};
	if constexpr (D == 0)
		column_terms();
	/* ---- this lane's positions: tile nh * 3 + j, position n of it ---- */
	int pp0[3];
#pragma unroll
	for (int j = 0; j < 3; j++) {
		const int pos = min((nh * 3 + j) * 32 + n, npos - 1);
		const int ly = cp_div(pos, p.m_cwl), lx = pos - ly * p.cwl;
		pp0[j] = (ly * p.pw + lx) * 16 + (2 * kp + h) * p.vp;	/* byte offset in a plane block: the vector plane this lane feeds to the matrix core */
	}
	intx16 acc[3];
#pragma unroll
	for (int j = 0; j < 3; j++)
#pragma unroll
		for (int r = 0; r < 16; r++)
			acc[j][r] = 0;
	intx4 bf[2][3];
	if constexpr (D == 0) {
		/* tiles of this wavefront that hold positions of the band */
		const int mytiles = min(3, max(0, (npos + 31) / 32 - nh * 3));
		/* the K-tile whose fragments are requested next: plane block, tap */
		int n_cb = 0, n_tap = 0, n_kh = 0, n_kw = 0;
		auto frags = [&](intx4 (&bb)[3]) {
			const unsigned char *pb = lds + n_cb * blk + (n_kh * p.pw + n_kw) * 16;
#pragma unroll
			for (int j = 0; j < 3; j++)
				bb[j] = *(const intx4 *)(pb + pp0[j]);
			if (++n_kw == p.kW) {
				n_kw = 0;
				++n_kh;
			}
			if (++n_tap == p.taps) {
				n_tap = n_kh = n_kw = 0;
				++n_cb;
			}
		};
		if (mytiles > 0) {
			/* Every step of the main loop issues the same memory operations whatever its K-tile: the compiler
			 * sets its waits for the worst of the paths that meet, and an operation on one path only makes
			 * every step wait for everything (measured: 390 -> 650 cycles a step). */
			frags(bf[0]);
			auto step = [&](int kt, auto slot_, auto par_, auto tail_) {
				constexpr int slot = decltype(slot_)::value;	/* kt % CP_DEPTH */
				constexpr int par = decltype(par_)::value;	/* kt % 2: the register set that holds K-tile kt */
				if (!decltype(tail_)::value || kt + 1 < p.nkt)
					frags(bf[par ^ 1]);	/* requested under this K-tile's MFMAs */
				const intx4 a = wr[slot];
#pragma unroll
				for (int j = 0; j < 3; j++)
					acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bf[par][j], acc[j], 0, 0, 0);
				CP_WFETCH(slot, kt + CP_DEPTH);
			};
			typedef std::integral_constant<int, 0> I0;
			typedef std::integral_constant<int, 1> I1;
			typedef std::integral_constant<int, 2> I2;
			typedef std::integral_constant<int, 3> I3;
			typedef std::integral_constant<int, 4> I4;
			typedef std::integral_constant<int, 5> I5;
			int kt = 0;
			for (; kt + 6 < p.nkt; kt += 6) {	/* (kt + 6 < nkt: the K-tile after these six exists) */
				step(kt, I0{}, I0{}, I0{});
				step(kt + 1, I1{}, I1{}, I0{});
				step(kt + 2, I2{}, I0{}, I0{});
				step(kt + 3, I3{}, I1{}, I0{});
				step(kt + 4, I4{}, I0{}, I0{});
				step(kt + 5, I5{}, I1{}, I0{});
			}
			if (kt < p.nkt)
				step(kt, I0{}, I0{}, I1{});
			if (kt + 1 < p.nkt)
				step(kt + 1, I1{}, I1{}, I1{});
			if (kt + 2 < p.nkt)
				step(kt + 2, I2{}, I0{}, I1{});
			if (kt + 3 < p.nkt)
				step(kt + 3, I3{}, I1{}, I1{});
			if (kt + 4 < p.nkt)
				step(kt + 4, I4{}, I0{}, I1{});
			if (kt + 5 < p.nkt)
				step(kt + 5, I5{}, I1{}, I1{});
		}
	} else {
		/* Streamed: a block's taps are groups of D steps, step i of a group on weight slot i; the fragments
		 * of the next K-tile of the block are requested under a step's MFMAs (past a block's last tap: its
		 * last tap's again, which nothing uses).  The first group after a block's patch loads went out is
		 * straight-line code of its own: its waits count the patch loads as younger than the weights they
		 * wait for; from the second group on the patch loads are older than every weight in flight. */
		static_assert(D % 2 == 1, "taps / D odd and D odd: a block has an odd number of steps");
		int c_kh = 0, c_kw = 0;		/* kernel row and column of the K-tile whose fragments were requested last */
		auto frags = [&](intx4 (&bb)[3], int cb, int kh, int kw) {
			const unsigned char *pb = lds + cb * blk + (kh * p.pw + kw) * 16;
#pragma unroll
			for (int j = 0; j < 3; j++)
				bb[j] = *(const intx4 *)(pb + pp0[j]);
		};
		/* one step: K-tile (cb, tap t) on slot `slot`, its fragments in bf[par] */
		auto step = [&](int cb, int t, auto slot_, auto par_) {
			constexpr int slot = decltype(slot_)::value, par = decltype(par_)::value;
			if (c_kw + 1 < p.kW)
				++c_kw;
			else if (c_kh + 1 < p.kH) {
				c_kw = 0;
				++c_kh;
			}
			frags(bf[par ^ 1], cb, c_kh, c_kw);
			const intx4 a = wr[slot];
#pragma unroll
			for (int j = 0; j < 3; j++)
				acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bf[par][j], acc[j], 0, 0, 0);
			CP_WFETCH(slot, cb * p.taps + t + D);
		};
		const int groups = p.taps / D;	/* odd */
		auto block = [&](int cb, auto more_) {
			constexpr bool more = decltype(more_)::value;	/* another block follows: its patch is streamed */
			c_kh = c_kw = 0;
			frags(bf[0], cb, 0, 0);
			if constexpr (more)
				patch_fetch(cb + 1);
			cp_static_for<0, D>([&](auto i_) {
				constexpr int i = decltype(i_)::value;
				step(cb, i, i_, std::integral_constant<int, i % 2>{});
			});
			for (int g = 1; g < groups; g += 2)
				cp_static_for<0, 2 * D>([&](auto i_) {
					constexpr int i = decltype(i_)::value;
					step(cb, g * D + i, std::integral_constant<int, i % D>{}, std::integral_constant<int, (i + 1) % 2>{});
				});
			if constexpr (more) {
				patch_store(cb + 1);
				__syncthreads();
			}
		};
		for (int cb = 0; cb + 1 < nblocks; cb++)
			block(cb, std::true_type{});
		column_terms();
		block(nblocks - 1, std::false_type{});
	}
#undef CP_WFETCH
	__syncthreads();	/* everybody is done with the patch (and the tables are written) */

	/* ---- the two chunks' sums.  Units u = 2 j + (upper half of the registers): wavefront kp finishes units
	 * 3 kp .. 3 kp + 2 and hands the other three to its partner (wave ^ 4) ---- */
	{
		int *mine = (int *)lds + wave * (24 * 64);
#pragma unroll
		for (int u = 0; u < 3; u++)	/* the units the partner finishes (kp is uniform in a wavefront) */
#pragma unroll
			for (int r = 0; r < 8; r++)
				mine[(u * 8 + r) * 64 + lane] = kp ? (u == 0 ? acc[0][r] : u == 1 ? acc[0][8 + r] : acc[1][r])
								   : (u == 0 ? acc[1][8 + r] : u == 1 ? acc[2][r] : acc[2][8 + r]);
	}
	__syncthreads();
	int fin[3][8];	/* the three units this wavefront finishes */
	{
		const int *other = (const int *)lds + (wave ^ 4) * (24 * 64);
#pragma unroll
		for (int u = 0; u < 3; u++)
#pragma unroll
			for (int r = 0; r < 8; r++) {
				const int own = kp ? (u == 0 ? acc[1][8 + r] : u == 1 ? acc[2][r] : acc[2][8 + r])
						   : (u == 0 ? acc[0][r] : u == 1 ? acc[0][8 + r] : acc[1][r]);
				fin[u][r] = own + other[(u * 8 + r) * 64 + lane];
			}
	}

	/* ---- requantise ---- */
	unsigned char *cbuf = lds + CP_XCH;	/* pooling: [position][64 planes], 16-byte pieces swapped around by the position */
	const int tail0 = (p.oH * p.oW / 8) * 8;	/* lowpadd's unclamped tail starts here */
	const bool has_add = p.addend != 0;
	const int athr = p.act ? p.ithr : -1;	/* no threshold: every code passes */
#pragma unroll
	for (int u = 0; u < 3; u++) {
		const int uu = 3 * kp + u, j = uu >> 1, gh = uu & 1;	/* tile, register half */
		const int pos = (nh * 3 + j) * 32 + n;
		const int posc = min(pos, npos - 1);
		const int ly = cp_div(posc, p.m_cwl), lx = posc - ly * p.cwl;
		const int rem = (row0 + ly) * p.oW + lx;
		/* lowpadd (lowp_SpatialConvolution.c:71-88): min(sum, 255), then the lower clamp at 0 - except for the
		 * last oH oW % 8 positions of a plane, whose negative sums wrap (the low byte is taken): a lower bound
		 * per lane and the mask do both without a branch */
		const int lo = has_add && rem >= tail0 ? (int)0x80000000 : 0;
		const int ct = colterm[pos];
		unsigned word[2];
#pragma unroll
		for (int g2 = 0; g2 < 2; g2++) {
			const int ml = ri * 32 + 8 * (2 * gh + g2) + 4 * h;
			const intx4 rt = *(const intx4 *)(rowterm + ml), ra4 = *(const intx4 *)(rowadd + ml);
			unsigned packed = 0;
#pragma unroll
			for (int e = 0; e < 4; e++) {
				/* gemmlowp's output stage in wrapping int32: (acc + row term + column term) mult + round,
				 * the constant parts multiplied before */
				const unsigned uq = (unsigned)fin[u][4 * g2 + e] * (unsigned)p.c_mult + (unsigned)rt[e] + (unsigned)ct;
				int q = (int)uq >> p.c_shift;
				q = q < 0 ? 0 : q > 255 ? 255 : q;
				q = max(min(q + ra4[e], 255), lo) & 255;	/* (no addend: 0, and nothing changes) */
				q = q > athr ? q : p.ival;
				packed |= (unsigned)q << (8 * e);
			}
			word[g2] = packed;
		}
		/* lane (n, h) holds planes 16 gh + 4 h .. + 3 and 16 gh + 8 + 4 h .. + 3 of the row half; after the
		 * swap lane n holds planes 16 gh .. + 7 and lane n + 32 planes 16 gh + 8 .. + 15 as 8 bytes */
		cp_swap32(word[0], word[1]);
		const uintx2 v = { word[0], word[1] };
		const int piece = 2 * ri + gh;		/* which 16 of the 64 planes */
		if (pos < npos) {
			if (POOL)
				*(uintx2 *)(cbuf + posc * CP_PLANES + ((piece ^ (posc >> 2)) & 3) * 16 + h * 8) = v;
			else
				*(uintx2 *)(p.y + ((size_t)b * p.oH * p.oW + rem) * p.Co + mz * CP_PLANES + piece * 16 + h * 8) = v;
		}
	}
	if (!POOL)
		return;
	__syncthreads();
	/* ---- 3x3 / stride 2 maximum, sixteen planes per thread ---- */
	for (int it = tid; it < pra * p.pW * 4; it += CP_THREADS) {
		const int c16 = it & 3, t = it >> 2;
		const int prl = cp_div(t, p.m_pW), pcl = t - prl * p.pW;
		cp_us2 me[4], mo[4];	/* byte-wise maxima as packed 16-bit maxima of the even and of the odd bytes */
#pragma unroll
		for (int d = 0; d < 4; d++)
			me[d] = mo[d] = cp_us2{ 0, 0 };
#pragma unroll
		for (int dy = 0; dy < 3; dy++)
#pragma unroll
			for (int dx = 0; dx < 3; dx++) {
				const int pos = (2 * prl + dy) * p.cwl + 2 * pcl + dx;
				const uintx4 v = *(const uintx4 *)(cbuf + pos * CP_PLANES + ((c16 ^ (pos >> 2)) & 3) * 16);
#pragma unroll
				for (int d = 0; d < 4; d++) {
					me[d] = __builtin_elementwise_max(me[d], __builtin_bit_cast(cp_us2, v[d] & 0x00ff00ffu));
					mo[d] = __builtin_elementwise_max(mo[d], __builtin_bit_cast(cp_us2, (v[d] >> 8) & 0x00ff00ffu));
				}
			}
		uintx4 m;
#pragma unroll
		for (int d = 0; d < 4; d++)
			m[d] = __builtin_bit_cast(unsigned, me[d]) | (__builtin_bit_cast(unsigned, mo[d]) << 8);
		*(uintx4 *)(p.y + (((size_t)b * p.pH + band * p.rb + prl) * p.pW + pcl) * p.Co + mz * CP_PLANES + c16 * 16) = m;
	}
}

/* x / d == __umulhi(x, cp_magic(d)) for 0 <= x < 2^32 / d (round-up reciprocal); 0 stands for d = 1 */
static unsigned cp_magic(int d)
{
	return d <= 1 ? 0u : (unsigned)((((unsigned long long)1 << 32) + d - 1) / d);
}

/* Geometry of a launch; returns 0 when the kernel does not take the layer, else the bytes of LDS. */
static int cp_plan(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int pool,
	ConvPatchParams *p)
{
	if (B < 1 || Ci < 64 || Ci % 64 || Co < 64 || Co % 64 || dH != 1 || dW != 1 || kH < 1 || kW < 1 ||
	    padH < 0 || padW < 0)
		return 0;
	const int oW = W + 2 * padW - kW + 1, oH = H + 2 * padH - kH + 1;
	if (oW < 1 || oH < 1)
		return 0;
	const int nblocks = Ci / 64;
	int cwl = oW, rb, pH = 0, pW = 0;
	/* bytes of LDS a band of `rows` output rows needs */
	auto lds_of = [&](int rows, int *vp_out) {
		const int npix = (rows + kH - 1) * (cwl + kW - 1);
		const int vp = (npix * 16 + 255) / 256 * 256 + 64;	/* 64 past a multiple of 256: the two halves of a fragment read fall on different banks */
		int front = nblocks * 4 * vp;
		if (npix > CP_MAXPIX)
			return 1 << 30;
		const int need = CP_XCH + (pool ? CP_CBUF : 0);
		if (front < need)
			front = need;
		front = (front + 15) / 16 * 16;
		if (vp_out)
			*vp_out = vp;
		return front + CP_TABLES;
	};
	if (pool) {
		if (oW < 3 || oH < 3)
			return 0;
		pH = (oH - 3) / 2 + 1;
		pW = (oW - 3) / 2 + 1;
		cwl = 2 * pW + 1;
		if (3 * cwl > CP_MAXPOS)
			return 0;
		rb = (CP_MAXPOS / cwl - 1) / 2;		/* pooled rows: 2 rb + 1 convolution rows */
		if (rb > pH)
			rb = pH;
		while (rb > 1 && lds_of(2 * rb + 1, 0) > CP_LDS_MAX)
			rb--;
		if (lds_of(2 * rb + 1, 0) > CP_LDS_MAX)
			return 0;
		/* bands of equal height rather than full ones and a short last one */
		const int bands = (pH + rb - 1) / rb;
		rb = (pH + bands - 1) / bands;
	} else {
		if (oW > CP_MAXPOS)
			return 0;
		rb = CP_MAXPOS / oW;
		if (rb > oH)
			rb = oH;
		while (rb > 1 && lds_of(rb, 0) > CP_LDS_MAX)
			rb--;
		if (lds_of(rb, 0) > CP_LDS_MAX)
			return 0;
		const int bands = (oH + rb - 1) / rb;
		rb = (oH + bands - 1) / bands;
	}
	if ((double)B * Ci * H * W >= 2147483000.0 || B > 65535 || Co / 64 > 65535)
		return 0;
	int vp = 0;
	const int total = lds_of(pool ? 2 * rb + 1 : rb, &vp);
	if (p) {
		p->B = B; p->Ci = Ci; p->H = H; p->W = W; p->Co = Co; p->kH = kH; p->kW = kW; p->padH = padH; p->padW = padW;
		p->oH = oH; p->oW = oW; p->pH = pH; p->pW = pW; p->pool = pool; p->rb = rb; p->cwl = cwl; p->pw = cwl + kW - 1;
		p->taps = kH * kW;
		p->nkt = Ci / 64 * kH * kW;
		p->K = Ci * kH * kW;
		p->vp = vp;
		p->front = total - CP_TABLES;
		p->m_pw = cp_magic(p->pw);
		p->m_cwl = cp_magic(cwl);
		p->m_pW = cp_magic(pW);
	}
	return total;
}

/* Whether thhip_conv2d_u8_patch takes the layer (pool = 1: together with a 3x3 / stride 2
 * max pooling without padding in floor mode). */
extern "C" int thhip_conv2d_u8_patch_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pool)
{
	return cp_plan(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pool, 0) > 0;
}

/* Codes [Co][Ci][kH][kW] -> per 64 output planes and K-tile (block of 64 input planes, tap)
 * the four fragments (row half i, chunk c) of v_mfma_i32_32x32x32_i8: lane = row % 32 +
 * 32 * (k half), 16 bytes each, re-centred to signed bytes; the per-row sums of the
 * re-centred codes follow.  Co % 64 == 0, Ci % 64 == 0. */
extern "C" void *thhip_conv_pack_weight_u8_patch(const unsigned char *w, int Co, int Ci, int kH, int kW)
{
	if (Co % 64 || Ci % 64 || Co < 64 || Ci < 64)
		THError("thhip_conv_pack_weight_u8_patch: Co = %d and Ci = %d must be multiples of 64", Co, Ci);
	const int taps = kH * kW, nkt = Ci / 64 * taps;
	const size_t bytes = (size_t)(Co / 64) * nkt * 4096, total = bytes + sizeof(int) * (size_t)Co;
	unsigned char *host = (unsigned char *)malloc(total);
	if (!host)
		THError("thhip_conv_pack_weight_u8_patch: out of host memory (%zu bytes)", total);
	int *rowsum = (int *)(host + bytes);
	for (int m = 0; m < Co; m++) {
		int sum = 0;
		for (int c = 0; c < Ci; c++)
			for (int t = 0; t < taps; t++) {
				const int v = (int)w[((size_t)m * Ci + c) * taps + t] - 128;
				const int kt = (c / 64) * taps + t, kk = c % 64;	/* K-tile, position in it */
				const int i = (m % 64) / 32, ch = kk / 32, hh = (kk % 32) / 16;
				const size_t idx = ((size_t)(m / 64) * nkt + kt) * 4096 + (size_t)(i * 2 + ch) * 1024 +
					(size_t)(hh * 32 + m % 32) * 16 + kk % 16;
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

/* x: codes [B][H][W][Ci]; wpatch: thhip_conv_pack_weight_u8_patch; y: [B][oH][oW][Co], or
 * [B][pH][pW][Co] with pool = 1 (pH = (oH - 3) / 2 + 1).  Same quantisation parameters as
 * thhip_conv2d_u8; `zero` is the padding code. */
extern "C" void thhip_conv2d_u8_patch(const unsigned char *x, const void *wpatch, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val, int pool)
{
	ConvPatchParams p;
	memset(&p, 0, sizeof(p));
	const int ldsbytes = cp_plan(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pool, &p);
	if (!ldsbytes)
		THError("thhip_conv2d_u8_patch: layer not supported (see thhip_conv2d_u8_patch_supported)");
	if (c_shift < 0 || c_shift > 31)
		THError("thhip_conv2d_u8_patch: shift %d out of range", c_shift);
	if (((size_t)x & 15) || ((size_t)y & 15))
		THError("thhip_conv2d_u8_patch: x and y must be 16-byte aligned");
	p.x = x;
	p.wp = (const unsigned char *)wpatch;
	p.rowsum = (const int *)(p.wp + (size_t)(Co / 64) * p.nkt * 4096);
	p.addend = addend;
	p.y = y;
	p.zero = zero & 255;
	p.offA = 128 + a_off;
	p.offB = 128 + b_off;
	p.c_off = c_off; p.c_mult = c_mult; p.c_shift = c_shift;
	p.act = act; p.ithr = thr; p.ival = val;
	const int bands = pool ? (p.pH + p.rb - 1) / p.rb : (p.oH + p.rb - 1) / p.rb;
	/* the patch streamed block by block where the kernel's taps come in an odd number of groups of 3 or 5,
	 * there are at least two plane blocks and a thread moves a block in two loads */
	const int npix_max = ((pool ? 2 * p.rb + 1 : p.rb) + kH - 1) * p.pw;
	const bool can_stream = Ci >= 128 && npix_max * 4 <= 2 * CP_THREADS;
	const int D = !can_stream ? 0 : p.taps % 5 == 0 && (p.taps / 5) % 2 ? 5 : p.taps % 3 == 0 && (p.taps / 3) % 2 ? 3 : 0;
	ThhipLaunchScope scope(THHIP_FAM_CONV_I8, 2.0 * Co * (double)p.K * B * p.oH * p.oW);
	const dim3 grid(bands, Co / 64, B);
	static bool attr_set[6];
#define CP_GO(POOL_, D_, I_) do { \
		if (!attr_set[I_]) {	/* more than 64 KiB of dynamic LDS has to be asked for */ \
			hipcheck(hipFuncSetAttribute((const void *)conv_u8_patch_kernel<POOL_, D_>, hipFuncAttributeMaxDynamicSharedMemorySize, CP_LDS_MAX)); \
			attr_set[I_] = true; \
		} \
		conv_u8_patch_kernel<POOL_, D_><<<grid, dim3(CP_THREADS), ldsbytes, thhip_stream()>>>(p); \
	} while (0)
	if (pool) {
		if (D == 5)
			CP_GO(true, 5, 0);
		else if (D == 3)
			CP_GO(true, 3, 1);
		else
			CP_GO(true, 0, 2);
	} else {
		if (D == 5)
			CP_GO(false, 5, 3);
		else if (D == 3)
			CP_GO(false, 3, 4);
		else
			CP_GO(false, 0, 5);
	}
#undef CP_GO
}
