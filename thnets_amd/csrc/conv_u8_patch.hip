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
 * output planes; per block of 64 input planes it copies the band's input patch (with its
 * halo) into LDS once and takes the B fragments of every tap from it; only the weights
 * stream.
 *
 *  - K order: (block of 64 planes, tap, plane in the block); a K-tile is one tap of one
 *    block: 64 codes = two chunks of 32.  thhip_conv_pack_weight_u8_patch stores, per 64
 *    output planes and K-tile, the four 1 KiB fragments (row half i, chunk c) the matrix
 *    core wants, re-centred to signed bytes.
 *  - Four wavefronts: (chunk c, half nh of the position tiles).  A wavefront multiplies
 *    both row halves with three position tiles: 5 fragment reads for 6 MFMAs per K-tile;
 *    the two chunks' partial sums are added through LDS at the end (integers: exact).
 *  - Weights: every wavefront fetches one fragment of a K-tile into registers three
 *    K-tiles ahead and passes it on through one of three LDS stages; one barrier per K-tile.
 *    The patch of the next plane block is fetched at the start of a block and stored a few
 *    K-tiles later into the second patch buffer.
 *  - A patch pixel is 64 bytes = four 16-byte vectors; the patch is kept vector plane by
 *    vector plane, so the 32 positions of a fragment read (neighbouring pixels, one vector
 *    each) are 512 contiguous bytes and a tap is an offset.  Pixels outside the image hold
 *    the padding code.  The codes are re-centred (x ^ 0x80) when the patch is stored, and
 *    the sum of each pixel's 64 codes is kept with it: the column sums of the expanded
 *    offset term are gathered from those, one value per position and tap.
 *  - The fragments of K-tile kt + 1 are requested before K-tile kt is multiplied.
 *  - Epilogue as in the other uint8 kernels (expanded offset terms, gemmlowp's output stage
 *    in wrapping int32, bias add with its unclamped tail, threshold); then either 16-byte
 *    channels-last stores, or the codes go to LDS and every thread takes the maximum of a
 *    3x3 window for 16 planes.
 */
#include <stdlib.h>
#include <string.h>
#include <type_traits>
#include "thhip_internal.h"

#define CP_THREADS 256
#define CP_MAXPOS 192		/* positions of a workgroup: six tiles of 32 */
#define CP_MAXPIX 384		/* pixels of a patch (24 KiB) */
#define CP_PL (CP_MAXPIX * 4 / CP_THREADS)	/* patch vectors per thread */
#define CP_PLANES 64

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
	int zero, offA, offB, c_off, c_mult, c_shift, act, ithr, ival;
};

typedef unsigned short cp_us2 __attribute__((ext_vector_type(2)));

/* v_permlane32_swap(x, y) exchanges x of lanes 32..63 with y of lanes 0..31. */
__device__ __forceinline__ void cp_swap32(unsigned &x, unsigned &y)
{
	const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
	x = r[0];
	y = r[1];
}

#define CP_VP (CP_MAXPIX * 16 + 64)	/* bytes between the vector planes of a patch: 64 past a multiple of 256 */

/* two workgroups per CU (LDS allows no more): 256 registers per lane */
template <bool POOL>
__global__ __launch_bounds__(CP_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_u8_patch_kernel(ConvPatchParams p)
{
	/* patch buffers 2 x 4 vector planes | pixel sums 2 x 384 | weight stages 3 x 4 KiB | row terms
	 * (the front is reused for the exchange of sums and for the codes at the end) */
	__shared__ __align__(16) unsigned char lds[2 * 4 * CP_VP + 2 * CP_MAXPIX * 4 + 3 * 4096 + 2 * CP_PLANES * 4];
	unsigned char *const patch0 = lds;
	int *const psum0 = (int *)(lds + 2 * 4 * CP_VP);
	unsigned char *const wst = (unsigned char *)(psum0 + 2 * CP_MAXPIX);
	int *const rowterm = (int *)(wst + 3 * 4096);
	int *const rowadd = rowterm + CP_PLANES;

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int kp = wave >> 1, nh = wave & 1;	/* this wavefront's chunk of every K-tile, its half of the position tiles */
	const int n = lane & 31, h = lane >> 5;
	const int band = blockIdx.x, mz = blockIdx.y, b = blockIdx.z;
	/* the band: output rows row0 .. row0 + rows - 1 */
	const int row0 = POOL ? 2 * band * p.rb : band * p.rb;
	const int pra = POOL ? min(p.rb, p.pH - band * p.rb) : 0;	/* pooled rows of this band */
	const int rows = POOL ? 2 * pra + 1 : min(p.rb, p.oH - row0);
	const int npos = rows * p.cwl;
	const int prows = rows + p.kH - 1;
	const int npix = prows * p.pw;

	/* ---- what this thread moves of a patch: vectors s = tid + 256 u = vector s % 4 of pixel s / 4
	 * (a wavefront's load covers 16 whole pixels: 64 contiguous bytes each) ---- */
	int psrc[CP_PL];	/* byte offset in x of the vector (without the plane block), or -1: outside the image */
#pragma unroll
	for (int u = 0; u < CP_PL; u++) {
		const int s = tid + CP_THREADS * u, pp = s >> 2;
		const int pr = pp / p.pw, pc = pp - pr * p.pw;
		const int iy = row0 - p.padH + pr, ix = pc - p.padW;
		const bool in = pp < npix && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W;
		psrc[u] = in ? (((b * p.H + iy) * p.W + ix) * p.Ci + (s & 3) * 16) : -1;
	}
	const int zero4 = p.zero * 0x01010101;
	intx4 pv[CP_PL];
	auto patch_fetch = [&](int cb) {
#pragma unroll
		for (int u = 0; u < CP_PL; u++)
			pv[u] = *(const intx4 *)(p.x + (psrc[u] >= 0 ? psrc[u] + cb * 64 : 0));
	};
	/* The patch is stored re-centred (code - 128 as signed bytes: x ^ 0x80), vector plane by
	 * vector plane ([vector][pixel][16 bytes]: the 32 positions of a fragment read are then
	 * 512 contiguous bytes), and with it the sum of every pixel's 64 re-centred codes, from
	 * which the column sums of the expanded offset term are gathered tap by tap. */
	auto patch_store = [&](int buf) {
#pragma unroll
		for (int u = 0; u < CP_PL; u++) {
			const int s = tid + CP_THREADS * u;
			intx4 v = psrc[u] >= 0 ? pv[u] : intx4{ zero4, zero4, zero4, zero4 };
			int part = 0;
#pragma unroll
			for (int d = 0; d < 4; d++) {
				v[d] ^= (int)0x80808080;
				part = __builtin_amdgcn_sdot4(v[d], 0x01010101, part, false);
			}
			part += __shfl_xor(part, 1, 64);	/* the four vectors of a pixel sit in four neighbouring lanes */
			part += __shfl_xor(part, 2, 64);
			if (s < npix * 4) {
				*(intx4 *)(patch0 + buf * (4 * CP_VP) + (s & 3) * CP_VP + (s >> 2) * 16) = v;
				if ((s & 3) == 0)
					psum0[buf * CP_MAXPIX + (s >> 2)] = part;
			}
		}
	};

	/* ---- weights: fragment `wave` (row half wave / 2, chunk wave % 2) of every K-tile ---- */
	const unsigned char *wsrc = p.wp + ((size_t)mz * p.nkt) * 4096 + wave * 1024 + lane * 16;
	intx4 wr[3];
#define CP_WFETCH(SLOT_, KT_) (wr[SLOT_] = *(const intx4 *)(wsrc + (size_t)min((KT_), p.nkt - 1) * 4096))
#define CP_WSTORE(SLOT_, KT_) (*(intx4 *)(wst + ((KT_) % 3) * 4096 + wave * 1024 + lane * 16) = wr[SLOT_])

	/* ---- this lane's positions: tile nh * 3 + j, position n of it ---- */
	int pp0[3];
#pragma unroll
	for (int j = 0; j < 3; j++) {
		const int pos = min((nh * 3 + j) * 32 + n, npos - 1);
		const int ly = pos / p.cwl, lx = pos - ly * p.cwl;
		pp0[j] = ly * p.pw + lx;
	}
	const int vbase = (2 * kp + h) * CP_VP;	/* the vector plane this lane feeds to the matrix core */

	intx16 acc[2][3];
	int cs[3] = { 0, 0, 0 };
#pragma unroll
	for (int i = 0; i < 2; i++)
#pragma unroll
		for (int j = 0; j < 3; j++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[i][j][r] = 0;

	/* prologue: patch of block 0, weights of K-tiles 0 and 1 in LDS, 2..4 on their way */
	patch_fetch(0);
	CP_WFETCH(0, 0);
	CP_WFETCH(1, 1);
	CP_WFETCH(2, 2);
	if (tid < CP_PLANES) {
		const int m = mz * CP_PLANES + tid;
		rowterm[tid] = p.offB * p.rowsum[m] + p.K * p.offA * p.offB + p.c_off;	/* (wrapping, like the sum it joins) */
		rowadd[tid] = p.addend ? p.addend[m] : 0;
	}
	patch_store(0);
	CP_WSTORE(0, 0);
	CP_WSTORE(1, 1);
	CP_WFETCH(0, 3);
	CP_WFETCH(1, 4);
	/* ring: K-tile t + 2 is in slot (t + 2) % 3 when step t begins */

	const int nblocks = p.Ci / 64;
	/* the K-tile whose fragments are requested next: plane block, tap, its offset in the patch */
	int n_cb = 0, n_tap = 0, n_kh = 0, n_kw = 0;
	/* the K-tile being multiplied */
	int c_cb = 0, c_tap = 0, c_toff = 0;
	intx4 af[2][2], bf[2][3];
	auto frags = [&](int kt, intx4 (&a)[2], intx4 (&bb)[3]) {
		const unsigned char *ws = wst + (kt % 3) * 4096 + kp * 1024 + lane * 16;
#pragma unroll
		for (int i = 0; i < 2; i++)
			a[i] = *(const intx4 *)(ws + i * 2048);
		const unsigned char *pb = patch0 + (n_cb & 1) * (4 * CP_VP) + vbase + (n_kh * p.pw + n_kw) * 16;
#pragma unroll
		for (int j = 0; j < 3; j++)
			bb[j] = *(const intx4 *)(pb + pp0[j] * 16);
	};
	auto advance = [&]() {		/* current <- next, next <- the K-tile after it */
		c_cb = n_cb;
		c_tap = n_tap;
		c_toff = n_kh * p.pw + n_kw;
		if (++n_kw == p.kW) {
			n_kw = 0;
			++n_kh;
		}
		if (++n_tap == p.taps) {
			n_tap = n_kh = n_kw = 0;
			++n_cb;
		}
	};
	__syncthreads();
	frags(0, af[0], bf[0]);
	advance();
	auto step = [&](int kt, auto slot_, auto par_) {
		constexpr int slot = decltype(slot_)::value;	/* (kt + 2) % 3 */
		constexpr int par = decltype(par_)::value;	/* kt % 2: the register set that holds K-tile kt */
		__syncthreads();	/* K-tile kt + 1 (and a patch stored before) is in LDS; stage (kt + 2) % 3 is free */
		/* column sums: this tap's pixel of every position (lanes n and n + 32 twice the same);
		 * requested first and added last, so that nothing this K-tile's MFMAs need waits for LDS */
		int pst[3] = { 0, 0, 0 };
		if (kp == 0) {
			const int *ps = psum0 + (c_cb & 1) * CP_MAXPIX + c_toff;
#pragma unroll
			for (int j = 0; j < 3; j++)
				pst[j] = ps[pp0[j]];
		}
		if (kt + 1 < p.nkt)
			frags(kt + 1, af[par ^ 1], bf[par ^ 1]);	/* requested under this K-tile's MFMAs */
		/* pass K-tile kt + 2 on, request K-tile kt + 5; the next block's patch early in a block */
		CP_WSTORE(slot, kt + 2);
		CP_WFETCH(slot, kt + 5);
		if (c_tap == 0 && c_cb + 1 < nblocks)
			patch_fetch(c_cb + 1);
#pragma unroll
		for (int j = 0; j < 3; j++)
#pragma unroll
			for (int i = 0; i < 2; i++)
				acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[par][i], bf[par][j], acc[i][j], 0, 0, 0);
		if (c_tap == 2 && c_cb + 1 < nblocks)
			patch_store((c_cb + 1) & 1);
#pragma unroll
		for (int j = 0; j < 3; j++)
			cs[j] += pst[j];
		advance();
	};
	typedef std::integral_constant<int, 0> I0;
	typedef std::integral_constant<int, 1> I1;
	typedef std::integral_constant<int, 2> I2;
	int kt = 0;
	for (; kt + 5 < p.nkt; kt += 6) {
		step(kt, I2{}, I0{});
		step(kt + 1, I0{}, I1{});
		step(kt + 2, I1{}, I0{});
		step(kt + 3, I2{}, I1{});
		step(kt + 4, I0{}, I0{});
		step(kt + 5, I1{}, I1{});
	}
	if (kt < p.nkt)
		step(kt, I2{}, I0{});
	if (kt + 1 < p.nkt)
		step(kt + 1, I0{}, I1{});
	if (kt + 2 < p.nkt)
		step(kt + 2, I1{}, I0{});
	if (kt + 3 < p.nkt)
		step(kt + 3, I2{}, I1{});
	if (kt + 4 < p.nkt)
		step(kt + 4, I0{}, I0{});
#undef CP_WFETCH
#undef CP_WSTORE
	__syncthreads();	/* everybody is done with the patches and the weight stages */

	/* ---- the two chunks' sums: wavefront (kp, nh) keeps row half kp, gets it from (1 - kp, nh) ---- */
	{
		int *xch = (int *)lds;		/* [wave][3 tiles][16][64 lanes]: 12 KiB per wavefront */
		int *mine = xch + wave * (3 * 16 * 64);
#pragma unroll
		for (int j = 0; j < 3; j++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				mine[(j * 16 + r) * 64 + lane] = kp ? acc[0][j][r] : acc[1][j][r];	/* the half the other one keeps */
		int *csx = xch + 4 * (3 * 16 * 64) + wave * (3 * 64);
#pragma unroll
		for (int j = 0; j < 3; j++)
			csx[j * 64 + lane] = cs[j];
	}
	__syncthreads();
	{
		const int *xch = (const int *)lds;
		const int *other = xch + (wave ^ 2) * (3 * 16 * 64);
#pragma unroll
		for (int j = 0; j < 3; j++)
#pragma unroll
			for (int r = 0; r < 16; r++) {
				const int o = other[(j * 16 + r) * 64 + lane];
				if (kp)
					acc[1][j][r] += o;
				else
					acc[0][j][r] += o;
			}
		/* column sums: gathered by the wavefront (0, nh), per position */
		const int *cso = xch + 4 * (3 * 16 * 64);
#pragma unroll
		for (int j = 0; j < 3; j++)
			cs[j] = cso[(nh * 3 + j) * 64 + n];
	}
	__syncthreads();	/* the exchange area becomes the code buffer */

	/* ---- requantise: this wavefront's row half kp of its three position tiles ---- */
	unsigned char *cbuf = lds;	/* pooling: [position][64 planes], 16-byte pieces swapped around by the position */
	const int tail0 = (p.oH * p.oW / 8) * 8;	/* lowpadd's unclamped tail starts here */
	const bool has_add = p.addend != 0;
	const unsigned round = p.c_shift < 1 ? 0u : 1u << (p.c_shift - 1);
#pragma unroll
	for (int j = 0; j < 3; j++) {
		const int pos = (nh * 3 + j) * 32 + n;
		const int posc = min(pos, npos - 1);
		const int ly = posc / p.cwl, lx = posc - ly * p.cwl;
		const int rem = (row0 + ly) * p.oW + lx;
		const bool tail = has_add && rem >= tail0;
		const int colterm = p.offA * cs[j];
		unsigned word[4];
#pragma unroll
		for (int g = 0; g < 4; g++) {
			const int ml = kp * 32 + 8 * g + 4 * h;
			const intx4 rt = *(const intx4 *)(rowterm + ml), ra = *(const intx4 *)(rowadd + ml);
			unsigned packed = 0;
#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int a = kp ? acc[1][j][4 * g + e] : acc[0][j][4 * g + e];
				/* gemmlowp's output stage in wrapping int32 (c_off is in the row term) */
				const unsigned u = (unsigned)(a + rt[e] + colterm) * (unsigned)p.c_mult + round;
				int q = (int)u >> p.c_shift;
				q = q < 0 ? 0 : q > 255 ? 255 : q;
				const int sum = q + ra[e];	/* (no addend: 0, and the clamp changes nothing) */
				q = tail ? (sum > 255 ? 255 : (sum & 255)) : (sum < 0 ? 0 : sum > 255 ? 255 : sum);	/* lowp_SpatialConvolution.c:71-88 */
				if (p.act)
					q = q > p.ithr ? q : p.ival;
				packed |= (unsigned)q << (8 * e);
			}
			word[g] = packed;
		}
		/* lane (n, h) holds planes 8 g + 4 h .. + 3 of the row half; after the swaps lane n holds
		 * planes 0..15 and lane n + 32 planes 16..31 as 16 bytes */
		cp_swap32(word[0], word[1]);
		cp_swap32(word[2], word[3]);
		cp_swap32(word[0], word[2]);
		cp_swap32(word[1], word[3]);
		const uintx4 v = { word[0], word[1], word[2], word[3] };
		const int piece = 2 * kp + h;		/* which 16 of the 64 planes */
		if (pos < npos) {
			if (POOL)
				*(uintx4 *)(cbuf + posc * CP_PLANES + ((piece ^ (posc >> 2)) & 3) * 16) = v;
			else
				*(uintx4 *)(p.y + ((size_t)b * p.oH * p.oW + rem) * p.Co + mz * CP_PLANES + piece * 16) = v;
		}
	}
	if (!POOL)
		return;
	__syncthreads();
	/* ---- 3x3 / stride 2 maximum, sixteen planes per thread ---- */
	for (int it = tid; it < pra * p.pW * 4; it += CP_THREADS) {
		const int c16 = it & 3, t = it >> 2;
		const int prl = t / p.pW, pcl = t - prl * p.pW;
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

/* Geometry of a launch; returns 0 when the kernel does not take the layer. */
static int cp_plan(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int pool,
	ConvPatchParams *p)
{
	if (B < 1 || Ci < 64 || Ci % 64 || Co < 64 || Co % 64 || dH != 1 || dW != 1 || kH < 1 || kW < 1 || kH * kW < 4 ||
	    padH < 0 || padW < 0)
		return 0;	/* (fewer than four taps: the next block's patch would not be stored in time) */
	const int oW = W + 2 * padW - kW + 1, oH = H + 2 * padH - kH + 1;
	if (oW < 1 || oH < 1)
		return 0;
	int cwl = oW, rb, pH = 0, pW = 0;
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
		while (rb > 1 && (2 * rb + kH) * (cwl + kW - 1) > CP_MAXPIX)
			rb--;
		if ((2 * rb + kH) * (cwl + kW - 1) > CP_MAXPIX)
			return 0;
	} else {
		if (oW > CP_MAXPOS)
			return 0;
		rb = CP_MAXPOS / oW;
		if (rb > oH)
			rb = oH;
		while (rb > 1 && (rb + kH - 1) * (oW + kW - 1) > CP_MAXPIX)
			rb--;
		if ((rb + kH - 1) * (oW + kW - 1) > CP_MAXPIX)
			return 0;
	}
	if ((double)B * Ci * H * W >= 2147483000.0 || B > 65535 || Co / 64 > 65535)
		return 0;
	if (p) {
		p->B = B; p->Ci = Ci; p->H = H; p->W = W; p->Co = Co; p->kH = kH; p->kW = kW; p->padH = padH; p->padW = padW;
		p->oH = oH; p->oW = oW; p->pH = pH; p->pW = pW; p->pool = pool; p->rb = rb; p->cwl = cwl; p->pw = cwl + kW - 1;
		p->taps = kH * kW;
		p->nkt = Ci / 64 * kH * kW;
		p->K = Ci * kH * kW;
	}
	return 1;
}

/* Whether thhip_conv2d_u8_patch takes the layer (pool = 1: together with a 3x3 / stride 2
 * max pooling without padding in floor mode). */
extern "C" int thhip_conv2d_u8_patch_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pool)
{
	return cp_plan(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pool, 0);
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
	if (!cp_plan(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, pool, &p))
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
	ThhipLaunchScope scope(THHIP_FAM_CONV_I8, 2.0 * Co * (double)p.K * B * p.oH * p.oW);
	const dim3 grid(bands, Co / 64, B);
	if (pool)
		conv_u8_patch_kernel<true><<<grid, dim3(CP_THREADS), 0, thhip_stream()>>>(p);
	else
		conv_u8_patch_kernel<false><<<grid, dim3(CP_THREADS), 0, thhip_stream()>>>(p);
}
