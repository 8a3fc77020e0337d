/*
 * Half types (fp16 / bf16 storage, fp32 accumulation on the matrix cores):
 * 3x3 / stride 1 convolutions of channels-last tensors with every tap read from
 * one input patch in LDS.  The layer, its bias (and folded batch norm factor),
 * the Threshold and a 2x2 max pooling that follow are one kernel
 * (modules/SpatialConvolutionMM.c:126-225, modules/Threshold.c:38-63,
 * modules/SpatialMaxPooling.c:6-98; the half storage is the counterpart of the
 * reference's cudnn/cudnn_basic.c:208-218).
 */
#include <float.h>
#include <stdlib.h>
#include <string.h>
#include "conv_common.h"

/* With 64 input planes a K-tile of the generic kernels moves 64 bytes per
 * position from L2 for 32 multiply-adds per output plane, nine times per
 * pixel (once per tap), and the path from L2 to LDS, not the matrix core, sets
 * their time.  Here a workgroup owns 8 rows x 32 columns of one image's output,
 * copies the 10 x 34 pixel patch those positions read once per block of 32
 * planes (21 KiB, straight to LDS), and takes the B fragments of all nine taps
 * from it: a fragment of tap (kh, kw) is the patch shifted by (kh, kw).  Two
 * patch buffers, the next block's loads spread over the first steps of this one,
 * the weights (K-tiles of one tap x 32 planes) through a ring of NST stages, the
 * nine steps of a block straight-line code with constant wait counts.
 *
 * Patch layout: 1 KiB blocks of sixteen pixels x four 16-byte vectors, pixel pp
 * of the patch (row-major, 34 wide) in block pp / 16; vector v of pixel pp sits
 * in slot 4 pp + (v ^ ((pp / 4) % 4)).  A fragment read takes one vector index
 * from 32 consecutive pixels, sixteen lanes (256 bytes, every bank once) a cycle;
 * pixels four apart share their banks, and the swizzle gives any four such in a
 * run of sixteen four different slots, wherever the run starts.  Pixels outside
 * the image are fetched out of the buffer's range and arrive as zeros.
 *
 * Four waves; wave w computes all BM planes of tile rows 2w and 2w+1.
 *
 * A workgroup walks several tiles (tile l, l + n, l + 2n, ... of its XCD's run, n
 * workgroups per XCD) without draining the pipeline: the blocks of its tiles are
 * one sequence, so the first patch and weights of the next tile are fetched under
 * the last steps of this one and land while the results are stored.  (One tile per
 * workgroup and two workgroups per CU, started together, spent as long waiting for
 * their first patch and storing as multiplying: 64 -> 64 @224^2 kept the matrix
 * cores 44 % busy.)  The per-plane constants of every plane block sit in LDS from
 * the start, so that nothing the epilogue needs queues behind those loads.
 *
 * WHOLE: outputs of at most 14 x 14 (VGG-16's last three layers, ResNet's 14 x 14
 * ones), where 32 x 8 tiles would be three fifths empty: a workgroup takes a whole
 * image, its 16 x 16 patch (16 KiB per block of 32 planes) and 256 position slots,
 * wave w slots 64 w .. 64 w + 63.  Slot s is position s of the image in row-major
 * order; with the pooling, member s % 4 of window s / 4, so that a window's four
 * values sit in neighbouring lanes.  Slots past the last position compute pixel 0
 * again and store nothing.  With few images such a layer has few workgroups (batch
 * 16, 512 planes: 128 of 64 planes), so BM may be 32 here: then two of the four
 * waves' weight loads repeat the other two's (same bytes to the same place), which
 * keeps every wave's count of outstanding loads the same.
 *
 * STEM: the layer in front is the network's image layer (3 planes -> 64, 3x3 / stride 1 / padding 1, with its
 * factor, bias and Threshold), whose output would be written by one kernel only to be read back by this one
 * (128 bytes a pixel: 411 MB for a batch of 64 at 224 x 224).  Here a workgroup computes the two 32-plane
 * patches of a tile from the image instead of loading them: the 12 x 36 pixels of the three image planes
 * under the patch go to LDS (a fourth plane of zeros beside them), a wave takes blocks of 32 patch pixels,
 * builds its B operand from 24 two-byte reads at constant offsets (lane half h reads planes 2h and 2h + 1, so
 * that the halves differ by a constant: K = 2 x 18 taps in three chunks, packed that way by
 * thhip_conv_pack_weight_image_front), multiplies with the 64 x 48 weights kept in LDS, applies factor, bias
 * and Threshold, writes zeros for pixels outside the image (this layer's padding) and puts the rounded
 * values where the loads would have put them.  The image pixels of the next tile are requested before the
 * stores of this one.  Every tile then starts its own weight ring (the patch computation covers its latency). */
#define PATCH_ROWC 1024	/* output planes (in whole blocks) whose constants the kernel keeps in LDS */

template <int DT, bool CLO, int BM, int CI, bool POOL, bool WHOLE, bool STEM = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv_patch_kernel(ConvParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)	/* as for conv_wide_kernel: the host pass gets the stub only */
	typedef ConvTraits<DT> TR;
	typedef typename TR::elem elem;
	static_assert(TR::CHUNK == 16 && sizeof(elem) == 2, "a half type");
	constexpr int TW = WHOLE ? 14 : PATCH_TW, TH = WHOLE ? 14 : PATCH_TH, PW = TW + 2, PH = TH + 2, PCI = 32, NB = CI / PCI;
	constexpr int NPIX = PW * PH, WAVES = 4;
	constexpr int BL = ((NPIX + 15) / 16 + WAVES - 1) / WAVES;	/* patch loads (sixteen pixels x four vectors) per wave and block */
	constexpr int B_VECS = STEM ? 22 * 64 : BL * WAVES * 64;	/* a buffer: every load's 1 KiB, the unused ones' too (STEM: 22 blocks of 16 pixels) */
	constexpr int MB = BM / 32, TM = MB, TN = 2, KCH = 2, NST = WHOLE ? 9 : 6;	/* NST: weight stages */
	constexpr int A_VECS = MB * KCH * 64, A_PW = (MB * KCH + WAVES - 1) / WAVES;
	static_assert(CI % (2 * PCI) == 0 && (MB * KCH % WAVES == 0 || WAVES % (MB * KCH) == 0) && (WHOLE || TH == 2 * WAVES) && BL <= 8, "shape");
	static_assert(!WHOLE || (NPIX == 256 && WAVES * TN * 32 == 256), "a whole image: 256 patch pixels, 256 position slots");
	static_assert(18 % NST == 0 && NST >= 3, "K-tile k of a pair of blocks in stage k % NST");
	/* Walking several tiles pays with 64 input planes, where a tile's eighteen steps are as long as its first
	 * loads and its stores (64 -> 64 @224^2 with the pooling, batch 64: 264 -> 241 us; 64 -> 128 @112^2:
	 * 167 -> 156 us); longer K loops lose more to the fixed tile order than they gain (3-7 %) and take one
	 * tile per workgroup, which the dispatcher hands to the CUs as they come free. */
	constexpr bool WALK = CI == 64;
	constexpr int ROWC = STEM ? 256 : WALK ? PATCH_ROWC : BM;	/* planes whose constants sit in LDS */
	static_assert(!STEM || (CI == 64 && !WHOLE && BM == 64), "the image layer in front: 64 planes into 32 x 8 tiles");
	/* STEM: the image patch (four planes of 12 x 36 halfs), the image layer's weights (2 x 3 fragments of 1 KiB) and constants */
	constexpr int IMG_ROWS = PH + 2, IMG_W = PW + 2, IMG_PLANE = IMG_ROWS * IMG_W;
	constexpr int IMG_VECS = (4 * IMG_PLANE * 2 + 15) / 16, WST_VECS = 2 * 3 * 64, SC_VECS = 2 * 64 / 4;
	/* (one array, every stage and buffer at a constant offset: conv_f32_patch_kernel says why) */
	__shared__ floatx4 lds[NST * A_VECS + 2 * B_VECS + 2 * ROWC / 4 + (STEM ? IMG_VECS + WST_VECS + SC_VECS : 0)];
	floatx4 *const astage = lds;
	floatx4 *const patch0 = lds + NST * A_VECS, *const patch1 = patch0 + B_VECS;
	float *const rowc = (float *)(patch1 + B_VECS);	/* bias[ROWC], factor[ROWC] */
	unsigned short *const imgl = (unsigned short *)(rowc + 2 * ROWC);	/* (STEM) */
	floatx4 *const wstl = (floatx4 *)imgl + IMG_VECS;
	float *const stemc = (float *)(wstl + WST_VECS);

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

	/* ---- this workgroup's tiles: number local0, local0 + nloc, ... of its XCD's.  32 x 8 tiles: consecutive
	 * tiles (plane block fastest, then along the row) share halo pixels, each XCD takes one run of them.
	 * WHOLE: every XCD a rectangle of the (plane block, image) grid, mparts x 8 / mparts of them; its
	 * workgroups run side by side and share the rectangle's weights and images through its L2. ---- */
	const int tx_n = (p.oW + TW - 1) / TW, ty_n = (p.oH + TH - 1) / TH;
	const int xcd = blockIdx.x & 7, nloc = gridDim.x >> 3;
	int first, cnt, mw = 1, m0 = 0, n0 = 0;
	if constexpr (WHOLE) {
		const int mp = xcd % p.mparts, np = xcd / p.mparts, nparts = 8 / p.mparts;
		m0 = p.tiles_m * mp / p.mparts;
		mw = p.tiles_m * (mp + 1) / p.mparts - m0;
		n0 = p.tiles_n * np / nparts;
		cnt = mw * (p.tiles_n * (np + 1) / nparts - n0);
		first = 0;
	} else {
		const int total = p.tiles_m * p.tiles_n, per_xcd = (total + 7) / 8;
		first = xcd * per_xcd;
		cnt = min(per_xcd, total - first);
	}
	struct Tile { int tile_m, tx, ty, img; bool ok; };
	auto decode = [&](int local) {
		Tile T;
		T.ok = local < cnt;
		const int l = T.ok ? local : 0;
		if constexpr (WHOLE) {
			T.tile_m = m0 + l % mw;
			T.img = n0 + l / mw;
			T.tx = T.ty = 0;
		} else {
			const int t = first + l;
			T.tile_m = t % p.tiles_m;
			const int sp = t / p.tiles_m;
			T.tx = sp % tx_n;
			T.ty = (sp / tx_n) % ty_n;
			T.img = sp / (tx_n * ty_n);
		}
		return T;
	};
	int nlocal = blockIdx.x >> 3;
	Tile cur = decode(nlocal);
	if (!cur.ok)
		return;
	nlocal += nloc;
	Tile nxt = decode(nlocal);
	if constexpr (!WALK)
		nxt.ok = false;

	const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes, 0x00020000);
	const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.wp, 0, p.w_bytes, 0x00020000);
	/* ---- what this lane fetches of every block of 32 planes of a tile: load t of the wave covers pixels
	 * 16 (wave + 4 t) .. + 15 of the patch, this lane pixel lane / 4 of them, vector lane % 4 through the
	 * swizzle; and the wave's weight blocks of a K-tile: wave + 4 i counts (chunk, 32-row block).  Of a
	 * tile that does not exist everything is out of range (and arrives as zeros). ---- */
	int a_lds_[A_PW];
#pragma unroll
	for (int i = 0; i < A_PW; i++) {
		const int idx = (wave + WAVES * i) % (MB * KCH);
		a_lds_[i] = ((idx / MB) * MB + idx % MB) * 64;
	}
	auto offsets = [&](const Tile &T, unsigned (&voff)[BL], unsigned (&aoff)[A_PW]) {
#pragma unroll
		for (int t = 0; t < BL; t++) {
			const int pp = (wave + WAVES * t) * 16 + (lane >> 2);
			const int v = (lane & 3) ^ ((pp >> 2) & 3);
			const int pr = pp / PW, pc = pp - pr * PW;
			const int iy = T.ty * TH - p.padH + pr, ix = T.tx * TW - p.padW + pc;
			const bool ok = T.ok && pp < NPIX && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
			voff[t] = ok ? (unsigned)((((T.img * p.H + iy) * p.W + ix) * CI + v * 8) * (int)sizeof(elem)) : 0x80000000u;
		}
#pragma unroll
		for (int i = 0; i < A_PW; i++) {
			const int idx = (wave + WAVES * i) % (MB * KCH), mbi = idx % MB, kci = idx / MB;
			aoff[i] = ((unsigned)(T.tile_m * MB + mbi) * (unsigned)p.KC + kci) * 1024u;
		}
	};
	unsigned voff_[BL], voffn_[BL], a_off_[A_PW], a_offn_[A_PW];
	offsets(cur, voff_, a_off_);
	offsets(nxt, voffn_, a_offn_);

	/* the weights of K-tile (block hb of 32 planes, tap): K runs (block, tap, plane) in chunks of 16.
	 * Block NB is block 0 of the next tile. */
	auto issue_a = [&](auto st_, int hb, int tap) {
		constexpr int st = decltype(st_)::value;
		const bool here = hb < NB;
		const unsigned kc = (unsigned)(((here || !WALK ? hb : 0) * 9 + tap) * KCH);
#pragma unroll
		for (int i = 0; i < A_PW; i++)
			__builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, WIDE_LDS(astage + st * A_VECS + a_lds_[i]), 16,
				here || (WALK && !STEM && nxt.ok) ? lane * 16 : 0x80000000u, (here || !WALK ? a_off_[i] : a_offn_[i]) + kc * 1024u, 0, 0);
	};
	auto issue_b = [&](auto t_, int hb, auto buf_) {
		constexpr int buf = decltype(buf_)::value, t = decltype(t_)::value;
		const bool here = hb < NB;
		if constexpr (WALK)
			__builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, WIDE_LDS((buf ? patch1 : patch0) + (wave + WAVES * t) * 64), 16,
				here ? voff_[t] : voffn_[t], here ? hb * PCI * (int)sizeof(elem) : 0, 0, 0);
		else
			__builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, WIDE_LDS((buf ? patch1 : patch0) + (wave + WAVES * t) * 64), 16,
				here ? voff_[t] : 0x80000000u, here ? hb * PCI * (int)sizeof(elem) : 0, 0, 0);
	};

	/* patch pixel of this lane's position at tap (0, 0), for its two tile rows */
	int pbase_[TN];
	int oy_[TN], ox_[TN];	/* WHOLE: the slot's output position (pooling: of its window member), -1: none */
#pragma unroll
	for (int j = 0; j < TN; j++) {
		if constexpr (WHOLE) {
			const int s = (wave * TN + j) * 32 + (lane & 31);
			int r, c;
			bool live;
			if constexpr (POOL) {
				const int pW = p.oW / 2, wd = s >> 2, wr = wd / pW, wc = wd - wr * pW;
				r = 2 * wr + ((s >> 1) & 1);
				c = 2 * wc + (s & 1);
				live = wd < p.pHW;
			} else {
				r = s / p.oW;
				c = s - r * p.oW;
				live = s < p.oHW;
			}
			oy_[j] = live ? r : -1;
			ox_[j] = live ? c : 0;
			pbase_[j] = live ? r * PW + c : 0;
		} else {
			pbase_[j] = (2 * wave + j) * PW + (lane & 31);
			oy_[j] = ox_[j] = 0;
		}
	}
	/* four fragment sets: two chunks each of this K-tile and the next (below) */
	floatx4 af[4][TM], bf[4][TN];
	auto read_frags = [&](auto st_, auto buf_, auto tap_, int c, floatx4 (&a)[TM], floatx4 (&b)[TN]) {
		constexpr int st = decltype(st_)::value, buf = decltype(buf_)::value, tap = decltype(tap_)::value;
		const floatx4 *la = astage + st * A_VECS;
#pragma unroll
		for (int i = 0; i < TM; i++)
			a[i] = la[(c * MB + i) * 64 + lane];
		const int v = c * 2 + (lane >> 5);
#pragma unroll
		for (int j = 0; j < TN; j++) {
			const int pp = pbase_[j] + (tap / 3) * PW + tap % 3;
			b[j] = (buf ? patch1 : patch0)[pp * 4 + (v ^ ((pp >> 2) & 3))];
		}
	};

	typename ConvAcc<DT>::T acc[TM][TN];
	auto clear = [&]() {
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					acc[i][j][r] = 0;
	};
	clear();
	auto mma = [&](int set) {
#pragma unroll
		for (int i = 0; i < TM; i++)
#pragma unroll
			for (int j = 0; j < TN; j++)
				conv_mma<DT>(acc[i][j], af[set][i], bf[set][j]);
	};

	typedef std::integral_constant<int, 0> C0;
	typedef std::integral_constant<int, 1> C1;
	/* patch loads of the next block: one in each of the first BL steps of this one (step `tap` issues
	 * numbers [PB(tap), PB(tap + 1))) */
#define CONV_PATCH_PB(tap) (STEM ? 0 : (tap) < BL ? (tap) : BL)
#define CONV_PATCH_NB(tap) (CONV_PATCH_PB(((tap) + 9) % 9 + 1) - CONV_PATCH_PB(((tap) + 9) % 9))
	/* The pipeline.  A wave with the SIMD to itself gets what it asks of LDS before a group of MFMAs only
	 * after them, so the fragments of a K-tile are fetched a whole step ahead, into four register sets.
	 * Step t (K-tile t of the workgroup's sequence, tap t % 9) starts with the wait and the barrier: K-tile
	 * t + 1 is in LDS, and every wave has issued the MFMAs of K-tile t - 1, whose stage the weights of K-tile
	 * t - 1 + NST now overwrite; then it alternates the reads of K-tile t + 1 with the MFMAs of K-tile t.
	 * The loads of a wave complete in the order of their issue, and a wait names how many of the latest may
	 * still be outstanding: the weights of K-tile t + 1 were issued in step t + 2 - NST, what steps
	 * t + 3 - NST .. t - 1 issued may be; the step that reads the next patch's first fragments (tap 8) needs
	 * that patch too, whose last load step BL - 1 issued before its weights.  The prologue issues what
	 * steps -9 .. -1 would have, in their order, so the counts hold from the first step.  (Stores count as
	 * loads do: after an epilogue the first steps of the next tile wait for most of its stores as well.) */
	constexpr auto allowed = [](int tap) {
		int n = 0;
		for (int t = tap + 3 - NST; t <= tap - 1; t++)
			n += A_PW + CONV_PATCH_NB(t + 18);
		if (tap == 8 && !STEM) {
			const int np = (8 - (BL - 1)) * A_PW;
			n = n < np ? n : np;
		}
		return n;
	};
	/* what steps -9 .. -1 would have issued: the first patch, the weights of K-tiles 0 .. NST - 2 */
	auto ring_start = [&]() {
		auto virt = [&](auto self, auto v_) {
			constexpr int v = decltype(v_)::value;	/* step v - 9, tap v */
			if constexpr (v < 9) {
				if constexpr (CONV_PATCH_NB(v) >= 1)
					issue_b(std::integral_constant<int, CONV_PATCH_PB(v)>{}, 0, C0{});
				if constexpr (v - 10 + NST >= 0)
					issue_a(std::integral_constant<int, v - 10 + NST>{}, 0, v - 10 + NST);
				self(self, std::integral_constant<int, v + 1>{});
			}
		};
		virt(virt, C0{});
	};
	/* ... and once the patch (its last load: step BL - 10) and K-tile 0 (step 1 - NST) are there (what the steps
	 * after both issued may be outstanding), the first fragments */
	auto ring_first = [&]() {
		wide_wait<(!STEM && BL - 10 > 1 - NST ? 10 - BL : NST - 2) * A_PW, true>();
		__builtin_amdgcn_s_barrier();
		read_frags(C0{}, C0{}, C0{}, 0, af[0], bf[0]);
		read_frags(C0{}, C0{}, C0{}, 1, af[1], bf[1]);
	};
	/* the per-plane constants of every plane block, or of this tile's if it is the only one (behind the
	 * first loads: they are waited for anyway) */
	auto fill_rowc = [&]() {
		const int row0 = WALK ? 0 : cur.tile_m * BM;
		for (int i = tid; i < (WALK ? p.tiles_m * BM : BM); i += 256) {
			const int mc = min(row0 + i, p.Co - 1);
			rowc[i] = p.bias ? p.bias[mc] : 0.0f;
			rowc[ROWC + i] = p.scale ? p.scale[mc] : 1.0f;
		}
	};

	/* ---- STEM: the image pixels a tile's patch is computed from, three dwords a thread ---- */
	const __amdgpu_buffer_rsrc_t irsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(STEM ? p.img : p.x), 0, STEM ? p.img_bytes : 0, 0x00020000);
	unsigned imgv[3];
	auto image_request = [&](const Tile &T) {
#pragma unroll
		for (int u = 0; u < 3; u++) {
			const int idx = tid + 256 * u, c = idx / (IMG_ROWS * (IMG_W / 2)), r = (idx / (IMG_W / 2)) % IMG_ROWS, d = idx % (IMG_W / 2);
			const int iy = T.ty * TH - p.padH - 1 + r, ix = T.tx * TW - p.padW - 1 + 2 * d;
			const bool ok = c < 3 && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
			imgv[u] = __builtin_amdgcn_raw_buffer_load_b32(irsrc, ok ? (((T.img * 3 + c) * p.H + iy) * p.W + ix) * 2 : (int)0x80000000, 0, 0);
		}
	};
	/* A tile's start with the image layer in front: image pixels to LDS, the weight ring started, the two
	 * patches computed, the first fragments read. */
	auto stem_tile = [&](const Tile &T) {
#pragma unroll
		for (int u = 0; u < 3; u++) {
			const int idx = tid + 256 * u;
			if (idx < 3 * IMG_ROWS * (IMG_W / 2))
				((unsigned *)imgl)[idx] = imgv[u];
		}
		wide_wait<48, true>();	/* (the LDS writes; every wave is past its last tile's reads of stages and patches) */
		__builtin_amdgcn_s_barrier();
		ring_start();
		/* Three blocks of 32 patch pixels a wave (the last wave: two).  Everything the blocks read from LDS is
		 * requested before the first MFMA -- the other workgroup of the CU keeps LDS busy with its K loop, and
		 * a wave that asks for a block's operands, waits, multiplies, asks for the constants, waits, ... spent
		 * 12 000 cycles here where its instructions need 2 000. */
		const int n = lane & 31, h = lane >> 5;
		constexpr int NBW = ((NPIX + 31) / 32 + WAVES - 1) / WAVES;
		uintx4 bw[NBW][3];
		int pp_[NBW];
		bool inside_[NBW];
#pragma unroll
		for (int t = 0; t < NBW; t++) {
			const int pp = (wave + WAVES * t) * 32 + n, ppc = min(pp, NPIX - 1);
			const int pr = ppc / PW, pc = ppc - pr * PW;
			const unsigned short *src = imgl + pr * IMG_W + pc + h * (2 * IMG_PLANE);
#pragma unroll
			for (int sc = 0; sc < 3; sc++)
#pragma unroll
				for (int d = 0; d < 4; d++) {
					unsigned two[2];
#pragma unroll
					for (int e = 0; e < 2; e++) {
						const int j = 8 * sc + 2 * d + e;	/* tap j of this lane half's two planes: (plane, kh, kw) = (j / 9, j % 9 / 3, j % 3) */
						two[e] = src[j < 18 ? ((j / 9) * IMG_ROWS + (j % 9) / 3) * IMG_W + j % 3 : 0];
					}
					bw[t][sc][d] = two[0] | (two[1] << 16);
				}
			const int iy = T.ty * TH - p.padH + pr, ix = T.tx * TW - p.padW + pc;
			pp_[t] = pp;
			inside_[t] = pp < NPIX && (unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W;
		}
		const bool relu = p.sact && p.sthr == 0.0f && p.sval == 0.0f;
#pragma unroll
		for (int mb = 0; mb < 2; mb++) {
			floatx4 wa[3], rb[4], rs[4];
#pragma unroll
			for (int sc = 0; sc < 3; sc++)
				wa[sc] = wstl[(mb * 3 + sc) * 64 + lane];
#pragma unroll
			for (int g = 0; g < 4; g++) {
				const int ml = mb * 32 + 8 * g + 4 * h;
				rb[g] = *(const floatx4 *)(stemc + ml);
				rs[g] = *(const floatx4 *)(stemc + 64 + ml);
			}
			floatx16 sacc[NBW];
#pragma unroll
			for (int t = 0; t < NBW; t++)
#pragma unroll
				for (int r = 0; r < 16; r++)
					sacc[t][r] = 0.0f;
#pragma unroll
			for (int sc = 0; sc < 3; sc++)
#pragma unroll
				for (int t = 0; t < NBW; t++)
					conv_mma<DT>(sacc[t], wa[sc], __builtin_bit_cast(floatx4, bw[t][sc]));
			/* register 4 g + e of block mb is plane 32 mb + 8 g + 4 h + e of pixel pp: half of vector g */
#pragma unroll
			for (int t = 0; t < NBW; t++) {
				if (wave + WAVES * t >= (NPIX + 31) / 32)
					continue;	/* (the last wave's third block does not exist) */
				const int pp = pp_[t];
				const bool inside = inside_[t];
#pragma unroll
				for (int g = 0; g < 4; g++) {
					char *const dst = (char *)(mb ? patch1 : patch0) + (4 * pp + (g ^ ((pp >> 2) & 3))) * 16 + 8 * h;
					if (relu) {
						/* on packed pairs: a ReLU of rounded values is an integer maximum with zero */
						typedef short shortx2 __attribute__((ext_vector_type(2)));
						typedef elem elemx2 __attribute__((ext_vector_type(2)));
						uintx2 out;
#pragma unroll
						for (int e2 = 0; e2 < 2; e2++) {
							const elemx2 v = { (elem)__builtin_fmaf(sacc[t][4 * g + 2 * e2], rs[g][2 * e2], rb[g][2 * e2]),
								(elem)__builtin_fmaf(sacc[t][4 * g + 2 * e2 + 1], rs[g][2 * e2 + 1], rb[g][2 * e2 + 1]) };
							const shortx2 zero = { 0, 0 };
							const unsigned u = __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(shortx2, v), zero));
							out[e2] = inside ? u : 0u;
						}
						*(uintx2 *)dst = out;
					} else {
						struct alignas(8) Quad { elem v[4]; } quad;
#pragma unroll
						for (int e = 0; e < 4; e++) {
							float v = __builtin_fmaf(sacc[t][4 * g + e], rs[g][e], rb[g][e]);
							if (p.sact)
								v = v > p.sthr ? v : p.sval;
							quad.v[e] = inside ? (elem)v : (elem)0.0f;
						}
						*(Quad *)dst = quad;
					}
				}
			}
		}
		ring_first();
	};
	if constexpr (STEM) {
		for (int i = tid; i < WST_VECS; i += 256)
			wstl[i] = ((const floatx4 *)p.wstem)[i];
		if (tid < 64) {
			stemc[tid] = p.sbias ? p.sbias[tid] : 0.0f;
			stemc[64 + tid] = p.sscale ? p.sscale[tid] : 1.0f;
		}
		for (int i = tid; i < IMG_PLANE / 2; i += 256)
			((unsigned *)imgl)[3 * IMG_PLANE / 2 + i] = 0;	/* the fourth plane */
		image_request(cur);
		fill_rowc();
	} else {
		ring_start();
		fill_rowc();
		ring_first();
	}
	auto step = [&](int hb, auto buf_, auto tap_) {
		constexpr int tap = decltype(tap_)::value, buf = decltype(buf_)::value;
		constexpr int par = (tap + buf) & 1;
		typedef std::integral_constant<int, (9 * buf + tap + 1) % NST> ST1;
		typedef std::integral_constant<int, (9 * buf + tap + NST - 1) % NST> STP;
		typedef std::integral_constant<int, (tap + 1) % 9> TAP1;
		typedef std::integral_constant<int, buf ^ 1> OTHER;
		typedef std::integral_constant<int, tap == 8 ? buf ^ 1 : buf> BUF1;
		wide_wait<allowed(tap), false>();
		__builtin_amdgcn_s_barrier();
		if constexpr (CONV_PATCH_NB(tap) >= 1)
			issue_b(std::integral_constant<int, CONV_PATCH_PB(tap)>{}, hb + 1, OTHER{});
		issue_a(STP{}, hb + (tap + NST - 1) / 9, (tap + NST - 1) % 9);
		read_frags(ST1{}, BUF1{}, TAP1{}, 0, af[2 * (par ^ 1)], bf[2 * (par ^ 1)]);
		__builtin_amdgcn_sched_barrier(0);	/* (the fragments are asked for before the MFMAs that follow in the source) */
		mma(2 * par);
		read_frags(ST1{}, BUF1{}, TAP1{}, 1, af[2 * (par ^ 1) + 1], bf[2 * (par ^ 1) + 1]);
		__builtin_amdgcn_sched_barrier(0);
		mma(2 * par + 1);
	};
#undef CONV_PATCH_NB
#undef CONV_PATCH_PB
	auto block = [&](int hb, auto buf_) {
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

	/* ---- (factor,) bias, Threshold, (pooling,) store of a finished tile ---- */
	elem *y = (elem *)p.y;
	auto store_tile = [&](const Tile &T) {
		const float *lrow = rowc + (WALK ? T.tile_m * BM : 0);
		/* The usual case, channels-last output after a ReLU (Threshold(0, 0)), on packed pairs: a rounded
		 * value at or above zero orders as its bits do, and a negative one is a negative 16-bit integer, so
		 * the pooling is an integer maximum and the ReLU one more against zero afterwards (the results are
		 * those of the general code below; a finished tile costs a quarter of its instructions, which with
		 * 64 input planes was two fifths of a tile's time).  The two lanes of a position then exchange groups
		 * and each writes 16 bytes (conv_store_cl_half). */
		if constexpr (CLO) {
			if (p.act && p.thr == 0.0f && p.val == 0.0f && p.Co % 8 == 0) {
				typedef short shortx2 __attribute__((ext_vector_type(2)));
				typedef elem elemx2 __attribute__((ext_vector_type(2)));
				auto pack2 = [](float a, float b) {
					const elemx2 v = { (elem)a, (elem)b };
					return __builtin_bit_cast(unsigned, v);
				};
				auto max2 = [](unsigned a, unsigned b) {
					return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(shortx2, a), __builtin_bit_cast(shortx2, b)));
				};
				/* accumulator i of tile row / slot block j as eight packed pairs: lo[g], hi[g] = planes 0..1, 2..3 of group g */
				auto packed = [&](int i, int j, unsigned (&lo)[4], unsigned (&hi)[4]) {
#pragma unroll
					for (int g = 0; g < 4; g++) {
						const int ml = i * 32 + 4 * (lane >> 5) + 8 * g;
						const floatx4 rb = *(const floatx4 *)(lrow + ml), rs = *(const floatx4 *)(lrow + ROWC + ml);
						lo[g] = pack2(__builtin_fmaf(acc[i][j][4 * g], rs[0], rb[0]), __builtin_fmaf(acc[i][j][4 * g + 1], rs[1], rb[1]));
						hi[g] = pack2(__builtin_fmaf(acc[i][j][4 * g + 2], rs[2], rb[2]), __builtin_fmaf(acc[i][j][4 * g + 3], rs[3], rb[3]));
					}
				};
				unsigned short *const yh = (unsigned short *)y;
#pragma unroll
				for (int i = 0; i < TM; i++) {
					const int mt = T.tile_m * BM + i * 32;
					if constexpr (POOL && WHOLE) {
						const int pH = p.oH / 2, pW = p.oW / 2;
#pragma unroll
						for (int j = 0; j < TN; j++) {
							unsigned lo[4], hi[4];
							packed(i, j, lo, hi);
#pragma unroll
							for (int g = 0; g < 4; g++) {
								lo[g] = max2(lo[g], (unsigned)__builtin_amdgcn_update_dpp(0, (int)lo[g], 0xB1, 0xF, 0xF, false));
								hi[g] = max2(hi[g], (unsigned)__builtin_amdgcn_update_dpp(0, (int)hi[g], 0xB1, 0xF, 0xF, false));
								lo[g] = max2(max2(lo[g], (unsigned)__builtin_amdgcn_update_dpp(0, (int)lo[g], 0x4E, 0xF, 0xF, false)), 0u);
								hi[g] = max2(max2(hi[g], (unsigned)__builtin_amdgcn_update_dpp(0, (int)hi[g], 0x4E, 0xF, 0xF, false)), 0u);
							}
							const int py = oy_[j] >> 1, px = ox_[j] >> 1;
							const size_t n = ((size_t)T.img * pH + py) * pW + px;
							conv_store_cl_half(yh + n * p.Co + mt, p.Co - mt, !(lane & 3) && oy_[j] >= 0, lo, hi, lane);
						}
					} else if constexpr (POOL) {
						const int pH = p.oH / 2, pW = p.oW / 2;
						const int py = T.ty * (TH / 2) + wave, px = T.tx * (TW / 2) + ((lane & 31) >> 1);
						const size_t n = ((size_t)T.img * pH + py) * pW + px;
						unsigned lo[4], hi[4], lo1[4], hi1[4];
						packed(i, 0, lo, hi);
						packed(i, 1, lo1, hi1);
#pragma unroll
						for (int g = 0; g < 4; g++) {
							lo[g] = max2(lo[g], lo1[g]);
							hi[g] = max2(hi[g], hi1[g]);
							lo[g] = max2(max2(lo[g], (unsigned)__builtin_amdgcn_update_dpp(0, (int)lo[g], 0xB1, 0xF, 0xF, false)), 0u);
							hi[g] = max2(max2(hi[g], (unsigned)__builtin_amdgcn_update_dpp(0, (int)hi[g], 0xB1, 0xF, 0xF, false)), 0u);
						}
						conv_store_cl_half(yh + n * p.Co + mt, p.Co - mt, !(lane & 1) && py < pH && px < pW, lo, hi, lane);
					} else {
#pragma unroll
						for (int j = 0; j < TN; j++) {
							const int oy = WHOLE ? oy_[j] : T.ty * TH + 2 * wave + j, ox = WHOLE ? ox_[j] : T.tx * TW + (lane & 31);
							const bool valid = oy >= 0 && oy < p.oH && ox < p.oW;
							const size_t n = (size_t)T.img * p.oHW + (valid ? oy * p.oW + ox : 0);
							unsigned lo[4], hi[4];
							packed(i, j, lo, hi);
#pragma unroll
							for (int g = 0; g < 4; g++) {
								lo[g] = max2(lo[g], 0u);
								hi[g] = max2(hi[g], 0u);
							}
							conv_store_cl_half(yh + n * p.Co + mt, p.Co - mt, valid, lo, hi, lane);
						}
					}
				}
				return;
			}
		}
		/* (one fused multiply-add in both forms of the epilogue: they must round alike; the factor is 1 without a batch norm) */
		auto finish = [&](float a, float s, float b) {
			float v = __builtin_fmaf(a, s, b);
			if (p.act)
				v = v > p.thr ? v : p.val;
			return v;
		};
		if constexpr (POOL && WHOLE) {
			/* a window's four members in four neighbouring lanes; the first one stores */
			const int pH = p.oH / 2, pW = p.oW / 2;
#pragma unroll
			for (int j = 0; j < TN; j++) {
				const int py = oy_[j] >> 1, px = ox_[j] >> 1;
				const bool store = !(lane & 3) && oy_[j] >= 0;
				const size_t n = ((size_t)T.img * pH + py) * pW + px;
				const size_t ybase = (size_t)T.img * p.Co * pH * pW + (size_t)py * pW + px;
#pragma unroll
				for (int i = 0; i < TM; i++) {
					const int m0 = T.tile_m * BM + i * 32 + 4 * (lane >> 5);
#pragma unroll
					for (int g = 0; g < 4; g++) {
						struct alignas(4 * sizeof(elem)) Quad { elem v[4]; } quad;
						const int ml = i * 32 + 4 * (lane >> 5) + 8 * g;
						const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
						const floatx4 rowscale = *(const floatx4 *)(lrow + ROWC + ml);
#pragma unroll
						for (int e = 0; e < 4; e++) {
							const int m = m0 + 8 * g + e;
							float v = finish(acc[i][j][4 * g + e], rowscale[e], rowbias[e]);
							v = (float)(elem)v;	/* the pooling compares the stored (rounded) values */
							v = fmaxf(v, __shfl_xor(v, 1));
							v = fmaxf(v, __shfl_xor(v, 2));
							if constexpr (!CLO) {
								if (store && m < p.Co)
									y[ybase + (size_t)m * pH * pW] = (elem)v;
							}
							quad.v[e] = (elem)v;
						}
						if constexpr (CLO) {
							if (store && m0 + 8 * g < p.Co)
								*(Quad *)(y + n * p.Co + m0 + 8 * g) = quad;
						}
					}
				}
			}
		} else if constexpr (POOL) {
			/* The 2x2 / stride 2 max pooling that follows, here: the two rows of a
			 * window are this wave's two tile rows (the same accumulator index), its
			 * two columns neighbouring lanes.  Threshold first, as the modules run. */
			const int pH = p.oH / 2, pW = p.oW / 2;
			const int py = T.ty * (TH / 2) + wave, px = T.tx * (TW / 2) + ((lane & 31) >> 1);
			const bool store = !(lane & 1) && py < pH && px < pW;
			const size_t n = ((size_t)T.img * pH + py) * pW + px;
			const size_t ybase = (size_t)T.img * p.Co * pH * pW + (size_t)py * pW + px;
#pragma unroll
			for (int i = 0; i < TM; i++) {
				const int m0 = T.tile_m * BM + i * 32 + 4 * (lane >> 5);
#pragma unroll
				for (int g = 0; g < 4; g++) {
					struct alignas(4 * sizeof(elem)) Quad { elem v[4]; } quad;
					const int ml = i * 32 + 4 * (lane >> 5) + 8 * g;
					const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
					const floatx4 rowscale = *(const floatx4 *)(lrow + ROWC + ml);
#pragma unroll
					for (int e = 0; e < 4; e++) {
						const int m = m0 + 8 * g + e;
						const float v0 = finish(acc[i][0][4 * g + e], rowscale[e], rowbias[e]);
						const float v1 = finish(acc[i][1][4 * g + e], rowscale[e], rowbias[e]);
						/* the pooling compares the stored (rounded) values */
						float v = fmaxf((float)(elem)v0, (float)(elem)v1);
						v = fmaxf(v, __shfl_xor(v, 1));
						if constexpr (!CLO) {
							if (store && m < p.Co)
								y[ybase + (size_t)m * pH * pW] = (elem)v;
						}
						quad.v[e] = (elem)v;
					}
					if constexpr (CLO) {
						if (store && m0 + 8 * g < p.Co)
							*(Quad *)(y + n * p.Co + m0 + 8 * g) = quad;
					}
				}
			}
		} else {
#pragma unroll
			for (int j = 0; j < TN; j++) {
				const int oy = WHOLE ? oy_[j] : T.ty * TH + 2 * wave + j, ox = WHOLE ? ox_[j] : T.tx * TW + (lane & 31);
				if (oy < 0 || oy >= p.oH || ox >= p.oW)
					continue;
				const int rem = oy * p.oW + ox;
				const size_t n = (size_t)T.img * p.oHW + rem;
				const size_t ybase = (size_t)T.img * p.Co * p.oHW + rem;
#pragma unroll
				for (int i = 0; i < TM; i++) {
					const int m0 = T.tile_m * BM + i * 32 + 4 * (lane >> 5);
#pragma unroll
					for (int g = 0; g < 4; g++) {
						struct alignas(4 * sizeof(elem)) Quad { elem v[4]; } quad;
						const int ml = i * 32 + 4 * (lane >> 5) + 8 * g;
						const floatx4 rowbias = *(const floatx4 *)(lrow + ml);
						const floatx4 rowscale = *(const floatx4 *)(lrow + ROWC + ml);
#pragma unroll
						for (int e = 0; e < 4; e++) {
							const int m = m0 + 8 * g + e;
							const float v = finish(acc[i][j][4 * g + e], rowscale[e], rowbias[e]);
							if constexpr (!CLO) {
								if (m < p.Co)
									y[ybase + (size_t)m * p.oHW] = (elem)v;
							}
							quad.v[e] = (elem)v;
						}
						if constexpr (CLO) {
							if (m0 + 8 * g < p.Co)
								*(Quad *)(y + n * p.Co + m0 + 8 * g) = quad;
						}
					}
				}
			}
		}
	};

	for (;;) {
		if constexpr (STEM)
			stem_tile(cur);
		for (int hb = 0; hb < NB; hb += 2) {
			block(hb, C0{});
			block(hb + 1, C1{});
		}
		if constexpr (STEM)
			if (nxt.ok)
				image_request(nxt);
		store_tile(cur);
		if (!WALK || !nxt.ok)
			break;
		cur = nxt;
#pragma unroll
		for (int t = 0; t < BL; t++)
			voff_[t] = voffn_[t];
#pragma unroll
		for (int i = 0; i < A_PW; i++)
			a_off_[i] = a_offn_[i];
		nlocal += nloc;
		nxt = decode(nlocal);
		offsets(nxt, voffn_, a_offn_);
		clear();
	}
	wide_wait<0, false>();	/* (the loads past the end bring zeros into LDS) */
#endif
}

/* Whether conv_patch_kernel can run this layer (a test may still force the generic kernels). */
bool thhip_conv_half_patch_ok(const ConvParams &p, int dtype)
{
	if (dtype != THHIP_F16 && dtype != THHIP_BF16)
		return false;
	return p.x_cl == 1 && (p.Ci == 64 || p.Ci == 128 || p.Ci == 256 || p.Ci == 512) && p.kH == 3 && p.kW == 3 && p.dH == 1 && p.dW == 1 &&
		p.x_bytes < 0x7fffffffu && (!p.y_cl || p.Co % 4 == 0) && (p.Ci != 64 || p.Co <= PATCH_ROWC);
}

/* Whether the whole-image form is the one to run: an output of at most 14 x 14 that fills at least five of
 * the eight blocks of 32 position slots, 256 or 512 input planes (a K loop long enough to pay for the patch),
 * and enough images and planes for 128 workgroups. */
bool thhip_conv_half_patch_flat_ok(const ConvParams &p, int dtype)
{
	if (!thhip_conv_half_patch_ok(p, dtype) || (p.Ci != 256 && p.Ci != 512) || p.padH != 1 || p.padW != 1)
		return false;
	if (p.oH > 14 || p.oW > 14 || p.Co % 32)
		return false;
	const int slots = p.pool ? 4 * (p.oH / 2) * (p.oW / 2) : p.oH * p.oW;
	return slots > 128 && (long)p.B * (p.Co / 32) >= 128;
}

/* Workgroups of a kernel that one CU holds at once (by its registers and LDS), asked once per kernel. */
template <void (*kernel)(ConvParams)>
static int patch_residents()
{
	static int n;
	if (!n) {
		hipcheck(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0));
		if (n < 1)
			THError("thhip_conv2d: the patch kernel does not fit a CU");
	}
	return n;
}

static int patch_cus()
{
	static int n;
	if (!n) {
		int dev;
		hipcheck(hipGetDevice(&dev));
		hipcheck(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
	}
	return n;
}

template <void (*kernel)(ConvParams)>
static void patch_go(ConvParams &p, long per_xcd, bool walk)
{
	/* walk: as many workgroups per XCD as it holds at once, or fewer when that spreads its tiles as evenly:
	 * each then walks rounds = ceil(tiles / workgroups) tiles or one less.  Else one workgroup per tile,
	 * which the dispatcher hands to the CUs as they come free. */
	long n = per_xcd;
	if (walk) {
		const long slots = (long)(patch_cus() / 8) * patch_residents<kernel>();
		n = per_xcd < slots ? per_xcd : slots;
		const long rounds = (per_xcd + n - 1) / n;
		n = (per_xcd + rounds - 1) / rounds;
	}
	kernel<<<dim3((unsigned)(8 * n)), dim3(256), 0, thhip_stream()>>>(p);
}

template <int DT, int BM, bool WHOLE>
static void conv_launch_patch(ConvParams &p)
{
	p.tiles_m = (p.Co + BM - 1) / BM;
	p.tiles_n = WHOLE ? p.B : p.B * ((p.oW + PATCH_TW - 1) / PATCH_TW) * ((p.oH + PATCH_TH - 1) / PATCH_TH);
	p.splitk = 1;
	if ((size_t)p.tiles_m * BM / 32 * p.KC * 1024 > p.w_bytes)
		THError("thhip_conv2d: packed weights shorter than the tile grid");
	const bool walk = p.Ci == 64;	/* (the kernel's WALK) */
	if (walk && p.tiles_m * BM > PATCH_ROWC)
		THError("thhip_conv2d: the patch kernel keeps the constants of at most %d planes", PATCH_ROWC);
	const long total = (long)p.tiles_m * p.tiles_n;
	long per_xcd = (total + 7) / 8;
	if constexpr (WHOLE) {
		/* The (plane block, image) grid in mparts x 8 / mparts rectangles, one per XCD: an XCD's L2 then
		 * fetches 1 / mparts of the weights and mparts / 8 of the images; the split that fetches least. */
		const double wbytes = (double)p.Co * p.K * 2, xbytes = (double)p.B * p.Ci * p.H * p.W * 2;
		double best = 0;
		p.mparts = 1;
		for (int mp = 1; mp <= 8; mp *= 2) {
			if (mp > p.tiles_m || 8 / mp > p.tiles_n)
				continue;
			const double cost = 8.0 * wbytes / mp + xbytes * mp;
			if (best == 0 || cost < best)
				best = cost, p.mparts = mp;
		}
		per_xcd = 0;
		for (int x = 0; x < 8; x++) {
			const int mp = x % p.mparts, np = x / p.mparts, nparts = 8 / p.mparts;
			const long cnt = (long)(p.tiles_m * (mp + 1) / p.mparts - p.tiles_m * mp / p.mparts) *
				(p.tiles_n * (np + 1) / nparts - p.tiles_n * np / nparts);
			per_xcd = cnt > per_xcd ? cnt : per_xcd;
		}
	}
#define CONV_PATCH_GO(CLO, CI)                                                              \
	do {                                                                               \
		if (p.pool)                                                                \
			patch_go<conv_patch_kernel<DT, CLO, BM, CI, true, WHOLE>>(p, per_xcd, walk);  \
		else                                                                       \
			patch_go<conv_patch_kernel<DT, CLO, BM, CI, false, WHOLE>>(p, per_xcd, walk); \
	} while (0)
	if constexpr (!WHOLE && BM == 64) {
		if (p.img) {	/* the image layer in front */
			if (p.Ci != 64 || !p.y_cl || p.tiles_m * BM > 256 || p.W % 2 || p.padH != 1 || p.padW != 1 || !p.wstem)
				THError("thhip_conv2d: the image layer goes in front of a 3x3 / padding 1 layer of 64 input and at most 256 output planes, channels-last, on images of even width");
			if (p.pool)
				patch_go<conv_patch_kernel<DT, true, BM, 64, true, false, true>>(p, per_xcd, true);
			else
				patch_go<conv_patch_kernel<DT, true, BM, 64, false, false, true>>(p, per_xcd, true);
			return;
		}
	}
	if constexpr (!WHOLE) {
		if (p.Ci == 64 && p.y_cl)
			CONV_PATCH_GO(true, 64);
		else if (p.Ci == 64)
			CONV_PATCH_GO(false, 64);
		else if (p.Ci == 128 && p.y_cl)
			CONV_PATCH_GO(true, 128);
		else if (p.Ci == 128)
			CONV_PATCH_GO(false, 128);
	}
	if (p.Ci == 256 && p.y_cl)
		CONV_PATCH_GO(true, 256);
	else if (p.Ci == 256)
		CONV_PATCH_GO(false, 256);
	else if (p.Ci == 512 && p.y_cl)
		CONV_PATCH_GO(true, 512);
	else if (p.Ci == 512)
		CONV_PATCH_GO(false, 512);
#undef CONV_PATCH_GO
}

/* flat: the whole-image form, with bm = 32 or 64 output planes per workgroup (the 32 x 8 tiles: always 64) */
void thhip_conv_half_patch_launch(ConvParams &p, int dtype, int bm, int flat)
{
	if (!thhip_conv_half_patch_ok(p, dtype))
		THError("thhip_conv2d: the patch kernel needs a half type, channels-last input of 64, 128, 256 or 512 planes, 3x3, stride 1, at most %d output planes",
			PATCH_ROWC);
	if (flat && !thhip_conv_half_patch_flat_ok(p, dtype))
		THError("thhip_conv2d: the whole-image patch kernel needs 256 or 512 input planes, padding 1 and an output of at most 14 x 14");
	if (dtype == THHIP_F16) {
		if (flat)
			return bm == 32 ? conv_launch_patch<THHIP_F16, 32, true>(p) : conv_launch_patch<THHIP_F16, 64, true>(p);
		return conv_launch_patch<THHIP_F16, 64, false>(p);
	}
	if (flat)
		return bm == 32 ? conv_launch_patch<THHIP_BF16, 32, true>(p) : conv_launch_patch<THHIP_BF16, 64, true>(p);
	return conv_launch_patch<THHIP_BF16, 64, false>(p);
}
