/*
 * The image layer of a VGG-style network: SpatialConvolution(3 -> 64 n planes, 3x3, stride 1,
 * padding 1) on plane-major input (modules/SpatialConvolutionMM.c:153-215: im2col + sgemm +
 * bias; cudnn/cudnn_SpatialConvolution.c for the half types), with the folded batch norm
 * factor and Threshold of the generic kernel's epilogue.
 *
 * K = 27 is one or two MFMAs deep, so the layer is bound by writing its output (64 planes
 * per pixel: 205 MB in fp32 at batch 16 against 10 MB read), and what a kernel can lose
 * time on is the gather.  Here a workgroup owns a band of whole output rows: it copies the
 * band's input rows (three planes, one row above and below, a zero column left and right)
 * into LDS once, with loads that run along the rows, and every B operand is that patch read
 * at a fixed offset per k: no tap decode, no bounds test.  The weights (64 rows x 27) live
 * in registers as A fragments for the whole kernel.  A wavefront multiplies tiles of 32
 * neighbouring positions of a row with all 64 planes and stores them: plane-major fp32 as
 * 128-byte runs per plane, channels-last half types as 16-byte pieces of a pixel's planes.
 */
#include <type_traits>
#include "thhip_internal.h"

#define STEM_THREADS 256
#define STEM_K 27

struct StemParams {
	const void *x;
	const void *wp;
	const float *bias, *scale;
	void *y;
	int B, H, W, Co, KC;
	int rows;	/* output rows per workgroup */
	int tpr;	/* tiles of 32 positions per row */
	int pw;		/* elements per patch row: 32 tpr + 2 */
	unsigned magic_pw;	/* floor(2^32 / pw) + 1: e / pw = umulhi(e, magic) for the e of a patch */
	int act;
	float thr, val;
};

__device__ __forceinline__ void stem_swap32(unsigned &x, unsigned &y)
{
	const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
	x = r[0];
	y = r[1];
}

/* offset of k = (plane, kh, kw) in a patch of prows rows of pw elements per plane */
__device__ __forceinline__ int stem_koff(int k, int prows, int pw)
{
	const int c = k / 9, t = k - 9 * c, kh = t / 3, kw = t - 3 * kh;
	return k < STEM_K ? (c * prows + kh) * pw + kw : 0;
}

template <int DT, bool CLO>
__global__ __launch_bounds__(STEM_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void conv_stem_kernel(StemParams p)
{
	typedef typename ThhipElem<DT>::T elem;
	constexpr bool F32 = DT == THHIP_F32;
	constexpr int NS = F32 ? 14 : 2;	/* MFMAs along K (K padded to 28 / 32) */
	extern __shared__ __align__(16) unsigned char stem_lds[];
	float *const rowc = (float *)stem_lds;	/* bias[64], factor[64] */
	elem *const patch = (elem *)(stem_lds + 512 + (CLO ? 4 * 4096 : 0));

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int n = lane & 31, h = lane >> 5;
	unsigned char *const stage = stem_lds + 512 + wave * 4096;	/* (channels-last output) */
	const int b = blockIdx.z, mz = blockIdx.y;
	const int row0 = blockIdx.x * p.rows;
	const int rows = min(p.rows, p.H - row0);
	const int prows = p.rows + 2;

	/* ---- the patch: rows row0 - 1 .. row0 + rows of the three planes, columns -1 .. 32 tpr;
	 * eight loads in flight per thread (a load that waits for the one before it costs a
	 * trip to memory each, and this prologue is most of what the kernel can lose) ---- */
	{
		const int total = 3 * prows * p.pw;
		/* this image's three planes; an offset past them reads as zero (the padding) */
		const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
			(void *)((const elem *)p.x + (size_t)b * 3 * p.H * p.W), 0, 3 * p.H * p.W * (int)sizeof(elem), 0x00020000);
		for (int e0 = 0; e0 < total; e0 += 8 * STEM_THREADS) {
			elem v[8];
#pragma unroll
			for (int u = 0; u < 8; u++) {
				const int e = e0 + u * STEM_THREADS + tid;
				const int r = __umulhi((unsigned)e, p.magic_pw), pc = e - r * p.pw;	/* e / pw, e % pw */
				const int c = r >= 2 * prows ? 2 : r >= prows ? 1 : 0, pr = r - c * prows;
				const int iy = row0 - 1 + pr, ix = pc - 1;
				const bool in = r < 3 * prows && iy >= 0 && iy < p.H && pr < rows + 2 && ix >= 0 && ix < p.W;
				const int voff = in ? ((c * p.H + iy) * p.W + ix) * (int)sizeof(elem) : (int)0x80000000;
				if constexpr (F32)
					v[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xrsrc, voff, 0, 0));
				else
					v[u] = __builtin_bit_cast(elem, __builtin_amdgcn_raw_buffer_load_b16(xrsrc, voff, 0, 0));
			}
#pragma unroll
			for (int u = 0; u < 8; u++) {
				const int e = e0 + u * STEM_THREADS + tid;
				if (e < total)
					patch[e] = v[u];
			}
		}
	}
	if (tid < 64) {
		rowc[tid] = p.bias ? p.bias[mz * 64 + tid] : 0.0f;
		rowc[64 + tid] = p.scale ? p.scale[mz * 64 + tid] : 1.0f;
	}
	__syncthreads();

	/* ---- weights: this lane's A fragments of both 32-row blocks (packed [32-row block][chunk][h][32][16 B]) ---- */
	float af[F32 ? 2 * NS : 1];
	halfx8 ah[F32 ? 1 : 2 * NS];
#pragma unroll
	for (int mb = 0; mb < 2; mb++)
#pragma unroll
		for (int s = 0; s < NS; s++) {
			const int blk = mz * 2 + mb;
			if constexpr (F32) {
				const int kp = 2 * s + h;	/* the MFMA contracts the two lane halves */
				af[mb * NS + s] = ((const float *)p.wp)[((((size_t)blk * p.KC + kp / 8) * 2 + (kp % 8) / 4) * 32 + n) * 4 + kp % 4];
			} else {
				ah[mb * NS + s] = ((const halfx8 *)p.wp)[(((size_t)blk * p.KC + s) * 2 + h) * 32 + n];
			}
		}
	/* ---- where this lane reads its B values: k = 2 s + h (fp32), 16 s + 8 h + e (half types) ---- */
	int off[F32 ? NS : 16];
#pragma unroll
	for (int i = 0; i < (F32 ? NS : 16); i++)
		off[i] = stem_koff(F32 ? 2 * i + h : 16 * (i / 8) + 8 * h + i % 8, prows, p.pw);

	const bool has_scale = p.scale != 0;
	const int ntiles = rows * p.tpr;
	constexpr int NB = F32 ? NS : 16;	/* B values a lane reads per tile */
	typedef typename std::conditional<F32, float, unsigned short>::type bval;
	bval bcur[NB];
	auto fetch = [&](int t, bval (&bv)[NB]) {
		const int ly = t / p.tpr, tx = t - ly * p.tpr;
		const bval *pb = (const bval *)patch + ly * p.pw + tx * 32 + n;
#pragma unroll
		for (int i = 0; i < NB; i++)
			bv[i] = pb[off[i]];
	};
	if (wave < ntiles)
		fetch(wave, bcur);
	/* the output of this image (channels-last) or of this image's 64 planes (plane-major) as a buffer:
	 * a store is then one instruction with a 32-bit offset per lane and the plane's offset from the
	 * scalar unit, and a lane past the row's end stores out of range, that is nowhere */
	const int HW = p.H * p.W;
	const __amdgpu_buffer_rsrc_t yrsrc = CLO
		? __builtin_amdgcn_make_buffer_rsrc((void *)((elem *)p.y + (size_t)b * HW * p.Co), 0, HW * p.Co * (int)sizeof(elem), 0x00020000)
		: __builtin_amdgcn_make_buffer_rsrc((void *)((elem *)p.y + ((size_t)b * p.Co + mz * 64) * HW), 0, 64 * HW * (int)sizeof(elem), 0x00020000);
	for (int t = wave; t < ntiles; t += STEM_THREADS / 64) {
		const int ly = t / p.tpr, tx = t - ly * p.tpr;
		floatx16 acc[2];
#pragma unroll
		for (int mb = 0; mb < 2; mb++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[mb][r] = 0.0f;
		if constexpr (F32) {
			if (h)
				bcur[NS - 1] = 0.0f;	/* k = 27 does not exist (its weight is zero, the patch value might not be finite) */
#pragma unroll
			for (int s = 0; s < NS; s++)
#pragma unroll
				for (int mb = 0; mb < 2; mb++)
					acc[mb] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[mb * NS + s], bcur[s], acc[mb], 0, 0, 0);
		} else {
#pragma unroll
			for (int i = 11; i < 16; i++)
				bcur[i] = h ? (unsigned short)0 : bcur[i];	/* k = 27 .. 31 */
#pragma unroll
			for (int s = 0; s < NS; s++) {
				uintx4 bw;
#pragma unroll
				for (int d = 0; d < 4; d++)
					bw[d] = (unsigned)bcur[8 * s + 2 * d] | ((unsigned)bcur[8 * s + 2 * d + 1] << 16);
#pragma unroll
				for (int mb = 0; mb < 2; mb++) {
					if constexpr (DT == THHIP_F16)
						acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[mb * NS + s], __builtin_bit_cast(halfx8, bw), acc[mb], 0, 0, 0);
					else
						acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ah[mb * NS + s]),
							__builtin_bit_cast(bf16x8, bw), acc[mb], 0, 0, 0);
				}
			}
		}
		/* the next tile's values are requested as soon as the MFMAs have taken this tile's, and arrive under the stores */
		fetch(min(t + STEM_THREADS / 64, ntiles - 1), bcur);
		/* ---- (factor,) bias, Threshold, store: register 4 g + e of block mb is plane 32 mb + 8 g + 4 h + e.
		 * Plane-major: a wave-uniform pointer per register plus one 32-bit offset per lane and tile. ---- */
		const int oy = row0 + ly, ox = tx * 32 + n;
		const bool valid = ox < p.W;
		/* (the per-plane constants are read from LDS again for every tile: kept in registers
		 * they would be 64 of them, and the weights would go to scratch memory) */
		asm volatile("" ::: "memory");
		const int laneoff = !valid ? (int)0x80000000
			: CLO ? ((oy * p.W + ox) * p.Co + mz * 64 + 8 * h) * (int)sizeof(elem) : ((4 * h * p.H + oy) * p.W + ox) * (int)sizeof(elem);
#pragma unroll
		for (int mb = 0; mb < 2; mb++) {
			unsigned lo[4], hi[4];
#pragma unroll
			for (int g = 0; g < 4; g++) {
				const int ml = mb * 32 + 8 * g + 4 * h;
				const floatx4 rb = *(const floatx4 *)(rowc + ml), rs = *(const floatx4 *)(rowc + 64 + ml);
				struct alignas(4 * sizeof(elem)) Quad { elem v[4]; } quad;
#pragma unroll
				for (int e = 0; e < 4; e++) {
					float v = has_scale ? acc[mb][4 * g + e] * rs[e] + rb[e] : acc[mb][4 * g + e] + rb[e];
					if (p.act)
						v = v > p.thr ? v : p.val;
					quad.v[e] = (elem)v;
					if constexpr (!CLO) {
						const int soff = (mb * 32 + 8 * g + e) * HW * (int)sizeof(elem);
						if constexpr (F32)
							__builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), yrsrc, laneoff, soff, 0);
						else
							__builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, quad.v[e]), yrsrc, laneoff, soff, 0);
					}
				}
				if constexpr (CLO) {
					unsigned pair[2];
					__builtin_memcpy(pair, &quad, 8);
					lo[g] = pair[0];
					hi[g] = pair[1];
				}
			}
			if constexpr (CLO) {
				/* into this wave's 4 KiB of LDS, [position][64 planes] with the 16-byte pieces of a
				 * position exchanged by its number (the 32 positions would otherwise share banks) */
#pragma unroll
				for (int g = 0; g < 4; g++) {
					const uintx2 v = { lo[g], hi[g] };
					*(uintx2 *)(stage + n * 128 + (((mb * 4 + g) ^ (n & 7)) * 16) + 8 * h) = v;
				}
			}
		}
		if constexpr (CLO) {
			/* ... and out again in memory order: an instruction stores eight positions' 128 bytes each
			 * (1 KiB in one piece when the layer has 64 planes) */
			const int obase = ((oy * p.W + tx * 32) * p.Co + mz * 64) * (int)sizeof(elem);
#pragma unroll
			for (int i = 0; i < 4; i++) {
				const int u = i * 64 + lane, px = u >> 3, slot = u & 7;
				const uintx4 v = *(const uintx4 *)(stage + px * 128 + ((slot ^ (px & 7)) * 16));
				const int goff = tx * 32 + px < p.W ? obase + px * p.Co * (int)sizeof(elem) + slot * 16 : (int)0x80000000;
				__builtin_amdgcn_raw_buffer_store_b128(v, yrsrc, goff, 0, 0);
			}
		}
	}
}

static int stem_rows(int B, int H)
{
	int rows = 4;
	while (rows > 1 && (long)B * ((H + rows - 1) / rows) < 512)
		rows /= 2;
	return rows;
}

static size_t stem_lds_bytes(int rows, int W, int esize, int y_cl)
{
	const int tpr = (W + 31) / 32;
	return 512 + (y_cl ? 4 * 4096 : 0) + (size_t)3 * (rows + 2) * (32 * tpr + 2) * esize;
}

/* The layers this kernel takes: 3 planes in, whole blocks of 64 planes out, 3x3, stride 1,
 * padding 1, float types, a patch that fits in 64 KiB of LDS; channels-last output for the
 * half types only. */
bool thhip_conv_stem_ok(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int dtype, int y_cl)
{
	if (Ci != 3 || Co % 64 || kH != 3 || kW != 3 || dH != 1 || dW != 1 || padH != 1 || padW != 1)
		return false;
	if (dtype != THHIP_F32 && dtype != THHIP_F16 && dtype != THHIP_BF16)
		return false;
	if (y_cl && dtype == THHIP_F32)
		return false;
	if (B > 65535 || Co / 64 > 65535)
		return false;
	return stem_lds_bytes(stem_rows(B, H), W, thhip_esize(dtype), y_cl) <= 65536;
}

template <int DT, bool CLO>
static void stem_launch(const StemParams &p, size_t lds)
{
	const dim3 grid((p.H + p.rows - 1) / p.rows, p.Co / 64, p.B);
	conv_stem_kernel<DT, CLO><<<grid, dim3(STEM_THREADS), lds, thhip_stream()>>>(p);
}

/* wpacked: the weights as thhip_conv_pack_weight_layout packs them for plane-major input
 * (K order plane, tap; KC chunks per 32-row block).  The caller brackets the launch. */
void thhip_conv_stem(const void *x, const void *wpacked, int KC, const float *scale, const float *bias, void *y,
	int B, int H, int W, int Co, int act, float thr, float val, int dtype, int y_cl)
{
	if (!thhip_conv_stem_ok(B, 3, H, W, Co, 3, 3, 1, 1, 1, 1, dtype, y_cl))
		THError("thhip_conv_stem: unsupported layer");
	StemParams p;
	p.x = x; p.wp = wpacked; p.bias = bias; p.scale = scale; p.y = y;
	p.B = B; p.H = H; p.W = W; p.Co = Co; p.KC = KC;
	p.rows = stem_rows(B, H);
	p.tpr = (W + 31) / 32;
	p.pw = 32 * p.tpr + 2;
	p.magic_pw = (unsigned)((1ull << 32) / p.pw + 1);
	p.act = act; p.thr = thr; p.val = val;
	const size_t lds = stem_lds_bytes(p.rows, W, thhip_esize(dtype), y_cl);
	if (dtype == THHIP_F32)
		stem_launch<THHIP_F32, false>(p, lds);
	else if (dtype == THHIP_F16)
		y_cl ? stem_launch<THHIP_F16, true>(p, lds) : stem_launch<THHIP_F16, false>(p, lds);
	else
		y_cl ? stem_launch<THHIP_BF16, true>(p, lds) : stem_launch<THHIP_BF16, false>(p, lds);
}
