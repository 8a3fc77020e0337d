/*
 * The image layer of a uint8 network with the Threshold and the 3x3 / stride 2 max
 * pooling that follow it, in one kernel:
 *
 *   Lowp_SpatialConvolution_updateOutput (lowp/lowp_SpatialConvolution.c:124-187: uint8
 *   im2col with the padding code, gemmlowp GEMM, saturating bias add with its unclamped
 *   tail) -> Lowp_Threshold_updateOutput (lowp_Threshold.c:3-28) ->
 *   Lowp_SpatialMaxPooling_updateOutput (lowp_SpatialMaxPooling.c:45-108)
 *
 * for inputs of at most four planes in the reference's plane-major order, a horizontal
 * stride of four (AlexNet's 11x11 / stride 4 stem) and a pooling of 3x3 / stride 2
 * without padding.  The convolution output is never written: 12.4 MB per batch of 64 for
 * AlexNet, and two launches, are saved.
 *
 * A workgroup owns up to 4 x 27 pooled positions of one image and 64 output planes,
 * i.e. up to 9 x 55 = 495 convolution positions (16 MFMA tiles of 32).
 *  1. The input patch those positions read is copied into LDS once, as pixels of four
 *     bytes (the planes of a pixel; missing planes hold code 128, pixels outside the image
 *     the padding code): aligned words from each plane in, 8-byte LDS writes out.
 *  2. The packed weights of the 64 planes (the layout of the four-plane pixel path:
 *     k = (kernel row, group of four pixels, pixel, plane), re-centred, zero where a
 *     group reaches past the kernel row) are copied into LDS.
 *  3. Eight wavefronts take two position tiles each.  With the horizontal stride of four
 *     a group of four pixels of a kernel row is 16 aligned bytes of the patch, so a B
 *     fragment of v_mfma_i32_32x32x32_i8 is one ds_read_b128 per lane at
 *     (position base) + (group offset), the group offsets coming from a small table.
 *     The patch holds re-centred codes (x ^ 0x80); the column sums of the expanded
 *     offset term are taken with v_dot4 over the bytes that belong to real taps.
 *  4. The epilogue applies gemmlowp's output stage in wrapping int32, the saturating
 *     bias add (unclamped below for the last oH * oW % 8 positions of a plane,
 *     lowp_SpatialConvolution.c:71-88) and the threshold, and puts the codes into LDS
 *     (over the weights, which are no longer needed) as [position][64 planes].
 *  5. Every thread takes the maximum of a 3x3 window for 16 planes and writes 16 bytes
 *     of the channels-last result [B][pH][pW][Co].
 */
#include <stdlib.h>
#include <type_traits>
#include "thhip_internal.h"

#define CI_THREADS 512
#define CI_WAVES 8
#define CI_PR 4		/* pooled rows per workgroup */
#define CI_PC 27	/* pooled columns per workgroup: (2 * 4 + 1) * (2 * 27 + 1) = 495 <= 512 positions */
#define CI_MAXPOS 512
#define CI_PLANES 64

struct ConvImgParams {
	const unsigned char *x;		/* [B][Ci][H][W] codes */
	const unsigned char *wp;	/* packed weights, [Co / 32][KC][2][32][16] */
	const int *rowsum;		/* per output plane: sum of the re-centred weight codes */
	const int *addend;		/* per output plane bias addend, or NULL */
	unsigned char *y;		/* [B][pH][pW][Co] */
	int B, Ci, H, W, Co, kH, kW, dH, padH, padW, oH, oW, pH, pW;
	int KC, kwv, K;
	int rin;			/* patch rows: 2 * CI_PR * dH + kH */
	int rowb;			/* bytes per patch row (a multiple of 16) */
	unsigned fill;			/* one pixel outside the image */
	int offA, offB, c_off, c_mult, c_shift, act, ithr, ival;
};

typedef unsigned short ci_us2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(CI_THREADS) void conv_u8_image_pool_kernel(ConvImgParams p)
{
	extern __shared__ __align__(16) unsigned char lds[];
	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int pc0 = blockIdx.x * CI_PC, pr0 = blockIdx.y * CI_PR;
	const int zgroups = p.Co / CI_PLANES;
	const int b = blockIdx.z / zgroups, cz = blockIdx.z - b * zgroups;
	const int pra = min(CI_PR, p.pH - pr0), pca = min(CI_PC, p.pW - pc0);	/* pooled rows / columns of this workgroup */
	const int chl = 2 * pra + 1, cwl = 2 * pca + 1;				/* its convolution rows / columns */
	const int npos = chl * cwl;
	const int y0 = 2 * pr0, x0 = 2 * pc0;
	/* LDS: patch | weights (later: codes) | group table | row terms | addends */
	const int patch_bytes = p.rin * p.rowb;
	const int w_bytes = 2 * p.KC * 1024;
	unsigned char *patch = lds;
	unsigned char *wl = lds + patch_bytes;
	const int cbuf_bytes = CI_MAXPOS * CI_PLANES;
	int *gtab = (int *)(wl + (w_bytes > cbuf_bytes ? w_bytes : cbuf_bytes));
	int *rowterm = gtab + 2 * p.KC;
	int *rowadd = rowterm + CI_PLANES;

	/* 1. + 2. the patch (row r is input row iy0 + r, byte 4 c of a row is input column
	 * ix0 + c) and the weights.  Every thread requests all it will move before it
	 * touches any of it: a loop of load, wait, store would cost a memory round trip
	 * per turn. */
	{
		const int iy0 = y0 * p.dH - p.padH, ix0 = x0 * 4 - p.padW;
		const int pcols = (cwl - 1) * 4 + p.kwv * 4;			/* pixels of a patch row that are read */
		const int q0 = ix0 >> 2;					/* first aligned input quad (floor) */
		const int nq = ((ix0 + pcols + 3) >> 2) - q0;
		const int rows = (chl - 1) * p.dH + p.kH;
		const size_t plane = (size_t)p.H * p.W;
		const unsigned char *xb = p.x + (size_t)b * p.Ci * plane;
		const uintx4 *wsrc = (const uintx4 *)(p.wp + (size_t)cz * 2 * p.KC * 1024);
		constexpr int WMAX = 6, PMAX = 6;	/* per round: 6 * 512 * 16 bytes of weights, 6 * 8 rows of the patch */
		for (int w0 = 0; w0 < w_bytes / 16; w0 += WMAX * CI_THREADS) {
			uintx4 wv[WMAX];
#pragma unroll
			for (int u = 0; u < WMAX; u++)
				wv[u] = wsrc[min(w0 + u * CI_THREADS + tid, w_bytes / 16 - 1)];
#pragma unroll
			for (int u = 0; u < WMAX; u++)
				if (w0 + u * CI_THREADS + tid < w_bytes / 16)
					((uintx4 *)wl)[w0 + u * CI_THREADS + tid] = wv[u];
		}
		/* a wavefront takes patch rows wave, wave + 8, ..., a lane one aligned quad of a row
		 * (no divisions; a row of 224 + 12 pixels is 59 quads at most -- wider rows take
		 * several turns) */
		for (int q1 = 0; q1 < nq; q1 += 64) {
			const int q = q1 + lane;
			const int ixq = (q0 + q) * 4, c0 = ixq - ix0;	/* patch column of the quad's first pixel; only 0 .. pcols - 1 exist */
			const bool colin = q < nq && ixq >= 0 && ixq < p.W;	/* W % 4 == 0: a quad is all in or all out */
			for (int r0 = 0; r0 < rows; r0 += PMAX * CI_WAVES) {
				unsigned pl[PMAX][4];
#pragma unroll
				for (int u = 0; u < PMAX; u++) {
					const int iy = iy0 + r0 + u * CI_WAVES + wave;
					const bool in = colin && iy >= 0 && iy < p.H && r0 + u * CI_WAVES + wave < rows;
					const unsigned char *src = xb + (in ? (size_t)iy * p.W + ixq : 0);
#pragma unroll
					for (int c = 0; c < 4; c++)
						pl[u][c] = c < p.Ci ? *(const unsigned *)(src + c * plane) : 0x80808080u;
				}
#pragma unroll
				for (int u = 0; u < PMAX; u++) {
					const int r = r0 + u * CI_WAVES + wave;
					const int iy = iy0 + r;
					const bool in = colin && iy >= 0 && iy < p.H;
					/* 4 x 4 byte transpose: plane words -> pixels (bytes plane 0..3) */
					const unsigned lo01 = __builtin_amdgcn_perm(pl[u][1], pl[u][0], 0x05010400u);	/* p0b0 p1b0 p0b1 p1b1 */
					const unsigned hi01 = __builtin_amdgcn_perm(pl[u][1], pl[u][0], 0x07030602u);	/* p0b2 p1b2 p0b3 p1b3 */
					const unsigned lo23 = __builtin_amdgcn_perm(pl[u][3], pl[u][2], 0x05010400u);
					const unsigned hi23 = __builtin_amdgcn_perm(pl[u][3], pl[u][2], 0x07030602u);
					unsigned px[4];
					px[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
					px[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
					px[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
					px[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
					if (r < rows && q < nq) {
						unsigned char *dst = patch + r * p.rowb + c0 * 4;
#pragma unroll
						for (int e = 0; e < 4; e++)
							if (c0 + e >= 0 && c0 + e < pcols)
								*(unsigned *)(dst + 4 * e) = (in ? px[e] : p.fill) ^ 0x80808080u;	/* code - 128 as a signed byte */
					}
				}
			}
		}
	}
	/* the group table, the per-plane terms */
	{
		const int ngroups = p.kH * p.kwv;
		for (int g = tid; g < 2 * p.KC; g += CI_THREADS) {
			const int kh = g / p.kwv, jj = g - kh * p.kwv;
			const int nvalid = g >= ngroups ? 0 : (jj == p.kwv - 1 && (p.kW & 3)) ? (p.kW & 3) : 4;
			gtab[g] = (g >= ngroups ? 0 : kh * p.rowb + jj * 16) | (nvalid << 24);
		}
		if (tid < CI_PLANES) {
			const int m = cz * CI_PLANES + tid;
			rowterm[tid] = p.offB * p.rowsum[m] + p.K * p.offA * p.offB + p.c_off;	/* (wrapping, like the sum it joins) */
			rowadd[tid] = p.addend ? p.addend[m] : 0;
		}
	}
	__syncthreads();

	/* 3. two position tiles per wavefront */
	const int n = lane & 31, h = lane >> 5;
	int pbase[2];
#pragma unroll
	for (int j = 0; j < 2; j++) {
		const int pos = min((2 * wave + j) * 32 + n, npos - 1);
		const int ly = pos / cwl, lx = pos - ly * cwl;
		pbase[j] = ly * p.dH * p.rowb + lx * 16;
	}
	intx16 acc[2][2];
	int cs[2] = { 0, 0 };
#pragma unroll
	for (int i = 0; i < 2; i++)
#pragma unroll
		for (int j = 0; j < 2; j++)
#pragma unroll
			for (int r = 0; r < 16; r++)
				acc[i][j][r] = 0;
	const bool busy = 2 * wave * 32 < npos;		/* (a wavefront without positions still joins the barriers) */
	if (busy) {
		/* The patch holds re-centred codes, so a fragment goes to the matrix core as it is
		 * read.  The column sums count real taps only: a group's pixels past the kernel row
		 * (weight 0) are left out through the second operand of v_dot4.  The fragments of
		 * chunk kc + 1 and the table entry of chunk kc + 2 are requested before chunk kc is
		 * multiplied (an LDS round trip per chunk would set the pace); two chunks per turn,
		 * so that the two register sets swap roles without copies. */
		intx4 a0[2], b0[2], a1[2], b1[2];
		int ge0 = gtab[h], ge1 = gtab[min(2, 2 * p.KC - 2) + h];
#define CI_FETCH(A_, B_, KC_, GE_)                                                                 \
		do {                                                                               \
			_Pragma("unroll") for (int i = 0; i < 2; i++)                              \
				A_[i] = *(const intx4 *)(wl + ((i * p.KC + (KC_)) * 1024) + lane * 16); \
			_Pragma("unroll") for (int j = 0; j < 2; j++)                              \
				B_[j] = *(const intx4 *)(patch + pbase[j] + ((GE_) & 0xffffff));   \
		} while (0)
#define CI_MMA(A_, B_, GE_)                                                                        \
		do {                                                                               \
			const int nv_ = (GE_) >> 24;                                               \
			int mk_[4];                                                                \
			_Pragma("unroll") for (int d = 0; d < 4; d++)                              \
				mk_[d] = d < nv_ ? 0x01010101 : 0;                                 \
			_Pragma("unroll") for (int j = 0; j < 2; j++) {                            \
				_Pragma("unroll") for (int d = 0; d < 4; d++)                      \
					cs[j] = __builtin_amdgcn_sdot4(B_[j][d], mk_[d], cs[j], false); \
				_Pragma("unroll") for (int i = 0; i < 2; i++)                      \
					acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A_[i], B_[j], acc[i][j], 0, 0, 0); \
			}                                                                          \
		} while (0)
		CI_FETCH(a0, b0, 0, ge0);
		for (int kc = 0; kc < p.KC; kc += 2) {		/* KC is even */
			const int ge2 = gtab[2 * min(kc + 2, p.KC - 1) + h];
			CI_FETCH(a1, b1, kc + 1, ge1);
			CI_MMA(a0, b0, ge0);
			const int ge3 = gtab[2 * min(kc + 3, p.KC - 1) + h];
			CI_FETCH(a0, b0, min(kc + 2, p.KC - 1), ge2);
			CI_MMA(a1, b1, ge1);
			ge0 = ge2;
			ge1 = ge3;
		}
#undef CI_FETCH
#undef CI_MMA
	}
	__syncthreads();	/* the weights are done with: their LDS becomes the code buffer */

	/* 4. requantise into [position][64 planes] */
	unsigned char *cbuf = wl;
	if (busy) {
		const int tail0 = (p.oH * p.oW / 8) * 8;	/* lowpadd's unclamped tail starts here */
		const bool has_add = p.addend != 0;
		const unsigned round = p.c_shift < 1 ? 0u : 1u << (p.c_shift - 1);
#pragma unroll
		for (int j = 0; j < 2; j++) {
			const int pos = (2 * wave + j) * 32 + n;
			const int colsum = cs[j] + __shfl_xor(cs[j], 32, 64);
			const int posc = min(pos, npos - 1);
			const int ly = posc / cwl, lx = posc - ly * cwl;
			const bool tail = has_add && (y0 + ly) * p.oW + x0 + lx >= tail0;
			/* the few tail positions of an image (if any) are in one wavefront of its last
			 * workgroup: everybody else takes the clamped add without asking per value */
			const bool any_tail = __builtin_amdgcn_ballot_w64(tail) != 0;
			const int colterm = p.offA * colsum;
			/* 16-byte pieces of a position's 64 codes are swapped around by the position, so
			 * that the lanes of a store (positions 64 bytes apart) spread over the banks */
			unsigned char *crow = cbuf + posc * CI_PLANES;
			const int sw = (posc >> 2) & 3;
			auto finish = [&](auto tails_, auto act_) {
				constexpr bool tails = decltype(tails_)::value, act = decltype(act_)::value;
#pragma unroll
				for (int i = 0; i < 2; i++)
#pragma unroll
					for (int g = 0; g < 4; g++) {
						const int ml = i * 32 + 8 * g + 4 * h;
						const intx4 rt = *(const intx4 *)(rowterm + ml), ra = *(const intx4 *)(rowadd + ml);
						unsigned packed = 0;
#pragma unroll
						for (int e = 0; e < 4; e++) {
							/* gemmlowp's output stage in wrapping int32 (c_off is in the row term) */
							const unsigned u = (unsigned)(acc[i][j][4 * g + e] + rt[e] + colterm) * (unsigned)p.c_mult + round;
							int q = (int)u >> p.c_shift;
							q = q < 0 ? 0 : q > 255 ? 255 : q;
							const int sum = q + ra[e];	/* (no addend: 0, and the clamp changes nothing) */
							q = sum < 0 ? 0 : sum > 255 ? 255 : sum;
							if (tails)
								q = tail ? (sum > 255 ? 255 : (sum & 255)) : q;	/* lowp_SpatialConvolution.c:86-87 */
							if (act)
								q = q > p.ithr ? q : p.ival;
							packed |= (unsigned)q << (8 * e);
						}
						if (pos < npos)
							*(unsigned *)(crow + ((((ml >> 4) ^ sw) << 4) | (ml & 15))) = packed;
					}
			};
			if (any_tail) {
				if (p.act)
					finish(std::true_type{}, std::true_type{});
				else
					finish(std::true_type{}, std::false_type{});
			} else if (p.act)
				finish(std::false_type{}, std::true_type{});
			else
				finish(std::false_type{}, std::false_type{});
		}
	}
	__syncthreads();

	/* 5. 3x3 / stride 2 maximum, sixteen planes per thread */
	for (int it = tid; it < pra * pca * 4; it += CI_THREADS) {
		const int c16 = it & 3, t = it >> 2;
		const int prl = t / pca, pcl = t - prl * pca;
		/* byte-wise maxima as packed 16-bit maxima of the even and of the odd bytes */
		ci_us2 me[4], mo[4];
#pragma unroll
		for (int d = 0; d < 4; d++)
			me[d] = mo[d] = ci_us2{ 0, 0 };
#pragma unroll
		for (int dy = 0; dy < 3; dy++)
#pragma unroll
			for (int dx = 0; dx < 3; dx++) {
				const int pos = (2 * prl + dy) * cwl + 2 * pcl + dx;
				const uintx4 v = *(const uintx4 *)(cbuf + pos * CI_PLANES + ((c16 ^ (pos >> 2)) & 3) * 16);
#pragma unroll
				for (int d = 0; d < 4; d++) {
					me[d] = __builtin_elementwise_max(me[d], __builtin_bit_cast(ci_us2, v[d] & 0x00ff00ffu));
					mo[d] = __builtin_elementwise_max(mo[d], __builtin_bit_cast(ci_us2, (v[d] >> 8) & 0x00ff00ffu));
				}
			}
		uintx4 m;
#pragma unroll
		for (int d = 0; d < 4; d++)
			m[d] = __builtin_bit_cast(unsigned, me[d]) | (__builtin_bit_cast(unsigned, mo[d]) << 8);
		*(uintx4 *)(p.y + (((size_t)b * p.pH + pr0 + prl) * p.pW + pc0 + pcl) * p.Co + cz * CI_PLANES + c16 * 16) = m;
	}
}

static size_t ci_lds_bytes(int Ci, int kH, int kW, int dH, int *rin, int *rowb)
{
	const int kwv = (kW + 3) / 4, KC = thhip_conv_u8_packed_chunks(Ci, kH, kW, 2);
	*rin = 2 * CI_PR * dH + kH;
	*rowb = (((2 * CI_PC) * 4 + kwv * 4) * 4 + 15) / 16 * 16 + 16;
	const size_t w = (size_t)2 * KC * 1024, c = (size_t)CI_MAXPOS * CI_PLANES;
	return (size_t)*rin * *rowb + (w > c ? w : c) + sizeof(int) * (2 * KC + 2 * CI_PLANES);
}

/* Whether thhip_conv2d_u8_image_pool takes the layer: at most four input planes in whole
 * words per row (W % 4 == 0), horizontal stride 4, output planes in groups of 64, a
 * 3x3 / stride 2 pooling without padding in floor mode, and a patch that fits in LDS. */
extern "C" int thhip_conv2d_u8_image_pool_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode)
{
	if (B < 1 || Ci < 1 || Ci > 4 || W % 4 || dW != 4 || dH < 1 || Co % CI_PLANES || Co < CI_PLANES || kH < 1 || kW < 1 ||
	    padH < 0 || padW < 0)
		return 0;
	if (pkH != 3 || pkW != 3 || pdH != 2 || pdW != 2 || ppadH || ppadW || ceil_mode)
		return 0;
	const int oW = (W + 2 * padW - kW) / dW + 1, oH = (H + 2 * padH - kH) / dH + 1;
	if (oW < 3 || oH < 3)
		return 0;
	if ((double)B * Ci * H * W >= 2147483000.0 || (long)B * (Co / CI_PLANES) > 65535)
		return 0;
	int rin, rowb;
	return ci_lds_bytes(Ci, kH, kW, dH, &rin, &rowb) <= 150 * 1024;
}

/* x: codes [B][Ci][H][W]; wpacked: thhip_conv_pack_weight_u8_layout(w, Co, Ci, kH, kW, 2)
 * (the per-row sums follow the packed codes); y: [B][pH][pW][Co] with
 * pH = (oH - 3) / 2 + 1, pW likewise.  Same parameters as thhip_conv2d_u8. */
extern "C" void thhip_conv2d_u8_image_pool(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val)
{
	if (!thhip_conv2d_u8_image_pool_supported(B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, 3, 3, 2, 2, 0, 0, 0))
		THError("thhip_conv2d_u8_image_pool: layer not supported (see thhip_conv2d_u8_image_pool_supported)");
	if (c_shift < 0 || c_shift > 31)
		THError("thhip_conv2d_u8_image_pool: shift %d out of range", c_shift);
	if (((size_t)x & 3) || ((size_t)y & 15))
		THError("thhip_conv2d_u8_image_pool: x must be 4-byte and y 16-byte aligned");
	ConvImgParams p;
	p.x = x;
	p.wp = (const unsigned char *)wpacked;
	p.B = B; p.Ci = Ci; p.H = H; p.W = W; p.Co = Co; p.kH = kH; p.kW = kW; p.dH = dH; p.padH = padH; p.padW = padW;
	p.oW = (W + 2 * padW - kW) / dW + 1;
	p.oH = (H + 2 * padH - kH) / dH + 1;
	p.pH = (p.oH - 3) / 2 + 1;
	p.pW = (p.oW - 3) / 2 + 1;
	p.KC = thhip_conv_u8_packed_chunks(Ci, kH, kW, 2);
	p.kwv = (kW + 3) / 4;
	p.K = Ci * kH * kW;
	p.rowsum = (const int *)(p.wp + thhip_conv_u8_packed_code_bytes(Co, Ci, kH, kW, 2));
	p.addend = addend;
	p.y = y;
	const size_t bytes = ci_lds_bytes(Ci, kH, kW, dH, &p.rin, &p.rowb);
	unsigned fill = 0x80808080u;
	for (int c = 0; c < Ci; c++)
		fill = (fill & ~(255u << (8 * c))) | ((unsigned)(zero & 255) << (8 * c));
	p.fill = fill;
	p.offA = 128 + a_off;
	p.offB = 128 + b_off;
	p.c_off = c_off; p.c_mult = c_mult; p.c_shift = c_shift;
	p.act = act; p.ithr = thr; p.ival = val;
	static size_t lds_set;
	if (bytes > lds_set) {
		hipcheck(hipFuncSetAttribute((const void *)conv_u8_image_pool_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
		lds_set = bytes;
	}
	ThhipLaunchScope scope(THHIP_FAM_CONV_I8, 2.0 * Co * (double)p.K * B * p.oH * p.oW);
	const dim3 grid((p.pW + CI_PC - 1) / CI_PC, (p.pH + CI_PR - 1) / CI_PR, B * (Co / CI_PLANES));
	conv_u8_image_pool_kernel<<<grid, dim3(CI_THREADS), bytes, thhip_stream()>>>(p);
}
