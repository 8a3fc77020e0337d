/*
 * thnets_hip.h -- C ABI of the MI355X (gfx950) engine for thnets.
 *
 * Three layers, all plain C (extern "C" when included from C++/HIP):
 *
 *  1. The thnets tensor / module / network structures, laid out field for
 *     field like the reference's default (non -DLOWP, non -DOPENCL) build so
 *     that a `struct module[]` built by an existing thnets caller can be
 *     handed to this library unchanged (thnets.h:104-120, 122-130, 140-232,
 *     250-336, 401-407, 571-580).
 *  2. The high level calls a thnets user already knows (thnets.h:582-598)
 *     plus the new constructors THCreateHipNetwork / THCreateHipLowpNetwork
 *     that sit beside THCreateCudaNetwork / THCreateLowpNetwork
 *     (thapi.c:730-742, 784-796).
 *  3. The kernel level entry points (thhip_*): plain device pointers and
 *     sizes, one per hand written HIP kernel.  These are what the module
 *     glue calls and what a foreign-function binding would bind.
 *
 * Every entry point that touches the GPU aborts through THError when a HIP
 * call fails; there is no CPU fallback in this library.
 */
#ifndef THNETS_HIP_H
#define THNETS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ */
/* 1. thnets ABI                                                       */
/* ------------------------------------------------------------------ */

#ifdef THNETS_IN_TREE
/* Built inside the thnets tree (its Makefile's HIP=1 option): structures, module
 * types, tensor helpers and the high level prototypes come from the tree's own
 * thnets.h, so the engine sees exactly the layout every other translation unit of
 * libthnets sees (all of them must agree on -DLOWP / -DOPENCL, thnets.h:117-119,
 * 300-303).  The tree appends ENGINE_HIP, ENGINE_HIPLOWP to the enum at thnets.h:401
 * and defines THNETS_HAS_ENGINE_HIP; against an unpatched header the two values are
 * declared here. */
#include "thnets.h"
#ifndef THNETS_HAS_ENGINE_HIP
enum { ENGINE_HIP = ENGINE_LOWP + 1, ENGINE_HIPLOWP = ENGINE_LOWP + 2 };
#endif
#ifndef MAXMODULEINPUTS
#define MAXMODULEINPUTS 16	/* int inputs[16], thnets.h:310 */
#endif
extern int th_debug, th_profile, th_minmax;
extern double th_convtot, th_convflops;
#else
/* thnets.h:16-22 */
enum therror {
	ERR_OPENFILE = -1,
	ERR_READFILE = -2,
	ERR_NOTIMPLEMENTED = -3,
	ERR_CORRUPTED = -4,
	ERR_WRONGOBJECT = -5
};

/* thnets.h:104-108.  mustfree: 0 borrowed, 1 free(), 2 cudaFree (unused
 * here), 3 OpenCL (unused here), 4..7 = device memory owned by this engine,
 * holding elements of type (mustfree - 4) of enum thhip_dtype: a device tensor
 * says what it holds, so a tensor made for one network type is refused by
 * another instead of being read with the wrong element size. */
typedef struct THFloatStorage {
	float *data;
	int nref, mustfree;
} THFloatStorage;


/* thnets.h:110-120 (default build: no sub/mult members). */
typedef struct THFloatTensor {
	long size[4];
	long stride[4];
	int nDimension;
	THFloatStorage *storage;
	long storageOffset;
} THFloatTensor;

/* Per-module parameter blocks, thnets.h:122-248.  Only the members of the
 * union that this engine reads are spelled out; the union is padded to the
 * reference's size so that modules[i] indexes identically. */
struct SpatialConvolution {
	THFloatTensor *bias, *weight, *finput;
	int dW, dH, padW, padH, kW, kH, nInputPlane, nOutputPlane;
	int refl_pad;
	int padW2, padH2;
	int autopad;
	int dlH, dlW;
};

/* thnets.h:132-138; weight is [nInputPlane][nOutputPlane][kH][kW] */
struct SpatialFullConvolution {
	THFloatTensor *bias, *weight;
	int dW, dH, padW, padH, kW, kH, nInputPlane, nOutputPlane;
	int adjW, adjH;
	THFloatTensor *ones, *columns;
};

/* thnets.h:191-194: `pooling` names the SpatialMaxPooling whose indices are
 * used, by the value of that module's `nnmodule` member */
struct SpatialMaxUnpooling {
	void *pooling;
};

struct SpatialMaxPooling {
	int padW, padH, dW, dH, kW, kH, ceil_mode;
	int iwidth, iheight;
	THFloatTensor *indices;
	int padW2, padH2;
};

struct SpatialAveragePooling {
	int padW, padH, dW, dH, kW, kH, ceil_mode;
	int iwidth, iheight, count_include_pad;
	int padW2, padH2;
};

struct Linear {
	THFloatTensor *bias, *weight, *addBuffer;
	int commute;
};

struct Threshold {
	float threshold, val, alpha;
	int inplace;
};

struct View {
	int numElements, nDimension;
	long size[4];
};

struct Dropout {
	float p;
	int inplace, v2;
};

struct SpatialBatchNormalization {
	THFloatTensor *running_mean, *running_var, *weight, *bias;
	double eps;
};

struct network;

struct Sequential {
	struct network *net;
};

struct Concat {
	struct network *net;
	int dimension;
};

/* thnets.h:250-288 -- numeric values are part of the ABI. */
enum moduletype {
	MT_Nil,
	MT_SpatialConvolutionMM,
	MT_SpatialConvolutionVirtMM,
	MT_SpatialConvolution,
	MT_SpatialMaxPooling,
	MT_SpatialAveragePooling,
	MT_Linear,
	MT_SoftMax,
	MT_Threshold,
	MT_View,
	MT_Dropout,
	MT_SpatialZeroPadding,
	MT_Reshape,
	MT_Normalize,
	MT_SpatialFullConvolution,
	MT_SpatialMaxUnpooling,
	MT_SpatialBatchNormalization,
	MT_Sequential,
	MT_Concat,
	MT_ConcatTable,
	MT_JoinTable,
	MT_CAddTable,
	MT_CSubTable,
	MT_PReLU,
	MT_Identity,
	MT_Padding,
	MT_LogSoftMax,
	MT_Slice,
	MT_Cmax,
	MT_Upsample,
	MT_LSTM,
	MT_GRU,
	MT_Squeeze,
	MT_Unsqueeze,
	MT_Sigmoid,
	MT_Tanh,
	MT_Transpose
};

#define MAXMODULEINPUTS 16
#define TH_MODULE_UNION_BYTES 80

/* thnets.h:292-336 */
struct module {
	int type;
	THFloatTensor *(*updateOutput)(struct module *m, THFloatTensor *in);
	void (*nnfree)(struct module *m);
	THFloatTensor *output;
	struct network *net;
	void *nnmodule;			/* struct nnmodule * of the .t7 loader */
	char *outputname;
	int ninputs;
	int inputs[MAXMODULEINPUTS];
	union {
		struct SpatialConvolution SpatialConvolution;
		struct SpatialFullConvolution SpatialFullConvolution;
		struct SpatialMaxUnpooling SpatialMaxUnpooling;
		struct SpatialMaxPooling SpatialMaxPooling;
		struct SpatialAveragePooling SpatialAveragePooling;
		struct Linear Linear;
		struct Threshold Threshold;
		struct View View;
		struct Dropout Dropout;
		struct SpatialBatchNormalization SpatialBatchNormalization;
		struct Sequential Sequential;
		struct Concat Concat;
		struct Sequential ConcatTable;
		char abi_pad[TH_MODULE_UNION_BYTES];
	};
};

/* thnets.h:401; the two HIP engines are appended. */
enum {
	ENGINE_CPU, ENGINE_CUDA, ENGINE_OPENCL, ENGINE_OPENCLINIT, ENGINE_LOWP,
	ENGINE_HIP, ENGINE_HIPLOWP
};

/* thnets.h:403-407 */
struct network {
	int nelem, engine;
	struct module *modules;
};

/* thnets.h:571-580 */
typedef struct thnetwork {
	void *netobj;			/* struct thobject * */
	void *statobj;			/* struct thobject * */
	struct network *net;
	void *pynet;			/* struct pyelement * */
	void **allpynodes;		/* struct pyelement ** */
	THFloatTensor *out;
	float mean[3], std[3];
} THNETWORK;

/* Tensor helpers with the reference's semantics (thbasic.c:17-460). */
void THError(const char *fmt, ...);
THFloatTensor *THFloatTensor_new(void);
THFloatStorage *THFloatStorage_new(long size);
THFloatStorage *THFloatStorage_newwithbuffer(void *buffer);
THFloatTensor *THFloatTensor_newWithStorage1d(THFloatStorage *storage, long storageOffset, long size0, long stride0);
THFloatTensor *THFloatTensor_newWithStorage2d(THFloatStorage *storage, long storageOffset, long size0, long stride0, long size1, long stride1);
THFloatTensor *THFloatTensor_newWithTensor(THFloatTensor *tensor);
float *THFloatTensor_data(THFloatTensor *tensor);
long THFloatTensor_nElement(THFloatTensor *t);
void THFloatTensor_resize(THFloatTensor *t, long *size, int nDimension);
void THFloatTensor_resize4d(THFloatTensor *t, long size0, long size1, long size2, long size3);
void THFloatTensor_resize3d(THFloatTensor *t, long size0, long size1, long size2);
void THFloatTensor_resize2d(THFloatTensor *t, long size0, long size1);
void THFloatTensor_resize1d(THFloatTensor *t, long size0);
void THFloatTensor_set(THFloatTensor *tdst, THFloatTensor *tsrc);
void THFloatTensor_free(THFloatTensor *t);

/* ------------------------------------------------------------------ */
/* 2. High level API                                                   */
/* ------------------------------------------------------------------ */

/* thapi.c:335-361 */
void THInit(void);
/* thapi.c:237-242.  `in` must live where the network's engine lives: a
 * device tensor for ENGINE_HIP / ENGINE_HIPLOWP. */
THFloatTensor *THForward(THNETWORK *net, THFloatTensor *in);
/* thapi.c:363-450.  Normalises the caller's buffer in place with
 * mean/std, uploads, runs, downloads; *result is library owned. */
int THProcessFloat(THNETWORK *network, float *data, int batchsize, int width, int height, int nplanes,
	float **result, int *outwidth, int *outheight);
/* thapi.c:452-563.  8-bit HWC images; conversion + normalisation run on the
 * device for the HIP engines. */
int THProcessImages(THNETWORK *network, unsigned char **images, int batchsize, int width, int height, int stride,
	float **result, int *outwidth, int *outheight, int bgr);
/* thapi.c:642-690 */
void THMakeSpatial(THNETWORK *network, int size);
/* thapi.c:692-728.  Only switches the module type tag (MM <-> VirtMM);
 * this library carries no direct-convolution path, mm_type 0 is refused. */
int THUseSpatialConvolutionMM(THNETWORK *network, int mm_type);
/* thapi.c:244-333 for Torch7 model directories: reads <path>/model.net (an
 * nn.Sequential saved with torch.save, binary mode, 8- or 4-byte longs) and,
 * when present, <path>/stat.t7 ({mean = FloatTensor(3), std = FloatTensor(3)})
 * into a host description (engine ENGINE_CPU) for THCreateHipNetwork /
 * THCreateHipLowpNetwork.  Returns 0 with the reason in THLastError() when a
 * file cannot be read; module types the engine does not run are fatal
 * (thload.c:776).  PyTorch dumps and ONNX files are not read. */
THNETWORK *THLoadNetwork(const char *path);
/* A Float / Double tensor saved with torch.save, as a new contiguous host
 * tensor (what thnets-test.c:166-178 does for `-i input.t7` with loadtorch +
 * THFloatTensor_newFromObject, thload.c:408-426, 701-711).  0 on failure. */
THFloatTensor *THLoadTensor(const char *path);
/* thapi.c:601-635: engine networks (frees device state) and the host networks
 * THLoadNetwork returns. */
void THFreeNetwork(THNETWORK *network);
/* thapi.c:637-640 */
int THLastError(void);
/* thapi.c:12; th_profile makes forward() print per-module seconds. */
extern int th_debug, th_profile, th_minmax;
extern double th_convtot, th_convflops;

#endif /* THNETS_IN_TREE */

#define TH_MUSTFREE_HIP 4
#define TH_MUSTFREE_HIP_OF(dtype) (TH_MUSTFREE_HIP + (dtype))
#define TH_IS_HIP_STORAGE(mustfree) ((mustfree) >= TH_MUSTFREE_HIP && (mustfree) <= TH_MUSTFREE_HIP + 3)
#define TH_HIP_STORAGE_DTYPE(mustfree) ((mustfree) - TH_MUSTFREE_HIP)

/* New: the MI355X engine.  Same shape as THCreateCudaNetwork
 * (thapi.c:730-742): returns a new THNETWORK whose modules own device
 * copies of every weight; the source network may be freed afterwards.
 * Conv+Threshold pairs are fused; Linear becomes a 1x1 convolution
 * (cudnn_basic.c:244-265). */
THNETWORK *THCreateHipNetwork(THNETWORK *net);
/* New: counterpart of THCudaHalfFloat (thapi.c:744-755).  0 = fp32,
 * 1 = fp16 storage + fp16 MFMA, 2 = bf16 storage + bf16 MFMA.  Read at
 * engine creation.  Returns 0, or ERR_NOTIMPLEMENTED for other values. */
int THHipHalfFloat(int enable);
/* 1 (default): SpatialBatchNormalization directly after a convolution is folded
 * into the convolution's epilogue at engine creation (the reference folds at
 * load time, absorb_bn, onnx.cc:472-570); 0: it runs as its own kernel like
 * nn_SpatialBatchNormalization_updateOutput.  Applies to engines created
 * afterwards; returns the previous setting. */
int THHipFoldBatchNorm(int enable);
/* Half engines: whether the image layer (3 -> 64 planes, 3x3 / stride 1 / padding 1) is computed by the
 * 3x3 layer after it instead of by a kernel of its own (thhip_conv2d_image_pair; nothing in the reference:
 * its engines run module by module, cudnn/cudnn_basic.c:189-303).  0: never; 2: always; 1 (default): for
 * batches of up to 2048 of that layer's 32 x 8 tiles, where one launch beats two.  The results are the same
 * within the last bit of a half value (another order of the 27 products' sum).  Read at every forward;
 * returns the previous setting. */
int THHipImageLayerInFront(int mode);
/* fp32 convolutions cut the tiles an XCD could not spread evenly over its CUs into parts along K, computed
 * by several workgroups of that XCD (nothing in the reference: its GEMM is one sgemm call per image,
 * modules/SpatialConvolutionMM.c:136-150).  1 (default): the workgroup whose part is ready last adds the
 * parts, in their order, and finishes the tile; the parts meet in the XCD's L2.  That is right while the
 * hardware hands workgroup b of a launch to XCD (b + r) % 8 with one r for the whole launch (r itself
 * changes as queues come and go: other streams, other processes), which every launch checks for itself:
 * its part workgroups record the r they see, and the one that finishes a tile looks at the record.  A
 * launch that saw two is never a silently wrong sum: it switches this setting to 0 for the rest of the
 * process, and THProcessFloat / THProcessImages then run their forward pass once more and return the
 * right values, while a plain synchronisation after THForward reports it as an error (the forward pass
 * has to be run again by the caller).  0: a second launch adds the parts.  The same bits either way.  Read
 * at every launch; returns the previous setting. */
int THHipSumPartsInKernel(int enable);
/* 0 (default): CAddTable / CSubTable compute what the reference's shipped modules
 * compute (modules/CAddTable.c:59-84: with two inputs CAddTable gives a - b and
 * CSubTable a + b; with more, 2a + b + c + ... and 0 - b - c - ...).  1: what the
 * modules' names say (the sum of all inputs; the first minus the others), for
 * networks trained against Torch's modules.  Applies to engines created
 * afterwards; returns the previous setting. */
int THHipTableArithmetic(int as_named);
/* New: the uint8 engine on the GPU, counterpart of THCreateLowpNetwork
 * (thapi.c:784-796, lowp_basic.c:133-212): activations quantised to
 * [-range/2, range/2) in 255 steps, int8 MFMA GEMM with gemmlowp offsets
 * and (multiplier, shift) requantisation (lowp_basic.c:299-321). */
THNETWORK *THCreateHipLowpNetwork(THNETWORK *net, float range);
/* Device <-> host tensors (cudnn_basic.c:64-97 are the CUDA analogues). */
THFloatTensor *THHipTensor_newFromFloatTensor(THFloatTensor *t);
THFloatTensor *THFloatTensor_newFromHipTensor(THFloatTensor *t);
/* Copies module `idx`'s current output of an engine network to the host as
 * float (half / uint8 activations are widened; uint8 codes are returned as
 * code values, not de-quantised).  Returns element count; *dst is malloc'd. */
long THHipNetwork_copyModuleOutput(THNETWORK *net, int idx, float **dst, long size[4], int *ndim);
/* Quantisation (mult, sub) of module `idx`'s output in a HIPLOWP network. */
int THHipNetwork_getModuleQuant(THNETWORK *net, int idx, float *mult, float *sub);
/* Declares the quantisation of the uint8 device tensor the next THForward of
 * a HIPLOWP network will be given (THProcessFloat derives it by itself). */
int THHipNetwork_setInputQuant(THNETWORK *net, float mult, float sub);
/* Device counterpart of THLowpTensor_newFromFloatTensor (lowp_basic.c:5-38):
 * upload, quantise with one min/max over the tensor, and record the result
 * as the quantisation of `net`'s next input. */
THFloatTensor *THHipLowpTensor_newFromFloatTensor(THNETWORK *net, THFloatTensor *t);

/* Drop-in for the reference's only call into gemmlowp (gemm8.cc:4-17,
 * declared lowp_basic.c:290-297): host pointers in and out, the GEMM and
 * requantisation run on the GPU.  Only the all-"transposed" (row-major)
 * form the reference uses is accepted. */
void lowpgemm(const int is_a_transposed, const int is_b_transposed, const int is_c_transposed,
	const int m, const int n, const int k,
	const unsigned char *a, const unsigned char *b, unsigned char *c,
	const int lda, const int ldb, const int ldc,
	const int a_offset, const int b_offset, const int c_offset,
	const int c_mult, const int c_shift);

/* ------------------------------------------------------------------ */
/* 3. Kernel level C ABI (device pointers unless stated)               */
/* ------------------------------------------------------------------ */

/* Element types of device activations / weights. */
enum thhip_dtype { THHIP_F32 = 0, THHIP_F16 = 1, THHIP_BF16 = 2, THHIP_U8 = 3 };

/* Runtime plumbing. */
int thhip_device_count(void);
void *thhip_malloc(size_t bytes);
void thhip_free(void *p);
void thhip_memcpy_h2d(void *dst, const void *src, size_t bytes);
void thhip_memcpy_d2h(void *dst, const void *src, size_t bytes);
void thhip_memcpy_d2d(void *dst, const void *src, size_t bytes);
/* Page-locked host memory and copies that are queued on the engine's stream
 * without waiting for them (the host side must be such memory); what the
 * ENGINE_HIP branches of THProcessFloat / THProcessImages stage their data
 * through (the CUDA engine copies from pageable memory, cudnn_basic.c:64-80). */
void *thhip_host_malloc(size_t bytes);
void thhip_host_free(void *p);
void thhip_memcpy_h2d_async(void *dst, const void *src_pinned, size_t bytes);
void thhip_memcpy_d2h_async(void *dst_pinned, const void *src, size_t bytes);
void thhip_memset(void *dst, int value, size_t bytes);
/* How many allocating requests (device or page-locked memory taken or given
 * back, events created) the library has made of the HIP runtime so far: a test
 * aid for the entry point that promises none. */
long thhip_alloc_calls(void);
void thhip_sync(void);
/* Events on the engine's stream: slots 0..63. thhip_event_ms(a,b) syncs b. */
void thhip_event_record(int slot);
float thhip_event_ms(int slot_start, int slot_stop);
/* Per-kernel-family accumulated time (ms) and launch count measured with
 * events around every launch while profiling is on (family ids below).
 * thhip_profile_enable: 0 off, 1 every family, otherwise the sum of
 * 2 << family over the families to time (an event pair costs a few
 * microseconds of stream time per launch). */
enum thhip_family { THHIP_FAM_CONV = 0, THHIP_FAM_GEMV = 1, THHIP_FAM_CONV_I8 = 2, THHIP_FAM_OTHER = 3, THHIP_FAM_COUNT = 4 };
void thhip_profile_enable(int on);
void thhip_profile_reset(void);
void thhip_profile_get(int family, double *ms, long *launches, double *work);
/* What the matrix cores sustain from registers alone on this device: a loop of
 * MFMAs (fp32 32x32x2, fp16 32x32x16 or int8 32x32x32; dtype THHIP_F32 /
 * THHIP_F16 / THHIP_U8) on four accumulators per wavefront, `waves_per_simd`
 * (1..8) wavefronts resident per SIMD, run for about `ms` milliseconds; returns
 * operations per second (two per multiply-add).  A measurement aid (the
 * reference has none: its thnets-test.c:214-235 prints GFLOP/s of whole layers). */
double thhip_probe_mfma(int dtype, int waves_per_simd, double ms);

/* Weight packing for the implicit-GEMM convolution: row-major
 * [Co][Ci][kHW = kH*kW] (SpatialConvolutionMM.c:141-144) -> the K-chunked,
 * M-interleaved layout the kernel streams (tap-major along K when Ci is a
 * multiple of the kernel's plane block).  Returns a device buffer. */
void *thhip_conv_pack_weight(const float *w_host, int Co, int Ci, int kHW, int dtype);
size_t thhip_conv_packed_bytes(int Co, int Ci, int kHW, int dtype);
/* The inverse: packed -> row-major [Co][Ci*kHW] in the same dtype (new device buffer). */
void *thhip_conv_unpack_rows(const void *wpacked, int Co, int Ci, int kHW, int dtype);

/* Replaces nn_SpatialConvolutionMM_updateOutput's per-image
 * im2col + sgemm + bias (SpatialConvolutionMM.c:75-109, 126-225) and, when
 * `act` != 0, the following nn_Threshold_updateOutput
 * (Threshold.c:38-63): y = x > thr ? x : val applied to the sum.
 * x: [B,Ci,H,W], y: [B,Co,oH,oW], both NCHW contiguous in `dtype`;
 * wpacked from thhip_conv_pack_weight; bias fp32 [Co] or NULL. */
void thhip_conv2d(const void *x, const void *wpacked, const float *bias, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype);

/* The same convolution with a per-plane factor before the bias:
 *     y = act(scale[o] * sum + shift[o]),
 * which is a convolution followed by SpatialBatchNormalization with
 * scale = invstd * weight and shift = (bias - mean) * scale + bn_bias
 * (SpatialBatchNormalization.c:57-116; the reference's own folding is
 * absorb_bn, onnx.cc:529-557).  scale == NULL is thhip_conv2d. */
void thhip_conv2d_affine(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype);

/* Half types (fp16 / bf16) with the memory order chosen per side, as for the
 * uint8 entry points below: x_layout 0 = the reference's [B][C][H][W],
 * 1 = channels-last [B][H][W][C] (Ci % 8 == 0; weights packed with
 * thhip_conv_pack_weight_layout for it); y_channels_last likewise (Co % 4 == 0).
 * The half engines keep activations channels-last between convolutions so
 * that the eight values of one MFMA operand vector are one 16-byte load.
 * Same arithmetic and reference lines as thhip_conv2d_affine. */
void *thhip_conv_pack_weight_layout(const float *w_host, int Co, int Ci, int kH, int kW, int dtype, int x_layout);
void thhip_conv2d_layout(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype, int x_layout, int y_channels_last);

/* thhip_conv2d_layout followed by a 2x2 / stride 2 max pooling without padding
 * (floor mode) in one kernel: y is [B][Co][oH/2][oW/2] (or channels-last), the
 * Threshold applied before the pooling as the modules run.  Replaces the module
 * sequence SpatialConvolutionMM -> Threshold -> SpatialMaxPooling
 * (modules/SpatialMaxPooling.c:6-98 after SpatialConvolutionMM.c:111-225) for the
 * layers thhip_conv2d_pool2_supported accepts: half types, channels-last input
 * with planes in blocks of 32 (the kernel that keeps an input patch in LDS for
 * 3x3 / stride 1 layers of 64, 128, 256 or 512 planes with enough tiles, else the tiles
 * loaded straight into LDS); fp32, plane-major tensors, planes in blocks of 32, any
 * kernel size and stride, more than 512 tiles of 64 planes x 64 positions (the
 * layers that run without a K split): the kernel then walks the positions window
 * by window, the four of a window in neighbouring lanes, and a last odd row or
 * column of the convolution, which the pooling drops, is never computed. */
int thhip_conv2d_pool2_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int dtype, int x_layout, int y_channels_last);
void thhip_conv2d_layout_pool2(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype, int x_layout, int y_channels_last);

/* Replaces SpatialConvolutionMM -> (SpatialBatchNormalization, folded) -> Threshold ->
 * SpatialMaxPooling(3, 3, 2, 2, ppad, ppad) (modules/SpatialConvolutionMM.c:126-225,
 * modules/SpatialMaxPooling.c:168-247) for an fp32 image layer: at most four
 * plane-major input planes, whole blocks of 64 output planes, strides up to 4,
 * pooled rows of whole groups of 14 positions (ResNet-18's 7x7 / stride 2 stem
 * at 224 x 224).  One kernel; the convolution's output is never written.  y is
 * [B][Co][pH][pW]. */
int thhip_conv2d_image_pool_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode, int dtype, int x_layout);
void thhip_conv2d_image_pool(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int ppad,
	int act, float thr, float val, int dtype);

/* Replaces two modules and what is folded into them: the image layer
 * SpatialConvolutionMM(3 -> 64, 3x3, stride 1, padding 1) (-> batch norm, folded) -> Threshold,
 * and the 3x3 / stride 1 / padding 1 layer of 64 input planes that follows with its own
 * (-> SpatialMaxPooling(2, 2, 2, 2) when pool2 is set), for the half types
 * (modules/SpatialConvolutionMM.c:126-225 twice, modules/Threshold.c:38-63,
 * modules/SpatialMaxPooling.c:6-98).  One kernel: the first layer's output, 64 planes a
 * pixel, is computed patch by patch in LDS and never written.  img: [B][3][H][W]
 * plane-major, W even; wfront: the first layer's [64][3][3][3] weights from
 * thhip_conv_pack_weight_image_front (6 KiB on the device, thhip_free); wpacked: the second
 * layer's weights as for thhip_conv2d_layout with channels-last input; y: channels-last,
 * [B][H][W][Co] or [B][H/2][W/2][Co]; Co at most 256, a multiple of 8. */
void *thhip_conv_pack_weight_image_front(const float *w, int dtype);
int thhip_conv2d_image_pair_supported(int B, int H, int W, int Co1, int Co2, int dtype, int y_channels_last);
void thhip_conv2d_image_pair(const void *img, const void *wfront, const float *scale1, const float *shift1,
	int act1, float thr1, float val1, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int H, int W, int Co, int act, float thr, float val, int pool2, int dtype);

/* Two convolutions that do not depend on each other as one launch (nothing in the reference, whose
 * modules run one after the other, thapi.c:158-235: the shortcut's 1x1 projection of a residual block
 * beside the block's first convolution, modules/ConcatTable.c).  The convolution call right after _begin
 * is held back if its kernel can run it whole (fp32, no K split, no cut tiles) and goes out in one grid
 * with the next call if that runs on the same kernel; otherwise right after that call, or at _end.  The
 * caller guarantees that neither of the two layers reads the other's output. */
void thhip_conv_pair_begin(void);
void thhip_conv_pair_end(void);

/* thhip_conv2d_affine followed by a max pooling of any window, stride, padding and
 * rounding (modules/SpatialMaxPooling.c:6-98; the module sequence SpatialConvolutionMM
 * -> Threshold -> SpatialMaxPooling), y = [B][Co][pH][pW] from thhip_pool_outsize of the
 * convolution's output.  For the layers thhip_conv2d_poolk_supported accepts: fp32,
 * plane-major, at most 512 tiles of 64 planes x 64 positions (a batch of one or a few
 * images), i.e. the layers whose K is split over workgroups and whose parts a second
 * kernel adds: that kernel takes the maximum of every window too, and the pooling's own
 * launch is saved.  The same values, bit for bit, as thhip_conv2d_affine followed by
 * thhip_maxpool. */
int thhip_conv2d_poolk_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppH, int ppW, int ceil_mode, int dtype);
void thhip_conv2d_poolk(const void *x, const void *wpacked, const float *scale, const float *shift, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int pkH, int pkW, int pdH, int pdW, int ppH, int ppW, int ceil_mode,
	int act, float thr, float val, int dtype);

/* thhip_conv2d_affine followed by the two-input table add of a residual block and
 * the Threshold(0, 0) after it, in the convolution's epilogue.  With v = the
 * convolution's result (after factor, bias and its own Threshold) and r = res (a
 * device tensor of y's shape): y = v + c r (mode 1) or r + c v (mode 2), then
 * max(y, 0) if res_act.  Replaces SpatialConvolutionMM -> CAddTable -> Threshold
 * (modules/CAddTable.c:59-70; c = -1 is the reference's two-input CAddTable, which
 * subtracts) for the layers thhip_conv2d_residual_supported accepts (fp32,
 * plane-major tensors, input planes in blocks of 32); bit for bit the values of
 * thhip_conv2d_affine followed by thhip_axpby2. */
int thhip_conv2d_residual_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int dtype);
void thhip_conv2d_residual(const void *x, const void *wpacked, const float *scale, const float *shift,
	const void *res, int mode, float c, int res_act, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int act, float thr, float val, int dtype);


/* Replaces nn_Linear_updateOutput's 1-D branch (Linear.c:86-90 ->
 * thbasic.c:713-741 -> sgemv.c:48-105): y = bias + W x, W row-major
 * [nOut][nIn] fp32/fp16/bf16, optional fused threshold. */
void thhip_gemv(const void *x, const void *w, const float *bias, void *y,
	int nIn, int nOut, int act, float thr, float val, int dtype);

/* Replaces nn_Linear_updateOutput's matrix branch for a small batch
 * (Linear.c:92-108: addmm with beta 0, then the rank-1 bias update through
 * addr / sger, thbasic.c:757-789): Y[b][o] = bias[o] + sum_k W[o][k] X[b][k],
 * X [B][nIn], W row-major [nOut][nIn], Y [B][nOut].  thhip_linear_batched_supported
 * says whether the shape is taken (B <= 128, run in slices of 64 that each read
 * the weights; rows in 16-byte vectors: nIn % 4 == 0 for fp32, % 8 for the half
 * types); other shapes run as a 1x1 convolution through thhip_conv2d. */
int thhip_linear_batched_supported(int B, int nIn, int nOut, int dtype);
void thhip_linear_batched(const void *x, const void *wrow, const float *bias, void *y,
	int B, int nIn, int nOut, int act, float thr, float val, int dtype);

/* thhip_linear_batched for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same arguments, same kernels and the same bits
 * as thhip_linear_batched; the partial sums of the K slices go to a fixed array of
 * thhip_linear_batched_noalloc_limit() bytes (8 MiB) that every GPU the library
 * runs on holds until the process ends, instead of a buffer that grows on demand.
 * The call allocates and frees nothing on the device or through the runtime.
 * Returns 0, or (with a message on stderr, nothing launched) -1 for a shape
 * thhip_linear_batched_supported refuses, -2 when a slice of 64 batch rows needs
 * more than the array holds (K slices x rows x nOut x 4 bytes; e.g. 25088 -> 4096
 * at batch 16 needs 2 MiB), -3 when the array's address cannot be resolved.
 * thhip_linear_batched_noalloc_init() resolves the address for the current device
 * ahead of the first call (THInit calls it).  Calls that overlap on one GPU share
 * the array and race; calls on the library's stream, one after the other, do not. */
int thhip_linear_batched_noalloc(const void *x, const void *wrow, const float *bias, void *y,
	int B, int nIn, int nOut, int act, float thr, float val, int dtype);
int thhip_linear_batched_noalloc_init(void);
size_t thhip_linear_batched_noalloc_limit(void);

/* Replaces FindMinMax (thapi.c:141-154), which the executor prints after every
 * module when th_minmax is set (thapi.c:197-202): smallest and largest of n
 * elements of the given type on the device (codes as numbers for uint8),
 * +inf / -inf for n = 0, NaNs skipped as the reference's comparisons skip them. */
void thhip_minmax(const void *x, long n, int dtype, float *min_out, float *max_out);

/* Replaces nn_Threshold_updateOutput (Threshold.c:38-63), out of place or
 * in place (y == x).  alpha != 0 selects the LeakyReLU branch. */
void thhip_threshold(const void *x, void *y, long n, float thr, float val, float alpha, int inplace, int dtype);

/* Replaces nn_SpatialMaxPooling_updateOutput (SpatialMaxPooling.c:168-247)
 * and Lowp_SpatialMaxPooling_updateOutput (lowp_SpatialMaxPooling.c:45-108);
 * oH/oW come from thhip_pool_outsize. */
void thhip_maxpool(const void *x, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype);
void thhip_pool_outsize(int H, int W, int kH, int kW, int dH, int dW, int padH, int padW, int ceil_mode,
	int *oH, int *oW);
/* nn_SpatialMaxPooling_updateOutput including its `indices` output
 * (SpatialMaxPooling.c:100-114), fp32 / fp16 / bf16: ind[i] = position of the
 * first maximum inside the input plane (the reference stores position + 1 as a
 * float), -1 for an empty window. */
void thhip_maxpool_indices(const void *x, void *y, int *ind, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype);
/* Replaces nn_SpatialMaxUnpooling_updateOutput (SpatialMaxUnpooling.c:43-120):
 * x [B][C][oH][oW] and the indices of the pooling described by the geometry
 * arguments (H x W in, oH x oW out) -> y [B][C][H][W], zero where no window's
 * maximum sat; of several windows naming one element the last in row-major
 * order gives the value, as in the reference's serial loop.  An index outside
 * the plane (THError in the reference) matches nothing. */
void thhip_maxunpool(const void *x, const int *ind, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype);

/* Replaces nn_SpatialFullConvolution_updateOutput
 * (SpatialFullConvolution.c:136-250) for fp32 / fp16 / bf16: x [B][Ci][H][W],
 * w [Ci][Co][kH][kW] -> y [B][Co][oH][oW], oH = (H-1)*dH - 2*padH + kH + adjH.
 * thhip_fullconv_pack_weight packs the host weights once (device pointer,
 * thhip_free); thhip_fullconv2d multiplies (the MFMA convolution kernel as a
 * 1x1 convolution with Co*kH*kW output planes, into `col`: device scratch of
 * B*Co*kH*kW*H*W elements) and gathers (thhip_col2im, the reference's col2im
 * :104-134 without scatter).  With a bias the result is beta * sum + bias[o]
 * -- the reference passes beta = 11 to its bias GEMM (:231-237), so 11
 * reproduces it and 1 is the textbook operator; without a bias the plain sum.
 * act / thr / val: fused Threshold as in thhip_conv2d. */
void *thhip_fullconv_pack_weight(const float *w, int Ci, int Co, int kH, int kW, int dtype);
void thhip_fullconv2d(const void *x, const void *wp, const float *bias, float beta, void *col, void *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW, int adjH, int adjW,
	int act, float thr, float val, int dtype);
void thhip_col2im(const void *col, const float *bias, float beta, void *y, int B, int Co, int H, int W,
	int kH, int kW, int dH, int dW, int padH, int padW, int adjH, int adjW, int act, float thr, float val, int dtype);

/* Replaces nn_SpatialAveragePooling_updateOutput
 * (SpatialAveragePooling.c:71-207). */
void thhip_avgpool(const void *x, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int count_include_pad, int dtype);

/* Replaces nn_SoftMax_updateOutput (SoftMax.c:24-90) with the reference's
 * polynomial exp approximation (thbasic.c:462-491). */
void thhip_softmax(const void *x, void *y, long nframe, long dim, long stride, int dtype);

/* Replaces nn_SpatialBatchNormalization_updateOutput
 * (SpatialBatchNormalization.c:57-116); scale/shift are fp32 device arrays
 * holding mean, invstd, weight, bias per plane. */
void thhip_batchnorm(const void *x, void *y, long B, long C, long HW,
	const float *mean, const float *invstd, const float *weight, const float *bias, int dtype);

/* Replaces nn_CAddTable_updateOutput's two-input branch
 * (CAddTable.c:59-70): y[j] = a[j] + sign*b[j] for j < nb, y[j] = a[j]
 * beyond; sign = -1 reproduces the reference's MT_CAddTable arithmetic. */
void thhip_axpby2(const void *a, const void *b, void *y, long na, long nb, float sign, int act, int dtype);

/* fp32 host-layout conversions on the device. */
void thhip_convert(const void *src, int src_dtype, void *dst, int dst_dtype, long n);

/* The normalisation loop of THProcessFloat (thapi.c:389-403) on a device copy
 * of the caller's [B][C][HW] fp32 data: planes 0..2 become (x - mean) / std,
 * further planes pass through; dst takes the engine's float dtype.  Same bits
 * as the host loop (fp32 subtraction, correctly rounded division). */
void thhip_normalize(const float *src, void *dst, int B, int C, long HW, const float *mean3, const float *std3,
	int dtype);

/* Replaces rgb2float / bgr2float (thapi.c:20-46; CUDA analogue
 * cudnn_copy.cu:13-116): one interleaved 8-bit image (device copy, `stride`
 * bytes per row, cp planes) -> normalised planar dst in `dtype`. */
void thhip_rgb2float(void *dst, const unsigned char *src, int width, int height, int stride, int cp,
	const float *mean, const float *std, int bgr, int dtype);
/* The loop over the images of THProcessImages (thapi.c:489-496, 509-515) as one
 * launch: n images, `src_pitch` bytes apart in src, -> n consecutive planar
 * tensors in dst. */
void thhip_rgb2float_batch(void *dst, const unsigned char *src, int n, long src_pitch, int width, int height,
	int stride, int cp, const float *mean, const float *std, int bgr, int dtype);

/* ---- uint8 (LOWP) path ---- */

/* Replaces THLowpTensor_newFromFloatTensor's arithmetic
 * (lowp_basic.c:15-35) on the device: min/max (including 0) over n floats,
 * then q = roundf(v*mult) - roundf(min*mult).  mult/sub returned to host. */
void thhip_quantize(const float *x, unsigned char *q, long n, float *mult, float *sub);
/* Replaces THFloatTensor_newFromLowpTensor (lowp_basic.c:40-58). */
void thhip_dequantize(const unsigned char *q, float *x, long n, float mult, float sub);

/* Weight packing for the int8 kernel: uint8 codes [Co][Ci][kHW] -> signed
 * (code-128) K-chunked layout + per-row sums.  Returns a device buffer. */
void *thhip_conv_pack_weight_u8(const unsigned char *w_host, int Co, int Ci, int kHW);
/* The same for a stated way of reading the input (codes [Co][Ci][kH][kW]):
 *   x_layout 0  plane-major [B][C][H][W], as thhip_conv_pack_weight_u8;
 *   x_layout 1  channels-last [B][H][W][C] in memory (K runs tap-major,
 *               k = tap * Ci + plane; Ci % 16 == 0);
 *   x_layout 2  plane-major in memory with Ci <= 4 (the image layer): the
 *               convolution first copies it to [B][H][W][4] so that four
 *               neighbouring pixels of a kernel row are one operand vector.
 * The packed buffer is only valid for calls with the same x_layout. */
void *thhip_conv_pack_weight_u8_layout(const unsigned char *w_host, int Co, int Ci, int kH, int kW, int x_layout);

/* Replaces Lowp_SpatialConvolution_updateOutput's per-image
 * uint8 im2col + THLowpTensor_mm/lowpgemm + lowpadd
 * (lowp_SpatialConvolution.c:5-120, lowp_basic.c:299-321, gemm8.cc:13-16):
 * acc = sum_k (w+a_off)(x+b_off) with x = `zero` in the padding,
 * c = clamp(((acc+c_off)*c_mult + round) >> c_shift, 0, 255),
 * then per-plane saturating add of addend[o] with the reference's
 * unclamped-below tail for the last (oH*oW)%8 elements of each plane,
 * then (act != 0) the uint8 threshold q > thr ? q : val. */
void thhip_conv2d_u8(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift,
	int act, int thr, int val);

/* thhip_conv2d_u8 with the memory order chosen per side.  x_layout as in
 * thhip_conv_pack_weight_u8_layout (and the weights packed for it);
 * y_channels_last 0 = the reference's [B][C][H][W], 1 = [B][H][W][C], the
 * order the uint8 engine keeps between convolutions so that the 16 codes of
 * one MFMA operand vector are one 16-byte load.  Same arithmetic and the same
 * reference lines; the tail rule of lowpadd still goes by the position inside
 * the plane.  Channels-last y needs Co % 4 == 0. */
void thhip_conv2d_u8_layout(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift,
	int act, int thr, int val, int x_layout, int y_channels_last);

/* The same when x is followed by x_tail_bytes (>= 64 to matter) bytes holding the
 * code `zero`: channels-last layers with Ci % 64 == 0 then run on the kernel
 * that loads its operands straight into LDS and fetches its padding from that
 * tail (a load out of the buffer's range would give code 0 instead).  No
 * counterpart in the reference: its im2col fills the padding itself
 * (lowp_SpatialConvolution.c:90-134). */
void thhip_conv2d_u8_layout_tail(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift,
	int act, int thr, int val, int x_layout, int y_channels_last, int x_tail_bytes);

/* Lowp_SpatialMaxPooling_updateOutput (lowp_SpatialMaxPooling.c:45-108) on
 * channels-last codes, C % 4 == 0. */
void thhip_maxpool_u8_cl(const unsigned char *x, unsigned char *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW);

/* Codes from [B][C][HW] to [B][HW][C] memory order (to_channels_last = 1) or
 * back (0).  No counterpart in the reference, whose tensors are always
 * plane-major; used where the engine's internal order meets the API. */
void thhip_relayout_u8(const unsigned char *x, unsigned char *y, int B, int C, int HW, int to_channels_last);
/* The same for any element type of the engine (dtype gives the element size),
 * and max pooling on channels-last tensors of the half types (C % 8 == 0) or
 * codes (SpatialMaxPooling.c:168-247 / lowp_SpatialMaxPooling.c:45-108). */
void thhip_relayout(const void *x, void *y, int B, int C, int HW, int to_channels_last, int dtype);
void thhip_maxpool_cl(const void *x, void *y, int B, int C, int H, int W, int oH, int oW,
	int kH, int kW, int dH, int dW, int padH, int padW, int dtype);

/* thhip_conv2d_u8 for an image layer (at most four planes, plane-major x
 * [B][Ci][H][W], W % 4 == 0, horizontal stride 4, Co % 64 == 0, wpacked from
 * thhip_conv_pack_weight_u8_layout(..., 2)) followed by the uint8 Threshold and a
 * 3x3 / stride 2 max pooling without padding (floor mode), in one kernel: replaces
 * Lowp_SpatialConvolution_updateOutput -> Lowp_Threshold_updateOutput ->
 * Lowp_SpatialMaxPooling_updateOutput (lowp_SpatialConvolution.c:124-187,
 * lowp_Threshold.c:3-28, lowp_SpatialMaxPooling.c:45-108) for AlexNet's stem.  y is
 * channels-last [B][pH][pW][Co], pH = (oH - 3) / 2 + 1; the convolution output is
 * never written.  thhip_conv2d_u8_image_pool_supported says whether the shapes
 * (convolution, then the pooling's kH kW dH dW padH padW ceil_mode) are taken. */
int thhip_conv2d_u8_image_pool_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pkH, int pkW, int pdH, int pdW, int ppadH, int ppadW, int ceil_mode);
void thhip_conv2d_u8_image_pool(const unsigned char *x, const void *wpacked, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val);

/* thhip_conv2d_u8 for stride-1 layers on small channels-last images (x [B][H][W][Ci],
 * Ci % 64 == 0, Co % 64 == 0, at least four taps, output rows of at most 64 positions when
 * pooling and 192 otherwise), by a kernel that copies the input patch of a band of output
 * rows into LDS once per block of 64 planes and takes every tap's operand from there, so
 * that only the weights stream; optionally (pool = 1) with the 3x3 / stride 2 max pooling
 * without padding (floor mode) that follows.  Replaces the same reference lines as
 * thhip_conv2d_u8_image_pool.  wpatch comes from thhip_conv_pack_weight_u8_patch (host codes
 * [Co][Ci][kH][kW]; K order: block of 64 planes, tap, plane).  y is channels-last,
 * [B][oH][oW][Co] or the pooled [B][(oH - 3) / 2 + 1][(oW - 3) / 2 + 1][Co]. */
int thhip_conv2d_u8_patch_supported(int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW,
	int padH, int padW, int pool);
void *thhip_conv_pack_weight_u8_patch(const unsigned char *w, int Co, int Ci, int kH, int kW);
void thhip_conv2d_u8_patch(const unsigned char *x, const void *wpatch, const int *addend, unsigned char *y,
	int B, int Ci, int H, int W, int Co, int kH, int kW, int dH, int dW, int padH, int padW,
	int zero, int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val, int pool);

/* The same arithmetic as thhip_conv2d_u8 for layers with one output position
 * per image (Linear, or a window covering its whole input): x [B][K] codes,
 * wfrag from thhip_linear_pack_weight_u8 (row-major [nOut][K] host codes ->
 * device copy re-centred to signed bytes, in the order the kernel streams them:
 * 16-row blocks x 64-code K-steps, one matrix-core fragment after the other),
 * rowsum from thhip_u8_rowsums, y [B][nOut].  Replaces the same reference
 * lines; B <= 64, K % 16 == 0.  One kernel: a workgroup owns 16 rows and all of
 * K, sums its wavefronts' tiles through LDS and requantises. */
int thhip_linear_batched_u8_supported(int B, int K, int nOut);
unsigned char *thhip_linear_pack_weight_u8(const unsigned char *w_host, int nOut, int K);
int *thhip_u8_rowsums(const unsigned char *w_host, int nOut, int K);
void thhip_linear_batched_u8(const unsigned char *x, const unsigned char *wfrag, const int *rowsum,
	const int *addend, unsigned char *y, int B, int K, int nOut,
	int a_off, int b_off, int c_off, int c_mult, int c_shift, int act, int thr, int val);

/* Replaces Lowp_LoadImages (lowp_basic.c:60-131) for one image: interleaved
 * 8-bit pixels (device copy, `stride` bytes per row, 3 planes) -> planar uint8
 * codes [3][height][width] in the fixed input range the reference derives from
 * mean / std; (*mult, *sub) receive that range's quantisation. */
void thhip_rgb2code(unsigned char *dst, const unsigned char *src_dev, int width, int height, int stride,
	const float *mean, const float *std, int bgr, float *mult, float *sub);
/* All n images of Lowp_LoadImages' loop (lowp_basic.c:113-130) in one launch. */
void thhip_rgb2code_batch(unsigned char *dst, const unsigned char *src_dev, int n, long src_pitch, int width,
	int height, int stride, const float *mean, const float *std, int bgr, float *mult, float *sub);

/* Replaces Lowp_Threshold_updateOutput (lowp_Threshold.c:3-28) on codes. */
void thhip_threshold_u8(const unsigned char *x, unsigned char *y, long n, int thr, int val, int inplace);

/* Replaces Lowp_SoftMax_updateOutput (lowp_SoftMax.c:3-89); returns the
 * output (mult) it derives (sub is 0). */
float thhip_softmax_u8(const unsigned char *x, unsigned char *y, long nframe, long dim, long stride,
	float in_mult, float in_sub);

#ifdef __cplusplus
}
#endif

#endif
