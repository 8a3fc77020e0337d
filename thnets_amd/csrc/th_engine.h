/* Engine-private declarations shared by the host C files (not installed). */
#ifndef TH_ENGINE_H
#define TH_ENGINE_H

#include "../../include/thnets_hip.h"

/* Per-module state the engine keeps beside `struct module` (index-parallel to
 * network.modules), so that the public structure keeps the reference layout. */
/* uint8 outputs: bytes of the code of 0.0 (128 for every convolution output) kept after the tensor */
#define TH_U8_TAIL 64
#define TH_U8_TAIL_CODE 128

struct hipmod {
	int fused_act;		/* the following Threshold is applied in this module's epilogue */
	float thr, val;
	int passthrough;	/* a Threshold whose work was folded into its producer */
	int pool_next;		/* convolution: index of a 2x2 / stride 2 max pooling its epilogue may do (0: none) */
	int pooled_by_producer;	/* max pooling: the convolution before it did the pooling in this forward */
	/* fp32 residual blocks: the table add (and the Threshold folded into it) done by the epilogue of the
	 * last convolution that runs in the ConcatTable before it */
	int res_mode;		/* convolution: 1: result + res_c * other branch, 2: other branch + res_c * result; 0: none */
	float res_c;
	int res_act;
	struct hipmod *res_add;	/* convolution: the table add's state, told when the epilogue did its work */
	const void *res_ptr;	/* convolution: the other branch's values for this forward (set by the ConcatTable) */
	long res_n;
	struct hipmod *res_target;	/* ConcatTable: the convolution planned to do the add, or NULL */
	int res_from_input;	/* ConcatTable: the other branch is the identity (the table's input), else branch 0's output */
	int shortcut_first;	/* ConcatTable: the shortcut (one convolution) runs first, in one launch with the main branch's first
				 * convolution, and the main branch's last convolution adds its output */
	int added_by_producer;	/* table add: 1 + the branch whose convolution did the add in this forward */
	int table_named;	/* table add / subtract: what the module's name says instead of the shipped arithmetic (THHipTableArithmetic) */
	int is_linear;		/* MT_Linear in the source network */
	int owns_output;	/* output storage was allocated by this module */
	size_t cap;		/* bytes allocated for the output */
	size_t tail_at;		/* uint8: offset at which the padding-code tail was last written */
	void *wpacked;		/* convolution weights in the kernel's packed layout (device) */
	void *wrow;		/* the same weights row-major, made on first matrix-vector use (device) */
	float *bias;		/* fp32 bias (device) */
	float *scale;		/* fp32 per-plane factor of a folded batch norm, applied before the bias (device), or NULL */
	float *bn[4];		/* mean, invstd, weight, bias per plane (device) */
	long bn_planes;
	/* uint8 engine */
	int *addend;		/* per-plane bias addend (device) */
	unsigned char *wrow_u8;	/* row-major weight codes for one-position layers (device) */
	void *wpatch_u8;	/* the weights packed for the kernel that keeps the input patch in LDS (device), or NULL */
	int *rowsum_u8;		/* their re-centred row sums (device) */
	unsigned char *wq_host;	/* weight codes on the host, only while the network is being built */
	/* SpatialFullConvolution: columns scratch; SpatialMaxPooling feeding a SpatialMaxUnpooling: its indices */
	void *col;
	size_t col_cap;
	int *pool_ind;
	size_t pool_ind_cap;
	int want_indices;	/* a SpatialMaxUnpooling of this network reads this pooling's indices */
	int pool_index;		/* SpatialMaxUnpooling: position of its pooling in the network */
	/* half engines: the network's image layer (3 -> 64 planes, 3x3 / stride 1 / padding 1) may be computed by the
	 * 3x3 layer that follows it, patch by patch in LDS, and then writes nothing (thhip_conv2d_image_pair) */
	int front_of;		/* image layer: position of that following convolution (0: none) */
	int front;		/* that convolution: position of the image layer + 1 (0: none) */
	void *wfront;		/* image layer: its weights packed for that kernel (device) */
	int deferred;		/* image layer: in this forward its output was left to the convolution after it (not written) */
	const void *front_img;	/* image layer: its input of this forward, [B][3][H][W] */
	int front_B, front_H, front_W;
	int in_cl, out_cl;	/* input / output codes are channels-last [B][H][W][C] in memory */
	int x_layout;		/* how the convolution reads its input: thhip_conv_pack_weight_u8_layout */
	float wm, wsub;		/* weight quantisation */
	float q_mult, q_sub;	/* quantisation of this module's output */
};

/* Staging memory of THProcessFloat / THProcessImages, kept with the top-level network
 * between calls (th_io.c). */
struct hipio_buf { THFloatTensor *t; size_t cap; };	/* a device tensor and the bytes behind it */
struct hipio_pin { void *ptr; size_t cap; };		/* page-locked host memory */
struct hipio {
	struct hipio_buf in_raw;	/* the caller's floats as uploaded */
	struct hipio_buf in_dev;	/* normalised input in a half type; planes made from 8-bit images */
	struct hipio_buf in_q;		/* uint8 engine: input codes */
	struct hipio_buf out_f;		/* a half or uint8 result as floats */
	struct hipio_buf img;		/* 8-bit images as uploaded */
	struct hipio_pin pin_in, pin_out;
};

/* A `struct network` with the engine's state behind it. */
struct hipnet {
	struct network pub;	/* must be first */
	struct hipmod *hm;
	int dtype;		/* enum thhip_dtype of activations */
	float range;
	float cur_mult, cur_sub;	/* uint8 engine: quantisation of the tensor in flight */
	int cur_cl;		/* uint8 engine: the tensor in flight is channels-last in memory */
	int dag;		/* modules name their inputs (ninputs / inputs[]): the list is a graph */
	int no_windows;		/* the first modules do not all honour a window of the batch (found on the first try) */
	struct hipio io;
};

struct hipnet *hipnet_of(struct module *m);
struct hipmod *hipmod_of(struct module *m);
void *thhip_tensor_ptr(THFloatTensor *t, int dtype);
int thhip_engine_dtype(void);
struct network *THHip_ToHip(struct network *net, int lowp, float range);
THFloatTensor *thhip_forward(struct network *net, THFloatTensor *in);
void thhip_free_network(struct network *net);
void thhip_materialize_output(struct network *net, int idx);
/* th_io.c */
void thhip_storage_release(THFloatStorage *s);
THFloatTensor *thhip_device_tensor_like(THFloatTensor *t, int dtype);
THFloatTensor *thhip_upload_as(THFloatTensor *t, int dtype);
THFloatTensor *thhip_download_as_float(THFloatTensor *t, int dtype);
THFloatTensor *thhip_process_float(THNETWORK *network, float *data, int batchsize, int width, int height, int nplanes);
THFloatTensor *thhip_process_images(THNETWORK *network, unsigned char **images, int batchsize, int width, int height,
	int stride, int bgr);
void thhip_io_free(struct hipnet *hn);
/* th_load.c */
int thhip_load_error(void);
/* hip_rt.hip: whether the GPU hands the workgroups of a launch to the XCDs in order (probed once); the flag
 * a kernel raises when it finds that its launch was not (a repeat or an error at the next synchronisation) */
unsigned thhip_xcd_map(void);
int *thhip_fault_flag(void);
/* hip_rt.hip: a caller that can repeat its forward pass holds the error of such a report back (1 / 0) and
 * asks afterwards whether one came (the fault's code, 0: none) */
void thhip_fault_hold(int on);
int thhip_fault_take(void);
/* hip_rt.hip: a window of the batch for the convolution entry points (0 images: none); whether anything
 * was launched outside them while one was set (clears the note); a host -> device copy on the copy stream
 * followed by event `event`, and the engine's stream made to wait for that event */
void thhip_batch_window(int b0, int n);
int thhip_batch_window_violated(void);
void thhip_memcpy_h2d_piece(void *dst, const void *src_pinned, size_t bytes, int event);
void thhip_wait_h2d_piece(int event);
/* th_engine.c: thhip_forward with the first modules run window by window; before(ctx, w) is called
 * before the modules see window w (to make its images ready) */
THFloatTensor *thhip_forward_windows(struct network *net, THFloatTensor *in, int nwin, const int *b0, const int *bn,
	void (*before)(void *ctx, int w), void *ctx);
void thhip_free_loaded_network(THNETWORK *n);

#endif
