/*
 * onenew_hip.h -- C ABI of the MI355X (gfx950) Conv / MatMul / Gemm backend.
 *
 * Two levels:
 *
 *  1. Plugin level (what the oneNew host binds).  Three shared objects, libConv_hip.so,
 *     libMatMul_hip.so and libGemm_hip.so, each export `eval` with the signature of
 *     onenew_abi.h; they forward to onhip_conv_eval / onhip_matmul_eval / onhip_gemm_eval below.
 *     These replace device/x86/Conv/conv.c:13 `eval`, device/x86/MatMul/mat_mul.c:10 `eval`
 *     and device/x86/Gemm/gemm.c:9 `eval` of the reference.
 *
 *  2. Kernel level: explicit shapes, device pointers and a HIP stream, no host<->device copies
 *     and no synchronisation.  This is what benchmarks and parity tests time and check.
 *
 * Every function returns 0 on success and a negative code on failure; the text of the last
 * failure on the calling thread is returned by onhip_last_error().  Nothing throws.
 *
 * Like the reference's kernels, which share one scratch buffer (host/net.h:419-429), the convolution and matrix
 * entry points share per-process device workspaces (split-K partial sums, arrival counters, the plugin level's staging
 * buffers): launches that may overlap on the device, i.e. on different streams without an ordering between them,
 * race.  One stream at a time, as the single-threaded reference host calls its operators, is the contract.
 */
#ifndef ONENEW_HIP_H
#define ONENEW_HIP_H

#include <stddef.h>
#include <stdint.h>
#include "onenew_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

#define ONHIP_OK 0
#define ONHIP_ERR_ARG (-1)        /* shape / argument the path does not support */
#define ONHIP_ERR_RUNTIME (-2)    /* a HIP call failed */
#define ONHIP_ERR_WORKSPACE (-3)  /* caller workspace missing or too small */

/* arithmetic of the multiply-accumulate; accumulation is always fp32 (int32 for W8A32) */
enum {
    ONHIP_COMPUTE_F32 = 0,   /* fp32 operands, fp32 MFMA */
    ONHIP_COMPUTE_BF16 = 1,  /* operands rounded to bf16 (RNE) on the way into LDS */
    ONHIP_COMPUTE_F16 = 2    /* operands rounded to fp16 (RNE) on the way into LDS */
};

/*
 * Geometry and epilogue of one convolution.  Field meaning follows CONV_CONFIG_S and the
 * OPERAND_S shapes the reference kernel reads (device/x86/Conv/conv.c:77-104,328-350):
 * activations NCHW, weights [cout, cin/group, kh, kw], pads = top/left/bottom/right,
 * dilation 1.  group == 1 is a dense convolution, any other value a depthwise convolution with
 * cin == cout (conv.c:29,597-612).  n is the batch: the result equals n independent batch-1
 * evaluations of the reference.
 */
typedef struct {
    int32_t n, cin, h, w;
    int32_t cout, kh, kw;
    int32_t stride_h, stride_w;
    int32_t pad_t, pad_l, pad_b, pad_r;
    int32_t group;
    int32_t has_bias;       /* 0: no bias and -- as in conv.c:18-27 -- no activation either */
    int32_t act_type;       /* ACT_TYPE_E */
    float clip_min, clip_max;
    float leaky_relu_alpha;
    float hard_sigmoid_alpha, hard_sigmoid_beta;
    float input_scale;      /* W8A32 only: activation quantisation step */
    int32_t compute;        /* ONHIP_COMPUTE_*; dense fp32-storage convolutions only */
    int32_t out_s8;         /* W8A32 only: 1 = write int8 NCHW, re-quantised with output_scale */
    float output_scale;
} onhip_conv_desc_t;

/*
 * out[b] = A[b] (M x K, row-major) * B (K x N, row-major, shared when b_shared else per batch),
 * optionally + bias[n] and then the table GELU of device/x86/Gelu/gelu.c:22-38.
 * Plain MatMul (mat_mul.c:10-102) is bias == NULL, gelu_lut == NULL.
 */
typedef struct {
    int32_t batch, m, k, n;
    int32_t b_shared;
    int32_t compute;        /* ONHIP_COMPUTE_* */
} onhip_matmul_desc_t;

/* ---- library -------------------------------------------------------------------------- */

/* Selects the device, checks it is gfx950 and loads the kernels.  Idempotent. */
int onhip_init(int device);
/* Text of the last error on this thread ("" if none). */
const char *onhip_last_error(void);
/* Tile / split-K selection.  mode 0: cost model only.  mode 1: the first call for each problem
 * signature times the candidate launches on the caller's stream (it synchronises that stream once)
 * and the winner is cached for the life of the process -- the counterpart of the reference's GEMM tile
 * search (tools/optimize/auto_tuning.hpp:9-75).  Default: the ONHIP_TUNE environment variable, else 0.
 * Returns the previous mode. */
int onhip_set_tuning(int mode);
/* Diagnostic, no counterpart in the reference: how many launches so far cut their leftover tiles (those beyond a
 * whole number of rounds of 256 tiles) into K slices next to the whole tiles of the same launch. */
long long onhip_split_tail_launches(void);
/* Diagnostic, no counterpart in the reference: how many int8 launches so far ran the kernel that loads its operand tiles
 * from global memory straight into LDS (NHWC int8 activations with a multiple of 64 padded channels). */
long long onhip_direct_lds_launches(void);
/* Diagnostic, no counterpart in the reference: how the calling thread's last dense convolution / MatMul launch ran:
 * out = {tile rows, tile columns, K slices of every tile (1 = none), K slices of the leftover tiles only (0 = none),
 * 1 if the fp32 kernel that reads B straight from memory ran, 1 if the slices were added up inside the launch,
 * 1 / 2 if the kernel that loads operand tiles straight into LDS ran (short / long ring)}; zeros before the first such
 * launch; launches of the other kernel families (depthwise, first-layer, few-channel int8) leave it as it is. */
void onhip_last_launch_choice(int32_t out[7]);
/* Diagnostic, no counterpart in the reference: how many launches of onhip_conv2d_f32_noalloc so far cut K into slices and
 * therefore put their partial sums into the library's built-in scratch array (a call the cost model gives a single
 * slice never touches the array). */
long long onhip_noalloc_scratch_launches(void);
/* The model-wide GEMM tile of a .one file: BLOCK_INFO_S.cuda_gemm_tile_{m,n} (common/nn_common.h:28-39), which the
 * reference's tuner fills for its x86 kernels (tools/optimize/auto_tuning.hpp:9-75) and its converter defaults to
 * 16 x 16 (tools/onnx2one/onnx2one.cpp:1346-1349).  onhip_set_tile_hint(bm, bn) makes the cost model of the calling
 * thread choose among the K splits of that workgroup tile only, when bm x bn is a tile this library has kernels for
 * (returns 1); any other pair, 16 x 16 included, clears the hint (returns 0).  Measured choices (onhip_set_tuning(1))
 * and ONHIP_TILE take precedence.  The Conv plugin sets it around each call from params[11] (USEFUL_INFO_S).
 * onhip_tile_candidate(idx, ...) lists the tiles (ONHIP_ERR_ARG past the last one). */
int onhip_set_tile_hint(int32_t bm, int32_t bn);
int onhip_tile_candidate(int32_t idx, int32_t *bm, int32_t *bn);
/* Diagnostic, no counterpart in the reference: size in bytes of the library's split-K scratch block (0 before the first
 * split launch).  The block grows by allocating a larger one; an outgrown block is kept until the process ends, because
 * a HIP graph recorded by the caller may hold its address. */
long long onhip_scratch_bytes(void);
/* Output height / width of a convolution (host/ops/conv.h:43-50). Returns 0 or ONHIP_ERR_ARG. */
int onhip_conv_out_shape(const onhip_conv_desc_t *d, int32_t *oh, int32_t *ow);

/* ---- kernel level: device pointers, asynchronous on `stream` (a hipStream_t, NULL = default) - */

/* fp32 convolution + bias + activation.  Replaces conv.c eval_1x1j1 (:68), eval_mxn_img2col
 * (:300), eval_mxn_img2col_no_bias (:417), eval_depthwise_conv_mxn_img2col (:527),
 * eval_depthwise_conv_3x3_pad1 (:757) and do_act (:1216).  silu_lut (8192 floats) is required
 * for act_type SILU only. */
int onhip_conv2d_f32(const onhip_conv_desc_t *d, const float *x, const float *w, const float *bias,
                     const float *silu_lut, float *y, void *stream);

/* Weights packed once at load time.  For dense convolutions other than unpadded 1x1 the kernel
 * runs fastest on weights re-laid out tap-major, [cout][kh*kw][cin padded to the MFMA unit]: every
 * group of input channels then shares one filter tap and the im2col arithmetic shrinks to one
 * scalar description per group.  onhip_conv2d_packed_weight_bytes returns the size of that copy
 * (0 when the convolution takes its weights as they are: 1x1 without padding, depthwise, and, first
 * layers with three input channels apart, fewer than four input channels or more than 64 filter taps);
 * onhip_conv2d_pack_weights writes it (device kernel on `stream`); onhip_conv2d_f32_packed is
 * onhip_conv2d_f32 on such a copy.  Results of the two entry points agree to fp32 rounding (the
 * summation order over K differs).  No counterpart in the reference, whose only weight
 * re-layout is the offline int8 packing of tools/optimize/model_quant.hpp:14-25. */
size_t onhip_conv2d_packed_weight_bytes(const onhip_conv_desc_t *d);
int onhip_conv2d_pack_weights(const onhip_conv_desc_t *d, const float *w, float *packed, void *stream);
int onhip_conv2d_f32_packed(const onhip_conv_desc_t *d, const float *x, const float *w_packed, const float *bias,
                            const float *silu_lut, float *y, void *stream);

/* onhip_conv2d_f32 (packed == 0) or onhip_conv2d_f32_packed (packed != 0) for callers that cannot allocate device
 * memory: code under HIP graph capture, serving loops, harnesses that forbid it.  No counterpart in the reference.
 * It calls no allocating routine: the partial sums of a split-K launch go to a 32 MiB array built into the library's
 * code object (one copy per GPU, held until the process ends), tile and split come from the cost model only, and the
 * slices are added up by a finishing launch.  A problem whose chosen split needs more than 32 MiB of partial sums
 * (split x output bytes) is refused with ONHIP_ERR_WORKSPACE.  The array keeps the last call's contents; every
 * element read is written first by the same call, so nothing needs clearing.  All calls on one GPU share the array:
 * calls that may overlap there (different streams without an ordering between them) race.  Same results as the entry
 * point it mirrors when that one runs the cost model's choice (tuning off). */
int onhip_conv2d_f32_noalloc(const onhip_conv_desc_t *d, const float *x, const float *w, int32_t packed, const float *bias,
                             const float *silu_lut, float *y, void *stream);

/* The convolution that ends a residual block with the operators after it folded into its store:
 * y = conv(x) as onhip_conv2d_f32 (packed != 0: as onhip_conv2d_f32_packed), then y += addend (a tensor of
 * y's shape, not y itself) as device/x86/Add/add.c:96, then, with relu_after != 0, relu as
 * device/x86/Relu/relu.c:27-52 (both of its rules, by element index).  Bit-identical to the three operators
 * run one after the other when the convolution runs the same tile and split in both (always so with the cost model's
 * choice; with measured choices, onhip_set_tuning(1), the two may be measured differently and then differ in the
 * rounding of the sums, within the fp32 tolerance).  The reference fuses activations into Conv (tools/optimize/op_fusion.hpp:47-222)
 * but not the Add; this is the same idea one operator further. */
int onhip_conv2d_f32_add(const onhip_conv_desc_t *d, const float *x, const float *w, int32_t packed, const float *bias,
                         const float *silu_lut, const float *addend, int32_t relu_after, float *y, void *stream);

/* Bytes of device scratch onhip_conv2d_w8a32 (and onhip_conv2d_w8_link on fp32 activations) needs for `d`: the int8
 * copy of the activations.  A depthwise convolution uses it only in onhip_conv2d_w8_link with fp32 in and int8 out. */
size_t onhip_conv2d_w8a32_workspace(const onhip_conv_desc_t *d);

/* W8A32 convolution: fp32 activations quantised with d->input_scale, int8 weights
 * [cout, cin/group, kh, kw], int32 bias, int32 accumulation, fp32 de-quantisation with
 * weight_aux[oc] / 127, activation.  Replaces conv.c eval_mxn_img2col_W8A32_with_input_scale
 * (:901), ..._no_bias (:1061), eval_depthwise_conv_mxn_img2col_W8A32 (:617) and do_act.
 * y is float* (d->out_s8 == 0) or int8_t* (d->out_s8 == 1).  acc32, when not NULL, receives
 * the raw int32 accumulators (NCHW) for bit-exactness checks. */
int onhip_conv2d_w8a32(const onhip_conv_desc_t *d, const float *x, const int8_t *w8,
                       const int32_t *bias32, const float *weight_aux, const float *silu_lut,
                       void *y, int32_t *acc32, void *workspace, size_t workspace_bytes,
                       void *stream);

/* The int8 weights re-laid out once per layer for the kernel (rows of kh*kw taps x 16-byte channel
 * blocks, zero padded), so that a call does not repeat it: same role as the weight buffer the
 * reference keeps for the lifetime of the net (host/ops/conv.h:148-154).  Bytes needed (0 for
 * depthwise, which reads the reference layout), the packing, and the convolution on packed weights
 * (w8_packed 16-byte aligned; the workspace then only holds the int8 activations, the size
 * onhip_conv2d_w8a32_workspace reports is enough).  Results are identical to onhip_conv2d_w8a32. */
size_t onhip_conv2d_w8a32_packed_weight_bytes(const onhip_conv_desc_t *d);
int onhip_conv2d_w8a32_pack_weights(const onhip_conv_desc_t *d, const int8_t *w8, int8_t *packed,
                                    void *stream);
int onhip_conv2d_w8a32_packed(const onhip_conv_desc_t *d, const float *x, const int8_t *w8_packed,
                              const int32_t *bias32, const float *weight_aux,
                              const float *silu_lut, void *y, int32_t *acc32, void *workspace,
                              size_t workspace_bytes, void *stream);

/* The int8 chain form of the W8A32 convolution: activations stay int8 between layers.  Layout of
 * both xq and yq: NHWC, channels padded with anything to a multiple of 16 ([n][h][w][cp], 16-byte
 * aligned).  yq = quantise(y, d->output_scale) where y is exactly what onhip_conv2d_w8a32 computes
 * from the activations de-quantised with d->input_scale — the quantiser every reference Conv applies
 * to its input (conv.c:961-973), moved into the producer's epilogue, so a chain of these calls gives
 * the consumer the same int8 values as a chain of reference convolutions.  No counterpart as a
 * separate function in the reference.  Dense convolutions take their weights from
 * onhip_conv2d_w8a32_pack_weights; depthwise convolutions (d->group == d->cin, the arithmetic of
 * conv.c:617-755) take them as the reference holds them, [c][1][kh][kw] int8, and write padding
 * channels as zero.  onhip_quantize_nhwc_s8 makes the first xq of a chain from
 * NCHW fp32 (q 16-byte aligned, n*h*w*round_up(c,16) bytes). */
int onhip_quantize_nhwc_s8(const float *x, int32_t n, int32_t c, int32_t h, int32_t w, float scale,
                           int8_t *q, void *stream);
int onhip_conv2d_w8a8_nhwc(const onhip_conv_desc_t *d, const int8_t *xq, const int8_t *w8_packed,
                           const int32_t *bias32, const float *weight_aux, const float *silu_lut,
                           int8_t *yq, void *stream);

/* 1 when the depthwise convolution `d` is available with int8 NHWC activations (onhip_conv2d_w8a8_nhwc,
 * onhip_conv2d_w8_link): any stride, uniform padding, filters of up to 225 taps, tensors below 2 GiB; 0 otherwise and
 * for dense convolutions.  No counterpart in the reference. */
int onhip_conv2d_w8a8_depthwise_supported(const onhip_conv_desc_t *d);

/* One link of an int8 chain inside a model: the activations come as fp32 NCHW (x, quantised with d->input_scale into the
 * workspace as in onhip_conv2d_w8a32) or as int8 NHWC with channels padded to 16 (xq), exactly one of the two; the
 * result leaves as fp32 NCHW (d->out_s8 == 0) or as int8 NHWC quantised with d->output_scale (d->out_s8 == 1: what a
 * consumer whose input_scale is that value would make of the fp32 result, conv.c:961-973).  Weights packed by
 * onhip_conv2d_w8a32_pack_weights; for a depthwise convolution w8_packed is the weights as the reference holds them,
 * and no addend or twin.  addend, when not null (fp32 results only): a tensor of the
 * result's shape added to it in the store (device/x86/Add/add.c:96), followed, with relu_after != 0, by relu as
 * device/x86/Relu/relu.c:27-52 (both of its rules, by element index): the three operators' bytes in one pass.  y_twin,
 * when not null (with an addend, cout a multiple of 16, d->out_s8 == 0): the fp32 result is also stored there as int8
 * NHWC quantised with d->output_scale, for the int8 convolutions among the tensor's readers.  No
 * counterpart in the reference, whose W8A32 operators (device/x86/Conv/conv.c:939-1067) always take and return fp32; the
 * device-resident runtime calls it for edges between two int8 convolutions and for the one that closes a residual block. */
int onhip_conv2d_w8_link(const onhip_conv_desc_t *d, const float *x, const int8_t *xq, const int8_t *w8_packed,
                         const int32_t *bias32, const float *weight_aux, const float *silu_lut, const float *addend,
                         int32_t relu_after, void *y, int8_t *y_twin, void *workspace, size_t workspace_bytes, void *stream);

/* ---- bf16 / fp16 with 16-bit storage --------------------------------------------------------------------------
 * The reference has the two types as enumerators only (ELEM_TYPE_E TYPE_FP16 / the cuda tile fields,
 * common/nn_common.h:102,107) and no kernel that stores them, so the layouts are this library's: activations NHWC
 * with the channel count padded to onhip_h16_pitch(c) (a multiple of 32; padding channels hold zeros), 16-byte
 * aligned; weights [cout][kh*kw][pitch(cin)] from the pack functions; accumulation in fp32 on the matrix cores
 * (v_mfma_f32_32x32x16_bf16 / _f16); bias, activation (the fp32 convolution's, same tables) in fp32 on the sums,
 * then one rounding to nearest even into the output type.  d->compute (ONHIP_COMPUTE_BF16 or _F16) names the type
 * of x, the weights, the residual operand and the 16-bit output.  Arithmetic replaced: the multiply-accumulate of
 * device/x86/Conv/conv.c:1024-1056 (its fp32 form) and device/x86/MatMul/mat_mul.c:10-102 on rounded operands.
 *
 * y_kind: where the result goes.  _NHWC: 16-bit, pitch(cout) channels per pixel, the input of the next 16-bit
 * layer; `residual`, when not NULL, is a tensor of that type and layout that is added to the rounded result in
 * fp32 (followed by a ReLU when residual_relu != 0) and the sum rounded again: what separate Add and Relu operators
 * (device/x86/Add/add.c, Relu/relu.c) would store on 16-bit tensors.  _F32_NHWC: fp32, cout channels per pixel, no
 * padding (the rows of a MatMul result).  _F32_NCHW: fp32 in the reference's own layout, the way back out of a
 * 16-bit chain. */
enum { ONHIP_H16_OUT_NHWC = 0, ONHIP_H16_OUT_F32_NHWC = 1, ONHIP_H16_OUT_F32_NCHW = 2 };
int32_t onhip_h16_pitch(int32_t channels);
/* bytes of a packed weight tensor of `rows` filters (or MatMul columns) of cin channels and `taps` filter taps */
size_t onhip_h16_packed_weight_bytes(int32_t rows, int32_t cin, int32_t taps);
/* fp32 OIHW weights -> packed 16-bit (once per tensor) */
int onhip_h16_pack_conv_weights(const onhip_conv_desc_t *d, const float *w, void *packed, void *stream);
/* the right operand b [k][n] (row-major fp32) of a MatMul -> packed 16-bit [n][pitch(k)] */
int onhip_h16_pack_matmul_weights(const float *b, int32_t k, int32_t n, int32_t compute, void *packed, void *stream);
/* fp32 NCHW <-> 16-bit NHWC with padded channels; fp32 rows [rows][k] <-> 16-bit rows [rows][pitch(k)] */
int onhip_h16_from_nchw_f32(const float *x, int32_t n, int32_t c, int32_t h, int32_t w, int32_t compute, void *y, void *stream);
int onhip_h16_to_nchw_f32(const void *x, int32_t n, int32_t c, int32_t h, int32_t w, int32_t compute, float *y, void *stream);
int onhip_h16_from_rows_f32(const float *x, long long rows, int32_t k, int32_t compute, void *y, void *stream);
int onhip_h16_to_rows_f32(const void *x, long long rows, int32_t k, int32_t compute, float *y, void *stream);
/* dense convolution, at most 64 filter taps, tensors below 2 GiB */
int onhip_conv2d_h16(const onhip_conv_desc_t *d, const void *x, const void *w_packed, const float *bias, const float *lut,
                     const void *residual, int32_t residual_relu, void *y, int32_t y_kind, void *stream);
/* First layers (dense, at most 8 input channels, filter rows of at most 8 columns, any stride and padding) in a storage
 * form of their own: with the 32-channel pitch above a three-channel image is 29/32 zeros, in memory and in the
 * arithmetic.  Here the image is stored [n][h][wp][cpp] (wp = onhip_h16_first_width: the padded row, an even number of
 * columns; cpp = onhip_h16_first_channels: 4 channels per pixel for up to four input channels, else 8; stored column s =
 * image column s - pad_l, zeros outside) and the weights [cout][kh][8 columns][cpp], so that a filter row meets 16 cpp
 * contiguous bytes of the stored row and the reduction runs over kh x 8 cpp values.  The same
 * arithmetic as onhip_conv2d_h16 (device/x86/Conv/conv.c:300-415 on operands rounded to the 16-bit type, fp32 sums, bias
 * and activation in fp32); the result leaves in the layouts of y_kind, i.e. as the next layer's ordinary input. */
int32_t onhip_h16_first_width(const onhip_conv_desc_t *d);            /* 0: not a shape of this form */
int32_t onhip_h16_first_channels(const onhip_conv_desc_t *d);
size_t onhip_h16_first_input_bytes(const onhip_conv_desc_t *d);
size_t onhip_h16_first_weight_bytes(const onhip_conv_desc_t *d);
int onhip_h16_first_from_nchw_f32(const onhip_conv_desc_t *d, const float *x, void *x_first, void *stream);
int onhip_h16_first_pack_weights(const onhip_conv_desc_t *d, const float *w, void *packed, void *stream);
int onhip_conv2d_h16_first(const onhip_conv_desc_t *d, const void *x_first, const void *w_packed, const float *bias,
                           const float *lut, void *y, int32_t y_kind, void *stream);
/* y[rows][n] = x[rows][k] * b[k][n] (+ bias[n]) (then the table GELU of device/x86/Gelu/gelu.c when gelu_lut is given):
 * the MatMul -> Add -> Gelu chain of a transformer's linear layers with x, b and (for _NHWC) y in 16 bits */
int onhip_linear_h16(long long rows, int32_t k, int32_t n, int32_t compute, const void *x, const void *w_packed,
                     const float *bias, const float *gelu_lut, const void *residual, void *y, int32_t y_kind, void *stream);

/* Batched MatMul with optional fused bias and table GELU.  Replaces mat_mul.c eval (:10) and,
 * with bias/gelu_lut, the chain MatMul -> Add -> Gelu (device/x86/Gelu/gelu.c:9). */
int onhip_matmul(const onhip_matmul_desc_t *d, const float *a, const float *b, const float *bias,
                 const float *gelu_lut, float *out, void *stream);
/* MatMul -> Add of a bias over the last axis (bias may be NULL) -> Add of a tensor shaped like the result (the skip
 * connection of a transformer block), the sum formed in the product's store: mat_mul.c eval (:10) followed by two
 * device/x86/Add/add.c evals, bit-equal to them.  addend must not be the output buffer. */
int onhip_matmul_add(const onhip_matmul_desc_t *d, const float *a, const float *b, const float *bias,
                     const float *addend, float *out, void *stream);

/* A whole inverted-residual block in one launch: 1x1 convolution (bias, activation) -> depthwise 3x3 (pads 1, stride 1 or
 * 2, bias, activation) -> 1x1 convolution (bias, activation) [-> Add of a residual tensor shaped like the output].
 * Replaces three (four) operator evaluations, device/x86/Conv/conv.c 1x1 path :1024-1056 twice and depthwise path :757-899
 * (and device/x86/Add/add.c); neither wide tensor of the block is written to memory.  fp32; the depthwise stage performs
 * the separate operator's operations in its order, the two 1x1 stages sum in MFMA order, so the block equals the chain of
 * operators within fp32 summation error.  No counterpart as one function in the reference.
 * onhip_ir_block_supported: 0 = this triple is not taken (16, 24, 32 or 64 input channels, expanded channels a multiple
 * of 16, at most 64 output channels, rows of a multiple of 2 and at most 128 output pixels, biases on the first two
 * convolutions), 1 = taken, 2 = taken and expected to be faster than the three launches (at most 32 input channels and at
 * least 256 bands of output rows over the batch).  packed: both 1x1 weight tensors ([ce][cin] and [co][ce]) re-laid once by
 * onhip_ir_block_pack_weights (onhip_ir_block_packed_weight_bytes(cin, ce, co) bytes, 16-byte aligned). */
int onhip_ir_block_supported(const onhip_conv_desc_t *expand, const onhip_conv_desc_t *dw, const onhip_conv_desc_t *project);
size_t onhip_ir_block_packed_weight_bytes(int32_t cin, int32_t ce, int32_t co);
int onhip_ir_block_pack_weights(const float *expand_w, const float *project_w, int32_t cin, int32_t ce, int32_t co, float *packed,
                                void *stream);
int onhip_ir_block_f32(const onhip_conv_desc_t *expand, const onhip_conv_desc_t *dw, const onhip_conv_desc_t *project, const float *x,
                       const float *packed, const float *expand_b, const float *dw_w, const float *dw_b, const float *project_b,
                       const float *residual, float *y, void *stream);

/* A dense convolution and the 1x1 convolution that reads its result, in one launch:  y = b(a(x)) [+ addend, then Relu].
 * Replaces two operator evaluations (device/x86/Conv/conv.c:300-415 twice: im2col + SGEMM + bias + activation, the second
 * with a 1x1 filter) and, with `addend`, the Add and Relu after them (device/x86/Add/add.c, device/x86/Relu/relu.c:27-52);
 * the tensor between the two convolutions is never written to memory: a workgroup holds all of a's output channels for its
 * 64 pixels and multiplies them by b's weights before it stores.  fp32; both products sum in MFMA order, so the pair equals
 * the two operators within fp32 summation error.  No counterpart as one function in the reference.
 * a: dense, at most 64 output channels, not a plain 1x1 and not a first layer (three input channels),
 * weights in the tap-major packed form of onhip_conv2d_pack_weights; b: 1x1, stride 1, no padding, over a's result, weights
 * ([cout][cin]) re-laid once by onhip_conv2d_pw_pack_weights into the order the kernel's matrix instructions read them
 * (onhip_conv2d_pw_packed_weight_bytes(b) bytes, 16-byte aligned); activations none, Relu or Clip.
 * onhip_conv2d_pw_supported: 0 = not taken, 1 = taken, 2 = taken and expected to be faster than the two launches (at least
 * 16384 output pixels over the batch).  addend (may be NULL): a tensor shaped like y, added after b's activation;
 * relu_after != 0: relu.c's rule on the sum.  addend must not be y. */
int onhip_conv2d_pw_supported(const onhip_conv_desc_t *a, const onhip_conv_desc_t *b);
size_t onhip_conv2d_pw_packed_weight_bytes(const onhip_conv_desc_t *b);
int onhip_conv2d_pw_pack_weights(const onhip_conv_desc_t *b, const float *wb, float *packed, void *stream);
int onhip_conv2d_pw_f32(const onhip_conv_desc_t *a, const onhip_conv_desc_t *b, const float *x, const float *wa_packed,
                        const float *bias_a, const float *wb_packed, const float *bias_b, const float *addend,
                        int32_t relu_after, float *y, void *stream);

/* Attention of every (batch, head) in one launch:  out = Softmax(q k^T * scale) v, Softmax over the keys.  Replaces the
 * operator chain MatMul (device/x86/MatMul/mat_mul.c:10-102) -> [Mul by a constant] -> Softmax (device/x86/Softmax/
 * softmax.c:26-59) -> MatMul of a transformer block, together with the Transposes (device/x86/Transpose/transpose.c)
 * that split q, k, v into heads, transpose k and merge the heads again: every operand is addressed through the element
 * strides of (batch, head, token), the head dimension being contiguous, so q, k and v may be slices of one projection
 * output [batch][tokens][3 * heads * head_dim] and out the merged [batch][tokens][heads * head_dim].  The scores stay in
 * registers.  compute ONHIP_COMPUTE_F32: fp32 tensors, head_dim 32 or 64.  ONHIP_COMPUTE_BF16 / _F16: q, k, v and out
 * are tensors of that 16-bit type (e.g. slices of a 16-bit projection output), head_dim 64; products on the 16-bit
 * matrix-core instructions with fp32 accumulation, scores and Softmax in fp32, the probabilities rounded to the operand
 * type for the second product.  At most 256 tokens, rows 16-byte aligned (strides multiples of a 16-byte vector); other
 * shapes are refused and stay with the separate operators. */
typedef struct onhip_attention_desc {
    int32_t batch, heads, tokens, head_dim;
    long long q_strides[3], k_strides[3], v_strides[3], out_strides[3];
    float scale;      /* 1.0f when the graph has no Mul between the first MatMul and the Softmax */
    int32_t compute;
} onhip_attention_desc_t;
int onhip_attention(const onhip_attention_desc_t *d, const void *q, const void *k, const void *v, void *out,
                    void *stream);

/* out[m][n] = sum_k a[m][k] * w[n][k] + bias[n].  Replaces gemm.c eval (:9). */
int onhip_gemm_f32(int32_t m, int32_t k, int32_t n, const float *a, const float *w,
                   const float *bias, float *out, void *stream);

/* ---- the operators around the convolutions of a residual network (device pointers) ------------ */

/* Broadcasting add: out = large + small, out has the shape of `large`; `small` is aligned to the
 * same rank (host pads its shape with leading 1s) and each of its extents is 1 or equal.  relu == 1
 * applies "x > 0 ? x : 0" to the sum: the Add -> Relu pair that closes a residual block, in one pass; relu == 2 applies
 * the Relu operator's own two rules by element index (device/x86/Relu/relu.c:27-52: "0 > x ? 0 : x" below n - n % 32,
 * "x > 0 ? x : 0" from there on; they differ on NaN and negative zero), what a separate Relu would store.
 * Replaces device/x86/Add/add.c eval (:18-80) and fun_0 / fun_1 / fun_2_dim3..6 (:87-365). */
typedef struct {
    int32_t ndim;            /* 1..6 */
    int32_t large_shape[6];
    int32_t small_shape[6];
    int32_t relu;
} onhip_add_desc_t;
int onhip_add_f32(const onhip_add_desc_t *d, const float *large, const float *small, float *out,
                  void *stream);

/* y = relu(x) over n floats (16-byte aligned).  Replaces device/x86/Relu/relu.c eval (:8-55),
 * including its two rules: the first n - n % 32 elements keep a NaN or a negative zero. */
int onhip_relu_f32(const float *x, float *y, long long n, void *stream);

/* Max pooling over NCHW planes, every side padded by `pad`; oh x ow is the extent of the output
 * operand (at most the floor-mode shape onhip_maxpool_out_shape reports).  Replaces
 * device/x86/MaxPool/maxpool.c eval (:7-92) with pad_maxpool.h; the running maximum starts at
 * -3276800 as there. */
typedef struct {
    int32_t n, c, h, w;
    int32_t kh, kw;
    int32_t stride_w, stride_h;   /* strides[0] moves along w, strides[1] along h (maxpool.c:20-21,72) */
    int32_t pad;
} onhip_pool_desc_t;
int onhip_maxpool_out_shape(const onhip_pool_desc_t *d, int32_t *oh, int32_t *ow);
int onhip_maxpool_f32(const onhip_pool_desc_t *d, int32_t oh, int32_t ow, const float *x, float *y,
                      void *stream);
/* The same on int8 NHWC activations (element (image, row, column, channel) at ((image * h + row) * w + column) * cp +
 * channel, cp = c rounded up to 16; 16-byte aligned): y = the byte-wise maximum over the window.  Because the activation
 * quantiser (device/x86/Conv/conv.c:961-973) is monotonic, this is what that quantiser makes of maxpool.c's fp32 result
 * on the de-quantised input: a MaxPool between int8 convolutions needs no fp32 tensor.  No counterpart in the reference. */
int onhip_maxpool_s8_nhwc(const onhip_pool_desc_t *d, int32_t oh, int32_t ow, const int8_t *x, int8_t *y, void *stream);

/* y[n][c] = (sum of the plane in memory order) * (1.0f / (h*w)).  Replaces
 * device/x86/GlobalAveragePool/global_avgpool.c eval (:7-45). */
int onhip_global_avgpool_f32(int32_t n, int32_t c, int32_t h, int32_t w, const float *x, float *y,
                             void *stream);

/* ---- the operators around the MatMuls of a transformer block (device pointers) ----------------- */

/* y = table GELU of x: 0 below -8, x from 8 up, else gelu_lut[(int)((x + 8) * 512)] (8192 floats,
 * host/ops/gelu.h:80-96).  Replaces device/x86/Gelu/gelu.c eval (:9-42). */
int onhip_gelu_lut_f32(const float *x, const float *gelu_lut, float *y, long long n, void *stream);

/* Layer normalisation of `rows` rows of `reduce` elements with per-element weight and bias, eps 1e-20.
 * strided == 0: rows are contiguous (the last non-1 dimension is normalised,
 * layer_normalization.c:62-97); strided != 0: element i of row r lies at i * rows + r (the "axes[0]
 * == 1" form, :28-60).  Replaces device/x86/LayerNormalization/layer_normalization.c eval (:10-101). */
int onhip_layernorm_f32(int32_t rows, int32_t reduce, int32_t strided, const float *x,
                        const float *weight, const float *bias, float *y, void *stream);

/* Softmax over `reduce` elements, `rows` times; strided as above (axis 1 of a batch-1 tensor).
 * Replaces device/x86/Softmax/softmax.c eval_dim_last (:26-59) and eval_dim_1 (:62-118). */
int onhip_softmax_f32(int32_t rows, int32_t reduce, int32_t strided, const float *x, float *y,
                      void *stream);

/* y = x with output dimension k taken from input dimension perm[k].  Replaces
 * device/x86/Transpose/transpose.c eval_perm_num4 (:24-79) and eval_perm_num6 (:81-140). */
typedef struct {
    int32_t ndim;            /* 1..6 */
    int32_t in_shape[6];
    int32_t perm[6];
} onhip_transpose_desc_t;
int onhip_transpose_f32(const onhip_transpose_desc_t *d, const float *x, float *y, void *stream);

/* ---- offline quantisation: what produces the operands of onhip_conv2d_w8a32 ------------------ */

/* Per output channel: weight_aux = max|w|, w8 = (int8)(w * 127 / aux) (truncating),
 * bias32 = (int32)(b * 127 / aux).  Replaces quant_weight_bias,
 * tools/optimize/model_quant.hpp:6-29.  Host arrays (runs once per model); bias may be NULL. */
int onhip_quant_weight_bias(const float *w, const float *bias, int32_t cout, int32_t per_channel,
                            int8_t *w8, int32_t *bias32, float *weight_aux);

/* Activation-scale calibration, the data passes of quant_kl / quant_mse / quant_percent
 * (model_quant.hpp:197-435, :437-623, :83-185) over device-resident activations x:
 *  - onhip_calib_abs_max: *max_abs (host, in/out) = max(*max_abs, max|x|)          (:287-296)
 *  - onhip_calib_histogram: adds the 2048-bin histogram of |x| over [0, max_abs] (zeros skipped) to
 *    hist (host, ONHIP_CALIB_BINS floats, counted like the reference's float counters) (:325-332)
 *  - onhip_calib_threshold: the clipping threshold from such a histogram; elem_count is the
 *    reference's "elements per image x images"                                   (:345-431, :585-618)
 *  - onhip_calib_percentile: x holds `images` tensors of `elems` values; the 99.998 % magnitude (:99-183)
 * The layer's input_scale is threshold / 127 (model_quant.hpp:668).  All four synchronise.  The three passes over
 * device data allocate nothing: they work in `workspace`, device memory of at least onhip_calib_workspace_bytes(images)
 * bytes (images = 1 for abs_max and histogram), 8-byte aligned, which the caller may reuse from call to call. */
#define ONHIP_CALIB_BINS 2048
#define ONHIP_CALIB_KL 0
#define ONHIP_CALIB_MSE 1
size_t onhip_calib_workspace_bytes(int images);
int onhip_calib_abs_max(const float *x, long long n, float *max_abs, void *workspace, size_t workspace_bytes, void *stream);
int onhip_calib_histogram(const float *x, long long n, float max_abs, float *hist, void *workspace, size_t workspace_bytes,
                          void *stream);
int onhip_calib_threshold(int method, const float *hist, long long elem_count, float max_abs,
                          float *threshold);
int onhip_calib_percentile(const float *x, int images, int elems, float *threshold, void *workspace, size_t workspace_bytes,
                           void *stream);

/* Plain device-to-device copy of n floats (n % 4 == 0, 16-byte aligned).  A measuring aid with no
 * counterpart in the reference: HBM traffic counters of the other kernels are scaled by what the
 * same counters read for this copy of known size. */
int onhip_copy_f32(const float *src, float *dst, long long n, void *stream);

/* ---- plugin level: the reference slot arrays; host or device pointers; synchronous --------- */

int onhip_conv_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* Conv with the Add (and Relu) that follow it in a residual block: slots as for Conv, inputs[3] = the other operand
 * of the Add, outputs[0] = the block's result.  No counterpart in the reference; exported by libConv_hip.so as
 * `eval_add` and `eval_add_relu` beside `eval`, for the device-resident runtime. */
int onhip_conv_add_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_conv_add_relu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_block` / `eval_block_takes` of libConv_hip.so: Conv (1x1) -> Conv (depthwise 3x3) -> Conv (1x1) [-> Add] in one
 * call (onhip_ir_block_f32).  Slots as for the first convolution's `eval` (host/op.h:109-168), the block's result operand
 * in params[4] and outputs[0]; inputs[3] = the addend or null; params[5], params[6], inputs[5], inputs[6] = the depthwise
 * convolution's CONV_CONFIG_S, weight operand, weights and bias; params[7], params[8], inputs[7], inputs[8] = the same of
 * the last convolution.  onhip_conv_block_takes reads the params only and returns 1 when onhip_ir_block_supported says 2
 * for these shapes, else 0.  No counterpart in the reference, whose host runs the operators one by one. */
int onhip_conv_block_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_pair` / `eval_pair_relu` / `eval_pair_takes` of libConv_hip.so: Conv (dense, at most 64 output channels, not a plain
 * 1x1) -> Conv (1x1) [-> Add [-> Relu]] in one call (onhip_conv2d_pw_f32).  Slots as for the first convolution's `eval`, the
 * pair's result operand in params[4] and outputs[0]; inputs[3] = the addend or null; params[5], params[6], inputs[5],
 * inputs[6] = the second convolution's CONV_CONFIG_S, weight operand, weights and bias.  onhip_conv_pair_relu_eval applies
 * relu.c's rule to the sum (an addend is required); onhip_conv_pair_takes reads the params only and returns 1 when
 * onhip_conv2d_pw_supported says 2 for these shapes, else 0.  No counterpart in the reference. */
int onhip_conv_pair_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_conv_pair_relu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_conv_pair_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_link` of libConv_hip.so: an int8 (W8A32) Conv, dense or depthwise, whose input and/or result travel as int8 NHWC (channels padded
 * to 16) instead of fp32 NCHW, see onhip_conv2d_w8_link.  Slots as for `eval`; inputs[4] = host pointer to
 * {int32 in_s8, int32 out_s8, float out_scale, int32 twin} (twin != 0: outputs[1] = device buffer for the int8 copy of an
 * fp32 result with a folded Add); inputs[5] = null, or host pointer to an int32 1 / 2 for the Add (and
 * Relu) of a residual block with its other operand in inputs[3] (fp32 results only).  No counterpart in the reference. */
int onhip_conv_link_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_link_takes` of libConv_hip.so: reads params[0..2] only (CONV_CONFIG_S, input operand, weight operand) and returns
 * 1 when `eval_link` can run this convolution with int8 NHWC activations on either side (every dense int8 convolution;
 * depthwise ones where onhip_conv2d_w8a8_depthwise_supported says so), else 0.  No counterpart in the reference. */
int onhip_conv_link_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_conv_block_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_matmul_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* Add (add.c:18), Relu (relu.c:8), MaxPool (maxpool.c:7), GlobalAveragePool (global_avgpool.c:7) */
int onhip_add_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_relu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_maxpool_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_s8` of libMaxPool_hip.so: slots and operand descriptors as for `eval` (NCHW shapes), the tensors int8 NHWC with
 * channels padded to 16 (onhip_maxpool_s8_nhwc).  For the device-resident runtime, between int8 convolutions. */
int onhip_maxpool_s8_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_global_avgpool_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* Gelu (gelu.c:9), LayerNormalization (layer_normalization.c:10), Softmax (softmax.c:12), Transpose (transpose.c:13) */
int onhip_gelu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_layernorm_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_softmax_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_transpose_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_gemm_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_attention` of libMatMul_hip.so: MatMul(q, Transpose(k)) -> Softmax (last axis) -> MatMul(., v) in one call
 * (onhip_attention with scale 1).  params[1..3] / inputs[0..2]: q, k (before its Transpose), v, all
 * [..., tokens, head_dim]; params[4] / outputs[0]: the result.  inputs[4]: null, or the address of four int32 flags (q, k,
 * v, result); non-zero = that rank-4 tensor is stored [batch, tokens, heads, head_dim], as on the other side of a
 * head-split / head-merge Transpose (0, 2, 1, 3), and its operand carries that shape.  No counterpart in the reference, whose host runs the four
 * operators one after the other (mat_mul.c, transpose.c, softmax.c). */
int onhip_matmul_attention_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_bias` / `eval_bias_gelu` of libMatMul_hip.so: MatMul -> Add of a bias over the last axis (-> Gelu) in one call
 * (onhip_matmul with bias and table).  Slots as for the MatMul `eval` plus params[3] / inputs[2] = the bias, the
 * result's operand in params[4], the Gelu table in inputs[11].  Bit-equal to the three reference operators in sequence
 * (mat_mul.c, add.c, gelu.c) as this library computes them. */
int onhip_matmul_bias_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
int onhip_matmul_bias_gelu_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/* `eval_bias_add` of libMatMul_hip.so: MatMul -> Add of a bias over the last axis -> Add of a tensor shaped like the
 * result, in one call (onhip_matmul_add).  Slots as for `eval_bias`; the second addend travels in inputs[3] (it has the
 * result's operand, so no params slot of its own), as the addend of the Conv plugin's `eval_add` does. */
int onhip_matmul_bias_add_eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
/*
 * No counterpart in the reference, whose operators always finish before eval returns (device/cuda/MaxPool/
 * maxpool.cu:76).  on != 0: an eval whose output is device memory returns as soon as its kernels are queued on
 * the default stream; the caller orders its own reads after them (a blocking hipMemcpy, hipStreamSynchronize).
 * Used by the device-resident runtime (onenew_rt.h) between the operators of one inference.  Outputs in host
 * memory are still complete on return.
 */
int onhip_plugin_set_async(int on);
/* The stream the evals queue their kernels on; NULL (the initial state) is the default stream.  No counterpart in the
 * reference.  The device-resident runtime names its own stream for the length of a run so that the run can be
 * recorded into a HIP graph.  Results into host buffers are still complete on return. */
int onhip_plugin_set_stream(void *stream);
/* For a caller that hands `eval` weights or activation tables in device memory and is about to free or overwrite them:
 * drops the re-laid-out copies the library made of weights (and the quantised copies of tables) whose address lies in
 * [base, base + bytes), so that other data at the same address later is packed afresh.  The device-resident runtime calls it when a net is freed.  No counterpart in the
 * reference (its weights live in host vectors for the life of the process). */
int onhip_plugin_forget(const void *base, size_t bytes);
/* `eval` keeps a device copy of every weight and table it was handed in host memory and, on each call, hashes the host
 * buffer to see whether the copy is still current: all of it by default (about 0.05 ms per MiB), so weights updated in
 * place are picked up.  on != 0: only 4096 sampled words are hashed, for a caller whose weights never change while the
 * library is loaded (the reference keeps them in vectors filled once at load, host/op.h).  No counterpart in the
 * reference. */
int onhip_plugin_trust_weights(int on);
/* Drops the device copies of weights the plugin level keeps between calls. */
int onhip_plugin_release(void);

#ifdef __cplusplus
}
#endif
#endif /* ONENEW_HIP_H */
