/*
 * onenew_rt.h -- device-resident execution of a .one model: the part of the oneNew host runtime that sits
 * either side of the operator plugins, with every operand buffer and every initialiser in HBM.
 *
 * It restates the calling sequence of the reference host (host/net.h): load the file, build one operator
 * object per node, order them, infer shapes, allocate one buffer per operand, fill the plugin slot arrays and
 * call each plugin's `eval` in order.  What differs is where the bytes live: initialisers are uploaded once
 * at load time, operand buffers are device memory, and between two operators nothing crosses PCIe.  Only the
 * net's inputs are copied in and its outputs copied out.
 *
 * Operators: Conv, MatMul, Gemm, Add, Relu, MaxPool, GlobalAveragePool, Gelu, LayerNormalization, Softmax,
 * Transpose through `lib<Op>_hip.so`; Flatten and Reshape as views (no buffer, no call: host/op.h:149-154); Clip,
 * LeakyRelu, Sigmoid x Mul and HardSigmoid x Mul only as the activation of the Conv in front of them.
 * A model with any other node type is refused at load time.
 *
 * All functions return 0 on success or a negative ONRT_ERR_* code; onrt_last_error() describes the failure.
 */
#ifndef ONENEW_RT_H
#define ONENEW_RT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ONRT_OK 0
#define ONRT_ERR_ARG (-1)       /* null pointer, bad index, unknown operand name */
#define ONRT_ERR_FORMAT (-2)    /* not a .one file, truncated file, node of an unsupported type */
#define ONRT_ERR_PLUGIN (-3)    /* lib<Op>_hip.so not found, no `eval` in it, or eval returned non-zero */
#define ONRT_ERR_RUNTIME (-4)   /* HIP call failed, out of memory */

typedef struct onrt_net onrt_net_t;

/* Message of the last failure on the calling thread. */
const char *onrt_last_error(void);

/*
 * Loads a model and makes it ready to run: host/net.h:101-131 (load_one_model) or :133-136 (load_one_buf),
 * :138-189 (instantiate_op), :191-221 (initialiser list), :378-389 (build_graph: order, operand list, shapes),
 * :419-452 (new_output_buf) and :629-640 (prepare_for_op).  The buffer is copied; the caller may free it.
 *
 * op_lib_dir: where the operator plugins are looked up, in the order of host/op.h:41-80 with the HIP
 * library in the place of the x86 one: <dir>/<Op>/lib<Op>_hip.so, then <dir>/lib<Op>_hip.so.  NULL means
 * the environment variable ONENEW_OP_LIB_DIR, and without it the directory this library was loaded from.
 */
int onrt_net_load_file(const char *one_path, const char *op_lib_dir, onrt_net_t **net);
int onrt_net_load_buf(const void *one_buf, size_t bytes, const char *op_lib_dir, onrt_net_t **net);

/*
 * The host-side half of loading, without plugins, device or memory: reads the file, orders the nodes, infers the
 * shapes and folds what the loader folds when the Conv plugin of this package is bound.  The result answers
 * onrt_net_io_count / _io_info / _op_count / _op_info / _operand (addresses NULL) / _fused_count and is released
 * with onrt_net_free; onrt_net_run refuses it.  For tools that want to know what a model will run as, and for
 * checking a file on a machine without a GPU.
 */
int onrt_net_plan_buf(const void *one_buf, size_t bytes, onrt_net_t **net);

/* Releases the device memory of the net and its operator objects (host/net.h:401-416). */
void onrt_net_free(onrt_net_t *net);

/* Counts of the io nodes named "input" / "output" (host/ops/io.h:56-70), in file order. */
int onrt_net_io_count(const onrt_net_t *net, int32_t *n_inputs, int32_t *n_outputs);

/* Name, rank and shape (SHAPE_LEN entries, unused ones 1) of input or output number idx. */
int onrt_net_io_info(const onrt_net_t *net, int32_t is_output, int32_t idx, const char **name, int32_t *ndim,
                     int32_t shape[8]);

/*
 * Residual blocks.  Where a Conv's result is read only by an Add whose other operand has the same shape (and
 * that sum perhaps only by a Relu), the loader folds the Add (and the Relu) into the convolution's store through
 * the Conv plugin's `eval_add` / `eval_add_relu` entry points, when the plugin has them: one launch instead of
 * three, and the tensors in between are never written.  The reference's offline optimiser folds the activation
 * after a Conv the same way (tools/optimize/op_fusion.hpp:47-222).  Results are bit-identical to the separate
 * operators as long as the convolution runs the same tile and split either way (the cost model's choice always does;
 * measured choices may differ between the two forms, and the sums then differ in their rounding).  The fused call runs at the Add's place in the order; the operands folded away stay in the operand
 * table and read as the block's result.  Setting the environment variable ONENEW_RT_FUSE=0 before loading keeps
 * every operator separate, for layer-by-layer comparison.
 *
 * A Relu that alone reads the result of a Conv with a bias and no activation is folded first, the way that
 * optimiser does it: the node goes and the Conv's act_type becomes RELU (a file that has been through the optimiser
 * has none left).  n_blocks / n_relus (either may be NULL): how many residual blocks / Relu nodes were folded.
 */
int onrt_net_fused_count(const onrt_net_t *net, int32_t *n_blocks, int32_t *n_relus);

/*
 * The other activations the offline optimiser folds into a Conv are folded the same way at load time: Conv -> Clip
 * (act_type CLIP with the node's min / max, tools/optimize/op_fusion.hpp:75-103), Conv -> LeakyRelu (:105-132), Conv ->
 * Sigmoid and Mul of the two (SILU, evaluated through the 8192-entry table like any fused SiLU, :134-160), Conv ->
 * HardSigmoid and Mul (HARDSILU with the node's alpha / beta, :162-192); patterns as in :485-539, for a Conv with a bias
 * and no activation yet.  This runtime has no operators of these five types: they are folded whatever ONENEW_RT_FUSE
 * says, and a model in which one of them does not follow such a Conv is refused at load time.  n: how many Conv nodes
 * took an activation this way.
 */
int onrt_net_folded_activations(const onrt_net_t *net, int32_t *n);

/*
 * Inverted-residual blocks: Conv (1x1) -> Conv (depthwise 3x3) -> Conv (1x1) [-> Add], each result read by the next
 * alone, run as one call of the Conv plugin's `eval_block` (libConv_hip.so; neither wide tensor in between is written)
 * where its `eval_block_takes` recommends that for the shapes: MobileNetV2's blocks on the 112, 56 and 28 pixel planes at
 * large batch.  The reference's host runs the operators one after the other (host/net.h:613-618).  The operands folded
 * away have no buffer.  ONENEW_RT_FUSE=0 keeps the operators separate.  n: how many blocks.
 */
int onrt_net_fused_ir_blocks(const onrt_net_t *net, int32_t *n);

/*
 * Convolution pairs: Conv (dense, at most 64 output channels, not a plain 1x1) -> Conv (1x1) [-> Add [-> Relu], folded into
 * the second convolution], the first result read by the second alone, run as one call of the Conv plugin's `eval_pair` /
 * `eval_pair_relu` (libConv_hip.so; the tensor in between is not written) where its `eval_pair_takes` recommends that for
 * the shapes: the 3x3 and the last convolution of ResNet-50's first-stage bottlenecks at large batch.  The reference's host
 * runs the operators one after the other (host/net.h:613-618).  The operand folded away has no buffer.  ONENEW_RT_FUSE=0
 * keeps the operators separate, ONENEW_RT_FUSE_PAIRS=0 these pairs alone.  n: how many pairs.
 */
int onrt_net_fused_pairs(const onrt_net_t *net, int32_t *n);

/*
 * int8 edges: the result of a dense int8 (W8A32) Conv that only dense int8 Convs with one and the same input_scale read
 * travels as int8 NHWC, quantised in the producer's store exactly as each consumer would have quantised the fp32 tensor
 * (device/x86/Conv/conv.c:961-973), through the Conv plugin's `eval_link`: a quarter of the bytes, no staging pass in the
 * consumers, the same results.  Likewise the int8 copy that the store of an int8 Conv with a folded Add leaves for the
 * int8 readers of its fp32 result, and both operands of a MaxPool between int8 convolutions (pooled as bytes: the
 * quantiser is monotonic).  The reference's operators always exchange fp32 (conv.c:939-1067).  ONENEW_RT_FUSE=0
 * keeps every operand fp32.  n: how many operands travel that way.
 */
int onrt_net_quantised_links(const onrt_net_t *net, int32_t *n);

/*
 * Attention blocks: MatMul(q, Transpose(k)) -> Softmax (last axis) -> MatMul(., v), where nothing else reads the operands
 * in between, run as one call of the MatMul plugin's `eval_attention` (libMatMul_hip.so; the scores stay on the chip, the
 * transposed k is never written) when q, k and v are [..., tokens, head_dim] with head_dim 32 or 64 and at most 256
 * tokens.  The reference's host runs the four operators one after the other (host/net.h:613-618); its optimiser has
 * no such pattern (tools/optimize/op_fusion.hpp:477-591).  A head-split Transpose (0, 2, 1, 3) that only feeds q, k or v
 * of such a block, and a head-merge one that alone reads its result, go as well: the call walks the [batch, tokens, heads,
 * head_dim] tensor on their far side through strides (device/x86/Transpose/transpose.c never runs for them).
 * The operands folded away have no buffer
 * (onrt_net_operand gives a null pointer for them).  ONENEW_RT_FUSE=0 keeps the operators separate.  n: how many blocks.
 */
int onrt_net_fused_attentions(const onrt_net_t *net, int32_t *n);

/*
 * Linear layers: MatMul -> Add of an initialiser over the last axis (-> Gelu), where nothing else reads the operands in
 * between, run as one call of the MatMul plugin's `eval_bias` / `eval_bias_gelu`, bit-equal to the separate operators
 * (device/x86/MatMul/mat_mul.c, Add/add.c:56-70, Gelu/gelu.c).  The operands folded away read as the layer's result.
 * ONENEW_RT_FUSE=0 keeps the operators separate.  n: how many layers.
 */
int onrt_net_fused_linears(const onrt_net_t *net, int32_t *n);
/* Of those layers, the ones (without Gelu) whose result goes, with no other reader, into an Add with an activation of the
 * same shape (the skip connection around a transformer block's projection): that Add joins the call (`eval_bias_add`,
 * the addend in inputs[3]), which then runs where the second Add stood.  n: how many. */
int onrt_net_fused_skips(const onrt_net_t *net, int32_t *n);

/*
 * One inference as a HIP graph, on request: with ONENEW_RT_GRAPH=1 in the environment at load time.  The operators
 * of a net are the same launches with the same addresses on every run, so the second call of onrt_net_run records
 * them (stream capture on a stream the net owns; the first call has packed the weights, sized the workspaces and
 * chosen the tiles) and later calls replay the recording with one hipGraphLaunch.  The recorded kernels and their
 * order are those of the plain run, so are the results.  It is not the default because onrt_net_run returns when
 * the outputs are complete: launched one by one the first operator starts while the host is still queueing the
 * rest, a replay starts nothing before the whole graph is submitted, and measured per-inference latency is higher
 * with it (ResNet-50 batch 1: 0.64 against 0.56 ms).  It pays where the host thread is the bottleneck.  Needs
 * plugins that export onhip_plugin_set_stream; when recording fails every run launches the operators one by one.
 * n: replays so far.
 */
int onrt_net_graph_launches(const onrt_net_t *net, int64_t *n);

/* Operators in execution order (host/net.h:309-330): type and name of number idx, count through n_ops. */
int onrt_net_op_count(const onrt_net_t *net, int32_t *n_ops);
int onrt_net_op_info(const onrt_net_t *net, int32_t idx, const char **op_type, const char **op_name);

/*
 * Shape and device address of any operand by name, after shape inference: the counterpart of the per-layer
 * dump mode (host/net.h:456-537), which reads operand_buf_map.  dev_ptr may be NULL.
 */
int onrt_net_operand(const onrt_net_t *net, const char *name, int32_t *ndim, int32_t shape[8], void **dev_ptr);

/*
 * One inference (extractor::impl, host/net.h:613-627).  inputs[i] / outputs[i] belong to input / output
 * number i and hold fp32 elements of that operand's shape; each may be host or device memory.  Inputs are
 * copied into the net's buffers, the operators run back to back on the device without a host wait in
 * between, outputs are copied out and are complete on return.  An outputs[i] of NULL skips that copy
 * (read the result in place through onrt_net_operand).
 */
int onrt_net_run(onrt_net_t *net, const void *const *inputs, void *const *outputs);
/*
 * The same inference without the wait at its end, for callers that keep the device busy with one batch after the other:
 * the copies into the net's input buffers, the operators and the copies of the outputs are queued on the default stream
 * (where the plugins launch) and the call returns; results are complete once that stream is (hipStreamSynchronize(NULL),
 * or any later work queued on it).  Every inputs[i] and non-NULL outputs[i] must be device memory; handed the net's own
 * buffers (onrt_net_operand) the call copies nothing.  A call must not be handed input memory that an earlier, still
 * running call is writing as its output.  Not for a net loaded with ONENEW_RT_GRAPH=1.  No counterpart in the reference,
 * whose host waits for every operator (host/net.h:613-627).
 */
int onrt_net_enqueue(onrt_net_t *net, const void *const *inputs, void *const *outputs);

/*
 * The model-wide GEMM tile: BLOCK_INFO_S.cuda_gemm_tile_{m,n,k} in the file header (common/nn_common.h:28-39;
 * the converter writes 16 / 16 / 16, tools/onnx2one/onnx2one.cpp:1346-1349), which every Conv call finds in its last
 * params slot (host/ops/conv.h:65-68).  The reference's tuner searches the tiles of its x86 GEMM on one 1024-cubed
 * product and writes them to the header (tools/optimize/auto_tuning.hpp:9-75); this one measures the loaded model
 * itself: onrt_net_tune_tiles runs the net with every workgroup tile the Conv plugin's library has kernels for, and
 * with none (each layer's tile from the cost model), `reps` timed inferences each on whatever the input buffers hold,
 * keeps the fastest (a candidate must win by 2 %, as auto_tuning.hpp:41) and leaves it set on the net; best_ms /
 * default_ms (may be NULL) are the fastest inference with it and with the converter's default.  tiles[2] is the depth
 * of a K tile in fp32 values (16), informational.  onrt_one_set_tiles writes a triple into the header of a file
 * image, so that every later load (onrt_net_load_*) starts from it; onrt_net_get_tiles / _set_tiles read and replace
 * the triple of a loaded net or a plan (a recorded graph is dropped and recorded again).
 */
int onrt_net_tune_tiles(onrt_net_t *net, int32_t reps, int32_t tiles[3], float *best_ms, float *default_ms);
int onrt_net_get_tiles(const onrt_net_t *net, int32_t tiles[3]);
int onrt_net_set_tiles(onrt_net_t *net, const int32_t tiles[3]);
int onrt_one_set_tiles(void *one_buf, size_t bytes, const int32_t tiles[3]);

/*
 * Model-level quantisation, the counterpart of model_quant (tools/optimize/model_quant.hpp:625-679): from an fp32 .one
 * image and calibration inputs to the W8A32 image the reference's optimiser writes.  The fp32 model is loaded with every
 * operator separate and run on each calibration input; for the input operand of every Conv the statistics of `method`
 * are taken on the device (the calibration passes of the kernel library, libonenew_hip.so beside the plugins):
 *   ONRT_QUANT_KL / ONRT_QUANT_MSE: the largest magnitude over `images` (first pass, :276-300), then the 2048-bin
 *     histogram of |x| over `images2` (second pass, :302-337; NULL = the same inputs again - the reference goes on
 *     reading its image list where the first pass stopped), then the KL (:345-431) or MSE (:585-618) threshold search;
 *   ONRT_QUANT_PERCENT: the 99.998 % magnitude over all of `images` (:83-185).
 * Then, as :657-670 and :31-81, every Conv gets input_scale = threshold / 127 and ifmap_quant2 = int8, its weights become
 * int8 (at the front of the initialiser, which keeps its fp32 size and type) with weight_aux = max |w| per output channel,
 * its bias int32 (quant_weight_bias, :6-29).  images / images2: n_images x (number of model inputs) pointers, input k of
 * calibration item i at [i * inputs + k], each a tensor of that input's shape in host or device memory.
 * quant_one_buf receives `bytes` bytes: the quantised image, loadable like any other.  A Conv that is int8 already is
 * refused.  The bytes behind the int8 weights inside their initialiser are zero here (the reference leaves the remains of
 * its in-place conversion there; nothing reads them).
 */
#define ONRT_QUANT_KL 0
#define ONRT_QUANT_MSE 1
#define ONRT_QUANT_PERCENT 2
int onrt_one_quantise(const void *one_buf, size_t bytes, const char *op_lib_dir, int32_t method,
                      const void *const *images, int32_t n_images, const void *const *images2, int32_t n_images2,
                      void *quant_one_buf);

#ifdef __cplusplus
}
#endif
#endif /* ONENEW_RT_H */
