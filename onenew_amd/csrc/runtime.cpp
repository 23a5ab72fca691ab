// Device-resident execution of a .one model (include/onenew_rt.h): file reader, operator objects, execution
// order, shape inference, buffers in HBM and the calls into the operator plugins.  Host code only; the
// kernels live behind `eval` in lib<Op>_hip.so.
//
// Follows the reference host step by step (host/net.h, host/op.h, host/ops/*.h), with three deliberate
// differences, all invisible to a batch-1 model the reference can run:
//   * operand buffers and initialisers are device memory, carved out of two allocations made at load time
//     (the reference makes one aligned_alloc per operand, host/net.h:434-449);
//   * Conv and GlobalAveragePool keep the batch dimension of their input (the reference writes 1,
//     host/ops/conv.h:43, host/ops/global_avgpool.h:33-36);
//   * an initialiser goes to the slot with the index it has among the node's inputs (for every operator and
//     operand order the reference host handles, this is the slot prepare_init_operand_data picks).
#include <dlfcn.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <array>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../../include/onenew_abi.h"
#include "../../include/onenew_rt.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define ONRT_HIP(expr)                                                                                     \
    do {                                                                                                   \
        hipError_t e_ = (expr);                                                                            \
        if (e_ != hipSuccess) return fail(ONRT_ERR_RUNTIME, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

// common/utils_c.h:4-7
inline size_t align64(size_t n) { return (n + 63) & ~(size_t) 63; }

// bytes per element of the data types an initialiser may carry (ONNX numbering, common/nn_common.h:92-110)
int elem_bytes(int32_t t) {
    switch (t) {
        case TYPE_FP32: case TYPE_INT32: return 4;
        case TYPE_UINT8: case TYPE_INT8: return 1;
        case TYPE_UINT16: case TYPE_INT16: case TYPE_FP16: case TYPE_BF16: return 2;
        case TYPE_INT64: case TYPE_FP64: return 8;
        default: return 0;
    }
}

// common/utils_c.h:9-16: all SHAPE_LEN entries are multiplied, unused ones hold 1.  -1 for a descriptor no tensor
// can have (an entry below 1, or more than 2^40 elements), so that a damaged file is refused instead of followed.
long long numel(const OPERAND_S &o) {
    long long n = 1;
    for (int i = 0; i < SHAPE_LEN; ++i) {
        if (o.shapes[i] < 1) return -1;
        n *= o.shapes[i];
        if (n > (1LL << 40)) return -1;
    }
    return n;
}

bool sane_rank(const OPERAND_S &o) { return o.dim_num_of_shapes >= 1 && o.dim_num_of_shapes <= SHAPE_LEN; }

// the node types this runtime runs, with the size of their config struct (the reference keeps this table in
// Manager::op_cfg_size_map, filled by OP_REGISTER_GLOBAL in each host/ops/*.h)
struct OpKind {
    const char *type;
    size_t cfg_size;
    bool view;   // no buffer of its own, no plugin call
    bool fold_only = false;   // runs only as part of the Conv in front of it (fold_activations_into_conv), no plugin of its own
};
const OpKind kOps[] = {
    {"Conv", sizeof(CONV_CONFIG_S), false},
    {"MatMul", sizeof(MATMUL_CONFIG_S), false},
    {"Gemm", sizeof(GEMM_CONFIG_S), false},
    {"Add", sizeof(ADD_CONFIG_S), false},
    {"Relu", sizeof(RELU_CONFIG_S), false},
    {"MaxPool", sizeof(MAX_POOL_CONFIG_S), false},
    {"GlobalAveragePool", sizeof(GLOBAL_AVGPOOL_CONFIG_S), false},
    {"Gelu", sizeof(GELU_CONFIG_S), false},
    {"LayerNormalization", sizeof(LAYERNORMALIZATION_CONFIG_S), false},
    {"Softmax", sizeof(SOFTMAX_CONFIG_S), false},
    {"Transpose", sizeof(TRANSPOSE_CONFIG_S), false},
    {"Flatten", sizeof(FLATTEN_CONFIG_S), true},
    {"Reshape", sizeof(RESHAPE_CONFIG_S), true},
    // what the offline optimiser folds into a Conv (tools/optimize/op_fusion.hpp:75-192), for files that have not been through it
    {"Clip", sizeof(CLIP_CONFIG_S), false, true},
    {"LeakyRelu", sizeof(LEAKYRELU_CONFIG_S), false, true},
    {"Sigmoid", sizeof(SIGMOID_CONFIG_S), false, true},
    {"HardSigmoid", sizeof(HARD_SIGMOID_CONFIG_S), false, true},
    {"Mul", sizeof(MUL_CONFIG_S), false, true},
};
const OpKind *find_kind(const char *type) {
    for (const OpKind &k : kOps)
        if (!strcmp(k.type, type)) return &k;
    return nullptr;
}

struct Tensor {
    OPERAND_S desc;
    void *dev = nullptr;
    size_t bytes = 0;
    bool is_init = false;
    bool produced = false;   // an io input, an initialiser or the output of an operator already ordered
    std::string alias;       // an operand folded away with its producer reads as this one (fuse_residual_blocks)
    bool never_written = false;   // an operand inside a fused attention block: it has no buffer and no value
    bool as_s8 = false;           // written and read as int8 NHWC, channels padded to 16 (link_int8_convs)
    bool has_twin = false;        // fp32, and stored once more as int8 NHWC for the int8 convolutions among its readers
    void *twin_dev = nullptr;
};

struct Node {
    const OpKind *kind = nullptr;
    std::vector<char> cfg;   // the node's config struct, as in the file
    std::vector<std::string> in, out;
    onenew_eval_fn eval = nullptr;
    int fuse = 0;            // Conv: 1 = the Add after it is folded in, 2 = and the Relu after that
    std::string addend, fused_out;
    int32_t token_major[4] = {0, 0, 0, 0};   // fused attention: q, k, v, result stored [batch, tokens, heads, head_dim]
    int block_dw = -1, block_pw = -1;        // fused inverted-residual block (fuse 7): its depthwise and last convolutions;
                                             // fused pair (fuse 8): block_pw is its 1x1 convolution
    // an int8 convolution whose input and/or result travel as int8 NHWC (link_int8_convs): what `eval_link` reads from
    // inputs[4] ({in_s8, out_s8, out_scale}) and inputs[5] (the fold code, when an Add is folded in)
    struct { int32_t in_s8, out_s8; float out_scale; int32_t twin; } link = {0, 0, 0.0f, 0};
    int32_t link_fuse = 0;
    bool reads_twin = false;   // its input is the int8 copy of an fp32 operand
    BUFFER_INFO_S params[BUF_MAXNUM], inputs[BUF_MAXNUM], outputs[BUF_MAXNUM];
    const BASE_CONFIG_S *base() const { return reinterpret_cast<const BASE_CONFIG_S *>(cfg.data()); }
};

typedef int (*set_async_fn)(int);
typedef int (*forget_fn)(const void *, size_t);
typedef int (*set_stream_fn)(void *);

}  // namespace

struct onrt_net {
    std::vector<char> file;
    std::vector<Node> nodes;
    std::vector<int> order;
    std::map<std::string, Tensor> tensors;   // operand_stu_map and operand_buf_map of the reference in one
    std::vector<std::string> in_names, out_names;
    USEFUL_INFO_S useful;
    std::string lib_dir;
    std::map<std::string, void *> handles;
    std::vector<set_async_fn> async_switches;
    std::set<forget_fn> forgetters;   // plugins that keep re-laid-out copies of device-resident weights
    std::set<set_stream_fn> stream_setters;
    size_t plugin_libs = 0;           // libraries bound; a graph needs every one of them to follow set_stream
    // one inference as a HIP graph: recorded on the net's own stream during the second run (the first one packs
    // weights, sizes workspaces and measures tile choices, none of which can be recorded), replayed from then on
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    bool graph_wanted = false, graph_failed = false;   // asked for with ONENEW_RT_GRAPH=1
    bool graph_refused = false;
    bool plan_only = false;           // onrt_net_plan_buf: no plugins, no device memory
    long long runs = 0, graph_launches = 0;
    size_t init_bytes = 0;
    onenew_eval_fn conv_add = nullptr, conv_add_relu = nullptr;   // optional entry points of the Conv plugin
    onenew_eval_fn conv_block = nullptr, conv_block_takes = nullptr, conv_link = nullptr, conv_link_takes = nullptr;
    onenew_eval_fn conv_pair = nullptr, conv_pair_relu = nullptr, conv_pair_takes = nullptr;
    onenew_eval_fn maxpool_s8 = nullptr;   // optional entry point of the MaxPool plugin
    onenew_eval_fn matmul_attention = nullptr, matmul_bias = nullptr, matmul_bias_gelu = nullptr, matmul_bias_add = nullptr;   // optional entry points of the MatMul plugin
    int fused_blocks = 0, folded_relus = 0, folded_acts = 0, fused_attentions = 0, fused_linears = 0, fused_skips = 0, fused_ir_blocks = 0, fused_pairs = 0, int8_links = 0;
    void *init_arena = nullptr, *act_arena = nullptr, *tables = nullptr;
    std::vector<float> silu_lut, gelu_lut;
};

namespace {

const ONE_MODEL_DESC_S *header(const onrt_net &n) { return reinterpret_cast<const ONE_MODEL_DESC_S *>(n.file.data()); }

// ---- reading the file (host/net.h:138-221) ------------------------------------------------------------
int read_model(onrt_net &net) {
    const size_t size = net.file.size();
    if (size < sizeof(ONE_MODEL_DESC_S)) return fail(ONRT_ERR_FORMAT, "file of %zu bytes is shorter than the header", size);
    const ONE_MODEL_DESC_S *h = header(net);
    if (h->one_model_magic_num != ONE_MAGIC_NUM)
        return fail(ONRT_ERR_FORMAT, "one_model_magic_num is 0x%x, a .one file starts with 0x%x", h->one_model_magic_num, ONE_MAGIC_NUM);
    if (h->node_cnt < 0 || h->init_cnt < 0 || h->io_cfg_cnt < 0 || h->node_cfg_offset < 0 || h->init_info_offset < 0 ||
        h->io_cfg_offset < 0)
        return fail(ONRT_ERR_FORMAT, "negative count or offset in the header");
    net.useful = h->useful_info;

    // initialisers first: the operators look their inputs up among them
    size_t off = (size_t) h->init_info_offset;
    for (int i = 0; i < h->init_cnt; ++i) {
        if (off + sizeof(OPERAND_S) > size) return fail(ONRT_ERR_FORMAT, "initialiser %d starts past the end of the file", i);
        Tensor t;
        memcpy(&t.desc, net.file.data() + off, sizeof(OPERAND_S));
        t.desc.operand_name[OPERAND_NAME_LEN - 1] = 0;
        const int eb = elem_bytes(t.desc.data_type);
        const long long n = numel(t.desc);
        if (!eb || n < 0 || !sane_rank(t.desc))
            return fail(ONRT_ERR_FORMAT, "initialiser %s: data type %d, rank %d, %lld elements", t.desc.operand_name, t.desc.data_type,
                        t.desc.dim_num_of_shapes, n);
        t.bytes = (size_t) n * eb;
        if (off + sizeof(OPERAND_S) + t.bytes > size)
            return fail(ONRT_ERR_FORMAT, "initialiser %s ends past the end of the file", t.desc.operand_name);
        t.is_init = true;
        t.produced = true;
        t.desc.p_data = (int64_t) (off + sizeof(OPERAND_S));   // offset of the data in the file until uploaded
        net.tensors[t.desc.operand_name] = t;
        off += align64(sizeof(OPERAND_S) + t.bytes);
    }

    // io nodes (host/ops/io.h:56-70): "input" produces its operand, "output" names one to hand back
    off = (size_t) h->io_cfg_offset;
    for (int i = 0; i < h->io_cfg_cnt; ++i) {
        if (off + sizeof(IO_CONFIG_S) > size) return fail(ONRT_ERR_FORMAT, "io config %d ends past the end of the file", i);
        IO_CONFIG_S io;
        memcpy(&io, net.file.data() + off, sizeof(io));
        io.op_type[OP_TYPE_LEN - 1] = io.op_name[OP_NAME_LEN - 1] = io.operand.operand_name[OPERAND_NAME_LEN - 1] = 0;
        if (strcmp(io.op_type, "io")) return fail(ONRT_ERR_FORMAT, "io config %d has op_type '%s'", i, io.op_type);
        const std::string name(io.operand.operand_name);
        if (!strcmp(io.op_name, "input")) {
            if (io.operand.data_type != TYPE_FP32) return fail(ONRT_ERR_FORMAT, "input %s is not fp32", name.c_str());
            if (!sane_rank(io.operand) || numel(io.operand) < 1 || numel(io.operand) >= (1LL << 31))
                return fail(ONRT_ERR_FORMAT, "input %s: rank %d, %lld elements", name.c_str(), io.operand.dim_num_of_shapes, numel(io.operand));
            Tensor t;
            t.desc = io.operand;
            t.produced = true;
            net.tensors[name] = t;
            net.in_names.push_back(name);
        } else if (!strcmp(io.op_name, "output")) {
            net.out_names.push_back(name);
        } else {
            return fail(ONRT_ERR_FORMAT, "io config %d is neither input nor output ('%s')", i, io.op_name);
        }
        off += align64(sizeof(IO_CONFIG_S));
    }

    // operator nodes
    off = (size_t) h->node_cfg_offset;
    for (int i = 0; i < h->node_cnt; ++i) {
        if (off + sizeof(BASE_CONFIG_S) > size) return fail(ONRT_ERR_FORMAT, "node %d starts past the end of the file", i);
        char type[OP_TYPE_LEN];
        memcpy(type, net.file.data() + off, OP_TYPE_LEN);
        type[OP_TYPE_LEN - 1] = 0;
        const OpKind *kind = find_kind(type);
        if (!kind) return fail(ONRT_ERR_FORMAT, "node %d: no HIP operator for type '%s'", i, type);
        if (off + kind->cfg_size > size) return fail(ONRT_ERR_FORMAT, "node %d (%s) ends past the end of the file", i, type);
        Node nd;
        nd.kind = kind;
        nd.cfg.assign(net.file.data() + off, net.file.data() + off + kind->cfg_size);
        BASE_CONFIG_S *b = reinterpret_cast<BASE_CONFIG_S *>(nd.cfg.data());
        b->op_name[OP_NAME_LEN - 1] = 0;
        if (b->in_operand_num < 1 || b->in_operand_num > OPERAND_MAXNUM || b->out_operand_num < 1 || b->out_operand_num > OPERAND_MAXNUM)
            return fail(ONRT_ERR_FORMAT, "node %s: %d inputs, %d outputs", b->op_name, b->in_operand_num, b->out_operand_num);
        for (int k = 0; k < b->in_operand_num; ++k) {
            b->in_operand_name[k][OPERAND_NAME_LEN - 1] = 0;
            nd.in.push_back(b->in_operand_name[k]);
        }
        for (int k = 0; k < b->out_operand_num; ++k) {
            b->out_operand_name[k][OPERAND_NAME_LEN - 1] = 0;
            nd.out.push_back(b->out_operand_name[k]);
        }
        memset(nd.params, 0, sizeof(nd.params));
        memset(nd.inputs, 0, sizeof(nd.inputs));
        memset(nd.outputs, 0, sizeof(nd.outputs));
        net.nodes.push_back(std::move(nd));
        off += align64(kind->cfg_size);
    }
    return ONRT_OK;
}

// ---- execution order (host/net.h:274-330) -------------------------------------------------------------
// A node is ready when every non-empty input is an initialiser, a net input or the output of a node already
// placed; among ready nodes the first in file order goes next.
int order_nodes(onrt_net &net) {
    std::vector<bool> placed(net.nodes.size(), false);
    for (size_t done = 0; done < net.nodes.size(); ++done) {
        int pick = -1;
        for (size_t i = 0; i < net.nodes.size() && pick < 0; ++i) {
            if (placed[i]) continue;
            bool ready = true;
            for (const std::string &name : net.nodes[i].in) {
                if (name.empty()) continue;
                auto it = net.tensors.find(name);
                if (it == net.tensors.end() || !it->second.produced) { ready = false; break; }
            }
            if (ready) pick = (int) i;
        }
        if (pick < 0) return fail(ONRT_ERR_FORMAT, "the graph has a cycle or an operand nobody produces (%zu of %zu nodes ordered)", done, net.nodes.size());
        placed[pick] = true;
        net.order.push_back(pick);
        for (const std::string &name : net.nodes[pick].out) {
            Tensor &t = net.tensors[name];
            memset(&t.desc, 0, sizeof(t.desc));
            snprintf(t.desc.operand_name, OPERAND_NAME_LEN, "%s", name.c_str());
            t.desc.data_type = TYPE_FP32;
            t.produced = true;
        }
    }
    for (const std::string &name : net.out_names)
        if (!net.tensors.count(name)) return fail(ONRT_ERR_FORMAT, "output %s is not produced by any node", name.c_str());
    return ONRT_OK;
}

// ---- shape inference (shape_infer of each host/ops/*.h) -----------------------------------------------
int infer_shapes(onrt_net &net) {
    for (int idx : net.order) {
        Node &nd = net.nodes[idx];
        const char *type = nd.kind->type;
        const Tensor &in0 = net.tensors[nd.in[0]];
        const OPERAND_S &in = in0.desc;
        OPERAND_S &out = net.tensors[nd.out[0]].desc;
        auto init_at = [&](size_t k) -> const Tensor * {
            if (k >= nd.in.size()) return nullptr;
            auto it = net.tensors.find(nd.in[k]);
            return it != net.tensors.end() && it->second.is_init ? &it->second : nullptr;
        };
        if (nd.in[0].empty() || !sane_rank(in))
            return fail(ONRT_ERR_FORMAT, "%s %s: first input of rank %d", type, nd.base()->op_name, in.dim_num_of_shapes);
        memcpy(out.shapes, in.shapes, sizeof(out.shapes));
        out.dim_num_of_shapes = in.dim_num_of_shapes;
        if (!strcmp(type, "Conv")) {   // host/ops/conv.h:31-58
            const CONV_CONFIG_S *c = reinterpret_cast<const CONV_CONFIG_S *>(nd.cfg.data());
            const Tensor *w = init_at(1);
            if (!w) return fail(ONRT_ERR_FORMAT, "Conv %s: the weight is not an initialiser", nd.base()->op_name);
            if (in.dim_num_of_shapes != 4) return fail(ONRT_ERR_FORMAT, "Conv %s: input of rank %d", nd.base()->op_name, in.dim_num_of_shapes);
            if (c->has_bias && !init_at(2)) return fail(ONRT_ERR_FORMAT, "Conv %s: the bias is not an initialiser", nd.base()->op_name);
            if (c->strides[0] < 1 || c->strides[1] < 1) return fail(ONRT_ERR_FORMAT, "Conv %s: stride below 1", nd.base()->op_name);
            out.shapes[1] = w->desc.shapes[0];
            out.shapes[2] = (int32_t) ((in.shapes[2] + c->pads[0] + c->pads[2] - c->kernel_shape[0]) / c->strides[0] + 1);
            out.shapes[3] = (int32_t) ((in.shapes[3] + c->pads[1] + c->pads[3] - c->kernel_shape[1]) / c->strides[1] + 1);
        } else if (!strcmp(type, "MaxPool")) {   // host/ops/maxpool.h:29-53
            const MAX_POOL_CONFIG_S *c = reinterpret_cast<const MAX_POOL_CONFIG_S *>(nd.cfg.data());
            if (c->strides[0] < 1 || c->strides[1] < 1) return fail(ONRT_ERR_FORMAT, "MaxPool %s: stride below 1", nd.base()->op_name);
            out.shapes[2] = (int32_t) ((in.shapes[2] + c->pads[0] + c->pads[2] - c->kernel_shape[0]) / c->strides[0] + 1);
            out.shapes[3] = (int32_t) ((in.shapes[3] + c->pads[1] + c->pads[3] - c->kernel_shape[1]) / c->strides[1] + 1);
        } else if (!strcmp(type, "GlobalAveragePool")) {   // host/ops/global_avgpool.h:29-45
            for (int i = 2; i < SHAPE_LEN; ++i) out.shapes[i] = 1;
        } else if (!strcmp(type, "Gemm")) {   // host/ops/gemm.h:28-48: the last dimension becomes the bias length
            const Tensor *b = init_at(2);
            if (!init_at(1) || !b) return fail(ONRT_ERR_FORMAT, "Gemm %s: weight and bias must be initialisers", nd.base()->op_name);
            out.shapes[out.dim_num_of_shapes - 1] = (int32_t) numel(b->desc);
        } else if (!strcmp(type, "MatMul")) {   // host/ops/mat_mul.h:32-57
            if (nd.in.size() < 2) return fail(ONRT_ERR_FORMAT, "MatMul %s: one input", nd.base()->op_name);
            const OPERAND_S &b = net.tensors[nd.in[1]].desc;
            if (nd.in[1].empty() || !sane_rank(b))
                return fail(ONRT_ERR_FORMAT, "MatMul %s: second input of rank %d", nd.base()->op_name, b.dim_num_of_shapes);
            out.shapes[out.dim_num_of_shapes - 1] = b.shapes[b.dim_num_of_shapes - 1];
        } else if (!strcmp(type, "Add")) {   // host/ops/add.h:32-57
            if (nd.in.size() < 2) return fail(ONRT_ERR_FORMAT, "Add %s: one input", nd.base()->op_name);
            const Tensor &t1 = net.tensors[nd.in[1]];
            if (in0.is_init) {
                memcpy(out.shapes, t1.desc.shapes, sizeof(out.shapes));
                out.dim_num_of_shapes = t1.desc.dim_num_of_shapes;
            } else if (!t1.is_init && t1.desc.dim_num_of_shapes == in.dim_num_of_shapes) {
                for (int i = 0; i < out.dim_num_of_shapes; ++i) out.shapes[i] = in.shapes[i] > t1.desc.shapes[i] ? in.shapes[i] : t1.desc.shapes[i];
            }
        } else if (!strcmp(type, "Transpose")) {   // host/ops/transpose.h:32-49
            const TRANSPOSE_CONFIG_S *c = reinterpret_cast<const TRANSPOSE_CONFIG_S *>(nd.cfg.data());
            if (c->perm_num < 0 || c->perm_num > SHAPE_LEN) return fail(ONRT_ERR_FORMAT, "Transpose %s: perm_num %lld", nd.base()->op_name, (long long) c->perm_num);
            for (int i = 0; i < c->perm_num; ++i) {
                if (c->perm[i] < 0 || c->perm[i] >= SHAPE_LEN) return fail(ONRT_ERR_FORMAT, "Transpose %s: perm[%d] = %lld", nd.base()->op_name, i, (long long) c->perm[i]);
                out.shapes[i] = in.shapes[c->perm[i]];
            }
        } else if (!strcmp(type, "Flatten")) {   // host/ops/flatten.h:29-62
            const FLATTEN_CONFIG_S *c = reinterpret_cast<const FLATTEN_CONFIG_S *>(nd.cfg.data());
            if (c->axis < 0 || c->axis >= SHAPE_LEN) return fail(ONRT_ERR_FORMAT, "Flatten %s: axis %lld", nd.base()->op_name, (long long) c->axis);
            out.not_need_buf = 1;
            for (int i = 0; i < SHAPE_LEN; ++i) out.shapes[i] = 1;
            for (int i = 0; i < c->axis; ++i) out.shapes[i] = in.shapes[i];
            out.dim_num_of_shapes = (int32_t) c->axis + 1;
            for (int i = (int) c->axis; i < SHAPE_LEN; ++i) out.shapes[c->axis] *= in.shapes[i];
            if (in.dim_num_of_shapes == 3 && in.shapes[0] == 1 && c->axis == 2) {   // the reference's special case
                out.shapes[0] = in.shapes[1];
                out.shapes[1] = in.shapes[2];
                out.shapes[2] = 1;
                out.dim_num_of_shapes = 2;
            }
        } else if (!strcmp(type, "Reshape")) {   // host/ops/reshape.h:31-70
            const RESHAPE_CONFIG_S *c = reinterpret_cast<const RESHAPE_CONFIG_S *>(nd.cfg.data());
            if (c->dst_shape_num < 1 || c->dst_shape_num > SHAPE_LEN) return fail(ONRT_ERR_FORMAT, "Reshape %s: dst_shape_num %lld", nd.base()->op_name, (long long) c->dst_shape_num);
            out.not_need_buf = 1;
            const long long total = numel(in);
            long long known = 1;
            for (int i = 0; i < SHAPE_LEN; ++i) out.shapes[i] = 1;
            for (int i = 0; i < c->dst_shape_num; ++i) {
                if (c->dst_shape[i] != -1 && (c->dst_shape[i] < 1 || c->dst_shape[i] > total))
                    return fail(ONRT_ERR_FORMAT, "Reshape %s: dimension %d is %lld", nd.base()->op_name, i, (long long) c->dst_shape[i]);
                out.shapes[i] = (int32_t) c->dst_shape[i];
                if (c->dst_shape[i] != -1) known *= c->dst_shape[i];
            }
            for (int i = 0; i < c->dst_shape_num; ++i)
                if (out.shapes[i] == -1) out.shapes[i] = known ? (int32_t) (total / known) : 0;
            out.dim_num_of_shapes = (int32_t) c->dst_shape_num;
            if (numel(out) != total) return fail(ONRT_ERR_FORMAT, "Reshape %s changes the element count (%lld to %lld)", nd.base()->op_name, total, numel(out));
        }
        // Relu, Gelu, LayerNormalization, Softmax: the input's shape
        const long long n = numel(out);
        if (n <= 0 || n >= (1LL << 31) || !sane_rank(out))
            return fail(ONRT_ERR_FORMAT, "%s %s: output of rank %d, %lld elements", type, nd.base()->op_name, out.dim_num_of_shapes, n);
    }
    return ONRT_OK;
}

// ---- buffers (host/net.h:419-452) ---------------------------------------------------------------------
int allocate(onrt_net &net) {
    // initialisers: one allocation, uploaded once
    size_t init_total = 0, act_total = 0;
    for (auto &kv : net.tensors)
        if (kv.second.is_init) init_total += (kv.second.bytes + 255) & ~(size_t) 255;
    if (init_total) {
        ONRT_HIP(hipMalloc(&net.init_arena, init_total));
        net.init_bytes = init_total;
        size_t off = 0;
        for (auto &kv : net.tensors) {
            Tensor &t = kv.second;
            if (!t.is_init) continue;
            t.dev = static_cast<char *>(net.init_arena) + off;
            if (t.bytes) ONRT_HIP(hipMemcpy(t.dev, net.file.data() + (size_t) t.desc.p_data, t.bytes, hipMemcpyHostToDevice));
            t.desc.p_data = 0;
            off += (t.bytes + 255) & ~(size_t) 255;
        }
    }
    // operands: fp32 elements (elem_size * sizeof(float) in the reference), views excepted
    for (auto &kv : net.tensors) {
        Tensor &t = kv.second;
        if (t.is_init || t.desc.not_need_buf || !t.alias.empty() || t.never_written) continue;
        t.bytes = (size_t) numel(t.desc) * 4;
        if (t.as_s8) {   // [n, h, w, channels padded to 16] bytes, where that is more
            const size_t s8 = (size_t) t.desc.shapes[0] * t.desc.shapes[2] * t.desc.shapes[3] * (((size_t) t.desc.shapes[1] + 15) / 16 * 16);
            if (s8 > t.bytes) t.bytes = s8;
        }
        act_total += (t.bytes + 255) & ~(size_t) 255;
        if (t.has_twin) act_total += ((size_t) numel(t.desc) + 255) & ~(size_t) 255;   // a byte per element, no padding channels
    }
    if (act_total) {
        ONRT_HIP(hipMalloc(&net.act_arena, act_total));
        size_t off = 0;
        for (auto &kv : net.tensors) {
            Tensor &t = kv.second;
            if (t.is_init || t.desc.not_need_buf || !t.alias.empty() || t.never_written) continue;
            t.dev = static_cast<char *>(net.act_arena) + off;
            off += (t.bytes + 255) & ~(size_t) 255;
            if (t.has_twin) {
                t.twin_dev = static_cast<char *>(net.act_arena) + off;
                off += ((size_t) numel(t.desc) + 255) & ~(size_t) 255;
            }
        }
    }
    for (auto &kv : net.tensors) {
        Tensor &t = kv.second;
        if (t.alias.empty()) continue;
        const Tensor *target = &net.tensors[t.alias];
        while (!target->alias.empty()) target = &net.tensors[target->alias];   // a folded Relu inside a folded block
        t.dev = target->dev;
        t.bytes = target->bytes;
    }
    // a view shares the buffer of its input (host/op.h:149-154), in execution order so that chains resolve
    for (int idx : net.order) {
        const Node &nd = net.nodes[idx];
        if (!nd.kind->view) continue;
        const Tensor &src = net.tensors[nd.in[0]];
        Tensor &dst = net.tensors[nd.out[0]];
        dst.dev = src.dev;
        dst.bytes = src.bytes;
    }
    return ONRT_OK;
}

// ---- activation tables (host/ops/conv.h:178-194, host/ops/gelu.h:80-96), built with the host's libm like
// the reference host does, then kept on the device
int build_tables(onrt_net &net) {
    bool need_silu = false, need_gelu = false;
    for (const Node &nd : net.nodes) {
        if (!strcmp(nd.kind->type, "Conv") && reinterpret_cast<const CONV_CONFIG_S *>(nd.cfg.data())->act_type == SILU) need_silu = true;
        if (!strcmp(nd.kind->type, "Gelu")) need_gelu = true;
    }
    if (!need_silu && !need_gelu) return ONRT_OK;
    const float single_limit = 8.0f;
    const float step = 1.0 / 512;
    const int32_t lut_len = (int32_t) (2.0f * single_limit / step);
    net.silu_lut.resize(lut_len);
    net.gelu_lut.resize(lut_len);
    const float inv_sqrt2 = 1.0f / 1.4142f;
    for (int i = 0; i < lut_len; ++i) {
        const float x = i * step - single_limit;
        net.silu_lut[i] = x / (1 + expf(-x));
        net.gelu_lut[i] = x * 0.5 * (1 + erf(x * inv_sqrt2));
    }
    ONRT_HIP(hipMalloc(&net.tables, 2 * (size_t) lut_len * 4));
    ONRT_HIP(hipMemcpy(net.tables, net.silu_lut.data(), (size_t) lut_len * 4, hipMemcpyHostToDevice));
    ONRT_HIP(hipMemcpy(static_cast<float *>(net.tables) + lut_len, net.gelu_lut.data(), (size_t) lut_len * 4, hipMemcpyHostToDevice));
    return ONRT_OK;
}

// ---- plugins (host/op.h:41-80) ------------------------------------------------------------------------
std::string own_directory() {
    Dl_info info;
    if (dladdr(reinterpret_cast<void *>(&own_directory), &info) && info.dli_fname) {
        std::string p(info.dli_fname);
        const size_t slash = p.rfind('/');
        return slash == std::string::npos ? std::string(".") : p.substr(0, slash);
    }
    return ".";
}

int bind_plugins(onrt_net &net) {
    for (Node &nd : net.nodes) {
        if (nd.kind->view || nd.kind->fold_only) continue;
        const std::string type(nd.kind->type);
        auto it = net.handles.find(type);
        if (it == net.handles.end()) {
            const std::string nested = net.lib_dir + "/" + type + "/lib" + type + "_hip.so";
            const std::string flat = net.lib_dir + "/lib" + type + "_hip.so";
            void *h = dlopen(nested.c_str(), RTLD_LAZY | RTLD_LOCAL);
            if (!h) h = dlopen(flat.c_str(), RTLD_LAZY | RTLD_LOCAL);
            if (!h) return fail(ONRT_ERR_PLUGIN, "the handle of %s op is not found: tried %s and %s (%s)", type.c_str(), nested.c_str(), flat.c_str(), dlerror());
            it = net.handles.emplace(type, h).first;
            // our plugins can leave a device-resident output to stream order instead of waiting for it
            if (set_async_fn f = reinterpret_cast<set_async_fn>(dlsym(h, "onhip_plugin_set_async"))) net.async_switches.push_back(f);
            if (forget_fn f = reinterpret_cast<forget_fn>(dlsym(h, "onhip_plugin_forget"))) net.forgetters.insert(f);
            ++net.plugin_libs;
            if (set_stream_fn f = reinterpret_cast<set_stream_fn>(dlsym(h, "onhip_plugin_set_stream"))) net.stream_setters.insert(f);
            else net.graph_refused = true;   // a plugin that launches where it likes cannot be recorded
        }
        nd.eval = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval"));
        if (!nd.eval) return fail(ONRT_ERR_PLUGIN, "no eval in the %s plugin", type.c_str());
        if (type == "Conv") {
            net.conv_add = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_add"));
            net.conv_add_relu = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_add_relu"));
            net.conv_block = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_block"));
            net.conv_block_takes = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_block_takes"));
            net.conv_pair = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_pair"));
            net.conv_pair_relu = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_pair_relu"));
            net.conv_pair_takes = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_pair_takes"));
            net.conv_link = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_link"));
            net.conv_link_takes = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_link_takes"));
        }
        if (type == "MaxPool") net.maxpool_s8 = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_s8"));
        if (type == "MatMul") {
            net.matmul_attention = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_attention"));
            net.matmul_bias = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_bias"));
            net.matmul_bias_gelu = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_bias_gelu"));
            net.matmul_bias_add = reinterpret_cast<onenew_eval_fn>(dlsym(it->second, "eval_bias_add"));
        }
    }
    return ONRT_OK;
}

// ---- Relu after Conv ------------------------------------------------------------------------------------
// What the reference's offline optimiser does to Conv -> Relu (tools/optimize/op_fusion.hpp:47-222: the Relu node goes
// and the Conv's act_type becomes RELU), done at load time for a file that has not been through it.  Only where the
// reference's kernel would apply the activation: a convolution with a bias (conv.c:18-27 returns before do_act without
// one) and no activation yet, whose result only the Relu reads.  As in the optimised file, the activation is then
// do_act's "x > 0 ? x : 0" (a NaN becomes 0) instead of relu.c's vector rule.  ONENEW_RT_FUSE=0 leaves the file as it is.
thread_local bool tl_load_unfused = false;   // set around the load inside onrt_one_quantise: every operand gets a buffer
bool fusing_enabled() {
    if (tl_load_unfused) return false;
    const char *env = getenv("ONENEW_RT_FUSE");
    return !(env && !strcmp(env, "0"));
}

bool is_net_output(const onrt_net &net, const std::string &name) {
    return std::find(net.out_names.begin(), net.out_names.end(), name) != net.out_names.end();
}

// index of the only node reading `name`, if it is of the given type and the operand is not a net output; else -1.
// The other operand of an Add folded into a convolution or a MatMul (Node::addend) is a read like any input: the Add
// itself is no longer in the order, and what it read must still be written.
int sole_reader(const onrt_net &net, const std::string &name, const char *type) {
    if (is_net_output(net, name)) return -1;
    int found = -1;
    for (int idx : net.order) {
        const Node &nd = net.nodes[idx];
        for (const std::string &in : nd.in)
            if (in == name) {
                if (found >= 0) return -1;   // a second reader, or the same node twice
                found = idx;
            }
        if (!nd.addend.empty() && nd.addend == name) {
            if (found >= 0) return -1;
            found = idx;
        }
    }
    if (found < 0 || strcmp(net.nodes[found].kind->type, type)) return -1;
    return found;
}

// every node that reads `name` (as an input or as the other operand of a folded Add), in execution order
std::vector<int> readers_of(const onrt_net &net, const std::string &name) {
    std::vector<int> out;
    for (int idx : net.order) {
        const Node &nd = net.nodes[idx];
        for (const std::string &in : nd.in)
            if (in == name) out.push_back(idx);
        if (!nd.addend.empty() && nd.addend == name) out.push_back(idx);
    }
    return out;
}

// The activation after a Conv becomes the Conv's act_type, as the offline optimiser does it (tools/optimize/
// op_fusion.hpp: Relu :47-73, Clip :75-103, LeakyRelu :105-132, Sigmoid x Mul = SiLU :134-160, HardSigmoid x Mul
// :162-192; sub-graph patterns :485-539), so a file that has not been through the optimiser runs like one that has.
// Only for a Conv with a bias and no activation yet: a Conv without bias returns before the activation in the
// reference's kernel (device/x86/Conv/conv.c:18-27).  The Relu fold obeys ONENEW_RT_FUSE (this package has a Relu
// operator to run instead); the other node types exist here only folded, so they are folded whatever the switch
// says, and one that no Conv takes is refused.
int fold_activations_into_conv(onrt_net &net) {
    std::vector<bool> dropped(net.nodes.size(), false);
    auto unary = [&](int ni) { return net.nodes[ni].in.size() == 1 && net.nodes[ni].out.size() == 1; };
    for (int idx : net.order) {
        Node &conv = net.nodes[idx];
        if (strcmp(conv.kind->type, "Conv") || conv.out.size() != 1) continue;
        CONV_CONFIG_S *cfg = reinterpret_cast<CONV_CONFIG_S *>(conv.cfg.data());
        if (!cfg->has_bias || cfg->act_type != NOT_ACT) continue;
        const std::string &mid = conv.out[0];
        if (is_net_output(net, mid)) continue;
        const std::vector<int> rd = readers_of(net, mid);
        std::string result;
        if (rd.size() == 1 && unary(rd[0])) {
            Node &act = net.nodes[rd[0]];
            const char *t = act.kind->type;
            if (!strcmp(t, "Relu")) {
                if (!fusing_enabled()) continue;
                cfg->act_type = RELU;
                ++net.folded_relus;
            } else if (!strcmp(t, "Clip")) {
                const CLIP_CONFIG_S *c = reinterpret_cast<const CLIP_CONFIG_S *>(act.cfg.data());
                cfg->act_type = CLIP;
                cfg->clip_min = c->min;
                cfg->clip_max = c->max;
                ++net.folded_acts;
            } else if (!strcmp(t, "LeakyRelu")) {
                cfg->act_type = LEAKYRELU;
                cfg->leaky_relu_alpha = reinterpret_cast<const LEAKYRELU_CONFIG_S *>(act.cfg.data())->alpha;
                ++net.folded_acts;
            } else {
                continue;
            }
            result = act.out[0];
            dropped[rd[0]] = true;
        } else if (rd.size() == 2 && rd[0] != rd[1]) {
            // x -> gate(x), then x * gate(x): the gate reads the convolution alone, the Mul reads the convolution and the gate
            int gi = rd[0], mi = rd[1];
            if (!strcmp(net.nodes[gi].kind->type, "Mul")) std::swap(gi, mi);
            Node &gate = net.nodes[gi], &mul = net.nodes[mi];
            const bool sig = !strcmp(gate.kind->type, "Sigmoid"), hard = !strcmp(gate.kind->type, "HardSigmoid");
            if ((!sig && !hard) || strcmp(mul.kind->type, "Mul") || !unary(gi) || mul.in.size() != 2 || mul.out.size() != 1) continue;
            const std::string &g = gate.out[0];
            if (!((mul.in[0] == mid && mul.in[1] == g) || (mul.in[1] == mid && mul.in[0] == g))) continue;
            if (is_net_output(net, g) || readers_of(net, g).size() != 1) continue;
            if (sig) {
                cfg->act_type = SILU;
            } else {
                const HARD_SIGMOID_CONFIG_S *c = reinterpret_cast<const HARD_SIGMOID_CONFIG_S *>(gate.cfg.data());
                cfg->act_type = HARDSILU;
                cfg->hard_sigmoid_alpha = c->alpha;
                cfg->hard_sigmoid_beta = c->beta;
            }
            ++net.folded_acts;
            result = mul.out[0];
            net.tensors[g].alias = result;
            dropped[gi] = dropped[mi] = true;
        } else {
            continue;
        }
        conv.fused_out = result;
        net.tensors[mid].alias = result;
    }
    std::vector<int> order;
    for (int idx : net.order) {
        if (dropped[idx]) continue;
        const Node &nd = net.nodes[idx];
        if (nd.kind->fold_only)
            return fail(ONRT_ERR_FORMAT, "%s %s does not follow a Conv (with bias, without activation) it can be folded into, and this "
                        "runtime has no %s operator of its own", nd.kind->type, nd.base()->op_name, nd.kind->type);
        order.push_back(idx);
    }
    net.order.swap(order);
    return ONRT_OK;
}

// ---- residual blocks ------------------------------------------------------------------------------------
// Conv -> Add (-> Relu), where the convolution's result has no other reader and the other operand of the Add has the
// same shape, becomes one call of the Conv plugin's `eval_add` / `eval_add_relu`: the sum is formed in the
// convolution's store and the operands in between are never written.  The reference's optimiser does this for the
// activation after a Conv (tools/optimize/op_fusion.hpp:47-222); here it goes one operator further, at load time.
// The fused call takes the place of the Add in the order, where both of its inputs are complete.  The operands
// folded away read as the block's result.  ONENEW_RT_FUSE=0 keeps every operator separate (layer-by-layer dumps).
int fuse_residual_blocks(onrt_net &net) {
    if (!fusing_enabled() || !net.conv_add) return ONRT_OK;
    std::map<int, int> runs_instead;   // Add node -> the Conv that takes its place
    std::vector<bool> dropped(net.nodes.size(), false);
    for (int idx : net.order) {
        Node &conv = net.nodes[idx];
        if (strcmp(conv.kind->type, "Conv") || conv.out.size() != 1 || conv.in.size() > 3) continue;
        const std::string mid = conv.fused_out.empty() ? conv.out[0] : conv.fused_out;   // after a folded Relu
        const int ai = sole_reader(net, mid, "Add");
        if (ai < 0 || runs_instead.count(ai)) continue;
        Node &add = net.nodes[ai];
        if (add.in.size() != 2 || add.out.size() != 1 || add.in[0] == add.in[1]) continue;
        const std::string &other = add.in[0] == mid ? add.in[1] : add.in[0];
        const Tensor &ot = net.tensors[other], &mt = net.tensors[mid], &st = net.tensors[add.out[0]];
        if (ot.is_init || !ot.alias.empty() || memcmp(ot.desc.shapes, mt.desc.shapes, sizeof(mt.desc.shapes)) ||
            memcmp(st.desc.shapes, mt.desc.shapes, sizeof(mt.desc.shapes)))
            continue;
        conv.fuse = 1;
        conv.addend = other;
        conv.fused_out = add.out[0];
        const int ri = net.conv_add_relu ? sole_reader(net, add.out[0], "Relu") : -1;
        if (ri >= 0 && net.nodes[ri].in.size() == 1 && net.nodes[ri].out.size() == 1) {
            conv.fuse = 2;
            conv.fused_out = net.nodes[ri].out[0];
            dropped[ri] = true;
            net.tensors[add.out[0]].alias = conv.fused_out;
        }
        // everything folded away on the way reads as the block's result
        net.tensors[conv.out[0]].alias = conv.fused_out;
        net.tensors[mid].alias = conv.fused_out;
        conv.eval = conv.fuse == 2 ? net.conv_add_relu : net.conv_add;
        dropped[idx] = true;
        runs_instead[ai] = idx;
        ++net.fused_blocks;
    }
    std::vector<int> order;
    for (int idx : net.order) {
        auto it = runs_instead.find(idx);
        if (it != runs_instead.end()) order.push_back(it->second);
        else if (!dropped[idx]) order.push_back(idx);
    }
    net.order.swap(order);
    return ONRT_OK;
}

// ---- inverted-residual blocks ---------------------------------------------------------------------------
// Conv (1x1) -> Conv (depthwise) -> Conv (1x1) [-> Add, already folded into the last convolution], each result read by
// the next alone, becomes one call of the Conv plugin's `eval_block` where the plugin's `eval_block_takes` recommends it
// for the shapes (large batches of MobileNetV2's early blocks): neither wide tensor in between is written.  The call
// takes the place of the last convolution in the order.  Runs after the residual fold; ONENEW_RT_FUSE=0 keeps every
// operator separate, and a plan without plugins (no device) folds none.
void block_slots(onrt_net &net, Node &a, const Node &b, const Node &c, const Tensor &result) {
    a.params[0].addr = (int64_t) a.cfg.data();
    a.params[1].addr = (int64_t) &net.tensors[a.in[0]].desc;
    a.params[2].addr = (int64_t) &net.tensors[a.in[1]].desc;
    a.params[3].addr = (int64_t) &net.tensors[a.in[2]].desc;
    a.params[4].addr = (int64_t) &result.desc;
    a.params[5].addr = (int64_t) b.cfg.data();
    a.params[6].addr = (int64_t) &net.tensors[b.in[1]].desc;
    a.params[7].addr = (int64_t) c.cfg.data();
    a.params[8].addr = (int64_t) &net.tensors[c.in[1]].desc;
}

int fuse_ir_blocks(onrt_net &net) {
    if (!fusing_enabled() || !net.conv_block || !net.conv_block_takes) return ONRT_OK;
    auto result_of = [](const Node &n) { return n.fused_out.empty() ? n.out[0] : n.fused_out; };
    auto plain_conv = [&](const Node &n, size_t min_in) {
        if (strcmp(n.kind->type, "Conv") || n.out.size() != 1 || n.in.size() < min_in || n.in.size() > 3) return false;
        for (size_t k = 1; k < n.in.size(); ++k)
            if (n.in[k].empty() || !net.tensors[n.in[k]].is_init) return false;
        return !net.tensors[n.in[0]].is_init;
    };
    std::map<int, int> runs_instead;   // last convolution -> the first one, which takes its place
    std::vector<bool> dropped(net.nodes.size(), false);
    for (int idx : net.order) {
        Node &a = net.nodes[idx];
        // a convolution that already closes a fused block keeps that role: its result is that block's output
        if (a.fuse || dropped[idx] || runs_instead.count(idx) || !plain_conv(a, 3)) continue;
        const int bi = sole_reader(net, result_of(a), "Conv");
        if (bi < 0 || dropped[bi] || runs_instead.count(bi)) continue;
        Node &b = net.nodes[bi];
        if (b.fuse || !plain_conv(b, 3) || b.in[0] != result_of(a)) continue;
        const int ci = sole_reader(net, result_of(b), "Conv");
        if (ci < 0 || dropped[ci] || runs_instead.count(ci)) continue;
        Node &c = net.nodes[ci];
        if (c.fuse > 1 || !plain_conv(c, 2) || c.in[0] != result_of(b)) continue;
        const Tensor &result = net.tensors[result_of(c)];
        for (BUFFER_INFO_S &s : a.params) s.addr = 0;
        block_slots(net, a, b, c, result);
        const bool takes = net.conv_block_takes(a.params, a.inputs, a.outputs) == 1;
        for (BUFFER_INFO_S &s : a.params) s.addr = 0;
        if (!takes) continue;
        for (const std::string &gone : {a.out[0], result_of(a), b.out[0], result_of(b)}) {
            net.tensors[gone].never_written = true;
            net.tensors[gone].alias.clear();
        }
        a.fuse = 7;
        a.block_dw = bi;
        a.block_pw = ci;
        a.addend = c.fuse == 1 ? c.addend : std::string();
        a.fused_out = result_of(c);
        if (c.out[0] != a.fused_out) net.tensors[c.out[0]].alias = a.fused_out;
        a.eval = net.conv_block;
        dropped[idx] = dropped[bi] = true;
        runs_instead[ci] = idx;
        ++net.fused_ir_blocks;
    }
    std::vector<int> order;
    for (int idx : net.order) {
        auto it = runs_instead.find(idx);
        if (it != runs_instead.end()) order.push_back(it->second);
        else if (!dropped[idx]) order.push_back(idx);
    }
    net.order.swap(order);
    return ONRT_OK;
}

// ---- a convolution and the 1x1 convolution after it ---------------------------------------------------------
// Conv -> Conv (1x1) [-> Add [-> Relu], already folded into the second convolution], the first result read by the second
// alone, becomes one call of the Conv plugin's `eval_pair` (`eval_pair_relu`) where the plugin's `eval_pair_takes`
// recommends it for the shapes (the 3x3 and the last convolution of ResNet-50's 64-channel bottlenecks at a batch that
// fills the chip): the tensor in between is not written.  The call takes the place of the second convolution in the
// order.  Runs after the residual and the inverted-residual folds, whose convolutions it leaves alone as first ones;
// ONENEW_RT_FUSE=0 keeps every operator separate, ONENEW_RT_FUSE_PAIRS=0 these pairs alone.
void pair_slots(onrt_net &net, Node &a, const Node &b, const Tensor &result) {
    a.params[0].addr = (int64_t) a.cfg.data();
    a.params[1].addr = (int64_t) &net.tensors[a.in[0]].desc;
    a.params[2].addr = (int64_t) &net.tensors[a.in[1]].desc;
    a.params[3].addr = (int64_t) &net.tensors[a.in[2]].desc;
    a.params[4].addr = (int64_t) &result.desc;
    a.params[5].addr = (int64_t) b.cfg.data();
    a.params[6].addr = (int64_t) &net.tensors[b.in[1]].desc;
}

int fuse_conv_pairs(onrt_net &net) {
    if (!fusing_enabled() || !net.conv_pair || !net.conv_pair_relu || !net.conv_pair_takes) return ONRT_OK;
    if (const char *env = getenv("ONENEW_RT_FUSE_PAIRS"))   // "0": this fold alone switched off
        if (!strcmp(env, "0")) return ONRT_OK;
    auto result_of = [](const Node &n) { return n.fused_out.empty() ? n.out[0] : n.fused_out; };
    auto plain_conv = [&](const Node &n, size_t min_in) {
        if (strcmp(n.kind->type, "Conv") || n.out.size() != 1 || n.in.size() < min_in || n.in.size() > 3) return false;
        for (size_t k = 1; k < n.in.size(); ++k)
            if (n.in[k].empty() || !net.tensors[n.in[k]].is_init) return false;
        return !net.tensors[n.in[0]].is_init;
    };
    std::map<int, int> runs_instead;   // second convolution -> the first one, which takes its place
    std::vector<bool> dropped(net.nodes.size(), false);
    for (int idx : net.order) {
        Node &a = net.nodes[idx];
        if (a.fuse || dropped[idx] || runs_instead.count(idx) || !plain_conv(a, 3)) continue;
        const int bi = sole_reader(net, result_of(a), "Conv");
        if (bi < 0 || dropped[bi] || runs_instead.count(bi)) continue;
        Node &b = net.nodes[bi];
        if (b.fuse > 2 || !plain_conv(b, 2) || b.in[0] != result_of(a)) continue;
        // the other operand of a folded Add must not be the tensor that disappears
        if (b.fuse && (b.addend == a.out[0] || b.addend == result_of(a))) continue;
        const Tensor &result = net.tensors[result_of(b)];
        for (BUFFER_INFO_S &s : a.params) s.addr = 0;
        pair_slots(net, a, b, result);
        const bool takes = net.conv_pair_takes(a.params, a.inputs, a.outputs) == 1;
        for (BUFFER_INFO_S &s : a.params) s.addr = 0;
        if (!takes) continue;
        for (const std::string &gone : {a.out[0], result_of(a)}) {
            net.tensors[gone].never_written = true;
            net.tensors[gone].alias.clear();
        }
        a.fuse = 8;
        a.block_pw = bi;
        a.addend = b.fuse ? b.addend : std::string();
        a.fused_out = result_of(b);
        if (b.out[0] != a.fused_out) net.tensors[b.out[0]].alias = a.fused_out;
        a.eval = b.fuse == 2 ? net.conv_pair_relu : net.conv_pair;
        dropped[idx] = true;
        runs_instead[bi] = idx;
        ++net.fused_pairs;
    }
    std::vector<int> order;
    for (int idx : net.order) {
        auto it = runs_instead.find(idx);
        if (it != runs_instead.end()) order.push_back(it->second);
        else if (!dropped[idx]) order.push_back(idx);
    }
    net.order.swap(order);
    return ONRT_OK;
}

// ---- int8 edges -------------------------------------------------------------------------------------------
// The reference's W8A32 convolution takes fp32, quantises it with its input_scale (device/x86/Conv/conv.c:961-973) and
// returns fp32 (:1049-1056).  Where the result of a dense int8 Conv is read by dense int8 Convs only, all with the same
// input_scale, that quantisation moves into the producer's store: the operand travels as int8 NHWC (a quarter of the
// bytes, and no staging pass in the consumers), holding exactly the bytes each consumer would have made of the fp32
// tensor, so the model's results do not change.  The Conv plugin's `eval_link` runs both ends.  Depthwise int8
// convolutions (device/x86/Conv/conv.c:617-755) take part where the plugin's `eval_link_takes` says its NHWC kernel has
// the shape, so a quantised MobileNetV2 moves int8 from the stem to the last projection.  Not for results that an Add is
// folded into, model outputs, or operands any other operator reads.  Runs after the other folds; ONENEW_RT_FUSE=0 keeps every operand fp32 (layer-by-layer comparisons), and so
// does ONENEW_RT_LINK=0 with the other folds in place.
int link_int8_convs(onrt_net &net) {
    if (!fusing_enabled() || !net.conv_link) return ONRT_OK;
    if (const char *env = getenv("ONENEW_RT_LINK"))   // "0": the other folds without this one (measurements)
        if (!strcmp(env, "0")) return ONRT_OK;
    auto result_of = [](const Node &n) { return n.fused_out.empty() ? n.out[0] : n.fused_out; };
    // an int8 convolution `eval_link` can run: dense, or (with_depthwise) a depthwise one without a folded Add that the
    // plugin's NHWC kernel takes
    auto int8_conv = [&](const Node &n, bool with_depthwise) -> const CONV_CONFIG_S * {
        if (strcmp(n.kind->type, "Conv") || n.out.size() != 1 || n.in.size() < 2 || n.in.size() > 3 || n.fuse > 2) return nullptr;
        for (size_t k = 1; k < n.in.size(); ++k)
            if (n.in[k].empty() || !net.tensors[n.in[k]].is_init) return nullptr;
        if (net.tensors[n.in[0]].is_init) return nullptr;
        const CONV_CONFIG_S *cfg = reinterpret_cast<const CONV_CONFIG_S *>(n.cfg.data());
        if (cfg->ifmap_quant2 != TYPE_INT8) return nullptr;
        if (cfg->has_bias && cfg->group != 1) {   // conv.c:18-29: depthwise
            if (!with_depthwise || n.fuse != 0 || !net.conv_link_takes) return nullptr;
            BUFFER_INFO_S prm[BUF_MAXNUM], none[BUF_MAXNUM];
            memset(prm, 0, sizeof(prm));
            memset(none, 0, sizeof(none));
            prm[0].addr = (int64_t) n.cfg.data();
            prm[1].addr = (int64_t) &net.tensors[n.in[0]].desc;
            prm[2].addr = (int64_t) &net.tensors[n.in[1]].desc;
            if (net.conv_link_takes(prm, none, none) != 1) return nullptr;
        }
        return cfg;
    };
    auto dense_int8 = [&](const Node &n) { return int8_conv(n, false); };
    auto any_int8 = [&](const Node &n) { return int8_conv(n, true); };
    for (int idx : net.order) {
        Node &p = net.nodes[idx];
        if (!any_int8(p) || p.fuse != 0) continue;
        const std::string name = result_of(p);
        if (is_net_output(net, name) || net.tensors[name].desc.not_need_buf) continue;
        const std::vector<int> readers = readers_of(net, name);
        bool ok = !readers.empty();
        float scale = 0.0f;
        for (int ri : readers) {
            const Node &c = net.nodes[ri];
            const CONV_CONFIG_S *cc = any_int8(c);
            if (!cc || c.in[0] != name || !(cc->input_scale > 0.0f) || (scale != 0.0f && cc->input_scale != scale)) { ok = false; break; }
            scale = cc->input_scale;
        }
        for (int oi : net.order)   // nor may it be the other operand of a folded Add
            if (net.nodes[oi].addend == name) ok = false;
        if (!ok) continue;
        p.link.out_s8 = 1;
        p.link.out_scale = scale;
        p.eval = net.conv_link;
        for (int ri : readers) {
            Node &c = net.nodes[ri];
            c.link.in_s8 = 1;
            c.link_fuse = c.fuse;
            c.eval = net.conv_link;
        }
        net.tensors[name].as_s8 = true;
        ++net.int8_links;
    }
    // A MaxPool between int8 convolutions (the pooling behind a quantised stem): the quantiser is monotonic, so pooling the
    // producer's int8 result gives the bytes the consumers would make of the pooled fp32 tensor; both operands travel
    // as int8 and the MaxPool plugin's `eval_s8` runs.  Producer: a dense int8 Conv whose result only the MaxPool reads;
    // readers of the MaxPool: dense int8 Convs with one input_scale.
    for (int idx : net.order) {
        Node &p = net.nodes[idx];
        if (!net.maxpool_s8 || !dense_int8(p) || p.fuse != 0 || p.link.out_s8) continue;
        const std::string name = result_of(p);
        const int mi = sole_reader(net, name, "MaxPool");
        if (mi < 0 || net.tensors[name].desc.not_need_buf) continue;
        Node &mp = net.nodes[mi];
        if (mp.in.size() != 1 || mp.out.size() != 1 || mp.in[0] != name) continue;
        const std::string pooled = mp.out[0];
        if (is_net_output(net, pooled) || net.tensors[pooled].desc.not_need_buf) continue;
        const std::vector<int> readers = readers_of(net, pooled);
        bool ok = !readers.empty();
        float scale = 0.0f;
        for (int ri : readers) {
            const Node &c = net.nodes[ri];
            const CONV_CONFIG_S *cc = dense_int8(c);
            if (!cc || c.in[0] != pooled || !(cc->input_scale > 0.0f) || (scale != 0.0f && cc->input_scale != scale)) { ok = false; break; }
            scale = cc->input_scale;
        }
        for (int oi : net.order)
            if (net.nodes[oi].addend == pooled || net.nodes[oi].addend == name) ok = false;
        if (!ok) continue;
        p.link.out_s8 = 1;
        p.link.out_scale = scale;
        p.eval = net.conv_link;
        mp.eval = net.maxpool_s8;
        for (int ri : readers) {
            Node &c = net.nodes[ri];
            c.link.in_s8 = 1;
            c.link_fuse = c.fuse;
            c.eval = net.conv_link;
        }
        net.tensors[name].as_s8 = net.tensors[pooled].as_s8 = true;
        net.int8_links += 2;
    }
    // The result of an int8 Conv with a folded Add (the output of a residual block) stays fp32, because the next block's
    // Add reads it; the int8 Convs among its readers get an int8 copy, written by the same store (outputs[1] of
    // `eval_link`), instead of each quantising the fp32 tensor again.  Output channels in sixteens, so that the copy has
    // no padding channels.
    for (int idx : net.order) {
        Node &p = net.nodes[idx];
        const CONV_CONFIG_S *pc = dense_int8(p);
        if (!pc || (p.fuse != 1 && p.fuse != 2) || p.link.out_s8) continue;
        const std::string name = result_of(p);
        Tensor &t = net.tensors[name];
        if (t.desc.not_need_buf || t.desc.shapes[1] % 16 || !t.alias.empty()) continue;
        float scale = 0.0f;
        bool ok = true;
        std::vector<int> takers;
        for (int ri : readers_of(net, name)) {
            const Node &c = net.nodes[ri];
            const CONV_CONFIG_S *cc = any_int8(c);
            if (!cc || c.in[0] != name || c.link.in_s8) continue;            // reads the fp32 tensor
            if (!(cc->input_scale > 0.0f) || (scale != 0.0f && cc->input_scale != scale)) { ok = false; break; }
            scale = cc->input_scale;
            takers.push_back(ri);
        }
        if (!ok || takers.empty()) continue;
        p.link.twin = 1;
        p.link.out_scale = scale;
        p.link_fuse = p.fuse;
        p.eval = net.conv_link;
        t.has_twin = true;
        for (int ri : takers) {
            Node &c = net.nodes[ri];
            c.link.in_s8 = 1;
            c.link_fuse = c.fuse;
            c.reads_twin = true;
            c.eval = net.conv_link;
        }
        ++net.int8_links;
    }
    return ONRT_OK;
}

// ---- attention ------------------------------------------------------------------------------------------
// MatMul(q, Transpose(k)) -> Softmax (last axis) -> MatMul(., v), with nothing else reading the operands in between,
// becomes one call of the MatMul plugin's `eval_attention` on q, k (as it is before the Transpose) and v: the scores
// stay on the chip and the Transpose of k is never materialised.  Only for the shapes the fused kernel takes (q, k, v
// all [..., tokens, head_dim] with head_dim 32 or 64 and at most 256 tokens); every other attention block keeps its four
// operators (device/x86/MatMul/mat_mul.c, Transpose/transpose.c, Softmax/softmax.c).  The fused call takes the place of
// the second MatMul in the order, where q, k and v are all complete.  ONENEW_RT_FUSE=0 keeps every operator separate.
// Head-split and head-merge Transposes around the block fold into the call's strides (see below).
int fuse_attention(onrt_net &net) {
    if (!fusing_enabled() || !net.matmul_attention) return ONRT_OK;
    auto producer_of = [&](const std::string &name) {
        for (int idx : net.order)
            for (const std::string &o : net.nodes[idx].out)
                if (o == name) return idx;
        return -1;
    };
    std::map<int, int> runs_instead;   // second MatMul -> the first one, which takes its place
    std::vector<bool> dropped(net.nodes.size(), false);
    for (int idx : net.order) {
        Node &m1 = net.nodes[idx];
        if (strcmp(m1.kind->type, "MatMul") || m1.in.size() != 2 || m1.out.size() != 1 || m1.fuse) continue;
        // the second operand comes from a Transpose of the last two axes that nothing else reads
        const int ti = producer_of(m1.in[1]);
        if (ti < 0 || strcmp(net.nodes[ti].kind->type, "Transpose") || sole_reader(net, m1.in[1], "MatMul") != idx) continue;
        const Node &tr = net.nodes[ti];
        const TRANSPOSE_CONFIG_S *tc = reinterpret_cast<const TRANSPOSE_CONFIG_S *>(tr.cfg.data());
        const std::string &q = m1.in[0], &k = tr.in[0];
        const Tensor &qt = net.tensors[q], &kt = net.tensors[k];
        const int nd = qt.desc.dim_num_of_shapes;
        if (nd < 2 || tc->perm_num != nd || kt.desc.dim_num_of_shapes != nd || qt.is_init || kt.is_init) continue;
        bool swap_last = tc->perm[nd - 1] == nd - 2 && tc->perm[nd - 2] == nd - 1;
        for (int i = 0; i < nd - 2; ++i) swap_last = swap_last && tc->perm[i] == i;
        if (!swap_last || memcmp(qt.desc.shapes, kt.desc.shapes, nd * sizeof(qt.desc.shapes[0]))) continue;
        const int tokens = qt.desc.shapes[nd - 2], head_dim = qt.desc.shapes[nd - 1];
        if ((head_dim != 32 && head_dim != 64) || tokens > 256) continue;
        long long pairs = 1;
        for (int i = 0; i < nd - 2; ++i) pairs *= qt.desc.shapes[i];
        if (pairs > 65535) continue;
        // scores -> Softmax over the keys -> second MatMul with v
        const int si = sole_reader(net, m1.out[0], "Softmax");
        if (si < 0 || net.nodes[si].in.size() != 1 || net.nodes[si].out.size() != 1) continue;
        const SOFTMAX_CONFIG_S *sc = reinterpret_cast<const SOFTMAX_CONFIG_S *>(net.nodes[si].cfg.data());
        if (sc->axis != -1 && sc->axis != nd - 1) continue;
        const int m2i = sole_reader(net, net.nodes[si].out[0], "MatMul");
        if (m2i < 0 || runs_instead.count(m2i)) continue;
        Node &m2 = net.nodes[m2i];
        if (m2.in.size() != 2 || m2.out.size() != 1 || m2.in[0] != net.nodes[si].out[0] || m2.in[1] == m2.in[0]) continue;
        const Tensor &vt = net.tensors[m2.in[1]], &ot = net.tensors[m2.out[0]];
        if (vt.is_init || vt.desc.dim_num_of_shapes != nd || ot.desc.dim_num_of_shapes != nd ||
            memcmp(vt.desc.shapes, qt.desc.shapes, nd * sizeof(qt.desc.shapes[0])) ||
            memcmp(ot.desc.shapes, qt.desc.shapes, nd * sizeof(qt.desc.shapes[0])))
            continue;
        // A head-split Transpose (0, 2, 1, 3) in front of q, k or v that nothing else reads, and a head-merge one behind the
        // result: the call reads / writes the [batch, tokens, heads, head_dim] tensor on the other side of it through
        // strides (flags in inputs[4]), and the Transpose goes.
        auto swaps_heads = [&](int node) {
            if (node < 0 || dropped[node] || nd != 4 || strcmp(net.nodes[node].kind->type, "Transpose")) return false;
            const TRANSPOSE_CONFIG_S *c = reinterpret_cast<const TRANSPOSE_CONFIG_S *>(net.nodes[node].cfg.data());
            return c->perm_num == 4 && c->perm[0] == 0 && c->perm[1] == 2 && c->perm[2] == 1 && c->perm[3] == 3 &&
                   !net.tensors[net.nodes[node].in[0]].is_init;
        };
        std::string src[3] = {q, k, m2.in[1]}, result = m2.out[0];
        const int reader[3] = {idx, ti, m2i};
        const char *reader_type[3] = {"MatMul", "Transpose", "MatMul"};
        for (int i = 0; i < 3; ++i) {
            const int pi = producer_of(src[i]);
            if (!swaps_heads(pi) || sole_reader(net, src[i], reader_type[i]) != reader[i]) continue;
            net.tensors[src[i]].never_written = true;
            src[i] = net.nodes[pi].in[0];
            m1.token_major[i] = 1;
            dropped[pi] = true;
        }
        const int oi = sole_reader(net, result, "Transpose");
        if (swaps_heads(oi)) {
            net.tensors[result].never_written = true;
            result = net.nodes[oi].out[0];
            m1.token_major[3] = 1;
            dropped[oi] = true;
        }
        m1.fuse = 3;
        m1.in = {src[0], src[1], src[2]};
        m1.fused_out = result;
        m1.eval = net.matmul_attention;
        for (const std::string &gone : {tr.out[0], m1.out[0], net.nodes[si].out[0]}) net.tensors[gone].never_written = true;
        dropped[ti] = dropped[idx] = dropped[si] = true;
        runs_instead[m2i] = idx;
        ++net.fused_attentions;
    }
    std::vector<int> order;
    for (int idx : net.order) {
        auto it = runs_instead.find(idx);
        if (it != runs_instead.end()) order.push_back(it->second);
        else if (!dropped[idx]) order.push_back(idx);
    }
    net.order.swap(order);
    return ONRT_OK;
}

// ---- linear layers ----------------------------------------------------------------------------------------
// MatMul -> Add of an initialiser over the last axis (-> Gelu), where nothing else reads the operands in between, becomes
// one call of the MatMul plugin's `eval_bias` / `eval_bias_gelu`: bias and table activation are applied in the store of
// the product, bit-equal to the separate operators (device/x86/MatMul/mat_mul.c, Add/add.c:56-70 broadcast of the smaller
// operand along the leading axes, Gelu/gelu.c).  The reference's optimiser builds the Gelu node itself out of five
// primitives (tools/optimize/op_fusion.hpp:195-222); folding it into the MatMul goes one operator further, at load time.
// Only a bias that add.c would broadcast: rank 3 to 6 result, bias [n] (leading axes of extent 1 allowed).
// A second Add after the bias (no Gelu in between) whose other operand is an activation shaped like the result, the skip
// connection around a transformer block's projection, goes into the same call (`eval_bias_add`, the addend in
// inputs[3]); that call takes the place of the second Add in the order, where the addend is complete.
int fuse_linear(onrt_net &net) {
    if (!fusing_enabled() || !net.matmul_bias) return ONRT_OK;
    std::vector<bool> dropped(net.nodes.size(), false);
    std::map<int, int> runs_instead;   // second Add -> the MatMul that takes its place
    for (int idx : net.order) {
        Node &mm = net.nodes[idx];
        if (strcmp(mm.kind->type, "MatMul") || mm.in.size() != 2 || mm.out.size() != 1 || mm.fuse) continue;
        const int ai = sole_reader(net, mm.out[0], "Add");
        if (ai < 0) continue;
        const Node &add = net.nodes[ai];
        if (add.in.size() != 2 || add.out.size() != 1 || add.in[0] == add.in[1]) continue;
        const std::string &bias = add.in[0] == mm.out[0] ? add.in[1] : add.in[0];
        const Tensor &bt = net.tensors[bias], &yt = net.tensors[mm.out[0]], &st = net.tensors[add.out[0]];
        const int rank = yt.desc.dim_num_of_shapes, brank = bt.desc.dim_num_of_shapes;
        if (!bt.is_init || rank < 3 || rank > 6 || brank < 1 || brank > rank) continue;
        const int n = yt.desc.shapes[rank - 1];
        bool last_axis_only = bt.desc.shapes[brank - 1] == n && numel(bt.desc) == n && numel(yt.desc) > n;
        if (!last_axis_only || memcmp(st.desc.shapes, yt.desc.shapes, sizeof(yt.desc.shapes))) continue;
        mm.fuse = 4;
        mm.in.push_back(bias);
        mm.fused_out = add.out[0];
        mm.eval = net.matmul_bias;
        net.tensors[mm.out[0]].alias = mm.fused_out;
        dropped[ai] = true;
        const int gi = net.matmul_bias_gelu ? sole_reader(net, add.out[0], "Gelu") : -1;
        if (gi >= 0 && net.nodes[gi].in.size() == 1 && net.nodes[gi].out.size() == 1) {
            mm.fuse = 5;
            mm.fused_out = net.nodes[gi].out[0];
            mm.eval = net.matmul_bias_gelu;
            net.tensors[add.out[0]].alias = mm.fused_out;
            net.tensors[mm.out[0]].alias = mm.fused_out;
            dropped[gi] = true;
        }
        ++net.fused_linears;
        if (mm.fuse != 4 || !net.matmul_bias_add) continue;
        const int si = sole_reader(net, add.out[0], "Add");
        if (si < 0 || runs_instead.count(si)) continue;
        const Node &skip = net.nodes[si];
        if (skip.in.size() != 2 || skip.out.size() != 1 || skip.in[0] == skip.in[1]) continue;
        const std::string &other = skip.in[0] == add.out[0] ? skip.in[1] : skip.in[0];
        const Tensor &ot = net.tensors[other], &rt = net.tensors[skip.out[0]];
        if (ot.is_init || !ot.alias.empty() || memcmp(ot.desc.shapes, st.desc.shapes, sizeof(st.desc.shapes)) ||
            ot.desc.dim_num_of_shapes != st.desc.dim_num_of_shapes || memcmp(rt.desc.shapes, st.desc.shapes, sizeof(st.desc.shapes)))
            continue;
        mm.fuse = 6;
        mm.addend = other;
        mm.fused_out = skip.out[0];
        mm.eval = net.matmul_bias_add;
        net.tensors[add.out[0]].alias = mm.fused_out;
        net.tensors[mm.out[0]].alias = mm.fused_out;
        dropped[idx] = true;
        runs_instead[si] = idx;
        ++net.fused_skips;
    }
    std::vector<int> order;
    for (int idx : net.order) {
        auto it = runs_instead.find(idx);
        if (it != runs_instead.end()) order.push_back(it->second);
        else if (!dropped[idx]) order.push_back(idx);
    }
    net.order.swap(order);
    return ONRT_OK;
}

// ---- slot arrays (op::rt_prepare, host/op.h:109-168, and prepare_init_operand_data of each operator) ----
int fill_slots(onrt_net &net) {
    const size_t lut_len = net.silu_lut.size();
    for (int idx : net.order) {
        Node &nd = net.nodes[idx];
        if (nd.kind->view) continue;
        nd.params[0].addr = (int64_t) nd.cfg.data();
        int act_slot = 0;   // activations are packed from slot 0 in input order (host/op.h:118-147) ...
        for (size_t k = 0; k < nd.in.size(); ++k) {
            if (nd.in[k].empty()) continue;
            Tensor &t = net.tensors[nd.in[k]];
            // ... and an initialiser sits at its own input index
            const int slot = t.is_init ? (int) k : act_slot++;
            if (1 + slot >= BUF_MAXNUM - 1) return fail(ONRT_ERR_FORMAT, "%s: too many inputs", nd.base()->op_name);
            nd.params[1 + slot].addr = (int64_t) &t.desc;
            nd.inputs[slot].addr = (int64_t) t.dev;
        }
        if (nd.fuse == 3) nd.inputs[4].addr = (int64_t) nd.token_major;
        if (nd.fuse == 7) {
            const Node &b = net.nodes[nd.block_dw], &c = net.nodes[nd.block_pw];
            block_slots(net, nd, b, c, net.tensors[nd.fused_out]);
            nd.inputs[3].addr = nd.addend.empty() ? 0 : (int64_t) net.tensors[nd.addend].dev;
            nd.inputs[5].addr = (int64_t) net.tensors[b.in[1]].dev;
            nd.inputs[6].addr = (int64_t) net.tensors[b.in[2]].dev;
            nd.inputs[7].addr = (int64_t) net.tensors[c.in[1]].dev;
            nd.inputs[8].addr = c.in.size() > 2 ? (int64_t) net.tensors[c.in[2]].dev : 0;
        }
        if (nd.fuse == 8) {
            const Node &b = net.nodes[nd.block_pw];
            pair_slots(net, nd, b, net.tensors[nd.fused_out]);
            nd.inputs[3].addr = nd.addend.empty() ? 0 : (int64_t) net.tensors[nd.addend].dev;
            nd.inputs[5].addr = (int64_t) net.tensors[b.in[1]].dev;
            nd.inputs[6].addr = b.in.size() > 2 ? (int64_t) net.tensors[b.in[2]].dev : 0;
        }
        if (nd.fuse == 1 || nd.fuse == 2 || nd.fuse == 6) nd.inputs[3].addr = (int64_t) net.tensors[nd.addend].dev;
        // the other operand of a folded Add must be a tensor some operator writes (or an input): one that a later fold
        // took the buffer away from would be added as zeros, silently
        if (!nd.addend.empty() && !net.plan_only) {
            const Tensor &ad = net.tensors[nd.addend];
            if (!ad.dev || ad.never_written)
                return fail(ONRT_ERR_FORMAT, "%s: the operand %s of the Add folded into it has no buffer", nd.base()->op_name, nd.addend.c_str());
        }
        if (nd.link.in_s8 || nd.link.out_s8 || nd.link.twin) {
            nd.inputs[4].addr = (int64_t) &nd.link;
            nd.inputs[5].addr = nd.link_fuse ? (int64_t) &nd.link_fuse : 0;
            if (nd.reads_twin) nd.inputs[0].addr = (int64_t) net.tensors[nd.in[0]].twin_dev;
        }
        int out_slot = 1 + (int) nd.in.size();   // host/op.h:131-137
        for (size_t k = 0; k < nd.out.size(); ++k, ++out_slot) {
            Tensor &t = net.tensors[nd.fused_out.empty() ? nd.out[k] : nd.fused_out];
            if (out_slot >= BUF_MAXNUM - 1) return fail(ONRT_ERR_FORMAT, "%s: too many operands", nd.base()->op_name);
            nd.params[out_slot].addr = (int64_t) &t.desc;
            nd.outputs[k].addr = (int64_t) t.dev;
        }
        if (nd.link.twin) nd.outputs[1].addr = (int64_t) net.tensors[nd.fused_out.empty() ? nd.out[0] : nd.fused_out].twin_dev;
        // per-model tunables in the last params slot (host/ops/conv.h:66-69, host/ops/maxpool.h:57-62); the
        // HIP operators bring their own workspace, so the shared scratch buffer stays unallocated
        nd.params[BUF_MAXNUM - 1].addr = (int64_t) &net.useful;
        if (!strcmp(nd.kind->type, "Conv") && reinterpret_cast<const CONV_CONFIG_S *>(nd.cfg.data())->act_type == SILU)
            nd.inputs[BUF_MAXNUM - 1].addr = (int64_t) net.tables;
        if (!strcmp(nd.kind->type, "Gelu") || nd.fuse == 5) nd.inputs[BUF_MAXNUM - 1].addr = (int64_t) (static_cast<float *>(net.tables) + lut_len);
    }
    return ONRT_OK;
}

int prepare(onrt_net &net, const char *op_lib_dir) {
    if (op_lib_dir && *op_lib_dir) net.lib_dir = op_lib_dir;
    else if (const char *env = getenv("ONENEW_OP_LIB_DIR")) net.lib_dir = env;
    else net.lib_dir = own_directory();
    int rc = read_model(net);
    if (!rc) rc = order_nodes(net);
    if (!rc) rc = infer_shapes(net);
    if (!rc) rc = bind_plugins(net);
    if (!rc) rc = fold_activations_into_conv(net);
    if (!rc) rc = fuse_residual_blocks(net);
    if (!rc) rc = fuse_ir_blocks(net);
    if (!rc) rc = fuse_conv_pairs(net);
    if (!rc) rc = fuse_attention(net);
    if (!rc) rc = fuse_linear(net);
    if (!rc) rc = link_int8_convs(net);
    if (!rc) rc = allocate(net);
    if (!rc) rc = build_tables(net);
    if (!rc) rc = fill_slots(net);
    net.useful.public_buf_info.public_buf_ptr = 0;
    net.useful.public_buf_info.public_buf_size = 0;
    if (const char *env = getenv("ONENEW_RT_GRAPH")) net.graph_wanted = !strcmp(env, "1");
    if (net.stream_setters.empty() || net.graph_refused) net.graph_wanted = false;
    // a stream of the blocking kind: the synchronous copies either side of a run order themselves against it
    if (!rc && net.graph_wanted) ONRT_HIP(hipStreamCreate(&net.stream));
    return rc;
}

int plan_stub_eval(BUFFER_INFO_S *, BUFFER_INFO_S *, BUFFER_INFO_S *) { return ONRT_ERR_ARG; }

// stands in for the Conv plugin's `eval_block_takes` in a plan made with ONENEW_RT_PLAN_BLOCKS=1: every 1x1 -> depthwise ->
// 1x1 chain counts as taken, whatever its size (the plugin's own answer depends on the batch and the device)
int plan_block_takes(BUFFER_INFO_S *params, BUFFER_INFO_S *, BUFFER_INFO_S *) {
    const CONV_CONFIG_S *a = reinterpret_cast<const CONV_CONFIG_S *>(params[0].addr);
    const CONV_CONFIG_S *b = reinterpret_cast<const CONV_CONFIG_S *>(params[5].addr);
    const CONV_CONFIG_S *c = reinterpret_cast<const CONV_CONFIG_S *>(params[7].addr);
    if (!a || !b || !c) return 0;
    const bool one_by_one = a->kernel_shape[0] == 1 && a->kernel_shape[1] == 1 && c->kernel_shape[0] == 1 && c->kernel_shape[1] == 1;
    return one_by_one && a->group == 1 && c->group == 1 && b->group > 1 ? 1 : 0;
}

// the host-side part of prepare: what would run, in which order, on which shapes
int plan(onrt_net &net) {
    net.plan_only = true;
    int rc = read_model(net);
    if (!rc) rc = order_nodes(net);
    if (!rc) rc = infer_shapes(net);
    net.conv_add = net.conv_add_relu = net.matmul_attention = net.matmul_bias = net.matmul_bias_gelu = net.matmul_bias_add = plan_stub_eval;   // as with the plugins of this package
    if (!rc) rc = fold_activations_into_conv(net);
    if (!rc) rc = fuse_residual_blocks(net);
    if (const char *env = getenv("ONENEW_RT_PLAN_BLOCKS"))   // "1": the inverted-residual fold as well, on the graph's shape alone
        if (!rc && !strcmp(env, "1")) {
            net.conv_block = plan_stub_eval;
            net.conv_block_takes = plan_block_takes;
            rc = fuse_ir_blocks(net);
        }
    if (!rc) rc = fuse_attention(net);
    if (!rc) rc = fuse_linear(net);
    return rc;
}

void set_async(onrt_net &net, int on) {
    for (set_async_fn f : net.async_switches) f(on);
}

void set_stream(onrt_net &net, hipStream_t s) {
    for (set_stream_fn f : net.stream_setters) f(s);
}

// every operator once, in order, on whatever stream the plugins currently launch on
int run_operators(onrt_net &net) {
    for (int idx : net.order) {
        Node &nd = net.nodes[idx];
        if (nd.kind->view) continue;
        const int r = nd.eval(nd.params, nd.inputs, nd.outputs);
        if (r) return fail(ONRT_ERR_PLUGIN, "%s %s: eval returned %d", nd.kind->type, nd.base()->op_name, r);
    }
    return ONRT_OK;
}

// Records one inference into net.graph_exec.  Relaxed capture mode: the plugins look pointers up
// (hipPointerGetAttributes) while they queue their kernels.  Any failure leaves the net on plain launches for good.
int record_graph(onrt_net &net) {
    if (hipStreamBeginCapture(net.stream, hipStreamCaptureModeRelaxed) != hipSuccess) {
        (void) hipGetLastError();
        net.graph_failed = true;
        return ONRT_OK;
    }
    const int rc = run_operators(net);
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture(net.stream, &g);
    if (rc || e != hipSuccess || !g) {
        (void) hipGetLastError();
        if (g) (void) hipGraphDestroy(g);
        net.graph_failed = true;
        return rc;
    }
    if (hipGraphInstantiate(&net.graph_exec, g, nullptr, nullptr, 0) != hipSuccess) {
        (void) hipGetLastError();
        (void) hipGraphDestroy(g);
        net.graph_exec = nullptr;
        net.graph_failed = true;
        return ONRT_OK;
    }
    net.graph = g;
    return ONRT_OK;
}

}  // namespace

#define ONRT_API __attribute__((visibility("default")))

extern "C" {

ONRT_API const char *onrt_last_error(void) { return g_err; }

ONRT_API int onrt_net_load_buf(const void *one_buf, size_t bytes, const char *op_lib_dir, onrt_net_t **out) {
    if (!one_buf || !out) return fail(ONRT_ERR_ARG, "load: null argument");
    *out = nullptr;
    std::unique_ptr<onrt_net> net(new onrt_net);
    net->file.assign(static_cast<const char *>(one_buf), static_cast<const char *>(one_buf) + bytes);
    const int rc = prepare(*net, op_lib_dir);
    if (rc) {
        onrt_net_free(net.release());
        return rc;
    }
    *out = net.release();
    return ONRT_OK;
}

ONRT_API int onrt_net_plan_buf(const void *one_buf, size_t bytes, onrt_net_t **out) {
    if (!one_buf || !out) return fail(ONRT_ERR_ARG, "plan: null argument");
    *out = nullptr;
    std::unique_ptr<onrt_net> net(new onrt_net);
    net->file.assign(static_cast<const char *>(one_buf), static_cast<const char *>(one_buf) + bytes);
    const int rc = plan(*net);
    if (rc) return rc;
    *out = net.release();
    return ONRT_OK;
}

ONRT_API int onrt_net_load_file(const char *one_path, const char *op_lib_dir, onrt_net_t **out) {
    if (!one_path || !out) return fail(ONRT_ERR_ARG, "load: null argument");
    FILE *f = fopen(one_path, "rb");
    if (!f) return fail(ONRT_ERR_FORMAT, "can't open the one file %s", one_path);
    std::vector<char> buf;
    char chunk[1 << 16];
    size_t got;
    while ((got = fread(chunk, 1, sizeof(chunk), f)) > 0) buf.insert(buf.end(), chunk, chunk + got);
    fclose(f);
    return onrt_net_load_buf(buf.data(), buf.size(), op_lib_dir, out);
}

ONRT_API void onrt_net_free(onrt_net_t *net) {
    if (!net) return;
    if (net->plan_only) {
        delete net;
        return;
    }
    (void) hipDeviceSynchronize();
    if (net->graph_exec) (void) hipGraphExecDestroy(net->graph_exec);
    if (net->graph) (void) hipGraphDestroy(net->graph);
    if (net->stream) (void) hipStreamDestroy(net->stream);
    // the plugins key their packed copies of the weights by device address: that address is about to be free for reuse
    if (net->init_arena)
        for (forget_fn f : net->forgetters) (void) f(net->init_arena, net->init_bytes);
    if (net->tables)   // and the quantised copies of the activation tables by theirs
        for (forget_fn f : net->forgetters) (void) f(net->tables, 2 * net->silu_lut.size() * sizeof(float));
    if (net->init_arena) (void) hipFree(net->init_arena);
    if (net->act_arena) (void) hipFree(net->act_arena);
    if (net->tables) (void) hipFree(net->tables);
    // plugin libraries stay loaded: they keep process-wide state (packed weights, staging buffers)
    delete net;
}

ONRT_API int onrt_net_io_count(const onrt_net_t *net, int32_t *n_inputs, int32_t *n_outputs) {
    if (!net) return fail(ONRT_ERR_ARG, "null net");
    if (n_inputs) *n_inputs = (int32_t) net->in_names.size();
    if (n_outputs) *n_outputs = (int32_t) net->out_names.size();
    return ONRT_OK;
}

ONRT_API int onrt_net_io_info(const onrt_net_t *net, int32_t is_output, int32_t idx, const char **name, int32_t *ndim, int32_t shape[8]) {
    if (!net) return fail(ONRT_ERR_ARG, "null net");
    const std::vector<std::string> &names = is_output ? net->out_names : net->in_names;
    if (idx < 0 || idx >= (int32_t) names.size()) return fail(ONRT_ERR_ARG, "%s index %d of %zu", is_output ? "output" : "input", idx, names.size());
    if (name) *name = names[idx].c_str();
    return onrt_net_operand(net, names[idx].c_str(), ndim, shape, nullptr);
}

ONRT_API int onrt_net_op_count(const onrt_net_t *net, int32_t *n_ops) {
    if (!net || !n_ops) return fail(ONRT_ERR_ARG, "null argument");
    *n_ops = (int32_t) net->order.size();
    return ONRT_OK;
}

ONRT_API int onrt_net_fused_count(const onrt_net_t *net, int32_t *n_blocks, int32_t *n_relus) {
    if (!net) return fail(ONRT_ERR_ARG, "null argument");
    if (n_blocks) *n_blocks = (int32_t) net->fused_blocks;
    if (n_relus) *n_relus = (int32_t) net->folded_relus;
    return ONRT_OK;
}

ONRT_API int onrt_net_graph_launches(const onrt_net_t *net, int64_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "null argument");
    *n = net->graph_launches;
    return ONRT_OK;
}

ONRT_API int onrt_net_op_info(const onrt_net_t *net, int32_t idx, const char **op_type, const char **op_name) {
    if (!net) return fail(ONRT_ERR_ARG, "null net");
    if (idx < 0 || idx >= (int32_t) net->order.size()) return fail(ONRT_ERR_ARG, "operator index %d of %zu", idx, net->order.size());
    const Node &nd = net->nodes[net->order[idx]];
    if (op_type) *op_type = nd.kind->type;
    if (op_name) *op_name = nd.base()->op_name;
    return ONRT_OK;
}

ONRT_API int onrt_net_operand(const onrt_net_t *net, const char *name, int32_t *ndim, int32_t shape[8], void **dev_ptr) {
    if (!net || !name) return fail(ONRT_ERR_ARG, "null argument");
    auto it = net->tensors.find(name);
    if (it == net->tensors.end()) return fail(ONRT_ERR_ARG, "no operand named %s", name);
    if (ndim) *ndim = it->second.desc.dim_num_of_shapes;
    if (shape) memcpy(shape, it->second.desc.shapes, sizeof(int32_t) * SHAPE_LEN);
    if (dev_ptr) *dev_ptr = it->second.dev;
    return ONRT_OK;
}

// ---- the model-wide GEMM tile (tools/optimize/auto_tuning.hpp:9-75 is the reference's search for its x86 kernels) ----

// drops a recorded graph: its launches were chosen under another tile
static void forget_graph(onrt_net &net) {
    if (net.graph_exec) (void) hipGraphExecDestroy(net.graph_exec);
    if (net.graph) (void) hipGraphDestroy(net.graph);
    net.graph_exec = nullptr;
    net.graph = nullptr;
    net.graph_launches = 0;
    net.runs = 0;
}

ONRT_API int onrt_net_folded_activations(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "folded activations: null argument");
    *n = (int32_t) net->folded_acts;
    return ONRT_OK;
}

ONRT_API int onrt_net_fused_attentions(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "fused attentions: null argument");
    *n = (int32_t) net->fused_attentions;
    return ONRT_OK;
}

ONRT_API int onrt_net_fused_linears(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "fused linear layers: null argument");
    *n = (int32_t) net->fused_linears;
    return ONRT_OK;
}

ONRT_API int onrt_net_quantised_links(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "null argument");
    *n = (int32_t) net->int8_links;
    return ONRT_OK;
}

ONRT_API int onrt_net_fused_ir_blocks(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "fused inverted-residual blocks: null argument");
    *n = (int32_t) net->fused_ir_blocks;
    return ONRT_OK;
}

ONRT_API int onrt_net_fused_pairs(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "fused convolution pairs: null argument");
    *n = (int32_t) net->fused_pairs;
    return ONRT_OK;
}

ONRT_API int onrt_net_fused_skips(const onrt_net_t *net, int32_t *n) {
    if (!net || !n) return fail(ONRT_ERR_ARG, "fused skip connections: null argument");
    *n = (int32_t) net->fused_skips;
    return ONRT_OK;
}

ONRT_API int onrt_net_get_tiles(const onrt_net_t *net, int32_t tiles[3]) {
    if (!net || !tiles) return fail(ONRT_ERR_ARG, "tiles: null argument");
    const BLOCK_INFO_S &b = net->useful.block_info;
    tiles[0] = b.cuda_gemm_tile_m; tiles[1] = b.cuda_gemm_tile_n; tiles[2] = b.cuda_gemm_tile_k;
    return ONRT_OK;
}

ONRT_API int onrt_net_set_tiles(onrt_net_t *net, const int32_t tiles[3]) {
    if (!net || !tiles) return fail(ONRT_ERR_ARG, "tiles: null argument");
    BLOCK_INFO_S &b = net->useful.block_info;   // the struct every Conv call finds in its last params slot
    b.cuda_gemm_tile_m = tiles[0]; b.cuda_gemm_tile_n = tiles[1]; b.cuda_gemm_tile_k = tiles[2];
    if (!net->plan_only) {
        (void) hipDeviceSynchronize();
        forget_graph(*net);
    }
    return ONRT_OK;
}

ONRT_API int onrt_one_set_tiles(void *one_buf, size_t bytes, const int32_t tiles[3]) {
    if (!one_buf || !tiles) return fail(ONRT_ERR_ARG, "tiles: null argument");
    if (bytes < sizeof(ONE_MODEL_DESC_S)) return fail(ONRT_ERR_FORMAT, "the buffer is shorter than a .one header");
    ONE_MODEL_DESC_S *h = static_cast<ONE_MODEL_DESC_S *>(one_buf);
    if (h->one_model_magic_num != ONE_MAGIC_NUM)
        return fail(ONRT_ERR_FORMAT, "one_model_magic_num is 0x%x, a .one file starts with 0x%x", h->one_model_magic_num, ONE_MAGIC_NUM);
    BLOCK_INFO_S &b = h->useful_info.block_info;
    b.cuda_gemm_tile_m = tiles[0]; b.cuda_gemm_tile_n = tiles[1]; b.cuda_gemm_tile_k = tiles[2];
    return ONRT_OK;
}

ONRT_API int onrt_net_tune_tiles(onrt_net_t *net, int32_t reps, int32_t tiles[3], float *best_ms, float *default_ms) {
    if (!net || !tiles) return fail(ONRT_ERR_ARG, "tune: null argument");
    if (net->plan_only) return fail(ONRT_ERR_ARG, "tune: this net is a plan (onrt_net_plan_buf): load it to tune it");
    if (reps < 1) reps = 5;
    // the candidates come from the Conv plugin's library when it lists them (onhip_tile_candidate), in the process
    // already; a library without the list has nothing to choose from
    typedef int (*cand_fn)(int32_t, int32_t *, int32_t *);
    cand_fn cand = nullptr;
    auto conv = net->handles.find("Conv");   // a handle's lookup covers the libraries it depends on
    if (conv != net->handles.end()) cand = reinterpret_cast<cand_fn>(dlsym(conv->second, "onhip_tile_candidate"));
    std::vector<std::array<int32_t, 3>> options;
    options.push_back({16, 16, 16});   // the converter's default: no tile this library has, every layer by the cost model
    for (int32_t i = 0; cand; ++i) {
        int32_t bm = 0, bn = 0;
        if (cand(i, &bm, &bn) != 0) break;
        options.push_back({bm, bn, 16});   // a K tile is four 16-byte units: 16 fp32 values
    }
    std::vector<const void *> ins;
    for (const std::string &name : net->in_names) ins.push_back(net->tensors[name].dev);   // whatever the buffers hold
    std::vector<void *> outs(net->out_names.size(), nullptr);
    hipEvent_t e0, e1;
    ONRT_HIP(hipEventCreate(&e0));
    ONRT_HIP(hipEventCreate(&e1));
    const bool graph_wanted = net->graph_wanted;
    net->graph_wanted = false;
    hipStream_t keep = net->stream;
    net->stream = nullptr;            // plain launches on the default stream while measuring
    int rc = ONRT_OK;
    float best = 1e30f, deflt = 0.f;
    std::array<int32_t, 3> best_opt = options[0];
    for (const auto &o : options) {
        rc = onrt_net_set_tiles(net, o.data());
        for (int i = 0; i < 2 && !rc; ++i) rc = onrt_net_run(net, ins.data(), outs.data());   // packs weights, warms caches
        float fastest = 1e30f;
        for (int i = 0; i < reps && !rc; ++i) {
            if (hipEventRecord(e0, nullptr) != hipSuccess) { rc = fail(ONRT_ERR_RUNTIME, "hipEventRecord failed"); break; }
            rc = onrt_net_run(net, ins.data(), outs.data());
            if (rc) break;
            float ms = 0.f;
            if (hipEventRecord(e1, nullptr) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
                hipEventElapsedTime(&ms, e0, e1) != hipSuccess) { rc = fail(ONRT_ERR_RUNTIME, "event timing failed"); break; }
            fastest = ms < fastest ? ms : fastest;
        }
        if (rc) break;
        if (&o == &options[0]) deflt = fastest;
        // like the reference's search (auto_tuning.hpp:41), a candidate has to win by 2 % to replace the one before it
        if (fastest < 0.98f * best) { best = fastest; best_opt = o; }
    }
    (void) hipEventDestroy(e0);
    (void) hipEventDestroy(e1);
    net->stream = keep;
    net->graph_wanted = graph_wanted;
    if (rc) return rc;
    rc = onrt_net_set_tiles(net, best_opt.data());
    for (int k = 0; k < 3; ++k) tiles[k] = best_opt[k];
    if (best_ms) *best_ms = best;
    if (default_ms) *default_ms = deflt;
    return rc;
}

namespace {
bool on_device(const void *p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void) hipGetLastError();   // plain host memory: clear the sticky error
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}
}  // namespace

ONRT_API int onrt_net_enqueue(onrt_net_t *net, const void *const *inputs, void *const *outputs) {
    if (!net || (!inputs && !net->in_names.empty()) || (!outputs && !net->out_names.empty())) return fail(ONRT_ERR_ARG, "enqueue: null argument");
    if (net->plan_only) return fail(ONRT_ERR_ARG, "enqueue: this net is a plan (onrt_net_plan_buf): load it to run it");
    if (net->stream) return fail(ONRT_ERR_ARG, "enqueue: not for a net loaded with ONENEW_RT_GRAPH=1, whose runs go to a stream of its own");
    for (size_t i = 0; i < net->in_names.size(); ++i)
        if (!inputs[i] || !on_device(inputs[i])) return fail(ONRT_ERR_ARG, "enqueue: input %zu is not device memory", i);
    for (size_t i = 0; i < net->out_names.size(); ++i)
        if (outputs[i] && !on_device(outputs[i])) return fail(ONRT_ERR_ARG, "enqueue: output %zu is not device memory", i);
    // everything in the order of the default stream, where the plugins launch: copies in, operators, copies out
    for (size_t i = 0; i < net->in_names.size(); ++i) {
        const Tensor &t = net->tensors[net->in_names[i]];
        if (inputs[i] != t.dev) ONRT_HIP(hipMemcpyAsync(t.dev, inputs[i], t.bytes, hipMemcpyDeviceToDevice, nullptr));
    }
    set_async(*net, 1);
    const int rc = run_operators(*net);
    set_async(*net, 0);
    ++net->runs;
    if (rc) {
        (void) hipDeviceSynchronize();
        return rc;
    }
    for (size_t i = 0; i < net->out_names.size(); ++i) {
        if (!outputs[i]) continue;
        const Tensor &t = net->tensors[net->out_names[i]];
        if (outputs[i] != t.dev) ONRT_HIP(hipMemcpyAsync(outputs[i], t.dev, t.bytes, hipMemcpyDeviceToDevice, nullptr));
    }
    return ONRT_OK;
}

ONRT_API int onrt_net_run(onrt_net_t *net, const void *const *inputs, void *const *outputs) {
    if (!net || (!inputs && !net->in_names.empty()) || (!outputs && !net->out_names.empty())) return fail(ONRT_ERR_ARG, "run: null argument");
    if (net->plan_only) return fail(ONRT_ERR_ARG, "run: this net is a plan (onrt_net_plan_buf): load it to run it");
    for (size_t i = 0; i < net->in_names.size(); ++i) {
        if (!inputs[i]) return fail(ONRT_ERR_ARG, "run: input %zu is null", i);
        const Tensor &t = net->tensors[net->in_names[i]];
        if (inputs[i] != t.dev) ONRT_HIP(hipMemcpy(t.dev, inputs[i], t.bytes, hipMemcpyDefault));
    }
    set_async(*net, 1);
    set_stream(*net, net->stream);
    int rc = ONRT_OK;
    if (net->stream && !net->graph_exec && !net->graph_failed && net->runs >= 1) rc = record_graph(*net);
    if (!rc) {
        if (net->graph_exec) {
            if (hipGraphLaunch(net->graph_exec, net->stream) != hipSuccess) rc = fail(ONRT_ERR_RUNTIME, "hipGraphLaunch failed");
            else ++net->graph_launches;
        } else {
            rc = run_operators(*net);
        }
    }
    set_stream(*net, nullptr);
    set_async(*net, 0);
    ++net->runs;
    if (rc) {
        (void) hipDeviceSynchronize();
        return rc;
    }
    if (net->stream) ONRT_HIP(hipStreamSynchronize(net->stream));
    bool copied = false;
    for (size_t i = 0; i < net->out_names.size(); ++i) {
        if (!outputs[i]) continue;
        const Tensor &t = net->tensors[net->out_names[i]];
        if (outputs[i] != t.dev) {
            ONRT_HIP(hipMemcpy(outputs[i], t.dev, t.bytes, hipMemcpyDefault));
            copied = true;
        }
    }
    // a blocking copy has already waited for the operators; otherwise wait here: results are complete on return
    if (!copied) ONRT_HIP(hipStreamSynchronize(nullptr));
    return ONRT_OK;
}

// ---- model-level quantisation (tools/optimize/model_quant.hpp:625-679) ----------------------------------------------
// The reference copies the fp32 file, runs it on the calibration images collecting, for the input operand of every Conv,
// the statistics of the chosen method (abs-max and a 2048-bin histogram for KL :197-435 and MSE :437-623; the largest
// magnitudes for the percentile :83-185), turns them into a clipping threshold per operand, writes
// input_scale = threshold / 127 and ifmap_quant2 = int8 into every Conv (:657-670) and quantises every Conv's weights and
// bias in place (:31-81, :6-29).  Here the fp32 model runs on the device through the operator plugins with every
// operator separate, the statistics are taken where the operands lie (the calibration kernels of the kernel library),
// and the file image is rewritten on the host.
namespace {
typedef size_t (*calib_ws_fn)(int);
typedef int (*calib_absmax_fn)(const float *, long long, float *, void *, size_t, void *);
typedef int (*calib_hist_fn)(const float *, long long, float, float *, void *, size_t, void *);
typedef int (*calib_thr_fn)(int, const float *, long long, float, float *);
typedef int (*calib_pct_fn)(const float *, int, int, float *, void *, size_t, void *);
typedef int (*quant_wb_fn)(const float *, const float *, int32_t, int32_t, int8_t *, int32_t *, float *);
typedef const char *(*last_error_fn)(void);

struct KernelLib {
    calib_ws_fn ws = nullptr;
    calib_absmax_fn abs_max = nullptr;
    calib_hist_fn hist = nullptr;
    calib_thr_fn thr = nullptr;
    calib_pct_fn pct = nullptr;
    quant_wb_fn quant_wb = nullptr;
    last_error_fn err = nullptr;
};

int bind_kernel_lib(const std::string &dir, KernelLib *k) {
    const std::string path = dir + "/libonenew_hip.so";
    void *h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!h) return fail(ONRT_ERR_PLUGIN, "quantise: %s", dlerror());
    k->ws = reinterpret_cast<calib_ws_fn>(dlsym(h, "onhip_calib_workspace_bytes"));
    k->abs_max = reinterpret_cast<calib_absmax_fn>(dlsym(h, "onhip_calib_abs_max"));
    k->hist = reinterpret_cast<calib_hist_fn>(dlsym(h, "onhip_calib_histogram"));
    k->thr = reinterpret_cast<calib_thr_fn>(dlsym(h, "onhip_calib_threshold"));
    k->pct = reinterpret_cast<calib_pct_fn>(dlsym(h, "onhip_calib_percentile"));
    k->quant_wb = reinterpret_cast<quant_wb_fn>(dlsym(h, "onhip_quant_weight_bias"));
    k->err = reinterpret_cast<last_error_fn>(dlsym(h, "onhip_last_error"));
    if (!k->ws || !k->abs_max || !k->hist || !k->thr || !k->pct || !k->quant_wb || !k->err)
        return fail(ONRT_ERR_PLUGIN, "quantise: %s lacks the calibration entry points", path.c_str());
    return ONRT_OK;
}

// offset in the file of the data of the initialiser called `name` and its descriptor, or 0
size_t find_initialiser(const std::vector<char> &file, const char *name, OPERAND_S *desc) {
    const ONE_MODEL_DESC_S *h = reinterpret_cast<const ONE_MODEL_DESC_S *>(file.data());
    size_t off = (size_t) h->init_info_offset;
    for (int i = 0; i < h->init_cnt; ++i) {
        OPERAND_S d;
        memcpy(&d, file.data() + off, sizeof(d));
        d.operand_name[OPERAND_NAME_LEN - 1] = 0;
        if (!strcmp(d.operand_name, name)) {
            *desc = d;
            return off + sizeof(OPERAND_S);
        }
        off += align64(sizeof(OPERAND_S) + (size_t) numel(d) * elem_bytes(d.data_type));
    }
    return 0;
}
}  // namespace

ONRT_API int onrt_one_quantise(const void *one_buf, size_t bytes, const char *op_lib_dir, int32_t method,
                               const void *const *images, int32_t n_images, const void *const *images2, int32_t n_images2,
                               void *quant_one_buf) {
    if (!one_buf || !quant_one_buf || !images || n_images < 1) return fail(ONRT_ERR_ARG, "quantise: null argument or no calibration image");
    if (method != ONRT_QUANT_KL && method != ONRT_QUANT_MSE && method != ONRT_QUANT_PERCENT) return fail(ONRT_ERR_ARG, "quantise: unknown method %d", method);
    if (!images2) { images2 = images; n_images2 = n_images; }
    if (n_images2 < 1) return fail(ONRT_ERR_ARG, "quantise: no image for the second pass");
    // the fp32 model with every operator separate: each Conv's input operand is a tensor of its own in device memory
    onrt_net_t *net = nullptr;
    tl_load_unfused = true;
    int rc = onrt_net_load_buf(one_buf, bytes, op_lib_dir, &net);
    tl_load_unfused = false;
    if (rc) return rc;
    struct Guard { onrt_net_t *n; void *ws = nullptr; std::vector<void *> bufs; ~Guard() { for (void *b : bufs) (void) hipFree(b); if (ws) (void) hipFree(ws); onrt_net_free(n); } } guard{net};
    KernelLib k;
    rc = bind_kernel_lib(net->lib_dir, &k);
    if (rc) return rc;
    // the input operands of the Conv nodes, in file order, each once
    std::vector<std::string> names;
    for (const Node &nd : net->nodes) {
        if (strcmp(nd.kind->type, "Conv")) continue;
        if (reinterpret_cast<const CONV_CONFIG_S *>(nd.cfg.data())->ifmap_quant2 == TYPE_INT8)
            return fail(ONRT_ERR_ARG, "quantise: Conv %s is quantised already", nd.base()->op_name);
        if (std::find(names.begin(), names.end(), nd.in[0]) == names.end()) names.push_back(nd.in[0]);
    }
    if (names.empty()) return fail(ONRT_ERR_ARG, "quantise: the model has no Conv");
    for (const std::string &nm : names) {
        const Tensor &t = net->tensors[nm];
        if (!t.dev || numel(t.desc) < 1 || numel(t.desc) >= (1LL << 31)) return fail(ONRT_ERR_FORMAT, "quantise: operand %s has no buffer", nm.c_str());
    }
    const size_t n_in = net->in_names.size();
    std::vector<void *> outs(net->out_names.size(), nullptr);
    const size_t ws_bytes = k.ws(method == ONRT_QUANT_PERCENT ? n_images : 1);
    ONRT_HIP(hipMalloc(&guard.ws, ws_bytes ? ws_bytes : 16));
    std::map<std::string, float> threshold;
    auto lib_fail = [&](const char *what) { return fail(ONRT_ERR_RUNTIME, "quantise: %s: %s", what, k.err()); };
    if (method == ONRT_QUANT_PERCENT) {
        // one pass: every image's copy of every operand is kept, [image][element], for the selection over all of them
        std::map<std::string, float *> store;
        for (const std::string &nm : names) {
            void *b = nullptr;
            ONRT_HIP(hipMalloc(&b, (size_t) n_images * numel(net->tensors[nm].desc) * 4));
            guard.bufs.push_back(b);
            store[nm] = static_cast<float *>(b);
        }
        for (int i = 0; i < n_images; ++i) {
            rc = onrt_net_run(net, images + (size_t) i * n_in, outs.data());
            if (rc) return rc;
            for (const std::string &nm : names) {
                const size_t n = (size_t) numel(net->tensors[nm].desc);
                ONRT_HIP(hipMemcpy(store[nm] + (size_t) i * n, net->tensors[nm].dev, n * 4, hipMemcpyDeviceToDevice));
            }
        }
        for (const std::string &nm : names) {
            float thr = 0.0f;
            if (k.pct(store[nm], n_images, (int) numel(net->tensors[nm].desc), &thr, guard.ws, ws_bytes, nullptr)) return lib_fail("percentile");
            threshold[nm] = thr;
        }
    } else {
        std::map<std::string, float> max_abs;
        std::map<std::string, std::vector<float>> hist;
        for (const std::string &nm : names) { max_abs[nm] = 0.0f; hist[nm].assign(2048, 0.0f); }
        for (int i = 0; i < n_images; ++i) {          // model_quant.hpp:276-300: the largest magnitude of every operand
            rc = onrt_net_run(net, images + (size_t) i * n_in, outs.data());
            if (rc) return rc;
            for (const std::string &nm : names)
                if (k.abs_max(static_cast<const float *>(net->tensors[nm].dev), numel(net->tensors[nm].desc), &max_abs[nm], guard.ws, ws_bytes, nullptr)) return lib_fail("abs-max");
        }
        for (int i = 0; i < n_images2; ++i) {         // :302-337: the histogram of every operand over [0, that maximum]
            rc = onrt_net_run(net, images2 + (size_t) i * n_in, outs.data());
            if (rc) return rc;
            for (const std::string &nm : names)
                if (k.hist(static_cast<const float *>(net->tensors[nm].dev), numel(net->tensors[nm].desc), max_abs[nm], hist[nm].data(), guard.ws, ws_bytes, nullptr)) return lib_fail("histogram");
        }
        for (const std::string &nm : names) {
            float thr = 0.0f;
            // the reference counts "elements per image x calibrate_img_num" (:341, :583)
            if (k.thr(method == ONRT_QUANT_KL ? 0 : 1, hist[nm].data(), numel(net->tensors[nm].desc) * (long long) n_images2, max_abs[nm], &thr)) return lib_fail("threshold");
            threshold[nm] = thr;
        }
    }
    // the quantised image: the file with every Conv's scale, type and weight_aux set and its weights and bias rewritten
    std::vector<char> out(net->file);
    const ONE_MODEL_DESC_S *h = reinterpret_cast<const ONE_MODEL_DESC_S *>(out.data());
    size_t off = (size_t) h->node_cfg_offset;
    for (int i = 0; i < h->node_cnt; ++i) {
        const OpKind *kind = find_kind(out.data() + off);
        if (!kind) return fail(ONRT_ERR_FORMAT, "quantise: node %d has an unknown type", i);
        if (!strcmp(kind->type, "Conv")) {
            CONV_CONFIG_S *cfg = reinterpret_cast<CONV_CONFIG_S *>(out.data() + off);
            const std::string in0(cfg->op_base_cfg.in_operand_name[0]);
            cfg->input_scale = threshold[in0] / 127;      // model_quant.hpp:668
            cfg->ifmap_quant2 = TYPE_INT8;
            OPERAND_S wd, bd;
            const size_t w_off = find_initialiser(out, cfg->op_base_cfg.in_operand_name[1], &wd);
            if (!w_off || wd.data_type != TYPE_FP32 || wd.dim_num_of_shapes != 4) return fail(ONRT_ERR_FORMAT, "quantise: Conv %s has no fp32 weight initialiser of rank 4", cfg->op_base_cfg.op_name);
            const int cout = wd.shapes[0], inner = wd.shapes[1] * wd.shapes[2] * wd.shapes[3];
            if (cout < 1 || cout > 4096 || inner < 1) return fail(ONRT_ERR_FORMAT, "quantise: Conv %s has %d output channels (weight_aux holds 4096)", cfg->op_base_cfg.op_name, cout);
            size_t b_off = 0;
            if (cfg->has_bias) {
                b_off = find_initialiser(out, cfg->op_base_cfg.in_operand_name[2], &bd);
                if (!b_off || numel(bd) != cout) return fail(ONRT_ERR_FORMAT, "quantise: Conv %s has no bias initialiser of %d elements", cfg->op_base_cfg.op_name, cout);
            }
            std::vector<float> w((size_t) cout * inner), b(cout);
            memcpy(w.data(), out.data() + w_off, w.size() * 4);
            if (b_off) memcpy(b.data(), out.data() + b_off, b.size() * 4);
            std::vector<int8_t> w8(w.size());
            std::vector<int32_t> b32(cout);
            if (k.quant_wb(w.data(), b_off ? b.data() : nullptr, cout, inner, w8.data(), b32.data(), cfg->weight_aux)) return lib_fail("weight quantiser");
            // int8 weights at the front of the fp32-sized initialiser, int32 bias in the fp32 bias (:16-25); the bytes behind
            // the weights, which nothing reads, are cleared (the reference leaves what the in-place conversion left there)
            memset(out.data() + w_off, 0, w.size() * 4);
            memcpy(out.data() + w_off, w8.data(), w8.size());
            if (b_off) memcpy(out.data() + b_off, b32.data(), b32.size() * 4);
        }
        off += align64(kind->cfg_size);
    }
    memcpy(quant_one_buf, out.data(), out.size());
    return ONRT_OK;
}

}  // extern "C"
