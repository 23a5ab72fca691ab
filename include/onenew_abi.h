/*
 * onenew_abi.h -- binary contract between the oneNew host runtime and an operator plugin.
 *
 * A plugin is a shared object exporting one C symbol
 *
 *     int eval(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);
 *
 * The structs below are layout-identical (x86-64, LP64) to the ones the reference host fills
 * (reference: common/nn_common.h:20-26 constants, :28-62 USEFUL_INFO_S, :77-82 BUFFER_INFO_S,
 * :92-110 ELEM_TYPE_E, :129-138 ACT_TYPE_E, :146-155 OPERAND_S, :164-182 BASE_CONFIG_S,
 * :222-243 CONV_CONFIG_S, :312-320 GEMM_CONFIG_S, :366-369 MATMUL_CONFIG_S, :371-379 MAX_POOL_CONFIG_S).  Only the types the
 * Conv / MatMul / Gemm plugins read are declared.  The static assertions at the end pin every
 * size and offset a plugin depends on.
 */
#ifndef ONENEW_ABI_H
#define ONENEW_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* slot-array and string sizes */
#define BUF_MAXNUM 12        /* slots in params[] and inputs[] */
#define OPERAND_MAXNUM 8
#define SHAPE_LEN 8
#define OP_TYPE_LEN 256
#define OP_NAME_LEN 256
#define OPERAND_NAME_LEN 256
#define USEFUL_INFO_MAGIC_NUM (45678)

typedef int32_t ONENEW_BOOL;   /* the reference enum BOOL {FALSE, TRUE}: a 4-byte int */
typedef int32_t ELEM_TYPE_E;   /* 4-byte enum in the reference */
typedef int32_t ACT_TYPE_E;    /* 4-byte enum in the reference */

enum {
    TYPE_UNKNOWN = 0, TYPE_FP32 = 1, TYPE_UINT8 = 2, TYPE_INT8 = 3, TYPE_UINT16 = 4,
    TYPE_INT16 = 5, TYPE_INT32 = 6, TYPE_INT64 = 7, TYPE_FP16 = 10, TYPE_FP64 = 11,
    TYPE_BF16 = 16
};

/* activation fused into Conv by the offline optimiser */
enum {
    NOT_ACT = 0,
    RELU = 1,
    RELU6 = 2,      /* declared by the reference, never produced and never applied */
    SILU = 3,       /* 8192-entry table on [-8, 8), step 1/512 */
    CLIP = 4,       /* ReLU6 arrives as CLIP(0, 6) */
    HARDSILU = 5,
    LEAKYRELU = 6
};

/* one slot of params[] / inputs[] / outputs[]; only addr is filled for most slots */
typedef struct {
    int64_t addr;
    int32_t elem_size;
    int32_t buf_size;
} BUFFER_INFO_S;

typedef struct {
    int32_t x86_gemm_single_threads_tile_m;
    int32_t x86_gemm_single_threads_tile_n;
    int32_t x86_gemm_single_threads_tile_k;
    int32_t x86_gemm_multi_threads_tile_m;
    int32_t x86_gemm_multi_threads_tile_n;
    int32_t x86_gemm_multi_threads_tile_k;
    int32_t cuda_gemm_tile_m;
    int32_t cuda_gemm_tile_n;
    int32_t cuda_gemm_tile_k;
} BLOCK_INFO_S;

typedef struct {
    int64_t public_buf_size;   /* bytes of shared scratch the host lends to a kernel */
    int64_t public_buf_ptr;
} PUBLIC_BUF_INFO_S;

typedef struct {
    int64_t kv_cache_buf_size;
    int64_t kv_cache_buf_ptr;
    int64_t prompts_amount;
    int64_t max_token_supported;
    int64_t cur_token_index;
} KV_CACHE_INFO_S;

/* per-model tunables; Conv receives a pointer to it in params[BUF_MAXNUM - 1] */
typedef struct {
    int32_t useful_info_magic_num;
    BLOCK_INFO_S block_info;
    PUBLIC_BUF_INFO_S public_buf_info;
    KV_CACHE_INFO_S kv_cache_info;
} USEFUL_INFO_S;

/* tensor descriptor; unused trailing dims of shapes[] hold 1 */
typedef struct {
    char operand_name[OPERAND_NAME_LEN];
    ONENEW_BOOL is_fixed_val;
    ONENEW_BOOL not_need_buf;
    int64_t p_data;
    int32_t dim_num_of_shapes;
    int32_t shapes[SHAPE_LEN];
    ELEM_TYPE_E data_type;
} OPERAND_S;

typedef struct {
    char op_type[OP_TYPE_LEN];
    char op_name[OP_NAME_LEN];
} NODE_INFO_S;

/* common head of every operator config */
typedef struct {
    char op_type[OP_TYPE_LEN];
    char op_name[OP_NAME_LEN];
    char in_operand_name[OPERAND_MAXNUM][OPERAND_NAME_LEN];
    char out_operand_name[OPERAND_MAXNUM][OPERAND_NAME_LEN];
    int32_t in_operand_num;
    int32_t out_operand_num;
    NODE_INFO_S producer[OPERAND_MAXNUM];
    NODE_INFO_S consumer[OPERAND_MAXNUM];
    int32_t producer_num;
    int32_t consumer_num;
    int32_t fusion_op_type;
    int64_t fusion_op_cnt_in_entire_net;
    int64_t cur_op_cnt_in_fusion_op;
} BASE_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
    ONENEW_BOOL has_bias;
    int64_t dilations[2];       /* stored, never honoured: dilation is always 1 */
    int64_t group;              /* 1 = dense; anything else = depthwise, multiplier 1 */
    int64_t kernel_shape[2];    /* kh, kw */
    int64_t pads[4];            /* top, left, bottom, right */
    int64_t strides[4];         /* [0] vertical, [1] horizontal */
    ACT_TYPE_E act_type;
    float clip_min;
    float clip_max;
    float leaky_relu_alpha;
    float hard_sigmoid_alpha;
    float hard_sigmoid_beta;
    ELEM_TYPE_E ifmap_quant2;   /* TYPE_INT8 selects the W8A32 path */
    float input_scale;          /* activation threshold / 127 */
    float output_scale;         /* never read by the reference kernels */
    float weight_aux[4096];     /* per output channel max|w| */
} CONV_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
    ONENEW_BOOL has_bias;
    float alpha;                /* ignored: 1 */
    float beta;                 /* ignored: 1 */
    int64_t transB;             /* ignored: the weight is always [N, K] */
} GEMM_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
} MATMUL_CONFIG_S;

/* common/nn_common.h:184-187, :327-330, :481-484: operators without parameters of their own */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
} ADD_CONFIG_S;
typedef struct {
    BASE_CONFIG_S op_base_cfg;
} GLOBAL_AVGPOOL_CONFIG_S;
typedef struct {
    BASE_CONFIG_S op_base_cfg;
} RELU_CONFIG_S;

/* The activation nodes the offline optimiser folds into the Conv in front of them (tools/optimize/op_fusion.hpp:75-192):
 * common/nn_common.h:208-213 (Clip), :340-351 (HardSigmoid, LeakyRelu), :381-384 (Mul), :524-527 (Sigmoid). */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    float min;
    float max;
} CLIP_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
    float alpha;
    float beta;
} HARD_SIGMOID_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
    float alpha;
} LEAKYRELU_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
} MUL_CONFIG_S;

typedef struct {
    BASE_CONFIG_S op_base_cfg;
} SIGMOID_CONFIG_S;

/* common/nn_common.h:371-379 */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    int64_t ceil_mode;          /* not read by the kernel */
    int64_t kernel_shape[2];
    int64_t pads[4];            /* the kernel pads all four sides by pads[0] */
    int64_t strides[2];         /* [0] steps along w, [1] along h (maxpool.c:20-21,72) */
} MAX_POOL_CONFIG_S;

/* common/nn_common.h:322-325 */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
} GELU_CONFIG_S;

/* common/nn_common.h:353-359 */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    int32_t axes[8];            /* axes[0] == 1 selects the strided form */
    int32_t axes_num;
    int32_t keepdims;
} LAYERNORMALIZATION_CONFIG_S;

/* common/nn_common.h:545-550 */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    int64_t dims;
    int64_t axis;
} SOFTMAX_CONFIG_S;

/* common/nn_common.h:584-590 */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    int64_t perm[8];
    int64_t perm_num;
} TRANSPOSE_CONFIG_S;

/* common/nn_common.h:296-300: Flatten keeps the data and only changes the shape (host/ops/flatten.h:29-62) */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    int64_t axis;
} FLATTEN_CONFIG_S;

/* common/nn_common.h:486-493: Reshape, likewise a view (host/ops/reshape.h:31-70) */
typedef struct {
    BASE_CONFIG_S op_base_cfg;
    int64_t allowzero;
    int64_t dst_shape[8];
    int64_t dst_shape_num;
} RESHAPE_CONFIG_S;

/* ---- the .one model file (tools/onnx2one/onnx2one.cpp:1294-1355, host/net.h:101-196) -------------------
 * [ONE_MODEL_DESC_S][node configs][initialisers][io configs], every piece padded to 64 bytes:
 *   node config   the op's *_CONFIG_S, BASE_CONFIG_S first (op_type selects the struct)
 *   initialiser   OPERAND_S followed by the raw data (shape product * element size bytes)
 *   io config     IO_CONFIG_S, op_type "io", op_name "input" or "output"
 */
#define ONE_MAGIC_NUM (0x6F6E65)

/* common/nn_common.h:64-75 */
typedef struct {
    int32_t one_model_magic_num;
    int32_t version;
    int32_t node_cnt;
    int32_t node_cfg_offset;
    int32_t init_cnt;
    int32_t init_info_offset;
    int32_t io_cfg_cnt;
    int32_t io_cfg_offset;
    USEFUL_INFO_S useful_info;
} ONE_MODEL_DESC_S;

/* common/nn_common.h:157-162 */
typedef struct {
    char op_type[OP_TYPE_LEN];   /* "io" */
    char op_name[OP_NAME_LEN];   /* "input" or "output" */
    OPERAND_S operand;
} IO_CONFIG_S;

/* the one symbol a plugin exports */
typedef int (*onenew_eval_fn)(BUFFER_INFO_S *params, BUFFER_INFO_S *inputs, BUFFER_INFO_S *outputs);

#ifdef __cplusplus
#define ONENEW_SA(c, m) static_assert(c, m)
#else
#define ONENEW_SA(c, m) _Static_assert(c, m)
#endif
ONENEW_SA(sizeof(BUFFER_INFO_S) == 16, "BUFFER_INFO_S");
ONENEW_SA(sizeof(ONE_MODEL_DESC_S) == 32 + sizeof(USEFUL_INFO_S) && offsetof(ONE_MODEL_DESC_S, useful_info) == 32,
          "ONE_MODEL_DESC_S");
ONENEW_SA(sizeof(IO_CONFIG_S) == 512 + sizeof(OPERAND_S), "IO_CONFIG_S");
ONENEW_SA(sizeof(FLATTEN_CONFIG_S) == sizeof(BASE_CONFIG_S) + 8, "FLATTEN_CONFIG_S");
ONENEW_SA(sizeof(RESHAPE_CONFIG_S) == sizeof(BASE_CONFIG_S) + 80, "RESHAPE_CONFIG_S");
ONENEW_SA(sizeof(OPERAND_S) == 312, "OPERAND_S");
ONENEW_SA(offsetof(OPERAND_S, p_data) == 264, "OPERAND_S.p_data");
ONENEW_SA(offsetof(OPERAND_S, dim_num_of_shapes) == 272, "OPERAND_S.dim_num_of_shapes");
ONENEW_SA(offsetof(OPERAND_S, shapes) == 276, "OPERAND_S.shapes");
ONENEW_SA(offsetof(OPERAND_S, data_type) == 308, "OPERAND_S.data_type");
ONENEW_SA(sizeof(BASE_CONFIG_S) == 12840, "BASE_CONFIG_S");
ONENEW_SA(offsetof(BASE_CONFIG_S, in_operand_num) == 4608, "BASE_CONFIG_S.in_operand_num");
ONENEW_SA(sizeof(CONV_CONFIG_S) == 29376, "CONV_CONFIG_S");
ONENEW_SA(offsetof(CONV_CONFIG_S, has_bias) == 12840, "CONV.has_bias");
ONENEW_SA(offsetof(CONV_CONFIG_S, dilations) == 12848, "CONV.dilations");
ONENEW_SA(offsetof(CONV_CONFIG_S, group) == 12864, "CONV.group");
ONENEW_SA(offsetof(CONV_CONFIG_S, kernel_shape) == 12872, "CONV.kernel_shape");
ONENEW_SA(offsetof(CONV_CONFIG_S, pads) == 12888, "CONV.pads");
ONENEW_SA(offsetof(CONV_CONFIG_S, strides) == 12920, "CONV.strides");
ONENEW_SA(offsetof(CONV_CONFIG_S, act_type) == 12952, "CONV.act_type");
ONENEW_SA(offsetof(CONV_CONFIG_S, clip_min) == 12956, "CONV.clip_min");
ONENEW_SA(offsetof(CONV_CONFIG_S, ifmap_quant2) == 12976, "CONV.ifmap_quant2");
ONENEW_SA(offsetof(CONV_CONFIG_S, input_scale) == 12980, "CONV.input_scale");
ONENEW_SA(offsetof(CONV_CONFIG_S, output_scale) == 12984, "CONV.output_scale");
ONENEW_SA(offsetof(CONV_CONFIG_S, weight_aux) == 12988, "CONV.weight_aux");
ONENEW_SA(sizeof(GEMM_CONFIG_S) == 12864, "GEMM_CONFIG_S");
ONENEW_SA(offsetof(GEMM_CONFIG_S, transB) == 12856, "GEMM.transB");
ONENEW_SA(sizeof(MATMUL_CONFIG_S) == 12840, "MATMUL_CONFIG_S");
ONENEW_SA(sizeof(ADD_CONFIG_S) == 12840 && sizeof(RELU_CONFIG_S) == 12840 && sizeof(GLOBAL_AVGPOOL_CONFIG_S) == 12840,
          "parameterless configs");
ONENEW_SA(sizeof(MAX_POOL_CONFIG_S) == 12912, "MAX_POOL_CONFIG_S");
ONENEW_SA(offsetof(MAX_POOL_CONFIG_S, kernel_shape) == 12848, "MAX_POOL.kernel_shape");
ONENEW_SA(offsetof(MAX_POOL_CONFIG_S, pads) == 12864, "MAX_POOL.pads");
ONENEW_SA(offsetof(MAX_POOL_CONFIG_S, strides) == 12896, "MAX_POOL.strides");
ONENEW_SA(sizeof(GELU_CONFIG_S) == 12840, "GELU_CONFIG_S");
ONENEW_SA(sizeof(LAYERNORMALIZATION_CONFIG_S) == 12880 && offsetof(LAYERNORMALIZATION_CONFIG_S, axes) == 12840, "LAYERNORMALIZATION_CONFIG_S");
ONENEW_SA(sizeof(SOFTMAX_CONFIG_S) == 12856 && offsetof(SOFTMAX_CONFIG_S, axis) == 12848, "SOFTMAX_CONFIG_S");
ONENEW_SA(sizeof(TRANSPOSE_CONFIG_S) == 12912 && offsetof(TRANSPOSE_CONFIG_S, perm_num) == 12904, "TRANSPOSE_CONFIG_S");
ONENEW_SA(sizeof(USEFUL_INFO_S) == 96, "USEFUL_INFO_S");
ONENEW_SA(sizeof(CLIP_CONFIG_S) == 12848 && offsetof(CLIP_CONFIG_S, min) == sizeof(BASE_CONFIG_S), "CLIP_CONFIG_S");
ONENEW_SA(sizeof(HARD_SIGMOID_CONFIG_S) == 12848 && offsetof(HARD_SIGMOID_CONFIG_S, alpha) == sizeof(BASE_CONFIG_S), "HARD_SIGMOID_CONFIG_S");
ONENEW_SA(sizeof(LEAKYRELU_CONFIG_S) == 12848 && offsetof(LEAKYRELU_CONFIG_S, alpha) == 12840, "LEAKYRELU_CONFIG_S");
ONENEW_SA(sizeof(MUL_CONFIG_S) == sizeof(BASE_CONFIG_S) && sizeof(SIGMOID_CONFIG_S) == sizeof(BASE_CONFIG_S), "MUL / SIGMOID CONFIG");
ONENEW_SA(offsetof(USEFUL_INFO_S, block_info) == 4, "USEFUL.block_info");
ONENEW_SA(offsetof(USEFUL_INFO_S, public_buf_info) == 40, "USEFUL.public_buf_info");
ONENEW_SA(offsetof(USEFUL_INFO_S, kv_cache_info) == 56, "USEFUL.kv_cache_info");

#ifdef __cplusplus
}
#endif
#endif /* ONENEW_ABI_H */
