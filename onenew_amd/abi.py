"""ctypes mirror of include/onenew_abi.h and include/onenew_hip.h.

The structures are layout-identical to the ones the reference host fills
(reference: common/nn_common.h:56-62,77-82,146-155,164-182,222-243,312-320,366-369);
``check_layout`` asserts the sizes and offsets a plugin depends on.
"""
import ctypes as C

BUF_MAXNUM = 12
OPERAND_MAXNUM = 8
SHAPE_LEN = 8
NAME_LEN = 256
USEFUL_INFO_MAGIC_NUM = 45678

# ELEM_TYPE_E
TYPE_UNKNOWN, TYPE_FP32, TYPE_UINT8, TYPE_INT8 = 0, 1, 2, 3
TYPE_INT32 = 6
# ACT_TYPE_E
NOT_ACT, RELU, RELU6, SILU, CLIP, HARDSILU, LEAKYRELU = 0, 1, 2, 3, 4, 5, 6
ACT_NAMES = {NOT_ACT: "none", RELU: "relu", RELU6: "relu6", SILU: "silu", CLIP: "clip",
             HARDSILU: "hardsilu", LEAKYRELU: "leakyrelu"}
# ONHIP_COMPUTE_*
COMPUTE_F32, COMPUTE_BF16, COMPUTE_F16 = 0, 1, 2


class BUFFER_INFO_S(C.Structure):
    _fields_ = [("addr", C.c_int64), ("elem_size", C.c_int32), ("buf_size", C.c_int32)]


class BLOCK_INFO_S(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "x86_gemm_single_threads_tile_m", "x86_gemm_single_threads_tile_n", "x86_gemm_single_threads_tile_k",
        "x86_gemm_multi_threads_tile_m", "x86_gemm_multi_threads_tile_n", "x86_gemm_multi_threads_tile_k",
        "cuda_gemm_tile_m", "cuda_gemm_tile_n", "cuda_gemm_tile_k")]


class PUBLIC_BUF_INFO_S(C.Structure):
    _fields_ = [("public_buf_size", C.c_int64), ("public_buf_ptr", C.c_int64)]


class KV_CACHE_INFO_S(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("kv_cache_buf_size", "kv_cache_buf_ptr", "prompts_amount",
                                         "max_token_supported", "cur_token_index")]


class USEFUL_INFO_S(C.Structure):
    _fields_ = [("useful_info_magic_num", C.c_int32), ("block_info", BLOCK_INFO_S),
                ("public_buf_info", PUBLIC_BUF_INFO_S), ("kv_cache_info", KV_CACHE_INFO_S)]


class OPERAND_S(C.Structure):
    _fields_ = [("operand_name", C.c_char * NAME_LEN), ("is_fixed_val", C.c_int32), ("not_need_buf", C.c_int32),
                ("p_data", C.c_int64), ("dim_num_of_shapes", C.c_int32), ("shapes", C.c_int32 * SHAPE_LEN),
                ("data_type", C.c_int32)]


class NODE_INFO_S(C.Structure):
    _fields_ = [("op_type", C.c_char * NAME_LEN), ("op_name", C.c_char * NAME_LEN)]


class BASE_CONFIG_S(C.Structure):
    _fields_ = [("op_type", C.c_char * NAME_LEN), ("op_name", C.c_char * NAME_LEN),
                ("in_operand_name", (C.c_char * NAME_LEN) * OPERAND_MAXNUM),
                ("out_operand_name", (C.c_char * NAME_LEN) * OPERAND_MAXNUM),
                ("in_operand_num", C.c_int32), ("out_operand_num", C.c_int32),
                ("producer", NODE_INFO_S * OPERAND_MAXNUM), ("consumer", NODE_INFO_S * OPERAND_MAXNUM),
                ("producer_num", C.c_int32), ("consumer_num", C.c_int32), ("fusion_op_type", C.c_int32),
                ("fusion_op_cnt_in_entire_net", C.c_int64), ("cur_op_cnt_in_fusion_op", C.c_int64)]


class CONV_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("has_bias", C.c_int32), ("dilations", C.c_int64 * 2),
                ("group", C.c_int64), ("kernel_shape", C.c_int64 * 2), ("pads", C.c_int64 * 4),
                ("strides", C.c_int64 * 4), ("act_type", C.c_int32), ("clip_min", C.c_float),
                ("clip_max", C.c_float), ("leaky_relu_alpha", C.c_float), ("hard_sigmoid_alpha", C.c_float),
                ("hard_sigmoid_beta", C.c_float), ("ifmap_quant2", C.c_int32), ("input_scale", C.c_float),
                ("output_scale", C.c_float), ("weight_aux", C.c_float * 4096)]


class GEMM_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("has_bias", C.c_int32), ("alpha", C.c_float),
                ("beta", C.c_float), ("transB", C.c_int64)]


class MATMUL_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S)]


class PLAIN_CONFIG_S(C.Structure):
    """ADD_CONFIG_S, RELU_CONFIG_S, GLOBAL_AVGPOOL_CONFIG_S: the base config and nothing else"""
    _fields_ = [("op_base_cfg", BASE_CONFIG_S)]


class CLIP_CONFIG_S(C.Structure):
    """common/nn_common.h:208-213"""
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("min", C.c_float), ("max", C.c_float)]


class HARD_SIGMOID_CONFIG_S(C.Structure):
    """common/nn_common.h:340-345"""
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("alpha", C.c_float), ("beta", C.c_float)]


class LEAKYRELU_CONFIG_S(C.Structure):
    """common/nn_common.h:347-351"""
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("alpha", C.c_float)]


class MAX_POOL_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("ceil_mode", C.c_int64), ("kernel_shape", C.c_int64 * 2),
                ("pads", C.c_int64 * 4), ("strides", C.c_int64 * 2)]


class LAYERNORMALIZATION_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("axes", C.c_int32 * 8), ("axes_num", C.c_int32), ("keepdims", C.c_int32)]


class SOFTMAX_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("dims", C.c_int64), ("axis", C.c_int64)]


class TRANSPOSE_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("perm", C.c_int64 * 8), ("perm_num", C.c_int64)]


class FLATTEN_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("axis", C.c_int64)]


class RESHAPE_CONFIG_S(C.Structure):
    _fields_ = [("op_base_cfg", BASE_CONFIG_S), ("allowzero", C.c_int64), ("dst_shape", C.c_int64 * 8),
                ("dst_shape_num", C.c_int64)]


ONE_MAGIC_NUM = 0x6F6E65


class ONE_MODEL_DESC_S(C.Structure):
    """header of a .one file (common/nn_common.h:64-75)"""
    _fields_ = [("one_model_magic_num", C.c_int32), ("version", C.c_int32), ("node_cnt", C.c_int32),
                ("node_cfg_offset", C.c_int32), ("init_cnt", C.c_int32), ("init_info_offset", C.c_int32),
                ("io_cfg_cnt", C.c_int32), ("io_cfg_offset", C.c_int32), ("useful_info", USEFUL_INFO_S)]


class IO_CONFIG_S(C.Structure):
    _fields_ = [("op_type", C.c_char * NAME_LEN), ("op_name", C.c_char * NAME_LEN), ("operand", OPERAND_S)]


class TransposeDesc(C.Structure):
    """onhip_transpose_desc_t"""
    _fields_ = [("ndim", C.c_int32), ("in_shape", C.c_int32 * 6), ("perm", C.c_int32 * 6)]


class AddDesc(C.Structure):
    """onhip_add_desc_t"""
    _fields_ = [("ndim", C.c_int32), ("large_shape", C.c_int32 * 6), ("small_shape", C.c_int32 * 6),
                ("relu", C.c_int32)]


class PoolDesc(C.Structure):
    """onhip_pool_desc_t"""
    _fields_ = [("n", C.c_int32), ("c", C.c_int32), ("h", C.c_int32), ("w", C.c_int32), ("kh", C.c_int32),
                ("kw", C.c_int32), ("stride_w", C.c_int32), ("stride_h", C.c_int32), ("pad", C.c_int32)]

    def out_hw(self):
        return ((self.h + 2 * self.pad - self.kh) // self.stride_h + 1,
                (self.w + 2 * self.pad - self.kw) // self.stride_w + 1)


class ConvDesc(C.Structure):
    """onhip_conv_desc_t"""
    _fields_ = [("n", C.c_int32), ("cin", C.c_int32), ("h", C.c_int32), ("w", C.c_int32),
                ("cout", C.c_int32), ("kh", C.c_int32), ("kw", C.c_int32),
                ("stride_h", C.c_int32), ("stride_w", C.c_int32),
                ("pad_t", C.c_int32), ("pad_l", C.c_int32), ("pad_b", C.c_int32), ("pad_r", C.c_int32),
                ("group", C.c_int32), ("has_bias", C.c_int32), ("act_type", C.c_int32),
                ("clip_min", C.c_float), ("clip_max", C.c_float), ("leaky_relu_alpha", C.c_float),
                ("hard_sigmoid_alpha", C.c_float), ("hard_sigmoid_beta", C.c_float),
                ("input_scale", C.c_float), ("compute", C.c_int32), ("out_s8", C.c_int32),
                ("output_scale", C.c_float)]

    def out_hw(self):
        oh = (self.h + self.pad_t + self.pad_b - self.kh) // self.stride_h + 1
        ow = (self.w + self.pad_l + self.pad_r - self.kw) // self.stride_w + 1
        return oh, ow

    def k_per_out(self):
        return (self.cin if self.group == 1 else 1) * self.kh * self.kw

    def flops(self):
        """2 per multiply-accumulate; bias and activation not counted (host/ops/conv.h:159-176)."""
        oh, ow = self.out_hw()
        return 2 * self.n * self.cout * oh * ow * self.k_per_out()

    def algorithmic_bytes(self, eb_x=4, eb_w=4, eb_y=4):
        """every tensor touched exactly once"""
        oh, ow = self.out_hw()
        return (eb_x * self.n * self.cin * self.h * self.w + eb_w * self.cout * self.k_per_out()
                + 4 * self.cout + eb_y * self.n * self.cout * oh * ow)


class MatmulDesc(C.Structure):
    """onhip_matmul_desc_t"""
    _fields_ = [("batch", C.c_int32), ("m", C.c_int32), ("k", C.c_int32), ("n", C.c_int32),
                ("b_shared", C.c_int32), ("compute", C.c_int32)]

    def flops(self):
        return 2 * self.batch * self.m * self.n * self.k

    def algorithmic_bytes(self, eb=4, bias=False):
        nb = 1 if self.b_shared else self.batch
        return eb * (self.batch * self.m * self.k + nb * self.k * self.n + self.batch * self.m * self.n) \
            + (4 * self.n if bias else 0)


class AttentionDesc(C.Structure):
    """onhip_attention_desc_t"""
    _fields_ = [("batch", C.c_int32), ("heads", C.c_int32), ("tokens", C.c_int32), ("head_dim", C.c_int32),
                ("q_strides", C.c_longlong * 3), ("k_strides", C.c_longlong * 3), ("v_strides", C.c_longlong * 3),
                ("out_strides", C.c_longlong * 3), ("scale", C.c_float), ("compute", C.c_int32)]


def check_layout():
    assert C.sizeof(BUFFER_INFO_S) == 16
    assert C.sizeof(OPERAND_S) == 312 and OPERAND_S.shapes.offset == 276 and OPERAND_S.data_type.offset == 308
    assert C.sizeof(BASE_CONFIG_S) == 12840
    assert C.sizeof(CONV_CONFIG_S) == 29376
    assert CONV_CONFIG_S.has_bias.offset == 12840 and CONV_CONFIG_S.group.offset == 12864
    assert CONV_CONFIG_S.kernel_shape.offset == 12872 and CONV_CONFIG_S.pads.offset == 12888
    assert CONV_CONFIG_S.strides.offset == 12920 and CONV_CONFIG_S.act_type.offset == 12952
    assert CONV_CONFIG_S.ifmap_quant2.offset == 12976 and CONV_CONFIG_S.input_scale.offset == 12980
    assert CONV_CONFIG_S.weight_aux.offset == 12988
    assert C.sizeof(GEMM_CONFIG_S) == 12864 and GEMM_CONFIG_S.transB.offset == 12856
    assert C.sizeof(MATMUL_CONFIG_S) == 12840
    assert C.sizeof(MAX_POOL_CONFIG_S) == 12912 and MAX_POOL_CONFIG_S.strides.offset == 12896
    assert C.sizeof(LAYERNORMALIZATION_CONFIG_S) == 12880 and C.sizeof(SOFTMAX_CONFIG_S) == 12856
    assert C.sizeof(TRANSPOSE_CONFIG_S) == 12912 and TRANSPOSE_CONFIG_S.perm_num.offset == 12904
    assert C.sizeof(USEFUL_INFO_S) == 96 and USEFUL_INFO_S.public_buf_info.offset == 40
    assert C.sizeof(ONE_MODEL_DESC_S) == 128 and C.sizeof(IO_CONFIG_S) == 824
    assert C.sizeof(FLATTEN_CONFIG_S) == 12848 and C.sizeof(RESHAPE_CONFIG_S) == 12920
    assert C.sizeof(ConvDesc) == 25 * 4
    assert C.sizeof(MatmulDesc) == 24


check_layout()
