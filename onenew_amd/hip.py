"""Loader and thin Python front end of the gfx950 kernel library (include/onenew_hip.h).

The shared objects are built in place by ``python -m onenew_amd.build``.  Nothing here falls back to
another implementation: a missing library or a failing call raises.

Tensor arguments are torch CUDA tensors (PyTorch is used for device memory and streams only) or
raw integer device addresses; launches go to torch's current stream.
"""
import ctypes as C
import os

from . import abi
from .abi import ConvDesc, MatmulDesc, BUFFER_INFO_S

LIBDIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
_lib = None


class OnhipError(RuntimeError):
    pass


def lib_path(name="libonenew_hip.so"):
    return os.path.join(LIBDIR, name)


def plugin_path(op):
    """libConv_hip.so / libMatMul_hip.so / libGemm_hip.so"""
    return os.path.join(LIBDIR, f"lib{op}_hip.so")


EXPORTS = ["onhip_init", "onhip_last_error", "onhip_set_tuning", "onhip_split_tail_launches", "onhip_direct_lds_launches", "onhip_noalloc_scratch_launches", "onhip_last_launch_choice", "onhip_scratch_bytes", "onhip_set_tile_hint", "onhip_tile_candidate", "onhip_conv_out_shape", "onhip_conv2d_f32",
           "onhip_conv2d_packed_weight_bytes", "onhip_conv2d_pack_weights", "onhip_conv2d_f32_packed",
           "onhip_conv2d_f32_add", "onhip_conv2d_f32_noalloc", "onhip_conv_add_eval", "onhip_conv_add_relu_eval", "onhip_conv_block_eval", "onhip_conv_block_takes", "onhip_conv_pair_eval", "onhip_conv_pair_relu_eval", "onhip_conv_pair_takes", "onhip_conv_link_eval", "onhip_conv_link_takes", "onhip_conv2d_w8_link", "onhip_conv2d_w8a8_depthwise_supported",
           "onhip_conv2d_w8a32_workspace", "onhip_conv2d_w8a32", "onhip_conv2d_w8a32_packed_weight_bytes",
           "onhip_conv2d_w8a32_pack_weights", "onhip_conv2d_w8a32_packed", "onhip_quantize_nhwc_s8",
           "onhip_conv2d_w8a8_nhwc", "onhip_quant_weight_bias",
           "onhip_calib_workspace_bytes", "onhip_calib_abs_max", "onhip_calib_histogram", "onhip_calib_threshold", "onhip_calib_percentile",
           "onhip_matmul", "onhip_matmul_add", "onhip_gemm_f32", "onhip_copy_f32",
           "onhip_h16_pitch", "onhip_h16_packed_weight_bytes", "onhip_h16_pack_conv_weights", "onhip_h16_pack_matmul_weights",
           "onhip_h16_from_nchw_f32", "onhip_h16_to_nchw_f32", "onhip_h16_from_rows_f32", "onhip_h16_to_rows_f32",
           "onhip_conv2d_h16", "onhip_h16_first_width", "onhip_h16_first_channels", "onhip_h16_first_input_bytes", "onhip_h16_first_weight_bytes", "onhip_h16_first_from_nchw_f32", "onhip_h16_first_pack_weights", "onhip_conv2d_h16_first", "onhip_linear_h16", "onhip_attention", 
           "onhip_ir_block_supported", "onhip_ir_block_packed_weight_bytes", "onhip_ir_block_pack_weights", "onhip_ir_block_f32",
           "onhip_conv2d_pw_supported", "onhip_conv2d_pw_packed_weight_bytes", "onhip_conv2d_pw_pack_weights", "onhip_conv2d_pw_f32",
           "onhip_add_f32", "onhip_relu_f32", "onhip_maxpool_out_shape", "onhip_maxpool_f32", "onhip_maxpool_s8_nhwc", "onhip_maxpool_s8_eval", "onhip_global_avgpool_f32",
           "onhip_gelu_lut_f32", "onhip_layernorm_f32", "onhip_softmax_f32", "onhip_transpose_f32",
           "onhip_conv_eval", "onhip_matmul_eval", "onhip_matmul_attention_eval", "onhip_matmul_bias_eval", "onhip_matmul_bias_gelu_eval", "onhip_matmul_bias_add_eval", "onhip_gemm_eval", "onhip_add_eval", "onhip_relu_eval",
           "onhip_maxpool_eval", "onhip_global_avgpool_eval", "onhip_gelu_eval", "onhip_layernorm_eval",
           "onhip_softmax_eval", "onhip_transpose_eval", "onhip_plugin_set_async", "onhip_plugin_set_stream", "onhip_plugin_forget", "onhip_plugin_trust_weights", "onhip_plugin_release"]


def load():
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise OnhipError(f"{path} is missing: build it with `python -m onenew_amd.build`")
    L = C.CDLL(path, mode=C.RTLD_GLOBAL)
    L.onhip_split_tail_launches.restype = C.c_longlong
    L.onhip_direct_lds_launches.restype = C.c_longlong
    L.onhip_noalloc_scratch_launches.restype = C.c_longlong
    L.onhip_scratch_bytes.restype = C.c_longlong
    vp = C.c_void_p
    L.onhip_init.argtypes = [C.c_int]
    L.onhip_last_error.restype = C.c_char_p
    L.onhip_conv_out_shape.argtypes = [C.POINTER(ConvDesc), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    L.onhip_conv2d_f32.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, vp]
    L.onhip_conv2d_packed_weight_bytes.argtypes = [C.POINTER(ConvDesc)]
    L.onhip_conv2d_packed_weight_bytes.restype = C.c_size_t
    L.onhip_conv2d_pack_weights.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    L.onhip_conv2d_f32_packed.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, vp]
    L.onhip_conv2d_f32_add.argtypes = [C.POINTER(ConvDesc), vp, vp, C.c_int32, vp, vp, vp, C.c_int32, vp, vp]
    L.onhip_conv2d_f32_noalloc.argtypes = [C.POINTER(ConvDesc), vp, vp, C.c_int32, vp, vp, vp, vp]
    L.onhip_conv2d_w8a32_workspace.argtypes = [C.POINTER(ConvDesc)]
    L.onhip_conv2d_w8a32_workspace.restype = C.c_size_t
    L.onhip_conv2d_w8a32.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, vp, vp, vp, C.c_size_t, vp]
    L.onhip_conv2d_w8a32_packed_weight_bytes.argtypes = [C.POINTER(ConvDesc)]
    L.onhip_conv2d_w8a32_packed_weight_bytes.restype = C.c_size_t
    L.onhip_conv2d_w8a32_pack_weights.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    L.onhip_conv2d_w8a32_packed.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, vp, vp, vp, C.c_size_t, vp]
    L.onhip_add_f32.argtypes = [vp, vp, vp, vp, vp]
    L.onhip_relu_f32.argtypes = [vp, vp, C.c_longlong, vp]
    L.onhip_maxpool_f32.argtypes = [vp, C.c_int32, C.c_int32, vp, vp, vp]
    L.onhip_maxpool_s8_nhwc.argtypes = [vp, C.c_int32, C.c_int32, vp, vp, vp]
    L.onhip_global_avgpool_f32.argtypes = [C.c_int32] * 4 + [vp, vp, vp]
    L.onhip_gelu_lut_f32.argtypes = [vp, vp, vp, C.c_longlong, vp]
    L.onhip_layernorm_f32.argtypes = [C.c_int32, C.c_int32, C.c_int32, vp, vp, vp, vp, vp]
    L.onhip_softmax_f32.argtypes = [C.c_int32, C.c_int32, C.c_int32, vp, vp, vp]
    L.onhip_transpose_f32.argtypes = [vp, vp, vp, vp]
    L.onhip_quant_weight_bias.argtypes = [vp, vp, C.c_int32, C.c_int32, vp, vp, vp]
    L.onhip_calib_workspace_bytes.argtypes = [C.c_int]
    L.onhip_calib_workspace_bytes.restype = C.c_size_t
    L.onhip_calib_abs_max.argtypes = [vp, C.c_longlong, C.POINTER(C.c_float), vp, C.c_size_t, vp]
    L.onhip_calib_histogram.argtypes = [vp, C.c_longlong, C.c_float, vp, vp, C.c_size_t, vp]
    L.onhip_calib_threshold.argtypes = [C.c_int, vp, C.c_longlong, C.c_float, C.POINTER(C.c_float)]
    L.onhip_calib_percentile.argtypes = [vp, C.c_int, C.c_int, C.POINTER(C.c_float), vp, C.c_size_t, vp]
    L.onhip_quantize_nhwc_s8.argtypes = [vp, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_float, vp, vp]
    L.onhip_conv2d_w8a8_nhwc.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, vp, vp]
    L.onhip_conv2d_w8_link.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, vp, vp, C.c_int32, vp, vp, vp, C.c_size_t, vp]
    L.onhip_matmul.argtypes = [C.POINTER(MatmulDesc), vp, vp, vp, vp, vp, vp]
    L.onhip_matmul_add.argtypes = [C.POINTER(MatmulDesc), vp, vp, vp, vp, vp, vp]
    L.onhip_gemm_f32.argtypes = [C.c_int32, C.c_int32, C.c_int32, vp, vp, vp, vp, vp]
    L.onhip_copy_f32.argtypes = [vp, vp, C.c_longlong, vp]
    L.onhip_plugin_forget.argtypes = [vp, C.c_size_t]
    i32 = C.c_int32
    L.onhip_h16_pitch.argtypes = [i32]
    L.onhip_h16_packed_weight_bytes.argtypes = [i32, i32, i32]
    L.onhip_h16_packed_weight_bytes.restype = C.c_size_t
    L.onhip_h16_pack_conv_weights.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    L.onhip_h16_pack_matmul_weights.argtypes = [vp, i32, i32, i32, vp, vp]
    L.onhip_h16_from_nchw_f32.argtypes = [vp, i32, i32, i32, i32, i32, vp, vp]
    L.onhip_h16_to_nchw_f32.argtypes = [vp, i32, i32, i32, i32, i32, vp, vp]
    L.onhip_h16_from_rows_f32.argtypes = [vp, C.c_longlong, i32, i32, vp, vp]
    L.onhip_h16_to_rows_f32.argtypes = [vp, C.c_longlong, i32, i32, vp, vp]
    L.onhip_conv2d_h16.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, i32, vp, i32, vp]
    L.onhip_h16_first_width.argtypes = [C.POINTER(ConvDesc)]
    L.onhip_h16_first_width.restype = i32
    L.onhip_h16_first_channels.argtypes = [C.POINTER(ConvDesc)]
    L.onhip_h16_first_channels.restype = i32
    for f in (L.onhip_h16_first_input_bytes, L.onhip_h16_first_weight_bytes):
        f.argtypes = [C.POINTER(ConvDesc)]
        f.restype = C.c_size_t
    L.onhip_h16_first_from_nchw_f32.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    L.onhip_h16_first_pack_weights.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    L.onhip_conv2d_h16_first.argtypes = [C.POINTER(ConvDesc), vp, vp, vp, vp, vp, i32, vp]
    L.onhip_attention.argtypes = [C.POINTER(abi.AttentionDesc), vp, vp, vp, vp, vp]
    L.onhip_ir_block_supported.argtypes = [C.POINTER(ConvDesc)] * 3
    L.onhip_ir_block_packed_weight_bytes.argtypes = [i32, i32, i32]
    L.onhip_ir_block_packed_weight_bytes.restype = C.c_size_t
    L.onhip_ir_block_pack_weights.argtypes = [vp, vp, i32, i32, i32, vp, vp]
    L.onhip_ir_block_f32.argtypes = [C.POINTER(ConvDesc)] * 3 + [vp] * 9
    L.onhip_conv2d_pw_supported.argtypes = [C.POINTER(ConvDesc)] * 2
    L.onhip_conv2d_pw_packed_weight_bytes.argtypes = [C.POINTER(ConvDesc)]
    L.onhip_conv2d_pw_packed_weight_bytes.restype = C.c_size_t
    L.onhip_conv2d_pw_pack_weights.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    L.onhip_conv2d_pw_f32.argtypes = [C.POINTER(ConvDesc)] * 2 + [vp] * 6 + [i32, vp, vp]
    L.onhip_linear_h16.argtypes = [C.c_longlong, i32, i32, i32, vp, vp, vp, vp, vp, vp, i32, vp]
    for name in ("onhip_conv_eval", "onhip_matmul_eval", "onhip_matmul_attention_eval", "onhip_matmul_bias_eval", "onhip_matmul_bias_gelu_eval", "onhip_matmul_bias_add_eval", "onhip_gemm_eval"):
        getattr(L, name).argtypes = [C.POINTER(BUFFER_INFO_S)] * 3
    _lib = L
    return L


def forget(t):
    """tell the library that the device tensor t (weights or an activation table it may hold copies of) is about to be
    freed or rewritten"""
    _check(load().onhip_plugin_forget(_ptr(t), t.numel() * t.element_size()), "onhip_plugin_forget")


def _check(rc, what):
    if rc != 0:
        raise OnhipError(f"{what} failed ({rc}): {load().onhip_last_error().decode()}")


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def init(device=0):
    _check(load().onhip_init(device), "onhip_init")


def set_tuning(mode):
    """0: cost model; 1: time tile / split-K candidates on first use of each problem shape"""
    return load().onhip_set_tuning(int(mode))


def conv2d_f32(d, x, w, bias=None, silu_lut=None, out=None, packed=False):
    """fused Conv2d (+bias, +activation); returns the fp32 NCHW output tensor.  packed=True: `w` is
    the result of pack_conv_weights"""
    import torch
    oh, ow = d.out_hw()
    if out is None:
        out = torch.empty((d.n, d.cout, oh, ow), dtype=torch.float32, device=x.device)
    fn = load().onhip_conv2d_f32_packed if packed else load().onhip_conv2d_f32
    _check(fn(C.byref(d), _ptr(x), _ptr(w), _ptr(bias), _ptr(silu_lut), _ptr(out), _stream()), "onhip_conv2d_f32")
    return out


def conv2d_f32_noalloc(d, x, w, out, bias=None, silu_lut=None, packed=False):
    """conv2d_f32 through the entry point that allocates nothing: the caller brings the output tensor, split-K partial
    sums go to the array built into the library"""
    _check(load().onhip_conv2d_f32_noalloc(C.byref(d), _ptr(x), _ptr(w), int(bool(packed)), _ptr(bias), _ptr(silu_lut),
                                           _ptr(out), _stream()), "onhip_conv2d_f32_noalloc")
    return out


def conv2d_f32_add(d, x, w, addend, bias=None, silu_lut=None, relu=False, out=None, packed=False):
    """conv2d_f32 with `addend` (a tensor of the output's shape) added in the convolution's store, then ReLU if asked:
    the last convolution of a residual block with the Add and the Relu after it"""
    import torch
    oh, ow = d.out_hw()
    if out is None:
        out = torch.empty((d.n, d.cout, oh, ow), dtype=torch.float32, device=x.device)
    _check(load().onhip_conv2d_f32_add(C.byref(d), _ptr(x), _ptr(w), int(bool(packed)), _ptr(bias), _ptr(silu_lut),
                                       _ptr(addend), int(bool(relu)), _ptr(out), _stream()), "onhip_conv2d_f32_add")
    return out


def pack_conv_weights(d, w):
    """tap-major copy of the weights for conv2d_f32(..., packed=True); None if the layer takes them as they are"""
    import torch
    nbytes = int(load().onhip_conv2d_packed_weight_bytes(C.byref(d)))
    if nbytes == 0:
        return None
    packed = torch.empty(nbytes // 4, dtype=torch.float32, device=w.device)
    _check(load().onhip_conv2d_pack_weights(C.byref(d), _ptr(w), _ptr(packed), _stream()), "onhip_conv2d_pack_weights")
    return packed


def add_f32(large, small, relu=False, out=None):
    """out = large + small (small broadcast onto large, numpy rules), optionally followed by ReLU"""
    import torch
    from onenew_amd.abi import AddDesc
    d = AddDesc()
    ls, ss = list(large.shape), list(small.shape)
    if large.numel() == small.numel() or small.numel() == 1:
        ls, ss = [large.numel()], [small.numel()]
    ss = [1] * (len(ls) - len(ss)) + ss
    d.ndim, d.relu = len(ls), int(relu)
    for i, (a, b) in enumerate(zip(ls, ss)):
        d.large_shape[i], d.small_shape[i] = a, b
    if out is None:
        out = torch.empty_like(large)
    _check(load().onhip_add_f32(C.byref(d), _ptr(large), _ptr(small), _ptr(out), _stream()), "onhip_add_f32")
    return out


def maxpool_s8_nhwc(d, xq, out=None):
    """max pooling (PoolDesc d) on int8 NHWC activations [n, h, w, c rounded up to 16]"""
    import torch
    oh, ow = d.out_hw()
    if out is None:
        out = torch.empty((d.n, oh, ow, xq.shape[3]), dtype=torch.int8, device=xq.device)
    _check(load().onhip_maxpool_s8_nhwc(C.byref(d), oh, ow, _ptr(xq), _ptr(out), _stream()), "onhip_maxpool_s8_nhwc")
    return out


def relu_f32(x, out=None):
    import torch
    if out is None:
        out = torch.empty_like(x)
    _check(load().onhip_relu_f32(_ptr(x), _ptr(out), x.numel(), _stream()), "onhip_relu_f32")
    return out


def maxpool_f32(d, x, out=None):
    import torch
    oh, ow = d.out_hw()
    if out is None:
        out = torch.empty((d.n, d.c, oh, ow), dtype=torch.float32, device=x.device)
    _check(load().onhip_maxpool_f32(C.byref(d), out.shape[2], out.shape[3], _ptr(x), _ptr(out), _stream()),
           "onhip_maxpool_f32")
    return out


def global_avgpool_f32(x, out=None):
    import torch
    n, c, h, w = x.shape
    if out is None:
        out = torch.empty((n, c, 1, 1), dtype=torch.float32, device=x.device)
    _check(load().onhip_global_avgpool_f32(n, c, h, w, _ptr(x), _ptr(out), _stream()), "onhip_global_avgpool_f32")
    return out


def gelu_lut_f32(x, lut, out=None):
    import torch
    if out is None:
        out = torch.empty_like(x)
    _check(load().onhip_gelu_lut_f32(_ptr(x), _ptr(lut), _ptr(out), x.numel(), _stream()), "onhip_gelu_lut_f32")
    return out


def layernorm_f32(x, weight, bias, axis1=False, out=None):
    """normalises the last dimension of x, or (axis1) dimension 1 of a batch-1 tensor"""
    import torch
    reduce = x.shape[1] if axis1 else next((d for d in reversed(x.shape) if d != 1), 1)
    rows = x.numel() // reduce
    if out is None:
        out = torch.empty_like(x)
    _check(load().onhip_layernorm_f32(rows, reduce, int(axis1), _ptr(x), _ptr(weight), _ptr(bias), _ptr(out), _stream()),
           "onhip_layernorm_f32")
    return out


def softmax_f32(x, axis1=False, out=None):
    import torch
    reduce = x.shape[1] if axis1 else x.shape[-1]
    rows = x.numel() // reduce
    if out is None:
        out = torch.empty_like(x)
    _check(load().onhip_softmax_f32(rows, reduce, int(axis1), _ptr(x), _ptr(out), _stream()), "onhip_softmax_f32")
    return out


def transpose_f32(x, perm, out=None):
    import torch
    from onenew_amd.abi import TransposeDesc
    d = TransposeDesc()
    d.ndim = x.dim()
    for i in range(x.dim()):
        d.in_shape[i], d.perm[i] = x.shape[i], perm[i]
    if out is None:
        out = torch.empty([x.shape[p] for p in perm], dtype=torch.float32, device=x.device)
    _check(load().onhip_transpose_f32(C.byref(d), _ptr(x), _ptr(out), _stream()), "onhip_transpose_f32")
    return out


CALIB_BINS, CALIB_KL, CALIB_MSE = 2048, 0, 1


def quant_weight_bias(w, bias=None):
    """host arrays: (w8, bias32, weight_aux) of model_quant.hpp:6-29"""
    import numpy as np
    w = np.ascontiguousarray(w, dtype=np.float32)
    cout = w.shape[0]
    per = w.size // cout
    w8 = np.empty(w.shape, np.int8)
    aux = np.empty(cout, np.float32)
    b32 = None
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
        b32 = np.empty(cout, np.int32)
    _check(load().onhip_quant_weight_bias(w.ctypes.data, bias.ctypes.data if bias is not None else None, cout, per,
                                          w8.ctypes.data, b32.ctypes.data if b32 is not None else None,
                                          aux.ctypes.data), "onhip_quant_weight_bias")
    return w8, b32, aux


_calib_ws = None


def calib_workspace(images=1):
    """device workspace of the calibration passes: allocated by the caller (here: once per process, grown on demand)"""
    import torch
    global _calib_ws
    L = load()
    need = int(L.onhip_calib_workspace_bytes(int(images)))
    if _calib_ws is None or _calib_ws.numel() < need:
        _calib_ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    return _calib_ws


def calib_abs_max(x, running=0.0):
    m = C.c_float(running)
    ws = calib_workspace()
    _check(load().onhip_calib_abs_max(_ptr(x), x.numel(), C.byref(m), _ptr(ws), ws.numel(), _stream()),
           "onhip_calib_abs_max")
    return m.value


def calib_histogram(x, max_abs, hist=None):
    """adds to (or creates) the host histogram of 2048 float counters"""
    import numpy as np
    if hist is None:
        hist = np.zeros(CALIB_BINS, np.float32)
    ws = calib_workspace()
    _check(load().onhip_calib_histogram(_ptr(x), x.numel(), max_abs, hist.ctypes.data, _ptr(ws),
                                        C.c_size_t(ws.numel()), _stream()), "onhip_calib_histogram")
    return hist


def calib_threshold(method, hist, elem_count, max_abs):
    t = C.c_float(0.0)
    _check(load().onhip_calib_threshold(method, hist.ctypes.data, elem_count, max_abs, C.byref(t)),
           "onhip_calib_threshold")
    return t.value


def calib_percentile(x, images, elems):
    t = C.c_float(0.0)
    ws = calib_workspace(images)
    _check(load().onhip_calib_percentile(_ptr(x), int(images), int(elems), C.byref(t), _ptr(ws), ws.numel(), _stream()),
           "onhip_calib_percentile")
    return t.value


def conv2d_w8a32_workspace(d):
    return int(load().onhip_conv2d_w8a32_workspace(C.byref(d)))


def pack_conv_weights_w8(d, w8):
    """the int8 weights in the kernel's layout (None for depthwise, which reads the reference layout)"""
    import torch
    nbytes = int(load().onhip_conv2d_w8a32_packed_weight_bytes(C.byref(d)))
    if nbytes == 0:
        return None
    packed = torch.empty(nbytes, dtype=torch.int8, device=w8.device)
    _check(load().onhip_conv2d_w8a32_pack_weights(C.byref(d), _ptr(w8), _ptr(packed), _stream()),
           "onhip_conv2d_w8a32_pack_weights")
    return packed


def quantize_nhwc_s8(x, scale, out=None):
    """NCHW fp32 -> NHWC int8 with channels padded to 16: the input form of conv2d_w8a8_nhwc"""
    import torch
    n, c, h, w = x.shape
    if out is None:
        out = torch.empty((n, h, w, (c + 15) // 16 * 16), dtype=torch.int8, device=x.device)
    _check(load().onhip_quantize_nhwc_s8(_ptr(x), n, c, h, w, scale, _ptr(out), _stream()), "onhip_quantize_nhwc_s8")
    return out


def conv2d_w8a8_nhwc(d, xq, w8_packed, bias32, weight_aux, silu_lut=None, out=None):
    """int8 NHWC in, int8 NHWC out (d.input_scale, d.output_scale); out[..., :cout] holds the result"""
    import torch
    oh, ow = d.out_hw()
    if out is None:
        out = torch.empty((d.n, oh, ow, (d.cout + 15) // 16 * 16), dtype=torch.int8, device=xq.device)
    _check(load().onhip_conv2d_w8a8_nhwc(C.byref(d), _ptr(xq), _ptr(w8_packed), _ptr(bias32), _ptr(weight_aux),
                                         _ptr(silu_lut), _ptr(out), _stream()), "onhip_conv2d_w8a8_nhwc")
    return out


def conv2d_w8_link(d, w8_packed, bias32, weight_aux, silu_lut=None, x=None, xq=None, addend=None, relu_after=False, out=None, twin=None):
    """one link of an int8 chain: fp32 NCHW (x) or int8 NHWC (xq) in; fp32 NCHW out, optionally with an addend (and a
    Relu) folded into the store and an int8 NHWC copy quantised with d.output_scale in `twin`, or int8 NHWC out
    (d.out_s8 = 1, d.output_scale)"""
    import torch
    oh, ow = d.out_hw()
    src = x if x is not None else xq
    if out is None:
        if d.out_s8:
            out = torch.empty((d.n, oh, ow, (d.cout + 15) // 16 * 16), dtype=torch.int8, device=src.device)
        else:
            out = torch.empty((d.n, d.cout, oh, ow), dtype=torch.float32, device=src.device)
    need = conv2d_w8a32_workspace(d)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=src.device)
    _check(load().onhip_conv2d_w8_link(C.byref(d), _ptr(x), _ptr(xq), _ptr(w8_packed), _ptr(bias32), _ptr(weight_aux), _ptr(silu_lut),
                                       _ptr(addend), int(relu_after), _ptr(out), _ptr(twin), _ptr(ws), ws.numel(), _stream()), "onhip_conv2d_w8_link")
    return out


def conv2d_w8a32(d, x, w8, bias32, weight_aux, silu_lut=None, out=None, acc32=None, workspace=None, packed=False):
    import torch
    oh, ow = d.out_hw()
    if out is None:
        out = torch.empty((d.n, d.cout, oh, ow), dtype=torch.int8 if d.out_s8 else torch.float32, device=x.device)
    need = conv2d_w8a32_workspace(d)
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    fn = load().onhip_conv2d_w8a32_packed if packed else load().onhip_conv2d_w8a32
    _check(fn(C.byref(d), _ptr(x), _ptr(w8), _ptr(bias32), _ptr(weight_aux), _ptr(silu_lut),
              _ptr(out), _ptr(acc32), _ptr(workspace), nbytes, _stream()),
           "onhip_conv2d_w8a32_packed" if packed else "onhip_conv2d_w8a32")
    return out


def matmul(a, b, bias=None, gelu_lut=None, compute=abi.COMPUTE_F32, out=None, addend=None):
    """out = a @ b (b either [K, N] or batched like a), optional fused bias over N and table GELU, or (addend given) bias
    and the Add of a tensor shaped like the result"""
    import torch
    M, K = a.shape[-2], a.shape[-1]
    N = b.shape[-1]
    batch = 1
    for s in a.shape[:-2]:
        batch *= s
    d = MatmulDesc(batch=batch, m=M, k=K, n=N, b_shared=int(b.numel() == K * N), compute=compute)
    if out is None:
        out = torch.empty(tuple(a.shape[:-1]) + (N,), dtype=torch.float32, device=a.device)
    if addend is not None:
        if gelu_lut is not None or tuple(addend.shape) != tuple(out.shape):
            raise ValueError("matmul: an addend takes the result's shape and excludes the GELU table")
        _check(load().onhip_matmul_add(C.byref(d), _ptr(a), _ptr(b), _ptr(bias), _ptr(addend), _ptr(out), _stream()),
               "onhip_matmul_add")
        return out
    _check(load().onhip_matmul(C.byref(d), _ptr(a), _ptr(b), _ptr(bias), _ptr(gelu_lut), _ptr(out), _stream()),
           "onhip_matmul")
    return out


# ---- bf16 / fp16 with 16-bit storage: tensors travel as torch.bfloat16 / torch.float16, NHWC with padded channels ----
H16_OUT_NHWC, H16_OUT_F32_NHWC, H16_OUT_F32_NCHW = 0, 1, 2


def h16_pitch(c):
    return (c + 31) // 32 * 32


def _h16_torch_dtype(compute):
    import torch
    if compute == abi.COMPUTE_BF16:
        return torch.bfloat16
    if compute == abi.COMPUTE_F16:
        return torch.float16
    raise OnhipError(f"16-bit storage: compute type {compute} is neither bf16 nor fp16")


def h16_pack_conv_weights(d, w):
    """fp32 OIHW weights -> [cout][kh*kw][pitch(cin)] in d.compute's 16-bit type"""
    import torch
    out = torch.empty((d.cout, d.kh * d.kw, h16_pitch(d.cin)), dtype=_h16_torch_dtype(d.compute), device=w.device)
    _check(load().onhip_h16_pack_conv_weights(C.byref(d), _ptr(w), _ptr(out), _stream()), "onhip_h16_pack_conv_weights")
    return out


def h16_pack_matmul_weights(b, compute):
    """the right operand [K, N] (fp32) of a MatMul -> [N][pitch(K)] 16-bit"""
    import torch
    k, n = b.shape
    out = torch.empty((n, h16_pitch(k)), dtype=_h16_torch_dtype(compute), device=b.device)
    _check(load().onhip_h16_pack_matmul_weights(_ptr(b), k, n, compute, _ptr(out), _stream()), "onhip_h16_pack_matmul_weights")
    return out


def h16_from_nchw(x, compute):
    import torch
    n, c, h, w = x.shape
    out = torch.empty((n, h, w, h16_pitch(c)), dtype=_h16_torch_dtype(compute), device=x.device)
    _check(load().onhip_h16_from_nchw_f32(_ptr(x), n, c, h, w, compute, _ptr(out), _stream()), "onhip_h16_from_nchw_f32")
    return out


def h16_to_nchw(x, c, compute):
    import torch
    n, h, w, cp = x.shape
    assert cp == h16_pitch(c)
    out = torch.empty((n, c, h, w), dtype=torch.float32, device=x.device)
    _check(load().onhip_h16_to_nchw_f32(_ptr(x), n, c, h, w, compute, _ptr(out), _stream()), "onhip_h16_to_nchw_f32")
    return out


def h16_from_rows(x, compute):
    import torch
    rows, k = x.shape
    out = torch.empty((rows, h16_pitch(k)), dtype=_h16_torch_dtype(compute), device=x.device)
    _check(load().onhip_h16_from_rows_f32(_ptr(x), rows, k, compute, _ptr(out), _stream()), "onhip_h16_from_rows_f32")
    return out


def h16_to_rows(x, k, compute):
    import torch
    rows = x.shape[0]
    out = torch.empty((rows, k), dtype=torch.float32, device=x.device)
    _check(load().onhip_h16_to_rows_f32(_ptr(x), rows, k, compute, _ptr(out), _stream()), "onhip_h16_to_rows_f32")
    return out


def conv2d_h16(d, x, w_packed, bias=None, lut=None, residual=None, residual_relu=False, y_kind=H16_OUT_NHWC, out=None):
    """x: 16-bit NHWC [n][h][w][pitch(cin)]; result by y_kind: 16-bit NHWC, fp32 NHWC [n][oh][ow][cout] or fp32 NCHW"""
    import torch
    oh, ow = d.out_hw()
    if out is None:
        if y_kind == H16_OUT_NHWC:
            out = torch.empty((d.n, oh, ow, h16_pitch(d.cout)), dtype=x.dtype, device=x.device)
        elif y_kind == H16_OUT_F32_NHWC:
            out = torch.empty((d.n, oh, ow, d.cout), dtype=torch.float32, device=x.device)
        else:
            out = torch.empty((d.n, d.cout, oh, ow), dtype=torch.float32, device=x.device)
    _check(load().onhip_conv2d_h16(C.byref(d), _ptr(x), _ptr(w_packed), _ptr(bias), _ptr(lut), _ptr(residual),
                                   int(residual_relu), _ptr(out), y_kind, _stream()), "onhip_conv2d_h16")
    return out


def h16_first_from_nchw(d, x):
    """fp32 NCHW image of a first layer -> its 16-bit storage form [n][h][wp][4 or 8]"""
    import torch
    lib = load()
    wp = lib.onhip_h16_first_width(C.byref(d))
    if wp < 1:
        raise OnhipError("16-bit first layer: " + load().onhip_last_error().decode())
    out = torch.empty((d.n, d.h, wp, lib.onhip_h16_first_channels(C.byref(d))), dtype=_h16_torch_dtype(d.compute), device=x.device)
    _check(lib.onhip_h16_first_from_nchw_f32(C.byref(d), _ptr(x), _ptr(out), _stream()), "onhip_h16_first_from_nchw_f32")
    return out


def h16_first_pack_weights(d, w):
    """fp32 OIHW weights of a first layer -> [cout][kh][8][4 or 8] 16-bit"""
    import torch
    out = torch.empty((d.cout, d.kh, 8, load().onhip_h16_first_channels(C.byref(d))), dtype=_h16_torch_dtype(d.compute), device=w.device)
    _check(load().onhip_h16_first_pack_weights(C.byref(d), _ptr(w), _ptr(out), _stream()), "onhip_h16_first_pack_weights")
    return out


def conv2d_h16_first(d, x_first, w_packed, bias=None, lut=None, y_kind=H16_OUT_NHWC, out=None):
    """conv2d_h16 on the first-layer storage form (h16_first_from_nchw, h16_first_pack_weights)"""
    import torch
    oh, ow = d.out_hw()
    if out is None:
        if y_kind == H16_OUT_NHWC:
            out = torch.empty((d.n, oh, ow, h16_pitch(d.cout)), dtype=x_first.dtype, device=x_first.device)
        elif y_kind == H16_OUT_F32_NHWC:
            out = torch.empty((d.n, oh, ow, d.cout), dtype=torch.float32, device=x_first.device)
        else:
            out = torch.empty((d.n, d.cout, oh, ow), dtype=torch.float32, device=x_first.device)
    _check(load().onhip_conv2d_h16_first(C.byref(d), _ptr(x_first), _ptr(w_packed), _ptr(bias), _ptr(lut), _ptr(out), y_kind,
                                         _stream()), "onhip_conv2d_h16_first")
    return out


def linear_h16(x, w_packed, k, n, compute, bias=None, gelu_lut=None, residual=None, y_kind=H16_OUT_NHWC, out=None):
    """x: 16-bit rows [rows][pitch(k)], w_packed from h16_pack_matmul_weights; y = x @ b (+ bias) (GELU table)"""
    import torch
    rows = x.shape[0]
    if out is None:
        if y_kind == H16_OUT_NHWC:
            out = torch.empty((rows, h16_pitch(n)), dtype=x.dtype, device=x.device)
        else:
            out = torch.empty((rows, n), dtype=torch.float32, device=x.device)
    _check(load().onhip_linear_h16(rows, k, n, compute, _ptr(x), _ptr(w_packed), _ptr(bias), _ptr(gelu_lut), _ptr(residual),
                                   _ptr(out), y_kind, _stream()), "onhip_linear_h16")
    return out


def ir_block_supported(ex, dw, pw):
    return load().onhip_ir_block_supported(C.byref(ex), C.byref(dw), C.byref(pw))


def ir_block_pack_weights(expand_w, project_w):
    """the two 1x1 weight tensors of an inverted-residual block, [ce, cin(, 1, 1)] and [cout, ce(, 1, 1)] -> the layout of
    the one-launch block kernel"""
    import torch
    ce, cin, co = expand_w.shape[0], expand_w.shape[1], project_w.shape[0]
    out = torch.empty(load().onhip_ir_block_packed_weight_bytes(cin, ce, co) // 4, dtype=torch.float32, device=expand_w.device)
    _check(load().onhip_ir_block_pack_weights(_ptr(expand_w), _ptr(project_w), cin, ce, co, _ptr(out), _stream()),
           "onhip_ir_block_pack_weights")
    return out


def ir_block_f32(ex, dw, pw, x, packed, expand_b, dw_w, dw_b, project_b=None, residual=None, out=None):
    """1x1 expansion -> depthwise 3x3 -> 1x1 projection [-> Add of residual] in one launch"""
    import torch
    oh, ow = dw.out_hw()
    if out is None:
        out = torch.empty((dw.n, pw.cout, oh, ow), dtype=torch.float32, device=x.device)
    _check(load().onhip_ir_block_f32(C.byref(ex), C.byref(dw), C.byref(pw), _ptr(x), _ptr(packed), _ptr(expand_b), _ptr(dw_w), _ptr(dw_b),
                                     _ptr(project_b), _ptr(residual), _ptr(out), _stream()), "onhip_ir_block_f32")
    return out


def conv2d_pw_supported(a, b):
    """0: the pair is not taken; 1: taken; 2: taken and expected to beat the two launches"""
    return load().onhip_conv2d_pw_supported(C.byref(a), C.byref(b))


def conv2d_pw_pack_weights(b, wb):
    """the 1x1 convolution's weights in the order conv2d_pw_f32 reads them"""
    import torch
    out = torch.empty(load().onhip_conv2d_pw_packed_weight_bytes(C.byref(b)) // 4, dtype=torch.float32, device=wb.device)
    _check(load().onhip_conv2d_pw_pack_weights(C.byref(b), _ptr(wb), _ptr(out), _stream()), "onhip_conv2d_pw_pack_weights")
    return out


def conv2d_pw_f32(a, b, x, wa_packed, bias_a, wb_packed, bias_b, addend=None, relu_after=False, out=None):
    """convolution a (packed weights) and the 1x1 convolution b over its result (weights from conv2d_pw_pack_weights)
    [-> Add of addend -> Relu] in one launch"""
    import torch
    oh, ow = a.out_hw()
    if out is None:
        out = torch.empty((a.n, b.cout, oh, ow), dtype=torch.float32, device=x.device)
    _check(load().onhip_conv2d_pw_f32(C.byref(a), C.byref(b), _ptr(x), _ptr(wa_packed), _ptr(bias_a), _ptr(wb_packed), _ptr(bias_b),
                                      _ptr(addend), 1 if relu_after else 0, _ptr(out), _stream()), "onhip_conv2d_pw_f32")
    return out


def attention(q, k, v, scale=1.0, out=None, merged_out=True):
    """out = Softmax(q k^T * scale) v per (batch, head).  q, k, v: views [batch, heads, tokens, head_dim] of fp32 tensors in
    any (batch, head, token) stride order with a contiguous head dimension (e.g. slices of a [batch, tokens, 3, heads,
    head_dim] projection output, permuted), fp32 or both operands and result in bfloat16 / float16; the result is [batch, tokens, heads * head_dim] (heads merged) or, with
    merged_out=False, [batch, heads, tokens, head_dim]"""
    import torch
    b, h, t, hd = q.shape
    compute = {torch.float32: abi.COMPUTE_F32, torch.bfloat16: abi.COMPUTE_BF16, torch.float16: abi.COMPUTE_F16}[q.dtype]
    if out is None:
        out = torch.empty((b, t, h * hd) if merged_out else (b, h, t, hd), dtype=q.dtype, device=q.device)
    d = abi.AttentionDesc(batch=b, heads=h, tokens=t, head_dim=hd, scale=scale, compute=compute)
    for name, ten in (("q_strides", q), ("k_strides", k), ("v_strides", v)):
        if ten.stride(3) != 1:
            raise OnhipError("attention: the head dimension must be contiguous")
        setattr(d, name, (C.c_longlong * 3)(ten.stride(0), ten.stride(1), ten.stride(2)))
    if out.dim() == 3 and merged_out:   # [b, t, pitch]: the merged layout, possibly with a channel pitch above heads * head_dim
        d.out_strides = (C.c_longlong * 3)(out.stride(0), hd, out.stride(1))
    else:
        d.out_strides = (C.c_longlong * 3)(h * t * hd, t * hd, hd)
    _check(load().onhip_attention(C.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _stream()), "onhip_attention")
    return out


def gemm_f32(a, w, bias, out=None):
    import torch
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    _check(load().onhip_gemm_f32(M, K, N, _ptr(a), _ptr(w), _ptr(bias), _ptr(out), _stream()), "onhip_gemm_f32")
    return out


def copy_f32(src, dst):
    """plain device copy (the yardstick for HBM traffic counters)"""
    _check(load().onhip_copy_f32(_ptr(src), _ptr(dst), src.numel(), _stream()), "onhip_copy_f32")
    return dst


def last_launch_choice():
    """(bm, bn, split, tail, rowb, fin, dma) of the calling thread's last dense convolution / MatMul launch"""
    v = (C.c_int32 * 7)()
    load().onhip_last_launch_choice(v)
    return tuple(int(t) for t in v)


def split_tail_launches():
    """launches so far whose leftover column blocks ran as a second, K-split launch"""
    return int(load().onhip_split_tail_launches())

