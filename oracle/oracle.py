"""ctypes front end of the CPU oracle (oracle/liboracle.so) and of the compiled reference kernels
(oracle/_ref/*.so, present only where `make -C oracle ref` could see the reference sources).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg; never by the onenew_amd package."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from onenew_amd.abi import ConvDesc  # noqa: E402

_lib = None
f32p, s8p, s32p = C.POINTER(C.c_float), C.POINTER(C.c_int8), C.POINTER(C.c_int32)


def build(force=False):
    so = os.path.join(HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", HERE, "liboracle.so"] + (["-B"] if force else []))
    return so


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.oracle_conv2d_f32.argtypes = [C.POINTER(ConvDesc), f32p, f32p, f32p, f32p, f32p]
        _lib.oracle_conv2d_w8a32.argtypes = [C.POINTER(ConvDesc), f32p, s8p, s32p, f32p, f32p, C.c_void_p, s32p]
        _lib.oracle_matmul_f32.argtypes = [C.c_int] * 5 + [f32p] * 3
        _lib.oracle_gemm_f32.argtypes = [C.c_int] * 3 + [f32p] * 4
        _lib.oracle_matmul_bias_gelu_f32.argtypes = [C.c_int] * 5 + [f32p] * 5
        _lib.oracle_quantize_s8.argtypes = [f32p, C.c_float, s8p, C.c_int64]
        _lib.oracle_lut_act_f32.argtypes = [f32p, f32p, f32p, C.c_int64]
        _lib.oracle_quant_weight_bias.argtypes = [f32p, f32p, C.c_int, C.c_int, s8p, s32p, f32p]
        _lib.oracle_round_bf16.argtypes = [f32p, f32p, C.c_int64]
        _lib.oracle_round_f16.argtypes = [f32p, f32p, C.c_int64]
        _lib.oracle_build_silu_lut.argtypes = [f32p]
        _lib.oracle_build_gelu_lut.argtypes = [f32p]
    return _lib


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    lib().oracle_set_threads(int(n))


def silu_lut():
    t = np.empty(8192, np.float32)
    lib().oracle_build_silu_lut(_p(t, f32p))
    return t


def gelu_lut():
    t = np.empty(8192, np.float32)
    lib().oracle_build_gelu_lut(_p(t, f32p))
    return t


def conv2d_f32(d, x, w, bias=None, lut=None):
    x, w, bias, lut = _f32(x), _f32(w), _f32(bias), _f32(lut)
    oh, ow = d.out_hw()
    y = np.empty((d.n, d.cout, oh, ow), np.float32)
    rc = lib().oracle_conv2d_f32(C.byref(d), _p(x, f32p), _p(w, f32p), _p(bias, f32p), _p(lut, f32p), _p(y, f32p))
    if rc:
        raise ValueError(f"oracle_conv2d_f32 rc={rc}")
    return y


def conv2d_w8a32(d, x, w8, bias32, weight_aux, lut=None, want_acc=False):
    x, weight_aux, lut = _f32(x), _f32(weight_aux), _f32(lut)
    w8 = np.ascontiguousarray(w8, dtype=np.int8)
    bias32 = None if bias32 is None else np.ascontiguousarray(bias32, dtype=np.int32)
    oh, ow = d.out_hw()
    y = np.empty((d.n, d.cout, oh, ow), np.int8 if d.out_s8 else np.float32)
    acc = np.empty((d.n, d.cout, oh, ow), np.int32) if want_acc else None
    rc = lib().oracle_conv2d_w8a32(C.byref(d), _p(x, f32p), _p(w8, s8p), _p(bias32, s32p), _p(weight_aux, f32p),
                                   _p(lut, f32p), y.ctypes.data, _p(acc, s32p))
    if rc:
        raise ValueError(f"oracle_conv2d_w8a32 rc={rc}")
    return (y, acc) if want_acc else y


def matmul_f32(a, b, bias=None, gelu=None):
    a, b, bias, gelu = _f32(a), _f32(b), _f32(bias), _f32(gelu)
    M, K = a.shape[-2:]
    N = b.shape[-1]
    batch = int(np.prod(a.shape[:-2])) if a.ndim > 2 else 1
    shared = int(b.size == K * N)
    out = np.empty(a.shape[:-1] + (N,), np.float32)
    if bias is None and gelu is None:
        rc = lib().oracle_matmul_f32(batch, M, K, N, shared, _p(a, f32p), _p(b, f32p), _p(out, f32p))
    else:
        rc = lib().oracle_matmul_bias_gelu_f32(batch, M, K, N, shared, _p(a, f32p), _p(b, f32p), _p(bias, f32p),
                                               _p(gelu, f32p), _p(out, f32p))
    if rc:
        raise ValueError(f"oracle_matmul rc={rc}")
    return out


def gemm_f32(a, w, bias):
    a, w, bias = _f32(a), _f32(w), _f32(bias)
    M, K = a.shape
    N = w.shape[0]
    out = np.empty((M, N), np.float32)
    rc = lib().oracle_gemm_f32(M, K, N, _p(a, f32p), _p(w, f32p), _p(bias, f32p), _p(out, f32p))
    if rc:
        raise ValueError(f"oracle_gemm rc={rc}")
    return out


def quantize_s8(x, scale):
    x = _f32(x)
    q = np.empty(x.shape, np.int8)
    lib().oracle_quantize_s8(_p(x, f32p), float(scale), _p(q, s8p), x.size)
    return q


def lut_act(x, lut):
    x, lut = _f32(x), _f32(lut)
    y = np.empty_like(x)
    lib().oracle_lut_act_f32(_p(x, f32p), _p(lut, f32p), _p(y, f32p), x.size)
    return y


def quant_weight_bias(w, bias):
    w = _f32(w)
    bias = _f32(bias)
    cout = w.shape[0]
    per = w.size // cout
    w8 = np.empty(w.shape, np.int8)
    b32 = np.empty(cout, np.int32)
    aux = np.empty(cout, np.float32)
    lib().oracle_quant_weight_bias(_p(w, f32p), _p(bias, f32p), cout, per, _p(w8, s8p), _p(b32, s32p), _p(aux, f32p))
    return w8, b32, aux


def add_f32(a, b):
    """device/x86/Add semantics: the operand with fewer elements (the second on a tie) is broadcast"""
    a, b = _f32(a), _f32(b)
    large, small = (b, a) if a.size < b.size else (a, b)
    ls, ss = list(large.shape), list(small.shape)
    if large.size == small.size or small.size == 1:
        ls, ss = [large.size], [small.size]
    ss = [1] * (len(ls) - len(ss)) + ss
    out = np.empty(large.shape, np.float32)
    i32 = C.c_int32 * len(ls)
    rc = lib().oracle_add_f32(len(ls), i32(*ls), i32(*ss), _p(large, f32p), _p(small, f32p), _p(out, f32p))
    assert rc == 0, "shapes do not broadcast"
    return out


def relu_f32(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_relu_f32(_p(x, f32p), _p(y, f32p), C.c_int64(x.size))
    return y


def maxpool_f32(x, kernel, stride, pad):
    x = _f32(x)
    n, c, h, w = x.shape
    oh, ow = (h + 2 * pad - kernel) // stride + 1, (w + 2 * pad - kernel) // stride + 1
    y = np.empty((n, c, oh, ow), np.float32)
    rc = lib().oracle_maxpool_f32(n, c, h, w, kernel, kernel, stride, stride, pad, oh, ow, _p(x, f32p), _p(y, f32p))
    assert rc == 0
    return y


def global_avgpool_f32(x):
    x = _f32(x)
    n, c, h, w = x.shape
    y = np.empty((n, c, 1, 1), np.float32)
    lib().oracle_global_avgpool_f32(n, c, h, w, _p(x, f32p), _p(y, f32p))
    return y


def layernorm_f32(x, weight, bias, axis1=False):
    x, weight, bias = _f32(x), _f32(weight), _f32(bias)
    # the reference normalises the last dimension that is not 1 (layer_normalization.c:63-68)
    reduce = x.shape[1] if axis1 else next((d for d in reversed(x.shape) if d != 1), 1)
    y = np.empty_like(x)
    lib().oracle_layernorm_f32(x.size // reduce, reduce, int(axis1), _p(x, f32p), _p(weight, f32p), _p(bias, f32p),
                               _p(y, f32p))
    return y


def softmax_f32(x, axis1=False):
    x = _f32(x)
    reduce = x.shape[1] if axis1 else x.shape[-1]
    y = np.empty_like(x)
    lib().oracle_softmax_f32(x.size // reduce, reduce, int(axis1), _p(x, f32p), _p(y, f32p))
    return y


def transpose_f32(x, perm):
    x = _f32(x)
    i32 = C.c_int32 * x.ndim
    y = np.empty([x.shape[p] for p in perm], np.float32)
    rc = lib().oracle_transpose_f32(x.ndim, i32(*x.shape), i32(*perm), _p(x, f32p), _p(y, f32p))
    assert rc == 0
    return y


def calib_abs_max(x, running=0.0):
    x = _f32(x)
    fn = lib().oracle_calib_abs_max
    fn.restype = C.c_float
    return float(fn(_p(x, f32p), C.c_int64(x.size), C.c_float(running)))


def calib_histogram(x, max_abs, hist=None):
    x = _f32(x)
    if hist is None:
        hist = np.zeros(2048, np.float32)
    lib().oracle_calib_histogram(_p(x, f32p), C.c_int64(x.size), C.c_float(max_abs), _p(hist, f32p))
    return hist


def calib_threshold(method, hist, elem_count, max_abs):
    fn = lib().oracle_calib_threshold_kl if method == "kl" else lib().oracle_calib_threshold_mse
    fn.restype = C.c_float
    hist = _f32(hist)
    return float(fn(_p(hist, f32p), C.c_int64(elem_count), C.c_float(max_abs)))


def calib_curve(method, hist, elem_count):
    """the search's value for every candidate clipping range (128 ... 2047 bins)"""
    fn = lib().oracle_calib_kl_curve if method == "kl" else lib().oracle_calib_mse_curve
    fn.restype = None
    hist = _f32(hist)
    out = np.empty(2048 - 128, np.float32)
    fn(_p(hist, f32p), C.c_int64(elem_count), _p(out, f32p))
    return out


def calib_percentile(x, images, elems):
    x = _f32(x)
    fn = lib().oracle_calib_threshold_percent
    fn.restype = C.c_float
    return float(fn(_p(x, f32p), int(images), C.c_int32(elems)))


def round_bf16(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_round_bf16(_p(x, f32p), _p(y, f32p), x.size)
    return y


def round_f16(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_round_f16(_p(x, f32p), _p(y, f32p), x.size)
    return y


# ---- compiled reference kernels (oracle/_ref) -------------------------------------------------

def ref_path(op):
    return os.path.join(HERE, "_ref", f"lib{op}_x86.so")


def have_ref():
    return all(os.path.exists(ref_path(op)) for op in ("Conv", "MatMul", "Gemm"))


def ref_scratch_bytes(d):
    """scratch the reference Conv bump-allocates from (conv.c:353-380, :945-1010), generously"""
    oh, ow = d.out_hw()
    ph, pw = d.h + d.pad_t + d.pad_b, d.w + d.pad_l + d.pad_r
    col = d.cin * d.kh * d.kw * oh * ow
    return 4 * (d.cin * ph * pw + col) + 2 * 5 * d.cin * d.h * d.w + d.cin * (d.h + 2 * d.pad_t) * (d.w + 2 * d.pad_t) + col + 4096
