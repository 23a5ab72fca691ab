"""Host side of the operator plugin boundary: the slot arrays the oneNew runtime hands to a
plugin's ``eval`` and operator objects that fill them the way the reference host classes do.

Mirrors, for the Conv / MatMul / Gemm path only:
  host/op.h:35-39,109-185     params_vec / inputs_vec / outputs_vec, rt_prepare, forward
  host/ops/conv.h:31-58,60-157,178-194   shape inference, slot filling, SiLU table
  host/ops/mat_mul.h:32-57, host/ops/gemm.h:28-48    output shapes
An operator object owns host buffers exactly like the reference (weights live for the lifetime of
the object, activations are caller buffers) and calls whatever ``eval`` it is given: the HIP plugin
of this package or any other shared object with the same symbol.
"""
import ctypes as C
import numpy as np

from . import abi
from .abi import (BUFFER_INFO_S, OPERAND_S, CONV_CONFIG_S, GEMM_CONFIG_S, MATMUL_CONFIG_S, USEFUL_INFO_S,
                  BUF_MAXNUM, ConvDesc)

EVAL_T = C.CFUNCTYPE(C.c_int, C.POINTER(BUFFER_INFO_S), C.POINTER(BUFFER_INFO_S), C.POINTER(BUFFER_INFO_S))


class Plugin:
    """A shared object exporting ``eval`` (host/op.h:41-80 find_handle)."""

    def __init__(self, path):
        self.path = str(path)
        self.lib = C.CDLL(self.path, mode=C.RTLD_LOCAL)
        self.eval = self.lib.eval
        self.eval.restype = C.c_int
        self.eval.argtypes = [C.POINTER(BUFFER_INFO_S)] * 3
        # entry points beside `eval` that the HIP Conv plugin has and the reference's plugins do not: the convolution
        # with the Add (and Relu) of a residual block folded in, the other operand of the Add in inputs[3]
        # and a whole inverted-residual block (eval_block, eval_block_takes) or a convolution and the 1x1 convolution after
        # it (eval_pair, eval_pair_relu, eval_pair_takes); the MatMul plugin's fused forms
        # (eval_link: an int8 convolution whose activations travel as int8 NHWC on one or both sides)
        for extra in ("eval_add", "eval_add_relu", "eval_block", "eval_block_takes", "eval_pair", "eval_pair_relu", "eval_pair_takes", "eval_link", "eval_attention", "eval_bias", "eval_bias_gelu",
                      "eval_bias_add"):
            fn = getattr(self.lib, extra, None) if hasattr(self.lib, extra) else None
            if fn is not None:
                fn.restype = C.c_int
                fn.argtypes = [C.POINTER(BUFFER_INFO_S)] * 3
            setattr(self, extra, fn)


def aligned_empty(shape, dtype=np.float32, align=64, extra=16):
    """host buffer aligned like the runtime's aligned_alloc(32, ...) (host/net.h:434-449), with a few
    spare elements because the reference int8 quantiser reads past the end (conv.c:967-973)"""
    dtype = np.dtype(dtype)
    n = int(np.prod(shape))
    raw = np.zeros((n + extra) * dtype.itemsize + align, dtype=np.uint8)
    off = (-raw.ctypes.data) % align
    return raw[off:off + n * dtype.itemsize].view(dtype).reshape(shape)


def make_operand(shape, name=b"", fixed=False, dtype=abi.TYPE_FP32):
    o = OPERAND_S()
    o.operand_name = name
    o.is_fixed_val = int(fixed)
    o.dim_num_of_shapes = len(shape)
    for i in range(abi.SHAPE_LEN):
        o.shapes[i] = int(shape[i]) if i < len(shape) else 1
    o.data_type = dtype
    return o


def make_useful_info(scratch_bytes=0):
    """per-model tunables with the defaults onnx2one writes (tools/onnx2one/onnx2one.cpp:1332-1350);
    returns (struct, scratch array or None)"""
    u = USEFUL_INFO_S()
    u.useful_info_magic_num = abi.USEFUL_INFO_MAGIC_NUM
    bi = u.block_info
    bi.x86_gemm_single_threads_tile_m, bi.x86_gemm_single_threads_tile_n, bi.x86_gemm_single_threads_tile_k = 32, 1024, 8
    bi.x86_gemm_multi_threads_tile_m, bi.x86_gemm_multi_threads_tile_n, bi.x86_gemm_multi_threads_tile_k = 32, 1024, 8
    bi.cuda_gemm_tile_m = bi.cuda_gemm_tile_n = bi.cuda_gemm_tile_k = 16
    scratch = None
    if scratch_bytes:
        scratch = aligned_empty((scratch_bytes,), np.uint8, extra=0)
        u.public_buf_info.public_buf_size = scratch_bytes
        u.public_buf_info.public_buf_ptr = scratch.ctypes.data
    return u, scratch


def build_silu_lut():
    """host/ops/conv.h:178-194, all-float: x = i/512 - 8, x / (1 + expf(-x)).  The table handed to a
    plugin in production is built by the oneNew host with its libm; this numpy form is for callers
    that have none.  Parity tests use the committed table in tests/golden."""
    x = (np.arange(8192, dtype=np.float32) * np.float32(1.0 / 512) - np.float32(8.0)).astype(np.float32)
    return (x / (np.float32(1.0) + np.exp(-x, dtype=np.float32))).astype(np.float32)


class _Op:
    def __init__(self, evalfn):
        self.eval = evalfn
        self.params_vec = (BUFFER_INFO_S * BUF_MAXNUM)()
        self.inputs_vec = (BUFFER_INFO_S * BUF_MAXNUM)()
        self.outputs_vec = (BUFFER_INFO_S * BUF_MAXNUM)()
        self._keep = []

    def _slot(self, vec, i, obj):
        """obj: ctypes struct (address of), numpy array (data pointer) or int (raw address)"""
        if isinstance(obj, np.ndarray):
            addr = obj.ctypes.data
        elif isinstance(obj, int):
            addr = obj
        else:
            addr = C.addressof(obj)
        self._keep.append(obj)
        vec[i].addr = addr

    def forward(self):
        """host/op.h:171-185"""
        return self.eval(self.params_vec, self.inputs_vec, self.outputs_vec)


class Conv(_Op):
    """host/ops/conv.h.  ``desc`` carries geometry and epilogue; weights are fp32 [cout, cin/g, kh, kw]
    or, for the W8A32 form, int8 packed at the front of the fp32-sized buffer with an int32 bias
    (tools/optimize/model_quant.hpp:14-25)."""

    def __init__(self, evalfn, desc, weight, bias=None, weight_aux=None, silu_lut=None, scratch_bytes=0):
        super().__init__(evalfn)
        d = self.desc = ConvDesc.from_buffer_copy(desc)
        cfg = self.conv_cfg = CONV_CONFIG_S()
        cfg.op_base_cfg.op_type = b"Conv"
        cfg.op_base_cfg.in_operand_num = 3 if d.has_bias else 2
        cfg.op_base_cfg.out_operand_num = 1
        cfg.has_bias = d.has_bias
        cfg.dilations[0] = cfg.dilations[1] = 1
        cfg.group = d.group
        cfg.kernel_shape[0], cfg.kernel_shape[1] = d.kh, d.kw
        cfg.pads[0], cfg.pads[1], cfg.pads[2], cfg.pads[3] = d.pad_t, d.pad_l, d.pad_b, d.pad_r
        cfg.strides[0], cfg.strides[1] = d.stride_h, d.stride_w
        cfg.act_type = d.act_type
        cfg.clip_min, cfg.clip_max = d.clip_min, d.clip_max
        cfg.leaky_relu_alpha = d.leaky_relu_alpha
        cfg.hard_sigmoid_alpha, cfg.hard_sigmoid_beta = d.hard_sigmoid_alpha, d.hard_sigmoid_beta
        self.int8 = weight_aux is not None
        if self.int8:
            cfg.ifmap_quant2 = abi.TYPE_INT8
            cfg.input_scale = d.input_scale
            aux = np.asarray(weight_aux, dtype=np.float32)
            assert aux.shape == (d.cout,) and d.cout <= 4096
            C.memmove(cfg.weight_aux, aux.ctypes.data, aux.nbytes)
        kc = d.cin if d.group == 1 else 1
        wshape = (d.cout, kc, d.kh, d.kw)
        # weight / bias storage is always sized as fp32, as in std::vector<float> initial_datas
        self.weight = aligned_empty(wshape, np.float32)
        if self.int8:
            w8 = np.ascontiguousarray(weight, dtype=np.int8).reshape(-1)
            self.weight.reshape(-1).view(np.int8)[:w8.size] = w8
        else:
            self.weight[...] = np.asarray(weight, dtype=np.float32).reshape(wshape)
        self.weight_operand = make_operand(wshape, b"weight", fixed=True)
        self.useful, self._scratch = make_useful_info(scratch_bytes)
        oh, ow = d.out_hw()
        self.in_operand = make_operand((d.n, d.cin, d.h, d.w), b"in")
        self.out_operand = make_operand((d.n, d.cout, oh, ow), b"out")
        self._slot(self.params_vec, 0, cfg)
        self._slot(self.params_vec, 1, self.in_operand)
        self._slot(self.params_vec, 2, self.weight_operand)
        self._slot(self.inputs_vec, 1, self.weight)
        if d.has_bias:
            self.bias = aligned_empty((d.cout,), np.float32)
            if self.int8:
                self.bias.view(np.int32)[...] = np.asarray(bias, dtype=np.int32)
            else:
                self.bias[...] = np.asarray(bias, dtype=np.float32)
            self.bias_operand = make_operand((d.cout,), b"bias", fixed=True)
            self._slot(self.params_vec, 3, self.bias_operand)
            self._slot(self.inputs_vec, 2, self.bias)
            self._slot(self.params_vec, 4, self.out_operand)
        else:
            self._slot(self.params_vec, 3, self.out_operand)
        self._slot(self.params_vec, BUF_MAXNUM - 1, self.useful)
        if d.act_type == abi.SILU:
            self.lut = np.ascontiguousarray(silu_lut if silu_lut is not None else build_silu_lut(), dtype=np.float32)
            self._slot(self.inputs_vec, BUF_MAXNUM - 1, self.lut)

    def __call__(self, x, out=None, addend=None):
        """addend: the tensor of the output's shape that `eval_add` / `eval_add_relu` add to the result (inputs[3])"""
        d = self.desc
        oh, ow = d.out_hw()
        xin = x if isinstance(x, int) else np.ascontiguousarray(x, dtype=np.float32)
        if out is None:
            out = aligned_empty((d.n, d.cout, oh, ow), np.float32)
        self._slot(self.inputs_vec, 0, xin)
        self._slot(self.outputs_vec, 0, out)
        kept = 2
        if addend is not None:
            self._slot(self.inputs_vec, 3, addend if isinstance(addend, int) else np.ascontiguousarray(addend, dtype=np.float32))
            kept = 3
        rc = self.forward()
        del self._keep[-kept:]
        self.inputs_vec[3].addr = 0
        if rc != 0:
            raise RuntimeError(f"Conv eval returned {rc}")
        return out


class ConvLink(Conv):
    """A dense W8A32 Conv through the HIP Conv plugin's `eval_link`: the slots of `eval` plus inputs[4] = {int32 in_s8,
    int32 out_s8, float out_scale, int32 twin} and inputs[5] = null or an int32 fold code (1: Add, 2: Add + Relu, the
    other operand in inputs[3]).  in_s8: x is int8 [n, h, w, channels padded to 16]; out_s8: the result is stored that
    way, quantised with out_scale.  No counterpart among the reference's host classes."""

    class _Flags(C.Structure):
        _fields_ = [("in_s8", C.c_int32), ("out_s8", C.c_int32), ("out_scale", C.c_float), ("twin", C.c_int32)]

    def __init__(self, plugin, desc, weight, bias, weight_aux, silu_lut=None):
        super().__init__(plugin.eval_link, desc, weight, bias, weight_aux=weight_aux, silu_lut=silu_lut)

    def __call__(self, x, in_s8=False, out_scale=None, addend=None, relu_after=False):
        d = self.desc
        oh, ow = d.out_hw()
        flags = self._Flags(int(in_s8), int(out_scale is not None), float(out_scale or 0.0), 0)
        fold = C.c_int32(0 if addend is None else 2 if relu_after else 1)
        xin = np.ascontiguousarray(x, dtype=np.int8 if in_s8 else np.float32)
        if out_scale is not None:
            out = aligned_empty((d.n, oh, ow, (d.cout + 15) // 16 * 16), np.int8)
        else:
            out = aligned_empty((d.n, d.cout, oh, ow), np.float32)
        self._slot(self.inputs_vec, 0, xin)
        self._slot(self.outputs_vec, 0, out)
        self._slot(self.inputs_vec, 4, flags)
        kept = 3
        if addend is not None:
            self._slot(self.inputs_vec, 3, np.ascontiguousarray(addend, dtype=np.float32))
            self._slot(self.inputs_vec, 5, fold)
            kept = 5
        rc = self.forward()
        del self._keep[-kept:]
        self.inputs_vec[3].addr = self.inputs_vec[4].addr = self.inputs_vec[5].addr = 0
        if rc != 0:
            raise RuntimeError(f"Conv eval_link returned {rc}")
        return out


class ConvBlock(_Op):
    """Conv (1x1) -> Conv (depthwise 3x3) -> Conv (1x1) [-> Add] through the HIP Conv plugin's `eval_block`: the slots of the
    first convolution's `eval` with the block's result operand in params[4], then the depthwise convolution's CONV_CONFIG_S,
    weight operand, weights and bias in params[5], params[6], inputs[5], inputs[6] and the last convolution's in params[7],
    params[8], inputs[7], inputs[8]; the addend in inputs[3].  No counterpart among the reference's host classes."""

    def __init__(self, plugin, descs, weights, biases):
        super().__init__(plugin.eval_block)
        self.takes_fn = plugin.eval_block_takes
        self.convs = [Conv(None, d, w, b) for d, w, b in zip(descs, weights, biases)]
        ex, dw, pw = self.convs
        oh, ow = pw.desc.out_hw()
        self.out_shape = (pw.desc.n, pw.desc.cout, oh, ow)
        self.out_operand = make_operand(self.out_shape, b"out")
        self._slot(self.params_vec, 0, ex.conv_cfg)
        self._slot(self.params_vec, 1, ex.in_operand)
        self._slot(self.params_vec, 2, ex.weight_operand)
        self._slot(self.params_vec, 3, ex.bias_operand)
        self._slot(self.params_vec, 4, self.out_operand)
        self._slot(self.inputs_vec, 1, ex.weight)
        self._slot(self.inputs_vec, 2, ex.bias)
        for base, conv in ((5, dw), (7, pw)):
            self._slot(self.params_vec, base, conv.conv_cfg)
            self._slot(self.params_vec, base + 1, conv.weight_operand)
            self._slot(self.inputs_vec, base, conv.weight)
            if conv.desc.has_bias:
                self._slot(self.inputs_vec, base + 1, conv.bias)

    def takes(self):
        """1 when the library recommends the one-launch kernel for these shapes"""
        return self.takes_fn(self.params_vec, self.inputs_vec, self.outputs_vec)

    def __call__(self, x, addend=None, out=None):
        xin = np.ascontiguousarray(x, dtype=np.float32)
        if out is None:
            out = aligned_empty(self.out_shape, np.float32)
        self._slot(self.inputs_vec, 0, xin)
        self._slot(self.outputs_vec, 0, out)
        kept = 2
        if addend is not None:
            self._slot(self.inputs_vec, 3, np.ascontiguousarray(addend, dtype=np.float32))
            kept = 3
        rc = self.forward()
        del self._keep[-kept:]
        self.inputs_vec[3].addr = 0
        if rc != 0:
            raise RuntimeError(f"Conv eval_block returned {rc}")
        return out


class ConvPair(_Op):
    """Conv (dense, at most 64 output channels) -> Conv (1x1) [-> Add [-> Relu]] through the HIP Conv plugin's `eval_pair` /
    `eval_pair_relu`: the slots of the first convolution's `eval` with the pair's result operand in params[4], then the second
    convolution's CONV_CONFIG_S, weight operand, weights and bias in params[5], params[6], inputs[5], inputs[6]; the addend
    in inputs[3].  No counterpart among the reference's host classes."""

    def __init__(self, plugin, descs, weights, biases):
        super().__init__(plugin.eval_pair)
        self.relu_fn, self.takes_fn = plugin.eval_pair_relu, plugin.eval_pair_takes
        self.convs = [Conv(None, d, w, b) for d, w, b in zip(descs, weights, biases)]
        first, second = self.convs
        oh, ow = second.desc.out_hw()
        self.out_shape = (second.desc.n, second.desc.cout, oh, ow)
        self.out_operand = make_operand(self.out_shape, b"out")
        self._slot(self.params_vec, 0, first.conv_cfg)
        self._slot(self.params_vec, 1, first.in_operand)
        self._slot(self.params_vec, 2, first.weight_operand)
        self._slot(self.params_vec, 3, first.bias_operand)
        self._slot(self.params_vec, 4, self.out_operand)
        self._slot(self.inputs_vec, 1, first.weight)
        if first.desc.has_bias:
            self._slot(self.inputs_vec, 2, first.bias)
        self._slot(self.params_vec, 5, second.conv_cfg)
        self._slot(self.params_vec, 6, second.weight_operand)
        self._slot(self.inputs_vec, 5, second.weight)
        if second.desc.has_bias:
            self._slot(self.inputs_vec, 6, second.bias)

    def takes(self):
        """1 when the library recommends the one-launch kernel for these shapes"""
        return self.takes_fn(self.params_vec, self.inputs_vec, self.outputs_vec)

    def __call__(self, x, addend=None, relu=False, out=None):
        xin = np.ascontiguousarray(x, dtype=np.float32)
        if out is None:
            out = aligned_empty(self.out_shape, np.float32)
        self._slot(self.inputs_vec, 0, xin)
        self._slot(self.outputs_vec, 0, out)
        kept = 2
        if addend is not None:
            self._slot(self.inputs_vec, 3, np.ascontiguousarray(addend, dtype=np.float32))
            kept = 3
        rc = (self.relu_fn if relu else self.eval)(self.params_vec, self.inputs_vec, self.outputs_vec)
        del self._keep[-kept:]
        self.inputs_vec[3].addr = 0
        if rc != 0:
            raise RuntimeError(f"Conv eval_pair returned {rc}")
        return out


class MatMul(_Op):
    """host/ops/mat_mul.h: out = A[..., M, K] @ B, B either [K, N] shared or batched like A."""

    def __init__(self, evalfn):
        super().__init__(evalfn)
        self.mat_mul_cfg = MATMUL_CONFIG_S()
        self.mat_mul_cfg.op_base_cfg.op_type = b"MatMul"
        self.mat_mul_cfg.op_base_cfg.in_operand_num = 2
        self.mat_mul_cfg.op_base_cfg.out_operand_num = 1
        self._slot(self.params_vec, 0, self.mat_mul_cfg)

    def __call__(self, a, b, out=None):
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        oshape = a.shape[:-1] + (b.shape[-1],)
        if out is None:
            out = aligned_empty(oshape, np.float32)
        ops = [make_operand(a.shape, b"a"), make_operand(b.shape, b"b"), make_operand(oshape, b"out")]
        for i, o in enumerate(ops):
            self._slot(self.params_vec, 1 + i, o)
        self._slot(self.inputs_vec, 0, a)
        self._slot(self.inputs_vec, 1, b)
        self._slot(self.outputs_vec, 0, out)
        rc = self.forward()
        del self._keep[-6:]
        if rc != 0:
            raise RuntimeError(f"MatMul eval returned {rc}")
        return out


class MatMulFused(_Op):
    """The HIP MatMul plugin's entry points beside `eval` (no counterpart among the reference's host classes):
    linear(): MatMul -> Add of a bias [-> Gelu | -> Add of a tensor shaped like the result] through eval_bias /
    eval_bias_gelu / eval_bias_add (bias in params[3] / inputs[2], result operand in params[4], Gelu table in inputs[11],
    second addend in inputs[3]); attention(): MatMul(q, Transpose(k)) -> Softmax -> MatMul(., v) through eval_attention
    (q, k, v in params[1..3] / inputs[0..2], result in params[4], four int32 layout flags behind inputs[4])."""

    def __init__(self, plugin):
        super().__init__(None)
        self.plugin = plugin
        self.cfg = MATMUL_CONFIG_S()
        self.cfg.op_base_cfg.op_type = b"MatMul"
        self._slot(self.params_vec, 0, self.cfg)

    def _run(self, fn, what):
        rc = fn(self.params_vec, self.inputs_vec, self.outputs_vec)
        for vec in (self.params_vec, self.inputs_vec, self.outputs_vec):
            for i in range(1 if vec is self.params_vec else 0, BUF_MAXNUM):
                vec[i].addr = 0
        del self._keep[1:]
        if rc != 0:
            raise RuntimeError(f"MatMul {what} returned {rc}")

    def linear(self, a, w, bias, gelu_lut=None, addend=None):
        a, w, bias = (np.ascontiguousarray(t, dtype=np.float32) for t in (a, w, bias))
        oshape = a.shape[:-1] + (w.shape[-1],)
        out = aligned_empty(oshape, np.float32)
        for i, o in enumerate([make_operand(a.shape, b"a"), make_operand(w.shape, b"w", fixed=True),
                               make_operand(bias.shape, b"bias", fixed=True), make_operand(oshape, b"out")]):
            self._slot(self.params_vec, 1 + i, o)
        for i, t in enumerate((a, w, bias)):
            self._slot(self.inputs_vec, i, t)
        self._slot(self.outputs_vec, 0, out)
        fn, what = self.plugin.eval_bias, "eval_bias"
        if gelu_lut is not None:
            self._slot(self.inputs_vec, BUF_MAXNUM - 1, np.ascontiguousarray(gelu_lut, dtype=np.float32))
            fn, what = self.plugin.eval_bias_gelu, "eval_bias_gelu"
        elif addend is not None:
            self._slot(self.inputs_vec, 3, np.ascontiguousarray(addend, dtype=np.float32))
            fn, what = self.plugin.eval_bias_add, "eval_bias_add"
        self._run(fn, what)
        return out

    def attention(self, q, k, v, token_major=(0, 0, 0, 0)):
        """q, k, v: [batch, heads, tokens, head_dim], or [batch, tokens, heads, head_dim] where the flag is set; so the
        result (flag 3)"""
        q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
        b, h, t, d = q.shape if not token_major[0] else (q.shape[0], q.shape[2], q.shape[1], q.shape[3])
        oshape = (b, t, h, d) if token_major[3] else (b, h, t, d)
        out = aligned_empty(oshape, np.float32)
        for i, o in enumerate([make_operand(q.shape, b"q"), make_operand(k.shape, b"k"), make_operand(v.shape, b"v"),
                               make_operand(oshape, b"out")]):
            self._slot(self.params_vec, 1 + i, o)
        for i, tns in enumerate((q, k, v)):
            self._slot(self.inputs_vec, i, tns)
        if any(token_major):
            self._slot(self.inputs_vec, 4, np.asarray(token_major, dtype=np.int32))
        self._slot(self.outputs_vec, 0, out)
        self._run(self.plugin.eval_attention, "eval_attention")
        return out


class Gemm(_Op):
    """host/ops/gemm.h: out[M, N] = A[M, K] @ W[N, K]^T + bias[N]; alpha, beta, transB ignored."""

    def __init__(self, evalfn, weight, bias):
        super().__init__(evalfn)
        self.gemm_cfg = GEMM_CONFIG_S()
        self.gemm_cfg.op_base_cfg.op_type = b"Gemm"
        self.gemm_cfg.op_base_cfg.in_operand_num = 3
        self.gemm_cfg.op_base_cfg.out_operand_num = 1
        self.gemm_cfg.has_bias = 1
        self.gemm_cfg.alpha = self.gemm_cfg.beta = 1.0
        self.gemm_cfg.transB = 1
        self.weight = aligned_empty(np.shape(weight), np.float32)
        self.weight[...] = weight
        self.bias = aligned_empty(np.shape(bias), np.float32)
        self.bias[...] = bias
        self.w_operand = make_operand(self.weight.shape, b"w", fixed=True)
        self.b_operand = make_operand(self.bias.shape, b"bias", fixed=True)
        self._slot(self.params_vec, 0, self.gemm_cfg)
        self._slot(self.params_vec, 2, self.w_operand)
        self._slot(self.params_vec, 3, self.b_operand)
        self._slot(self.inputs_vec, 1, self.weight)
        self._slot(self.inputs_vec, 2, self.bias)

    def __call__(self, a, out=None):
        a = np.ascontiguousarray(a, dtype=np.float32)
        oshape = a.shape[:-1] + (self.bias.shape[0],)
        if out is None:
            out = aligned_empty(oshape, np.float32)
        ain, aout = make_operand(a.shape, b"a"), make_operand(oshape, b"out")
        self._slot(self.params_vec, 1, ain)
        self._slot(self.params_vec, 4, aout)
        self._slot(self.inputs_vec, 0, a)
        self._slot(self.outputs_vec, 0, out)
        rc = self.forward()
        del self._keep[-4:]
        if rc != 0:
            raise RuntimeError(f"Gemm eval returned {rc}")
        return out


class Add(_Op):
    """host/ops/add.h: out = in0 + in1 with numpy broadcasting of the smaller operand (device/x86/Add/add.c)."""

    def __init__(self, evalfn):
        super().__init__(evalfn)
        self.cfg = abi.PLAIN_CONFIG_S()
        self.cfg.op_base_cfg.op_type = b"Add"
        self.cfg.op_base_cfg.in_operand_num = 2
        self.cfg.op_base_cfg.out_operand_num = 1
        self._slot(self.params_vec, 0, self.cfg)

    def __call__(self, a, b, out=None):
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        oshape = a.shape if a.size >= b.size else b.shape
        if out is None:
            out = aligned_empty(oshape, np.float32)
        descs = [make_operand(a.shape, b"a"), make_operand(b.shape, b"b"), make_operand(oshape, b"out")]
        for i, o in enumerate(descs):
            self._slot(self.params_vec, 1 + i, o)
        self._slot(self.inputs_vec, 0, a)
        self._slot(self.inputs_vec, 1, b)
        self._slot(self.outputs_vec, 0, out)
        rc = self.forward()
        del self._keep[-6:]
        if rc != 0:
            raise RuntimeError(f"Add eval returned {rc}")
        return out


class _Unary(_Op):
    op_type = b""

    def __init__(self, evalfn, cfg=None):
        super().__init__(evalfn)
        self.cfg = cfg if cfg is not None else abi.PLAIN_CONFIG_S()
        self.cfg.op_base_cfg.op_type = self.op_type
        self.cfg.op_base_cfg.in_operand_num = 1
        self.cfg.op_base_cfg.out_operand_num = 1
        self._slot(self.params_vec, 0, self.cfg)

    def out_shape(self, shape):
        return shape

    def __call__(self, x, out=None):
        x = np.ascontiguousarray(x, dtype=np.float32)
        oshape = self.out_shape(x.shape)
        if out is None:
            out = aligned_empty(oshape, np.float32)
        descs = [make_operand(x.shape, b"in"), make_operand(oshape, b"out")]
        self._slot(self.params_vec, 1, descs[0])
        self._slot(self.params_vec, 2, descs[1])
        self._slot(self.inputs_vec, 0, x)
        self._slot(self.outputs_vec, 0, out)
        rc = self.forward()
        del self._keep[-4:]
        if rc != 0:
            raise RuntimeError(f"{self.op_type.decode()} eval returned {rc}")
        return out


class Relu(_Unary):
    """host/ops/relu.h (device/x86/Relu/relu.c)"""
    op_type = b"Relu"


class GlobalAveragePool(_Unary):
    """host/ops/global_avgpool.h (device/x86/GlobalAveragePool/global_avgpool.c)"""
    op_type = b"GlobalAveragePool"

    def out_shape(self, shape):
        return (shape[0], shape[1], 1, 1)


class MaxPool(_Unary):
    """host/ops/max_pool.h (device/x86/MaxPool/maxpool.c): square padding pads[0], floor-mode output shape;
    the kernel takes its scratch for the padded copy from USEFUL_INFO_S in params[11]."""
    op_type = b"MaxPool"

    def __init__(self, evalfn, kernel, stride, pad, scratch_bytes=0):
        cfg = abi.MAX_POOL_CONFIG_S()
        cfg.kernel_shape[0], cfg.kernel_shape[1] = kernel, kernel
        cfg.strides[0], cfg.strides[1] = stride, stride
        for i in range(4):
            cfg.pads[i] = pad
        super().__init__(evalfn, cfg)
        self.kernel, self.stride, self.pad = kernel, stride, pad
        self.useful, self._scratch = make_useful_info(scratch_bytes)
        self._slot(self.params_vec, BUF_MAXNUM - 1, self.useful)

    def out_shape(self, shape):
        n, c, h, w = shape
        return (n, c, (h + 2 * self.pad - self.kernel) // self.stride + 1,
                (w + 2 * self.pad - self.kernel) // self.stride + 1)


class Gelu(_Unary):
    """host/ops/gelu.h: table GELU, the 8192-entry table travels in inputs[11] (device/x86/Gelu/gelu.c)"""
    op_type = b"Gelu"

    def __init__(self, evalfn, gelu_lut):
        super().__init__(evalfn)
        self.lut = np.ascontiguousarray(gelu_lut, dtype=np.float32)
        self._slot(self.inputs_vec, BUF_MAXNUM - 1, self.lut)


class LayerNormalization(_Unary):
    """host/ops/layer_normalization.h: weight in inputs[1], bias in inputs[2]; axes[0] == 1 normalises dimension 1
    (device/x86/LayerNormalization/layer_normalization.c)"""
    op_type = b"LayerNormalization"

    def __init__(self, evalfn, weight, bias, axis=-1):
        cfg = abi.LAYERNORMALIZATION_CONFIG_S()
        cfg.axes[0] = axis
        cfg.axes_num = 1
        super().__init__(evalfn, cfg)
        self.weight = np.ascontiguousarray(weight, dtype=np.float32)
        self.bias = np.ascontiguousarray(bias, dtype=np.float32)
        self._slot(self.inputs_vec, 1, self.weight)
        self._slot(self.inputs_vec, 2, self.bias)


class Softmax(_Unary):
    """host/ops/softmax.h (device/x86/Softmax/softmax.c): the last axis, or axis 1 of a batch-1 tensor"""
    op_type = b"Softmax"

    def __init__(self, evalfn, axis=-1):
        cfg = abi.SOFTMAX_CONFIG_S()
        cfg.axis = axis
        super().__init__(evalfn, cfg)


class Transpose(_Unary):
    """host/ops/transpose.h (device/x86/Transpose/transpose.c): out dim k = in dim perm[k]"""
    op_type = b"Transpose"

    def __init__(self, evalfn, perm):
        cfg = abi.TRANSPOSE_CONFIG_S()
        for i, p in enumerate(perm):
            cfg.perm[i] = p
        cfg.perm_num = len(perm)
        super().__init__(evalfn, cfg)
        self.perm = tuple(perm)

    def out_shape(self, shape):
        return tuple(shape[p] for p in self.perm)
