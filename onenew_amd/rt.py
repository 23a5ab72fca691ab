"""ctypes binding of the device-resident model runtime (include/onenew_rt.h, libonenew_rt.so)."""
import ctypes as C
import os

import numpy as np

from . import hip

EXPORTS = ["onrt_last_error", "onrt_net_load_file", "onrt_net_load_buf", "onrt_net_free", "onrt_net_io_count",
           "onrt_net_io_info", "onrt_net_op_count", "onrt_net_op_info", "onrt_net_operand", "onrt_net_run", "onrt_net_enqueue", "onrt_net_fused_count", "onrt_net_graph_launches", "onrt_net_plan_buf",
           "onrt_net_folded_activations", "onrt_net_fused_attentions", "onrt_net_fused_linears", "onrt_net_fused_skips", "onrt_net_fused_ir_blocks", "onrt_net_fused_pairs", "onrt_net_quantised_links", "onrt_net_tune_tiles", "onrt_net_get_tiles", "onrt_net_set_tiles", "onrt_one_set_tiles", "onrt_one_quantise"]

_lib = None


class OnrtError(RuntimeError):
    pass


def lib_path():
    return os.path.join(os.path.dirname(hip.lib_path()), "libonenew_rt.so")


def load():
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise OnrtError(f"{path} is missing: build it with `python -m onenew_amd.build`")
    L = C.CDLL(path)
    vp, i32p = C.c_void_p, C.POINTER(C.c_int32)
    L.onrt_last_error.restype = C.c_char_p
    L.onrt_net_load_file.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(vp)]
    L.onrt_net_load_buf.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.POINTER(vp)]
    L.onrt_net_free.argtypes = [vp]
    L.onrt_net_free.restype = None
    L.onrt_net_io_count.argtypes = [vp, i32p, i32p]
    L.onrt_net_io_info.argtypes = [vp, C.c_int32, C.c_int32, C.POINTER(C.c_char_p), i32p, i32p]
    L.onrt_net_op_count.argtypes = [vp, i32p]
    L.onrt_net_op_info.argtypes = [vp, C.c_int32, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p)]
    L.onrt_net_plan_buf.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(vp)]
    L.onrt_net_graph_launches.argtypes = [vp, C.POINTER(C.c_int64)]
    L.onrt_net_fused_count.argtypes = [vp, i32p, i32p]
    L.onrt_net_folded_activations.argtypes = [vp, i32p]
    L.onrt_net_fused_attentions.argtypes = [vp, i32p]
    L.onrt_net_fused_linears.argtypes = [vp, i32p]
    L.onrt_net_fused_skips.argtypes = [vp, i32p]
    L.onrt_net_fused_ir_blocks.argtypes = [vp, i32p]
    L.onrt_net_fused_pairs.argtypes = [vp, i32p]
    L.onrt_net_quantised_links.argtypes = [vp, i32p]
    L.onrt_net_operand.argtypes = [vp, C.c_char_p, i32p, i32p, C.POINTER(vp)]
    L.onrt_net_run.argtypes = [vp, C.POINTER(vp), C.POINTER(vp)]
    L.onrt_net_enqueue.argtypes = [vp, C.POINTER(vp), C.POINTER(vp)]
    L.onrt_net_tune_tiles.argtypes = [vp, C.c_int32, i32p, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.onrt_net_get_tiles.argtypes = [vp, i32p]
    L.onrt_net_set_tiles.argtypes = [vp, i32p]
    L.onrt_one_set_tiles.argtypes = [C.c_char_p, C.c_size_t, i32p]
    L.onrt_one_quantise.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.c_int32, C.POINTER(vp), C.c_int32, C.POINTER(vp), C.c_int32, C.c_char_p]
    _lib = L
    return L


def _check(rc, what):
    if rc != 0:
        raise OnrtError(f"{what} failed ({rc}): {load().onrt_last_error().decode(errors='replace')}")


def with_tiles(one_bytes, tiles):
    """a copy of a .one file image with BLOCK_INFO_S.cuda_gemm_tile_{m,n,k} of its header set to `tiles`"""
    buf = C.create_string_buffer(bytes(one_bytes), len(one_bytes))
    t = (C.c_int32 * 3)(*tiles)
    _check(load().onrt_one_set_tiles(buf, len(one_bytes), t), "onrt_one_set_tiles")
    return buf.raw


QUANT_KL, QUANT_MSE, QUANT_PERCENT = 0, 1, 2


def quantise(one_bytes, images, method=QUANT_KL, images2=None, op_lib_dir=None):
    """the W8A32 image of an fp32 .one model (onrt_one_quantise, the counterpart of tools/optimize/model_quant.hpp:625-679).
    images: calibration items, each a numpy array (one-input models) or a list of arrays in input order, or device
    addresses given as ints; images2: the items of the second pass of KL / MSE (default: the same ones)."""
    vp = C.c_void_p
    keep = []

    def pointers(items):
        flat = []
        for item in items:
            for a in (item if isinstance(item, (list, tuple)) else [item]):
                if isinstance(a, int):
                    flat.append(a)
                else:
                    a = np.ascontiguousarray(a, dtype=np.float32)
                    keep.append(a)
                    flat.append(a.ctypes.data)
        return (vp * len(flat))(*[vp(p) for p in flat])

    one_bytes = bytes(one_bytes)
    p1 = pointers(images)
    p2 = pointers(images2) if images2 is not None else None
    out = C.create_string_buffer(len(one_bytes))
    lib_dir = (op_lib_dir or os.path.dirname(lib_path())).encode()
    _check(load().onrt_one_quantise(one_bytes, len(one_bytes), lib_dir, int(method), p1, len(images), p2,
                                    len(images2) if images2 is not None else 0, out), "onrt_one_quantise")
    return out.raw


class Net:
    """A loaded model.  ``model`` is a path or the bytes of a .one file; ``op_lib_dir`` defaults to the directory
    of the built plugins."""

    def __init__(self, model, op_lib_dir=None, plan_only=False):
        """plan_only: the host-side half only (order, shapes, folding) -- needs no GPU, cannot run"""
        L = load()
        self._h = C.c_void_p()
        d = (op_lib_dir or os.path.dirname(lib_path())).encode()
        if plan_only:
            data = bytes(model) if isinstance(model, (bytes, bytearray, memoryview)) else open(os.fspath(model), "rb").read()
            _check(L.onrt_net_plan_buf(data, len(data), C.byref(self._h)), "onrt_net_plan_buf")
        elif isinstance(model, (bytes, bytearray, memoryview)):
            data = bytes(model)
            _check(L.onrt_net_load_buf(data, len(data), d, C.byref(self._h)), "onrt_net_load_buf")
        else:
            _check(L.onrt_net_load_file(os.fspath(model).encode(), d, C.byref(self._h)), "onrt_net_load_file")
        ni, no = C.c_int32(), C.c_int32()
        _check(L.onrt_net_io_count(self._h, C.byref(ni), C.byref(no)), "onrt_net_io_count")
        self.inputs = [self._io(0, i) for i in range(ni.value)]
        self.outputs = [self._io(1, i) for i in range(no.value)]

    def _io(self, is_output, idx):
        name, nd, shape = C.c_char_p(), C.c_int32(), (C.c_int32 * 8)()
        _check(load().onrt_net_io_info(self._h, is_output, idx, C.byref(name), C.byref(nd), shape), "onrt_net_io_info")
        return name.value.decode(), tuple(shape[i] for i in range(nd.value))

    def ops(self):
        """(type, name) of every operator in execution order"""
        L, n = load(), C.c_int32()
        _check(L.onrt_net_op_count(self._h, C.byref(n)), "onrt_net_op_count")
        out = []
        for i in range(n.value):
            t, nm = C.c_char_p(), C.c_char_p()
            _check(L.onrt_net_op_info(self._h, i, C.byref(t), C.byref(nm)), "onrt_net_op_info")
            out.append((t.value.decode(), nm.value.decode()))
        return out

    def fused_blocks(self):
        """number of Conv -> Add (-> Relu) groups the loader folded into one call"""
        n = C.c_int32()
        _check(load().onrt_net_fused_count(self._h, C.byref(n), None), "onrt_net_fused_count")
        return n.value

    def graph_launches(self):
        """runs so far that replayed the recorded HIP graph of the net"""
        n = C.c_int64()
        _check(load().onrt_net_graph_launches(self._h, C.byref(n)), "onrt_net_graph_launches")
        return n.value

    def folded_activations(self):
        """number of Conv nodes that took a Clip / LeakyRelu / Sigmoid x Mul / HardSigmoid x Mul after them as act_type"""
        n = C.c_int32()
        _check(load().onrt_net_folded_activations(self._h, C.byref(n)), "onrt_net_folded_activations")
        return n.value

    def fused_attentions(self):
        """number of MatMul -> Softmax -> MatMul blocks (with the Transpose of k) that run as one attention call"""
        n = C.c_int32()
        _check(load().onrt_net_fused_attentions(self._h, C.byref(n)), "onrt_net_fused_attentions")
        return n.value

    def fused_linears(self):
        """number of MatMul -> Add of a bias (-> Gelu) groups that run as one call"""
        n = C.c_int32()
        _check(load().onrt_net_fused_linears(self._h, C.byref(n)), "onrt_net_fused_linears")
        return n.value

    def fused_skips(self):
        """number of those groups that also take in the Add of a skip connection after them"""
        n = C.c_int32()
        _check(load().onrt_net_fused_skips(self._h, C.byref(n)), "onrt_net_fused_skips")
        return n.value

    def fused_ir_blocks(self):
        """number of Conv (1x1) -> depthwise Conv -> Conv (1x1) [-> Add] blocks that run as one call"""
        n = C.c_int32()
        _check(load().onrt_net_fused_ir_blocks(self._h, C.byref(n)), "onrt_net_fused_ir_blocks")
        return n.value

    def fused_pairs(self):
        """number of Conv -> Conv (1x1) [-> Add [-> Relu]] pairs that run as one call"""
        n = C.c_int32()
        _check(load().onrt_net_fused_pairs(self._h, C.byref(n)), "onrt_net_fused_pairs")
        return n.value

    def int8_links(self):
        """number of operands between int8 convolutions that travel as int8 NHWC instead of fp32"""
        n = C.c_int32()
        _check(load().onrt_net_quantised_links(self._h, C.byref(n)), "onrt_net_quantised_links")
        return n.value

    def folded_relus(self):
        """number of Relu nodes folded into the Conv in front of them (act_type RELU, as the offline optimiser does)"""
        n = C.c_int32()
        _check(load().onrt_net_fused_count(self._h, None, C.byref(n)), "onrt_net_fused_count")
        return n.value

    def tiles(self):
        """the model-wide GEMM tile (m, n, k) the net runs with: BLOCK_INFO_S.cuda_gemm_tile_* of its file, or what
        tune_tiles / set_tiles left"""
        t = (C.c_int32 * 3)()
        _check(load().onrt_net_get_tiles(self._h, t), "onrt_net_get_tiles")
        return tuple(t)

    def set_tiles(self, tiles):
        t = (C.c_int32 * 3)(*tiles)
        _check(load().onrt_net_set_tiles(self._h, t), "onrt_net_set_tiles")

    def tune_tiles(self, reps=5):
        """measures the net with every workgroup tile of the Conv plugin's library and with none; leaves the fastest
        set and returns (tiles, ms with it, ms with the converter's default)"""
        t, best, deflt = (C.c_int32 * 3)(), C.c_float(), C.c_float()
        _check(load().onrt_net_tune_tiles(self._h, reps, t, C.byref(best), C.byref(deflt)), "onrt_net_tune_tiles")
        return tuple(t), best.value, deflt.value

    def operand(self, name):
        """(shape, device address) of an operand"""
        nd, shape, ptr = C.c_int32(), (C.c_int32 * 8)(), C.c_void_p()
        _check(load().onrt_net_operand(self._h, name.encode(), C.byref(nd), shape, C.byref(ptr)), "onrt_net_operand")
        return tuple(shape[i] for i in range(nd.value)), ptr.value

    def fetch(self, name):
        """host copy of an operand's current contents (fp32)"""
        shape, ptr = self.operand(name)
        n = int(np.prod(shape)) if shape else 1
        out = np.empty(n, dtype=np.float32)
        rt = C.CDLL("libamdhip64.so")
        rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        rc = rt.hipMemcpy(out.ctypes.data, ptr, out.nbytes, 2)   # blocking device-to-host copy
        if rc != 0:
            raise OnrtError(f"hipMemcpy of operand {name} failed ({rc})")
        return out.reshape(shape)

    def run_raw(self, in_ptrs, out_ptrs):
        """addresses (host or device) in input / output order; 0 / None among the outputs skips that copy"""
        vp = C.c_void_p
        ins = (vp * max(1, len(in_ptrs)))(*[vp(p) for p in in_ptrs])
        outs = (vp * max(1, len(out_ptrs)))(*[vp(p or 0) for p in out_ptrs])
        _check(load().onrt_net_run(self._h, ins, outs), "onrt_net_run")

    def enqueue_raw(self, in_ptrs, out_ptrs):
        """run_raw without the wait at the end: device addresses only, results complete when the default stream is"""
        vp = C.c_void_p
        ins = (vp * max(1, len(in_ptrs)))(*[vp(p) for p in in_ptrs])
        outs = (vp * max(1, len(out_ptrs)))(*[vp(p or 0) for p in out_ptrs])
        _check(load().onrt_net_enqueue(self._h, ins, outs), "onrt_net_enqueue")

    def run(self, *arrays):
        """numpy inputs in input order -> list of numpy outputs"""
        if len(arrays) != len(self.inputs):
            raise OnrtError(f"the net has {len(self.inputs)} inputs, {len(arrays)} given")
        ins = []
        for a, (name, shape) in zip(arrays, self.inputs):
            a = np.ascontiguousarray(a, dtype=np.float32)
            if a.size != int(np.prod(shape)):
                raise OnrtError(f"input {name} has shape {shape}, got {a.shape}")
            ins.append(a)
        outs = [np.empty(shape, dtype=np.float32) for _, shape in self.outputs]
        self.run_raw([a.ctypes.data for a in ins], [o.ctypes.data for o in outs])
        return outs

    def close(self):
        if self._h:
            load().onrt_net_free(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
