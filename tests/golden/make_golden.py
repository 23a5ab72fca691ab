"""Writes tests/golden/golden.npz and the two activation tables from the reference's own x86
kernels, compiled in place by `make -C oracle ref` (outputs in oracle/_ref).  Runs only where the
reference sources are mounted; the fixtures it writes are committed.

    python tests/golden/make_golden.py

For every case of tests/golden/cases.py the reference `eval` is called through the same slot
arrays the oneNew host fills (onenew_amd.ops) and the output is summarised by cases.summarize."""
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)
import cases  # noqa: E402
from onenew_amd import abi, ops  # noqa: E402
from oracle import oracle  # noqa: E402


def main():
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "ref"])
    ref = os.path.join(ROOT, "oracle", "_ref")
    subprocess.check_call([os.path.join(ref, "lutdump"), cases.SILU_LUT, cases.GELU_LUT])
    silu, gelu = cases.silu_lut(), cases.gelu_lut()
    conv = ops.Plugin(oracle.ref_path("Conv"))
    matmul = ops.Plugin(oracle.ref_path("MatMul"))
    gemm = ops.Plugin(oracle.ref_path("Gemm"))
    gelu_so = ops.Plugin(os.path.join(ref, "libGelu_x86.so"))
    out = {}

    def put(name, tensor):
        for k, v in cases.summarize(name, tensor).items():
            out[f"{name}/{k}"] = v

    for name, d in cases.conv_f32_cases().items():
        x, w, b = cases.conv_inputs(name, d)
        op = ops.Conv(conv.eval, d, w, b, silu_lut=silu, scratch_bytes=oracle.ref_scratch_bytes(d))
        put(name, op(x))
        print("conv f32", name, flush=True)
    for name, d in cases.conv_w8a32_cases().items():
        x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
        op = ops.Conv(conv.eval, d, w8, b32, weight_aux=aux, silu_lut=silu, scratch_bytes=oracle.ref_scratch_bytes(d))
        xin = ops.aligned_empty(x.shape)
        xin[...] = x
        put(name, op(xin))
        print("conv w8a32", name, flush=True)
    for name, (ash, bsh) in cases.matmul_cases().items():
        a, b = cases.matmul_inputs(name, ash, bsh)
        aa, bb = ops.aligned_empty(a.shape), ops.aligned_empty(b.shape)
        aa[...], bb[...] = a, b
        put(name, ops.MatMul(matmul.eval)(aa, bb))
        print("matmul", name, flush=True)
    for name, (M, K, N) in cases.gemm_cases().items():
        a, w, b = cases.gemm_inputs(name, M, K, N)
        put(name, ops.Gemm(gemm.eval, w, b)(a))
        print("gemm", name, flush=True)
    # the operators around the convolutions: Add, Relu, MaxPool, GlobalAveragePool
    add = ops.Plugin(os.path.join(ref, "libAdd_x86.so"))
    relu = ops.Plugin(os.path.join(ref, "libRelu_x86.so"))
    maxpool = ops.Plugin(os.path.join(ref, "libMaxPool_x86.so"))
    gap = ops.Plugin(os.path.join(ref, "libGlobalAveragePool_x86.so"))
    for name, (s0, s1) in cases.add_cases().items():
        a, b = cases.add_inputs(name, s0, s1)
        put(name, ops.Add(add.eval)(a, b))
        print("add", name, flush=True)
    for name, shape in cases.relu_cases().items():
        xin = ops.aligned_empty(shape)
        xin[...] = cases.relu_input(name, shape)
        put(name, ops.Relu(relu.eval)(xin))
        print("relu", name, flush=True)
    for name, (shape, k, st, pad) in cases.maxpool_cases().items():
        x = cases.maxpool_input(name, shape)
        scratch = 4 * x.size * 4 + (1 << 20)
        put(name, ops.MaxPool(maxpool.eval, k, st, pad, scratch_bytes=scratch)(x))
        print("maxpool", name, flush=True)
    for name, shape in cases.gap_cases().items():
        put(name, ops.GlobalAveragePool(gap.eval)(cases.gap_input(name, shape)))
        print("gap", name, flush=True)
    # the operators around the MatMuls: LayerNormalization, Softmax, Transpose
    ln = ops.Plugin(os.path.join(ref, "libLayerNormalization_x86.so"))
    sm = ops.Plugin(os.path.join(ref, "libSoftmax_x86.so"))
    tr = ops.Plugin(os.path.join(ref, "libTranspose_x86.so"))
    for name, (shape, axis) in cases.layernorm_cases().items():
        x, w, b = cases.layernorm_inputs(name, shape, axis)
        put(name, ops.LayerNormalization(ln.eval, w, b, axis)(x))
        print("layernorm", name, flush=True)
    for name, (shape, axis) in cases.softmax_cases().items():
        put(name, ops.Softmax(sm.eval, axis)(cases.softmax_input(name, shape)))
        print("softmax", name, flush=True)
    for name, (shape, perm) in cases.transpose_cases().items():
        put(name, ops.Transpose(tr.eval, perm)(cases.transpose_input(name, shape)))
        print("transpose", name, flush=True)
    # table GELU (device/x86/Gelu/gelu.c) on edge values
    x = cases.gelu_input()
    params = (abi.BUFFER_INFO_S * abi.BUF_MAXNUM)()
    inputs = (abi.BUFFER_INFO_S * abi.BUF_MAXNUM)()
    outputs = (abi.BUFFER_INFO_S * abi.BUF_MAXNUM)()
    cfg = abi.MATMUL_CONFIG_S()          # GELU_CONFIG_S is a bare BASE_CONFIG_S as well
    operand = ops.make_operand(x.shape)
    y = np.empty_like(x)
    import ctypes as C
    params[0].addr, params[1].addr = C.addressof(cfg), C.addressof(operand)
    inputs[0].addr, inputs[abi.BUF_MAXNUM - 1].addr = x.ctypes.data, gelu.ctypes.data
    outputs[0].addr = y.ctypes.data
    gelu_so.eval(params, inputs, outputs)
    put("gelu_edges", y)
    np.savez_compressed(cases.GOLDEN_NPZ, **out)
    print("wrote", cases.GOLDEN_NPZ, os.path.getsize(cases.GOLDEN_NPZ), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
