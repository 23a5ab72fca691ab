"""CPU checks of the boundary: struct layouts, exported symbols, slot filling, shape tables."""
import ctypes as C
import os
import re
import sys

import numpy as np

from onenew_amd import abi, hip, ops, stacks, datagen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_struct_layout_matches_reference_abi():
    abi.check_layout()
    # offsets a plugin reads (common/nn_common.h:222-243, probed with gcc on x86-64)
    assert abi.CONV_CONFIG_S.clip_min.offset == 12956 and abi.CONV_CONFIG_S.clip_max.offset == 12960
    assert abi.CONV_CONFIG_S.leaky_relu_alpha.offset == 12964
    assert abi.CONV_CONFIG_S.hard_sigmoid_alpha.offset == 12968 and abi.CONV_CONFIG_S.hard_sigmoid_beta.offset == 12972
    assert abi.CONV_CONFIG_S.output_scale.offset == 12984
    assert abi.GEMM_CONFIG_S.has_bias.offset == 12840 and abi.GEMM_CONFIG_S.alpha.offset == 12844
    assert abi.OPERAND_S.p_data.offset == 264 and abi.OPERAND_S.dim_num_of_shapes.offset == 272


def test_c_header_compiles_with_its_static_asserts(tmp_path):
    import subprocess
    src = tmp_path / "t.c"
    src.write_text('#include "onenew_hip.h"\nint main(void) { return sizeof(onhip_conv_desc_t) == 100 ? 0 : 1; }\n')
    exe = tmp_path / "t"
    subprocess.check_call(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    assert subprocess.call([str(exe)]) == 0
    subprocess.check_call(["g++", "-std=c++14", "-x", "c++", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])


def test_library_exports_every_declared_symbol():
    """every function include/onenew_hip.h declares is exported by libonenew_hip.so; each plugin exports eval"""
    text = open(os.path.join(ROOT, "include", "onenew_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(onhip_\w+)\s*\(", text))
    assert {"onhip_conv2d_f32", "onhip_conv2d_w8a32", "onhip_matmul", "onhip_gemm_f32", "onhip_conv_eval"} <= declared
    lib = hip.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared but not exported"
    assert declared == set(hip.EXPORTS), declared ^ set(hip.EXPORTS)
    for op in ("Conv", "MatMul", "Gemm"):
        assert ops.Plugin(hip.plugin_path(op)).eval is not None


def test_errors_without_gpu_are_codes_not_crashes():
    """argument errors are detected before any device work, so they can be checked on a CPU-only machine"""
    lib = hip.load()
    d = abi.ConvDesc(n=1, cin=4, h=8, w=8, cout=4, kh=3, kw=3, stride_h=0, stride_w=1, group=1, has_bias=1)
    oh, ow = C.c_int32(), C.c_int32()
    assert lib.onhip_conv_out_shape(C.byref(d), C.byref(oh), C.byref(ow)) == -1
    assert b"bad geometry" in lib.onhip_last_error()
    d.stride_h = 1
    d.pad_t = d.pad_l = d.pad_b = d.pad_r = 1
    assert lib.onhip_conv_out_shape(C.byref(d), C.byref(oh), C.byref(ow)) == 0 and (oh.value, ow.value) == (8, 8)
    d.group, d.cout = 4, 8       # depthwise needs cin == cout
    assert lib.onhip_conv_out_shape(C.byref(d), C.byref(oh), C.byref(ow)) == -1
    # tap-major [cout][taps][channels padded to 4] ...
    assert lib.onhip_conv2d_packed_weight_bytes(C.byref(abi.ConvDesc(n=1, cin=5, h=8, w=8, cout=8, kh=7, kw=7, stride_h=2,
                                                                      stride_w=2, group=1, has_bias=1))) == 8 * 49 * 8 * 4
    # ... except a first layer (three input channels, 7x7 or 3x3): [3 * taps rounded up to even][64], the layout of its kernel
    assert lib.onhip_conv2d_packed_weight_bytes(C.byref(abi.ConvDesc(n=1, cin=3, h=8, w=8, cout=8, kh=7, kw=7, stride_h=2,
                                                                      stride_w=2, group=1, has_bias=1))) == 148 * 64 * 4
    one = abi.ConvDesc(n=1, cin=8, h=8, w=8, cout=8, kh=1, kw=1, stride_h=1, stride_w=1, group=1, has_bias=1)
    assert lib.onhip_conv2d_packed_weight_bytes(C.byref(one)) == 0
    assert lib.onhip_conv_eval(None, None, None) == -1


def test_conv_operator_fills_slots_like_the_reference_host():
    """host/ops/conv.h:60-157 and host/op.h:109-168: where each descriptor and buffer goes"""
    seen = {}

    @ops.EVAL_T
    def fake_eval(params, inputs, outputs):
        cfg = C.cast(params[0].addr, C.POINTER(abi.CONV_CONFIG_S)).contents
        seen["has_bias"], seen["group"], seen["act"] = cfg.has_bias, cfg.group, cfg.act_type
        seen["pads"] = list(cfg.pads)
        seen["in"] = list(C.cast(params[1].addr, C.POINTER(abi.OPERAND_S)).contents.shapes)
        seen["w"] = list(C.cast(params[2].addr, C.POINTER(abi.OPERAND_S)).contents.shapes)
        seen["out"] = list(C.cast(params[4].addr, C.POINTER(abi.OPERAND_S)).contents.shapes)
        seen["useful_magic"] = C.cast(params[11].addr, C.POINTER(abi.USEFUL_INFO_S)).contents.useful_info_magic_num
        seen["x0"] = C.cast(inputs[0].addr, C.POINTER(C.c_float))[0]
        seen["lut"] = inputs[11].addr != 0
        C.cast(outputs[0].addr, C.POINTER(C.c_float))[0] = 42.0
        return 0

    d = abi.ConvDesc(n=1, cin=3, h=10, w=12, cout=5, kh=3, kw=3, stride_h=2, stride_w=2, pad_t=1, pad_l=1, pad_b=0,
                     pad_r=0, group=1, has_bias=1, act_type=abi.SILU)
    op = ops.Conv(fake_eval, d, np.zeros((5, 3, 3, 3), np.float32), np.zeros(5, np.float32))
    x = np.full((1, 3, 10, 12), 7.0, np.float32)
    y = op(x)
    assert seen == {"has_bias": 1, "group": 1, "act": abi.SILU, "pads": [1, 1, 0, 0], "in": [1, 3, 10, 12, 1, 1, 1, 1],
                    "w": [5, 3, 3, 3, 1, 1, 1, 1], "out": [1, 5, 5, 6, 1, 1, 1, 1], "useful_magic": 45678, "x0": 7.0,
                    "lut": True}
    assert y.shape == (1, 5, 5, 6) and y.reshape(-1)[0] == 42.0


def test_int8_weights_are_packed_at_the_front_of_the_float_buffer():
    """tools/optimize/model_quant.hpp:14-25: int8 weights in place, int32 bias in the fp32 bias buffer"""
    d = abi.ConvDesc(n=1, cin=2, h=4, w=4, cout=3, kh=1, kw=1, stride_h=1, stride_w=1, group=1, has_bias=1, input_scale=0.1)
    w8 = np.arange(-3, 3, dtype=np.int8).reshape(3, 2, 1, 1)
    op = ops.Conv(lambda *a: 0, d, w8, np.array([1, -2, 3], np.int32), weight_aux=np.ones(3, np.float32))
    assert op.conv_cfg.ifmap_quant2 == abi.TYPE_INT8 and abs(op.conv_cfg.input_scale - 0.1) < 1e-7
    assert list(op.weight.reshape(-1).view(np.int8)[:6]) == [-3, -2, -1, 0, 1, 2]
    assert list(op.bias.view(np.int32)) == [1, -2, 3] and op.conv_cfg.weight_aux[2] == 1.0


def test_layer_tables_match_published_counts():
    r = stacks.resnet50()
    assert len(r) == 53
    # 8174.3 MFLOP per image: sum of the Conv rows of tools/perf_profiling/timeline_info/resnet50.csv
    assert abs(sum(d.flops() for _, d in r) / 1e6 - 8174.27) < 0.01
    assert r[2][1].flops() == 231211008          # Conv2d+ReLU 64->64 56x56 3x3, batch 1: 2 * 64 * 56 * 56 * 64 * 9
    m = stacks.mobilenet_v2()
    assert len(m) == 52 and sum(1 for _, d in m if d.group != 1) == 17
    assert len(stacks.yolov8s()) == 63
    assert [n for n, *_ in stacks.vit_tiny()] == ["qkv", "scores", "context", "proj", "fc1", "fc2"]
    assert stacks.with_batch(r, 32)[0][1].n == 32 and r[0][1].n == 1


def test_datagen_is_deterministic_and_distributed():
    a = datagen.uniform(datagen.seed_for("t", 1, "x"), (1000,))
    b = datagen.uniform(datagen.seed_for("t", 1, "x"), (1000,))
    assert np.array_equal(a, b) and a.min() >= -1 and a.max() <= 1
    assert a[:3].tolist() == datagen.uniform(datagen.seed_for("t", 1, "x"), (3,)).tolist()   # counter-based
    z = datagen.normal(7, (200000,), 0.0, 2.0)
    assert abs(z.mean()) < 0.02 and abs(z.std() - 2.0) < 0.02
    i = datagen.integers(9, (10000,), -127, 127)
    assert i.min() == -127 and i.max() == 127


def test_bench_refuses_more_than_one_gpu():
    """the benchmark measures one GPU; asked for more it says so and exits before touching a device"""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0
    assert "one GPU" in (res.stderr + res.stdout)

