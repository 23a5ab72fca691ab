"""CPU checks of the .one file path: the writer against the reference's own reader (its host operator classes,
compiled into oracle/_ref/ref_run_one), the oracle's graph executor against the reference's x86 kernels run by
those classes, and the loader's error paths (which end before any device call)."""
import ctypes as C
import os
import re
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, ROOT)
from oracle import one_model  # noqa: E402
import one_models  # noqa: E402
from onenew_amd import abi, onefile, rt  # noqa: E402

needs_ref = pytest.mark.skipif(not one_model.have_ref_runner(), reason="oracle/_ref/ref_run_one is not built")


@pytest.mark.parametrize("name", list(one_models.MODELS))
def test_writer_and_reader_round_trip(name):
    data, _ = one_models.MODELS[name]()
    m = onefile.parse(data)
    h = m["header"]
    assert h.one_model_magic_num == 0x6F6E65 and len(data) % 64 == 0
    assert h.node_cfg_offset == 128 and h.node_cfg_offset < h.init_info_offset <= h.io_cfg_offset <= len(data)
    assert h.useful_info.public_buf_info.public_buf_size == 512 * 1024 * 1024     # onnx2one.cpp:1332-1336
    assert len(m["nodes"]) == h.node_cnt and len(m["inits"]) == h.init_cnt
    assert len(m["inputs"]) + len(m["outputs"]) == h.io_cfg_cnt
    for op_type, cfg in m["nodes"]:
        b = cfg.op_base_cfg
        assert b.op_type.decode() == op_type and 1 <= b.in_operand_num <= 8 and b.out_operand_num == 1
        # every node but the first of a chain has a producer, every output is consumed (onnx2one.cpp:1117-1227)
        assert b.consumer_num >= 1


@needs_ref
@pytest.mark.parametrize("name", list(one_models.MODELS))
def test_oracle_executor_matches_reference_host_classes(name):
    """the same file through the reference's fill_operands / shape_infer / rt_prepare / forward and x86 kernels:
    shapes and values of every output are identical to the oracle executor's, bit for bit"""
    data, ins = one_models.MODELS[name]()
    mine = one_model.run(data, ins)
    ref = one_model.run_reference(data, ins)
    names = [n for n, _ in onefile.parse(data)["outputs"]]
    assert [n for n, _ in ref] == names
    for a, (n, b) in zip(mine, ref):
        assert a.shape == b.shape, n
        assert np.array_equal(a, b), n


def test_flatten_and_reshape_are_views():
    m = onefile.OneModel()
    m.input("x", (1, 4, 3, 2))
    m.flatten("f", "x", "f_out", axis=1)
    m.reshape("r", "f_out", "r_out", (1, 2, -1))
    m.relu("relu", "r_out", "y")
    m.output("y", (1, 2, 12))
    x = np.arange(-12, 12, dtype=np.float32).reshape(1, 4, 3, 2)
    (y,) = one_model.run(m.tobytes(), [x])
    assert y.shape == (1, 2, 12) and np.array_equal(y.reshape(-1), np.maximum(x, 0).reshape(-1))
    if one_model.have_ref_runner():
        (n, ref), = one_model.run_reference(m.tobytes(), [x])
        assert ref.shape == (1, 2, 12) and np.array_equal(ref, y)


def test_runtime_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "onenew_rt.h")).read()
    declared = sorted(set(re.findall(r"\b(onrt_[a-z_]+)\s*\(", header)))
    assert declared == sorted(rt.EXPORTS)
    lib = C.CDLL(rt.lib_path())
    for sym in declared:
        assert hasattr(lib, sym), sym


def _load_error(data):
    L = rt.load()
    h = C.c_void_p()
    rc = L.onrt_net_load_buf(bytes(data), len(data), b"/nonexistent", C.byref(h))
    assert not h.value
    return rc, L.onrt_last_error().decode()


def test_loader_rejects_what_is_not_a_model():
    data, _ = one_models.resnet_block()
    rc, msg = _load_error(b"\0" * 64)
    assert rc == -2 and "shorter than the header" in msg
    bad = bytearray(data)
    bad[0] ^= 0xFF
    rc, msg = _load_error(bad)
    assert rc == -2 and "magic" in msg
    rc, msg = _load_error(data[:len(data) // 2])
    assert rc == -2 and "past the end" in msg


def test_loader_rejects_an_operator_without_a_plugin():
    data, _ = one_models.resnet_block()
    m = onefile.parse(data)
    bad = bytearray(data)
    off = m["header"].node_cfg_offset
    bad[off:off + 8] = b"Einsum\0\0"
    rc, msg = _load_error(bad)
    assert rc == -2 and "Einsum" in msg


def test_loader_reports_a_missing_plugin_directory():
    data, _ = one_models.two_inputs()
    rc, msg = _load_error(data)
    assert rc == -3 and "not found" in msg and "/nonexistent/Add/libAdd_hip.so" in msg


def test_loader_rejects_damaged_descriptors():
    """ranks and extents no tensor can have are refused before anything is indexed with them"""
    import ctypes
    data, _ = one_models.resnet_block()
    m = onefile.parse(data)
    io_off = m["header"].io_cfg_offset + 512                     # OPERAND_S of the first io config (the input)
    for field, value, word in (("dim_num_of_shapes", 100, "rank"), ("dim_num_of_shapes", 0, "rank"), ("shapes", -3, "elements")):
        bad = bytearray(data)
        pos = io_off + getattr(abi.OPERAND_S, field).offset
        bad[pos:pos + 4] = int(value & 0xffffffff).to_bytes(4, "little")
        rc, msg = _load_error(bad)
        assert rc == -2 and word in msg, (field, value, msg)
    view = onefile.OneModel()
    view.input("x", (1, 4, 3, 2))
    view.reshape("r", "x", "y", (1, 0, 24))
    view.relu("relu", "y", "z")
    view.output("z", (1, 1, 24))
    rc, msg = _load_error(view.tobytes())
    assert rc == -2 and "Reshape" in msg

