"""GPU parity of the device-resident model runtime (include/onenew_rt.h): .one models through libonenew_rt.so and
the HIP operator plugins against the oracle's CPU execution of the same file (itself pinned, bit for bit, against
the reference's host classes and x86 kernels in tests/test_one_model_cpu.py).

Tolerances: a chain that contains Conv / MatMul / Gemm accumulates in a different order than the CPU, fp32
relative 1e-4 of the output's largest magnitude per operator it passes through (stated per test); chains of the
exact operators (Add, Relu, MaxPool, Transpose, views) are bit-exact."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle import one_model  # noqa: E402
import one_models  # noqa: E402
from onenew_amd import hip, onefile, rt  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    hip.init(0)
    return torch


def _close(got, ref, rel):
    scale = max(float(np.abs(ref).max()), 1e-6)
    return float(np.abs(got - ref).max()) <= rel * scale


@pytest.mark.parametrize("name", list(one_models.MODELS))
def test_model_outputs_match_oracle(name, torch_dev):
    data, ins = one_models.MODELS[name]()
    net = rt.Net(data)
    m = onefile.parse(data)
    assert [n for n, _ in net.inputs] == [n for n, _ in m["inputs"]]
    assert net.outputs == [(n, tuple(s)) for n, s in m["outputs"]]          # inferred shapes equal the declared ones
    ref = one_model.run(data, ins, keep_all=True)
    outs = net.run(*ins)
    for (oname, _), got in zip(net.outputs, outs):
        assert got.shape == ref[oname].shape
        assert _close(got, ref[oname], 5e-4), oname                          # up to five MFMA operators deep, 1e-4 each
        if name == "quantised_block":
            assert np.array_equal(got, ref[oname])                           # integer accumulation: the chain is exact
    # every intermediate operand sits in device memory and holds what the oracle computed at that point
    for op_type, cfg in m["nodes"]:
        oname = cfg.op_base_cfg.out_operand_name[0].value.decode()
        shape, ptr = net.operand(oname)
        assert ptr and int(np.prod(shape)) == ref[oname].size
        assert _close(net.fetch(oname).reshape(ref[oname].shape), ref[oname], 5e-4), (op_type, oname)
    # the order is a topological one with as many operators as nodes, views included
    assert sorted(t for t, _ in net.ops()) == sorted(t for t, _ in m["nodes"])
    net.close()


def test_exact_operators_are_bit_exact_through_the_runtime(torch_dev):
    m = onefile.OneModel()
    m.input("a", (1, 6, 9, 9))
    m.input("b", (1, 6, 9, 9))
    m.add("sum", "a", "b", "s")
    m.relu("relu", "s", "r")
    m.maxpool("pool", "r", "p", 3, 2, 1)
    m.transpose("tr", "p", "t", (0, 2, 3, 1))
    m.flatten("fl", "t", "f", axis=1)
    m.output("f", (1, 150))
    data = m.tobytes()
    rng = np.random.default_rng(5)
    ins = [rng.normal(size=(1, 6, 9, 9)).astype(np.float32) for _ in range(2)]
    (ref,) = one_model.run(data, ins)
    net = rt.Net(data)
    (got,) = net.run(*ins)
    assert got.shape == (1, 150) and np.array_equal(got, ref)
    # a view shares its input's buffer (host/op.h:149-154)
    assert net.operand("f")[1] == net.operand("t")[1]


def test_second_run_and_device_pointers(torch_dev):
    """buffers are reused between runs; inputs and outputs may be device memory"""
    torch = torch_dev
    data, ins = one_models.resnet_block()
    net = rt.Net(data)
    (first,) = net.run(*ins)
    x2 = (ins[0] * np.float32(-0.5) + np.float32(0.25)).astype(np.float32)
    (ref2,) = one_model.run(data, [x2])
    xd = torch.from_numpy(x2).cuda()
    yd = torch.empty((1, 10), dtype=torch.float32, device="cuda")
    net.run_raw([xd.data_ptr()], [yd.data_ptr()])
    assert _close(yd.cpu().numpy(), ref2, 5e-4)
    (again,) = net.run(*ins)
    assert np.array_equal(again, first)                                      # same input, same kernels, same bits
    # output left in place: read it through the operand table
    net.run_raw([xd.data_ptr()], [None])
    assert _close(net.fetch("logits"), ref2, 5e-4)


def test_batched_input_keeps_its_batch(torch_dev):
    """the reference host fixes Conv and GlobalAveragePool outputs to batch 1; this runtime carries the input's batch
    through (the plugins already take it from the operand descriptor), image by image equal to batch-1 runs"""
    m = onefile.OneModel()
    rng = np.random.default_rng(11)
    m.input("x", (3, 4, 10, 10))
    m.conv("c", "x", rng.normal(size=(8, 4, 3, 3)).astype(np.float32) * 0.2, rng.normal(size=8).astype(np.float32), "y",
           pad=1, act=1)
    m.global_avgpool("g", "y", "z")
    m.output("z", (3, 8, 1, 1))
    x = rng.normal(size=(3, 4, 10, 10)).astype(np.float32)
    net = rt.Net(m.tobytes())
    assert net.outputs == [("z", (3, 8, 1, 1))]
    (z,) = net.run(x)
    ref = one_model.run(m.tobytes(), [x])[0]
    assert _close(z, ref, 2e-4)


def test_plugin_lookup_prefers_the_per_operator_directory(torch_dev, tmp_path):
    """host/op.h:41-80 looks in <dir>/<Op>/lib<Op>_x86.so; here <dir>/<Op>/lib<Op>_hip.so, then <dir>/lib<Op>_hip.so"""
    libdir = os.path.dirname(rt.lib_path())
    (tmp_path / "Relu").mkdir()
    os.symlink(os.path.join(libdir, "libRelu_hip.so"), tmp_path / "Relu" / "libRelu_hip.so")
    os.symlink(os.path.join(libdir, "libAdd_hip.so"), tmp_path / "libAdd_hip.so")
    m = onefile.OneModel()
    m.input("a", (1, 2, 3, 3))
    m.add("sum", "a", "a", "s")
    m.relu("relu", "s", "r")
    m.output("r", (1, 2, 3, 3))
    a = np.linspace(-1, 1, 18, dtype=np.float32).reshape(1, 2, 3, 3)
    net = rt.Net(m.tobytes(), op_lib_dir=str(tmp_path))
    assert np.array_equal(net.run(a)[0], np.maximum(a + a, 0))


@pytest.mark.parametrize("model", ["resnet50", "mobilenetv2"])
def test_whole_model_matches_the_reference_host_run(model, torch_dev):
    """the full-size network at batch 1 (89 / 65 operators) through the runtime against the same file run by the
    reference's host operator classes and x86 kernels on the CPU: logits within 1e-3 of their largest magnitude
    (53 / 52 convolutions deep with fp32 sums in another order), same top-5 classes"""
    from onenew_amd import stacks
    if not one_model.have_ref_runner():
        pytest.skip("oracle/_ref/ref_run_one is not built")
    make = stacks.resnet50_model if model == "resnet50" else stacks.mobilenet_v2_model
    data, shape, _ = make(1)
    x = np.random.default_rng(3).normal(size=shape).astype(np.float32)
    (_, ref), = one_model.run_reference(data, [x])
    net = rt.Net(data)
    (got,) = net.run(x)
    assert got.shape == ref.shape == (1, 1000)
    assert np.isfinite(got).all()
    assert _close(got, ref, 1e-3)
    assert set(np.argsort(got[0])[-5:]) == set(np.argsort(ref[0])[-5:])

