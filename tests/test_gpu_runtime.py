"""GPU parity of the device-resident model runtime (include/onenew_rt.h): .one models through libonenew_rt.so and
the HIP operator plugins against the oracle's CPU execution of the same file (itself pinned, bit for bit, against
the reference's host classes and x86 kernels in tests/test_one_model_cpu.py).

Tolerances: a chain that contains Conv / MatMul / Gemm accumulates in a different order than the CPU, fp32
relative 1e-4 of the output's largest magnitude per operator it passes through (stated per test); chains of the
exact operators (Add, Relu, MaxPool, Transpose, views) are bit-exact."""
import ctypes as C
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle import one_model  # noqa: E402
import one_models  # noqa: E402
from onenew_amd import abi, hip, onefile, rt  # noqa: E402

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
def test_model_outputs_match_oracle(name, torch_dev, monkeypatch):
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")          # operator by operator, so that every operand can be compared
    data, ins = one_models.MODELS[name]()
    net = rt.Net(data)
    assert net.fused_blocks() == 0
    m = onefile.parse(data)
    assert [n for n, _ in net.inputs] == [n for n, _ in m["inputs"]]
    assert net.outputs == [(n, tuple(s)) for n, s in m["outputs"]]          # inferred shapes equal the declared ones
    ref = one_model.run(data, ins, keep_all=True)
    outs = net.run(*ins)
    for (oname, _), got in zip(net.outputs, outs):
        assert got.shape == ref[oname].shape
        assert _close(got, ref[oname], 5e-4), oname                          # up to five MFMA operators deep, 1e-4 each
        if name in ("quantised_block", "quantised_chain", "quantised_stem", "quantised_mobile"):
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


def test_weights_of_a_freed_net_are_forgotten(torch_dev):
    """nets of one shape with different weights, loaded and freed one after the other: the allocator hands the next
    net the address the last one's weights had, and the Conv plugin must not run it on the packed copy it kept of
    those"""
    for seed in range(4):
        rng = np.random.default_rng(100 + seed)
        m = onefile.OneModel()
        m.input("x", (1, 8, 10, 10))
        m.conv("c", "x", (rng.normal(size=(8, 8, 3, 3)) * 0.2).astype(np.float32), rng.normal(size=8).astype(np.float32),
               "y", pad=1)
        m.output("y", (1, 8, 10, 10))
        x = rng.normal(size=(1, 8, 10, 10)).astype(np.float32)
        net = rt.Net(m.tobytes())
        (y,) = net.run(x)
        assert _close(y, one_model.run(m.tobytes(), [x])[0], 2e-4), seed
        net.close()


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


def _both_ways(data, ins, monkeypatch):
    """outputs of the net loaded with residual blocks folded and with every operator separate"""
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    plain = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_FUSE")
    fused = rt.Net(data)
    return fused, plain, fused.run(*ins), plain.run(*ins)


def test_residual_block_is_folded_into_the_convolution(torch_dev, monkeypatch):
    """Conv -> Add -> Relu of the small ResNet block runs as one call of the Conv plugin: two operators fewer, the
    operands in between share the block's buffer, and the net's output has the same bits as operator by operator"""
    data, ins = one_models.resnet_block()
    fused, plain, got, want = _both_ways(data, ins, monkeypatch)
    assert plain.fused_blocks() == 0 and fused.fused_blocks() == 1
    assert len(fused.ops()) == len(plain.ops()) - 2
    assert [t for t, _ in fused.ops()].count("Add") == 0 and [t for t, _ in fused.ops()].count("Relu") == 0
    assert np.array_equal(got[0], want[0])
    assert fused.operand("c2_out")[1] == fused.operand("res_out")[1] == fused.operand("relu_out")[1]
    assert np.array_equal(fused.fetch("relu_out"), plain.fetch("relu_out"))
    (ref,) = one_model.run(data, ins)
    assert _close(got[0], ref, 5e-4)
    # a second run on another input: the folded call reads the addend afresh
    x2 = (ins[0] * np.float32(0.5) - np.float32(0.1)).astype(np.float32)
    assert np.array_equal(fused.run(x2)[0], plain.run(x2)[0])


def test_vit_encoder_through_the_runtime(torch_dev, monkeypatch):
    """a ViT-Tiny encoder (two of its twelve blocks) as a .one file: logits against the CPU restatement of the graph, with
    every attention block and every linear layer folded into one call each and with every operator on its own"""
    from onenew_amd import stacks
    data, shape, _ = stacks.vit_tiny_model(2, blocks=2)
    x = np.random.default_rng(5).normal(size=shape).astype(np.float32)
    ref = one_model.run(data, [x])[0]
    fused = rt.Net(data)
    assert fused.fused_attentions() == 2 and fused.fused_linears() == 12 and fused.fused_skips() == 4
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    plain = rt.Net(data)
    assert len(plain.ops()) == len(onefile.parse(data)["nodes"]) and len(fused.ops()) == len(plain.ops()) - 2 * 7 - 14 - 4
    for net in (fused, plain):
        got = net.run(x)[0]
        assert got.shape == ref.shape and _close(got, ref, 1e-3), float(np.abs(got - ref).max())
        assert np.array_equal(np.argsort(got, axis=1)[:, -5:], np.argsort(ref, axis=1)[:, -5:])
        net.close()


def test_linear_layers_run_as_one_call_bit_for_bit(torch_dev, monkeypatch):
    """MatMul -> Add of a bias -> Gelu, MatMul -> Add of a bias, and MatMul -> Add of a bias -> Add of a skip connection as
    one call each: the operands behind them hold exactly what the separate operators produce (the bias is added to the
    finished sum, the table is read with the same index, the skip tensor is added last)"""
    m = onefile.OneModel()
    rng = np.random.default_rng(3)
    w = lambda *s: (rng.normal(size=s) * 0.2).astype(np.float32)   # noqa: E731
    m.input("x", (2, 50, 48))
    m.matmul("fc1", "x", w(48, 96), "fc1_out")
    m.add("fc1_bias", "fc1_out", w(96), "fc1_b")
    m.gelu("act", "fc1_b", "act_out")
    m.matmul("fc2", "act_out", w(96, 40), "fc2_out")
    m.add("fc2_bias", "fc2_out", w(1, 1, 40), "fc2_b")                # leading axes of extent 1
    m.matmul("fc3", "fc2_b", w(40, 24), "fc3_out")
    m.add("not_a_bias", "fc3_out", w(2, 50, 24), "y")                 # a full tensor: stays an Add
    m.matmul("proj", "act_out", w(96, 48), "proj_out")
    m.add("proj_bias", "proj_out", w(48), "proj_b")
    m.add("skip", "x", "proj_b", "z")                                  # the block's input around it
    m.matmul("fc4", "z", w(48, 48), "fc4_out")
    m.add("fc4_bias", "fc4_out", w(48), "fc4_b")
    m.add("skip_with_two_readers", "fc4_b", "z", "z2")                 # fc4_b is also an output: that Add stays
    m.output("act_out", (2, 50, 96))
    m.output("y", (2, 50, 24))
    m.output("z", (2, 50, 48))
    m.output("fc4_b", (2, 50, 48))
    m.output("z2", (2, 50, 48))
    data, x = m.tobytes(), rng.normal(size=(2, 50, 48)).astype(np.float32)
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    plain = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_FUSE")
    fused = rt.Net(data)
    assert plain.fused_linears() == 0 and fused.fused_linears() == 4
    assert plain.fused_skips() == 0 and fused.fused_skips() == 1
    assert [t for t, _ in fused.ops()] == ["MatMul", "MatMul", "MatMul", "Add", "MatMul", "MatMul", "Add"]
    for got, ref in zip(fused.run(x), plain.run(x)):
        assert np.array_equal(got, ref)
    assert np.array_equal(fused.fetch("fc2_b"), plain.fetch("fc2_b"))
    assert fused.operand("fc1_out")[1] == fused.operand("fc1_b")[1] == fused.operand("act_out")[1]
    assert fused.operand("proj_out")[1] == fused.operand("proj_b")[1] == fused.operand("z")[1]
    # a second run on another input: the folded call reads the skip tensor afresh
    x2 = (x * np.float32(-0.5) + np.float32(0.1)).astype(np.float32)
    for got, ref in zip(fused.run(x2), plain.run(x2)):
        assert np.array_equal(got, ref)
    plain.close()
    fused.close()


def test_inverted_residual_blocks_run_as_one_call(torch_dev, monkeypatch):
    """Conv 1x1 -> depthwise Conv -> Conv 1x1 (-> Add) of two MobileNetV2-style blocks as one call of the Conv plugin's
    eval_block each, where the plugin recommends it (enough bands of rows over the batch): against the net run operator by
    operator within 1e-4 and against the CPU restatement of the graph; at a small batch the operators stay separate"""
    data, ins = one_models.inverted_residual_blocks(batch=16, size=32)
    fused, plain, got, want = _both_ways(data, ins, monkeypatch)
    assert plain.fused_ir_blocks() == 0 and fused.fused_ir_blocks() == 2
    assert [t for t, _ in fused.ops()] == ["Conv", "Conv"] and len(plain.ops()) == 7
    for name in ("e1_out", "d1_out", "e2_out", "d2_out"):
        assert fused.operand(name)[1] is None
    ref = one_model.run(data, ins)
    for g, w_, r in zip(got, want, ref):
        assert g.shape == w_.shape and np.all(np.abs(g - w_) <= 1e-4 * np.abs(w_) + 1e-5 * np.abs(w_).max())
        assert _close(g, r, 5e-4)
    x2 = [(ins[0] * np.float32(-0.7) + np.float32(0.2)).astype(np.float32)]
    for g, w_ in zip(fused.run(*x2), plain.run(*x2)):
        assert np.all(np.abs(g - w_) <= 1e-4 * np.abs(w_) + 1e-5 * np.abs(w_).max())
    fused.close()
    plain.close()
    small = rt.Net(one_models.inverted_residual_blocks(batch=1, size=32)[0])
    assert small.fused_ir_blocks() == 0 and len(small.ops()) == 6
    small.close()


def test_inferences_queued_without_a_wait(torch_dev, monkeypatch):
    """onrt_net_enqueue: the same inference queued on the default stream, no wait at its end.  Three of them back to back
    on the net's own buffers (nothing copied) and on caller tensors (copies queued in stream order) give the bits of
    onrt_net_run; host memory and a net with a stream of its own are refused"""
    torch = torch_dev
    data, ins = one_models.resnet_block()
    net = rt.Net(data)
    (want,) = net.run(*ins)
    x = torch.from_numpy(ins[0]).cuda()
    y = torch.zeros(want.shape, dtype=torch.float32, device="cuda")
    for _ in range(3):
        net.enqueue_raw([x.data_ptr()], [y.data_ptr()])
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), want)
    (_, in_dev), (_, out_dev) = net.operand(net.inputs[0][0]), net.operand(net.outputs[0][0])
    x2 = (ins[0] * np.float32(0.5) - np.float32(0.25)).astype(np.float32)
    (want2,) = net.run(x2)                       # leaves x2 in the net's input buffer
    for _ in range(3):
        net.enqueue_raw([in_dev], [out_dev])
    torch.cuda.synchronize()
    assert np.array_equal(net.fetch(net.outputs[0][0]).reshape(want2.shape), want2)
    with pytest.raises(rt.OnrtError):
        net.enqueue_raw([ins[0].ctypes.data], [y.data_ptr()])
    host_out = np.empty(want.shape, np.float32)
    with pytest.raises(rt.OnrtError):
        net.enqueue_raw([x.data_ptr()], [host_out.ctypes.data])
    net.close()
    monkeypatch.setenv("ONENEW_RT_GRAPH", "1")
    graphed = rt.Net(data)
    with pytest.raises(rt.OnrtError):
        graphed.enqueue_raw([x.data_ptr()], [y.data_ptr()])
    graphed.close()


def test_convolution_pairs_run_as_one_call(torch_dev, monkeypatch):
    """Conv (3x3) -> Conv (1x1) of two ResNet-style bottlenecks as one call of the Conv plugin's eval_pair / eval_pair_relu
    each, where the plugin recommends it: the pair of the first block without an Add (the projection on the skip path took
    it), the pair of the second with the Add and the Relu; the same bits as the net run operator by operator on the tile the
    pair's kernel uses, within 1e-4 of it whatever tiles it picks, and close to the CPU restatement of the graph; at a
    small batch the operators stay separate"""
    data, ins = one_models.bottleneck_pairs(batch=16, size=32)
    fused, plain, got, want = _both_ways(data, ins, monkeypatch)
    assert plain.fused_pairs() == 0 and fused.fused_pairs() == 2
    assert [n for _, n in fused.ops()] == ["c1", "c2", "dn", "c4", "c5"] and len(plain.ops()) == 11
    assert fused.fused_blocks() == 2   # the two Adds (and Relus) were folded first: into dn and into c6
    for name in ("c2_out", "c5_out"):
        assert fused.operand(name)[1] is None
    assert fused.operand("c6_out")[1] == fused.operand("add2_out")[1] == fused.operand("out")[1]
    ref = one_model.run(data, ins)
    for g, w_, r in zip(got, want, ref):
        assert g.shape == w_.shape and np.all(np.abs(g - w_) <= 1e-4 * np.abs(w_) + 1e-5 * np.abs(w_).max())
        assert _close(g, r, 5e-4)
    x2 = [(ins[0] * np.float32(-0.7) + np.float32(0.2)).astype(np.float32)]
    for g, w_ in zip(fused.run(*x2), plain.run(*x2)):
        assert np.all(np.abs(g - w_) <= 1e-4 * np.abs(w_) + 1e-5 * np.abs(w_).max())
    fused.close()
    plain.close()
    monkeypatch.setenv("ONHIP_TILE", "64x64x1")
    tiled = rt.Net(data)
    monkeypatch.setenv("ONENEW_RT_FUSE_PAIRS", "0")
    tiled_plain = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_FUSE_PAIRS")
    assert tiled.fused_pairs() == 2 and tiled_plain.fused_pairs() == 0 and tiled_plain.fused_blocks() == 2
    for g, w_ in zip(tiled.run(*ins), tiled_plain.run(*ins)):
        assert np.array_equal(g, w_)
    tiled.close()
    tiled_plain.close()
    monkeypatch.delenv("ONHIP_TILE")
    small = rt.Net(one_models.bottleneck_pairs(batch=1, size=32)[0])
    assert small.fused_pairs() == 0 and len(small.ops()) == 7
    small.close()


def test_one_launch_blocks_do_not_overlap_nor_swallow_a_folded_adds_operand(torch_dev, monkeypatch):
    """pw -> dw -> pw -> dw -> pw with at most 64 channels at a batch where the plugin recommends the block kernel: one block
    is folded (the middle 1x1 closes it and opens no second one), the output equals the operator-by-operator run within
    1e-4; a triple whose first result the folded Add of its last convolution reads keeps its operators and its values"""
    data, ins = one_models.separable_chain(batch=16, size=32)
    fused, plain, got, want = _both_ways(data, ins, monkeypatch)
    assert plain.fused_ir_blocks() == 0 and fused.fused_ir_blocks() == 1
    assert [n for _, n in fused.ops()] == ["pw1", "dw2", "pw3"]
    for g, w_ in zip(got, want):
        assert g.shape == w_.shape and np.all(np.abs(g - w_) <= 1e-4 * np.abs(w_) + 1e-5 * np.abs(w_).max())
    assert _close(got[0], one_model.run(data, ins)[0], 5e-4)
    fused.close()
    plain.close()
    data, ins = one_models.block_with_inner_skip(batch=16, size=32)
    fused, plain, got, want = _both_ways(data, ins, monkeypatch)
    assert fused.fused_ir_blocks() == 0 and fused.fused_blocks() == 1
    assert [n for _, n in fused.ops()] == ["a", "b", "c"]
    assert np.all(np.abs(got[0] - want[0]) <= 1e-4 * np.abs(want[0]) + 1e-5 * np.abs(want[0]).max())
    assert _close(got[0], one_model.run(data, ins)[0], 5e-4)
    fused.close()
    plain.close()


def test_mobilenetv2_batch64_with_its_blocks_in_one_call(torch_dev, monkeypatch):
    """the whole MobileNetV2 model at batch 64, where the early inverted-residual blocks run as one call each: logits
    against the same file run operator by operator (1e-3 of the largest logit, same top-5 on every image)"""
    from onenew_amd import stacks
    data, shape, _ = stacks.mobilenet_v2_model(64)
    x = np.random.default_rng(64).uniform(-1.0, 1.0, size=shape).astype(np.float32)
    fused = rt.Net(data)
    assert fused.fused_ir_blocks() == 6
    got = fused.run(x)[0]
    fused.close()
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    plain = rt.Net(data)
    assert plain.fused_ir_blocks() == 0
    want = plain.run(x)[0]
    plain.close()
    assert got.shape == want.shape == (64, 1000)
    assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max()
    assert np.array_equal(np.argsort(got, axis=1)[:, -5:], np.argsort(want, axis=1)[:, -5:])


@pytest.mark.parametrize("split", ["qkvo", "kv", "qo", "o"])
def test_attention_block_takes_in_the_head_transposes(split, torch_dev, monkeypatch):
    """head-split Transposes (0, 2, 1, 3) in front of q, k, v and the head-merge one behind the result fold into the
    attention call's strides: as many operators fewer, the net's output within 1e-4 of the net run operator by operator
    (which has the same values as the plain attention block, in another order in memory)"""
    data, ins = one_models.attention_heads(heads=3, tokens=50, head_dim=64, batch=2, split_heads=tuple(split))
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    plain = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_FUSE")
    fused = rt.Net(data)
    assert fused.fused_attentions() == 1 and [t for t, _ in fused.ops()] == ["MatMul"]
    assert len(plain.ops()) == 4 + len(split)
    for name in [n for n in "qkv" if n in split]:
        assert fused.operand(name)[1] is None
    for scale in (1.0, -0.6):
        xs = [x * np.float32(scale) for x in ins]
        for got, ref in zip(fused.run(*xs), plain.run(*xs)):
            assert got.shape == ref.shape and np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-5)
    plain.close()
    fused.close()


@pytest.mark.parametrize("model", ["attention_heads", "vit_block", "ragged"])
def test_attention_block_runs_as_one_call(model, torch_dev, monkeypatch):
    """the net loaded with the attention block folded into one call of the MatMul plugin's eval_attention against the
    same net run operator by operator: outputs within 1e-4, the operands in between have no buffer, a second run on
    another input reads its operands afresh"""
    data, ins = {"attention_heads": one_models.attention_heads, "vit_block": one_models.vit_block,
                 "ragged": lambda: one_models.attention_heads(heads=2, tokens=197, head_dim=32, batch=1)}[model]()
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    plain = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_FUSE")
    fused = rt.Net(data)
    assert plain.fused_attentions() == 0 and fused.fused_attentions() == 1
    # vit_block also has two linear layers (MatMul -> Add -> Gelu and MatMul -> Add -> Add of the skip connection): four
    # more operators folded away
    linears = 2 if model == "vit_block" else 0
    assert plain.fused_linears() == 0 and fused.fused_linears() == linears
    assert len(fused.ops()) == len(plain.ops()) - 3 - (4 if linears else 0)
    assert fused.operand("scores_out")[1] is None and fused.operand("attn_out")[1] is None
    for scale in (1.0, -0.7):
        xs = [x * np.float32(scale) for x in ins]
        for got, ref in zip(fused.run(*xs), plain.run(*xs)):
            assert _close(got, ref, 1e-4)
            assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-5)
    plain.close()
    fused.close()


@pytest.mark.parametrize("name", list(one_models.MODELS) + ["resnet50", "mobilenetv2"])
def test_graph_replay_matches_plain_launches(name, torch_dev, monkeypatch):
    """loaded with ONENEW_RT_GRAPH=1 a net replays a recorded HIP graph of its operators from its second run on: five runs on changing inputs, with
    unrelated eager work and a device-wide wait between them, each against a net of the same file that launches its
    operators one by one -- the same bits every time"""
    torch = torch_dev
    if name in one_models.MODELS:
        data, ins = one_models.MODELS[name]()
    else:
        from onenew_amd import stacks
        data, shape, _ = (stacks.resnet50_model if name == "resnet50" else stacks.mobilenet_v2_model)(1)
        ins = [np.random.default_rng(41).normal(size=shape).astype(np.float32)]
    plain = rt.Net(data)
    monkeypatch.setenv("ONENEW_RT_GRAPH", "1")
    graphed = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_GRAPH")
    scratch = torch.zeros(1 << 20, device="cuda")
    for rep in range(5):
        cur = [(a * np.float32(1.0 - 0.3 * rep) + np.float32(0.05 * rep)).astype(np.float32) for a in ins]
        got = graphed.run(*cur)
        scratch.add_(1.0)                       # the program's own work on another stream between the replays
        torch.cuda.synchronize()
        want = plain.run(*cur)
        for g, w_ in zip(got, want):
            assert np.array_equal(g, w_), (name, rep)
    assert graphed.graph_launches() == 4 and plain.graph_launches() == 0
    assert float(scratch[0]) == 5.0


def test_recorded_graph_survives_growth_of_the_shared_workspaces(torch_dev, monkeypatch):
    """net A (a split-K convolution and a W8A32 convolution) records its graph; then a net with larger operands makes
    the library's split-K scratch and the plugin's int8 workspace grow; replays of A afterwards still equal plain
    launches bit for bit, because the blocks its recording points at are retired, not freed"""
    from oracle import oracle as orc
    torch = torch_dev
    rng = np.random.default_rng(77)

    def model(n, c, hw, q_hw):
        m = onefile.OneModel()
        m.input("x", (n, c, hw, hw))
        m.conv("c1", "x", _w(rng, c, c, 3, 3) * 0.2, _w(rng, c), "c1_out", pad=1, act=abi.RELU)
        w8, b32, aux = orc.quant_weight_bias(_w(rng, 32, c, 3, 3), _w(rng, 32))
        m.conv("q1", "c1_out", w8, b32, "out", pad=1, act=abi.RELU, quant=(aux, 0.05))
        m.output("out", (n, 32, hw, hw))
        return m.tobytes(), rng.normal(size=(n, c, hw, hw)).astype(np.float32)

    data_a, xa = model(1, 256, 14, 14)          # 256 -> 256 3x3 on 14 x 14: sixteen tiles, the cost model splits K
    plain = rt.Net(data_a)
    monkeypatch.setenv("ONENEW_RT_GRAPH", "1")
    graphed = rt.Net(data_a)
    monkeypatch.delenv("ONENEW_RT_GRAPH")
    for rep in range(2):                        # the second run records
        got = graphed.run(xa * np.float32(1.0 + rep))
    before = hip.load().onhip_scratch_bytes()
    assert before > 0, "net A did not use the split-K scratch"
    # a larger net, every convolution forced to eight K slices: 8 x n x 64 x 56 x 56 x 4 B of partial sums, with the batch
    # n chosen so that they exceed the block the process has so far (other tests may have grown it already)
    n_b = before // (8 * 64 * 56 * 56 * 4) + 2
    data_b, xb = model(int(n_b), 64, 56, 56)
    monkeypatch.setenv("ONHIP_TILE", "64x64x8")
    big = rt.Net(data_b)
    big.run(xb)
    monkeypatch.delenv("ONHIP_TILE")
    torch.cuda.synchronize()
    assert hip.load().onhip_scratch_bytes() > before, "the scratch did not grow: the test does not test what it says"
    filler = torch.full((64 << 20,), 3.0, device="cuda")      # whatever the allocator hands out next
    for rep in range(3):
        cur = (xa * np.float32(0.5 + rep)).astype(np.float32)
        got = graphed.run(cur)
        filler.mul_(1.0)
        torch.cuda.synchronize()
        want = plain.run(cur)
        assert np.array_equal(got[0], want[0]), rep
    assert graphed.graph_launches() >= 3


def _w(rng, *shape):
    return (rng.normal(size=shape) * 0.2).astype(np.float32)


def _residual_variants():
    rng = np.random.default_rng(23)
    out = {}

    def base():
        m = onefile.OneModel()
        m.input("x", (2, 8, 12, 12))
        return m

    # the shortcut is itself a convolution that comes later in the file than the main branch (ResNet's first block of
    # a stage): the folded call runs where the Add was, after both
    m = base()
    m.conv("main", "x", _w(rng, 8, 8, 3, 3), _w(rng, 8), "main_out", pad=1)
    m.conv("short", "x", _w(rng, 8, 8, 1, 1), _w(rng, 8), "short_out")
    m.add("sum", "main_out", "short_out", "s")
    m.relu("relu", "s", "y")
    m.output("y", (2, 8, 12, 12))
    out["shortcut_conv_later_in_the_file"] = (m.tobytes(), 1, 2)
    # the Add without a Relu (MobileNetV2), addend first
    m = base()
    m.conv("main", "x", _w(rng, 8, 8, 1, 1), _w(rng, 8), "main_out")
    m.add("sum", "x", "main_out", "y")
    m.output("y", (2, 8, 12, 12))
    out["add_only_addend_first"] = (m.tobytes(), 1, 1)
    # the sum is read twice: the Add is folded, the Relu stays an operator
    m = base()
    m.conv("main", "x", _w(rng, 8, 8, 3, 3), None, "main_out", pad=1, act=abi.RELU)
    m.add("sum", "main_out", "x", "s")
    m.relu("relu", "s", "r")
    m.add("again", "s", "r", "y")
    m.output("y", (2, 8, 12, 12))
    out["sum_read_twice"] = (m.tobytes(), 1, 1)
    # depthwise convolution in front of the Add: the plugin runs the passes itself
    m = base()
    m.conv("main", "x", _w(rng, 8, 1, 3, 3), _w(rng, 8), "main_out", pad=1, group=8)
    m.add("sum", "main_out", "x", "s")
    m.relu("relu", "s", "y")
    m.output("y", (2, 8, 12, 12))
    out["depthwise_main_branch"] = (m.tobytes(), 1, 2)
    # nothing to fold: the convolution's result is a net output / is read twice / the Add broadcasts a vector
    m = base()
    m.conv("main", "x", _w(rng, 8, 8, 1, 1), _w(rng, 8), "main_out")
    m.add("sum", "main_out", "x", "y")
    m.output("y", (2, 8, 12, 12))
    m.output("main_out", (2, 8, 12, 12))
    out["conv_result_is_an_output"] = (m.tobytes(), 0, 0)
    m = base()
    m.conv("main", "x", _w(rng, 8, 8, 1, 1), _w(rng, 8), "main_out")
    m.add("sum", "main_out", "x", "s")
    m.add("again", "s", "main_out", "y")
    m.output("y", (2, 8, 12, 12))
    out["conv_result_read_twice"] = (m.tobytes(), 0, 0)
    m = base()
    m.conv("main", "x", _w(rng, 8, 8, 1, 1), _w(rng, 8), "main_out")
    m.add("sum", "main_out", _w(rng, 1, 8, 1, 1), "y")
    m.output("y", (2, 8, 12, 12))
    out["add_of_a_broadcast_initialiser"] = (m.tobytes(), 0, 0)
    # a Relu right after a convolution with a bias becomes the convolution's activation, as the offline optimiser
    # does it; here in front of a residual Add, so the block folds on top of it: three operators fewer
    m = base()
    m.conv("pre", "x", _w(rng, 8, 8, 3, 3), _w(rng, 8), "pre_out", pad=1)
    m.relu("pre_relu", "pre_out", "pre_act")
    m.add("sum", "pre_act", "x", "s")
    m.relu("relu", "s", "y")
    m.output("y", (2, 8, 12, 12))
    out["relu_folded_then_block_folded"] = (m.tobytes(), 1, 3)
    # the same Relu after a convolution without a bias stays: the reference's kernel returns before the activation
    m = base()
    m.conv("pre", "x", _w(rng, 8, 8, 3, 3), None, "pre_out", pad=1)
    m.relu("pre_relu", "pre_out", "y")
    m.output("y", (2, 8, 12, 12))
    out["relu_after_a_convolution_without_bias"] = (m.tobytes(), 0, 0)
    m = base()
    m.conv("pre", "x", _w(rng, 8, 8, 3, 3), _w(rng, 8), "pre_out", pad=1)
    m.relu("pre_relu", "pre_out", "mid")
    m.conv("post", "mid", _w(rng, 8, 8, 1, 1), _w(rng, 8), "y", act=abi.RELU)
    m.output("y", (2, 8, 12, 12))
    out["relu_between_two_convolutions"] = (m.tobytes(), 0, 1)
    # two convolutions into one Add: one of them is folded, the other runs before it
    m = base()
    m.conv("a", "x", _w(rng, 8, 8, 1, 1), _w(rng, 8), "a_out")
    m.conv("b", "x", _w(rng, 8, 8, 3, 3), _w(rng, 8), "b_out", pad=1)
    m.add("sum", "a_out", "b_out", "y")
    m.output("y", (2, 8, 12, 12))
    out["two_convolutions_into_one_add"] = (m.tobytes(), 1, 1)
    return out


@pytest.mark.parametrize("name", list(_residual_variants()))
def test_folding_rules(name, torch_dev, monkeypatch):
    data, blocks, fewer_ops = _residual_variants()[name]
    x = np.random.default_rng(29).normal(size=(2, 8, 12, 12)).astype(np.float32)
    fused, plain, got, want = _both_ways(data, [x], monkeypatch)
    assert fused.fused_blocks() == blocks
    assert len(fused.ops()) == len(plain.ops()) - fewer_ops
    assert fused.folded_relus() == (1 if name in ("relu_folded_then_block_folded", "relu_between_two_convolutions") else 0)
    for g, w_ in zip(got, want):
        assert np.array_equal(g, w_)
    ref = one_model.run(data, [x])
    for g, r in zip(got, ref):
        assert _close(g, r, 3e-4)


def test_relu_after_a_quantised_convolution_is_folded(torch_dev, monkeypatch):
    """the W8A32 convolution takes the Relu as its activation too, and the integer chain stays exact"""
    data, ins = one_models.quantised_block()
    fused, plain, got, want = _both_ways(data, ins, monkeypatch)
    assert fused.folded_relus() == 1 and len(fused.ops()) == len(plain.ops()) - 1
    assert np.array_equal(got[0], want[0])
    assert np.array_equal(got[0], one_model.run(data, ins)[0])


def _random_residual_graph(seed):
    """convolutions (dense and depthwise, 1x1 and 3x3, with and without bias and activation), Relu and Add nodes over
    tensors of one shape, wired at random: residual adds in either operand order, results read twice, results that are
    net outputs, chains of folded blocks"""
    rng = np.random.default_rng(13000 + seed)
    C, H, W, N = int(rng.choice([4, 8, 12])), int(rng.integers(5, 14)), int(rng.integers(5, 14)), int(rng.integers(1, 3))
    m = onefile.OneModel()
    m.input("x", (N, C, H, W))
    tensors, outs, nid = ["x"], [], 0

    def w(*shape):
        return (rng.normal(size=shape) * 0.2).astype(np.float32)

    for _ in range(int(rng.integers(2, 7))):
        kind = rng.random()
        src = tensors[int(rng.integers(len(tensors)))] if rng.random() < 0.3 else tensors[-1]
        nid += 1
        if kind < 0.55:
            k = int(rng.choice([1, 3]))
            bias = w(C) if rng.random() < 0.8 else None
            act = int(rng.choice([abi.NOT_ACT, abi.NOT_ACT, abi.RELU, abi.CLIP]))
            group = C if (rng.random() < 0.2 and bias is not None) else 1
            m.conv(f"c{nid}", src, w(C, 1 if group != 1 else C, k, k), bias, f"t{nid}", pad=k // 2, act=act,
                   clip=(-0.5, 0.8), group=group)
            cur = f"t{nid}"
            if rng.random() < 0.3:
                m.relu(f"r{nid}", cur, f"t{nid}r")
                cur = f"t{nid}r"
            if rng.random() < 0.6:
                other = tensors[int(rng.integers(len(tensors)))]
                if rng.random() < 0.5:
                    m.add(f"a{nid}", cur, other, f"t{nid}a")
                else:
                    m.add(f"a{nid}", other, cur, f"t{nid}a")
                if rng.random() < 0.2:
                    outs.append(cur)
                cur = f"t{nid}a"
                if rng.random() < 0.6:
                    m.relu(f"ar{nid}", cur, f"t{nid}ar")
                    cur = f"t{nid}ar"
            tensors.append(cur)
        elif kind < 0.75:
            m.add(f"a{nid}", src, tensors[int(rng.integers(len(tensors)))], f"t{nid}")
            tensors.append(f"t{nid}")
        else:
            m.relu(f"r{nid}", src, f"t{nid}")
            tensors.append(f"t{nid}")
    outs.append(tensors[-1])
    if rng.random() < 0.3 and len(tensors) > 2:
        outs.append(tensors[int(rng.integers(1, len(tensors)))])
    outs = list(dict.fromkeys(o for o in outs if o != "x"))
    for o in outs:
        m.output(o, (N, C, H, W))
    return (m.tobytes() if outs else None), rng.normal(size=(N, C, H, W)).astype(np.float32)


@pytest.mark.parametrize("seed", range(30))
def test_random_residual_graphs_fold_without_changing_a_bit(seed, torch_dev, monkeypatch):
    data, x = _random_residual_graph(seed)
    if data is None:
        pytest.skip("the draw has no output")
    fused, plain, got, want = _both_ways(data, [x], monkeypatch)
    ref = one_model.run(data, [x])
    for g, w_, r in zip(got, want, ref):
        assert np.array_equal(g, w_)
        assert _close(w_, r, 5e-4)


@pytest.mark.parametrize("model", ["resnet50", "mobilenetv2"])
def test_whole_model_folds_every_residual_block(model, torch_dev, monkeypatch):
    """16 bottleneck blocks of ResNet-50 (Add + Relu) and the 10 residual connections of MobileNetV2 (Add), batch 2:
    the same logits, bit for bit, as operator by operator"""
    from onenew_amd import stacks
    make = stacks.resnet50_model if model == "resnet50" else stacks.mobilenet_v2_model
    data, shape, _ = make(2)
    x = np.random.default_rng(31).normal(size=shape).astype(np.float32)
    fused, plain, got, want = _both_ways(data, [x], monkeypatch)
    assert fused.fused_blocks() == (16 if model == "resnet50" else 10)
    assert len(fused.ops()) == len(plain.ops()) - (32 if model == "resnet50" else 10)
    assert np.array_equal(got[0], want[0])


@pytest.mark.parametrize("model", ["resnet50", "mobilenetv2"])
def test_whole_model_matches_the_reference_host_run(model, torch_dev):
    """the full-size network at batch 1 (89 / 65 operators) through the runtime against the logits the reference's
    host operator classes and x86 kernels gave for the same file and input (tests/golden/model_logits.npz, written by
    tests/golden/make_model_logits.py): within 1e-3 of their largest magnitude (53 / 52 convolutions deep with fp32
    sums in another order), same top-5 classes"""
    import hashlib
    import make_model_logits
    data, x = make_model_logits.model_and_input(model)
    fix = np.load(make_model_logits.OUT)
    assert hashlib.sha256(data).digest() == fix[model + "_sha256"].tobytes(), "the model file changed: regenerate the fixture"
    ref = fix[model + "_logits"]
    net = rt.Net(data)
    (got,) = net.run(x)
    assert got.shape == ref.shape == (1, 1000)
    assert np.isfinite(got).all()
    assert _close(got, ref, 1e-3)
    assert set(np.argsort(got[0])[-5:]) == set(np.argsort(ref[0])[-5:])


def test_tile_tuner_writes_the_header_and_the_runtime_reads_it_back(torch_dev):
    """onrt_net_tune_tiles measures the loaded model under every workgroup tile of the library and leaves the fastest
    set; written into the file header (BLOCK_INFO_S.cuda_gemm_tile_*) it is what the next load runs with; whatever the
    tile, the results stay those of the oracle"""
    from onenew_amd import stacks
    data, ins = one_models.resnet_block()
    ref = one_model.run(data, ins)
    net = rt.Net(data)
    assert net.tiles() == (16, 16, 16)
    tiles, best_ms, default_ms = net.tune_tiles(reps=3)
    cands = [(16, 16, 16)]
    i, bm, bn = 0, C.c_int32(), C.c_int32()
    while hip.load().onhip_tile_candidate(i, C.byref(bm), C.byref(bn)) == 0:
        cands.append((bm.value, bn.value, 16))
        i += 1
    assert len(cands) >= 4 and tiles in cands and net.tiles() == tiles
    assert 0 < best_ms <= default_ms
    for g, r in zip(net.run(*ins), ref):
        assert _close(g, r, 5e-4)
    # every tile, forced through the header of the file: same results within the fp32 bar, and the tile is really used
    # (a 3x3 convolution on 20 x 20 pixels and 16 channels under 128 x 128 and 32 x 128 tiles sums in another order)
    outs = {}
    for t in cands[1:]:
        n2 = rt.Net(rt.with_tiles(data, t))
        assert n2.tiles() == t
        outs[t] = n2.run(*ins)
        for g, r in zip(outs[t], ref):
            assert _close(g, r, 5e-4), t
    # the full-size model: the tuner's choice is at least as fast as the default and keeps the logits
    data, shape, _ = stacks.resnet50_model(1)
    x = np.random.default_rng(5).normal(size=shape).astype(np.float32)
    net = rt.Net(data)
    (before,) = net.run(x)
    tiles, best_ms, default_ms = net.tune_tiles(reps=3)
    print("ResNet-50 batch 1: tile", tiles, "best", best_ms, "ms, default", default_ms, "ms", flush=True)
    (after,) = net.run(x)
    assert best_ms <= default_ms and _close(after, before, 1e-3)
    assert set(np.argsort(after[0])[-5:]) == set(np.argsort(before[0])[-5:])


def test_unoptimised_file_runs_like_the_optimised_one(torch_dev, monkeypatch):
    """a file with Clip / LeakyRelu / Sigmoid x Mul / HardSigmoid x Mul / Relu nodes after its convolutions, loaded as
    it is: the same bits as the file the offline optimiser would have made of it, which in turn matches the oracle;
    also with ONENEW_RT_FUSE=0, which cannot leave these nodes unfolded"""
    raw, ins = one_models.unfused_activations()
    opt, _ = one_models.unfused_activations(optimised=True)
    want = rt.Net(opt).run(*ins)
    ref = one_model.run(opt, ins)
    assert _close(want[0], ref[0], 5e-4)
    net = rt.Net(raw)
    assert net.folded_activations() == 4 and [t for t, _ in net.ops()] == ["Conv"] * 5
    got = net.run(*ins)
    assert np.array_equal(got[0], want[0])
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    unfused = rt.Net(raw)                       # the Relu stays a node of its own here, the other four are folded
    monkeypatch.delenv("ONENEW_RT_FUSE")
    assert unfused.folded_activations() == 4 and [t for t, _ in unfused.ops()] == ["Conv"] * 5 + ["Relu"]
    assert np.array_equal(unfused.run(*ins)[0], want[0])


@pytest.mark.gpu
def test_int8_convolutions_exchange_int8_operands(torch_dev, monkeypatch):
    """dense int8 convolutions that feed each other hand their operand over as int8 NHWC, quantised by the producer with
    the consumers' input_scale: three operands in the chain model (one with two readers, one into a convolution with a
    folded Add + Relu), the results equal to the oracle's and to the runtime's with every operand fp32, bit for bit;
    at batch 3 too.  Consumers with different scales, or any other reader, keep the operand fp32"""
    for n in (1, 3):
        data, ins = one_models.quantised_chain(n=n)
        net = rt.Net(data)
        assert net.int8_links() == 3 and net.fused_blocks() == 1
        outs = net.run(*ins)
        outs2 = net.run(*ins)                       # buffers reused
        ref = one_model.run(data, ins, keep_all=True)
        for (oname, _), got, got2 in zip(net.outputs, outs, outs2):
            assert np.array_equal(got, ref[oname]), oname
            assert np.array_equal(got2, got)
        net.close()
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    data, ins = one_models.quantised_chain()
    plain = rt.Net(data)
    assert plain.int8_links() == 0
    plain_outs = plain.run(*ins)
    plain.close()
    monkeypatch.delenv("ONENEW_RT_FUSE")
    net = rt.Net(data)
    for a, b in zip(net.run(*ins), plain_outs):
        assert np.array_equal(a, b)
    net.close()
    # the fp32 result of the residual block, read by two more int8 convolutions: they get its int8 copy from the same store
    for n in (1, 2):
        data, ins = one_models.quantised_chain(n=n, tail=True)
        net = rt.Net(data)
        assert net.int8_links() == 4
        ref = one_model.run(data, ins, keep_all=True)
        for (oname, _), got in zip(net.outputs, net.run(*ins)):
            assert np.array_equal(got, ref[oname]), ("tail", oname)
        net.close()
    for kw, links in (({"different_scales": True}, 2), ({"extra_reader": True}, 2)):
        data, ins = one_models.quantised_chain(**kw)
        net = rt.Net(data)
        assert net.int8_links() == links, kw
        ref = one_model.run(data, ins, keep_all=True)
        for (oname, _), got in zip(net.outputs, net.run(*ins)):
            assert np.array_equal(got, ref[oname]), (kw, oname)
        net.close()


@pytest.mark.gpu
def test_maxpool_between_int8_convolutions_runs_on_int8(torch_dev):
    """Conv (int8) -> MaxPool -> two int8 convolutions with one input_scale: both operands around the MaxPool travel as
    int8 NHWC and the pooling runs on bytes; the outputs equal the oracle's fp32 evaluation bit for bit"""
    for n, hw in ((2, 21), (1, 40)):
        data, ins = one_models.quantised_stem(n=n, hw=hw)
        net = rt.Net(data)
        assert net.int8_links() == 2
        ref = one_model.run(data, ins, keep_all=True)
        for (oname, _), got in zip(net.outputs, net.run(*ins)):
            assert np.array_equal(got, ref[oname]), oname
        net.close()


@pytest.mark.gpu
def test_depthwise_int8_convolutions_take_part_in_the_int8_edges(torch_dev, monkeypatch):
    """a quantised MobileNetV2-style model: the operands around its depthwise convolutions (conv.c:617-755) travel as int8
    NHWC like those between dense ones, so everything from the stem to the last projection is int8 except the sum of the
    skip connection; the outputs equal the oracle's evaluation with every operand fp32 and the runtime's own with the
    edges off, bit for bit.  A reader with another input_scale keeps that one operand fp32."""
    for n, hw in ((2, 24), (1, 37)):
        data, ins = one_models.quantised_mobile(n=n, hw=hw)
        net = rt.Net(data)
        # stem, dw0, pw0, e1, dw1 | p1 (read by e2 and, as the Add's operand, by p2: stays fp32), e2, dw2 | e3, dw3
        assert net.int8_links() == 9, net.int8_links()
        outs = net.run(*ins)
        outs2 = net.run(*ins)
        ref = one_model.run(data, ins, keep_all=True)
        for (oname, _), got, got2 in zip(net.outputs, outs, outs2):
            assert np.array_equal(got, ref[oname]), oname
            assert np.array_equal(got2, got)
        net.close()
    data, ins = one_models.quantised_mobile()
    monkeypatch.setenv("ONENEW_RT_LINK", "0")
    plain = rt.Net(data)
    assert plain.int8_links() == 0
    want = plain.run(*ins)
    plain.close()
    monkeypatch.delenv("ONENEW_RT_LINK")
    net = rt.Net(data)
    for a, b in zip(net.run(*ins), want):
        assert np.array_equal(a, b)
    net.close()
    data, ins = one_models.quantised_mobile(scales_differ=True)
    net = rt.Net(data)
    assert net.int8_links() == 8
    ref = one_model.run(data, ins, keep_all=True)
    for (oname, _), got in zip(net.outputs, net.run(*ins)):
        assert np.array_equal(got, ref[oname]), ("scales differ", oname)
    net.close()


def _conv_nodes(parsed):
    return [cfg for t, cfg in parsed["nodes"] if t == "Conv"]


@pytest.mark.gpu
@pytest.mark.parametrize("method", ["kl", "mse", "percent"])
@pytest.mark.parametrize("model", ["resnet_block", "mobile_block", "unfused_activations", "ir_blocks"])
def test_model_level_quantisation_writes_what_the_oracles_steps_give(model, method, torch_dev, oracle, monkeypatch):
    """onrt_one_quantise (tools/optimize/model_quant.hpp:625-679) on small fp32 models: every Conv of the image it returns
    carries input_scale = threshold / 127 with the threshold the oracle's calibrators compute from the same activations
    (the fp32 net's own operands on the calibration inputs), int8 weights, int32 bias and weight_aux equal to the oracle's
    quant_weight_bias, and nothing else in the file differs; the quantised image then runs through the runtime with the
    results of the oracle's executor (bit for bit where every operator after the first Conv is exact)"""
    builder = {"resnet_block": one_models.resnet_block, "mobile_block": one_models.mobile_block,
               "unfused_activations": one_models.unfused_activations,
               "ir_blocks": lambda: one_models.inverted_residual_blocks(batch=2, size=32)}[model]
    if method == "percent" and model != "ir_blocks":
        # model_quant.hpp:107-118 keeps (1 - 0.99998) * 10 * elements values per image: nothing below 5000 elements, and the
        # threshold of such an operand is 0
        pytest.skip("the percentile rule keeps no value of operands this small")
    data, ins = builder()
    rng = np.random.default_rng(77)
    images = [[(a * np.float32(s) + rng.normal(size=a.shape).astype(np.float32) * np.float32(0.1)).astype(np.float32) for a in ins]
              for s in (1.0, 0.7, -1.2)]
    second = [[(a * np.float32(0.9)).astype(np.float32) for a in item] for item in images[:2]]
    code = {"kl": rt.QUANT_KL, "mse": rt.QUANT_MSE, "percent": rt.QUANT_PERCENT}[method]
    q = rt.quantise(data, images, code, images2=None if method == "percent" else second)
    assert len(q) == len(data)
    src, dst = onefile.parse(data), onefile.parse(q)
    # the activations the calibration saw: the fp32 net, operator by operator
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    net = rt.Net(data)
    monkeypatch.delenv("ONENEW_RT_FUSE")
    names = []
    for cfg in _conv_nodes(src):
        n = cfg.op_base_cfg.in_operand_name[0].value.decode()
        if n not in names:
            names.append(n)
    seen = {n: [] for n in names}
    seen2 = {n: [] for n in names}
    for store, items in ((seen, images), (seen2, second)):
        for item in items:
            net.run(*item)
            for n in names:
                store[n].append(net.fetch(n).copy())
    net.close()
    thr = {}
    for n in names:
        if method == "percent":
            x = np.stack(seen[n])
            thr[n] = oracle.calib_percentile(x, len(images), x[0].size)
        else:
            mx = 0.0
            for a in seen[n]:
                mx = oracle.calib_abs_max(a, mx)
            hist = None
            for a in seen2[n]:
                hist = oracle.calib_histogram(a, mx, hist)
            thr[n] = oracle.calib_threshold(method, hist, seen2[n][0].size * len(second), mx)
    assert [t for t, _ in src["nodes"]] == [t for t, _ in dst["nodes"]]
    touched = set()
    for (t, a), (_, b) in zip(src["nodes"], dst["nodes"]):
        if t != "Conv":
            assert bytes(a) == bytes(b)
            continue
        name = a.op_base_cfg.op_name.decode()
        want_scale = np.float32(thr[a.op_base_cfg.in_operand_name[0].value.decode()]) / np.float32(127)
        assert np.float32(b.input_scale) == want_scale, (name, b.input_scale, want_scale)
        assert b.ifmap_quant2 == abi.TYPE_INT8 and b.input_scale > 0
        wname = a.op_base_cfg.in_operand_name[1].value.decode()
        w = src["inits"][wname]
        bias = src["inits"][a.op_base_cfg.in_operand_name[2].value.decode()] if a.has_bias else None
        w8, b32, aux = oracle.quant_weight_bias(w, bias)
        got_w = dst["inits"][wname]
        assert got_w.shape == w.shape and got_w.dtype == np.float32
        raw = got_w.reshape(-1).view(np.int8)
        assert np.array_equal(raw[:w.size], w8.reshape(-1)) and not raw[w.size:].any(), name
        assert np.array_equal(np.array(b.weight_aux[:w.shape[0]], np.float32), aux), name
        touched.add(wname)
        if bias is not None:
            bname = a.op_base_cfg.in_operand_name[2].value.decode()
            assert np.array_equal(dst["inits"][bname].view(np.int32), b32), name
            touched.add(bname)
        # everything else of the node is as it was
        a2 = type(a).from_buffer_copy(a)
        a2.input_scale, a2.ifmap_quant2 = b.input_scale, b.ifmap_quant2
        for i in range(len(a2.weight_aux)):
            a2.weight_aux[i] = b.weight_aux[i]
        assert bytes(a2) == bytes(b), name
    for n, arr in src["inits"].items():
        if n not in touched:
            assert np.array_equal(arr.view(np.uint8), dst["inits"][n].view(np.uint8)), n
    assert src["inputs"] == dst["inputs"] and src["outputs"] == dst["outputs"]
    # the quantised image runs: against the oracle's executor on the same image
    qnet = rt.Net(q)
    if model == "unfused_activations":
        # the oracle's executor has no Clip / Sigmoid / Mul nodes (it reads optimised files); the same model written by the
        # optimiser carries the same weights and, given the same scales, must give the same results
        opt, _ = one_models.unfused_activations(optimised=True)
        buf = bytearray(opt)
        po, off = onefile.parse(opt), onefile.parse(opt)["header"].node_cfg_offset
        scales = {b.op_base_cfg.op_name.decode(): b for b in _conv_nodes(dst)}
        for t, cfg in po["nodes"]:
            assert t == "Conv"
            qc = scales[cfg.op_base_cfg.op_name.decode()]
            cfg.input_scale, cfg.ifmap_quant2 = qc.input_scale, qc.ifmap_quant2
            for i in range(len(cfg.weight_aux)):
                cfg.weight_aux[i] = qc.weight_aux[i]
            buf[off:off + C.sizeof(cfg)] = bytes(cfg)
            off += onefile.align64(C.sizeof(cfg))
        ref_model = bytes(buf)
        # weights and biases: the optimised builder draws the same ones, so copy the quantised initialisers over by name
        pq = onefile.parse(ref_model)
        m2 = bytearray(ref_model)
        ioff = pq["header"].init_info_offset
        for name, arr in pq["inits"].items():
            start = ioff + C.sizeof(abi.OPERAND_S)
            m2[start:start + arr.nbytes] = dst["inits"][name].tobytes()
            ioff += onefile.align64(C.sizeof(abi.OPERAND_S) + arr.nbytes)
        ref = one_model.run(bytes(m2), ins)
    else:
        ref = one_model.run(q, ins)
    for got, want in zip(qnet.run(*ins), ref):
        if model == "resnet_block":          # a Gemm (MFMA summation order) ends this one
            assert _close(got, want, 1e-4)
        else:
            assert np.array_equal(got, want)
    qnet.close()
    # and an image that is quantised already is refused
    with pytest.raises(rt.OnrtError, match="quantised already"):
        rt.quantise(q, images, code)
