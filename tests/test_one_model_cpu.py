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



# ---- the host-side half of the runtime (order, shape inference, folding) on the CPU -----------------------------

@pytest.mark.parametrize("name", list(one_models.MODELS))
def test_plan_infers_the_shapes_the_oracle_computes(name, monkeypatch):
    """onrt_net_plan_buf needs no GPU: with folding off every operand of every test model gets the shape the oracle's
    execution of the file produces, in an order in which every input is ready"""
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    data, ins = one_models.MODELS[name]()
    net = rt.Net(data, plan_only=True)
    m = onefile.parse(data)
    ref = one_model.run(data, ins, keep_all=True)
    assert net.outputs == [(n, tuple(s)) for n, s in m["outputs"]]
    assert sorted(t for t, _ in net.ops()) == sorted(t for t, _ in m["nodes"])
    produced = {n for n, _ in m["inputs"]}
    by_name = {cfg.op_base_cfg.op_name.decode(): cfg for _, cfg in m["nodes"]}
    for _, op_name in net.ops():
        cfg = by_name[op_name].op_base_cfg
        for k in range(cfg.in_operand_num):
            iname = cfg.in_operand_name[k].value.decode()
            assert iname in produced or iname not in ref or iname.startswith(op_name + "."), (op_name, iname)
        oname = cfg.out_operand_name[0].value.decode()
        produced.add(oname)
        shape, ptr = net.operand(oname)
        assert ptr is None and tuple(shape) == tuple(ref[oname].shape), oname
    with pytest.raises(rt.OnrtError, match="plan"):
        net.run(*ins)
    net.close()


def test_plan_folds_residual_blocks_and_relus():
    from onenew_amd import stacks
    data, _ = one_models.resnet_block()
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 1 and net.folded_relus() == 0
    types = [t for t, _ in net.ops()]
    assert "Add" not in types and types.count("Relu") == 0 and len(types) == len(onefile.parse(data)["nodes"]) - 2
    data, _ = one_models.quantised_block()
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 0 and net.folded_relus() == 1
    # the full-size models: 16 bottleneck blocks, 10 inverted-residual connections
    data, shape, _ = stacks.resnet50_model(2)
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 16 and len(net.ops()) == 89 - 32
    assert net.inputs[0][1] == tuple(shape) and net.outputs[0][1] == (2, 1000)
    data, shape, _ = stacks.mobilenet_v2_model(3)
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 10 and len(net.ops()) == 65 - 10
    assert net.outputs[0][1] == (3, 1000)


def test_plan_keeps_one_launch_blocks_apart_and_counts_folded_adds_as_reads(monkeypatch):
    """the inverted-residual fold on the graph alone (ONENEW_RT_PLAN_BLOCKS=1 takes every 1x1 -> depthwise -> 1x1 chain):
    in pw -> dw -> pw -> dw -> pw the middle 1x1 closes the first block and must not open a second one over it; a triple
    whose first result is also the other operand of the Add folded into its last convolution stays three operators"""
    monkeypatch.setenv("ONENEW_RT_PLAN_BLOCKS", "1")
    data, _ = one_models.separable_chain()
    net = rt.Net(data, plan_only=True)
    assert net.fused_ir_blocks() == 1
    assert [n for _, n in net.ops()] == ["pw1", "dw2", "pw3"]
    data, _ = one_models.block_with_inner_skip()
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 1 and net.fused_ir_blocks() == 0
    assert [n for _, n in net.ops()] == ["a", "b", "c"]
    # MobileNetV2's blocks: the skip connection reads the block's input, not an operand inside it; all 16 expanding
    # blocks are chains of this shape (the first block has no expansion)
    from onenew_amd import stacks
    data, _, _ = stacks.mobilenet_v2_model(2)
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 10 and net.fused_ir_blocks() == 16
    monkeypatch.delenv("ONENEW_RT_PLAN_BLOCKS")
    assert rt.Net(one_models.separable_chain()[0], plan_only=True).fused_ir_blocks() == 0


def test_plan_runs_an_attention_block_as_one_call(monkeypatch):
    """MatMul(q, Transpose(k)) -> Softmax -> MatMul(., v): one call where the fused kernel takes the shape, four operators
    where it does not (head dimension, token count), where an operand in between has another reader, or with fusing off"""
    data, _ = one_models.attention_heads()
    net = rt.Net(data, plan_only=True)
    assert net.fused_attentions() == 1 and [t for t, _ in net.ops()] == ["MatMul"]
    data, _ = one_models.vit_block()                       # q = k = v = one tensor, behind a Reshape
    net = rt.Net(data, plan_only=True)
    # and two linear layers in front: MatMul -> Add -> Gelu, MatMul -> Add -> Add of the skip connection (four more
    # operators folded away)
    assert net.fused_attentions() == 1 and net.fused_linears() == 2 and net.fused_skips() == 1
    assert len(net.ops()) == len(onefile.parse(data)["nodes"]) - 3 - 4
    # head-split Transposes in front of q, k, v and the head-merge one behind the result go into the same call
    for split in ("qkvo", "k", "qo"):
        net = rt.Net(one_models.attention_heads(split_heads=tuple(split))[0], plan_only=True)
        assert net.fused_attentions() == 1 and [t for t, _ in net.ops()] == ["MatMul"], split
    for kw in (dict(head_dim=48), dict(tokens=300), dict(scores_also_output=True)):
        net = rt.Net(one_models.attention_heads(**kw)[0], plan_only=True)
        assert net.fused_attentions() == 0 and len(net.ops()) == 4, kw
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    net = rt.Net(one_models.attention_heads()[0], plan_only=True)
    assert net.fused_attentions() == 0 and len(net.ops()) == 4


def test_plan_keeps_what_must_not_be_folded(monkeypatch):
    """a convolution whose result is a net output, or has two readers, or meets a broadcast Add, stays as it is; with
    ONENEW_RT_FUSE=0 so does everything"""
    rng = np.random.default_rng(1)
    w = lambda *s: (rng.normal(size=s) * 0.2).astype(np.float32)   # noqa: E731
    m = onefile.OneModel()
    m.input("x", (1, 4, 6, 6))
    m.conv("a", "x", w(4, 4, 1, 1), w(4), "a_out")
    m.add("s1", "a_out", "x", "y1")                    # a_out is also an output
    m.conv("b", "x", w(4, 4, 1, 1), w(4), "b_out")
    m.add("s2", "b_out", w(1, 4, 1, 1), "y2")          # broadcast of a per-channel initialiser
    m.conv("c", "x", w(4, 4, 1, 1), w(4), "c_out")
    m.add("s3", "c_out", "x", "t3")
    m.add("s4", "t3", "c_out", "y3")                   # c_out read twice
    m.conv("d", "x", w(4, 4, 1, 1), None, "d_out")
    m.relu("r", "d_out", "y4")                         # no bias: the reference kernel skips the activation
    for n in ("a_out", "y1", "y2", "y3", "y4"):
        m.output(n, (1, 4, 6, 6))
    net = rt.Net(m.tobytes(), plan_only=True)
    assert net.fused_blocks() == 0 and net.folded_relus() == 0 and len(net.ops()) == 9
    data, _ = one_models.resnet_block()
    monkeypatch.setenv("ONENEW_RT_FUSE", "0")
    net = rt.Net(data, plan_only=True)
    assert net.fused_blocks() == 0 and len(net.ops()) == len(onefile.parse(data)["nodes"])


def test_plan_refuses_a_node_whose_first_input_is_unnamed():
    """found by fuzzing the plan under the host sanitizers: an empty first input name made a rank-0 operand whose last
    dimension Gemm and MatMul then indexed"""
    data, _ = one_models.resnet_block()
    m = onefile.parse(data)
    off = m["header"].node_cfg_offset
    for op_type, cfg in m["nodes"]:
        if op_type == "Gemm":
            name_off = off + abi.BASE_CONFIG_S.in_operand_name.offset
            bad = bytearray(data)
            bad[name_off:name_off + 8] = b"\0" * 8
            h = C.c_void_p()
            rc = rt.load().onrt_net_plan_buf(bytes(bad), len(bad), C.byref(h))
            assert rc == -2 and not h.value and "first input" in rt.load().onrt_last_error().decode()
            return
        off += onefile.align64(C.sizeof(cfg))
    raise AssertionError("the test model has no Gemm")


@pytest.mark.parametrize("seed", range(30))
def test_plan_of_random_residual_graphs(seed):
    """the folding passes on the random graphs of the GPU suite, without a GPU: the plan loads, keeps every output, and
    never runs more operators than the file has"""
    sys.path.insert(0, HERE)
    from test_gpu_runtime import _random_residual_graph
    data, _ = _random_residual_graph(seed)
    if data is None:
        pytest.skip("the draw has no output")
    m = onefile.parse(data)
    net = rt.Net(data, plan_only=True)
    assert net.outputs == [(n, tuple(s)) for n, s in m["outputs"]]
    folded = len(m["nodes"]) - len(net.ops())
    assert 0 <= folded <= 2 * net.fused_blocks() + net.folded_relus()
    assert folded >= net.fused_blocks() + net.folded_relus()


@pytest.mark.parametrize("model", ["resnet50", "mobilenetv2"])
def test_full_size_model_oracle_reproduces_the_reference_logits(model):
    """the CPU restatement of the runtime on the full-size model files against the logits the reference's host classes
    gave for them (tests/golden/model_logits.npz): the same convolution arithmetic, so the same bits"""
    import hashlib
    import make_model_logits
    data, x = make_model_logits.model_and_input(model)
    fix = np.load(make_model_logits.OUT)
    assert hashlib.sha256(data).digest() == fix[model + "_sha256"].tobytes(), "the model file changed: regenerate the fixture"
    (got,) = one_model.run(data, [x])
    assert np.array_equal(got, fix[model + "_logits"])


def test_header_tiles_are_written_and_read_back():
    """BLOCK_INFO_S.cuda_gemm_tile_{m,n,k} of the file header (common/nn_common.h:28-39): the writer's default is the
    converter's 16 / 16 / 16, onrt_one_set_tiles changes those three fields and nothing else, a plan reads them back"""
    data, _ = one_models.resnet_block()
    assert rt.Net(data, plan_only=True).tiles() == (16, 16, 16)
    tuned = rt.with_tiles(data, (64, 128, 16))
    assert len(tuned) == len(data)
    h0, h1 = abi.ONE_MODEL_DESC_S.from_buffer_copy(data), abi.ONE_MODEL_DESC_S.from_buffer_copy(tuned)
    b = h1.useful_info.block_info
    assert (b.cuda_gemm_tile_m, b.cuda_gemm_tile_n, b.cuda_gemm_tile_k) == (64, 128, 16)
    assert (b.x86_gemm_multi_threads_tile_m, b.x86_gemm_multi_threads_tile_n, b.x86_gemm_multi_threads_tile_k) == (32, 1024, 8)
    off = abi.ONE_MODEL_DESC_S.useful_info.offset + abi.USEFUL_INFO_S.block_info.offset + 6 * 4
    assert tuned[:off] == data[:off] and tuned[off + 12:] == data[off + 12:]
    assert h0.node_cnt == h1.node_cnt
    plan = rt.Net(tuned, plan_only=True)
    assert plan.tiles() == (64, 128, 16)
    plan.set_tiles((128, 128, 16))
    assert plan.tiles() == (128, 128, 16)
    with pytest.raises(rt.OnrtError):
        rt.with_tiles(b"\0" * 4096, (64, 64, 16))


def test_plan_folds_the_optimisers_activation_patterns():
    """Conv -> Clip / LeakyRelu / Sigmoid x Mul / HardSigmoid x Mul / Relu of a file that has not been through the
    offline optimiser: the plan runs five Conv calls and nothing else, exactly as for the optimised file, with the
    activation parameters in the convolutions' configuration (tools/optimize/op_fusion.hpp:47-192)"""
    raw, _ = one_models.unfused_activations()
    opt, _ = one_models.unfused_activations(optimised=True)
    p_raw, p_opt = rt.Net(raw, plan_only=True), rt.Net(opt, plan_only=True)
    assert [t for t, _ in p_raw.ops()] == ["Conv"] * 5 == [t for t, _ in p_opt.ops()]
    assert p_raw.folded_activations() == 4 and p_raw.folded_relus() == 1
    assert p_opt.folded_activations() == 0 and p_opt.folded_relus() == 0
    # the folded-away operands read as the activation's result
    for name in ("c1_raw", "c3_raw", "c3_gate", "c4_gate"):
        assert p_raw.operand(name)[0] == p_raw.operand({"c1_raw": "a1", "c3_raw": "a3", "c3_gate": "a3", "c4_gate": "a4"}[name])[0]
    assert p_raw.operand("out")[0] == (2, 12, 12, 12)


def test_plan_refuses_an_activation_node_no_conv_takes():
    """a Clip after a MaxPool, a Sigmoid whose Mul partner is missing, a Clip after a Conv without bias: refused"""
    def base():
        m = onefile.OneModel()
        m.input("x", (1, 4, 8, 8))
        return m
    w, b = np.ones((4, 4, 1, 1), np.float32), np.zeros(4, np.float32)
    m = base()
    m.maxpool("pool", "x", "p", 3, 1, 1)
    m.clip("clip", "p", "out", 0.0, 6.0)
    m.output("out", (1, 4, 8, 8))
    with pytest.raises(rt.OnrtError, match="Clip"):
        rt.Net(m.tobytes(), plan_only=True)
    m = base()
    m.conv("c", "x", w, b, "c_out")
    m.sigmoid("sig", "c_out", "out")
    m.output("out", (1, 4, 8, 8))
    with pytest.raises(rt.OnrtError, match="Sigmoid"):
        rt.Net(m.tobytes(), plan_only=True)
    m = base()
    m.conv("c", "x", w, None, "c_out")
    m.clip("clip", "c_out", "out", 0.0, 6.0)
    m.output("out", (1, 4, 8, 8))
    with pytest.raises(rt.OnrtError, match="Clip"):
        rt.Net(m.tobytes(), plan_only=True)
    # the convolution's own result is also read elsewhere: the Clip cannot be folded
    m = base()
    m.conv("c", "x", w, b, "c_out")
    m.clip("clip", "c_out", "y", 0.0, 6.0)
    m.add("sum", "y", "c_out", "out")
    m.output("out", (1, 4, 8, 8))
    with pytest.raises(rt.OnrtError, match="Clip"):
        rt.Net(m.tobytes(), plan_only=True)
