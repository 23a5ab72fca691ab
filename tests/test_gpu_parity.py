"""GPU parity: the HIP kernels against the CPU oracle on the same seeded inputs and against the
fixtures made from the reference's own compiled kernels.  Everything goes through the C ABI
(kernel level via onenew_amd.hip, plugin level via `eval`).

Bars: depthwise and W8A32 bit-exact (int32 accumulators included); fp32 MFMA paths
max|a-b| / max|b| <= 1e-4 and |a-b| <= 1e-4 * |b| + 1e-5 element-wise; table activations are
checked exactly on the kernel's own pre-activation; bf16 / fp16 modes within 1e-2 of the fp32
reference."""
import numpy as np
import pytest

import cases
from onenew_amd import abi, datagen, hip, ops
from onenew_amd.abi import ConvDesc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    hip.init(0)
    return torch


def dev(torch, a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close_f32(got, ref, rel=1e-4, tag="", elementwise=True):
    """max|a-b| / max|b| <= rel, and (fp32 paths) |a-b| <= rel*|b| + rel/10 for every element.  The
    reduced-precision modes are judged on the normalised maximum only: with 8 mantissa bits the
    rounding noise of a K-term sum exceeds any per-element bound near zero crossings."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape
    scale = np.abs(ref).max() if ref.size else 0.0
    diff = np.abs(got - ref)
    assert diff.max() <= rel * max(scale, 1e-30), f"{tag}: max diff {diff.max():.3e} vs max|ref| {scale:.3e}"
    if not elementwise:
        return
    bad = diff > rel * np.abs(ref) + rel * 0.1
    assert not bad.any(), f"{tag}: {bad.sum()} elements outside |a-b| <= {rel}*|b| + {rel * 0.1}"


def run_conv_f32(torch, name, d, compute=abi.COMPUTE_F32):
    x, w, b = cases.conv_inputs(name, d)
    dd = ConvDesc.from_buffer_copy(d)
    dd.compute = compute
    lut = dev(torch, cases.silu_lut())
    y = hip.conv2d_f32(dd, dev(torch, x), dev(torch, w), dev(torch, b), lut)
    torch.cuda.synchronize()
    return x, w, b, y.cpu().numpy()


@pytest.mark.parametrize("name", list(cases.conv_f32_cases()))
def test_conv_f32(name, torch_dev, oracle, golden):
    torch = torch_dev
    d = cases.conv_f32_cases()[name]
    print(f"case {name}", flush=True)
    x, w, b, y = run_conv_f32(torch, name, d)
    ref = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    if d.group != 1:
        # depthwise: same operation order as the reference, bit-identical
        assert np.array_equal(y, ref), f"{name}: {(y != ref).sum()} elements differ"
        cases.check_against(golden, name, y, exact=True)
        return
    if d.has_bias and d.act_type == abi.SILU:
        # table activation: compare the pre-activation, then the table applied to the kernel's own pre-activation
        dn = ConvDesc.from_buffer_copy(d)
        dn.act_type = abi.NOT_ACT
        _, _, _, pre = run_conv_f32(torch, name, dn)
        assert_close_f32(pre, oracle.conv2d_f32(dn, x, w, b), tag=name + " pre-activation")
        assert np.array_equal(y, oracle.lut_act(pre, cases.silu_lut())), f"{name}: table lookup differs"
        return
    assert_close_f32(y, ref, tag=name)
    scale = float(np.abs(ref).max())
    cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-4 * scale)


def _random_conv(rng, quant):
    """a convolution the path accepts, drawn at random: filter 1..5 (rectangular now and then), stride 1..3, padding up
    to the filter's reach, odd channel counts and image sides, batch 1..3, dense or depthwise, any activation"""
    kh = int(rng.choice([1, 1, 3, 3, 3, 5, 2]))
    kw = kh if rng.random() < 0.8 else int(rng.choice([1, 3]))
    s = int(rng.choice([1, 1, 2, 3]))
    pad = int(rng.integers(0, max(kh, kw) // 2 + 1))
    depthwise = rng.random() < 0.25
    cin = int(rng.integers(1, 70))
    cout = cin if depthwise else int(rng.integers(1, 140))
    h = int(rng.integers(max(kh, 1), 40))
    w = int(rng.integers(max(kw, 1), 40))
    acts = [abi.NOT_ACT, abi.RELU, abi.CLIP, abi.SILU, abi.LEAKYRELU, abi.HARDSILU]
    act = int(rng.choice(acts))
    bias = 1 if (depthwise or rng.random() < 0.8) else 0
    kw_args = dict(clip_min=-0.3, clip_max=0.6, leaky_relu_alpha=0.1, hard_sigmoid_alpha=1.0 / 6, hard_sigmoid_beta=0.5)
    if quant:
        pad = min(pad, kh // 2)
        kw_args["input_scale"] = float(rng.uniform(0.005, 0.05))
    return cases.cd(cin, cout, (kh, kw), s, pad, h, w, act=act, group=cin if depthwise else 1, bias=bias,
                    n=int(rng.integers(1, 4)), **kw_args)


@pytest.mark.parametrize("seed", range(40))
def test_conv_f32_random_shapes(seed, torch_dev, oracle):
    """forty seeded random convolutions through the measured tile choice and through the cost model's"""
    torch = torch_dev
    rng = np.random.default_rng(1000 + seed)
    d = _random_conv(rng, quant=False)
    name = f"random_f32_{seed}"
    x, w, b = cases.conv_inputs(name, d)
    lut = cases.silu_lut()
    xd, wd, ld = dev(torch, x), dev(torch, w), dev(torch, lut)
    bd = dev(torch, b) if b is not None else None
    table = bool(d.has_bias) and d.act_type == abi.SILU
    dn = ConvDesc.from_buffer_copy(d)
    if table:
        dn.act_type = abi.NOT_ACT                          # judged on the pre-activation: the table is a step function
    ref = oracle.conv2d_f32(dn, x, w, b, lut)
    for tune in (0, 1):
        hip.set_tuning(tune)
        try:
            y = hip.conv2d_f32(dn, xd, wd, bd, ld).cpu().numpy()
            yt = hip.conv2d_f32(d, xd, wd, bd, ld).cpu().numpy() if table else None
        finally:
            hip.set_tuning(0)
        if d.group != 1:
            assert np.array_equal(y, ref), f"{name}: depthwise differs from the reference's order of operations"
        else:
            assert_close_f32(y, ref, tag=f"{name} tuning {tune}", elementwise=False)
        if table:
            assert np.array_equal(yt, oracle.lut_act(y, lut)), f"{name}: table lookup differs"


@pytest.mark.parametrize("seed", range(24))
def test_conv_w8a32_random_shapes_bit_exact(seed, torch_dev, oracle):
    torch = torch_dev
    rng = np.random.default_rng(2000 + seed)
    d = _random_conv(rng, quant=True)
    if not d.has_bias:
        d.act_type = abi.NOT_ACT
    name = f"random_q_{seed}"
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    oh, ow = d.out_hw()
    acc = torch.empty((d.n, d.cout, oh, ow), dtype=torch.int32, device="cuda")
    y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32) if b32 is not None else None, dev(torch, aux),
                         dev(torch, cases.silu_lut()), acc32=acc)
    torch.cuda.synchronize()
    ref, ref_acc = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut(), want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), ref_acc), f"{name}: int32 accumulators differ"
    assert np.array_equal(y.cpu().numpy(), ref), f"{name}: de-quantised outputs differ"


@pytest.mark.parametrize("seed", range(24))
def test_conv_w8a8_chain_random_shapes(seed, torch_dev, oracle):
    """the int8 NHWC chain form on seeded random dense convolutions: the reference's int8 values exactly"""
    torch = torch_dev
    rng = np.random.default_rng(9000 + seed)
    d = _random_conv(rng, quant=True)
    if d.group != 1:
        d.group, d.cout = 1, int(rng.integers(1, 100))
    if not d.has_bias:
        d.act_type = abi.NOT_ACT
    d.out_s8, d.output_scale = 1, float(rng.uniform(0.01, 0.08))
    x, w8, b32, aux = cases.conv_inputs(f"random_chain_{seed}", d, quant=True)
    ref = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut())
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale)
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    oh, ow = d.out_hw()
    out = torch.full((d.n, oh, ow, (d.cout + 15) // 16 * 16), 77, dtype=torch.int8, device="cuda")
    yq = hip.conv2d_w8a8_nhwc(d, xq, wp, dev(torch, b32) if b32 is not None else None, dev(torch, aux),
                              dev(torch, cases.silu_lut()), out=out)
    torch.cuda.synchronize()
    assert np.array_equal(yq.cpu().numpy()[..., :d.cout], np.transpose(ref, (0, 2, 3, 1)))


@pytest.mark.parametrize("seed", range(24))
def test_conv_add_random_shapes(seed, torch_dev):
    """the folded residual store on seeded random convolutions (cost model's tile choice, the same for both forms):
    the bits of conv, Add and Relu run one after the other"""
    torch = torch_dev
    rng = np.random.default_rng(5000 + seed)
    d = _random_conv(rng, quant=False)
    x, w, b = cases.conv_inputs(f"random_res_{seed}", d)
    oh, ow = d.out_hw()
    r = rng.normal(size=(d.n, d.cout, oh, ow)).astype(np.float32)
    lut = dev(torch, cases.silu_lut())
    xd, wd, rd = dev(torch, x), dev(torch, w), dev(torch, r)
    bd = dev(torch, b) if b is not None else None
    for relu in (False, True):
        want = hip.add_f32(hip.conv2d_f32(d, xd, wd, bd, lut), rd)
        if relu:
            want = hip.relu_f32(want)
        got = hip.conv2d_f32_add(d, xd, wd, rd, bias=bd, silu_lut=lut, relu=relu)
        torch.cuda.synchronize()
        assert _same_bits(got.cpu().numpy(), want.cpu().numpy()), (seed, relu)


@pytest.mark.parametrize("shape", [(58, 13, 32, 3, 3, 0), (39, 33, 11, 3, 3, 0), (4, 22, 36, 1, 3, 0), (31, 39, 20, 3, 2, 0),
                                   (64, 29, 23, 5, 3, 1), (30, 14, 12, 3, 3, 1), (7, 16, 32, 5, 2, 0), (9, 61, 100, 3, 3, 1)])
@pytest.mark.parametrize("quant", [False, True])
def test_depthwise_stride_leaves_rows_and_columns_unread(shape, quant, torch_dev, oracle):
    """a stride above 1 whose last window ends before the image does (found by the random sweep: the copy of the image
    into the LDS tile had no cells for those rows and columns and wrote over its neighbours); small planes staged flat
    and a plane wide enough for the row-walking copy, fp32 and W8A32, bit for bit"""
    torch = torch_dev
    c, h, w, k, s, pad = shape
    d = cases.cd(c, c, k, s, pad, h, w, act=abi.RELU, group=c, n=2, input_scale=0.02)
    name = f"dw_unread_{shape}_{quant}"
    if quant:
        x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
        y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, cases.silu_lut()))
        ref = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut())
    else:
        x, wt, b = cases.conv_inputs(name, d)
        y = hip.conv2d_f32(d, dev(torch, x), dev(torch, wt), dev(torch, b))
        ref = oracle.conv2d_f32(d, x, wt, b, cases.silu_lut())
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), ref)


def _has_packed_form(d):
    """dense, not a plain 1x1; the first-layer kernel's shapes, or at least four input channels and at most 64 taps"""
    if d.group != 1 or (d.kh == 1 and d.kw == 1 and d.pad_t == 0):
        return False
    first_layer = d.cin == 3 and d.cout <= 64 and d.kh == d.kw and d.kh in (3, 7) and d.stride_h == d.stride_w and d.stride_h <= 2
    return first_layer or (d.cin >= 4 and d.kh * d.kw <= 64)


PACKED_CASES = [n for n, d in cases.conv_f32_cases().items() if _has_packed_form(d)]
UNPACKED_DENSE_CASES = [n for n, d in cases.conv_f32_cases().items()
                        if d.group == 1 and not (d.kh == 1 and d.kw == 1 and d.pad_t == 0) and not _has_packed_form(d)]


@pytest.mark.parametrize("name", PACKED_CASES)
def test_conv_f32_packed_weights(name, torch_dev, oracle):
    """tap-major packed weights: same convolution, the reduction merely runs in another order"""
    torch = torch_dev
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    wd = dev(torch, w)
    wp = hip.pack_conv_weights(d, wd)
    assert wp is not None
    dn = ConvDesc.from_buffer_copy(d)
    if d.has_bias and d.act_type == abi.SILU:
        dn.act_type = abi.NOT_ACT      # judged on the pre-activation; the table lookup is tested elsewhere
    y = hip.conv2d_f32(dn, dev(torch, x), wp, dev(torch, b), None, packed=True)
    torch.cuda.synchronize()
    assert_close_f32(y.cpu().numpy(), oracle.conv2d_f32(dn, x, w, b), tag=name + " packed")


@pytest.mark.parametrize("name", UNPACKED_DENSE_CASES)
def test_conv_f32_shapes_without_a_packed_form(name, torch_dev):
    """fewer than four input channels or more than 64 filter taps (first-layer shapes apart): the library says that the
    weights are taken as they are, and refuses to pack them or to be handed packed ones"""
    torch = torch_dev
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    wd = dev(torch, w)
    assert hip.pack_conv_weights(d, wd) is None
    with pytest.raises(hip.OnhipError):
        hip.conv2d_f32(d, dev(torch, x), wd, dev(torch, b), None, packed=True)


@pytest.mark.parametrize("compute", [abi.COMPUTE_BF16, abi.COMPUTE_F16])
def test_conv_packed_reduced_precision(compute, torch_dev, oracle):
    torch = torch_dev
    for name in ("cfg1_64x56_3x3", "c7x7_s2_p3"):
        d = ConvDesc.from_buffer_copy(cases.conv_f32_cases()[name])
        d.compute = compute
        x, w, b = cases.conv_inputs(name, d)
        wp = hip.pack_conv_weights(d, dev(torch, w))
        assert (wp is None) == (d.cin < 4)   # three input channels at reduced precision: no packed form, the element gather
        y = hip.conv2d_f32(d, dev(torch, x), wp if wp is not None else dev(torch, w), dev(torch, b), None, packed=wp is not None)
        torch.cuda.synchronize()
        rnd = oracle.round_bf16 if compute == abi.COMPUTE_BF16 else oracle.round_f16
        assert_close_f32(y.cpu().numpy(), oracle.conv2d_f32(d, rnd(x), rnd(w), b), rel=1e-4, tag=name + " packed")


@pytest.mark.parametrize("name", list(cases.conv_w8a32_cases()))
def test_conv_w8a32_bit_exact(name, torch_dev, oracle, golden):
    torch = torch_dev
    d = cases.conv_w8a32_cases()[name]
    print(f"case {name}", flush=True)
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    oh, ow = d.out_hw()
    acc = torch.empty((d.n, d.cout, oh, ow), dtype=torch.int32, device="cuda")
    y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux),
                         dev(torch, cases.silu_lut()), acc32=acc)
    torch.cuda.synchronize()
    ref, ref_acc = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut(), want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), ref_acc), f"{name}: int32 accumulators differ"
    y = y.cpu().numpy()
    assert np.array_equal(y, ref), f"{name}: {(y != ref).sum()} de-quantised outputs differ"
    cases.check_against(golden, name, y, exact=True)
    # the same through weights laid out once for the kernel
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    assert (wp is None) == (d.group != 1)
    if wp is not None:
        y2 = hip.conv2d_w8a32(d, dev(torch, x), wp, dev(torch, b32), dev(torch, aux), dev(torch, cases.silu_lut()),
                              packed=True)
        torch.cuda.synchronize()
        assert np.array_equal(y2.cpu().numpy(), ref), f"{name}: packed weights give other results"


@pytest.mark.parametrize("name", ["q3x3_silu", "q3x3_s2", "qdw3x3", "yolo_c2f_3x3_64_80"])
def test_conv_w8a32_requant_s8(name, torch_dev, oracle):
    """int8 output = the consumer's input quantisation of the fp32 result: exact, so <= 1 LSB"""
    torch = torch_dev
    d = ConvDesc.from_buffer_copy(cases.conv_w8a32_cases()[name])
    d.out_s8, d.output_scale = 1, 0.037
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, cases.silu_lut()))
    torch.cuda.synchronize()
    ref = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut())
    assert y.dtype == torch.int8 and np.array_equal(y.cpu().numpy(), ref)


@pytest.mark.parametrize("name,batch", [("c3x3_tiny_relu", 3), ("c1x1_unaligned_clip", 5), ("c7x7_s2_p3", 2),
                                        ("dw3x3_s2_odd", 4), ("cfg1_64x56_3x3", 2), ("rn50_l4_3x3", 33)])
def test_conv_f32_batched(name, batch, torch_dev, oracle):
    """a batch is that many independent batch-1 evaluations of the reference"""
    torch = torch_dev
    d = ConvDesc.from_buffer_copy(cases.conv_f32_cases()[name])
    d.n = batch
    x, w, b, y = run_conv_f32(torch, name + "_batched", d)
    ref = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    if d.group != 1:
        assert np.array_equal(y, ref)
    else:
        assert_close_f32(y, ref, tag=name)


@pytest.mark.parametrize("tile", ["64x64x1", "64x64x3", "32x128x2", "64x128x5", "128x128x4", "128x128x1",
                                  # the same splits with the slices added up inside the launch by the last to arrive
                                  "64x64x3x0x0x1", "32x128x2x0x0x1", "64x128x5x0x0x1", "128x128x4x0x0x1"])
@pytest.mark.parametrize("kind", ["1x1_ragged_k", "3x3_packed"])
def test_forced_tile_and_split_many_items(tile, kind, torch_dev, oracle, monkeypatch):
    """every tile shape, with and without split-K, on problems with more work items than resident
    workgroups (each workgroup walks through several tiles) and a K that ends inside a K tile;
    run twice: the split-K arrival counters must be back at zero after a launch"""
    torch = torch_dev
    if kind == "1x1_ragged_k":
        d = cases.cd(198, 96, 1, 1, 0, 48, n=24, act=abi.RELU)         # K = 198: ragged, odd
    else:
        d = cases.cd(24, 80, 3, 1, 1, 40, n=40, act=abi.CLIP, clip_min=-0.5, clip_max=0.7)
    x, w, b = cases.conv_inputs("forced_" + kind, d)
    ref = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    monkeypatch.setenv("ONHIP_TILE", tile)
    xd, wd, bd = dev(torch, x), dev(torch, w), dev(torch, b)
    wp = hip.pack_conv_weights(d, wd) if kind == "3x3_packed" else None
    for rep in range(2):
        if wp is not None:
            y = hip.conv2d_f32(d, xd, wp, bd, packed=True)
        else:
            y = hip.conv2d_f32(d, xd, wd, bd)
        torch.cuda.synchronize()
        assert_close_f32(y.cpu().numpy(), ref, tag=f"{kind} {tile} run {rep}")


@pytest.mark.parametrize("tile", ["64x64x4x0x0x1", "64x128x3x0x0x1", "64x64x16x0x0x1"])
def test_split_k_added_up_inside_the_launch_is_the_finishing_pass_bit_for_bit(tile, torch_dev, monkeypatch):
    """the last slice of a tile to arrive adds the partial sums up in slice order, as the finishing kernel does: the same
    bits as that kernel on the same split, two hundred launches in a row (whichever slice arrives last), with a launch
    of another shape in between so that the counters and the workspace are reused"""
    torch = torch_dev
    d = cases.cd(200, 100, 3, 1, 1, 14, 15, n=6, act=abi.RELU)           # K = 1800: 113 K tiles, ragged rows and columns
    x, w, b = cases.conv_inputs("inlaunch_" + tile, d)
    xd, wd, bd = dev(torch, x), dev(torch, w), dev(torch, b)
    wp = hip.pack_conv_weights(d, wd)
    d2 = cases.cd(64, 40, 1, 1, 0, 9, n=2, act=abi.NOT_ACT)
    x2, w2, b2 = cases.conv_inputs("inlaunch_other", d2)
    x2d, w2d, b2d = dev(torch, x2), dev(torch, w2), dev(torch, b2)
    monkeypatch.setenv("ONHIP_TILE", tile.rsplit("x", 3)[0])               # the same tile and split, finishing launch
    want = hip.conv2d_f32(d, xd, wp, bd, packed=True).cpu().numpy()
    want2 = hip.conv2d_f32(d2, x2d, w2d, b2d).cpu().numpy()
    monkeypatch.setenv("ONHIP_TILE", tile)
    for rep in range(200):
        y = hip.conv2d_f32(d, xd, wp, bd, packed=True)
        if rep % 10 == 0:
            y2 = hip.conv2d_f32(d2, x2d, w2d, b2d)
            assert _same_bits(y2.cpu().numpy(), want2), rep
        assert _same_bits(y.cpu().numpy(), want), rep


@pytest.mark.parametrize("tile,shape", [("64x64x1x8", (20, 30, 29)), ("64x64x1x16", (17, 32, 32)), ("64x128x1x4", (34, 32, 34)),
                                        ("32x128x1x8", (33, 32, 33)), ("128x128x1x2", (80, 24, 36)),
                                        # the same through the kernel that reads B straight from memory (1x1 and matmul;
                                        # the 3x3 case falls back to the tiled kernel with the same split)
                                        ("64x128x1x4x1", (34, 32, 34)), ("128x128x1x2x1", (80, 24, 36)),
                                        ("64x256x1x4x1", (34, 32, 36)), ("96x128x1x4x1", (34, 32, 34)),
                                        ("32x512x1x8x1", (34, 32, 32)),
                                        # leftover tiles whose slices are added up inside the launch
                                        ("64x64x1x8x0x1", (20, 30, 29)), ("64x128x1x4x0x1", (34, 32, 34))])
@pytest.mark.parametrize("kind", ["3x3_packed", "1x1", "matmul"])
def test_leftover_tiles_as_a_split_launch(tile, shape, kind, torch_dev, oracle, monkeypatch):
    """the launch cut along N: whole rounds of 256 tiles unsplit on the caller's stream, the leftover column blocks
    split along K on the side stream, joined by events.  Shapes with more than 256 tiles, a ragged last column
    block and (100 output channels) a ragged last row block; run three times, interleaved with an ordinary launch
    on the same stream that reads the result"""
    torch = torch_dev
    n, h, w_ = shape
    monkeypatch.setenv("ONHIP_TILE", tile)
    if kind == "matmul":
        rng = np.random.default_rng(7)
        a = (rng.normal(size=(100, 528)) * 0.05).astype(np.float32)          # 100 rows, as many columns as the conv has pixels
        b = rng.normal(size=(528, n * h * w_)).astype(np.float32)
        ref = oracle.matmul_f32(a, b)
        before = hip.split_tail_launches()
        for rep in range(2):
            y = hip.matmul(dev(torch, a), dev(torch, b))
            torch.cuda.synchronize()
            assert_close_f32(y.cpu().numpy(), ref, tag=f"matmul {tile} run {rep}")
        assert hip.split_tail_launches() == before + 2
        return
    if kind == "3x3_packed":
        d = cases.cd(64, 100, 3, 1, 1, h, w_, n=n, act=abi.RELU)              # K = 576: 36 K tiles, enough for 16 slices
    else:
        d = cases.cd(520, 100, 1, 1, 0, h, w_, n=n, act=abi.CLIP, clip_min=-0.4, clip_max=0.9)
    x, w, b = cases.conv_inputs(f"tail_{kind}_{tile}", d)
    ref = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    xd, wd, bd = dev(torch, x), dev(torch, w), dev(torch, b)
    wp = hip.pack_conv_weights(d, wd) if kind == "3x3_packed" else None
    before = hip.split_tail_launches()
    for rep in range(3):
        y = hip.conv2d_f32(d, xd, wp, bd, packed=True) if wp is not None else hip.conv2d_f32(d, xd, wd, bd)
        doubled = hip.add_f32(y, y)                                            # stream-ordered consumer of the result
        torch.cuda.synchronize()
        assert_close_f32(y.cpu().numpy(), ref, tag=f"{kind} {tile} run {rep}")
        assert np.array_equal(doubled.cpu().numpy(), 2 * y.cpu().numpy())
    assert hip.split_tail_launches() == before + 3                             # the shape does have leftover tiles


@pytest.mark.parametrize("tile", ["64x128x1x0x1", "128x128x1x0x1", "64x256x1x0x1", "96x128x1x0x1", "32x256x1x0x1", "32x512x1x0x1"])
@pytest.mark.parametrize("kind", ["conv_k200_m100", "conv_silu_k64", "conv_nobias", "matmul_batched_bias_gelu", "matmul_shared",
                                  "not_applicable"])
def test_kernel_with_b_straight_from_memory(tile, kind, torch_dev, oracle, monkeypatch):
    """the fp32 kernel whose B operand never passes through LDS: 1x1 stride-1 convolutions and matrix products with K,
    N and the pixels per image multiples of 4.  Ragged rows (100 channels), a last K tile of 8, column counts that end
    inside a tile, several images, every epilogue; a problem it cannot take falls back to the tiled kernel."""
    torch = torch_dev
    monkeypatch.setenv("ONHIP_TILE", tile)
    if kind.startswith("matmul"):
        rng = np.random.default_rng(21)
        if kind == "matmul_batched_bias_gelu":
            a = (rng.normal(size=(3, 70, 136)) * 0.1).astype(np.float32)
            b = rng.normal(size=(3, 136, 300)).astype(np.float32)
            bias = rng.normal(size=(300,)).astype(np.float32)
            lut = cases.gelu_lut()
            ref = oracle.matmul_f32(a, b, bias, lut)
            y = hip.matmul(dev(torch, a), dev(torch, b), bias=dev(torch, bias), gelu_lut=dev(torch, lut))
        else:
            a = (rng.normal(size=(2, 197, 192)) * 0.1).astype(np.float32)
            b = rng.normal(size=(192, 576)).astype(np.float32)
            ref = oracle.matmul_f32(a, b)
            y = hip.matmul(dev(torch, a), dev(torch, b))
        torch.cuda.synchronize()
        if kind == "matmul_batched_bias_gelu":   # table activation: a step function of the sum (see the SILU case below)
            err = np.abs(y.cpu().numpy() - ref)
            assert err.max() <= 1.2 / 512 + 1e-4 * np.abs(ref).max() and np.mean(err > 1e-4 * np.abs(ref).max()) < 2e-3
        else:
            assert_close_f32(y.cpu().numpy(), ref, tag=f"{kind} {tile}")
        return
    d = {"conv_k200_m100": cases.cd(200, 100, 1, 1, 0, 20, 18, n=5, act=abi.RELU),
         "conv_silu_k64": cases.cd(64, 256, 1, 1, 0, 28, 28, n=3, act=abi.SILU),
         "conv_nobias": cases.cd(32, 48, 1, 1, 0, 12, 12, n=2, bias=0, act=abi.NOT_ACT),
         "not_applicable": cases.cd(30, 40, 1, 1, 0, 7, 7, n=3, act=abi.RELU)}[kind]       # K = 30, 49 pixels per image
    x, w, b = cases.conv_inputs(f"rowb_{kind}", d)
    ref = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    y = hip.conv2d_f32(d, dev(torch, x), dev(torch, w), dev(torch, b), dev(torch, cases.silu_lut()))
    torch.cuda.synchronize()
    if d.act_type == abi.SILU:
        # the table is a step function of the pre-activation: a last-bit difference in the sum may move an output to
        # the neighbouring entry (slope below 1.1, step 1/512)
        assert np.abs(y.cpu().numpy() - ref).max() <= 1.1 / 512 + 1e-4 * np.abs(ref).max()
        assert np.mean(np.abs(y.cpu().numpy() - ref) > 1e-4 * np.abs(ref).max()) < 2e-3
    else:
        assert_close_f32(y.cpu().numpy(), ref, tag=f"{kind} {tile}")


@pytest.mark.parametrize("tile", ["64x64x4", "128x128x2", "32x128x1"])
def test_forced_split_w8a32_bit_exact(tile, torch_dev, oracle, monkeypatch):
    """integer partial sums add up exactly whatever the split"""
    torch = torch_dev
    d = ConvDesc.from_buffer_copy(cases.conv_w8a32_cases()["q3x3_silu"])
    d.n = 6
    x, w8, b32, aux = cases.conv_inputs("q_forced_split", d, quant=True)
    ref = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut())
    monkeypatch.setenv("ONHIP_TILE", tile)
    for rep in range(2):
        y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, cases.silu_lut()))
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), ref), f"{tile} run {rep}"


def test_conv_w8a32_batched(torch_dev, oracle):
    torch = torch_dev
    d = ConvDesc.from_buffer_copy(cases.conv_w8a32_cases()["q3x3_s2_odd"])
    d.n = 5
    x, w8, b32, aux = cases.conv_inputs("q_batched", d, quant=True)
    y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, cases.silu_lut()))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut()))


@pytest.mark.parametrize("shape", [(2, 64, 7, 2, 3, 224, 224, abi.RELU, 1), (1, 32, 3, 2, 1, 224, 224, abi.CLIP, 1),
                                   (1, 40, 3, 1, 1, 20, 200, abi.RELU, 1), (1, 8, 7, 1, 3, 9, 130, abi.NOT_ACT, 1),
                                   (2, 33, 3, 2, 1, 37, 300, abi.LEAKYRELU, 1), (1, 64, 7, 2, 3, 64, 260, abi.RELU, 0)])
@pytest.mark.parametrize("packed", [False, True])
def test_conv_f32_first_layer_kernel(shape, packed, torch_dev, oracle):
    """three input channels, rows of at least 96 output pixels: the kernel that multiplies out of an LDS patch of the
    input (one and several 128-pixel segments per row, ragged last segment, both filter sizes, both strides, with and
    without bias, weights as given and tap-major packed); 1e-4 against the oracle like every fp32 convolution"""
    torch = torch_dev
    n, cout, k, stride, pad, h, w, act, bias = shape
    d = cases.cd(3, cout, k, stride, pad, h, w=w, n=n, act=act, bias=bias, clip_min=0.0, clip_max=0.8, leaky_relu_alpha=0.1)
    name = f"stem_{cout}_{k}_{stride}_{h}x{w}"
    x, wt, b = cases.conv_inputs(name, d)
    wd = dev(torch, wt)
    if packed:
        y = hip.conv2d_f32(d, dev(torch, x), hip.pack_conv_weights(d, wd), dev(torch, b), packed=True)
    else:
        y = hip.conv2d_f32(d, dev(torch, x), wd, dev(torch, b))
    torch.cuda.synchronize()
    assert_close_f32(y.cpu().numpy(), oracle.conv2d_f32(d, x, wt, b), tag=name)


@pytest.mark.parametrize("compute,name", [(abi.COMPUTE_BF16, "cfg1_64x56_3x3"), (abi.COMPUTE_F16, "cfg1_64x56_3x3"),
                                          (abi.COMPUTE_BF16, "c7x7_s2_p3"), (abi.COMPUTE_F16, "c1x1_unaligned_clip")])
def test_conv_reduced_precision_modes(compute, name, torch_dev, oracle):
    """bf16 / fp16 MFMA with fp32 accumulation: equals the reference arithmetic on operands rounded
    to that type (tight), and stays within 1e-2 of the fp32 reference"""
    torch = torch_dev
    d = cases.conv_f32_cases()[name]
    x, w, b, y = run_conv_f32(torch, name, d, compute=compute)
    rnd = oracle.round_bf16 if compute == abi.COMPUTE_BF16 else oracle.round_f16
    assert_close_f32(y, oracle.conv2d_f32(d, rnd(x), rnd(w), b, cases.silu_lut()), rel=1e-4, tag=name + " rounded operands")
    assert_close_f32(y, oracle.conv2d_f32(d, x, w, b, cases.silu_lut()), rel=1e-2, tag=name + " vs fp32",
                     elementwise=False)


@pytest.mark.parametrize("name", list(cases.matmul_cases()))
def test_matmul_f32(name, torch_dev, oracle, golden):
    torch = torch_dev
    a, b = cases.matmul_inputs(name, *cases.matmul_cases()[name])
    y = hip.matmul(dev(torch, a), dev(torch, b))
    torch.cuda.synchronize()
    y = y.cpu().numpy()
    ref = oracle.matmul_f32(a, b)
    assert_close_f32(y, ref, tag=name)
    cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-4 * float(np.abs(ref).max()))


@pytest.mark.parametrize("compute", [abi.COMPUTE_F32, abi.COMPUTE_BF16, abi.COMPUTE_F16])
@pytest.mark.parametrize("batch", [1, 4])
def test_matmul_bias_gelu_fused(compute, batch, torch_dev, oracle):
    """fused MatMul + bias + table GELU == the reference chain MatMul -> Add -> Gelu (ViT MLP fc1)"""
    torch = torch_dev
    a, w = cases.matmul_inputs("vit_fc1", (batch, 197, 192), (192, 768))
    bias = cases.datagen.normal(cases.datagen.seed_for("vit_fc1", "bias"), (768,), 0.0, 0.02)
    lut = cases.gelu_lut()
    pre = hip.matmul(dev(torch, a), dev(torch, w), bias=dev(torch, bias), compute=compute)
    y = hip.matmul(dev(torch, a), dev(torch, w), bias=dev(torch, bias), gelu_lut=dev(torch, lut), compute=compute)
    torch.cuda.synchronize()
    pre, y = pre.cpu().numpy(), y.cpu().numpy()
    ref_pre = oracle.matmul_f32(a, w, bias=bias)
    assert_close_f32(pre, ref_pre, rel=1e-4 if compute == abi.COMPUTE_F32 else 1e-2, tag="fc1 pre-activation",
                     elementwise=compute == abi.COMPUTE_F32)
    assert np.array_equal(y, oracle.lut_act(pre, lut)), "table GELU differs from the table applied to the kernel's sum"
    if compute == abi.COMPUTE_F32:
        # away from bin edges the fused result equals the reference chain
        ref = oracle.matmul_f32(a, w, bias=bias, gelu=lut)
        assert np.mean(y == ref) > 0.98 and np.abs(y - ref).max() < 5e-3


@pytest.mark.parametrize("compute", [abi.COMPUTE_F32, abi.COMPUTE_BF16])
@pytest.mark.parametrize("shape", [((4, 197, 192), (192, 192)), ((2, 196, 768), (768, 192)), ((3, 37, 50), (3, 50, 21))])
def test_matmul_bias_add_fused(shape, compute, torch_dev, oracle):
    """MatMul -> Add of a bias -> Add of a skip tensor in one call == the three operators one after the other (the sums are
    formed in the same order on the same values: bit for bit), and, in fp32, the oracle's chain within 1e-4"""
    torch = torch_dev
    a, w = cases.matmul_inputs("vit_proj", *shape)
    n = shape[1][-1]
    bias = cases.datagen.normal(cases.datagen.seed_for("vit_proj", "bias", n), (n,), 0.0, 0.05)
    skip = cases.datagen.normal(cases.datagen.seed_for("vit_proj", "skip", n), shape[0][:-1] + (n,), 0.0, 1.0)
    for b in (bias, None):
        kw = dict(bias=dev(torch, b)) if b is not None else {}
        y = hip.matmul(dev(torch, a), dev(torch, w), addend=dev(torch, skip), compute=compute, **kw)
        pre = hip.matmul(dev(torch, a), dev(torch, w), compute=compute, **kw)
        torch.cuda.synchronize()
        y, pre = y.cpu().numpy(), pre.cpu().numpy()
        assert np.array_equal(y, oracle.add_f32(pre, skip))
        if compute == abi.COMPUTE_F32:
            assert_close_f32(y, oracle.add_f32(oracle.matmul_f32(a, w, bias=b), skip), rel=1e-4, tag="proj + skip")
    with pytest.raises(hip.OnhipError):
        out = dev(torch, skip)
        hip.matmul(dev(torch, a), dev(torch, w), addend=out, out=out)


def test_plugin_matmul_fused_entries_host_buffers(torch_dev, oracle):
    """eval_bias, eval_bias_gelu and eval_bias_add of the MatMul plugin on tensors in host memory: each equal, bit for bit,
    to the operators it replaces as this library computes them (MatMul through `eval`, then the oracle's Add / table Gelu /
    Add on that result)"""
    a, w = cases.matmul_inputs("plug_linear", (3, 37, 48), (48, 40))
    bias = cases.datagen.normal(cases.datagen.seed_for("plug_linear", "bias"), (40,), 0.0, 0.2)
    skip = cases.datagen.normal(cases.datagen.seed_for("plug_linear", "skip"), (3, 37, 40), 0.0, 1.0)
    lut = cases.gelu_lut()
    plug = ops.Plugin(hip.plugin_path("MatMul"))
    plain = ops.MatMul(plug.eval)(a, w)
    fused = ops.MatMulFused(plug)
    with_bias = oracle.add_f32(plain, bias)
    assert np.array_equal(fused.linear(a, w, bias), with_bias)
    assert np.array_equal(fused.linear(a, w, bias, gelu_lut=lut), oracle.lut_act(with_bias, lut))
    assert np.array_equal(fused.linear(a, w, bias, addend=skip), oracle.add_f32(with_bias, skip))
    assert_close_f32(with_bias, oracle.matmul_f32(a, w, bias=bias), rel=1e-4, tag="plugin linear")


@pytest.mark.parametrize("name", list(cases.gemm_cases()))
def test_gemm_f32(name, torch_dev, oracle, golden):
    torch = torch_dev
    a, w, b = cases.gemm_inputs(name, *cases.gemm_cases()[name])
    y = hip.gemm_f32(dev(torch, a), dev(torch, w), dev(torch, b))
    torch.cuda.synchronize()
    y = y.cpu().numpy()
    ref = oracle.gemm_f32(a, w, b)
    assert_close_f32(y, ref, tag=name)
    cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-4 * float(np.abs(ref).max()))


@pytest.mark.parametrize("shape", [(9, 2048, 1000), (32, 2048, 1000), (33, 1283, 37), (200, 64, 5), (8, 300, 70)])
def test_gemm_many_rows_runs_as_a_matrix_product(shape, torch_dev, oracle):
    """more than eight rows of A go through the MFMA kernel (the rows as one-pixel images of a 1x1 convolution), eight
    and fewer through the skinny kernel; odd K, N below a tile, ragged M"""
    torch = torch_dev
    a, w, b = cases.gemm_inputs(f"gemm_rows_{shape}", *shape)
    y = hip.gemm_f32(dev(torch, a), dev(torch, w), dev(torch, b))
    torch.cuda.synchronize()
    assert_close_f32(y.cpu().numpy(), oracle.gemm_f32(a, w, b), tag=str(shape))


# ---- the last convolution of a residual block with the Add and the Relu folded into its store ------------------

def _residual_case(kind):
    if kind == "1x1_resnet":          # a ResNet conv3: 1x1, no activation of its own
        return cases.cd(64, 256, 1, 1, 0, 28, act=abi.NOT_ACT, n=2)
    if kind == "1x1_ragged":          # 100 channels, 29x29: ragged tiles both ways, element count not a multiple of 32
        return cases.cd(72, 100, 1, 1, 0, 29, act=abi.NOT_ACT, n=3)
    if kind == "3x3_packed_relu":     # activation before the Add, then the block's Relu
        return cases.cd(32, 48, 3, 1, 1, 19, 23, act=abi.RELU, n=2)
    if kind == "3x3_s2_gather":       # weights as they are: the gathering loader
        return cases.cd(24, 40, 3, 2, 1, 30, act=abi.CLIP, n=2, clip_min=-0.2, clip_max=0.5)
    if kind == "mobilenet_project":   # MobileNetV2 project layer: few output channels, linear
        return cases.cd(144, 24, 1, 1, 0, 56, act=abi.NOT_ACT, n=2)
    if kind == "depthwise":           # no folded store on this path: the entry point runs the passes itself
        return cases.cd(48, 48, 3, 1, 1, 20, act=abi.NOT_ACT, group=48, n=2)
    if kind == "nobias":
        return cases.cd(64, 64, 1, 1, 0, 16, act=abi.NOT_ACT, bias=0, n=1)
    raise KeyError(kind)


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("tile", [None, "64x64x1", "64x64x3", "32x128x2", "128x128x1", "64x128x1x4", "64x128x1x0x1",
                                  "64x64x3x0x0x1", "128x128x2x0x0x1"])
@pytest.mark.parametrize("kind", ["1x1_resnet", "1x1_ragged", "3x3_packed_relu", "3x3_s2_gather", "mobilenet_project",
                                  "depthwise", "nobias"])
def test_conv_with_add_and_relu_folded_in(kind, tile, relu, torch_dev, oracle, monkeypatch):
    """onhip_conv2d_f32_add against the three operators run one after the other on the same launch configuration:
    the same bits, whichever kernel stores the result (whole tiles, split K with its finishing pass, leftover tiles;
    a forced row-B tile falls back to the tiled kernel).  The addend holds NaNs in the part of the tensor that
    relu.c's vector body covers and in its scalar tail, where the two rules of that operator differ."""
    torch = torch_dev
    if tile is not None:
        monkeypatch.setenv("ONHIP_TILE", tile)
    d = _residual_case(kind)
    if kind == "depthwise" and tile is not None:
        pytest.skip("one kernel only")
    x, w, b = cases.conv_inputs(f"res_{kind}", d)
    oh, ow = d.out_hw()
    r = datagen.uniform(datagen.seed_for(f"res_{kind}", "r"), (d.n, d.cout, oh, ow), -1.0, 1.0)
    flat = r.reshape(-1)
    flat[5] = np.nan
    flat[-1] = np.nan                      # in the tail whenever the element count is not a multiple of 32
    flat[7] = -0.0
    xd, wd, rd = dev(torch, x), dev(torch, w), dev(torch, r)
    bd = dev(torch, b) if b is not None else None
    packed = kind.startswith("3x3_packed")
    if packed:
        wd = hip.pack_conv_weights(d, wd)
    plain = hip.conv2d_f32(d, xd, wd, bd, packed=packed)
    want = hip.add_f32(plain, rd)
    if relu:
        want = hip.relu_f32(want)
    for rep in range(2):
        got = hip.conv2d_f32_add(d, xd, wd, rd, bias=bd, relu=relu, packed=packed)
        torch.cuda.synchronize()
        assert _same_bits(got.cpu().numpy(), want.cpu().numpy()), f"{kind} tile {tile} relu {relu} run {rep}"
    # and the sum is the sum: against the oracle's convolution, away from the planted NaNs
    ref = oracle.conv2d_f32(d, x, w, b, cases.silu_lut()) + r
    if relu:
        ref = np.where(ref > 0, ref, 0).astype(np.float32)
    ok = ~np.isnan(r)
    assert_close_f32(np.where(ok, got.cpu().numpy(), 0), np.where(ok, ref, 0), tag=f"{kind} against the oracle")


@pytest.mark.parametrize("relu", [False, True])
def test_conv_with_add_folded_in_leftover_tiles(relu, torch_dev, monkeypatch):
    """more tiles than one round of the chip: whole tiles store the sum themselves, the finishing pass of the split
    leftover tiles adds it for its columns"""
    torch = torch_dev
    monkeypatch.setenv("ONHIP_TILE", "64x64x1x8")
    d = cases.cd(520, 100, 1, 1, 0, 30, 29, n=20, act=abi.NOT_ACT)
    x, w, b = cases.conv_inputs("res_tail", d)
    r = datagen.uniform(datagen.seed_for("res_tail", "r"), (20, 100, 30, 29), -1.0, 1.0)
    xd, wd, bd, rd = dev(torch, x), dev(torch, w), dev(torch, b), dev(torch, r)
    before = hip.split_tail_launches()
    want = hip.add_f32(hip.conv2d_f32(d, xd, wd, bd), rd)
    if relu:
        want = hip.relu_f32(want)
    got = hip.conv2d_f32_add(d, xd, wd, rd, bias=bd, relu=relu)
    torch.cuda.synchronize()
    assert hip.split_tail_launches() == before + 2
    assert _same_bits(got.cpu().numpy(), want.cpu().numpy())


def test_conv_add_refuses_the_output_as_addend(torch_dev):
    torch = torch_dev
    d = _residual_case("nobias")
    x, w, _ = cases.conv_inputs("res_alias", d)
    y = torch.zeros((1, 64, 16, 16), dtype=torch.float32, device="cuda")
    with pytest.raises(hip.OnhipError):
        hip.conv2d_f32_add(d, dev(torch, x), dev(torch, w), y, out=y)


@pytest.mark.parametrize("name", ["c3x3_tiny_relu", "c1x1_unaligned_clip", "dw3x3_s2_even", "rn50_l4_1x1_2048_512"])
def test_plugin_conv_eval_add_host_buffers(name, torch_dev):
    """libConv_hip.so's eval_add / eval_add_relu: slots as for eval plus the addend in inputs[3]; against eval
    followed by the Add and Relu plugins"""
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    oh, ow = d.out_hw()
    r = datagen.uniform(datagen.seed_for(name, "residual"), (d.n, d.cout, oh, ow), -1.0, 1.0)
    plug = ops.Plugin(hip.plugin_path("Conv"))
    assert plug.eval_add is not None and plug.eval_add_relu is not None
    y = ops.Conv(plug.eval, d, w, b, silu_lut=cases.silu_lut())(x)
    add = ops.Add(ops.Plugin(hip.plugin_path("Add")).eval)
    relu = ops.Relu(ops.Plugin(hip.plugin_path("Relu")).eval)
    summed = add(y, r)
    got = ops.Conv(plug.eval_add, d, w, b, silu_lut=cases.silu_lut())(x, addend=r)
    assert _same_bits(got, summed)
    got = ops.Conv(plug.eval_add_relu, d, w, b, silu_lut=cases.silu_lut())(x, addend=r)
    assert _same_bits(got, relu(summed))


def test_plugin_conv_eval_add_w8a32(torch_dev):
    """the int8 convolution has no folded store: the plugin runs the Add and the Relu as passes over its output"""
    name = "q3x3_silu"
    d = cases.conv_w8a32_cases()[name]
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    oh, ow = d.out_hw()
    r = datagen.uniform(datagen.seed_for(name, "residual"), (d.n, d.cout, oh, ow), -1.0, 1.0)
    plug = ops.Plugin(hip.plugin_path("Conv"))
    y = ops.Conv(plug.eval, d, w8, b32, weight_aux=aux, silu_lut=cases.silu_lut())(x)
    got = ops.Conv(plug.eval_add_relu, d, w8, b32, weight_aux=aux, silu_lut=cases.silu_lut())(x, addend=r)
    want = y + r
    want = np.concatenate([np.where(0.0 > want.reshape(-1)[:want.size // 32 * 32], 0.0, want.reshape(-1)[:want.size // 32 * 32]),
                           np.where(want.reshape(-1)[want.size // 32 * 32:] > 0, want.reshape(-1)[want.size // 32 * 32:], 0.0)])
    assert _same_bits(got, want.astype(np.float32).reshape(got.shape))


# ---- plugin level: host pointers through `eval`, as the oneNew runtime calls it -------------------------

@pytest.mark.parametrize("name", ["c3x3_tiny_relu", "c1x1_unaligned_clip", "c3x3_silu", "c3x3_nobias", "dw3x3_s2_even",
                                  "dw3x3_group0", "cfg1_64x56_3x3", "rn50_l4_1x1_2048_512"])
def test_plugin_conv_eval_host_buffers(name, torch_dev, golden):
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    plug = ops.Plugin(hip.plugin_path("Conv"))
    op = ops.Conv(plug.eval, d, w, b, silu_lut=cases.silu_lut())
    y = op(x)
    y2 = op(x)  # second call: cached weights
    assert np.array_equal(y, y2)
    exact = d.group != 1
    # the SiLU case can flip a table bin on a last-bit difference of the sum
    atol = 5e-3 if d.act_type == abi.SILU and d.has_bias else 1e-4 * float(np.abs(y).max())
    cases.check_against(golden, name, y, exact=exact, rtol=1e-4, atol=atol)


def test_plugin_conv_eval_sees_a_weight_changed_in_place(torch_dev, oracle):
    """the device copy of host weights is checked against all of the host buffer on every call: one weight changed in
    place, at a position a sparse sample of the buffer would skip, must show in the next result"""
    d = cases.conv_f32_cases()["cfg1_64x56_3x3"]
    x, w, b = cases.conv_inputs("plugin_inplace", d)
    op = ops.Conv(ops.Plugin(hip.plugin_path("Conv")).eval, d, w, b)
    y0 = op(x).copy()
    flat = op.weight.reshape(-1)
    assert flat.size // 2 > 4096                      # large enough for a 4096-word sample to have gaps
    flat[3] += np.float32(0.75)                       # word 1 of the buffer: between two sampled words
    y1 = op(x).copy()
    w2 = w.copy()
    w2.reshape(-1)[3] += np.float32(0.75)
    ref = oracle.conv2d_f32(d, x, w2, b)
    assert not np.array_equal(y0, y1), "the stale device copy of the weights was used"
    assert_close_f32(y1, ref, tag="weights changed in place")


@pytest.mark.parametrize("name", ["q3x3_silu", "q3x3_nobias", "qdw3x3_s2", "q3x3_bigacc", "yolo_sppf_1x1_1024"])
def test_plugin_conv_eval_w8a32(name, torch_dev, golden):
    d = cases.conv_w8a32_cases()[name]
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    plug = ops.Plugin(hip.plugin_path("Conv"))
    op = ops.Conv(plug.eval, d, w8, b32, weight_aux=aux, silu_lut=cases.silu_lut())
    cases.check_against(golden, name, op(x), exact=True)


def test_plugin_matmul_and_gemm_eval(torch_dev, golden):
    mm = ops.MatMul(ops.Plugin(hip.plugin_path("MatMul")).eval)
    for name in ("mm_batched_shared", "mm_batched_b", "vit_scores", "mm_many_batches"):
        a, b = cases.matmul_inputs(name, *cases.matmul_cases()[name])
        y = mm(a, b)
        cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-4 * float(np.abs(y).max()))
    for name in ("gemm_n_tail", "rn50_fc"):
        a, w, b = cases.gemm_inputs(name, *cases.gemm_cases()[name])
        y = ops.Gemm(ops.Plugin(hip.plugin_path("Gemm")).eval, w, b)(a)
        cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-4 * float(np.abs(y).max()))


def test_plugin_evals_on_a_named_stream(torch_dev):
    """onhip_plugin_set_stream: the evals queue their kernels on a caller's stream (here one created non-blocking, which
    a blocking copy does not wait for by itself) and results in host buffers are still complete on return"""
    import ctypes as C
    torch = torch_dev
    name = "c3x3_tiny_relu"
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    plug = ops.Plugin(hip.plugin_path("Conv"))
    op = ops.Conv(plug.eval, d, w, b)
    want = op(x).copy()
    lib = hip.load()
    lib.onhip_plugin_set_stream.argtypes = [C.c_void_p]
    s = torch.cuda.Stream()
    assert lib.onhip_plugin_set_stream(C.c_void_p(s.cuda_stream)) == 0
    try:
        for _ in range(3):
            assert np.array_equal(op(x), want)
        relu = ops.Relu(ops.Plugin(hip.plugin_path("Relu")).eval)
        assert np.array_equal(relu(x), np.maximum(x, 0))
    finally:
        assert lib.onhip_plugin_set_stream(None) == 0
    assert np.array_equal(op(x), want)


def test_plugin_conv_eval_device_buffers(torch_dev, golden):
    """activation and output already in device memory: used in place, no staging"""
    torch = torch_dev
    name = "c3x3_s2_p1_even"
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    oh, ow = d.out_hw()
    xd = dev(torch, x)
    yd = torch.zeros((1, d.cout, oh, ow), dtype=torch.float32, device="cuda")
    op = ops.Conv(ops.Plugin(hip.plugin_path("Conv")).eval, d, w, b)
    op(xd.data_ptr(), out=yd.data_ptr())
    y = yd.cpu().numpy()
    cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-4 * float(np.abs(y).max()))


def test_errors_are_reported_not_thrown(torch_dev):
    d = cases.cd(4, 4, 3, 1, 1, 8)
    d.stride_h = 0
    import ctypes as C
    L = hip.load()
    rc = L.onhip_conv2d_f32(C.byref(d), 1, 1, 1, None, 1, None)
    assert rc == -1 and b"bad geometry" in L.onhip_last_error()
    q = cases.cd(4, 4, 3, 1, (1, 0, 1, 0), 8, input_scale=0.1)
    rc = L.onhip_conv2d_w8a32(C.byref(q), 1, 1, 1, 1, None, 1, None, None, 0, None)
    assert rc == -1 and b"uniform" in L.onhip_last_error()


# ---- full-size properties ------------------------------------------------------------------------------

def _sampled_conv_f64(d, x, w, b, idx):
    """float64 cross-correlation at the sampled flat output indices (dense convolution, ReLU)"""
    oh, ow = d.out_hw()
    out = np.empty(len(idx))
    xp = np.zeros((d.n, d.cin, d.h + d.pad_t + d.pad_b, d.w + d.pad_l + d.pad_r))
    xp[:, :, d.pad_t:d.pad_t + d.h, d.pad_l:d.pad_l + d.w] = x
    for t, f in enumerate(idx):
        n, r = divmod(int(f), d.cout * oh * ow)
        m, r = divmod(r, oh * ow)
        i, j = divmod(r, ow)
        patch = xp[n, :, i * d.stride_h:i * d.stride_h + d.kh, j * d.stride_w:j * d.stride_w + d.kw]
        out[t] = max((patch * w[m].astype(np.float64)).sum() + float(b[m]), 0.0)
    return out


@pytest.mark.parametrize("layer", [0, 2, 13, 15, 26, 44, 49, 52])
def test_resnet50_layers_batch32_sampled_f64(layer, torch_dev):
    """ResNet-50 layers at their real shapes, batch 32: 1500 sampled outputs against float64"""
    torch = torch_dev
    from onenew_amd import stacks
    name, d = stacks.with_batch(stacks.resnet50(), 32)[layer]
    x, w, b = cases.conv_inputs("rn50b32_" + name, d)
    wp = hip.pack_conv_weights(d, dev(torch, w))
    if wp is not None:
        y = hip.conv2d_f32(d, dev(torch, x), wp, dev(torch, b), packed=True)
    else:
        y = hip.conv2d_f32(d, dev(torch, x), dev(torch, w), dev(torch, b))
    torch.cuda.synchronize()
    y = y.cpu().numpy().reshape(-1)
    idx = cases.datagen.integers(cases.datagen.seed_for(name, "probe"), (1500,), 0, y.size - 1)
    ref = _sampled_conv_f64(d, x, w, b, idx)
    assert np.abs(y[idx] - ref).max() <= 1e-4 * max(np.abs(ref).max(), 1e-6), name
    # image 7 of the batch equals the batch-1 evaluation of image 7
    d1 = ConvDesc.from_buffer_copy(d)
    d1.n = 1
    y1 = hip.conv2d_f32(d1, dev(torch, x[7:8]), dev(torch, w), dev(torch, b))
    torch.cuda.synchronize()
    per = y.size // 32
    assert_close_f32(y[7 * per:8 * per], y1.cpu().numpy(), tag=name + " batch slice")


def test_linearity_and_zero_input(torch_dev):
    """conv(a*x) - bias == a * (conv(x) - bias) up to rounding; zero input gives act(bias)"""
    torch = torch_dev
    d = cases.cd(64, 128, 3, 1, 1, 28, act=abi.NOT_ACT, n=4)
    x, w, b = cases.conv_inputs("lin", d)
    xd, wd, bd = dev(torch, x), dev(torch, w), dev(torch, b)
    y1 = hip.conv2d_f32(d, xd, wd, bd).cpu().numpy()
    y2 = hip.conv2d_f32(d, xd * 2.0, wd, bd).cpu().numpy()
    bb = b.reshape(1, -1, 1, 1)
    assert_close_f32(y2 - bb, 2.0 * (y1 - bb), rel=1e-5, tag="linearity")
    d.act_type = abi.RELU
    y0 = hip.conv2d_f32(d, torch.zeros_like(xd), wd, bd).cpu().numpy()
    assert np.array_equal(y0, np.broadcast_to(np.maximum(bb, 0), y0.shape))


def _calib_tensor(seed, n):
    x = cases.datagen.normal(seed, (n,), 1.0)
    x[::997] *= 9.0
    x[5::1231] = 0.0
    return x.astype(np.float32)


def test_calibration_passes_match_oracle(torch_dev, oracle):
    """running max |x|, the 2048-bin histogram (two images accumulated) and the KL / MSE thresholds are the
    oracle's, bit for bit; so is the weight / bias quantiser"""
    torch = torch_dev
    imgs = [_calib_tensor(cases.datagen.seed_for("calib_gpu", str(i)), 300000 + 1000 * i) for i in range(2)]
    mx_ref, mx = 0.0, 0.0
    for x in imgs:
        mx_ref = oracle.calib_abs_max(x, mx_ref)
        mx = hip.calib_abs_max(dev(torch, x), mx)
    assert mx == mx_ref == max(float(np.abs(x).max()) for x in imgs)
    h_ref, h = None, None
    for x in imgs:
        h_ref = oracle.calib_histogram(x, mx_ref, h_ref)
        h = hip.calib_histogram(dev(torch, x), mx, h)
    assert np.array_equal(h, h_ref)
    count = sum(x.size for x in imgs)
    for name, method in (("kl", hip.CALIB_KL), ("mse", hip.CALIB_MSE)):
        assert hip.calib_threshold(method, h, count, mx) == oracle.calib_threshold(name, h_ref, count, mx_ref), name
    w = cases.datagen.normal(21, (7, 5, 3, 3), 0.0, 0.1)
    b = cases.datagen.normal(22, (7,), 0.0, 0.05)
    got, ref = hip.quant_weight_bias(w, b), oracle.quant_weight_bias(w, b)
    assert all(np.array_equal(g, r) for g, r in zip(got, ref))


@pytest.mark.parametrize("images,elems,step", [(3, 400000, 0.0), (1, 100000, 0.0), (5, 70001, 0.0), (7, 50000, 0.125),
                                               (4, 250000, 0.5), (2, 1000000, 0.03125), (16, 50001, 0.25)])
def test_calibration_percentile_matches_oracle(images, elems, step, torch_dev, oracle):
    """the radix selection against the oracle's sort, also on data with many equal magnitudes (values rounded to a
    step, so the kept set of an image ends inside a run of ties) and with zeros"""
    torch = torch_dev
    x = _calib_tensor(cases.datagen.seed_for("calib_gpu", "pct", images, elems), images * elems)
    if step:
        x = (np.round(x / np.float32(step)) * np.float32(step)).astype(np.float32)
    assert hip.calib_percentile(dev(torch, x), images, elems) == oracle.calib_percentile(x, images, elems)


def test_calibration_passes_refuse_a_missing_workspace(torch_dev):
    import ctypes as C
    torch = torch_dev
    x = torch.ones(1000, device="cuda")
    m, t = C.c_float(0.0), C.c_float(0.0)
    L = hip.load()
    assert L.onhip_calib_abs_max(x.data_ptr(), 1000, C.byref(m), None, 0, None) == -3
    hist = np.zeros(2048, np.float32)
    assert L.onhip_calib_histogram(x.data_ptr(), 1000, 1.0, hist.ctypes.data, None, 0, None) == -3
    small = torch.empty(64, dtype=torch.uint8, device="cuda")
    big = torch.ones(4 * 300000, device="cuda")
    assert L.onhip_calib_percentile(big.data_ptr(), 4, 300000, C.byref(t), small.data_ptr(), 64, None) == -3
    assert b"onhip_calib_workspace_bytes" in L.onhip_last_error()


def _same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).reshape(-1).view(np.uint32),
                          np.ascontiguousarray(b).reshape(-1).view(np.uint32))


@pytest.mark.parametrize("name", list(cases.add_cases()))
def test_add_matches_oracle_and_plugin(name, torch_dev, oracle, golden):
    """kernel level (incl. the fused ReLU) and the Add plugin on host buffers: bit-identical to the reference"""
    torch = torch_dev
    a, b = cases.add_inputs(name, *cases.add_cases()[name])
    ref = oracle.add_f32(a, b)
    large, small = (b, a) if a.size < b.size else (a, b)
    y = hip.add_f32(dev(torch, large), dev(torch, small))
    yr = hip.add_f32(dev(torch, large), dev(torch, small), relu=True)
    torch.cuda.synchronize()
    assert _same_bits(y.cpu().numpy(), ref)
    assert _same_bits(yr.cpu().numpy(), np.where(ref > 0, ref, np.float32(0)))
    cases.check_against(golden, name, y.cpu().numpy(), exact=True)
    assert _same_bits(ops.Add(ops.Plugin(hip.plugin_path("Add")).eval)(a, b), ref)


@pytest.mark.parametrize("name", list(cases.relu_cases()))
def test_relu_matches_oracle_and_plugin(name, torch_dev, oracle):
    torch = torch_dev
    x = cases.relu_input(name, cases.relu_cases()[name])
    ref = oracle.relu_f32(x)
    y = hip.relu_f32(dev(torch, x))
    torch.cuda.synchronize()
    assert _same_bits(y.cpu().numpy(), ref)          # signed zeros and NaNs included
    xin = ops.aligned_empty(x.shape)
    xin[...] = x
    assert _same_bits(ops.Relu(ops.Plugin(hip.plugin_path("Relu")).eval)(xin), ref)


@pytest.mark.parametrize("name", list(cases.maxpool_cases()))
def test_maxpool_matches_oracle_and_plugin(name, torch_dev, oracle, golden):
    torch = torch_dev
    shape, k, st, pad = cases.maxpool_cases()[name]
    x = cases.maxpool_input(name, shape)
    ref = oracle.maxpool_f32(x, k, st, pad)
    d = abi.PoolDesc(shape[0], shape[1], shape[2], shape[3], k, k, st, st, pad)
    y = hip.maxpool_f32(d, dev(torch, x))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), ref)
    cases.check_against(golden, name, y.cpu().numpy(), exact=True)
    assert np.array_equal(ops.MaxPool(ops.Plugin(hip.plugin_path("MaxPool")).eval, k, st, pad)(x), ref)
    # a batch is that many independent images
    xb = np.concatenate([x, x[:, ::-1].copy()], axis=0)
    db = abi.PoolDesc(2, shape[1], shape[2], shape[3], k, k, st, st, pad)
    yb = hip.maxpool_f32(db, dev(torch, xb)).cpu().numpy()
    assert np.array_equal(yb[0], ref[0]) and np.array_equal(yb[1], oracle.maxpool_f32(xb[1:2], k, st, pad)[0])


@pytest.mark.parametrize("shape", [(2, 3, 9, 8), (1, 5, 16, 4), (3, 2, 7, 20), (1, 1, 2, 12), (2, 4, 10, 10)])
def test_maxpool_3x3_stride2_two_outputs_per_thread(shape, torch_dev, oracle):
    """the stem pooling (3x3, stride 2, padding 1) on rows of a multiple of four floats runs a kernel of its own:
    odd and even heights, a single column pair, inputs below the reference's start value, NaNs (which never win),
    and a width that is not a multiple of four (the general kernel) -- all equal to the oracle bit for bit"""
    torch = torch_dev
    rng = np.random.default_rng(sum(shape))
    x = rng.normal(size=shape).astype(np.float32)
    x[0, 0, 0, :] = -5e6                                   # below -3276800: the start value wins
    x[-1, -1, -1, 1::3] = np.nan
    ref = oracle.maxpool_f32(x, 3, 2, 1)
    d = abi.PoolDesc(shape[0], shape[1], shape[2], shape[3], 3, 3, 2, 2, 1)
    y = hip.maxpool_f32(d, dev(torch, x))
    torch.cuda.synchronize()
    assert _same_bits(y.cpu().numpy(), ref)


@pytest.mark.parametrize("name", list(cases.gap_cases()))
def test_global_avgpool_matches_oracle_and_plugin(name, torch_dev, oracle, golden):
    torch = torch_dev
    x = cases.gap_input(name, cases.gap_cases()[name])
    ref = oracle.global_avgpool_f32(x)
    y = hip.global_avgpool_f32(dev(torch, x))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), ref)      # same summation order: bit-identical
    cases.check_against(golden, name, y.cpu().numpy(), exact=True)
    assert np.array_equal(ops.GlobalAveragePool(ops.Plugin(hip.plugin_path("GlobalAveragePool")).eval)(x), ref)
    xb = np.concatenate([x] * 3, axis=0)
    yb = hip.global_avgpool_f32(dev(torch, xb)).cpu().numpy()
    assert np.array_equal(yb, np.concatenate([ref] * 3, axis=0))


def test_gelu_table_matches_oracle_and_plugin(torch_dev, oracle, golden):
    torch = torch_dev
    x = cases.gelu_input()
    lut = cases.gelu_lut()
    ref = oracle.lut_act(x, lut)
    y = hip.gelu_lut_f32(dev(torch, x), dev(torch, lut))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), ref)
    cases.check_against(golden, "gelu_edges", y.cpu().numpy(), exact=True)
    xin = ops.aligned_empty(x.shape)
    xin[...] = x
    assert np.array_equal(ops.Gelu(ops.Plugin(hip.plugin_path("Gelu")).eval, lut)(xin), ref)


@pytest.mark.parametrize("name", list(cases.layernorm_cases()))
def test_layernorm_matches_oracle_and_plugin(name, torch_dev, oracle, golden):
    """sums in memory order, every operation rounded as in the reference: bit-identical"""
    torch = torch_dev
    shape, axis = cases.layernorm_cases()[name]
    x, w, b = cases.layernorm_inputs(name, shape, axis)
    ref = oracle.layernorm_f32(x, w, b, axis1=(axis == 1))
    y = hip.layernorm_f32(dev(torch, x), dev(torch, w), dev(torch, b), axis1=(axis == 1))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), ref), f"{name}: {(y.cpu().numpy() != ref).sum()} elements differ"
    cases.check_against(golden, name, y.cpu().numpy(), exact=True)
    plug = ops.LayerNormalization(ops.Plugin(hip.plugin_path("LayerNormalization")).eval, w, b, axis)
    assert np.array_equal(plug(x), ref)


@pytest.mark.parametrize("shape", [(64 * 196, 192), (7, 128), (300, 32), (5, 2044), (1000, 768), (515, 36), (41, 192)])
def test_layernorm_rows_of_16_byte_pieces(shape, torch_dev, oracle):
    """rows of a multiple of four floats take the kernel that stages them with 16-byte accesses: the same sums in the same
    order, bit-identical to the oracle, whatever the number of rows per workgroup and the ragged last workgroup"""
    torch = torch_dev
    x = cases.datagen.normal(cases.datagen.seed_for("ln_rows4", *shape), shape, -0.2, 2.0)
    w = cases.datagen.normal(cases.datagen.seed_for("ln_rows4", "w", shape[1]), (shape[1],), 1.0, 0.2)
    b = cases.datagen.normal(cases.datagen.seed_for("ln_rows4", "b", shape[1]), (shape[1],), 0.0, 0.2)
    y = hip.layernorm_f32(dev(torch, x), dev(torch, w), dev(torch, b))
    torch.cuda.synchronize()
    ref = oracle.layernorm_f32(x, w, b)
    assert np.array_equal(y.cpu().numpy(), ref), f"{(y.cpu().numpy() != ref).sum()} elements differ"


@pytest.mark.parametrize("name", list(cases.softmax_cases()))
def test_softmax_matches_oracle_and_plugin(name, torch_dev, oracle, golden):
    """expf on the GPU and in glibc agree to a few ulp: fp32 tolerance 1e-4 of the row maximum, rows sum to 1"""
    torch = torch_dev
    shape, axis = cases.softmax_cases()[name]
    x = cases.softmax_input(name, shape)
    ref = oracle.softmax_f32(x, axis1=(axis == 1))
    y = hip.softmax_f32(dev(torch, x), axis1=(axis == 1)).cpu().numpy()
    assert np.abs(y - ref).max() <= 1e-4 * ref.max() and np.allclose(y, ref, rtol=1e-4, atol=1e-9)
    ax = 1 if axis == 1 else x.ndim - 1
    assert np.allclose(y.sum(axis=ax), 1.0, atol=1e-5)
    cases.check_against(golden, name, y, exact=False, rtol=1e-4, atol=1e-9)
    yp = ops.Softmax(ops.Plugin(hip.plugin_path("Softmax")).eval, axis)(x)
    assert np.array_equal(yp, y)


@pytest.mark.parametrize("name", list(cases.transpose_cases()))
def test_transpose_matches_numpy_and_plugin(name, torch_dev):
    torch = torch_dev
    shape, perm = cases.transpose_cases()[name]
    x = cases.transpose_input(name, shape)
    y = hip.transpose_f32(dev(torch, x), perm)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), np.transpose(x, perm))
    if len(shape) in (4, 6):
        assert np.array_equal(ops.Transpose(ops.Plugin(hip.plugin_path("Transpose")).eval, perm)(x), np.transpose(x, perm))


# shapes that reduce to a batch of plain matrix transposes (the LDS-tile kernel): ViT's tokens <-> channels with its unit
# dimension, ragged tiles, a single matrix, batch dimensions that merge, rows of fewer than 8 floats (element-wise kernel)
TRANSPOSE_EXTRA = [((3, 192, 196, 1), (0, 2, 1, 3)), ((3, 196, 192, 1), (0, 2, 1, 3)), ((2, 37, 65), (0, 2, 1)), ((100, 70), (1, 0)),
                   ((2, 3, 33, 40), (0, 1, 3, 2)), ((5, 1, 64, 9), (0, 1, 3, 2)), ((4, 300, 5), (0, 2, 1)), ((1, 32, 32), (0, 2, 1)),
                   ((2, 8, 1, 50, 1), (0, 3, 2, 1, 4))]


@pytest.mark.parametrize("shape,perm", TRANSPOSE_EXTRA)
def test_transpose_batches_of_matrices(shape, perm, torch_dev):
    torch = torch_dev
    x = cases.transpose_input(f"tr_extra{shape}{perm}", shape)
    y = hip.transpose_f32(dev(torch, x), perm)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), np.transpose(x, perm))


# chain-form shapes beyond the W8A32 case list: output channels that end inside a 16-channel group and inside a
# row tile, channel counts whose K tiles do / do not straddle filter taps (64-channel multiples or not)
CHAIN_EXTRA = {
    "chain_128_80_3x3": cases.cd(128, 80, 3, 1, 1, 13, act=abi.SILU, input_scale=0.017),
    "chain_48_24_3x3_s2": cases.cd(48, 24, 3, 2, 1, 17, act=abi.CLIP, clip_min=-0.5, clip_max=2.0, input_scale=0.02),
    "chain_192_200_1x1": cases.cd(192, 200, 1, 1, 0, 9, act=abi.LEAKYRELU, leaky_relu_alpha=0.1, input_scale=0.012),
    "chain_64_33_5x5": cases.cd(64, 33, 5, 1, 2, 11, act=abi.HARDSILU, hard_sigmoid_alpha=0.2, hard_sigmoid_beta=0.5, input_scale=0.015),
}


def _chain_desc(name):
    if name in CHAIN_EXTRA:
        return ConvDesc.from_buffer_copy(CHAIN_EXTRA[name])
    return ConvDesc.from_buffer_copy(cases.conv_w8a32_cases()[name])


def test_quantised_copy_of_a_table_is_dropped_with_the_table(torch_dev, oracle):
    """the chain form keeps a quantised copy of the activation table by the table's address; once the caller says
    that address is being rewritten, the next call quantises what is there now"""
    torch = torch_dev
    d = _chain_desc("q3x3_silu")
    d.n = 2
    d.out_s8, d.output_scale = 1, 0.041
    x, w8, b32, aux = cases.conv_inputs("q3x3_silu_table", d, quant=True)
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale)
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    lut = dev(torch, cases.silu_lut())
    other = -cases.silu_lut()
    args = (d, xq, wp, dev(torch, b32), dev(torch, aux), lut)
    got = hip.conv2d_w8a8_nhwc(*args).cpu().numpy()
    assert np.array_equal(got[..., :d.cout], np.transpose(oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut()), (0, 2, 3, 1)))
    hip.forget(lut)
    lut.copy_(dev(torch, other))
    got = hip.conv2d_w8a8_nhwc(*args).cpu().numpy()
    want = np.transpose(oracle.conv2d_w8a32(d, x, w8, b32, aux, other), (0, 2, 3, 1))
    assert np.array_equal(got[..., :d.cout], want)
    assert not np.array_equal(got[..., :d.cout], np.transpose(oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut()), (0, 2, 3, 1)))
    hip.forget(lut)


@pytest.mark.parametrize("tile", [None, "128x128", "64x128", "32x128", "64x64x2"])
@pytest.mark.parametrize("name", ["q3x3_silu", "q3x3_s2", "yolo_c2f_3x3_64_80", "yolo_sppf_1x1_1024", "q3x3_bigacc"]
                         + list(CHAIN_EXTRA))
def test_conv_w8a8_nhwc_chain_form(name, tile, torch_dev, oracle, monkeypatch):
    """int8 NHWC in / int8 NHWC out: the same int8 values as quantising the reference's fp32 result, and the
    quantised input equals the reference's own input quantiser; every tile shape and the split-K path"""
    torch = torch_dev
    if tile is not None and name in ("yolo_sppf_1x1_1024", "q3x3_silu", "q3x3_s2"):
        pytest.skip("forced tiles run on the shapes with ragged rows and columns")
    if tile:
        monkeypatch.setenv("ONHIP_TILE", tile)
    d = _chain_desc(name)
    d.n = 3
    d.out_s8, d.output_scale = 1, 0.041
    x, w8, b32, aux = cases.conv_inputs(name + "_chain", d, quant=True)
    ref = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut())          # int8 NCHW
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale)
    q_ref = oracle.quantize_s8(x, d.input_scale)                              # NCHW
    assert np.array_equal(xq.cpu().numpy()[..., :d.cin], np.transpose(q_ref, (0, 2, 3, 1)))
    assert not xq.cpu().numpy()[..., d.cin:].any()                            # channel padding is zero
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    oh, ow = d.out_hw()
    out = torch.full((d.n, oh, ow, (d.cout + 15) // 16 * 16), 77, dtype=torch.int8, device="cuda")
    yq = hip.conv2d_w8a8_nhwc(d, xq, wp, dev(torch, b32), dev(torch, aux), dev(torch, cases.silu_lut()), out=out)
    torch.cuda.synchronize()
    got = yq.cpu().numpy()
    assert np.array_equal(got[..., :d.cout], np.transpose(ref, (0, 2, 3, 1)))
    if tile is None or "x2" not in tile:
        assert not got[..., d.cout:].any()                                    # unsplit launches zero the channel padding


@pytest.mark.parametrize("tile", ["128x128", "128x64", "64x128", "64x64"])
@pytest.mark.parametrize("shape", [(2, 64, 19, 72, 3, 1, 1), (1, 128, 23, 200, 3, 2, 1), (3, 192, 9, 130, 1, 1, 0), (2, 128, 12, 64, 5, 1, 2),
                                   (1, 256, 7, 33, 3, 1, 1), (2, 64, 16, 128, 1, 2, 0),
                                   # fewer than 64 channels: stages that hold several filter taps, ragged last stage
                                   (2, 3, 30, 40, 3, 2, 1), (1, 32, 21, 64, 3, 1, 1), (2, 16, 17, 72, 5, 1, 2), (1, 32, 16, 100, 1, 1, 0),
                                   (1, 8, 12, 33, 7, 2, 3), (1, 20, 9, 130, 3, 1, 1)])
@pytest.mark.parametrize("act", [abi.SILU, abi.RELU, abi.NOT_ACT])
@pytest.mark.parametrize("ring", [1, 2])
def test_conv_int8_direct_to_lds_kernel_every_tile(ring, tile, shape, act, torch_dev, oracle, monkeypatch):
    """the int8 kernel that loads its tiles from global memory straight into LDS, every tile it has, on shapes with ragged
    rows and columns, strides, padding, 64- and 128-byte stages (channels a multiple of 64 / of 128) and 64-byte stages of
    two or four short taps (up to 32 / 16 channels), one and many taps, a single stage and many: int8 NHWC chain form and the fp32 / int32-accumulator form, both equal to the oracle"""
    torch = torch_dev
    n, cin, hw, cout, k, stride, pad = shape
    monkeypatch.setenv("ONHIP_TILE", tile + f"x1x0x0x0x{ring}")   # ring 2: the long ring of stage buffers (more than 64 KiB of LDS)
    d = cases.cd(cin, cout, k, stride, pad, hw, n=n, act=act, input_scale=0.037)
    name = f"dma_{tile}_{cin}_{cout}_{k}_{stride}"
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    lut = cases.silu_lut()
    oh, ow = d.out_hw()
    launches = hip.load().onhip_direct_lds_launches()
    # fp32 NCHW out with the raw accumulators
    acc = torch.empty((d.n, d.cout, oh, ow), dtype=torch.int32, device="cuda")
    y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, lut), acc32=acc)
    torch.cuda.synchronize()
    ref, ref_acc = oracle.conv2d_w8a32(d, x, w8, b32, aux, lut, want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), ref_acc), "int32 accumulators differ"
    assert np.array_equal(y.cpu().numpy(), ref), "de-quantised outputs differ"
    # int8 NHWC in and out
    dq = ConvDesc.from_buffer_copy(d)
    dq.out_s8, dq.output_scale = 1, 0.045
    refq = oracle.conv2d_w8a32(dq, x, w8, b32, aux, lut)
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale)
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    out = torch.full((d.n, oh, ow, (d.cout + 15) // 16 * 16), 77, dtype=torch.int8, device="cuda")
    hip.conv2d_w8a8_nhwc(dq, xq, wp, dev(torch, b32), dev(torch, aux), dev(torch, lut), out=out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got[..., :d.cout], np.transpose(refq, (0, 2, 3, 1)))
    assert not got[..., d.cout:].any()
    assert hip.load().onhip_direct_lds_launches() == launches + 2, "the forced tile did not run the direct-to-LDS kernel"


_TUNE_CHILD = r"""
import sys, numpy as np, torch
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests/golden")
import cases
from onenew_amd import abi, hip
hip.init(0)
d = cases.cd(96, 80, 3, 1, 1, 20, n=4, act=abi.NOT_ACT)
x, w, b = cases.conv_inputs("tune_cache_file", d)
y = hip.conv2d_f32(d, torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda()).cpu()
ref = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(b).double(), padding=1)
print("ERR", float((y.double() - ref).abs().max() / ref.abs().max()))
"""


@pytest.mark.gpu
def test_tune_cache_file_is_validated_and_rewritten(tmp_path):
    """measured choices persist in the file ONHIP_TUNE_CACHE names; lines that are not choices of this build (garbage,
    or a choice the problem does not admit) are passed over and the problem is measured again"""
    import os, subprocess, sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cache = tmp_path / "tune.txt"
    env = dict(os.environ, ONHIP_TUNE="1", ONHIP_TUNE_CACHE=str(cache))
    env.pop("ONHIP_TILE", None)

    def run():
        out = subprocess.run([sys.executable, "-c", _TUNE_CHILD, root], env=env, capture_output=True, text=True, timeout=100)
        assert out.returncode == 0, out.stderr[-2000:]
        err = [float(l.split()[1]) for l in out.stdout.splitlines() if l.startswith("ERR")]
        assert err and err[0] <= 1e-4
        return [l for l in cache.read_text().splitlines() if l.strip()]

    lines = run()                                   # measured and written
    assert len(lines) == 1 and ":" in lines[0]
    assert run() == lines                           # read back: nothing measured, nothing appended
    key = lines[0].split(":")[0]
    cache.write_text("not a line of this file\n" + key + ": 64 64 0 0 0 0\n" + key + ": 64 64 1 0 0 1\n")
    after = run()       # split 0 is no choice; in-launch reduction without slices is none either: measured again
    assert len(after) == 4 and after[3].startswith(key + ":")
    assert run() == after                           # the last line for a problem is the one that counts


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [
    # (n, cin, h, w, cout, k, stride, pad): 16 bytes per pixel (two taps per MFMA step), first layers
    (2, 3, 30, 30, 32, 3, 2, 1), (1, 3, 33, 47, 16, 3, 2, 1), (3, 8, 17, 21, 40, 3, 1, 1), (2, 16, 12, 19, 64, 3, 2, 0), (1, 4, 9, 70, 24, 3, 1, 2),
    # 32 bytes per pixel: stride 1 with pads 1 (the rows of a band kept in LDS), other strides and pads (loaded per tap)
    (2, 32, 20, 20, 32, 3, 1, 1), (1, 24, 13, 37, 16, 3, 1, 1), (2, 32, 16, 160, 32, 3, 1, 1), (1, 32, 7, 256, 24, 3, 1, 1), (3, 20, 5, 6, 64, 3, 1, 1),
    (2, 32, 21, 23, 64, 3, 2, 1), (1, 32, 18, 18, 48, 3, 1, 0), (2, 17, 15, 15, 32, 3, 2, 1), (1, 32, 40, 80, 64, 3, 1, 1),
    # 7x7 first layers (49 taps of 16 bytes, 25 MFMA steps), one and two row tiles
    (2, 3, 30, 30, 64, 7, 2, 3), (1, 3, 33, 47, 24, 7, 2, 3), (1, 8, 20, 20, 32, 7, 1, 3), (2, 16, 9, 9, 40, 7, 2, 0),
    # rows too long for a band in LDS (loaded per tap instead); fewer blocks than XCDs; one pixel
    (1, 32, 4, 300, 32, 3, 1, 1), (3, 32, 3, 3, 16, 3, 1, 1), (1, 16, 1, 1, 32, 3, 1, 1),
    # 64 bytes per pixel, stride 1, pads 1
    (2, 64, 20, 20, 64, 3, 1, 1), (1, 48, 11, 80, 32, 3, 1, 1), (1, 64, 9, 13, 40, 3, 1, 1),
    # 1x1 with 64, 96 or 128 bytes per pixel, a stride, a pad; more than 64 output channels (the implicit-GEMM kernels')
    (2, 64, 20, 20, 64, 1, 1, 0), (1, 50, 13, 37, 40, 1, 1, 0), (2, 96, 9, 31, 48, 1, 1, 0), (1, 90, 16, 16, 64, 1, 2, 0),
    (3, 128, 7, 11, 33, 1, 1, 0), (1, 128, 24, 24, 64, 1, 1, 1), (2, 100, 5, 5, 16, 1, 1, 0), (1, 128, 12, 12, 80, 1, 1, 0)])
@pytest.mark.parametrize("act", [abi.SILU, abi.RELU, abi.NOT_ACT])
def test_conv_int8_chain_3x3_with_few_channels(shape, act, torch_dev, oracle, monkeypatch):
    """3x3 convolutions of the int8 NHWC chain form with at most 64 input channels and 64 output channels, 7x7 first
    layers, and 1x1 convolutions with at most 128 and 64: whichever kernel
    takes them (input rows of a band in LDS, or windows loaded per tap, or the implicit-GEMM kernels), the bytes are the
    oracle's, and the same with the LDS kernel given every shape it can take and with those two kernels switched off; ragged sizes, pixels past the last block, pads 0 to 2"""
    torch = torch_dev
    n, cin, h, w, cout, k, stride, pad = shape
    d = cases.cd(cin, cout, k, stride, pad, h, w=w, n=n, act=act, input_scale=0.041, out_s8=1, output_scale=0.052)
    x, w8, b32, aux = cases.conv_inputs(f"few_{cin}_{cout}_{h}_{w}_{k}_{stride}_{pad}", d, quant=True)
    lut = cases.silu_lut()
    oh, ow = d.out_hw()
    ref = np.transpose(oracle.conv2d_w8a32(d, x, w8, b32, aux, lut), (0, 2, 3, 1))
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale)
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    for off in (False, "ONHIP_PATCH_ALL", "ONHIP_NO_PATCH"):   # the default choice; every shape the LDS kernel takes; neither kernel
        if off:
            monkeypatch.setenv(off, "1")
        out = torch.full((d.n, oh, ow, (d.cout + 15) // 16 * 16), 77, dtype=torch.int8, device="cuda")
        hip.conv2d_w8a8_nhwc(d, xq, wp, dev(torch, b32), dev(torch, aux), dev(torch, lut), out=out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.array_equal(got[..., :d.cout], ref), f"kernels off: {off}"
        assert not got[..., d.cout:].any()


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 8, 7, 9), (1, 3, 5, 5), (4, 64), (1, 32, 14, 14)])
def test_add_then_relu_by_the_relu_operators_own_rules(shape, torch_dev):
    """onhip_add_f32 with relu = 2: the Relu operator's two rules by element index (relu.c:27-52) in the same pass, equal
    bit for bit to onhip_add_f32 followed by onhip_relu_f32, NaNs and negative zeros included, before and after the
    boundary at n - n % 32"""
    torch = torch_dev
    rng = np.random.default_rng(11)
    a = rng.normal(size=shape).astype(np.float32)
    b = rng.normal(size=shape).astype(np.float32)
    fa, fb = a.reshape(-1), b.reshape(-1)
    n = fa.size
    for i in (0, 5, n - n % 32 - 1, n - n % 32, n - 1):     # sums that are NaN and -0 on both sides of the boundary
        if 0 <= i < n:
            fa[i], fb[i] = np.float32("nan"), np.float32(1.0)
    for i in (1, 6, n - n % 32 - 2, n - n % 32 + 1, n - 2):
        if 0 <= i < n and not np.isnan(fa[i]):
            fa[i], fb[i] = np.float32(-0.0), np.float32(-0.0)
    ta, tb = dev(torch, a), dev(torch, b)
    two = hip.relu_f32(hip.add_f32(ta, tb))
    one = hip.add_f32(ta, tb, relu=2)
    torch.cuda.synchronize()
    assert np.array_equal(one.cpu().numpy().view(np.uint32), two.cpu().numpy().view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 64, 14, 14, 256, 1, 1, 0), (1, 32, 9, 11, 40, 3, 1, 1), (3, 128, 7, 7, 100, 1, 1, 0), (1, 16, 20, 20, 64, 3, 2, 1),
                                   (2, 256, 6, 6, 33, 1, 1, 0)])
@pytest.mark.parametrize("act", [abi.NOT_ACT, abi.RELU, abi.SILU])
@pytest.mark.parametrize("relu_after", [False, True])
def test_int8_convolution_with_the_add_and_relu_in_its_store(shape, act, relu_after, torch_dev, oracle):
    """onhip_conv2d_w8_link with an addend: fp32 or int8 NHWC activations in, the Add (and the Relu, by its own two rules)
    of a residual block in the convolution's fp32 store, equal bit for bit to the W8A32 convolution followed by the Add
    and Relu operators; NaN and negative-zero sums included"""
    torch = torch_dev
    n, cin, h, w, cout, k, stride, pad = shape
    d = cases.cd(cin, cout, k, stride, pad, h, w=w, n=n, act=act, input_scale=0.043)
    x, w8, b32, aux = cases.conv_inputs(f"resq_{cin}_{cout}_{h}_{w}_{k}_{stride}", d, quant=True)
    lut = cases.silu_lut()
    oh, ow = d.out_hw()
    y = hip.conv2d_w8a32(d, dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, lut))
    torch.cuda.synchronize()
    yh = y.cpu().numpy()
    rng = np.random.default_rng(3)
    addend = rng.normal(size=yh.shape).astype(np.float32)
    fa, fy = addend.reshape(-1), yh.reshape(-1)
    nel = fa.size
    for i in (0, 7, nel - nel % 32 - 1, nel - nel % 32, nel - 1):
        if 0 <= i < nel:
            fa[i] = np.float32("nan")
    for i in (3, nel - nel % 32 - 2, nel - nel % 32 + 1, nel - 2):
        if 0 <= i < nel and fy[i] == 0:
            fa[i] = np.float32(-0.0)
    ta = dev(torch, addend)
    want = hip.add_f32(y, ta)
    if relu_after:
        want = hip.relu_f32(want)
    wp = hip.pack_conv_weights_w8(d, dev(torch, w8))
    got = hip.conv2d_w8_link(d, wp, dev(torch, b32), dev(torch, aux), dev(torch, lut), x=dev(torch, x), addend=ta, relu_after=relu_after)
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale)
    got_q = hip.conv2d_w8_link(d, wp, dev(torch, b32), dev(torch, aux), dev(torch, lut), xq=xq, addend=ta, relu_after=relu_after)
    plain = hip.conv2d_w8_link(d, wp, dev(torch, b32), dev(torch, aux), dev(torch, lut), xq=xq)
    torch.cuda.synchronize()
    bits = lambda t: t.cpu().numpy().view(np.uint32)   # noqa: E731
    assert np.array_equal(bits(got), bits(want))
    assert np.array_equal(bits(got_q), bits(want))
    assert np.array_equal(bits(plain), bits(y))
    if cout % 16 == 0:
        # the same store also leaves the result as int8 NHWC, as the input quantiser of a reader would make it (the NaN
        # sums aside: no quantiser is defined on them)
        dt = ConvDesc.from_buffer_copy(d)
        dt.output_scale = 0.06
        twin = torch.full((n, oh, ow, cout), 77, dtype=torch.int8, device="cuda")
        got_t = hip.conv2d_w8_link(dt, wp, dev(torch, b32), dev(torch, aux), dev(torch, lut), xq=xq, addend=ta, relu_after=relu_after, twin=twin)
        ref_t = hip.quantize_nhwc_s8(want, 0.06)
        torch.cuda.synchronize()
        assert np.array_equal(bits(got_t), bits(want))
        ok = ~np.isnan(np.transpose(want.cpu().numpy(), (0, 2, 3, 1)))
        assert np.array_equal(twin.cpu().numpy()[ok], ref_t.cpu().numpy()[ok])


@pytest.mark.gpu
def test_plugin_eval_link_host_buffers(torch_dev, oracle):
    """eval_link of the Conv plugin on tensors in host memory: fp32 in / int8 NHWC out equals the consumer's quantiser on
    the W8A32 result of `eval`; int8 NHWC in / fp32 out with the Add and Relu folded equals Add and Relu on it, bit for bit"""
    torch = torch_dev
    d = cases.cd(24, 40, 3, 1, 1, 13, n=2, act=abi.SILU, input_scale=0.037)
    x, w8, b32, aux = cases.conv_inputs("plug_link", d, quant=True)
    lut = cases.silu_lut()
    plug = ops.Plugin(hip.plugin_path("Conv"))
    y = ops.Conv(plug.eval, d, w8, b32, weight_aux=aux, silu_lut=lut)(x)
    assert np.array_equal(y, oracle.conv2d_w8a32(d, x, w8, b32, aux, lut))
    link = ops.ConvLink(plug, d, w8, b32, aux, silu_lut=lut)
    yq = link(x, out_scale=0.052)
    dq = ConvDesc.from_buffer_copy(d)
    dq.out_s8, dq.output_scale = 1, 0.052
    refq = np.transpose(oracle.conv2d_w8a32(dq, x, w8, b32, aux, lut), (0, 2, 3, 1))
    assert yq.shape == (2, 13, 13, 48) and np.array_equal(yq[..., :40], refq) and not yq[..., 40:].any()
    xq = hip.quantize_nhwc_s8(dev(torch, x), d.input_scale).cpu().numpy()
    skip = cases.datagen.normal(cases.datagen.seed_for("plug_link", "skip"), y.shape, 0.0, 1.0)
    assert np.array_equal(link(xq, in_s8=True), y)
    assert np.array_equal(link(xq, in_s8=True, addend=skip), oracle.add_f32(y, skip))
    assert np.array_equal(link(x, addend=skip, relu_after=True), oracle.relu_f32(oracle.add_f32(y, skip)))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 24, 11, 11, 3, 2, 1), (1, 64, 56, 56, 3, 2, 1), (3, 5, 9, 14, 2, 2, 0), (1, 16, 7, 7, 3, 1, 1), (2, 40, 6, 6, 5, 1, 2)])
def test_maxpool_on_int8_nhwc_is_the_quantised_fp32_maxpool(shape, torch_dev):
    """onhip_maxpool_s8_nhwc on the quantised tensor equals the quantiser applied to onhip_maxpool_f32's result (the
    quantiser is monotonic), padding channels stay zero... except where a window holds no input at all"""
    torch = torch_dev
    n, c, h, w, k, stride, pad = shape
    x = cases.datagen.normal(cases.datagen.seed_for("mp8", str(shape)), (n, c, h, w), 0.0, 1.5)
    d = abi.PoolDesc(n=n, c=c, h=h, w=w, kh=k, kw=k, stride_w=stride, stride_h=stride, pad=pad)
    scale = 0.031
    y = hip.maxpool_f32(d, dev(torch, x))
    want = hip.quantize_nhwc_s8(y, scale)
    got = hip.maxpool_s8_nhwc(d, hip.quantize_nhwc_s8(dev(torch, x), scale))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy()[..., :c], want.cpu().numpy()[..., :c])


# ---- depthwise convolutions in the int8 NHWC chain form ---------------------------------------------------------
# (channels, height, width, filter, stride, pad, activation, batch): channel counts inside and beyond one 16-channel
# group, MobileNetV2's (32, 96, 144, 960), strides 1 / 2 (the unrolled 3x3 kernels) and 3, 5x5 and 7x7 (the generic one),
# planes narrower than a wavefront and wider, output rows that do not fill the last strip of a lane
DW_CHAIN = [(12, 11, 11, 3, 1, 1, abi.SILU, 2), (10, 14, 14, 3, 2, 1, abi.CLIP, 3), (6, 9, 9, 5, 1, 2, abi.NOT_ACT, 2),
            (32, 28, 28, 3, 1, 1, abi.CLIP, 2), (96, 30, 26, 3, 2, 1, abi.CLIP, 2), (144, 13, 17, 3, 1, 1, abi.RELU, 1),
            (960, 7, 7, 3, 1, 1, abi.CLIP, 3), (24, 70, 70, 3, 1, 1, abi.LEAKYRELU, 1), (40, 15, 15, 3, 3, 1, abi.HARDSILU, 2),
            (17, 12, 12, 7, 2, 3, abi.RELU, 2), (48, 5, 5, 3, 1, 1, abi.SILU, 9), (200, 9, 20, 5, 2, 2, abi.CLIP, 2),
            (16, 6, 130, 3, 2, 1, abi.NOT_ACT, 1), (64, 1, 1, 3, 1, 1, abi.RELU, 70),
            # 3x3 without padding and with more than it needs; 33 channels: Clip bounds inside the int8 range (see below)
            (20, 9, 9, 3, 1, 0, abi.RELU, 2), (33, 10, 8, 3, 2, 2, abi.CLIP, 2), (272, 31, 33, 3, 1, 1, abi.CLIP, 1)]


def _dw_chain_desc(shape):
    c, h, w, k, s, pad, act, n = shape
    # 33 channels: Clip to [-1, 2.5], i.e. to [-27, 68] output steps, so that the activation's bounds and not the
    # quantiser's are what clamps
    lo, hi = (-1.0, 2.5) if c == 33 else (0.0, 6.0)
    d = cases.cd(c, c, k, s, pad, h, w, act=act, group=c, n=n, input_scale=0.013, clip_min=lo, clip_max=hi,
                 leaky_relu_alpha=0.1, hard_sigmoid_alpha=0.2, hard_sigmoid_beta=0.5)
    return d


@pytest.mark.parametrize("shape", DW_CHAIN, ids=["x".join(map(str, s)) for s in DW_CHAIN])
def test_depthwise_w8a8_nhwc_chain_form(shape, torch_dev, oracle):
    """depthwise int8 convolutions with int8 NHWC on both sides (conv.c:617-755 followed by the consumer's quantiser,
    :961-973): the reference's int8 values exactly, padding channels zero, and the two mixed forms of a model edge (fp32
    NCHW in / int8 NHWC out, int8 NHWC in / fp32 NCHW out) equal to the reference's fp32 result and its quantisation"""
    torch = torch_dev
    d = _dw_chain_desc(shape)
    name = "dwchain_" + "x".join(map(str, shape))
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    lut = cases.silu_lut()
    ref32 = oracle.conv2d_w8a32(d, x, w8, b32, aux, lut)                    # fp32 NCHW
    dq = ConvDesc.from_buffer_copy(d)
    dq.out_s8, dq.output_scale = 1, 0.037
    ref8 = oracle.conv2d_w8a32(dq, x, w8, b32, aux, lut)                    # int8 NCHW
    assert np.array_equal(ref8, oracle.quantize_s8(ref32, dq.output_scale))
    xd, wd, bd, ad, ld = dev(torch, x), dev(torch, w8), dev(torch, b32), dev(torch, aux), dev(torch, lut)
    xq = hip.quantize_nhwc_s8(xd, d.input_scale)
    oh, ow = d.out_hw()
    cp = (d.cout + 15) // 16 * 16
    out = torch.full((d.n, oh, ow, cp), 77, dtype=torch.int8, device="cuda")
    hip.conv2d_w8a8_nhwc(dq, xq, wd, bd, ad, ld, out=out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got[..., :d.cout], np.transpose(ref8, (0, 2, 3, 1))), f"{name}: int8 values differ"
    assert not got[..., d.cout:].any(), f"{name}: padding channels are not zero"
    # int8 in, fp32 out
    y32 = hip.conv2d_w8_link(d, wd, bd, ad, ld, xq=xq)
    torch.cuda.synchronize()
    assert np.array_equal(y32.cpu().numpy(), ref32), f"{name}: fp32 result from int8 activations differs"
    # fp32 in, int8 out
    y8 = hip.conv2d_w8_link(dq, wd, bd, ad, ld, x=xd)
    torch.cuda.synchronize()
    assert np.array_equal(y8.cpu().numpy(), got), f"{name}: int8 result from fp32 activations differs"
    # and the fp32 form is untouched by all this
    y = hip.conv2d_w8a32(d, xd, wd, bd, ad, ld)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), ref32)
