"""The benchmark configurations at their stated sizes, every layer: ResNet-50 batch 32 (53 convolutions), MobileNetV2
batch 64 (52, of which 17 depthwise), the ViT-Tiny MatMuls at B = 64 in fp32 and bf16, YOLOv8s int8 batch 16 (63
convolutions, fp32-in/out W8A32 form and int8 NHWC chain form).  The dense fp32 layers are checked twice: with the tile
and split the cost model gives (a host calling `eval` gets those) and with the ones the library measures when tuning is
on, which is what the benchmark times; and, on the layers where the measured choice varies from box to box, under
each kernel variant it can fall on (B straight from memory, K slices added up inside the launch, leftover tiles cut
along K).

Tensors of this size are drawn on the device (seeded) and only what the check needs comes back to the host: for a
dense convolution the input patches of a few thousand sampled outputs, which are then evaluated on the CPU - float64
cross-correlation for fp32 (bar 1e-4 of the largest sampled value), the exact integer closed form of
device/x86/Conv/conv.c:961-973,1024-1056 for int8 (int64 sum, then the three separately rounded fp32 operations,
the table and the re-quantisation through the oracle's own functions; bar: equality).  Depthwise layers are compared
bit for bit with the oracle on whole images of the batch; the MatMuls with the oracle on the whole product."""
import numpy as np
import pytest

import cases
from onenew_amd import abi, datagen, hip, stacks
from onenew_amd.abi import ConvDesc

pytestmark = pytest.mark.gpu

SAMPLES = 2000


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    assert torch.cuda.is_available(), "no GPU visible"
    hip.init(0)
    return torch


def _seed(*parts):
    return datagen.seed_for("fullsize", *parts) & 0x7FFFFFFFFFFF


def _device_uniform(torch, seed, shape, lo=-1.0, hi=1.0):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.rand(shape, generator=g, device="cuda", dtype=torch.float32) * (hi - lo) + lo


def _sample_index(seed, d, count=SAMPLES):
    """sampled outputs as (image, channel, row, column) index arrays; corners and edges of the first and last image and
    channel are always among them (padding, the last tile's ragged rows and columns)"""
    oh, ow = d.out_hw()
    total = d.n * d.cout * oh * ow
    flat = datagen.integers(seed, (min(count, total),), 0, total - 1)
    fixed = [((n * d.cout + m) * oh + i) * ow + j for n in (0, d.n - 1) for m in (0, d.cout - 1)
             for i in (0, oh - 1) for j in (0, ow - 1)]
    flat = np.unique(np.concatenate([flat, np.array(fixed, np.int64)]))
    n, r = np.divmod(flat, d.cout * oh * ow)
    m, r = np.divmod(r, oh * ow)
    i, j = np.divmod(r, ow)
    return flat, n, m, i, j


def _patches(torch, x, d, n, i, j):
    """input patches [S, cin, kh, kw] of the sampled outputs, zero where the window hangs over the padding; pure data
    movement on the device, returned as a host array"""
    dv = x.device
    n_t = torch.from_numpy(n).to(dv)
    ih = torch.from_numpy(i * d.stride_h - d.pad_t).to(dv)[:, None] + torch.arange(d.kh, device=dv)[None, :]
    iw = torch.from_numpy(j * d.stride_w - d.pad_l).to(dv)[:, None] + torch.arange(d.kw, device=dv)[None, :]
    ok = ((ih >= 0) & (ih < d.h))[:, :, None] & ((iw >= 0) & (iw < d.w))[:, None, :]           # [S, kh, kw]
    ihc, iwc = ih.clamp(0, d.h - 1), iw.clamp(0, d.w - 1)
    c = torch.arange(d.cin, device=dv)
    p = x[n_t[:, None, None, None], c[None, :, None, None], ihc[:, None, :, None], iwc[:, None, None, :]]
    p = p * ok[:, None, :, :].to(p.dtype)
    return p.cpu().numpy()


def _act_f64(d, v):
    if not d.has_bias or d.act_type == abi.NOT_ACT:
        return v
    if d.act_type == abi.RELU:
        return np.maximum(v, 0.0)
    if d.act_type == abi.CLIP:
        return np.minimum(np.maximum(v, d.clip_min), d.clip_max)
    raise AssertionError("activation not used by these stacks")


def _check_dense_f32(torch, tag, name, d, w_std=None):
    x = _device_uniform(torch, _seed(tag, name, "x"), (d.n, d.cin, d.h, d.w))
    fan_in = d.cin * d.kh * d.kw
    w = datagen.normal(_seed(tag, name, "w"), (d.cout, d.cin, d.kh, d.kw), 0.0, w_std or float(np.sqrt(2.0 / fan_in)))
    b = datagen.normal(_seed(tag, name, "b"), (d.cout,), 0.0, 0.01)
    wd, bd = torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda()
    wp = hip.pack_conv_weights(d, wd)
    y = hip.conv2d_f32(d, x, wp if wp is not None else wd, bd, packed=wp is not None)
    torch.cuda.synchronize()
    flat, n, m, i, j = _sample_index(_seed(tag, name, "probe"), d)
    got = y.reshape(-1)[torch.from_numpy(flat).cuda()].cpu().numpy().astype(np.float64)
    p = _patches(torch, x, d, n, i, j).astype(np.float64)
    ref = _act_f64(d, np.einsum("sckl,sckl->s", p, w[m].astype(np.float64)) + b[m].astype(np.float64))
    scale = max(float(np.abs(ref).max()), 1e-6)
    assert np.abs(got - ref).max() <= 1e-4 * scale, f"{name}: {np.abs(got - ref).max():.3e} against {scale:.3e}"
    assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-5), name
    assert bool(torch.isfinite(y).all())


def _check_depthwise_f32(torch, oracle, tag, name, d):
    x = _device_uniform(torch, _seed(tag, name, "x"), (d.n, d.cin, d.h, d.w))
    w = datagen.normal(_seed(tag, name, "w"), (d.cout, 1, d.kh, d.kw), 0.0, 0.05)
    b = datagen.normal(_seed(tag, name, "b"), (d.cout,), 0.0, 0.01)
    y = hip.conv2d_f32(d, x, torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda())
    torch.cuda.synchronize()
    d1 = ConvDesc.from_buffer_copy(d)
    d1.n = 1
    pick = sorted({0, d.n - 1, int(datagen.integers(_seed(tag, name, "img"), (1,), 0, d.n - 1)[0])})
    for img in pick:
        ref = oracle.conv2d_f32(d1, x[img:img + 1].cpu().numpy(), w, b)
        assert np.array_equal(y[img:img + 1].cpu().numpy(), ref), f"{name}: image {img} differs from the oracle"
    # the images the oracle did not see: each is a function of its own input alone, so a copy of image `a` put
    # in place of image `c` must reproduce image a's result there
    a, c = pick[0], (pick[0] + 1) % d.n
    x2 = x.clone()
    x2[c] = x[a]
    y2 = hip.conv2d_f32(d, x2, torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda())
    torch.cuda.synchronize()
    assert torch.equal(y2[c], y[a])
    keep = [k for k in range(d.n) if k != c]
    assert torch.equal(y2[keep], y[keep])


@pytest.fixture
def measured_choices():
    """tile, split and kernel variant measured per problem shape on first use, as bench.py runs the stacks"""
    prev = hip.set_tuning(1)
    yield
    hip.set_tuning(prev)


RESNET = stacks.with_batch(stacks.resnet50(), 32)
MOBILENET = stacks.with_batch(stacks.mobilenet_v2(), 64)
YOLO = stacks.with_batch(stacks.yolov8s(), 16)


@pytest.mark.parametrize("layer", range(len(RESNET)), ids=[n for n, _ in RESNET])
def test_resnet50_batch32_every_layer(layer, torch_dev):
    name, d = RESNET[layer]
    print(f"resnet50 b32 {name}", flush=True)
    _check_dense_f32(torch_dev, "rn50b32", name, d)


@pytest.mark.parametrize("layer", range(len(RESNET)), ids=[n for n, _ in RESNET])
def test_resnet50_batch32_every_layer_measured_choice(layer, torch_dev, measured_choices):
    """the same check with the launch the library measures to be the fastest for the shape: what bench.py times"""
    name, d = RESNET[layer]
    _check_dense_f32(torch_dev, "rn50b32", name, d)
    print(f"resnet50 b32 {name}: measured choice (bm, bn, split, tail, rowb, fin, dma) = {hip.last_launch_choice()}", flush=True)


def _layer(stack, name):
    return next(d for n, d in stack if n == name)


# (layer, ONHIP_TILE, what must have run): the kernel variants the measured choice takes on these layers on one box or
# another - B straight from memory (rowb) on 1x1 stride-1 layers, K slices reduced by the last slice to arrive (fin)
# or by a finishing launch, the leftover tiles alone cut along K (tail)
FORCED = [("l1.0.conv1", "64x256x1x0x1", dict(rowb=1)), ("l1.0.conv3", "64x128x1x0x1", dict(rowb=1)),
          ("l1.1.conv1", "128x128x1x0x1", dict(rowb=1)), ("l2.0.conv1", "128x128x1x0x1", dict(rowb=1)),
          ("l2.1.conv3", "64x128x1x0x1", dict(rowb=1)), ("l3.0.conv1", "128x128x1x0x1", dict(rowb=1)),
          ("l4.0.conv1", "128x128x1x0x1", dict(rowb=1)), ("l2.0.down", "64x128", dict(rowb=0, split=1)),
          ("l3.1.conv2", "64x64x3x0x0x1", dict(split=3, fin=1)), ("l3.1.conv2", "64x64x3", dict(split=3, fin=0)),
          ("l3.0.conv2", "64x64x3x0x0x1", dict(split=3, fin=1)), ("l3.1.conv1", "64x64x2x0x0x1", dict(split=2, fin=1)),
          ("l3.1.conv3", "64x128x1x2x0x1", dict()), ("l4.0.conv2", "64x64x6x0x0x1", dict(split=6, fin=1)),
          ("l4.1.conv2", "64x64x6x0x0x1", dict(split=6, fin=1)), ("l4.1.conv2", "128x128x12x0x0x1", dict(split=12, fin=1)),
          ("l4.1.conv1", "64x64x4x0x0x1", dict(split=4, fin=1)), ("l4.1.conv3", "64x64x2x0x0x1", dict(split=2, fin=1)),
          ("l4.0.down", "64x64x2x0x0x1", dict(split=2, fin=1)), ("l2.1.conv2", "64x64x1x4x0x1", dict(tail=4, fin=1)),
          ("l2.1.conv2", "64x64x1x4", dict(tail=4, fin=0)), ("l1.1.conv2", "64x64x1x8x0x1", dict(tail=8, fin=1)),
          ("l2.1.conv1", "64x64x1x2x0x1", dict()), ("l3.0.conv1", "64x128x1x2x0x1", dict())]


@pytest.mark.parametrize("name,tile,ran", FORCED, ids=[f"{n}-{t}" for n, t, _ in FORCED])
def test_resnet50_batch32_forced_kernel_variants(name, tile, ran, torch_dev, monkeypatch):
    monkeypatch.setenv("ONHIP_TILE", tile)
    print(f"resnet50 b32 {name} forced {tile}", flush=True)
    _check_dense_f32(torch_dev, "rn50b32", name, _layer(RESNET, name))
    got = dict(zip(("bm", "bn", "split", "tail", "rowb", "fin", "dma"), hip.last_launch_choice()))
    print(f"  ran as {got}", flush=True)
    want = [int(v) for v in tile.split("x")[:2]]
    assert [got["bm"], got["bn"]] == want, (tile, got)
    for key, v in ran.items():
        assert got[key] == v, f"{name} {tile}: {key} = {got[key]}, expected {v} ({got})"


@pytest.mark.parametrize("layer", [i for i, (_, d) in enumerate(MOBILENET) if d.group == 1], ids=[n for n, d in MOBILENET if d.group == 1])
def test_mobilenetv2_batch64_every_dense_layer_measured_choice(layer, torch_dev, measured_choices):
    name, d = MOBILENET[layer]
    _check_dense_f32(torch_dev, "mbv2b64", name, d, w_std=0.05)
    print(f"mobilenetv2 b64 {name}: measured choice = {hip.last_launch_choice()}", flush=True)


@pytest.mark.parametrize("layer", range(len(MOBILENET)), ids=[n for n, _ in MOBILENET])
def test_mobilenetv2_batch64_every_layer(layer, torch_dev, oracle):
    name, d = MOBILENET[layer]
    print(f"mobilenetv2 b64 {name}", flush=True)
    if d.group != 1:
        _check_depthwise_f32(torch_dev, oracle, "mbv2b64", name, d)
    else:
        _check_dense_f32(torch_dev, "mbv2b64", name, d, w_std=0.05)


# the inverted-residual blocks the benchmark runs as one launch each (expansion, depthwise, projection)
IR_BLOCKS = [i for i in range(len(MOBILENET) - 2)
             if MOBILENET[i][1].group == 1 and MOBILENET[i + 1][1].group != 1 and MOBILENET[i][1].kh == 1]


@pytest.mark.parametrize("first", IR_BLOCKS, ids=[MOBILENET[i][0].replace(".expand", "") for i in IR_BLOCKS])
def test_mobilenetv2_batch64_blocks_in_one_launch(first, torch_dev, oracle):
    """every block the library recommends for the one-launch kernel at batch 64: three whole images against the oracle's
    chain of the three convolutions (1e-4 of the largest value), and the other images through the fact that an image's
    result depends on its own input alone"""
    torch = torch_dev
    (name, ex), (_, dw), (_, pw) = MOBILENET[first], MOBILENET[first + 1], MOBILENET[first + 2]
    want = hip.ir_block_supported(ex, dw, pw)
    print(f"mobilenetv2 b64 block {name}: supported = {want}", flush=True)
    if want < 2:
        pytest.skip("not a shape of the one-launch block kernel: the benchmark runs its three convolutions")
    x = _device_uniform(torch, _seed("mbv2blk", name, "x"), (ex.n, ex.cin, ex.h, ex.w))
    r = lambda role, shape, std, mean=0.0: datagen.normal(_seed("mbv2blk", name, role), shape, mean, std)   # noqa: E731
    ex_w, ex_b = r("exw", (ex.cout, ex.cin, 1, 1), float(np.sqrt(2.0 / ex.cin))), r("exb", (ex.cout,), 0.3, 0.3)
    dw_w, dw_b = r("dww", (dw.cout, 1, 3, 3), 0.4), r("dwb", (dw.cout,), 0.2)
    pw_w, pw_b = r("pww", (pw.cout, pw.cin, 1, 1), float(np.sqrt(1.0 / pw.cin))), r("pwb", (pw.cout,), 0.1)
    cu = lambda a: torch.from_numpy(a).cuda()   # noqa: E731
    packed = hip.ir_block_pack_weights(cu(ex_w), cu(pw_w))
    args = (packed, cu(ex_b), cu(dw_w), cu(dw_b), cu(pw_b))
    y = hip.ir_block_f32(ex, dw, pw, x, *args)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all())
    one = [ConvDesc.from_buffer_copy(d) for d in (ex, dw, pw)]
    for d in one:
        d.n = 1
    pick = sorted({0, ex.n - 1, int(datagen.integers(_seed("mbv2blk", name, "img"), (1,), 0, ex.n - 1)[0])})
    for img in pick:
        wide = oracle.conv2d_f32(one[0], x[img:img + 1].cpu().numpy(), ex_w, ex_b)
        ref = oracle.conv2d_f32(one[2], oracle.conv2d_f32(one[1], wide, dw_w, dw_b), pw_w, pw_b).astype(np.float64)
        got = y[img:img + 1].cpu().numpy().astype(np.float64)
        top = np.abs(ref).max()
        assert np.abs(got - ref).max() <= 1e-4 * top, f"{name} image {img}: {np.abs(got - ref).max():.3e} against {top:.3e}"
        assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-5 * top), name
    a, c = pick[0], (pick[0] + 1) % ex.n
    x2 = x.clone()
    x2[c] = x[a]
    y2 = hip.ir_block_f32(ex, dw, pw, x2, *args)
    torch.cuda.synchronize()
    assert torch.equal(y2[c], y[a])
    keep = [k for k in range(ex.n) if k != c]
    assert torch.equal(y2[keep], y[keep])


# ---- ViT-Tiny MatMuls at B = 64 -------------------------------------------------------------------------------

VIT = stacks.vit_tiny(64)


@pytest.mark.parametrize("tuned", [0, 1], ids=["cost_model", "measured_choice"])
@pytest.mark.parametrize("compute", [abi.COMPUTE_F32, abi.COMPUTE_BF16, abi.COMPUTE_F16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("layer", range(len(VIT)), ids=[v[0] for v in VIT])
def test_vit_tiny_batch64_every_matmul(layer, compute, tuned, torch_dev, oracle, request):
    torch = torch_dev
    prev = hip.set_tuning(tuned)
    request.addfinalizer(lambda: hip.set_tuning(prev))
    name, md, has_bias, gelu = VIT[layer]
    print(f"vit b64 {name} compute {compute}", flush=True)
    ashape = (md.batch, md.m, md.k)
    bshape = (md.k, md.n) if md.b_shared else (md.batch, md.k, md.n)
    a = datagen.normal(_seed("vit", name, "a"), ashape, 0.0, 1.0)
    b = datagen.normal(_seed("vit", name, "b"), bshape, 0.0, 0.02)
    bias = datagen.normal(_seed("vit", name, "bias"), (md.n,), 0.0, 0.02) if has_bias else None
    lut = cases.gelu_lut() if gelu else None
    cu = lambda t: None if t is None else torch.from_numpy(t).cuda()
    y = hip.matmul(cu(a), cu(b), bias=cu(bias), compute=compute)          # pre-activation
    torch.cuda.synchronize()
    y = y.cpu().numpy()

    def full(aa, bb):
        r = oracle.matmul_f32(aa, bb)
        return r + bias if has_bias else r

    ref32 = full(a, b)
    scale = float(np.abs(ref32).max())
    if compute == abi.COMPUTE_F32:
        assert np.abs(y - ref32).max() <= 1e-4 * scale, name
        assert np.all(np.abs(y - ref32) <= 1e-4 * np.abs(ref32) + 1e-5), name
    else:
        rnd = oracle.round_bf16 if compute == abi.COMPUTE_BF16 else oracle.round_f16
        ref16 = full(rnd(a), rnd(b))                 # operands rounded to the 16-bit type, fp32 accumulation
        assert np.abs(y - ref16).max() <= 1e-4 * scale, name
        assert np.abs(y - ref32).max() <= 1e-2 * scale, name
    if gelu:
        # the fused table activation, judged exactly on the kernel's own pre-activation
        yg = hip.matmul(cu(a), cu(b), bias=cu(bias), gelu_lut=cu(lut), compute=compute)
        torch.cuda.synchronize()
        assert np.array_equal(yg.cpu().numpy(), oracle.lut_act(y, lut)), name


# ---- 16-bit storage at full size ---------------------------------------------------------------------------------------
def _round16(torch, t, compute):
    """the operand as the 16-bit kernels see it, back in fp32 (torch's conversion is round-to-nearest-even, the
    oracle's rule; the small tests compare the library's conversions with the oracle's bit for bit)"""
    return t.to(torch.bfloat16 if compute == abi.COMPUTE_BF16 else torch.float16).float()


@pytest.mark.parametrize("compute", [abi.COMPUTE_BF16, abi.COMPUTE_F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("layer", [i for i, v in enumerate(VIT) if v[1].b_shared], ids=[v[0] for v in VIT if v[1].b_shared])
def test_vit_tiny_batch64_linear_layers_16bit_storage(layer, compute, torch_dev, oracle):
    """qkv / proj / fc1 / fc2 at batch 64 with operands and result stored in 16 bits: the fp32 output against the oracle on
    rounded operands (1e-4) and on the unrounded ones (1e-2); the 16-bit output is the rounding of the fp32 one"""
    torch = torch_dev
    name, md, has_bias, gelu = VIT[layer]
    print(f"vit b64 {name} 16-bit storage compute {compute}", flush=True)
    rows = md.batch * md.m
    a = datagen.normal(_seed("vit", name, "a"), (rows, md.k), 0.0, 1.0)
    b = datagen.normal(_seed("vit", name, "b"), (md.k, md.n), 0.0, 0.02)
    bias = datagen.normal(_seed("vit", name, "bias"), (md.n,), 0.0, 0.02) if has_bias else None
    lut = cases.gelu_lut() if gelu else None
    cu = lambda t: None if t is None else torch.from_numpy(t).cuda()
    ah, bp = hip.h16_from_rows(cu(a), compute), hip.h16_pack_matmul_weights(cu(b), compute)
    pre = hip.linear_h16(ah, bp, md.k, md.n, compute, bias=cu(bias), y_kind=hip.H16_OUT_F32_NHWC)
    y32 = hip.linear_h16(ah, bp, md.k, md.n, compute, bias=cu(bias), gelu_lut=cu(lut), y_kind=hip.H16_OUT_F32_NHWC)
    y16 = hip.linear_h16(ah, bp, md.k, md.n, compute, bias=cu(bias), gelu_lut=cu(lut))
    torch.cuda.synchronize()
    rnd = oracle.round_bf16 if compute == abi.COMPUTE_BF16 else oracle.round_f16
    ref16 = oracle.matmul_f32(rnd(a), rnd(b), bias=bias)
    ref32 = oracle.matmul_f32(a, b, bias=bias)
    scale = float(np.abs(ref32).max())
    pre = pre.cpu().numpy()
    assert np.abs(pre - ref16).max() <= 1e-4 * scale, name
    assert np.abs(pre - ref32).max() <= 1e-2 * scale, name
    y32 = y32.cpu().numpy()
    assert np.array_equal(y32, oracle.lut_act(pre, lut) if gelu else pre)
    got = y16.float().cpu().numpy()
    assert np.array_equal(got[:, :md.n], rnd(y32)) and not got[:, md.n:].any()


@pytest.mark.parametrize("layer", range(len(RESNET)), ids=[n for n, _ in RESNET])
def test_resnet50_batch32_every_layer_bf16_storage(layer, torch_dev):
    """every convolution of the stack with bf16 NHWC tensors: sampled outputs of the fp32 form against the float64 sum over
    the rounded operands; the bf16 output (what the next layer reads) is the rounding of the fp32 one everywhere"""
    torch = torch_dev
    name, d = RESNET[layer]
    print(f"resnet50 b32 bf16 {name}", flush=True)
    d = ConvDesc.from_buffer_copy(d)
    d.compute = abi.COMPUTE_BF16
    x = _device_uniform(torch, _seed("rn50b32h", name, "x"), (d.n, d.cin, d.h, d.w))
    w = datagen.normal(_seed("rn50b32h", name, "w"), (d.cout, d.cin, d.kh, d.kw), 0.0, float(np.sqrt(2.0 / (d.cin * d.kh * d.kw))))
    b = datagen.normal(_seed("rn50b32h", name, "b"), (d.cout,), 0.0, 0.01)
    wd, bd = torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda()
    xh, wp = hip.h16_from_nchw(x, d.compute), hip.h16_pack_conv_weights(d, wd)
    y32 = hip.conv2d_h16(d, xh, wp, bd, y_kind=hip.H16_OUT_F32_NCHW)
    y16 = hip.conv2d_h16(d, xh, wp, bd)
    torch.cuda.synchronize()
    flat, n, m, i, j = _sample_index(_seed("rn50b32h", name, "probe"), d)
    got = y32.reshape(-1)[torch.from_numpy(flat).cuda()].cpu().numpy().astype(np.float64)
    p = _patches(torch, _round16(torch, x, d.compute), d, n, i, j).astype(np.float64)
    wr = _round16(torch, wd, d.compute).cpu().numpy().astype(np.float64)
    ref = _act_f64(d, np.einsum("sckl,sckl->s", p, wr[m]) + b[m].astype(np.float64))
    scale = max(float(np.abs(ref).max()), 1e-6)
    assert np.abs(got - ref).max() <= 1e-4 * scale, f"{name}: {np.abs(got - ref).max():.3e} against {scale:.3e}"
    want16 = y32.permute(0, 2, 3, 1).to(torch.bfloat16)
    assert torch.equal(y16[..., :d.cout], want16), name
    assert not bool(y16[..., d.cout:].any())


def test_resnet50_batch32_stem_bf16_in_the_first_layer_form(torch_dev):
    """the stem as the bf16 benchmark runs it (8 channels per pixel, a filter row per tap): sampled outputs against the
    float64 sum over the rounded operands; the bf16 store is the rounding of the fp32 one"""
    torch = torch_dev
    name, d = RESNET[0]
    assert d.cin == 3 and d.kh == 7
    d = ConvDesc.from_buffer_copy(d)
    d.compute = abi.COMPUTE_BF16
    x = _device_uniform(torch, _seed("rn50b32h", name, "x"), (d.n, d.cin, d.h, d.w))
    w = datagen.normal(_seed("rn50b32h", name, "w"), (d.cout, d.cin, d.kh, d.kw), 0.0, float(np.sqrt(2.0 / (d.cin * d.kh * d.kw))))
    b = datagen.normal(_seed("rn50b32h", name, "b"), (d.cout,), 0.0, 0.01)
    wd, bd = torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda()
    xf, wp = hip.h16_first_from_nchw(d, x), hip.h16_first_pack_weights(d, wd)
    y32 = hip.conv2d_h16_first(d, xf, wp, bd, y_kind=hip.H16_OUT_F32_NCHW)
    y16 = hip.conv2d_h16_first(d, xf, wp, bd)
    torch.cuda.synchronize()
    flat, n, m, i, j = _sample_index(_seed("rn50b32h", name, "probe"), d)
    got = y32.reshape(-1)[torch.from_numpy(flat).cuda()].cpu().numpy().astype(np.float64)
    p = _patches(torch, _round16(torch, x, d.compute), d, n, i, j).astype(np.float64)
    wr = _round16(torch, wd, d.compute).cpu().numpy().astype(np.float64)
    ref = _act_f64(d, np.einsum("sckl,sckl->s", p, wr[m]) + b[m].astype(np.float64))
    scale = max(float(np.abs(ref).max()), 1e-6)
    assert np.abs(got - ref).max() <= 1e-4 * scale, f"{name}: {np.abs(got - ref).max():.3e} against {scale:.3e}"
    assert torch.equal(y16[..., :d.cout], y32.permute(0, 2, 3, 1).to(torch.bfloat16))
    assert not bool(y16[..., d.cout:].any())


# ---- YOLOv8s int8, batch 16 ---------------------------------------------------------------------------------------

def _yolo_operands(torch, i, name, d):
    d = ConvDesc.from_buffer_copy(d)
    d.input_scale = float(datagen.uniform(_seed("yolo", i, "s_in"), (1,), 0.005, 0.05)[0])
    # activations as the configuration draws them: U(-1, 1), scaled so that a few per cent clip at +-127 steps
    x = _device_uniform(torch, _seed("yolo", name, "x"), (d.n, d.cin, d.h, d.w)) * float(d.input_scale * 140.0)
    w8 = datagen.integers(_seed("yolo", name, "w"), (d.cout, d.cin, d.kh, d.kw), -127, 127).astype(np.int8)
    b32 = datagen.integers(_seed("yolo", name, "b"), (d.cout,), -100, 100).astype(np.int32)
    s_w = float(datagen.uniform(_seed("yolo", name, "aux"), (1,), 0.005, 0.05)[0])
    aux = np.full((d.cout,), np.float32(127.0) * np.float32(s_w), np.float32)      # per-tensor weight scale
    return d, x, w8, b32, aux


def _int8_closed_form(oracle, d, patches, w8, b32, aux, m, lut):
    """conv.c:961-973 (quantise), :1024-1039 (int32 sum), :1041-1056 (three rounded fp32 operations), do_act"""
    q = oracle.quantize_s8(patches, d.input_scale).astype(np.int64)
    acc = np.einsum("sckl,sckl->s", q, w8[m].astype(np.int64))
    assert np.abs(acc).max() < 2 ** 31
    f = acc.astype(np.int32).astype(np.float32)
    f = f * np.float32(d.input_scale)
    f = f + b32[m].astype(np.float32)
    y = f * (aux[m] * np.float32(1.0) / np.float32(127.0))
    if d.act_type == abi.SILU:
        y = oracle.lut_act(y, lut)
    return acc.astype(np.int32), y.astype(np.float32)


@pytest.mark.parametrize("layer", range(len(YOLO)), ids=[n for n, _ in YOLO])
def test_yolov8s_int8_batch16_every_layer(layer, torch_dev, oracle):
    torch = torch_dev
    name, d0 = YOLO[layer]
    print(f"yolov8s b16 {name}", flush=True)
    d, x, w8, b32, aux = _yolo_operands(torch, layer, name, d0)
    lut = cases.silu_lut()
    cu = lambda t: torch.from_numpy(t).cuda()
    w8d, b32d, auxd, lutd = cu(w8), cu(b32), cu(aux), cu(lut)
    oh, ow = d.out_hw()
    flat, n, m, i, j = _sample_index(_seed("yolo", name, "probe"), d)
    flat_t = torch.from_numpy(flat).cuda()
    acc_ref, y_ref = _int8_closed_form(oracle, d, _patches(torch, x, d, n, i, j), w8, b32, aux, m, lut)

    # the reference's form: fp32 NCHW in and out, int32 accumulators on request
    wp = hip.pack_conv_weights_w8(d, w8d)
    acc = torch.empty((d.n, d.cout, oh, ow), dtype=torch.int32, device="cuda")
    y = hip.conv2d_w8a32(d, x, wp, b32d, auxd, lutd, acc32=acc, packed=True)
    torch.cuda.synchronize()
    assert np.array_equal(acc.reshape(-1)[flat_t].cpu().numpy(), acc_ref), f"{name}: int32 accumulators differ"
    assert np.array_equal(y.reshape(-1)[flat_t].cpu().numpy(), y_ref), f"{name}: de-quantised outputs differ"
    y_full = y
    del acc

    # the chain form: int8 NHWC in, int8 NHWC out; equals the consumer's own quantisation of the fp32 result
    dq = ConvDesc.from_buffer_copy(d)
    dq.out_s8, dq.output_scale = 1, 0.03
    xq = hip.quantize_nhwc_s8(x, d.input_scale)
    cpo = (d.cout + 15) // 16 * 16
    out = torch.full((d.n, oh, ow, cpo), 77, dtype=torch.int8, device="cuda")
    hip.conv2d_w8a8_nhwc(dq, xq, wp, b32d, auxd, lutd, out=out)
    torch.cuda.synchronize()
    q_ref = oracle.quantize_s8(y_ref, dq.output_scale)
    nhwc = ((n * oh + i) * ow + j) * cpo + m
    assert np.array_equal(out.reshape(-1)[torch.from_numpy(nhwc).cuda()].cpu().numpy(), q_ref), f"{name}: chain form differs"
    # and, over the whole tensor, the chain form is the quantisation of the fp32 form's result (same accumulators)
    want = hip.quantize_nhwc_s8(y_full, dq.output_scale)
    assert torch.equal(out[..., :d.cout], want[..., :d.cout]), f"{name}: chain form is not the quantised fp32 form everywhere"


# ---- MobileNetV2 depthwise layers in the int8 NHWC chain form, batch 64 -------------------------------------------------
DW_LAYERS = [i for i, (_, d) in enumerate(MOBILENET) if d.group != 1]


@pytest.mark.parametrize("layer", DW_LAYERS, ids=[MOBILENET[i][0] for i in DW_LAYERS])
def test_mobilenetv2_batch64_depthwise_int8_chain_form(layer, torch_dev, oracle):
    """every depthwise layer with int8 NHWC activations in and out (conv.c:617-755 + the consumer's quantiser :961-973):
    three whole images against the oracle bit for bit, and over the whole batch the int8 result is the quantisation of what
    the fp32-in / fp32-out form of the same layer returns (that form is checked against the oracle the same way)"""
    torch = torch_dev
    name, d0 = MOBILENET[layer]
    print(f"mobilenetv2 b64 int8 {name}", flush=True)
    d = ConvDesc.from_buffer_copy(d0)
    d.input_scale = 0.021
    x = _device_uniform(torch, _seed("mbv2q", name, "x"), (d.n, d.cin, d.h, d.w)) * 3.0      # a few per cent clip at +-127
    w8 = datagen.integers(_seed("mbv2q", name, "w"), (d.cout, 1, d.kh, d.kw), -127, 127).astype(np.int8)
    b32 = datagen.integers(_seed("mbv2q", name, "b"), (d.cout,), -300, 300).astype(np.int32)
    aux = datagen.uniform(_seed("mbv2q", name, "aux"), (d.cout,), 0.5, 3.0)
    cu = lambda t: torch.from_numpy(t).cuda()   # noqa: E731
    w8d, b32d, auxd = cu(w8), cu(b32), cu(aux)
    y32 = hip.conv2d_w8a32(d, x, w8d, b32d, auxd)
    dq = ConvDesc.from_buffer_copy(d)
    dq.out_s8, dq.output_scale = 1, 0.045
    xq = hip.quantize_nhwc_s8(x, d.input_scale)
    oh, ow = d.out_hw()
    cp = (d.cout + 15) // 16 * 16
    out = torch.full((d.n, oh, ow, cp), 77, dtype=torch.int8, device="cuda")
    hip.conv2d_w8a8_nhwc(dq, xq, w8d, b32d, auxd, out=out)
    torch.cuda.synchronize()
    d1 = ConvDesc.from_buffer_copy(dq)
    d1.n = 1
    for img in sorted({0, d.n - 1, int(datagen.integers(_seed("mbv2q", name, "img"), (1,), 0, d.n - 1)[0])}):
        ref = oracle.conv2d_w8a32(d1, x[img:img + 1].cpu().numpy(), w8, b32, aux)            # int8 NCHW
        assert np.array_equal(out[img, :, :, :d.cout].cpu().numpy(), np.transpose(ref[0], (1, 2, 0))), f"{name}: image {img}"
    want = hip.quantize_nhwc_s8(y32, dq.output_scale)
    assert torch.equal(out[..., :d.cout], want[..., :d.cout]), f"{name}: not the quantised fp32 form everywhere"
    assert not bool(out[..., d.cout:].any())
