"""bf16 / fp16 with 16-bit storage (onhip_conv2d_h16, onhip_linear_h16 and the conversions around them), through the
C-ABI, against the oracle on operands rounded with its own bf16 / fp16 rounding.

What is asserted:
  * conversions and weight packing: bit-equal to the oracle's round-to-nearest-even, channel padding zero;
  * fp32 outputs: within 1e-4 (normalised) of the oracle's fp32 convolution / MatMul on the rounded operands, and within
    1e-2 of the same on the unrounded operands (the tolerance the reduced-precision modes are specified with);
  * 16-bit outputs: bit-equal to the rounding of the fp32 output of the same problem (one rounding after bias and
    activation), and with a residual operand bit-equal to round(relu(round(y) + r)) computed in fp32;
  * every tile of the kernel, 64- and 128-byte stages, ragged rows and columns, strides and padding.
"""
import numpy as np
import pytest

import cases
from onenew_amd import abi, hip
from onenew_amd.abi import ConvDesc

pytestmark = pytest.mark.gpu

TYPES = [abi.COMPUTE_BF16, abi.COMPUTE_F16]


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    hip.init(0)
    return torch


def dev(torch, a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rounder(oracle, compute):
    return oracle.round_bf16 if compute == abi.COMPUTE_BF16 else oracle.round_f16


def norm_diff(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30)


def with_compute(d, compute):
    dd = ConvDesc.from_buffer_copy(d)
    dd.compute = compute
    return dd


@pytest.mark.parametrize("compute", TYPES)
@pytest.mark.parametrize("shape", [(2, 3, 9, 11), (1, 40, 5, 7), (3, 64, 4, 4), (1, 100, 17, 3)])
def test_layout_conversions_round_like_the_oracle(compute, shape, torch_dev, oracle):
    torch = torch_dev
    x = cases.datagen.normal(cases.datagen.seed_for("h16conv", *shape), shape, 0.0, 3.0)
    x.reshape(-1)[::7] *= np.float32(1e-3)
    xh = hip.h16_from_nchw(dev(torch, x), compute)
    back = hip.h16_to_nchw(xh, shape[1], compute)
    torch.cuda.synchronize()
    ref = rounder(oracle, compute)(x)
    nhwc = xh.float().cpu().numpy()
    assert nhwc.shape == (shape[0], shape[2], shape[3], hip.h16_pitch(shape[1]))
    assert np.array_equal(nhwc[..., :shape[1]], np.transpose(ref, (0, 2, 3, 1)))
    assert not nhwc[..., shape[1]:].any(), "channel padding must be zero"
    assert np.array_equal(back.cpu().numpy(), ref)
    rows = x.reshape(-1, shape[3])
    rh = hip.h16_from_rows(dev(torch, rows), compute)
    rb = hip.h16_to_rows(rh, shape[3], compute)
    torch.cuda.synchronize()
    assert np.array_equal(rb.cpu().numpy(), ref.reshape(-1, shape[3]))
    assert not rh.float().cpu().numpy()[:, shape[3]:].any()


@pytest.mark.parametrize("compute", TYPES)
def test_weight_packing_is_tap_major_and_rounded(compute, torch_dev, oracle):
    torch = torch_dev
    d = with_compute(cases.cd(13, 9, 3, 1, 1, 7), compute)
    _, w, _ = cases.conv_inputs("h16pack", d)
    wp = hip.h16_pack_conv_weights(d, dev(torch, w)).float().cpu().numpy()
    ref = rounder(oracle, compute)(w)
    assert wp.shape == (9, 9, 32)
    assert np.array_equal(wp[..., :13], np.transpose(ref.reshape(9, 13, 9), (0, 2, 1)))
    assert not wp[..., 13:].any()
    b = cases.datagen.normal(cases.datagen.seed_for("h16pack", "b"), (50, 24), 0.0, 1.0)
    bp = hip.h16_pack_matmul_weights(dev(torch, b), compute).float().cpu().numpy()
    assert bp.shape == (24, 64)
    assert np.array_equal(bp[:, :50], rounder(oracle, compute)(b).T)
    assert not bp[:, 50:].any()


# (n, cin, hw, cout, k, stride, pad): ragged rows / columns, 64-byte stages (cin <= 32 or 96), 128-byte stages (64, 128),
# one tap and many, strides, a single stage per tap and several
CONV_SHAPES = [(1, 64, 56, 64, 3, 1, 1), (2, 13, 9, 9, 1, 1, 0), (1, 3, 30, 8, 7, 2, 3), (2, 96, 13, 72, 3, 2, 1),
               (3, 128, 9, 130, 1, 1, 0), (1, 256, 7, 33, 3, 1, 1), (2, 32, 16, 200, 5, 1, 2)]


def run_conv_h16(torch, oracle, d, name, tile, monkeypatch, lut=None):
    """-> (x, w, b rounded as the kernel sees them, fp32 NHWC result, fp32 NCHW result, 16-bit NHWC result as fp32)"""
    if tile:
        monkeypatch.setenv("ONHIP_TILE", tile)
    rnd = rounder(oracle, d.compute)
    x, w, b = cases.conv_inputs(name, d)
    xh = hip.h16_from_nchw(dev(torch, x), d.compute)
    wp = hip.h16_pack_conv_weights(d, dev(torch, w))
    launches = hip.load().onhip_direct_lds_launches()
    args = (d, xh, wp, dev(torch, b), dev(torch, lut))
    y_nhwc = hip.conv2d_h16(*args, y_kind=hip.H16_OUT_F32_NHWC)
    y_nchw = hip.conv2d_h16(*args, y_kind=hip.H16_OUT_F32_NCHW)
    oh, ow = d.out_hw()
    out16 = torch.full((d.n, oh, ow, hip.h16_pitch(d.cout)), 7.0, dtype=xh.dtype, device="cuda")
    hip.conv2d_h16(*args, y_kind=hip.H16_OUT_NHWC, out=out16)
    torch.cuda.synchronize()
    assert hip.load().onhip_direct_lds_launches() == launches + 3
    return x, w, b, rnd, y_nhwc.cpu().numpy(), y_nchw.cpu().numpy(), out16


@pytest.mark.parametrize("compute", TYPES)
@pytest.mark.parametrize("ring", [1, 2])
@pytest.mark.parametrize("tile", ["128x128", "128x64", "64x128", "64x64"])
@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv_h16_every_tile(compute, ring, tile, shape, torch_dev, oracle, monkeypatch):
    """ring: 1 = stage buffers within 64 KiB of LDS, 2 = the long ring (up to 144 KiB)"""
    torch = torch_dev
    tile = f"{tile}x1x0x0x0x{ring}"
    n, cin, hw, cout, k, stride, pad = shape
    d = with_compute(cases.cd(cin, cout, k, stride, pad, hw, n=n, act=abi.RELU), compute)
    name = f"h16_{cin}_{cout}_{k}_{stride}"
    print(f"case {name} tile {tile} compute {compute}", flush=True)
    x, w, b, rnd, y_nhwc, y_nchw, out16 = run_conv_h16(torch, oracle, d, name, tile, monkeypatch)
    ref = oracle.conv2d_f32(d, rnd(x), rnd(w), b)
    assert np.array_equal(y_nhwc, np.transpose(y_nchw, (0, 2, 3, 1))), "the two fp32 layouts hold different values"
    assert norm_diff(y_nchw, ref) <= 1e-4, f"vs oracle on rounded operands: {norm_diff(y_nchw, ref):.3e}"
    assert norm_diff(y_nchw, oracle.conv2d_f32(d, x, w, b)) <= 1e-2
    got16 = out16.float().cpu().numpy()
    assert np.array_equal(got16[..., :cout], rnd(y_nhwc)), "16-bit store is not the rounding of the fp32 result"
    assert not got16[..., cout:].any(), "channel padding of the output must be zero"


# (n, cin, h, w, cout, kh, kw, stride, pad): first layers in their own storage form; the ResNet-50 / MobileNetV2 / YOLOv8
# stems in small, a ragged one (cin 1, 5 x 8 filter, stride 3, more padding than the filter needs), stride 1
FIRST_SHAPES = [(2, 3, 30, 30, 64, 7, 7, 2, 3), (1, 3, 20, 36, 32, 3, 3, 2, 1), (2, 1, 17, 23, 9, 5, 8, 3, 4),
                (1, 8, 12, 12, 40, 3, 3, 1, 1), (3, 4, 9, 40, 130, 1, 2, 1, 0), (2, 3, 11, 13, 24, 3, 3, 1, 1),
                (1, 5, 15, 15, 16, 4, 4, 3, 2)]


@pytest.mark.parametrize("compute", TYPES)
@pytest.mark.parametrize("tile", [None, "128x128", "128x64", "64x128", "64x64x1x0x0x0x2"])
@pytest.mark.parametrize("shape", FIRST_SHAPES)
def test_conv_h16_first_layer_form(compute, tile, shape, torch_dev, oracle, monkeypatch):
    """onhip_conv2d_h16_first against the oracle on rounded operands, and bit for bit against onhip_conv2d_h16 on the
    32-channel form where both take the shape with the same tile (same products, zeros added in between)"""
    torch = torch_dev
    if tile:
        monkeypatch.setenv("ONHIP_TILE", tile)
    n, cin, h, w, cout, kh, kw, stride, pad = shape
    d = ConvDesc(n=n, cin=cin, h=h, w=w, cout=cout, kh=kh, kw=kw, stride_h=stride, stride_w=stride, pad_t=pad, pad_l=pad,
                 pad_b=pad, pad_r=pad, group=1, has_bias=1, act_type=abi.RELU, compute=compute)
    name = f"h16first_{cin}_{cout}_{kh}x{kw}_{stride}"
    print(f"case {name} tile {tile} compute {compute}", flush=True)
    rnd = rounder(oracle, compute)
    x, wt, b = cases.conv_inputs(name, d)
    xf = hip.h16_first_from_nchw(d, dev(torch, x))
    wp_cols = xf.shape[2]
    oh, ow = d.out_hw()
    cpp = 4 if cin <= 4 else 8
    assert wp_cols == hip.load().onhip_h16_first_width(d) >= max(w + 2 * pad, (ow - 1) * stride + 8) and wp_cols % 2 == 0
    assert xf.shape[3] == hip.load().onhip_h16_first_channels(d) == cpp
    # the storage form itself: rounded pixels at column + pad_l, zeros around them and in the channels past cin
    got = xf.float().cpu().numpy()
    want = np.zeros((n, h, wp_cols, cpp), np.float32)
    want[:, :, pad:pad + w, :cin] = np.transpose(rnd(x), (0, 2, 3, 1))
    assert np.array_equal(got, want)
    wpk = hip.h16_first_pack_weights(d, dev(torch, wt))
    wwant = np.zeros((cout, kh, 8, cpp), np.float32)
    wwant[:, :, :kw, :cin] = np.transpose(rnd(wt), (0, 2, 3, 1))
    assert np.array_equal(wpk.float().cpu().numpy(), wwant)
    launches = hip.load().onhip_direct_lds_launches()
    y_nchw = hip.conv2d_h16_first(d, xf, wpk, dev(torch, b), y_kind=hip.H16_OUT_F32_NCHW).cpu().numpy()
    out16 = torch.full((n, oh, ow, hip.h16_pitch(cout)), 7.0, dtype=xf.dtype, device="cuda")
    hip.conv2d_h16_first(d, xf, wpk, dev(torch, b), y_kind=hip.H16_OUT_NHWC, out=out16)
    torch.cuda.synchronize()
    assert hip.load().onhip_direct_lds_launches() == launches + 2, "the first-layer form did not run on the direct-to-LDS kernel"
    ref = oracle.conv2d_f32(d, rnd(x), rnd(wt), b)
    assert norm_diff(y_nchw, ref) <= 1e-4, f"vs oracle on rounded operands: {norm_diff(y_nchw, ref):.3e}"
    assert norm_diff(y_nchw, oracle.conv2d_f32(d, x, wt, b)) <= 1e-2
    got16 = out16.float().cpu().numpy()
    assert np.array_equal(got16[..., :cout], rnd(np.transpose(y_nchw, (0, 2, 3, 1))))
    assert not got16[..., cout:].any(), "channel padding of the output must be zero"


def test_conv_h16_first_layer_form_refuses_what_it_cannot_store(torch_dev):
    d = ConvDesc(n=1, cin=9, h=8, w=8, cout=8, kh=3, kw=3, stride_h=1, stride_w=1, pad_t=1, pad_l=1, pad_b=1, pad_r=1,
                 group=1, has_bias=0, act_type=abi.NOT_ACT, compute=abi.COMPUTE_BF16)
    assert hip.load().onhip_h16_first_width(d) == 0          # nine channels
    d.cin, d.kw, d.pad_l, d.pad_r = 3, 9, 4, 4
    assert hip.load().onhip_h16_first_width(d) == 0          # filter rows of nine columns
    d.kw, d.pad_l, d.pad_r, d.compute = 3, 1, 1, abi.COMPUTE_F32
    x = torch_dev.zeros((1, 3, 8, 8), device="cuda")
    with pytest.raises(hip.OnhipError):
        hip.h16_first_from_nchw(d, x)                        # not a 16-bit type


@pytest.mark.parametrize("compute", TYPES)
@pytest.mark.parametrize("act", ["none", "clip", "silu", "leaky", "nobias"])
def test_conv_h16_activations(compute, act, torch_dev, oracle, monkeypatch):
    torch = torch_dev
    kw = {"none": dict(act=abi.NOT_ACT), "clip": dict(act=abi.CLIP, clip_min=0.0, clip_max=0.5), "silu": dict(act=abi.SILU),
          "leaky": dict(act=abi.LEAKYRELU, leaky_relu_alpha=0.1), "nobias": dict(act=abi.RELU, bias=0)}[act]
    d = with_compute(cases.cd(40, 50, 3, 1, 1, 14, n=2, **kw), compute)
    lut = cases.silu_lut() if act == "silu" else None
    x, w, b, rnd, y_nhwc, y_nchw, out16 = run_conv_h16(torch, oracle, d, f"h16act_{act}", None, monkeypatch, lut=lut)
    if act == "silu":
        # the table applied to the kernel's own sums (bin edges make a direct comparison ill-conditioned)
        dn = with_compute(d, compute)
        dn.act_type = abi.NOT_ACT
        _, _, _, _, _, pre, _ = run_conv_h16(torch, oracle, dn, f"h16act_{act}", None, monkeypatch)
        assert norm_diff(pre, oracle.conv2d_f32(dn, rnd(x), rnd(w), b)) <= 1e-4
        assert np.array_equal(y_nchw, oracle.lut_act(pre, lut))
    else:
        assert norm_diff(y_nchw, oracle.conv2d_f32(d, rnd(x), rnd(w), b)) <= 1e-4
    assert np.array_equal(out16.float().cpu().numpy()[..., :d.cout], rnd(y_nhwc))


@pytest.mark.parametrize("compute", TYPES)
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("tile", ["128x128", "64x64"])
def test_conv_h16_residual_operand(compute, relu, tile, torch_dev, oracle, monkeypatch):
    torch = torch_dev
    monkeypatch.setenv("ONHIP_TILE", tile)
    d = with_compute(cases.cd(64, 136, 1, 1, 0, 14, n=3, act=abi.NOT_ACT), compute)
    rnd = rounder(oracle, compute)
    x, w, b = cases.conv_inputs("h16res", d)
    r = cases.datagen.normal(cases.datagen.seed_for("h16res", "r"), (3, 136, 14, 14), 0.0, 1.0)
    xh, wp = hip.h16_from_nchw(dev(torch, x), compute), hip.h16_pack_conv_weights(d, dev(torch, w))
    rh = hip.h16_from_nchw(dev(torch, r), compute)
    y32 = hip.conv2d_h16(d, xh, wp, dev(torch, b), y_kind=hip.H16_OUT_F32_NHWC)
    y16 = hip.conv2d_h16(d, xh, wp, dev(torch, b), residual=rh, residual_relu=relu)
    torch.cuda.synchronize()
    want = rnd(y32.cpu().numpy()) + np.transpose(rnd(r), (0, 2, 3, 1))
    if relu:
        want = np.maximum(want, np.float32(0.0))
    got = y16.float().cpu().numpy()
    assert np.array_equal(got[..., :136], rnd(want.astype(np.float32)))
    assert not got[..., 136:].any()


VIT_LINEARS = [("qkv", 192, 576, False, False), ("proj", 192, 192, True, True), ("fc1", 192, 768, True, False), ("fc2", 768, 192, True, True)]


@pytest.mark.parametrize("compute", TYPES)
@pytest.mark.parametrize("layer", VIT_LINEARS, ids=[v[0] for v in VIT_LINEARS])
@pytest.mark.parametrize("batch", [1, 3])
def test_linear_h16_vit_layers(compute, layer, batch, torch_dev, oracle):
    """the four linear layers of a ViT-Tiny block with 16-bit operands: MatMul (+ bias) (+ table GELU for fc1) (+ the
    residual stream for proj and fc2)"""
    torch = torch_dev
    name, k, n, has_bias, has_res = layer
    rows = batch * 197
    rnd = rounder(oracle, compute)
    a = cases.datagen.normal(cases.datagen.seed_for("h16vit", name, "a"), (rows, k), 0.0, 1.0)
    bmat = cases.datagen.normal(cases.datagen.seed_for("h16vit", name, "b"), (k, n), 0.0, 0.05)
    bias = cases.datagen.normal(cases.datagen.seed_for("h16vit", name, "bias"), (n,), 0.0, 0.02) if has_bias else None
    lut = cases.gelu_lut() if name == "fc1" else None
    ah, bp = hip.h16_from_rows(dev(torch, a), compute), hip.h16_pack_matmul_weights(dev(torch, bmat), compute)
    pre = hip.linear_h16(ah, bp, k, n, compute, bias=dev(torch, bias), y_kind=hip.H16_OUT_F32_NHWC)
    y32 = hip.linear_h16(ah, bp, k, n, compute, bias=dev(torch, bias), gelu_lut=dev(torch, lut), y_kind=hip.H16_OUT_F32_NHWC)
    y16 = hip.linear_h16(ah, bp, k, n, compute, bias=dev(torch, bias), gelu_lut=dev(torch, lut))
    torch.cuda.synchronize()
    pre, y32 = pre.cpu().numpy(), y32.cpu().numpy()
    assert norm_diff(pre, oracle.matmul_f32(rnd(a), rnd(bmat), bias=bias)) <= 1e-4
    assert norm_diff(pre, oracle.matmul_f32(a, bmat, bias=bias)) <= 1e-2
    if lut is not None:
        assert np.array_equal(y32, oracle.lut_act(pre, lut))
    else:
        assert np.array_equal(y32, pre)
    got = y16.float().cpu().numpy()
    assert np.array_equal(got[:, :n], rnd(y32)) and not got[:, n:].any()
    if has_res:
        r = cases.datagen.normal(cases.datagen.seed_for("h16vit", name, "r"), (rows, n), 0.0, 1.0)
        rh = hip.h16_from_rows(dev(torch, r), compute)
        yr = hip.linear_h16(ah, bp, k, n, compute, bias=dev(torch, bias), residual=rh)
        torch.cuda.synchronize()
        assert np.array_equal(yr.float().cpu().numpy()[:, :n], rnd((rnd(y32) + rnd(r)).astype(np.float32)))


def test_h16_argument_errors(torch_dev):
    torch = torch_dev
    d = with_compute(cases.cd(32, 32, 3, 1, 1, 8), abi.COMPUTE_BF16)
    x = torch.zeros((1, 8, 8, 32), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((32, 9, 32), dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(32, device="cuda")
    r = torch.zeros((1, 8, 8, 32), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(hip.OnhipError, match="neither bf16 nor fp16"):
        hip.conv2d_h16(with_compute(d, abi.COMPUTE_F32), x, w, b)
    with pytest.raises(hip.OnhipError, match="residual operand goes with the 16-bit output"):
        hip.conv2d_h16(d, x, w, b, residual=r, y_kind=hip.H16_OUT_F32_NCHW)
    with pytest.raises(hip.OnhipError, match="16-byte aligned"):
        hip.conv2d_h16(d, torch.zeros(2048 + 8, dtype=torch.bfloat16, device="cuda")[4:4 + 2048], w, b)
    dw = with_compute(cases.cd(32, 32, 3, 1, 1, 8, group=32), abi.COMPUTE_BF16)
    with pytest.raises(hip.OnhipError, match="dense convolutions only"):
        hip.conv2d_h16(dw, x, w, b)
    big = with_compute(cases.cd(32, 32, 9, 1, 4, 12), abi.COMPUTE_BF16)
    with pytest.raises(hip.OnhipError, match="64 taps"):
        hip.conv2d_h16(big, torch.zeros((1, 12, 12, 32), dtype=torch.bfloat16, device="cuda"),
                       torch.zeros((32, 81, 32), dtype=torch.bfloat16, device="cuda"), b)
