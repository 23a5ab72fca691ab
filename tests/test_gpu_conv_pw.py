"""onhip_conv2d_pw_f32 (a convolution with at most 64 output channels and the 1x1 convolution over its result, [+ Add of a
residual tensor, + Relu], in one launch) through the C-ABI: against the oracle's chain of the two (three, four) separate
operators within 1e-4, and bit for bit against the library's own two launches on the tile the fused kernel uses.
"""
import numpy as np
import pytest

import cases
from onenew_amd import abi, hip

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    hip.init(0)
    return torch


def dev(torch, a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def descs(n, cin, cmid, h, w, cout, k, s, p, act_a, act_b, bias_a=1, bias_b=1):
    a = cases.cd(cin, cmid, k, s, p, h, w=w, n=n, act=act_a, bias=bias_a, clip_min=0.0, clip_max=6.0)
    oh, ow = a.out_hw()
    b = cases.cd(cmid, cout, 1, 1, 0, oh, w=ow, n=n, act=act_b, bias=bias_b, clip_min=-1.0, clip_max=2.5)
    return a, b


def operands(tag, a, b):
    g = cases.datagen
    x = g.uniform(g.seed_for(tag, "x"), (a.n, a.cin, a.h, a.w), -2.0, 2.0)
    wa = g.normal(g.seed_for(tag, "wa"), (a.cout, a.cin, a.kh, a.kw), 0.0, float(np.sqrt(2.0 / (a.cin * a.kh * a.kw))))
    ba = g.normal(g.seed_for(tag, "ba"), (a.cout,), 0.3, 0.5) if a.has_bias else None
    wb = g.normal(g.seed_for(tag, "wb"), (b.cout, b.cin, 1, 1), 0.0, float(np.sqrt(1.0 / b.cin)))
    bb = g.normal(g.seed_for(tag, "bb"), (b.cout,), 0.0, 0.2) if b.has_bias else None
    return x, wa, ba, wb, bb


def close(got, ref):
    got = got.astype(np.float64)
    top = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-4 * top, f"{np.abs(got - ref).max():.3e} against {top:.3e}"
    assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-4 * 0.1 * top)


# (n, cin, cmid, h, w, cout, filter, stride, pad, first activation, second activation, residual, relu after it):
# ResNet-50's first-stage pair at batch 2, then ragged ones: pixels not a multiple of 64 (and fewer than 64), middle
# channels below 64 and not a multiple of 32 or of 4, output channels not a multiple of 64 or of 32, strides, a 5x5 and a 1x3
# filter, asymmetric padding, a padded 1x1, and every activation pair the entry point takes
N, R, CL = abi.NOT_ACT, abi.RELU, abi.CLIP
SHAPES = [(2, 64, 64, 56, 56, 256, 3, 1, 1, R, N, True, True), (2, 64, 64, 56, 56, 256, 3, 1, 1, R, R, False, False),
          (1, 16, 32, 20, 20, 64, 3, 1, 1, R, N, False, False), (1, 8, 48, 9, 11, 100, 3, 1, 1, CL, CL, True, False),
          (3, 20, 60, 13, 7, 17, 3, 2, 1, N, R, True, True), (1, 32, 4, 15, 15, 300, 5, 1, 2, R, CL, False, False),
          (1, 5, 35, 12, 30, 33, (1, 3), 1, (0, 1, 0, 1), R, R, True, True), (2, 24, 64, 6, 6, 128, 3, 1, (1, 0, 1, 2), CL, N, False, False),
          (1, 12, 20, 10, 10, 40, 1, 1, 1, R, N, True, False), (1, 64, 64, 7, 9, 64, 3, 2, 1, R, R, False, False)]


@pytest.mark.parametrize("shape", SHAPES)
def test_pair_equals_the_operator_chain(shape, torch_dev, oracle):
    torch = torch_dev
    n, cin, cmid, h, w, cout, k, s, p, act_a, act_b, with_res, relu = shape
    print(f"conv + 1x1 {shape}", flush=True)
    a, b = descs(n, cin, cmid, h, w, cout, k, s, p, act_a, act_b)
    assert hip.conv2d_pw_supported(a, b) >= 1
    x, wa, ba, wb, bb = operands(f"convpw{shape}", a, b)
    oh, ow = a.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("convpw", "res", *shape[:6]), (n, cout, oh, ow), 0.0, 1.0) if with_res else None
    packed = hip.pack_conv_weights(a, dev(torch, wa))
    y = hip.conv2d_pw_f32(a, b, dev(torch, x), packed, dev(torch, ba), hip.conv2d_pw_pack_weights(b, dev(torch, wb)), dev(torch, bb), dev(torch, res), relu)
    torch.cuda.synchronize()
    mid = oracle.conv2d_f32(a, x, wa, ba)
    if act_a != N:
        assert 0.02 < np.mean(mid == 0.0) < 0.9   # the first activation's lower bound is in play
    ref = oracle.conv2d_f32(b, mid, wb, bb).astype(np.float64)
    if with_res:
        ref = ref + res
        if relu:
            ref = np.maximum(ref, 0.0)
    close(y.cpu().numpy(), ref)


def _random_shapes(count=24):
    """seeded draws over everything the entry point takes: 1-64 middle channels, 1-200 output channels, 1-3 images, filters
    of 1-5 rows and columns (never a plain 1x1), strides 1-3, paddings up to the filter's reach, every activation pair"""
    rng = np.random.default_rng(20251)
    out = []
    while len(out) < count:
        n, cin, cmid, cout = int(rng.integers(1, 4)), int(rng.integers(4, 40)), int(rng.integers(1, 65)), int(rng.integers(1, 201))
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        pads = tuple(int(rng.integers(0, k)) for k in (kh, kw, kh, kw))
        if kh == 1 and kw == 1 and not any(pads):
            continue
        h, w, s = int(rng.integers(kh, 24)), int(rng.integers(kw, 24)), int(rng.integers(1, 4))
        act_a, act_b = (int(rng.choice([N, R, CL])) for _ in range(2))
        out.append((n, cin, cmid, h, w, cout, (kh, kw), s, pads, act_a, act_b, bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("shape", _random_shapes())
def test_pair_random_shapes(shape, torch_dev, oracle):
    torch = torch_dev
    n, cin, cmid, h, w, cout, k, s, p, act_a, act_b, with_res, relu = shape
    print(f"conv + 1x1, drawn shape {shape}", flush=True)
    a, b = descs(n, cin, cmid, h, w, cout, k, s, p, act_a, act_b)
    assert hip.conv2d_pw_supported(a, b) >= 1
    x, wa, ba, wb, bb = operands(f"convpw_rand{shape}", a, b)
    oh, ow = a.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("convpw_rand", "res", *shape[:6]), (n, cout, oh, ow), 0.0, 1.0) if with_res else None
    y = hip.conv2d_pw_f32(a, b, dev(torch, x), hip.pack_conv_weights(a, dev(torch, wa)), dev(torch, ba),
                          hip.conv2d_pw_pack_weights(b, dev(torch, wb)), dev(torch, bb), dev(torch, res), relu and with_res)
    torch.cuda.synchronize()
    ref = oracle.conv2d_f32(b, oracle.conv2d_f32(a, x, wa, ba), wb, bb).astype(np.float64)
    if with_res:
        ref = ref + res
        if relu:
            ref = np.maximum(ref, 0.0)
    close(y.cpu().numpy(), ref)


@pytest.mark.parametrize("bias_a,bias_b", [(0, 1), (1, 0), (0, 0)])
def test_pair_without_biases(bias_a, bias_b, torch_dev, oracle):
    """a convolution without bias has no activation either (conv.c:18-27), in both places"""
    torch = torch_dev
    a, b = descs(1, 16, 40, 12, 12, 96, 3, 1, 1, R, R, bias_a, bias_b)
    x, wa, ba, wb, bb = operands(f"convpw_nobias{bias_a}{bias_b}", a, b)
    packed = hip.pack_conv_weights(a, dev(torch, wa))
    y = hip.conv2d_pw_f32(a, b, dev(torch, x), packed, dev(torch, ba), hip.conv2d_pw_pack_weights(b, dev(torch, wb)), dev(torch, bb))
    torch.cuda.synchronize()
    mid = oracle.conv2d_f32(a, x, wa, ba)
    ref = oracle.conv2d_f32(b, mid, wb, bb).astype(np.float64)
    assert (mid < 0).any() == (not bias_a) and (ref < 0).any() == (not bias_b)
    close(y.cpu().numpy(), ref)


@pytest.mark.parametrize("shape", [(2, 64, 64, 56, 56, 256, 3, 1, 1, R, N, True, True), (1, 8, 48, 9, 11, 100, 3, 1, 1, CL, CL, True, False),
                                   (3, 20, 60, 13, 7, 17, 3, 2, 1, N, R, False, False)])
def test_pair_has_the_bits_of_the_two_launches_on_its_tile(shape, torch_dev, monkeypatch):
    """both products of the fused kernel sum in the order of the 64 x 64 tile's K loop, so with that tile forced on the two
    separate launches (whole K, no split) the results are the same bits, residual Add and Relu included"""
    torch = torch_dev
    n, cin, cmid, h, w, cout, k, s, p, act_a, act_b, with_res, relu = shape
    a, b = descs(n, cin, cmid, h, w, cout, k, s, p, act_a, act_b)
    x, wa, ba, wb, bb = operands(f"convpw_bits{shape}", a, b)
    oh, ow = a.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("convpw_bits", "res", *shape[:6]), (n, cout, oh, ow), 0.0, 1.0) if with_res else None
    packed = hip.pack_conv_weights(a, dev(torch, wa))
    dx, dba, dwb, dbb, dres = dev(torch, x), dev(torch, ba), dev(torch, wb), dev(torch, bb), dev(torch, res)
    y = hip.conv2d_pw_f32(a, b, dx, packed, dba, hip.conv2d_pw_pack_weights(b, dwb), dbb, dres, relu)
    monkeypatch.setenv("ONHIP_TILE", "64x64x1")
    mid = hip.conv2d_f32(a, dx, packed, dba, packed=True)
    assert list(hip.last_launch_choice())[:3] == [64, 64, 1]
    if with_res:
        two = hip.conv2d_f32_add(b, mid, dwb, dres, dbb, relu=relu)
    else:
        two = hip.conv2d_f32(b, mid, dwb, dbb)
    assert list(hip.last_launch_choice())[:5] == [64, 64, 1, 0, 0]
    torch.cuda.synchronize()
    assert torch.equal(y, two), f"{(y != two).sum().item()} of {y.numel()} values differ"


def test_resnet50_first_stage_pair_at_batch_32(torch_dev, monkeypatch):
    """the pair the benchmark runs (3x3 64 -> 64 with Relu, then 1x1 64 -> 256, on 56 x 56 at batch 32; with and without
    the block's Add and Relu), tensors drawn on the device: the same bits as the two launches on the 64 x 64 tile, which the
    full-size tests check against float64 sums"""
    torch = torch_dev
    a, b = descs(32, 64, 64, 56, 56, 256, 3, 1, 1, R, R)
    g = torch.Generator(device="cuda")
    g.manual_seed(20240)
    draw = lambda shape, std: torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * std
    x, res = draw((32, 64, 56, 56), 1.0), draw((32, 256, 56, 56), 1.0)
    wa, ba, wb, bb = draw((64, 64, 3, 3), 0.06), draw((64,), 0.1), draw((256, 64, 1, 1), 0.12), draw((256,), 0.1)
    packed, wb_packed = hip.pack_conv_weights(a, wa), hip.conv2d_pw_pack_weights(b, wb)
    assert hip.conv2d_pw_supported(a, b) == 2
    y = hip.conv2d_pw_f32(a, b, x, packed, ba, wb_packed, bb)
    y_res = hip.conv2d_pw_f32(a, b, x, packed, ba, wb_packed, bb, res, True)
    monkeypatch.setenv("ONHIP_TILE", "64x64x1")
    mid = hip.conv2d_f32(a, x, packed, ba, packed=True)
    two = hip.conv2d_f32(b, mid, wb, bb)
    two_res = hip.conv2d_f32_add(b, mid, wb, res, bb, relu=True)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all()) and 0.2 < float((y == 0).float().mean()) < 0.8
    assert torch.equal(y, two), f"{(y != two).sum().item()} of {y.numel()} values differ"
    assert torch.equal(y_res, two_res), f"{(y_res != two_res).sum().item()} of {y.numel()} values differ"


@pytest.mark.parametrize("shape", [(2, 16, 32, 20, 20, 64, 3, 1, 1, R, N, True, True), (1, 8, 48, 9, 11, 100, 3, 2, 1, CL, R, False, False)])
def test_plugin_eval_pair_host_buffers(shape, torch_dev, oracle):
    """the Conv plugin's eval_pair / eval_pair_relu on tensors in host memory, slots filled like the host fills a Conv's
    (weights and biases as fixed operands, the pair's result operand in params[4]): within 1e-4 of the oracle's operator
    chain, a second call (cached weights) identical, and eval_pair_takes saying that so small a batch is not recommended"""
    from onenew_amd import ops
    n, cin, cmid, h, w, cout, k, s, p, act_a, act_b, with_res, relu = shape
    a, b = descs(n, cin, cmid, h, w, cout, k, s, p, act_a, act_b)
    x, wa, ba, wb, bb = operands(f"convpw_plugin{shape}", a, b)
    oh, ow = a.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("convpw_plugin", "res", *shape[:6]), (n, cout, oh, ow), 0.0, 1.0) if with_res else None
    pair = ops.ConvPair(ops.Plugin(hip.plugin_path("Conv")), (a, b), (wa, wb), (ba, bb))
    assert pair.takes() == 0
    y = pair(x, addend=res, relu=relu).copy()
    assert np.array_equal(pair(x, addend=res, relu=relu), y)
    ref = oracle.conv2d_f32(b, oracle.conv2d_f32(a, x, wa, ba), wb, bb).astype(np.float64)
    if with_res:
        ref = np.maximum(ref + res, 0.0) if relu else ref + res
    close(y, ref)


def test_pair_refuses_what_it_cannot_run(torch_dev):
    torch = torch_dev
    ok_a, ok_b = descs(1, 16, 32, 10, 10, 64, 3, 1, 1, R, N)
    assert hip.conv2d_pw_supported(ok_a, ok_b) == 1
    big_a, big_b = descs(8, 64, 64, 56, 56, 256, 3, 1, 1, R, N)
    assert hip.conv2d_pw_supported(big_a, big_b) == 2
    bad = [descs(1, 16, 96, 10, 10, 64, 3, 1, 1, R, N),          # more than 64 middle channels
           descs(1, 16, 32, 10, 10, 64, 1, 1, 0, R, N),          # the first convolution is a plain 1x1
           descs(1, 3, 32, 32, 32, 64, 7, 2, 3, R, N),           # a first layer
           descs(1, 3, 32, 10, 10, 64, 5, 1, 2, R, N),           # fewer than four input channels: no tap-major weights
           descs(1, 16, 32, 10, 10, 64, 3, 1, 1, abi.SILU, N),   # a table activation
           descs(1, 16, 32, 10, 10, 64, 3, 1, 1, R, abi.LEAKYRELU)]
    for a, b in bad:
        assert hip.conv2d_pw_supported(a, b) == 0
    a, b = ok_a, ok_b
    b2 = cases.cd(32, 64, 1, 2, 0, 10, n=1, act=N)               # second convolution with a stride
    assert hip.conv2d_pw_supported(a, b2) == 0
    b3 = cases.cd(32, 64, 1, 1, 0, 12, n=1, act=N)               # does not read the first one's result
    assert hip.conv2d_pw_supported(a, b3) == 0
    x, wa, ba, wb, bb = operands("convpw_refuse", a, b)
    packed = hip.pack_conv_weights(a, dev(torch, wa))
    with pytest.raises(hip.OnhipError):
        hip.conv2d_pw_f32(a, b2, dev(torch, x), packed, dev(torch, ba), hip.conv2d_pw_pack_weights(b, dev(torch, wb)), dev(torch, bb))
    y = torch.empty((1, 64, 10, 10), dtype=torch.float32, device="cuda")
    with pytest.raises(hip.OnhipError):
        hip.conv2d_pw_f32(a, b, dev(torch, x), packed, dev(torch, ba), hip.conv2d_pw_pack_weights(b, dev(torch, wb)), dev(torch, bb), addend=y, out=y)
