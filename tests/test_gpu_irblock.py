"""onhip_ir_block_f32 (1x1 expansion -> depthwise 3x3 -> 1x1 projection [+ residual Add] in one launch) against the
oracle's chain of the three (four) separate operators, through the C-ABI, within 1e-4; and, stage by stage, against the
oracle with identity matrices in the places of the other two stages.
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


def descs(n, cin, ce, h, w, co, stride, act=abi.CLIP, pw_bias=1, clip=(0.0, 6.0)):
    ex = cases.cd(cin, ce, 1, 1, 0, h, w=w, n=n, act=act, clip_min=clip[0], clip_max=clip[1])
    dw = cases.cd(ce, ce, 3, stride, 1, h, w=w, n=n, group=ce, act=act, clip_min=clip[0], clip_max=clip[1])
    oh, ow = dw.out_hw()
    pw = cases.cd(ce, co, 1, 1, 0, oh, w=ow, n=n, act=abi.NOT_ACT, bias=pw_bias)
    return ex, dw, pw


def operands(tag, ex, dw, pw):
    g = cases.datagen
    x = g.uniform(g.seed_for(tag, "x"), (ex.n, ex.cin, ex.h, ex.w), -3.0, 3.0)
    ex_w = g.normal(g.seed_for(tag, "exw"), (ex.cout, ex.cin, 1, 1), 0.0, float(np.sqrt(2.0 / ex.cin)))
    ex_b = g.normal(g.seed_for(tag, "exb"), (ex.cout,), 0.5, 0.5)
    dw_w = g.normal(g.seed_for(tag, "dww"), (dw.cin, 1, 3, 3), 0.0, 0.5)
    dw_b = g.normal(g.seed_for(tag, "dwb"), (dw.cin,), 0.0, 0.3)
    pw_w = g.normal(g.seed_for(tag, "pww"), (pw.cout, pw.cin, 1, 1), 0.0, float(np.sqrt(1.0 / pw.cin)))
    pw_b = g.normal(g.seed_for(tag, "pwb"), (pw.cout,), 0.0, 0.1) if pw.has_bias else None
    return x, ex_w, ex_b, dw_w, dw_b, pw_w, pw_b


# (n, input channels, expanded channels, h, w, output channels, stride, residual): MobileNetV2's blocks on the 112, 56 and
# 28 pixel planes at a small batch (and one on the 14 pixel plane, rows of an even number of floats that is not a multiple
# of four), then ragged ones (odd heights, a last band shorter than the others, bands of one row
# and of the whole image, output channels not a multiple of 32, 64 input channels)
SHAPES = [(2, 16, 96, 112, 112, 24, 2, False), (1, 24, 144, 56, 56, 24, 1, True), (2, 24, 144, 56, 56, 32, 2, False),
          (2, 32, 192, 28, 28, 32, 1, True), (2, 32, 192, 28, 28, 64, 2, False), (1, 16, 48, 20, 20, 40, 1, False),
          (2, 32, 64, 9, 12, 64, 2, False), (1, 24, 32, 37, 36, 24, 1, True), (1, 64, 128, 8, 8, 64, 1, True),
          (1, 64, 128, 16, 16, 33, 1, False), (1, 16, 16, 5, 128, 8, 1, False), (3, 32, 160, 11, 44, 17, 2, False),
          (2, 64, 384, 14, 14, 64, 1, True), (1, 32, 64, 9, 18, 40, 2, False), (1, 16, 32, 6, 6, 16, 1, False)]


@pytest.mark.parametrize("shape", SHAPES)
def test_block_equals_the_operator_chain(shape, torch_dev, oracle):
    torch = torch_dev
    n, cin, ce, h, w, co, stride, with_res = shape
    print(f"inverted-residual block {shape}", flush=True)
    ex, dw, pw = descs(n, cin, ce, h, w, co, stride)
    assert hip.ir_block_supported(ex, dw, pw) >= 1
    x, ex_w, ex_b, dw_w, dw_b, pw_w, pw_b = operands(f"irblock{shape}", ex, dw, pw)
    oh, ow = dw.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("irblock", "res", *shape[:7]), (n, co, oh, ow), 0.0, 1.0) if with_res else None
    packed = hip.ir_block_pack_weights(dev(torch, ex_w), dev(torch, pw_w))
    y = hip.ir_block_f32(ex, dw, pw, dev(torch, x), packed, dev(torch, ex_b), dev(torch, dw_w), dev(torch, dw_b), dev(torch, pw_b),
                         dev(torch, res))
    torch.cuda.synchronize()
    wide = oracle.conv2d_f32(ex, x, ex_w, ex_b)
    assert 0.05 < np.mean(wide == 0.0) < 0.6 and np.mean(wide == 6.0) > 1e-3   # both clip bounds are in play
    mid = oracle.conv2d_f32(dw, wide, dw_w, dw_b)
    ref = oracle.conv2d_f32(pw, mid, pw_w, pw_b)
    if with_res:
        ref = ref + res
    got = y.cpu().numpy().astype(np.float64)
    top = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-4 * top, f"{np.abs(got - ref).max():.3e} against {top:.3e}"
    assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-4 * 0.1 * top)


@pytest.mark.parametrize("shape", [(2, 16, 28, 28, 1), (1, 32, 30, 32, 2), (1, 64, 9, 16, 1), (1, 32, 56, 56, 2)])
@pytest.mark.parametrize("act", [abi.CLIP, abi.RELU, abi.LEAKYRELU])
def test_depthwise_stage_is_the_reference_depthwise_bit_for_bit(shape, act, torch_dev, oracle):
    """expansion = identity matrix with zero bias on an input inside the activation's linear range, projection = identity
    without bias: every output is the depthwise value of the input itself, which must equal the oracle's depthwise
    convolution bit for bit (1 * x + zeros is x in any summation order)"""
    torch = torch_dev
    n, c, h, w, stride = shape
    ex, dw, pw = descs(n, c, c, h, w, c, stride, act=act, pw_bias=0, clip=(0.0, 6.0))
    ex.leaky_relu_alpha = dw.leaky_relu_alpha = 0.1
    g = cases.datagen
    x = g.uniform(g.seed_for("irid", *shape), (n, c, h, w), 0.25, 5.0)   # CLIP, RELU and LEAKYRELU leave these as they are
    dw_w = g.normal(g.seed_for("irid", "dww", *shape), (c, 1, 3, 3), 0.0, 0.5)
    dw_b = g.normal(g.seed_for("irid", "dwb", *shape), (c,), 0.0, 0.3)
    eye = np.eye(c, dtype=np.float32).reshape(c, c, 1, 1)
    zero_b = np.zeros(c, np.float32)
    packed = hip.ir_block_pack_weights(dev(torch, eye), dev(torch, eye))
    y = hip.ir_block_f32(ex, dw, pw, dev(torch, x), packed, dev(torch, zero_b), dev(torch, dw_w), dev(torch, dw_b))
    torch.cuda.synchronize()
    ref = oracle.conv2d_f32(dw, x, dw_w, dw_b)
    got = y.cpu().numpy()
    assert np.array_equal(got, ref), f"{(got != ref).sum()} of {ref.size} depthwise values differ"


@pytest.mark.parametrize("shape", [(2, 16, 96, 28, 28, 24, 2, False), (1, 32, 64, 20, 20, 32, 1, True)])
def test_plugin_eval_block_host_buffers(shape, torch_dev, oracle):
    """the Conv plugin's eval_block on tensors in host memory, slots filled like the host fills a Conv's (weights and
    biases as fixed operands, the block's result operand in params[4]): within 1e-4 of the oracle's operator chain, a second
    call (cached weights) identical, and eval_block_takes saying that so small a batch is not recommended"""
    from onenew_amd import ops
    n, cin, ce, h, w, co, stride, with_res = shape
    ex, dw, pw = descs(n, cin, ce, h, w, co, stride)
    x, ex_w, ex_b, dw_w, dw_b, pw_w, pw_b = operands(f"irplugin{shape}", ex, dw, pw)
    oh, ow = dw.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("irplugin", "res", *shape[:7]), (n, co, oh, ow), 0.0, 1.0) if with_res else None
    block = ops.ConvBlock(ops.Plugin(hip.plugin_path("Conv")), (ex, dw, pw), (ex_w, dw_w, pw_w), (ex_b, dw_b, pw_b))
    assert block.takes() == 0
    y = block(x, addend=res).copy()
    assert np.array_equal(block(x, addend=res), y)
    ref = oracle.conv2d_f32(pw, oracle.conv2d_f32(dw, oracle.conv2d_f32(ex, x, ex_w, ex_b), dw_w, dw_b), pw_w, pw_b)
    if with_res:
        ref = ref + res
    top = np.abs(ref).max()
    assert np.abs(y.astype(np.float64) - ref).max() <= 1e-4 * top


def test_block_says_what_it_does_not_take(torch_dev):
    torch = torch_dev
    z = torch.zeros(64, device="cuda")
    ex, dw, pw = descs(1, 64, 128, 7, 7, 64, 1)            # rows of 7 pixels: an odd number of floats
    assert hip.ir_block_supported(ex, dw, pw) == 0
    with pytest.raises(hip.OnhipError, match="band of output rows"):
        hip.ir_block_f32(ex, dw, pw, z, z, z, z, z, z)
    ex, dw, pw = descs(1, 48, 96, 16, 16, 24, 1)           # an input channel count without a kernel
    assert hip.ir_block_supported(ex, dw, pw) == 0
    ex, dw, pw = descs(1, 32, 96, 16, 16, 128, 1)          # too many output channels
    assert hip.ir_block_supported(ex, dw, pw) == 0
    ex, dw, pw = descs(1, 32, 96, 16, 16, 24, 1)
    ex.has_bias = 0                                        # the expansion's activation hangs on its bias (conv.c:18-27)
    assert hip.ir_block_supported(ex, dw, pw) == 0
    ex, dw, pw = descs(64, 16, 96, 112, 112, 24, 2)        # MobileNetV2's first expanding block at batch 64: recommended
    assert hip.ir_block_supported(ex, dw, pw) == 2
    ex, dw, pw = descs(1, 16, 96, 112, 112, 24, 2)         # at batch 1: taken, but the three launches are faster
    assert hip.ir_block_supported(ex, dw, pw) == 1
