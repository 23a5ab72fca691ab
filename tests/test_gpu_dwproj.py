"""onhip_dw_project_f32 (depthwise 3x3 + activation -> 1x1 convolution [+ residual Add] in one launch) against the oracle's
chain of the separate operators, through the C-ABI.

  * with an identity matrix as the 1x1 weights the output IS the depthwise result: it must equal the oracle's depthwise
    convolution bit for bit (same operations in the same order as the reference's depthwise path);
  * with real weights: within 1e-4 of the oracle chain  conv (depthwise) -> conv (1x1) -> add.
"""
import numpy as np
import pytest

import cases
from onenew_amd import abi, hip

# The kernel these tests cover (depthwise 3x3 + 1x1 projection in one launch, onhip_dw_project_f32) was taken out of the
# library: the whole-block kernel (onhip_ir_block_f32, tests/test_gpu_irblock.py) runs every block it was faster on, and
# on every other shape it lost to the two separate launches.  The tests stay as the record of what it had to satisfy.
pytestmark = [pytest.mark.gpu, pytest.mark.skip(reason="onhip_dw_project_f32 is no longer part of the library: superseded by the "
                                                       "one-launch block kernel, slower than two launches elsewhere")]


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    hip.init(0)
    return torch


def dev(torch, a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def descs(n, ce, hw, co, stride, dw_act=abi.CLIP, pw_bias=1):
    dw = cases.cd(ce, ce, 3, stride, 1, hw, n=n, group=ce, act=dw_act, clip_min=0.0, clip_max=6.0)
    oh, ow = dw.out_hw()
    pw = cases.cd(ce, co, 1, 1, 0, oh, w=ow, n=n, act=abi.NOT_ACT, bias=pw_bias)
    return dw, pw


def operands(tag, dw, pw):
    x = cases.datagen.uniform(cases.datagen.seed_for(tag, "x"), (dw.n, dw.cin, dw.h, dw.w), -3.0, 3.0)
    dw_w = cases.datagen.normal(cases.datagen.seed_for(tag, "dww"), (dw.cin, 1, 3, 3), 0.0, 0.5)
    dw_b = cases.datagen.normal(cases.datagen.seed_for(tag, "dwb"), (dw.cin,), 0.0, 0.3)
    pw_w = cases.datagen.normal(cases.datagen.seed_for(tag, "pww"), (pw.cout, pw.cin, 1, 1), 0.0, float(np.sqrt(1.0 / pw.cin)))
    pw_b = cases.datagen.normal(cases.datagen.seed_for(tag, "pwb"), (pw.cout,), 0.0, 0.1) if pw.has_bias else None
    return x, dw_w, dw_b, pw_w, pw_b


# (n, expanded channels, input size, output channels, stride, residual): the MobileNetV2 pairs at a small batch, and
# ragged ones (pixels not a multiple of 64, output channels not a multiple of 32, odd sizes with stride 2)
SHAPES = [(2, 32, 28, 16, 1, False), (2, 96, 28, 24, 2, False), (1, 144, 28, 24, 1, True), (2, 192, 14, 64, 2, False),
          (1, 384, 14, 96, 1, True), (1, 576, 7, 96, 2, False), (2, 960, 7, 128, 1, False), (3, 48, 9, 40, 1, True),
          (1, 16, 15, 8, 2, False), (1, 64, 5, 100, 1, False), (1, 32, 112, 16, 1, False), (1, 96, 112, 24, 2, True),
          (2, 16, 30, 33, 1, False), (1, 32, 128, 8, 1, False)]


@pytest.mark.parametrize("shape", SHAPES)
def test_dw_project_equals_the_operator_chain(shape, torch_dev, oracle):
    torch = torch_dev
    n, ce, hw, co, stride, with_res = shape
    print(f"dw+project {shape}", flush=True)
    dw, pw = descs(n, ce, hw, co, stride)
    assert hip.dw_project_supported(dw, pw) >= 1
    x, dw_w, dw_b, pw_w, pw_b = operands(f"dwproj{shape}", dw, pw)
    oh, ow = dw.out_hw()
    res = cases.datagen.normal(cases.datagen.seed_for("dwproj", "res", *shape[:5]), (n, co, oh, ow), 0.0, 1.0) if with_res else None
    packed = hip.dw_project_pack_weights(dev(torch, pw_w))
    y = hip.dw_project_f32(dw, pw, dev(torch, x), dev(torch, dw_w), dev(torch, dw_b), packed, dev(torch, pw_b), dev(torch, res))
    torch.cuda.synchronize()
    mid = oracle.conv2d_f32(dw, x, dw_w, dw_b)
    ref = oracle.conv2d_f32(pw, mid, pw_w, pw_b)
    if with_res:
        ref = ref + res
    got = y.cpu().numpy().astype(np.float64)
    top = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-4 * top, f"{np.abs(got - ref).max():.3e} against {top:.3e}"
    assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-4 * 0.1 * top)


@pytest.mark.parametrize("shape", [(2, 32, 28, 1), (1, 96, 30, 2), (2, 128, 14, 1), (1, 112, 7, 2), (1, 16, 9, 1), (1, 32, 112, 2)])
@pytest.mark.parametrize("act", [abi.CLIP, abi.RELU, abi.NOT_ACT, abi.LEAKYRELU])
def test_depthwise_half_is_the_reference_depthwise_bit_for_bit(shape, act, torch_dev, oracle):
    """1x1 weights = identity, no bias: every output is 1 * (one depthwise value) + zeros, i.e. the depthwise result itself"""
    torch = torch_dev
    n, ce, hw, stride = shape
    dw, pw = descs(n, ce, hw, ce, stride, dw_act=act, pw_bias=0)
    dw.leaky_relu_alpha = 0.1
    x, dw_w, dw_b, _, _ = operands(f"dwid{shape}", dw, pw)
    eye = np.eye(ce, dtype=np.float32).reshape(ce, ce, 1, 1)
    packed = hip.dw_project_pack_weights(dev(torch, eye))
    y = hip.dw_project_f32(dw, pw, dev(torch, x), dev(torch, dw_w), dev(torch, dw_b), packed)
    torch.cuda.synchronize()
    ref = oracle.conv2d_f32(dw, x, dw_w, dw_b)
    got = y.cpu().numpy()
    assert np.array_equal(got, ref), f"{(got != ref).sum()} of {ref.size} depthwise values differ"


def test_dw_project_says_what_it_does_not_take(torch_dev):
    torch = torch_dev
    dw, pw = descs(1, 24, 8, 8, 1)                       # channels not a multiple of 16
    assert hip.dw_project_supported(dw, pw) == 0
    z = torch.zeros(16, device="cuda")
    with pytest.raises(hip.OnhipError, match="multiple of 16"):
        hip.dw_project_f32(dw, pw, z, z, z, z, z)
    dw, pw = descs(1, 32, 8, 400, 1)                     # too many output channels
    assert hip.dw_project_supported(dw, pw) == 0
    dw5 = cases.cd(32, 32, 5, 1, 2, 8, group=32)
    assert hip.dw_project_supported(dw5, pw) == 0
    dw, pw = descs(64, 96, 112, 24, 2)
    assert hip.dw_project_supported(dw, pw) == 2         # MobileNetV2's first strided block at batch 64: recommended
