"""onhip_attention against the oracle's operator chain  Transpose -> MatMul -> [Mul] -> Softmax -> MatMul -> Transpose
(the reference's ViT block runs exactly these operators one after the other), through the C-ABI; the first case is the
ViT-Tiny configuration at its full batch of 64.  Tolerance 1e-4
(normalised maximum and per element), the tolerance of the fp32 MatMul and of the Softmax's expf."""
import numpy as np
import pytest

import cases
from onenew_amd import hip

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_dev():
    import torch
    hip.init(0)
    return torch


def oracle_chain(oracle, qkv, b, t, h, hd, scale):
    """qkv: [b, t, 3, h, hd] as the projection writes it -> merged context [b, t, h * hd]"""
    x = oracle.transpose_f32(qkv.reshape(b, t, 3 * h, hd), (0, 2, 1, 3)).reshape(b, 3, h, t, hd)   # head split
    q, k, v = x[:, 0], x[:, 1], x[:, 2]
    kt = oracle.transpose_f32(np.ascontiguousarray(k), (0, 1, 3, 2))
    s = oracle.matmul_f32(np.ascontiguousarray(q).reshape(b * h, t, hd), kt.reshape(b * h, hd, t))
    if scale != 1.0:
        s = (s * np.float32(scale)).astype(np.float32)
    p = oracle.softmax_f32(s)
    ctx = oracle.matmul_f32(p, np.ascontiguousarray(v).reshape(b * h, t, hd)).reshape(b, h, t, hd)
    return oracle.transpose_f32(ctx, (0, 2, 1, 3)).reshape(b, t, h * hd)                            # head merge


@pytest.mark.parametrize("shape", [(64, 3, 197, 64, 0.125), (2, 3, 197, 64, 0.125), (1, 1, 17, 32, 1.0), (3, 2, 64, 64, 0.125), (1, 4, 129, 32, 0.25),
                                   (2, 1, 256, 64, 0.125), (1, 2, 5, 64, 1.0), (1, 3, 224, 64, 0.125), (2, 2, 33, 32, 0.5)])
def test_attention_equals_the_operator_chain(shape, torch_dev, oracle):
    torch = torch_dev
    b, h, t, hd, scale = shape
    print(f"attention {shape}", flush=True)
    qkv = cases.datagen.normal(cases.datagen.seed_for("attn", *shape[:4]), (b, t, 3, h, hd), 0.0, 1.5)
    dev = torch.from_numpy(qkv).cuda()
    q, k, v = (dev[:, :, i].permute(0, 2, 1, 3) for i in range(3))       # views [b, h, t, hd] of the projection output
    out = hip.attention(q, k, v, scale=scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    ref = oracle_chain(oracle, qkv, b, t, h, hd, scale).astype(np.float64)
    top = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-4 * top, f"{np.abs(got - ref).max():.3e} against {top:.3e}"
    assert np.all(np.abs(got - ref) <= 1e-4 * np.abs(ref) + 1e-5)
    # heads kept apart, operands as separate contiguous tensors
    out2 = hip.attention(q.contiguous(), k.contiguous(), v.contiguous(), scale=scale, merged_out=False)
    torch.cuda.synchronize()
    assert torch.equal(out2.permute(0, 2, 1, 3).reshape(b, t, h * hd), out)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("shape", [(64, 3, 197, 64, 0.125), (2, 3, 197, 64, 0.125), (1, 2, 40, 64, 1.0), (3, 1, 256, 64, 0.125),
                                   (1, 4, 129, 64, 0.25), (2, 2, 7, 64, 0.5)])
def test_attention_with_16_bit_operands(shape, dtype, torch_dev, oracle):
    """q, k, v and the result in bf16 / fp16: within 1e-2 of the oracle's fp32 operator chain on the same (rounded)
    operands, and within one and a half units in the last place of the 16-bit type (normalised) of a float64 model of what
    the kernel is specified to compute: exact scores and Softmax, probabilities rounded to the operand type, exact second
    product, one rounding of the result"""
    torch = torch_dev
    b, h, t, hd, scale = shape
    tdt = getattr(torch, dtype)
    print(f"attention {dtype} {shape}", flush=True)
    qkv = cases.datagen.normal(cases.datagen.seed_for("attn16", *shape[:4]), (b, t, 3, h, hd), 0.0, 1.0)
    dev = torch.from_numpy(qkv).cuda().to(tdt)
    rounded = dev.float().cpu().numpy()
    q, k, v = (dev[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    out = hip.attention(q, k, v, scale=scale)
    torch.cuda.synchronize()
    assert out.dtype == tdt
    got = out.float().cpu().numpy().astype(np.float64)
    ref = oracle_chain(oracle, rounded, b, t, h, hd, scale).astype(np.float64)
    top = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-2 * top, f"{np.abs(got - ref).max():.3e} against {top:.3e}"
    # the float64 model
    x = rounded.astype(np.float64).transpose(0, 2, 3, 1, 4)                      # [b, 3, h, t, hd]
    qq, kk, vv = x[:, 0], x[:, 1], x[:, 2]
    sc = np.einsum("bhqd,bhkd->bhqk", qq, kk) * scale
    pr = np.exp(sc - sc.max(-1, keepdims=True))
    pr = pr / pr.sum(-1, keepdims=True)
    pr16 = torch.from_numpy(pr).to(tdt).double().numpy()
    model = np.einsum("bhqk,bhkd->bhqd", pr16, vv).transpose(0, 2, 1, 3).reshape(b, t, h * hd)
    ulp = 2.0 ** -8 if dtype == "bfloat16" else 2.0 ** -11
    assert np.abs(got - model).max() <= 1.5 * ulp * top + 1e-6, f"{np.abs(got - model).max():.3e} against {ulp * top:.3e}"


def test_attention_rows_are_probabilities(torch_dev):
    """v = identity columns: the output is the Softmax itself; rows sum to one, and large scores do not overflow"""
    torch = torch_dev
    t, hd = 64, 64
    q = torch.randn((1, 1, t, hd), generator=torch.Generator().manual_seed(5)).cuda() * 30.0
    k = torch.randn((1, 1, t, hd), generator=torch.Generator().manual_seed(6)).cuda()
    v = torch.eye(t, hd, device="cuda").reshape(1, 1, t, hd).contiguous()
    p = hip.attention(q, k, v, merged_out=False)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(p).all()) and bool((p >= 0).all())
    assert torch.allclose(p.sum(-1), torch.ones(1, 1, t, device="cuda"), atol=1e-5)


def test_attention_refuses_what_it_does_not_fuse(torch_dev):
    torch = torch_dev
    z = lambda *s: torch.zeros(s, device="cuda")
    with pytest.raises(hip.OnhipError, match="head dimension 48"):
        hip.attention(z(1, 1, 8, 48), z(1, 1, 8, 48), z(1, 1, 8, 48))
    with pytest.raises(hip.OnhipError, match="at most 256"):
        hip.attention(z(1, 1, 257, 64), z(1, 1, 257, 64), z(1, 1, 257, 64))
    with pytest.raises(hip.OnhipError, match="multiples of 4"):
        base = z(1, 1, 8, 66)
        hip.attention(base[..., :64], z(1, 1, 8, 64), z(1, 1, 8, 64))


@pytest.mark.parametrize("flags", [(0, 0, 0, 0), (1, 1, 1, 1), (0, 1, 0, 1)])
def test_plugin_eval_attention_host_buffers(flags, torch_dev, oracle):
    """the MatMul plugin's eval_attention on tensors in host memory, with and without the layout flags that say a tensor
    is stored [batch, tokens, heads, head_dim] (the far side of a head-split / head-merge Transpose): 1e-4 against the
    oracle's chain Transpose -> MatMul -> Softmax -> MatMul"""
    from onenew_amd import ops
    b, h, t, hd = 2, 3, 50, 64
    g = cases.datagen
    q, k, v = (g.normal(g.seed_for("plug_attn", n, *flags), (b, h, t, hd), 0.0, 0.5) for n in "qkv")
    kt = oracle.transpose_f32(k, (0, 1, 3, 2))
    p = oracle.softmax_f32(oracle.matmul_f32(q.reshape(b * h, t, hd), kt.reshape(b * h, hd, t)))
    ref = oracle.matmul_f32(p, v.reshape(b * h, t, hd)).reshape(b, h, t, hd)
    given = [np.ascontiguousarray(x.transpose(0, 2, 1, 3)) if f else x for x, f in zip((q, k, v), flags)]
    op = ops.MatMulFused(ops.Plugin(hip.plugin_path("MatMul")))
    got = op.attention(*given, token_major=flags)
    if flags[3]:
        got = got.transpose(0, 2, 1, 3)
    assert got.shape == ref.shape
    assert np.abs(got.astype(np.float64) - ref).max() <= 1e-4 * np.abs(ref).max()


def test_plugin_eval_attention_result_does_not_share_a_staging_buffer_with_v(torch_dev, oracle):
    """host buffers, the result token-major and v head-major, many heads and tokens: the result of one head is written while
    v of the next is still being read, so the two must not sit in one staging buffer (they once did: now and then wrong)"""
    from onenew_amd import ops
    b, h, t, hd = 3, 6, 200, 64
    g = cases.datagen
    q, k, v = (g.normal(g.seed_for("plug_attn_big", n), (b, h, t, hd), 0.0, 0.5) for n in "qkv")
    kt = oracle.transpose_f32(k, (0, 1, 3, 2))
    p = oracle.softmax_f32(oracle.matmul_f32(q.reshape(b * h, t, hd), kt.reshape(b * h, hd, t)))
    ref = oracle.matmul_f32(p, v.reshape(b * h, t, hd)).reshape(b, h, t, hd)
    op = ops.MatMulFused(ops.Plugin(hip.plugin_path("MatMul")))
    for _ in range(3):
        got = op.attention(q, k, v, token_major=(0, 0, 0, 1)).transpose(0, 2, 1, 3)
        assert np.abs(got.astype(np.float64) - ref).max() <= 1e-4 * np.abs(ref).max()
