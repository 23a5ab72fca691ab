"""Pins the CPU oracle against what the mathematics fixes, independently of the reference build:
float64 brute force on small inputs, algebraic invariants, and the closed form of the W8A32 path."""
import numpy as np
import pytest

import cases
from onenew_amd import abi, datagen
from onenew_amd.abi import ConvDesc


def conv_f64(d, x, w, b):
    """textbook cross-correlation with zero padding, float64, dense or depthwise"""
    oh, ow = d.out_hw()
    xp = np.zeros((d.n, d.cin, d.h + d.pad_t + d.pad_b, d.w + d.pad_l + d.pad_r))
    xp[:, :, d.pad_t:d.pad_t + d.h, d.pad_l:d.pad_l + d.w] = x
    y = np.zeros((d.n, d.cout, oh, ow))
    w = w.astype(np.float64)
    for i in range(d.kh):
        for j in range(d.kw):
            patch = xp[:, :, i:i + (oh - 1) * d.stride_h + 1:d.stride_h, j:j + (ow - 1) * d.stride_w + 1:d.stride_w]
            if d.group == 1:
                y += np.einsum("nchw,mc->nmhw", patch, w[:, :, i, j])
            else:
                y += patch * w[:, 0, i, j][None, :, None, None]
    if b is not None:
        y += b.astype(np.float64)[None, :, None, None]
    return y


@pytest.mark.parametrize("name", ["c3x3_tiny_relu", "c1x1_unaligned_clip", "c7x7_s2_p3", "c1x1_s2", "c3x3_s2_asym_pad",
                                  "c5x5_p2_hardsilu", "c3x3_nobias", "dw3x3_s2_odd", "dw5x5_p2", "dw3x3_p0", "c1x1_pad1"])
def test_conv_matches_float64_closed_form(name, oracle):
    d = ConvDesc.from_buffer_copy(cases.conv_f32_cases()[name])
    d.n = 2
    x, w, b = cases.conv_inputs(name + "_f64", d)
    y = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    ref = conv_f64(d, x, w, b)
    if d.has_bias:
        if d.act_type == abi.RELU:
            ref = np.maximum(ref, 0)
        elif d.act_type == abi.CLIP:
            ref = np.clip(ref, d.clip_min, d.clip_max)
        elif d.act_type == abi.LEAKYRELU:
            ref = np.where(ref > 0, ref, d.leaky_relu_alpha * ref)
        elif d.act_type == abi.HARDSILU:
            ref = ref * np.clip(d.hard_sigmoid_alpha * ref + d.hard_sigmoid_beta, 0, 1)
    assert np.abs(y - ref).max() <= 2e-6 * max(1.0, np.abs(ref).max())


def test_conv_invariants(oracle):
    d = cases.cd(6, 10, 3, 1, 1, 9, act=abi.NOT_ACT)
    x, w, b = cases.conv_inputs("inv", d)
    y = oracle.conv2d_f32(d, x, w, b)
    # zero input -> bias
    y0 = oracle.conv2d_f32(d, np.zeros_like(x), w, b)
    assert np.array_equal(y0, np.broadcast_to(b.reshape(1, -1, 1, 1), y0.shape))
    # linearity in x (up to rounding)
    y2 = oracle.conv2d_f32(d, 2 * x, w, b)
    assert np.allclose(y2 - b.reshape(1, -1, 1, 1), 2 * (y - b.reshape(1, -1, 1, 1)), atol=1e-6)
    # stride-2 output = subsampled stride-1 output (same padding)
    d2 = cases.cd(6, 10, 3, 2, 1, 9, act=abi.NOT_ACT)
    assert np.array_equal(oracle.conv2d_f32(d2, x, w, b), y[:, :, ::2, ::2])
    # 1x1 convolution == MatMul of the weight matrix with the [C, H*W] image, plus bias: same rounding chain
    d1 = cases.cd(6, 10, 1, 1, 0, 9, act=abi.NOT_ACT)
    w1 = w[:, :, 1:2, 1:2].copy()
    y1 = oracle.conv2d_f32(d1, x, w1, b)
    mm = oracle.matmul_f32(w1.reshape(10, 6), x.reshape(6, 81)) + b.reshape(-1, 1)
    assert np.array_equal(y1.reshape(10, 81), mm.astype(np.float32))
    # batch B = B independent batch-1 evaluations
    d3 = ConvDesc.from_buffer_copy(d)
    d3.n = 3
    xb = np.concatenate([x, 2 * x, -x])
    yb = oracle.conv2d_f32(d3, xb, w, b)
    assert np.array_equal(yb[1:2], y2) and np.array_equal(yb[0:1], y)


def test_depthwise_equals_grouped_dense(oracle):
    """a depthwise convolution is the dense one with a block-diagonal weight"""
    dd = cases.cd(5, 5, 3, 1, 1, 8, group=5, act=abi.NOT_ACT)
    x, w, b = cases.conv_inputs("dwdense", dd)
    wd = np.zeros((5, 5, 3, 3), np.float32)
    for c in range(5):
        wd[c, c] = w[c, 0]
    dn = cases.cd(5, 5, 3, 1, 1, 8, act=abi.NOT_ACT)
    assert np.allclose(oracle.conv2d_f32(dd, x, w, b), oracle.conv2d_f32(dn, x, wd, b), atol=1e-6)


def test_matmul_and_gemm_closed_forms(oracle):
    a = datagen.normal(1, (3, 7, 11))
    b = datagen.normal(2, (11, 5))
    assert np.allclose(oracle.matmul_f32(a, b), a.astype(np.float64) @ b.astype(np.float64), atol=1e-5)
    bb = datagen.normal(3, (3, 11, 5))
    assert np.allclose(oracle.matmul_f32(a, bb), np.einsum("bmk,bkn->bmn", a.astype(np.float64), bb.astype(np.float64)), atol=1e-5)
    w = datagen.normal(4, (9, 11))
    bias = datagen.normal(5, (9,))
    assert np.allclose(oracle.gemm_f32(a[0], w, bias), a[0].astype(np.float64) @ w.astype(np.float64).T + bias, atol=1e-5)
    # Gemm is MatMul against the transposed weight plus bias, with the same rounding chain
    assert np.array_equal(oracle.gemm_f32(a[0], w, bias), (oracle.matmul_f32(a[0], np.ascontiguousarray(w.T)) + bias).astype(np.float32))


def test_w8a32_closed_form_and_special_cases(oracle):
    """the integer path restated in numpy: quantise (ties away from zero, saturating), exact int32 sum,
    three separately rounded fp32 operations"""
    d = cases.cd(6, 4, 3, 1, 1, 7, act=abi.NOT_ACT, input_scale=0.05)
    x, w8, b32, aux = cases.conv_inputs("q_closed", d, quant=True)
    x = x * np.float32(8.0)          # |x / s| up to 160: exercises saturation at -128 / 127
    x.reshape(-1)[:8] = np.array([0.025, -0.025, 0.075, -0.075, 6.35, 6.375, -6.4, -6.425], np.float32)  # ties, edges
    y, acc = oracle.conv2d_w8a32(d, x, w8, b32, aux, want_acc=True)
    r = np.float32(1.0) / np.float32(0.05)
    t = np.clip(x * r, np.float32(-128), np.float32(127))
    q = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int64)      # roundf
    assert q.min() == -128 and q.max() == 127
    assert np.array_equal(oracle.quantize_s8(x, 0.05).astype(np.int64), q)
    qp = np.zeros((1, 6, 9, 9), np.int64)
    qp[:, :, 1:8, 1:8] = q
    ref_acc = np.zeros((1, 4, 7, 7), np.int64)
    for i in range(3):
        for j in range(3):
            ref_acc += np.einsum("nchw,mc->nmhw", qp[:, :, i:i + 7, j:j + 7], w8[:, :, i, j].astype(np.int64))
    assert np.array_equal(acc.astype(np.int64), ref_acc)
    f = ref_acc.astype(np.float32) * np.float32(0.05)
    f = f + b32.astype(np.float32).reshape(1, -1, 1, 1)
    coeff = (aux / np.float32(127.0)).astype(np.float32).reshape(1, -1, 1, 1)
    assert np.array_equal(y, (f * coeff).astype(np.float32))
    # re-quantised output is the consumer's quantisation of y
    d8 = ConvDesc.from_buffer_copy(d)
    d8.out_s8, d8.output_scale = 1, 0.7
    assert np.array_equal(oracle.conv2d_w8a32(d8, x, w8, b32, aux), oracle.quantize_s8(y, 0.7))
    # non-uniform padding is rejected (the reference pads all sides by pads[0])
    bad = cases.cd(6, 4, 3, 1, (1, 0, 1, 0), 7, input_scale=0.05)
    with pytest.raises(ValueError):
        oracle.conv2d_w8a32(bad, x, w8, b32, aux)


def test_weight_quantiser_truncates_toward_zero(oracle):
    """tools/optimize/model_quant.hpp:6-29: aux = max|w| per output channel, w8 = trunc(w * 127 / aux)"""
    w = datagen.normal(11, (5, 3, 3, 3), 0.0, 0.1)
    b = datagen.normal(12, (5,), 0.0, 0.05)
    w8, b32, aux = oracle.quant_weight_bias(w, b)
    assert np.array_equal(aux, np.abs(w).reshape(5, -1).max(axis=1))
    # "w * 127 / max": the product is rounded to float before the division
    a4 = aux.reshape(5, 1, 1, 1)
    assert np.array_equal(w8, np.trunc((w * np.float32(127.0)) / a4).astype(np.int8))
    assert np.array_equal(b32, np.trunc((b * np.float32(127.0)) / aux).astype(np.int32))
    assert np.abs(w8).max() == 127
    back = w8.astype(np.float32) * (aux / np.float32(127.0)).reshape(5, 1, 1, 1)
    assert np.all(np.abs(back) <= np.abs(w) + 1e-7) and np.abs(back - w).max() <= (aux / 127).max() + 1e-7


def test_table_activation_rule(oracle):
    lut = cases.silu_lut()
    x = np.array([-9.0, -8.0, -8.0 + 1 / 512, 0.0, 1.0, 8.0 - 1 / 512, 8.0, 9.5, 1.0 + 1 / 1024], np.float32)
    y = oracle.lut_act(x, lut)
    assert y[0] == 0.0 and y[1] == lut[0] and y[2] == lut[1] and y[3] == lut[4096] and y[4] == lut[4608]
    assert y[5] == lut[8191] and y[6] == 8.0 and y[7] == 9.5 and y[8] == lut[4608]      # truncation, not rounding
    xs = np.linspace(-8, 7.99, 1000).astype(np.float32)
    exact = xs / (1 + np.exp(-xs.astype(np.float64)))
    assert np.abs(oracle.lut_act(xs, lut) - exact).max() < 2.2e-3
    g = oracle.lut_act(xs, cases.gelu_lut())
    from math import erf
    gexact = np.array([0.5 * v * (1 + erf(v / 2 ** 0.5)) for v in xs.astype(np.float64)])
    assert np.abs(g - gexact).max() < 2.5e-3


def test_bf16_f16_rounding_helpers(oracle):
    x = np.array([1.0, 1.00390625, 1.005859375, 3.1415927, -2.7182817, 65504.0, 1e-3], np.float32)
    b = oracle.round_bf16(x)
    assert b[0] == 1.0 and b[1] == 1.0 and b[2] == 1.0078125      # ties to even on the 8-bit mantissa
    assert np.all((b.view(np.uint32) & 0xFFFF) == 0)
    h = oracle.round_f16(x)
    assert np.array_equal(h, x.astype(np.float16).astype(np.float32))


def _calib_data(seed, n):
    # a bell around zero with a few far outliers: the case clipping calibration exists for
    x = datagen.normal(seed, (n,), 1.0)
    x[::997] *= 9.0
    x[5::1231] = 0.0
    return x.astype(np.float32)


def test_calibration_histogram_and_max(oracle):
    """abs-max and the 2048-bin histogram against numpy; zeros are skipped, the top bin catches the maximum"""
    x = _calib_data(datagen.seed_for("calib", "x"), 200000)
    mx = oracle.calib_abs_max(x)
    assert mx == np.abs(x).max()
    assert oracle.calib_abs_max(x[:10], running=1e9) == np.float32(1e9)
    h = oracle.calib_histogram(x, mx)
    nz = np.abs(x[x != 0.0])
    idx = np.minimum((nz * np.float32(2048) * np.float32(1.0) / np.float32(mx)).astype(np.int32), 2047)
    assert np.array_equal(h, np.bincount(idx, minlength=2048).astype(np.float32))
    assert h.sum() == nz.size and h[2047] >= 1
    # a second call accumulates
    h2 = oracle.calib_histogram(x, mx, hist=h.copy())
    assert np.array_equal(h2, 2 * h)


def test_calibration_thresholds_closed_cases(oracle):
    """cases the definitions fix: (1) KL: a jagged distribution that lives in the first 128 bins is reproduced
    exactly by 128 levels over 128 bins and blurred by every wider clipping range (neighbouring bins merge),
    so the first candidate wins: threshold = 128.5 * max / 2048; (2) MSE: a single occupied
    bin b has squared error (b + 0.5 - level)^2 minimised over the candidates - brute-forced in float64;
    (3) thresholds scale linearly with max_abs; (4) outliers beyond the bulk are clipped: the KL threshold of a
    bell with far outliers lies well below the maximum"""
    h = np.zeros(2048, np.float32)
    h[:128] = datagen.integers(datagen.seed_for("calib", "jagged"), (128,), 1, 2000).astype(np.float32)
    t = oracle.calib_threshold("kl", h, int(h.sum()), 4.0)
    assert t == np.float32((128 + 0.5) * 4.0 / 2048)
    for b in (300, 1000, 2047):
        h = np.zeros(2048, np.float32)
        h[b] = 50.0
        losses = []
        for bins in range(128, 2048):
            step = np.float32(bins) / np.float32(127)
            level = min(np.floor((b + 0.5) / float(step) + 0.5), 127.0) * float(step)
            losses.append((b + 0.5 - level) ** 2)
        losses = np.array(losses)
        t = oracle.calib_threshold("mse", h, 50, 2.0)
        got_bins = round(t * 2048 / 2.0 - 0.5)
        # float32 rounding of the step decides between candidates that both sit within 1e-3 bin^2 of zero error
        assert losses[got_bins - 128] <= losses.min() + 1e-3, (b, got_bins, int(losses.argmin()) + 128)
    x = _calib_data(datagen.seed_for("calib", "thr"), 400000)
    mx = oracle.calib_abs_max(x)
    h = oracle.calib_histogram(x, mx)
    for method in ("kl", "mse"):
        t1 = oracle.calib_threshold(method, h, x.size, mx)
        t2 = oracle.calib_threshold(method, h, x.size, 2 * mx)
        assert t2 == 2 * t1
        assert 128.5 * mx / 2048 <= t1 <= mx
    assert oracle.calib_threshold("kl", h, x.size, mx) < 0.8 * mx


def _tailed_histogram(tag, n, tail_frac, tail_scale):
    """2048-bin histogram of a half-normal bulk with an exponential tail from 4 sigma outwards: the bulk fills a few
    hundred bins, the tail reaches the last one, so every candidate range leaves mass beyond itself"""
    x = np.abs(datagen.normal(datagen.seed_for("calib", tag, "bulk"), (n,), 0.0, 1.0).astype(np.float64))
    k = int(n * tail_frac)
    x[:k] = 4.0 - tail_scale * np.log(datagen.unit(datagen.seed_for("calib", tag, "tail"), k))
    idx = np.minimum((x * 2048 / x.max()).astype(np.int64), 2047)
    return np.bincount(idx, minlength=2048).astype(np.float32)


def _overlap(bins, shift_last=False):
    """W[i, j] = length of [i r, (i + 1) r) inside bin [j, j + 1), r = bins / 128: the 128 levels as intervals"""
    r = bins / 128.0
    i = np.arange(128)[:, None]
    j = np.arange(bins)[None, :]
    w = np.clip(np.minimum((i + 1) * r, j + 1.0) - np.maximum(i * r, j * 1.0), 0.0, None)
    if shift_last:          # the mistake of giving a level's last, fractional piece to the bin before it
        e = np.floor((np.arange(128) + 1) * r).astype(int)
        for lvl in range(127):
            if 0 < e[lvl] < bins and w[lvl, e[lvl]] > 0:
                w[lvl, e[lvl] - 1] += w[lvl, e[lvl]]
                w[lvl, e[lvl]] = 0.0
    return w


def _kl_curve_f64(h, n, fold=True, shift_last=False, eps=1e-7):
    """the entropy calibration as its definition reads, in float64, for every clipping range: P = the range's bins
    with everything beyond folded into the last one; Q = the same bins (not folded) averaged over 128 equal
    intervals and spread back over the bins by interval overlap; KL(P || Q)"""
    h = h.astype(np.float64)
    out = np.empty(2048 - 128)
    for bins in range(128, 2048):
        p = (eps + h[:bins]) / n
        P = p.copy()
        if fold:
            P[bins - 1] += h[bins:].sum() / n
        w = _overlap(bins, shift_last)
        q = (w @ p) / (bins / 128.0)
        Q = eps + w.T @ q
        out[bins - 128] = (P * np.log(P / Q)).sum()
    return out


def _mse_curve_f64(h, n, levels=128):
    """squared distance of every bin centre to the nearest of `levels` equidistant levels from 0 to the clipping
    point (centres beyond it are nearest to the top level), weighted by the histogram; float64"""
    h = h.astype(np.float64)
    c = np.arange(2048) + 0.5
    out = np.empty(2048 - 128)
    for bins in range(128, 2048):
        grid = np.arange(levels) * (bins / (levels - 1.0))
        d = np.abs(c[:, None] - grid[None, :]).min(axis=1)
        out[bins - 128] = (h * d * d).sum() / n
    return out


# histograms on which the winner of the float64 search stands clear of its runner-up by more than ten times the
# float32 rounding noise of the search under test
_TAILED = [("t1", 0.002, 3.0), ("t2", 0.0005, 6.0), ("t6", 0.02, 1.0), ("t4", 0.0001, 10.0)]
_TAILED_MSE = [("t1", 0.002, 3.0), ("t2", 0.0005, 6.0), ("t3", 0.01, 1.5), ("t7", 0.001, 4.0)]


@pytest.mark.parametrize("tag,frac,scale", _TAILED)
def test_kl_search_matches_float64_definition(oracle, tag, frac, scale):
    """the KL value of every one of the 1920 candidates against the float64 definition written with an
    interval-overlap matrix; the winner lies inside the range, is not a multiple of 128 (fractional level edges
    decide) and has mass beyond it (the fold into the last bin decides).  Two plausible mistakes - leaving the
    mass beyond the range out of P, giving a level's fractional last piece to the neighbouring bin - are shown to
    move the curve by orders of magnitude more than the tolerance, and the first also moves the winner."""
    h = _tailed_histogram(tag, 300000, frac, scale)
    n = int(h.sum())
    got = oracle.calib_curve("kl", h, n).astype(np.float64)
    want = _kl_curve_f64(h, n)
    tol = 2e-6 + 2e-5 * np.abs(want)
    assert np.all(np.abs(got - want) <= tol), float(np.abs(got - want).max())
    best = int(want.argmin()) + 128
    srt = np.sort(want)
    assert srt[1] - srt[0] > 10 * np.abs(got - want).max()          # the winner is decided beyond float32 noise
    assert int(got.argmin()) + 128 == best
    assert 128 < best < 2047 and best % 128 != 0 and h[best:].sum() > 0
    t = oracle.calib_threshold("kl", h, n, 6.5)
    assert t == np.float32(np.float32(best + 0.5) * np.float32(6.5) / np.float32(2048))
    nofold = _kl_curve_f64(h, n, fold=False)
    assert np.abs(nofold - want).max() > 1e3 * tol.max() and int(nofold.argmin()) + 128 != best
    shifted = _kl_curve_f64(h, n, shift_last=True)
    assert np.abs(shifted - want).max() > 1e2 * tol.max()


@pytest.mark.parametrize("tag,frac,scale", _TAILED_MSE)
def test_mse_search_matches_float64_definition(oracle, tag, frac, scale):
    """the loss of every candidate against nearest-level quantisation brute-forced in float64 over a histogram with
    hundreds of occupied bins; same winner, decided beyond float32 noise.  A 128-interval grid (step = range / 128
    instead of range / 127) is shown to fail the same comparison."""
    h = _tailed_histogram(tag, 300000, frac, scale)
    n = int(h.sum())
    got = oracle.calib_curve("mse", h, n).astype(np.float64)
    want = _mse_curve_f64(h, n)
    assert np.all(np.abs(got - want) <= 2e-5 * want), float((np.abs(got - want) / want).max())
    best = int(want.argmin()) + 128
    srt = np.sort(want)
    assert (srt[1] - srt[0]) / srt[0] > 10 * (np.abs(got - want) / want).max()
    assert int(got.argmin()) + 128 == best and 128 < best < 2047
    t = oracle.calib_threshold("mse", h, n, 3.25)
    assert t == np.float32(np.float32(best + 0.5) * np.float32(3.25) / np.float32(2048))
    wrong = _mse_curve_f64(h, n, levels=129)
    assert (np.abs(wrong - want) / want).max() > 1e-2


def test_calibration_percentile_rank(oracle):
    """the 99.998 % rule against a numpy sort: rank (1-p)*images*elems among the kept largest magnitudes"""
    images, elems = 3, 500000
    x = _calib_data(datagen.seed_for("calib", "pct"), images * elems)
    t = oracle.calib_percentile(x, images, elems)
    p = np.float32(99.998 / 100)
    keep = int(np.float32(elems) * (np.float32(1) - p) * 10)
    kept = np.concatenate([np.sort(np.abs(x[i * elems:(i + 1) * elems]))[::-1][:keep] for i in range(images)])
    rank = int((np.float32(1) - p) * images * elems)
    assert t == np.sort(kept)[::-1][rank]


def test_cheap_rounding_of_the_quantisers_is_roundf():
    """the device quantisers round with (int) (t + copysign(0.49999997, t)) instead of roundf: the same integer for every
    float the clamp lets through.  All ties k + 0.5, their float neighbours, the values around one half, and ten million
    random floats in [-128.5, 128.5]; the exhaustive check of all 2.2e9 floats in that range was run once in C."""
    half = np.float32(np.frombuffer(np.uint32(0x3EFFFFFF).tobytes(), np.float32)[0])
    assert half == np.nextafter(np.float32(0.5), np.float32(0))
    ties = (np.arange(-129, 129, dtype=np.float32) + np.float32(0.5))
    pts = np.concatenate([ties, np.nextafter(ties, np.float32(1e9)), np.nextafter(ties, np.float32(-1e9)),
                          np.arange(-129, 130, dtype=np.float32), np.array([0.0, -0.0, 1e-40, -1e-40, 0.49999997, -0.49999997], np.float32)])
    u = datagen.unit(datagen.seed_for("round", "t"), 10_000_000)
    pts = np.concatenate([pts, ((u - 0.5) * 257.0).astype(np.float32)])
    pts = pts[np.abs(pts) <= 128.5]
    cheap = np.trunc(pts + np.copysign(half, pts)).astype(np.int64)          # float32 addition, then truncation
    want = (np.sign(pts) * np.floor(np.abs(pts.astype(np.float64)) + 0.5)).astype(np.int64)   # round half away from zero
    assert np.array_equal(cheap, want)
