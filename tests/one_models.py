"""Small .one models for the runtime tests: every operator of the package, initialisers in each position the
reference host handles, views, two inputs and two outputs.  Weights and inputs are seeded."""
import numpy as np

from onenew_amd import abi, onefile, datagen


def _r(tag, shape, scale=1.0):
    return (datagen.normal(datagen.seed_for("one_models", tag), shape, 0.0, 1.0) * np.float32(scale)).astype(np.float32)


def resnet_block():
    """conv+relu, conv, residual add, relu, maxpool, strided 1x1, global pool, flatten, gemm"""
    m = onefile.OneModel()
    m.input("x", (1, 16, 20, 20))
    m.conv("c1", "x", _r("c1w", (16, 16, 3, 3), 0.08), _r("c1b", (16,), 0.1), "c1_out", pad=1, act=abi.RELU)
    m.conv("c2", "c1_out", _r("c2w", (16, 16, 3, 3), 0.08), _r("c2b", (16,), 0.1), "c2_out", pad=1)
    m.add("res", "c2_out", "x", "res_out")
    m.relu("relu", "res_out", "relu_out")
    m.maxpool("pool", "relu_out", "pool_out", 3, 2, 1)
    m.conv("down", "pool_out", _r("dw", (40, 16, 1, 1), 0.2), None, "down_out", stride=2)
    m.global_avgpool("gap", "down_out", "gap_out")
    m.flatten("flat", "gap_out", "flat_out", axis=1)
    m.gemm("fc", "flat_out", _r("fcw", (10, 40), 0.15), _r("fcb", (10,), 0.1), "logits")
    m.output("logits", (1, 10))
    return m.tobytes(), [_r("x", (1, 16, 20, 20))]


def mobile_block():
    """pointwise + CLIP, depthwise + CLIP, pointwise, SiLU conv: the fused activations and group != 1"""
    m = onefile.OneModel()
    m.input("x", (1, 8, 14, 14))
    m.conv("expand", "x", _r("ew", (24, 8, 1, 1), 0.3), _r("eb", (24,), 0.1), "e", act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("dw", "e", _r("dww", (24, 1, 3, 3), 0.3), _r("dwb", (24,), 0.1), "d", stride=2, pad=1, group=24,
           act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("project", "d", _r("pw", (12, 24, 1, 1), 0.2), _r("pb", (12,), 0.1), "p")
    m.conv("silu", "p", _r("sw", (12, 12, 3, 3), 0.1), _r("sb", (12,), 0.1), "out", pad=1, act=abi.SILU)
    m.output("out", (1, 12, 7, 7))
    return m.tobytes(), [_r("xm", (1, 8, 14, 14))]


def inverted_residual_blocks(batch=8, size=32):
    """two MobileNetV2-style blocks on a plane large enough for the one-launch block kernel to be recommended at this batch:
    1x1 expansion + CLIP, depthwise 3x3 + CLIP (stride 1, then 2), linear 1x1 projection; the first with the skip connection"""
    m = onefile.OneModel()
    m.input("x", (batch, 16, size, size))
    m.conv("e1", "x", _r("e1w", (64, 16, 1, 1), 0.3), _r("e1b", (64,), 0.3), "e1_out", act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("d1", "e1_out", _r("d1w", (64, 1, 3, 3), 0.3), _r("d1b", (64,), 0.1), "d1_out", pad=1, group=64, act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("p1", "d1_out", _r("p1w", (16, 64, 1, 1), 0.15), _r("p1b", (16,), 0.1), "p1_out")
    m.add("skip", "p1_out", "x", "b1_out")
    m.conv("e2", "b1_out", _r("e2w", (96, 16, 1, 1), 0.3), _r("e2b", (96,), 0.3), "e2_out", act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("d2", "e2_out", _r("d2w", (96, 1, 3, 3), 0.3), _r("d2b", (96,), 0.1), "d2_out", stride=2, pad=1, group=96, act=abi.CLIP,
           clip=(0.0, 6.0))
    m.conv("p2", "d2_out", _r("p2w", (24, 96, 1, 1), 0.1), None, "out")
    m.output("out", (batch, 24, size // 2, size // 2))
    m.output("b1_out", (batch, 16, size, size))
    return m.tobytes(), [_r("xir", (batch, 16, size, size))]


def bottleneck_pairs(batch=16, size=32):
    """two ResNet-style bottlenecks with 16 channels inside, on a plane large enough at this batch for the library to
    recommend the 3x3 convolution and the 1x1 after it as one launch: the first with a projection on the skip path (which
    comes before the last convolution in the file, as in ResNet-50, so the Add is folded into the projection and the pair
    has none), the second with the identity skip (the pair takes the Add and the Relu)"""
    m = onefile.OneModel()
    m.input("x", (batch, 32, size, size))
    m.conv("c1", "x", _r("bp_c1w", (16, 32, 1, 1), 0.25), _r("bp_c1b", (16,), 0.2), "c1_out", act=abi.RELU)
    m.conv("c2", "c1_out", _r("bp_c2w", (16, 16, 3, 3), 0.12), _r("bp_c2b", (16,), 0.2), "c2_out", pad=1, act=abi.RELU)
    m.conv("dn", "x", _r("bp_dnw", (64, 32, 1, 1), 0.2), _r("bp_dnb", (64,), 0.1), "dn_out")
    m.conv("c3", "c2_out", _r("bp_c3w", (64, 16, 1, 1), 0.2), _r("bp_c3b", (64,), 0.1), "c3_out")
    m.add("add1", "c3_out", "dn_out", "add1_out")
    m.relu("relu1", "add1_out", "r1")
    m.conv("c4", "r1", _r("bp_c4w", (16, 64, 1, 1), 0.2), _r("bp_c4b", (16,), 0.2), "c4_out", act=abi.RELU)
    m.conv("c5", "c4_out", _r("bp_c5w", (16, 16, 3, 3), 0.12), _r("bp_c5b", (16,), 0.2), "c5_out", pad=1, act=abi.RELU)
    m.conv("c6", "c5_out", _r("bp_c6w", (64, 16, 1, 1), 0.2), _r("bp_c6b", (64,), 0.1), "c6_out")
    m.add("add2", "c6_out", "r1", "add2_out")
    m.relu("relu2", "add2_out", "out")
    m.output("out", (batch, 64, size, size))
    m.output("r1", (batch, 64, size, size))
    return m.tobytes(), [_r("xbp", (batch, 32, size, size))]


def separable_chain(batch=16, size=32, ch=32):
    """a depthwise-separable stack pw -> dw -> pw -> dw -> pw (MobileNetV1 style, at most 64 channels): the last 1x1 of the
    first triple is also the first 1x1 of the next, so one-launch blocks must not overlap"""
    m = onefile.OneModel()
    m.input("x", (batch, 16, size, size))
    act = dict(act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("pw1", "x", _r("s_pw1w", (ch, 16, 1, 1), 0.3), _r("s_pw1b", (ch,), 0.3), "pw1_out", **act)
    m.conv("dw1", "pw1_out", _r("s_dw1w", (ch, 1, 3, 3), 0.3), _r("s_dw1b", (ch,), 0.1), "dw1_out", pad=1, group=ch, **act)
    m.conv("pw2", "dw1_out", _r("s_pw2w", (ch, ch, 1, 1), 0.2), _r("s_pw2b", (ch,), 0.2), "pw2_out", **act)
    m.conv("dw2", "pw2_out", _r("s_dw2w", (ch, 1, 3, 3), 0.3), _r("s_dw2b", (ch,), 0.1), "dw2_out", pad=1, group=ch, **act)
    m.conv("pw3", "dw2_out", _r("s_pw3w", (24, ch, 1, 1), 0.2), _r("s_pw3b", (24,), 0.1), "out")
    m.output("out", (batch, 24, size, size))
    return m.tobytes(), [_r("xsep", (batch, 16, size, size))]


def block_with_inner_skip(batch=16, size=32, ch=32):
    """1x1 -> depthwise -> 1x1 whose result is added to the FIRST convolution's result: that operand has a second reader
    (the Add folded into the last convolution), so the triple must stay three operators"""
    m = onefile.OneModel()
    m.input("x", (batch, 16, size, size))
    act = dict(act=abi.CLIP, clip=(0.0, 6.0))
    m.conv("a", "x", _r("k_aw", (ch, 16, 1, 1), 0.3), _r("k_ab", (ch,), 0.3), "a_out", **act)
    m.conv("b", "a_out", _r("k_bw", (ch, 1, 3, 3), 0.3), _r("k_bb", (ch,), 0.1), "b_out", pad=1, group=ch, **act)
    m.conv("c", "b_out", _r("k_cw", (ch, ch, 1, 1), 0.2), _r("k_cb", (ch,), 0.2), "c_out")
    m.add("skip", "c_out", "a_out", "out")
    m.output("out", (batch, ch, size, size))
    return m.tobytes(), [_r("xskip", (batch, 16, size, size))]


def vit_block():
    """layer norm, projection with a weight initialiser and a bias Add, table GELU, residual, then a token-mixing
    pair of MatMuls over two activations with Transpose and Softmax, and a Reshape view"""
    t, c = 17, 32
    m = onefile.OneModel()
    m.input("x", (1, t, c))
    m.layernorm("ln1", "x", 1.0 + _r("g", (c,), 0.1), _r("b", (c,), 0.1), "ln1_out")
    m.matmul("fc1", "ln1_out", _r("w1", (c, 64), 0.2), "fc1_out")
    m.add("fc1_bias", "fc1_out", _r("b1", (64,), 0.1), "fc1_b")
    m.gelu("gelu", "fc1_b", "gelu_out")
    m.matmul("fc2", "gelu_out", _r("w2", (64, c), 0.2), "fc2_out")
    m.add("fc2_bias", "fc2_out", _r("b2", (c,), 0.1), "fc2_b")
    m.add("res", "fc2_b", "x", "h")
    m.reshape("heads", "h", "h4", (1, 1, t, c))
    m.transpose("kt", "h4", "h4_t", (0, 1, 3, 2))
    m.matmul("scores", "h4", "h4_t", "scores_out")
    m.softmax("attn", "scores_out", "attn_out")
    m.matmul("ctx", "attn_out", "h4", "ctx_out")
    m.output("ctx_out", (1, 1, t, c))
    m.output("h", (1, t, c))
    return m.tobytes(), [_r("xv", (1, t, c))]


def two_inputs():
    """two net inputs, an Add of them, a channel Softmax (axis 1) and an axis-1 layer norm"""
    m = onefile.OneModel()
    m.input("a", (1, 6, 5, 5))
    m.input("b", (1, 6, 5, 5))
    m.add("sum", "a", "b", "s")
    m.softmax("sm", "s", "sm_out", axis=1)
    m.output("sm_out", (1, 6, 5, 5))
    m.relu("r", "s", "r_out")
    m.output("r_out", (1, 6, 5, 5))
    return m.tobytes(), [_r("a", (1, 6, 5, 5)), _r("b", (1, 6, 5, 5))]


def quantised_block():
    """W8A32 convolutions as the offline quantiser leaves them (int8 weights, int32 bias, per-channel weight_aux,
    input_scale), dense with SiLU and RELU and one depthwise, between fp32 operators"""
    from oracle import oracle
    m = onefile.OneModel()
    m.input("x", (1, 16, 18, 18))

    def q(tag, shape, scale):
        w = _r(tag + "w", shape, scale)
        b = _r(tag + "b", (shape[0],), 0.2)
        return oracle.quant_weight_bias(w, b)

    w8, b32, aux = q("q1", (32, 16, 3, 3), 0.1)
    m.conv("q1", "x", w8, b32, "q1_out", pad=1, act=abi.SILU, quant=(aux, 0.031))
    w8, b32, aux = q("qd", (32, 1, 3, 3), 0.3)
    m.conv("qd", "q1_out", w8, b32, "qd_out", stride=2, pad=1, group=32, act=abi.RELU, quant=(aux, 0.024))
    w8, b32, aux = q("q2", (24, 32, 1, 1), 0.2)
    m.conv("q2", "qd_out", w8, b32, "q2_out", act=abi.NOT_ACT, quant=(aux, 0.017))
    m.relu("relu", "q2_out", "out")
    m.output("out", (1, 24, 9, 9))
    return m.tobytes(), [_r("xq", (1, 16, 18, 18))]


def quantised_chain(n=1, hw=18, different_scales=False, extra_reader=False, tail=False):
    """dense W8A32 convolutions feeding each other: q1 -> (q2, q2b with one input_scale) , q2 -> q3, and a residual
    block qa -> qb + skip -> Relu behind q3; the operands between them can travel as int8.  different_scales: q2b
    quantises its input differently from q2; extra_reader: a Relu also reads q1's result; tail: two more int8
    convolutions read the residual block's fp32 result (which stays an output)"""
    from oracle import oracle
    m = onefile.OneModel()
    m.input("x", (n, 16, hw, hw))

    def q(tag, shape, scale):
        w = _r(tag + "w", shape, scale)
        b = _r(tag + "b", (shape[0],), 0.2)
        return oracle.quant_weight_bias(w, b)

    w8, b32, aux = q("c1", (32, 16, 3, 3), 0.1)
    m.conv("q1", "x", w8, b32, "q1_out", pad=1, act=abi.SILU, quant=(aux, 0.031))
    w8, b32, aux = q("c2", (64, 32, 1, 1), 0.2)
    m.conv("q2", "q1_out", w8, b32, "q2_out", act=abi.RELU, quant=(aux, 0.024))
    w8, b32, aux = q("c2b", (24, 32, 3, 3), 0.1)
    m.conv("q2b", "q1_out", w8, b32, "q2b_out", stride=2, pad=1, act=abi.NOT_ACT, quant=(aux, 0.029 if different_scales else 0.024))
    m.relu("relu_b", "q2b_out", "out_b")
    oh = (hw + 2 - 3) // 2 + 1
    m.output("out_b", (n, 24, oh, oh))
    if extra_reader:
        m.relu("relu_x", "q1_out", "out_x")
        m.output("out_x", (n, 32, hw, hw))
    w8, b32, aux = q("c3", (32, 64, 3, 3), 0.08)
    m.conv("q3", "q2_out", w8, b32, "q3_out", pad=1, act=abi.NOT_ACT, quant=(aux, 0.04))
    # a residual block of int8 convolutions on q3's fp32 result
    w8, b32, aux = q("ca", (32, 32, 1, 1), 0.2)
    m.conv("qa", "q3_out", w8, b32, "qa_out", act=abi.RELU, quant=(aux, 0.06))
    w8, b32, aux = q("cb", (32, 32, 3, 3), 0.1)
    m.conv("qb", "qa_out", w8, b32, "qb_out", pad=1, act=abi.NOT_ACT, quant=(aux, 0.035))
    m.add("sum", "qb_out", "q3_out", "sum_out")
    m.relu("relu_s", "sum_out", "out")
    m.output("out", (n, 32, hw, hw))
    if tail:
        w8, b32, aux = q("ct", (48, 32, 3, 3), 0.1)
        m.conv("qt", "out", w8, b32, "out_t", pad=1, act=abi.RELU, quant=(aux, 0.045))
        m.output("out_t", (n, 48, hw, hw))
        w8, b32, aux = q("cu", (16, 32, 1, 1), 0.2)
        m.conv("qu", "out", w8, b32, "out_u", stride=2, act=abi.NOT_ACT, quant=(aux, 0.045))
        m.output("out_u", (n, 16, (hw - 1) // 2 + 1, (hw - 1) // 2 + 1))
    return m.tobytes(), [_r("xqc", (n, 16, hw, hw))]


def quantised_mobile(n=1, hw=24, scales_differ=False):
    """MobileNetV2 in small, every convolution W8A32: dense 3x3 stride-2 stem, a depthwise + projection pair, an expanding
    block with a stride-2 depthwise layer and one with the skip connection (its sum is read by an int8 convolution and is
    a net output), 5x5 depthwise in the last block.  Every operand between two convolutions can travel as int8, the
    depthwise ones included.  scales_differ: the second depthwise layer quantises its input with another scale than the
    expansion's other reader, so that operand stays fp32"""
    from oracle import oracle
    m = onefile.OneModel()
    m.input("x", (n, 3, hw, hw))
    clip = dict(act=abi.CLIP, clip=(0.0, 6.0))

    def q(tag, shape, scale):
        w = _r("qm_" + tag + "w", shape, scale)
        b = _r("qm_" + tag + "b", (shape[0],), 0.2)
        return oracle.quant_weight_bias(w, b)

    def cv(name, x, out, shape, wscale, in_scale, **kw):
        w8, b32, aux = q(name, shape, wscale)
        m.conv(name, x, w8, b32, out, quant=(aux, in_scale), **kw)

    h1 = (hw + 2 - 3) // 2 + 1
    cv("stem", "x", "stem_out", (20, 3, 3, 3), 0.3, 0.02, stride=2, pad=1, **clip)
    cv("dw0", "stem_out", "dw0_out", (20, 1, 3, 3), 0.3, 0.03, pad=1, group=20, **clip)
    cv("pw0", "dw0_out", "pw0_out", (16, 20, 1, 1), 0.2, 0.04)
    cv("e1", "pw0_out", "e1_out", (48, 16, 1, 1), 0.3, 0.05, **clip)
    cv("dw1", "e1_out", "dw1_out", (48, 1, 3, 3), 0.3, 0.035, stride=2, pad=1, group=48, **clip)
    if scales_differ:   # a second reader of the expansion with another input_scale: e1_out stays fp32
        cv("side", "e1_out", "side_out", (8, 48, 1, 1), 0.2, 0.05, act=abi.RELU)
        m.output("side_out", (n, 8, h1, h1))
    h2 = (h1 + 2 - 3) // 2 + 1
    cv("p1", "dw1_out", "p1_out", (24, 48, 1, 1), 0.2, 0.045)
    cv("e2", "p1_out", "e2_out", (72, 24, 1, 1), 0.3, 0.05, **clip)
    cv("dw2", "e2_out", "dw2_out", (72, 1, 3, 3), 0.3, 0.04, pad=1, group=72, **clip)
    cv("p2", "dw2_out", "p2_out", (24, 72, 1, 1), 0.2, 0.045)
    m.add("skip", "p2_out", "p1_out", "b2_out")
    m.output("b2_out", (n, 24, h2, h2))
    cv("e3", "b2_out", "e3_out", (40, 24, 1, 1), 0.3, 0.06, act=abi.SILU)
    cv("dw3", "e3_out", "dw3_out", (40, 1, 5, 5), 0.2, 0.03, pad=2, group=40, act=abi.RELU)
    cv("p3", "dw3_out", "out", (32, 40, 1, 1), 0.2, 0.05)
    m.output("out", (n, 32, h2, h2))
    return m.tobytes(), [_r("xqm", (n, 3, hw, hw))]


def quantised_stem(n=1, hw=21):
    """a quantised stem: dense int8 Conv (7x7 stride 2, Relu) -> MaxPool 3x3 stride 2 -> two dense int8 convolutions with
    one input_scale; the operands either side of the MaxPool can travel as int8"""
    from oracle import oracle
    m = onefile.OneModel()
    m.input("x", (n, 3, hw, hw))

    def q(tag, shape, scale):
        w = _r(tag + "w", shape, scale)
        b = _r(tag + "b", (shape[0],), 0.2)
        return oracle.quant_weight_bias(w, b)

    w8, b32, aux = q("s0", (24, 3, 7, 7), 0.1)
    m.conv("stem", "x", w8, b32, "stem_out", stride=2, pad=3, act=abi.RELU, quant=(aux, 0.02))
    h1 = (hw + 6 - 7) // 2 + 1
    m.maxpool("pool", "stem_out", "pool_out", 3, 2, 1)
    h2 = (h1 + 2 - 3) // 2 + 1
    w8, b32, aux = q("s1", (32, 24, 1, 1), 0.2)
    m.conv("c1", "pool_out", w8, b32, "out_a", act=abi.RELU, quant=(aux, 0.03))
    m.output("out_a", (n, 32, h2, h2))
    w8, b32, aux = q("s2", (16, 24, 3, 3), 0.1)
    m.conv("c2", "pool_out", w8, b32, "out_b", pad=1, act=abi.NOT_ACT, quant=(aux, 0.03))
    m.output("out_b", (n, 16, h2, h2))
    return m.tobytes(), [_r("xstem", (n, 3, hw, hw))]


def attention_heads(heads=3, tokens=40, head_dim=64, batch=2, scores_also_output=False, split_heads=()):
    """q, k, v as three inputs [batch, heads, tokens, head_dim]: Transpose of k, MatMul, Softmax, MatMul, the pattern the
    runtime runs as one attention call (unless the scores are also a net output).  split_heads: which of "q", "k", "v"
    arrive as [batch, tokens, heads, head_dim] and go through a head-split Transpose (0, 2, 1, 3) first, and whether the
    result ("o") goes through the head-merge Transpose afterwards."""
    m = onefile.OneModel()
    shape = (batch, heads, tokens, head_dim)
    flat = (batch, tokens, heads, head_dim)
    if split_heads:
        for n in ("q", "k", "v"):
            if n in split_heads:
                m.input(n + "_flat", flat)
                m.transpose(n + "_split", n + "_flat", n, (0, 2, 1, 3))
            else:
                m.input(n, shape)
        m.transpose("kt", "k", "k_t", (0, 1, 3, 2))
        m.matmul("scores", "q", "k_t", "scores_out")
        m.softmax("attn", "scores_out", "attn_out")
        m.matmul("ctx", "attn_out", "v", "ctx_out")
        if "o" in split_heads:
            m.transpose("merge", "ctx_out", "merged", (0, 2, 1, 3))
            m.output("merged", flat)
        else:
            m.output("ctx_out", shape)
        return m.tobytes(), [_r(n + str(tokens), flat if n in split_heads else shape, 0.5) for n in ("q", "k", "v")]
    for n in ("q", "k", "v"):
        m.input(n, shape)
    m.transpose("kt", "k", "k_t", (0, 1, 3, 2))
    m.matmul("scores", "q", "k_t", "scores_out")
    m.softmax("attn", "scores_out", "attn_out")
    m.matmul("ctx", "attn_out", "v", "ctx_out")
    m.output("ctx_out", shape)
    if scores_also_output:
        m.output("scores_out", (batch, heads, tokens, tokens))
    return m.tobytes(), [_r(n + str(tokens), shape, 0.5) for n in ("q", "k", "v")]


MODELS = {"quantised_block": quantised_block, "quantised_mobile": quantised_mobile, "quantised_chain": quantised_chain, "quantised_stem": quantised_stem, "resnet_block": resnet_block, "mobile_block": mobile_block, "vit_block": vit_block, "two_inputs": two_inputs}


def unfused_activations(optimised=False):
    """A file as the converter leaves it, before tools/optimize: every activation a node of its own after its Conv
    (Clip, LeakyRelu, Sigmoid and Mul, HardSigmoid and Mul, Relu).  optimised=True: the same model as the optimiser
    writes it, the activations in the convolutions' act_type (tools/optimize/op_fusion.hpp:47-192)."""
    m = onefile.OneModel()
    m.input("x", (2, 8, 12, 12))

    def cv(name, x, cin, cout, k, act, out, **kw):
        w, b = _r(name + "w", (cout, cin, k, k), 0.25), _r(name + "b", (cout,), 0.2)
        if optimised:
            return m.conv(name, x, w, b, out, pad=k // 2, act=act, **kw)
        return m.conv(name, x, w, b, name + "_raw", pad=k // 2)

    cv("c1", "x", 8, 16, 3, abi.CLIP, "a1", clip=(0.0, 6.0))
    if not optimised:
        m.clip("clip", "c1_raw", "a1", 0.0, 6.0)
    cv("c2", "a1", 16, 16, 1, abi.LEAKYRELU, "a2", leaky=0.1)
    if not optimised:
        m.leaky_relu("leaky", "c2_raw", "a2", 0.1)
    cv("c3", "a2", 16, 16, 3, abi.SILU, "a3")
    if not optimised:
        m.sigmoid("sig", "c3_raw", "c3_gate")
        m.mul("silu_mul", "c3_raw", "c3_gate", "a3")
    cv("c4", "a3", 16, 12, 3, abi.HARDSILU, "a4", hard=(0.2, 0.5))
    if not optimised:
        m.hard_sigmoid("hsig", "c4_raw", "c4_gate", 0.2, 0.5)
        m.mul("hsilu_mul", "c4_gate", "c4_raw", "a4")          # operands the other way round
    cv("c5", "a4", 12, 12, 1, abi.RELU, "out")
    if not optimised:
        m.relu("relu", "c5_raw", "out")
    m.output("out", (2, 12, 12, 12))
    return m.tobytes(), [_r("xu", (2, 8, 12, 12))]
