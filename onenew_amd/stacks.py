"""Layer-shape tables of the benchmark configurations (convolutions and matmuls at their real
shapes).  ResNet-50 follows the torchvision v1.5 layout that the reference's recorded trace
(tools/perf_profiling/timeline_info/resnet50.csv) confirms through its per-layer MFLOP counts."""
from .abi import ConvDesc, MatmulDesc, NOT_ACT, RELU, CLIP, SILU


def conv(name, cin, cout, k, s, p, hw, act=RELU, group=1, clip=(0.0, 6.0)):
    d = ConvDesc(n=1, cin=cin, h=hw, w=hw, cout=cout, kh=k, kw=k, stride_h=s, stride_w=s,
                 pad_t=p, pad_l=p, pad_b=p, pad_r=p, group=group, has_bias=1, act_type=act)
    if act == CLIP:
        d.clip_min, d.clip_max = clip
    return name, d


def resnet50(relu_everywhere=True):
    """53 convolutions; 8174.3 MFLOP per image.  The real graph fuses ReLU into 33 of them (stem,
    conv1, conv2); relu_everywhere=True applies it to all, as the benchmark configuration states."""
    L = [conv("stem", 3, 64, 7, 2, 3, 224)]
    lin = RELU if relu_everywhere else NOT_ACT
    inplanes, hw = 64, 56
    for li, (planes, blocks, stride) in enumerate([(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)], 1):
        for b in range(blocks):
            s = stride if b == 0 else 1
            p = f"l{li}.{b}"
            L.append(conv(p + ".conv1", inplanes, planes, 1, 1, 0, hw))
            L.append(conv(p + ".conv2", planes, planes, 3, s, 1, hw))
            if b == 0:
                L.append(conv(p + ".down", inplanes, planes * 4, 1, s, 0, hw, act=lin))
            hw //= s
            L.append(conv(p + ".conv3", planes, planes * 4, 1, 1, 0, hw, act=lin))
            inplanes = planes * 4
    return L


def mobilenet_v2():
    """52 convolutions, 17 of them depthwise 3x3 pad 1; ReLU6 arrives as CLIP(0, 6)."""
    L = [conv("stem", 3, 32, 3, 2, 1, 224, act=CLIP)]
    cin, hw = 32, 112
    cfg = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]
    bi = 0
    for t, c, n, s in cfg:
        for i in range(n):
            bi += 1
            stride = s if i == 0 else 1
            hidden = cin * t
            if t != 1:
                L.append(conv(f"b{bi}.expand", cin, hidden, 1, 1, 0, hw, act=CLIP))
            L.append(conv(f"b{bi}.dw", hidden, hidden, 3, stride, 1, hw, act=CLIP, group=hidden))
            hw //= stride
            L.append(conv(f"b{bi}.project", hidden, c, 1, 1, 0, hw, act=NOT_ACT))
            cin = c
    L.append(conv("last", 320, 1280, 1, 1, 0, 7, act=CLIP))
    return L


def vit_tiny(batch=1):
    """MatMuls of one ViT-Tiny/16 block at 197 tokens, dim 192, 3 heads x 64.
    Returns (name, MatmulDesc, has_bias, gelu)."""
    T, D, H = 197, 192, 3
    return [
        ("qkv", MatmulDesc(batch=batch, m=T, k=D, n=3 * D, b_shared=1), False, False),
        ("scores", MatmulDesc(batch=batch * H, m=T, k=D // H, n=T, b_shared=0), False, False),
        ("context", MatmulDesc(batch=batch * H, m=T, k=T, n=D // H, b_shared=0), False, False),
        ("proj", MatmulDesc(batch=batch, m=T, k=D, n=D, b_shared=1), False, False),
        ("fc1", MatmulDesc(batch=batch, m=T, k=D, n=4 * D, b_shared=1), True, True),
        ("fc2", MatmulDesc(batch=batch, m=T, k=4 * D, n=D, b_shared=1), True, False),
    ]


def yolov8s():
    """Convolutions of YOLOv8s at 640x640 (public ultralytics yolov8.yaml, scale s: widths
    32/64/128/256/512, depth 1/2/2/1 bottlenecks).  SiLU everywhere except the final 1x1
    predictors.  The reference ships no YOLO graph; this list restates the public definition."""
    L = []

    def cv(name, cin, cout, k, s, hw, act=SILU):
        L.append(conv(name, cin, cout, k, s, k // 2, hw, act=act))

    def c2f(name, cin, cout, n, hw):
        c = cout // 2
        cv(name + ".cv1", cin, cout, 1, 1, hw)
        for i in range(n):
            cv(f"{name}.m{i}.cv1", c, c, 3, 1, hw)
            cv(f"{name}.m{i}.cv2", c, c, 3, 1, hw)
        cv(name + ".cv2", (2 + n) * c, cout, 1, 1, hw)

    cv("b0", 3, 32, 3, 2, 640)
    cv("b1", 32, 64, 3, 2, 320)
    c2f("b2", 64, 64, 1, 160)
    cv("b3", 64, 128, 3, 2, 160)
    c2f("b4", 128, 128, 2, 80)
    cv("b5", 128, 256, 3, 2, 80)
    c2f("b6", 256, 256, 2, 40)
    cv("b7", 256, 512, 3, 2, 40)
    c2f("b8", 512, 512, 1, 20)
    cv("sppf.cv1", 512, 256, 1, 1, 20)
    cv("sppf.cv2", 1024, 512, 1, 1, 20)
    c2f("n12", 768, 256, 1, 40)
    c2f("n15", 384, 128, 1, 80)
    cv("n16", 128, 128, 3, 2, 80)
    c2f("n18", 384, 256, 1, 40)
    cv("n19", 256, 256, 3, 2, 40)
    c2f("n21", 768, 512, 1, 20)
    for c, hw in ((128, 80), (256, 40), (512, 20)):
        cv(f"det{hw}.box0", c, 64, 3, 1, hw)
        cv(f"det{hw}.box1", 64, 64, 3, 1, hw)
        cv(f"det{hw}.box2", 64, 64, 1, 1, hw, act=NOT_ACT)
        cv(f"det{hw}.cls0", c, 128, 3, 1, hw)
        cv(f"det{hw}.cls1", 128, 128, 3, 1, hw)
        cv(f"det{hw}.cls2", 128, 80, 1, 1, hw, act=NOT_ACT)
    return L


def with_batch(layers, n):
    out = []
    for name, d in layers:
        e = ConvDesc.from_buffer_copy(d)
        e.n = n
        out.append((name, e))
    return out


def resnet50_model(batch=1, classes=1000, tag="resnet50_model"):
    """The whole ResNet-50 as a .one file, in the form the offline optimiser leaves it: batch norm folded into the
    convolutions, ReLU fused into stem / conv1 / conv2 (33 of the 53), the residual Add and its ReLU as nodes of
    their own, MaxPool 3x3 s2 after the stem, GlobalAveragePool, Flatten, Gemm.  Seeded He-scaled weights.
    Returns (bytes, input shape, multiply-accumulates x 2 per inference)."""
    import numpy as np
    from . import datagen, onefile

    def weights(name, shape, fan_in):
        return datagen.normal(datagen.seed_for(tag, name), shape, 0.0, float(np.sqrt(2.0 / fan_in)))

    m = onefile.OneModel()
    flops = 0

    def cv(name, x, cin, cout, k, s, p, hw, act, gain=1.0):
        nonlocal flops
        out_hw = (hw + 2 * p - k) // s + 1
        flops += 2 * batch * cout * out_hw * out_hw * cin * k * k
        w = weights(name + ".w", (cout, cin, k, k), cin * k * k) * gain   # the residual branch is damped: no batch norm here
        b = datagen.normal(datagen.seed_for(tag, name + ".b"), (cout,), 0.0, 0.01)
        return m.conv(name, x, w, b, name + "_out", stride=s, pad=p, act=act)

    x = m.input("input", (batch, 3, 224, 224))
    x = cv("stem", x, 3, 64, 7, 2, 3, 224, RELU)
    x = m.maxpool("maxpool", x, "maxpool_out", 3, 2, 1)
    inplanes, hw = 64, 56
    for li, (planes, blocks, stride) in enumerate([(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)], 1):
        for b in range(blocks):
            s = stride if b == 0 else 1
            p = f"l{li}.{b}"
            y = cv(p + ".conv1", x, inplanes, planes, 1, 1, 0, hw, RELU)
            y = cv(p + ".conv2", y, planes, planes, 3, s, 1, hw, RELU)
            skip = cv(p + ".down", x, inplanes, planes * 4, 1, s, 0, hw, NOT_ACT) if b == 0 else x
            hw //= s
            y = cv(p + ".conv3", y, planes, planes * 4, 1, 1, 0, hw, NOT_ACT, gain=0.3)
            y = m.add(p + ".add", y, skip, p + ".add_out")
            x = m.relu(p + ".relu", y, p + ".relu_out")
            inplanes = planes * 4
    x = m.global_avgpool("avgpool", x, "avgpool_out")
    x = m.flatten("flatten", x, "flatten_out", axis=1)
    flops += 2 * batch * classes * inplanes
    x = m.gemm("fc", x, weights("fc.w", (classes, inplanes), inplanes) * 0.5,
               datagen.normal(datagen.seed_for(tag, "fc.b"), (classes,), 0.0, 0.01), "logits")
    m.output("logits", (batch, classes))
    return m.tobytes(), (batch, 3, 224, 224), flops


def mobilenet_v2_model(batch=1, classes=1000, tag="mobilenetv2_model"):
    """The whole MobileNetV2 as a .one file in its optimised form: batch norm folded, ReLU6 fused as CLIP(0, 6) into
    the stem, the expand and the depthwise convolutions, linear projections, residual Adds where stride is 1 and
    the width does not change, the last 1x1 convolution, GlobalAveragePool, Flatten, Gemm.  Seeded weights.
    Returns (bytes, input shape, multiply-accumulates x 2 per inference)."""
    import numpy as np
    from . import datagen, onefile

    m = onefile.OneModel()
    flops = 0

    def cv(name, x, cin, cout, k, s, hw, act, group=1, gain=1.0):
        nonlocal flops
        p = k // 2
        out_hw = (hw + 2 * p - k) // s + 1
        kc = cin if group == 1 else 1
        flops += 2 * batch * cout * out_hw * out_hw * kc * k * k
        w = datagen.normal(datagen.seed_for(tag, name + ".w"), (cout, kc, k, k), 0.0, float(np.sqrt(2.0 / (kc * k * k)))) * gain
        b = datagen.normal(datagen.seed_for(tag, name + ".b"), (cout,), 0.0, 0.01)
        return m.conv(name, x, w, b, name + "_out", stride=s, pad=p, group=group, act=act, clip=(0.0, 6.0))

    x = m.input("input", (batch, 3, 224, 224))
    x = cv("stem", x, 3, 32, 3, 2, 224, CLIP)
    cin, hw, bi = 32, 112, 0
    for t, c, n, s in [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]:
        for i in range(n):
            bi += 1
            stride = s if i == 0 else 1
            hidden = cin * t
            y = x
            if t != 1:
                y = cv(f"b{bi}.expand", y, cin, hidden, 1, 1, hw, CLIP)
            y = cv(f"b{bi}.dw", y, hidden, hidden, 3, stride, hw, CLIP, group=hidden)
            hw //= stride
            y = cv(f"b{bi}.project", y, hidden, c, 1, 1, hw, NOT_ACT, gain=0.5)
            x = m.add(f"b{bi}.add", y, x, f"b{bi}.add_out") if stride == 1 and cin == c else y
            cin = c
    x = cv("last", x, 320, 1280, 1, 1, hw, CLIP)
    x = m.global_avgpool("avgpool", x, "avgpool_out")
    x = m.flatten("flatten", x, "flatten_out", axis=1)
    flops += 2 * batch * classes * 1280
    x = m.gemm("fc", x, datagen.normal(datagen.seed_for(tag, "fc.w"), (classes, 1280), 0.0, 0.03),
               datagen.normal(datagen.seed_for(tag, "fc.b"), (classes,), 0.0, 0.01), "logits")
    m.output("logits", (batch, classes))
    return m.tobytes(), (batch, 3, 224, 224), flops



def vit_tiny_model(batch=1, blocks=12, classes=1000, tag="vit_tiny_model"):
    """A ViT-Tiny/16 encoder as a .one file with the operators this package runs: 16x16 stride-16 patch convolution,
    position embedding, `blocks` pre-norm encoder blocks (LayerNormalization, three projections with bias, head split
    Transposes, MatMul / Softmax / MatMul attention over 3 heads of 64 with the 1/8 scale folded into the q projection,
    head merge, output projection, residual Add, LayerNormalization, MLP with table Gelu, residual Add), final
    LayerNormalization, mean over the 196 tokens (no class token: the package has no Concat), Gemm head.  Seeded weights.
    Returns (bytes, input shape, multiply-accumulates x 2 per inference)."""
    import numpy as np
    from . import datagen, onefile

    m = onefile.OneModel()
    T, D, H, hd = 196, 192, 3, 64
    flops = 0

    def w(name, shape, std):
        return datagen.normal(datagen.seed_for(tag, name), shape, 0.0, std)

    def linear(name, x, k, n, gain=1.0, gelu=False):
        nonlocal flops
        flops += 2 * batch * T * k * n
        y = m.matmul(name, x, w(name + ".w", (k, n), gain / float(np.sqrt(k))), name + "_mm")
        y = m.add(name + ".bias", y, w(name + ".b", (n,), 0.02), name + "_out")
        return m.gelu(name + ".gelu", y, name + "_act") if gelu else y

    x = m.input("input", (batch, 3, 224, 224))
    flops += 2 * batch * D * T * 3 * 256
    x = m.conv("patch", x, w("patch.w", (D, 3, 16, 16), 1.0 / float(np.sqrt(768))), w("patch.b", (D,), 0.02), "patch_out", stride=16)
    x = m.reshape("tokens.flat", x, "tokens_flat", (batch, D, T, 1))
    x = m.transpose("tokens.t", x, "tokens_t", (0, 2, 1, 3))
    x = m.reshape("tokens", x, "tokens", (batch, T, D))
    x = m.add("pos", x, w("pos", (T, D), 0.02), "embedded")
    for b in range(blocks):
        p = f"b{b}."
        y = m.layernorm(p + "ln1", x, 1.0 + w(p + "ln1.g", (D,), 0.05), w(p + "ln1.b", (D,), 0.05), p + "ln1_out")
        heads = {}
        for which in ("q", "k", "v"):
            t = linear(p + which, y, D, D, gain=0.125 if which == "q" else 1.0)
            t = m.reshape(p + which + ".split", t, p + which + "_split", (batch, T, H, hd))
            heads[which] = m.transpose(p + which + ".heads", t, p + which + "_heads", (0, 2, 1, 3))
        flops += 2 * 2 * batch * H * T * T * hd
        kt = m.transpose(p + "k.t", heads["k"], p + "k_t", (0, 1, 3, 2))
        s = m.matmul(p + "scores", heads["q"], kt, p + "scores_out")
        a = m.softmax(p + "attn", s, p + "attn_out")
        c = m.matmul(p + "ctx", a, heads["v"], p + "ctx_out")
        c = m.transpose(p + "merge", c, p + "merged", (0, 2, 1, 3))
        c = m.reshape(p + "merge.flat", c, p + "merged_flat", (batch, T, D))
        c = linear(p + "proj", c, D, D, gain=0.5)
        x = m.add(p + "res1", c, x, p + "res1_out")
        y = m.layernorm(p + "ln2", x, 1.0 + w(p + "ln2.g", (D,), 0.05), w(p + "ln2.b", (D,), 0.05), p + "ln2_out")
        y = linear(p + "fc1", y, D, 4 * D, gelu=True)
        y = linear(p + "fc2", y, 4 * D, D, gain=0.5)
        x = m.add(p + "res2", y, x, p + "res2_out")
    x = m.layernorm("ln", x, 1.0 + w("ln.g", (D,), 0.05), w("ln.b", (D,), 0.05), "ln_out")
    x = m.reshape("pool.shape", x, "pool_in_t", (batch, T, D, 1))
    x = m.transpose("pool.t", x, "pool_in", (0, 2, 1, 3))
    x = m.reshape("pool.grid", x, "pool_grid", (batch, D, 14, 14))
    x = m.global_avgpool("pool", x, "pooled")
    x = m.flatten("flatten", x, "flat", axis=1)
    flops += 2 * batch * classes * D
    m.gemm("head", x, w("head.w", (classes, D), 0.05), w("head.b", (classes,), 0.01), "logits")
    m.output("logits", (batch, classes))
    return m.tobytes(), (batch, 3, 224, 224), flops
