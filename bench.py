#!/usr/bin/env python3
"""Benchmark of the Conv / MatMul / Gemm hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50_b32] [--layers]

Workloads: resnet50_b{1,32} (default: the ResNet-50 conv stack, fp32, batch 32),
cfg1, resnet50_net_b{1,32}, mobilenetv2_net_b{1,64} and vit_tiny_net_b{1,64} (the whole model as a .one file through the runtime), resnet50_int8_net_b{1,32} and mobilenetv2_int8_net_b{1,64} (the same files through the model-level quantisation step: W8A32 convolutions with calibrated scales), mobilenetv2_b{1,64}, yolov8s_int8_b{1,16}, vit_tiny_b{1,64}[_bf16|_f16], and `copy` (the yardstick
the HBM traffic counters are scaled by).

A step is one pass over every layer of the workload: one launch per layer, inputs, weights and outputs
resident in HBM, synthetic seeded data.  Prints ONE JSON line: whole-stack throughput (`value`, TFLOP/s
or TOP/s with 2 operations per multiply-accumulate; bias, activation and (de)quantisation not counted),
the roofline position of the dominant kernel measured with HIP events on the launch stream, and the CPU
baseline (the reference's own x86 kernels when their build is present, else the CPU restatement) timed on
this machine's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

import numpy as np  # noqa: E402

PEAK = {"f32": 157.3, "bf16": 2500.0, "f16": 2500.0, "i8": 5000.0}   # dense MFMA, TFLOP/s (TOP/s)
HBM_PEAK_GBS = 8000.0


# ---- layers: device-resident operands + one launch -------------------------------------------------------

def device_uniform(torch, seed, shape, lo=-1.0, hi=1.0):
    """activations U(lo, hi) drawn on the device from a seeded generator (the large tensors of batch 16 to 64 take
    longer to draw on the host than the whole measurement)"""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed & 0x7FFFFFFFFFFF)
    return torch.rand(shape, generator=g, device="cuda", dtype=torch.float32) * (hi - lo) + lo


class ConvF32Layer:
    kind = "conv_f32"

    def __init__(self, torch, hip, name, d, tag):
        from onenew_amd import datagen
        kc = d.cin if d.group == 1 else 1
        w = datagen.normal(datagen.seed_for(f"{tag}/{name}", "w"), (d.cout, kc, d.kh, d.kw), 0.0, float(np.sqrt(2.0 / (kc * d.kh * d.kw))))
        b = datagen.normal(datagen.seed_for(f"{tag}/{name}", "b"), (d.cout,), 0.0, 0.01)
        self.name, self.d = name, d
        self.x = device_uniform(torch, datagen.seed_for(f"{tag}/{name}", "x"), (d.n, d.cin, d.h, d.w))
        self.w, self.b = torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda()
        self.y = torch.empty((d.n, d.cout) + d.out_hw(), dtype=torch.float32, device="cuda")
        # k x k weights are re-laid out once at load time (tap-major), as an inference runtime would
        self.wp = hip.pack_conv_weights(d, self.w)
        self.flops, self.bytes = d.flops(), d.algorithmic_bytes()
        self.dense = d.group == 1
        oh, ow = d.out_hw()
        self.shape = f"M={d.cout} N={d.n * oh * ow} K={d.k_per_out()}"

    def launch(self, hip):
        if self.wp is not None:
            hip.conv2d_f32(self.d, self.x, self.wp, self.b, None, out=self.y, packed=True)
        else:
            hip.conv2d_f32(self.d, self.x, self.w, self.b, None, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        import cases
        from onenew_amd import abi
        d1 = abi.ConvDesc.from_buffer_copy(self.d)
        d1.n = 1
        x, w, b = cases.conv_inputs(f"{tag}/cpu/{self.name}", d1)
        if oracle.have_ref():
            op = ops.Conv(ops.Plugin(oracle.ref_path("Conv")).eval, d1, w, b, silu_lut=cases.silu_lut(),
                          scratch_bytes=oracle.ref_scratch_bytes(d1))
            xin = ops.aligned_empty(x.shape)
            xin[...] = x
            out = ops.aligned_empty((1, d1.cout) + d1.out_hw())
            return d1.flops(), lambda: op(xin, out=out)
        return d1.flops(), lambda: oracle.conv2d_f32(d1, x, w, b, cases.silu_lut())


class ConvW8A32Layer:
    kind = "conv_w8a32"

    def __init__(self, torch, hip, name, d, tag):
        import cases
        from onenew_amd import datagen
        d1 = type(d).from_buffer_copy(d)
        d1.n, d1.h, d1.w = 1, d.kh, d.kw          # the weight-side operands of the case, without its activations
        _, w8, b32, aux = cases.conv_inputs(f"{tag}/{name}", d1, quant=True)
        self.name, self.d = name, d
        self.x = device_uniform(torch, datagen.seed_for(f"{tag}/{name}", "x"), (d.n, d.cin, d.h, d.w))
        self.w8, self.b32, self.aux = (torch.from_numpy(t).cuda() for t in (w8, b32, aux))
        self.lut = torch.from_numpy(cases.silu_lut()).cuda()
        self.y = torch.empty((d.n, d.cout) + d.out_hw(), dtype=torch.float32, device="cuda")
        self.ws = torch.empty(max(16, hip.conv2d_w8a32_workspace(d)), dtype=torch.uint8, device="cuda")
        # weights are laid out for the kernel once, as a runtime does when it loads the layer
        self.wp = hip.pack_conv_weights_w8(d, self.w8)
        self.flops, self.bytes = d.flops(), d.algorithmic_bytes(eb_x=4, eb_w=1, eb_y=4)
        self.dense = d.group == 1
        oh, ow = d.out_hw()
        self.shape = f"M={d.cout} N={d.n * oh * ow} K={d.k_per_out()}"

    def launch(self, hip):
        if self.wp is not None:
            hip.conv2d_w8a32(self.d, self.x, self.wp, self.b32, self.aux, self.lut, out=self.y, workspace=self.ws,
                             packed=True)
        else:
            hip.conv2d_w8a32(self.d, self.x, self.w8, self.b32, self.aux, self.lut, out=self.y, workspace=self.ws)

    def cpu_runner(self, ops, oracle, tag):
        import cases
        from onenew_amd import abi
        d1 = abi.ConvDesc.from_buffer_copy(self.d)
        d1.n = 1
        x, w8, b32, aux = cases.conv_inputs(f"{tag}/cpu/{self.name}", d1, quant=True)
        if oracle.have_ref():
            op = ops.Conv(ops.Plugin(oracle.ref_path("Conv")).eval, d1, w8, b32, weight_aux=aux, silu_lut=cases.silu_lut(),
                          scratch_bytes=oracle.ref_scratch_bytes(d1))
            xin = ops.aligned_empty(x.shape)
            xin[...] = x
            out = ops.aligned_empty((1, d1.cout) + d1.out_hw())
            return d1.flops(), lambda: op(xin, out=out)
        return d1.flops(), lambda: oracle.conv2d_w8a32(d1, x, w8, b32, aux, cases.silu_lut())


class ConvW8A8Layer(ConvW8A32Layer):
    """the int8 chain form: int8 NHWC activations in and out, quantisation fused into the producer's epilogue"""
    kind = "conv_w8a8"

    def __init__(self, torch, hip, name, d, tag):
        super().__init__(torch, hip, name, d, tag)
        self.d.out_s8, self.d.output_scale = 1, 0.03
        self.xq = hip.quantize_nhwc_s8(self.x, d.input_scale)
        oh, ow = d.out_hw()
        self.yq = torch.empty((d.n, oh, ow, (d.cout + 15) // 16 * 16), dtype=torch.int8, device="cuda")
        self.bytes = d.algorithmic_bytes(eb_x=1, eb_w=1, eb_y=1)
        del self.x, self.y

    def launch(self, hip):
        hip.conv2d_w8a8_nhwc(self.d, self.xq, self.wp, self.b32, self.aux, self.lut, out=self.yq)

    def cpu_runner(self, ops, oracle, tag):
        import cases
        from onenew_amd import abi
        d1 = abi.ConvDesc.from_buffer_copy(self.d)
        d1.n, d1.out_s8 = 1, 0
        x, w8, b32, aux = cases.conv_inputs(f"{tag}/cpu/{self.name}", d1, quant=True)
        if oracle.have_ref():
            # the reference has no int8-to-int8 form: its W8A32 convolution (fp32 in and out) is the baseline
            op = ops.Conv(ops.Plugin(oracle.ref_path("Conv")).eval, d1, w8, b32, weight_aux=aux, silu_lut=cases.silu_lut(),
                          scratch_bytes=oracle.ref_scratch_bytes(d1))
            xin = ops.aligned_empty(x.shape)
            xin[...] = x
            out = ops.aligned_empty((1, d1.cout) + d1.out_hw())
            return d1.flops(), lambda: op(xin, out=out)
        return d1.flops(), lambda: oracle.conv2d_w8a32(d1, x, w8, b32, aux, cases.silu_lut())


class GlueLayer:
    """the memory-bound operators between the convolutions of ResNet-50: MaxPool after the stem, the residual
    Add + ReLU of every block (one fused pass), GlobalAveragePool at the end"""
    kind = "glue"
    dense = False

    def __init__(self, torch, hip, name, op, shape, tag):
        from onenew_amd import abi, datagen
        self.name, self.op = name, op
        n, c, h, w = shape
        rnd = lambda role: torch.from_numpy(datagen.normal(datagen.seed_for(f"{tag}/{name}", role), shape, 0.0, 1.0)).cuda()
        self.x = rnd("x")
        if op == "add_relu":
            self.r = rnd("r")
            self.y = torch.empty_like(self.x)
            self.flops, self.bytes = 2 * self.x.numel(), 12 * self.x.numel()
        elif op == "maxpool":
            self.pd = abi.PoolDesc(n, c, h, w, 3, 3, 2, 2, 1)
            oh, ow = self.pd.out_hw()
            self.y = torch.empty((n, c, oh, ow), dtype=torch.float32, device="cuda")
            self.flops, self.bytes = 9 * self.y.numel(), 4 * (self.x.numel() + self.y.numel())
        else:
            self.y = torch.empty((n, c, 1, 1), dtype=torch.float32, device="cuda")
            self.flops, self.bytes = self.x.numel(), 4 * (self.x.numel() + self.y.numel())
        self.shape = f"{op} {n}x{c}x{h}x{w}"

    def launch(self, hip):
        if self.op == "add_relu":
            hip.add_f32(self.x, self.r, relu=True, out=self.y)
        elif self.op == "maxpool":
            hip.maxpool_f32(self.pd, self.x, out=self.y)
        else:
            hip.global_avgpool_f32(self.x, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        """the reference's own Add then Relu (two passes), MaxPool, GlobalAveragePool on one image"""
        import os
        x = self.x[:1].cpu().numpy()
        ref = lambda op: ops.Plugin(os.path.join(os.path.dirname(oracle.ref_path("Conv")), f"lib{op}_x86.so")).eval
        if self.op == "add_relu":
            r = self.r[:1].cpu().numpy()
            if oracle.have_ref():
                add, relu = ops.Add(ref("Add")), ops.Relu(ref("Relu"))
                buf = ops.aligned_empty(x.shape)
                return self.flops // self.x.shape[0], lambda: relu(add(x, r, out=buf))
            return self.flops // self.x.shape[0], lambda: oracle.relu_f32(oracle.add_f32(x, r))
        if self.op == "maxpool":
            if oracle.have_ref():
                mp = ops.MaxPool(ref("MaxPool"), 3, 2, 1, scratch_bytes=8 * x.size + (1 << 20))
                return self.flops // self.x.shape[0], lambda: mp(x)
            return self.flops // self.x.shape[0], lambda: oracle.maxpool_f32(x, 3, 2, 1)
        if oracle.have_ref():
            gp = ops.GlobalAveragePool(ref("GlobalAveragePool"))
            return self.flops // self.x.shape[0], lambda: gp(x)
        return self.flops // self.x.shape[0], lambda: oracle.global_avgpool_f32(x)


class VitGlueLayer:
    """the memory-bound operators around the MatMuls of one ViT-Tiny block"""
    kind = "glue"
    dense = False

    def __init__(self, torch, hip, name, op, shape, tag, perm=None):
        import cases
        from onenew_amd import datagen
        self.name, self.op, self.perm = name, op, perm
        rnd = lambda role, shp, sd=1.0: torch.from_numpy(datagen.normal(datagen.seed_for(f"{tag}/{name}", role), shp, 0.0, sd)).cuda()
        self.x = rnd("x", shape)
        self.y = torch.empty([shape[p] for p in perm] if perm else shape, dtype=torch.float32, device="cuda")
        n = self.x.numel()
        self.bytes, self.flops = 8 * n, n
        if op == "layernorm":
            self.w, self.b = rnd("w", (shape[-1],)), rnd("b", (shape[-1],))
            self.flops = 8 * n
        elif op == "bias_add":
            self.b = rnd("b", (shape[-1],))
        elif op == "residual_add":
            self.r = rnd("r", shape)
            self.bytes = 12 * n
        elif op == "gelu":
            self.lut = torch.from_numpy(cases.gelu_lut()).cuda()
        elif op == "softmax":
            self.flops = 4 * n
        self.shape = f"{op} {'x'.join(map(str, shape))}"

    def launch(self, hip):
        if self.op == "layernorm":
            hip.layernorm_f32(self.x, self.w, self.b, out=self.y)
        elif self.op == "bias_add":
            hip.add_f32(self.x, self.b, out=self.y)
        elif self.op == "residual_add":
            hip.add_f32(self.x, self.r, out=self.y)
        elif self.op == "gelu":
            hip.gelu_lut_f32(self.x, self.lut, out=self.y)
        elif self.op == "softmax":
            hip.softmax_f32(self.x, out=self.y)
        else:
            hip.transpose_f32(self.x, self.perm, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        import cases
        x = self.x[:1].cpu().numpy()
        fl = self.flops // self.x.shape[0]
        if self.op == "layernorm":
            w, b = self.w.cpu().numpy(), self.b.cpu().numpy()
            return fl, lambda: oracle.layernorm_f32(x, w, b)
        if self.op == "bias_add":
            b = self.b.cpu().numpy()
            return fl, lambda: oracle.add_f32(x, b)
        if self.op == "residual_add":
            r = self.r[:1].cpu().numpy()
            return fl, lambda: oracle.add_f32(x, r)
        if self.op == "gelu":
            lut = cases.gelu_lut()
            return fl, lambda: oracle.lut_act(x, lut)
        if self.op == "softmax":
            return fl, lambda: oracle.softmax_f32(x)
        return fl, lambda: oracle.transpose_f32(x, self.perm)


class IrBlockLayer:
    """a whole inverted-residual block (1x1 expansion + CLIP, depthwise 3x3 + CLIP, 1x1 projection) in one launch: neither
    wide tensor leaves the chip.  Work is counted as the three convolutions'; bytes as what the launch itself has to move
    (input, weights, output), with the bytes of the three-launch chain it replaces kept beside them (`chain_bytes`)"""
    kind = "ir_block"

    def __init__(self, torch, hip, name, ex, dw, pw, tag):
        from onenew_amd import datagen
        self.name, self.ex, self.dw, self.pw = name.replace(".expand", "") + ".block", ex, dw, pw
        self.x = device_uniform(torch, datagen.seed_for(f"{tag}/{name}", "x"), (ex.n, ex.cin, ex.h, ex.w))
        g = lambda role, shape, std: torch.from_numpy(datagen.normal(datagen.seed_for(f"{tag}/{name}", role), shape, 0.0, std)).cuda()
        self.ex_w, self.ex_b = g("w", (ex.cout, ex.cin, 1, 1), float(np.sqrt(2.0 / ex.cin))), g("b", (ex.cout,), 0.01)
        self.dw_w, self.dw_b = g("dw", (dw.cout, 1, 3, 3), float(np.sqrt(2.0 / 9))), g("db", (dw.cout,), 0.01)
        self.pw_w, self.pw_b = g("pw", (pw.cout, pw.cin, 1, 1), float(np.sqrt(2.0 / pw.cin))), g("pb", (pw.cout,), 0.01)
        self.packed = hip.ir_block_pack_weights(self.ex_w, self.pw_w)
        oh, ow = dw.out_hw()
        self.y = torch.empty((dw.n, pw.cout, oh, ow), dtype=torch.float32, device="cuda")
        self.flops = ex.flops() + dw.flops() + pw.flops()
        # what this launch has to move: the block's input, its weights and biases, its output (every tensor once) ...
        self.bytes = 4 * (self.x.numel() + self.y.numel() + self.ex_w.numel() + self.ex_b.numel() + self.dw_w.numel()
                          + self.dw_b.numel() + self.pw_w.numel() + self.pw_b.numel())
        # ... and what the three separate convolutions it replaces move (both wide tensors written and read back)
        self.chain_bytes = ex.algorithmic_bytes() + dw.algorithmic_bytes() + pw.algorithmic_bytes()
        self.dense = False           # grouped with the depthwise layers: the memory-bound part of the network
        self.shape = f"C={ex.cin}>{dw.cin}>{pw.cout} N={dw.n * oh * ow} s{dw.stride_h}"

    def launch(self, hip):
        hip.ir_block_f32(self.ex, self.dw, self.pw, self.x, self.packed, self.ex_b, self.dw_w, self.dw_b, self.pw_b, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        runs = [ConvF32Layer.cpu_runner(type("L", (), {"d": d, "name": self.name + sfx})(), ops, oracle, tag)
                for d, sfx in ((self.ex, "/ex"), (self.dw, "/dw"), (self.pw, "/pw"))]
        return sum(f for f, _ in runs), lambda: [r() for _, r in runs]


class ConvPwLayer:
    """a convolution with at most 64 output channels and the 1x1 convolution over its result in one launch
    (onhip_conv2d_pw_f32): the tensor between them stays on the chip.  Operands are seeded as the two separate layers'
    are; work is counted as the two convolutions', bytes as what the launch itself has to move (input, both weight
    tensors and biases, output), with the bytes of the two launches it replaces kept beside them (`chain_bytes`)"""
    kind = "conv_pw"

    def __init__(self, torch, hip, name_a, da, name_b, db, tag):
        from onenew_amd import datagen
        self.name, self.d, self.db = name_a + "+" + name_b.rsplit(".", 1)[-1], da, db
        self.x = device_uniform(torch, datagen.seed_for(f"{tag}/{name_a}", "x"), (da.n, da.cin, da.h, da.w))
        g = lambda name, role, shape, std: torch.from_numpy(datagen.normal(datagen.seed_for(f"{tag}/{name}", role), shape, 0.0, std)).cuda()
        self.wa = g(name_a, "w", (da.cout, da.cin, da.kh, da.kw), float(np.sqrt(2.0 / (da.cin * da.kh * da.kw))))
        self.ba = g(name_a, "b", (da.cout,), 0.01)
        self.wb, self.bb = g(name_b, "w", (db.cout, db.cin, 1, 1), float(np.sqrt(2.0 / db.cin))), g(name_b, "b", (db.cout,), 0.01)
        self.wa_packed, self.wb_packed = hip.pack_conv_weights(da, self.wa), hip.conv2d_pw_pack_weights(db, self.wb)
        self.y = torch.empty((db.n, db.cout) + db.out_hw(), dtype=torch.float32, device="cuda")
        self.flops = da.flops() + db.flops()
        self.bytes = 4 * (self.x.numel() + self.y.numel() + self.wa.numel() + self.ba.numel() + self.wb.numel() + self.bb.numel())
        self.chain_bytes = da.algorithmic_bytes() + db.algorithmic_bytes()
        self.dense = True
        oh, ow = da.out_hw()
        self.shape = f"M={da.cout}>{db.cout} N={da.n * oh * ow} K={da.k_per_out()}"

    def launch(self, hip):
        hip.conv2d_pw_f32(self.d, self.db, self.x, self.wa_packed, self.ba, self.wb_packed, self.bb, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        runs = [ConvF32Layer.cpu_runner(type("L", (), {"d": d, "name": self.name + sfx})(), ops, oracle, tag)
                for d, sfx in ((self.d, "/a"), (self.db, "/b"))]
        return sum(f for f, _ in runs), lambda: [r() for _, r in runs]


class ConvH16Layer:
    """dense convolution with bf16 / fp16 storage: 16-bit NHWC in, 16-bit NHWC out, weights packed once"""
    kind = "conv_h16"

    def __init__(self, torch, hip, name, d, compute, tag):
        from onenew_amd import abi, datagen
        d = abi.ConvDesc.from_buffer_copy(d)
        d.compute = compute
        w = datagen.normal(datagen.seed_for(f"{tag}/{name}", "w"), (d.cout, d.cin, d.kh, d.kw), 0.0, float(np.sqrt(2.0 / (d.cin * d.kh * d.kw))))
        b = datagen.normal(datagen.seed_for(f"{tag}/{name}", "b"), (d.cout,), 0.0, 0.01)
        self.name, self.d = name, d
        x = device_uniform(torch, datagen.seed_for(f"{tag}/{name}", "x"), (d.n, d.cin, d.h, d.w))
        # a first layer (at most 8 input channels, filter rows of at most 8 columns) is kept in the storage form made for
        # it, 8 channels per pixel instead of 32: what a 16-bit pipeline is fed with at its head
        self.first = hip.load().onhip_h16_first_width(d) > 0
        if self.first:
            self.x = hip.h16_first_from_nchw(d, x)
            self.wp = hip.h16_first_pack_weights(d, torch.from_numpy(w).cuda())
        else:
            self.x = hip.h16_from_nchw(x, compute)
            self.wp = hip.h16_pack_conv_weights(d, torch.from_numpy(w).cuda())
        del x
        self.b = torch.from_numpy(b).cuda()
        oh, ow = d.out_hw()
        self.y = torch.empty((d.n, oh, ow, hip.h16_pitch(d.cout)), dtype=self.x.dtype, device="cuda")
        # every tensor once at 2 bytes per element, unpadded (the channel padding the layout adds is not counted as work)
        self.flops, self.bytes = d.flops(), d.algorithmic_bytes(eb_x=2, eb_w=2, eb_y=2)
        self.dense = True
        self.shape = f"M={d.cout} N={d.n * oh * ow} K={d.k_per_out()}"

    def launch(self, hip):
        if self.first:
            hip.conv2d_h16_first(self.d, self.x, self.wp, self.b, out=self.y)
        else:
            hip.conv2d_h16(self.d, self.x, self.wp, self.b, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        return ConvF32Layer.cpu_runner(self, ops, oracle, tag)


class LinearH16Layer:
    """a transformer's linear layer with bf16 / fp16 storage: rows in, rows out, fused bias and table GELU"""
    kind = "linear_h16"

    def __init__(self, torch, hip, name, md, has_bias, gelu, compute, tag):
        import cases
        from onenew_amd import datagen
        self.name, self.md, self.compute = name, md, compute
        rows = md.batch * md.m
        a = datagen.normal(datagen.seed_for(tag, name, "a"), (md.batch, md.m, md.k), 0.0, 1.0)
        b = datagen.normal(datagen.seed_for(tag, name, "b"), (md.k, md.n), 0.0, 0.02)
        self.host = (a, b)
        self.a = hip.h16_from_rows(torch.from_numpy(a.reshape(rows, md.k)).cuda(), compute)
        self.bp = hip.h16_pack_matmul_weights(torch.from_numpy(b).cuda(), compute)
        self.bias = torch.from_numpy(datagen.normal(datagen.seed_for(tag, name, "bias"), (md.n,), 0.0, 0.02)).cuda() \
            if has_bias else None
        self.lut = torch.from_numpy(cases.gelu_lut()).cuda() if gelu else None
        self.y = torch.empty((rows, hip.h16_pitch(md.n)), dtype=self.a.dtype, device="cuda")
        self.flops, self.bytes = md.flops(), md.algorithmic_bytes(eb=2, bias=has_bias)
        self.dense = True
        self.shape = f"B={md.batch} M={md.m} N={md.n} K={md.k}"

    def launch(self, hip):
        hip.linear_h16(self.a, self.bp, self.md.k, self.md.n, self.compute, bias=self.bias, gelu_lut=self.lut, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        return MatmulLayer.cpu_runner(self, ops, oracle, tag)


class AttentionLayer:
    """scores = q k^T * scale, Softmax, context = scores v of every (batch, head) in one launch, q / k / v read as slices of
    the qkv projection's output and the context written with the heads merged; counted as the two MatMuls it replaces"""
    kind = "attention"

    def __init__(self, torch, hip, name, md_scores, md_context, heads, tag, dtype=None):
        from onenew_amd import datagen
        self.name = name
        bh, t, hd = md_scores.batch, md_scores.m, md_scores.k
        b = bh // heads
        self.qkv = device_uniform(torch, datagen.seed_for(tag, name, "qkv"), (b, t, 3, heads, hd), -1.5, 1.5)
        if dtype is not None:   # 16-bit storage: q, k, v slices of a 16-bit projection output, 16-bit result
            self.qkv = self.qkv.to(dtype)
        self.q, self.k, self.v = (self.qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        self.scale = 1.0 / float(np.sqrt(hd))
        self.y = torch.empty((b, t, heads * hd), dtype=self.qkv.dtype, device="cuda")
        self.mds = (md_scores, md_context)
        self.flops = md_scores.flops() + md_context.flops()
        eb = 4 if dtype is None else 2
        self.bytes = md_scores.algorithmic_bytes(eb=eb) + md_context.algorithmic_bytes(eb=eb)   # of the unfused chain's two MatMuls
        self.dense = True
        self.shape = f"B={b} H={heads} T={t} D={hd}"

    def launch(self, hip):
        hip.attention(self.q, self.k, self.v, scale=self.scale, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        # reference semantics: the two MatMuls and the Softmax between them as separate operators
        ms, mc = self.mds
        from onenew_amd import datagen
        q = datagen.normal(datagen.seed_for(tag, self.name, "cq"), (ms.batch, ms.m, ms.k), 0.0, 1.0)
        kt = datagen.normal(datagen.seed_for(tag, self.name, "ck"), (ms.batch, ms.k, ms.n), 0.0, 1.0)
        v = datagen.normal(datagen.seed_for(tag, self.name, "cv"), (mc.batch, mc.k, mc.n), 0.0, 1.0)

        def run():
            return oracle.matmul_f32(oracle.softmax_f32(oracle.matmul_f32(q, kt)), v)
        return self.flops, run


class MatmulLayer:
    kind = "matmul"

    def __init__(self, torch, hip, name, md, has_bias, gelu, compute, tag):
        import cases
        from onenew_amd import datagen
        self.name, self.md, self.compute = name, md, compute
        ashape = (md.batch, md.m, md.k)
        bshape = (md.k, md.n) if md.b_shared else (md.batch, md.k, md.n)
        a = datagen.normal(datagen.seed_for(tag, name, "a"), ashape, 0.0, 1.0)
        b = datagen.normal(datagen.seed_for(tag, name, "b"), bshape, 0.0, 0.02)
        self.host = (a, b)
        self.a, self.b = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
        self.bias = torch.from_numpy(datagen.normal(datagen.seed_for(tag, name, "bias"), (md.n,), 0.0, 0.02)).cuda() \
            if has_bias else None
        self.lut = torch.from_numpy(cases.gelu_lut()).cuda() if gelu else None
        self.y = torch.empty((md.batch, md.m, md.n), dtype=torch.float32, device="cuda")
        self.flops, self.bytes = md.flops(), md.algorithmic_bytes(bias=has_bias)
        self.dense = True
        self.shape = f"B={md.batch} M={md.m} N={md.n} K={md.k}"

    def launch(self, hip):
        hip.matmul(self.a, self.b, bias=self.bias, gelu_lut=self.lut, compute=self.compute, out=self.y)

    def cpu_runner(self, ops, oracle, tag):
        # reference semantics: MatMul (+ Add + Gelu as separate sweeps); one image's worth of the batch
        md = self.md
        per_image = md.batch if md.b_shared else md.batch      # the ViT batch is already folded into `batch`
        a, b = self.host
        flops = md.flops()
        if oracle.have_ref():
            mm = ops.MatMul(ops.Plugin(oracle.ref_path("MatMul")).eval)
            aa, bb = ops.aligned_empty(a.shape), ops.aligned_empty(b.shape)
            aa[...], bb[...] = a, b
            out = ops.aligned_empty(a.shape[:-1] + (md.n,))
            return flops, lambda: mm(aa, bb, out=out)
        return flops, lambda: oracle.matmul_f32(a, b)


def make_workload(torch, hip, name):
    """-> (description, dtype, [layers])"""
    from onenew_amd import abi, stacks, datagen
    tag = name

    def conv_stack(layers):
        return [ConvF32Layer(torch, hip, n, d, tag) for n, d in layers]

    if name.startswith("resnet50_b") and name.endswith(("_bf16", "_f16")):
        n = int(name.split("_b")[1].split("_")[0])
        compute, dtype = (abi.COMPUTE_BF16, "bf16") if name.endswith("_bf16") else (abi.COMPUTE_F16, "f16")
        return (f"ResNet-50 conv stack {dtype} with 16-bit storage (NHWC in and out, fp32 accumulate), batch {n}, 224x224, "
                f"53 conv layers, fused ReLU", dtype,
                [ConvH16Layer(torch, hip, ln, d, compute, tag) for ln, d in stacks.with_batch(stacks.resnet50(), n)])
    if name in ("cfg1_bf16", "cfg1_f16"):
        import cases
        compute, dtype = (abi.COMPUTE_BF16, "bf16") if name.endswith("_bf16") else (abi.COMPUTE_F16, "f16")
        return (f"Conv2d+ReLU {dtype} with 16-bit storage 64->64 56x56 3x3 s1 p1, batch 1", dtype,
                [ConvH16Layer(torch, hip, "cfg1", cases.conv_f32_cases()["cfg1_64x56_3x3"], compute, tag)])
    if name.startswith("resnet50_b"):
        n = int(name.split("_b")[1].split("_")[0])
        spec = stacks.with_batch(stacks.resnet50(), n)
        # conv2 (3x3) and conv3 (1x1) of a block in one launch where the library takes the pair and expects it to pay
        # (the 64-channel blocks of the first stage at batch sizes that fill the chip)
        by_name = {ln: d for ln, d in spec}
        layers, taken, pairs = [], set(), 0
        for ln, d in spec:
            if ln in taken:
                continue
            other = ln[:-len("conv2")] + "conv3"
            if (not name.endswith("_unfused") and ln.endswith(".conv2") and other in by_name
                    and hip.conv2d_pw_supported(d, by_name[other]) >= 2):
                layers.append(ConvPwLayer(torch, hip, ln, d, other, by_name[other], tag))
                taken.add(other)
                pairs += 1
            else:
                layers.append(ConvF32Layer(torch, hip, ln, d, tag))
        return (f"ResNet-50 conv stack fp32, batch {n}, 224x224, 53 conv layers, fused ReLU"
                + (f"; {pairs} pairs of a 3x3 and the 1x1 convolution after it (64 channels between them) as one launch each" if pairs else ""),
                "f32", layers)
    if name.startswith("resnet50_glue_b"):
        n = int(name.split("_b")[1])
        spec = [("maxpool", "maxpool", (n, 64, 112, 112))]
        for stage, (c, hw, blocks) in enumerate([(256, 56, 3), (512, 28, 4), (1024, 14, 6), (2048, 7, 3)], 1):
            spec += [(f"l{stage}.{b}.add_relu", "add_relu", (n, c, hw, hw)) for b in range(blocks)]
        spec.append(("avgpool", "gap", (n, 2048, 7, 7)))
        return (f"ResNet-50 operators between the convolutions fp32, batch {n}: MaxPool 3x3 s2, 16 residual "
                f"Add + ReLU (fused), GlobalAveragePool", "f32",
                [GlueLayer(torch, hip, ln, op, shape, tag) for ln, op, shape in spec])
    if name.startswith("yolov8s_int8chain_b"):
        n = int(name.split("_b")[1])
        layers = []
        for i, (ln, d) in enumerate(stacks.with_batch(stacks.yolov8s(), n)):
            d.input_scale = float(datagen.uniform(datagen.seed_for(tag, i, "s_in"), (1,), 0.005, 0.05)[0])
            layers.append(ConvW8A8Layer(torch, hip, ln, d, tag))
        return (f"YOLOv8s conv stack int8 chain form (int8 NHWC activations in and out, int32 accumulate, SiLU table, "
                f"requantise), batch {n}, 640x640, {len(layers)} conv layers", "i8", layers)
    if name.startswith("vit_tiny_glue_b"):
        n = int(name.split("_b")[1])
        t, c, h, hd = 197, 192, 3, 64
        spec = [("ln1", "layernorm", (n, t, c), None), ("qkv.bias", "bias_add", (n, t, 3 * c), None),
                ("q.heads", "transpose", (n, t, h, hd), (0, 2, 1, 3)), ("k.t", "transpose", (n, h, t, hd), (0, 1, 3, 2)),
                ("softmax", "softmax", (n, h, t, t), None), ("ctx.merge", "transpose", (n, h, t, hd), (0, 2, 1, 3)),
                ("proj.bias", "bias_add", (n, t, c), None), ("res1", "residual_add", (n, t, c), None),
                ("ln2", "layernorm", (n, t, c), None), ("fc1.bias", "bias_add", (n, t, 4 * c), None),
                ("gelu", "gelu", (n, t, 4 * c), None), ("fc2.bias", "bias_add", (n, t, c), None),
                ("res2", "residual_add", (n, t, c), None)]
        return (f"ViT-Tiny block, operators around the MatMuls fp32, batch {n}: LayerNorm x2, bias adds, head "
                f"transposes, Softmax, table GELU, residual adds", "f32",
                [VitGlueLayer(torch, hip, ln, op, shape, tag, perm) for ln, op, shape, perm in spec])
    if name.startswith("mobilenetv2_b"):
        n = int(name.split("_b")[1].split("_")[0])
        spec = stacks.with_batch(stacks.mobilenet_v2(), n)
        layers, blocks, i = [], 0, 0
        while i < len(spec):
            ln, d = spec[i]
            # expansion, depthwise and projection in one launch where the block kernel takes the shapes
            if (not name.endswith("_unfused") and i + 2 < len(spec) and d.group == 1
                    and hip.ir_block_supported(d, spec[i + 1][1], spec[i + 2][1]) >= 2):
                layers.append(IrBlockLayer(torch, hip, ln, d, spec[i + 1][1], spec[i + 2][1], tag))
                blocks += 1
                i += 3
                continue
            layers.append(ConvF32Layer(torch, hip, ln, d, tag))
            i += 1
        return (f"MobileNetV2 conv stack fp32, batch {n}, 224x224, 52 conv layers (17 depthwise), ReLU6 as CLIP; {blocks} whole inverted-residual blocks "
                f"as one launch each", "f32", layers)
    if name == "cfg1":
        import cases
        return ("Conv2d+ReLU fp32 64->64 56x56 3x3 s1 p1, batch 1", "f32",
                conv_stack([("cfg1", cases.conv_f32_cases()["cfg1_64x56_3x3"])]))
    if name.startswith("yolov8s_int8_b"):
        n = int(name.split("_b")[1])
        layers = []
        for i, (lname, d) in enumerate(stacks.with_batch(stacks.yolov8s(), n)):
            d.input_scale = float(datagen.uniform(datagen.seed_for(tag, i, "s_in"), (1,), 0.005, 0.05)[0])
            layers.append(ConvW8A32Layer(torch, hip, lname, d, tag))
        return (f"YOLOv8s conv stack W8A32 int8, batch {n}, 640x640, 63 conv layers, SiLU table, fp32 in/out", "i8", layers)
    if name.startswith("vit_tiny_b"):
        rest = name[len("vit_tiny_b"):]
        compute, dtype = abi.COMPUTE_F32, "f32"
        if rest.endswith("_bf16"):
            compute, dtype, rest = abi.COMPUTE_BF16, "bf16", rest[:-5]
        elif rest.endswith("_f16"):
            compute, dtype, rest = abi.COMPUTE_F16, "f16", rest[:-4]
        n = int(rest)
        if compute != abi.COMPUTE_F32:
            # 16-bit storage throughout: the four linear layers and the attention between them
            tdt = torch.bfloat16 if compute == abi.COMPUTE_BF16 else torch.float16
            spec = {ln: md for ln, md, _, _ in stacks.vit_tiny(n)}
            layers = []
            for ln, md, hb, g in stacks.vit_tiny(n):
                if ln == "scores":
                    layers.append(AttentionLayer(torch, hip, "attention", md, spec["context"], 3, tag, dtype=tdt))
                elif ln != "context":
                    layers.append(LinearH16Layer(torch, hip, ln, md, hb, g, compute, tag))
            return (f"ViT-Tiny block MatMuls {dtype} with 16-bit storage, batch {n}, 197 tokens x 192, 3 heads: qkv, attention "
                    f"(scores, Softmax and context in one launch), proj, fc1 (fused bias + table GELU), fc2", dtype, layers)
        spec = {ln: (md, hb, g) for ln, md, hb, g in stacks.vit_tiny(n)}
        layers = []
        for ln, md, hb, g in stacks.vit_tiny(n):
            if ln == "scores":
                layers.append(AttentionLayer(torch, hip, "attention", md, spec["context"][0], 3, tag))
            elif ln != "context":
                layers.append(MatmulLayer(torch, hip, ln, md, hb, g, compute, tag))
        return (f"ViT-Tiny block MatMuls {dtype}, batch {n}, 197 tokens x 192, 3 heads: qkv, attention (scores, Softmax and "
                f"context in one launch, head split and merge in its strides), proj, fc1 with fused bias + table GELU, fc2",
                dtype, layers)
    raise SystemExit(f"unknown workload {name}")


def measured_traffic(workload, group):
    """HBM bytes per launch of a kernel group ("igemm" or "depthwise") from the committed counter summary
    (profiles/<workload>_traffic.json: FETCH_SIZE / WRITE_SIZE scaled by the copy yardstick), else None"""
    path = os.path.join(ROOT, "profiles", f"{workload}_traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f).get("groups", {}).get(group, {}).get("hbm_bytes_per_launch")


def time_layers(torch, hip, layers, reps):
    """average launch duration of every layer, HIP events on the launch stream"""
    out = []
    for L in layers:
        for _ in range(3):
            L.launch(hip)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            L.launch(hip)
        e1.record()
        e1.synchronize()
        out.append(e0.elapsed_time(e1) / reps)   # ms
    return out


def plugin_eval_latency(hip):
    """the drop-in boundary end to end: `eval` of libConv_hip.so on host buffers (Conv2d+ReLU 64->64 56x56 3x3), i.e. with the
    activation copied in and the result copied out over PCIe on every call; never part of `value`"""
    import cases
    from onenew_amd import ops
    d = cases.conv_f32_cases()["cfg1_64x56_3x3"]
    x, w, b = cases.conv_inputs("bench/plugin_cfg1", d)
    op = ops.Conv(ops.Plugin(hip.plugin_path("Conv")).eval, d, w, b, silu_lut=cases.silu_lut())
    xin = ops.aligned_empty(x.shape)
    xin[...] = x
    out = ops.aligned_empty((1, d.cout) + d.out_hw())
    for _ in range(5):
        op(xin, out=out)
    times = []
    for _ in range(30):
        t0 = time.perf_counter()
        op(xin, out=out)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"ms_per_call": round(med * 1e3, 4), "tflops": round(d.flops() / med / 1e12, 3),
            "note": "host buffers in and out (PCIe-inclusive), synchronous, weights cached on the device"}


def cpu_baseline(layers, tag, unit, budget_s=12.0):
    """the reference's x86 kernels (or the CPU restatement) on a bounded sample: passes over the same layer
    shapes at batch 1 (the reference evaluates one image per call), 8 threads as the reference builds"""
    from onenew_amd import ops
    from oracle import oracle
    threads = 8
    os.environ.setdefault("OMP_NUM_THREADS", str(threads))
    oracle.set_threads(threads)
    runs = [L.cpu_runner(ops, oracle, tag) for L in layers]
    flops = sum(f for f, _ in runs)
    for _, f in runs:
        f()                      # warm-up pass
    times = []
    t_start = time.perf_counter()
    # about budget_s seconds of CPU work, at least 10 and at most 2000 passes
    while len(times) < 2000 and (time.perf_counter() - t_start < budget_s or len(times) < 10):
        t0 = time.perf_counter()
        for _, f in runs:
            f()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(flops / med / 1e12, 5), "unit": unit, "cores": threads,
            "kind": "reference" if oracle.have_ref() else "port",
            "sample": f"{len(times)} passes over the {len(runs)} layer shapes, one image per call, median; "
                      f"{med * 1e3:.1f} ms per pass",
            "ms_per_pass": round(med * 1e3, 2), "host_cpus": os.cpu_count()}


def bench_net(torch, args):
    print(json.dumps(net_result(torch, args.workload, args.steps, args.warmup, not args.no_cpu)))


def net_result(torch, workload, steps, warmup, with_cpu):
    """A whole model (ResNet-50: 53 Conv, MaxPool, 16 Add, 16 Relu, GlobalAveragePool, Gemm; MobileNetV2: 52 Conv of
    which 17 depthwise, 10 Add, GlobalAveragePool, Gemm; ViT-Tiny: patch Conv, 12 encoder blocks of LayerNormalization /
    MatMul / Add / Transpose / Softmax / Gelu, mean over the tokens, Gemm) as a .one file through the device-resident runtime
    (libonenew_rt.so): every operator back to back on the device, input and output in device memory.  A step is one
    inference of the batch."""
    from onenew_amd import rt, stacks
    n = int(workload.split("_b")[1])
    model = "ResNet-50" if workload.startswith("resnet50") else "MobileNetV2" if workload.startswith("mobilenetv2") else "ViT-Tiny"
    make = {"ResNet-50": stacks.resnet50_model, "MobileNetV2": stacks.mobilenet_v2_model, "ViT-Tiny": stacks.vit_tiny_model}[model]
    int8 = "_int8_net_" in workload   # every convolution in the W8A32 form the offline quantiser writes
    data, in_shape, flops = make(n)
    x = torch.randn(in_shape, dtype=torch.float32, device="cuda")
    calibration = None
    if int8:
        # the model-level quantisation step on the fp32 file (tools/optimize/model_quant.hpp:625-679): activation scales
        # from the KL search over two calibration batches drawn like the input, weights / bias / weight_aux per channel
        g = torch.Generator(device="cuda")
        g.manual_seed(1234)
        cal = [torch.randn(in_shape, generator=g, dtype=torch.float32, device="cuda") for _ in range(2)]
        t0 = time.perf_counter()
        data = rt.quantise(data, [c.data_ptr() for c in cal], rt.QUANT_KL)
        calibration = {"method": "KL", "batches": len(cal), "seconds": round(time.perf_counter() - t0, 2)}
        del cal
    net = rt.Net(data)
    y = torch.empty((n, 1000), dtype=torch.float32, device="cuda")
    net.run_raw([x.data_ptr()], [y.data_ptr()])   # the input goes into the net's own input buffer, the logits come back
    # From here on the batch is where the first operator reads it and the logits stay where the last one writes them (the
    # runtime copies nothing when it is handed its own buffers): a caller that produces its batch on the device writes it
    # there directly.  The logits of the copying run above are kept to check the others against.
    (_, in_dev), (_, out_dev) = net.operand(net.inputs[0][0]), net.operand(net.outputs[0][0])
    ins, outs = [in_dev], [out_dev]
    for _ in range(max(2, warmup)):     # the first inferences measure tile choices and pack the weights
        net.run_raw(ins, outs)
    torch.cuda.synchronize()
    logits = torch.from_numpy(net.fetch(net.outputs[0][0]).reshape(n, 1000)).cuda()
    if not torch.equal(logits, y):
        raise SystemExit(f"{workload}: the logits in the net's own buffer differ from those of the run that copied them out")
    t0 = time.perf_counter()
    for _ in range(steps):
        net.enqueue_raw(ins, outs)      # one batch after the other, no host wait in between: throughput, as the stacks are timed
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    if not torch.equal(torch.from_numpy(net.fetch(net.outputs[0][0]).reshape(n, 1000)).cuda(), y):
        raise SystemExit(f"{workload}: the logits after the queued inferences differ from those of the first run")
    # device time of one inference: events around it on the default stream, where the plugins launch
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    dev_ms = []
    for _ in range(max(5, steps)):
        e0.record(torch.cuda.default_stream())
        net.run_raw(ins, outs)
        e1.record(torch.cuda.default_stream())
        e1.synchronize()
        dev_ms.append(e0.elapsed_time(e1))
    dev = float(np.median(dev_ms))
    ops = net.ops()
    cpu = None
    if with_cpu:
        from oracle import one_model
        if one_model.have_ref_runner():
            data1, shape1, flops1 = make(1)
            xin = np.random.default_rng(0).normal(size=shape1).astype(np.float32)
            ms = one_model.time_reference(data1, [xin], repeats=40)
            cpu = {"value": round(flops1 / (ms * 1e-3) / 1e12, 5), "unit": "TFLOP/s", "cores": 8, "kind": "reference",
                   "sample": f"40 inferences of the same model at batch 1 through the reference's host operator classes "
                             f"and x86 kernels, median {ms:.2f} ms", "ms_per_inference": round(ms, 3)}
    line = {"metric": f"{workload.split('_net_')[0]}_net_{'w8a32_tops' if int8 else 'fp32_tflops'}", "value": round(flops / (ms_per_step * 1e-3) / 1e12, 3), "unit": "TOP/s" if int8 else "TFLOP/s",
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8" if int8 else "f32", "data": "synthetic",
            "config": {"workload": f"{model} .one model {'W8A32 (int8 weights and activations, int32 accumulate; ' + str(net.int8_links()) + ' operands between convolutions travel as int8)' if int8 else 'fp32'}, batch {n}, 224x224, {len(ops)} operators through the "
                                   f"device-resident runtime, input and logits in HBM (the runtime's own buffers: nothing is copied)", "operators": len(ops),
                       "ops_per_step": flops, "model_bytes": len(data)},
            "roofline": {"kernel": "whole inference: every operator of the graph on the default stream", "bound": "mfma",
                         "achieved": round(flops / (dev * 1e-3) / 1e12, 3), "peak": PEAK["i8" if int8 else "f32"], "unit": "TOP/s" if int8 else "TFLOP/s",
                         "frac": round(flops / (dev * 1e-3) / 1e12 / PEAK["i8" if int8 else "f32"], 4), "traffic": None,
                         "launches": len(ops), "device_ms_per_inference": round(dev, 4)},
            "cpu_baseline": cpu, "images_per_s": round(n / (ms_per_step * 1e-3), 1)}
    if calibration:
        line["calibration"] = calibration
    net.close()
    return line


METRIC = {"resnet50_glue": "resnet50_glue_ops_fp32_tflops", "vit_tiny_glue": "vit_tiny_glue_ops_fp32_tflops",
          "resnet50": "resnet50_conv_stack_{dtype}_tflops", "mobilenetv2": "mobilenetv2_conv_stack_fp32_tflops",
          "yolov8s_int8chain": "yolov8s_conv_stack_w8a8_tops", "yolov8s": "yolov8s_conv_stack_w8a32_tops",
          "vit": "vit_tiny_matmul_{dtype}_tflops", "cfg1": "conv2d_relu_{dtype}_tflops"}

# the other configurations of the benchmark, timed after the headline one in a default run
NET_CONFIGS = ["resnet50_net_b32", "resnet50_int8_net_b32", "mobilenetv2_net_b64", "mobilenetv2_int8_net_b64", "vit_tiny_net_b64"]
OTHER_CONFIGS = ["cfg1", "cfg1_bf16", "resnet50_b1", "resnet50_b32_bf16", "mobilenetv2_b64", "mobilenetv2_b1", "vit_tiny_b64", "vit_tiny_b64_bf16", "vit_tiny_b1",
                 "yolov8s_int8_b16", "yolov8s_int8chain_b16", "yolov8s_int8chain_b1"]


def run_workload(torch, hip, name, steps, warmup, layers_table=False, graph=True):
    """times one workload: `warmup` untimed passes (tile choices are measured there when tuning is on), `steps` timed
    passes between two device synchronisations, then every layer on its own with HIP events on the launch stream"""
    desc, dtype, layers = make_workload(torch, hip, name)
    unit = "TOP/s" if dtype == "i8" else "TFLOP/s"
    flops = sum(L.flops for L in layers)
    abytes = sum(L.bytes for L in layers)           # what the launches of a pass have to move (fused launches: their own tensors)

    for _ in range(warmup):
        for L in layers:
            L.launch(hip)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        for L in layers:
            L.launch(hip)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    eager_ms = wall * 1e3 / steps
    ms_per_step, launch_mode = eager_ms, "one launch per layer from the host"
    # The same pass recorded once into a HIP graph and replayed: where the layers are shorter than the host needs to queue
    # one (about 7 us through this Python binding), the device otherwise idles between them.  The replayed pass is the
    # same launches with the same tile choices (made during the warm-up); its last layer's output is compared with the
    # eager pass before the figure is used.
    if graph:
        try:
            outs = [getattr(L, "yq", None) if getattr(L, "yq", None) is not None else L.y for L in layers]
            want = outs[-1].clone()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for L in layers:
                    L.launch(hip)
            for _ in range(2):
                g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                g.replay()
            torch.cuda.synchronize()
            graph_ms = (time.perf_counter() - t0) * 1e3 / steps
            same = bool(torch.equal(outs[-1], want))
            if same and graph_ms < eager_ms:
                ms_per_step, launch_mode = graph_ms, "one HIP graph replay per pass (the layers' launches recorded once)"
            elif not same:
                print(f"[bench] {name}: graph replay differs from the eager pass; eager timing kept", file=sys.stderr)
            del g
        except Exception as e:   # capture refused (e.g. an allocation inside a launch): the eager figure stands
            print(f"[bench] {name}: no graph replay ({type(e).__name__}: {e})", file=sys.stderr)
            torch.cuda.synchronize()

    # Roofline of the dominant kernel.  Dense layers all run onhip::igemm_kernel (MFMA-bound); depthwise layers run
    # onhip::depthwise_*_kernel (HBM-bound).  Whichever group takes more time is reported: algorithmic work of its
    # launches / their average durations, from events on the launch stream.
    per_layer_ms = time_layers(torch, hip, layers, reps=max(10, steps))
    groups = {True: [], False: []}
    for L, t in zip(layers, per_layer_ms):
        groups[L.dense].append((L, t))
    dom_dense = sum(t for _, t in groups[True]) >= sum(t for _, t in groups[False])
    grp = groups[dom_dense]
    g_ms = sum(t for _, t in grp)
    g_flops, g_bytes = sum(L.flops for L, _ in grp), sum(L.bytes for L, _ in grp)
    g_chain_bytes = sum(getattr(L, "chain_bytes", L.bytes) for L, _ in grp)
    kernel = ("onhip::igemm_dma_kernel (operand tiles straight into LDS, 16-bit storage, MFMA implicit GEMM)"
              if dom_dense and grp[0][0].kind in ("conv_h16", "linear_h16") else
              f"onhip::igemm_kernel ({dtype} MFMA implicit GEMM)" if dom_dense else
              "element-wise / pooling / normalisation kernels (elementwise.hip, vit_glue.hip)" if grp[0][0].kind == "glue"
              else "onhip::irblock_f32_kernel (expansion + depthwise + projection in one launch) and onhip::depthwise_tiled_kernel"
              if any(L.kind == "ir_block" for L, _ in grp) else "onhip::depthwise_tiled_kernel")
    # the bound is the roof the group's arithmetic intensity puts it under
    mfma_bound = dom_dense and g_flops / g_bytes >= PEAK[dtype] * 1e12 / (HBM_PEAK_GBS * 1e9)
    if mfma_bound:
        achieved, peak, r_unit, work = g_flops / (g_ms * 1e-3) / 1e12, PEAK[dtype], unit, g_flops
        step_frac = flops / (ms_per_step * 1e-3) / 1e12 / peak
    else:
        achieved, peak, r_unit, work = g_bytes / (g_ms * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s", g_bytes
        step_frac = abytes / (ms_per_step * 1e-3) / 1e9 / peak
    group = "igemm" if dom_dense else "glue" if grp[0][0].kind == "glue" else "depthwise"
    traffic = measured_traffic(name, group)
    roofline = {"kernel": kernel, "bound": "mfma" if mfma_bound else "hbm", "achieved": round(achieved, 3),
                "peak": peak, "unit": r_unit, "frac": round(achieved / peak, 4),
                "traffic": traffic,
                "traffic_source": None if traffic is None else
                f"profiles/{name}_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload, summarised by "
                f"onenew_amd/profile_summary.py; a committed figure, not measured in this run)",
                "launches": len(grp), "avg_launch_ms": round(g_ms / len(grp), 5),
                "work_per_launch": work / len(grp),
                "arithmetic_intensity": round(g_flops / g_bytes, 2),
                # the same fraction from the wall time of the timed passes (layers back to back, cold caches between them)
                "frac_whole_step": round(step_frac, 4)}
    if g_chain_bytes != g_bytes and not mfma_bound:
        # launches that replace a chain of operators: `achieved` / `frac` count the bytes those launches themselves move;
        # this is the rate at which the bytes of the chains they replace would have had to move in the same time
        roofline["unfused_chain_equivalent"] = {"achieved": round(g_chain_bytes / (g_ms * 1e-3) / 1e9, 3), "unit": "GB/s",
                                                "frac": round(g_chain_bytes / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                                "bytes_per_launch": g_chain_bytes / len(grp)}
    res = {"name": name, "desc": desc, "dtype": dtype, "unit": unit, "flops": flops, "abytes": abytes,
           "ms_per_step": ms_per_step, "eager_ms_per_step": eager_ms, "launch": launch_mode, "per_layer_ms": per_layer_ms,
           "roofline": roofline, "layers": layers,
           "value": flops / (ms_per_step * 1e-3) / 1e12}
    if layers_table:
        print(f"{'layer':<18}{'shape':<32}{'ms':>9}{unit:>9}{'%mfma':>7}{'GB/s':>8}{'%hbm':>6}", file=sys.stderr)
        for L, t in zip(layers, per_layer_ms):
            tf = L.flops / (t * 1e-3) / 1e12
            gb = L.bytes / (t * 1e-3) / 1e9
            print(f"{L.name:<18}{L.shape:<32}{t:>9.4f}{tf:>9.2f}{100 * tf / PEAK[dtype]:>7.1f}{gb:>8.0f}"
                  f"{100 * gb / HBM_PEAK_GBS:>6.1f}", file=sys.stderr)
    return res


def config_summary(res):
    """the short form of a workload's result for the `configs` array of the headline line"""
    rf = res["roofline"]
    per = res["per_layer_ms"]
    out = {"workload": res["name"], "what": res["desc"], "dtype": res["dtype"], "value": round(res["value"], 3), "unit": res["unit"],
           "ms_per_step": round(res["ms_per_step"], 4), "launch": res["launch"], "eager_ms_per_step": round(res["eager_ms_per_step"], 4),
           "ms_sum_of_layers": round(sum(per), 4), "layers": len(per),
           "roofline": {k: rf[k] for k in ("bound", "achieved", "peak", "unit", "frac", "frac_whole_step", "avg_launch_ms", "launches", "traffic",
                                           "unfused_chain_equivalent") if k in rf},
           "algorithmic_GBps": round(res["abytes"] / (res["ms_per_step"] * 1e-3) / 1e9, 1),
           "hbm_frac_whole_step": round(res["abytes"] / (res["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    lowai = [(L, t) for L, t in zip(res["layers"], per) if not L.dense]
    if lowai:
        out["depthwise_GBps"] = round(sum(L.bytes for L, _ in lowai) / (sum(t for _, t in lowai) * 1e-3) / 1e9, 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="resnet50_b32")
    ap.add_argument("--layers", action="store_true", help="also print a per-layer table on stderr")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-tune", action="store_true", help="use the cost model instead of measured tile choice")
    ap.add_argument("--no-batch1", action="store_true", help="skip the extra batch-1 pass over the same stack")
    ap.add_argument("--only", action="store_true", help="time the named workload only, not the other configurations after it")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only, no HIP graph replay of the pass")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the path runs on a single MI355X and nothing in this build "
                         "uses a second one; run with --gpus 1")
    import torch
    from onenew_amd import hip
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    hip.init(0)
    # tile / split-K per layer shape is measured on first use (during the warm-up steps) and cached
    hip.set_tuning(0 if args.no_tune else 1)

    if args.workload == "copy":
        # yardstick for the HBM traffic counters: a plain device copy of known size (1 GiB read + 1 GiB written)
        src = torch.rand(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            hip.copy_f32(src, dst)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "copy", "bytes_read_per_launch": src.numel() * 4,
                          "bytes_written_per_launch": src.numel() * 4, "launches": args.warmup + args.steps}))
        return

    if args.workload.startswith(("resnet50_net_b", "resnet50_int8_net_b", "mobilenetv2_net_b", "mobilenetv2_int8_net_b", "vit_tiny_net_b")):
        return bench_net(torch, args)

    res = run_workload(torch, hip, args.workload, args.steps, args.warmup, layers_table=args.layers, graph=not args.no_graph)
    layers, per_layer_ms, dtype, unit = res["layers"], res["per_layer_ms"], res["dtype"], res["unit"]

    extra = {"launch": res["launch"], "eager_ms_per_step": round(res["eager_ms_per_step"], 4),
             "tuning": "cost model only" if args.no_tune else
             "tile and split-K measured once per layer shape during the warm-up passes (onhip_set_tuning(1)); the library's "
             "default is the cost model"}
    if not args.no_tune and args.workload == "resnet50_b32" and not args.only:
        # the same stack with the choices a host gets by default: the cost model, nothing measured
        hip.set_tuning(0)
        for _ in range(2):
            for L in layers:
                L.launch(hip)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            for L in layers:
                L.launch(hip)
        torch.cuda.synchronize()
        ms_model = (time.perf_counter() - t0) * 1e3 / args.steps
        hip.set_tuning(1)
        extra["cost_model_choices"] = {"ms_per_step": round(ms_model, 4), "value": round(res["flops"] / (ms_model * 1e-3) / 1e12, 3)}
    if args.workload.startswith("resnet50_b") and args.workload != "resnet50_b1" and not args.no_batch1:
        # the same stack at batch 1 (the "conv stack ms" of the reference's recorded trace)
        _, _, layers1 = make_workload(torch, hip, "resnet50_b1")
        ms1 = time_layers(torch, hip, layers1, reps=20)
        extra["resnet50_conv_stack_ms_batch1"] = round(sum(ms1), 4)
        del layers1
    if args.workload.startswith("resnet50_b") or args.workload == "cfg1":
        extra["plugin_eval_cfg1"] = plugin_eval_latency(hip)
    extra["stack_ms_sum_of_layers"] = round(sum(per_layer_ms), 4)
    extra["algorithmic_GBps"] = round(res["abytes"] / (sum(per_layer_ms) * 1e-3) / 1e9, 1)
    lowai = [(L, t) for L, t in zip(layers, per_layer_ms) if not L.dense]
    if lowai:
        extra["depthwise_GBps"] = round(sum(L.bytes for L, _ in lowai) / (sum(t for _, t in lowai) * 1e-3) / 1e9, 1)
        extra["depthwise_ms"] = round(sum(t for _, t in lowai), 4)

    cpu = None if args.no_cpu else cpu_baseline(layers, args.workload, unit)

    key = next(k for k in METRIC if args.workload.startswith(k))
    line = {"metric": METRIC[key].format(dtype="fp32" if dtype == "f32" and "{dtype}_tflops" in METRIC[key] and key != "vit" else dtype), "value": round(res["value"], 3), "unit": unit, "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(res["ms_per_step"], 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
            "config": {"workload": res["desc"], "layers": len(layers), "ops_per_step": res["flops"],
                       "algorithmic_bytes_per_step": res["abytes"]},
            "roofline": res["roofline"], "cpu_baseline": cpu}
    line.update(extra)

    if args.workload == "resnet50_b32" and not args.only:
        # every other configuration of the benchmark, each timed the same way (fewer passes), as extra keys
        del layers, res, lowai
        configs = []
        for name in OTHER_CONFIGS:
            torch.cuda.empty_cache()
            t0 = time.perf_counter()
            r = run_workload(torch, hip, name, steps=10, warmup=3, graph=not args.no_graph)
            c = config_summary(r)
            c["bench_seconds"] = round(time.perf_counter() - t0, 1)
            configs.append(c)
            print(f"[bench] {name}: {c['value']} {c['unit']}, {c['ms_per_step']} ms per step, roofline {c['roofline']['bound']} "
                  f"{c['roofline']['frac']}", file=sys.stderr, flush=True)
            del r
        # whole models as .one files through the device-resident runtime (fewer inferences, no CPU leg)
        for name in NET_CONFIGS:
            torch.cuda.empty_cache()
            t0 = time.perf_counter()
            r = net_result(torch, name, steps=10, warmup=3, with_cpu=False)
            c = {"workload": name, "what": r["config"]["workload"], "dtype": r["dtype"], "value": r["value"], "unit": r["unit"],
                 "ms_per_step": r["ms_per_step"], "images_per_s": r["images_per_s"], "operators": r["config"]["operators"],
                 "device_ms_per_inference": r["roofline"]["device_ms_per_inference"], "bench_seconds": round(time.perf_counter() - t0, 1)}
            configs.append(c)
            print(f"[bench] {name}: {c['value']} {c['unit']}, {c['ms_per_step']} ms per inference of the batch", file=sys.stderr, flush=True)
        line["configs"] = configs
    print(json.dumps(line))


if __name__ == "__main__":
    main()
