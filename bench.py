#!/usr/bin/env python3
"""Benchmark of the Conv / MatMul / Gemm hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50_b32] [--layers]

A step is one pass over every layer of the workload: one launch per layer, inputs, weights and
outputs resident in HBM, synthetic seeded data (x ~ U(-1,1), He-normal weights, bias N(0, 0.01)).
Prints ONE JSON line: whole-stack throughput (`value`, TFLOP/s with 2 FLOP per multiply-accumulate,
bias and activation not counted), the roofline position of the dominant kernel measured with HIP
events on the launch stream, and the CPU baseline (the reference's own x86 kernels when their
build is present, else the CPU restatement) timed on this machine's host cores.
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


def make_workload(name):
    """-> (description, dtype, [(layer name, ConvDesc)])"""
    from onenew_amd import stacks
    if name.startswith("resnet50_b"):
        n = int(name.split("_b")[1])
        return f"ResNet-50 conv stack fp32, batch {n}, 224x224, 53 conv layers, fused ReLU", "f32", \
            stacks.with_batch(stacks.resnet50(), n)
    if name.startswith("mobilenetv2_b"):
        n = int(name.split("_b")[1])
        return f"MobileNetV2 conv stack fp32, batch {n}, 224x224, 52 conv layers", "f32", \
            stacks.with_batch(stacks.mobilenet_v2(), n)
    if name == "cfg1":
        import cases
        return "Conv2d+ReLU fp32 64->64 56x56 3x3 s1 p1, batch 1", "f32", [("cfg1", cases.conv_f32_cases()["cfg1_64x56_3x3"])]
    raise SystemExit(f"unknown workload {name}")


class DeviceLayer:
    """device-resident operands of one layer"""

    def __init__(self, torch, name, d, seed_tag):
        import cases
        x, w, b = cases.conv_inputs(f"{seed_tag}/{name}", d)
        self.name, self.d = name, d
        self.x, self.w, self.b = (torch.from_numpy(t).cuda() for t in (x, w, b))
        oh, ow = d.out_hw()
        self.y = torch.empty((d.n, d.cout, oh, ow), dtype=torch.float32, device="cuda")
        # weights are re-laid out once at load time (tap-major), as an inference runtime would
        from onenew_amd import hip
        self.wp = hip.pack_conv_weights(d, self.w)

    def launch(self, hip):
        if self.wp is not None:
            hip.conv2d_f32(self.d, self.x, self.wp, self.b, None, out=self.y, packed=True)
        else:
            hip.conv2d_f32(self.d, self.x, self.w, self.b, None, out=self.y)


def measured_traffic(workload):
    """HBM bytes per launch of the dominant kernel from the committed counter summary
    (profiles/<workload>_traffic.json: FETCH_SIZE / WRITE_SIZE scaled by the copy yardstick), else None"""
    path = os.path.join(ROOT, "profiles", f"{workload}_traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f).get("hbm_bytes_per_launch")


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


def cpu_baseline(layer_descs, seed_tag, budget_s=20.0):
    """the reference's x86 kernels (or the CPU restatement) on a bounded sample: batch-1 passes over the
    same layer shapes, 8 threads as the reference builds by default"""
    import cases
    from onenew_amd import abi, ops
    from oracle import oracle
    threads = 8
    os.environ.setdefault("OMP_NUM_THREADS", str(threads))
    use_ref = oracle.have_ref()
    oracle.set_threads(threads)
    runs = []
    for name, d in layer_descs:
        d1 = abi.ConvDesc.from_buffer_copy(d)
        d1.n = 1
        x, w, b = cases.conv_inputs(f"{seed_tag}/cpu/{name}", d1)
        if use_ref:
            op = ops.Conv(ops.Plugin(oracle.ref_path("Conv")).eval, d1, w, b, scratch_bytes=oracle.ref_scratch_bytes(d1))
            xin = ops.aligned_empty(x.shape)
            xin[...] = x
            out = ops.aligned_empty((1, d1.cout) + d1.out_hw())
            runs.append((d1, lambda op=op, xin=xin, out=out: op(xin, out=out)))
        else:
            runs.append((d1, lambda d1=d1, x=x, w=w, b=b: oracle.conv2d_f32(d1, x, w, b)))
    flops = sum(d1.flops() for d1, _ in runs)
    for _, f in runs:
        f()                      # warm-up pass
    times = []
    t_start = time.perf_counter()
    while len(times) < 10 and (time.perf_counter() - t_start < budget_s or len(times) < 2):
        t0 = time.perf_counter()
        for _, f in runs:
            f()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(flops / med / 1e12, 5), "unit": "TFLOP/s", "cores": threads,
            "kind": "reference" if use_ref else "port",
            "sample": f"{len(times)} batch-1 passes over the {len(runs)} layer shapes, median; {med * 1e3:.1f} ms per pass",
            "ms_per_pass": round(med * 1e3, 2), "host_cpus": os.cpu_count()}


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

    desc, dtype, layer_descs = make_workload(args.workload)
    layers = [DeviceLayer(torch, n, d, args.workload) for n, d in layer_descs]
    flops = sum(L.d.flops() for L in layers)
    abytes = sum(L.d.algorithmic_bytes() for L in layers)

    for _ in range(args.warmup):
        for L in layers:
            L.launch(hip)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        for L in layers:
            L.launch(hip)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # roofline of the dominant kernel (the implicit-GEMM MFMA kernel runs every dense layer):
    # algorithmic FLOPs of its launches / their average durations, from events on the launch stream
    per_layer_ms = time_layers(torch, hip, layers, reps=max(10, args.steps))
    dense = [(L, t) for L, t in zip(layers, per_layer_ms) if L.d.group == 1]
    dense_flops = sum(L.d.flops() for L, _ in dense)
    dense_ms = sum(t for _, t in dense)
    achieved = dense_flops / (dense_ms * 1e-3) / 1e12
    roofline = {"kernel": "onhip::igemm_kernel (fp32 MFMA implicit GEMM)", "bound": "mfma",
                "achieved": round(achieved, 3), "peak": PEAK[dtype], "unit": "TFLOP/s",
                "frac": round(achieved / PEAK[dtype], 4), "traffic": measured_traffic(args.workload),
                "launches": len(dense), "avg_launch_ms": round(dense_ms / len(dense), 5),
                "flops_per_launch": dense_flops / len(dense)}

    extra = {}
    if args.workload.startswith("resnet50_b") and args.workload != "resnet50_b1" and not args.no_batch1:
        # the same stack at batch 1 (the "conv stack ms" of the reference's recorded trace)
        _, _, l1 = make_workload("resnet50_b1")
        layers1 = [DeviceLayer(torch, n, d, "resnet50_b1") for n, d in l1]
        ms1 = time_layers(torch, hip, layers1, reps=20)
        extra["resnet50_conv_stack_ms_batch1"] = round(sum(ms1), 4)
    extra["conv_stack_ms_sum_of_layers"] = round(sum(per_layer_ms), 4)
    extra["algorithmic_GBps"] = round(abytes / (sum(per_layer_ms) * 1e-3) / 1e9, 1)

    if args.layers:
        print(f"{'layer':<18}{'M':>6}{'N':>9}{'K':>6}{'ms':>9}{'TFLOP/s':>9}{'%mfma':>7}{'GB/s':>8}", file=sys.stderr)
        for L, t in zip(layers, per_layer_ms):
            d = L.d
            oh, ow = d.out_hw()
            tf = d.flops() / (t * 1e-3) / 1e12
            print(f"{L.name:<18}{d.cout:>6}{d.n * oh * ow:>9}{d.k_per_out():>6}{t:>9.4f}{tf:>9.2f}"
                  f"{100 * tf / PEAK[dtype]:>7.1f}{d.algorithmic_bytes() / (t * 1e-3) / 1e9:>8.0f}", file=sys.stderr)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(layer_descs, args.workload)

    line = {"metric": "resnet50_conv_stack_fp32_tflops" if args.workload.startswith("resnet50") else
            f"{args.workload}_tflops",
            "value": round(flops / (ms_per_step * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
            "config": {"workload": desc, "layers": len(layers), "flops_per_step": flops,
                       "algorithmic_bytes_per_step": abytes},
            "roofline": roofline, "cpu_baseline": cpu}
    line.update(extra)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
