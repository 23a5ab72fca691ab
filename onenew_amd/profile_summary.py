"""Reduces the raw rocprofv3 output of a benchmark workload to the short summaries kept under profiles/.

    python -m onenew_amd.profile_summary <workload> --raw DIR [--out DIR]

DIR holds what the commands below wrote on the MI355X box; every command runs
committed files only.  With TMPDIR=/tmp, from a scratch directory, $R the repository root and $W the workload:

    export ONHIP_TUNE_CACHE=/tmp/tune_$W.txt      # tile / split-K choices measured once, reused by the traced runs
    python3 $R/bench.py --workload $W --only --no-graph --steps 2 --warmup 1 --no-cpu --no-batch1         # fills the cache
    rocprofv3 --kernel-trace --stats -d kt -o kt --output-format csv -- \\
        python3 $R/bench.py --workload $W --only --no-graph --steps 20 --warmup 5 --no-cpu --no-batch1 > bench_under_trace.json
    rocprofv3 --pmc FETCH_SIZE -d f -o pmc --output-format csv -- python3 $R/bench.py --workload $W --only --no-graph --steps 3 --warmup 1 --no-cpu --no-batch1
    rocprofv3 --pmc WRITE_SIZE -d w -o pmc --output-format csv -- python3 $R/bench.py --workload $W --only --no-graph --steps 3 --warmup 1 --no-cpu --no-batch1
    rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_WAIT_ANY \\
        -d sq -o pmc --output-format csv -- python3 $R/bench.py --workload $W --only --no-graph --steps 3 --warmup 1 --no-cpu --no-batch1
    rocprofv3 --pmc FETCH_SIZE -d cf -o pmc --output-format csv -- python3 $R/bench.py --workload copy --steps 3 --warmup 1
    rocprofv3 --pmc WRITE_SIZE -d cw -o pmc --output-format csv -- python3 $R/bench.py --workload copy --steps 3 --warmup 1

and DIR the files kt_kernel_stats.csv, bench_under_trace.json, pmc_FETCH_SIZE.csv, pmc_WRITE_SIZE.csv, pmc_SQ.csv,
pmc_copy_FETCH_SIZE.csv, pmc_copy_WRITE_SIZE.csv (the *_counter_collection.csv of each run under those names).

Written: profiles/<workload>_kernels.md (kernel statistics, HBM traffic per launch scaled by the copy yardstick, MFMA and
LDS counters) and profiles/<workload>_traffic.json (the figure bench.py quotes as roofline.traffic).
"""
import argparse
import collections
import csv
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SIMDS = 256 * 4            # MI355X: 256 compute units of 4 SIMDs
CLOCK_HZ = 2.4e9           # peak engine clock the MFMA peak is quoted at
GLUE = ("add_kernel", "relu_kernel", "maxpool", "gap_kernel", "layernorm", "softmax", "transpose_kernel", "gelu_lut")
LEGEND = ("Kernel names: `onhip::igemm_kernel<dtype, loader, BM, BN, WM, WN, PF, RES, PW2>` (dtype 0 fp32, 1 bf16, 2 f16, 3 int8; loader 0 "
          "gather, 1 int8 vectors, 2 plain, 3 tap-major packed, 4 int8 vectors with scalar taps; PF register sets of tiles in flight; "
          "RES the variant whose store adds a residual operand; PW2 the variant that multiplies its finished tile by a second, 1x1 weight "
          "matrix before storing: a convolution and the 1x1 convolution after it in one launch), `onhip::igemm_dma_kernel<dtype, BM, BN, WM, WN, KS, NST>` (int8 and "
          "16-bit storage: operand tiles loaded straight into LDS, KS bytes of K per stage, ring of NST stages), `onhip::rowb_f32_kernel<WM, WN>` (fp32, B "
          "straight from memory, tile 32 WM x 128 WN), `onhip::splitk_finish_kernel`, `onhip::depthwise_tiled_kernel<int8, stride, "
          "act>`, `onhip::quantize_nhwc_kernel<CBW>`, `onhip::stem_f32_kernel<filter size, act, two row tiles>` (first-layer "
          "convolutions from an LDS patch), `onhip::i8patch_kernel<bytes per pixel, WM, pixel tiles>` and `onhip::i8direct_kernel<bytes per pixel, taps, WM, TM, pixel "
          "tiles, workgroups per CU>` (int8 chain form, 3x3 with few channels: input rows in LDS / windows loaded per tap), `onhip::attention_f32_kernel<16-key tiles, head dim>`, `onhip::dw_s8_nhwc_kernel<3x3 stride, epilogue, fp32 out>` (depthwise on int8 NHWC), `onhip::irblock_f32_kernel<act, input channels / 4, row tiles, "
          "patches>` (1x1 expansion + depthwise 3x3 + 1x1 projection in one launch), and the element-wise kernels.")


def short(name):
    name = name.replace("void ", "").replace("onhip::", "")
    i = name.find("(")
    return name[:i] if i > 0 else name


def family(name):
    if "_pack_kernel" in name:   # weight re-layouts: once per model, not part of a pass
        return None
    if "igemm" in name or "splitk_finish" in name or "rowb_f32" in name or "attention" in name or "stem_f32" in name or "i8patch" in name or "i8direct" in name:
        return "igemm"
    if "depthwise" in name or "irblock" in name or "dw_s8" in name:
        return "depthwise"
    if "quantize_nhwc" in name:
        return "quantize"
    if any(g in name for g in GLUE):
        return "glue"
    return None


def counters(path):
    """kernel -> counter -> list of per-dispatch values"""
    out = collections.defaultdict(lambda: collections.defaultdict(list))
    if not os.path.exists(path):
        return out
    for r in csv.DictReader(open(path)):
        out[short(r["Kernel_Name"])][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return out


def mean(v):
    return sum(v) / len(v) if v else 0.0


def summarise(workload, raw, out_dir):
    bench = json.load(open(os.path.join(raw, "bench_under_trace.json")))
    stats = list(csv.DictReader(open(os.path.join(raw, "kt_kernel_stats.csv"))))
    fetch, write = counters(os.path.join(raw, "pmc_FETCH_SIZE.csv")), counters(os.path.join(raw, "pmc_WRITE_SIZE.csv"))
    cfetch, cwrite = counters(os.path.join(raw, "pmc_copy_FETCH_SIZE.csv")), counters(os.path.join(raw, "pmc_copy_WRITE_SIZE.csv"))
    sq = counters(os.path.join(raw, "pmc_SQ.csv"))
    copy_f = [mean(c["FETCH_SIZE"]) for k, c in cfetch.items() if "copy_f32" in k]
    copy_w = [mean(c["WRITE_SIZE"]) for k, c in cwrite.items() if "copy_f32" in k]
    L = [f"# rocprofv3 summary: {bench['config']['workload']}\n",
         f"Workload `{workload}` of `bench.py`. {LEGEND}\n",
         "Commands and the reduction to this file: the docstring of `onenew_amd/profile_summary.py` (run as "
         f"`python -m onenew_amd.profile_summary {workload} --raw <raw files>`).\n",
         "## Kernel statistics (`--kernel-trace --stats`)\n",
         "| kernel | calls | total ms | average us | % | min us | max us |\n|---|---:|---:|---:|---:|---:|---:|"]
    dur_us = {}
    for r in stats:
        n = short(r["Name"])
        dur_us[n] = float(r["AverageNs"]) / 1e3
        if float(r["Percentage"]) < 0.05:
            continue
        L.append(f"| `{n}` | {r['Calls']} | {float(r['TotalDurationNs']) / 1e6:.3f} | {float(r['AverageNs']) / 1e3:.2f} | "
                 f"{float(r['Percentage']):.2f} | {float(r['MinNs']) / 1e3:.2f} | {float(r['MaxNs']) / 1e3:.2f} |")
    whole_model = "layers" not in bench["config"]      # a .one file through the runtime: one timed loop, no per-layer timing
    passes = bench["warmup"] + bench["steps"] + (0 if whole_model else 3 + max(10, bench["steps"]))
    nl = bench["config"].get("layers", bench["config"].get("operators"))
    groups = collections.defaultdict(list)
    for r in stats:
        fam = family(r["Name"])
        if fam:
            groups[fam].append(r)
    L.append("")
    if whole_model:
        # the operator that runs once per inference has the fewest calls: that count is the number of inferences traced
        # (warm-up, timed steps, and the runs bench.py makes before them to fill the tile cache and check the outputs)
        passes = min([int(r["Calls"]) for rs in groups.values() for r in rs if "splitk_finish" not in r["Name"]] or [passes])
        L.append(f"The traced run makes {passes} inferences of the {nl} operators ({bench['warmup']} warm-up + {bench['steps']} timed, the rest "
                 f"before them: tile choices, output checks).")
    else:
        L.append(f"The traced run makes {passes} passes over the {nl} layers ({bench['warmup']} warm-up + {bench['steps']} timed steps, then "
                 f"3 + {max(10, bench['steps'])} per layer for the event-timed roofline figures), plus the launches that measure tile choices "
                 f"where the cache did not have them.")
    for g, rs in groups.items():
        ns = sum(float(r["TotalDurationNs"]) for r in rs)
        main = sum(int(r["Calls"]) for r in rs if "splitk_finish" not in r["Name"])
        L.append(f"- {g}: {main} layer launches, {ns / 1e6:.3f} ms in total (split-K reduction included) = "
                 f"**{ns / main / 1e3:.2f} us per layer launch**, {ns / passes / 1e6:.4f} ms per pass.")
    rf = bench["roofline"]
    if whole_model:
        L.append(f"- `bench.py` in the same run: {bench['ms_per_step']} ms per inference, {bench['value']} {bench['unit']} ({rf['kernel']}).")
    else:
        L.append(f"- `bench.py` in the same run (HIP events on the launch stream): roofline group `{rf['kernel']}`, "
                 f"{rf['launches']} launches per pass, average {rf['avg_launch_ms'] * 1e3:.2f} us per launch, "
                 f"{rf['achieved']} {rf['unit']}; whole pass {bench['ms_per_step']} ms wall, {bench['value']} {bench['unit']}.")
    L.append("")
    out = {"workload": workload, "groups": {}}
    if copy_f and copy_w and fetch:
        ff, wf = (1 << 20) / copy_f[0], (1 << 20) / copy_w[0]     # KiB per count, from 1 GiB in and 1 GiB out
        out["fetch_kib_per_count"], out["write_kib_per_count"] = ff, wf
        L.append("## HBM traffic (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`; counter units per dispatch)\n")
        L.append(f"Yardstick: `onhip::copy_f32_kernel` moving 1 GiB in and 1 GiB out reads FETCH_SIZE = {copy_f[0]:.0f} and WRITE_SIZE = "
                 f"{copy_w[0]:.0f}, so one FETCH_SIZE count = {ff:.3f} KiB and one WRITE_SIZE count = {wf:.3f} KiB.\n")
        L.append("| kernel | dispatches | FETCH_SIZE mean | WRITE_SIZE mean | read MiB / dispatch | written MiB / dispatch |\n|---|---:|---:|---:|---:|---:|")
        traffic, launches = collections.defaultdict(float), collections.defaultdict(int)
        for k in sorted(fetch):
            g = family(k)
            if g is None:
                continue
            fv, wv = fetch[k]["FETCH_SIZE"], write[k]["WRITE_SIZE"]
            L.append(f"| `{k}` | {len(fv)} | {mean(fv):.1f} | {mean(wv):.1f} | {mean(fv) * ff / 1024:.2f} | {mean(wv) * wf / 1024:.2f} |")
            traffic[g] += (sum(fv) * ff + sum(wv) * wf) * 1024
            if "splitk_finish" not in k:
                launches[g] += len(fv)
        L.append("")
        for g in traffic:
            per = traffic[g] / max(1, launches[g])
            L.append(f"- {g}: {launches[g]} layer launches, **{per / 1e6:.2f} MB of HBM traffic per layer launch** (reads + writes, split-K partials included).")
            out["groups"][g] = {"launches_counted": launches[g], "hbm_bytes_per_launch": round(per)}
        dom = "igemm" if "igemm" in rf["kernel"] else "depthwise" if "depthwise" in rf["kernel"] else "glue"
        out["hbm_bytes_per_launch"] = out["groups"].get(dom, {}).get("hbm_bytes_per_launch")
        if "algorithmic_bytes_per_step" in bench["config"]:
            L.append(f"- algorithmic bytes per step (every tensor once): {bench['config']['algorithmic_bytes_per_step'] / 1e6:.1f} MB over {nl} layers "
                     f"= {bench['config']['algorithmic_bytes_per_step'] / nl / 1e6:.2f} MB per layer launch.")
        L.append("")
    if sq:
        L.append("## Matrix-core and LDS counters (`--pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT SQ_WAVE_CYCLES "
                 "SQ_INSTS_VALU SQ_WAIT_ANY`, means per dispatch)\n")
        L.append("MFMA utilisation = SQ_VALU_MFMA_BUSY_CYCLES (summed over the SIMDs) / (kernel duration from the trace x "
                 f"{CLOCK_HZ / 1e9:.1f} GHz x {SIMDS} SIMDs); wait share = SQ_WAIT_ANY / SQ_WAVE_CYCLES; conflict share = "
                 "SQ_LDS_BANK_CONFLICT cycles / (4 x SQ_WAVE_CYCLES) is left out where no LDS instruction ran.\n")
        L.append("| kernel | dispatches | MFMA busy cycles | MFMA utilisation | LDS instructions | LDS bank-conflict cycles | VALU instructions | wait share |\n"
                 "|---|---:|---:|---:|---:|---:|---:|---:|")
        for k in sorted(sq):
            if family(k) is None:
                continue
            c = sq[k]
            busy = mean(c["SQ_VALU_MFMA_BUSY_CYCLES"])
            d = dur_us.get(k)
            util = busy / (d * 1e-6 * CLOCK_HZ * SIMDS) if d else float("nan")
            wave = mean(c["SQ_WAVE_CYCLES"])
            L.append(f"| `{k}` | {len(c['SQ_BUSY_CYCLES'])} | {busy:.4g} | {util:.3f} | {mean(c['SQ_INSTS_LDS']):.4g} | "
                     f"{mean(c['SQ_LDS_BANK_CONFLICT']):.4g} | {mean(c['SQ_INSTS_VALU']):.4g} | "
                     f"{(mean(c['SQ_WAIT_ANY']) / wave if wave else 0):.2f} |")
        L.append("")
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, f"{workload}_kernels.md"), "w") as f:
        f.write("\n".join(L) + "\n")
    if out["groups"]:
        with open(os.path.join(out_dir, f"{workload}_traffic.json"), "w") as f:
            json.dump(out, f, indent=1)
    return "\n".join(L)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("workload")
    ap.add_argument("--raw", required=True, help="directory with the raw rocprofv3 files of the workload")
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles"))
    args = ap.parse_args()
    print(summarise(args.workload, args.raw, args.out))


if __name__ == "__main__":
    sys.exit(main())
