"""Builds the gfx950 shared objects in place (onenew_amd/lib/): the kernel library
libonenew_hip.so, the model runtime libonenew_rt.so and the operator plugins lib{Conv,MatMul,Gemm,Add,Relu,MaxPool,GlobalAveragePool,Gelu,LayerNormalization,Softmax,Transpose}_hip.so.

    python -m onenew_amd.build [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 instructions are switched off for every device compile; floating-point contraction is
# off because the epilogues and the depthwise kernels reproduce the reference's separately rounded
# multiply and add (__fmul_rn / __fadd_rn are plain operators to this compiler, not barriers)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-c++20-extensions",
             "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
KERNEL_SOURCES = ["depthwise.hip", "dw_s8.hip", "igemm_f32.hip", "igemm_f32_res.hip", "igemm_f32_pw.hip", "igemm_bf16.hip", "igemm_f16.hip", "igemm_i8.hip", "igemm_i8_res.hip", "igemm_rowb.hip", "igemm_dma.hip", "igemm_dma_bf16.hip", "igemm_dma_f16.hip", "igemm.hip", "direct.hip", "h16.hip", "attention.hip", "attention_h16.hip", "stem.hip", "irblock.hip", "i8patch.hip", "calib.hip", "elementwise.hip", "vit_glue.hip", "api.hip",
                  "plugin.hip"]
# per-file compiler options.  The implicit-GEMM kernels keep their accumulators in ordinary vector registers (the
# compiler's default puts them into the accumulation half of the register file and copies them out, one instruction per
# register, for the store): the same kernels fit one more wavefront per SIMD (fp32 64 x 64: 75 registers instead of
# 75 + 16, six instead of five; with a residual operand five instead of four; int8 128 x 128 three instead of two)
EXTRA_FLAGS = {src: ["-mllvm", "-amdgpu-mfma-vgpr-form=1"] for src in KERNEL_SOURCES if src.startswith("igemm")}
PLUGINS = {"Conv": "plugin_conv.cpp", "MatMul": "plugin_matmul.cpp", "Gemm": "plugin_gemm.cpp",
           "Add": "plugin_add.cpp", "Relu": "plugin_relu.cpp", "MaxPool": "plugin_maxpool.cpp",
           "GlobalAveragePool": "plugin_global_avgpool.cpp", "Gelu": "plugin_gelu.cpp",
           "LayerNormalization": "plugin_layernorm.cpp", "Softmax": "plugin_softmax.cpp",
           "Transpose": "plugin_transpose.cpp"}
HEADERS = [os.path.join(CSRC, "onhip_internal.hpp"), os.path.join(CSRC, "igemm_kernel.hpp"), os.path.join(CSRC, "igemm_dma_kernel.hpp"), os.path.join(HERE, "..", "include", "onenew_hip.h"),
           os.path.join(HERE, "..", "include", "onenew_abi.h"), os.path.abspath(__file__)]


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def _scratch_users(text):
    """kernels that the compiler gave a stack frame (register arrays that fell out of registers): the resource
    remarks come as a 'Function Name' line followed by that function's figures"""
    bad, name = [], None
    for line in text.splitlines():
        if "remark:" not in line:
            continue
        body = line.split("remark:", 1)[1].strip()
        if body.startswith("Function Name:"):
            name = body.split(":", 1)[1].split("[")[0].strip()
        elif body.startswith("ScratchSize [bytes/lane]:"):
            # a few dozen bytes are reserved now and then without a single scratch instruction in the kernel;
            # operand arrays that fell out of registers take a kilobyte and more
            if int(body.split(":", 1)[1].split("[")[0]) > 256 and name:
                bad.append(name)
    return bad


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and "remark:" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if out.strip():
        print(out)
    # the MFMA kernels keep tiles, operands and prefetched units in registers by construction: a kernel of those
    # files that uses scratch memory has lost that (a lambda that was not inlined, an array indexed at run time)
    if any(os.path.basename(a).startswith("igemm_") for a in cmd):
        bad = _scratch_users(res.stdout)
        if bad:
            raise RuntimeError("kernels with a stack frame (scratch memory) in " + cmd[-3] + ":\n  " + "\n  ".join(bad))


def build(force=False, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    jobs = []
    objs = []
    for src in KERNEL_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJDIR, src + ".o")
        objs.append(o)
        if force or _stale(o, [s] + HEADERS):
            jobs.append([HIPCC] + HIP_FLAGS + EXTRA_FLAGS.get(src, []) + ["-Rpass-analysis=kernel-resource-usage", "-c", s, "-o", o])
    if verbose and jobs:
        print(f"[onenew_amd.build] compiling {len(jobs)} file(s) for gfx950", flush=True)
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(_run, jobs))
    core = os.path.join(LIBDIR, "libonenew_hip.so")
    if force or jobs or _stale(core, objs):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", core] + objs)
    for op, src in PLUGINS.items():
        so = os.path.join(LIBDIR, f"lib{op}_hip.so")
        s = os.path.join(CSRC, src)
        if force or _stale(so, [s, core] + HEADERS):
            _run(["g++", "-O2", "-fPIC", "-shared", "-fvisibility=hidden", s, "-o", so, "-L" + LIBDIR,
                  "-lonenew_hip", "-Wl,-rpath,$ORIGIN"])
    # the device-resident model runtime: host code over the HIP runtime API, it reaches the kernels through the plugins
    rt = os.path.join(LIBDIR, "libonenew_rt.so")
    rt_src = os.path.join(CSRC, "runtime.cpp")
    if force or _stale(rt, [rt_src, os.path.join(HERE, "..", "include", "onenew_rt.h")] + HEADERS):
        _run(["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__",
              "-I/opt/rocm/include", rt_src, "-o", rt, "-L/opt/rocm/lib", "-lamdhip64", "-ldl", "-Wl,-rpath,/opt/rocm/lib"])
    return LIBDIR


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    print("built in", LIBDIR)
