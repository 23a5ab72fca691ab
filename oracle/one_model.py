"""CPU execution of a .one model with the oracle's operators: the restatement of what the reference host does
between loading the file and returning the outputs (host/net.h:138-221 reading, :274-330 ordering, the
shape_infer of each host/ops/*.h, host/op.h:109-185 running every operator in order).

TEST INFRASTRUCTURE ONLY, like the rest of this directory.  Pinned by running the same files through the
reference's own operator classes and x86 kernels (oracle/_ref/ref_run_one, tests/test_one_model_cpu.py):
outputs and shapes agree bit for bit."""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle import oracle  # noqa: E402
from onenew_amd import abi, onefile  # noqa: E402
from onenew_amd.abi import ConvDesc  # noqa: E402

REF_RUNNER = os.path.join(HERE, "_ref", "ref_run_one")
REF_OPS = os.path.join(HERE, "_ref", "ops")


def _names(cfg):
    b = cfg.op_base_cfg
    return ([b.in_operand_name[i].value.decode() for i in range(b.in_operand_num)],
            [b.out_operand_name[i].value.decode() for i in range(b.out_operand_num)])


def _conv(cfg, x, w, bias):
    n, cin, h, wd = x.shape
    d = ConvDesc(n=n, cin=cin, h=h, w=wd, cout=w.shape[0], kh=cfg.kernel_shape[0], kw=cfg.kernel_shape[1],
                 stride_h=cfg.strides[0], stride_w=cfg.strides[1], pad_t=cfg.pads[0], pad_l=cfg.pads[1],
                 pad_b=cfg.pads[2], pad_r=cfg.pads[3], group=cfg.group, has_bias=cfg.has_bias, act_type=cfg.act_type,
                 clip_min=cfg.clip_min, clip_max=cfg.clip_max, leaky_relu_alpha=cfg.leaky_relu_alpha,
                 hard_sigmoid_alpha=cfg.hard_sigmoid_alpha, hard_sigmoid_beta=cfg.hard_sigmoid_beta)
    lut = oracle.silu_lut() if cfg.act_type == abi.SILU else None
    if cfg.ifmap_quant2 == abi.TYPE_INT8:
        # W8A32: int8 weights and int32 bias sit at the front of fp32-sized initialisers (conv.c:77-104)
        d.input_scale = cfg.input_scale
        w8 = np.ascontiguousarray(w).reshape(-1).view(np.int8)[:w.size].reshape(w.shape)
        b32 = None if bias is None else np.ascontiguousarray(bias).view(np.int32)
        aux = np.array([cfg.weight_aux[i] for i in range(d.cout)], dtype=np.float32)
        return oracle.conv2d_w8a32(d, x, w8, b32, aux, lut)
    return oracle.conv2d_f32(d, x, w, bias, lut)


def run(one_bytes, inputs, keep_all=False):
    """inputs: arrays in io order.  Returns the outputs in io order (keep_all: a dict of every operand)."""
    m = onefile.parse(one_bytes)
    env = {name: np.ascontiguousarray(a, dtype=np.float32).reshape(shape)
           for (name, shape), a in zip(m["inputs"], inputs)}
    inits = m["inits"]
    pending = list(m["nodes"])
    while pending:
        for k, (op_type, cfg) in enumerate(pending):
            ins, outs = _names(cfg)
            if all((not n) or n in env or n in inits for n in ins):
                break
        else:
            raise ValueError("graph cannot be ordered")
        pending.pop(k)
        arg = [env[n] if n in env else inits[n] for n in ins]
        x = arg[0]
        if op_type == "Conv":
            y = _conv(cfg, x, arg[1], arg[2] if cfg.has_bias else None)
        elif op_type == "Gemm":
            y = oracle.gemm_f32(x.reshape(-1, x.shape[-1]), arg[1], arg[2]).reshape(x.shape[:-1] + (arg[2].size,))
        elif op_type == "MatMul":
            y = oracle.matmul_f32(x, arg[1])
        elif op_type == "Add":
            y = oracle.add_f32(x, arg[1])
        elif op_type == "Relu":
            y = oracle.relu_f32(x)
        elif op_type == "Gelu":
            y = oracle.lut_act(x, oracle.gelu_lut())
        elif op_type == "MaxPool":
            y = oracle.maxpool_f32(x, cfg.kernel_shape[0], cfg.strides[0], cfg.pads[0])
        elif op_type == "GlobalAveragePool":
            y = oracle.global_avgpool_f32(x)
        elif op_type == "LayerNormalization":
            y = oracle.layernorm_f32(x, arg[1], arg[2], axis1=(cfg.axes[0] == 1))
        elif op_type == "Softmax":
            y = oracle.softmax_f32(x, axis1=not (cfg.axis == -1 or cfg.axis == x.ndim - 1))
        elif op_type == "Transpose":
            y = oracle.transpose_f32(x, [cfg.perm[i] for i in range(cfg.perm_num)])
        elif op_type == "Flatten":
            y = x.reshape(x.shape[:cfg.axis] + (-1,))
        elif op_type == "Reshape":
            y = x.reshape([cfg.dst_shape[i] for i in range(cfg.dst_shape_num)])
        else:
            raise ValueError(f"no oracle for {op_type}")
        env[outs[0]] = y
    return env if keep_all else [env[name] for name, _ in m["outputs"]]


def have_ref_runner():
    return os.path.exists(REF_RUNNER) and os.path.isdir(REF_OPS)


def time_reference(one_bytes, inputs, repeats, threads=8):
    """median milliseconds of one inference through the reference's operator classes and x86 kernels"""
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "m.one")
        with open(path, "wb") as f:
            f.write(one_bytes)
        files = []
        for i, a in enumerate(inputs):
            files.append(os.path.join(tmp, f"in{i}.bin"))
            np.ascontiguousarray(a, dtype=np.float32).tofile(files[-1])
        env = dict(os.environ, ONENEW_REF_OP_DIR=REF_OPS, REF_REPEAT=str(repeats), OMP_NUM_THREADS=str(threads))
        out = subprocess.run([REF_RUNNER, path, tmp] + files, check=True, env=env, capture_output=True, text=True).stdout
        for line in out.splitlines():
            if line.startswith("forward_ms"):
                return float(line.split()[1])
    raise RuntimeError("the reference runner printed no timing")


def run_reference(one_bytes, inputs):
    """The same model through the reference's operator classes and x86 kernels (CPU).  Returns
    [(name, array)] for the outputs in io order."""
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "m.one")
        with open(path, "wb") as f:
            f.write(one_bytes)
        files = []
        for i, a in enumerate(inputs):
            files.append(os.path.join(tmp, f"in{i}.bin"))
            np.ascontiguousarray(a, dtype=np.float32).tofile(files[-1])
        env = dict(os.environ, ONENEW_REF_OP_DIR=REF_OPS)
        subprocess.run([REF_RUNNER, path, tmp] + files, check=True, env=env, stdout=subprocess.DEVNULL)
        out = []
        for line in open(os.path.join(tmp, "shapes.txt")):
            parts = line.split()
            shape = tuple(int(v) for v in parts[3:3 + int(parts[2])])
            out.append((parts[1], np.fromfile(os.path.join(tmp, parts[0]), dtype=np.float32).reshape(shape)))
        return out
