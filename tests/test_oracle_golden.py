"""Pins the CPU oracle against outputs of the reference's own compiled x86 kernels
(tests/golden/golden.npz, written by tests/golden/make_golden.py): bit-identical for every fp32 and
W8A32 convolution path, MatMul, Gemm and the table activations."""
import numpy as np
import pytest

import cases


@pytest.mark.parametrize("name", list(cases.conv_f32_cases()))
def test_conv_f32_bit_exact(name, golden, oracle):
    d = cases.conv_f32_cases()[name]
    x, w, b = cases.conv_inputs(name, d)
    y = oracle.conv2d_f32(d, x, w, b, cases.silu_lut())
    cases.check_against(golden, name, y, exact=True)


@pytest.mark.parametrize("name", list(cases.conv_w8a32_cases()))
def test_conv_w8a32_bit_exact(name, golden, oracle):
    d = cases.conv_w8a32_cases()[name]
    x, w8, b32, aux = cases.conv_inputs(name, d, quant=True)
    y = oracle.conv2d_w8a32(d, x, w8, b32, aux, cases.silu_lut())
    cases.check_against(golden, name, y, exact=True)


@pytest.mark.parametrize("name", list(cases.matmul_cases()))
def test_matmul_bit_exact(name, golden, oracle):
    a, b = cases.matmul_inputs(name, *cases.matmul_cases()[name])
    cases.check_against(golden, name, oracle.matmul_f32(a, b), exact=True)


@pytest.mark.parametrize("name", list(cases.gemm_cases()))
def test_gemm_bit_exact(name, golden, oracle):
    a, w, b = cases.gemm_inputs(name, *cases.gemm_cases()[name])
    cases.check_against(golden, name, oracle.gemm_f32(a, w, b), exact=True)


def test_gelu_table_apply(golden, oracle):
    y = oracle.lut_act(cases.gelu_input(), cases.gelu_lut())
    cases.check_against(golden, "gelu_edges", y, exact=True)


def test_tables_regenerate(oracle):
    """the table builders reproduce the tables dumped from the reference host classes"""
    assert np.array_equal(oracle.silu_lut(), cases.silu_lut())
    assert np.array_equal(oracle.gelu_lut(), cases.gelu_lut())
    assert cases.silu_lut()[4608] == np.float32(0.731058598) and cases.gelu_lut()[4608] == np.float32(0.841347098)


@pytest.mark.parametrize("name", list(cases.add_cases()))
def test_add_bit_exact(name, golden, oracle):
    a, b = cases.add_inputs(name, *cases.add_cases()[name])
    y = oracle.add_f32(a, b)
    cases.check_against(golden, name, y, exact=True)
    if np.broadcast_shapes(a.shape, b.shape) == y.shape:
        assert np.array_equal(y, a + b)            # numpy's broadcasting is the closed form


@pytest.mark.parametrize("name", list(cases.relu_cases()))
def test_relu_bit_exact(name, golden, oracle):
    """bit patterns, so that the signed zeros and NaNs either side of the 32-element body count"""
    x = cases.relu_input(name, cases.relu_cases()[name])
    y = oracle.relu_f32(x)
    key = f"{name}/full" if f"{name}/full" in golden else None
    if key:
        assert np.array_equal(golden[key].view(np.uint32), y.reshape(-1).view(np.uint32))
    else:
        idx = cases.sample_indices(name, y.size)
        assert np.array_equal(golden[f"{name}/samples"].view(np.uint32), y.reshape(-1)[idx].view(np.uint32))


@pytest.mark.parametrize("name", list(cases.maxpool_cases()))
def test_maxpool_bit_exact(name, golden, oracle):
    shape, k, st, pad = cases.maxpool_cases()[name]
    y = oracle.maxpool_f32(cases.maxpool_input(name, shape), k, st, pad)
    cases.check_against(golden, name, y, exact=True)
    if name == "mp_deep_negative":
        assert y.min() == np.float32(-3276800.0)   # the start value of the running maximum shows through


@pytest.mark.parametrize("name", list(cases.gap_cases()))
def test_global_avgpool_bit_exact(name, golden, oracle):
    x = cases.gap_input(name, cases.gap_cases()[name])
    y = oracle.global_avgpool_f32(x)
    cases.check_against(golden, name, y, exact=True)
    assert np.allclose(y.reshape(x.shape[:2]), x.astype(np.float64).mean(axis=(2, 3)), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("name", list(cases.layernorm_cases()))
def test_layernorm_bit_exact(name, golden, oracle):
    shape, axis = cases.layernorm_cases()[name]
    x, w, b = cases.layernorm_inputs(name, shape, axis)
    y = oracle.layernorm_f32(x, w, b, axis1=(axis == 1))
    cases.check_against(golden, name, y, exact=True)
    # closed form in float64 (eps 1e-20 is invisible)
    ax = 1 if axis == 1 else max(i for i, d in enumerate(shape) if d != 1)
    x64 = x.astype(np.float64)
    norm = (x64 - x64.mean(axis=ax, keepdims=True)) / np.sqrt(x64.var(axis=ax, keepdims=True))
    bshape = [1] * x.ndim
    bshape[ax] = -1
    assert np.allclose(y, norm * w.reshape(bshape) + b.reshape(bshape), rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("name", list(cases.softmax_cases()))
def test_softmax_bit_exact(name, golden, oracle):
    """same libm as the reference build in this container, so the CPU restatement matches to the bit"""
    shape, axis = cases.softmax_cases()[name]
    x = cases.softmax_input(name, shape)
    y = oracle.softmax_f32(x, axis1=(axis == 1))
    cases.check_against(golden, name, y, exact=True)
    ax = 1 if axis == 1 else x.ndim - 1
    e = np.exp(x.astype(np.float64) - x.max(axis=ax, keepdims=True))
    assert np.allclose(y, e / e.sum(axis=ax, keepdims=True), rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("name", list(cases.transpose_cases()))
def test_transpose_bit_exact(name, golden, oracle):
    shape, perm = cases.transpose_cases()[name]
    x = cases.transpose_input(name, shape)
    y = oracle.transpose_f32(x, perm)
    assert np.array_equal(y, np.transpose(x, perm))
    if len(shape) in (4, 6) or len(perm) <= 4:
        cases.check_against(golden, name, y, exact=True)
