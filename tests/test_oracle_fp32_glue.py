"""Pins the oracle's fp32 glue (Softmax, Erf, Gelu, LayerNorm) -- CPU only.

Against the reference's own tests (test/backend/softmax.in.cpp, gelu.in.cpp, layer_norm.in.cpp),
against the reference kernels compiled from the nGraph tree (oracle/_ref: softmax.hpp, sum.hpp,
erf.hpp) where that library is present, and against float64 closed forms.
"""
import math

import numpy as np
import pytest

import oracle_lib as O
from ngraph_amd import synth

f32 = np.float32
needs_ref = pytest.mark.skipif(not (O.have_ref() and hasattr(O.ref(), "ref_softmax_f32")), reason="oracle/_ref not built with the fp32 kernels")


def expf(v):
    return f32(np.exp(f32(v)))


def close_f(a, b, tolerance_bits=2):
    """test::all_close_f's default: the floats agree in all but the last 2 of their 24 mantissa bits"""
    a, b = np.asarray(a, dtype=f32), np.asarray(b, dtype=f32)
    ai, bi = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = np.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    return bool(np.all(np.abs(ai - bi) <= (1 << tolerance_bits)))


def test_softmax_reference_tests():
    """test/backend/softmax.in.cpp:66-293 -- the expectations are written there as expf() formulas"""
    # softmax_all (:66-94), also with the empty axis set
    x = np.array([[-3, -2, -1], [0, 1, 2]], dtype=f32)
    d = sum((expf(v) for v in (-3, -2, -1, 0, 1, 2)), f32(0))
    exp = np.array([expf(v) / d for v in (-3, -2, -1, 0, 1, 2)], dtype=f32).reshape(2, 3)
    assert close_f(O.softmax(x, (0, 1)), exp) and close_f(O.softmax(x, ()), exp)
    # softmax_axis_3d (:96-131): axis 0 of [2,2,3]
    x = np.array([-10, -20, -30, -40, -50, -60, -1, -2, -3, -4, -5, -6], dtype=f32).reshape(2, 2, 3)
    ds = [expf(a) + expf(b) for a, b in zip((-10, -20, -30, -40, -50, -60), (-1, -2, -3, -4, -5, -6))]
    exp = np.array([expf(v) / ds[i % 6] for i, v in enumerate(x.ravel())], dtype=f32).reshape(2, 2, 3)
    assert np.allclose(O.softmax(x, (0,)), exp, rtol=1e-5, atol=1e-8)
    # softmax_axis (:170-194): axis 1 of [2,3]; softmax_axis_2 (:196-221): axis 0
    x = np.array([[-10, -20, -30], [-40, -50, -60]], dtype=f32)
    d0, d1 = expf(-10) + expf(-20) + expf(-30), expf(-40) + expf(-50) + expf(-60)
    exp = np.array([[expf(-10) / d0, expf(-20) / d0, expf(-30) / d0], [expf(-40) / d1, expf(-50) / d1, expf(-60) / d1]], dtype=f32)
    assert close_f(O.softmax(x, (1,)), exp)
    d = [expf(-10) + expf(-40), expf(-20) + expf(-50), expf(-30) + expf(-60)]
    exp = np.array([[expf(-10) / d[0], expf(-20) / d[1], expf(-30) / d[2]], [expf(-40) / d[0], expf(-50) / d[1], expf(-60) / d[2]]], dtype=f32)
    assert close_f(O.softmax(x, (0,)), exp)
    # softmax_axis_3d_trivial (:223-239): a single element along the axis gives 1
    assert np.array_equal(O.softmax(np.array([[[-10, -20, -30], [-40, -50, -60]]], dtype=f32), (0,)), np.ones((1, 2, 3), dtype=f32))
    # softmax_underflow / softmax_overflow (:241-293): the row maximum is subtracted first
    low, high = np.finfo(f32).min, np.finfo(f32).max
    x = np.array([[low, 1, 2], [3, 4, 5]], dtype=f32)
    d = [expf(low) + expf(3), expf(1) + expf(4), expf(2) + expf(5)]
    exp = np.array([[expf(low) / d[0], expf(1) / d[1], expf(2) / d[2]], [expf(3) / d[0], expf(4) / d[1], expf(5) / d[2]]], dtype=f32)
    assert close_f(O.softmax(x, (0,)), exp)
    x = np.array([[high, 1, 2], [3, 4, 5]], dtype=f32)
    d0 = expf(0) + expf(f32(3) - high)
    exp = np.array([[expf(0) / d0, expf(1) / d[1], expf(2) / d[2]], [expf(f32(3) - high) / d0, expf(4) / d[1], expf(5) / d[2]]], dtype=f32)
    got = O.softmax(x, (0,))
    assert close_f(got, exp) and np.all(np.isfinite(got))


@needs_ref
@pytest.mark.parametrize("shape,axes", [((7, 33), (1,)), ((5, 6, 9), (1,)), ((4, 3, 10), (0,)), ((3, 4, 5, 6), (2, 3)), ((2, 50), ()), ((3, 1, 7), (1,))])
def test_softmax_equals_compiled_reference(shape, axes):
    """runtime::reference::softmax<float> itself (max, exp, compensated sum, divide), bit for bit"""
    x = synth.normal_f32(11, shape) * f32(4.0)
    assert np.array_equal(O.softmax(x, axes), O.ref_softmax(x, axes))


@needs_ref
def test_erf_equals_compiled_reference():
    x = np.concatenate([synth.uniform_f32(12, (5000,), -6.0, 6.0), np.array([0.0, -0.0, np.inf, -np.inf, 1e-30, -1e-30], dtype=f32)])
    assert np.array_equal(O.erf(x), O.ref_erf(x))


def test_erf_closed_form():
    """against math.erf in float64 (test/backend/erf.in.cpp:47-66 compares with std::erf the same way)"""
    x = synth.uniform_f32(13, (4000,), -5.0, 5.0)
    exp = np.array([math.erf(float(v)) for v in x])
    assert np.max(np.abs(O.erf(x) - exp)) < 2e-7
    assert O.erf(np.array([0.0], dtype=f32))[0] == 0.0 and O.erf(np.array([np.inf], dtype=f32))[0] == 1.0


def test_gelu_reference_tests():
    """test/backend/gelu.in.cpp:49-108: 0.5 * x * (1 + erf(x / sqrt(2))), f32 on U(-100,100) to 0.007, and the eight f64 points"""
    x = synth.uniform_f32(14, (100000,), -100.0, 100.0)
    exp = np.array([0.5 * float(v) * (1.0 + math.erf(float(v) / math.sqrt(2.0))) for v in x[:20000]])
    got = O.gelu(x)
    assert np.all(np.abs(got[:20000] - exp) <= 0.007 + 0.007 * np.abs(exp))
    # f32 rounding of (1 + erf) is an absolute 6e-8, scaled by 0.5 |x|: that bounds the distance to the f64 value
    assert np.all(np.abs(got[:20000] - exp) <= 2e-7 * np.maximum(np.abs(x[:20000]), 1.0))
    pts = np.array([-4.0, -3.0, -2.0, -1.0, 0.0, 1.0, 2.0, 3.0], dtype=f32)
    exp = np.array([0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))) for v in pts.astype(np.float64)])
    assert np.allclose(O.gelu(pts), exp, rtol=2e-6, atol=1e-7)
    # the decomposition's order of operations (op/gelu.cpp:59): (half * data) * (one + erf(data / sqrt_two)) in f32
    for v in (f32(0.7), f32(-1.3), f32(2.5)):
        t = f32(v / f32(math.sqrt(2.0)))
        manual = f32(f32(0.5) * v) * f32(f32(1.0) + f32(math.erf(float(t))))
        assert abs(float(O.gelu(np.array([v]))[0]) - float(manual)) <= abs(float(manual)) * 2.4e-7


def test_layer_norm_reference_test():
    """test/backend/layer_norm.in.cpp:48-91 (layer_norm_affine_stats): literal vectors"""
    x = np.array([[-4, -3, -2, -1], [0, 1, 2, 3]], dtype=f32)
    scale = np.array([-1, 1, 2, 3], dtype=f32)
    bias = np.array([-4, -3, -2, -1], dtype=f32)
    norm, mean, var = O.layer_norm(x, scale, bias, begin_norm_axis=1, epsilon=1e-5)
    exp = np.array([-2.658364534378051758, -3.447211742401123047, -1.105576276779174805, 3.024906158447265625] * 2, dtype=f32).reshape(2, 4)
    assert close_f(norm, exp)
    assert close_f(mean, np.array([-2.5, 1.5], dtype=f32)) and close_f(var, np.array([1.25, 1.25], dtype=f32))


def test_layer_norm_closed_form_and_options():
    """float64 statistics; no affine; begin_norm_axis over several trailing axes and negative"""
    x = synth.normal_f32(15, (6, 5, 8)) * f32(3.0) + f32(1.5)
    norm, mean, var = O.layer_norm(x, None, None, begin_norm_axis=1, epsilon=1e-5)
    x64 = x.astype(np.float64).reshape(6, 40)
    mu, v = x64.mean(axis=1), x64.var(axis=1)
    assert np.allclose(mean, mu, rtol=1e-6, atol=1e-6) and np.allclose(var, v, rtol=1e-6)
    assert np.allclose(norm.reshape(6, 40), (x64 - mu[:, None]) / np.sqrt(v[:, None] + 1e-5), rtol=1e-5, atol=1e-5)
    scale, bias = synth.uniform_f32(16, (8,), 0.5, 2.0), synth.uniform_f32(17, (8,), -1.0, 1.0)
    n2, m2, v2 = O.layer_norm(x, scale, bias, begin_norm_axis=-1, epsilon=1e-3)
    assert m2.shape == (6, 5)
    x64 = x.astype(np.float64)
    exp = (x64 - x64.mean(-1, keepdims=True)) / np.sqrt(x64.var(-1, keepdims=True) + 1e-3) * scale + bias
    assert np.allclose(n2, exp, rtol=1e-5, atol=1e-5)


@needs_ref
def test_layer_norm_sums_equal_compiled_reference():
    """mean and variance are reference::sum (sequential, Kahan-compensated) divided by n: the oracle's row sums must be that sum bit for bit"""
    x = synth.normal_f32(18, (9, 700)) * f32(100.0)
    _, mean, var = O.layer_norm(x, None, None, begin_norm_axis=1)
    s = O.ref_sum(x, (1,))
    assert np.array_equal(mean, s / f32(700))
    d = (x - mean[:, None]).astype(f32)
    assert np.array_equal(var, O.ref_sum((d * d).astype(f32), (1,)) / f32(700))


def test_batch_matmul_reference_tests():
    """test/backend/batch_mat_mul.in.cpp:51-102: BatchMatMulTranspose without and with a transposed first operand"""
    a = np.array([1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4], dtype=f32)
    b = np.array([1, 1, 1, 1, 2, 2, 2, 2, 3, 3, 3, 3] * 2, dtype=f32).reshape(2, 3, 4)
    got = O.batch_matmul(a.reshape(2, 2, 3), b)
    assert np.array_equal(got.ravel(), [6, 6, 6, 6, 12, 12, 12, 12, 18, 18, 18, 18, 24, 24, 24, 24])
    got = O.batch_matmul(a.reshape(2, 3, 2), b, transpose_a=True)
    assert np.array_equal(got.ravel(), [9, 9, 9, 9, 11, 11, 11, 11, 21, 21, 21, 21, 23, 23, 23, 23])


@pytest.mark.skipif(not (O.have_ref() and hasattr(O.ref(), "ref_batch_mat_mul_f32")), reason="oracle/_ref not built with batch_mat_mul")
@pytest.mark.parametrize("batch,M,K,N", [(3, 5, 7, 4), (2, 16, 33, 9), (1, 1, 50, 1), (4, 8, 1, 8)])
def test_batch_matmul_equals_compiled_reference(batch, M, K, N):
    """runtime::reference::batch_mat_mul<float> (dot.hpp's sequential f32 sum) bit for bit; the transposed
    forms must give the same bits on operands transposed in numpy"""
    a, b = synth.normal_f32(41, (batch, M, K)), synth.normal_f32(42, (batch, K, N))
    exp = O.ref_batch_matmul(a, b)
    assert np.array_equal(O.batch_matmul(a, b), exp)
    at, bt = np.ascontiguousarray(a.transpose(0, 2, 1)), np.ascontiguousarray(b.transpose(0, 2, 1))
    assert np.array_equal(O.batch_matmul(at, b, transpose_a=True), exp)
    assert np.array_equal(O.batch_matmul(a, bt, transpose_b=True), exp)
    assert np.array_equal(O.batch_matmul(at, bt, transpose_a=True, transpose_b=True), exp)
    assert np.allclose(exp, np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64)), rtol=1e-5, atol=1e-5)
