"""fp32 glue of a transformer encoder on the device against the oracle: Softmax, Erf, Gelu, LayerNorm.

Floating point, so the bar is a tolerance: 1e-5 relative (the reference sums sequentially with Kahan
compensation and calls the host's expf / erff; the kernels reduce in parallel and call the
device's), with an absolute floor where a result is a difference of nearly equal numbers (stated
at each check).  The shapes cross every kernel variant: rows kept in registers, rows re-read,
ragged rows, strided axes, and the BERT-base sizes (batch 32, 12 heads, sequence 128, hidden 768,
FFN 3072).
"""
import numpy as np
import pytest

import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth

pytestmark = pytest.mark.gpu
f32 = np.float32
RTOL = 1e-5


def say(*a):
    print("[case]", *a, flush=True)


SOFTMAX_CASES = [
    ((32 * 12 * 128, 128), (1,)),   # BERT-base attention rows: kept in registers
    ((3, 5, 2048), (2,)),           # the longest row that stays in registers
    ((7, 2052), (1,)),              # longer: re-read
    ((9, 131), (1,)),               # not a multiple of four
    ((77, 64), (1,)),               # short rows: four to a wavefront
    ((50, 20), (1,)),               # eight to a wavefront, five of eight lanes used
    ((13, 4), (1,)),
    ((4, 6, 10), (1,)),             # strided axis
    ((5, 3, 4, 6), (1, 2)),         # a run of two axes with an inner extent
    ((2, 3), ()),                   # all axes (op::v0::Softmax with an empty AxisSet)
    ((6, 1, 5), (1,)),              # one element along the axis
    ((0, 8), (1,)),                 # empty
]


@pytest.mark.parametrize("shape,axes", SOFTMAX_CASES)
def test_softmax(gpu_lib, shape, axes):
    say("softmax", shape, axes)
    O.port().orc_set_threads(8)
    x = synth.normal_f32(21, shape) * f32(5.0)
    exp = O.softmax(x, axes)
    got = H.softmax(x, axes)
    O.port().orc_set_threads(1)
    assert got.shape == exp.shape
    if x.size == 0:
        return
    assert np.allclose(got, exp, rtol=RTOL, atol=1e-30), float(np.max(np.abs(got - exp) / np.maximum(exp, 1e-30)))
    # rows sum to one
    outer, axis, inner = H._axes_run(x.shape, axes)
    assert np.allclose(got.reshape(outer, axis, inner).astype(np.float64).sum(axis=1), 1.0, atol=1e-5)
    assert H.last_kernel() == ("softmax_rows" if inner == 1 else "softmax_strided")


def test_softmax_extremes(gpu_lib):
    """test/backend/softmax.in.cpp:241-293: lowest() and max() in a column neither underflow to NaN nor overflow"""
    say("softmax extremes")
    for v in (np.finfo(f32).min, np.finfo(f32).max):
        x = np.array([[v, 1, 2], [3, 4, 5]], dtype=f32)
        got, exp = H.softmax(x, (0,)), O.softmax(x, (0,))
        assert np.all(np.isfinite(got)) and np.allclose(got, exp, rtol=RTOL, atol=1e-30)
        got, exp = H.softmax(x, (1,)), O.softmax(x, (1,))
        assert np.all(np.isfinite(got)) and np.allclose(got, exp, rtol=RTOL, atol=1e-30)


@pytest.mark.parametrize("n", [1, 3, 4096, 4099, 4096 * 3072])
def test_erf_and_gelu(gpu_lib, n):
    say("erf / gelu", n)
    x = synth.uniform_f32(22, (n,), -6.0, 6.0)
    # erf: |erf| <= 1 and the functions agree to a couple of ulps of 1
    assert np.max(np.abs(H.erf(x) - O.erf(x))) <= 2.4e-7
    assert H.last_kernel() == "erf_vec"
    # gelu: the f32 rounding of (1 + erf) is an absolute ~1e-7 scaled by 0.5 |x|; relative elsewhere
    got, exp = H.gelu(x), O.gelu(x)
    assert np.all(np.abs(got - exp) <= RTOL * np.abs(exp) + 3e-7 * np.maximum(np.abs(x), 1.0))
    assert H.last_kernel() == "gelu_vec"
    # special values
    sp = np.array([0.0, -0.0, np.inf, -np.inf, 50.0, -50.0], dtype=f32)
    assert np.array_equal(H.erf(sp), np.array([0.0, -0.0, 1.0, -1.0, 1.0, -1.0], dtype=f32))
    g = H.gelu(sp[[0, 4, 5]])
    assert g[0] == 0.0 and g[1] == 50.0 and g[2] == 0.0


LN_CASES = [
    ((32 * 128, 768), 1, True),     # BERT-base hidden states
    ((4, 2048), 1, True),           # the longest row that stays in registers
    ((5, 2056), 1, True),           # longer: re-read
    ((6, 130), 1, False),           # ragged row, no affine
    ((2, 3, 4, 5), 2, True),        # several trailing axes
    ((3, 7, 64), -1, True),         # negative begin_norm_axis
    ((0, 16), 1, True),             # empty
]


@pytest.mark.parametrize("shape,axis,affine", LN_CASES)
def test_layer_norm(gpu_lib, shape, axis, affine):
    say("layer_norm", shape, axis, affine)
    O.port().orc_set_threads(8)
    x = synth.normal_f32(23, shape) * f32(2.0) + f32(0.75)
    n_axis = axis if axis >= 0 else len(shape) + axis
    cols = int(np.prod(shape[n_axis:]))
    scale = synth.uniform_f32(24, (cols,), 0.5, 1.5) if affine else None
    bias = synth.uniform_f32(25, (cols,), -0.5, 0.5) if affine else None
    en, em, ev = O.layer_norm(x, scale, bias, begin_norm_axis=axis, epsilon=1e-5)
    gn, gm, gv = H.layer_norm(x, scale, bias, begin_norm_axis=axis, epsilon=1e-5)
    O.port().orc_set_threads(1)
    assert gn.shape == en.shape and gm.shape == em.shape
    if x.size == 0:
        return
    # the mean is a difference-prone quantity only against |x| ~ 2: absolute floor 1e-6
    assert np.allclose(gm, em, rtol=RTOL, atol=1e-6) and np.allclose(gv, ev, rtol=RTOL, atol=1e-7)
    # (x - mean) cancels near the mean: absolute floor 1e-5 on values of order one
    assert np.allclose(gn, en, rtol=RTOL, atol=1e-5), float(np.max(np.abs(gn - en)))
    g2, m2, v2 = H.layer_norm(x, scale, bias, begin_norm_axis=axis, epsilon=1e-5, keep_stats=False)
    assert m2 is None and v2 is None and np.array_equal(g2, gn)
    assert H.last_kernel() == "layer_norm_rows"


def test_layer_norm_reference_vectors(gpu_lib):
    """test/backend/layer_norm.in.cpp:48-91"""
    say("layer_norm reference vectors")
    x = np.array([[-4, -3, -2, -1], [0, 1, 2, 3]], dtype=f32)
    norm, mean, var = H.layer_norm(x, np.array([-1, 1, 2, 3], dtype=f32), np.array([-4, -3, -2, -1], dtype=f32), begin_norm_axis=1, epsilon=1e-5)
    exp = np.array([-2.658364534378051758, -3.447211742401123047, -1.105576276779174805, 3.024906158447265625] * 2, dtype=f32).reshape(2, 4)
    assert np.allclose(norm, exp, rtol=RTOL) and np.array_equal(mean, [-2.5, 1.5]) and np.array_equal(var, [1.25, 1.25])


def test_argument_errors(gpu_lib):
    lib = gpu_lib
    lib.hipq_softmax_f32.argtypes = [H.C.c_void_p, H.C.c_void_p, H.C.c_int64, H.C.c_int64, H.C.c_int64, H.C.c_void_p]
    assert lib.hipq_softmax_f32(None, None, 2, 3, 1, None) == H.ERR_INVALID
    assert lib.hipq_softmax_f32(None, None, -1, 3, 1, None) == H.ERR_INVALID
    lib.hipq_layer_norm_f32.argtypes = [H.C.c_void_p] * 6 + [H.C.c_int64, H.C.c_int64, H.C.c_double, H.C.c_void_p]
    buf = H.DeviceBuffer(64)
    assert lib.hipq_layer_norm_f32(buf.ptr, buf.ptr, None, buf.ptr, None, None, 1, 4, 1e-5, None) == H.ERR_INVALID  # scale without bias


MATMUL_CASES = [
    # batch, M, K, N
    (32 * 12, 128, 64, 128),   # BERT-base attention scores (Q K^T takes transpose_b)
    (32 * 12, 128, 128, 64),   # attention context
    (3, 70, 37, 129),          # ragged on every side
    (2, 64, 16, 64),           # exactly one tile, one step
    (1, 200, 300, 100),        # op::v0::Dot of two matrices
    (5, 1, 9, 1),
    (2, 8, 0, 8),              # empty reduction: zeros
    (0, 4, 4, 4),
]


@pytest.mark.parametrize("batch,M,K,N", MATMUL_CASES)
def test_batch_matmul(gpu_lib, batch, M, K, N):
    """bit-exact: like the reference (dot.hpp:37, widen<float> = double) the kernel accumulates the exact
    products in double, k ascending, and rounds to f32 once"""
    say("batch_matmul", batch, M, K, N)
    O.port().orc_set_threads(8)
    a, b = synth.normal_f32(51, (batch, M, K)), synth.normal_f32(52, (batch, K, N))
    small = batch * M * N * max(K, 1) <= 40_000_000
    for ta in (False, True):
        for tb in (False, True):
            if not small and (ta, tb) not in ((False, False), (False, True)):
                continue
            aa = np.ascontiguousarray(a.transpose(0, 2, 1)) if ta else a
            bb = np.ascontiguousarray(b.transpose(0, 2, 1)) if tb else b
            got = H.batch_matmul(aa, bb, ta, tb)
            assert got.shape == (batch, M, N)
            if got.size == 0:
                continue
            exp = O.batch_matmul(aa, bb, ta, tb)
            assert np.array_equal(got, exp), (ta, tb, float(np.max(np.abs(got - exp))))
            assert H.last_kernel() == "batch_matmul_f32"
    O.port().orc_set_threads(1)


def test_batch_matmul_reference_vectors(gpu_lib):
    """test/backend/batch_mat_mul.in.cpp:51-102 (small integers: exact)"""
    a = np.array([1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4], dtype=f32)
    b = np.array([1, 1, 1, 1, 2, 2, 2, 2, 3, 3, 3, 3] * 2, dtype=f32).reshape(2, 3, 4)
    assert np.array_equal(H.batch_matmul(a.reshape(2, 2, 3), b).ravel(), [6, 6, 6, 6, 12, 12, 12, 12, 18, 18, 18, 18, 24, 24, 24, 24])
    assert np.array_equal(H.batch_matmul(a.reshape(2, 3, 2), b, transpose_a=True).ravel(), [9, 9, 9, 9, 11, 11, 11, 11, 21, 21, 21, 21, 23, 23, 23, 23])
    # two matrices
    x, y = synth.normal_f32(53, (10, 20)), synth.normal_f32(54, (20, 6))
    assert np.allclose(H.batch_matmul(x, y), x.astype(np.float64) @ y.astype(np.float64), rtol=1e-5, atol=1e-5)


# ---- fused forms: equal to the op-by-op sequence they replace, bit for bit ------------------------


@pytest.mark.parametrize("shape", [(32 * 12 * 128, 128), (7, 128), (5, 300), (3, 2052), (9, 131), (50, 20)])
def test_softmax_scaled_equals_multiply_then_softmax(gpu_lib, shape):
    say("softmax scaled", shape)
    x = synth.normal_f32(41, shape) * f32(7.0)
    for c in (0.125, 0.3):
        got = H.softmax_scaled(x, c)
        exp = H.softmax(H.binary("multiply", x, np.asarray([c], dtype=f32)), (len(shape) - 1,))
        assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), c


@pytest.mark.parametrize("shape", [(4096, 768), (9, 768), (5, 30), (3, 2050), (6, 4)])
def test_add_layer_norm_with_quantized_output(gpu_lib, shape):
    say("add + layer norm + quantize", shape)
    a, b = synth.normal_f32(42, shape), synth.normal_f32(43, shape) * f32(0.3)
    gamma, beta = synth.uniform_f32(44, (shape[-1],), 0.8, 1.2), synth.uniform_f32(45, (shape[-1],), -0.1, 0.1)
    summed = H.binary("add", a, b)
    exp = H.layer_norm(summed, gamma, beta, begin_norm_axis=len(shape) - 1, epsilon=1e-5, keep_stats=False)[0]
    got, q = H.add_layer_norm(a, b, gamma, beta, 1e-5)
    assert q is None and np.array_equal(got.view(np.uint32), exp.view(np.uint32))
    for quant_t, zp, s in (("i8", 0, 6.0 / 127.0), ("i8", -3, 0.02), ("u8", 128, 0.03)):
        got, q = H.add_layer_norm(a, b, gamma, beta, 1e-5, q_scale=s, q_zp=zp, quant_t=quant_t)
        assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), quant_t
        assert np.array_equal(q, H.quantize(exp, f32(s), zp, quant_t)), (quant_t, zp)
        assert len(np.unique(q)) > 5
    # without the addend: plain LayerNorm with the quantized copy
    plain = H.layer_norm(a, gamma, beta, begin_norm_axis=len(shape) - 1, epsilon=1e-5, keep_stats=False)[0]
    got, q = H.add_layer_norm(a, None, gamma, beta, 1e-5, q_scale=0.05)
    assert np.array_equal(got.view(np.uint32), plain.view(np.uint32)) and np.array_equal(q, H.quantize(plain, f32(0.05), 0, "i8"))


@pytest.mark.parametrize("n", [3, 4096, 4099, 4096 * 3072])
def test_gelu_with_quantized_output(gpu_lib, n):
    say("gelu + quantize", n)
    x = synth.normal_f32(46, (n,)) * f32(2.0)
    exp = H.gelu(x)
    for quant_t, zp, s in (("i8", 0, 4.0 * 0.02 * 27.7 / 127.0), ("u8", 7, 0.01)):
        g, q = H.gelu_quantize(x, s, zp, quant_t)
        assert np.array_equal(g.view(np.uint32), exp.view(np.uint32))
        assert np.array_equal(q, H.quantize(exp, f32(s), zp, quant_t)), (quant_t, zp)
        g, q2 = H.gelu_quantize(x, s, zp, quant_t, keep_f32=False)
        assert g is None and np.array_equal(q2, q)


@pytest.mark.parametrize("B,S,nh,hd", [(2, 128, 12, 64), (3, 9, 2, 8), (2, 7, 3, 5)])
def test_batch_matmul_views_are_attention_without_the_reshapes(gpu_lib, B, S, nh, hd):
    """scores and context of an attention layer straight from the fused [tokens, 3 * hidden] projection
    and into the merged-heads layout, against the same products on permuted copies"""
    say("matmul views", B, S, nh, hd)
    h = nh * hd
    qkv = synth.normal_f32(47, (B * S, 3 * h))
    heads = np.ascontiguousarray(qkv.reshape(B, S, 3, nh, hd).transpose(2, 0, 3, 1, 4))
    Q, K, V = (heads[i].reshape(B * nh, S, hd) for i in range(3))
    exp_scores = H.batch_matmul(Q, K, False, True)
    v_scores = H.MatmulView(nh, S * 3 * h, hd, 3 * h, S * 3 * h, hd, 3 * h, nh * S * S, S * S, S)
    got_scores, _ = H.batch_matmul_view(qkv, 0, qkv, h, B * nh * S * S, 0, v_scores, B * nh, S, hd, S, False, True)
    assert np.array_equal(got_scores.view(np.uint32), exp_scores.ravel().view(np.uint32))
    probs = H.softmax(exp_scores * f32(0.125), (2,))
    exp_ctx = H.batch_matmul(probs, V, False, False)
    exp_merged = np.ascontiguousarray(exp_ctx.reshape(B, nh, S, hd).transpose(0, 2, 1, 3)).reshape(B * S, h)
    v_ctx = H.MatmulView(nh, nh * S * S, S * S, S, S * 3 * h, hd, 3 * h, S * h, hd, h)
    s_c = 0.4 / 127.0
    got_ctx, q = H.batch_matmul_view(probs, 0, qkv, 2 * h, B * S * h, 0, v_ctx, B * nh, S, S, hd, False, False, q_scale=s_c)
    assert np.array_equal(got_ctx.view(np.uint32), exp_merged.ravel().view(np.uint32))
    assert np.array_equal(q, H.quantize(exp_merged, f32(s_c), 0, "i8").ravel())
    _, q_only = H.batch_matmul_view(probs, 0, qkv, 2 * h, B * S * h, 0, v_ctx, B * nh, S, S, hd, False, False, q_scale=s_c, keep_f32=False)
    assert np.array_equal(q_only, q)


@pytest.mark.parametrize("B,S,nh", [(2, 128, 12), (1, 128, 1), (5, 128, 3)])
def test_attention_in_one_kernel_equals_the_three_ops(gpu_lib, B, S, nh):
    """scores, scaled Softmax and context of every head in one launch, against the three launches it
    replaces (bit for bit: the same product chains, the same Softmax lanes), with and without the
    Multiply, the f32 result and the quantized copy"""
    say("attention", B, S, nh)
    hd = 64
    h = nh * hd
    qkv = synth.normal_f32(48, (B * S, 3 * h)) * f32(1.5)
    v_scores = H.MatmulView(nh, S * 3 * h, hd, 3 * h, S * 3 * h, hd, 3 * h, nh * S * S, S * S, S)
    v_ctx = H.MatmulView(nh, nh * S * S, S * S, S, S * 3 * h, hd, 3 * h, S * h, hd, h)
    v_att = H.AttentionView(nh, S * 3 * h, hd, 3 * h, S * 3 * h, hd, 3 * h, S * 3 * h, hd, 3 * h, S * h, hd, h)
    scores, _ = H.batch_matmul_view(qkv, 0, qkv, h, B * nh * S * S, 0, v_scores, B * nh, S, hd, S, False, True)
    s_c = 0.4 / 127.0
    for factor in (0.125, None):
        probs = H.softmax_scaled(scores.reshape(B * nh * S, S), factor) if factor is not None else H.softmax(scores.reshape(B * nh * S, S), (1,))
        exp, exp_q = H.batch_matmul_view(probs, 0, qkv, 2 * h, B * S * h, 0, v_ctx, B * nh, S, S, hd, False, False, q_scale=s_c)
        got, q = H.attention(qkv, 0, h, 2 * h, B * S * h, v_att, B * nh, S, S, hd, factor=factor, q_scale=s_c)
        assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), factor
        assert np.array_equal(q, exp_q) and len(np.unique(q)) > 5
        assert H.last_kernel() == "attention_f32"
    got, q = H.attention(qkv, 0, h, 2 * h, B * S * h, v_att, B * nh, S, S, hd, factor=0.125)
    assert q is None
    _, q_only = H.attention(qkv, 0, h, 2 * h, B * S * h, v_att, B * nh, S, S, hd, factor=0.125, q_scale=s_c, quant_t="u8", q_zp=128, keep_f32=False)
    assert np.array_equal(q_only, H.quantize(got, f32(s_c), 128, "u8"))


def test_attention_in_one_kernel_rejects_other_shapes(gpu_lib):
    say("attention shapes")
    qkv = synth.normal_f32(49, (2 * 64, 3 * 64))
    view = H.AttentionView(1, 64 * 192, 64, 192, 64 * 192, 64, 192, 64 * 192, 64, 192, 64 * 64, 64, 64)
    for queries, keys, depth in ((64, 64, 64), (128, 128, 32), (100, 128, 64)):
        with pytest.raises(H.HipqError) as e:
            H.attention(qkv, 0, 64, 128, 2 * 64 * 64, view, 2, queries, keys, depth)
        assert e.value.code == H.ERR_UNSUPPORTED


def test_attention_in_one_kernel_rejects_bad_arguments(gpu_lib):
    """nothing is launched on operands the kernel's 16-byte fetches and its views could not honour"""
    say("attention arguments")
    lib = H.load()
    import ctypes as C

    S, hd = 128, 64
    buf = H.DeviceBuffer(4 * (3 * S * hd + 8))
    out = H.DeviceBuffer(4 * S * hd)
    lib.hipq_attention_f32.argtypes = [C.c_void_p] * 7 + [C.c_int64] * 4 + [C.c_void_p]

    def call(q_off=0, view=None, out_ptr=out.ptr, quant=None, view_ptr=True):
        v = view or H.AttentionView(1, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd)
        return lib.hipq_attention_f32(buf.ptr + q_off, buf.ptr + 4 * S * hd, buf.ptr + 8 * S * hd, None, out_ptr, C.byref(v) if view_ptr else None, quant, 1, S, S, hd, None)

    class _H:  # (the library's last error text)
        @staticmethod
        def last_error():
            return lib.hipq_last_error().decode()

    assert call() == H.OK
    assert call(q_off=4) == H.ERR_INVALID and "16-byte aligned" in _H.last_error()
    assert call(view=H.AttentionView(1, S * hd, 0, hd - 4, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd)) == H.ERR_INVALID and "shorter than the row" in _H.last_error()
    assert call(view=H.AttentionView(1, S * hd, 0, hd + 2, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd)) == H.ERR_INVALID
    assert call(view=H.AttentionView(1, -1, 0, hd, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd)) == H.ERR_INVALID and "negative batch stride" in _H.last_error()
    assert call(view=H.AttentionView(0, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd, S * hd, 0, hd)) == H.ERR_INVALID
    assert call(out_ptr=None) == H.ERR_INVALID and "null pointer" in _H.last_error()
    assert call(view_ptr=False) == H.ERR_INVALID and "null view" in _H.last_error()
    bad_quant = H.QuantOut(out.ptr, None, None, H.I8, H.RNE)
    assert call(quant=C.byref(bad_quant)) == H.ERR_INVALID
    H.check(lib.hipq_stream_sync(None))


@pytest.mark.parametrize("M,K,N,kernel", [(4096, 768, 3072, "dot_gelu_q8"), (512, 256, 80, "dot_gelu_q8"), (1000, 320, 144, "dot_gelu_q8"), (4096, 768, 3000, "gelu_vec"), (128, 768, 3072, "gelu_vec"),
                                          (300, 64, 64, "gelu_vec"), (2048, 1024, 1024, "dot_gelu_q8"), (512, 4096, 128, "dot_gelu_q8"), (384, 8192, 256, "dot_gelu_q8")])
def test_dot_bias_gelu_quantize_equals_the_three_ops(gpu_lib, M, K, N, kernel):
    """the feed-forward block's first projection with Gelu and Quantize in its epilogue (or, where those
    kernels do not apply, through the workspace) against QuantizedDotBias -> Gelu -> Quantize, bit for bit"""
    say("dot + gelu + quantize", M, K, N)
    a = synth.uniform_int(60, (M, K), -127, 127, np.int8)
    w = synth.uniform_int(61, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(62, (N,), -3000, 3000, np.int32)
    scale = synth.uniform_f32(63, (N,), 0.5, 1.5) * f32(4.0 / (127.0 * 127.0 * np.sqrt(K)))
    d = H.make_dot_desc(M, K, N, a_t="i8", out_t="f32", b_layout=H.B_NK)
    fd = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=N)
    product = H.quantized_dot_bias(d, fd, a, w, bias, scale)
    for quant_t, zp, s, mode in (("i8", 0, 3.0 / 127.0, H.RNE), ("u8", 9, 0.02, H.RNE), ("i8", -5, 0.03, H.ROUND_MODES.index("ROUND_NEAREST_TOWARD_INFINITY"))):
        _, exp = H.gelu_quantize(product, s, zp, quant_t, round_mode=mode, keep_f32=False)
        got = H.quantized_dot_bias_gelu_quantize(d, fd, a, w, bias, scale, s, zp, quant_t, round_mode=mode)
        assert np.array_equal(got, exp), (quant_t, zp)
        assert kernel in H.last_kernel(), H.last_kernel()
        assert len(np.unique(got)) > 20
    # one scale for all channels, ReLU in front of the Gelu, u8 data
    au = synth.uniform_int(64, (M, K), 0, 255, np.uint8)
    du = H.make_dot_desc(M, K, N, a_t="u8", out_t="f32", b_layout=H.B_NK)
    f1 = H.make_fused_desc(has_bias=True, with_relu=True, scale_count=1)
    product = H.quantized_dot_bias(du, f1, au, w, bias, scale[:1])
    _, exp = H.gelu_quantize(product, 0.05, 0, "u8", keep_f32=False)
    assert np.array_equal(H.quantized_dot_bias_gelu_quantize(du, f1, au, w, bias, scale[:1], 0.05, 0, "u8"), exp)


def test_dot_bias_gelu_quantize_refuses_output_over_its_input(gpu_lib):
    """workgroups write output bytes while others still read rows of the data: an output that overlaps
    the data is refused before any launch"""
    say("dot + gelu + quantize in place")
    import ctypes as C

    lib = H.load()
    M, K, N = 512, 256, 128
    d = H.make_dot_desc(M, K, N, a_t="i8", out_t="f32", b_layout=H.B_NK)
    fd = H.make_fused_desc(has_bias=False, with_relu=False, scale_count=1)
    buf = H.DeviceBuffer(M * max(K, N) + M * N)
    w = H.DeviceBuffer.from_numpy(synth.uniform_int(65, (N, K), -127, 127, np.int8))
    scale = H.DeviceBuffer.from_numpy(np.asarray([0.001], np.float32))
    qs = H.DeviceBuffer.from_numpy(np.asarray([0.05], np.float32))
    lib.hipq_quantized_dot_bias_gelu_quantize.argtypes = [C.c_void_p] * 9
    for out_ptr, ok in ((buf.ptr, False), (buf.ptr + M * K - 16, False), (buf.ptr + M * K, True)):
        q = H.QuantOut(out_ptr, qs.ptr, None, H.I8, H.RNE)
        rc = lib.hipq_quantized_dot_bias_gelu_quantize(C.byref(d), C.byref(fd), buf.ptr, w.ptr, None, None, scale.ptr, C.byref(q), None)
        assert (rc == H.OK) == ok, (out_ptr - buf.ptr, rc)
        if not ok:
            assert rc == H.ERR_INVALID and "overlap" in lib.hipq_last_error().decode()
    H.check(lib.hipq_stream_sync(None))
