"""Parity of the HIP library (through the C ABI) with the oracle, on a real MI355X.

Bars: bit-exact for every integer output (int32 accumulators, int8 / uint8 results); Dequantize
f32 outputs within 1e-5 relative (they are in fact required to be bit-exact below, which is
stricter).  Every case prints its name before it touches the GPU.
"""
import ctypes as C

import numpy as np
import pytest

import cases
import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)


# ------------------------------------------------------------------ Quantize / Dequantize


def test_quantize_dequantize_kats(gpu_lib, qdq_kats):
    for t in qdq_kats:
        say(t["name"])
        shape = t["shape"]
        x = np.array(t["input"], dtype=H.NP_OF[H.dtype_code(t["input_type"])]).reshape(shape)
        if t["op"] == "quantize":
            got = H.quantize(x, t["scale"], t["offset"], t["output_type"], t["axes"], t["round_mode"])
            assert got.reshape(-1).astype(np.int64).tolist() == t["expected"], t["name"]
        else:
            got = H.dequantize(x, t["scale"], t["offset"], t["output_type"], t["axes"])
            assert np.array_equal(got.reshape(-1), np.array(t["expected"], dtype=got.dtype)), t["name"]


def test_quantize_reference_vectors(gpu_lib, ref_vectors):
    manifest, arrays = ref_vectors
    for m in manifest:
        if m["kind"] != "quantize":
            continue
        say(m["name"])
        x, s, z = arrays[m["name"] + "__x"], arrays[m["name"] + "__scale"], arrays[m["name"] + "__zp"]
        got = H.quantize(x, s, z, m["quant_t"], m["axes"], m["round_mode"])
        assert np.array_equal(got, arrays[m["name"]]), m["name"]
        dq = H.dequantize(got, s, z, m["real_t"], m["axes"])
        assert np.array_equal(dq, arrays[m["name"] + "__dq"]), m["name"]


@pytest.mark.parametrize("mode", range(9))
@pytest.mark.parametrize("qt", ["i8", "u8", "i32"])
def test_quantize_round_modes_dense(gpu_lib, mode, qt):
    """every half-integer neighbourhood, vectorised kernel (count % 4 == 0) and generic kernel"""
    base = np.arange(-600, 600, dtype=np.float32) * 0.25
    eps = np.float32(2.0**-20)
    x = np.concatenate([base, base + eps, base - eps, np.float32([8388607.5, 8388609.0, -8388609.0, 1e9, -1e9, 0.49999997, -0.49999997, 3e38])])
    assert x.size % 4 == 0
    for (s, z) in ((1.0, 0), (0.3, 3)):
        say("round modes", mode, qt, s, z)
        assert np.array_equal(H.quantize(x, s, z, qt, (), mode), O.quantize(x, s, z, qt, (), mode))
        assert np.array_equal(H.quantize(x[:-1], s, z, qt, (), mode), O.quantize(x[:-1], s, z, qt, (), mode))


@pytest.mark.parametrize(
    "shape,axes",
    [((8, 64, 128), (1,)), ((5, 7, 12), (1,)), ((6, 40), (0,)), ((6, 40), (1,)), ((3, 4, 5, 8), (1, 2)), ((3, 4, 5), (0, 2)), ((2, 3, 5, 7), ()), ((4096,), (0,))],
)
def test_quantize_axes_patterns(gpu_lib, shape, axes):
    say("axes", shape, axes)
    x = synth.normal_f32(7, shape) * 30
    sshape = [shape[a] for a in axes]
    scale = synth.uniform_f32(8, sshape, 0.05, 1.5)
    for qt in ("i8", "u8"):
        lo, hi = (-20, 20) if qt == "i8" else (0, 40)
        zp = synth.uniform_int(9, sshape, lo, hi, H.NP_OF[H.dtype_code(qt)])
        got = H.quantize(x, scale, zp, qt, axes)
        exp = O.quantize(x, scale, zp, qt, axes)
        assert np.array_equal(got, exp)
        dq = H.dequantize(got, scale, zp, "f32", axes)
        dexp = O.dequantize(exp, scale, zp, "f32", axes)
        assert np.array_equal(dq, dexp)
        # the 1e-5 relative bar of the specification, stated explicitly
        assert np.allclose(dq, dexp, rtol=1e-5, atol=0)


def test_quantize_dequantize_config3_shape(gpu_lib):
    """[8,1024,1024] slice of BASELINE config 3 (per-channel scales on axis 1 = max|x|/127, RNE)
    against the oracle, bit for bit"""
    shape = (8, 1024, 1024)
    say("config3 slice", shape)
    x = synth.normal_f32(11, shape)
    scale = (np.abs(x).max(axis=(0, 2)) / np.float32(127)).astype(np.float32)
    zp = np.zeros(1024, np.int8)
    O.port().orc_set_threads(8)
    got = H.quantize(x, scale, zp, "i8", (1,))
    assert H.last_kernel() == "quantize_vec4"
    exp = O.quantize(x, scale, zp, "i8", (1,))
    assert np.array_equal(got, exp)
    dq = H.dequantize(got, scale, zp, "f32", (1,))
    assert H.last_kernel() == "dequantize_vec4"
    assert np.array_equal(dq, O.dequantize(exp, scale, zp, "f32", (1,)))
    O.port().orc_set_threads(1)


def test_quantize_dequantize_config3_full_size_properties(gpu_lib):
    """full [64,1024,1024] of config 3 on the device: size-independent properties.
    |dq - x| <= scale/2 (+ rounding slack) inside the clamp range, re-quantizing the dequantized
    tensor reproduces q exactly (idempotence), and the 8 slices agree with the oracle-checked kernel
    run slice by slice (same kernel, different launch geometry)."""
    lib = gpu_lib
    shape = (64, 1024, 1024)
    say("config3 full", shape)
    n = int(np.prod(shape))
    x = synth.normal_f32(12, (8, 1024, 1024))
    scale = (np.abs(x).max(axis=(0, 2)) / np.float32(127)).astype(np.float32)
    zp = np.zeros(1024, np.int8)
    bx = H.DeviceBuffer(n * 4)
    for i in range(8):  # tile the 8-image block eight times
        H.check(lib.hipq_memcpy_h2d(bx.ptr + i * x.nbytes, x.ctypes.data, x.nbytes, None))
    bs, bz = H.DeviceBuffer.from_numpy(scale), H.DeviceBuffer.from_numpy(zp)
    bq, bdq, bq2 = H.DeviceBuffer(n), H.DeviceBuffer(n * 4), H.DeviceBuffer(n)
    d = H.make_quant_desc(shape, (1,), "f32", "i8")
    H.check(lib.hipq_quantize(C.byref(d), bx.ptr, bs.ptr, bz.ptr, bq.ptr, None))
    H.check(lib.hipq_dequantize(C.byref(d), bq.ptr, bs.ptr, bz.ptr, bdq.ptr, None))
    H.check(lib.hipq_quantize(C.byref(d), bdq.ptr, bs.ptr, bz.ptr, bq2.ptr, None))
    H.check(lib.hipq_stream_sync(None))
    q = bq.to_numpy(np.int8, shape)
    q2 = bq2.to_numpy(np.int8, shape)
    assert np.array_equal(q, q2)
    part = H.quantize(x, scale, zp, "i8", (1,))
    for i in range(8):
        assert np.array_equal(q[8 * i : 8 * i + 8], part)
    dq = bdq.to_numpy(np.float32, shape)[:8]
    err = np.abs(dq - x)
    # half a quantization step, plus the f32 roundings of x/scale and q*scale (a few ulp of |x| <= 127*scale)
    bound = scale[None, :, None] * np.float32(0.5 + 127 * 4 * 2.0**-24)
    assert np.all(err <= bound)


@pytest.mark.parametrize("inner", [1024, 1000])
@pytest.mark.parametrize("qt", ["i8", "u8"])
def test_quantize_division_bits_near_ties(gpu_lib, qt, inner):
    """The vectorised kernel shares one reciprocal among the four elements of a group when the
    exponents allow it: its quotients must still be the IEEE ones.  Dividends are placed on and a
    few ulp either side of scale * (k + 1/2), where one wrong last bit of the quotient changes the
    rounded integer; scales cover the range limits of the shared-reciprocal path (2^-30, 2^30), what
    lies beyond them (denormal, huge, negative, Inf, NaN, zero), and groups mix special dividends
    (NaN, Inf, denormals, -0, 1e35) with ordinary ones.  inner = 1024 takes the kernel form whose
    scale index is uniform over a workgroup step, inner = 1000 the per-lane form; the dequantize
    kernels have the same two forms and are checked on the result."""
    rng = np.random.default_rng(2024)
    chans = 256
    scale = rng.uniform(0.001, 3.0, chans).astype(np.float32)
    scale[:24] = np.float32(
        [2.0**-30, 2.0**-30 * (1 - 2.0**-24), 2.0**30, 2.0**30 * (1 + 2.0**-23), 1e-40, 3e38, -0.37, -(2.0**-31), np.inf, np.nan, 0.0, -0.0,
         1.0, 0.5, 3.0, 1 / 3, 0.1, 127.0, 1 / 127, 2.0**-29, 2.0**29, 1.9999999, 1.0000001, 0.99999994]
    )
    k = rng.integers(-140, 140, (chans, inner)).astype(np.float32) + np.float32(0.5)
    with np.errstate(all="ignore"):
        x = (scale[:, None] * k).astype(np.float32)
        ulps = rng.integers(-3, 4, x.shape).astype(np.int32)
        x = (x.view(np.int32) + ulps).view(np.float32)
    special = np.float32([np.nan, np.inf, -np.inf, 1e-42, -1e-42, -0.0, 1e35, -1e35, 2.0**30, 2.0**-60, 2.0**-61, 1e-30])
    pos = rng.integers(0, inner, (chans, special.size))
    for c in range(0, chans, 3):
        x[c, pos[c]] = special
    zp = rng.integers(-9, 9, chans).astype(np.int8) if qt == "i8" else rng.integers(0, 30, chans).astype(np.uint8)
    say("ties", qt)
    got = H.quantize(x, scale, zp, qt, (0,))
    assert H.last_kernel() == "quantize_vec4"
    with np.errstate(all="ignore"):
        exp = O.quantize(x, scale, zp, qt, (0,))
    assert np.array_equal(got, exp)
    with np.errstate(all="ignore"):
        dq = H.dequantize(got, scale, zp, "f32", (0,))
        assert H.last_kernel() == "dequantize_vec4"
        assert np.array_equal(dq, O.dequantize(exp, scale, zp, "f32", (0,)), equal_nan=True)
    # the same through the scalar-scale form, ordinary scales only
    for c in (12, 13, 15, 16, 40, 41):
        g1 = H.quantize(x[c], scale[c], zp[c], qt)
        with np.errstate(all="ignore"):
            assert np.array_equal(g1, O.quantize(x[c], scale[c], zp[c], qt)), c


def test_quantize_empty_and_scalar(gpu_lib):
    say("empty / rank-0")
    assert H.quantize(np.zeros((0, 3), np.float32), 1.0, 0, "i8").shape == (0, 3)
    assert H.quantize(np.float32(5.0).reshape(()), 2.0, 1, "u8").item() == 3
    assert H.dequantize(np.int8(-4).reshape(()), 0.5, 2, "f32").item() == -3.0


# ------------------------------------------------------------------ QuantizedConvolution


def _conv_both(desc, data, filt, s, z):
    """direct kernel and (where eligible) MFMA kernel"""
    outs = []
    got = H.quantized_convolution(desc, data, filt, s[0], z[0], s[1], z[1], s[2], z[2], use_packed=False)
    outs.append(("direct", got, H.last_kernel()))
    if H.load().hipq_conv_packed_filter_bytes(C.byref(desc)):
        got = H.quantized_convolution(desc, data, filt, s[0], z[0], s[1], z[1], s[2], z[2], use_packed=True)
        outs.append(("mfma", got, H.last_kernel()))
    return outs


def test_conv_kats(gpu_lib, kats):
    lib = O.port()
    for k in kats["conv"]:
        if k.get("policy") == "dnnl":
            continue
        say(k["name"])
        d, data, filt, exp = cases.kat_conv(k)
        if k.get("via_builder"):
            s = [lib.orc_get_scale(*k["in_range"], d.data_t, 0), lib.orc_get_scale(*k["filter_range"], d.filter_t, 0), lib.orc_get_scale(*k["out_range"], d.out_t, 0)]
            z = [0, 0, 0]
        else:
            s, z = k["scales"], k["zps"]
        for name, got, kern in _conv_both(d, data, filt, s, z):
            assert got.reshape(-1).astype(np.int64).tolist() == exp.astype(np.int64).tolist(), (k["name"], name)


def test_conv_reference_vectors(gpu_lib, ref_vectors):
    """compiled-reference outputs, including BASELINE config 1 with its wrapped outputs"""
    manifest, arrays = ref_vectors
    used = set()
    for m in manifest:
        if m["kind"] != "conv":
            continue
        say(m["name"])
        d, data, filt, s, z = cases.conv_from_manifest(m)
        for name, got, kern in _conv_both(d, data, filt, s, z):
            assert np.array_equal(got, arrays[m["name"]]), (m["name"], name, kern)
            used.add(kern)
        # channels-last descriptors on the same tensors (2-D MFMA-eligible cases included)
        dl = cases.conv_from_manifest(m, H.NXC, H.NXC)[0]
        for name, got, kern in _conv_both(dl, cases.to_nxc(data), filt, s, z):
            assert np.array_equal(cases.to_ncx(got), arrays[m["name"]]), (m["name"], name, "nxc")
    assert "conv_direct" in used and any(k.startswith(("conv_mfma", "dot_skinny")) for k in used), used


MFMA_SHAPES = [
    # N, C, K, in_sp, f_sp, kw : ResNet-50-like layers and ragged edges (K, pixels not multiples of the tile)
    (1, 64, 64, (56, 56), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),
    (3, 64, 64, (20, 20), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),
    (2, 64, 256, (14, 14), (1, 1), dict()),
    (2, 256, 64, (14, 14), (1, 1), dict()),
    (1, 128, 128, (28, 28), (3, 3), dict(stride=(2, 2), pad_below=(1, 1), pad_above=(1, 1))),
    (2, 256, 512, (14, 14), (1, 1), dict(stride=(2, 2))),
    (1, 16, 24, (9, 7), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),
    (1, 48, 40, (11, 13), (3, 2), dict(stride=(2, 1), dilation=(1, 2), pad_below=(2, 0), pad_above=(0, 3))),
    (2, 32, 200, (10, 10), (5, 5), dict(pad_below=(2, 2), pad_above=(2, 2))),
    (1, 80, 17, (6, 6), (3, 3), dict(pad_below=(-1, 1), pad_above=(1, -1))),
    (2, 32, 8, (33,), (5,), dict(stride=(2,), pad_below=(2,), pad_above=(2,))),
    (1, 512, 512, (7, 7), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),
]


@pytest.mark.parametrize("i", range(len(MFMA_SHAPES)))
def test_conv_mfma_shapes(gpu_lib, i):
    N, Cc, K, in_sp, f_sp, kw = MFMA_SHAPES[i]
    say("mfma conv", MFMA_SHAPES[i])
    for out_t, s, z in (("i32", (1.0, 1.0, 1.0), (0, 0, 0)), ("i8", (0.02, 0.005, 0.9), (0, 0, -3)), ("i8", (0.02, 0.005, 0.7), (131, 0, 0))):
        d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, data_layout=H.NXC, out_layout=H.NXC, **kw)
        data = synth.uniform_int(100 + i, d.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(200 + i, d.filter_shape(), -128, 127, np.int8)
        O.port().orc_set_threads(8)
        exp = O.quantized_convolution(d, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
        O.port().orc_set_threads(1)
        got = H.quantized_convolution(d, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
        assert H.last_kernel().startswith(("conv_mfma", "conv_band", "conv_regw", "dot_skinny")), H.last_kernel()
        assert np.array_equal(got, exp), (out_t, z)
    # reference layouts in and out (transposed through the workspace)
    d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="i8", **kw)
    data = synth.uniform_int(100 + i, d.data_shape(), 0, 255, np.uint8)
    O.port().orc_set_threads(8)
    exp = O.quantized_convolution(d, data, filt, 0.02, 0, 0.005, 0, 0.9, 0)
    O.port().orc_set_threads(1)
    got = H.quantized_convolution(d, data, filt, 0.02, 0, 0.005, 0, 0.9, 0)
    assert H.last_kernel().startswith(("conv_mfma", "conv_band", "conv_regw", "dot_skinny")), H.last_kernel()
    assert np.array_equal(got, exp)


def test_conv_mfma_nonzero_filter_zero_point(gpu_lib):
    """packed filter handed over although the filter zero point is not zero: the kernel's slow
    in-kernel path must still give the reference's numbers"""
    say("mfma conv, filter zp != 0")
    d = H.make_conv_desc(1, 32, 40, (9, 9), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_layout=H.NXC, out_layout=H.NXC)
    data = synth.uniform_int(31, d.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(32, d.filter_shape(), -128, 127, np.int8)
    exp = O.quantized_convolution(d, data, filt, 0.02, 7, 0.005, -9, 0.9, 1)
    got = H.quantized_convolution(d, data, filt, 0.02, 7, 0.005, -9, 0.9, 1)
    assert np.array_equal(got, exp)


def test_conv_i8_data(gpu_lib):
    say("i8 data")
    d = H.make_conv_desc(1, 32, 48, (9, 9), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_t="i8", out_t="i32", data_layout=H.NXC, out_layout=H.NXC)
    data = synth.uniform_int(41, d.data_shape(), -128, 127, np.int8)
    filt = synth.uniform_int(42, d.filter_shape(), -128, 127, np.int8)
    for zpd in (0, -5):
        exp = O.quantized_convolution(d, data, filt, 1.0, zpd, 1.0, 0, 1.0, 0)
        for packed in (False, True):
            got = H.quantized_convolution(d, data, filt, 1.0, zpd, 1.0, 0, 1.0, 0, use_packed=packed)
            assert np.array_equal(got, exp), (zpd, packed, H.last_kernel())


def test_conv_linearity_at_config1_batch(gpu_lib):
    """BASELINE config 1's layer at batch 32 (too slow for the CPU oracle in a test): int32
    accumulators are linear in the filter, conv(f1) + conv(f2) == conv(f1 + f2), and image 0
    equals the oracle-checked single-image result"""
    say("config1 batch 32 linearity")
    kw = dict(pad_below=(1, 1), pad_above=(1, 1), out_t="i32", data_layout=H.NXC, out_layout=H.NXC)
    d = H.make_conv_desc(32, 64, 64, (56, 56), (3, 3), **kw)
    data = synth.uniform_int(51, d.data_shape(), 0, 255, np.uint8)
    f1 = synth.uniform_int(52, d.filter_shape(), -60, 60, np.int8)
    f2 = synth.uniform_int(53, d.filter_shape(), -60, 60, np.int8)
    a = H.quantized_convolution(d, data, f1, 1.0, 0, 1.0, 0, 1.0, 0).astype(np.int64)
    b = H.quantized_convolution(d, data, f2, 1.0, 0, 1.0, 0, 1.0, 0).astype(np.int64)
    c = H.quantized_convolution(d, data, (f1 + f2).astype(np.int8), 1.0, 0, 1.0, 0, 1.0, 0).astype(np.int64)
    assert H.last_kernel().startswith(("conv_mfma", "conv_band", "conv_regw", "dot_skinny"))
    assert np.array_equal(a + b, c)
    d1 = H.make_conv_desc(1, 64, 64, (56, 56), (3, 3), **kw)
    O.port().orc_set_threads(8)
    exp0 = O.quantized_convolution(d1, data[:1], f1, 1.0, 0, 1.0, 0, 1.0, 0)
    exp31 = O.quantized_convolution(d1, data[31:], f1, 1.0, 0, 1.0, 0, 1.0, 0)
    O.port().orc_set_threads(1)
    assert np.array_equal(a[:1], exp0) and np.array_equal(a[31:], exp31)


# ------------------------------------------------------------------ fused convolutions


def test_fused_conv_kats(gpu_lib, kats):
    lib = O.port()
    for k in kats["fused_conv"]:
        say(k["name"])
        d, data, filt, exp = cases.kat_conv(k)
        builder_out_t = H.U8 if k["with_relu"] else H.I8
        scale = lib.orc_get_conv_requant_scale(*k["in_range"], H.U8, *k["filter_range"], H.I8, *k["out_range"], builder_out_t)
        bias = k.get("bias")
        if "bias_f32" in k:
            bs = lib.orc_get_bias_scale(*k["in_range"], *k["filter_range"])
            bias = H.quantize(np.float32(k["bias_f32"]), bs, 0, "i32", (), H.RNE).tolist()
        has_sum = "sum" in k
        sum_scale = sum_in = None
        if has_sum:
            sum_scale = lib.orc_get_sum_scale(*k["out_range"], *k["sum_range"])
            if k["op"] == "QuantizedConvolutionBiasSignedAdd" and builder_out_t == H.U8:
                sum_scale = np.float32(2.0) * np.float32(sum_scale)
            sum_in = np.array(k["sum"], dtype=H.NP_OF[H.dtype_code(k["sum_t"])]).reshape(d.out_shape())
        f = H.make_fused_desc(has_bias=bias is not None, has_sum=has_sum, sum_t=k.get("sum_t", "u8"), with_relu=k["with_relu"])
        got = H.quantized_convolution_fused(d, f, data, filt, bias, sum_in, scale, sum_scale)
        if k["out_t"] == "u8_via_i8_convert":
            got = got.astype(np.uint8)
        assert got.reshape(-1).astype(np.int64).tolist() == exp.tolist(), k["name"]


def test_quant_conv_linear_rne_kat(gpu_lib, kats):
    """ONNX QLinearConv vector (round-half-even): the fused entry point without bias"""
    k = next(x for x in kats["conv"] if x.get("policy") == "dnnl")
    say(k["name"])
    d, data, filt, exp = cases.kat_conv(k)
    f = H.make_fused_desc(has_bias=False)
    got = H.quantized_convolution_fused(d, f, data, filt, None, None, np.float32(1.0 / 16.0), None)
    assert got.reshape(-1).astype(np.int64).tolist() == exp.tolist()


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("has_sum", [False, True])
@pytest.mark.parametrize("layout", [H.NCX, H.NXC])
def test_fused_conv_random(gpu_lib, relu, has_sum, layout):
    """ResNet-style bottleneck piece: per-channel scales, bias, residual sum, relu; both kernels"""
    say("fused conv", relu, has_sum, layout)
    out_t = "u8" if relu else "i8"
    for (Cc, K, sp, fs, kw) in ((64, 96, (12, 12), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))), (3, 16, (17, 17), (7, 7), dict(stride=(2, 2), pad_below=(3, 3), pad_above=(3, 3)))):
        d = H.make_conv_desc(2, Cc, K, sp, fs, out_t=out_t, data_layout=layout, out_layout=layout, **kw)
        dn = H.make_conv_desc(2, Cc, K, sp, fs, out_t=out_t, **kw)
        data = synth.uniform_int(61, dn.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(62, d.filter_shape(), -127, 127, np.int8)
        bias = synth.uniform_int(63, (K,), -20000, 20000, np.int32)
        scales = synth.uniform_f32(64, (K,), 2e-4, 9e-4)
        summ = synth.uniform_int(65, dn.out_shape(), 0, 255, np.uint8) if has_sum else None
        if layout == H.NXC:
            data = cases.to_nxc(data)
            summ = cases.to_nxc(summ) if has_sum else None
        f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="u8", with_relu=relu, scale_count=K)
        ss = 0.37 if has_sum else None
        exp = O.quantized_convolution_fused(d, f, data, filt, bias, summ, scales, ss)
        for packed in (False, True):
            got = H.quantized_convolution_fused(d, f, data, filt, bias, summ, scales, ss, use_packed=packed)
            assert np.array_equal(got, exp), (Cc, packed, H.last_kernel())
    # signed sum input, scalar scale, output stays i8 (QuantizedConvolutionBiasSignedAdd)
    d = H.make_conv_desc(1, 32, 32, (8, 8), (1, 1), out_t="i8", data_layout=layout, out_layout=layout)
    data = synth.uniform_int(71, d.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(72, d.filter_shape(), -127, 127, np.int8)
    summ = synth.uniform_int(73, d.out_shape(), -128, 127, np.int8)
    f = H.make_fused_desc(has_bias=False, has_sum=True, sum_t="i8", with_relu=relu)
    exp = O.quantized_convolution_fused(d, f, data, filt, None, summ, 1.5e-3, 0.8)
    got = H.quantized_convolution_fused(d, f, data, filt, None, summ, 1.5e-3, 0.8)
    assert np.array_equal(got, exp)


BAND_SHAPES = [
    # N, K, in_sp, f_sp, kw : 64 input channels, filter resident in LDS
    (2, 64, (56, 56), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),  # 7 full bands an image
    (1, 64, (20, 20), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),  # one band, ragged last tile
    (3, 32, (30, 24), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),  # short last band, K < 64
    (2, 48, (14, 14), (1, 1), dict()),                                    # 1x1, K not a multiple of 32
    (1, 16, (12, 16), (3, 2), dict(pad_below=(1, 0), pad_above=(1, 1))),  # asymmetric filter and padding
    (1, 64, (9, 40), (3, 3), dict()),                                     # no padding
    (2, 32, (5, 60), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),   # 64-slot rows, one-row items with ragged tiles, K < 64
    (3, 48, (10, 48), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),  # 64-slot rows, short last band, idle wavefronts
]


@pytest.mark.parametrize("i", range(len(BAND_SHAPES)))
def test_conv_band(gpu_lib, i, monkeypatch):
    """the LDS-resident-filter kernel against the oracle: both requantization policies, both output
    layouts, both fixed-point and float requantization branches, i32 output, zero points (the
    filter-in-registers kernel, which would take the 3x3 shapes with an NCHW output, is switched off:
    tests/test_conv_regw.py is its own)"""
    monkeypatch.setenv("HIPQ_NO_REGW", "1")
    N, K, in_sp, f_sp, kw = BAND_SHAPES[i]
    say("band conv", BAND_SHAPES[i])
    O.port().orc_set_threads(8)
    kernels = set()
    for dl, ol in ((H.NXC, H.NXC), (H.NXC, H.NCX), (H.NCX, H.NCX)):
        for out_t, data_t, s, z in (
            ("i8", "u8", (0.02, 0.005, 0.9), (0, 0, -3)),     # fixed-point requantization
            ("u8", "u8", (0.02, 0.005, 0.7), (131, 0, 7)),    # padding materialised as the zero point
            ("i8", "u8", (1.0, 1.0, 1.0), (0, 0, 0)),         # |scale| too large for fixed point; wraps
            ("i32", "u8", (1.0, 1.0, 1.0), (3, 0, 11)),
            ("i8", "i8", (0.02, 0.005, 0.9), (-5, 0, 0)),
            ("u8", "u8", (0.02, 0.005, 0.9), (9, -7, 1)),     # filter zero point: exact slow path
        ):
            d = H.make_conv_desc(N, 64, K, in_sp, f_sp, data_t=data_t, out_t=out_t, data_layout=dl, out_layout=ol, **kw)
            dn = H.make_conv_desc(N, 64, K, in_sp, f_sp, data_t=data_t, out_t=out_t, **kw)
            lo, hi = (0, 255) if data_t == "u8" else (-128, 127)
            data = synth.uniform_int(300 + i, dn.data_shape(), lo, hi, H.NP_OF[H.dtype_code(data_t)])
            filt = synth.uniform_int(400 + i, d.filter_shape(), -128, 127, np.int8)
            exp = O.quantized_convolution(dn, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
            got = H.quantized_convolution(d, cases.to_nxc(data) if dl == H.NXC else data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
            kernels.add(H.last_kernel())
            got = cases.to_ncx(got) if ol == H.NXC else got
            assert np.array_equal(got, exp), (dl, ol, out_t, data_t, z, H.last_kernel())
        # fused policy: bias, per-channel scales, residual sum, relu
        for relu, has_sum, per_channel in ((True, True, True), (False, False, False), (True, False, True), (False, True, False)):
            out_t = "u8" if relu else "i8"
            d = H.make_conv_desc(N, 64, K, in_sp, f_sp, out_t=out_t, data_layout=dl, out_layout=ol, **kw)
            dn = H.make_conv_desc(N, 64, K, in_sp, f_sp, out_t=out_t, **kw)
            data = synth.uniform_int(500 + i, dn.data_shape(), 0, 255, np.uint8)
            filt = synth.uniform_int(600 + i, d.filter_shape(), -127, 127, np.int8)
            bias = synth.uniform_int(63, (K,), -20000, 20000, np.int32)
            scales = synth.uniform_f32(64, (K,), 2e-4, 9e-4) if per_channel else np.float32(5e-4)
            summ = synth.uniform_int(65, dn.out_shape(), -128, 127, np.int8) if has_sum else None
            f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="i8", with_relu=relu, scale_count=K if per_channel else 1)
            ss = 0.37 if has_sum else None
            exp = O.quantized_convolution_fused(dn, H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="i8", with_relu=relu, scale_count=K if per_channel else 1), data, filt, bias, summ, scales, ss)
            got = H.quantized_convolution_fused(
                d, f, cases.to_nxc(data) if dl == H.NXC else data, filt, bias, (cases.to_nxc(summ) if ol == H.NXC else summ) if has_sum else None, scales, ss
            )
            kernels.add(H.last_kernel())
            got = cases.to_ncx(got) if ol == H.NXC else got
            assert np.array_equal(got, exp), (dl, ol, relu, has_sum, per_channel, H.last_kernel())
    O.port().orc_set_threads(1)
    assert any(k.startswith("conv_band") for k in kernels), kernels


SKINNY_CONV_SHAPES = [
    # N, C, K, in_sp, f_sp, kw : at most 64 output pixels in all and a reduction of whole 64-byte steps
    (1, 256, 64, (8, 7), (1, 1), dict()),                                                    # the data is the matrix
    (1, 512, 512, (7, 7), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),                 # im2col, padding taps
    (1, 64, 96, (12, 12), (3, 3), dict(stride=(2, 2), pad_below=(1, 1), pad_above=(0, 1))),  # stride, ragged K
    (1, 128, 40, (7, 8), (2, 2), dict(dilation=(2, 1), pad_below=(1, 0), pad_above=(1, 0))),
    (3, 256, 1000, (1, 1), (1, 1), dict()),                                                  # a classifier as a convolution
]


@pytest.mark.parametrize("i", range(len(SKINNY_CONV_SHAPES)))
def test_conv_as_skinny_gemm(gpu_lib, i):
    """layers with few output pixels run as a GEMM over their receptive-field matrix on the
    weight-streaming kernels: both policies, zero points (padding holds the data zero point; a filter
    zero point takes the exact path), reference-layout input (transposed, then gathered), residual sum"""
    N, Cc, K, in_sp, f_sp, kw = SKINNY_CONV_SHAPES[i]
    say("skinny conv", SKINNY_CONV_SHAPES[i])
    O.port().orc_set_threads(8)
    for dl in (H.NXC, H.NCX):
        for out_t, z in (("i8", (0, 0, -3)), ("u8", (131, 0, 7)), ("i32", (3, 0, 0)), ("i8", (9, -7, 1))):
            d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, data_layout=dl, out_layout=H.NXC, **kw)
            dn = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, **kw)
            data = synth.uniform_int(1100 + i, dn.data_shape(), 0, 255, np.uint8)
            filt = synth.uniform_int(1200 + i, dn.filter_shape(), -128, 127, np.int8)
            s = (1.0, 1.0, 1.0) if out_t == "i32" else (0.02, 0.005, 0.9)
            exp = O.quantized_convolution(dn, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
            got = H.quantized_convolution(d, cases.to_nxc(data) if dl == H.NXC else data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
            assert H.last_kernel().startswith("dot_skinny"), H.last_kernel()
            assert np.array_equal(cases.to_ncx(got), exp), (dl, out_t, z)
        for relu, has_sum in ((True, True), (False, False)):
            out_t = "u8" if relu else "i8"
            d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, data_layout=dl, out_layout=H.NXC, **kw)
            dn = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, **kw)
            data = synth.uniform_int(1300 + i, dn.data_shape(), 0, 255, np.uint8)
            filt = synth.uniform_int(1400 + i, dn.filter_shape(), -127, 127, np.int8)
            bias = synth.uniform_int(1500, (K,), -20000, 20000, np.int32)
            scales = synth.uniform_f32(1501, (K,), 2e-4, 9e-4)
            summ = synth.uniform_int(1502, dn.out_shape(), 0, 255, np.uint8) if has_sum else None
            f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="u8", with_relu=relu, scale_count=K)
            exp = O.quantized_convolution_fused(dn, f, data, filt, bias, summ, scales, 0.37 if has_sum else None)
            got = H.quantized_convolution_fused(d, f, cases.to_nxc(data) if dl == H.NXC else data, filt, bias, cases.to_nxc(summ) if has_sum else None, scales, 0.37 if has_sum else None)
            assert H.last_kernel().startswith("dot_skinny"), H.last_kernel()
            assert np.array_equal(cases.to_ncx(got), exp), (dl, relu, has_sum)
    O.port().orc_set_threads(1)


SPLIT_CONV_SHAPES = [
    # N, C, K, in_sp, f_sp, kw : few output tiles, long reductions that divide into runs of slices
    (1, 256, 256, (14, 14), (3, 3), dict(pad_below=(1, 1), pad_above=(1, 1))),   # 36 slices, 2 x 2 tiles
    (1, 1024, 64, (14, 14), (1, 1), dict()),                                     # 16 slices, one narrow tile
    (2, 512, 144, (9, 9), (1, 1), dict()),                                       # ragged tiles on both sides
    (1, 128, 128, (10, 12), (4, 4), dict(stride=(1, 1), pad_below=(2, 1), pad_above=(1, 2))),
]


def test_conv_bias_in_accumulator(gpu_lib):
    """short reductions add small biases to the accumulators as integers (exact: no float rounding
    happens below 2^24); a column block holding a bias beyond 2^24 keeps the float add -- both kinds
    in one call, with and without a residual, against the oracle"""
    say("bias folding")
    O.port().orc_set_threads(8)
    N, Cc, K, sp = 2, 64, 256, (12, 11)
    dn = H.make_conv_desc(N, Cc, K, sp, (1, 1), out_t="u8")
    d = H.make_conv_desc(N, Cc, K, sp, (1, 1), out_t="u8", data_layout=H.NXC, out_layout=H.NXC)
    data = synth.uniform_int(3100, dn.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(3101, dn.filter_shape(), -127, 127, np.int8)
    bias = synth.uniform_int(3102, (K,), -(2**24), 2**24, np.int32)
    bias[5] = 2**24          # still exact
    bias[7] = -(2**24)
    bias[200] = 2**25 + 3    # second column block: rounds as a float, so that block must not fold
    bias[201] = -(2**26) - 5
    scales = synth.uniform_f32(3103, (K,), 2e-6, 6e-6)
    for has_sum in (False, True):
        summ = synth.uniform_int(3104, dn.out_shape(), 0, 255, np.uint8) if has_sum else None
        f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="u8", with_relu=True, scale_count=K)
        exp = O.quantized_convolution_fused(dn, f, data, filt, bias, summ, scales, 0.21 if has_sum else None)
        got = H.quantized_convolution_fused(d, f, cases.to_nxc(data), filt, bias, cases.to_nxc(summ) if has_sum else None, scales, 0.21 if has_sum else None)
        assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
        assert np.array_equal(cases.to_ncx(got), exp), has_sum
        assert len(np.unique(exp)) > 50  # the outputs are spread, not saturated
    O.port().orc_set_threads(1)


def _conv_sweep():
    """seeded channels-last layers of the kinds a ResNet holds -- 1 x 1 and 3 x 3, stride 1 and 2, 64 to
    512 channels either side, with and without a residual -- at image sizes and batches that put their
    tile counts on both sides of the dispatch edges (pointwise / tile kernels, 64- and 128-byte
    slices, 64 x 128 tiles, split reductions)"""
    rng = np.random.default_rng(777)
    out = []
    for _ in range(60):
        Cc = int(rng.choice([64, 128, 256, 512]))
        K = int(rng.choice([64, 128, 256, 512]))
        r = int(rng.choice([1, 1, 3]))
        st = int(rng.choice([1, 1, 2]))
        hw = int(rng.choice([7, 10, 14, 21, 28]))
        N = int(rng.choice([1, 2, 5, 9]))
        res = bool(rng.integers(0, 2)) and st == 1
        ho = (hw + 2 * (r // 2) - r) // st + 1
        if N * ho * ho * K * Cc * r * r <= 600_000_000:
            out.append((N, Cc, K, hw, r, st, res))
    return sorted(set(out))[:30]


@pytest.mark.parametrize("case", _conv_sweep())
def test_conv_fused_nxc_sweep(gpu_lib, case):
    """QuantizedConvolutionBias(+Add)+ReLU, channels-last in and out, over seeded ResNet-like layers, against the oracle"""
    N, Cc, K, hw, r, st, res = case
    say("conv fused nxc sweep", case)
    O.port().orc_set_threads(8)
    pad = (r // 2, r // 2)
    kw = dict(stride=(st, st), pad_below=pad, pad_above=pad, out_t="u8")
    dn = H.make_conv_desc(N, Cc, K, (hw, hw), (r, r), **kw)
    d = H.make_conv_desc(N, Cc, K, (hw, hw), (r, r), data_layout=H.NXC, out_layout=H.NXC, **kw)
    data = synth.uniform_int(3301, dn.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(3302, dn.filter_shape(), -127, 127, np.int8)
    bias = synth.uniform_int(3303, (K,), -20000, 20000, np.int32)
    scales = synth.uniform_f32(3304, (K,), 1e-3, 3e-3) * np.float32(8.0 / (r * np.sqrt(Cc)))
    summ = synth.uniform_int(3305, dn.out_shape(), 0, 255, np.uint8) if res else None
    f = H.make_fused_desc(has_bias=True, has_sum=res, sum_t="u8", with_relu=True, scale_count=K)
    exp = O.quantized_convolution_fused(dn, f, data, filt, bias, summ, scales, 0.3 if res else None)
    got = H.quantized_convolution_fused(d, f, cases.to_nxc(data), filt, bias, cases.to_nxc(summ) if res else None, scales, 0.3 if res else None)
    assert np.array_equal(cases.to_ncx(got), exp), (case, H.last_kernel())
    assert len(np.unique(exp)) > 20, case
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("i", range(len(SPLIT_CONV_SHAPES)))
def test_conv_register_staged(gpu_lib, i, monkeypatch):
    """the same shapes through the register-staged kernels (windows over multiples of 64 channels
    take the kernels whose loads go straight into LDS unless this switch is set; there, padding
    with a non-zero data zero point is patched in after the load)"""
    monkeypatch.setenv("HIPQ_NO_CONV_DMA", "1")
    test_conv_split_reduction(gpu_lib, i)


@pytest.mark.parametrize("stride", [1, 2])
def test_conv_deep_slices_padding(gpu_lib, stride, monkeypatch):
    """windows over 128 channels with enough tiles to take the 128-byte-deep slices (two operand
    buffers): padded borders with a non-zero data zero point are patched in after the loads land,
    one slice ahead instead of two; both policies, against the oracle and the regular slices"""
    say("conv deep slices with padding, stride", stride)
    N, Cc, K = (4, 128, 128) if stride == 1 else (16, 128, 256)
    in_sp, f_sp = (56, 56), (3, 3)
    kw = dict(stride=(stride, stride), pad_below=(1, 1), pad_above=(1, 1))
    O.port().orc_set_threads(8)
    d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="u8", data_layout=H.NXC, out_layout=H.NXC, **kw)
    dn = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="u8", **kw)
    data = synth.uniform_int(3100 + stride, dn.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(3200, dn.filter_shape(), -128, 127, np.int8)
    for z in ((131, 0, 7), (0, 0, 0)):
        s = (0.02, 0.005, 2.5)
        exp = O.quantized_convolution(dn, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
        got = H.quantized_convolution(d, cases.to_nxc(data), filt, s[0], z[0], s[1], z[1], s[2], z[2])
        assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
        assert np.array_equal(cases.to_ncx(got), exp), z
        assert len(np.unique(exp)) > 50
        monkeypatch.setenv("HIPQ_NO_DEEP_SLICES", "1")
        regular = H.quantized_convolution(d, cases.to_nxc(data), filt, s[0], z[0], s[1], z[1], s[2], z[2])
        monkeypatch.delenv("HIPQ_NO_DEEP_SLICES")
        assert np.array_equal(regular, got), z
    df = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="i8", data_layout=H.NXC, out_layout=H.NXC, **kw)
    dfn = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="i8", **kw)
    f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=K)
    bias = synth.uniform_int(3300, (K,), -20000, 20000, np.int32)
    scales = synth.uniform_f32(3301, (K,), 2e-4, 9e-4)
    exp = O.quantized_convolution_fused(dfn, f, data, filt, bias, None, scales, None)
    got = H.quantized_convolution_fused(df, f, cases.to_nxc(data), filt, bias, None, scales, None)
    assert np.array_equal(cases.to_ncx(got), exp)
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("i", range(len(SPLIT_CONV_SHAPES)))
def test_conv_split_forced(gpu_lib, i, monkeypatch):
    """the same shapes with every reduction cut in two whatever the launch heuristic would choose"""
    monkeypatch.setenv("HIPQ_SPLIT_K", "2")
    test_conv_split_reduction(gpu_lib, i)


@pytest.mark.parametrize("i", range(len(SPLIT_CONV_SHAPES)))
def test_conv_split_reduction(gpu_lib, i):
    """few tiles with long reductions: the pipelined kernel cuts each reduction over several
    workgroups, which meet through partial sums and a counter that the last one resets; called
    several times in a row (the counters must be back at zero), both policies, zero points, residual"""
    N, Cc, K, in_sp, f_sp, kw = SPLIT_CONV_SHAPES[i]
    say("split conv", SPLIT_CONV_SHAPES[i])
    O.port().orc_set_threads(8)
    d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="u8", data_layout=H.NXC, out_layout=H.NXC, **kw)
    dn = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t="u8", **kw)
    for rep, z in enumerate(((0, 0, 0), (131, 0, 7), (9, -7, 1))):
        data = synth.uniform_int(2100 + i + rep, dn.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(2200 + i, dn.filter_shape(), -128, 127, np.int8)
        s = (0.02, 0.005, 0.9)
        exp = O.quantized_convolution(dn, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
        got = H.quantized_convolution(d, cases.to_nxc(data), filt, s[0], z[0], s[1], z[1], s[2], z[2])
        assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
        assert np.array_equal(cases.to_ncx(got), exp), z
    for rep, (relu, has_sum) in enumerate(((True, True), (False, False), (True, True))):
        out_t = "u8" if relu else "i8"
        d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, data_layout=H.NXC, out_layout=H.NXC, **kw)
        dn = H.make_conv_desc(N, Cc, K, in_sp, f_sp, out_t=out_t, **kw)
        data = synth.uniform_int(2300 + i + rep, dn.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(2400 + i, dn.filter_shape(), -127, 127, np.int8)
        bias = synth.uniform_int(2500, (K,), -20000, 20000, np.int32)
        scales = synth.uniform_f32(2501, (K,), 2e-4, 9e-4)
        summ = synth.uniform_int(2502, dn.out_shape(), 0, 255, np.uint8) if has_sum else None
        f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="u8", with_relu=relu, scale_count=K)
        exp = O.quantized_convolution_fused(dn, f, data, filt, bias, summ, scales, 0.37 if has_sum else None)
        got = H.quantized_convolution_fused(d, f, cases.to_nxc(data), filt, bias, cases.to_nxc(summ) if has_sum else None, scales, 0.37 if has_sum else None)
        assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
        assert np.array_equal(cases.to_ncx(got), exp), (relu, has_sum)
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("image,pads", [((30, 26), ((3, 3), (3, 3))), ((30, 28), ((3, 3), (3, 3))), ((19, 32), ((2, 5), (4, 0)))], ids=["rows26", "rows28", "rows32_uneven_pads"])
@pytest.mark.parametrize("K", [24, 32])
@pytest.mark.parametrize("Cc", [1, 3, 4, 15])
def test_conv_few_input_channels(gpu_lib, Cc, K, image, pads):
    """a network's first layer (3 input channels, 7x7 stride 2): the data is padded to 16 channels on
    the way into the MFMA kernel, or -- at most four channels, channels-last 8-bit output in whole
    16-byte pixels (K = 32 here) -- staged with its padding so that a filter row is one 32-byte run;
    both policies, both layouts, zero points on every operand (a filter zero point takes the exact path);
    image rows of 28 and 32 bytes in NCHW take the staging kernel that moves whole dwords, rows of 26 the
    one that moves bytes"""
    say("first-layer conv", Cc, K, image, pads)
    O.port().orc_set_threads(8)
    kw = dict(stride=(2, 2), pad_below=pads[0], pad_above=pads[1])
    for dl, ol in ((H.NCX, H.NCX), (H.NXC, H.NXC), (H.NCX, H.NXC)):
        for out_t, z in (("i8", (0, 0, 0)), ("u8", (119, 0, 3)), ("i8", (7, -5, 0))):
            d = H.make_conv_desc(2, Cc, K, image, (7, 7), out_t=out_t, data_layout=dl, out_layout=ol, **kw)
            dn = H.make_conv_desc(2, Cc, K, image, (7, 7), out_t=out_t, **kw)
            data = synth.uniform_int(700 + Cc, dn.data_shape(), 0, 255, np.uint8)
            filt = synth.uniform_int(800 + Cc, dn.filter_shape(), -128, 127, np.int8)
            exp = O.quantized_convolution(dn, data, filt, 0.02, z[0], 0.01, z[1], 0.8, z[2])
            got = H.quantized_convolution(d, cases.to_nxc(data) if dl == H.NXC else data, filt, 0.02, z[0], 0.01, z[1], 0.8, z[2])
            assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
            assert np.array_equal(cases.to_ncx(got) if ol == H.NXC else got, exp), (dl, ol, out_t, z)
        d = H.make_conv_desc(2, Cc, K, image, (7, 7), out_t="u8", data_layout=dl, out_layout=ol, **kw)
        dn = H.make_conv_desc(2, Cc, K, image, (7, 7), out_t="u8", **kw)
        data = synth.uniform_int(900 + Cc, dn.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(901 + Cc, dn.filter_shape(), -127, 127, np.int8)
        bias = synth.uniform_int(902, (K,), -5000, 5000, np.int32)
        scales = synth.uniform_f32(903, (K,), 1e-4, 6e-4)
        f = H.make_fused_desc(has_bias=True, with_relu=True, scale_count=K)
        exp = O.quantized_convolution_fused(dn, f, data, filt, bias, None, scales, None)
        got = H.quantized_convolution_fused(d, f, cases.to_nxc(data) if dl == H.NXC else data, filt, bias, None, scales, None)
        assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
        assert np.array_equal(cases.to_ncx(got) if ol == H.NXC else got, exp), (dl, ol, "fused")
    O.port().orc_set_threads(1)


def test_first_layer_staging_kernels_agree(gpu_lib, monkeypatch):
    """the padded copy of a first layer written four pixels a lane (image rows of whole dwords) and
    pixel by pixel: same convolution, both data layouts, at ResNet-50's stem geometry (batch 2)"""
    say("first-layer staging, dwords vs bytes")
    kw = dict(stride=(2, 2), pad_below=(3, 3), pad_above=(3, 3))
    for dl in (H.NCX, H.NXC):
        d = H.make_conv_desc(2, 3, 64, (224, 224), (7, 7), out_t="u8", data_layout=dl, out_layout=H.NXC, **kw)
        dn = H.make_conv_desc(2, 3, 64, (224, 224), (7, 7), out_t="u8", **kw)
        data = synth.uniform_int(910, dn.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(911, dn.filter_shape(), -127, 127, np.int8)
        x = cases.to_nxc(data) if dl == H.NXC else data
        monkeypatch.delenv("HIPQ_NO_STAGE_QUADS", raising=False)
        a = H.quantized_convolution(d, x, filt, 0.02, 5, 0.01, 0, 0.9, 128)
        monkeypatch.setenv("HIPQ_NO_STAGE_QUADS", "1")
        b = H.quantized_convolution(d, x, filt, 0.02, 5, 0.01, 0, 0.9, 128)
        monkeypatch.delenv("HIPQ_NO_STAGE_QUADS")
        assert np.array_equal(a, b), dl
        assert len(np.unique(a)) > 50  # a real spread of outputs, not a saturated tensor


def test_conv_band_matches_generic_kernel(gpu_lib, monkeypatch):
    """the band kernel and the generic implicit-GEMM kernel agree byte for byte at a size the oracle
    does not reach (BASELINE config 1 at batch 16, wrapping requantization included)"""
    say("band vs generic")
    d = H.make_conv_desc(16, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    data = synth.uniform_int(701, d.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(702, d.filter_shape(), -127, 127, np.int8)
    r = H.quantized_convolution(d, data, filt, 0.02, 0, 0.005, 0, 0.1, 0)
    assert H.last_kernel().startswith("conv_regw"), H.last_kernel()  # NCHW out, 3x3 over 64 channels: filter in registers
    monkeypatch.setenv("HIPQ_NO_REGW", "1")
    a = H.quantized_convolution(d, data, filt, 0.02, 0, 0.005, 0, 0.1, 0)
    assert H.last_kernel().startswith("conv_band"), H.last_kernel()
    monkeypatch.setenv("HIPQ_NO_BAND", "1")
    b = H.quantized_convolution(d, data, filt, 0.02, 0, 0.005, 0, 0.1, 0)
    assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
    assert np.array_equal(a, b) and np.array_equal(r, a)


# ------------------------------------------------------------------ QuantizedDot


def test_dot_kats(gpu_lib, kats):
    for k in kats["dot"]:
        say(k["name"])
        M, K = k["a_shape"]
        N = k["b_shape"][1]
        d = H.make_dot_desc(M, K, N, a_t=k["a_t"], b_t=k["b_t"], out_t=k["out_t"])
        a = np.array(k["a"], dtype=H.NP_OF[d.a_t]).reshape(M, K)
        b = np.array(k["b"], dtype=H.NP_OF[d.b_t]).reshape(K, N)
        s, z = k["scales"], k["zps"]
        got = H.quantized_dot(d, a, b, s[0], z[0], s[1], z[1], s[2], z[2])
        assert got.reshape(-1).tolist() == k["expected"], k["name"]


def test_dot_reference_vectors(gpu_lib, ref_vectors):
    manifest, arrays = ref_vectors
    used = set()
    for m in manifest:
        if m["kind"] != "dot":
            continue
        say(m["name"])
        d, a, b, s, z = cases.dot_from_manifest(m)
        for prepare in (False, True):
            got = H.quantized_dot(d, a, b, s[0], z[0], s[1], z[1], s[2], z[2], prepare=prepare)
            used.add(H.last_kernel())
            assert np.array_equal(got, arrays[m["name"]]), (m["name"], prepare, H.last_kernel())
    assert "dot_direct" in used and any(k.startswith(("dot_mfma", "dot_skinny")) for k in used), used


@pytest.mark.parametrize("M", [1, 32, 256, 130])
def test_dot_mfma_vs_oracle(gpu_lib, M):
    say("dot mfma M", M)
    K, N = 512, 384
    a = synth.uniform_int(81, (M, K), 0, 255, np.uint8)
    b = synth.uniform_int(82, (K, N), -127, 127, np.int8)
    O.port().orc_set_threads(8)
    for out_t, s, z in (("i32", (1.0, 1.0, 1.0), (0, 0, 0)), ("i8", (0.01, 0.01, 2.5), (0, 0, 4)), ("i8", (0.01, 0.01, 2.5), (9, 0, 0)), ("i8", (0.01, 0.01, 2.5), (9, 3, 0))):
        d = H.make_dot_desc(M, K, N, out_t=out_t)
        exp = O.quantized_dot(d, a, b, s[0], z[0], s[1], z[1], s[2], z[2])
        got = H.quantized_dot(d, a, b, s[0], z[0], s[1], z[1], s[2], z[2])
        assert H.last_kernel().startswith(("dot_mfma", "dot_skinny", "dot_rows64")), H.last_kernel()
        assert np.array_equal(got, exp), (out_t, z)
    O.port().orc_set_threads(1)


def test_dot_bias_kat(gpu_lib, kats):
    k = kats["dot_bias"]
    say(k["name"])
    lib = O.port()
    M, K = k["a_shape"]
    N = k["w_shape"][0]
    a = np.array(k["a"], dtype=np.uint8).reshape(M, K)
    w = np.array(k["w"], dtype=np.int8).reshape(N, K)
    r = k["in_range"] + k["filter_range"] + k["out_range"]
    for requant, relu, key, out_t in ((0, 0, "expected_f32", "f32"), (0, 1, "expected_f32_relu", "f32"), (1, 0, "expected_i8", "i8"), (1, 1, "expected_u8_relu", "u8")):
        scale = lib.orc_get_dot_scale(*r, H.U8, H.U8 if relu else H.I8, requant)
        d = H.make_dot_desc(M, K, N, out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=bool(relu))
        got = H.quantized_dot_bias(d, f, a, w, k["bias"], scale)
        assert np.array_equal(got, np.array(k[key], dtype=got.dtype).reshape(M, N)), key


@pytest.mark.parametrize("M", [1, 32, 256])
def test_dot_bias_config2_shape(gpu_lib, M):
    """BASELINE config 2 at K = N = 1024 (the oracle needs minutes at 4096): per-output-channel
    scales, int32 bias, requantize to i8; and the f32 / relu variants"""
    say("config2 M", M)
    K = N = 1024
    a = synth.uniform_int(91, (M, K), 0, 255, np.uint8)
    w = synth.uniform_int(92, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(93, (N,), -(2**15), 2**15, np.int32)
    scales = synth.uniform_f32(94, (N,), 0.001, 0.01) * np.float32(0.02)
    O.port().orc_set_threads(8)
    for out_t, relu in (("i8", False), ("u8", True), ("f32", False), ("f32", True)):
        d = H.make_dot_desc(M, K, N, out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
        exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
        got = H.quantized_dot_bias(d, f, a, w, bias, scales)
        assert H.last_kernel().startswith(("dot_mfma", "dot_skinny", "dot_rows64")), H.last_kernel()
        assert np.array_equal(got, exp), (out_t, relu)
        assert len(np.unique(exp)) > 20  # the case is not degenerate (all saturated)
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("shape", [(200, 192, 144), (130, 4096, 64), (333, 768, 272), (4096, 64, 128)])
def test_dot_bias_f32_tiles(gpu_lib, shape, monkeypatch):
    """float outputs of QuantizedDotBias through the tile kernels: ragged row and column tiles, a
    long reduction that is split over workgroups, a single-slice reduction; small biases (added to
    the accumulators as integers) and one beyond 2^24 (kept as a float add); with and without relu"""
    M, K, N = shape
    say("dot bias f32 tiles", shape)
    O.port().orc_set_threads(8)
    for a_t, lo, hi in (("u8", 0, 255), ("i8", -128, 127)):
        a = synth.uniform_int(1201, (M, K), lo, hi, np.uint8 if a_t == "u8" else np.int8)
        w = synth.uniform_int(1202, (N, K), -127, 127, np.int8)
        for big_bias in (False, True):
            bias = synth.uniform_int(1203, (N,), -(2**15), 2**15, np.int32)
            if big_bias:
                bias[N // 2] = 2**26 + 12345
            scales = synth.uniform_f32(1204, (N,), 0.001, 0.01) * np.float32(0.03)
            for relu in (False, True):
                d = H.make_dot_desc(M, K, N, a_t=a_t, out_t="f32", b_layout=H.B_NK)
                f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
                exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
                got = H.quantized_dot_bias(d, f, a, w, bias, scales)
                # (up to 256 rows with a long reduction and few tiles: one workgroup per 64 x 64 tile, whole reduction)
                rows64 = 64 < M <= 256 and K >= 1024
                assert H.last_kernel().startswith("dot_rows64" if rows64 else "dot_mfma"), H.last_kernel()
                assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), (a_t, big_bias, relu)
                if rows64:
                    monkeypatch.setenv("HIPQ_NO_ROWS64", "1")
                    got = H.quantized_dot_bias(d, f, a, w, bias, scales)
                    monkeypatch.delenv("HIPQ_NO_ROWS64")
                    assert H.last_kernel().startswith("dot_mfma"), H.last_kernel()
                    assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), (a_t, big_bias, relu, "tiles")
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("shape", [(512, 256, 384), (1024, 128, 640), (12288, 64, 1024), (16384, 64, 1152), (5000, 192, 400), (2048, 512, 1152)])
def test_dot_tile_order(gpu_lib, shape):
    """the persistent tile kernels number their tiles in groups of column blocks (squares per
    compute die): full groups of 2, 4 and 8, a narrower last group, more tiles than resident
    workgroups, ragged edges -- every output element must still be written exactly once"""
    M, K, N = shape
    say("dot tile order", shape)
    O.port().orc_set_threads(8)
    a = synth.uniform_int(1301, (M, K), 0, 255, np.uint8)
    w = synth.uniform_int(1302, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(1303, (N,), -(2**15), 2**15, np.int32)
    scales = synth.uniform_f32(1304, (N,), 0.001, 0.01) * np.float32(0.05)
    for out_t, relu in (("i8", False), ("u8", True), ("f32", False)):
        d = H.make_dot_desc(M, K, N, a_t="u8", out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
        exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
        got = H.quantized_dot_bias(d, f, a, w, bias, scales)
        assert H.last_kernel().startswith("dot_mfma"), H.last_kernel()
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (out_t, relu)
        assert len(np.unique(exp)) > 20
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("shape", [(1000, 768, 400), (2000, 512, 1104), (4096, 768, 768)])
def test_dot_half_height_tiles(gpu_lib, shape, monkeypatch):
    """row matrices whose 128 x 128 tiles would leave compute units idle run on 64 x 128 tiles with
    whole reductions: ragged last tiles in both directions, 8-bit and float outputs, against the
    oracle and against the 128 x 128 tiles (reductions split over workgroups) behind the switch"""
    M, K, N = shape
    say("dot half-height tiles", shape)
    O.port().orc_set_threads(8)
    a = synth.uniform_int(1451, (M, K), 0, 255, np.uint8)
    w = synth.uniform_int(1452, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(1453, (N,), -(2**15), 2**15, np.int32)
    scales = synth.uniform_f32(1454, (N,), 0.001, 0.01) * np.float32(0.03)
    for out_t, relu in (("i8", False), ("u8", True), ("f32", False)):
        d = H.make_dot_desc(M, K, N, a_t="u8", out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
        exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
        got = H.quantized_dot_bias(d, f, a, w, bias, scales)
        assert H.last_kernel().startswith("dot_mfma"), H.last_kernel()
        monkeypatch.setenv("HIPQ_NO_HALF_TILES", "1")
        full = H.quantized_dot_bias(d, f, a, w, bias, scales)
        monkeypatch.delenv("HIPQ_NO_HALF_TILES")
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (out_t, relu)
        assert np.array_equal(full.view(np.uint8), exp.view(np.uint8)), (out_t, relu, "128 x 128")
        assert len(np.unique(exp)) > 20
    O.port().orc_set_threads(1)


def _sweep_shapes():
    """seeded shapes around the tile kernels' dispatch edges: rows just past 64 and 128, column counts
    that are not whole tiles, reductions from one 64-byte slice to 2048 bytes (whole 128-byte pieces and
    not), tile counts below and above the compute units"""
    rng = np.random.default_rng(20240)
    shapes = []
    for _ in range(28):
        M = int(rng.choice([65, 96, 129, 200, 257, 384, 640, 1000, 1536, 2500, 4100]))
        K = int(rng.choice([64, 128, 192, 256, 320, 512, 768, 1024, 1408, 2048]))
        N = int(rng.choice([16, 48, 64, 80, 128, 144, 256, 400, 768, 1104]))
        if M * K * N <= 1_500_000_000:
            shapes.append((M, K, N))
    return sorted(set(shapes))


@pytest.mark.parametrize("shape", _sweep_shapes())
def test_dot_dispatch_sweep(gpu_lib, shape):
    """QuantizedDotBias over shapes drawn around the dispatch edges, 8-bit and float outputs, against the oracle"""
    M, K, N = shape
    say("dot dispatch sweep", shape)
    O.port().orc_set_threads(8)
    a = synth.uniform_int(1501, (M, K), 0, 255, np.uint8)
    w = synth.uniform_int(1502, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(1503, (N,), -(2**15), 2**15, np.int32)
    scales = synth.uniform_f32(1504, (N,), 0.001, 0.01) * np.float32(40.0 / K)
    for out_t, relu in (("u8", True), ("f32", False)):
        d = H.make_dot_desc(M, K, N, a_t="u8", out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
        exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
        got = H.quantized_dot_bias(d, f, a, w, bias, scales)
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (shape, out_t, H.last_kernel())
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("split", ["2", "4"])
def test_dot_deep_slices_split(gpu_lib, split, monkeypatch):
    """reductions in whole 128-byte pieces run with slices twice as deep and two operand buffers;
    here with the reduction also cut over workgroups, and against the regular slices"""
    say("dot deep slices, split", split)
    M, K, N = 300, 1024, 272
    O.port().orc_set_threads(8)
    a = synth.uniform_int(1401, (M, K), -128, 127, np.int8)
    w = synth.uniform_int(1402, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(1403, (N,), -(2**15), 2**15, np.int32)
    scales = synth.uniform_f32(1404, (N,), 0.001, 0.01) * np.float32(0.05)
    for out_t in ("i8", "f32"):
        d = H.make_dot_desc(M, K, N, a_t="i8", out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=N)
        exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
        monkeypatch.setenv("HIPQ_SPLIT_K", split)
        got = H.quantized_dot_bias(d, f, a, w, bias, scales)
        monkeypatch.setenv("HIPQ_NO_DEEP_SLICES", "1")
        regular = H.quantized_dot_bias(d, f, a, w, bias, scales)
        monkeypatch.delenv("HIPQ_NO_DEEP_SLICES")
        monkeypatch.delenv("HIPQ_SPLIT_K")
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), out_t
        assert np.array_equal(regular.view(np.uint8), exp.view(np.uint8)), out_t
    O.port().orc_set_threads(1)


def test_dot_config2_full_size_properties(gpu_lib):
    """config 2 at its real size [256,4096] x [4096,4096]: rows of the M=256 result equal the
    M=1 / M=32 results (launch geometry independence), and int32 accumulators of a row subset
    match numpy's int64 matmul"""
    say("config2 full size")
    K = N = 4096
    a = synth.uniform_int(95, (256, K), 0, 255, np.uint8)
    w = synth.uniform_int(96, (N, K), -127, 127, np.int8)
    d = H.make_dot_desc(256, K, N, out_t="i32", b_layout=H.B_NK)
    got = H.quantized_dot(d, a, w, 1.0, 0, 1.0, 0, 1.0, 0)
    assert H.last_kernel().startswith("dot_rows64"), H.last_kernel()
    rows = [0, 1, 31, 32, 127, 128, 255]
    exp = a[rows].astype(np.int64) @ w.astype(np.int64).T
    assert np.array_equal(got[rows].astype(np.int64), exp)
    for M in (1, 32):
        dm = H.make_dot_desc(M, K, N, out_t="i32", b_layout=H.B_NK)
        gm = H.quantized_dot(dm, a[:M], w, 1.0, 0, 1.0, 0, 1.0, 0)
        assert np.array_equal(gm, got[:M])


@pytest.mark.parametrize("M", [1, 32, 256])
def test_dot_bias_config2_benchmarked_form(gpu_lib, M):
    """BASELINE config 2 exactly as bench.py times it: QuantizedDotBias u8 [M,4096] x i8 [4096,4096]
    ([N,K] weights, prepacked), int32 bias, per-output-channel scales, requantized to i8 -- on the
    kernel the bench reports for that M -- against the closed form of tests/cases.py (float64 BLAS
    sums, numpy float32 post-ops, rint + clip), which test_oracle_conv_dot.py also holds the oracle
    to.  The u8 + relu and f32 forms ride along."""
    say("config2 benchmarked form, M", M)
    K = N = 4096
    a = synth.uniform_int(2001, (M, K), 0, 255, np.uint8)
    w = synth.uniform_int(2002, (N, K), -127, 127, np.int8)
    bias = synth.uniform_int(2003, (N,), -(2**15), 2**15, np.int32)
    scales = synth.uniform_f32(2004, (N,), 0.001, 0.01)
    # BASELINE's weight scales; the data and output scales fold into the same per-channel factor
    scales = (scales * np.float32(0.02)).astype(np.float32)
    for out_t, relu in (("i8", False), ("u8", True), ("f32", False)):
        d = H.make_dot_desc(M, K, N, out_t=out_t, b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
        got = H.quantized_dot_bias(d, f, a, w, bias, scales)
        kernel = H.last_kernel()
        exp = cases.dot_bias_closed_form(a, w, bias, scales, out_t, relu)
        assert np.array_equal(got, exp), (out_t, relu, kernel, int(np.sum(got != exp)))
        if out_t == "i8":
            # the kernels bench.py's gemm_config2 entries name (prepacked weights: the fragment-ordered copy):
            # weight-streaming up to 32 rows, 64 x 64 tiles with the whole reduction above
            assert kernel == ("dot_skinnyf_i8_16x16x64" if M <= 32 else "dot_rows64w_i8_16x16x64"), kernel
            assert len(np.unique(exp)) > 100 and (exp == 127).any() and (exp == -128).any()


@pytest.mark.parametrize("M", [1, 7, 16, 17, 33, 64, 100, 129, 256])
def test_dot_skinny(gpu_lib, M):
    """the weight-streaming kernel for a handful of rows: ragged row and column tiles, a reduction
    that does not split evenly over the four wavefronts, signed and unsigned data, zero points,
    both requantization policies, f32 output, and the exact path for a non-zero weight zero point"""
    say("dot skinny M", M)
    O.port().orc_set_threads(8)

    def kernel_of(tiles, K, prepacked):
        # prepacked weights carry a fragment-ordered copy, which the kernels for up to 32 rows (reductions
        # up to 4096 bytes; 8192 with at most 16 rows) and for 65-256 rows read; weights packed on the fly
        # take the kernels that read the row-major matrix
        if M > 64 and K >= 1024:
            return "dot_rows64w_" if prepacked else "dot_rows64_"
        if tiles:
            return "dot_mfma"
        if prepacked and (M <= 16 and K <= 8192 or M <= 32 and K <= 4096):
            return "dot_skinnyf_"
        return "dot_skinny_"

    # (a reduction of five 64-byte steps, one that splits evenly, the shortest one, and -- for the
    # fragment-ordered kernels -- one of two 1 KB segments a wavefront and one that leaves a wavefront
    # a partial segment)
    shapes = ((320, 40), (1024, 100), (256, 16)) + (((8192, 24), (2880, 20)) if M <= 32 else ())
    for K, N in shapes:
        w = synth.uniform_int(802, (N, K), -128, 127, np.int8)
        for a_t, lo, hi in (("u8", 0, 255), ("i8", -128, 127)):
            a = synth.uniform_int(801, (M, K), lo, hi, H.NP_OF[H.dtype_code(a_t)])
            for prepacked in (True, False):
                if not prepacked and K > 1024:
                    continue
                for out_t, s, z in (("i32", (1.0, 1.0, 1.0), (0, 0, 0)), ("i8", (0.01, 0.01, 2.5), (5 if a_t == "u8" else -5, 0, 4)), ("u8", (0.01, 0.01, 2.5), (0, 3, 9))):
                    d = H.make_dot_desc(M, K, N, a_t=a_t, out_t=out_t, b_layout=H.B_NK)
                    exp = O.quantized_dot(d, a, w, s[0], z[0], s[1], z[1], s[2], z[2])
                    got = H.quantized_dot(d, a, w, s[0], z[0], s[1], z[1], s[2], z[2], prepare=prepacked)
                    # (more than 64 rows with an 8-bit output in whole 16-byte rows go to the tile kernels)
                    want = kernel_of(M > 64 and out_t != "i32" and N % 16 == 0, K, prepacked)
                    assert H.last_kernel().startswith(want), (H.last_kernel(), want)
                    assert np.array_equal(got, exp), (K, N, a_t, out_t, z, prepacked)
                bias = synth.uniform_int(803, (N,), -(2**15), 2**15, np.int32)
                scales = synth.uniform_f32(804, (N,), 0.001, 0.01) * np.float32(0.05)
                for out_t, relu in (("i8", False), ("u8", True), ("f32", True)):
                    d = H.make_dot_desc(M, K, N, a_t=a_t, out_t=out_t, b_layout=H.B_NK)
                    f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
                    exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
                    got = H.quantized_dot_bias(d, f, a, w, bias, scales, prepare=prepacked)
                    want = kernel_of(M > 64 and N % 16 == 0, K, prepacked)
                    assert H.last_kernel().startswith(want), (H.last_kernel(), want)
                    assert np.array_equal(got, exp), (K, N, a_t, out_t, relu, prepacked)
    O.port().orc_set_threads(1)


# ------------------------------------------------------------------ layout helpers


@pytest.mark.parametrize("eb", [1, 4])
def test_transposes(gpu_lib, eb):
    say("transpose", eb)
    dt = np.uint8 if eb == 1 else np.int32
    for (N, Cc, X) in ((2, 64, 3136), (3, 5, 7), (1, 130, 67), (3, 48, 80), (1, 256, 208), (2, 16, 16), (1, 144, 400)):
        a = synth.uniform_int(5, (N, Cc, X), 0, 255, np.uint8).astype(dt)
        src = H.DeviceBuffer.from_numpy(a)
        dst = H.DeviceBuffer(a.nbytes)
        H.check(gpu_lib.hipq_transpose_ncx_to_nxc(src.ptr, dst.ptr, N, Cc, X, eb, None))
        t = dst.to_numpy(dt, (N, X, Cc))
        assert np.array_equal(t, np.transpose(a, (0, 2, 1)))
        back = H.DeviceBuffer(a.nbytes)
        H.check(gpu_lib.hipq_transpose_nxc_to_ncx(dst.ptr, back.ptr, N, Cc, X, eb, None))
        assert np.array_equal(back.to_numpy(dt, (N, Cc, X)), a)


def test_mfma_requant_ties(gpu_lib):
    """exact .5 ties of both signs and both parities on the MFMA path: half away from zero for the
    INTERPRETER policy, half to even for the fused policy"""
    say("requant ties")
    K, N, M = 16, 64, 40
    a = np.zeros((M, K), np.uint8)
    a[:, 0] = 1  # acc[m, n] = w[n, 0]: every integer in [-32, 31]
    w = np.zeros((N, K), np.int8)
    w[:, 0] = np.arange(N) - 32
    exp_acc = np.tile(w[:, 0].astype(np.int32), (M, 1))
    d = H.make_dot_desc(M, K, N, out_t="i8", b_layout=H.B_NK)
    got = H.quantized_dot(d, a, w, 0.5, 0, 1.0, 0, 1.0, 0)
    assert H.last_kernel().startswith(("dot_mfma", "dot_skinny")), H.last_kernel()
    half_away = np.sign(exp_acc) * np.floor(np.abs(exp_acc) / 2 + 0.5)
    assert np.array_equal(got.astype(np.int64), half_away.astype(np.int64))
    assert np.array_equal(got, O.quantized_dot(d, a, w, 0.5, 0, 1.0, 0, 1.0, 0))
    f = H.make_fused_desc(has_bias=False)
    got = H.quantized_dot_bias(d, f, a, w, None, 0.5)
    assert np.array_equal(got.astype(np.int64), np.rint(exp_acc / 2).astype(np.int64))
    assert np.array_equal(got, O.quantized_dot_bias(d, f, a, w, None, 0.5))
    # a scale >= 1 takes the out-of-range-aware conversion; 2^31-sized products give INT32_MIN like x86
    d32 = H.make_dot_desc(M, K, N, out_t="i32", b_layout=H.B_NK)
    for s in (1.5, 3.0e8):
        assert np.array_equal(H.quantized_dot(d32, a, w, s, 0, 1.0, 0, 1.0, 0), O.quantized_dot(d32, a, w, s, 0, 1.0, 0, 1.0, 0)), s
        assert np.array_equal(H.quantized_dot(d, a, w, s, 0, 1.0, 0, 1.0, 5), O.quantized_dot(d, a, w, s, 0, 1.0, 0, 1.0, 5)), s


@pytest.mark.parametrize("shape", [(65, 1088, 64), (200, 1152, 130), (256, 2048, 48), (129, 1024, 1000), (192, 3008, 200), (72, 4096, 40), (130, 4160, 72)])
def test_dot_rows64(gpu_lib, shape):
    """the whole-reduction kernels for 65-256 rows (prepacked weights: the one that reads their
    fragment-ordered copy; weights packed on the fly: the one that reads the row-major matrix): ragged row and column tiles, reductions that end in
    half a 128-byte piece (K % 128 == 64) or leave wavefronts without a piece, signed and unsigned
    data with zero points, both requantization policies, every output type, and the exact path for a
    non-zero weight zero point"""
    M, K, N = shape
    say("dot rows64", shape)
    O.port().orc_set_threads(8)
    w = synth.uniform_int(1502, (N, K), -128, 127, np.int8)
    for a_t, lo, hi in (("u8", 0, 255), ("i8", -128, 127)):
        a = synth.uniform_int(1501, (M, K), lo, hi, H.NP_OF[H.dtype_code(a_t)])
        for out_t, s, z in (("i32", (1.0, 1.0, 1.0), (0, 0, 0)), ("i8", (0.01, 0.01, 2.5), (5 if a_t == "u8" else -5, 0, 4)), ("u8", (0.01, 0.01, 2.5), (0, 3, 9))):
            d = H.make_dot_desc(M, K, N, a_t=a_t, out_t=out_t, b_layout=H.B_NK)
            exp = O.quantized_dot(d, a, w, s[0], z[0], s[1], z[1], s[2], z[2])
            for prepacked, name in ((True, "dot_rows64w_" if K <= 4096 else "dot_rows64_"), (False, "dot_rows64_")):  # (the fragment-ordered kernel holds a reduction of 4096 bytes in registers)
                got = H.quantized_dot(d, a, w, s[0], z[0], s[1], z[1], s[2], z[2], prepare=prepacked)
                assert H.last_kernel().startswith(name), H.last_kernel()
                assert np.array_equal(got, exp), (a_t, out_t, z, prepacked)
        bias = synth.uniform_int(1503, (N,), -(2**15), 2**15, np.int32)
        scales = synth.uniform_f32(1504, (N,), 0.001, 0.01) * np.float32(0.05)
        for out_t, relu in (("i8", False), ("u8", True), ("f32", True)):
            d = H.make_dot_desc(M, K, N, a_t=a_t, out_t=out_t, b_layout=H.B_NK)
            f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N)
            exp = O.quantized_dot_bias(d, f, a, w, bias, scales)
            for prepacked, name in ((True, "dot_rows64w_" if K <= 4096 else "dot_rows64_"), (False, "dot_rows64_")):  # (the fragment-ordered kernel holds a reduction of 4096 bytes in registers)
                got = H.quantized_dot_bias(d, f, a, w, bias, scales, prepare=prepacked)
                assert H.last_kernel().startswith(name), H.last_kernel()
                assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (a_t, out_t, relu, prepacked)
    O.port().orc_set_threads(1)


def _random_conv_case(rng):
    """a random geometry the reference accepts: 1 to 3 spatial axes, strides, filter and data dilation,
    positive and negative padding, channel counts on and off the matrix kernels' multiples"""
    ns = int(rng.integers(1, 4))
    N = int(rng.integers(1, 4))
    Cc = int(rng.choice([1, 3, 4, 7, 16, 32, 48, 64, 96, 128]))
    K = int(rng.choice([1, 5, 16, 24, 32, 64, 80, 128]))
    limit = {1: 40, 2: 14, 3: 6}[ns]
    for _ in range(100):
        in_sp = [int(rng.integers(1, limit + 1)) for _ in range(ns)]
        f_sp = [int(rng.integers(1, 4)) for _ in range(ns)]
        kw = dict(
            stride=[int(rng.integers(1, 3)) for _ in range(ns)],
            dilation=[int(rng.integers(1, 3)) for _ in range(ns)],
            pad_below=[int(rng.integers(-1, 3)) for _ in range(ns)],
            pad_above=[int(rng.integers(-1, 3)) for _ in range(ns)],
            data_dilation=[int(rng.choice([1, 1, 1, 2])) for _ in range(ns)],
        )
        ok = True
        for i in range(ns):
            padded = (in_sp[i] - 1) * kw["data_dilation"][i] + 1 + kw["pad_below"][i] + kw["pad_above"][i]
            window = (f_sp[i] - 1) * kw["dilation"][i] + 1
            ok = ok and padded >= window and padded >= 1
        if ok:
            return N, Cc, K, in_sp, f_sp, kw
    return N, Cc, K, [4] * ns, [1] * ns, dict()


@pytest.mark.parametrize("block", range(6))
def test_conv_random_geometries(gpu_lib, block):
    """seeded sweep: every case against the oracle, bit for bit, in the reference's layouts and (2-D and
    below) channels-last; INTERPRETER arithmetic with zero points on all three tensors"""
    rng = np.random.default_rng(9000 + block)
    kernels = set()
    for case in range(12):
        N, Cc, K, in_sp, f_sp, kw = _random_conv_case(rng)
        data_t = "u8" if rng.integers(0, 4) else "i8"
        out_t = str(rng.choice(["i8", "u8", "i32"])) if data_t == "u8" else "i32"
        filter_t = "i8" if out_t != "u8" else "u8"
        zps = (int(rng.integers(0, 200)) if data_t == "u8" else int(rng.integers(-100, 100)), int(rng.choice([0, 0, 3])) if filter_t == "i8" else int(rng.choice([0, 130])),
               int(rng.integers(-20, 20)) if out_t != "u8" else int(rng.integers(0, 30)))
        scales = (1.0, 1.0, 1.0) if out_t == "i32" else (0.02, 0.005, float(rng.choice([0.9, 0.05, 2.5])))
        if out_t == "i32":
            zps = (zps[0], zps[1], 0)
        say("random conv", block, case, N, Cc, K, in_sp, f_sp, kw, data_t, filter_t, out_t, zps)
        layouts = [(H.NCX, H.NCX)] + ([(H.NXC, H.NXC), (H.NCX, H.NXC)] if K > 1 else [])
        d0 = H.make_conv_desc(N, Cc, K, in_sp, f_sp, data_t=data_t, filter_t=filter_t, out_t=out_t, **kw)
        data = synth.uniform_int(int(rng.integers(1 << 30)), d0.data_shape(), 0 if data_t == "u8" else -128, 255 if data_t == "u8" else 127, np.uint8 if data_t == "u8" else np.int8)
        filt = synth.uniform_int(int(rng.integers(1 << 30)), d0.filter_shape(), -128 if filter_t == "i8" else 0, 127 if filter_t == "i8" else 255, np.int8 if filter_t == "i8" else np.uint8)
        exp = O.quantized_convolution(d0, data, filt, scales[0], zps[0], scales[1], zps[1], scales[2], zps[2])
        for dl, ol in layouts:
            d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, data_t=data_t, filter_t=filter_t, out_t=out_t, data_layout=dl, out_layout=ol, **kw)
            x = cases.to_nxc(data) if dl == H.NXC else data
            got = H.quantized_convolution(d, x, filt, scales[0], zps[0], scales[1], zps[1], scales[2], zps[2])
            kernels.add(H.last_kernel())
            got = cases.to_ncx(got) if ol == H.NXC else got
            assert np.array_equal(got, exp), (block, case, dl, ol, H.last_kernel())
    print("kernels:", sorted(kernels), flush=True)


@pytest.mark.parametrize("block", range(3))
def test_dot_random_shapes(gpu_lib, block):
    """seeded sweep of QuantizedDot (INTERPRETER arithmetic, [K, N] weights, zero points) and
    QuantizedDotBias (fused arithmetic, [N, K] weights, per-channel scales) against the oracle"""
    rng = np.random.default_rng(9100 + block)
    kernels = set()
    for case in range(10):
        M = int(rng.choice([1, 2, 7, 16, 31, 64, 65, 100, 128, 200, 257, 384]))
        K = int(rng.choice([1, 5, 16, 48, 64, 100, 256, 512, 1024]))
        N = int(rng.choice([1, 3, 16, 40, 64, 100, 128, 208, 512]))
        say("random dot", block, case, M, K, N)
        a_t = "u8"
        b_t = str(rng.choice(["i8", "u8"]))
        out_t = str(rng.choice(["i8", "i32"])) if b_t == "i8" else str(rng.choice(["u8", "i32"]))
        d = H.make_dot_desc(M, K, N, a_t=a_t, b_t=b_t, out_t=out_t)
        a = synth.uniform_int(int(rng.integers(1 << 30)), (M, K), 0, 255, np.uint8)
        b = synth.uniform_int(int(rng.integers(1 << 30)), (K, N), -128 if b_t == "i8" else 0, 127 if b_t == "i8" else 255, np.int8 if b_t == "i8" else np.uint8)
        zps = (int(rng.integers(0, 200)), int(rng.choice([0, 0, 5])) if b_t == "i8" else int(rng.choice([0, 120])), 0 if out_t == "i32" else int(rng.integers(0, 20)))
        sc = (1.0, 1.0, 1.0) if out_t == "i32" else (0.01, 0.02, float(rng.choice([0.5, 4.0, 40.0])))
        exp = O.quantized_dot(d, a, b, sc[0], zps[0], sc[1], zps[1], sc[2], zps[2])
        got = H.quantized_dot(d, a, b, sc[0], zps[0], sc[1], zps[1], sc[2], zps[2])
        kernels.add(H.last_kernel())
        assert np.array_equal(got, exp), (block, case, "dot", H.last_kernel())
        # the fused op on the same extents
        fo = str(rng.choice(["i8", "u8", "f32"]))
        relu = fo == "u8" or bool(rng.integers(0, 2))
        db = H.make_dot_desc(M, K, N, a_t="u8", out_t=fo, b_layout=H.B_NK)
        per_channel = bool(rng.integers(0, 2))
        fd = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=N if per_channel else 1)
        w = synth.uniform_int(int(rng.integers(1 << 30)), (N, K), -127, 127, np.int8)
        bias = synth.uniform_int(int(rng.integers(1 << 30)), (N,), -5000, 5000, np.int32)
        scale = synth.uniform_f32(int(rng.integers(1 << 30)), (N if per_channel else 1,), 0.5, 1.5) * np.float32(1.0 / (40.0 * np.sqrt(K)))
        exp = O.quantized_dot_bias(db, fd, a, w, bias, scale)
        got = H.quantized_dot_bias(db, fd, a, w, bias, scale)
        kernels.add(H.last_kernel())
        if fo == "f32":
            assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), (block, case, "dot bias f32", H.last_kernel())
        else:
            assert np.array_equal(got, exp), (block, case, "dot bias", fo, H.last_kernel())
    print("kernels:", sorted(kernels), flush=True)
