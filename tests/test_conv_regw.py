"""The convolution kernel that keeps its filter in registers (3x3 over 64 channels, stride 1, pad 1,
NCHW output; BASELINE config 1's layer): against the oracle, bit for bit, with the input in either
layout, both requantization policies, signed and unsigned data, zero points, narrow outputs,
residual sums, bands that start and end inside the image, and the exact path for a non-zero filter
zero point."""
import numpy as np
import pytest

import cases
import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth

pytestmark = pytest.mark.gpu
KERNEL = "conv_regw_i8_32x32x32"


def say(*a):
    print("[case]", *a, flush=True)


def _inputs(seed, N, K, hw, data_t="u8"):
    ncx = H.make_conv_desc(N, 64, K, hw, (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_t=data_t)
    lo, hi, dt = (0, 255, np.uint8) if data_t == "u8" else (-128, 127, np.int8)
    data = synth.uniform_int(seed, ncx.data_shape(), lo, hi, dt)
    filt = synth.uniform_int(seed + 1, ncx.filter_shape(), -127, 127, np.int8)
    return ncx, data, filt


# (N, K, (H, W)): one band an image, several bands an image (bands that begin and end inside the image),
# widths whose rows end inside a 32-pixel tile, the narrowest and widest rows, fewer output channels
SHAPES = [(1, 64, (56, 56)), (3, 64, (56, 56)), (2, 64, (8, 8)), (5, 32, (12, 20)), (2, 16, (4, 64)), (1, 48, (16, 4)), (40, 64, (28, 28))]


@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_interpreter_policy_both_layouts(gpu_lib, shape):
    N, K, hw = shape
    ncx, data, filt = _inputs(7000 + N + K, N, K, hw)
    O.port().orc_set_threads(8)
    for s, z in (((0.02, 0.005, 0.1), (0, 0, 0)), ((0.02, 0.005, 0.9), (131, 0, -3)), ((0.5, 0.5, 1e-3), (0, 0, 0))):
        say("regw interp", shape, s, z)
        exp = O.quantized_convolution(ncx, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
        got = H.quantized_convolution(ncx, data, filt, s[0], z[0], s[1], z[1], s[2], z[2])
        assert H.last_kernel() == KERNEL, H.last_kernel()
        assert np.array_equal(got, exp), ("ncx in", s, z)
        nxc = H.make_conv_desc(N, 64, K, hw, (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_layout=H.NXC, out_layout=H.NCX)
        got = H.quantized_convolution(nxc, cases.to_nxc(data), filt, s[0], z[0], s[1], z[1], s[2], z[2])
        assert H.last_kernel() == KERNEL, H.last_kernel()
        assert np.array_equal(got, exp), ("nxc in", s, z)
    O.port().orc_set_threads(1)
    assert len(np.unique(exp)) > 3


def test_signed_data_and_u8_output(gpu_lib):
    ncx, data, filt = _inputs(7100, 2, 64, (16, 16), data_t="i8")
    O.port().orc_set_threads(8)
    for out_t, zpd in (("i8", 0), ("u8", -5), ("i8", 17)):
        say("regw i8 data", out_t, zpd)
        d = H.make_conv_desc(2, 64, 64, (16, 16), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_t="i8", out_t=out_t)
        exp = O.quantized_convolution(d, data, filt, 0.02, zpd, 0.005, 0, 0.3, 0)
        got = H.quantized_convolution(d, data, filt, 0.02, zpd, 0.005, 0, 0.3, 0)
        assert H.last_kernel() == KERNEL
        assert np.array_equal(got, exp), (out_t, zpd)
    O.port().orc_set_threads(1)


def test_nonzero_filter_zero_point(gpu_lib):
    say("regw filter zp != 0")
    ncx, data, filt = _inputs(7200, 2, 32, (8, 12))
    exp = O.quantized_convolution(ncx, data, filt, 0.02, 7, 0.005, -9, 0.9, 1)
    got = H.quantized_convolution(ncx, data, filt, 0.02, 7, 0.005, -9, 0.9, 1)
    assert H.last_kernel() == KERNEL
    assert np.array_equal(got, exp)
    nxc = H.make_conv_desc(2, 64, 32, (8, 12), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_layout=H.NXC, out_layout=H.NCX)
    assert np.array_equal(H.quantized_convolution(nxc, cases.to_nxc(data), filt, 0.02, 7, 0.005, -9, 0.9, 1), exp)


@pytest.mark.parametrize("shape", [(2, 64, (56, 56)), (3, 32, (12, 20)), (9, 64, (28, 28))], ids=str)
def test_fused_policy(gpu_lib, shape):
    """QuantizedConvolutionBias / Relu / BiasAdd / BiasSignedAdd: bias, scalar and per-channel scales,
    residual sums (u8 and i8), relu -- round half to even, saturate"""
    N, K, hw = shape
    ncx, data, filt = _inputs(7300 + N, N, K, hw)
    bias = synth.uniform_int(7310, (K,), -30000, 30000, np.int32)
    per = (synth.uniform_f32(7311, (K,), 0.5, 1.5) * np.float32(1.0 / 4000)).astype(np.float32)
    O.port().orc_set_threads(8)
    for relu, has_sum, sum_t, per_channel in ((True, False, "u8", True), (False, False, "u8", False), (True, True, "u8", True), (False, True, "i8", True), (True, True, "i8", False)):
        say("regw fused", shape, relu, has_sum, sum_t, per_channel)
        out_t = "u8" if (relu and sum_t == "u8") else "i8"
        d = H.make_conv_desc(N, 64, K, hw, (3, 3), pad_below=(1, 1), pad_above=(1, 1), out_t=out_t)
        f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t=sum_t, with_relu=relu, scale_count=K if per_channel else 1)
        sc = per if per_channel else np.float32(1.0 / 3500)
        summ = None
        if has_sum:
            summ = synth.uniform_int(7320, d.out_shape(), 0 if sum_t == "u8" else -128, 255 if sum_t == "u8" else 127, np.uint8 if sum_t == "u8" else np.int8)
        exp = O.quantized_convolution_fused(d, f, data, filt, bias, summ, sc, 0.37 if has_sum else None)
        got = H.quantized_convolution_fused(d, f, data, filt, bias, summ, sc, 0.37 if has_sum else None)
        assert H.last_kernel() == KERNEL, H.last_kernel()
        assert np.array_equal(got, exp), (relu, has_sum, sum_t, per_channel)
        nxc = H.make_conv_desc(N, 64, K, hw, (3, 3), pad_below=(1, 1), pad_above=(1, 1), out_t=out_t, data_layout=H.NXC, out_layout=H.NCX)
        got = H.quantized_convolution_fused(nxc, f, cases.to_nxc(data), filt, bias, summ, sc, 0.37 if has_sum else None)
        assert np.array_equal(got, exp), ("nxc in", relu, has_sum, sum_t, per_channel)
        assert len(np.unique(exp)) > 20
    O.port().orc_set_threads(1)


def test_config1_batch128_properties(gpu_lib):
    """BASELINE config 1's layer at the benchmarked batch (one band of 28 rows a workgroup, 256
    workgroups): images 0, 77 and 127 equal the oracle's single-image results, and the NCHW-in call
    equals the channels-last-in call on the same values"""
    say("regw config 1 at batch 128")
    N = 128
    ncx, data, filt = _inputs(7400, N, 64, (56, 56))
    got = H.quantized_convolution(ncx, data, filt, 0.02, 0, 0.005, 0, 0.1, 0)
    assert H.last_kernel() == KERNEL
    one = H.make_conv_desc(1, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    O.port().orc_set_threads(8)
    for i in (0, 77, 127):
        assert np.array_equal(got[i : i + 1], O.quantized_convolution(one, data[i : i + 1], filt, 0.02, 0, 0.005, 0, 0.1, 0)), i
    O.port().orc_set_threads(1)
    nxc = H.make_conv_desc(N, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_layout=H.NXC, out_layout=H.NCX)
    assert np.array_equal(H.quantized_convolution(nxc, cases.to_nxc(data), filt, 0.02, 0, 0.005, 0, 0.1, 0), got)
