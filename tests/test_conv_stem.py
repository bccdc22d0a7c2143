"""A network's first convolution on the band kernel that reads [N][C][H][W] bytes itself, alone and with
the MaxPool that follows it reduced in the same launch: bytes against the C restatement of
QuantizedConvolutionBias (quantized_conv.cpp:332-766 arithmetic) and of MaxPool (max_pool.hpp:127-222),
and against the library's own two-launch path.
"""
import numpy as np
import pytest

import cases
import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth

pytestmark = pytest.mark.gpu


def say(*a):
    print("[stem]", *a, flush=True)


# N, C, image, filter, conv stride, conv pads (below, above), pool window, pool stride, pool pads (below, above)
CASES = [
    (2, 3, (224, 224), (7, 7), (2, 2), ((3, 3), (3, 3)), (3, 3), (2, 2), ((1, 1), (1, 1))),  # ResNet-50's first two layers
    (3, 3, (64, 48), (7, 7), (2, 2), ((3, 3), (3, 3)), (3, 3), (2, 2), ((1, 1), (1, 1))),    # bands that end short
    (2, 1, (40, 36), (5, 5), (2, 2), ((2, 2), (2, 2)), (2, 2), (2, 2), ((0, 0), (0, 0))),    # one channel, 2 x 2 pool without padding
    (1, 4, (33, 52), (3, 3), (1, 2), ((1, 1), (1, 1)), (3, 3), (2, 2), ((0, 0), (1, 1))),    # row stride 1, four channels, odd rows, uneven pool pads
    (2, 3, (30, 40), (8, 8), (2, 2), ((4, 3), (3, 4)), (3, 2), (1, 2), ((1, 0), (1, 0))),    # 8 x 8 taps, uneven pads, pool row stride 1
    (5, 2, (18, 16), (3, 5), (2, 2), ((0, 2), (1, 2)), (1, 1), (1, 1), ((0, 0), (0, 0))),    # 1 x 1 "pool": the convolution itself
]


def _case(i, relu=True, scalar_scale=False, big_bias=False, data_t="u8"):
    N, Cc, image, fs, st, pads, pw, ps, pp = CASES[i]
    kw = dict(stride=st, pad_below=pads[0], pad_above=pads[1], out_t="u8", data_t=data_t)
    d = H.make_conv_desc(N, Cc, 64, image, fs, data_layout=H.NCX, out_layout=H.NXC, **kw)
    dn = H.make_conv_desc(N, Cc, 64, image, fs, **kw)
    lo, hi = (0, 255) if data_t == "u8" else (-128, 127)
    data = synth.uniform_int(4100 + i, dn.data_shape(), lo, hi, H.NP_OF[d.data_t])
    filt = synth.uniform_int(4200 + i, dn.filter_shape(), -127, 127, np.int8)
    bias = synth.uniform_int(4300 + i, (64,), -30000, 30000, np.int32)
    if big_bias:
        bias[5] = (1 << 24) + 12345  # beyond what the accumulators may carry: the exact scalar band
        bias[40] = -(1 << 25)
    taps = Cc * fs[0] * fs[1]
    scales = np.float32(0.9 / (40.0 * np.sqrt(taps))) if scalar_scale else synth.uniform_f32(4400 + i, (64,), 0.5 / (40.0 * np.sqrt(taps)), 1.5 / (40.0 * np.sqrt(taps)))
    f = H.make_fused_desc(has_bias=True, with_relu=relu, scale_count=1 if scalar_scale else 64)
    osp = dn.out_shape()[2:]
    pd = H.make_pool_desc("max", "u8", N, 64, osp, pw, ps, pp[0], pp[1], layout=H.NXC)
    pdn = H.make_pool_desc("max", "u8", N, 64, osp, pw, ps, pp[0], pp[1])
    return d, dn, f, pd, pdn, data, filt, bias, scales


@pytest.mark.parametrize("i", range(len(CASES)))
def test_stem_conv_alone(gpu_lib, i):
    """the convolution by itself through hipq_quantized_convolution_fused"""
    say("conv", CASES[i])
    O.port().orc_set_threads(8)
    for relu, scalar in ((True, False), (False, True)):
        d, dn, f, pd, pdn, data, filt, bias, scales = _case(i, relu=relu, scalar_scale=scalar)
        exp = O.quantized_convolution_fused(dn, f, data, filt, bias, None, scales, None)
        got = H.quantized_convolution_fused(d, f, data, filt, bias, None, scales, None)
        assert H.last_kernel() == "conv_stem_i8_32x32x32", H.last_kernel()
        assert np.array_equal(cases.to_ncx(got), exp), (i, relu, scalar)
        assert len(np.unique(got)) > 30
    O.port().orc_set_threads(1)


@pytest.mark.parametrize("i", range(len(CASES)))
def test_stem_conv_max_pool(gpu_lib, i, monkeypatch):
    """MaxPool(convolution) in one launch against the restatement of both ops and against the two launches"""
    say("conv + pool", CASES[i])
    O.port().orc_set_threads(8)
    d, dn, f, pd, pdn, data, filt, bias, scales = _case(i)
    assert H.conv_max_pool_fusable(d, f, pd)
    conv = O.quantized_convolution_fused(dn, f, data, filt, bias, None, scales, None)
    exp = O.pool(pdn, conv)
    got = H.quantized_convolution_fused_max_pool(d, f, pd, data, filt, bias, scales)
    assert H.last_kernel() == "conv_stem_pool_i8_32x32x32", H.last_kernel()
    assert np.array_equal(cases.to_ncx(got), exp), i
    monkeypatch.setenv("HIPQ_NO_STEM", "1")
    two = H.pool(pd, H.quantized_convolution_fused(d, f, data, filt, bias, None, scales, None))
    assert H.last_kernel().startswith("max_pool"), H.last_kernel()
    assert np.array_equal(two, got)
    O.port().orc_set_threads(1)


def test_stem_signed_data_and_large_bias(gpu_lib):
    """i8 data (no sign flip), and biases beyond 2^24, which the kernel computes in its exact scalar band"""
    say("i8 data, large bias")
    O.port().orc_set_threads(8)
    for kw in (dict(data_t="i8"), dict(big_bias=True), dict(big_bias=True, relu=False)):
        d, dn, f, pd, pdn, data, filt, bias, scales = _case(1, **kw)
        conv = O.quantized_convolution_fused(dn, f, data, filt, bias, None, scales, None)
        got = H.quantized_convolution_fused(d, f, data, filt, bias, None, scales, None)
        assert H.last_kernel() == "conv_stem_i8_32x32x32", H.last_kernel()
        assert np.array_equal(cases.to_ncx(got), conv), kw
        gp = H.quantized_convolution_fused_max_pool(d, f, pd, data, filt, bias, scales)
        assert np.array_equal(cases.to_ncx(gp), O.pool(pdn, conv)), kw
    O.port().orc_set_threads(1)


def test_stem_pairs_without_a_fused_kernel(gpu_lib):
    """pairs the fused kernel does not take are reported as such, by the query and by the call"""
    say("unsupported pairs")
    d, dn, f, pd, pdn, data, filt, bias, scales = _case(1)
    # an average pool, a pool over some other tensor, a convolution with 32 output channels
    avg = H.make_pool_desc("avg", "u8", pd.N, 64, list(pd.in_sp)[:2], (3, 3), (2, 2), (1, 1), (1, 1), layout=H.NXC)
    other = H.make_pool_desc("max", "u8", pd.N, 64, (pd.in_sp[0] + 1, pd.in_sp[1]), (3, 3), (2, 2), (1, 1), (1, 1), layout=H.NXC)
    assert not H.conv_max_pool_fusable(d, f, avg)
    assert not H.conv_max_pool_fusable(d, f, other)
    N, Cc, image, fs, st, pads, pw, ps, pp = CASES[1]
    d32 = H.make_conv_desc(N, Cc, 32, image, fs, stride=st, pad_below=pads[0], pad_above=pads[1], out_t="u8", data_layout=H.NCX, out_layout=H.NXC)
    p32 = H.make_pool_desc("max", "u8", N, 32, d32.out_shape()[1:3], pw, ps, pp[0], pp[1], layout=H.NXC)
    assert not H.conv_max_pool_fusable(d32, f, p32)
    with pytest.raises(H.HipqError):
        H.quantized_convolution_fused_max_pool(d, f, avg, data, filt, bias, scales)
