"""1 x 1 convolutions from 64 or 128 to 256 / 512 channels on the kernel that keeps its weights in registers and
loads a tile ahead (bottleneck blocks' last layer and projection shortcut): bytes against the C
restatement of the fused ops (quantized_conv.cpp:332-766 arithmetic) and against the tile kernel."""
import numpy as np
import pytest

import cases
import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth

pytestmark = pytest.mark.gpu


def say(*a):
    print("[pw64]", *a, flush=True)


# N, image, K, relu, residual (None / "u8" / "i8"), per-channel scales, bias magnitude, input channels
CASES = [
    (3, (40, 40), 256, True, "u8", True, 20000, 64),     # QuantizedConvolutionBiasAdd, 75 whole tiles
    (2, (37, 29), 256, False, "i8", False, 20000, 64),   # ...BiasSignedAdd without ReLU: i8 out, scalar scale, ragged last tile (2146 rows)
    (2, (33, 31), 256, True, None, True, 20000, 64),     # QuantizedConvolutionBias + ReLU, last tile 62 rows short of 64
    (1, (50, 41), 512, False, None, True, 20000, 64),    # two column blocks, i8 out
    (2, (20, 20), 256, True, "u8", True, 1 << 25, 64),   # biases beyond 2^24: added in float, not carried in the accumulators
    (2, (28, 28), 512, True, "u8", True, 20000, 128),    # 128 input channels (four reduction steps), two column blocks
    (1, (31, 23), 256, False, "i8", True, 20000, 128),   # ... signed residual, i8 out, ragged last tile
    (2, (19, 21), 256, True, None, False, 20000, 128),   # ... no residual, scalar scale
]


@pytest.mark.parametrize("i", range(len(CASES)))
def test_pw64_against_oracle_and_tile_kernel(gpu_lib, i, monkeypatch):
    N, image, K, relu, res, per_channel, bias_mag, Cc = CASES[i]
    say(CASES[i])
    O.port().orc_set_threads(8)
    out_t = "u8" if relu else "i8"
    d = H.make_conv_desc(N, Cc, K, image, (1, 1), out_t=out_t, data_layout=H.NXC, out_layout=H.NXC)
    dn = H.make_conv_desc(N, Cc, K, image, (1, 1), out_t=out_t)
    data = synth.uniform_int(5100 + i, dn.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(5200 + i, dn.filter_shape(), -127, 127, np.int8)
    bias = synth.uniform_int(5300 + i, (K,), -bias_mag, bias_mag, np.int32)
    scales = synth.uniform_f32(5400 + i, (K,), 1e-3, 3e-3) if per_channel else np.float32(2e-3)
    if bias_mag > (1 << 24):
        scales = scales * np.float32(2e-4)
    summ = None
    if res is not None:
        lo, hi = (0, 255) if res == "u8" else (-128, 127)
        summ = synth.uniform_int(5500 + i, dn.out_shape(), lo, hi, H.NP_OF[H.dtype_code(res)])
    f = H.make_fused_desc(has_bias=True, has_sum=res is not None, sum_t=res or "u8", with_relu=relu, scale_count=K if per_channel else 1)
    ss = 0.41 if res is not None else None
    exp = O.quantized_convolution_fused(dn, f, data, filt, bias, summ, scales, ss)
    x, sm = cases.to_nxc(data), (cases.to_nxc(summ) if summ is not None else None)
    monkeypatch.setenv("HIPQ_PW64_MIN_ROWS", "1")
    got = H.quantized_convolution_fused(d, f, x, filt, bias, sm, scales, ss)
    assert H.last_kernel() == "conv_pw64_i8_32x32x32", H.last_kernel()
    assert np.array_equal(cases.to_ncx(got), exp), CASES[i]
    assert len(np.unique(got)) > 30
    monkeypatch.setenv("HIPQ_NO_PW64", "1")
    other = H.quantized_convolution_fused(d, f, x, filt, bias, sm, scales, ss)
    assert H.last_kernel().startswith("conv_mfma"), H.last_kernel()
    assert np.array_equal(other, got)
    O.port().orc_set_threads(1)


def test_pw64_takes_the_layers_it_is_for(gpu_lib):
    """without the test's threshold override: 100352 pixels (a 56 x 56 stage at batch 32) go to this kernel, 3136 do not"""
    for N, want in ((32, "conv_pw64"), (1, "conv_mfma")):
        d = H.make_conv_desc(N, 64, 256, (56, 56), (1, 1), out_t="u8", data_layout=H.NXC, out_layout=H.NXC)
        data = synth.uniform_int(5600, d.data_shape(), 0, 255, np.uint8)
        filt = synth.uniform_int(5601, d.filter_shape(), -127, 127, np.int8)
        bias = synth.uniform_int(5602, (256,), -2000, 2000, np.int32)
        f = H.make_fused_desc(has_bias=True, with_relu=True, scale_count=1)
        H.quantized_convolution_fused(d, f, data, filt, bias, None, np.float32(2e-3), None)
        assert H.last_kernel().startswith(want), (N, H.last_kernel())
