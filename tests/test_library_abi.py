"""CPU-side checks of the C-ABI library: it loads, exports everything include/hipq.h declares, and
its argument validation answers before any GPU work is attempted."""
import ctypes as C
import os
import re

import numpy as np

from ngraph_amd import hipq as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "hipq.h")).read()
    return sorted(set(re.findall(r"HIPQ_API\s+[\w\s\*]+?\b(hipq_\w+)\s*\(", text)))


def test_exports_match_header():
    names = _declared()
    assert len(names) >= 30
    lib = H.load()
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(H.EXPORTS) == names


def test_product_library_exports_only_the_declared_abi():
    """libhipq.so exports what include/hipq.h declares (plus hipq_last_kernel, the tests' window on the
    dispatcher) and no development or measurement symbol; those live in libhipq_probe.so"""
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", H.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if " T " in line)
    assert not [n for n in exported if "debug" in n or "probe" in n], exported
    assert set(exported) - set(_declared()) <= {"hipq_last_kernel", "_init", "_fini"}, sorted(set(exported) - set(_declared()))
    probe = H.load_probe()
    for n in ("hipq_probe_mfma_i8", "hipq_probe_coissue", "hipq_probe_intake", "hipq_probe_atomic_tiles", "hipq_debug_fastdiv", "hipq_probe_last_error"):
        assert hasattr(probe, n), n


def test_struct_sizes_match_header():
    # sizes follow from the header's field lists (natural alignment)
    assert C.sizeof(H.QuantDesc) == 4 * 6 + 8 * 8
    assert C.sizeof(H.ConvDesc) == 4 * 6 + 8 * 3 + 8 * 3 * 8
    assert C.sizeof(H.FusedDesc) == 4 * 4 + 8
    assert C.sizeof(H.DotDesc) == 4 * 4 + 8 * 3
    assert C.sizeof(H.DeviceInfo) == 64 + 32 + 4 * 4 + 8


def test_argument_validation_without_gpu():
    lib = H.load()
    assert lib.hipq_quantize(None, None, None, None, None, None) == H.ERR_INVALID
    assert b"null" in lib.hipq_last_error()
    d = H.make_quant_desc((4, 4), (), "f32", "i8")
    d.real_t = H.I8
    assert lib.hipq_quantize(C.byref(d), None, None, None, None, None) == H.ERR_UNSUPPORTED
    d = H.make_quant_desc((4, 4), (3,), "f32", "i8")
    assert lib.hipq_quantize(C.byref(d), None, None, None, None, None) == H.ERR_INVALID
    d = H.make_quant_desc((0, 4), (), "f32", "i8")
    assert lib.hipq_quantize(C.byref(d), None, None, None, None, None) == H.OK  # empty tensor: nothing to do
    cd = H.make_conv_desc(1, 16, 16, (8, 8), (3, 3))
    cd.out_sp[0] = 7
    assert lib.hipq_quantized_convolution(C.byref(cd), *([None] * 11)) == H.ERR_INVALID
    assert b"inferred" in lib.hipq_last_error()
    cd = H.make_conv_desc(1, 16, 16, (8, 8), (3, 3), out_t="f32")
    assert lib.hipq_quantized_convolution(C.byref(cd), *([None] * 11)) == H.ERR_UNSUPPORTED
    dd = H.make_dot_desc(4, 16, 4, a_t="f32")
    assert lib.hipq_quantized_dot(C.byref(dd), *([None] * 11)) == H.ERR_UNSUPPORTED


def test_conv_infer_output_matches_oracle_formula():
    lib = H.load()
    for kw in (
        dict(in_sp=(56, 56), f_sp=(3, 3), pad_below=(1, 1), pad_above=(1, 1)),
        dict(in_sp=(224, 224), f_sp=(7, 7), stride=(2, 2), pad_below=(3, 3), pad_above=(3, 3)),
        dict(in_sp=(10, 9), f_sp=(3, 2), dilation=(2, 3), data_dilation=(2, 1), pad_below=(-1, 2), pad_above=(1, 0)),
    ):
        d = H.make_conv_desc(1, 16, 16, **kw)
        exp = [d.out_sp[i] for i in range(3)]
        for i in range(3):
            d.out_sp[i] = 0
        assert lib.hipq_conv_infer_output(C.byref(d)) == H.OK
        assert [d.out_sp[i] for i in range(2)] == exp[:2]
    bad = H.make_conv_desc(1, 1, 1, (8, 8), (3, 3))
    bad.in_sp[0] = 1
    assert lib.hipq_conv_infer_output(C.byref(bad)) == H.ERR_INVALID


def test_packed_sizes_and_eligibility():
    lib = H.load()
    d = H.make_conv_desc(1, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    assert lib.hipq_conv_packed_filter_bytes(C.byref(d)) == 64 * 64 * 9 + 64 * 4
    d3 = H.make_conv_desc(1, 3, 64, (224, 224), (7, 7))  # fewer than 16 channels: packed with the channels padded to 16
    assert lib.hipq_conv_packed_filter_bytes(C.byref(d3)) == 64 * 16 * 49 + 64 * 4
    # ... unless the output is 8-bit channels-last: then every filter row is packed as 8 taps x 4 channels (7 rows -> 224 -> 256 bytes)
    d3r = H.make_conv_desc(1, 3, 64, (224, 224), (7, 7), out_t="u8", out_layout=H.NXC)
    assert lib.hipq_conv_packed_filter_bytes(C.byref(d3r)) == 64 * 256 + 64 * 4
    d40 = H.make_conv_desc(1, 40, 64, (8, 8), (3, 3))  # 16 or more channels, not a multiple of 16: direct kernel
    assert lib.hipq_conv_packed_filter_bytes(C.byref(d40)) == 0
    du = H.make_conv_desc(1, 64, 64, (8, 8), (1, 1), filter_t="u8", out_t="u8")
    assert lib.hipq_conv_packed_filter_bytes(C.byref(du)) == 0
    # column sums, plus (up to 256 rows, reductions in whole 64-byte steps) the weights once more in fragment order
    dd = H.make_dot_desc(32, 4096, 4096, b_layout=H.B_NK)
    assert lib.hipq_dot_packed_bytes(C.byref(dd)) == 4096 * 4 + 4096 * 4096
    dk = H.make_dot_desc(32, 4096, 4096, b_layout=H.B_KN)
    assert lib.hipq_dot_packed_bytes(C.byref(dk)) == 4096 * 4096 + 4096 * 4 + 4096 * 4096
    assert lib.hipq_dot_packed_bytes(C.byref(H.make_dot_desc(512, 4096, 4096, b_layout=H.B_NK))) == 4096 * 4
    assert lib.hipq_dot_packed_bytes(C.byref(H.make_dot_desc(32, 4000, 100, b_layout=H.B_NK))) == 512  # 100 sums, padded to 256 bytes
    assert lib.hipq_dot_packed_bytes(C.byref(H.make_dot_desc(1, 30, 8))) == 0


def test_fastdiv_exact():
    lib = H.load_probe()  # the index division of the Quantize kernels, exported by the measurement-aid library
    rng = np.random.default_rng(0)
    ds = list(range(1, 130)) + [255, 256, 257, 1023, 1024, 1025, 65535, 65536, 65537, 2**30, 2**31 - 1] + rng.integers(1, 2**31, 50).tolist()
    for d in ds:
        ns = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 2**31 - 1, 2**31 - 2] + rng.integers(0, 2**31, 20).tolist()
        for n in ns:
            if 0 <= n < 2**31:
                assert lib.hipq_debug_fastdiv(n, d) == n // d, (n, d)
