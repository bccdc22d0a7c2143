"""Pins orc_quantize / orc_dequantize (oracle/hipq_oracle.c) and the builder scale algebra."""
import numpy as np
import pytest

import oracle_lib as O
from ngraph_amd import hipq as H


def _run_kat(t, quantize, dequantize):
    shape = t["shape"]
    if t["op"] == "quantize":
        x = np.array(t["input"], dtype=H.NP_OF[H.dtype_code(t["input_type"])]).reshape(shape)
        got = quantize(x, t["scale"], t["offset"], t["output_type"], t["axes"], t["round_mode"])
        exp = np.array(t["expected"], dtype=np.int64).reshape(shape)
        assert np.array_equal(got.astype(np.int64), exp), t["name"]
    else:
        q = np.array(t["input"], dtype=H.NP_OF[H.dtype_code(t["input_type"])]).reshape(shape)
        got = dequantize(q, t["scale"], t["offset"], t["output_type"], t["axes"])
        exp = np.array(t["expected"], dtype=got.dtype).reshape(shape)
        assert np.array_equal(got, exp), t["name"]


def test_backend_kats(qdq_kats):
    """the 28 literal vectors of test/backend/quantize_dequantize.in.cpp"""
    assert len(qdq_kats) == 28
    for t in qdq_kats:
        _run_kat(t, O.quantize, O.dequantize)


@pytest.mark.skipif(not O.have_ref(), reason="oracle/_ref not built (reference tree absent)")
def test_ref_build_matches_kats(qdq_kats):
    """sanity of the shim itself: the compiled reference reproduces its own test vectors"""
    for t in qdq_kats:
        _run_kat(t, O.ref_quantize, O.ref_dequantize)


def test_against_reference_vectors(ref_vectors):
    """outputs of the compiled reference kernels on seeded tensors (ties, per-axis, f64, i32)"""
    manifest, arrays = ref_vectors
    n = 0
    for m in manifest:
        if m["kind"] != "quantize":
            continue
        x, s, z = arrays[m["name"] + "__x"], arrays[m["name"] + "__scale"], arrays[m["name"] + "__zp"]
        got = O.quantize(x, s, z, m["quant_t"], m["axes"], m["round_mode"])
        assert np.array_equal(got, arrays[m["name"]]), m["name"]
        dq = O.dequantize(got, s, z, m["real_t"], m["axes"])
        assert np.array_equal(dq, arrays[m["name"] + "__dq"]), m["name"]
        n += 1
    assert n >= 16


@pytest.mark.skipif(not O.have_ref(), reason="oracle/_ref not built (reference tree absent)")
@pytest.mark.parametrize("mode", range(9))
def test_live_reference_sweep(mode):
    """dense sweep around every half-integer and the f32 integer boundary, all nine round modes"""
    base = np.arange(-600, 600, dtype=np.float32) * 0.25
    eps = np.float32(2.0 ** -20)
    x = np.concatenate([base, base + eps, base - eps, np.float32([8388607.5, 8388609.0, -8388609.0, 1e9, -1e9, 0.49999997, -0.49999997])])
    for qt in ("i8", "u8", "i32"):
        a = O.quantize(x, 1.0, 0, qt, (), mode)
        b = O.ref_quantize(x, 1.0, 0, qt, (), mode)
        assert np.array_equal(a, b), (mode, qt)
        a = O.quantize(x, 0.3, 3, qt, (), mode)
        b = O.ref_quantize(x, 0.3, 3, qt, (), mode)
        assert np.array_equal(a, b), (mode, qt)


def test_rne_closed_form():
    """independent pin: for |q| < 2^22 the reference's floor/ceil/fmod formula is IEEE
    round-half-to-even, i.e. numpy.rint of the f32 quotient"""
    x = (np.arange(-40000, 40000, dtype=np.float32) * np.float32(0.125))
    s = np.float32(0.75)
    got = O.quantize(x, s, 0, "i32", (), H.RNE)
    exp = np.rint(x / s).astype(np.int32)
    assert np.array_equal(got, exp)
    # clamp then cast for the narrow types
    got8 = O.quantize(x, s, 5, "i8", (), H.RNE)
    exp8 = np.clip(np.rint(x / s) + 5, -128, 127).astype(np.int8)
    assert np.array_equal(got8, exp8)


def test_dequantize_closed_form():
    q = np.arange(-128, 128, dtype=np.int8).reshape(4, 64)
    scale = np.float32([0.1, 0.25, 3.0, 1e-3])
    zp = np.int8([0, -7, 100, -128])
    got = O.dequantize(q, scale, zp, "f32", (0,))
    exp = (q.astype(np.int32) - zp.astype(np.int32)[:, None]).astype(np.float32) * scale[:, None]
    assert np.array_equal(got, exp)


def test_builder_scaled_quantize(kats):
    """test/builder_quantization.cpp:679-847 feed (min,max); scale = get_scale(..., bump_by_eps)"""
    lib = O.port()
    for k in kats["scaled_quantize"]:
        scale = lib.orc_get_scale(k["range"][0], k["range"][1], H.dtype_code(k["quant_t"]), 1)
        x = np.array(k["input"], dtype=np.float32).reshape(k["shape"])
        got = O.quantize(x, scale, 0, k["quant_t"], (), H.RNE)
        assert got.reshape(-1).tolist() == k["expected"], k["name"]
    for k in kats["scaled_dequantize"]:
        scale = lib.orc_get_scale(k["range"][0], k["range"][1], H.dtype_code(k["quant_t"]), 0)
        q = np.array(k["input"], dtype=H.NP_OF[H.dtype_code(k["quant_t"])]).reshape(k["shape"])
        got = O.dequantize(q, scale, 0, "f32", ())
        assert np.array_equal(got.reshape(-1), np.array(k["expected"], dtype=np.float32)), k["name"]


def test_empty_and_scalar():
    assert O.quantize(np.zeros((0, 3), np.float32), 1.0, 0, "i8").shape == (0, 3)
    assert O.quantize(np.float32(5.0).reshape(()), 2.0, 1, "u8").item() == 3  # 2.5 -> 2 (even) + 1
