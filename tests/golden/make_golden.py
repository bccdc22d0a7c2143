#!/usr/bin/env python3
"""Regenerates the fixtures of tests/golden/ that come from the nGraph reference tree.

Run in a container where the reference lies at $NGRAPH_SRC (default /root/reference) and
oracle/_ref has been built (`make -C oracle ref`).  The committed outputs are data only:

  quantize_dequantize_kats.json   inputs / attributes / expected outputs of the 28 tests of
                                  test/backend/quantize_dequantize.in.cpp, read from its literals
  qlinearconv{2d,3d}_{x,y}.bin    the byte fixtures of test/files/onnx/qlinearconv{2d,3d}/
  pool_vectors.npz + .json        outputs of the compiled reference max_pool / avg_pool (oracle/_ref)
                                  on seeded synthetic inputs (`--pool-only` writes just these)
  resnet50_logits.npz / .json     the synthetic int8 ResNet-50's logits and per-op byte sums on one seeded
                                  image, from the C restatement (`--resnet-only` writes just these)
  ref_vectors.npz + .json         outputs of the compiled reference kernels (oracle/_ref) on seeded
                                  synthetic inputs; inputs are regenerated from the seed by
                                  ngraph_amd.synth (or stored, where they are floating point)

reference_kats.json is transcribed by hand from the reference's tests and is not written here.
"""
import json
import os
import re
import shutil
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

NGRAPH_SRC = os.environ.get("NGRAPH_SRC", "/root/reference")

ET = {"f32": "f32", "f64": "f64", "u8": "u8", "i8": "i8", "i32": "i32"}
LIMITS = {"u8": (0, 255), "i8": (-128, 127), "i32": (-(2**31), 2**31 - 1)}


def _numbers(text, min_v=None, max_v=None):
    out = []
    for tok in text.split(","):
        tok = tok.strip()
        if not tok:
            continue
        if tok == "min":
            out.append(min_v)
        elif tok == "max":
            out.append(max_v)
        elif tok == "1.0 / (max + 1.0)":
            out.append(1.0 / (max_v + 1.0))
        else:
            tok = tok.rstrip("f")
            out.append(float(tok) if any(c in tok for c in ".e") else int(tok))
    return out


def parse_quantize_dequantize():
    path = os.path.join(NGRAPH_SRC, "test/backend/quantize_dequantize.in.cpp")
    src = open(path).read()
    # strip // comments, they carry worked arithmetic full of digits
    lines = src.split("\n")
    tests = []
    starts = [i for i, l in enumerate(lines) if l.startswith("NGRAPH_TEST(")]
    starts.append(len(lines))
    for a, b in zip(starts[:-1], starts[1:]):
        body = "\n".join(re.sub(r"//.*", "", l) for l in lines[a:b])
        name = re.search(r"NGRAPH_TEST\(\$\{BACKEND_NAME\},\s*(\w+)\)", body).group(1)
        t = {"name": name, "source": f"test/backend/quantize_dequantize.in.cpp:{a + 1}"}
        t["shape"] = _numbers(re.search(r"Shape input_shape\{([^}]*)\}", body).group(1))
        m = re.search(r"Shape scale_offset_shape(?:\s*=\s*)?\{([^}]*)\}", body)
        t["scale_shape"] = _numbers(m.group(1)) if m else []
        m = re.search(r"AxisSet quantization_axes\{([^}]*)\}", body)
        t["axes"] = _numbers(m.group(1)) if m else []
        t["input_type"] = re.search(r"auto input_type = element::(\w+);", body).group(1)
        t["output_type"] = re.search(r"auto output_type = element::(\w+);", body).group(1)
        m = re.search(r"RoundMode round_mode =\s*op::v0::Quantize::RoundMode::(\w+);", body)
        t["op"] = "quantize" if m else "dequantize"
        if m:
            t["round_mode"] = m.group(1)
        qt = t["output_type"] if t["op"] == "quantize" else t["input_type"]
        lo, hi = LIMITS[qt]
        if "numeric_limits" not in body:
            lo = hi = None
        m = re.search(r"auto scale = op::v0::Constant::create\(\w+, scale_offset_shape, \{([^}]*)\}\)", body)
        if m:
            t["scale"] = _numbers(m.group(1), lo, hi)
            t["offset"] = _numbers(
                re.search(r"auto offset = op::v0::Constant::create\(\w+, scale_offset_shape, \{([^}]*)\}\)", body).group(1), lo, hi
            )
            t["dynamic"] = False
        else:  # scale / offset are Parameters fed at call time
            t["scale"] = _numbers(re.search(r"copy_data\(Scale, vector<\w+>\{([^}]*)\}\)", body).group(1))
            t["offset"] = _numbers(re.search(r"copy_data\(Offset, vector<\w+>\{([^}]*)\}\)", body).group(1))
            t["dynamic"] = True
        t["input"] = _numbers(re.search(r"copy_data\(x, vector<input_c_type>\{([^}]*)\}\)", body, re.S).group(1), lo, hi)
        exp = re.findall(r"vector<output_c_type>\{([^}]*)\}", body, re.S)
        t["expected"] = _numbers(exp[-1], lo, hi)
        n = int(np.prod(t["shape"])) if t["shape"] else 1
        assert len(t["input"]) == n and len(t["expected"]) == n, name
        tests.append(t)
    assert len(tests) == 28, len(tests)
    with open(os.path.join(HERE, "quantize_dequantize_kats.json"), "w") as f:
        json.dump(tests, f, indent=1)
    print("quantize_dequantize_kats.json:", len(tests), "tests")


def copy_onnx_bins():
    for d in ("qlinearconv2d", "qlinearconv3d"):
        for n in ("x", "y"):
            shutil.copyfile(os.path.join(NGRAPH_SRC, "test/files/onnx", d, n + ".bin"), os.path.join(HERE, f"{d}_{n}.bin"))
            os.chmod(os.path.join(HERE, f"{d}_{n}.bin"), 0o644)
    print("copied ONNX QLinearConv byte fixtures")


def ref_vectors():
    import oracle_lib as O
    from ngraph_amd import hipq as H
    from ngraph_amd import synth

    if not O.have_ref():
        raise SystemExit("oracle/_ref is not built: make -C oracle ref")
    arrays, manifest = {}, []

    def conv_case(name, seed, N, Cc, K, in_sp, f_sp, types=("u8", "i8", "i8"), scales=(0.02, 0.005, 0.1), zps=(0, 0, 0), **kw):
        d = H.make_conv_desc(N, Cc, K, in_sp, f_sp, data_t=types[0], filter_t=types[1], out_t=types[2], **kw)
        dlo, dhi = (0, 255)
        flo, fhi = (-127, 127) if types[1] == "i8" else (0, 255)
        data = synth.uniform_int(seed, d.data_shape(), dlo, dhi, np.uint8)
        filt = synth.uniform_int(seed + 1, d.filter_shape(), flo, fhi, H.NP_OF[d.filter_t])
        out = O.ref_quantized_convolution(d, data, filt, scales[0], zps[0], scales[1], zps[1], scales[2], zps[2])
        arrays[name] = out
        manifest.append(
            dict(
                kind="conv",
                name=name,
                seed=seed,
                N=N,
                C=Cc,
                K=K,
                in_sp=list(in_sp),
                f_sp=list(f_sp),
                types=list(types),
                scales=list(scales),
                zps=list(zps),
                data_range=[dlo, dhi],
                filter_range=[flo, fhi],
                kw={k: list(v) for k, v in kw.items()},
            )
        )

    # BASELINE config 1 exactly (65 % of outputs wrap: the reference narrows without saturating)
    conv_case("c1", 1001, 1, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    # same layer with an in-range output scale
    conv_case("c1_inrange", 1001, 1, 64, 64, (56, 56), (3, 3), scales=(0.02, 0.005, 1.0), pad_below=(1, 1), pad_above=(1, 1))
    # raw accumulators
    conv_case("c1_small_i32", 1003, 2, 64, 64, (9, 11), (3, 3), types=("u8", "i8", "i32"), scales=(1.0, 1.0, 1.0), pad_below=(1, 1), pad_above=(1, 1))
    # parameter grid in the spirit of test/ref_generators/generate_convolution_ref.py:313-373
    conv_case("stride2", 1010, 2, 16, 8, (13, 12), (3, 3), stride=(2, 2), pad_below=(1, 1), pad_above=(1, 1))
    conv_case("stride_mixed", 1011, 1, 5, 7, (10, 9), (3, 2), stride=(3, 1), scales=(0.1, 0.01, 0.5))
    conv_case("dilation", 1012, 1, 4, 6, (12, 12), (3, 3), dilation=(2, 3), pad_below=(2, 3), pad_above=(2, 3), scales=(0.1, 0.01, 0.5))
    conv_case("data_dilation", 1013, 1, 3, 4, (6, 5), (3, 3), data_dilation=(2, 3), pad_below=(1, 0), pad_above=(0, 2), scales=(0.1, 0.01, 0.5))
    conv_case("neg_pad", 1014, 1, 3, 4, (10, 10), (3, 3), pad_below=(-1, 2), pad_above=(1, -2), scales=(0.1, 0.01, 0.5))
    conv_case("conv1d", 1015, 2, 6, 5, (17,), (4,), stride=(2,), pad_below=(1,), pad_above=(2,), scales=(0.1, 0.01, 0.5))
    conv_case("conv3d", 1016, 1, 3, 4, (5, 6, 4), (2, 3, 2), stride=(1, 2, 1), pad_below=(1, 0, 1), pad_above=(0, 1, 1), scales=(0.1, 0.01, 0.5))
    conv_case("u8u8_zp", 1017, 1, 4, 5, (8, 8), (3, 3), types=("u8", "u8", "u8"), scales=(0.0037, 0.0017, 0.02), zps=(132, 120, 123), pad_below=(1, 1), pad_above=(1, 1))
    conv_case("u8u8_i32_zp", 1018, 1, 4, 5, (8, 8), (3, 3), types=("u8", "u8", "i32"), scales=(1.0, 1.0, 1.0), zps=(7, 250, -9), pad_below=(1, 1), pad_above=(1, 1))
    conv_case("u8i8_zp", 1019, 1, 8, 8, (7, 7), (1, 1), scales=(0.05, 0.01, 0.3), zps=(128, -3, 5))
    conv_case("k1x1_c64", 1020, 1, 64, 128, (14, 14), (1, 1), scales=(0.02, 0.005, 1.0))
    conv_case("s2_c64", 1021, 1, 64, 64, (15, 15), (3, 3), stride=(2, 2), pad_below=(1, 1), pad_above=(1, 1), scales=(0.02, 0.005, 1.0))

    def dot_case(name, seed, M, K, N, types=("u8", "i8", "i8"), scales=(0.02, 0.005, 0.1), zps=(0, 0, 0)):
        d = H.make_dot_desc(M, K, N, a_t=types[0], b_t=types[1], out_t=types[2])
        blo, bhi = (-127, 127) if types[1] == "i8" else (0, 255)
        a = synth.uniform_int(seed, (M, K), 0, 255, np.uint8)
        b = synth.uniform_int(seed + 1, (K, N), blo, bhi, H.NP_OF[d.b_t])
        out = O.ref_quantized_dot(d, a, b, scales[0], zps[0], scales[1], zps[1], scales[2], zps[2])
        arrays[name] = out
        manifest.append(dict(kind="dot", name=name, seed=seed, M=M, K=K, N=N, types=list(types), scales=list(scales), zps=list(zps), b_range=[blo, bhi]))

    dot_case("dot_m1_k4096_n512", 2001, 1, 4096, 512, scales=(0.02, 0.005, 2.0))
    dot_case("dot_m5_wrap", 2002, 5, 300, 70)
    dot_case("dot_i32", 2003, 3, 257, 65, types=("u8", "i8", "i32"), scales=(1.0, 1.0, 1.0))
    dot_case("dot_u8u8_zp", 2004, 4, 128, 48, types=("u8", "u8", "u8"), scales=(0.0066, 0.00705, 0.0107), zps=(113, 114, 118))
    dot_case("dot_u8u8_i32_zp", 2005, 4, 100, 33, types=("u8", "u8", "i32"), scales=(1.0, 1.0, 1.0), zps=(3, 200, 11))
    dot_case("dot_m32_k1024_n256", 2006, 32, 1024, 256, scales=(0.02, 0.005, 1.5))

    def quant_case(name, seed, shape, axes, quant_t, mode, real="f32", spread=40.0):
        x = (synth.normal_f32(seed, shape) * spread).astype(H.NP_OF[H.dtype_code(real)])
        # exact .5 ties and a few large values so every branch of the rounding formulas is hit
        flat = x.reshape(-1)
        flat[:: 7] = np.round(flat[:: 7] * 2) / 2
        sshape = [shape[a] for a in axes]
        scale = synth.uniform_f32(seed + 1, sshape, 0.25, 2.0).astype(x.dtype)
        scale.reshape(-1)[::2] = 0.5
        lo, hi = LIMITS[quant_t]
        zp = synth.uniform_int(seed + 2, sshape, max(lo, -20), min(hi, 20), H.NP_OF[H.dtype_code(quant_t)])
        out = O.ref_quantize(x, scale, zp, quant_t, axes, mode)
        arrays[name + "__x"] = x
        arrays[name + "__scale"] = scale
        arrays[name + "__zp"] = zp
        arrays[name] = out
        manifest.append(dict(kind="quantize", name=name, shape=list(shape), axes=list(axes), quant_t=quant_t, round_mode=mode, real_t=real))
        dq = O.ref_dequantize(out, scale, zp, real, axes)
        arrays[name + "__dq"] = dq

    for i, mode in enumerate(H.ROUND_MODES):
        quant_case(f"q_i8_mode{i}", 3000 + 10 * i, (3, 5, 7), (), "i8", mode)
    quant_case("q_u8_axis1", 3100, (4, 6, 10), (1,), "u8", "ROUND_NEAREST_TOWARD_EVEN")
    quant_case("q_i8_axis0", 3110, (5, 33), (0,), "i8", "ROUND_NEAREST_TOWARD_EVEN")
    quant_case("q_i8_axis_last", 3120, (7, 9), (1,), "i8", "ROUND_NEAREST_TOWARD_EVEN")
    quant_case("q_u8_axes02", 3130, (3, 4, 5), (0, 2), "u8", "ROUND_NEAREST_TOWARD_INFINITY")
    quant_case("q_i32_f32", 3140, (64,), (), "i32", "ROUND_NEAREST_TOWARD_EVEN", spread=1e6)
    quant_case("q_i8_f64", 3150, (6, 11), (0,), "i8", "ROUND_NEAREST_TOWARD_EVEN", real="f64")
    quant_case("q_i32_f64", 3160, (40,), (), "i32", "ROUND_NEAREST_DOWNWARD", real="f64", spread=1e8)

    np.savez_compressed(os.path.join(HERE, "ref_vectors.npz"), **arrays)
    with open(os.path.join(HERE, "ref_vectors.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    print("ref_vectors:", len(manifest), "cases,", os.path.getsize(os.path.join(HERE, "ref_vectors.npz")), "bytes")


POOL_CASES = [
    # name, seed, op, dtype, N, C, in_sp, window, stride, pad_below, pad_above, include_padding
    ("max_u8_resnet_stem", 4001, "max", "u8", 1, 16, (28, 28), (3, 3), (2, 2), (1, 1), (1, 1), False),
    ("max_i8_pad", 4002, "max", "i8", 2, 5, (9, 7), (3, 2), (2, 1), (1, 0), (0, 1), False),
    ("max_i8_window_in_padding", 4003, "max", "i8", 1, 3, (4, 4), (2, 2), (3, 3), (2, 2), (2, 2), False),
    ("max_f32_3d", 4004, "max", "f32", 1, 2, (5, 6, 4), (2, 3, 2), (1, 2, 1), (1, 0, 1), (0, 1, 1), False),
    ("max_i32_1d", 4005, "max", "i32", 2, 3, (17,), (4,), (3,), (2,), (1,), False),
    ("avg_u8_global7x7_wraps", 4010, "avg", "u8", 2, 8, (7, 7), (7, 7), (1, 1), (0, 0), (0, 0), False),
    ("avg_i8_global7x7_wraps", 4011, "avg", "i8", 2, 8, (7, 7), (7, 7), (1, 1), (0, 0), (0, 0), False),
    ("avg_u8_pad_excluded", 4012, "avg", "u8", 1, 4, (6, 5), (3, 3), (2, 2), (1, 1), (1, 1), False),
    ("avg_u8_pad_included", 4013, "avg", "u8", 1, 4, (6, 5), (3, 3), (2, 2), (1, 1), (1, 1), True),
    ("avg_i8_ties", 4014, "avg", "i8", 1, 6, (8, 8), (2, 1), (2, 1), (0, 0), (0, 0), False),
    ("avg_f32", 4015, "avg", "f32", 1, 3, (6, 6), (3, 3), (1, 1), (1, 1), (1, 1), True),
]


def pool_input(seed, dtype, shape):
    from ngraph_amd import synth

    if dtype == "f32":
        return synth.normal_f32(seed, shape)
    lo, hi = {"u8": (0, 255), "i8": (-128, 127), "i32": (-(2**20), 2**20)}[dtype]
    return synth.uniform_int(seed, shape, lo, hi, {"u8": np.uint8, "i8": np.int8, "i32": np.int32}[dtype])


def pool_vectors():
    """outputs of runtime::reference::max_pool / avg_pool (oracle/_ref) on seeded inputs"""
    import oracle_lib as O
    from ngraph_amd import hipq as H

    if not O.have_ref():
        raise SystemExit("oracle/_ref is not built: make -C oracle ref")
    arrays, manifest = {}, []
    for name, seed, op, dtype, N, Cc, in_sp, win, st, pb, pa, incl in POOL_CASES:
        d = H.make_pool_desc(op, dtype, N, Cc, list(in_sp), list(win), list(st), list(pb), list(pa), incl)
        x = pool_input(seed, dtype, d.in_shape())
        arrays[name] = O.ref_pool(d, x)
        manifest.append(dict(name=name, seed=seed, op=op, dtype=dtype, N=N, C=Cc, in_sp=list(in_sp), window=list(win), stride=list(st), pad_below=list(pb), pad_above=list(pa), include_padding=incl))
    np.savez_compressed(os.path.join(HERE, "pool_vectors.npz"), **arrays)
    with open(os.path.join(HERE, "pool_vectors.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    print("pool_vectors:", len(manifest), "cases")


def resnet50_vectors():
    """The synthetic int8 ResNet-50 of ngraph_amd/resnet50.py on one seeded image, computed by the C
    restatement in oracle/ (the fused quantized ops it is made of exist only in the reference's CPU
    backend, which cannot be built here; the restatement of those ops is pinned on the reference's own
    test values).  Kept: the logits and a checksum of every op's output."""
    import oracle_lib as O
    from ngraph_amd import resnet50 as R

    class Oracle:
        quantize = staticmethod(lambda x, s, z, t: O.quantize(x, s, z, t))
        dequantize = staticmethod(lambda q, s, z: O.dequantize(q, s, z, "f32"))
        conv = staticmethod(lambda d, f, x, filt, bias, s, sc, ss: O.quantized_convolution_fused(d, f, x, filt, bias, s, sc, ss))
        pool = staticmethod(lambda d, x: O.pool(d, x))
        dot_bias = staticmethod(lambda d, f, a, w, bias, sc: O.quantized_dot_bias(d, f, a, w, bias, sc))

    O.port().orc_set_threads(8)
    image = R.synthetic_images(1)
    t = R.run(Oracle, image)
    O.port().orc_set_threads(1)
    sums = {op["name"]: int(t[op["name"]].view(np.uint8).astype(np.uint64).sum()) for op in R.layers()}
    np.savez_compressed(os.path.join(HERE, "resnet50_logits.npz"), logits=t["logits"])
    with open(os.path.join(HERE, "resnet50_logits.json"), "w") as f:
        # image_bit_sum: the f32 image is made with the host's log / cos / sin; a math library that rounds
        # one value differently changes this sum, and the tests say so instead of reporting wrong logits
        json.dump(dict(image_seed=42, image_bit_sum=int(image.view(np.uint32).astype(np.uint64).sum()), byte_sums=sums, logits=[float(v) for v in t["logits"].ravel()]), f, indent=0)
    print("resnet50_logits: 1000 logits,", len(sums), "byte sums")


if __name__ == "__main__":
    if "--resnet-only" in sys.argv:
        resnet50_vectors()
        sys.exit(0)
    if "--pool-only" not in sys.argv:
        parse_quantize_dequantize()
        copy_onnx_bins()
        ref_vectors()
    pool_vectors()
