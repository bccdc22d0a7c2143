"""MaxPool / AvgPool / Concat: the integer glue between quantized convolutions.

CPU: the C restatement against vectors written by the compiled reference kernels
(runtime::reference::max_pool / avg_pool, tests/golden/pool_vectors.*), against the compiled
reference itself where it is built, and against a numpy formulation that shares no code with it.
GPU: the HIP kernels against the restatement, in both tensor layouts.
"""
import json
import os

import numpy as np
import pytest

import cases
import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
NP = {"u8": np.uint8, "i8": np.int8, "i32": np.int32, "f32": np.float32}


def _input(seed, dtype, shape):
    if dtype == "f32":
        return synth.normal_f32(seed, shape)
    lo, hi = {"u8": (0, 255), "i8": (-128, 127), "i32": (-(2**20), 2**20)}[dtype]
    return synth.uniform_int(seed, shape, lo, hi, NP[dtype])


def _manifest():
    with open(os.path.join(GOLDEN, "pool_vectors.json")) as f:
        return json.load(f), np.load(os.path.join(GOLDEN, "pool_vectors.npz"))


def _desc(m, layout=H.NCX):
    return H.make_pool_desc(m["op"], m["dtype"], m["N"], m["C"], m["in_sp"], m["window"], m["stride"], m["pad_below"], m["pad_above"], m["include_padding"], layout)


def _numpy_pool(d, x):
    """independent formulation on NCX data: windows gathered with a padded array and a validity mask"""
    ns = d.n_spatial
    win, st, pb, pa = (list(v)[:ns] for v in (d.window, d.stride, d.pad_below, d.pad_above))
    xp = np.pad(x.astype(np.float64), [(0, 0), (0, 0)] + [(pb[i], pa[i]) for i in range(ns)])
    mask = np.pad(np.ones(x.shape, bool), [(0, 0), (0, 0)] + [(pb[i], pa[i]) for i in range(ns)])
    out = np.empty(d.out_shape(), dtype=x.dtype)
    for idx in np.ndindex(*[int(v) for v in list(d.out_sp)[:ns]]):
        sl = tuple(slice(idx[i] * st[i], idx[i] * st[i] + win[i]) for i in range(ns))
        w = xp[(slice(None), slice(None)) + sl].reshape(x.shape[0], x.shape[1], -1)
        mk = mask[(slice(None), slice(None)) + sl].reshape(x.shape[0], x.shape[1], -1)
        if d.op == H.POOL_MAX:
            lowest = np.finfo(np.float32).min if x.dtype == np.float32 else np.iinfo(x.dtype).min
            r = np.where(mk, w, float(lowest)).max(axis=-1)
            out[(slice(None), slice(None)) + idx] = r.astype(x.dtype)
        else:
            cnt = mk.shape[-1] if d.include_padding else mk[0, 0].sum()
            total = np.where(mk, w, 0.0).sum(axis=-1)
            if x.dtype.itemsize == 1:
                # the reference sums in the 8-bit type: wrap the exact sum, then nearbyint of the f32 quotient
                wrapped = total.astype(np.int64).astype(x.dtype)
                r = np.rint(wrapped.astype(np.float32) / np.float32(cnt))
                out[(slice(None), slice(None)) + idx] = r.astype(x.dtype)
            else:
                s = np.zeros(total.shape, np.float32)
                for j in range(w.shape[-1]):  # same left-to-right f32 summation order as the reference's window walk
                    s = (s + np.where(mk[..., j], w[..., j], 0.0).astype(np.float32)).astype(np.float32)
                out[(slice(None), slice(None)) + idx] = (s / np.float32(cnt)).astype(x.dtype)
    return out


def _known_answers():
    with open(os.path.join(GOLDEN, "pool_known_answers.json")) as f:
        return json.load(f)["cases"]


def test_oracle_pool_against_reference_test_values():
    """the values the reference's own backend tests expect (test/backend/pool.in.cpp)"""
    for m in _known_answers():
        d = _desc(m)
        x = np.array(m["x"], dtype=NP[m["dtype"]]).reshape(d.in_shape())
        y = np.array(m["y"], dtype=NP[m["dtype"]]).reshape(d.out_shape())
        assert np.array_equal(O.pool(d, x), y), m["name"]


def test_oracle_pool_against_reference_vectors():
    manifest, arrays = _manifest()
    assert len(manifest) >= 11
    for m in manifest:
        d = _desc(m)
        x = _input(m["seed"], m["dtype"], d.in_shape())
        got = O.pool(d, x)
        assert got.dtype == arrays[m["name"]].dtype
        assert np.array_equal(got, arrays[m["name"]]), m["name"]
        # channels-last descriptor on the same data
        dl = _desc(m, H.NXC)
        assert np.array_equal(cases.to_ncx(O.pool(dl, cases.to_nxc(x))), arrays[m["name"]]), (m["name"], "nxc")


def test_oracle_pool_against_numpy_formulation():
    manifest, _ = _manifest()
    for m in manifest:
        if m["dtype"] == "i32" and m["op"] == "avg":
            continue
        d = _desc(m)
        x = _input(m["seed"], m["dtype"], d.in_shape())
        assert np.array_equal(O.pool(d, x), _numpy_pool(d, x)), m["name"]


def test_pool_vectors_cover_the_traps():
    """the fixtures must contain what makes the reference's integer pooling peculiar"""
    manifest, arrays = _manifest()
    by = {m["name"]: m for m in manifest}
    # 8-bit sums of a 7x7 window wrap: the reference's result differs from the true mean
    m = by["avg_u8_global7x7_wraps"]
    d = _desc(m)
    x = _input(m["seed"], "u8", d.in_shape())
    true_mean = np.rint(x.reshape(m["N"], m["C"], -1).astype(np.float64).mean(axis=-1))
    assert (arrays[m["name"]].reshape(m["N"], m["C"]) != true_mean).any()
    # a window wholly inside the padding yields the type's lowest value
    assert (arrays["max_i8_window_in_padding"] == -128).any()
    # exact .5 quotients round to even
    m = by["avg_i8_ties"]
    d = _desc(m)
    x = _input(m["seed"], "i8", d.in_shape()).astype(np.int32)
    pair = x[:, :, 0::2, :] + x[:, :, 1::2, :]
    ties = (pair % 2 != 0) & (np.abs(pair) < 128)
    assert ties.any()
    assert np.array_equal(arrays[m["name"]].astype(np.int32)[ties], (np.rint(pair / 2.0)).astype(np.int32)[ties])


@pytest.mark.skipif(not O.have_ref(), reason="oracle/_ref not built")
def test_oracle_pool_against_compiled_reference_random():
    rng = np.random.RandomState(7)
    for trial in range(40):
        ns = int(rng.randint(1, 4))
        dtype = ["u8", "i8", "f32", "i32"][trial % 4]
        op = "max" if (dtype == "i32" or trial % 3 == 0) else "avg"
        in_sp = [int(rng.randint(3, 9)) for _ in range(ns)]
        win = [int(rng.randint(1, 4)) for _ in range(ns)]
        st = [int(rng.randint(1, 4)) for _ in range(ns)]
        pb = [int(rng.randint(0, w)) for w in win]
        pa = [int(rng.randint(0, w)) for w in win]
        d = H.make_pool_desc(op, dtype, int(rng.randint(1, 3)), int(rng.randint(1, 5)), in_sp, win, st, pb, pa, bool(trial & 1))
        x = _input(900 + trial, dtype, d.in_shape())
        try:
            exp = O.ref_pool(d, x)
        except RuntimeError:
            with pytest.raises(RuntimeError):
                O.pool(d, x)
            continue
        assert np.array_equal(O.pool(d, x), exp), (trial, op, dtype, in_sp, win, st, pb, pa)


def test_oracle_concat():
    a = synth.uniform_int(1, (2, 3, 4, 5), 0, 255, np.uint8)
    b = synth.uniform_int(2, (2, 7, 4, 5), 0, 255, np.uint8)
    c = synth.uniform_int(3, (2, 1, 4, 5), 0, 255, np.uint8)
    assert np.array_equal(O.concat([a, b, c], 1), np.concatenate([a, b, c], axis=1))
    f = [synth.normal_f32(4 + i, (3, 2 + i)) for i in range(3)]
    assert np.array_equal(O.concat(f, 1), np.concatenate(f, axis=1))
    assert np.array_equal(O.concat([a, a], 0), np.concatenate([a, a], axis=0))


# ------------------------------------------------------------------ GPU


@pytest.mark.gpu
def test_gpu_pool_vectors(gpu_lib):
    manifest, arrays = _manifest()
    for m in manifest:
        print("[case]", m["name"], flush=True)
        d = _desc(m)
        x = _input(m["seed"], m["dtype"], d.in_shape())
        assert np.array_equal(H.pool(d, x), arrays[m["name"]]), m["name"]
        assert H.last_kernel().startswith(("max_pool", "avg_pool"))
        dl = _desc(m, H.NXC)
        assert np.array_equal(cases.to_ncx(H.pool(dl, cases.to_nxc(x))), arrays[m["name"]]), (m["name"], "nxc")


@pytest.mark.gpu
def test_gpu_pool_reference_test_values(gpu_lib):
    for m in _known_answers():
        print("[case]", m["name"], flush=True)
        d = _desc(m)
        x = np.array(m["x"], dtype=NP[m["dtype"]]).reshape(d.in_shape())
        y = np.array(m["y"], dtype=NP[m["dtype"]]).reshape(d.out_shape())
        assert np.array_equal(H.pool(d, x), y), m["name"]


@pytest.mark.gpu
def test_gpu_pool_resnet_shapes(gpu_lib):
    """ResNet-50's two pools at batch 8, u8: the stem's 3x3/2 max pool and the 7x7 global average"""
    for op, Cc, sp, win, st, pb in (("max", 64, (112, 112), (3, 3), (2, 2), (1, 1)), ("avg", 2048, (7, 7), (7, 7), (1, 1), (0, 0))):
        print("[case] resnet pool", op, flush=True)
        for layout in (H.NCX, H.NXC):
            d = H.make_pool_desc(op, "u8", 8, Cc, list(sp), list(win), list(st), list(pb), list(pb), False, layout)
            dn = H.make_pool_desc(op, "u8", 8, Cc, list(sp), list(win), list(st), list(pb), list(pb), False)
            x = synth.uniform_int(77, dn.in_shape(), 0, 255, np.uint8)
            O.port().orc_set_threads(8)
            exp = O.pool(dn, x)
            got = H.pool(d, cases.to_nxc(x) if layout == H.NXC else x)
            assert np.array_equal(cases.to_ncx(got) if layout == H.NXC else got, exp), (op, layout)


# (N, C, in_sp, window, stride, pad_below, pad_above): chosen to reach every variant of the 8-bit
# kernels -- widths that are / are not multiples of 4 on either side, planes small enough to share a
# workgroup (with a ragged last group), channel counts that are multiples of 16, of 4 only, and of
# neither, one and three spatial axes, windows that hang into the padding on every side
POOL8_SHAPES = [
    (2, 16, (12, 16), (3, 3), (2, 2), (1, 1), (1, 1)),
    (3, 5, (7, 7), (7, 7), (1, 1), (0, 0), (0, 0)),
    (1, 67, (7, 7), (7, 7), (1, 1), (0, 0), (0, 0)),
    (2, 4, (9, 10), (2, 3), (1, 2), (0, 2), (1, 0)),
    (1, 32, (8, 8), (2, 2), (2, 2), (0, 0), (0, 0)),
    (2, 20, (6, 12), (3, 2), (1, 1), (2, 1), (2, 1)),
    (1, 3, (70, 72), (3, 3), (2, 2), (1, 1), (1, 1)),
    (1, 2, (200, 200), (3, 3), (2, 2), (1, 1), (0, 0)),
    (2, 8, (33,), (4,), (3,), (2,), (3,)),
    (2, 16, (4, 5, 6), (2, 3, 2), (1, 2, 2), (1, 1, 0), (0, 1, 1)),
    (1, 48, (5, 5), (3, 3), (1, 1), (2, 2), (2, 2)),
    (2, 6, (7, 7), (7, 7), (1, 1), (0, 0), (0, 0)),
    (1, 100, (7, 7), (3, 3), (2, 2), (1, 1), (1, 1)),
    (4, 25, (5, 6), (2, 2), (1, 1), (0, 0), (0, 0)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("shape_id", range(len(POOL8_SHAPES)))
def test_gpu_pool_8bit_kernels(gpu_lib, monkeypatch, shape_id):
    N, Cc, in_sp, win, st, pb, pa = POOL8_SHAPES[shape_id]
    seen = set()
    for dtype in ("u8", "i8"):
        for op, incl in (("max", False), ("avg", False), ("avg", True)):
            if op == "avg" and not incl and any(b >= w for b, w in zip(pb, win)):
                continue
            print("[case] pool8", shape_id, dtype, op, incl, flush=True)
            dn = H.make_pool_desc(op, dtype, N, Cc, list(in_sp), list(win), list(st), list(pb), list(pa), incl)
            x = _input(500 + shape_id, dtype, dn.in_shape())
            try:
                exp = O.pool(dn, x)
            except RuntimeError:
                continue
            for layout in (H.NCX, H.NXC):
                d = H.make_pool_desc(op, dtype, N, Cc, list(in_sp), list(win), list(st), list(pb), list(pa), incl, layout)
                xin = cases.to_nxc(x) if layout == H.NXC else x
                got = H.pool(d, xin)
                seen.add(H.last_kernel())
                assert np.array_equal(cases.to_ncx(got) if layout == H.NXC else got, exp), (dtype, op, incl, layout, H.last_kernel())
                monkeypatch.setenv("HIPQ_NO_FAST_POOL", "1")
                slow = H.pool(d, xin)
                assert H.last_kernel() in ("max_pool", "avg_pool")
                monkeypatch.delenv("HIPQ_NO_FAST_POOL")
                assert np.array_equal(slow, got)
    print("kernels", sorted(seen), flush=True)


@pytest.mark.gpu
def test_gpu_pool_errors_and_empty(gpu_lib):
    lib = gpu_lib
    d = H.make_pool_desc("avg", "u8", 1, 2, [4, 4], [2, 2], [3, 3], [2, 2], [2, 2])
    x = H.DeviceBuffer(64)
    assert lib.hipq_pool(d, x.ptr, x.ptr, None) != 0  # window wholly in the padding: the reference throws
    assert b"padding" in lib.hipq_last_error()
    d = H.make_pool_desc("avg", "i32", 1, 2, [4, 4], [2, 2])
    assert lib.hipq_pool(d, x.ptr, x.ptr, None) != 0
    d = H.make_pool_desc("max", "u8", 0, 2, [4, 4], [2, 2])
    assert lib.hipq_pool(d, None, None, None) == 0  # empty batch


@pytest.mark.gpu
def test_gpu_concat(gpu_lib):
    print("[case] concat", flush=True)
    parts = [synth.uniform_int(10 + i, (3, c, 6, 5), 0, 255, np.uint8) for i, c in enumerate((64, 32, 1, 96))]
    assert np.array_equal(H.concat(parts, 1), np.concatenate(parts, axis=1))
    assert H.last_kernel() == "concat"
    wide = [parts[0], parts[1], parts[3]]  # every piece a multiple of 16 bytes: the 16-byte copy
    assert np.array_equal(H.concat(wide, 1), np.concatenate(wide, axis=1))
    odd = [synth.uniform_int(30 + i, (5, c, 3), -128, 127, np.int8) for i, c in enumerate((3, 1, 7))]
    assert np.array_equal(H.concat(odd, 1), np.concatenate(odd, axis=1))
    nh = [cases.to_nxc(p) for p in parts]
    assert np.array_equal(H.concat(nh, 3), np.concatenate(nh, axis=3))
    f = [synth.normal_f32(20 + i, (4, 2 + i, 3)) for i in range(3)]
    assert np.array_equal(H.concat(f, 1), np.concatenate(f, axis=1))
    assert np.array_equal(H.concat([parts[0], parts[0]], 0), np.concatenate([parts[0], parts[0]], axis=0))
