"""Builds descriptors and inputs from the golden manifests; shared by the oracle tests (CPU) and
the parity tests (GPU) so that both sides see exactly the same cases."""
import os

import numpy as np

from ngraph_amd import hipq as H
from ngraph_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def conv_from_manifest(m, data_layout=H.NCX, out_layout=H.NCX):
    """-> (desc, data NCX, filter, scales, zps).  Inputs are always generated in the reference's
    NCX order; use to_layout() to hand them to a channels-last descriptor."""
    kw = {k: list(v) for k, v in m["kw"].items()}
    d = H.make_conv_desc(
        m["N"], m["C"], m["K"], m["in_sp"], m["f_sp"], data_t=m["types"][0], filter_t=m["types"][1], out_t=m["types"][2],
        data_layout=data_layout, out_layout=out_layout, **kw
    )
    ncx = H.make_conv_desc(m["N"], m["C"], m["K"], m["in_sp"], m["f_sp"], **kw)
    data = synth.uniform_int(m["seed"], ncx.data_shape(), m["data_range"][0], m["data_range"][1], np.uint8)
    filt = synth.uniform_int(m["seed"] + 1, ncx.filter_shape(), m["filter_range"][0], m["filter_range"][1], H.NP_OF[d.filter_t])
    return d, data, filt, m["scales"], m["zps"]


def to_nxc(a):
    """[N,C,spatial...] -> [N,spatial...,C]"""
    return np.ascontiguousarray(np.moveaxis(a, 1, -1))


def to_ncx(a):
    """[N,spatial...,C] -> [N,C,spatial...]"""
    return np.ascontiguousarray(np.moveaxis(a, -1, 1))


def dot_from_manifest(m):
    d = H.make_dot_desc(m["M"], m["K"], m["N"], a_t=m["types"][0], b_t=m["types"][1], out_t=m["types"][2])
    a = synth.uniform_int(m["seed"], (m["M"], m["K"]), 0, 255, np.uint8)
    b = synth.uniform_int(m["seed"] + 1, (m["K"], m["N"]), m["b_range"][0], m["b_range"][1], H.NP_OF[d.b_t])
    return d, a, b, m["scales"], m["zps"]


def kat_conv(k):
    """descriptor + arrays of one hand-transcribed convolution vector"""
    ds, fs = k["data_shape"], k["filter_shape"]
    ns = len(ds) - 2
    ones = [1] * ns
    out_t = k["out_t"]
    d = H.make_conv_desc(
        ds[0], ds[1], fs[0], ds[2:], fs[2:], stride=k.get("stride", ones), dilation=k.get("dilation", ones),
        pad_below=k.get("pad_below", [0] * ns), pad_above=k.get("pad_above", [0] * ns), data_dilation=k.get("data_dilation", ones),
        data_t=k.get("data_t", "u8"), filter_t=k.get("filter_t", "i8"), out_t="i8" if out_t == "u8_via_i8_convert" else out_t,
    )
    if "data_file" in k:
        data = np.fromfile(os.path.join(GOLDEN, k["data_file"]), dtype=np.uint8).reshape(ds)
    elif "data_iota_from" in k:
        data = (np.arange(int(np.prod(ds))) + k["data_iota_from"]).astype(np.uint8).reshape(ds)
    else:
        data = np.array(k["data"], dtype=H.NP_OF[d.data_t]).reshape(ds)
    filt = np.array(k["filter"], dtype=H.NP_OF[d.filter_t]).reshape(fs)
    if "expected_file" in k:
        exp = np.fromfile(os.path.join(GOLDEN, k["expected_file"]), dtype=np.uint8)
    else:
        exp = np.array(k["expected"])
    return d, data, filt, exp


def brute_conv_acc(d, data, filt, dzp=0, fzp=0):
    """Independent int64 convolution in numpy/pure Python on the NCX layout: pads and dilates the
    input explicitly with a validity mask instead of testing tap membership."""
    ns = d.n_spatial
    N, Cc, K = int(d.N), int(d.C), int(d.K)
    x = data.astype(np.int64) - dzp
    w = filt.astype(np.int64) - fzp
    # data dilation: scatter into a zero grid (gaps contribute nothing, like a mask of zeros)
    dil_shape = [(int(d.in_sp[i]) - 1) * int(d.data_dilation[i]) + 1 for i in range(ns)]
    xd = np.zeros([N, Cc] + dil_shape, dtype=np.int64)
    sl = (slice(None), slice(None)) + tuple(slice(None, None, int(d.data_dilation[i])) for i in range(ns))
    xd[sl] = x
    # padding (negative = crop)
    for i in range(ns):
        pb, pa = int(d.pad_below[i]), int(d.pad_above[i])
        ax = 2 + i
        if pb < 0:
            xd = np.take(xd, range(-pb, xd.shape[ax]), axis=ax)
            pb = 0
        if pa < 0:
            xd = np.take(xd, range(0, xd.shape[ax] + pa), axis=ax)
            pa = 0
        padw = [(0, 0)] * xd.ndim
        padw[ax] = (pb, pa)
        xd = np.pad(xd, padw)
    out_sp = [int(d.out_sp[i]) for i in range(ns)]
    out = np.zeros([N, K] + out_sp, dtype=np.int64)
    for taps in np.ndindex(*[int(d.f_sp[i]) for i in range(ns)]):
        sl = [slice(None), slice(None)]
        for i in range(ns):
            start = taps[i] * int(d.dilation[i])
            sl.append(slice(start, start + (out_sp[i] - 1) * int(d.stride[i]) + 1, int(d.stride[i])))
        patch = xd[tuple(sl)]  # N, C, out...
        wt = w[(slice(None), slice(None)) + taps]  # K, C
        out += np.einsum("nc...,kc->nk...", patch, wt)
    return out


def dot_bias_closed_form(a, w, bias, scales, out_t, relu):
    """QuantizedDotBias from first principles, independent of the oracle's loops: the integer sums
    through float64 BLAS (exact: 255 * 127 * K stays far below 2^53), then the three float32 steps
    the reference's CPU backend hands oneDNN (src/ngraph/runtime/cpu/builder/quantized_dot.cpp:36-125,
    dnnl_emitter.hpp:737-761) -- f32(acc) + f32(bias), times scale[n] (or the one scale), relu -- and
    round-half-to-even with saturation for 8-bit outputs.  a [M,K] u8/i8, w [N,K] i8."""
    acc = (a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64)
    assert np.all(np.abs(acc) < 2**31)
    v = acc.astype(np.float32)
    if bias is not None:
        v = v + np.asarray(bias, np.int32).astype(np.float32)[None, :]
    sc = np.asarray(scales, np.float32).reshape(-1)
    v = (v * (sc[None, :] if sc.size > 1 else sc[0])).astype(np.float32)
    if relu:
        v = np.maximum(v, np.float32(0))
    if out_t == "f32":
        return v
    lo, hi = (0, 255) if out_t == "u8" else (-128, 127)
    return np.clip(np.rint(v), lo, hi).astype(np.uint8 if out_t == "u8" else np.int8)
