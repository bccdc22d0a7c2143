"""ctypes access to the test oracle: oracle/libhipq_oracle.so (the C restatement) and, where it was
built, oracle/_ref/libngraph_ref.so (the real nGraph reference kernels).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from ngraph_amd import hipq as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PORT_PATH = os.path.join(ROOT, "oracle", "libhipq_oracle.so")
REF_PATH = os.path.join(ROOT, "oracle", "_ref", "libngraph_ref.so")

_port = None
_ref = None


def port():
    global _port
    if _port is None:
        if not os.path.exists(PORT_PATH):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "port"])
        lib = C.CDLL(PORT_PATH)
        vp = C.c_void_p
        lib.orc_set_threads.argtypes = [C.c_int]
        lib.orc_quantize.argtypes = [C.POINTER(H.QuantDesc), vp, vp, vp, vp]
        lib.orc_dequantize.argtypes = [C.POINTER(H.QuantDesc), vp, vp, vp, vp]
        lib.orc_conv_infer_output.argtypes = [C.POINTER(H.ConvDesc)]
        lib.orc_conv_accumulate.argtypes = [C.POINTER(H.ConvDesc), vp, vp, C.c_int32, C.c_int32, vp]
        lib.orc_quantized_convolution.argtypes = [C.POINTER(H.ConvDesc)] + [vp] * 9
        lib.orc_quantized_convolution_fused.argtypes = [C.POINTER(H.ConvDesc), C.POINTER(H.FusedDesc)] + [vp] * 7
        lib.orc_dot_accumulate.argtypes = [C.POINTER(H.DotDesc), vp, vp, C.c_int32, C.c_int32, vp]
        lib.orc_quantized_dot.argtypes = [C.POINTER(H.DotDesc)] + [vp] * 9
        lib.orc_quantized_dot_bias.argtypes = [C.POINTER(H.DotDesc), C.POINTER(H.FusedDesc)] + [vp] * 5
        lib.orc_pool.argtypes = [C.POINTER(H.PoolDesc), vp, vp]
        lib.orc_concat.argtypes = [C.c_int, C.c_int, C.POINTER(vp), C.POINTER(C.c_int64), C.c_int64, C.c_int64, vp]
        f = C.c_float
        lib.orc_get_scale.restype = f
        lib.orc_get_scale.argtypes = [f, f, C.c_int, C.c_int]
        lib.orc_get_bias_scale.restype = f
        lib.orc_get_bias_scale.argtypes = [f] * 4
        lib.orc_get_sum_scale.restype = f
        lib.orc_get_sum_scale.argtypes = [f] * 4
        lib.orc_get_dot_scale.restype = f
        lib.orc_get_dot_scale.argtypes = [f] * 6 + [C.c_int] * 3
        lib.orc_get_conv_requant_scale.restype = f
        lib.orc_get_conv_requant_scale.argtypes = [f, f, C.c_int, f, f, C.c_int, f, f, C.c_int]
        lib.orc_softmax_f32.argtypes = [vp, vp, C.c_int64, C.c_int64, C.c_int64]
        lib.orc_erf_f32.argtypes = [vp, vp, C.c_int64]
        lib.orc_gelu_f32.argtypes = [vp, vp, C.c_int64]
        lib.orc_layer_norm_f32.argtypes = [vp] * 6 + [C.c_int64, C.c_int64, C.c_double]
        lib.orc_batch_matmul_f32.argtypes = [vp] * 3 + [C.c_int64] * 4 + [C.c_int] * 2
        _port = lib
    return _port


def have_ref() -> bool:
    return os.path.exists(REF_PATH)


def ref():
    global _ref
    if _ref is None:
        lib = C.CDLL(REF_PATH)
        vp, i64p = C.c_void_p, C.POINTER(C.c_int64)
        lib.ref_quantized_convolution.argtypes = [C.c_int] + [i64p] * 8 + [C.c_int] * 3 + [vp] * 9
        lib.ref_quantized_dot.argtypes = [C.c_int64] * 3 + [C.c_int] * 3 + [vp] * 9
        lib.ref_quantize.argtypes = [C.c_int, i64p, C.c_uint32, C.c_int, C.c_int, C.c_int] + [vp] * 4
        lib.ref_dequantize.argtypes = [C.c_int, i64p, C.c_uint32, C.c_int, C.c_int] + [vp] * 4
        lib.ref_pool.argtypes = [C.c_int] * 3 + [i64p] * 6 + [C.c_int, vp, vp]
        if hasattr(lib, "ref_softmax_f32"):
            lib.ref_softmax_f32.argtypes = [vp, vp, i64p, C.c_int, C.c_uint32]
            lib.ref_sum_f32.argtypes = [vp, vp, i64p, C.c_int, C.c_uint32]
            lib.ref_erf_f32.argtypes = [vp, vp, C.c_int64]
        if hasattr(lib, "ref_batch_mat_mul_f32"):
            lib.ref_batch_mat_mul_f32.argtypes = [vp] * 3 + [C.c_int64] * 4
        _ref = lib
    return _ref


def _ptr(a):
    return None if a is None else a.ctypes.data


def _arr(x, dtype):
    return np.ascontiguousarray(np.asarray(x, dtype=dtype))


def _ok(rc):
    if rc != 0:
        raise RuntimeError(f"oracle returned status {rc}")


# ------------------------------------------------------------------ C restatement


def quantize(x, scale, zp, quant_t, axes=(), round_mode=H.RNE):
    x = np.ascontiguousarray(x)
    qt = H.dtype_code(quant_t)
    d = H.make_quant_desc(x.shape, axes, x.dtype, qt, round_mode)
    s, z = _arr(scale, x.dtype), _arr(zp, H.NP_OF[qt])
    out = np.empty(x.shape, dtype=H.NP_OF[qt])
    _ok(port().orc_quantize(C.byref(d), _ptr(x), _ptr(s), _ptr(z), _ptr(out)))
    return out


def dequantize(q, scale, zp, real_t=H.F32, axes=()):
    q = np.ascontiguousarray(q)
    rt = H.dtype_code(real_t)
    d = H.make_quant_desc(q.shape, axes, rt, q.dtype)
    s, z = _arr(scale, H.NP_OF[rt]), _arr(zp, q.dtype)
    out = np.empty(q.shape, dtype=H.NP_OF[rt])
    _ok(port().orc_dequantize(C.byref(d), _ptr(q), _ptr(s), _ptr(z), _ptr(out)))
    return out


def conv_accumulate(desc, data, filt, data_zp=0, filter_zp=0):
    data, filt = np.ascontiguousarray(data), np.ascontiguousarray(filt)
    out = np.empty(desc.out_shape(), dtype=np.int32)
    _ok(port().orc_conv_accumulate(C.byref(desc), _ptr(data), _ptr(filt), int(data_zp), int(filter_zp), _ptr(out)))
    return out


def quantized_convolution(desc, data, filt, data_scale, data_zp, filter_scale, filter_zp, out_scale, out_zp):
    data, filt = np.ascontiguousarray(data), np.ascontiguousarray(filt)
    s = [_arr(v, np.float32) for v in (data_scale, filter_scale, out_scale)]
    z = [_arr(data_zp, H.NP_OF[desc.data_t]), _arr(filter_zp, H.NP_OF[desc.filter_t]), _arr(out_zp, H.NP_OF[desc.out_t])]
    out = np.empty(desc.out_shape(), dtype=H.NP_OF[desc.out_t])
    _ok(
        port().orc_quantized_convolution(
            C.byref(desc), _ptr(data), _ptr(filt), _ptr(s[0]), _ptr(z[0]), _ptr(s[1]), _ptr(z[1]), _ptr(s[2]), _ptr(z[2]), _ptr(out)
        )
    )
    return out


def quantized_convolution_fused(desc, fused, data, filt, bias, sum_in, scale, sum_scale):
    data, filt = np.ascontiguousarray(data), np.ascontiguousarray(filt)
    b = None if bias is None else _arr(bias, np.int32)
    sm = None if sum_in is None else np.ascontiguousarray(sum_in)
    sc = _arr(scale, np.float32)
    ss = None if sum_scale is None else _arr(sum_scale, np.float32)
    out = np.empty(desc.out_shape(), dtype=H.NP_OF[desc.out_t])
    _ok(
        port().orc_quantized_convolution_fused(
            C.byref(desc), C.byref(fused), _ptr(data), _ptr(filt), _ptr(b), _ptr(sm), _ptr(sc), _ptr(ss), _ptr(out)
        )
    )
    return out


def dot_accumulate(desc, a, b, a_zp=0, b_zp=0):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    out = np.empty((int(desc.M), int(desc.N)), dtype=np.int32)
    _ok(port().orc_dot_accumulate(C.byref(desc), _ptr(a), _ptr(b), int(a_zp), int(b_zp), _ptr(out)))
    return out


def quantized_dot(desc, a, b, a_scale, a_zp, b_scale, b_zp, out_scale, out_zp):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    s = [_arr(v, np.float32) for v in (a_scale, b_scale, out_scale)]
    z = [_arr(a_zp, H.NP_OF[desc.a_t]), _arr(b_zp, H.NP_OF[desc.b_t]), _arr(out_zp, H.NP_OF[desc.out_t])]
    out = np.empty((int(desc.M), int(desc.N)), dtype=H.NP_OF[desc.out_t])
    _ok(
        port().orc_quantized_dot(
            C.byref(desc), _ptr(a), _ptr(b), _ptr(s[0]), _ptr(z[0]), _ptr(s[1]), _ptr(z[1]), _ptr(s[2]), _ptr(z[2]), _ptr(out)
        )
    )
    return out


def quantized_dot_bias(desc, fused, a, w, bias, scale):
    a, w = np.ascontiguousarray(a), np.ascontiguousarray(w)
    b = None if bias is None else _arr(bias, np.int32)
    sc = _arr(scale, np.float32)
    out = np.empty((int(desc.M), int(desc.N)), dtype=H.NP_OF[desc.out_t])
    _ok(port().orc_quantized_dot_bias(C.byref(desc), C.byref(fused), _ptr(a), _ptr(w), _ptr(b), _ptr(sc), _ptr(out)))
    return out


# ------------------------------------------------------------------ real reference (oracle/_ref)


def _i64(v):
    return (C.c_int64 * len(v))(*[int(x) for x in v])


def ref_quantized_convolution(desc, data, filt, data_scale, data_zp, filter_scale, filter_zp, out_scale, out_zp):
    """desc must use the reference's NCX layouts."""
    assert desc.data_layout == H.NCX and desc.out_layout == H.NCX
    ns = desc.n_spatial
    data, filt = np.ascontiguousarray(data), np.ascontiguousarray(filt)
    s = [_arr(v, np.float32) for v in (data_scale, filter_scale, out_scale)]
    z = [_arr(data_zp, H.NP_OF[desc.data_t]), _arr(filter_zp, H.NP_OF[desc.filter_t]), _arr(out_zp, H.NP_OF[desc.out_t])]
    out = np.empty(desc.out_shape(), dtype=H.NP_OF[desc.out_t])
    rc = ref().ref_quantized_convolution(
        ns,
        _i64(desc.data_shape()),
        _i64(desc.filter_shape()),
        _i64(desc.out_shape()),
        _i64(list(desc.stride)[:ns]),
        _i64(list(desc.dilation)[:ns]),
        _i64(list(desc.pad_below)[:ns]),
        _i64(list(desc.pad_above)[:ns]),
        _i64(list(desc.data_dilation)[:ns]),
        desc.data_t,
        desc.filter_t,
        desc.out_t,
        _ptr(data),
        _ptr(filt),
        _ptr(s[0]),
        _ptr(z[0]),
        _ptr(s[1]),
        _ptr(z[1]),
        _ptr(s[2]),
        _ptr(z[2]),
        _ptr(out),
    )
    _ok(rc)
    return out


def ref_quantized_dot(desc, a, b, a_scale, a_zp, b_scale, b_zp, out_scale, out_zp):
    assert desc.b_layout == H.B_KN
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    s = [_arr(v, np.float32) for v in (a_scale, b_scale, out_scale)]
    z = [_arr(a_zp, H.NP_OF[desc.a_t]), _arr(b_zp, H.NP_OF[desc.b_t]), _arr(out_zp, H.NP_OF[desc.out_t])]
    out = np.empty((int(desc.M), int(desc.N)), dtype=H.NP_OF[desc.out_t])
    rc = ref().ref_quantized_dot(
        desc.M, desc.K, desc.N, desc.a_t, desc.b_t, desc.out_t, _ptr(a), _ptr(b), _ptr(s[0]), _ptr(z[0]), _ptr(s[1]), _ptr(z[1]), _ptr(s[2]), _ptr(z[2]), _ptr(out)
    )
    _ok(rc)
    return out


def ref_quantize(x, scale, zp, quant_t, axes=(), round_mode=H.RNE):
    x = np.ascontiguousarray(x)
    qt = H.dtype_code(quant_t)
    s, z = _arr(scale, x.dtype), _arr(zp, H.NP_OF[qt])
    out = np.empty(x.shape, dtype=H.NP_OF[qt])
    mask = sum(1 << int(a) for a in axes)
    rm = round_mode if isinstance(round_mode, int) else H.ROUND_MODES.index(round_mode)
    _ok(ref().ref_quantize(x.ndim, _i64(x.shape), mask, H.dtype_code(x.dtype), qt, rm, _ptr(x), _ptr(s), _ptr(z), _ptr(out)))
    return out


def ref_dequantize(q, scale, zp, real_t=H.F32, axes=()):
    q = np.ascontiguousarray(q)
    rt = H.dtype_code(real_t)
    s, z = _arr(scale, H.NP_OF[rt]), _arr(zp, q.dtype)
    out = np.empty(q.shape, dtype=H.NP_OF[rt])
    mask = sum(1 << int(a) for a in axes)
    _ok(ref().ref_dequantize(q.ndim, _i64(q.shape), mask, rt, H.dtype_code(q.dtype), _ptr(q), _ptr(s), _ptr(z), _ptr(out)))
    return out


def pool(desc, x):
    """C restatement of MaxPool / AvgPool in either layout"""
    x = np.ascontiguousarray(x)
    out = np.empty(desc.out_shape(), dtype=x.dtype)
    rc = port().orc_pool(C.byref(desc), _ptr(x), _ptr(out))
    if rc == -2:
        raise RuntimeError("AvgPool elements == 0, must be non-zero")
    _ok(rc)
    return out


def ref_pool(desc, x):
    """runtime::reference::max_pool / avg_pool themselves (NCX tensors only)"""
    assert desc.layout == H.NCX
    ns = desc.n_spatial
    x = np.ascontiguousarray(x)
    out = np.empty(desc.out_shape(), dtype=x.dtype)
    rc = ref().ref_pool(
        desc.op, desc.dtype, ns, _i64(desc.in_shape()), _i64(desc.out_shape()), _i64(list(desc.window)[:ns]), _i64(list(desc.stride)[:ns]),
        _i64(list(desc.pad_below)[:ns]), _i64(list(desc.pad_above)[:ns]), desc.include_padding, _ptr(x), _ptr(out)
    )
    if rc == -2:
        raise RuntimeError("AvgPool elements == 0, must be non-zero")
    _ok(rc)
    return out


def concat(arrays, axis):
    arrays = [np.ascontiguousarray(a) for a in arrays]
    shape = list(arrays[0].shape)
    outer, inner = int(np.prod(shape[:axis])), int(np.prod(shape[axis + 1 :]))
    extents = [a.shape[axis] for a in arrays]
    shape[axis] = sum(extents)
    out = np.empty(shape, dtype=arrays[0].dtype)
    ptrs = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    ext = (C.c_int64 * len(arrays))(*extents)
    _ok(port().orc_concat(arrays[0].dtype.itemsize, len(arrays), ptrs, ext, outer, inner, _ptr(out)))
    return out


# ---- fp32 glue ------------------------------------------------------------------------------------

def softmax(x, axes=()):
    x = np.ascontiguousarray(x, dtype=np.float32)
    outer, axis, inner = H._axes_run(x.shape, axes)
    out = np.empty_like(x)
    _ok(port().orc_softmax_f32(_ptr(x), _ptr(out), outer, axis, inner))
    return out


def erf(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    _ok(port().orc_erf_f32(_ptr(x), _ptr(out), x.size))
    return out


def gelu(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    _ok(port().orc_gelu_f32(_ptr(x), _ptr(out), x.size))
    return out


def layer_norm(x, scale=None, bias=None, begin_norm_axis=1, epsilon=1e-5):
    x = np.ascontiguousarray(x, dtype=np.float32)
    n_axis = begin_norm_axis if begin_norm_axis >= 0 else x.ndim + begin_norm_axis
    rows = int(np.prod(x.shape[:n_axis], dtype=np.int64))
    cols = int(np.prod(x.shape[n_axis:], dtype=np.int64))
    sc = np.ascontiguousarray(scale, dtype=np.float32) if scale is not None else None
    bi = np.ascontiguousarray(bias, dtype=np.float32) if bias is not None else None
    out = np.empty_like(x)
    mean = np.empty(x.shape[:n_axis], dtype=np.float32)
    var = np.empty(x.shape[:n_axis], dtype=np.float32)
    _ok(port().orc_layer_norm_f32(_ptr(x), _ptr(sc), _ptr(bi), _ptr(out), _ptr(mean), _ptr(var), rows, cols, float(epsilon)))
    return out, mean, var


def _mask(axes):
    m = 0
    for a in axes:
        m |= 1 << a
    return m


def ref_softmax(x, axes):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    axes = range(x.ndim) if len(axes) == 0 else axes
    assert ref().ref_softmax_f32(_ptr(x), _ptr(out), _i64(x.shape), x.ndim, _mask(axes)) == 0
    return out


def ref_sum(x, axes):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty([d for i, d in enumerate(x.shape) if i not in axes], dtype=np.float32)
    assert ref().ref_sum_f32(_ptr(x), _ptr(out), _i64(x.shape), x.ndim, _mask(axes)) == 0
    return out


def ref_erf(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    assert ref().ref_erf_f32(_ptr(x), _ptr(out), x.size) == 0
    return out


def batch_matmul(a, b, transpose_a=False, transpose_b=False):
    a, b = np.ascontiguousarray(a, dtype=np.float32), np.ascontiguousarray(b, dtype=np.float32)
    batch = a.shape[0]
    M, K = (a.shape[2], a.shape[1]) if transpose_a else (a.shape[1], a.shape[2])
    N = b.shape[1] if transpose_b else b.shape[2]
    out = np.empty((batch, M, N), dtype=np.float32)
    _ok(port().orc_batch_matmul_f32(_ptr(a), _ptr(b), _ptr(out), batch, M, K, N, int(transpose_a), int(transpose_b)))
    return out


def ref_batch_matmul(a, b):
    a, b = np.ascontiguousarray(a, dtype=np.float32), np.ascontiguousarray(b, dtype=np.float32)
    batch, M, K = a.shape
    N = b.shape[2]
    out = np.empty((batch, M, N), dtype=np.float32)
    assert ref().ref_batch_mat_mul_f32(_ptr(a), _ptr(b), _ptr(out), batch, M, K, N) == 0
    return out
