"""ctypes view of libhipq.so (declared in include/hipq.h).

Plumbing for the Python tests and the benchmark: descriptor structs, dtype codes and a loader
that fails loudly when the HIP library has not been built.  There is no CPU fallback here or
anywhere else in the package.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "csrc", "libhipq.so")

U8, I8, I32, F32, F64 = 0, 1, 2, 3, 4
NCX, NXC = 0, 1
B_KN, B_NK = 0, 1
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP, ERR_LIMIT = 0, 1, 2, 3, 4

ROUND_MODES = [
    "ROUND_NEAREST_TOWARD_INFINITY",
    "ROUND_NEAREST_TOWARD_ZERO",
    "ROUND_NEAREST_UPWARD",
    "ROUND_NEAREST_DOWNWARD",
    "ROUND_NEAREST_TOWARD_EVEN",
    "ROUND_TOWARD_INFINITY",
    "ROUND_TOWARD_ZERO",
    "ROUND_UP",
    "ROUND_DOWN",
]
RNE = ROUND_MODES.index("ROUND_NEAREST_TOWARD_EVEN")

NP_OF = {U8: np.uint8, I8: np.int8, I32: np.int32, F32: np.float32, F64: np.float64}
CODE_OF = {np.dtype(v): k for k, v in NP_OF.items()}
NAME_OF = {U8: "u8", I8: "i8", I32: "i32", F32: "f32", F64: "f64"}
CODE_OF_NAME = {v: k for k, v in NAME_OF.items()}


def dtype_code(x) -> int:
    if isinstance(x, str):
        return CODE_OF_NAME[x]
    if isinstance(x, int):
        return x
    return CODE_OF[np.dtype(x)]


class QuantDesc(C.Structure):
    _fields_ = [
        ("real_t", C.c_int32),
        ("quant_t", C.c_int32),
        ("rank", C.c_int32),
        ("round_mode", C.c_int32),
        ("axes_mask", C.c_uint32),
        ("reserved", C.c_uint32),
        ("shape", C.c_int64 * 8),
    ]


class ConvDesc(C.Structure):
    _fields_ = [
        ("n_spatial", C.c_int32),
        ("data_t", C.c_int32),
        ("filter_t", C.c_int32),
        ("out_t", C.c_int32),
        ("data_layout", C.c_int32),
        ("out_layout", C.c_int32),
        ("N", C.c_int64),
        ("C", C.c_int64),
        ("K", C.c_int64),
        ("in_sp", C.c_int64 * 3),
        ("f_sp", C.c_int64 * 3),
        ("out_sp", C.c_int64 * 3),
        ("stride", C.c_int64 * 3),
        ("dilation", C.c_int64 * 3),
        ("data_dilation", C.c_int64 * 3),
        ("pad_below", C.c_int64 * 3),
        ("pad_above", C.c_int64 * 3),
    ]

    def out_shape(self):
        sp = [int(self.out_sp[i]) for i in range(self.n_spatial)]
        if self.out_layout == NXC:
            return [int(self.N)] + sp + [int(self.K)]
        return [int(self.N), int(self.K)] + sp

    def data_shape(self):
        sp = [int(self.in_sp[i]) for i in range(self.n_spatial)]
        if self.data_layout == NXC:
            return [int(self.N)] + sp + [int(self.C)]
        return [int(self.N), int(self.C)] + sp

    def filter_shape(self):
        return [int(self.K), int(self.C)] + [int(self.f_sp[i]) for i in range(self.n_spatial)]

    def ops(self):
        """2 * MACs of the dense contraction (padding taps counted, as rooflines do)."""
        n = 2 * int(self.N) * int(self.K) * int(self.C)
        for i in range(self.n_spatial):
            n *= int(self.out_sp[i]) * int(self.f_sp[i])
        return n


class FusedDesc(C.Structure):
    _fields_ = [
        ("has_bias", C.c_int32),
        ("has_sum", C.c_int32),
        ("sum_t", C.c_int32),
        ("with_relu", C.c_int32),
        ("scale_count", C.c_int64),
    ]


class DotDesc(C.Structure):
    _fields_ = [
        ("a_t", C.c_int32),
        ("b_t", C.c_int32),
        ("out_t", C.c_int32),
        ("b_layout", C.c_int32),
        ("M", C.c_int64),
        ("K", C.c_int64),
        ("N", C.c_int64),
    ]


class PoolDesc(C.Structure):
    _fields_ = [
        ("op", C.c_int32),
        ("dtype", C.c_int32),
        ("layout", C.c_int32),
        ("n_spatial", C.c_int32),
        ("include_padding", C.c_int32),
        ("N", C.c_int64),
        ("C", C.c_int64),
        ("in_sp", C.c_int64 * 3),
        ("window", C.c_int64 * 3),
        ("stride", C.c_int64 * 3),
        ("pad_below", C.c_int64 * 3),
        ("pad_above", C.c_int64 * 3),
        ("out_sp", C.c_int64 * 3),
    ]

    def in_shape(self):
        sp = list(self.in_sp)[: self.n_spatial]
        return (self.N, self.C, *sp) if self.layout == NCX else (self.N, *sp, self.C)

    def out_shape(self):
        sp = list(self.out_sp)[: self.n_spatial]
        return (self.N, self.C, *sp) if self.layout == NCX else (self.N, *sp, self.C)


POOL_MAX, POOL_AVG = 0, 1


class QuantOut(C.Structure):
    """hipq_quant_out_t: a Quantize of a kernel's f32 result written beside it"""

    _fields_ = [("out", C.c_void_p), ("scale", C.c_void_p), ("zero_point", C.c_void_p), ("quant_t", C.c_int32), ("round_mode", C.c_int32)]


class MatmulView(C.Structure):
    """hipq_matmul_view_t: batch strides (two levels) and row strides of a, b and out, in elements"""

    _fields_ = [(n, C.c_int64) for n in ("batch_inner", "a_outer", "a_inner", "lda", "b_outer", "b_inner", "ldb", "o_outer", "o_inner", "ldo")]


class AttentionView(C.Structure):
    """hipq_attention_view_t: batch strides (two levels) and row strides of Q, K, V and out, in elements"""

    _fields_ = [(n, C.c_int64) for n in ("batch_inner", "q_outer", "q_inner", "ldq", "k_outer", "k_inner", "ldk", "v_outer", "v_inner", "ldv", "o_outer", "o_inner", "ldo")]


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 64),
        ("arch", C.c_char * 32),
        ("compute_units", C.c_int32),
        ("clock_mhz", C.c_int32),
        ("lds_bytes_per_cu", C.c_int32),
        ("reserved", C.c_int32),
        ("hbm_bytes", C.c_uint64),
    ]


def make_quant_desc(shape, axes, real_t, quant_t, round_mode=RNE) -> QuantDesc:
    d = QuantDesc()
    d.real_t, d.quant_t = dtype_code(real_t), dtype_code(quant_t)
    d.rank = len(shape)
    d.round_mode = round_mode if isinstance(round_mode, int) else ROUND_MODES.index(round_mode)
    d.axes_mask = sum(1 << int(a) for a in axes)
    for i, s in enumerate(shape):
        d.shape[i] = int(s)
    return d


def make_conv_desc(
    N,
    C_,
    K,
    in_sp,
    f_sp,
    stride=None,
    dilation=None,
    pad_below=None,
    pad_above=None,
    data_dilation=None,
    data_t=U8,
    filter_t=I8,
    out_t=I8,
    data_layout=NCX,
    out_layout=NCX,
) -> ConvDesc:
    ns = len(in_sp)
    d = ConvDesc()
    d.n_spatial = ns
    d.data_t, d.filter_t, d.out_t = dtype_code(data_t), dtype_code(filter_t), dtype_code(out_t)
    d.data_layout, d.out_layout = data_layout, out_layout
    d.N, d.C, d.K = N, C_, K
    for i in range(3):
        d.in_sp[i] = d.f_sp[i] = d.out_sp[i] = 1
        d.stride[i] = d.dilation[i] = d.data_dilation[i] = 1
        d.pad_below[i] = d.pad_above[i] = 0
    for i in range(ns):
        d.in_sp[i] = in_sp[i]
        d.f_sp[i] = f_sp[i]
        d.stride[i] = (stride or [1] * ns)[i]
        d.dilation[i] = (dilation or [1] * ns)[i]
        d.data_dilation[i] = (data_dilation or [1] * ns)[i]
        d.pad_below[i] = (pad_below or [0] * ns)[i]
        d.pad_above[i] = (pad_above or [0] * ns)[i]
    for i in range(ns):
        eff_in = (d.in_sp[i] - 1) * d.data_dilation[i] + 1 + d.pad_below[i] + d.pad_above[i]
        eff_f = (d.f_sp[i] - 1) * d.dilation[i] + 1
        if eff_in < eff_f:
            raise ValueError("convolution window larger than padded input")
        d.out_sp[i] = (eff_in - eff_f) // d.stride[i] + 1
    return d


def make_fused_desc(has_bias=True, has_sum=False, sum_t=U8, with_relu=False, scale_count=1) -> FusedDesc:
    f = FusedDesc()
    f.has_bias, f.has_sum, f.sum_t = int(has_bias), int(has_sum), dtype_code(sum_t)
    f.with_relu, f.scale_count = int(with_relu), int(scale_count)
    return f


def make_pool_desc(op, dtype, N, Cc, in_sp, window, stride=None, pad_below=None, pad_above=None, include_padding=False, layout=NCX) -> PoolDesc:
    """out_sp follows the reference's rule (src/ngraph/validation_util.cpp, infer_batched_pooling_forward)"""
    ns = len(in_sp)
    d = PoolDesc()
    d.op = POOL_AVG if op in (POOL_AVG, "avg") else POOL_MAX
    d.dtype, d.layout, d.n_spatial, d.include_padding = dtype_code(dtype), layout, ns, int(include_padding)
    d.N, d.C = N, Cc
    stride = stride or [1] * ns
    pad_below = pad_below or [0] * ns
    pad_above = pad_above or [0] * ns
    for i in range(ns):
        d.in_sp[i], d.window[i], d.stride[i], d.pad_below[i], d.pad_above[i] = in_sp[i], window[i], stride[i], pad_below[i], pad_above[i]
        d.out_sp[i] = (in_sp[i] + pad_below[i] + pad_above[i] - window[i]) // stride[i] + 1
    return d


def make_dot_desc(M, K, N, a_t=U8, b_t=I8, out_t=I8, b_layout=B_KN) -> DotDesc:
    d = DotDesc()
    d.a_t, d.b_t, d.out_t, d.b_layout = dtype_code(a_t), dtype_code(b_t), dtype_code(out_t), b_layout
    d.M, d.K, d.N = M, K, N
    return d


EXPORTS = [
    "hipq_last_error",
    "hipq_version",
    "hipq_device_count",
    "hipq_set_device",
    "hipq_get_device_info",
    "hipq_malloc",
    "hipq_free",
    "hipq_memcpy_h2d",
    "hipq_memcpy_d2h",
    "hipq_memcpy_d2d",
    "hipq_fill_bytes",
    "hipq_stream_create",
    "hipq_stream_destroy",
    "hipq_stream_release_scratch",
    "hipq_stream_sync",
    "hipq_capture_begin",
    "hipq_capture_end",
    "hipq_graph_launch",
    "hipq_graph_destroy",
    "hipq_workspace_epoch",
    "hipq_event_create",
    "hipq_event_destroy",
    "hipq_event_record",
    "hipq_event_sync",
    "hipq_event_elapsed_ms",
    "hipq_quantize",
    "hipq_dequantize",
    "hipq_conv_infer_output",
    "hipq_conv_packed_filter_bytes",
    "hipq_conv_pack_filter",
    "hipq_quantized_convolution",
    "hipq_quantized_convolution_noalloc",
    "hipq_quantized_convolution_fused",
    "hipq_conv_max_pool_fusable",
    "hipq_quantized_convolution_fused_max_pool",
    "hipq_dot_packed_bytes",
    "hipq_dot_pack",
    "hipq_quantized_dot",
    "hipq_quantized_dot_bias",
    "hipq_quantized_dot_bias_gelu_quantize",
    "hipq_transpose_ncx_to_nxc",
    "hipq_transpose_nxc_to_ncx",
    "hipq_binary",
    "hipq_unary",
    "hipq_convert",
    "hipq_broadcast",
    "hipq_permute",
    "hipq_slice",
    "hipq_pool_infer_output",
    "hipq_pool",
    "hipq_concat",
    "hipq_last_kernel",
    "hipq_softmax_f32",
    "hipq_erf_f32",
    "hipq_gelu_f32",
    "hipq_layer_norm_f32",
    "hipq_batch_matmul_f32",
    "hipq_softmax_scaled_f32",
    "hipq_gelu_quantize_f32",
    "hipq_add_layer_norm_f32",
    "hipq_batch_matmul_view_f32",
    "hipq_attention_f32",
]

_lib = None


class HipqError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"hipq error {code}: {msg}")
        self.code = code


PROBE_LIB_PATH = os.path.join(os.path.dirname(LIB_PATH), "libhipq_probe.so")
_probe = None


def load_probe():
    """dlopen libhipq_probe.so, the measurement aids (ngraph_amd/csrc/probe/hipq_probe.h): bench.py's
    device ceilings and the host-side index-division check.  Not part of the product library."""
    global _probe
    if _probe is not None:
        return _probe
    if not os.path.exists(PROBE_LIB_PATH):
        raise RuntimeError(f"{PROBE_LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')")
    lib = C.CDLL(PROBE_LIB_PATH)
    vp, i32, sz = C.c_void_p, C.c_int32, C.c_size_t
    lib.hipq_probe_last_error.restype = C.c_char_p
    lib.hipq_probe_mfma_i8.argtypes = [vp, vp, i32, i32, vp]
    lib.hipq_probe_coissue.argtypes = [vp, vp, i32, i32, i32, i32, vp]
    lib.hipq_probe_intake.argtypes = [vp, sz, sz, i32, i32, i32, i32, i32, i32, vp, vp]
    lib.hipq_probe_atomic_tiles.argtypes = [vp, sz, i32, i32, i32, i32, vp]
    lib.hipq_probe_empty_chain.argtypes = [vp, i32, i32, i32, vp]
    lib.hipq_debug_fastdiv.restype = C.c_uint32
    lib.hipq_debug_fastdiv.argtypes = [C.c_uint32] * 2
    _probe = lib
    return lib


def check_probe(rc):
    if rc:
        raise RuntimeError("libhipq_probe: " + load_probe().hipq_probe_last_error().decode())


def load():
    """dlopen libhipq.so (built by __graft_entry__.build()); raises if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP library first (python -c 'import __graft_entry__ as g; g.build()')"
        )
    lib = C.CDLL(LIB_PATH)
    vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int32
    lib.hipq_last_error.restype = C.c_char_p
    lib.hipq_last_kernel.restype = C.c_char_p
    lib.hipq_conv_packed_filter_bytes.restype = C.c_size_t
    lib.hipq_conv_packed_filter_bytes.argtypes = [C.POINTER(ConvDesc)]
    lib.hipq_device_count.argtypes = [C.POINTER(C.c_int)]
    lib.hipq_set_device.argtypes = [C.c_int]
    lib.hipq_get_device_info.argtypes = [C.POINTER(DeviceInfo)]
    lib.hipq_malloc.argtypes = [C.POINTER(vp), C.c_size_t]
    lib.hipq_free.argtypes = [vp]
    for n in ("hipq_memcpy_h2d", "hipq_memcpy_d2h", "hipq_memcpy_d2d"):
        getattr(lib, n).argtypes = [vp, vp, C.c_size_t, vp]
    lib.hipq_fill_bytes.argtypes = [vp, C.c_int, C.c_size_t, vp]
    lib.hipq_stream_create.argtypes = [C.POINTER(vp)]
    lib.hipq_stream_destroy.argtypes = [vp]
    lib.hipq_stream_release_scratch.argtypes = [vp]
    lib.hipq_stream_sync.argtypes = [vp]
    lib.hipq_event_create.argtypes = [C.POINTER(vp)]
    lib.hipq_event_destroy.argtypes = [vp]
    lib.hipq_event_record.argtypes = [vp, vp]
    lib.hipq_event_sync.argtypes = [vp]
    lib.hipq_event_elapsed_ms.argtypes = [vp, vp, C.POINTER(C.c_float)]
    lib.hipq_quantize.argtypes = [C.POINTER(QuantDesc), vp, vp, vp, vp, vp]
    lib.hipq_dequantize.argtypes = [C.POINTER(QuantDesc), vp, vp, vp, vp, vp]
    lib.hipq_conv_infer_output.argtypes = [C.POINTER(ConvDesc)]
    lib.hipq_conv_pack_filter.argtypes = [C.POINTER(ConvDesc), vp, vp, vp]
    lib.hipq_quantized_convolution.argtypes = [C.POINTER(ConvDesc)] + [vp] * 11
    lib.hipq_quantized_convolution_noalloc.argtypes = [C.POINTER(ConvDesc)] + [vp] * 11
    lib.hipq_quantized_convolution_fused.argtypes = [C.POINTER(ConvDesc), C.POINTER(FusedDesc)] + [vp] * 9
    lib.hipq_conv_max_pool_fusable.argtypes = [C.POINTER(ConvDesc), C.POINTER(FusedDesc), C.POINTER(PoolDesc)]
    lib.hipq_quantized_convolution_fused_max_pool.argtypes = [C.POINTER(ConvDesc), C.POINTER(FusedDesc), C.POINTER(PoolDesc)] + [vp] * 6
    lib.hipq_dot_packed_bytes.restype = C.c_size_t
    lib.hipq_dot_packed_bytes.argtypes = [C.POINTER(DotDesc)]
    lib.hipq_dot_pack.argtypes = [C.POINTER(DotDesc), vp, vp, vp]
    lib.hipq_quantized_dot.argtypes = [C.POINTER(DotDesc)] + [vp] * 11
    lib.hipq_quantized_dot_bias.argtypes = [C.POINTER(DotDesc), C.POINTER(FusedDesc)] + [vp] * 7
    for n in ("hipq_transpose_ncx_to_nxc", "hipq_transpose_nxc_to_ncx"):
        getattr(lib, n).argtypes = [vp, vp, i64, i64, i64, i32, vp]
    lib.hipq_capture_begin.argtypes = [vp]
    lib.hipq_capture_end.argtypes = [vp, C.POINTER(vp)]
    lib.hipq_graph_launch.argtypes = [vp, vp]
    lib.hipq_graph_destroy.argtypes = [vp]
    lib.hipq_workspace_epoch.argtypes = []
    lib.hipq_workspace_epoch.restype = C.c_uint64
    lib.hipq_binary.argtypes = [i32, i32, vp, i64, vp, i64, vp, i64, vp]
    lib.hipq_unary.argtypes = [i32, i32, vp, vp, i64, vp]
    lib.hipq_convert.argtypes = [i32, i32, vp, vp, i64, vp]
    lib.hipq_broadcast.argtypes = [i32, vp, vp, i32, C.POINTER(C.c_int64), C.c_uint32, vp]
    lib.hipq_permute.argtypes = [i32, vp, vp, i32, C.POINTER(C.c_int64), C.POINTER(C.c_int32), vp]
    lib.hipq_pool_infer_output.argtypes = [C.POINTER(PoolDesc)]
    lib.hipq_pool.argtypes = [C.POINTER(PoolDesc), vp, vp, vp]
    lib.hipq_concat.argtypes = [i32, i32, C.POINTER(vp), C.POINTER(C.c_int64), i64, i64, vp, vp]
    _lib = lib
    return lib


def check(rc):
    if rc != OK:
        raise HipqError(rc, load().hipq_last_error().decode())


def last_kernel() -> str:
    return load().hipq_last_kernel().decode()


class DeviceBuffer:
    """Device allocation owned through hipq_malloc / hipq_free."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(load().hipq_malloc(C.byref(p), max(self.nbytes, 1)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        if a.nbytes:
            check(load().hipq_memcpy_h2d(b.ptr, a.ctypes.data, a.nbytes, None))
        return b

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(load().hipq_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes, None))
        return out

    def free(self):
        if self.ptr:
            load().hipq_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _dev(x):
    """numpy array / scalar -> DeviceBuffer (None stays None)."""
    if x is None:
        return None
    return DeviceBuffer.from_numpy(np.asarray(x))


def _p(b):
    return None if b is None else b.ptr


# ---- numpy-in / numpy-out conveniences (one call = upload, launch, sync, download) ----------


def quantize(x, scale, zp, quant_t, axes=(), round_mode=RNE):
    x = np.ascontiguousarray(x)
    qt = dtype_code(quant_t)
    d = make_quant_desc(x.shape, axes, x.dtype, qt, round_mode)
    bx, bs, bz = _dev(x), _dev(np.asarray(scale, dtype=x.dtype)), _dev(np.asarray(zp, dtype=NP_OF[qt]))
    out = DeviceBuffer(x.size * np.dtype(NP_OF[qt]).itemsize)
    check(load().hipq_quantize(C.byref(d), bx.ptr, bs.ptr, bz.ptr, out.ptr, None))
    check(load().hipq_stream_sync(None))
    return out.to_numpy(NP_OF[qt], x.shape)


def dequantize(q, scale, zp, real_t=F32, axes=()):
    q = np.ascontiguousarray(q)
    rt = dtype_code(real_t)
    d = make_quant_desc(q.shape, axes, rt, q.dtype)
    bq, bs, bz = _dev(q), _dev(np.asarray(scale, dtype=NP_OF[rt])), _dev(np.asarray(zp, dtype=q.dtype))
    out = DeviceBuffer(q.size * np.dtype(NP_OF[rt]).itemsize)
    check(load().hipq_dequantize(C.byref(d), bq.ptr, bs.ptr, bz.ptr, out.ptr, None))
    check(load().hipq_stream_sync(None))
    return out.to_numpy(NP_OF[rt], q.shape)


def pack_filter(desc: ConvDesc, filter_dev: DeviceBuffer):
    """Returns the packed-filter DeviceBuffer, or None when the MFMA path does not apply."""
    n = load().hipq_conv_packed_filter_bytes(C.byref(desc))
    if n == 0:
        return None
    packed = DeviceBuffer(n)
    check(load().hipq_conv_pack_filter(C.byref(desc), filter_dev.ptr, packed.ptr, None))
    return packed


def pack_dot(desc: DotDesc, b_dev: DeviceBuffer):
    """Returns the packed second operand, or None when the MFMA path does not apply."""
    n = load().hipq_dot_packed_bytes(C.byref(desc))
    if n == 0:
        return None
    packed = DeviceBuffer(n)
    check(load().hipq_dot_pack(C.byref(desc), b_dev.ptr, packed.ptr, None))
    return packed


def quantized_convolution(desc, data, filt, data_scale, data_zp, filter_scale, filter_zp, out_scale, out_zp, use_packed=True, noalloc=False):
    """noalloc=True goes through the entry point that takes its scratch from the library's fixed array"""
    lib = load()
    bd, bf = _dev(data), _dev(filt)
    packed = pack_filter(desc, bf) if use_packed else None
    s = [_dev(np.float32(v)) for v in (data_scale, filter_scale, out_scale)]
    z = [
        _dev(np.asarray(data_zp, dtype=NP_OF[desc.data_t])),
        _dev(np.asarray(filter_zp, dtype=NP_OF[desc.filter_t])),
        _dev(np.asarray(out_zp, dtype=NP_OF[desc.out_t])),
    ]
    oshape = desc.out_shape()
    out = DeviceBuffer(int(np.prod(oshape)) * np.dtype(NP_OF[desc.out_t]).itemsize)
    entry = lib.hipq_quantized_convolution_noalloc if noalloc else lib.hipq_quantized_convolution
    check(entry(C.byref(desc), bd.ptr, bf.ptr, _p(packed), s[0].ptr, z[0].ptr, s[1].ptr, z[1].ptr, s[2].ptr, z[2].ptr, out.ptr, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(NP_OF[desc.out_t], oshape)


def quantized_convolution_fused(desc, fused, data, filt, bias, sum_in, scale, sum_scale, use_packed=True):
    lib = load()
    bd, bf = _dev(data), _dev(filt)
    packed = pack_filter(desc, bf) if use_packed else None
    bb = _dev(None if bias is None else np.asarray(bias, dtype=np.int32))
    bsc = _dev(np.asarray(scale, dtype=np.float32))
    bss = _dev(None if sum_scale is None else np.float32(sum_scale))
    oshape = desc.out_shape()
    nbytes = int(np.prod(oshape)) * np.dtype(NP_OF[desc.out_t]).itemsize
    out = DeviceBuffer(nbytes)
    bsum = _dev(sum_in)
    check(
        lib.hipq_quantized_convolution_fused(
            C.byref(desc), C.byref(fused), bd.ptr, bf.ptr, _p(packed), _p(bb), _p(bsum), bsc.ptr, _p(bss), out.ptr, None
        )
    )
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(NP_OF[desc.out_t], oshape)


def conv_max_pool_fusable(desc, fused, pool_desc) -> bool:
    return bool(load().hipq_conv_max_pool_fusable(C.byref(desc), C.byref(fused), C.byref(pool_desc)))


def quantized_convolution_fused_max_pool(desc, fused, pool_desc, data, filt, bias, scale):
    """MaxPool(fused convolution) in one launch; raises HipqError (UNSUPPORTED) for pairs without a fused kernel"""
    lib = load()
    bd, bf = _dev(data), _dev(filt)
    packed = pack_filter(desc, bf)
    bb = _dev(None if bias is None else np.asarray(bias, dtype=np.int32))
    bsc = _dev(np.asarray(scale, dtype=np.float32))
    oshape = pool_desc.out_shape()
    out = DeviceBuffer(int(np.prod(oshape)) * np.dtype(NP_OF[desc.out_t]).itemsize)
    check(lib.hipq_quantized_convolution_fused_max_pool(C.byref(desc), C.byref(fused), C.byref(pool_desc), bd.ptr, _p(packed), _p(bb), bsc.ptr, out.ptr, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(NP_OF[desc.out_t], oshape)


def pool(desc, x):
    lib = load()
    bx = _dev(np.ascontiguousarray(x))
    oshape = desc.out_shape()
    out = DeviceBuffer(int(np.prod(oshape)) * x.dtype.itemsize)
    check(lib.hipq_pool(C.byref(desc), bx.ptr, out.ptr, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(x.dtype, oshape)


def concat(arrays, axis):
    lib = load()
    arrays = [np.ascontiguousarray(a) for a in arrays]
    bufs = [_dev(a) for a in arrays]
    shape = list(arrays[0].shape)
    outer = int(np.prod(shape[:axis]))
    inner = int(np.prod(shape[axis + 1 :]))
    extents = [a.shape[axis] for a in arrays]
    shape[axis] = sum(extents)
    out = DeviceBuffer(int(np.prod(shape)) * arrays[0].dtype.itemsize)
    ptrs = (C.c_void_p * len(bufs))(*[b.ptr for b in bufs])
    ext = (C.c_int64 * len(bufs))(*extents)
    check(lib.hipq_concat(arrays[0].dtype.itemsize, len(bufs), ptrs, ext, outer, inner, out.ptr, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(arrays[0].dtype, shape)


class GraphReplay:
    """One fixed launch sequence on a stream, captured into a HIP graph and replayed.

    `launch` issues the sequence on `stream`.  The graph points into the library's scratch blocks:
    it is captured again whenever hipq_workspace_epoch says a block of the device was reallocated
    since the capture, and destroyed by close() (or when the object goes away)."""

    def __init__(self, lib, stream, launch):
        self.lib, self.stream, self._launch = lib, stream, launch
        self.graph = None
        self.epoch = None

    def capture(self):
        self.close()
        self._launch()  # sizes the library's scratch blocks before anything is recorded
        check(self.lib.hipq_stream_sync(self.stream))
        check(self.lib.hipq_capture_begin(self.stream))
        g = C.c_void_p()
        try:
            self._launch()
        except Exception:
            self.lib.hipq_capture_end(self.stream, C.byref(g))  # leave the stream usable
            if g.value:
                self.lib.hipq_graph_destroy(g)
            raise
        check(self.lib.hipq_capture_end(self.stream, C.byref(g)))
        self.graph = g
        self.epoch = self.lib.hipq_workspace_epoch()

    def replay(self):
        if self.graph is None or self.lib.hipq_workspace_epoch() != self.epoch:
            self.capture()
        rc = self.lib.hipq_graph_launch(self.graph, self.stream)
        if rc:
            check(rc)

    def close(self):
        if self.graph is not None:
            g, self.graph = self.graph, None
            check(self.lib.hipq_stream_sync(self.stream))
            check(self.lib.hipq_graph_destroy(g))

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


BINARY_OPS = {"add": 0, "subtract": 1, "multiply": 2, "divide": 3, "maximum": 4, "minimum": 5, "divide_floor": 6}
UNARY_OPS = {"abs": 0, "relu": 1, "copy": 2}


def binary(op, a, b):
    """elementwise a (op) b; either side may be a single element"""
    lib = load()
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    big = a if a.size >= b.size else b
    ba, bb = _dev(a), _dev(b)
    out = DeviceBuffer(big.nbytes)
    check(lib.hipq_binary(BINARY_OPS[op], dtype_code(a.dtype), ba.ptr, a.size, bb.ptr, b.size, out.ptr, big.size, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(a.dtype, big.shape)


def unary(op, x):
    lib = load()
    x = np.ascontiguousarray(x)
    bx = _dev(x)
    out = DeviceBuffer(x.nbytes)
    check(lib.hipq_unary(UNARY_OPS[op], dtype_code(x.dtype), bx.ptr, out.ptr, x.size, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(x.dtype, x.shape)


def convert(x, out_dtype):
    lib = load()
    x = np.ascontiguousarray(x)
    out_dtype = np.dtype(out_dtype)
    bx = _dev(x)
    out = DeviceBuffer(x.size * out_dtype.itemsize)
    check(lib.hipq_convert(dtype_code(x.dtype), dtype_code(out_dtype), bx.ptr, out.ptr, x.size, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(out_dtype, x.shape)


def permute(x, order):
    """out = x with axes read in `order` (numpy's transpose(order), made contiguous)"""
    lib = load()
    x = np.ascontiguousarray(x)
    bx = _dev(x)
    out = DeviceBuffer(x.nbytes)
    shape = (C.c_int64 * x.ndim)(*x.shape)
    ordr = (C.c_int32 * x.ndim)(*order)
    check(lib.hipq_permute(x.dtype.itemsize, bx.ptr, out.ptr, x.ndim, shape, ordr, None))
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(x.dtype, [x.shape[i] for i in order])


def slice_(x, lower, upper, strides=None):
    """x[lower:upper:strides] along every axis (op::v0::Slice)"""
    lib = load()
    x = np.ascontiguousarray(x)
    strides = list(strides) if strides is not None else [1] * x.ndim
    bx = _dev(x)
    out = DeviceBuffer(max(x.nbytes, 1))  # (a slice is never larger than its input)
    i64 = C.c_int64 * x.ndim
    lib.hipq_slice.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_int32] + [C.c_void_p] * 5
    check(lib.hipq_slice(x.dtype.itemsize, bx.ptr, out.ptr, x.ndim, i64(*x.shape), i64(*lower), i64(*upper), i64(*strides), None))
    check(lib.hipq_stream_sync(None))
    out_shape = [(u - l + s - 1) // s for l, u, s in zip(lower, upper, strides)]
    return out.to_numpy(x.dtype, out_shape)


def quantized_dot(desc, a, b, a_scale, a_zp, b_scale, b_zp, out_scale, out_zp, prepare=True):
    lib = load()
    ba, bb = _dev(a), _dev(b)
    bsum = pack_dot(desc, bb) if prepare else None
    s = [_dev(np.float32(v)) for v in (a_scale, b_scale, out_scale)]
    z = [
        _dev(np.asarray(a_zp, dtype=NP_OF[desc.a_t])),
        _dev(np.asarray(b_zp, dtype=NP_OF[desc.b_t])),
        _dev(np.asarray(out_zp, dtype=NP_OF[desc.out_t])),
    ]
    out = DeviceBuffer(int(desc.M * desc.N) * np.dtype(NP_OF[desc.out_t]).itemsize)
    check(
        lib.hipq_quantized_dot(
            C.byref(desc), ba.ptr, bb.ptr, _p(bsum), s[0].ptr, z[0].ptr, s[1].ptr, z[1].ptr, s[2].ptr, z[2].ptr, out.ptr, None
        )
    )
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(NP_OF[desc.out_t], (int(desc.M), int(desc.N)))


def quantized_dot_bias(desc, fused, a, w, bias, scale, prepare=True):
    lib = load()
    ba, bw = _dev(a), _dev(w)
    wsum = pack_dot(desc, bw) if prepare else None
    bb = _dev(None if bias is None else np.asarray(bias, dtype=np.int32))
    bsc = _dev(np.asarray(scale, dtype=np.float32))
    out = DeviceBuffer(int(desc.M * desc.N) * np.dtype(NP_OF[desc.out_t]).itemsize)
    check(
        lib.hipq_quantized_dot_bias(C.byref(desc), C.byref(fused), ba.ptr, bw.ptr, _p(wsum), _p(bb), bsc.ptr, out.ptr, None)
    )
    check(lib.hipq_stream_sync(None))
    return out.to_numpy(NP_OF[desc.out_t], (int(desc.M), int(desc.N)))


def quantized_dot_bias_gelu_quantize(desc, fused, a, w, bias, scale, q_scale, q_zp=0, quant_t="i8", round_mode=RNE, prepare=True):
    """Quantize(Gelu(QuantizedDotBias(...) as f32)) through hipq_quantized_dot_bias_gelu_quantize: the [M, N] bytes"""
    lib = load()
    ba, bw = _dev(a), _dev(w)
    wsum = pack_dot(desc, bw) if prepare else None
    bb = _dev(None if bias is None else np.asarray(bias, dtype=np.int32))
    bsc = _dev(np.asarray(scale, dtype=np.float32))
    q, keep, qt = _quant_out(int(desc.M * desc.N), q_scale, q_zp, quant_t, round_mode)
    lib.hipq_quantized_dot_bias_gelu_quantize.argtypes = [C.c_void_p] * 9
    check(lib.hipq_quantized_dot_bias_gelu_quantize(C.byref(desc), C.byref(fused), ba.ptr, bw.ptr, _p(wsum), _p(bb), bsc.ptr, C.byref(q), None))
    check(lib.hipq_stream_sync(None))
    return keep[0].to_numpy(NP_OF[qt], (int(desc.M), int(desc.N)))


# ---- fp32 glue of a transformer encoder -----------------------------------------------------------

def _axes_run(shape, axes):
    """(outer, axis, inner) of a contiguous run of axes (all axes when `axes` is empty, as op::v0::Softmax reads it)"""
    rank = len(shape)
    axes = sorted(set(range(rank)) if len(axes) == 0 else set(axes))
    if axes != list(range(axes[0], axes[-1] + 1)):
        raise ValueError("the library takes a contiguous run of axes")
    outer = int(np.prod(shape[: axes[0]], dtype=np.int64))
    axis = int(np.prod(shape[axes[0] : axes[-1] + 1], dtype=np.int64))
    inner = int(np.prod(shape[axes[-1] + 1 :], dtype=np.int64))
    return outer, axis, inner


def softmax(x, axes=()):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    outer, axis, inner = _axes_run(x.shape, axes)
    src, dst = _dev(x), DeviceBuffer(max(x.nbytes, 4))
    lib.hipq_softmax_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]
    check(lib.hipq_softmax_f32(src.ptr, dst.ptr, outer, axis, inner, None))
    check(lib.hipq_stream_sync(None))
    return dst.to_numpy(np.float32, x.shape)


def _unary_f32(name, x):
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    src, dst = _dev(x), DeviceBuffer(max(x.nbytes, 4))
    fn = getattr(lib, name)
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    check(fn(src.ptr, dst.ptr, x.size, None))
    check(lib.hipq_stream_sync(None))
    return dst.to_numpy(np.float32, x.shape)


def erf(x):
    return _unary_f32("hipq_erf_f32", x)


def gelu(x):
    return _unary_f32("hipq_gelu_f32", x)


def layer_norm(x, scale=None, bias=None, begin_norm_axis=1, epsilon=1e-5, keep_stats=True):
    """op::v0::LayerNorm forward: returns (norm, mean, var), mean and var None without keep_stats"""
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    n_axis = begin_norm_axis if begin_norm_axis >= 0 else x.ndim + begin_norm_axis
    rows = int(np.prod(x.shape[:n_axis], dtype=np.int64))
    cols = int(np.prod(x.shape[n_axis:], dtype=np.int64))
    src, dst = _dev(x), DeviceBuffer(max(x.nbytes, 4))
    sc = _dev(np.ascontiguousarray(scale, dtype=np.float32)) if scale is not None else None
    bi = _dev(np.ascontiguousarray(bias, dtype=np.float32)) if bias is not None else None
    mean = DeviceBuffer(max(rows, 1) * 4) if keep_stats else None
    var = DeviceBuffer(max(rows, 1) * 4) if keep_stats else None
    lib.hipq_layer_norm_f32.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int64, C.c_double, C.c_void_p]
    check(lib.hipq_layer_norm_f32(src.ptr, sc.ptr if sc else None, bi.ptr if bi else None, dst.ptr, mean.ptr if mean else None, var.ptr if var else None, rows, cols, float(epsilon), None))
    check(lib.hipq_stream_sync(None))
    stats_shape = x.shape[:n_axis]
    return (dst.to_numpy(np.float32, x.shape), mean.to_numpy(np.float32, stats_shape) if keep_stats else None, var.to_numpy(np.float32, stats_shape) if keep_stats else None)


def batch_matmul(a, b, transpose_a=False, transpose_b=False):
    """out[i] = op(a[i]) @ op(b[i]) for f32 [batch, ., .] operands (two matrices: a batch of one)"""
    lib = load()
    a, b = np.ascontiguousarray(a, dtype=np.float32), np.ascontiguousarray(b, dtype=np.float32)
    squeeze = a.ndim == 2
    if squeeze:
        a, b = a[None], b[None]
    batch = a.shape[0]
    M, K = (a.shape[2], a.shape[1]) if transpose_a else (a.shape[1], a.shape[2])
    N = b.shape[1] if transpose_b else b.shape[2]
    assert (b.shape[2] if transpose_b else b.shape[1]) == K and b.shape[0] == batch
    da, db = _dev(a) if a.size else None, _dev(b) if b.size else None
    out = DeviceBuffer(max(batch * M * N * 4, 4))
    lib.hipq_batch_matmul_f32.argtypes = [C.c_void_p] * 3 + [C.c_int64] * 4 + [C.c_int32] * 2 + [C.c_void_p]
    check(lib.hipq_batch_matmul_f32(da.ptr if da else None, db.ptr if db else None, out.ptr, batch, M, K, N, int(transpose_a), int(transpose_b), None))
    check(lib.hipq_stream_sync(None))
    r = out.to_numpy(np.float32, (batch, M, N))
    return r[0] if squeeze else r


# ---- fused forms: each equals the op-by-op sequence it replaces bit for bit


def _quant_out(n, scale, zp, quant_t, round_mode):
    qt = dtype_code(quant_t)
    out = DeviceBuffer(max(n, 4))
    bs, bz = _dev(np.asarray(scale, dtype=np.float32)), _dev(np.asarray(zp, dtype=NP_OF[qt]))
    return QuantOut(out.ptr, bs.ptr, bz.ptr, qt, round_mode), (out, bs, bz), qt


def softmax_scaled(x, factor):
    """Softmax(x * factor) over the last axis in one launch"""
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    src, dst, fac = _dev(x), DeviceBuffer(max(x.nbytes, 4)), _dev(np.asarray(factor, dtype=np.float32))
    lib.hipq_softmax_scaled_f32.argtypes = [C.c_void_p] * 3 + [C.c_int64] * 3 + [C.c_void_p]
    check(lib.hipq_softmax_scaled_f32(src.ptr, fac.ptr, dst.ptr, int(np.prod(x.shape[:-1], dtype=np.int64)), x.shape[-1], 1, None))
    check(lib.hipq_stream_sync(None))
    return dst.to_numpy(np.float32, x.shape)


def add_layer_norm(a, b, scale, bias, epsilon=1e-5, q_scale=None, q_zp=0, quant_t="i8", round_mode=RNE):
    """LayerNorm(a + b) over the last axis (b may be None); with q_scale also Quantize of the result: returns (norm, q or None)"""
    lib = load()
    a = np.ascontiguousarray(a, dtype=np.float32)
    rows, cols = int(np.prod(a.shape[:-1], dtype=np.int64)), a.shape[-1]
    ba, bb = _dev(a), (_dev(np.ascontiguousarray(b, dtype=np.float32)) if b is not None else None)
    sc, bi = _dev(np.ascontiguousarray(scale, dtype=np.float32)), _dev(np.ascontiguousarray(bias, dtype=np.float32))
    dst = DeviceBuffer(max(a.nbytes, 4))
    q = keep = qt = None
    if q_scale is not None:
        q, keep, qt = _quant_out(a.size, q_scale, q_zp, quant_t, round_mode)
    lib.hipq_add_layer_norm_f32.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int64, C.c_double, C.c_void_p]
    check(lib.hipq_add_layer_norm_f32(ba.ptr, bb.ptr if bb else None, sc.ptr, bi.ptr, dst.ptr, C.byref(q) if q else None, rows, cols, float(epsilon), None))
    check(lib.hipq_stream_sync(None))
    return dst.to_numpy(np.float32, a.shape), (keep[0].to_numpy(NP_OF[qt], a.shape) if q else None)


def gelu_quantize(x, q_scale, q_zp=0, quant_t="i8", round_mode=RNE, keep_f32=True):
    """Gelu(x) and Quantize(Gelu(x)) in one launch: returns (gelu or None, q)"""
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    src = _dev(x)
    dst = DeviceBuffer(max(x.nbytes, 4)) if keep_f32 else None
    q, keep, qt = _quant_out(x.size, q_scale, q_zp, quant_t, round_mode)
    lib.hipq_gelu_quantize_f32.argtypes = [C.c_void_p] * 3 + [C.c_int64, C.c_void_p]
    check(lib.hipq_gelu_quantize_f32(src.ptr, dst.ptr if dst else None, C.byref(q), x.size, None))
    check(lib.hipq_stream_sync(None))
    return (dst.to_numpy(np.float32, x.shape) if dst else None), keep[0].to_numpy(NP_OF[qt], x.shape)


def attention(qkv, q_off, k_off, v_off, out_elems, view, batch, queries, keys, depth, factor=None, q_scale=None, q_zp=0, quant_t="i8", keep_f32=True):
    """hipq_attention_f32 on one flat f32 buffer holding Q, K and V (element offsets) into a flat zero-initialised
    output of out_elems elements: returns (out or None, q or None); raises HipqError (UNSUPPORTED) for shapes the
    one-kernel form does not take"""
    lib = load()
    buf = _dev(np.ascontiguousarray(qkv, dtype=np.float32).ravel())
    dst = DeviceBuffer.from_numpy(np.zeros(out_elems, np.float32)) if keep_f32 else None
    fac = _dev(np.asarray([factor], dtype=np.float32)) if factor is not None else None
    q = keep = qt = None
    if q_scale is not None:
        q, keep, qt = _quant_out(out_elems, q_scale, q_zp, quant_t, RNE)
        check(lib.hipq_fill_bytes(keep[0].ptr, 0, out_elems, None))
    lib.hipq_attention_f32.argtypes = [C.c_void_p] * 7 + [C.c_int64] * 4 + [C.c_void_p]
    check(lib.hipq_attention_f32(buf.ptr + 4 * q_off, buf.ptr + 4 * k_off, buf.ptr + 4 * v_off, fac.ptr if fac else None, dst.ptr if dst else None, C.byref(view),
                                 C.byref(q) if q else None, batch, queries, keys, depth, None))
    check(lib.hipq_stream_sync(None))
    return (dst.to_numpy(np.float32, (out_elems,)) if dst else None), (keep[0].to_numpy(NP_OF[qt], (out_elems,)) if q else None)


def batch_matmul_view(a, a_off, b, b_off, out_elems, out_off, view, batch, M, K, N, transpose_a=False, transpose_b=False, q_scale=None, q_zp=0, quant_t="i8", keep_f32=True):
    """hipq_batch_matmul_view_f32 on flat f32 buffers a and b (element offsets a_off, b_off) into a flat
    zero-initialised output of out_elems elements: returns (out or None, q or None)"""
    lib = load()
    a, b = np.ascontiguousarray(a, dtype=np.float32).ravel(), np.ascontiguousarray(b, dtype=np.float32).ravel()
    ba, bb = _dev(a), _dev(b)
    dst = DeviceBuffer.from_numpy(np.zeros(out_elems, np.float32)) if keep_f32 else None
    q = keep = qt = None
    if q_scale is not None:
        q, keep, qt = _quant_out(out_elems, q_scale, q_zp, quant_t, RNE)
        check(lib.hipq_fill_bytes(keep[0].ptr, 0, out_elems, None))
    lib.hipq_batch_matmul_view_f32.argtypes = [C.c_void_p] * 5 + [C.c_int64] * 4 + [C.c_int32] * 2 + [C.c_void_p]
    check(lib.hipq_batch_matmul_view_f32(ba.ptr + 4 * a_off, bb.ptr + 4 * b_off, (dst.ptr + 4 * out_off) if dst else None, C.byref(view), C.byref(q) if q else None, batch, M, K, N,
                                         1 if transpose_a else 0, 1 if transpose_b else 0, None))
    check(lib.hipq_stream_sync(None))
    return (dst.to_numpy(np.float32, (out_elems,)) if dst else None), (keep[0].to_numpy(NP_OF[qt], (out_elems,)) if q else None)
