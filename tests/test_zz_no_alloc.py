"""hipq_quantized_convolution_noalloc: the convolution entry point that takes its scratch from a
fixed per-device array instead of allocating.  Its outputs must be the regular entry point's bit
for bit -- on calls that need a layout copy of an NCX input, a first layer's padded copy, and
partial sums of a split reduction -- on two calls in a row, the second smaller (the array still
holds the first call's bytes), and a call beyond the array's size must be refused with nothing
launched."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O
from ngraph_amd import hipq as H
from ngraph_amd import synth


def say(*a):
    print("[case]", *a, flush=True)


def _pair(d, seed, out_scale=1.0, data_zp=0):
    data = synth.uniform_int(seed, d.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(seed + 1, d.filter_shape(), -127, 127, np.int8)
    args = (d, data, filt, 0.02, data_zp, 0.005, 0, out_scale, 0)
    regular = H.quantized_convolution(*args)
    k_regular = H.last_kernel()
    noalloc = H.quantized_convolution(*args, noalloc=True)
    assert H.last_kernel() == k_regular
    return regular, noalloc, k_regular, args


@pytest.mark.gpu
def test_noalloc_layout_copy_two_calls(gpu_lib, monkeypatch):
    """NCX in (the reference's layout): the channels-last copy lives in the scratch array (the kernel
    that reads NCHW itself is switched off for this test: it needs no scratch)"""
    monkeypatch.setenv("HIPQ_NO_REGW", "1")
    for N in (8, 3):  # the second call is smaller
        say("noalloc NCX conv, N", N)
        d = H.make_conv_desc(N, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
        regular, noalloc, kernel, args = _pair(d, 3100 + N, out_scale=0.1)
        assert kernel.startswith("conv_band"), kernel
        assert np.array_equal(noalloc, regular)
        if N == 3:
            O.port().orc_set_threads(8)
            assert np.array_equal(noalloc, O.quantized_convolution(*args))
            O.port().orc_set_threads(1)


@pytest.mark.gpu
def test_noalloc_generic_conv_and_first_layer(gpu_lib):
    """a strided 3x3 over 128 channels (generic tile kernels behind the transposition) with a
    non-zero data zero point, then a 3-channel 7x7 stem (padded / row-packed copy in the scratch)"""
    for N in (4, 1):
        say("noalloc strided conv, N", N)
        d = H.make_conv_desc(N, 128, 192, (28, 28), (3, 3), stride=(2, 2), pad_below=(1, 1), pad_above=(1, 1))
        regular, noalloc, kernel, _ = _pair(d, 3200 + N, out_scale=0.2, data_zp=7)
        assert kernel.startswith("conv_mfma"), kernel
        assert np.array_equal(noalloc, regular)
    for N in (2, 1):
        say("noalloc stem, N", N)
        d = H.make_conv_desc(N, 3, 64, (224, 224), (7, 7), stride=(2, 2), pad_below=(3, 3), pad_above=(3, 3), out_layout=H.NXC if N == 2 else H.NCX)
        regular, noalloc, kernel, _ = _pair(d, 3300 + N, out_scale=0.05)
        assert kernel.startswith("conv_mfma"), kernel
        assert np.array_equal(noalloc, regular)


@pytest.mark.gpu
def test_noalloc_split_reduction_two_calls(gpu_lib, monkeypatch):
    """few output tiles and a long reduction, cut over four workgroups a tile: partial sums and tile
    counters in the scratch array; channels-last in and out"""
    monkeypatch.setenv("HIPQ_SPLIT_K", "4")
    for N in (4, 1):
        say("noalloc split reduction, N", N)
        d = H.make_conv_desc(N, 512, 512, (7, 7), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_t="u8", out_t="i8", data_layout=H.NXC, out_layout=H.NXC)
        regular, noalloc, kernel, args = _pair(d, 3400 + N, out_scale=1.5)
        assert kernel.startswith(("conv_mfma", "dot_")), kernel
        assert np.array_equal(noalloc, regular)
        monkeypatch.delenv("HIPQ_SPLIT_K")
        unsplit = H.quantized_convolution(*args, noalloc=True)
        monkeypatch.setenv("HIPQ_SPLIT_K", "4")
        assert np.array_equal(unsplit, regular)
        assert len(np.unique(regular)) > 50


@pytest.mark.gpu
def test_noalloc_refuses_what_does_not_fit(gpu_lib, monkeypatch):
    monkeypatch.setenv("HIPQ_NO_REGW", "1")  # the kernel that reads NCHW itself needs no scratch and would take this call
    lib = gpu_lib
    N = 176  # 176 x 64 x 56 x 56 = 35.3 MB of NCX input: beyond the 32 MiB the array holds for the copy
    d = H.make_conv_desc(N, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    nbytes = int(np.prod(d.data_shape()))
    assert nbytes > 32 << 20
    data, out = H.DeviceBuffer(nbytes), H.DeviceBuffer(nbytes)
    H.check(lib.hipq_fill_bytes(out.ptr, 0x5A, nbytes, None))
    filt = H.DeviceBuffer.from_numpy(synth.uniform_int(1, d.filter_shape(), -127, 127, np.int8))
    packed = H.pack_filter(d, filt)
    s = [H.DeviceBuffer.from_numpy(np.float32(v)) for v in (0.02, 0.005, 0.1)]
    z = [H.DeviceBuffer.from_numpy(np.zeros(1, t)) for t in (np.uint8, np.int8, np.int8)]
    say("noalloc beyond the limit")
    rc = lib.hipq_quantized_convolution_noalloc(C.byref(d), data.ptr, filt.ptr, packed.ptr, s[0].ptr, z[0].ptr, s[1].ptr, z[1].ptr, s[2].ptr, z[2].ptr, out.ptr, None)
    assert rc == 4, rc  # HIPQ_ERR_LIMIT
    assert b"allocates nothing" in lib.hipq_last_error()
    H.check(lib.hipq_stream_sync(None))
    assert np.all(out.to_numpy(np.uint8, (nbytes,)) == 0x5A)  # nothing was launched
    # the regular entry point takes the same call
    H.check(lib.hipq_quantized_convolution(C.byref(d), data.ptr, filt.ptr, packed.ptr, s[0].ptr, z[0].ptr, s[1].ptr, z[1].ptr, s[2].ptr, z[2].ptr, out.ptr, None))
    H.check(lib.hipq_stream_sync(None))


@pytest.mark.gpu
def test_noalloc_first_on_a_fresh_stream_allocates_nothing_and_replays_from_a_graph(gpu_lib, monkeypatch):
    """The entry point is the first thing a new stream ever sees (no regular call has sized any scratch
    for that stream): the library's allocation epoch must not move.  Then the same call recorded into
    a HIP graph and replayed three times, with eager work of the program between the replays, gives
    the regular entry point's bytes every time (the layout copy into the scratch array is inside the
    graph)."""
    monkeypatch.setenv("HIPQ_NO_REGW", "1")
    lib = gpu_lib
    lib.hipq_workspace_epoch.restype = C.c_uint64
    d = H.make_conv_desc(2, 64, 64, (28, 28), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    nin, nout = int(np.prod(d.data_shape())), int(np.prod(d.out_shape()))
    filt = H.DeviceBuffer.from_numpy(synth.uniform_int(3501, d.filter_shape(), -127, 127, np.int8))
    packed = H.pack_filter(d, filt)
    s = [H.DeviceBuffer.from_numpy(np.float32(v)) for v in (0.02, 0.005, 0.3)]
    z = [H.DeviceBuffer.from_numpy(np.zeros(1, t)) for t in (np.uint8, np.int8, np.int8)]
    data, out, ref = H.DeviceBuffer(nin), H.DeviceBuffer(nout), H.DeviceBuffer(nout)
    sp = C.c_void_p()
    H.check(lib.hipq_stream_create(C.byref(sp)))
    stream = sp.value

    def upload(seed):
        x = synth.uniform_int(seed, d.data_shape(), 0, 255, np.uint8)
        H.check(lib.hipq_memcpy_h2d(data.ptr, x.ctypes.data, x.nbytes, None))

    def call(fn, dst, st):
        H.check(fn(C.byref(d), data.ptr, filt.ptr, packed.ptr, s[0].ptr, z[0].ptr, s[1].ptr, z[1].ptr, s[2].ptr, z[2].ptr, dst.ptr, st))

    say("noalloc first on a fresh stream")
    upload(3502)
    epoch = lib.hipq_workspace_epoch()
    call(lib.hipq_quantized_convolution_noalloc, out, stream)
    H.check(lib.hipq_stream_sync(stream))
    assert lib.hipq_workspace_epoch() == epoch, "the entry point that allocates nothing moved the allocation epoch"
    call(lib.hipq_quantized_convolution, ref, None)
    H.check(lib.hipq_stream_sync(None))
    first = out.to_numpy(np.uint8, (nout,))
    assert np.array_equal(first, ref.to_numpy(np.uint8, (nout,)))
    assert len(np.unique(first)) > 50

    say("noalloc recorded into a graph")
    H.check(lib.hipq_capture_begin(stream))
    call(lib.hipq_quantized_convolution_noalloc, out, stream)
    graph = C.c_void_p()
    H.check(lib.hipq_capture_end(stream, C.byref(graph)))
    try:
        for i in range(3):
            upload(3510 + i)  # eager work and a synchronisation between the replays
            call(lib.hipq_quantized_convolution, ref, None)
            H.check(lib.hipq_stream_sync(None))
            H.check(lib.hipq_fill_bytes(out.ptr, 0xA5, nout, stream))
            say("replay", i)
            H.check(lib.hipq_graph_launch(graph, stream))
            H.check(lib.hipq_stream_sync(stream))
            assert np.array_equal(out.to_numpy(np.uint8, (nout,)), ref.to_numpy(np.uint8, (nout,))), "replay %d differs from the eager result" % i
        assert lib.hipq_workspace_epoch() >= epoch
    finally:
        H.check(lib.hipq_graph_destroy(graph))
        H.check(lib.hipq_stream_destroy(stream))
