#!/usr/bin/env python3
"""Benchmark of the int8 hot path on one MI355X.

Headline step: one op::v0::QuantizedConvolution call on the layer of BASELINE config 1
(u8 [N,64,56,56] x i8 [64,64,3,3] -> i8, stride 1, pad 1) through the C ABI with the reference's
NCHW tensors already resident in HBM, filter prepacked once (as a backend does at compile time).
The batch defaults to 128, where a matrix-core fraction is meaningful; the N=1 and N=32 results
of the same layer, the int8 GEMM of config 2 and the Quantize/Dequantize chain of config 3 are
reported in the "results" object of the same JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch N] [--quick]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from ngraph_amd import hipq as H  # noqa: E402
from ngraph_amd import synth  # noqa: E402

PEAK_I8_TOPS = 5000.0  # MI355X dense int8 MFMA, published
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, published
# HBM bytes per launch of the headline kernel at batch 128: not measured by this run (counters need
# a profiler run of their own) but quoted from the FETCH_SIZE / WRITE_SIZE runs summarised in the
# file below (scaled by a 64 MiB copy in the same run); the JSON line names that file
MEASURED_TRAFFIC_BYTES = {("conv_regw_i8_32x32x32", 128): 52.0e6}
TRAFFIC_SOURCE = {"conv_regw_i8_32x32x32": "profiles/conv_regw_config1_batch128.md"}
_DATA_CACHE = {}


class Timer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self, lib, stream):
        self.lib, self.stream = lib, stream
        self.a, self.b = C.c_void_p(), C.c_void_p()
        H.check(lib.hipq_event_create(C.byref(self.a)))
        H.check(lib.hipq_event_create(C.byref(self.b)))

    def run(self, fn, steps, warmup):
        """-> (wall ms per step, event ms per step)"""
        for _ in range(warmup):
            fn()
        H.check(self.lib.hipq_stream_sync(self.stream))
        H.check(self.lib.hipq_event_record(self.a, self.stream))
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        H.check(self.lib.hipq_event_record(self.b, self.stream))
        H.check(self.lib.hipq_stream_sync(self.stream))
        t1 = time.perf_counter()
        ms = C.c_float()
        H.check(self.lib.hipq_event_elapsed_ms(self.a, self.b, C.byref(ms)))
        return (t1 - t0) * 1e3 / steps, ms.value / steps


def dev(a):
    return H.DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def scalar(v, dt):
    return dev(np.asarray(v, dtype=dt))


def bench_conv(lib, stream, timer, N, steps, warmup, layout, out_layout=None, sustained=False):
    out_layout = layout if out_layout is None else out_layout
    d = H.make_conv_desc(N, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1), data_layout=layout, out_layout=out_layout)
    # every image of the batch has bytes of its own (operand content moves this chip's clock: a
    # batch of copies of one image would flatter the kernel); the channels-last tensor holds the same
    # seeded values as the NCHW one, read in its own order
    if N not in _DATA_CACHE:
        _DATA_CACHE[N] = synth.uniform_int(1001, (N, 64, 56, 56), 0, 255, np.uint8)
    data = dev(_DATA_CACHE[N].reshape(d.data_shape()))
    filt = dev(synth.uniform_int(1002, d.filter_shape(), -127, 127, np.int8))
    packed = H.pack_filter(d, filt)
    assert packed is not None
    s = [scalar(v, np.float32) for v in (0.02, 0.005, 0.1)]
    z = [scalar(0, np.uint8), scalar(0, np.int8), scalar(0, np.int8)]
    out = H.DeviceBuffer(int(np.prod(d.out_shape())))

    def step():
        rc = lib.hipq_quantized_convolution(C.byref(d), data.ptr, filt.ptr, packed.ptr, s[0].ptr, z[0].ptr, s[1].ptr, z[1].ptr, s[2].ptr, z[2].ptr, out.ptr, stream)
        if rc:
            H.check(rc)

    wall, ev = timer.run(step, steps, warmup)
    kern = H.last_kernel()
    ops = d.ops()
    name = lambda l: "NCHW" if l == H.NCX else "NHWC"
    out_d = dict(N=N, layout=name(layout), out_layout=name(out_layout), ops=ops, ms_wall=wall, ms_event=ev, tops=ops / (wall * 1e-3) / 1e12, tops_event=ops / (ev * 1e-3) / 1e12, kernel=kern)
    if sustained:
        # the rate the device settles at once its clock has come down under the load: 2000 calls in a
        # row, the last 1000 of them timed, in this same process
        swall, sev = timer.run(step, 1000, 1000)
        out_d["sustained"] = dict(steps=1000, warmup=1000, ms_wall=swall, ms_event=sev, tops=ops / (swall * 1e-3) / 1e12, tops_event=ops / (sev * 1e-3) / 1e12,
                                  frac_of_peak=ops / (sev * 1e-3) / 1e12 / PEAK_I8_TOPS)
    return out_d


def bench_gemm(lib, stream, timer, M, steps, warmup):
    K = N = 4096
    d = H.make_dot_desc(M, K, N, out_t="i8", b_layout=H.B_NK)
    f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=N)
    a = dev(synth.uniform_int(2001, (M, K), 0, 255, np.uint8))
    w = dev(synth.uniform_int(2002, (N, K), -127, 127, np.int8))
    bias = dev(synth.uniform_int(2003, (N,), -(2**15), 2**15, np.int32))
    scale = dev(synth.uniform_f32(2004, (N,), 0.001, 0.01))
    packed = H.pack_dot(d, w)
    out = H.DeviceBuffer(M * N)

    def step():
        rc = lib.hipq_quantized_dot_bias(C.byref(d), C.byref(f), a.ptr, w.ptr, packed.ptr, bias.ptr, scale.ptr, out.ptr, stream)
        if rc:
            H.check(rc)

    wall, ev = timer.run(step, steps, warmup)
    ops = 2 * M * K * N
    nbytes = K * N + M * K + M * N + 4 * N + 4 * N
    return dict(M=M, ops=ops, bytes=nbytes, ms_wall=wall, ms_event=ev, tops=ops / (ev * 1e-3) / 1e12, gbs=nbytes / (ev * 1e-3) / 1e9, kernel=H.last_kernel())


def bench_qdq(lib, stream, timer, steps, warmup, rotate=4):
    """Quantize / Dequantize of f32[64,1024,1024] <-> i8.  Successive steps work on `rotate` distinct
    tensor sets (1.25 GiB of inputs and outputs between two visits of the same bytes at the default
    4), so that the chip's 256 MB memory-side cache cannot serve a step from what the step before
    left in it: the figure is an HBM figure."""
    shape = (64, 1024, 1024)
    n = int(np.prod(shape))
    block = synth.normal_f32(3001, (4, 1024, 1024))
    scale = (np.abs(block).max(axis=(0, 2)) / np.float32(127)).astype(np.float32)
    bxs = [H.DeviceBuffer(n * 4) for _ in range(rotate)]
    for bx in bxs:
        for i in range(16):
            H.check(lib.hipq_memcpy_h2d(bx.ptr + i * block.nbytes, block.ctypes.data, block.nbytes, None))
    bs, bz = dev(scale), dev(np.zeros(1024, np.int8))
    bqs = [H.DeviceBuffer(n) for _ in range(rotate)]
    bdqs = [H.DeviceBuffer(n * 4) for _ in range(rotate)]
    d = H.make_quant_desc(shape, (1,), "f32", "i8")
    turn = [0, 0]

    def q():
        i = turn[0] % rotate
        turn[0] += 1
        rc = lib.hipq_quantize(C.byref(d), bxs[i].ptr, bs.ptr, bz.ptr, bqs[i].ptr, stream)
        if rc:
            H.check(rc)

    def dq():
        i = turn[1] % rotate
        turn[1] += 1
        rc = lib.hipq_dequantize(C.byref(d), bqs[i].ptr, bs.ptr, bz.ptr, bdqs[i].ptr, stream)
        if rc:
            H.check(rc)

    for _ in range(rotate):  # every quantized tensor exists before Dequantize is timed
        q()
    _, evq = timer.run(q, steps, warmup)
    kq = H.last_kernel()
    _, evd = timer.run(dq, steps, warmup)
    kd = H.last_kernel()
    nbytes = 5 * n
    return dict(
        elements=n,
        tensor_sets=rotate,
        quantize=dict(ms_event=evq, gbs=nbytes / (evq * 1e-3) / 1e9, frac_hbm=nbytes / (evq * 1e-3) / 1e9 / PEAK_HBM_GBS, kernel=kq),
        dequantize=dict(ms_event=evd, gbs=nbytes / (evd * 1e-3) / 1e9, frac_hbm=nbytes / (evd * 1e-3) / 1e9 / PEAK_HBM_GBS, kernel=kd),
    )


def bench_pool(lib, stream, timer, steps, warmup, batch=128):
    """ResNet-50's two pools on u8 activations: 3x3/2 max pool after the stem, 7x7 global average"""
    out = []
    for op, Cc, sp, win, st, pad in (("max", 64, 112, 3, 2, 1), ("avg", 2048, 7, 7, 1, 0)):
        for layout, lname in ((H.NCX, "nchw"), (H.NXC, "nhwc")):
            d = H.make_pool_desc(op, "u8", batch, Cc, [sp, sp], [win, win], [st, st], [pad, pad], [pad, pad], False, layout)
            nin = batch * Cc * sp * sp
            nout = int(np.prod(d.out_shape()))
            bx, by = H.DeviceBuffer(nin), H.DeviceBuffer(nout)
            H.check(lib.hipq_fill_bytes(bx.ptr, 7, nin, stream))

            def step():
                rc = lib.hipq_pool(C.byref(d), bx.ptr, by.ptr, stream)
                if rc:
                    H.check(rc)

            _, ev = timer.run(step, steps, warmup)
            gbs = (nin + nout) / (ev * 1e-3) / 1e9
            out.append(dict(op=op + "_pool", layout=lname, shape=[batch, Cc, sp, sp], window=win, stride=st, ms_event=ev, gbs=gbs, frac_hbm=gbs / PEAK_HBM_GBS, kernel=H.last_kernel()))
    return out


def bench_glue(lib, stream, timer, steps, warmup, batch=128):
    """the elementwise / layout glue of an int8 ResNet-50 stage on u8[batch,256,56,56]"""
    n = batch * 256 * 56 * 56
    ba, bb, bo = H.DeviceBuffer(n), H.DeviceBuffer(n), H.DeviceBuffer(n)
    H.check(lib.hipq_fill_bytes(ba.ptr, 3, n, stream))
    H.check(lib.hipq_fill_bytes(bb.ptr, 5, n, stream))
    shape = (C.c_int64 * 4)(batch, 256, 56, 56)
    order = (C.c_int32 * 4)(0, 2, 3, 1)
    ops = {
        "add_u8": (lambda: lib.hipq_binary(0, H.U8, ba.ptr, n, bb.ptr, n, bo.ptr, n, stream), 3 * n),
        "relu_i8": (lambda: lib.hipq_unary(1, H.I8, ba.ptr, bo.ptr, n, stream), 2 * n),
        "convert_i8_u8": (lambda: lib.hipq_convert(H.I8, H.U8, ba.ptr, bo.ptr, n, stream), 2 * n),
        "reshape_nchw_to_nhwc_u8": (lambda: lib.hipq_permute(1, ba.ptr, bo.ptr, 4, shape, order, stream), 2 * n),
    }
    out = []
    for name, (fn, nbytes) in ops.items():
        def step():
            rc = fn()
            if rc:
                H.check(rc)

        _, ev = timer.run(step, steps, warmup)
        gbs = nbytes / (ev * 1e-3) / 1e9
        out.append(dict(op=name, elements=n, ms_event=ev, gbs=gbs, frac_hbm=gbs / PEAK_HBM_GBS, kernel=H.last_kernel()))
    return out


def bench_fp32_glue(lib, stream, timer, steps, warmup):
    """fp32 glue of a BERT-base encoder layer between its quantized projections (batch 32, sequence 128):
    attention softmax f32[32*12*128, 128], Gelu f32[4096, 3072], LayerNorm f32[4096, 768] with affine and stats"""
    f, vp, i64 = C.c_float, C.c_void_p, C.c_int64
    lib.hipq_softmax_f32.argtypes = [vp, vp, i64, i64, i64, vp]
    lib.hipq_gelu_f32.argtypes = [vp, vp, i64, vp]
    lib.hipq_layer_norm_f32.argtypes = [vp] * 6 + [i64, i64, C.c_double, vp]
    n_max = 4096 * 3072
    src = dev(synth.normal_f32(31, (n_max,)))
    dst = H.DeviceBuffer(n_max * 4)
    scale, bias = dev(synth.uniform_f32(32, (768,), 0.5, 1.5)), dev(synth.uniform_f32(33, (768,), -0.5, 0.5))
    mean, var = H.DeviceBuffer(4096 * 4), H.DeviceBuffer(4096 * 4)
    ops = {
        "softmax_f32[49152,128]": (lambda: lib.hipq_softmax_f32(src.ptr, dst.ptr, 32 * 12 * 128, 128, 1, stream), 32 * 12 * 128 * 128),
        "gelu_f32[4096,3072]": (lambda: lib.hipq_gelu_f32(src.ptr, dst.ptr, n_max, stream), n_max),
        "layer_norm_f32[4096,768]": (lambda: lib.hipq_layer_norm_f32(src.ptr, scale.ptr, bias.ptr, dst.ptr, mean.ptr, var.ptr, 4096, 768, 1e-5, stream), 4096 * 768),
    }
    out = []
    for name, (fn, n) in ops.items():
        def step():
            rc = fn()
            if rc:
                H.check(rc)

        _, ev = timer.run(step, steps, warmup)
        gbs = 8 * n / (ev * 1e-3) / 1e9  # one f32 read, one f32 written per element
        out.append(dict(op=name, elements=n, ms_event=ev, gbs=gbs, frac_hbm=gbs / PEAK_HBM_GBS, kernel=H.last_kernel()))
    # attention's two batched products per (image, head): scores = Q K^T [128,64]x[128,64]^T, context = P V [128,128]x[128,64]
    lib.hipq_batch_matmul_f32.argtypes = [vp] * 3 + [i64] * 4 + [C.c_int32] * 2 + [vp]
    heads = 32 * 12
    for name, (m, k, n, tb) in {"scores_f32[384x128x64x128]": (128, 64, 128, 1), "context_f32[384x128x128x64]": (128, 128, 64, 0)}.items():
        def step():
            rc = lib.hipq_batch_matmul_f32(src.ptr, src.ptr + 4 * heads * m * k, dst.ptr, heads, m, k, n, 0, tb, stream)
            if rc:
                H.check(rc)

        _, ev = timer.run(step, steps, warmup)
        nbytes = 4 * heads * (m * k + k * n + m * n)
        out.append(dict(op=name, elements=heads * m * n, ms_event=ev, gbs=nbytes / (ev * 1e-3) / 1e9, frac_hbm=nbytes / (ev * 1e-3) / 1e9 / PEAK_HBM_GBS,
                        tflops=2.0 * heads * m * k * n / (ev * 1e-3) / 1e12, kernel=H.last_kernel()))
    # ... and the whole attention of those heads in one launch: scores, scaled Softmax, context + Quantize,
    # Q, K, V read as views of a [4096, 2304] projection, the context written head-interleaved as i8
    lib.hipq_attention_f32.argtypes = [vp] * 7 + [i64] * 4 + [vp]
    S, nh, hd, h = 128, 12, 64, 768
    view = H.AttentionView(nh, S * 3 * h, hd, 3 * h, S * 3 * h, hd, 3 * h, S * 3 * h, hd, 3 * h, S * h, hd, h)
    inv, qscale, zero = dev(np.asarray([0.125], np.float32)), dev(np.asarray([0.4 / 127.0], np.float32)), dev(np.zeros(1, np.int8))
    qout = H.QuantOut(dst.ptr, qscale.ptr, zero.ptr, H.I8, H.RNE)

    def attention_step():
        rc = lib.hipq_attention_f32(src.ptr, src.ptr + 4 * h, src.ptr + 8 * h, inv.ptr, None, C.byref(view), C.byref(qout), heads, S, S, hd, stream)
        if rc:
            H.check(rc)

    _, ev = timer.run(attention_step, steps, warmup)
    nbytes = 4 * 4096 * 3 * h + 4096 * h
    out.append(dict(op="attention_f32[384x128x64]", elements=4096 * h, ms_event=ev, gbs=nbytes / (ev * 1e-3) / 1e9, frac_hbm=nbytes / (ev * 1e-3) / 1e9 / PEAK_HBM_GBS,
                    tflops=4.0 * heads * S * S * hd / (ev * 1e-3) / 1e12, kernel=H.last_kernel()))
    return out


def bench_bert(lib, stream, timer, batches=(1, 32), use_graph=True):
    """synthetic int8 BERT-base-shaped encoder (ngraph_amd/bert.py): 12 layers of QuantizedDotBias projections
    with f32 attention, Softmax, Gelu and LayerNorm between them, sequence 128, every tensor resident in HBM"""
    from ngraph_amd import bert as B

    out = []
    for n in batches:
        plan = B.DevicePlan(lib, stream, n)
        plan.set_input(B.embeddings(B.BASE, n))
        steps = 10 if n <= 8 else 5
        _, eager = timer.run(plan.launch, steps, 2)
        graph = None
        if use_graph:
            plan.capture()
            _, graph = timer.run(plan.replay, steps, 2)
            plan.close()
        best = eager if graph is None else min(eager, graph)
        out.append(dict(batch=n, ms_eager=eager, ms_graph=graph, sequences_per_s=n / (best * 1e-3), int8_tops=2 * B.BASE.macs_per_sequence() * n / (best * 1e-3) / 1e12, launches=len(plan.calls)))
        del plan
    return out


def bench_resnet50(lib, stream, timer, batches=(1, 32, 128), use_graph=True):
    """synthetic int8 ResNet-50 (ngraph_amd/resnet50.py), every tensor resident in HBM, channels-last,
    one forward pass = 53 convolutions, 2 pools, 1 GEMM; replayed as one HIP graph"""
    from ngraph_amd import resnet50 as R

    out = []
    for n in batches:
        plan = R.DevicePlan(lib, stream, n)
        plan.set_images_nchw(R.synthetic_images(min(n, 4)).repeat((n + 3) // 4, axis=0)[:n])
        steps = 30 if n <= 32 else 10
        _, eager = timer.run(plan.launch, steps, 2)
        graph = None
        if use_graph:
            plan.capture()
            _, graph = timer.run(plan.replay, steps, 2)
            plan.close()
        best = eager if graph is None else min(eager, graph)
        out.append(dict(batch=n, ms_eager=eager, ms_graph=graph, images_per_s=n / (best * 1e-3), tops=plan.ops_per_image * n / (best * 1e-3) / 1e12, launches=len(plan.calls)))
        del plan
    return out


def mfma_ceiling(lib, stream, timer, compute_units):
    """What the matrix cores sustain with nothing in their way: every wavefront of a full-chip launch
    issues one dependent chain of v_mfma_i32_32x32x32_i8 on operands it holds in registers (no memory,
    no LDS, no other instructions).  The rate depends on the operand bytes -- the device lowers its
    clock under the switching activity of dense data -- so it is measured for all-zero operands and
    for the kind the convolution multiplies (random bytes)."""
    probe = H.load_probe()
    iters, wgs = 400, int(compute_units)
    sink = H.DeviceBuffer(wgs * 256 * 4)
    out = {}
    rng = np.random.default_rng(4001)
    for kind, host in (("zero_bytes", np.zeros(8192, np.uint8)), ("random_bytes", rng.integers(0, 256, 8192, dtype=np.uint8))):
        ops = dev(host)

        def step():
            H.check_probe(probe.hipq_probe_mfma_i8(ops.ptr, sink.ptr, wgs, iters, stream))

        _, ev = timer.run(step, 5, 2)
        total = wgs * 4 * 64 * iters * 65536.0
        out[kind] = dict(ms_event=ev, tops=total / (ev * 1e-3) / 1e12, frac_of_published_peak=total / (ev * 1e-3) / 1e12 / PEAK_I8_TOPS)
    return out


def bench_coissue(lib, stream, timer, compute_units):
    """Do matrix and vector instructions share a SIMD's time?  One workgroup of eight wavefronts a
    compute unit (two a SIMD), every wavefront 16 x iters v_mfma_i32_32x32x32_i8 (32 cycles each) with 4, 8
    or 16 independent v_fma_f32 (4 cycles each) behind each of them -- 'both'; the same MFMAs alone;
    the same vector instructions alone; and 'split': four wavefronts issue only MFMAs, the other four
    only vector instructions (half the work of either kind); 'both_acc_regs': 'both' with the accumulators
    in the accumulation registers.  If the two kinds overlap, 'both' takes the longer of the two alone; if
    they take turns, their sum.  (Times move with the clock the chip holds under each mix; the counter run
    in profiles/ gives the same comparison in cycles.)"""
    probe = H.load_probe()
    iters, wgs = 400, int(compute_units)
    sink = H.DeviceBuffer(wgs * 512 * 4)
    ops = dev(np.random.default_rng(4002).integers(0, 256, 2048, dtype=np.uint8))
    out = []
    for v in (4, 8, 16):
        row = {"vector_per_mfma": v}
        for mode, name in ((0, "both"), (1, "mfma_alone"), (2, "vector_alone"), (3, "split"), (4, "both_acc_regs")):

            def step():
                H.check_probe(probe.hipq_probe_coissue(ops.ptr, sink.ptr, wgs, iters, v, mode, stream))

            _, ev = timer.run(step, 5, 2)
            row[name + "_us"] = ev * 1e3
        row["both_over_sum"] = row["both_us"] / (row["mfma_alone_us"] + row["vector_alone_us"])
        row["both_over_longer"] = row["both_us"] / max(row["mfma_alone_us"], row["vector_alone_us"])
        out.append(row)
    return out


def bench_intake(lib, stream, timer, compute_units):
    """What a compute unit takes in: 1 / 2 / 4 workgroups of four wavefronts a compute unit (by their LDS
    allocation) each read 8 MiB in 16-byte pieces -- a wavefront instruction covering 1 KiB contiguous,
    8 rows x 128 bytes, 16 rows x 64 bytes (rows 4096 bytes apart) or 64 rows x 16 bytes (every lane in
    a cache line of its own, rows 1024 bytes apart) -- into registers or straight into
    LDS, out of a 2 MiB window (served by the L2s after the first pass) or out of 2 GiB with a region
    per workgroup (served by HBM).  No division in the address stream; the launch is below 2 % of a sample."""
    probe = H.load_probe()
    cus = int(compute_units)
    total = 2 << 30
    buf = H.DeviceBuffer(total)
    H.check(lib.hipq_fill_bytes(buf.ptr, 5, total, stream))
    sink = H.DeviceBuffer(4 * cus * 256 * 4)
    steps = 256  # x 32 KiB = 8 MiB a workgroup
    out = []
    shapes = {0: "1024 B contiguous", 1: "8 rows x 128 B", 2: "16 rows x 64 B", 3: "64 rows x 16 B"}
    for source, window, spread in (("l2", 2 << 20, 0), ("hbm", total, 1)):
        for to_lds in (0, 1):
            for shape in (0, 1, 2, 3):
                for per_cu in (1, 2, 4):
                    wgs = cus * per_cu
                    lds_bytes = {1: 160 * 1024, 2: 80 * 1024, 4: 40 * 1024}[per_cu]

                    def step():
                        H.check_probe(probe.hipq_probe_intake(buf.ptr, total, window, spread, shape, to_lds, wgs, lds_bytes, steps, sink.ptr, stream))

                    _, ev = timer.run(step, 3, 1)
                    per_cu_gbs = per_cu * steps * 32768 / (ev * 1e-3) / 1e9
                    out.append(dict(source=source, dest="lds" if to_lds else "registers", shape=shapes[shape], workgroups_per_cu=per_cu, ms_event=ev,
                                    gbs_per_cu=per_cu_gbs, tbs_chip=per_cu_gbs * cus / 1e3))
    return out


def bench_atomic_tiles(lib, stream, timer, compute_units):
    """int32 atomic adds of whole 128 x 128 accumulator tiles into L2 (no return value): 256 workgroups,
    8 rounds each, 1 / 4 / 8 workgroups adding to the same tile, on one compute die or across the eight"""
    probe = H.load_probe()
    wgs, rounds = 256, 8
    dst = H.DeviceBuffer(wgs * rounds * 65536)
    H.check(lib.hipq_fill_bytes(dst.ptr, 0, wgs * rounds * 65536, stream))
    out = []
    for share in (1, 4, 8):
        for same_die in (1, 0):
            def step():
                H.check_probe(probe.hipq_probe_atomic_tiles(dst.ptr, wgs * rounds * 65536, wgs, share, same_die, rounds, stream))

            _, ev = timer.run(step, 5, 2)
            n = wgs * rounds * 16384
            out.append(dict(share=share, same_die=bool(same_die), ms_event=ev, giga_atomics_per_s=n / (ev * 1e-3) / 1e9, us_per_tile_per_workgroup=ev * 1e3 / rounds))
    return out


def bench_backend(calls=100, warmup=10):
    """The same workloads through the product boundary: ngraph_amd/host/hip_backend_tests --bench builds the
    graphs with the nGraph API and times Backend::create("HIP") -> compile -> Executable::call with nbench's
    protocol (inputs written once, `warmup` calls, `calls` timed calls, outputs not copied back).  Runs as a
    child process of its own, before this process touches the GPU."""
    import subprocess

    exe = os.path.join(ROOT, "ngraph_amd", "host", "hip_backend_tests")
    if not os.path.exists(exe):
        return dict(status="unavailable", reason="%s is not built" % exe)
    try:
        p = subprocess.run([exe, "--bench", "--calls", str(calls), "--warmup", str(warmup)], capture_output=True, text=True, timeout=600)
    except subprocess.TimeoutExpired:
        return dict(status="unavailable", reason="backend benchmark timed out")
    rows = []
    for line in p.stdout.splitlines():
        if line.startswith("{"):
            try:
                rows.append(json.loads(line))
            except ValueError:
                pass
    if p.returncode != 0 or not rows:
        return dict(status="failed", returncode=p.returncode, stderr=p.stderr[-400:])
    return dict(protocol="Backend::create(\"HIP\") -> compile -> Executable::call; nbench --no_copy_data protocol (src/tools/nbench/benchmark.cpp:141-176): %d warm-up, %d timed calls, "
                         "host stopwatch around the calls; a call returns when its results are in the output tensors" % (warmup, calls), rows=rows)


def bench_launch_floor(lib, stream, timer, launches=(58, 85)):
    """What a pass of n dependent launches costs before any of them computes: n launches in a row of a
    kernel that does nothing (256 workgroups; and 1 workgroup), eagerly and replayed as one HIP graph.
    58 = the launches of a ResNet-50 pass, 85 = of a BERT-base pass."""
    probe = H.load_probe()
    sink = H.DeviceBuffer(65536 * 4)
    out = []
    for n in launches:
        for wgs in (1, 256):
            def chain():
                H.check_probe(probe.hipq_probe_empty_chain(sink.ptr, n, wgs, 1, stream))

            _, eager = timer.run(chain, 20, 3)
            replay = H.GraphReplay(lib, stream, chain)
            replay.capture()
            _, graph = timer.run(replay.replay, 20, 3)
            replay.close()
            out.append(dict(launches=n, workgroups=wgs, ms_eager=eager, ms_graph=graph, us_per_launch_eager=eager * 1e3 / n, us_per_launch_graph=graph * 1e3 / n))
    return out


def under_profiler():
    """rocprofv3 (and its predecessors) announce themselves in the environment of the program they run"""
    pre = os.environ.get("LD_PRELOAD", "")
    return "rocprof" in pre or any(k.startswith(("ROCPROF", "ROCP_", "ROCPROFILER_")) for k in os.environ)


def copy_calibration(lib, stream, timer):
    """a plain device-to-device copy of known size: the yardstick for the FETCH_SIZE / WRITE_SIZE
    counters of a profiler run over this same command"""
    cal_bytes = 64 << 20
    ca, cb = H.DeviceBuffer(cal_bytes), H.DeviceBuffer(cal_bytes)
    H.check(lib.hipq_fill_bytes(ca.ptr, 1, cal_bytes, stream))

    def copy():
        rc = lib.hipq_memcpy_d2d(cb.ptr, ca.ptr, cal_bytes, stream)
        if rc:
            H.check(rc)

    _, cev = timer.run(copy, 10, 2)
    return dict(bytes=cal_bytes, ms_event=cev, gbs=2 * cal_bytes / (cev * 1e-3) / 1e9)


def host_threads():
    """threads for the host baselines: this process's share of the machine (OMP_NUM_THREADS when the
    environment sets it, never more than the CPUs the process may run on)"""
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS", "")
    want = int(env) if env.isdigit() and int(env) > 0 else allowed
    return max(1, min(want, allowed))


def cpu_onednn_conv(batch, threads, seconds=6.0):
    """The headline layer as an int8 convolution through the oneDNN that ships inside PyTorch, all of
    this process's cores.  A DNNL-class stand-in for the reference's CPU backend (which drives oneDNN
    1.6.2 and cannot be built offline) -- not nGraph's own code, and its u8 output saturates where the
    INTERPRETER wraps, so it is timed, not compared."""
    try:
        import torch

        if "onednn" not in torch.backends.quantized.supported_engines:
            return dict(status="unavailable", reason="torch has no onednn quantized engine")
        torch.set_num_threads(threads)
        torch.backends.quantized.engine = "onednn"
        g = torch.Generator().manual_seed(1001)
        x = torch.randint(0, 256, (batch, 64, 56, 56), dtype=torch.uint8, generator=g)
        w = torch.randint(-127, 128, (64, 64, 3, 3), dtype=torch.int8, generator=g)
        qx = torch._make_per_tensor_quantized_tensor(x, 0.02, 0)
        qw = torch._make_per_tensor_quantized_tensor(w, 0.005, 0)
        packed = torch.ops.quantized.conv2d_prepack(qw, None, [1, 1], [1, 1], [1, 1], 1)
        for _ in range(2):
            torch.ops.quantized.conv2d(qx, packed, 0.1, 0)
        calls, t0 = 0, time.perf_counter()
        while True:
            torch.ops.quantized.conv2d(qx, packed, 0.1, 0)
            calls += 1
            el = time.perf_counter() - t0
            if el >= seconds or calls >= 100000:
                break
        ops = 2 * batch * 64 * 64 * 9 * 56 * 56
        ver = [l.strip() for l in torch.__config__.show().splitlines() if "oneDNN" in l or "MKL-DNN" in l]
        return dict(value=ops * calls / el / 1e12, unit="TOP/s", cores=threads, kind="oneDNN via torch %s (quantized engine 'onednn'), not nGraph-CPU" % torch.__version__,
                    library=ver[0] if ver else "", sample="%d calls of quantized.conv2d u8[%d,64,56,56] x i8[64,64,3,3] -> u8, %.1f s" % (calls, batch, el))
    except Exception as e:  # informative only
        return dict(status="unavailable", reason=repr(e)[:200])


def cpu_baseline(batch, seconds=8.0):
    """Host baselines, timed on this machine in the same run, each on a bounded sample:
    * value: the C restatement of the reference kernel (oracle/, OpenMP over output planes) on the
      headline layer at batch `min(batch, 32)`, all of this process's cores -- "port";
    * reference_1core: runtime::reference::convolution itself (oracle/_ref, compiled from the nGraph
      tree) when it was built, config 1 at N=1, one core;
    * onednn_via_torch: the DNNL-class figure (see cpu_onednn_conv);
    * resnet50_int8: one image of the synthetic ResNet-50 through the C restatement, all cores."""
    import oracle_lib as O

    threads = host_threads()
    nb = min(batch, 32)
    d = H.make_conv_desc(nb, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    data = synth.uniform_int(1001, d.data_shape(), 0, 255, np.uint8)
    filt = synth.uniform_int(1002, d.filter_shape(), -127, 127, np.int8)
    O.port().orc_set_threads(threads)
    calls, t0 = 0, time.perf_counter()
    while True:
        O.quantized_convolution(d, data, filt, 0.02, 0, 0.005, 0, 0.1, 0)
        calls += 1
        el = time.perf_counter() - t0
        if el >= seconds or calls >= 100:
            break
    O.port().orc_set_threads(1)
    out = dict(
        value=d.ops() * calls / el / 1e12,
        unit="TOP/s",
        cores=threads,
        host_cpus=os.cpu_count(),
        kind="port",
        sample="%d calls of QuantizedConvolution u8[%d,64,56,56] x i8[64,64,3,3] -> i8 (the headline layer at batch %d), %.1f s, C restatement of runtime::reference::convolution with OpenMP"
        % (calls, nb, nb, el),
    )
    # the reference's own kernel, one core, config 1 as BASELINE states it (N=1)
    d1 = H.make_conv_desc(1, 64, 64, (56, 56), (3, 3), pad_below=(1, 1), pad_above=(1, 1))
    kind = "reference" if O.have_ref() else "port"
    fn = O.ref_quantized_convolution if kind == "reference" else O.quantized_convolution
    calls, t0 = 0, time.perf_counter()
    while True:
        fn(d1, data[:1], filt, 0.02, 0, 0.005, 0, 0.1, 0)
        calls += 1
        el = time.perf_counter() - t0
        if el >= seconds / 2 or calls >= 100:
            break
    out["reference_1core"] = dict(value=d1.ops() * calls / el / 1e12, unit="TOP/s", cores=1, kind=kind,
                                  sample="%d calls of config 1 at N=1, %.1f s, %s" % (calls, el, "runtime::reference::convolution compiled from the nGraph tree" if kind == "reference" else "C restatement of it"))
    out["onednn_via_torch"] = cpu_onednn_conv(nb, threads)
    # the synthetic ResNet-50 on the host: one image through the C restatement of its ops (the fused
    # ops exist only in the reference's CPU backend, which does not build here)
    try:
        from ngraph_amd import resnet50 as R

        class Port:
            quantize = staticmethod(lambda x, s, z, t: O.quantize(x, s, z, t))
            dequantize = staticmethod(lambda q, s, z: O.dequantize(q, s, z, "f32"))
            conv = staticmethod(lambda d, f, x, filt, bias, s, sc, ss: O.quantized_convolution_fused(d, f, x, filt, bias, s, sc, ss))
            pool = staticmethod(lambda d, x: O.pool(d, x))
            dot_bias = staticmethod(lambda d, f, a, w, bias, sc: O.quantized_dot_bias(d, f, a, w, bias, sc))

        O.port().orc_set_threads(threads)
        t0 = time.perf_counter()
        R.run(Port, R.synthetic_images(1))
        el = time.perf_counter() - t0
        O.port().orc_set_threads(1)
        out["resnet50_int8"] = dict(value=1.0 / el, unit="images/s", cores=threads, kind="port", sample="1 image, %.1f s" % el)
    except Exception as e:  # the baseline is informative: never fail the bench over it
        out["resnet50_int8"] = dict(error=str(e))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: 20, as the round-end driver runs it; 200 with --only)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps first (default: 5; 20 with --only)")
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--quick", action="store_true", help="headline workload only, no CPU baseline")
    ap.add_argument("--resnet-only", action="store_true", help="only the synthetic int8 ResNet-50 (for profiling); prints its results")
    ap.add_argument("--bert-only", action="store_true", help="only the synthetic int8 BERT-base encoder (for profiling); prints its results")
    ap.add_argument("--skip-models", action="store_true", help="leave out the BERT and ResNet-50 sections (kernel traces of the single operators; the models have runs of their own)")
    ap.add_argument("--only", choices=["gemm", "qdq", "glue", "intake"],
                    help="only config 2's GEMMs, config 3's Quantize / Dequantize, or the encoder's fp32 glue and attention (for counter runs under a profiler); prints their results")
    ap.add_argument("--no-graph", action="store_true", help="time the models' eager launch sequences only, no HIP-graph capture or replay (for runs under a profiler)")
    args = ap.parse_args()
    # The headline is timed the way the round-end driver times it unless told otherwise: a run of a few
    # hundred launches from idle sits in the power controller's transient (slower than both the first
    # 20 launches and launches 1000-2000, which `sustained` reports either way).  The single-operator
    # sections keep their longer runs.
    if args.steps is None:
        args.steps = 200 if args.only else 20
    if args.warmup is None:
        args.warmup = 20 if args.only else 5
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if under_profiler() and not args.no_graph:
        # graph replays of the models under a profiler's interception of graph launches once ended in a
        # crash whose cause was never established: profiled runs launch eagerly
        print("bench.py: running under a profiler -- models are launched eagerly (--no-graph)", file=sys.stderr)
        args.no_graph = True

    backend = None
    if not (args.quick or args.only or args.resnet_only or args.bert_only or args.skip_models or under_profiler()):
        backend = bench_backend()  # a child process with the GPU to itself: before this process opens the device

    lib = H.load()
    H.check(lib.hipq_set_device(0))
    info = H.DeviceInfo()
    H.check(lib.hipq_get_device_info(C.byref(info)))
    sp = C.c_void_p()
    H.check(lib.hipq_stream_create(C.byref(sp)))
    stream = sp.value
    timer = Timer(lib, stream)

    if args.only == "gemm":
        print(json.dumps({"gemm_config2": [bench_gemm(lib, stream, timer, m, args.steps, args.warmup) for m in (1, 32, 256)], "copy_calibration": copy_calibration(lib, stream, timer)}))
        return
    if args.only == "qdq":
        print(json.dumps({"quantize_dequantize_config3": bench_qdq(lib, stream, timer, args.steps, args.warmup), "copy_calibration": copy_calibration(lib, stream, timer)}))
        return
    if args.only == "intake":
        print(json.dumps({"l2_intake_per_cu": bench_intake(lib, stream, timer, info.compute_units), "atomic_tiles": bench_atomic_tiles(lib, stream, timer, info.compute_units),
                          "launch_floor": bench_launch_floor(lib, stream, timer), "matrix_vector_coissue": bench_coissue(lib, stream, timer, info.compute_units)}))
        return
    if args.only == "glue":
        print(json.dumps({"fp32_glue": bench_fp32_glue(lib, stream, timer, args.steps, args.warmup), "copy_calibration": copy_calibration(lib, stream, timer)}))
        return
    if args.resnet_only:
        print(json.dumps({"resnet50_int8": bench_resnet50(lib, stream, timer, use_graph=not args.no_graph)}))
        return
    if args.bert_only:
        print(json.dumps({"bert_base_int8": bench_bert(lib, stream, timer, use_graph=not args.no_graph)}))
        return

    # headline: the reference's NCHW tensors in, NCHW out
    head = bench_conv(lib, stream, timer, args.batch, args.steps, args.warmup, H.NCX, sustained=True)
    # the dominant kernel of that call alone: channels-last data in (what the call's transpose
    # hands it), NCHW out -- such a call launches only the MFMA kernel
    kern = bench_conv(lib, stream, timer, args.batch, args.steps, args.warmup, H.NXC, H.NCX)
    # channels-last in and out, the layout a backend keeps between layers
    nhwc = bench_conv(lib, stream, timer, args.batch, args.steps, args.warmup, H.NXC)

    results = {"conv_nchw": [head], "conv_kernel_nhwc_in_nchw_out": [kern], "conv_nhwc_kernel": [nhwc]}
    # when the headline call is a single launch (the kernel that reads NCHW itself), its own HIP-event
    # time per step is the dominant kernel's launch duration
    if head["kernel"] == kern["kernel"] and head["kernel"].startswith("conv_regw"):
        kern = head
    results["copy_calibration"] = copy_calibration(lib, stream, timer)
    results["mfma_ceiling_i8"] = mfma_ceiling(lib, stream, timer, info.compute_units)
    cpu = None
    if not args.quick:
        small = max(20, args.steps // 4)
        for n in (1, 32):
            results["conv_nchw"].append(bench_conv(lib, stream, timer, n, args.steps, args.warmup, H.NCX))
            results["conv_nhwc_kernel"].append(bench_conv(lib, stream, timer, n, args.steps, args.warmup, H.NXC))
        results["gemm_config2"] = [bench_gemm(lib, stream, timer, m, small, 5) for m in (1, 32, 256)]
        results["quantize_dequantize_config3"] = bench_qdq(lib, stream, timer, small, 5)
        results["pool_resnet50_u8"] = bench_pool(lib, stream, timer, small, 5, args.batch)
        results["glue_resnet50_u8"] = bench_glue(lib, stream, timer, small, 5, args.batch)
        results["fp32_glue_bert_base"] = bench_fp32_glue(lib, stream, timer, small, 5)
        results["launch_floor"] = bench_launch_floor(lib, stream, timer)
        if not args.skip_models:
            results["bert_base_int8"] = bench_bert(lib, stream, timer, use_graph=not args.no_graph)
            results["resnet50_int8"] = bench_resnet50(lib, stream, timer, use_graph=not args.no_graph)
        cpu = cpu_baseline(args.batch)
    if backend is not None:
        # next to each boundary figure, the same workload as this process timed it over the C ABI
        if "rows" in backend:
            for row in backend["rows"]:
                if row["workload"].startswith("QuantizedConvolution"):
                    row["c_abi_ms"] = head["ms_wall"]
                elif "resnet50_int8" in results:
                    match = [r for r in results["resnet50_int8"] if r["batch"] == row["batch"]]
                    if match:
                        row["c_abi_ms"] = min(v for v in (match[0]["ms_eager"], match[0]["ms_graph"]) if v is not None)
                if "c_abi_ms" in row:
                    row["boundary_over_c_abi"] = row["ms_per_call"] / row["c_abi_ms"]
            backend["gap"] = ("Executable::call replays one captured HIP graph and then waits for the stream (hipStreamSynchronize) before it returns, once per call; the C-ABI loop "
                              "of this process enqueues all its steps and waits once at the end.  The per-call wait and graph launch cost about the same few tens of microseconds at "
                              "every size: a large part of a 20 us convolution, a few per cent of a ResNet-50 pass.")
        results["backend"] = backend

    derived_peak = info.compute_units * info.clock_mhz * 1e6 * 8192 / 1e12
    line = {
        "metric": "QuantizedConvolution int8 TOPS",
        "value": head["tops"],
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_wall"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {
            "workload": "op::v0::QuantizedConvolution u8[%d,64,56,56] x i8[64,64,3,3] -> i8, stride 1, pad 1 (BASELINE config 1 layer at batch %d), NCHW in / NCHW out through the C ABI, filter prepacked; %d distinct seeded images"
            % (args.batch, args.batch, args.batch),
            "ops_per_step": head["ops"],
            "device": info.name.decode(),
            "compute_units": info.compute_units,
            "clock_mhz": info.clock_mhz,
            "derived_i8_peak_tops": derived_peak,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": kern["kernel"],
            "achieved": kern["tops_event"],
            "peak": PEAK_I8_TOPS,
            "unit": "TOP/s",
            "frac": kern["tops_event"] / PEAK_I8_TOPS,
            "traffic": MEASURED_TRAFFIC_BYTES.get((kern["kernel"], args.batch)),
            "traffic_source": TRAFFIC_SOURCE.get(kern["kernel"], "none") + " (counter runs of this command; not measured by this run)",
            "algorithmic_bytes": 2 * args.batch * 64 * 56 * 56 + 64 * 64 * 9,
            "kernel_ms": kern["ms_event"],
            "measured_ceiling_random_bytes": results["mfma_ceiling_i8"]["random_bytes"]["tops"],
            "frac_of_measured_ceiling": kern["tops_event"] / results["mfma_ceiling_i8"]["random_bytes"]["tops"],
        },
        "cpu_baseline": cpu,
        "results": results,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
