"""A synthetic int8 BERT-base-shaped encoder (12 layers, hidden 768, 12 heads, FFN 3072, sequence
128) made of the ops this library implements, the way a quantized nGraph graph expresses it: the
four projections of a layer are QuantizedDotBias (i8 activations, per-output-channel i8 weights,
i32 bias, f32 result) with a Quantize in front of each, and everything between them stays in f32 --
the attention products (BatchMatMul), Softmax, the residual Adds, LayerNorm and Gelu.

  layer   q   = Quantize(x)                         x f32 [T, H], T = batch * sequence
          qkv = QuantizedDotBias(q, Wqkv [3H, H])   f32 [T, 3H]
          Q, K, V = heads of qkv                    Reshape: [B, S, 3, heads, 64] -> [3, B, heads, S, 64]
          P   = Softmax(BatchMatMul(Q, K^T) / 8)    f32 [B * heads, S, S]
          c   = heads back of BatchMatMul(P, V)     [B, heads, S, 64] -> [T, H]
          a   = QuantizedDotBias(Quantize(c), Wo [H, H])
          x1  = LayerNorm(x + a)
          f   = Gelu(QuantizedDotBias(Quantize(x1), W1 [F, H]))
          x2  = LayerNorm(x1 + QuantizedDotBias(Quantize(f), W2 [H, F]))

Weights are N(0, 0.02) quantized per output channel, activations use fixed symmetric scales
(there is no trained checkpoint or calibration set here), token embeddings are N(0, 1).  The
activations are signed, so the projections take i8 data with zero point 0.  `run` executes the layer
list through any provider of the ops (the HIP library's numpy conveniences, or a CPU
implementation), recording every intermediate; `DevicePlan` executes it with every tensor
resident on the GPU for timing.
"""
import ctypes as C
import math

import numpy as np

from . import hipq as H
from . import synth


class Config:
    def __init__(self, layers=12, hidden=768, heads=12, ffn=3072, seq=128):
        assert hidden % heads == 0
        self.layers, self.hidden, self.heads, self.ffn, self.seq = layers, hidden, heads, ffn, seq
        self.head_dim = hidden // heads
        # fixed activation scales ("calibration" by construction): LayerNorm outputs are of order one; the
        # projections' outputs have deviation 0.02 * sqrt(hidden); a context is an average of ~seq values
        self.s_x = 6.0 / 127.0
        self.s_c = 0.4 / 127.0
        self.s_g = 4.0 * 0.02 * math.sqrt(hidden) / 127.0

    def macs_per_sequence(self):
        h, f, s = self.hidden, self.ffn, self.seq
        return self.layers * s * (4 * h * h + 2 * h * f)


BASE = Config()


def projection(seed, n_out, n_in, s_act):
    """(weights i8 [n_out, n_in], bias i32 [n_out], scale f32 [n_out]) of a QuantizedDotBias whose data
    was quantized with scale s_act: result = (acc + bias) * scale, scale = s_act * s_w[n]"""
    w = synth.normal_f32(seed, (n_out, n_in)) * np.float32(0.02)
    s_w = (np.max(np.abs(w), axis=1) / np.float32(127.0)).astype(np.float32)
    wq = np.clip(np.rint(w / s_w[:, None]), -127, 127).astype(np.int8)
    scale = (np.float32(s_act) * s_w).astype(np.float32)
    bias_f = synth.normal_f32(seed + 1, (n_out,)) * np.float32(0.02)
    bias = np.rint(bias_f / scale).astype(np.int32)
    return wq, bias, scale


def layer_weights(cfg, l):
    h, f = cfg.hidden, cfg.ffn
    seed = 1000 + 100 * l
    return dict(
        qkv=projection(seed, 3 * h, h, cfg.s_x),
        out=projection(seed + 10, h, h, cfg.s_c),
        ffn1=projection(seed + 20, f, h, cfg.s_x),
        ffn2=projection(seed + 30, h, f, cfg.s_g),
        ln1=(synth.uniform_f32(seed + 40, (h,), 0.8, 1.2), synth.uniform_f32(seed + 41, (h,), -0.1, 0.1)),
        ln2=(synth.uniform_f32(seed + 42, (h,), 0.8, 1.2), synth.uniform_f32(seed + 43, (h,), -0.1, 0.1)),
    )


def embeddings(cfg, batch, seed=7):
    return synth.normal_f32(seed, (batch * cfg.seq, cfg.hidden))


def run(provider, x, cfg=BASE, layers=None):
    """executes the encoder on f32 [batch * seq, hidden] through `provider`; returns (output, trace) where
    trace is a list of (name, op, inputs, output) for every op executed, in order"""
    B = x.shape[0] // cfg.seq
    h, hd, nh, S = cfg.hidden, cfg.head_dim, cfg.heads, cfg.seq
    trace = []

    def do(name, op, *args):
        out = getattr(provider, op)(*args)
        trace.append((name, op, args, out))
        return out

    for l in range(cfg.layers if layers is None else layers):
        w = layer_weights(cfg, l)
        p = "l%d_" % l
        q = do(p + "q_x", "quantize", x, cfg.s_x)
        qkv = do(p + "qkv", "dot_bias", q, *w["qkv"])
        heads = do(p + "split", "permute", qkv.reshape(B, S, 3, nh, hd), (2, 0, 3, 1, 4))
        Q, K, V = (heads[i].reshape(B * nh, S, hd) for i in range(3))
        sc = do(p + "scores", "batch_matmul", Q, K, True)
        sc = do(p + "scaled", "scale", sc, 1.0 / math.sqrt(hd))
        pr = do(p + "probs", "softmax", sc)
        ctx = do(p + "context", "batch_matmul", pr, V, False)
        ctx = do(p + "merge", "permute", ctx.reshape(B, nh, S, hd), (0, 2, 1, 3)).reshape(B * S, h)
        qc = do(p + "q_ctx", "quantize", ctx, cfg.s_c)
        att = do(p + "attn_out", "dot_bias", qc, *w["out"])
        x1 = do(p + "res1", "add", x, att)
        x1 = do(p + "ln1", "layer_norm", x1, *w["ln1"])
        q1 = do(p + "q_x1", "quantize", x1, cfg.s_x)
        f1 = do(p + "ffn1", "dot_bias", q1, *w["ffn1"])
        g = do(p + "gelu", "gelu", f1)
        qg = do(p + "q_gelu", "quantize", g, cfg.s_g)
        f2 = do(p + "ffn2", "dot_bias", qg, *w["ffn2"])
        x2 = do(p + "res2", "add", x1, f2)
        x = do(p + "ln2", "layer_norm", x2, *w["ln2"])
    return x, trace


class HipProvider:
    """the HIP library through its numpy-in / numpy-out conveniences (one upload and download per op)"""

    @staticmethod
    def quantize(x, scale):
        return H.quantize(x, np.float32(scale), 0, "i8")

    @staticmethod
    def dot_bias(a, w, bias, scales):
        d = H.make_dot_desc(a.shape[0], a.shape[1], w.shape[0], a_t="i8", out_t="f32", b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=w.shape[0])
        return H.quantized_dot_bias(d, f, a, w, bias, scales)

    @staticmethod
    def permute(x, order):
        return H.permute(x, order)

    @staticmethod
    def batch_matmul(a, b, transpose_b):
        return H.batch_matmul(a, b, False, transpose_b)

    @staticmethod
    def scale(x, c):
        return H.binary("multiply", x, np.asarray([c], dtype=np.float32))

    @staticmethod
    def softmax(x):
        return H.softmax(x, (x.ndim - 1,))

    @staticmethod
    def add(a, b):
        return H.binary("add", a, b)

    @staticmethod
    def layer_norm(x, gamma, beta):
        return H.layer_norm(x, gamma, beta, begin_norm_axis=1, epsilon=1e-5, keep_stats=False)[0]

    @staticmethod
    def gelu(x):
        return H.gelu(x)


class DevicePlan:
    """The encoder with every tensor resident in HBM and the weights prepared once: `launch()` issues
    the kernel launches of every layer on `stream`; `capture()` turns the pass into one HIP graph.

    fused=False launches the graph op by op, 19 launches a layer.  fused=True (what a backend's fusion
    pass makes of the same graph, 9 calls a layer, 7 where a head has 128 keys of depth 64) folds the ops that only re-read and re-write a
    tensor into their producers, each through an entry point whose result equals the op-by-op one bit
    for bit: the head split and merge become views of the attention products (scores, Softmax and
    context of a head are one kernel at 128 keys of depth 64), Multiply goes into Softmax, the residual Add into LayerNorm, Gelu into the projection in front of it, and every
    Quantize into the kernel that produces its input (the context product, LayerNorm, that projection)."""

    def __init__(self, lib, stream, batch, cfg=BASE, fused=True):
        self.lib, self.stream, self.batch, self.cfg = lib, stream, batch, cfg
        self.fused = fused
        self._replay = None
        self.calls, self.keep, self.graph = [], [], None
        vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int32
        lib.hipq_softmax_f32.argtypes = [vp, vp, i64, i64, i64, vp]
        lib.hipq_gelu_f32.argtypes = [vp, vp, i64, vp]
        lib.hipq_layer_norm_f32.argtypes = [vp] * 6 + [i64, i64, C.c_double, vp]
        lib.hipq_batch_matmul_f32.argtypes = [vp] * 3 + [i64] * 4 + [i32] * 2 + [vp]
        T, h, f, S, nh, hd = batch * cfg.seq, cfg.hidden, cfg.ffn, cfg.seq, cfg.heads, cfg.head_dim
        dev = lambda a: self._keep(H.DeviceBuffer.from_numpy(np.ascontiguousarray(a)))
        new = lambda nbytes: self._keep(H.DeviceBuffer(nbytes))
        self.x = new(T * h * 4)
        x8, qkv, heads = new(T * max(h, f)), new(T * 3 * h * 4), new(T * 3 * h * 4)
        scores, probs, ctx, merged = new(batch * nh * S * S * 4), new(batch * nh * S * S * 4), new(T * h * 4), new(T * h * 4)
        proj, res, x1, ffn, gel = new(T * h * 4), new(T * h * 4), new(T * h * 4), new(T * f * 4), new(T * f * 4)
        zero = dev(np.zeros(1, np.int8))
        inv = dev(np.asarray([1.0 / math.sqrt(hd)], np.float32))
        scales = {s: dev(np.asarray(s, np.float32)) for s in (cfg.s_x, cfg.s_c, cfg.s_g)}

        def call(fn, *args):
            self.calls.append((fn, args))

        def quantize(src, n_cols, s):
            d = self._keep(H.make_quant_desc((T, n_cols), (), np.float32, "i8"))
            call(lib.hipq_quantize, d, src, scales[s], zero, x8)

        def dot(wts, K, N, out, src=None):
            wq, bias, scale = wts
            src = x8 if src is None else src
            d = self._keep(H.make_dot_desc(T, K, N, a_t="i8", out_t="f32", b_layout=H.B_NK))
            fd = self._keep(H.make_fused_desc(has_bias=True, with_relu=False, scale_count=N))
            bw = dev(wq)
            call(lib.hipq_quantized_dot_bias, d, fd, src, bw, self._keep(H.pack_dot(d, bw)), dev(bias), dev(scale), out)

        def dot_gelu_quantize(wts, K, N, quant):
            # the projection with Gelu and the Quantize behind it in one call (in the product's epilogue where
            # the library's tile kernels take it, through its workspace otherwise)
            wq, bias, scale = wts
            d = self._keep(H.make_dot_desc(T, K, N, a_t="i8", out_t="f32", b_layout=H.B_NK))
            fd = self._keep(H.make_fused_desc(has_bias=True, with_relu=False, scale_count=N))
            bw = dev(wq)
            call(lib.hipq_quantized_dot_bias_gelu_quantize, d, fd, x8, bw, self._keep(H.pack_dot(d, bw)), dev(bias), dev(scale), quant)

        def permute(src, dst, shape, order):
            call(lib.hipq_permute, 4, src, dst, len(shape), self._keep((i64 * len(shape))(*shape)), self._keep((i32 * len(shape))(*order)))

        if fused:
            lib.hipq_softmax_scaled_f32.argtypes = [vp, vp, vp, i64, i64, i64, vp]
            lib.hipq_gelu_quantize_f32.argtypes = [vp, vp, vp, i64, vp]
            lib.hipq_add_layer_norm_f32.argtypes = [vp] * 6 + [i64, i64, C.c_double, vp]
            lib.hipq_batch_matmul_view_f32.argtypes = [vp] * 5 + [i64] * 4 + [i32] * 2 + [vp]
            lib.hipq_attention_f32.argtypes = [vp] * 7 + [i64] * 4 + [vp]
            lib.hipq_quantized_dot_bias_gelu_quantize.argtypes = [vp] * 9
            qout = {s: self._keep(H.QuantOut(x8.ptr, scales[s].ptr, zero.ptr, H.I8, H.RNE)) for s in scales}
            g8 = new(T * f)
            gelu_out = self._keep(H.QuantOut(g8.ptr, scales[cfg.s_g].ptr, zero.ptr, H.I8, H.RNE))
            H3 = 3 * h
            # Q, K, V of batch element (b, head): rows of the [T, 3H] projection, 3H apart, starting at column
            # {0, H, 2H} + head * hd; scores [B * heads, S, S] dense; the context goes straight into [T, H]
            v_scores = self._keep(H.MatmulView(nh, S * H3, hd, H3, S * H3, hd, H3, nh * S * S, S * S, S))
            v_context = self._keep(H.MatmulView(nh, nh * S * S, S * S, S, S * H3, hd, H3, S * h, hd, h))
            # 128 keys of depth 64: scores, Softmax and context of a head in one kernel
            self.one_kernel_attention = S == 128 and hd == 64
            v_attention = self._keep(H.AttentionView(nh, S * H3, hd, H3, S * H3, hd, H3, S * H3, hd, H3, S * h, hd, h))
            for l in range(cfg.layers):
                w = layer_weights(cfg, l)
                if l == 0:
                    quantize(self.x, h, cfg.s_x)
                dot(w["qkv"], h, H3, qkv)
                if self.one_kernel_attention:
                    call(lib.hipq_attention_f32, qkv, (qkv, h * 4), (qkv, 2 * h * 4), inv, None, v_attention, qout[cfg.s_c], batch * nh, S, S, hd)
                else:
                    call(lib.hipq_batch_matmul_view_f32, qkv, (qkv, h * 4), scores, v_scores, None, batch * nh, S, hd, S, 0, 1)
                    call(lib.hipq_softmax_scaled_f32, scores, inv, probs, batch * nh * S, S, 1)
                    call(lib.hipq_batch_matmul_view_f32, probs, (qkv, 2 * h * 4), None, v_context, qout[cfg.s_c], batch * nh, S, S, hd, 0, 0)
                dot(w["out"], h, h, proj)
                g1, b1 = dev(w["ln1"][0]), dev(w["ln1"][1])
                call(lib.hipq_add_layer_norm_f32, self.x, proj, g1, b1, x1, qout[cfg.s_x], T, h, 1e-5)
                dot_gelu_quantize(w["ffn1"], h, f, gelu_out)  # (reads x8: its bytes go to a tensor of their own)
                dot(w["ffn2"], f, h, proj, src=g8)
                g2, b2 = dev(w["ln2"][0]), dev(w["ln2"][1])
                call(lib.hipq_add_layer_norm_f32, x1, proj, g2, b2, self.x, qout[cfg.s_x] if l + 1 < cfg.layers else None, T, h, 1e-5)
            return
        for l in range(cfg.layers):
            w = layer_weights(cfg, l)
            quantize(self.x, h, cfg.s_x)
            dot(w["qkv"], h, 3 * h, qkv)
            permute(qkv, heads, (batch, S, 3, nh, hd), (2, 0, 3, 1, 4))
            one = T * h * 4  # bytes of one of Q, K, V
            call(lib.hipq_batch_matmul_f32, heads, (heads, one), scores, batch * nh, S, hd, S, 0, 1)
            call(lib.hipq_binary, 2, H.F32, scores, batch * nh * S * S, inv, 1, scores, batch * nh * S * S)
            call(lib.hipq_softmax_f32, scores, probs, batch * nh * S, S, 1)
            call(lib.hipq_batch_matmul_f32, probs, (heads, 2 * one), ctx, batch * nh, S, S, hd, 0, 0)
            permute(ctx, merged, (batch, nh, S, hd), (0, 2, 1, 3))
            quantize(merged, h, cfg.s_c)
            dot(w["out"], h, h, proj)
            call(lib.hipq_binary, 0, H.F32, self.x, T * h, proj, T * h, res, T * h)
            g1, b1 = dev(w["ln1"][0]), dev(w["ln1"][1])
            call(lib.hipq_layer_norm_f32, res, g1, b1, x1, None, None, T, h, 1e-5)
            quantize(x1, h, cfg.s_x)
            dot(w["ffn1"], h, f, ffn)
            call(lib.hipq_gelu_f32, ffn, gel, T * f)
            quantize(gel, f, cfg.s_g)
            dot(w["ffn2"], f, h, proj)
            call(lib.hipq_binary, 0, H.F32, x1, T * h, proj, T * h, res, T * h)
            g2, b2 = dev(w["ln2"][0]), dev(w["ln2"][1])
            call(lib.hipq_layer_norm_f32, res, g2, b2, self.x, None, None, T, h, 1e-5)

    def _keep(self, x):
        self.keep.append(x)
        return x

    def set_input(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        H.check(self.lib.hipq_memcpy_h2d(self.x.ptr, x.ctypes.data, x.nbytes, None))

    @staticmethod
    def _arg(a):
        if isinstance(a, C.Structure):
            return C.byref(a)
        if isinstance(a, tuple):  # (buffer, byte offset)
            return a[0].ptr + a[1]
        if isinstance(a, H.DeviceBuffer):
            return a.ptr
        return a

    def launch(self):
        """one forward pass; the result replaces the input buffer (call set_input before every pass that is to be read)"""
        for fn, args in self.calls:
            rc = fn(*[self._arg(a) for a in args], self.stream)
            if rc:
                H.check(rc)

    def capture(self):
        """records the pass into a HIP graph (after one eager pass that sizes the library's scratch)"""
        if self._replay is None:
            self._replay = H.GraphReplay(self.lib, self.stream, self.launch)
        self._replay.capture()

    def replay(self):
        """launches the recorded graph; records it again first if the library's scratch has moved"""
        if self._replay is None:
            self.capture()
        self._replay.replay()

    def close(self):
        """destroys the recorded graph (the buffers go with the object)"""
        if self._replay is not None:
            self._replay.close()
            self._replay = None

    def read_output(self):
        H.check(self.lib.hipq_stream_sync(self.stream))
        return self.x.to_numpy(np.float32, (self.batch * self.cfg.seq, self.cfg.hidden))
