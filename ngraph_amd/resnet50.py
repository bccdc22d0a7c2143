"""A synthetic int8 ResNet-50 (v1.5: the stride sits in the 3x3 convolution of a bottleneck) made
of the quantized ops this library implements, the way nGraph's quantized graphs express it after
the fusion passes:

  input       Quantize f32 [N,3,224,224] (N(0,1) images) -> u8, scale 1/32, zero point 128, round half to even
  stem        QuantizedConvolutionBias(relu) 7x7/2, 3 -> 64          u8 [N,3,224,224] -> u8
              MaxPool 3x3/2, pad 1
  bottleneck  QuantizedConvolutionBias(relu) 1x1, in -> mid
              QuantizedConvolutionBias(relu) 3x3/s, mid -> mid
              identity block:   QuantizedConvolutionBiasAdd(relu) 1x1, mid -> out, sum = block input (u8)
              first of a stage: QuantizedConvolutionBias 1x1/s, in -> out (i8, no relu) on the shortcut,
                                QuantizedConvolutionBiasSignedAdd(relu) 1x1 (i8), Convert -> u8
  head        AvgPool 7x7, QuantizedDotBias 2048 -> 1000 requantized to i8, Dequantize -> f32 logits

Weights, biases and scales are seeded pseudo-random numbers (there is no trained checkpoint here);
scales are chosen so that activations keep using the 8-bit range through all 16 blocks.  The layer
list is plain data: `run` executes it through any provider of the ops (the HIP library's numpy
conveniences, or a CPU implementation of the same ops), `DevicePlan` executes it with every tensor
resident on the GPU, channels-last, for timing.
"""
import ctypes as C
import math

import numpy as np

from . import hipq as H
from . import synth

STAGES = [(64, 256, 3, 1), (128, 512, 4, 2), (256, 1024, 6, 2), (512, 2048, 3, 2)]
CLASSES = 1000
INPUT_SCALE, INPUT_ZP = 1.0 / 32, 128  # N(0,1) images: +-4 sigma fill the 8-bit range around 128
LOGIT_SCALE = 0.05                      # scale of the i8 logits the Dequantize at the tail undoes


def _conv(name, seed, Cc, K, R, stride, relu, src, sum_src=None, signed_sum=False, gain=1.0, in_rms=None, fold_zp=0):
    kred = Cc * R * R
    # Weights are uniform in -127 .. 127 (rms 73.3).  With inputs of root mean square a the accumulators
    # have spread 73.3 a sqrt(kred); a ReLU output of spread s has root mean square s / sqrt(2): the scale
    # sqrt(2) / (73.3 sqrt(kred)) hands the next layer the root mean square this layer was given, so the
    # activations neither die out nor saturate over 16 blocks.  `in_rms` (the stem): the input's spread
    # is known, the output is given a spread of 36 (the max pool behind it raises the level again).
    scale = gain * math.sqrt(2.0) / (73.3 * math.sqrt(kred)) if in_rms is None else gain * 36.0 / (in_rms * 73.3 * math.sqrt(kred))
    return dict(op="conv", name=name, seed=seed, C=Cc, K=K, R=R, stride=stride, pad=R // 2, relu=relu, src=src, sum_src=sum_src, signed_sum=signed_sum, scale=scale,
                sum_scale=0.5 if sum_src is not None else None, fold_zp=fold_zp)


def layers():
    """the network as a list of ops; every op names its input(s) by the `name` of an earlier op ("input" for the image)"""
    ops = [dict(op="quantize", name="input_q", src="input", scale=INPUT_SCALE, zp=INPUT_ZP),
           _conv("stem", 1, 3, 64, 7, 2, True, "input_q", in_rms=1.0 / INPUT_SCALE, fold_zp=INPUT_ZP), dict(op="maxpool", name="pool1", src="stem", window=3, stride=2, pad=1)]
    prev, cin, seed = "pool1", 64, 10
    for si, (mid, cout, blocks, stride) in enumerate(STAGES):
        for b in range(blocks):
            s = stride if b == 0 else 1
            p = "s%d_b%d_" % (si + 2, b)
            ops.append(_conv(p + "c1", seed, cin, mid, 1, 1, True, prev))
            ops.append(_conv(p + "c2", seed + 1, mid, mid, 3, s, True, p + "c1"))
            if b == 0:
                ops.append(_conv(p + "down", seed + 2, cin, cout, 1, s, False, prev, gain=0.5))
                ops.append(_conv(p + "c3", seed + 3, mid, cout, 1, 1, True, p + "c2", sum_src=p + "down", signed_sum=True, gain=0.85))
                ops.append(dict(op="convert_u8", name=p + "out", src=p + "c3"))
            else:
                ops.append(_conv(p + "out", seed + 3, mid, cout, 1, 1, True, p + "c2", sum_src=prev, gain=0.85))
            prev, cin, seed = p + "out", cout, seed + 4
    ops.append(dict(op="avgpool", name="pool5", src=prev, window=7, stride=1, pad=0))
    ops.append(dict(op="fc", name="fc", seed=seed, K=2048, N=CLASSES, src="pool5", scale=1.0 / 400))
    ops.append(dict(op="dequantize", name="logits", src="fc", scale=LOGIT_SCALE))
    return ops


def conv_weights(op):
    filt = synth.uniform_int(1000 + op["seed"], (op["K"], op["C"], op["R"], op["R"]), -127, 127, np.int8)
    bias = synth.uniform_int(5000 + op["seed"], (op["K"],), -3000, 3000, np.int32)
    if op["fold_zp"]:
        # the input's zero point folded into the bias, as quantized graphs do for an asymmetric u8 input:
        # sum((x - zp) w) = sum(x w) - zp sum(w)
        bias = (bias - op["fold_zp"] * filt.astype(np.int32).sum(axis=(1, 2, 3))).astype(np.int32)
    scales = (synth.uniform_f32(7000 + op["seed"], (op["K"],), 0.8, 1.2) * np.float32(op["scale"])).astype(np.float32)
    return filt, bias, scales


def fc_weights(op):
    w = synth.uniform_int(1000 + op["seed"], (op["N"], op["K"]), -127, 127, np.int8)
    bias = synth.uniform_int(5000 + op["seed"], (op["N"],), -20000, 20000, np.int32)
    scales = (synth.uniform_f32(7000 + op["seed"], (op["N"],), 0.8, 1.2) * np.float32(op["scale"])).astype(np.float32)
    return w, bias, scales


def synthetic_images(N, seed=42, hw=224):
    """N(0,1) f32 images [N,3,hw,hw]; image i depends on (seed, i) only, so a batch's first images are
    the images of a smaller batch"""
    return np.stack([synth.normal_f32(seed * 1000 + i, (3, hw, hw)) for i in range(N)])


def out_hw(hw, R, stride, pad):
    return (hw + 2 * pad - R) // stride + 1


def run(provider, images, ops=None):
    """executes the network on NCHW numpy tensors through `provider`, which offers
    quantize(x, scale, zp, quant_t), conv(desc, fused_desc, data, filt, bias, sum_in, scales, sum_scale),
    pool(desc, x), dot_bias(desc, fused_desc, a, w, bias, scales), dequantize(q, scale, zp);
    returns {name: tensor} of every op"""
    ops = layers() if ops is None else ops
    t = {"input": np.ascontiguousarray(images)}
    for op in ops:
        x = t[op["src"]]
        N, hw = x.shape[0], x.shape[2] if x.ndim == 4 else 1
        if op["op"] == "quantize":
            t[op["name"]] = provider.quantize(x, np.float32(op["scale"]), np.uint8(op["zp"]), "u8")
        elif op["op"] == "dequantize":
            t[op["name"]] = provider.dequantize(x, np.float32(op["scale"]), np.int8(0))
        elif op["op"] == "conv":
            signed = op["signed_sum"] or not op["relu"]
            out_t = "i8" if signed else "u8"
            d = H.make_conv_desc(N, op["C"], op["K"], (hw, hw), (op["R"], op["R"]), stride=(op["stride"],) * 2, pad_below=(op["pad"],) * 2, pad_above=(op["pad"],) * 2, out_t=out_t)
            has_sum = op["sum_src"] is not None
            f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="i8" if op["signed_sum"] else "u8", with_relu=op["relu"], scale_count=op["K"])
            filt, bias, scales = conv_weights(op)
            t[op["name"]] = provider.conv(d, f, x, filt, bias, t[op["sum_src"]] if has_sum else None, scales, op["sum_scale"])
        elif op["op"] in ("maxpool", "avgpool"):
            d = H.make_pool_desc("max" if op["op"] == "maxpool" else "avg", "u8", N, x.shape[1], [hw, hw], [op["window"]] * 2, [op["stride"]] * 2, [op["pad"]] * 2, [op["pad"]] * 2, False)
            t[op["name"]] = provider.pool(d, x)
        elif op["op"] == "convert_u8":
            t[op["name"]] = x.view(np.uint8)  # static_cast between the 8-bit types keeps the bits
        elif op["op"] == "fc":
            w, bias, scales = fc_weights(op)
            d = H.make_dot_desc(N, op["K"], op["N"], out_t="i8", b_layout=H.B_NK)
            f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=op["N"])
            t[op["name"]] = provider.dot_bias(d, f, x.reshape(N, op["K"]), w, bias, scales)
    return t


class HipProvider:
    """the HIP library through its numpy-in / numpy-out conveniences (one upload and download per op)"""

    @staticmethod
    def quantize(x, scale, zp, quant_t):
        return H.quantize(x, scale, zp, quant_t)

    @staticmethod
    def dequantize(q, scale, zp):
        return H.dequantize(q, scale, zp, "f32")

    @staticmethod
    def conv(d, f, x, filt, bias, sum_in, scales, sum_scale):
        return H.quantized_convolution_fused(d, f, x, filt, bias, sum_in, scales, sum_scale)

    @staticmethod
    def pool(d, x):
        return H.pool(d, x)

    @staticmethod
    def dot_bias(d, f, a, w, bias, scales):
        return H.quantized_dot_bias(d, f, a, w, bias, scales)


class DevicePlan:
    """The network with every tensor resident in HBM, weights packed once: the f32 images arrive in the
    reference's NCHW order, Quantize writes u8 NCHW, the stem reads that and writes channels-last, and
    everything up to the logits stays channels-last.  `launch()` issues the kernel launches of one
    forward pass on `stream`; `capture()` turns them into one HIP graph for `replay()`."""

    def __init__(self, lib, stream, N, hw=224, fuse_pool=True):
        self.lib, self.stream, self.N = lib, stream, N
        self._replay = None
        self.calls, self.keep, self.graph = [], [], None
        dev = lambda a: self._keep(H.DeviceBuffer.from_numpy(np.ascontiguousarray(a)))
        buf = {"input": self._keep(H.DeviceBuffer(N * hw * hw * 3 * 4))}
        shape = {"input": (3, hw)}
        self.input = buf["input"]
        self.ops_per_image = 0
        ops = layers()
        readers = {}
        for op in ops:
            for key in ("src", "sum_src"):
                if op.get(key) is not None:
                    readers[op[key]] = readers.get(op[key], 0) + 1
        pending = None  # a convolution whose only reader is the MaxPool behind it, held back for the fused call
        for i, op in enumerate(ops):
            Cc, h = shape[op["src"]]
            src = buf.get(op["src"])
            if op["op"] == "quantize":
                d = H.make_quant_desc((N, Cc, h, h), (), "f32", "u8")
                out = self._keep(H.DeviceBuffer(N * Cc * h * h))
                bs, bz = dev(np.asarray([op["scale"]], np.float32)), dev(np.asarray([op["zp"]], np.uint8))
                self.calls.append((lib.hipq_quantize, (self._keep(d), src, bs, bz, out)))
                buf[op["name"]], shape[op["name"]] = out, (Cc, h)
            elif op["op"] == "dequantize":
                d = H.make_quant_desc((N, CLASSES), (), "f32", "i8")
                out = self._keep(H.DeviceBuffer(N * CLASSES * 4))
                bs, bz = dev(np.asarray([op["scale"]], np.float32)), dev(np.zeros(1, np.int8))
                self.calls.append((lib.hipq_dequantize, (self._keep(d), src, bs, bz, out)))
                buf[op["name"]] = out
            elif op["op"] == "conv":
                signed = op["signed_sum"] or not op["relu"]
                # the stem reads the Quantize's NCHW bytes itself; every later layer is channels-last
                d = H.make_conv_desc(N, op["C"], op["K"], (h, h), (op["R"], op["R"]), stride=(op["stride"],) * 2, pad_below=(op["pad"],) * 2, pad_above=(op["pad"],) * 2,
                                     out_t="i8" if signed else "u8", data_layout=H.NCX if op["src"] == "input_q" else H.NXC, out_layout=H.NXC)
                has_sum = op["sum_src"] is not None
                f = H.make_fused_desc(has_bias=True, has_sum=has_sum, sum_t="i8" if op["signed_sum"] else "u8", with_relu=op["relu"], scale_count=op["K"])
                filt, bias, scales = conv_weights(op)
                bf, bb, bs = dev(filt), dev(bias), dev(scales)
                packed = self._keep(H.pack_filter(d, bf))
                ho = out_hw(h, op["R"], op["stride"], op["pad"])
                self.ops_per_image += 2 * op["K"] * op["C"] * op["R"] * op["R"] * ho * ho
                shape[op["name"]] = (op["K"], ho)
                nxt = ops[i + 1] if i + 1 < len(ops) else None
                if nxt is not None and nxt["op"] == "maxpool" and nxt["src"] == op["name"] and readers.get(op["name"], 0) == 1 and not has_sum and fuse_pool:
                    pd = H.make_pool_desc("max", "u8", N, op["K"], [ho, ho], [nxt["window"]] * 2, [nxt["stride"]] * 2, [nxt["pad"]] * 2, [nxt["pad"]] * 2, False, H.NXC)
                    if H.conv_max_pool_fusable(d, f, pd):
                        # MaxPool(convolution) in one launch: the convolution's own output is never written
                        pending = (op["name"], self._keep(d), self._keep(f), self._keep(pd), src, packed, bb, bs)
                        continue
                out = self._keep(H.DeviceBuffer(N * op["K"] * ho * ho))
                ss = dev(np.asarray(op["sum_scale"], np.float32)) if has_sum else None
                sm = buf[op["sum_src"]] if has_sum else None
                self.calls.append((lib.hipq_quantized_convolution_fused, (self._keep(d), self._keep(f), src, bf, packed, bb, sm, bs, ss, out)))
                buf[op["name"]] = out
            elif op["op"] in ("maxpool", "avgpool"):
                ho = out_hw(h, op["window"], op["stride"], op["pad"])
                out = self._keep(H.DeviceBuffer(N * Cc * ho * ho))
                if pending is not None and pending[0] == op["src"]:
                    _, cd, cf, pd, csrc, cpacked, cbias, cscale = pending
                    self.calls.append((lib.hipq_quantized_convolution_fused_max_pool, (cd, cf, pd, csrc, cpacked, cbias, cscale, out)))
                    pending = None
                else:
                    d = H.make_pool_desc("max" if op["op"] == "maxpool" else "avg", "u8", N, Cc, [h, h], [op["window"]] * 2, [op["stride"]] * 2, [op["pad"]] * 2, [op["pad"]] * 2, False, H.NXC)
                    self.calls.append((lib.hipq_pool, (self._keep(d), src, out)))
                buf[op["name"]], shape[op["name"]] = out, (Cc, ho)
            elif op["op"] == "convert_u8":
                buf[op["name"]], shape[op["name"]] = src, (Cc, h)  # same bits: the buffer is shared
            elif op["op"] == "fc":
                w, bias, scales = fc_weights(op)
                d = H.make_dot_desc(N, op["K"], op["N"], out_t="i8", b_layout=H.B_NK)
                f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=op["N"])
                bw, bb, bs = dev(w), dev(bias), dev(scales)
                packed = self._keep(H.pack_dot(d, bw))
                out = self._keep(H.DeviceBuffer(N * op["N"]))
                self.calls.append((lib.hipq_quantized_dot_bias, (self._keep(d), self._keep(f), src, bw, packed, bb, bs, out)))
                buf[op["name"]], shape[op["name"]] = out, (op["N"], 1)
                self.ops_per_image += 2 * op["K"] * op["N"]
        self.logits = buf["logits"]
        self.buffers = buf

    def _keep(self, x):
        self.keep.append(x)
        return x

    def set_images_nchw(self, images):
        """uploads f32 [N,3,H,W] images, the tensor the Quantize at the head reads"""
        x = np.ascontiguousarray(images, dtype=np.float32)
        assert x.nbytes == self.input.nbytes
        H.check(self.lib.hipq_memcpy_h2d(self.input.ptr, x.ctypes.data, x.nbytes, None))

    def launch(self):
        for fn, args in self.calls:
            a = [C.byref(x) if isinstance(x, C.Structure) else (None if x is None else x.ptr) for x in args]
            rc = fn(*a, self.stream)
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

    def read_logits(self):
        H.check(self.lib.hipq_stream_sync(self.stream))
        return self.logits.to_numpy(np.float32, (self.N, CLASSES))

    def read(self, name, channels, hw, dtype=np.uint8):
        """a named activation as an NCHW numpy tensor"""
        H.check(self.lib.hipq_stream_sync(self.stream))
        return np.ascontiguousarray(np.moveaxis(self.buffers[name].to_numpy(dtype, (self.N, hw, hw, channels)), -1, 1))
