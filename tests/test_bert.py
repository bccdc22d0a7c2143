"""The synthetic int8 BERT-base-shaped encoder (ngraph_amd/bert.py; BASELINE's fifth configuration)
against the oracle.

The pipeline alternates int8 projections with f32 glue, and a Quantize sits in front of every
projection: a last-bit difference in an f32 value can move an int8 code by one, so the encoder is
checked op by op -- every op of the device run is fed the oracle's own inputs -- with the bar of each
op's kind: bit-exact for Quantize, QuantizedDotBias, the batched products, Reshape and the
elementwise ops; 1e-5 relative (with the absolute floors of tests/test_fp32_glue.py) for Softmax,
Gelu and LayerNorm.  The end-to-end device pass is then compared with the oracle's in distribution.
"""
import numpy as np
import pytest

import oracle_lib as O
from ngraph_amd import bert as B
from ngraph_amd import hipq as H

f32 = np.float32
SMALL = B.Config(layers=2, hidden=128, heads=2, ffn=256, seq=16)


class OracleProvider:
    """the same ops on the CPU: the C restatement for the library's ops, numpy for what is a single
    expression per element in the reference (multiply.hpp, add.hpp) or a pure index map (reshape.hpp)"""

    @staticmethod
    def quantize(x, scale):
        return O.quantize(x, f32(scale), 0, "i8")

    @staticmethod
    def dot_bias(a, w, bias, scales):
        d = H.make_dot_desc(a.shape[0], a.shape[1], w.shape[0], a_t="i8", out_t="f32", b_layout=H.B_NK)
        f = H.make_fused_desc(has_bias=True, with_relu=False, scale_count=w.shape[0])
        return O.quantized_dot_bias(d, f, a, w, bias, scales)

    @staticmethod
    def permute(x, order):
        return np.ascontiguousarray(x.transpose(order))

    @staticmethod
    def batch_matmul(a, b, transpose_b):
        return O.batch_matmul(a, b, False, transpose_b)

    @staticmethod
    def scale(x, c):
        return (x * f32(c)).astype(f32)

    @staticmethod
    def softmax(x):
        return O.softmax(x, (x.ndim - 1,))

    @staticmethod
    def add(a, b):
        return (a + b).astype(f32)

    @staticmethod
    def layer_norm(x, gamma, beta):
        return O.layer_norm(x, gamma, beta, begin_norm_axis=1, epsilon=1e-5)[0]

    @staticmethod
    def gelu(x):
        return O.gelu(x)


EXACT = {"quantize", "dot_bias", "permute", "batch_matmul", "scale", "add"}


def test_structure():
    cfg = B.BASE
    # 12 layers of 4 H^2 + 2 H F multiply-accumulates a token: 348 G for 32 sequences of 128 tokens
    assert 32 * cfg.macs_per_sequence() == 12 * 4096 * (4 * 768**2 + 2 * 768 * 3072)
    w = B.layer_weights(SMALL, 1)
    assert w["qkv"][0].shape == (384, 128) and w["qkv"][0].dtype == np.int8 and w["ffn2"][0].shape == (128, 256)
    assert w["qkv"][1].dtype == np.int32 and w["qkv"][2].dtype == f32 and np.all(w["qkv"][2] > 0)
    assert np.max(np.abs(w["ffn1"][0])) == 127  # every row uses the full int8 range


def test_oracle_pipeline_is_well_conditioned():
    """the fixed activation scales keep the int8 codes in range (few saturate) and spread (not a handful of codes)"""
    O.port().orc_set_threads(8)
    x = B.embeddings(SMALL, 3)
    out, trace = B.run(OracleProvider, x, SMALL)
    O.port().orc_set_threads(1)
    assert out.shape == x.shape and np.all(np.isfinite(out))
    assert len(trace) == 19 * SMALL.layers
    for name, op, args, res in trace:
        if op == "quantize":
            assert np.mean(np.abs(res.astype(np.int32)) == 127) < 0.02, name
            assert len(np.unique(res)) > 40, name
        if op == "softmax":
            assert np.allclose(res.sum(axis=-1), 1.0, atol=1e-5)


def _check(name, op, got, exp):
    assert got.shape == exp.shape and got.dtype == exp.dtype, name
    if op in EXACT:
        assert np.array_equal(got, exp), (name, float(np.max(np.abs(got.astype(np.float64) - exp.astype(np.float64)))))
    elif op == "softmax":
        assert np.allclose(got, exp, rtol=1e-5, atol=1e-30), name
    elif op == "gelu":
        x = None
        assert np.all(np.abs(got - exp) <= 1e-5 * np.abs(exp) + 3e-7 * np.maximum(np.abs(exp), 1.0)), name
    else:  # layer_norm: (x - mean) cancels near the mean, values are of order one
        assert np.allclose(got, exp, rtol=1e-5, atol=1e-5), name


@pytest.mark.gpu
@pytest.mark.parametrize("cfg,batch,layers", [(SMALL, 3, 2), (B.BASE, 2, 1)], ids=["small", "base-dims"])
def test_every_op_against_oracle(gpu_lib, cfg, batch, layers):
    print("[case] bert every op", cfg.hidden, batch, layers, flush=True)
    O.port().orc_set_threads(8)
    x = B.embeddings(cfg, batch)
    _, trace = B.run(OracleProvider, x, cfg, layers=layers)
    O.port().orc_set_threads(1)
    for name, op, args, exp in trace:
        got = getattr(B.HipProvider, op)(*args)
        _check(name, op, got, exp)


@pytest.mark.gpu
def test_device_plan_against_oracle_pipeline(gpu_lib):
    """the whole pass on the device (every tensor resident, 19 launches a layer), eager and as a HIP
    graph: equal to each other bit for bit, and to the oracle's pass in distribution -- a flipped int8
    code moves a projection's output by one quantization step, so single elements may differ"""
    print("[case] bert device plan", flush=True)
    O.port().orc_set_threads(8)
    x = B.embeddings(SMALL, 4)
    exp, _ = B.run(OracleProvider, x, SMALL)
    O.port().orc_set_threads(1)
    lib = gpu_lib
    sp = H.C.c_void_p()
    H.check(lib.hipq_stream_create(H.C.byref(sp)))
    plan = B.DevicePlan(lib, sp.value, 4, SMALL, fused=False)
    assert len(plan.calls) == 19 * SMALL.layers
    plan.set_input(x)
    plan.launch()
    eager = plan.read_output()
    plan.capture()
    for _ in range(3):
        plan.set_input(x)
        H.check(lib.hipq_stream_sync(None))
        plan.replay()
        assert np.array_equal(plan.read_output(), eager)
    plan.close()
    diff = np.abs(eager - exp)
    print("bert plan vs oracle: max", float(diff.max()), "mean", float(diff.mean()), "beyond 1e-3:", float(np.mean(diff > 1e-3)), flush=True)
    assert np.all(np.isfinite(eager))
    assert diff.mean() < 2e-3 and np.mean(diff > 0.05) < 0.01
    # the HIP provider's op-at-a-time pass takes the same kernels: identical to the plan
    hp, _ = B.run(B.HipProvider, x, SMALL)
    assert np.array_equal(hp, eager)
    # the fused plan (9 calls a layer: reshapes as views, Multiply in Softmax, Add in LayerNorm, every
    # Quantize in its producer) gives the same bits, eager and replayed
    fused = B.DevicePlan(lib, sp.value, 4, SMALL, fused=True)
    assert not fused.one_kernel_attention and len(fused.calls) == 9 * SMALL.layers + 1
    fused.set_input(x)
    fused.launch()
    assert np.array_equal(fused.read_output(), eager)
    fused.capture()
    for _ in range(2):
        fused.set_input(x)
        H.check(lib.hipq_stream_sync(None))
        fused.replay()
        assert np.array_equal(fused.read_output(), eager)
    fused.close()


@pytest.mark.gpu
def test_benchmarked_batch_base_dims(gpu_lib):
    """What the benchmark times: BASE dimensions, 12 layers, batch 32.  Kernel choice depends on the
    row count (tile shapes, split reductions, deep slices), so the batch-32 launches are not the
    batch-2 ones.  Every op is a function of one sequence alone, and every kernel's arithmetic per
    output is the same whatever the batch (exact integer sums; f32 rows reduced by one wavefront in a
    fixed order; products accumulated in double, k ascending): a batch of 16 copies of two sequences
    must reproduce the batch-2 pass bit for bit, eager and as a HIP graph.  The batch-2 pass is tied to
    the oracle op by op: every one of the 12 x 19 ops is run on the oracle's own inputs and held to the
    bar of its kind.  End to end the two passes agree only in distribution, and less tightly than two
    layers do: a last-bit difference in an f32 value flips an int8 code, and twelve layers compound
    the flips (the outputs are layer-normalised, of order one)."""
    lib = gpu_lib
    two = B.embeddings(B.BASE, 2)
    print("[case] bert base oracle pass, 2 sequences x 12 layers", flush=True)
    O.port().orc_set_threads(8)
    exp, trace = B.run(OracleProvider, two, B.BASE)
    O.port().orc_set_threads(1)
    assert len(trace) == 19 * 12
    print("[case] bert base every op of 12 layers on the oracle's inputs", flush=True)
    for name, op, args, res in trace:
        _check(name, op, getattr(B.HipProvider, op)(*args), res)
    sp = H.C.c_void_p()
    H.check(lib.hipq_stream_create(H.C.byref(sp)))
    print("[case] bert base plan, batch 2", flush=True)
    small = B.DevicePlan(lib, sp.value, 2, B.BASE, fused=False)
    assert len(small.calls) == 19 * 12
    small.set_input(two)
    small.launch()
    ref = small.read_output()
    assert np.all(np.isfinite(ref))
    diff = np.abs(ref - exp)
    print("bert base batch 2 vs oracle: max", float(diff.max()), "mean", float(diff.mean()), "beyond 0.05:", float(np.mean(diff > 0.05)), flush=True)
    assert diff.mean() < 0.05 and np.mean(diff > 0.5) < 0.001
    print("[case] bert base plan, batch 32", flush=True)
    x = np.ascontiguousarray(np.tile(two, (16, 1)))
    unfused = B.DevicePlan(lib, sp.value, 32, B.BASE, fused=False)
    unfused.set_input(x)
    unfused.launch()
    assert np.array_equal(unfused.read_output(), np.tile(ref, (16, 1)))
    del unfused
    # what bench.py times: the fused plan (7 calls a layer: a head's scores, Softmax and context are one
    # kernel at 128 keys of depth 64, Gelu and its Quantize ride in the projection in front of them), bit
    # for bit the op-by-op result
    plan = B.DevicePlan(lib, sp.value, 32, B.BASE)
    assert plan.fused and plan.one_kernel_attention and len(plan.calls) == 7 * 12 + 1
    plan.set_input(x)
    plan.launch()
    eager = plan.read_output()
    assert np.array_equal(eager, np.tile(ref, (16, 1)))
    plan.capture()
    for _ in range(2):
        plan.set_input(x)
        H.check(lib.hipq_stream_sync(None))
        plan.replay()
        assert np.array_equal(plan.read_output(), eager)
    plan.close()
    small.close()
    H.check(lib.hipq_stream_destroy(sp.value))
