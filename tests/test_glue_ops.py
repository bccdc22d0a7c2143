"""Elementwise and shape glue of int8 networks on the device: Add / Subtract / Multiply / Maximum /
Minimum, Abs, Relu, Convert, Reshape's transpositions.  The reference kernels are single
expressions on the element type (src/ngraph/runtime/reference/add.hpp:30-36 `arg0[i] + arg1[i]`,
relu.hpp:29-33 `arg[i] > 0 ? arg[i] : 0`, abs.hpp, maximum.hpp, minimum.hpp, convert.hpp:28-34
`static_cast<TO>`, reshape.hpp): numpy's same-dtype arithmetic wraps the way those do, so numpy is the
restatement here.  Sizes cross the 16-byte vector kernels, their scalar tails and the small-tensor path.
"""
import numpy as np
import pytest

from ngraph_amd import hipq as H
from ngraph_amd import synth

SIZES = [1, 15, 4096, 4099, 70001]


def _rand(seed, n, dtype):
    if dtype == np.float32:
        return synth.normal_f32(seed, (n,))
    info = np.iinfo(dtype)
    lo, hi = (info.min, info.max) if dtype != np.int32 else (-(2**31), 2**31 - 1)
    return synth.uniform_int(seed, (n,), lo, hi, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.int32, np.float32])
def test_binary_ops(gpu_lib, dtype):
    with np.errstate(over="ignore"):
        for n in SIZES:
            a, b = _rand(11, n, dtype), _rand(12, n, dtype)
            for op, fn in (("add", np.add), ("subtract", np.subtract), ("multiply", np.multiply), ("maximum", np.maximum), ("minimum", np.minimum)):
                print("[case] binary", np.dtype(dtype).name, op, n, flush=True)
                got = H.binary(op, a, b)
                assert got.dtype == a.dtype
                assert np.array_equal(got, fn(a, b).astype(dtype)), (op, n)
            # one side a single element
            assert np.array_equal(H.binary("add", a, b[:1]), (a + b[0]).astype(dtype))
            assert np.array_equal(H.binary("subtract", a[:1], b), (a[0] - b).astype(dtype))
    # the vector kernel was the one that ran for the bulk sizes
    H.binary("add", _rand(1, 70000 * 16, dtype), _rand(2, 70000 * 16, dtype))
    assert H.last_kernel() == "binary_vec"


@pytest.mark.gpu
def test_divide(gpu_lib):
    """op::v1::Divide: floor division for integers by default (is_pythondiv, src/ngraph/op/divide.hpp:72,
    reference/divide.hpp:41-60 -- numpy's `//`), C++ truncation with the flag off; floats divide the same
    way under both.  Mixed signs with a remainder are where the two differ by one."""
    for n in SIZES:
        a, b = synth.normal_f32(21, (n,)), synth.normal_f32(22, (n,))
        assert np.array_equal(H.binary("divide", a, b), a / b)
        assert np.array_equal(H.binary("divide_floor", a, b), a / b)
        ia = synth.uniform_int(23, (n,), -100000, 100000, np.int32)
        ib = synth.uniform_int(24, (n,), -300, 300, np.int32)
        ib[ib == 0] = 7
        trunc = (np.abs(ia) // np.abs(ib) * np.sign(ia) * np.sign(ib)).astype(np.int32)
        assert np.array_equal(H.binary("divide", ia, ib), trunc)
        assert np.array_equal(H.binary("divide_floor", ia, ib), ia // ib)
        if n > 1000:
            assert np.any(trunc != ia // ib)
        sa = synth.uniform_int(27, (n,), -128, 127, np.int8)
        sb = synth.uniform_int(28, (n,), -128, 127, np.int8)
        sb[sb == 0] = -3
        wide = sa.astype(np.int32) // sb.astype(np.int32)
        assert np.array_equal(H.binary("divide_floor", sa, sb), wide.astype(np.int8))  # -128 // -1 wraps like the reference's T quot
        ua = synth.uniform_int(25, (n,), 0, 255, np.uint8)
        ub = synth.uniform_int(26, (n,), 1, 255, np.uint8)
        assert np.array_equal(H.binary("divide", ua, ub), ua // ub)
        assert np.array_equal(H.binary("divide_floor", ua, ub), ua // ub)
    # hand-checked corners of the reference's rule: quot - 1 when rem != 0 and the signs differ
    a = np.array([7, -7, 7, -7, 6, -6, 0, -1], np.int32)
    b = np.array([2, 2, -2, -2, 3, 3, 5, 5], np.int32)
    assert H.binary("divide_floor", a, b).tolist() == [3, -4, -4, 3, 2, -2, 0, -1]
    assert H.binary("divide", a, b).tolist() == [3, -3, -3, 3, 2, -2, 0, 0]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.int32, np.float32])
def test_unary_ops(gpu_lib, dtype):
    with np.errstate(over="ignore"):
        for n in SIZES:
            x = _rand(31, n, dtype)
            print("[case] unary", np.dtype(dtype).name, n, flush=True)
            assert np.array_equal(H.unary("relu", x), np.maximum(x, 0).astype(dtype))
            # -(-128) wraps back to -128 in int8, as in the reference's `-x`
            assert np.array_equal(H.unary("abs", x), np.where(x < 0, (0 - x).astype(dtype), x))
            assert np.array_equal(H.unary("copy", x), x)
    H.unary("relu", _rand(1, 1 << 20, dtype))
    assert H.last_kernel() == "unary_vec"


@pytest.mark.gpu
def test_convert(gpu_lib):
    for n in SIZES:
        u = _rand(41, n, np.uint8)
        i = _rand(42, n, np.int8)
        assert np.array_equal(H.convert(u, np.int8), u.view(np.int8))
        assert np.array_equal(H.convert(i, np.uint8), i.view(np.uint8))
        assert np.array_equal(H.convert(u, np.float32), u.astype(np.float32))
        assert np.array_equal(H.convert(i, np.int32), i.astype(np.int32))
        w = _rand(43, n, np.int32)
        assert np.array_equal(H.convert(w, np.int8), w.astype(np.int8))
        f = (synth.normal_f32(44, (n,)) * np.float32(50)).astype(np.float32)
        assert np.array_equal(H.convert(f, np.int32), np.trunc(f).astype(np.int32))
        assert np.array_equal(H.convert(f, np.int8), np.trunc(f).astype(np.int32).astype(np.int8))


PERMUTES = [
    ((4, 32, 6, 8), (0, 2, 3, 1)),  # NCHW -> NHWC, every extent a multiple of 16 after grouping
    ((4, 6, 8, 32), (0, 3, 1, 2)),  # NHWC -> NCHW
    ((3, 5, 7, 9), (0, 2, 3, 1)),
    ((3, 5, 7), (2, 0, 1)),         # two blocks without a leading batch
    ((6, 10), (1, 0)),
    ((2, 3, 4, 5), (0, 1, 2, 3)),   # identity
    ((2, 3, 4, 5), (3, 1, 0, 2)),   # a general permutation
    ((2, 3, 4, 5), (0, 2, 1, 3)),   # middle axes swapped: not a two-block order
    ((2, 5, 3, 4, 16), (2, 0, 3, 1, 4)),  # attention heads split: innermost axis kept, rows of whole 16-byte pieces
    ((3, 4, 6, 64), (0, 2, 1, 3)),        # heads merged
    ((3, 4, 6, 12), (0, 2, 1, 3)),        # the same with rows that are whole pieces for f32 only
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", range(len(PERMUTES)))
@pytest.mark.parametrize("dtype", [np.uint8, np.float32])
def test_permute(gpu_lib, case, dtype):
    shape, order = PERMUTES[case]
    x = _rand(50 + case, int(np.prod(shape)), dtype).reshape(shape)
    got = H.permute(x, order)
    assert np.array_equal(got, np.ascontiguousarray(np.transpose(x, order)))


# op::v0::Slice (src/ngraph/runtime/reference/slice.hpp:30-66): (shape, lower, upper, strides); the first
# three are the shapes of test/backend/slice.in.cpp (matrix, vector, strided 3-D)
SLICES = [
    ((4, 4), (0, 1), (3, 3), (1, 1)),
    ((16,), (2,), (14,), (1,)),
    ((4, 4, 4), (0, 0, 0), (4, 4, 4), (2, 2, 3)),
    ((2, 8, 5, 5), (0, 4, 0, 0), (2, 8, 5, 5), (1, 1, 1, 1)),
    ((3, 7, 9), (1, 2, 3), (3, 7, 8), (1, 3, 2)),
    ((5, 6), (2, 3), (2, 6), (1, 1)),
    ((1, 2, 3, 4, 5, 2), (0, 1, 0, 1, 2, 0), (1, 2, 3, 4, 5, 2), (1, 1, 2, 2, 1, 1)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", range(len(SLICES)))
@pytest.mark.parametrize("dtype", [np.uint8, np.float32, np.float64])
def test_slice(gpu_lib, case, dtype):
    shape, lower, upper, strides = SLICES[case]
    x = (_rand(70 + case, int(np.prod(shape)), np.float32).astype(np.float64) if dtype == np.float64 else _rand(70 + case, int(np.prod(shape)), dtype)).reshape(shape)
    got = H.slice_(x, lower, upper, strides)
    exp = x[tuple(slice(l, u, s) for l, u, s in zip(lower, upper, strides))]
    assert got.shape == exp.shape and np.array_equal(got, exp)


@pytest.mark.gpu
def test_slice_rejects_bounds_outside_the_tensor(gpu_lib):
    x = np.zeros((4, 4), np.float32)
    for lower, upper, strides in (((0, 0), (5, 4), (1, 1)), ((3, 0), (2, 4), (1, 1)), ((0, 0), (4, 4), (0, 1)), ((-1, 0), (4, 4), (1, 1))):
        with pytest.raises(H.HipqError) as e:
            H.slice_(x, lower, upper, strides)
        assert e.value.code == H.ERR_INVALID
