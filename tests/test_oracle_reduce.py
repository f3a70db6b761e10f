"""The oracle's single-block reductions against independent routines: numpy's reductions (library
code, not the oracle's formula), math.fsum for the rounding bound of float sums, and hand-made
known answers for what only the IR fixes (wraparound at the accumulate width, per-step rounding of a
bf16 sum, the tie rules of the (value, index) combine, the two NaN rules)."""
import math

import numpy as np
import pytest

from oracle import oracle as orc

INTS = {orc.I8: np.int8, orc.I16: np.int16, orc.I32: np.int32, orc.I64: np.int64, orc.U8: np.uint8, orc.U16: np.uint16,
        orc.U32: np.uint32, orc.U64: np.uint64}
SHAPES = [1, 32, 64, 128, 512, 1000]     # 32..512: test_core.py::test_reduce1d


def _ints(rng, dt, n, narrow=False):
    info = np.iinfo(INTS[dt])
    lo, hi = (max(info.min, -5), min(info.max, 5)) if narrow else (info.min, info.max)
    return rng.integers(lo, hi, n, dtype=INTS[dt], endpoint=True)


@pytest.mark.parametrize("dt", list(INTS))
@pytest.mark.parametrize("n", SHAPES)
def test_integer_reductions_match_numpy(dt, n):
    rng = np.random.default_rng(100 * dt + n)
    for narrow in (False, True):            # narrow: many ties
        x = _ints(rng, dt, n, narrow)
        assert orc.reduce1d(x, "min", dt) == x.min() and orc.reduce1d(x, "max", dt) == x.max()
        assert orc.reduce1d(x, "argmin", dt) == np.argmin(x) and orc.reduce1d(x, "argmax", dt) == np.argmax(x)
        assert orc.reduce1d(x, "xor_sum", dt) == np.bitwise_xor.reduce(x)
        # numpy sums in the array's own width when told to: the same wraparound
        assert orc.reduce1d(x, "sum", dt) == x.sum(dtype=INTS[dt])
        # narrow integers summed in 32 bits, as tl.sum does
        if np.dtype(INTS[dt]).itemsize < 4:
            acc = orc.U32 if dt in (orc.U8, orc.U16) else orc.I32
            assert int(orc.reduce1d(x, "sum", dt, acc_dt=acc)) == int(x.astype(np.int64).sum())


def test_integer_known_answers():
    # wraparound at the accumulate width
    assert orc.reduce1d(np.array([2**31 - 1, 1], np.int32), "sum", orc.I32) == -2**31
    assert orc.reduce1d(np.array([200, 100], np.uint8), "sum", orc.U8) == 44
    assert orc.reduce1d(np.array([200, 100], np.uint8), "sum", orc.U8, acc_dt=orc.U32) == 300
    # u8 max runs in i32 after a zero extension and is truncated again: 200 beats 100 (a sign extension would not)
    assert orc.reduce1d(np.array([100, 200], np.uint8), "max", orc.U8, acc_dt=orc.I32, out_dt=orc.U8) == 200
    assert orc.reduce1d(np.array([100, -56], np.int8), "max", orc.I8, acc_dt=orc.I32, out_dt=orc.I8) == 100
    # ties: the left one with tie_break_left; the left fold of the bare combine keeps the last
    x = np.array([3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 9], np.int32)
    assert orc.reduce1d(x, "argmin", orc.I32) == 1 and orc.reduce1d(x, "argmax", orc.I32) == 5
    assert orc.reduce1d(x, "argmin", orc.I32, tie_break_left=False) == 3
    assert orc.reduce1d(x, "argmax", orc.I32, tie_break_left=False) == 11
    assert orc.reduce1d(x, "argmax", orc.I32, out_dt=orc.I64) == 5
    # what the IR cannot hold
    with pytest.raises(ValueError):
        orc.reduce1d(np.zeros(4, np.float32), "xor_sum", orc.F32)
    with pytest.raises(ValueError):
        orc.reduce1d(np.zeros(4, np.int32), "sum", orc.I32, out_dt=orc.I64)


@pytest.mark.parametrize("n", SHAPES)
def test_float_reductions(n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 100).astype(np.float32)
    assert orc.reduce1d(x, "min", orc.F32) == x.min() and orc.reduce1d(x, "max", orc.F32) == x.max()
    assert orc.reduce1d(x, "argmin", orc.F32) == np.argmin(x) and orc.reduce1d(x, "argmax", orc.F32) == np.argmax(x)
    exact = math.fsum(float(v) for v in x)
    bound = n * 2.0**-24 * math.fsum(abs(float(v)) for v in x)       # first-order bound of any fp32 summation order
    assert abs(float(orc.reduce1d(x, "sum", orc.F32)) - exact) <= bound
    xd = rng.standard_normal(n)
    assert abs(float(orc.reduce1d(xd, "sum", orc.F64)) - math.fsum(xd)) <= n * 2.0**-53 * np.abs(xd).sum()
    assert orc.reduce1d(xd, "max", orc.F64) == xd.max()
    # half types: min / max run in fp32 (exact), the result is the element itself
    for dt, conv in ((orc.BF16, orc.to_bf16), (orc.F16, orc.to_f16)):
        h = conv(x)
        as_f32 = orc.convert(h, dt, orc.F32)
        assert orc.reduce1d(h, "max", dt, acc_dt=orc.F32) == as_f32.max()
        assert orc.reduce1d(h, "min", dt, acc_dt=orc.F32, out_dt=dt) == h[np.argmin(as_f32)]
        assert orc.reduce1d(h, "argmax", dt) == np.argmax(as_f32)


def test_float_known_answers():
    one = orc.to_bf16(np.array([256.0, 1.0, 1.0, 1.0], np.float32))
    # a bf16 sum rounds after every addition: 256 + 1 is a tie that goes to even (256) each time
    assert orc.convert(np.array([orc.reduce1d(one, "sum", orc.BF16)], np.uint16), orc.BF16, orc.F32)[0] == 256.0
    # run in fp32 instead, the sum is 259, which rounds to 260 in bf16 (8 significant bits: multiples of 2 up to 512)
    got = orc.reduce1d(one, "sum", orc.BF16, acc_dt=orc.F32, out_dt=orc.BF16)
    assert orc.convert(np.array([got], np.uint16), orc.BF16, orc.F32)[0] == 260.0
    half = orc.to_f16(np.array([2048.0, 1.0, 1.0], np.float32))
    assert orc.convert(np.array([orc.reduce1d(half, "sum", orc.F16)], np.uint16), orc.F16, orc.F32)[0] == 2048.0
    # NaN: dropped by minnumf / maxnumf, kept by minimumf / maximumf
    x = np.array([1.0, np.nan, -3.0, 2.0], np.float32)
    assert orc.reduce1d(x, "max", orc.F32) == 2.0 and orc.reduce1d(x, "min", orc.F32) == -3.0
    assert np.isnan(orc.reduce1d(x, "max", orc.F32, propagate_nan=True))
    assert np.isnan(orc.reduce1d(x, "min", orc.F32, propagate_nan=True))
    assert np.isnan(orc.reduce1d(np.full(3, np.nan, np.float32), "max", orc.F32))
    # signed zeros and infinities
    assert orc.reduce1d(np.array([np.inf, -np.inf, 0.0], np.float32), "argmin", orc.F32) == 1
    assert orc.reduce1d(np.array([-0.0, 0.0, -0.0], np.float32), "argmax", orc.F32) == 0      # -0 == +0: a tie
