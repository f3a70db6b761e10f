"""Pins for the oracle's unary / binary / narrowing operations
(npu/lib/Dialect/TritonTenstorrent/Transforms/ConvertComputeOps.cpp:162-182)."""
import numpy as np
import pytest

from oracle import oracle as orc

RNG = np.random.default_rng(5)
X = np.concatenate([RNG.standard_normal(5000).astype(np.float32) * 10,
                    np.array([0.0, -0.0, 1.0, -1.0, 0.5, 2.5, -2.5, 1e-40, -1e-40, 3.4e38, -3.4e38, np.inf, -np.inf, np.nan],
                             dtype=np.float32)])
Y = np.concatenate([RNG.standard_normal(5000).astype(np.float32) * 3,
                    np.array([-0.0, 0.0, np.nan, 2.0, 0.0, np.inf, -np.inf, 1e-40, 1e-40, 3.4e38, 3.4e38, np.inf, np.inf, 1.0],
                             dtype=np.float32)])


def _same(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32)) or (
        np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~np.isnan(a)].view(np.uint32), b[~np.isnan(b)].view(np.uint32)))


@pytest.mark.parametrize("op,ref", [("abs", np.abs), ("ceil", np.ceil), ("floor", np.floor), ("sqrt", np.sqrt)])
def test_exact_unary_ops_equal_numpy_float32(op, ref):
    with np.errstate(all="ignore"):
        assert _same(orc.unary(op, X), ref(X).astype(np.float32))


@pytest.mark.parametrize("op,ref", [("cos", np.cos), ("sin", np.sin), ("exp", np.exp), ("exp2", np.exp2), ("log", np.log),
                                    ("log2", np.log2), ("rsqrt", lambda v: 1.0 / np.sqrt(v))])
def test_transcendental_unary_ops_are_float64_rounded_once(op, ref):
    with np.errstate(all="ignore"):
        want = ref(X.astype(np.float64)).astype(np.float32)
        got = orc.unary(op, X)
    # glibc's and numpy's float64 routines may differ in the last place of the float64 result; after rounding to
    # fp32 that shows as at most one fp32 ulp, and only on ties
    ok = np.isnan(want) == np.isnan(got)
    fin = np.isfinite(want) & np.isfinite(got)
    assert ok.all() and np.array_equal(np.isinf(want), np.isinf(got))
    assert np.all(np.abs(got[fin].astype(np.float64) - want[fin].astype(np.float64)) <= np.spacing(np.abs(want[fin])))
    assert np.mean(got[fin] == want[fin]) > 0.999


@pytest.mark.parametrize("op,ref", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)])
def test_arithmetic_equals_numpy_float32(op, ref):
    with np.errstate(all="ignore"):
        assert _same(orc.binary(op, X, Y), ref(X, Y))


def test_maximum_minimum_nan_and_signed_zero_tables():
    nan, inf = np.float32(np.nan), np.float32(np.inf)
    a = np.array([1, 2, nan, 1, nan, 0.0, -0.0, -inf, inf, -0.0], dtype=np.float32)
    b = np.array([2, 1, 1, nan, nan, -0.0, 0.0, 5, 5, -0.0], dtype=np.float32)
    mx, mn = orc.binary("maximum", a, b), orc.binary("minimum", a, b)
    assert np.array_equal(np.isnan(mx), [0, 0, 1, 1, 1, 0, 0, 0, 0, 0]) and np.array_equal(np.isnan(mn), np.isnan(mx))
    assert list(mx[[0, 1, 7, 8]]) == [2, 2, 5, inf] and list(mn[[0, 1, 7, 8]]) == [1, 1, -inf, 5]
    # -0 is below +0 whichever side it is on
    assert not np.signbit(mx[5]) and not np.signbit(mx[6]) and np.signbit(mx[9])
    assert np.signbit(mn[5]) and np.signbit(mn[6]) and np.signbit(mn[9])
    # away from NaN and zero ties it is numpy's maximum / minimum
    with np.errstate(all="ignore"):
        plain = ~(np.isnan(X) | np.isnan(Y) | ((X == 0) & (Y == 0)))
        assert np.array_equal(orc.binary("maximum", X, Y)[plain], np.maximum(X, Y)[plain])
        assert np.array_equal(orc.binary("minimum", X, Y)[plain], np.minimum(X, Y)[plain])


def test_masked_block_form_and_partial_grid():
    x = np.arange(1, 3001, dtype=np.float32)
    out = np.full(3000, -7.0, dtype=np.float32)
    orc.unary("sqrt", x, block=1024, grid=2, out=out)
    assert np.array_equal(out[:2048], np.sqrt(x[:2048])) and np.all(out[2048:] == -7.0)
    out2 = np.full(3000, -7.0, dtype=np.float32)
    orc.binary("mul", x, x, block=1024, grid=3, out=out2, nthreads=3)
    assert np.array_equal(out2, x * x)


def test_trunci_keeps_low_bits():
    x = np.array([0, 1, -1, 127, 128, 255, 256, 32767, 32768, 65535, 65536, -32769, 2**31 - 1, -2**31], dtype=np.int32)
    assert np.array_equal(orc.trunci(x, 16), x.astype(np.int16))
    assert np.array_equal(orc.trunci(x, 8), x.astype(np.int8))


@pytest.mark.parametrize("op,ref", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)])
@pytest.mark.parametrize("c", [2.0, -0.75, 0.0, np.inf])
def test_constant_operand_forms_equal_numpy_float32(op, ref, c):
    # x OP c and c OP x against numpy's own float32 arithmetic (not the oracle's formula); in place as well
    cf = np.float32(c)
    with np.errstate(all="ignore"):
        assert _same(orc.binary_const(op, X, c), ref(X, cf).astype(np.float32))
        assert _same(orc.binary_const(op, X, c, flip=True), ref(cf, X).astype(np.float32))
        buf = X.copy()
        assert orc.binary_const(op, buf, c, out=buf) is buf and _same(buf, ref(X, cf).astype(np.float32))
    # and it is the two-operand oracle with a constant second array
    assert _same(orc.binary_const(op, X, c), orc.binary(op, X, np.full_like(X, cf)))


def test_constant_operand_max_min_and_one_element_per_program():
    for op in ("maximum", "minimum"):
        for c in (0.5, np.nan, -0.0):
            assert _same(orc.binary_const(op, X, c), orc.binary(op, X, np.full_like(X, np.float32(c))))
            assert _same(orc.binary_const(op, X, c, flip=True), orc.binary(op, np.full_like(X, np.float32(c)), X))
    # test_core.py::test_load_store_same_ptr: 65536 programs, one element each, x * 2 in place
    x = np.ones(65536, np.float32)
    orc.binary_const("mul", x, 2.0, block=1, grid=65536, out=x)
    assert np.all(x == 2.0)
    y = np.ones(10, np.float32)
    orc.binary_const("mul", y, 2.0, block=1, grid=4, out=y)       # a smaller grid touches its own elements only
    assert np.array_equal(y, [2, 2, 2, 2, 1, 1, 1, 1, 1, 1])


def test_copy_moves_the_masked_block_and_nothing_else():
    """Pinned by what a masked copy must do: the first min(n, grid*block) elements are the source's, bit for bit
    (NaN payloads included), the rest of the destination is untouched; a ragged last block and a short grid."""
    rng = np.random.default_rng(11)
    for dt in (np.uint8, np.int16, np.float32, np.int64):
        x = rng.integers(0, 255, 5000 * np.dtype(dt).itemsize, dtype=np.uint8).view(dt)
        for n, block, grid in ((5000, 1024, None), (4097, 1024, None), (5000, 1024, 3), (10, 16, 10), (0, 16, 1)):
            out = np.full(5000, 7, dtype=dt)
            orc.copy(x, out, n, block=block, grid=grid)
            moved = min(n, (orc.cdiv(n, block) if grid is None else grid) * block)
            assert out[:moved].tobytes() == x[:moved].tobytes() and np.all(out[moved:] == 7), (dt, n, block, grid)

