"""Pins the oracle's elementwise kernels against closed forms."""
import numpy as np
import pytest

from oracle import oracle as orc


@pytest.mark.parametrize("n", [0, 1, 32, 1023, 1024, 1025, 98432])
def test_add_f32_bit_exact_and_masked(n):
    rng = np.random.default_rng(0)
    pad = 64
    x = rng.random(n + pad, dtype=np.float32)
    y = rng.random(n + pad, dtype=np.float32)
    out = np.full(n + pad, 7.5, dtype=np.float32)
    orc.add(x, y, out, n=n)
    assert np.array_equal(out[:n].view(np.uint32), (x[:n] + y[:n]).view(np.uint32))
    assert np.all(out[n:] == 7.5), "lanes with offset >= n must not be stored"


def test_add_f32_specials_are_ieee():
    x = np.array([np.inf, -np.inf, np.nan, 1e38, -0.0, 1e-45, 3.0e38], dtype=np.float32)
    y = np.array([-np.inf, -np.inf, 1.0, 3e38, 0.0, 1e-45, 3.0e38], dtype=np.float32)
    with np.errstate(all="ignore"):
        want = x + y
    got = orc.add(x, y)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    m = ~np.isnan(want)
    assert np.array_equal(got[m].view(np.uint32), want[m].view(np.uint32))


def test_add_i32_wraps():
    x = np.array([2**31 - 1, -2**31, 5, -(2**20)], dtype=np.int32)
    y = np.array([1, -1, -7, 2**20 - 1], dtype=np.int32)
    got = orc.add(x, y)
    assert got.tolist() == [-2**31, 2**31 - 1, -2, -1]
    rng = np.random.default_rng(1)
    a = rng.integers(-2**31, 2**31, 5000, dtype=np.int64).astype(np.int32)
    b = rng.integers(-2**31, 2**31, 5000, dtype=np.int64).astype(np.int32)
    want = (a.astype(np.int64) + b.astype(np.int64)).astype(np.uint64).astype(np.uint32).view(np.int32)
    assert np.array_equal(orc.add(a, b), want)


def test_partial_grid_leaves_the_rest_untouched():
    n = 5000
    x = np.arange(n, dtype=np.float32)
    out = np.full(n, -1.0, dtype=np.float32)
    orc.add(x, x, out, grid=2)  # programs 0,1 only
    assert np.array_equal(out[:2048], 2 * x[:2048]) and np.all(out[2048:] == -1.0)


def test_result_independent_of_worker_count():
    rng = np.random.default_rng(2)
    x = rng.standard_normal(98432).astype(np.float32)
    y = rng.standard_normal(98432).astype(np.float32)
    ref = orc.add(x, y, nthreads=1)
    for t in (2, 3, 8):
        assert np.array_equal(orc.add(x, y, nthreads=t), ref)


def test_sin_is_correctly_rounded_float64_sin():
    rng = np.random.default_rng(3)
    x = ((rng.random(98432, dtype=np.float32) * 2 - 1) * np.float32(8 * np.pi)).astype(np.float32)
    got = orc.sin(x)
    want = np.sin(x.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # textbook identities on exactly known points
    assert orc.sin(np.array([0.0], dtype=np.float32))[0] == 0.0
    s = orc.sin(np.array([np.pi / 2, -np.pi / 2, np.pi / 6], dtype=np.float32))
    assert abs(s[0] - 1) < 1e-7 and abs(s[1] + 1) < 1e-7 and abs(s[2] - 0.5) < 1e-7
    # libm fp32 variant (the timed CPU baseline) stays within 1 ulp-ish of it
    assert np.max(np.abs(orc.sin(x, libm_f32=True) - want)) <= 2e-7


def test_muladd_fused_vs_unfused():
    x = np.array([1.0 + 2**-12], dtype=np.float32)
    y = np.array([1.0 + 2**-12], dtype=np.float32)
    z = np.array([-(1.0 + 2**-11)], dtype=np.float32)
    fused = orc.muladd(x, y, z, fused=True)[0]
    unfused = orc.muladd(x, y, z, fused=False)[0]
    assert fused == np.float32(2**-24) and unfused == 0.0


def test_pcc_definition():
    a = np.linspace(-1, 1, 100)
    assert orc.pcc(a, a) == pytest.approx(1.0)
    assert orc.pcc(a, -a) == pytest.approx(-1.0)
    assert orc.pcc(np.ones(4), np.ones(4)) == 1.0
    assert orc.pcc(np.ones(4), np.zeros(4)) == 0.0
