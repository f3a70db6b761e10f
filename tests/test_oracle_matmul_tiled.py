"""Pins for the oracle's tile-major matmul_kernel restatement
(examples/matmul/03-matrix-multiplication.py:242-391)."""
import numpy as np
import pytest

from oracle import oracle as orc


def _rand_f16(shape, seed):
    rng = np.random.default_rng(seed)
    return (rng.random(shape, dtype=np.float32) - 0.5).astype(np.float16)


def _brute_tilize(x, TR, TC):
    # the kernel's own index map (:326-337), one element at a time
    R, C = x.shape
    ntc = -(-C // TC)
    out = np.zeros((-(-R // TR)) * ntc * TR * TC, dtype=x.dtype)
    for r in range(R):
        for c in range(C):
            out[((r // TR) * ntc + c // TC) * TR * TC + (r % TR) * TC + c % TC] = x[r, c]
    return out


@pytest.mark.parametrize("R,C,TR,TC", [(32, 64, 32, 32), (70, 45, 32, 32), (64, 96, 32, 64), (5, 3, 4, 2)])
def test_tilize_matches_the_kernel_index_map_and_round_trips(R, C, TR, TC):
    x = np.arange(R * C, dtype=np.uint16).reshape(R, C) + 1
    t = orc.tilize(x, TR, TC)
    assert np.array_equal(t, _brute_tilize(x, TR, TC))
    assert np.array_equal(orc.untilize(t, R, C, TR, TC), x)


@pytest.mark.parametrize("M,N,K,BM,BN,BK,G", [(32, 32, 64, 32, 32, 32, 1), (96, 64, 128, 32, 32, 32, 1),
                                              (70, 45, 50, 32, 32, 32, 2), (128, 192, 64, 64, 32, 64, 4),
                                              (33, 31, 17, 32, 64, 16, 1)])
@pytest.mark.parametrize("leaky", [False, True])
def test_tiled_equals_row_major_oracle_bit_for_bit(M, N, K, BM, BN, BK, G, leaky):
    a, b = _rand_f16((M, K), 1), _rand_f16((K, N), 2)
    ab, bb = a.view(np.uint16), b.view(np.uint16)
    ct = orc.matmul_tiled(orc.tilize(ab, BM, BK), orc.tilize(bb, BK, BN), M, N, K, in_dt=orc.F16, BM=BM, BN=BN, BK=BK,
                          group_m=G, leaky_relu=leaky)
    ref = orc.matmul(ab, bb, in_dt=orc.F16, out_dt=orc.F16, BM=BM, BN=BN, BK=BK, group_m=G,
                     epi=orc.EPI_LEAKY_RELU if leaky else orc.EPI_NONE)
    assert np.array_equal(orc.untilize(ct, M, N, BM, BN), ref)


def test_reference_self_check_shape_and_tolerance():
    # 03-matrix-multiplication.py:428-438: rand(32,64)-0.5 @ rand(64,32)-0.5 in fp16, atol 1e-2
    a, b = _rand_f16((32, 64), 0), _rand_f16((64, 32), 3)
    ct = orc.matmul_tiled(orc.tilize(a.view(np.uint16), 32, 32), orc.tilize(b.view(np.uint16), 32, 32), 32, 32, 64)
    got = orc.untilize(ct, 32, 32, 32, 32).view(np.float16).astype(np.float64)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert np.max(np.abs(got - want)) <= 1e-2
    # and to within fp16 rounding of the exact product
    assert np.max(np.abs(got - want)) <= 2.0 ** -11 * np.max(np.abs(want)) + 1e-6


def test_leaky_relu_acts_on_the_accumulator():
    a, b = _rand_f16((32, 32), 4), _rand_f16((32, 32), 5)
    at, bt = orc.tilize(a.view(np.uint16), 32, 32), orc.tilize(b.view(np.uint16), 32, 32)
    plain = orc.matmul_tiled(at, bt, 32, 32, 32, acc64=True).view(np.float16).astype(np.float64)
    leaky = orc.matmul_tiled(at, bt, 32, 32, 32, acc64=True, leaky_relu=True).view(np.float16).astype(np.float64)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    want = np.where(exact >= 0, exact, 0.01 * exact).astype(np.float32).astype(np.float16).astype(np.float64)
    assert np.array_equal(leaky.reshape(32, 32), want)
    assert np.array_equal(plain[plain >= 0], leaky[plain >= 0])


def test_partial_grid_leaves_other_tiles_untouched():
    M = N = 64
    a, b = _rand_f16((M, 32), 6), _rand_f16((32, N), 7)
    out = np.full(4 * 32 * 32, 0x7e00, dtype=np.uint16)
    orc.matmul_tiled(orc.tilize(a.view(np.uint16), 32, 32), orc.tilize(b.view(np.uint16), 32, 32), M, N, 32, grid=3, out=out)
    assert np.all(out[3 * 1024:] == 0x7e00) and not np.any(out[:3 * 1024] == 0x7e00)


def test_partial_grid_writes_the_tiles_the_pointer_decode_names():
    """matmul_kernel takes its row from the position inside the group (03-matrix-multiplication.py:281); on 5x3 tiles
    in groups of 3 the first 12 programs therefore write tiles (3,0), (4,0), (3,1) of the last group, not
    (4,0), (3,0), (4,1) as the descriptor kernels' decode would."""
    M, N, K = 160, 96, 32
    rng = np.random.default_rng(5)
    a = rng.integers(1, 4, (M, K)).astype(np.float16).view(np.uint16)
    b = rng.integers(1, 4, (K, N)).astype(np.float16).view(np.uint16)
    c = orc.matmul_tiled(orc.tilize(a, 32, 32), orc.tilize(b, 32, 32), M, N, K, group_m=3, grid=12)
    written = {(t // 3, t % 3) for t in range(15) if c[t * 1024:(t + 1) * 1024].any()}
    assert written == {(i, j) for i in range(3) for j in range(3)} | {(3, 0), (4, 0), (3, 1)}
    want = a.view(np.float16).astype(np.float32) @ b.view(np.float16).astype(np.float32)
    got = orc.untilize(c, M, N, 32, 32).view(np.float16).astype(np.float32)
    for (i, j) in written:
        assert np.array_equal(got[i * 32:(i + 1) * 32, j * 32:(j + 1) * 32], want[i * 32:(i + 1) * 32, j * 32:(j + 1) * 32])
