"""Pins the oracle's conversions and tile-matmul family against independent
library routines (torch CPU dtypes, numpy float64 matmul) and invariants."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc


def _bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.view(torch.uint8).numpy()


def test_bf16_f16_fp8_rounding_matches_torch_cpu():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 3,
        (rng.standard_normal(5000) * 1e-6).astype(np.float32),
        (rng.standard_normal(5000) * 300).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 448.0, 447.9, 464.0, 1e6, -1e6, 65504.0, 65519.9, 65520.0, 2**-24, 2**-25,
                  1.5 * 2**-25, 2**-9, 2**-10, 1.5 * 2**-10, 0.0156, 1.00390625, 1.01171875], dtype=np.float32),
    ])
    t = torch.from_numpy(x)
    assert np.array_equal(orc.to_bf16(x), _bits(t.to(torch.bfloat16)))
    assert np.array_equal(orc.to_f16(x), _bits(t.to(torch.float16)))
    # e4m3fn: torch does not saturate, the oracle's quantiser does -> compare in range
    inr = np.abs(x) <= 448
    assert np.array_equal(orc.to_fp8(x[inr]), _bits(t[torch.from_numpy(inr)].to(torch.float8_e4m3fn)))
    assert orc.from_fp8(orc.to_fp8(np.array([1e6, -1e6], dtype=np.float32))).tolist() == [448.0, -448.0]
    # decode of every code point
    codes8 = np.arange(256, dtype=np.uint8)
    want8 = torch.from_numpy(codes8).view(torch.float8_e4m3fn).float().numpy()
    got8 = orc.from_fp8(codes8)
    assert np.array_equal(np.isnan(got8), np.isnan(want8))
    assert np.array_equal(got8[~np.isnan(want8)], want8[~np.isnan(want8)])
    codes16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    for dec, tdt in ((orc.from_bf16, torch.bfloat16), (orc.from_f16, torch.float16)):
        want = torch.from_numpy(codes16.view(np.int16)).view(tdt).float().numpy()
        got = dec(codes16)
        ok = ~np.isnan(want)
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[ok], want[ok])


def _rand_bf16(rng, shape, scale=1.0):
    return orc.to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


# the reference's own validate shapes (09-persistent-matmul.py:326-327, .ttnn.py:334-336)
@pytest.mark.parametrize("M,N,K", [(32, 32, 32), (64, 32, 32), (64, 32, 64), (256, 192, 320)])
@pytest.mark.parametrize("BM,BN,BK,G", [(64, 64, 64, 1), (32, 32, 32, 1), (128, 128, 64, 8)])
def test_matmul_is_the_textbook_sum(M, N, K, BM, BN, BK, G):
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a, b = _rand_bf16(rng, (M, K)), _rand_bf16(rng, (K, N), K ** -0.5)
    want64 = orc.from_bf16(a).astype(np.float64) @ orc.from_bf16(b).astype(np.float64)
    # fp64-accumulating oracle must be the correctly rounded textbook sum
    got64 = orc.matmul(a, b, BM=BM, BN=BN, BK=BK, group_m=G, acc64=True)
    assert np.array_equal(got64, orc.to_bf16(want64.astype(np.float32)))
    # fp32-accumulating oracle (the parity target) differs from it by at most 1 bf16 ulp
    got32 = orc.from_bf16(orc.matmul(a, b, BM=BM, BN=BN, BK=BK, group_m=G))
    ref = orc.from_bf16(got64)
    assert np.all(np.abs(got32 - ref) <= 2.0 ** -7 * np.abs(ref) + 1e-6)
    assert orc.pcc(want64, got32) > 0.9999


def test_matmul_small_integers_are_exact_whatever_the_tiling():
    # small-integer inputs: every partial sum is exact in fp32, so all tilings,
    # group sizes and worker counts agree bit for bit with the integer product
    rng = np.random.default_rng(5)
    M, N, K = 192, 128, 256
    ai = rng.integers(-4, 5, (M, K))
    bi = rng.integers(-4, 5, (K, N))
    a, b = orc.to_bf16(ai.astype(np.float32)), orc.to_bf16(bi.astype(np.float32))
    want = orc.to_bf16((ai @ bi).astype(np.float32))  # |c| <= 4096: bf16 rounding applies, same everywhere
    for BM, BN, BK, G, t in [(64, 64, 64, 1, 1), (32, 64, 128, 2, 3), (128, 128, 64, 8, 8), (64, 32, 32, 5, 2)]:
        assert np.array_equal(orc.matmul(a, b, BM=BM, BN=BN, BK=BK, group_m=G, nthreads=t), want)


def test_matmul_identity_and_transposition_sensitivity():
    rng = np.random.default_rng(6)
    a = _rand_bf16(rng, (64, 64))
    eye = orc.to_bf16(np.eye(64, dtype=np.float32))
    assert np.array_equal(orc.matmul(a, eye), a)        # B = I  =>  C = A
    assert np.array_equal(orc.matmul(eye, a), a)
    # B is [K,N] row-major, not transposed: a permutation matrix tells the two apart
    p = np.zeros((64, 64), dtype=np.float32)
    p[np.arange(64), (np.arange(64) + 1) % 64] = 1
    got = orc.from_bf16(orc.matmul(a, orc.to_bf16(p)))
    assert np.array_equal(got, np.roll(orc.from_bf16(a), 1, axis=1))


def test_matmul_ragged_edges_zero_pad_and_clip():
    rng = np.random.default_rng(7)
    M, N, K = 70, 45, 100
    a, b = _rand_bf16(rng, (M, K)), _rand_bf16(rng, (K, N), 0.1)
    out = np.full((M + 3, N + 5), 0x40F0, dtype=np.uint16)  # 7.5 sentinel
    view = out[:M, :N]
    orc.matmul(a, b, BM=64, BN=64, BK=64, out=view, acc64=True)
    want = orc.to_bf16((orc.from_bf16(a).astype(np.float64) @ orc.from_bf16(b).astype(np.float64)).astype(np.float32))
    assert np.array_equal(view, want)
    assert np.all(out[M:, :] == 0x40F0) and np.all(out[:, N:] == 0x40F0)


def test_matmul_partial_grid_writes_only_its_tiles():
    rng = np.random.default_rng(8)
    a, b = _rand_bf16(rng, (128, 64)), _rand_bf16(rng, (64, 128))
    out = np.full((128, 128), 0x40F0, dtype=np.uint16)
    orc.matmul(a, b, BM=64, BN=64, BK=64, grid=3, out=out)
    full = orc.matmul(a, b, BM=64, BN=64, BK=64)
    assert np.all(out[64:, 64:] == 0x40F0)  # pid 3 = tile (1,1) never ran
    assert np.array_equal(out[:64, :], full[:64, :]) and np.array_equal(out[64:, :64], full[64:, :64])
    with pytest.raises(ValueError):
        orc.matmul(a, b, BM=64, BN=64, BK=64, grid=5)


def test_fused_full_bias_is_a_half_precision_add_after_the_cast():
    # 09-matmul-fused.py:139-146: c = acc.to(half); c = c + bias
    rng = np.random.default_rng(9)
    M = N = K = 64
    for dt, tdt, enc in ((orc.F16, torch.float16, orc.to_f16), (orc.BF16, torch.bfloat16, orc.to_bf16)):
        a = enc(rng.standard_normal((M, K)).astype(np.float32))
        b = enc((rng.standard_normal((K, N)) / 8).astype(np.float32))
        bias = enc(rng.standard_normal((M, N)).astype(np.float32))
        got = orc.matmul(a, b, in_dt=dt, out_dt=dt, bias=bias, epi=orc.EPI_BIAS_FULL)
        plain = orc.matmul(a, b, in_dt=dt, out_dt=dt)
        tp = torch.from_numpy(plain.view(np.int16)).view(tdt)
        tb = torch.from_numpy(bias.view(np.int16)).view(tdt)
        assert np.array_equal(got, _bits(tp + tb))


def test_row_bias_gelu_epilogue_matches_torch_fp32():
    # not in the reference ("parity unpinned" there): pinned to torch's exact-erf GELU
    rng = np.random.default_rng(10)
    M, N, K = 64, 128, 96
    a, b = _rand_bf16(rng, (M, K)), _rand_bf16(rng, (K, N), K ** -0.5)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float32)
    got = orc.from_bf16(orc.matmul(a, b, bias=bias, epi=orc.EPI_BIAS_ROW_GELU, acc64=True))
    acc = torch.from_numpy(orc.from_bf16(a)).double() @ torch.from_numpy(orc.from_bf16(b)).double()
    want = torch.nn.functional.gelu((acc + torch.from_numpy(bias).double()).float()).to(torch.bfloat16).float().numpy()
    assert np.max(np.abs(got - want)) <= 2.0 ** -7 * np.max(np.abs(want))
    assert np.mean(got != want) < 0.01  # at most the odd 1-ulp flip from erff vs torch erf


def test_leaky_relu_on_the_fp32_accumulator():
    a = orc.to_bf16(np.array([[1.0, -2.0]], dtype=np.float32))
    b = orc.to_bf16(np.array([[3.0], [4.0]], dtype=np.float32))
    got = orc.from_bf16(orc.matmul(a, b, BM=32, BN=32, BK=32, epi=orc.EPI_LEAKY_RELU))
    assert got[0, 0] == orc.from_bf16(orc.to_bf16(np.array([-0.05], dtype=np.float32)))[0]


def test_fp8_scaled_matmul_is_exact_dequant_then_scale():
    rng = np.random.default_rng(11)
    M, N, K = 64, 64, 128
    qa, sa = orc.quantize_fp8(rng.standard_normal((M, K)).astype(np.float32))
    qb, sb = orc.quantize_fp8(rng.standard_normal((K, N)).astype(np.float32))
    assert np.max(np.abs(orc.from_fp8(qa))) == 448.0
    got = orc.from_bf16(orc.matmul(qa, qb, in_dt=orc.FP8E4M3, out_dt=orc.BF16, scale=sa * sb, acc64=True))
    want = (orc.from_fp8(qa).astype(np.float64) @ orc.from_fp8(qb).astype(np.float64)) * (np.float32(sa * sb))
    assert np.array_equal(got, orc.from_bf16(orc.to_bf16(want.astype(np.float32))))
