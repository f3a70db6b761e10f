"""Pins the oracle's fused-attention forward against what the mathematics
fixes: float64 softmax attention, closed-form rows, the base-2 LSE identity."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc


def _qkv(seed, Z, H, S, D, scale=1.0):
    rng = np.random.default_rng(seed)
    return [orc.to_bf16((rng.standard_normal((Z, H, S, D)) * scale).astype(np.float32)) for _ in range(3)]


def _textbook(q, k, v, sm_scale, causal):
    qf, kf, vf = (orc.from_bf16(t).astype(np.float64) for t in (q, k, v))
    s = np.einsum("zhid,zhjd->zhij", qf, kf) * sm_scale
    if causal:
        S = s.shape[-1]
        s = np.where(np.tril(np.ones((S, S), dtype=bool)), s, -np.inf)
    m = s.max(-1, keepdims=True)
    p = np.exp(s - m)
    l = p.sum(-1, keepdims=True)
    o = (p / l) @ vf
    lse2 = (m[..., 0] + np.log(l[..., 0])) / np.log(2.0)  # base-2 log-sum-exp of the scaled scores
    return o, lse2


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("BM,BN", [(32, 32), (64, 32), (64, 64), (128, 64)])
def test_attention_matches_float64_softmax_attention(causal, BM, BN):
    Z, H, S, D = 1, 2, 256, 64
    q, k, v = _qkv(0, Z, H, S, D)
    sm = D ** -0.5
    o, M = orc.attn_fwd(q, k, v, sm, causal=causal, BLOCK_M=BM, BLOCK_N=BN)
    wo, wM = _textbook(q, k, v, sm, causal)
    assert np.max(np.abs(orc.from_bf16(o) - wo)) <= 2e-2   # bf16 P rounding dominates
    assert np.max(np.abs(M - wM)) <= 1e-3
    assert orc.pcc(wo, orc.from_bf16(o)) > 0.9999


def test_non_causal_vs_torch_sdpa():
    Z, H, S, D = 2, 2, 128, 32
    q, k, v = _qkv(1, Z, H, S, D)
    tq, tk, tv = (torch.from_numpy(orc.from_bf16(t)) for t in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, scale=0.25).numpy()
    o, _ = orc.attn_fwd(q, k, v, 0.25, causal=False, BLOCK_M=32, BLOCK_N=32)
    assert np.max(np.abs(orc.from_bf16(o) - want)) <= 2e-2


def test_causal_row0_closed_form():
    # row 0 attends to key 0 only: O[0] = bf16(V[0]) and M[0] = qk_scale * q0.k0
    Z, H, S, D = 1, 3, 64, 32
    q, k, v = _qkv(2, Z, H, S, D)
    sm = 0.3
    o, M = orc.attn_fwd(q, k, v, sm, causal=True, BLOCK_M=32, BLOCK_N=32)
    assert np.array_equal(o[:, :, 0, :], v[:, :, 0, :])
    dot = np.einsum("zhd,zhd->zh", orc.from_bf16(q)[:, :, 0].astype(np.float64), orc.from_bf16(k)[:, :, 0].astype(np.float64))
    assert np.allclose(M[:, :, 0], dot * sm * 1.44269504, rtol=1e-5, atol=1e-5)


def test_uniform_keys_give_the_running_mean_of_v():
    Z, H, S, D = 1, 1, 128, 32
    q, _, v = _qkv(3, Z, H, S, D)
    k = np.zeros_like(q)  # all scores equal
    o, M = orc.attn_fwd(q, k, v, 1.0, causal=True, BLOCK_M=64, BLOCK_N=32)
    vf = orc.from_bf16(v).astype(np.float64)[0, 0]
    mean = np.cumsum(vf, 0) / np.arange(1, S + 1)[:, None]
    assert np.max(np.abs(orc.from_bf16(o)[0, 0] - mean)) <= 2e-2
    assert np.allclose(M[0, 0], np.log2(np.arange(1, S + 1)), atol=1e-5)


def test_mask_value_is_additive_minus_1e6_not_minus_inf():
    # with scores ~ +2e6 above the band the additive -1e6 no longer hides them: the oracle
    # must reproduce that (06-fused-attention.py:59), a -inf mask would not
    Z, H, S, D = 1, 1, 32, 32
    q = orc.to_bf16(np.zeros((Z, H, S, D), dtype=np.float32))
    k = orc.to_bf16(np.zeros((Z, H, S, D), dtype=np.float32))
    qf = np.zeros((S, D), dtype=np.float32); qf[0, 0] = 2048.0
    kf = np.zeros((S, D), dtype=np.float32); kf[1, 0] = 1024.0   # q0.k1 = 2^21 > 1e6/ (scale*log2e)
    q[0, 0], k[0, 0] = orc.to_bf16(qf), orc.to_bf16(kf)
    v = orc.to_bf16(np.arange(S * D, dtype=np.float32).reshape(1, 1, S, D) % 7)
    o, _ = orc.attn_fwd(q, k, v, 1.0, causal=True, BLOCK_M=32, BLOCK_N=32)
    assert np.array_equal(o[0, 0, 0], v[0, 0, 1]), "row 0 must leak to the masked key 1"


def test_result_does_not_depend_on_workers_and_grid_subset():
    Z, H, S, D = 1, 2, 128, 32
    q, k, v = _qkv(4, Z, H, S, D)
    o1, M1 = orc.attn_fwd(q, k, v, 0.2, BLOCK_M=32, BLOCK_N=32, nthreads=1)
    o8, M8 = orc.attn_fwd(q, k, v, 0.2, BLOCK_M=32, BLOCK_N=32, nthreads=5)
    assert np.array_equal(o1, o8) and np.array_equal(M1, M8)
    o = np.full_like(q, 0x40F0)
    orc.attn_fwd(q, k, v, 0.2, BLOCK_M=32, BLOCK_N=32, grid=(2, 1), o=o)
    assert np.array_equal(o[0, 0, :64], o1[0, 0, :64]) and np.all(o[0, 0, 64:] == 0x40F0) and np.all(o[0, 1] == 0x40F0)


def test_rejects_block_n_above_head_dim():
    q, k, v = _qkv(5, 1, 1, 64, 32)
    with pytest.raises(ValueError):
        orc.attn_fwd(q, k, v, 1.0, BLOCK_M=64, BLOCK_N=64)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("BM,BN", [(32, 32), (64, 32)])
def test_p_is_rounded_to_bf16_and_l_is_summed_before_the_cast(causal, BM, BN):
    """06-fused-attention.py:65-83: l_ij = sum(p) in fp32, then p.to(bf16) feeds the second dot.  On the constructed
    input an oracle that left P in fp32 puts 0.2-1.7 into the last row of O where the source gives 0, and one that
    summed l after the cast moves M by 5e-3."""
    from util import p_cast_case
    S, D = 64, 32
    q, k, v, sm, models = p_cast_case(S, D)
    o, M = orc.attn_fwd(q, k, v, sm, causal=causal, BLOCK_M=BM, BLOCK_N=BN)
    o, M = orc.from_bf16(o)[0, 0], M[0, 0]
    wo, wM = models[("faithful", causal)]
    assert np.all(np.abs(o - wo) <= 2.0 ** -8 * np.abs(wo) + 2e-2) and np.max(np.abs(M - wM)) <= 1e-3
    assert np.all(o[-1] == 0.0)
    # the construction discriminates: each wrong reading is far outside those bars
    assert np.min(np.abs(models[("p_not_rounded", causal)][0][-1])) > 0.2
    assert abs(models[("l_after_cast", causal)][1][-1] - wM[-1]) > 4e-3
