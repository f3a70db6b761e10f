"""GPU parity: _attn_fwd through the launcher and the C ABI against the CPU oracle.
Tolerances: O max-abs <= 2e-2 (bf16 rounding of P dominates), M (base-2 LSE) max-abs <= 1e-3."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from triton_tenstorrent_amd import kernels as K
from util import bits, decode

pytestmark = pytest.mark.gpu
O_ATOL, M_ATOL = 2e-2, 1e-3


def _qkv(Z, H, S, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(Z, H, S, D, generator=g).to(torch.bfloat16) for _ in range(3)]


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Z,H,S,D", [(1, 2, 128, 64), (2, 3, 256, 128), (1, 1, 512, 32), (1, 2, 384, 16), (1, 1, 128, 256)])
def test_attention_vs_oracle(causal, Z, H, S, D):
    q, k, v = _qkv(Z, H, S, D)
    sm = D ** -0.5
    o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), causal, sm, return_lse=True)
    bn = min(64, D)
    wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), sm, causal=causal, BLOCK_M=128 if S % 128 == 0 else 64, BLOCK_N=bn)
    assert np.max(np.abs(decode(o) - orc.from_bf16(wo))) <= O_ATOL
    assert np.max(np.abs(M.cpu().numpy() - wM)) <= M_ATOL


def test_attention_matches_reference_pytest_config_32x32():
    # the reference's single testing config: BLOCK_M = BLOCK_N = 32 (06-fused-attention.py:117-121)
    q, k, v = _qkv(1, 2, 256, 64, seed=1)
    o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), True, 0.125, return_lse=True, BLOCK_M=32, BLOCK_N=32)
    wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), 0.125, causal=True, BLOCK_M=32, BLOCK_N=32)
    assert np.max(np.abs(decode(o) - orc.from_bf16(wo))) <= O_ATOL and np.max(np.abs(M.cpu().numpy() - wM)) <= M_ATOL


def test_causal_closed_forms():
    q, k, v = _qkv(1, 2, 256, 64, seed=2)
    o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), True, 0.3, return_lse=True)
    # row 0 sees key 0 only
    assert torch.equal(o[:, :, 0].cpu(), v[:, :, 0])
    dot = (q[:, :, 0].double() * k[:, :, 0].double()).sum(-1)
    assert torch.allclose(M[:, :, 0].cpu().double(), dot * 0.3 * 1.44269504, rtol=1e-5, atol=1e-5)
    # uniform keys: running mean of V, M = log2(i+1)
    kz = torch.zeros_like(k)
    o, M = K.attention(q.cuda(), kz.cuda(), v.cuda(), True, 1.0, return_lse=True)
    mean = torch.cumsum(v.double(), 2) / torch.arange(1, 257).double()[None, None, :, None]
    assert (o.cpu().double() - mean).abs().max() <= O_ATOL
    assert torch.allclose(M.cpu(), torch.log2(torch.arange(1, 257).float()).expand(1, 2, 256), atol=1e-5)


def test_partial_grid_produces_only_its_rows_and_heads():
    q, k, v = _qkv(1, 3, 256, 64, seed=3)
    from triton_tenstorrent_amd.tensor_descriptor import TensorDescriptor as TD
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    o = torch.full_like(qc, 7.5)
    M = torch.full((1, 3, 256), -3.0, device="cuda")
    y = 3 * 256
    dq, dk, dv, do = (TD(t, [y, 64], [64, 1], [1, 1]) for t in (qc, kc, vc, o))
    K._attn_fwd[(2, 2, 1)](0.125, M, 1, 3, dq, dk, dv, do, N_CTX=256, HEAD_DIM=64, BLOCK_M=64, BLOCK_N=64,
                           FP8_OUTPUT=False, STAGE=3, warp_specialize=False, IS_HOPPER=False)
    wo = np.full((1, 3, 256, 64), 0x40F0, dtype=np.uint16)
    wM = np.full((1, 3, 256), -3.0, dtype=np.float32)
    orc.attn_fwd(bits(q), bits(k), bits(v), 0.125, causal=True, BLOCK_M=64, BLOCK_N=64, grid=(2, 2), o=wo, M=wM)
    touched = wo != 0x40F0
    assert np.array_equal(bits(o) != 0x40F0, touched)
    assert np.max(np.abs(decode(o)[touched] - orc.from_bf16(wo)[touched])) <= O_ATOL
    assert np.array_equal(M.cpu().numpy() == -3.0, wM == -3.0)


def test_attention_errors():
    q, k, v = _qkv(1, 1, 128, 64)
    with pytest.raises(ValueError):
        K.attention(q.cuda(), k.cuda(), v.cuda(), True, 1.0, BLOCK_M=64, BLOCK_N=128)  # BLOCK_N > HEAD_DIM
    with pytest.raises(NotImplementedError):
        K.attention(q.cuda().half(), k.cuda().half(), v.cuda().half(), True, 1.0)
    q2, k2, v2 = _qkv(1, 1, 96, 64)
    with pytest.raises(NotImplementedError):
        K.attention(q2.cuda(), k2.cuda(), v2.cuda(), True, 1.0, BLOCK_M=64, BLOCK_N=64)  # N_CTX % BLOCK_M
