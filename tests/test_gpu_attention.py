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


# ---- the 256-query / 64-key tile fast path ---------------------------------
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Z,H,S,D", [(1, 2, 256, 128), (2, 2, 512, 128), (1, 3, 768, 64), (1, 1, 1024, 128), (2, 2, 512, 32),
                                     (1, 1, 1024, 32), (1, 2, 256, 256), (2, 1, 640, 256)])
def test_fast_attention_vs_oracle(causal, Z, H, S, D):
    from triton_tenstorrent_amd import runtime as rt
    q, k, v = _qkv(Z, H, S, D, seed=S + D)
    sm = D ** -0.5
    o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), causal, sm, return_lse=True)
    assert rt.last_kernel_name() == f"attn_tile_d{D}", rt.last_kernel_name()
    wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), sm, causal=causal, BLOCK_M=128, BLOCK_N=min(64, D))
    assert np.max(np.abs(decode(o) - orc.from_bf16(wo))) <= O_ATOL
    assert np.max(np.abs(M.cpu().numpy() - wM)) <= M_ATOL


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Z,H,S,D", [(1, 2, 32, 128), (2, 2, 96, 64), (1, 3, 160, 128), (1, 2, 288, 128), (1, 2, 480, 64),
                                     (1, 1, 992, 128), (1, 1, 4064, 128), (1, 2, 32, 32), (2, 1, 352, 32),
                                     (1, 2, 160, 256), (1, 1, 864, 256)])
def test_fast_attention_ragged_sequence_lengths(causal, Z, H, S, D):
    # N_CTX in whole wavefronts of 32 queries but not whole 256-query blocks: the fast kernel with a clipped tail.
    # q, k, v end exactly where a buffer of NaN begins: a fetch past the last head's rows would show
    from triton_tenstorrent_amd import runtime as rt
    g = torch.Generator().manual_seed(S + D + causal)
    rows = Z * H * S
    bufs = []
    for _ in range(3):
        buf = torch.full((rows + 64, D), float("nan"), dtype=torch.bfloat16)
        buf[:rows] = torch.randn(rows, D, generator=g).to(torch.bfloat16)
        bufs.append(buf)
    q, k, v = (b.cuda()[:rows].view(Z, H, S, D) for b in bufs)
    sm = D ** -0.5
    o, M = K.attention(q, k, v, causal, sm, return_lse=True)
    assert rt.last_kernel_name() == f"attn_ragged_d{D}", rt.last_kernel_name()
    bm = 32 if S % 64 else 64
    wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), sm, causal=causal, BLOCK_M=bm, BLOCK_N=min(bm, 64, D))
    assert np.max(np.abs(decode(o) - orc.from_bf16(wo))) <= O_ATOL
    assert np.max(np.abs(M.cpu().numpy() - wM)) <= M_ATOL


def test_fast_attention_random_lengths_and_head_dims():
    # a seeded sweep: N_CTX any multiple of 32 up to 800, every head dim of the fast kernel, both mask modes
    from triton_tenstorrent_amd import runtime as rt
    rng = np.random.default_rng(31)
    for case in range(16):
        D = int(rng.choice([32, 64, 128, 256]))
        S = 32 * int(rng.integers(1, 26))
        Z, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        causal = bool(case % 2)
        q, k, v = _qkv(Z, H, S, D, seed=100 + case)
        sm = D ** -0.5
        o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), causal, sm, return_lse=True)
        per_wg = 128 if D == 256 else 256
        assert rt.last_kernel_name() == f"attn_{'tile' if S % per_wg == 0 else 'ragged'}_d{D}", (S, D)
        bm = 128 if S % 128 == 0 else (64 if S % 64 == 0 else 32)
        wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), sm, causal=causal, BLOCK_M=bm, BLOCK_N=min(bm, 64, D))
        assert np.max(np.abs(decode(o) - orc.from_bf16(wo))) <= O_ATOL, (Z, H, S, D, causal)
        assert np.max(np.abs(M.cpu().numpy() - wM)) <= M_ATOL, (Z, H, S, D, causal)


def test_fast_attention_closed_forms_and_any_path_agreement():
    from triton_tenstorrent_amd import runtime as rt
    q, k, v = _qkv(1, 2, 512, 128, seed=7)
    o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), True, 0.3, return_lse=True)
    assert rt.last_kernel_name() == "attn_tile_d128"
    assert torch.equal(o[:, :, 0].cpu(), v[:, :, 0])      # row 0 sees key 0 only
    kz = torch.zeros_like(k)
    o2, M2 = K.attention(q.cuda(), kz.cuda(), v.cuda(), True, 1.0, return_lse=True)
    mean = torch.cumsum(v.double(), 2) / torch.arange(1, 513).double()[None, None, :, None]
    assert (o2.cpu().double() - mean).abs().max() <= O_ATOL
    assert torch.allclose(M2.cpu(), torch.log2(torch.arange(1, 513).float()).expand(1, 2, 512), atol=1e-5)
    # a one-hot V column picks out P itself: every probability row sums to 1
    ones = torch.ones_like(v)
    o3 = K.attention(q.cuda(), k.cuda(), ones.cuda(), True, 0.3)
    assert (o3.float() - 1).abs().max() <= 1e-2


def test_full_size_attention_properties():
    """BASELINE's 4x32x4096x128 causal config through size-independent properties: row 0 of every
    head copies V[0]; V = ones gives ones; sampled heads against the oracle on a 512-row prefix
    (causal attention of a prefix does not depend on what follows it)."""
    from triton_tenstorrent_amd import runtime as rt
    Z, H, S, D = 4, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(Z, H, S, D, device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
    sm = D ** -0.5
    o, M = K.attention(q, k, v, True, sm, return_lse=True)
    assert rt.last_kernel_name() == "attn_tile_d128"
    assert torch.equal(o[:, :, 0], v[:, :, 0])
    for (z, h) in [(0, 0), (3, 31), (1, 17)]:
        qs, ks, vs = (t[z:z + 1, h:h + 1, :512].contiguous().cpu() for t in (q, k, v))
        wo, wM = orc.attn_fwd(bits(qs), bits(ks), bits(vs), sm, causal=True, BLOCK_M=128, BLOCK_N=64)
        assert np.max(np.abs(decode(o[z:z + 1, h:h + 1, :512]) - orc.from_bf16(wo))) <= O_ATOL
        assert np.max(np.abs(M[z:z + 1, h:h + 1, :512].cpu().numpy() - wM)) <= M_ATOL
    # last rows against float64 attention over the full context, two heads
    for (z, h) in [(2, 5), (0, 31)]:
        qf, kf, vf = q[z, h, -64:].double(), k[z, h].double(), v[z, h].double()
        s = qf @ kf.T * sm
        mask = torch.arange(S - 64, S, device="cuda")[:, None] >= torch.arange(S, device="cuda")[None, :]
        s = s.masked_fill(~mask, float("-inf"))
        ref = torch.softmax(s, -1) @ vf
        assert (o[z, h, -64:].double() - ref).abs().max() <= O_ATOL
        lse2 = torch.logsumexp(s, -1) / np.log(2.0)
        assert (M[z, h, -64:].double() - lse2).abs().max() <= M_ATOL
    del o, M
    o1 = K.attention(q, k, torch.ones_like(v), True, sm)
    assert (o1.float() - 1).abs().max() <= 1e-2


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("S,D,kernel", [(256, 128, "attn_tile_d128"), (256, 64, "attn_tile_d64"), (224, 128, "attn_ragged_d128"),
                                        (128, 256, "attn_tile_d256"), (64, 16, "attn_any_d16")])
def test_p_is_rounded_to_bf16_and_l_is_summed_before_the_cast(causal, S, D, kernel):
    """06-fused-attention.py:65-83 on the constructed input of util.p_cast_case: a kernel that fed fp32 P into the
    second product would put 0.2-1.7 where the last row of O is exactly 0, and one that summed l after the cast would
    move M by 5e-3 (the bar is 1e-3)."""
    from triton_tenstorrent_amd import runtime as rt
    from util import from_bits, p_cast_case
    q, k, v, sm, models = p_cast_case(S, D)
    tq, tk, tv = (from_bits(t, torch.bfloat16) for t in (q, k, v))
    o, M = K.attention(tq, tk, tv, causal, sm, return_lse=True)
    assert rt.last_kernel_name() == kernel
    wo, wM = models[("faithful", causal)]
    o, M = decode(o)[0, 0], M.cpu().numpy()[0, 0]
    assert np.all(np.abs(o - wo) <= 2.0 ** -8 * np.abs(wo) + O_ATOL) and np.max(np.abs(M - wM)) <= M_ATOL
    assert np.all(o[-1] == 0.0)
    bm = 32 if S % 64 else 64
    ro, rM = orc.attn_fwd(q, k, v, sm, causal=causal, BLOCK_M=bm, BLOCK_N=min(bm, D))
    assert np.all(np.abs(o - orc.from_bf16(ro)[0, 0]) <= 2.0 ** -8 * np.abs(wo) + O_ATOL) and np.max(np.abs(M - rM[0, 0])) <= M_ATOL


@pytest.mark.parametrize("S,D,kernel", [(256, 128, "attn_tile_d128"), (512, 128, "attn_tile_d128"), (224, 128, "attn_ragged_d128"),
                                        (256, 64, "attn_tile_d64"), (128, 256, "attn_tile_d256"), (128, 16, "attn_any_d16")])
def test_causal_mask_is_the_sources_at_block_m_32(S, D, kernel):
    """The source masks with an ADDITIVE -1.0e6 inside the diagonal block (06-fused-attention.py:58-59), so a masked
    score more than 1e6 above the unmasked ones leaks.  The kernels evaluate the mask as the source does at
    BLOCK_M = 32, whatever BLOCK_M the launch names: row 40 against key 41 (same 32x32 tile, 2^21 * log2e above the
    rest) leaks exactly as in the oracle; row 70 against key 100 (a later tile) does not, where the source at
    BLOCK_M = 128 would leak too.  Both stated in the kernels' headers."""
    from triton_tenstorrent_amd import runtime as rt
    g = torch.Generator().manual_seed(S + D)
    q = torch.zeros(1, 1, S, D)
    k = torch.zeros(1, 1, S, D)
    q[0, 0, 40, 0], k[0, 0, 41, 0] = 2048.0, 1024.0
    q[0, 0, 70, 1], k[0, 0, 100, 1] = 2048.0, 1024.0
    v = torch.randn(1, 1, S, D, generator=g)
    q, k, v = (t.to(torch.bfloat16) for t in (q, k, v))
    wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), 1.0, causal=True, BLOCK_M=32, BLOCK_N=min(32, D))
    wo = orc.from_bf16(wo)
    assert np.array_equal(wo[0, 0, 40], decode(v)[0, 0, 41])                       # the oracle leaks inside the tile
    for bm in (32, 64, 128):
        if S % bm:
            continue
        o, M = K.attention(q.cuda(), k.cuda(), v.cuda(), True, 1.0, return_lse=True, BLOCK_M=bm, BLOCK_N=min(32, D))
        assert rt.last_kernel_name() == kernel
        assert np.max(np.abs(decode(o) - wo)) <= O_ATOL and np.max(np.abs(M.cpu().numpy() - wM)) <= M_ATOL * max(1.0, 2.0 ** 21 * 2 ** -20)
        assert torch.equal(o[0, 0, 40].cpu(), v[0, 0, 41])                         # row 40 copies the masked key's value
        mean70 = v[0, 0, :71].double().mean(0)
        assert (o[0, 0, 70].cpu().double() - mean70).abs().max() <= O_ATOL          # row 70 does not see key 100
    if S % 128 == 0:
        # the stated difference: at BLOCK_M = 128 the source itself would leak row 70 to key 100
        o128, _ = orc.attn_fwd(bits(q), bits(k), bits(v), 1.0, causal=True, BLOCK_M=128, BLOCK_N=min(32, D))
        assert np.array_equal(orc.from_bf16(o128)[0, 0, 70], decode(v)[0, 0, 100])


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Z,H,S,D", [(2, 32, 2304, 128), (1, 40, 3328, 128), (3, 3, 768, 128), (2, 32, 2272, 128),
                                     (1, 33, 4000, 128), (5, 8, 1056, 128), (2, 32, 2304, 64), (3, 11, 3328, 64), (1, 5, 512, 64),
                                     (2, 32, 1152, 256), (1, 40, 1664, 256), (3, 3, 384, 256), (1, 5, 128, 256),
                                     (2, 32, 1056, 256), (1, 33, 2016, 256), (5, 8, 544, 256), (1, 3, 32, 256), (2, 3, 96, 256),
                                     (2, 32, 2272, 64), (1, 33, 4000, 64), (5, 8, 1056, 64), (1, 3, 32, 64), (2, 3, 96, 64), (1, 2, 224, 64)])
def test_items_chained_inside_a_workgroup(causal, Z, H, S, D):
    """The head dim 128, 64 and 256 kernels walk (head, pair of query blocks) items on a persistent grid (256-query blocks;
    128-query blocks at head dim 256) and let each item's last
    copies fetch the first key blocks of the next one, which may belong to another head.  Shapes with more items
    than CUs (288 and 280 against 256), an odd number of query blocks (9, 13: the middle block is an item on its own,
    so items of one and of two blocks alternate), a head count that is not a multiple of 8, and lengths that are not
    whole 256-query blocks (the last block's wavefronts past the end only keep up with the barriers, and the stream of
    an item is padded to whole turns of the stage ring); every row of sampled
    heads and of the heads where a workgroup changes head, against float64."""
    from triton_tenstorrent_amd import runtime as rt
    g = torch.Generator(device="cuda").manual_seed(Z * 1000 + S)
    q, k, v = (torch.randn(Z, H, S, D, device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
    # every head gets its own offset in V, so that output rows computed from another head's keys or values show
    v = (v.float() + torch.arange(Z * H, device="cuda").view(Z, H, 1, 1).float() * 0.25).to(torch.bfloat16)
    sm = D ** -0.5
    o, M = K.attention(q, k, v, causal, sm, return_lse=True)
    assert rt.last_kernel_name() == (f"attn_tile_d{D}" if S % (128 if D == 256 else 256) == 0 else f"attn_ragged_d{D}")
    heads = sorted({0, 1, Z * H // 2, Z * H - 2, Z * H - 1, 7, 8} & set(range(Z * H)))
    rows = torch.arange(S, device="cuda")
    for hh in heads:
        z, h = divmod(hh, H)
        s = (q[z, h].double() @ k[z, h].double().T) * sm
        if causal:
            s = s.masked_fill(rows[:, None] < rows[None, :], float("-inf"))
        ref = torch.softmax(s, -1) @ v[z, h].double()
        assert (o[z, h].double() - ref).abs().max() <= O_ATOL * max(1.0, float(v[z, h].float().abs().max()))
        assert (M[z, h].double() - torch.logsumexp(s, -1) / np.log(2.0)).abs().max() <= M_ATOL


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("S,D,kernel", [(1024, 128, "attn_tile_d128"), (1024, 256, "attn_tile_d256"), (1024, 64, "attn_tile_d64")])
def test_row_maxima_that_climb_slowly_and_in_jumps(causal, S, D, kernel):
    """The pipelined kernels keep a row's exponent reference until some row of the wavefront outgrows it by 2^8 and
    only then rescale (a stated difference from a literal evaluation).  Scores that rise by 0.1 log2 units per key
    (6.4 per 64-key block: several blocks pass between two rescales, and p reaches 2^8 in between), with a jump of 60
    units at key 700 and another of 20 at key 900, against float64."""
    from triton_tenstorrent_amd import runtime as rt
    g = torch.Generator().manual_seed(S + D)
    q = torch.randn(1, 2, S, D, generator=g) * 0.05
    k = torch.randn(1, 2, S, D, generator=g) * 0.05
    ramp = 0.1 / 1.44269504 * torch.arange(S).float()
    ramp[700:] += 60 / 1.44269504
    ramp[900:] += 20 / 1.44269504
    q[..., 0] = 1.0
    k[..., 0] = ramp
    v = torch.randn(1, 2, S, D, generator=g)
    q, k, v = (t.to(torch.bfloat16).cuda() for t in (q, k, v))
    o, M = K.attention(q, k, v, causal, 1.0, return_lse=True)
    assert rt.last_kernel_name() == kernel
    rows = torch.arange(S, device="cuda")
    for h in range(2):
        s_ = q[0, h].double() @ k[0, h].double().T
        if causal:
            s_ = s_.masked_fill(rows[:, None] < rows[None, :], float("-inf"))
        ref = torch.softmax(s_, -1) @ v[0, h].double()
        assert (o[0, h].double() - ref).abs().max() <= O_ATOL
        assert (M[0, h].double() - torch.logsumexp(s_, -1) / np.log(2.0)).abs().max() <= M_ATOL


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Z,H,S,sm", [(3, 2, 1216, 0.125), (2, 4, 1184, 0.0625), (1, 6, 160, 0.125), (2, 3, 1152, 0.125)])
def test_the_wavefront_that_ends_an_item_reads_finished_accumulators(causal, Z, H, S, sm):
    """Head dim 256.  The last wavefront of a full 128-query block runs its last block period and goes straight to
    the epilogue, with no idle period in between; in the other periods outside the main loop (a number of key blocks
    that is not a multiple of four leaves up to three) the compiler may move accumulator tiles between register
    sets.  Wherever such a read follows the MFMA that writes the tile, the MFMA carries its wait states itself.
    A length with nine full blocks and a part (every block but the last is full while the launch takes the ragged
    kernel), one more ragged length, a short one and a whole one: every row of every head against float64, and three
    launches on the same operands give the same bits."""
    from triton_tenstorrent_amd import runtime as rt
    g = torch.Generator(device="cuda").manual_seed(S + Z)
    q, k, v = (torch.randn(Z, H, S, 256, device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
    o, M = K.attention(q, k, v, causal, sm, return_lse=True)
    assert rt.last_kernel_name() == ("attn_tile_d256" if S % 128 == 0 else "attn_ragged_d256")
    for _ in range(2):
        o2, M2 = K.attention(q, k, v, causal, sm, return_lse=True)
        assert torch.equal(o2, o) and torch.equal(M2, M)
    s = (q.double() @ k.double().transpose(-1, -2)) * sm
    if causal:
        rows = torch.arange(S, device="cuda")
        s = s.masked_fill(rows[:, None] < rows[None, :], float("-inf"))
    ref = torch.softmax(s, -1) @ v.double()
    assert (o.double() - ref).abs().max() <= O_ATOL
    assert (M.double() - torch.logsumexp(s, -1) / np.log(2.0)).abs().max() <= M_ATOL


def test_repeat_launches_take_the_cached_path_and_keep_the_checks():
    """From the second call of a shape on, `_attn_fwd` is launched through a cached closure (N_CTX and the block
    sizes arrive by keyword and are part of what makes two calls alike).  Batch, heads, operands and the mask may
    change under it; whatever it does not recognise falls back to the full path."""
    Z, H, S, D = 2, 3, 256, 128
    q, k, v = (t.cuda() for t in _qkv(Z, H, S, D, seed=3))
    sm = D ** -0.5
    first_o, first_m = K.attention(q, k, v, True, sm, return_lse=True)
    for _ in range(2):
        o, m = K.attention(q, k, v, True, sm, return_lse=True)
        assert torch.equal(o, first_o) and torch.equal(m, first_m)
    assert K._attn_fwd._plan is not None
    wo, wM = orc.attn_fwd(bits(q.cpu()), bits(k.cpu()), bits(v.cpu()), sm, causal=True, BLOCK_M=128, BLOCK_N=64)
    assert np.max(np.abs(decode(first_o) - orc.from_bf16(wo))) <= O_ATOL
    assert np.max(np.abs(first_m.cpu().numpy() - wM)) <= M_ATOL
    # other operands, one head of one batch (Z = H = 1: values that Triton folds), the other mask, another length
    q1, k1, v1 = q[:1, :1].contiguous(), k[:1, :1].contiguous(), v[:1, :1].contiguous()
    o1 = K.attention(q1, k1, v1, True, sm)
    assert torch.equal(o1, first_o[:1, :1])
    of = K.attention(q, k, v, False, sm)
    wo, _ = orc.attn_fwd(bits(q.cpu()), bits(k.cpu()), bits(v.cpu()), sm, causal=False, BLOCK_M=128, BLOCK_N=64)
    assert np.max(np.abs(decode(of) - orc.from_bf16(wo))) <= O_ATOL
    q2, k2, v2 = (t.cuda() for t in _qkv(1, 2, 384, D, seed=4))
    o2 = K.attention(q2, k2, v2, True, sm)
    wo, _ = orc.attn_fwd(bits(q2.cpu()), bits(k2.cpu()), bits(v2.cpu()), sm, causal=True, BLOCK_M=128, BLOCK_N=64)
    assert np.max(np.abs(decode(o2) - orc.from_bf16(wo))) <= O_ATOL
    assert torch.equal(K.attention(q, k, v, True, sm), first_o)
    # and the same refusals
    with pytest.raises(NotImplementedError):
        K.attention(q.half(), k.half(), v.half(), True, sm)
    assert torch.equal(K.attention(q, k, v, True, sm), first_o)
