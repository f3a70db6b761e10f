"""matmul_kernel on tile-major buffers (examples/matmul/03-matrix-multiplication.py:242-391) through
the launcher and the C ABI, against the oracle's restatement."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(shape, generator=g) - 0.5).to(dtype)


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _f16(buf_u16):
    return buf_u16.view(np.float16).astype(np.float32)


def _close(got, ref):
    # the tile-matmul bar: |err| <= 1e-2*|ref| + 1e-4 against the fp64-accumulating oracle
    return np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-4)


@pytest.mark.parametrize("M,N,K_,cfg", [
    (32, 32, 64, {}),                                               # the reference's self-check shape
    (70, 45, 50, {}),                                               # ragged in all three
    (128, 192, 96, {"BLOCK_SIZE_M": 64, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 4}),
    (33, 31, 17, {"BLOCK_SIZE_M": 32, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 16}),
    (257, 31, 33, {}), (300, 333, 200, {}), (1000, 1000, 1000, {}), (256, 256, 96, {}),   # the clamping fast kernel
])
@pytest.mark.parametrize("act", ["", "leaky_relu"])
def test_tiled_matmul_vs_oracle(M, N, K_, cfg, act):
    c = {**K.MATMUL_POINTER_CONFIG, **cfg}
    BM, BN, BK = c["BLOCK_SIZE_M"], c["BLOCK_SIZE_N"], c["BLOCK_SIZE_K"]
    a, b = _rand((M, K_), 1), _rand((K_, N), 2)
    at, bt = K.tilize(a, BM, BK), K.tilize(b, BK, BN)
    assert np.array_equal(_bits(at), orc.tilize(_bits(a), BM, BK))          # same tiling as the oracle's
    ct = K.matmul_tiled(at.cuda(), bt.cuda(), M, N, K_, activation=act, **cfg)
    # the reference's 32x32x32 tiling takes the fast kernel's clamping instantiation, other tilings the any-shape one
    assert rt.last_kernel_name() == (f"gemm_tiledragged_f16_epi{3 if act else 0}" if not cfg else "gemm_anytiled_f16_f16")
    ref = orc.matmul_tiled(_bits(at), _bits(bt), M, N, K_, in_dt=orc.F16, BM=BM, BN=BN, BK=BK,
                           group_m=c["GROUP_SIZE_M"], leaky_relu=bool(act), acc64=True)
    got = _bits(ct.cpu())
    gm, rm = orc.untilize(got, M, N, BM, BN), orc.untilize(ref, M, N, BM, BN)
    assert _close(_f16(gm), _f16(rm))
    # the reference's own bar for this kernel: atol 1e-2 against a plain matmul (:438)
    want = a.double() @ b.double()
    want = torch.where(want >= 0, want, 0.01 * want) if act else want
    assert np.max(np.abs(_f16(gm) - want.numpy())) <= 1e-2
    assert torch.equal(K.untilize(ct.cpu(), M, N, BM, BN).view(torch.int16), torch.from_numpy(gm.view(np.int16)))


def test_tiled_matmul_small_integers_are_exact_and_padding_is_untouched():
    M, N, K_ = 70, 45, 50
    g = torch.Generator().manual_seed(3)
    a = torch.randint(-4, 5, (M, K_), generator=g).to(torch.float16)
    b = torch.randint(-4, 5, (K_, N), generator=g).to(torch.float16)
    ct = K.matmul_tiled(K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), M, N, K_)
    assert torch.equal(K.untilize(ct.cpu(), M, N, 32, 32).float(), a.float() @ b.float())
    # masked store (:387-388): elements of the padded C tiles beyond M, N are never written
    c = torch.full((3 * 2 * 1024, ), float("nan"), dtype=torch.float16, device="cuda")
    grid = (6, )
    K.matmul_kernel[grid](K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), c, M, N, K_, K_, 1, N, 1, N, 1)
    full = c.cpu().reshape(3, 2, 32, 32).permute(0, 2, 1, 3).reshape(96, 64)
    assert not torch.isnan(full[:M, :N]).any() and torch.isnan(full[M:, :]).all() and torch.isnan(full[:, N:]).all()


def test_tiled_matmul_random_shapes_exact_and_padding_untouched():
    # a seeded sweep over any M, N, K at the reference's 32x32x32 tiling: small integers, bit for bit; the padding of
    # the C tiles keeps the NaN it was filled with
    rng = np.random.default_rng(77)
    for case in range(16):
        M, N, K_ = (int(rng.integers(1, 600)) for _ in range(3))
        g = torch.Generator().manual_seed(case)
        a = torch.randint(-3, 4, (M, K_), generator=g).to(torch.float16)
        b = torch.randint(-3, 4, (K_, N), generator=g).to(torch.float16)
        tm, tn = K.cdiv(M, 32), K.cdiv(N, 32)
        c = torch.full((tm * tn * 1024, ), float("nan"), dtype=torch.float16, device="cuda")
        act = "leaky_relu" if case % 3 == 0 else ""
        K.matmul_kernel[(tm * tn, )](K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), c, M, N, K_, K_, 1, N, 1, N, 1,
                                     ACTIVATION=act)
        whole = M % 256 == 0 and N % 256 == 0 and K_ % 128 == 0
        assert rt.last_kernel_name().startswith("gemm_tiled_f16" if whole else "gemm_tiledragged_f16"), (M, N, K_)
        full = c.cpu().reshape(tm, tn, 32, 32).permute(0, 2, 1, 3).reshape(tm * 32, tn * 32)
        want = a.float() @ b.float()
        if act:
            want = torch.where(want >= 0, want, 0.01 * want)
        assert torch.equal(full[:M, :N], want.to(torch.float16)), (M, N, K_)
        assert torch.isnan(full[M:, :]).all() and torch.isnan(full[:, N:]).all(), (M, N, K_)


@pytest.mark.parametrize("M,N,K_", [(70, 45, 50), (300, 333, 200), (256, 256, 1), (515, 260, 31), (64, 64, 161), (1000, 1000, 1000)])
def test_tiled_matmul_ignores_what_the_padding_holds(M, N, K_):
    """The source masks k >= K to zero and never stores rows >= M or columns >= N (03-matrix-multiplication.py:340-342,
    359-361, 387-388), so the result must not depend on the padding of the tile-major buffers: here it is NaN in A
    (rows past M, columns past K) and in B (rows past K, columns past N), and the result equals the zero-padded one
    bit for bit and meets the bar against the oracle run on the same NaN-padded buffers."""
    a, b = _rand((M, K_), 20), _rand((K_, N), 21)
    Mp, Np, Kp = (K.cdiv(x, 32) * 32 for x in (M, N, K_))
    an = torch.full((Mp, Kp), float("nan"), dtype=torch.float16); an[:M, :K_] = a
    bn = torch.full((Kp, Np), float("nan"), dtype=torch.float16); bn[:K_, :N] = b
    at, bt = K.tilize(an, 32, 32), K.tilize(bn, 32, 32)
    for act in ("", "leaky_relu"):
        ct = K.matmul_tiled(at.cuda(), bt.cuda(), M, N, K_, activation=act)
        assert rt.last_kernel_name() == f"gemm_tiledragged_f16_epi{3 if act else 0}"
        c0 = K.matmul_tiled(K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), M, N, K_, activation=act)
        got, got0 = (orc.untilize(_bits(t.cpu()), M, N, 32, 32) for t in (ct, c0))
        assert np.array_equal(got, got0)
        ref = orc.matmul_tiled(_bits(at), _bits(bt), M, N, K_, leaky_relu=bool(act), acc64=True)
        assert _close(_f16(got), _f16(orc.untilize(ref, M, N, 32, 32)))


def test_tiled_matmul_bf16_inputs_give_fp16():
    M, N, K_ = 64, 96, 128
    a, b = _rand((M, K_), 4, torch.bfloat16), _rand((K_, N), 5, torch.bfloat16)
    ct = K.matmul_tiled(K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), M, N, K_)
    assert ct.dtype == torch.float16 and rt.last_kernel_name() == "gemm_anytiled_bf16_f16"
    ref = orc.matmul_tiled(_bits(K.tilize(a, 32, 32)), _bits(K.tilize(b, 32, 32)), M, N, K_, in_dt=orc.BF16, acc64=True)
    assert _close(_f16(_bits(ct.cpu())), _f16(ref))


def test_partial_grid_and_errors():
    M = N = 64
    a, b = _rand((M, 32), 6), _rand((32, N), 7)
    c = torch.full((4 * 1024, ), float("nan"), dtype=torch.float16, device="cuda")
    K.matmul_kernel[(3, )](K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), c, M, N, 32, 32, 1, N, 1, N, 1)
    assert torch.isnan(c[3 * 1024:]).all() and not torch.isnan(c[:3 * 1024]).any()
    with pytest.raises(rt.InvalidLaunch):
        K.matmul_kernel[(5, )](K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), c, M, N, 32, 32, 1, N, 1, N, 1)
    with pytest.raises(rt.InvalidLaunch):   # the kernel asserts positive strides
        K.matmul_kernel[(4, )](K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), c, M, N, 32, 0, 1, N, 1, N, 1)
    with pytest.raises(rt.Unsupported):
        K.matmul_tiled(K.tilize(a, 48, 32).cuda(), K.tilize(b, 32, 32).cuda(), M, N, 32, BLOCK_SIZE_M=48)


def test_partial_grid_in_a_short_last_group_follows_the_pointer_decode():
    """5x3 tiles in groups of 3: the last group has 2 rows and starts at an odd program id, where the row taken from
    the position inside the group (03-matrix-multiplication.py:281) and the row taken from the program id itself
    (the descriptor kernels) name different tiles.  12 of 15 programs: the oracle and the kernel must leave the same
    three tiles of the result untouched."""
    M, N, K_ = 160, 96, 64
    a, b = _rand((M, K_), 12), _rand((K_, N), 13)
    at, bt = K.tilize(a, 32, 32), K.tilize(b, 32, 32)
    for grid in (10, 12, 14):
        c = torch.full((15 * 1024, ), float("nan"), dtype=torch.float16, device="cuda")
        K.matmul_kernel[(grid, )](at.cuda(), bt.cuda(), c, M, N, K_, K_, 1, N, 1, N, 1, GROUP_SIZE_M=3)
        assert rt.last_kernel_name() == "gemm_anytiled_f16_f16"
        ref = orc.matmul_tiled(_bits(at), _bits(bt), M, N, K_, group_m=3, grid=grid, acc64=True,
                               out=np.full(15 * 1024, 0x7e00, dtype=np.uint16))
        got = _bits(c.cpu())
        untouched = np.isnan(_f16(ref))
        assert np.array_equal(np.isnan(_f16(got)), untouched) and untouched.sum() == (15 - grid) * 1024
        assert _close(_f16(got)[~untouched], _f16(ref)[~untouched])
        if grid == 12:
            # hand-worked: programs 9, 10, 11 are tiles (3,0), (4,0), (3,1); in the tile-major result tile (i,j) is
            # block i*3 + j, so blocks 12 (4,0) and 9, 10 are written and 11, 13, 14 are not
            blocks = {t for t in range(15) if not np.isnan(_f16(got[t * 1024:(t + 1) * 1024])).any()}
            assert blocks == set(range(9)) | {9, 12, 10}


@pytest.mark.parametrize("act", ["", "leaky_relu"])
def test_fast_path_tiled(act):
    M, N, K_ = 512, 768, 256
    a, b = _rand((M, K_), 8), _rand((K_, N), 9)
    at, bt = K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda()
    ct = K.matmul_tiled(at, bt, M, N, K_, activation=act)
    assert rt.last_kernel_name() == ("gemm_tiled_f16_epi3" if act else "gemm_tiled_f16_epi0")
    ref = orc.matmul_tiled(_bits(at.cpu()), _bits(bt.cpu()), M, N, K_, leaky_relu=bool(act), acc64=True)
    assert _close(_f16(_bits(ct.cpu())), _f16(ref))
    # and the reference wrapper on whole tiles: tensors handed over as they lie in memory
    c2 = K.matmul(at.reshape(M, K_), bt.reshape(K_, N), activation=act)
    assert torch.equal(c2.reshape(-1), ct)


def test_fast_path_tiled_small_integers_exact_and_equal_to_any_path():
    M, N, K_ = 256, 512, 384
    g = torch.Generator().manual_seed(10)
    a = torch.randint(-3, 4, (M, K_), generator=g).to(torch.float16)
    b = torch.randint(-3, 4, (K_, N), generator=g).to(torch.float16)
    at, bt = K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda()
    ct = K.matmul_tiled(at, bt, M, N, K_)
    assert rt.last_kernel_name() == "gemm_tiled_f16_epi0"
    assert torch.equal(K.untilize(ct.cpu(), M, N, 32, 32).float(), a.float() @ b.float())
    # one program short of the full grid takes the any-shape kernel; with GROUP_SIZE_M = 1 program p writes
    # tile p of the tile-major result, so all tiles but the last must agree bit for bit
    tiles = (M // 32) * (N // 32)
    ca = torch.zeros_like(ct)
    K.matmul_kernel[(tiles - 1, )](at, bt, ca, M, N, K_, K_, 1, N, 1, N, 1)
    assert rt.last_kernel_name() == "gemm_anytiled_f16_f16"
    assert torch.equal(ca[:(tiles - 1) * 1024], ct[:(tiles - 1) * 1024]) and not ca[(tiles - 1) * 1024:].any()


def test_full_size_tiled_identity_and_scaling():
    # 8192^3 through size-independent properties: B = I gives C = A bit for bit; 2A gives 2C
    n = 8192
    g = torch.Generator(device="cuda").manual_seed(11)
    a = ((torch.rand((n, n), device="cuda", generator=g) - 0.5) / 8).to(torch.float16)
    at = K.tilize(a, 32, 32)
    eye_t = K.tilize(torch.eye(n, device="cuda", dtype=torch.float16), 32, 32)
    c = K.matmul_tiled(at, eye_t, n, n, n)
    assert rt.last_kernel_name() == "gemm_tiled_f16_epi0"
    assert torch.equal(c, at)
    del eye_t
    b = ((torch.rand((n, n), device="cuda", generator=g) - 0.5) / 8).to(torch.float16)
    bt = K.tilize(b, 32, 32)
    c1 = K.matmul_tiled(at, bt, n, n, n)
    c2 = K.matmul_tiled(at * 2, bt, n, n, n)
    # exact wherever c1 is clear of fp16's subnormal range (a value that rounded UP to 2^-14 counts as inside it);
    # below, doubling the input keeps a bit that the rounded c1 lost
    normal = c1.abs() >= 2.0 ** -13
    assert torch.equal(c2[normal], c1[normal] * 2)
    assert torch.all((c2[~normal].float() - 2 * c1[~normal].float()).abs() <= 2.0 ** -24)
    rows = torch.randint(0, n, (32, ), device="cuda")
    ref = (a[rows].double() @ b.double()).float()
    got = K.untilize(c1, n, n, 32, 32)[rows].float()
    assert torch.all((got - ref).abs() <= 1e-2 * ref.abs() + 1e-4)


@pytest.mark.parametrize("M,N,K_", [(4352, 4096, 256), (4352, 4352, 128), (1024, 2048, 384)])
def test_tiled_fast_kernel_half_tile_tail(M, N, K_):
    """Macro-tile counts that leave a short last round (272 and 289 tiles on 256 CUs) or no whole round at all
    (32): the tail runs as half tiles.  Small integers, so the result is exact whatever the order."""
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-3, 4, (M, K_), generator=g).to(torch.float16)
    b = torch.randint(-3, 4, (K_, N), generator=g).to(torch.float16)
    for act in ("", "leaky_relu"):
        ct = K.matmul_tiled(K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), M, N, K_, activation=act)
        assert rt.last_kernel_name() == f"gemm_tiled_f16_epi{3 if act else 0}"
        want = a.cuda().float() @ b.cuda().float()
        want = torch.where(want >= 0, want, 0.01 * want) if act else want
        assert torch.equal(K.untilize(ct, M, N, 32, 32), want.to(torch.float16))


@pytest.mark.parametrize("M,N,K_", [(4300, 4090, 100), (4481, 4000, 40)])
def test_tiled_clamping_kernel_half_tile_tail(M, N, K_):
    """The same for the clamping instantiation: 272 and 288 macro tiles, the second with a last row of tiles
    whose lower halves lie wholly past the matrix."""
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-3, 4, (M, K_), generator=g).to(torch.float16)
    b = torch.randint(-3, 4, (K_, N), generator=g).to(torch.float16)
    ct = K.matmul_tiled(K.tilize(a, 32, 32).cuda(), K.tilize(b, 32, 32).cuda(), M, N, K_)
    assert rt.last_kernel_name() == "gemm_tiledragged_f16_epi0"
    assert torch.equal(K.untilize(ct, M, N, 32, 32), (a.cuda().float() @ b.cuda().float()).to(torch.float16))



# ---- few tiles under a long K: slices of K (the tile-major kernel's own instantiation, a row-major workspace) -----
@pytest.mark.parametrize("M,N,K_", [(64, 45, 2048), (1, 77, 2048), (300, 200, 3072), (200, 520, 2048), (256, 256, 4096)])
@pytest.mark.parametrize("act", ["", "leaky_relu"])
def test_tiled_k_slices_vs_oracle(M, N, K_, act):
    a, b = _rand((M, K_), 31), _rand((K_, N), 32)
    at, bt = K.tilize(a, 32, 32), K.tilize(b, 32, 32)
    ct = K.matmul_tiled(at.cuda(), bt.cuda(), M, N, K_, activation=act)
    assert rt.last_kernel_name() == "gemm_splitk_reduce_f16"
    ref = orc.matmul_tiled(_bits(at), _bits(bt), M, N, K_, in_dt=orc.F16, leaky_relu=bool(act), acc64=True)
    gm, rm = orc.untilize(_bits(ct.cpu()), M, N, 32, 32), orc.untilize(ref, M, N, 32, 32)
    assert _close(_f16(gm), _f16(rm))
    again = K.matmul_tiled(at.cuda(), bt.cuda(), M, N, K_, activation=act)      # slabs added in slice order: the same bits
    assert np.array_equal(orc.untilize(_bits(again.cpu()), M, N, 32, 32), gm)


def test_tiled_k_slices_exact_padding_untouched_and_ignored():
    """Small integers, bit for bit; the padding of the C tiles keeps the NaN it was filled with; NaN in the padding
    of A (rows past M) and of B (columns past N) does not reach the result (K is whole tiles on this route)."""
    rng = np.random.default_rng(5)
    for case in range(8):
        M, N = int(rng.integers(1, 400)), int(rng.integers(1, 600))
        K_ = int(rng.integers(8, 24)) * 256
        g = torch.Generator().manual_seed(case)
        a = torch.randint(-3, 4, (M, K_), generator=g).to(torch.float16)
        b = torch.randint(-3, 4, (K_, N), generator=g).to(torch.float16)
        Mp, Np = K.cdiv(M, 32) * 32, K.cdiv(N, 32) * 32
        an = torch.full((Mp, K_), float("nan"), dtype=torch.float16); an[:M] = a
        bn = torch.full((K_, Np), float("nan"), dtype=torch.float16); bn[:, :N] = b
        tm, tn = Mp // 32, Np // 32
        c = torch.full((tm * tn * 1024, ), float("nan"), dtype=torch.float16, device="cuda")
        act = "leaky_relu" if case % 3 == 0 else ""
        K.matmul_kernel[(tm * tn, )](K.tilize(an, 32, 32).cuda(), K.tilize(bn, 32, 32).cuda(), c, M, N, K_, K_, 1, N, 1, N, 1,
                                     ACTIVATION=act)
        assert rt.last_kernel_name() == "gemm_splitk_reduce_f16", (M, N, K_)
        full = c.cpu().reshape(tm, tn, 32, 32).permute(0, 2, 1, 3).reshape(Mp, Np)
        want = a.float() @ b.float()
        if act:
            want = torch.where(want >= 0, want, 0.01 * want)
        assert torch.equal(full[:M, :N], want.to(torch.float16)), (M, N, K_)
        assert torch.isnan(full[M:, :]).all() and torch.isnan(full[:, N:]).all(), (M, N, K_)
