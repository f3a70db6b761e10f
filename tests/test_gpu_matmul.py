"""GPU parity: the tile-matmul family through the launcher and the C ABI against the CPU
oracle.  Tolerance (bf16/fp16/fp8 inputs, fp32 accumulate): abs(err) <= 1e-2*abs(ref) + 1e-4
against the fp64-accumulated oracle, and PCC >= 0.9999 (the reference's bar is 0.97)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt
from triton_tenstorrent_amd.tensor_descriptor import TensorDescriptor
from util import ORC_DT, bits, close_bf16, decode

pytestmark = pytest.mark.gpu
RTOL, ATOL, PCC = 1e-2, 1e-4, 0.9999


def fp8_atol(ref):
    """fp8 products summed over K grow like sqrt(K): the absolute slack is 1e-4 of the output's rms
    (elements that cancel to ~0 cannot be held to a relative bound by any fp32-accumulating kernel)."""
    return ATOL * max(1.0, float(np.sqrt(np.mean(np.square(ref)))))


def _ab(M, N, K_, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn(M, K_, generator=g) / K_ ** 0.5 * 4).to(dtype)
    b = (torch.randn(K_, N, generator=g)).to(dtype)
    return a, b


def _check(c, a, b, **okw):
    dt = ORC_DT[a.dtype]
    ref = orc.matmul(bits(a), bits(b), in_dt=dt, out_dt=ORC_DT[c.dtype], acc64=True, **okw)
    ref = orc.decode(ref, ORC_DT[c.dtype])
    got = decode(c)
    assert close_bf16(got, ref, RTOL, ATOL), f"max err {np.max(np.abs(got - ref))}"
    assert orc.pcc(ref, got) >= PCC


# the reference's validate shapes (09-persistent-matmul.py:326-327, .ttnn.py:334-336) and more
@pytest.mark.parametrize("M,N,K_", [(32, 32, 32), (64, 32, 32), (64, 32, 64), (256, 256, 256), (1024, 1024, 1024), (384, 640, 192)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matmul_tma(M, N, K_, dtype):
    a, b = _ab(M, N, K_, dtype)
    c = K.matmul_tma(a.cuda(), b.cuda())
    _check(c, a, b)


@pytest.mark.parametrize("cfg", [dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64, GROUP_SIZE_M=1),
                                 dict(BLOCK_SIZE_M=32, BLOCK_SIZE_N=32, BLOCK_SIZE_K=32, GROUP_SIZE_M=3),
                                 dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=256, BLOCK_SIZE_K=64, GROUP_SIZE_M=8),
                                 dict(BLOCK_SIZE_M=256, BLOCK_SIZE_N=128, BLOCK_SIZE_K=32, GROUP_SIZE_M=2)])
def test_matmul_small_integers_exact_for_every_tiling(cfg):
    # every partial sum is exact in fp32 => bit-exact against the oracle for any tile size/order
    g = torch.Generator().manual_seed(3)
    M, N, K_ = 320, 448, 256
    a = torch.randint(-4, 5, (M, K_), generator=g).to(torch.bfloat16)
    b = torch.randint(-4, 5, (K_, N), generator=g).to(torch.bfloat16)
    c = K.matmul_tma(a.cuda(), b.cuda(), **cfg)
    want = orc.matmul(bits(a), bits(b), BM=cfg["BLOCK_SIZE_M"], BN=cfg["BLOCK_SIZE_N"], BK=cfg["BLOCK_SIZE_K"],
                      group_m=cfg["GROUP_SIZE_M"])
    assert np.array_equal(bits(c), want)


def test_matmul_ragged_shapes_strided_views_and_sentinel():
    # descriptor zero-padding on loads, clipped stores, non-contiguous rows; sentinel proves
    # nothing outside C[:M,:N] is written
    M, N, K_ = 200, 136, 104
    a, b = _ab(M + 8, N + 8, K_ + 8)
    a, b = a.cuda()[:M, :K_], b.cuda()[:K_, :N]
    cbuf = torch.full((M + 8, N + 8), 7.5, dtype=torch.bfloat16, device="cuda")
    c = cbuf[:M, :N]
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
    K.matmul_kernel_tma[(K.cdiv(M, 64) * K.cdiv(N, 64), )](ad, bd, cd, M, N, K_, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64,
                                                          BLOCK_SIZE_K=64, GROUP_SIZE_M=2, FP8_OUTPUT=False,
                                                          WARP_SPECIALIZE=False)
    _check(c, a.cpu(), b.cpu(), BM=64, BN=64, BK=64, group_m=2)
    assert torch.all(cbuf[M:, :] == 7.5) and torch.all(cbuf[:, N:] == 7.5)


# Shapes in whole 8-element chunks of N and K that are not whole 256x256x128 macro tiles take the fast kernel's
# clamping variant: rows / chunks past the edge are fetched from inside the matrix, a last 32-deep K step that ends
# past K is cleared from K on, K is padded with steps of zeros, stores are clipped.
RAGGED_SHAPES = [(33, 8, 32), (256, 256, 32), (260, 264, 160), (511, 520, 96), (1000, 1000, 992), (257, 1032, 4128),
                 (4000, 4096, 1024), (33, 8, 8), (256, 256, 40), (300, 328, 72), (1000, 1000, 1000), (257, 1032, 4104),
                 (4000, 4096, 1048)]


@pytest.mark.parametrize("M,N,K_", RAGGED_SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matmul_ragged_fast_path(M, N, K_, dtype):
    a, b = _ab(M, N, K_, dtype, seed=M + N)
    # C sits inside a larger buffer: the sentinel shows that nothing outside C[:M,:N] is written
    cbuf = torch.full((M + 3, N + 16), 7.5, dtype=dtype, device="cuda")
    c = cbuf[:M, :N]
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a.cuda(), b.cuda(), c))
    K.matmul_kernel_tma[(K.cdiv(M, 64) * K.cdiv(N, 64), )](ad, bd, cd, M, N, K_, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64,
                                                          BLOCK_SIZE_K=32, GROUP_SIZE_M=1, FP8_OUTPUT=False,
                                                          WARP_SPECIALIZE=False)
    assert rt.last_kernel_name() == f"gemm_ragged_{'bf16' if dtype == torch.bfloat16 else 'f16'}_epi0"
    _check(c, a, b, BM=64, BN=64, BK=32)
    assert torch.all(cbuf[M:, :] == 7.5) and torch.all(cbuf[:, N:] == 7.5)


def test_matmul_ragged_fast_path_random_shapes_exact():
    # a seeded sweep over shapes (M anything, N and K in steps of 8), small integers: bit for bit, with
    # a sentinel frame around C and NaN frames around A and B
    rng = np.random.default_rng(2025)
    for case in range(32):
        M = int(rng.integers(1, 700))
        N = 8 * int(rng.integers(1, 90))
        K_ = 8 * int(rng.integers(1, 48))
        dtype = torch.bfloat16 if case % 2 else torch.float16
        g = torch.Generator().manual_seed(case)
        abuf = torch.full((M + 2, K_ + 8), float("nan"), dtype=dtype)
        bbuf = torch.full((K_ + 2, N + 8), float("nan"), dtype=dtype)
        abuf[:M, :K_] = torch.randint(-3, 4, (M, K_), generator=g).to(dtype)
        bbuf[:K_, :N] = torch.randint(-3, 4, (K_, N), generator=g).to(dtype)
        cbuf = torch.full((M + 2, N + 8), 7.5, dtype=dtype, device="cuda")
        c = cbuf[:M, :N]
        ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (abuf.cuda()[:M, :K_], bbuf.cuda()[:K_, :N], c))
        K.matmul_kernel_tma[(K.cdiv(M, 32) * K.cdiv(N, 32), )](ad, bd, cd, M, N, K_, BLOCK_SIZE_M=32, BLOCK_SIZE_N=32,
                                                              BLOCK_SIZE_K=32, GROUP_SIZE_M=1, FP8_OUTPUT=False,
                                                              WARP_SPECIALIZE=False)
        whole = M % 256 == 0 and N % 256 == 0 and K_ % 128 == 0
        assert rt.last_kernel_name().startswith("gemm_tile_" if whole else "gemm_ragged_"), (M, N, K_)
        want = abuf[:M, :K_].float() @ bbuf[:K_, :N].float()            # exact in fp32, and in the half types up to 2^8
        assert torch.equal(c.float().cpu(), want.to(dtype).float()), (M, N, K_)
        assert torch.all(cbuf[M:, :] == 7.5) and torch.all(cbuf[:, N:] == 7.5), (M, N, K_)


def test_matmul_ragged_fast_path_every_k_in_steps_of_eight():
    # K = 8 .. 328: every length of the last step (8, 16, 24, 32) at every depth of the copy ring's fill (one to ten
    # steps); small integers, bit for bit.  The operands end where their buffers end, next to NaN rows of the
    # neighbouring allocation-sized frame: a chunk fetched past K would bring NaN (A) or the next row in
    M, N = 261, 264
    for K_ in range(8, 336, 8):
        g = torch.Generator().manual_seed(K_)
        abuf = torch.full((M + 1, K_), float("nan"), dtype=torch.bfloat16)
        bbuf = torch.full((K_ + 1, N), float("nan"), dtype=torch.bfloat16)
        abuf[:M] = torch.randint(-3, 4, (M, K_), generator=g).to(torch.bfloat16)
        bbuf[:K_] = torch.randint(-3, 4, (K_, N), generator=g).to(torch.bfloat16)
        # column K-1 large: a chunk of A cleared one element too early, or a row of B dropped, shows at once
        abuf[:M, K_ - 1] = 64
        c = K.matmul_tma(abuf.cuda()[:M], bbuf.cuda()[:K_])
        assert rt.last_kernel_name() == "gemm_ragged_bf16_epi0", K_
        want = (abuf[:M].float() @ bbuf[:K_].float()).to(torch.bfloat16)
        assert torch.equal(c.cpu(), want), K_


def test_matmul_ragged_fast_path_exact_and_with_wild_values_next_door():
    # small integers: bit for bit against the oracle.  The operands are views into larger buffers whose
    # neighbouring rows and columns hold inf and NaN: whatever the clamped fetches and the padding steps
    # read, none of it may reach C
    g = torch.Generator().manual_seed(12)
    M, N, K_ = 300, 328, 224
    abuf = torch.full((M + 5, K_ + 8), float("nan"), dtype=torch.bfloat16)
    bbuf = torch.full((K_ + 7, N + 8), float("inf"), dtype=torch.bfloat16)
    abuf[:M, :K_] = torch.randint(-4, 5, (M, K_), generator=g).to(torch.bfloat16)
    bbuf[:K_, :N] = torch.randint(-4, 5, (K_, N), generator=g).to(torch.bfloat16)
    a, b = abuf.cuda()[:M, :K_], bbuf.cuda()[:K_, :N]
    c = K.matmul_tma(a, b)
    assert rt.last_kernel_name() == "gemm_ragged_bf16_epi0"
    want = orc.matmul(bits(abuf[:M, :K_]), bits(bbuf[:K_, :N]), BM=64, BN=64, BK=64)
    assert np.array_equal(bits(c), want)


@pytest.mark.parametrize("epilogue", [None, "gelu", "bias_row", "leaky_relu"])
def test_matmul_ragged_fast_path_epilogues(epilogue):
    M, N, K_ = 390, 520, 160
    a, b = _ab(M, N, K_, seed=21)
    gen = torch.Generator().manual_seed(22)
    if epilogue is None:
        bias = torch.randn(M, N, generator=gen).to(torch.bfloat16)
        okw = dict(bias=bits(bias), epi=orc.EPI_BIAS_FULL)
    else:
        bias = torch.randn(N, generator=gen) * 0.02
        okw = dict(bias=bias.numpy(), epi={"gelu": orc.EPI_BIAS_ROW_GELU, "bias_row": orc.EPI_BIAS_ROW,
                                          "leaky_relu": orc.EPI_LEAKY_RELU}[epilogue])
        if epilogue == "leaky_relu":
            okw.pop("bias")
    c = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda(), epilogue=epilogue)
    assert rt.last_kernel_name().startswith("gemm_ragged_bf16_epi")
    ref = orc.from_bf16(orc.matmul(bits(a), bits(b), acc64=True, **okw))
    assert close_bf16(decode(c), ref, RTOL, 1e-2 if epilogue is None else ATOL)


@pytest.mark.parametrize("M,N,K_", [(40, 16, 64), (300, 336, 192), (1000, 1008, 960), (4000, 4096, 1088)])
def test_fp8_scaled_ragged_fast_path(M, N, K_):
    g = torch.Generator().manual_seed(M)
    x, w = torch.randn(M, K_, generator=g), torch.randn(K_, N, generator=g)
    qa, sa = K.quantize_fp8(x)
    qb, sb = K.quantize_fp8(w)
    # operands are views into buffers whose surroundings are NaN codes (0x7f): none of it may reach C
    abuf = torch.full((M + 2, K_ + 16), 0x7f, dtype=torch.uint8).view(torch.float8_e4m3fn)
    bbuf = torch.full((K_ + 2, N + 16), 0x7f, dtype=torch.uint8).view(torch.float8_e4m3fn)
    abuf[:M, :K_] = qa
    bbuf[:K_, :N] = qb
    c = K.matmul_fp8_scaled(abuf.cuda()[:M, :K_], bbuf.cuda()[:K_, :N], sa, sb)
    assert rt.last_kernel_name() == "gemm_ragged_fp8_bf16"
    ref = orc.from_bf16(orc.matmul(bits(qa), bits(qb), in_dt=orc.FP8E4M3, out_dt=orc.BF16,
                                   scale=float(np.float32(sa) * np.float32(sb)), acc64=True))
    assert close_bf16(decode(c), ref, RTOL, fp8_atol(ref))


@pytest.mark.parametrize("M,N,K_", [(100, 336, 4096), (16, 512, 4096), (300, 208, 3072), (256, 256, 4096), (130, 1024, 8192)])
def test_fp8_scaled_k_slices(M, N, K_):
    """fp8 launches of few tiles under a long K (a multiple of 512) run in slices of K too: half tiles as parts, the
    same workspace and adding kernel, the scales applied to the whole sum.  Operands are views into buffers whose
    surroundings are NaN codes; two launches give the same bits."""
    g = torch.Generator().manual_seed(M + K_)
    qa, sa = K.quantize_fp8(torch.randn(M, K_, generator=g))
    qb, sb = K.quantize_fp8(torch.randn(K_, N, generator=g))
    abuf = torch.full((M + 2, K_ + 16), 0x7f, dtype=torch.uint8).view(torch.float8_e4m3fn)
    bbuf = torch.full((K_ + 2, N + 16), 0x7f, dtype=torch.uint8).view(torch.float8_e4m3fn)
    abuf[:M, :K_] = qa
    bbuf[:K_, :N] = qb
    a, b = abuf.cuda()[:M, :K_], bbuf.cuda()[:K_, :N]
    c = K.matmul_fp8_scaled(a, b, sa, sb)
    assert rt.last_kernel_name() == "gemm_splitk_reduce_bf16"
    ref = orc.from_bf16(orc.matmul(bits(qa), bits(qb), in_dt=orc.FP8E4M3, out_dt=orc.BF16,
                                   scale=float(np.float32(sa) * np.float32(sb)), acc64=True))
    assert close_bf16(decode(c), ref, RTOL, fp8_atol(ref))
    assert torch.equal(K.matmul_fp8_scaled(a, b, sa, sb), c)


def test_matmul_partial_grid_runs_only_its_programs():
    a, b = _ab(256, 256, 128)
    c = torch.full((256, 256), 7.5, dtype=torch.bfloat16, device="cuda")
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a.cuda(), b.cuda(), c))
    K.matmul_kernel_tma[(5, )](ad, bd, cd, 256, 256, 128, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64,
                               GROUP_SIZE_M=2, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    want = np.full((256, 256), 0x40F0, dtype=np.uint16)
    orc.matmul(bits(a), bits(b), BM=64, BN=64, BK=64, group_m=2, grid=5, out=want, acc64=True)
    touched = want != 0x40F0
    assert np.array_equal(bits(c) != 0x40F0, touched)
    assert close_bf16(decode(c)[touched], orc.from_bf16(want)[touched], RTOL, ATOL)
    with pytest.raises(ValueError):
        K.matmul_kernel_tma[(17, )](ad, bd, cd, 256, 256, 128, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64,
                                    GROUP_SIZE_M=2, FP8_OUTPUT=False, WARP_SPECIALIZE=False)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_full_bias_adds_in_half_after_the_cast(dtype):
    M, N, K_ = 192, 256, 128
    a, b = _ab(M, N, K_, dtype, seed=4)
    bias = torch.randn(M, N, generator=torch.Generator().manual_seed(5)).to(dtype)
    c = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda())
    dt = ORC_DT[dtype]
    ref = orc.decode(orc.matmul(bits(a), bits(b), in_dt=dt, out_dt=dt, bias=bits(bias), epi=orc.EPI_BIAS_FULL, acc64=True), dt)
    assert close_bf16(decode(c), ref, RTOL, 1e-2)
    # identity on the epilogue: exactly half(c0) + bias in the half type
    c0 = K.matmul_tma(a.cuda(), b.cuda())
    assert torch.equal(c, c0 + bias.cuda())


def test_fused_row_bias_gelu():
    # BASELINE's fused-epilogue config shape class; erf-form GELU in fp32 on the accumulator (the oracle uses
    # libm's erf, the kernel a polynomial within 1.5e-7 of it: far inside the bf16 output's rounding)
    M, N, K_ = 256, 512, 256
    a, b = _ab(M, N, K_, seed=6)
    bias = torch.randn(N, generator=torch.Generator().manual_seed(7)) * 0.02
    c = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda(), epilogue="gelu")
    ref = orc.from_bf16(orc.matmul(bits(a), bits(b), bias=bias.numpy(), epi=orc.EPI_BIAS_ROW_GELU, acc64=True))
    assert close_bf16(decode(c), ref, RTOL, ATOL)
    tref = torch.nn.functional.gelu(a.double() @ b.double() + bias.double()).float().numpy()
    assert close_bf16(decode(c), tref, RTOL, 1e-3)
    c2 = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda(), epilogue="bias_row")
    ref2 = orc.from_bf16(orc.matmul(bits(a), bits(b), bias=bias.numpy(), epi=orc.EPI_BIAS_ROW, acc64=True))
    assert close_bf16(decode(c2), ref2, RTOL, ATOL)
    c3 = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda(), epilogue="leaky_relu")
    ref3 = orc.from_bf16(orc.matmul(bits(a), bits(b), epi=orc.EPI_LEAKY_RELU, acc64=True))
    assert close_bf16(decode(c3), ref3, RTOL, ATOL)


@pytest.mark.parametrize("M,N,K_", [(64, 64, 64), (256, 384, 512), (1024, 1024, 1024)])
def test_fp8_scaled(M, N, K_):
    g = torch.Generator().manual_seed(8)
    x, w = torch.randn(M, K_, generator=g), torch.randn(K_, N, generator=g)
    qa, sa = K.quantize_fp8(x)
    qb, sb = K.quantize_fp8(w)
    # host quantiser agrees with the oracle's
    oa, osa = orc.quantize_fp8(x.numpy())
    assert np.array_equal(bits(qa), oa) and abs(sa - osa) <= 1e-9
    c = K.matmul_fp8_scaled(qa.cuda(), qb.cuda(), sa, sb)
    ref = orc.from_bf16(orc.matmul(bits(qa), bits(qb), in_dt=orc.FP8E4M3, out_dt=orc.BF16,
                                   scale=float(np.float32(sa) * np.float32(sb)), acc64=True))
    assert close_bf16(decode(c), ref, RTOL, fp8_atol(ref))
    assert orc.pcc(ref, decode(c)) >= PCC


def test_fp8_inputs_fp8_output_unscaled():
    g = torch.Generator().manual_seed(9)
    a = (torch.randn(128, 64, generator=g) * 0.5).to(torch.float8_e4m3fn)
    b = (torch.randn(64, 96, generator=g) * 0.5).to(torch.float8_e4m3fn)
    c = K.matmul_tma(a.cuda(), b.cuda(), BLOCK_SIZE_M=32, BLOCK_SIZE_N=32, BLOCK_SIZE_K=32, GROUP_SIZE_M=1)
    assert c.dtype == torch.float8_e4m3fn
    want = orc.matmul(bits(a), bits(b), in_dt=orc.FP8E4M3, out_dt=orc.FP8E4M3, BM=32, BN=32, BK=32, acc64=True)
    got = bits(c)
    # fp8 output: one e4m3 ulp of slack where fp32 vs fp64 accumulation straddles a rounding boundary
    assert np.mean(got != want) < 0.02
    assert np.max(np.abs(orc.from_fp8(got) - orc.from_fp8(want))) <= 0.125 * np.max(np.abs(orc.from_fp8(want)))


@pytest.mark.parametrize("M,N,K_", [(256, 256, 256), (512, 768, 512), (300, 336, 192)])
def test_fp8_output_fast_path_exact_on_small_integers(M, N, K_):
    # FP8_OUTPUT (09-persistent-matmul.py:116,173) on the fast kernel: exact sums, one rounding to e4m3 (saturating)
    g = torch.Generator().manual_seed(M + K_)
    a = torch.randint(-2, 3, (M, K_), generator=g).float().to(torch.float8_e4m3fn)
    b = torch.randint(-2, 3, (K_, N), generator=g).float().to(torch.float8_e4m3fn)
    c = K.matmul_tma(a.cuda(), b.cuda())
    assert c.dtype == torch.float8_e4m3fn
    assert rt.last_kernel_name() == ("gemm_tile_fp8_fp8" if M % 256 == 0 and N % 256 == 0 and K_ % 256 == 0 else "gemm_ragged_fp8_fp8")
    want = orc.matmul(bits(a), bits(b), in_dt=orc.FP8E4M3, out_dt=orc.FP8E4M3, acc64=True)
    assert np.array_equal(bits(c), want)


def test_matmul_errors():
    a, b = _ab(64, 64, 64)
    with pytest.raises(NotImplementedError):
        K.matmul_tma(a.cuda(), b.cuda(), BLOCK_SIZE_M=48, BLOCK_SIZE_N=64)   # not a multiple of 32
    with pytest.raises(NotImplementedError):
        K.matmul_tma(a.cuda().float(), b.cuda().float())
    ad, bd = (TensorDescriptor.from_tensor(t.cuda(), [32, 32]) for t in (a, b))
    c = torch.empty(64, 32, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        K.matmul_kernel_tma[(1, )](ad, bd, TensorDescriptor.from_tensor(c, [32, 32]), 64, 64, 64, FP8_OUTPUT=False,
                                   WARP_SPECIALIZE=False)
    assert rt.last_error() != ""


# ---- the 256x256x64 macro-tile fast path -----------------------------------
@pytest.mark.parametrize("M,N,K_", [(256, 256, 128), (256, 256, 256), (512, 768, 384), (1024, 256, 2048), (768, 1280, 640)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fast_path_matches_oracle(M, N, K_, dtype):
    a, b = _ab(M, N, K_, dtype, seed=M + N + K_)
    c = K.matmul_tma(a.cuda(), b.cuda())
    # (four tiles under K = 2048: the launch that is finished in slices of K)
    assert rt.last_kernel_name().startswith("gemm_splitk_reduce_" if K_ == 2048 else "gemm_tile_"), rt.last_kernel_name()
    _check(c, a, b)


# ---- few tiles under a long K: slices of K as work items, fp32 sums through a workspace -------------------------
@pytest.mark.parametrize("M,N,K_", [(64, 256, 2048), (1, 512, 4096), (200, 520, 2048), (256, 256, 4096), (300, 264, 3072),
                                    (130, 1024, 8192), (700, 256, 2560)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_k_slices_match_oracle(M, N, K_, dtype):
    """Shapes of one to twelve macro tiles with K a multiple of 256: matrices of one row of tiles with 1, 64, 130, 200
    and 256 live rows (one to four live quarters per tile), two and three rows of tiles, N not a whole tile.  The
    result is the fp32 sum over all of K rounded once, as without slices, so the same bounds hold; two launches give
    the same bits (the slabs are added in slice order)."""
    a, b = _ab(M, N, K_, dtype, seed=M + N + K_)
    c = K.matmul_tma(a.cuda(), b.cuda())
    assert rt.last_kernel_name() == ("gemm_splitk_reduce_bf16" if dtype == torch.bfloat16 else "gemm_splitk_reduce_f16")
    _check(c, a, b)
    assert torch.equal(K.matmul_tma(a.cuda(), b.cuda()), c)


def test_k_slices_small_integers_bit_exact_and_output_strides():
    g = torch.Generator().manual_seed(5)
    M, N, K_ = 190, 520, 4096
    a = torch.randint(-4, 5, (M, K_), generator=g).to(torch.bfloat16)
    b = torch.randint(-4, 5, (K_, N), generator=g).to(torch.bfloat16)
    cbuf = torch.full((M + 3, N + 24), 7.5, dtype=torch.bfloat16, device="cuda")
    c = cbuf[:M, :N]
    from triton_tenstorrent_amd.tensor_descriptor import TensorDescriptor as TD
    ad, bd, cd = TD.from_tensor(a.cuda(), [128, 64]), TD.from_tensor(b.cuda(), [64, 128]), TD.from_tensor(c, [128, 128])
    K.matmul_kernel_tma[(2 * 5, )](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False, BLOCK_SIZE_M=128,
                                   BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, GROUP_SIZE_M=8)
    assert rt.last_kernel_name() == "gemm_splitk_reduce_bf16"
    assert np.array_equal(bits(c), orc.matmul(bits(a), bits(b), BM=64, BN=64, BK=64))
    # nothing outside the [M, N] window of the output buffer was written
    assert torch.all(cbuf[M:, :] == 7.5) and torch.all(cbuf[:, N:] == 7.5)


@pytest.mark.parametrize("epilogue", [None, "gelu", "bias_row", "leaky_relu"])
def test_k_slices_epilogues(epilogue):
    """The epilogue is applied by the kernel that adds the slabs, on the whole sum: same results as in one pass."""
    M, N, K_ = 100, 520, 4096
    a, b = _ab(M, N, K_, seed=31)
    gen = torch.Generator().manual_seed(32)
    if epilogue is None:
        bias = torch.randn(M, N, generator=gen).to(torch.bfloat16)
        okw = dict(bias=bits(bias), epi=orc.EPI_BIAS_FULL)
    else:
        bias = torch.randn(N, generator=gen) * 0.02
        okw = dict(bias=bias.numpy(), epi={"gelu": orc.EPI_BIAS_ROW_GELU, "bias_row": orc.EPI_BIAS_ROW,
                                          "leaky_relu": orc.EPI_LEAKY_RELU}[epilogue])
        if epilogue == "leaky_relu":
            okw.pop("bias")
    c = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda(), epilogue=epilogue)
    assert rt.last_kernel_name() == "gemm_splitk_reduce_bf16"
    ref = orc.from_bf16(orc.matmul(bits(a), bits(b), acc64=True, **okw))
    assert close_bf16(decode(c), ref, RTOL, 1e-2 if epilogue is None else ATOL)


def test_k_slices_workspace_per_stream_growth_release_and_graphs():
    """The workspace belongs to a (device, stream) pair: launches on two streams do not share one, a launch that
    needs more than the stream's has grows it, rt_release_stream gives it back (and the next launch takes a new
    one), and a launch that is being recorded into a graph runs in one pass and holds no address of the library's."""
    shapes = [(64, 256, 2048), (200, 1024, 4096), (64, 256, 2048)]      # small, larger, small again
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    data = [[_ab(M, N, K_, seed=7 * i + j) for j, (M, N, K_) in enumerate(shapes)] for i in range(2)]
    dev = [[(a.cuda(), b.cuda()) for a, b in row] for row in data]
    torch.cuda.synchronize()
    out = [[None] * len(shapes) for _ in range(2)]
    for j in range(len(shapes)):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                out[i][j] = K.matmul_tma(*dev[i][j])
                assert rt.last_kernel_name() == "gemm_splitk_reduce_bf16"
    torch.cuda.synchronize()
    for i in range(2):
        for j in range(len(shapes)):
            _check(out[i][j], *data[i][j])
    for st in streams:
        assert rt.load().rt_release_stream(C.c_void_p(st.cuda_stream)) == rt.RT_OK
    with torch.cuda.stream(streams[0]):
        c = K.matmul_tma(*dev[0][1])
    streams[0].synchronize()
    assert torch.equal(c, out[0][1])
    assert rt.load().rt_release_stream(C.c_void_p(streams[0].cuda_stream)) == rt.RT_OK
    # under capture: one pass, same bounds; replays agree with each other
    a, b = dev[1][1]
    cg = torch.empty(a.shape[0], b.shape[1], dtype=torch.bfloat16, device="cuda")
    ad, bd, cd = (TensorDescriptor.from_tensor(t, blk) for t, blk in ((a, [128, 64]), (b, [64, 128]), (cg, [128, 128])))
    M, K_ = a.shape
    N = b.shape[1]
    grid = ((M + 127) // 128 * ((N + 127) // 128), )
    st = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        K.matmul_kernel_tma[grid](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False, BLOCK_SIZE_M=128,
                                  BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, GROUP_SIZE_M=8)      # warm: modules loaded
        st.synchronize()
        with torch.cuda.graph(graph, stream=st):
            K.matmul_kernel_tma[grid](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False, BLOCK_SIZE_M=128,
                                      BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, GROUP_SIZE_M=8)
            assert rt.last_kernel_name() == "gemm_ragged_bf16_epi0"
    for _ in range(3):
        cg.zero_()
        graph.replay()
        torch.cuda.synchronize()
        _check(cg, *data[1][1])


def test_fast_path_small_integers_bit_exact():
    g = torch.Generator().manual_seed(11)
    M, N, K_ = 512, 512, 640
    a = torch.randint(-4, 5, (M, K_), generator=g).to(torch.bfloat16)
    b = torch.randint(-4, 5, (K_, N), generator=g).to(torch.bfloat16)
    c = K.matmul_tma(a.cuda(), b.cuda())
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi0"
    assert np.array_equal(bits(c), orc.matmul(bits(a), bits(b), BM=128, BN=128, BK=64, group_m=8))
    # a permutation matrix tells B from B^T and exposes any mis-indexed fragment
    p = torch.zeros(512, 512)
    p[torch.arange(512), (torch.arange(512) * 37 + 5) % 512] = 1
    x = torch.randn(512, 512, generator=g).to(torch.bfloat16)
    c = K.matmul_tma(x.cuda(), p.to(torch.bfloat16).cuda())
    assert torch.equal(c.cpu(), (x.float() @ p).to(torch.bfloat16))
    c = K.matmul_tma(p.to(torch.bfloat16).cuda(), x.cuda())
    assert torch.equal(c.cpu(), (p @ x.float()).to(torch.bfloat16))


def test_fast_path_strided_rows_and_epilogues():
    M, N, K_ = 512, 512, 256
    a, b = _ab(M, N + 64, K_ + 64, seed=12)
    a = a.cuda()[:, :K_]                 # lda = K+64
    b = b.cuda()[:K_ , :N]               # ldb = N+64
    cbuf = torch.full((M, N + 64), 7.5, dtype=torch.bfloat16, device="cuda")
    c = cbuf[:, :N]
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
    K.matmul_kernel_tma[(16, )](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi0"
    _check(c, a.cpu(), b.cpu())
    assert torch.all(cbuf[:, N:] == 7.5)
    ac, bc = a.contiguous(), b.contiguous()
    bias_full = torch.randn(M, N, generator=torch.Generator().manual_seed(13)).to(torch.bfloat16).cuda()
    cf = K.matmul_fused(ac, bc, bias_full)
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi1"
    assert torch.equal(cf, c + bias_full)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(14)) * 0.02).cuda()
    cg = K.matmul_fused(ac, bc, bias, epilogue="gelu")
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi2"
    ref = orc.from_bf16(orc.matmul(bits(ac), bits(bc), bias=bias.cpu().numpy(), epi=orc.EPI_BIAS_ROW_GELU, acc64=True))
    assert close_bf16(decode(cg), ref, RTOL, ATOL)
    cl = K.matmul_fused(ac, bc, bias, epilogue="leaky_relu")
    ref = orc.from_bf16(orc.matmul(bits(ac), bits(bc), epi=orc.EPI_LEAKY_RELU, acc64=True))
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi3" and close_bf16(decode(cl), ref, RTOL, ATOL)
    cr = K.matmul_fused(ac, bc, bias, epilogue="bias_row")
    ref = orc.from_bf16(orc.matmul(bits(ac), bits(bc), bias=bias.cpu().numpy(), epi=orc.EPI_BIAS_ROW, acc64=True))
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi4" and close_bf16(decode(cr), ref, RTOL, ATOL)


# Shapes whose macro tiles do not fill the last round of the persistent grid: the kernel finishes the tail as
# half tiles, two workgroups per tile.  With 256 CUs: 272 tiles = one round + 16 (dealt in groups of 8 tiles),
# 289 = one round + 33 (dealt in pairs), 64 and 15 tiles = tail only.
@pytest.mark.parametrize("M,N,K_", [(4352, 4096, 256), (4352, 4352, 128), (2048, 2048, 256), (768, 1280, 640)])
def test_fast_path_half_tile_tail(M, N, K_):
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-4, 5, (M, K_), generator=g).to(torch.bfloat16).cuda()
    b = torch.randint(-4, 5, (K_, N), generator=g).to(torch.bfloat16).cuda()
    c = K.matmul_tma(a, b)
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi0"
    assert torch.equal(c, (a.float() @ b.float()).to(torch.bfloat16))       # small integers: every sum is exact in fp32
    # random operands against the oracle, with the GELU epilogue (row bias indexed by the half tile's columns)
    a, b = _ab(M, N, K_, seed=M * 3 + N)
    bias = (torch.randn(N, generator=g) * 0.02)
    cg = K.matmul_fused(a.cuda(), b.cuda(), bias.cuda(), epilogue="gelu")
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi2"
    ref = orc.from_bf16(orc.matmul(bits(a), bits(b), bias=bias.numpy(), epi=orc.EPI_BIAS_ROW_GELU, acc64=True))
    assert close_bf16(decode(cg), ref, RTOL, ATOL)
    # strided C with a sentinel beside it: the half tiles store their own rows only
    cbuf = torch.full((M, N + 8), 7.5, dtype=torch.float16, device="cuda")
    ah, bh = a.to(torch.float16).cuda(), b.to(torch.float16).cuda()
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (ah, bh, cbuf[:, :N]))
    K.matmul_kernel_tma[((M // 128) * (N // 128), )](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert rt.last_kernel_name() == "gemm_tile_f16_epi0" and torch.all(cbuf[:, N:] == 7.5)
    _check(cbuf[:, :N].cpu(), ah.cpu(), bh.cpu())


@pytest.mark.parametrize("M,N,K_", [(4300, 4096, 160), (4225, 4104, 96), (2000, 2056, 224), (4481, 4096, 64)])
def test_ragged_fast_path_half_tile_tail(M, N, K_):
    """The clamping instantiation with a short last round: 272 and 289 macro tiles, 72 (tail only), and 288 with a
    last row of tiles that holds one row of C, so every lower half there lies past the matrix and stores nothing."""
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-4, 5, (M, K_), generator=g).to(torch.bfloat16).cuda()
    b = torch.randint(-4, 5, (K_, N), generator=g).to(torch.bfloat16).cuda()
    cbuf = torch.full((M + 1, N + 8), 7.5, dtype=torch.bfloat16, device="cuda")
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, cbuf[:M, :N]))
    K.matmul_kernel_tma[(-(-M // 128) * -(-N // 128), )](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert rt.last_kernel_name() == "gemm_ragged_bf16_epi0"
    assert torch.equal(cbuf[:M, :N], (a.float() @ b.float()).to(torch.bfloat16))
    assert torch.all(cbuf[M:] == 7.5) and torch.all(cbuf[:, N:] == 7.5)


def test_full_size_gelu_row_bias_4096x14336x4096():
    """BASELINE's fused-epilogue shape, D = GELU(A.B + bias[N]) with M, N, K = 4096, 14336, 4096: 896 macro tiles on
    256 CUs, i.e. three whole rounds and a tail that runs as half tiles, at 32 turns of the ring per tile.  Small
    integers with an integer row bias are exact in fp32 whatever the order (the GELU of an integer >= 6 in magnitude
    is the integer or 0 to bf16 precision, and in between the bar is the bf16 rounding of the exact value); random
    operands on sampled rows and columns against float64 erf-GELU; a sentinel column block beside C."""
    M, N, K_ = 4096, 14336, 4096
    g = torch.Generator(device="cuda").manual_seed(21)
    a = torch.randint(-2, 3, (M, K_), device="cuda", generator=g).to(torch.bfloat16)
    b = torch.randint(-2, 3, (K_, N), device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randint(-3, 4, (N, ), device="cuda", generator=g).float()
    c = K.matmul_fused(a, b, bias, epilogue="bias_row")
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi4"
    want = a.float() @ b.float() + bias                      # |sums| < 2^24: exact in fp32 in any order
    assert torch.equal(c, want.to(torch.bfloat16))
    cg = K.matmul_fused(a, b, bias, epilogue="gelu")
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi2"
    ref = torch.nn.functional.gelu(want.double())
    assert bool(torch.all((cg.double() - ref).abs() <= RTOL * ref.abs() + ATOL))
    del c, cg, want, ref
    # random operands as BASELINE draws them, sampled rows and columns against float64
    a = (torch.randn(M, K_, device="cuda", generator=g) / K_ ** 0.5).to(torch.bfloat16)
    b = torch.randn(K_, N, device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randn(N, device="cuda", generator=g) * 0.02
    cbuf = torch.full((M, N + 8), 7.5, dtype=torch.bfloat16, device="cuda")
    cg = cbuf[:, :N]
    ad, bd, cd, biasd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, cg, bias.reshape(1, N)))
    K.matmul_kernel_fused[((M // 128) * (N // 128), )](ad, bd, cd, biasd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False,
                                                        EPILOGUE="gelu")
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi2"
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 2047, 2048, 3839, 3840, 3967, 3968, 4095, 1234], device="cuda")
    ref = torch.nn.functional.gelu(a[rows].double() @ b.double() + bias.double())
    assert bool(torch.all((cg[rows].double() - ref).abs() <= RTOL * ref.abs() + ATOL))
    cols = torch.tensor([0, 7, 8, 255, 256, 14079, 14080, 14207, 14208, 14335, 9999], device="cuda")
    ref = torch.nn.functional.gelu(a.double() @ b[:, cols].double() + bias[cols].double())
    assert bool(torch.all((cg[:, cols].double() - ref).abs() <= RTOL * ref.abs() + ATOL))
    assert torch.all(cbuf[:, N:] == 7.5)


def test_full_size_8192_properties():
    """BASELINE's 8192^3: checked through size-independent properties -- B = I gives C = A
    bit for bit, linearity in A, and sampled rows against fp64 on the host."""
    n = 8192
    g = torch.Generator(device="cuda").manual_seed(0)
    a = (torch.randn(n, n, device="cuda", generator=g) / n ** 0.5).to(torch.bfloat16)
    eye = torch.eye(n, device="cuda", dtype=torch.bfloat16)
    c = K.matmul_tma(a, eye)
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi0"
    assert torch.equal(c, a)
    assert torch.equal(K.matmul_tma(eye, a), a)
    del eye
    b = (torch.randn(n, n, device="cuda", generator=g) / n ** 0.5).to(torch.bfloat16)
    c = K.matmul_tma(a, b)
    rows = torch.tensor([0, 1, 255, 256, 4095, 4096, 8191, 5000, 77], device="cuda")
    ref = (a[rows].double() @ b.double()).float()
    err = (c[rows].float() - ref).abs()
    assert bool(torch.all(err <= RTOL * ref.abs() + ATOL))
    cols = torch.tensor([0, 31, 32, 255, 256, 8191, 6007], device="cuda")
    ref = (a.double() @ b[:, cols].double()).float()
    assert bool(torch.all((c[:, cols].float() - ref).abs() <= RTOL * ref.abs() + ATOL))
    # scaling A by 2 scales C by 2 exactly (powers of two commute with every rounding)
    assert torch.equal(K.matmul_tma(a * 2, b), c * 2)


def test_streaming_stores_of_an_output_beyond_the_memory_side_cache():
    """A C of more than 256 MiB with K <= 2048 goes to the kernels whose stores bypass the caches: small integers
    make every element exact, so the whole 512 MiB output is compared, ragged edge included."""
    g = torch.Generator(device="cuda").manual_seed(5)
    for (M, N, K_), kernel in (((16384, 16384, 256), "gemm_tile_bf16_epi0_stream"), ((16380, 16392, 136), "gemm_ragged_bf16_epi0_stream")):
        a = torch.randint(-3, 4, (M, K_), device="cuda", generator=g).to(torch.bfloat16)
        b = torch.randint(-3, 4, (K_, N), device="cuda", generator=g).to(torch.bfloat16)
        cbuf = torch.full((M, N + 8), 7.5, device="cuda", dtype=torch.bfloat16)
        c = cbuf[:, :N]
        ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
        K.matmul_kernel_tma[(-(-M // 128) * -(-N // 128), )](ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
        assert rt.last_kernel_name() == kernel
        for r0 in range(0, M, 4096):          # (by slabs: the float reference of a slab is 256 MiB)
            r1 = min(r0 + 4096, M)
            assert torch.equal(c[r0:r1], (a[r0:r1].float() @ b.float()).to(torch.bfloat16))   # (sums < 2^24: exact in fp32)
        assert torch.all(cbuf[:, N:] == 7.5)
        del a, b, c, cbuf


# ---- the fp8 fast path (scaled 32x32x64 MFMA, transposing byte reads) --------
@pytest.mark.parametrize("M,N,K_", [(256, 256, 256), (512, 768, 512), (1024, 1024, 1024), (256, 512, 2048)])
def test_fp8_fast_path(M, N, K_):
    g = torch.Generator().manual_seed(M + K_)
    x, w = torch.randn(M, K_, generator=g), torch.randn(K_, N, generator=g)
    qa, sa = K.quantize_fp8(x)
    qb, sb = K.quantize_fp8(w)
    c = K.matmul_fp8_scaled(qa.cuda(), qb.cuda(), sa, sb)
    assert rt.last_kernel_name() == "gemm_tile_fp8_bf16", rt.last_kernel_name()
    ref = orc.from_bf16(orc.matmul(bits(qa), bits(qb), in_dt=orc.FP8E4M3, out_dt=orc.BF16,
                                   scale=float(np.float32(sa) * np.float32(sb)), acc64=True))
    assert close_bf16(decode(c), ref, RTOL, fp8_atol(ref))
    assert orc.pcc(ref, decode(c)) >= PCC


def test_fp8_fast_path_small_integers_bit_exact_and_permutations():
    g = torch.Generator().manual_seed(21)
    M, N, K_ = 512, 512, 768
    a = torch.randint(-4, 5, (M, K_), generator=g).float().to(torch.float8_e4m3fn)
    b = torch.randint(-4, 5, (K_, N), generator=g).float().to(torch.float8_e4m3fn)
    c = K.matmul_fp8_scaled(a.cuda(), b.cuda(), 1.0, 1.0)
    assert rt.last_kernel_name() == "gemm_tile_fp8_bf16"
    want = orc.matmul(bits(a), bits(b), in_dt=orc.FP8E4M3, out_dt=orc.BF16, BM=128, BN=128, BK=64, group_m=8)
    assert np.array_equal(bits(c), want)
    # permutation matrices expose a mis-indexed fragment or a transposed operand
    p = torch.zeros(512, 512)
    p[torch.arange(512), (torch.arange(512) * 37 + 5) % 512] = 1
    x = torch.randint(-8, 9, (512, 512), generator=g).float()
    p8, x8 = p.to(torch.float8_e4m3fn).cuda(), x.to(torch.float8_e4m3fn).cuda()
    assert torch.equal(K.matmul_fp8_scaled(x8, p8, 1.0, 1.0).cpu().float(), x @ p)
    assert torch.equal(K.matmul_fp8_scaled(p8, x8, 1.0, 1.0).cpu().float(), p @ x)
    # scales are applied once, in fp32, before the rounding
    assert torch.equal(K.matmul_fp8_scaled(x8, p8, 0.5, 4.0).cpu().float(), (x @ p) * 2)


@pytest.mark.parametrize("M,N,K_", [(4352, 4096, 256), (4352, 4352, 256), (2048, 2048, 512), (4300, 4096, 192), (4481, 4112, 128)])
def test_fp8_fast_path_half_tile_tail(M, N, K_):
    """fp8 with a short last round of macro tiles (272, 289, 64 tiles on 256 CUs; the last two shapes take the
    clamping instantiation, the very last with lower halves that lie wholly past the matrix).  Small integers: exact."""
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-4, 5, (M, K_), generator=g).float()
    b = torch.randint(-4, 5, (K_, N), generator=g).float()
    c = K.matmul_fp8_scaled(a.to(torch.float8_e4m3fn).cuda(), b.to(torch.float8_e4m3fn).cuda(), 0.5, 4.0)
    assert rt.last_kernel_name() == ("gemm_tile_fp8_bf16" if M % 256 == 0 and N % 256 == 0 and K_ % 256 == 0 else "gemm_ragged_fp8_bf16")
    assert torch.equal(c, ((a.cuda() @ b.cuda()) * 2).to(torch.bfloat16))


def test_fp8_full_size_8192_properties():
    n = 8192
    g = torch.Generator(device="cuda").manual_seed(0)
    qa, sa = K.quantize_fp8(torch.randn(n, n, device="cuda", generator=g))
    qb, sb = K.quantize_fp8(torch.randn(n, n, device="cuda", generator=g))
    c = K.matmul_fp8_scaled(qa, qb, sa, sb)
    assert rt.last_kernel_name() == "gemm_tile_fp8_bf16"
    rows = torch.tensor([0, 255, 256, 4097, 8191], device="cuda")
    ref = ((qa[rows].double() @ qb.double()) * float(np.float32(sa) * np.float32(sb))).float()
    assert bool(torch.all((c[rows].float() - ref).abs() <= RTOL * ref.abs() + 1e-4 * ref.square().mean().sqrt()))
    cols = torch.tensor([0, 33, 4096, 8191], device="cuda")
    ref = ((qa.double() @ qb[:, cols].double()) * float(np.float32(sa) * np.float32(sb))).float()
    assert bool(torch.all((c[:, cols].float() - ref).abs() <= RTOL * ref.abs() + 1e-4 * ref.square().mean().sqrt()))
    eye = torch.eye(n, device="cuda").to(torch.float8_e4m3fn)
    assert torch.equal(K.matmul_fp8_scaled(qa, eye, 1.0, 1.0), qa.to(torch.bfloat16))   # e4m3 values are exact in bf16


def test_fp8_streaming_stores_of_an_output_beyond_the_memory_side_cache():
    """The fp8 kernels' cache-bypassing variants (a 16-bit C of more than 256 MiB, K <= 4096): small integers, so
    the whole 512 MiB output is compared bit for bit, whole tiles and clamped."""
    g = torch.Generator(device="cuda").manual_seed(6)
    for (M, N, K_), kernel in (((16384, 16384, 256), "gemm_tile_fp8_bf16_stream"), ((16380, 16400, 192), "gemm_ragged_fp8_bf16_stream")):
        a = torch.randint(-4, 5, (M, K_), device="cuda", generator=g).float()
        b = torch.randint(-4, 5, (K_, N), device="cuda", generator=g).float()
        c = K.matmul_fp8_scaled(a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn), 0.5, 4.0)
        assert rt.last_kernel_name() == kernel
        for r0 in range(0, M, 4096):
            r1 = min(r0 + 4096, M)
            assert torch.equal(c[r0:r1], ((a[r0:r1] @ b) * 2).to(torch.bfloat16))   # (sums < 2^24: exact in fp32)
        del a, b, c


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_nan_padded_descriptors(dtype):
    """`padding="nan"` (reference backend/driver.py:322-329): elements of A and B outside the matrix read as NaN.
    Rows past M and columns past N only reach results that are not stored, so the option shows exactly when K is not
    a whole number of BLOCK_SIZE_K steps, and then in every stored element (NaN * x in each sum)."""
    torch.manual_seed(5)

    def run(M, N, Kd, pad_a, pad_b, bk=64):
        a = (torch.randn(M, Kd, device="cuda") / 8).to(dtype)
        b = (torch.randn(Kd, N, device="cuda") / 8).to(dtype)
        c = torch.full((M + 1, N), 7.0, device="cuda", dtype=dtype)
        ad = TensorDescriptor.from_tensor(a, [128, bk], padding=pad_a)
        bd = TensorDescriptor.from_tensor(b, [bk, 128], padding=pad_b)
        cd = TensorDescriptor.from_tensor(c[:M], [128, 128])
        grid = (K.cdiv(M, 128) * K.cdiv(N, 128), )
        K.matmul_kernel_tma[grid](ad, bd, cd, M, N, Kd, BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=bk,
                                  GROUP_SIZE_M=8, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
        assert torch.all(c[M] == 7.0)                                 # nothing past the last row
        return a, b, c[:M], rt.last_kernel_name()

    # K a whole number of steps: the option changes nothing, ragged M and N included, and the fast kernels still run
    for shape in ((512, 512, 256), (300, 264, 128)):
        a, b, c_nan, name = run(*shape, "nan", "nan")
        ref = (a.double() @ b.double()).float()
        assert not torch.isnan(c_nan).any()
        assert torch.all((c_nan.float() - ref).abs() <= 1e-2 * ref.abs() + 1e-4)
        assert name.startswith(("gemm_tile_", "gemm_ragged_"))
    # K = 96 with 64-deep steps: the second step is half padding.  NaN on either operand poisons every element
    for pads in (("nan", "zero"), ("zero", "nan"), ("nan", "nan")):
        _, _, c, name = run(256, 256, 96, *pads)
        assert torch.isnan(c).all() and name.startswith("gemm_any_")
    # the same shape with zero padding on both is an ordinary product
    a, b, c, _ = run(256, 256, 96, "zero", "zero")
    ref = (a.double() @ b.double()).float()
    assert torch.all((c.float() - ref).abs() <= 1e-2 * ref.abs() + 1e-4)
    # 32-deep steps divide 96: no padding along K, no NaN
    _, _, c, _ = run(256, 256, 96, "nan", "nan", bk=32)
    assert not torch.isnan(c).any()


def test_repeat_launches_take_the_cached_path_and_keep_the_checks():
    """From the second launch of a call shape on, the descriptor matmuls go through a cached closure (the
    configuration's pre_hook, then one C call).  Whatever the closure does not recognise falls back to the full path:
    same results, same refusals."""
    g = torch.Generator().manual_seed(5)
    M, N, K_ = 300, 328, 224
    a = torch.randint(-3, 4, (M, K_), generator=g).to(torch.bfloat16).cuda()
    b = torch.randint(-3, 4, (K_, N), generator=g).to(torch.bfloat16).cuda()
    want = (a.float() @ b.float()).to(torch.bfloat16)
    for _ in range(3):
        assert torch.equal(K.matmul_tma(a, b), want)
    assert K.matmul_kernel_tma._plan is not None
    # the pre_hook still patches the descriptors it is handed (09-persistent-matmul.py:90-100)
    c = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
    launch = K.matmul_kernel_tma[(K.cdiv(M, 128) * K.cdiv(N, 128), )]
    launch(ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert torch.equal(c, want)
    assert ad.block_shape == [128, 64] and bd.block_shape == [64, 128] and cd.block_shape == [128, 128]
    # another dtype, another shape, a strided view, a dimension of 1: same answers as a first launch
    a16, b16 = a.half(), b.half()
    assert torch.equal(K.matmul_tma(a16, b16), (a16.float() @ b16.float()).half())
    assert torch.equal(K.matmul_tma(a[:40], b), want[:40])
    abuf = torch.zeros(M, K_ + 8, dtype=torch.bfloat16, device="cuda")
    abuf[:, :K_] = a
    assert torch.equal(K.matmul_tma(abuf[:, :K_], b), want)
    assert torch.equal(K.matmul_tma(a[:1], b), want[:1])
    assert torch.equal(K.matmul_tma(a, b), want)
    # a dimension of 1 is another specialisation (Triton folds the value): it gets a closure of its own, which serves
    # the launches that have the 1 in the same places and hands every other one back to the full path
    plans = []
    for rows in (1, 1, 1, 40, 1, 1):
        assert torch.equal(K.matmul_tma(a[:rows], b), want[:rows])
        plans.append(K.matmul_kernel_tma._plan[3])
    assert plans[1] is plans[2] and plans[4] is plans[5] and plans[3] is not plans[2]
    assert torch.equal(K.matmul_tma(a, b[:, :8])[:, :1], want[:, :1])
    # and the same refusals
    c.fill_(7.5)
    with pytest.raises(ValueError):
        launch(ad, bd, cd, M, N, K_ + 8, FP8_OUTPUT=False, WARP_SPECIALIZE=False)      # K that the descriptors do not have
    with pytest.raises(ValueError):
        launch(ad, bd, TensorDescriptor.from_tensor(c[:, :64], [32, 32]), M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    with pytest.raises((ValueError, TypeError)):
        launch(ad, bd, c, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)           # a tensor where a descriptor belongs
    assert torch.all(c == 7.5)
    # a side stream is picked up by the cached path too
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        launch(ad, bd, cd, M, N, K_, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    side.synchronize()
    assert torch.equal(c, want)
    # the fused kernel with a named epilogue and the scaled fp8 kernel have the closure too
    bias = torch.randn(N, generator=g).cuda()
    first = K.matmul_fused(a, b, bias, epilogue="bias_row")
    for _ in range(2):
        assert torch.equal(K.matmul_fused(a, b, bias, epilogue="bias_row"), first)
    assert K.matmul_kernel_fused._plan is not None
    assert torch.equal(first, ((a.float() @ b.float()) + bias).to(torch.bfloat16))
    qa, sa = K.quantize_fp8(a[:, :192].float())           # fp8 rows must be whole 16-byte pieces
    qb, sb = K.quantize_fp8(b[:192, :320].float())
    first = K.matmul_fp8_scaled(qa, qb, sa, sb)
    for _ in range(2):
        assert torch.equal(K.matmul_fp8_scaled(qa, qb, sa, sb), first)
    assert K.matmul_kernel_tma_fp8_scaled._plan is not None


@pytest.mark.gpu
def test_clock_probe_reports_a_plausible_core_clock_and_leaves_results_alone():
    """rt_gemm_clock_probe arms ONE launch of the 16-bit macro-tile GEMM: that launch records workgroup 0's core
    cycles and wall ticks (the clock granted under load), computes what it always computes, and the launches after
    it are not probed."""
    torch.manual_seed(5)
    a = (torch.randn(4096, 4096, device="cuda") / 64).to(torch.bfloat16)
    b = (torch.randn(4096, 4096, device="cuda") / 64).to(torch.bfloat16)
    want = K.matmul_tma(a, b)
    assert rt.last_kernel_name() == "gemm_tile_bf16_epi0"
    for _ in range(10):
        K.matmul_tma(a, b)
    rt.gemm_clock_probe(arm=True)
    got = K.matmul_tma(a, b)
    torch.cuda.synchronize()
    cycles, ticks, ghz = rt.gemm_clock_probe()
    assert cycles > 0 and ticks > 0 and 0.4 < ghz < 2.6, (cycles, ticks, ghz)
    assert torch.equal(got, want)
    K.matmul_tma(a, b)                       # not armed any more: the record stays as it is
    torch.cuda.synchronize()
    assert rt.gemm_clock_probe()[:2] == (cycles, ticks)
