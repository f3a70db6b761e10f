"""Randomised parity on the GPU: seeded draws of shapes, dtypes, epilogues and masks for the tile matmuls, the fp8
scaled matmul and fused attention, through the reference-style wrappers, each against a float64 evaluation of the
same formula on the same inputs (computed with torch on the device).  The fixed cases of the other files pin the
corners one at a time; these draws cover the combinations in between (odd M, K that is not a multiple of 8 behind a
padded view, sequence lengths that are whole 32-query tiles but not whole blocks, every head dim), and report which
device kernels they reached."""
import math
import random

import pytest
import torch

from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu


def _close(got, ref, rtol, atol):
    return bool(torch.all((got.double() - ref).abs() <= rtol * ref.abs() + atol))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_matmuls_against_float64(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    seen = set()
    for case in range(60):
        dt = rnd.choice([torch.bfloat16, torch.float16])
        M, N, Kd = rnd.randrange(1, 1500), rnd.randrange(8, 1400, 8), rnd.randrange(8, 1600, 8)
        if rnd.random() < 0.15:
            Kd += rnd.choice([2, 4, 6])          # rows stay 16-byte aligned through a padded view; K itself is odd
        if rnd.random() < 0.3:
            M, N, Kd = rnd.randrange(256, 2049, 256), rnd.randrange(256, 2049, 256), rnd.randrange(128, 2049, 128)
        k_pad = (Kd + 7) // 8 * 8
        a = (torch.randn(M, k_pad, device="cuda") / math.sqrt(Kd)).to(dt)[:, :Kd]
        b = torch.randn(Kd, N, device="cuda").to(dt)
        what = (seed, case, dt, M, N, Kd)
        ref = a.double() @ b.double()
        c = K.matmul_tma(a, b)
        seen.add(rt.last_kernel_name())
        assert _close(c, ref, 1e-2, 1e-4), (what, rt.last_kernel_name())
        epi = rnd.choice([None, "gelu", "bias_row"])
        if epi is None:
            bias = torch.randn(M, N, device="cuda").to(dt)
            c = K.matmul_fused(a, b, bias)
            want = (ref.to(dt).double() + bias.double()).to(dt).double()      # the add happens in half precision, after the cast
            assert _close(c, want, 2e-2, 2e-2), (what, "full bias", rt.last_kernel_name())
        else:
            bias = torch.randn(N, device="cuda") * 0.5
            c = K.matmul_fused(a, b, bias, epilogue=epi)
            x = ref + bias.double()[None, :]
            want = torch.nn.functional.gelu(x) if epi == "gelu" else x
            assert _close(c, want, 1e-2, 2e-3), (what, epi, rt.last_kernel_name())
        seen.add(rt.last_kernel_name())
        # fp8 e4m3 with per-tensor scales
        M, N, Kd = rnd.randrange(1, 1200), rnd.randrange(16, 1300, 16), rnd.randrange(64, 1500, 64)
        if rnd.random() < 0.3:
            M, N, Kd = rnd.randrange(256, 1537, 256), rnd.randrange(256, 1537, 256), rnd.randrange(256, 2049, 256)
        aq, sa = K.quantize_fp8(torch.randn(M, Kd, device="cuda"))
        bq, sb = K.quantize_fp8(torch.randn(Kd, N, device="cuda"))
        c = K.matmul_fp8_scaled(aq, bq, sa, sb)
        seen.add(rt.last_kernel_name())
        ref = (aq.double() @ bq.double()) * (sa * sb)
        assert _close(c, ref, 1e-2, 1e-3 * math.sqrt(Kd)), ((seed, case, "fp8", M, N, Kd), rt.last_kernel_name())
    # the draws reach the whole-tile, the clamping and the any-shape kernels
    assert {"gemm_ragged_bf16_epi0", "gemm_tile_fp8_bf16", "gemm_ragged_fp8_bf16"} <= seen, seen
    assert any(k.startswith("gemm_any_") for k in seen) and any(k.startswith("gemm_tile_") and "fp8" not in k for k in seen), seen


@pytest.mark.parametrize("seed", [21, 22])
def test_random_attention_against_float64(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    seen = set()
    for case in range(50):
        D = rnd.choice([32, 64, 128, 128, 128, 256])
        Z, H = rnd.randint(1, 3), rnd.randint(1, 5)
        S = rnd.choice([rnd.randrange(32, 1537, 32), rnd.randrange(256, 2049, 256), rnd.randrange(128, 1025, 128)])
        causal = rnd.random() < 0.6
        sm = rnd.choice([1.0, 0.5, 2.0]) / math.sqrt(D)
        q, k, v = (torch.randn(Z, H, S, D, device="cuda").to(torch.bfloat16) for _ in range(3))
        o, lse = K.attention(q, k, v, causal, sm, return_lse=True)
        seen.add(rt.last_kernel_name())
        sc = (q.double() @ k.double().transpose(-1, -2)) * sm
        if causal:
            sc = sc.masked_fill(torch.ones(S, S, device="cuda", dtype=torch.bool).triu(1), float("-inf"))
        ref_o = torch.softmax(sc, -1) @ v.double()
        ref_m = torch.logsumexp(sc, -1) / math.log(2.0)
        what = (seed, case, Z, H, S, D, causal, rt.last_kernel_name())
        assert float((o.double() - ref_o).abs().max()) <= 2e-2, what       # the bar of tests/test_gpu_attention.py
        assert float((lse.double() - ref_m).abs().max()) <= 1e-3, what
    assert {"attn_tile_d128", "attn_ragged_d128"} <= seen, seen
