"""GPU parity on random shapes, one launch after the other in one process: every kernel family against float64
evaluated by torch on the device.  What it is for: faults that depend on what ran before (an accumulator read too
early showed only behind a certain sequence of other launches) and shapes nobody thought of.  Bounds: matmul
abs(err) <= 1e-2*abs(ref) + 1e-4 (fp8: + 1e-3*sqrt(K)); attention O max-abs <= 3e-2 against the exact softmax (P is
rounded to bf16 and O to bf16 of values up to 4), M <= 1e-3; elementwise and reductions as in their own tests."""
import math
import random

import pytest
import torch

from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu


def _close(got, ref, rtol=1e-2, atol=1e-4):
    return bool(torch.all((got.double() - ref).abs() <= rtol * ref.abs() + atol))


@pytest.mark.parametrize("seed", [21, 105, 406])
def test_random_shapes_in_sequence(seed):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    rdim = lambda lo, hi, mult=1: rnd.randrange(lo, hi + 1, mult)
    seen = set()
    for i in range(100):
        # 16-bit matmul: any M; N, K multiples of 8 (sometimes not: the any-shape kernel), sometimes whole tiles
        dt = rnd.choice([torch.bfloat16, torch.float16])
        M, N, Kd = rdim(1, 1500), rdim(8, 1400, 8), rdim(8, 1600, 8)
        if rnd.random() < 0.15:
            Kd += rnd.choice([2, 4, 6])
        if rnd.random() < 0.3:
            M, N, Kd = rdim(256, 2048, 256), rdim(256, 2048, 256), rdim(128, 2048, 128)
        N8, K8 = (N + 7) // 8 * 8, (Kd + 7) // 8 * 8      # descriptors need 16-byte leading strides: views of padded buffers
        a = (torch.randn(M, K8, device="cuda") / math.sqrt(Kd)).to(dt)[:, :Kd]
        b = torch.randn(Kd, N8, device="cuda").to(dt)[:, :N]
        c = K.matmul_tma(a, b)
        seen.add(rt.last_kernel_name())
        ref = a.double() @ b.double()
        assert _close(c, ref), ("matmul", i, dt, M, N, Kd, rt.last_kernel_name(), float((c.double() - ref).abs().max()))
        bias = torch.randn(N, device="cuda") * 0.5
        epi = rnd.choice(["gelu", "bias_row"])
        c = K.matmul_fused(a, b, bias, epilogue=epi)
        seen.add(rt.last_kernel_name())
        x = ref + bias.double()[None, :]
        want = torch.nn.functional.gelu(x) if epi == "gelu" else x
        assert _close(c, want, 1e-2, 2e-3), ("fused", i, epi, dt, M, N, Kd, rt.last_kernel_name())
        # few tiles under a long K
        M, N, Kd = rnd.choice([rdim(1, 300), rdim(1, 1100)]), rdim(8, 2048, 8), rdim(1024, 8192, 256)
        a = (torch.randn(M, Kd, device="cuda") / math.sqrt(Kd)).to(dt)
        b = torch.randn(Kd, N, device="cuda").to(dt)
        c = K.matmul_tma(a, b)
        seen.add(rt.last_kernel_name())
        ref = a.double() @ b.double()
        assert _close(c, ref), ("few tiles", i, dt, M, N, Kd, rt.last_kernel_name(), float((c.double() - ref).abs().max()))
        # the same for fp8 and for the tile-major kernel
        M, N, Kd = rnd.choice([rdim(1, 300), rdim(1, 1100)]), rdim(16, 2048, 16), rdim(2048, 8192, 512)
        aq, sa = K.quantize_fp8(torch.randn(M, Kd, device="cuda"))
        bq, sb = K.quantize_fp8(torch.randn(Kd, N, device="cuda"))
        c = K.matmul_fp8_scaled(aq, bq, sa, sb)
        seen.add(rt.last_kernel_name())
        ref = (aq.double() @ bq.double()) * (sa * sb)
        assert _close(c, ref, 1e-2, 1e-3 * math.sqrt(Kd)), ("fp8 few tiles", i, M, N, Kd, rt.last_kernel_name())
        M, N, Kd = rnd.choice([rdim(1, 300), rdim(1, 1100)]), rdim(1, 1500), rdim(1024, 6144, 256)
        a = (torch.randn(M, Kd, device="cuda") / math.sqrt(Kd)).to(torch.float16)
        b = torch.randn(Kd, N, device="cuda").to(torch.float16)
        act = rnd.choice(["", "leaky_relu"])
        ct = K.matmul_tiled(K.tilize(a, 32, 32), K.tilize(b, 32, 32), M, N, Kd, activation=act)
        seen.add(rt.last_kernel_name())
        ref = a.double() @ b.double()
        if act:
            ref = torch.where(ref >= 0, ref, 0.01 * ref)
        assert _close(K.untilize(ct, M, N, 32, 32), ref, 1e-2, 2e-3), ("tile-major few tiles", i, M, N, Kd, act, rt.last_kernel_name())
        # fp8 with scales
        M, N, Kd = rdim(1, 1200), rdim(16, 1300, 16), rdim(64, 1500, 64)
        if rnd.random() < 0.3:
            M, N, Kd = rdim(256, 1536, 256), rdim(256, 1536, 256), rdim(256, 2048, 256)
        aq, sa = K.quantize_fp8(torch.randn(M, Kd, device="cuda"))
        bq, sb = K.quantize_fp8(torch.randn(Kd, N, device="cuda"))
        c = K.matmul_fp8_scaled(aq, bq, sa, sb)
        seen.add(rt.last_kernel_name())
        ref = (aq.double() @ bq.double()) * (sa * sb)
        assert _close(c, ref, 1e-2, 1e-3 * math.sqrt(Kd)), ("fp8", i, M, N, Kd, rt.last_kernel_name())
        # attention
        D, Z, H = rnd.choice([32, 64, 128, 128, 128, 256, 256]), rnd.randint(1, 3), rnd.randint(1, 5)
        S = rnd.choice([rdim(32, 1536, 32), rdim(256, 2048, 256), rdim(128, 1024, 128)])
        causal = rnd.random() < 0.6
        q, k, v = (torch.randn(Z, H, S, D, device="cuda").to(torch.bfloat16) for _ in range(3))
        sm = 1.0 / math.sqrt(D) * rnd.choice([1.0, 0.5, 2.0])
        o, lse = K.attention(q, k, v, causal, sm, return_lse=True)
        seen.add(rt.last_kernel_name())
        sc = (q.double() @ k.double().transpose(-1, -2)) * sm
        if causal:
            sc = sc.masked_fill(torch.ones(S, S, device="cuda", dtype=torch.bool).triu(1), float("-inf"))
        eo = float((o.double() - torch.softmax(sc, -1) @ v.double()).abs().max())
        em = float((lse.double() - torch.logsumexp(sc, -1) / math.log(2.0)).abs().max())
        assert eo <= 3e-2 and em <= 1e-3, ("attention", i, Z, H, S, D, causal, sm, rt.last_kernel_name(), eo, em)
        # elementwise, views that start off a 16-byte boundary among them, and a reduction
        n, off = rnd.choice([rdim(1, 5000), rdim(1, 2_000_000)]), rnd.choice([0, 0, 1, 3])
        x, y = (torch.randn(n + off, device="cuda")[off:] for _ in range(2))
        assert torch.equal(K.add(x, y), x + y), ("add", i, n, off)
        seen.add(rt.last_kernel_name())
        op = rnd.choice(["exp", "sqrt", "sin", "abs", "floor"])
        xin = x.abs() + 0.01 if op == "sqrt" else x
        want = getattr(torch, op)(xin.double())
        got = K.unary(op, xin)
        assert bool(torch.all((got.double() - want).abs() <= 2e-6 * want.abs() + 2e-6)), ("unary", i, op, n, off)
        xr = torch.randn(rnd.choice([rdim(1, 4096), 2 ** rnd.randint(0, 20)]), device="cuda")
        assert int(K.reduce1d("argmax", xr)) == int(xr.argmax()), ("argmax", i, xr.numel())
        assert abs(float(K.reduce1d("sum", xr)) - float(xr.double().sum())) <= 1e-5 * float(xr.double().abs().sum()) + 1e-6
    # the sweep reached the hand-scheduled kernels it is meant for
    for name in ("gemm_splitk_reduce_bf16", "gemm_splitk_reduce_f16", "gemm_ragged_bf16_epi0", "attn_ragged_d256", "attn_tile_d128"):
        assert name in seen, (name, sorted(seen))
