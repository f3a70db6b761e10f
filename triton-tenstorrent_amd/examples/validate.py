"""Self-checks in the style of the reference's example scripts: run a kernel through the host wrapper,
compare with torch, print and bound the Pearson correlation (their acceptance bar is PCC > 0.97;
examples/01-sin-kernel.py:40-63, examples/matmul_tensor_descriptor/09-persistent-matmul.ttnn.py:256-280).

    python -m triton_tenstorrent_amd.examples.validate          # every example, on cuda:0
"""
from __future__ import annotations

import math

import torch

from .. import kernels as K

PCC_BAR = 0.97


def torch_pcc(golden: torch.Tensor, result: torch.Tensor) -> float:
    """Pearson correlation of the two tensors over the positions where both are finite.  A degenerate
    pair (fewer than two values, or either side constant) counts as 1.0 when the values agree and 0.0
    when they do not (01-sin-kernel.py:40-50)."""
    g = golden.detach().reshape(-1).to("cpu", torch.float64)
    r = result.detach().reshape(-1).to("cpu", torch.float64)
    keep = torch.isfinite(g) & torch.isfinite(r)
    g, r = g[keep], r[keep]
    if g.numel() < 2:
        return 1.0 if torch.allclose(g, r) else 0.0
    dg, dr = g - g.mean(), r - r.mean()
    sg, sr = dg.square().sum().sqrt().item(), dr.square().sum().sqrt().item()
    if sg == 0.0 or sr == 0.0:
        return 1.0 if torch.allclose(g.float(), r.float()) else 0.0
    return float((dg * dr).sum().item() / (sg * sr))


def _report(what: str, golden: torch.Tensor, result: torch.Tensor, verbose: bool) -> float:
    pcc = torch_pcc(golden, result)
    err = (golden.double().cpu() - result.double().cpu()).abs()
    err = err[torch.isfinite(err)]
    if verbose:
        print(f"{what}: PCC = {pcc:.6f}, max abs err = {err.max().item() if err.numel() else 0.0:.3e}")
    assert pcc > PCC_BAR, f"{what}: PCC too low: {pcc:.6f} (expected > {PCC_BAR})"
    return pcc


def validate_add(size: int = 98432, verbose: bool = True) -> float:
    """python/tutorials/01-vector-add.py:83-102."""
    x, y = torch.rand(size, device="cuda"), torch.rand(size, device="cuda")
    return _report(f"add size={size}", x + y, K.add(x, y), verbose)


def validate_sin(size: int, dtype=torch.float32, verbose: bool = True) -> float:
    """examples/01-sin-kernel.py:52-63."""
    x = torch.randn(size, dtype=torch.float32).to(dtype).cuda()
    return _report(f"sin size={size}", torch.sin(x.float()), K.sin(x).float(), verbose)


def validate_matmul(M: int, N: int, Kd: int, dtype=torch.bfloat16, verbose: bool = True) -> float:
    """09-persistent-matmul.ttnn.py:267-280: random A [M,K] and B [K,N] against a float32 product."""
    a = torch.randn(M, Kd).to(dtype).cuda()
    b = torch.randn(Kd, N).to(dtype).cuda()
    return _report(f"matmul_tma M={M} N={N} K={Kd}", a.float() @ b.float(), K.matmul_tma(a, b).float(), verbose)


def validate_matmul_fused(M: int, N: int, Kd: int, dtype=torch.float16, verbose: bool = True) -> float:
    """python/tutorials/09-matmul-fused.py:151-181: C = (A.B).to(dtype) + bias, bias a full [M,N] matrix."""
    a = torch.randn(M, Kd).to(dtype).cuda()
    b = torch.randn(Kd, N).to(dtype).cuda()
    bias = torch.randn(M, N).to(dtype).cuda()
    want = (a.float() @ b.float()).to(dtype).float() + bias.float()
    return _report(f"matmul_fused M={M} N={N} K={Kd}", want, K.matmul_fused(a, b, bias).float(), verbose)


def validate_matmul_pointer(M: int = 32, N: int = 32, Kd: int = 64, verbose: bool = True) -> float:
    """examples/matmul/03-matrix-multiplication.py:424-440: fp16, tile-major operands, atol 1e-2."""
    a = (torch.randn(M, Kd) / 4).to(torch.float16).cuda()
    b = (torch.randn(Kd, N) / 4).to(torch.float16).cuda()
    got = K.untilize(K.matmul_tiled(K.tilize(a, 32, 32), K.tilize(b, 32, 32), M, N, Kd), M, N, 32, 32)
    want = (a.float() @ b.float())
    assert torch.allclose(got.float(), want, atol=1e-2, rtol=0), "matmul_kernel: atol 1e-2 exceeded"
    return _report(f"matmul_kernel M={M} N={N} K={Kd}", want, got.float(), verbose)


def validate_attention(Z: int = 1, H: int = 2, N_CTX: int = 256, D: int = 64, causal: bool = True,
                       verbose: bool = True) -> float:
    """examples/fused-attn/06-fused-attention.py:224-273 against softmax(Q.K^T * sm_scale [+ causal mask]).V."""
    q, k, v = (torch.randn(Z, H, N_CTX, D).to(torch.bfloat16).cuda() for _ in range(3))
    sm_scale = 1.0 / math.sqrt(D)
    s = (q.float() @ k.float().transpose(-1, -2)) * sm_scale
    if causal:
        s = s.masked_fill(~torch.tril(torch.ones(N_CTX, N_CTX, dtype=torch.bool, device="cuda")), float("-inf"))
    want = torch.softmax(s, dim=-1) @ v.float()
    return _report(f"_attn_fwd Z={Z} H={H} N_CTX={N_CTX} D={D} causal={causal}", want,
                   K.attention(q, k, v, causal, sm_scale).float(), verbose)


def main() -> int:
    torch.manual_seed(0)
    validate_add()
    for size in (32, 1024, 98432):                                   # 01-sin-kernel.py:66-71
        validate_sin(size)
    for M, N, Kd in ((32, 32, 32), (64, 32, 32), (64, 32, 64), (1024, 1024, 1024)):   # 09-persistent-matmul.py:326-327
        validate_matmul(M, N, Kd)
    validate_matmul_fused(512, 512, 512)
    validate_matmul_pointer()
    validate_attention(causal=True)
    validate_attention(causal=False)
    print("Success!")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
