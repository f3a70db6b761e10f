"""Helpers shared by the GPU parity tests: torch <-> oracle bit-pattern glue."""
import numpy as np
import torch

from oracle import oracle as orc


def bits(t: torch.Tensor) -> np.ndarray:
    """CPU numpy view of a tensor's raw element bits (uint16 / uint8 / native)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    return t.numpy()


def from_bits(a: np.ndarray, dtype: torch.dtype, device="cuda") -> torch.Tensor:
    a = np.ascontiguousarray(a)
    if dtype in (torch.bfloat16, torch.float16):
        return torch.from_numpy(a.view(np.int16)).view(dtype).to(device)
    if dtype == torch.float8_e4m3fn:
        return torch.from_numpy(a).view(dtype).to(device)
    return torch.from_numpy(a).to(device)


ORC_DT = {torch.bfloat16: orc.BF16, torch.float16: orc.F16, torch.float8_e4m3fn: orc.FP8E4M3, torch.float32: orc.F32}


def decode(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def close_bf16(got: np.ndarray, ref: np.ndarray, rtol=1e-2, atol=1e-4) -> bool:
    """The tile-matmul tolerance: abs(err) <= rtol*abs(ref) + atol."""
    return bool(np.all(np.abs(got - ref) <= rtol * np.abs(ref) + atol))


def p_cast_case(S: int, D: int):
    """A constructed attention input on which the placement of the bf16 cast of P (06-fused-attention.py:65-83:
    `l_ij = sum(p)` in fp32 BEFORE `p = p.to(dtype)`, and the cast itself) shows in the outputs.

    Every query is (1, 2^-8, 0, ...); key 0 is zero (score 0, the row maximum, p = 1) and every other key has a score
    whose p = exp2(score * log2e) lies just BELOW the bf16 rounding tie above 0.5 (p = 0.5 + 0.45 * 2^-8, which
    rounds to 0.5: a relative error of 3.5e-3).  V is a constant c_d in every row but row 0, which holds
    -(S-1)/2 * c_d: with P rounded, the last row's (and, unmasked, every row's) numerator 1*v_0 + 0.5*(S-1)*c_d cancels
    exactly and O = 0; with P left in fp32 it is c_d*(S-1)*0.45*2^-8 / l, tens of tolerances away.  M = log2(1 + i*p)
    from the unrounded p; summed after the cast it would be log2(1 + i/2), 5e-3 lower at the last row.

    Returns q, k, v as uint16 bf16 patterns [1,1,S,D], sm_scale, and the float64 model's (O, M) for the causal and
    the full mask under three readings: faithful, P never rounded, l summed after the cast."""
    assert (S - 1) < 256 and D >= 2
    log2e = float(np.float32(1.44269504))
    t = np.log2(0.5 + 0.45 * 2.0 ** -8) / log2e
    c0 = float(orc.from_bf16(orc.to_bf16(np.array([t], dtype=np.float32)))[0])
    c1 = float(orc.from_bf16(orc.to_bf16(np.array([(t - c0) * 256.0], dtype=np.float32)))[0])
    q = np.zeros((S, D), dtype=np.float32); q[:, 0] = 1.0; q[:, 1] = 2.0 ** -8
    k = np.zeros((S, D), dtype=np.float32); k[1:, 0] = c0; k[1:, 1] = c1
    c = np.array([(-1.0) ** d * 2.0 ** (6 + d % 4) for d in range(D)])
    v = np.tile(c, (S, 1)); v[0] = -(S - 1) / 2 * c
    p = 2.0 ** ((c0 + c1 / 256.0) * log2e)
    p_hat = float(orc.from_bf16(orc.to_bf16(np.array([p], dtype=np.float32)))[0])
    assert p_hat == 0.5 and 1e-4 < (0.5 + 2.0 ** -9) - p < 1e-3, "p must sit clear of the tie, on its lower side"

    def model(p_num, p_den, causal):
        n = np.arange(S) if causal else np.full(S, S - 1)     # keys j >= 1 a row sees
        l = 1.0 + n * p_den
        o = (v[0][None, :] + (p_num * n)[:, None] * c[None, :]) / l[:, None]
        return o, np.log2(l)

    models = {(name, causal): model(pn, pd, causal)
              for name, pn, pd in (("faithful", p_hat, p), ("p_not_rounded", p, p), ("l_after_cast", p_hat, p_hat))
              for causal in (True, False)}
    as_bits = lambda a: orc.to_bf16(a.astype(np.float32)).reshape(1, 1, S, D)
    assert np.array_equal(orc.from_bf16(as_bits(v)).reshape(S, D), v), "V must be exact in bf16"
    return as_bits(q), as_bits(k), as_bits(v), 1.0, models
