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
