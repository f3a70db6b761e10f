"""Host-side tensor descriptor with the five fields the launcher reads
(``base, shape, strides, block_shape, padding``).

When Triton is importable its own ``triton.tools.tensor_descriptor.TensorDescriptor``
works just as well: the launcher only looks at these attributes.  This class
exists so that the C-ABI path has no Triton dependency.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List


@dataclass
class TensorDescriptor:
    base: Any
    shape: List[int]
    strides: List[int]
    block_shape: List[int]
    padding: str = "zero"

    def __post_init__(self):
        rank = len(self.shape)
        if not (0 < rank <= 5):
            raise AssertionError(f"descriptor rank must be 1..5, got {rank}")
        if len(self.strides) != rank or len(self.block_shape) != rank:
            raise AssertionError(f"shape/strides/block_shape ranks differ: {self.shape} {self.strides} {self.block_shape}")
        if self.padding not in ("zero", "nan"):
            raise AssertionError(f"padding must be 'zero' or 'nan', got {self.padding!r}")
        if any(int(s) <= 0 for s in self.shape):
            raise AssertionError(f"every dimension must be positive: {self.shape}")
        if int(self.strides[-1]) != 1:
            raise AssertionError("the last dimension must be contiguous")
        itemsize = self.base.dtype.itemsize
        if self.base.data_ptr() % 16:
            raise AssertionError("base must be 16-byte aligned")
        for s in self.strides[:-1]:
            if (int(s) * itemsize) % 16:
                raise AssertionError("leading strides must be 16-byte aligned")
        if self.padding == "nan" and not self.base.dtype.is_floating_point:
            raise AssertionError("'nan' padding needs a floating point tensor")

    @staticmethod
    def from_tensor(tensor: Any, block_shape: List[int], padding: str = "zero") -> "TensorDescriptor":
        return TensorDescriptor(tensor, list(tensor.shape), list(tensor.stride()), list(block_shape), padding)


def is_tensor_descriptor(obj: Any) -> bool:
    """Duck-typed check accepting this class and Triton's."""
    if type(obj) is TensorDescriptor:
        return True
    # block_shape first: tensors and scalars do not have it, so the common case is one lookup
    return (hasattr(obj, "block_shape") and hasattr(obj, "base") and hasattr(obj, "shape") and hasattr(obj, "strides")
            and hasattr(obj, "padding"))
