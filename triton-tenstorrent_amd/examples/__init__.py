"""User-side scripts: the example kernels as ``@triton.jit`` sources, launched
through Triton's own JIT with this backend active."""
