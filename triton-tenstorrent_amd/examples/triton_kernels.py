"""The example kernels written as ordinary ``@triton.jit`` functions, with the
names and signatures of the reference's tutorials
(python/tutorials/01-vector-add.py:29, examples/01-sin-kernel.py:17,
examples/matmul_tensor_descriptor/09-persistent-matmul.py:102).

With ``backend.compiler.register()`` in effect Triton's JIT parses these on the
host, the backend binds each by name to its prebuilt gfx950 kernel and the
launcher runs it: a user script written against the reference needs no change
beyond the device its tensors live on.
"""
import triton
import triton.language as tl


@triton.jit
def add_kernel(x_ptr, y_ptr, output_ptr, n_elements, BLOCK_SIZE: tl.constexpr):
    pid = tl.program_id(axis=0)
    offsets = pid * BLOCK_SIZE + tl.arange(0, BLOCK_SIZE)
    mask = offsets < n_elements
    x = tl.load(x_ptr + offsets, mask=mask)
    y = tl.load(y_ptr + offsets, mask=mask)
    tl.store(output_ptr + offsets, x + y, mask=mask)


@triton.jit
def sin_kernel(x_ptr, output_ptr, n_elements, BLOCK_SIZE: tl.constexpr):
    pid = tl.program_id(axis=0)
    offsets = pid * BLOCK_SIZE + tl.arange(0, BLOCK_SIZE)
    mask = offsets < n_elements
    tl.store(output_ptr + offsets, tl.sin(tl.load(x_ptr + offsets, mask=mask)), mask=mask)


@triton.jit
def matmul_kernel_tma(a_desc, b_desc, c_desc, M, N, K, BLOCK_SIZE_M: tl.constexpr, BLOCK_SIZE_N: tl.constexpr,
                      BLOCK_SIZE_K: tl.constexpr, GROUP_SIZE_M: tl.constexpr, FP8_OUTPUT: tl.constexpr,
                      WARP_SPECIALIZE: tl.constexpr):
    pid = tl.program_id(axis=0)
    num_pid_m = tl.cdiv(M, BLOCK_SIZE_M)
    num_pid_n = tl.cdiv(N, BLOCK_SIZE_N)
    width = GROUP_SIZE_M * num_pid_n
    first_pid_m = (pid // width) * GROUP_SIZE_M
    rows = min(num_pid_m - first_pid_m, GROUP_SIZE_M)
    pid_m = first_pid_m + (pid % rows)
    pid_n = (pid % width) // rows
    acc = tl.zeros((BLOCK_SIZE_M, BLOCK_SIZE_N), dtype=tl.float32)
    for k in range(tl.cdiv(K, BLOCK_SIZE_K)):
        a = a_desc.load([pid_m * BLOCK_SIZE_M, k * BLOCK_SIZE_K])
        b = b_desc.load([k * BLOCK_SIZE_K, pid_n * BLOCK_SIZE_N])
        acc = tl.dot(a, b, acc)
    c_desc.store([pid_m * BLOCK_SIZE_M, pid_n * BLOCK_SIZE_N], acc.to(tl.bfloat16))
