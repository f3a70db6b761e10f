"""The example kernels written as ordinary ``@triton.jit`` functions, with the
names and signatures of the reference's tutorials
(python/tutorials/01-vector-add.py:29, 01-vector-mul-add.py:30, 09-matmul-fused.py:100, examples/01-sin-kernel.py:17,
examples/matmul_tensor_descriptor/09-persistent-matmul.py:102,
examples/matmul/03-matrix-multiplication.py:242, examples/fused-attn/06-fused-attention.py:143).

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


@triton.jit
def matmul_kernel(a_ptr, b_ptr, c_ptr, M, N, K, stride_am, stride_ak, stride_bk, stride_bn, stride_cm, stride_cn,
                  BLOCK_SIZE_M: tl.constexpr, BLOCK_SIZE_N: tl.constexpr, BLOCK_SIZE_K: tl.constexpr,
                  GROUP_SIZE_M: tl.constexpr, ACTIVATION: tl.constexpr):
    # tile-major operands: tile (i, j) of a matrix with nt tiles per tile row starts at (i*nt + j) * tile elements
    pid = tl.program_id(axis=0)
    num_pid_m = tl.cdiv(M, BLOCK_SIZE_M)
    num_pid_n = tl.cdiv(N, BLOCK_SIZE_N)
    width = GROUP_SIZE_M * num_pid_n
    first_pid_m = (pid // width) * GROUP_SIZE_M
    rows = min(num_pid_m - first_pid_m, GROUP_SIZE_M)
    pid_m = first_pid_m + ((pid % width) % rows)
    pid_n = (pid % width) // rows
    num_k = tl.cdiv(K, BLOCK_SIZE_K)
    im = tl.arange(0, BLOCK_SIZE_M)
    jn = tl.arange(0, BLOCK_SIZE_N)
    kk = tl.arange(0, BLOCK_SIZE_K)
    acc = tl.zeros((BLOCK_SIZE_M, BLOCK_SIZE_N), dtype=tl.float32)
    for kt in range(num_k):
        live = kt * BLOCK_SIZE_K + kk < K
        a_tile = a_ptr + (pid_m * num_k + kt) * (BLOCK_SIZE_M * BLOCK_SIZE_K)
        b_tile = b_ptr + (kt * num_pid_n + pid_n) * (BLOCK_SIZE_K * BLOCK_SIZE_N)
        a = tl.load(a_tile + im[:, None] * BLOCK_SIZE_K + kk[None, :], mask=live[None, :], other=0.0)
        b = tl.load(b_tile + kk[:, None] * BLOCK_SIZE_N + jn[None, :], mask=live[:, None], other=0.0)
        acc = tl.dot(a, b, acc)
    if ACTIVATION == "leaky_relu":
        acc = tl.where(acc >= 0, acc, 0.01 * acc)
    c_tile = c_ptr + (pid_m * num_pid_n + pid_n) * (BLOCK_SIZE_M * BLOCK_SIZE_N)
    keep = (pid_m * BLOCK_SIZE_M + im[:, None] < M) & (pid_n * BLOCK_SIZE_N + jn[None, :] < N)
    tl.store(c_tile + im[:, None] * BLOCK_SIZE_N + jn[None, :], acc.to(tl.float16), mask=keep)


@triton.jit
def muladd_kernel(x_ptr, y_ptr, z_ptr, output_ptr, n_elements, BLOCK_SIZE: tl.constexpr):
    # python/tutorials/01-vector-mul-add.py:30-57
    pid = tl.program_id(axis=0)
    offsets = pid * BLOCK_SIZE + tl.arange(0, BLOCK_SIZE)
    mask = offsets < n_elements
    x = tl.load(x_ptr + offsets, mask=mask)
    y = tl.load(y_ptr + offsets, mask=mask)
    z = tl.load(z_ptr + offsets, mask=mask)
    tl.store(output_ptr + offsets, x * y + z, mask=mask)


@triton.jit
def matmul_kernel_fused(a_desc, b_desc, c_desc, bias_desc, M, N, K, BLOCK_SIZE_M: tl.constexpr, BLOCK_SIZE_N: tl.constexpr,
                        BLOCK_SIZE_K: tl.constexpr, GROUP_SIZE_M: tl.constexpr, FP8_OUTPUT: tl.constexpr,
                        WARP_SPECIALIZE: tl.constexpr):
    # python/tutorials/09-matmul-fused.py:100-148: the bias is a full [M,N] matrix, added in the output type after the cast
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
    c = acc.to(tl.float16)
    bias = bias_desc.load([pid_m * BLOCK_SIZE_M, pid_n * BLOCK_SIZE_N])
    c_desc.store([pid_m * BLOCK_SIZE_M, pid_n * BLOCK_SIZE_N], c + bias)


@triton.jit
def _attn_fwd(sm_scale, M, Z, H, desc_q, desc_k, desc_v, desc_o, N_CTX, HEAD_DIM: tl.constexpr, BLOCK_M: tl.constexpr,
              BLOCK_N: tl.constexpr, FP8_OUTPUT: tl.constexpr, STAGE: tl.constexpr, warp_specialize: tl.constexpr,
              IS_HOPPER: tl.constexpr):
    # examples/fused-attn/06-fused-attention.py:143-215 with its inner loop (:33-90) written out: an online softmax in
    # base 2 over key blocks; STAGE 3 is causal (whole blocks below the diagonal, then the one on it with an additive
    # -1.0e6 above the diagonal), STAGE 1 takes every key block.  M receives m_i + log2(l_i).
    tl.static_assert(BLOCK_N <= HEAD_DIM)
    start_m = tl.program_id(0)
    off_hz = tl.program_id(1)
    offset_y = (off_hz // H) * (N_CTX * H) + (off_hz % H) * N_CTX
    qo_offset_y = offset_y + start_m * BLOCK_M
    offs_m = start_m * BLOCK_M + tl.arange(0, BLOCK_M)
    offs_n = tl.arange(0, BLOCK_N)
    m_i = tl.zeros([BLOCK_M], dtype=tl.float32) - float("inf")
    l_i = tl.zeros([BLOCK_M], dtype=tl.float32) + 1.0
    acc = tl.zeros([BLOCK_M, HEAD_DIM], dtype=tl.float32)
    qk_scale = sm_scale * 1.44269504
    q = desc_q.load([qo_offset_y, 0])
    below_diagonal = start_m * BLOCK_M if STAGE == 3 else N_CTX      # keys [0, below_diagonal) need no mask
    for start_n in range(0, below_diagonal, BLOCK_N):
        k = desc_k.load([offset_y + start_n, 0]).T
        qk = tl.dot(q, k)
        m_ij = tl.maximum(m_i, tl.max(qk, 1) * qk_scale)
        qk = qk * qk_scale - m_ij[:, None]
        p = tl.math.exp2(qk)
        alpha = tl.math.exp2(m_i - m_ij)
        l_ij = tl.sum(p, 1)
        acc = acc * alpha[:, None]
        v = desc_v.load([offset_y + start_n, 0])
        acc = tl.dot(p.to(tl.bfloat16), v, acc)
        l_i = l_i * alpha + l_ij
        m_i = m_ij
    if STAGE == 3:
        for start_n in range(start_m * BLOCK_M, (start_m + 1) * BLOCK_M, BLOCK_N):
            k = desc_k.load([offset_y + start_n, 0]).T
            qk = tl.dot(q, k)
            qk = qk * qk_scale + tl.where(offs_m[:, None] >= (start_n + offs_n[None, :]), 0, -1.0e6)
            m_ij = tl.maximum(m_i, tl.max(qk, 1))
            qk -= m_ij[:, None]
            p = tl.math.exp2(qk)
            alpha = tl.math.exp2(m_i - m_ij)
            l_ij = tl.sum(p, 1)
            acc = acc * alpha[:, None]
            v = desc_v.load([offset_y + start_n, 0])
            acc = tl.dot(p.to(tl.bfloat16), v, acc)
            l_i = l_i * alpha + l_ij
            m_i = m_ij
    m_i += tl.math.log2(l_i)
    acc = acc / l_i[:, None]
    tl.store(M + off_hz * N_CTX + offs_m, m_i)
    desc_o.store([qo_offset_y, 0], acc.to(tl.bfloat16))
