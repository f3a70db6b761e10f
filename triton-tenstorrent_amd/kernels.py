"""The example kernels by name and signature, and their host wrappers.

Kernel objects take the arguments of the reference's ``@triton.jit`` functions
in the same order; host wrappers mirror the reference's own
(``add`` 01-vector-add.py:62-78, ``sin`` 01-sin-kernel.py:32-37, ``matmul_tma``
09-persistent-matmul.py:148-176, fused ``matmul_tma`` 09-matmul-fused.py:151-181,
``_attention.forward`` 06-fused-attention.py:224-273, pointer ``matmul``
03-matrix-multiplication.py:403-421).
"""
from __future__ import annotations


import torch

from .jit import Config, PrebuiltKernel
from .tensor_descriptor import TensorDescriptor, is_tensor_descriptor


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


# ---- elementwise -----------------------------------------------------------
add_kernel = PrebuiltKernel("add_kernel", ["x_ptr", "y_ptr", "output_ptr", "n_elements", "BLOCK_SIZE"], ["BLOCK_SIZE"])
add_kernel_loop = PrebuiltKernel("add_kernel", ["x_ptr", "y_ptr", "output_ptr", "n_elements", "row_count", "BLOCK_SIZE"],
                                 ["BLOCK_SIZE"])
muladd_kernel = PrebuiltKernel("muladd_kernel", ["x_ptr", "y_ptr", "z_ptr", "output_ptr", "n_elements", "BLOCK_SIZE"],
                               ["BLOCK_SIZE"])
sin_kernel = PrebuiltKernel("sin_kernel", ["x_ptr", "output_ptr", "n_elements", "BLOCK_SIZE"], ["BLOCK_SIZE"])

# the rest of the operation set the reference's compute lowering accepts (ConvertComputeOps.cpp:162-182),
# in the same masked-block form; OP is the operation's mnemonic ("exp", "maximum", ...)
unary_kernel = PrebuiltKernel("unary_kernel", ["x_ptr", "output_ptr", "n_elements", "BLOCK_SIZE", "OP"], ["BLOCK_SIZE", "OP"])
binary_kernel = PrebuiltKernel("binary_kernel", ["x_ptr", "y_ptr", "output_ptr", "n_elements", "BLOCK_SIZE", "OP"],
                               ["BLOCK_SIZE", "OP"])
cast_kernel = PrebuiltKernel("cast_kernel", ["x_ptr", "output_ptr", "n_elements", "BLOCK_SIZE"], ["BLOCK_SIZE"])


def unary(op: str, x: torch.Tensor) -> torch.Tensor:
    """``op`` in abs, ceil, cos, exp, exp2, floor, log, log2, rsqrt, sin, sqrt; fp32."""
    out = torch.empty_like(x)
    n = out.numel()
    unary_kernel[lambda meta: (cdiv(n, meta["BLOCK_SIZE"]), )](x, out, n, BLOCK_SIZE=1024, OP=op)
    return out


def binary(op: str, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """``op`` in add, sub, mul, div, maximum, minimum; fp32."""
    out = torch.empty_like(x)
    n = out.numel()
    binary_kernel[lambda meta: (cdiv(n, meta["BLOCK_SIZE"]), )](x, y, out, n, BLOCK_SIZE=1024, OP=op)
    return out


binary_const_kernel = PrebuiltKernel("binary_const_kernel", ["x_ptr", "output_ptr", "n_elements", "BLOCK_SIZE", "OP", "C", "FLIP"],
                                     ["BLOCK_SIZE", "OP", "C", "FLIP"], defaults={"FLIP": False})


def binary_const(op: str, x: torch.Tensor, c: float, flip: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """``x OP c`` (``c OP x`` with ``flip``) for ``op`` in add, sub, mul, div, maximum, minimum; fp32.  ``out`` may be
    ``x`` itself (test_core.py::test_load_store_same_ptr updates its buffer in place)."""
    out = torch.empty_like(x) if out is None else out
    n = out.numel()
    binary_const_kernel[lambda meta: (cdiv(n, meta["BLOCK_SIZE"]), )](x, out, n, BLOCK_SIZE=1024, OP=op, C=float(c), FLIP=flip)
    return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """fp32 -> bf16 / fp16 (round to nearest even) or int32 -> int16 / int8 (low bits kept)."""
    out = torch.empty(x.shape, device=x.device, dtype=dtype)
    n = out.numel()
    cast_kernel[lambda meta: (cdiv(n, meta["BLOCK_SIZE"]), )](x, out, n, BLOCK_SIZE=1024)
    return out


copy_kernel = PrebuiltKernel("copy_kernel", ["x_ptr", "output_ptr", "n_elements", "BLOCK_SIZE"], ["BLOCK_SIZE"])


def copy(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``out[i] = x[i]``: the masked block loaded and stored back unchanged, any element type."""
    out = torch.empty_like(x) if out is None else out
    n = x.numel()
    copy_kernel[lambda meta: (cdiv(n, meta["BLOCK_SIZE"]), )](x, out, n, BLOCK_SIZE=1024)
    return out


reduce1d_kernel = PrebuiltKernel("reduce1d_kernel", ["X", "Z", "BLOCK", "OP", "PROPAGATE_NAN"], ["BLOCK", "OP", "PROPAGATE_NAN"],
                                 defaults={"PROPAGATE_NAN": False})


def reduce1d(op: str, x: torch.Tensor, out_dtype: torch.dtype | None = None, propagate_nan: bool = False) -> torch.Tensor:
    """``tl.<op>(x, axis=0)`` of one block: ``op`` in sum, min, max, argmin, argmax, xor_sum
    (test_core.py::test_reduce1d).  The result has the dtype the reduction runs in (int32 for the
    index reductions and for sums of narrow integers, fp32 for min / max of bf16 and fp16) unless
    ``out_dtype`` names a narrower one."""
    from .backend.driver import reduce_acc_dtype, _torch_dtype_code
    if out_dtype is None:
        if op in ("argmin", "argmax"):
            out_dtype = torch.int32
        else:
            code = reduce_acc_dtype(op, _torch_dtype_code(x))
            from .backend import driver as _d
            out_dtype = next(k for k, v in _d._DTYPE_CODES.items() if v == code)
    z = torch.empty(1, device=x.device, dtype=out_dtype)
    reduce1d_kernel[(1, )](x, z, BLOCK=x.numel(), OP=op, PROPAGATE_NAN=propagate_nan)
    return z


def add(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    output = torch.empty_like(x)
    n_elements = output.numel()
    grid = lambda meta: (cdiv(n_elements, meta["BLOCK_SIZE"]), )
    add_kernel[grid](x, y, output, n_elements, BLOCK_SIZE=1024)
    return output


def add_loop(x: torch.Tensor, y: torch.Tensor, n_cores: int | None = None) -> torch.Tensor:
    """The loop variant: one program per core, ``row_count`` blocks each
    (01-vector-add.loop.py:68-93; the reference uses its 130 Tensix cores)."""
    from .jit import active_driver
    output = torch.empty_like(x)
    n_elements = output.numel()
    if n_cores is None:
        n_cores = active_driver().utils.get_device_properties()["multiprocessor_count"]
    BLOCK_SIZE = 1024
    n_rows = cdiv(n_elements, BLOCK_SIZE)
    row_count = cdiv(n_rows, n_cores)
    n_cores = min(n_cores, n_rows)
    add_kernel_loop[(n_cores, )](x, y, output, n_elements, row_count, BLOCK_SIZE=BLOCK_SIZE)
    return output


def muladd(x, y, z):
    output = torch.empty_like(x)
    n_elements = output.numel()
    muladd_kernel[lambda meta: (cdiv(n_elements, meta["BLOCK_SIZE"]), )](x, y, z, output, n_elements, BLOCK_SIZE=1024)
    return output


def sin(x: torch.Tensor) -> torch.Tensor:
    output = torch.empty_like(x)
    n_elements = output.numel()
    grid = lambda meta: (cdiv(n_elements, meta["BLOCK_SIZE"]), )
    sin_kernel[grid](x, output, n_elements, BLOCK_SIZE=1024)
    return output


# ---- tile matmul family ----------------------------------------------------
def _matmul_launch_metadata(grid, kernel, args):
    """flops/bytes record for profilers (09-persistent-matmul.py:60-71)."""
    M, N, K = args["M"], args["N"], args["K"]
    bytes_per_elem = 1 if args.get("FP8_OUTPUT") else 2
    return {"name": f"{kernel.name} [M={M}, N={N}, K={K}]", f"flops{bytes_per_elem * 8}": 2.0 * M * N * K,
            "bytes": bytes_per_elem * (M * K + N * K + M * N)}


def matmul_tma_set_block_size_hook(nargs):
    """Autotune pre_hook: patch the descriptors' block shapes from the chosen
    config (09-persistent-matmul.py:90-100, 09-matmul-fused.py:85-97)."""
    BM, BN, BK = nargs["BLOCK_SIZE_M"], nargs["BLOCK_SIZE_N"], nargs["BLOCK_SIZE_K"]
    nargs["a_desc"].block_shape = [BM, BK]
    nargs["b_desc"].block_shape = [BK, BN]
    nargs["c_desc"].block_shape = [BM, BN]
    if "bias_desc" in nargs and is_tensor_descriptor(nargs["bias_desc"]):
        bias = nargs["bias_desc"]
        bias.block_shape = [BM, BN] if len(bias.shape) == 2 and bias.shape[0] != 1 else ([1, BN] if len(bias.shape) == 2 else [BN])


# the MI355X configuration of BASELINE: 128x128x64 tiles; the reference's own is 64x64x64, G=1
MATMUL_CONFIG = {"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 8}
_MM_CONSTEXPRS = ["BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "GROUP_SIZE_M", "FP8_OUTPUT", "WARP_SPECIALIZE"]


def _mm_configs():
    return [Config(dict(MATMUL_CONFIG), num_stages=2, num_warps=4, pre_hook=matmul_tma_set_block_size_hook)]


matmul_kernel_tma = PrebuiltKernel("matmul_kernel_tma", ["a_desc", "b_desc", "c_desc", "M", "N", "K"] + _MM_CONSTEXPRS,
                                   _MM_CONSTEXPRS, configs=_mm_configs(), launch_metadata=_matmul_launch_metadata)
matmul_kernel_fused = PrebuiltKernel("matmul_kernel_fused",
                                     ["a_desc", "b_desc", "c_desc", "bias_desc", "M", "N", "K"] + _MM_CONSTEXPRS + ["EPILOGUE"],
                                     _MM_CONSTEXPRS + ["EPILOGUE"], configs=_mm_configs(),
                                     launch_metadata=_matmul_launch_metadata, defaults={"EPILOGUE": None})
matmul_kernel_tma_fp8_scaled = PrebuiltKernel(
    "matmul_kernel_tma_fp8_scaled", ["a_desc", "b_desc", "c_desc", "M", "N", "K", "scale_a", "scale_b"] + _MM_CONSTEXPRS,
    _MM_CONSTEXPRS, configs=_mm_configs(), launch_metadata=_matmul_launch_metadata)


def _mm_grid(M, N):
    return lambda META: (cdiv(M, META["BLOCK_SIZE_M"]) * cdiv(N, META["BLOCK_SIZE_N"]), )


def matmul_tma(a: torch.Tensor, b: torch.Tensor, warp_specialize: bool = False, **meta) -> torch.Tensor:
    assert a.dtype == b.dtype, "Incompatible dtypes"
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    M, K = a.shape
    K, N = b.shape
    c = torch.empty((M, N), device=a.device, dtype=a.dtype)
    dummy_block = [32, 32]
    a_desc = TensorDescriptor.from_tensor(a, dummy_block)
    b_desc = TensorDescriptor.from_tensor(b, dummy_block)
    c_desc = TensorDescriptor.from_tensor(c, dummy_block)
    matmul_kernel_tma[_mm_grid(M, N)](a_desc, b_desc, c_desc, M, N, K, FP8_OUTPUT=a.dtype == torch.float8_e4m3fn,
                                      WARP_SPECIALIZE=warp_specialize, **meta)
    return c


def matmul_fused(a: torch.Tensor, b: torch.Tensor, bias: torch.Tensor, warp_specialize: bool = False,
                 epilogue: str | None = None, **meta) -> torch.Tensor:
    """``epilogue=None`` with a full [M,N] bias is the reference kernel
    (c = acc.to(dtype) + bias); ``"gelu"`` / ``"bias_row"`` take an fp32 bias[N]."""
    assert a.dtype == b.dtype, "Incompatible dtypes"
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    M, K = a.shape
    K, N = b.shape
    c = torch.empty((M, N), device=a.device, dtype=a.dtype)
    if epilogue in (None, "bias", "bias_full"):
        assert bias.shape == (M, N), "Incompatible bias dimensions"
    else:
        assert bias.numel() == N, "Incompatible bias dimensions"
        bias = bias.reshape(1, N)
    dummy_block = [32, 32]
    a_desc = TensorDescriptor.from_tensor(a, dummy_block)
    b_desc = TensorDescriptor.from_tensor(b, dummy_block)
    c_desc = TensorDescriptor.from_tensor(c, dummy_block)
    bias_desc = TensorDescriptor.from_tensor(bias, dummy_block)
    matmul_kernel_fused[_mm_grid(M, N)](a_desc, b_desc, c_desc, bias_desc, M, N, K,
                                        FP8_OUTPUT=a.dtype == torch.float8_e4m3fn, WARP_SPECIALIZE=warp_specialize,
                                        EPILOGUE=epilogue, **meta)
    return c


def quantize_fp8(x: torch.Tensor) -> tuple[torch.Tensor, float]:
    """Per-tensor e4m3 quantiser: s = amax/448, q = saturating RNE(x/s)."""
    amax = x.abs().max().float().item()
    s = amax / 448.0 if amax > 0 else 1.0
    q = (x.float() / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q, s


def matmul_fp8_scaled(a_q: torch.Tensor, b_q: torch.Tensor, scale_a: float, scale_b: float,
                      out_dtype=torch.bfloat16, **meta) -> torch.Tensor:
    assert a_q.dtype == torch.float8_e4m3fn and b_q.dtype == torch.float8_e4m3fn
    M, K = a_q.shape
    K, N = b_q.shape
    c = torch.empty((M, N), device=a_q.device, dtype=out_dtype)
    dummy_block = [32, 32]
    a_desc = TensorDescriptor.from_tensor(a_q, dummy_block)
    b_desc = TensorDescriptor.from_tensor(b_q, dummy_block)
    c_desc = TensorDescriptor.from_tensor(c, dummy_block)
    matmul_kernel_tma_fp8_scaled[_mm_grid(M, N)](a_desc, b_desc, c_desc, M, N, K, float(scale_a), float(scale_b),
                                                 FP8_OUTPUT=False, WARP_SPECIALIZE=False, **meta)
    return c


# ---- fused attention -------------------------------------------------------
def _host_descriptor_pre_hook(nargs):
    """06-fused-attention.py:93-105."""
    BLOCK_M, BLOCK_N, HEAD_DIM = nargs["BLOCK_M"], nargs["BLOCK_N"], nargs["HEAD_DIM"]
    if not is_tensor_descriptor(nargs["desc_q"]):
        return
    nargs["desc_q"].block_shape = [BLOCK_M, HEAD_DIM]
    nargs["desc_v"].block_shape = [BLOCK_N, HEAD_DIM]
    nargs["desc_k"].block_shape = [BLOCK_N, HEAD_DIM]
    nargs["desc_o"].block_shape = [BLOCK_M, HEAD_DIM]


_ATTN_CONSTEXPRS = ["HEAD_DIM", "BLOCK_M", "BLOCK_N", "FP8_OUTPUT", "STAGE", "warp_specialize", "IS_HOPPER"]
# ---- pointer-based matmul_kernel on tile-major buffers ----------------------
# the reference's configuration for this backend (03-matrix-multiplication.py:213-218)
MATMUL_POINTER_CONFIG = {"BLOCK_SIZE_M": 32, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 1}
_MMP_CONSTEXPRS = ["BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "GROUP_SIZE_M", "ACTIVATION"]
matmul_kernel = PrebuiltKernel(
    "matmul_kernel", ["a_ptr", "b_ptr", "c_ptr", "M", "N", "K", "stride_am", "stride_ak", "stride_bk", "stride_bn",
                      "stride_cm", "stride_cn"] + _MMP_CONSTEXPRS, _MMP_CONSTEXPRS,
    configs=[Config(dict(MATMUL_POINTER_CONFIG), num_stages=1, num_warps=1)], defaults={"ACTIVATION": ""})


def tilize(x: torch.Tensor, TR: int, TC: int) -> torch.Tensor:
    """Row-major [R,C] -> the flat tile-major buffer ``matmul_kernel`` addresses
    (03-matrix-multiplication.py:326-337): TR x TC tiles, row-major inside a tile,
    tiles in row-major order, ragged edges zero-filled."""
    R, C_ = x.shape
    tr, tc = cdiv(R, TR), cdiv(C_, TC)
    if (tr * TR, tc * TC) != (R, C_):
        x = torch.nn.functional.pad(x, (0, tc * TC - C_, 0, tr * TR - R))
    return x.reshape(tr, TR, tc, TC).permute(0, 2, 1, 3).contiguous().reshape(-1)


def untilize(flat: torch.Tensor, R: int, C_: int, TR: int, TC: int) -> torch.Tensor:
    """Inverse of :func:`tilize`, dropping the padding."""
    tr, tc = cdiv(R, TR), cdiv(C_, TC)
    return flat.reshape(tr, tc, TR, TC).permute(0, 2, 1, 3).reshape(tr * TR, tc * TC)[:R, :C_].contiguous()


def matmul_tiled(a_buf: torch.Tensor, b_buf: torch.Tensor, M: int, N: int, K: int, activation: str = "",
                 **meta) -> torch.Tensor:
    """Launch ``matmul_kernel`` on tile-major buffers (as :func:`tilize` makes them) and
    return the flat tile-major fp16 result; any M, N, K."""
    cfg = {**MATMUL_POINTER_CONFIG, **meta}
    BM, BN = cfg["BLOCK_SIZE_M"], cfg["BLOCK_SIZE_N"]
    c = torch.empty(cdiv(M, BM) * cdiv(N, BN) * BM * BN, device=a_buf.device, dtype=torch.float16)
    grid = lambda META: (cdiv(M, META["BLOCK_SIZE_M"]) * cdiv(N, META["BLOCK_SIZE_N"]), )
    # strides as the reference's wrapper passes them: those of row-major [M,K], [K,N], [M,N] views
    matmul_kernel[grid](a_buf, b_buf, c, M, N, K, K, 1, N, 1, N, 1, ACTIVATION=activation, **meta)
    return c


def matmul(a: torch.Tensor, b: torch.Tensor, activation: str = "", **meta) -> torch.Tensor:
    """The reference's wrapper (03-matrix-multiplication.py:403-421): ``a`` [M,K] and ``b``
    [K,N] are handed to the kernel as they lie in memory, and the kernel reads that memory
    tile-major; so is the [M,N] fp16 result laid out.  Without padding that needs whole tiles."""
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.is_contiguous(), "Matrix A must be contiguous"
    M, K = a.shape
    K, N = b.shape
    cfg = {**MATMUL_POINTER_CONFIG, **meta}
    assert M % cfg["BLOCK_SIZE_M"] == 0 and N % cfg["BLOCK_SIZE_N"] == 0 and K % cfg["BLOCK_SIZE_K"] == 0, \
        "tile-major operands without padding need whole tiles; use matmul_tiled on padded buffers"
    c = torch.empty((M, N), device=a.device, dtype=torch.float16)
    grid = lambda META: (cdiv(M, META["BLOCK_SIZE_M"]) * cdiv(N, META["BLOCK_SIZE_N"]), )
    matmul_kernel[grid](a, b, c, M, N, K, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                        ACTIVATION=activation, **meta)
    return c


_attn_fwd = PrebuiltKernel("_attn_fwd", ["sm_scale", "M", "Z", "H", "desc_q", "desc_k", "desc_v", "desc_o", "N_CTX"] +
                           _ATTN_CONSTEXPRS, _ATTN_CONSTEXPRS,
                           configs=[Config({"BLOCK_M": 128, "BLOCK_N": 64}, num_warps=4, pre_hook=_host_descriptor_pre_hook)])


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, causal: bool, sm_scale: float,
              warp_specialize: bool = False, return_lse: bool = False, **meta):
    """``_attention.forward`` (06-fused-attention.py:224-273): q,k,v [Z,H,N_CTX,D] bf16."""
    HEAD_DIM_Q, HEAD_DIM_K, HEAD_DIM_V = q.shape[-1], k.shape[-1], v.shape[-1]
    assert HEAD_DIM_Q == HEAD_DIM_K and HEAD_DIM_K == HEAD_DIM_V
    assert HEAD_DIM_K in {16, 32, 64, 128, 256}
    o = torch.empty_like(q)
    stage = 3 if causal else 1
    M = torch.empty((q.shape[0], q.shape[1], q.shape[2]), device=q.device, dtype=torch.float32)
    y_dim = q.shape[0] * q.shape[1] * q.shape[2]
    dummy_block = [1, 1]
    desc_q = TensorDescriptor(q, shape=[y_dim, HEAD_DIM_K], strides=[HEAD_DIM_K, 1], block_shape=dummy_block)
    desc_v = TensorDescriptor(v, shape=[y_dim, HEAD_DIM_K], strides=[HEAD_DIM_K, 1], block_shape=dummy_block)
    desc_k = TensorDescriptor(k, shape=[y_dim, HEAD_DIM_K], strides=[HEAD_DIM_K, 1], block_shape=dummy_block)
    desc_o = TensorDescriptor(o, shape=[y_dim, HEAD_DIM_K], strides=[HEAD_DIM_K, 1], block_shape=dummy_block)
    if "BLOCK_M" not in meta and q.shape[2] % 128:
        meta["BLOCK_M"] = 32 if q.shape[2] % 64 else 64      # the largest of the reference's block sizes that divides N_CTX
    if "BLOCK_N" not in meta:
        meta["BLOCK_N"] = min(meta.get("BLOCK_M", 128), 64, HEAD_DIM_K)

    def grid(META):
        return (cdiv(q.shape[2], META["BLOCK_M"]), q.shape[0] * q.shape[1], 1)

    _attn_fwd[grid](sm_scale, M, q.shape[0], q.shape[1], desc_q, desc_k, desc_v, desc_o, N_CTX=q.shape[2],
                    HEAD_DIM=HEAD_DIM_K, FP8_OUTPUT=False, STAGE=stage, warp_specialize=warp_specialize,
                    IS_HOPPER=False, **meta)
    return (o, M) if return_lse else o
