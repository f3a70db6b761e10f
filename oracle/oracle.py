"""ctypes front-end of the CPU oracle (``liboracle.so`` built from ``oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The shipped package never
imports this module.

All array arguments are numpy arrays.  16-bit float types travel as
``uint16`` bit patterns and fp8 as ``uint8`` (numpy has no such dtypes); the
helpers ``to_bf16`` / ``from_bf16`` etc. convert through the same C routines
the oracle itself uses.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle.so"

F32, I32, BF16, F16, FP8E4M3 = 0, 1, 2, 3, 4
EPI_NONE, EPI_BIAS_FULL, EPI_BIAS_ROW_GELU, EPI_LEAKY_RELU, EPI_BIAS_ROW = 0, 1, 2, 3, 4

_NP_OF = {F32: np.float32, I32: np.int32, BF16: np.uint16, F16: np.uint16, FP8E4M3: np.uint8}


def build(force: bool = False) -> Path:
    """Compile ``oracle.c`` with the Makefile beside it."""
    if force and LIB_PATH.exists():
        LIB_PATH.unlink()
    subprocess.run(["make", "-C", str(HERE), "--no-print-directory"], check=True,
                   stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        L = C.CDLL(str(LIB_PATH))
        vp, i32, i64, f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float
        L.orc_convert.argtypes = [vp, C.c_int, vp, C.c_int, i64]
        L.orc_convert.restype = None
        L.orc_block_range.argtypes = [i64, C.c_int, C.c_int, C.POINTER(i64), C.POINTER(i64)]
        L.orc_block_range.restype = None
        L.orc_pid_decode.argtypes = [i64, C.c_int, C.c_int] + [C.POINTER(C.c_int)] * 3
        L.orc_pid_decode.restype = None
        L.orc_tile_of_pid.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_int)] * 2
        L.orc_tile_of_pid.restype = None
        L.orc_tile_of_pid_pointer.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_int)] * 2
        L.orc_tile_of_pid_pointer.restype = None
        for name in ("orc_add_f32", "orc_add_i32"):
            f = getattr(L, name)
            f.argtypes = [vp, vp, vp, i32, i32, i32, C.c_int]
            f.restype = None
        L.orc_muladd_f32.argtypes = [vp, vp, vp, vp, i32, i32, i32, C.c_int, C.c_int]
        L.orc_muladd_f32.restype = None
        for name in ("orc_sin_f32", "orc_sinf_f32"):
            f = getattr(L, name)
            f.argtypes = [vp, vp, i32, i32, i32, C.c_int]
            f.restype = None
        L.orc_matmul.argtypes = [vp, i64, vp, i64, vp, i64, vp, i64, i32, i32, i32, i32, i32, i32,
                                 i32, i32, C.c_int, C.c_int, C.c_int, f32, C.c_int, C.c_int]
        L.orc_matmul.restype = C.c_int
        L.orc_unary_f32.argtypes = [C.c_int, vp, vp, i32, i32, i32, C.c_int]
        L.orc_unary_f32.restype = C.c_int
        L.orc_binary_f32.argtypes = [C.c_int, vp, vp, vp, i32, i32, i32, C.c_int]
        L.orc_binary_f32.restype = C.c_int
        L.orc_binary_const_f32.argtypes = [C.c_int, vp, f32, C.c_int, vp, i32, i32, i32]
        L.orc_binary_const_f32.restype = C.c_int
        L.orc_trunci.argtypes = [vp, vp, C.c_int, i32, i32, i32]
        L.orc_reduce1d.restype = C.c_int
        L.orc_reduce1d.argtypes = [C.c_int, vp, i32, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, vp]
        L.orc_matmul_tiled.argtypes = [vp, vp, vp] + [i32] * 8 + [C.c_int] * 4
        L.orc_matmul_tiled.restype = C.c_int
        L.orc_attn_fwd.argtypes = [f32, vp, i32, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32,
                                   i32, C.c_int]
        L.orc_attn_fwd.restype = C.c_int
        L.orc_num_threads.argtypes = []
        L.orc_num_threads.restype = C.c_int
        _lib = L
    return _lib


def _p(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"] or a.ndim == 2, "oracle wants contiguous rows"
    return a.ctypes.data_as(C.c_void_p)


def num_threads() -> int:
    return int(lib().orc_num_threads())


# --------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------
def convert(src: np.ndarray, src_dt: int, dst_dt: int) -> np.ndarray:
    src = np.ascontiguousarray(src)
    dst = np.empty(src.shape, dtype=_NP_OF[dst_dt])
    lib().orc_convert(_p(src), src_dt, _p(dst), dst_dt, src.size)
    return dst


def to_bf16(x):
    return convert(np.asarray(x, dtype=np.float32), F32, BF16)


def from_bf16(x):
    return convert(np.asarray(x, dtype=np.uint16), BF16, F32)


def to_f16(x):
    return convert(np.asarray(x, dtype=np.float32), F32, F16)


def from_f16(x):
    return convert(np.asarray(x, dtype=np.uint16), F16, F32)


def to_fp8(x):
    return convert(np.asarray(x, dtype=np.float32), F32, FP8E4M3)


def from_fp8(x):
    return convert(np.asarray(x, dtype=np.uint8), FP8E4M3, F32)


def decode(x: np.ndarray, dt: int) -> np.ndarray:
    """Bit pattern array of element type ``dt`` -> float32 values."""
    return x.astype(np.float32) if dt in (F32, I32) else convert(x, dt, F32)


# --------------------------------------------------------------------------
# SPMD plumbing
# --------------------------------------------------------------------------
def block_range(num_blocks: int, num_workers: int, worker: int) -> tuple[int, int]:
    s, e = C.c_int64(), C.c_int64()
    lib().orc_block_range(num_blocks, num_workers, worker, C.byref(s), C.byref(e))
    return s.value, e.value


def pid_decode(b: int, gx: int, gy: int) -> tuple[int, int, int]:
    x, y, z = C.c_int(), C.c_int(), C.c_int()
    lib().orc_pid_decode(b, gx, gy, C.byref(x), C.byref(y), C.byref(z))
    return x.value, y.value, z.value


def tile_of_pid(pid: int, num_pid_m: int, num_pid_n: int, group_m: int) -> tuple[int, int]:
    m, n = C.c_int(), C.c_int()
    lib().orc_tile_of_pid(pid, num_pid_m, num_pid_n, group_m, C.byref(m), C.byref(n))
    return m.value, n.value


def tile_of_pid_pointer(pid: int, num_pid_m: int, num_pid_n: int, group_m: int) -> tuple[int, int]:
    """The pointer-based matmul_kernel's decode (03-matrix-multiplication.py:273-282)."""
    m, n = C.c_int(), C.c_int()
    lib().orc_tile_of_pid_pointer(pid, num_pid_m, num_pid_n, group_m, C.byref(m), C.byref(n))
    return m.value, n.value


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


# --------------------------------------------------------------------------
# kernels
# --------------------------------------------------------------------------
def add(x: np.ndarray, y: np.ndarray, out: np.ndarray | None = None, n: int | None = None,
        block: int = 1024, grid: int | None = None, nthreads: int = 0) -> np.ndarray:
    """add_kernel; dtype float32 or int32.  ``out`` keeps its contents where no
    program writes (pass a sentinel-filled array to see the mask)."""
    n = x.size if n is None else n
    grid = cdiv(n, block) if grid is None else grid
    out = np.empty_like(x) if out is None else out
    fn = {np.dtype(np.float32): lib().orc_add_f32, np.dtype(np.int32): lib().orc_add_i32}[x.dtype]
    assert y.dtype == x.dtype and out.dtype == x.dtype
    fn(_p(x), _p(y), _p(out), n, block, grid, nthreads)
    return out


def muladd(x, y, z, out=None, n=None, block=1024, grid=None, fused=True, nthreads=0):
    n = x.size if n is None else n
    grid = cdiv(n, block) if grid is None else grid
    out = np.empty_like(x) if out is None else out
    lib().orc_muladd_f32(_p(x), _p(y), _p(z), _p(out), n, block, grid, int(fused), nthreads)
    return out


def sin(x: np.ndarray, out: np.ndarray | None = None, n: int | None = None, block: int = 1024,
        grid: int | None = None, nthreads: int = 0, libm_f32: bool = False) -> np.ndarray:
    n = x.size if n is None else n
    grid = cdiv(n, block) if grid is None else grid
    out = np.empty_like(x) if out is None else out
    fn = lib().orc_sinf_f32 if libm_f32 else lib().orc_sin_f32
    fn(_p(x), _p(out), n, block, grid, nthreads)
    return out


def matmul(a: np.ndarray, b: np.ndarray, *, in_dt: int = BF16, out_dt: int = BF16,
           BM: int = 64, BN: int = 64, BK: int = 64, group_m: int = 1, grid: int | None = None,
           bias: np.ndarray | None = None, epi: int = EPI_NONE, scale: float = 1.0,
           acc64: bool = False, out: np.ndarray | None = None, nthreads: int = 0) -> np.ndarray:
    """matmul_kernel_tma / matmul_kernel_fused.  ``a`` is [M,K], ``b`` is [K,N]
    (bit patterns of ``in_dt``); returns [M,N] bit patterns of ``out_dt``."""
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    grid = cdiv(M, BM) * cdiv(N, BN) if grid is None else grid
    if out is None:
        out = np.zeros((M, N), dtype=_NP_OF[out_dt])
    ldbias = 0
    if bias is not None:
        ldbias = bias.strides[0] // bias.itemsize if bias.ndim == 2 else 0
    rc = lib().orc_matmul(_p(a), a.strides[0] // a.itemsize, _p(b), b.strides[0] // b.itemsize,
                          _p(out), out.strides[0] // out.itemsize, _p(bias), ldbias, M, N, K, BM, BN,
                          BK, group_m, grid, in_dt, out_dt, epi, scale, int(acc64), nthreads)
    if rc != 0:
        raise ValueError(f"orc_matmul rejected the launch (code {rc})")
    return out


UNARY_OPS = {"abs": 0, "ceil": 1, "cos": 2, "exp": 3, "exp2": 4, "floor": 5, "log": 6, "log2": 7, "rsqrt": 8, "sin": 9,
             "sqrt": 10}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "maximum": 4, "minimum": 5}


def unary(op: str, x: np.ndarray, *, block: int = 1024, grid: int | None = None, out: np.ndarray | None = None,
          nthreads: int = 0) -> np.ndarray:
    """out[i] = op(x[i]) in the masked-block form (ConvertComputeOps.cpp:170-180)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros_like(x) if out is None else out
    grid = cdiv(x.size, block) if grid is None else grid
    if lib().orc_unary_f32(UNARY_OPS[op], _p(x), _p(out), x.size, block, grid, nthreads):
        raise ValueError("orc_unary_f32 rejected the launch")
    return out


def binary(op: str, x: np.ndarray, y: np.ndarray, *, block: int = 1024, grid: int | None = None,
           out: np.ndarray | None = None, nthreads: int = 0) -> np.ndarray:
    """out[i] = x[i] op y[i] (ConvertComputeOps.cpp:162-167)."""
    x, y = np.ascontiguousarray(x, dtype=np.float32), np.ascontiguousarray(y, dtype=np.float32)
    out = np.zeros_like(x) if out is None else out
    grid = cdiv(x.size, block) if grid is None else grid
    if lib().orc_binary_f32(BINARY_OPS[op], _p(x), _p(y), _p(out), x.size, block, grid, nthreads):
        raise ValueError("orc_binary_f32 rejected the launch")
    return out


def binary_const(op: str, x: np.ndarray, c: float, *, flip: bool = False, block: int = 1024, grid: int | None = None,
                 out: np.ndarray | None = None) -> np.ndarray:
    """out[i] = x[i] OP c (c OP x[i] with ``flip``) in fp32; ``out`` may be ``x`` itself."""
    x = np.ascontiguousarray(x, dtype=np.float32) if out is not x else x
    if out is None:
        out = np.zeros_like(x)
    rc = lib().orc_binary_const_f32(BINARY_OPS[op], _p(x), float(np.float32(c)), int(flip), _p(out), x.size, block,
                                    cdiv(x.size, block) if grid is None else grid)
    if rc:
        raise ValueError(f"unknown binary operation {op!r}")
    return out


def copy(x: np.ndarray, out: np.ndarray, n: int, *, block: int = 1024, grid: int | None = None) -> np.ndarray:
    """The masked block moved unchanged: program p of ``grid`` stores out[i] = x[i] for the i of
    [p*block, (p+1)*block) with i < n, and every other element of ``out`` keeps what it held
    (masked load and store, cpu/lib/TritonCPUToLLVM/MaskedOpsToLLVM.cpp:33-114).  Any element type; bits move."""
    grid = cdiv(max(n, 0), block) if grid is None else grid
    x, out = x.reshape(-1), out.reshape(-1)
    for p in range(grid):
        lo, hi = p * block, min((p + 1) * block, n)
        if lo < hi:
            out[lo:hi] = x[lo:hi]
    return out


def trunci(x: np.ndarray, bits: int, *, block: int = 1024, grid: int | None = None) -> np.ndarray:
    """arith.trunci int32 -> int16 / int8 (ConvertComputeOps.cpp:182)."""
    x = np.ascontiguousarray(x, dtype=np.int32)
    out = np.zeros(x.shape, dtype=np.int16 if bits == 16 else np.int8)
    lib().orc_trunci(_p(x), _p(out), bits, x.size, block, cdiv(x.size, block) if grid is None else grid)
    return out


REDUCE_OPS = {"sum": 0, "min": 1, "max": 2, "argmin": 3, "argmax": 4, "xor_sum": 5}
I16, I8, I64, F64, U8, U16, U32, U64 = 5, 6, 7, 8, 9, 10, 11, 12
_RED_NP = {F32: np.float32, I32: np.int32, BF16: np.uint16, F16: np.uint16, I16: np.int16, I8: np.int8, I64: np.int64,
           F64: np.float64, U8: np.uint8, U16: np.uint16, U32: np.uint32, U64: np.uint64}


def reduce1d(x: np.ndarray, op: str, in_dt: int, *, acc_dt: int | None = None, out_dt: int | None = None,
             tie_break_left: bool = True, propagate_nan: bool = False):
    """tl.<op>(x, axis=0) of one BLOCK-sized tensor, folded from the left in the accumulate type of
    the IR (test_core.py::test_reduce1d, run by .github/workflows/integration-tests-cpu.yml:105).
    bf16 / f16 data travel as uint16 bit patterns.  Returns a numpy scalar of the output type."""
    acc_dt = in_dt if acc_dt is None else acc_dt
    if out_dt is None:
        out_dt = I32 if op in ("argmin", "argmax") else acc_dt
    x = np.ascontiguousarray(x, dtype=_RED_NP[in_dt])
    z = np.zeros(1, dtype=_RED_NP[out_dt])
    rc = lib().orc_reduce1d(REDUCE_OPS[op], _p(x), x.size, in_dt, acc_dt, out_dt, int(tie_break_left),
                            int(propagate_nan), _p(z))
    if rc:
        raise ValueError(f"reduce1d: {op} of dtype {in_dt} accumulated in {acc_dt} stored as {out_dt} is not expressible")
    return z[0]


def tilize(x: np.ndarray, TR: int, TC: int) -> np.ndarray:
    """Row-major [R,C] -> the tile-major buffer matmul_kernel addresses
    (03-matrix-multiplication.py:326-337): tiles of TR x TC, row-major inside a tile,
    tiles in row-major order; ragged edges are zero-filled."""
    R, C = x.shape
    tr, tc = cdiv(R, TR), cdiv(C, TC)
    pad = np.zeros((tr * TR, tc * TC), dtype=x.dtype)
    pad[:R, :C] = x
    return np.ascontiguousarray(pad.reshape(tr, TR, tc, TC).transpose(0, 2, 1, 3)).reshape(-1)


def untilize(flat: np.ndarray, R: int, C: int, TR: int, TC: int) -> np.ndarray:
    """Inverse of :func:`tilize` (drops the padding)."""
    tr, tc = cdiv(R, TR), cdiv(C, TC)
    return np.ascontiguousarray(flat.reshape(tr, tc, TR, TC).transpose(0, 2, 1, 3).reshape(tr * TR, tc * TC)[:R, :C])


def matmul_tiled(a_tiled: np.ndarray, b_tiled: np.ndarray, M: int, N: int, K: int, *, in_dt: int = F16,
                 BM: int = 32, BN: int = 32, BK: int = 32, group_m: int = 1, grid: int | None = None,
                 leaky_relu: bool = False, acc64: bool = False, out: np.ndarray | None = None,
                 nthreads: int = 0) -> np.ndarray:
    """matmul_kernel (03-matrix-multiplication.py:242-391) on tile-major buffers;
    returns the tile-major fp16 C buffer (uint16 patterns)."""
    assert a_tiled.size >= cdiv(M, BM) * cdiv(K, BK) * BM * BK and b_tiled.size >= cdiv(K, BK) * cdiv(N, BN) * BK * BN
    grid = cdiv(M, BM) * cdiv(N, BN) if grid is None else grid
    if out is None:
        out = np.zeros(cdiv(M, BM) * cdiv(N, BN) * BM * BN, dtype=np.uint16)
    rc = lib().orc_matmul_tiled(_p(a_tiled), _p(b_tiled), _p(out), M, N, K, BM, BN, BK, group_m, grid, in_dt,
                                int(leaky_relu), int(acc64), nthreads)
    if rc != 0:
        raise ValueError(f"orc_matmul_tiled rejected the launch (code {rc})")
    return out


def attn_fwd(q: np.ndarray, k: np.ndarray, v: np.ndarray, sm_scale: float, *, causal: bool = True,
             BLOCK_M: int = 64, BLOCK_N: int = 64, grid: tuple[int, int] | None = None,
             o: np.ndarray | None = None, M: np.ndarray | None = None, nthreads: int = 0):
    """_attn_fwd.  q,k,v: uint16 bf16 patterns shaped [Z,H,N_CTX,D].
    Returns (o [Z,H,N_CTX,D] uint16, M [Z,H,N_CTX] float32)."""
    Z, H, N_CTX, D = q.shape
    q, k, v = (np.ascontiguousarray(t) for t in (q, k, v))
    o = np.zeros_like(q) if o is None else o
    M = np.zeros((Z, H, N_CTX), dtype=np.float32) if M is None else M
    gx, gy = (cdiv(N_CTX, BLOCK_M), Z * H) if grid is None else grid
    rc = lib().orc_attn_fwd(sm_scale, _p(M), Z, H, _p(q), _p(k), _p(v), _p(o), N_CTX, D, BLOCK_M,
                            BLOCK_N, 3 if causal else 1, gx, gy, nthreads)
    if rc != 0:
        raise ValueError(f"orc_attn_fwd rejected the launch (code {rc})")
    return o, M


def quantize_fp8(x: np.ndarray) -> tuple[np.ndarray, float]:
    """Per-tensor e4m3 quantiser of the fp8 config: s = amax/448,
    q = saturating RNE(x / s).  Returns (uint8 codes, fp32 scale)."""
    x = np.asarray(x, dtype=np.float32)
    amax = float(np.max(np.abs(x))) if x.size else 0.0
    s = np.float32(amax / 448.0) if amax > 0 else np.float32(1.0)
    return to_fp8((x / s).astype(np.float32)), float(s)


def pcc(golden: np.ndarray, result: np.ndarray) -> float:
    """Pearson correlation on finite entries; degenerate inputs give 1.0 when
    equal and 0.0 otherwise (the acceptance measure of
    examples/01-sin-kernel.py:40-50)."""
    x = np.asarray(golden, dtype=np.float64).reshape(-1)
    y = np.asarray(result, dtype=np.float64).reshape(-1)
    m = np.isfinite(x) & np.isfinite(y)
    x, y = x[m], y[m]
    if x.size < 2 or x.std() == 0 or y.std() == 0:
        return 1.0 if np.allclose(x, y) else 0.0
    return float(np.corrcoef(x, y)[0, 1])
