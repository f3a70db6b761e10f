"""Driver and launcher of the plugin surface, MI355X edition.

Mirrors the reference's ``backend/driver.py``: ``TTUtils`` (:63-82),
``TTLauncher`` (:85-170), ``TTDeviceInterface`` (:390-442) and ``TTDriver``
(:445-535), with the knexus/ttrt device replaced by ``libttamd_rt.so``.  The
launcher keeps the reference's call signature and argument walk, then binds the
kernel NAME to the matching ``tt_*`` entry point of the C ABI.
"""
from __future__ import annotations

import ctypes as C
import functools
import json
import threading
import time
from typing import Callable

from .. import runtime as rt
from ..tensor_descriptor import is_tensor_descriptor

try:  # Triton present: be a real DriverBase so set_active()/backends discovery accept us
    from triton.backends.driver import DriverBase as _DriverBase
    from triton.backends.compiler import GPUTarget
    _HAVE_TRITON = True
except Exception:  # C-ABI-only use
    _HAVE_TRITON = False

    class _DriverBase:  # type: ignore
        def __init__(self) -> None:
            pass

    class GPUTarget:  # type: ignore
        def __init__(self, backend, arch, warp_size):
            self.backend, self.arch, self.warp_size = backend, arch, warp_size

        def __repr__(self):
            return f"GPUTarget(backend={self.backend!r}, arch={self.arch!r}, warp_size={self.warp_size})"


BINARY_EXT = "ttamd"  # the "binary" of a kernel is a small JSON record naming the prebuilt kernel


# --------------------------------------------------------------------------
# signature handling
# --------------------------------------------------------------------------
def _typestr_dtype(ty: str) -> int:
    """'*fp32' / '*bf16' / 'tensordesc<bf16[128,64]>' -> tt_dtype."""
    t = ty
    if t.startswith("tensordesc<"):
        t = t[len("tensordesc<"):].split("[")[0]
    t = t.lstrip("*")
    if t not in rt.DTYPE_OF_TYPESTR:
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, f"element type {ty!r} has no kernel")
    return rt.DTYPE_OF_TYPESTR[t]


_DTYPE_CODES: dict | None = None


def _torch_dtype_code(t) -> int:
    global _DTYPE_CODES
    if _DTYPE_CODES is None:
        import torch
        _DTYPE_CODES = {torch.float32: rt.TT_F32, torch.int32: rt.TT_I32, torch.bfloat16: rt.TT_BF16,
                        torch.float16: rt.TT_F16, torch.float8_e4m3fn: rt.TT_FP8E4M3, torch.int16: rt.TT_I16,
                        torch.int8: rt.TT_I8, torch.int64: rt.TT_I64, torch.float64: rt.TT_F64, torch.uint8: rt.TT_U8,
                        torch.uint16: rt.TT_U16, torch.uint32: rt.TT_U32, torch.uint64: rt.TT_U64}
    code = _DTYPE_CODES.get(t.dtype)
    if code is None:
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, f"tensor dtype {t.dtype} has no kernel")
    return code


def flatten_launch_args(sig_types: list[str], args: tuple, ranks_out: list | None = None) -> list:
    """The reference launcher's argument walk (backend/driver.py:134-164):
    constexprs are skipped, a tensor contributes itself, a rank-r descriptor
    contributes ``base, shape*r, strides*r, pad, shape*r, strides*r`` and
    anything else is passed through.  The pad flag is 1 for ``padding == "nan"``
    (driver.py:326).  ``ranks_out`` receives the rank of each descriptor met."""
    flat: list = []
    for ty, arg in zip(sig_types, args):
        if ty == "constexpr":
            continue
        if is_tensor_descriptor(arg):
            if ranks_out is not None:
                ranks_out.append(len(arg.shape))
            flat.append(arg.base)
            flat.extend(int(d) for d in arg.shape)
            flat.extend(int(s) for s in arg.strides)
            flat.append(1 if arg.padding == "nan" else 0)
            flat.extend(int(d) for d in arg.shape)
            flat.extend(int(s) for s in arg.strides)
        else:
            flat.append(arg)
    return flat


class _Cursor:
    """Reads the flattened argument list back in signature order."""

    def __init__(self, flat: list, keep: list, ranks: list | None = None, consts: dict | None = None,
                 arg_names: list | None = None):
        self.flat, self.i, self.keep = flat, 0, keep
        self.ranks = ranks if ranks is not None else []     # consumed from the front by desc()
        self.consts = consts if consts is not None else {}
        self.arg_names = arg_names if arg_names is not None else []
        self.direct = None      # set by a binder that offers a repeat-launch closure (_streaming_direct)

    def _next(self):
        if self.i >= len(self.flat):
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "the launch arguments ran out before the kernel's parameters did "
                                   "(a tensor where a tensor descriptor belongs?)")
        v = self.flat[self.i]
        self.i += 1
        return v

    def tensor(self, dtype_hint: int | None = None):
        t = self._next()
        if not hasattr(t, "data_ptr"):
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"expected a tensor argument, got {type(t).__name__}")
        if not t.is_cuda:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "tensor arguments must live on the GPU")
        self.keep.append(t)
        return t

    def scalar(self, name: str | None = None):
        """Next launch-time scalar; a parameter that Triton specialised to a
        constexpr (an int equal to 1) is absent from the launch list and is
        read from the constants instead."""
        if name is not None and name in self.consts:
            return self.consts[name]
        return self._next()

    def has(self, name: str) -> bool:
        return name in self.arg_names

    def named(self) -> dict:
        """Every parameter by name: constexprs from the constants, the rest from the launch list in order
        (no descriptors: used for the pointer-and-scalar kernels matched by shape)."""
        out = {}
        for name in self.arg_names:
            out[name] = self.consts[name] if name in self.consts else self._next()
        return out

    def desc(self) -> rt.tt_desc2d:
        rank = self.ranks.pop(0) if self.ranks else 2
        base = self.tensor()
        shape = [self._next() for _ in range(rank)]
        strides = [self._next() for _ in range(rank)]
        pad = self._next()
        shape2 = [self._next() for _ in range(rank)]
        strides2 = [self._next() for _ in range(rank)]
        assert shape == shape2 and strides == strides2
        if rank == 1:  # a vector is the [1, n] matrix
            shape, strides = [1, shape[0]], [shape[0], 1]
        return rt.make_desc(base.data_ptr(), shape, strides, None, _torch_dtype_code(base),
                            "nan" if pad else "zero")

    def done(self):
        if self.i != len(self.flat):
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID,
                                   f"{len(self.flat) - self.i} launch arguments left over for this kernel")


def _contiguous_1d(t):
    if t.dim() > 1 and not t.is_contiguous():
        raise ValueError("elementwise kernels index their operands linearly: pass contiguous tensors")  # driver.py:272-274
    return t


def _check_extent(who: str, n: int, grid, per_program: int, *tensors):
    """The launch touches elements [0, min(n, grid * per_program)) of every operand: each tensor has to hold that
    many, or the kernel would read or write past an allocation (a GPU memory fault, not a Python error)."""
    touched = min(max(int(n), 0), int(grid[0]) * int(per_program))
    for t in tensors:
        if t.numel() < touched:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"{who}: the launch covers {touched} elements, an operand holds "
                                                      f"{t.numel()}")


def _tensor_type():
    """The class a repeat-launch closure accepts as a tensor operand (exactly this class: a subclass may override
    what the closure reads).  Looked up when a closure is built."""
    import torch
    return torch.Tensor


def _desc_blocks_per_thread(dtype_codes: tuple):
    """``get()`` -> (blocks, refs): one set of ``tt_desc2d`` blocks, and the ``byref`` handles to pass, PER CALLING
    THREAD.  A closure refills its blocks on every call and ``ctypes`` releases the interpreter lock for the duration
    of the C call, so blocks shared between threads would let one thread's launch read another's descriptors."""
    tls = threading.local()

    def get():
        try:
            return tls.state
        except AttributeError:
            blocks = [rt.tt_desc2d() for _ in dtype_codes]
            for blk, code in zip(blocks, dtype_codes):
                blk.dtype = code
            tls.state = (blocks, tuple(C.byref(b) for b in blocks))
            return tls.state

    return get


def _streaming_direct(fn, n_tensors: int, dtype, tail: tuple, per_program: int):
    """Repeat-launch closure for a kernel whose launch arguments are ``n_tensors`` tensors and ``n_elements``:
    ``direct(args, grid, stream)`` makes the same checks as the binder that built it (operand type, dtype, device,
    contiguity, extent) and the one C call, or returns False for anything it does not recognise, so that the
    caller takes the ordinary path (which also words the errors).  ``n_elements == 1`` is refused here because
    Triton folds that value into the specialisation: it belongs to another launcher."""
    tensor_type, grid3, check = _tensor_type(), rt.Grid3, rt.check

    def direct(args, grid, stream):
        n = args[n_tensors]
        if type(n) is not int or not 1 < n < 2147483648 or len(grid) != 1:
            return False
        gx = grid[0]
        if type(gx) is not int:
            return False
        touched = gx * per_program
        if touched > n:
            touched = n
        ptrs = []
        for t in args[:n_tensors]:
            if (type(t) is not tensor_type or t.dtype is not dtype or not t.is_cuda or t.numel() < touched
                    or not t.is_contiguous()):
                return False
            ptrs.append(t.data_ptr())
        rc = fn(*ptrs, n, *tail, grid3(gx, 1, 1), stream)
        if rc:
            check(rc)
        return True

    return direct


def _desc_matmul_direct(fn, bases: list, n_floats: int, tail: tuple, mnk: tuple = (0, 0, 0)):
    """Repeat-launch closure of the descriptor matmuls (see ``_streaming_direct``): the launch arguments are
    ``len(dtypes)`` rank-2 descriptors, then M, N, K, then ``n_floats`` floats.  The closure re-checks what selects
    the specialisation it was built under (descriptor class, rank, base dtype and device, integer M, N, K of which
    those that were 1 at the launch that built this, ``mnk``, are 1 again and the others are not: Triton folds the value
    1 into the specialisation, so a launch that differs there belongs to another launcher) and fills the calling thread's own ``tt_desc2d`` blocks, which the library reads during the call
    only; shapes, strides, alignment and the grid are validated by the library as on the ordinary path."""
    from ..tensor_descriptor import TensorDescriptor
    dtypes = tuple(t.dtype for t in bases)      # of the descriptors' base tensors at the launch that built this
    tensor_type, grid3, check, n_desc = _tensor_type(), rt.Grid3, rt.check, len(dtypes)
    my_blocks = _desc_blocks_per_thread(tuple(_torch_dtype_code(t) for t in bases))
    n_args = n_desc + 3 + n_floats
    folded = tuple(v == 1 for v in mnk)

    def direct(args, grid, stream):
        if len(args) != n_args or len(grid) != 1 or type(grid[0]) is not int:
            return False
        M, N, K = args[n_desc], args[n_desc + 1], args[n_desc + 2]
        for v, one in zip((M, N, K), folded):
            if type(v) is not int or not 0 < v < 2147483648 or (v == 1) is not one:
                return False
        blocks, refs = my_blocks()
        for blk, d, dt in zip(blocks, args, dtypes):
            if type(d) is not TensorDescriptor:
                return False
            base, shape, strides = d.base, d.shape, d.strides
            if (type(base) is not tensor_type or base.dtype is not dt or not base.is_cuda or len(shape) != 2
                    or len(strides) != 2):
                return False
            blk.base = base.data_ptr()
            blk.shape[0], blk.shape[1] = shape
            blk.strides[0], blk.strides[1] = strides
            blk.padding_nan = d.padding == "nan"
        floats = args[n_desc + 3:]
        for f in floats:
            if type(f) is not float:
                return False
        rc = fn(*refs, M, N, K, *floats, *tail, grid3(grid[0], 1, 1), stream)
        if rc:
            check(rc)
        return True

    return direct


def _attn_direct(fn, bases: list, tail: tuple):
    """Repeat-launch closure of ``_attn_fwd`` (see ``_streaming_direct``): launch arguments sm_scale, M, Z, H, four
    rank-2 descriptors, N_CTX; ``tail`` = (HEAD_DIM, BLOCK_M, BLOCK_N, STAGE).  The checks of the binder that the
    library does not repeat (M: fp32, contiguous, Z*H*N_CTX elements) are made here; the rest is the library's."""
    import torch
    from ..tensor_descriptor import TensorDescriptor
    dtypes = tuple(t.dtype for t in bases)
    tensor_type, grid3, check, f32 = _tensor_type(), rt.Grid3, rt.check, torch.float32
    my_blocks = _desc_blocks_per_thread(tuple(_torch_dtype_code(t) for t in bases))

    def direct(args, grid, stream):
        if len(args) != 9 or not 1 <= len(grid) <= 3:
            return False
        sm_scale, M, Z, H, n_ctx = args[0], args[1], args[2], args[3], args[8]
        if (type(sm_scale) is not float or type(Z) is not int or type(H) is not int or type(n_ctx) is not int
                or Z < 1 or H < 1 or not 0 < n_ctx < 2147483648 or Z * H >= 2147483648):
            return False
        if (type(M) is not tensor_type or M.dtype is not f32 or not M.is_cuda or M.numel() < Z * H * n_ctx
                or not M.is_contiguous()):
            return False
        for g in grid:
            if type(g) is not int:
                return False
        blocks, refs = my_blocks()
        for blk, d, dt in zip(blocks, args[4:8], dtypes):
            if type(d) is not TensorDescriptor:
                return False
            base, shape, strides = d.base, d.shape, d.strides
            if (type(base) is not tensor_type or base.dtype is not dt or not base.is_cuda or len(shape) != 2
                    or len(strides) != 2):
                return False
            blk.base = base.data_ptr()
            blk.shape[0], blk.shape[1] = shape
            blk.strides[0], blk.strides[1] = strides
            blk.padding_nan = d.padding == "nan"
        rc = fn(sm_scale, M.data_ptr(), Z, H, *refs, n_ctx, *tail, grid3(*(grid + (1, 1, 1))[:3]), stream)
        if rc:
            check(rc)
        return True

    return direct


def _reduce_direct(fn, op_code: int, x_dtype, z_dtype, fixed: tuple):
    """Repeat-launch closure of ``reduce1d_kernel`` (see ``_streaming_direct``): the same checks as its binder for
    a call of the same shape, then the one C call.  ``fixed`` = (BLOCK, input, accumulate and output dtype codes,
    NaN flag), all set by the constexprs and dtypes that the closure re-checks."""
    tensor_type, grid3, check, block = _tensor_type(), rt.Grid3, rt.check, fixed[0]

    def direct(args, grid, stream):
        x, z = args
        if (type(x) is not tensor_type or type(z) is not tensor_type or x.dtype is not x_dtype or z.dtype is not z_dtype
                or not x.is_cuda or not z.is_cuda or x.numel() < block or z.numel() < 1 or not x.is_contiguous()
                or not 1 <= len(grid) <= 3):
            return False
        rc = fn(op_code, x.data_ptr(), z.data_ptr(), *fixed, grid3(*grid, *(1, 1, 1)[len(grid):]), stream)
        if rc:
            check(rc)
        return True

    return direct


# --------------------------------------------------------------------------
# kernel name -> C entry point
# --------------------------------------------------------------------------
def _bind_add(lib, cur: _Cursor, consts: dict, grid, stream):
    x, y, out = cur.tensor(), cur.tensor(), cur.tensor()
    n = int(cur.scalar("n_elements"))
    block = int(consts["BLOCK_SIZE"])
    for t in (x, y, out):
        _contiguous_1d(t)
    dt = _torch_dtype_code(x)
    if y.dtype != x.dtype or out.dtype != x.dtype:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "add_kernel: operand dtypes differ")
    if cur.has("row_count"):  # the loop variant
        row_count = int(cur.scalar("row_count"))
        cur.done()
        _check_extent("add_kernel", n, grid, block * max(row_count, 0), x, y, out)
        return lib.tt_add_kernel_loop(x.data_ptr(), y.data_ptr(), out.data_ptr(), n, row_count, block, dt, grid, stream)
    cur.done()
    _check_extent("add_kernel", n, grid, block, x, y, out)
    cur.direct = _streaming_direct(lib.tt_add_kernel, 3, x.dtype, (block, dt), block)
    return lib.tt_add_kernel(x.data_ptr(), y.data_ptr(), out.data_ptr(), n, block, dt, grid, stream)


def _bind_muladd(lib, cur, consts, grid, stream):
    x, y, z, out = (_contiguous_1d(cur.tensor()) for _ in range(4))
    n = int(cur.scalar("n_elements"))
    cur.done()
    for t in (x, y, z, out):
        if _torch_dtype_code(t) != rt.TT_F32:
            raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, "muladd_kernel computes in fp32")
    _check_extent("muladd_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, y, z, out)
    cur.direct = _streaming_direct(lib.tt_muladd_kernel, 4, x.dtype, (int(consts["BLOCK_SIZE"]), ),
                                   int(consts["BLOCK_SIZE"]))
    return lib.tt_muladd_kernel(x.data_ptr(), y.data_ptr(), z.data_ptr(), out.data_ptr(), n,
                                int(consts["BLOCK_SIZE"]), grid, stream)


def _bind_sin(lib, cur, consts, grid, stream):
    x, out = _contiguous_1d(cur.tensor()), _contiguous_1d(cur.tensor())
    n = int(cur.scalar("n_elements"))
    cur.done()
    if _torch_dtype_code(x) != rt.TT_F32 or _torch_dtype_code(out) != rt.TT_F32:
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, "sin_kernel computes in fp32")
    _check_extent("sin_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, out)
    cur.direct = _streaming_direct(lib.tt_sin_kernel, 2, x.dtype, (int(consts["BLOCK_SIZE"]), ),
                                   int(consts["BLOCK_SIZE"]))
    return lib.tt_sin_kernel(x.data_ptr(), out.data_ptr(), n, int(consts["BLOCK_SIZE"]), grid, stream)


def _op_code(table: dict, consts: dict, who: str) -> int:
    op = consts.get("OP")
    if op not in table:
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, f"{who}: OP {op!r}; one of {sorted(table)}")
    return table[op]


def _bind_unary(lib, cur, consts, grid, stream):
    """out[i] = OP(x[i]) for the unary operations of ConvertComputeOps.cpp:170-180."""
    x, out = _contiguous_1d(cur.tensor()), _contiguous_1d(cur.tensor())
    n = int(cur.scalar("n_elements"))
    cur.done()
    if _torch_dtype_code(x) != rt.TT_F32 or _torch_dtype_code(out) != rt.TT_F32:
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, "unary_kernel computes in fp32")
    _check_extent("unary_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, out)
    return lib.tt_unary_kernel(_op_code(rt.UNARY_OPS, consts, "unary_kernel"), x.data_ptr(), out.data_ptr(), n,
                               int(consts["BLOCK_SIZE"]), grid, stream)


def _bind_binary(lib, cur, consts, grid, stream):
    """out[i] = x[i] OP y[i] for the binary operations of ConvertComputeOps.cpp:162-167."""
    x, y, out = (_contiguous_1d(cur.tensor()) for _ in range(3))
    n = int(cur.scalar("n_elements"))
    cur.done()
    for t in (x, y, out):
        if _torch_dtype_code(t) != rt.TT_F32:
            raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, "binary_kernel computes in fp32")
    _check_extent("binary_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, y, out)
    return lib.tt_binary_kernel(_op_code(rt.BINARY_OPS, consts, "binary_kernel"), x.data_ptr(), y.data_ptr(),
                                out.data_ptr(), n, int(consts["BLOCK_SIZE"]), grid, stream)


def _bind_binary_const(lib, cur, consts, grid, stream):
    """out[i] = x[i] OP C, or C OP x[i] with FLIP: a binary operation of ConvertComputeOps.cpp:162-167 against a
    constant of the kernel."""
    x, out = _contiguous_1d(cur.tensor()), _contiguous_1d(cur.tensor())
    n = int(cur.scalar("n_elements"))
    cur.done()
    if _torch_dtype_code(x) != rt.TT_F32 or _torch_dtype_code(out) != rt.TT_F32:
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, "binary_const_kernel computes in fp32")
    _check_extent("binary_const_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, out)
    return lib.tt_binary_const_kernel(_op_code(rt.BINARY_OPS, consts, "binary_const_kernel"), x.data_ptr(), float(consts["C"]),
                                      int(bool(consts.get("FLIP", False))), out.data_ptr(), n, int(consts["BLOCK_SIZE"]),
                                      grid, stream)


def _bind_cast(lib, cur, consts, grid, stream):
    """out[i] = x[i].to(out dtype): arith.truncf / arith.trunci (ConvertComputeOps.cpp:181-182)."""
    x, out = _contiguous_1d(cur.tensor()), _contiguous_1d(cur.tensor())
    n = int(cur.scalar("n_elements"))
    cur.done()
    _check_extent("cast_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, out)
    return lib.tt_cast_kernel(x.data_ptr(), out.data_ptr(), n, int(consts["BLOCK_SIZE"]), _torch_dtype_code(x),
                              _torch_dtype_code(out), grid, stream)


def _bind_copy(lib, cur, consts, grid, stream):
    """out[i] = x[i] for i < n_elements: a masked block loaded and stored back unchanged, any element type
    (the kernel of test_launch.py::test_memory_leak, .github/workflows/integration-tests-cpu.yml:106)."""
    x, out = _contiguous_1d(cur.tensor()), _contiguous_1d(cur.tensor())
    n = int(cur.scalar("n_elements"))
    cur.done()
    if x.dtype != out.dtype:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"copy_kernel moves one element type, got {x.dtype} and {out.dtype}")
    _check_extent("copy_kernel", n, grid, int(consts["BLOCK_SIZE"]), x, out)
    return lib.tt_copy_kernel(x.data_ptr(), out.data_ptr(), n, int(consts["BLOCK_SIZE"]), _torch_dtype_code(x), grid, stream)


def _bind_empty(lib, cur, consts, grid, stream):
    """A kernel with an empty body: the launch hooks run, nothing is sent to the device."""
    return rt.RT_OK


_FLOATS = (rt.TT_F32, rt.TT_BF16, rt.TT_F16, rt.TT_F64)
_UNSIGNED = (rt.TT_U8, rt.TT_U16, rt.TT_U32, rt.TT_U64)
_NARROW = (rt.TT_I8, rt.TT_I16, rt.TT_U8, rt.TT_U16, rt.TT_BF16, rt.TT_F16)


def reduce_acc_dtype(op: str, in_dtype: int) -> int:
    """The element type Triton's front end runs ``tl.<op>`` in (triton/language/standard.py): sums of
    integers narrower than 32 bits run in (u)int32, min / max promote every type narrower than 32 bits
    to int32 or fp32, xor_sum and the index reductions keep the type."""
    if in_dtype not in _NARROW:
        return in_dtype
    if op == "sum":
        if in_dtype in _FLOATS:
            return in_dtype
        return rt.TT_U32 if in_dtype in _UNSIGNED else rt.TT_I32
    if op in ("xor_sum", "argmin", "argmax"):
        return in_dtype
    return rt.TT_F32 if in_dtype in _FLOATS else rt.TT_I32


def _bind_reduce1d(lib, cur, consts, grid, stream):
    """Z[0] = tl.<OP>(X[0:BLOCK], axis=0): the single-block reductions of test_core.py::test_reduce1d."""
    x, z = _contiguous_1d(cur.tensor()), cur.tensor()
    cur.done()
    op = consts.get("OP")
    if op not in rt.REDUCE_OPS:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"reduce1d_kernel: OP {op!r}, have {sorted(rt.REDUCE_OPS)}")
    block = int(consts["BLOCK"])
    if x.numel() < block or z.numel() < 1:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"reduce1d_kernel: X holds {x.numel()} elements, BLOCK is {block}")
    in_dt = _torch_dtype_code(x)
    fixed = (block, in_dt, reduce_acc_dtype(op, in_dt), _torch_dtype_code(z), int(bool(consts.get("PROPAGATE_NAN", False))))
    cur.direct = _reduce_direct(lib.tt_reduce1d_kernel, rt.REDUCE_OPS[op], x.dtype, z.dtype, fixed)
    return lib.tt_reduce1d_kernel(rt.REDUCE_OPS[op], x.data_ptr(), z.data_ptr(), *fixed, grid, stream)


def _mnk(cur: _Cursor, a: rt.tt_desc2d, b: rt.tt_desc2d):
    """M, N, K follow the descriptors when the signature carries them; the
    minimal variant reads them from ``desc.shape`` (kernel_matmul_tma.py:71-75).
    An int equal to 1 is specialised to a constexpr by Triton and is then
    absent from the launch list; the caller passes those through consts."""
    if cur.has("M"):
        return int(cur.scalar("M")), int(cur.scalar("N")), int(cur.scalar("K"))
    return a.shape[0], b.shape[1], a.shape[1]


def _block_consts(consts: dict, a: rt.tt_desc2d):
    bm = int(consts.get("BLOCK_SIZE_M", consts.get("BLOCK_M", 0)) or 0)
    bn = int(consts.get("BLOCK_SIZE_N", consts.get("BLOCK_N", 0)) or 0)
    bk = int(consts.get("BLOCK_SIZE_K", consts.get("BLOCK_K", 0)) or 0)
    return bm, bn, bk, int(consts.get("GROUP_SIZE_M", 1) or 1)


def _bind_matmul_tma(lib, cur, consts, grid, stream):
    a, b, c = cur.desc(), cur.desc(), cur.desc()
    M, N, K = _mnk(cur, a, b)
    bm, bn, bk, g = _block_consts(consts, a)
    bases = cur.keep[-3:]      # the three descriptors' base tensors, in order
    with_mnk = cur.has("M")    # (the minimal variant reads M, N, K from the descriptors: no closure for it)
    if cur.has("scale_a"):
        sa, sb = float(cur.scalar("scale_a")), float(cur.scalar("scale_b"))
        cur.done()
        if with_mnk:
            cur.direct = _desc_matmul_direct(lib.tt_matmul_kernel_tma_fp8_scaled, bases, 2, (bm, bn, bk, g), (M, N, K))
        return lib.tt_matmul_kernel_tma_fp8_scaled(C.byref(a), C.byref(b), C.byref(c), M, N, K, sa, sb, bm, bn, bk,
                                                   g, grid, stream)
    cur.done()
    if with_mnk:
        cur.direct = _desc_matmul_direct(lib.tt_matmul_kernel_tma, bases, 0, (bm, bn, bk, g), (M, N, K))
    return lib.tt_matmul_kernel_tma(C.byref(a), C.byref(b), C.byref(c), M, N, K, bm, bn, bk, g, grid, stream)


_EPILOGUES = {None: None, "": None, "bias": rt.TT_EPI_BIAS_FULL, "bias_full": rt.TT_EPI_BIAS_FULL,
              "bias_row": rt.TT_EPI_BIAS_ROW, "bias_row_gelu": rt.TT_EPI_BIAS_ROW_GELU, "gelu": rt.TT_EPI_BIAS_ROW_GELU,
              "leaky_relu": rt.TT_EPI_LEAKY_RELU}


def _bind_matmul_fused(lib, cur, consts, grid, stream):
    a, b, c, bias = cur.desc(), cur.desc(), cur.desc(), cur.desc()
    M, N, K = _mnk(cur, a, b)
    cur.done()
    bm, bn, bk, g = _block_consts(consts, a)
    epi = _EPILOGUES.get(consts.get("EPILOGUE"))
    if epi is None:
        # the reference kernel: full [M,N] bias of the output type; a [1,N]/[N] fp32 bias selects the row form
        full = (bias.shape[0], bias.shape[1]) == (c.shape[0], c.shape[1]) and bias.dtype == c.dtype
        epi = rt.TT_EPI_BIAS_FULL if full else rt.TT_EPI_BIAS_ROW
    # (the epilogue chosen from the bias's shape and dtype holds for repeat launches only while those stay as they
    # are: the closure is offered for the named epilogues, which do not look at the bias)
    if _EPILOGUES.get(consts.get("EPILOGUE")) is not None and "M" in cur.arg_names:
        cur.direct = _desc_matmul_direct(lib.tt_matmul_kernel_fused, cur.keep[-4:], 0, (bm, bn, bk, g, epi), (M, N, K))
    return lib.tt_matmul_kernel_fused(C.byref(a), C.byref(b), C.byref(c), C.byref(bias), M, N, K, bm, bn, bk, g, epi,
                                      grid, stream)


def _bind_matmul(lib, cur, consts, grid, stream):
    """matmul_kernel (examples/matmul/03-matrix-multiplication.py:242-260): three pointers, M, N, K and six
    strides, of which the unit ones arrive as constexprs (Triton folds an int equal to 1)."""
    a, b, c = cur.tensor(), cur.tensor(), cur.tensor()
    M, N, K = (int(cur.scalar(n)) for n in ("M", "N", "K"))
    strides = [int(cur.scalar(n)) for n in ("stride_am", "stride_ak", "stride_bk", "stride_bn", "stride_cm", "stride_cn")]
    cur.done()
    bm, bn, bk, g = _block_consts(consts, None)
    act = consts.get("ACTIVATION", "") or ""
    if act not in ("", "leaky_relu"):
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, f"matmul_kernel: ACTIVATION {act!r}; '' and 'leaky_relu' exist")
    dt = _torch_dtype_code(a)
    if _torch_dtype_code(b) != dt:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "matmul_kernel: a and b dtypes differ")
    if _torch_dtype_code(c) != rt.TT_F16:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "matmul_kernel: c must be fp16 (the kernel casts to tl.float16)")
    need = (-(-M // bm) * -(-K // bk) * bm * bk, -(-K // bk) * -(-N // bn) * bk * bn,
            -(-M // bm) * -(-N // bn) * bm * bn) if min(bm, bn, bk) > 0 else (0, 0, 0)
    for name, t, n in zip("abc", (a, b, c), need):
        if not t.is_contiguous() or t.numel() < n:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"matmul_kernel: {name} must be a contiguous tile-major buffer of "
                                   f"at least {n} elements, got {t.numel()}")
    return lib.tt_matmul_kernel(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, *strides, bm, bn, bk, g,
                                int(act == "leaky_relu"), dt, grid, stream)


def _bind_attn_fwd(lib, cur, consts, grid, stream):
    sm_scale = float(cur.scalar("sm_scale"))
    M = cur.tensor()
    Z, H = int(cur.scalar("Z")), int(cur.scalar("H"))
    q, k, v, o = cur.desc(), cur.desc(), cur.desc(), cur.desc()
    n_ctx = int(cur.scalar("N_CTX"))
    cur.done()
    if _torch_dtype_code(M) != rt.TT_F32:
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "_attn_fwd: M must be fp32")
    if M.numel() < Z * H * n_ctx or not M.is_contiguous():
        raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "_attn_fwd: M must be a contiguous [Z,H,N_CTX] tensor")
    if consts.get("FP8_OUTPUT"):
        raise rt.Unsupported(rt.RT_ERR_UNSUPPORTED, "_attn_fwd: FP8_OUTPUT is not supported")
    tail = (int(consts["HEAD_DIM"]), int(consts["BLOCK_M"]), int(consts["BLOCK_N"]), int(consts["STAGE"]))
    cur.direct = _attn_direct(lib.tt_attn_fwd, cur.keep[-4:], tail)
    return lib.tt_attn_fwd(sm_scale, M.data_ptr(), Z, H, C.byref(q), C.byref(k), C.byref(v), C.byref(o), n_ctx, *tail,
                           grid, stream)


def _bind_matched(match: dict, lib, cur, consts, grid, stream):
    """A kernel recognised by ``patterns.match_streaming``: operands by the names the IR gave, operation
    and BLOCK from the IR."""
    vals = cur.named()
    cur.done()
    if match["kernel"] == "empty_kernel":
        return rt.RT_OK
    tensors = [vals[n] for n in match["inputs"]] + [vals[match["output"]]]
    for t in tensors:
        if not hasattr(t, "data_ptr") or not t.is_cuda:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "tensor arguments must live on the GPU")
        _contiguous_1d(t)
    cur.keep.extend(tensors)
    if match.get("n") is not None:
        n = int(vals[match["n"]])
    else:
        n = int(match["n_const"]) if match.get("n_const") is not None else None     # None: one element per program
    block = int(match["block"])
    ptrs = [t.data_ptr() for t in tensors]
    if match["kernel"] == "reduce1d_kernel":
        if tensors[0].numel() < block:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"the kernel reads {block} elements, its input holds {tensors[0].numel()}")
        return lib.tt_reduce1d_kernel(rt.REDUCE_OPS[match["op"]], ptrs[0], ptrs[1], block, match["in_dtype"],
                                      match["acc_dtype"], match["out_dtype"], int(match["propagate_nan"]), grid, stream)
    if match["kernel"] == "binary_const_kernel":
        if match.get("n") is None and match.get("n_const") is None:      # one element per program: n is the grid
            n = int(grid[0])
        return lib.tt_binary_const_kernel(rt.BINARY_OPS[match["op"]], ptrs[0], float(match["c"]), int(match["flip"]), ptrs[1],
                                          n, block, grid, stream)
    if match["kernel"] == "copy_kernel":
        if tensors[0].dtype != tensors[1].dtype:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, "copy_kernel moves one element type")
        touched = min(max(n, 0), int(grid[0]) * block)
        if min(t.numel() for t in tensors) < touched:
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID, f"the kernel moves {touched} elements, a tensor holds fewer")
        return lib.tt_copy_kernel(ptrs[0], ptrs[1], n, block, match["dtype"], grid, stream)
    if match["kernel"] == "muladd_kernel":
        return lib.tt_muladd_kernel(ptrs[0], ptrs[1], ptrs[2], ptrs[3], n, block, grid, stream)
    if match["kernel"] == "add_kernel":
        return lib.tt_add_kernel(ptrs[0], ptrs[1], ptrs[2], n, block, rt.TT_I32, grid, stream)
    if match["kernel"] == "unary_kernel":
        return lib.tt_unary_kernel(rt.UNARY_OPS[match["op"]], ptrs[0], ptrs[1], n, block, grid, stream)
    if match["kernel"] == "binary_kernel":
        return lib.tt_binary_kernel(rt.BINARY_OPS[match["op"]], ptrs[0], ptrs[1], ptrs[2], n, block, grid, stream)
    return lib.tt_cast_kernel(ptrs[0], ptrs[1], n, block, _torch_dtype_code(tensors[0]), _torch_dtype_code(tensors[1]),
                              grid, stream)


KERNEL_TABLE: dict[str, Callable] = {
    "add_kernel": _bind_add,
    "muladd_kernel": _bind_muladd,
    "sin_kernel": _bind_sin,
    "unary_kernel": _bind_unary,
    "binary_kernel": _bind_binary,
    "cast_kernel": _bind_cast,
    "binary_const_kernel": _bind_binary_const,
    "copy_kernel": _bind_copy,
    "empty_kernel": _bind_empty,
    "reduce1d_kernel": _bind_reduce1d,
    "matmul_kernel_tma": _bind_matmul_tma,
    "matmul_kernel_tma_fp8_scaled": _bind_matmul_tma,
    "matmul_kernel_fused": _bind_matmul_fused,
    "matmul_kernel": _bind_matmul,
    "_attn_fwd": _bind_attn_fwd,
}


class BoundKernel:
    """What ``load_binary`` hands back as ``function``: the kernel name and its binder."""

    host = False        # (cpu_abi.HostFunction, the other kind of ``function``, says True)

    def __init__(self, name: str, record: dict):
        if name not in KERNEL_TABLE:
            raise rt.RuntimeError_(rt.RT_ERR_NOT_FOUND, f"no prebuilt kernel named {name!r}; have {sorted(KERNEL_TABLE)}")
        self.name = name
        self.record = record
        match = record.get("match")
        self.bind = functools.partial(_bind_matched, match) if match else KERNEL_TABLE[name]

    def __repr__(self):
        return f"<BoundKernel {self.name}>"


# --------------------------------------------------------------------------
# reference classes
# --------------------------------------------------------------------------
class TTUtils:
    """load_binary / get_device_properties (backend/driver.py:63-82)."""

    def __init__(self, driver: "TTDriver"):
        self.driver = driver

    def load_binary(self, name, kernel, shared_mem, device_id):
        """``kernel`` is the JSON record of a prebuilt gfx950 kernel (what ``TTBackend`` emits), or an ELF shared
        object that the CALLER built with the reference's cpu/ kernel ABI (what its ``make_library`` stage emits,
        backend/compiler.py:452-466).  The second kind is loaded as the reference loads one
        (``device.load_library(kernel, len(kernel))``, ``lib.get_kernel(name)``, backend/driver.py:68-74) and runs on
        the host, on host tensors; it needs no GPU and is never chosen for a kernel of the first kind."""
        from .. import cpu_abi
        if cpu_abi.is_elf_image(kernel):
            lib = cpu_abi.load_image(kernel)
            return (lib, cpu_abi.HostFunction(lib, name), 1, shared_mem, 2**12)
        rt.init(int(device_id or 0))
        record = json.loads(kernel.decode() if isinstance(kernel, (bytes, bytearray)) else kernel) if kernel else {}
        fn = BoundKernel(record.get("kernel", name), record)
        # (module, function, n_regs, n_spills, n_max_threads); Triton checks
        # num_warps * warp_size <= n_max_threads
        return (rt.load(), fn, 0, 0, 1024)

    def get_device_properties(self, *args):
        p = rt.device_props()
        return {"max_num_regs": p["max_num_regs"], "max_shared_mem": p["max_shared_mem"],
                "multiprocessor_count": p["multiprocessor_count"], "warpSize": p["warp_size"],
                "sm_clock_rate": p["clock_khz"], "mem_clock_rate": p["mem_clock_khz"], "mem_bus_width": p["mem_bus_bits"],
                "arch": p["arch"], "name": p["name"]}


class TTLauncher:
    """``__init__(src, metadata)`` / ``__call__(gridX, gridY, gridZ, stream,
    function, packed_metadata, launch_metadata, enter_hook, exit_hook, *args)``
    (backend/driver.py:87-111)."""

    def __init__(self, src, metadata):
        constants = src.constants if hasattr(src, "constants") else dict()
        arg_names = list(src.fn.arg_names)
        arg_idx = lambda x: (arg_names.index(x), ) if isinstance(x, str) else x
        self.constants = {arg_idx(idx): value for idx, value in constants.items()}
        self.signature = {idx: value for idx, value in src.signature.items()}
        self.arg_names = arg_names
        # One launcher serves every thread that launches this specialisation, so what a launch leaves behind is kept
        # per thread: its operands (launches are asynchronous) and the repeat-launch closure its binder offered,
        # which carries the constexprs of THAT launch (two threads may launch with different BLOCK sizes).
        self._tls = threading.local()
        # fixed per (kernel, specialisation): computed once, used on every launch
        self._sig_types = list(self.signature.values())
        self._constexpr_pos = [(i, n) for i, (n, ty) in enumerate(zip(arg_names, self._sig_types)) if ty == "constexpr"]
        self._folded = [(arg_names[idx[0]], val) for idx, val in self.constants.items()
                        if len(idx) == 1 and idx[0] < len(arg_names)]
        # a signature without descriptors flattens to "every non-constexpr argument, in order"
        self._plain_pos = None
        if not any(str(ty).startswith("tensordesc") for ty in self._sig_types):
            self._plain_pos = [i for i, ty in enumerate(self._sig_types) if ty != "constexpr"]

    @property
    def direct(self):
        """The repeat-launch closure of this thread's last launch, when its binder offers one."""
        return getattr(self._tls, "direct", None)

    @property
    def keepalive(self) -> list:
        """The operands of this thread's last launch."""
        return getattr(self._tls, "keepalive", [])

    def __call__(self, gridX, gridY, gridZ, stream, function, *args):
        kernel_metadata, launch_metadata, launch_enter_hook, launch_exit_hook = args[0], args[1], args[2], args[3]
        user_args = args[4:]
        sig_types = self._sig_types
        if len(user_args) != len(sig_types):
            raise rt.InvalidLaunch(rt.RT_ERR_INVALID,
                                   f"{function.name}: {len(user_args)} arguments for a {len(sig_types)}-entry signature")
        if function.host:
            # a caller-supplied shared object with the cpu/ kernel ABI: num_warps and the shared-memory size are
            # the launch's own (packed metadata entries 0 and 2, backend/driver.py:103-106); host tensors only
            from .. import cpu_abi
            if launch_enter_hook is not None:
                launch_enter_hook(launch_metadata)
            cpu_abi.launch_host(function, sig_types, (gridX, gridY, gridZ), user_args, kernel_metadata[0],
                                kernel_metadata[2], persistent=getattr(function, "persistent", True))
            if launch_exit_hook is not None:
                launch_exit_hook(launch_metadata)
            return
        # (num_warps / shared describe Triton codegen; the prebuilt gfx950 kernels fix their own)
        ranks: list = []
        if self._plain_pos is not None:
            flat = [user_args[i] for i in self._plain_pos]
        else:
            flat = flatten_launch_args(sig_types, user_args, ranks)
        # constexprs by name: explicit constexpr parameters plus ints Triton specialised away (value 1)
        consts = {name: user_args[i] for i, name in self._constexpr_pos}
        for name, val in self._folded:
            consts.setdefault(name, val)
        keep: list = []
        cur = _Cursor(flat, keep, ranks, consts, self.arg_names)
        lib = rt.init(0)
        grid = rt.Grid3(gridX, gridY, gridZ)
        if launch_enter_hook is not None:
            launch_enter_hook(launch_metadata)
        rc = function.bind(lib, cur, consts, grid, stream or 0)
        if rc:
            rt.check(rc)
        tls = self._tls
        tls.direct = cur.direct
        # launches are asynchronous: keep operands referenced until this thread's next launch replaces them
        tls.keepalive = keep
        if launch_exit_hook is not None:
            launch_exit_hook(launch_metadata)


class TTDeviceInterface:
    """What ``triton.testing.do_bench`` drives (backend/driver.py:390-442):
    ``Event(enable_timing)``, ``synchronize()``, optional hook timing.  Events
    are hipEvents on the current torch stream."""

    class HooksTimeAccessor:

        def __init__(self, di):
            self.di = di
            self.record_idx = 0

        def elapsed_time(self, end_event) -> float:
            return sum(self.di.kernel_times[self.record_idx:end_event.record_idx]) * 1000

        def record(self):
            self.record_idx = len(self.di.kernel_times)

    class DeviceEvent:

        def __init__(self):
            self.ev = rt.Event()

        def record(self):
            import torch
            self.ev.record(torch.cuda.current_stream().cuda_stream)

        def elapsed_time(self, end_event) -> float:
            return self.ev.elapsed_time(end_event.ev)

        def synchronize(self):
            self.ev.synchronize()

    def __init__(self):
        self.kernel_times: list[float] = []
        self.last_start = 0.0
        self.use_hooks = False

    def enable_hook_timing(self):
        self.use_hooks = True
        if _HAVE_TRITON:
            import triton
            triton.compiler.CompiledKernel.launch_enter_hook = lambda arg: self._enter_hook()
            triton.compiler.CompiledKernel.launch_exit_hook = lambda arg: self._exit_hook()

    def synchronize(self):
        import torch
        torch.cuda.synchronize()

    def _enter_hook(self):
        self.synchronize()
        self.last_start = time.perf_counter()

    def _exit_hook(self):
        self.synchronize()
        self.kernel_times.append(time.perf_counter() - self.last_start)

    def Event(self, enable_timing=True):
        if self.use_hooks:
            return TTDeviceInterface.HooksTimeAccessor(self)
        return TTDeviceInterface.DeviceEvent()


_OPTED_IN = False


def opt_in(on: bool = True) -> None:
    """Let :meth:`TTDriver.is_active` answer true in this process (``register()`` and ``activate()`` call it)."""
    global _OPTED_IN
    _OPTED_IN = bool(on)


class TTDriver(_DriverBase):
    """backend/driver.py:445-535 on an MI355X."""

    @staticmethod
    def is_active():
        """True only where this backend was asked for: after ``register()`` / ``activate()`` in this process, or
        with ``TRITON_TENSTORRENT_AMD=1`` in the environment.  Triton refuses to start with two active drivers
        (triton/runtime/driver.py:6-10), and on a ROCm box the stock HIP driver is active already, so a package
        that is merely installed (its entry point makes Triton import this module) must stay passive, as the
        reference's driver does wherever its own runtime is absent (backend/driver.py:449-467)."""
        import os
        if not (_OPTED_IN or os.environ.get("TRITON_TENSTORRENT_AMD", "") == "1"):
            return False
        try:
            import torch
            return bool(torch.cuda.is_available()) and rt.LIB_PATH.exists()
        except Exception:
            return False

    def __init__(self):
        super().__init__()
        self.utils = TTUtils(self)
        self.launcher_cls = TTLauncher

    def get_device(self, device_id=0):
        return device_id

    def get_current_device(self):
        import torch
        return torch.cuda.current_device()

    def set_current_device(self, device):
        import torch
        torch.cuda.set_device(device)

    def get_current_stream(self, device_id=None):
        import torch
        return torch.cuda.current_stream(device_id).cuda_stream

    def get_device_interface(self):
        return TTDeviceInterface()

    def get_current_target(self):
        # same backend name as the reference (driver.py:509-512) so that
        # TTBackend.supports_target and `--target tenstorrent:...` keep working;
        # arch and wavefront size are the MI355X's
        return GPUTarget("tenstorrent", "gfx950", 64)

    def get_active_torch_device(self):
        import torch
        return torch.device("cuda", self.get_current_device())

    def map_python_to_cpp_type(self, ty: str) -> str:
        return ty

    def get_benchmarker(self):
        from triton.testing import do_bench
        return do_bench

    def get_empty_cache_for_benchmark(self):
        import torch
        # 512 MiB: twice the 256 MiB last-level cache, so a clear really evicts
        return torch.empty(512 * 1024 * 1024 // 4, dtype=torch.int, device="cuda")

    def clear_cache(self, cache):
        cache.zero_()

    def get_empty_device_buffer(self, size, dtype):
        """Output allocation used by the loop/mul-add tutorials
        (python/tutorials/01-vector-add.loop.py:70)."""
        import torch
        return torch.empty(size, dtype=dtype, device="cuda")


def activate() -> TTDriver:
    """Make this driver Triton's active one (Triton allows a single active
    driver; on a ROCm box the stock HIP driver would otherwise win)."""
    opt_in()
    drv = TTDriver()
    if _HAVE_TRITON:
        import triton
        triton.runtime.driver.set_active(drv)
    return drv
