"""Host launcher for kernels built with the reference's cpu/ calling convention.

The reference's cpu/ lowering turns a Triton kernel into a host function

    kernel(user args..., i32* launch_sz, i32* launch_id, i8* smem, void* barrier)

(cpu/lib/TritonCPUToLLVM/FuncOpToLLVM.cpp:44-65, Utility.h:14-19) with

    launch_sz = [gridX, gridY, gridZ, blockX, blockY, blockZ]
    launch_id = [block_start, block_end, thread_id, 0, 0]          (GPUOpToLLVM.cpp:16-22)

and wraps its body in ``for block in [block_start, block_end)`` (Dialect/TritonCPU/Transforms/
MakePersistentKernel.cpp:144-198; a kernel without that wrapper runs the one block ``block_start``,
GPUOpToLLVM.cpp:121-129).  Program ids are decoded from the linear block index inside the kernel
(``x = b % gridX``, ``y = (b % (gridX*gridY)) / gridX``, ``z = b / (gridX*gridY)``, GPUOpToLLVM.cpp:73-101);
shared memory is 64-byte aligned (FuncOpToLLVM.cpp:150-162); every ``gpu.barrier`` calls the external
``_cpu_barrier(barrier)``, which the host supplies (GPUOpToLLVM.cpp:196-237).

The host side of this convention is not in the reference's tree (its launcher hands the shared object to the
knexus runtime, backend/driver.py:68-74, 114-170).  This module is that host side for a shared object the CALLER
supplies: ``dlopen``, look the kernel up, marshal the arguments by the launcher's type strings
(backend/driver.py:141-159: constexprs skipped, tensors as pointers), give every worker one contiguous
``[block_start, block_end)`` and run one host thread per (worker, thread_id).

The same launcher is reached through the plugin surface: ``TTUtils.load_binary`` given an ELF image (what the
reference's ``make_library`` stage produces, backend/compiler.py:452-466) loads it with ``load_image`` and hands back
a ``HostFunction``, and ``TTLauncher.__call__`` launches that on host tensors with ``launch_host`` (the launcher's
own argument walk, descriptors decomposed as Triton decomposes them).

It runs host code on host memory and nothing else: it is not a fallback for the gfx950 kernels (those fail loudly
without their library or a GPU), it refuses device tensors, and it never loads anything but the file it is given
and ``libttamd_cpuabi.so`` (the barrier).
"""
from __future__ import annotations

import ctypes as C
import os
import threading
from pathlib import Path
from typing import Any, Sequence

SUPPORT_LIB_PATH = Path(__file__).resolve().parent / "lib" / "libttamd_cpuabi.so"
SUPPORT_SYMBOLS = {
    "_cpu_barrier": (None, [C.c_void_p]),
    "ttamd_cpu_barrier_create": (C.c_void_p, [C.c_int32]),
    "ttamd_cpu_barrier_destroy": (None, [C.c_void_p]),
    "ttamd_cpu_smem_alloc": (C.c_void_p, [C.c_uint64]),
    "ttamd_cpu_smem_free": (None, [C.c_void_p]),
    "ttamd_cpu_block_range": (None, [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
}

_support = None
_support_lock = threading.Lock()


def support() -> C.CDLL:
    """``libttamd_cpuabi.so``, loaded with global symbol visibility so that a kernel library's undefined
    ``_cpu_barrier`` resolves against it."""
    global _support
    with _support_lock:
        if _support is None:
            if not SUPPORT_LIB_PATH.exists():
                raise FileNotFoundError(f"{SUPPORT_LIB_PATH} is missing: build it with "
                                        "`python -c 'import __graft_entry__ as g; g.build()'`")
            lib = C.CDLL(str(SUPPORT_LIB_PATH), mode=C.RTLD_GLOBAL)
            for name, (res, args) in SUPPORT_SYMBOLS.items():
                fn = getattr(lib, name)
                fn.restype, fn.argtypes = res, args
            _support = lib
    return _support


# launch-time type strings of the launcher (backend/driver.py:141-159) -> how the value crosses the C ABI
_SCALARS = {"i1": C.c_bool, "i8": C.c_int8, "i16": C.c_int16, "i32": C.c_int32, "i64": C.c_int64,
            "u8": C.c_uint8, "u16": C.c_uint16, "u32": C.c_uint32, "u64": C.c_uint64,
            "fp32": C.c_float, "f32": C.c_float, "fp64": C.c_double}


def _ctype_of(ty: str):
    if ty.startswith("*"):
        return C.c_void_p
    if ty in _SCALARS:
        return _SCALARS[ty]
    raise TypeError(f"Unsupported scalar type: {ty}")        # the reference launcher's wording, driver.py:295


def block_range(blocks: int, workers: int, worker: int) -> tuple[int, int]:
    """Blocks ``[start, end)`` of worker ``worker``: contiguous, in worker order, the first ``blocks % workers``
    workers one block longer (the split of npu/lib/TritonNPUToTenstorrent/D2M/SPMDOpToD2M.cpp:38-112)."""
    s, e = C.c_int32(), C.c_int32()
    support().ttamd_cpu_block_range(blocks, workers, worker, C.byref(s), C.byref(e))
    return s.value, e.value


class CPUKernel:
    """One kernel of a caller-supplied shared object, typed by its launch signature."""

    def __init__(self, library: "CPULibrary", name: str, signature: Sequence[str]):
        try:
            fn = getattr(library.handle, name)
        except AttributeError:
            raise LookupError(f"{library.path}: no kernel '{name}'") from None
        self.library, self.name = library, name
        self.signature = list(signature)
        self._launch_types = [t for t in self.signature if t != "constexpr"]
        fn.restype = None
        fn.argtypes = [_ctype_of(t) for t in self._launch_types] + [C.c_void_p] * 4
        self._fn = fn

    def _marshal(self, args: Sequence[Any]) -> tuple[list, list]:
        """User arguments in signature order (constexprs included, and skipped as the reference's launcher skips
        them) -> C values; the second list keeps tensors alive for the duration of the launch."""
        if len(args) != len(self.signature):
            raise ValueError(f"{self.name}: {len(args)} arguments for a {len(self.signature)}-entry signature")
        out, keep = [], []
        for ty, a in zip(self.signature, args):
            if ty == "constexpr":
                continue
            if ty.startswith("*"):
                if hasattr(a, "data_ptr"):
                    if getattr(a, "is_cuda", False):
                        raise ValueError(f"{self.name}: a host kernel cannot dereference device memory; "
                                         "pass CPU tensors (the gfx950 kernels are reached through TTDriver)")
                    keep.append(a)
                    out.append(a.data_ptr())
                elif hasattr(a, "ctypes") and hasattr(a, "dtype"):      # numpy array
                    keep.append(a)
                    out.append(a.ctypes.data)
                elif isinstance(a, int):
                    out.append(a)
                else:
                    raise TypeError(f"{self.name}: pointer argument of type {type(a).__name__}")
            else:
                out.append(a)
        return out, keep

    def launch(self, grid: Sequence[int], *args, shared: int = 0, num_warps: int = 1, workers: int | None = None,
               persistent: bool = True):
        """Run programs ``[0, gridX*gridY*gridZ)``: worker w gets ``block_range(blocks, workers, w)`` and runs it on
        ``num_warps`` host threads (``thread_id`` 0 .. num_warps-1; the cpu/ path has one thread per warp,
        backend/compiler.py:131-134) that share the worker's shared memory and barrier.  Returns when every
        thread has; an exception in argument marshalling is raised before anything runs.

        ``persistent``: the kernel carries the loop over ``[block_start, block_end)`` that MakePersistentKernel
        wraps around its body, so it is called once per (worker, thread) with the worker's whole range.  A kernel
        built WITHOUT that pass runs the one block ``block_start`` per call (GPUOpToLLVM.cpp:121-129): say
        ``persistent=False`` and it is called once per block, with ``[b, b + 1)``, the threads of a team meeting at
        the team's barrier between blocks (they share the worker's shared memory)."""
        g = [int(x) for x in grid] + [1, 1, 1]
        gx, gy, gz = g[:3]
        if min(gx, gy, gz) < 0 or gx * gy * gz >= 2**31:
            raise ValueError(f"{self.name}: grid {tuple(g[:3])} out of range")
        if num_warps < 1 or shared < 0:
            raise ValueError(f"{self.name}: num_warps and shared must not be negative")
        blocks = gx * gy * gz
        if blocks == 0:
            return
        if workers is None:
            workers = min(blocks, max(1, (os.cpu_count() or 1) // num_warps))
        workers = max(1, min(int(workers), blocks))
        cargs, keep = self._marshal(args)
        sup = support()
        launch_sz = (C.c_int32 * 6)(gx, gy, gz, num_warps, 1, 1)
        teams, threads, errors = [], [], []

        def run(ids, smem, barrier):
            try:
                if persistent:
                    self._fn(*cargs, C.addressof(launch_sz), C.addressof(ids), smem, barrier)
                    return
                first, last = ids[0], ids[1]
                for b in range(first, last):
                    ids[0], ids[1] = b, b + 1
                    self._fn(*cargs, C.addressof(launch_sz), C.addressof(ids), smem, barrier)
                    if num_warps > 1 and b + 1 < last:
                        sup._cpu_barrier(barrier)      # nobody starts block b+1 on shared memory that block b still reads
            except BaseException as e:      # ctypes.ArgumentError and the like: report, do not lose the thread
                errors.append(e)

        try:
            for w in range(workers):
                start, end = block_range(blocks, workers, w)
                smem = sup.ttamd_cpu_smem_alloc(shared)
                barrier = sup.ttamd_cpu_barrier_create(num_warps)
                if not smem or not barrier:
                    raise MemoryError(f"{self.name}: shared memory or barrier allocation failed")
                teams.append((smem, barrier))
                for t in range(num_warps):
                    ids = (C.c_int32 * 5)(start, end, t, 0, 0)
                    keep.append(ids)
                    threads.append(threading.Thread(target=run, args=(ids, smem, barrier), daemon=True))
            # a thread that raised before reaching a barrier would leave its team waiting: check the argument
            # conversion once, on this thread, before any team starts
            for ct, v in zip(self._fn.argtypes, cargs):
                ct(v) if ct is not C.c_void_p else C.c_void_p(v)
            if len(threads) == 1:
                run(keep[-1], *teams[0])
            else:
                for th in threads:
                    th.start()
                for th in threads:
                    th.join()
        finally:
            for smem, barrier in teams:
                sup.ttamd_cpu_smem_free(smem)
                sup.ttamd_cpu_barrier_destroy(barrier)
        if errors:
            raise errors[0]


class CPULibrary:
    """A caller-supplied shared object of cpu/-convention kernels."""

    def __init__(self, path: str | os.PathLike):
        support()        # first, so that the object's `_cpu_barrier` resolves
        self.path = str(path)
        if not Path(self.path).exists():
            raise FileNotFoundError(self.path)
        self.handle = C.CDLL(self.path)

    def get_kernel(self, name: str, signature: Sequence[str]) -> CPUKernel:
        """``signature``: the kernel's type strings in parameter order, as Triton writes them (``*fp32``, ``i32``,
        ``fp32``, ``constexpr`` ...)."""
        return CPUKernel(self, name, signature)


def load_library(path: str | os.PathLike) -> CPULibrary:
    return CPULibrary(path)


def is_elf_image(kernel) -> bool:
    """Is this ``load_binary`` payload a shared object (as opposed to the JSON record of a prebuilt gfx950 kernel)?"""
    return isinstance(kernel, (bytes, bytearray, memoryview)) and bytes(kernel[:4]) == b"\x7fELF"


def load_image(image: bytes) -> CPULibrary:
    """A shared object handed over as bytes, the way the reference's launcher hands one to its runtime
    (``device.load_library(kernel, len(kernel))``, backend/driver.py:72).  The image is written to a file of its own
    in the temporary directory, mapped by ``dlopen`` and unlinked at once: the mapping keeps the pages, nothing is left
    on disk, and two images never meet under one path name (``dlopen`` answers a path it has seen before with the
    library it loaded then)."""
    import tempfile
    if not is_elf_image(image):
        raise ValueError("not an ELF image")
    fd, path = tempfile.mkstemp(prefix="ttamd_cpu_kernel_", suffix=".so")
    try:
        with os.fdopen(fd, "wb") as f:
            f.write(bytes(image))
        return CPULibrary(path)
    finally:
        os.unlink(path)


def expand_signature(sig_types: Sequence[str]) -> list[str]:
    """Launch signature -> the types that cross the C ABI, one per value of the launcher's argument walk
    (backend/driver.py:141-159): a rank-r ``tensordesc<dtype[...]>`` becomes ``*dtype``, r shapes and r strides as
    i64, the padding flag as i1, then r shapes as i32 and r strides as i64, which is how Triton decomposes a
    descriptor that has no hardware form (triton/backends/amd/driver.py:229-256)."""
    out: list[str] = []
    for ty in sig_types:
        if isinstance(ty, str) and ty.startswith("tensordesc<"):
            dtype = ty[len("tensordesc<"):].split("[")[0]
            r = ty.count(",") + 1
            out += ["*" + dtype] + ["i64"] * (2 * r) + ["i1"] + ["i32"] * r + ["i64"] * r
        else:
            out.append(ty)
    return out


class HostFunction:
    """What ``TTUtils.load_binary`` returns as ``function`` for an ELF image: the kernel's name in a loaded
    library.  The launch signature is the launcher's, so the typed kernel is made (and kept) at the first launch."""

    host = True

    def __init__(self, library: CPULibrary, name: str):
        self.library, self.name = library, name
        self._typed: dict = {}
        if not hasattr(library.handle, name):
            raise LookupError(f"{library.path}: no kernel '{name}'")

    def typed(self, flat_types: Sequence[str]) -> CPUKernel:
        key = tuple(flat_types)
        k = self._typed.get(key)
        if k is None:
            k = self._typed[key] = CPUKernel(self.library, self.name, key)
        return k

    def __repr__(self):
        return f"<HostFunction {self.name}>"


def launch_host(function: HostFunction, sig_types: Sequence[str], grid: Sequence[int], user_args: Sequence[Any],
                num_warps: int, shared: int, persistent: bool = True) -> None:
    """``TTLauncher.__call__`` for a host kernel: the reference's argument walk (constexprs skipped, a tensor as
    its address, a descriptor as base, shape, strides, padding flag, shape, strides), then ``CPUKernel.launch``."""
    from .tensor_descriptor import is_tensor_descriptor
    flat_types = [t for t in expand_signature(sig_types) if t != "constexpr"]
    flat: list = []
    for ty, a in zip(sig_types, user_args):
        if ty == "constexpr":
            continue
        if is_tensor_descriptor(a):
            shape, strides = [int(d) for d in a.shape], [int(x) for x in a.strides]
            flat += [a.base, *shape, *strides, a.padding == "nan", *shape, *strides]
        else:
            flat.append(a)
    if len(flat) != len(flat_types):
        raise ValueError(f"{function.name}: the arguments flatten to {len(flat)} values, the signature to {len(flat_types)}")
    function.typed(flat_types).launch(grid, *flat, shared=int(shared), num_warps=max(1, int(num_warps)), persistent=persistent)
