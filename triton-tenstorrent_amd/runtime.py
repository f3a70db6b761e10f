"""ctypes binding of ``libttamd_rt.so`` (declared in ``include/ttamd_rt.h``).

There is no CPU fallback: if the library has not been built, or no gfx950
device is present, every entry point raises.
"""
from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libttamd_rt.so"

RT_OK, RT_ERR_INVALID, RT_ERR_HIP, RT_ERR_NOT_FOUND, RT_ERR_UNSUPPORTED, RT_ERR_NOT_INIT = 0, -1, -2, -3, -4, -5
TT_F32, TT_I32, TT_BF16, TT_F16, TT_FP8E4M3, TT_I16, TT_I8 = 0, 1, 2, 3, 4, 5, 6
TT_I64, TT_F64, TT_U8, TT_U16, TT_U32, TT_U64 = 7, 8, 9, 10, 11, 12
# tt_unary_op / tt_binary_op of the header, by the name of the MLIR operation's mnemonic
UNARY_OPS = {"abs": 0, "ceil": 1, "cos": 2, "exp": 3, "exp2": 4, "floor": 5, "log": 6, "log2": 7, "rsqrt": 8, "sin": 9,
             "sqrt": 10}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "maximum": 4, "minimum": 5}
# tt_reduce_op of the header, by the name of the tl.* reduction
REDUCE_OPS = {"sum": 0, "min": 1, "max": 2, "argmin": 3, "argmax": 4, "xor_sum": 5}
# element type names (numpy / torch spelling) -> tt_dtype, for the reductions
DTYPE_OF_NAME = {"float32": TT_F32, "int32": TT_I32, "bfloat16": TT_BF16, "float16": TT_F16, "int16": TT_I16,
                 "int8": TT_I8, "int64": TT_I64, "float64": TT_F64, "uint8": TT_U8, "uint16": TT_U16,
                 "uint32": TT_U32, "uint64": TT_U64}
TT_EPI_NONE, TT_EPI_BIAS_FULL, TT_EPI_BIAS_ROW_GELU, TT_EPI_LEAKY_RELU, TT_EPI_BIAS_ROW = 0, 1, 2, 3, 4

# Triton pointer type strings -> tt_dtype
DTYPE_OF_TYPESTR = {"fp32": TT_F32, "i32": TT_I32, "bf16": TT_BF16, "fp16": TT_F16, "fp8e4nv": TT_FP8E4M3}


class RuntimeError_(RuntimeError):
    """A tt_*/rt_* call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[ttamd_rt {code}] {message}")
        self.code = code


class InvalidLaunch(RuntimeError_, ValueError):
    pass


class Unsupported(RuntimeError_, NotImplementedError):
    pass


class rt_props(C.Structure):
    _fields_ = [("device", C.c_int32), ("multiprocessor_count", C.c_int32), ("warp_size", C.c_int32),
                ("max_shared_mem", C.c_int32), ("max_num_regs", C.c_int32), ("clock_khz", C.c_int32),
                ("mem_clock_khz", C.c_int32), ("mem_bus_bits", C.c_int32), ("l2_bytes", C.c_int32),
                ("reserved", C.c_int32), ("total_mem", C.c_uint64), ("name", C.c_char * 128),
                ("arch", C.c_char * 64)]


class tt_desc2d(C.Structure):
    _fields_ = [("base", C.c_void_p), ("shape", C.c_int32 * 2), ("strides", C.c_int64 * 2),
                ("block_shape", C.c_int32 * 2), ("padding_nan", C.c_int32), ("dtype", C.c_int32)]


Grid3 = C.c_uint32 * 3

# name -> (restype, argtypes); must list every symbol include/ttamd_rt.h declares
_vp, _i32, _f32 = C.c_void_p, C.c_int32, C.c_float
_DP = C.POINTER(tt_desc2d)
_G = C.POINTER(C.c_uint32)
SYMBOLS = {
    "rt_init": (C.c_int, [C.c_int]),
    "rt_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "rt_device_props": (C.c_int, [C.POINTER(rt_props)]),
    "rt_malloc": (C.c_int, [C.POINTER(_vp), C.c_size_t]),
    "rt_free": (C.c_int, [_vp]),
    "rt_memcpy": (C.c_int, [_vp, _vp, C.c_size_t, C.c_int]),
    "rt_memset": (C.c_int, [_vp, C.c_int, C.c_size_t, _vp]),
    "rt_module_load": (C.c_int, [_vp, C.c_size_t, C.POINTER(_vp)]),
    "rt_module_unload": (C.c_int, [_vp]),
    "rt_builtin_module": (C.c_int, [C.c_char_p, C.POINTER(_vp)]),
    "rt_get_kernel": (C.c_int, [_vp, C.c_char_p, C.POINTER(_vp)]),
    "rt_launch": (C.c_int, [_vp, _G, _G, C.c_uint32, _vp, C.POINTER(_vp), C.c_size_t]),
    "rt_sync": (C.c_int, [_vp]),
    "rt_event_create": (C.c_int, [C.POINTER(_vp)]),
    "rt_event_record": (C.c_int, [_vp, _vp]),
    "rt_event_sync": (C.c_int, [_vp]),
    "rt_event_elapsed_ms": (C.c_int, [_vp, _vp, C.POINTER(C.c_float)]),
    "rt_event_destroy": (C.c_int, [_vp]),
    "rt_last_error": (C.c_char_p, []),
    "tt_add_kernel": (C.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _G, _vp]),
    "tt_add_kernel_loop": (C.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_muladd_kernel": (C.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _G, _vp]),
    "tt_sin_kernel": (C.c_int, [_vp, _vp, _i32, _i32, _G, _vp]),
    "tt_unary_kernel": (C.c_int, [_i32, _vp, _vp, _i32, _i32, _G, _vp]),
    "tt_binary_kernel": (C.c_int, [_i32, _vp, _vp, _vp, _i32, _i32, _G, _vp]),
    "tt_binary_const_kernel": (C.c_int, [_i32, _vp, _f32, _i32, _vp, _i32, _i32, _G, _vp]),
    "tt_cast_kernel": (C.c_int, [_vp, _vp, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_copy_kernel": (C.c_int, [_vp, _vp, _i32, _i32, _i32, _G, _vp]),
    "tt_reduce1d_kernel": (C.c_int, [_i32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_reduce1d_kernel_noalloc": (C.c_int, [_i32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _G, _vp]),
    "rt_release_stream": (C.c_int, [_vp]),
    "tt_matmul_kernel_tma": (C.c_int, [_DP, _DP, _DP, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_matmul_kernel_fused": (C.c_int, [_DP, _DP, _DP, _DP, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_matmul_kernel_tma_fp8_scaled": (C.c_int, [_DP, _DP, _DP, _i32, _i32, _i32, _f32, _f32, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_matmul_kernel": (C.c_int, [_vp, _vp, _vp, _i32, _i32, _i32] + [C.c_int64] * 6 + [_i32] * 6 + [_G, _vp]),
    "tt_attn_fwd": (C.c_int, [_f32, _vp, _i32, _i32, _DP, _DP, _DP, _DP, _i32, _i32, _i32, _i32, _i32, _G, _vp]),
    "tt_last_kernel_name": (C.c_char_p, []),
    "rt_gemm_clock_probe": (C.c_int, [_i32, C.POINTER(C.c_uint64)]),
}

_lib = None
_lock = threading.Lock()
_inited_device = None


def load() -> C.CDLL:
    """dlopen the runtime library and type every exported symbol."""
    global _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise FileNotFoundError(
                    f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                    "(there is no CPU fallback)")
            lib = C.CDLL(str(LIB_PATH))
            for name, (res, args) in SYMBOLS.items():
                fn = getattr(lib, name)  # AttributeError here = header and library disagree
                fn.restype, fn.argtypes = res, args
            _lib = lib
    return _lib


def last_error() -> str:
    return load().rt_last_error().decode(errors="replace")


def check(rc: int) -> None:
    if rc == RT_OK:
        return
    msg = last_error()
    if rc == RT_ERR_INVALID:
        raise InvalidLaunch(rc, msg)
    if rc == RT_ERR_UNSUPPORTED:
        raise Unsupported(rc, msg)
    raise RuntimeError_(rc, msg)


def init(device: int = 0) -> C.CDLL:
    """rt_init on ``device`` (idempotent) and return the library."""
    global _inited_device
    lib = load()
    if _inited_device != device:
        check(lib.rt_init(device))
        _inited_device = device
    return lib


def device_props() -> dict:
    lib = init(0 if _inited_device is None else _inited_device)
    p = rt_props()
    check(lib.rt_device_props(C.byref(p)))
    d = {name: getattr(p, name) for name, _ in rt_props._fields_ if name != "reserved"}
    d["name"] = p.name.decode()
    d["arch"] = p.arch.decode()
    return d


def last_kernel_name() -> str:
    return load().tt_last_kernel_name().decode()


def gemm_clock_probe(arm: bool = False):
    """``arm``: the next launch of the 16-bit macro-tile GEMM records its clock (and is synchronous).  Returns the
    last record as (core cycles, 100 MHz ticks, GHz) or None."""
    r = (C.c_uint64 * 2)()
    check(load().rt_gemm_clock_probe(1 if arm else 0, r))
    return (int(r[0]), int(r[1]), r[0] / r[1] / 10.0) if r[1] else None


def grid3(gx: int, gy: int = 1, gz: int = 1):
    return Grid3(int(gx), int(gy), int(gz))


def make_desc(base_ptr: int, shape, strides, block_shape, dtype: int, padding: str = "zero") -> tt_desc2d:
    if len(shape) != 2 or len(strides) != 2:
        raise Unsupported(RT_ERR_UNSUPPORTED, f"rank-{len(shape)} tensor descriptor; rank 2 is supported")
    d = tt_desc2d()
    d.base = base_ptr
    d.shape[0], d.shape[1] = int(shape[0]), int(shape[1])
    d.strides[0], d.strides[1] = int(strides[0]), int(strides[1])
    bs = list(block_shape) if block_shape is not None else [0, 0]
    d.block_shape[0], d.block_shape[1] = int(bs[0]), int(bs[1])
    d.padding_nan = 1 if padding == "nan" else 0
    d.dtype = dtype
    return d


class Event:
    """hipEvent with torch.cuda.Event's record/elapsed_time/synchronize surface."""

    def __init__(self, enable_timing: bool = True):
        self._lib = init(0 if _inited_device is None else _inited_device)
        h = C.c_void_p()
        check(self._lib.rt_event_create(C.byref(h)))
        self._h = h

    def record(self, stream: int | None = None):
        check(self._lib.rt_event_record(self._h, C.c_void_p(stream or 0)))

    def synchronize(self):
        check(self._lib.rt_event_sync(self._h))

    def elapsed_time(self, end: "Event") -> float:
        ms = C.c_float()
        check(self._lib.rt_event_sync(end._h))
        check(self._lib.rt_event_elapsed_ms(self._h, end._h, C.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            if self._h:
                self._lib.rt_event_destroy(self._h)
        except Exception:
            pass
