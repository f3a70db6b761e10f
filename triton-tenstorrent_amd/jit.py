"""``kernel[grid](*args, **constexprs)`` for the prebuilt kernels, without
Triton's JIT in the loop.

It reproduces the part of Triton's runtime that sits between a user script and
the plugin's launcher (triton/runtime/jit.py:695-745): bind the arguments,
specialise the signature (tensors -> ``*fp32``, ints -> ``i32`` with the value 1
folded to ``constexpr``, floats -> ``fp32``, descriptors ->
``tensordesc<dtype[b0,b1]>``), run the autotune config's ``pre_hook``, evaluate
the grid callable on the meta-parameters, obtain ``function`` from
``driver.utils.load_binary`` and call ``driver.launcher_cls(src, metadata)`` with
``(gridX, gridY, gridZ, stream, function, packed_metadata, launch_metadata,
enter_hook, exit_hook, *args)``.
"""
from __future__ import annotations

import functools
import json
import threading
from types import SimpleNamespace
from typing import Any, Callable, Sequence

from .backend.driver import BINARY_EXT, TTDriver
from .tensor_descriptor import is_tensor_descriptor

_TORCH_TYPESTR = None


def _typestr_of_torch(dtype) -> str:
    global _TORCH_TYPESTR
    if _TORCH_TYPESTR is None:
        import torch
        _TORCH_TYPESTR = {torch.float32: "fp32", torch.int32: "i32", torch.bfloat16: "bf16", torch.float16: "fp16",
                          torch.float8_e4m3fn: "fp8e4nv", torch.float8_e5m2: "fp8e5", torch.int64: "i64",
                          torch.float64: "fp64", torch.int8: "i8", torch.uint8: "u8", torch.int16: "i16",
                          torch.uint16: "u16", torch.uint32: "u32", torch.uint64: "u64"}
    return _TORCH_TYPESTR[dtype]


_TENSOR_TYPE = None
_PTR_TYPESTR: dict = {}


def specialize(arg: Any, is_constexpr: bool) -> str:
    """Type string of one bound argument, as Triton's specializer writes it."""
    if is_constexpr or arg is None:
        return "constexpr"
    ta = type(arg)
    if ta is _TENSOR_TYPE:  # a plain torch tensor: one dictionary lookup
        ts = _PTR_TYPESTR.get(arg.dtype)
        if ts is None:
            ts = _PTR_TYPESTR[arg.dtype] = "*" + _typestr_of_torch(arg.dtype)
        return ts
    if ta is int:  # the common scalar, ahead of the duck-typed checks
        if arg == 1:
            return "constexpr"  # Triton folds the value 1 into the specialisation
        return "i32" if -2**31 <= arg < 2**31 else "i64"
    if is_tensor_descriptor(arg):
        block = ",".join(str(int(b)) for b in arg.block_shape)
        return f"tensordesc<{_typestr_of_torch(arg.base.dtype)}[{block}]>"
    if hasattr(arg, "data_ptr"):
        return "*" + _typestr_of_torch(arg.dtype)
    if isinstance(arg, bool):
        return "i1"
    if isinstance(arg, int):
        if arg == 1:
            return "constexpr"  # Triton folds the value 1 into the specialisation
        return "i32" if -2**31 <= arg < 2**31 else "i64"
    if isinstance(arg, float):
        return "fp32"
    raise TypeError(f"Unsupported scalar type: {type(arg)}")  # backend/driver.py:295


class Config:
    """One autotune configuration: meta-parameters plus an optional ``pre_hook(nargs)``."""

    def __init__(self, kwargs: dict, num_warps: int = 4, num_stages: int = 1, pre_hook: Callable | None = None):
        self.kwargs, self.num_warps, self.num_stages, self.pre_hook = dict(kwargs), num_warps, num_stages, pre_hook


_MISSING = object()
_PLAIN_VALUES = (int, float, str, bool, type(None))      # constexpr values a plan compares with ==

_driver: TTDriver | None = None
_STOCK_GET_STREAM = TTDriver.get_current_stream      # a driver whose stream lookup was replaced is asked, not bypassed
_raw_stream = None      # (current device, its current stream) without building torch.cuda.Stream objects


def active_driver() -> TTDriver:
    global _driver, _TENSOR_TYPE, _raw_stream
    if _driver is None:
        _driver = TTDriver()
        try:
            import torch
            _TENSOR_TYPE = torch.Tensor
            get_dev, get_raw = torch._C._cuda_getDevice, torch._C._cuda_getCurrentRawStream
            get_raw(get_dev())

            def _raw_stream_fn():
                d = get_dev()
                return d, get_raw(d)
            _raw_stream = _raw_stream_fn
        except Exception:       # no GPU here (host tests), or a torch without these entry points
            _raw_stream = None
    return _driver


class PrebuiltKernel:
    """A kernel of the prebuilt table with a Triton-style call surface."""

    launch_enter_hook: Callable | None = None
    launch_exit_hook: Callable | None = None

    def __init__(self, name: str, arg_names: Sequence[str], constexprs: Sequence[str], *,
                 configs: Sequence[Config] | None = None, launch_metadata: Callable | None = None,
                 defaults: dict | None = None):
        self.name = name
        self.arg_names = list(arg_names)
        self.constexprs = set(constexprs)
        self.configs = list(configs or [])
        self.launch_metadata = launch_metadata
        self.defaults = dict(defaults or {})
        self.fn = SimpleNamespace(arg_names=self.arg_names, __name__=name)
        self._cache: dict = {}
        # repeat launches: (number of positional arguments, the keyword arguments that are not launch arguments
        # (constexprs, num_warps ...) with their values, device, closure, the configuration's pre_hook or None, the
        # arguments after the positional ones by name for that hook and for a callable grid, the launch arguments
        # among them in order as (name, given by keyword?, value at the launch that built the plan) or None, the
        # number of keyword arguments).  The tuple is replaced as a whole and never modified, and everything a launch
        # writes (the closure's descriptor blocks, the operands kept alive) is per thread: any thread may take a plan
        # that another one built.
        self._plan = None
        self._tls = threading.local()
        n_lead = next((i for i, n in enumerate(self.arg_names) if n in self.constexprs), len(self.arg_names))
        # a plan needs "launch arguments first, positionally; constexprs after them, by keyword or default"
        self._lead = n_lead if all(n in self.constexprs for n in self.arg_names[n_lead:]) else None

    def __getitem__(self, grid):
        return functools.partial(self.run, grid=grid)

    def _bind(self, args, kwargs) -> dict:
        if len(args) > len(self.arg_names):
            raise TypeError(f"{self.name}() takes {len(self.arg_names)} arguments, {len(args)} given")
        bound = dict(zip(self.arg_names, args))
        for k, v in kwargs.items():
            if k in ("num_warps", "num_stages", "num_ctas"):
                continue
            if k not in self.arg_names:
                raise TypeError(f"{self.name}() got an unexpected keyword argument {k!r}")
            if k in bound:
                raise TypeError(f"{self.name}() got multiple values for argument {k!r}")
            bound[k] = v
        config = self.configs[0] if self.configs else None
        for src in ((config.kwargs if config else {}), self.defaults):
            for k, v in src.items():
                bound.setdefault(k, v)
        missing = [n for n in self.arg_names if n not in bound]
        if missing:
            raise TypeError(f"{self.name}() missing arguments: {missing}")
        return {n: bound[n] for n in self.arg_names}

    @property
    def _keep(self):
        """The operands of the calling thread's last repeat launch."""
        return getattr(self._tls, "keep", None)

    def _plan_applies(self, plan, kwargs):
        """-> (True, launch arguments given by keyword in their positions) when this call's keyword arguments are
        the plan's: the same names, the same VALUES for those that select the kernel (constexprs, compared only
        where they are plain Python values), and whatever the caller passes now for the launch arguments among
        them (a tensor given by keyword is a different tensor every call)."""
        for k, v in plan[1].items():
            w = kwargs.get(k, _MISSING)
            if w is not v and (type(w) is not type(v) or type(v) not in _PLAIN_VALUES or w != v):
                return False, None
        tail = plan[6]
        if tail is None:
            return True, None
        try:
            return True, tuple([kwargs[n] if from_kw else v for n, from_kw, v in tail])
        except KeyError:
            return False, None

    def run(self, *args, grid, **kwargs):
        plan = self._plan
        if (plan is not None and TTDriver.get_current_stream is _STOCK_GET_STREAM and len(args) == plan[0]
                and len(kwargs) == plan[7] and (type(grid) is tuple or callable(grid))
                and PrebuiltKernel.launch_enter_hook is None and PrebuiltKernel.launch_exit_hook is None):
            device, stream = _raw_stream()
            ok, by_keyword = self._plan_applies(plan, kwargs) if device == plan[2] else (False, None)
            if ok:
                g = grid
                if plan[4] is not None or type(g) is not tuple:
                    # the configuration's pre_hook and a callable grid see every argument by name, as on the ordinary path
                    named = dict(zip(self.arg_names, args))
                    named.update(plan[5])
                    if by_keyword is not None:
                        for (n, _, _), v in zip(plan[6], by_keyword):
                            named[n] = v
                    if plan[4] is not None:
                        plan[4](named)
                    if type(g) is not tuple:
                        g = g(named)
                # launch arguments that came by keyword go to the closure in their positions
                full = args if by_keyword is None else args + by_keyword
                if type(g) is tuple and plan[3](full, g, stream):
                    self._tls.keep = full   # launches are asynchronous: operands stay referenced until this thread's next one
                    return self
        user_grid = grid
        bound = self._bind(args, kwargs)
        config = self.configs[0] if self.configs else None
        if config is not None and config.pre_hook is not None:
            config.pre_hook(bound)
        if callable(grid):
            grid = grid(bound)
        grid = tuple(int(g) for g in grid)
        gx, gy, gz = (grid + (1, 1, 1))[:3]
        constexprs = self.constexprs
        drv = active_driver()
        types = tuple([specialize(v, n in constexprs) for n, v in bound.items()])
        if _raw_stream is not None and type(drv).get_current_stream is _STOCK_GET_STREAM:
            device, stream = _raw_stream()
        else:
            device = drv.get_current_device()
            stream = drv.get_current_stream(device)
        key = (types, device)
        entry = self._cache.get(key)
        if entry is None:
            signature = dict(zip(self.arg_names, types))
            constants = {(i, ): bound[n] for i, (n, t) in enumerate(zip(self.arg_names, types))
                         if t == "constexpr" and not hasattr(bound[n], "data_ptr")}
            src = SimpleNamespace(fn=self.fn, signature=signature, constants=constants, name=self.name)
            metadata = SimpleNamespace(name=self.name, shared=0, num_warps=config.num_warps if config else 4,
                                       num_ctas=1, cluster_dims=(1, 1, 1), target=drv.get_current_target())
            binary = json.dumps({"kernel": self.name, "ext": BINARY_EXT}).encode()
            _, function, _, _, _ = drv.utils.load_binary(self.name, binary, metadata.shared, device)
            packed = (metadata.num_warps, metadata.num_ctas, metadata.shared, *metadata.cluster_dims)
            entry = (drv.launcher_cls(src, metadata), function, packed)
            self._cache[key] = entry
        launcher, function, packed = entry
        enter, exit_ = PrebuiltKernel.launch_enter_hook, PrebuiltKernel.launch_exit_hook
        launch_md = None
        if self.launch_metadata is not None and (enter is not None or exit_ is not None):
            launch_md = self.launch_metadata(grid, SimpleNamespace(name=self.name), bound)
        launcher(gx, gy, gz, stream, function, packed, launch_md, enter, exit_, *bound.values())
        direct = getattr(launcher, "direct", None)
        if (direct is not None and _raw_stream is not None and self._lead is not None and len(args) <= self._lead
                and (type(user_grid) is tuple or callable(user_grid)) and stream == _raw_stream()[1]):
            hook = config.pre_hook if config is not None else None
            rest = {n: bound[n] for n in self.arg_names[len(args):]}
            tail = tuple((n, n in kwargs, bound[n]) for n in self.arg_names[len(args):self._lead]) or None
            selecting = {k: v for k, v in kwargs.items() if k not in self.arg_names[len(args):self._lead]}
            self._plan = (len(args), selecting, device, direct, hook, rest, tail, len(kwargs))
        return self
