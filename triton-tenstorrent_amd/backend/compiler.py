"""Compiler half of the plugin surface, MI355X edition.

Keeps the reference's ``TTOptions`` / ``TTBackend`` method surface
(backend/compiler.py:21-105, 474-502) and target name, but there is no code
generation for the device: Triton's own front end still turns the ``@triton.jit``
source into TTIR on the host (``src.make_ir``), the ``ttir`` stage tidies it with
stock passes, and the last stage emits a small JSON record that names the
prebuilt gfx950 kernel the launcher will bind (``backend/driver.py``).  A kernel
name with no prebuilt counterpart is a compile error, not a silent fallback.
"""
from __future__ import annotations

import functools
import hashlib
import json
import os
import re
from dataclasses import dataclass
from types import ModuleType
from typing import Dict, Tuple

from .driver import BINARY_EXT, KERNEL_TABLE, GPUTarget, TTDriver
from .patterns import match_empty, match_per_program, match_reduce1d, match_streaming, verify_named

try:
    from triton.backends.compiler import BaseBackend, Language
    _HAVE_TRITON = True
except Exception:  # importable without Triton: the C-ABI path needs none of this
    _HAVE_TRITON = False

    class BaseBackend:  # type: ignore
        def __init__(self, target) -> None:
            self.target = target
            assert self.supports_target(target)

        @staticmethod
        def parse_attr(desc):
            return [["tt.divisibility", 16]] if "D" in desc else []

    class Language:  # type: ignore
        TRITON, GLUON = 0, 1


@dataclass(frozen=True)
class TTOptions:
    # the reference's fields (backend/compiler.py:21-38) ...
    num_warps: int = 4
    num_ctas: int = 1
    num_stages: int = 1
    cluster_dims: tuple = (1, 1, 1)
    debug: bool = False
    arch: str = None
    enable_fp_fusion: bool = True
    backend_name: str = "tenstorrent"
    sanitize_overflow: bool = True
    instrumentation_mode: str = ""
    allowed_dot_input_precisions: Tuple[str] = ("ieee", )
    matrix_instr_nonkdim: int = 32
    warp_size: int = 64
    min_dot_size: int = 1
    enable_dot_op_multicast: bool = False
    ttmlir_target: str = "gfx950"
    # ... plus what the Triton 3.6 front end reads from every backend's options
    supported_fp8_dtypes: Tuple[str] = ("fp8e4nv", "fp8e5")
    deprecated_fp8_dot_operand_dtypes: Tuple[str] = ()
    default_dot_input_precision: str = "ieee"
    max_num_imprecise_acc_default: int = 0
    launch_cooperative_grid: bool = False
    extern_libs: dict = None

    def hash(self):
        hash_dict = dict(self.__dict__)
        key = "_".join([f"{name}-{val}" for name, val in sorted(hash_dict.items())])
        return hashlib.sha256(key.encode("utf-8")).hexdigest()


class TTBackend(BaseBackend):
    instrumentation = None

    @staticmethod
    def supports_target(target: GPUTarget):
        return target.backend == "tenstorrent"

    def get_driver(self):
        return TTDriver()

    def get_target_name(self, options) -> str:
        return "tenstorrent"

    def __init__(self, target: GPUTarget) -> None:
        super().__init__(target)
        self.binary_ext = BINARY_EXT
        self.device = "MI355X"

    def parse_options(self, options):
        args = {"arch": "gfx950"}
        if "enable_fp_fusion" not in options:
            args["enable_fp_fusion"] = True
        if "enable_dot_op_multicast" not in options:
            args["enable_dot_op_multicast"] = os.environ.get("TRITON_ENABLE_DOT_OP_MULTICAST", "0") == "1"
        args.update({k: options[k] for k in TTOptions.__dataclass_fields__.keys() if k in options if options[k] is not None})
        return TTOptions(**args)

    def pack_metadata(self, metadata):
        return (
            metadata.num_warps,
            metadata.num_ctas,
            metadata.shared,
            metadata.cluster_dims[0],
            metadata.cluster_dims[1],
            metadata.cluster_dims[2],
        )

    def get_codegen_implementation(self, options):
        return {"min_dot_size": lambda lhs, rhs: (1, 1, 1)}

    def get_module_map(self) -> Dict[str, ModuleType]:
        return {}

    def load_dialects(self, ctx):
        pass  # stock Triton dialects only; there is no backend dialect

    @staticmethod
    def parse_attr(desc):
        ret = []
        if "D" in desc:
            ret += [["tt.divisibility", 8]]
        desc = desc.replace("D", "")
        ret += BaseBackend.parse_attr(desc)
        return ret

    # ---- stages -------------------------------------------------------------
    @staticmethod
    def make_ttir(mod, metadata, options):
        """Host-side clean-up of the front end's TTIR with stock passes (the
        target-independent part of backend/compiler.py:107-125)."""
        from triton._C.libtriton import ir, passes
        pm = ir.pass_manager(mod.context)
        passes.common.add_inliner(pm)
        passes.common.add_canonicalizer(pm)
        passes.ttir.add_combine(pm)
        passes.common.add_cse(pm)
        passes.common.add_symbol_dce(pm)
        pm.run(mod, "make_ttir")
        return mod

    @staticmethod
    def kernel_name_of(ttir_text: str) -> str:
        names = re.findall(r"tt\.func\s+public\s+@([A-Za-z_][A-Za-z0-9_]*)", ttir_text)
        if len(names) != 1:
            raise RuntimeError(f"expected exactly one public kernel in the module, found {names}")
        return names[0]

    @staticmethod
    def make_binary(src, metadata, options):
        """Final stage: bind the kernel to the prebuilt table, by name where the IR under that name is the
        table's kernel and by what the IR does otherwise, and return the record the launcher loads.  No device
        code is generated; a kernel that matches nothing is a compile error."""
        text = str(src)
        name = TTBackend.kernel_name_of(text)
        record = {"kernel": name, "ext": BINARY_EXT, "arch": options.arch}
        if name not in KERNEL_TABLE:
            # not one of the example kernels by name: a kernel of the masked-block elementwise form is
            # bound by what its IR says it does (one operation of the reference's opcode set)
            match = match_streaming(text) or match_reduce1d(text) or match_per_program(text) or match_empty(text)
            if match is None:
                raise RuntimeError(f"kernel '{name}' has no prebuilt gfx950 implementation; this backend runs "
                                   f"{sorted(KERNEL_TABLE)}, and elementwise kernels of the masked-block form with "
                                   f"one supported operation; it does no code generation")
            record.update(kernel=match["kernel"], match=match)
        else:
            # a table name does not vouch for the body: the IR has to be that kernel (raises otherwise)
            match = verify_named(name, text)
            if match is not None:
                record.update(kernel=match["kernel"], match=match)
        metadata["name"] = name
        metadata["shared"] = 0
        metadata["warp_size"] = 64
        # read by triton/tools/compile.py after an ahead-of-time compile (backend/compiler.py:385-386)
        metadata["global_scratch_size"] = 0
        metadata["global_scratch_align"] = 1
        metadata["profile_scratch_size"] = 0
        metadata["profile_scratch_align"] = 1
        return json.dumps(record).encode()

    def add_stages(self, stages, options, language=None):
        if language is not None and language == getattr(Language, "GLUON", object()):
            raise NotImplementedError("Gluon language support is not implemented for this backend")
        if options.ttmlir_target != "gfx950":
            raise ValueError(f"Unsupported TTMLIR target: {options.ttmlir_target}")
        stages["ttir"] = lambda src, metadata: self.make_ttir(src, metadata, options)
        stages[BINARY_EXT] = lambda src, metadata: self.make_binary(src, metadata, options)

    @functools.lru_cache()
    def hash(self):
        version = 0.1
        return f"{version}-{self.target.arch}"


def register() -> None:
    """Make Triton see this backend without an installed entry point, and make its
    driver the active one (a ROCm box has the stock HIP driver active otherwise)."""
    if not _HAVE_TRITON:
        raise RuntimeError("Triton is not importable; use triton_tenstorrent_amd.kernels (the C-ABI path) instead")
    import triton
    from triton.backends import Backend, backends
    from . import driver as _drv
    _drv.opt_in()
    backends["tenstorrent"] = Backend(compiler=TTBackend, driver=TTDriver)
    triton.runtime.driver.set_active(TTDriver())
