"""Build recipe: gfx950 code objects (hipcc --genco) and libttamd_rt.so.

    python -m triton_tenstorrent_amd.build        # rebuild everything

Every kernels/*.hip becomes one code object under build/, and the host runtime
embeds them, so the shared library is the only file that has to travel.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
BUILD = PKG / "build"
LIB = PKG / "lib" / "libttamd_rt.so"
CPUABI_LIB = PKG / "lib" / "libttamd_cpuabi.so"
ARCH = "gfx950"

CODE_OBJECTS = ["elementwise", "gemm", "attention", "reduce"]
RT_SOURCES = ["ttamd_rt.cpp", "tt_elementwise.cpp", "tt_gemm.cpp", "tt_attention.cpp", "tt_reduce.cpp",
              "tt_reduce_static.hip"]

# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 on this target
DEVICE_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-ffp-contract=on", "-fno-fast-math", "-Wall", "-Wno-unused-function", "-Wno-inline-asm"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; the runtime cannot be built without ROCm")
    return exe


def _run(cmd: list[str], cwd: str | None = None) -> None:
    r = subprocess.run(cmd, capture_output=True, text=True, cwd=cwd)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + r.stderr)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    noise = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if noise and os.environ.get("TTAMD_BUILD_VERBOSE"):
        sys.stderr.write("\n".join(noise) + "\n")


def build_code_object(name: str, extra: list[str] | None = None) -> Path:
    """Compile kernels/<name>.hip and check the assembly listing of that same compilation (kept with -save-temps
    in a directory of its own, deleted afterwards) for reads of an MFMA result that the compiler placed too close
    behind an inline-assembly MFMA: see listing_check."""
    from . import listing_check
    BUILD.mkdir(exist_ok=True)
    out = BUILD / f"{name}.hsaco"
    with tempfile.TemporaryDirectory(prefix=f"ttamd_{name}_") as tmp:
        _run([hipcc(), "--genco", *DEVICE_FLAGS, "-save-temps", *(extra or []), str(CSRC / "kernels" / f"{name}.hip"),
              "-o", str(out)], cwd=tmp)
        listings = list(Path(tmp).glob(f"{name}-hip-amdgcn-*{ARCH}.s"))
        if len(listings) != 1:
            raise RuntimeError(f"{name}: expected one {ARCH} listing from -save-temps, found {len(listings)}")
        text = listings[0].read_text()
        bad = listing_check.check_listing(text)
        # not an error, but worth a line: the hand-scheduled K loops should hold no wait of the compiler's for memory
        for kernel, lines in listing_check.split_kernels(text).items():
            n = listing_check.vmcnt_waits_in_mfma_blocks(lines) if kernel.startswith(("gemm_tile", "gemm_ragged", "gemm_splitk_b", "gemm_splitk_f")) else 0
            if n:
                sys.stderr.write(f"[build] {kernel}: {n} compiler-placed vmcnt wait(s) inside an MFMA loop (a spill in the K loop?)\n")
    if bad:
        out.unlink()
        lines = [f"{k}: {len(v)} (first: {v[0]})" for k, v in bad.items()]
        raise RuntimeError(f"{name}.hip: an MFMA result is touched too early in\n  " + "\n  ".join(lines))
    return out


def build_runtime() -> Path:
    LIB.parent.mkdir(exist_ok=True)
    # tt_reduce_static.hip carries a __device__ array, so the library holds a small gfx950 image of its own
    cmd = [hipcc(), "-shared", "-fPIC", "-O2", "-std=c++17", "-fvisibility=hidden", "-Wall", f"--offload-arch={ARCH}",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           f"-I{ROOT / 'include'}", f"-I{CSRC / 'rt'}", f'-DTTAMD_CO_DIR="{BUILD}"',
           *[str(CSRC / "rt" / s) for s in RT_SOURCES], "-o", str(LIB)]
    _run(cmd)
    return LIB


def build_cpu_abi() -> Path:
    """libttamd_cpuabi.so: host-only support (the barrier) for kernels with the reference's cpu/ calling
    convention; plain g++, no ROCm."""
    CPUABI_LIB.parent.mkdir(exist_ok=True)
    cxx = shutil.which("g++") or "g++"
    _run([cxx, "-shared", "-fPIC", "-O2", "-std=c++17", "-fvisibility=hidden", "-Wall", "-Wextra", "-pthread",
          f"-I{ROOT / 'include'}", str(CSRC / "cpuabi" / "cpu_abi.cpp"), "-o", str(CPUABI_LIB)])
    return CPUABI_LIB


def build_all(jobs: int = 4) -> Path:
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(build_code_object, CODE_OBJECTS))
    build_cpu_abi()
    return build_runtime()


if __name__ == "__main__":
    print(build_all())
