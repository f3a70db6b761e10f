"""The C ABI from plain C.  Not marked gpu: include/ttamd_rt.h compiles as C (gcc -std=c99 -pedantic -Werror) and
tests/c_abi_consumer.c links against libttamd_rt.so, i.e. the boundary has C linkage, plain pointers and sizes
only.  Marked gpu: the program runs and its three kernels agree with the values it computes on the host."""
import shutil
import subprocess
from pathlib import Path

import pytest

from triton_tenstorrent_amd import runtime as rt

ROOT = Path(__file__).resolve().parent.parent
SRC = ROOT / "tests" / "c_abi_consumer.c"


def _build(out: Path) -> Path:
    lib = Path(rt.LIB_PATH)
    cmd = ["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O1", f"-I{ROOT / 'include'}", str(SRC), "-o", str(out),
           f"-L{lib.parent}", "-lttamd_rt", f"-Wl,-rpath,{lib.parent}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return out


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_header_is_c_and_the_consumer_links(tmp_path):
    rt.load()                                  # the library exists (built by conftest when missing)
    exe = _build(tmp_path / "c_abi_consumer")
    assert exe.exists()
    # and the header alone, as a C translation unit with nothing else in it
    tu = tmp_path / "only_header.c"
    tu.write_text('#include "ttamd_rt.h"\nint main(void) { return (int)sizeof(tt_desc2d) == 0; }\n')
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", f"-I{ROOT / 'include'}", str(tu)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


@pytest.mark.gpu
@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_c_consumer_runs(tmp_path):
    exe = _build(tmp_path / "c_abi_consumer")
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "add_kernel ok via ew_add_f32" in r.stdout and "reduce1d ok via reduce1d_i32" in r.stdout
    assert "matmul_kernel_tma ok via gemm_" in r.stdout and r.stdout.rstrip().endswith("C ABI ok")
