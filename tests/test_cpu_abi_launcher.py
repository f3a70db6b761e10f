"""The host launcher for the reference's cpu/ kernel calling convention
(``kernel(user args..., launch_sz, launch_id, smem, barrier)``, cpu/lib/TritonCPUToLLVM/FuncOpToLLVM.cpp:44-65),
driven with small C kernels compiled here: what a caller's shared object sees must be what the convention says.
Nothing of the GPU runtime and nothing of the oracle is involved."""
import subprocess
import sys

import numpy as np
import pytest
import torch

from triton_tenstorrent_amd import cpu_abi

KERNELS_C = r"""
#include <stdint.h>
extern void _cpu_barrier(void *barrier);

/* add_kernel as the cpu/ lowering shapes it: the persistent wrapper's loop over [block_start, block_end)
   around the body of python/tutorials/01-vector-add.py:29-54 */
void add_kernel(const float *x, const float *y, float *out, int32_t n,
                int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier) {
  (void)launch_sz; (void)smem; (void)barrier;
  for (int32_t pid = launch_id[0]; pid < launch_id[1]; ++pid)
    for (int32_t i = pid * 1024; i < (pid + 1) * 1024 && i < n; ++i) out[i] = x[i] + y[i];
}

/* one record per (block, thread): what the kernel was handed */
void probe_kernel(int32_t *rec, int64_t tag, float scale, double bias,
                  int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier) {
  (void)barrier;
  const int32_t gx = launch_sz[0], gy = launch_sz[1], threads = launch_sz[3];
  for (int32_t b = launch_id[0]; b < launch_id[1]; ++b) {
    int32_t *r = rec + ((int64_t)b * threads + launch_id[2]) * 12;
    r[0] += 1;                               /* visits */
    r[1] = b % gx;                           /* program ids, decoded as GPUOpToLLVM.cpp:73-101 */
    r[2] = (b % (gx * gy)) / gx;
    r[3] = b / (gx * gy);
    r[4] = launch_sz[2];
    r[5] = launch_id[0];
    r[6] = launch_id[1];
    r[7] = (int32_t)((uintptr_t)smem % 64);
    r[8] = (int32_t)(tag >> 32);
    r[9] = (int32_t)(scale * 4.0f);
    r[10] = (int32_t)(bias * 8.0);
    r[11] = launch_id[3] | launch_id[4];
  }
}

/* every thread of a block writes its slot of shared memory, waits, and sums all of them: a wrong thread id, a
   barrier that lets a thread through early, or shared memory that is not shared shows in the sum */
void team_kernel(int32_t *out, int32_t rounds,
                 int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier) {
  const int32_t threads = launch_sz[3], t = launch_id[2];
  int32_t *slots = (int32_t *)smem;
  for (int32_t b = launch_id[0]; b < launch_id[1]; ++b) {
    int32_t acc = 0;
    for (int32_t r = 0; r < rounds; ++r) {
      slots[t] = (b + 1) * 1000 + r * 10 + t;
      _cpu_barrier(barrier);
      for (int32_t i = 0; i < threads; ++i) acc += slots[i];
      _cpu_barrier(barrier);                /* nobody overwrites a slot that is still being read */
    }
    out[b * threads + t] = acc;
  }
}

/* a kernel without the persistent wrapper runs the one block block_start (GPUOpToLLVM.cpp:121-129) */
void single_block_kernel(int32_t *out, int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier) {
  (void)launch_sz; (void)smem; (void)barrier;
  out[launch_id[0]] += 1;
}
"""


@pytest.fixture(scope="module")
def lib(tmp_path_factory):
    d = tmp_path_factory.mktemp("cpu_abi")
    src, so = d / "kernels.c", d / "libkernels.so"
    src.write_text(KERNELS_C)
    # `_cpu_barrier` stays undefined in the object, as in the reference's output: the launcher's support library
    # has to resolve it
    subprocess.run(["gcc", "-shared", "-fPIC", "-O2", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(so)], check=True)
    return cpu_abi.load_library(so)


def test_support_library_exports_every_declared_symbol():
    import re
    from pathlib import Path
    header = (Path(__file__).resolve().parents[1] / "include" / "ttamd_cpu_abi.h").read_text()
    declared = set(re.findall(r"^\w[\w\s\*]*?\b(\w+)\(", header, re.M))
    assert declared == set(cpu_abi.SUPPORT_SYMBOLS)
    sup = cpu_abi.support()
    for name in declared:
        assert getattr(sup, name)


@pytest.mark.parametrize("blocks,workers", [(152, 40), (7, 3), (3, 7), (64, 8), (1, 1), (0, 4)])
def test_block_ranges_are_contiguous_balanced_and_larger_first(blocks, workers):
    ranges = [cpu_abi.block_range(blocks, workers, w) for w in range(workers)]
    assert ranges[0][0] == 0 and ranges[-1][1] == blocks
    assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:]))
    sizes = [e - s for s, e in ranges]
    assert max(sizes) - min(sizes) <= 1 and sizes == sorted(sizes, reverse=True)


@pytest.mark.parametrize("n,workers", [(98432, None), (98432, 1), (5000, 3), (1, 4), (1024 * 7, 16)])
def test_add_kernel_over_worker_ranges(lib, n, workers):
    k = lib.get_kernel("add_kernel", ["*fp32", "*fp32", "*fp32", "i32", "constexpr"])
    torch.manual_seed(0)
    x, y = torch.rand(n), torch.rand(n)
    out = torch.full((n + 8, ), -1.0)
    grid = ((n + 1023) // 1024, )
    k.launch(grid, x, y, out, n, 1024, workers=workers)
    assert torch.equal(out[:n], x + y) and torch.all(out[n:] == -1.0)
    # numpy arrays are pointers too; a partial grid leaves the rest alone
    o2 = np.full(n, -1.0, dtype=np.float32)
    k.launch((1, ), x.numpy(), y.numpy(), o2, n, 1024)
    m = min(n, 1024)
    assert np.array_equal(o2[:m], (x + y).numpy()[:m]) and np.all(o2[m:] == -1.0)


@pytest.mark.parametrize("grid,threads,workers", [((5, 3, 2), 1, 4), ((4, 1, 1), 3, 2), ((2, 7), 2, 5), ((9, ), 1, 9)])
def test_what_a_kernel_is_handed(lib, grid, threads, workers):
    k = lib.get_kernel("probe_kernel", ["*i32", "i64", "fp32", "fp64"])
    g = list(grid) + [1] * (3 - len(grid))
    blocks = g[0] * g[1] * g[2]
    rec = torch.zeros(blocks * threads, 12, dtype=torch.int32)
    k.launch(grid, rec, 7 << 32, 2.75, -1.5, shared=100, num_warps=threads, workers=workers)
    rec = rec.view(blocks, threads, 12).numpy()
    assert np.all(rec[..., 0] == 1)                                   # every (block, thread) exactly once
    b = np.arange(blocks)[:, None]
    assert np.array_equal(rec[..., 1], np.broadcast_to(b % g[0], rec[..., 1].shape))
    assert np.array_equal(rec[..., 2], np.broadcast_to((b % (g[0] * g[1])) // g[0], rec[..., 2].shape))
    assert np.array_equal(rec[..., 3], np.broadcast_to(b // (g[0] * g[1]), rec[..., 3].shape))
    assert np.all(rec[..., 4] == g[2])
    ranges = [cpu_abi.block_range(blocks, min(workers, blocks), w) for w in range(min(workers, blocks))]
    for s, e in ranges:                                               # a block's range is its worker's
        assert np.all(rec[s:e, :, 5] == s) and np.all(rec[s:e, :, 6] == e)
    assert np.all(rec[..., 7] == 0)                                   # shared memory on a cache line
    assert np.all(rec[..., 8] == 7) and np.all(rec[..., 9] == 11) and np.all(rec[..., 10] == -12)
    assert np.all(rec[..., 11] == 0)


@pytest.mark.parametrize("threads,workers,blocks", [(4, 2, 6), (8, 1, 3), (2, 3, 3), (1, 2, 5)])
def test_threads_of_a_block_share_memory_and_meet_at_the_barrier(lib, threads, workers, blocks):
    k = lib.get_kernel("team_kernel", ["*i32", "i32"])
    rounds = 50
    out = torch.zeros(blocks * threads, dtype=torch.int32)
    k.launch((blocks, ), out, rounds, shared=4 * threads, num_warps=threads, workers=workers)
    want = [sum((b + 1) * 1000 + r * 10 + t for r in range(rounds) for t in range(threads))
            for b in range(blocks) for _ in range(threads)]
    assert out.tolist() == want


def test_a_kernel_without_the_block_loop_runs_block_start(lib):
    k = lib.get_kernel("single_block_kernel", ["*i32"])
    out = torch.zeros(6, dtype=torch.int32)
    k.launch((6, ), out, workers=6)            # one block per worker: every block is somebody's block_start
    assert out.tolist() == [1] * 6
    out.zero_()
    k.launch((6, ), out, workers=2)            # such a kernel sees only the first block of each range
    assert out.tolist() == [1, 0, 0, 1, 0, 0]


def test_errors_before_anything_runs(lib, tmp_path):
    with pytest.raises(LookupError):
        lib.get_kernel("no_such_kernel", ["*fp32"])
    with pytest.raises(TypeError, match="Unsupported scalar type"):
        lib.get_kernel("add_kernel", ["*fp32", "*fp32", "*fp32", "tensordesc<fp32[1,1]>"])
    with pytest.raises(FileNotFoundError):
        cpu_abi.load_library(tmp_path / "absent.so")
    k = lib.get_kernel("add_kernel", ["*fp32", "*fp32", "*fp32", "i32", "constexpr"])
    x = torch.zeros(8)
    with pytest.raises(ValueError):
        k.launch((1, ), x, x, x, 8)                               # constexpr missing from the argument list
    with pytest.raises(ValueError):
        k.launch((-1, ), x, x, x, 8, 1024)
    with pytest.raises(TypeError):
        k.launch((1, ), x, x, "not a pointer", 8, 1024)
    with pytest.raises(TypeError):
        k.launch((1, ), x, x, x, "eight", 1024)
    k.launch((0, ), x, x, x, 8, 1024)                             # an empty grid runs nothing
    k.launch((1, ), x, x, x, 8, 1024)                             # and the library still works
    assert torch.all(x == 0)


def test_device_tensors_are_refused(lib):
    class DeviceTensor:
        is_cuda = True

        def data_ptr(self):
            raise AssertionError("must not be asked for an address")

    k = lib.get_kernel("add_kernel", ["*fp32", "*fp32", "*fp32", "i32", "constexpr"])
    with pytest.raises(ValueError, match="device memory"):
        k.launch((1, ), DeviceTensor(), DeviceTensor(), DeviceTensor(), 8, 1024)


def test_the_launcher_stands_apart_from_the_gpu_runtime_and_the_oracle():
    """It must work where no GPU library can be loaded, and nothing of it may reach into the oracle."""
    code = ("import sys; sys.path.insert(0, '.'); import __graft_entry__ as g; g._package();"
            "from triton_tenstorrent_amd import cpu_abi; cpu_abi.support();"
            "bad = [m for m in sys.modules if m.startswith('oracle') or m.endswith('.runtime')];"
            "assert not bad, bad")
    from pathlib import Path
    root = Path(__file__).resolve().parents[1]
    subprocess.run([sys.executable, "-c", code], check=True, cwd=root)
    text = (root / "triton-tenstorrent_amd" / "cpu_abi.py").read_text()
    assert "import oracle" not in text and "from oracle" not in text and "libttamd_rt" not in text
