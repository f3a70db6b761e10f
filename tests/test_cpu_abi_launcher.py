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


def test_a_kernel_without_the_block_loop_covers_its_grid_when_the_launcher_is_told(lib):
    k = lib.get_kernel("single_block_kernel", ["*i32"])
    out = torch.zeros(6, dtype=torch.int32)
    k.launch((6, ), out, workers=2, persistent=False)          # called once per block with [b, b + 1)
    assert out.tolist() == [1] * 6
    # threads of a team still share memory and barriers from block to block
    k = lib.get_kernel("team_kernel", ["*i32", "i32"])
    threads, blocks, rounds = 3, 5, 20
    out = torch.zeros(blocks * threads, dtype=torch.int32)
    k.launch((blocks, ), out, rounds, shared=4 * threads, num_warps=threads, workers=2, persistent=False)
    want = [sum((b + 1) * 1000 + r * 10 + t for r in range(rounds) for t in range(threads))
            for b in range(blocks) for _ in range(threads)]
    assert out.tolist() == want


# --------------------------------------------------------------------------
# the same kernels through the plugin surface: TTUtils.load_binary + TTLauncher
# --------------------------------------------------------------------------
DESC_KERNEL_C = r"""
#include <stdint.h>
/* a rank-2 descriptor arrives decomposed: base, shape x2 and strides x2 as i64, the padding flag, shape x2 as i32,
   strides x2 as i64; then the launch scalars */
void desc_kernel(const float *base, int64_t s0, int64_t s1, int64_t st0, int64_t st1, int8_t pad,
                 int32_t t0, int32_t t1, int64_t tt0, int64_t tt1, float *out, int32_t n,
                 int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier) {
  (void)launch_sz; (void)smem; (void)barrier;
  if (launch_id[0] != 0) return;
  out[0] = (float)s0; out[1] = (float)s1; out[2] = (float)st0; out[3] = (float)st1; out[4] = (float)pad;
  out[5] = (float)t0; out[6] = (float)t1; out[7] = (float)tt0; out[8] = (float)tt1; out[9] = (float)n;
  out[10] = base[st0 * (s0 - 1) + (s1 - 1)];          /* the last element, through the descriptor */
}
"""


def _launcher_for(arg_names, signature, constants=None):
    from types import SimpleNamespace
    from triton_tenstorrent_amd.backend import driver as drv
    src = SimpleNamespace(fn=SimpleNamespace(arg_names=list(arg_names)), signature=dict(zip(arg_names, signature)),
                          constants=constants or {})
    return drv.TTLauncher(src, SimpleNamespace())


def test_an_elf_image_goes_through_load_binary_and_the_launcher(tmp_path):
    """The reference hands a shared object to its runtime inside TTUtils.load_binary and launches it from
    TTLauncher.__call__ (backend/driver.py:68-74, 98-170).  Here an ELF image given to load_binary comes back as a
    host function, and the launcher runs it on host tensors with the cpu/ kernel ABI: no GPU, no GPU library."""
    from triton_tenstorrent_amd.backend import driver as drv
    src, so = tmp_path / "k.c", tmp_path / "libk.so"
    src.write_text(KERNELS_C + DESC_KERNEL_C)
    subprocess.run(["gcc", "-shared", "-fPIC", "-O2", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(so)], check=True)
    image = so.read_bytes()
    utils = drv.TTDriver().utils
    module, function, n_regs, shared, max_threads = utils.load_binary("add_kernel", image, 0, 0)
    assert isinstance(function, cpu_abi.HostFunction) and function.host and (n_regs, shared, max_threads) == (1, 0, 4096)

    n = 5000
    torch.manual_seed(1)
    x, y, out = torch.rand(n), torch.rand(n), torch.full((n + 4, ), -1.0)
    launcher = _launcher_for(["x_ptr", "y_ptr", "output_ptr", "n_elements", "BLOCK_SIZE"],
                             ["*fp32", "*fp32", "*fp32", "i32", "constexpr"])
    seen = []
    packed = (1, 1, 0, 1, 1, 1)              # num_warps, num_ctas, shared, cluster dims (backend/compiler.py:96-104)
    launcher((n + 1023) // 1024, 1, 1, 0, function, packed, {"name": "add"}, lambda md: seen.append(("enter", md["name"])),
             lambda md: seen.append(("exit", md["name"])), x, y, out, n, 1024)
    assert torch.equal(out[:n], x + y) and torch.all(out[n:] == -1.0)
    assert seen == [("enter", "add"), ("exit", "add")]

    # threads, shared memory and the barrier come from the packed metadata
    _, team, _, _, _ = utils.load_binary("team_kernel", image, 16, 0)
    threads, blocks, rounds = 4, 3, 10
    res = torch.zeros(blocks * threads, dtype=torch.int32)
    _launcher_for(["out", "rounds"], ["*i32", "i32"])(blocks, 1, 1, 0, team, (threads, 1, 4 * threads, 1, 1, 1), None, None, None,
                                                      res, rounds)
    want = [sum((b + 1) * 1000 + r * 10 + t for r in range(rounds) for t in range(threads))
            for b in range(blocks) for _ in range(threads)]
    assert res.tolist() == want

    # a descriptor is decomposed the way the reference's argument walk lists it
    from triton_tenstorrent_amd.tensor_descriptor import TensorDescriptor
    _, dk, _, _, _ = utils.load_binary("desc_kernel", image, 0, 0)
    base = torch.arange(8 * 12, dtype=torch.float32).reshape(8, 12)
    d = TensorDescriptor(base, [8, 12], [12, 1], [4, 4])
    rec = torch.zeros(11)
    _launcher_for(["d", "out", "n"], ["tensordesc<fp32[4,4]>", "*fp32", "i32"])(2, 1, 1, 0, dk, packed, None, None, None, d, rec, 77)
    assert rec.tolist() == [8, 12, 12, 1, 0, 8, 12, 12, 1, 77, 95]

    # device tensors are still refused, a missing kernel is an error at load_binary, and a JSON record is still the
    # other kind of binary
    class DeviceTensor:
        is_cuda = True

        def data_ptr(self):
            raise AssertionError("must not be asked for an address")

    with pytest.raises(ValueError, match="device memory"):
        launcher(1, 1, 1, 0, function, packed, None, None, None, DeviceTensor(), y, out, 8, 1024)
    with pytest.raises(LookupError):
        utils.load_binary("no_such_kernel", image, 0, 0)
    assert not cpu_abi.is_elf_image(b'{"kernel": "add_kernel"}')


def test_two_images_loaded_one_after_the_other_are_two_libraries(tmp_path):
    """dlopen answers a path name it has seen with the library it loaded then, so images must never share one."""
    libs = []
    for value in (11, 22):
        src, so = tmp_path / f"k{value}.c", tmp_path / f"libk{value}.so"
        src.write_text("#include <stdint.h>\nvoid which(int32_t *out, int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier) "
                       f"{{ (void)launch_sz; (void)launch_id; (void)smem; (void)barrier; out[0] = {value}; }}\n")
        subprocess.run(["gcc", "-shared", "-fPIC", "-O2", "-std=c99", str(src), "-o", str(so)], check=True)
        libs.append(cpu_abi.load_image(so.read_bytes()))
    outs = []
    for lib_ in libs:
        o = torch.zeros(1, dtype=torch.int32)
        lib_.get_kernel("which", ["*i32"]).launch((1, ), o)
        outs.append(int(o[0]))
    assert outs == [11, 22]


def test_the_elf_route_loads_neither_the_gpu_library_nor_the_oracle(tmp_path):
    src, so = tmp_path / "k.c", tmp_path / "libk.so"
    src.write_text(KERNELS_C)
    subprocess.run(["gcc", "-shared", "-fPIC", "-O2", "-std=c99", str(src), "-o", str(so)], check=True)
    code = ("import sys; sys.path.insert(0, '.'); import __graft_entry__ as g; g._package();"
            "import torch;"
            "from types import SimpleNamespace as NS;"
            "from triton_tenstorrent_amd.backend import driver as drv;"
            f"img = open({str(so)!r}, 'rb').read();"
            "_, fn, _, _, _ = drv.TTDriver().utils.load_binary('add_kernel', img, 0, 0);"
            "names = ['x', 'y', 'o', 'n', 'B'];"
            "src = NS(fn=NS(arg_names=names), signature=dict(zip(names, ['*fp32', '*fp32', '*fp32', 'i32', 'constexpr'])), constants={});"
            "x = torch.ones(2048); o = torch.zeros(2048);"
            "drv.TTLauncher(src, NS())(2, 1, 1, 0, fn, (1, 1, 0, 1, 1, 1), None, None, None, x, x, o, 2048, 1024);"
            "assert bool((o == 2).all());"
            "maps = open('/proc/self/maps').read();"
            "assert 'libttamd_rt' not in maps and 'liboracle' not in maps, 'a GPU or oracle library was mapped';"
            "assert not [m for m in sys.modules if m.startswith('oracle')]")
    from pathlib import Path
    subprocess.run([sys.executable, "-c", code], check=True, cwd=Path(__file__).resolve().parents[1])
