"""tt_reduce1d_kernel_noalloc through the C ABI against tt_reduce1d_kernel: the entry point for callers that cannot
allocate device memory keeps its partial results in a device array inside the library.  Bit for bit on integers
and on min / max / the index reductions; float sums fold in the same tree, so they are bit-equal too."""
import ctypes as C

import numpy as np
import pytest
import torch

from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu

OPS = {"sum": 0, "min": 1, "max": 2, "argmin": 3, "argmax": 4, "xor_sum": 5}
GRID = (C.c_uint32 * 3)(1, 1, 1)


def _pair(lib, op, x, in_dt, acc_dt, out_dt, out_torch, stream=None):
    """(existing entry point's result, new entry point's result) as raw bytes"""
    outs = []
    for fn in (lib.tt_reduce1d_kernel, lib.tt_reduce1d_kernel_noalloc):
        z = torch.full((2, ), -77, dtype=out_torch, device="cuda")
        rt.check(fn(OPS[op], x.data_ptr(), z.data_ptr(), x.numel(), in_dt, acc_dt, out_dt, 0, GRID, stream))
        torch.cuda.synchronize()
        outs.append(z.cpu().numpy().tobytes())
    return outs


def test_no_alloc_entry_point_matches_the_allocating_one_on_two_calls_in_a_row():
    lib = rt.init(0)
    g = torch.Generator(device="cuda").manual_seed(5)
    big = torch.randint(-2**31, 2**31 - 1, (1 << 20, ), dtype=torch.int32, device="cuda", generator=g)
    fbig = torch.randn(1 << 20, device="cuda", generator=g) * 100
    # first a block that takes 256 workgroups, then a smaller one (12 workgroups), then one below the
    # several-workgroup threshold: the array keeps the first call's partial results and counter state
    for n in (1 << 20, 200_000, 1000):
        x, xf = big[:n], fbig[:n]
        for op in OPS:
            out_t, out_dt = (torch.int32, rt.TT_I32)
            a, b = _pair(lib, op, x, rt.TT_I32, rt.TT_I32, out_dt, out_t)
            assert a == b, (op, n)
            if op != "xor_sum":
                is_arg = op.startswith("arg")
                a, b = _pair(lib, op, xf, rt.TT_F32, rt.TT_F32, rt.TT_I32 if is_arg else rt.TT_F32,
                             torch.int32 if is_arg else torch.float32)
                assert a == b, (op, n, "f32")
    # the results are right, not merely equal: against torch
    z = torch.zeros(2, dtype=torch.int64, device="cuda")
    rt.check(lib.tt_reduce1d_kernel_noalloc(OPS["argmax"], fbig.data_ptr(), z.data_ptr(), fbig.numel(), rt.TT_F32, rt.TT_F32,
                                            rt.TT_I64, 0, GRID, None))
    assert int(z.cpu()[0]) == int(torch.argmax(fbig))
    zi = torch.zeros(2, dtype=torch.int32, device="cuda")
    rt.check(lib.tt_reduce1d_kernel_noalloc(OPS["sum"], big.data_ptr(), zi.data_ptr(), big.numel(), rt.TT_I32, rt.TT_I32,
                                            rt.TT_I32, 0, GRID, None))
    want = int(big.cpu().numpy().astype(np.int64).sum() & 0xFFFFFFFF)
    assert int(zi.cpu().numpy().view(np.uint32)[0]) == want


def test_no_alloc_entry_point_rejects_sizes_beyond_its_scratch_and_allocates_nothing():
    lib = rt.init(0)
    x = torch.zeros(64, device="cuda")
    z = torch.zeros(2, device="cuda")
    rc = lib.tt_reduce1d_kernel_noalloc(0, x.data_ptr(), z.data_ptr(), (1 << 20) + 1, rt.TT_F32, rt.TT_F32, rt.TT_F32, 0, GRID, None)
    assert rc == rt.RT_ERR_INVALID and "1048576" in rt.last_error()
    big = torch.ones(1 << 20, device="cuda")
    s = torch.cuda.Stream()        # a stream the allocating entry point has never seen
    with torch.cuda.stream(s):
        z.zero_()                  # the stream's own first-use set-up (its queue) is not the entry point's
    host = torch.empty(2).pin_memory()
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        rt.check(lib.tt_reduce1d_kernel_noalloc(0, big.data_ptr(), z.data_ptr(), big.numel(), rt.TT_F32, rt.TT_F32, rt.TT_F32,
                                                0, GRID, s.cuda_stream))
    s.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, "device memory was allocated behind the entry point"
    host.copy_(z)
    assert float(host[0]) == float(1 << 20)
    assert rt.last_kernel_name() == "reduce1d_f32"
