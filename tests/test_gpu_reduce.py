"""tt_reduce1d_kernel through the launcher and the C ABI against the oracle.  Integer reductions, min / max
and the index reductions (tie_break_left): bit for bit.  Float sums: the oracle folds from the left, the
kernel in a tree, so they agree to the first-order bound of fp32 summation, n * 2^-24 * sum|x|
(test_core.py::test_reduce1d itself allows rtol 1e-2)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu

TORCH_OF = {orc.I8: torch.int8, orc.I16: torch.int16, orc.I32: torch.int32, orc.I64: torch.int64, orc.U8: torch.uint8,
            orc.U16: torch.uint16, orc.U32: torch.uint32, orc.U64: torch.uint64}
NP_OF = {orc.I8: np.int8, orc.I16: np.int16, orc.I32: np.int32, orc.I64: np.int64, orc.U8: np.uint8, orc.U16: np.uint16,
         orc.U32: np.uint32, orc.U64: np.uint64}
# 32..512: test_core.py::test_reduce1d; 2^20: Triton's largest tensor; 131072 and up: from 128 KiB of input on the
# block is shared between workgroups (131072 int8 is the first such size, 131075 and 1048575 leave a ragged end)
SHAPES = [1, 32, 64, 128, 512, 1000, 4096, 131072, 131075, 1048575, 1 << 20]


def _acc_for(op, dt):
    from triton_tenstorrent_amd.backend.driver import reduce_acc_dtype
    return reduce_acc_dtype(op, dt)


@pytest.mark.parametrize("dt", list(NP_OF))
@pytest.mark.parametrize("n", SHAPES)
def test_integer_reductions_bit_exact(dt, n):
    rng = np.random.default_rng(7 * dt + n)
    info = np.iinfo(NP_OF[dt])
    for lo, hi in ((info.min, info.max), (max(info.min, -3), min(info.max, 3))):       # the second: ties everywhere
        x = rng.integers(lo, hi, n, dtype=NP_OF[dt], endpoint=True)
        xg = torch.from_numpy(x).cuda()
        for op in ("sum", "min", "max", "argmin", "argmax", "xor_sum"):
            got = K.reduce1d(op, xg).cpu().numpy()[0]
            assert rt.last_kernel_name().startswith("reduce1d_")
            acc = _acc_for(op, dt)
            want = orc.reduce1d(x, op, dt, acc_dt=acc)
            assert got.dtype == want.dtype and got == want, (op, dt, n, got, want)


@pytest.mark.parametrize("n", SHAPES)
def test_float_reductions(n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 100).astype(np.float32)
    x[rng.integers(0, n, max(1, n // 50))] = x[0]                  # ties
    xg = torch.from_numpy(x).cuda()
    for op in ("min", "max", "argmin", "argmax"):
        assert K.reduce1d(op, xg).cpu().numpy()[0] == orc.reduce1d(x, op, orc.F32), op
    bound = n * 2.0**-24 * float(np.abs(x).astype(np.float64).sum())
    assert abs(float(K.reduce1d("sum", xg).cpu()[0]) - float(orc.reduce1d(x, "sum", orc.F32))) <= 2 * bound
    xd = rng.standard_normal(n)
    dg = torch.from_numpy(xd).cuda()
    assert K.reduce1d("max", dg).cpu().numpy()[0] == xd.max() and K.reduce1d("argmin", dg).cpu().numpy()[0] == np.argmin(xd)
    assert abs(float(K.reduce1d("sum", dg).cpu()[0]) - float(orc.reduce1d(xd, "sum", orc.F64))) <= 2 * n * 2.0**-53 * np.abs(xd).sum()
    for dt, tdt in ((orc.BF16, torch.bfloat16), (orc.F16, torch.float16)):
        hg = (xg * (2.0**-8 if dt == orc.F16 else 1.0)).to(tdt)          # keeps the largest sum inside fp16's range
        h = hg.cpu().view(torch.uint16).numpy()
        # min / max of a half type run in fp32 and may be stored back to the half type: the element itself
        assert K.reduce1d("max", hg).cpu().numpy()[0] == orc.reduce1d(h, "max", dt, acc_dt=orc.F32)
        got = K.reduce1d("min", hg, out_dtype=tdt).cpu().view(torch.uint16).numpy()[0]
        assert got == orc.reduce1d(h, "min", dt, acc_dt=orc.F32, out_dt=dt)
        assert K.reduce1d("argmax", hg).cpu().numpy()[0] == orc.reduce1d(h, "argmax", dt)
        # a half sum: the IR rounds after every addition, the kernel carries fp32 and rounds once, so the
        # kernel is compared with the exact sum at half a unit in the last place of the result plus the fp32 bound
        exact = float(hg.cpu().double().sum())
        got = float(K.reduce1d("sum", hg).cpu().float()[0])
        ulp = 2.0 ** (np.floor(np.log2(max(abs(exact), 1e-30))) - (7 if dt == orc.BF16 else 10))
        assert abs(exact) < 60000 or dt == orc.BF16
        assert abs(got - exact) <= 0.5 * ulp + 2 * bound + 1e-30, (dt, n, got, exact)


def test_nan_rules_and_special_values():
    x = torch.tensor([1.0, float("nan"), -3.0, 2.0] * 100, device="cuda")
    assert float(K.reduce1d("max", x).cpu()[0]) == 2.0 and float(K.reduce1d("min", x).cpu()[0]) == -3.0
    assert torch.isnan(K.reduce1d("max", x, propagate_nan=True).cpu()[0])
    assert torch.isnan(K.reduce1d("min", x, propagate_nan=True).cpu()[0])
    assert torch.isnan(K.reduce1d("max", torch.full((300, ), float("nan"), device="cuda")).cpu()[0])
    assert int(K.reduce1d("argmin", torch.tensor([float("inf"), float("-inf"), 0.0], device="cuda")).cpu()[0]) == 1
    assert int(K.reduce1d("argmax", torch.tensor([-0.0, 0.0, -0.0], device="cuda")).cpu()[0]) == 0
    i64 = K.reduce1d("argmax", torch.arange(1000, device="cuda", dtype=torch.int32), out_dtype=torch.int64)
    assert i64.dtype == torch.int64 and int(i64.cpu()[0]) == 999


def test_error_paths_return_codes():
    lib = rt.init(0)
    x = torch.zeros(64, device="cuda")
    z = torch.zeros(2, device="cuda", dtype=torch.float64)
    grid = (C.c_uint32 * 3)(1, 1, 1)
    call = lambda op, block, i, a, o, nan=0, g=grid: lib.tt_reduce1d_kernel(op, x.data_ptr(), z.data_ptr(), block, i, a, o, nan, g, None)
    assert call(0, 0, rt.TT_F32, rt.TT_F32, rt.TT_F32) == rt.RT_ERR_INVALID                 # empty block
    assert call(0, (1 << 20) + 1, rt.TT_F32, rt.TT_F32, rt.TT_F32) == rt.RT_ERR_INVALID     # beyond Triton's largest tensor
    assert call(6, 64, rt.TT_F32, rt.TT_F32, rt.TT_F32) == rt.RT_ERR_INVALID                # unknown reduction
    assert call(5, 64, rt.TT_F32, rt.TT_F32, rt.TT_F32) == rt.RT_ERR_INVALID                # xor_sum of floats
    assert call(0, 64, rt.TT_I32, rt.TT_I32, rt.TT_I64) == rt.RT_ERR_UNSUPPORTED            # widening after the reduction
    assert call(0, 64, rt.TT_F32, rt.TT_I32, rt.TT_I32) == rt.RT_ERR_UNSUPPORTED            # float data, integer accumulate
    assert call(0, 64, rt.TT_FP8E4M3, rt.TT_F32, rt.TT_F32) == rt.RT_ERR_UNSUPPORTED
    assert call(3, 64, rt.TT_F32, rt.TT_F32, rt.TT_F32) == rt.RT_ERR_UNSUPPORTED            # index result into a float
    assert call(0, 64, rt.TT_I32, rt.TT_I32, rt.TT_I32, nan=1) == rt.RT_ERR_INVALID
    assert call(0, 64, rt.TT_F32, rt.TT_F32, rt.TT_F32, g=(C.c_uint32 * 3)(0, 1, 1)) == rt.RT_ERR_INVALID
    assert "reduce1d" in rt.last_error()
    assert call(0, 64, rt.TT_F32, rt.TT_F32, rt.TT_F32, g=(C.c_uint32 * 3)(7, 1, 1)) == rt.RT_OK   # every program stores the same
    torch.cuda.synchronize()


def test_first_large_launch_on_a_new_stream():
    """The buffer of partial results of a stream is allocated and cleared at the stream's first large launch; the
    clearing is ordered in that stream (a clear in the null stream is not waited for by a non-blocking stream and
    could reset the arrival counter under the first launch).  Eight new streams, the first launch of each checked."""
    rng = np.random.default_rng(11)
    x = rng.integers(-2**31, 2**31 - 1, 1 << 20, dtype=np.int64).astype(np.int32)
    xg = torch.from_numpy(x).cuda()
    want = orc.reduce1d(x, "sum", orc.I32)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(8)]
    outs = []
    for st in streams:
        with torch.cuda.stream(st):
            outs.append(K.reduce1d("sum", xg))
            outs.append(K.reduce1d("sum", xg))
    torch.cuda.synchronize()
    for got in outs:
        assert got.cpu().numpy()[0] == want
    for st in streams:
        assert rt.load().rt_release_stream(C.c_void_p(st.cuda_stream)) == rt.RT_OK


def test_large_blocks_across_workgroups_streams_and_repeats():
    """A block of 128 KiB and more is folded by several workgroups through a per-stream buffer of partial results:
    repeated launches on one stream, launches on two streams at once, an operand off the 16-byte grid (one
    workgroup) and the one-workgroup switch all give the same exact answers."""
    rng = np.random.default_rng(3)
    x = rng.integers(-2**31, 2**31 - 1, (1 << 20) + 4, dtype=np.int64).astype(np.int32)
    xg = torch.from_numpy(x).cuda()
    want = {op: orc.reduce1d(x[:1 << 20], op, orc.I32) for op in ("sum", "argmax", "xor_sum", "min")}
    for _ in range(5):
        for op, w in want.items():
            assert K.reduce1d(op, xg[:1 << 20]).cpu().numpy()[0] == w, op
    off = xg[1:(1 << 20) + 1]                                          # 4 bytes off a 16-byte boundary
    for op in want:
        assert K.reduce1d(op, off).cpu().numpy()[0] == orc.reduce1d(x[1:(1 << 20) + 1], op, orc.I32), op
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    y = torch.from_numpy(x[::-1].copy()).cuda()
    torch.cuda.synchronize()
    outs = []
    for i in range(20):
        with torch.cuda.stream(s1):
            outs.append((K.reduce1d("sum", xg[:1 << 20]), want["sum"]))
        with torch.cuda.stream(s2):
            outs.append((K.reduce1d("argmax", y[4:]), orc.reduce1d(np.ascontiguousarray(x[::-1][4:]), "argmax", orc.I32)))
    torch.cuda.synchronize()
    for got, w in outs:
        assert got.cpu().numpy()[0] == w



def test_repeat_launches_take_the_cached_path_and_keep_the_checks():
    """From the second call of one shape on, the launch is a cached closure; another dtype, operation or block size,
    a short operand or a host tensor must come out as on a first call."""
    n = 4096
    x = torch.randn(n, device="cuda")
    z = torch.empty(1, device="cuda")
    launch = K.reduce1d_kernel[(1, )]
    for _ in range(3):
        z.zero_()
        launch(x, z, BLOCK=n, OP="max")
        assert z.item() == x.max().item()
    assert K.reduce1d_kernel._plan is not None
    zi = torch.empty(1, device="cuda", dtype=torch.int32)
    launch(x, zi, BLOCK=n, OP="argmax")
    assert zi.item() == int(torch.argmax(x))
    launch(x, z, BLOCK=512, OP="max")
    assert z.item() == x[:512].max().item()
    xi = torch.arange(n, device="cuda", dtype=torch.int32)
    launch(xi, zi, BLOCK=n, OP="sum")
    launch(xi, zi, BLOCK=n, OP="sum")
    assert zi.item() == n * (n - 1) // 2
    launch(x, z, BLOCK=n, OP="max")
    with pytest.raises(ValueError):
        launch(x[:100], z, BLOCK=n, OP="max")
    with pytest.raises(ValueError):
        launch(x.cpu(), z, BLOCK=n, OP="max")
    launch(x, z, BLOCK=n, OP="max")
    assert z.item() == x.max().item()
