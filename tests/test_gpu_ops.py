"""The unary / binary / narrowing operations of ConvertComputeOps.cpp:162-182 through the launcher and
the C ABI against the oracle.  Exact operations: bit for bit.  Transcendental ones: within 2 fp32 ulp of
the float64 result rounded once (the oracle), NaN / inf / domain errors in the same places."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu

G = torch.Generator().manual_seed(9)
SPECIAL = torch.tensor([0.0, -0.0, 1.0, -1.0, 0.5, 2.5, -2.5, 1e-40, -1e-40, 3.4e38, -3.4e38, float("inf"), float("-inf"),
                        float("nan"), 88.7, -103.9, -95.0, 127.5, -149.5, -140.25, 1e-30, 6.1e-5], dtype=torch.float32)
X = torch.cat([torch.randn(70000, generator=G) * 10, SPECIAL])
Y = torch.cat([torch.randn(70000, generator=G) * 3, SPECIAL.flip(0)])


def _bits_equal(got: np.ndarray, want: np.ndarray) -> bool:
    nan_g, nan_w = np.isnan(got), np.isnan(want)
    return bool(np.array_equal(nan_g, nan_w) and np.array_equal(got[~nan_g].view(np.uint32), want[~nan_w].view(np.uint32)))


@pytest.mark.parametrize("op", ["abs", "ceil", "floor", "sqrt"])
def test_exact_unary(op):
    got = K.unary(op, X.cuda()).cpu().numpy()
    assert rt.last_kernel_name() == f"ew_{op}_f32"
    assert _bits_equal(got, orc.unary(op, X.numpy()))


@pytest.mark.parametrize("op", ["cos", "sin", "exp", "exp2", "log", "log2", "rsqrt"])
def test_transcendental_unary_within_two_ulp(op):
    x = X if op in ("exp", "exp2") else torch.cat([X, (torch.rand(50000, generator=G) * 2 - 1) * 8 * np.pi])
    got = K.unary(op, x.cuda()).cpu().numpy()
    want = orc.unary(op, x.numpy())
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
    fin = np.isfinite(want)
    normal = fin & (np.abs(want) >= 2.0 ** -126)     # a result that rounds to the smallest subnormal may round to 0
    assert np.array_equal(np.sign(got[normal]), np.sign(want[normal]))
    err = np.abs(got[fin].astype(np.float64) - want[fin].astype(np.float64))
    if op in ("sin", "cos"):
        # near a zero of sin / cos the result is tiny and a relative bound would ask for more than fp32 range
        # reduction gives: the bar there is absolute, 2e-6 as for sin_kernel
        assert np.all((err <= 2 * np.spacing(np.abs(want[fin]))) | (err <= 2e-6))
    else:
        assert np.all(err <= 2 * np.spacing(np.abs(want[fin])))


@pytest.mark.parametrize("op", ["cos", "sin"])
def test_trig_on_both_sides_of_the_library_threshold(op):
    """Below 2^17 the kernels reduce the argument themselves; from 2^17 on, inf and NaN included, a wavefront
    branches to the library routine for the lanes that need it.  Blocks in which no lane, some lanes and every lane
    take that branch, and the values right at the threshold."""
    g = torch.Generator().manual_seed(17)
    small = (torch.rand(64 * 300, generator=g) * 2 - 1) * 1.3e5
    large = torch.randn(64 * 300, generator=g) * 1e7
    mixed = torch.where(torch.rand(64 * 300, generator=g) < 0.03, large, small)
    edge = torch.tensor([131071.99, 131072.0, 131072.01, -131071.99, -131072.0, 1e30, -1e30, float("inf"), float("nan")])
    x = torch.cat([small, mixed, large, edge])
    got = K.unary(op, x.cuda()).cpu().numpy()
    want = orc.unary(op, x.numpy())
    assert np.array_equal(np.isnan(got), np.isnan(want))
    fin = np.isfinite(want)
    assert np.max(np.abs(got[fin].astype(np.float64) - want[fin].astype(np.float64))) <= 2e-6


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "maximum", "minimum"])
def test_binary_bit_exact(op):
    got = K.binary(op, X.cuda(), Y.cuda()).cpu().numpy()
    assert _bits_equal(got, orc.binary(op, X.numpy(), Y.numpy()))
    # signed zeros and NaN of maximum / minimum, both operand orders
    a = torch.tensor([0.0, -0.0, float("nan"), 1.0, -0.0, float("inf"), float("-inf"), float("nan")], dtype=torch.float32)
    b = torch.tensor([-0.0, 0.0, 1.0, float("nan"), -0.0, float("nan"), 5.0, float("inf")], dtype=torch.float32)
    got = K.binary(op, a.cuda(), b.cuda()).cpu().numpy()
    assert _bits_equal(got, orc.binary(op, a.numpy(), b.numpy()))


def test_masked_tail_partial_grid_and_unaligned():
    n = 5000
    x = torch.rand(n + 8) + 0.5
    for off in (0, 1):                          # 16-byte aligned and not
        xd = x.cuda()[off:off + n]
        out = torch.full((n + 8, ), -7.0, device="cuda")[off:off + n]
        K.unary_kernel[(3, )](xd, out, n, BLOCK_SIZE=1024, OP="sqrt")   # programs 0..2 of 5
        assert rt.last_kernel_name() == ("ew_sqrt_f32" if off == 0 else "ew_sqrt_f32_unaligned")
        assert torch.equal(out[:3072], torch.sqrt(xd[:3072])) and torch.all(out[3072:] == -7.0)
        out2 = torch.full((n + 8, ), -7.0, device="cuda")[off:off + n]
        K.binary_kernel[(5, )](xd, xd, out2, n - 3, BLOCK_SIZE=1024, OP="mul")   # n_elements masks the last three
        assert torch.equal(out2[:n - 3], xd[:n - 3] * xd[:n - 3]) and torch.all(out2[n - 3:] == -7.0)
    with pytest.raises(rt.Unsupported):
        K.unary("tanh", x.cuda())
    with pytest.raises(rt.Unsupported):
        K.unary("sqrt", x.cuda().half())


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "maximum", "minimum"])
def test_constant_operand_forms_exact(op):
    for c in (2.0, -0.75, 0.0, float("inf"), float("nan")):
        for flip in (False, True):
            got = K.binary_const(op, X.cuda(), c, flip=flip).cpu().numpy()
            assert rt.last_kernel_name() == f"ew_{ {'maximum': 'max', 'minimum': 'min'}.get(op, op)}c_f32"
            assert _bits_equal(got, orc.binary_const(op, X.numpy(), c, flip=flip)), (op, c, flip)
    # in place, an odd length and an operand off the 16-byte grid
    buf = torch.cat([torch.zeros(1), X]).cuda()
    view = buf[1:]
    K.binary_const(op, view, 1.5, out=view)
    assert rt.last_kernel_name().endswith("_unaligned")
    assert _bits_equal(view.cpu().numpy(), orc.binary_const(op, X.numpy(), 1.5)) and float(buf[0]) == 0.0


def test_narrowing_casts_exact():
    xf = torch.cat([X, torch.tensor([65504.0, 65520.0, 65519.99, 1e-8, 3.3895e38], dtype=torch.float32)])
    for dt, code in ((torch.bfloat16, orc.BF16), (torch.float16, orc.F16)):
        got = K.cast(xf.cuda(), dt).cpu()
        want = np.zeros(xf.numel(), dtype=np.uint16)
        orc.lib().orc_convert(orc._p(xf.numpy()), orc.F32, orc._p(want), code, xf.numel())
        g = got.view(torch.int16).numpy().view(np.uint16)
        nan = np.isnan(xf.numpy())
        assert np.array_equal(g[~nan], want[~nan]) and torch.isnan(got.float()[torch.from_numpy(nan)]).all()
        assert torch.equal(got[~torch.from_numpy(nan)], xf.to(dt)[~torch.from_numpy(nan)])   # torch's RNE cast agrees
    xi = torch.randint(-2**31, 2**31 - 1, (70001, ), dtype=torch.int64).to(torch.int32)
    assert np.array_equal(K.cast(xi.cuda(), torch.int16).cpu().numpy(), orc.trunci(xi.numpy(), 16))
    assert np.array_equal(K.cast(xi.cuda(), torch.int8).cpu().numpy(), orc.trunci(xi.numpy(), 8))
    with pytest.raises(rt.Unsupported):
        K.cast(xf.cuda(), torch.int8)


@pytest.mark.parametrize("n", [1, 7, 16, 8191, 8192, 16384, 32768 + 5, 131072 + 17, 1 << 22])
@pytest.mark.parametrize("offset", [0, 1, 4])
def test_narrowing_casts_sizes_alignments_and_sentinel(n, offset):
    # whole runs of the 16-byte path, ragged ends, operands off the 16-byte grid (element offsets 1) and on it (4);
    # nothing is written past n
    g = torch.Generator().manual_seed(n + offset)
    xf = (torch.randn(n + offset, generator=g) * 100)[offset:]
    xi = torch.randint(-2**31, 2**31 - 1, (n + offset, ), dtype=torch.int64, generator=g).to(torch.int32)[offset:]
    for src, dt, want in ((xf, torch.bfloat16, xf.to(torch.bfloat16)), (xf, torch.float16, xf.to(torch.float16)),
                          (xi, torch.int16, torch.from_numpy(orc.trunci(xi.numpy(), 16))),
                          (xi, torch.int8, torch.from_numpy(orc.trunci(xi.numpy(), 8)))):
        sent = 77 if dt in (torch.int16, torch.int8) else 7.5
        buf = torch.full((n + offset + 40, ), sent, dtype=dt, device="cuda")
        out = buf[offset:offset + n]
        xs = src.cuda()
        xs = torch.cat([torch.zeros(offset, dtype=xs.dtype, device="cuda"), xs])[offset:]      # same misalignment on the input
        K.cast_kernel[lambda meta: (K.cdiv(n, meta["BLOCK_SIZE"]), )](xs, out, n, BLOCK_SIZE=1024)
        aligned = xs.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0
        assert rt.last_kernel_name().endswith("_unaligned") != aligned
        assert torch.equal(out.cpu(), want), (dt, n, offset)
        assert torch.all(buf[:offset] == sent) and torch.all(buf[offset + n:] == sent)


def test_full_size_streaming_properties():
    # 2^28 elements: exp(log(x)) ~ x, sqrt(x)^2 ~ x, x/x == 1, max(x,y)+min(x,y) == x+y bit for bit
    n = 1 << 28
    x = torch.rand(n, device="cuda") + 0.5
    y = torch.rand(n, device="cuda") + 0.5
    one = K.binary("div", x, x)
    assert rt.last_kernel_name() == "ew_div_f32" and bool((one == 1.0).all())
    del one
    s = K.binary("add", K.binary("maximum", x, y), K.binary("minimum", x, y))
    assert torch.equal(s, x + y)
    del s
    r = K.unary("exp", K.unary("log", x))
    assert float(((r - x).abs() / x).max()) <= 4 * 2.0 ** -23
    del r
    q = K.unary("sqrt", x)
    assert float(((q * q - x).abs() / x).max()) <= 2 * 2.0 ** -23


@pytest.mark.parametrize("dt", [torch.uint8, torch.int8, torch.int16, torch.bfloat16, torch.float16, torch.int32, torch.float32,
                                torch.int64, torch.float64, torch.float8_e4m3fn])
def test_copy_exact(dt):
    """Bits move unchanged for every element width, every length around the vector and workgroup boundaries, and
    operands off the 16-byte grid; what lies past the masked range keeps its contents."""
    width = torch.empty(0, dtype=dt).element_size()
    g = torch.Generator().manual_seed(5)
    raw = torch.randint(0, 256, ((70001 + 64) * width, ), generator=g, dtype=torch.uint8)       # every bit pattern, NaNs included
    for n in (1, 15, 16, 17, 4095, 4096, 4097, 16384, 16385, 70001):
        x = raw[:n * width].cuda().view(dt)
        out = torch.zeros(n + 8, dtype=torch.uint8).repeat_interleave(width).view(dt).cuda()
        K.copy_kernel[(-(-n // 1024), )](x, out, n, BLOCK_SIZE=1024)
        assert rt.last_kernel_name() == "ew_copy_b128"
        want = np.zeros((n + 8) * width, dtype=np.uint8)
        orc.copy(raw[:n * width].numpy(), want, n * width, block=1024 * width)
        assert np.array_equal(out.view(torch.uint8).cpu().numpy(), want), (dt, n)
    # off the 16-byte grid: one element in
    n = 70001
    src = raw[:(n + 1) * width].cuda().view(dt)[1:]
    dst = torch.zeros((n + 2) * width, dtype=torch.uint8).cuda().view(dt)
    K.copy_kernel[(-(-n // 1024), )](src, dst[1:], n, BLOCK_SIZE=1024)
    assert rt.last_kernel_name() == f"ew_copy_b{8 * width}_unaligned"
    got = dst.view(torch.uint8).cpu()
    assert torch.equal(got[width:(n + 1) * width], raw[width:(n + 1) * width]) and not got[:width].any() and not got[(n + 1) * width:].any()
    # a grid shorter than the data: three programs move 3072 elements
    out = torch.zeros(n * width, dtype=torch.uint8).cuda().view(dt)
    K.copy_kernel[(3, )](raw[:n * width].cuda().view(dt), out, n, BLOCK_SIZE=1024)
    got = out.view(torch.uint8).cpu()
    assert torch.equal(got[:3072 * width], raw[:3072 * width]) and not got[3072 * width:].any()
    assert torch.equal(K.copy(x).view(torch.uint8), x.view(torch.uint8))

