"""GPU parity: add_kernel / sin_kernel / muladd_kernel through the launcher and the C ABI
against the CPU oracle.  add is bit-exact; sin is within 2e-6 absolute."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu
SIN_ATOL = 2e-6


def _dev(a):
    return torch.from_numpy(a).cuda()


@pytest.mark.parametrize("n", [1, 31, 1023, 1024, 1025, 4099, 98432, 1 << 20, (1 << 22) + 3])
def test_add_f32_bit_exact(n):
    torch.manual_seed(0)
    x, y = torch.rand(n), torch.rand(n)
    got = K.add(x.cuda(), y.cuda()).cpu().numpy()
    want = orc.add(x.numpy(), y.numpy())
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert rt.last_kernel_name() == "ew_add_f32"


@pytest.mark.parametrize("n", [5, 98432, (1 << 21) + 1])
def test_add_i32_bit_exact_with_wraparound(n):
    g = torch.Generator().manual_seed(0)
    a = torch.randint(-2**31, 2**31 - 1, (n, ), dtype=torch.int32, generator=g)
    b = torch.randint(-2**31, 2**31 - 1, (n, ), dtype=torch.int32, generator=g)
    got = K.add(a.cuda(), b.cuda()).cpu().numpy()
    assert np.array_equal(got, orc.add(a.numpy(), b.numpy()))
    assert rt.last_kernel_name() == "ew_add_i32"


def test_add_mask_never_touches_past_n_and_partial_grid():
    n, pad = 98432, 4096
    x = torch.rand(n + pad).cuda()
    y = torch.rand(n + pad).cuda()
    out = torch.full((n + pad, ), 7.5, device="cuda")
    K.add_kernel[(K.cdiv(n, 1024), )](x, y, out, n, BLOCK_SIZE=1024)
    assert torch.equal(out[:n], x[:n] + y[:n]) and torch.all(out[n:] == 7.5)
    out.fill_(7.5)
    K.add_kernel[(3, )](x, y, out, n, BLOCK_SIZE=1024)  # programs 0..2 only
    want = np.full(n + pad, 7.5, dtype=np.float32)
    orc.add(x.cpu().numpy(), y.cpu().numpy(), want, n=n, grid=3)
    assert np.array_equal(out.cpu().numpy(), want)


def test_add_unaligned_views_take_the_scalar_kernel():
    x = torch.rand(10001).cuda()
    y = torch.rand(10001).cuda()
    out = torch.zeros(10001, device="cuda")
    K.add_kernel[(K.cdiv(10000, 1024), )](x[1:], y[1:], out[1:], 10000, BLOCK_SIZE=1024)
    assert rt.last_kernel_name() == "ew_add_f32_unaligned"
    assert torch.equal(out[1:], x[1:] + y[1:]) and out[0] == 0


def test_add_specials():
    x = torch.tensor([float("inf"), float("-inf"), float("nan"), 1e38, -0.0, 1e-45, 3.0e38] * 3)
    y = torch.tensor([float("-inf"), float("-inf"), 1.0, 3e38, 0.0, 1e-45, 3.0e38] * 3)
    got = K.add(x.cuda(), y.cuda()).cpu().numpy()
    want = orc.add(x.numpy(), y.numpy())
    m = ~np.isnan(want)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[m].view(np.uint32), want[m].view(np.uint32))


def test_add_loop_variant_matches_plain():
    n = 98432 * 3 + 17
    x, y = torch.rand(n).cuda(), torch.rand(n).cuda()
    assert torch.equal(K.add_loop(x, y), x + y)
    assert torch.equal(K.add_loop(x, y, n_cores=130), x + y)


def test_muladd_is_one_fma():
    n = 98432
    g = torch.Generator().manual_seed(1)
    x, y, z = (torch.randn(n, generator=g) for _ in range(3))
    got = K.muladd(x.cuda(), y.cuda(), z.cuda()).cpu().numpy()
    want = orc.muladd(x.numpy(), y.numpy(), z.numpy(), fused=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("n", [32, 1024, 98432, (1 << 22) + 5])
def test_sin_within_tolerance_of_correctly_rounded(n):
    torch.manual_seed(0)
    x = (torch.rand(n) * 2 - 1) * (8 * np.pi)
    got = K.sin(x.cuda()).cpu().numpy()
    want = orc.sin(x.numpy())
    assert np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) <= SIN_ATOL
    assert orc.pcc(want, got) > 0.97  # the reference's own bar (examples/01-sin-kernel.py:61)


def test_sin_wide_range_and_specials():
    x = torch.cat([torch.randn(100000) * 1e4, torch.randn(100000) * 1e7,
                   torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 1e30, 131071.9, 131072.0])])
    got = K.sin(x.cuda()).cpu().numpy()
    want = orc.sin(x.numpy())
    fin = np.isfinite(want)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.max(np.abs(got[fin].astype(np.float64) - want[fin])) <= SIN_ATOL
    assert got[200000] == 0.0 and got[200001] == 0.0 and np.signbit(got[200001]) and not np.signbit(got[200000])


def test_full_size_streaming_properties():
    """N = 2^28 (BASELINE streaming config): checked through size-independent properties
    (commutativity, x + 0 = x, sampled windows against the oracle, sin odd symmetry)."""
    n = 1 << 28
    g = torch.Generator(device="cuda").manual_seed(0)
    a = torch.randint(-2**20, 2**20, (n, ), dtype=torch.int32, device="cuda", generator=g)
    b = torch.randint(-2**20, 2**20, (n, ), dtype=torch.int32, device="cuda", generator=g)
    c = K.add(a, b)
    assert torch.equal(c, K.add(b, a))
    assert torch.equal(K.add(a, torch.zeros_like(a)), a)
    assert int(c.sum(dtype=torch.int64)) == int(a.sum(dtype=torch.int64)) + int(b.sum(dtype=torch.int64))
    for lo in (0, 123456789, n - 98432):
        sl = slice(lo, lo + 98432)
        assert np.array_equal(c[sl].cpu().numpy(), orc.add(a[sl].cpu().numpy(), b[sl].cpu().numpy()))
    del a, b, c
    x = (torch.rand(n, device="cuda", generator=g) * 2 - 1) * (8 * np.pi)
    s = K.sin(x)
    assert torch.equal(K.sin(-x), -s)
    for lo in (0, 200000001, n - 98432):
        sl = slice(lo, lo + 98432)
        assert np.max(np.abs(s[sl].cpu().numpy() - orc.sin(x[sl].cpu().numpy()))) <= SIN_ATOL


def test_launch_errors_are_reported_not_fatal():
    x = torch.rand(100).cuda()
    with pytest.raises(ValueError):
        K.add_kernel[(1, 2, 1)](x, x, x, 100, BLOCK_SIZE=1024)  # 2-D grid
    with pytest.raises(ValueError):
        K.add_kernel[(1, )](x, x, x, -5, BLOCK_SIZE=1024)
    with pytest.raises(NotImplementedError):
        K.add(x.double(), x.double())
    with pytest.raises(ValueError):
        K.add_kernel[(1, )](x.cpu(), x, x, 100, BLOCK_SIZE=1024)
    # still healthy afterwards
    assert torch.equal(K.add(x, x), x + x)


def test_repeat_launches_keep_every_check_of_the_first():
    """The second launch of the same call shape goes through a cached closure (one C call); whatever that
    closure does not recognise has to fall back to the full path, with the same results and the same errors."""
    n = 98432
    x, y = torch.rand(n).cuda(), torch.rand(n).cuda()
    out = torch.zeros(n, device="cuda")
    launch = K.add_kernel[(K.cdiv(n, 1024), )]
    for _ in range(3):
        out.zero_()
        launch(x, y, out, n, BLOCK_SIZE=1024)
        assert torch.equal(out, x + y)
    assert K.add_kernel._plan is not None
    # another dtype, another BLOCK_SIZE, a partial grid, n == 1: same answers as a first launch
    xi = torch.arange(n, dtype=torch.int32).cuda()
    oi = torch.zeros_like(xi)
    launch(xi, xi, oi, n, BLOCK_SIZE=1024)
    assert torch.equal(oi, xi + xi)
    out.zero_()
    K.add_kernel[(K.cdiv(n, 512), )](x, y, out, n, BLOCK_SIZE=512)
    assert torch.equal(out, x + y)
    out.fill_(7.5)
    K.add_kernel[(3, )](x, y, out, n, BLOCK_SIZE=1024)
    K.add_kernel[(3, )](x, y, out, n, BLOCK_SIZE=1024)
    assert torch.equal(out[:3072], (x + y)[:3072]) and torch.all(out[3072:] == 7.5)
    out.fill_(7.5)
    launch(x, y, out, 1, BLOCK_SIZE=1024)
    assert out[0] == x[0] + y[0] and torch.all(out[1:] == 7.5)
    # and the same refusals
    launch(x, y, out, n, BLOCK_SIZE=1024)
    with pytest.raises(ValueError):
        launch(x[:1000], y, out, n, BLOCK_SIZE=1024)            # an operand shorter than the launch covers
    with pytest.raises(ValueError):
        launch(x.cpu(), y, out, n, BLOCK_SIZE=1024)
    with pytest.raises(ValueError):
        launch(x, y, out, -5, BLOCK_SIZE=1024)
    with pytest.raises(ValueError):
        launch(x, y, out.double(), n, BLOCK_SIZE=1024)
    m = torch.rand(512, 512).cuda()
    with pytest.raises(ValueError):
        K.add_kernel[(256, )](m.t(), m, torch.empty_like(m), 512 * 512, BLOCK_SIZE=1024)
    # a side stream is picked up by the cached path too
    side = torch.cuda.Stream()
    out.zero_()
    with torch.cuda.stream(side):
        launch(x, y, out, n, BLOCK_SIZE=1024)
    side.synchronize()
    assert torch.equal(out, x + y)
    s = torch.zeros(n, device="cuda")
    for _ in range(2):
        K.sin_kernel[(K.cdiv(n, 1024), )](x, s, n, BLOCK_SIZE=1024)
    assert K.sin_kernel._plan is not None
    assert np.max(np.abs(s.cpu().numpy() - orc.sin(x.cpu().numpy()))) <= SIN_ATOL
