"""Launches are plain hipModuleLaunchKernel calls on the caller's stream with no allocation, memset or
synchronisation inside, so a caller can record them into a HIP graph.  Each graph is replayed several times
with eager work and synchronisations in between, and every replay is checked against the eager result."""
import pytest
import torch

from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu


def _capture(fn):
    fn()                                    # warm-up outside the graph: library and code objects are loaded here
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


def test_elementwise_chain_in_a_graph():
    n = 98432
    x, y = torch.rand(n, device="cuda"), torch.rand(n, device="cuda")
    t, out = torch.empty_like(x), torch.empty_like(x)
    grid = (K.cdiv(n, 1024), )

    def chain():
        K.add_kernel[grid](x, y, t, n, BLOCK_SIZE=1024)
        K.sin_kernel[grid](t, out, n, BLOCK_SIZE=1024)
        K.binary_kernel[grid](out, x, t, n, BLOCK_SIZE=1024, OP="mul")

    g = _capture(chain)
    for rep in range(4):
        x.copy_(torch.rand(n, device="cuda"))          # eager work between replays, new inputs each time
        torch.cuda.synchronize()
        t.fill_(-1.0)
        out.fill_(-1.0)
        g.replay()
        torch.cuda.synchronize()
        want_out = K.sin(x + y)
        assert torch.equal(out, want_out) and torch.equal(t, want_out * x), rep


def test_matmul_and_attention_in_a_graph():
    M = N = Kd = 512
    a = (torch.randn(M, Kd, device="cuda") / 16).to(torch.bfloat16)
    b = torch.randn(Kd, N, device="cuda").to(torch.bfloat16)
    bias = torch.randn(N, device="cuda") * 0.02
    q, k, v = (torch.randn(1, 2, 512, 128, device="cuda").to(torch.bfloat16) for _ in range(3))
    res = {}

    def work():
        res["c"] = K.matmul_fused(a, b, bias, epilogue="gelu")
        res["o"] = K.attention(q, k, v, True, 128 ** -0.5)

    eager = {}
    work()
    torch.cuda.synchronize()
    eager["c"], eager["o"] = res["c"].clone(), res["o"].clone()
    g = _capture(work)                      # outputs are allocated by torch inside the capture: graph-private memory
    for rep in range(3):
        res["c"].zero_()
        res["o"].zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert rt.last_kernel_name() is not None
        assert torch.equal(res["c"], eager["c"]) and torch.equal(res["o"], eager["o"]), rep


def test_large_reduction_in_a_graph():
    """A reduction of 128 KiB and more runs on several workgroups through a per-stream buffer that the first
    eager call on a stream allocates.  Recorded into a graph it takes the one-workgroup form, whether the stream
    has such a buffer or not, so the graph holds no address of the library's."""
    n = 1 << 20
    x = torch.randint(-2**31, 2**31 - 1, (n, ), device="cuda", dtype=torch.int64).to(torch.int32)
    z = torch.zeros(1, device="cuda", dtype=torch.int32)
    za = torch.zeros(1, device="cuda", dtype=torch.int32)

    def work():
        K.reduce1d_kernel[(1, )](x, z, BLOCK=n, OP="sum")
        K.reduce1d_kernel[(1, )](x, za, BLOCK=n, OP="argmax")

    # a fresh side stream: nothing may be allocated while it records
    fresh = torch.cuda.Stream()
    torch.cuda.synchronize()
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1, stream=fresh):
        work()
    # a side stream that has run the reduction before
    warm = torch.cuda.Stream()
    with torch.cuda.stream(warm):
        work()
    torch.cuda.synchronize()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=warm):
        work()
    for rep in range(4):
        x.copy_(torch.randint(-2**31, 2**31 - 1, (n, ), device="cuda", dtype=torch.int64).to(torch.int32))
        torch.cuda.synchronize()
        want_sum = int(x.sum(dtype=torch.int64).item()) & 0xffffffff
        want_arg = int(torch.argmax(x).item())           # ties are as good as impossible in 2^20 draws from 2^32
        for g in (g1, g2):
            z.fill_(-7)
            za.fill_(-7)
            g.replay()
            torch.cuda.synchronize()
            assert int(z.item()) & 0xffffffff == want_sum and int(za.item()) == want_arg, rep
        work()                                           # and eagerly, between the replays
        torch.cuda.synchronize()
        assert int(z.item()) & 0xffffffff == want_sum and int(za.item()) == want_arg


def test_graph_with_a_large_reduction_replayed_on_another_stream_beside_eager_calls():
    """A graph recorded on stream A (which owns a buffer of partial results from earlier eager calls) is replayed on
    stream B while eager several-workgroup reductions of other data run on A: the graph shares nothing with them,
    so both give their own right answers every time.  Bounded: 100 rounds, stops at the first mismatch."""
    n = 1 << 20
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randint(-2**31, 2**31 - 1, (n, ), device="cuda", dtype=torch.int64, generator=g).to(torch.int32)
    y = torch.randint(-2**31, 2**31 - 1, (n, ), device="cuda", dtype=torch.int64, generator=g).to(torch.int32)
    zx = torch.zeros(1, device="cuda", dtype=torch.int32)
    zy = torch.zeros(1, device="cuda", dtype=torch.int32)
    want_x = int(x.sum(dtype=torch.int64).item()) & 0xffffffff
    want_y = int(y.sum(dtype=torch.int64).item()) & 0xffffffff
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(a):
        K.reduce1d_kernel[(1, )](x, zx, BLOCK=n, OP="sum")     # a now owns a buffer
    torch.cuda.synchronize()
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr, stream=a):
        K.reduce1d_kernel[(1, )](x, zx, BLOCK=n, OP="sum")
    for rep in range(100):
        zx.fill_(-7)
        zy.fill_(-7)
        torch.cuda.synchronize()
        with torch.cuda.stream(b):
            gr.replay()
        with torch.cuda.stream(a):
            for _ in range(4):
                K.reduce1d_kernel[(1, )](y, zy, BLOCK=n, OP="sum")
        torch.cuda.synchronize()
        assert int(zx.item()) & 0xffffffff == want_x and int(zy.item()) & 0xffffffff == want_y, rep
