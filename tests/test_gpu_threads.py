"""The C ABI from several host threads, each on its own stream: kernels are immutable after load, the lookup
tables are locked, errors and "last kernel" are per thread, so concurrent launches on distinct streams are safe."""
import threading

import pytest
import torch

from triton_tenstorrent_amd import kernels as K
from triton_tenstorrent_amd import runtime as rt

pytestmark = pytest.mark.gpu


def test_concurrent_launches_from_four_threads():
    rt.init(0)
    n_threads, rounds = 4, 40
    errors: list = []
    results: dict = {}

    def worker(tid: int):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            g = torch.Generator(device="cuda").manual_seed(tid)
            with torch.cuda.stream(stream):
                x = torch.randn(70001 + tid, device="cuda", generator=g)
                y = torch.randn(70001 + tid, device="cuda", generator=g)
                a = torch.randint(-3, 4, (256, 128), device="cuda", generator=g).to(torch.bfloat16)
                b = torch.randint(-3, 4, (128, 264), device="cuda", generator=g).to(torch.bfloat16)
                outs = []
                for _ in range(rounds):
                    s = K.add(x, y)
                    assert rt.last_kernel_name() == "ew_add_f32"            # this thread's own last launch
                    c = K.matmul_tma(a, b)
                    assert rt.last_kernel_name().startswith("gemm_")
                    z = K.reduce1d("argmax", x[:4096])
                    outs.append((s, c, z))
                # an error in this thread stays in this thread
                with pytest.raises(rt.InvalidLaunch):
                    K.add_kernel[(1, )](x, y, s, -5, BLOCK_SIZE=1024)
                assert "n_elements" in rt.last_error()
                stream.synchronize()
                want_s, want_c, want_z = x + y, (a.float() @ b.float()).to(torch.bfloat16), torch.argmax(x[:4096])
                for s, c, z in outs:
                    assert torch.equal(s, want_s) and torch.equal(c, want_c) and int(z) == int(want_z)
            results[tid] = True
        except BaseException as e:      # noqa: BLE001 - reported in the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(i, )) for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert len(results) == n_threads and not any(t.is_alive() for t in threads)


def test_matmuls_in_slices_of_k_from_threads_that_share_a_stream():
    """A matmul of few tiles under a long K is two launches that share the stream's workspace.  Threads that feed ONE
    stream (each orders its own work with the others' only through that stream) must not interleave their pairs:
    small-integer operands, so every result is exact and a slab of another thread's slices would show."""
    rt.init(0)
    n_threads, rounds = 4, 30
    stream = torch.cuda.Stream()
    errors: list = []
    done: list = []
    g = torch.Generator(device="cuda").manual_seed(3)
    shapes = [(64, 256, 2048), (200, 520, 2048), (130, 264, 4096), (16, 512, 4096)]
    data = []
    for (M, N, Kd) in shapes:
        a = torch.randint(-3, 4, (M, Kd), device="cuda", generator=g).to(torch.bfloat16)
        b = torch.randint(-3, 4, (Kd, N), device="cuda", generator=g).to(torch.bfloat16)
        data.append((a, b, (a.float() @ b.float()).to(torch.bfloat16)))
    torch.cuda.synchronize()

    def worker(tid: int):
        try:
            torch.cuda.set_device(0)
            a, b, want = data[tid]
            with torch.cuda.stream(stream):
                outs = []
                for _ in range(rounds):
                    outs.append(K.matmul_tma(a, b))
                    assert rt.last_kernel_name() == "gemm_splitk_reduce_bf16"
                stream.synchronize()
                for c in outs:
                    assert torch.equal(c, want)
            done.append(tid)
        except BaseException as e:      # noqa: BLE001 - reported in the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(i, )) for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert len(done) == n_threads and not any(t.is_alive() for t in threads)
