#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only gemm,add,...] [--no-cpu]

One "step" is one launch of the persistent bf16 GEMM, M=N=K=8192 (BASELINE
configs[2], the configuration the metric's TFLOP/s figure is quoted on), with
inputs resident in HBM.  The other configurations of the metric (elementwise
streaming, fused epilogue, fp8, attention) are measured beside it and reported
under "extra", each with its own roofline fraction.  Kernel durations come from
HIP events recorded on the stream the kernels are launched on.  Prints ONE JSON
line.
"""
from __future__ import annotations

import argparse
import json
import math
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBS = 8000.0        # MI355X HBM3E
PEAK_BF16_TFLOPS = 2500.0    # dense MFMA bf16 / fp16
PEAK_FP8_TFLOPS = 5000.0     # dense MFMA fp8


SPINUP_MS = 30.0      # set from --spinup-ms
SPINUP_LAUNCHES: dict = {}


def _events_time(fn, steps: int, warmup: int, stream: int, tag: str | None = None):
    """Run fn() warmup+steps times; returns (avg_ms over the K-step region, list of per-launch ms, wall ms per step).

    Before the warm-up steps the same fn() is launched for SPINUP_MS of wall time: the part's clock climbs
    from its idle state over the first tens of milliseconds of load (the 8192^3 GEMM measures 0.95-1.2 ms for
    its first ~25 launches and 0.84 ms from then on), and a sub-benchmark that follows host-side set-up would
    otherwise be timed on that slope.  Untimed, like the warm-up; the count goes into extra['spinup_launches']."""
    import torch
    from triton_tenstorrent_amd import runtime as rt
    spun = 0
    t_spin = time.perf_counter()
    while (time.perf_counter() - t_spin) * 1e3 < SPINUP_MS:
        for _ in range(8):
            fn()
        spun += 8
        torch.cuda.synchronize()
    if tag is not None:
        SPINUP_LAUNCHES[tag] = spun
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [rt.Event() for _ in range(steps + 1)]
    t0 = time.perf_counter()
    evs[0].record(stream)
    for i in range(steps):
        fn()
        evs[i + 1].record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per = [evs[i].elapsed_time(evs[i + 1]) for i in range(steps)]
    total = evs[0].elapsed_time(evs[steps])
    return total / steps, per, wall_ms / steps


# HBM-side bytes per launch, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this file (KiB per
# dispatch, FETCH_SIZE scaled by 2.0 and WRITE_SIZE by 1.0: what the same counters read for the int32 add, a
# plain copy-like kernel of known size).  Not measured live: the counters need the profiler around the process.
# profiles/bench_all_kernels_rocprofv3.md holds the raw readings and the commands.
TRAFFIC_FROM_COMMIT = "fddd240"   # the tree the readings below were taken from
TRAFFIC_KERNELS_SHA = "7b15c66926959939"   # _kernel_sources_sha() of that tree: a kernel edit after the readings shows in the JSON
MEASURED_TRAFFIC_BYTES = {
    "gemm_tile_bf16_epi0": int((2 * 795938 + 134110) * 1024),
    "gemm_tile_bf16_epi2": int((2 * 385288 + 117760) * 1024),
    "gemm_tile_fp8_bf16": int((2 * 407758 + 157285) * 1024),
    "gemm_tiled_f16_epi0": int((2 * 790342 + 132864) * 1024),
    "attn_tile_d128": int((2 * 306392 + 133123) * 1024),     # the causal launches
    "ew_add_i32": int((2 * 1048588 + 1048576) * 1024),
    "ew_sin_f32": int((2 * 524332 + 1048578) * 1024),
}


def _kernel_sources_sha() -> str:
    """Digest of the kernel sources (names and contents of csrc/kernels), to tell whether the traffic readings above
    still describe the kernels that run."""
    import hashlib
    h = hashlib.sha256()
    for f in sorted((ROOT / "triton-tenstorrent_amd" / "csrc" / "kernels").iterdir()):
        if f.is_file():
            h.update(f.name.encode())
            h.update(f.read_bytes())
    return h.hexdigest()[:16]


def _roof(bound: str, achieved: float, peak: float, unit: str, kernel: str = ""):
    return {"bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(kernel)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--spinup-ms", type=float, default=30.0,
                    help="untimed run of each kernel before its warm-up steps, so that the clock has left its idle state")
    ap.add_argument("--only", type=str, default="", help="comma list of: gemm,add,sin,ops,ew_ceiling,fused,fp8,tiled,attn,add0")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE MI355X; every kernel here shards without communication "
              "and no multi-GPU figure is produced (--gpus must be 1)", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    import __graft_entry__ as ge
    ge._package()
    from triton_tenstorrent_amd import kernels as K
    from triton_tenstorrent_amd import runtime as rt
    from triton_tenstorrent_amd.tensor_descriptor import TensorDescriptor

    if not torch.cuda.is_available():
        print("bench.py needs the GPU (no CPU fallback exists)", file=sys.stderr)
        return 2
    only = set(filter(None, args.only.split(",")))
    want = lambda name: not only or name in only
    props = rt.device_props()
    stream = torch.cuda.current_stream().cuda_stream
    steps, warmup = args.steps, args.warmup
    global SPINUP_MS
    SPINUP_MS = max(0.0, args.spinup_ms)
    extra: dict = {"device": props["name"], "arch": props["arch"], "cus": props["multiprocessor_count"],
                   "clock_mhz": props["clock_khz"] // 1000,
                   "peaks": {"hbm_GBs": PEAK_HBM_GBS, "bf16_TFLOPs": PEAK_BF16_TFLOPS, "fp8_TFLOPs": PEAK_FP8_TFLOPS}}
    extra["traffic_from_commit"] = TRAFFIC_FROM_COMMIT
    extra["traffic_kernels_unchanged"] = _kernel_sources_sha() == TRAFFIC_KERNELS_SHA
    rooflines: dict = {}
    parity_failed = False
    torch.manual_seed(0)

    # ---------------- primary: persistent bf16 GEMM 8192^3 -----------------
    M = N = Kd = 8192
    value = ms_per_step = None
    primary_roof = None
    if want("gemm"):
        a = (torch.randn(M, Kd, device="cuda") / math.sqrt(Kd)).to(torch.bfloat16)
        b = (torch.randn(Kd, N, device="cuda") / math.sqrt(Kd)).to(torch.bfloat16)
        c = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
        grid = (K.cdiv(M, 128) * K.cdiv(N, 128), )

        def gemm_step():
            K.matmul_kernel_tma[grid](ad, bd, cd, M, N, Kd, FP8_OUTPUT=False, WARP_SPECIALIZE=False)

        # barrier + synchronize on both sides of exactly K timed steps
        avg_ms, per, wall_ms = _events_time(gemm_step, steps, warmup, stream, "gemm_tile_bf16_epi0")
        flops = 2.0 * M * N * Kd
        value = flops / (avg_ms * 1e-3) / 1e12
        ms_per_step = avg_ms
        primary_roof = _roof("mfma", value, PEAK_BF16_TFLOPS, "TFLOP/s", "gemm_tile_bf16_epi0")
        extra["gemm_bf16_8192"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4),
                                   "ms_min": round(min(per), 4), "ms_median": round(statistics.median(per), 4),
                                   "wall_ms_per_step": round(wall_ms, 4), "TFLOPs": round(value, 2),
                                   "TFLOPs_best": round(flops / (min(per) * 1e-3) / 1e12, 2)}
        # spot parity on the benchmark's own output: 64 random rows against fp64 on the host
        rows = torch.randint(0, M, (64, ), device="cuda")
        ref = (a[rows].double() @ b.double()).float()
        err = (c[rows].float() - ref).abs()
        ok = bool(torch.all(err <= 1e-2 * ref.abs() + 1e-4))
        extra["gemm_bf16_8192"]["parity_rows_ok"] = ok
        if not ok:
            print("bench.py: GEMM output failed its parity spot check", file=sys.stderr)
            return 1
        # The kernel is bounded by power, so its rate follows the core clock the box grants under it (1.6-1.8 GHz
        # against the 2.4 GHz the peak is quoted at), and boxes differ.  One untimed launch behind a run of ordinary
        # ones reports workgroup 0's core cycles and wall ticks: with it two lines from two boxes can be compared.
        readings = []
        for _ in range(5):          # five probed launches, each behind a run of ordinary ones; the median clock
            for _ in range(8):
                gemm_step()
            rt.gemm_clock_probe(arm=True)
            gemm_step()
            torch.cuda.synchronize()
            r = rt.gemm_clock_probe()
            if r is not None:
                readings.append(r[2])
        if readings:
            ghz = statistics.median(readings)
            extra["gemm_bf16_8192"]["clock_under_load_GHz"] = round(ghz, 3)
            extra["gemm_bf16_8192"]["clock_under_load_GHz_minmax"] = [round(min(readings), 3), round(max(readings), 3)]
            # the MFMA peak at the granted clock, and the kernel against that
            extra["gemm_bf16_8192"]["peak_at_granted_clock_TFLOPs"] = round(PEAK_BF16_TFLOPS * ghz / (props["clock_khz"] / 1e6), 1)
            extra["gemm_bf16_8192"]["frac_at_granted_clock"] = round(value / (PEAK_BF16_TFLOPS * ghz / (props["clock_khz"] / 1e6)), 4)
        # ... and the ceiling to lay it against: the same MFMAs alone (no LDS, no copies, no barrier) on the
        # benchmark's own operand values, one wavefront per SIMD on every CU, and the clock the box grants under THAT
        import ctypes as C
        lib = rt.init(0)
        mod, kh = C.c_void_p(), C.c_void_p()
        rt.check(lib.rt_builtin_module(b"gemm", C.byref(mod)))
        rt.check(lib.rt_get_kernel(mod, b"gemm_mfma_ceiling_bf16", C.byref(kh)))
        sink = torch.zeros(4, device="cuda")
        probe = torch.zeros(2, device="cuda", dtype=torch.int64)
        iters = 3000
        vals = [C.c_int(iters), C.c_void_p(a.data_ptr()), C.c_void_p(sink.data_ptr()), C.c_void_p(probe.data_ptr())]
        kargs = (C.c_void_p * 4)(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])     # (src: 64 x 16 x 256 fragments of A)
        cus = props["multiprocessor_count"]
        g3, b3 = rt.grid3(cus), rt.grid3(256)
        avg_c, per_c, _ = _events_time(lambda: rt.check(lib.rt_launch(kh, g3, b3, 0, C.c_void_p(stream), kargs, 4)),
                                       max(5, steps // 2), 3, stream)
        extra["gemm_bf16_8192"]["mfma_only_TFLOPs"] = round(4 * cus * iters * 2.0 ** 20 / (avg_c * 1e-3) / 1e12, 1)
        pr = probe.tolist()
        if pr[1]:
            extra["gemm_bf16_8192"]["mfma_only_clock_GHz"] = round(pr[0] / pr[1] / 10.0, 3)
        extra["gemm_bf16_8192"]["kernel_over_mfma_only"] = round(value / extra["gemm_bf16_8192"]["mfma_only_TFLOPs"], 4)
        del a, b, c, ad, bd, cd, sink, probe
        # shapes that are not whole 256x256x128 macro tiles run the same kernel's clamping instantiation
        ragged = {}
        for (m_, n_, k_) in ((8000, 8192, 8192), (8192, 8192, 8160)):
            a = (torch.randn(m_, k_, device="cuda") / math.sqrt(k_)).to(torch.bfloat16)
            b = (torch.randn(k_, n_, device="cuda") / math.sqrt(k_)).to(torch.bfloat16)
            avg_ms, per, _ = _events_time(lambda: K.matmul_tma(a, b), max(3, steps // 4), 2, stream)
            ragged[f"{m_}x{n_}x{k_}"] = {"kernel": rt.last_kernel_name(), "TFLOPs": round(2.0 * m_ * n_ * k_ / (avg_ms * 1e-3) / 1e12, 1)}
            del a, b
        extra["gemm_bf16_ragged_shapes"] = ragged
        # few output tiles under a long K: computed in slices of K (two launches; the time is that of the pair).  These
        # are bounded by the one pass over B: GB/s of A + B + C against the HBM peak
        skinny = {}
        for (m_, n_, k_) in ((16, 8192, 8192), (128, 8192, 8192), (64, 4096, 8192)):
            a = (torch.randn(m_, k_, device="cuda") / math.sqrt(k_)).to(torch.bfloat16)
            b = (torch.randn(k_, n_, device="cuda") / math.sqrt(k_)).to(torch.bfloat16)
            avg_ms, per, _ = _events_time(lambda: K.matmul_tma(a, b), max(3, steps // 4), 2, stream)
            byts = 2.0 * (m_ * k_ + k_ * n_ + m_ * n_)
            skinny[f"{m_}x{n_}x{k_}"] = {"kernel": rt.last_kernel_name(), "us": round(avg_ms * 1e3, 1),
                                         "TFLOPs": round(2.0 * m_ * n_ * k_ / (avg_ms * 1e-3) / 1e12, 1),
                                         "GBs": round(byts / (avg_ms * 1e-3) / 1e9, 0),
                                         "frac_of_hbm_peak": round(byts / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 3)}
            del a, b
        extra["gemm_bf16_few_tiles_long_k"] = skinny

    # ---------------- elementwise streaming, N = 2^28 ----------------------
    n_el = 1 << 28
    if want("add"):
        g = torch.Generator(device="cuda").manual_seed(0)
        x = torch.randint(-2**20, 2**20, (n_el, ), dtype=torch.int32, device="cuda", generator=g)
        y = torch.randint(-2**20, 2**20, (n_el, ), dtype=torch.int32, device="cuda", generator=g)
        out = torch.empty_like(x)
        egrid = (K.cdiv(n_el, 1024), )
        avg_ms, per, _ = _events_time(lambda: K.add_kernel[egrid](x, y, out, n_el, BLOCK_SIZE=1024), steps, warmup, stream, "ew_add_i32")
        gbs = 3 * 4 * n_el / (avg_ms * 1e-3) / 1e9
        assert torch.equal(out[:1 << 20], x[:1 << 20] + y[:1 << 20])
        extra["add_i32_2p28"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4), "ms_min": round(min(per), 4),
                                 "GBs": round(gbs, 1)}
        rooflines["add_i32_2p28"] = _roof("hbm", gbs, PEAK_HBM_GBS, "GB/s", "ew_add_i32")
        del x, y, out
    if want("sin"):
        xs = (torch.rand(n_el, device="cuda") * 2 - 1) * (8 * math.pi)
        outs = torch.empty_like(xs)
        egrid = (K.cdiv(n_el, 1024), )
        avg_ms, per, _ = _events_time(lambda: K.sin_kernel[egrid](xs, outs, n_el, BLOCK_SIZE=1024), steps, warmup, stream, "ew_sin_f32")
        gbs = 2 * 4 * n_el / (avg_ms * 1e-3) / 1e9
        extra["sin_f32_2p28"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4), "ms_min": round(min(per), 4),
                                 "GBs": round(gbs, 1),
                                 "max_abs_err_vs_f64": float((outs[:1 << 20].double() - torch.sin(xs[:1 << 20].double())).abs().max())}
        rooflines["sin_f32_2p28"] = _roof("hbm", gbs, PEAK_HBM_GBS, "GB/s", "ew_sin_f32")
        del xs, outs
    if want("ops"):
        # the other operations of the elementwise family at the streaming size: they have to stay under the HBM shadow
        xs = torch.rand(n_el, device="cuda") + 0.5
        ys = torch.rand(n_el, device="cuda") + 0.5
        outs = torch.empty_like(xs)
        egrid = (K.cdiv(n_el, 1024), )
        ops = {}
        for op in ("exp", "log", "cos", "rsqrt", "sqrt"):
            avg_ms, per, _ = _events_time(lambda: K.unary_kernel[egrid](xs, outs, n_el, BLOCK_SIZE=1024, OP=op),
                                          max(3, steps // 4), 2, stream)
            ops[op] = round(2 * 4 * n_el / (avg_ms * 1e-3) / 1e9, 1)
        for op in ("div", "maximum"):
            avg_ms, per, _ = _events_time(lambda: K.binary_kernel[egrid](xs, ys, outs, n_el, BLOCK_SIZE=1024, OP=op),
                                          max(3, steps // 4), 2, stream)
            ops[op] = round(3 * 4 * n_el / (avg_ms * 1e-3) / 1e9, 1)
        ob = torch.empty(n_el, device="cuda", dtype=torch.bfloat16)
        avg_ms, per, _ = _events_time(lambda: K.cast_kernel[egrid](xs, ob, n_el, BLOCK_SIZE=1024), max(3, steps // 4), 2, stream)
        ops["truncf_bf16"] = round((4 + 2) * n_el / (avg_ms * 1e-3) / 1e9, 1)
        del ob
        avg_ms, per, _ = _events_time(lambda: K.copy_kernel[egrid](xs, outs, n_el, BLOCK_SIZE=1024), max(3, steps // 4), 2, stream)
        ops["copy"] = round(2 * 4 * n_el / (avg_ms * 1e-3) / 1e9, 1)
        extra["elementwise_ops_2p28_GBs"] = ops
        del xs, ys, outs
    if "ew_ceiling" in only or not only:
        # what the streaming geometry reaches when it only reads, only writes, or copies: the bounds the 2-read/1-write
        # add and the 1-read/1-write sin sit under (the kernels are diagnostics inside the elementwise code object)
        import ctypes as C
        lib = rt.init(0)
        mod = C.c_void_p()
        rt.check(lib.rt_builtin_module(b"elementwise", C.byref(mod)))
        xs = torch.randint(-2**20, 2**20, (n_el, ), dtype=torch.int32, device="cuda")
        outs = torch.empty_like(xs)
        nvec = n_el // 4
        ceil = {}
        for kname, per_wg in (("ew_ceiling_read_b128", 1024), ("ew_ceiling_write_b128", 256)):
            nbytes = 4 * n_el
            kh = C.c_void_p()
            rt.check(lib.rt_get_kernel(mod, kname.encode(), C.byref(kh)))
            vals = [C.c_void_p(xs.data_ptr()), C.c_void_p(outs.data_ptr()), C.c_uint32(nvec)]
            kargs = (C.c_void_p * 3)(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])
            g3, b3 = rt.grid3(nvec // per_wg), rt.grid3(256)
            avg_ms, per, _ = _events_time(lambda: rt.check(lib.rt_launch(kh, g3, b3, 0, C.c_void_p(stream), kargs, 3)),
                                          max(3, steps // 2), 3, stream)
            ceil[kname] = round(nbytes / (avg_ms * 1e-3) / 1e9, 1)
        egrid = (K.cdiv(n_el, 1024), )
        avg_ms, per, _ = _events_time(lambda: K.copy_kernel[egrid](xs, outs, n_el, BLOCK_SIZE=1024), max(3, steps // 2), 3, stream)
        ceil["ew_copy_b128"] = round(2 * 4 * n_el / (avg_ms * 1e-3) / 1e9, 1)
        r, w = ceil["ew_ceiling_read_b128"], ceil["ew_ceiling_write_b128"]
        # bytes move at the read rate or at the write rate: the harmonic mix for a kernel's read:write ratio
        ceil["bound_2r1w_GBs"] = round(3.0 / (2.0 / r + 1.0 / w), 1)
        ceil["bound_1r1w_GBs"] = round(2.0 / (1.0 / r + 1.0 / w), 1)
        extra["ew_ceiling_2p28_GBs"] = ceil
        del xs, outs
    if want("add0"):
        n0 = 98432
        x0, y0 = torch.rand(n0, device="cuda"), torch.rand(n0, device="cuda")
        o0 = torch.empty_like(x0)
        launch0 = K.add_kernel[(97, )]
        avg_ms, per, _ = _events_time(lambda: launch0(x0, y0, o0, n0, BLOCK_SIZE=1024), 200, 20, stream)
        # host time per launch: the loop alone, no events between the launches, the clock stopped before the sync
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5000):
            launch0(x0, y0, o0, n0, BLOCK_SIZE=1024)
        host_us = (time.perf_counter() - t0) / 5000 * 1e6
        torch.cuda.synchronize()
        extra["add_f32_98432"] = {"us_avg": round(avg_ms * 1e3, 2), "us_min": round(min(per) * 1e3, 2),
                                  "host_us_per_launch": round(host_us, 2), "GBs": round(3 * 4 * n0 / (avg_ms * 1e-3) / 1e9, 1)}
        # the same launch recorded 100 times into a HIP graph: what is left when the host is out of the loop
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for _ in range(100):
                K.add_kernel[(97, )](x0, y0, o0, n0, BLOCK_SIZE=1024)
        gr.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            gr.replay()
        e1.record()
        torch.cuda.synchronize()
        extra["add_f32_98432"]["us_per_launch_in_hip_graph"] = round(e0.elapsed_time(e1) * 1e3 / 1000, 2)
        # the single-block reductions: one program by construction, so a latency figure, not a roofline one
        red = {}
        for nr in (512, 1 << 20):
            xr = torch.randn(nr, device="cuda")
            zr = torch.empty(1, device="cuda")
            for op in ("sum", "argmax"):
                zi = zr if op == "sum" else torch.empty(1, device="cuda", dtype=torch.int32)
                avg_ms, per, _ = _events_time(lambda: K.reduce1d_kernel[(1, )](xr, zi, BLOCK=nr, OP=op), 50, 5, stream)
                red[f"{op}_f32_{nr}"] = {"us_avg": round(avg_ms * 1e3, 2), "us_min": round(min(per) * 1e3, 2)}
        extra["reduce1d"] = red
        del gr
        # a matmul small enough that the launch path is what is timed (the kernel itself takes about 5 us): the
        # reference-style wrapper (three descriptors made per call, a callable grid) and the bare launch
        a512 = torch.randn(512, 512, device="cuda").to(torch.bfloat16)
        b512 = torch.randn(512, 512, device="cuda").to(torch.bfloat16)
        for _ in range(20):
            K.matmul_tma(a512, b512)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(2000):
            K.matmul_tma(a512, b512)
        wrap_us = (time.perf_counter() - t0) / 2000 * 1e6
        torch.cuda.synchronize()
        c512 = torch.empty(512, 512, device="cuda", dtype=torch.bfloat16)
        d512 = [TensorDescriptor.from_tensor(t, [32, 32]) for t in (a512, b512, c512)]
        launch_m = K.matmul_kernel_tma[(16, )]
        for _ in range(20):
            launch_m(*d512, 512, 512, 512, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(2000):
            launch_m(*d512, 512, 512, 512, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
        bare_us = (time.perf_counter() - t0) / 2000 * 1e6
        torch.cuda.synchronize()
        extra["matmul_bf16_512"] = {"host_us_per_launch": round(bare_us, 2), "host_us_per_wrapper_call": round(wrap_us, 2)}

    # ---------------- fused epilogue: GELU(A.B + bias) ----------------------
    if want("fused"):
        Mf, Nf, Kf = 4096, 14336, 4096
        a = (torch.randn(Mf, Kf, device="cuda") / math.sqrt(Kf)).to(torch.bfloat16)
        b = (torch.randn(Kf, Nf, device="cuda") / math.sqrt(Kf)).to(torch.bfloat16)
        bias = (torch.randn(Nf, device="cuda") * 0.02).reshape(1, Nf)
        c = torch.empty(Mf, Nf, device="cuda", dtype=torch.bfloat16)
        ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
        biasd = TensorDescriptor.from_tensor(bias, [1, 32])
        grid = (K.cdiv(Mf, 128) * K.cdiv(Nf, 128), )
        avg_ms, per, _ = _events_time(
            lambda: K.matmul_kernel_fused[grid](ad, bd, cd, biasd, Mf, Nf, Kf, FP8_OUTPUT=False, WARP_SPECIALIZE=False,
                                                EPILOGUE="gelu"), steps, warmup, stream, "gemm_tile_bf16_epi2")
        tf = 2.0 * Mf * Nf * Kf / (avg_ms * 1e-3) / 1e12
        extra["gemm_gelu_4096x14336x4096"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4),
                                              "ms_min": round(min(per), 4), "TFLOPs": round(tf, 2)}
        rooflines["gemm_gelu_4096x14336x4096"] = _roof("mfma", tf, PEAK_BF16_TFLOPS, "TFLOP/s", "gemm_tile_bf16_epi2")
        # spot parity on the timed output: 64 random rows against float64 erf-GELU
        rows = torch.randint(0, Mf, (64, ), device="cuda")
        ref = torch.nn.functional.gelu(a[rows].double() @ b.double() + bias.double()).float()
        ok = bool(torch.all((c[rows].float() - ref).abs() <= 1e-2 * ref.abs() + 1e-4))
        extra["gemm_gelu_4096x14336x4096"]["parity_rows_ok"] = ok
        # the same shape without the epilogue: what the bias and the GELU cost, apart from what the shape costs
        # (896 macro tiles on 256 CUs are 3.5 rounds, the last one run as half tiles)
        c2 = torch.empty_like(c)
        c2d = TensorDescriptor.from_tensor(c2, [32, 32])
        avg0, _, _ = _events_time(
            lambda: K.matmul_kernel_tma[grid](ad, bd, c2d, Mf, Nf, Kf, FP8_OUTPUT=False, WARP_SPECIALIZE=False),
            steps, warmup, stream)
        tf0 = 2.0 * Mf * Nf * Kf / (avg0 * 1e-3) / 1e12
        extra["gemm_gelu_4096x14336x4096"]["plain_same_shape_TFLOPs"] = round(tf0, 2)
        extra["gemm_gelu_4096x14336x4096"]["gelu_over_plain"] = round(tf / tf0, 4)
        del c2, c2d
        parity_failed |= not ok
        del a, b, c, bias, ref
    if want("fp8"):
        xa = torch.randn(M, Kd, device="cuda")
        qa, sa = K.quantize_fp8(xa)
        del xa
        xb = torch.randn(Kd, N, device="cuda")
        qb, sb = K.quantize_fp8(xb)
        del xb
        c = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (qa, qb, c))
        grid = (K.cdiv(M, 128) * K.cdiv(N, 128), )
        avg_ms, per, _ = _events_time(
            lambda: K.matmul_kernel_tma_fp8_scaled[grid](ad, bd, cd, M, N, Kd, sa, sb, FP8_OUTPUT=False, WARP_SPECIALIZE=False),
            steps, warmup, stream, "gemm_tile_fp8_bf16")
        tf = 2.0 * M * N * Kd / (avg_ms * 1e-3) / 1e12
        extra["gemm_fp8_8192"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4), "ms_min": round(min(per), 4),
                                  "TFLOPs": round(tf, 2)}
        rooflines["gemm_fp8_8192"] = _roof("mfma", tf, PEAK_FP8_TFLOPS, "TFLOP/s", "gemm_tile_fp8_bf16")
        # spot parity: 64 random rows against float64 on the dequantised operands; the absolute slack follows the
        # output's rms, since fp8 products summed over K cancel to values no relative bound can hold
        rows = torch.randint(0, M, (64, ), device="cuda")
        ref = ((qa[rows].double() @ qb.double()) * (sa * sb)).float()
        atol = 1e-4 * max(1.0, float(ref.square().mean().sqrt()))
        ok = bool(torch.all((c[rows].float() - ref).abs() <= 1e-2 * ref.abs() + atol))
        extra["gemm_fp8_8192"]["parity_rows_ok"] = ok
        parity_failed |= not ok
        del qa, qb, c, ref
        # few output tiles under a long K, in slices of K: bounded by the one pass over B (one byte an element)
        skinny8 = {}
        for (m_, n_, k_) in ((16, 8192, 8192), (128, 8192, 8192)):
            qa, sa = K.quantize_fp8(torch.randn(m_, k_, device="cuda"))
            qb, sb = K.quantize_fp8(torch.randn(k_, n_, device="cuda"))
            avg_ms, per, _ = _events_time(lambda: K.matmul_fp8_scaled(qa, qb, sa, sb), max(3, steps // 4), 2, stream)
            byts = 1.0 * (m_ * k_ + k_ * n_) + 2.0 * m_ * n_
            skinny8[f"{m_}x{n_}x{k_}"] = {"kernel": rt.last_kernel_name(), "us": round(avg_ms * 1e3, 1),
                                          "GBs": round(byts / (avg_ms * 1e-3) / 1e9, 0),
                                          "frac_of_hbm_peak": round(byts / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 3)}
            del qa, qb
        extra["gemm_fp8_few_tiles_long_k"] = skinny8
    if want("tiled"):
        # the pointer-based matmul_kernel on tile-major fp16 buffers, 32x32x32 tiles, same 8192^3 problem
        at = K.tilize((torch.randn(M, Kd, device="cuda") / math.sqrt(Kd)).to(torch.float16), 32, 32)
        bt = K.tilize((torch.randn(Kd, N, device="cuda") / math.sqrt(Kd)).to(torch.float16), 32, 32)
        ct = torch.empty(M * N, device="cuda", dtype=torch.float16)
        grid = (K.cdiv(M, 32) * K.cdiv(N, 32), )
        avg_ms, per, _ = _events_time(lambda: K.matmul_kernel[grid](at, bt, ct, M, N, Kd, Kd, 1, N, 1, N, 1), steps, warmup,
                                      stream, "gemm_tiled_f16_epi0")
        tf = 2.0 * M * N * Kd / (avg_ms * 1e-3) / 1e12
        extra["gemm_tiled_f16_8192"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4),
                                        "ms_min": round(min(per), 4), "TFLOPs": round(tf, 2)}
        rooflines["gemm_tiled_f16_8192"] = _roof("mfma", tf, PEAK_BF16_TFLOPS, "TFLOP/s", "gemm_tiled_f16_epi0")
        # spot parity: 64 random rows of the un-tiled result against float64 on the un-tiled operands
        rows = torch.randint(0, M, (64, ), device="cuda")
        a_rows = K.untilize(at, M, Kd, 32, 32)[rows].double()
        ref = (a_rows @ K.untilize(bt, Kd, N, 32, 32).double()).float()
        got = K.untilize(ct, M, N, 32, 32)[rows].float()
        ok = bool(torch.all((got - ref).abs() <= 1e-2 * ref.abs() + 1e-4))
        extra["gemm_tiled_f16_8192"]["parity_rows_ok"] = ok
        parity_failed |= not ok
        del at, bt, ct, ref, got, a_rows
    if want("attn"):
        Z, H, S, D = 4, 32, 4096, 128
        q, k, v = (torch.randn(Z, H, S, D, device="cuda").to(torch.bfloat16) for _ in range(3))
        sm = 1.0 / math.sqrt(D)
        o_buf = []

        def attn_step():
            o_buf[:] = [K.attention(q, k, v, True, sm)]

        avg_ms, per, _ = _events_time(attn_step, steps, warmup, stream, "attn_tile_d128")
        fl = 4.0 * Z * H * S * S * D / 2  # lower triangle only
        tf = fl / (avg_ms * 1e-3) / 1e12
        extra["attn_fwd_causal_4x32x4096x128"] = {"kernel": rt.last_kernel_name(), "ms_avg": round(avg_ms, 4),
                                                  "ms_min": round(min(per), 4), "TFLOPs": round(tf, 2)}
        rooflines["attn_fwd_causal_4x32x4096x128"] = _roof("mfma", tf, PEAK_BF16_TFLOPS, "TFLOP/s", "attn_tile_d128")
        # spot parity on the last timed output: 64 random rows of two heads against float64 softmax attention
        ok = True
        for (z, h) in ((1, 7), (3, 31)):
            rows = torch.randint(0, S, (64, ), device="cuda")
            sc = (q[z, h, rows].double() @ k[z, h].double().T) * sm
            sc = sc.masked_fill(rows[:, None] < torch.arange(S, device="cuda")[None, :], float("-inf"))
            ref = torch.softmax(sc, -1) @ v[z, h].double()
            ok &= bool((o_buf[0][z, h, rows].double() - ref).abs().max() <= 2e-2)
        extra["attn_fwd_causal_4x32x4096x128"]["parity_rows_ok"] = ok
        parity_failed |= not ok
        del q, k, v, o_buf
        # the other instantiations of the same kernel, for the record (few launches each; not roofline lines)
        others = {}
        for (z, h, s_, d, causal) in ((4, 32, 4096, 128, False), (4, 32, 4064, 128, True), (4, 32, 4096, 64, True),
                                      (4, 32, 4096, 32, True), (2, 16, 4096, 256, True)):
            q, k, v = (torch.randn(z, h, s_, d, device="cuda").to(torch.bfloat16) for _ in range(3))
            avg_ms, per, _ = _events_time(lambda: K.attention(q, k, v, causal, 1.0 / math.sqrt(d)), max(3, steps // 4), 2, stream)
            fl = 4.0 * z * h * s_ * s_ * d * (0.5 if causal else 1.0)
            others[f"{z}x{h}x{s_}x{d}_{'causal' if causal else 'full'}"] = {"kernel": rt.last_kernel_name(),
                                                                          "TFLOPs": round(fl / (avg_ms * 1e-3) / 1e12, 1)}
            del q, k, v
        extra["attn_fwd_other_shapes"] = others

    # ---------------- CPU baseline: the oracle on a bounded sample ---------
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import oracle as orc
        cores = orc.num_threads()
        rng = np.random.default_rng(0)
        ms = 8192  # the benchmark's own problem; repeated until about 10 s of CPU work have been timed
        ah = orc.to_bf16((rng.standard_normal((ms, ms)) / math.sqrt(ms)).astype(np.float32))
        bh = orc.to_bf16((rng.standard_normal((ms, ms)) / math.sqrt(ms)).astype(np.float32))
        ch = np.zeros((ms, ms), dtype=np.uint16)
        runs, total = 0, 0.0
        while runs < 8 and total < 10.0:
            t0 = time.perf_counter()
            orc.matmul(ah, bh, BM=128, BN=128, BK=64, group_m=8, out=ch)
            total += time.perf_counter() - t0
            runs += 1
        dt = total / runs
        cpu_baseline = {"value": round(2.0 * ms ** 3 / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                        "sample": f"oracle matmul_kernel_tma restatement (C, OpenMP, fp32 accumulate), bf16 M=N=K={ms}, "
                                  f"128x128x64 tiles, mean of {runs} runs, {total:.1f} s in all; built -O3 "
                                  "-march=x86-64-v3 -ffp-contract=off (a checker first: plain IEEE sums, no FMA contraction)"}
        del ah, bh, ch
        ne = 1 << 26
        xh = rng.integers(-2**20, 2**20, ne).astype(np.int32)
        yh = rng.integers(-2**20, 2**20, ne).astype(np.int32)
        oh = np.empty_like(xh)
        orc.add(xh, yh, oh)
        t0 = time.perf_counter()
        for _ in range(3):
            orc.add(xh, yh, oh)
        dt = (time.perf_counter() - t0) / 3
        extra["cpu_add_i32"] = {"GBs": round(3 * 4 * ne / dt / 1e9, 2), "cores": cores, "sample": f"N=2^26, mean of 3"}
        xf = ((rng.random(1 << 24, dtype=np.float32) * 2 - 1) * np.float32(8 * math.pi)).astype(np.float32)
        of = np.empty_like(xf)
        t0 = time.perf_counter()
        orc.sin(xf, of, libm_f32=True)
        dt = time.perf_counter() - t0
        extra["cpu_sin_f32"] = {"GBs": round(2 * 4 * xf.size / dt / 1e9, 3), "cores": cores, "sample": "N=2^24, libm sinf, one run"}
        # fused attention (configs[4]) on a bounded sample of the same shape: one batch entry, four heads
        za, ha, sa, da = 1, 4, 4096, 128
        qh, kh_, vh = (orc.to_bf16(rng.standard_normal((za, ha, sa, da)).astype(np.float32)) for _ in range(3))
        orc.attn_fwd(qh, kh_, vh, 1.0 / math.sqrt(da), causal=True, BLOCK_M=128, BLOCK_N=64)
        runs_a, total_a = 0, 0.0
        while runs_a < 8 and total_a < 4.0:
            t0 = time.perf_counter()
            orc.attn_fwd(qh, kh_, vh, 1.0 / math.sqrt(da), causal=True, BLOCK_M=128, BLOCK_N=64)
            total_a += time.perf_counter() - t0
            runs_a += 1
        fl_a = 4.0 * za * ha * sa * sa * da / 2
        tq, tk, tv = (torch.from_numpy(orc.from_bf16(t)).to(torch.bfloat16) for t in (qh, kh_, vh))
        torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)
        t0 = time.perf_counter()
        for _ in range(2):
            torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)
        dt_sdpa = (time.perf_counter() - t0) / 2
        extra["cpu_attn"] = {"TFLOPs": round(fl_a / (total_a / runs_a) / 1e12, 4), "cores": cores, "kind": "port",
                             "torch_sdpa_bf16_TFLOPs": round(fl_a / dt_sdpa / 1e12, 4), "torch_threads": torch.get_num_threads(),
                             "sample": f"oracle _attn_fwd restatement (C, OpenMP), causal, bf16 {za}x{ha}x{sa}x{da} (one batch entry and "
                                       f"four heads of configs[4]), BLOCK_M=128 BLOCK_N=64, mean of {runs_a} runs; beside it torch's "
                                       "CPU scaled_dot_product_attention on the same tensors, mean of 2; lower-triangle flops"}
        del qh, kh_, vh, tq, tk, tv
        # Library-grade CPU line: the same operations through torch's CPU kernels, as the reference's examples
        # compare against torch (01-vector-add.py:129-138).  Bounded samples, host tensors only.
        tx, ty = torch.from_numpy(xh), torch.from_numpy(yh)
        to = torch.empty_like(tx)
        torch.add(tx, ty, out=to)
        t0 = time.perf_counter()
        for _ in range(3):
            torch.add(tx, ty, out=to)
        dt_add = (time.perf_counter() - t0) / 3
        tf32 = torch.from_numpy(xf)
        tof = torch.empty_like(tf32)
        torch.sin(tf32, out=tof)
        t0 = time.perf_counter()
        torch.sin(tf32, out=tof)
        dt_sin = time.perf_counter() - t0
        mt = 4096
        ta = torch.randn(mt, mt) / math.sqrt(mt)
        tb = torch.randn(mt, mt) / math.sqrt(mt)
        torch.matmul(ta, tb)
        t0 = time.perf_counter()
        torch.matmul(ta, tb)
        dt_mm = time.perf_counter() - t0
        extra["cpu_torch"] = {"threads": torch.get_num_threads(),
                              "add_i32_GBs": round(3 * 4 * ne / dt_add / 1e9, 2),
                              "sin_f32_GBs": round(2 * 4 * xf.size / dt_sin / 1e9, 3),
                              "matmul_f32_4096_TFLOPs": round(2.0 * mt ** 3 / dt_mm / 1e12, 4),
                              "sample": "torch CPU kernels: add N=2^26 (mean of 3), sin N=2^24, fp32 matmul 4096^3 (one run each)"}

    line = {
        "metric": "GEMM TFLOP/s @8192^3 bf16 + elementwise GB/s, % of MI355X roofline",
        "value": None if value is None else round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": None if ms_per_step is None else round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "persistent GEMM C=A.B, bf16 in/out, fp32 accumulate, M=N=K=8192, logical tiles 128x128x64, "
                               "persistent grid = CU count (BASELINE configs[2]); elementwise int32 add / fp32 sin at N=2^28 "
                               "(configs[1]), GELU-fused GEMM and fp8 GEMM (configs[3]) and causal attention (configs[4]) under 'extra'"},
        "roofline": primary_roof,
        "cpu_baseline": cpu_baseline,
        "rooflines": rooflines,
        "extra": extra,
    }
    extra["spinup_ms"] = SPINUP_MS
    extra["spinup_launches"] = dict(SPINUP_LAUNCHES)
    print(json.dumps(line))
    if parity_failed:
        print("bench.py: a timed output failed its parity spot check (see parity_rows_ok under 'extra')", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
