#!/usr/bin/env python3
"""Writes the fixtures of this directory: seeded inputs and the outputs the CPU oracle gives for them.

    python tests/golden/make_golden.py            # rewrites tests/golden/*.npz

The reference holds no numeric vectors for these kernels (its tests compare against torch with PCC / atol
bars), so the expected values here come from this repository's oracle, whose functions are pinned against
independent routines in tests/test_oracle_*.py.  The fixtures freeze those outputs: tests/test_golden.py
checks that the oracle still reproduces them (a change of the oracle shows) and that the HIP kernels
meet each kernel's bar against the stored values with no oracle in the loop.

Every array is stored as plain numpy data (bf16 / fp16 / fp8 as their bit patterns); files load with
numpy.load(allow_pickle=False).
"""
from __future__ import annotations

import math
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))
from oracle import oracle as orc  # noqa: E402


def elementwise() -> dict:
    rng = np.random.default_rng(2024)
    n = 2500                                                   # 2 full blocks of 1024 and a tail of 452
    special = np.array([0.0, -0.0, 1.0, -1.0, 0.5, 2.5, -2.5, 1e-40, -1e-40, 3.4e38, -3.4e38, np.inf, -np.inf, np.nan,
                        88.7, -103.9, 127.5, -149.5, 6.1e-5], np.float32)
    x = np.concatenate([(rng.standard_normal(n - special.size) * 10).astype(np.float32), special])
    y = np.concatenate([(rng.standard_normal(n - special.size) * 3).astype(np.float32), special[::-1]])
    z = (rng.standard_normal(n) * 2).astype(np.float32)
    xi = rng.integers(-2**31, 2**31 - 1, n, dtype=np.int64).astype(np.int32)
    yi = rng.integers(-2**31, 2**31 - 1, n, dtype=np.int64).astype(np.int32)
    xs = ((rng.random(n, dtype=np.float32) * 2 - 1) * np.float32(8 * math.pi)).astype(np.float32)
    out = {"x": x, "y": y, "z": z, "xi": xi, "yi": yi, "xs": xs,
           "add_f32": orc.add(x, y), "add_i32": orc.add(xi, yi), "muladd": orc.muladd(x, y, z), "sin": orc.sin(xs),
           "trunci16": orc.trunci(xi, 16), "trunci8": orc.trunci(xi, 8),
           "truncf_bf16": orc.to_bf16(x), "truncf_f16": orc.to_f16(x)}
    for op in orc.UNARY_OPS:
        out[f"unary_{op}"] = orc.unary(op, x)
    for op in orc.BINARY_OPS:
        out[f"binary_{op}"] = orc.binary(op, x, y)
    return out


def matmul() -> dict:
    rng = np.random.default_rng(7)
    out = {}
    # small integers: every partial sum is exact, so the stored product is the answer for any tiling and order
    M, N, K = 96, 160, 64
    ai = orc.to_bf16(rng.integers(-4, 5, (M, K)).astype(np.float32))
    bi = orc.to_bf16(rng.integers(-4, 5, (K, N)).astype(np.float32))
    out.update(int_a=ai, int_b=bi, int_c=orc.matmul(ai, bi, BM=32, BN=32, BK=32))
    # the reference's validate shape 64x32x64 (09-persistent-matmul.py:326-327) on random data, fp64-accumulated
    a = orc.to_bf16((rng.standard_normal((64, 64)) / 8).astype(np.float32))
    b = orc.to_bf16(rng.standard_normal((64, 32)).astype(np.float32))
    out.update(a=a, b=b, c=orc.matmul(a, b, acc64=True))
    # fused: full [M,N] bias added in half precision after the cast (09-matmul-fused.py:139-146)
    bias_full = orc.to_bf16(rng.standard_normal((64, 32)).astype(np.float32))
    out.update(bias_full=bias_full, c_bias_full=orc.matmul(a, b, bias=bias_full, epi=orc.EPI_BIAS_FULL, acc64=True))
    # GELU(A.B + bias[N]) in fp32, one rounding
    bias_row = (rng.standard_normal(32) * 0.02).astype(np.float32)
    out.update(bias_row=bias_row, c_gelu=orc.matmul(a, b, bias=bias_row, epi=orc.EPI_BIAS_ROW_GELU, acc64=True))
    # fp8 e4m3 with per-tensor scales
    aq, sa = orc.quantize_fp8(rng.standard_normal((64, 64)).astype(np.float32))
    bq, sb = orc.quantize_fp8(rng.standard_normal((64, 32)).astype(np.float32))
    out.update(aq=aq, bq=bq, scales=np.array([sa, sb], np.float32),
               c_fp8=orc.matmul(aq, bq, in_dt=orc.FP8E4M3, out_dt=orc.BF16, scale=float(np.float32(sa) * np.float32(sb)),
                                acc64=True))
    # pointer-based matmul_kernel on tile-major fp16 buffers, ragged sizes, leaky_relu
    Mt, Nt, Kt = 70, 45, 50
    at = orc.to_f16((rng.standard_normal((Mt, Kt)) / 4).astype(np.float32))
    bt = orc.to_f16(rng.standard_normal((Kt, Nt)).astype(np.float32))
    a_tiled, b_tiled = orc.tilize(at, 32, 32), orc.tilize(bt, 32, 32)
    out.update(a_tiled=a_tiled, b_tiled=b_tiled, tiled_shape=np.array([Mt, Nt, Kt], np.int32),
               c_tiled=orc.matmul_tiled(a_tiled, b_tiled, Mt, Nt, Kt, acc64=True),
               c_tiled_leaky=orc.matmul_tiled(a_tiled, b_tiled, Mt, Nt, Kt, leaky_relu=True, acc64=True))
    return out


def attention() -> dict:
    rng = np.random.default_rng(11)
    Z, H, N, D = 1, 2, 128, 64
    q, k, v = (orc.to_bf16(rng.standard_normal((Z, H, N, D)).astype(np.float32)) for _ in range(3))
    sm = 1.0 / math.sqrt(D)
    oc, mc = orc.attn_fwd(q, k, v, sm, causal=True, BLOCK_M=32, BLOCK_N=32)     # the reference's pytest config
    of, mf = orc.attn_fwd(q, k, v, sm, causal=False, BLOCK_M=32, BLOCK_N=32)
    return {"q": q, "k": k, "v": v, "sm_scale": np.array([sm], np.float32), "o_causal": oc, "m_causal": mc,
            "o_full": of, "m_full": mf}


def reductions() -> dict:
    rng = np.random.default_rng(5)
    out = {}
    for name, dt, npdt in (("i8", orc.I8, np.int8), ("u8", orc.U8, np.uint8), ("i16", orc.I16, np.int16),
                           ("i32", orc.I32, np.int32), ("u32", orc.U32, np.uint32), ("i64", orc.I64, np.int64)):
        info = np.iinfo(npdt)
        x = rng.integers(info.min, info.max, 512, dtype=npdt, endpoint=True)
        out[f"x_{name}"] = x
        narrow = np.dtype(npdt).itemsize < 4
        sum_acc = (orc.U32 if dt == orc.U8 else orc.I32) if narrow else dt
        mm_acc = orc.I32 if narrow else dt
        out[f"sum_{name}"] = np.array([orc.reduce1d(x, "sum", dt, acc_dt=sum_acc)])
        for op in ("min", "max"):
            out[f"{op}_{name}"] = np.array([orc.reduce1d(x, op, dt, acc_dt=mm_acc)])
        for op in ("argmin", "argmax", "xor_sum"):
            out[f"{op}_{name}"] = np.array([orc.reduce1d(x, op, dt)])
    xf = (rng.standard_normal(512) * 100).astype(np.float32)
    xf[100] = xf[7] = xf.max()                                  # a tie for argmax
    out["x_f32"] = xf
    for op in ("sum", "min", "max", "argmin", "argmax"):
        out[f"{op}_f32"] = np.array([orc.reduce1d(xf, op, orc.F32)])
    return out


FIXTURES = {"elementwise": elementwise, "matmul": matmul, "attention": attention, "reductions": reductions}

if __name__ == "__main__":
    for name, make in FIXTURES.items():
        data = make()
        np.savez_compressed(HERE / f"{name}.npz", **data)
        print(f"{name}.npz: {len(data)} arrays, {(HERE / f'{name}.npz').stat().st_size} bytes")
