"""The plugin surface under real Triton: target registration, option parsing, the stage pipeline
on the host (no GPU needed to compile: nothing is generated for the device), and -- on the GPU --
launching ``@triton.jit`` kernels through Triton's own JIT onto the prebuilt kernels."""
import json

import numpy as np
import pytest
import torch

triton = pytest.importorskip("triton")

import triton.language as tl  # noqa: E402
from triton.backends.compiler import GPUTarget  # noqa: E402

from triton_tenstorrent_amd.backend import compiler as ttc  # noqa: E402
from triton_tenstorrent_amd.backend import driver as ttd  # noqa: E402

TARGET = GPUTarget("tenstorrent", "gfx950", 64)


def test_backend_surface():
    assert ttc.TTBackend.supports_target(TARGET)
    assert not ttc.TTBackend.supports_target(GPUTarget("hip", "gfx950", 64))
    b = ttc.TTBackend(TARGET)
    assert b.get_target_name(None) == "tenstorrent" and b.binary_ext == ttd.BINARY_EXT
    o = b.parse_options({"num_warps": 8, "bogus": 1, "num_stages": None})
    assert (o.num_warps, o.num_stages, o.arch, o.allowed_dot_input_precisions) == (8, 1, "gfx950", ("ieee", ))
    assert len(o.hash()) == 64 and o.hash() != b.parse_options({}).hash()
    md = type("M", (), dict(num_warps=4, num_ctas=1, shared=0, cluster_dims=(1, 1, 1)))
    assert b.pack_metadata(md) == (4, 1, 0, 1, 1, 1)
    assert b.get_codegen_implementation(o)["min_dot_size"](None, None) == (1, 1, 1)
    assert ["tt.divisibility", 8] in ttc.TTBackend.parse_attr("D")     # the reference's 8, not upstream's 16
    assert b.hash() == "0.1-gfx950"
    stages = {}
    b.add_stages(stages, o, triton.backends.compiler.Language.TRITON)
    assert list(stages) == ["ttir", ttd.BINARY_EXT]
    with pytest.raises(NotImplementedError):
        b.add_stages({}, o, triton.backends.compiler.Language.GLUON)
    with pytest.raises(ValueError):
        b.add_stages({}, b.parse_options({"ttmlir_target": "d2m"}), triton.backends.compiler.Language.TRITON)
    # every field the Triton front end reads from a backend's options exists
    for f in ("supported_fp8_dtypes", "deprecated_fp8_dot_operand_dtypes", "default_dot_input_precision",
              "max_num_imprecise_acc_default", "launch_cooperative_grid", "extern_libs", "sanitize_overflow",
              "enable_fp_fusion", "num_ctas", "num_stages", "num_warps", "debug", "arch"):
        assert hasattr(o, f)


def _compile(fn, signature, constexprs):
    from triton.backends import Backend, backends
    from triton.compiler import ASTSource
    backends["tenstorrent"] = Backend(compiler=ttc.TTBackend, driver=ttd.TTDriver)
    try:
        src = ASTSource(fn=fn, signature=signature, constexprs=constexprs)
        return triton.compile(src, target=TARGET)
    finally:
        backends.pop("tenstorrent", None)


def test_compile_on_host_binds_by_name(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton_tenstorrent_amd.examples import triton_kernels as tk
    k = _compile(tk.add_kernel, {"x_ptr": "*fp32", "y_ptr": "*fp32", "output_ptr": "*fp32", "n_elements": "i32",
                                 "BLOCK_SIZE": "constexpr"}, {"BLOCK_SIZE": 1024})
    assert k.name == "add_kernel" and k.metadata.shared == 0
    assert json.loads(k.kernel)["kernel"] == "add_kernel"
    assert "tt.func public @add_kernel" in k.asm["ttir"]
    assert k.packed_metadata[:3] == (4, 1, 0)

    # the pointer-based matmul_kernel: its unit strides are constexprs, as Triton's specialiser makes them
    sig = {"a_ptr": "*fp16", "b_ptr": "*fp16", "c_ptr": "*fp16", "M": "i32", "N": "i32", "K": "i32", "stride_am": "i32",
           "stride_ak": "constexpr", "stride_bk": "i32", "stride_bn": "constexpr", "stride_cm": "i32",
           "stride_cn": "constexpr", "BLOCK_SIZE_M": "constexpr", "BLOCK_SIZE_N": "constexpr",
           "BLOCK_SIZE_K": "constexpr", "GROUP_SIZE_M": "constexpr", "ACTIVATION": "constexpr"}
    k = _compile(tk.matmul_kernel, sig, {"stride_ak": 1, "stride_bn": 1, "stride_cn": 1, "BLOCK_SIZE_M": 32,
                                         "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 1,
                                         "ACTIVATION": "leaky_relu"})
    assert k.name == "matmul_kernel" and "tt.dot" in k.asm["ttir"]

    @triton.jit
    def unknown_kernel(x_ptr, n):
        tl_pid = triton.language.program_id(0)
        triton.language.store(x_ptr + tl_pid, n)

    with pytest.raises(Exception, match="no prebuilt gfx950 implementation"):
        _compile(unknown_kernel, {"x_ptr": "*i32", "n": "i32"}, {})


@pytest.mark.gpu
def test_triton_jit_launches_prebuilt_kernels(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton.tools.tensor_descriptor import TensorDescriptor
    from oracle import oracle as orc
    from triton_tenstorrent_amd import runtime as rt
    from triton_tenstorrent_amd.examples import triton_kernels as tk
    ttc.register()
    try:
        n = 98432
        x, y = torch.rand(n, device="cuda"), torch.rand(n, device="cuda")
        out = torch.empty_like(x)
        tk.add_kernel[lambda meta: (triton.cdiv(n, meta["BLOCK_SIZE"]), )](x, y, out, n, BLOCK_SIZE=1024)
        assert rt.last_kernel_name() == "ew_add_f32"
        assert np.array_equal(out.cpu().numpy().view(np.uint32), orc.add(x.cpu().numpy(), y.cpu().numpy()).view(np.uint32))
        s = torch.empty_like(x)
        tk.sin_kernel[(triton.cdiv(n, 1024), )](x, s, n, BLOCK_SIZE=1024)
        assert np.max(np.abs(s.cpu().numpy() - orc.sin(x.cpu().numpy()))) <= 2e-6
        M = N = Kd = 512
        a = (torch.randn(M, Kd, device="cuda") / 16).to(torch.bfloat16)
        b = torch.randn(Kd, N, device="cuda").to(torch.bfloat16)
        c = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        ad, bd, cd = (TensorDescriptor.from_tensor(a, [128, 64]), TensorDescriptor.from_tensor(b, [64, 128]),
                      TensorDescriptor.from_tensor(c, [128, 128]))
        tk.matmul_kernel_tma[(16, )](ad, bd, cd, M, N, Kd, BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64,
                                     GROUP_SIZE_M=8, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
        assert rt.last_kernel_name().startswith("gemm_tile_bf16")
        ref = (a.double() @ b.double()).float()
        assert torch.all((c.float() - ref).abs() <= 1e-2 * ref.abs() + 1e-4)
        # the pointer-based kernel on tile-major fp16 buffers; its unit strides reach the launcher as constexprs
        from triton_tenstorrent_amd import kernels as K
        M, N, Kd = 256, 512, 128
        ah = (torch.rand(M, Kd, device="cuda") - 0.5).to(torch.float16)
        bh = (torch.rand(Kd, N, device="cuda") - 0.5).to(torch.float16)
        ct = torch.empty(M * N, device="cuda", dtype=torch.float16)
        tk.matmul_kernel[(M // 32 * (N // 32), )](K.tilize(ah, 32, 32), K.tilize(bh, 32, 32), ct, M, N, Kd, Kd, 1, N, 1,
                                                  N, 1, BLOCK_SIZE_M=32, BLOCK_SIZE_N=32, BLOCK_SIZE_K=32,
                                                  GROUP_SIZE_M=1, ACTIVATION="leaky_relu")
        assert rt.last_kernel_name() == "gemm_tiled_f16_epi3"
        ref = ah.double() @ bh.double()
        ref = torch.where(ref >= 0, ref, 0.01 * ref).float()
        assert torch.all((K.untilize(ct, M, N, 32, 32).float() - ref).abs() <= 1e-2 * ref.abs() + 1e-4)
        # do_bench drives the device interface of the active driver
        ms = triton.testing.do_bench(lambda: tk.add_kernel[(97, )](x, y, out, n, BLOCK_SIZE=1024), warmup=5, rep=20)
        assert 0 < ms < 10
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None  # back to the stock driver, lazily


# ---- kernels bound by the shape of their IR ---------------------------------------------------------
@triton.jit
def user_exp2(src_ptr, dst_ptr, count, BLOCK_SIZE: tl.constexpr):
    pid = tl.program_id(axis=0)
    offsets = pid * BLOCK_SIZE + tl.arange(0, BLOCK_SIZE)
    mask = offsets < count
    tl.store(dst_ptr + offsets, tl.exp2(tl.load(src_ptr + offsets, mask=mask)), mask=mask)


@triton.jit
def user_sub_swapped(out_ptr, a_ptr, b_ptr, n, BLOCK: tl.constexpr):
    # output first, and the second tensor is the minuend: operand order must come from the IR, not the signature
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(out_ptr + offs, tl.load(b_ptr + offs, mask=m) - tl.load(a_ptr + offs, mask=m), mask=m)


@triton.jit
def user_to_bf16(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(y_ptr + offs, tl.load(x_ptr + offs, mask=m).to(tl.bfloat16), mask=m)


@triton.jit
def user_fma(o_ptr, p_ptr, q_ptr, r_ptr, n, BLOCK: tl.constexpr):
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(o_ptr + offs, tl.load(r_ptr + offs, mask=m) + tl.load(p_ptr + offs, mask=m) * tl.load(q_ptr + offs, mask=m), mask=m)


@triton.jit
def user_iadd(a_ptr, b_ptr, c_ptr, n, BLOCK: tl.constexpr):
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(c_ptr + offs, tl.load(a_ptr + offs, mask=m) + tl.load(b_ptr + offs, mask=m), mask=m)


@triton.jit
def user_two_ops(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(y_ptr + offs, tl.exp(tl.sqrt(tl.load(x_ptr + offs, mask=m))), mask=m)


@triton.jit
def user_strided(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(y_ptr + offs, tl.exp(tl.load(x_ptr + 2 * offs, mask=m)), mask=m)


def test_elementwise_kernels_are_recognised_by_shape(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    f32 = "*fp32"
    k = _compile(user_exp2, {"src_ptr": f32, "dst_ptr": f32, "count": "i32", "BLOCK_SIZE": "constexpr"}, {"BLOCK_SIZE": 512})
    rec = json.loads(k.kernel)
    assert k.name == "user_exp2" and rec["kernel"] == "unary_kernel"
    assert rec["match"] == {"kernel": "unary_kernel", "op": "exp2", "inputs": ["src_ptr"], "output": "dst_ptr",
                            "n": "count", "n_const": None, "block": 512}
    k = _compile(user_sub_swapped, {"out_ptr": f32, "a_ptr": f32, "b_ptr": f32, "n": "i32", "BLOCK": "constexpr"},
                 {"BLOCK": 1024})
    m = json.loads(k.kernel)["match"]
    assert (m["kernel"], m["op"], m["inputs"], m["output"]) == ("binary_kernel", "sub", ["b_ptr", "a_ptr"], "out_ptr")
    k = _compile(user_to_bf16, {"x_ptr": f32, "y_ptr": "*bf16", "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 1024})
    assert json.loads(k.kernel)["match"]["kernel"] == "cast_kernel"
    k = _compile(user_fma, {"o_ptr": f32, "p_ptr": f32, "q_ptr": f32, "r_ptr": f32, "n": "i32", "BLOCK": "constexpr"},
                 {"BLOCK": 1024})
    m = json.loads(k.kernel)["match"]
    assert m["kernel"] == "muladd_kernel" and sorted(m["inputs"][:2]) == ["p_ptr", "q_ptr"] and m["inputs"][2] == "r_ptr"
    k = _compile(user_iadd, {"a_ptr": "*i32", "b_ptr": "*i32", "c_ptr": "*i32", "n": "i32", "BLOCK": "constexpr"},
                 {"BLOCK": 1024})
    m = json.loads(k.kernel)["match"]
    assert (m["kernel"], m["op"], m["inputs"], m["output"]) == ("add_kernel", "i32", ["a_ptr", "b_ptr"], "c_ptr")
    # not of the form: two operations, or addressing other than base + offsets
    for fn in (user_two_ops, user_strided):
        with pytest.raises(Exception, match="no prebuilt gfx950 implementation"):
            _compile(fn, {"x_ptr": f32, "y_ptr": f32, "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 1024})
    # wrong element type for the operation set
    with pytest.raises(Exception, match="no prebuilt gfx950 implementation"):
        _compile(user_sub_swapped, {"out_ptr": "*fp16", "a_ptr": "*fp16", "b_ptr": "*fp16", "n": "i32",
                                    "BLOCK": "constexpr"}, {"BLOCK": 1024})


@pytest.mark.gpu
def test_shape_matched_kernels_run(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from oracle import oracle as orc
    from triton_tenstorrent_amd import runtime as rt
    ttc.register()
    try:
        n = 70001
        a = torch.randn(n, device="cuda") * 3
        b = torch.randn(n, device="cuda")
        out = torch.full((n + 5, ), -7.0, device="cuda")
        user_exp2[(triton.cdiv(n, 512), )](a, out, n, BLOCK_SIZE=512)
        assert rt.last_kernel_name() == "ew_exp2_f32"
        want = orc.unary("exp2", a.cpu().numpy())
        got = out[:n].cpu().numpy()
        assert np.all(np.abs(got.astype(np.float64) - want) <= 2 * np.spacing(np.abs(want))) and torch.all(out[n:] == -7.0)
        user_sub_swapped[(triton.cdiv(n, 1024), )](out, a, b, n, BLOCK=1024)
        assert torch.equal(out[:n], b - a)
        c = torch.randn(n, device="cuda")
        user_fma[(triton.cdiv(n, 1024), )](out, a, b, c, n, BLOCK=1024)
        assert rt.last_kernel_name() == "ew_muladd_f32"
        assert torch.equal(out[:n].cpu(), torch.from_numpy(np.float32(np.float64(a.cpu().numpy()) * np.float64(b.cpu().numpy())
                                                                       + np.float64(c.cpu().numpy()))))
        ia = torch.randint(-2**31, 2**31 - 1, (n, ), device="cuda", dtype=torch.int64).to(torch.int32)
        ic = torch.empty_like(ia)
        user_iadd[(triton.cdiv(n, 1024), )](ia, ia, ic, n, BLOCK=1024)
        assert rt.last_kernel_name() == "ew_add_i32" and torch.equal(ic, ia + ia)
        h = torch.empty(n, device="cuda", dtype=torch.bfloat16)
        user_to_bf16[(triton.cdiv(n, 1024), )](a, h, n, BLOCK=1024)
        assert rt.last_kernel_name() == "ew_cast_f32_bf16" and torch.equal(h, a.to(torch.bfloat16))
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None


# --- the single-block reductions of test_core.py::test_reduce1d (the reference's CI: integration-tests-cpu.yml:105) ---
def _reduce_kernel(expr: str):
    """The test's kernel with its GENERATE_TEST_HERE line filled in, as the test does by patching the source."""
    src = ("import triton\nimport triton.language as tl\n\n@triton.jit\ndef kernel(X, Z, BLOCK: tl.constexpr):\n"
           "    x = tl.load(X + tl.arange(0, BLOCK))\n" f"    {expr}\n" "    tl.store(Z, z)\n")
    import importlib.util, tempfile, hashlib, os
    path = os.path.join(tempfile.gettempdir(), f"ttamd_reduce_{hashlib.sha1(expr.encode()).hexdigest()[:12]}.py")
    with open(path, "w") as f:
        f.write(src)
    spec = importlib.util.spec_from_file_location(os.path.basename(path)[:-3], path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.kernel


REDUCE_FORMS = {
    "sum": "z = tl.sum(x, axis=0)",
    "min": "z = tl.min(x, axis=0)",
    "max": "z = tl.max(x, axis=0)",
    "min-with-indices": "z, _ = tl.min(x, axis=0, return_indices=True)",
    "max-with-indices": "z, _ = tl.max(x, axis=0, return_indices=True)",
    "argmin-tie-break-left": "z = tl.argmin(x, axis=0, tie_break_left=True)",
    "argmax-tie-break-left": "z = tl.argmax(x, axis=0, tie_break_left=True)",
    "xor_sum": "z = tl.xor_sum(x, axis=0)",
}


def test_reductions_are_recognised_by_shape(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton_tenstorrent_amd import runtime as rt

    def match(form, x, z, block=512):
        k = _compile(_reduce_kernel(REDUCE_FORMS[form]), {"X": x, "Z": z, "BLOCK": "constexpr"}, {"BLOCK": block})
        rec = json.loads(k.kernel)
        assert k.name == "kernel" and rec["kernel"] == "reduce1d_kernel"
        m = rec["match"]
        assert (m["inputs"], m["output"], m["block"]) == (["X"], "Z", block)
        return m["op"], m["in_dtype"], m["acc_dtype"], m["out_dtype"], m["tie_break_left"]

    assert match("sum", "*fp32", "*fp32") == ("sum", rt.TT_F32, rt.TT_F32, rt.TT_F32, False)
    assert match("sum", "*i8", "*i32", 32) == ("sum", rt.TT_I8, rt.TT_I32, rt.TT_I32, False)        # narrow sums run in i32
    assert match("sum", "*u16", "*u32") == ("sum", rt.TT_U16, rt.TT_I32, rt.TT_U32, False)      # zero-extended
    assert match("sum", "*bf16", "*bf16") == ("sum", rt.TT_BF16, rt.TT_BF16, rt.TT_BF16, False)
    assert match("max", "*bf16", "*fp32") == ("max", rt.TT_BF16, rt.TT_F32, rt.TT_F32, False)       # promoted to fp32
    assert match("max", "*u8", "*u8") == ("max", rt.TT_U8, rt.TT_I32, rt.TT_U8, False)          # extui, maxsi, trunci
    assert match("min", "*u32", "*u32") == ("min", rt.TT_U32, rt.TT_U32, rt.TT_U32, False)      # minui
    assert match("min", "*i64", "*i64") == ("min", rt.TT_I64, rt.TT_I64, rt.TT_I64, False)
    assert match("max", "*fp64", "*fp64") == ("max", rt.TT_F64, rt.TT_F64, rt.TT_F64, False)
    assert match("min-with-indices", "*fp32", "*fp32") == ("min", rt.TT_F32, rt.TT_F32, rt.TT_F32, True)
    assert match("max-with-indices", "*i32", "*i32") == ("max", rt.TT_I32, rt.TT_I32, rt.TT_I32, True)
    assert match("argmin-tie-break-left", "*fp32", "*i32") == ("argmin", rt.TT_F32, rt.TT_F32, rt.TT_I32, True)
    assert match("argmax-tie-break-left", "*i16", "*i32", 128)[0:2] == ("argmax", rt.TT_I16)
    assert match("xor_sum", "*i32", "*i32") == ("xor_sum", rt.TT_I32, rt.TT_I32, rt.TT_I32, False)
    # a reduction outside the set stays a compile error
    with pytest.raises(Exception, match="no prebuilt gfx950 implementation"):
        _compile(_reduce_kernel("z = tl.sum(x * x, axis=0)"), {"X": "*fp32", "Z": "*fp32", "BLOCK": "constexpr"}, {"BLOCK": 64})


@pytest.mark.gpu
def test_reductions_run_through_triton(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from oracle import oracle as orc
    from triton_tenstorrent_amd import runtime as rt
    ttc.register()
    try:
        rng = np.random.default_rng(3)
        for form, np_dt, dt, shape in (("sum", np.int8, orc.I8, 512), ("max", np.uint8, orc.U8, 64),
                                       ("argmin-tie-break-left", np.int32, orc.I32, 128), ("xor_sum", np.int32, orc.I32, 32),
                                       ("min-with-indices", np.int16, orc.I16, 512)):
            info = np.iinfo(np_dt)
            x = rng.integers(info.min, info.max, shape, dtype=np_dt, endpoint=True)
            op = form.split("-")[0]
            narrow_sum = op == "sum" and np.dtype(np_dt).itemsize < 4
            z_dt = torch.int32 if (op.startswith("arg") or narrow_sum) else torch.from_numpy(x).dtype
            z = torch.zeros(1, device="cuda", dtype=z_dt)
            _reduce_kernel(REDUCE_FORMS[form])[(1, )](torch.from_numpy(x).cuda(), z, BLOCK=shape)
            assert rt.last_kernel_name().startswith("reduce1d_")
            want = {"sum": lambda: x.astype(np.int64).sum(), "max": x.max, "min": x.min, "argmin": lambda: np.argmin(x),
                    "xor_sum": lambda: np.bitwise_xor.reduce(x)}[op]()
            assert int(z.cpu()[0]) == int(want), (form, np_dt)
        xf = (rng.standard_normal(512) * 10).astype(np.float32)
        z = torch.zeros(1, device="cuda")
        _reduce_kernel(REDUCE_FORMS["sum"])[(1, )](torch.from_numpy(xf).cuda(), z, BLOCK=512)
        np.testing.assert_allclose(float(z.cpu()[0]), float(np.sum(xf.astype(np.float64))), rtol=1e-5, atol=1e-3)
        _reduce_kernel(REDUCE_FORMS["max"])[(1, )](torch.from_numpy(xf).cuda().to(torch.bfloat16), z, BLOCK=512)
        assert float(z.cpu()[0]) == float(torch.from_numpy(xf).to(torch.bfloat16).float().max())
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None


def test_offline_compile_tool_accepts_the_tenstorrent_target(tmp_path, monkeypatch):
    """README.md:74-77 of the reference: `compile.py --target tenstorrent:0:1 --signature "*fp32,*fp32,*fp32,i32,1024"
    --grid 1,1,1 -n add_kernel <source>` prints nothing and leaves its artefacts in the Triton cache."""
    import sys
    import triton.tools.compile as aot
    from triton_tenstorrent_amd.examples import triton_kernels as tk
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path / "cache"))
    monkeypatch.setattr(sys, "argv", ["compile.py", "--target", "tenstorrent:0:1", "--signature", "*fp32,*fp32,*fp32,i32,1024",
                                      "--grid", "1,1,1", "-n", "add_kernel", "-o", str(tmp_path / "out"), tk.__file__])
    ttc.register()
    try:
        aot.main()
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None
    made = {p.name for p in (tmp_path / "cache").rglob("add_kernel.*")}
    assert {"add_kernel.ttir", "add_kernel.ttamd", "add_kernel.json"} <= made
    record = json.loads(next((tmp_path / "cache").rglob("add_kernel.ttamd")).read_text())
    assert record["kernel"] == "add_kernel" and record["arch"] == "gfx950"


# --- a constant operand, and the one-element-per-program form of test_core.py::test_load_store_same_ptr ---
@triton.jit
def kernel_same_ptr(in_out_ptr):
    pid = tl.program_id(axis=0)
    x = tl.load(in_out_ptr + pid)
    out = x * 2
    tl.store(in_out_ptr + pid, out)


@triton.jit
def user_rsub_const(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    pid = tl.program_id(axis=0)
    offs = pid * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    tl.store(y_ptr + offs, 3.5 - tl.load(x_ptr + offs, mask=m), mask=m)


def test_constant_operand_forms_are_recognised(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    m = json.loads(_compile(kernel_same_ptr, {"in_out_ptr": "*fp32"}, {}).kernel)["match"]
    assert m == {"kernel": "binary_const_kernel", "op": "mul", "inputs": ["in_out_ptr"], "output": "in_out_ptr", "n": None,
                 "n_const": None, "block": 1, "c": 2.0, "flip": False}
    m = json.loads(_compile(user_rsub_const, {"x_ptr": "*fp32", "y_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"},
                            {"BLOCK": 1024}).kernel)["match"]
    assert (m["kernel"], m["op"], m["inputs"], m["output"], m["n"], m["block"], m["c"], m["flip"]) == \
        ("binary_const_kernel", "sub", ["x_ptr"], "y_ptr", "n", 1024, 3.5, True)


@pytest.mark.gpu
def test_load_store_same_ptr_runs(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton_tenstorrent_amd import runtime as rt
    ttc.register()
    try:
        for _ in range(20):                                  # the upstream test repeats the launch 1000 times
            x = torch.ones((65536, ), device="cuda", dtype=torch.float32)
            kernel_same_ptr[(65536, )](x, num_warps=16)
            assert torch.all(x == 2)
        assert rt.last_kernel_name() == "ew_mulc_f32"
        x = torch.ones(100, device="cuda")
        kernel_same_ptr[(40, )](x)                           # 40 programs touch 40 elements
        assert torch.all(x[:40] == 2) and torch.all(x[40:] == 1)
        a = torch.randn(70001, device="cuda")
        y = torch.full((70001 + 3, ), -7.0, device="cuda")
        user_rsub_const[(triton.cdiv(70001, 1024), )](a, y, 70001, BLOCK=1024)
        assert rt.last_kernel_name() == "ew_subc_f32" and torch.equal(y[:70001], 3.5 - a) and torch.all(y[70001:] == -7.0)
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None


# --- the kernels of test_launch.py, which the reference's CI runs on its cpu/ path
# (.github/workflows/integration-tests-cpu.yml:106): an empty kernel under the launch hooks and a masked copy whose
# bound is a constant of the kernel, launched in a loop under tracemalloc ---
@triton.jit
def copy_first_ten(src_ptr, dst_ptr, count, BLOCK: tl.constexpr):
    count = 10
    idx = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    keep = idx < count
    v = tl.load(src_ptr + idx, keep)
    tl.store(dst_ptr + (idx + tl.zeros([BLOCK], tl.int32)), v, keep)


@triton.jit
def user_copy(src_ptr, dst_ptr, n, BLOCK: tl.constexpr):
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    tl.store(dst_ptr + offs, tl.load(src_ptr + offs, mask=offs < n), mask=offs < n)


def _describe_launch(grid, kernel, args):
    return {"grid": grid, "value": args["x"]}


@triton.jit(launch_metadata=_describe_launch)
def does_nothing(x):
    pass


def test_copy_and_empty_kernels_are_recognised(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    m = json.loads(_compile(copy_first_ten, {"src_ptr": "*fp32", "dst_ptr": "*fp32", "count": "i32", "BLOCK": "constexpr"},
                            {"BLOCK": 16}).kernel)["match"]
    assert m == {"kernel": "copy_kernel", "op": None, "inputs": ["src_ptr"], "output": "dst_ptr", "n": None, "n_const": 10,
                 "block": 16, "dtype": 0}
    for ty, code in (("*i8", 6), ("*u8", 6), ("*bf16", 2), ("*i64", 7), ("*fp64", 8), ("*u16", 5)):
        m = json.loads(_compile(user_copy, {"src_ptr": ty, "dst_ptr": ty, "n": "i32", "BLOCK": "constexpr"},
                                {"BLOCK": 256}).kernel)["match"]
        assert (m["kernel"], m["n"], m["block"], m["dtype"]) == ("copy_kernel", "n", 256, code), ty
    k = _compile(does_nothing, {"x": "i32"}, {})
    assert json.loads(k.kernel)["match"] == {"kernel": "empty_kernel"}

    @triton.jit
    def copy_between_types(src_ptr, dst_ptr, n, BLOCK: tl.constexpr):     # the store widens: neither a copy nor a narrowing cast
        offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
        tl.store(dst_ptr + offs, tl.load(src_ptr + offs, mask=offs < n), mask=offs < n)

    with pytest.raises(RuntimeError, match="no prebuilt gfx950 implementation"):
        _compile(copy_between_types, {"src_ptr": "*fp16", "dst_ptr": "*fp32", "n": "i32", "BLOCK": "constexpr"}, {"BLOCK": 256})


@pytest.mark.gpu
def test_launch_hooks_and_no_leak_through_the_jit(tmp_path, monkeypatch):
    import gc
    import tracemalloc
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton_tenstorrent_amd import runtime as rt
    ttc.register()
    seen = []

    def first(launch_metadata):
        md = launch_metadata.get()
        assert md["grid"] == (1, 3, 2) and md["value"] == 6
        seen.append("first")

    def second(launch_metadata):
        seen.append("second")

    def after(launch_metadata):
        seen.append("after")

    def load_start(module, function, name, metadata_group, hash):
        seen.append(("load start", name, repr(function)))

    def load_end(module, function, name, metadata_group, hash):
        seen.append(("load end", name))

    try:
        triton.knobs.runtime.launch_enter_hook.add(first)
        triton.knobs.runtime.launch_enter_hook.add(second)
        triton.knobs.runtime.launch_exit_hook.add(after)
        triton.knobs.runtime.kernel_load_start_hook.add(load_start)
        triton.knobs.runtime.kernel_load_end_hook.add(load_end)
        try:
            does_nothing[(1, 3, 2)](6)
        finally:
            triton.knobs.runtime.launch_enter_hook.remove(first)
            triton.knobs.runtime.launch_enter_hook.remove(second)
            triton.knobs.runtime.launch_exit_hook.remove(after)
            triton.knobs.runtime.kernel_load_start_hook.remove(load_start)
            triton.knobs.runtime.kernel_load_end_hook.remove(load_end)
        # the load hooks bracket load_binary on the first launch (test_launch.py::test_load_hook), then the launch hooks
        assert seen[0][:2] == ("load start", "does_nothing") and seen[1] == ("load end", "does_nothing")
        assert "BoundKernel empty_kernel" in repr(seen[0][2]) or seen[0][2] == "None"
        del seen[:2]
        assert seen == ["first", "second", "after"]
        does_nothing[(1, 3, 2)](6)
        assert seen == ["first", "second", "after"]                    # removed hooks stay removed

        inp, out = torch.randn(10, device="cuda"), torch.randn(10, device="cuda")
        tracemalloc.start()
        try:
            copy_first_ten[(10, )](inp, out, 10, BLOCK=16)
            gc.collect()
            begin, _ = tracemalloc.get_traced_memory()
            for _ in range(100):
                copy_first_ten[(10, )](inp, out, 10, BLOCK=16)
            gc.collect()
            end, _ = tracemalloc.get_traced_memory()
        finally:
            tracemalloc.stop()
        assert end - begin < 30000                                     # the upstream test's bound
        assert torch.equal(out, inp) and rt.last_kernel_name() == "ew_copy_b128"

        # the bound is the kernel's constant, not the argument: 10 of 64 elements move
        src = torch.arange(64, device="cuda", dtype=torch.int16)
        dst = torch.full((64, ), -1, device="cuda", dtype=torch.int16)
        copy_first_ten[(4, )](src, dst, 64, BLOCK=16)
        assert torch.equal(dst[:10], src[:10]) and torch.all(dst[10:] == -1)
        with pytest.raises(Exception, match="holds fewer"):
            copy_first_ten[(1, )](src[:4], dst, 64, BLOCK=16)

        big = torch.randint(-2**62, 2**62, (70001, ), device="cuda", dtype=torch.int64)
        got = torch.zeros(70001 + 5, device="cuda", dtype=torch.int64)
        user_copy[(triton.cdiv(70001, 512), )](big, got, 70001, BLOCK=512)
        assert torch.equal(got[:70001], big) and not got[70001:].any()
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None


# --- autotune and do_bench through the plugin's device interface (driver.py:390-442 of the reference) ---
@triton.autotune(configs=[triton.Config({"BLOCK_SIZE": 512}), triton.Config({"BLOCK_SIZE": 1024}),
                          triton.Config({"BLOCK_SIZE": 2048})], key=["n_elements"])
@triton.jit
def add_kernel_autotuned(x_ptr, y_ptr, output_ptr, n_elements, BLOCK_SIZE: tl.constexpr):
    pid = tl.program_id(axis=0)
    block_start = pid * BLOCK_SIZE
    offsets = block_start + tl.arange(0, BLOCK_SIZE)
    mask = offsets < n_elements
    x = tl.load(x_ptr + offsets, mask=mask)
    y = tl.load(y_ptr + offsets, mask=mask)
    tl.store(output_ptr + offsets, x + y, mask=mask)


@pytest.mark.gpu
def test_autotune_and_do_bench_through_the_plugin(tmp_path, monkeypatch):
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton_tenstorrent_amd import runtime as rt
    ttc.register()
    try:
        n = 1 << 22
        x, y = torch.rand(n, device="cuda"), torch.rand(n, device="cuda")
        out = torch.empty_like(x)
        grid = lambda meta: (triton.cdiv(n, meta["BLOCK_SIZE"]), )
        add_kernel_autotuned[grid](x, y, out, n)             # times the three configurations with the driver's benchmarker
        assert torch.equal(out, x + y) and rt.last_kernel_name() == "ew_add_f32"
        assert add_kernel_autotuned.best_config.kwargs["BLOCK_SIZE"] in (512, 1024, 2048)
        assert len(add_kernel_autotuned.cache) == 1
        # do_bench drives Event / synchronize / the cache-clearing buffer of the device interface
        ms = triton.testing.do_bench(lambda: add_kernel_autotuned[grid](x, y, out, n), warmup=5, rep=20)
        assert 0.0 < ms < 5.0, ms                                             # 48 MiB of traffic: a few tens of microseconds
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None


@pytest.mark.gpu
def test_triton_jit_launches_the_fused_matmul_muladd_and_attention(tmp_path, monkeypatch):
    """The remaining example kernels as @triton.jit sources through Triton's own JIT: descriptors, scalars and
    constexprs reach the launcher as Triton passes them."""
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton.tools.tensor_descriptor import TensorDescriptor
    from oracle import oracle as orc
    from triton_tenstorrent_amd import runtime as rt
    from triton_tenstorrent_amd.examples import triton_kernels as tk
    from util import bits
    ttc.register()
    try:
        n = 70001
        x, y, z = (torch.randn(n, device="cuda") for _ in range(3))
        out = torch.empty_like(x)
        tk.muladd_kernel[(triton.cdiv(n, 1024), )](x, y, z, out, n, BLOCK_SIZE=1024)
        assert rt.last_kernel_name() == "ew_muladd_f32"
        want = orc.muladd(x.cpu().numpy(), y.cpu().numpy(), z.cpu().numpy())
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))
        # fused matmul: fp16, full bias added in fp16 after the cast
        M, N, Kd = 256, 384, 128
        a = (torch.randn(M, Kd, device="cuda") / 8).to(torch.float16)
        b = torch.randn(Kd, N, device="cuda").to(torch.float16)
        bias = torch.randn(M, N, device="cuda").to(torch.float16)
        c = torch.empty(M, N, device="cuda", dtype=torch.float16)
        descs = [TensorDescriptor.from_tensor(t, blk) for t, blk in ((a, [64, 64]), (b, [64, 64]), (c, [64, 64]), (bias, [64, 64]))]
        tk.matmul_kernel_fused[(M // 64 * (N // 64), )](*descs, M, N, Kd, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64,
                                                        GROUP_SIZE_M=1, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
        assert rt.last_kernel_name().startswith("gemm_") and rt.last_kernel_name().endswith("_epi1")
        c0 = (a.double() @ b.double()).to(torch.float16)
        assert torch.all((c.float() - (c0 + bias).float()).abs() <= 1e-2 * (c0 + bias).float().abs() + 2e-2)
        # attention, causal and not, through 2-D descriptors over [Z*H*N_CTX, D]
        Z, H, S, D = 1, 2, 256, 64
        q, k, v = (torch.randn(Z, H, S, D, device="cuda").to(torch.bfloat16) for _ in range(3))
        o = torch.empty_like(q)
        Mlse = torch.empty(Z, H, S, device="cuda", dtype=torch.float32)
        for causal in (True, False):
            dq, dk, dv, do = (TensorDescriptor(t, shape=[Z * H * S, D], strides=[D, 1], block_shape=blk)
                              for t, blk in ((q, [64, D]), (k, [64, D]), (v, [64, D]), (o, [64, D])))
            tk._attn_fwd[(S // 64, Z * H, 1)](0.125, Mlse, Z, H, dq, dk, dv, do, S, HEAD_DIM=D, BLOCK_M=64, BLOCK_N=64,
                                              FP8_OUTPUT=False, STAGE=3 if causal else 1, warp_specialize=False,
                                              IS_HOPPER=False)
            assert rt.last_kernel_name() == "attn_tile_d64"
            wo, wM = orc.attn_fwd(bits(q), bits(k), bits(v), 0.125, causal=causal, BLOCK_M=64, BLOCK_N=64)
            assert np.max(np.abs(o.float().cpu().numpy() - orc.from_bf16(wo))) <= 2e-2
            assert np.max(np.abs(Mlse.cpu().numpy() - wM)) <= 1e-3
    finally:
        from triton.backends import backends
        backends.pop("tenstorrent", None)
        triton.runtime.driver._active = None


def test_installed_but_not_asked_for_the_driver_stays_passive(monkeypatch):
    """An installed package reaches Triton through its entry point whether or not anyone wants it, and Triton refuses
    to start with two active drivers (triton/runtime/driver.py:6-10).  Without register() / activate() or
    TRITON_TENSTORRENT_AMD=1 the driver therefore reports itself inactive, as the reference's does where its
    runtime is missing (backend/driver.py:449-467)."""
    from triton_tenstorrent_amd.backend import driver as drv
    monkeypatch.delenv("TRITON_TENSTORRENT_AMD", raising=False)
    monkeypatch.setattr(drv, "_OPTED_IN", False)
    assert drv.TTDriver.is_active() is False
    monkeypatch.setattr(drv.rt, "LIB_PATH", drv.rt.LIB_PATH.parent / "missing.so")
    monkeypatch.setenv("TRITON_TENSTORRENT_AMD", "1")
    assert drv.TTDriver.is_active() is False      # asked for, but nothing to run on


@pytest.mark.gpu
def test_entry_point_coexists_with_the_stock_driver(tmp_path, monkeypatch):
    """Both backends in Triton's table, as after `pip install`: driver selection must not raise, must pick the stock
    HIP driver while nobody asked for this one, and register() must still route add_kernel to ew_add_f32."""
    import importlib
    trd = importlib.import_module("triton.runtime.driver")    # the module (the package attribute of that name is its DriverConfig)
    from triton.backends import Backend, backends
    from triton_tenstorrent_amd import runtime as rt
    from triton_tenstorrent_amd.backend import driver as drv
    from triton_tenstorrent_amd.examples import triton_kernels as tk
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("TRITON_TENSTORRENT_AMD", raising=False)
    monkeypatch.setattr(drv, "_OPTED_IN", False)
    backends["tenstorrent"] = Backend(compiler=ttc.TTBackend, driver=drv.TTDriver)
    try:
        assert "amd" in backends and backends["amd"].driver.is_active()
        picked = trd._create_driver()                         # raises "2 active drivers" if both answer true
        assert type(picked).__name__ != "TTDriver"
        monkeypatch.setenv("TRITON_TENSTORRENT_AMD", "1")
        with pytest.raises(RuntimeError, match="active drivers"):
            trd._create_driver()                              # the opt-in is exclusive by Triton's own rule
        monkeypatch.delenv("TRITON_TENSTORRENT_AMD")
        ttc.register()
        n = 5000
        x, y = torch.rand(n, device="cuda"), torch.rand(n, device="cuda")
        out = torch.empty_like(x)
        tk.add_kernel[(triton.cdiv(n, 1024), )](x, y, out, n, BLOCK_SIZE=1024)
        assert rt.last_kernel_name() == "ew_add_f32" and torch.equal(out, x + y)
    finally:
        backends.pop("tenstorrent", None)
        triton.runtime.driver.reset_active()
        drv.opt_in(False)


def test_a_table_name_does_not_vouch_for_the_body(tmp_path, monkeypatch):
    """The reference generates code from the IR, so a kernel's name means nothing there.  Here a user kernel that
    merely carries the name of a prebuilt one (a `sin_kernel` that computes a cosine, an `add_kernel` that subtracts,
    upstream Triton's row-major `matmul_kernel`, which shares name and signature with the reference's tile-major
    one) must be a compile error, never a silent run of the prebuilt kernel."""
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    f32 = "*fp32"

    def one_op(name, expr, nin=1):
        ns = {"triton": triton, "tl": tl}
        ins = ", ".join(f"p{i}" for i in range(nin))
        loads = "\n".join(f"    v{i} = tl.load(p{i} + offs, mask=mask)" for i in range(nin))
        src = (f"@triton.jit\ndef {name}({ins}, out_ptr, n_elements, BLOCK_SIZE: tl.constexpr):\n"
               f"    pid = tl.program_id(axis=0)\n    offs = pid * BLOCK_SIZE + tl.arange(0, BLOCK_SIZE)\n"
               f"    mask = offs < n_elements\n{loads}\n    tl.store(out_ptr + offs, {expr}, mask=mask)\n")
        import linecache, hashlib
        fname = f"<wrong_body_{hashlib.md5(src.encode()).hexdigest()[:8]}>"
        linecache.cache[fname] = (len(src), None, src.splitlines(True), fname)
        exec(compile(src, fname, "exec"), ns)
        return ns[name]

    sig1 = {"p0": f32, "out_ptr": f32, "n_elements": "i32", "BLOCK_SIZE": "constexpr"}
    sig2 = {"p0": f32, "p1": f32, "out_ptr": f32, "n_elements": "i32", "BLOCK_SIZE": "constexpr"}
    with pytest.raises(Exception, match="does not match"):
        _compile(one_op("sin_kernel", "tl.cos(v0)"), sig1, {"BLOCK_SIZE": 1024})
    with pytest.raises(Exception, match="does not match"):
        _compile(one_op("add_kernel", "v0 - v1", 2), sig2, {"BLOCK_SIZE": 1024})
    with pytest.raises(Exception, match="does not match"):
        _compile(one_op("unary_kernel", "v0 * v1", 2), sig2, {"BLOCK_SIZE": 1024})
    # the right bodies under those names still bind
    assert json.loads(_compile(one_op("sin_kernel", "tl.sin(v0)"), sig1, {"BLOCK_SIZE": 1024}).kernel)["kernel"] == "sin_kernel"
    assert json.loads(_compile(one_op("add_kernel", "v0 + v1", 2), sig2, {"BLOCK_SIZE": 1024}).kernel)["kernel"] == "add_kernel"
    rec = json.loads(_compile(one_op("unary_kernel", "tl.exp(v0)"), sig1, {"BLOCK_SIZE": 1024}).kernel)
    assert rec["kernel"] == "unary_kernel" and rec["match"]["op"] == "exp"

    # upstream Triton's tutorial matmul: row-major, addressed through the strides
    @triton.jit
    def matmul_kernel(a_ptr, b_ptr, c_ptr, M, N, K, stride_am, stride_ak, stride_bk, stride_bn, stride_cm, stride_cn,
                      BLOCK_SIZE_M: tl.constexpr, BLOCK_SIZE_N: tl.constexpr, BLOCK_SIZE_K: tl.constexpr,
                      GROUP_SIZE_M: tl.constexpr, ACTIVATION: tl.constexpr):
        pid = tl.program_id(axis=0)
        num_pid_n = tl.cdiv(N, BLOCK_SIZE_N)
        pid_m = pid // num_pid_n
        pid_n = pid % num_pid_n
        offs_am = (pid_m * BLOCK_SIZE_M + tl.arange(0, BLOCK_SIZE_M)) % M
        offs_bn = (pid_n * BLOCK_SIZE_N + tl.arange(0, BLOCK_SIZE_N)) % N
        offs_k = tl.arange(0, BLOCK_SIZE_K)
        a_ptrs = a_ptr + (offs_am[:, None] * stride_am + offs_k[None, :] * stride_ak)
        b_ptrs = b_ptr + (offs_k[:, None] * stride_bk + offs_bn[None, :] * stride_bn)
        acc = tl.zeros((BLOCK_SIZE_M, BLOCK_SIZE_N), dtype=tl.float32)
        for k in range(0, tl.cdiv(K, BLOCK_SIZE_K)):
            a = tl.load(a_ptrs, mask=offs_k[None, :] < K - k * BLOCK_SIZE_K, other=0.0)
            b = tl.load(b_ptrs, mask=offs_k[:, None] < K - k * BLOCK_SIZE_K, other=0.0)
            acc = tl.dot(a, b, acc)
            a_ptrs += BLOCK_SIZE_K * stride_ak
            b_ptrs += BLOCK_SIZE_K * stride_bk
        c = acc.to(tl.float16)
        offs_cm = pid_m * BLOCK_SIZE_M + tl.arange(0, BLOCK_SIZE_M)
        offs_cn = pid_n * BLOCK_SIZE_N + tl.arange(0, BLOCK_SIZE_N)
        c_ptrs = c_ptr + stride_cm * offs_cm[:, None] + stride_cn * offs_cn[None, :]
        tl.store(c_ptrs, c, mask=(offs_cm[:, None] < M) & (offs_cn[None, :] < N))

    sig = {"a_ptr": "*fp16", "b_ptr": "*fp16", "c_ptr": "*fp16", "M": "i32", "N": "i32", "K": "i32", "stride_am": "i32",
           "stride_ak": "constexpr", "stride_bk": "i32", "stride_bn": "constexpr", "stride_cm": "i32",
           "stride_cn": "constexpr", "BLOCK_SIZE_M": "constexpr", "BLOCK_SIZE_N": "constexpr",
           "BLOCK_SIZE_K": "constexpr", "GROUP_SIZE_M": "constexpr", "ACTIVATION": "constexpr"}
    with pytest.raises(Exception, match="does not match"):
        _compile(matmul_kernel, sig, {"stride_ak": 1, "stride_bn": 1, "stride_cn": 1, "BLOCK_SIZE_M": 32, "BLOCK_SIZE_N": 32,
                                      "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 1, "ACTIVATION": ""})

    # upstream Triton's descriptor matmul (python/tutorials/09-persistent-matmul.py): same name and signature as
    # the reference's, but B is [N, K] and the product is A.B^T; the reference removed that transpose
    # (examples/matmul_tensor_descriptor/09-persistent-matmul.py:139), and with N == K the shapes would pass
    @triton.jit
    def matmul_kernel_tma(a_desc, b_desc, c_desc, M, N, K, BLOCK_SIZE_M: tl.constexpr, BLOCK_SIZE_N: tl.constexpr,
                          BLOCK_SIZE_K: tl.constexpr, GROUP_SIZE_M: tl.constexpr, FP8_OUTPUT: tl.constexpr,
                          WARP_SPECIALIZE: tl.constexpr):
        pid = tl.program_id(axis=0)
        num_pid_n = tl.cdiv(N, BLOCK_SIZE_N)
        pid_m = pid // num_pid_n
        pid_n = pid % num_pid_n
        acc = tl.zeros((BLOCK_SIZE_M, BLOCK_SIZE_N), dtype=tl.float32)
        for k in range(tl.cdiv(K, BLOCK_SIZE_K)):
            a = a_desc.load([pid_m * BLOCK_SIZE_M, k * BLOCK_SIZE_K])
            b = b_desc.load([pid_n * BLOCK_SIZE_N, k * BLOCK_SIZE_K])
            acc = tl.dot(a, b.T, acc)
        c_desc.store([pid_m * BLOCK_SIZE_M, pid_n * BLOCK_SIZE_N], acc.to(tl.bfloat16))

    tma_sig = {"a_desc": "tensordesc<bf16[128,64]>", "b_desc": "tensordesc<bf16[128,64]>", "c_desc": "tensordesc<bf16[128,128]>",
               "M": "i32", "N": "i32", "K": "i32", "BLOCK_SIZE_M": "constexpr", "BLOCK_SIZE_N": "constexpr",
               "BLOCK_SIZE_K": "constexpr", "GROUP_SIZE_M": "constexpr", "FP8_OUTPUT": "constexpr", "WARP_SPECIALIZE": "constexpr"}
    with pytest.raises(Exception, match="does not match"):
        _compile(matmul_kernel_tma, tma_sig, {"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 8,
                                              "FP8_OUTPUT": False, "WARP_SPECIALIZE": False})

    # a module named like the descriptor matmul whose body is something else
    from triton_tenstorrent_amd.backend.patterns import verify_named
    ttir_cos = _compile(one_op("cos_user", "tl.cos(v0)"), sig1, {"BLOCK_SIZE": 1024}).asm["ttir"]
    for table_name in ("matmul_kernel_tma", "matmul_kernel_fused", "matmul_kernel_tma_fp8_scaled", "_attn_fwd", "matmul_kernel"):
        with pytest.raises(RuntimeError, match="does not match"):
            verify_named(table_name, ttir_cos.replace("@cos_user", "@" + table_name))


def test_every_example_kernel_passes_the_check_of_its_own_name(tmp_path, monkeypatch):
    """The fingerprints that guard the prebuilt names must accept the kernels they are taken from, compiled by the
    real front end at the tilings the examples launch."""
    monkeypatch.setenv("TRITON_CACHE_DIR", str(tmp_path))
    from triton_tenstorrent_amd.examples import triton_kernels as tk
    mm = {"BLOCK_SIZE_M": "constexpr", "BLOCK_SIZE_N": "constexpr", "BLOCK_SIZE_K": "constexpr",
          "GROUP_SIZE_M": "constexpr", "FP8_OUTPUT": "constexpr", "WARP_SPECIALIZE": "constexpr"}
    mmc = {"BLOCK_SIZE_M": 128, "BLOCK_SIZE_N": 128, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 8, "FP8_OUTPUT": False,
           "WARP_SPECIALIZE": False}
    descs = {"a_desc": "tensordesc<bf16[128,64]>", "b_desc": "tensordesc<bf16[64,128]>", "c_desc": "tensordesc<bf16[128,128]>"}
    dims = {"M": "i32", "N": "i32", "K": "i32"}
    k = _compile(tk.matmul_kernel_tma, {**descs, **dims, **mm}, mmc)
    assert json.loads(k.kernel)["kernel"] == "matmul_kernel_tma"
    k = _compile(tk.matmul_kernel_fused, {**descs, "bias_desc": "tensordesc<bf16[128,128]>", **dims, **mm}, mmc)
    assert json.loads(k.kernel)["kernel"] == "matmul_kernel_fused"
    qd = "tensordesc<bf16[64,64]>"
    attn = {"sm_scale": "fp32", "M": "*fp32", "Z": "i32", "H": "i32", "desc_q": qd, "desc_k": qd, "desc_v": qd,
            "desc_o": qd, "N_CTX": "i32", "HEAD_DIM": "constexpr", "BLOCK_M": "constexpr", "BLOCK_N": "constexpr",
            "FP8_OUTPUT": "constexpr", "STAGE": "constexpr", "warp_specialize": "constexpr", "IS_HOPPER": "constexpr"}
    for stage in (1, 3):
        k = _compile(tk._attn_fwd, attn, {"HEAD_DIM": 64, "BLOCK_M": 64, "BLOCK_N": 64, "FP8_OUTPUT": False,
                                          "STAGE": stage, "warp_specialize": False, "IS_HOPPER": False})
        assert json.loads(k.kernel)["kernel"] == "_attn_fwd"
    k = _compile(tk.muladd_kernel, {"x_ptr": "*fp32", "y_ptr": "*fp32", "z_ptr": "*fp32", "output_ptr": "*fp32",
                                    "n_elements": "i32", "BLOCK_SIZE": "constexpr"}, {"BLOCK_SIZE": 1024})
    assert json.loads(k.kernel)["kernel"] == "muladd_kernel"
    k = _compile(tk.sin_kernel, {"x_ptr": "*fp32", "output_ptr": "*fp32", "n_elements": "i32", "BLOCK_SIZE": "constexpr"},
                 {"BLOCK_SIZE": 1024})
    assert json.loads(k.kernel)["kernel"] == "sin_kernel"
