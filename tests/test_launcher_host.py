"""Host-side logic of the plugin surface, no GPU: signature specialisation, the reference's
argument flattening, constexpr folding, binding of kernel names to C entry points (against a
recording stand-in for the library), and that libttamd_rt.so exports what the header declares."""
import ctypes as C
import re
from pathlib import Path

import pytest
import torch

from triton_tenstorrent_amd import jit, kernels as K, runtime as rt
from triton_tenstorrent_amd.backend import driver as drv
from triton_tenstorrent_amd.tensor_descriptor import TensorDescriptor

ROOT = Path(__file__).resolve().parent.parent


class FakeTensor:
    """Looks like a CUDA tensor to the launcher; never dereferenced."""

    def __init__(self, shape, dtype, ptr=0x7f0000000000):
        self.shape, self.dtype, self._ptr = tuple(shape), dtype, ptr
        self.is_cuda = True

    def data_ptr(self):
        return self._ptr

    def dim(self):
        return len(self.shape)

    def is_contiguous(self):
        return True

    def stride(self):
        st, acc = [], 1
        for d in reversed(self.shape):
            st.insert(0, acc)
            acc *= d
        return tuple(st)

    def numel(self):
        n = 1
        for d in self.shape:
            n *= d
        return n


class RecordingLib:
    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def fn(*args):
            self.calls.append((name, args))
            return 0
        return fn


@pytest.fixture
def fake(monkeypatch):
    lib = RecordingLib()
    monkeypatch.setattr(rt, "init", lambda device=0: lib)
    monkeypatch.setattr(drv.TTDriver, "get_current_device", lambda self: 0)
    monkeypatch.setattr(drv.TTDriver, "get_current_stream", lambda self, d=None: 0x1234)
    for k in (K.add_kernel, K.add_kernel_loop, K.sin_kernel, K.matmul_kernel_tma, K.matmul_kernel_fused, K._attn_fwd,
              K.matmul_kernel_tma_fp8_scaled, K.muladd_kernel, K.matmul_kernel, K.unary_kernel, K.binary_kernel,
              K.cast_kernel, K.reduce1d_kernel, K.binary_const_kernel, K.copy_kernel):
        k._cache.clear()
        k._plan = None
    return lib


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "ttamd_rt.h").read_text()
    declared = set(re.findall(r"TTAMD_API\s+(?:const\s+char\s*\*|int)\s*(\w+)\s*\(", header))
    assert declared == set(rt.SYMBOLS), declared ^ set(rt.SYMBOLS)
    lib = rt.load()
    for name in declared:
        assert getattr(lib, name) is not None


def test_calls_before_init_return_errors_instead_of_aborting():
    if rt._inited_device is not None:
        pytest.skip("an earlier test of this process has initialised the runtime")
    lib = rt.load()
    g = rt.grid3(1)
    assert lib.tt_add_kernel(None, None, None, 4, 1024, rt.TT_F32, g, None) == rt.RT_ERR_NOT_INIT
    assert "rt_init" in rt.last_error()
    p = rt.rt_props()
    assert lib.rt_device_props(C.byref(p)) == rt.RT_ERR_NOT_INIT
    assert lib.rt_launch(None, g, g, 0, None, None, 0) == rt.RT_ERR_INVALID
    if not torch.cuda.is_available():
        with pytest.raises(rt.RuntimeError_):
            rt.init(0)  # no device here: a HIP error string, not a crash


def test_specialize_matches_tritons_type_strings():
    x = FakeTensor((8, ), torch.float32)
    assert jit.specialize(x, False) == "*fp32"
    assert jit.specialize(FakeTensor((8, ), torch.bfloat16), False) == "*bf16"
    assert jit.specialize(FakeTensor((8, ), torch.float8_e4m3fn), False) == "*fp8e4nv"
    assert jit.specialize(98432, False) == "i32" and jit.specialize(2**31, False) == "i64"
    assert jit.specialize(1, False) == "constexpr"       # the value 1 is folded
    assert jit.specialize(0.5, False) == "fp32" and jit.specialize(1024, True) == "constexpr"
    d = TensorDescriptor(FakeTensor((256, 64), torch.bfloat16), [256, 64], [64, 1], [128, 64])
    assert jit.specialize(d, False) == "tensordesc<bf16[128,64]>"
    with pytest.raises(TypeError):
        jit.specialize("nope", False)


def test_descriptor_flattening_is_the_references_ten_scalars():
    # base, shape0, shape1, stride0, stride1, pad, shape0, shape1, stride0, stride1 (backend/driver.py:141-159)
    t = FakeTensor((64, 2560), torch.bfloat16)
    d = TensorDescriptor(t, [64, 2560], [2560, 1], [64, 64])
    flat = drv.flatten_launch_args(["tensordesc<bf16[64,64]>", "i32", "constexpr"], (d, 7, 64))
    assert flat == [t, 64, 2560, 2560, 1, 0, 64, 2560, 2560, 1, 7]
    d.padding = "nan"
    assert drv.flatten_launch_args(["tensordesc<bf16[64,64]>"], (d, ))[5] == 1
    # matmul_kernel_tma: 3 descriptors + M,N,K = 33 scalars (matmul_multi_core_tma.cpp:307-339)
    sig = ["tensordesc<bf16[64,64]>"] * 3 + ["i32"] * 3 + ["constexpr"] * 6
    assert len(drv.flatten_launch_args(sig, (d, d, d, 64, 2560, 9728, 64, 64, 64, 1, False, False))) == 33


def test_descriptor_asserts():
    t = FakeTensor((64, 64), torch.bfloat16)
    with pytest.raises(AssertionError):
        TensorDescriptor(t, [64, 64], [64, 2], [32, 32])            # last stride
    with pytest.raises(AssertionError):
        TensorDescriptor(FakeTensor((64, 64), torch.bfloat16, ptr=0x1008), [64, 64], [64, 1], [32, 32])  # 16 B base
    with pytest.raises(AssertionError):
        TensorDescriptor(t, [64, 60], [60, 1], [32, 32])            # 16 B leading stride
    with pytest.raises(AssertionError):
        TensorDescriptor(t, [64, 64], [64, 1], [32, 32], padding="inf")


def test_add_binds_and_folds_n_equal_one(fake):
    x = FakeTensor((98432, ), torch.float32)
    K.add_kernel[lambda meta: (K.cdiv(98432, meta["BLOCK_SIZE"]), )](x, x, x, 98432, BLOCK_SIZE=1024)
    name, a = fake.calls[-1]
    assert name == "tt_add_kernel" and a[3:6] == (98432, 1024, rt.TT_F32) and list(a[6]) == [97, 1, 1]
    assert a[7] == 0x1234          # the stream handle, as the integer ctypes converts to void*
    K.add_kernel[(1, )](x, x, x, 1, BLOCK_SIZE=1024)     # n_elements == 1 arrives as a constexpr
    assert fake.calls[-1][1][3] == 1
    xi = FakeTensor((10, ), torch.int32)
    K.add_kernel[(1, )](xi, xi, xi, 10, BLOCK_SIZE=1024)
    assert fake.calls[-1][1][5] == rt.TT_I32
    K.add_kernel_loop[(130, )](x, x, x, 98432, 1, BLOCK_SIZE=1024)  # row_count == 1 folded too
    assert fake.calls[-1][0] == "tt_add_kernel_loop" and fake.calls[-1][1][3:6] == (98432, 1, 1024)


def test_matmul_binding_pre_hook_and_grid(fake):
    a, b, c = FakeTensor((256, 128), torch.bfloat16), FakeTensor((128, 512), torch.bfloat16), FakeTensor((256, 512), torch.bfloat16)
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
    K.matmul_kernel_tma[lambda META: (K.cdiv(256, META["BLOCK_SIZE_M"]) * K.cdiv(512, META["BLOCK_SIZE_N"]), )](
        ad, bd, cd, 256, 512, 128, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert ad.block_shape == [128, 64] and bd.block_shape == [64, 128] and cd.block_shape == [128, 128]  # pre_hook ran
    name, args = fake.calls[-1]
    assert name == "tt_matmul_kernel_tma" and args[3:10] == (256, 512, 128, 128, 128, 64, 8) and list(args[10]) == [8, 1, 1]
    d = args[0]._obj
    assert (d.shape[0], d.shape[1], d.strides[0], d.strides[1], d.dtype) == (256, 128, 128, 1, rt.TT_BF16)
    # reference configuration by keyword
    K.matmul_kernel_tma[(32, )](ad, bd, cd, 256, 512, 128, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64, GROUP_SIZE_M=1,
                                FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert fake.calls[-1][1][6:10] == (64, 64, 64, 1)


def test_fused_and_attention_binding(fake):
    a, b, c = FakeTensor((256, 128), torch.bfloat16), FakeTensor((128, 512), torch.bfloat16), FakeTensor((256, 512), torch.bfloat16)
    ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
    full = TensorDescriptor.from_tensor(FakeTensor((256, 512), torch.bfloat16), [32, 32])
    K.matmul_kernel_fused[(8, )](ad, bd, cd, full, 256, 512, 128, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    assert fake.calls[-1][0] == "tt_matmul_kernel_fused" and fake.calls[-1][1][11] == rt.TT_EPI_BIAS_FULL
    row = TensorDescriptor.from_tensor(FakeTensor((1, 512), torch.float32), [1, 32])
    K.matmul_kernel_fused[(8, )](ad, bd, cd, row, 256, 512, 128, FP8_OUTPUT=False, WARP_SPECIALIZE=False, EPILOGUE="gelu")
    assert fake.calls[-1][1][11] == rt.TT_EPI_BIAS_ROW_GELU
    q = FakeTensor((1, 1, 256, 64), torch.bfloat16)
    M = FakeTensor((1, 1, 256), torch.float32)
    dq = TensorDescriptor(q, [256, 64], [64, 1], [1, 1])
    K._attn_fwd[(2, 1, 1)](0.125, M, 1, 1, dq, dq, dq, dq, N_CTX=256, HEAD_DIM=64, BLOCK_M=128, BLOCK_N=64, FP8_OUTPUT=False,
                           STAGE=3, warp_specialize=False, IS_HOPPER=False)   # Z = H = 1 are folded to constexprs
    name, args = fake.calls[-1]
    assert name == "tt_attn_fwd" and args[2:4] == (1, 1) and args[8:13] == (256, 64, 128, 64, 3)
    assert dq.block_shape == [128, 64]


def test_launch_hooks_and_metadata(fake):
    seen = []
    jit.PrebuiltKernel.launch_enter_hook = lambda md: seen.append(("enter", md))
    jit.PrebuiltKernel.launch_exit_hook = lambda md: seen.append(("exit", md))
    try:
        a, b, c = FakeTensor((128, 128), torch.bfloat16), FakeTensor((128, 128), torch.bfloat16), FakeTensor((128, 128), torch.bfloat16)
        ad, bd, cd = (TensorDescriptor.from_tensor(t, [32, 32]) for t in (a, b, c))
        K.matmul_kernel_tma[(1, )](ad, bd, cd, 128, 128, 128, FP8_OUTPUT=False, WARP_SPECIALIZE=False)
    finally:
        jit.PrebuiltKernel.launch_enter_hook = jit.PrebuiltKernel.launch_exit_hook = None
    assert [s[0] for s in seen] == ["enter", "exit"]
    assert seen[0][1]["flops16"] == 2.0 * 128 ** 3 and seen[0][1]["bytes"] == 2 * 3 * 128 * 128


def test_unknown_kernel_and_bad_arguments(fake):
    with pytest.raises(rt.RuntimeError_):
        drv.BoundKernel("no_such_kernel", {})
    x = FakeTensor((8, ), torch.float32)
    with pytest.raises(TypeError):
        K.add_kernel[(1, )](x, x, x, 8)                      # BLOCK_SIZE missing
    with pytest.raises(TypeError):
        K.add_kernel[(1, )](x, x, x, 8, BLOCK_SIZE=1024, bogus=3)
    with pytest.raises(ValueError):
        cpu = torch.zeros(8)
        K.add_kernel[(1, )](cpu, cpu, cpu, 8, BLOCK_SIZE=1024)   # host tensor


def test_driver_surface():
    d = drv.TTDriver()
    t = d.get_current_target()
    assert (t.backend, t.arch, t.warp_size) == ("tenstorrent", "gfx950", 64)
    assert d.map_python_to_cpp_type("*fp32") == "*fp32"
    assert d.launcher_cls is drv.TTLauncher and isinstance(d.utils, drv.TTUtils)
    di = d.get_device_interface()
    assert hasattr(di, "Event") and hasattr(di, "synchronize") and hasattr(di, "enable_hook_timing")


def test_pointer_matmul_binds_with_unit_strides_folded(fake):
    # matmul_kernel(a,b,c, M,N,K, six strides, constexprs): the unit strides arrive as constexprs
    # (03-matrix-multiplication.py:403-421 passes a.stride(1) == 1)
    a, b, c = FakeTensor((64, 96), torch.float16), FakeTensor((96, 32), torch.float16), FakeTensor((64, 32), torch.float16)
    launch = K.matmul_kernel[lambda META: (K.cdiv(64, META["BLOCK_SIZE_M"]) * K.cdiv(32, META["BLOCK_SIZE_N"]), )]
    launch(a, b, c, 64, 32, 96, 96, 1, 32, 1, 32, 1, ACTIVATION="leaky_relu")
    name, args = fake.calls[-1]
    assert name == "tt_matmul_kernel"
    assert args[3:6] == (64, 32, 96) and args[6:12] == (96, 1, 32, 1, 32, 1)
    assert args[12:16] == (32, 32, 32, 1) and args[16] == 1 and args[17] == rt.TT_F16
    assert list(args[18]) == [2, 1, 1]
    launch(a, b, c, 64, 32, 96, 96, 1, 32, 1, 32, 1)
    assert fake.calls[-1][1][16] == 0
    with pytest.raises(rt.Unsupported):
        launch(a, b, c, 64, 32, 96, 96, 1, 32, 1, 32, 1, ACTIVATION="relu")
    with pytest.raises(rt.InvalidLaunch):      # c must be fp16
        launch(a, b, FakeTensor((64, 32), torch.bfloat16), 64, 32, 96, 96, 1, 32, 1, 32, 1)
    with pytest.raises(rt.InvalidLaunch):      # ragged M needs a buffer padded to whole tiles
        launch(FakeTensor((60, 96), torch.float16), b, c, 60, 32, 96, 96, 1, 32, 1, 32, 1)


def test_packaging_declares_the_triton_backends_entry_point():
    # Triton 3.6 finds out-of-tree backends in the "triton.backends" entry-point group; the value must be a
    # package with compiler.py and driver.py (triton/backends/__init__.py)
    import importlib
    import tomli
    meta = tomli.loads((ROOT / "pyproject.toml").read_text())
    ep = meta["project"]["entry-points"]["triton.backends"]
    assert list(ep) == ["tenstorrent"]
    pkg = importlib.import_module(ep["tenstorrent"])
    comp, drv_mod = importlib.import_module(pkg.__name__ + ".compiler"), importlib.import_module(pkg.__name__ + ".driver")
    assert hasattr(comp, "TTBackend") and hasattr(drv_mod, "TTDriver")
    assert meta["tool"]["setuptools"]["package-dir"]["triton_tenstorrent_amd"] == "triton-tenstorrent_amd"
    assert (ROOT / "triton-tenstorrent_amd" / "backend" / "name.conf").exists()


def test_generic_elementwise_ops_bind_by_mnemonic(fake):
    x, o = FakeTensor((5000, ), torch.float32), FakeTensor((5000, ), torch.float32)
    K.unary_kernel[(5, )](x, o, 5000, BLOCK_SIZE=1024, OP="exp2")
    name, a = fake.calls[-1]
    assert name == "tt_unary_kernel" and a[0] == rt.UNARY_OPS["exp2"] and a[3:5] == (5000, 1024) and list(a[5]) == [5, 1, 1]
    K.binary_kernel[(5, )](x, x, o, 5000, BLOCK_SIZE=1024, OP="minimum")
    name, a = fake.calls[-1]
    assert name == "tt_binary_kernel" and a[0] == rt.BINARY_OPS["minimum"] and a[4:6] == (5000, 1024)
    K.cast_kernel[(5, )](x, FakeTensor((5000, ), torch.bfloat16), 5000, BLOCK_SIZE=1024)
    name, a = fake.calls[-1]
    assert name == "tt_cast_kernel" and a[4:6] == (rt.TT_F32, rt.TT_BF16)
    K.cast_kernel[(5, )](FakeTensor((5000, ), torch.int32), FakeTensor((5000, ), torch.int8), 5000, BLOCK_SIZE=1024)
    assert fake.calls[-1][1][4:6] == (rt.TT_I32, rt.TT_I8)
    with pytest.raises(rt.Unsupported):
        K.unary_kernel[(5, )](x, o, 5000, BLOCK_SIZE=1024, OP="tanh")
    with pytest.raises(rt.Unsupported):
        K.binary_kernel[(5, )](x, FakeTensor((5000, ), torch.float16), o, 5000, BLOCK_SIZE=1024, OP="add")
    # the op tables here, in the oracle and in the header agree
    from oracle import oracle as orc
    assert orc.UNARY_OPS == rt.UNARY_OPS and orc.BINARY_OPS == rt.BINARY_OPS
    header = (ROOT / "include" / "ttamd_rt.h").read_text()
    for name, code in rt.UNARY_OPS.items():
        assert re.search(rf"TT_OP_{name.upper()} = {code}\b", header), name
    for name, code in rt.BINARY_OPS.items():
        assert re.search(rf"TT_OP_{name.upper()} = {code}\b", header), name


def test_reduce1d_binds_with_tritons_accumulate_types(fake):
    z = FakeTensor((1, ), torch.int32)
    K.reduce1d_kernel[(1, )](FakeTensor((512, ), torch.int8), z, BLOCK=512, OP="sum")
    name, a = fake.calls[-1]
    assert name == "tt_reduce1d_kernel" and a[0] == rt.REDUCE_OPS["sum"] and a[3] == 512
    assert a[4:8] == (rt.TT_I8, rt.TT_I32, rt.TT_I32, 0) and list(a[8]) == [1, 1, 1]
    K.reduce1d_kernel[(1, )](FakeTensor((512, ), torch.uint8), FakeTensor((1, ), torch.uint32), BLOCK=512, OP="sum")
    assert fake.calls[-1][1][4:7] == (rt.TT_U8, rt.TT_U32, rt.TT_U32)
    K.reduce1d_kernel[(1, )](FakeTensor((64, ), torch.bfloat16), FakeTensor((1, ), torch.float32), BLOCK=64, OP="max",
                             PROPAGATE_NAN=True)
    assert fake.calls[-1][1][4:8] == (rt.TT_BF16, rt.TT_F32, rt.TT_F32, 1)
    K.reduce1d_kernel[(1, )](FakeTensor((64, ), torch.bfloat16), FakeTensor((1, ), torch.bfloat16), BLOCK=64, OP="sum")
    assert fake.calls[-1][1][4:7] == (rt.TT_BF16, rt.TT_BF16, rt.TT_BF16)
    K.reduce1d_kernel[(1, )](FakeTensor((64, ), torch.float16), z, BLOCK=64, OP="argmin")
    assert fake.calls[-1][1][0] == rt.REDUCE_OPS["argmin"] and fake.calls[-1][1][4:7] == (rt.TT_F16, rt.TT_F16, rt.TT_I32)
    with pytest.raises(rt.InvalidLaunch):
        K.reduce1d_kernel[(1, )](FakeTensor((64, ), torch.float32), z, BLOCK=64, OP="prod")
    with pytest.raises(rt.InvalidLaunch):
        K.reduce1d_kernel[(1, )](FakeTensor((32, ), torch.float32), z, BLOCK=64, OP="sum")     # reads past X
    from oracle import oracle as orc
    assert orc.REDUCE_OPS == rt.REDUCE_OPS
    header = (ROOT / "include" / "ttamd_rt.h").read_text()
    for name, code in rt.REDUCE_OPS.items():
        assert re.search(rf"TT_REDUCE_{name.upper()} = {code}\b", header), name
    for name, code in rt.DTYPE_OF_NAME.items():
        short = {"float32": "F32", "int32": "I32", "bfloat16": "BF16", "float16": "F16", "int16": "I16", "int8": "I8",
                 "int64": "I64", "float64": "F64", "uint8": "U8", "uint16": "U16", "uint32": "U32", "uint64": "U64"}[name]
        assert re.search(rf"TT_{short} = {code}\b", header), name
        assert getattr(orc, short) == code


def test_constant_operand_kernel_binds(fake):
    x, o = FakeTensor((5000, ), torch.float32), FakeTensor((5000, ), torch.float32)
    K.binary_const_kernel[(5, )](x, o, 5000, BLOCK_SIZE=1024, OP="sub", C=3.5, FLIP=True)
    name, a = fake.calls[-1]
    assert name == "tt_binary_const_kernel" and a[0] == rt.BINARY_OPS["sub"] and a[2:4] == (3.5, 1) and a[5:7] == (5000, 1024)
    K.binary_const_kernel[(5, )](x, x, 5000, BLOCK_SIZE=1024, OP="mul", C=2)          # in place, FLIP defaults to False
    name, a = fake.calls[-1]
    assert a[1] == a[4] and a[2:4] == (2.0, 0)
    with pytest.raises(rt.Unsupported):
        K.binary_const_kernel[(5, )](x, o, 5000, BLOCK_SIZE=1024, OP="pow", C=2.0)


def test_copy_kernel_binds(fake):
    for dt, code in ((torch.float32, rt.TT_F32), (torch.int8, rt.TT_I8), (torch.int64, rt.TT_I64), (torch.bfloat16, rt.TT_BF16)):
        x, o = FakeTensor((5000, ), dt), FakeTensor((5000, ), dt)
        K.copy_kernel[(5, )](x, o, 5000, BLOCK_SIZE=1024)
        name, a = fake.calls[-1]
        assert name == "tt_copy_kernel" and a[2:5] == (5000, 1024, code)
    with pytest.raises(rt.InvalidLaunch):
        K.copy_kernel[(5, )](FakeTensor((5000, ), torch.float32), FakeTensor((5000, ), torch.int32), 5000, BLOCK_SIZE=1024)



def test_elementwise_binders_refuse_a_launch_that_runs_past_an_operand(fake):
    """The launch touches min(n_elements, grid * BLOCK) elements of every operand; a tensor that holds fewer would be
    read or written out of bounds on the device, so the binder raises before anything is launched."""
    big, small = FakeTensor((4096, ), torch.float32), FakeTensor((1000, ), torch.float32)
    before = len(fake.calls)
    with pytest.raises(rt.InvalidLaunch, match="covers 4096"):
        K.add_kernel[(4, )](big, small, big, 4096, BLOCK_SIZE=1024)
    with pytest.raises(rt.InvalidLaunch):
        K.sin_kernel[(4, )](big, small, 4096, BLOCK_SIZE=1024)
    with pytest.raises(rt.InvalidLaunch):
        K.unary_kernel[(2, )](small, small, 2048, BLOCK_SIZE=1024, OP="exp")
    with pytest.raises(rt.InvalidLaunch):
        K.binary_kernel[(4, )](big, big, small, 4096, BLOCK_SIZE=1024, OP="mul")
    with pytest.raises(rt.InvalidLaunch):
        K.muladd_kernel[(4, )](big, big, small, big, 4096, BLOCK_SIZE=1024)
    with pytest.raises(rt.InvalidLaunch):
        K.copy_kernel[(4, )](small, big, 4096, BLOCK_SIZE=1024)
    with pytest.raises(rt.InvalidLaunch):
        K.add_kernel_loop[(2, )](big, big, small, 4096, 2, BLOCK_SIZE=1024)      # 2 programs x 2 rows x 1024
    assert len(fake.calls) == before
    # the mask and the grid both clip: a short grid or a small n_elements makes the same tensors legal
    K.add_kernel[(1, )](big, small, big, 4096, BLOCK_SIZE=512)
    K.add_kernel[(4, )](big, small, big, 1000, BLOCK_SIZE=1024)
    assert len(fake.calls) == before + 2


# --------------------------------------------------------------------------
# the cached repeat-launch path under threads (no GPU: stand-ins for the library and for tensors)
# --------------------------------------------------------------------------
import threading


def _descriptors(ptr, shape=(256, 128), dtype=torch.bfloat16):
    t = FakeTensor(shape, dtype, ptr)
    return TensorDescriptor(t, list(shape), [shape[1], 1], [32, 32])


def test_a_closure_parked_inside_the_c_call_keeps_its_own_descriptors(monkeypatch):
    """ctypes releases the interpreter lock for the duration of a C call, so a second thread can run the same
    closure while the first one's call is still reading its descriptor blocks.  The stand-in for the C entry point
    parks thread A inside the call until thread B has launched with other operands, and then looks at the blocks it
    was handed: they must still be A's."""
    monkeypatch.setattr(drv, "_tensor_type", lambda: FakeTensor)
    a_inside, b_done = threading.Event(), threading.Event()
    seen = {}

    def fn(da, db, dc, M, N, K_, bm, bn, bk, g, grid, stream):
        who = threading.current_thread().name
        if who == "A":
            a_inside.set()
            assert b_done.wait(10)
        seen[who] = tuple(r._obj.base for r in (da, db, dc)) + (da._obj.shape[0], M)
        return 0

    bases = [FakeTensor((256, 128), torch.bfloat16)] * 3
    direct = drv._desc_matmul_direct(fn, bases, 0, (128, 128, 64, 8))
    ops = {"A": (0x1000, 0x2000, 0x3000, 256), "B": (0x5000, 0x6000, 0x7000, 512)}
    ok = {}

    def launch(who):
        pa, pb, pc, M = ops[who]
        ok[who] = direct((_descriptors(pa, (M, 128)), _descriptors(pb, (128, 128)), _descriptors(pc, (M, 128)), M, 128, 128),
                         (4, ), 0)

    ta = threading.Thread(target=launch, args=("A", ), name="A")
    ta.start()
    assert a_inside.wait(10)
    tb = threading.Thread(target=launch, args=("B", ), name="B")
    tb.start()
    tb.join(10)
    b_done.set()
    ta.join(10)
    assert ok == {"A": True, "B": True}
    assert seen["A"] == (0x1000, 0x2000, 0x3000, 256, 256), seen
    assert seen["B"] == (0x5000, 0x6000, 0x7000, 512, 512), seen


def test_attention_closure_is_per_thread_too(monkeypatch):
    monkeypatch.setattr(drv, "_tensor_type", lambda: FakeTensor)
    a_inside, b_done = threading.Event(), threading.Event()
    seen = {}

    def fn(sm, m_ptr, Z, H, dq, dk, dv, do, n_ctx, hd, bm, bn, stage, grid, stream):
        who = threading.current_thread().name
        if who == "A":
            a_inside.set()
            assert b_done.wait(10)
        seen[who] = tuple(r._obj.base for r in (dq, dk, dv, do)) + (m_ptr, )
        return 0

    direct = drv._attn_direct(fn, [FakeTensor((512, 64), torch.bfloat16)] * 4, (64, 128, 64, 3))
    ok = {}

    def launch(who, p0):
        M = FakeTensor((2, 256), torch.float32, p0 + 0x900)
        ds = [_descriptors(p0 + i * 0x100, (512, 64)) for i in range(4)]
        ok[who] = direct((0.125, M, 1, 2, *ds, 256), (2, 2, 1), 0)

    ta = threading.Thread(target=launch, args=("A", 0x10000), name="A")
    ta.start()
    assert a_inside.wait(10)
    tb = threading.Thread(target=launch, args=("B", 0x20000), name="B")
    tb.start()
    tb.join(10)
    b_done.set()
    ta.join(10)
    assert ok == {"A": True, "B": True}
    assert seen["A"] == (0x10000, 0x10100, 0x10200, 0x10300, 0x10900), seen
    assert seen["B"] == (0x20000, 0x20100, 0x20200, 0x20300, 0x20900), seen


@pytest.fixture
def fast(monkeypatch):
    """The recording library with the cached repeat-launch path left ON: tensors are FakeTensors, the stream
    lookup is the stock one (so plans are built and taken) and answers a fixed handle."""
    lib = RecordingLib()
    monkeypatch.setattr(rt, "init", lambda device=0: lib)
    monkeypatch.setattr(drv, "_tensor_type", lambda: FakeTensor)
    jit.active_driver()
    monkeypatch.setattr(jit, "_raw_stream", lambda: (0, 0x1234))
    for k in (K.add_kernel, K.matmul_kernel_tma, K._attn_fwd):
        k._cache.clear()
        k._plan = None
    yield lib
    for k in (K.add_kernel, K.matmul_kernel_tma, K._attn_fwd):
        k._cache.clear()
        k._plan = None


def test_a_tensor_given_by_keyword_is_taken_from_the_call_not_from_the_plan(fast):
    """Launch arguments may arrive by keyword.  A second call with ANOTHER output tensor under the same keyword
    has to write there: the cached path compares only the values that select the kernel and reads the launch
    arguments from the call in hand (comparing whole keyword dictionaries would compare tensors, and taking the
    stored ones would write the previous call's buffer)."""
    x, y = FakeTensor((4096, ), torch.float32, 0x1000), FakeTensor((4096, ), torch.float32, 0x2000)
    out1, out2 = FakeTensor((4096, ), torch.float32, 0x3000), FakeTensor((4096, ), torch.float32, 0x4000)
    K.add_kernel[(4, )](x, y, output_ptr=out1, n_elements=4096, BLOCK_SIZE=1024)
    assert K.add_kernel._plan is not None
    n0 = len(fast.calls)
    K.add_kernel[(4, )](x, y, output_ptr=out2, n_elements=4096, BLOCK_SIZE=1024)
    name, a = fast.calls[-1]
    assert len(fast.calls) == n0 + 1 and name == "tt_add_kernel" and a[:4] == (0x1000, 0x2000, 0x4000, 4096)
    assert K.add_kernel._keep[2] is out2                     # and that is the tensor kept alive
    K.add_kernel[(2, )](x, y, output_ptr=out1, n_elements=2000, BLOCK_SIZE=1024)   # another n by keyword as well
    assert fast.calls[-1][1][:4] == (0x1000, 0x2000, 0x3000, 2000)
    K.add_kernel[(4, )](x, y, output_ptr=out2, n_elements=4096, BLOCK_SIZE=512)    # another constexpr: not the plan's kernel
    assert fast.calls[-1][1][2:5] == (0x4000, 4096, 512)
    K.add_kernel[(4, )](x, y, out1, n_elements=4096, BLOCK_SIZE=512)               # another split of the arguments
    assert fast.calls[-1][1][2:5] == (0x3000, 4096, 512)


def test_threads_with_different_constexprs_never_take_each_others_closure(fast):
    """One launcher serves every thread that launches a specialisation, and the closure a binder leaves carries the
    constexprs of ITS launch.  Two threads that launch the same kernel with different BLOCK sizes, again and again,
    each have to see their own BLOCK in every C call."""
    x = FakeTensor((1 << 16, ), torch.float32, 0x1000)
    errors = []
    start = threading.Barrier(2)

    def worker(block, out_ptr):
        out = FakeTensor((1 << 16, ), torch.float32, out_ptr)
        start.wait()
        for _ in range(300):
            K.add_kernel[(8, )](x, x, out, 1 << 16, BLOCK_SIZE=block)

    threads = [threading.Thread(target=worker, args=(256, 0xA000)), threading.Thread(target=worker, args=(1024, 0xB000))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(30)
    for name, a in fast.calls:
        if (a[2], a[4]) not in ((0xA000, 256), (0xB000, 1024)):
            errors.append((name, a[2], a[4]))
    assert len(fast.calls) == 600 and not errors, errors[:3]


def test_launcher_keeps_operands_and_closure_per_thread(fake):
    x = FakeTensor((4096, ), torch.float32)
    K.add_kernel[(4, )](x, x, x, 4096, BLOCK_SIZE=1024)
    launcher = next(iter(K.add_kernel._cache.values()))[0]
    assert launcher.direct is not None and len(launcher.keepalive) == 3
    other = {}
    t = threading.Thread(target=lambda: other.update(direct=launcher.direct, keep=list(launcher.keepalive)))
    t.start()
    t.join(10)
    assert other == {"direct": None, "keep": []}             # a thread that has not launched holds nothing
