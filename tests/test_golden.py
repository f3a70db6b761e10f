"""The committed fixtures of tests/golden/ (made by tests/golden/make_golden.py from seeds).

Not marked gpu: the oracle of today still reproduces every stored output, so a change to the oracle's
arithmetic shows up as a diff against data in the repository, and the generator is deterministic.
Marked gpu: the HIP kernels, through the launcher and the C ABI, against the stored outputs with no
oracle in the loop, to each kernel's bar (bit-exact for exact operations, integer work and small-integer
products; the stated tolerances elsewhere)."""
import importlib.util
from pathlib import Path

import numpy as np
import pytest
import torch

GOLDEN = Path(__file__).resolve().parent / "golden"


def _load(name):
    with np.load(GOLDEN / f"{name}.npz", allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


def _same(a: np.ndarray, b: np.ndarray) -> bool:
    """Equal as bit patterns, any NaN matching any NaN."""
    if a.dtype.kind == "f":
        nan = np.isnan(a)
        return bool(np.array_equal(nan, np.isnan(b)) and np.array_equal(a[~nan].view(np.uint32 if a.itemsize == 4 else np.uint64),
                                                                         b[~nan].view(np.uint32 if a.itemsize == 4 else np.uint64)))
    return bool(np.array_equal(a, b))


@pytest.mark.parametrize("name", ["elementwise", "matmul", "attention", "reductions"])
def test_oracle_reproduces_the_fixtures(name):
    spec = importlib.util.spec_from_file_location("make_golden", GOLDEN / "make_golden.py")
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    want, got = _load(name), mg.FIXTURES[name]()
    assert sorted(want) == sorted(got)
    for k in want:
        g = np.asarray(got[k])
        assert g.dtype == want[k].dtype and g.shape == want[k].shape, k
        assert _same(g, want[k]), k


# ----------------------------------------------------------------------------------------------------------
gpu = pytest.mark.gpu


def _bf16(bits_):
    return torch.from_numpy(bits_.view(np.int16).copy()).view(torch.bfloat16)


def _f16(bits_):
    return torch.from_numpy(bits_.view(np.int16).copy()).view(torch.float16)


def _bits16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _f32_of_bf16(bits_):
    return (bits_.astype(np.uint32) << 16).view(np.float32)


@gpu
def test_elementwise_fixture_on_the_gpu():
    from triton_tenstorrent_amd import kernels as K
    g = _load("elementwise")
    x, y, z = (torch.from_numpy(g[k]).cuda() for k in ("x", "y", "z"))
    xi, yi, xs = (torch.from_numpy(g[k]).cuda() for k in ("xi", "yi", "xs"))
    assert _same(K.add(x, y).cpu().numpy(), g["add_f32"])
    assert _same(K.add(xi, yi).cpu().numpy(), g["add_i32"])
    assert _same(K.muladd(x, y, z).cpu().numpy(), g["muladd"])
    assert np.max(np.abs(K.sin(xs).cpu().numpy().astype(np.float64) - g["sin"])) <= 2e-6
    assert _same(K.cast(xi, torch.int16).cpu().numpy(), g["trunci16"]) and _same(K.cast(xi, torch.int8).cpu().numpy(), g["trunci8"])
    got_bf16, got_f16 = _bits16(K.cast(x, torch.bfloat16)), _bits16(K.cast(x, torch.float16))
    nan = np.isnan(g["x"])
    assert np.array_equal(got_bf16[~nan], g["truncf_bf16"][~nan]) and np.array_equal(got_f16[~nan], g["truncf_f16"][~nan])
    for op in ("abs", "ceil", "floor", "sqrt"):
        assert _same(K.unary(op, x).cpu().numpy(), g[f"unary_{op}"]), op
    for op in ("add", "sub", "mul", "div", "maximum", "minimum"):
        assert _same(K.binary(op, x, y).cpu().numpy(), g[f"binary_{op}"]), op
    for op in ("cos", "sin", "exp", "exp2", "log", "log2", "rsqrt"):
        got, want = K.unary(op, x).cpu().numpy(), g[f"unary_{op}"]
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want)), op
        ok = np.isfinite(want) & (np.abs(want) >= 2.0**-126)
        err = np.abs(got[ok].astype(np.float64) - want[ok].astype(np.float64))
        slack = 2 * np.spacing(np.abs(want[ok])).astype(np.float64)
        if op in ("cos", "sin"):
            slack = np.maximum(slack, 2e-6)          # near a zero of the function the bar is absolute
        assert np.all(err <= slack), op


@gpu
def test_matmul_fixture_on_the_gpu():
    from triton_tenstorrent_amd import kernels as K
    g = _load("matmul")
    close = lambda got, want: bool(np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-4))
    # small integers: bit for bit, in two tilings
    a, b = _bf16(g["int_a"]).cuda(), _bf16(g["int_b"]).cuda()
    for cfg in (dict(BLOCK_SIZE_M=32, BLOCK_SIZE_N=32, BLOCK_SIZE_K=32, GROUP_SIZE_M=1),
                dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=32, BLOCK_SIZE_K=64, GROUP_SIZE_M=2)):
        assert np.array_equal(_bits16(K.matmul_tma(a, b, **cfg)), g["int_c"])
    a, b = _bf16(g["a"]).cuda(), _bf16(g["b"]).cuda()
    assert close(_f32_of_bf16(_bits16(K.matmul_tma(a, b))), _f32_of_bf16(g["c"]))
    got = _f32_of_bf16(_bits16(K.matmul_fused(a, b, _bf16(g["bias_full"]).cuda())))
    assert close(got, _f32_of_bf16(g["c_bias_full"]))
    got = _f32_of_bf16(_bits16(K.matmul_fused(a, b, torch.from_numpy(g["bias_row"]).cuda(), epilogue="gelu")))
    assert close(got, _f32_of_bf16(g["c_gelu"]))
    aq = torch.from_numpy(g["aq"]).view(torch.float8_e4m3fn).cuda()
    bq = torch.from_numpy(g["bq"]).view(torch.float8_e4m3fn).cuda()
    got = _f32_of_bf16(_bits16(K.matmul_fp8_scaled(aq, bq, float(g["scales"][0]), float(g["scales"][1]))))
    assert close(got, _f32_of_bf16(g["c_fp8"]))
    M, N, Kd = (int(v) for v in g["tiled_shape"])
    at, bt = _f16(g["a_tiled"]).cuda(), _f16(g["b_tiled"]).cuda()
    for key, act in (("c_tiled", ""), ("c_tiled_leaky", "leaky_relu")):
        got = K.matmul_tiled(at, bt, M, N, Kd, activation=act)
        want = _f16(g[key]).float().numpy()
        # the padding of C is never written: compare the tiles' live parts
        live = K.untilize(got, M, N, 32, 32).float().cpu().numpy()
        assert close(live, K.untilize(torch.from_numpy(want), M, N, 32, 32).numpy()), key


@gpu
def test_attention_fixture_on_the_gpu():
    from triton_tenstorrent_amd import kernels as K
    g = _load("attention")
    q, k, v = (_bf16(g[n]).cuda() for n in ("q", "k", "v"))
    for causal, tag in ((True, "causal"), (False, "full")):
        o, m = K.attention(q, k, v, causal, float(g["sm_scale"][0]), return_lse=True)
        assert np.max(np.abs(o.float().cpu().numpy() - _f32_of_bf16(g[f"o_{tag}"]))) <= 2e-2
        assert np.max(np.abs(m.cpu().numpy() - g[f"m_{tag}"])) <= 1e-3


@gpu
def test_reduction_fixture_on_the_gpu():
    from triton_tenstorrent_amd import kernels as K
    g = _load("reductions")
    for name in ("i8", "u8", "i16", "i32", "u32", "i64"):
        x = torch.from_numpy(g[f"x_{name}"]).cuda()
        for op in ("sum", "min", "max", "argmin", "argmax", "xor_sum"):
            got = K.reduce1d(op, x).cpu().numpy()
            assert got.dtype == g[f"{op}_{name}"].dtype and got[0] == g[f"{op}_{name}"][0], (op, name)
    x = torch.from_numpy(g["x_f32"]).cuda()
    for op in ("min", "max", "argmin", "argmax"):
        assert K.reduce1d(op, x).cpu().numpy()[0] == g[f"{op}_f32"][0], op
    bound = 512 * 2.0**-24 * float(np.abs(g["x_f32"]).astype(np.float64).sum())
    assert abs(float(K.reduce1d("sum", x).cpu()[0]) - float(g["sum_f32"][0])) <= 2 * bound
