"""Recognise the masked-block elementwise form in TTIR.

The operations the reference's compute lowering accepts
(npu/lib/Dialect/TritonTenstorrent/Transforms/ConvertComputeOps.cpp:162-182) reach it inside kernels of one
shape, the one of ``sin_kernel`` and ``add_kernel`` (examples/01-sin-kernel.py:17-29,
python/tutorials/01-vector-add.py:29-54):

    pid = program_id(0); offsets = pid * BLOCK + arange(0, BLOCK); mask = offsets < n
    store(out + offsets, OP(load(x + offsets, mask) [, load(y + offsets, mask)]), mask)

A kernel of that shape, whatever it is called, is bound to the prebuilt ``unary_kernel`` / ``binary_kernel`` /
``cast_kernel`` with the operation read off the IR.  Nothing is generated: anything that is not exactly this
shape over fp32 (or the two narrowing casts) is not matched and stays a compile error.

The second form is the single-block reduction the reference's CI runs on its cpu/ path
(.github/workflows/integration-tests-cpu.yml:105, test_core.py::test_reduce1d):

    x = load(X + arange(0, BLOCK)); store(Z, reduce(x, axis=0))

bound to ``reduce1d_kernel`` with the reduction, the element types and the NaN rule read off the ``tt.reduce``.
"""
from __future__ import annotations

import re

UNARY = {"math.absf": "abs", "math.ceil": "ceil", "math.cos": "cos", "math.exp": "exp", "math.exp2": "exp2",
         "math.floor": "floor", "math.log": "log", "math.log2": "log2", "math.rsqrt": "rsqrt", "math.sin": "sin",
         "math.sqrt": "sqrt"}
BINARY = {"arith.addf": "add", "arith.subf": "sub", "arith.mulf": "mul", "arith.divf": "div",
          "arith.maximumf": "maximum", "arith.minimumf": "minimum"}
CASTS = {"arith.truncf", "arith.trunci"}
# element types a copy moves, as tt_dtype codes (unsigned integers arrive as the signed type of their width)
_COPY_ELEM = {"f32": 0, "i32": 1, "bf16": 2, "f16": 3, "f8E4M3FN": 4, "i16": 5, "i8": 6, "i64": 7, "f64": 8}
_PLUMBING = {"tt.get_program_id", "arith.constant", "arith.muli", "tt.make_range", "tt.splat", "arith.addi",
             "arith.cmpi", "tt.addptr", "tt.load", "tt.store", "tt.return"}

_LOC = re.compile(r"\s*loc\(.*\)\s*$")
_OP = re.compile(r"^\s*(?:(%[\w.#]+)\s*=\s*)?([a-z_]+\.[a-z_0-9.]+)\s*(.*)$")
_SSA = re.compile(r"%[\w.#]+")


def _strip_locs(text: str) -> str:
    """Drop every ``loc(...)`` annotation (they nest: ``loc("x"(#loc))``)."""
    out, i, n = [], 0, len(text)
    while i < n:
        j = text.find("loc(", i)
        if j < 0 or (j > 0 and (text[j - 1].isalnum() or text[j - 1] in "_#")):
            if j < 0:
                out.append(text[i:])
                break
            out.append(text[i:j + 4])
            i = j + 4
            continue
        out.append(text[i:j])
        depth, k = 1, j + 4
        while k < n and depth:
            depth += text[k] == "("
            depth -= text[k] == ")"
            k += 1
        i = k
    return "".join(out)


def _body(ttir: str):
    ttir = _strip_locs(ttir)
    m = re.search(r"tt\.func\s+public\s+@(\w+)\((.*?)\)\s*(?:attributes\s*\{.*?\}\s*)?\{\s*\n(.*?)\n\s*\}", ttir, re.S)
    if not m:
        return None
    args = re.findall(r"(%[\w.]+)\s*:\s*([^,{]+?)\s*(?:\{[^}]*\})?\s*(?:,|$)", m.group(2))
    return m.group(1), [(a, t.strip()) for a, t in args], m.group(3).splitlines()


def match_streaming(ttir: str) -> dict | None:
    """``{"kernel", "op", "inputs": [arg names], "output": name, "n": name, "block": int}`` or None."""
    parsed = _body(ttir)
    if parsed is None:
        return None
    _, args, lines = parsed
    arg_types = dict(args)
    defs: dict[str, tuple[str, list[str], str]] = {}
    compute, store = [], []
    for raw in lines:
        line = _LOC.sub("", raw).strip()
        if not line:
            continue
        m = _OP.match(line)
        if not m:
            return None
        res, op, rest = m.groups()
        operands = _SSA.findall(rest.split(" : ")[0])
        is_int_add = op == "arith.addi" and operands and all(defs.get(o, ("",))[0] == "tt.load" for o in operands)
        if op in UNARY or op in BINARY or op in CASTS or is_int_add:
            compute.append((res, op, operands, rest))
        elif op == "tt.store":
            store.append((operands, rest))
        elif op not in _PLUMBING:
            return None
        if res:
            defs[res] = (op, operands, rest)
    if len(store) != 1 or len(compute) not in (0, 1, 2):
        return None
    if not compute:
        # the loaded block stored back unchanged: the copy kernel of test_launch.py::test_memory_leak
        # (.github/workflows/integration-tests-cpu.yml:106)
        if len(store[0][0]) != 3:
            return None
        res, op, operands = store[0][0][1], "copy", [store[0][0][1]]
    elif len(compute) == 2:
        # x * y + z, contracted to one fused multiply-add (01-vector-mul-add.py:30-57; enable_fp_fusion)
        (mres, mop, mops, _), (ares, aop, aops, _) = compute
        if mop != "arith.mulf" or aop != "arith.addf" or mres not in aops or len(aops) != 2:
            return None
        z = aops[0] if aops[1] == mres else aops[1]
        res, op, operands = ares, "muladd", list(mops) + [z]
    else:
        res, op, operands, rest = compute[0]

    def pointer_arg(ptr_ssa):
        # %p = tt.addptr %splat, %offsets ; %splat = tt.splat %arg
        d = defs.get(ptr_ssa)
        if not d or d[0] != "tt.addptr" or len(d[1]) != 2:
            return None, None
        s = defs.get(d[1][0])
        if not s or s[0] != "tt.splat" or s[1][0] not in arg_types:
            return None, None
        return s[1][0], d[1][1]

    (st_ops, _), = store
    if len(st_ops) != 3 or st_ops[1] != res:
        return None
    out_arg, offsets = pointer_arg(st_ops[0])
    mask = st_ops[2]
    if out_arg is None:
        return None
    inputs = []
    const_operand = None       # (position, value) of a splat constant among the operands of a binary operation
    for pos, o in enumerate(operands):
        d = defs.get(o)
        if d and d[0] == "arith.constant" and op in BINARY and const_operand is None and len(operands) == 2:
            cm = re.match(r"\s*dense<([^>]+)>\s*:\s*tensor<\d+xf32>", d[2])
            if not cm:
                return None
            const_operand = (pos, float(cm.group(1)))
            continue
        if not d or d[0] != "tt.load" or len(d[1]) < 2 or d[1][1] != mask:
            return None
        a, offs = pointer_arg(d[1][0])
        if a is None or offs != offsets:
            return None
        inputs.append(a)
    # mask = offsets < splat(n)
    md = defs.get(mask)
    if not md or md[0] != "arith.cmpi" or not md[2].lstrip().startswith("slt") or md[1][0] != offsets:
        return None
    ns = defs.get(md[1][1])
    n_src, n_const = None, None
    if ns and ns[0] == "arith.constant":       # the bound is a constant of the kernel: dense<N> : tensor<BLOCKxi32>
        cm = re.match(r"\s*dense<(-?\d+)>\s*:\s*tensor<\d+xi32>", ns[2])
        if not cm:
            return None
        n_const = int(cm.group(1))
    elif ns and ns[0] == "tt.splat":
        n_src = ns[1][0] if ns[1] else None
        if n_src not in arg_types:             # n_elements folded to a constant (the value 1)
            c = defs.get(n_src)
            if not c or c[0] != "arith.constant":
                return None
            n_const = int(re.match(r"\s*(-?\d+)", c[2]).group(1))
    else:
        return None
    # offsets = splat(pid * BLOCK) + make_range(0, BLOCK), either order
    od = defs.get(offsets)
    if not od or od[0] != "arith.addi" or len(od[1]) != 2:
        return None
    kinds = {defs[x][0]: x for x in od[1] if x in defs}
    if set(kinds) != {"tt.splat", "tt.make_range"}:
        return None
    rng = re.search(r"end\s*=\s*(\d+)\s*:\s*i32,\s*start\s*=\s*(\d+)", defs[kinds["tt.make_range"]][2])
    if not rng or int(rng.group(2)) != 0:
        return None
    block = int(rng.group(1))
    mul = defs.get(defs[kinds["tt.splat"]][1][0])
    if not mul or mul[0] != "arith.muli" or len(mul[1]) != 2:
        return None
    mk = {defs[x][0]: x for x in mul[1] if x in defs}
    if set(mk) != {"tt.get_program_id", "arith.constant"} or not defs[mk["tt.get_program_id"]][2].lstrip().startswith("x"):
        return None
    if int(re.match(r"\s*(-?\d+)", defs[mk["arith.constant"]][2]).group(1)) != block:
        return None
    # element types
    in_types = {arg_types[a] for a in inputs}
    out_type = arg_types[out_arg]
    if op == "copy":
        elem = re.fullmatch(r"!tt\.ptr<(\w+)>", out_type)
        if in_types != {out_type} or len(inputs) != 1 or not elem or elem.group(1) not in _COPY_ELEM:
            return None
        kernel, opname = "copy_kernel", None
    elif op == "muladd":
        if in_types != {"!tt.ptr<f32>"} or out_type != "!tt.ptr<f32>" or len(inputs) != 3:
            return None
        kernel, opname = "muladd_kernel", None
    elif op == "arith.addi":
        if in_types != {"!tt.ptr<i32>"} or out_type != "!tt.ptr<i32>" or len(inputs) != 2:
            return None
        kernel, opname = "add_kernel", "i32"
    elif op in CASTS:
        ok = (in_types, out_type) in (({"!tt.ptr<f32>"}, "!tt.ptr<bf16>"), ({"!tt.ptr<f32>"}, "!tt.ptr<f16>"),
                                      ({"!tt.ptr<i32>"}, "!tt.ptr<i16>"), ({"!tt.ptr<i32>"}, "!tt.ptr<i8>"))
        if not ok or len(inputs) != 1:
            return None
        kernel, opname = "cast_kernel", None
    else:
        if in_types != {"!tt.ptr<f32>"} or out_type != "!tt.ptr<f32>":
            return None
        if op in UNARY:
            if len(inputs) != 1:
                return None
            kernel, opname = "unary_kernel", UNARY[op]
        elif const_operand is not None:
            if len(inputs) != 1:
                return None
            kernel, opname = "binary_const_kernel", BINARY[op]
        else:
            if len(inputs) != 2:
                return None
            kernel, opname = "binary_kernel", BINARY[op]
    strip = lambda a: a.lstrip("%")
    rec = {"kernel": kernel, "op": opname, "inputs": [strip(a) for a in inputs], "output": strip(out_arg),
           "n": strip(n_src) if n_const is None else None, "n_const": n_const, "block": block}
    if kernel == "binary_const_kernel":
        rec.update(c=const_operand[1], flip=const_operand[0] == 0)
    if kernel == "copy_kernel":
        rec.update(dtype=_COPY_ELEM[elem.group(1)])
    return rec


def match_empty(ttir: str) -> dict | None:
    """A kernel whose body is ``tt.return`` alone (``def kernel(x): pass``, the kernel the hook tests of
    test_launch.py launch, .github/workflows/integration-tests-cpu.yml:106): nothing to run on the device."""
    parsed = _body(ttir)
    if parsed is None:
        return None
    body = [l for l in (_LOC.sub("", raw).strip() for raw in parsed[2]) if l]
    return {"kernel": "empty_kernel"} if body == ["tt.return"] else None


_ELEM = {"f32": 0, "i32": 1, "bf16": 2, "f16": 3, "i16": 5, "i8": 6, "i64": 7, "f64": 8}
_UNSIGNED_OF = {6: 9, 5: 10, 1: 11, 7: 12}
_REDUCE = re.compile(r'(%[\w.#]+)(?::(\d))?\s*=\s*"tt\.reduce"\(([^)]*)\)\s*<\{axis = 0 : i32\}>\s*\(\{\s*\n(.*?)\n\s*\}\)'
                     r'\s*:\s*\(([^)]*)\)\s*->\s*([^\n]*)\n', re.S)
_FOLDS = {"arith.addf": ("sum", None), "arith.addi": ("sum", None), "arith.xori": ("xor_sum", None),
          "arith.maxnumf": ("max", None), "arith.minnumf": ("min", None),
          "arith.maximumf": ("max", "nan"), "arith.minimumf": ("min", "nan"),
          "arith.maxsi": ("max", "s"), "arith.minsi": ("min", "s"), "arith.maxui": ("max", "u"), "arith.minui": ("min", "u")}


def _ops_of(lines):
    out = []
    for raw in lines:
        line = raw.strip()
        if not line or line.startswith("^bb") or line == "}":
            continue
        m = _OP.match(line)
        if not m:
            return None
        res, op, rest = m.groups()
        out.append((res, op, _SSA.findall(rest.split(" : ")[0]), rest))
    return out


def match_reduce1d(ttir: str) -> dict | None:
    """``{"kernel": "reduce1d_kernel", "op", "inputs": [X], "output": Z, "block", "in_dtype", "acc_dtype",
    "out_dtype", "propagate_nan", "tie_break_left"}`` (dtypes as tt_dtype codes) or None."""
    text = _strip_locs(ttir)
    f = re.search(r"tt\.func\s+public\s+@(\w+)\((.*?)\)\s*(?:attributes\s*\{.*?\}\s*)?\{\s*\n", text, re.S)
    if not f:
        return None
    arg_types = {a: t.strip() for a, t in re.findall(r"(%[\w.]+)\s*:\s*([^,{]+?)\s*(?:\{[^}]*\})?\s*(?:,|$)", f.group(2))}
    body = text[f.end():]
    r = _REDUCE.search(body)
    if not r or _REDUCE.search(body, r.end()):
        return None
    res, nres, red_operands, region, in_tensors, out_types = r.groups()
    red_operands = _SSA.findall(red_operands)
    tail = body[r.end():]
    end = tail.find("tt.return")
    if end < 0:
        return None
    pre, fold, post = (_ops_of(t.splitlines()) for t in (body[:r.start()], region, tail[:end + len("tt.return")]))
    if pre is None or fold is None or post is None or len(red_operands) not in (1, 2):
        return None
    defs = {o[0]: o for o in pre if o[0]}
    if any(o[1] not in ("tt.make_range", "tt.splat", "tt.addptr", "tt.load", "arith.extsi", "arith.extui", "arith.extf")
           for o in pre):
        return None
    # value operand: [ext of] load(addptr(splat(X), make_range(0, BLOCK))), no mask
    v = defs.get(red_operands[0])
    ext = None
    if v and v[1].startswith("arith.ext"):
        ext, v = v[1], defs.get(v[2][0])
    if not v or v[1] != "tt.load" or len(v[2]) != 1:
        return None
    ap = defs.get(v[2][0])
    if not ap or ap[1] != "tt.addptr" or len(ap[2]) != 2:
        return None
    sp, rg = defs.get(ap[2][0]), defs.get(ap[2][1])
    if not sp or sp[1] != "tt.splat" or sp[2][0] not in arg_types or not rg or rg[1] != "tt.make_range":
        return None
    x_arg = sp[2][0]
    span = re.search(r"end\s*=\s*(\d+)\s*:\s*i32,\s*start\s*=\s*(\d+)", rg[3])
    if not span or int(span.group(2)) != 0:
        return None
    block = int(span.group(1))
    if len(red_operands) == 2 and red_operands[1] != rg[0]:      # the index operand is the same arange
        return None
    # element types: X's, the one the reduction runs in, Z's
    pe = re.fullmatch(r"!tt\.ptr<(\w+)>", arg_types[x_arg])
    te = re.match(r"tensor<%dx(\w+)>" % block, in_tensors.strip())
    if not pe or not te or pe.group(1) not in _ELEM or te.group(1) not in _ELEM:
        return None
    in_dt, acc_dt = _ELEM[pe.group(1)], _ELEM[te.group(1)]
    if (ext is None) != (in_dt == acc_dt):
        return None
    kinds = [o[1] for o in fold if o[1] != "tt.reduce.return"]
    unsigned, nan, tie = ext == "arith.extui", False, False
    if len(red_operands) == 1:
        if len(kinds) != 1 or kinds[0] not in _FOLDS:
            return None
        op, rule = _FOLDS[kinds[0]]
        unsigned |= rule == "u"
        nan = rule == "nan"
        want = None
    else:
        # the (value, index) combine of triton/language/standard.py: compares, and / or, two selects
        if any(k not in ("arith.cmpf", "arith.cmpi", "arith.andi", "arith.ori", "arith.select") for k in kinds) \
                or kinds.count("arith.select") != 2:
            return None
        preds = [o[3].split()[0].rstrip(",") for o in fold if o[1] in ("arith.cmpf", "arith.cmpi")]
        order = [p for p in preds if p in ("olt", "ogt", "slt", "sgt", "ult", "ugt")]
        # with tie_break_left the index compare adds one `slt`; the value compare is the last one written
        tie = any(p in ("oeq", "eq") for p in preds)
        if not order or len(order) != (2 if tie else 1) or (tie and order[0] != "slt"):
            return None
        unsigned |= order[-1] in ("ult", "ugt")
        op = "min" if order[-1].endswith("lt") else "max"
        want = {"0": "value", "1": "index"}
    if unsigned:
        if in_dt not in _UNSIGNED_OF:
            return None
        in_dt = _UNSIGNED_OF[in_dt]
        acc_dt = _UNSIGNED_OF.get(acc_dt, acc_dt) if ext is None else acc_dt
    # after the reduction: [trunc] then store(Z, result)
    if not post or post[-1][1] != "tt.return" or len(post) not in (2, 3):
        return None
    st = post[-2]
    if st[1] != "tt.store" or len(st[2]) != 2 or st[2][0] not in arg_types:
        return None
    stored = st[2][1]
    if len(post) == 3:
        if post[0][1] not in ("arith.trunci", "arith.truncf") or post[0][0] != stored or len(post[0][2]) != 1:
            return None
        stored = post[0][2][0]
    if want is None:
        if stored != res:
            return None
    else:
        which = stored.split("#")
        if len(which) != 2 or which[0] != res or which[1] not in want:
            return None
        if which[1] == "1":
            op = "arg" + op
    ze = re.fullmatch(r"!tt\.ptr<(\w+)>", arg_types[st[2][0]])
    if not ze or ze.group(1) not in _ELEM:
        return None
    out_dt = _ELEM[ze.group(1)]
    if unsigned and not op.startswith("arg"):
        out_dt = _UNSIGNED_OF.get(out_dt, out_dt)
    strip = lambda a: a.lstrip("%")
    return {"kernel": "reduce1d_kernel", "op": op, "inputs": [strip(x_arg)], "output": strip(st[2][0]), "n": None,
            "n_const": block, "block": block, "in_dtype": in_dt, "acc_dtype": acc_dt, "out_dtype": out_dt,
            "propagate_nan": nan, "tie_break_left": tie}


def match_per_program(ttir: str) -> dict | None:
    """The one-element-per-program form of test_core.py::test_load_store_same_ptr:

        pid = program_id(0); x = load(p + pid); store(q + pid, x OP constant)

    (p and q may be the same argument) -> ``binary_const_kernel`` with BLOCK = 1 and n = the grid, or None."""
    parsed = _body(ttir)
    if parsed is None:
        return None
    _, args, lines = parsed
    arg_types = dict(args)
    defs, order = {}, []
    for raw in lines:
        line = _LOC.sub("", raw).strip()
        if not line:
            continue
        m = _OP.match(line)
        if not m:
            return None
        res, op, rest = m.groups()
        operands = _SSA.findall(rest.split(" : ")[0])
        order.append((res, op, operands, rest))
        if res:
            defs[res] = (op, operands, rest)
    kinds = [o[1] for o in order]
    compute = [o for o in order if o[1] in BINARY]
    if sorted(k for k in kinds if k not in BINARY) != sorted(["tt.get_program_id", "tt.addptr", "tt.load", "arith.constant",
                                                             "tt.addptr", "tt.store", "tt.return"]) and \
            sorted(k for k in kinds if k not in BINARY) != sorted(["tt.get_program_id", "tt.addptr", "tt.load", "arith.constant",
                                                                 "tt.store", "tt.return"]):
        return None
    if len(compute) != 1:
        return None
    res, op, operands, _ = compute[0]
    if len(operands) != 2:
        return None

    def pointer_arg(ssa):      # %p = tt.addptr %arg, %pid with %pid = tt.get_program_id x
        d = defs.get(ssa)
        if not d or d[0] != "tt.addptr" or len(d[1]) != 2 or d[1][0] not in arg_types:
            return None
        pid = defs.get(d[1][1])
        if not pid or pid[0] != "tt.get_program_id" or not pid[2].lstrip().startswith("x"):
            return None
        return d[1][0]

    x_arg = c = flip = None
    for pos, o in enumerate(operands):
        d = defs.get(o)
        if d and d[0] == "tt.load" and len(d[1]) == 1:
            x_arg = pointer_arg(d[1][0])
        elif d and d[0] == "arith.constant":
            cm = re.match(r"\s*([-+0-9.eE]+(?:inf|nan)?)\s*:\s*f32", d[2])
            if not cm:
                return None
            c, flip = float(cm.group(1)), pos == 0
    st = next(o for o in order if o[1] == "tt.store")
    if x_arg is None or c is None or len(st[2]) != 2 or st[2][1] != res:
        return None
    out_arg = pointer_arg(st[2][0])
    if out_arg is None or arg_types[x_arg] != "!tt.ptr<f32>" or arg_types[out_arg] != "!tt.ptr<f32>":
        return None
    strip = lambda a: a.lstrip("%")
    return {"kernel": "binary_const_kernel", "op": BINARY[op], "inputs": [strip(x_arg)], "output": strip(out_arg), "n": None,
            "n_const": None, "block": 1, "c": c, "flip": flip}


# --------------------------------------------------------------------------
# kernels bound by NAME: does the IR under that name do what the prebuilt kernel does?
# --------------------------------------------------------------------------
def _op_counts(ttir: str) -> dict:
    text = _strip_locs(ttir)
    ops = re.findall(r"=\s*\"?([a-z_]+\.[a-z_0-9.]+)", text) + re.findall(r"^\s*([a-z_]+\.[a-z_0-9.]+)", text, re.M)
    counts: dict = {}
    for o in ops:
        counts[o] = counts.get(o, 0) + 1
    return counts


def verify_named(name: str, ttir: str) -> dict | None:
    """A kernel whose NAME is in the prebuilt table still has to be that kernel: the reference generates code from
    the IR, so there a name carries no meaning, and a user's ``sin_kernel`` that computes a cosine, or upstream
    Triton's row-major ``matmul_kernel`` (same name and signature as the reference's tile-major one), must not run
    the prebuilt kernel silently.  Returns the IR match to bind by (elementwise, copy and reduction forms), or None
    to bind by name (the matmul and attention kernels, checked by a structural fingerprint); raises on a mismatch."""
    def bad(why):
        return RuntimeError(f"kernel '{name}' carries the name of a prebuilt gfx950 kernel but its IR does not match it "
                            f"({why}); this backend does no code generation, rename the kernel or use the reference's source")

    c = _op_counts(ttir)
    n = lambda op: c.get(op, 0)
    if name in ("add_kernel", "sin_kernel", "muladd_kernel", "unary_kernel", "binary_kernel", "cast_kernel",
                "binary_const_kernel", "copy_kernel", "empty_kernel", "reduce1d_kernel"):
        if name == "add_kernel" and n("scf.for") == 1:
            # the loop variant (01-vector-add.loop.py:30-62): two loads, one add, one store inside one loop
            if n("tt.load") == 2 and n("tt.store") == 1 and n("arith.addf") + n("arith.addi") >= 1 and n("tt.dot") == 0 \
                    and not any(k.startswith("math.") for k in c) and n("arith.mulf") == 0 and n("arith.subf") == 0:
                return None
            raise bad("a loop, but not two loads, one addition and one store")
        m = match_streaming(ttir) or match_reduce1d(ttir) or match_per_program(ttir) or match_empty(ttir)
        if m is None:
            raise bad("not a masked-block elementwise, copy, reduction or empty kernel of a supported operation")
        want = {"add_kernel": lambda m: (m["kernel"] == "binary_kernel" and m["op"] == "add") or m["kernel"] == "add_kernel",
                "sin_kernel": lambda m: m["kernel"] == "unary_kernel" and m["op"] == "sin",
                "muladd_kernel": lambda m: m["kernel"] == "muladd_kernel"}.get(name, lambda m: m["kernel"] == name)
        if not want(m):
            raise bad(f"the IR is a {m['kernel']}" + (f" computing {m['op']}" if m.get("op") else ""))
        # the three example kernels keep their own binders (argument order is theirs); the generic names bind by the IR
        return None if name in ("add_kernel", "sin_kernel", "muladd_kernel") else m
    # descriptor PARAMETERS: counted in the function header only (an op's result or operand type reads the same)
    plain = _strip_locs(ttir)
    head = plain[plain.find("tt.func"):]
    head = head[:head.find("\n")] if "\n" in head else head
    descs = len(re.findall(r"%[\w.]+\s*:\s*!tt\.tensordesc<", head))
    foreign = [k for k in c if k.startswith("math.")]
    if name in ("matmul_kernel_tma", "matmul_kernel_tma_fp8_scaled"):
        # no tt.trans: upstream Triton's tutorial kernel of the same name and signature loads B as [N, K] and
        # multiplies by its transpose; the reference took that transpose out (09-persistent-matmul.py:139) and the
        # prebuilt kernel computes A.B
        ok = (n("tt.dot") == 1 and n("tt.descriptor_load") == 2 and n("tt.descriptor_store") == 1 and descs == 3
              and n("tt.load") == 0 and n("tt.store") == 0 and not foreign and n("arith.addf") == 0
              and n("tt.trans") == 0 and n("arith.mulf") <= (2 if name.endswith("fp8_scaled") else 0))
        if not ok:
            raise bad("expected one tt.dot over two descriptor loads with B as [K, N] (no transpose), one descriptor "
                      "store and no epilogue")
    elif name == "matmul_kernel_fused":
        ok = (n("tt.dot") == 1 and n("tt.descriptor_load") in (2, 3) and n("tt.descriptor_store") == 1 and descs == 4
              and n("tt.load") == 0 and n("tt.store") == 0 and n("tt.trans") == 0
              and all(k in ("math.erf", "math.exp", "math.tanh") for k in foreign))
        if not ok:
            raise bad("expected one tt.dot with B as [K, N] (no transpose), a bias descriptor and one descriptor store")
    elif name == "matmul_kernel":
        body = _body(ttir)
        # the reference's kernel reads tile-major buffers and never uses the strides of its signature
        # (03-matrix-multiplication.py:251-253); upstream's row-major kernel of the same name multiplies by them
        unused = body is not None and all(not re.search(re.escape(a) + r"\b", "\n".join(body[2]))
                                          for a, t in body[1] if "stride" in a)
        ok = (n("tt.dot") == 1 and n("tt.load") == 2 and n("tt.store") == 1 and n("tt.descriptor_load") == 0 and descs == 0
              and n("arith.remsi") >= 2 and unused and not foreign)
        if not ok:
            raise bad("expected the tile-major pointer kernel: one tt.dot over two masked loads, offsets wrapped with "
                      "% M and % N, and the stride arguments unused")
    elif name == "_attn_fwd":
        d = n("tt.dot")
        ok = (d in (2, 4) and n("math.exp2") == d and n("math.log2") == 1 and n("tt.descriptor_load") == d + 1
              and n("tt.descriptor_store") == 1 and n("tt.store") == 1 and descs == 4 and n("tt.reduce") == d
              and set(foreign) <= {"math.exp2", "math.log2"})
        if not ok:
            raise bad("expected online-softmax attention: Q.K^T and P.V per stage, exp2, log2, M stored through a pointer")
    return None
