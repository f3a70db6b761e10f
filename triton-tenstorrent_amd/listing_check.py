"""Static checks of a gfx950 assembly listing around MFMAs issued from inline assembly: nothing but another MFMA
touches an MFMA's result too early, and no vector ALU result lands right in front of the MFMA that reads it.

The hot kernels issue their MFMAs from inline assembly (that is how the accumulators stay in AGPRs and a
direct-to-LDS copy rides behind an MFMA).  The compiler does not look inside such a statement, so it does not know
that the registers the statement writes are an MFMA's result, and it leaves none of the wait states that a VALU,
memory or export read (or a write) of an MFMA result needs: passes + 3 for an MFMA of `passes` passes (eleven for
v_mfma_f32_32x32x16_bf16).  Where the register allocator places a copy of such registers directly behind the
statement (a move of an accumulator tile to VGPRs for an epilogue, a copy between register sets where control flow
joins), the copy reads what the registers held before the MFMA and the kernel returns wrong values now and then.
The kernels leave idle states where they read results themselves; this check covers what the compiler adds, on the
listing of the very compilation that produced the code object, and the build fails if it finds anything.

    python -m triton_tenstorrent_amd.listing_check file.s
"""
from __future__ import annotations

import re
import sys

# passes of the MFMA forms the kernels use (an MFMA occupies the matrix pipe for four cycles a pass); any other
# form is taken at sixteen, the longest there is
PASSES = {"32x32x16_bf16": 8, "32x32x16_f16": 8, "16x16x32_bf16": 4, "16x16x32_f16": 4, "32x32x64_f8f6f4": 16,
          "16x16x128_f8f6f4": 8}

_RANGE = re.compile(r"^(v|a)\[(\d+):(\d+)\]$")
_ONE = re.compile(r"^-?\|?(v|a)(\d+)\|?$")
_KERNEL = re.compile(r"^([A-Za-z_]\w*):\s*(;.*)?$")
_LABEL = re.compile(r"^(\.LBB\w+):")


def _regs(tok: str) -> set[tuple[str, int]]:
    tok = tok.strip().rstrip(",")
    m = _RANGE.match(tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = _ONE.match(tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def passes(op: str) -> int:
    m = re.match(r"^v_mfma_[a-z0-9]+_(\w+)$", op)
    return PASSES.get(m.group(1), 16) if m else 16


def _states(op: str, ops: list[str]) -> int:
    if op == "s_nop":
        return int(ops[0], 0) + 1
    if op.startswith("v_mfma"):
        return passes(op)      # the next instruction issues when the pipe has taken this one
    return 1


def split_kernels(listing: str) -> dict[str, list[str]]:
    """The lines of each function of the listing, by name."""
    out: dict[str, list[str]] = {}
    cur = None
    for line in listing.split("\n"):
        m = _KERNEL.match(line)
        if m and not line.startswith(".L"):
            cur = m.group(1)
            out[cur] = []
        if cur is not None:
            out[cur].append(line)
        if line.startswith(".Lfunc_end"):
            cur = None
    return out


def mfma_result_hazards(lines: list[str]) -> list[str]:
    """One message per instruction that reads or writes an MFMA's destination registers within passes + 3 wait
    states behind it, along any path (both sides of a conditional branch are followed)."""
    ins: list[tuple[str, list[str], str]] = []
    label_at: dict[str, int] = {}
    for line in lines:
        m = _LABEL.match(line)
        if m:
            label_at[m.group(1)] = len(ins)
            continue
        if not line.startswith("\t"):
            continue
        text = line.strip()
        if not text or text[0] in ";.":
            continue
        parts = text.split(None, 1)
        ops = [o.strip().split(" ")[0] for o in parts[1].split(",")] if len(parts) > 1 else []
        ins.append((parts[0], ops, text))
    found: list[str] = []
    for i, (op, ops, text) in enumerate(ins):
        if not op.startswith("v_mfma"):
            continue
        dst = _regs(ops[0])
        window = passes(op) + 3
        best: dict[int, int] = {}
        stack = [(i + 1, 0)]
        while stack:
            k, st = stack.pop()
            while k < len(ins) and st < window:
                if best.get(k, window) <= st:
                    break
                best[k] = st
                op2, ops2, text2 = ins[k]
                if op2.startswith("v_mfma"):
                    # as the addend the result may be named again (the hardware orders that; the kernels keep chains
                    # apart themselves); as a multiplicand it is a read like any other
                    if (_regs(ops2[1]) | _regs(ops2[2])) & dst:
                        found.append(f"{st} states behind `{text}`: `{text2}`")
                    st += _states(op2, ops2)
                    k += 1
                    continue
                if op2 == "s_endpgm":
                    break
                if op2 == "s_branch":
                    k = label_at.get(ops2[0], len(ins))
                    st += 1
                    continue
                if op2.startswith("s_cbranch") and ops2 and ops2[0] in label_at:
                    stack.append((label_at[ops2[0]], st + 1))
                if not op2.startswith("s_"):
                    touched: set[tuple[str, int]] = set()
                    for o in ops2:
                        touched |= _regs(o)
                    if touched & dst:
                        found.append(f"{st} states behind `{text}`: `{text2}`")
                st += _states(op2, ops2)
                k += 1
    return found


def valu_writes_in_front_of_an_mfma(lines: list[str], states: int = 2) -> list[str]:
    """One message per vector ALU instruction (register-file copies v_accvgpr_read / _write / _mov above all) whose
    result an inline-assembly MFMA reads fewer than `states` wait states later (straight-line: such an instruction
    sits in the MFMA's own block).  The compiler moves operands between the register files where it likes, and in front
    of an inline-assembly MFMA it leaves no distance: the MFMA then read the register before the copy had arrived
    (attention, head dim 256: scores off by a few per cent, exact with one idle state in between; that kernel's MFMAs
    carry two).  Held for every vector ALU write, not only the copies it was seen with: the kernels that feed an MFMA
    from the ALU pad their MFMAs, the others feed theirs from LDS reads."""
    ins, in_asm = [], False
    for line in lines:
        if _LABEL.match(line):
            ins.append(None)       # a block boundary ends the look-back
            continue
        if "ASMSTART" in line or "ASMEND" in line:
            in_asm = "ASMSTART" in line
            continue
        if not line.startswith("\t"):
            continue
        text = line.strip()
        if not text or text[0] in ";.":
            continue
        parts = text.split(None, 1)
        ops = [o.strip().split(" ")[0] for o in parts[1].split(",")] if len(parts) > 1 else []
        ins.append((parts[0], ops, text, in_asm))
    found = []
    for i, cur in enumerate(ins):
        # (an MFMA that the compiler issued itself has the distance the hardware asks for)
        if cur is None or not cur[0].startswith("v_mfma") or not cur[3]:
            continue
        reads = set()
        for o in cur[1][1:]:
            reads |= _regs(o)
        st, k = 0, i - 1
        while k >= 0 and st < states and ins[k] is not None:
            op2, ops2, text2, _ = ins[k]
            if op2.startswith("v_") and not op2.startswith("v_mfma") and ops2 and _regs(ops2[0]) & reads:
                found.append(f"{st} states in front of `{cur[2]}`: `{text2}`")
            st += _states(op2, ops2)
            k -= 1
    return found


def vmcnt_waits_in_mfma_blocks(lines: list[str], min_mfma: int = 32) -> int:
    """Number of `s_waitcnt vmcnt(...)` that the compiler placed (outside inline assembly) in basic blocks with at
    least `min_mfma` MFMAs, i.e. in the K loops.  The kernels track their direct-to-LDS copies by hand; a wait the
    compiler adds there (it reloads a spilled register and waits for the reload with vmcnt(0)) also waits for every
    copy in flight and flattens the prefetch: not wrong, but 5-7 % slower where it happened."""
    count, block, in_asm = 0, [], False

    def close(block):
        if sum("v_mfma" in t for t, _ in block) < min_mfma:
            return 0
        return sum(1 for t, a in block if not a and re.search(r"s_waitcnt.*vmcnt\(", t))

    for line in lines:
        if _LABEL.match(line):
            count += close(block)
            block = []
        if "ASMSTART" in line:
            in_asm = True
        elif "ASMEND" in line:
            in_asm = False
        else:
            block.append((line, in_asm))
    return count + close(block)


def check_listing(listing: str) -> dict[str, list[str]]:
    """Kernel name -> hazards, for the kernels of the listing that have any."""
    out = {}
    for name, lines in split_kernels(listing).items():
        if any("v_mfma" in l for l in lines):
            h = mfma_result_hazards(lines) + valu_writes_in_front_of_an_mfma(lines)
            if h:
                out[name] = h
    return out


if __name__ == "__main__":
    bad = check_listing(open(sys.argv[1]).read())
    for name, h in bad.items():
        print(f"{name}: {len(h)}")
        for msg in h[:8]:
            print("   ", msg)
    sys.exit(1 if bad else 0)
