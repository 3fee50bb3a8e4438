"""Build-time check of the generated GCN assembly of the GEMM kernels.

The kernels issue global loads from inline assembly and wait for them by count (`s_waitcnt
vmcnt(N)`), so the compiler does not know when a load's destination registers become valid.  It
is free to copy or reuse such a register between the load and the wait - which reads a stale value
or, worse, lets the load land on an unrelated value such as an address.  This pass builds the
control-flow graph of every kernel, propagates "VGPR v is the destination of the p-th youngest
load in flight" to a fixed point (a wait for vmcnt(N) retires every load with p > N; where paths
join, the younger position wins), and reports any compiler-generated instruction that touches a
register whose load may still be in flight.

LDS reads issued from inline assembly (`ds_read_*`) are tracked the same way, more coarsely: their
destinations stay in flight until a wait for lgkmcnt(0).  (A destination that nothing reads any
more is the dangerous one: the compiler hands the register to another value at once, and the
read lands on it later.)

MFMAs issued from inline assembly hide a third hazard: the hardware does not interlock a matrix
instruction's result against vector instructions, the compiler normally pads with s_nop, and it
cannot see into inline assembly.  Compiler-generated accumulator moves (`v_accvgpr_*`) must
therefore not follow an inline-assembly MFMA that writes the same AGPR within `_MFMA_SETTLE` wait
states, nor write an AGPR that an inline-assembly MFMA reads within the next two.
"""
from __future__ import annotations

import re
from typing import Dict, List, Tuple

_LOAD = re.compile(r"^\s*global_load_(?:lds_)?dword(?:x2|x3|x4)?\s+v(?:\[(\d+):(\d+)\]|(\d+))\s*,")
_DSREAD = re.compile(r"^\s*ds_read\w*\s+v(?:\[(\d+):(\d+)\]|(\d+))\s*,")
_STORE = re.compile(r"^\s*global_(?:store|atomic)\w*\s")
_VMCNT = re.compile(r"vmcnt\((\d+)\)")
_VREG = re.compile(r"\bv(?:\[(\d+):(\d+)\]|(\d+))\b")
_FUNC = re.compile(r"^(_Z\w+):")
_LABEL = re.compile(r"^(\.LBB\w+):")
_BRANCH = re.compile(r"^\s*s_(c?branch)\w*\s+(\.LBB\w+)")


def _regs(m) -> range:
    if m.group(1) is not None:
        return range(int(m.group(1)), int(m.group(2)) + 1)
    return range(int(m.group(3)), int(m.group(3)) + 1)


class _Ins:
    __slots__ = ("kind", "regs", "n", "text", "line")

    def __init__(self, kind, regs, n, text, line):
        self.kind, self.regs, self.n, self.text, self.line = kind, regs, n, text, line


def _parse(lines: List[Tuple[int, str]]):
    """-> blocks: list of (label, [ins], successors-by-label, falls_through)"""
    blocks, cur, label, in_asm = [], [], "<entry>", False

    def close(succ, fall):
        nonlocal cur, label
        blocks.append([label, cur, succ, fall])
        cur, label = [], None

    for ln, raw in lines:
        s = raw.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = _LABEL.match(raw)
        if m:
            if label is not None:
                close([], True)
            label = m.group(1)
            continue
        code = raw.split(";")[0].strip()
        if not code or code.startswith("."):
            continue
        if label is None:
            label = "<anon%d>" % ln
        m = _BRANCH.match(code)
        if m:
            close([m.group(2)], m.group(1) == "cbranch")
            continue
        if code.startswith("s_endpgm"):
            close([], False)
            continue
        m = _LOAD.match(code)
        if m:
            regs = [] if "_lds_" in code else list(_regs(m))
            cur.append(_Ins("load", regs, 0, code, ln))
            continue
        if _STORE.match(code):
            cur.append(_Ins("load", [], 0, code, ln))  # stores count in vmcnt too: only makes waits conservative
            continue
        if in_asm:
            m = _DSREAD.match(code)
            if m:
                cur.append(_Ins("ldsread", list(_regs(m)), 0, code, ln))
                continue
        if code.startswith("s_waitcnt"):
            everything = re.match(r"s_waitcnt\s+(0|0x0)\s*$", code) is not None
            v = _VMCNT.search(code)
            if v is not None or everything:
                cur.append(_Ins("wait", [], 0 if everything else int(v.group(1)), code, ln))
            if everything or "lgkmcnt(0)" in code:
                cur.append(_Ins("ldswait", [], 0, code, ln))
            continue
        if in_asm:
            continue  # hand-written: assumed to respect the waits it places
        regs = [r for m in _VREG.finditer(code) for r in _regs(m)]
        if regs:
            cur.append(_Ins("use", regs, 0, code, ln))
    if label is not None:
        close([], False)
    return blocks


def _transfer(state: Dict[int, int], ins: List[_Ins], report=None) -> Dict[int, int]:
    """state: register -> position of its load among those in flight (1 = youngest); a register
    with an LDS read in flight is kept under the key -(register + 1)."""
    st = dict(state)
    for i in ins:
        if i.kind == "load":
            st = {r: (p + 1 if r >= 0 else p) for r, p in st.items()}
            for r in i.regs:
                st[r] = 1
        elif i.kind == "wait":
            st = {r: p for r, p in st.items() if r < 0 or p <= i.n}
        elif i.kind == "ldsread":
            for r in i.regs:
                st[-(r + 1)] = 0
        elif i.kind == "ldswait":
            st = {r: p for r, p in st.items() if r >= 0}
        elif report is not None:
            for r in i.regs:
                if r in st or -(r + 1) in st:
                    report(i, r)
                    break
    return st


_MFMA_SETTLE = 20  # wait states after which the result of the longest MFMA used here (8 passes) is readable
_MFMA = re.compile(r"^\s*v_mfma\w*\s+a\[(\d+):(\d+)\]\s*,(.*)$")
_AREG = re.compile(r"\ba(?:\[(\d+):(\d+)\]|(\d+))\b")
_NOP = re.compile(r"^\s*s_nop\s+(\d+)")


def _mfma_hazards(name: str, lines: List[Tuple[int, str]]) -> List[str]:
    """Textual (fall-through order) check of compiler-generated AGPR moves next to inline-assembly MFMAs."""
    seq, in_asm = [], False  # (line, code, in_asm)
    for ln, raw in lines:
        s = raw.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        code = raw.split(";")[0].strip()
        if not code or (code.startswith(".") and not code.endswith(":")):
            continue
        seq.append((ln, code, in_asm))  # (labels stay in the sequence: they delimit loops)
    out = []
    # A loop whose body holds inline-assembly MFMAs must not move accumulators at all: across the
    # back edge the MFMAs at the bottom of the body precede whatever stands at its top.  Blocks and
    # edges of the function; a branch back to a label closes a loop only if the branch can be
    # reached from that label (out-of-line blocks at the end of a function also jump backwards).
    starts = sorted({0} | {k for k, (_, c, _) in enumerate(seq) if c.endswith(":")}
                    | {k + 1 for k, (_, c, _) in enumerate(seq) if _BRANCH.match(c) or c.startswith("s_endpgm")})
    starts = [k for k in starts if k < len(seq)]
    block_of = {}
    for bi, k0 in enumerate(starts):
        for k in range(k0, starts[bi + 1] if bi + 1 < len(starts) else len(seq)):
            block_of[k] = bi
    label_block = {c[:-1]: block_of[k] for k, (_, c, _) in enumerate(seq) if c.endswith(":")}
    succ = [set() for _ in starts]
    for bi, k0 in enumerate(starts):
        k1 = (starts[bi + 1] if bi + 1 < len(starts) else len(seq)) - 1
        last = seq[k1][1]
        m = _BRANCH.match(last)
        if m and m.group(2) in label_block:
            succ[bi].add(label_block[m.group(2)])
        if not last.startswith("s_endpgm") and not (m and m.group(1) == "branch") and bi + 1 < len(starts):
            succ[bi].add(bi + 1)

    def reach(src, edges):
        seen, work = {src}, [src]
        while work:
            for nb in edges[work.pop()]:
                if nb not in seen:
                    seen.add(nb)
                    work.append(nb)
        return seen

    pred = [set() for _ in starts]
    for bi, ss in enumerate(succ):
        for t in ss:
            pred[t].add(bi)
    for bi in range(len(starts)):
        for h in succ[bi]:
            if h > bi or bi not in reach(h, succ):
                continue  # not a back edge of a loop
            body = reach(h, succ) & reach(bi, pred)
            ks = [k for k in range(len(seq)) if block_of[k] in body]
            if any(seq[k][2] and _MFMA.match(seq[k][1]) for k in ks):
                for k in ks:
                    bl, bc, ba = seq[k]
                    if not ba and bc.startswith("v_accvgpr"):
                        out.append("%s: line %d moves an accumulator inside a loop of inline-assembly MFMAs: %s"
                                   % (name, bl, bc))
    for k, (ln, code, asm) in enumerate(seq):
        if asm or not code.startswith("v_accvgpr"):
            continue
        mine = {r for m in _AREG.finditer(code) for r in _regs(m)}
        waited, j = 0, k - 1
        while j >= 0 and waited < _MFMA_SETTLE:
            pl, pc, pasm = seq[j]
            if pc.startswith("s_branch") or pc.startswith("s_endpgm"):
                break  # not reached from the text above
            m = _MFMA.match(pc) if pasm else None
            if m and mine & set(range(int(m.group(1)), int(m.group(2)) + 1)):
                out.append("%s: line %d moves an accumulator %d wait states after the MFMA of line %d wrote it: %s"
                           % (name, ln, waited, pl, code))
                break
            n = _NOP.match(pc)
            if not pc.endswith(":"):
                waited += int(n.group(1)) + 1 if n else 1
            j -= 1
        if code.startswith("v_accvgpr_write") or code.startswith("v_accvgpr_mov"):
            dst = next(iter(_regs(_AREG.search(code))))
            for pl, pc, pasm in [x for x in seq[k + 1:k + 6] if not x[1].endswith(":")][:2]:
                m = _MFMA.match(pc) if pasm else None
                if m and dst in {r for a in _AREG.finditer(m.group(3)) for r in _regs(a)}:
                    out.append("%s: line %d writes a%d right before the MFMA of line %d reads it: %s"
                               % (name, ln, dst, pl, code))
                    break
    return out


def lint(asm_text: str, only_if_name_has: str = "kernel") -> List[str]:
    """Returns one message per violation (empty list: clean)."""
    out: List[str] = []
    funcs, cur, name = [], [], None
    for ln, raw in enumerate(asm_text.split("\n"), 1):
        m = _FUNC.match(raw)
        if m:
            name, cur = m.group(1), []
            continue
        if raw.startswith(".Lfunc_end"):
            if name is not None and only_if_name_has in name:
                funcs.append((name, cur))
            name = None
            continue
        if name is not None:
            cur.append((ln, raw))
    for name, lines in funcs:
        out.extend(_mfma_hazards(name, lines))
        blocks = _parse(lines)
        index = {b[0]: k for k, b in enumerate(blocks)}
        entry: List[Dict[int, int]] = [None] * len(blocks)  # type: ignore
        entry[0] = {}
        work = [0]
        while work:
            k = work.pop()
            label, ins, succ, fall = blocks[k]
            st = _transfer(entry[k], ins)
            nxt = [index[s] for s in succ if s in index]
            if fall and k + 1 < len(blocks):
                nxt.append(k + 1)
            for j in nxt:
                if entry[j] is None:
                    entry[j] = dict(st)
                    work.append(j)
                else:
                    merged, changed = entry[j], False
                    for r, p in st.items():
                        if r not in merged or p < merged[r]:
                            merged[r] = p
                            changed = True
                    if changed:
                        work.append(j)
        for k, (label, ins, succ, fall) in enumerate(blocks):
            if entry[k] is None:
                continue
            _transfer(entry[k], ins, lambda i, r: out.append(
                "%s: line %d touches v%d while a load into it may be in flight: %s" % (name, i.line, r, i.text)))
    return out
