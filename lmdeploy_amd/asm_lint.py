"""Build-time check of the generated GCN assembly of the GEMM kernels.

The kernels issue global loads from inline assembly and wait for them by count (`s_waitcnt
vmcnt(N)`), so the compiler does not know when a load's destination registers become valid.  It
is free to copy or reuse such a register between the load and the wait - which reads a stale value
or, worse, lets the load land on an unrelated value such as an address.  This pass builds the
control-flow graph of every kernel, propagates "VGPR v is the destination of the p-th youngest
load in flight" to a fixed point (a wait for vmcnt(N) retires every load with p > N; where paths
join, the younger position wins), and reports any compiler-generated instruction that touches a
register whose load may still be in flight.
"""
from __future__ import annotations

import re
from typing import Dict, List, Tuple

_LOAD = re.compile(r"^\s*global_load_(?:lds_)?dword(?:x2|x3|x4)?\s+v(?:\[(\d+):(\d+)\]|(\d+))\s*,")
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
        if code.startswith("s_waitcnt"):
            v = _VMCNT.search(code)
            if v is not None:
                cur.append(_Ins("wait", [], int(v.group(1)), code, ln))
            elif re.match(r"s_waitcnt\s+(0|0x0)\s*$", code):
                cur.append(_Ins("wait", [], 0, code, ln))
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
    st = dict(state)
    for i in ins:
        if i.kind == "load":
            st = {r: p + 1 for r, p in st.items()}
            for r in i.regs:
                st[r] = 1
        elif i.kind == "wait":
            st = {r: p for r, p in st.items() if p <= i.n}
        elif report is not None:
            for r in i.regs:
                if r in st:
                    report(i, r)
                    break
    return st


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
