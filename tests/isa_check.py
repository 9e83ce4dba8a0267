"""Static check of gfx950 assembly for reads of registers whose load is still in flight.

The streaming kernel issues its vector-memory loads from inline assembly and waits for
them with hand-counted `s_waitcnt vmcnt(N)`.  The compiler does not know those registers
are pending, so a copy, spill or reuse it inserts between a load and the wait that covers
it would silently read or clobber garbage.  This walks every path of a kernel's control-flow
graph with the hardware's rule (vector-memory operations retire in order; after
`vmcnt(N)` only the N youngest can still be outstanding) and reports every instruction
that touches the destination of an outstanding load.
"""
from __future__ import annotations

import re
from typing import Dict, List, Optional, Tuple

_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_FUNC = re.compile(r"^(_Z\w+):")
_VREG_RANGE = re.compile(r"\bv\[(\d+):(\d+)\]")
_VREG = re.compile(r"\bv(\d+)\b")
_VMCNT = re.compile(r"vmcnt\((\d+)\)")
_VMEM_PREFIXES = ("global_load", "global_store", "global_atomic", "buffer_load", "buffer_store", "buffer_atomic",
                  "scratch_load", "scratch_store", "flat_load", "flat_store", "flat_atomic")


def _regs(text: str) -> set:
    out = set()
    for a, b in _VREG_RANGE.findall(text):
        out.update(range(int(a), int(b) + 1))
    for a in _VREG.findall(_VREG_RANGE.sub(" ", text)):
        out.add(int(a))
    return out


class Inst:
    __slots__ = ("line", "text", "mnemonic", "is_vmem", "dest", "touched", "vmcnt", "target", "kind")

    def __init__(self, line: int, text: str):
        self.line, self.text = line, text
        body = text.split(";")[0].strip()
        parts = body.split(None, 1)
        self.mnemonic = parts[0]
        ops = parts[1] if len(parts) > 1 else ""
        self.is_vmem = self.mnemonic.startswith(_VMEM_PREFIXES)
        self.dest = frozenset()
        if self.is_vmem and "_load" in self.mnemonic and "_lds_" not in self.mnemonic:
            first = ops.split(",")[0]
            self.dest = frozenset(_regs(first))
        self.touched = frozenset(_regs(ops))
        m = _VMCNT.search(body) if self.mnemonic == "s_waitcnt" else None
        self.vmcnt = int(m.group(1)) if m else None
        self.target = None
        self.kind = "plain"
        if self.mnemonic == "s_branch":
            self.kind, self.target = "jump", ops.strip()
        elif self.mnemonic.startswith("s_cbranch"):
            self.kind, self.target = "cond", ops.strip()
        elif self.mnemonic == "s_endpgm":
            self.kind = "end"


def split_kernels(asm: str) -> Dict[str, List[str]]:
    kernels, name, cur = {}, None, []
    for raw in asm.split("\n"):
        m = _FUNC.match(raw)
        if m:
            if name:
                kernels[name] = cur
            name, cur = m.group(1), []
            continue
        if name is not None:
            if raw.startswith(".Lfunc_end"):
                kernels[name] = cur
                name, cur = None, []
            else:
                cur.append(raw)
    if name:
        kernels[name] = cur
    return kernels


def check_kernel(lines: List[str], max_states: int = 200000) -> List[str]:
    """Returns a list of hazard descriptions (empty = clean)."""
    insts: List[Inst] = []
    label_at: Dict[str, int] = {}
    for n, raw in enumerate(lines):
        m = _LABEL.match(raw)
        if m:
            label_at[m.group(1)] = len(insts)
            continue
        t = raw.strip()
        if not t or t.startswith((";", ".")) or not raw.startswith("\t"):
            continue
        insts.append(Inst(n, t))
    hazards: Dict[Tuple[int, int], str] = {}
    # state: tuple of destination sets (frozenset, line) of outstanding vector-memory ops, oldest first
    start: Tuple = ()
    seen = set()
    work: List[Tuple[int, Tuple]] = [(0, start)]
    while work:
        pc, state = work.pop()
        while pc < len(insts):
            key = (pc, state)
            if key in seen:
                break
            seen.add(key)
            if len(seen) > max_states:
                raise RuntimeError("state explosion in isa_check")
            ins = insts[pc]
            if ins.vmcnt is not None:
                n = ins.vmcnt
                state = state[len(state) - n:] if n < len(state) else state
                if n == 0:
                    state = ()
            else:
                for dest, where in state:
                    if dest and (dest & ins.touched):
                        hazards.setdefault((where, ins.line),
                                           f"line {ins.line}: `{ins.text}` touches v{sorted(dest & ins.touched)} "
                                           f"while the load at line {where} may be outstanding")
                if ins.is_vmem:
                    state = state + ((ins.dest, ins.line if ins.dest else 0),)
                    if len(state) > 64:  # vmcnt is a 6-bit counter; the hardware stalls the issue beyond it
                        state = state[-64:]
            # operations older than the oldest outstanding load cannot matter any more
            first = next((i for i, (d, _) in enumerate(state) if d), len(state))
            state = state[first:]
            if ins.kind == "end":
                break
            if ins.kind == "jump":
                pc = label_at[ins.target]
                continue
            if ins.kind == "cond":
                work.append((label_at[ins.target], state))
            pc += 1
    return [hazards[k] for k in sorted(hazards)]


def check_asm(asm: str, name_filter: Optional[str] = None) -> Dict[str, List[str]]:
    out = {}
    for name, lines in split_kernels(asm).items():
        if name_filter and name_filter not in name:
            continue
        out[name] = check_kernel(lines)
    return out
