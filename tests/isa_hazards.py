"""Reads gfx950 assembly text and reports reads of an MFMA result that come too early.

The score MFMAs of the attention kernels are inline assembly with an ordinary VGPR tuple as
destination.  The compiler inserts the wait states a VALU / memory read of an MFMA result needs
only for MFMAs it knows; for the assembly ones the source has to keep the distance itself, and a
register copy the compiler places on its own can break it without any warning.  This checker walks
the emitted assembly in program order and, for every MFMA whose destination is a VGPR tuple,
counts wait states until something other than an MFMA accumulating into the very same tuple
touches one of its registers.

Wait states: one per instruction, n + 1 for `s_nop n`, and 8 for an MFMA in between (a 32x32x16
MFMA is 8 passes on gfx950, and the matrix pipe runs a wave's MFMAs in order, one behind the
other).  A result may be read or overwritten 12 wait states after its MFMA: the distance the
compiler's own hazard recogniser keeps on this target between such an MFMA and a
`v_accvgpr_read` of its result (it pads with `s_nop` up to exactly that).  MFMAs the compiler
knows are walked as well: the reader may be assembly (`v_accvgpr_read` of O in the epilogues).
"""
from __future__ import annotations

import re
from dataclasses import dataclass

_MFMA = re.compile(r"^\s*v_mfma_\w+\s+(v|a)\[(\d+):(\d+)\]\s*,(.*)$")
_REG_RANGE = re.compile(r"\b([va])\[(\d+):(\d+)\]")
_REG_ONE = re.compile(r"\b([va])(\d+)\b")
_NOP = re.compile(r"^\s*s_nop\s+(\d+)")


def _vgprs(text: str) -> set:
    """The vector registers an instruction names: ("v", n) ordinary, ("a", n) accumulation."""
    regs: set = set()
    for c, a, b in _REG_RANGE.findall(text):
        regs.update((c, i) for i in range(int(a), int(b) + 1))
    for c, a in _REG_ONE.findall(_REG_RANGE.sub(" ", text)):
        regs.add((c, int(a)))
    return regs


def _tuple(cls: str, lo: str, hi: str) -> set:
    return {(cls, i) for i in range(int(lo), int(hi) + 1)}


@dataclass
class Finding:
    function: str
    line_no: int
    mfma: str
    reader: str
    wait_states: dict

    def __str__(self):
        return (f"{self.function}: line {self.line_no}: `{self.reader.strip()}` touches the result of "
                f"`{self.mfma.strip()}` after {self.wait_states} wait states (passes: have)")


def _parse(asm_text: str):
    """Per function: the list of ("label", name, line number) and ("ins", text, line number) entries in order."""
    funcs: dict[str, list] = {}
    cur = None
    for no, raw in enumerate(asm_text.splitlines(), 1):
        line = raw.split(";", 1)[0].rstrip()
        s = line.strip()
        if not s:
            continue
        if not line.startswith((" ", "\t")) and s.endswith(":"):
            name = s[:-1]
            if name.startswith(".L"):
                if cur is not None:
                    funcs[cur].append(("label", name, no))
            else:
                cur = name
                funcs[cur] = []
            continue
        if s.startswith(".") or cur is None:
            continue
        funcs[cur].append(("ins", line, no))
    return funcs


_LIMIT = {8: 12}   # MFMA passes -> wait states before its result may be read or overwritten
_BRANCH = re.compile(r"^\s*s_(c?branch\w*)\s+(\.L\w+)")


def _walk(items, labels, pos, dest, have, mfma_line, func, findings, seen):
    """Follows program order from items[pos] (both ways at a conditional branch) until the distance is safe."""
    while pos < len(items):
        if all(have[p] >= _LIMIT[p] for p in have):
            return
        key = (pos, have[8])
        if key in seen:
            return
        seen.add(key)
        kind, text, no = items[pos]
        pos += 1
        if kind == "label":
            continue
        s = text.strip()
        if s.startswith("s_endpgm"):
            return
        br = _BRANCH.match(text)
        if br:
            target = labels.get(br.group(2))
            nxt = {p: have[p] + 1 for p in have}
            if target is not None:
                _walk(items, labels, target, dest, dict(nxt), mfma_line, func, findings, seen)
            if br.group(1) == "branch":
                return
            have = nxt
            continue
        nop = _NOP.match(text)
        if nop:
            have = {p: have[p] + int(nop.group(1)) + 1 for p in have}
            continue
        m2 = _MFMA.match(text)
        if m2:
            ab, c = m2.group(4).rsplit(",", 1)
            same = _tuple(m2.group(1), m2.group(2), m2.group(3)) == dest
            if same and not (_vgprs(ab) & dest) and _vgprs(c) in (dest, set()):
                return   # accumulates into (or restarts) the same tuple: back to back is fine, and it has its own turn
            if _vgprs(text) & dest:
                findings.append(Finding(func, no, mfma_line, text, dict(have)))
                return
            have = {p: have[p] + p for p in have}
            continue
        if _vgprs(text) & dest:
            findings.append(Finding(func, no, mfma_line, text, dict(have)))
            return
        have = {p: have[p] + 1 for p in have}


def check(asm_text: str, only_functions: str | None = None, all_mfmas: bool = True) -> list[Finding]:
    findings: list[Finding] = []
    for func, items in _parse(asm_text).items():
        if only_functions is not None and not re.search(only_functions, func):
            continue
        labels = {text: i for i, (kind, text, _) in enumerate(items) if kind == "label"}
        for i, (kind, text, no) in enumerate(items):
            m = _MFMA.match(text) if kind == "ins" else None
            if not m or (m.group(1) != "v" and not all_mfmas):
                continue
            dest = _tuple(m.group(1), m.group(2), m.group(3))
            _walk(items, labels, i + 1, dest, {8: 0}, text, func, findings, set())
    return findings


def count_vgpr_mfmas(asm_text: str, only_functions: str | None = None) -> int:
    n = 0
    for func, items in _parse(asm_text).items():
        if only_functions is None or re.search(only_functions, func):
            n += sum(1 for kind, text, _ in items if kind == "ins" and (m := _MFMA.match(text)) and m.group(1) == "v")
    return n
