"""Build-time check of the hand-issued matrix instructions in the dK/dV kernel.

``bwd.hip`` issues the S and dO V^T products of ``bwd_dkv_kernel`` as inline assembly so that their results
land in vector registers (``mfma32_into_vgprs`` in ``csrc/common.h``).  The compiler does not know that such a
statement is a matrix instruction and inserts no wait states behind it, while the hardware needs 11 of them
between a 32x32x16 MFMA and any other access to its result (a chained accumulation into the same registers
excepted).  The kernel keeps that distance by construction; this module measures it in the generated assembly,
along every control-flow path, so that a compiler that schedules differently fails the build instead of
producing a kernel that reads registers too early.
"""

from __future__ import annotations

import re
import subprocess
from collections import deque

# wait states the hardware needs behind an 8-pass MFMA before another instruction may touch its result,
# plus a margin of one
MIN_DISTANCE = 12
_LOOKAHEAD = 24  # paths are followed this many instructions: anything later is far enough

_LABEL = re.compile(r"^([A-Za-z_.$][\w.$]*):")


def _vregs(text: str) -> set[int]:
    out: set[int] = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def _function(asm: str, symbol: str) -> list[str]:
    """Instruction and label lines of the first function whose (mangled) name contains `symbol`."""
    lines = asm.split("\n")
    start = None
    for i, l in enumerate(lines):
        m = _LABEL.match(l)
        if m and symbol in m.group(1) and not m.group(1).startswith(".L"):
            start = i + 1
            break
    if start is None:
        raise ValueError(f"no function containing {symbol!r} in the assembly")
    out = []
    for l in lines[start:]:
        t = l.split(";")[0].strip()
        if not t:
            continue
        m = _LABEL.match(t)
        if m:
            if m.group(1).startswith(".Lfunc_end"):
                break
            out.append(t)
        elif not t.startswith("."):  # directives are not instructions
            out.append(t)
    return out


def min_result_distance(asm: str, symbol: str) -> tuple[int, int, str]:
    """Smallest number of wait states (instructions, an `s_nop n` counting n + 1) between an MFMA with a
    vector-register destination in the function `symbol` and the first other instruction that reads or writes
    that destination, over all paths.

    Returns (distance, number of such MFMAs, description of the closest pair); distance is _LOOKAHEAD when
    nothing comes closer than that."""
    body = _function(asm, symbol)
    ins: list[str] = []
    labels: dict[str, int] = {}
    for t in body:
        m = _LABEL.match(t)
        if m:
            labels[m.group(1)] = len(ins)
        else:
            ins.append(t)

    def successors(i: int) -> list[int]:
        t = ins[i]
        op = t.split()[0]
        if op == "s_endpgm":
            return []
        if op == "s_branch":
            return [labels[t.split()[1]]]
        if op.startswith("s_cbranch"):
            return [i + 1, labels[t.split()[-1]]]
        return [i + 1]

    best, count, where = _LOOKAHEAD, 0, ""
    for i, t in enumerate(ins):
        if not t.startswith("v_mfma"):
            continue
        dst = t.split(None, 1)[1].split(",")[0].strip()
        if not dst.startswith("v["):
            continue
        count += 1
        d = _vregs(dst)
        seen = {}
        queue = deque((s, 0) for s in successors(i))
        while queue:
            j, gap = queue.popleft()
            if j >= len(ins) or gap >= _LOOKAHEAD or seen.get(j, _LOOKAHEAD + 1) <= gap:
                continue
            seen[j] = gap
            u = ins[j]
            if u.startswith("v_mfma") and u.split(None, 1)[1].split(",")[0].strip() == dst:
                continue  # chained into the same registers: ordered by the hardware
            if _vregs(u) & d:
                if gap < best:
                    best, where = gap, f"{t}  ->  {u}"
                continue
            cost = int(u.split()[1], 0) + 1 if u.startswith("s_nop") else 1  # s_nop n stands for n + 1 wait states
            for s in successors(j):
                queue.append((s, gap + cost))
    return best, count, where


def device_assembly(hipcc: str, flags: list[str], source: str) -> str:
    r = subprocess.run([hipcc, *flags, "-S", "--offload-device-only", source, "-o", "-"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {source}:\n{r.stderr[-4000:]}")
    return r.stdout


def dkv_kernel_symbols(asm: str) -> list[str]:
    """Names (up to the template arguments) of every instantiation of bwd_dkv_kernel in the assembly."""
    out = []
    for l in asm.split("\n"):
        m = _LABEL.match(l)
        if m and "bwd_dkv_kernel" in m.group(1) and not m.group(1).startswith(".L"):
            name = m.group(1)
            cut = name.find("EEEv")
            name = name[name.index("bwd_dkv_kernel"):cut if cut > 0 else len(name)]
            if name not in out:
                out.append(name)
    return out


def check_dkv_kernel(asm: str) -> str:
    """Raises if a hand-issued MFMA result of bwd_dkv_kernel is touched too early; returns a one-line report."""
    lines = []
    symbols = dkv_kernel_symbols(asm)
    if not symbols:
        raise RuntimeError("no bwd_dkv_kernel in the assembly (the check looks at nothing)")
    for sym in symbols:
        dist, count, where = min_result_distance(asm, sym)
        if count == 0:
            raise RuntimeError(f"{sym}: no MFMA with a vector-register destination found (the check looks at nothing)")
        if dist < MIN_DISTANCE:
            raise RuntimeError(f"{sym}: an MFMA result is touched {dist} instructions later, {MIN_DISTANCE} needed: {where}")
        lines.append(f"{sym}: {count} MFMAs, nearest use {'>=' if dist >= _LOOKAHEAD else ''}{dist} instructions later")
    return "; ".join(lines)
