"""Checks the gfx950 assembly of kernels that keep loads in flight behind hand-placed waits (stream_kernel.hpp).

The compiler takes the result of an inline-assembly load for present as soon as the statement has run.  The kernels
rely on every such register staying untouched until an `s_waitcnt vmcnt(n)` that covers the load; a register copy,
a spill or a reuse in between reads stale data or -- when the late data lands in a register that meanwhile holds an
address -- sends a later access astray.  This pass walks each kernel's instructions in program order, keeps the queue
of outstanding vector-memory loads (they return in order), retires all but the last n at every vmcnt(n), and reports
any instruction that reads or writes a register of a load still in the queue.  Branches are not followed: the kernels'
loads and waits sit in straight-line code, and the walk restarts its queue at every label that a backward branch
targets, so loops are neither mis-tracked nor checked.
"""
from __future__ import annotations

import re
from typing import Dict, List, Tuple

_REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
_LOAD = re.compile(r"^\s*(global_load_\w+|buffer_load_\w+|flat_load_\w+)\s+(v\d+|v\[\d+:\d+\])")
_VMCNT = re.compile(r"s_waitcnt\s+.*vmcnt\((\d+)\)")
_LABEL = re.compile(r"^([.\w$]+):")
_BRANCH = re.compile(r"^\s*s_c?branch\w*\s+([.\w$]+)")


def _regs(text: str) -> set:
    out = set()
    for m in _REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def lint(asm: str, kernel_substring: str) -> List[str]:
    """Violations found in the kernels of `asm` (text of a .s file) whose symbol contains `kernel_substring`."""
    problems: List[str] = []
    lines = asm.splitlines()
    # kernel bodies: from "<symbol>:" to "s_endpgm" ... up to the next ".Lfunc_end"
    starts = [i for i, l in enumerate(lines) if _LABEL.match(l) and kernel_substring in l and not l.startswith(".L")]
    for start in starts:
        name = lines[start].rstrip(":")
        end = next((i for i in range(start, len(lines)) if lines[i].startswith(".Lfunc_end")), len(lines))
        body = lines[start + 1:end]
        labels = {m.group(1): i for i, l in enumerate(body) if (m := _LABEL.match(l))}
        loop_heads = set()
        for i, l in enumerate(body):
            b = _BRANCH.match(l)
            if b and b.group(1) in labels and labels[b.group(1)] <= i:
                loop_heads.add(labels[b.group(1)])
        queue: List[Tuple[int, set, str]] = []  # (line, destination registers, text)
        for i, raw in enumerate(body):
            l = raw.split(";")[0].strip()
            if not l or l.startswith("."):
                if i in loop_heads:
                    queue.clear()
                continue
            if _LABEL.match(l):
                if i in loop_heads:
                    queue.clear()
                continue
            w = _VMCNT.search(l)
            if w:
                keep = int(w.group(1))
                queue = queue[len(queue) - keep:] if keep < len(queue) else queue
                if keep == 0:
                    queue = []
                continue
            used = _regs(l)
            ld = _LOAD.match(l)
            for at, dest, text in queue:
                hit = used & dest
                if hit:
                    problems.append(f"{name}: '{l}' touches v{sorted(hit)[0]} while '{text}' (instruction {at}) is still in flight")
                    break
            if ld:
                queue.append((i, _regs(ld.group(2)), l))
            elif l.startswith(("global_store", "buffer_store", "flat_store", "global_atomic", "buffer_atomic", "flat_atomic")):
                queue.append((i, set(), l))  # counted by vmcnt on this target, no destination to protect
    return problems


if __name__ == "__main__":
    import sys

    found = lint(open(sys.argv[1]).read(), sys.argv[2] if len(sys.argv) > 2 else "gemv_stream_kernel")
    print("\n".join(found) if found else "clean")
    sys.exit(1 if found else 0)
