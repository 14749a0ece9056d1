"""Checks the compiler's assembly of the HIP kernels for register spills that lose lanes.

The kernels of this package are allowed to spill a few vector registers in their tightest instances.  A spill store
writes the lanes that are active when it executes; the compiler places spill code per basic block and does not ask which
lanes are active there.  Two placements lose data silently:

* at the top of the block where divergent lanes rejoin, BEFORE the instruction that restores the exec mask
  (``s_or_b64 exec, exec, ...``): the store (or the reload) runs with the mask of the branch that was just left;
* a spill STORE anywhere between an instruction that narrows exec and the one that widens it again.

Both were seen with this compiler (the per-block, per-channel V scale instances at head_dim 256 wrote a wrong LSE for
the waves whose lanes had been masked off around a scale fetch).  The kernels avoid per-thread branches around their
global loads for that reason (they branch on the wave index, a scalar); this scan runs at build time over every kernel
and fails the build if such a placement appears again.
"""
from __future__ import annotations

import re
from typing import List

_LABEL = re.compile(r"^\.LBB\d+_\d+:")
_KERNEL = re.compile(r"^(_Z\w+):")
_BLOCK_END = re.compile(r"^\s+(s_cbranch\w*|s_branch|s_endpgm|s_setpc_b64)\b")
_EXEC_RESTORE = re.compile(r"^\s+(s_or_b64 exec, exec,|s_mov_b64 exec, -1)")
_EXEC_NARROW = re.compile(r"^\s+(s_and_saveexec_b64|s_or_saveexec_b64|s_and_b64 exec, exec,|s_andn2_b64 exec, exec,|s_xor_b64 exec, exec,)")
_SPILL = re.compile(r"^\s+(scratch_|buffer_)\w+.*Folded (Spill|Reload)")


def scan(asm: str) -> List[str]:
    """Returns one line per suspicious spill / reload in the assembly text of one translation unit."""
    findings: List[str] = []
    kernel = "?"
    block: List[tuple] = []          # (line number, text) of the current basic block
    narrowed_at = 0                    # line of the last exec-narrowing instruction not yet undone (linear order)

    def close_block():
        restore = next((i for i, (_, t) in enumerate(block) if _EXEC_RESTORE.match(t)), None)
        if restore is not None:
            for n, t in block[:restore]:
                if _SPILL.match(t):
                    findings.append(f"{kernel}: line {n}: `{t.strip()}` runs before exec is restored at line {block[restore][0]}")
        block.clear()

    for n, line in enumerate(asm.split("\n"), 1):
        m = _KERNEL.match(line)
        if m:
            close_block()
            kernel, narrowed_at = m.group(1), 0
            continue
        if _LABEL.match(line):
            close_block()
        block.append((n, line))
        if _EXEC_NARROW.match(line):
            narrowed_at = n
        elif _EXEC_RESTORE.match(line):
            narrowed_at = 0
        elif narrowed_at and _SPILL.match(line) and "Folded Spill" in line:
            findings.append(f"{kernel}: line {n}: `{line.strip()}` stores while exec is narrowed (since line {narrowed_at})")
        if _BLOCK_END.match(line):
            close_block()
            if line.split()[0] in ("s_endpgm", "s_setpc_b64"):
                narrowed_at = 0          # nothing falls through: what follows is reached by branches, each with its own mask
    close_block()
    return findings
