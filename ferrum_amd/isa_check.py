"""Build-time check of the hand-scheduled loads in this library's own kernels.

Three sources issue memory instructions through ``asm volatile`` that the compiler
cannot see the timing of:

* LDS-direct loads (``s_mov_b32 m0, <lds address>`` followed by
  ``global_load_lds_dwordx4``): the statement writes M0, which an asm statement cannot
  name as a clobber on this target.  The invariant is that the compiler keeps nothing of
  its own in M0 inside these kernels: every mention of M0 in a kernel's code must be one
  of these statements.
* register loads (``global_load_dwordx2/x4 vDST, vADDR, off`` in gemv_stream.hip): the
  destination registers hold the data only after the hand-placed ``s_waitcnt vmcnt(n)``
  that follows.  The invariant is that nothing between the load and that wait reads or
  writes the destination registers (no copy, no spill), and that the kernel has no
  scratch at all, so that no spill code can exist.
* ``s_waitcnt vmcnt(n)`` counts are the author's: they are right only if the compiler
  has put no vector-memory load of its own between the counted loads and the
  wait.  The check counts the vector-memory instructions outside asm statements between
  a hand-issued load and the hand-placed wait that covers it; there must be none, except
  stores behind LDS-direct loads, which can only lengthen the wait.

The check reads the assembly hipcc writes with ``-S`` for this library's own sources
(text, before it becomes a code object) and returns every violation it finds.  It is a
linear scan in program-text order, which is the order these straight-line stretches are
laid out in.  ``ferrum_amd.build.build`` runs it and refuses to produce a library when
it fails; the hipcc release the kernels were validated with is recorded in
``VALIDATED_HIPCC`` and any other release is reported.
"""
from __future__ import annotations

import re

# `hipcc --version` of the toolchain every kernel here was validated with on gfx950
VALIDATED_HIPCC = "7.2.26015"

CHECKED_SOURCES = ("gemm.hip", "gemv_stream.hip", "gemm_skinny.hip", "probe.hip")

_KERNEL_LABEL = re.compile(r"^(_Z\w+|\w+):\s*(;.*)?$")
_VREG_RANGE = re.compile(r"\bv\[(\d+):(\d+)\]")
_VREG_ONE = re.compile(r"\bv(\d+)\b")
_REG_LOAD = re.compile(r"^global_load_dwordx[234]\s+(v\[\d+:\d+\]|v\d+)\s*,")
_VMEM = re.compile(r"^(global_|buffer_|flat_|scratch_)(load|store|atomic)")
_STORE = re.compile(r"^(global_|buffer_|flat_)store")


def _vregs(text: str) -> set[int]:
    regs: set[int] = set()
    for lo, hi in _VREG_RANGE.findall(text):
        regs.update(range(int(lo), int(hi) + 1))
    for one in _VREG_ONE.findall(_VREG_RANGE.sub(" ", text)):
        regs.add(int(one))
    return regs


def _functions(asm: str):
    """Yields (name, [(line number, instruction text, inside an asm statement)]) per function."""
    name, body, in_asm = None, [], False
    for number, raw in enumerate(asm.splitlines(), 1):
        line = raw.strip()
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        if not line or line.startswith(";") or line.startswith("//"):
            continue
        if line.startswith(".Lfunc_end"):
            if name is not None:
                yield name, body
            name, body = None, []
            continue
        if line.startswith("."):
            continue
        label = _KERNEL_LABEL.match(line)
        if label and not line.startswith(".L"):
            name, body, in_asm = label.group(1), [], False
            continue
        if name is not None:
            body.append((number, line.split(";")[0].strip(), in_asm))


def violations(asm: str, source: str = "") -> list[str]:
    """Every break of the invariants in the module docstring found in `asm` (the text
    `hipcc -S --offload-device-only` writes for one source)."""
    found: list[str] = []
    where = (source + ":") if source else ""
    scratch = {}
    current = None
    for raw in asm.splitlines():
        line = raw.strip()
        if line.startswith(".amdhsa_kernel"):
            current = line.split()[1]
        elif line.startswith(".amdhsa_private_segment_fixed_size") and current:
            scratch[current] = int(line.split()[1])
    for name, body in _functions(asm):
        hand_loads = False
        for at, (number, text, in_asm) in enumerate(body):
            if not text:
                continue
            mentions_m0 = re.search(r"\bm0\b", text) is not None
            if mentions_m0:
                nxt = body[at + 1][1] if at + 1 < len(body) else ""
                nxt2 = body[at + 2][1] if at + 2 < len(body) else ""
                ours = in_asm and text.startswith("s_mov_b32 m0,") and (
                    nxt.startswith("global_load_lds_") or (nxt.startswith("s_nop") and nxt2.startswith("global_load_lds_")))
                if not ours:
                    found.append(f"{where}{number}: {name}: M0 is used outside an LDS-direct load statement: {text}")
            if in_asm and text.startswith("global_load_lds_"):
                hand_loads = True
                found.extend(_scan_to_wait(body, at, set(), name, where))
            match = _REG_LOAD.match(text) if in_asm else None
            if match:
                hand_loads = True
                found.extend(_scan_to_wait(body, at, _vregs(match.group(1)), name, where))
        if hand_loads and scratch.get(name, 0) != 0:
            found.append(f"{where}{name}: a kernel with hand-scheduled loads uses {scratch[name]} bytes of scratch")
    return found


def _scan_to_wait(body, at, dst: set[int], name: str, where: str) -> list[str]:
    found = []
    number0 = body[at][0]
    for number, text, in_asm in body[at + 1:]:
        if in_asm and text.startswith("s_waitcnt") and "vmcnt" in text:
            return found
        if text.startswith("s_endpgm") or text.startswith("s_setpc"):
            break
        if in_asm and (_REG_LOAD.match(text) or text.startswith("global_load_lds_") or text.startswith("s_mov_b32 m0,")
                       or text.startswith("s_nop")):
            # the following hand-issued loads of the same run; a destination may not be reused
            if dst and _REG_LOAD.match(text) and dst & _vregs(_REG_LOAD.match(text).group(1)):
                found.append(f"{where}{number}: {name}: a second load targets registers still in flight since line {number0}")
            continue
        if dst and dst & _vregs(text):
            found.append(f"{where}{number}: {name}: '{text}' touches registers loaded at line {number0} before the wait")
        # A store of the compiler's between an LDS-direct load and its wait can only lengthen the wait:
        # loads retire in order among themselves, so "at most n operations outstanding", n the later
        # loads, still means the awaited load has landed whether or not a store is among the n.
        if not dst and not in_asm and _STORE.match(text):
            continue
        if not in_asm and _VMEM.match(text):
            found.append(f"{where}{number}: {name}: the compiler's '{text.split()[0]}' sits between the load at line "
                         f"{number0} and its hand-counted wait")
    # no hand-placed wait follows: LDS-direct loads at the end of a kernel's text are waited
    # for by a later stretch the scan cannot order; register loads must always find theirs
    if dst:
        found.append(f"{where}{number0}: {name}: no hand-placed s_waitcnt vmcnt follows this register load")
    return found


def hipcc_release(version_text: str) -> str:
    match = re.search(r"HIP version:\s*([0-9.]+)", version_text)
    return match.group(1) if match else ""
