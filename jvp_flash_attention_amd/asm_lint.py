"""Lint of the compiled kernels around their inline-asm matrix instructions.

The tuned kernels issue some ``v_mfma`` instructions through inline asm (result tile in ordinary
vector registers, B operand resident in the accumulation file).  The compiler schedules and
allocates registers around inline asm but does not look inside it, so it cannot add the idle issue
slots that the hardware needs

1. between a vector-ALU write to a register (for instance ``v_accvgpr_read_b32`` bringing back a
   value the allocator parked in the accumulation file) and a matrix instruction that reads it, and
2. between a matrix instruction and anything else that reads its result (a vector instruction reading a score
   tile, or ``v_accvgpr_read_b32`` reading an accumulator: the compiler may schedule the epilogue's reads in front
   of a wait that is not tied to the registers).

Likewise for the LDS reads issued through inline asm (``ds_read_b128``, ``ds_read_b64_tr_b16``): to the
compiler the destination holds its value as soon as the statement is over, while the hardware delivers it
some cycles later, and only the ``s_waitcnt lgkmcnt`` that the sources tie to the register (``lds_wait``)
says when.  Under register pressure the allocator has been seen to give several such reads one destination
and to copy each result away at once, in front of the wait: the copy holds whatever the register held before.

3. No instruction may read a register while an inline-asm LDS read into it is still in flight.

The forward kernels rescale and re-centre their accumulators in place with an asm statement that names the
accumulator elements as inputs and writes them all the same (``acc_move_in_place``: as in/out operands the
compiler gives the tiles a second home behind the rarely taken block and copies them there on every half
tile).  That is sound only while the registers the statement is handed are the very ones the in-place matrix
instructions (``mfma_acc``) accumulate into:

4. In a kernel that contains such a statement (an asm block with two ``v_accvgpr_write_b32``), the registers those
   blocks write must be exactly the destinations of the kernel's in-place inline-asm matrix instructions, and behind
   the first of those no ``v_accvgpr_mov_b32`` outside asm may read or write one of them (a copy would mean a
   second home; in front of it the compiler zeroes the tiles that way).

The sources provide those slots themselves (``s_nop 1`` in front of the matrix instructions whose
operands live long enough to be parked, ``tiles_ready()`` = ``s_nop 15; s_nop 3`` after each group).
A result also counts as written once two further 32x32 matrix instructions have been issued behind its
producer: the matrix pipe takes them one after another, each for its 8 or 16 passes, so the second cannot
start before the producer has been through (the one-pass backward reads its dq tile that way, with atomic
adds placed between the matrix instructions of the next phase).
``scan()`` checks the ISA text of a translation unit for both; ``build()`` runs it on every kernel unit it
compiles and fails on a finding.  ``python -m jvp_flash_attention_amd.asm_lint [unit names]`` compiles
units to ISA text on its own and scans them.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor



def _regs(tok: str) -> set[tuple[str, int]]:
    """Registers named by an operand: ('v', n) ordinary, ('a', n) accumulation file."""
    tok = tok.strip()
    m = re.fullmatch(r"([va])(\d+)", tok)
    if m:
        return {(m.group(1), int(m.group(2)))}
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), n) for n in range(int(m.group(2)), int(m.group(3)) + 1)}
    return set()


def scan(isa_text: str, where: str = "") -> list[str]:
    """Findings (one line each) in the ISA text of one translation unit."""
    out = []
    kern, inasm, hist, pending = "?", False, [], {}  # pending: register -> matrix instructions issued since
    flying: list[set] = []  # destinations of the inline-asm LDS reads in flight, oldest first
    # rule 4, per kernel: destinations of in-place asm matrix instructions, registers written by in-place-move
    # blocks, accumulation-file copies made by the compiler
    acc_dst, moved, copies, block_writes = set(), set(), [], []

    def rule4():
        if not moved:
            return
        if moved != acc_dst:
            extra, missing = sorted(moved - acc_dst), sorted(acc_dst - moved)
            out.append(f"{where} {kern}: in-place accumulator moves write a{[r[1] for r in extra]} outside, and miss "
                       f"a{[r[1] for r in missing]} of, the in-place matrix instructions' destinations")
        for line, regs in copies:
            if regs & acc_dst:
                out.append(f"{where} {kern}: '{line[:60]}' copies an accumulator that is also moved in place")

    for ln in isa_text.splitlines():
        t = ln.strip()
        if t.startswith("_Z") and ":" in t and "$" not in t.split(":")[0]:
            rule4()
            kern, hist, pending, flying = t.split(":")[0], [], {}, []
            acc_dst, moved, copies, block_writes = set(), set(), [], []
            continue
        if "ASMSTART" in t:
            inasm = True
            block_writes = []
            continue
        if "ASMEND" in t:
            inasm = False
            if len(block_writes) == 2:  # acc_move_in_place
                moved |= set(block_writes)
            continue
        if not t or t[0] in ";.":
            continue
        t = t.split(";")[0].strip()
        if not t:
            continue
        op = t.split()[0]
        ops = [x.strip() for x in t.split(None, 1)[1].split(",")] if " " in t else []
        if op == "v_accvgpr_write_b32" and inasm:
            block_writes += list(_regs(ops[0]))
        if op == "v_accvgpr_mov_b32" and not inasm and acc_dst:  # (before the first accumulation: the zeroing)
            copies.append((t, _regs(ops[0]) | _regs(ops[1])))
        if op == "s_nop" and ops and int(ops[0]) >= 15:
            pending = {}  # tiles_ready(): results of the group are readable from here on
        if op.startswith("ds_read") and inasm:
            flying.append(_regs(ops[0]))
            hist.append((op, ops))
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", t)
            if m:  # LDS reads return in order: the N youngest may still be in flight
                n = int(m.group(1))
                flying = flying[len(flying) - n:] if n and n < len(flying) else ([] if n == 0 else flying)
        elif flying and op.startswith(("v_", "ds_", "global_", "buffer_", "scratch_")):
            srcs = set()
            for o in (ops[1:] if op.startswith("v_") else ops):
                srcs |= _regs(o)
            if any(srcs & f for f in flying):
                out.append(f"{where} {kern}: '{t[:60]}' reads the destination of an LDS read that is still in flight")
        if op.startswith("v_mfma"):
            dst, srcs = _regs(ops[0]), set()
            for o in ops[1:4]:
                srcs |= _regs(o)
            if op.startswith("v_mfma_f32_32x32"):  # two younger ones: the producer has written its result
                pending = {r: n + 1 for r, n in pending.items() if n + 1 < 2}
            if inasm:
                guarded = bool(hist) and hist[-1][0] == "s_nop"
                if not guarded:
                    for pop, pops in hist[-2:]:
                        if pop.startswith("v_") and not pop.startswith("v_mfma") and pops and (_regs(pops[0]) & srcs):
                            out.append(f"{where} {kern}: '{pop} {pops[0]}' feeds '{t[:60]}' without idle slots")
                for r in dst:  # vector registers, and accumulation registers (read back by v_accvgpr_read)
                    pending[r] = 0
                if len(ops) >= 4 and ops[0] == ops[3] and ops[0].startswith("a"):
                    acc_dst |= dst  # accumulation in place (mfma_acc)
            else:
                for r in dst:
                    pending.pop(r, None)
        elif pending and op.startswith(("v_", "ds_write", "global_store", "buffer_store", "scratch_store", "global_atomic")):
            srcs = set()
            for o in (ops[1:] if op.startswith("v_") else ops):
                srcs |= _regs(o)
            if srcs & pending.keys():
                out.append(f"{where} {kern}: '{t[:60]}' reads a matrix result before the wait that follows its group")
        hist.append((op, ops))
    rule4()
    return out


def isa_of(unit) -> str:
    """Device ISA text of one translation unit of ``build.units()``."""
    from . import build as _build

    name, src, defs = unit
    with tempfile.TemporaryDirectory() as td:
        path = os.path.join(td, name + ".s")
        cmd = [_build.HIPCC, *_build.FLAGS, *defs, "-S", "--cuda-device-only", src, "-o", path]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc -S failed for {name}:\n{r.stderr[-4000:]}")
        with open(path) as f:
            return f.read()


def lint(names=None, jobs: int | None = None) -> list[str]:
    """Compile the named units (default: every kernel unit) to ISA and scan them."""
    from . import build as _build

    units = [u for u in _build.units() if u[0].startswith(("fwd_", "bwd_")) and (not names or u[0] in names)]
    with ThreadPoolExecutor(max_workers=jobs or min(8, os.cpu_count() or 1)) as ex:
        texts = list(ex.map(isa_of, units))
    findings = []
    for u, text in zip(units, texts):
        findings += scan(text, u[0])
    return findings


if __name__ == "__main__":
    found = lint(sys.argv[1:] or None)
    print("\n".join(found) if found else "asm lint: clean")
    sys.exit(1 if found else 0)
