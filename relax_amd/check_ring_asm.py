"""Build-time check of the generated code of ``csrc/q4g32_gemv_list.hip`` and ``csrc/q4g32_batch_list.hip``.

The compute wavefronts of those kernels load their weight stream with inline-assembly loads into a
ring of registers and wait for them by hand, so the compiler does not know that those registers are
in flight between a load and its wait.  The source makes every read of a ring register an asm
statement that depends on the wait; what is left to chance is register allocation (a copy or a
spill of a ring register inserted between load and wait would read it too early).  This script
compiles the file to assembly and verifies, in the kernel's text, that

* every ring register (destination of a ``global_load_* ... nt`` or ``buffer_load_* ... nt`` instruction) is read only by the
  instructions the source uses for it (``v_and_or_b32``, ``v_lshrrev_b32 .., 8 | 16, ..``, ``v_cvt_f32_f16``,
  and the cross-lane ``v_mov_b32_dpp`` of the batch kernel's lane exchange, which the compiler never
  generates by itself), never by a plain move, a store or anything else, and
* each ring slot keeps one register in the prologue and in the loop (no renaming copies).

What the text cannot show is a slot abandoned on the way out of the loop: its load is still in flight, and
a register the compiler reuses behind the loop would receive the data on top of its new value.  The
sources therefore wait for all loads (``s_waitcnt vmcnt(0)``) where the ring's loop ends.

Registers that the compiler also uses for short-lived temporaries while a slot is empty are
recognised by being written by another instruction first.

Kernels with such a ring must also be free of register spills (no ``scratch_*`` instruction).

A second check (``check_asm_results``) covers what inline assembly costs besides: the compiler does
not keep the hardware's wait states between an inline-assembly VALU result and an MFMA or DPP
instruction that reads it.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ("q4g32_gemv_list.hip", "q4g32_batch_list.hip")
ALLOWED_READERS = ("v_and_or_b32", "v_lshrrev_b32", "v_cvt_f32_f16", "v_mov_b32_dpp")


def _is_ring_load(l: str) -> bool:
    """A load of the weight stream: the only non-temporal loads of these kernels."""
    return l.startswith(("global_load_", "buffer_load_")) and l.endswith(" nt")


def _regs(tok: str):
    """'v[4:7]' -> {4,5,6,7}; 'v12' -> {12}; anything else -> empty."""
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"v(\d+)", tok)
    return {int(m.group(1))} if m else set()


def _check_function(body: list[str]) -> list[str]:
    errors = []
    ring = set()
    for l in body:
        if _is_ring_load(l):
            ring |= _regs(l.split()[1].rstrip(","))
    if not ring:
        return []
    # walk the text; a ring register is "loaded" after a ring load wrote it and until something else writes it
    loaded = set()
    for l in body:
        parts = l.replace(",", " ").split()
        op, ops = parts[0], parts[1:]
        if _is_ring_load(l):
            loaded |= _regs(ops[0])
            continue
        if not ops:
            continue
        stores = ("global_store", "ds_write", "buffer_store", "scratch_store", "global_atomic", "ds_add")
        writes = _regs(ops[0]) if not op.startswith(("s_",) + stores) else set()
        reads = set()
        for t in (ops if not writes else ops[1:]):
            reads |= _regs(t)
        if op.startswith(stores):
            reads |= _regs(ops[0])
        hit = reads & loaded
        if hit and not op.startswith(ALLOWED_READERS):
            errors.append(f"ring register(s) {sorted(hit)} read by `{l}`")
        if op.startswith("v_lshrrev_b32") and hit and ops[1] not in ("8", "16"):
            errors.append(f"unexpected shift of a ring register: `{l}`")
        loaded -= writes  # now a temporary of the compiler
    return errors


HAZARD_WINDOW = 3  # instructions: the hardware wants up to 2 wait states, one instruction may be a zero-cycle s_nop


def check_asm_results(asm_text: str) -> list[str]:
    """The compiler inserts the wait states between a VALU result and an MFMA or DPP instruction that reads it
    only when it issued the VALU instruction itself: the text of an inline-assembly statement is opaque to its
    hazard recognizer.  So no register written inside an ASMSTART / ASMEND block may be read by a v_mfma* or
    *_dpp instruction within the next HAZARD_WINDOW instructions, unless an s_nop of the block itself follows
    the write (loads are exempt: their results are waited for with s_waitcnt)."""
    errors = []
    recent = []  # (instructions ago, set of registers) written by inline assembly
    in_asm = False
    for raw in asm_text.splitlines():
        t = raw.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        l = t.split(";")[0].strip()
        if not l or l.startswith(".") or l.endswith(":"):
            if l.endswith(":") and not l.startswith("."):
                recent = []
            continue
        parts = l.replace(",", " ").split()
        op, ops = parts[0], parts[1:]
        if in_asm and op.startswith("s_nop"):
            recent = []  # the statement brings its own wait states
            continue
        reads_all = set()
        for tok in ops[1:] if ops else []:
            reads_all |= _regs(tok)
        if (op.startswith("v_mfma") or op.endswith("_dpp") or "_dpp " in l) and not in_asm:
            for age, regs in recent:
                hit = regs & (reads_all | (_regs(ops[0]) if op.endswith("_dpp") else set()))
                if hit:
                    errors.append(f"`{l}` reads v{sorted(hit)} written by inline assembly {age} instruction(s) before")
        recent = [(a + 1, r) for a, r in recent if a + 1 < HAZARD_WINDOW]
        if in_asm and ops and op.startswith("v_") and not op.startswith("v_cmp"):
            recent.append((0, _regs(ops[0])))
    return errors


def check(asm_text: str) -> list[str]:
    """Checks every kernel of the file on its own (register names mean nothing across kernels)."""
    lines = [l.split(";")[0].strip() for l in asm_text.splitlines()]
    functions, cur = [], None
    for l in lines:
        if not l:
            continue
        if l.endswith(":") and not l.startswith("."):  # a function label
            cur = []
            functions.append(cur)
        elif l.startswith(".Lfunc_end"):
            cur = None
        elif cur is not None and not l.startswith(".") and not l.endswith(":"):
            cur.append(l)
    errors, with_ring = [], 0
    for body in functions:
        if any(_is_ring_load(l) for l in body):
            with_ring += 1
            errors += _check_function(body)
            # These kernels are written to fit their register budget.  A spill anywhere in them (also in a service
            # wavefront's path: one extra branch there once sent 64 load registers through scratch memory and
            # cost the 4-linear step 3 of 21 us) is a regression the tests do not show.
            spills = [l for l in body if l.startswith(("scratch_load", "scratch_store"))]
            if spills:
                errors.append(f"{len(spills)} scratch accesses (register spills), the first: `{spills[0]}`")
    if with_ring == 0:
        return ["no ring loads found (expected global_load_* / buffer_load_* ... nt in the kernel)"]
    return errors


def main(hipcc="/opt/rocm/bin/hipcc", flags=(), sources=SOURCES):
    for name in sources:
        with tempfile.TemporaryDirectory() as td:
            out = os.path.join(td, "k.s")
            subprocess.check_call([hipcc, *flags, "-S", "--cuda-device-only", os.path.join(HERE, "csrc", name), "-o", out],
                                  stderr=subprocess.DEVNULL)
            text = open(out).read()
            errs = check(text)
            hazards = check_asm_results(text)
        if errs:
            raise RuntimeError(f"{name}: the generated code touches in-flight ring registers:\n  " + "\n  ".join(errs[:20]))
        if hazards:
            raise RuntimeError(f"{name}: an inline-assembly result reaches an MFMA / DPP instruction without wait states:\n  "
                               + "\n  ".join(hazards[:20]))
    return True


if __name__ == "__main__":
    from relax_amd import build as _b  # noqa: E402

    main(_b.HIPCC, [f for f in _b.FLAGS if f != "-fPIC"])
    print("ring registers: ok")
