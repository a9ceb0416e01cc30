"""Static check of the gfx950 assembly of the attention kernels.

The transposing LDS reads (``ds_read_b64_tr_b16``) of these kernels are inline assembly, and the ``s_waitcnt
lgkmcnt(0)`` that makes their results usable is written out by hand (csrc/common.h: ``lds_read_tr16_b64``,
``lds_tr_wait``; csrc/attention_sweep.h).  The compiler neither counts these reads nor protects their destination
registers, so two properties that it guarantees for its own instructions have to be checked on what it emitted:

1. pending result: between a transposing read and the next ``s_waitcnt`` with ``lgkmcnt(0)`` no instruction names one
   of the read's destination registers (it would see the old value, or be overwritten when the read returns).  The
   scan is linear; forward branches inside such a window (the mask's if-then) are covered because both paths are
   scanned, and a backward branch from outside a window to a label inside it - a second way in that the scan does not
   follow - is reported;
2. MFMA write-after-write: no transposing read is issued within ``MFMA_WINDOW`` instructions after an MFMA whose
   destination registers overlap the read's (the compiler may hand registers it can prove dead to the read while the
   MFMA that last wrote them is still running; the MFMA's late write then replaces what the read returned).

3. counted wait behind loads into LDS: a ``s_waitcnt vmcnt(N) lgkmcnt(0)`` with N > 0 stands where a kernel waits for
   its ``buffer_load ... lds`` loads but lets the N stores issued after them drain later (vector memory operations
   complete in order, so "at most N outstanding" covers everything older than the N youngest).  That only holds if N
   vector memory instructions really follow the loads on every path: the N youngest ones before the wait must be
   stores in the wait's own basic block (no label in between), so that no path can skip them.  (Checked wherever a
   store is among them; the counted waits of the k-loops stand between loads only.)

    python aeris-gb_amd/asm_check.py file.s [...]      # exit status 1 if a rule is broken

``check_text`` is what build.py runs on the device assembly of every source that contains such reads.
"""
from __future__ import annotations

import re
import sys

MFMA_WINDOW = 24  # instructions; an MFMA of these kernels is done at most 16 passes after it issued
_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
_TAIL_WAIT = re.compile(r"^s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)$")
_VMEM = ("global_", "buffer_", "flat_", "scratch_")
_KERNEL_LABEL = re.compile(r"^(_Z\w+):")


def _regs(text):
    out = set()
    for a, b, c in _REG.findall(text):
        out |= set(range(int(a), int(b) + 1)) if a else {int(c)}
    return out


def _first_operand(instr):
    parts = instr.split(None, 1)
    return parts[1].split(",")[0] if len(parts) > 1 else ""


def check_text(asm: str):
    """-> (problems, transposing reads seen); ``problems`` is a list of strings naming kernel, line and rule."""
    problems, n_reads = [], 0
    kernel, pending, recent_mfma, n_ins = None, {}, [], 0
    labels_in_window, window_id = {}, 0
    block_vmem = []  # vector memory instructions of the current basic block, in order
    for ln, raw in enumerate(asm.splitlines(), 1):
        m = _KERNEL_LABEL.match(raw)
        if m:
            kernel, pending, recent_mfma, n_ins = m.group(1), {}, [], 0
            labels_in_window = {}
            continue
        t = raw.split(";")[0].strip()
        if not t or kernel is None:
            continue
        if t.endswith(":"):
            if pending:
                labels_in_window[t[:-1]] = window_id
            block_vmem = []
            continue
        if t.startswith("."):
            continue
        n_ins += 1
        if t.startswith(_VMEM):
            block_vmem.append(t)
        m = _TAIL_WAIT.match(t)
        if m and int(m.group(1)) > 0:
            n = int(m.group(1))
            tail = block_vmem[-n:]
            is_store = [x.split()[0].startswith(("global_store", "buffer_store")) for x in tail]
            # (a counted wait with no store among the youngest operations is one of the k-loops' waits between loads)
            if any(is_store) and (len(tail) < n or not all(is_store)):
                problems.append(f"{kernel} line {ln}: `{t}` is not preceded by {n} stores in its basic block "
                                f"(found {[x.split()[0] for x in tail]})")
        if t.startswith(("s_cbranch", "s_branch")) and t.split()[-1] in labels_in_window:
            if not pending or labels_in_window[t.split()[-1]] != window_id:
                problems.append(f"{kernel} line {ln}: `{t}` jumps back into the window of a transposing read")
        if t.startswith("s_endpgm"):
            if pending:
                problems.append(f"{kernel} line {ln}: kernel ends with a transposing read not waited for")
            kernel = None
            continue
        if t.startswith("v_mfma"):
            recent_mfma = (recent_mfma + [(n_ins, _regs(_first_operand(t)))])[-16:]
        if t.startswith("ds_read_b64_tr_b16"):
            n_reads += 1
            dst = _regs(_first_operand(t))
            for at, mfma_dst in recent_mfma:
                if n_ins - at <= MFMA_WINDOW and dst & mfma_dst:
                    problems.append(f"{kernel} line {ln}: `{t}` returns into registers that an MFMA {n_ins - at} "
                                    f"instructions earlier is still writing")
            busy = dst & set(pending)
            if busy:
                problems.append(f"{kernel} line {ln}: `{t}` reuses destination registers {sorted(busy)} of a read not waited for")
            for r in dst:
                pending[r] = ln
            continue
        if t.startswith("s_waitcnt") and "lgkmcnt(0)" in t:
            if pending:
                window_id += 1
            pending = {}
            continue
        if pending:
            hit = _regs(t) & set(pending)
            if hit:
                problems.append(f"{kernel} line {ln}: `{t}` touches registers {sorted(hit)} of a transposing read "
                                f"(line {min(pending[r] for r in hit)}) before its wait")
    return problems, n_reads


def main(argv):
    bad = 0
    for path in argv:
        with open(path) as f:
            problems, n = check_text(f.read())
        print(f"{path}: {n} transposing reads, {len(problems)} problems")
        for p in problems:
            print("  " + p)
        bad += len(problems)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
