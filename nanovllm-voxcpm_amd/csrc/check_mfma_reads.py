"""Check of the compiler's assembly output for this library's kernels (`make check`).

An MFMA's result may not be read by another kind of instruction for some cycles after the MFMA
was issued.  The compiler spaces them out along straight-line code.  Where a run of MFMAs can be
left through a branch (rank blocks or k-steps that are skipped at run time) and the branch lands
on code that reads the last result, it was seen to provide for the longest way to that code only:
the result was read two instructions after its MFMA and came out incomplete or not depending on
where the code lay in memory.  The kernels therefore call `mfma_settle` behind such runs; this
script finds places where that was forgotten: an MFMA followed within NEED wait states by a
branch whose target reads the MFMA's destination registers after fewer than NEED wait states.
NEED follows from the MFMA's mnemonic: the number of passes of the variant plus three, which is
what the instruction set's table of software-inserted wait states asks for between a matrix
instruction's write and a vector instruction's read of the same register, and never less than the
eight states the compiler was seen to leave along straight-line code.  Passes (four cycles each)
of the 16-bit variants on this chip, from their FLOP count at 1024 FLOP per cycle and SIMD:
16x16x32 and 16x16x16 four, 32x32x16 eight; a mnemonic the table below does not know is given the
largest value.  A wait instruction or a barrier is not taken for a delay: it may return at once.

usage: check_mfma_reads.py file.s [file.s ...]    (exit status 1 if anything is found)
"""
import re
import sys

ANY_USE = False  # True: an early overwrite of the result counts as well as an early read
PASSES = {"16x16x32": 4, "16x16x16": 4, "32x32x16": 8, "32x32x8": 8, "4x4x4": 2}
NEED_MIN, NEED_MAX = 8, 19


def need_of(mnemonic):
    """Wait states between this MFMA and a read of its result by another kind of instruction."""
    for shape, passes in PASSES.items():
        if f"_{shape}" in mnemonic:
            return max(passes + 3, NEED_MIN)
    return NEED_MAX


def vgprs(text):
    out = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def is_code(line):
    return bool(line) and not line.endswith(":") and not line.startswith(".")


def early_read(lines, start, dst, states, need):
    """First instruction from `start` on that reads `dst` before `need` wait states have passed."""
    k, seen = start, 0
    while k < len(lines) and states < need and seen < 60:
        w = lines[k].strip()
        k += 1
        if not is_code(w):
            continue
        seen += 1
        if w.startswith("s_nop"):
            states += int(w.split()[1]) + 1
            continue
        if w.startswith(("s_endpgm", "v_mfma")):
            return None  # the end, or the matrix pipeline's own ordering
        if w.startswith(("s_branch", "s_cbranch", "s_waitcnt", "s_barrier")):
            states += 1  # (a wait or a barrier may return at once: one state, no more)
            continue
        operands = w.split(None, 1)[1].split(",") if " " in w else []
        stores = w.startswith(("global_store", "buffer_store", "ds_write", "scratch_store"))
        if vgprs(",".join(operands if stores or ANY_USE else operands[1:])) & dst:
            return states, w
        states += 1
    return None


def scan(path):
    lines = [l.split(";")[0].rstrip() for l in open(path)]
    labels = {l[:-1]: i for i, l in enumerate(lines) if l.endswith(":") and not l.startswith("\t")}
    found, func = 0, "?"
    for i, l in enumerate(lines):
        if l.endswith(":") and l.startswith("_Z"):
            func = l[:-1]
        t = l.strip()
        if not t.startswith("v_mfma"):
            continue
        dst = vgprs(t.split(",")[0])
        need = need_of(t.split()[0])
        # walk on from the MFMA; every branch met before `need` wait states have passed is followed
        j, states = i + 1, 0
        while j < len(lines) and states < need:
            u = lines[j].strip()
            j += 1
            if not is_code(u):
                continue
            if u.startswith("s_nop"):
                states += int(u.split()[1]) + 1
                continue
            if u.startswith(("s_endpgm", "v_mfma")):
                break
            if u.startswith(("s_waitcnt", "s_barrier")):
                states += 1
                continue
            if u.startswith(("s_branch", "s_cbranch")):
                hit = early_read(lines, labels.get(u.split()[-1], len(lines)), dst, states + 1, need)
                if hit:
                    print(f"{path}:{i + 1}: {func[:70]}\n    {t}\n    -> {u.split()[-1]}: read after {hit[0]} wait states: {hit[1]}")
                    found += 1
                if u.startswith("s_branch"):
                    break
            states += 1
    return found


if __name__ == "__main__":
    total = sum(scan(p) for p in sys.argv[1:])
    print(f"{total} early reads of MFMA results")
    sys.exit(1 if total else 0)
