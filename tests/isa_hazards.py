"""Checks gfx950 assembly for one class of hazard: a vector (or LDS / memory) instruction that reads (or
overwrites) the result of a matrix instruction, in another basic block, before the matrix pipeline has written it.

Matrix instructions are not interlocked against such readers; the required distance is padded with wait
states by the compiler, which only looks inside one basic block. A reader reached through a branch (or
past a label) sooner than the instruction's latency takes the accumulator as it was before the last
instruction landed. Required distances (CDNA3 ISA guide, "XDL write VGPR" followed by a VALU / LDS /
memory read of it): 7 wait states for a 4-pass instruction (the 16x16 shapes here), 11 for an 8-pass one
(32x32x16). Every instruction issued in between counts as one wait state, `s_nop N` as N + 1, a following
matrix instruction as its own passes.
"""
import re

NEED = {"32x32": 11, "16x16": 7}
HORIZON = 20  # wait states walked behind each matrix instruction


def _regs(tok):
    m = re.match(r"([av])\[(\d+):(\d+)\]$", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"([av])(\d+)$", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def _parse(line):
    line = line.split(";")[0].strip()
    if not line or (line.startswith(".") and not line.startswith(".LBB")):
        return None
    if line.endswith(":"):
        return ("label", line[:-1], [])
    parts = line.replace(",", " ").split()
    return ("ins", parts[0], parts[1:])


def kernels(text):
    """Yields (mangled name, [parsed lines]) for every kernel body of an assembly listing."""
    name, lines = None, []
    for raw in text.splitlines():
        if re.match(r"^_Z\w+:", raw):
            name, lines = raw.strip()[:-1], []
            continue
        if name is None:
            continue
        p = _parse(raw)
        if p:
            lines.append(p)
        if "s_endpgm" in raw:
            yield name, lines
            name = None


def violations(lines):
    """[(index of the matrix instruction, its text, index of the reader, its text, wait states between)]"""
    labels = {l[1]: i for i, l in enumerate(lines) if l[0] == "label"}
    found = []
    for i, l in enumerate(lines):
        if l[0] != "ins" or not l[1].startswith("v_mfma"):
            continue
        need = NEED["32x32"] if "32x32" in l[1] else NEED["16x16"]
        dst = _regs(l[2][0])

        def walk(j, left, crossed, seen):
            while j < len(lines) and left > 0:
                kind, op, args = lines[j]
                if kind == "label":
                    crossed, j = True, j + 1
                    continue
                if op.startswith("s_cbranch") or op == "s_branch":
                    tgt = args[0]
                    if tgt in labels and (tgt, left) not in seen:
                        seen.add((tgt, left))
                        walk(labels[tgt], left - 1, True, seen)
                    if op == "s_branch":
                        return
                    crossed, j, left = True, j + 1, left - 1
                    continue
                if op == "s_nop":
                    left, j = left - int(args[0]) - 1, j + 1
                    continue
                if op.startswith("v_mfma"):
                    left, j = left - (8 if "32x32" in op else 4), j + 1
                    continue
                stores = op.startswith(("ds_write", "global_store", "buffer_store", "scratch_store"))
                srcs = set()
                for a in (args if stores else args[1:]):
                    srcs |= _regs(a)
                # (an instruction that overwrites the result registers while the matrix instruction is still in the
                # pipeline is as bad as one that reads them early: its value is overwritten when the result lands)
                if not stores and args and not op.startswith("s_"):
                    srcs |= _regs(args[0])
                if srcs & dst:
                    if crossed and HORIZON - left < need and not any(f[0] == i and f[2] == j for f in found):
                        found.append((i, " ".join([l[1]] + l[2]), j, " ".join([op] + args), HORIZON - left))
                    return  # the first reader decides; one in the same block is the compiler's to pad
                left, j = left - 1, j + 1

        walk(i + 1, HORIZON, False, set())
    return found
