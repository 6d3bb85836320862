"""A lint over compiled gfx950 assembly for one hazard that hipcc's wait-state insertion leaves open: a vector
instruction that reads an MFMA's result registers needs the MFMA's passes behind it, and the compiler counts the
wait states between the two within one basic block only.  Where a branch or a label lies between them (a
conditional piece of work placed behind an MFMA), the reader can come out a few instructions behind the MFMA and
see the registers before they are written.  An MFMA that takes the result as its own accumulator is not a reader in
this sense (the matrix core orders those itself).

violations(asm) walks forward from every MFMA along the fall-through path and the targets of the branches it meets,
for as many wait states as the longest MFMA needs, and reports readers reached across a block boundary."""
import re

WAIT_STATES = 18  # a 16-pass MFMA's result is readable by the vector ALU 18 wait states behind it


def _regs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def _is_instruction(line):
    t = line.strip()
    return bool(t) and not t.startswith(";") and not t.startswith(".") and not t.endswith(":")


def violations(asm):
    lines = [l.rstrip() for l in asm.split("\n")]
    labels = {l.split(":")[0]: i for i, l in enumerate(lines) if l.startswith(".LBB")}
    found = []

    def walk(i, dst, budget, crossed, origin, seen):
        while budget > 0 and i < len(lines):
            line = lines[i]
            if line.startswith(".LBB"):
                crossed = True
                i += 1
                continue
            if not _is_instruction(line):
                i += 1
                continue
            t = line.strip()
            op = t.split()[0]
            if op == "s_endpgm" or op == "s_setpc_b64":
                return
            if op == "s_nop":
                budget -= int(t.split()[1]) + 1
                i += 1
                continue
            if op == "s_sleep":
                budget -= 64 * max(int(t.split()[1]), 1)
                i += 1
                continue
            if op.startswith("s_cbranch") or op == "s_branch":
                target = t.split()[1]
                if target in labels and (origin, target) not in seen:
                    seen.add((origin, target))
                    walk(labels[target], dst, budget - 1, True, origin, seen)
                if op == "s_branch":
                    return
                crossed = True
                budget -= 1
                i += 1
                continue
            operands = t[len(op):]
            parts = operands.split(",")
            if op.startswith("v_mfma"):
                read = _regs(parts[1]) | _regs(parts[2]) if len(parts) > 2 else set()
                budget -= 4
            elif op.startswith("v_"):
                # the first operand is written; v_fmac / v_mac forms accumulate into it, so they read it too
                read = _regs(",".join(parts[1:])) | (_regs(parts[0]) if "mac" in op else set())
                budget -= 1
            elif op.startswith(("global_", "ds_", "buffer_", "scratch_")):
                # (a load's destination is a write: only its address and data operands are read)
                read = _regs(",".join(parts[1:])) if op.startswith(("ds_read", "global_load", "buffer_load", "scratch_load")) else _regs(operands)
                budget -= 1
            else:
                read = set()
                budget -= 1
            if crossed and read & dst:
                found.append("MFMA at line %d: its result is read at line %d, across a block boundary: %s" % (origin + 1, i + 1, t))
                return
            if op.startswith("v_") and not op.startswith("v_mfma"):
                dst = dst - _regs(parts[0])  # (overwritten: no longer the MFMA's result)
                if not dst:
                    return
            i += 1

    for i, line in enumerate(lines):
        t = line.strip()
        if t.startswith("v_mfma"):
            walk(i + 1, _regs(t.split()[1].rstrip(",")), WAIT_STATES, False, i, set())
    return sorted(set(found))
