"""Checker for kernels that issue LDS reads from inline assembly and place the waits by hand.

The compiler does not know that the registers such a read names are filled later: anything it puts
between the read and the hand-written s_waitcnt that releases them (a register copy where two
branches meet, a spill) reads or overwrites them too early, silently.  This scans a kernel's
assembly in program order, keeps the LDS reads in flight according to the s_waitcnt lgkmcnt(N)
bookkeeping (LDS operations of a wavefront complete in order) and reports every instruction that
touches a register still in flight.  Test infrastructure: nothing in the library uses it."""
import re


def _regs(text):
    out = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    rest = re.sub(r"v\[\d+:\d+\]", "", text)
    for m in re.finditer(r"\bv(\d+)\b", rest):
        out.add(int(m.group(1)))
    return out


def kernels(asm_text):
    """names of the kernels (global function symbols followed by code) in an assembly listing"""
    return re.findall(r"^\s*\.amdhsa_kernel\s+(\S+)", asm_text, flags=re.M)


def violations(asm_text, kernel):
    lines = asm_text.split("\n")
    inside = False
    in_flight = []  # (registers, line number) of LDS reads, oldest first
    found = []
    for n, line in enumerate(lines, 1):
        if line.startswith(kernel + ":"):
            inside = True
            continue
        if not inside:
            continue
        code = line.split(";")[0].strip()
        if not code or code.startswith("."):
            continue
        if code.startswith("s_endpgm"):
            break
        op = code.split()[0]
        args = code[len(op):].strip()
        if op.startswith("ds_read"):
            in_flight.append((_regs(args.split(",")[0]), n))
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", args)
            if m:
                keep = int(m.group(1))
                in_flight = in_flight[len(in_flight) - keep:] if keep else []
            continue
        parts = args.split(",")
        writes_first = op.startswith(("v_", "global_load", "scratch_load", "buffer_load"))
        read = _regs(",".join(parts[1:]) if writes_first else args)
        written = _regs(parts[0]) if writes_first else set()
        for regs, since in in_flight:
            if regs & read:
                found.append("line %d: `%s` reads v%d, in flight since line %d" % (n, code, min(regs & read), since))
            if regs & written:
                found.append("line %d: `%s` overwrites v%d, in flight since line %d" % (n, code, min(regs & written), since))
    return found
