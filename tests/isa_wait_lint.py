"""Checker for kernels that issue LDS reads and global loads from inline assembly and place the
waits by hand.

The compiler does not know that the registers such an instruction names are filled later: anything
it puts between the request and the hand-written s_waitcnt that releases them (a register copy where
two branches meet, a spill, a multiply it hoisted) reads or overwrites them too early, silently.
This walks a kernel's assembly along its control flow, keeps two queues of what is in flight
according to the s_waitcnt bookkeeping -- lgkmcnt for LDS operations (reads, writes, lane permutes), vmcnt for global/buffer/scratch
loads, stores and loads that land in LDS (each queue completes in order on this target) -- and
reports every instruction that touches a register still in flight.  Test infrastructure: nothing in
the library uses it."""
import re


def _regs(text):
    out = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    rest = re.sub(r"v\[\d+:\d+\]", "", text)
    for m in re.finditer(r"\bv(\d+)\b", rest):
        out.add(int(m.group(1)))
    return out


_VM_OPS = ("global_load", "buffer_load", "scratch_load", "global_store", "buffer_store", "scratch_store",
           "global_atomic", "buffer_atomic")


_MAX_VISITS = 256  # of one block, with different things in flight: enough for every loop here to settle


def kernels(asm_text):
    """names of the kernels (global function symbols followed by code) in an assembly listing"""
    return re.findall(r"^\s*\.amdhsa_kernel\s+(\S+)", asm_text, flags=re.M)


def _kernel_code(asm_text, kernel):
    """[(line number, code)] of a kernel: instructions and labels, comments and directives dropped"""
    out = []
    inside = False
    for n, line in enumerate(asm_text.split("\n"), 1):
        if line.startswith(kernel + ":"):
            inside = True
            continue
        if not inside:
            continue
        code = line.split(";")[0].strip()
        if not code or (code.startswith(".") and not code.endswith(":")):
            continue
        if code.startswith(".Lfunc_end"):  # (blocks may follow an s_endpgm; the symbol's end is the end)
            break
        out.append((n, code))
    return out


def violations(asm_text, kernel):
    """Walks the kernel's control flow graph: a block is scanned once per distinct set of LDS reads that
    can be in flight where it starts (a loop head is entered with the reads its back edge leaves)."""
    code = _kernel_code(asm_text, kernel)
    label_at = {c[:-1]: i for i, (_, c) in enumerate(code) if c.endswith(":")}
    found = []
    seen = set()
    visits = {}
    # (index into code, LDS reads in flight there, memory operations in flight there); a queue holds
    # (registers to be written, line) oldest first
    todo = [(0, (), ())]
    while todo:
        i, lds_state, vm_state = todo.pop()
        lds, vm = list(lds_state), list(vm_state)
        while i < len(code):
            n, text = code[i]
            if text.endswith(":"):  # a block starts here
                key = (i, tuple(lds), tuple(vm))
                if key in seen or visits.get(i, 0) >= _MAX_VISITS:
                    break
                seen.add(key)
                visits[i] = visits.get(i, 0) + 1
                i += 1
                continue
            op = text.split()[0]
            args = text[len(op):].strip()
            if op.startswith("s_endpgm"):
                break
            if op == "s_branch":
                i = label_at[args]
                continue
            if op.startswith("s_cbranch"):
                todo.append((label_at[args], tuple(lds), tuple(vm)))
                i += 1
                continue
            i += 1
            if op == "s_waitcnt":
                for name, queue in (("lgkmcnt", lds), ("vmcnt", vm)):
                    m = re.search(name + r"\((\d+)\)", args)
                    if m:
                        keep = int(m.group(1))
                        del queue[:len(queue) - keep if keep else len(queue)]
                continue
            parts = args.split(",")
            is_vm = op.startswith(_VM_OPS)
            is_lds = op.startswith("ds_")  # every LDS operation counts in lgkmcnt, writes and lane permutes included
            lds_fills = is_lds and any(k in op for k in ("read", "permute", "swizzle", "_rtn", "consume", "append"))
            fills = lds_fills or (is_vm and "_load" in op and "_lds" not in op)
            writes_first = fills or op.startswith("v_")
            read = _regs(",".join(parts[1:]) if writes_first else args)
            written = _regs(parts[0]) if writes_first else set()
            own = lds if lds_fills else vm if fills else None
            for queue in (lds, vm):
                for regs, since in queue:
                    if regs & read:
                        found.append("line %d: `%s` reads v%d, in flight since line %d" % (n, text, min(regs & read), since))
                    # (a second fill of a register from the same queue lands after the first: in order)
                    if regs & written and queue is not own:
                        found.append("line %d: `%s` overwrites v%d, in flight since line %d" % (n, text, min(regs & written), since))
            if is_lds:
                lds.append((frozenset(written), n) if lds_fills else (frozenset(), 0))
                del lds[:-15]  # (the hardware's counter holds 4 bits)
            elif is_vm:
                # (what fills no register only counts: its line is left out, so that states that differ
                # in nothing else are one state; the hardware's counter holds 6 bits)
                vm.append((frozenset(written), n) if fills else (frozenset(), 0))
                del vm[:-63]
    return sorted(set(found), key=lambda f: int(f.split()[1][:-1]))
