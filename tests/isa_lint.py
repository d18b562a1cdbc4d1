"""Check of the generated gfx950 code for one hazard of hand-written asynchronous loads.

Several kernels issue a load with an inline-asm instruction and wait for it later with a second asm statement that
names the destination registers as read-write operands.  Between the two the compiler takes the registers for
defined: if it moves them (a copy at a control-flow join, live-range splitting under register pressure), the copy
runs before the data has landed, the later code reads the copy, and the result is wrong now and then, with no error.
The check walks the assembly of every kernel in program order, keeps the destination registers of asm loads
(`global_load*`, `ds_read*` between ASMSTART / ASMEND) until a wait counter retires them or an instruction overwrites
them, and reports every register move whose source is still in flight.  Program order is an approximation of
control flow, good enough for the straight-line pipelines these kernels are.
"""
import re


def _regs(tok):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", tok):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def copies_of_inflight_registers(asm_text):
    """[(kernel, line number, instruction, line of the load)] for every move of a register whose load is in flight."""
    lines = asm_text.split("\n")
    starts = [(i, l.split(":")[0]) for i, l in enumerate(lines) if re.match(r"^_Z\w+:", l)]
    found = []
    for idx, (st, name) in enumerate(starts):
        en = starts[idx + 1][0] if idx + 1 < len(starts) else len(lines)
        vm, lg, inasm = [], [], False
        for i in range(st, en):
            l = lines[i].strip()
            if l.startswith(";;#ASMSTART"):
                inasm = True
                continue
            if l.startswith(";;#ASMEND"):
                inasm = False
                continue
            if not l or l[0] in ";.":
                continue
            op = l.split()[0]
            if op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", l)
                if m:
                    n = int(m.group(1))
                    vm = vm[len(vm) - n:] if n > 0 else []
                m = re.search(r"lgkmcnt\((\d+)\)", l)
                if m:
                    n = int(m.group(1))
                    lg = lg[len(lg) - n:] if n > 0 else []
                continue
            if inasm:
                if op.startswith("global_load_lds"):
                    vm.append((i + 1, set()))
                elif op.startswith("global_load"):
                    vm.append((i + 1, _regs(l.split(",")[0])))
                elif op.startswith("ds_read"):
                    lg.append((i + 1, _regs(l.split(",")[0])))
                elif op.startswith("ds_write"):
                    lg.append((i + 1, set()))
                continue
            if op.startswith(("global_load", "buffer_load", "flat_load", "global_store", "buffer_store", "flat_store",
                              "global_atomic")):
                vm.append((i + 1, set()))
                continue
            if op.startswith(("ds_", "s_load", "s_buffer_load")):
                lg.append((i + 1, set()))
                continue
            parts = l.split(",")
            src = _regs(",".join(parts[1:])) if len(parts) > 1 else set()
            if op.startswith(("v_mov", "v_accvgpr", "v_swap", "scratch_store")):
                for ln, rs in vm + lg:
                    if src & rs:
                        found.append((name, i + 1, l, ln))
                        break
            if op.startswith("v_") and not op.startswith("v_cmp"):
                dst = _regs(parts[0]) - src
                if dst:  # written again: this path no longer waits for the load into it
                    vm = [(ln, rs - dst) for ln, rs in vm]
                    lg = [(ln, rs - dst) for ln, rs in lg]
    return found


def scratch_bytes_per_kernel(asm_text):
    """{kernel symbol: scratch bytes per lane} from the resource comments hipcc writes behind every kernel."""
    out, name = {}, None
    for l in asm_text.split("\n"):
        m = re.match(r"^(_Z\w+):", l)
        if m:
            name = m.group(1)
        m = re.match(r"^; ScratchSize: (\d+)", l)
        if m and name:
            out[name] = int(m.group(1))
            name = None
    return out
