#!/usr/bin/env python3
"""Static check of kernels whose vector-memory instructions and waits are written by hand.

    python3 check_vmem_asm.py file.s kernel_name_substring [...]

The streaming kernels issue their global loads from asm statements and place `s_waitcnt vmcnt(N)`
themselves, so the compiler does not know that a load's destination registers are still being
filled.  Correctness then rests on two facts about the generated code which this script proves on
the compiler's assembly output, over every path through the kernel:

  * between a load (or returning atomic) and the wait that covers it, no instruction reads or
    writes the destination registers (a register copy inserted by the register allocator would);
  * no wave ends with a load in flight;
  * no vector instruction overwrites the data registers of a store of more than 8 bytes within
    two wait states of it (the store still reads them then; the compiler pads this hazard for its
    own stores only).

A wait `vmcnt(N)` is taken to cover exactly the operations that have at least N vector-memory
operations issued after them on every path (loads, stores and atomics count alike) — the weakest
reading of the counter.  The analysis is a forward data-flow over the control-flow graph; the state
maps each in-flight register to the least number of operations issued behind it.
"""
import re
import sys

VREG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
VMCNT = re.compile(r"vmcnt\((\d+)\)")
CAP = 64


def vregs(text):
    out = set()
    for m in VREG.finditer(text):
        if m.group(1) is not None:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def parse_kernel(lines, start):
    """Instructions of the kernel whose label is at lines[start]: list of (label_or_None, text)."""
    insts, labels = [], {}
    for raw in lines[start + 1:]:
        text = raw.split(";")[0].strip()
        if raw.startswith(".Lfunc_end"):
            break
        if raw.startswith(".LBB") or re.match(r"^\.L\w+:", raw):
            labels[raw.split(":")[0].strip()] = len(insts)
            continue
        if not text or text.startswith(".") or text.startswith(";"):
            continue
        insts.append(text)
    return insts, labels


SREG_PAIR = re.compile(r"\bs\[(\d+):(\d+)\]")


class State:
    """in_flight: VGPR -> least number of vector-memory operations issued behind its load.
    exec_nz: the exec mask is known to be non-zero.  nz: SGPR pairs known to hold a non-zero mask."""

    def __init__(self, in_flight=None, exec_nz=True, nz=frozenset(), ones=frozenset(), vcc_nz=False):
        self.in_flight = dict(in_flight or {})
        self.exec_nz = exec_nz
        self.nz = frozenset(nz)
        self.ones = frozenset(ones)      # SGPR pairs known to hold -1
        self.vcc_nz = vcc_nz             # vcc is known to be non-zero

    def key(self):
        return (tuple(sorted(self.in_flight.items())), self.exec_nz, self.nz, self.ones, self.vcc_nz)

    def copy(self):
        return State(self.in_flight, self.exec_nz, self.nz, self.ones, self.vcc_nz)


def merge(a, b):
    if a is None:
        return b.copy()
    out = dict(a.in_flight)
    for r, k in b.in_flight.items():
        out[r] = min(out[r], k) if r in out else k
    return State(out, a.exec_nz and b.exec_nz, a.nz & b.nz, a.ones & b.ones, a.vcc_nz and b.vcc_nz)


def successors(insts, labels, i, state):
    """Where control can go after instruction i.  A branch on `exec == 0` is not followed when the mask
    is known to be non-zero, nor one on vcc when vcc is known to be `exec & -1` with exec non-zero (the compiler
    emits both around uniform loop exits)."""
    text = insts[i]
    op = text.split()[0]
    if op == "s_endpgm":
        return []
    if op == "s_branch":
        return [labels[text.split()[1]]]
    if op == "s_cbranch_execz":
        return [i + 1] if state.exec_nz else [labels[text.split()[1]], i + 1]
    if op == "s_cbranch_execnz":
        return [labels[text.split()[1]]] if state.exec_nz else [labels[text.split()[1]], i + 1]
    if op == "s_cbranch_vccnz" and state.vcc_nz:
        return [labels[text.split()[1]]]
    if op == "s_cbranch_vccz" and state.vcc_nz:
        return [i + 1]
    if op.startswith("s_cbranch"):
        return [labels[text.split()[1]], i + 1]
    return [i + 1]


def is_vmem(op):
    return op.startswith(("global_", "flat_", "buffer_", "scratch_"))


def scalar_effects(text, st):
    """Tracks whether exec is known non-zero through the save / restore idiom of divergent branches."""
    op = text.split()[0]
    parts = [p.strip() for p in text[len(op):].split(",")]
    dest = parts[0] if parts else ""
    pairs = lambda t: {int(m.group(1)) for m in SREG_PAIR.finditer(t)}
    # vcc: known non-zero only right after `s_and_b64 vcc, exec, <pair holding -1>` with exec non-zero; anything
    # else that may write it (every mention outside pure readers, every v_cmp) makes it unknown again
    if op == "s_and_b64" and dest == "vcc" and parts[1] == "exec" and pairs(parts[2]) & st.ones and st.exec_nz:
        st.vcc_nz = True
    elif op.startswith("v_cmp") or ("vcc" in text and not op.startswith(("s_cbranch", "v_cndmask", "v_div_fmas"))):
        st.vcc_nz = False
    if not op.startswith("s_"):
        return
    if op == "s_mov_b64" and dest != "exec" and parts[1] == "-1":
        st.ones = st.ones | pairs(dest)
    elif pairs(dest) & st.ones:
        st.ones = st.ones - pairs(dest)
    if op == "s_and_saveexec_b64" or op == "s_or_saveexec_b64":
        saved = pairs(dest)
        st.nz = (st.nz - saved) | (saved if st.exec_nz else set())
        st.exec_nz = False
        return
    if dest == "exec":
        if op == "s_or_b64":
            srcs = pairs(",".join(parts[1:]))
            st.exec_nz = st.exec_nz or bool(srcs & st.nz)
        elif op == "s_mov_b64":
            st.exec_nz = bool(pairs(parts[1]) & st.nz)
        else:
            st.exec_nz = False
        return
    written = pairs(dest)
    if written & st.nz:
        st.nz = st.nz - written
    # a 32-bit scalar write into half of a tracked pair
    m = re.match(r"^s(\d+)$", dest)
    if m:
        n = int(m.group(1))
        st.nz = frozenset(x for x in st.nz if x != n and x + 1 != n)
        st.ones = frozenset(x for x in st.ones if x != n and x + 1 != n)


def transfer(text, st, where, problems):
    """Applies one instruction to the state."""
    op = text.split()[0]
    operands = text[len(op):]
    scalar_effects(text, st)
    if op == "s_waitcnt":
        m = VMCNT.search(text)
        if m:
            n = int(m.group(1))
            st.in_flight = {r: k for r, k in st.in_flight.items() if k < n}
        return st
    if is_vmem(op) and not op.startswith(("buffer_wbl2", "buffer_inv")):
        parts = [p.strip() for p in operands.split(",")]
        returns = op.startswith(("global_load", "flat_load", "buffer_load")) or ("atomic" in op and " sc0" in text)
        dest = vregs(parts[0]) if returns else set()
        srcs = vregs(",".join(parts[1:] if returns else parts))
        hit = (srcs | dest) & set(st.in_flight)
        if hit:
            problems.append(f"{where}: `{text}` uses v{sorted(hit)} while a load into it is in flight")
        st.in_flight = {r: min(k + 1, CAP) for r, k in st.in_flight.items()}
        for r in dest:
            st.in_flight[r] = 0
        return st
    hit = vregs(operands) & set(st.in_flight)
    if hit:
        problems.append(f"{where}: `{text}` touches v{sorted(hit)} while a load into it is in flight")
    if op == "s_endpgm" and st.in_flight:
        problems.append(f"{where}: the wave ends with loads in flight into v{sorted(st.in_flight)}")
    return st


def store_data_hazards(insts, name):
    """A store of more than 8 bytes reads its data registers for two wait states after issue."""
    problems = []
    for i, text in enumerate(insts):
        op = text.split()[0]
        if not (is_vmem(op) and "store" in op and op.endswith(("dwordx3", "dwordx4"))):
            continue
        data = vregs(text[len(op):].split(",")[1])
        waited, j = 0, i + 1
        while waited < 2 and j < len(insts):
            nxt = insts[j]
            nop = nxt.split()[0]
            if nop == "s_nop":
                waited += int(nxt.split()[1]) + 1
            else:
                if nop.startswith("v_") and vregs(nxt[len(nop):].split(",")[0]) & data:
                    problems.append(f"{name} instruction {j}: `{nxt}` overwrites data of `{text}` {waited} wait state(s) after it")
                if nop.startswith(("s_branch", "s_cbranch", "s_endpgm")):
                    break
                waited += 1
            j += 1
    return problems


def check(lines, start, name):
    """Forward data-flow.  States that differ in what is known about scalar registers (exec, vcc, pairs holding
    -1 or a non-zero mask) are kept apart at joins, so that a branch decided by such a fact on one incoming path
    only is followed correctly; states that agree in those facts are merged."""
    insts, labels = parse_kernel(lines, start)
    facts = lambda st: (st.exec_nz, st.nz, st.ones, st.vcc_nz)
    state_in = [dict() for _ in range(len(insts) + 1)]
    state_in[0][facts(State())] = State()
    work = [(0, facts(State()))]
    steps = 0
    while work:
        i, f = work.pop()
        steps += 1
        if i >= len(insts) or steps > 2_000_000:
            continue
        out = transfer(insts[i], state_in[i][f].copy(), "", [])
        for j in successors(insts, labels, i, out):
            fj = facts(out)
            merged = merge(state_in[j].get(fj), out)
            if fj not in state_in[j] or merged.key() != state_in[j][fj].key():
                state_in[j][fj] = merged
                work.append((j, fj))
    problems = store_data_hazards(insts, name)
    if steps > 2_000_000:
        problems.append(f"{name}: analysis did not converge")
    seen = set()
    loads = waits = 0
    for i, text in enumerate(insts):
        for st in state_in[i].values():
            found = []
            transfer(text, st.copy(), f"{name} instruction {i}", found)
            for msg in found:
                if msg not in seen:
                    seen.add(msg)
                    problems.append(msg)
        loads += text.startswith("global_load")
        waits += text.startswith("s_waitcnt") and "vmcnt" in text
    return problems, len(insts), loads, waits


def main():
    path, wanted = sys.argv[1], sys.argv[2:]
    lines = open(path).read().split("\n")
    found = 0
    failed = False
    for i, line in enumerate(lines):
        m = re.match(r"^(\w+):\s*;\s*@", line)
        if not m or not any(w in m.group(1) for w in wanted):
            continue
        found += 1
        problems, n, loads, waits = check(lines, i, m.group(1))
        print(f"{m.group(1)}: {n} instructions, {loads} global loads, {waits} vmcnt waits: "
              + ("ok" if not problems else f"{len(problems)} problem(s)"))
        for p in problems[:20]:
            print("   ", p)
        failed |= bool(problems)
    if found == 0:
        print(f"no kernel matching {wanted} in {path}")
        failed = True
    sys.exit(1 if failed else 0)


if __name__ == "__main__":
    main()
