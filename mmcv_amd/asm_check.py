"""Build-time check of the device assembly the compiler emitted for libmdcn_hip.so.

The kernels issue their vector-memory instructions from inline assembly.  On
this hardware a vector-memory instruction must not read a scalar register that a
vector instruction (v_readlane_b32 / v_readfirstlane_b32: a reload of spilled
scalars, a broadcast) wrote within the previous five issue slots.  The compiler
keeps that distance for the instructions it emits itself, but it does not look
into assembly text, so a reload it places right in front of an asm statement
would make the statement read a stale base address.  This scan fails the build
when it finds such a pair; the cure is an ``s_nop`` at the head of the asm
statement or fewer live scalars around it.

Second check: the loads (global_load, ds_read) those asm statements issue
complete asynchronously, and the code waits for them with explicit ``s_waitcnt``
counts.  The compiler believes an asm statement's outputs are valid when the
statement ends, so it is free to copy such a register elsewhere, or to reuse it
as a temporary, between the load and the wait -- reading stale data, or having
the landing load overwrite an address.  The waits of the kernels therefore name
the registers they release in a trailing comment (``s_waitcnt vmcnt(32) ; v[4:7]
...``).  The scan follows every path through a kernel's basic blocks with the
set of registers that may still be locked -- locked by an asm-issued load,
released by an asm wait that names them or by any wait for count 0 -- and
fails the build when an instruction touches a locked register.

Third check: whether the count of such a wait is right.  ``s_waitcnt vmcnt(N)``
returns once at most N vector-memory operations of the wave are outstanding, and
loads complete in the order of issue, so the load into a register has landed for
sure when at least N loads were issued behind it.  The scan follows the same
paths with, per locked register, the smallest number of loads issued since its
own, and reports every wait that names a register with fewer than N loads behind
it (a count that is too large: the wait may return before the data is there), and
-- as a note, not a finding -- the slack of every wait (loads behind the register
minus N: 0 is a count that is exactly right on its shortest path).  Stores are
not counted: they only ever make a wait stricter.  Paths are followed without
regard to what the branches test, so the check suits kernels whose loads are
issued unconditionally; a kernel asks for it with an asm statement that is nothing
but the comment ``; mdcn-counted-waits``.
Paths are followed without regard to what the branches test, with one
exception: code that only one kind of wave executes can say so with an asm
statement that is nothing but the comment ``; mdcn-role <name>``.  A wave keeps
its role for the whole kernel, so a path that passes markers of two different
roles cannot occur and is dropped; without this, a kernel that branches on the
role in several places (first gather sets in another order, barrier at another
place) is reported for paths that mix the two.
"""
import re
import sys

_SREG = re.compile(r'\bs\[(\d+):(\d+)\]|\bs(\d+)\b')
_VMEM = ('global_', 'buffer_', 'flat_', 'scratch_')
WAIT_STATES = 5


def _sregs(text):
    regs = set()
    for m in _SREG.finditer(text):
        if m.group(1):
            regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            regs.add(int(m.group(3)))
    return regs


def violations(asm_text):
    """[(line number, instruction, scalar registers, distance, writer)] for every
    vector-memory instruction inside an inline-asm block that breaks the rule.
    Distances are counted backwards along every way into the instruction: through
    the instructions in front of it and, at a label, through every branch that
    targets the label as well as the code that falls into it."""
    found = []
    for name, ins, labels in _kernels(asm_text, keep_nops=True):
        n = len(ins)
        # predecessors of every instruction index
        label_at = {}
        for lab, idx in labels.items():
            label_at.setdefault(idx, []).append(lab)
        branches_to = {}
        falls_through = [True] * n
        for k, (no, t, _, _) in enumerate(ins):
            m = _BRANCH.match(t)
            if m:
                tgt = labels.get(m.group(1))
                if tgt is not None and tgt < n:
                    branches_to.setdefault(tgt, []).append(k)
                if not t.startswith('s_cbranch'):
                    falls_through[k] = False
            elif t.startswith(('s_endpgm', 's_setpc', 's_swappc')):
                falls_through[k] = False
        for k, (no, t, _, in_asm) in enumerate(ins):
            if not in_asm or not t.startswith(_VMEM):
                continue
            used = _sregs(t.split(None, 1)[1] if ' ' in t else '')
            if not used:
                continue
            # walk backwards: (index of the instruction to look at next, wait states collected so far)
            seen = {}
            work = [(k - 1, 0, k)]
            while work:
                j, dist, came_from = work.pop()
                if dist >= WAIT_STATES:
                    continue
                # ways into instruction `came_from`: falling in from j (if j falls through) and branches to it
                preds = []
                if j >= 0 and falls_through[j]:
                    preds.append(j)
                for b in branches_to.get(came_from, []):
                    preds.append(b)
                for pj in preds:
                    if seen.get(pj, WAIT_STATES) <= dist:
                        continue
                    seen[pj] = dist
                    pt = ins[pj][1]
                    d = dist
                    if pt.startswith('s_nop'):
                        d += int(pt.split()[1], 0) + 1
                    else:
                        if pt.startswith(('v_readlane_b32', 'v_readfirstlane_b32')):
                            hit = _sregs(pt.split(None, 1)[1].split(',')[0]) & used
                            if hit:
                                found.append((no, t, sorted(hit), dist, pt))
                                continue
                        d += 1
                    work.append((pj - 1, d, pj))
    return [(a, b, list(c), d, e) for a, b, c, d, e in sorted(set((a, b, tuple(c), d, e) for a, b, c, d, e in found))]


_VREG = re.compile(r'\bv\[(\d+):(\d+)\]|\bv(\d+)\b')
_VMCNT = re.compile(r'vmcnt\((\d+)\)')
_LGKMCNT = re.compile(r'lgkmcnt\((\d+)\)')
_BRANCH = re.compile(r'^s_c?branch\w*\s+(\.?\w+)')


def _vregs(text):
    regs = set()
    for m in _VREG.finditer(text):
        if m.group(1):
            regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            regs.add(int(m.group(3)))
    return regs


def _wait_counts(t):
    """(vmcnt, lgkmcnt) of an s_waitcnt; None for a counter it leaves alone."""
    vm, lg = _VMCNT.search(t), _LGKMCNT.search(t)
    if vm or lg or 'expcnt' in t:
        return (int(vm.group(1)) if vm else None, int(lg.group(1)) if lg else None)
    try:
        imm = int(t.split(None, 1)[1].strip(), 0)
    except (ValueError, IndexError):
        return (None, None)
    vmc = (imm & 0xF) | (((imm >> 14) & 0x3) << 4)
    lgc = (imm >> 8) & 0xF
    return (None if vmc == 63 else vmc, None if lgc == 15 else lgc)


def _kernels(asm_text, keep_nops=False):
    """[(name, [(line number, instruction, comment, inside inline asm)], {label: index})] per function."""
    out, cur, labels, in_asm = [], None, None, False
    for no, line in enumerate(asm_text.split('\n'), 1):
        t = line.strip()
        if t.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if t.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if in_asm and t.startswith('; mdcn-role ') and cur is not None:
            cur.append((no, 'role ' + t[len('; mdcn-role '):].strip(), '', True))
            continue
        if in_asm and t.startswith('; mdcn-counted-waits') and cur is not None:
            cur.append((no, 'counted-waits', '', True))
            continue
        if not t or t[0] == ';':
            continue
        code, _, comment = t.partition(';')
        code = code.strip()
        if code.endswith(':') and t[0] != '.':
            cur, labels = [], {}
            out.append((code[:-1], cur, labels))
            continue
        if cur is None:  # text that starts without a function label: one nameless function
            cur, labels = [], {}
            out.append(('', cur, labels))
        if code.endswith(':') and t.startswith('.L'):
            labels[code[:-1]] = len(cur)
            continue
        if t[0] == '.':
            continue
        cur.append((no, code, comment, in_asm))
    return out


def inflight_violations(asm_text):
    """[(kernel, line number, instruction, registers)] for every instruction that
    touches a register which a load issued from inline asm may still be writing."""
    found = set()
    for name, ins, labels in _kernels(asm_text):
        if not any(a and (c.startswith('ds_read') or (c.startswith(_VMEM) and 'load' in c and '_lds_' not in c))
                   for _, c, _, a in ins):
            continue
        n = len(ins)
        leaders = {0} | {i for i in labels.values() if i < n}
        succ_of = {}
        for k, (no, t, _, _) in enumerate(ins):
            m = _BRANCH.match(t)
            if m:
                tgt = labels.get(m.group(1))
                nxt = [tgt] if tgt is not None and tgt < n else []
                if t.startswith('s_cbranch') and k + 1 < n:
                    nxt.append(k + 1)
                succ_of[k] = nxt
                if k + 1 < n:
                    leaders.add(k + 1)
            elif t.startswith(('s_endpgm', 's_setpc', 's_swappc')):
                succ_of[k] = []
                if k + 1 < n:
                    leaders.add(k + 1)
        starts = sorted(leaders)
        end_of = {b: (starts[i + 1] if i + 1 < len(starts) else n) for i, b in enumerate(starts)}
        at_entry = {(0, None): (frozenset(), frozenset())}  # (block, role of the wave so far) -> locked registers
        work = [(0, None)]
        while work:
            b, role = work.pop()
            vm, lg = set(at_entry[(b, role)][0]), set(at_entry[(b, role)][1])
            feasible = True
            for k in range(b, end_of[b]):
                no, t, comment, in_asm = ins[k]
                if t == 'counted-waits':
                    continue
                if t.startswith('role '):
                    if role is not None and role != t[5:]:
                        feasible = False  # a wave of one role never reaches code of another
                        break
                    role = t[5:]
                    continue
                if t.startswith('s_waitcnt'):
                    vmc, lgc = _wait_counts(t)
                    named = _vregs(comment) if in_asm else set()
                    if vmc == 0:
                        vm.clear()
                    elif vmc is not None:
                        vm -= named
                    if lgc == 0:
                        lg.clear()
                    elif lgc is not None:
                        lg -= named
                    continue
                touched = _vregs(t.split(None, 1)[1]) if ' ' in t else set()
                hit = touched & (vm | lg)
                if hit:
                    found.add((name, no, t, tuple(sorted(hit))))
                if in_asm:
                    op, _, rest = t.partition(' ')
                    if op.startswith(_VMEM) and 'load' in op and '_lds_' not in op:
                        vm |= _vregs(rest.split(',')[0])
                    elif op.startswith('ds_read'):
                        lg |= _vregs(rest.split(',')[0])
            if not feasible:
                continue
            last = end_of[b] - 1
            out_state = (frozenset(vm), frozenset(lg))
            for nb in succ_of.get(last, [end_of[b]] if end_of[b] < n else []):
                old = at_entry.get((nb, role))
                new = out_state if old is None else (old[0] | out_state[0], old[1] | out_state[1])
                if new != old:
                    at_entry[(nb, role)] = new
                    work.append((nb, role))
    return sorted(found, key=lambda v: (v[0], v[1]))


_VM_LOAD = re.compile(r'^(global|buffer|flat|scratch)_(load|atomic)')
AGE_CAP = 64


def wait_count_findings(asm_text, notes=None):
    """[(kernel, line number, wait instruction, register, loads issued behind it)] for every
    wait inside inline asm whose vmcnt is larger than the number of loads issued behind
    the load of a register it names (or, for a wait whose comment says `lds-copies`, behind
    the youngest direct-to-LDS copy).  `notes`, a list, receives (kernel, line number, count,
    slack) for every such wait that names locked registers."""
    found = set()
    for name, ins, labels in _kernels(asm_text):
        if not any(t == 'counted-waits' for _, t, _, _ in ins):
            continue
        n = len(ins)
        leaders = {0} | {i for i in labels.values() if i < n}
        succ_of = {}
        for k, (no, t, _, _) in enumerate(ins):
            m = _BRANCH.match(t)
            if m:
                tgt = labels.get(m.group(1))
                nxt = [tgt] if tgt is not None and tgt < n else []
                if t.startswith('s_cbranch') and k + 1 < n:
                    nxt.append(k + 1)
                succ_of[k] = nxt
                if k + 1 < n:
                    leaders.add(k + 1)
            elif t.startswith(('s_endpgm', 's_setpc', 's_swappc')):
                succ_of[k] = []
                if k + 1 < n:
                    leaders.add(k + 1)
        starts = sorted(leaders)
        end_of = {b: (starts[i + 1] if i + 1 < len(starts) else n) for i, b in enumerate(starts)}
        # state at block entry: {register: fewest loads issued since the load into it}
        at_entry = {(0, None): {}}
        work = [(0, None)]
        slack = {}
        while work:
            b, role = work.pop()
            age = dict(at_entry[(b, role)])
            feasible = True
            for k in range(b, end_of[b]):
                no, t, comment, in_asm = ins[k]
                if t == 'counted-waits':
                    continue
                if t.startswith('role '):
                    if role is not None and role != t[5:]:
                        feasible = False
                        break
                    role = t[5:]
                    continue
                if t.startswith('s_waitcnt'):
                    vmc, _ = _wait_counts(t)
                    if vmc is None:
                        continue
                    if in_asm:
                        regs = sorted(_vregs(comment)) + (['lds'] if 'lds-copies' in comment else [])
                        for r in regs:
                            if r in age:
                                if age[r] < vmc:
                                    found.add((name, no, t, r, age[r]))
                                key = (name, no, vmc)
                                slack[key] = min(slack.get(key, AGE_CAP), age[r] - vmc)
                                del age[r]
                    if vmc == 0:
                        age.clear()
                    continue
                if _VM_LOAD.match(t):
                    for r in age:
                        if age[r] < AGE_CAP:
                            age[r] += 1
                    if in_asm and '_lds_' in t.split()[0]:
                        age['lds'] = 0   # the youngest direct-to-LDS copy (a wait marked `lds-copies` is about it)
                    elif in_asm and 'load' in t.split()[0]:
                        for r in _vregs(t.split(None, 1)[1].split(',')[0]):
                            age[r] = 0
            if not feasible:
                continue
            last = end_of[b] - 1
            for nb in succ_of.get(last, [end_of[b]] if end_of[b] < n else []):
                old = at_entry.get((nb, role))
                if old is None:
                    new = dict(age)
                else:
                    new = dict(old)
                    for r, a in age.items():
                        new[r] = min(a, old[r]) if r in old else a
                if new != old:
                    at_entry[(nb, role)] = new
                    work.append((nb, role))
        if notes is not None:
            notes.extend((k[0], k[1], k[2], v) for k, v in sorted(slack.items()))
    return sorted(found)


def check_file(path):
    with open(path) as f:
        text = f.read()
    bad = violations(text)
    for no, t, regs, dist, writer in bad:
        print(f'{path}:{no}: "{t}" reads s{regs} {dist} slot(s) after "{writer}"', file=sys.stderr)
    early = inflight_violations(text)
    for name, no, t, regs in early:
        print(f'{path}:{no}: {name}: "{t}" touches v{list(regs)} while a load issued from inline asm may still '
              'be writing it', file=sys.stderr)
    late = wait_count_findings(text)
    for name, no, t, reg, behind in late:
        print(f'{path}:{no}: {name}: "{t.split(";")[0].strip()}" names v{reg}, whose load has only {behind} load(s) issued '
              'behind it', file=sys.stderr)
    return len(bad) + len(early) + len(late)


if __name__ == '__main__':
    sys.exit(1 if sum(check_file(p) for p in sys.argv[1:]) else 0)
