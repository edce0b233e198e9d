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
    vector-memory instruction inside an inline-asm block that breaks the rule."""
    ins = []
    in_asm = False
    for no, line in enumerate(asm_text.split('\n'), 1):
        t = line.strip()
        if t.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if t.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if not t or t[0] in ';.' or t.endswith(':'):
            continue
        ins.append((no, t.split(';')[0].strip(), in_asm))
    found = []
    for k, (no, t, in_asm) in enumerate(ins):
        if not in_asm or not t.startswith(_VMEM):
            continue
        used = _sregs(t.split(None, 1)[1] if ' ' in t else '')
        if not used:
            continue
        dist = 0
        for j in range(k - 1, -1, -1):
            _, pt, _ = ins[j]
            if dist >= WAIT_STATES:
                break
            if pt.startswith('s_nop'):
                dist += int(pt.split()[1], 0) + 1
                continue
            if pt.startswith(('v_readlane_b32', 'v_readfirstlane_b32')):
                hit = _sregs(pt.split(None, 1)[1].split(',')[0]) & used
                if hit:
                    found.append((no, t, sorted(hit), dist, pt))
                    break
            if pt.startswith(('s_cbranch', 's_branch', 's_endpgm', 's_setpc', 's_swappc')):
                break  # (straight-line distance only; a branch target starts a new count)
            dist += 1
    return found


def check_file(path):
    with open(path) as f:
        bad = violations(f.read())
    for no, t, regs, dist, writer in bad:
        print(f'{path}:{no}: "{t}" reads s{regs} {dist} slot(s) after "{writer}"', file=sys.stderr)
    return len(bad)


if __name__ == '__main__':
    sys.exit(1 if sum(check_file(p) for p in sys.argv[1:]) else 0)
