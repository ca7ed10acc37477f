#!/usr/bin/env python3
"""Static check of gfx950 device assembly for one hazard of hand-issued loads.

The recurrence kernels request their operand fragments (`global_load_dwordx4 ... sc1`) and the operands they stream
from memory (`... nt`) in inline assembly and wait for them later with an explicit `s_waitcnt vmcnt(n)`.  The compiler does not know that the destination registers are
still being written in between; if it copies, reads or reuses them there (a copy at a join of two definitions, a split
live range) the kernel multiplies garbage.  This script walks the control-flow graph of the assembly from every such
load and reports any instruction that names a destination register on a path before the first wait for vector memory.
Branches on flags that the path itself has set to a constant are followed only the way the flag points.

usage: check_inflight.py file.s [...]      exit status 1 if a hazard is found
"""
import re
import sys

# hand-issued loads carry a cache policy the compiler never emits for its own loads of these kernels: sc1 (device
# scope: the exchanged fragments) or nt (the operands streamed from memory one or two phases ahead)
LOAD = re.compile(r'^\s+global_load_dword(?:x2|x4)? v\[(\d+):(\d+)\], .*\b(?:sc1|nt)\s*$')
LABEL = re.compile(r'^([.\w$]+):')
REG = re.compile(r'\bv\[(\d+):(\d+)\]|\bv(\d+)\b')


SPAIR = re.compile(r'^s\[(\d+):(\d+)\]$')
SREG = re.compile(r'^s(\d+)$')


def check(path):
    lines = open(path).read().split('\n')
    label_at = {}
    for i, l in enumerate(lines):
        m = LABEL.match(l)
        if m:
            label_at[m.group(1)] = i
    hazards = []

    # The compiler lowers structured control flow to flags: a block sets a pair of scalar registers to 0 or -1 and a
    # later block branches on `exec & flag`.  Paths are followed with the flags that are known constants (and what
    # they make of vcc), so that a path the flags rule out is not walked.
    def step(i, known, vcc):
        """-> list of (next line, known, vcc) after executing line i"""
        t = lines[i].split(';')[0].strip()
        if not t or t.startswith('.') or LABEL.match(lines[i]):
            return [(i + 1, known, vcc)]
        parts = t.replace(',', ' ').split()
        op, ops = parts[0], parts[1:]
        if op == 's_endpgm':
            return []
        if op == 's_branch':
            return [(label_at[ops[0]], known, vcc)] if ops[0] in label_at else []
        if op.startswith('s_cbranch'):
            tgt = label_at.get(ops[0])
            taken = None
            if op == 's_cbranch_vccnz' and vcc is not None:
                taken = (vcc == 'nz')
            if op == 's_cbranch_vccz' and vcc is not None:
                taken = (vcc == 'z')
            out = []
            if taken is not True:
                out.append((i + 1, known, vcc))
            if taken is not False and tgt is not None:
                out.append((tgt, known, vcc))
            return out
        # writes: the first operand (conservatively also for compares, whose first operand is only read)
        if ops:
            d = ops[0]
            if d == 'vcc' or d.startswith('vcc_'):
                vcc = None
                if op in ('s_andn2_b64', 's_and_b64') and len(ops) == 3 and ops[1] == 'exec':
                    m = SPAIR.match(ops[2])
                    if m and (int(m.group(1)), int(m.group(2))) in known:
                        val = known[(int(m.group(1)), int(m.group(2)))]
                        vcc = ('nz' if val == 0 else 'z') if op == 's_andn2_b64' else ('z' if val == 0 else 'nz')
            m = SPAIR.match(d)
            m1 = SREG.match(d)
            if m or m1:
                lo, hi = (int(m.group(1)), int(m.group(2))) if m else (int(m1.group(1)), int(m1.group(1)))
                known = {k: v for k, v in known.items() if k[1] < lo or k[0] > hi}
                if op == 's_mov_b64' and m and len(ops) == 2:
                    if ops[1] in ('0', '-1'):
                        known = dict(known)
                        known[(lo, hi)] = 0 if ops[1] == '0' else -1
                    else:
                        ms = SPAIR.match(ops[1])
                        if ms and (int(ms.group(1)), int(ms.group(2))) in known:
                            known = dict(known)
                            known[(lo, hi)] = known[(int(ms.group(1)), int(ms.group(2)))]
        return [(i + 1, known, vcc)]

    for i, l in enumerate(lines):
        m = LOAD.match(l)
        if not m:
            continue
        a, b = int(m.group(1)), int(m.group(2))
        seen = set()
        stack = step(i, {}, None)
        while stack:
            k, known, vcc = stack.pop()
            key = (k, tuple(sorted(known.items())), vcc)
            if key in seen or k >= len(lines):
                continue
            seen.add(key)
            t = lines[k].strip()
            if not t or t.startswith(';') or t.startswith('.') or LABEL.match(lines[k]):
                stack.extend(step(k, known, vcc))
                continue
            if t.startswith('s_waitcnt') and 'vmcnt' in t:
                continue   # the path ends at the first wait for vector memory
            m2 = LOAD.match(lines[k])
            if m2 and int(m2.group(1)) == a and int(m2.group(2)) == b:
                continue   # requested again into the same registers (a reload loop)
            code = t.split(';')[0]
            hit = False
            for r in REG.finditer(code):
                lo = int(r.group(1) or r.group(3))
                hi = int(r.group(2) or r.group(3))
                if lo <= b and hi >= a:
                    hazards.append((i + 1, a, b, k + 1, code.strip()))
                    hit = True
                    break
            if hit:
                continue   # (one report per path)
            stack.extend(step(k, known, vcc))
    for h in hazards[:40]:
        print('%s: load at line %d into v[%d:%d] is in flight when line %d runs: %s' % ((path,) + h))
    return len(hazards)


if __name__ == '__main__':
    total = sum(check(p) for p in sys.argv[1:])
    print('check_inflight: %d hazard(s)' % total)
    sys.exit(1 if total else 0)
