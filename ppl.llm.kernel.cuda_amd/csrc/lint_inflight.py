#!/usr/bin/env python3
"""Build-time check of the hand-scheduled decode kernels.

Their cache loads are inline assembly with explicit wait counts, so the compiler does not know which
registers are the target of a load still in flight.  This script reads the gfx950 assembly of a
translation unit (hipcc -S) and, with the in-order completion model of vector memory operations,
reports every instruction that reads or writes such a register before a wait covers it (a spill, a
copy, a reuse).  It also reports an inline-assembly vector instruction that reads the result of the
transcendental instruction (v_exp_f32, v_rcp_f32, ...) issued directly before it: that use needs a wait
state, which the compiler inserts for its own instructions but not for the opaque text of an asm
statement.  Exit status 1 when it finds either: such a kernel must not run.

    hipcc ... --cuda-device-only -S file.hip -o file.s && python3 lint_inflight.py file.s
"""
import re
import sys


def registers(text):
    out = set()
    for m in re.finditer(r'\bv\[(\d+):(\d+)\]', text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r'(?<![\w\[:])v(\d+)\b', text):
        out.add(int(m.group(1)))
    return out


TRANS = ('v_exp_', 'v_log_', 'v_rcp_', 'v_rsq_', 'v_sqrt_', 'v_sin_', 'v_cos_')
LOADS = ('global_load', 'scratch_load', 'buffer_load', 'flat_load')
STORES = ('global_store', 'scratch_store', 'buffer_store', 'flat_store', 'global_atomic', 'flat_atomic', 'buffer_atomic')


def lint(name, lines):
    queue = []  # outstanding vector memory operations, oldest first: (destination registers, from inline asm)
    in_asm = False
    problems = 0
    hazards = 0
    asm_loads = 0
    trans_dst = set()  # destination of the previous instruction when that was a transcendental one
    for no, raw in enumerate(lines):
        t = raw.strip()
        if t.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if t.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if not t or t.startswith(';') or t.startswith('.') or t.endswith(':'):
            continue
        t = t.split(';')[0].strip()
        op = t.split()[0]
        if in_asm and op.startswith('v_') and ',' in t and registers(t.split(',', 1)[1]) & trans_dst:
            print("  %s:%d: asm instruction reads a transcendental result without a wait state: %s" % (name, no, t[:90]))
            hazards += 1
        trans_dst = registers(t.split(',')[0]) if op.startswith(TRANS) else set()
        if op == 's_waitcnt':
            m = re.search(r'vmcnt\((\d+)\)', t)
            if m:
                del queue[:max(0, len(queue) - int(m.group(1)))]
            continue
        pending = set().union(*[d for d, from_asm in queue if from_asm]) if queue else set()
        if op.startswith(LOADS):
            dst = registers(t.split(',')[0])
            if in_asm:
                asm_loads += 1
                if dst & set().union(*[d for d, _ in queue]) if queue else False:
                    print("  %s:%d: load into a register with a load in flight: %s" % (name, no, t))
                    problems += 1
            elif dst & pending:
                print("  %s:%d: load into a register with a hand-scheduled load in flight: %s" % (name, no, t))
                problems += 1
            if registers(t.split(',', 1)[1] if ',' in t else '') & pending:
                print("  %s:%d: address from a register with a load in flight: %s" % (name, no, t))
                problems += 1
            queue.append((dst, in_asm))
            continue
        if op.startswith(STORES):
            if registers(t) & pending:
                print("  %s:%d: store reads a register with a load in flight: %s" % (name, no, t))
                problems += 1
            queue.append((set(), in_asm))
            continue
        bad = registers(t) & pending
        if bad:
            print("  %s:%d: touches v%s with a load in flight: %s" % (name, no, sorted(bad)[:6], t[:90]))
            problems += 1
    return problems, asm_loads, hazards


def main():
    total = 0
    checked = 0
    for path in sys.argv[1:]:
        src = open(path).read().split('\n')
        i = 0
        while i < len(src):
            m = re.match(r'^(_Z\S+):', src[i])
            if m and '.' not in m.group(1):
                j = i + 1
                while j < len(src) and 's_endpgm' not in src[j]:
                    j += 1
                problems, asm_loads, hazards = lint(m.group(1), src[i:j])
                if asm_loads:
                    checked += 1
                total += (problems if asm_loads else 0) + hazards
                i = j
            i += 1
    print("lint_inflight: %d hand-scheduled kernels checked, %d problems" % (checked, total))
    return 1 if total or not checked else 0


if __name__ == '__main__':
    sys.exit(main())
