"""Reads the compiler's output (gfx950 assembly of this package's own kernels) for what hand-written waits promise.

Kernels that write MFMAs and LDS reads as instructions count their waits by hand; the compiler neither sees the
latency of such an instruction nor keeps other uses of its registers away.  This walks every path through a function
with a small model of the counters and reports
 (1) an instruction that touches a register while an LDS read into it is still out by the count of s_waitcnt lgkmcnt
     (scalar loads are left out of the count: they may return out of order, so the model takes the careful side),
 (2) an instruction other than an MFMA that touches an MFMA's result before the wait states it needs have passed
     (an MFMA behind another goes out when the matrix pipe has finished the passes of the one before),
 (3) in loops that wait for direct loads into LDS by count in front of a barrier: that the loads which the wait
     leaves in flight were all issued behind the last direct load of the stage that is read next (loads return in
     order; `stages` is the number of LDS stages the loop rotates through).
Used by tests/test_kernel_waits.py; no product code imports it."""
import re, sys
from collections import deque

NEED = {'32x32x16': 11, '16x16x32': 7, '32x32x8': 19, '16x16x16': 11}  # wait states issue -> result readable (8/4/16/8 passes)
PASSES = {'32x32x16': 8, '16x16x32': 4, '32x32x8': 16, '16x16x16': 8}

reg_re = re.compile(r'\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]')

def regs_of(tok):
    out = set()
    for m in reg_re.finditer(tok):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            for k in range(int(m.group(4)), int(m.group(5)) + 1):
                out.add((m.group(3), k))
    return out

def parse(path):
    funcs, cur, name = {}, None, None
    for raw in open(path):
        line = raw.split(';')[0].rstrip()
        if not line.strip():
            continue
        m = re.match(r'^(_Z\w+):', line)
        if m:
            name = m.group(1); cur = []; funcs[name] = cur; continue
        if cur is None:
            continue
        if re.match(r'^\.Lfunc_end', line):
            cur = None; continue
        m = re.match(r'^(\.LBB\d+_\d+):', line)
        if m:
            cur.append(('label', m.group(1))); continue
        s = line.strip()
        if s.startswith('.'):
            continue
        cur.append(('ins', s))
    return funcs

def audit(name, items, verbose=True):
    # basic blocks
    label_at = {}
    for i, (k, v) in enumerate(items):
        if k == 'label':
            label_at[v] = i
    n = len(items)
    problems = []
    seen = {}
    # state: (lds fifo tuple of frozenset regs, mfma pending tuple of (ready_time_rel...)) -- times relative: keep 'age'
    # we keep: lds = tuple of frozensets; mf = tuple of (frozenset regs, remaining wait states); pipe = states until the matrix pipe takes the next MFMA
    work = deque([(0, (), (), 0)])
    visits = {}
    while work:
        pc, lds, mf, pipe = work.pop()
        while pc < n:
            kind, text = items[pc]
            if kind == 'label':
                key = (pc, lds, tuple((r, min(w, 32)) for r, w in mf), min(pipe, 32))
                if key in seen:
                    break
                seen[key] = 1
                visits[pc] = visits.get(pc, 0) + 1
                if visits[pc] > 64:
                    break
                pc += 1
                continue
            ins = text
            op = ins.split()[0]
            args = ins[len(op):]
            toks = [t.strip() for t in args.split(',')] if args.strip() else []
            dst = regs_of(toks[0]) if toks else set()
            srcs = set()
            for t in toks[1:]:
                srcs |= regs_of(t)
            is_store = op.startswith(('ds_write', 'buffer_store', 'global_store', 'scratch_store', 'flat_store', 'ds_store'))
            if is_store or op.startswith(('buffer_load', 'global_load', 'scratch_load')) and 'lds' in ins.split():
                srcs |= dst
                dst = set()
            if op.startswith(('s_', 'v_cmp', 'v_cmpx')) and not op.startswith('s_waitcnt'):
                # scalar op / compare: may read vgprs (v_cmp, v_readlane..)
                if op.startswith('v_cmp'):
                    srcs |= dst; dst = set()
            touched = dst | srcs
            adv = 1
            if op == 's_nop':
                adv = int(toks[0], 0) + 1
            is_mfma = op.startswith('v_mfma')
            # ---- (1) outstanding LDS reads
            if op == 's_waitcnt':
                m = re.search(r'lgkmcnt\((\d+)\)', ins)
                if m:
                    k = int(m.group(1))
                    if len(lds) > k:
                        lds = lds[len(lds) - k:] if k else ()
                if re.fullmatch(r's_waitcnt\s+(0x)?[0-9a-f]+', ins):
                    v = int(ins.split()[1], 0)
                    k = (v >> 8) & 15
                    if len(lds) > k:
                        lds = lds[len(lds) - k:] if k else ()
            else:
                for pend, origin in lds:
                    if pend & touched:
                        problems.append((origin, 'LDS read at item %d (%s) still out at' % (origin, items[origin][1]), '%d: %s' % (pc, ins), sorted(pend & touched)[:4]))
                        break
            # ---- (2) MFMA results
            if is_mfma:
                shape = re.search(r'(\d+x\d+x\d+)', op).group(1)
                # the matrix pipe takes this MFMA when the one before has made its passes
                stall = pipe
                mf = tuple((r, w - stall) for r, w in mf if w - stall > 0)
                # srcA/B from an MFMA result too early? srcC exact overlap is the hardware's business
                a_b = set()
                for t in toks[1:3]:
                    a_b |= regs_of(t)
                for r, w in mf:
                    if r & a_b:
                        problems.append((pc, 'MFMA->MFMA A/B', ins, sorted(r & a_b)[:4]))
                    c = regs_of(toks[3]) if len(toks) > 3 else set()
                    if (r & c) and r != c:
                        problems.append((pc, 'MFMA->MFMA C partly', ins, sorted(r & c)[:4]))
                    if (r & dst) and r != dst:
                        problems.append((pc, 'MFMA->MFMA D partly', ins, sorted(r & dst)[:4]))
                mf = tuple((r, w) for r, w in mf if not (r == dst)) + ((frozenset(dst), NEED[shape]),)
                pipe = PASSES[shape]
                adv = 1
            elif op != 's_waitcnt':
                for r, w in mf:
                    if r & touched:
                        problems.append((pc, 'MFMA %d short' % w, ins, sorted(r & touched)[:4]))
            if not is_mfma:
                pass
            # time passes
            mf = tuple((r, w - adv) for r, w in mf if w - adv > 0)
            pipe = max(0, pipe - adv)
            # new LDS read
            if op.startswith('ds_read'):
                lds = lds + ((frozenset(dst), pc),)
            elif op.startswith(('ds_write', 'ds_store', 'ds_')) and not op.startswith('ds_read'):
                lds = lds + ((frozenset(), pc),)
            # control flow
            if op == 's_endpgm':
                break
            if op == 's_branch':
                pc = label_at[toks[0]]
                continue
            if op.startswith('s_cbranch'):
                work.append((label_at[toks[0]], lds, mf, pipe))
            if op == 's_barrier':
                pass
            pc += 1
    uniq = {}
    for p in problems:
        uniq.setdefault((p[0], p[1].split()[0]), p)
    if verbose:
        print(f'{name[:90]}: {len(uniq)} findings')
        for (pc, _), p in sorted(uniq.items())[:40]:
            print('   item %d: %s: %s  regs %s' % (pc, p[1], p[2], p[3]))
    return uniq



def _loops(items):
    lab = {v: i for i, (k, v) in enumerate(items) if k == 'label'}
    out = []
    for i, (k, t) in enumerate(items):
        if k == 'ins':
            m = re.match(r's_c?branch\S*\s+(\.LBB\d+_\d+)', t)
            if m and lab.get(m.group(1), 1 << 30) < i:
                out.append((lab[m.group(1)], i))
    return out


def _memory_sequence(items, a, b):
    s = []
    for k, t in items[a:b]:
        if k != 'ins':
            continue
        if t.startswith('buffer_load') and t.split()[-1] == 'lds':
            s.append('D')
        elif t.startswith(('buffer_load', 'global_load', 'scratch_load', 'buffer_store', 'global_store', 'scratch_store')):
            s.append('R')
        elif t.startswith('s_waitcnt'):
            m = re.search(r'vmcnt\((\d+)\)', t)
            if m:
                s.append('W%d' % int(m.group(1)))
        elif t.startswith('s_barrier'):
            s.append('B')
    return s


def direct_load_counts(items, stages):
    """[(loop start, loop end, loads left in flight N, loads issued behind the last direct load needed)] for every
    counted wait (N > 0) that stands in front of a barrier in a loop with direct loads, in the loop's steady state."""
    out = []
    for a, b in _loops(items):
        s = _memory_sequence(items, a, b)
        if 'B' not in s or 'D' not in s:
            continue
        # only loops all of whose barriers stand behind a counted wait (a barrier on a side path, behind a full
        # wait, would be counted as a stage), and no loop around other loops
        if any(a < a2 and b2 < b for a2, b2 in _loops(items)):
            continue
        if any(x == 'B' and not (i > 0 and s[i - 1].startswith('W') and s[i - 1] != 'W0') for i, x in enumerate(s)):
            continue
        rep = s * (stages + 3)
        for i in range(len(s) * (stages + 1), len(s) * (stages + 2)):
            if rep[i] != 'B':
                continue
            j = i - 1
            while j >= 0 and rep[j] in ('D', 'R'):
                j -= 1
            if j < 0 or not rep[j].startswith('W'):
                continue
            n = int(rep[j][1:])
            if n == 0:
                continue
            k, crossed, found = i, 0, None
            while k > 0:
                k -= 1
                if rep[k] == 'B':
                    crossed += 1
                    if crossed > stages - 2:
                        break
                if crossed == stages - 2 and rep[k] == 'D':
                    found = k
                    break
            behind = -1 if found is None else sum(1 for x in rep[found + 1:j] if x in 'DR')
            out.append((a, b, n, behind))
    return out


if __name__ == '__main__':
    fs = parse(sys.argv[1])
    pick = sys.argv[2] if len(sys.argv) > 2 else ''
    for nm, items in fs.items():
        if pick in nm:
            audit(nm, items)
            print('   direct loads:', direct_load_counts(items, 4))
