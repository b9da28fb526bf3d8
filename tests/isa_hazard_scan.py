"""Scans the gfx950 assembly hipcc generates for the matrix-core kernels for reads of an MFMA destination that follow
the MFMA by fewer wait states than the result latency, following both directions of every branch.

Why it exists: the compiler's own hazard handling lost track of a matrix instruction whose result read it had sunk
behind the branches of a loop (single-tile decode kernel: rows 4 kq + 3 came out wrong).  The kernels now avoid the
pattern; this check keeps it from coming back unnoticed.  One instruction = one wait state, `s_nop N` = N + 1, as in
the compiler's own model; the thresholds are the ones the compiler applies in straight-line code on this target
(4-pass 16x16x32: 8, 8-pass 32x32x16: 12, the 8-pass fp32 16x16x4 outside the dense-math pipe: 10).  A dependent MFMA that takes the result as its C operand is interlocked
by the hardware and is not a finding."""
import re

_REG = re.compile(r'\b([av])\[(\d+):(\d+)\]|\b([av])(\d+)\b')
NEED = {"16x16x32": 8, "32x32x16": 12, "16x16x4_f32": 10}


def _regs(tok):
    out = set()
    for m in _REG.finditer(tok):
        if m.group(1):
            out |= {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
        else:
            out.add((m.group(4), int(m.group(5))))
    return out


def _need(mfma):
    for k, v in NEED.items():
        if k in mfma:
            return v
    return max(NEED.values())


def scan(text):
    """Returns a list of (function, wait_states, mfma, reader)."""
    findings = []
    lines = text.split('\n')
    i = 0
    while i < len(lines):
        m = re.match(r'^(_Z\w+):', lines[i])
        if not m:
            i += 1
            continue
        name = m.group(1)
        j = i + 1
        ins, labels = [], {}
        while j < len(lines) and not lines[j].strip().startswith('s_endpgm'):
            s = lines[j].split(';')[0].strip()
            j += 1
            if not s:
                continue
            lm = re.match(r'^(\.LBB\w+):', s)
            if lm:
                labels[lm.group(1)] = len(ins)
            elif not s.startswith('.'):
                ins.append(s)
        i = j + 1

        def succ(k):
            parts = ins[k].split()
            if parts[0] == 's_branch':
                return [labels[parts[1]]] if parts[1] in labels else []
            if parts[0].startswith('s_cbranch'):
                return ([labels[parts[1]]] if parts[1] in labels else []) + [k + 1]
            return [k + 1]

        for k, s in enumerate(ins):
            if not s.startswith('v_mfma'):
                continue
            need = _need(s)
            dst = _regs(s.split(None, 1)[1].split(',')[0])
            stack = [(n, 0) for n in succ(k)]
            seen = {}
            while stack:
                n, w = stack.pop()
                if n >= len(ins) or w >= need or seen.get(n, 1 << 30) <= w:
                    continue
                seen[n] = w
                t = ins[n]
                op = t.split()[0]
                rest = t.split(None, 1)[1] if ' ' in t else ''
                if op == 's_nop':
                    stack += [(x, w + int(rest) + 1) for x in succ(n)]
                    continue
                ops = rest.split(',')
                if op.startswith('v_mfma'):
                    if _regs(','.join(ops[1:3])) & dst:       # result used as an A / B operand
                        findings.append((name, w, s, t))
                    if _regs(ops[0]) & dst:                   # overwritten (dependent chain): interlocked
                        continue
                elif op.startswith(('ds_write', 'global_store', 'buffer_store', 'scratch_store')):
                    if _regs(rest) & dst:
                        findings.append((name, w, s, t))
                        continue
                elif op.startswith('v_'):
                    if _regs(','.join(ops[1:])) & dst:
                        findings.append((name, w, s, t))
                        continue
                stack += [(x, w + 1) for x in succ(n)]
    return findings
