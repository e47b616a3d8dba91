"""Static check of gfx950 assembly (hipcc -S) for one hazard of hand-placed LDS reads.

TEST INFRASTRUCTURE. The kernels read MFMA fragments from LDS with inline-assembly ``ds_read_*`` and wait for them with
their own ``s_waitcnt lgkmcnt(N)`` (daceml_amd/csrc/lds_ops.h). The compiler does not know that the destination
registers are written some time AFTER the instruction issues: if a read's result is unused on some path, or a copy is
placed before the wait, the register allocator may give those registers to something else - an address, say - that the
late-arriving LDS data then overwrites. This walks every kernel's control-flow graph with the queue of outstanding LDS
operations as state (they complete in order; ``lgkmcnt(N)`` leaves at most the N youngest outstanding) and reports
every instruction that reads or writes a VGPR while an LDS read into it is outstanding.

Branches are explored independently of their conditions, so a kernel whose wait sits in one of two branches whose
conditions are complementary is reported although it is safe: use the check on code that waits unconditionally."""
import re

_VREG = re.compile(r'(?<![\w\]])v\[(\d+):(\d+)\]|(?<![\w\]])v(\d+)\b')
_LGKM = re.compile(r'lgkmcnt\((\d+)\)')
_RETURNING = ('ds_read', 'ds_bpermute', 'ds_permute', 'ds_swizzle')


def _vregs(text):
    out = set()
    for m in _VREG.finditer(text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return frozenset(out)


def kernels(path):
    """Yield (symbol, [(line number, 'label' | 'ins', text)]) for every function of an assembly file."""
    name, body = None, []
    with open(path) as f:
        for ln, line in enumerate(f, 1):
            s = line.strip()
            m = re.match(r'^(_Z\w+):', s)
            if m:
                if name:
                    yield name, body
                name, body = m.group(1), []
                continue
            if s.startswith(('.end_amdhsa_kernel', '.section', '.Lfunc_end')):
                if name:
                    yield name, body
                name, body = None, []
                continue
            if name is None or not s or s.startswith((';', '//')):
                continue
            m = re.match(r'^(\.LBB\w+):', s)
            if m:
                body.append((ln, 'label', m.group(1)))
                continue
            if s.startswith('.'):
                continue
            code = s.split(';')[0].split('//')[0].strip()
            if code:
                body.append((ln, 'ins', code))
    if name:
        yield name, body


def check_kernel(body):
    """Returns {line: (instruction, registers, lines of the reads in flight)} for one kernel."""
    labels = {b[2]: i for i, b in enumerate(body) if b[1] == 'label'}
    n = len(body)
    seen, work, bad = set(), [(0, ())], {}
    while work:
        i, q = work.pop()
        while i < n:
            if body[i][1] == 'label':
                if (i, q) in seen:
                    break
                seen.add((i, q))
                i += 1
                continue
            ln, _, code = body[i]
            op = code.split()[0]
            rest = code[len(op):]
            if op == 's_waitcnt':
                m = _LGKM.search(code)
                if m:
                    k = int(m.group(1))
                    q = () if k == 0 else q[-k:]
                i += 1
                continue
            if op == 's_endpgm':
                break
            pending = frozenset().union(*[e[0] for e in q]) if q else frozenset()
            is_read = op.startswith('ds_read')
            # a later LDS read into the same registers completes after the earlier one: only its address matters
            touched = _vregs(','.join(rest.split(',')[1:])) if is_read else _vregs(rest)
            if touched & pending:
                bad.setdefault(ln, (code, sorted(touched & pending), [e[1] for e in q if e[0] & touched]))
            if op.startswith('ds_'):
                dst = _vregs(rest.split(',')[0]) if op.startswith(_RETURNING) else frozenset()
                q = (q + ((dst, ln), ))[-64:]
            elif op.startswith(('s_load', 's_buffer_load')):
                q = (q + ((frozenset(), ln), ))[-64:]
            if op == 's_branch':
                i = labels.get(rest.strip(), n)
                continue
            if op.startswith('s_cbranch') and rest.strip() in labels:
                work.append((labels[rest.strip()], q))
            i += 1
    return bad


def check_file(path):
    """Returns (number of kernels, {symbol: hazards}) with only the kernels that have any."""
    count, found = 0, {}
    for name, body in kernels(path):
        count += 1
        bad = check_kernel(body)
        if bad:
            found[name] = bad
    return count, found


_WIDE_STORE = re.compile(r'^(global|flat|buffer|scratch)_store_(dwordx3|dwordx4|b96|b128)\b')
_VALU_OR_LOAD = re.compile(r'^(v_|ds_read|ds_bpermute|global_load|flat_load|buffer_load|scratch_load)')


def check_store_data(path):
    """A second hazard of the same kind. A memory store of more than 64 bits reads its data registers up to two wait
    states after it issues; the compiler's hazard recognizer keeps vector writes to those registers away for that long,
    but it does not look into inline assembly. Reports, per kernel, every store of more than 64 bits that sits in an
    inline-assembly block (between #ASMSTART and #ASMEND markers the compiler writes) and is not followed, inside the
    block, by ``s_nop 1`` or more. Returns {kernel: [line numbers]}."""
    found = {}
    name, in_asm, pending = None, False, None
    with open(path) as f:
        for ln, line in enumerate(f, 1):
            s = line.strip()
            m = re.match(r'^(_Z\w+):', s)
            if m:
                name, in_asm, pending = m.group(1), False, None
                continue
            if name is None:
                continue
            if '#ASMSTART' in s:
                in_asm, pending = True, None
                continue
            if '#ASMEND' in s:
                if pending is not None:
                    found.setdefault(name, []).append(pending)
                in_asm, pending = False, None
                continue
            if not in_asm:
                continue
            code = s.split(';')[0].strip()
            if not code:
                continue
            if pending is not None:
                m = re.match(r'^s_nop\s+(\d+)', code)
                if m and int(m.group(1)) >= 1:
                    pending = None
                else:
                    found.setdefault(name, []).append(pending)
                    pending = None
            if _WIDE_STORE.match(code):
                pending = ln
    return found
