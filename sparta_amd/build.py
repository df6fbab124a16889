"""Ahead-of-time build of libsparta_hip.so for gfx950 with hipcc.

Every ``csrc/*.hip`` translation unit is compiled to an object (in parallel) and
linked into ``sparta_amd/lib/libsparta_hip.so``.  Run as
``python -m sparta_amd.build`` or through ``__graft_entry__.build()``.
"""
import concurrent.futures
import os
import re
import shutil
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, 'csrc')
OBJ = os.path.join(ROOT, 'build', 'obj')
LIB_DIR = os.path.join(ROOT, 'lib')
LIB = os.path.join(LIB_DIR, 'libsparta_hip.so')

HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wno-unused-command-line-argument',
]


def _hipcc() -> str:
    exe = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
    if not os.path.exists(exe):
        raise RuntimeError('hipcc not found; a ROCm toolchain is required to build libsparta_hip.so')
    return exe


# Kernels that prefetch into registers through inline assembly (``global_load_dwordx4 %0``
# with an explicit ``s_waitcnt vmcnt(N)`` later) rely on the compiler not touching those
# registers while the loads are in flight.  Nothing in the language promises that: a copy
# the register allocator inserts, or a spill, would read them before the data has arrived.
# Translation units with such loads are therefore compiled with their device assembly kept,
# and the assembly is checked.
_ASM_LOAD_MARKS = ('global_load_dwordx4 %0', 'buffer_load_dwordx4 %0')


def _has_register_prefetch(src: str, _seen=None) -> bool:
    """True if the file, or a header of this directory that it includes (at any depth),
    issues loads into registers through inline assembly."""
    seen = set() if _seen is None else _seen
    if src in seen or not os.path.exists(src):
        return False
    seen.add(src)
    text = open(src).read()
    if any(mark in text for mark in _ASM_LOAD_MARKS):
        return True
    return any(_has_register_prefetch(os.path.join(CSRC, name), seen)
               for name in re.findall(r'#include "([^"]+)"', text))


def _registers(token: str) -> set:
    m = re.match(r'v\[(\d+):(\d+)\]$', token)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r'v(\d+)$', token)
    return {int(m.group(1))} if m else set()


def check_inflight_registers_in_text_order(asm: str) -> list:
    """Scan device assembly for compiler-generated instructions that touch a VGPR between the
    inline-assembly load that targets it and the inline-assembly wait that covers it.

    The text of each kernel is walked in order.  An inline ``global_load_*`` / ``buffer_load_*``
    makes its destination registers pending; a memory instruction of the compiler's own takes
    a place in the same queue; ``s_waitcnt vmcnt(N)``, inline or not, leaves the N newest
    entries pending (vector memory operations retire in order); an unconditional branch or the
    end of the kernel clears the state (what follows in the text is not what runs next).
    Returns a list of (kernel, line number, instruction).
    """
    findings = []
    kernel, pending, in_asm = None, [], False
    for number, line in enumerate(asm.split('\n'), 1):
        m = re.match(r'^(_Z\w+):', line)
        if m:
            kernel, pending = m.group(1), []
            continue
        text = line.strip()
        if kernel is None or not text or text[0] in '.;' and not text.startswith(';;#ASM'):
            continue
        if text.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if text.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if in_asm:
            if text.startswith(('global_load_', 'buffer_load_')):
                # (a load that lands in LDS writes no register but takes its place in the queue)
                pending.append(set() if 'lds' in text.split()[0] else _registers(text.split()[1].rstrip(',')))
            elif text.startswith('s_waitcnt') and 'vmcnt' in text:
                n = int(re.search(r'vmcnt\((\d+)\)', text).group(1))
                pending = pending[len(pending) - n:] if n else []
            continue
        if text.startswith('s_endpgm'):
            kernel = None
            continue
        if text.startswith(('s_branch', 's_setpc')):
            pending = []
            continue
        if text.startswith('s_waitcnt') and 'vmcnt(' in text:
            n = int(re.search(r'vmcnt\((\d+)\)', text).group(1))
            pending = pending[len(pending) - n:] if n else []
            continue
        if not pending:
            continue
        if text.startswith(('global_', 'buffer_', 'scratch_', 'flat_')):
            # a memory instruction of the compiler's own takes a place in the same queue
            pending.append(set())
        used = set()
        for token in re.findall(r'v\[\d+:\d+\]|v\d+', text):
            used |= _registers(token)
        if used & set().union(*pending):
            findings.append((kernel, number, text))
    return findings



STRICT_MARKER = 'spx-uniform-waits'
_LABEL, _WAIT, _ASM_LOAD, _END, _BRANCH, _CBRANCH, _MEM, _OTHER = range(8)


def _parse_kernels(asm: str) -> list:
    """[(kernel, [(line number, kind, payload, registers named)])] with inline-assembly text
    reduced to its loads and waits.  Only kernels that carry the marker comment
    ``spx-uniform-waits`` (emitted by the kernel source through an inline-assembly comment) are
    returned."""
    kernels, body, in_asm, marked = [], None, False, set()
    for number, line in enumerate(asm.split('\n'), 1):
        m = re.match(r'^(_Z\w+):', line)
        if m:
            body, in_asm = [], False
            kernels.append((m.group(1), body))
            continue
        if body is None:
            continue
        label = re.match(r'^(\.L\w+):', line)
        if label:
            body.append((number, _LABEL, label.group(1), None))
            continue
        text = line.strip()
        if STRICT_MARKER in text:
            marked.add(id(body))
            continue
        if text.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if text.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if not text or text[0] in '.;':
            continue
        text = text.split(';')[0].strip()
        wait = re.search(r'vmcnt\((\d+)\)', text) if text.startswith('s_waitcnt') else None
        if wait:
            body.append((number, _WAIT, int(wait.group(1)), None))
        elif in_asm:
            if text.startswith(('global_load_', 'buffer_load_')):
                # a load that lands in LDS writes no register but takes its place in the queue
                to_lds = 'lds' in text.split()[0]
                body.append((number, _ASM_LOAD, frozenset() if to_lds else frozenset(_registers(text.split()[1].rstrip(','))), None))
            elif text.startswith(('global_store_', 'buffer_store_')):
                body.append((number, _ASM_LOAD, frozenset(), None))
        elif text.startswith(('s_endpgm', 's_setpc')):
            body.append((number, _END, text, None))
            if text.startswith('s_endpgm'):
                body = None
        else:
            target = re.match(r's_(c?branch)\w*\s+(\.L\w+)', text)
            if target:
                body.append((number, _BRANCH if target.group(1) == 'branch' else _CBRANCH, target.group(2), None))
                continue
            used = set()
            for token in re.findall(r'v\[\d+:\d+\]|v\d+', text):
                used |= _registers(token)
            kind = _MEM if text.startswith(('global_', 'buffer_', 'scratch_', 'flat_')) else _OTHER
            if used or kind == _MEM:
                body.append((number, kind, text, frozenset(used)))
    return [(name, items) for name, items in kernels if id(items) in marked]


def check_inflight_registers_along_control_flow(asm: str, max_states: int = 500000) -> list:
    """The stricter check, for kernels that declare (marker comment ``spx-uniform-waits``) that
    every path issues the same loads and waits with one fixed count per wait: compiler-generated
    instructions that touch a VGPR between the inline-assembly load that targets it and the
    wait that covers it, on ANY path - feasible or not, the walk does not evaluate conditions,
    which is why a kernel has to be written for it.

    Every kernel is walked along its control flow, not in text order: labels start blocks, a
    conditional branch continues on both sides, an unconditional one only at its target, and a
    (block, queue) pair is walked once.  The queue holds the vector-memory operations in
    flight, oldest first: an inline ``global_load_*`` / ``buffer_load_*`` enters with its
    destination registers, a memory instruction of the compiler's own with none;
    ``s_waitcnt vmcnt(N)``, inline or not, leaves the N newest entries (vector memory
    operations retire in order).  An instruction outside inline assembly that names a register
    of a queued load is a finding - in particular code after a loop that reuses the registers
    of loads the loop left in flight.  Returns a list of (kernel, line number, instruction).
    """
    findings, seen_findings = [], set()
    for kernel, body in _parse_kernels(asm):
        if not any(item[1] == _ASM_LOAD and item[2] for item in body):
            continue
        labels = {item[2]: i for i, item in enumerate(body) if item[1] == _LABEL}
        work, visited = [(0, ())], set()
        while work:
            if len(visited) > max_states:
                raise RuntimeError(f'{kernel}: too many (block, queue) states while checking the register prefetch')
            pos, pending = work.pop()
            pending = list(pending)
            busy = frozenset().union(*pending) if pending else frozenset()
            while pos < len(body):
                number, kind, payload, used = body[pos]
                pos += 1
                if kind == _OTHER:
                    if busy and used & busy and (kernel, number) not in seen_findings:
                        seen_findings.add((kernel, number))
                        findings.append((kernel, number, payload))
                elif kind == _LABEL:
                    # entries older than the oldest pending load carry no information
                    # (and the counter itself holds 63: older operations have retired)
                    pending = pending[-63:]
                    while pending and not pending[0]:
                        pending.pop(0)
                    key = (payload, tuple(pending))
                    if key in visited:
                        break
                    visited.add(key)
                elif kind == _WAIT:
                    pending = pending[len(pending) - payload:] if payload else []
                    busy = frozenset().union(*pending) if pending else frozenset()
                elif kind == _ASM_LOAD:
                    pending.append(payload)
                    busy = busy | payload
                elif kind == _MEM:
                    if busy:
                        if used & busy and (kernel, number) not in seen_findings:
                            seen_findings.add((kernel, number))
                            findings.append((kernel, number, payload))
                        pending.append(frozenset())   # takes a place in the same queue
                elif kind == _CBRANCH:
                    if payload in labels:
                        work.append((labels[payload], tuple(pending)))
                elif kind == _BRANCH:
                    if payload in labels:
                        work.append((labels[payload], tuple(pending)))
                    break
                else:   # _END
                    break
    return findings


def check_inflight_registers(asm: str) -> list:
    """Both checks of the register prefetch: every kernel in text order, and the kernels that
    declare uniform wait counts (the marker comment) along their control flow as well."""
    return check_inflight_registers_in_text_order(asm) + check_inflight_registers_along_control_flow(asm)


def _compile_checked(src: str, obj: str) -> None:
    """Compile with the intermediate files kept (in a scratch directory) and check the device
    assembly the object was assembled from."""
    with tempfile.TemporaryDirectory() as tmp:
        cmd = [_hipcc(), *HIPCC_FLAGS, '-save-temps=cwd', '-c', src, '-o', obj]
        proc = subprocess.run(cmd, capture_output=True, text=True, cwd=tmp)
        if proc.returncode != 0:
            raise RuntimeError(f'hipcc failed on {src}:\n{proc.stderr}')
        listings = [f for f in os.listdir(tmp) if f.endswith('.s') and 'amdgcn' in f]
        if not listings:
            raise RuntimeError(f'no device assembly was kept for {src}; the register prefetch cannot be checked')
        for name in listings:
            findings = check_inflight_registers(open(os.path.join(tmp, name)).read())
            if findings:
                os.remove(obj)
                shown = '\n'.join(f'  {k}: line {n}: {t}' for k, n, t in findings[:20])
                raise RuntimeError(
                    f'{src}: the compiler touches registers that inline-assembly loads are still filling '
                    f'({len(findings)} instructions); restructure the prefetch or lower the register pressure:\n{shown}')


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + '.o')
    if not force and os.path.exists(obj):
        # an object is current when it is newer than its own source and every header
        deps = [src] + [os.path.join(d, f)
                        for d in (CSRC, os.path.join(ROOT, '..', 'include'))
                        for f in os.listdir(d) if f.endswith(('.hpp', '.h'))]
        if os.path.getmtime(obj) >= max(os.path.getmtime(d) for d in deps):
            return obj
    if _has_register_prefetch(src):
        _compile_checked(src, obj)
        return obj
    cmd = [_hipcc(), *HIPCC_FLAGS, '-c', src, '-o', obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f'hipcc failed on {src}:\n{proc.stderr}')
    return obj


def build(force: bool = True, jobs: int = 8, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    sources = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith('.hip'))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), sources))
    cmd = [_hipcc(), '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f'link failed:\n{proc.stderr}')
    if verbose:
        print(f'built {LIB} from {len(sources)} translation units')
    return LIB


if __name__ == '__main__':
    build(force='--incremental' not in sys.argv)
