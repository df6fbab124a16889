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


def check_inflight_registers(asm: str) -> list:
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
            if text.startswith(('global_load_', 'buffer_load_')) and 'lds' not in text.split()[0]:
                pending.append(_registers(text.split()[1].rstrip(',')))
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
