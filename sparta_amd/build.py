"""Ahead-of-time build of libsparta_hip.so for gfx950 with hipcc.

Every ``csrc/*.hip`` translation unit is compiled to an object (in parallel) and
linked into ``sparta_amd/lib/libsparta_hip.so``.  Run as
``python -m sparta_amd.build`` or through ``__graft_entry__.build()``.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

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


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + '.o')
    if not force and os.path.exists(obj):
        # an object is current when it is newer than its own source and every header
        deps = [src] + [os.path.join(d, f)
                        for d in (CSRC, os.path.join(ROOT, '..', 'include'))
                        for f in os.listdir(d) if f.endswith(('.hpp', '.h'))]
        if os.path.getmtime(obj) >= max(os.path.getmtime(d) for d in deps):
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
