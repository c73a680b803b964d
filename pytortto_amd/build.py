"""Builds ``libtortto_hip.so`` (gfx950 only) from ``csrc/*.hip`` with hipcc.

    python -m pytortto_amd.build        # compile every source, link, report

Objects go to ``csrc/build/`` and the library to ``pytortto_amd/lib/``; both are kept out of
version control but travel with the working tree.  hipcc cross-compiles, so no GPU is needed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

from pytortto_amd._paths import CSRC, LIB_DIR, LIB_PATH, OBJ_DIR

ARCH = 'gfx950'
# packed-fp32 instructions are switched off for the device code of every kernel in this library
HIPCC_FLAGS = ['--offload-arch=' + ARCH, '-O3', '-std=c++17', '-fPIC', '-Wall', '-Wno-unused-function',
               '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith('.hip'))


def _compile(src, verbose):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + '.o')
    cmd = ['hipcc', *HIPCC_FLAGS, '-c', src, '-o', obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only target feature and says so; nothing else is filtered
    err = '\n'.join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed for {src}:\n{err}')
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return obj


def build_library(verbose=False, jobs=None):
    """Compile every HIP source and link the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), os.cpu_count() or 1, 8)
    with ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), srcs))
    tmp = LIB_PATH + '.tmp'
    cmd = ['hipcc', '--offload-arch=' + ARCH, '-shared', '-fPIC', '-o', tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f'link failed:\n{res.stderr}')
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(verbose=True))
