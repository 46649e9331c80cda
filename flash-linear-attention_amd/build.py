"""Compiles csrc/*.hip into fla_hip/_C/libgdn_hip.so for gfx950 with hipcc.

    python flash-linear-attention_amd/build.py [--force]

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is
installed.  Objects are rebuilt when their source (or a header) is newer.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
OUT_DIR = os.path.join(HERE, 'fla_hip', '_C')
LIB = os.path.join(OUT_DIR, 'libgdn_hip.so')
OBJ_DIR = os.path.join(HERE, 'build', 'obj')

HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++20', '-fPIC', '-fvisibility=default',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    # keep MFMA accumulators in ordinary VGPRs: the state and the products are read by vector ALU
    # instructions every chunk, and the AGPR form costs a copy per register each time
    '-mllvm', '-amdgpu-mfma-vgpr-form',
    '-Wno-unused-result', '-Wno-unknown-attributes',
]


def _newer(src_list, target):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in src_list)


def _compile(src, obj):
    cmd = [HIPCC, *FLAGS, '-c', src, '-o', obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l)
    if r.returncode != 0:
        raise RuntimeError(f'hipcc failed for {src}:\n{err}')
    if err.strip():
        sys.stderr.write(err + '\n')


def build(force: bool = False, verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, '*.hip')))
    hdrs = sorted(glob.glob(os.path.join(CSRC, '*.h'))) + [os.path.join(HERE, '..', 'include', 'gdn_hip.h')]
    jobs, objs = [], []
    for s in srcs:
        o = os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + '.o')
        objs.append(o)
        if force or _newer([s, *hdrs], o):
            jobs.append((s, o))
    if verbose and jobs:
        print(f'[build] compiling {len(jobs)} file(s) for gfx950', flush=True)
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(lambda a: _compile(*a), jobs))
    if jobs or force or _newer(objs, LIB):
        cmd = [HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB, *objs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f'link failed:\n{r.stderr}')
        if verbose:
            print(f'[build] linked {LIB}', flush=True)
    return LIB


if __name__ == '__main__':
    build(force='--force' in sys.argv)
