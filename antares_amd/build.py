"""Builds libantares_amd.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m antares_amd.build
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
OUT = os.path.join(CSRC, 'libantares_amd.so')

# packed-FP32 instruction selection is switched off for all device code
FLAGS = ['--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared',
         '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops', '-Wno-unused-result']


def build(verbose: bool = True) -> str:
    sources = sorted(glob.glob(os.path.join(CSRC, '*.hip')))
    cmd = ['hipcc'] + FLAGS + sources + ['-o', OUT + '.tmp', '-lhiprtc']
    if verbose:
        print('[antares_amd.build]', ' '.join(cmd), flush=True)
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = '\n'.join(l for l in p.stderr.splitlines() if 'packed-fp32-ops' not in l)
    if p.returncode != 0:
        raise RuntimeError(f'hipcc failed:\n{p.stdout}\n{err}')
    if err.strip() and verbose:
        print(err)
    os.replace(OUT + '.tmp', OUT)
    return OUT


if __name__ == '__main__':
    build()
    print('built', OUT)
