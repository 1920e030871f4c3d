"""Compiles the HIP sources in d2dmoe_amd/csrc into d2dmoe_amd/libd2dmoe_hip.so for gfx950 (in-tree).

    python -m d2dmoe_amd.build

hipcc cross-compiles without a GPU.  Packed-FP32 instruction selection is switched off for all device code.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
SOURCES = ('api.hip', 'kernels_generic.hip', 'kernels_mfma.hip', 'kernels_sparse.hip', 'kernels_decode.hip', 'kernels_gemm.hip')
OUTPUT = os.path.join(HERE, 'libd2dmoe_hip.so')
ARCH = 'gfx950'


def hipcc_path() -> str:
    for cand in (os.environ.get('HIPCC'), shutil.which('hipcc'), '/opt/rocm/bin/hipcc'):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError('hipcc not found')


def build(verbose: bool = False) -> str:
    cmd = [hipcc_path(), f'--offload-arch={ARCH}', '-O3', '-std=c++17', '-fPIC', '-shared',
           '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
           *[os.path.join(CSRC, s) for s in SOURCES], '-o', OUTPUT + '.tmp']
    if verbose:
        print(' '.join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    err = '\n'.join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed ({res.returncode}):\n{err}')
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(OUTPUT + '.tmp', OUTPUT)
    return OUTPUT


if __name__ == '__main__':
    print(build(verbose=True))
