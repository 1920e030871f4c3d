"""Compiles the HIP sources in d2dmoe_amd/csrc into d2dmoe_amd/libd2dmoe_hip.so for gfx950 (in-tree).

    python -m d2dmoe_amd.build

hipcc cross-compiles without a GPU.  Packed-FP32 instruction selection is switched off for all device code.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
SOURCES = ('api.hip', 'kernels_generic.hip', 'kernels_mfma.hip', 'kernels_dense_wide.hip', 'kernels_sparse.hip', 'kernels_decode.hip', 'kernels_gemm.hip', 'kernels_norms.hip', 'kernels_mid.hip')
OUTPUT = os.path.join(HERE, 'libd2dmoe_hip.so')
ARCH = 'gfx950'


def hipcc_path() -> str:
    for cand in (os.environ.get('HIPCC'), shutil.which('hipcc'), '/opt/rocm/bin/hipcc'):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError('hipcc not found')


def _run(cmd, verbose):
    if verbose:
        print(' '.join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    err = '\n'.join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f'hipcc failed ({res.returncode}):\n{err}')
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False) -> str:
    """One object per source, compiled side by side (a handful of processes), then one link."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = hipcc_path()
    flags = [f'--offload-arch={ARCH}', '-O3', '-std=c++17', '-fPIC', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']
    objdir = tempfile.mkdtemp(prefix='d2dmoe_build_')
    try:
        objs = [os.path.join(objdir, s.replace('.hip', '.o')) for s in SOURCES]
        jobs = [[hipcc, *flags, '-c', os.path.join(CSRC, s), '-o', o] for s, o in zip(SOURCES, objs)]
        with ThreadPoolExecutor(max_workers=min(len(jobs), max(1, min(os.cpu_count() or 1, 8)))) as pool:
            list(pool.map(lambda c: _run(c, verbose), jobs))
        _run([hipcc, f'--offload-arch={ARCH}', '-shared', '-fPIC', *objs, '-o', OUTPUT + '.tmp'], verbose)
    finally:
        shutil.rmtree(objdir, ignore_errors=True)
    os.replace(OUTPUT + '.tmp', OUTPUT)
    return OUTPUT


if __name__ == '__main__':
    print(build(verbose=True))
