"""Builds ``libelx_hip.so`` in-tree with hipcc for gfx950.

    python -m elixir_amd.build

-ffp-contract=off keeps the kernels' arithmetic to the fused multiply-adds that are written out;
packed fp32 instructions are switched off for the device pass.
"""
import os
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
SOURCES = [os.path.join(_HERE, 'csrc', 'elx_kernels.hip')]
OUTPUT = os.path.join(_HERE, 'libelx_hip.so')

HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared', '-ffp-contract=off', '-Xclang', '-target-feature',
    '-Xclang', '-packed-fp32-ops', '-Wno-unused-command-line-argument'
]


def hipcc_path() -> str:
    for cand in (shutil.which('hipcc'), '/opt/rocm/bin/hipcc'):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError('hipcc not found: the HIP extension cannot be built')


def build(verbose: bool = True) -> str:
    cmd = [hipcc_path()] + HIPCC_FLAGS + ['-I', os.path.join(_ROOT, 'include'), '-o', OUTPUT] + SOURCES
    if verbose:
        print(' '.join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so; that is harmless
    out = '\n'.join(l for l in proc.stdout.splitlines() if 'packed-fp32-ops' not in l)
    if proc.returncode != 0:
        raise RuntimeError(f'hipcc failed ({proc.returncode}):\n{out}')
    if verbose and out.strip():
        print(out)
    return OUTPUT


def ensure_built(verbose: bool = False) -> str:
    """For test runs, the smoke check and the benchmark: compiles the library only when no built one is
    there (a tree that was never built).  The product itself never builds behind the caller's back:
    ``elixir_amd._abi.load`` raises when the library is missing."""
    if not os.path.exists(OUTPUT):
        build(verbose=verbose)
    return OUTPUT


if __name__ == '__main__':
    build()
    sys.exit(0)
