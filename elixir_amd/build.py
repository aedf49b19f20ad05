"""Builds ``libelx_hip.so`` in-tree with hipcc for gfx950.

    python -m elixir_amd.build

-ffp-contract=off keeps the kernels' arithmetic to the fused multiply-adds that are written out;
packed fp32 instructions are switched off for the device pass.  The digest of the sources is compiled
in (``elx_source_sha``), so that a binding can tell a library built from other sources.
"""
import os
import shutil
import subprocess
import sys

from ._abi import LIB_PATH, built_source_sha, source_sha16

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
SOURCES = [os.path.join(_HERE, 'csrc', 'elx_kernels.hip'), os.path.join(_HERE, 'csrc', 'elx_host.cpp')]
HOST_SOURCE = os.path.join(_HERE, 'csrc', 'elx_host.cpp')
OUTPUT = LIB_PATH

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
    cmd = ([hipcc_path()] + HIPCC_FLAGS + [f'-DELX_SOURCE_SHA="{source_sha16()}"', '-I', os.path.join(_ROOT, 'include'),
                                           '-o', OUTPUT] + SOURCES)
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


def build_host_checked(out_path: str, verbose: bool = False) -> str:
    """The host-only part of the library (table validators, unscale mode, LDS reservation) compiled alone
    by g++ with AddressSanitizer and UBSan, for the tests of the validators: what is accepted or refused
    there is decided by the same source file that is linked into ``libelx_hip.so``."""
    cmd = ['g++', '-std=c++17', '-O1', '-g', '-fPIC', '-shared', '-fno-omit-frame-pointer',
           '-fsanitize=address,undefined', '-fno-sanitize-recover=all', '-Wall', '-Wextra', '-Werror',
           '-I', os.path.join(_ROOT, 'include'), '-o', out_path, HOST_SOURCE]
    if verbose:
        print(' '.join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out_path


def is_stale() -> bool:
    """The built library is missing, or was built from other sources than the ones beside it."""
    return not os.path.exists(OUTPUT) or built_source_sha(OUTPUT) != source_sha16()


def ensure_built(verbose: bool = False) -> str:
    """For test runs, the smoke check and the benchmark: compiles the library when none is there or when
    the one that is there was built from other sources (an edited kernel must never be measured through
    an old binary); a library that matches its sources is loaded as it is.  The product itself never
    builds behind the caller's back: ``elixir_amd._abi.load`` raises when the library is missing or stale."""
    if is_stale():
        if os.path.exists(OUTPUT):
            print(f'{OUTPUT} was built from other sources: rebuilding', file=sys.stderr, flush=True)
        build(verbose=verbose)
    return OUTPUT


if __name__ == '__main__':
    build()
    sys.exit(0)
