"""
Builds libattorch_hip.so (the C-ABI library of gfx950 kernels) in-tree with hipcc.

Usage: ``python -m attorch_amd.build`` or ``attorch_amd.build.build()``.
Each ``csrc/*.hip`` translation unit is compiled to an object file in parallel and the
objects are linked into ``attorch_amd/lib/libattorch_hip.so``.  Nothing here needs a GPU:
hipcc cross-compiles for gfx950.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import List

PKG_DIR = Path(__file__).resolve().parent
SRC_DIR = PKG_DIR / 'csrc'
OBJ_DIR = SRC_DIR / 'build'
LIB_PATH = PKG_DIR / 'lib' / 'libattorch_hip.so'

HIPCC_FLAGS = ['--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC',
               '-Wall', '-Wno-pass-failed', '-Wno-unused-function',
               # packed fp32 VALU forms are kept out of generated code on purpose
               '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']


def find_hipcc() -> str:
    for cand in (os.environ.get('HIPCC'), shutil.which('hipcc'), '/opt/rocm/bin/hipcc'):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError('hipcc not found; set HIPCC or install ROCm under /opt/rocm')


def _run(cmd: List[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = '\n'.join(line for line in proc.stdout.splitlines()
                    if "'-packed-fp32-ops' is not a recognized feature" not in line)
    if proc.returncode != 0:
        raise RuntimeError(f'command failed ({proc.returncode}): {" ".join(cmd)}\n{out}')
    if out.strip():
        print(out, file=sys.stderr)


def build(jobs: int = 8, verbose: bool = True) -> Path:
    """
    Compiles every HIP source for gfx950 and links the shared library.

    Args:
        jobs: Number of translation units compiled at once.
        verbose: Prints one line per step.

    Returns:
        Path of the built shared library.
    """
    hipcc = find_hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    LIB_PATH.parent.mkdir(parents=True, exist_ok=True)
    sources = sorted(SRC_DIR.glob('*.hip'))
    if not sources:
        raise RuntimeError(f'no HIP sources under {SRC_DIR}')

    def compile_one(src: Path) -> Path:
        obj = OBJ_DIR / (src.stem + '.o')
        if verbose:
            print(f'[attorch_amd.build] hipcc {src.name}', file=sys.stderr)
        _run([hipcc, *HIPCC_FLAGS, '-c', str(src), '-o', str(obj)])
        return obj

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objects = list(pool.map(compile_one, sources))

    tmp = LIB_PATH.with_suffix('.so.tmp')
    _run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', str(tmp),
          *[str(o) for o in objects]])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f'[attorch_amd.build] linked {LIB_PATH}', file=sys.stderr)
    return LIB_PATH


if __name__ == '__main__':
    build()
