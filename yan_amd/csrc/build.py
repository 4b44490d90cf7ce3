#!/usr/bin/env python3
"""Builds yan_amd/csrc/libyan_gemm.so, the ahead-of-time C-ABI library (declared in include/yan_gemm.h), with
hipcc for gfx950. Cross-compiles: needs no GPU. `--force` rebuilds even when the library is newer than its sources."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SRC = os.path.join(HERE, 'yan_gemm_capi.hip')
OUT = os.path.join(HERE, 'libyan_gemm.so')
INCLUDE = os.path.join(ROOT, 'yan_amd', 'include')


def sources():
    return [SRC, os.path.join(ROOT, 'include', 'yan_gemm.h')] + glob.glob(os.path.join(INCLUDE, 'gemm', '*.hpp'))


def up_to_date() -> bool:
    return os.path.exists(OUT) and all(os.path.getmtime(OUT) >= os.path.getmtime(s) for s in sources())


def build(force: bool = False) -> str:
    if not force and up_to_date():
        return OUT
    hipcc = os.getenv('YAN_HIPCC_COMPILER') or os.path.join(os.getenv('ROCM_PATH', '/opt/rocm'), 'bin', 'hipcc')
    cmd = [hipcc, SRC, '-o', OUT + '.tmp', '-std=c++20', '-O3', '--offload-arch=gfx950', '-shared', '-fPIC', '-fno-gpu-rdc',
           '-fvisibility=hidden', '-Wno-unused-command-line-argument',
           '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops', f'-I{INCLUDE}']
    done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    if done.returncode != 0:
        raise RuntimeError(f'hipcc failed:\n{done.stdout[-4000:]}')
    os.replace(OUT + '.tmp', OUT)
    return OUT


if __name__ == '__main__':
    print(build(force='--force' in sys.argv))
