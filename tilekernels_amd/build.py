"""Ahead-of-time build of libtk_quant.so (hipcc, gfx950 only).

    python -m tilekernels_amd.build [--force]

The library is written to tilekernels_amd/lib/ inside the source tree so that it travels with
the checkout; nothing is JIT-compiled at run time.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, 'csrc')
LIB_DIR = os.path.join(PKG, 'lib')
LIB_PATH = os.path.join(LIB_DIR, 'libtk_quant.so')
SOURCES = ['api.hip', 'per_token_cast.hip', 'per_block_cast.hip', 'swiglu_cast.hip', 'cast_back.hip', 'moe_layout.hip',
           'swiglu_backward.hip', 'per_channel_cast.hip', 'lossless_cast.hip', 'stream_floor.hip', 'swiglu_cast_variants.hip']

HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
FLAGS = [
    '-O3', '-std=c++17', '-fPIC', '--offload-arch=gfx950',
    # every fp32 operation is a single IEEE rounding unless the source asks for an fma
    '-ffp-contract=off', '-fno-fast-math', '-fhip-fp32-correctly-rounded-divide-sqrt',
    '-fno-gpu-flush-denormals-to-zero',
    # keep packed-fp32 VALU instructions out of the generated code
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    # the first 16 dwords of kernel arguments arrive preloaded in SGPRs at wave start
    '-mllvm', '-amdgpu-kernarg-preload-count=16',
    '-Wall', '-Wno-unused-command-line-argument',
]


def _compile(src: str) -> str:
    obj = os.path.join(LIB_DIR, src.replace('.hip', '.o'))
    cmd = [HIPCC, *FLAGS, '-c', os.path.join(CSRC, src), '-o', obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l and 'not a recognized feature' not in l)
    if r.returncode != 0:
        raise RuntimeError(f'hipcc failed on {src}:\n{err}')
    if err.strip():
        sys.stderr.write(err + '\n')
    return obj


def build_library(force: bool = True) -> str:
    """Compile every HIP source and link libtk_quant.so.  Returns its path."""
    if not force and os.path.exists(LIB_PATH):
        return LIB_PATH
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, '-shared', '-fPIC', '--offload-arch=gfx950', '-Wno-unused-command-line-argument', '-o', LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f'link failed:\n{r.stderr}')
    for o in objs:
        os.remove(o)
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(force=True))
