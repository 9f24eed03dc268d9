"""Compiles libsub1_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_PATH = os.path.join(HERE, 'libsub1_hip.so')
SOURCES = [os.path.join(HERE, 'csrc', 'sub1_kernels.hip'),
           os.path.join(HERE, 'csrc', 'sub1_prepared.hip'),
           os.path.join(HERE, 'csrc', 'sub1_tiles.hip'),
           os.path.join(HERE, 'csrc', 'sub1_tables.cpp')]

HIPCC_FLAGS = [
    '-O3', '--offload-arch=gfx950', '-fPIC', '-shared', '-std=c++17',
    # keep the compiler from forming packed fp32 instructions
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-I' + os.path.join(ROOT, 'include'), '-I' + os.path.join(HERE, 'csrc'),
]


def build_library(verbose=False):
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    cmd = [hipcc] + HIPCC_FLAGS + SOURCES + ['-o', LIB_PATH]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError('hipcc failed:\n' + res.stdout)
    if verbose:
        print(res.stdout)
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(verbose=True))
