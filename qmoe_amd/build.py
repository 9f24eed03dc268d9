"""Compiles libsub1_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import re
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
    # registers and scratch memory per kernel, read back below
    '-Rpass-analysis=kernel-resource-usage',
    '-I' + os.path.join(ROOT, 'include'), '-I' + os.path.join(HERE, 'csrc'),
]


def kernels_with_scratch(compiler_output):
    """{kernel: bytes of scratch memory per lane} for the kernels that spill
    registers, from the compiler's resource-usage remarks."""
    found, name = {}, None
    for line in compiler_output.splitlines():
        m = re.search(r'remark: Function Name: (\S+)', line)
        if m:
            name = m.group(1)
        m = re.search(r'remark:\s+ScratchSize \[bytes/lane\]: (\d+)', line)
        if m and name and int(m.group(1)):
            found[name] = int(m.group(1))
    return found


# Kernels known to spill, and how many bytes per lane: the fused kernel's form for
# tokens grouped by expert keeps four tokens' sums per lane.
SPILLS_ACCEPTED = {'_ZN12_GLOBAL__N_125moe_prepared_fused_kernelILb1ELb0EEEvNS_12PreparedArgsE': 36}


def build_library(verbose=False):
    """Builds the library; refuses a build in which a kernel spills registers
    to scratch memory beyond what SPILLS_ACCEPTED lists.  The kernels are
    written to fit their registers (72 to 96 of the 128 that 16 wavefronts per
    compute unit leave a lane), and a spill in a walk costs more than any of
    the tunings measured; one build of the one-token launch that spilled 12
    registers also gave results that differed from run to run (cause not
    established; the code was restructured to fit)."""
    hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
    cmd = [hipcc] + HIPCC_FLAGS + SOURCES + ['-o', LIB_PATH]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError('hipcc failed:\n' + res.stdout)
    spilling = {k: v for k, v in kernels_with_scratch(res.stdout).items()
                if v > SPILLS_ACCEPTED.get(k, 0)}
    if spilling:
        os.remove(LIB_PATH)
        raise RuntimeError('kernels that spill registers to scratch memory: %s' % spilling)
    if verbose:
        print('\n'.join(l for l in res.stdout.splitlines() if 'kernel-resource-usage' not in l
                        and not l.lstrip().startswith(('|', '^')) and '__global__' not in l))
    return LIB_PATH


if __name__ == '__main__':
    print(build_library(verbose=True))
