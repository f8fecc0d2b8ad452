"""Build the CPU oracle (test infrastructure) and, when the reference checkout is present, the compiled reference codec.

  python oracle/build.py            # builds oracle/liborc.so (+ oracle/_ref/libref_kv_codec.so if /root/reference exists)

liborc.so      : oracle/camx_oracle.c with gcc, contraction off (every fma is explicit), OpenMP over rows.
_ref/...       : the reference's kernels/own_kv_codec.h compiled as host C++ from where it lies (never copied), wrapped by
                 a three-line extern "C" shim kept here; the recipe follows the reference's own host test
                 (tests/io/test_own_kv_codec.py:88-96). Needs clang++ (g++ 11 has no _Float16).
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = os.environ.get('CAMX_REFERENCE', '/root/reference')
CLANGXX = os.environ.get('CAMX_CLANGXX', '/opt/rocm/lib/llvm/bin/clang++')
ORC_SO = os.path.join(HERE, 'liborc.so')
REF_DIR = os.path.join(HERE, '_ref')
REF_SO = os.path.join(REF_DIR, 'libref_kv_codec.so')

REF_SHIM = '''#include "own_kv_codec.h"
extern "C" void ref_kv_q8_encode(const float * x, unsigned char * y, unsigned char * ok, long n) {
    for (long i = 0; i < n; i++) ok[i] = own_kv_q8_encode(x + (size_t)i * 32, (OwnKvQ8Block *)(y + (size_t)i * 34));
}
'''


def build_oracle(fast=False, out=None):
    """fast: -O3 -march=native for the benchmark's CPU-baseline leg (same source, same contraction setting), built on the host that
    times it and written to `out` (the tests keep oracle/liborc.so, the -O2 build)"""
    if fast and out is None:
        raise ValueError('the -march=native build goes to a path of its own, never over oracle/liborc.so')
    out = out or ORC_SO
    cmd = ['gcc', '-std=c11', '-O3' if fast else '-O2', '-ffp-contract=off', '-fno-fast-math', '-fopenmp', '-fvisibility=hidden',
           '-shared', '-fPIC', os.path.join(HERE, 'camx_oracle.c'), '-o', out, '-lm']
    if fast: cmd.insert(3, '-march=native')
    subprocess.run(cmd, check=True)
    return out


def build_ref():
    """the compiled reference codec, or None when the checkout or the compiler is absent"""
    hdr = os.path.join(REFERENCE, 'kernels', 'own_kv_codec.h')
    if not os.path.isfile(hdr) or not shutil.which(CLANGXX):
        return None
    os.makedirs(REF_DIR, exist_ok=True)
    shim = os.path.join(REF_DIR, 'ref_kv_codec_shim.cpp')
    with open(shim, 'w') as f:
        f.write(REF_SHIM)
    subprocess.run([CLANGXX, '-std=c++17', '-O3', '-fno-fast-math', '-ffp-contract=off', '-shared', '-fPIC',
                    '-I', os.path.join(REFERENCE, 'kernels'), shim, '-o', REF_SO], check=True)
    return REF_SO


if __name__ == '__main__':
    print(build_oracle())
    print(build_ref())
