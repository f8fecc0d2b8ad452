"""Build tests/native/libcpp_caller.so: a C++ caller of the C ABI (host code only: the HIP runtime API, include/camx.h and, as the
checker, the CPU oracle). Linked against caminus_amd/libcamx.so and oracle/liborc.so, found at run time relative to this folder.

  python tests/native/build.py
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
SO = os.path.join(HERE, 'libcpp_caller.so')


def build():
    cmd = [HIPCC, '--offload-arch=gfx950', '-std=c++17', '-O2', '-fPIC', '-shared', '-fvisibility=hidden', '-Wall', '-Wno-unknown-cuda-version',
           os.path.join(HERE, 'cpp_caller.cpp'), '-I', os.path.join(ROOT, 'include'),
           '-L', os.path.join(ROOT, 'caminus_amd'), '-lcamx', '-L', os.path.join(ROOT, 'oracle'), '-lorc',
           '-Wl,-rpath,$ORIGIN/../../caminus_amd', '-Wl,-rpath,$ORIGIN/../../oracle', '-o', SO]
    subprocess.run(cmd, check=True)
    return SO


if __name__ == '__main__':
    print(build())
