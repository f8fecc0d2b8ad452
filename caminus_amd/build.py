"""Compile the HIP sources under caminus_amd/csrc into libcamx.so for gfx950 (in-tree, next to this file).

  python -m caminus_amd.build

Flags: contraction off (every fused multiply-add in the kernels is an explicit fma), IEEE divide and square root (hipcc's
default), packed-fp32 instruction selection off.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB = os.path.join(HERE, 'libcamx.so')
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
FLAGS = ['--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared', '-ffp-contract=off', '-fno-fast-math',
         '-fhip-fp32-correctly-rounded-divide-sqrt', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
         '-Wall', '-Wno-unused-function', '-Wno-unknown-cuda-version']


def sources():
    return sorted(glob.glob(os.path.join(CSRC, '*.hip')))


def build(verbose=False):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, 'build'), exist_ok=True)
    for src in sources():
        obj = os.path.join(HERE, 'build', os.path.basename(src)[:-4] + '.o')
        cmd = [HIPCC] + [f for f in FLAGS if f != '-shared'] + ['-c', src, '-o', obj, '-I', CSRC, '-I', os.path.join(os.path.dirname(HERE), 'include')]
        if verbose: print(' '.join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    bad = False
    for src, p in procs:
        out, _ = p.communicate()
        out = '\n'.join(l for l in out.splitlines() if "is not a recognized feature" not in l and l.strip())
        if out and (verbose or p.returncode): print(out, flush=True)
        if p.returncode: bad = True; print(f'FAILED: {src}', file=sys.stderr)
    if bad: raise RuntimeError('hipcc failed')
    subprocess.run([HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB] + objs, check=True)
    return LIB


if __name__ == '__main__':
    print(build(verbose='-v' in sys.argv))
