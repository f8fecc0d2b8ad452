#!/usr/bin/env python3
"""Writes tests/golden/kv_q8_blocks.npz: Q8 KV wire blocks encoded by the REFERENCE's own encoder.

The encoder is the reference header kernels/own_kv_codec.h, compiled for the host from where it lies in the reference
checkout by oracle/build.py (never copied here); this script runs in a container that has the checkout and commits only
the resulting data. Inputs: the reference's fixed regression blocks and the first blocks of its seeded generator
(tests/io/test_own_kv_codec.py:24-68, restated in tests/vectors.py), then the blocks its encoder must refuse.

  x   float32 [n, 32]   inputs
  raw uint8   [n, 34]   encoder output; a refused block keeps the 0xa5 fill
  ok  uint8   [n]       1 = encoded, 0 = refused

  python tests/golden/make_kv_q8_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.dirname(os.path.dirname(HERE)), os.path.dirname(HERE)]

import oracle as O                      # noqa: E402
from oracle import build as B           # noqa: E402
from vectors import kv_invalid_blocks, kv_valid_blocks    # noqa: E402

N_VALID = 13 + 1024                     # every fixed block + 1024 generator blocks


def main():
    if B.build_ref() is None:
        raise SystemExit('the reference checkout (or clang++) is absent: the golden file can only be made where it is present')
    x = np.concatenate([kv_valid_blocks()[:N_VALID], kv_invalid_blocks()]).astype(np.float32)
    raw, ok = O.ref_kv_q8_encode(x)
    out = os.path.join(HERE, 'kv_q8_blocks.npz')
    np.savez_compressed(out, x=x, raw=raw, ok=ok)
    print(out, x.shape, int(ok.sum()), 'encoded', int((ok == 0).sum()), 'refused')


if __name__ == '__main__':
    main()
