"""Writes tests/golden/dequant_rows.npz: blocks of the embedding-row formats and the reference's own decoding of them.

The reference's host decoders (python/caminus/own_dequant.py: numpy only, declared bit-equal to gguf-py by its
tests/io/test_own_dequant.py) are imported from a checkout at /root/reference (or $CAMINUS_REFERENCE) and run on random blocks
whose fp16 scales include negative values, subnormals, infinities and NaN, the cases no per-value definition in the
reference's CPU tests covers; the IQ formats have no such definition there at all. The product's kernels and the oracle are
then held to these outputs. Run once where the checkout exists:  python tests/golden/make_dequant_golden.py
"""
import os
import sys

import numpy as np

FORMATS = {'Q4_K': (256, 144, (0, 2)), 'Q8_0': (32, 34, (0,)), 'IQ4_XS': (256, 136, (0,)), 'IQ2_S': (256, 82, (0,))}


def blocks(rng, n, bs, dpos):
    raw = rng.integers(0, 256, (n, bs), dtype=np.uint8)
    d = (rng.standard_normal((n, len(dpos))) * 0.01).astype(np.float16)
    special = np.array([0.0, -0.0, 6e-8, -6e-8, 6.1e-5, 65504, -65504, np.inf, -np.inf, np.nan], np.float16)
    d[:special.size, 0] = special                                # the first scale of the first blocks: the special values
    if len(dpos) > 1: d[special.size:2 * special.size, 1] = special
    for k, o in enumerate(dpos):
        raw[:, o:o + 2] = d[:, k:k + 1].view(np.uint8).reshape(n, 2)
    return raw


def main():
    ref = os.environ.get('CAMINUS_REFERENCE', '/root/reference')
    sys.path.insert(0, os.path.join(ref, 'python'))
    from caminus import own_dequant
    rng = np.random.default_rng(20261125)
    out = {}
    for name, (qk, bs, dpos) in FORMATS.items():
        raw = blocks(rng, 48, bs, dpos)
        with np.errstate(all='ignore'):
            y = own_dequant.dequant(raw.reshape(-1), name, 48 * qk)
        out[name + '_raw'] = raw
        out[name + '_y'] = np.asarray(y, np.float32).view(np.uint32)            # bits: NaN payloads survive the file
    here = os.path.dirname(os.path.abspath(__file__))
    np.savez_compressed(os.path.join(here, 'dequant_rows.npz'), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == '__main__':
    main()
