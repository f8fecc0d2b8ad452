"""Writes tests/golden/yarn_tables.npz: the exact fp32 bits of the reference's YaRN tables for a set of parameters.

The table (64 per-pair frequencies + the attention factor, computed in float64 and rounded to fp32) is the one input of the
rotary kernels whose last bits nothing in the reference's tests pins (they check the correction range, which pairs are
scaled and the factor's value). This script imports the reference's numpy-only module python/caminus/rope.py from a
checkout at /root/reference (or $CAMINUS_REFERENCE) and records its outputs; the product's caminus_amd.rope.yarn_table is
then held to those bits by tests/test_oracle_pins.py. Run once where the checkout exists:  python tests/golden/make_yarn_table_golden.py
"""
import os
import sys

import numpy as np

CASES = [(128, 1e6, 4.0, 32768), (128, 1e6, 2.0, 32768), (128, 1e6, 8.0, 32768), (128, 1e7, 4.0, 65536), (128, 5e5, 4.0, 8192), (128, 1e4, 16.0, 4096),
         (128, 1e6, 1.5, 40960), (128, 1e6, 4.0, 131072)]


def main():
    ref = os.environ.get('CAMINUS_REFERENCE', '/root/reference')
    sys.path.insert(0, os.path.join(ref, 'python'))
    from caminus import rope as ref_rope
    tabs = np.stack([np.asarray(ref_rope.yarn_table(*c), np.float32) for c in CASES])
    here = os.path.dirname(os.path.abspath(__file__))
    np.savez(os.path.join(here, 'yarn_tables.npz'), cases=np.array(CASES, np.float64), tables=tabs,
             corr=np.array([ref_rope.corr_dims(c[0], c[3], c[1]) for c in CASES], np.float64), mscale=np.array([ref_rope.mscale(c[2]) for c in CASES], np.float64))
    print('wrote', tabs.shape)


if __name__ == '__main__':
    main()
