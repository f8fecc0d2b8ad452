"""The committed golden file tests/golden/kv_q8_blocks.npz holds Q8 KV blocks encoded by the reference's own encoder
(kernels/own_kv_codec.h compiled for the host; see tests/golden/make_kv_q8_golden.py). The CPU oracle and the device
kernel must both reproduce its bytes and its refusals, with nothing from the reference checkout present at run time."""
import os

import numpy as np
import pytest

import oracle as O

GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'kv_q8_blocks.npz'))


def test_oracle_reproduces_the_reference_encoder_bytes():
    x, raw, ok = GOLDEN['x'], GOLDEN['raw'], GOLDEN['ok']
    assert x.shape == (1044, 32) and ok.sum() == 1037
    got, gok = O.kv_q8_encode(x)
    assert np.array_equal(gok, ok) and np.array_equal(got, raw)


@pytest.mark.gpu
def test_device_append_reproduces_the_reference_encoder_bytes():
    from gpu_util import I, call, dev, host, ptr
    x, raw, ok = GOLDEN['x'], GOLDEN['raw'], GOLDEN['ok']
    # one block per K part and the same block per V part: rows of M = 32 values, cache rows [K block | V block]
    n = len(x)
    cache = dev(np.full(n * 68, 0xa5, np.uint8)); err = dev(np.zeros(1, np.int32)); xd = dev(x)
    call('camx_own_kv_q8_append', ptr(xd), I(32), ptr(xd), I(32), I(32), ptr(cache), I(0), I(n), ptr(err), I(n))
    got = host(cache).reshape(n, 2, 34)
    assert np.array_equal(got[:, 0], raw) and np.array_equal(got[:, 1], raw)
    assert int(host(err)[0]) == 2                                        # the refused blocks raised the numerical bit
    assert (got[ok == 0] == 0xa5).all()
