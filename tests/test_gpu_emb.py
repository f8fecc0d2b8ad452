"""GPU parity of the quantized embedding gather (+ fused add + RMSNorm + q8_1) against the CPU oracle (bit-exact)."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, dev, host, outliers, ptr
from vectors import q4k_table, q80_table

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('N,vocab,n', [(2048, 1000, 256), (256, 17, 5), (5120, 64, 7)])
def test_gather_q4k_q80(N, vocab, n):
    rng = np.random.default_rng(1002 + N)
    toks = rng.integers(0, vocab, n).astype(np.int32); toks[:3] = [-5, vocab + 7, vocab - 1][:min(3, n)]     # clamped ids
    for fmt, table, orc in ((0, q4k_table(rng, vocab, N), O.emb_q4k), (1, q80_table(rng, vocab, N), O.emb_q8_0)):
        rb = table.shape[1]
        ref_x, ref_bf = orc(table, vocab, toks, N)
        Wd, td = dev(table), dev(toks)
        x = dev(np.zeros((n, N), np.float32)); xbf = dev(np.zeros((n, N), np.uint16))
        call('camx_emb_gather', ptr(Wd), L64(rb), I(vocab), ptr(td), ptr(x), ptr(xbf), I(N), I(n), I(fmt))
        assert bits_equal(host(x), ref_x) and bits_equal(host(xbf, np.uint16), ref_bf)
        if fmt == 0:
            x2 = dev(np.zeros((n, N), np.float32))
            call('camx_q3p_emb', ptr(Wd), I(rb), I(vocab), ptr(td), ptr(x2), I(N), I(n))
            assert bits_equal(host(x2), ref_x)


@pytest.mark.parametrize('fmt', [0, 1])
@pytest.mark.parametrize('with_add', [False, True])
def test_gather_add_rms_q8_1(fmt, with_add):
    """config-2 op-set: gather + dequant -> fp32 + bf16, then (add +) RMSNorm + q8_1 from the same registers"""
    rng = np.random.default_rng(1002 + fmt)
    N, vocab, n = 2048, 4096, 256
    table = (q4k_table if fmt == 0 else q80_table)(rng, vocab, N)
    toks = rng.integers(0, vocab, n).astype(np.int32)
    nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    d = outliers(rng, (n, 1, N)) * np.float32(0.01)
    gx, gbf = (O.emb_q4k if fmt == 0 else O.emb_q8_0)(table, vocab, toks, N)
    ref = O.add_rms16(gx, nw, 1e-6, d=d if with_add else None, S=1 if with_add else 0, want_q8=True)
    x = dev(np.zeros((n, N), np.float32)); xbf = dev(np.zeros((n, N), np.uint16)); h = dev(np.zeros((n, N), np.float32))
    h16 = dev(np.zeros((n, N), np.uint16)); q8 = dev(np.zeros((n, N // 32, 36), np.uint8))
    call('camx_emb_gather_add_rms', ptr(dev(table)), L64(table.shape[1]), I(vocab), ptr(dev(toks)), ptr(x), ptr(xbf),
         ptr(dev(d)) if with_add else NULL, ptr(dev(nw)), F(1e-6), ptr(h), ptr(h16), ptr(q8), I(N), I(n), I(fmt))
    assert bits_equal(host(xbf, np.uint16), gbf)
    assert bits_equal(host(x), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16, np.uint16), ref['h16'])
    assert bits_equal(host(q8), ref['q8'])
