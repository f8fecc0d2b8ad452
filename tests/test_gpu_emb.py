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
@pytest.mark.parametrize('N,n', [(2048, 256), (1024, 37), (4096, 130), (5120, 19), (2560, 40), (2048, 300)])
def test_gather_add_rms_q8_1(fmt, with_add, N, n):
    """config-2 op-set: gather + dequant -> fp32 + bf16, then (add +) RMSNorm + q8_1 from the same registers; every row width of the
    workgroup-per-row form (up to 256 rows) and one batch beyond it"""
    rng = np.random.default_rng(1002 + fmt + N)
    vocab = 4096 if N == 2048 else 300
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


# ---- IQ4_XS / IQ2_S token rows, IQ4_NL feed rows ------------------------------------------------------------------------------

@pytest.mark.parametrize('N,vocab,n', [(2048, 500, 256), (256, 9, 5), (5120, 40, 7), (8192, 12, 33), (1536, 30, 64)])
def test_gather_iq4xs_iq2s(N, vocab, n):
    from vectors import iq_table
    rng = np.random.default_rng(2002 + N)
    toks = rng.integers(0, vocab, n).astype(np.int32); toks[:3] = [-5, vocab + 7, vocab - 1][:min(3, n)]
    for fmt, name in ((2, 'IQ4_XS'), (3, 'IQ2_S')):
        table = iq_table(rng, vocab, N, name)
        if fmt == 2: ref_x, ref_bf, _ = O.emb_iq4xs(table, vocab, toks, N)
        else: ref_x, ref_bf = O.emb_iq2s(table, vocab, toks, N)
        Wd, td = dev(table), dev(toks)
        x = dev(np.zeros((n, N), np.float32)); xbf = dev(np.zeros((n, N), np.uint16))
        call('camx_emb_gather', ptr(Wd), L64(table.shape[1]), I(vocab), ptr(td), ptr(x), ptr(xbf), I(N), I(n), I(fmt))
        assert bits_equal(host(x), ref_x) and bits_equal(host(xbf, np.uint16), ref_bf)
        if fmt == 2:                                                    # the reference's own entry point, with its error word
            x2 = dev(np.zeros((n, N), np.float32)); err = dev(np.zeros(1, np.int32))
            call('camx_embd_rows_iq4xs', ptr(Wd), ptr(td), I(vocab), I(n), I(N // 256), ptr(x2), ptr(err))
            assert bits_equal(host(x2), ref_x) and int(host(err)[0]) == 2
            good = dev(np.clip(toks, 0, vocab - 1)); err.zero_()
            call('camx_embd_rows_iq4xs', ptr(Wd), ptr(good), I(vocab), I(n), I(N // 256), ptr(x2), ptr(err))
            assert bits_equal(host(x2), ref_x) and int(host(err)[0]) == 0


@pytest.mark.parametrize('fmt', [2, 3])
def test_gather_add_rms_q8_1_iq(fmt):
    from vectors import iq_table
    rng = np.random.default_rng(2100 + fmt)
    N, vocab, n = 2048, 300, 64
    table = iq_table(rng, vocab, N, 'IQ4_XS' if fmt == 2 else 'IQ2_S')
    toks = rng.integers(0, vocab, n).astype(np.int32)
    nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    d = outliers(rng, (n, 1, N)) * np.float32(0.01)
    gx, gbf = O.emb_iq4xs(table, vocab, toks, N)[:2] if fmt == 2 else O.emb_iq2s(table, vocab, toks, N)
    ref = O.add_rms16(gx, nw, 1e-6, d=d, S=1, want_q8=True)
    x = dev(np.zeros((n, N), np.float32)); xbf = dev(np.zeros((n, N), np.uint16)); h = dev(np.zeros((n, N), np.float32))
    h16 = dev(np.zeros((n, N), np.uint16)); q8 = dev(np.zeros((n, N // 32, 36), np.uint8))
    call('camx_emb_gather_add_rms', ptr(dev(table)), L64(table.shape[1]), I(vocab), ptr(dev(toks)), ptr(x), ptr(xbf), ptr(dev(d)), ptr(dev(nw)),
         F(1e-6), ptr(h), ptr(h16), ptr(q8), I(N), I(n), I(fmt))
    assert bits_equal(host(xbf, np.uint16), gbf) and bits_equal(host(x), ref['x']) and bits_equal(host(h), ref['h'])
    assert bits_equal(host(h16, np.uint16), ref['h16']) and bits_equal(host(q8), ref['q8'])


@pytest.mark.parametrize('nuniq,nrows,bpr', [(40, 2048 * 2, 5), (3, 7, 1), (64, 300, 8)])
def test_ple_rows_iq4nl(nuniq, nrows, bpr):
    """the feed's IQ4_NL rows through the reference's launcher surface, with its negative controls (tests/prefill/test_prefill_feed.py:189-199)"""
    import ctypes
    import torch
    from caminus_amd.device.hip import Module
    from vectors import iq_table
    rng = np.random.default_rng(2200 + bpr)
    raw = iq_table(rng, nuniq, 32 * bpr, 'IQ4_NL'); inv = rng.integers(0, nuniq, nrows).astype(np.int32)
    want, e0 = O.ple_rows_iq4nl(raw, inv, nuniq, bpr)
    out = dev(np.zeros((nrows, 32 * bpr), np.float32)); err = dev(np.zeros(1, np.int32))
    mod = Module('prefill_feed')
    N = nrows * 32 * bpr
    rawd, invd = dev(raw), dev(inv)
    mod.ple_rows_iq4nl(((N + 255) // 256,), (256,), rawd, invd, ctypes.c_int(nuniq), ctypes.c_int(nrows), ctypes.c_int(bpr), out, err)
    torch.cuda.synchronize()
    assert e0 == 0 and int(host(err)[0]) == 0 and bits_equal(host(out), want)
    bad = inv.copy(); bad[min(3, nrows - 1)] = nuniq; bad[min(5, nrows - 1)] = -7
    want, e1 = O.ple_rows_iq4nl(raw, bad, nuniq, bpr)
    badd = dev(bad)
    mod.ple_rows_iq4nl(((N + 255) // 256,), (256,), rawd, badd, ctypes.c_int(nuniq), ctypes.c_int(nrows), ctypes.c_int(bpr), out, err)
    torch.cuda.synchronize()
    assert e1 == 1 and int(host(err)[0]) == 1 and bits_equal(host(out), want)
    with pytest.raises(ValueError):
        mod.ple_rows_iq4nl((1,), (256,), rawd, invd, ctypes.c_int(nuniq), ctypes.c_int(nrows + 300), ctypes.c_int(bpr), out, err)


def test_op_own_emb_tape_fields():
    """OP_OWN_EMB with the Seg's fields: the same rows as the prefill entry points; the drafter's key form (the token is the complement
    of the low half of a 64-bit argmax key); a format the op does not have is refused"""
    rng = np.random.default_rng(77)
    N, vocab, n = 2048, 500, 9
    table = q4k_table(rng, vocab, N); rb = table.shape[1]
    toks = rng.integers(0, vocab, n).astype(np.int32); toks[:2] = [-3, vocab + 1]
    ref_x, _ = O.emb_q4k(table, vocab, toks, N)
    Wd = dev(table); x = dev(np.zeros((n, N), np.float32))
    call('camx_op_own_emb', ptr(Wd), ptr(dev(toks)), ptr(x), I(N), I(rb), I(4), I(0), I(vocab), I(n))
    assert bits_equal(host(x), ref_x)
    tok = 123
    key = np.array([(0x3f80_0000 << 32) | (~tok & 0xffffffff)], np.uint64)
    x1 = dev(np.zeros((1, N), np.float32))
    call('camx_op_own_emb', ptr(Wd), ptr(dev(key.view(np.int64))), ptr(x1), I(N), I(rb), I(4), I(1), I(vocab), I(1))
    assert bits_equal(host(x1), O.emb_q4k(table, vocab, np.array([tok], np.int32), N)[0])
    import ctypes as C
    from gpu_util import camx
    dp = lambda t: C.c_void_p(t.data_ptr())
    td, kd = dev(toks), dev(key.view(np.int64))
    assert camx().camx_op_own_emb(dp(Wd), dp(td), dp(x), I(N), I(rb), I(9), I(0), I(vocab), I(n), NULL) == 1            # a format the op does not have
    assert camx().camx_op_own_emb(dp(Wd), dp(kd), dp(x), I(N), I(rb), I(4), I(1), I(vocab), I(2), NULL) == 1            # the key form is one token
    t80 = q80_table(rng, vocab, N)
    x2 = dev(np.zeros((n, N), np.float32))
    call('camx_op_own_emb', ptr(dev(t80)), ptr(dev(toks)), ptr(x2), I(N), I(t80.shape[1]), I(3), I(0), I(vocab), I(n))
    assert bits_equal(host(x2), O.emb_q8_0(t80, vocab, toks, N)[0])
