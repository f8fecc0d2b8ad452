"""Embedding-row formats against the reference's own decoders' outputs (tests/golden/dequant_rows.npz, written once from the
reference's numpy-only python/caminus/own_dequant.py by tests/golden/make_dequant_golden.py): blocks with ordinary, negative,
subnormal, infinite and NaN scales. Bits must agree wherever the expected value is a number; where it is NaN, a NaN (the sign
and payload of an invalid operation's NaN are the machine's: x86 and gfx950 differ)."""
import os

import numpy as np
import pytest

import oracle as O
from oracle import np_dequant

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'dequant_rows.npz'))
FMT = {'Q4_K': 0, 'Q8_0': 1, 'IQ4_XS': 2, 'IQ2_S': 3}


def _same(got, want_bits):
    got = np.ascontiguousarray(got, np.float32).reshape(-1); want = want_bits.view(np.float32)
    nan = np.isnan(want)
    return bool(np.array_equal(np.isnan(got), nan) and np.array_equal(got.view(np.uint32)[~nan], want_bits[~nan]))


def _rows(name):
    raw = G[name + '_raw']
    return raw.reshape(-1, 272) if name == 'Q8_0' else raw          # one row of 256 values per table row


@pytest.mark.parametrize('name', list(FMT))
def test_oracle_and_numpy_decoders_against_the_reference_outputs(name):
    table = _rows(name); vocab = table.shape[0]; toks = np.arange(vocab, dtype=np.int32)
    with np.errstate(all='ignore'):
        if name == 'Q4_K': x = O.emb_q4k(table, vocab, toks, 256)[0]; y = np_dequant.q4_k(table.reshape(-1))
        elif name == 'Q8_0': x = O.emb_q8_0(table, vocab, toks, 256)[0]; y = np_dequant.q8_0(table.reshape(-1))
        elif name == 'IQ4_XS': x = O.emb_iq4xs(table, vocab, toks, 256)[0]; y = np_dequant.iq4_xs(table.reshape(-1))
        else: x = O.emb_iq2s(table, vocab, toks, 256)[0]; y = np_dequant.iq2_s(table.reshape(-1), O.iq2s_grid())
    assert _same(x, G[name + '_y']) and _same(y, G[name + '_y'])
    assert np.isnan(G[name + '_y'].view(np.float32)).any()              # the fixture does hold the hard cases


@pytest.mark.gpu
@pytest.mark.parametrize('name', list(FMT))
def test_gather_kernels_against_the_reference_outputs(name):
    from gpu_util import I, L64, call, dev, host, ptr
    table = _rows(name); vocab = table.shape[0]; toks = np.arange(vocab, dtype=np.int32)
    x = dev(np.zeros((vocab, 256), np.float32)); xbf = dev(np.zeros((vocab, 256), np.uint16))
    call('camx_emb_gather', ptr(dev(table)), L64(table.shape[1]), I(vocab), ptr(dev(toks)), ptr(x), ptr(xbf), I(256), I(vocab), I(FMT[name]))
    got = host(x)
    assert _same(got, G[name + '_y'])
    fin = ~np.isnan(got)
    assert np.array_equal(host(xbf, np.uint16)[fin], O.f2bf(got)[fin])
