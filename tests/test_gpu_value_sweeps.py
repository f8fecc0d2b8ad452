"""Values from the whole exponent range of fp32 / bf16 (subnormals, +-0, blocks and rows that sit entirely at one extreme, sums of
squares that overflow) through the integer-exact kernels, and every byte pattern through the quantized-embedding decoders: the
same bits as the oracle (where the oracle's value is a NaN: a NaN). Seeded."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, dev, host, ptr

pytestmark = pytest.mark.gpu
f32 = np.float32


def values(rng, shape, emin=-149.0, emax=127.9):
    """magnitudes 2 ** e with e uniform over [emin, emax], or (half of the draws) a 40-binade window placed anywhere in it"""
    e = rng.uniform(emin, emax, shape)
    if rng.random() < 0.5:
        e = np.clip(rng.uniform(-20, 20, shape) + rng.uniform(emin + 20, emax - 20), emin, emax)
    x = np.clip(np.exp2(e) * rng.choice([-1.0, 1.0], shape) * rng.uniform(1, 2, shape), -3.4e38, 3.4e38).astype(f32)
    x[rng.random(shape) < 0.05] = 0.0
    x[rng.random(shape) < 0.02] = -0.0
    return x


def same_or_nan(got, want):
    if got.dtype != f32: return bits_equal(got, want)
    nan = np.isnan(want)
    return np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan]) and bool(np.isnan(got[nan]).all())


@pytest.mark.parametrize('N,S', [(2048, 1), (1024, 3), (4096, 0)])
def test_norm_chunk_forms_on_extreme_values(N, S):
    """the same value classes through the forms that take 1024 and more rows (a wave per row, and a row divided over the waves of a
    workgroup when a q8_1 copy is asked for): every copy against the oracle, NaN for NaN"""
    rng = np.random.default_rng(4000 + N + S)
    rows = 1100
    with np.errstate(all='ignore'):
        xx = values(rng, (rows, N)); dd = values(rng, (rows, max(S, 1), N)); w = rng.standard_normal((rows, max(S, 1))).astype(f32)
        nw = (1 + 0.1 * rng.standard_normal(N)).astype(f32)
        ref = O.add_rms16(xx.copy(), nw, 1e-6, d=dd if S else None, w=w if S else None, S=S, want_q8=True)
        finite_rows = ~np.isnan(ref['h']).any(1)
        for with_q8 in (True, False):
            xd = dev(xx.copy()); h = dev(np.zeros((rows, N), f32)); h16 = dev(np.zeros((rows, N), np.uint16)); q8 = dev(np.zeros((rows, N // 32, 36), np.uint8))
            if with_q8:
                call('camx_add_rms_q8_1', ptr(xd), ptr(dev(dd)) if S else NULL, ptr(dev(w)) if S else NULL, I(S), ptr(dev(nw)), F(1e-6), ptr(h), ptr(h16), ptr(q8), I(N), I(rows))
                assert bits_equal(host(q8)[finite_rows], ref['q8'][finite_rows])
            elif N <= 2048:
                call('camx_q3p_add_rms16', ptr(xd), ptr(dev(dd)) if S else NULL, ptr(dev(w)) if S else NULL, I(S), ptr(dev(nw)), F(1e-6), ptr(h), ptr(h16), I(N), I(rows))
            else:
                continue
            assert same_or_nan(host(xd), ref['x']) and same_or_nan(host(h), ref['h'])
            assert bits_equal(host(h16, np.uint16)[finite_rows], ref['h16'][finite_rows])


@pytest.mark.parametrize('seed', range(8))
def test_quantizers_and_norms(seed):
    rng = np.random.default_rng(1000 + seed)
    with np.errstate(all='ignore'):
        n = int(rng.integers(1, 40000)); x = values(rng, n)
        y = dev(np.zeros(((n + 31) // 32) * 36, np.uint8))
        call('camx_gg_quantize_q8_1', ptr(dev(x)), ptr(y), L64(n), I(0), F(0), NULL)
        assert bits_equal(host(y), O.q8_1(x).reshape(-1))
        K = 4 * int(rng.integers(1, 600)); nc = int(rng.choice([3, 17, 300])); layout = int(rng.integers(0, 2)); x = values(rng, (nc, K))
        y = dev(np.zeros((O.k_pad(K) // 128, nc, 144), np.uint8))
        call('camx_quantize_mmq_q8_1', ptr(dev(x)), NULL, ptr(y), L64(K), L64(K), L64(0), L64(0), L64(O.k_pad(K)), I(nc), I(1), I(0), I(layout))
        assert bits_equal(host(y), O.mmq_q8_1(x, K, nc, layout))
        N = 256 * int(rng.integers(1, 9)); rows = int(rng.choice([1, 5, 300])); S = int(rng.integers(0, 4))
        xx = values(rng, (rows, N)); dd = values(rng, (rows, max(S, 1), N)); w = rng.standard_normal((rows, max(S, 1))).astype(f32)
        nw = (1 + 0.1 * rng.standard_normal(N)).astype(f32)
        ref = O.add_rms16(xx.copy(), nw, 1e-6, d=dd if S else None, w=w if S else None, S=S, want_q8=True)
        finite_rows = ~np.isnan(ref['h']).any(1)                           # (a row whose sum of squares overflows: inf * 0)
        xd = dev(xx.copy()); h = dev(np.zeros((rows, N), f32)); h16 = dev(np.zeros((rows, N), np.uint16)); q8 = dev(np.zeros((rows, N // 32, 36), np.uint8))
        call('camx_add_rms_q8_1', ptr(xd), ptr(dev(dd)) if S else NULL, ptr(dev(w)) if S else NULL, I(S), ptr(dev(nw)), F(1e-6), ptr(h), ptr(h16), ptr(q8), I(N), I(rows))
        assert same_or_nan(host(xd), ref['x']) and same_or_nan(host(h), ref['h'])
        assert bits_equal(host(h16, np.uint16)[finite_rows], ref['h16'][finite_rows]) and bits_equal(host(q8)[finite_rows], ref['q8'][finite_rows])
        db = O.f2bf(values(rng, (rows, N)))
        refb = O.add_rms_bf16(xx.copy(), db, nw, 1e-6)
        xd = dev(xx.copy()); hb = dev(np.zeros((rows, N), np.uint16))
        call('camx_add_rms_bf16', ptr(xd), ptr(dev(db)), ptr(dev(nw)), F(1e-6), ptr(h), ptr(hb), I(N), I(rows))
        ok_rows = ~np.isnan(refb['h']).any(1)
        assert same_or_nan(host(xd), refb['x']) and same_or_nan(host(h), refb['h']) and bits_equal(host(hb, np.uint16)[ok_rows], refb['hbf'][ok_rows])


@pytest.mark.parametrize('seed', range(8))
def test_kv_hadamard_actq_swiglu(seed):
    rng = np.random.default_rng(7000 + seed)
    with np.errstate(all='ignore'):
        M = 32 * int(rng.integers(1, 20)); T = int(rng.integers(1, 50))
        k = values(rng, (T, M)); v = values(rng, (T, M))
        cache0 = np.full(T * 2 * (M // 32) * 34, 0xa5, np.uint8)
        want, werr = O.kv_q8_append(k, M, v, M, M, cache0, 0, T)
        cd = dev(cache0); err = dev(np.zeros(1, np.int32))
        call('camx_own_kv_q8_append', ptr(dev(k)), I(M), ptr(dev(v)), I(M), I(M), ptr(cd), I(0), I(T), ptr(err), I(T))
        assert bits_equal(host(cd), want) and int(host(err)[0]) == werr       # blocks whose scale underflows are refused on both sides
        H = int(rng.integers(1, 3000)); x = values(rng, (H, 128), emax=115.0)
        y = dev(np.zeros((H, 128), f32))
        call('camx_hadamard128', ptr(dev(x)), ptr(y), L64(H))
        assert bits_equal(host(y), O.hadamard128(x))
        Kq = 128 * int(rng.integers(1, 40)); Mq = int(rng.integers(1, 40))
        xa = values(rng, (Mq, Kq), emin=-60.0, emax=40.0); g = O.f2bf(values(rng, (Mq, Kq), emin=-40.0, emax=20.0))
        for bf in (False, True):
            src = O.f2bf(xa) if bf else xa
            ry, rs, rc = O.actq_fwd(src, clip=0.9, qmax=7, bf16=bf)
            yq = dev(np.zeros((Mq, Kq), np.uint16)); s = dev(np.zeros(Mq, f32)); c = dev(np.zeros((Mq, Kq // 2), np.uint8))
            call('camx_actq_fwd', ptr(dev(src)), I(int(bf)), ptr(yq), ptr(s), ptr(c), I(Kq), F(0.9), I(7), I(Mq))
            assert bits_equal(host(s), rs) and bits_equal(host(yq, np.uint16), ry) and bits_equal(host(c), rc)
            dx = dev(np.zeros((Mq, Kq), np.uint16 if bf else f32))
            call('camx_actq_bwd', ptr(dev(src)), I(int(bf)), ptr(dev(g)), ptr(dx), I(Kq), F(0.9), I(7), I(Mq))
            assert bits_equal(host(dx, np.uint16) if bf else host(dx), O.actq_bwd(src, g, clip=0.9, qmax=7, bf16=bf))
        T2 = int(rng.integers(1, 60)); Fh = 8 * int(rng.integers(1, 300)); layout = int(rng.integers(0, 2))
        gu = O.f2bf(values(rng, (T2, 2 * Fh), emin=-130.0, emax=60.0))
        wa = O.silu_mul_bf16(gu)
        y = dev(np.zeros((O.k_pad(Fh) // 128, T2, 144), np.uint8)); act = dev(np.zeros((T2, Fh), np.uint16))
        call('camx_swiglu_mmq_q8_1', ptr(dev(gu)), L64(2 * Fh), L64(Fh), ptr(y), ptr(act), I(T2), I(layout))
        assert bits_equal(host(act, np.uint16), wa) and bits_equal(host(y), O.mmq_q8_1(O.bf2f(wa), Fh, T2, layout))


@pytest.mark.parametrize('T2,layout', [(40, 1), (40, 0), (300, 1), (2100, 1), (2100, 0)])
def test_swiglu_mmq_nonfinite_activations(T2, layout):
    """+-inf and NaN gate / up values (and inf * 0 products): the activation is the canonical NaN 0x7fc0 that silu_mul_bf16 stores, in every
    batch-size form of the fused kernel, and the blocks are the quantizer's of that activation (a block sum that is a NaN: a NaN)"""
    rng = np.random.default_rng(4200 + T2 + layout)
    Fh = 8 * 80
    with np.errstate(all='ignore'):
        gu = O.f2bf(values(rng, (T2, 2 * Fh), emin=-130.0, emax=60.0))
        for pat in (0x7f80, 0xff80, 0x7fc0, 0xffc1, 0x7fff, 0x7f81):
            gu[rng.random(gu.shape) < 2e-3] = pat
        wa = O.silu_mul_bf16(gu)
        want = O.mmq_q8_1(O.bf2f(wa), Fh, T2, layout)
    assert (wa == 0x7fc0).any()
    y = dev(np.zeros((O.k_pad(Fh) // 128, T2, 144), np.uint8)); act = dev(np.zeros((T2, Fh), np.uint16))
    call('camx_swiglu_mmq_q8_1', ptr(dev(gu)), L64(2 * Fh), L64(Fh), ptr(y), ptr(act), I(T2), I(layout))
    assert bits_equal(host(act, np.uint16), wa)
    got = host(y)
    if layout == 1:                                  # the half-precision sums: a NaN for a NaN, everything else bit for bit
        gs = got[:, :, :16].copy().view(np.float16)[..., 1::2]; ws = want[:, :, :16].copy().view(np.float16)[..., 1::2]
        nan = np.isnan(ws)
        assert np.isnan(gs[nan]).all() and np.array_equal(gs[~nan].view(np.uint16), ws[~nan].view(np.uint16))
        got = got.copy(); want = want.copy()
        for k in range(4): got[:, :, 4 * k + 2:4 * k + 4] = 0; want[:, :, 4 * k + 2:4 * k + 4] = 0
    assert bits_equal(got, want)
    silu = dev(np.zeros((T2, Fh), np.uint16))
    call('camx_silu_mul_bf16', ptr(dev(gu)), ptr(silu), I(Fh), L64(T2 * Fh))
    assert bits_equal(host(silu, np.uint16), wa)


@pytest.mark.parametrize('seed', range(6))
def test_embedding_blocks_of_random_bytes(seed):
    """every scale pattern (negative, subnormal, infinite, NaN) and every code byte"""
    rng = np.random.default_rng(9000 + seed)
    N = 256 * int(rng.integers(1, 20)); vocab = int(rng.integers(3, 200)); n = int(rng.integers(1, 300))
    toks = rng.integers(0, vocab, n).astype(np.int32)
    for fmt, bpb, per, orc in ((0, 144, 256, O.emb_q4k), (1, 34, 32, O.emb_q8_0), (2, 136, 256, lambda t, v, k, m: O.emb_iq4xs(t, v, k, m)[:2]), (3, 82, 256, O.emb_iq2s)):
        rb = N // per * bpb
        table = rng.integers(0, 256, (vocab, rb), dtype=np.uint8)
        with np.errstate(all='ignore'):
            ref_x, ref_bf = orc(table, vocab, toks, N)
        x = dev(np.zeros((n, N), f32)); xbf = dev(np.zeros((n, N), np.uint16))
        call('camx_emb_gather', ptr(dev(table)), L64(rb), I(vocab), ptr(dev(toks)), ptr(x), ptr(xbf), I(N), I(n), I(fmt))
        assert same_or_nan(host(x), ref_x), fmt
        gb = host(xbf, np.uint16); nanb = np.isnan(O.bf2f(ref_bf))
        assert np.array_equal(gb[~nanb], ref_bf[~nanb]) and np.isnan(O.bf2f(gb[nanb])).all(), fmt
