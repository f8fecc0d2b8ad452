"""GPU parity of the residual add + RMSNorm family against the CPU oracle (bit-exact under the contract tree)."""
import numpy as np
import pytest

import oracle as O
import ctypes as C

from gpu_util import F, I, NULL, bits_equal, call, camx, dev, host, outliers, ptr, stream

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('n,N,S,weighted', [(1, 2048, 1, False), (5, 2048, 8, True), (3, 256, 0, False), (7, 1024, 3, True), (256, 2048, 1, False),
                                                (1027, 2048, 2, True), (1024, 1024, 1, False), (1030, 2048, 8, False), (16385, 2048, 1, False), (16384, 1024, 3, True)])
def test_q3p_add_rms16(n, N, S, weighted):
    rng = np.random.default_rng(1001 + n + N + S)
    x = outliers(rng, (n, N)); d = outliers(rng, (n, max(S, 1), N)); w = rng.random((n, max(S, 1))).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    ref = O.add_rms16(x, nw, 1e-6, d=d if S else None, w=w if weighted else None, S=S)
    xd, dd, wd, nwd = dev(x), dev(d), dev(w), dev(nw)
    h = dev(np.zeros((n, N), np.float32)); h16 = dev(np.zeros((n, N), np.uint16))
    call('camx_q3p_add_rms16', ptr(xd), ptr(dd) if S else NULL, ptr(wd) if weighted else NULL, I(S), ptr(nwd), F(1e-6), ptr(h), ptr(h16), I(N), I(n))
    assert bits_equal(host(xd), ref['x'])
    assert bits_equal(host(h), ref['h'])
    assert bits_equal(host(h16, np.uint16), ref['h16'])
    # without the fp32 copy (the layers whose consumer reads fp16 only)
    xd = dev(x); h16 = dev(np.zeros((n, N), np.uint16))
    call('camx_q3p_add_rms16', ptr(xd), ptr(dd) if S else NULL, ptr(wd) if weighted else NULL, I(S), ptr(nwd), F(1e-6), NULL, ptr(h16), I(N), I(n))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(h16, np.uint16), ref['h16'])
    # the tape's form: the fp16 copy at its own token stride (the Seg's K), the elements between the rows untouched
    K = N + 64
    xd = dev(x); h = dev(np.zeros((n, N), np.float32)); h16 = dev(np.full((n, K), 0x5a5a, np.uint16))
    call('camx_op_own_add_rms16', ptr(xd), ptr(dd) if S else NULL, ptr(wd) if weighted else NULL, I(S), ptr(nwd), F(1e-6), ptr(h), ptr(h16), I(N), I(K), I(n))
    got = host(h16, np.uint16)
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(got[:, :N], ref['h16']) and (got[:, N:] == 0x5a5a).all()


@pytest.mark.parametrize('n,N', [(2, 5120), (3, 2560), (1, 8192), (2, 16384), (4, 4096), (520, 4096), (513, 8192), (600, 3072), (1030, 2560), (1025, 5120), (1024, 4096), (16385, 1024), (16384, 5120)])
def test_q35p_add_rms16(n, N):
    rng = np.random.default_rng(7 + N)
    x = outliers(rng, (n, N)); d = outliers(rng, (n, N)); nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    for dd_ in (d, None):
        ref = O.add_rms16_q35(x, nw, 1e-6, d=dd_)
        xd = dev(x); h = dev(np.zeros((n, N), np.float32)); h16 = dev(np.zeros((n, N), np.uint16)); nwd = dev(nw)
        ddv = dev(dd_) if dd_ is not None else None
        call('camx_q35p_add_rms16', ptr(xd), ptr(ddv), ptr(nwd), F(1e-6), ptr(h), ptr(h16), I(N), I(n))
        assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16, np.uint16), ref['h16'])
        # the tape's form of the same op (OP_OWN_ADD_RMS16 on the dense line: rows longer than 2048, one addend or none), h16 at its own stride
        K = N + 64
        for sym in ('camx_op_q35_add_rms16',) + (('camx_op_own_add_rms16',) if N > 2048 else ()):
            xd = dev(x); h = dev(np.zeros((n, N), np.float32)); h16 = dev(np.full((n, K), 0x5a5a, np.uint16))
            extra = (NULL,) if sym == 'camx_op_own_add_rms16' else ()
            call(sym, ptr(xd), ptr(ddv), *extra, I(1 if dd_ is not None else 0), ptr(nwd), F(1e-6), ptr(h), ptr(h16), I(N), I(K), I(n))
            got = host(h16, np.uint16)
            assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(got[:, :N], ref['h16']) and (got[:, N:] == 0x5a5a).all(), sym
    if N > 2048:                                                      # what the long-row form does not take: weights, more than one addend, no fp32 copy
        L = camx(); p = lambda t: C.c_void_p(t.data_ptr()); ddv = dev(d)
        assert L.camx_op_own_add_rms16(p(xd), p(ddv), p(nwd), I(1), p(nwd), F(1e-6), p(h), p(h16), I(N), I(K), I(1), stream()) == 1
        assert L.camx_op_own_add_rms16(p(xd), p(ddv), NULL, I(2), p(nwd), F(1e-6), p(h), p(h16), I(N), I(K), I(1), stream()) == 1
        assert L.camx_op_own_add_rms16(p(xd), p(ddv), NULL, I(1), p(nwd), F(1e-6), NULL, p(h16), I(N), I(K), I(1), stream()) == 1


@pytest.mark.parametrize('n,N', [(4, 2048), (256, 2048), (2, 5120), (1026, 2048), (1024, 4096)])
def test_add_rms_q8_1(n, N):
    rng = np.random.default_rng(1002 + N)
    x = outliers(rng, (n, N)); d = outliers(rng, (n, 1, N)); nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    ref = O.add_rms16(x, nw, 1e-6, d=d, S=1, want_q8=True)
    xd, dd, nwd = dev(x), dev(d), dev(nw)
    h = dev(np.zeros((n, N), np.float32)); q8 = dev(np.zeros((n, N // 32, 36), np.uint8))
    call('camx_add_rms_q8_1', ptr(xd), ptr(dd), NULL, I(1), ptr(nwd), F(1e-6), ptr(h), NULL, ptr(q8), I(N), I(n))
    assert bits_equal(host(h), ref['h'])
    assert bits_equal(host(q8), ref['q8'])
    # the q8_1 copy alone, and with both float copies
    xd = dev(x); q8 = dev(np.zeros((n, N // 32, 36), np.uint8))
    call('camx_add_rms_q8_1', ptr(xd), ptr(dd), NULL, I(1), ptr(nwd), F(1e-6), NULL, NULL, ptr(q8), I(N), I(n))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(q8), ref['q8'])
    xd = dev(x); q8 = dev(np.zeros((n, N // 32, 36), np.uint8)); h = dev(np.zeros((n, N), np.float32)); h16 = dev(np.zeros((n, N), np.uint16))
    call('camx_add_rms_q8_1', ptr(xd), ptr(dd), NULL, I(1), ptr(nwd), F(1e-6), ptr(h), ptr(h16), ptr(q8), I(N), I(n))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(q8), ref['q8']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16, np.uint16), ref['h16'])


@pytest.mark.parametrize('n,N', [(3, 5120), (64, 5120), (2, 2048), (600, 5120), (515, 6144), (512, 7168)])
def test_add_rms_bf16(n, N):
    rng = np.random.default_rng(1003 + N)
    x = outliers(rng, (n, N)); d = O.f2bf(outliers(rng, (n, N))); nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    ref = O.add_rms_bf16(x, d, nw, 1e-6)
    xd, dd, nwd = dev(x), dev(d), dev(nw)
    h = dev(np.zeros((n, N), np.float32)); hbf = dev(np.zeros((n, N), np.uint16))
    call('camx_add_rms_bf16', ptr(xd), ptr(dd), ptr(nwd), F(1e-6), ptr(h), ptr(hbf), I(N), I(n))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(hbf, np.uint16), ref['hbf'])


@pytest.mark.parametrize('R,K,wr', [(8, 2560, 4), (3, 2048, 1), (5, 100, 1), (2, 896, 2), (516, 3072, 4), (512, 5120, 1), (1028, 2560, 4), (1029, 2560, 1), (1026, 2048, 1), (1024, 5120, 4), (16388, 2048, 4)])
def test_rms_mul_and_rmsnorm(R, K, wr):
    rng = np.random.default_rng(R * K)
    x = outliers(rng, (R, K)); w = (1 + 0.1 * rng.standard_normal((wr, K))).astype(np.float32)
    if R % wr: R = R // wr * wr; x = x[:R]
    ref = O.rms_mul(x, w, 1e-6, want_q8=K % 32 == 0)
    xd, wd = dev(x), dev(w)
    y = dev(np.zeros((R, K), np.float32)); ybf = dev(np.zeros((R, K), np.uint16)); scl = dev(np.zeros(R, np.float32))
    call('camx_pf_rms_mul', ptr(xd), ptr(wd), ptr(y), ptr(ybf), ptr(scl), I(R), I(wr), F(1e-6), I(K))
    assert bits_equal(host(y), ref['y']) and bits_equal(host(ybf, np.uint16), ref['ybf']) and bits_equal(host(scl), ref['scale'])
    # each copy set the prefill callers ask for on its own (python/caminus/prefill/glue.py:153: absent copies are null)
    ybf = dev(np.zeros((R, K), np.uint16)); scl = dev(np.zeros(R, np.float32)); y = dev(np.zeros((R, K), np.float32))
    call('camx_pf_rms_mul', ptr(xd), ptr(wd), NULL, ptr(ybf), ptr(scl), I(R), I(wr), F(1e-6), I(K))
    call('camx_pf_rms_mul', ptr(xd), ptr(wd), ptr(y), NULL, NULL, I(R), I(wr), F(1e-6), I(K))
    assert bits_equal(host(y), ref['y']) and bits_equal(host(ybf, np.uint16), ref['ybf']) and bits_equal(host(scl), ref['scale'])
    xnan = x.copy(); xnan[R // 2, 3] = np.nan; xnd = dev(xnan); ybf = dev(np.zeros((R, K), np.uint16))
    call('camx_pf_rms_mul', ptr(xnd), ptr(wd), NULL, ptr(ybf), NULL, I(R), I(wr), F(1e-6), I(K))
    assert bits_equal(host(ybf, np.uint16), O.rms_mul(xnan, w, 1e-6)['ybf'])         # a NaN row takes the reference's integer rounding
    if K % 32 == 0:
        q8 = dev(np.zeros((R, K // 32, 36), np.uint8)); y2 = dev(np.zeros((R, K), np.float32))
        call('camx_op_rms_mul', ptr(xd), ptr(wd), ptr(y2), ptr(q8), I(R), I(wr), I(K), F(1e-6))
        assert bits_equal(host(y2), ref['y']) and bits_equal(host(q8), ref['q8'])
    if wr == 1:
        out = dev(np.zeros((R, K), np.float32))
        call('camx_rmsnorm_f32', ptr(xd), ptr(wd), ptr(out), I(K), F(1e-6), I(R))
        assert bits_equal(host(out), O.rmsnorm_f32(x, w[0], 1e-6))


@pytest.mark.parametrize('T,HC,N', [(5, 4, 2560), (2048, 4, 2560), (3, 2, 2048), (7, 3, 100), (130, 4, 5120), (601, 2, 2048), (1100, 1, 2560)])
def test_hc_glue(T, HC, N):
    """hyper-connection glue: the residual update passes expf (tolerance class: 1e-5 x max), everything behind it is exact given
    the updated residual; inj = 0 makes the gate exactly 1, so those rows are compared bit for bit"""
    from gpu_util import close_16, close_fp32
    rng = np.random.default_rng(T + N)
    b = outliers(rng, (T, N)); inj = rng.standard_normal((T, HC)).astype(np.float32); inj[0] = 0.0
    res = outliers(rng, (T, HC, N)); w = (1 + 0.1 * rng.standard_normal((HC, N))).astype(np.float32)
    ref = O.hc_post_rms(b, inj, res, w, 1e-6)
    rd = dev(res); xn = dev(np.zeros((T, HC, N), np.float32)); xnbf = dev(np.zeros((T, HC, N), np.uint16)); scl = dev(np.zeros(T * HC, np.float32))
    bd, injd, wd = dev(b), dev(inj), dev(w)
    call('camx_pf_hc_post_rms', ptr(bd), ptr(injd), ptr(rd), ptr(wd), ptr(xn), ptr(xnbf), ptr(scl), I(T), I(HC), F(0.25), F(1e-6), I(N))
    gres, gxn = host(rd), host(xn)
    assert close_fp32(gres, ref['res']) and close_fp32(gxn, ref['xn']) and close_16(host(xnbf, np.uint16), ref['xnbf'], 'bf16')
    assert bits_equal(gres[0], ref['res'][0]) and bits_equal(gxn[0], ref['xn'][0]) and bits_equal(host(scl)[:HC], ref['scale'][:HC])
    # exact given the device's own residual: the norm of it by the oracle's rms_mul
    again = O.rms_mul(gres.reshape(T * HC, N), w, 1e-6)
    assert bits_equal(gxn.reshape(T * HC, N), again['y']) and bits_equal(host(scl), again['scale']) and bits_equal(host(xnbf, np.uint16).reshape(T * HC, N), again['ybf'])
    # the prefill caller's copy set (bf16 + row scale, no fp32 copy): the same bits
    r3 = dev(res); xnbf3 = dev(np.zeros((T, HC, N), np.uint16)); scl3 = dev(np.zeros(T * HC, np.float32))
    call('camx_pf_hc_post_rms', ptr(bd), ptr(injd), ptr(r3), ptr(wd), NULL, ptr(xnbf3), ptr(scl3), I(T), I(HC), F(0.25), F(1e-6), I(N))
    assert bits_equal(host(r3), gres) and bits_equal(host(xnbf3, np.uint16), host(xnbf, np.uint16)) and bits_equal(host(scl3), host(scl))
    r2 = dev(res)
    call('camx_pf_hc_post', ptr(bd), ptr(injd), ptr(r2), I(T), I(HC), I(N), F(0.25))
    assert bits_equal(host(r2), gres)                                      # the same statements: the same bits as the fused kernel
    g = outliers(rng, (T, HC, N))
    out = dev(np.zeros((T, N), np.float32)); out2 = dev(np.zeros((T, N), np.float32))
    call('camx_pf_hc_mean', ptr(xn), NULL, NULL, ptr(dev(g)), ptr(out), I(T), I(HC), I(N), F(0.25))
    call('camx_pf_hc_mean', ptr(rd), ptr(scl), ptr(wd), ptr(dev(g)), ptr(out2), I(T), I(HC), I(N), F(0.25))
    assert close_fp32(host(out), O.hc_mean(gxn, g)) and bits_equal(host(out2), host(out))
