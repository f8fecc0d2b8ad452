"""GPU parity of the activation fake-quant forward kernels against the CPU oracle: codes, scales and bf16 values bit-exact
for the plain and RMSNorm sources; the SiLU source carries expf and is compared through its own activation bits."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, close_16, dev, host, outliers, ptr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('M,K,qmax', [(5, 896, 7), (3, 2048, 7), (2, 8192, 7), (4, 128, 3), (3, 768, 127), (9, 1152, 7), (6, 1920, 7), (301, 1024, 7),
                                      (5, 2176, 7)])
def test_actq_fwd(M, K, qmax):
    """rows of at most 2048 values take the wave-per-row kernel when the outputs are 16-byte (values) and 4-byte (codes) aligned,
    the workgroup-per-row kernel otherwise: both against the oracle"""
    import ctypes
    rng = np.random.default_rng(K + qmax)
    x = outliers(rng, (M, K)); x[0] = 0
    for bf in (False, True):
        src = O.f2bf(x) if bf else x
        ry, rs, rc = O.actq_fwd(src, clip=0.9, qmax=qmax, bf16=bf)
        srcd = dev(src)
        for shift in (0, 1):                                            # shift: outputs moved off their 16- / 4-byte alignment
            y = dev(np.zeros(M * K + 8, np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros(M * K // 2 + 8, np.uint8))
            yp = ctypes.c_void_p(y.data_ptr() + 8 * shift); cp = ctypes.c_void_p(c.data_ptr() + 2 * shift)
            call('camx_actq_fwd', ptr(srcd), I(int(bf)), yp, ptr(s), cp if qmax <= 7 else NULL, I(K), F(0.9), I(qmax), I(M))
            assert bits_equal(host(s), rs) and bits_equal(host(y, np.uint16)[4 * shift:4 * shift + M * K].reshape(M, K), ry)
            if qmax <= 7: assert bits_equal(host(c)[2 * shift:2 * shift + M * K // 2].reshape(M, K // 2), rc)


@pytest.mark.parametrize('M,d,nab', [(6, 896, 8), (5, 1024, 16), (3, 2048, 5), (2, 4096, 2), (130, 1024, 14), (4, 128, 1), (3, 8192, 3), (7, 768, 0),
                                     (9, 512, 6), (5, 256, 16), (300, 640, 3), (4, 1152, 9)])
def test_block_entry_fwd(M, d, nab):
    """rows of at most 1024 values: one wave per row, every round count; longer rows: a workgroup per row. The projections run one
    per wave (rows w, w + W, ... of wab): counts that are not multiples of four, rows that keep bf16(h) in registers and longer ones"""
    rng = np.random.default_rng(11 + d + nab)
    x = outliers(rng, (M, d)); nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32); wab = O.f2bf(rng.standard_normal((nab, d)) * 0.05)
    ry, rs, rc, rab, rstd = O.block_entry_fwd(x, nw, wab if nab else None, 1e-6)
    y = dev(np.zeros((M, d), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, d // 2), np.uint8))
    ab = dev(np.zeros((M, max(nab, 1)), np.uint16)); rstd_d = dev(np.zeros(M, np.float32))
    call('camx_block_entry_fwd', ptr(dev(x)), ptr(dev(nw)), ptr(dev(wab)) if nab else NULL, I(nab), F(1e-6), ptr(y), ptr(s), ptr(c),
         ptr(ab) if nab else NULL, ptr(rstd_d), I(d), F(1.0), I(7), I(M))
    assert bits_equal(host(rstd_d), rstd) and bits_equal(host(s), rs) and bits_equal(host(c), rc) and bits_equal(host(y, np.uint16), ry)
    if nab: assert bits_equal(host(ab, np.uint16), rab)


@pytest.mark.parametrize('M,Fh', [(5, 768), (2100, 1024), (2050, 1920), (2049, 2176), (4099, 128), (5, 2304), (303, 2048)])
def test_silu_mul_actq_fwd(M, Fh):
    rng = np.random.default_rng(12 + M)
    gu = O.f2bf(outliers(rng, (M, 2 * Fh)))
    gu[M - 1, :10] = O.f2bf(np.array([256., -256., 255., -255., 2.0 ** -24, -2.0 ** -24, 2.0 ** -25, -2.0 ** -25, 1e4, -1e-30], np.float32))      # the edges of the small table
    y = dev(np.zeros((M, Fh), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, Fh // 2), np.uint8))
    gud = dev(gu)
    call('camx_silu_mul_actq_fwd', ptr(gud), I(2 * Fh), I(Fh), ptr(y), ptr(s), ptr(c), F(1.0), I(7), I(M))
    # the activation is the table's (the oracle's bits), then the exact stages on it
    act = dev(np.zeros((M, Fh), np.uint16))
    call('camx_silu_mul_bf16', ptr(gud), ptr(act), I(Fh), L64(M * Fh))
    assert bits_equal(host(act, np.uint16), O.silu_mul_bf16(gu))
    ry, rs, rc = O.actq_fwd(host(act, np.uint16), bf16=True)
    assert bits_equal(host(s), rs) and bits_equal(host(c), rc) and bits_equal(host(y, np.uint16), ry)
    fy, fs, fc = O.silu_mul_actq_fwd(gu)
    assert bits_equal(host(s), fs) and bits_equal(host(c), fc) and bits_equal(host(y, np.uint16), fy)


# ---- backward ----------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize('M,K,qmax', [(5, 896, 7), (3, 2048, 7), (2, 8192, 7), (4, 128, 3), (3, 768, 127), (300, 1024, 7), (7, 5120, 7), (9, 1152, 7), (6, 1920, 7),
                                      (5, 1536, 15)])
def test_actq_bwd(M, K, qmax):
    rng = np.random.default_rng(100 + K + qmax)
    x = outliers(rng, (M, K)); x[0] = 0
    if M > 2: x[2, :] = 0; x[2, 7] = 3.0                                   # rotates to a constant row: every element ties for the max
    g = O.f2bf(rng.standard_normal((M, K)).astype(np.float32))
    for bf in (False, True):
        src = O.f2bf(x) if bf else x
        want = O.actq_bwd(src, g, clip=0.9, qmax=qmax, bf16=bf)
        dx = dev(np.zeros((M, K), np.uint16 if bf else np.float32))
        call('camx_actq_bwd', ptr(dev(src)), I(int(bf)), ptr(dev(g)), ptr(dx), I(K), F(0.9), I(qmax), I(M))
        assert bits_equal(host(dx, np.uint16) if bf else host(dx), want)


@pytest.mark.parametrize('K', [1024, 2048, 2560])
def test_actq_bwd_quotients_at_the_exponent_limits(K):
    """u / s where the quotient, the scale or their ratio leaves the range in which the kernel divides by a refined reciprocal:
    rows scaled to 1e-30 and 1e30, a row of 1e-12 with one chunk at 1e20 (quotients near 1e-32), a row whose values span
    1e-38 .. 1e38, inf and NaN entries, and a clip of 1e-20 (quotients near 1e21): the IEEE quotient in every case"""
    rng = np.random.default_rng(500 + K)
    M = 8
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[0] *= 1e-30; x[1] *= 1e30
    x[2] *= 1e-12; x[2, 128:256] *= 1e32
    x[3] *= (10.0 ** rng.uniform(-38, 38, K)).astype(np.float32)
    x[4, 5] = np.inf; x[5, 130] = np.nan
    x[6] *= 1e-12; x[6, :128] = 0; x[6, 300] = 1e25
    x[7] = 0; x[7, 128:256] = 1e-30 * rng.standard_normal(128)
    g = O.f2bf(rng.standard_normal((M, K)).astype(np.float32))
    for bf in (False, True):
        src = O.f2bf(x) if bf else x
        for clip in (1.0, 1e-20):
            want = O.actq_bwd(src, g, clip=clip, qmax=7, bf16=bf)
            dx = dev(np.zeros((M, K), np.uint16 if bf else np.float32))
            call('camx_actq_bwd', ptr(dev(src)), I(int(bf)), ptr(dev(g)), ptr(dx), I(K), F(clip), I(7), I(M))
            got = host(dx, np.uint16) if bf else host(dx)
            nan_w = np.isnan(O.bf2f(want)) if bf else np.isnan(want); nan_g = np.isnan(O.bf2f(got)) if bf else np.isnan(got)
            assert np.array_equal(nan_w, nan_g) and bits_equal(np.where(nan_w, 0, got), np.where(nan_w, 0, want))


@pytest.mark.parametrize('M,d,nab', [(6, 896, 14), (5, 1024, 0), (9, 256, 2), (130, 896, 16), (7, 1024, 16), (3, 128, 4), (171, 896, 8), (12, 640, 6), (9, 384, 0)])
def test_block_entry_bwd(M, d, nab):
    """every round count of the wave-per-row kernel; row 1 has one value in the row's last chunk and one in chunk 1 with the same
    |h|: their chunks rotate to constants, so 256 elements tie for the row's maximum across rounds that not all lanes take part in"""
    rng = np.random.default_rng(200 + d + nab)
    x = outliers(rng, (M, d)); nw = (0.5 + rng.random(d)).astype(np.float32)
    if d >= 384 and M > 1:
        last = d - 128 + 5
        nw[last] = nw[128 + 7]; x[1] = 0; x[1, 128 + 7] = 3.0; x[1, last] = -3.0
    wab = O.f2bf((rng.standard_normal((max(nab, 2), d)) / 30).astype(np.float32))[:nab]
    dy = O.f2bf(rng.standard_normal((M, d)).astype(np.float32)); dab = O.f2bf(rng.standard_normal((M, max(nab, 1))).astype(np.float32))[:, :nab]
    rstd = O.block_entry_fwd(x, nw, wab if nab else None, 1e-6)[4]
    want = O.block_entry_bwd(x, nw, rstd, wab if nab else None, dy, dab if nab else None)
    dx = dev(np.zeros((M, d), np.float32))
    call('camx_block_entry_bwd', ptr(dev(x)), ptr(dev(nw)), ptr(dev(rstd)), ptr(dev(wab)) if nab else NULL, I(nab), ptr(dev(dy)),
         ptr(dev(np.ascontiguousarray(dab))) if nab else NULL, ptr(dx), I(d), F(1.0), I(7), I(M))
    assert bits_equal(host(dx), want)


@pytest.mark.parametrize('M,Fh,ld', [(24, 768, 1536), (12, 2048, 4608), (9, 256, 512), (1100, 256, 520), (2300, 1024, 2048), (4099, 128, 256),
                                      (24, 768, 1540), (1030, 2304, 4608), (7, 2304, 4612), (1500, 640, 1284)])
def test_silu_mul_actq_bwd(M, Fh, ld):
    """the recomputed activation is the table's (the oracle's bits); the sigmoid of silu's derivative comes from a table of the correctly
    rounded expf, the oracle's from the C library's (within an ulp of it): one bf16 step at most. Row widths and strides that take
    the wave-per-row form (tables in LDS, gates at their edges in the last row) and the workgroup-per-row form (longer or unaligned rows)"""
    rng = np.random.default_rng(300 + Fh)
    base = O.f2bf((rng.standard_normal((M, ld)) * 2).astype(np.float32))
    base[0, :8] = O.f2bf(np.array([30., -30., 0., -0.0, 1e-3, -88., 88., 3.], np.float32))
    base[M - 1, :10] = O.f2bf(np.array([256., -256., 255., -255., 2.0 ** -24, -2.0 ** -24, 2.0 ** -25, -2.0 ** -25, 1e4, -1e-30], np.float32))    # the edges of the small tables
    g = O.f2bf(rng.standard_normal((M, Fh)).astype(np.float32))
    bd = dev(base)
    dgu = dev(np.zeros((M, 2 * Fh), np.uint16))
    call('camx_silu_mul_actq_bwd', ptr(bd), I(ld), I(Fh), ptr(dev(g)), ptr(dgu), F(1.0), I(7), I(M))
    gu = np.ascontiguousarray(base[:, :2 * Fh])
    act = dev(np.zeros((M, Fh), np.uint16))
    call('camx_silu_mul_bf16', ptr(dev(gu)), ptr(act), I(Fh), L64(M * Fh))
    assert bits_equal(host(act, np.uint16), O.silu_mul_bf16(gu))
    want = O.silu_mul_actq_bwd(gu, g)
    got = host(dgu, np.uint16)
    assert close_16(got, want, 'bf16')
    assert (got == want).mean() > 0.99
    assert bits_equal(got, O.silu_mul_actq_bwd(gu, g, table=True))        # bit for bit against the table's own definition (every gate here is finite)


@pytest.mark.parametrize('M,Fh', [(6, 1024), (1200, 256), (5, 2304)])
def test_silu_mul_actq_gates_of_every_magnitude(M, Fh):
    """gates and multipliers over the whole bf16 exponent range (most gates outside the small tables the wave-per-row kernels hold in
    LDS), +-inf gates, a NaN gate and a NaN multiplier: the forward bit for bit, the backward within a bf16 step, NaN for NaN"""
    from test_gpu_value_sweeps import values
    rng = np.random.default_rng(900 + M)
    with np.errstate(all='ignore'):
        gu = O.f2bf(values(rng, (M, 2 * Fh), emin=-130.0, emax=120.0))
        gu[1, :Fh] = O.f2bf(values(rng, Fh, emin=-30.0, emax=12.0))
        gu[2, 5] = 0x7f80; gu[2, 6] = 0xff80; gu[3, 9] = 0x7fc1; gu[4, Fh + 3] = 0xffc0
        g = O.f2bf(rng.standard_normal((M, Fh)).astype(np.float32))
        fy, fs, fc = O.silu_mul_actq_fwd(gu)
        want = O.silu_mul_actq_bwd(gu, g)
    gud = dev(gu)
    y = dev(np.zeros((M, Fh), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, Fh // 2), np.uint8))
    call('camx_silu_mul_actq_fwd', ptr(gud), I(2 * Fh), I(Fh), ptr(y), ptr(s), ptr(c), F(1.0), I(7), I(M))
    nan_s = np.isnan(fs)
    assert np.array_equal(np.isnan(host(s)), nan_s) and bits_equal(host(s)[~nan_s], fs[~nan_s])
    assert bits_equal(host(y, np.uint16)[~nan_s], fy[~nan_s]) and bits_equal(host(c)[~nan_s], fc[~nan_s])
    dgu = dev(np.zeros((M, 2 * Fh), np.uint16))
    call('camx_silu_mul_actq_bwd', ptr(gud), I(2 * Fh), I(Fh), ptr(dev(g)), ptr(dgu), F(1.0), I(7), I(M))
    got = host(dgu, np.uint16)
    nan_w = np.isnan(O.bf2f(want)); nan_g = np.isnan(O.bf2f(got))
    assert np.array_equal(nan_w, nan_g)
    assert close_16(np.where(nan_w, 0, got).astype(np.uint16), np.where(nan_w, 0, want).astype(np.uint16), 'bf16')


def test_actq_autograd_wrappers():
    """caminus_amd.train.actq end to end: values, codes, scales and every gradient equal the C entry points' results"""
    import torch
    from caminus_amd.train import actq as A
    rng = np.random.default_rng(7)
    M, K = 33, 1024
    x = outliers(rng, (M, K)); gy = rng.standard_normal((M, K)).astype(np.float32)
    for bf in (False, True):
        xt = torch.from_numpy(x).to('cuda:0'); xt = (xt.bfloat16() if bf else xt).requires_grad_()
        src = host(xt.detach().view(torch.int16), np.uint16) if bf else x
        y, c, s = A.actq_codes(xt.view(3, 11, K), 4, 0.9)
        ry, rs, rc = O.actq_fwd(src, clip=0.9, qmax=7, bf16=bf)
        assert y.shape == (3, 11, K) and bits_equal(host(y.view(torch.int16), np.uint16).reshape(M, K), ry) and bits_equal(host(s), rs) and bits_equal(host(c), rc)
        gt = torch.from_numpy(gy).to('cuda:0').view(3, 11, K)
        y.backward(gt)
        want = O.actq_bwd(src, O.f2bf(gy), clip=0.9, qmax=7, bf16=bf)
        assert xt.grad.dtype == xt.dtype
        assert bits_equal(host(xt.grad.view(torch.int16), np.uint16) if bf else host(xt.grad), want)
        x2 = xt.detach().clone().requires_grad_()
        A.actq(x2, 4, 0.9).backward(gt.view(M, K))
        assert torch.equal(x2.grad, xt.grad)
        assert torch.equal(A.scales(xt.detach(), 4, 0.9), s) and torch.equal(A.codes(xt.detach(), 4, 0.9)[0], c)
    # block entry
    d, nab = 896, 14
    xb = outliers(rng, (M, d)); nw = (0.5 + rng.random(d)).astype(np.float32); wab = O.f2bf((rng.standard_normal((nab, d)) / 30).astype(np.float32))
    dy = rng.standard_normal((M, d)).astype(np.float32); dab = rng.standard_normal((M, nab)).astype(np.float32)
    xt = torch.from_numpy(xb).to('cuda:0').requires_grad_(); nwt = torch.from_numpy(nw).to('cuda:0'); wt = dev(wab).view(torch.bfloat16)
    y, c, s, ab = A.block_entry(xt, nwt, wt, 1e-6)
    ry, rs, rc, rab, rstd = O.block_entry_fwd(xb, nw, wab, 1e-6)
    assert bits_equal(host(y.view(torch.int16), np.uint16), ry) and bits_equal(host(ab.view(torch.int16), np.uint16), rab) and bits_equal(host(c), rc)
    torch.autograd.backward([y, ab], [torch.from_numpy(dy).to('cuda:0'), torch.from_numpy(dab).to('cuda:0')])
    assert bits_equal(host(xt.grad), O.block_entry_bwd(xb, nw, rstd, wab, O.f2bf(dy), O.f2bf(dab)))
    # silu-mul: gradient has gu's shape and dtype, strided input accepted
    base = torch.randn(M, 4608, device='cuda:0').bfloat16()
    gu = base[:, 256:256 + 2048].detach().requires_grad_()
    yq, cq, sq = A.silu_mul_actq(gu)
    yq.backward(torch.randn(M, 1024, device='cuda:0').bfloat16())
    assert gu.grad.shape == (M, 2048) and gu.grad.dtype == torch.bfloat16 and torch.isfinite(gu.grad.float()).all()


@pytest.mark.parametrize('bf', [False, True])
def test_actq_fwd_and_bwd_four_million_values(bf):
    """enough values that the forward's division-free rounding meets its fallback thousands of times"""
    rng = np.random.default_rng(5150)
    M, K = 2048, 2048
    x = (rng.standard_normal((M, K)) * np.exp(rng.standard_normal((M, 1)))).astype(np.float32)
    g = O.f2bf(rng.standard_normal((M, K)).astype(np.float32))
    src = O.f2bf(x) if bf else x
    ry, rs, rc = O.actq_fwd(src, clip=0.95, qmax=7, bf16=bf)
    y = dev(np.zeros((M, K), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, K // 2), np.uint8))
    xd = dev(src)
    call('camx_actq_fwd', ptr(xd), I(int(bf)), ptr(y), ptr(s), ptr(c), I(K), F(0.95), I(7), I(M))
    assert bits_equal(host(s), rs) and bits_equal(host(c), rc) and bits_equal(host(y, np.uint16), ry)
    dx = dev(np.zeros((M, K), np.uint16 if bf else np.float32))
    call('camx_actq_bwd', ptr(xd), I(int(bf)), ptr(dev(g)), ptr(dx), I(K), F(0.95), I(7), I(M))
    assert bits_equal(host(dx, np.uint16) if bf else host(dx), O.actq_bwd(src, g, clip=0.95, qmax=7, bf16=bf))
