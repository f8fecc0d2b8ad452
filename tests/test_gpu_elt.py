"""GPU parity of the elementwise / small row kernels against the CPU oracle: exact where no transcendental is involved,
1e-5 relative (fp32) / one 16-bit ulp otherwise."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, close_16, close_fp32, dev, host, outliers, ptr

pytestmark = pytest.mark.gpu
EXTREMES = np.array([30, -30, 0, -0.0, 1e-3, -88, 88, 5], np.float32)


@pytest.mark.parametrize('n', [8 * 768, 1001, 7])
def test_swiglu(n):
    rng = np.random.default_rng(n)
    g = outliers(rng, n); u = outliers(rng, n); g[:min(8, n)] = EXTREMES[:min(8, n)]
    y16 = dev(np.zeros(n, np.uint16)); y32 = dev(np.zeros(n, np.float32)); gd, ud = dev(g), dev(u)
    call('camx_q3p_swiglu', ptr(gd), ptr(ud), ptr(y16), I(n))
    call('camx_gg_silu_mul', ptr(gd), ptr(ud), ptr(y32), I(n))
    assert close_16(host(y16, np.uint16), O.swiglu16(g, u), 'f16')
    assert close_fp32(host(y32), O.silu_mul_f32(g, u))


@pytest.mark.parametrize('R,H', [(4, 17408), (3, 7), (256, 17408), (1100, 4096)])
def test_silu_mul_bf16(R, H):
    """bf16(silu g) comes from the table of the correctly rounded value at every size (in device memory for small inputs, in LDS
    from 2^22 values on): bit-equal to the oracle, NaN (canonical) and infinities included"""
    rng = np.random.default_rng(H)
    gu = O.f2bf(outliers(rng, (R, 2 * H)) * np.float32(2))
    gu[0, :6] = [0x7fc0, 0xffc1, 0x7f80, 0xff80, 0x0000, 0x8000]; gu[0, H:H + 6] = [0x3f80, 0x3f80, 0x0000, 0x3f80, 0x7f80, 0x7fa5]
    act = dev(np.zeros((R, H), np.uint16))
    call('camx_silu_mul_bf16', ptr(dev(gu)), ptr(act), I(H), L64(R * H))
    want = O.silu_mul_bf16(gu); got = host(act, np.uint16)
    assert np.array_equal(got, want)


def test_gate_mul():
    rng = np.random.default_rng(1004)
    T, H, D = 16, 24, 256
    a = outliers(rng, (T * H, D)); qg = outliers(rng, (T * H, 2 * D)); qg[0, D:D + 8] = EXTREMES
    ad, gd = dev(a), dev(qg)
    y = dev(np.zeros_like(a)); y16 = dev(np.zeros(a.shape, np.uint16))
    call('camx_gate_mul', ptr(ad), ptr(gd), ptr(y), L64(a.size), I(D), I(2 * D), I(D), I(0))
    call('camx_gate_mul', ptr(ad), ptr(gd), ptr(y16), L64(a.size), I(D), I(2 * D), I(D), I(1))
    assert close_fp32(host(y), O.gate_mul(a, qg, D, 2 * D, D))
    assert close_16(host(y16, np.uint16), O.gate_mul(a, qg, D, 2 * D, D, f16=True), 'f16')
    abf, gbf = O.f2bf(a), O.f2bf(qg)
    ybf = dev(np.zeros(a.shape, np.uint16))
    call('camx_gate_mul', ptr(dev(abf)), ptr(dev(gbf)), ptr(ybf), L64(a.size), I(D), I(2 * D), I(D), I(2))
    assert close_16(host(ybf, np.uint16), O.f2bf(O.gate_mul(O.bf2f(abf), O.bf2f(gbf), D, 2 * D, D)), 'bf16')


@pytest.mark.parametrize('T,C', [(16, 10240), (1, 64), (2, 100), (5, 256), (37, 512), (3, 6), (520, 8192), (130, 8200)])
def test_gdn_conv(T, C):
    rng = np.random.default_rng(C)
    ldx = C + 4
    x = outliers(rng, (T, ldx)); w = rng.standard_normal((C, 4)).astype(np.float32); st = rng.standard_normal((C, 3)).astype(np.float32)
    ref_y, ref_st = O.gdn_conv(x, w, st, ldx=ldx)
    xd, wd, sd = dev(x), dev(w), dev(st); y = dev(np.zeros((T, C), np.float32))
    call('camx_pf_gdn_conv', ptr(xd), ptr(wd), ptr(sd), ptr(y), I(C), I(T), I(ldx), I(C), I(0))
    call('camx_pf_conv_state', ptr(xd), ptr(sd), I(C), I(T), I(ldx), I(0))
    assert close_fp32(host(y), ref_y) and bits_equal(host(sd), ref_st)


@pytest.mark.parametrize('T,heads,K', [(16, 32, 128), (16, 48, 128), (3, 5, 256), (2, 3, 96), (1030, 32, 128), (683, 48, 128), (2049, 32, 128), (1401, 48, 128)])
def test_gdn_l2(T, heads, K):
    rng = np.random.default_rng(K + heads)
    ldx = heads * K + 64
    x = outliers(rng, (T, ldx))
    y = dev(np.zeros((T * heads, K), np.float32))
    call('camx_pf_gdn_l2', ptr(dev(x)), ptr(y), I(heads), I(K), I(ldx), F(np.float32(1e-6 / K)), I(T), I(0))
    ref = O.gdn_l2(x, T, heads, K, 1e-6, ldx=ldx)
    assert bits_equal(host(y), ref)
    if K == 128:                                                       # bf16 in / out (a prefill chunk's form)
        xb = O.f2bf(x); yb = dev(np.zeros((T * heads, K), np.uint16))
        call('camx_pf_gdn_l2', ptr(dev(xb)), ptr(yb), I(heads), I(K), I(ldx), F(np.float32(1e-6 / K)), I(T), I(1))
        assert bits_equal(host(yb, np.uint16), O.f2bf(O.gdn_l2(O.bf2f(xb), T, heads, K, 1e-6, ldx=ldx)))


def test_core_and_fuse():
    rng = np.random.default_rng(5)
    T, D, V = 9, 896, 50
    emb = rng.standard_normal((V, D)).astype(np.float32); tok = rng.integers(0, V, T).astype(np.int32)
    out = dev(np.zeros((T, D), np.float32))
    call('camx_embedding_f32', ptr(dev(tok)), ptr(dev(emb)), ptr(out), I(D), I(T))
    assert bits_equal(host(out), O.embedding_f32(tok, emb))
    x = outliers(rng, (T, D))
    m = O.f2bf(outliers(rng, (T, D))); y = O.f2bf(outliers(rng, (T, D)))
    o = dev(np.zeros((T, D), np.float32))
    call('camx_residual3', ptr(dev(x)), ptr(dev(m)), ptr(dev(y)), ptr(o), L64(T * D))
    assert bits_equal(host(o), O.residual3(x, m, y))
    o1 = dev(np.zeros(T * D - 3, np.float32))                          # a length that is no multiple of four: the element-wise form
    call('camx_residual3', ptr(dev(x)), ptr(dev(m)), ptr(dev(y)), ptr(o1), L64(T * D - 3))
    assert bits_equal(host(o1), O.residual3(x, m, y).reshape(-1)[:T * D - 3])
    x[0, :6] = [np.nan, np.inf, -np.inf, 1e-40, -np.nan, 3.3895314e38]
    c = dev(np.zeros((T, D), np.uint16))
    call('camx_cast_bf16', ptr(dev(x)), ptr(c), L64(T * D))
    assert bits_equal(host(c, np.uint16), O.f2bf(x))
    c1 = dev(np.zeros(T * D - 5, np.uint16))
    call('camx_cast_bf16', ptr(dev(x)), ptr(c1), L64(T * D - 5))
    assert bits_equal(host(c1, np.uint16), O.f2bf(x).reshape(-1)[:T * D - 5])
    dst = rng.integers(0, 65536, (T, 64)).astype(np.uint16); dd = dev(dst)
    call('camx_copy_cols_bf16', ptr(dev(m)), I(D), I(5), ptr(dd), I(64), I(3), I(40), L64(T))
    assert bits_equal(host(dd, np.uint16), O.copy_cols_bf16(m, 5, dst, 3, 40))
    dd2 = dev(dst)                                                     # offsets and width in whole 16-byte units
    call('camx_copy_cols_bf16', ptr(dev(m)), I(D), I(8), ptr(dd2), I(64), I(16), I(40), L64(T))
    assert bits_equal(host(dd2, np.uint16), O.copy_cols_bf16(m, 8, dst, 16, 40))
    whole = rng.integers(0, 65536, (517, 64)).astype(np.uint16); dd3 = dev(np.zeros((517, 64), np.uint16))     # whole contiguous rows: the flat copy
    call('camx_copy_cols_bf16', ptr(dev(whole)), I(64), I(0), ptr(dd3), I(64), I(0), I(64), L64(517))
    assert bits_equal(host(dd3, np.uint16), whole)
    ys = O.f2bf(outliers(rng, (4, D))); pos = np.array([-1, 0, 3, -1, 2, 1, -1, -1, 0], np.int32)
    x2 = outliers(rng, (T, D))
    for has in (True, False):
        o2 = dev(np.zeros((T, D), np.float32))
        call('camx_residual_slices_fwd', ptr(dev(x2)), ptr(dev(m)), ptr(dev(y)), ptr(dev(ys)) if has else NULL, ptr(dev(pos)) if has else NULL,
             ptr(o2), I(D), L64(T * D // 4))
        assert bits_equal(host(o2), O.residual_slices_fwd(x2, m, y, ys if has else None, pos if has else None))


@pytest.mark.parametrize('T,D', [(9, 896), (300, 2048), (7, 892), (33, 100), (5, 8)])
def test_residual_slices_widths(T, D):
    """several row widths and counts, forward and backward, with and without slices, non-finite and subnormal values"""
    rng = np.random.default_rng(60 + D)
    nys = 4
    x = outliers(rng, (T, D)); m = O.f2bf(outliers(rng, (T, D))); mlp = O.f2bf(outliers(rng, (T, D))); ys = O.f2bf(outliers(rng, (nys, D)))
    pos = rng.integers(-1, nys, T).astype(np.int32); pos[rng.random(T) < 0.5] = -1
    taken = pos[pos >= 0]; pos[pos >= 0] = np.where(np.arange(len(taken)) < nys, rng.permutation(nys)[np.arange(len(taken)) % nys], -1)   # each slice at most once
    seen = set()
    for r in range(T):
        if pos[r] >= 0 and int(pos[r]) in seen: pos[r] = -1
        elif pos[r] >= 0: seen.add(int(pos[r]))
    x[0, :4] = [np.nan, np.inf, -0.0, 1e-40]
    for has in (True, False):
        o = dev(np.zeros((T, D), np.float32))
        call('camx_residual_slices_fwd', ptr(dev(x)), ptr(dev(m)), ptr(dev(mlp)), ptr(dev(ys)) if has else NULL, ptr(dev(pos)) if has else NULL, ptr(o), I(D), L64(T * D // 4))
        want = O.residual_slices_fwd(x, m, mlp, ys if has else None, pos if has else None)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(host(o)), nan) and bits_equal(np.where(nan, 0, host(o)), np.where(nan, 0, want))
    rdm, rdmlp, rdys = O.residual_slices_bwd(x, pos, nys)
    dm = dev(np.zeros((T, D), np.uint16)); dmlp = dev(np.zeros((T, D), np.uint16)); dys = dev(np.zeros((nys, D), np.uint16))
    call('camx_residual_slices_bwd', ptr(dev(x)), ptr(dev(pos)), ptr(dm), ptr(dmlp), ptr(dys), I(D), L64(T * D // 4))
    used = sorted(seen)
    assert bits_equal(host(dm, np.uint16), rdm) and bits_equal(host(dmlp, np.uint16), rdmlp) and bits_equal(host(dys, np.uint16)[used], rdys[used])


def test_residual_slices_bwd_and_autograd():
    """the backward kernel against the oracle, and the autograd wrapper end to end against torch's own graph of the same sum"""
    import torch
    from caminus_amd.train.fuse import residual_slices
    rng = np.random.default_rng(6)
    T, D, nys = 11, 896, 5
    dout = outliers(rng, (T, D)); dout[0, :3] = [np.nan, np.inf, 3.3895314e38]
    pos = np.array([-1, 0, 3, -1, 2, 1, -1, -1, 4, -1, -1], np.int32)
    rdm, rdmlp, rdys = O.residual_slices_bwd(dout, pos, nys)
    dm = dev(np.zeros((T, D), np.uint16)); dmlp = dev(np.zeros((T, D), np.uint16)); dys = dev(np.zeros((nys, D), np.uint16))
    call('camx_residual_slices_bwd', ptr(dev(dout)), ptr(dev(pos)), ptr(dm), ptr(dmlp), ptr(dys), I(D), L64(T * D // 4))
    assert bits_equal(host(dm, np.uint16), rdm) and bits_equal(host(dmlp, np.uint16), rdmlp) and bits_equal(host(dys, np.uint16), rdys)
    x = torch.randn(T, D, device='cuda:0', requires_grad=True)
    m = torch.randn(T, D, device='cuda:0').bfloat16().requires_grad_(); mlp = torch.randn(T, D, device='cuda:0').bfloat16().requires_grad_()
    ys = torch.randn(nys, D, device='cuda:0').bfloat16().requires_grad_(); pd = torch.from_numpy(pos).to('cuda:0')
    out = residual_slices(x, m, mlp, ys, pd)
    gsel = torch.zeros(T, D, device='cuda:0'); sel = pd >= 0
    gsel[sel] = ys.detach().float()[pd[sel].long()]
    want = ((x.detach() + m.detach().float()) + mlp.detach().float()) + gsel
    assert torch.equal(out.detach(), want)
    go = torch.randn(T, D, device='cuda:0')
    out.backward(go)
    assert torch.equal(x.grad, go) and torch.equal(m.grad, go.bfloat16()) and torch.equal(mlp.grad, go.bfloat16())
    assert torch.equal(ys.grad[pd[sel].long()], go[sel].bfloat16())


def test_cast_bf16_every_upper_half_with_edge_lower_halves():
    """fp32 -> bf16 over every sign / exponent / top-mantissa pattern combined with the lower halves where rounding decides
    (ties, one off a tie, all ones), NaN payloads and denormals included: 0x7fc0 for every NaN, nearest-even elsewhere"""
    hi = np.arange(65536, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7fff, 0x8000, 0x8001, 0xffff, 0x4000, 0xc000, 0x8000 - 2, 0x1234, 0xfedc, 0x8002], np.uint32)
    x = (hi[:, None] | lows[None, :]).reshape(-1).view(np.float32)
    c = dev(np.zeros(x.size, np.uint16))
    call('camx_cast_bf16', ptr(dev(x)), ptr(c), L64(x.size))
    assert bits_equal(host(c, np.uint16), O.f2bf(x))
    c1 = dev(np.zeros(x.size - 1, np.uint16))                             # the element-wise form
    call('camx_cast_bf16', ptr(dev(x)), ptr(c1), L64(x.size - 1))
    assert bits_equal(host(c1, np.uint16), O.f2bf(x)[:-1])


@pytest.mark.parametrize('C,T', [(10240, 16), (96, 5), (300, 1)])
def test_op_gdn_conv_lazy_commit(C, T):
    """OP_GDN_CONV: two passes with every commit count; the state after the commit and the next pass's xprev bit for bit, the outputs
    within the FP class (silu) and equal to the chunk kernel's on the same state"""
    from gpu_util import close_fp32
    rng = np.random.default_rng(C + T)
    w = rng.standard_normal((C, 4)).astype(np.float32); st0 = rng.standard_normal((C, 3)).astype(np.float32)
    x1 = outliers(rng, (T, C)); x2 = outliers(rng, (T, C)); junk = rng.standard_normal((T, C)).astype(np.float32)
    wd = dev(w)
    for m in sorted({0, 1, T // 2, T}):
        std = dev(st0); xp = dev(junk); y = dev(np.zeros((T, C), np.float32))
        call('camx_op_gdn_conv', ptr(wd), ptr(std), ptr(dev(x1)), ptr(dev(np.array([0, 0, 0, 0], np.int32))), ptr(y), ptr(xp), I(C), I(T))
        ry1, rst1, rxp1 = O.op_gdn_conv(w, st0, x1, 0, junk)
        assert bits_equal(host(std), rst1) and bits_equal(host(xp), rxp1) and close_fp32(host(y), ry1)
        y2 = dev(np.zeros((T, C), np.float32))
        call('camx_op_gdn_conv', ptr(wd), ptr(std), ptr(dev(x2)), ptr(dev(np.array([7, m, 0, 0], np.int32))), ptr(y2), ptr(xp), I(C), I(T))
        ry2, rst2, rxp2 = O.op_gdn_conv(w, rst1, x2, m, rxp1)
        assert bits_equal(host(std), rst2) and bits_equal(host(xp), rxp2) and close_fp32(host(y2), ry2)
        yc = dev(np.zeros((T, C), np.float32))                      # the chunk kernel from the committed state: the same bits
        call('camx_pf_gdn_conv', ptr(dev(x2)), ptr(wd), ptr(std), ptr(yc), I(C), I(T), I(C), I(C), I(0))
        assert bits_equal(host(yc), host(y2))
