"""GPU parity of the second batch of prefill row kernels (gated GDN norm, GDN gates, fp16 KV append, add_sum, bf16 operand copies,
hyper-connection average, per-layer-embedding gate / conv / history) against the CPU oracle: bit-exact wherever no transcendental
function is involved, the fp32 / 16-bit tolerance classes elsewhere."""
import ctypes

import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, close_16, close_fp32, dev, host, outliers, ptr

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.mark.parametrize('rows,K', [(16 * 48, 128), (5, 256), (3, 96), (7, 640), (4096 * 9 + 3, 128), (2, 1024)])
def test_gdn_norm(rows, K):
    rng = np.random.default_rng(K + rows)
    o = outliers(rng, (rows, K)); z = (rng.standard_normal((rows, K)) * 3).astype(f32); w = (1 + 0.1 * rng.standard_normal(K)).astype(f32)
    od, wd, zd = dev(o), dev(w), dev(z)
    for silu in (0, 1):
        ry, ry16 = O.gdn_norm(o, w, z, 1e-6, silu=bool(silu))
        y = dev(np.zeros((rows, K), f32))
        call('camx_pf_gdn_norm', ptr(od), ptr(wd), ptr(zd), ptr(y), I(K), F(1e-6), ctypes.c_long(rows), I(silu))
        assert close_fp32(host(y), ry)
    y16 = dev(np.zeros((rows, K), np.uint16))
    call('camx_q35p_gdn_norm16', ptr(od), ptr(wd), ptr(zd), ptr(y16), I(K), F(1e-6), ctypes.c_long(rows))
    assert close_16(host(y16, np.uint16), ry16, 'f16')
    # the norm itself carries no transcendental: with z = 0 the sigmoid gate is exactly 1 / 2
    y = dev(np.zeros((rows, K), f32))
    call('camx_pf_gdn_norm', ptr(od), ptr(wd), ptr(dev(np.zeros((rows, K), f32))), ptr(y), I(K), F(1e-6), ctypes.c_long(rows), I(0))
    assert bits_equal(host(y), O.gdn_norm(o, w, np.zeros((rows, K), f32), 1e-6)[0])


def test_gdn_gates_and_kv_append16():
    rng = np.random.default_rng(3)
    T, H = 300, 48
    al = (rng.standard_normal((T, H + 5)) * 8).astype(f32); be = (rng.standard_normal((T, H)) * 4).astype(f32)
    dt = rng.standard_normal(H).astype(f32); A = -np.exp(rng.standard_normal(H)).astype(f32)
    y = dev(np.zeros((T, 2 * H), f32))
    call('camx_pf_gdn_gates', ptr(dev(al)), I(H + 5), ptr(dev(be)), I(H), ptr(dev(dt)), ptr(dev(A)), ptr(y), I(H), I(T))
    ref = O.gdn_gates(al, be, dt, A)
    assert np.allclose(host(y)[:, :H], ref[:, :H], rtol=1e-5, atol=3e-7 * np.abs(A).max()) and close_fp32(host(y)[:, H:], ref[:, H:])
    for M, ldk, ldv in ((512, 512, 520), (100, 101, 100)):
        Tk = 37
        k = outliers(rng, (Tk, ldk)) * f32(30); v = outliers(rng, (Tk, ldv)); k[0, :3] = [np.inf, np.nan, 1e6]
        cache0 = np.full((Tk + 9, 2 * M), 0x1234, np.uint16)
        for pos0, want_err in ((4, 0), (20, 1)):
            cd = dev(cache0); err = dev(np.zeros(1, np.int32))
            call('camx_q35p_kv_append16', ptr(dev(k)), I(ldk), ptr(dev(v)), I(ldv), ptr(cd), I(M), I(pos0), I(Tk + 9), ptr(err), I(Tk))
            rc, rerr = O.kv_append16(k, v, M, cache0, pos0)
            assert rerr == want_err and int(host(err)[0]) == want_err and bits_equal(host(cd, np.uint16), rc)


def test_add_sum_bf16_copies_hc_avg():
    rng = np.random.default_rng(4)
    for n in (2048 * 2560, 1001):
        a = outliers(rng, (n,)); b = outliers(rng, (n,)); y0 = outliers(rng, (n,))
        yd = dev(y0)
        call('camx_pf_add_sum', ptr(dev(a)), ptr(dev(b)), ptr(yd), L64(n))
        assert bits_equal(host(yd), O.add_sum(a, b, y0))
    for T, Tpad, K, ldx in ((37, 64, 2560, 2560), (5, 5, 33, 40), (100, 128, 512, 516)):
        x = outliers(rng, (T, ldx)); x[0, :4] = [np.nan, np.inf, -0.0, 1e-41]
        y = dev(np.full((Tpad, K), 0x7777, np.uint16))
        call('camx_pf_to_bf16', ptr(dev(x)), I(ldx), ptr(y), I(T), I(Tpad), I(K))
        assert bits_equal(host(y, np.uint16), O.to_bf16_rows(x, T, Tpad, K))
        y = dev(np.full((Tpad, K), 0x7777, np.uint16))
        xs = x.copy(); xs[0, :2] = 0
        call('camx_pf_silu_bf16', ptr(dev(xs)), I(ldx), ptr(y), I(T), I(Tpad), I(K), F(0.25))
        assert close_16(host(y, np.uint16), O.to_bf16_rows(xs, T, Tpad, K, rs=0.25, silu=True), 'bf16')
    for T, hc, D, ldo in ((2048, 4, 2560, 2560), (7, 3, 50, 64)):
        r = outliers(rng, (T, hc, D))
        y = dev(np.zeros((T, ldo), f32))
        call('camx_pf_hc_avg', ptr(dev(r)), ptr(y), I(T), I(hc), I(D), I(ldo))
        assert bits_equal(host(y), O.hc_avg(r, ldo=ldo))


@pytest.mark.parametrize('T,HC,D,dil', [(50, 4, 256, 3), (9, 2, 96, 1), (300, 4, 640, 10), (40, 3, 6, 2), (2, 1, 1030, 4)])        # (D % 4 != 0: the one-channel-per-thread conv)
def test_ple_gate_conv_hist(T, HC, D, dil):
    rng = np.random.default_rng(T + D)
    kn = rng.standard_normal((T, HC, D)).astype(f32); q = rng.standard_normal((T, HC, D)).astype(f32); val = rng.standard_normal((T, D + 4)).astype(f32)
    qscl = (0.5 + rng.random(T * HC)).astype(f32); qw = (1 + 0.1 * rng.standard_normal((HC, D))).astype(f32)
    for rec in (False, True):
        rg, rgate = O.ple_gate(kn, q, val, qscl if rec else None, qw if rec else None)
        gated = dev(np.zeros((T, HC, D), f32)); gate = dev(np.zeros((T, HC), f32))
        call('camx_pf_ple_gate', ptr(dev(kn)), ptr(dev(q)), ptr(dev(qscl)) if rec else NULL, ptr(dev(qw)) if rec else NULL, ptr(dev(val)), I(D + 4),
             ptr(gated), ptr(gate), I(HC), I(D), I(T))
        g = host(gate)
        assert close_fp32(g, rgate) and bits_equal(host(gated), (val[:, None, :D] * g[:, :, None]).astype(f32))     # the products from the device's own gates
    knd = dev(kn); gate = dev(np.zeros((T, HC), f32))                         # in place: gated written over kn
    call('camx_pf_ple_gate', ptr(knd), ptr(dev(q)), NULL, NULL, ptr(dev(val)), I(D + 4), ptr(knd), ptr(gate), I(HC), I(D), I(T))
    assert bits_equal(host(knd), (val[:, None, :D] * host(gate)[:, :, None]).astype(f32)) and close_fp32(host(gate), O.ple_gate(kn, q, val)[1])
    C = HC * D
    x = rng.standard_normal((T, C)).astype(f32); w16 = (rng.standard_normal((C, 4)) * 0.5).astype(np.float16).view(np.uint16)
    hist = rng.standard_normal((C, 3 * dil)).astype(f32); xscl = (0.5 + rng.random(T * HC)).astype(f32); xw = (1 + 0.1 * rng.standard_normal(C)).astype(f32)
    a = rng.standard_normal((T, C)).astype(f32); res = rng.standard_normal((T, C)).astype(f32)
    for rec in (False, True):
        ry, rres = O.ple_conv(x, w16, hist, D, dil, xscl if rec else None, xw if rec else None, a=a, res=res)
        y = dev(np.zeros((T, C), f32)); rd = dev(res)
        sc, sw = (ptr(dev(xscl)), ptr(dev(xw))) if rec else (NULL, NULL)
        call('camx_pf_ple_conv', ptr(dev(x)), sc, sw, ptr(dev(w16)), ptr(dev(hist)), ptr(y), ptr(dev(a)), ptr(rd), I(C), I(T), I(D), I(dil))
        assert close_fp32(host(y), ry) and bits_equal(host(rd), (res + (a + host(y))).astype(f32))
        hd = dev(hist)
        call('camx_pf_ple_hist', ptr(dev(x)), sc, sw, ptr(hd), I(C), I(T), I(D), I(dil))
        assert bits_equal(host(hd), O.ple_hist(x, hist, D, dil, xscl if rec else None, xw if rec else None))
    hd = dev(hist)                                                            # a chunk shorter than the history keeps its tail
    call('camx_pf_ple_hist', ptr(dev(x)), NULL, NULL, ptr(hd), I(C), I(2), I(D), I(dil))
    assert bits_equal(host(hd), O.ple_hist(x[:2], hist, D, dil))


def test_launcher_surface_of_the_new_symbols():
    """the reference's module and symbol names reach the entry points with the reference's argument lists"""
    import torch
    from caminus_amd.device.hip import Module
    rng = np.random.default_rng(8)
    rows, K = 64, 128
    o = outliers(rng, (rows, K)); z = rng.standard_normal((rows, K)).astype(f32); w = np.ones(K, f32)
    od, wd, zd = dev(o), dev(w), dev(z)
    for module, silu in (('prefill_gdn', False), ('prefill_gdn_q35', True)):
        y = dev(np.zeros((rows, K), f32))
        Module(module).pf_gdn_norm((rows,), (256,), od, wd, zd, y, ctypes.c_int(K), ctypes.c_float(1e-6))
        torch.cuda.synchronize()
        assert close_fp32(host(y), O.gdn_norm(o, w, z, 1e-6, silu=silu)[0])
    y16 = dev(np.zeros((rows, K), np.uint16))
    Module('q35_prefill').q35p_gdn_norm16((rows,), (256,), od, wd, zd, y16, ctypes.c_int(K), ctypes.c_float(1e-6))
    a = dev(o); b = dev(z); yy = dev(o)
    Module('prefill_glue').pf_add_sum(((rows * K + 255) // 256,), (256,), a, b, yy, ctypes.c_long(rows * K))
    torch.cuda.synchronize()
    assert close_16(host(y16, np.uint16), O.gdn_norm(o, w, z, 1e-6, silu=True)[1], 'f16') and bits_equal(host(yy), O.add_sum(o, z, o))


def test_host_wrappers_of_the_new_ops():
    """Glue / Gdn / Attn / q35 Ops methods with the reference's argument lists, against the oracle"""
    import torch
    from caminus_amd.prefill import attn as A, gdn as G, glue as GL, q35_ops
    rng = np.random.default_rng(9)
    T, HC, D = 12, 4, 2560
    gl = GL.Glue('cuda:0')
    a = outliers(rng, (T * D,)); b = outliers(rng, (T * D,)); y0 = outliers(rng, (T * D,))
    yd = dev(y0); gl.add_sum(dev(a), dev(b), yd, T * D)
    x = outliers(rng, (T, D)); ybf = dev(np.zeros((GL.tpad(T), D), np.uint16)).view(torch.bfloat16)
    gl.to_bf16(dev(x), ybf, T, D)
    kn = rng.standard_normal((T, HC, D)).astype(f32); q = rng.standard_normal((T, HC, D)).astype(f32); val = rng.standard_normal((T, D)).astype(f32)
    gated = dev(np.zeros((T, HC, D), f32)); gate = dev(np.zeros((T, HC), f32))
    gl.ple_gate(dev(kn), dev(q), dev(val), gated, gate, T, HC)
    C = HC * D
    xc = rng.standard_normal((T, C)).astype(f32); w16 = (rng.standard_normal((C, 4)) * 0.5).astype(np.float16); hist = rng.standard_normal((C, 9)).astype(f32)
    yc = dev(np.zeros((T, C), f32)); hd = dev(hist)
    gl.ple_conv(dev(xc), torch.from_numpy(w16).to('cuda:0'), hd, C, T, y=yc)
    with pytest.raises(ValueError):
        gl.ple_conv(dev(xc), torch.from_numpy(w16).to('cuda:0'), hd, C, T)                  # neither y nor res
    with pytest.raises(ValueError):
        gl.ple_gate(dev(kn), dev(q), dev(val), gated, gate, T, 9)                         # more than eight streams
    torch.cuda.synchronize()
    assert bits_equal(host(yd), O.add_sum(a, b, y0)) and bits_equal(host(ybf.view(torch.int16), np.uint16), O.to_bf16_rows(x, T, GL.tpad(T), D))
    assert close_fp32(host(gate), O.ple_gate(kn, q, val)[1])
    assert close_fp32(host(yc), O.ple_conv(xc, w16.view(np.uint16), hist, D, 3)[0]) and bits_equal(host(hd), O.ple_hist(xc, hist, D, 3))
    H, K = 6, 128
    o = outliers(rng, (T * H, K)); z = rng.standard_normal((T * H, K)).astype(f32); w = (1 + 0.1 * rng.standard_normal(K)).astype(f32)
    for module, silu in (('prefill_gdn', False), ('prefill_gdn_q35', True)):
        g = G.Gdn('cuda:0', module=module); y = dev(np.zeros((T * H, K), f32))
        g.norm(dev(o), dev(w), dev(z), y, T, H, 1e-6)
        torch.cuda.synchronize()
        assert close_fp32(host(y), O.gdn_norm(o, w, z, 1e-6, silu=silu)[0])
    al = rng.standard_normal((T, H)).astype(f32); be = rng.standard_normal((T, H)).astype(f32); dt = rng.standard_normal(H).astype(f32); Aa = -np.ones(H, f32)
    out = dev(np.zeros((T, 2 * H), f32)); g.gates(dev(al), dev(be), dev(dt), dev(Aa), out, T, H)
    r = outliers(rng, (T, 4, 64)); ya = dev(np.zeros((T, 64), f32))
    A.Attn('cuda:0').hc_avg(dev(r), ya, T, 4, 64)
    ops = q35_ops.Ops('cuda:0')
    y16 = dev(np.zeros((T * H, K), np.uint16)).view(torch.float16)
    ops.gdn_norm16(dev(o), dev(w), dev(z), y16, T, H, K, 1e-6)
    M = 256; k = outliers(rng, (T, M)); v = outliers(rng, (T, M)); cache = dev(np.zeros((T + 4, 2 * M), np.uint16)).view(torch.float16); err = dev(np.zeros(1, np.int32))
    ops.kv_append16(dev(k), M, dev(v), M, cache, M, 2, T, T + 4, err)
    with pytest.raises(IndexError):
        ops.kv_append16(dev(k), M, dev(v), M, cache, M, 5, T, T + 4, err)                   # rows 5 .. 16 of 16
    torch.cuda.synchronize()
    assert np.allclose(host(out), O.gdn_gates(al, be, dt, Aa), rtol=1e-5, atol=1e-6) and bits_equal(host(ya), O.hc_avg(r))
    assert close_16(host(y16.view(torch.int16), np.uint16), O.gdn_norm(o, w, z, 1e-6, silu=True)[1], 'f16')
    assert bits_equal(host(cache.view(torch.int16), np.uint16), O.kv_append16(k, v, M, np.zeros((T + 4, 2 * M), np.uint16), 2)[0]) and int(host(err)[0]) == 0
