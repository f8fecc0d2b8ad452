"""The same tokens in one launch and split over several give the same bits (the reference's chunk-geometry gate, e.g.
tests/prefill/test_prefill_glue.py): entry points whose kernel depends on the batch size (streaming / wide kernels from some size
on, decode-sized kernels below) and whose outputs pass a transcendental, so that agreement with the oracle within a tolerance
would not imply it."""
import ctypes

import numpy as np
import pytest

import oracle as O
from caminus_amd import rope
from gpu_util import F, I, L64, NULL, bits_equal, call, dev, host, outliers, ptr
from vectors import qk_par

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.mark.parametrize('bf16', [0, 1])
def test_gdn_conv_chunks(bf16):
    """600 tokens at once (the streaming kernel) and in chunks of 37 and 1 with the state carried between them"""
    rng = np.random.default_rng(5)
    T, C = 600, 2048
    x = outliers(rng, (T, C)); w = rng.standard_normal((C, 4)).astype(f32); st0 = rng.standard_normal((C, 3)).astype(f32)
    xin = O.f2bf(x) if bf16 else x
    ydt = np.uint16 if bf16 else f32
    xd, wd = dev(xin), dev(w)
    results = []
    for chunk in (T, 37, 1):
        if chunk == 1 and not bf16: continue
        sd = dev(st0.copy()); y = dev(np.zeros((T, C), ydt))
        for t in range(0, T, chunk):
            m = min(chunk, T - t)
            call('camx_pf_gdn_conv', ptr(xd[t:]), ptr(wd), ptr(sd), ptr(y[t:]), I(C), I(m), I(C), I(C), I(bf16))
            call('camx_pf_conv_state', ptr(xd[t:]), ptr(sd), I(C), I(m), I(C), I(bf16))
        results.append((host(y, ydt) if bf16 else host(y), host(sd)))
    for y, s in results[1:]:
        assert bits_equal(y, results[0][0]) and bits_equal(s, results[0][1])


def test_gdn_norm_chunks():
    """40000 rows of 128 (the four-rows-per-half-wave kernel) and chunks of 5000 (the row kernel): fp16 and fp32 outputs"""
    rng = np.random.default_rng(6)
    rows, K = 40000, 128
    o = outliers(rng, (rows, K)); z = (rng.standard_normal((rows, K)) * 3).astype(f32); w = (1 + 0.1 * rng.standard_normal(K)).astype(f32)
    od, wd, zd = dev(o), dev(w), dev(z)
    for name, dt, extra in (('camx_q35p_gdn_norm16', np.uint16, ()), ('camx_pf_gdn_norm', f32, (I(1),)), ('camx_pf_gdn_norm', f32, (I(0),))):
        outs = []
        for chunk in (rows, 5000):
            y = dev(np.zeros((rows, K), dt))
            for r in range(0, rows, chunk):
                m = min(chunk, rows - r)
                call(name, ptr(od[r:]), ptr(wd), ptr(zd[r:]), ptr(y[r:]), I(K), F(1e-6), ctypes.c_long(m), *extra)
            outs.append(host(y, dt) if dt == np.uint16 else host(y))
        assert bits_equal(outs[0], outs[1]), name


@pytest.mark.parametrize('io,D,n_rot', [(0, 256, 64), (1, 256, 64), (1, 128, 128), (0, 96, 32), (0, 512, 128), (1, 200, 48), (0, 256, 256)])
def test_qk_nr_chunks(io, D, n_rot):
    """600 tokens x 8 heads at once (the per-token kernels) and in chunks of 100 (the per-head kernel)"""
    rng = np.random.default_rng(7 + D)
    T, heads, stride, pos0 = 600, 8, D + 8, 4000
    x = outliers(rng, (T * heads, stride)); w = (1 + 0.1 * rng.standard_normal(D)).astype(f32)
    ts = float(f32(f32(1e6) ** f32(-2.0 / n_rot)))
    xin = O.f2bf(x) if io else x
    dt = np.uint16 if io else f32
    xd, wd = dev(xin), dev(w)
    outs = []
    for chunk in (T, 100):
        y = dev(np.zeros((T * heads, D), dt))
        for t in range(0, T, chunk):
            m = min(chunk, T - t)
            call('camx_pf_qk_nr', ptr(xd[t * heads:]), I(stride), I(heads), ptr(wd), I(D), I(n_rot), F(ts), F(1e-6), I(pos0 + t), ptr(y[t * heads:]), I(m), I(io))
        outs.append(host(y, dt) if io else host(y))
    assert bits_equal(outs[0], outs[1])


@pytest.mark.parametrize('yarn', [False, True])
def test_qk_rope_bf16_chunks(yarn):
    """2049 tokens of bf16 rows at once (four tokens per workgroup) and in chunks of 500 (one)"""
    rng = np.random.default_rng(8)
    nh, nkv, n, pos0 = 20, 4, 2049, 3
    tab = rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None
    par = qk_par(rng, yarn_table=tab)
    ldq = (nh + 2 * nkv) * 128
    qkv = O.f2bf(outliers(rng, (n, ldq)) * f32(1.3))
    M = nkv * 128; rows = pos0 + n + 1
    qd, pd = dev(qkv), dev(par)
    outs = []
    for chunk in (n, 500):
        q16 = dev(np.zeros((n, nh, 128), np.uint16)); c16 = dev(np.zeros((rows, 2 * M), np.uint16))
        for t in range(0, n, chunk):
            m = min(chunk, n - t)
            call('camx_qk_rope_bf16', ptr(qd[t:]), I(ldq), I(nh), I(nkv), ptr(pd), I(pos0 + t), ptr(q16[t:]), ptr(c16), I(m), I(int(yarn)))
        outs.append((host(q16, np.uint16), host(c16, np.uint16)))
    assert bits_equal(outs[0][0], outs[1][0]) and bits_equal(outs[0][1], outs[1][1])
    # the same rows at a stride that rules out 128-bit loads (the half-wave-per-head kernel)
    ld2 = ldq + 4
    wide = np.zeros((n, ld2), np.uint16); wide[:, :ldq] = qkv
    q16 = dev(np.zeros((n, nh, 128), np.uint16)); c16 = dev(np.zeros((rows, 2 * M), np.uint16))
    call('camx_qk_rope_bf16', ptr(dev(wide)), I(ld2), I(nh), I(nkv), ptr(pd), I(pos0), ptr(q16), ptr(c16), I(n), I(int(yarn)))
    assert bits_equal(host(q16, np.uint16), outs[0][0]) and bits_equal(host(c16, np.uint16), outs[0][1])


def test_elementwise_chunks():
    """SwiGLU to fp16 and fp32, the sigmoid gate in its three forms, and bf16 SwiGLU across the size where the table moves into LDS"""
    rng = np.random.default_rng(9)
    n = 3 << 20
    g = outliers(rng, n) * f32(2); u = outliers(rng, n)
    gd, ud = dev(g), dev(u)
    for name, dt in (('camx_q3p_swiglu', np.uint16), ('camx_gg_silu_mul', f32)):
        outs = []
        for chunk in (n, 4096 + 7 * 4):
            y = dev(np.zeros(n, dt))
            for t in range(0, n, chunk):
                call(name, ptr(gd[t:]), ptr(ud[t:]), ptr(y[t:]), I(min(chunk, n - t)))
            outs.append(host(y, dt) if dt == np.uint16 else host(y))
        assert bits_equal(outs[0], outs[1]), name
    T, H, D = 4096, 8, 256
    a = outliers(rng, (T * H, D)); qg = outliers(rng, (T * H, 2 * D))
    for io, src_a, src_g, dt in ((0, a, qg, f32), (1, a, qg, np.uint16), (2, O.f2bf(a), O.f2bf(qg), np.uint16)):
        ad, qd = dev(src_a), dev(src_g)
        outs = []
        for chunk in (T * H, 16 * H):
            y = dev(np.zeros((T * H, D), dt))
            for r in range(0, T * H, chunk):
                m = min(chunk, T * H - r)
                call('camx_gate_mul', ptr(ad[r:]), ptr(qd[r:]), ptr(y[r:]), L64(m * D), I(D), I(2 * D), I(D), I(io))
            outs.append(host(y, dt) if dt == np.uint16 else host(y))
        assert bits_equal(outs[0], outs[1]), io
    R, Hh = 1040, 4096                                                   # 4.26 M values: the LDS-table kernel; chunks of 16 rows: the small one
    gu = O.f2bf(outliers(rng, (R, 2 * Hh)) * f32(2))
    gud = dev(gu)
    outs = []
    for chunk in (R, 16):
        act = dev(np.zeros((R, Hh), np.uint16))
        for r in range(0, R, chunk):
            m = min(chunk, R - r)
            call('camx_silu_mul_bf16', ptr(gud[r:]), ptr(act[r:]), I(Hh), L64(m * Hh))
        outs.append(host(act, np.uint16))
    assert bits_equal(outs[0], outs[1])
