"""The five workload configurations at their full sizes, seeded as the measurement plan states (seeds 1001 .. 1005), each
op-set through the C ABI against the CPU oracle on the same inputs, plus the size-independent properties the domain
offers (chunk-split invariance, paged rows equal unpaged rows, a checksum over the untouched part of the paged cache).

Tolerances: bit-exact for everything that does not pass a transcendental (norms, q8_1 / MMQ / Q8 KV bytes given their
fp16 / bf16 inputs, dequantized rows); one fp16 / bf16 unit in the last place + 1e-5 x max for rotary, SwiGLU, gates, conv.
"""
import numpy as np
import pytest
import torch

import oracle as O
from caminus_amd import rope
from gpu_util import F, I, L64, NULL, bits_equal, call, close_16, close_fp32, dev, host, outliers, ptr
from vectors import q4k_table, q80_table, qk_par

pytestmark = pytest.mark.gpu


def _gamma(rng, n):
    return (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)


def test_config1_decode_token():
    """Qwen3-30B-A3B-shaped single decode token: add + RMSNorm over 2048, q8_1 of the normed row, QK-norm + NeoX rotary on
    32 Q + 4 KV heads of 128 at a random position below 4096 (theta 1e6), SwiGLU for 8 experts x 768"""
    rng = np.random.default_rng(1001)
    N, nh, nkv = 2048, 32, 4
    x = outliers(rng, (1, N)); d = outliers(rng, (1, 1, N)); nw = _gamma(rng, N)
    ref = O.add_rms16(x, nw, 1e-6, d=d, S=1, want_q8=True)
    xd = dev(x); h = dev(np.zeros((1, N), np.float32)); h16 = dev(np.zeros((1, N), np.uint16)); q8 = dev(np.zeros((N // 32, 36), np.uint8))
    call('camx_q3p_add_rms16', ptr(xd), ptr(dev(d)), NULL, I(1), ptr(dev(nw)), F(1e-6), ptr(h), ptr(h16), I(N), I(1))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16, np.uint16), ref['h16'])
    call('camx_gg_quantize_q8_1', ptr(h), ptr(q8), L64(N), I(0), F(0), NULL)
    assert bits_equal(host(q8), ref['q8'][0]) and bits_equal(host(q8), O.q8_1(ref['h'][0]))
    # the fused form gives the same blocks in one launch
    x2 = dev(x); q8b = dev(np.zeros((N // 32, 36), np.uint8))
    call('camx_add_rms_q8_1', ptr(x2), ptr(dev(d)), NULL, I(1), ptr(dev(nw)), F(1e-6), NULL, NULL, ptr(q8b), I(N), I(1))
    assert bits_equal(host(q8b), host(q8))

    par = qk_par(rng, theta_base=1e6)
    pos = int(rng.integers(0, 4096))
    ldq = (nh + 2 * nkv) * 128
    qkv = outliers(rng, (1, ldq)); M = nkv * 128
    q16 = dev(np.zeros((1, nh, 128), np.uint16)); c16 = dev(np.zeros((4096, 2 * M), np.uint16))
    call('camx_q3p_qk_rope', ptr(dev(qkv)), I(ldq), I(nh), I(nkv), ptr(dev(par)), I(pos), ptr(q16), ptr(c16), I(1), I(0))
    rq, rc, _ = O.qk_rope(qkv, nh, nkv, par, 1, pos0=pos, rows=4096)
    gc = host(c16, np.uint16)
    assert close_16(host(q16, np.uint16), rq, 'f16') and close_16(gc[pos, :M], rc[pos, :M], 'f16') and bits_equal(gc[pos, M:], rc[pos, M:])
    gc[pos] = 0
    assert not gc.any()

    n = 8 * 768
    g = outliers(rng, n); u = outliers(rng, n)
    y16 = dev(np.zeros(n, np.uint16))
    call('camx_q3p_swiglu', ptr(dev(g)), ptr(dev(u)), ptr(y16), I(n))
    assert close_16(host(y16, np.uint16), O.swiglu16(g, u), 'f16')


@pytest.mark.parametrize('T', [1, 4])
def test_config1_decode_tape_row_ops(T):
    """The qwen3moe decode tape at config 1's shapes through the host mirror's TapeOps (python/caminus/engine/q3moe_one.py:308-334, 352-377): the
    three-stage entry (expert sum -> RMS norm -> fp16) and its one-launch form, the fp16-cache attention inputs as one launch (QK-norm + NeoX
    rotary of 4 k heads into the cache beside v, and of 32 q heads), the own line's norm + rotary + append behind OP_OWN_ATTS, the
    attention output's fp16 copy, and SwiGLU over 8 experts x 768. T = 4: the verify module's pass."""
    from caminus_amd.engine.k3 import TapeOps
    rng = np.random.default_rng(1001 + T)
    D, hd, nh, nkv, KU, FF, rows = 2048, 128, 32, 4, 8, 768, 4096
    M = nkv * hd; eps = 1e-6; ts = float(np.float32(np.float32(1e6) ** np.float32(-2.0 / hd)))
    p0 = int(rng.integers(0, rows - T))
    err = dev(np.zeros(1, np.int32)); pos = dev(np.array([p0], np.int32))
    E = TapeOps(T=T, kv_error=err)
    nw = _gamma(rng, D); nwd = dev(nw)
    # experts' sum -> norm -> fp16 as three segments, token by token as the one-token statements have it
    x = outliers(rng, (T, D)); dexp = outliers(rng, (T, KU, D)); wts = rng.random((T, KU)).astype(np.float32)
    xs = x.copy(); hs = np.zeros((T, D), np.float32)
    for t in range(T):
        xt = dev(x[t]); ht = dev(np.zeros((1, D), np.float32)); h16t = torch.zeros(D, dtype=torch.float16, device=xt.device)
        one = TapeOps(T=1, kv_error=err)
        one.own_moe_sum(dev(dexp[t]), xt, slots=KU, w=dev(wts[t])); one.rms_mul(xt.view(1, D), nwd.view(1, D), ht, eps); one.own_f16(ht, h16t)
        xs[t] = O.own_moe_sum(dexp[t], wts[t], x[t], KU); hs[t] = O.rms_mul(xs[t].reshape(1, D), nw.reshape(1, D), eps)['y'][0]
        assert bits_equal(host(xt), xs[t]) and bits_equal(host(ht)[0], hs[t]) and bits_equal(host(h16t.view(torch.int16), np.uint16), O.own_f16(hs[t]))
    # the same as one segment (equal to the three to rounding: its own statements, the oracle's add_rms16)
    xd = dev(x); h = dev(np.zeros((T, D), np.float32)); h16 = torch.zeros((T, D), dtype=torch.float16, device=xd.device)
    E.own_add_rms16(xd, nwd, h, h16, eps, d=dev(dexp), slots=KU, w=dev(wts), tokens=T)
    ref = O.add_rms16(x, nw, eps, d=dexp, w=wts, S=KU)
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16.view(torch.int16), np.uint16), ref['h16'])
    assert close_fp32(ref['h'], hs)
    # the fp16-cache attention inputs in one launch
    q = outliers(rng, (T * nh, hd)); k = outliers(rng, (T * nkv, hd)); v = outliers(rng, (T, M)); qn = _gamma(rng, hd); kn = _gamma(rng, hd)
    qo = dev(np.zeros((T * nh, hd), np.float32)); ko = dev(np.zeros((T * nkv, hd), np.float32)); cache = dev(np.zeros((rows, 2 * M), np.uint16))
    E.qk_nr_kv(dev(q), hd, nh, dev(k), hd, dev(v), nkv, hd, dev(qn), dev(kn), pos, qo, cache, hd, ts, eps, ko=ko)
    wq_, wk_, cref, werr = O.qk_nr_kv(q, hd, nh, qn, k, hd, v, nkv, kn, hd, hd, ts, eps, p0, T, np.zeros((rows, 2 * M), np.uint16), False, ko=host(ko))
    assert close_fp32(host(qo), wq_) and close_fp32(host(ko), wk_) and werr == 0 and bits_equal(host(cache.view(torch.int16), np.uint16), cref)
    # the own line: norm + rotary + append of the token's q | k | v row at the device position
    par = qk_par(rng, theta_base=1e6); ldq = (nh + 2 * nkv) * hd
    qkv = outliers(rng, (T, ldq)); q16 = dev(np.zeros((T, nh, hd), np.uint16)); c16 = dev(np.zeros((rows, 2 * M), np.uint16))
    call('camx_op_own_qk_rope', ptr(dev(qkv)), I(ldq), I(nh), I(nkv), ptr(dev(par)), ptr(pos), ptr(q16), ptr(c16), I(rows), ptr(err), I(T), I(0), I(0))
    rq, rc, _ = O.qk_rope(qkv, nh, nkv, par, T, pos0=p0, rows=rows)
    gc = host(c16, np.uint16)
    assert close_16(host(q16, np.uint16), rq, 'f16') and close_16(gc[p0:p0 + T, :M], rc[p0:p0 + T, :M], 'f16') and bits_equal(gc[p0:p0 + T, M:], rc[p0:p0 + T, M:])
    # the attention output's fp16 copy and the experts' activation
    att = outliers(rng, (T * nh * hd,)); a16 = torch.zeros(T * nh * hd, dtype=torch.float16, device=xd.device)
    E.own_f16(dev(att), a16)
    assert bits_equal(host(a16.view(torch.int16), np.uint16), O.own_f16(att))
    g = outliers(rng, (T * KU * FF,)); u = outliers(rng, (T * KU * FF,)); y16 = torch.zeros(T * KU * FF, dtype=torch.float16, device=xd.device)
    E.own_swiglu16(dev(g), dev(u), y16)
    assert close_16(host(y16.view(torch.int16), np.uint16), O.swiglu16(g, u), 'f16')
    assert int(host(err)[0]) == 0


@pytest.mark.parametrize('fmt', [0, 1])
def test_config2_embedding_gather_full_table(fmt):
    """151936 x 2048 table, Q4_K (175 MB) or Q8_0 (331 MB): 256 uniformly drawn ids to fp32 and bf16, then add + RMSNorm +
    q8_1 of the gathered rows, every output bit-exact"""
    rng = np.random.default_rng(1002)
    V, N, n = 151936, 2048, 256
    table = (q4k_table if fmt == 0 else q80_table)(rng, V, N)
    toks = rng.integers(0, V, n).astype(np.int32)
    nw = _gamma(rng, N); d = outliers(rng, (n, 1, N))
    orc = O.emb_q4k if fmt == 0 else O.emb_q8_0
    ref_x, ref_bf = orc(table, V, toks, N)
    Wd, td = dev(table), dev(toks)
    x = dev(np.zeros((n, N), np.float32)); xbf = dev(np.zeros((n, N), np.uint16))
    call('camx_emb_gather', ptr(Wd), L64(table.shape[1]), I(V), ptr(td), ptr(x), ptr(xbf), I(N), I(n), I(fmt))
    assert bits_equal(host(x), ref_x) and bits_equal(host(xbf, np.uint16), ref_bf)
    # the independent numpy decoder on the same rows
    from oracle import np_dequant
    want = np.stack([np_dequant.dequant(table[t], 'Q4_K' if fmt == 0 else 'Q8_0', N) for t in toks[:16]])
    assert bits_equal(host(x)[:16], want)
    for addend in (None, d):
        ref = O.add_rms16(ref_x, nw, 1e-6, d=addend, S=0 if addend is None else 1, want_q8=True)
        xr = dev(np.zeros((n, N), np.float32)); q8 = dev(np.zeros((n, N // 32, 36), np.uint8)); h = dev(np.zeros((n, N), np.float32))
        call('camx_emb_gather_add_rms', ptr(Wd), L64(table.shape[1]), I(V), ptr(td), ptr(xr), NULL, ptr(dev(addend)) if addend is not None else NULL,
             ptr(dev(nw)), F(1e-6), ptr(h), NULL, ptr(q8), I(N), I(n), I(fmt))
        assert bits_equal(host(xr), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(q8), ref['q8'])


def test_config3_add_rms_full_chunk():
    """4096 x 5120, fp32 residual + bf16 addend -> fp32 residual + bf16 normed rows, bit-exact; the same rows in two launches
    of 1000 and 3096 tokens give the same bits (chunk geometry does not matter)"""
    rng = np.random.default_rng(1003)
    T, H = 4096, 5120
    x = outliers(rng, (T, H)); d = O.f2bf(outliers(rng, (T, H))); nw = _gamma(rng, H)
    ref = O.add_rms_bf16(x, d, nw, 1e-6)
    xd, dd, nwd = dev(x), dev(d), dev(nw); hbf = dev(np.zeros((T, H), np.uint16))
    call('camx_add_rms_bf16', ptr(xd), ptr(dd), ptr(nwd), F(1e-6), NULL, ptr(hbf), I(H), I(T))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(hbf, np.uint16), ref['hbf'])
    x2 = dev(x); h2 = dev(np.zeros((T, H), np.uint16))
    call('camx_add_rms_bf16', ptr(x2), ptr(dd), ptr(nwd), F(1e-6), NULL, ptr(h2), I(H), I(1000))
    call('camx_add_rms_bf16', ptr(x2[1000:]), ptr(dd[1000:]), ptr(nwd), F(1e-6), NULL, ptr(h2[1000:]), I(H), I(T - 1000))
    assert torch.equal(x2, xd) and torch.equal(h2, hbf)


def test_config3_qk_rope_yarn_full_chunk():
    """64 Q + 8 KV (+ 8 V) heads of 128 in bf16, YaRN factor 4 from 32768, theta 1e6, positions 0 .. 4095"""
    rng = np.random.default_rng(1003)
    T, nh, nkv = 4096, 64, 8
    par = qk_par(rng, theta_base=1e6, yarn_table=rope.yarn_table(128, 1e6, 4.0, 32768))
    ldq = (nh + 2 * nkv) * 128; M = nkv * 128
    qkv = O.f2bf(outliers(rng, (T, ldq)))
    q16 = dev(np.zeros((T, nh, 128), np.uint16)); c16 = dev(np.zeros((T, 2 * M), np.uint16))
    call('camx_qk_rope_bf16', ptr(dev(qkv)), I(ldq), I(nh), I(nkv), ptr(dev(par)), I(0), ptr(q16), ptr(c16), I(T), I(1))
    rq, rc, _ = O.qk_rope(O.bf2f(qkv), nh, nkv, par, T, pos0=0, yarn=True, rows=T)
    gq, gc = host(q16, np.uint16), host(c16, np.uint16)
    assert close_16(gq, rq, 'f16') and close_16(gc[:, :M], rc[:, :M], 'f16') and bits_equal(gc[:, M:], rc[:, M:])
    # position 0 is the identity rotation times mscale: norm preserved per pair up to mscale^2
    ms = float(par[322])
    k0 = O.h2f(gc[0, :M]).reshape(nkv, 128).astype(np.float64)
    xk = O.bf2f(qkv[0, nh * 128:(nh + nkv) * 128]).reshape(nkv, 128).astype(np.float64)
    want = xk / np.sqrt((xk * xk).mean(1, keepdims=True) + 1e-6) * par[128:256] * ms
    assert np.abs(k0 - want).max() <= 2.0 ** -10 * np.abs(want).max() + 1e-5


def test_config3_swiglu_mmq_full_chunk():
    """4096 x 17408 gate / up pair in bf16 -> q8_1 blocks in the MMQ layout (DS4): activation and blocks bit-equal to the
    oracle's; without the activation output the blocks are the same"""
    rng = np.random.default_rng(1003)
    T, Fh = 4096, 17408
    gu = O.f2bf(outliers(rng, (T, 2 * Fh)))
    gud = dev(gu)
    y = dev(np.zeros((O.k_pad(Fh) // 128, T, 144), np.uint8)); act = dev(np.zeros((T, Fh), np.uint16))
    call('camx_swiglu_mmq_q8_1', ptr(gud), L64(2 * Fh), L64(Fh), ptr(y), ptr(act), I(T), I(1))
    a = O.silu_mul_bf16(gu)
    assert bits_equal(host(act, np.uint16), a)
    assert bits_equal(host(y), O.mmq_q8_1(O.bf2f(a), Fh, T, 1))
    y2 = dev(np.zeros((O.k_pad(Fh) // 128, T, 144), np.uint8))
    call('camx_swiglu_mmq_q8_1', ptr(gud), L64(2 * Fh), L64(Fh), ptr(y2), NULL, I(T), I(1))
    assert torch.equal(y2, y)
    # q * d reconstructs the activation within half a quantization step, block by block (layout-independent invariant)
    blocks = host(y).reshape(-1, T, 144)
    dsc = blocks[:, :, :16].copy().view(np.float16).reshape(-1, T, 4, 2)[..., 0].astype(np.float32)       # [kb][t][group]
    q = blocks[:, :, 16:].view(np.int8).reshape(-1, T, 4, 32).astype(np.float32)
    recon = (q * dsc[..., None]).transpose(1, 0, 2, 3).reshape(T, -1)[:, :Fh]
    af = O.bf2f(a)
    step = np.repeat(dsc.transpose(1, 0, 2).reshape(T, -1), 32, axis=1)[:, :Fh]
    assert (np.abs(recon - af) <= 0.57 * step + 1e-30).all()            # d / 2, plus 127 codes x the half rounding of the stored d


def test_config4_hybrid_verify_batch():
    """16-token verify batch: 24 Q heads (stride 512: q | gate) and 4 KV heads of 256 with rotary over the first 64 dims
    (theta 1e7), sigmoid output gate, SiLU short conv of width 4 over 10240 channels, L2 norm of 32 (and 48) heads of 128;
    bf16 activations, positions uniform below 65536"""
    rng = np.random.default_rng(1004)
    T, D, nrot = 16, 256, 64
    ts = float(np.float32(np.float32(1e7) ** np.float32(-2.0 / nrot)))
    pos = rng.integers(0, 65536, T).astype(np.int32)
    w = _gamma(rng, D)
    for heads, stride in ((24, 512), (4, 256)):
        xb = O.f2bf(outliers(rng, (T * heads, stride)))
        out = dev(np.zeros((T * heads, D), np.uint16))
        call('camx_qk_nr_pos', ptr(dev(xb)), I(stride), I(heads), ptr(dev(w)), I(D), I(nrot), F(ts), F(1e-6), ptr(dev(pos)), ptr(out), I(T), I(1))
        ref = np.concatenate([O.qk_nr(O.bf2f(xb)[t * heads:(t + 1) * heads], stride, heads, w, D, nrot, ts, 1e-6, int(pos[t]), 1) for t in range(T)])
        got = host(out, np.uint16)
        assert close_16(got, O.f2bf(ref), 'bf16')
        assert bits_equal(got[:, nrot:], O.f2bf(ref)[:, nrot:])                 # the pass-through dims carry no transcendental
    a = O.f2bf(outliers(rng, (T * 24, D))); qg = O.f2bf(outliers(rng, (T * 24, 2 * D)))
    y = dev(np.zeros((T * 24, D), np.uint16))
    call('camx_gate_mul', ptr(dev(a)), ptr(dev(qg)), ptr(y), L64(a.size), I(D), I(2 * D), I(D), I(2))
    assert close_16(host(y, np.uint16), O.f2bf(O.gate_mul(O.bf2f(a), O.bf2f(qg), D, 2 * D, D)), 'bf16')
    C = 10240
    xc = O.f2bf(outliers(rng, (T, C))); wc = rng.standard_normal((C, 4)).astype(np.float32); st = rng.standard_normal((C, 3)).astype(np.float32)
    ry, rst = O.gdn_conv(O.bf2f(xc), wc, st)
    xcd, std = dev(xc), dev(st); yc = dev(np.zeros((T, C), np.uint16))
    call('camx_pf_gdn_conv', ptr(xcd), ptr(dev(wc)), ptr(std), ptr(yc), I(C), I(T), I(C), I(C), I(1))
    call('camx_pf_conv_state', ptr(xcd), ptr(std), I(C), I(T), I(C), I(1))
    assert close_16(host(yc, np.uint16), O.f2bf(ry), 'bf16') and bits_equal(host(std), rst)
    # the same 16 tokens as two passes of 5 and 11 (state carried between them) give the same outputs
    st2 = dev(st); y2 = dev(np.zeros((T, C), np.uint16))
    for lo, hi in ((0, 5), (5, 16)):
        call('camx_pf_gdn_conv', ptr(xcd[lo:]), ptr(dev(wc)), ptr(st2), ptr(y2[lo:]), I(C), I(hi - lo), I(C), I(C), I(1))
        call('camx_pf_conv_state', ptr(xcd[lo:]), ptr(st2), I(C), I(hi - lo), I(C), I(1))
    assert torch.equal(y2, yc) and torch.equal(st2, std)
    for heads in (32, 48):
        xl = O.f2bf(outliers(rng, (T, heads * 128)))
        yl = dev(np.zeros((T * heads, 128), np.uint16))
        call('camx_pf_gdn_l2', ptr(dev(xl)), ptr(yl), I(heads), I(128), I(heads * 128), F(np.float32(1e-6 / 128)), I(T), I(1))
        assert bits_equal(host(yl, np.uint16), O.f2bf(O.gdn_l2(O.bf2f(xl), T, heads, 128, 1e-6)))


@pytest.mark.parametrize('T', [1, 16])
def test_config4_decode_tape_row_ops_of_both_layer_kinds(T):
    """The dense line's decode / verify tape at config 4's shapes, fp32 as the tape runs it (python/caminus/engine/q35_dense.py:389-425), through the
    host mirror's TapeOps(q35=True) with the fused launches: per layer the add + norm of 5120-wide rows, then either the linear-attention
    row ops (gates | conv4 + SiLU with the lazy commit | L2 norm of 32 key heads; the gated norm of 48 value heads to fp16) or the
    full-attention ones (QK-norm + partial rotary of 4 k heads into the fp16 cache beside v, and of 24 q heads; the sigmoid gate to fp16),
    and the SwiGLU of the 17408-wide FFN. Two passes, the second committing part of the first."""
    from caminus_amd.engine.k3 import TapeOps
    rng = np.random.default_rng(1004 + T)
    D, CH, NK, NV, S, nh, nkv, hd, nrot, FF, rows = 5120, 10240, 16, 48, 128, 24, 4, 256, 64, 17408, 64
    M = nkv * hd; eps = 1e-6
    ts = float(np.float32(np.float32(1e7) ** np.float32(-2.0 / nrot)))
    err = dev(np.zeros(1, np.int32)); pos = dev(np.array([0], np.int32)); par = dev(np.zeros(4, np.int32))
    E = TapeOps(T=T, kv_error=err, q35=True); E.params = par
    nw = _gamma(rng, D); wc = rng.standard_normal((CH, 4)).astype(np.float32); st = rng.standard_normal((CH, 3)).astype(np.float32)
    dt = rng.standard_normal(NV).astype(np.float32); A = -np.abs(rng.standard_normal(NV)).astype(np.float32); gw = _gamma(rng, S)
    qn = _gamma(rng, hd); kn = _gamma(rng, hd)
    nwd, wcd, std, dtd, Ad, gwd, qnd, knd = (dev(a) for a in (nw, wc, st, dt, A, gw, qn, kn))
    xprev_ref = np.zeros((T, CH), np.float32); xpd = dev(xprev_ref); st_ref = st
    cache = dev(np.zeros((rows, 2 * M), np.uint16)); cache_ref = np.zeros((rows, 2 * M), np.uint16)
    mprev = 0
    for step, p0 in enumerate((7, 7 + T)):
        pos.fill_(p0); par.copy_(dev(np.array([0, mprev, 0, 0], np.int32)))
        # the layer's entry: x += blk, h = rms_norm(x) * w, h16 (rounded once)
        x = outliers(rng, (T, D)); blk = outliers(rng, (T, D))
        xd = dev(x); h = dev(np.zeros((T, D), np.float32)); h16 = torch.zeros((T, D), dtype=torch.float16, device=xd.device)
        E.own_add_rms16(xd, nwd, h, h16, eps, d=dev(blk), slots=1, tokens=T)
        ref = O.add_rms16_q35(x, nw, eps, d=blk)
        assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16.view(torch.int16), np.uint16), ref['h16'])
        # a linear-attention layer
        qkv = outliers(rng, (T, CH)); al = outliers(rng, (T, NV)) * np.float32(6); be = outliers(rng, (T, NV))
        conv = dev(np.zeros((T, CH), np.float32)); qk = dev(np.zeros((T * 2 * NK, S), np.float32)); gates = dev(np.zeros((T, 2 * NV), np.float32))
        E.gdn_conv_l2_gates(dev(qkv), wcd, std, conv, xpd, qk, 2 * NK, S, eps, dev(al), dev(be), dtd, Ad, gates)
        ry, st_ref, xprev_ref = O.op_gdn_conv(wc, st_ref, qkv, mprev, xprev_ref)
        got_y = host(conv)
        assert close_fp32(got_y, ry) and bits_equal(host(std), st_ref) and bits_equal(host(xpd), xprev_ref)
        assert bits_equal(host(qk), O.gdn_l2(got_y, T, 2 * NK, S, eps, ldx=CH)) and close_fp32(host(gates), O.gdn_gates(al, be, dt, A))
        o = outliers(rng, (T * NV, S)); z = outliers(rng, (T * NV, S)); fin16 = torch.zeros((T * NV, S), dtype=torch.float16, device=xd.device)
        E.gdn_norm16(dev(o), gwd, dev(z), fin16, NV, S, eps)
        assert close_16(host(fin16.view(torch.int16), np.uint16), O.gdn_norm(o, gw, z, eps, silu=True)[1], 'f16')
        # a full-attention layer
        kr = outliers(rng, (T, M)); vr = outliers(rng, (T, M)); qf = outliers(rng, (T * nh, 2 * hd))
        qo = dev(np.zeros((T * nh, hd), np.float32)); ko = dev(np.zeros((T * nkv, hd), np.float32))
        E.qk_nr_kv(dev(qf), 2 * hd, nh, dev(kr), hd, dev(vr), nkv, hd, qnd, knd, pos, qo, cache, nrot, ts, eps, ko=ko)
        wq_, wk_, cache_ref, werr = O.qk_nr_kv(qf, 2 * hd, nh, qn, kr.reshape(T * nkv, hd), hd, vr, nkv, kn, hd, nrot, ts, eps, p0, T, cache_ref, False, ko=host(ko))
        assert close_fp32(host(qo), wq_) and close_fp32(host(ko), wk_) and werr == 0 and bits_equal(host(cache.view(torch.int16), np.uint16), cache_ref)
        att = outliers(rng, (T * nh, hd)); gat16 = torch.zeros((T * nh, hd), dtype=torch.float16, device=xd.device)
        E.gate_mul16(dev(att), dev(qf), 2 * hd, hd, gat16, hd)
        assert close_16(host(gat16.view(torch.int16), np.uint16), O.gate_mul(att, qf, hd, 2 * hd, hd, f16=True), 'f16')
        # the FFN's activation
        g = outliers(rng, (T * FF,)); u = outliers(rng, (T * FF,)); y16 = torch.zeros(T * FF, dtype=torch.float16, device=xd.device)
        E.own_swiglu16(dev(g), dev(u), y16)
        assert close_16(host(y16.view(torch.int16), np.uint16), O.swiglu16(g, u), 'f16')
        mprev = int(rng.integers(0, T + 1))
    torch.cuda.synchronize()
    assert int(host(err)[0]) == 0 and E.n == 2 * 6


def test_q3m_prefill_chunk_through_the_host_wrappers():
    """A 4096-token prefill chunk of the qwen3moe own prefill (python/caminus/prefill/q3m.py's layer loop: the call stack of the 2048-wide
    configurations) through the host mirror's wrapper classes: Q4_K embedding rows of a 32768-row table, the layer entry with the 8 weighted
    expert rows added, QK-norm + rotary into the fp16 cache, the router's scatter of the normed rows into the MMQ layout, SwiGLU of 8 x 768 per
    token. The first and last 8 tokens against the oracle; the scatter block for block."""
    from caminus_amd.prefill import mmq, q3m_ops
    rng = np.random.default_rng(1033)
    n, N, nh, nkv, KU, FF, vocab, rows, p0 = 4096, 2048, 32, 4, 8, 768, 32768, 8192, 1000
    M = nkv * 128; eps = 1e-6; devname = 'cuda:0'
    Oq = q3m_ops.Ops(devname); Q = mmq.MMQ(devname)
    ends = np.r_[0:8, n - 8:n]
    f16 = lambda t: host(t.view(torch.int16), np.uint16)
    tab = q4k_table(rng, vocab, N); toks = rng.integers(-3, vocab + 3, n).astype(np.int32)
    x = dev(np.zeros((n, N), np.float32))
    Oq.emb(dev(tab), tab.shape[1], vocab, dev(toks), x, n, N)
    assert bits_equal(host(x)[ends], O.emb_q4k(tab, vocab, toks[ends], N)[0])
    x0 = host(x).copy()
    dexp = outliers(rng, (n, KU, N)); wts = rng.random((n, KU)).astype(np.float32); nw = _gamma(rng, N)
    h = dev(np.zeros((n, N), np.float32)); h16 = torch.zeros((n, N), dtype=torch.float16, device=devname)
    Oq.add_rms16(x, dev(nw), eps, h16, n, N, d=dev(dexp), w=dev(wts), S=KU, h=h)
    ref = O.add_rms16(x0[ends], nw, eps, d=dexp[ends], w=wts[ends], S=KU)
    assert bits_equal(host(x)[ends], ref['x']) and bits_equal(host(h)[ends], ref['h']) and bits_equal(f16(h16)[ends], ref['h16'])
    par = qk_par(rng, theta_base=1e6); ldq = (nh + 2 * nkv) * 128
    qkv = outliers(rng, (n, ldq)); q16 = torch.zeros((n, nh, 128), dtype=torch.float16, device=devname); cache = torch.zeros((rows, 2 * M), dtype=torch.float16, device=devname)
    Oq.qk_rope(dev(qkv), ldq, nh, nkv, dev(par), p0, q16, cache, n)
    rq, rc, _ = O.qk_rope(qkv[ends[:8]], nh, nkv, par, 8, pos0=p0, rows=rows)
    gc = f16(cache)
    assert close_16(f16(q16).reshape(n, -1)[:8], rq.reshape(8, -1), 'f16') and close_16(gc[p0:p0 + 8, :M], rc[p0:p0 + 8, :M], 'f16') and bits_equal(gc[p0:p0 + 8, M:], rc[p0:p0 + 8, M:])
    assert not gc[:p0].any() and not gc[p0 + n:].any() and gc[p0 + n - 1].any()
    # the router's compact columns: grouped by expert, a group's tokens in order
    ex = np.argsort(-rng.random((n, 128)), axis=1)[:, :KU].reshape(-1)
    order = np.argsort(ex, kind='stable'); ids_inv = np.empty(n * KU, np.int32); ids_inv[order] = np.arange(n * KU, dtype=np.int32)
    y = torch.zeros(mmq.y_bytes(N, n * KU), dtype=torch.uint8, device=devname)
    Q.quantize_scatter(h, N, n, dev(ids_inv), KU, y, 1)
    assert bits_equal(host(y)[:(N // 128) * n * KU * 144].reshape(N // 128, n * KU, 144), O.mmq_q8_1_scatter(host(h), N, n, ids_inv, KU, 1))
    g = outliers(rng, (n * KU * FF,)); u = outliers(rng, (n * KU * FF,)); a16 = torch.zeros(n * KU * FF, dtype=torch.float16, device=devname)
    Oq.swiglu(dev(g), dev(u), a16, n * KU * FF)
    e = np.r_[0:8 * KU * FF, (n - 8) * KU * FF:n * KU * FF]
    assert close_16(f16(a16)[e], O.swiglu16(g[e], u[e]), 'f16')


def test_coder_glue_chunk_through_the_host_wrappers():
    """A 2048-token chunk of the hyper-connection model's prefill glue at the shape the reference publishes its times on (4 streams of
    2560: SURVEY's perf table), through the host mirror's Glue wrappers in the layer's order (python/caminus/prefill/glue.py): the block's
    output into the four residual streams + their norms (fp32, bf16 and the row scale), the gated mean of the streams from the norm and
    again from the residual with the scale, the norm alone with a per-stream gamma, the bf16 operand copies. First and last 8 tokens."""
    from caminus_amd.prefill import glue
    rng = np.random.default_rng(1055)
    T, HC, D, eps = 2048, 4, 2560, 1e-6
    G = glue.Glue('cuda:0')
    ends = np.r_[0:8, T - 8:T]
    b = outliers(rng, (T, D)); inj = outliers(rng, (T, HC)); res = outliers(rng, (T, HC, D)); w = (1 + 0.1 * rng.standard_normal((HC, D))).astype(np.float32)
    resd = dev(res); xn = dev(np.zeros((T, HC, D), np.float32)); xnbf = torch.zeros((T, HC, D), dtype=torch.bfloat16, device='cuda:0'); scl = dev(np.zeros(T * HC, np.float32))
    G.hc_post_rms(dev(b), dev(inj), resd, dev(w), T, HC, eps, xn=xn, xnbf=xnbf, scale=scl)
    ref = O.hc_post_rms(b[ends], inj[ends], res[ends], w, eps)
    bfb = lambda t: host(t.view(torch.int16), np.uint16)
    assert close_fp32(host(resd)[ends], ref['res']) and close_fp32(host(xn)[ends], ref['xn']) and close_16(bfb(xnbf)[ends], ref['xnbf'], 'bf16')
    assert close_fp32(host(scl).reshape(T, HC)[ends], ref['scale'].reshape(len(ends), HC))
    gate = outliers(rng, (T, HC, D)); out1 = dev(np.zeros((T, D), np.float32)); out2 = dev(np.zeros((T, D), np.float32))
    G.hc_mean(xn, dev(gate), out1, T, HC)
    G.hc_mean(resd, dev(gate), out2, T, HC, scale=scl, w=dev(w))
    gxn = host(xn)
    assert close_fp32(host(out1)[ends], O.hc_mean(gxn[ends], gate[ends])) and close_fp32(host(out2)[ends], host(out1)[ends])
    y = dev(np.zeros((T * HC, D), np.float32)); ybf = torch.zeros((T * HC, D), dtype=torch.bfloat16, device='cuda:0')
    G.rms_mul(resd.view(T * HC, D), dev(w), y, T * HC, eps, ybf=ybf)
    gres = host(resd).reshape(T * HC, D); r2 = np.r_[0:8 * HC, (T - 8) * HC:T * HC]
    rr = O.rms_mul(gres[r2], w, eps)
    assert bits_equal(host(y)[r2], rr['y']) and bits_equal(bfb(ybf)[r2], rr['ybf'])
    xb = torch.zeros((T, D), dtype=torch.bfloat16, device='cuda:0'); sb = torch.zeros((T, D), dtype=torch.bfloat16, device='cuda:0')
    G.to_bf16(out1, xb, T, D); G.silu_bf16(out1, sb, T, D, 0.5)
    g1 = host(out1)
    assert bits_equal(bfb(xb)[ends], O.to_bf16_rows(g1[ends], len(ends), len(ends), D)) and close_16(bfb(sb)[ends], O.to_bf16_rows(g1[ends], len(ends), len(ends), D, rs=0.5, silu=True), 'bf16')


def test_config4_prefill_chunk_through_the_host_wrappers():
    """A 2048-token prefill chunk of the dense line's own prefill (python/caminus/prefill/q35own.py:352-389), fp32 as it runs there, through
    the host mirror's wrapper classes with the reference's call sequence: add + norm of 5120-wide rows; gates, conv4 + SiLU with its carried
    state, L2 norm of the 32 key heads, gated norm of the 48 value heads; QK-norm + partial rotary of the 4 k heads, the fp16 append, the
    24 q heads, the sigmoid gate. The first and last 8 tokens of every output against the oracle."""
    from caminus_amd.prefill import attn, gdn, glue, q35_ops
    rng = np.random.default_rng(1044)
    n, D, CH, NK, NV, S, nh, nkv, hd, nrot, p0, rows = 2048, 5120, 10240, 16, 48, 128, 24, 4, 256, 64, 100, 4096
    M = nkv * hd; eps = 1e-6; ts = float(np.float32(np.float32(1e7) ** np.float32(-2.0 / nrot)))
    devname = 'cuda:0'
    Oq = q35_ops.Ops(devname); A = attn.Attn(devname); Gd = gdn.Gdn(devname, 'prefill_gdn_q35'); Gl = glue.Glue(devname)
    ends = np.r_[0:8, n - 8:n]
    zeros16 = lambda *sh: torch.zeros(sh, dtype=torch.float16, device=devname)
    f16 = lambda t: host(t.view(torch.int16), np.uint16)
    x = outliers(rng, (n, D)); blk = outliers(rng, (n, D)); nw = _gamma(rng, D)
    xd = dev(x); h = dev(np.zeros((n, D), np.float32)); h16 = zeros16(n, D)
    Oq.add_rms16(xd, dev(nw), eps, h16, n, D, d=dev(blk), h=h)
    ref = O.add_rms16_q35(x[ends], nw, eps, d=blk[ends])
    assert bits_equal(host(xd)[ends], ref['x']) and bits_equal(host(h)[ends], ref['h']) and bits_equal(f16(h16)[ends], ref['h16'])
    al = outliers(rng, (n, NV)) * np.float32(6); be = outliers(rng, (n, NV)); dt = rng.standard_normal(NV).astype(np.float32); Aa = -np.abs(rng.standard_normal(NV)).astype(np.float32)
    gt = dev(np.zeros((n, 2 * NV), np.float32))
    Gd.gates(dev(al), dev(be), dev(dt), dev(Aa), gt, n, NV)
    assert close_fp32(host(gt)[ends], O.gdn_gates(al[ends], be[ends], dt, Aa))
    qkv = outliers(rng, (n, CH)); wc = rng.standard_normal((CH, 4)).astype(np.float32); st = rng.standard_normal((CH, 3)).astype(np.float32)
    conv = dev(np.zeros((n, CH), np.float32)); std = dev(st); qk = dev(np.zeros((n * 2 * NK, S), np.float32))
    Gl.gdn_conv(dev(qkv), dev(wc), std, conv, CH, n)
    Gd.l2(conv, qk, n, 2 * NK, eps, ldx=CH)
    ry, rst = O.gdn_conv(qkv, wc, st)
    gy = host(conv)
    assert close_fp32(gy[ends], ry[ends]) and bits_equal(host(std), rst)
    assert bits_equal(host(qk).reshape(n, -1)[ends], O.gdn_l2(gy[ends], len(ends), 2 * NK, S, eps, ldx=CH).reshape(len(ends), -1))
    o = outliers(rng, (n * NV, S)); z = outliers(rng, (n * NV, S)); gw = _gamma(rng, S); fin16 = zeros16(n * NV, S)
    Oq.gdn_norm16(dev(o), dev(gw), dev(z), fin16, n, NV, S, eps)
    rows_ = np.r_[0:8 * NV, (n - 8) * NV:n * NV]
    assert close_16(f16(fin16)[rows_], O.gdn_norm(o[rows_], gw, z[rows_], eps, silu=True)[1], 'f16')
    kr = outliers(rng, (n, M)); vr = outliers(rng, (n, M)); qf = outliers(rng, (n * nh, 2 * hd)); kn = _gamma(rng, hd); qn = _gamma(rng, hd)
    ko = dev(np.zeros((n * nkv, hd), np.float32)); qo = dev(np.zeros((n * nh, hd), np.float32))
    cache = zeros16(rows, 2 * M); err = dev(np.zeros(1, np.int32))
    A.qk_nr(dev(kr), hd, nkv, hd, dev(kn), nrot, ts, eps, p0, ko, n)
    Oq.kv_append16(ko, M, dev(vr), M, cache, M, p0, n, rows, err)
    A.qk_nr(dev(qf), 2 * hd, nh, hd, dev(qn), nrot, ts, eps, p0, qo, n)
    gko = host(ko).reshape(n, M)
    for t in (0, 5, n - 1):
        assert close_fp32(gko[t].reshape(nkv, hd), O.qk_nr(kr[t].reshape(nkv, hd), hd, nkv, kn, hd, nrot, ts, eps, p0 + t, 1))
        assert close_fp32(host(qo)[t * nh:(t + 1) * nh], O.qk_nr(qf[t * nh:(t + 1) * nh], 2 * hd, nh, qn, hd, nrot, ts, eps, p0 + t, 1))
    want, werr = O.kv_append16(gko, vr, M, np.zeros((rows, 2 * M), np.uint16), p0)
    assert werr == 0 and int(host(err)[0]) == 0 and bits_equal(f16(cache), want)
    att = outliers(rng, (n * nh, hd)); x16 = zeros16(n * nh, hd)
    Oq.gate_mul16(dev(att), dev(qf), x16, n * nh * hd, hd, 2 * hd, hd)
    r2 = np.r_[0:8 * nh, (n - 8) * nh:n * nh]
    assert close_16(f16(x16)[r2], O.gate_mul(att, qf, hd, 2 * hd, hd, f16=True)[r2], 'f16')


def test_config5_batched_decode_paged_q8():
    """256 sequences at the Qwen3-30B-A3B shape: add + RMSNorm, then QK-norm -> rotary at each sequence's own position below
    131072 -> fp16 -> Hadamard-128 -> Q8 blocks into a paged cache (page 256 tokens, random table over 65536 pages, 18 GB).
    Row bytes equal the unpaged kernel's rows, which equal the oracle codec applied to the fp16 rows the F16 form wrote; restoring
    the fill in the written rows leaves the whole cache uniform: nothing else was touched."""
    rng = np.random.default_rng(1005)
    S, N, nh, nkv, page, n_pages = 256, 2048, 32, 4, 256, 65536
    x = outliers(rng, (S, N)); d = outliers(rng, (S, 1, N)); nw = _gamma(rng, N)
    ref = O.add_rms16(x, nw, 1e-6, d=d, S=1)
    xd = dev(x); h = dev(np.zeros((S, N), np.float32)); h16 = dev(np.zeros((S, N), np.uint16))
    call('camx_q3p_add_rms16', ptr(xd), ptr(dev(d)), NULL, I(1), ptr(dev(nw)), F(1e-6), ptr(h), ptr(h16), I(N), I(S))
    assert bits_equal(host(xd), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16, np.uint16), ref['h16'])

    par = qk_par(rng, theta_base=1e6)
    M = nkv * 128; rb = 2 * (M // 32) * 34; ldq = (nh + 2 * nkv) * 128
    qkv = outliers(rng, (S, ldq))
    pos = rng.choice(131072, S, replace=False).astype(np.int32)          # distinct: the unpaged comparison run below shares one flat cache
    table = rng.integers(0, n_pages, (S, 512)).astype(np.int32)
    table[np.arange(S), pos // page] = rng.permutation(n_pages)[:S]                # the pages this batch writes are distinct
    qd, pd, posd, td = dev(qkv), dev(par), dev(pos), dev(table)
    cache = torch.full((n_pages * page * rb,), 0xa5, dtype=torch.uint8, device='cuda:0')
    err = dev(np.zeros(1, np.int32)); q16 = dev(np.zeros((S, nh, 128), np.uint16))
    call('camx_qk_rope_paged', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(q16), ptr(cache), ptr(err), ptr(td), I(512), I(page),
         I(n_pages), I(S), I(0), I(1))
    assert int(host(err)[0]) == 0
    rowid = table[np.arange(S), pos // page].astype(np.int64) * page + pos % page
    rows = host(cache.view(-1, rb)[torch.from_numpy(rowid).to('cuda:0')])
    # everything else still holds the fill: put the fill back into the written rows and the whole 18 GB must be uniform
    assert not (rows == 0xa5).all(axis=1).any()
    cache.view(-1, rb)[torch.from_numpy(rowid).to('cuda:0')] = 0xa5
    fill_word = int(np.frombuffer(bytes([0xa5] * 8), np.int64)[0])
    assert bool((cache.view(torch.int64) == fill_word).all())
    del cache
    # the unpaged F16 form at the same positions: the stage boundary the Q8 bytes are defined from
    c16 = dev(np.zeros((131072, 2 * M), np.uint16)); q16f = dev(np.zeros((S, nh, 128), np.uint16)); e2 = dev(np.zeros(1, np.int32))
    call('camx_qk_rope_paged', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(q16f), ptr(c16), ptr(e2), NULL, I(0), I(0), I(131072), I(S), I(0), I(0))
    rows16 = host(c16, np.uint16)[pos]
    rq, rc, _ = O.qk_rope(qkv, nh, nkv, par, S, pos=pos, rows=131072)
    assert close_16(host(q16f, np.uint16), rq, 'f16') and close_16(rows16[:, :M], rc[pos][:, :M], 'f16') and bits_equal(rows16[:, M:], rc[pos][:, M:])
    k16 = O.h2f(rows16[:, :M]).reshape(S * nkv, 128); v16 = O.h2f(rows16[:, M:]).reshape(-1, 32)
    kb, ok1 = O.kv_q8_encode(O.hadamard128(k16).reshape(-1, 32)); vb, ok2 = O.kv_q8_encode(v16)
    assert ok1.all() and ok2.all()
    assert bits_equal(rows, np.concatenate([kb.reshape(S, -1), vb.reshape(S, -1)], axis=1))
    assert bits_equal(host(q16, np.uint16), O.f2h(O.hadamard128(O.h2f(host(q16f, np.uint16)).reshape(-1, 128))).reshape(S, nh, 128))
