"""The reference's own entry points on the GPU: every kernel is launched the way the reference launches it,
`Module(name).<symbol>(grid, block, *args)` with the reference's module names, symbol names, launch geometry and argument
lists (python/caminus/device/hip.py:90-99; runtime/s1.cpp:97-106; python/caminus/train/actq.py:24-33;
python/caminus/device/kv_codec.py:79-83; python/caminus/prefill/q3m_ops.py:86-139; python/caminus/prefill/mmq.py:245-276),
or through the wrapper classes of the same files (Q8KVCodec, q3m Ops, MMQ), and the bytes are compared with the oracle.
A wrong trailing argument in one of the launcher's adapters fails here and nowhere else."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import bits_equal, close_16, close_fp32, dev, host, outliers

pytestmark = pytest.mark.gpu
f32 = np.float32
I, F, L, L64 = C.c_int, C.c_float, C.c_long, C.c_int64
NULL = C.c_void_p(None)
DEV = 'cuda:0'


def sync():
    torch.cuda.synchronize()


def qk_par(rng, base=1e6, eps=1e-6, yarn=False):
    from caminus_amd import rope
    qn = (1 + 0.1 * rng.standard_normal(128)).astype(f32); kn = (1 + 0.1 * rng.standard_normal(128)).astype(f32)
    ts = f32(f32(base) ** f32(-2.0 / 128))
    par = np.concatenate([qn, kn, np.array([ts, eps], f32)])
    if yarn: par = np.concatenate([par, rope.yarn_table(128, base, 4.0, 32768)])
    return par.astype(f32)


def test_module_core_with_the_s1_runtime_launch_tuples():
    from caminus_amd.device import hip
    m = hip.Module('core')
    rng = np.random.default_rng(31)
    T, D, V = 7, 896, 40
    emb = rng.standard_normal((V, D)).astype(f32); tok = rng.integers(0, V, T).astype(np.int32)
    out = dev(np.zeros((T, D), f32))
    m.embedding_f32((T,), (256,), dev(tok), dev(emb), out, I(D))
    x = outliers(rng, (T, D)); w = (1 + 0.1 * rng.standard_normal(D)).astype(f32)
    nrm = dev(np.zeros((T, D), f32))
    m.rmsnorm_f32((T,), (256,), dev(x), dev(w), nrm, I(D), F(1e-6))
    H = 448
    gu = O.f2bf(outliers(rng, (T, 2 * H))); act = dev(np.zeros((T, H), np.uint16)); n = T * H
    m.silu_mul_bf16(((n + 255) // 256,), (256,), dev(gu), act, I(H), L64(n))
    mm = O.f2bf(outliers(rng, (T, D))); yy = O.f2bf(outliers(rng, (T, D))); r3 = dev(np.zeros((T, D), f32)); n = T * D
    m.residual3(((n + 255) // 256,), (256,), dev(x), dev(mm), dev(yy), r3, L64(n))
    cb = dev(np.zeros((T, D), np.uint16))
    m.cast_bf16(((n + 255) // 256,), (256,), dev(x), cb, L64(n))
    dst = rng.integers(0, 65536, (T, 64)).astype(np.uint16); dd = dev(dst)
    m.copy_cols_bf16(((T * 40 + 255) // 256,), (256,), dev(mm), I(D), I(5), dd, I(64), I(3), I(40), L64(T))
    sync()
    assert bits_equal(host(out), O.embedding_f32(tok, emb)) and bits_equal(host(nrm), O.rmsnorm_f32(x, w, 1e-6))
    assert bits_equal(host(act, np.uint16), O.silu_mul_bf16(gu)) and bits_equal(host(r3), O.residual3(x, mm, yy))
    assert bits_equal(host(cb, np.uint16), O.f2bf(x)) and bits_equal(host(dd, np.uint16), O.copy_cols_bf16(mm, 5, dst, 3, 40))
    assert 'core' in hip.LOADED
    with pytest.raises(AttributeError):
        m.no_such_kernel
    with pytest.raises(FileNotFoundError):
        hip.Module('no_such_module')


def test_module_fuse_and_actq_symbols():
    from caminus_amd.device import hip
    rng = np.random.default_rng(32)
    T, D = 9, 896
    x = outliers(rng, (T, D)); m_ = O.f2bf(outliers(rng, (T, D))); mlp = O.f2bf(outliers(rng, (T, D)))
    ys = O.f2bf(outliers(rng, (4, D))); pos = np.array([-1, 0, 3, -1, 2, 1, -1, -1, 0], np.int32)
    o = dev(np.zeros((T, D), f32)); n4 = T * D // 4
    hip.Module('fuse').residual_slices_fwd(((n4 + 255) // 256,), (256,), dev(x), dev(m_), dev(mlp), dev(ys), dev(pos), o, I(D), L(n4))
    M, K = 5, 256
    xa = outliers(rng, (M, K)); y = dev(np.zeros((M, K), np.uint16)); s = dev(np.zeros(M, f32)); c = dev(np.zeros((M, K // 2), np.uint8))
    am = hip.Module('actq')
    am.actq_fwd_codes_f32((M,), (256,), dev(xa), y, s, c, I(K), F(0.9), I(7))
    y2 = dev(np.zeros((M, K), np.uint16))
    am.actq_fwd_bf16((M,), (256,), dev(O.f2bf(xa)), y2, NULL, I(K), F(0.9), I(7))
    sync()
    assert bits_equal(host(o), O.residual_slices_fwd(x, m_, mlp, ys, pos))
    ry, rs, rc = O.actq_fwd(xa, clip=0.9, qmax=7)
    assert bits_equal(host(y, np.uint16), ry) and bits_equal(host(s), rs) and bits_equal(host(c), rc)
    assert bits_equal(host(y2, np.uint16), O.actq_fwd(O.f2bf(xa), clip=0.9, qmax=7, bf16=True)[0])


def test_module_k3_gguf_quantizer_and_silu():
    from caminus_amd.device import hip
    rng = np.random.default_rng(33)
    for name in ('k3_gguf', 'k3_gguf_swiglu'):
        m = hip.Module(name)
        n = 2048 + 37
        x = outliers(rng, n); y = dev(np.zeros(((n + 31) // 32) * 36, np.uint8))
        m.gg_quantize_q8_1(((n + 255) // 256,), (256,), dev(x), y, I(n))
        g = outliers(rng, n); u = outliers(rng, n); h = dev(np.zeros(n, f32))
        m.gg_silu_mul(((n + 255) // 256,), (256,), dev(g), dev(u), h, I(n))
        sync()
        assert bits_equal(host(y), O.q8_1(x).reshape(-1)) and close_fp32(host(h), O.silu_mul_f32(g, u))
        with pytest.raises(ValueError):
            m.gg_quantize_q8_1((1,), (256,), dev(x), y, I(n))               # a grid that does not cover n


def test_module_kv_codec_and_q8kvcodec_append_check_read():
    from caminus_amd.device import hip
    from caminus_amd.device.kv_codec import Q8KVCodec
    rng = np.random.default_rng(34)
    M, T, rows, pos0 = 512, 11, 20, 4
    ldk, ldv = M + 32, M
    k = outliers(rng, (T, ldk)); v = outliers(rng, (T, ldv))
    rb = 2 * (M // 32) * 34
    fill = np.full(rows * rb, 0xa5, np.uint8)
    want, werr = O.kv_q8_append(k, ldk, v, ldv, M, fill, pos0, T, rows=rows)
    assert werr == 0
    # the launcher tuple of the reference wrapper: ((T,), (256,), k, ldk, v, ldv, M, cache, pos0, rows, err)
    cd = dev(fill); err = dev(np.zeros(1, np.int32))
    hip.Module('kv_codec').own_kv_q8_append((T,), (256,), dev(k), I(ldk), dev(v), I(ldv), I(M), cd, I(pos0), I(rows), err)
    sync()
    assert bits_equal(host(cd), want) and int(host(err)[0]) == 0
    # the wrapper class: append -> check -> read (fp32 and fp16), every refusal before the first launch
    codec = Q8KVCodec(DEV)
    cd = dev(fill); err = dev(np.zeros(1, np.int32)); kd, vd = dev(k), dev(v)
    codec.append(kd, ldk, vd, ldv, M, cd, pos0, T, err, rows=rows)
    codec.check(err)
    assert bits_equal(host(cd), want)
    rk, rv, _ = O.kv_q8_read(want.reshape(rows, rb), M, T, pos0=pos0, rows=rows)
    ko = dev(np.zeros((T, M), f32)); vo = dev(np.zeros((T, M), f32))
    codec.read(cd, M, ko, M, vo, M, pos0, T, err, rows=rows)
    codec.check(err)
    assert bits_equal(host(ko), rk) and bits_equal(host(vo), rv)
    k16 = torch.zeros((T, M), dtype=torch.float16, device=DEV); v16 = torch.zeros((T, M), dtype=torch.float16, device=DEV)
    codec.read(cd, M, k16, M, v16, M, pos0, T, err, rows=rows)
    codec.check(err)
    hk, hv, _ = O.kv_q8_read(want.reshape(rows, rb), M, T, pos0=pos0, rows=rows, f16=True)
    assert bits_equal(host(k16.view(torch.int16), np.uint16), hk) and bits_equal(host(v16.view(torch.int16), np.uint16), hv)
    ids = np.array([5, 4, 9, 14, 6], np.int32); ko2 = dev(np.zeros((5, M), f32)); vo2 = dev(np.zeros((5, M), f32))
    codec.read(cd, M, ko2, M, vo2, M, 0, 5, err, rows=rows, row_ids=dev(ids))
    codec.check(err)
    assert bits_equal(host(ko2), O.kv_q8_read(want.reshape(rows, rb), M, 5, row_ids=ids, rows=rows)[0])
    with pytest.raises(ValueError):
        codec.read(cd, M, k16, M + 2, v16, M, pos0, 2, err, rows=rows)      # fp16 rows: the stride must keep 8-byte alignment
    with pytest.raises(IndexError):
        codec.append(kd, ldk, vd, ldv, M, cd, rows - 3, T, err, rows=rows)  # span before any launch
    # a refused block: the error word carries bit 2, check() raises, the block keeps its bytes, its neighbours are written
    kb = k.copy(); kb[2, 40] = np.inf
    cd2 = dev(fill); err2 = dev(np.zeros(1, np.int32))
    codec.append(dev(kb), ldk, vd, ldv, M, cd2, pos0, T, err2, rows=rows)
    with pytest.raises(RuntimeError, match='numerical'):
        codec.check(err2)
    want2, werr2 = O.kv_q8_append(kb, ldk, v, ldv, M, fill, pos0, T, rows=rows)
    assert werr2 == 2 and bits_equal(host(cd2), want2)


@pytest.mark.parametrize('q8,yarn', [(False, False), (True, False), (False, True), (True, True)])
def test_q3m_ops_emb_add_rms16_swiglu_qk_rope(q8, yarn):
    """q3m_ops.Ops as the prefill driver uses it (python/caminus/prefill/q3m_ops.py:86-139): the four q3m_prefill module variants"""
    from caminus_amd.device import hip
    from caminus_amd.prefill.q3m_ops import Ops
    rng = np.random.default_rng(35 + 2 * int(q8) + int(yarn))
    ops = Ops(DEV, q8=q8, yarn=yarn)
    n, N, vocab = 6, 2048, 50
    rb = N // 256 * 144
    W = rng.integers(0, 256, (vocab, rb), dtype=np.uint8)
    sc = rng.uniform(1e-3, 1e-2, (vocab, rb // 144, 2)).astype(np.float16)
    W.reshape(vocab, rb // 144, 144)[:, :, :4] = sc.view(np.uint8).reshape(vocab, rb // 144, 4)
    toks = rng.integers(-2, vocab + 2, n).astype(np.int32)                # ids outside the vocabulary are clamped
    x = dev(np.zeros((n, N), f32))
    ops.emb(dev(W), rb, vocab, dev(toks), x, n, N)
    sync()
    ref_x, _ = O.emb_q4k(W, vocab, toks, N)
    assert bits_equal(host(x), ref_x)
    S = 3
    d = outliers(rng, (n, S, N)); w = rng.standard_normal((n, S)).astype(f32); nw = (1 + 0.1 * rng.standard_normal(N)).astype(f32)
    ref = O.add_rms16(ref_x.copy(), nw, 1e-6, d=d, w=w, S=S)
    h16 = dev(np.zeros((n, N), np.uint16)); h = dev(np.zeros((n, N), f32))
    ops.add_rms16(x, dev(nw), 1e-6, h16, n, N, d=dev(d), w=dev(w), S=S, h=h)
    sync()
    assert bits_equal(host(x), ref['x']) and bits_equal(host(h), ref['h']) and bits_equal(host(h16, np.uint16), ref['h16'])
    with pytest.raises(ValueError):
        ops.add_rms16(x, dev(nw), 1e-6, h16, n, 4096)
    ng = 8 * 768
    g = outliers(rng, ng); u = outliers(rng, ng); y16 = dev(np.zeros(ng, np.uint16))
    ops.swiglu(dev(g), dev(u), y16, ng)
    sync()
    assert close_16(host(y16, np.uint16), O.swiglu16(g, u), 'f16')
    nh, nkv, pos0, rows = 8, 2, 5, 16
    M = nkv * 128; ldq = (nh + 2 * nkv) * 128 + 64
    qkv = outliers(rng, (n, ldq)); par = qk_par(rng, yarn=yarn)
    q16 = torch.zeros((n, nh, 128), dtype=torch.float16, device=DEV)
    if q8:
        rbq = 2 * (M // 32) * 34
        fill = np.full((rows, rbq), 0xa5, np.uint8); cache = dev(fill); err = dev(np.zeros(1, np.int32))
        ops.qk_rope(dev(qkv), ldq, nh, nkv, dev(par), pos0, q16, cache, n, rows=rows, err=err)
        sync()
        rq, _, _ = O.qk_rope(qkv, nh, nkv, par, n, pos0=pos0, yarn=yarn, q8=True, cache=fill)
        assert int(host(err)[0]) == 0 and close_16(host(q16.view(torch.int16), np.uint16), rq, 'f16')
        # the row bytes from the fp16 stage the same launch defines (its F16 twin): K16 -> Hadamard -> Q8, V16 -> Q8
        c16 = torch.zeros((rows, 2 * M), dtype=torch.float16, device=DEV); q16f = torch.zeros_like(q16)
        Ops(DEV, yarn=yarn).qk_rope(dev(qkv), ldq, nh, nkv, dev(par), pos0, q16f, c16, n, rows=rows)
        sync()
        kv16 = host(c16.view(torch.int16), np.uint16)[pos0:pos0 + n]
        k16 = O.h2f(kv16[:, :M]).reshape(n * nkv, 128); v16 = O.h2f(kv16[:, M:])
        wantrows, werr = O.kv_q8_append(O.hadamard128(k16).reshape(n, M), M, v16, M, M, fill.reshape(-1), pos0, n, rows=rows)
        assert werr == 0 and bits_equal(host(cache).reshape(-1), wantrows)
        with pytest.raises(ValueError):
            ops.qk_rope(dev(qkv), ldq, nh, nkv, dev(par), pos0, q16, cache, n, rows=rows)          # a Q8 cache needs its error word
    else:
        cache = torch.zeros((rows, 2 * M), dtype=torch.float16, device=DEV)
        ops.qk_rope(dev(qkv), ldq, nh, nkv, dev(par), pos0, q16, cache, n, rows=rows)
        sync()
        rq, rc, _ = O.qk_rope(qkv, nh, nkv, par, n, pos0=pos0, yarn=yarn, rows=rows)
        got = host(cache.view(torch.int16), np.uint16)
        assert close_16(host(q16.view(torch.int16), np.uint16), rq, 'f16') and close_16(got[:, :M], rc[:, :M], 'f16') and bits_equal(got[:, M:], rc[:, M:])
        with pytest.raises(IndexError):
            ops.qk_rope(dev(qkv), ldq, nh, nkv, dev(par), rows - 2, q16, cache, n, rows=rows)      # positions past the cache
    # the same kernel by its reference symbol and launch tuple: grid (n, nh + nkv), block 128
    name = {(False, False): 'q3m_prefill', (True, False): 'q3m_prefill_kvq8', (False, True): 'q3m_prefill_yarn', (True, True): 'q3m_prefill_kvq8_yarn'}[(q8, yarn)]
    mod = hip.Module(name)
    q16b = torch.zeros_like(q16)
    if q8:
        cache2 = dev(np.full((rows, 2 * (M // 32) * 34), 0xa5, np.uint8)); err = dev(np.zeros(1, np.int32))
        mod.q3p_qk_rope_q8((n, nh + nkv), (128,), dev(qkv), I(ldq), I(nh), I(nkv), dev(par), I(pos0), q16b, cache2, err)
    else:
        cache2 = torch.zeros((rows, 2 * M), dtype=torch.float16, device=DEV)
        mod.q3p_qk_rope((n, nh + nkv), (128,), dev(qkv), I(ldq), I(nh), I(nkv), dev(par), I(pos0), q16b, cache2)
    sync()
    assert torch.equal(q16b, q16) and torch.equal(cache2.view(torch.uint8), cache.view(torch.uint8))
    with pytest.raises(ValueError):
        mod.__getattr__('q3p_qk_rope_q8' if q8 else 'q3p_qk_rope')((n, nh), (128,), dev(qkv), I(ldq), I(nh), I(nkv), dev(par), I(pos0), q16b, cache2, *([err] if q8 else []))


def test_module_prefill_attn_and_glue_symbols():
    """pf_qk_nr, pf_gate_mul, pf_hadamard, pf_kv_append (kernels/prefill_attn.hip:106-181,379-386) and pf_rms_mul, pf_gdn_conv,
    pf_conv_state (kernels/prefill_glue.hip:94-124,314-341) with the reference's launch tuples; q35p_add_rms16 and q35p_gate_mul16"""
    from caminus_amd.device import hip
    rng = np.random.default_rng(36)
    A = hip.Module('prefill_attn')
    T, heads, D, nrot, stride = 5, 6, 256, 64, 512
    x = outliers(rng, (T * heads, stride)); w = (1 + 0.1 * rng.standard_normal(D)).astype(f32)
    ts = float(f32(f32(1e7) ** f32(-2.0 / nrot)))
    out = dev(np.zeros((T * heads, D), f32))
    A.pf_qk_nr((T * heads,), (256,), dev(x), I(stride), I(heads), dev(w), I(D), I(nrot), F(ts), F(1e-6), I(9), out)
    a = outliers(rng, (T * heads, D)); y = dev(np.zeros((T * heads, D), f32)); N = T * heads * D
    A.pf_gate_mul(((N + 255) // 256,), (256,), dev(a), dev(x), y, L(N), I(D), I(stride), I(D))
    hx = outliers(rng, (12, 128)); hd = dev(hx)
    A.pf_hadamard((12,), (256,), hd, I(12), I(128), I(1))
    M, rows, pos0 = 256, 9, 3
    k = outliers(rng, (T, M)); v = outliers(rng, (T, M)); rbq = 2 * (M // 32) * 34
    fill = np.full(rows * rbq, 0xa5, np.uint8); cd = dev(fill); err = dev(np.zeros(1, np.int32))
    A.pf_kv_append((T,), (256,), dev(k), I(M), dev(v), I(M), I(M), cd, I(pos0), I(rows), err)
    sync()
    assert close_fp32(host(out), O.qk_nr(x, stride, heads, w, D, nrot, ts, 1e-6, 9, T)) and close_fp32(host(y), O.gate_mul(a, x, D, stride, D))
    assert bits_equal(host(hd), O.hadamard_n(hx, 128))
    wantc, werr = O.pf_kv_append(k, M, v, M, M, fill, pos0, T, rows=rows)
    assert bits_equal(host(cd), wantc) and int(host(err)[0]) == werr == 0
    with pytest.raises(ValueError):
        A.pf_qk_nr((T * heads + 1,), (256,), dev(x), I(stride), I(heads), dev(w), I(D), I(nrot), F(ts), F(1e-6), I(9), out)
    G = hip.Module('prefill_glue')                                        # the build with rows of 2560 values
    R, K, wr = 8, 2560, 4
    xr = outliers(rng, (R, K)); wg = (1 + 0.1 * rng.standard_normal((wr, K))).astype(f32)
    yn = dev(np.zeros((R, K), f32)); ybf = dev(np.zeros((R, K), np.uint16)); scl = dev(np.zeros(R, f32))
    G.pf_rms_mul((R,), (256,), dev(xr), dev(wg), yn, ybf, scl, I(R), I(wr), F(1e-6))
    Cc, Tc = 512, 7
    xc = outliers(rng, (Tc, Cc)); wc = rng.standard_normal((Cc, 4)).astype(f32); st = rng.standard_normal((Cc, 3)).astype(f32)
    yc = dev(np.zeros((Tc, Cc), f32)); sd = dev(st); xcd = dev(xc)
    G.pf_gdn_conv(((Tc * Cc + 255) // 256,), (256,), xcd, dev(wc), sd, yc, I(Cc), I(Tc), I(Cc), I(Cc))
    G.pf_conv_state(((Cc + 255) // 256,), (256,), xcd, sd, I(Cc), I(Tc), I(Cc))
    sync()
    ref = O.rms_mul(xr, wg, 1e-6)
    assert bits_equal(host(yn), ref['y']) and bits_equal(host(ybf, np.uint16), ref['ybf']) and bits_equal(host(scl), ref['scale'])
    ry, rst = O.gdn_conv(xc, wc, st)
    assert close_fp32(host(yc), ry) and bits_equal(host(sd), rst)
    Q = hip.Module('q35_prefill')
    n, N5 = 5, 5120
    x5 = outliers(rng, (n, N5)); d5 = outliers(rng, (n, N5)); nw5 = (1 + 0.1 * rng.standard_normal(N5)).astype(f32)
    xd = dev(x5); h = dev(np.zeros((n, N5), f32)); h16 = dev(np.zeros((n, N5), np.uint16))
    Q.q35p_add_rms16((n,), (256,), xd, dev(d5), dev(nw5), F(1e-6), h, h16, I(N5))
    y16 = dev(np.zeros((T * heads, D), np.uint16))
    Q.q35p_gate_mul16(((N + 255) // 256,), (256,), dev(a), dev(x), y16, L(N), I(D), I(stride), I(D))
    sync()
    r5 = O.add_rms16_q35(x5.copy(), nw5, 1e-6, d=d5)
    assert bits_equal(host(xd), r5['x']) and bits_equal(host(h), r5['h']) and bits_equal(host(h16, np.uint16), r5['h16'])
    assert close_16(host(y16, np.uint16), O.gate_mul(a, x, D, stride, D, f16=True), 'f16')


def test_mmq_wrapper_quantize_scatter_and_fused_swiglu():
    """MMQ.quantize / quantize_scatter (python/caminus/prefill/mmq.py:245-276) and the fused SwiGLU form, small and chunk-sized"""
    from caminus_amd.prefill import mmq
    rng = np.random.default_rng(37)
    q = mmq.MMQ(DEV)
    for ncols, K, layout in ((9, 1000, mmq.DS4), (300, 768, mmq.D4)):
        s01 = K + 8
        x = outliers(rng, (ncols, s01)); x[3, :64] = 0
        y = dev(np.zeros(mmq.y_bytes(K, ncols), np.uint8))
        q.quantize(dev(x), K, ncols, y, layout, s01=s01)
        sync()
        nb = mmq.k_pad(K) // 128 * ncols * 144
        assert bits_equal(host(y)[:nb], O.mmq_q8_1(x, K, ncols, layout, s01=s01).reshape(-1))
        ids = rng.integers(0, ncols, ncols).astype(np.int32)
        y2 = dev(np.zeros(mmq.y_bytes(K, ncols), np.uint8))
        q.quantize(dev(x), K, ncols, y2, layout, s01=s01, ids=dev(ids))
        sync()
        assert bits_equal(host(y2)[:nb], O.mmq_q8_1(x, K, ncols, layout, s01=s01, ids=ids).reshape(-1))
    ntok, k, K = 7, 3, 512
    x = outliers(rng, (ntok, K)); inv = rng.permutation(ntok * k).astype(np.int32)
    y = dev(np.zeros(mmq.y_bytes(K, ntok * k), np.uint8))
    q.quantize_scatter(dev(x), K, ntok, dev(inv), k, y, mmq.DS4)
    sync()
    assert bits_equal(host(y)[:K // 128 * ntok * k * 144], O.mmq_q8_1_scatter(x, K, ntok, inv, k, mmq.DS4).reshape(-1))
    for T, Fh in ((5, 640), (2100, 256)):
        gu = O.f2bf(outliers(rng, (T, 2 * Fh)) * f32(2))
        y = dev(np.zeros(mmq.y_bytes(Fh, T), np.uint8)); act = torch.zeros((T, Fh), dtype=torch.bfloat16, device=DEV)
        q.swiglu_quantize(dev(gu).view(torch.bfloat16), Fh, T, y, mmq.DS4, act=act)
        sync()
        wa = O.silu_mul_bf16(gu)
        assert bits_equal(host(act.view(torch.int16), np.uint16), wa)
        assert bits_equal(host(y)[:mmq.k_pad(Fh) // 128 * T * 144], O.mmq_q8_1(O.bf2f(wa), Fh, T, mmq.DS4).reshape(-1))
    with pytest.raises(ValueError):
        q.quantize(dev(x), K, ntok, dev(np.zeros(16, np.uint8)), mmq.DS4)                          # y too small


def test_record_hook_and_loaded_list():
    """hip.RECORD (python/caminus/device/hip.py:12-14,96-99): a recorder may take a launch over (nothing runs) or watch it go through"""
    from caminus_amd.device import hip

    class Recorder:
        def __init__(self): self.taken, self.seen = [], []

        def intercept(self, kernel, grid, block, vals, shmem, stream):
            if kernel.name == 'cast_bf16':
                self.taken.append((kernel.name, grid, block, len(vals))); return True
            return False

        def launched(self, kernel, grid, block, vals, shmem, stream):
            self.seen.append((kernel.name, grid, block, len(vals), stream))

    rng = np.random.default_rng(38)
    m = hip.Module('core')
    x = outliers(rng, 1024); n = x.size
    c = dev(np.full(n, 0x1234, np.uint16)); mm = O.f2bf(outliers(rng, n)); r3 = dev(np.zeros(n, f32))
    rec = Recorder()
    hip.RECORD = rec
    try:
        m.cast_bf16(((n + 255) // 256,), (256,), dev(x), c, L64(n))                       # taken over: the kernel does not run
        m.residual3(((n + 255) // 256,), (256,), dev(x), dev(mm), dev(mm), r3, L64(n))    # goes through and is reported
    finally:
        hip.RECORD = None
    sync()
    assert rec.taken == [('cast_bf16', (4, 1, 1), (256, 1, 1), 3)] and (host(c, np.uint16) == 0x1234).all()
    assert len(rec.seen) == 1 and rec.seen[0][:4] == ('residual3', (4, 1, 1), (256, 1, 1), 5) and rec.seen[0][4] == torch.cuda.current_stream().cuda_stream
    assert bits_equal(host(r3), O.residual3(x, mm, mm))
    m.cast_bf16(((n + 255) // 256,), (256,), dev(x), c, L64(n))                           # no recorder: the launch goes straight through
    sync()
    assert bits_equal(host(c, np.uint16), O.f2bf(x))
    assert hip.LOADED.index('core') >= 0 and len(set(hip.LOADED)) == len(hip.LOADED)
