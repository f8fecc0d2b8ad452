"""numpy front end of the CPU oracle (oracle/camx_oracle.c). TEST INFRASTRUCTURE ONLY: tests, the smoke check and the
benchmark's cpu_baseline leg import this; nothing in the product package does.

Every wrapper takes and returns numpy arrays; in/out arguments are copied first, so callers' arrays never change.
"""
import ctypes as C
import os

import numpy as np

from . import build as _build

_lib = None
_ref = None


_path = None


def use_library(path):
    """load the oracle from another build of the same source (the benchmark's -O3 -march=native build)"""
    global _lib, _path
    _lib, _path = None, path


def lib():
    global _lib
    if _lib is None:
        if _path is None and not os.path.isfile(_build.ORC_SO):
            _build.build_oracle()
        L = C.CDLL(_path or _build.ORC_SO)
        for n, r in (('orc_bf2f', C.c_float), ('orc_h2f', C.c_float), ('orc_row_ss', C.c_float), ('orc_bfly32_sum', C.c_float)):
            getattr(L, n).restype = r
        for n in ('orc_f2bf', 'orc_to_bf16', 'orc_f2h'):
            getattr(L, n).restype = C.c_uint16
            getattr(L, n).argtypes = [C.c_float]
        L.orc_bf2f.argtypes = [C.c_uint16]; L.orc_h2f.argtypes = [C.c_uint16]
        L.orc_row_ss.argtypes = [C.c_void_p, C.c_int]
        L.orc_bfly32_sum.argtypes = [C.c_void_p]
        _lib = L
    return _lib


def ref_codec():
    """the reference's own_kv_codec.h compiled for the host (oracle/_ref), or None when it was never built here"""
    global _ref
    if _ref is None and os.path.isfile(_build.REF_SO):
        _ref = C.CDLL(_build.REF_SO)
    return _ref


def _p(a):
    return C.c_void_p(a.ctypes.data) if a is not None else C.c_void_p(None)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


I, F, L64 = C.c_int, C.c_float, C.c_int64

# ---- conversions -------------------------------------------------------------------------------------------------------


def f2h(x):
    x = _c(x, np.float32); y = np.empty(x.shape, np.uint16)
    lib().orc_f2h_n(_p(x), _p(y), L64(x.size)); return y


def h2f(h):
    h = _c(h, np.uint16); y = np.empty(h.shape, np.float32)
    lib().orc_h2f_n(_p(h), _p(y), L64(h.size)); return y


def f2bf(x):
    x = _c(x, np.float32); y = np.empty(x.shape, np.uint16)
    lib().orc_cast_bf16(_p(x), _p(y), L64(x.size)); return y


def bf2f(h):
    return (_c(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def set_threads(n):
    """threads the row loops run on (timing only); returns the previous setting"""
    return int(lib().orc_set_threads(C.c_int(n)))


def row_ss(x):
    x = _c(x, np.float32); return np.float32(lib().orc_row_ss(_p(x), I(x.size)))


# ---- q8_1 ----------------------------------------------------------------------------------------------------------------


def q8_1(x, mode=0, rs=0.0, g=None):
    """uint8 [ceil(n / 32), 36]"""
    x = _c(x, np.float32).reshape(-1); n = x.size
    g = _c(g, np.float32).reshape(-1) if g is not None else None
    y = np.zeros(((n + 31) // 32, 36), np.uint8)
    lib().orc_q8_1(_p(x), _p(y), L64(n), I(mode), F(rs), _p(g)); return y


def k_pad(K):
    return (int(K) + 511) // 512 * 512


def mmq_q8_1(x, K, ncols, layout, s01=None, ids=None):
    """uint8 [K_pad / 128, ncols, 144]"""
    x = _c(x, np.float32); s01 = K if s01 is None else s01
    ids = _c(ids, np.int32) if ids is not None else None
    y = np.zeros((k_pad(K) // 128, ncols, 144), np.uint8)
    lib().orc_mmq_q8_1(_p(x), _p(ids), _p(y), L64(K), L64(s01), I(ncols), I(layout)); return y


def mmq_q8_1_scatter(x, K, ntok, ids_inv, k, layout, s_tok=None, fill=0):
    x = _c(x, np.float32); s_tok = K if s_tok is None else s_tok
    ids_inv = _c(ids_inv, np.int32)
    y = np.full((k_pad(K) // 128, ntok * k, 144), fill, np.uint8)
    lib().orc_mmq_q8_1_scatter(_p(x), _p(ids_inv), _p(y), L64(K), L64(s_tok), I(ntok), I(k), I(layout)); return y


# ---- norms ---------------------------------------------------------------------------------------------------------------


def add_rms16(x, nw, eps, d=None, w=None, S=0, want_q8=False):
    """-> dict(x, h, h16[, q8]); x [n, N]"""
    x = _c(x, np.float32).copy(); n, N = x.shape
    d = _c(d, np.float32) if d is not None else None
    w = _c(w, np.float32) if w is not None else None
    nw = _c(nw, np.float32)
    h = np.empty_like(x); h16 = np.empty(x.shape, np.uint16)
    q8 = np.zeros((n, N // 32, 36), np.uint8) if want_q8 else None
    lib().orc_add_rms16(_p(x), _p(d), _p(w), I(S), _p(nw), F(eps), _p(h), _p(h16), _p(q8), I(N), I(n))
    out = dict(x=x, h=h, h16=h16)
    if want_q8: out['q8'] = q8
    return out


def add_rms16_q35(x, nw, eps, d=None):
    x = _c(x, np.float32).copy(); n, N = x.shape
    d = _c(d, np.float32) if d is not None else None
    h = np.empty_like(x); h16 = np.empty(x.shape, np.uint16)
    lib().orc_add_rms16_q35(_p(x), _p(d), _p(_c(nw, np.float32)), F(eps), _p(h), _p(h16), I(N), I(n))
    return dict(x=x, h=h, h16=h16)


def add_rms_bf16(x, d, nw, eps):
    x = _c(x, np.float32).copy(); n, N = x.shape
    d = _c(d, np.uint16) if d is not None else None
    h = np.empty_like(x); hbf = np.empty(x.shape, np.uint16)
    lib().orc_add_rms_bf16(_p(x), _p(d), _p(_c(nw, np.float32)), F(eps), _p(h), _p(hbf), I(N), I(n))
    return dict(x=x, h=h, hbf=hbf)


def rms_mul(x, w, eps, want_q8=False):
    x = _c(x, np.float32); R, K = x.shape
    w = _c(w, np.float32).reshape(-1, K); wr = w.shape[0]
    y = np.empty_like(x); ybf = np.empty(x.shape, np.uint16); scl = np.empty(R, np.float32)
    q8 = np.zeros((R, K // 32, 36), np.uint8) if want_q8 else None
    lib().orc_rms_mul(_p(x), _p(w), _p(y), _p(ybf), _p(scl), _p(q8), I(R), I(wr), I(K), F(eps))
    out = dict(y=y, ybf=ybf, scale=scl)
    if want_q8: out['q8'] = q8
    return out


def hc_post_rms(b, inj, res, w, eps, rs=0.25):
    """-> dict(res, xn, xnbf, scale); b [T, N], inj [T, HC], res [T, HC, N], w [HC, N]"""
    b = _c(b, np.float32); inj = _c(inj, np.float32); res = _c(res, np.float32).copy(); w = _c(w, np.float32)
    T, HC, N = res.shape
    xn = np.empty_like(res); xnbf = np.empty(res.shape, np.uint16); scl = np.empty(T * HC, np.float32)
    lib().orc_hc_post_rms(_p(b), _p(inj), _p(res), _p(w), _p(xn), _p(xnbf), _p(scl), I(T), I(HC), I(N), F(rs), F(eps))
    return dict(res=res, xn=xn, xnbf=xnbf, scale=scl)


def hc_post(b, inj, res, rs=0.25):
    b = _c(b, np.float32); inj = _c(inj, np.float32); res = _c(res, np.float32).copy()
    T, HC, D = res.shape
    lib().orc_hc_post(_p(b), _p(inj), _p(res), I(T), I(HC), I(D), F(rs))
    return res


def hc_mean(x, g, rs=0.25, scale=None, w=None):
    x = _c(x, np.float32); g = _c(g, np.float32)
    T, HC, D = x.shape
    out = np.empty((T, D), np.float32)
    lib().orc_hc_mean(_p(x), _p(_c(scale, np.float32)) if scale is not None else _p(None), _p(_c(w, np.float32)) if w is not None else _p(None),
                      _p(g), _p(out), I(T), I(HC), I(D), F(rs))
    return out


def rmsnorm_f32(x, w, eps):
    x = _c(x, np.float32); rows, D = x.shape; out = np.empty_like(x)
    lib().orc_rmsnorm_f32(_p(x), _p(_c(w, np.float32)), _p(out), I(D), F(eps), I(rows)); return out


# ---- core / fuse -----------------------------------------------------------------------------------------------------------


def embedding_f32(tok, emb):
    tok = _c(tok, np.int32); emb = _c(emb, np.float32); out = np.empty((tok.size, emb.shape[1]), np.float32)
    lib().orc_embedding_f32(_p(tok), _p(emb), _p(out), I(emb.shape[1]), I(tok.size)); return out


def silu_mul_bf16(gu):
    gu = _c(gu, np.uint16); R, H2 = gu.shape; H = H2 // 2; act = np.empty((R, H), np.uint16)
    lib().orc_silu_mul_bf16(_p(gu), _p(act), I(H), L64(R * H)); return act


def residual3(x, m, y):
    x = _c(x, np.float32); out = np.empty_like(x)
    lib().orc_residual3(_p(x), _p(_c(m, np.uint16)), _p(_c(y, np.uint16)), _p(out), L64(x.size)); return out


def copy_cols_bf16(inp, c_in, out, c_out, n):
    inp = _c(inp, np.uint16); out = _c(out, np.uint16).copy()
    lib().orc_copy_cols_bf16(_p(inp), I(inp.shape[1]), I(c_in), _p(out), I(out.shape[1]), I(c_out), I(n), L64(inp.shape[0])); return out


def residual_slices_bwd(dout, pos, nys):
    """-> (dm, dmlp, dys) bf16 bits; dys [nys, d] rows that no pos names stay 0"""
    dout = _c(dout, np.float32); d = dout.shape[-1]
    dm = np.empty(dout.shape, np.uint16); dmlp = np.empty(dout.shape, np.uint16); dys = np.zeros((nys, d), np.uint16)
    lib().orc_residual_slices_bwd(_p(dout), _p(_c(pos, np.int32)) if pos is not None else _p(None), _p(dm), _p(dmlp), _p(dys), I(d), L64(dout.size))
    return dm, dmlp, dys


def residual_slices_fwd(x, m, mlp, ys, pos):
    x = _c(x, np.float32); d = x.shape[-1]; out = np.empty_like(x)
    ys = _c(ys, np.uint16) if ys is not None else None
    pos = _c(pos, np.int32) if pos is not None else None
    lib().orc_residual_slices_fwd(_p(x), _p(_c(m, np.uint16)), _p(_c(mlp, np.uint16)), _p(ys), _p(pos), _p(out), I(d), L64(x.size // 4))
    return out


# ---- SwiGLU / gates / GDN ----------------------------------------------------------------------------------------------------


def swiglu16(g, u):
    g = _c(g, np.float32); y = np.empty(g.shape, np.uint16)
    lib().orc_swiglu16(_p(g), _p(_c(u, np.float32)), _p(y), L64(g.size)); return y


def silu_mul_f32(g, u):
    g = _c(g, np.float32); y = np.empty_like(g)
    lib().orc_silu_mul_f32(_p(g), _p(_c(u, np.float32)), _p(y), L64(g.size)); return y


def gate_mul(a, gate, D, stride, off, f16=False):
    a = _c(a, np.float32); gate = _c(gate, np.float32)
    y = np.empty(a.shape, np.float32); y16 = np.empty(a.shape, np.uint16) if f16 else None
    lib().orc_gate_mul(_p(a), _p(gate), _p(y), _p(y16), L64(a.size), I(D), I(stride), I(off))
    return y16 if f16 else y


def gdn_conv(x, w, st, ldx=None, ldy=None):
    """-> (y [T, C], new state [C, 3]); x [T, ldx]"""
    x = _c(x, np.float32); w = _c(w, np.float32); st = _c(st, np.float32).copy()
    T = x.shape[0]; C_ = w.shape[0]; ldx = x.shape[1] if ldx is None else ldx; ldy = C_ if ldy is None else ldy
    y = np.zeros((T, ldy), np.float32)
    lib().orc_gdn_conv(_p(x), _p(w), _p(st), _p(y), I(C_), I(T), I(ldx), I(ldy))
    lib().orc_conv_state(_p(x), _p(st), I(C_), I(T), I(ldx))
    return y, st


def op_gdn_conv(w, st, x, mprev, xprev):
    """OP_GDN_CONV -> (y [T, C], state after the commit [C, 3], xprev for the next pass [T, C])"""
    x = _c(x, np.float32); w = _c(w, np.float32); st = _c(st, np.float32).copy(); xprev = _c(xprev, np.float32).copy()
    T, C_ = x.shape
    params = np.array([0, mprev, 0, 0], np.int32); y = np.zeros((T, C_), np.float32)
    lib().orc_op_gdn_conv(_p(w), _p(st), _p(x), _p(params), _p(y), _p(xprev), I(C_), I(T))
    return y, st, xprev


def gdn_l2(x, T, heads, K, eps, ldx=None):
    x = _c(x, np.float32); ldx = heads * K if ldx is None else ldx
    y = np.empty((T * heads, K), np.float32)
    lib().orc_gdn_l2(_p(x), _p(y), I(T), I(heads), I(K), I(ldx), F(np.float32(eps / K))); return y


def gdn_conv_l2(x, w, st, heads, eps, bf16=False):
    """OP_GDN_CONV then OP_GDN_L2 as the reference's dense engine appends them (python/caminus/engine/q35_dense.py:399-400): the L2 norm reads
    the first heads * 128 channels of the convolution's stored output (bf16: rounded first). -> (y [T, C], qk [T * heads, 128])"""
    y, _ = gdn_conv(x, w, st)
    if bf16: y = bf2f(f2bf(y))
    T, C_ = y.shape
    return y, gdn_l2(y, T, heads, 128, eps, ldx=C_)


def qk_nr_q8(q, q_stride, nh, k, v, nkv, qn, kn, n_rot, theta_scale, eps, pos, cache, rows):
    """the dense Q8 line's chain (python/caminus/engine/q35_dense.py:409-418): qo = H256(qk_nr(q)); cache row pos[t] = Q8 blocks of
    H256(qk_nr(k)) | Q8 blocks of H64(v) with the codec's refusals (kernels/k3_q35_kvq8_ops.h:16-50). pos: one position per token.
    -> (qo [T * nh, 256], cache bytes, err)"""
    T = len(pos); M = nkv * 256; err = 0
    k = _c(k, np.float32).reshape(T, M); v = _c(v, np.float32).reshape(T, M)
    qo = np.concatenate([hadamard_n(qk_nr(_c(q, np.float32)[t * nh:(t + 1) * nh], q_stride, nh, qn, 256, n_rot, theta_scale, eps, int(pos[t]), 1), 256) for t in range(T)])
    cache = _c(cache, np.uint8).copy()
    for t in range(T):
        ko = hadamard_n(qk_nr(k[t].reshape(nkv, 256), 256, nkv, kn, 256, n_rot, theta_scale, eps, int(pos[t]), 1), 256).reshape(1, M)
        vo = hadamard_n(v[t], 64).reshape(1, M)
        cache, e = kv_q8_append(ko, M, vo, M, M, cache, int(pos[t]), 1, rows=rows)
        err |= e
    return qo, cache, err


def qk_nr_kv(q, q_stride, nh, wq, k, k_stride, v, nkv, wk, D, n_rot, theta_scale, eps, pos0, T, cache, q8, ko=None):
    """the fp16 / q8_0 cache lines' chain (python/caminus/engine/q3moe_one.py:316-318): OP_QK_NR of k -> OP_KV_APPEND (rows pos0 + t) and
    OP_QK_NR of q. ko: the normed k to append instead of this function's own (a caller that holds another implementation's fp32 result and
    wants the cache bytes that follow from it). -> (qo [T * nh, D], ko [T * nkv, D], cache after the append, err)"""
    M = nkv * D
    qo = qk_nr(q, q_stride, nh, wq, D, n_rot, theta_scale, eps, pos0, T)
    kn = qk_nr(k, k_stride, nkv, wk, D, n_rot, theta_scale, eps, pos0, T)
    ka = _c(kn if ko is None else ko, np.float32).reshape(T, M); v = _c(v, np.float32).reshape(T, M)
    if q8: cache, err = pf_kv_append(ka, M, v, M, M, cache, pos0, T)
    else: cache, err = kv_append16(ka, v, M, cache, pos0)
    return qo, kn, cache, err


# ---- rotary ---------------------------------------------------------------------------------------------------------------


def qk_nr(x, head_stride, heads, w, D, n_rot, theta_scale, eps, pos0, T):
    x = _c(x, np.float32); out = np.empty((T * heads, D), np.float32)
    lib().orc_qk_nr(_p(x), I(head_stride), I(heads), _p(_c(w, np.float32)), I(D), I(n_rot), F(theta_scale), F(eps), I(pos0), _p(out), I(T))
    return out


def qk_rope(qkv, nh, nkv, par, n, pos0=0, pos=None, yarn=False, q8=False, cache=None, rows=None,
            page_table=None, page=256, n_pages=0):
    """-> (q16 uint16 [n, nh, 128], cache, err). cache: given (copied) or zeros of `rows` rows; fp16 rows as uint16
    [rows, 2 M], Q8 rows as uint8 [rows, row_bytes]."""
    qkv = _c(qkv, np.float32); ldq = qkv.shape[1]; M = nkv * 128
    par = _c(par, np.float32)
    q16 = np.zeros((n, nh, 128), np.uint16)
    if cache is None:
        cache = np.zeros((rows, 2 * (M // 32) * 34), np.uint8) if q8 else np.zeros((rows, 2 * M), np.uint16)
    else:
        cache = cache.copy()
    err = np.zeros(1, np.int32)
    pos = _c(pos, np.int32) if pos is not None else None
    pt = _c(page_table, np.int32) if page_table is not None else None
    lib().orc_qk_rope(_p(qkv), I(ldq), I(nh), I(nkv), _p(par), I(pos0), _p(pos), _p(q16), _p(cache), I(n), I(int(yarn)), I(int(q8)),
                      _p(err), _p(pt), I(pt.shape[1] if pt is not None else 0), I(page), I(n_pages))
    return q16, cache, int(err[0])


# ---- Hadamard / KV codec ------------------------------------------------------------------------------------------------------


def hadamard128(x):
    x = _c(x, np.float32); y = np.empty_like(x)
    lib().orc_hadamard128(_p(x), _p(y), L64(x.size // 128)); return y


def hadamard_n(x, n):
    x = _c(x, np.float32).copy()
    lib().orc_hadamard_n(_p(x), L64(x.size // n), I(n)); return x


def kv_q8_encode(blocks, fill=0xa5):
    """blocks float32 [nb, 32] -> (bytes uint8 [nb, 34] (refused blocks keep `fill`), ok uint8 [nb])"""
    b = _c(blocks, np.float32).reshape(-1, 32); raw = np.full((b.shape[0], 34), fill, np.uint8); ok = np.zeros(b.shape[0], np.uint8)
    lib().orc_kv_q8_encode(_p(b), _p(raw), _p(ok), L64(b.shape[0])); return raw, ok


def ref_kv_q8_encode(blocks, fill=0xa5):
    """the same through the compiled reference header (None when oracle/_ref was not built)"""
    r = ref_codec()
    if r is None: return None
    b = _c(blocks, np.float32).reshape(-1, 32); raw = np.full((b.shape[0], 34), fill, np.uint8); ok = np.zeros(b.shape[0], np.uint8)
    r.ref_kv_q8_encode(_p(b), _p(raw), _p(ok), C.c_long(b.shape[0])); return raw, ok


def kv_q8_append(k, ldk, v, ldv, M, cache, pos0, T, rows=None):
    """-> (cache bytes (copy), err)"""
    k = _c(k, np.float32); v = _c(v, np.float32); cache = _c(cache, np.uint8).copy()
    rb = 2 * (M // 32) * 34 if M >= 32 else 1
    rows = cache.size // rb if rows is None else rows
    err = np.zeros(1, np.int32)
    lib().orc_kv_q8_append(_p(k), I(ldk), _p(v), I(ldv), I(M), _p(cache), I(pos0), I(rows), I(T), _p(err))
    return cache, int(err[0])


def kv_q8_read(cache, M, T, pos0=0, row_ids=None, rows=None, f16=False, fill=None):
    """-> (k, v, err): [T, M] float32, or fp16 bits (uint16) when f16; rows outside [0, rows) keep `fill`"""
    cache = _c(cache, np.uint8).reshape(-1); rb = 2 * (M // 32) * 34
    rows = cache.size // rb if rows is None else rows
    dt = np.uint16 if f16 else np.float32
    k = np.zeros((T, M), dt); v = np.zeros((T, M), dt)
    if fill is not None: k[:] = fill; v[:] = fill
    err = np.zeros(1, np.int32)
    ids = _c(row_ids, np.int32) if row_ids is not None else None
    lib().orc_kv_q8_read(_p(cache), _p(ids), I(pos0), I(rows), I(M), _p(k), I(M), _p(v), I(M), I(T), I(int(f16)), _p(err))
    return k, v, int(err[0])


def pf_kv_append(k, ldk, v, ldv, M, cache, pos0, T, rows=None):
    k = _c(k, np.float32); v = _c(v, np.float32); cache = _c(cache, np.uint8).copy()
    rb = 2 * (M // 32) * 34
    rows = cache.size // rb if rows is None else rows
    err = np.zeros(1, np.int32)
    lib().orc_pf_kv_append(_p(k), I(ldk), _p(v), I(ldv), I(M), _p(cache), I(pos0), I(rows), I(T), _p(err))
    return cache, int(err[0])


# ---- quantized embedding rows ---------------------------------------------------------------------------------------------------


def emb_q4k(W, vocab, toks, N):
    W = _c(W, np.uint8); toks = _c(toks, np.int32); rb = N // 256 * 144
    x = np.empty((toks.size, N), np.float32); xbf = np.empty((toks.size, N), np.uint16)
    lib().orc_emb_q4k(_p(W), I(rb), I(vocab), _p(toks), _p(x), _p(xbf), I(N), I(toks.size)); return x, xbf


def emb_q8_0(W, vocab, toks, N):
    W = _c(W, np.uint8); toks = _c(toks, np.int32); rb = N // 32 * 34
    x = np.empty((toks.size, N), np.float32); xbf = np.empty((toks.size, N), np.uint16)
    lib().orc_emb_q8_0(_p(W), I(rb), I(vocab), _p(toks), _p(x), _p(xbf), I(N), I(toks.size)); return x, xbf


def emb_iq4xs(W, vocab, toks, N):
    """-> (x fp32 [n, N], xbf bf16 bits, err word)"""
    W = _c(W, np.uint8); toks = _c(toks, np.int32)
    x = np.empty((toks.size, N), np.float32); xbf = np.empty((toks.size, N), np.uint16); err = np.zeros(1, np.int32)
    lib().orc_emb_iq4xs(_p(W), I(vocab), _p(toks), _p(x), _p(xbf), I(N // 256), I(toks.size), _p(err)); return x, xbf, int(err[0])


def ple_rows_iq4nl(raw, inv, nuniq, bpr):
    """-> (out fp32 [nrows, 32 bpr], err word)"""
    raw = _c(raw, np.uint8); inv = _c(inv, np.int32)
    out = np.empty((inv.size, 32 * bpr), np.float32); err = np.zeros(1, np.int32)
    lib().orc_ple_rows_iq4nl(_p(raw), _p(inv), I(nuniq), I(inv.size), I(bpr), _p(out), _p(err)); return out, int(err[0])


_IQ2S = None


def iq2s_grid():
    """the IQ2_S codebook, uint8 [1024, 8] (ggml's iq2s_grid as magnitude bytes; oracle/iq2s_grid.npy)"""
    global _IQ2S
    if _IQ2S is None:
        _IQ2S = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'iq2s_grid.npy'))
    return _IQ2S


def emb_iq2s(W, vocab, toks, N):
    W = _c(W, np.uint8); toks = _c(toks, np.int32); grid = _c(iq2s_grid(), np.uint8)
    x = np.empty((toks.size, N), np.float32); xbf = np.empty((toks.size, N), np.uint16)
    lib().orc_emb_iq2s(_p(W), I(vocab), _p(toks), _p(x), _p(xbf), I(N), I(toks.size), _p(grid)); return x, xbf


# ---- more row kernels of the batched prefill ---------------------------------------------------------------------------------


def gdn_norm(o, w, z, eps, silu=False):
    """-> (y fp32 [rows, K], y16 fp16 bits)"""
    o = _c(o, np.float32); rows, K = o.shape; w = _c(w, np.float32); z = _c(z, np.float32)
    y = np.empty((rows, K), np.float32); y16 = np.empty((rows, K), np.uint16)
    lib().orc_gdn_norm(_p(o), _p(w), _p(z), _p(y), _p(y16), I(K), F(eps), C.c_long(rows), I(int(silu))); return y, y16


def gdn_gates(al, be, dt, A):
    al = _c(al, np.float32); be = _c(be, np.float32); T, H = al.shape[0], dt.size
    dt = _c(dt, np.float32); A = _c(A, np.float32); y = np.empty((T, 2 * H), np.float32)
    lib().orc_gdn_gates(_p(al), I(al.shape[1]), _p(be), I(be.shape[1]), _p(dt), _p(A), _p(y), I(H), I(T)); return y


def kv_append16(k, v, M, cache, pos0):
    """-> (cache fp16 bits [rows, 2 M] after the append, err word)"""
    k = _c(k, np.float32); v = _c(v, np.float32); cache = _c(cache, np.uint16).copy(); err = np.zeros(1, np.int32)
    lib().orc_kv_append16(_p(k), I(k.shape[1]), _p(v), I(v.shape[1]), _p(cache), I(M), I(pos0), I(cache.shape[0]), _p(err), I(k.shape[0]))
    return cache, int(err[0])


def own_moe_sum(d, w, x, slots):
    """OP_OWN_MOE_SUM (kernels/k3_own_ops.h:263-271): x += the slot-ordered fma chain (w None: plain adds) -> x"""
    d = _c(d, np.float32); x = _c(x, np.float32).copy(); w = None if w is None else _c(w, np.float32)
    lib().orc_own_moe_sum(_p(d), _p(w), _p(x), C.c_long(x.size), I(slots)); return x


def shexp_add(moe, shexp, logit, T):
    """OP_SHEXP_ADD (kernels/k3_gguf_ops.h:1220-1229) -> out"""
    moe = _c(moe, np.float32); shexp = _c(shexp, np.float32); logit = _c(logit, np.float32); out = np.empty_like(moe)
    lib().orc_shexp_add(_p(moe), _p(shexp), _p(logit), _p(out), C.c_long(moe.size), I(T)); return out


def own_f16(x):
    """OP_OWN_F16 (kernels/k3_own_ops.h:247-252) -> fp16 bits"""
    return f2h(x)


def add_sum(a, b, y):
    a = _c(a, np.float32); b = _c(b, np.float32); y = _c(y, np.float32).copy()
    lib().orc_add_sum(_p(a), _p(b), _p(y), C.c_long(y.size)); return y


def to_bf16_rows(x, T, Tpad, K, rs=0.0, silu=False):
    x = _c(x, np.float32); y = np.empty((Tpad, K), np.uint16)
    lib().orc_to_bf16_rows(_p(x), I(x.shape[1]), _p(y), I(T), I(Tpad), I(K), F(rs), I(int(silu))); return y


def hc_avg(r, ldo=None):
    r = _c(r, np.float32); T, hc, D = r.shape; ldo = ldo or D
    y = np.zeros((T, ldo), np.float32)
    lib().orc_hc_avg(_p(r), _p(y), I(T), I(hc), I(D), I(ldo)); return y


def ple_gate(kn, q, val, qscl=None, qw=None):
    """-> (gated [T, HC, D], gate [T, HC])"""
    kn = _c(kn, np.float32); q = _c(q, np.float32); val = _c(val, np.float32); T, HC, D = kn.shape
    qscl = _c(qscl, np.float32) if qscl is not None else None; qw = _c(qw, np.float32) if qw is not None else None
    gated = np.empty((T, HC, D), np.float32); gate = np.empty((T, HC), np.float32)
    lib().orc_ple_gate(_p(kn), _p(q), _p(qscl), _p(qw), _p(val), I(val.shape[1]), _p(gated), _p(gate), I(HC), I(D), I(T)); return gated, gate


def ple_conv(x, w16, hist, D, dil, xscl=None, xw=None, a=None, res=None):
    """-> (y [T, C], res after the fused add or None); w16: fp16 bits [C, 4]"""
    x = _c(x, np.float32); T, Cc = x.shape; w16 = _c(w16, np.uint16); hist = _c(hist, np.float32)
    xscl = _c(xscl, np.float32) if xscl is not None else None; xw = _c(xw, np.float32) if xw is not None else None
    a = _c(a, np.float32) if a is not None else None; res = _c(res, np.float32).copy() if res is not None else None
    y = np.empty((T, Cc), np.float32)
    lib().orc_ple_conv(_p(x), _p(xscl), _p(xw), _p(w16), _p(hist), _p(y), _p(a), _p(res), I(Cc), I(T), I(D), I(dil)); return y, res


def ple_hist(x, hist, D, dil, xscl=None, xw=None):
    x = _c(x, np.float32); T, Cc = x.shape; hist = _c(hist, np.float32).copy()
    xscl = _c(xscl, np.float32) if xscl is not None else None; xw = _c(xw, np.float32) if xw is not None else None
    lib().orc_ple_hist(_p(x), _p(xscl), _p(xw), _p(hist), I(Cc), I(T), I(D), I(dil)); return hist


# ---- actq -----------------------------------------------------------------------------------------------------------------------


def actq_fwd(x, clip=1.0, qmax=7, bf16=False):
    """-> (y bf16 bits [M, K], s [M], codes uint8 [M, K / 2])"""
    x = _c(x, np.uint16 if bf16 else np.float32); M, K = x.shape
    y = np.empty((M, K), np.uint16); s = np.empty(M, np.float32); c = np.zeros((M, K // 2), np.uint8)
    lib().orc_actq_fwd(_p(x), I(int(bf16)), _p(y), _p(s), _p(c), I(M), I(K), F(clip), I(qmax)); return y, s, c


def silu_mul_actq_fwd(gu, clip=1.0, qmax=7):
    gu = _c(gu, np.uint16); M, F2 = gu.shape; Fh = F2 // 2
    y = np.empty((M, Fh), np.uint16); s = np.empty(M, np.float32); c = np.zeros((M, Fh // 2), np.uint8)
    lib().orc_silu_mul_actq_fwd(_p(gu), I(F2), I(Fh), _p(y), _p(s), _p(c), I(M), F(clip), I(qmax)); return y, s, c


def block_entry_fwd(x, nw, wab, eps, clip=1.0, qmax=7):
    x = _c(x, np.float32); M, d = x.shape
    nab = 0 if wab is None else wab.shape[0]
    wab = _c(wab, np.uint16) if nab else None
    y = np.empty((M, d), np.uint16); s = np.empty(M, np.float32); c = np.zeros((M, d // 2), np.uint8)
    ab = np.zeros((M, max(nab, 1)), np.uint16); rstd = np.empty(M, np.float32)
    lib().orc_block_entry_fwd(_p(x), _p(_c(nw, np.float32)), _p(wab), I(nab), F(eps), _p(y), _p(s), _p(c), _p(ab), _p(rstd),
                              I(M), I(d), F(clip), I(qmax))
    return y, s, c, ab[:, :nab], rstd


def actq_rotate(x):
    """u = bf16(H128 . bf16 x) per 128-chunk, bf16 bits [M, K] (the forward's first stage; also the backward's last)"""
    x = _c(x, np.uint16); M, K = x.shape
    u = np.empty((M, K), np.uint16)
    lib().orc_actq_rotate(_p(x), _p(u), I(M), I(K)); return u


def actq_bwd(x, g, clip=1.0, qmax=7, bf16=False):
    """-> dx [M, K]: fp32, or bf16 bits when x is bf16 bits"""
    x = _c(x, np.uint16 if bf16 else np.float32); M, K = x.shape
    dx = np.empty((M, K), np.uint16 if bf16 else np.float32); g = _c(g, np.uint16)
    lib().orc_actq_bwd(_p(x), I(int(bf16)), _p(g), _p(dx), I(M), I(K), F(clip), I(qmax)); return dx


def silu_mul_actq_bwd(gu, g, clip=1.0, qmax=7, table=False):
    """-> dgu bf16 bits [M, 2F]. table: the derivative's sigmoid from the correctly rounded single-precision exponential (the definition of
    the HIP kernel's table) instead of the C library's expf"""
    gu = _c(gu, np.uint16); M, F2 = gu.shape
    dgu = np.empty((M, F2), np.uint16); g = _c(g, np.uint16)
    fn = lib().orc_silu_mul_actq_bwd_tab if table else lib().orc_silu_mul_actq_bwd
    fn(_p(gu), I(F2), I(F2 // 2), _p(g), _p(dgu), I(M), F(clip), I(qmax)); return dgu


def block_entry_bwd(x, nw, rstd, wab, dy, dab, clip=1.0, qmax=7):
    """-> dx fp32 [M, d]"""
    x = _c(x, np.float32); M, d = x.shape
    nab = 0 if wab is None else wab.shape[0]
    nw = _c(nw, np.float32); rstd = _c(rstd, np.float32); dy = _c(dy, np.uint16)
    wab = _c(wab, np.uint16) if nab else None; dab = _c(dab, np.uint16) if nab else None
    dx = np.empty((M, d), np.float32)
    lib().orc_block_entry_bwd(_p(x), _p(nw), _p(rstd), _p(wab), I(nab), _p(dy), _p(dab), _p(dx), I(M), I(d), F(clip), I(qmax))
    return dx
