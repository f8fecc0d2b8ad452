"""GPU parity of the fused chains (conv4 + SiLU + L2 norm; QK-norm + partial rotary + Hadamard + Q8 blocks), of the tape-shaped entry
points that read their position from a device word, and of camx_init. A fused launch must leave the bytes of the separate launches it
replaces (that is its contract); the separate launches are held to the oracle by their own tests, and the fused outputs are checked
against the oracle's composition as well."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O
from gpu_util import F, HADAMARD_FLOOR, I, L64, NULL, bits_equal, call, camx, close_16, close_fp32, dev, host, outliers, ptr, stream
from vectors import qk_par

pytestmark = pytest.mark.gpu
RS = np.float32(1e-6 / 128)


def _theta(base, n_rot):
    return float(np.float32(np.float32(base) ** np.float32(-2.0 / n_rot)))


# ---- conv4 + SiLU + L2 ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize('T,C,heads', [(16, 10240, 32), (16, 10240, 48), (1, 128, 1), (5, 1024, 3), (3, 384, 3), (300, 4096, 16), (4096, 10240, 32), (1100, 1024, 8)])
@pytest.mark.parametrize('bf16', [0, 1])
def test_gdn_conv_l2_equals_the_two_launches(T, C, heads, bf16):
    rng = np.random.default_rng(T + C + heads)
    pad = 8
    x = outliers(rng, (T, C + pad)); w = rng.standard_normal((C, 4)).astype(np.float32); st = rng.standard_normal((C, 3)).astype(np.float32)
    xin = O.f2bf(x) if bf16 else x
    dt = np.uint16 if bf16 else np.float32
    xd, wd, sd = dev(xin), dev(w), dev(st)
    y1 = dev(np.zeros((T, C), dt)); q1 = dev(np.zeros((T * heads, 128), dt))
    call('camx_pf_gdn_conv', ptr(xd), ptr(wd), ptr(sd), ptr(y1), I(C), I(T), I(C + pad), I(C), I(bf16))
    call('camx_pf_gdn_l2', ptr(y1), ptr(q1), I(heads), I(128), I(C), F(RS), I(T), I(bf16))
    y2 = dev(np.full((T, C), 7, dt)); q2 = dev(np.full((T * heads, 128), 7, dt))
    call('camx_gdn_conv_l2', ptr(xd), ptr(wd), ptr(sd), ptr(y2), ptr(q2), I(C), I(T), I(C + pad), I(C), I(heads), F(RS), I(bf16))
    assert torch.equal(y1, y2) and torch.equal(q1, q2)
    q3 = dev(np.full((T * heads, 128), 7, dt))                      # without the convolution's own output
    call('camx_gdn_conv_l2', ptr(xd), ptr(wd), ptr(sd), NULL, ptr(q3), I(C), I(T), I(C + pad), I(C), I(heads), F(RS), I(bf16))
    assert torch.equal(q1, q3)
    if T * C <= 16 * 10240 or (T, C) == (300, 4096):                # against the oracle (the big shapes are covered by the equality above)
        xs = O.bf2f(xin) if bf16 else x
        ry, _ = O.gdn_conv(xs, w, st, ldx=C + pad)
        if bf16:
            assert close_16(host(y2, np.uint16), O.f2bf(ry), 'bf16')
            assert bits_equal(host(q2, np.uint16), O.f2bf(O.gdn_l2(O.bf2f(host(y2, np.uint16)), T, heads, 128, 1e-6, ldx=C)))   # exact from the stored y on
        else:
            assert close_fp32(host(y2), ry)
            assert bits_equal(host(q2), O.gdn_l2(host(y2), T, heads, 128, 1e-6, ldx=C))


def test_gdn_conv_l2_refuses_shapes_it_does_not_cover():
    L = camx(); z = dev(np.zeros(1024, np.float32))
    p = lambda t: C.c_void_p(t.data_ptr())
    assert L.camx_gdn_conv_l2(p(z), p(z), p(z), p(z), p(z), I(200), I(1), I(200), I(200), I(1), F(RS), I(0), stream()) == 1      # C % 128
    assert L.camx_gdn_conv_l2(p(z), p(z), p(z), p(z), p(z), I(256), I(1), I(256), I(256), I(3), F(RS), I(0), stream()) == 1      # more heads than channels
    assert L.camx_gdn_conv_l2(p(z), p(z), p(z), p(z), NULL, I(256), I(1), I(256), I(256), I(1), F(RS), I(0), stream()) == 1     # no qk


@pytest.mark.parametrize('C_,T,heads', [(10240, 16, 32), (256, 4, 2), (128, 1, 1), (1024, 7, 5)])
def test_op_gdn_conv_l2_equals_the_two_tape_ops(C_, T, heads):
    rng = np.random.default_rng(C_ + T)
    w = rng.standard_normal((C_, 4)).astype(np.float32); st0 = rng.standard_normal((C_, 3)).astype(np.float32)
    junk = rng.standard_normal((T, C_)).astype(np.float32)
    wd = dev(w)
    s1, s2 = dev(st0), dev(st0); xp1, xp2 = dev(junk), dev(junk)
    m = 0
    for step in range(3):                                           # three passes; the second and third commit m tokens of the one before
        x = outliers(rng, (T, C_)); xd = dev(x)
        par = dev(np.array([7, m, 0, 0], np.int32))
        ya = dev(np.zeros((T, C_), np.float32)); qa = dev(np.zeros((T * heads, 128), np.float32))
        call('camx_op_gdn_conv', ptr(wd), ptr(s1), ptr(xd), ptr(par), ptr(ya), ptr(xp1), I(C_), I(T))
        call('camx_op_gdn_l2', ptr(ya), ptr(qa), I(heads), I(128), F(RS), I(C_), I(T))
        yb = dev(np.full((T, C_), 3, np.float32)); qb = dev(np.full((T * heads, 128), 3, np.float32))
        call('camx_op_gdn_conv_l2', ptr(wd), ptr(s2), ptr(xd), ptr(par), ptr(yb), ptr(xp2), ptr(qb), I(C_), I(T), I(heads), F(RS))
        assert torch.equal(ya, yb) and torch.equal(qa, qb) and torch.equal(s1, s2) and torch.equal(xp1, xp2), f'pass {step}'
        assert bits_equal(host(qb), O.gdn_l2(host(yb), T, heads, 128, 1e-6, ldx=C_))
        m = int(rng.integers(0, T + 1))


@pytest.mark.parametrize('C_,T,heads,H', [(10240, 16, 32, 48), (10240, 1, 32, 48), (256, 4, 2, 3), (1024, 7, 5, 300)])
def test_op_gdn_conv_l2_gates_equals_the_three_tape_ops(C_, T, heads, H):
    """OP_GDN_GATES beside OP_GDN_CONV -> OP_GDN_L2 in one launch: every output and the carried state as the separate tape ops leave them"""
    rng = np.random.default_rng(C_ + T + H)
    w = rng.standard_normal((C_, 4)).astype(np.float32); st0 = rng.standard_normal((C_, 3)).astype(np.float32)
    junk = rng.standard_normal((T, C_)).astype(np.float32)
    dt = rng.standard_normal(H).astype(np.float32); A = -np.abs(rng.standard_normal(H)).astype(np.float32)
    wd, dtd, Ad = dev(w), dev(dt), dev(A)
    s1, s2 = dev(st0), dev(st0); xp1, xp2 = dev(junk), dev(junk)
    m = 0
    for step in range(3):
        x = outliers(rng, (T, C_)); xd = dev(x); al = outliers(rng, (T, H)) * np.float32(8); be = outliers(rng, (T, H)); ald, bed = dev(al), dev(be)
        par = dev(np.array([7, m, 0, 0], np.int32))
        ya = dev(np.zeros((T, C_), np.float32)); qa = dev(np.zeros((T * heads, 128), np.float32)); ga = dev(np.zeros((T, 2 * H), np.float32))
        call('camx_op_gdn_gates', ptr(ald), ptr(bed), ptr(dtd), ptr(Ad), ptr(ga), I(H), I(T))
        call('camx_op_gdn_conv_l2', ptr(wd), ptr(s1), ptr(xd), ptr(par), ptr(ya), ptr(xp1), ptr(qa), I(C_), I(T), I(heads), F(RS))
        yb = dev(np.full((T, C_), 3, np.float32)); qb = dev(np.full((T * heads, 128), 3, np.float32)); gb = dev(np.full((T, 2 * H), 3, np.float32))
        call('camx_op_gdn_conv_l2_gates', ptr(wd), ptr(s2), ptr(xd), ptr(par), ptr(yb), ptr(xp2), ptr(qb), I(C_), I(T), I(heads), F(RS),
             ptr(ald), ptr(bed), ptr(dtd), ptr(Ad), ptr(gb), I(H))
        assert torch.equal(ya, yb) and torch.equal(qa, qb) and torch.equal(ga, gb) and torch.equal(s1, s2) and torch.equal(xp1, xp2), f'pass {step}'
        m = int(rng.integers(0, T + 1))
    assert close_fp32(host(gb), O.gdn_gates(al, be, dt, A))
    L = camx(); p = lambda t: C.c_void_p(t.data_ptr())
    args = [p(wd), p(s2), p(xd), p(par), p(yb), p(xp2), p(qb), I(C_), I(T), I(heads), F(RS), p(ald), p(bed), p(dtd), p(Ad), p(gb), I(H)]
    for i, bad in ((11, NULL), (15, NULL), (16, I(0)), (7, I(C_ + 64))):
        a2 = list(args); a2[i] = bad
        assert L.camx_op_gdn_conv_l2_gates(*a2, stream()) == 1


# ---- the dense Q8 line: QK-norm + partial rotary + Hadamard + Q8 blocks ---------------------------------------------------------------
def _dense_q8_inputs(rng, T, nh, nkv):
    q = outliers(rng, (T * nh, 512)); k = outliers(rng, (T, nkv * 256)); v = outliers(rng, (T, nkv * 256))
    qn = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32); kn = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
    return q, k, v, qn, kn


def _dense_q8_separate(qd, kd, vd, qnd, knd, nh, nkv, nrot, ts, pos0, T, rows, fill=0xa5):
    """the six launches of the reference's chain, through their own entry points"""
    M = nkv * 256; rb = 2 * (M // 32) * 34
    ko = dev(np.zeros((T * nkv, 256), np.float32)); qo = dev(np.zeros((T * nh, 256), np.float32)); vr = vd.clone()
    cache = dev(np.full((rows, rb), fill, np.uint8)); err = dev(np.zeros(1, np.int32))
    call('camx_pf_qk_nr', ptr(kd), I(256), I(nkv), ptr(knd), I(256), I(nrot), F(ts), F(1e-6), I(pos0), ptr(ko), I(T), I(0))
    call('camx_pf_hadamard', ptr(ko), I(T * nkv), I(256), I(1))
    call('camx_pf_hadamard', ptr(vr), I(T * M // 64), I(64), I(1))
    call('camx_own_kv_q8_append', ptr(ko), I(M), ptr(vr), I(M), I(M), ptr(cache), I(pos0), I(rows), ptr(err), I(T))
    call('camx_pf_qk_nr', ptr(qd), I(512), I(nh), ptr(qnd), I(256), I(nrot), F(ts), F(1e-6), I(pos0), ptr(qo), I(T), I(0))
    call('camx_pf_hadamard', ptr(qo), I(T * nh), I(256), I(1))
    return qo, cache, err


@pytest.mark.parametrize('T,nh,nkv,nrot,pos0', [(16, 24, 4, 64, 40000), (1, 24, 4, 64, 65535), (3, 5, 3, 256, 7), (2, 1, 1, 16, 0), (4096, 24, 4, 64, 100), (700, 8, 2, 128, 60000)])
def test_qk_nr_q8_equals_the_six_launches(T, nh, nkv, nrot, pos0):
    rng = np.random.default_rng(1004 + T + nh)
    q, k, v, qn, kn = _dense_q8_inputs(rng, T, nh, nkv)
    ts = _theta(1e7, nrot); rows = pos0 + T + 3
    qd, kd, vd, qnd, knd = (dev(a) for a in (q, k, v, qn, kn))
    qo1, c1, e1 = _dense_q8_separate(qd, kd, vd, qnd, knd, nh, nkv, nrot, ts, pos0, T, rows)
    M = nkv * 256; rb = 2 * (M // 32) * 34
    for mode in ('host', 'device', 'array'):
        qo2 = dev(np.full((T * nh, 256), 9, np.float32)); c2 = dev(np.full((rows, rb), 0xa5, np.uint8)); e2 = dev(np.zeros(1, np.int32))
        pd = dev(np.array([pos0], np.int32)) if mode == 'device' else None
        pa = dev((pos0 + np.arange(T)).astype(np.int32)) if mode == 'array' else None
        call('camx_qk_nr_q8', ptr(qd), I(512), I(nh), ptr(kd), I(M), ptr(vd), I(M), I(nkv), ptr(qnd), ptr(knd), I(nrot), F(ts), F(1e-6),
             I(pos0 if mode == 'host' else 0), ptr(pd), ptr(pa), ptr(qo2), ptr(c2), I(rows), ptr(e2), I(T))
        assert torch.equal(qo1, qo2) and torch.equal(c1, c2) and int(host(e2)[0]) == int(host(e1)[0]) == 0, mode
    assert torch.equal(vd, dev(v))                                  # the fused launch leaves v alone (the chain rotates it in place)
    if T <= 16:                                                     # the oracle's composition: q within the rotary tolerance behind a Hadamard transform
        rq, rc, rerr = O.qk_nr_q8(q, 512, nh, k, v, nkv, qn, kn, nrot, ts, 1e-6, pos0 + np.arange(T), np.full((rows, rb), 0xa5, np.uint8), rows)
        assert rerr == 0 and close_fp32(host(qo2), rq, floor=HADAMARD_FLOOR)
        got = host(c2).reshape(rows, rb)
        assert bits_equal(got[:pos0], rc.reshape(rows, rb)[:pos0]) and bits_equal(got[pos0 + T:], rc.reshape(rows, rb)[pos0 + T:])    # rows outside the span untouched
        assert bits_equal(got[:, M // 32 * 34:], rc.reshape(rows, rb)[:, M // 32 * 34:])          # V: no transcendental before the codec, exact
        # K: exact from the fp32 rotary output on; take that from the separate kernel (held to the oracle by its own test)
        ko = dev(np.zeros((T * nkv, 256), np.float32))
        call('camx_pf_qk_nr', ptr(kd), I(256), I(nkv), ptr(knd), I(256), I(nrot), F(ts), F(1e-6), I(pos0), ptr(ko), I(T), I(0))
        kb, ok = O.kv_q8_encode(O.hadamard_n(host(ko), 256).reshape(-1, 32))
        assert ok.all() and bits_equal(got[pos0:pos0 + T, :M // 32 * 34], kb.reshape(T, -1))


def test_qk_nr_q8_refusals():
    rng = np.random.default_rng(5)
    T, nh, nkv, nrot, rows = 6, 4, 2, 64, 10
    q, k, v, qn, kn = _dense_q8_inputs(rng, T, nh, nkv)
    v[1, 300] = np.inf                                              # one V block of token 1 is refused; its 34 bytes stay
    k[2, 5] = np.nan                                                # a NaN in a k head poisons the whole head's 8 blocks (norm, then the transform)
    ts = _theta(1e7, nrot); M = nkv * 256; rb = 2 * (M // 32) * 34
    pos = np.array([3, 9, 0, 10, -1, 5], np.int32)                  # tokens 3 and 4 sit outside [0, 10)
    qd, kd, vd, qnd, knd = (dev(a) for a in (q, k, v, qn, kn))
    qo = dev(np.zeros((T * nh, 256), np.float32)); c = dev(np.full((rows, rb), 0xa5, np.uint8)); e = dev(np.zeros(1, np.int32))
    call('camx_qk_nr_q8', ptr(qd), I(512), I(nh), ptr(kd), I(M), ptr(vd), I(M), I(nkv), ptr(qnd), ptr(knd), I(nrot), F(ts), F(1e-6), I(0), NULL, ptr(dev(pos)),
         ptr(qo), ptr(c), I(rows), ptr(e), I(T))
    rq, rc, rerr = O.qk_nr_q8(q, 512, nh, k, v, nkv, qn, kn, nrot, ts, 1e-6, pos, np.full((rows, rb), 0xa5, np.uint8), rows)
    assert int(host(e)[0]) == rerr == 3
    got = host(c).reshape(rows, rb); want = rc.reshape(rows, rb)
    assert bits_equal(got[:, M // 32 * 34:], want[:, M // 32 * 34:])                                # V blocks, the refused one untouched
    written = got[:, :M // 32 * 34] != 0xa5
    assert not written[[1, 2, 4, 6, 7, 8]].any()                                                       # rows no token goes to
    assert (got[0, :8 * 34] == 0xa5).all() and not (got[0, 8 * 34:M // 32 * 34] == 0xa5).all()       # token 2's first k head refused, its second written
    assert close_fp32(host(qo), rq, floor=HADAMARD_FLOOR)                                              # every q row is written, also of the tokens outside


@pytest.mark.parametrize('io', [0, 1])
@pytest.mark.parametrize('T,nh,nkv,D,nrot', [(16, 24, 4, 256, 64), (1, 24, 4, 256, 64), (3, 5, 2, 128, 128), (2, 3, 1, 96, 32), (300, 8, 2, 256, 64), (520, 24, 4, 256, 64), (400, 32, 4, 128, 128)])
def test_qk_nr_qk_equals_two_launches(T, nh, nkv, D, nrot, io):
    rng = np.random.default_rng(T + nh + D)
    qs, ks = 2 * D, D + (8 if D % 8 == 0 else 4)
    xq = outliers(rng, (T * nh, qs)); xk = outliers(rng, (T * nkv, ks))
    wq = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32); wk = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    ts = _theta(1e7, nrot); pos = rng.integers(0, 65536, T).astype(np.int32)
    dt = np.uint16 if io else np.float32
    xqd, xkd = dev(O.f2bf(xq) if io else xq), dev(O.f2bf(xk) if io else xk)
    wqd, wkd, posd = dev(wq), dev(wk), dev(pos)
    oq1 = dev(np.zeros((T * nh, D), dt)); ok1 = dev(np.zeros((T * nkv, D), dt))
    call('camx_qk_nr_pos', ptr(xqd), I(qs), I(nh), ptr(wqd), I(D), I(nrot), F(ts), F(1e-6), ptr(posd), ptr(oq1), I(T), I(io))
    call('camx_qk_nr_pos', ptr(xkd), I(ks), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6), ptr(posd), ptr(ok1), I(T), I(io))
    oq2 = dev(np.full((T * nh, D), 5, dt)); ok2 = dev(np.full((T * nkv, D), 5, dt))
    call('camx_qk_nr_qk', ptr(xqd), I(qs), I(nh), ptr(wqd), ptr(xkd), I(ks), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6), I(0), NULL, ptr(posd),
         ptr(oq2), ptr(ok2), I(T), I(io))
    assert torch.equal(oq1, oq2) and torch.equal(ok1, ok2)
    # contiguous positions from a device word and from the host
    p0 = 1234
    call('camx_pf_qk_nr', ptr(xqd), I(qs), I(nh), ptr(wqd), I(D), I(nrot), F(ts), F(1e-6), I(p0), ptr(oq1), I(T), I(io))
    call('camx_pf_qk_nr', ptr(xkd), I(ks), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6), I(p0), ptr(ok1), I(T), I(io))
    for pd, ph in ((dev(np.array([p0], np.int32)), 0), (None, p0)):
        call('camx_qk_nr_qk', ptr(xqd), I(qs), I(nh), ptr(wqd), ptr(xkd), I(ks), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6), I(ph), ptr(pd), NULL,
             ptr(oq2), ptr(ok2), I(T), I(io))
        assert torch.equal(oq1, oq2) and torch.equal(ok1, ok2)


@pytest.mark.parametrize('work', [0, 1])
@pytest.mark.parametrize('T,nh,nkv,D,nrot', [(1, 32, 4, 128, 128), (16, 24, 4, 256, 64), (3, 5, 2, 96, 32), (2, 3, 1, 512, 64), (5, 2, 3, 32, 8), (300, 8, 2, 128, 128), (300, 16, 2, 128, 64), (520, 24, 1, 256, 64)])
def test_qk_nr_kv_equals_the_three_tape_ops(T, nh, nkv, D, nrot, work):
    """q and k norm + rotary and the cache append in one launch against OP_QK_NR (k), OP_KV_APPEND, OP_QK_NR (q) one after another:
    the fp32 outputs and every byte of the cache (fp16 rows and q8_0 rows), with the position on the device, on the host, per row,
    and with tokens that fall outside the cache."""
    rng = np.random.default_rng(T + nh + D + work)
    M = nkv * D; qs, ks, ldv = 2 * D, D + 8, M + 4
    xq = outliers(rng, (T * nh, qs)); xk = outliers(rng, (T * nkv, ks)); xv = outliers(rng, (T, ldv))
    wq = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32); wk = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    ts = _theta(1e7, nrot); eb = int(np.array([1e-6], np.float32).view(np.int32)[0])
    xqd, xkd, xvd, wqd, wkd = dev(xq), dev(xk), dev(xv), dev(wq), dev(wk)
    vc = dev(np.ascontiguousarray(xv[:, :M]))                          # OP_KV_APPEND reads v at stride M
    rows = 40 + T; rb = 2 * M * 2 if work == 0 else 2 * (M // 32) * 34
    def three(p0):
        pd = dev(np.array([p0], np.int32))
        oq = dev(np.zeros((T * nh, D), np.float32)); ok = dev(np.zeros((T * nkv, D), np.float32))
        c = dev(np.full((rows, rb), 0xa5, np.uint8)); e = dev(np.zeros(1, np.int32))
        call('camx_op_qk_nr', ptr(xkd), I(ks), I(nkv), I(D), ptr(wkd), ptr(pd), ptr(ok), I(nrot), F(ts), I(eb), I(T))
        call('camx_op_kv_append', ptr(ok), ptr(vc), ptr(c), ptr(pd), I(M), I(work), ptr(e), I(rows), I(T))
        call('camx_op_qk_nr', ptr(xqd), I(qs), I(nh), I(D), ptr(wqd), ptr(pd), ptr(oq), I(nrot), F(ts), I(eb), I(T))
        return oq, ok, c, int(host(e)[0])
    for p0 in (0, 17, 40, 40 + T - 1 if T > 1 else 39):              # the last ones push tokens past the cache's end
        oq1, ok1, c1, e1 = three(p0)
        assert e1 == (1 if p0 + T > rows else 0)
        for pd, ph, keep in ((dev(np.array([p0], np.int32)), 0, True), (None, p0, True), (None, p0, False)):
            oq2 = dev(np.full((T * nh, D), 5, np.float32)); ok2 = dev(np.full((T * nkv, D), 5, np.float32))
            c2 = dev(np.full((rows, rb), 0xa5, np.uint8)); e2 = dev(np.zeros(1, np.int32))
            call('camx_qk_nr_kv', ptr(xqd), I(qs), I(nh), ptr(wqd), ptr(xkd), I(ks), ptr(xvd), I(ldv), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6),
                 I(ph), ptr(pd), NULL, ptr(oq2), ptr(ok2) if keep else NULL, ptr(c2), I(work), I(rows), ptr(e2), I(T))
            assert torch.equal(oq1, oq2) and torch.equal(c1, c2) and int(host(e2)[0]) == e1
            assert torch.equal(ok1, ok2) if keep else bool((ok2 == 5).all())
    # against the oracle's composition: the fp32 outputs within the rotary's tolerance, and the cache bytes that follow from the launch's own k
    oq2 = dev(np.zeros((T * nh, D), np.float32)); ok2 = dev(np.zeros((T * nkv, D), np.float32)); c2 = dev(np.full((rows, rb), 0xa5, np.uint8)); e2 = dev(np.zeros(1, np.int32))
    call('camx_qk_nr_kv', ptr(xqd), I(qs), I(nh), ptr(wqd), ptr(xkd), I(ks), ptr(xvd), I(ldv), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6),
         I(17), NULL, NULL, ptr(oq2), ptr(ok2), ptr(c2), I(work), I(rows), ptr(e2), I(T))
    c0 = np.full((rows, rb), 0xa5, np.uint8)
    wq_, wk_, wc, werr = O.qk_nr_kv(xq, qs, nh, wq, xk, ks, xv[:, :M], nkv, wk, D, nrot, ts, 1e-6, 17, T, c0.view(np.uint16) if work == 0 else c0, work == 1, ko=host(ok2))
    assert close_fp32(host(oq2), wq_) and close_fp32(host(ok2), wk_) and werr == 0 and int(host(e2)[0]) == 0
    assert bits_equal(host(c2).reshape(-1), np.ascontiguousarray(wc).view(np.uint8).reshape(-1))
    # one position per row (a verify batch): the cache row is the token's position
    pos = rng.permutation(rows + 3)[:T].astype(np.int32) - 1         # distinct; may hold -1 and rows .. rows + 1
    posd = dev(pos)
    oq1 = dev(np.zeros((T * nh, D), np.float32)); ok1 = dev(np.zeros((T * nkv, D), np.float32)); c1 = dev(np.full((rows, rb), 0xa5, np.uint8))
    call('camx_qk_nr_pos', ptr(xqd), I(qs), I(nh), ptr(wqd), I(D), I(nrot), F(ts), F(1e-6), ptr(posd), ptr(oq1), I(T), I(0))
    call('camx_qk_nr_pos', ptr(xkd), I(ks), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6), ptr(posd), ptr(ok1), I(T), I(0))
    bad = False
    for t in range(T):
        if 0 <= pos[t] < rows:
            e = dev(np.zeros(1, np.int32))
            call('camx_op_kv_append', ptr(ok1[t * nkv:(t + 1) * nkv]), ptr(vc[t:t + 1]), ptr(c1), ptr(posd[t:t + 1]), I(M), I(work), ptr(e), I(rows), I(1))
            assert int(host(e)[0]) == 0
        else:
            bad = True
    oq2 = dev(np.full((T * nh, D), 5, np.float32)); ok2 = dev(np.full((T * nkv, D), 5, np.float32))
    c2 = dev(np.full((rows, rb), 0xa5, np.uint8)); e2 = dev(np.zeros(1, np.int32))
    call('camx_qk_nr_kv', ptr(xqd), I(qs), I(nh), ptr(wqd), ptr(xkd), I(ks), ptr(xvd), I(ldv), I(nkv), ptr(wkd), I(D), I(nrot), F(ts), F(1e-6),
         I(0), NULL, ptr(posd), ptr(oq2), ptr(ok2), ptr(c2), I(work), I(rows), ptr(e2), I(T))
    assert torch.equal(oq1, oq2) and torch.equal(ok1, ok2) and torch.equal(c1, c2) and int(host(e2)[0]) == (1 if bad else 0)


def test_qk_nr_kv_refusals():
    D, nh, nkv, T = 128, 4, 2, 2; M = nkv * D
    L = camx(); p = lambda t: C.c_void_p(t.data_ptr())
    q = dev(np.zeros((T * nh, D), np.float32)); k = dev(np.zeros((T * nkv, D), np.float32)); v = dev(np.zeros((T, M), np.float32)); w = dev(np.ones(D, np.float32))
    qo = dev(np.zeros((T * nh, D), np.float32)); c = dev(np.zeros((8, 4 * M), np.uint8)); e = dev(np.zeros(1, np.int32))
    def rc(**kw):
        a = dict(q=p(q), qs=D, k=p(k), ks=D, v=p(v), ldv=M, D=D, nrot=64, pos0=0, cache=p(c), work=0, rows=8, err=p(e), T=T)
        a.update(kw)
        r = L.camx_qk_nr_kv(a['q'], I(a['qs']), I(nh), p(w), a['k'], I(a['ks']), a['v'], I(a['ldv']), I(nkv), p(w), I(a['D']), I(a['nrot']), F(1e-4), F(1e-6),
                            I(a['pos0']), NULL, NULL, p(qo), NULL, a['cache'], I(a['work']), I(a['rows']), a['err'], I(a['T']), stream())
        torch.cuda.synchronize()
        return r
    assert rc() == 0 and rc(T=0) == 0 and rc(work=1) == 0
    for kw in (dict(D=126), dict(D=80, work=1), dict(qs=D + 2), dict(ks=D - 4), dict(ldv=M - 4), dict(nrot=D + 2), dict(nrot=3), dict(work=2), dict(rows=0),
               dict(pos0=-1), dict(pos0=0x7fffffff), dict(cache=NULL), dict(err=NULL), dict(q=C.c_void_p(q.data_ptr() + 4)), dict(cache=C.c_void_p(c.data_ptr() + 2)),
               dict(T=-1)):
        assert rc(**kw) == 1, kw


# ---- tape-shaped entry points: the position is a device word --------------------------------------------------------------------------
@pytest.mark.parametrize('T,heads,D,nrot,stride', [(1, 24, 256, 64, 512), (16, 4, 256, 64, 256), (3, 5, 128, 128, 128), (2, 3, 96, 32, 100), (600, 8, 256, 64, 256)])
def test_op_qk_nr_reads_its_position_on_the_device(T, heads, D, nrot, stride):
    rng = np.random.default_rng(D + T)
    x = outliers(rng, (T * heads, stride)); w = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32); ts = _theta(1e7, nrot)
    xd, wd = dev(x), dev(w)
    pd = dev(np.array([0], np.int32))
    eb = int(np.array([1e-6], np.float32).view(np.int32)[0])
    for p0 in (0, 777, 65000):
        a = dev(np.zeros((T * heads, D), np.float32)); b = dev(np.ones((T * heads, D), np.float32))
        call('camx_pf_qk_nr', ptr(xd), I(stride), I(heads), ptr(wd), I(D), I(nrot), F(ts), F(1e-6), I(p0), ptr(a), I(T), I(0))
        pd.fill_(p0)
        call('camx_op_qk_nr', ptr(xd), I(stride), I(heads), I(D), ptr(wd), ptr(pd), ptr(b), I(nrot), F(ts), I(eb), I(T))
        assert torch.equal(a, b)
    assert close_fp32(host(b), O.qk_nr(x, stride, heads, w, D, nrot, ts, 1e-6, 65000, T))


@pytest.mark.parametrize('M,T', [(1024, 1), (512, 16), (64, 3), (512, 1100)])
def test_op_kv_append_three_row_formats(M, T):
    rng = np.random.default_rng(M + T)
    k = outliers(rng, (T, M)); v = outliers(rng, (T, M)); kd, vd = dev(k), dev(v)
    rows = T + 9; p0 = 5
    pd = dev(np.array([p0], np.int32))
    for work, entry, rbytes in ((0, 'camx_q35p_kv_append16', 4 * M), (1, 'camx_pf_kv_append', 2 * (M // 32) * 34), (2, 'camx_own_kv_q8_append', 2 * (M // 32) * 34)):
        c1 = dev(np.full((rows, rbytes), 0x5a, np.uint8)); c2 = dev(np.full((rows, rbytes), 0x5a, np.uint8)); e1 = dev(np.zeros(1, np.int32)); e2 = dev(np.zeros(1, np.int32))
        if work == 0: call(entry, ptr(kd), I(M), ptr(vd), I(M), ptr(c1), I(M), I(p0), I(rows), ptr(e1), I(T))
        else: call(entry, ptr(kd), I(M), ptr(vd), I(M), I(M), ptr(c1), I(p0), I(rows), ptr(e1), I(T))
        call('camx_op_kv_append', ptr(kd), ptr(vd), ptr(c2), ptr(pd), I(M), I(work), ptr(e2), I(rows), I(T))
        assert torch.equal(c1, c2) and int(host(e1)[0]) == int(host(e2)[0]) == 0, work
        assert (host(c2)[:p0] == 0x5a).all() and (host(c2)[p0 + T:] == 0x5a).all()
        # a position word that runs the pass over the end of the cache: bit 1, the rows inside are written, nothing else
        pd2 = dev(np.array([rows - 1], np.int32)); c3 = dev(np.full((rows, rbytes), 0x5a, np.uint8)); e3 = dev(np.zeros(1, np.int32))
        call('camx_op_kv_append', ptr(kd), ptr(vd), ptr(c3), ptr(pd2), I(M), I(work), ptr(e3), I(rows), I(T))
        assert int(host(e3)[0]) == (1 if T > 1 else 0) and (host(c3)[:rows - 1] == 0x5a).all() and bits_equal(host(c3)[rows - 1], host(c1)[p0])
    # against the oracle's writers
    c = dev(np.zeros((rows, 2 * (M // 32) * 34), np.uint8)); e = dev(np.zeros(1, np.int32))
    call('camx_op_kv_append', ptr(kd), ptr(vd), ptr(c), ptr(pd), I(M), I(2), ptr(e), I(rows), I(T))
    rc, rerr = O.kv_q8_append(k, M, v, M, M, np.zeros((rows, 2 * (M // 32) * 34), np.uint8), p0, T, rows=rows)
    assert rerr == 0 and bits_equal(host(c).reshape(-1), rc.reshape(-1))


@pytest.mark.parametrize('T,nh,D,n', [(16, 24, 256, 64), (1, 24, 256, 64), (3, 5, 256, 256), (7, 12, 128, 128), (300, 24, 256, 64)])
def test_hadamard_gate_mul16_equals_the_two_tape_ops(T, nh, D, n):
    """the attention output's Hadamard and the gate multiply behind it in one launch: out16 and the transformed values carry the bits of
    camx_op_hadamard followed by camx_op_gate_mul16; with a_out NULL the input is left as it was"""
    rng = np.random.default_rng(420 + T + n)
    a = outliers(rng, (T * nh, D)); qg = outliers(rng, (T * nh, 2 * D))
    a1 = dev(a); qgd = dev(qg); y1 = dev(np.zeros((T * nh, D), np.uint16))
    call('camx_op_hadamard', ptr(a1), I(a.size // n), I(n), I(1))
    call('camx_op_gate_mul16', ptr(a1), ptr(qgd), I(2 * D), I(D), ptr(y1), I(a.size), I(D))
    a2 = dev(a); y2 = dev(np.ones((T * nh, D), np.uint16))
    call('camx_op_hadamard_gate_mul16', ptr(a2), ptr(a2), ptr(qgd), I(2 * D), I(D), ptr(y2), I(a.size), I(D), I(n))
    assert torch.equal(y1, y2) and torch.equal(a1, a2)
    a3 = dev(a); y3 = dev(np.ones((T * nh, D), np.uint16))
    call('camx_op_hadamard_gate_mul16', ptr(a3), NULL, ptr(qgd), I(2 * D), I(D), ptr(y3), I(a.size), I(D), I(n))
    assert torch.equal(y1, y3) and bits_equal(host(a3), a)
    ref = O.gate_mul(O.hadamard_n(a, n).reshape(a.shape), qg, D, 2 * D, D, f16=True)
    assert close_16(host(y2, np.uint16), ref, 'f16')
    for bad in ((I(a.size), I(D), I(32)), (I(a.size), I(D + 32), I(n)), (I(a.size - 4), I(D), I(n))):          # a chunk size, a head and a length that do not fit
        p = lambda t: C.c_void_p(t.data_ptr())
        assert camx().camx_op_hadamard_gate_mul16(p(a2), NULL, p(qgd), I(2 * D), I(D), p(y2), *bad, stream()) == 1


@pytest.mark.parametrize('n,slots,T', [(2048, 8, 1), (2048, 1, 1), (4 * 2048, 8, 4), (1000, 3, 2), (37, 64, 1), (16 * 5120, 1, 16)])
def test_op_own_f16_moe_sum_shexp_add_against_the_oracle(n, slots, T):
    """the tape's elementwise ops beside the row ops: OP_OWN_MOE_SUM (slot-ordered fma chain, and the plain adds without weights) and
    OP_OWN_F16 bit for bit, OP_SHEXP_ADD within the gate's exponential"""
    rng = np.random.default_rng(n + slots)
    d = outliers(rng, (slots, n)); w = rng.standard_normal(slots).astype(np.float32); x = outliers(rng, (n,))
    for wt in (w, None):
        xd = dev(x)
        call('camx_op_own_moe_sum', ptr(dev(d)), ptr(dev(wt)) if wt is not None else NULL, ptr(xd), I(n), I(slots))
        assert bits_equal(host(xd), O.own_moe_sum(d, wt, x, slots))
    base = dev(np.concatenate([x, np.zeros(4, np.float32)]))          # an unaligned view: the scalar form
    if n % 4 == 0:
        xu = base[1:1 + n]; xu.copy_(dev(x))
        call('camx_op_own_moe_sum', ptr(dev(d)), ptr(dev(w)), ptr(xu), I(n), I(slots))
        assert bits_equal(host(xu), O.own_moe_sum(d, w, x, slots))
    v = np.concatenate([outliers(rng, (n - 8,)) * np.float32(300), np.array([65504, 65519.99, 65520, 1 + 2.0 ** -11, 2.0 ** -25, -0.0, 1e-8, np.inf], np.float32)]) if n > 8 else x
    y = dev(np.zeros(n, np.uint16))
    call('camx_op_own_f16', ptr(dev(v)), ptr(y), I(n))
    assert bits_equal(host(y, np.uint16), O.own_f16(v))
    moe = outliers(rng, (n,)); sh = outliers(rng, (n,)); lg = (4 * rng.standard_normal(T)).astype(np.float32); out = dev(np.zeros(n, np.float32))
    if n % T == 0:
        call('camx_op_shexp_add', ptr(dev(moe)), ptr(dev(sh)), ptr(dev(lg)), ptr(out), I(n), I(T))
        assert close_fp32(host(out).reshape(T, -1), O.shexp_add(moe, sh, lg, T).reshape(T, -1))
    L = camx(); p = lambda t: C.c_void_p(t.data_ptr())
    assert L.camx_op_own_moe_sum(p(out), NULL, p(out), I(n), I(65), stream()) == 1 and L.camx_op_own_moe_sum(p(out), NULL, p(out), I(n), I(0), stream()) == 1
    assert L.camx_op_shexp_add(p(out), p(out), p(out), p(out), I(n), I(0), stream()) == 1 and L.camx_op_own_f16(NULL, p(y), I(n), stream()) == 1
    if n % 7: assert L.camx_op_shexp_add(p(out), p(out), p(out), p(out), I(n), I(7), stream()) == 1


def test_tape_ops_of_the_gdn_and_gate_rows_equal_their_prefill_namesakes():
    """OP_GDN_GATES, OP_GDN_NORM (+ its q8_1 copy), OP_GDN_NORM16, OP_GATE_MUL (+ q8_1 copy) and OP_ADD_SUM by their Seg fields: the bits of the
    prefill entry points the reference states the same arithmetic in, and the oracle's q8_1 blocks of the stored values"""
    rng = np.random.default_rng(55)
    T, H, S = 3, 48, 128
    al = outliers(rng, (T, H)); be = outliers(rng, (T, H)); dt = rng.standard_normal(H).astype(np.float32); A = -np.abs(rng.standard_normal(H)).astype(np.float32)
    ald, bed, dtd, Ad = dev(al), dev(be), dev(dt), dev(A)
    g1 = dev(np.zeros((T, 2 * H), np.float32)); g2 = dev(np.ones((T, 2 * H), np.float32))
    call('camx_pf_gdn_gates', ptr(ald), I(H), ptr(bed), I(H), ptr(dtd), ptr(Ad), ptr(g1), I(H), I(T))
    call('camx_op_gdn_gates', ptr(ald), ptr(bed), ptr(dtd), ptr(Ad), ptr(g2), I(H), I(T))
    assert torch.equal(g1, g2)
    o = outliers(rng, (T * H, S)); z = outliers(rng, (T * H, S)); w = (1 + 0.1 * rng.standard_normal(S)).astype(np.float32)
    od, zd, wd = dev(o), dev(z), dev(w)
    for silu in (0, 1):
        y1 = dev(np.zeros((T * H, S), np.float32)); y2 = dev(np.ones((T * H, S), np.float32)); q8 = dev(np.zeros(T * H * S // 32 * 36, np.uint8))
        call('camx_pf_gdn_norm', ptr(od), ptr(wd), ptr(zd), ptr(y1), I(S), F(1e-6), L64(T * H), I(silu))
        call('camx_op_gdn_norm', ptr(od), ptr(wd), ptr(zd), ptr(y2), ptr(q8), I(T * H), I(S), F(1e-6), I(silu))
        assert torch.equal(y1, y2) and bits_equal(host(q8).reshape(-1, 36), O.q8_1(host(y2).reshape(-1)))
        y3 = dev(np.ones((T * H, S), np.float32))
        call('camx_op_gdn_norm', ptr(od), ptr(wd), ptr(zd), ptr(y3), NULL, I(T * H), I(S), F(1e-6), I(silu))
        assert torch.equal(y1, y3)
    h1 = dev(np.zeros((T * H, S), np.uint16)); h2 = dev(np.ones((T * H, S), np.uint16))
    call('camx_q35p_gdn_norm16', ptr(od), ptr(wd), ptr(zd), ptr(h1), I(S), F(1e-6), L64(T * H))
    call('camx_op_gdn_norm16', ptr(od), ptr(wd), ptr(zd), ptr(h2), I(T * H), I(S), F(1e-6))
    assert torch.equal(h1, h2)
    nh, D = 24, 256
    a = outliers(rng, (T * nh, D)); qg = outliers(rng, (T * nh, 2 * D)); ad, qgd = dev(a), dev(qg)
    m1 = dev(np.zeros((T * nh, D), np.float32)); m2 = dev(np.ones((T * nh, D), np.float32)); q8 = dev(np.zeros(T * nh * D // 32 * 36, np.uint8))
    call('camx_gate_mul', ptr(ad), ptr(qgd), ptr(m1), L64(a.size), I(D), I(2 * D), I(D), I(0))
    call('camx_op_gate_mul', ptr(ad), ptr(qgd), I(2 * D), I(D), ptr(m2), ptr(q8), I(a.size), I(D))
    assert torch.equal(m1, m2) and bits_equal(host(q8).reshape(-1, 36), O.q8_1(host(m2).reshape(-1)))
    ya = outliers(rng, (5000,)); s1, s2 = dev(ya), dev(ya); aa, bb = dev(outliers(rng, (5000,))), dev(outliers(rng, (5000,)))
    call('camx_pf_add_sum', ptr(aa), ptr(bb), ptr(s1), L64(5000)); call('camx_op_add_sum', ptr(aa), ptr(bb), ptr(s2), I(5000))
    assert torch.equal(s1, s2)
    L = camx(); p = lambda t: C.c_void_p(t.data_ptr())
    assert L.camx_op_gdn_norm(p(od), p(wd), p(zd), p(y1), p(q8), I(T * H), I(S), F(1e-6), I(2), stream()) == 1        # a gate form that does not exist
    assert L.camx_op_gate_mul(p(ad), p(qgd), I(2 * D), I(D), p(m2), p(q8), I(a.size - 8), I(D), stream()) == 1        # a q8_1 copy of a partial block


def test_thin_tape_ops_equal_their_prefill_namesakes():
    rng = np.random.default_rng(31)
    x = outliers(rng, (64, 256)); xa, xb = dev(x), dev(x)
    call('camx_pf_hadamard', ptr(xa), I(64), I(256), I(1)); call('camx_op_hadamard', ptr(xb), I(64), I(256), I(4))
    assert torch.equal(xa, xb)
    T, nh, D = 3, 24, 256
    a = outliers(rng, (T * nh, D)); qg = outliers(rng, (T * nh, 2 * D)); ad, qgd = dev(a), dev(qg)
    y1 = dev(np.zeros((T * nh, D), np.uint16)); y2 = dev(np.ones((T * nh, D), np.uint16))
    call('camx_gate_mul', ptr(ad), ptr(qgd), ptr(y1), L64(a.size), I(D), I(2 * D), I(D), I(1))
    call('camx_op_gate_mul16', ptr(ad), ptr(qgd), I(2 * D), I(D), ptr(y2), I(a.size), I(D))
    assert torch.equal(y1, y2) and close_16(host(y2, np.uint16), O.gate_mul(a, qg, D, 2 * D, D, f16=True), 'f16')
    g = outliers(rng, (6144,)); u = outliers(rng, (6144,)); gd, ud = dev(g), dev(u)
    s1 = dev(np.zeros(6144, np.uint16)); s2 = dev(np.ones(6144, np.uint16))
    call('camx_q3p_swiglu', ptr(gd), ptr(ud), ptr(s1), I(6144)); call('camx_op_own_swiglu16', ptr(gd), ptr(ud), ptr(s2), I(6144))
    assert torch.equal(s1, s2)
    xl = outliers(rng, (T, 10240)); l1 = dev(np.zeros((T * 32, 128), np.float32)); l2 = dev(np.ones((T * 32, 128), np.float32))
    call('camx_pf_gdn_l2', ptr(dev(xl)), ptr(l1), I(32), I(128), I(10240), F(RS), I(T), I(0))
    call('camx_op_gdn_l2', ptr(dev(xl)), ptr(l2), I(32), I(128), F(RS), I(10240), I(T))
    assert torch.equal(l1, l2) and bits_equal(host(l2), O.gdn_l2(xl, T, 32, 128, 1e-6, ldx=10240))
    xc = outliers(rng, (T, 32 * 128)); l3 = dev(np.ones((T * 32, 128), np.float32))
    call('camx_op_gdn_l2', ptr(dev(xc)), ptr(l3), I(32), I(128), F(RS), I(0), I(T))            # x_stride 0: heads * dim
    assert bits_equal(host(l3), O.gdn_l2(xc, T, 32, 128, 1e-6))


@pytest.mark.parametrize('n,q8,yarn', [(1, 1, 0), (1, 0, 0), (7, 1, 1), (16, 0, 1), (2100, 1, 0), (2100, 0, 0)])
def test_op_own_qk_rope_reads_its_position_on_the_device(n, q8, yarn):
    rng = np.random.default_rng(n + q8)
    nh, nkv = 32, 4; ldq = (nh + 2 * nkv) * 128; M = nkv * 128
    from caminus_amd import rope as _rope
    qkv = outliers(rng, (n, ldq)); par = qk_par(rng, yarn_table=_rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None)
    rows = n + 40; p0 = 33
    rbytes = 2 * (M // 32) * 34 if q8 else 4 * M
    qd, pd = dev(qkv), dev(par)
    q1 = dev(np.zeros((n, nh, 128), np.uint16)); c1 = dev(np.full((rows, rbytes), 0x11, np.uint8)); e1 = dev(np.zeros(1, np.int32))
    if q8: call('camx_q3p_qk_rope_q8', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), I(p0), ptr(q1), ptr(c1), ptr(e1), I(n), I(yarn))
    else: call('camx_q3p_qk_rope', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), I(p0), ptr(q1), ptr(c1), I(n), I(yarn))
    pw = dev(np.array([p0], np.int32))
    q2 = dev(np.ones((n, nh, 128), np.uint16)); c2 = dev(np.full((rows, rbytes), 0x11, np.uint8)); e2 = dev(np.zeros(1, np.int32))
    call('camx_op_own_qk_rope', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), ptr(pw), ptr(q2), ptr(c2), I(rows), ptr(e2), I(n), I(yarn), I(q8))
    assert torch.equal(q1, q2) and torch.equal(c1, c2) and int(host(e2)[0]) == 0
    pw.fill_(rows - 1)                                              # the pass runs over the end of the cache: bit 1, q16 still written
    c3 = dev(np.full((rows, rbytes), 0x11, np.uint8)); e3 = dev(np.zeros(1, np.int32)); q3 = dev(np.ones((n, nh, 128), np.uint16))
    call('camx_op_own_qk_rope', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), ptr(pw), ptr(q3), ptr(c3), I(rows), ptr(e3), I(n), I(yarn), I(q8))
    assert int(host(e3)[0]) == (1 if n > 1 else 0) and (host(c3)[:rows - 1] == 0x11).all() and not (host(c3)[rows - 1] == 0x11).all()
    assert not (host(q3) == 1).all(axis=-1).any()


def test_pos0_forms_refuse_a_negative_position():
    L = camx(); z = dev(np.zeros(4096 * 6, np.float32)); par = dev(qk_par(np.random.default_rng(1)))
    p = lambda t: C.c_void_p(t.data_ptr())
    for n in (1, 2048):
        assert L.camx_q3p_qk_rope(p(z), I(768), I(4), I(1), p(par), I(-1), p(z), p(z), I(n), I(0), stream()) == 1
        assert L.camx_q3p_qk_rope_q8(p(z), I(768), I(4), I(1), p(par), I(-1), p(z), p(z), p(z), I(n), I(0), stream()) == 1
        assert L.camx_qk_rope_bf16(p(z), I(768), I(4), I(1), p(par), I(-5), p(z), p(z), I(n), I(0), stream()) == 1
        assert L.camx_q3p_qk_rope(p(z), I(768), I(4), I(1), p(par), I(2 ** 31 - 3), p(z), p(z), I(n + 8), I(0), stream()) == 1
    torch.cuda.synchronize()


# ---- camx_init and a captured decode step whose position lives on the device ----------------------------------------------------------
def test_init_then_graph_replays_at_three_positions():
    from caminus_amd.device import lib as _lib
    L = camx()
    _lib.check(L.camx_init(stream())); _lib.check(L.camx_init(stream()))              # idempotent
    rng = np.random.default_rng(9)
    nh, nkv, T, rows = 24, 4, 1, 64
    q, k, v, qn, kn = _dense_q8_inputs(rng, T, nh, nkv)
    M = nkv * 256; rb = 2 * (M // 32) * 34; ts = _theta(1e7, 64)
    Cc, heads = 1024, 4
    xc = outliers(rng, (T, Cc)); wc = rng.standard_normal((Cc, 4)).astype(np.float32); st0 = rng.standard_normal((Cc, 3)).astype(np.float32)
    gu = O.f2bf(outliers(rng, (T, 2 * 512)))
    qd, kd, vd, qnd, knd, xcd, wcd, gud = (dev(a) for a in (q, k, v, qn, kn, xc, wc, gu))
    pos = dev(np.array([0], np.int32)); par = dev(np.array([0, 0, 0, 0], np.int32))
    qo = dev(np.zeros((T * nh, 256), np.float32)); cache = dev(np.zeros((rows, rb), np.uint8)); err = dev(np.zeros(1, np.int32))
    std = dev(st0); yc = dev(np.zeros((T, Cc), np.float32)); xp = dev(np.zeros((T, Cc), np.float32)); qk = dev(np.zeros((T * heads, 128), np.float32))
    act = dev(np.zeros((T, 512), np.uint16)); mmq = dev(np.zeros(4 * T * 144, np.uint8))
    c16 = dev(np.zeros((rows, 2 * M), np.uint16)); qo2 = dev(np.zeros((T * nh, 256), np.float32)); g16 = dev(np.zeros((T * nh, 256), np.uint16))

    def launch_all():
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        p = lambda t: C.c_void_p(t.data_ptr())
        _lib.check(L.camx_qk_nr_q8(p(qd), I(512), I(nh), p(kd), I(M), p(vd), I(M), I(nkv), p(qnd), p(knd), I(64), F(ts), F(1e-6), I(0), p(pos), NULL, p(qo), p(cache), I(rows), p(err), I(T), s))
        _lib.check(L.camx_op_gdn_conv_l2(p(wcd), p(std), p(xcd), p(par), p(yc), p(xp), p(qk), I(Cc), I(T), I(heads), F(RS), s))
        _lib.check(L.camx_swiglu_mmq_q8_1(p(gud), L64(1024), L64(512), p(mmq), p(act), I(T), I(1), s))     # a table reader: no fill, no wait after camx_init
        _lib.check(L.camx_qk_nr_kv(p(qd), I(512), I(nh), p(qnd), p(kd), I(256), p(vd), I(M), I(nkv), p(knd), I(256), I(64), F(ts), F(1e-6), I(0), p(pos), NULL, p(qo2), NULL,
                                   p(c16), I(0), I(rows), p(err), I(T), s))
        _lib.check(L.camx_op_hadamard_gate_mul16(p(qo2), NULL, p(qd), I(512), I(256), p(g16), I(T * nh * 256), I(256), I(64), s))

    def reset():
        cache.zero_(); err.zero_(); std.copy_(dev(st0))
        for t in (qo, yc, xp, qk, act, mmq, c16, qo2, g16): t.zero_()
        torch.cuda.synchronize()

    def snapshot():
        torch.cuda.synchronize()
        return [host(t).copy() for t in (qo, cache, err, std, yc, xp, qk, act, mmq, c16, qo2, g16)]

    eager = {}
    for p0 in (5, 40, 63):
        reset(); pos.fill_(p0); launch_all(); eager[p0] = snapshot()
        assert eager[p0][1][p0].any() and not eager[p0][1][:p0].any() and eager[p0][9][p0].any() and not eager[p0][9][:p0].any()
    reset(); pos.fill_(5)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch_all()
    for p0 in (40, 5, 63, 40):                                      # one capture, replayed after the position word changed
        reset(); pos.fill_(p0)
        torch.zeros(1 << 20, device=qo.device).add_(1.0)
        g.replay()
        for a, b in zip(snapshot(), eager[p0]):
            assert bits_equal(a, b), f'replay at {p0}'


def test_tape_ops_object_and_f16_module():
    """the host mirror: TapeOps' methods (the reference's K3 op methods, launched at once) and Module('prefill_attn_f16').pf_kv_append"""
    from caminus_amd.device.hip import LOADED, Module
    from caminus_amd.engine.k3 import TapeOps
    rng = np.random.default_rng(12)
    T, nh, nkv = 2, 4, 1
    M = nkv * 256; rows = 16
    q, k, v, qn, kn = _dense_q8_inputs(rng, T, nh, nkv)
    qd, kd, vd, qnd, knd = (dev(a) for a in (q, k, v, qn, kn))
    err = dev(np.zeros(1, np.int32)); pos = dev(np.array([3], np.int32))
    ops = TapeOps(T=T, kv_q8_dense=True, kv_error=err)
    ts = _theta(1e7, 64)
    ko = dev(np.zeros((T * nkv, 256), np.float32)); vr = vd.clone(); qo = dev(np.zeros((T * nh, 256), np.float32))
    cache = torch.full((rows * 2 * (M // 32) * 34,), 0x22, dtype=torch.uint8, device=qd.device)
    i0 = ops.qk_nr(kd, 256, nkv, 256, knd, pos, ko, 64, ts, 1e-6)
    ops.hadamard(ko, 256); ops.hadamard(vr, 64)
    ops.kv_append(ko, vr, cache, pos, q8=True)
    ops.qk_nr(qd, 512, nh, 256, qnd, pos, qo, 64, ts, 1e-6); i5 = ops.hadamard(qo, 256)
    assert i5 == i0 + 5
    qo2 = dev(np.zeros((T * nh, 256), np.float32)); cache2 = torch.full_like(cache, 0x22)
    ops.qk_nr_q8(qd, 512, nh, kd, vd, nkv, qnd, knd, pos, qo2, cache2, 64, ts, 1e-6)
    torch.cuda.synchronize()
    assert torch.equal(qo, qo2) and torch.equal(cache, cache2) and int(host(err)[0]) == 0
    with pytest.raises(ValueError): ops.hadamard(qo, 256, rows_per_task=0)
    with pytest.raises(ValueError): TapeOps(T=1, kv_q8_dense=True)
    # the fp16 / q8_0 cache lines: qk_nr(k) -> kv_append and qk_nr(q) against qk_nr_kv
    po = TapeOps(T=T, kv_error=err)
    for q8 in (False, True):
        rb = 2 * (M // 32) * 34 if q8 else 4 * M
        ca = torch.full((rows * rb,), 0x22, dtype=torch.uint8, device=qd.device); cb = torch.full_like(ca, 0x22)
        po.qk_nr(kd, 256, nkv, 256, knd, pos, ko, 64, ts, 1e-6); po.kv_append(ko, vd, ca, pos, q8=q8); po.qk_nr(qd, 512, nh, 256, qnd, pos, qo, 64, ts, 1e-6)
        ko2 = torch.zeros_like(ko); qo2.zero_()
        po.qk_nr_kv(qd, 512, nh, kd, 256, vd, nkv, 256, qnd, knd, pos, qo2, cb, 64, ts, 1e-6, ko=ko2, q8=q8)
        torch.cuda.synchronize()
        assert torch.equal(qo, qo2) and torch.equal(ko, ko2) and torch.equal(ca, cb) and int(host(err)[0]) == 0
    with pytest.raises(ValueError): ops.qk_nr_kv(qd, 512, nh, kd, 256, vd, nkv, 256, qnd, knd, pos, qo2, cb, 64, ts, 1e-6, q8=True)
    # the elementwise tape ops through the host mirror
    xs = dev(outliers(rng, (T * 512,))); ds_ = dev(outliers(rng, (3, T * 512))); ws = dev(rng.standard_normal(3).astype(np.float32)); x0 = host(xs).copy()
    po.own_moe_sum(ds_, xs, slots=3, w=ws); h16 = torch.zeros(T * 512, dtype=torch.float16, device=qd.device); po.own_f16(xs, h16)
    torch.cuda.synchronize()
    want = O.own_moe_sum(host(ds_), host(ws), x0, 3)
    assert bits_equal(host(xs), want) and bits_equal(host(h16.view(torch.int16), np.uint16), O.own_f16(want))
    lg = dev(np.array([0.0, -200.0], np.float32)); so = torch.zeros_like(xs); po.shexp_add(xs, ds_[0], lg, so); po.add_sum(ds_[1], ds_[2], so)
    torch.cuda.synchronize()
    sh_ = want.reshape(T, -1) + np.stack([host(ds_[0]).reshape(T, -1)[0] * np.float32(0.5), np.zeros(512, np.float32)])
    assert bits_equal(host(so), (sh_.reshape(-1) + (host(ds_[1]) + host(ds_[2]))).astype(np.float32))
    # the fp16-cache build of the prefill attention module
    m = Module('prefill_attn_f16'); assert 'prefill_attn_f16' in LOADED
    c16 = torch.zeros((rows, 2 * M), dtype=torch.float16, device=qd.device); e16 = dev(np.zeros(1, np.int32))
    m.pf_kv_append((T,), (256,), kd, I(M), vd, I(M), I(M), c16, I(3), I(rows), e16)
    torch.cuda.synchronize()
    want, werr = O.kv_append16(k, v, M, np.zeros((rows, 2 * M), np.uint16), 3)
    assert werr == 0 and bits_equal(host(c16.view(torch.int16), np.uint16), want)
