"""Pins of the oracle's activation fake-quant, forward and backward, against torch on the CPU.

The reference states what its kernels compute (kernels/actq.hip:1-12, python/caminus/train/actq.py:1): under bf16 autocast,
u = bf16(bf16(x) @ H128) per 128-chunk with H the normalized Sylvester matrix in bf16, then in fp32 s = max(amax|u| clip / qmax,
1e-8), y = bf16(clamp(round(u / s), -qmax - 1, qmax) s), a straight-through rounding whose clamp passes no gradient at the
bounds, s not detached. Here that graph is written with torch ops and differentiated by autograd, which derives the backward
on its own: the hand-derived dL/ds, tie split, sign and mask of the oracle must agree with it. The two sides round a few
fp32 sums in different orders, so agreement is bit-equality of nearly all bf16 values and one bf16 step for the rest.
"""
import numpy as np
import torch
import torch.nn.functional as TF

import oracle as O

f32 = np.float32


def _bits(t):
    return t.detach().contiguous().view(torch.int16).numpy().view(np.uint16)


def _bf(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)


def _h128():
    i = np.arange(128)
    sign = 1 - 2 * (np.bitwise_count(i[:, None] & i[None, :]).astype(np.int64) & 1)
    return (torch.from_numpy(sign.astype(f32)) / 128 ** 0.5).to(torch.bfloat16)


def _fake_quant(src, clip, qmax):
    """src: any float tensor [M, K] in the autograd graph -> y bf16 [M, K]"""
    M, K = src.shape
    u = (src.to(torch.bfloat16).view(M, K // 128, 128) @ _h128()).view(M, K)
    uf = u.float()
    s = (uf.abs().amax(-1, keepdim=True) * clip / qmax).clamp_min(1e-8)
    t = uf / s
    r = t.round()
    lo, hi = float(-qmax - 1), float(qmax)
    m = ((r > lo) & (r < hi)).float()
    q = r.clamp(lo, hi)
    q_ste = (q - m * t).detach() + m * t
    return (q_ste * s).to(torch.bfloat16), s[:, 0].detach()


def _agree(got_bits, want_bits, share=0.995, what=''):
    """bf16 bit patterns: nearly all equal, the rest one step apart (or a zero of either sign)"""
    got = O.bf2f(got_bits).astype(np.float64); want = O.bf2f(want_bits).astype(np.float64)
    same = (got_bits == want_bits) | ((got == 0) & (want == 0))
    assert same.mean() >= share, (what, same.mean())
    step = np.maximum(np.abs(want), np.abs(got)) * 2.0 ** -7 + 1e-30
    assert (np.abs(got - want)[~same] <= step[~same] * 1.01).all(), what


def _inputs(seed, M, K, heavy=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K)).astype(f32) * (np.exp(rng.standard_normal((M, 1))).astype(f32) * 3 if heavy else 2)
    g = O.f2bf(rng.standard_normal((M, K)).astype(f32))
    return rng, x, g


def test_forward_against_torch_bf16_graph():
    for seed, (M, K, qmax, clip) in enumerate([(16, 512, 7, 1.0), (8, 2048, 7, 0.9), (8, 896, 127, 1.0), (8, 128, 3, 0.8)]):
        _, x, _ = _inputs(seed, M, K, heavy=seed == 1)
        for bf in (False, True):
            src = O.f2bf(x) if bf else x
            y, s, c = O.actq_fwd(src, clip=clip, qmax=qmax, bf16=bf)
            xt = _bf(src) if bf else torch.from_numpy(x)
            yt, st = _fake_quant(xt, clip, qmax)
            u = O.actq_rotate(O.f2bf(x))
            ut = (_bf(O.f2bf(x)).view(M, K // 128, 128) @ _h128()).view(M, K)
            _agree(u, _bits(ut), 0.999, 'rotation')
            rows = (u == _bits(ut)).all(1)                               # rows whose rotation agrees bit for bit: everything after is exact
            assert rows.sum() >= M // 2
            assert np.array_equal(s[rows], st.numpy()[rows])
            assert np.array_equal(y[rows] & 0x7fff, _bits(yt)[rows] & 0x7fff)    # (the sign of a zero aside: rint keeps -0)
            if qmax <= 7:
                q = np.stack([c & 0xF, c >> 4], -1).reshape(M, K).astype(np.int16); q = np.where(q > 7, q - 16, q)
                want = np.rint(yt.float().numpy() / st.numpy()[:, None])
                assert np.array_equal(q[rows], want[rows])


def test_actq_backward_against_autograd():
    for seed, (M, K, qmax, clip) in enumerate([(16, 512, 7, 1.0), (8, 2048, 7, 0.9), (6, 896, 127, 1.0), (8, 128, 3, 0.8), (4, 8192, 7, 1.0)]):
        _, x, g = _inputs(10 + seed, M, K, heavy=seed == 1)
        x[0, :3] = 0
        for bf in (False, True):
            src = O.f2bf(x) if bf else x
            xt = (_bf(src) if bf else torch.from_numpy(x)).clone().requires_grad_()
            yt, _ = _fake_quant(xt, clip, qmax)
            yt.backward(_bf(g))
            dx = O.actq_bwd(src, g, clip=clip, qmax=qmax, bf16=bf)
            want = _bits(xt.grad) if bf else O.f2bf(xt.grad.numpy())
            got = dx if bf else O.f2bf(dx)
            if not bf: assert np.array_equal(O.bf2f(got), dx)               # fp32 dx carries bf16 values (the matmul's dtype)
            _agree(got, want, 0.99, f'dx K {K} bf16 {bf}')


def test_actq_backward_special_rows():
    """a zero row sits on the scale's floor: only the straight-through term passes (a constant gradient comes back as one
    spike); a single spike rotates to a constant row whose 128 tied maxima share the scale's gradient"""
    K, qmax = 128, 7
    g = O.f2bf(np.ones((1, K), f32))
    dz = O.actq_bwd(np.zeros((1, K), f32), g, qmax=qmax)
    assert dz[0, 0] == O.bf2f(O.f2bf(np.array([128 * 0.08837890625], f32)))[0] and not dz[0, 1:].any()
    x = np.zeros((3, K), f32); x[0, 0] = 4.0; x[1, 5] = -2.0
    gt = O.f2bf(np.random.default_rng(3).standard_normal((3, K)).astype(f32))
    xt = torch.from_numpy(x).clone().requires_grad_()
    yt, _ = _fake_quant(xt, 1.0, qmax); yt.backward(_bf(gt))
    _agree(O.f2bf(O.actq_bwd(x, gt, qmax=qmax)), O.f2bf(xt.grad.numpy()), 0.98, 'ties')


def test_silu_mul_actq_backward_against_autograd():
    for seed, (M, Fh, ld) in enumerate([(12, 768, 1536), (6, 2048, 4096), (5, 256, 640)]):
        rng = np.random.default_rng(20 + seed)
        base = O.f2bf((rng.standard_normal((M, ld)) * 2).astype(f32))
        base[0, :8] = O.f2bf(np.array([30., -30., 0., -0.0, 1e-3, -88., 88., 3.], f32))      # silu extremes (tests/train/test_silu_mul_actq.py:26)
        gu = base[:, :2 * Fh] if ld == 2 * Fh else np.ascontiguousarray(base[:, 64:64 + 2 * Fh])
        g = O.f2bf(rng.standard_normal((M, Fh)).astype(f32))
        gut = _bf(gu).clone().requires_grad_()
        a, b = gut.chunk(2, -1)
        yt, _ = _fake_quant(TF.silu(a) * b, 1.0, 7)
        yt.backward(_bf(g))
        dgu = O.silu_mul_actq_bwd(gu, g)
        _agree(dgu, _bits(gut.grad), 0.99, f'dgu F {Fh}')


def test_block_entry_backward_against_autograd():
    for seed, (M, d, nab, heavy) in enumerate([(16, 896, 14, False), (8, 896, 14, True), (6, 1024, 0, False), (4, 256, 2, False)]):
        rng, x, dy = _inputs(30 + seed, M, d, heavy)
        nw = (rng.random(d) + 0.5).astype(f32)
        wab = O.f2bf((rng.standard_normal((max(nab, 2), d)) / 30).astype(f32))[:nab]
        dab = O.f2bf(rng.standard_normal((M, max(nab, 1))).astype(f32))[:, :nab]
        y, s, c, ab, rstd = O.block_entry_fwd(x, nw, wab if nab else None, 1e-6)
        dx = O.block_entry_bwd(x, nw, rstd, wab if nab else None, dy, dab if nab else None)
        xt = torch.from_numpy(x).clone().requires_grad_()
        h = TF.rms_norm(xt, (d,), torch.from_numpy(nw), 1e-6)
        yt, _ = _fake_quant(h, 1.0, 7)
        outs, grads = [yt], [_bf(dy)]
        if nab:
            hb = h.to(torch.bfloat16)                                    # autocast's cast: each projection's input gradient is rounded to bf16
            half = nab // 2
            outs += [TF.linear(hb, _bf(wab[:half])), TF.linear(hb, _bf(wab[half:]))]
            grads += [_bf(np.ascontiguousarray(dab[:, :half])), _bf(np.ascontiguousarray(dab[:, half:]))]
        torch.autograd.backward(outs, grads)
        want = xt.grad.numpy()
        rel = np.linalg.norm(dx - want, axis=1) / np.linalg.norm(want, axis=1)
        assert rel.max() < 2e-2 and np.median(rel) < 5e-3, (d, nab, rel)   # the reference's own bar is 1e-2 on the whole tensor (tests/train/test_block_entry.py:33)
        # the forward's gate projections against the same graph
        if nab:
            _agree(ab, np.concatenate([_bits(outs[1]), _bits(outs[2])], 1), 0.98, 'ab')
