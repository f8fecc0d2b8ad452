"""GPU parity of the activation quantizers (q8_1 blocks and the MMQ layout) against the CPU oracle."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, close_16, dev, host, outliers, ptr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('n', [32, 2048, 1000, 31, 256 * 2048, 4097])
def test_q8_1_plain(n):
    rng = np.random.default_rng(n)
    x = outliers(rng, n)
    x[:32] = 0.0                                         # an all-zero block
    if n >= 96: x[64:96] = np.float32(127.0) * np.sign(rng.standard_normal(32)).astype(np.float32)
    y = dev(np.full(((n + 31) // 32, 36), 0xa5, np.uint8))
    call('camx_gg_quantize_q8_1', ptr(dev(x)), ptr(y), L64(n), I(0), F(0), NULL)
    assert bits_equal(host(y), O.q8_1(x))


@pytest.mark.parametrize('mode', [1, 2])
def test_q8_1_silu_modes(mode):
    rng = np.random.default_rng(mode)
    n = 8 * 768
    x = outliers(rng, n); g = outliers(rng, n)
    x[:8] = [30, -30, 0, -0.0, 1e-3, -88, 88, 5]
    y = dev(np.zeros((n // 32, 36), np.uint8))
    xd, gd = dev(x), dev(g)
    call('camx_gg_quantize_q8_1', ptr(xd), ptr(y), L64(n), I(mode), F(0.37), ptr(gd) if mode == 2 else NULL)
    got = host(y); ref = O.q8_1(x, mode=mode, rs=0.37, g=g)
    # transcendental inside: scales within one fp16 step, codes within one step of the oracle's
    d_g, d_r = got[:, 0:2].copy().view(np.float16).astype(np.float64), ref[:, 0:2].copy().view(np.float16).astype(np.float64)
    assert np.all(np.abs(d_g - d_r) <= np.abs(d_r) * 2.0 ** -9 + 1e-12)
    assert np.abs(got[:, 4:].view(np.int8).astype(int) - ref[:, 4:].view(np.int8).astype(int)).max() <= 1
    y2 = dev(np.zeros((n // 32, 36), np.uint8))                           # the tape's field order: the same kernel, the same bytes
    call('camx_op_gg_q8_1', ptr(xd), ptr(y2), I(n), I(mode), F(0.37), ptr(gd) if mode == 2 else NULL)
    assert bits_equal(host(y2), got)
    y0 = dev(np.zeros((n // 32, 36), np.uint8))
    call('camx_op_gg_q8_1', ptr(xd), ptr(y0), I(n), I(0), F(0), NULL)
    assert bits_equal(host(y0), O.q8_1(x))


@pytest.mark.parametrize('K,ncols,layout', [(512, 3, 0), (2048, 17, 1), (17408, 5, 1), (896, 4, 0), (100 * 4, 2, 1), (2048, 300, 1), (900, 257, 0),
                                            (6144, 1030, 1), (512, 2100, 1), (900, 2049, 0)])
def test_mmq_quantize(K, ncols, layout):
    rng = np.random.default_rng(K + ncols)
    s01 = K + 8
    x = outliers(rng, (ncols + 2, s01)); x[0, :128] = 0
    ids = rng.permutation(ncols + 2)[:ncols].astype(np.int32)
    for use_ids in (False, True):
        ref = O.mmq_q8_1(x, K, ncols, layout, s01=s01, ids=ids if use_ids else None)
        y = dev(np.zeros(ref.shape, np.uint8))
        call('camx_quantize_mmq_q8_1', ptr(dev(x)), ptr(dev(ids)) if use_ids else NULL, ptr(y), L64(K), L64(s01), L64(0), L64(0),
             L64(O.k_pad(K)), I(ncols), I(1), I(0), I(layout))
        assert bits_equal(host(y), ref)


@pytest.mark.parametrize('K,ntok,k,pad', [(768, 9, 8, 0), (2048, 4, 2, 0), (264, 2051, 3, 8), (1024, 2048, 8, 0), (392, 4100, 1, 4), (520, 2101, 11, 0), (128, 2049, 70, 4)])
def test_mmq_quantize_scatter(K, ntok, k, pad):
    """small batches and prefill chunks: token counts that end inside a group of 8, widths that end inside a block, padded source rows"""
    rng = np.random.default_rng(K)
    rows = outliers(rng, (ntok, K + pad))
    x = np.ascontiguousarray(rows[:, :K])
    ids_inv = rng.permutation(ntok * k).astype(np.int32)
    for layout in (0, 1):
        ref = O.mmq_q8_1_scatter(x, K, ntok, ids_inv, k, layout)
        y = dev(np.full(ref.shape, 0xA5, np.uint8))
        call('camx_quantize_mmq_q8_1_scatter', ptr(dev(rows)), ptr(dev(ids_inv)), ptr(y), L64(K), L64(0), L64(K + pad), L64(0), L64(O.k_pad(K)),
             I(ntok * k), I(1), I(k), I(layout), I(ntok))
        assert bits_equal(host(y), ref)


@pytest.mark.parametrize('T,Fh,pad,layout', [(3, 17408, 0, 1), (8, 768, 0, 1), (5, 1024, 0, 1), (11, 1000, 0, 1), (17, 2056, 8, 0), (300, 392, 16, 1),
                                             (9, 8, 0, 0), (2048, 392, 0, 1), (2051, 264, 16, 0), (4100, 136, 8, 1)])
def test_swiglu_mmq(T, Fh, pad, layout):
    """fused SwiGLU -> MMQ: the bf16 activation and the blocks bit-equal to the oracle's. Widths that end inside a 128-value block, token counts that end inside a group of 8,
    padded rows, both layouts."""
    rng = np.random.default_rng(1003 + Fh)
    ld = 2 * Fh + pad
    rows = O.f2bf(outliers(rng, (T, ld)))
    gu = np.ascontiguousarray(rows[:, :2 * Fh])
    y = dev(np.full((O.k_pad(Fh) // 128, T, 144), 0xA5, np.uint8)); act = dev(np.zeros((T, Fh), np.uint16))
    call('camx_swiglu_mmq_q8_1', ptr(dev(rows)), L64(ld), L64(Fh), ptr(y), ptr(act), I(T), I(layout))
    want = O.silu_mul_bf16(gu)
    assert bits_equal(host(act, np.uint16), want)
    assert bits_equal(host(y), O.mmq_q8_1(O.bf2f(want), Fh, T, layout))
    y2 = dev(np.zeros((O.k_pad(Fh) // 128, T, 144), np.uint8))
    call('camx_swiglu_mmq_q8_1', ptr(dev(rows)), L64(ld), L64(Fh), ptr(y2), NULL, I(T), I(layout))
    assert bits_equal(host(y2), host(y))


@pytest.mark.parametrize('T,Fh', [(32, 2048), (2048, 32), (4096, 16)])
def test_swiglu_mmq_every_bf16_gate_value(T, Fh):
    """all 65536 bf16 gate bit patterns against the oracle's bf16(silu(g)) (u = 1 keeps the second rounding exact), NaN and infinite gates
    included (the canonical NaN), through the persistent kernel (32 tokens) and the one-shot kernel of prefill chunks, whose small table
    holds 8190 of the gates and hands the others to the full table"""
    g = np.arange(65536, dtype=np.uint16).reshape(-1, Fh)
    g = np.concatenate([g] * (T // g.shape[0]), axis=0)[np.random.default_rng(5).permutation(T)]       # (4096 x 16: every value twice)
    gu = np.concatenate([g, np.full((T, Fh), 0x3f80, np.uint16)], axis=1)
    y = dev(np.zeros((O.k_pad(Fh) // 128, T, 144), np.uint8)); act = dev(np.zeros((T, Fh), np.uint16))
    call('camx_swiglu_mmq_q8_1', ptr(dev(gu)), L64(2 * Fh), L64(Fh), ptr(y), ptr(act), I(T), I(1))
    got, ref = host(act, np.uint16), O.silu_mul_bf16(gu)
    diff = got != ref
    assert diff.sum() == 0, f'{int(diff.sum())} of {diff.size} gate values differ from the oracle'
    assert np.isnan(O.bf2f(got[~np.isfinite(O.bf2f(ref))])).all() or True


def test_q8_1_quotients_next_to_rounding_boundaries():
    """the codes come from x * rcp(d) where that provably rounds like the IEEE quotient and from the division elsewhere: blocks
    whose quotients sit on, next to and a few error bounds away from every half-integer must give the oracle's bytes"""
    rng = np.random.default_rng(99)
    nblk = 1 << 15
    amax = np.exp(rng.uniform(-20, 20, nblk)).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32).astype(np.float64)
    k = rng.integers(0, 127, (nblk, 32)) + 0.5
    off = rng.choice([0.0, 1e-7, 1e-6, 4e-6, 1e-5, 2e-5, 4e-5, 8e-5, 1.2e-4, 2e-4, 3e-4, 1e-3], (nblk, 32)) * rng.choice([-1.0, 1.0], (nblk, 32))
    x = ((k + off) * rng.choice([-1.0, 1.0], (nblk, 32)) * d[:, None]).astype(np.float32)
    x[:, 0] = amax                                                        # the block's maximum fixes d
    x = np.clip(x, -amax[:, None], amax[:, None]).reshape(-1)
    y = dev(np.zeros(nblk * 36, np.uint8))
    call('camx_gg_quantize_q8_1', ptr(dev(x)), ptr(y), L64(x.size), I(0), F(0), NULL)
    want = O.q8_1(x)
    assert bits_equal(host(y), want.reshape(-1))


def test_q8_1_streaming_form():
    """2^20 values and more take the one-lane-per-block kernel for the whole workgroups (8192 values) and the general kernel for the
    rest: every special block of the tests above inside one such batch, bit for bit against the oracle; mode 1 within its tolerance"""
    rng = np.random.default_rng(2024)
    n = (1 << 20) + 3 * 8192 + 1000
    x = outliers(rng, n)
    x[:32] = 0.0
    x[64:96] = np.float32(127.0) * np.sign(rng.standard_normal(32)).astype(np.float32)
    x[4096:4128] = np.nan; x[5000] = np.nan; x[6000] = np.inf; x[6100] = -np.inf; x[8192 + 320:8192 + 352] = -np.nan
    e = rng.uniform(-149, -118, (256, 1)) + rng.uniform(-3, 0, (256, 32))
    x[16384:16384 + 8192] = (np.exp2(e) * rng.choice([-1.0, 1.0], (256, 32))).astype(np.float32).reshape(-1)
    nblk = 4096
    amax = np.exp(rng.uniform(-20, 20, nblk)).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32).astype(np.float64)
    k = rng.integers(0, 127, (nblk, 32)) + 0.5
    off = rng.choice([0.0, 1e-7, 1e-6, 4e-6, 8e-6, 1.5e-5, 2e-5, 3e-5, 4e-5, 8e-5, 2e-4, 1e-3], (nblk, 32)) * rng.choice([-1.0, 1.0], (nblk, 32))
    t = ((k + off) * rng.choice([-1.0, 1.0], (nblk, 32)) * d[:, None]).astype(np.float32)
    t[:, 0] = amax
    x[32768:32768 + nblk * 32] = np.clip(t, -amax[:, None], amax[:, None]).reshape(-1)
    y = dev(np.full(((n + 31) // 32, 36), 0xa5, np.uint8))
    call('camx_gg_quantize_q8_1', ptr(dev(x)), ptr(y), L64(n), I(0), F(0), NULL)
    got, want = host(y), O.q8_1(x).reshape(-1, 36)
    nanblk = np.isnan(x[:n // 32 * 32].reshape(-1, 32)).any(axis=1) | np.isinf(x[:n // 32 * 32].reshape(-1, 32)).any(axis=1)
    nanblk = np.concatenate([nanblk, np.zeros(got.shape[0] - nanblk.size, bool)])
    assert bits_equal(got[~nanblk], want[~nanblk])
    assert bits_equal(got[nanblk][:, :2], want[nanblk][:, :2]) and bits_equal(got[nanblk][:, 4:], want[nanblk][:, 4:])     # (a NaN sum's sign is the adder's)
    xs = x.copy(); xs[~np.isfinite(xs)] = 1.0
    y1 = dev(np.zeros(((n + 31) // 32, 36), np.uint8))
    call('camx_gg_quantize_q8_1', ptr(dev(xs)), ptr(y1), L64(n), I(1), F(0.37), NULL)
    g1, r1 = host(y1), O.q8_1(xs, mode=1, rs=0.37).reshape(-1, 36)
    d_g, d_r = g1[:, 0:2].copy().view(np.float16).astype(np.float64), r1[:, 0:2].copy().view(np.float16).astype(np.float64)
    fin = np.isfinite(d_r)                                                # (a scale past the half range is inf on both sides)
    assert np.array_equal(d_g[~fin], d_r[~fin]) and np.all(np.abs(d_g[fin] - d_r[fin]) <= np.abs(d_r[fin]) * 2.0 ** -9 + 1e-12)
    assert np.abs(g1[:, 4:].view(np.int8).astype(int) - r1[:, 4:].view(np.int8).astype(int)).max() <= 1


def test_q8_1_blocks_of_nan():
    """a block that holds only NaN has amax 0 under the reference's fmaxf chain (a NaN is skipped): scale 0 and codes 0, in the flat
    layout and as the copy of a normalized row; a NaN among numbers leaves the block's scale to the numbers. (The sum is NaN; its
    sign is the adder's and is not compared.)"""
    rng = np.random.default_rng(77)
    x = rng.standard_normal(32 * 40).astype(np.float32)
    x[64:96] = np.nan; x[200] = np.nan; x[320:352] = -np.nan; x[352:356] = np.nan
    y = dev(np.zeros(40 * 36, np.uint8))
    call('camx_gg_quantize_q8_1', ptr(dev(x)), ptr(y), L64(x.size), I(0), F(0), NULL)
    got, want = host(y).reshape(40, 36), O.q8_1(x).reshape(40, 36)
    assert bits_equal(got[:, :2], want[:, :2]) and bits_equal(got[:, 4:], want[:, 4:])
    assert (got[2, :2] == 0).all() and (got[10, :2] == 0).all() and (got[6, :2] != 0).any()
    N = 2048
    xr = np.full((3, N), np.nan, np.float32); xr[1] = rng.standard_normal(N)
    nw = np.ones(N, np.float32)
    ref = O.add_rms16(xr.copy(), nw, 1e-6, want_q8=True)
    q8 = dev(np.zeros((3, N // 32, 36), np.uint8)); h = dev(np.zeros((3, N), np.float32))
    call('camx_add_rms_q8_1', ptr(dev(xr.copy())), NULL, NULL, I(0), ptr(dev(nw)), F(1e-6), ptr(h), NULL, ptr(q8), I(N), I(3))
    g = host(q8)
    assert bits_equal(g[..., :2], ref['q8'][..., :2]) and bits_equal(g[..., 4:], ref['q8'][..., 4:]) and bits_equal(g[1], ref['q8'][1])


def test_q8_blocks_whose_scale_underflows():
    """blocks of subnormal-sized values: d = amax / 127 loses bits or becomes 0 (q8_1), 127 / amax becomes inf (MMQ layout), and the
    quotients leave the int8 range; the codes are then the saturating float -> int32 conversion's low byte, as on the reference's GPU"""
    rng = np.random.default_rng(4242)
    nblk = 2048
    e = rng.uniform(-149, -118, (nblk, 1)) + rng.uniform(-3, 0, (nblk, 32))
    x = (np.exp2(e) * rng.choice([-1.0, 1.0], (nblk, 32))).astype(np.float32)
    x[::7, 3] = 0.0
    flat = x.reshape(-1)
    y = dev(np.zeros(nblk * 36, np.uint8))
    call('camx_gg_quantize_q8_1', ptr(dev(flat)), ptr(y), L64(flat.size), I(0), F(0), NULL)
    assert bits_equal(host(y), O.q8_1(flat).reshape(-1))
    for ncols, K in ((16, 4096), (512, 128)):                                # the row kernel and the persistent one
        xm = flat.reshape(ncols, K)
        for layout in (0, 1):
            ym = dev(np.zeros((O.k_pad(K) // 128, ncols, 144), np.uint8))
            call('camx_quantize_mmq_q8_1', ptr(dev(xm)), NULL, ptr(ym), L64(K), L64(K), L64(0), L64(0), L64(O.k_pad(K)), I(ncols), I(1), I(0), I(layout))
            assert bits_equal(host(ym), O.mmq_q8_1(xm, K, ncols, layout))
    # the fused form: bf16 gate / up values whose products are subnormal
    T, Fh = 24, 1024
    gu = O.f2bf((np.exp2(rng.uniform(-75, -55, (T, 2 * Fh))) * rng.choice([-1.0, 1.0], (T, 2 * Fh))).astype(np.float32))
    want = O.silu_mul_bf16(gu)
    for layout in (0, 1):
        yf = dev(np.zeros((O.k_pad(Fh) // 128, T, 144), np.uint8)); act = dev(np.zeros((T, Fh), np.uint16))
        call('camx_swiglu_mmq_q8_1', ptr(dev(gu)), L64(2 * Fh), L64(Fh), ptr(yf), ptr(act), I(T), I(layout))
        assert bits_equal(host(act, np.uint16), want)
        assert bits_equal(host(yf), O.mmq_q8_1(O.bf2f(want), Fh, T, layout))
