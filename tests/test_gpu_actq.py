"""GPU parity of the activation fake-quant forward kernels against the CPU oracle: codes, scales and bf16 values bit-exact
for the plain and RMSNorm sources; the SiLU source carries expf and is compared through its own activation bits."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, L64, NULL, bits_equal, call, dev, host, outliers, ptr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('M,K,qmax', [(5, 896, 7), (3, 2048, 7), (2, 8192, 7), (4, 128, 3), (3, 768, 127)])
def test_actq_fwd(M, K, qmax):
    rng = np.random.default_rng(K + qmax)
    x = outliers(rng, (M, K)); x[0] = 0
    for bf in (False, True):
        src = O.f2bf(x) if bf else x
        ry, rs, rc = O.actq_fwd(src, clip=0.9, qmax=qmax, bf16=bf)
        y = dev(np.zeros((M, K), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, K // 2), np.uint8))
        call('camx_actq_fwd', ptr(dev(src)), I(int(bf)), ptr(y), ptr(s), ptr(c) if qmax <= 7 else NULL, I(K), F(0.9), I(qmax), I(M))
        assert bits_equal(host(s), rs) and bits_equal(host(y, np.uint16), ry)
        if qmax <= 7: assert bits_equal(host(c), rc)


def test_block_entry_fwd():
    rng = np.random.default_rng(11)
    M, d, nab = 6, 896, 8
    x = outliers(rng, (M, d)); nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32); wab = O.f2bf(rng.standard_normal((nab, d)) * 0.05)
    ry, rs, rc, rab, rstd = O.block_entry_fwd(x, nw, wab, 1e-6)
    y = dev(np.zeros((M, d), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, d // 2), np.uint8))
    ab = dev(np.zeros((M, nab), np.uint16)); rstd_d = dev(np.zeros(M, np.float32))
    call('camx_block_entry_fwd', ptr(dev(x)), ptr(dev(nw)), ptr(dev(wab)), I(nab), F(1e-6), ptr(y), ptr(s), ptr(c), ptr(ab), ptr(rstd_d),
         I(d), F(1.0), I(7), I(M))
    assert bits_equal(host(rstd_d), rstd) and bits_equal(host(s), rs) and bits_equal(host(c), rc) and bits_equal(host(y, np.uint16), ry)
    assert bits_equal(host(ab, np.uint16), rab)


def test_silu_mul_actq_fwd():
    rng = np.random.default_rng(12)
    M, Fh = 5, 768
    gu = O.f2bf(outliers(rng, (M, 2 * Fh)))
    y = dev(np.zeros((M, Fh), np.uint16)); s = dev(np.zeros(M, np.float32)); c = dev(np.zeros((M, Fh // 2), np.uint8))
    gud = dev(gu)
    call('camx_silu_mul_actq_fwd', ptr(gud), I(2 * Fh), I(Fh), ptr(y), ptr(s), ptr(c), F(1.0), I(7), I(M))
    # the kernel's own activation, then the exact stages on it
    act = dev(np.zeros((M, Fh), np.uint16))
    call('camx_silu_mul_bf16', ptr(gud), ptr(act), I(Fh), L64(M * Fh))
    ry, rs, rc = O.actq_fwd(host(act, np.uint16), bf16=True)
    assert bits_equal(host(s), rs) and bits_equal(host(c), rc) and bits_equal(host(y, np.uint16), ry)
