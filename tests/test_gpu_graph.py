"""The entry points under HIP graph capture: a decode-shaped op-set (add + RMSNorm + q8_1, QK-norm + rotary + Q8 rows, SwiGLU)
captured once and replayed, with eager work and synchronizations between the replays; every replay must leave the bytes the
eager launches leave."""
import numpy as np
import pytest

import oracle as O
from gpu_util import F, I, NULL, bits_equal, camx, dev, host, outliers, ptr
from vectors import qk_par

pytestmark = pytest.mark.gpu


def test_decode_opset_graph_replays_equal_eager():
    import ctypes as C
    import torch
    from caminus_amd.device import lib as _lib
    rng = np.random.default_rng(77)
    N, nh, nkv, rows = 2048, 32, 4, 64
    ldq = (nh + 2 * nkv) * 128
    x0 = outliers(rng, (1, N)); d = outliers(rng, (1, 1, N)); nw = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
    qkv = outliers(rng, (1, ldq)); par = qk_par(rng)
    gq = outliers(rng, (8 * 768,)); up = outliers(rng, (8 * 768,))
    xd, dd, nwd, qkvd, pard, gd, ud = (dev(a) for a in (x0, d, nw, qkv, par, gq, up))
    h = dev(np.zeros((1, N), np.float32)); q8 = dev(np.zeros(N // 32 * 36, np.uint8)); q16 = dev(np.zeros((1, nh, 128), np.uint16))
    rb = 2 * (nkv * 128 // 32) * 34
    cache = dev(np.zeros(rows * rb, np.uint8)); err = dev(np.zeros(1, np.int32)); y16 = dev(np.zeros(8 * 768, np.uint16))

    def launch_all(pos):
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        p = lambda t: C.c_void_p(t.data_ptr())
        L = camx()
        _lib.check(L.camx_add_rms_q8_1(p(xd), p(dd), NULL, I(1), p(nwd), F(1e-6), p(h), NULL, p(q8), I(N), I(1), st))
        _lib.check(L.camx_q3p_qk_rope_q8(p(qkvd), I(ldq), I(nh), I(nkv), p(pard), I(pos), p(q16), p(cache), p(err), I(1), I(0), st))
        _lib.check(L.camx_q3p_swiglu(p(gd), p(ud), p(y16), I(8 * 768), st))

    def snapshot():
        torch.cuda.synchronize()
        return [host(t).copy() for t in (xd, h, q8, q16, cache, y16, err)]

    def reset():
        xd.copy_(torch.from_numpy(x0).to(xd.device)); cache.zero_(); err.zero_()
        for t in (h, q8, q16, y16): t.zero_()
        torch.cuda.synchronize()

    reset(); launch_all(5); eager = snapshot()
    assert eager[6][0] == 0 and eager[4].any()
    reset()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        launch_all(5)                                              # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(s)
    reset()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch_all(5)
    for rep in range(4):
        reset()                                                   # eager fills and copies between the replays
        torch.zeros(1 << 20, device=xd.device).add_(1.0)
        g.replay()
        got = snapshot()
        for a, b in zip(got, eager):
            assert bits_equal(a, b), f'replay {rep}'
