"""Launch wrappers of the batched prefill's row kernels for the dense / hybrid line (qwen35 shapes): the subset of the
reference's python/caminus/prefill/q35own.py Ops that this library provides on top of the own line's - add_rms16 with rows
up to 65536, the IQ2_S embedding rows, the gated GDN norm with fp16 output, the fp16 KV append and the fp16 sigmoid gate
(:130-150, 211-212) - with the same arguments and refusals. GEMMs and attention belong to other kernels and are not here."""
import ctypes

from ..device import hip
from ..engine import k3
from . import q3m_ops

I, F = ctypes.c_int, ctypes.c_float
NULL = ctypes.c_void_p(0)
MODULE = 'q35_prefill'
FMT_IQ2_S = 3


class Ops(q3m_ops.Ops):
    def __init__(self, dev, module=MODULE):
        if module != MODULE:
            raise ValueError(f'q35 Ops: module {module!r} (this library provides {MODULE})')
        super().__init__(dev, module='q3m_prefill')
        self.module = module
        import torch
        with torch.cuda.device(self.dev):
            self.mod35 = hip.Module(MODULE)
            self.camx = hip.Module('camx')

    def emb_iq2s(self, W, rb, vocab, toks, x, n, N):
        """x [n][N] = the IQ2_S embedding rows toks[i] (82-byte blocks; bit for bit the host decoder)"""
        self.camx.camx_emb_gather((int(n),), (256,), W, ctypes.c_long(int(rb)), I(vocab), toks, x, NULL, I(N), I(int(n)), I(FMT_IQ2_S))

    def add_rms16(self, x, nw, eps, h16, n, N, d=None, h=None):
        """per row: x += d (d None: no add); h = rms_norm(x) * nw (fp32, required); h16 its fp16 copy"""
        if N % 256 or not 256 <= N <= 65536:
            raise ValueError(f'q35 add_rms16: N {N} (a multiple of 256)')
        if h is None:
            raise ValueError('q35 add_rms16: h (the fp32 output) is required')
        self.mod35.q35p_add_rms16((int(n),), (256,), x, NULL if d is None else d, nw, F(eps), h, h16, I(N))

    def gdn_norm16(self, o, w, z, y16, n, H, K, eps):
        self.mod35.q35p_gdn_norm16((int(n) * int(H),), (256,), o, w, z, y16, I(K), F(eps))

    def kv_append16(self, k, ldk, v, ldv, cache, M, pos0, n, rows, err):
        """cache rows pos0 .. pos0 + n - 1 = (k, v) as fp16; rows: the positions the cache holds"""
        alloc = cache.numel() // (2 * int(M))
        if not 0 < int(rows) <= alloc:
            raise ValueError(f'q35 kv_append16: rows {rows} of a cache of {alloc}')
        k3.check_span(pos0, n, int(rows), what='q35 kv_append16')
        self.mod35.q35p_kv_append16((int(n),), (256,), k, I(ldk), v, I(ldv), cache, I(M), I(pos0), I(rows), err)

    def gate_mul16(self, a, gate, y16, N, D, stride, off):
        self.mod35.q35p_gate_mul16((min(-(-int(N) // 256), 8192),), (256,), a, gate, y16, ctypes.c_longlong(int(N)), I(D), I(stride), I(off))
