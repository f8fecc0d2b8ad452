"""The activation side of the quantized GEMM feed: fp32 rows -> q8_1 blocks in the MMQ layout (144 bytes per 128 values,
[K_pad / 128][ncols] block order), plain, gathered, scattered to expert columns, and fused behind SwiGLU. Mirrors the
quantizer part of the reference's python/caminus/prefill/mmq.py (k_pad :90, y_bytes :94, quantize :245-261,
quantize_scatter :263-276; same arguments, checks and refusals). The quantized GEMMs themselves are not in this library."""
import ctypes

import torch

from ..device.bufcheck import ALIGN, aligned, disjoint, view_bytes   # noqa: F401
from ..device.hip import Module

MATRIX_ROW_PADDING = 512
QK8_1_MMQ, Y_BLOCK = 128, 144
QUANT_BLOCK = 128
Y_TAIL = 18432
D4, DS4 = 0, 1            # per 32 values: fp32 scale / half2(scale, partial sum)


def k_pad(K):
    return -(-int(K) // MATRIX_ROW_PADDING) * MATRIX_ROW_PADDING


def y_bytes(K, ncols):
    """bytes of a quantized activation buffer for ncols columns of K values (K padded to 512, plus the GEMM's tail)"""
    return k_pad(K) // QK8_1_MMQ * int(ncols) * Y_BLOCK + Y_TAIL


class MMQ:
    def __init__(self, device):
        self.dev = torch.device(device)
        with torch.cuda.device(self.dev):
            self.m = Module('camx')

    def _chk_dev(self, t, what):
        if not isinstance(t, torch.Tensor) or t.device != self.dev or not t.is_contiguous():
            raise ValueError(f'mmq: {what} must be a contiguous tensor on {self.dev}')

    def _chk_f32(self, t, what):
        self._chk_dev(t, what)
        if t.dtype != torch.float32:
            raise ValueError(f'mmq: {what} must be float32 (is {t.dtype})')

    def _chk_i32(self, t, n, what):
        self._chk_dev(t, what)
        if t.dtype != torch.int32 or t.numel() < n:
            raise ValueError(f'mmq: {what} must be int32 with >= {n} elements')

    def _launch(self, name, *args, stream=None):
        with torch.cuda.device(self.dev):
            getattr(self.m, name)((1,), (1,), *args, stream=stream)

    def quantize(self, x, K, ncols, y, layout, s01=None, ids=None, stream=None):
        """column c of y = x row (ids[c] if ids else c) (x fp32, row stride s01 floats, default K); the K padding is zeros"""
        K, ncols = int(K), int(ncols); s01 = K if s01 is None else int(s01)
        self._chk_f32(x, 'x'); self._chk_dev(y, 'y')
        if K % 4 or ncols < 1 or s01 < K:
            raise ValueError(f'mmq.quantize: K {K} (a multiple of 4), ncols {ncols}, s01 {s01}')
        if view_bytes(y) < y_bytes(K, ncols):
            raise ValueError(f'mmq.quantize: y holds {view_bytes(y)} B < {y_bytes(K, ncols)}')
        xb = 4 * ((ncols - 1) * s01 + K)
        if view_bytes(x) < xb:
            raise ValueError(f'mmq.quantize: x holds {view_bytes(x)} B < {ncols} rows ({xb} B)')
        if ids is not None: self._chk_i32(ids, ncols, 'ids')
        disjoint('mmq.quantize', dict(x=(x, xb), ids=(ids, 4 * ncols), y=(y, y_bytes(K, ncols))), ('y',))
        self._launch('camx_quantize_mmq_q8_1', x, ids if ids is not None else ctypes.c_void_p(0), y, ctypes.c_int64(K), ctypes.c_int64(s01),
                     ctypes.c_int64(0), ctypes.c_int64(0), ctypes.c_int64(k_pad(K)), ctypes.c_int(ncols), ctypes.c_int(1), ctypes.c_int(0),
                     ctypes.c_int(int(layout)), stream=stream)

    def quantize_scatter(self, x, K, ntok, ids_inv, k, y, layout, s_tok=None, stream=None):
        """each token's row of x quantized once and written to its k compact columns ids_inv[t * k + slot] of y"""
        K, ntok, k = int(K), int(ntok), int(k); s_tok = K if s_tok is None else int(s_tok)
        self._chk_f32(x, 'x'); self._chk_dev(y, 'y'); self._chk_i32(ids_inv, ntok * k, 'ids_inv')
        if K % 4 or ntok < 1 or k < 1 or s_tok < K:
            raise ValueError(f'mmq.quantize_scatter: K {K}, ntok {ntok}, k {k}, s_tok {s_tok}')
        xb = 4 * ((ntok - 1) * s_tok + K)
        if view_bytes(x) < xb:
            raise ValueError(f'mmq.quantize_scatter: x holds {view_bytes(x)} B < {ntok} rows ({xb} B)')
        if view_bytes(y) < y_bytes(K, ntok * k):
            raise ValueError(f'mmq.quantize_scatter: y holds {view_bytes(y)} B < {y_bytes(K, ntok * k)}')
        disjoint('mmq.quantize_scatter', dict(x=(x, xb), ids_inv=(ids_inv, 4 * ntok * k), y=(y, y_bytes(K, ntok * k))), ('y',))
        self._launch('camx_quantize_mmq_q8_1_scatter', x, ids_inv, y, ctypes.c_int64(K), ctypes.c_int64(0), ctypes.c_int64(s_tok), ctypes.c_int64(0),
                     ctypes.c_int64(k_pad(K)), ctypes.c_int(ntok * k), ctypes.c_int(1), ctypes.c_int(k), ctypes.c_int(int(layout)), ctypes.c_int(ntok),
                     stream=stream)

    def swiglu_quantize(self, gu, F, T, y, layout, ld=None, act=None, stream=None):
        """fused: act = bf16(bf16(silu(g)) * u) of gu bf16 [T, ld] = [g (F) | u (F)], quantized as quantize() of the widened
        act; act (optional, bf16 [T, F]) receives the activation itself"""
        F, T = int(F), int(T); ld = 2 * F if ld is None else int(ld)
        self._chk_dev(gu, 'gu'); self._chk_dev(y, 'y')
        if gu.dtype != torch.bfloat16 or F % 4 or T < 1 or ld < 2 * F:
            raise ValueError(f'mmq.swiglu_quantize: gu {gu.dtype}, F {F}, T {T}, ld {ld}')
        if view_bytes(gu) < 2 * ((T - 1) * ld + 2 * F) or view_bytes(y) < y_bytes(F, T):
            raise ValueError(f'mmq.swiglu_quantize: gu holds {view_bytes(gu)} B, y {view_bytes(y)} B < {y_bytes(F, T)}')
        if act is not None and (act.dtype != torch.bfloat16 or act.numel() < T * F):
            raise ValueError('mmq.swiglu_quantize: act must be bf16 [T, F]')
        disjoint('mmq.swiglu_quantize', dict(gu=(gu, 2 * ((T - 1) * ld + 2 * F)), y=(y, y_bytes(F, T)), act=(act, 2 * T * F)), ('y', 'act'))
        self._launch('camx_swiglu_mmq_q8_1', gu, ctypes.c_int64(ld), ctypes.c_int64(F), y, act if act is not None else ctypes.c_void_p(0),
                     ctypes.c_int(T), ctypes.c_int(int(layout)), stream=stream)
