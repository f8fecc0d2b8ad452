"""Fused activation fake-quant, forward: per row a 128-point Hadamard rotation per chunk in bf16 steps, one scale per row,
int codes packed two per byte. Mirrors the forward entry points of the reference's python/caminus/train/actq.py:24-169
(actq, scales, codes, actq_codes, silu_mul_actq, block_entry; same arguments and results). The backward kernels are not
part of this library: these functions return plain tensors and do not record autograd history."""
import ctypes

import torch

from ..device.hip import Module

_mod = {}


def _m():
    dev = torch.cuda.current_device()
    if dev not in _mod:
        _mod[dev] = Module('actq')
    return _mod[dev]


def _sfx(x):
    if x.dtype == torch.bfloat16: return 'bf16'
    if x.dtype == torch.float32: return 'f32'
    raise TypeError(f'actq: unsupported dtype {x.dtype}')


def _rows(x):
    K = x.shape[-1]
    assert K % 128 == 0 and K <= 8192, K
    return x.reshape(-1, K).contiguous(), K


def _qmax(bits):
    return 2 ** (bits - 1) - 1


def actq(x, bits=4, clip=1.0):
    """bf16 fake-quantized x (same shape)"""
    x2, K = _rows(x); M = x2.shape[0]
    y = torch.empty(M, K, device=x.device, dtype=torch.bfloat16)
    if M:
        getattr(_m(), f'actq_fwd_{_sfx(x2)}')((M,), (256,), x2, y, ctypes.c_void_p(None), ctypes.c_int(K), ctypes.c_float(clip), ctypes.c_int(_qmax(bits)))
    return y.reshape(*x.shape[:-1], K)


def scales(x, bits=4, clip=1.0):
    """the per-row scales [M] fp32"""
    x2, K = _rows(x); M = x2.shape[0]
    y = torch.empty(M, K, device=x.device, dtype=torch.bfloat16); s = torch.empty(M, device=x.device)
    getattr(_m(), f'actq_fwd_{_sfx(x2)}')((M,), (256,), x2, y, s, ctypes.c_int(K), ctypes.c_float(clip), ctypes.c_int(_qmax(bits)))
    return s


def codes(x, bits=4, clip=1.0, dequant=False):
    """(packed codes [M, K / 2] uint8, row scales [M]); dequant=True adds the bf16 values"""
    assert bits <= 4
    x2, K = _rows(x); M = x2.shape[0]
    c = torch.empty(M, K // 2, device=x.device, dtype=torch.uint8); s = torch.empty(M, device=x.device)
    y = torch.empty(M, K, device=x.device, dtype=torch.bfloat16) if dequant else None
    getattr(_m(), f'actq_fwd_codes_{_sfx(x2)}')((M,), (256,), x2, y if y is not None else ctypes.c_void_p(None), s, c, ctypes.c_int(K),
                                                ctypes.c_float(clip), ctypes.c_int(_qmax(bits)))
    return (c, s, y) if dequant else (c, s)


def actq_codes(x, bits=4, clip=1.0):
    """(bf16 fake-quantized x, packed codes [M, K / 2], row scales [M]) from one pass"""
    c, s, y = codes(x, bits, clip, dequant=True)
    return y.reshape(*x.shape[:-1], x.shape[-1]), c, s


def silu_mul_actq(gu, bits=4, clip=1.0):
    """(xq, codes, scales) of act = bf16(bf16(silu(g)) * u) for gu [M, 2F] bf16 = [g | u]; gu may be a row-strided view"""
    M, F2 = gu.shape; Fh = F2 // 2
    assert gu.dtype == torch.bfloat16 and gu.stride(1) == 1 and Fh % 128 == 0 and Fh <= 8192 and bits <= 4
    y = torch.empty(M, Fh, device=gu.device, dtype=torch.bfloat16)
    c = torch.empty(M, Fh // 2, device=gu.device, dtype=torch.uint8); s = torch.empty(M, device=gu.device)
    if M:
        _m().silu_mul_actq_fwd((M,), (256,), gu, ctypes.c_int(gu.stride(0)), ctypes.c_int(Fh), y, s, c, ctypes.c_float(clip), ctypes.c_int(_qmax(bits)))
    return y, c, s


def block_entry(x, nw, wab, eps, bits=4, clip=1.0):
    """(xq, codes, scales, ab) for h = RMSNorm(x; nw, eps) without materializing h; wab bf16 [nab, d] or None"""
    d = x.shape[-1]; x2 = x.reshape(-1, d).contiguous(); M = x2.shape[0]
    assert x2.dtype == torch.float32 and d % 128 == 0 and d <= 1024 and bits <= 4
    nab = 0 if wab is None else wab.shape[0]
    assert nab <= 16 and nab % 2 == 0
    y = torch.empty(M, d, device=x.device, dtype=torch.bfloat16)
    c = torch.empty(M, d // 2, device=x.device, dtype=torch.uint8); s = torch.empty(M, device=x.device)
    ab = torch.empty(M, nab, device=x.device, dtype=torch.bfloat16); rstd = torch.empty(M, device=x.device)
    nul = ctypes.c_void_p(None)
    if M:
        _m().block_entry_fwd((M,), (256,), x2, nw, wab if nab else nul, ctypes.c_int(nab), ctypes.c_float(eps), y, s, c, ab if nab else nul, rstd,
                             ctypes.c_int(d), ctypes.c_float(clip), ctypes.c_int(_qmax(bits)))
    return y.view(*x.shape), c, s, ab.view(*x.shape[:-1], nab)
