"""Fused activation fake-quant with autograd: per row a 128-point Hadamard rotation per chunk in bf16 steps, one scale per
row, int codes packed two per byte; the backward passes the straight-through gradient and the scale's gradient back through
the rotation in one kernel per call.

Offers the entry points of the reference's python/caminus/train/actq.py:46-169 with the same arguments and results:
actq, scales, codes, actq_codes, silu_mul_actq, block_entry, and the autograd classes ActQ, ActQCodes, SiluMulActQ,
BlockEntry. Values (y) are always bf16; gradients come back in the input's dtype; codes and scales carry no gradient.
"""
import ctypes

import torch

from ..device.hip import Module

_NULL = ctypes.c_void_p(None)
_modules = {}


def _kernels():
    dev = torch.cuda.current_device()
    mod = _modules.get(dev)
    if mod is None:
        mod = _modules[dev] = Module('actq')
    return mod


def _suffix(t):
    try:
        return {torch.bfloat16: 'bf16', torch.float32: 'f32'}[t.dtype]
    except KeyError:
        raise TypeError(f'actq: unsupported dtype {t.dtype}') from None


def _as_rows(x, limit=8192):
    K = x.shape[-1]
    assert K % 128 == 0 and K <= limit, K
    return x.reshape(-1, K).contiguous()


def _scalars(K, clip, bits):
    return ctypes.c_int(K), ctypes.c_float(clip), ctypes.c_int(2 ** (bits - 1) - 1)


def _forward(x2, bits, clip, want_y=True, want_scales=False, want_codes=False):
    """one launch of actq_fwd[_codes]_{f32,bf16} over rows x2 -> (y | None, s | None, codes | None)"""
    M, K = x2.shape
    dev = x2.device
    y = torch.empty(M, K, device=dev, dtype=torch.bfloat16) if want_y else None
    s = torch.empty(M, device=dev, dtype=torch.float32) if (want_scales or want_codes) else None
    c = torch.empty(M, K // 2, device=dev, dtype=torch.uint8) if want_codes else None
    if M:
        k, clipf, qmax = _scalars(K, clip, bits)
        if want_codes:
            getattr(_kernels(), 'actq_fwd_codes_' + _suffix(x2))((M,), (256,), x2, y if want_y else _NULL, s, c, k, clipf, qmax)
        else:
            getattr(_kernels(), 'actq_fwd_' + _suffix(x2))((M,), (256,), x2, y, s if s is not None else _NULL, k, clipf, qmax)
    return y, s, c


def _backward(x2, gy, bits, clip):
    M, K = x2.shape
    g2 = gy.reshape(M, K).to(torch.bfloat16).contiguous()
    dx = torch.empty_like(x2)
    if M:
        getattr(_kernels(), 'actq_bwd_' + _suffix(x2))((M,), (256,), x2, g2, dx, *_scalars(K, clip, bits))
    return dx


class ActQ(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bits, clip):
        x2 = _as_rows(x)
        y, _, _ = _forward(x2, bits, clip)
        ctx.save_for_backward(x2)
        ctx.quant = (bits, clip)
        ctx.in_shape = x.shape
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, gy):
        (x2,) = ctx.saved_tensors
        return _backward(x2, gy, *ctx.quant).view(ctx.in_shape), None, None


class ActQCodes(torch.autograd.Function):
    """ActQ that also hands out the packed codes and the row scales of the same pass"""
    @staticmethod
    def forward(ctx, x, bits, clip):
        assert bits <= 4
        x2 = _as_rows(x)
        y, s, c = _forward(x2, bits, clip, want_codes=True)
        ctx.save_for_backward(x2)
        ctx.quant = (bits, clip)
        ctx.in_shape = x.shape
        ctx.mark_non_differentiable(c, s)
        return y.view(x.shape), c, s

    @staticmethod
    def backward(ctx, gy, _gc, _gs):
        (x2,) = ctx.saved_tensors
        return _backward(x2, gy, *ctx.quant).view(ctx.in_shape), None, None


class SiluMulActQ(torch.autograd.Function):
    """gu [M, 2F] bf16 = [g | u] (rows may be strided) -> the fake-quant of act = bf16(bf16(silu g) * u) without writing act;
    the backward recomputes act and returns d gu = [dg | du] with torch's bf16 roundings of the product and of silu's derivative"""
    @staticmethod
    def forward(ctx, gu, bits, clip):
        M, F2 = gu.shape
        Fh = F2 // 2
        assert gu.dtype == torch.bfloat16 and gu.stride(1) == 1 and Fh % 128 == 0 and Fh <= 8192 and bits <= 4
        y = torch.empty(M, Fh, device=gu.device, dtype=torch.bfloat16)
        c = torch.empty(M, Fh // 2, device=gu.device, dtype=torch.uint8)
        s = torch.empty(M, device=gu.device, dtype=torch.float32)
        if M:
            _, clipf, qmax = _scalars(Fh, clip, bits)
            _kernels().silu_mul_actq_fwd((M,), (256,), gu, ctypes.c_int(gu.stride(0)), ctypes.c_int(Fh), y, s, c, clipf, qmax)
        ctx.save_for_backward(gu)
        ctx.quant = (bits, clip)
        ctx.mark_non_differentiable(c, s)
        return y, c, s

    @staticmethod
    def backward(ctx, gy, _gc, _gs):
        (gu,) = ctx.saved_tensors
        M, F2 = gu.shape
        Fh = F2 // 2
        g2 = gy.to(torch.bfloat16).contiguous()
        dgu = torch.empty(M, F2, device=gu.device, dtype=torch.bfloat16)
        if M:
            _, clipf, qmax = _scalars(Fh, ctx.quant[1], ctx.quant[0])
            _kernels().silu_mul_actq_bwd((M,), (256,), gu, ctypes.c_int(gu.stride(0)), ctypes.c_int(Fh), g2, dgu, clipf, qmax)
        return dgu, None, None


class BlockEntry(torch.autograd.Function):
    """x fp32 [..., d] -> for h = RMSNorm(x; nw, eps), never written: h's fake-quant (values, codes, scales) and the gate
    projections ab = bf16(bf16(h) @ wab^T), wab bf16 [nab, d] (two projections of nab / 2 rows each) or None. The norm
    weight and the projections are frozen: only x receives a gradient."""
    @staticmethod
    def forward(ctx, x, nw, wab, eps, bits, clip):
        d = x.shape[-1]
        x2 = _as_rows(x, limit=1024)
        assert x2.dtype == torch.float32 and bits <= 4
        nab = 0 if wab is None else wab.shape[0]
        assert nab <= 16 and nab % 2 == 0
        M, dev = x2.shape[0], x.device
        y = torch.empty(M, d, device=dev, dtype=torch.bfloat16)
        c = torch.empty(M, d // 2, device=dev, dtype=torch.uint8)
        s = torch.empty(M, device=dev, dtype=torch.float32)
        rstd = torch.empty(M, device=dev, dtype=torch.float32)
        ab = torch.empty(M, nab, device=dev, dtype=torch.bfloat16)
        if M:
            k, clipf, qmax = _scalars(d, clip, bits)
            _kernels().block_entry_fwd((M,), (256,), x2, nw, wab if nab else _NULL, ctypes.c_int(nab), ctypes.c_float(eps), y, s, c,
                                       ab if nab else _NULL, rstd, k, clipf, qmax)
        ctx.save_for_backward(x2, nw, rstd, wab if nab else None)
        ctx.quant = (bits, clip)
        ctx.in_shape = x.shape
        ctx.mark_non_differentiable(c, s)
        return y.view(x.shape), c, s, ab.view(*x.shape[:-1], nab)

    @staticmethod
    def backward(ctx, dy, _dc, _ds, dab):
        x2, nw, rstd, wab = ctx.saved_tensors
        M, d = x2.shape
        nab = 0 if wab is None else wab.shape[0]
        dy2 = dy.reshape(M, d).to(torch.bfloat16).contiguous()
        dab2 = None
        if nab:
            dab2 = (torch.zeros(M, nab, device=x2.device, dtype=torch.bfloat16) if dab is None
                    else dab.reshape(M, nab).to(torch.bfloat16).contiguous())
        dx = torch.empty_like(x2)
        if M:
            k, clipf, qmax = _scalars(d, ctx.quant[1], ctx.quant[0])
            _kernels().block_entry_bwd((M,), (256,), x2, nw, rstd, wab if nab else _NULL, ctypes.c_int(nab), dy2, dab2 if nab else _NULL, dx,
                                       k, clipf, qmax)
        return dx.view(ctx.in_shape), None, None, None, None, None


def actq(x, bits=4, clip=1.0):
    """bf16 fake-quantized x (same shape), differentiable"""
    return ActQ.apply(x, bits, clip)


def scales(x, bits=4, clip=1.0):
    """the per-row scales [M] fp32"""
    return _forward(_as_rows(x), bits, clip, want_scales=True)[1]


def codes(x, bits=4, clip=1.0, dequant=False):
    """(packed codes [M, K / 2] uint8, row scales [M]); dequant=True adds the bf16 values y = codes * s"""
    assert bits <= 4
    y, s, c = _forward(_as_rows(x), bits, clip, want_y=dequant, want_codes=True)
    return (c, s, y) if dequant else (c, s)


def actq_codes(x, bits=4, clip=1.0):
    """(differentiable bf16 fake-quantized x, packed codes [M, K / 2], row scales [M]) from one pass"""
    return ActQCodes.apply(x, bits, clip)


def silu_mul_actq(gu, bits=4, clip=1.0):
    """(xq, codes, scales) = actq_codes(silu(g) * u) for gu [M, 2F] bf16, fused"""
    return SiluMulActQ.apply(gu, bits, clip)


def block_entry(x, nw, wab, eps, bits=4, clip=1.0):
    """(xq, codes, scales, ab) for h = RMSNorm(x; nw, eps), fused"""
    return BlockEntry.apply(x, nw, wab, eps, bits, clip)
