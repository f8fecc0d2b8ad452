"""Residual sum fused with the scatter of routed rows: out = ((x + m) + mlp) + ys[pos] in one pass over the rows.

Offers the reference's entry point residual_slices(x, m, mlp, ys, pos) (python/caminus/train/fuse.py:16-45) on top of this
library's residual_slices_fwd / residual_slices_bwd. Backward: dx = dout, dm = dmlp = bf16(dout), dys[pos[r]] = bf16(dout[r]).

  x    fp32  [..., d]      residual stream
  m    bf16  [..., d]      first addend (mixer output)
  mlp  bf16  [..., d]      second addend
  ys   bf16  [n, d] | None outputs of the routed rows, compact
  pos  int32 [rows] | None row r adds ys[pos[r]] when pos[r] >= 0
"""
import ctypes

import torch

from ..device.hip import Module

_BLOCK = 256
_modules = {}


def _module():
    dev = torch.cuda.current_device()
    mod = _modules.get(dev)
    if mod is None:
        mod = _modules[dev] = Module('fuse')
    return mod


def _launch_forward(x, m, mlp, ys, pos):
    d = x.shape[-1]
    assert x.dtype == torch.float32 and m.dtype == mlp.dtype == torch.bfloat16 and d % 4 == 0
    routed = ys is not None and ys.numel() > 0
    if routed:
        assert ys.dtype == torch.bfloat16
    bufs = [t.contiguous() for t in (x, m, mlp)]
    tail = [ys.contiguous(), pos] if routed else [ctypes.c_void_p(None), ctypes.c_void_p(None)]
    out = torch.empty_like(bufs[0])
    quads = out.numel() // 4                                 # the kernel moves four values per thread
    grid = (quads + _BLOCK - 1) // _BLOCK
    _module().residual_slices_fwd((grid,), (_BLOCK,), *bufs, *tail, out, ctypes.c_int(d), ctypes.c_long(quads))
    return out


def _launch_backward(dout, pos, nys):
    dout = dout.contiguous()
    d = dout.shape[-1]
    quads = dout.numel() // 4
    dm = torch.empty(dout.shape, device=dout.device, dtype=torch.bfloat16)
    dmlp = torch.empty_like(dm)
    routed = pos is not None
    dys = torch.empty(nys, d, device=dout.device, dtype=torch.bfloat16) if routed else None      # every row of ys is named by one pos
    null = ctypes.c_void_p(None)
    grid = (quads + _BLOCK - 1) // _BLOCK
    _module().residual_slices_bwd((grid,), (_BLOCK,), dout, pos if routed else null, dm, dmlp, dys if routed else null,
                                  ctypes.c_int(d), ctypes.c_long(quads))
    return dout, dm, dmlp, dys


class ResidualSlices(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, m, mlp, ys, pos):
        routed = ys is not None and ys.numel() > 0
        ctx.save_for_backward(pos if routed else None)
        ctx.nys = ys.shape[0] if routed else 0
        return _launch_forward(x, m, mlp, ys, pos)

    @staticmethod
    def backward(ctx, dout):
        (pos,) = ctx.saved_tensors
        dx, dm, dmlp, dys = _launch_backward(dout, pos, ctx.nys)
        return dx, dm, dmlp, dys, None


def residual_slices(x, m, mlp, ys, pos):
    return ResidualSlices.apply(x, m, mlp, ys, pos)
