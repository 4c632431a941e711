"""Assembly of a depth shard's halo-extended slab, the local step of the forward halo exchange.

``halo_assemble(x, lo, hi, halo)`` returns ``cat([lo, x, hi], dim=2)`` for channels-last 5-D tensors, with zeros for a
missing neighbour (``lo`` / ``hi`` = ``None``) -- the slab the reference builds after its receives
(``ScaFFold/unet/conv3d.py:769-776``) and then convolves at depth padding 0.  One streaming kernel instead of a fill
and up to three strided copies.  Differentiable: the gradient of the slab is sliced back to the shard and to the two
borrowed boundary slabs (which ``backward_halo_exchange`` would send to their owners, ``conv3d.py:779-812``).
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import HaloDesc

__all__ = ["halo_assemble", "is_supported_halo"]

_CL3D = torch.channels_last_3d


def is_supported_halo(x, lo=None, hi=None, halo: int = 1) -> bool:
    """Total gate: never raises."""
    try:
        if not isinstance(x, torch.Tensor) or x.dim() != 5 or not x.is_cuda or x.dtype not in _lib.SUPPORTED_DTYPES:
            return False
        if not isinstance(halo, int) or isinstance(halo, bool) or halo < 0 or min(x.shape[1:]) < 1:
            return False
        n, c, d, h, w = x.shape
        for t in (lo, hi):
            if t is None:
                continue
            if not isinstance(t, torch.Tensor) or t.dtype is not x.dtype or t.device != x.device \
                    or tuple(t.shape) != (n, c, halo, h, w):
                return False
        return True
    except Exception:
        return False


class _HaloAssembleFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, lo, hi, halo):
        x = x.contiguous(memory_format=_CL3D)
        lo = None if lo is None else lo.contiguous(memory_format=_CL3D)
        hi = None if hi is None else hi.contiguous(memory_format=_CL3D)
        n, c, d, h, w = (int(v) for v in x.shape)
        out = torch.empty((n, c, d + 2 * halo, h, w), dtype=x.dtype, device=x.device, memory_format=_CL3D)
        desc = HaloDesc(n, c, d, h, w, halo)
        with _lib.device_guard(x.device):
            rc = _lib.lib().sfh_halo_assemble(ctypes.byref(desc), _lib.dtype_code(x.dtype), _lib.ptr(x), _lib.ptr(lo), _lib.ptr(hi),
                                              _lib.ptr(out), _lib.stream_ptr(x.device))
        _lib.check(rc, "halo_assemble")
        ctx.halo_args = (d, halo, lo is not None, hi is not None)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        d, halo, has_lo, has_hi = ctx.halo_args
        gx = grad.narrow(2, halo, d) if ctx.needs_input_grad[0] else None
        glo = grad.narrow(2, 0, halo) if (has_lo and ctx.needs_input_grad[1]) else None
        ghi = grad.narrow(2, halo + d, halo) if (has_hi and ctx.needs_input_grad[2]) else None
        return gx, glo, ghi, None


def halo_assemble(x: torch.Tensor, lo: Optional[torch.Tensor] = None, hi: Optional[torch.Tensor] = None,
                  halo: int = 1) -> torch.Tensor:
    """``[lo | x | hi]`` along depth; ``None`` stands for ``halo`` planes of zeros. The result is channels-last."""
    if not is_supported_halo(x, lo, hi, halo):
        raise NotImplementedError(
            f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)} halo={halo} "
            f"lo={None if lo is None else tuple(lo.shape)} hi={None if hi is None else tuple(hi.shape)}")
    if halo == 0:
        return x
    return _HaloAssembleFn.apply(x, lo, hi, halo)
