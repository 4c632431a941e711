"""The skip connection's channel concatenation as one streaming kernel, optionally into a depth slab.

``skip_concat(skip, upsampled)`` is ``torch.cat([skip, upsampled], dim=1)`` (``ScaFFold/unet/unet_parts.py:107-120``) for
channels-last 5-D tensors: one launch instead of two strided copies, and one for the backward split.  With
``out_halo=h`` (one sample) the result is the interior view of a slab with ``h`` zero depth planes on each face, carried
as ``result._sfh_slab = (slab, h)``: the tensor a following ``FastConv3d.shard_halo`` reads, so the concatenation and
the slab assembly of the halo exchange (``ScaFFold/unet/conv3d.py:769-776``) are one pass over the data.
"""

from __future__ import annotations

import ctypes

import torch
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import ConcatDesc

__all__ = ["skip_concat", "is_supported_concat"]

_CL3D = torch.channels_last_3d


def is_supported_concat(skip, upsampled) -> bool:
    """Total gate: never raises."""
    try:
        for t in (skip, upsampled):
            if not isinstance(t, torch.Tensor) or t.dim() != 5 or not t.is_cuda or t.dtype not in _lib.SUPPORTED_DTYPES:
                return False
        if skip.dtype is not upsampled.dtype or skip.device != upsampled.device:
            return False
        if skip.shape[0] != upsampled.shape[0] or skip.shape[2:] != upsampled.shape[2:] or skip.numel() == 0 or upsampled.numel() == 0:
            return False
        es = skip.dtype.itemsize
        return (skip.shape[1] * es) % 16 == 0 and (upsampled.shape[1] * es) % 16 == 0
    except Exception:
        return False


class _SkipConcatFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, out_halo):
        a = a.contiguous(memory_format=_CL3D)
        b = b.contiguous(memory_format=_CL3D)
        n, ca, d, h, w = (int(v) for v in a.shape)
        cb = int(b.shape[1])
        halo = out_halo if n == 1 else 0
        desc = ConcatDesc(n, ca, cb, d * h * w, halo * h * w)
        slab = torch.empty((n, ca + cb, d + 2 * halo, h, w), dtype=a.dtype, device=a.device, memory_format=_CL3D)
        with _lib.device_guard(a.device):
            rc = _lib.lib().sfh_skip_concat_fwd(ctypes.byref(desc), _lib.dtype_code(a.dtype), _lib.ptr(a), _lib.ptr(b), _lib.ptr(slab),
                                                _lib.stream_ptr(a.device))
        _lib.check(rc, "skip_concat")
        ctx.cat_args = (n, ca, cb, d, h, w)
        if halo == 0:
            return slab
        out = slab.narrow(2, halo, d)
        out._sfh_slab = (slab, halo)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        n, ca, cb, d, h, w = ctx.cat_args
        grad = grad.contiguous(memory_format=_CL3D)
        ga = torch.empty((n, ca, d, h, w), dtype=grad.dtype, device=grad.device, memory_format=_CL3D)
        gb = torch.empty((n, cb, d, h, w), dtype=grad.dtype, device=grad.device, memory_format=_CL3D)
        desc = ConcatDesc(n, ca, cb, d * h * w, 0)   # `grad` is dense: the interior itself
        with _lib.device_guard(grad.device):
            rc = _lib.lib().sfh_skip_concat_bwd(ctypes.byref(desc), _lib.dtype_code(grad.dtype), _lib.ptr(grad), _lib.ptr(ga),
                                                _lib.ptr(gb), _lib.stream_ptr(grad.device))
        _lib.check(rc, "skip_concat backward")
        return ga, gb, None


def skip_concat(skip: torch.Tensor, upsampled: torch.Tensor, out_halo: int = 0) -> torch.Tensor:
    """``torch.cat([skip, upsampled], 1)``, channels-last; see the module text for ``out_halo``."""
    if not is_supported_concat(skip, upsampled):
        raise NotImplementedError(
            f"unsupported: skip={tuple(getattr(skip, 'shape', ()))}/{getattr(skip, 'dtype', None)} "
            f"upsampled={tuple(getattr(upsampled, 'shape', ()))}/{getattr(upsampled, 'dtype', None)}")
    return _SkipConcatFn.apply(skip, upsampled, int(out_halo))
