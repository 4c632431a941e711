"""Assembly of a depth shard's halo-extended slab, the local step of the forward halo exchange.

``halo_assemble(x, lo, hi, halo)`` returns ``cat([lo, x, hi], dim=2)`` for channels-last 5-D tensors, with zeros for a
missing neighbour (``lo`` / ``hi`` = ``None``) -- the slab the reference builds after its receives
(``ScaFFold/unet/conv3d.py:769-776``) and then convolves at depth padding 0.  One streaming kernel instead of a fill
and up to three strided copies.  Differentiable: the gradient of the slab is sliced back to the shard and to the two
borrowed boundary slabs (which ``backward_halo_exchange`` would send to their owners, ``conv3d.py:779-812``).

The other local steps are here too.  ``halo_pack(x, halo)`` gathers the boundary planes a shard sends into plain dense
wire buffers (``_packed_slab`` + ``view.copy_(x.narrow(...))``, ``conv3d.py:710-731,757-768``); ``halo_accumulate_(g,
lo, hi, halo)`` adds what the backward exchange received into the shard's own boundary planes in place
(``conv3d.py:838-841``).  ``halo_exchange(x, halo, wire)`` strings them together as one autograd node the way the
reference's ``_Halo3d`` does (``conv3d.py:844-900``): pack, hand the two wire buffers to ``wire`` (the caller's sends and
receives; this build runs one GPU and ships none), assemble; in the backward pack the slab gradient's outer planes, ``wire``
again, accumulate.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import HaloDesc

__all__ = ["halo_assemble", "is_supported_halo", "halo_pack", "halo_accumulate_", "halo_exchange"]

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


def _wire_buffer(x: torch.Tensor, halo: int):
    """A plain-contiguous (N, halo, H, W, C) allocation and its (N, C, halo, H, W) view: what goes on the wire must be
    plain contiguous (``conv3d.py:710-731``), and the view has exactly channels-last strides."""
    n, c, _, h, w = (int(v) for v in x.shape)
    base = torch.empty((n, halo, h, w, c), dtype=x.dtype, device=x.device)
    return base.permute(0, 4, 1, 2, 3)


def halo_pack(x: torch.Tensor, halo: int = 1, lo: bool = True, hi: bool = True):
    """``(x[:, :, :halo], x[:, :, -halo:])`` copied into wire buffers in one launch; a face not asked for is ``None``.
    Not differentiable by itself (``halo_exchange`` is the differentiable form)."""
    if not is_supported_halo(x, None, None, halo) or halo > x.shape[2]:
        raise NotImplementedError(f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)} halo={halo}")
    if halo == 0 or not (lo or hi):
        return None, None
    x = x.detach().contiguous(memory_format=_CL3D)
    n, c, d, h, w = (int(v) for v in x.shape)
    out_lo = _wire_buffer(x, halo) if lo else None
    out_hi = _wire_buffer(x, halo) if hi else None
    desc = HaloDesc(n, c, d, h, w, halo)
    with _lib.device_guard(x.device):
        rc = _lib.lib().sfh_halo_pack(ctypes.byref(desc), _lib.dtype_code(x.dtype), _lib.ptr(x), _lib.ptr(out_lo), _lib.ptr(out_hi),
                                      _lib.stream_ptr(x.device))
    _lib.check(rc, "halo_pack")
    return out_lo, out_hi


def halo_accumulate_(g: torch.Tensor, lo: Optional[torch.Tensor] = None, hi: Optional[torch.Tensor] = None, halo: int = 1):
    """In place: ``g[:, :, :halo] += lo``, ``g[:, :, -halo:] += hi`` (``None``: nothing received). ``g`` must be dense
    channels-last or the interior view of a dense one-sample slab; returns ``g``."""
    if not is_supported_halo(g, lo, hi, halo):
        raise NotImplementedError(
            f"unsupported: g={tuple(getattr(g, 'shape', ()))}/{getattr(g, 'dtype', None)} halo={halo} "
            f"lo={None if lo is None else tuple(lo.shape)} hi={None if hi is None else tuple(hi.shape)}")
    if 2 * halo > g.shape[2]:
        raise NotImplementedError(f"unsupported: depth {g.shape[2]} is thinner than two halos of {halo}")
    if halo == 0 or (lo is None and hi is None):
        return g
    if not g.is_contiguous(memory_format=_CL3D):
        raise ValueError("halo_accumulate_ works in place: g must be channels-last contiguous (a one-sample depth slice of a "
                         "channels-last tensor is)")
    lo = None if lo is None else lo.contiguous(memory_format=_CL3D)
    hi = None if hi is None else hi.contiguous(memory_format=_CL3D)
    n, c, d, h, w = (int(v) for v in g.shape)
    desc = HaloDesc(n, c, d, h, w, halo)
    with _lib.device_guard(g.device):
        rc = _lib.lib().sfh_halo_accumulate(ctypes.byref(desc), _lib.dtype_code(g.dtype), _lib.ptr(g), _lib.ptr(lo), _lib.ptr(hi),
                                            _lib.stream_ptr(g.device))
    _lib.check(rc, "halo_accumulate_")
    return g


class _HaloExchangeFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, halo, wire, has_lo, has_hi):
        x = x.contiguous(memory_format=_CL3D)
        send_lo, send_hi = halo_pack(x, halo, lo=has_lo, hi=has_hi)
        recv_lo, recv_hi = wire(send_lo, send_hi)
        ctx.exchange = (halo, wire, has_lo, has_hi, int(x.shape[2]))
        return _HaloAssembleFn.forward(_NoCtx(), x, recv_lo if has_lo else None, recv_hi if has_hi else None, halo)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad):
        halo, wire, has_lo, has_hi, d = ctx.exchange
        grad = grad.contiguous(memory_format=_CL3D)
        # the outer planes belong to the neighbours that lent them; what they return was borrowed from this shard
        send_lo, send_hi = halo_pack(grad, halo, lo=has_lo, hi=has_hi)
        recv_lo, recv_hi = wire(send_lo, send_hi)
        inner = grad.narrow(2, halo, d)
        if grad.shape[0] != 1:          # a batch's interior is strided by sample: accumulate into a dense copy
            inner = inner.contiguous(memory_format=_CL3D)
        halo_accumulate_(inner, recv_lo if has_lo else None, recv_hi if has_hi else None, halo)
        return inner, None, None, None, None


class _NoCtx:
    """Stand-in context for calling another node's forward from inside this one."""
    halo_args = None


def halo_exchange(x: torch.Tensor, halo: int, wire, has_lo: bool = True, has_hi: bool = True) -> torch.Tensor:
    """The depth halo exchange around one convolution as a single autograd node.

    ``wire(send_lo, send_hi) -> (recv_lo, recv_hi)`` performs the communication: it is given the planes for the lower and
    the upper neighbour (``None`` for a face with ``has_lo`` / ``has_hi`` false, i.e. no neighbour) and returns the planes
    received from them; it is called once in the forward and once in the backward, like the two ``batch_isend_irecv``
    rounds of the reference.  The result is the slab ``[recv_lo | x | recv_hi]`` (zeros for a missing neighbour) to be
    convolved at depth padding 0.  The backward mutates the incoming slab gradient in place, as the reference does.
    """
    if not is_supported_halo(x, None, None, halo) or halo < 1 or 2 * halo > x.shape[2]:
        raise NotImplementedError(f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)} halo={halo}")
    return _HaloExchangeFn.apply(x, int(halo), wire, bool(has_lo), bool(has_hi))
