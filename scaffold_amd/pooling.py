"""``MaxPool3d(2)`` on channels-last volumes: the down-sampling step of the U-Net's ``Down`` block.

The reference calls the stock module there (``ScaFFold/unet/unet_parts.py:165``).  This op keeps its
semantics (floor mode, ties to the first voxel of the cell, NaN wins) and its result bit for bit, but reads the
NDHWC tensor where it lies, keeps one byte per output element for the backward instead of an int64 index, and
writes the input gradient in one pass.
"""

from __future__ import annotations

import ctypes

import torch
import torch.nn as nn
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import PoolDesc

__all__ = ["max_pool3d_2x_with_skip", "max_pool3d_2x", "is_supported_pool", "FastMaxPool3d"]

_CL3D = torch.channels_last_3d


def is_supported_pool(x) -> bool:
    """Total gate: never raises."""
    try:
        return (isinstance(x, torch.Tensor) and x.dim() == 5 and x.is_cuda and x.dtype in _lib.SUPPORTED_DTYPES
                and x.shape[1] >= 1 and min(x.shape[2:]) >= 1)
    except Exception:
        return False


class _MaxPool2Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, out_halo=0):
        x = x.contiguous(memory_format=_CL3D)
        n, c, d, h, w = (int(v) for v in x.shape)
        idx = torch.empty((n, d // 2, h // 2, w // 2, c), dtype=torch.uint8, device=x.device)
        desc = PoolDesc(n, c, d, h, w)
        y = None
        if out_halo > 0 and n == 1 and min(d, h, w) >= 2:
            # the result in the interior of a depth slab with zero faces (the launch zeroes them), for a following
            # FastConv3d.shard_halo; where the library does not offer it for these extents, the plain launch below
            slab = torch.empty((1, c, d // 2 + 2 * out_halo, h // 2, w // 2), dtype=x.dtype, device=x.device, memory_format=_CL3D)
            with _lib.device_guard(x.device):
                rc = _lib.lib().sfh_maxpool2_fwd_slab(ctypes.byref(desc), _lib.dtype_code(x.dtype), _lib.ptr(x), _lib.ptr(slab),
                                                      out_halo * (h // 2) * (w // 2) * c, _lib.ptr(idx), _lib.stream_ptr(x.device))
            if rc != _lib.SFH_ERR_UNSUPPORTED:
                _lib.check(rc, "max_pool3d_2x")
                y = slab.narrow(2, out_halo, d // 2)
                y._sfh_slab = (slab, out_halo)
        if y is None:
            y = torch.empty((n, c, d // 2, h // 2, w // 2), dtype=x.dtype, device=x.device, memory_format=_CL3D)
            with _lib.device_guard(x.device):
                rc = _lib.lib().sfh_maxpool2_fwd(ctypes.byref(desc), _lib.dtype_code(x.dtype), _lib.ptr(x), _lib.ptr(y), _lib.ptr(idx),
                                                 _lib.stream_ptr(x.device))
            _lib.check(rc, "max_pool3d_2x")
        ctx.save_for_backward(idx)
        ctx.pool_shape = (n, c, d, h, w)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_y):
        (idx,) = ctx.saved_tensors
        n, c, d, h, w = ctx.pool_shape
        gy = grad_y.contiguous(memory_format=_CL3D)
        gx = torch.empty((n, c, d, h, w), dtype=gy.dtype, device=gy.device, memory_format=_CL3D)
        desc = PoolDesc(n, c, d, h, w)
        with _lib.device_guard(gy.device):
            rc = _lib.lib().sfh_maxpool2_bwd(ctypes.byref(desc), _lib.dtype_code(gy.dtype), _lib.ptr(gy), _lib.ptr(idx), _lib.ptr(gx),
                                             _lib.stream_ptr(gy.device))
        _lib.check(rc, "max_pool3d_2x backward")
        return gx, None


class _MaxPool2SkipFn(torch.autograd.Function):
    """Pooling of a tensor that is also carried on as a skip connection: returns ``(pooled, x)``; the two gradients
    of ``x`` (through the pooling and through the skip) are summed inside the pooling-gradient kernel instead of by a
    separate addition over the full-size tensor."""

    @staticmethod
    def forward(ctx, x, out_halo=0):
        y = _MaxPool2Fn.forward(ctx, x, out_halo)
        return y, x  # autograd hands out an alias of x with this node as its history

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_y, grad_skip):
        if grad_skip is None:
            return _MaxPool2Fn.backward(ctx, grad_y)
        if grad_y is None:
            return grad_skip, None
        (idx,) = ctx.saved_tensors
        n, c, d, h, w = ctx.pool_shape
        gy = grad_y.contiguous(memory_format=_CL3D)
        gs = grad_skip.contiguous(memory_format=_CL3D)
        if gs.dtype is not gy.dtype:
            gs = gs.to(gy.dtype)
        gx = torch.empty((n, c, d, h, w), dtype=gy.dtype, device=gy.device, memory_format=_CL3D)
        desc = PoolDesc(n, c, d, h, w)
        with _lib.device_guard(gy.device):
            rc = _lib.lib().sfh_maxpool2_bwd_add(ctypes.byref(desc), _lib.dtype_code(gy.dtype), _lib.ptr(gy), _lib.ptr(idx),
                                                 _lib.ptr(gs), _lib.ptr(gx), _lib.stream_ptr(gy.device))
        _lib.check(rc, "max_pool3d_2x backward")
        return gx, None


def max_pool3d_2x_with_skip(x: torch.Tensor, out_halo: int = 0):
    """``(F.max_pool3d(x, 2), x)``: use the returned ``x`` for the skip connection and the gradients of both uses are
    combined in one kernel (same values as autograd's own addition: one fp32 sum, one rounding)."""
    if not is_supported_pool(x):
        raise NotImplementedError(f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)}")
    if not x.is_contiguous(memory_format=_CL3D):
        return _MaxPool2Fn.apply(x, int(out_halo)), x
    pooled, skip = _MaxPool2SkipFn.apply(x, int(out_halo))
    slab = getattr(x, "_sfh_slab", None)
    if slab is not None:  # the alias is the same memory: still the interior of the slab its producer wrote it into
        skip._sfh_slab = slab
    return pooled, skip


def max_pool3d_2x(x: torch.Tensor, out_halo: int = 0) -> torch.Tensor:
    """``F.max_pool3d(x, 2)`` for a 5-D GPU tensor; the result is channels-last.  ``out_halo=h`` (one sample): the result is
    the interior view of a slab with ``h`` zero depth planes on each face (``result._sfh_slab``), for ``FastConv3d.shard_halo``."""
    if not is_supported_pool(x):
        raise NotImplementedError(f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)}")
    return _MaxPool2Fn.apply(x, int(out_halo))


def _all_equal(v, want) -> bool:
    if isinstance(v, (tuple, list)):
        return len(v) == 3 and all(int(e) == want for e in v)
    return int(v) == want


class FastMaxPool3d(nn.MaxPool3d):
    """``nn.MaxPool3d`` whose forward runs the HIP kernel. Only the configuration the U-Net uses exists:
    ``kernel_size == stride == 2``, no padding, no dilation, floor mode, no returned indices; anything else
    raises ``NotImplementedError`` at call time."""

    #: depth planes of zero halo to leave around the output for a following ``FastConv3d.shard_halo`` (0: none)
    out_halo = 0

    def _is_pool2(self) -> bool:
        stride = self.kernel_size if self.stride is None else self.stride
        return (_all_equal(self.kernel_size, 2) and _all_equal(stride, 2) and _all_equal(self.padding, 0)
                and _all_equal(self.dilation, 1) and not self.ceil_mode and not self.return_indices)

    def serves(self, input) -> bool:
        """Whether :meth:`with_skip` applies to this module and tensor."""
        return self._is_pool2() and is_supported_pool(input) and input.is_contiguous(memory_format=_CL3D)

    def with_skip(self, input):
        """``(self(input), input)`` for an input that is also used elsewhere (the U-Net's skip connection): use the
        returned pair and the two gradients of ``input`` are summed inside the pooling-gradient kernel."""
        if not self._is_pool2():
            raise NotImplementedError("FastMaxPool3d.with_skip supports MaxPool3d(2) only")
        return max_pool3d_2x_with_skip(input, self.out_halo)

    def forward(self, input):
        if not self._is_pool2():
            raise NotImplementedError(
                f"FastMaxPool3d supports MaxPool3d(2) only, got kernel_size={self.kernel_size} stride={self.stride} "
                f"padding={self.padding} dilation={self.dilation} ceil_mode={self.ceil_mode} "
                f"return_indices={self.return_indices}")
        return max_pool3d_2x(input, self.out_halo)
