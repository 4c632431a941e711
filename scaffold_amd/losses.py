"""Fused loss head of the U-Net train step: fp32 log-softmax, cross entropy and soft Dice in one pass.

Mirrors the loss block of the reference's trainer (``ScaFFold/utils/trainer.py:634-663``): the logits are
upcast to fp32 once, ``CE = sum_v w[y_v] * -log p_v[y_v] / normaliser`` (``ScaFFold/utils/losses.py:119-214``;
the normaliser is the voxel count, or ``sum_v w[y_v]`` with class weights), the Dice score of every (sample, class)
is ``(2 I + eps) / (P + T + eps)`` over the softmax probabilities (``ScaFFold/utils/dice_score.py:101-136``), and the
loss is ``CE + 1 - mean foreground Dice`` (``trainer.py:331-333,660-663``).  One HIP kernel pass produces all
sums (fixed-order reductions, no atomics), a second one the gradient; nothing of size ``N*C*D*H*W`` is
materialised in fp32.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch
from torch.autograd.function import once_differentiable

from . import _lib
from ._lib import LossDesc

__all__ = ["ce_dice_loss", "is_supported_loss"]

_CL3D = torch.channels_last_3d


def is_supported_loss(logits, labels, class_weight=None) -> bool:
    """Total gate: never raises."""
    try:
        if not isinstance(logits, torch.Tensor) or not isinstance(labels, torch.Tensor):
            return False
        if logits.dim() != 5 or labels.dim() != 4 or not logits.is_cuda or labels.device != logits.device:
            return False
        if logits.dtype not in _lib.SUPPORTED_DTYPES or labels.dtype is not torch.int64:
            return False
        n, c, d, h, w = logits.shape
        if tuple(labels.shape) != (n, d, h, w) or not 2 <= c <= 32 or n < 1 or d * h * w < 1:
            return False
        if class_weight is not None:
            if not isinstance(class_weight, torch.Tensor) or class_weight.device != logits.device \
                    or tuple(class_weight.shape) != (c,) or not class_weight.dtype.is_floating_point:
                return False
        return True
    except Exception:
        return False


class _CeDiceFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, class_weight, eps):
        x = logits.contiguous(memory_format=_CL3D)
        lab = labels.contiguous()
        cw = None if class_weight is None else class_weight.detach().to(torch.float32).contiguous()
        n, c, d, h, w = (int(v) for v in x.shape)
        desc = LossDesc(n, c, d * h * w, float(eps))
        L = _lib.lib()
        loss = torch.empty((), dtype=torch.float32, device=x.device)
        stats = torch.empty((n * 3 * c + 2,), dtype=torch.float32, device=x.device)
        with _lib.device_guard(x.device):
            ws = _lib.workspace(int(L.sfh_ce_dice_workspace_bytes(ctypes.byref(desc))), x.device)
            rc = L.sfh_ce_dice_fwd(ctypes.byref(desc), _lib.dtype_code(x.dtype), _lib.ptr(x), _lib.ptr(lab), _lib.ptr(cw),
                                   _lib.ptr(loss), _lib.ptr(stats), _lib.ptr(ws), 0 if ws is None else ws.numel(),
                                   _lib.stream_ptr(x.device))
        _lib.check(rc, "ce_dice_loss")
        ctx.save_for_backward(x, lab, stats) if cw is None else ctx.save_for_backward(x, lab, stats, cw)
        ctx.loss_args = (n, c, d * h * w, float(eps), cw is not None)
        return loss

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_loss):
        n, c, s, eps, weighted = ctx.loss_args
        saved = ctx.saved_tensors
        x, lab, stats = saved[:3]
        cw = saved[3] if weighted else None
        desc = LossDesc(n, c, s, eps)
        g = grad_loss.detach().to(device=x.device, dtype=torch.float32).reshape(1).contiguous()
        dx = torch.empty_like(x, memory_format=_CL3D)
        L = _lib.lib()
        with _lib.device_guard(x.device):
            rc = L.sfh_ce_dice_bwd(ctypes.byref(desc), _lib.dtype_code(x.dtype), _lib.ptr(x), _lib.ptr(lab), _lib.ptr(cw),
                                   _lib.ptr(stats), _lib.ptr(g), _lib.ptr(dx), _lib.stream_ptr(x.device))
        _lib.check(rc, "ce_dice_loss backward")
        return dx, None, None, None


def ce_dice_loss(logits: torch.Tensor, labels: torch.Tensor, class_weight: Optional[torch.Tensor] = None,
                 eps: float = 1e-6) -> torch.Tensor:
    """``CE(logits, labels[, class_weight]) + 1 - mean foreground soft Dice`` as a 0-dim fp32 tensor.

    ``logits``: ``(N, C, D, H, W)`` bf16 / fp16 / fp32 on the GPU (any memory format; channels-last is read in
    place); ``labels``: ``(N, D, H, W)`` int64 class ids, ids outside ``[0, C)`` contribute nothing."""
    if not is_supported_loss(logits, labels, class_weight):
        raise NotImplementedError(
            f"unsupported: logits={tuple(getattr(logits, 'shape', ()))}/{getattr(logits, 'dtype', None)} "
            f"labels={tuple(getattr(labels, 'shape', ()))}/{getattr(labels, 'dtype', None)}")
    return _CeDiceFn.apply(logits, labels, class_weight, eps)
