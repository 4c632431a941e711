"""Channels-last GroupNorm (+ fused ReLU) forward / backward on the HIP library.

Mirrors ``ScaFFold/unet/triton_group_norm.py``: the dispatcher ops
``torch.ops.scaffold_gn.group_norm`` / ``group_norm_backward`` (:1339-1436) with fake kernels and
an autograd formula (:1439-1479), the gate ``is_supported`` (:1541) and the public
``group_norm`` function (there called ``triton_group_norm``, :1610; the old name is kept as an
alias so callers can switch by changing an import).

Contract kept from the reference:

* statistics and the normalisation are fp32 whatever the storage dtype; the result is rounded once;
* ``out_dtype=MATCH_STOCK_DTYPE`` reproduces ``F.group_norm`` (fp32 inside autocast, the input's
  dtype outside), ``None`` means the input's dtype, an explicit dtype is honoured;
* ``activation="relu"`` is fused into the store and the backward gates on the recomputed
  pre-activation; NaN propagates like ``F.relu`` / ``threshold_backward``;
* ``mean`` / ``rstd`` are non-differentiable backward state; the backward op has no autograd
  formula, so double backward raises;
* every shape ``F.group_norm`` rejects is rejected with the same exception type.

Difference from the reference: inputs the gate refuses are **not** routed to ``F.group_norm``.
``group_norm`` raises ``NotImplementedError`` for them -- this package has no second backend.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import GroupNormDesc

__all__ = [
    "group_norm",
    "triton_group_norm",
    "is_supported",
    "SUPPORTED_ACTIVATIONS",
    "SUPPORTED_DTYPES",
    "MATCH_STOCK_DTYPE",
]

SUPPORTED_ACTIVATIONS = (None, "relu")
SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16)
_CL3D = torch.channels_last_3d


def _one_value_per_channel(input, num_groups: int) -> bool:
    """``F.group_norm`` raises for ``N * (C/G) * S == 1``, i.e. numel == C == num_groups."""
    channels = input.shape[1]
    return channels == num_groups and input.numel() == channels


def _validate(input, num_groups, weight, bias, activation) -> None:
    if activation not in SUPPORTED_ACTIVATIONS:
        raise ValueError(f"activation must be one of {SUPPORTED_ACTIVATIONS}, got {activation!r}")
    if input.dim() != 5:
        raise ValueError(f"expected a 5-D NCDHW tensor, got {tuple(input.shape)}")
    if num_groups <= 0 or input.shape[1] % num_groups != 0:
        raise ValueError(f"num_channels={input.shape[1]} is not divisible by num_groups={num_groups}")
    if _one_value_per_channel(input, num_groups):
        raise ValueError(
            f"Expected more than 1 value per channel when training, got input size {tuple(input.shape)} "
            f"with num_groups={num_groups}"
        )
    if input.dtype not in SUPPORTED_DTYPES:
        raise ValueError(f"unsupported input dtype {input.dtype}")
    if not input.is_contiguous(memory_format=_CL3D):
        raise ValueError("input must be channels_last_3d-contiguous")
    for name, t in (("weight", weight), ("bias", bias)):
        if t is not None and t.numel() != input.shape[1]:
            raise ValueError(f"{name} has {t.numel()} elements, expected {input.shape[1]}")


def _param_dtype(weight, bias, input) -> torch.dtype:
    for t in (weight, bias):
        if t is not None:
            return t.dtype
    return input.dtype


def _desc(input, num_groups: int, eps: float, activation) -> GroupNormDesc:
    n, c = int(input.shape[0]), int(input.shape[1])
    spatial = int(input.shape[2]) * int(input.shape[3]) * int(input.shape[4])
    return GroupNormDesc(n, c, int(num_groups), 1 if activation == "relu" else 0, spatial, float(eps))


_PLANS: dict = {}


def _plan(input, num_groups: int, eps: float, activation, backward: bool):
    """``(descriptor, dtype code, workspace bytes)`` of a call, cached by shape: one dictionary lookup per call."""
    key = (input.shape, input.dtype, num_groups, eps, activation, backward)
    plan = _PLANS.get(key)
    if plan is None:
        desc = _desc(input, num_groups, eps, activation)
        code = _lib.dtype_code(input.dtype)
        L = _lib.lib()
        need = (L.sfh_groupnorm_bwd_workspace_bytes if backward else L.sfh_groupnorm_fwd_workspace_bytes)(ctypes.byref(desc), code)
        if len(_PLANS) > 4096:
            _PLANS.clear()
        plan = _PLANS[key] = (desc, code, int(need))
    return plan


def _launch_forward(L, desc, xcode, odt, need, input, weight, bias, out, slab, out_halo, mean, rstd):
    """The statistics pass + normalisation; returns the status, or ``(status, output)`` when the slab form was refused and
    a plain output took its place."""
    ws = _lib.workspace(need, input.device)
    if slab is None:
        return L.sfh_groupnorm_fwd(
            ctypes.byref(desc), xcode, _lib.dtype_code(odt), _lib.dtype_code(_param_dtype(weight, bias, input)),
            _lib.ptr(input), _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(out), _lib.ptr(mean), _lib.ptr(rstd),
            _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.stream_ptr(input.device))
    rc = L.sfh_groupnorm_fwd_slab(
        ctypes.byref(desc), xcode, _lib.dtype_code(odt), _lib.dtype_code(_param_dtype(weight, bias, input)),
        _lib.ptr(input), _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(slab), out_halo * int(input.shape[3]) * int(input.shape[4]),
        _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.stream_ptr(input.device))
    if rc == _lib.SFH_ERR_UNSUPPORTED:  # channel counts off the vector path: the plain form
        out = torch.empty_like(input, dtype=odt)
        rc = L.sfh_groupnorm_fwd(
            ctypes.byref(desc), xcode, _lib.dtype_code(odt), _lib.dtype_code(_param_dtype(weight, bias, input)),
            _lib.ptr(input), _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(out), _lib.ptr(mean), _lib.ptr(rstd),
            _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.stream_ptr(input.device))
        return rc, out
    return rc


def _forward_impl(input, num_groups, weight, bias, eps, activation, out_dtype, out_halo: int = 0):
    """The forward launch: ``(output, mean, rstd)``; shared by the registered operator and the eager autograd node.

    ``out_halo > 0`` (one sample, output of the input's element width): the output is the interior view of a slab with
    ``out_halo`` zero depth planes on each face, which rides along as ``output._sfh_slab = (slab, out_halo)`` for a
    consumer that wants the extended tensor (a depth shard's convolution) without copying the interior."""
    _validate(input, num_groups, weight, bias, activation)
    weight = None if weight is None else weight.contiguous()
    bias = None if bias is None else bias.contiguous()
    if weight is not None and bias is not None and weight.dtype != bias.dtype:
        bias = bias.to(weight.dtype)
    odt = out_dtype or input.dtype
    n = int(input.shape[0])
    slab = None
    if out_halo > 0 and n == 1 and odt.itemsize == input.dtype.itemsize and input.numel() > 0:
        c, d, h, w = (int(v) for v in input.shape[1:])
        slab = torch.empty((1, c, d + 2 * out_halo, h, w), dtype=odt, device=input.device, memory_format=_CL3D)
        out = slab.narrow(2, out_halo, d)
        out._sfh_slab = (slab, out_halo)
    else:
        out = torch.empty_like(input, dtype=odt)  # keeps the channels_last_3d strides
    mean = torch.empty((n, num_groups), dtype=torch.float32, device=input.device)
    rstd = torch.empty((n, num_groups), dtype=torch.float32, device=input.device)
    if input.numel() == 0:
        return out, mean, rstd
    L = _lib.lib()
    desc, xcode, need = _plan(input, num_groups, eps, activation, False)
    with _lib.device_guard(input.device):
        rc = _lib.SFH_ERR_UNSUPPORTED
        given = getattr(input, "_sfh_gn_partials", None)
        if given is not None and given[2] == num_groups and given[3] == input._version and given[0].device == input.device:
            # the producer of `input` left per-group Welford records of these very bits: no statistics pass
            rc = L.sfh_groupnorm_fwd_from_partials(
                ctypes.byref(desc), xcode, _lib.dtype_code(odt), _lib.dtype_code(_param_dtype(weight, bias, input)),
                _lib.ptr(input), _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(out if slab is None else slab),
                0 if slab is None else out_halo * int(input.shape[3]) * int(input.shape[4]),
                _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(given[0]), given[0].numel() * 4, given[1],
                _lib.stream_ptr(input.device))
        if rc == _lib.SFH_ERR_UNSUPPORTED:
            rc = _launch_forward(L, desc, xcode, odt, need, input, weight, bias, out, slab, out_halo, mean, rstd)
            if isinstance(rc, tuple):
                rc, out = rc
    _lib.check(rc, "group_norm")
    return out, mean, rstd


@torch.library.custom_op("scaffold_gn::group_norm", mutates_args=(), device_types="cuda")
def _group_norm_op(
    input: torch.Tensor,
    num_groups: int,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
    activation: Optional[str],
    out_dtype: Optional[torch.dtype],
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Channels-last GroupNorm forward: ``(output, mean, rstd)``; mean/rstd are ``(N, G)`` fp32."""
    return _forward_impl(input, num_groups, weight, bias, eps, activation, out_dtype)


@_group_norm_op.register_fake
def _(input, num_groups, weight, bias, eps, activation, out_dtype):
    out = torch.empty_like(input, dtype=out_dtype or input.dtype)
    mean = input.new_empty((input.shape[0], num_groups), dtype=torch.float32)
    rstd = input.new_empty((input.shape[0], num_groups), dtype=torch.float32)
    return out, mean, rstd


def _backward_impl(grad_out, input, weight, bias, mean, rstd, num_groups, activation):
    """The backward launch: ``(d_input, d_weight, d_bias)``."""
    if not grad_out.is_contiguous(memory_format=_CL3D):
        grad_out = grad_out.contiguous(memory_format=_CL3D)
    if not input.is_contiguous(memory_format=_CL3D):
        input = input.contiguous(memory_format=_CL3D)
    if grad_out.dtype != input.dtype and grad_out.dtype != torch.float32:
        grad_out = grad_out.to(input.dtype)
    weight = None if weight is None else weight.contiguous()
    bias = None if bias is None else bias.contiguous()
    if weight is not None and bias is not None and weight.dtype != bias.dtype:
        bias = bias.to(weight.dtype)
    channels = int(input.shape[1])
    d_input = torch.empty_like(input, memory_format=_CL3D)
    dw32 = torch.empty(channels, dtype=torch.float32, device=input.device) if weight is not None else None
    db32 = torch.empty(channels, dtype=torch.float32, device=input.device) if bias is not None else None
    if input.numel() > 0:
        L = _lib.lib()
        desc, xcode, need = _plan(input, num_groups, 0.0, activation, True)
        with _lib.device_guard(input.device):
            ws = _lib.workspace(need, input.device)
            rc = L.sfh_groupnorm_bwd(
                ctypes.byref(desc), xcode, _lib.dtype_code(grad_out.dtype),
                _lib.dtype_code(_param_dtype(weight, bias, input)), _lib.ptr(grad_out), _lib.ptr(input), _lib.ptr(weight),
                _lib.ptr(bias), _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(d_input), _lib.ptr(dw32), _lib.ptr(db32),
                _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.stream_ptr(input.device))
        _lib.check(rc, "group_norm_backward")
    else:
        if dw32 is not None:
            dw32.zero_()
        if db32 is not None:
            db32.zero_()
    d_weight = input.new_empty(0, dtype=torch.float32) if weight is None else dw32.to(weight.dtype)
    d_bias = input.new_empty(0, dtype=torch.float32) if bias is None else db32.to(bias.dtype)
    return d_input, d_weight, d_bias


@torch.library.custom_op("scaffold_gn::group_norm_backward", mutates_args=(), device_types="cuda")
def _group_norm_backward_op(
    grad_out: torch.Tensor,
    input: torch.Tensor,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    mean: torch.Tensor,
    rstd: torch.Tensor,
    num_groups: int,
    activation: Optional[str],
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(d_input, d_weight, d_bias)``; the parameter gradients are empty when the parameter is None.
    ``d_input`` has the input's dtype and is channels_last_3d."""
    return _backward_impl(grad_out, input, weight, bias, mean, rstd, num_groups, activation)


@_group_norm_backward_op.register_fake
def _(grad_out, input, weight, bias, mean, rstd, num_groups, activation):
    channels = input.shape[1]
    d_input = torch.empty_like(input, memory_format=_CL3D)
    d_weight = input.new_empty(channels if weight is not None else 0,
                               dtype=weight.dtype if weight is not None else torch.float32)
    d_bias = input.new_empty(channels if bias is not None else 0,
                             dtype=bias.dtype if bias is not None else torch.float32)
    return d_input, d_weight, d_bias


# Positions of the operator's arguments that can carry a gradient (the schema order of scaffold_gn::group_norm).
_ARG_INPUT, _ARG_WEIGHT, _ARG_BIAS, _N_ARGS = 0, 2, 3, 7


def _remember_for_backward(ctx, inputs, output):
    """What the backward launch reads: x, the affine parameters and the statistics the forward produced (they carry no
    gradient of their own); which of the three gradients autograd asked for is kept per argument position."""
    ctx.mark_non_differentiable(output[1], output[2])
    ctx.save_for_backward(inputs[_ARG_INPUT], inputs[_ARG_WEIGHT], inputs[_ARG_BIAS], output[1], output[2])
    ctx.gn_groups, ctx.gn_activation = inputs[1], inputs[5]
    ctx.gn_wanted = tuple(pos for pos in (_ARG_INPUT, _ARG_WEIGHT, _ARG_BIAS) if ctx.needs_input_grad[pos])


def _gradients_through_the_op(ctx, grad_out, _grad_mean, _grad_rstd):
    """One backward launch produces all three gradients; they are handed out at the positions that were asked for."""
    grads = [None] * _N_ARGS
    if ctx.gn_wanted:
        x, gamma, beta, mean, rstd = ctx.saved_tensors
        produced = torch.ops.scaffold_gn.group_norm_backward(grad_out, x, gamma, beta, mean, rstd, ctx.gn_groups, ctx.gn_activation)
        for pos, grad in zip((_ARG_INPUT, _ARG_WEIGHT, _ARG_BIAS), produced):
            if pos in ctx.gn_wanted:
                grads[pos] = grad
    return tuple(grads)


torch.library.register_autograd("scaffold_gn::group_norm", _gradients_through_the_op, setup_context=_remember_for_backward)


class _EagerGroupNormFn(torch.autograd.Function):
    """The same two launches as the registered operators, as a plain autograd node: outside ``torch.compile`` the
    operator registry's dispatch costs more host time per call than both launches together."""

    @staticmethod
    def forward(ctx, input, num_groups, weight, bias, eps, activation, out_dtype, out_halo=0):
        out, mean, rstd = _forward_impl(input, num_groups, weight, bias, eps, activation, out_dtype, out_halo)
        ctx.save_for_backward(input, weight, bias, mean, rstd)
        ctx.num_groups = num_groups
        ctx.activation = activation
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out):
        input, weight, bias, mean, rstd = ctx.saved_tensors
        need_x, need_w, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[2], ctx.needs_input_grad[3]
        if not (need_x or need_w or need_b):
            return None, None, None, None, None, None, None, None
        d_input, d_weight, d_bias = _backward_impl(grad_out, input, weight, bias, mean, rstd, ctx.num_groups, ctx.activation)
        return (d_input if need_x else None, None, d_weight if need_w else None, d_bias if need_b else None, None, None, None, None)


# ---------------------------------------------------------------------------------------------
# public API
# ---------------------------------------------------------------------------------------------
def _autocast_active(input: torch.Tensor) -> bool:
    try:
        return bool(torch.is_autocast_enabled(input.device.type))
    except (RuntimeError, TypeError):
        return False


class _MatchStockDtype:
    __slots__ = ()

    def __repr__(self):
        return "MATCH_STOCK_DTYPE"


#: default ``out_dtype``: what ``F.group_norm`` would return (fp32 inside autocast, else the input's dtype)
MATCH_STOCK_DTYPE = _MatchStockDtype()


def _resolve_out_dtype(input: torch.Tensor, out_dtype) -> Optional[torch.dtype]:
    if out_dtype is MATCH_STOCK_DTYPE:
        if input.dtype is not torch.float32 and _autocast_active(input):
            return torch.float32
        return None
    return out_dtype


@_lib.memoized_gate
def is_supported(input, num_groups: int, weight=None, bias=None, activation: Optional[str] = None) -> bool:
    """Whether the HIP kernels serve this call: a 5-D CUDA tensor, ``channels_last_3d``-contiguous,
    fp32/bf16/fp16, C divisible by ``num_groups``, affine parameters of the input's dtype (or fp32 under
    autocast), and not one of the shapes ``F.group_norm`` itself rejects.  Total and side-effect free."""
    try:
        if activation not in SUPPORTED_ACTIVATIONS:
            return False
        if not isinstance(input, torch.Tensor) or input.device.type != "cuda":
            return False
        if input.dim() != 5 or input.dtype not in SUPPORTED_DTYPES:
            return False
        if not isinstance(num_groups, int) or isinstance(num_groups, bool) or num_groups <= 0:
            return False
        channels = input.shape[1]
        if channels % num_groups != 0 or input.numel() == 0:
            return False
        if _one_value_per_channel(input, num_groups):
            return False
        if not input.is_contiguous(memory_format=_CL3D):
            return False
        for t in (weight, bias):
            if t is None:
                continue
            if not isinstance(t, torch.Tensor) or t.dim() != 1 or t.numel() != channels or t.device != input.device:
                return False
            if t.dtype is not input.dtype:
                if t.dtype is not torch.float32 or not _autocast_active(input):
                    return False
        return True
    except (TypeError, ValueError, AttributeError):
        return False


def group_norm(input, num_groups: int, weight=None, bias=None, eps: float = 1e-5, activation: Optional[str] = None, *,
               out_dtype=MATCH_STOCK_DTYPE, out_halo: int = 0):
    """``F.group_norm(input, num_groups, weight, bias, eps)`` (then ``F.relu`` when ``activation="relu"``)
    on a channels_last_3d CUDA tensor.  Raises ``NotImplementedError`` for calls :func:`is_supported` refuses.

    ``out_halo`` (eager calls on one sample) asks for the result as the interior of a depth slab with that many zero
    planes on each face (``result._sfh_slab``), for ``FastConv3d.shard_halo``; values and gradients are unchanged."""
    if activation not in SUPPORTED_ACTIVATIONS:
        raise ValueError(f"activation must be one of {SUPPORTED_ACTIVATIONS}, got {activation!r}")
    if not (out_dtype is MATCH_STOCK_DTYPE or out_dtype is None or out_dtype in SUPPORTED_DTYPES):
        raise ValueError(
            f"out_dtype must be MATCH_STOCK_DTYPE, None (the input's dtype) or one of {SUPPORTED_DTYPES}, got {out_dtype!r}"
        )
    if not is_supported(input, num_groups, weight, bias, activation):
        if isinstance(input, torch.Tensor) and input.dim() == 5 and input.is_cuda:
            # shapes F.group_norm rejects keep F.group_norm's own exception type
            if isinstance(num_groups, int) and num_groups > 0 and input.shape[1] % num_groups == 0 \
                    and _one_value_per_channel(input, num_groups):
                raise ValueError(
                    f"Expected more than 1 value per channel when training, got input size {tuple(input.shape)}"
                )
        raise NotImplementedError(
            f"unsupported group_norm call: input={tuple(getattr(input, 'shape', ()))}/{getattr(input, 'dtype', None)} on "
            f"{getattr(input, 'device', None)}, num_groups={num_groups}; needs a channels_last_3d CUDA tensor"
        )
    if torch.compiler.is_compiling():
        out, _mean, _rstd = torch.ops.scaffold_gn.group_norm(
            input, num_groups, weight, bias, float(eps), activation, _resolve_out_dtype(input, out_dtype)
        )
        return out
    return _EagerGroupNormFn.apply(input, num_groups, weight, bias, float(eps), activation, _resolve_out_dtype(input, out_dtype),
                                   int(out_halo))


#: the reference's name for :func:`group_norm`
triton_group_norm = group_norm
