"""Drop-in ``nn.Module``s over the HIP ops: ``FastConv3d``, ``FastConvTranspose3d``, ``FastGroupNorm``.

They stand where the reference's adapters stand (``ScaFFold/unet/conv3d.py:1235-1479,1790-1904``,
``ScaFFold/unet/group_norm.py:556-808``) and keep their contract:

* same parameters under the same names and no buffers, so ``state_dict`` keys and shapes are
  those of ``nn.Conv3d`` / ``nn.ConvTranspose3d`` / ``nn.GroupNorm`` in both directions;
* under ``torch.autocast`` only exactly-fp32 operands are cast, and the cast is an ordinary
  autograd node *outside* the kernel's node, so an fp32 parameter receives an fp32 gradient
  (``conv3d.py:446-480``);
* the autograd nodes save ``(x, weight)`` after the launch, compute the bias gradient as
  ``grad_output.sum((0, 2, 3, 4))`` (``conv3d.py:1231``) and are once-differentiable: a second
  differentiation raises instead of returning zeros;
* ``FastGroupNorm`` returns its input's dtype (not fp32) inside autocast and applies the ReLU
  when ``activation="relu"``.

What is deliberately absent: the reference's fallback ladder (Triton -> MIOpen, compiled ->
eager), its latches, the hardware allowlist and the mesh-wide vote.  There is one backend here;
a call it does not serve raises ``NotImplementedError``.

``FastConv3d.shard_halo`` reproduces the compute shape of one DistConv depth shard on a single
GPU: the input is extended by one voxel of (zero) halo on each depth face and the convolution
runs with depth padding 0, which is what the reference's own halo exchange hands its kernel
(``conv3d.py:648-677,748-792``); with no neighbour the halo is zero and the result equals the
ordinary padded convolution.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd.function import once_differentiable

from . import conv3d as _c3
from . import groupnorm as _gn
from . import halo as _halo
from . import transposed as _ct

__all__ = ["FastConv3d", "FastConvTranspose3d", "FastGroupNorm", "autocast_dtype", "cast_operand", "compute_copy",
           "flush_weight_gradients"]

_CL3D = torch.channels_last_3d

#: pack each convolution weight once per step for forward and data gradient also outside graph capture
PACK_WEIGHTS_ONCE = False


def autocast_dtype(tensor: torch.Tensor) -> Optional[torch.dtype]:
    """The dtype autocast would cast a convolution's operands to on this device, or ``None``."""
    try:
        if not torch.is_autocast_enabled(tensor.device.type):
            return None
        return torch.get_autocast_dtype(tensor.device.type)
    except (RuntimeError, TypeError):
        return None


def cast_operand(tensor: Optional[torch.Tensor], dtype: Optional[torch.dtype]):
    """ATen's ``cached_cast`` rule: only an exactly-fp32 tensor is narrowed."""
    if tensor is None or dtype is None or tensor.dtype is not torch.float32:
        return tensor
    return tensor.to(dtype)


def compute_copy(param: Optional[torch.Tensor], dtype: Optional[torch.dtype]):
    """A current half-precision copy of an fp32 parameter kept by the optimizer (``FusedClipAdam(shadow_dtype=...)``
    refreshes it inside its update kernel), or ``None``.  It is used only while the parameter has not been written
    by anything else since the copy was made (torch's version counter), so a stale copy is never read."""
    if param is None or dtype is None or param.dtype is not torch.float32:
        return None
    copy = getattr(param, "_sfh_shadow", None)
    if copy is None or copy.dtype is not dtype or getattr(param, "_sfh_shadow_version", None) != param._version:
        return None
    return copy


def _current_packs(owner: torch.Tensor, source: torch.Tensor, in_shape, stride, padding, dilation):
    """The packed forms of a parameter's weight for this problem, or ``None`` when the problem reads no packed weight.

    They are kept on the parameter (``owner._sfh_packs``) and trusted without a launch only under the rule that also
    guards the optimizer's half-precision copies: the optimizer that writes the parameter refreshes them inside its
    step (``maintained``) and nothing else has written the parameter since (torch's version counter).  Otherwise they
    are packed again here, in one launch for both directions."""
    if source.dtype is torch.float32:
        return None
    table = owner.__dict__.get("_sfh_packs")
    if table is None:
        table = owner._sfh_packs = {}
    key = (in_shape, padding)
    e = table.get(key)
    if e is None:
        if len(table) >= 8:  # a parameter meets few problems; shapes that keep changing are not worth the buffers
            table.clear()
        e = table[key] = _c3.PackedWeights(source, in_shape, stride, padding, dilation)
        e.version = owner._version
        return e if e else None
    if not e:
        return None
    if not (e.maintained and e.version == owner._version and e.source is source):
        e.repack(source)
        e.version = owner._version
    return e


def _fp32_weight_grad(fn, *args, **kwargs):
    """Weight gradient straight in fp32 where the tiled kernels serve the shape, else in the operands' dtype and
    widened afterwards (what autocast's cast node would have done)."""
    try:
        return fn(*args, grad_dtype=torch.float32, **kwargs)
    except NotImplementedError:
        return fn(*args, **kwargs).to(torch.float32)


# ---- weight gradients of a backward pass in one launch -----------------------------------------------------------------
# Nothing reads a weight gradient before the optimizer (``ScaFFold/utils/trainer.py:678-694``), and a launch of the
# weight-gradient kernel costs 15-20 us whatever the problem.  A convolution whose module has ``defer_weight_grad`` set
# therefore does not compute its weight gradient in its own backward node: the node leaves (parameter, operands) in a
# queue and returns no gradient for the weight, and a callback the autograd engine runs when the backward pass has
# finished -- still inside ``backward()`` -- computes all queued gradients with :func:`conv3d_backward_weight_batch` and
# adds them to the parameters' ``.grad``.  After ``backward()`` returns the gradients are where they always are.  What
# differs: hooks on the parameter's gradient accumulation do not see these gradients, and the operands stay alive until
# the end of the pass.
class _QueuedWeightGrad:
    __slots__ = ("param", "inp", "wshape", "gy", "padding", "grad_dtype", "family", "early")

    def __init__(self, param, inp, wshape, gy, padding, grad_dtype, family=1, early=False):
        self.param, self.inp, self.wshape, self.gy, self.padding, self.grad_dtype = param, inp, wshape, gy, padding, grad_dtype
        self.family, self.early = family, early  # the launch that takes it (1: large rows, 2: small volumes); early mode


_WEIGHT_GRAD_QUEUE: list = []
_BATCHABLE: dict = {}


def _deferrable(param, in_shape, wshape, stride, padding, dilation, dtype) -> int:
    """Whether a weight gradient can wait for the end of the pass: the parameter is a leaf that takes a ``.grad`` and the
    library batches the problem.  0, or the launch of the batch that takes it (``conv3d.weight_grad_batch_family``)."""
    if param is None or not param.is_leaf or not param.requires_grad:
        return 0
    key = (in_shape, wshape, stride, padding, dilation, dtype)
    ok = _BATCHABLE.get(key)
    if ok is None:
        ok = _c3.weight_grad_batch_family(in_shape, wshape, stride, padding, dilation, dtype)
        if len(_BATCHABLE) > 256:
            _BATCHABLE.clear()
        _BATCHABLE[key] = ok
    return ok


def _queue_weight_grad(item: _QueuedWeightGrad) -> None:
    _WEIGHT_GRAD_QUEUE.append(item)
    # one callback per queued gradient: the first to run takes the whole queue, the others find it empty (a pass that
    # raised before its callbacks ran leaves its entries to the next pass's callbacks, or to flush_weight_gradients())
    torch.autograd.Variable._execution_engine.queue_callback(flush_weight_gradients)
    if item.early and item.family == 2:
        # The pass has reached a small volume: the deep levels, whose kernels are bound by latency and leave most of the
        # device idle. The large-row gradients queued so far (the decoder's upper levels) go out now, on a stream of their own
        # and on half of the compute units, beside the rest of the pass; flush_weight_gradients() joins them.
        waiting = [it for it in _WEIGHT_GRAD_QUEUE if it.family == 1 and it.early and it.gy.device == item.gy.device and
                   it.gy.dtype is item.gy.dtype and it.grad_dtype is item.grad_dtype]
        if len(waiting) >= 2:
            for it in waiting:
                _WEIGHT_GRAD_QUEUE.remove(it)
            _send_early(waiting)


_EARLY_STREAMS: dict = {}
_EARLY_DONE: list = []


def _send_early(items) -> None:
    dev = items[0].gy.device
    side = _EARLY_STREAMS.get(dev)
    if side is None:
        side = _EARLY_STREAMS[dev] = torch.cuda.Stream(device=dev)
    # Every use of the side stream starts by waiting for the current one and ends (in flush_weight_gradients) with the
    # current one waiting for it, and the operands stay referenced until then: memory the caching allocator hands to
    # either stream is never in use on the other.
    side.wait_stream(torch.cuda.current_stream(dev))
    gdt, dt = items[0].grad_dtype, items[0].gy.dtype
    with torch.no_grad(), torch.cuda.stream(side):
        grads = _c3.conv3d_backward_weight_batch([(it.inp, it.wshape, it.gy, it.padding) for it in items],
                                                 grad_dtype=None if gdt is dt else gdt, share_device=True)
    _EARLY_DONE.append((items, grads, side))


def _add_to_grads(items, grads) -> None:
    for it, gw in zip(items, grads):
        p = it.param
        if p.grad is None:
            # in the parameter's own layout, as the engine's accumulation would leave it
            p.grad = gw if gw.stride() == p.stride() else torch.empty_like(p).copy_(gw)
        else:
            p.grad.add_(gw)


def flush_weight_gradients() -> None:
    """Compute the queued weight gradients and add them to their parameters' ``.grad`` (runs by itself at the end of a
    backward pass; callable by hand after a pass that raised)."""
    while _EARLY_DONE:
        items, grads, side = _EARLY_DONE.pop(0)
        torch.cuda.current_stream(items[0].gy.device).wait_stream(side)
        with torch.no_grad():
            _add_to_grads(items, grads)
    if not _WEIGHT_GRAD_QUEUE:
        return
    queue = list(_WEIGHT_GRAD_QUEUE)
    _WEIGHT_GRAD_QUEUE.clear()
    groups: dict = {}
    for it in queue:
        groups.setdefault((it.gy.device, it.gy.dtype, it.grad_dtype), []).append(it)
    with torch.no_grad():
        for (_, dt, gdt), items in groups.items():
            grads = _c3.conv3d_backward_weight_batch([(it.inp, it.wshape, it.gy, it.padding) for it in items],
                                                     grad_dtype=None if gdt is dt else gdt)
            _add_to_grads(items, grads)


# positions in _Conv3dFn.forward's argument list (after ctx): the gradients come back in this order
_ARG_SECOND, _N_ARGS = 11, 14


class _Conv3dFn(torch.autograd.Function):
    """The caller (``FastConv3d.forward``) has passed the gate for all three directions with these very operands, and
    autograd hands ``backward`` a gradient of the output's shape and dtype: the per-call gates are not repeated."""

    @staticmethod
    def forward(ctx, x, weight, bias, stride, padding, dilation, weight_compute=None, bias_compute=None, packs=None, slab=None,
                gn_groups=0, second=None, slab2=None, defer_weight_grad=False):
        # weight / bias are the tensors that receive gradients; when half-precision copies of fp32 masters are
        # given, the kernels read those and the gradients are produced in the masters' dtype directly
        wc = weight if weight_compute is None else weight_compute
        bc = bias if bias_compute is None else bias_compute
        # `slab` = (tensor, halo): x is the depth interior of that tensor, whose faces already hold the halo; the
        # kernels read the whole of it and the data gradient of its interior is x's
        ctx.halo = 0
        if slab is not None:
            ctx.halo, ctx.depth = slab[1], x.shape[2]
            x = slab[0]
        # `second`: the input is the pair (x, second) whose channels follow each other -- a skip connection and the
        # upsampled tensor, never concatenated; `slab2` is to `second` what `slab` is to x
        ctx.pair = second is not None
        if slab2 is not None:
            second = slab2[0]
        in_shape = x.shape if second is None else torch.Size((x.shape[0], x.shape[1] + second.shape[1], *x.shape[2:]))
        pf = pd = None
        if packs is not None:
            # packed forms that are current (kept by the module, refreshed by whoever writes the weight)
            pf, pd = packs.fwd, packs.dgrad
        elif ctx.needs_input_grad[0] and (PACK_WEIGHTS_ONCE or torch.cuda.is_current_stream_capturing()):
            # When the data gradient will be wanted too, the weight can be packed for both directions in one launch.
            # That saves a launch per convolution on the GPU and costs a little more host time, so it is done where
            # host time is free (under graph capture) or when asked for (PACK_WEIGHTS_ONCE).
            pf, pd = _c3.pack_weights(wc, in_shape, stride, padding, dilation)
        # gn_groups: a GroupNorm of that many groups follows; the launch leaves its statistics on y where it can
        if second is None:
            y = _c3.conv3d_forward(x, wc, bc, stride, padding, dilation, 1, packed_weight=pf, gn_groups=gn_groups, _checked=True)
            ctx.save_for_backward(x, wc) if pd is None else ctx.save_for_backward(x, wc, pd)
        else:
            y = _c3.conv3d_forward_pair(x, second, wc, bc, stride, padding, dilation, packed_weight=pf, gn_groups=gn_groups,
                                        _checked=True)
            ctx.save_for_backward(x, wc, second) if pd is None else ctx.save_for_backward(x, wc, second, pd)
        ctx.conv_args = (stride, padding, dilation, bias is not None, None if bias is None else bias.dtype,
                         weight.dtype is not wc.dtype)
        # the parameter whose .grad a deferred weight gradient is added to (see flush_weight_gradients)
        ctx.defer_param = weight if defer_weight_grad else None
        ctx.defer_early = defer_weight_grad == 2
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        if ctx.pair:
            return _Conv3dFn._backward_pair(ctx, grad_output)
        x, weight, *packed = ctx.saved_tensors
        stride, padding, dilation, has_bias, bias_dtype, master = ctx.conv_args
        needs_x, needs_w, needs_b = ctx.needs_input_grad[:3]
        grad_output = grad_output.contiguous(memory_format=_CL3D)
        grad_x = _c3.conv3d_backward_data(grad_output, weight, x.shape, stride, padding, dilation, 1,
                                          packed_weight=packed[0] if packed else None, _checked=True) if needs_x else None
        if ctx.halo and grad_x is not None:
            grad_x = grad_x.narrow(2, ctx.halo, ctx.depth)
        grad_w = None
        if needs_w and has_bias and needs_b:
            # both parameter gradients from one pass over grad_output where the library offers it (the 1x1x1 head)
            both = _c3.conv3d_backward_weight_bias(x, weight.shape, grad_output, stride, padding, dilation, 1,
                                                   grad_dtype=torch.float32 if master else None, _checked=True)
            if both is not None:
                grad_w, grad_b = both
                if grad_b.dtype is not bias_dtype:
                    grad_b = grad_b.to(bias_dtype)
                return grad_x, grad_w, grad_b, None, None, None, None, None, None, None, None, None, None, None
        family = _deferrable(ctx.defer_param, x.shape, weight.shape, stride, padding, dilation, x.dtype) if needs_w else 0
        if family:
            _queue_weight_grad(_QueuedWeightGrad(ctx.defer_param, x, weight.shape, grad_output, padding,
                                                 torch.float32 if master else x.dtype, family, ctx.defer_early))
        elif needs_w:
            if master:
                grad_w = _fp32_weight_grad(_c3.conv3d_backward_weight, x, weight.shape, grad_output, stride, padding, dilation, 1,
                                           _checked=True)
            else:
                grad_w = _c3.conv3d_backward_weight(x, weight.shape, grad_output, stride, padding, dilation, 1, _checked=True)
        grad_b = _c3.bias_grad(grad_output, bias_dtype) if (has_bias and needs_b) else None
        return grad_x, grad_w, grad_b, None, None, None, None, None, None, None, None, None, None, None

    @staticmethod
    def _backward_pair(ctx, grad_output):
        """The three gradients of the convolution over (x, second): the data gradient comes back as the two tensors the
        concatenation's backward would have cut it into."""
        x, weight, second, *packed = ctx.saved_tensors
        stride, padding, dilation, has_bias, bias_dtype, master = ctx.conv_args
        needs_x, needs_w, needs_b = ctx.needs_input_grad[:3]
        needs_second = ctx.needs_input_grad[_ARG_SECOND]
        grad_output = grad_output.contiguous(memory_format=_CL3D)
        grad_x = grad_second = None
        if needs_x or needs_second:
            in_shape = torch.Size((x.shape[0], x.shape[1] + second.shape[1], *x.shape[2:]))
            grad_x, grad_second = _c3.conv3d_backward_data_pair(grad_output, weight, in_shape, int(x.shape[1]), stride, padding,
                                                                dilation, packed_weight=packed[0] if packed else None, _checked=True)
            if ctx.halo:  # both tensors are slabs of the same depth: the interiors are the inputs' gradients
                grad_x = grad_x.narrow(2, ctx.halo, ctx.depth)
                grad_second = grad_second.narrow(2, ctx.halo, ctx.depth)
        grad_w = None
        family = 0
        if needs_w:
            family = _deferrable(ctx.defer_param, torch.Size((x.shape[0], x.shape[1] + second.shape[1], *x.shape[2:])), weight.shape,
                                 stride, padding, dilation, x.dtype)
        if family:
            _queue_weight_grad(_QueuedWeightGrad(ctx.defer_param, (x, second), weight.shape, grad_output, padding,
                                                 torch.float32 if master else x.dtype, family, ctx.defer_early))
        elif needs_w:
            if master:
                grad_w = _fp32_weight_grad(_c3.conv3d_backward_weight_pair, x, second, weight.shape, grad_output, stride, padding,
                                           dilation, _checked=True)
            else:
                grad_w = _c3.conv3d_backward_weight_pair(x, second, weight.shape, grad_output, stride, padding, dilation, _checked=True)
        grad_b = _c3.bias_grad(grad_output, bias_dtype) if (has_bias and needs_b) else None
        grads = [None] * _N_ARGS
        grads[0], grads[1], grads[2] = (grad_x if needs_x else None), grad_w, grad_b
        grads[_ARG_SECOND] = grad_second if needs_second else None
        return tuple(grads)


class _ConvTranspose3dFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, stride, weight_compute=None, bias_compute=None, packs=None, out_halo=0):
        wc = weight if weight_compute is None else weight_compute
        bc = bias if bias_compute is None else bias_compute
        # `out_halo` (one sample): the result is written into the interior of a depth slab with that many zero planes on
        # each face, which rides along as y._sfh_slab for a following FastConv3d.shard_halo
        # `packs`: kept packed forms of the kernel == stride convolution this op transposes; its data-gradient form is
        # what this forward reads, its forward form what the data gradient below reads
        y = _ct.conv_transpose3d_forward(x, wc, bc, stride, 0, 0, 1, 1, packed_weight=None if packs is None else packs.dgrad,
                                         out_halo=out_halo)
        pf = None if packs is None else packs.fwd
        ctx.save_for_backward(x, wc) if pf is None else ctx.save_for_backward(x, wc, pf)
        ctx.conv_args = (stride, bias is not None, None if bias is None else bias.dtype, weight.dtype is not wc.dtype)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        x, weight, *packed = ctx.saved_tensors
        stride, has_bias, bias_dtype, master = ctx.conv_args
        needs_x, needs_w, needs_b = ctx.needs_input_grad[:3]
        grad_output = grad_output.contiguous(memory_format=_CL3D)
        grad_x = _ct.conv_transpose3d_backward_data(grad_output, weight, x.shape, stride, 0, 0, 1, 1,
                                                    packed_weight=packed[0] if packed else None) if needs_x else None
        grad_w = grad_b = None
        if needs_w and has_bias and needs_b:
            # both from one pass over grad_output where the library offers it (the 2x2x2 matrix-core problems)
            both = _ct.conv_transpose3d_backward_weight_bias(x, weight.shape, grad_output, stride, 0, 0, 1, 1,
                                                             grad_dtype=torch.float32 if master else None)
            if both is not None:
                grad_w, grad_b = both
                if grad_b.dtype is not bias_dtype:
                    grad_b = grad_b.to(bias_dtype)
                return grad_x, grad_w, grad_b, None, None, None, None, None
        if needs_w:
            if master:
                grad_w = _fp32_weight_grad(_ct.conv_transpose3d_backward_weight, x, weight.shape, grad_output, stride, 0, 0, 1, 1)
            else:
                grad_w = _ct.conv_transpose3d_backward_weight(x, weight.shape, grad_output, stride, 0, 0, 1, 1)
        grad_b = _c3.bias_grad(grad_output, bias_dtype) if (has_bias and needs_b) else None
        return grad_x, grad_w, grad_b, None, None, None, None, None


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class FastConv3d(nn.Conv3d):
    """``nn.Conv3d`` served by the HIP kernels.  ``__init__`` is inherited unchanged."""

    #: emulate one depth shard: zero halo on both depth faces + depth padding 0
    shard_halo = False
    #: groups of a GroupNorm that reads this module's output next (0: none): the forward launch then also leaves that
    #: GroupNorm's statistics on its result, where the kernel offers it, and the normalisation skips its statistics pass
    gn_groups = 0
    #: leave this module's weight gradient to the end of the backward pass, where all such gradients come from one launch
    #: (see flush_weight_gradients); taken up only where the weight is the parameter itself and the library batches the shape.
    #: 2 instead of True: besides, the large-row gradients queued when the pass reaches its first small volume are computed
    #: there and then on a stream of their own, on half of the device, beside the rest of the pass
    defer_weight_grad = False

    def _pair_operands(self, x, second):
        """The tensors the kernels would read for ``forward(x, second)`` and the padding they would run with, or ``None``
        when the pair is not served as it stands: ``(x_read, second_read, padding, slab, slab2)``.  In the depth-shard
        form both tensors must already lie in slabs with zero faces (their producers wrote them there)."""
        if self.padding_mode != "zeros" or isinstance(self.padding, str) or self.groups != 1:
            return None
        if not isinstance(x, torch.Tensor) or not isinstance(second, torch.Tensor) or x.dtype is not second.dtype:
            return None
        dt = autocast_dtype(x)
        if dt is not None and x.dtype is torch.float32:
            return None  # the casts would make new tensors (outside the slabs); the caller concatenates instead
        if (dt if (dt is not None and self.weight.dtype is torch.float32) else self.weight.dtype) is not x.dtype:
            return None  # the weight the kernel would read (autocast narrows an fp32 parameter) is of another dtype
        padding = tuple(self.padding)
        slab = slab2 = None
        if self.shard_halo and padding[0] > 0:
            slab, slab2 = getattr(x, "_sfh_slab", None), getattr(second, "_sfh_slab", None)
            if slab is None or slab2 is None or slab[1] != padding[0] or slab2[1] != padding[0]:
                return None
            if slab[0].dtype is not x.dtype or slab2[0].dtype is not x.dtype:
                return None
            x_read, second_read = slab[0], slab2[0]
            padding = (0, padding[1], padding[2])
        else:
            x_read, second_read = x, second
        if not (x_read.is_contiguous(memory_format=_CL3D) and second_read.is_contiguous(memory_format=_CL3D)):
            return None
        return x_read, second_read, padding, slab, slab2

    def takes_pair(self, x, second) -> bool:
        """Whether ``forward(x, second)`` is served: the convolution of ``torch.cat([x, second], 1)`` read from the two
        tensors themselves, all three directions.  Total: never raises."""
        try:
            ops = self._pair_operands(x, second)
            return ops is not None and self._pair_gate(ops[0], ops[1], ops[2])
        except (TypeError, ValueError, AttributeError, RuntimeError):
            return False

    def _pair_gate(self, x_read, second_read, padding) -> bool:
        """The library's answer for the tensors the kernels would read, remembered per shape (the parameters' shapes and
        the module's geometry do not change; their dtypes under autocast are the activations')."""
        key = (x_read.shape, second_read.shape, x_read.dtype, x_read.device, padding, self.bias is None)
        table = self.__dict__.get("_pair_ok")
        if table is None:
            table = self.__dict__["_pair_ok"] = {}
        ok = table.get(key)
        if ok is None:
            # stand-ins with the dtype the kernel's operands will have (metadata only)
            w = self.weight if self.weight.dtype is x_read.dtype else self.weight.new_empty((1, 1, 1, 1, 1), dtype=x_read.dtype).expand(
                self.weight.shape)
            b = None
            if self.bias is not None:
                b = self.bias if self.bias.dtype is x_read.dtype else torch.empty(self.bias.shape, dtype=x_read.dtype, device=x_read.device)
            ok = _c3.is_supported_pair(x_read, second_read, w, b, tuple(self.stride), padding, tuple(self.dilation))
            if len(table) > 64:
                table.clear()
            table[key] = ok
        return ok

    def _forward_pair(self, x, second):
        ops = self._pair_operands(x, second)
        if ops is None:
            raise NotImplementedError(f"FastConv3d: the pair x={tuple(x.shape)}/{x.dtype}, second={tuple(second.shape)}/{second.dtype} "
                                      "is not served as it stands (see takes_pair); concatenate instead")
        x_read, second_read, padding, slab, slab2 = ops
        dt = autocast_dtype(x)
        weight, bias = self.weight, self.bias  # (each lookup of a parameter is a call into Module.__getattr__)
        wc = compute_copy(weight, dt)
        bc = compute_copy(bias, dt) if wc is not None else None
        master = wc is not None and (bias is None or bc is not None)
        w = wc if master else cast_operand(weight, dt)
        b = bc if master else cast_operand(bias, dt)
        stride, dilation = tuple(self.stride), tuple(self.dilation)
        if w.dtype is not x_read.dtype or not self._pair_gate(x_read, second_read, padding):
            raise NotImplementedError(
                f"FastConv3d: pair not served: x={tuple(x_read.shape)}/{x_read.dtype} second={tuple(second_read.shape)} on {x.device}, "
                f"weight={tuple(w.shape)}/{w.dtype}, stride={stride} padding={padding} dilation={dilation}")
        in_shape = torch.Size((x_read.shape[0], x_read.shape[1] + second_read.shape[1], *x_read.shape[2:]))
        if master:
            return _Conv3dFn.apply(x, weight, bias, stride, padding, dilation, w, b,
                                   _current_packs(weight, w, in_shape, stride, padding, dilation), slab, self.gn_groups,
                                   second, slab2, self.defer_weight_grad)
        packs = _current_packs(w, w, in_shape, stride, padding, dilation) if w is weight else None
        return _Conv3dFn.apply(x, w, b, stride, padding, dilation, None, None, packs, slab, self.gn_groups, second,
                               slab2, self.defer_weight_grad if w is weight else False)

    def forward(self, x: torch.Tensor, second: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``second``: the input is ``torch.cat([x, second], 1)``, read from the two tensors themselves (the decoder's skip
        connection and upsampled tensor, ``ScaFFold/unet/unet_parts.py:107-120``); ask :meth:`takes_pair` first."""
        if second is not None:
            return self._forward_pair(x, second)
        if self.padding_mode != "zeros" or isinstance(self.padding, str):
            raise NotImplementedError(f"FastConv3d: padding_mode={self.padding_mode!r} padding={self.padding!r}")
        dt = autocast_dtype(x)
        x = cast_operand(x, dt)
        weight, bias = self.weight, self.bias  # (each lookup of a parameter is a call into Module.__getattr__)
        # under autocast, an up-to-date half-precision copy kept by the optimizer replaces the per-call cast
        wc = compute_copy(weight, dt)
        bc = compute_copy(bias, dt) if wc is not None else None
        master = wc is not None and (bias is None or bc is not None)
        w = wc if master else cast_operand(weight, dt)
        b = bc if master else cast_operand(bias, dt)
        padding = tuple(self.padding)
        inner, slab = x, None
        if self.shard_halo and padding[0] > 0:
            # (N, C, D, H, W): extend D by the halo the neighbours would have sent (none here: zeros). A producer that
            # already wrote x into the interior of such a slab (zero faces) has left it on the tensor.
            slab = getattr(x, "_sfh_slab", None)
            if slab is not None and slab[1] == padding[0] and slab[0].dtype is x.dtype:
                x = slab[0]
            else:
                slab = None
                x = inner = _halo.halo_assemble(x, None, None, int(padding[0]))
            padding = (0, padding[1], padding[2])
        x = x.contiguous(memory_format=_CL3D)
        # the node below skips its own gates on the strength of this one (a call that will be differentiated is
        # gated for all three directions here)
        gate = _c3.is_supported_all if _wants_grad(inner, w, b) else _c3.is_supported
        if not gate(x, w, b, self.stride, padding, self.dilation, self.groups):
            raise NotImplementedError(
                f"FastConv3d: not served: x={tuple(x.shape)}/{x.dtype} on {x.device}, weight={tuple(w.shape)}/{w.dtype}, "
                f"stride={self.stride} padding={padding} dilation={self.dilation} groups={self.groups}"
            )
        stride, dilation = tuple(self.stride), tuple(self.dilation)
        if slab is None:
            inner = x
        if master:
            return _Conv3dFn.apply(inner, weight, bias, stride, padding, dilation, w, b,
                                   _current_packs(weight, w, x.shape, stride, padding, dilation), slab, self.gn_groups,
                                   None, None, self.defer_weight_grad)
        if w is weight:
            return _Conv3dFn.apply(inner, w, b, stride, padding, dilation, None, None,
                                   _current_packs(w, w, x.shape, stride, padding, dilation), slab, self.gn_groups,
                                   None, None, self.defer_weight_grad)
        return _Conv3dFn.apply(inner, w, b, stride, padding, dilation, None, None, None, slab, self.gn_groups)


class FastConvTranspose3d(nn.ConvTranspose3d):
    """``nn.ConvTranspose3d`` at ``kernel == stride`` served by the HIP kernels."""

    #: depth planes of zero halo to leave around the output for a following ``FastConv3d.shard_halo`` (0: none)
    out_halo = 0

    def forward(self, x: torch.Tensor, output_size=None) -> torch.Tensor:
        if output_size is not None:
            raise NotImplementedError("FastConvTranspose3d: output_size is not supported")
        dt = autocast_dtype(x)
        x = cast_operand(x, dt)
        weight, bias = self.weight, self.bias
        wc = compute_copy(weight, dt)
        bc = compute_copy(bias, dt) if wc is not None else None
        master = wc is not None and (bias is None or bc is not None)
        w = wc if master else cast_operand(weight, dt)
        b = bc if master else cast_operand(bias, dt)
        x = x.contiguous(memory_format=_CL3D)
        gate = _ct.is_supported_transposed_all if _wants_grad(x, w, b) else _ct.is_supported_transposed
        if not gate(x, w, b, self.stride, self.padding, self.output_padding, self.dilation, self.groups):
            raise NotImplementedError(
                f"FastConvTranspose3d: not served: x={tuple(x.shape)}/{x.dtype} on {x.device}, weight={tuple(w.shape)}, "
                f"stride={self.stride} padding={self.padding} output_padding={self.output_padding} "
                f"dilation={self.dilation} groups={self.groups}"
            )
        stride = tuple(self.stride)
        if master or w is weight:
            # the problem the packed forms belong to: the stride-k convolution over this op's output
            n, _, d, h, wd = x.shape
            big = torch.Size((n, w.shape[1], d * stride[0], h * stride[1], wd * stride[2]))
            packs = _current_packs(weight, w, big, stride, (0, 0, 0), (1, 1, 1))
            if packs is not None and (packs.fwd is None or packs.dgrad is None):
                packs = None
            if master:
                return _ConvTranspose3dFn.apply(x, weight, bias, stride, w, b, packs, self.out_halo)
            return _ConvTranspose3dFn.apply(x, w, b, stride, None, None, packs, self.out_halo)
        return _ConvTranspose3dFn.apply(x, w, b, stride, None, None, None, self.out_halo)


class FastGroupNorm(nn.GroupNorm):
    """``nn.GroupNorm`` (+ optional fused ReLU) served by the HIP kernels; output dtype = input dtype."""

    activation = None  # class-level default: not a parameter, buffer or state-dict key
    #: depth planes of zero halo to leave around the output for a following ``FastConv3d.shard_halo`` (0: none)
    out_halo = 0

    def __init__(self, num_groups, num_channels, eps=1e-5, affine=True, device=None, dtype=None, activation=None):
        super().__init__(num_groups, num_channels, eps=eps, affine=affine, device=device, dtype=dtype)
        if activation not in _gn.SUPPORTED_ACTIVATIONS:
            raise ValueError(f"activation must be one of {_gn.SUPPORTED_ACTIVATIONS}, got {activation!r}")
        self.activation = activation

    def extra_repr(self) -> str:
        base = super().extra_repr()
        return base if self.activation is None else f"{base}, activation={self.activation!r}"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dim() == 5 and not x.is_contiguous(memory_format=_CL3D):
            x = x.contiguous(memory_format=_CL3D)
        return _gn.group_norm(x, self.num_groups, self.weight, self.bias, self.eps, self.activation, out_dtype=None,
                              out_halo=self.out_halo)
