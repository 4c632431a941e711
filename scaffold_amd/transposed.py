"""kernel == stride transposed conv3d (the U-Net up-convolution) on the HIP library.

Mirrors ``triton_conv3d/transposed.py``: ``conv_transpose3d_forward`` (:941),
``conv_transpose3d_backward_data`` (:1073), ``conv_transpose3d_backward_weight`` (:1113), the four
gates (:739-938) and ``grad_transposed_weight_empty`` (:1170).

With ``kernel == stride``, ``padding == output_padding == 0`` and ``dilation == 1`` the output
windows tile the output exactly once, so every output voxel has a single contributing input voxel
and tap:  ``y[n, oc, d*k+a, h*k+b, w*k+c] = bias[oc] + sum_ic x[n, ic, d, h, w] * w[ic, oc, a, b, c]``.
The data gradient is an ordinary convolution of ``grad_output`` at stride ``k`` with the weight
passed unpermuted (a ``ConvTranspose3d`` weight ``(Cin, Cout, k, k, k)`` already is the
``(out, in, k, k, k)`` weight of that convolution), and the weight gradient is the ordinary weight
gradient of the same convolution with the two activations swapped.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from . import conv3d as _c3
from ._lib import ConvTDesc, SUPPORTED_DTYPES
from .conv3d import (
    _CL3D,
    _check_out,
    _flags,
    _no_config,
    _triple,
    conv3d_backward_weight,
    conv3d_forward,
    is_supported,
    is_supported_bwd_weight,
)

__all__ = [
    "conv_transpose3d_forward",
    "conv_transpose3d_backward_data",
    "conv_transpose3d_backward_weight",
    "conv_transpose3d_backward_weight_bias",
    "is_supported_transposed",
    "is_supported_transposed_all",
    "is_supported_transposed_bwd_data",
    "is_supported_transposed_bwd_weight",
    "grad_transposed_weight_empty",
]


def _kernel_if_tiling(x_dim: int, w, stride, padding, output_padding, dilation, groups):
    """The kernel triple when the problem is a ``k == s`` upsample, else ``None`` (total)."""
    try:
        if groups != 1 or x_dim != 5:
            return None
        wshape = tuple(int(v) for v in (w.shape if isinstance(w, torch.Tensor) else w))
        if len(wshape) != 5:
            return None
        s = _triple(stride, "stride")
        p = _triple(padding, "padding")
        op = _triple(output_padding, "output_padding")
        d = _triple(dilation, "dilation")
        k = wshape[2:]
        if s != k or p != (0, 0, 0) or op != (0, 0, 0) or d != (1, 1, 1):
            return None
        if min(k) < 1 or wshape[0] < 1 or wshape[1] < 1:
            return None
        return k
    except (TypeError, ValueError, AttributeError):
        return None


@_lib.memoized_gate
def is_supported_transposed(x, w, bias=None, stride=1, padding=0, output_padding=0, dilation=1, groups: int = 1) -> bool:
    """Whether :func:`conv_transpose3d_forward` serves this call.  ``w`` is ``(Cin, Cout, kd, kh, kw)``."""
    try:
        if not isinstance(x, torch.Tensor) or not isinstance(w, torch.Tensor):
            return False
        k = _kernel_if_tiling(x.dim(), w, stride, padding, output_padding, dilation, groups)
        if k is None:
            return False
        if min(int(v) for v in x.shape[2:]) < 1:
            return False
        if x.dtype != w.dtype or x.dtype not in SUPPORTED_DTYPES:
            return False
        if not x.is_cuda or not w.is_cuda or x.device != w.device:
            return False
        if x.shape[1] != w.shape[0]:
            return False
        if bias is not None:
            if not isinstance(bias, torch.Tensor) or bias.dim() != 1 or bias.shape[0] != w.shape[1]:
                return False
            if bias.dtype != x.dtype or bias.device != x.device or bias.stride(0) != 1:
                return False
        return True
    except (TypeError, ValueError, AttributeError):
        return False


@_lib.memoized_gate
def is_supported_transposed_bwd_data(grad_output, w, input_shape, stride=1, padding=0, output_padding=0, dilation=1,
                                     groups: int = 1) -> bool:
    """Whether :func:`conv_transpose3d_backward_data` serves this call."""
    try:
        if not isinstance(grad_output, torch.Tensor) or not isinstance(w, torch.Tensor):
            return False
        k = _kernel_if_tiling(grad_output.dim(), w, stride, padding, output_padding, dilation, groups)
        if k is None:
            return False
        shape = tuple(int(v) for v in input_shape)
        if len(shape) != 5 or shape[1] != w.shape[0] or shape[0] != grad_output.shape[0]:
            return False
        if grad_output.shape[1] != w.shape[1]:
            return False
        if any(int(grad_output.shape[2 + i]) != shape[2 + i] * k[i] for i in range(3)):
            return False
        if shape[0] < 0 or min(shape[2:]) < 1:
            return False
        # the strided convolution that computes it
        return is_supported(grad_output, w, None, k, 0, 1, 1)
    except (TypeError, ValueError, AttributeError):
        return False


@_lib.memoized_gate
def is_supported_transposed_bwd_weight(x, weight_shape, grad_output, stride=1, padding=0, output_padding=0, dilation=1,
                                       groups: int = 1) -> bool:
    """Whether :func:`conv_transpose3d_backward_weight` serves this call."""
    try:
        if not isinstance(x, torch.Tensor) or not isinstance(grad_output, torch.Tensor):
            return False
        k = _kernel_if_tiling(x.dim(), tuple(weight_shape), stride, padding, output_padding, dilation, groups)
        if k is None:
            return False
        return is_supported_bwd_weight(grad_output, tuple(weight_shape), x, k, 0, 1, 1)
    except (TypeError, ValueError, AttributeError):
        return False


@_lib.memoized_gate
def is_supported_transposed_all(x, w, bias=None, stride=1, padding=0, output_padding=0, dilation=1, groups: int = 1) -> bool:
    """All three directions; asked for real rather than assumed to agree."""
    if not is_supported_transposed(x, w, bias, stride, padding, output_padding, dilation, groups):
        return False
    try:
        k = tuple(int(v) for v in w.shape[2:])
        gshape = (int(x.shape[0]), int(w.shape[1])) + tuple(int(x.shape[2 + i]) * k[i] for i in range(3))
        grad = x.new_empty((1, 1, 1, 1, 1)).expand(gshape)
        return is_supported_transposed_bwd_data(grad, w, tuple(x.shape), stride, padding, output_padding, dilation, groups) \
            and is_supported_transposed_bwd_weight(x, tuple(w.shape), grad, stride, padding, output_padding, dilation, groups)
    except (TypeError, ValueError, AttributeError, RuntimeError):
        return False


def grad_transposed_weight_empty(cin: int, cout: int, kernel: Sequence[int], *, dtype, device) -> torch.Tensor:
    """An empty ``(Cin, Cout, kd, kh, kw)`` gradient, ``channels_last_3d`` (memory ``[Cin][tap][Cout]``)."""
    k = _triple(kernel, "kernel")
    return torch.empty((cin, cout, *k), dtype=dtype, device=device, memory_format=_CL3D)


def conv_transpose3d_forward(
    x: torch.Tensor,
    w: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    stride=1,
    padding=0,
    output_padding=0,
    dilation=1,
    groups: int = 1,
    *,
    config=None,
    out: Optional[torch.Tensor] = None,
    force_generic: bool = False,
    packed_weight: Optional[torch.Tensor] = None,
    out_halo: int = 0,
) -> torch.Tensor:
    """Transposed 3-D convolution at ``kernel == stride``; NDHWC in and out; the bias is per
    output channel (not per tap column).  ``packed_weight``: the data-gradient form from
    ``pack_weights(w, output_shape, stride=kernel, padding=0)`` -- this op is the data gradient of that convolution.
    ``out_halo=h`` (one sample, the 2x2x2 matrix-core problems): the result is the interior view of a slab with ``h`` zero
    depth planes on each face, carried as ``result._sfh_slab = (slab, h)`` for a following ``FastConv3d.shard_halo``; the
    launch zeroes the faces itself.  Where the kernel does not offer it the result is the plain tensor."""
    if not is_supported_transposed(x, w, bias, stride, padding, output_padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)} w={tuple(getattr(w, 'shape', ()))} "
            f"stride={stride} padding={padding} output_padding={output_padding} dilation={dilation} groups={groups}"
        )
    _no_config(config)
    k = tuple(int(v) for v in w.shape[2:])
    x = x.contiguous(memory_format=_CL3D)
    n, cin, *in_sp = (int(v) for v in x.shape)
    cout = int(w.shape[1])
    y_shape = (n, cout, in_sp[0] * k[0], in_sp[1] * k[1], in_sp[2] * k[2])
    L = _lib.lib()
    desc = ConvTDesc(n, cin, in_sp[0], in_sp[1], in_sp[2], cout, k[0], k[1], k[2])
    code = _lib.dtype_code(x.dtype)
    if out_halo > 0 and out is None and n == 1 and not force_generic and min(in_sp) > 0:
        done = _forward_into_slab(L, desc, code, x, w, bias, packed_weight, y_shape, k, int(out_halo))
        if done is not None:
            return done
    if out is None:
        y = torch.empty(y_shape, device=x.device, dtype=x.dtype, memory_format=_CL3D)
    else:
        y = out
        _check_out(y, y_shape, x)
    if n == 0:
        return y
    with _lib.device_guard(x.device):
        if packed_weight is not None:
            if force_generic:
                raise ValueError("packed_weight= cannot be combined with force_generic=")
            # the up-convolution is the data gradient of the stride-k convolution of its OUTPUT: that problem's form
            _c3._problem(torch.Size(y_shape), torch.Size((cin, cout, *k)), k, 0, 1, x.dtype).check_packed(packed_weight, True, x)
            rc = L.sfh_convT3d_fwd(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(packed_weight), None, _lib.ptr(bias),
                                   _lib.ptr(y), None, 0, _lib.SFH_FLAG_WEIGHT_PACKED, _lib.stream_ptr(x.device))
        else:
            ws = _lib.workspace(L.sfh_convT3d_fwd_workspace_bytes(ctypes.byref(desc), code), x.device)
            rc = L.sfh_convT3d_fwd(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(w), _lib.strides5(w), _lib.ptr(bias),
                                   _lib.ptr(y), _lib.ptr(ws), 0 if ws is None else ws.numel(), _flags(force_generic),
                                   _lib.stream_ptr(x.device))
    _lib.check(rc, "conv_transpose3d_forward")
    return y


def conv_transpose3d_backward_weight_bias(x: torch.Tensor, weight_shape: Sequence[int], grad_output: torch.Tensor, stride=1, padding=0,
                                          output_padding=0, dilation=1, groups: int = 1, *, grad_dtype: Optional[torch.dtype] = None):
    """``(grad_weight, grad_bias)`` of the transposed convolution from ONE pass over ``grad_output``: the weight gradient of
    :func:`conv_transpose3d_backward_weight` (same bits) and ``grad_output.sum((0, 2, 3, 4))`` (fp32 accumulation in a fixed
    order, one rounding; ``ScaFFold/unet/conv3d.py:1786``) from the tiles the weight gradient reads anyway.  Both come in
    ``grad_dtype`` (default: the operands' dtype).  Returns ``None`` where the library does not offer the fused form (anything
    but the 2x2x2 matrix-core problems): the caller then computes the two apart."""
    if not is_supported_transposed_bwd_weight(x, weight_shape, grad_output, stride, padding, output_padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: x={tuple(getattr(x, 'shape', ()))} weight_shape={tuple(weight_shape)} "
            f"grad_output={tuple(getattr(grad_output, 'shape', ()))} stride={stride}")
    ws_shape = tuple(int(v) for v in weight_shape)
    x = x.contiguous(memory_format=_CL3D)
    gy = grad_output.contiguous(memory_format=_CL3D)
    n, cin, *in_sp = (int(v) for v in x.shape)
    cout, k = ws_shape[1], ws_shape[2:]
    if n == 0:
        return None
    gdt = x.dtype if grad_dtype is None else grad_dtype
    if gdt is not x.dtype and gdt is not torch.float32:
        raise ValueError(f"grad_dtype must be the operands' dtype or torch.float32, got {grad_dtype}")
    L = _lib.lib()
    desc = ConvTDesc(n, cin, in_sp[0], in_sp[1], in_sp[2], cout, k[0], k[1], k[2])
    code = _lib.dtype_code(x.dtype)
    need = int(L.sfh_convT3d_wgrad_bias_workspace_bytes(ctypes.byref(desc), code))
    if need == 0:
        return None
    gw = torch.empty(ws_shape, dtype=gdt, device=x.device, memory_format=_CL3D)
    gb = torch.empty((cout,), dtype=gdt, device=x.device)
    with _lib.device_guard(x.device):
        ws = _lib.workspace(need, x.device)
        rc = L.sfh_convT3d_wgrad_bias(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(gy), _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(ws), need,
                                      _lib.SFH_FLAG_GRAD_FP32 if gdt is not x.dtype else 0, _lib.stream_ptr(x.device))
    if rc == _lib.SFH_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "conv_transpose3d_backward_weight_bias")
    return gw, gb


def _forward_into_slab(L, desc, code, x, w, bias, packed_weight, y_shape, k, halo):
    """The forward launch with its result in the interior of a fresh depth slab, or ``None`` where the library does not
    offer that for the problem (the caller then runs the plain launch)."""
    _, cout, d, h, wd = y_shape
    slab = torch.empty((1, cout, d + 2 * halo, h, wd), dtype=x.dtype, device=x.device, memory_format=_CL3D)
    halo_elems = halo * h * wd * cout
    with _lib.device_guard(x.device):
        if packed_weight is not None:
            _c3._problem(torch.Size(y_shape), torch.Size((int(x.shape[1]), cout, *k)), k, 0, 1, x.dtype).check_packed(packed_weight, True, x)
            rc = L.sfh_convT3d_fwd_slab(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(packed_weight), None, _lib.ptr(bias),
                                        _lib.ptr(slab), halo_elems, None, 0, _lib.SFH_FLAG_WEIGHT_PACKED, _lib.stream_ptr(x.device))
        else:
            ws = _lib.workspace(L.sfh_convT3d_fwd_workspace_bytes(ctypes.byref(desc), code), x.device)
            rc = L.sfh_convT3d_fwd_slab(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(w), _lib.strides5(w), _lib.ptr(bias),
                                        _lib.ptr(slab), halo_elems, _lib.ptr(ws), 0 if ws is None else ws.numel(), 0,
                                        _lib.stream_ptr(x.device))
    if rc == _lib.SFH_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "conv_transpose3d_forward")
    y = slab.narrow(2, halo, d)
    y._sfh_slab = (slab, halo)
    return y


def conv_transpose3d_backward_data(
    grad_output: torch.Tensor,
    w: torch.Tensor,
    input_shape: Sequence[int],
    stride=1,
    padding=0,
    output_padding=0,
    dilation=1,
    groups: int = 1,
    *,
    config=None,
    out: Optional[torch.Tensor] = None,
    force_generic: bool = False,
    packed_weight: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``grad_input = conv3d(grad_output, w, stride=k)`` with ``w`` unpermuted (``packed_weight``: that convolution's
    forward form from ``pack_weights``)."""
    if not is_supported_transposed_bwd_data(grad_output, w, input_shape, stride, padding, output_padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: grad_output={tuple(getattr(grad_output, 'shape', ()))} w={tuple(getattr(w, 'shape', ()))} "
            f"input_shape={tuple(input_shape)} stride={stride} padding={padding} output_padding={output_padding} "
            f"dilation={dilation} groups={groups}"
        )
    k = tuple(int(v) for v in w.shape[2:])
    return conv3d_forward(grad_output, w, None, k, 0, 1, 1, config=config, out=out, force_generic=force_generic,
                          packed_weight=packed_weight)


def conv_transpose3d_backward_weight(
    x: torch.Tensor,
    weight_shape: Sequence[int],
    grad_output: torch.Tensor,
    stride=1,
    padding=0,
    output_padding=0,
    dilation=1,
    groups: int = 1,
    *,
    config=None,
    workspace: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    deterministic: bool = True,
    force_generic: bool = False,
    grad_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """Weight gradient ``(Cin, Cout, k, k, k)``, ``channels_last_3d``: the ordinary weight gradient of
    the stride-``k`` convolution whose input is ``grad_output`` and whose output gradient is ``x``."""
    if not is_supported_transposed_bwd_weight(x, weight_shape, grad_output, stride, padding, output_padding, dilation,
                                              groups):
        raise NotImplementedError(
            f"unsupported: x={tuple(getattr(x, 'shape', ()))} weight_shape={tuple(weight_shape)} "
            f"grad_output={tuple(getattr(grad_output, 'shape', ()))} stride={stride} padding={padding} "
            f"output_padding={output_padding} dilation={dilation} groups={groups}"
        )
    ws = tuple(int(v) for v in weight_shape)
    return conv3d_backward_weight(grad_output, ws, x, ws[2:], 0, 1, 1, config=config, workspace=workspace, out=out,
                                  deterministic=deterministic, force_generic=force_generic, grad_dtype=grad_dtype)
