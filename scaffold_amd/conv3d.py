"""Channels-last conv3d forward / data-gradient / weight-gradient on the HIP library.

Same call signatures, argument meaning and error behaviour as the reference's kernel package:

====================================  ==========================================================
this module                           reference (LBANN/ScaFFold)
====================================  ==========================================================
``conv3d_forward``                    ``triton_conv3d/gather_gemm.py:1187``
``conv3d_backward_data``              ``triton_conv3d/bwd_data.py:275``
``conv3d_backward_weight``            ``triton_conv3d/reduce_gemm.py:1177``
``is_supported`` / ``_all``           ``triton_conv3d/gather_gemm.py:945,1036``
``is_supported_bwd_data``             ``triton_conv3d/bwd_data.py:201``
``is_supported_bwd_weight``           ``triton_conv3d/reduce_gemm.py:1112``
``grad_weight_empty``                 ``triton_conv3d/reduce_gemm.py:1023``
``bwd_data_padding``                  ``triton_conv3d/bwd_data.py:84``
====================================  ==========================================================

Tensors are PyTorch NCDHW-shaped; memory is ``channels_last_3d`` (NDHWC).  Inputs in another
layout are converted, never misread.  Outputs are allocated once, directly in the layout the
kernels store.  ``out=`` / ``workspace=`` are validated, not trusted.  A call the library does
not serve raises ``NotImplementedError``; a contract violation raises ``ValueError``; the gates
never raise.  There is no fallback to another backend: a CPU tensor is simply not served.

``config=`` and ``weight_rsck=`` are accepted for signature compatibility.  Tile selection here
is a pure function of shape inside the library, so ``config`` must be ``None``; ``weight_rsck``
(the forward's ``(kd, kh, kw, Cin, Cout)`` weight copy) is validated and then read through its
strides like any other weight layout.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import ConvDesc, SUPPORTED_DTYPES

__all__ = [
    "conv3d_forward",
    "conv3d_backward_data",
    "conv3d_backward_weight",
    "bias_grad",
    "is_supported",
    "is_supported_all",
    "is_supported_bwd_data",
    "is_supported_bwd_weight",
    "bwd_data_padding",
    "grad_weight_empty",
    "workspace_elements",
    "pack_weights", "pack_weights_batch", "PackedWeights",
    "packed_weight_bytes",
    "split_count",
    "uses_mfma",
    "output_shape",
    "is_supported_pair",
    "conv3d_forward_pair",
    "conv3d_backward_data_pair",
    "conv3d_backward_weight_pair",
    "conv3d_backward_weight_bias",
]

_CL3D = torch.channels_last_3d


def _triple(value, name: str) -> tuple[int, int, int]:
    """``int`` or length-3 sequence of ints -> 3-tuple; anything else is a ValueError/TypeError."""
    if isinstance(value, bool):
        raise TypeError(f"{name} must be an int or three ints, got {value!r}")
    if isinstance(value, int):
        return (value, value, value)
    seq = tuple(value)  # TypeError for non-iterables such as None or 1.5
    if len(seq) != 3 or not all(isinstance(v, int) and not isinstance(v, bool) for v in seq):
        raise ValueError(f"{name} must be an int or three ints, got {value!r}")
    return seq  # type: ignore[return-value]


def output_shape(in_shape: Sequence[int], weight_shape: Sequence[int], stride, padding, dilation) -> tuple[int, ...]:
    """NCDHW output shape of a conv3d, ``floor((in + 2p - dil(k-1) - 1)/s) + 1`` per axis."""
    s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
    n, cout = int(in_shape[0]), int(weight_shape[0])
    sp = tuple(
        (int(in_shape[2 + i]) + 2 * p[i] - d[i] * (int(weight_shape[2 + i]) - 1) - 1) // s[i] + 1 for i in range(3)
    )
    return (n, cout) + sp


def bwd_data_padding(padding, dilation, kernel) -> tuple[int, int, int]:
    """Padding of the gather that computes the data gradient: ``dil*(k-1) - p`` per axis."""
    p, d, k = _triple(padding, "padding"), _triple(dilation, "dilation"), _triple(kernel, "kernel")
    return (d[0] * (k[0] - 1) - p[0], d[1] * (k[1] - 1) - p[1], d[2] * (k[2] - 1) - p[2])


def _desc(n, cin, in_sp, cout, k, s, p, d) -> ConvDesc:
    return ConvDesc(n, cin, in_sp[0], in_sp[1], in_sp[2], cout, k[0], k[1], k[2], s[0], s[1], s[2],
                    p[0], p[1], p[2], d[0], d[1], d[2])


class _Problem:
    """Everything about one convolution problem that does not depend on the tensors: parsed geometry, the descriptor
    the library takes, and (filled on first use) the workspace bytes of each direction."""

    __slots__ = ("s", "p", "d", "k", "n", "cin", "in_sp", "cout", "y_shape", "desc", "code", "need", "packed", "gn")

    def __init__(self, in_shape, w_shape, stride, padding, dilation, dtype):
        self.s, self.p, self.d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
        self.n, self.cin, *in_sp = (int(v) for v in in_shape)
        self.in_sp = tuple(in_sp)
        self.cout = int(w_shape[0])
        self.k = tuple(int(v) for v in w_shape[2:])
        self.y_shape = output_shape(in_shape, w_shape, self.s, self.p, self.d)
        self.desc = _desc(self.n, self.cin, self.in_sp, self.cout, self.k, self.s, self.p, self.d)
        self.code = _lib.dtype_code(dtype)
        self.need = {}
        self.packed = None
        self.gn = {}

    def gn_records(self, groups: int) -> int:
        """Records of GroupNorm partial sums per sample the forward launch leaves for ``groups`` groups (0: not offered)."""
        rec = self.gn.get(groups)
        if rec is None:
            rec = self.gn[groups] = int(_lib.lib().sfh_conv3d_fwd_gn_records(ctypes.byref(self.desc), self.code, int(groups)))
        return rec

    def packed_bytes(self, backward_data: bool) -> int:
        """Bytes of the packed weight this direction of the problem reads (0: it reads the weight where it lies)."""
        if self.packed is None:
            L = _lib.lib()
            self.packed = (int(L.sfh_conv3d_packed_weight_bytes(ctypes.byref(self.desc), self.code, 0)),
                           int(L.sfh_conv3d_packed_weight_bytes(ctypes.byref(self.desc), self.code, 1)))
        return self.packed[1 if backward_data else 0]

    def check_packed(self, packed, backward_data: bool, like: torch.Tensor) -> int:
        """A caller's ``packed_weight=`` is validated, not trusted: the MFMA kernels index it by fragment, so a pack made for
        another shape, direction or dtype would be read out of bounds.  Returns its size in bytes."""
        want = self.packed_bytes(backward_data)
        what = "data-gradient" if backward_data else "forward"
        if want == 0:
            raise ValueError(f"packed_weight=: the {what} direction of this problem does not read a packed weight")
        if not isinstance(packed, torch.Tensor) or packed.dtype is not torch.uint8 or packed.dim() != 1 or not packed.is_contiguous():
            raise ValueError(f"packed_weight= must be the contiguous uint8 buffer pack_weights() returned, got "
                             f"{getattr(packed, 'dtype', type(packed))} of shape {tuple(getattr(packed, 'shape', ()))}")
        if packed.device != like.device:
            raise ValueError(f"packed_weight= is on {packed.device}, the operands on {like.device}")
        if packed.numel() != want:
            raise ValueError(f"packed_weight= holds {packed.numel()} bytes, the {what} form of this problem has {want}: "
                             "it was packed for another shape, direction or dtype")
        return want

    def workspace_bytes(self, direction: str) -> int:
        need = self.need.get(direction)
        if need is None:
            fn = getattr(_lib.lib(), f"sfh_conv3d_{direction}_workspace_bytes")
            need = self.need[direction] = int(fn(ctypes.byref(self.desc), self.code))
        return need


_PROBLEMS: dict = {}


def _problem(in_shape, w_shape, stride, padding, dilation, dtype) -> _Problem:
    """The cached :class:`_Problem` of a call (one dictionary lookup per call once a shape has been seen)."""
    key = (in_shape, w_shape, stride, padding, dilation, dtype)
    try:
        prob = _PROBLEMS.get(key)
    except TypeError:  # unhashable spelling of a shape, stride, padding or dilation
        return _Problem(in_shape, w_shape, stride, padding, dilation, dtype)
    if prob is None:
        prob = _Problem(in_shape, w_shape, stride, padding, dilation, dtype)
        if len(_PROBLEMS) > 4096:
            _PROBLEMS.clear()
        _PROBLEMS[key] = prob
    return prob


# ---------------------------------------------------------------------------------------------
# gates
# ---------------------------------------------------------------------------------------------
@_lib.memoized_gate
def is_supported(x, w, bias=None, stride=1, padding=0, dilation=1, groups: int = 1) -> bool:
    """Whether :func:`conv3d_forward` serves this call.  Total: never raises."""
    try:
        if groups != 1:
            return False
        if not isinstance(x, torch.Tensor) or not isinstance(w, torch.Tensor):
            return False
        if x.dim() != 5 or w.dim() != 5:
            return False
        if x.dtype != w.dtype or x.dtype not in SUPPORTED_DTYPES:
            return False
        if not x.is_cuda or not w.is_cuda or x.device != w.device:
            return False
        if bias is not None:
            if not isinstance(bias, torch.Tensor) or bias.dim() != 1 or bias.shape[0] != w.shape[0]:
                return False
            if bias.dtype != x.dtype or bias.device != x.device or bias.stride(0) != 1:
                return False
        if x.shape[1] != w.shape[1]:
            return False
        s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
        k = tuple(int(v) for v in w.shape[2:])
        if min(s + d) < 1 or min(p) < 0:
            return False
        if min(int(v) for v in x.shape[2:]) < 1 or min(k) < 1:
            return False
        if w.shape[0] < 1 or w.shape[1] < 1:
            return False
        for i in range(3):
            if int(x.shape[2 + i]) + 2 * p[i] < d[i] * (k[i] - 1) + 1:
                return False
        return True
    except (TypeError, ValueError, AttributeError):
        return False


@_lib.memoized_gate
def is_supported_bwd_data(grad_output, weight, input_shape, stride=1, padding=0, dilation=1, groups: int = 1) -> bool:
    """Whether :func:`conv3d_backward_data` serves this call: stride 1 and ``p <= dil*(k-1)`` only."""
    try:
        if groups != 1:
            return False
        if not isinstance(grad_output, torch.Tensor) or not isinstance(weight, torch.Tensor):
            return False
        shape = tuple(int(v) for v in input_shape)
        if grad_output.dim() != 5 or weight.dim() != 5 or len(shape) != 5:
            return False
        if grad_output.dtype != weight.dtype or grad_output.dtype not in SUPPORTED_DTYPES:
            return False
        if not grad_output.is_cuda or not weight.is_cuda or grad_output.device != weight.device:
            return False
        s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
        k = tuple(int(v) for v in weight.shape[2:])
        if min(d) < 1 or min(p) < 0 or min(k) < 1 or s != (1, 1, 1):
            return False
        if any(p[i] > d[i] * (k[i] - 1) for i in range(3)):
            return False
        n, cin, *in_sp = shape
        if weight.shape[0] != grad_output.shape[1] or weight.shape[1] != cin or grad_output.shape[0] != n:
            return False
        if n < 1 or min(in_sp) < 1:
            return False
        for i in range(3):
            if int(grad_output.shape[2 + i]) != in_sp[i] + 2 * p[i] - d[i] * (k[i] - 1):
                return False
        return True
    except (TypeError, ValueError, AttributeError):
        return False


@_lib.memoized_gate
def is_supported_bwd_weight(input, weight_shape, grad_output, stride=1, padding=0, dilation=1, groups: int = 1) -> bool:
    """Whether :func:`conv3d_backward_weight` serves this call (any stride)."""
    try:
        if groups != 1:
            return False
        if not isinstance(input, torch.Tensor) or not isinstance(grad_output, torch.Tensor):
            return False
        ws = tuple(int(v) for v in weight_shape)
        if input.dim() != 5 or grad_output.dim() != 5 or len(ws) != 5:
            return False
        if input.dtype != grad_output.dtype or input.dtype not in SUPPORTED_DTYPES:
            return False
        if not input.is_cuda or not grad_output.is_cuda or input.device != grad_output.device:
            return False
        s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
        cout, cin, *k = ws
        if min(s + d + tuple(k)) < 1 or min(p) < 0 or cout < 1 or cin < 1:
            return False
        n, in_c, *in_sp = (int(v) for v in input.shape)
        if in_c != cin or grad_output.shape[1] != cout or grad_output.shape[0] != n:
            return False
        for i in range(3):
            eff = d[i] * (k[i] - 1) + 1
            if in_sp[i] + 2 * p[i] < eff:
                return False
            if int(grad_output.shape[2 + i]) != (in_sp[i] + 2 * p[i] - eff) // s[i] + 1:
                return False
        return True
    except (TypeError, ValueError, AttributeError):
        return False


@_lib.memoized_gate
def is_supported_all(x, w, bias=None, stride=1, padding=0, dilation=1, groups: int = 1) -> bool:
    """Whether all three directions of this convolution are served (the gate for a caller
    that will differentiate): the forward accepts strides the data gradient refuses."""
    if not is_supported(x, w, bias, stride, padding, dilation, groups):
        return False
    try:
        gshape = output_shape(x.shape, w.shape, stride, padding, dilation)
        grad = x.new_empty((1, 1, 1, 1, 1)).expand(gshape)  # metadata-only stand-in
        return is_supported_bwd_data(grad, w, tuple(x.shape), stride, padding, dilation, groups) and \
            is_supported_bwd_weight(x, tuple(w.shape), grad, stride, padding, dilation, groups)
    except (TypeError, ValueError, AttributeError, RuntimeError):
        return False


# ---------------------------------------------------------------------------------------------
# helpers
# ---------------------------------------------------------------------------------------------
def _check_out(y: torch.Tensor, shape: tuple[int, ...], like: torch.Tensor) -> None:
    if tuple(y.shape) != tuple(shape):
        raise ValueError(f"out= must have shape {tuple(shape)}, got {tuple(y.shape)}")
    if y.dtype != like.dtype:
        raise ValueError(f"out= must have dtype {like.dtype}, got {y.dtype}")
    if y.device != like.device:
        raise ValueError(f"out= must be on {like.device}, got {y.device}")
    if not y.is_contiguous(memory_format=_CL3D):
        raise ValueError(f"out= must be channels_last_3d (channel stride 1); got strides {tuple(y.stride())}")


def _check_weight_rsck(wr: torch.Tensor, shape: tuple[int, ...], like: torch.Tensor) -> None:
    if tuple(wr.shape) != tuple(shape):
        raise ValueError(f"weight_rsck= must have shape {tuple(shape)} (kd, kh, kw, Cin, Cout), got {tuple(wr.shape)}")
    if wr.dtype != like.dtype:
        raise ValueError(f"weight_rsck= must have dtype {like.dtype}, got {wr.dtype}")
    if wr.device != like.device:
        raise ValueError(f"weight_rsck= must be on {like.device}, got {wr.device}")
    if not wr.is_contiguous():
        raise ValueError(f"weight_rsck= must be contiguous; got strides {tuple(wr.stride())}")


def _no_config(config) -> None:
    if config is not None:
        raise ValueError("config= is not supported: tile selection is a pure function of shape inside the HIP library")


def _flags(force_generic: bool) -> int:
    return _lib.SFH_FLAG_FORCE_GENERIC if force_generic else 0


def uses_mfma(in_shape, weight_shape, stride, padding, dilation, dtype, direction: str = "fwd") -> bool:
    """Whether the MFMA implicit-GEMM kernels (rather than the direct ones) serve a problem."""
    s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
    n, cin, *in_sp = (int(v) for v in in_shape)
    cout, _, *k = (int(v) for v in weight_shape)
    desc = _desc(n, cin, in_sp, cout, k, s, p, d)
    code = {"fwd": 0, "bwd-data": 1, "bwd-weight": 2}[direction]
    return bool(_lib.lib().sfh_conv3d_uses_mfma(ctypes.byref(desc), _lib.dtype_code(dtype), code))


KERNEL_NAMES = ("direct", "persist", "brick", "wide", "wgrad", "other-matrix", "split")


def launch_geometry(in_shape, weight_shape, stride, padding, dilation, dtype, direction: str = "fwd") -> dict:
    """Which kernel serves a problem and with what launch geometry: ``{"kernel", "voxels", "blocks", "slices"}`` (the
    kernel by name; output voxels per workgroup step; 32-channel output blocks per workgroup; slices of the reduction whose
    fp32 partials are summed in fixed order). A pure function of the problem, never of the device or the run."""
    s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
    n, cin, *in_sp = (int(v) for v in in_shape)
    cout, _, *k = (int(v) for v in weight_shape)
    desc = _desc(n, cin, in_sp, cout, k, s, p, d)
    code = {"fwd": 0, "bwd-data": 1, "bwd-weight": 2}[direction]
    geom = (ctypes.c_int32 * 4)()
    _lib.check(_lib.lib().sfh_conv3d_launch_geometry(ctypes.byref(desc), _lib.dtype_code(dtype), code, geom), "launch_geometry")
    return {"kernel": KERNEL_NAMES[geom[0]], "voxels": int(geom[1]), "blocks": int(geom[2]), "slices": int(geom[3])}


def split_count(in_shape, weight_shape, stride, padding, dilation, dtype) -> int:
    """Number of fp32 partial slices the weight gradient reduces (1 = no workspace)."""
    s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
    n, cin, *in_sp = (int(v) for v in in_shape)
    cout, _, *k = (int(v) for v in weight_shape)
    desc = _desc(n, cin, in_sp, cout, k, s, p, d)
    return int(_lib.lib().sfh_conv3d_wgrad_splits(ctypes.byref(desc), _lib.dtype_code(dtype)))


def workspace_elements(splits: int, cout: int, cin: int, kernel: Sequence[int]) -> int:
    """fp32 elements :func:`conv3d_backward_weight` needs for ``splits`` partial slices."""
    k = _triple(kernel, "kernel")
    return int(splits) * int(cout) * int(cin) * k[0] * k[1] * k[2]


def grad_weight_empty(cout: int, cin: int, kernel: Sequence[int], *, dtype, device) -> torch.Tensor:
    """An empty ``(Cout, Cin, kd, kh, kw)`` gradient in the layout the kernel writes:
    ``[Cout][kd][kh][kw][Cin]`` in memory, i.e. ``channels_last_3d``."""
    k = _triple(kernel, "kernel")
    return torch.empty((cout, cin, *k), dtype=dtype, device=device, memory_format=_CL3D)


def bias_grad(grad_output: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Bias gradient of a (transposed) convolution: ``grad_output.sum((0, 2, 3, 4))`` with fp32 accumulation in a
    fixed order, rounded once to ``dtype`` (default: ``grad_output``'s) -- the expression the reference's autograd
    functions use (``ScaFFold/unet/conv3d.py:1231``, ``:1786``)."""
    if not isinstance(grad_output, torch.Tensor) or grad_output.dim() != 5 or not grad_output.is_cuda \
            or grad_output.dtype not in _lib.SUPPORTED_DTYPES:
        raise NotImplementedError(f"unsupported: grad_output={getattr(grad_output, 'shape', None)}/"
                                  f"{getattr(grad_output, 'dtype', None)}")
    out_dtype = grad_output.dtype if dtype is None else dtype
    if out_dtype not in _lib.SUPPORTED_DTYPES:
        raise NotImplementedError(f"unsupported bias dtype {out_dtype}")
    g = grad_output.contiguous(memory_format=_CL3D)
    n, c, d, h, w = (int(v) for v in g.shape)
    gb = torch.empty((c,), dtype=out_dtype, device=g.device)
    rows = n * d * h * w
    if rows == 0:
        return gb.zero_()
    L = _lib.lib()
    with _lib.device_guard(g.device):
        ws = _lib.workspace(int(L.sfh_bias_grad_workspace_bytes(rows, c)), g.device)
        rc = L.sfh_bias_grad(_lib.dtype_code(g.dtype), _lib.dtype_code(out_dtype), _lib.ptr(g), rows, c, _lib.ptr(gb),
                             _lib.ptr(ws), 0 if ws is None else ws.numel(), _lib.stream_ptr(g.device))
    _lib.check(rc, "bias_grad")
    return gb


_PACKED_BYTES_CACHE: dict = {}


def packed_weight_bytes(in_shape, weight_shape, stride, padding, dilation, dtype) -> tuple[int, int]:
    """Bytes of the packed weight the forward and the data gradient of this problem read (0 where a direction does
    not read one)."""
    s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
    key = (tuple(int(v) for v in in_shape), tuple(int(v) for v in weight_shape), s, p, d, dtype)
    hit = _PACKED_BYTES_CACHE.get(key)
    if hit is None:
        n, cin, *in_sp = key[0]
        cout, _, *k = key[1]
        desc = _desc(n, cin, in_sp, cout, k, s, p, d)
        L = _lib.lib()
        try:
            code = _lib.dtype_code(dtype)
            hit = (int(L.sfh_conv3d_packed_weight_bytes(ctypes.byref(desc), code, 0)),
                   int(L.sfh_conv3d_packed_weight_bytes(ctypes.byref(desc), code, 1)))
        except NotImplementedError:
            hit = (0, 0)
        if len(_PACKED_BYTES_CACHE) > 4096:
            _PACKED_BYTES_CACHE.clear()
        _PACKED_BYTES_CACHE[key] = hit
    return hit


_PACK_PLAN_CACHE: dict = {}


def _pack_plan(w, in_shape, stride, padding, dilation):
    key = (in_shape, w.shape, stride, padding, dilation, w.dtype)
    try:
        plan = _PACK_PLAN_CACHE.get(key)
    except TypeError:  # unhashable spelling of stride / padding / dilation
        key, plan = None, None
    if plan is None:
        s, p, d = _triple(stride, "stride"), _triple(padding, "padding"), _triple(dilation, "dilation")
        nbf, nbd = packed_weight_bytes(in_shape, w.shape, s, p, d, w.dtype)
        n, cin, *in_sp = (int(v) for v in in_shape)
        k = tuple(int(v) for v in w.shape[2:])
        plan = (nbf, nbd, _desc(n, cin, in_sp, int(w.shape[0]), k, s, p, d), _lib.dtype_code(w.dtype) if (nbf or nbd) else -1)
        if key is not None:
            if len(_PACK_PLAN_CACHE) > 4096:
                _PACK_PLAN_CACHE.clear()
            _PACK_PLAN_CACHE[key] = plan
    return plan


def pack_weights(w: torch.Tensor, in_shape, stride=1, padding=0, dilation=1, *, forward: bool = True, backward_data: bool = True,
                 out=None):
    """Packs ``w`` once, in one launch, for the forward and / or the data gradient of the convolution of an input of
    ``in_shape``: returns ``(packed_fwd, packed_dgrad)`` to pass as ``packed_weight=``; an entry is ``None`` when it
    was not asked for or when that direction of the problem does not read a packed weight (it then takes ``w``).
    ``out=(packed_fwd, packed_dgrad)`` reuses the buffers of an earlier call for the same problem.
    The default entry points repack on every call; a train step that packs once here saves a launch per convolution."""
    nbf, nbd, desc, code = _pack_plan(w, in_shape, stride, padding, dilation)
    if out is not None:
        pf, pd = out
        if (pf is not None and pf.numel() != nbf) or (pd is not None and pd.numel() != nbd):
            raise ValueError("pack_weights: out= buffers are not those of this problem")
    else:
        pf = torch.empty(nbf, dtype=torch.uint8, device=w.device) if (forward and nbf) else None
        pd = torch.empty(nbd, dtype=torch.uint8, device=w.device) if (backward_data and nbd) else None
    if pf is None and pd is None:
        return None, None
    with _lib.device_guard(w.device):
        rc = _lib.lib().sfh_conv3d_pack_weights(ctypes.byref(desc), code, _lib.ptr(w), _lib.strides5(w), _lib.ptr(pf), _lib.ptr(pd),
                                                _lib.stream_ptr(w.device))
    if rc:
        _lib.check(rc, "pack_weights")
    return pf, pd


class PackedWeights:
    """Both packed forms of one convolution weight for one problem, in buffers that live as long as this object, so
    that whoever changes the weight can refresh them in place (``repack`` / ``pack_weights_batch``).

    ``source`` is the tensor the forms were packed from; ``version`` is a stamp for the caller's own validity rule
    (``FastConv3d`` stores the version counter of the parameter there); ``maintained`` says that the writer of the
    weight refreshes the forms itself after every change."""

    __slots__ = ("source", "problem", "fwd", "dgrad", "version", "maintained")

    #: bumped whenever an instance is created or packs from another source: holders of batch plans rebuild on change
    generation = 0

    def __init__(self, w: torch.Tensor, in_shape, stride=1, padding=0, dilation=1):
        self.problem = (tuple(int(v) for v in in_shape), stride, padding, dilation)
        self.source = None
        self.version = None
        self.maintained = False
        self.fwd, self.dgrad = pack_weights(w, self.problem[0], stride, padding, dilation)
        self.source = w
        PackedWeights.generation += 1

    def __bool__(self):
        return self.fwd is not None or self.dgrad is not None

    def repack(self, w: Optional[torch.Tensor] = None) -> None:
        """Packs again from ``w`` (default: the same source) into the same buffers."""
        if w is not None and w is not self.source:
            if w.shape != self.source.shape or w.dtype is not self.source.dtype or w.device != self.source.device:
                raise ValueError("PackedWeights.repack: the new source is a different problem")
            self.source = w
            PackedWeights.generation += 1
        if self:
            pack_weights(self.source, self.problem[0], *self.problem[1:], out=(self.fwd, self.dgrad))


def pack_weights_batch(packs):
    """Refreshes many ``PackedWeights`` in as few launches as possible.  Returns a plan to pass back as ``packs`` the
    next time (it holds the prepared argument list; valid while no source tensor is replaced)."""
    if not isinstance(packs, _PackBatchPlan):
        packs = _PackBatchPlan(packs)
    packs.run()
    return packs


class _PackBatchPlan:
    def __init__(self, packs):
        self.generation = PackedWeights.generation
        groups = {}
        for e in packs:
            if e:
                groups.setdefault((e.source.device, e.source.dtype), []).append(e)
        self.groups = []
        for (device, dtype), entries in groups.items():
            items = (_lib.PackItem * len(entries))()
            for it, e in zip(items, entries):
                w = e.source
                _, _, desc, _ = _pack_plan(w, e.problem[0], *e.problem[1:])
                it.desc = desc
                it.w = w.data_ptr()
                for i, v in enumerate(_lib.strides5(w)):
                    it.w_stride[i] = v
                it.packed_fwd = None if e.fwd is None else e.fwd.data_ptr()
                it.packed_dgrad = None if e.dgrad is None else e.dgrad.data_ptr()
            # the entries are held so that the addresses in `items` stay valid
            self.groups.append((device, _lib.dtype_code(dtype), items, len(entries), entries))

    def run(self):
        L = _lib.lib()
        for device, code, items, n, _ in self.groups:
            with _lib.device_guard(device):
                rc = L.sfh_conv3d_pack_weights_batch(items, n, code, _lib.stream_ptr(device))
            if rc:
                _lib.check(rc, "pack_weights_batch")


# ---------------------------------------------------------------------------------------------
# forward
# ---------------------------------------------------------------------------------------------
def conv3d_forward(
    x: torch.Tensor,
    w: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    stride=1,
    padding=0,
    dilation=1,
    groups: int = 1,
    *,
    config=None,
    weight_rsck: Optional[torch.Tensor] = None,
    weight_flip: bool = False,
    out: Optional[torch.Tensor] = None,
    force_generic: bool = False,
    packed_weight: Optional[torch.Tensor] = None,
    gn_groups: int = 0,
    _checked: bool = False,
    _second: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Forward 3-D convolution; input and output are ``channels_last_3d``.

    The weight is read where it lies (its strides are handed to the library), so a
    ``channels_last_3d`` parameter, PyTorch's default layout and an RSCK copy all work without
    a host-side transform and give bitwise identical results.  ``weight_flip`` consumes the
    taps mirrored in all three axes (the data gradient's view of the weight).

    ``gn_groups > 0`` announces a GroupNorm of that many groups on the result: where the kernel that serves the problem
    offers it, the launch also leaves per-group Welford records (count, mean, M2) of its rounded output, which ride along
    as ``result._sfh_gn_partials`` and spare :func:`scaffold_amd.group_norm` its statistics pass. The result itself is the
    same bits either way, and the records are a function of the result alone (no state from earlier calls).
    """
    if not _checked and not is_supported(x, w, bias, stride, padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: x={tuple(getattr(x, 'shape', ()))}/{getattr(x, 'dtype', None)} "
            f"w={tuple(getattr(w, 'shape', ()))} stride={stride} padding={padding} dilation={dilation} groups={groups}"
        )
    _no_config(config)
    x = x.contiguous(memory_format=_CL3D)
    if _second is None:
        prob = _problem(x.shape, w.shape, stride, padding, dilation, x.dtype)
    else:  # conv3d_forward_pair: x holds the first channels of the input, _second the rest
        _second = _second.contiguous(memory_format=_CL3D)
        prob = _problem(_pair_shape(x, _second), w.shape, stride, padding, dilation, x.dtype)
    if out is None:
        y = torch.empty(prob.y_shape, device=x.device, dtype=x.dtype, memory_format=_CL3D)
    else:
        y = out
        _check_out(y, prob.y_shape, x)
    if weight_rsck is not None:
        _check_weight_rsck(weight_rsck, (*prob.k, prob.cin, prob.cout), x)
        w_eff = weight_rsck.permute(4, 3, 0, 1, 2)  # (Cout, Cin, kd, kh, kw) view of the RSCK buffer
    else:
        w_eff = w
    if weight_flip:
        w_eff = w_eff.flip(2, 3, 4)  # small copy; the data-gradient entry point flips inside the library instead
    if prob.n == 0:
        return y
    L = _lib.lib()
    desc, code = prob.desc, prob.code
    with _lib.device_guard(x.device):
        need = prob.workspace_bytes("fwd")
        flags = _flags(force_generic)
        if packed_weight is not None:
            # ``packed_weight`` comes from pack_weights() for this very problem: the library reads it in place of w
            if weight_rsck is not None or weight_flip or force_generic:
                raise ValueError("packed_weight= cannot be combined with weight_rsck=, weight_flip= or force_generic=")
            need -= prob.check_packed(packed_weight, False, x)
            flags |= _lib.SFH_FLAG_WEIGHT_PACKED
            w_eff = packed_weight
        ws = _lib.workspace(need, x.device)
        records = prob.gn_records(gn_groups) if gn_groups > 0 and not force_generic else 0
        if records > 0:
            partials = torch.empty(prob.n * records * gn_groups * 4, dtype=torch.float32, device=x.device)
            if _second is None:
                rc = L.sfh_conv3d_fwd_gn(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(w_eff),
                                         None if packed_weight is not None else _lib.strides5(w_eff), _lib.ptr(bias),
                                         _lib.ptr(y), _lib.ptr(ws), 0 if ws is None else ws.numel(), flags, int(gn_groups),
                                         _lib.ptr(partials), partials.numel() * 4, _lib.stream_ptr(x.device))
            else:
                rc = L.sfh_conv3d_fwd_pair(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(_second), int(x.shape[1]), _lib.ptr(w_eff),
                                           None if packed_weight is not None else _lib.strides5(w_eff), _lib.ptr(bias),
                                           _lib.ptr(y), _lib.ptr(ws), 0 if ws is None else ws.numel(), flags, int(gn_groups),
                                           _lib.ptr(partials), partials.numel() * 4, _lib.stream_ptr(x.device))
            if rc == _lib.SFH_ERR_UNSUPPORTED:  # e.g. an out= view off the 16-byte grid: the plain launch
                records = 0
            else:
                # valid for these bits of y only: the version lets the consumer see an in-place change
                y._sfh_gn_partials = (partials, records, int(gn_groups), y._version)
        if records == 0 and _second is not None:
            rc = L.sfh_conv3d_fwd_pair(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(_second), int(x.shape[1]), _lib.ptr(w_eff),
                                       None if packed_weight is not None else _lib.strides5(w_eff), _lib.ptr(bias),
                                       _lib.ptr(y), _lib.ptr(ws), 0 if ws is None else ws.numel(), flags, 0, None, 0,
                                       _lib.stream_ptr(x.device))
        elif records == 0:
            rc = L.sfh_conv3d_fwd(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(w_eff),
                                  None if packed_weight is not None else _lib.strides5(w_eff), _lib.ptr(bias),
                                  _lib.ptr(y), _lib.ptr(ws), 0 if ws is None else ws.numel(), flags, _lib.stream_ptr(x.device))
    _lib.check(rc, "conv3d_forward")
    return y


# ---------------------------------------------------------------------------------------------
# data gradient
# ---------------------------------------------------------------------------------------------
def conv3d_backward_data(
    grad_output: torch.Tensor,
    weight: torch.Tensor,
    input_shape: Sequence[int],
    stride=1,
    padding=0,
    dilation=1,
    groups: int = 1,
    *,
    config=None,
    weight_rsck: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    force_generic: bool = False,
    packed_weight: Optional[torch.Tensor] = None,
    _checked: bool = False,
    _cin_first: int = 0,
):
    """Gradient of a conv3d with respect to its input (stride 1 only).

    Computed as a gather over ``grad_output`` with the channel roles of the weight swapped, the
    taps mirrored and padding ``dil*(k-1) - p``; the swap and the mirror happen while the library
    repacks the weight, so no transformed copy of the weight is made here.
    """
    if not _checked and not is_supported_bwd_data(grad_output, weight, input_shape, stride, padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: grad_output={tuple(getattr(grad_output, 'shape', ()))}/{getattr(grad_output, 'dtype', None)} "
            f"w={tuple(getattr(weight, 'shape', ()))} input_shape={tuple(input_shape)} stride={stride} "
            f"padding={padding} dilation={dilation} groups={groups}"
        )
    _no_config(config)
    gy = grad_output.contiguous(memory_format=_CL3D)
    prob = _problem(input_shape if isinstance(input_shape, torch.Size) else tuple(input_shape), weight.shape, stride, padding,
                    dilation, gy.dtype)
    gx_shape = (prob.n, prob.cin, *prob.in_sp)
    gx_second = None
    if _cin_first:  # conv3d_backward_data_pair: the gradient as two tensors, cut at that channel
        gx = torch.empty((prob.n, _cin_first, *prob.in_sp), device=gy.device, dtype=gy.dtype, memory_format=_CL3D)
        gx_second = torch.empty((prob.n, prob.cin - _cin_first, *prob.in_sp), device=gy.device, dtype=gy.dtype, memory_format=_CL3D)
    elif out is None:
        gx = torch.empty(gx_shape, device=gy.device, dtype=gy.dtype, memory_format=_CL3D)
    else:
        gx = out
        _check_out(gx, gx_shape, gy)
    if weight_rsck is not None:
        _check_weight_rsck(weight_rsck, (*prob.k, prob.cin, prob.cout), gy)
        w_eff = weight_rsck.permute(4, 3, 0, 1, 2)
    else:
        w_eff = weight
    L = _lib.lib()
    desc, code = prob.desc, prob.code
    with _lib.device_guard(gy.device):
        need = prob.workspace_bytes("dgrad")
        flags = _flags(force_generic)
        if packed_weight is not None:
            if weight_rsck is not None or force_generic:
                raise ValueError("packed_weight= cannot be combined with weight_rsck= or force_generic=")
            need -= prob.check_packed(packed_weight, True, gy)
            flags |= _lib.SFH_FLAG_WEIGHT_PACKED
            w_eff = packed_weight
        ws = _lib.workspace(need, gy.device)
        if gx_second is None:
            rc = L.sfh_conv3d_dgrad(ctypes.byref(desc), code, _lib.ptr(gy), _lib.ptr(w_eff),
                                    None if packed_weight is not None else _lib.strides5(w_eff), _lib.ptr(gx),
                                    _lib.ptr(ws), 0 if ws is None else ws.numel(), flags, _lib.stream_ptr(gy.device))
        else:
            rc = L.sfh_conv3d_dgrad_pair(ctypes.byref(desc), code, _lib.ptr(gy), _lib.ptr(w_eff),
                                         None if packed_weight is not None else _lib.strides5(w_eff), _lib.ptr(gx), _lib.ptr(gx_second),
                                         int(_cin_first), _lib.ptr(ws), 0 if ws is None else ws.numel(), flags,
                                         _lib.stream_ptr(gy.device))
    _lib.check(rc, "conv3d_backward_data")
    return gx if gx_second is None else (gx, gx_second)


# ---------------------------------------------------------------------------------------------
# weight gradient
# ---------------------------------------------------------------------------------------------
def _validate_gw_out(gw: torch.Tensor, cout: int, cin: int, k, dtype, device) -> Optional[str]:
    want_shape = (cout, cin, *k)
    if tuple(gw.shape) != want_shape:
        return f"shape must be {want_shape} (Cout x Cin x kernel); got {tuple(gw.shape)}"
    if gw.device != device:
        return f"device must be {device}; got {gw.device}"
    if gw.dtype != dtype:
        return f"dtype must match the operands' {dtype}; got {gw.dtype}"
    taps = k[0] * k[1] * k[2]
    want = (taps * cin, 1, k[1] * k[2] * cin, k[2] * cin, cin)
    got = tuple(gw.stride())
    # A size-1 dimension's stride is unobservable; compare only the ones that matter.
    if not all(g == w for g, w, extent in zip(got, want, want_shape) if extent > 1):
        return f"must have channels_last_3d strides ([Cout][tap][Cin] in memory); want {want}, got {got}"
    return None


def conv3d_backward_weight(
    input: torch.Tensor,
    weight_shape: Sequence[int],
    grad_output: torch.Tensor,
    stride=1,
    padding=0,
    dilation=1,
    groups: int = 1,
    *,
    deterministic: bool = True,
    config=None,
    workspace: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    force_generic: bool = False,
    grad_dtype: Optional[torch.dtype] = None,
    _checked: bool = False,
    _second: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Gradient of a conv3d with respect to its weight, returned ``channels_last_3d``.

    Split-K over the output voxels with fp32 partial slices at fixed workspace slots and an
    ordered reduction; there is no atomic variant, so ``deterministic=False`` is refused rather
    than silently served by the deterministic path.  ``grad_dtype=torch.float32`` with 16-bit operands returns
    the fp32 sum of the slices unrounded (the gradient of an fp32 master weight under autocast, without the
    rounding and the up-cast); shapes only the untiled kernel serves raise ``NotImplementedError`` for it.
    """
    if not _checked and not is_supported_bwd_weight(input, weight_shape, grad_output, stride, padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: input={tuple(getattr(input, 'shape', ()))}/{getattr(input, 'dtype', None)} "
            f"weight_shape={tuple(weight_shape)} grad_output={tuple(getattr(grad_output, 'shape', ()))} "
            f"stride={stride} padding={padding} dilation={dilation} groups={groups}"
        )
    _no_config(config)
    if not deterministic:
        raise NotImplementedError("deterministic=False: this library has no atomic weight-gradient path")
    x = input.contiguous(memory_format=_CL3D)
    gy = grad_output.contiguous(memory_format=_CL3D)
    if _second is not None:  # conv3d_backward_weight_pair: x holds the first channels of the input, _second the rest
        _second = _second.contiguous(memory_format=_CL3D)
    prob = _problem(x.shape if _second is None else _pair_shape(x, _second),
                    weight_shape if isinstance(weight_shape, torch.Size) else tuple(weight_shape), stride, padding, dilation, x.dtype)
    cout, cin, k, n = prob.cout, prob.cin, prob.k, prob.n
    gdt = x.dtype if grad_dtype is None else grad_dtype
    if gdt is not x.dtype and gdt is not torch.float32:
        raise ValueError(f"grad_dtype must be the operands' dtype or torch.float32, got {grad_dtype}")
    if out is None:
        gw = torch.empty((cout, cin, *k), dtype=gdt, device=x.device, memory_format=_CL3D)
    else:
        gw = out
        why = _validate_gw_out(gw, cout, cin, tuple(k), gdt, x.device)
        if why is not None:
            raise ValueError(f"out= is not usable for this problem: {why}")
    L = _lib.lib()
    desc, code = prob.desc, prob.code
    if n == 0:
        return gw.zero_()
    with _lib.device_guard(x.device):
        need = 0 if force_generic else prob.workspace_bytes("wgrad")
        if workspace is None:
            ws = _lib.workspace(need, x.device)
            ws_bytes = 0 if ws is None else ws.numel()
        else:
            have = workspace.numel() * workspace.element_size()
            if workspace.dtype is not torch.float32 or have < need or workspace.device != x.device \
                    or not workspace.is_contiguous():
                splits = int(L.sfh_conv3d_wgrad_splits(ctypes.byref(desc), code))
                raise ValueError(
                    f"workspace must be a contiguous float32 tensor on {x.device} of at least {need // 4} elements "
                    f"({need / 2**20:.1f} MiB) -- {splits} splits x {cout} Cout x {k[0] * k[1] * k[2]} taps x {cin} Cin; "
                    f"got {workspace.numel()} of {workspace.dtype}"
                )
            ws, ws_bytes = workspace, have
        flags = _flags(force_generic) | (_lib.SFH_FLAG_GRAD_FP32 if gdt is not x.dtype else 0)
        if _second is None:
            rc = L.sfh_conv3d_wgrad(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(gy), _lib.ptr(gw), _lib.ptr(ws), ws_bytes,
                                    flags, _lib.stream_ptr(x.device))
        else:
            rc = L.sfh_conv3d_wgrad_pair(ctypes.byref(desc), code, _lib.ptr(x), _lib.ptr(_second), int(x.shape[1]), _lib.ptr(gy),
                                         _lib.ptr(gw), _lib.ptr(ws), ws_bytes, flags, _lib.stream_ptr(x.device))
    _lib.check(rc, "conv3d_backward_weight")
    return gw


WGRAD_BATCH_MAX = 16  # SFH_WGRAD_BATCH_MAX


def weight_grad_batch_family(input_shape, weight_shape, stride, padding, dilation, dtype) -> int:
    """Which launch of :func:`conv3d_backward_weight_batch` takes this problem: 1, the one of the problems with output rows of
    more than 16 voxels; 2, the one of the small volumes (at most 32 tiles of 256 voxels); 0, neither (it is not 3x3x3 at
    unit stride and dilation in bf16 / fp16 with channel counts multiples of 32, or fits neither family).  A pure function
    of the problem."""
    if dtype not in (torch.bfloat16, torch.float16):
        return 0
    try:
        prob = _problem(torch.Size(input_shape), torch.Size(weight_shape), stride, padding, dilation, dtype)
    except (ValueError, NotImplementedError):
        return 0
    if prob.n == 0:
        return 0
    return int(_lib.lib().sfh_conv3d_wgrad_batch_supported(ctypes.byref(prob.desc), prob.code))


def weight_grad_batchable(input_shape, weight_shape, stride, padding, dilation, dtype) -> bool:
    """Whether :func:`conv3d_backward_weight_batch` takes this problem (see :func:`weight_grad_batch_family`)."""
    return weight_grad_batch_family(input_shape, weight_shape, stride, padding, dilation, dtype) != 0


def conv3d_backward_weight_batch(problems, *, grad_dtype: Optional[torch.dtype] = None, outs=None, share_device: bool = False):
    """The weight gradients of several convolutions from one launch of the weight-gradient kernel and one sum pass.

    ``problems``: a sequence of ``(input, weight_shape, grad_output, padding)`` or ``((first, second), weight_shape,
    grad_output, padding)`` -- the arguments of :func:`conv3d_backward_weight` / :func:`conv3d_backward_weight_pair` at unit
    stride and dilation -- every one of them a problem :func:`weight_grad_batchable` accepts, all of one dtype and device.
    What a single launch costs whatever the problem (first fetch, slices written and read back, launch gaps: 15-20 us on
    MI355X) is paid once for the list.  Returns the gradients (``channels_last_3d``, ``grad_dtype`` or the operands' dtype)
    in order; ``outs`` supplies the tensors to write.  Each gradient is a fixed-order fp32 sum that depends on the LIST of
    shapes only: the same bits on every run, within summation-order rounding of the one-problem call's.

    ``share_device``: the launch of the problems with rows of more than 16 voxels takes half of the compute units -- for a
    batch issued on a stream of its own while the current stream has other work (the deferred weight gradients of a
    backward pass, see ``modules.flush_weight_gradients``)."""
    problems = list(problems)
    if not problems:
        return []
    L = _lib.lib()
    keep, gws = [], []
    dev = dt = None
    for i, (inp, wshape, gy, padding) in enumerate(problems):
        first, second = inp if isinstance(inp, (tuple, list)) else (inp, None)
        x = first.contiguous(memory_format=_CL3D)
        x2 = None if second is None else second.contiguous(memory_format=_CL3D)
        g = gy.contiguous(memory_format=_CL3D)
        if dev is None:
            dev, dt = x.device, x.dtype
        if x.device != dev or x.dtype is not dt or g.dtype is not dt or g.device != dev or (x2 is not None and (x2.dtype is not dt or x2.device != dev)):
            raise ValueError("conv3d_backward_weight_batch: all operands share one dtype and one device")
        in_shape = x.shape if x2 is None else _pair_shape(x, x2)
        wshape = wshape if isinstance(wshape, torch.Size) else torch.Size(wshape)
        prob = _problem(in_shape, wshape, 1, padding, 1, dt)
        if tuple(g.shape) != tuple(prob.y_shape):
            raise ValueError(f"conv3d_backward_weight_batch: problem {i}: grad_output {tuple(g.shape)} does not match {tuple(prob.y_shape)}")
        gdt = dt if grad_dtype is None else grad_dtype
        if gdt is not dt and gdt is not torch.float32:
            raise ValueError(f"grad_dtype must be the operands' dtype or torch.float32, got {grad_dtype}")
        if outs is None:
            gw = torch.empty((prob.cout, prob.cin, *prob.k), dtype=gdt, device=dev, memory_format=_CL3D)
        else:
            gw = outs[i]
            why = _validate_gw_out(gw, prob.cout, prob.cin, tuple(prob.k), gdt, dev)
            if why is not None:
                raise ValueError(f"outs[{i}] is not usable for this problem: {why}")
        keep.append((prob, x, x2, g))
        gws.append(gw)
    flags = _lib.SFH_FLAG_GRAD_FP32 if (grad_dtype is not None and grad_dtype is not dt) else 0
    if share_device:
        flags |= _lib.SFH_FLAG_SHARE_DEVICE
    # calls of at most WGRAD_BATCH_MAX problems, filled family by family (the problems of a family share a launch)
    family = [int(L.sfh_conv3d_wgrad_batch_supported(ctypes.byref(k[0].desc), k[0].code)) for k in keep]
    if 0 in family:
        raise NotImplementedError(f"conv3d_backward_weight_batch: problem {family.index(0)} of the list is not served in a batch "
                                  "(weight_grad_batchable says which)")
    calls = []
    for f in (1, 2):
        members = [i for i in range(len(keep)) if family[i] == f]
        calls += [members[lo:lo + WGRAD_BATCH_MAX] for lo in range(0, len(members), WGRAD_BATCH_MAX)]
    with _lib.device_guard(dev):
        for idx in calls:
            part = [keep[i] for i in idx]
            items = (_lib.WgradItem * len(part))()
            for it, (prob, x, x2, g), gw in zip(items, part, [gws[i] for i in idx]):
                it.desc = prob.desc
                it.x, it.x_second, it.cin_first = _lib.ptr(x), (None if x2 is None else _lib.ptr(x2)), (0 if x2 is None else int(x.shape[1]))
                it.gy, it.gw = _lib.ptr(g), _lib.ptr(gw)
            code = part[0][0].code
            need = int(L.sfh_conv3d_wgrad_batch_workspace_bytes(items, len(part), code, flags))
            if need == 0:
                raise NotImplementedError("conv3d_backward_weight_batch: a problem of the list is not served in a batch "
                                          "(weight_grad_batchable says which)")
            ws = _lib.workspace(need, dev)
            _lib.check(L.sfh_conv3d_wgrad_batch(items, len(part), code, _lib.ptr(ws), need, flags, _lib.stream_ptr(dev)),
                       "conv3d_backward_weight_batch")
    return gws


def conv3d_backward_weight_bias(input: torch.Tensor, weight_shape: Sequence[int], grad_output: torch.Tensor, stride=1, padding=0,
                                dilation=1, groups: int = 1, *, grad_dtype: Optional[torch.dtype] = None, _checked: bool = False):
    """``(grad_weight, grad_bias)`` from ONE pass over ``grad_output`` where the kernel that serves the problem reads it tile
    by tile anyway (the 1x1x1 convolutions with few output channels: the U-Net's head): the weight gradient of
    :func:`conv3d_backward_weight` (same bits) and ``grad_output.sum((0, 2, 3, 4))`` (``ScaFFold/unet/conv3d.py:1231``; fp32
    slices summed in a fixed order, one rounding), both in ``grad_dtype`` (default: the operands' dtype).  ``None`` where the
    library does not offer the fused form: the caller then computes the two apart."""
    if not _checked and not is_supported_bwd_weight(input, weight_shape, grad_output, stride, padding, dilation, groups):
        raise NotImplementedError(
            f"unsupported: input={tuple(getattr(input, 'shape', ()))}/{getattr(input, 'dtype', None)} "
            f"weight_shape={tuple(weight_shape)} grad_output={tuple(getattr(grad_output, 'shape', ()))}")
    x = input.contiguous(memory_format=_CL3D)
    gy = grad_output.contiguous(memory_format=_CL3D)
    prob = _problem(x.shape, weight_shape if isinstance(weight_shape, torch.Size) else tuple(weight_shape), stride, padding,
                    dilation, x.dtype)
    if prob.n == 0:
        return None
    need = prob.workspace_bytes("wgrad_bias")
    if need == 0:
        return None
    gdt = x.dtype if grad_dtype is None else grad_dtype
    if gdt is not x.dtype and gdt is not torch.float32:
        raise ValueError(f"grad_dtype must be the operands' dtype or torch.float32, got {grad_dtype}")
    gw = torch.empty((prob.cout, prob.cin, *prob.k), dtype=gdt, device=x.device, memory_format=_CL3D)
    gb = torch.empty((prob.cout,), dtype=gdt, device=x.device)
    with _lib.device_guard(x.device):
        ws = _lib.workspace(need, x.device)
        rc = _lib.lib().sfh_conv3d_wgrad_bias(ctypes.byref(prob.desc), prob.code, _lib.ptr(x), _lib.ptr(gy), _lib.ptr(gw), _lib.ptr(gb),
                                              _lib.ptr(ws), need, _lib.SFH_FLAG_GRAD_FP32 if gdt is not x.dtype else 0,
                                              _lib.stream_ptr(x.device))
    if rc == _lib.SFH_ERR_UNSUPPORTED:  # e.g. operands off the 16-byte grid
        return None
    _lib.check(rc, "conv3d_backward_weight_bias")
    return gw, gb


# ---------------------------------------------------------------------------------------------
# a convolution over two tensors whose channels follow each other
# ---------------------------------------------------------------------------------------------
def _pair_shape(first: torch.Tensor, second: torch.Tensor) -> torch.Size:
    return torch.Size((first.shape[0], first.shape[1] + second.shape[1], *first.shape[2:]))


_PAIR_GATE: dict = {}


def is_supported_pair(x_first, x_second, w, bias=None, stride=1, padding=0, dilation=1) -> bool:
    """Whether all three directions of ``conv3d(torch.cat([x_first, x_second], 1), w)`` are served from the two tensors
    themselves (:func:`conv3d_forward_pair` and its two gradients).  Total: never raises."""
    try:
        if not isinstance(x_first, torch.Tensor) or not isinstance(x_second, torch.Tensor) or x_first.dim() != 5 or x_second.dim() != 5:
            return False
        if x_first.dtype is not x_second.dtype or x_first.device != x_second.device:
            return False
        if x_first.shape[0] != x_second.shape[0] or x_first.shape[2:] != x_second.shape[2:] or x_first.shape[0] < 1:
            return False
        shape = _pair_shape(x_first, x_second)
        stand_in = x_first.new_empty((1, 1, 1, 1, 1)).expand(shape)  # metadata only
        if not is_supported_all(stand_in, w, bias, stride, padding, dilation, 1):
            return False
        key = (shape, int(x_first.shape[1]), w.shape, stride, padding, dilation, x_first.dtype)
        hit = _PAIR_GATE.get(key)
        if hit is None:
            prob = _problem(shape, w.shape, stride, padding, dilation, x_first.dtype)
            L = _lib.lib()
            hit = all(L.sfh_conv3d_pair_supported(ctypes.byref(prob.desc), prob.code, int(x_first.shape[1]), d) == 1 for d in (0, 1, 2))
            if len(_PAIR_GATE) > 4096:
                _PAIR_GATE.clear()
            _PAIR_GATE[key] = hit
        return hit
    except (TypeError, ValueError, AttributeError, RuntimeError, NotImplementedError):
        return False


def _refuse_pair(x_first, x_second, w):
    raise NotImplementedError(
        f"unsupported pair: x_first={tuple(getattr(x_first, 'shape', ()))}/{getattr(x_first, 'dtype', None)} "
        f"x_second={tuple(getattr(x_second, 'shape', ()))} w={tuple(getattr(w, 'shape', ()))}: concatenate and use conv3d_forward")


def conv3d_forward_pair(x_first, x_second, w, bias=None, stride=1, padding=0, dilation=1, *, packed_weight=None, gn_groups: int = 0,
                        _checked: bool = False) -> torch.Tensor:
    """``conv3d_forward(torch.cat([x_first, x_second], 1), w, ...)`` without the concatenation
    (``ScaFFold/unet/unet_parts.py:107-120`` writes that tensor for the decoder's first convolution): the kernel stages each
    32-channel chunk of its reduction from the tensor that holds it.  Same bits as the call on the concatenated tensor;
    ``packed_weight`` / ``gn_groups`` as there.  ``NotImplementedError`` where :func:`is_supported_pair` says no."""
    if not _checked and not is_supported_pair(x_first, x_second, w, bias, stride, padding, dilation):
        _refuse_pair(x_first, x_second, w)
    return conv3d_forward(x_first, w, bias, stride, padding, dilation, 1, packed_weight=packed_weight, gn_groups=gn_groups,
                          _checked=True, _second=x_second)


def conv3d_backward_data_pair(grad_output, weight, input_shape, cin_first: int, stride=1, padding=0, dilation=1, *,
                              packed_weight=None, _checked: bool = False):
    """The data gradient of that convolution as the two tensors the concatenation's backward would have split it into:
    ``(grad_first, grad_second)`` with ``cin_first`` and ``Cin - cin_first`` channels; ``input_shape`` is the
    concatenation's.  Same bits as ``conv3d_backward_data(...)`` split along the channels."""
    cin_first = int(cin_first)
    if not _checked:
        shape = tuple(int(v) for v in input_shape)
        ok = isinstance(grad_output, torch.Tensor) and len(shape) == 5 and 0 < cin_first < shape[1] and \
            is_supported_bwd_data(grad_output, weight, shape, stride, padding, dilation, 1)
        if ok:
            prob = _problem(torch.Size(shape), weight.shape, stride, padding, dilation, grad_output.dtype)
            ok = _lib.lib().sfh_conv3d_pair_supported(ctypes.byref(prob.desc), prob.code, cin_first, 1) == 1
        if not ok:
            raise NotImplementedError(f"unsupported pair: grad_output={tuple(getattr(grad_output, 'shape', ()))} "
                                      f"input_shape={tuple(input_shape)} cut at channel {cin_first}")
    return conv3d_backward_data(grad_output, weight, input_shape, stride, padding, dilation, 1, packed_weight=packed_weight,
                                _checked=True, _cin_first=cin_first)


def conv3d_backward_weight_pair(x_first, x_second, weight_shape, grad_output, stride=1, padding=0, dilation=1, *,
                                grad_dtype=None, _checked: bool = False) -> torch.Tensor:
    """``conv3d_backward_weight(torch.cat([x_first, x_second], 1), ...)`` without the concatenation; same bits."""
    if not _checked:
        ok = isinstance(x_first, torch.Tensor) and isinstance(x_second, torch.Tensor) and x_first.dim() == 5 and x_second.dim() == 5 \
            and x_first.dtype is x_second.dtype and x_first.device == x_second.device and x_first.shape[0] == x_second.shape[0] \
            and x_first.shape[2:] == x_second.shape[2:]
        if ok:
            shape = _pair_shape(x_first, x_second)
            stand_in = x_first.new_empty((1, 1, 1, 1, 1)).expand(shape)
            ok = is_supported_bwd_weight(stand_in, tuple(weight_shape), grad_output, stride, padding, dilation, 1)
        if ok:
            prob = _problem(shape, torch.Size(tuple(weight_shape)), stride, padding, dilation, x_first.dtype)
            ok = _lib.lib().sfh_conv3d_pair_supported(ctypes.byref(prob.desc), prob.code, int(x_first.shape[1]), 2) == 1
        if not ok:
            _refuse_pair(x_first, x_second, None)
    return conv3d_backward_weight(x_first, weight_shape, grad_output, stride, padding, dilation, 1, grad_dtype=grad_dtype,
                                  _checked=True, _second=x_second)
