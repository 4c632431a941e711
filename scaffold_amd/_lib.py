"""ctypes binding of ``libscaffold_hip.so`` (the C ABI declared in ``include/scaffold_hip.h``).

The library is the product: there is no Python or CPU fallback behind it.  If the shared
object has not been built, :func:`lib` raises ``ScaffoldLibraryError`` with the build command,
and every op that needs it fails with that error.

Error codes map onto the exception classes the reference's entry points raise
(``triton_conv3d/gather_gemm.py:1228-1232``, ``ScaFFold/unet/triton_group_norm.py:253-277``):
``SFH_ERR_UNSUPPORTED`` -> ``NotImplementedError``, ``SFH_ERR_INVALID`` / ``SFH_ERR_WORKSPACE``
-> ``ValueError``, ``SFH_ERR_LAUNCH`` -> :class:`ScaffoldKernelError`.
"""

from __future__ import annotations

import ctypes
import os
import threading
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_size_t, c_uint32, c_void_p

import torch

__all__ = [
    "ScaffoldLibraryError",
    "ScaffoldKernelError",
    "lib",
    "lib_path",
    "check",
    "ConvDesc",
    "ConvTDesc",
    "GroupNormDesc",
    "LossDesc",
    "PoolDesc",
    "AdamDesc",
    "HaloDesc",
    "dtype_code",
    "SUPPORTED_DTYPES",
    "EXPORTED_SYMBOLS",
]

SFH_OK, SFH_ERR_INVALID, SFH_ERR_UNSUPPORTED, SFH_ERR_WORKSPACE, SFH_ERR_LAUNCH = range(5)
SFH_FLAG_FORCE_GENERIC = 1
SFH_FLAG_GRAD_FP32 = 2
SFH_FLAG_WEIGHT_PACKED = 4
SFH_FLAG_SHARE_DEVICE = 8

_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
SUPPORTED_DTYPES = tuple(_DTYPE_CODE)


class ScaffoldLibraryError(RuntimeError):
    """libscaffold_hip.so is missing or does not export the declared ABI."""


class ScaffoldKernelError(RuntimeError):
    """The HIP runtime refused a kernel launch (distinct from a contract violation)."""


class ConvDesc(ctypes.Structure):
    _fields_ = [(k, c_int32) for k in (
        "n", "cin", "in_d", "in_h", "in_w", "cout", "kd", "kh", "kw",
        "sd", "sh", "sw", "pd", "ph", "pw", "dd", "dh", "dw")]


class PackItem(ctypes.Structure):
    _fields_ = [("desc", ConvDesc), ("w", c_void_p), ("w_stride", c_int64 * 5), ("packed_fwd", c_void_p),
                ("packed_dgrad", c_void_p)]


class WgradItem(ctypes.Structure):
    _fields_ = [("desc", ConvDesc), ("x", c_void_p), ("x_second", c_void_p), ("cin_first", c_int32), ("gy", c_void_p),
                ("gw", c_void_p)]


class ConvTDesc(ctypes.Structure):
    _fields_ = [(k, c_int32) for k in ("n", "cin", "in_d", "in_h", "in_w", "cout", "kd", "kh", "kw")]


class ConcatDesc(ctypes.Structure):
    _fields_ = [("n", c_int32), ("c_a", c_int32), ("c_b", c_int32), ("rows", c_int64), ("halo_rows", c_int64)]


class IngestDesc(ctypes.Structure):
    _fields_ = [("n", c_int32), ("c", c_int32), ("mask_signed", c_int32), ("rows", c_int64), ("halo_rows", c_int64)]


class LossDesc(ctypes.Structure):
    _fields_ = [("n", c_int32), ("classes", c_int32), ("spatial", c_int64), ("eps", c_float)]


class PoolDesc(ctypes.Structure):
    _fields_ = [(k, c_int32) for k in ("n", "c", "in_d", "in_h", "in_w")]


class HaloDesc(ctypes.Structure):
    _fields_ = [(k, c_int32) for k in ("n", "c", "d", "h", "w", "halo")]


class AdamDesc(ctypes.Structure):
    _fields_ = [(k, c_float) for k in ("lr", "beta1", "beta2", "eps", "weight_decay", "max_norm")] + [("shadow_dtype", c_int32)]


class GroupNormDesc(ctypes.Structure):
    _fields_ = [("n", c_int32), ("c", c_int32), ("groups", c_int32), ("relu", c_int32),
                ("spatial", c_int64), ("eps", c_float)]


_I64x5 = c_int64 * 5

# name -> (restype, argtypes); every symbol include/scaffold_hip.h declares.
_SIGNATURES = {
    "sfh_version": (c_int, []),
    "sfh_last_error": (c_char_p, []),
    "sfh_device_info": (c_int, [c_char_p, c_size_t, POINTER(c_int32), POINTER(c_int32)]),
    "sfh_tuned_compute_units": (c_int, []),
    "sfh_conv3d_out_shape": (c_int, [POINTER(ConvDesc), POINTER(c_int32)]),
    "sfh_conv3d_uses_mfma": (c_int, [POINTER(ConvDesc), c_int, c_int]),
    "sfh_conv3d_launch_geometry": (c_int, [POINTER(ConvDesc), c_int, c_int, POINTER(c_int32)]),
    "sfh_mfma_ceiling_probe_flops": (c_double, [c_int32, c_int32]),
    "sfh_mfma_ceiling_probe": (c_int, [c_int32, c_int32, c_int32, c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_void_p]),
    "sfh_conv3d_fwd_workspace_bytes": (c_size_t, [POINTER(ConvDesc), c_int]),
    "sfh_conv3d_fwd": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_void_p,
                               c_void_p, c_size_t, c_uint32, c_void_p]),
    "sfh_conv3d_fwd_gn_records": (c_int32, [POINTER(ConvDesc), c_int, c_int]),
    "sfh_conv3d_fwd_gn": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_void_p,
                                  c_void_p, c_size_t, c_uint32, c_int, c_void_p, c_size_t, c_void_p]),
    "sfh_conv3d_dgrad_workspace_bytes": (c_size_t, [POINTER(ConvDesc), c_int]),
    "sfh_conv3d_dgrad": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_void_p,
                                 c_size_t, c_uint32, c_void_p]),
    "sfh_conv3d_packed_weight_bytes": (c_size_t, [POINTER(ConvDesc), c_int, c_int]),
    "sfh_conv3d_pack_weights": (c_int, [POINTER(ConvDesc), c_int, c_void_p, POINTER(c_int64), c_void_p, c_void_p, c_void_p]),
    "sfh_conv3d_pack_weights_batch": (c_int, [POINTER(PackItem), c_int32, c_int, c_void_p]),
    "sfh_conv3d_wgrad_splits": (c_int, [POINTER(ConvDesc), c_int]),
    "sfh_conv3d_wgrad_workspace_bytes": (c_size_t, [POINTER(ConvDesc), c_int]),
    "sfh_conv3d_wgrad": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_uint32,
                                 c_void_p]),
    "sfh_conv3d_pair_supported": (c_int, [POINTER(ConvDesc), c_int, c_int32, c_int]),
    "sfh_conv3d_fwd_pair": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, c_int32, c_void_p, POINTER(c_int64), c_void_p,
                                    c_void_p, c_void_p, c_size_t, c_uint32, c_int, c_void_p, c_size_t, c_void_p]),
    "sfh_conv3d_dgrad_pair": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_void_p, c_int32,
                                      c_void_p, c_size_t, c_uint32, c_void_p]),
    "sfh_conv3d_wgrad_batch_supported": (c_int, [POINTER(ConvDesc), c_int]),
    "sfh_conv3d_wgrad_batch_workspace_bytes": (c_size_t, [POINTER(WgradItem), c_int32, c_int, c_uint32]),
    "sfh_conv3d_wgrad_batch": (c_int, [POINTER(WgradItem), c_int32, c_int, c_void_p, c_size_t, c_uint32, c_void_p]),
    "sfh_conv3d_wgrad_pair": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_size_t,
                                      c_uint32, c_void_p]),
    "sfh_convT3d_fwd_workspace_bytes": (c_size_t, [POINTER(ConvTDesc), c_int]),
    "sfh_convT3d_fwd": (c_int, [POINTER(ConvTDesc), c_int, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_void_p,
                                c_void_p, c_size_t, c_uint32, c_void_p]),
    "sfh_conv3d_wgrad_bias_workspace_bytes": (c_size_t, [POINTER(ConvDesc), c_int]),
    "sfh_conv3d_wgrad_bias": (c_int, [POINTER(ConvDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_uint32,
                                      c_void_p]),
    "sfh_convT3d_wgrad_bias_workspace_bytes": (c_size_t, [POINTER(ConvTDesc), c_int]),
    "sfh_convT3d_wgrad_bias": (c_int, [POINTER(ConvTDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_uint32,
                                       c_void_p]),
    "sfh_convT3d_fwd_slab": (c_int, [POINTER(ConvTDesc), c_int, c_void_p, c_void_p, POINTER(c_int64), c_void_p, c_void_p, c_int64,
                                     c_void_p, c_size_t, c_uint32, c_void_p]),
    "sfh_groupnorm_fwd_workspace_bytes": (c_size_t, [POINTER(GroupNormDesc), c_int]),
    "sfh_groupnorm_fwd": (c_int, [POINTER(GroupNormDesc), c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "sfh_groupnorm_fwd_noalloc_max_bytes": (c_size_t, []),
    "sfh_groupnorm_fwd_noalloc_prepare": (c_int, []),
    "sfh_groupnorm_fwd_noalloc": (c_int, [POINTER(GroupNormDesc), c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p]),
    "sfh_shard_ingest": (c_int, [POINTER(IngestDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_skip_concat_fwd": (c_int, [POINTER(ConcatDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_skip_concat_bwd": (c_int, [POINTER(ConcatDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_groupnorm_fwd_slab": (c_int, [POINTER(GroupNormDesc), c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "sfh_groupnorm_fwd_from_partials": (c_int, [POINTER(GroupNormDesc), c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                                c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_int32, c_void_p]),
    "sfh_groupnorm_bwd_workspace_bytes": (c_size_t, [POINTER(GroupNormDesc), c_int]),
    "sfh_groupnorm_bwd": (c_int, [POINTER(GroupNormDesc), c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "sfh_bias_grad_workspace_bytes": (c_size_t, [c_int64, c_int32]),
    "sfh_bias_grad": (c_int, [c_int, c_int, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_size_t, c_void_p]),
    "sfh_ce_dice_workspace_bytes": (c_size_t, [POINTER(LossDesc)]),
    "sfh_ce_dice_fwd": (c_int, [POINTER(LossDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                c_void_p]),
    "sfh_ce_dice_bwd": (c_int, [POINTER(LossDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_maxpool2_fwd": (c_int, [POINTER(PoolDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_maxpool2_fwd_slab": (c_int, [POINTER(PoolDesc), c_int, c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "sfh_maxpool2_bwd": (c_int, [POINTER(PoolDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_maxpool2_bwd_add": (c_int, [POINTER(PoolDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_halo_assemble": (c_int, [POINTER(HaloDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_halo_pack": (c_int, [POINTER(HaloDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_halo_accumulate": (c_int, [POINTER(HaloDesc), c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sfh_adam_slots": (c_int64, [c_int32, POINTER(c_int64)]),
    "sfh_adam_grad_sumsq": (c_int, [c_int32, POINTER(c_void_p), POINTER(c_int64), c_void_p, c_void_p, c_void_p]),
    "sfh_adam_clip_step": (c_int, [POINTER(AdamDesc), c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                   POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "sfh_stream_copy": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lock = threading.Lock()
_lib = None


def lib_path() -> str:
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "libscaffold_hip.so")


def lib() -> ctypes.CDLL:
    """The loaded library; raises :class:`ScaffoldLibraryError` if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = lib_path()
        if not os.path.exists(path):
            raise ScaffoldLibraryError(
                f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C scaffold_amd/csrc -j8` (needs hipcc, targets gfx950). There is no fallback path."
            )
        try:
            handle = ctypes.CDLL(path)
        except OSError as exc:  # missing ROCm runtime, wrong arch, ...
            raise ScaffoldLibraryError(f"cannot load {path}: {exc}") from exc
        for name, (restype, argtypes) in _SIGNATURES.items():
            try:
                fn = getattr(handle, name)
            except AttributeError as exc:
                raise ScaffoldLibraryError(f"{path} does not export {name}; rebuild it") from exc
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
        return _lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise NotImplementedError(f"unsupported dtype {dtype}; supported: {SUPPORTED_DTYPES}") from None


def check(rc: int, what: str) -> None:
    """Turn a non-zero return code into the matching exception."""
    if rc == SFH_OK:
        return
    msg = lib().sfh_last_error()
    msg = msg.decode("utf-8", "replace") if msg else "unknown error"
    text = f"{what}: {msg}"
    if rc == SFH_ERR_UNSUPPORTED:
        raise NotImplementedError(text)
    if rc in (SFH_ERR_INVALID, SFH_ERR_WORKSPACE):
        raise ValueError(text)
    raise ScaffoldKernelError(text)


def strides5(t: torch.Tensor):
    return _I64x5(*[int(s) for s in t.stride()])


_devices_seen: set = set()


def _note_device(device: torch.device) -> None:
    """Once per device: compares its compute-unit count with the one the library's launch geometry is written for.
    Split counts are functions of the problem shape and that compiled-in count, so results do not depend on the device;
    on a device of another size the geometry is only not the best one, which is worth a warning, not an error."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index in _devices_seen:
        return
    _devices_seen.add(index)
    units, lds = c_int32(0), c_int32(0)
    with torch.cuda.device(index):
        rc = lib().sfh_device_info(None, 0, ctypes.byref(units), ctypes.byref(lds))
    tuned = int(lib().sfh_tuned_compute_units())
    if rc == SFH_OK and units.value != tuned:
        import warnings

        warnings.warn(f"libscaffold_hip's launch geometry is written for {tuned} compute units; device {index} has "
                      f"{units.value}: results are unaffected, launch shapes are not the best ones for it", RuntimeWarning, stacklevel=3)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """The HIP stream handle torch is issuing work to on ``device`` (one C call where torch offers the raw query;
    a ``torch.cuda.Stream`` object per launch costs several microseconds, which a step of a few hundred launches feels)."""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    if index not in _devices_seen:
        _note_device(device)
    if _raw_stream is not None:
        return int(_raw_stream(index))
    return int(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


class _NoGuard:
    __slots__ = ()

    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device: torch.device):
    """``torch.cuda.device(device)`` only when ``device`` is not already current (the common case costs one query)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


def _meta(v):
    """Everything a gate may look at, as a hashable value: tensors by their metadata, sequences as tuples. The common
    argument kinds are told apart by exact type first: a gate runs in front of every launch."""
    t = type(v)
    if t is int or v is None:
        return v
    if t is tuple or t is list:
        return tuple([e if type(e) is int else _meta(e) for e in v])
    if isinstance(v, torch.Tensor):
        return (torch.Tensor, v.shape, v.dtype, v.device, v.stride(), v.layout)
    return (t, v)


def memoized_gate(fn):
    """Caches a gate's verdict by the metadata of its arguments and the autocast state (gates are pure functions of
    those). Unhashable or exotic arguments simply take the uncached path."""
    cache = {}

    def wrapper(*args, **kwargs):
        try:
            key = (tuple([_meta(a) for a in args]), tuple([(k, _meta(v)) for k, v in kwargs.items()]) if kwargs else (),
                   torch.is_autocast_enabled("cuda"))
            hit = cache.get(key)
        except Exception:
            return fn(*args, **kwargs)
        if hit is None:
            hit = fn(*args, **kwargs)
            if len(cache) > 4096:
                cache.clear()
            cache[key] = hit
        return hit

    wrapper.__name__ = fn.__name__
    wrapper.__doc__ = fn.__doc__
    wrapper.__wrapped__ = fn
    return wrapper


def workspace(nbytes: int, device: torch.device):
    """A scratch buffer from torch's caching allocator (None when nothing is needed)."""
    if nbytes <= 0:
        return None
    return torch.empty(int(nbytes), dtype=torch.uint8, device=device)
