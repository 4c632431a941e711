"""scaffold_amd -- MI355X (gfx950) kernels for the ScaFFold 3D U-Net compute hot path.

A thin host-side mirror of the reference's operator interface (``triton_conv3d/__init__.py:60-107``,
``ScaFFold/unet/triton_group_norm.py``, ``ScaFFold/unet/{conv3d,group_norm,unet_model,unet_parts}.py``)
over one C-ABI shared library of hand-written HIP kernels (``libscaffold_hip.so``, declared in
``include/scaffold_hip.h``).  Importing the package loads nothing; the library is loaded on first
use and its absence is an error, never a fallback.
"""

from __future__ import annotations

import importlib

__version__ = "0.1.0"

_EXPORTS = {
    # conv3d family (triton_conv3d public names)
    "conv3d_forward": "conv3d", "conv3d_backward_data": "conv3d", "conv3d_backward_weight": "conv3d",
    "is_supported": "conv3d", "is_supported_all": "conv3d", "is_supported_bwd_data": "conv3d",
    "is_supported_bwd_weight": "conv3d", "bwd_data_padding": "conv3d", "grad_weight_empty": "conv3d",
    "workspace_elements": "conv3d", "split_count": "conv3d", "bias_grad": "conv3d",
    "conv3d_backward_weight_batch": "conv3d", "weight_grad_batchable": "conv3d", "weight_grad_batch_family": "conv3d",
    "pack_weights": "conv3d", "packed_weight_bytes": "conv3d", "pack_weights_batch": "conv3d", "PackedWeights": "conv3d",
    "conv_transpose3d_forward": "transposed", "conv_transpose3d_backward_data": "transposed",
    "conv_transpose3d_backward_weight": "transposed", "is_supported_transposed": "transposed",
    "is_supported_transposed_all": "transposed", "is_supported_transposed_bwd_data": "transposed",
    "is_supported_transposed_bwd_weight": "transposed", "grad_transposed_weight_empty": "transposed",
    # GroupNorm
    "group_norm": "groupnorm", "triton_group_norm": "groupnorm", "MATCH_STOCK_DTYPE": "groupnorm",
    # loss head
    "ce_dice_loss": "losses", "is_supported_loss": "losses",
    # pooling
    "max_pool3d_2x": "pooling", "is_supported_pool": "pooling", "FastMaxPool3d": "pooling",
    # halo slab of a depth shard
    "halo_assemble": "halo", "is_supported_halo": "halo", "halo_pack": "halo", "halo_accumulate_": "halo",
    "halo_exchange": "halo",
    # skip connection concat
    "skip_concat": "concat", "is_supported_concat": "concat",
    # dataset shards: file layout, reader, device ingest
    "ingest": "shards", "is_supported_ingest": "shards", "ShardReader": "shards",
    # optimizer step
    "FusedClipAdam": "optim",
    # modules / model
    "FastConv3d": "modules", "FastConvTranspose3d": "modules", "FastGroupNorm": "modules",
    "UNet": "unet",
    # errors
    "ScaffoldKernelError": "_lib", "ScaffoldLibraryError": "_lib",
}

__all__ = sorted(_EXPORTS)


def __getattr__(name):
    try:
        module = _EXPORTS[name]
    except KeyError:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}") from None
    value = getattr(importlib.import_module(f".{module}", __name__), name)
    globals()[name] = value
    return value
