"""The ScaFFold 3D U-Net over the HIP ops, with the widths of the benchmark configurations as arguments.

Structure, child names and therefore ``state_dict`` keys follow the reference model
(``ScaFFold/unet/unet_model.py:27-162``, ``ScaFFold/unet/unet_parts.py:107-240``):
``down_list[0]`` is a DoubleConv, ``down_list[i]`` is MaxPool3d(2) + DoubleConv, ``up_list[i]`` is
ConvTranspose3d(k=2, s=2) -> pad -> skip concat -> DoubleConv, ``up_list[-1]`` is the 1x1x1 head.
DoubleConv is ``(conv3 -> GroupNorm(+ReLU) -> Identity) x 2``: the ReLU is fused into the GroupNorm
and ``nn.Identity`` keeps the positional names of a conv/norm/relu Sequential.

The reference hard-codes a base width of 64 (``unet_model.py:68``); here ``base_width`` is an
argument (32 for the benchmark configuration).  ``stock=True`` builds the identical architecture
from ``nn.Conv3d`` / ``nn.ConvTranspose3d`` / ``nn.GroupNorm`` + ``F.relu``: the comparison arm of the
parity tests, with interchangeable state dicts.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F
import torch.utils.checkpoint

from . import concat as _cat
from .modules import FastConv3d, FastConvTranspose3d, FastGroupNorm, autocast_dtype
from .pooling import FastMaxPool3d

__all__ = ["UNet", "DoubleConv", "Down", "Up", "OutConv", "skip_concat"]


class _StockGroupNormRelu(nn.GroupNorm):
    """Stock arm: ``F.group_norm`` then ``F.relu``, returned in the input's dtype (the contract of
    ``FastGroupNorm``, ``ScaFFold/unet/group_norm.py:572-599``)."""

    activation = None

    def __init__(self, num_groups, num_channels, eps=1e-5, affine=True, device=None, dtype=None, activation=None):
        super().__init__(num_groups, num_channels, eps=eps, affine=affine, device=device, dtype=dtype)
        self.activation = activation

    def forward(self, x):
        y = F.group_norm(x, self.num_groups, self.weight, self.bias, self.eps)
        if self.activation == "relu":
            y = F.relu(y)
        return y if y.dtype is x.dtype else y.to(x.dtype)


def _conv3d(stock, cin, cout, **kw):
    return (nn.Conv3d if stock else FastConv3d)(cin, cout, **kw)


def _conv_transpose3d(stock, cin, cout, **kw):
    return (nn.ConvTranspose3d if stock else FastConvTranspose3d)(cin, cout, **kw)


def _max_pool(stock):
    return (nn.MaxPool3d if stock else FastMaxPool3d)(2)


def _group_norm(stock, groups, channels, activation=None):
    if channels % groups != 0:
        raise ValueError(f"group_norm_groups={groups} must evenly divide num_channels={channels}")
    return (_StockGroupNormRelu if stock else FastGroupNorm)(groups, channels, activation=activation)


def _consumer_dtype(*tensors):
    """The dtype the convolution after a concat will read: autocast's when it narrows, else the widest."""
    dtype = tensors[0].dtype
    for t in tensors[1:]:
        dtype = torch.promote_types(dtype, t.dtype)
    ac = autocast_dtype(tensors[0])
    if ac is None or dtype is not torch.float32:
        return dtype
    return ac


def skip_concat(skip, upsampled, out_halo=0):
    """``torch.cat([skip, upsampled], 1)`` at the consumer's dtype (``unet_parts.py:107-120``): the one-pass kernel
    where it serves the tensors (``out_halo``: into the slab of a following depth-shard convolution), else ``torch.cat``."""
    dtype = _consumer_dtype(skip, upsampled)
    skip, upsampled = skip.to(dtype), upsampled.to(dtype)
    if _cat.is_supported_concat(skip, upsampled):
        return _cat.skip_concat(skip, upsampled, out_halo)
    return torch.cat([skip, upsampled], dim=1)


class DoubleConv(nn.Module):
    def __init__(self, in_channels, out_channels, group_norm_groups, mid_channels=None, stock=False):
        super().__init__()
        mid = mid_channels or out_channels
        self.double_conv = nn.Sequential(
            _conv3d(stock, in_channels, mid, kernel_size=3, padding=1, bias=False),
            _group_norm(stock, group_norm_groups, mid, activation="relu"),
            nn.Identity(),
            _conv3d(stock, mid, out_channels, kernel_size=3, padding=1, bias=False),
            _group_norm(stock, group_norm_groups, out_channels, activation="relu"),
            nn.Identity(),
        )

        self._pairs = () if stock else ((0, 1), (3, 4))
        # each convolution announces the GroupNorm that reads its output: its launch leaves the statistics
        for c, g in self._pairs:
            self.double_conv[c].gn_groups = self.double_conv[g].num_groups

    def forward(self, x, second=None):
        """``second``: the input is ``torch.cat([x, second], 1)``, handed over as the two tensors (the first convolution
        must have said ``takes_pair``)."""
        if not self._pairs:
            return self.double_conv(x if second is None else torch.cat([x, second], dim=1))
        for c, g in self._pairs:  # the Identity modules between the pairs only keep the reference's state-dict indices
            conv, norm = self.double_conv[c], self.double_conv[g]
            x = norm(conv(x) if second is None else conv(x, second))
            second = None
        return x


class Down(nn.Module):
    def __init__(self, in_channels, out_channels, group_norm_groups, stock=False):
        super().__init__()
        self.maxpool_conv = nn.Sequential(_max_pool(stock), DoubleConv(in_channels, out_channels, group_norm_groups, stock=stock))

    def forward(self, x):
        return self.maxpool_conv(x)


class Up(nn.Module):
    #: let the first convolution read [skip, upsampled] as two tensors where it serves them (False: always concatenate)
    read_skip_in_place = True

    def __init__(self, in_channels, out_channels, group_norm_groups, stock=False):
        super().__init__()
        self.up = _conv_transpose3d(stock, in_channels, in_channels // 2, kernel_size=2, stride=2)
        self.conv = DoubleConv(in_channels, out_channels, group_norm_groups, stock=stock)

    def forward(self, x1, x2):
        x1 = self.up(x1)
        dz, dy, dx = (x2.size(i) - x1.size(i) for i in (2, 3, 4))
        if dx or dy or dz:
            x1 = F.pad(x1, [dx // 2, dx - dx // 2, dy // 2, dy - dy // 2, dz // 2, dz - dz // 2])
        first = self.conv.double_conv[0]
        if self.read_skip_in_place and isinstance(first, FastConv3d):
            # the convolution reads the skip connection and the upsampled tensor where they lie: nothing is concatenated
            dtype = _consumer_dtype(x2, x1)
            skip, up = (x2 if x2.dtype is dtype else x2.to(dtype)), (x1 if x1.dtype is dtype else x1.to(dtype))
            if first.takes_pair(skip, up):
                return self.conv(skip, up)
        halo = int(first.padding[0]) if getattr(first, "shard_halo", False) else 0
        return self.conv(skip_concat(x2, x1, halo))


class OutConv(nn.Module):
    def __init__(self, in_channels, out_channels, stock=False):
        super().__init__()
        self.conv = _conv3d(stock, in_channels, out_channels, kernel_size=1)

    def forward(self, x):
        return self.conv(x)


class UNet(nn.Module):
    """``layers`` down/up stages (4 at problem scale 7), widths ``base_width * 2**i``."""

    def __init__(self, n_channels, n_classes, layers=4, group_norm_groups=8, base_width=32, stock=False):
        super().__init__()
        if layers < 1:
            raise ValueError(f"UNet requires layers >= 1, got layers={layers}")
        self.n_channels, self.n_classes, self.layers = n_channels, n_classes, layers
        self.group_norm_groups, self.base_width, self.stock = group_norm_groups, base_width, stock
        self.checkpointing = False
        g = group_norm_groups
        width = base_width
        self.down_list = nn.ModuleList([DoubleConv(n_channels, width, g, stock=stock)])
        for _ in range(layers):
            self.down_list.append(Down(width, width * 2, g, stock=stock))
            width *= 2
        self.up_list = nn.ModuleList()
        for _ in range(layers):
            self.up_list.append(Up(width, width // 2, g, stock=stock))
            width //= 2
        self.up_list.append(OutConv(width, n_classes, stock=stock))

    def use_checkpointing(self):
        self.checkpointing = True

    def set_shard_halo(self, enabled: bool = True):
        """Run every 3x3x3 convolution in the depth-shard form (zero halo + depth padding 0)."""
        for m in self.modules():
            if isinstance(m, FastConv3d):
                m.shard_halo = bool(enabled)
            if isinstance(m, DoubleConv):
                # the first GroupNorm writes straight into the slab the second convolution reads
                norm, conv = m.double_conv[1], m.double_conv[3]
                if isinstance(norm, FastGroupNorm) and isinstance(conv, FastConv3d):
                    norm.out_halo = int(conv.padding[0]) if enabled else 0
        # the pooling writes into the slab the first convolution of its level reads
        for down in self.down_list[1:]:
            pool, block = down.maxpool_conv
            if isinstance(pool, FastMaxPool3d) and isinstance(block.double_conv[0], FastConv3d):
                pool.out_halo = int(block.double_conv[0].padding[0]) if enabled else 0
        # The decoder's first convolutions read the skip connection and the upsampled tensor as they lie: their
        # producers (the encoder blocks' last GroupNorm, the up-convolutions) write them into slabs as well.
        for i, up in enumerate(self.up_list[:-1]):
            first = up.conv.double_conv[0]
            if not isinstance(first, FastConv3d):
                continue
            halo = int(first.padding[0]) if enabled else 0
            if isinstance(up.up, FastConvTranspose3d):
                up.up.out_halo = halo
            enc = self.down_list[self.layers - 1 - i]
            block = enc if isinstance(enc, DoubleConv) else enc.maxpool_conv[1]
            if isinstance(block.double_conv[4], FastGroupNorm):
                block.double_conv[4].out_halo = halo
        return self

    def defer_weight_gradients(self, enabled: bool = True, early: bool = False):
        """Leave the weight gradients of the 3x3x3 convolutions to the end of the backward pass, where one launch computes
        all that the library batches (``modules.flush_weight_gradients``): ``.grad`` is complete when ``backward()``
        returns, as always; hooks on the parameters' gradient accumulation do not see these gradients.

        ``early``: the gradients of the decoder's upper levels do not wait for the end: when the backward pass reaches the
        deep levels (small volumes: kernels bound by latency, most of the device idle) they are computed on a stream of
        their own, on half of the compute units, beside the rest of the pass, and joined where the others are computed."""
        for m in self.modules():
            if isinstance(m, FastConv3d):
                m.defer_weight_grad = (2 if early else True) if enabled else False
        return self

    def _run(self, block, *inputs):
        if self.checkpointing:
            return torch.utils.checkpoint.checkpoint(block, *inputs, use_reentrant=False)
        return block(*inputs)

    def forward(self, x):
        feats = [self._run(self.down_list[0], x)]
        for i in range(1, self.layers + 1):
            pool, block = self.down_list[i].maxpool_conv
            if isinstance(pool, FastMaxPool3d) and not self.checkpointing and pool.serves(feats[-1]):
                # the tensor that is pooled is also the skip connection: both gradients meet in the pooling kernel
                pooled, feats[-1] = pool.with_skip(feats[-1])
                feats.append(block(pooled))
            else:
                feats.append(self._run(self.down_list[i], feats[-1]))
        feats.reverse()
        out = feats[0]
        for i in range(self.layers):
            out = self._run(self.up_list[i], out, feats[i + 1])
        return self._run(self.up_list[-1], out)
