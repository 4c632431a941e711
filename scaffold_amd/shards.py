"""Dataset shards: the on-disk format of a spatially sharded volume and its way onto the device.

The generator writes every logical volume as one pair of ``.npy`` files per physical shard
(``ScaFFold/datagen/volumegen.py:259-292``): ``{id}_shard{k:06d}.npy`` holds the float32 volume ``(3, d, h, w)`` of
shard ``k`` and ``{id}_shard{k:06d}_mask.npy`` its uint16 class ids ``(d, h, w)``
(``ScaFFold/utils/spatial_sharding.py:130-133``, ``ScaFFold/utils/data_loading.py:308-317``).  Shard ids count the
shard grid row-major, and a sharded axis is cut the way ``torch.chunk`` cuts it
(``ScaFFold/utils/spatial_sharding.py:48-127``).  The layout functions below keep the reference's names and argument
meaning so that a caller of ``ScaFFold.utils.spatial_sharding`` finds them here.

``ingest`` is the device half: what ``images.to(float32, memory_format=channels_last_3d)``, ``masks.to(torch.long)``
(``ScaFFold/utils/trainer.py:572-589``) and autocast's cast in front of the first convolution do in three passes, done
in one kernel, optionally straight into the depth slab the first convolution of a shard reads.  ``ShardReader`` is the
host half for one rank: it indexes a directory pair, memory-maps a shard's two files (never unpickling anything), stages
them in pinned memory and hands them to ``ingest``.
"""

from __future__ import annotations

import ctypes
import os
import re
from typing import Dict, Iterable, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from ._lib import IngestDesc

__all__ = [
    "normalize_sharding", "total_shards", "shard_id_to_indices", "shard_indices_to_id", "chunk_slice", "spatial_slices",
    "shard_file_suffix", "is_supported_ingest", "ingest", "ShardReader", "VOLUME_DTYPE", "MASK_DTYPE",
]

VOLUME_DTYPE = np.float32   # ScaFFold/utils/data_types.py:20-25
MASK_DTYPE = np.uint16
MAX_INGEST_CHANNELS = 4

_CL3D = torch.channels_last_3d
_SPATIAL_DIMS = (2, 3, 4)   # tensor dimensions of (N, C, D, H, W) that may be sharded


# ---------------------------------------------------------------------------------------------
# layout arithmetic (pure functions of the shard grid)
# ---------------------------------------------------------------------------------------------
def _ints(values: Iterable[int]) -> Tuple[int, ...]:
    return tuple(int(v) for v in values)


def normalize_sharding(num_shards: Iterable[int], shard_dims: Iterable[int]):
    """``(num_shards, shard_dims)`` as int tuples; ``ValueError`` for a malformed grid
    (``spatial_sharding.py:19-41``): lengths differ, a dimension twice, a count below 1, a non-spatial dimension."""
    counts, dims = _ints(num_shards), _ints(shard_dims)
    if len(counts) != len(dims):
        raise ValueError(f"num_shards {counts} must have same length as shard_dims {dims}")
    if len(dims) != len(set(dims)):
        raise ValueError(f"Shard dimensions must be unique: {dims}")
    for count, dim in zip(counts, dims):
        if count < 1:
            raise ValueError(f"Invalid num_shards value {count}")
        if dim not in _SPATIAL_DIMS:
            raise ValueError(f"Invalid shard_dim {dim}: only 3D spatial dimensions 2, 3, and 4 are supported")
    return counts, dims


def total_shards(num_shards: Iterable[int]) -> int:
    """Number of cells of the shard grid."""
    n = 1
    for count in _ints(num_shards):
        n *= count
    return n


def shard_id_to_indices(shard_id: int, num_shards: Iterable[int]) -> Tuple[int, ...]:
    """Row-major shard id -> grid indices (``spatial_sharding.py:50-68``)."""
    counts = _ints(num_shards)
    shard_id = int(shard_id)
    if not 0 <= shard_id < total_shards(counts):
        raise ValueError(f"shard_id {shard_id} out of range for num_shards={counts}")
    digits = []
    for count in reversed(counts):      # the last grid axis is the fastest digit
        shard_id, digit = divmod(shard_id, count)
        digits.append(digit)
    return tuple(reversed(digits))


def shard_indices_to_id(shard_indices: Iterable[int], num_shards: Iterable[int]) -> int:
    """Grid indices -> row-major shard id (``spatial_sharding.py:71-93``)."""
    idx, counts = _ints(shard_indices), _ints(num_shards)
    if len(idx) != len(counts):
        raise ValueError(f"shard_indices {idx} must match num_shards {counts}")
    shard_id = 0
    for i, count in zip(idx, counts):   # Horner form of the row-major number
        if not 0 <= i < count:
            raise ValueError(f"Invalid shard index {i} for num_shards={counts}")
        shard_id = shard_id * count + i
    return shard_id


def chunk_slice(size: int, num_shards: int, shard_index: int) -> slice:
    """The piece ``torch.chunk(size, num_shards)[shard_index]`` covers: every piece ``ceil(size / num_shards)`` long, the
    last one shorter, trailing pieces possibly empty — those raise (``spatial_sharding.py:96-106``)."""
    size, num_shards, shard_index = int(size), int(num_shards), int(shard_index)
    piece = -(-size // num_shards)
    begin = piece * shard_index
    if begin >= size:
        raise ValueError(f"Empty local shard: dim size {size}, num_shards {num_shards}, shard_index {shard_index}")
    return slice(begin, min(begin + piece, size))


def spatial_slices(spatial_shape: Iterable[int], shard_dims: Iterable[int], num_shards: Iterable[int],
                   shard_indices: Iterable[int]) -> Tuple[slice, slice, slice]:
    """Local ``(D, H, W)`` slices of the shard at ``shard_indices``; ``shard_dims`` name tensor dimensions 2/3/4
    (``spatial_sharding.py:109-127``)."""
    shape = _ints(spatial_shape)
    if len(shape) != 3:
        raise ValueError(f"Expected 3D spatial shape, got {shape}")
    local = [slice(0, extent) for extent in shape]
    for dim, count, index in zip(_ints(shard_dims), _ints(num_shards), _ints(shard_indices)):
        axis = dim - 2
        local[axis] = chunk_slice(shape[axis], count, index)
    return tuple(local)


def shard_file_suffix(shard_id: int) -> str:
    """``_shard000007`` for shard 7 (``spatial_sharding.py:130-133``)."""
    return "_shard%06d" % int(shard_id)


# ---------------------------------------------------------------------------------------------
# device: planar float32 + 16-bit mask -> channels-last compute tensor (+ slab) and int64 labels
# ---------------------------------------------------------------------------------------------
def is_supported_ingest(volume, mask=None, dtype: torch.dtype = torch.float32) -> bool:
    """Total gate: never raises."""
    try:
        if not isinstance(volume, torch.Tensor) or volume.dim() != 5 or not volume.is_cuda or volume.dtype is not torch.float32:
            return False
        if dtype not in _lib.SUPPORTED_DTYPES or volume.numel() == 0 or not 1 <= volume.shape[1] <= MAX_INGEST_CHANNELS:
            return False
        if mask is not None:
            if not isinstance(mask, torch.Tensor) or mask.device != volume.device or mask.dtype not in (torch.int16, torch.uint16):
                return False
            if tuple(mask.shape) != (volume.shape[0],) + tuple(volume.shape[2:]):
                return False
        return True
    except Exception:
        return False


def ingest(volume: torch.Tensor, mask: Optional[torch.Tensor] = None, *, dtype: torch.dtype = torch.float32, out_halo: int = 0):
    """``(x, labels)`` for a batch ``volume (N, C, D, H, W)`` float32 (any strides; relaid out if not dense planar) and
    ``mask (N, D, H, W)`` int16 / uint16, both on the device.

    ``x`` equals ``volume.to(dtype, memory_format=torch.channels_last_3d)`` bit for bit and ``labels`` equals
    ``mask.to(torch.long)`` (``None`` without a mask).  With ``out_halo=h`` (one sample) ``x`` is the interior view of a
    slab with ``h`` zero depth planes on each face, carried as ``x._sfh_slab = (slab, h)`` for a
    ``FastConv3d.shard_halo`` stem.  Nothing here is differentiable: these are the step's inputs.
    """
    if not is_supported_ingest(volume, mask, dtype):
        raise NotImplementedError(
            f"unsupported: volume={tuple(getattr(volume, 'shape', ()))}/{getattr(volume, 'dtype', None)} "
            f"mask={tuple(getattr(mask, 'shape', ()))}/{getattr(mask, 'dtype', None)} dtype={dtype}")
    out_halo = int(out_halo)
    if out_halo < 0:
        raise ValueError(f"out_halo must be >= 0, got {out_halo}")
    volume = volume.detach().contiguous()
    n, c, d, h, w = (int(v) for v in volume.shape)
    halo = out_halo if n == 1 else 0
    labels = None
    if mask is not None:
        mask = mask.detach().contiguous()
        labels = torch.empty((n, d, h, w), dtype=torch.long, device=volume.device)
    slab = torch.empty((n, c, d + 2 * halo, h, w), dtype=dtype, device=volume.device, memory_format=_CL3D)
    desc = IngestDesc(n, c, int(mask is not None and mask.dtype is torch.int16), d * h * w, halo * h * w)
    with _lib.device_guard(volume.device):
        rc = _lib.lib().sfh_shard_ingest(ctypes.byref(desc), _lib.dtype_code(dtype), _lib.ptr(volume),
                                         _lib.ptr(mask) if mask is not None else None, _lib.ptr(slab),
                                         _lib.ptr(labels) if labels is not None else None, _lib.stream_ptr(volume.device))
    _lib.check(rc, "shard ingest")
    if halo == 0:
        return slab, labels
    x = slab.narrow(2, halo, d)
    x._sfh_slab = (slab, halo)
    return x, labels


# ---------------------------------------------------------------------------------------------
# host: one rank's view of a sharded dataset directory
# ---------------------------------------------------------------------------------------------
class ShardReader:
    """Index of the shard files one rank reads, and their way to the device.

    ``images_dir`` / ``mask_dir`` hold ``{id}{suffix}.npy`` / ``{id}{suffix}{mask_suffix}.npy`` with
    ``suffix = shard_file_suffix(shard_id)``; other files are ignored, hidden files too, and two files that reduce to
    the same id are an error, as in ``ScaFFold/utils/data_loading.py:296-340``.  ``shard_id`` is either given or derived
    from the rank's position in the shard grid (``shard_indices`` + ``num_shards``, ``data_loading.py:421-437``).
    """

    def __init__(self, images_dir, mask_dir, *, shard_id: Optional[int] = None, shard_indices: Optional[Sequence[int]] = None,
                 num_shards: Optional[Sequence[int]] = None, mask_suffix: str = "_mask"):
        if shard_id is None:
            if shard_indices is None or num_shards is None:
                raise ValueError("give shard_id, or shard_indices together with num_shards")
            shard_id = shard_indices_to_id(shard_indices, num_shards)
        elif num_shards is not None and not 0 <= int(shard_id) < total_shards(num_shards):
            raise ValueError(f"shard_id {shard_id} out of range for num_shards={_ints(num_shards)}")
        self.shard_id = int(shard_id)
        self.suffix = shard_file_suffix(self.shard_id)
        self.mask_suffix = str(mask_suffix)
        self.images_dir, self.mask_dir = os.fspath(images_dir), os.fspath(mask_dir)
        tail = re.escape(self.suffix)
        self._images = self._index(self.images_dir, re.compile(rf"^(?P<id>.+){tail}\.npy$"), "image")
        self._masks = self._index(self.mask_dir, re.compile(rf"^(?P<id>.+){tail}{re.escape(self.mask_suffix)}\.npy$"), "mask")
        if not self._images:
            raise RuntimeError(f"No input file found in {self.images_dir}, make sure you put your images there")
        self.ids = sorted(self._images)
        self._staging: Dict[Tuple, torch.Tensor] = {}

    @staticmethod
    def _index(directory: str, pattern, label: str) -> Dict[str, str]:
        found: Dict[str, str] = {}
        for entry in sorted(os.scandir(directory), key=lambda e: e.name):
            if not entry.is_file() or entry.name.startswith("."):
                continue
            m = pattern.match(entry.name)
            if m is None:
                continue
            sample = m.group("id")
            if sample in found:
                raise RuntimeError(f"Ambiguous {label} id '{sample}' in {directory}: matches both "
                                   f"{os.path.basename(found[sample])} and {entry.name}. Every id must map to exactly one file.")
            found[sample] = entry.path
        return found

    def __len__(self) -> int:
        return len(self.ids)

    def paths(self, sample_id: str) -> Tuple[str, str]:
        """``(volume file, mask file)`` of a sample; ``KeyError`` names the missing one."""
        if sample_id not in self._images:
            raise KeyError(f"No image file found for the ID {sample_id} in {self.images_dir}")
        if sample_id not in self._masks:
            raise KeyError(f"No mask file found for the ID {sample_id} in {self.mask_dir}")
        return self._images[sample_id], self._masks[sample_id]

    def read(self, sample_id: str):
        """The two arrays of a sample, memory-mapped: ``volume (C, d, h, w)`` float32, ``mask (d, h, w)`` uint16.
        Files of another dtype or rank are refused rather than converted silently."""
        volume_path, mask_path = self.paths(sample_id)
        volume = np.load(volume_path, mmap_mode="r", allow_pickle=False)
        mask = np.load(mask_path, mmap_mode="r", allow_pickle=False)
        if volume.dtype != VOLUME_DTYPE or volume.ndim != 4:
            raise ValueError(f"{volume_path}: expected a float32 (C, D, H, W) volume, found {volume.dtype} {volume.shape}")
        if mask.dtype != MASK_DTYPE or mask.ndim != 3:
            raise ValueError(f"{mask_path}: expected a uint16 (D, H, W) mask, found {mask.dtype} {mask.shape}")
        if tuple(mask.shape) != tuple(volume.shape[1:]):
            raise ValueError(f"{mask_path}: mask extent {mask.shape} does not match the volume's {volume.shape[1:]}")
        return volume, mask

    # -- the reference dataset's host-side protocol (``BasicDataset``, data_loading.py:535-576) --------------------
    @staticmethod
    def _mask_carrier(mask) -> torch.Tensor:
        # class ids travel as int16 and are widened on the device (data_loading.py:540-545)
        return torch.from_numpy(np.array(mask, dtype=MASK_DTYPE, order="C").astype(np.int16, copy=False)).contiguous()

    def load_mask_only(self, idx: int) -> torch.Tensor:
        """The int16 mask of sample ``idx`` without touching its volume (what the class-weight estimate reads,
        ``ScaFFold/utils/losses.py:76-85``)."""
        _, mask_path = self.paths(self.ids[idx])
        mask = np.load(mask_path, mmap_mode="r", allow_pickle=False)
        if mask.dtype != MASK_DTYPE or mask.ndim != 3:
            raise ValueError(f"{mask_path}: expected a uint16 (D, H, W) mask, found {mask.dtype} {mask.shape}")
        return self._mask_carrier(mask)

    def __getitem__(self, idx: int):
        """``{"image": float32 (C, d, h, w), "mask": int16 (d, h, w)}`` on the host, as the reference's dataset returns
        it to a ``DataLoader`` (``data_loading.py:560-576``)."""
        volume, mask = self.read(self.ids[idx])
        return {"image": torch.from_numpy(np.array(volume, dtype=VOLUME_DTYPE, order="C")).contiguous().float(),
                "mask": self._mask_carrier(mask)}

    def _pinned(self, key, shape, dtype) -> torch.Tensor:
        buf = self._staging.get(key)
        if buf is None or tuple(buf.shape) != tuple(shape):
            buf = torch.empty(shape, dtype=dtype, pin_memory=True)   # allocated pinned; never a registration of pageable memory
            self._staging[key] = buf
        return buf

    def load(self, sample_ids, device, *, dtype: torch.dtype = torch.float32, out_halo: int = 0):
        """``(x, labels)`` on ``device`` for one id or a list of ids (a batch; all shards of one rank have one extent).

        File bytes go through a pinned staging buffer (kept and reused) and one asynchronous copy each for volumes and
        masks, then through ``ingest``.  The host waits for the copies before returning, so the staging buffers may be
        refilled by the next call.
        """
        if isinstance(sample_ids, str):
            sample_ids = [sample_ids]
        arrays = [self.read(s) for s in sample_ids]
        if not arrays:
            raise ValueError("no sample ids given")
        vshape = arrays[0][0].shape
        for (volume, _), s in zip(arrays, sample_ids):
            if volume.shape != vshape:
                raise ValueError(f"sample {s}: extent {volume.shape} differs from the batch's {vshape}")
        n = len(arrays)
        device = torch.device(device)
        hv = self._pinned(("v", device), (n,) + tuple(vshape), torch.float32)
        hm = self._pinned(("m", device), (n,) + tuple(vshape[1:]), torch.int16)
        hv_np, hm_np = hv.numpy(), hm.numpy().view(np.uint16)
        for i, (volume, mask) in enumerate(arrays):
            np.copyto(hv_np[i], volume)
            np.copyto(hm_np[i], mask)
        dv = hv.to(device, non_blocking=True)
        dm = hm.to(device, non_blocking=True).view(torch.uint16)
        x, labels = ingest(dv, dm, dtype=dtype, out_halo=out_halo)
        torch.cuda.current_stream(device).synchronize()
        return x, labels
