"""The shard format's layout arithmetic, the directory index and the ingest oracle (no GPU).

Pins: ``chunk_slice`` against ``torch.chunk`` itself (the routine ``ScaFFold/utils/spatial_sharding.py:96-106`` says it
matches), the id <-> index maps against numpy's row-major unravel and each other, ``spatial_slices`` by counting that the
shards of a grid cover every voxel exactly once, the oracle's relayout against index-by-index loops and a round trip
through real ``.npy`` files."""

import ctypes
import itertools
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from scaffold_amd import _lib, shards


def test_chunk_slice_is_torch_chunk():
    for size in range(1, 41):
        line = torch.arange(size)
        for count in range(1, 10):
            pieces = torch.chunk(line, count)
            for index in range(count):
                if index < len(pieces):
                    s = shards.chunk_slice(size, count, index)
                    assert (s.start, s.stop) == (int(pieces[index][0]), int(pieces[index][-1]) + 1)
                else:   # torch.chunk returned fewer pieces: that cell of the grid would be empty
                    with pytest.raises(ValueError, match="Empty local shard"):
                        shards.chunk_slice(size, count, index)


@pytest.mark.parametrize("grid", [(1,), (4,), (2, 3), (3, 1, 2), (2, 2, 2)])
def test_shard_ids_count_the_grid_row_major(grid):
    total = shards.total_shards(grid)
    assert total == int(np.prod(grid))
    for shard_id in range(total):
        idx = shards.shard_id_to_indices(shard_id, grid)
        assert idx == tuple(int(v) for v in np.unravel_index(shard_id, grid))
        assert shards.shard_indices_to_id(idx, grid) == shard_id
    for bad in (-1, total):
        with pytest.raises(ValueError):
            shards.shard_id_to_indices(bad, grid)
    with pytest.raises(ValueError):
        shards.shard_indices_to_id(tuple(grid), grid)          # every index one past its range
    with pytest.raises(ValueError):
        shards.shard_indices_to_id((0,) * (len(grid) + 1), grid)


@pytest.mark.parametrize("shape, dims, grid", [((8, 8, 8), (2,), (2,)), ((7, 5, 9), (2, 4), (3, 2)), ((6, 10, 4), (4, 3, 2), (2, 3, 3)),
                                               ((5, 5, 5), (), ())])
def test_shards_of_a_grid_cover_every_voxel_once(shape, dims, grid):
    seen = np.zeros(shape, dtype=np.int32)
    for shard_id in range(shards.total_shards(grid)):
        sl = shards.spatial_slices(shape, dims, grid, shards.shard_id_to_indices(shard_id, grid))
        seen[sl] += 1
    assert (seen == 1).all()
    with pytest.raises(ValueError):
        shards.spatial_slices(shape[:2], dims, grid, (0,) * len(grid))


def test_grid_validation_and_file_suffix():
    assert shards.normalize_sharding([2, 2], (2, 3)) == ((2, 2), (2, 3))
    for counts, dims in [((2,), (2, 3)), ((2, 2), (2, 2)), ((0,), (2,)), ((2,), (1,)), ((2,), (5,))]:
        with pytest.raises(ValueError):
            shards.normalize_sharding(counts, dims)
    assert shards.shard_file_suffix(0) == "_shard000000"
    assert shards.shard_file_suffix(7) == "_shard000007"
    assert shards.shard_file_suffix(1234567) == "_shard1234567"


def _write_dataset(root, ids, shard_ids, shape=(3, 4, 5, 6), seed=0):
    rng = np.random.default_rng(seed)
    images, masks = os.path.join(root, "volumes"), os.path.join(root, "masks")
    os.makedirs(images), os.makedirs(masks)
    data = {}
    for sample, k in itertools.product(ids, shard_ids):
        v = rng.random(shape, dtype=np.float32)
        m = rng.integers(0, 12, size=shape[1:]).astype(np.uint16)
        np.save(os.path.join(images, f"{sample}{shards.shard_file_suffix(k)}.npy"), v)
        np.save(os.path.join(masks, f"{sample}{shards.shard_file_suffix(k)}_mask.npy"), m)
        data[sample, k] = (v, m)
    return images, masks, data


def test_reader_indexes_one_shard_of_every_sample(tmp_path):
    images, masks, data = _write_dataset(str(tmp_path), ["7", "12", "a_b"], [0, 1, 2, 3])
    open(os.path.join(images, ".hidden_shard000002.npy"), "w").close()
    open(os.path.join(images, "notes.txt"), "w").close()
    r = shards.ShardReader(images, masks, shard_indices=(1, 0), num_shards=(2, 2))
    assert r.shard_id == 2 and r.suffix == "_shard000002" and len(r) == 3
    assert r.ids == ["12", "7", "a_b"]                      # sorted as strings, as the reference sorts its ids
    for sample in r.ids:
        v, m = r.read(sample)
        assert v.dtype == np.float32 and m.dtype == np.uint16
        np.testing.assert_array_equal(v, data[sample, 2][0])
        np.testing.assert_array_equal(m, data[sample, 2][1])
    with pytest.raises(KeyError, match="No image file"):
        r.read("nope")
    os.remove(os.path.join(masks, "7_shard000002_mask.npy"))
    r = shards.ShardReader(images, masks, shard_id=2)
    with pytest.raises(KeyError, match="No mask file"):
        r.read("7")
    with pytest.raises(ValueError):
        shards.ShardReader(images, masks)                    # neither id nor grid position
    with pytest.raises(ValueError):
        shards.ShardReader(images, masks, shard_id=4, num_shards=(2, 2))
    with pytest.raises(RuntimeError, match="No input file"):
        shards.ShardReader(images, masks, shard_id=9)


def test_reader_speaks_the_reference_datasets_protocol(tmp_path):
    """Indexable like the reference's dataset (a DataLoader and the class-weight estimate of ScaFFold/utils/losses.py:42-114
    can be pointed at it): float32 image + int16 mask carrier per item, masks alone on request."""
    images, masks, data = _write_dataset(str(tmp_path), ["0", "1", "2"], [0, 1])
    r = shards.ShardReader(images, masks, shard_id=1)
    counts = torch.zeros(12, dtype=torch.long)
    for idx in range(len(r)):
        item = r[idx]
        v, m = data[r.ids[idx], 1]
        assert item["image"].dtype is torch.float32 and item["mask"].dtype is torch.int16
        assert item["image"].is_contiguous() and item["mask"].is_contiguous()
        np.testing.assert_array_equal(item["image"].numpy(), v)
        np.testing.assert_array_equal(item["mask"].numpy(), m.astype(np.int16))
        only = r.load_mask_only(idx)
        assert torch.equal(only, item["mask"])
        counts += torch.bincount(only.reshape(-1).long(), minlength=12)      # losses.py:83-85
    want = sum(np.bincount(data[s, 1][1].reshape(-1), minlength=12) for s in r.ids)
    np.testing.assert_array_equal(counts.numpy(), want)
    batch = next(iter(torch.utils.data.DataLoader(r, batch_size=2)))
    assert batch["image"].shape == (2, 3, 4, 5, 6) and batch["mask"].shape == (2, 4, 5, 6) and batch["mask"].dtype is torch.int16


def test_reader_refuses_files_of_another_type(tmp_path):
    images, masks, _ = _write_dataset(str(tmp_path), ["s"], [0])
    np.save(os.path.join(images, "d_shard000000.npy"), np.zeros((3, 4, 5, 6), dtype=np.float64))
    np.save(os.path.join(masks, "d_shard000000_mask.npy"), np.zeros((4, 5, 6), dtype=np.uint16))
    np.save(os.path.join(images, "m_shard000000.npy"), np.zeros((3, 4, 5, 6), dtype=np.float32))
    np.save(os.path.join(masks, "m_shard000000_mask.npy"), np.zeros((4, 5, 6), dtype=np.int64))
    np.save(os.path.join(images, "e_shard000000.npy"), np.zeros((3, 4, 5, 6), dtype=np.float32))
    np.save(os.path.join(masks, "e_shard000000_mask.npy"), np.zeros((4, 5, 7), dtype=np.uint16))
    np.save(os.path.join(images, "o_shard000000.npy"), np.array([{"a": 1}], dtype=object), allow_pickle=True)
    np.save(os.path.join(masks, "o_shard000000_mask.npy"), np.zeros((4, 5, 6), dtype=np.uint16))
    r = shards.ShardReader(images, masks, shard_id=0)
    for sample in ("d", "m", "e"):
        with pytest.raises(ValueError):
            r.read(sample)
    with pytest.raises(ValueError):                           # a pickled array is never loaded
        r.read("o")
    r.read("s")


def test_ingest_oracle_against_index_loops_and_the_file_round_trip(tmp_path):
    images, masks, data = _write_dataset(str(tmp_path), ["s"], [0], shape=(3, 2, 3, 4), seed=3)
    r = shards.ShardReader(images, masks, shard_id=0)
    v, m = r.read("s")
    volume = torch.from_numpy(np.array(v))[None]
    mask = torch.from_numpy(np.array(m).astype(np.int16))[None]
    for dtype in (torch.float32, torch.bfloat16):
        x, labels = orc.shard_ingest(volume, mask, dtype=dtype, halo=1)
        assert x.shape == (1, 3, 4, 3, 4) and x.is_contiguous(memory_format=torch.channels_last_3d)
        flat = x.permute(0, 2, 3, 4, 1).contiguous().view(-1)     # memory order of a channels-last tensor
        at = 0
        for d in range(4):
            for h in range(3):
                for w in range(4):
                    for c in range(3):
                        want = 0.0 if d in (0, 3) else float(torch.tensor(data["s", 0][0][c, d - 1, h, w]).to(dtype))
                        assert float(flat[at]) == want
                        at += 1
        assert labels.dtype is torch.long and labels.shape == (1, 2, 3, 4)
        np.testing.assert_array_equal(labels[0].numpy(), data["s", 0][1].astype(np.int64))
    # the unsigned file type and the loader's signed carrier differ above 32767
    big = torch.from_numpy(np.array([[[[40000, 7]]]], dtype=np.uint16))
    one = torch.zeros((1, 1, 1, 1, 2))
    assert orc.shard_ingest(one, big)[1].tolist() == [[[[40000, 7]]]]
    assert orc.shard_ingest(one, big.view(torch.int16))[1].tolist() == [[[[40000 - 65536, 7]]]]


def test_argument_checks_of_the_ingest_entry_point():
    """Rejected before anything is launched, so this runs without a GPU."""
    from scaffold_amd._lib import IngestDesc

    L = _lib.lib()
    bf16 = 0
    one = ctypes.c_void_p(16)   # never dereferenced
    good = IngestDesc(1, 3, 0, 64, 0)
    assert L.sfh_shard_ingest(None, bf16, one, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_shard_ingest(ctypes.byref(good), 9, one, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_shard_ingest(ctypes.byref(IngestDesc(1, 0, 0, 64, 0)), bf16, one, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_shard_ingest(ctypes.byref(IngestDesc(1, 3, 0, 0, 0)), bf16, one, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_shard_ingest(ctypes.byref(IngestDesc(1, 3, 0, 64, -1)), bf16, one, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_shard_ingest(ctypes.byref(IngestDesc(1, 5, 0, 64, 0)), bf16, one, one, one, one, None) == _lib.SFH_ERR_UNSUPPORTED
    assert b"channels" in L.sfh_last_error()
    assert L.sfh_shard_ingest(ctypes.byref(good), bf16, one, one, one, None, None) == _lib.SFH_ERR_INVALID   # mask without labels
    assert L.sfh_shard_ingest(ctypes.byref(good), bf16, None, None, one, None, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_shard_ingest(ctypes.byref(good), bf16, ctypes.c_void_p(18), None, one, None, None) == _lib.SFH_ERR_INVALID
    assert b"aligned" in L.sfh_last_error()
    assert L.sfh_shard_ingest(ctypes.byref(IngestDesc(0, 3, 0, 64, 0)), bf16, None, None, None, None, None) == _lib.SFH_OK
