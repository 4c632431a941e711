"""The C-ABI library without a GPU: it loads, exports every symbol include/scaffold_hip.h declares, and its
pure host entry points (shape, plan and workspace queries, argument checking) behave."""

import ctypes
import os
import re

import pytest
import torch

from scaffold_amd import _lib
from scaffold_amd._lib import ConvDesc, ConvTDesc, GroupNormDesc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "scaffold_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sfh_[a-zA-Z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = header_symbols()
    assert len(names) >= 18
    handle = ctypes.CDLL(_lib.lib_path())
    for name in names:
        assert hasattr(handle, name), f"{name} is declared in scaffold_hip.h but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names, "the ctypes binding and the header disagree"
    assert _lib.lib().sfh_version() >= 100


def conv_desc(n=1, cin=32, sp=(16, 16, 16), cout=32, k=(3, 3, 3), s=(1, 1, 1), p=(1, 1, 1), d=(1, 1, 1)):
    return ConvDesc(n, cin, *sp, cout, *k, *s, *p, *d)


def test_out_shape_and_argument_checks():
    L = _lib.lib()
    out = (ctypes.c_int32 * 3)()
    assert L.sfh_conv3d_out_shape(ctypes.byref(conv_desc(p=(0, 1, 1))), out) == 0 and list(out) == [14, 16, 16]
    assert L.sfh_conv3d_out_shape(ctypes.byref(conv_desc(sp=(7, 8, 9), k=(2, 3, 1), s=(2, 1, 3), p=(1, 0, 2), d=(1, 2, 1))), out) == 0
    assert list(out) == list(torch.nn.functional.conv3d(torch.empty((1, 32, 7, 8, 9), device="meta"),
                                                        torch.empty((32, 32, 2, 3, 1), device="meta"), None, (2, 1, 3),
                                                        (1, 0, 2), (1, 2, 1)).shape[2:])
    # kernel wider than the padded input, zero stride, null descriptor: contract violations with a message
    assert L.sfh_conv3d_out_shape(ctypes.byref(conv_desc(sp=(2, 2, 2), p=(0, 0, 0))), out) == _lib.SFH_ERR_INVALID
    assert b"wider" in L.sfh_last_error()
    assert L.sfh_conv3d_out_shape(ctypes.byref(conv_desc(s=(0, 1, 1))), out) == _lib.SFH_ERR_INVALID
    assert L.sfh_conv3d_out_shape(None, out) == _lib.SFH_ERR_INVALID
    with pytest.raises(ValueError):
        _lib.check(_lib.SFH_ERR_INVALID, "x")
    with pytest.raises(NotImplementedError):
        _lib.check(_lib.SFH_ERR_UNSUPPORTED, "x")
    with pytest.raises(_lib.ScaffoldKernelError):
        _lib.check(_lib.SFH_ERR_LAUNCH, "x")


def test_kernel_selection_is_a_pure_function_of_the_problem():
    L = _lib.lib()
    bf16, fp32 = 0, 2
    d = conv_desc(sp=(128, 128, 128))
    assert [L.sfh_conv3d_uses_mfma(ctypes.byref(d), bf16, i) for i in range(3)] == [1, 1, 1]
    assert [L.sfh_conv3d_uses_mfma(ctypes.byref(d), fp32, i) for i in range(3)] == [1, 1, 1]          # fp32: the fp32 matrix pipe
    assert L.sfh_conv3d_uses_mfma(ctypes.byref(conv_desc(cin=8)), fp32, 0) == 0                         # not a multiple of 16
    assert L.sfh_conv3d_uses_mfma(ctypes.byref(conv_desc(cin=3)), bf16, 0) == 0                         # odd channels
    assert L.sfh_conv3d_uses_mfma(ctypes.byref(conv_desc(s=(2, 2, 2))), bf16, 0) == 0                   # strided
    assert L.sfh_conv3d_uses_mfma(ctypes.byref(conv_desc(p=(0, 1, 1))), bf16, 1) == 1                   # shard form dgrad
    # workspace sizes: packed weight for fwd/dgrad, splits * Cout * 27 * Cin fp32 for wgrad
    assert L.sfh_conv3d_fwd_workspace_bytes(ctypes.byref(d), bf16) == 32 * 32 * 27 * 2
    assert L.sfh_conv3d_fwd_workspace_bytes(ctypes.byref(d), fp32) == 32 * 32 * 27 * 4              # fp32 packed weight
    splits = L.sfh_conv3d_wgrad_splits(ctypes.byref(d), bf16)
    assert splits >= 1 and splits == L.sfh_conv3d_wgrad_splits(ctypes.byref(d), bf16)
    assert L.sfh_conv3d_wgrad_workspace_bytes(ctypes.byref(d), bf16) == splits * 32 * 27 * 32 * 4
    splits32 = L.sfh_conv3d_wgrad_splits(ctypes.byref(d), fp32)
    assert splits32 >= 1 and L.sfh_conv3d_wgrad_workspace_bytes(ctypes.byref(d), fp32) == splits32 * 32 * 27 * 32 * 4
    assert L.sfh_conv3d_wgrad_splits(ctypes.byref(conv_desc(cin=8)), fp32) == 1                         # untiled: one pass, no slices


def test_launch_geometry_is_stated_and_agrees_with_the_workspace():
    """The geometry query names the kernel and its tile / block / slice counts; the workspace sizes follow from it."""
    L = _lib.lib()
    bf16, fp32 = 0, 2

    def geometry(desc, dtype, direction):
        out = (ctypes.c_int32 * 4)()
        assert L.sfh_conv3d_launch_geometry(ctypes.byref(desc), dtype, direction, out) == 0
        assert list(out) == list(geometry_again(desc, dtype, direction))
        return list(out)

    def geometry_again(desc, dtype, direction):
        out = (ctypes.c_int32 * 4)()
        L.sfh_conv3d_launch_geometry(ctypes.byref(desc), dtype, direction, out)
        return out

    DIRECT, PERSIST, BRICK, WIDE, WGRAD, OTHER, SPLIT = range(7)
    cube = conv_desc(sp=(128, 128, 128))
    assert geometry(cube, bf16, 0) == [PERSIST, 512, 1, 1] and geometry(cube, bf16, 1) == [PERSIST, 512, 1, 1]
    assert geometry(cube, bf16, 2) == [WGRAD, 256, 1, L.sfh_conv3d_wgrad_splits(ctypes.byref(cube), bf16)]
    assert geometry(cube, fp32, 0)[0] == OTHER and geometry(conv_desc(cin=3), bf16, 0)[0] == DIRECT
    assert geometry(conv_desc(cin=128, cout=64, sp=(64, 64, 64)), bf16, 0) == [WIDE, 1024, 2, 1]
    # the data gradient of a depth shard's slab (D + 2 planes): 256-voxel tiles, or a ninth of the workgroups would run a
    # round of their own
    assert geometry(conv_desc(cin=64, cout=64, sp=(34, 64, 64), p=(0, 1, 1)), bf16, 1) == [BRICK, 256, 1, 1]
    assert geometry(conv_desc(cin=64, cout=64, sp=(64, 64, 64)), bf16, 0) == [BRICK, 512, 2, 1]
    # a small-volume level: 64-voxel bricks, the reduction cut over the wavefronts of a workgroup -- no slices, no partials
    small = conv_desc(cin=256, cout=256, sp=(10, 16, 16), p=(0, 1, 1))
    assert geometry(small, bf16, 0) == [SPLIT, 64, 2, 1] and geometry(small, bf16, 1) == [SPLIT, 64, 2, 1]
    assert L.sfh_conv3d_fwd_workspace_bytes(ctypes.byref(small), bf16) == 256 * 256 * 27 * 2
    # the deepest level: too few bricks for that, the reduction channels are cut into slices and the workspace holds their
    # fp32 partials
    deep = conv_desc(cin=256, cout=512, sp=(6, 8, 8), p=(0, 1, 1))
    kernel, voxels, blocks, slices = geometry(deep, bf16, 0)
    assert (kernel, voxels, blocks) == (BRICK, 256, 1) and 1 < slices <= 8 and slices & (slices - 1) == 0
    packed = 256 * 512 * 27 * 2
    assert L.sfh_conv3d_fwd_workspace_bytes(ctypes.byref(deep), bf16) == packed + slices * 4 * 8 * 8 * 512 * 4
    out = (ctypes.c_int32 * 4)()
    assert L.sfh_conv3d_launch_geometry(ctypes.byref(cube), bf16, 3, out) == _lib.SFH_ERR_INVALID
    assert L.sfh_conv3d_launch_geometry(ctypes.byref(cube), bf16, 0, None) == _lib.SFH_ERR_INVALID


def test_which_problems_take_a_skip_connection_as_two_tensors():
    """``sfh_conv3d_pair_supported`` is a pure function of problem, dtype, cut and direction; the entry points refuse what it
    refuses before anything is launched."""
    L = _lib.lib()
    bf16, fp16, fp32 = 0, 1, 2

    def offered(desc, dtype, first):
        return [L.sfh_conv3d_pair_supported(ctypes.byref(desc), dtype, first, d) for d in (0, 1, 2)]

    level0 = conv_desc(cin=64, cout=32, sp=(66, 128, 128), p=(0, 1, 1))   # the decoder's first convolution on a depth shard
    assert offered(level0, bf16, 32) == [1, 1, 1] and offered(level0, fp16, 32) == [1, 1, 1]
    assert offered(level0, fp32, 32) == [0, 0, 0]                        # the fp32 tiles read one tensor
    assert offered(level0, bf16, 16) == [0, 0, 0] and offered(level0, bf16, 48) == [0, 0, 0]  # a cut off the 32-channel grid
    assert offered(level0, bf16, 0) == [0, 0, 0] and offered(level0, bf16, 64) == [0, 0, 0]   # nothing on one side
    assert L.sfh_conv3d_pair_supported(ctypes.byref(level0), bf16, 32, 3) == 0
    wide = conv_desc(cin=128, cout=64, sp=(34, 64, 64), p=(0, 1, 1))      # forward on the wide-tile kernel: equal halves only
    assert offered(wide, bf16, 64) == [1, 1, 1] and offered(wide, bf16, 32) == [0, 1, 1]
    assert offered(conv_desc(cin=96, cout=32, sp=(8, 16, 16)), bf16, 64) == [1, 1, 1]        # an unequal cut elsewhere is fine
    deep = conv_desc(cin=512, cout=256, sp=(8, 16, 16))                   # both directions sliced: the slice sum writes the pair
    assert offered(deep, bf16, 256) == [1, 1, 1]
    assert offered(conv_desc(cin=64, cout=32, k=(1, 1, 1), p=(0, 0, 0)), bf16, 32) == [0, 0, 0]      # not a 3x3x3 problem
    assert offered(conv_desc(cin=64, cout=32, s=(2, 2, 2)), bf16, 32)[1] == 0                        # strided: no data gradient at all
    assert offered(conv_desc(cin=64, cout=32, n=0), bf16, 32) == [0, 0, 0]
    # refused calls launch nothing: null tensors are never touched
    assert L.sfh_conv3d_fwd_pair(ctypes.byref(level0), bf16, None, None, 16, None, None, None, None, None, 0, 0, 0, None, 0,
                                 None) == _lib.SFH_ERR_INVALID
    one = ctypes.c_void_p(16)  # a non-null stand-in that must not be dereferenced
    assert L.sfh_conv3d_fwd_pair(ctypes.byref(level0), bf16, one, one, 16, one, None, None, one, None, 0, 0, 0, None, 0,
                                 None) == _lib.SFH_ERR_UNSUPPORTED
    assert L.sfh_conv3d_dgrad_pair(ctypes.byref(level0), bf16, one, one, None, one, one, 48, None, 0, 0, None) == _lib.SFH_ERR_UNSUPPORTED
    assert L.sfh_conv3d_wgrad_pair(ctypes.byref(level0), fp32, one, one, 32, one, one, None, 0, 0, None) == _lib.SFH_ERR_UNSUPPORTED
    assert L.sfh_conv3d_wgrad_pair(ctypes.byref(level0), bf16, one, one, 32, one, one, None, 0, _lib.SFH_FLAG_FORCE_GENERIC,
                                   None) == _lib.SFH_ERR_INVALID


def test_wgrad_split_plan_partitions_the_bricks():
    """Every brick belongs to exactly one split: splits * ceil(bricks / splits) covers, (splits-1) * that does not."""
    L = _lib.lib()
    for sp in [(128, 128, 128), (64, 64, 64), (9, 10, 16), (5, 7, 33), (8, 8, 8), (2, 2, 2)]:
        for cin, cout in [(32, 32), (64, 128), (512, 512)]:
            d = conv_desc(cin=cin, cout=cout, sp=sp)
            splits = L.sfh_conv3d_wgrad_splits(ctypes.byref(d), 0)
            tw, td, th = (32, 2, 4) if sp[2] > 16 else ((16, 2, 8) if sp[2] > 8 else (8, 4, 8))
            bricks = -(-sp[0] // td) * -(-sp[1] // th) * -(-sp[2] // tw)
            per = -(-bricks // splits)
            assert 1 <= splits <= bricks and splits * per >= bricks and (splits - 1) * per < bricks


def test_weight_gradient_batch_plan_and_refusals():
    """The batched weight gradient without a GPU: which problems join which launch, the workspace of a list (a pure
    function of its shapes, never 0 for a served list), and the refusals that come before any launch."""
    L = _lib.lib()
    bf16, fp32 = 0, 2
    ring = conv_desc(cin=64, cout=32, sp=(18, 32, 64), p=(0, 1, 1))      # rows of more than 16 voxels
    small = conv_desc(cin=256, cout=256, sp=(10, 16, 16), p=(0, 1, 1))   # a small volume: 8 tiles under a block
    large16 = conv_desc(cin=32, cout=32, sp=(64, 64, 16))                  # rows of 16 voxels, hundreds of tiles
    strided = conv_desc(cin=32, cout=32, sp=(8, 8, 32)); strided.sd = 2
    assert L.sfh_conv3d_wgrad_batch_supported(ctypes.byref(ring), bf16) == 1
    assert L.sfh_conv3d_wgrad_batch_supported(ctypes.byref(small), bf16) == 2
    assert L.sfh_conv3d_wgrad_batch_supported(ctypes.byref(large16), bf16) == 0
    assert L.sfh_conv3d_wgrad_batch_supported(ctypes.byref(strided), bf16) == 0
    assert L.sfh_conv3d_wgrad_batch_supported(ctypes.byref(ring), fp32) == 0
    assert L.sfh_conv3d_wgrad_batch_supported(None, bf16) == 0

    def items(*descs):
        arr = (_lib.WgradItem * len(descs))()
        for it, d in zip(arr, descs):
            it.desc = d
        return arr

    one = L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring), 1, bf16, 0)
    two = L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring, ring), 2, bf16, 0)
    mixed = L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring, small), 2, bf16, 0)
    assert one > 0 and two > 0 and mixed > 0
    # every workgroup writes one 32 x 32 x 27 fp32 slice per unit it touches: at least a slice a block, a few hundred at most
    block = 32 * 32 * 27 * 4
    assert 2 * block <= one <= 1024 * block
    assert L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring), 1, bf16, 0) == one        # a pure function of the list
    assert L.sfh_conv3d_wgrad_batch_workspace_bytes(items(small, small), 2, bf16, 0) > 0   # nothing needed, still not 0
    assert L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring, large16), 2, bf16, 0) == 0
    assert L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring), 0, bf16, 0) == 0
    # half of the compute units for a batch that runs beside other work: fewer workgroups, no more slices
    shared = L.sfh_conv3d_wgrad_batch_workspace_bytes(items(ring, ring), 2, bf16, _lib.SFH_FLAG_SHARE_DEVICE)
    assert 0 < shared <= two
    assert L.sfh_conv3d_wgrad_batch_workspace_bytes(items(*([ring] * 17)), 17, bf16, 0) == 0
    addr = ctypes.c_void_p(256)  # never dereferenced: every call below is refused before a launch
    bad = items(ring, large16)
    for it in bad:
        it.x, it.gy, it.gw = addr, addr, addr
    assert L.sfh_conv3d_wgrad_batch(bad, 2, bf16, addr, 1 << 30, 0, None) == _lib.SFH_ERR_UNSUPPORTED
    ok = items(ring)
    assert L.sfh_conv3d_wgrad_batch(ok, 1, bf16, addr, 1 << 30, 0, None) == _lib.SFH_ERR_INVALID          # null tensors
    ok[0].x, ok[0].gy, ok[0].gw = addr, addr, addr
    assert L.sfh_conv3d_wgrad_batch(ok, 1, bf16, addr, one - 256, 0, None) == _lib.SFH_ERR_WORKSPACE
    assert L.sfh_conv3d_wgrad_batch(ok, 1, bf16, None, 0, 0, None) == _lib.SFH_ERR_WORKSPACE
    assert L.sfh_conv3d_wgrad_batch(ok, 1, bf16, addr, one, _lib.SFH_FLAG_FORCE_GENERIC, None) == _lib.SFH_ERR_INVALID
    ok[0].x_second, ok[0].cin_first = addr, 16                                                             # a cut off the 32-channel grid
    assert L.sfh_conv3d_wgrad_batch(ok, 1, bf16, addr, one, 0, None) == _lib.SFH_ERR_UNSUPPORTED


def test_groupnorm_workspace_and_checks():
    L = _lib.lib()
    d = GroupNormDesc(2, 64, 8, 1, 64 ** 3, 1e-5)
    fwd = L.sfh_groupnorm_fwd_workspace_bytes(ctypes.byref(d), 0)
    bwd = L.sfh_groupnorm_bwd_workspace_bytes(ctypes.byref(d), 0)
    assert fwd > 0 and bwd > fwd and fwd % 256 == 0
    assert L.sfh_groupnorm_fwd_workspace_bytes(ctypes.byref(GroupNormDesc(2, 64, 7, 0, 8, 1e-5)), 0) == 0   # C % G != 0
    rc = L.sfh_groupnorm_fwd(ctypes.byref(d), 0, 0, 2, None, None, None, None, None, None, None, 0, None)
    assert rc == _lib.SFH_ERR_INVALID and b"null" in L.sfh_last_error()


def test_groupnorm_from_records_checks_their_size_before_launching():
    """The records a producer left are bounded by their byte size: a count that does not fit is refused, nothing is read."""
    L = _lib.lib()
    d = GroupNormDesc(1, 32, 8, 1, 8 * 8 * 32, 1e-5)
    one = ctypes.c_void_p(256)  # non-null, 16-byte aligned stand-ins that must not be dereferenced
    need = 1 * 16 * 8 * 4 * 4   # N x records x groups x 4 floats
    call = lambda nbytes, records, rec=one: L.sfh_groupnorm_fwd_from_partials(
        ctypes.byref(d), 0, 0, 2, one, None, None, one, 0, one, one, rec, nbytes, records, None)
    assert call(need - 1, 16) == _lib.SFH_ERR_WORKSPACE and b"records" in L.sfh_last_error()
    assert call(need, 0) == _lib.SFH_ERR_INVALID and call(need, 16, None) == _lib.SFH_ERR_INVALID
    assert call(need, 16, ctypes.c_void_p(260)) == _lib.SFH_ERR_INVALID   # off the 16-byte grid
    # the producer side: too few bytes for the records of the problem
    conv = conv_desc(cin=32, cout=32, sp=(8, 8, 32))
    records = L.sfh_conv3d_fwd_gn_records(ctypes.byref(conv), 0, 8)
    assert records > 0
    rc = L.sfh_conv3d_fwd_gn(ctypes.byref(conv), 0, one, one, None, None, one, None, 0, 0, 8, one, records * 8 * 16 - 1, None)
    assert rc == _lib.SFH_ERR_WORKSPACE


def test_transposed_and_copy_entry_points_check_arguments():
    L = _lib.lib()
    d = ConvTDesc(1, 128, 32, 32, 32, 64, 2, 2, 2)
    assert L.sfh_convT3d_fwd_workspace_bytes(ctypes.byref(d), 0) >= 0
    strides = (ctypes.c_int64 * 5)(512, 1, 256, 128, 64)
    assert L.sfh_convT3d_fwd(ctypes.byref(d), 0, None, None, strides, None, None, None, 0, 0, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_stream_copy(None, None, 64, None) == _lib.SFH_ERR_INVALID


def test_argument_checks_of_the_rows_beside_the_convolutions():
    """Loss head, pooling, halo slab, bias gradient and optimizer entry points reject bad arguments with a message
    before anything is launched (so this runs without a GPU)."""
    from scaffold_amd._lib import AdamDesc, HaloDesc, LossDesc, PoolDesc

    L = _lib.lib()
    bf16 = 0
    one = ctypes.c_void_p(16)  # never dereferenced: every call below fails its checks first

    # loss head: classes in [2, 32], positive extents, non-null tensors
    assert L.sfh_ce_dice_workspace_bytes(ctypes.byref(LossDesc(1, 11, 64, 1e-6))) > 0
    assert L.sfh_ce_dice_workspace_bytes(ctypes.byref(LossDesc(1, 1, 64, 1e-6))) == 0
    assert L.sfh_ce_dice_workspace_bytes(ctypes.byref(LossDesc(1, 33, 64, 1e-6))) == 0
    assert L.sfh_ce_dice_fwd(ctypes.byref(LossDesc(1, 11, 64, 1e-6)), bf16, None, one, None, one, one, one, 1 << 20, None) \
        == _lib.SFH_ERR_INVALID
    assert L.sfh_ce_dice_fwd(ctypes.byref(LossDesc(1, 11, 64, 1e-6)), bf16, one, one, None, one, one, None, 0, None) \
        == _lib.SFH_ERR_WORKSPACE
    assert L.sfh_ce_dice_bwd(ctypes.byref(LossDesc(0, 11, 64, 1e-6)), bf16, one, one, None, one, one, one, None) != _lib.SFH_OK

    # pooling
    assert L.sfh_maxpool2_fwd(None, bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_maxpool2_fwd(ctypes.byref(PoolDesc(1, 0, 4, 4, 4)), bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_maxpool2_fwd(ctypes.byref(PoolDesc(1, 8, 4, 4, 4)), 7, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_maxpool2_fwd(ctypes.byref(PoolDesc(1, 8, 4, 4, 4)), bf16, None, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_maxpool2_fwd(ctypes.byref(PoolDesc(1, 8, 1, 4, 4)), bf16, None, None, None, None) == _lib.SFH_OK  # empty output
    assert L.sfh_maxpool2_bwd(ctypes.byref(PoolDesc(1, 8, 4, 4, 4)), bf16, one, None, one, None) == _lib.SFH_ERR_INVALID

    # halo slab
    assert L.sfh_halo_assemble(None, bf16, one, None, None, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_halo_assemble(ctypes.byref(HaloDesc(1, 8, 4, 4, 4, -1)), bf16, one, None, None, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_halo_assemble(ctypes.byref(HaloDesc(1, 8, 4, 4, 4, 1)), bf16, None, None, None, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_halo_assemble(ctypes.byref(HaloDesc(0, 8, 4, 4, 4, 1)), bf16, None, None, None, None, None) == _lib.SFH_OK

    # bias gradient
    assert L.sfh_bias_grad_workspace_bytes(0, 32) == 0 and L.sfh_bias_grad_workspace_bytes(4096, 32) > 0
    assert L.sfh_bias_grad(bf16, bf16, one, 0, 32, one, one, 1 << 20, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_bias_grad(bf16, bf16, one, 4096, 32, one, None, 0, None) == _lib.SFH_ERR_WORKSPACE

    # optimizer: slot count = sum of ceil(numel / 8192); hyperparameter and pointer checks
    numel = (ctypes.c_int64 * 3)(1, 8192, 8193)
    assert L.sfh_adam_slots(3, numel) == 1 + 1 + 2
    assert L.sfh_adam_slots(0, numel) == 0
    ptrs = (ctypes.c_void_p * 3)(16, 16, 16)
    nulls = (ctypes.c_void_p * 3)(16, None, 16)
    assert L.sfh_adam_grad_sumsq(3, nulls, numel, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_adam_grad_sumsq(3, ptrs, (ctypes.c_int64 * 3)(1, 0, 1), one, one, None) == _lib.SFH_ERR_INVALID
    good = AdamDesc(1e-3, 0.9, 0.999, 1e-8, 0.0, 1.0, -1)
    assert L.sfh_adam_clip_step(ctypes.byref(good), 3, ptrs, ptrs, ptrs, nulls, None, numel, one, 4, one, None, None) \
        == _lib.SFH_ERR_INVALID
    bad_beta = AdamDesc(1e-3, 1.0, 0.999, 1e-8, 0.0, 1.0, -1)
    assert L.sfh_adam_clip_step(ctypes.byref(bad_beta), 3, ptrs, ptrs, ptrs, ptrs, None, numel, one, 4, one, None, None) \
        == _lib.SFH_ERR_INVALID
    assert L.sfh_adam_clip_step(ctypes.byref(good), 3, ptrs, ptrs, ptrs, ptrs, ptrs, numel, one, 4, one, None, None) \
        == _lib.SFH_ERR_INVALID  # shadow copies without a shadow dtype
    assert L.sfh_adam_clip_step(ctypes.byref(good), 3, ptrs, ptrs, ptrs, ptrs, None, numel, one, 0, one, None, None) \
        == _lib.SFH_ERR_INVALID  # no slots to fold


def test_argument_checks_of_the_slab_concat_and_batch_packing_entry_points():
    """Rejected before anything is launched, so this runs without a GPU."""
    from scaffold_amd._lib import ConcatDesc, GroupNormDesc, PackItem

    L = _lib.lib()
    bf16 = 0
    one = ctypes.c_void_p(16)  # never dereferenced: every call below fails its checks first

    # skip concat: both channel counts must fill 16-byte pieces; extents positive; tensors non-null
    assert L.sfh_skip_concat_fwd(None, bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_skip_concat_fwd(ctypes.byref(ConcatDesc(1, 32, 0, 64, 0)), bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_skip_concat_fwd(ctypes.byref(ConcatDesc(1, 32, 32, 64, -1)), bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_skip_concat_fwd(ctypes.byref(ConcatDesc(1, 32, 4, 64, 0)), bf16, one, one, one, None) == _lib.SFH_ERR_UNSUPPORTED
    assert b"16-byte" in L.sfh_last_error()
    assert L.sfh_skip_concat_fwd(ctypes.byref(ConcatDesc(1, 32, 32, 64, 8)), bf16, one, None, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_skip_concat_bwd(ctypes.byref(ConcatDesc(1, 32, 32, 64, 8)), bf16, None, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_skip_concat_bwd(ctypes.byref(ConcatDesc(0, 32, 32, 64, 8)), bf16, None, None, None, None) == _lib.SFH_OK  # empty batch

    # GroupNorm into a slab: same checks as the plain forward, plus the halo
    gd = GroupNormDesc(1, 64, 8, 1, 512, 1e-5)
    assert L.sfh_groupnorm_fwd_slab(ctypes.byref(gd), bf16, bf16, bf16, one, None, None, one, -1, one, one, one, 1 << 20, None) \
        == _lib.SFH_ERR_INVALID
    assert L.sfh_groupnorm_fwd_slab(ctypes.byref(gd), bf16, bf16, bf16, one, None, None, None, 64, one, one, one, 1 << 20, None) \
        == _lib.SFH_ERR_INVALID
    assert L.sfh_groupnorm_fwd_slab(None, bf16, bf16, bf16, one, None, None, one, 64, one, one, one, 1 << 20, None) == _lib.SFH_ERR_INVALID

    # batch packing: an empty batch is fine, a bad list or a problem that reads no packed weight is not
    assert L.sfh_conv3d_pack_weights_batch(None, 0, bf16, None) == _lib.SFH_OK
    assert L.sfh_conv3d_pack_weights_batch(None, 2, bf16, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_conv3d_pack_weights_batch(None, -1, bf16, None) == _lib.SFH_ERR_INVALID
    items = (PackItem * 1)()
    items[0].desc = conv_desc(cin=3)
    items[0].w = 16
    items[0].packed_fwd = 16
    assert L.sfh_conv3d_pack_weights_batch(items, 1, bf16, None) == _lib.SFH_ERR_UNSUPPORTED
    items[0].desc = conv_desc()
    items[0].w = None
    assert L.sfh_conv3d_pack_weights_batch(items, 1, bf16, None) == _lib.SFH_ERR_INVALID
    items[0].w = 16
    items[0].packed_fwd = None                      # nothing asked for: nothing launched
    assert L.sfh_conv3d_pack_weights_batch(items, 1, bf16, None) == _lib.SFH_OK


def test_argument_checks_of_the_halo_pack_and_accumulate_entry_points():
    """Rejected (or accepted as empty) before anything is launched, so this runs without a GPU."""
    from scaffold_amd._lib import HaloDesc

    L = _lib.lib()
    bf16 = 0
    one = ctypes.c_void_p(16)  # never dereferenced
    good = HaloDesc(1, 32, 8, 4, 4, 1)
    for fn in (L.sfh_halo_pack, L.sfh_halo_accumulate):
        assert fn(None, bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
        assert fn(ctypes.byref(good), 7, one, one, one, None) == _lib.SFH_ERR_INVALID
        assert fn(ctypes.byref(HaloDesc(1, 0, 8, 4, 4, 1)), bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
        assert fn(ctypes.byref(HaloDesc(1, 32, 8, 4, 4, -1)), bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
        assert fn(ctypes.byref(good), bf16, None, one, one, None) == _lib.SFH_ERR_INVALID
        assert fn(ctypes.byref(HaloDesc(0, 32, 8, 4, 4, 1)), bf16, None, None, None, None) == _lib.SFH_OK   # empty batch
        assert fn(ctypes.byref(HaloDesc(1, 32, 8, 4, 4, 0)), bf16, None, None, None, None) == _lib.SFH_OK   # no halo
    assert L.sfh_halo_pack(ctypes.byref(HaloDesc(1, 32, 2, 4, 4, 3)), bf16, one, one, one, None) == _lib.SFH_ERR_INVALID
    assert L.sfh_halo_accumulate(ctypes.byref(HaloDesc(1, 32, 3, 4, 4, 2)), bf16, one, one, one, None) == _lib.SFH_ERR_UNSUPPORTED
    assert b"overlap" in L.sfh_last_error()


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 and as C++, and a C caller links and runs -- here only calls
    that need no GPU (version, an argument check, the error string)."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no C compiler here")
    include = os.path.join(ROOT, "include")
    libdir = os.path.dirname(_lib.lib_path())
    src = tmp_path / "caller.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "scaffold_hip.h"\n'
        "int main(void) {\n"
        "  sfh_ingest_desc d = {1, 9, 0, 64, 0};  /* nine channels: refused before any launch */\n"
        "  char one[16] = {0};\n"
        "  int rc = sfh_shard_ingest(&d, SFH_BF16, one, NULL, one, NULL, NULL);\n"
        '  printf("%d %d %s\\n", sfh_version(), rc, sfh_last_error());\n'
        "  return rc == SFH_ERR_UNSUPPORTED && strstr(sfh_last_error(), \"channels\") != NULL ? 0 : 1;\n"
        "}\n")
    exe = tmp_path / "caller"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", f"-I{include}", str(src), "-o", str(exe), f"-L{libdir}",
                    "-lscaffold_hip", f"-Wl,-rpath,{libdir}"], check=True, capture_output=True, text=True)
    if shutil.which("g++") is not None:
        cpp = tmp_path / "caller.cpp"
        cpp.write_text('#include "scaffold_hip.h"\nint main() { return sfh_version() > 0 ? 0 : 1; }\n')
        subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", f"-I{include}", str(cpp)], check=True,
                       capture_output=True, text=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, (out.stdout, out.stderr)
    assert out.stdout.split()[0] == str(_lib.lib().sfh_version())
