"""The convolution over a skip connection that is never concatenated (``conv3d_forward_pair`` and its two gradients),
through the C ABI.

The reference writes ``torch.cat([skip, upsampled], dim=1)`` (``ScaFFold/unet/unet_parts.py:107-120``) and convolves that
tensor.  The pair entry points read / write the two tensors themselves, and what they are held to is the strongest
statement available: every result is the SAME BITS as the ordinary entry point on the concatenated tensor (which the
convolution parity tests hold to the oracle), on Gaussian operands, for every kernel that can serve such a problem --
the brick-per-workgroup kernel with and without a sliced reduction, the wide-tile kernel, the persistent kernel (data
gradient of a 32-channel output) and the weight-gradient kernel -- with ragged extents, several samples, the depth-shard
form and unequal cuts.  One case per kernel is also checked directly against the fp64 oracle.
"""

import pytest
import torch

import scaffold_amd as sa
from oracle import oracle as orc
from scaffold_amd import conv3d as c3

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d

# (n, c_first, c_second, cout, spatial, padding, forward kernel, data-gradient kernel)
CASES = [
    (1, 32, 32, 32, (8, 16, 64), (1, 1, 1), "brick", "persist"),     # the level-0 decoder shape: 64 -> 32
    (2, 32, 32, 32, (5, 7, 33), (0, 1, 1), "brick", "persist"),      # two samples, ragged, shard form
    (1, 32, 64, 32, (6, 8, 16), (1, 1, 1), "brick", "persist"),      # unequal cut, rows of 16
    (1, 64, 32, 32, (9, 8, 8), (1, 1, 1), "brick", "persist"),       # unequal cut the other way, rows of 8
    (1, 64, 64, 64, (32, 64, 64), (0, 1, 1), "wide", "brick"),       # the level-1 decoder shape: wide forward
    (1, 64, 64, 64, (31, 61, 65), (1, 1, 1), "wide", "brick"),       # ragged on every axis
    (1, 32, 96, 64, (32, 64, 64), (1, 1, 1), None, "brick"),         # wide forward takes equal halves only: not offered
    (1, 64, 64, 128, (9, 192, 16), (1, 1, 1), "brick", "brick"),     # rows of 16: the brick kernel, two blocks a workgroup
    (1, 64, 64, 128, (16, 32, 16), (1, 1, 1), "split", "split"),     # a small volume: the reduction cut over the wavefronts
    (2, 128, 128, 128, (10, 20, 32), (1, 1, 1), "split", "split"),   # the level-2 decoder shape, two rounds of four chunks
    (1, 256, 256, 256, (10, 16, 16), (0, 1, 1), "brick", "split"),   # level 3 on a shard: forward sliced
    (1, 256, 256, 256, (8, 16, 16), (1, 1, 1), "brick", "split"),    # ... and as a cube
    (1, 128, 128, 256, (8, 16, 16), (1, 1, 1), "split", "split"),    # two rounds of four chunks from the two tensors in turn
    (1, 96, 160, 128, (7, 13, 35), (1, 1, 1), "split", "split"),     # unequal cut inside a round, ragged
    (1, 256, 256, 512, (4, 8, 8), (1, 1, 1), "brick", "brick"),      # level 4: both directions sliced
    (1, 128, 64, 96, (4, 8, 8), (1, 1, 1), "brick", "brick"),        # sliced, unequal cut, 96 output channels
    (3, 32, 32, 64, (4, 8, 24), (1, 1, 1), "brick", "brick"),        # three samples, two output blocks
]


def _operands(case, dtype, device, seed=11):
    n, c0, c1, cout, spatial, padding, _, _ = case
    prob = orc.ConvProblem(n=n, cin=c0 + c1, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    ops = orc.make_inputs(prob, seed=seed)
    x = ops["input"].to(device).contiguous(memory_format=CL)
    w = ops["weight"].to(device)
    gy = ops["grad_output"].to(device).contiguous(memory_format=CL)
    first = x[:, :c0].contiguous(memory_format=CL)
    second = x[:, c0:].contiguous(memory_format=CL)
    return prob, x, first, second, w, gy


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[1]}+{c[2]}->{c[3]}@{'x'.join(map(str, c[4]))}")
def test_pair_is_bitwise_the_concatenation(device, dtype, case):
    n, c0, c1, cout, spatial, padding, fwd_kernel, dgrad_kernel = case
    prob, x, first, second, w, gy = _operands(case, dtype, device)
    offered = c3.is_supported_pair(first, second, w, None, 1, padding, 1)
    assert offered == (fwd_kernel is not None)
    if fwd_kernel is not None:
        assert c3.launch_geometry(x.shape, w.shape, 1, padding, 1, dtype, "fwd")["kernel"] == fwd_kernel
        bias = (torch.arange(cout, device=device) % 7 - 3).to(dtype) / 4
        want = sa.conv3d_forward(x, w, bias, 1, padding, 1)
        got = c3.conv3d_forward_pair(first, second, w, bias, 1, padding, 1)
        assert torch.equal(got, want)
        # with a packed weight and the statistics of a following GroupNorm
        pf, _ = c3.pack_weights(w, x.shape, 1, padding, 1)
        want = sa.conv3d_forward(x, w, None, 1, padding, 1, packed_weight=pf, gn_groups=8)
        got = c3.conv3d_forward_pair(first, second, w, None, 1, padding, 1, packed_weight=pf, gn_groups=8)
        assert torch.equal(got, want)
        assert hasattr(got, "_sfh_gn_partials") == hasattr(want, "_sfh_gn_partials")
        if hasattr(want, "_sfh_gn_partials"):
            assert torch.equal(got._sfh_gn_partials[0], want._sfh_gn_partials[0]) and got._sfh_gn_partials[1] == want._sfh_gn_partials[1]
    else:
        with pytest.raises(NotImplementedError):
            c3.conv3d_forward_pair(first, second, w, None, 1, padding, 1)
    # data gradient: the two tensors are the channel split of the ordinary result
    assert c3.launch_geometry(x.shape, w.shape, 1, padding, 1, dtype, "bwd-data")["kernel"] == dgrad_kernel
    want = sa.conv3d_backward_data(gy, w, x.shape, 1, padding, 1)
    g0, g1 = c3.conv3d_backward_data_pair(gy, w, x.shape, c0, 1, padding, 1)
    assert g0.shape == first.shape and g1.shape == second.shape
    assert g0.is_contiguous(memory_format=CL) and g1.is_contiguous(memory_format=CL)
    assert torch.equal(g0, want[:, :c0]) and torch.equal(g1, want[:, c0:])
    # weight gradient, in the operands' dtype and in fp32
    for grad_dtype in (None, torch.float32):
        want = sa.conv3d_backward_weight(x, w.shape, gy, 1, padding, 1, grad_dtype=grad_dtype)
        got = c3.conv3d_backward_weight_pair(first, second, w.shape, gy, 1, padding, 1, grad_dtype=grad_dtype)
        assert got.dtype is want.dtype and torch.equal(got, want)


@pytest.mark.parametrize("case", [CASES[0], CASES[4], CASES[10], CASES[12], CASES[13], CASES[14], CASES[15]],
                         ids=["brick-persist", "wide", "sliced-shard", "split", "split-unequal", "sliced", "sliced-unequal"])
def test_pair_against_the_oracle(device, case):
    """Straight to the fp64 oracle on the concatenated operands, with the error bound of the convolution parity tests."""
    n, c0, c1, cout, spatial, padding, _, _ = case
    dtype = torch.bfloat16
    prob = orc.ConvProblem(n=n, cin=c0 + c1, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    ops = orc.make_inputs(prob, seed=5)
    ops["weight"] = (ops["weight"].float() / (prob.cin * 27) ** 0.5).to(dtype)
    x = ops["input"].to(device)
    first, second = x[:, :c0].contiguous(memory_format=CL), x[:, c0:].contiguous(memory_format=CL)
    w, gy = ops["weight"].to(device), ops["grad_output"].to(device)
    y = c3.conv3d_forward_pair(first, second, w, None, 1, padding, 1)
    g0, g1 = c3.conv3d_backward_data_pair(gy, w, x.shape, c0, 1, padding, 1)
    gw = c3.conv3d_backward_weight_pair(first, second, w.shape, gy, 1, padding, 1)
    orc.assert_close(y, orc.conv_reference(prob, ops, "fwd"), prob, "fwd")
    orc.assert_close(torch.cat([g0, g1], 1), orc.conv_reference(prob, ops, "bwd-data"), prob, "bwd-data")
    orc.assert_close(gw, orc.conv_reference(prob, ops, "bwd-weight"), prob, "bwd-weight")


def test_what_is_refused(device):
    dtype = torch.bfloat16
    mk = lambda c, sp=(4, 8, 32): torch.randn(1, c, *sp, device=device, dtype=dtype).contiguous(memory_format=CL)
    w = torch.randn(32, 64, 3, 3, 3, device=device, dtype=dtype)
    assert c3.is_supported_pair(mk(32), mk(32), w, None, 1, 1, 1)
    assert not c3.is_supported_pair(mk(16), mk(48), w, None, 1, 1, 1)               # a cut off the 32-channel grid
    assert not c3.is_supported_pair(mk(32), mk(32, (4, 8, 16)), w, None, 1, 1, 1)    # different voxels
    assert not c3.is_supported_pair(mk(32), mk(32).float(), w, None, 1, 1, 1)        # different dtypes
    assert not c3.is_supported_pair(mk(32).float(), mk(32).float(), w.float(), None, 1, 1, 1)  # the fp32 tiles read one tensor
    assert not c3.is_supported_pair(mk(32), mk(32), w, None, 2, 1, 1)                # strided: no data gradient
    w1 = torch.randn(32, 64, 1, 1, 1, device=device, dtype=dtype)
    assert not c3.is_supported_pair(mk(32), mk(32), w1, None, 1, 0, 1)               # not a 3x3x3 problem
    with pytest.raises(NotImplementedError):
        c3.conv3d_forward_pair(mk(16), mk(48), w, None, 1, 1, 1)
    with pytest.raises(NotImplementedError):
        c3.conv3d_backward_data_pair(mk(32), w, (1, 64, 4, 8, 32), 16, 1, 1, 1)
    with pytest.raises(NotImplementedError):
        c3.conv3d_backward_weight_pair(mk(16), mk(48), w.shape, mk(32), 1, 1, 1)
