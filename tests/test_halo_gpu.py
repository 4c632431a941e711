"""Halo slab assembly against torch.cat: a pure data movement, so results and gradients must be bitwise equal."""

import pytest
import torch

import scaffold_amd as sa

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,halo", [((1, 32, 8, 8, 16), 1), ((2, 5, 3, 4, 7), 1), ((1, 64, 4, 6, 6), 2),
                                        ((3, 1, 5, 5, 5), 1), ((1, 8, 1, 2, 2), 3)])
@pytest.mark.parametrize("neighbours", ["none", "lo", "hi", "both"])
def test_equals_cat_with_zeros_for_missing_neighbours(device, shape, halo, dtype, neighbours):
    g = torch.Generator().manual_seed(41)
    n, c, d, h, w = shape
    x = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    mk = lambda: torch.randn((n, c, halo, h, w), generator=g).to(dtype).contiguous(memory_format=CL).to(device)  # noqa: E731
    lo = mk() if neighbours in ("lo", "both") else None
    hi = mk() if neighbours in ("hi", "both") else None
    zeros = torch.zeros((n, c, halo, h, w), dtype=dtype, device=device)
    want = torch.cat([zeros if lo is None else lo, x, zeros if hi is None else hi], dim=2)
    got = sa.halo_assemble(x, lo, hi, halo)
    assert got.shape == want.shape and got.is_contiguous(memory_format=CL)
    assert torch.equal(got, want)


def test_gradient_is_sliced_back_to_the_shard_and_the_borrowed_slabs(device):
    g = torch.Generator().manual_seed(42)
    x = torch.randn((2, 16, 4, 5, 6), generator=g).contiguous(memory_format=CL).to(device).requires_grad_(True)
    lo = torch.randn((2, 16, 1, 5, 6), generator=g).contiguous(memory_format=CL).to(device).requires_grad_(True)
    hi = torch.randn((2, 16, 1, 5, 6), generator=g).contiguous(memory_format=CL).to(device).requires_grad_(True)
    gout = torch.randn((2, 16, 6, 5, 6), generator=g).contiguous(memory_format=CL).to(device)
    sa.halo_assemble(x, lo, hi, 1).backward(gout)
    assert torch.equal(x.grad, gout[:, :, 1:5]) and torch.equal(lo.grad, gout[:, :, :1]) and torch.equal(hi.grad, gout[:, :, 5:])


def test_feeding_a_convolution_equals_ordinary_padding(device):
    """The slab convolved at depth padding 0 is the shard convolved at padding 1 (zero neighbours): bit for bit."""
    g = torch.Generator().manual_seed(43)
    x = torch.randn((1, 32, 8, 8, 16), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    w = (torch.randn((32, 32, 3, 3, 3), generator=g) * 0.05).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    y_pad = sa.conv3d_forward(x, w, None, 1, 1, 1)
    y_slab = sa.conv3d_forward(sa.halo_assemble(x, None, None, 1), w, None, 1, (0, 1, 1), 1)
    assert torch.equal(y_pad, y_slab)


def test_gates(device):
    x = torch.randn((1, 4, 2, 2, 2), device=device)
    assert sa.halo_assemble(x, None, None, 0) is x
    assert not sa.is_supported_halo(torch.randn(1, 4, 2, 2, 2))
    assert not sa.is_supported_halo(x, torch.zeros((1, 4, 2, 2, 2), device=device), None, 1)   # slab of the wrong depth
    assert not sa.is_supported_halo(x, None, None, -1)
    with pytest.raises(NotImplementedError):
        sa.halo_assemble(x, torch.zeros((1, 4, 1, 2, 2), device=device, dtype=torch.bfloat16), None, 1)
