"""MaxPool3d(2) kernels against the stock op: values and routed gradients must be bitwise equal (pooling selects,
it never rounds), on even, odd, tiny and full-size volumes, with ties and NaNs."""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import scaffold_amd as sa

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d

SHAPES = [
    # n, c, d, h, w
    (1, 32, 8, 8, 16),
    (2, 64, 6, 10, 12),
    (1, 8, 5, 7, 9),       # odd everywhere: trailing planes dropped, their gradient is zero
    (3, 5, 4, 6, 8),       # channel count with no vector form
    (1, 1, 2, 2, 2),
    (1, 12, 3, 2, 5),
    (1, 256, 4, 8, 8),
    (2, 17, 7, 3, 4),
]


def _stock(x, gy=None):
    xr = x.detach().clone().requires_grad_(True)
    y = F.max_pool3d(xr, 2)
    if gy is None:
        return y.detach(), None
    y.backward(gy)
    return y.detach(), xr.grad


def _ours(x, gy=None):
    xr = x.detach().clone().requires_grad_(True)
    y = sa.max_pool3d_2x(xr)
    if gy is None:
        return y.detach(), None
    y.backward(gy)
    return y.detach(), xr.grad


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
def test_matches_stock_bitwise(device, shape, dtype):
    g = torch.Generator().manual_seed(hash(shape) % 1000)
    n, c, d, h, w = shape
    x = torch.randn((n, c, d, h, w), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    gy = torch.randn((n, c, d // 2, h // 2, w // 2), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    y0, gx0 = _stock(x, gy)
    y1, gx1 = _ours(x, gy)
    assert y1.shape == y0.shape and y1.dtype == dtype
    assert y1.is_contiguous(memory_format=CL) or y1.numel() <= c
    assert torch.equal(y1, y0)
    assert gx1.shape == x.shape and torch.equal(gx1, gx0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ties_route_to_the_first_voxel_like_stock(device, dtype):
    """Few distinct values: most cells hold ties; every tie must send its gradient where the stock op sends it."""
    g = torch.Generator().manual_seed(11)
    x = torch.randint(0, 3, (2, 16, 6, 8, 10), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    gy = torch.randint(1, 5, (2, 16, 3, 4, 5), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    y0, gx0 = _stock(x, gy)
    y1, gx1 = _ours(x, gy)
    assert torch.equal(y1, y0) and torch.equal(gx1, gx0)
    # closed form for an all-equal input: the whole gradient lands on the cell's first voxel
    ones = torch.ones((1, 8, 4, 4, 4), dtype=dtype, device=device).contiguous(memory_format=CL)
    _, gx = _ours(ones, torch.full((1, 8, 2, 2, 2), 3.0, dtype=dtype, device=device).contiguous(memory_format=CL))
    want = torch.zeros_like(ones)
    want[:, :, ::2, ::2, ::2] = 3.0
    assert torch.equal(gx, want)


def test_nan_and_infinities_follow_stock(device):
    g = torch.Generator().manual_seed(12)
    x = torch.randn((1, 8, 4, 4, 8), generator=g)
    x[0, 0, 0, 0, 1] = float("nan")
    x[0, 1, 1, 1, 0] = float("nan")
    x[0, 1, 0, 1, 1] = float("nan")   # two NaNs in one cell
    x[0, 2, :2, :2, :2] = float("-inf")
    x[0, 3, 2, 2, 2] = float("inf")
    x = x.contiguous(memory_format=CL).to(device)
    gy = torch.ones((1, 8, 2, 2, 4), device=device).contiguous(memory_format=CL)
    y0, gx0 = _stock(x, gy)
    y1, gx1 = _ours(x, gy)
    assert torch.equal(torch.isnan(y1), torch.isnan(y0))
    assert torch.equal(torch.nan_to_num(y1, nan=7.0), torch.nan_to_num(y0, nan=7.0))
    assert torch.equal(gx1, gx0)


def test_accepts_any_memory_format_and_returns_channels_last(device):
    x = torch.randn((2, 16, 4, 6, 8), device=device)  # NCDHW-contiguous
    y = sa.max_pool3d_2x(x)
    assert torch.equal(y, F.max_pool3d(x, 2))
    assert y.is_contiguous(memory_format=CL)


def test_empty_output_and_gates(device):
    x = torch.randn((1, 4, 1, 4, 4), device=device).contiguous(memory_format=CL).requires_grad_(True)
    y = sa.max_pool3d_2x(x)
    assert y.shape == (1, 4, 0, 2, 2)
    y.sum().backward()
    assert torch.equal(x.grad, torch.zeros_like(x))
    assert not sa.is_supported_pool(torch.randn(2, 3, 4, 4))
    assert not sa.is_supported_pool(torch.randn(1, 2, 4, 4, 4))            # host tensor
    assert not sa.is_supported_pool(torch.zeros((1, 2, 4, 4, 4), dtype=torch.int32, device=device))
    with pytest.raises(NotImplementedError):
        sa.max_pool3d_2x(torch.randn(1, 2, 4, 4, 4))


def test_module_is_a_drop_in_and_rejects_other_configurations(device):
    m = sa.FastMaxPool3d(2)
    assert isinstance(m, nn.MaxPool3d) and not list(m.state_dict())
    x = torch.randn((1, 32, 8, 8, 8), device=device).contiguous(memory_format=CL)
    assert torch.equal(m(x), nn.MaxPool3d(2)(x))
    for bad in (sa.FastMaxPool3d(3), sa.FastMaxPool3d(2, stride=1), sa.FastMaxPool3d(2, padding=1),
                sa.FastMaxPool3d(2, ceil_mode=True), sa.FastMaxPool3d(2, return_indices=True)):
        with pytest.raises(NotImplementedError):
            bad(x)


def test_second_order_differentiation_raises(device):
    x = torch.randn((1, 8, 4, 4, 4), device=device).contiguous(memory_format=CL).requires_grad_(True)
    y = sa.max_pool3d_2x(x)
    (gx,) = torch.autograd.grad(y.sum(), x, create_graph=True)
    with pytest.raises(RuntimeError):
        gx.sum().backward()


def test_full_size_level0_properties(device):
    """The U-Net's largest pooling (32 channels, 64x128x128): the gradient of sum(y) is a 0/1 mask with exactly
    one hit per cell and channel, the hit voxel holds the pooled value, and the values equal the stock op's."""
    g = torch.Generator(device=device).manual_seed(13)
    x = torch.randn((1, 32, 64, 128, 128), generator=g, device=device, dtype=torch.bfloat16).contiguous(memory_format=CL)
    xr = x.clone().requires_grad_(True)
    y = sa.max_pool3d_2x(xr)
    y.backward(torch.ones_like(y))
    gx = xr.grad
    cells = gx.reshape(1, 32, 32, 2, 64, 2, 64, 2).float().sum(dim=(3, 5, 7))
    assert torch.equal(cells, torch.ones_like(cells))
    picked = (gx.float() * x.float()).reshape(1, 32, 32, 2, 64, 2, 64, 2).sum(dim=(3, 5, 7))
    assert torch.equal(picked, y.detach().float())
    assert torch.equal(y.detach(), F.max_pool3d(x, 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32, 6, 8, 10), (2, 16, 5, 7, 9), (1, 3, 4, 4, 6)])
def test_pool_with_skip_sums_both_gradients_in_one_kernel(device, dtype, shape):
    """``max_pool3d_2x_with_skip``: the pooled tensor and an alias of the input for the skip connection; the input's
    gradient is the bits autograd's own accumulation gives (one fp32 sum, one rounding)."""
    from scaffold_amd.pooling import max_pool3d_2x_with_skip

    g = torch.Generator().manual_seed(17)
    x0 = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    n, c, d, h, w = shape
    gy = torch.randn((n, c, d // 2, h // 2, w // 2), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    gs = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    a = x0.clone().requires_grad_(True)
    pooled, skip = max_pool3d_2x_with_skip(a)
    assert skip is not a and skip.data_ptr() == a.data_ptr() and torch.equal(pooled, F.max_pool3d(x0, 2))
    torch.autograd.backward([pooled, skip], [gy, gs])
    b = x0.clone().requires_grad_(True)
    torch.autograd.backward([sa.max_pool3d_2x(b), b * 1], [gy, gs])
    assert torch.equal(a.grad, b.grad)
    # only one of the two uses differentiated
    c1 = x0.clone().requires_grad_(True)
    p1, s1 = max_pool3d_2x_with_skip(c1)
    p1.backward(gy)
    d1 = x0.clone().requires_grad_(True)
    sa.max_pool3d_2x(d1).backward(gy)
    assert torch.equal(c1.grad, d1.grad)
    c2 = x0.clone().requires_grad_(True)
    _, s2 = max_pool3d_2x_with_skip(c2)
    s2.backward(gs)
    assert torch.equal(c2.grad, gs)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,halo", [((1, 32, 8, 12, 20), 1), ((1, 64, 5, 9, 7), 1), ((1, 8, 4, 4, 6), 2), ((1, 3, 6, 6, 6), 1), ((2, 32, 4, 8, 8), 1)])
def test_pooling_into_a_depth_slab_is_bitwise_the_plain_result(device, dtype, shape, halo):
    """``max_pool3d_2x(x, out_halo=h)`` / ``with_skip``: the result lies in the interior of a slab whose faces the launch
    zeroes, and is the plain result in values and gradients; where the library does not offer a slab (a batch, faces off the
    16-byte grid) the plain tensor comes back."""
    torch.manual_seed(7)
    x0 = torch.randn(shape, device=device).to(dtype).contiguous(memory_format=CL)
    n, c, d, h, w = shape
    gy = torch.randn((n, c, d // 2, h // 2, w // 2), device=device).to(dtype).contiguous(memory_format=CL)
    gs = torch.randn(shape, device=device).to(dtype).contiguous(memory_format=CL)
    from scaffold_amd import pooling

    def run(out_halo, with_skip):
        x = x0.clone().requires_grad_(True)
        if with_skip:
            y, skip = pooling.max_pool3d_2x_with_skip(x, out_halo)
            (y * gy).sum().backward(retain_graph=True)
            skip.backward(gs)
        else:
            y = pooling.max_pool3d_2x(x, out_halo)
            y.backward(gy)
        return y, x.grad

    for with_skip in (False, True):
        y_plain, g_plain = run(0, with_skip)
        y_slab, g_slab = run(halo, with_skip)
        assert torch.equal(y_plain, y_slab) and torch.equal(g_plain, g_slab)
        offered = n == 1 and (halo * (h // 2) * (w // 2) * c * x0.element_size()) % 16 == 0 and (y_plain.numel() * x0.element_size()) % 16 == 0
        assert hasattr(y_slab, "_sfh_slab") == offered
        if offered:
            slab, hh = y_slab._sfh_slab
            assert hh == halo and slab.shape == (1, c, d // 2 + 2 * halo, h // 2, w // 2)
            assert y_slab.is_contiguous(memory_format=CL) and torch.equal(slab[:, :, halo:halo + d // 2], y_plain)
            assert not slab[:, :, :halo].any() and not slab[:, :, halo + d // 2:].any()
