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


# ---- the sending side, the backward's accumulation, and the exchange as one node ----------------------------------
PACK_SHAPES = [((1, 32, 8, 8, 16), 1), ((2, 5, 3, 4, 7), 1), ((1, 64, 4, 6, 6), 2), ((3, 1, 5, 5, 5), 2), ((1, 8, 6, 2, 2), 3),
               ((1, 3, 2, 5, 3), 1)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,halo", PACK_SHAPES)
def test_pack_copies_the_boundary_planes_into_plain_wire_buffers(device, shape, halo, dtype):
    g = torch.Generator().manual_seed(43)
    x = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    lo, hi = sa.halo_pack(x, halo)
    assert torch.equal(lo, x[:, :, :halo]) and torch.equal(hi, x[:, :, -halo:])
    for t in (lo, hi):      # what goes on the wire is plain contiguous as (N, halo, H, W, C)
        assert t.permute(0, 2, 3, 4, 1).is_contiguous() and t.shape == (shape[0], shape[1], halo) + shape[3:]
    only_lo, none = sa.halo_pack(x, halo, hi=False)
    assert none is None and torch.equal(only_lo, lo)
    none, only_hi = sa.halo_pack(x, halo, lo=False)
    assert none is None and torch.equal(only_hi, hi)
    # from an NCDHW-contiguous tensor: relaid out, not misread
    lo2, hi2 = sa.halo_pack(x.contiguous(), halo)
    assert torch.equal(lo2, lo) and torch.equal(hi2, hi)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,halo", PACK_SHAPES)
@pytest.mark.parametrize("neighbours", ["lo", "hi", "both"])
def test_accumulate_is_add_in_place_on_the_boundary_planes(device, shape, halo, dtype, neighbours):
    g = torch.Generator().manual_seed(44)
    n, c, d, h, w = shape
    grad = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    mk = lambda: torch.randn((n, c, halo, h, w), generator=g).to(dtype).contiguous(memory_format=CL).to(device)  # noqa: E731
    lo = mk() if neighbours in ("lo", "both") else None
    hi = mk() if neighbours in ("hi", "both") else None
    want = grad.clone()
    if lo is not None:
        want[:, :, :halo].add_(lo)          # the reference's own two statements (conv3d.py:838-841)
    if hi is not None:
        want[:, :, -halo:].add_(hi)
    got = sa.halo_accumulate_(grad, lo, hi, halo)
    assert got is grad and torch.equal(grad, want)


def test_accumulate_on_the_interior_of_a_slab_and_its_refusals(device):
    g = torch.Generator().manual_seed(45)
    slab = torch.randn((1, 16, 8, 4, 6), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    lo = torch.randn((1, 16, 1, 4, 6), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    want = slab.clone()
    want[:, :, 1:2].add_(lo)
    inner = slab[:, :, 1:7]
    sa.halo_accumulate_(inner, lo, None, 1)
    assert torch.equal(slab, want)          # through the view, nothing outside the interior touched
    batch = torch.zeros((2, 16, 8, 4, 6), dtype=torch.bfloat16, device=device).contiguous(memory_format=CL)
    with pytest.raises(ValueError):         # a batch's interior is not dense: refused rather than copied silently
        sa.halo_accumulate_(batch[:, :, 1:7], torch.cat([lo, lo]), None, 1)
    with pytest.raises(NotImplementedError):
        sa.halo_accumulate_(slab[:, :, :1], lo, lo, 1)      # thinner than two halos
    with pytest.raises(NotImplementedError):
        sa.halo_accumulate_(slab, lo[:, :8], None, 1)       # face of another shape
    with pytest.raises(NotImplementedError):
        sa.halo_pack(slab, 9)


def _conv_args(device, cin=32, cout=32, dtype=torch.bfloat16, seed=46):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn((cout, cin, 3, 3, 3), generator=g) / (27 * cin) ** 0.5).to(dtype).contiguous(memory_format=CL).to(device)
    b = torch.randn(cout, generator=g).to(dtype).to(device)
    return w, b


@pytest.mark.parametrize("dtype, tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_exchange_node_with_itself_as_both_neighbours_is_circular_padding(device, dtype, tol):
    """A shard whose two neighbours are itself sees a volume that is periodic in depth, and torch can state that
    directly: the node's forward and backward against F.pad(mode="circular") + F.conv3d under autograd, in fp64."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(47)
    x = torch.randn((1, 32, 6, 8, 16), generator=g).to(dtype).contiguous(memory_format=CL)
    gy = torch.randn((1, 32, 6, 8, 16), generator=g).to(dtype).contiguous(memory_format=CL)
    w, b = _conv_args(device, dtype=dtype)
    calls = []

    def myself(send_lo, send_hi):
        calls.append((send_lo.shape, send_hi.shape))
        return send_hi, send_lo             # what I send down comes back from above, and the other way round

    xd = x.to(device).requires_grad_(True)
    slab = sa.halo_exchange(xd, 1, myself)
    y = sa.conv3d_forward(slab.detach(), w, b, 1, (0, 1, 1))
    assert torch.equal(slab.detach()[:, :, 0], xd.detach()[:, :, -1]) and torch.equal(slab.detach()[:, :, -1], xd.detach()[:, :, 0])
    gslab = sa.conv3d_backward_data(gy.to(device), w, slab.shape, 1, (0, 1, 1))
    slab.backward(gslab)
    assert len(calls) == 2                  # one round of communication per direction

    x64 = x.double().requires_grad_(True)
    ref = F.conv3d(F.pad(x64, (0, 0, 0, 0, 1, 1), mode="circular"), w.cpu().double(), b.cpu().double(), padding=(0, 1, 1))
    ref.backward(gy.double())
    ref = ref.detach()
    scale = lambda t: float(t.abs().max())  # noqa: E731
    assert float((y.cpu().double() - ref).abs().max()) <= tol * scale(ref) + (1e-2 if dtype is torch.bfloat16 else 0)
    # bf16: the slab gradient is rounded once before the two boundary sums and once after
    assert float((xd.grad.cpu().double() - x64.grad).abs().max()) <= 2 * tol * scale(x64.grad) + (1e-2 if dtype is torch.bfloat16 else 0)


@pytest.mark.parametrize("dtype, tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_two_depth_shards_on_one_gpu_reproduce_the_unsharded_convolution(device, dtype, tol):
    """Both halves of a volume as two shards of one process, the wire replaced by handing the packed buffers across:
    forward slabs and outputs, and the data gradient after the backward exchange, against the unsharded convolution
    (how the reference checks its two-rank run, triton_conv3d/bench/conv3d_shards_2rank.py:96-98)."""
    g = torch.Generator().manual_seed(48)
    full = torch.randn((1, 32, 12, 8, 16), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    gy = torch.randn((1, 32, 12, 8, 16), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    w, b = _conv_args(device, dtype=dtype, seed=49)
    top, bottom = full[:, :, :6].contiguous(memory_format=CL), full[:, :, 6:].contiguous(memory_format=CL)

    # forward exchange: each shard sends its boundary planes towards the other
    _, top_down = sa.halo_pack(top, 1, lo=False)
    bottom_up, _ = sa.halo_pack(bottom, 1, hi=False)
    slab_top = sa.halo_assemble(top, None, bottom_up, 1)
    slab_bottom = sa.halo_assemble(bottom, top_down, None, 1)
    assert torch.equal(slab_top[:, :, 1:], full[:, :, :7]) and torch.equal(slab_bottom[:, :, :-1], full[:, :, 5:])
    y = torch.cat([sa.conv3d_forward(slab_top, w, b, 1, (0, 1, 1)), sa.conv3d_forward(slab_bottom, w, b, 1, (0, 1, 1))], dim=2)
    y_full = sa.conv3d_forward(full, w, b, 1, 1)
    assert torch.equal(y, y_full)           # same taps in the same order for every output voxel

    # backward exchange: the outer planes of each slab gradient return to the shard they were borrowed from
    g_top = sa.conv3d_backward_data(gy[:, :, :6].contiguous(memory_format=CL), w, slab_top.shape, 1, (0, 1, 1))
    g_bottom = sa.conv3d_backward_data(gy[:, :, 6:].contiguous(memory_format=CL), w, slab_bottom.shape, 1, (0, 1, 1))
    _, top_returns = sa.halo_pack(g_top, 1, lo=False)          # gradient of the plane borrowed from `bottom`
    bottom_returns, _ = sa.halo_pack(g_bottom, 1, hi=False)    # gradient of the plane borrowed from `top`
    gx_top = sa.halo_accumulate_(g_top[:, :, 1:7], None, bottom_returns, 1)
    gx_bottom = sa.halo_accumulate_(g_bottom[:, :, 1:7], top_returns, None, 1)
    gx = torch.cat([gx_top, gx_bottom], dim=2)
    gx_full = sa.conv3d_backward_data(gy, w, full.shape, 1, 1)
    err = float((gx.float() - gx_full.float()).abs().max())
    assert err <= tol * float(gx_full.float().abs().max()) + (1e-2 if dtype is torch.bfloat16 else 0)
    if dtype is torch.float32:              # away from the cut nothing was added: bitwise the unsharded gradient
        assert torch.equal(gx[:, :, :5], gx_full[:, :, :5]) and torch.equal(gx[:, :, 7:], gx_full[:, :, 7:])
