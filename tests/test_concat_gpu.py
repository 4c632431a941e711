"""GPU parity of the skip-connection concat kernel: bit for bit ``torch.cat`` and its backward slices."""

import pytest
import torch

import scaffold_amd as sa

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,ca,cb,sp,halo", [
    (1, 32, 32, (6, 10, 12), 1),
    (1, 64, 8, (3, 5, 7), 2),
    (1, 8, 40, (1, 1, 3), 1),
    (2, 16, 24, (4, 6, 5), 1),      # a batch keeps the plain form
    (1, 32, 32, (5, 4, 9), 0),
])
def test_concat_and_split_are_bitwise_torch(device, dtype, n, ca, cb, sp, halo):
    g = torch.Generator().manual_seed(5)
    a0 = torch.randn((n, ca, *sp), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    b0 = torch.randn((n, cb, *sp), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    gy = torch.randn((n, ca + cb, *sp), generator=g).to(dtype).contiguous(memory_format=CL).to(device)
    a, b = a0.clone().requires_grad_(True), b0.clone().requires_grad_(True)
    y = sa.skip_concat(a, b, halo)
    assert y.is_contiguous(memory_format=CL) and torch.equal(y, torch.cat([a0, b0], 1))
    if halo and n == 1:
        slab, h = y._sfh_slab
        assert h == halo and slab.shape[2] == sp[0] + 2 * halo and slab.is_contiguous(memory_format=CL)
        assert y.data_ptr() == slab[:, :, halo:].data_ptr()
        assert not slab[:, :, :halo].any() and not slab[:, :, -halo:].any()
    else:
        assert not hasattr(y, "_sfh_slab")
    y.backward(gy)
    assert torch.equal(a.grad, gy[:, :ca]) and torch.equal(b.grad, gy[:, ca:])
    assert a.grad.is_contiguous(memory_format=CL) and b.grad.is_contiguous(memory_format=CL)


def test_concat_gate(device):
    x = torch.randn(1, 16, 2, 3, 4, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    assert sa.is_supported_concat(x, x)
    assert not sa.is_supported_concat(x, x.float())                              # dtypes differ
    assert not sa.is_supported_concat(x, x[:, :, :1])                            # extents differ
    assert not sa.is_supported_concat(x[:, :4], x)                               # 4 bf16 channels: half a 16-byte piece
    assert not sa.is_supported_concat(x.cpu(), x.cpu())
    assert not sa.is_supported_concat(None, x)
    with pytest.raises(NotImplementedError):
        sa.skip_concat(x[:, :4], x)


def test_decoder_stage_with_the_fused_concat_matches_torch_cat(device):
    """Up = transposed conv -> concat -> DoubleConv in the depth-shard form: the slab path (concat and first GroupNorm
    writing into the slabs the convolutions read) against the same modules fed by torch.cat and explicit assembly."""
    from scaffold_amd.unet import Up

    torch.manual_seed(3)
    up = Up(64, 32, 8).to(device).to(torch.bfloat16).to(memory_format=CL)
    for m in up.modules():
        if isinstance(m, sa.FastConv3d):
            m.shard_halo = True
    x1 = torch.randn(1, 64, 4, 4, 8, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    x2 = torch.randn(1, 32, 8, 8, 16, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn(1, 32, 8, 8, 16, device=device).to(torch.bfloat16).contiguous(memory_format=CL)

    def run(fused):
        up.conv.double_conv[1].out_halo = 1 if fused else 0
        a, b = x1.clone().requires_grad_(True), x2.clone().requires_grad_(True)
        up.zero_grad(set_to_none=True)
        y = up(a, b) if fused else up.conv(torch.cat([b, up.up(a)], dim=1))
        y.backward(gy)
        return [y.detach(), a.grad, b.grad] + [p.grad.clone() for p in up.parameters()]

    assert all(torch.equal(p, q) for p, q in zip(run(True), run(False)))
