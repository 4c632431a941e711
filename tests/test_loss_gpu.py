"""GPU parity of the fused cross-entropy + soft-Dice loss head against the oracle (fp64 torch restatement of
``ScaFFold/utils/trainer.py:634-663``), through the C ABI."""

import pytest
import torch

import scaffold_amd as sa
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d


def reference(logits, labels, cw, grad=True):
    x = logits.detach().cpu().double().requires_grad_(grad)
    w = None if cw is None else cw.detach().cpu().double()
    loss = orc.train_step_loss(x, labels.cpu(), logits.shape[1], class_weight=w, dtype=torch.float64)
    if not grad:
        return loss, None
    (g,) = torch.autograd.grad(loss, x)
    return loss.detach(), g


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 11, 6, 9, 13), (2, 11, 4, 5, 70), (1, 2, 3, 3, 3), (3, 17, 2, 8, 9), (1, 32, 5, 5, 5),
                                   (2, 11, 3, 3, 3)])  # the last: samples that do not start on 16-byte boundaries
def test_loss_and_gradient_match_oracle(device, dtype, shape, weighted):
    g = torch.Generator().manual_seed(31)
    n, c = shape[:2]
    logits = (torch.randn(shape, generator=g) * 3).to(dtype).contiguous(memory_format=CL)
    labels = torch.randint(0, c, (n, *shape[2:]), generator=g)
    labels[:, 0, 0, :2] = 0  # some background
    cw = (0.5 + torch.rand(c, generator=g)) if weighted else None
    ref_loss, ref_grad = reference(logits, labels, cw)
    x = logits.to(device).requires_grad_(True)
    loss = sa.ce_dice_loss(x, labels.to(device), None if cw is None else cw.to(device))
    assert loss.dtype is torch.float32 and loss.dim() == 0
    assert abs(loss.item() - ref_loss.item()) <= 2e-5 * max(1.0, abs(ref_loss.item()))
    (grad,) = torch.autograd.grad(loss * 2.5, x)  # an upstream factor must scale the gradient
    assert grad.dtype is dtype and grad.shape == x.shape
    err = (grad.cpu().double() / 2.5 - ref_grad).abs().max().item()
    scale = ref_grad.abs().max().item()
    tol = {torch.float32: 2e-5, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]  # one rounding of the gradient
    assert err <= tol * scale, (err, scale)


def test_matches_the_torch_recipe_on_device(device):
    """The same recipe built from torch ops on the GPU (what the reference runs) agrees to fp32 rounding."""
    g = torch.Generator().manual_seed(5)
    logits = torch.randn((1, 11, 8, 16, 16), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    labels = torch.randint(0, 11, (1, 8, 16, 16), generator=g).to(device)
    a = logits.clone().requires_grad_(True)
    b = logits.clone().requires_grad_(True)
    la = sa.ce_dice_loss(a, labels)
    lb = orc.train_step_loss(b, labels, 11)
    assert abs(la.item() - lb.item()) <= 1e-5 * abs(lb.item())
    la.backward()
    lb.backward()
    assert (a.grad.float() - b.grad.float()).abs().max() <= 1e-2 * b.grad.float().abs().max()


def test_extreme_logits_and_ignored_labels(device):
    """A huge margin must not overflow (max-subtracted softmax); out-of-range labels contribute nothing."""
    logits = torch.zeros((1, 3, 1, 2, 2), dtype=torch.float32)
    logits[0, 0] = 80.0
    logits[0, 1] = -80.0
    labels = torch.tensor([[[[0, 1], [2, 0]]]])
    ref, _ = reference(logits, labels, None, grad=False)
    got = sa.ce_dice_loss(logits.to(device).contiguous(memory_format=CL), labels.to(device))
    assert torch.isfinite(got) and abs(got.item() - ref.item()) <= 1e-4 * abs(ref.item())
    bad = labels.clone()
    bad[0, 0, 0, 0] = -100
    x = logits.to(device).contiguous(memory_format=CL).requires_grad_(True)
    loss = sa.ce_dice_loss(x, bad.to(device))
    loss.backward()
    assert torch.isfinite(loss) and torch.isfinite(x.grad).all()


def test_gate_and_determinism(device):
    g = torch.Generator().manual_seed(2)
    logits = torch.randn((1, 11, 4, 8, 8), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    labels = torch.randint(0, 11, (1, 4, 8, 8), generator=g).to(device)
    assert sa.is_supported_loss(logits, labels)
    assert not sa.is_supported_loss(logits.cpu(), labels.cpu())
    assert not sa.is_supported_loss(logits, labels.int())
    assert not sa.is_supported_loss(logits[:, :1], labels)
    with pytest.raises(NotImplementedError):
        sa.ce_dice_loss(logits, labels.int())
    outs = []
    for _ in range(3):
        junk = torch.full((1 << 20,), float("nan"), device=device)
        del junk
        x = logits.clone().requires_grad_(True)
        loss = sa.ce_dice_loss(x, labels)
        loss.backward()
        outs.append((loss.clone(), x.grad.clone()))
    for l, gr in outs[1:]:
        assert torch.equal(l, outs[0][0]) and torch.equal(gr, outs[0][1])
    with pytest.raises(RuntimeError):
        x = logits.clone().requires_grad_(True)
        loss = sa.ce_dice_loss(x, labels)
        (g1,) = torch.autograd.grad(loss, x, create_graph=True)
        g1.sum().backward()
