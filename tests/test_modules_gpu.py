"""GPU parity at the module / network level, and of the kernels against the committed golden vectors.

Mirrors the reference's module-level tests: all three directions through autograd against the stock op
(``tests/test_conv3d.py:1170-1217``), autocast dtypes (``:1248-1284``), second-order differentiation raising
(``:1733-1739``), and whole-network gradients with the two-arm structure of ``tests/test_groupnorm.py:1174-1228``
(fp32: per-parameter relative L2 < 1e-4; bf16 autocast: relative L2 of the concatenated gradient < 5e-2)."""

import os

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import scaffold_amd as sa
from oracle import oracle as orc
from scaffold_amd.modules import FastConv3d, FastConvTranspose3d, FastGroupNorm
from scaffold_amd.unet import UNet

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "hotpath_small.npz"))


def g(name, device, dtype=torch.float32):
    t = torch.from_numpy(GOLD[name]).to(dtype)
    return (t.contiguous(memory_format=CL) if t.dim() == 5 else t).to(device)


def test_kernels_reproduce_the_golden_vectors(device):
    """Small-integer problems: fp32 results must equal the committed brute-force answers exactly."""
    x, w, b, gy = (g(k, device) for k in ("conv_x", "conv_w", "conv_b", "conv_gy"))
    assert torch.equal(sa.conv3d_forward(x, w, b, 1, (0, 1, 1)).cpu().double(), torch.from_numpy(GOLD["conv_y"]))
    assert torch.equal(sa.conv3d_backward_data(gy, w, x.shape, 1, (0, 1, 1)).cpu().double(), torch.from_numpy(GOLD["conv_gx"]))
    assert torch.equal(sa.conv3d_backward_weight(x, w.shape, gy, 1, (0, 1, 1)).cpu().double(), torch.from_numpy(GOLD["conv_gw"]))
    x2, w2, gy2 = g("sconv_x", device), g("sconv_w", device), g("sconv_gy", device)
    assert torch.equal(sa.conv3d_forward(x2, w2, None, (2, 1, 3), (1, 0, 2), (1, 2, 1)).cpu().double(), torch.from_numpy(GOLD["sconv_y"]))
    assert torch.equal(sa.conv3d_backward_weight(x2, w2.shape, gy2, (2, 1, 3), (1, 0, 2), (1, 2, 1)).cpu().double(),
                       torch.from_numpy(GOLD["sconv_gw"]))
    xt, wt, bt = g("convt_x", device), g("convt_w", device), g("convt_b", device)
    assert torch.equal(sa.conv_transpose3d_forward(xt, wt, bt, 2).cpu().double(), torch.from_numpy(GOLD["convt_y"]))
    xg, gamma, beta, dy = g("gn_x", device), g("gn_gamma", device), g("gn_beta", device), g("gn_dy", device)
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(xg, 4, gamma, beta, 1e-5, "relu", None)
    dx, dgamma, dbeta = torch.ops.scaffold_gn.group_norm_backward(dy, xg, gamma, beta, mean, rstd, 4, "relu")
    for got, name in ((out, "gn_y"), (mean, "gn_mean"), (rstd, "gn_rstd"), (dx, "gn_dx"), (dgamma, "gn_dgamma"), (dbeta, "gn_dbeta")):
        assert orc.gn_rel_error(got, torch.from_numpy(GOLD[name])) <= 1e-5, name


def _grads(module, x, gy):
    x = x.clone().requires_grad_(True)
    y = module(x)
    y.backward(gy)
    return y.detach(), x.grad, {k: p.grad for k, p in module.named_parameters()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fastconv3d_matches_stock_in_all_directions(device, dtype):
    torch.manual_seed(0)
    stock = nn.Conv3d(32, 64, 3, padding=1, bias=True).double()
    fast = FastConv3d(32, 64, 3, padding=1, bias=True).to(device).to(dtype).to(memory_format=CL)
    fast.load_state_dict({k: v.to(dtype) for k, v in stock.state_dict().items()})
    stock.load_state_dict({k: v.double() for k, v in fast.state_dict().items()})  # identical (rounded) parameters
    x = torch.randn(2, 32, 6, 10, 12).to(dtype)
    gy = torch.randn(2, 64, 6, 10, 12).to(dtype)
    y0, gx0, gp0 = _grads(stock, x.double(), gy.double())
    y1, gx1, gp1 = _grads(fast, x.to(device).contiguous(memory_format=CL), gy.to(device).contiguous(memory_format=CL))
    prob = orc.ConvProblem(n=2, cin=32, cout=64, spatial=(6, 10, 12), bias=True, dtype=dtype)
    orc.assert_close(y1, y0, prob, "fwd")
    orc.assert_close(gx1, gx0, prob, "bwd-data")
    orc.assert_close(gp1["weight"], gp0["weight"], prob, "bwd-weight")
    assert orc.gn_rel_error(gp1["bias"], gp0["bias"]) <= (1e-5 if dtype is torch.float32 else 2e-2)   # gy.sum((0,2,3,4))
    assert y1.dtype is dtype and gx1.dtype is dtype and gp1["weight"].dtype is dtype and y1.is_contiguous(memory_format=CL)


@pytest.mark.parametrize("cin,cout,spatial", [(32, 32, (16, 32, 32)), (64, 64, (8, 16, 32))])
def test_no_worse_than_the_incumbent_in_all_directions(device, cin, cout, spatial):
    """The reference's module-level standard (tests/test_conv3d.py:1170-1217, triton_conv3d/reference.py:241-261): the
    error against fp64 may not exceed max(error_bound, 4 x the incumbent's error), the incumbent being the stock module
    on the same GPU (MIOpen) with the same rounded parameters and inputs, in all three directions."""
    torch.manual_seed(12)
    dtype = torch.bfloat16
    truth = nn.Conv3d(cin, cout, 3, padding=1, bias=True).double()
    fast = FastConv3d(cin, cout, 3, padding=1, bias=True).to(device).to(dtype).to(memory_format=CL)
    fast.load_state_dict({k: v.to(dtype) for k, v in truth.state_dict().items()})
    truth.load_state_dict({k: v.double() for k, v in fast.state_dict().items()})
    incumbent = nn.Conv3d(cin, cout, 3, padding=1, bias=True).to(device).to(dtype).to(memory_format=CL)
    incumbent.load_state_dict(fast.state_dict())
    x = torch.randn(1, cin, *spatial).to(dtype)
    gy = torch.randn(1, cout, *spatial).to(dtype)
    xd, gyd = x.to(device).contiguous(memory_format=CL), gy.to(device).contiguous(memory_format=CL)
    y0, gx0, gp0 = _grads(truth, x.double(), gy.double())
    y1, gx1, gp1 = _grads(fast, xd, gyd)
    y2, gx2, gp2 = _grads(incumbent, xd, gyd)
    prob = orc.ConvProblem(n=1, cin=cin, cout=cout, spatial=spatial, bias=True, dtype=dtype)
    for direction, ours, theirs, ref in (("fwd", y1, y2, y0), ("bwd-data", gx1, gx2, gx0),
                                         ("bwd-weight", gp1["weight"], gp2["weight"], gp0["weight"])):
        stock_error = orc.compare(theirs, ref)
        orc.assert_close(ours, ref, prob, direction, incumbent_error=stock_error)
        # and without the incumbent's allowance: ours holds the bound on its own account
        orc.assert_close(ours, ref, prob, direction)


def test_autocast_casts_outside_the_node_and_returns_fp32_parameter_grads(device):
    fast = FastConv3d(32, 32, 3, padding=1, bias=False).to(device).to(memory_format=CL)
    up = FastConvTranspose3d(32, 32, 2, stride=2).to(device).to(memory_format=CL)
    gn = FastGroupNorm(8, 32, activation="relu").to(device)
    x = torch.randn(1, 32, 4, 8, 8, device=device).contiguous(memory_format=CL).requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        h = fast(x)
        assert h.dtype is torch.bfloat16
        h = gn(h)
        assert h.dtype is torch.bfloat16           # the input's dtype, not autocast's fp32 policy
        y = up(h)
        assert y.dtype is torch.bfloat16 and y.shape == (1, 32, 8, 16, 16)
    y.float().sum().backward()
    assert x.grad.dtype is torch.float32 and fast.weight.grad.dtype is torch.float32
    assert up.weight.grad.dtype is torch.float32 and up.bias.grad.dtype is torch.float32 and gn.weight.grad.dtype is torch.float32
    # outside autocast an fp32 model computes in fp32
    assert fast(x.detach()).dtype is torch.float32


def test_second_order_differentiation_raises(device):
    fast = FastConv3d(8, 8, 3, padding=1).to(device)
    x = torch.randn(1, 8, 4, 4, 4, device=device).requires_grad_(True)
    (gx,) = torch.autograd.grad(fast(x).sum(), x, create_graph=True)
    with pytest.raises(RuntimeError):
        gx.sum().backward()
    with torch.no_grad():
        assert fast(x).shape == (1, 8, 4, 4, 4)
    with torch.inference_mode():
        assert fast(x).shape == (1, 8, 4, 4, 4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transposed_module_matches_stock(device, dtype):
    torch.manual_seed(1)
    stock = nn.ConvTranspose3d(64, 32, 2, stride=2).double()
    fast = FastConvTranspose3d(64, 32, 2, stride=2).to(device).to(dtype).to(memory_format=CL)
    fast.load_state_dict({k: v.to(dtype) for k, v in stock.state_dict().items()})
    stock.load_state_dict({k: v.double() for k, v in fast.state_dict().items()})
    x = torch.randn(1, 64, 4, 5, 6).to(dtype)
    gy = torch.randn(1, 32, 8, 10, 12).to(dtype)
    y0, gx0, gp0 = _grads(stock, x.double(), gy.double())
    y1, gx1, gp1 = _grads(fast, x.to(device).contiguous(memory_format=CL), gy.to(device).contiguous(memory_format=CL))
    tol = 1e-5 if dtype is torch.float32 else 2e-2
    for a, b in ((y1, y0), (gx1, gx0), (gp1["weight"], gp0["weight"]), (gp1["bias"], gp0["bias"])):
        assert orc.gn_rel_error(a, b) <= tol
    assert gp1["weight"].shape == (64, 32, 2, 2, 2)


def _two_arms(device, dtype_autocast, layers=2, base=32, size=(16, 16, 32), shard=False):
    torch.manual_seed(7)
    stock = UNet(1, 5, layers=layers, base_width=base, stock=True)
    ours = UNet(1, 5, layers=layers, base_width=base).to(device).to(memory_format=CL)
    ours.load_state_dict(stock.state_dict())
    if shard:
        ours.set_shard_halo(True)
    g0 = torch.Generator().manual_seed(8)
    x = (torch.rand((1, 1, *size), generator=g0) < 0.05).float()
    lab = torch.randint(0, 5, (1, *size), generator=g0)
    return stock, ours, x, lab


def _step(model, x, lab, autocast_device=None):
    if autocast_device is None:
        logits = model(x)
    else:
        with torch.autocast(autocast_device, dtype=torch.bfloat16):
            logits = model(x)
    loss = orc.train_step_loss(logits, lab, 5)
    loss.backward()
    return loss.detach(), logits.detach()


def test_unet_fp32_gradients_match_stock_per_parameter(device):
    stock, ours, x, lab = _two_arms(device, None)
    stock = stock.double()
    l0, y0 = _step(stock, x.double(), lab)
    l1, y1 = _step(ours, x.to(device).contiguous(memory_format=CL), lab.to(device))
    assert abs(l0.item() - l1.item()) <= 1e-5 * abs(l0.item())
    assert orc.gn_rel_error(y1, y0) <= 1e-4
    worst = 0.0
    for (k, p0), (_, p1) in zip(stock.named_parameters(), ours.named_parameters()):
        rel = (p1.grad.cpu().double() - p0.grad).norm() / p0.grad.norm().clamp_min(1e-30)
        worst = max(worst, rel.item())
        assert rel < 1e-4, (k, rel.item())


def test_unet_bf16_autocast_train_step_matches_stock(device):
    """Config 5 in small: bf16 autocast, fp32 master weights, CE + Dice, clip 1.0, one Adam step; our arm on the
    GPU against the stock-module arm on the host cores."""
    stock, ours, x, lab = _two_arms(device, torch.bfloat16)
    opt0 = torch.optim.Adam(stock.parameters(), lr=1e-3)
    opt1 = torch.optim.Adam(ours.parameters(), lr=1e-3)
    l0, _ = _step(stock, x, lab, "cpu")
    l1, _ = _step(ours, x.to(device).contiguous(memory_format=CL), lab.to(device), "cuda")
    assert abs(l0.item() - l1.item()) <= 2e-2 * abs(l0.item())
    g0 = torch.cat([p.grad.flatten().double() for p in stock.parameters()])
    g1 = torch.cat([p.grad.flatten().cpu().double() for p in ours.parameters()])
    assert all(p.grad.dtype is torch.float32 for p in ours.parameters())
    assert ((g1 - g0).norm() / g0.norm()).item() < 5e-2
    init = torch.cat([p.detach().flatten().double() for p in stock.parameters()])
    for m, o in ((stock, opt0), (ours, opt1)):
        torch.nn.utils.clip_grad_norm_(m.parameters(), 1.0)
        o.step()
    w0 = torch.cat([p.detach().flatten().double() for p in stock.parameters()])
    w1 = torch.cat([p.detach().flatten().cpu().double() for p in ours.parameters()])
    # Adam's first update is lr * sign(g): it amplifies the sign of gradients that are noise in bf16, so the
    # bounded quantities are the step size and the agreement of the two update directions, not w itself.
    u0, u1 = w0 - init, w1 - init
    assert u0.abs().max() <= 1.001e-3 and u1.abs().max() <= 1.001e-3
    assert (torch.dot(u0, u1) / (u0.norm() * u1.norm())).item() > 0.9


# ---- config 5's architecture: 5 levels, base width 32 doubling to 512, 11 classes, depth-shard form ------------------
def _cfg5_arms(device, grid, iterations):
    """Stock-module arm on the host and ours on the GPU in shard form (zero depth halo, padding (0, 1, 1)), the same seeded
    weights; input = the first half along depth of an IFS sample (occupancy in, class ids 0..10 as labels)."""
    torch.manual_seed(5001)
    stock = UNet(1, 11, layers=4, base_width=32, stock=True)
    ours = UNet(1, 11, layers=4, base_width=32).to(device).to(memory_format=CL).set_shard_halo(True)
    ours.load_state_dict(stock.state_dict())
    occ, lab = orc.ifs_volume(grid, iterations=iterations, seed=5000)
    x, lab = occ[:, :, : grid // 2].contiguous(), lab[:, : grid // 2].contiguous()
    assert 0.01 < x.mean() < 0.5 and lab.unique().numel() >= 3
    return stock, ours, x, lab


def test_cfg5_architecture_fp32_gradients_match_stock_per_parameter(device):
    """The reference's fp32 arm (`tests/test_groupnorm.py:1174-1228`: worst per-parameter relative L2 < 1e-4) on the
    5-level / 11-class network: every kernel family of the step chained at widths 32..512, fp64 stock modules as truth,
    the fused loss head against the loss recipe."""
    stock, ours, x, lab = _cfg5_arms(device, 32, 20000)
    assert sum(isinstance(m, FastConv3d) for m in ours.modules()) == 19 and sum(isinstance(m, FastGroupNorm) for m in ours.modules()) == 18
    stock = stock.double()
    l0 = orc.train_step_loss(stock(x.double()), lab, 11, dtype=torch.float64)
    l0.backward()
    l1 = sa.ce_dice_loss(ours(x.to(device).contiguous(memory_format=CL)), lab.to(device))
    l1.backward()
    assert abs(l0.item() - l1.item()) <= 1e-5 * abs(l0.item())
    for (k, p0), (_, p1) in zip(stock.named_parameters(), ours.named_parameters()):
        rel = (p1.grad.cpu().double() - p0.grad).norm() / p0.grad.norm().clamp_min(1e-30)
        assert rel < 1e-4, (k, rel.item())


@pytest.mark.parametrize("grid,iterations", [(32, 20000), (64, 60000)])
def test_cfg5_architecture_bf16_train_step_matches_stock(device, grid, iterations):
    """The reference's bf16 arm (aggregate relative L2 of the concatenated gradient < 5e-2) plus the loss within 2e-2 and the
    clipped Adam step, for the step exactly as the bench runs it: bf16 autocast over fp32 master weights, every convolution
    reading a depth slab, fused CE + Dice, `FusedClipAdam` with bf16 shadow weights.  Truth is the stock-module arm in
    fp32 on the host (no autocast), with `clip_grad_norm_(1.0)` + `torch.optim.Adam` (`ScaFFold/utils/trainer.py:640-694`)."""
    stock, ours, x, lab = _cfg5_arms(device, grid, iterations)
    opt0 = torch.optim.Adam(stock.parameters(), lr=1e-3)
    opt1 = sa.FusedClipAdam(ours.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
    l0 = orc.train_step_loss(stock(x), lab, 11)
    l0.backward()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        logits = ours(x.to(device).contiguous(memory_format=CL))
    assert logits.dtype is torch.bfloat16 and logits.shape == (1, 11, grid // 2, grid, grid)
    l1 = sa.ce_dice_loss(logits, lab.to(device))
    l1.backward()
    assert abs(l0.item() - l1.item()) <= 2e-2 * abs(l0.item()), (l0.item(), l1.item())
    assert all(p.grad.dtype is torch.float32 for p in ours.parameters())
    g0 = torch.cat([p.grad.flatten().double() for p in stock.parameters()])
    g1 = torch.cat([p.grad.flatten().cpu().double() for p in ours.parameters()])
    assert ((g1 - g0).norm() / g0.norm()).item() < 5e-2
    init = torch.cat([p.detach().flatten().double() for p in stock.parameters()])
    want_norm = torch.nn.utils.clip_grad_norm_(stock.parameters(), 1.0)
    opt0.step()
    opt1.step()
    assert abs(opt1.grad_norm.item() - want_norm.item()) <= 5e-2 * want_norm.item()
    u0 = torch.cat([p.detach().flatten().double() for p in stock.parameters()]) - init
    u1 = torch.cat([p.detach().flatten().cpu().double() for p in ours.parameters()]) - init
    # Adam's first update is lr * sign(g) (amplifying the sign of gradients that are noise in bf16): bounded are the step
    # size and the agreement of the two update directions
    assert u0.abs().max() <= 1.001e-3 and u1.abs().max() <= 1.001e-3
    assert (torch.dot(u0, u1) / (u0.norm() * u1.norm())).item() > 0.9
    # the bf16 copies the next step's convolutions read are the rounded new weights
    for p in ours.parameters():
        assert torch.equal(opt1.shadow[p], p.detach().to(torch.bfloat16))


def test_shard_halo_form_is_bitwise_the_padded_form(device):
    """Zero depth halo + depth padding 0 (what a single DistConv shard computes) equals padding 1."""
    _, ours, x, _ = _two_arms(device, torch.bfloat16)
    xd = x.to(device).contiguous(memory_format=CL)
    with torch.autocast("cuda", dtype=torch.bfloat16), torch.no_grad():
        y_pad = ours(xd)
        ours.set_shard_halo(True)
        y_halo = ours(xd)
    assert torch.equal(y_pad, y_halo)


def test_up_equals_explicit_cat(device):
    from scaffold_amd.unet import Up

    torch.manual_seed(3)
    up = Up(64, 32, 8).to(device).to(memory_format=CL)
    x1 = torch.randn(1, 64, 4, 4, 8, device=device).contiguous(memory_format=CL)
    x2 = torch.randn(1, 32, 8, 8, 16, device=device).contiguous(memory_format=CL)
    want = up.conv(torch.cat([x2, up.up(x1)], dim=1))
    assert torch.equal(up(x1, x2), want)


def test_train_step_as_a_hip_graph_replays_to_the_eager_result(device):
    """The whole step (forward, fused loss, backward, clipping, Adam) captured once and replayed: every replay, with
    eager work and synchronisations between replays, must give the loss the eager step gives from the same state."""
    def make():
        _, ours, x, lab = _two_arms(device, torch.bfloat16, shard=True)
        opt = torch.optim.Adam(ours.parameters(), lr=1e-3, fused=True, capturable=True)
        xd, labd = x.to(device).contiguous(memory_format=CL), lab.to(device)

        def step():
            with torch.autocast("cuda", dtype=torch.bfloat16):
                logits = ours(xd)
            loss = sa.ce_dice_loss(logits, labd)
            loss.backward()
            torch.nn.utils.clip_grad_norm_(ours.parameters(), 1.0)
            opt.step()
            opt.zero_grad(set_to_none=True)
            return loss.detach()
        return ours, opt, step

    _, _, eager = make()
    want = [eager().item() for _ in range(4)]
    model, opt, step = make()
    init = {k: v.clone() for k, v in model.state_dict().items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    model.load_state_dict(init)
    for st in opt.state.values():
        for v in st.values():
            if torch.is_tensor(v):
                v.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_loss = step()
    got = []
    for _ in range(4):
        graph.replay()
        torch.cuda.synchronize()
        got.append(static_loss.item())
        torch.randn(1 << 16, device=device).sum().item()
    assert got == want
    assert want[0] != want[1]


def test_packing_the_weight_once_per_step_changes_no_bits(device):
    import scaffold_amd.modules as mods

    def grads(flag):
        mods.PACK_WEIGHTS_ONCE = flag
        try:
            _, ours, x, lab = _two_arms(device, torch.bfloat16, shard=True)
            _step(ours, x.to(device).contiguous(memory_format=CL), lab.to(device), "cuda")
            return [p.grad.clone() for p in ours.parameters()]
        finally:
            mods.PACK_WEIGHTS_ONCE = False

    a, b = grads(False), grads(True)
    assert all(torch.equal(p, q) for p, q in zip(a, b))


def _fused_adam_run(device, steps):
    _, ours, x, lab = _two_arms(device, torch.bfloat16, shard=True)
    opt = sa.FusedClipAdam(ours.parameters(), lr=1e-2, max_norm=1.0, shadow_dtype=torch.bfloat16)
    xd, labd = x.to(device).contiguous(memory_format=CL), lab.to(device)
    losses = []
    for _ in range(steps):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = ours(xd)
        loss = sa.ce_dice_loss(logits, labd)
        loss.backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
        losses.append(loss.item())
    return ours, losses


def test_packed_weights_kept_by_the_optimizer_change_no_bits(device, monkeypatch):
    """FusedClipAdam repacks the convolution weights inside its step and the modules then launch no packing of their
    own: the run must equal, bit for bit, one in which every call packs for itself."""
    import scaffold_amd.modules as mods
    kept, a = _fused_adam_run(device, 4)
    entries = [e for p in kept.parameters() for e in getattr(p, "_sfh_packs", {}).values() if e]
    assert entries and all(e.maintained for e in entries)
    assert all(e.version == p._version for p in kept.parameters() for e in getattr(p, "_sfh_packs", {}).values() if e)
    monkeypatch.setattr(mods, "_current_packs", lambda *args, **kwargs: None)
    plain, b = _fused_adam_run(device, 4)
    assert not any(hasattr(p, "_sfh_packs") for p in plain.parameters())
    assert a == b and a[0] != a[-1]
    assert all(torch.equal(p, q) for p, q in zip(kept.parameters(), plain.parameters()))


def test_kept_packed_weights_are_not_trusted_after_a_foreign_write(device):
    torch.manual_seed(3)
    conv = sa.FastConv3d(32, 32, 3, padding=1, bias=False).to(device).to(memory_format=CL)
    opt = sa.FusedClipAdam(conv.parameters(), lr=1e-2, shadow_dtype=torch.bfloat16)
    x = torch.randn(1, 32, 8, 16, 16, device=device).to(torch.bfloat16).contiguous(memory_format=CL).requires_grad_()
    for _ in range(2):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = conv(x)
        y.float().square().mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
    (entry,) = conv.weight._sfh_packs.values()
    assert entry.maintained and entry.version == conv.weight._version
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(conv(x), sa.conv3d_forward(x.detach(), conv.weight.detach().to(torch.bfloat16), None, 1, 1, 1))
    with torch.no_grad():
        conv.weight.mul_(-0.5)                    # not the optimizer: the copies and packed forms are stale now
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = conv(x)                               # the per-call cast path
    want = sa.conv3d_forward(x.detach(), conv.weight.detach().to(torch.bfloat16), None, 1, 1, 1)
    assert torch.equal(y, want)
    opt.refresh_shadows()                         # the copies are current again, the packed forms are repacked on use
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = conv(x)
    assert torch.equal(y, want)
    x.grad = None
    y.float().sum().backward()
    assert torch.equal(x.grad, sa.conv3d_backward_data(torch.ones_like(want), conv.weight.detach().to(torch.bfloat16), x.shape, 1, 1, 1))


def test_conv_reading_the_producers_slab_is_bitwise_the_assembled_form(device):
    """GroupNorm -> FastConv3d(shard_halo): with ``out_halo`` the norm writes into the slab the convolution reads; the
    result and every gradient equal the form that assembles the slab with a copy."""
    torch.manual_seed(11)
    x0 = torch.randn(1, 32, 6, 12, 20, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn(1, 64, 6, 12, 20, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    results = []
    for out_halo in (0, 1):
        torch.manual_seed(12)
        norm = FastGroupNorm(8, 32, activation="relu").to(device).to(torch.bfloat16)
        conv = FastConv3d(32, 64, 3, padding=1, bias=False).to(device).to(torch.bfloat16).to(memory_format=CL)
        conv.shard_halo = True
        norm.out_halo = out_halo
        x = x0.clone().requires_grad_(True)
        h = norm(x)
        assert hasattr(h, "_sfh_slab") == bool(out_halo)
        y = conv(h)
        y.backward(gy)
        results.append((y.detach(), x.grad, conv.weight.grad, norm.weight.grad, norm.bias.grad))
    assert all(torch.equal(a, b) for a, b in zip(*results))


@pytest.mark.parametrize("batch,size,checkpoint", [(1, (12, 20, 36), False), (2, (8, 12, 20), False), (1, (8, 16, 32), True)])
def test_shard_form_gradients_equal_the_padded_form(device, batch, size, checkpoint):
    """Every route of the depth-shard form -- slabs written by GroupNorm and by the fused concat (one sample), assembled
    slabs (a batch), sizes that make the decoder pad, activation checkpointing -- gives the padded form's loss and
    parameter gradients bit for bit."""
    torch.manual_seed(5)
    model = UNet(1, 5, layers=2, base_width=32).to(device).to(memory_format=CL)
    if checkpoint:
        model.use_checkpointing()
    g0 = torch.Generator().manual_seed(6)
    x = (torch.rand((batch, 1, *size), generator=g0) < 0.1).float().contiguous(memory_format=CL).to(device)
    lab = torch.randint(0, 5, (batch, *size), generator=g0).to(device)

    def grads(shard):
        model.set_shard_halo(shard)
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = model(x)
        loss = sa.ce_dice_loss(logits, lab)
        loss.backward()
        return [loss.detach().clone()] + [p.grad.clone() for p in model.parameters()]

    a, b = grads(False), grads(True)
    assert all(torch.equal(p, q) for p, q in zip(a, b))


@pytest.mark.parametrize("layers,base,size,shard,batch", [
    (3, 32, (16, 32, 64), False, 1),   # brick forward at every level, persist / brick data gradients, the deepest level sliced
    (3, 32, (16, 32, 64), True, 1),    # the same on a depth shard: every source lies in a slab its producer wrote
    (2, 32, (8, 12, 24), False, 2),    # a batch
    (2, 32, (8, 12, 24), True, 2),     # a batch on a shard: no slabs, so the decoder concatenates into one
    (1, 64, (32, 64, 64), True, 1),    # 128 -> 64 at 32 x 64 x 64: the wide-tile forward reads the pair
    (2, 32, (10, 12, 20), False, 1),   # an odd level: the upsampled tensor is padded (unet_parts.py:212-223) before it is read
    (2, 32, (10, 12, 20), True, 1),    # ... on a shard the padded tensor lies in no slab: that stage concatenates
])
def test_decoder_reading_the_skip_in_place_changes_no_bits(device, monkeypatch, layers, base, size, shard, batch):
    """The decoder's first convolution reads [skip, upsampled] as two tensors instead of their concatenation
    (``unet_parts.py:107-120``): loss and every parameter gradient are the bits of the concatenating form."""
    from scaffold_amd import conv3d as c3
    from scaffold_amd.unet import Up

    torch.manual_seed(21)
    model = UNet(1, 5, layers=layers, base_width=base).to(device).to(memory_format=CL).set_shard_halo(shard)
    g0 = torch.Generator().manual_seed(22)
    x = (torch.rand((batch, 1, *size), generator=g0) < 0.1).float().contiguous(memory_format=CL).to(device)
    lab = torch.randint(0, 5, (batch, *size), generator=g0).to(device)
    calls = []
    real = c3.conv3d_forward_pair
    monkeypatch.setattr(c3, "conv3d_forward_pair", lambda *a, **k: (calls.append(1), real(*a, **k))[1])

    def grads(in_place):
        monkeypatch.setattr(Up, "read_skip_in_place", in_place)
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = model(x)
        loss = sa.ce_dice_loss(logits, lab)
        loss.backward()
        return [loss.detach().clone(), logits.detach().clone()] + [p.grad.clone() for p in model.parameters()]

    want = grads(False)
    assert not calls
    got = grads(True)
    padded_stages = sum(1 for i in range(1, layers + 1) if any((v >> (i - 1)) % 2 for v in size))  # levels with an odd extent
    assert len(calls) == (0 if (shard and batch > 1) else layers - (padded_stages if shard else 0))
    assert all(torch.equal(p, q) for p, q in zip(want, got))


def test_up_convolution_into_a_depth_slab_is_bitwise_the_plain_output(device):
    """``FastConvTranspose3d.out_halo``: the result lies in the interior of a slab with zero faces and is otherwise the
    plain result, values and gradients."""
    torch.manual_seed(31)
    x0 = torch.randn(1, 64, 3, 5, 9, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn(1, 32, 6, 10, 18, device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    results = []
    for halo in (0, 1, 2):
        torch.manual_seed(32)
        up = FastConvTranspose3d(64, 32, kernel_size=2, stride=2).to(device).to(torch.bfloat16)
        up.out_halo = halo
        x = x0.clone().requires_grad_(True)
        y = up(x)
        assert hasattr(y, "_sfh_slab") == bool(halo) and y.is_contiguous(memory_format=CL)
        if halo:
            slab, h = y._sfh_slab
            assert h == halo and slab.shape == (1, 32, 6 + 2 * halo, 10, 18) and slab.data_ptr() < y.data_ptr()
            assert torch.equal(slab[:, :, halo:halo + 6], y)
            assert not slab[:, :, :halo].any() and not slab[:, :, halo + 6:].any()
        y.backward(gy)
        results.append((y.detach().clone(), x.grad, up.weight.grad, up.bias.grad))
    for other in results[1:]:
        assert all(torch.equal(a, b) for a, b in zip(results[0], other))


def test_where_the_decoder_still_concatenates(device):
    """``FastConv3d.takes_pair`` says no -- and ``Up`` concatenates, with the concatenating form's result -- for fp32
    operands, a cut off the 32-channel grid, tensors outside their slabs on a depth shard, and other voxels."""
    from scaffold_amd.unet import Up

    torch.manual_seed(41)
    conv = FastConv3d(64, 32, 3, padding=1, bias=False).to(device).to(memory_format=CL)
    mk = lambda c, dtype=torch.bfloat16, sp=(4, 8, 32): torch.randn(1, c, *sp, device=device).to(dtype).contiguous(memory_format=CL)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert conv.takes_pair(mk(32), mk(32))
        assert not conv.takes_pair(mk(32, torch.float32), mk(32, torch.float32))  # autocast would cast: new tensors
        assert not conv.takes_pair(mk(32), mk(32, torch.float32))
        assert not conv.takes_pair(mk(16), mk(48))
        assert not conv.takes_pair(mk(32), mk(32, sp=(4, 8, 16)))
        assert not conv.takes_pair(mk(32), None)
        conv.shard_halo = True
        assert not conv.takes_pair(mk(32), mk(32))  # no producer wrote them into slabs
        with pytest.raises(NotImplementedError):
            conv(mk(32), mk(32))
        conv.shard_halo = False
    assert not conv.takes_pair(mk(32), mk(32))  # outside autocast the fp32 weight does not match bf16 tensors
    # Up with fp32 tensors: the concatenating form, same result as torch.cat by hand
    up = Up(64, 32, 8).to(device).to(memory_format=CL)
    x1 = torch.randn(1, 64, 4, 4, 8, device=device).contiguous(memory_format=CL)
    x2 = torch.randn(1, 32, 8, 8, 16, device=device).contiguous(memory_format=CL)
    assert torch.equal(up(x1, x2), up.conv(torch.cat([x2, up.up(x1)], dim=1)))


def test_from_shard_files_to_updated_weights(device, tmp_path):
    """The whole path on one rank's share: a volume / mask pair as the generator writes it (float32 (3, d, h, w) + uint16),
    read and ingested into the stem's slab, the 3-channel U-Net in shard form under bf16 autocast, the fused loss head and
    one clipped Adam step -- against stock modules in fp32 on the host, fed the reference's way
    (ScaFFold/utils/trainer.py:572-694)."""
    import numpy as np

    from scaffold_amd import shards

    size = (8, 16, 32)
    rng = np.random.default_rng(12)
    volume = (rng.random((3,) + size, dtype=np.float32) * (rng.random(size) < 0.1)).astype(np.float32)   # sparse, coloured
    mask = (rng.integers(1, 5, size=size) * (volume.sum(0) > 0)).astype(np.uint16)
    images, masks = tmp_path / "volumes", tmp_path / "masks"
    images.mkdir(), masks.mkdir()
    np.save(images / "0_shard000000.npy", volume)
    np.save(masks / "0_shard000000_mask.npy", mask)

    torch.manual_seed(9)
    stock = UNet(3, 5, layers=2, base_width=32, stock=True)
    ours = UNet(3, 5, layers=2, base_width=32).to(device).to(memory_format=CL)
    ours.load_state_dict(stock.state_dict())
    ours.set_shard_halo(True)
    init = torch.cat([p.detach().flatten().double() for p in stock.parameters()])

    # the reference's arm: host tensors, channels_last_3d float32 image, long mask, torch loss recipe, clip + Adam
    x0 = torch.from_numpy(volume)[None].contiguous(memory_format=CL)
    lab0 = torch.from_numpy(mask.astype(np.int16))[None].long()
    opt0 = torch.optim.Adam(stock.parameters(), lr=1e-3)
    l0, _ = _step(stock, x0, lab0)          # in fp32: the host's bf16 kernels are not the oracle here
    g0 = torch.cat([p.grad.flatten().double() for p in stock.parameters()])     # before the clipping scales them in place
    torch.nn.utils.clip_grad_norm_(stock.parameters(), 1.0)
    opt0.step()

    # this build's arm: files -> pinned staging -> one ingest kernel (bf16 slab + int64 labels) -> HIP ops
    reader = shards.ShardReader(images, masks, shard_id=0)
    x1, lab1 = reader.load("0", device, dtype=torch.bfloat16, out_halo=1)
    assert x1._sfh_slab[1] == 1 and torch.equal(lab1.cpu(), lab0)
    opt1 = sa.FusedClipAdam(ours.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        logits = ours(x1)
    l1 = sa.ce_dice_loss(logits, lab1)
    l1.backward()
    g1 = torch.cat([p.grad.flatten().cpu().double() for p in ours.parameters()])
    opt1.step()

    assert abs(l0.item() - l1.item()) <= 2e-2 * abs(l0.item())
    assert ((g1 - g0).norm() / g0.norm()).item() < 5e-2          # aggregate bf16 tolerance of the reference's own suite
    u0 = torch.cat([p.detach().flatten().double() for p in stock.parameters()]) - init
    u1 = torch.cat([p.detach().flatten().cpu().double() for p in ours.parameters()]) - init
    assert u0.abs().max() <= 1.001e-3 and u1.abs().max() <= 1.001e-3
    assert (torch.dot(u0, u1) / (u0.norm() * u1.norm())).item() > 0.9
