"""Fused gradient clipping + Adam against torch's own pair (clip_grad_norm_ + optim.Adam) on the same tensors:
parameters and moments within fp32 rounding of the stock single-tensor implementation after several steps."""

import copy

import pytest
import torch

import scaffold_amd as sa

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d

SIZES = [(32, 32, 3, 3, 3), (64,), (1,), (7, 5), (513,), (8192,), (8193,), (3, 16385), (11, 32, 1, 1, 1), (100000,)]


def _make(device, sizes=SIZES, seed=0, channels_last=True):
    g = torch.Generator().manual_seed(seed)
    ps = []
    for s in sizes:
        t = torch.randn(s, generator=g)
        if channels_last and len(s) == 5:
            t = t.contiguous(memory_format=CL)
        ps.append(t.to(device).requires_grad_(True))
    return ps


def _set_grads(params, step, scale):
    g = torch.Generator().manual_seed(1000 + step)
    for p in params:
        gr = (torch.randn(p.shape, generator=g) * scale).to(p.device)
        p.grad = gr.contiguous(memory_format=CL) if p.dim() == 5 and p.is_contiguous(memory_format=CL) else gr


def _run_pair(device, steps, max_norm, scale, **kw):
    ours, stock = _make(device), _make(device)
    opt_o = sa.FusedClipAdam(ours, max_norm=max_norm, **kw)
    opt_s = torch.optim.Adam(stock, foreach=False, fused=False, **kw)
    norms = []
    for step in range(steps):
        _set_grads(ours, step, scale)
        _set_grads(stock, step, scale)
        before = [p.grad.clone() for p in ours]
        opt_o.step()
        assert all(torch.equal(p.grad, b) for p, b in zip(ours, before)), "gradients must not be rewritten"
        want_norm = torch.nn.utils.clip_grad_norm_(stock, max_norm) if max_norm is not None else \
            torch.linalg.vector_norm(torch.stack([torch.linalg.vector_norm(p.grad) for p in stock]))
        opt_s.step()
        norms.append((opt_o.grad_norm.item(), want_norm.item()))
    return ours, stock, opt_o, opt_s, norms


@pytest.mark.parametrize("max_norm,scale", [(1.0, 1.0), (1.0, 1e-4), (None, 1.0), (0.05, 3.0)])
def test_matches_clip_grad_norm_plus_adam(device, max_norm, scale):
    ours, stock, opt_o, opt_s, norms = _run_pair(device, 5, max_norm, scale, lr=1e-2)
    for got, want in norms:
        assert abs(got - want) <= 1e-5 * want
    for p, q in zip(ours, stock):
        assert torch.allclose(p, q, rtol=1e-5, atol=1e-6), (p.shape, (p - q).abs().max().item())
        so, ss = opt_o.state[p], opt_s.state[q]
        assert torch.allclose(so["exp_avg"], ss["exp_avg"], rtol=1e-5, atol=1e-6 * max(scale, 1e-3))
        assert torch.allclose(so["exp_avg_sq"], ss["exp_avg_sq"], rtol=1e-5, atol=1e-7 * max(scale, 1e-3) ** 2)
        assert so["step"].item() == 5.0 == float(ss["step"])


def test_weight_decay_betas_eps(device):
    ours, stock, *_ = _run_pair(device, 4, 1.0, 1.0, lr=3e-3, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.1)
    for p, q in zip(ours, stock):
        assert torch.allclose(p, q, rtol=1e-5, atol=1e-6)


def test_first_step_is_lr_times_sign_and_clipping_scales_the_moments(device):
    """Closed forms: after one step from zero moments the update is lr * g / (|g| + eps*...) ~ lr * sign(g); the first
    moment equals (1 - beta1) * clip * g with clip = max_norm / (norm + 1e-6)."""
    p = torch.zeros(1000, device=device, requires_grad=True)
    g = torch.linspace(-2, 2, 1000, device=device)
    p.grad = g.clone()
    opt = sa.FusedClipAdam([p], lr=0.5, max_norm=1.0)
    opt.step()
    norm = g.norm().item()
    assert abs(opt.grad_norm.item() - norm) <= 1e-5 * norm
    clip = 1.0 / (norm + 1e-6)
    assert torch.allclose(opt.state[p]["exp_avg"], 0.1 * clip * g, rtol=1e-5, atol=1e-9)
    big = g.abs() * clip > 1e-4
    assert torch.allclose(p.detach()[big], -0.5 * torch.sign(g[big]), rtol=1e-3)


def test_more_tensors_than_one_launch_holds_and_missing_gradients(device):
    sizes = [(i % 7 + 1, 33) for i in range(130)]
    ours, stock = _make(device, sizes), _make(device, sizes)
    opt_o = sa.FusedClipAdam(ours, lr=1e-2, max_norm=1.0)
    opt_s = torch.optim.Adam(stock, lr=1e-2, foreach=False, fused=False)
    for step in range(3):
        _set_grads(ours, step, 1.0)
        _set_grads(stock, step, 1.0)
        for i in (5, 77):  # parameters without a gradient are left alone and do not count in the norm
            ours[i].grad = None
            stock[i].grad = None
        opt_o.step()
        torch.nn.utils.clip_grad_norm_(stock, 1.0)
        opt_s.step()
    for p, q in zip(ours, stock):
        assert torch.allclose(p, q, rtol=1e-5, atol=1e-6)


def test_parameter_groups_share_one_norm(device):
    ours, stock = _make(device), _make(device)
    opt_o = sa.FusedClipAdam([{"params": ours[:4], "lr": 1e-2}, {"params": ours[4:], "lr": 1e-3, "weight_decay": 0.05}], max_norm=1.0)
    opt_s = torch.optim.Adam([{"params": stock[:4], "lr": 1e-2}, {"params": stock[4:], "lr": 1e-3, "weight_decay": 0.05}],
                             foreach=False, fused=False)
    for step in range(3):
        _set_grads(ours, step, 1.0)
        _set_grads(stock, step, 1.0)
        opt_o.step()
        torch.nn.utils.clip_grad_norm_(stock, 1.0)
        opt_s.step()
    for p, q in zip(ours, stock):
        assert torch.allclose(p, q, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_shadow_copy_is_the_rounded_parameter(device, dtype):
    ours = _make(device)
    opt = sa.FusedClipAdam(ours, lr=1e-2, max_norm=1.0, shadow_dtype=dtype)
    for step in range(2):
        _set_grads(ours, step, 1.0)
        opt.step()
    for p in ours:
        sh = opt.shadow[p]
        assert sh.dtype is dtype and sh.stride() == p.stride()
        assert torch.equal(sh, p.detach().to(dtype))


def test_same_inputs_same_bits_and_state_dict_round_trip(device):
    a, b = _make(device), _make(device)
    oa, ob = sa.FusedClipAdam(a, lr=1e-2, max_norm=1.0), sa.FusedClipAdam(b, lr=1e-2, max_norm=1.0)
    for step in range(3):
        _set_grads(a, step, 1.0)
        _set_grads(b, step, 1.0)
        oa.step()
        ob.step()
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    # continue b from a checkpoint loaded into a fresh optimizer, and into torch's Adam
    sd = oa.state_dict()  # holds references: every consumer below gets its own deep copy
    c = [p.detach().clone().requires_grad_(True) for p in a]
    oc = sa.FusedClipAdam(c, lr=1e-2, max_norm=1.0)
    oc.load_state_dict(copy.deepcopy(sd))
    d = [p.detach().clone().requires_grad_(True) for p in a]
    od = torch.optim.Adam(d, lr=1e-2, foreach=False, fused=False)
    od.load_state_dict(copy.deepcopy(sd))
    for params, opt in ((a, oa), (c, oc)):
        _set_grads(params, 9, 1.0)
        opt.step()
    _set_grads(d, 9, 1.0)
    torch.nn.utils.clip_grad_norm_(d, 1.0)
    od.step()
    assert all(torch.equal(p, q) for p, q in zip(a, c))
    assert all(torch.allclose(p, q, rtol=1e-5, atol=1e-6) for p, q in zip(a, d))


def test_rejects_what_it_cannot_serve(device):
    with pytest.raises(ValueError):
        sa.FusedClipAdam([torch.zeros(4, device=device, requires_grad=True)], lr=-1.0)
    with pytest.raises(ValueError):
        sa.FusedClipAdam([torch.zeros(4, device=device, requires_grad=True)], max_norm=0.0)
    half = torch.zeros(4, device=device, dtype=torch.bfloat16, requires_grad=True)
    half.grad = torch.ones_like(half)
    with pytest.raises(NotImplementedError):
        sa.FusedClipAdam([half]).step()
    host = torch.zeros(4, requires_grad=True)
    host.grad = torch.ones(4)
    with pytest.raises(NotImplementedError):
        sa.FusedClipAdam([host]).step()
    strided = torch.zeros(8, 8, device=device)[:, ::2].requires_grad_(True)
    strided.grad = torch.ones_like(strided)
    with pytest.raises(NotImplementedError):
        sa.FusedClipAdam([strided]).step()


def test_step_captured_in_a_graph_replays_to_the_eager_result(device):
    eager = _make(device)
    oe = sa.FusedClipAdam(eager, lr=1e-2, max_norm=1.0)
    graphed = _make(device)
    og = sa.FusedClipAdam(graphed, lr=1e-2, max_norm=1.0)
    static = [torch.zeros_like(p) for p in graphed]
    for p, s in zip(graphed, static):
        p.grad = s
    # warm up on a side stream (allocates state), then rewind it
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        og.step()
    torch.cuda.current_stream().wait_stream(side)
    fresh = _make(device)
    with torch.no_grad():
        for p, f in zip(graphed, fresh):
            p.copy_(f)
            og.state[p]["exp_avg"].zero_()
            og.state[p]["exp_avg_sq"].zero_()
        og.state[graphed[0]]["step"].zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        og.step()
    for step in range(4):
        _set_grads(eager, step, 1.0)
        oe.step()
        for p, s in zip(eager, static):
            s.copy_(p.grad)
        graph.replay()
        torch.cuda.synchronize()
        torch.randn(1 << 14, device=device).sum().item()
        assert all(torch.equal(p, q) for p, q in zip(eager, graphed)), step


# ---- half-precision parameter copies feeding the modules, fp32 weight gradients ---------------------------------
@pytest.mark.parametrize("shape", [
    # cin, cout, spatial, kernel, stride, padding     (tiled MFMA, 2x2x2 stride-2, thin head, thin stem)
    (32, 32, (8, 16, 32), 3, 1, 1),
    (64, 128, (4, 8, 8), 3, 1, 1),
    (256, 512, (4, 8, 8), 3, 1, 1),   # one voxel slice: the fp32 gradient is written in place, no sum pass
    (32, 64, (8, 8, 16), 2, 2, 0),
    (32, 11, (8, 8, 16), 1, 1, 0),
    (1, 32, (8, 16, 32), 3, 1, 1),
])
def test_fp32_weight_gradient_is_the_unrounded_sum(device, shape):
    """grad_dtype=float32 stores the fp32 slice sum the 16-bit path rounds: rounding it must give the 16-bit result
    bit for bit."""
    cin, cout, sp, k, stride, pad = shape
    g = torch.Generator().manual_seed(21)
    x = torch.randn((1, cin, *sp), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    osp = tuple((s + 2 * pad - k) // stride + 1 for s in sp)
    gy = torch.randn((1, cout, *osp), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    wshape = (cout, cin, k, k, k)
    g16 = sa.conv3d_backward_weight(x, wshape, gy, stride, pad, 1)
    g32 = sa.conv3d_backward_weight(x, wshape, gy, stride, pad, 1, grad_dtype=torch.float32)
    assert g32.dtype is torch.float32 and g32.stride() == g16.stride()
    assert torch.equal(g32.to(torch.bfloat16), g16)
    assert not torch.equal(g32, g16.float())  # it really carries more bits


def test_fp32_weight_gradient_refused_where_only_the_untiled_kernel_applies(device):
    x = torch.randn((1, 5, 6, 6, 6), device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn((1, 7, 6, 6, 6), device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    with pytest.raises(NotImplementedError):
        sa.conv3d_backward_weight(x, (7, 5, 3, 3, 3), gy, 1, 1, 1, grad_dtype=torch.float32)
    with pytest.raises(ValueError):
        sa.conv3d_backward_weight(x, (7, 5, 3, 3, 3), gy, 1, 1, 1, grad_dtype=torch.float16)


def _tiny_unet(device):
    torch.manual_seed(31)
    model = sa.UNet(1, 5, layers=2, base_width=32).to(device).to(memory_format=CL)
    g = torch.Generator().manual_seed(32)
    x = (torch.rand((1, 1, 16, 16, 32), generator=g) < 0.05).float().contiguous(memory_format=CL).to(device)
    lab = torch.randint(0, 5, (1, 16, 16, 32), generator=g).to(device)
    return model, x, lab


def _train(model, opt, x, lab, steps):
    losses, grads = [], None
    for _ in range(steps):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = model(x)
        loss = sa.ce_dice_loss(logits, lab)
        loss.backward()
        if grads is None:
            grads = {k: p.grad.clone() for k, p in model.named_parameters()}
        opt.step()
        opt.zero_grad(set_to_none=True)
        losses.append(loss.item())
    return losses, grads


def test_modules_read_the_optimizers_copies_and_get_fp32_gradients(device):
    """Same model trained with and without the optimizer's bf16 copies: the first forward is bitwise the same (the
    copy is the cast autocast would make), every parameter gradient is fp32 and equals the cast path's up to the one
    bf16 rounding that path applies, and training stays together."""
    plain, x, lab = _tiny_unet(device)
    fused, _, _ = _tiny_unet(device)
    opt_p = sa.FusedClipAdam(plain.parameters(), lr=1e-3, max_norm=1.0)
    opt_f = sa.FusedClipAdam(fused.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
    from scaffold_amd.modules import compute_copy
    convs = [m for m in fused.modules() if isinstance(m, (sa.FastConv3d, sa.FastConvTranspose3d))]
    assert convs and all(compute_copy(m.weight, torch.bfloat16) is not None for m in convs)
    lp, gp = _train(plain, opt_p, x, lab, 4)
    lf, gf = _train(fused, opt_f, x, lab, 4)
    assert lp[0] == lf[0]
    for k in gp:
        assert gf[k].dtype is torch.float32
        # conv weights and biases: the cast path rounded to bf16 once; GroupNorm parameters: fp32 in both
        assert torch.equal(gf[k].to(torch.bfloat16), gp[k].to(torch.bfloat16)) or \
            torch.allclose(gf[k], gp[k], rtol=1e-5, atol=1e-7), k
    assert all(abs(a - b) <= 2e-3 * abs(a) for a, b in zip(lp, lf))
    # after the steps the copies are still current and equal to the rounded parameters
    for m in convs:
        c = compute_copy(m.weight, torch.bfloat16)
        assert c is not None and torch.equal(c, m.weight.detach().to(torch.bfloat16))


def test_a_parameter_written_by_someone_else_is_not_read_through_a_stale_copy(device):
    model, x, lab = _tiny_unet(device)
    opt = sa.FusedClipAdam(model.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
    from scaffold_amd.modules import compute_copy
    conv = next(m for m in model.modules() if isinstance(m, sa.FastConv3d))
    assert compute_copy(conv.weight, torch.bfloat16) is not None
    with torch.no_grad():
        conv.weight.mul_(0.5)  # version counter moves
    assert compute_copy(conv.weight, torch.bfloat16) is None
    with torch.autocast("cuda", dtype=torch.bfloat16), torch.no_grad():
        y_after = model(x)
    ref, _, _ = _tiny_unet(device)
    with torch.no_grad():
        next(m for m in ref.modules() if isinstance(m, sa.FastConv3d)).weight.mul_(0.5)
    with torch.autocast("cuda", dtype=torch.bfloat16), torch.no_grad():
        assert torch.equal(y_after, ref(x))
    opt.refresh_shadows()
    assert compute_copy(conv.weight, torch.bfloat16) is not None


def _to_host(obj):
    """The reference's restore path: every tensor of the optimizer state dict moved to the host before it is loaded
    back (`ScaFFold/utils/checkpointing.py:309-340`)."""
    if torch.is_tensor(obj):
        return obj.detach().cpu()
    if isinstance(obj, dict):
        return {k: _to_host(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return type(obj)(_to_host(v) for v in obj)
    return obj


def _assign_grads(params, values):
    """The same logical gradient values for every arm, each in its parameter's own memory layout."""
    for p, v in zip(params, values):
        fmt = CL if p.dim() == 5 and not p.is_contiguous() else torch.contiguous_format
        p.grad = v.to(p.device).contiguous(memory_format=fmt)


@pytest.mark.parametrize("source", ["stock_adam", "ours_through_the_host"])
def test_resume_from_a_checkpoint_whose_step_counters_live_on_the_host(device, source):
    """A checkpoint of a non-fused torch.optim.Adam (host `step`, contiguous moments for a weight we keep channels-last) or
    our own state dict after a round trip through host memory: the resumed run must continue like stock clip + Adam."""
    sizes = [(8, 4, 3, 3, 3), (33,), (8193,)]
    gen = torch.Generator().manual_seed(5)
    a = _make(device, sizes, channels_last=source != "stock_adam")   # the stock run keeps its 5-d weight contiguous
    stock = [p.detach().clone().requires_grad_(True) for p in a]
    opt_a = torch.optim.Adam(a, lr=1e-2, foreach=False, fused=False) if source == "stock_adam" else sa.FusedClipAdam(a, lr=1e-2, max_norm=1.0)
    opt_s = torch.optim.Adam(stock, lr=1e-2, foreach=False, fused=False)
    for _ in range(3):
        values = [torch.randn(s, generator=gen) for s in sizes]
        _assign_grads(stock, values)
        _assign_grads(a, values)
        torch.nn.utils.clip_grad_norm_(stock, 1.0)
        opt_s.step()
        if source == "stock_adam":
            torch.nn.utils.clip_grad_norm_(a, 1.0)
        opt_a.step()
    sd = _to_host(copy.deepcopy(opt_a.state_dict()))
    assert sd["state"][0]["step"].device.type == "cpu"
    # resume into our optimizer with the 5-d weight channels-last
    mine = [p.detach().clone().contiguous(memory_format=CL).requires_grad_(True) if p.dim() == 5 else p.detach().clone().requires_grad_(True)
            for p in a]
    opt_m = sa.FusedClipAdam(mine, lr=1e-2, max_norm=1.0)
    opt_m.load_state_dict(sd)
    for p in mine:
        st = opt_m.state[p]
        assert st["step"].is_cuda and st["step"].dtype is torch.float32 and st["exp_avg"].stride() == p.stride()
    for _ in range(2):
        values = [torch.randn(s, generator=gen) for s in sizes]
        _assign_grads(stock, values)
        _assign_grads(mine, values)
        torch.nn.utils.clip_grad_norm_(stock, 1.0)
        opt_s.step()
        opt_m.step()
    for p, q in zip(mine, stock):
        assert torch.allclose(p, q, rtol=1e-5, atol=1e-6)
        assert torch.allclose(opt_m.state[p]["exp_avg"], opt_s.state[q]["exp_avg"], rtol=1e-5, atol=1e-7)
        assert torch.allclose(opt_m.state[p]["exp_avg_sq"], opt_s.state[q]["exp_avg_sq"], rtol=1e-5, atol=1e-9)
        assert opt_m.state[p]["step"].item() == 5.0
