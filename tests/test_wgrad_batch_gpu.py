"""Several weight gradients from one launch (``conv3d_backward_weight_batch``, ``sfh_conv3d_wgrad_batch``), and the
backward pass that uses it (``FastConv3d.defer_weight_grad``).

The reference computes each weight gradient with a launch of its own (``triton_conv3d/reduce_gemm.py:1177``); the batch is
the same arithmetic -- fp32 partial sums over voxel ranges, added in a fixed order -- with the ranges cut differently, so
what it is held to is: the fp64 oracle's error bound for every problem of a list (ragged extents, several samples, the
depth-shard form, inputs handed over as two tensors, lists long enough that a workgroup covers parts of several problems
and lists so short that a problem spans many workgroups, small volumes whose blocks are walked whole, both kinds in one
list), agreement with the one-problem entry point to fp32
summation-order rounding, the same bits on every run and for every list with the same shapes, and refusal -- before any
launch -- of a list with a problem the batch does not serve.
"""

import pytest
import torch

import scaffold_amd as sa
from oracle import oracle as orc
from scaffold_amd import _lib
from scaffold_amd import conv3d as c3
from scaffold_amd import modules

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d

# (n, cin, cout, spatial of the output, padding, cut of the input into two tensors or 0)
LISTS = {
    "one-small": [(1, 32, 32, (4, 8, 32), (1, 1, 1), 0)],
    "one-large": [(1, 32, 32, (24, 64, 96), (0, 1, 1), 0)],                          # many workgroups per block
    "ragged": [(2, 32, 64, (5, 7, 33), (1, 1, 1), 0), (1, 64, 32, (3, 9, 47), (0, 1, 1), 32)],
    "levels": [(1, 32, 32, (16, 32, 64), (0, 1, 1), 0), (1, 64, 32, (16, 32, 64), (0, 1, 1), 32),
               (1, 32, 64, (8, 16, 32), (0, 1, 1), 0), (1, 64, 64, (8, 16, 32), (0, 1, 1), 0),
               (1, 128, 64, (8, 16, 32), (0, 1, 1), 64), (1, 64, 128, (4, 8, 32), (1, 1, 1), 0),
               (1, 128, 128, (4, 8, 32), (1, 1, 1), 0), (1, 256, 128, (4, 8, 32), (1, 1, 1), 128)],
    "many-blocks": [(1, 128, 256, (2, 4, 32), (1, 1, 1), 0), (1, 96, 160, (3, 5, 40), (1, 1, 1), 32),
                    (1, 32, 32, (2, 4, 17), (1, 1, 1), 0)],                          # more blocks than workgroups
    # small volumes (rows of 16 and of 8 voxels): whole blocks per workgroup, no slices
    "deep": [(1, 128, 256, (8, 16, 16), (0, 1, 1), 0), (1, 256, 256, (8, 16, 16), (0, 1, 1), 0),
             (1, 512, 256, (8, 16, 16), (0, 1, 1), 256), (1, 256, 512, (4, 8, 8), (0, 1, 1), 0)],
    "deep-ragged": [(2, 32, 64, (3, 5, 7), (1, 1, 1), 0), (1, 64, 32, (5, 9, 13), (1, 1, 1), 32), (3, 32, 32, (1, 1, 1), (1, 1, 1), 0),
                    (1, 96, 64, (9, 16, 16), (0, 1, 1), 64)],
    # both families in one list (two launches and a sum pass)
    "mixed": [(1, 64, 64, (8, 16, 32), (0, 1, 1), 0), (1, 128, 256, (4, 8, 16), (1, 1, 1), 0), (1, 64, 128, (4, 8, 32), (1, 1, 1), 32),
              (1, 256, 256, (4, 8, 8), (1, 1, 1), 128)],
}


def _make(lst, dtype, device, seed=3):
    problems, refs = [], []
    for i, (n, cin, cout, spatial, padding, cut) in enumerate(lst):
        prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=tuple(s + 2 - 2 * p for s, p in zip(spatial, padding)),
                               padding=padding, dtype=dtype)
        ops = orc.make_inputs(prob, seed=seed + i)
        x, gy = ops["input"].to(device), ops["grad_output"].to(device)
        assert tuple(gy.shape[2:]) == tuple(spatial)
        inp = x if cut == 0 else (x[:, :cut].contiguous(memory_format=CL), x[:, cut:].contiguous(memory_format=CL))
        problems.append((inp, (cout, cin, 3, 3, 3), gy, padding))
        refs.append((prob, ops, x))
    return problems, refs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("name", list(LISTS))
def test_batch_against_the_oracle_and_the_single_calls(device, dtype, name):
    problems, refs = _make(LISTS[name], dtype, device)
    for (inp, wshape, gy, padding), (prob, ops, x) in zip(problems, refs):
        assert c3.weight_grad_batchable(x.shape, wshape, 1, padding, 1, dtype)
    got = sa.conv3d_backward_weight_batch(problems, grad_dtype=torch.float32)
    again = sa.conv3d_backward_weight_batch(problems, grad_dtype=torch.float32)
    rounded = sa.conv3d_backward_weight_batch(problems)
    for (inp, wshape, gy, padding), (prob, ops, x), g, g2, r in zip(problems, refs, got, again, rounded):
        assert g.dtype is torch.float32 and r.dtype is dtype and g.is_contiguous(memory_format=CL)
        assert torch.equal(g, g2)                                   # the same bits on every run
        assert torch.equal(r, g.to(dtype))                          # one rounding of the same sum
        orc.assert_close(r, orc.conv_reference(prob, ops, "bwd-weight"), prob, "bwd-weight")
        single = sa.conv3d_backward_weight(x, wshape, gy, 1, padding, 1, grad_dtype=torch.float32)
        # the two sum the same products in different orders: fp32 rounding of sums of up to ~1e5 terms
        scale = single.abs().max().item()
        assert (g - single).abs().max().item() <= 2e-5 * scale
    # on half of the compute units (a batch meant to run beside other work): another cut, the same sums
    shared = sa.conv3d_backward_weight_batch(problems, grad_dtype=torch.float32, share_device=True)
    shared2 = sa.conv3d_backward_weight_batch(problems, grad_dtype=torch.float32, share_device=True)
    for g, s1, s2 in zip(got, shared, shared2):
        assert torch.equal(s1, s2)
        assert (g - s1).abs().max().item() <= 2e-5 * g.abs().max().item()


def test_the_cut_depends_on_the_shapes_alone(device):
    """Other tensors of the same shapes, in the same order, are cut the same way: a problem's gradient does not depend on
    what the other problems' operands hold, and depends on their shapes only through the fixed cut."""
    dtype = torch.bfloat16
    problems, _ = _make(LISTS["levels"], dtype, device, seed=3)
    others, _ = _make(LISTS["levels"], dtype, device, seed=50)
    base = sa.conv3d_backward_weight_batch(problems, grad_dtype=torch.float32)
    mixed = [problems[0]] + others[1:]
    assert torch.equal(sa.conv3d_backward_weight_batch(mixed, grad_dtype=torch.float32)[0], base[0])
    mixed = others[:-1] + [problems[-1]]
    assert torch.equal(sa.conv3d_backward_weight_batch(mixed, grad_dtype=torch.float32)[-1], base[-1])
    outs = [torch.full_like(g, float("nan")) for g in base]         # caller-supplied outputs, overwritten whole
    back = sa.conv3d_backward_weight_batch(problems, grad_dtype=torch.float32, outs=outs)
    assert all(b is o and torch.equal(b, g) for b, o, g in zip(back, outs, base))


def test_more_problems_than_a_launch_takes(device):
    dtype = torch.bfloat16
    lst = [(1, 32, 32, (2, 4, 32), (1, 1, 1), 0)] * (c3.WGRAD_BATCH_MAX + 3)
    problems, refs = _make(lst, dtype, device)
    got = sa.conv3d_backward_weight_batch(problems)
    for (prob, ops, x), g in zip(refs, got):
        orc.assert_close(g, orc.conv_reference(prob, ops, "bwd-weight"), prob, "bwd-weight")


def test_what_is_refused(device):
    dtype = torch.bfloat16
    ok = (1, 32, 32, (4, 8, 32), (1, 1, 1), 0)
    assert c3.weight_grad_batchable((1, 32, 4, 8, 16), (32, 32, 3, 3, 3), 1, 1, 1, dtype)            # rows of 16 voxels, two tiles
    assert not c3.weight_grad_batchable((1, 32, 40, 64, 16), (32, 32, 3, 3, 3), 1, 1, 1, dtype)      # ... and 160 tiles
    assert not c3.weight_grad_batchable((1, 32, 4, 8, 32), (32, 32, 1, 1, 1), 1, 0, 1, dtype)        # not 3x3x3
    assert not c3.weight_grad_batchable((1, 32, 4, 8, 32), (32, 32, 3, 3, 3), 2, 1, 1, dtype)        # strided
    assert not c3.weight_grad_batchable((1, 48, 4, 8, 32), (32, 48, 3, 3, 3), 1, 1, 1, dtype)        # channels off the grid
    assert not c3.weight_grad_batchable((1, 32, 4, 8, 32), (32, 32, 3, 3, 3), 1, 1, 1, torch.float32)
    problems, _ = _make([ok, (1, 32, 32, (40, 64, 16), (1, 1, 1), 0)], dtype, device)
    with pytest.raises(NotImplementedError):
        sa.conv3d_backward_weight_batch(problems)
    # through the C ABI: the list is refused as a whole, with the library's own code, and a short workspace is an error
    L = _lib.lib()
    good, _ = _make([ok, ok], dtype, device)
    items = (_lib.WgradItem * 2)()
    gws = []
    for it, (x, wshape, gy, padding) in zip(items, good):
        prob = c3._problem(x.shape, torch.Size(wshape), 1, padding, 1, dtype)
        gw = torch.empty((32, 32, 3, 3, 3), dtype=dtype, device=device).contiguous(memory_format=CL)
        gws.append(gw)
        it.desc, it.x, it.x_second, it.cin_first, it.gy, it.gw = prob.desc, _lib.ptr(x), None, 0, _lib.ptr(gy), _lib.ptr(gw)
    code = c3._problem(good[0][0].shape, torch.Size(good[0][1]), 1, (1, 1, 1), 1, dtype).code
    need = int(L.sfh_conv3d_wgrad_batch_workspace_bytes(items, 2, code, 0))
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    stream = _lib.stream_ptr(device)
    assert L.sfh_conv3d_wgrad_batch(items, 2, code, _lib.ptr(ws), need - 256, 0, stream) == _lib.SFH_ERR_WORKSPACE
    assert L.sfh_conv3d_wgrad_batch(items, 0, code, _lib.ptr(ws), need, 0, stream) == _lib.SFH_ERR_INVALID
    assert L.sfh_conv3d_wgrad_batch(items, 2, code, _lib.ptr(ws), need, _lib.SFH_FLAG_FORCE_GENERIC, stream) == _lib.SFH_ERR_INVALID
    assert L.sfh_conv3d_wgrad_batch(items, 2, code, _lib.ptr(ws), need, 0, stream) == _lib.SFH_OK
    torch.cuda.synchronize()
    assert torch.equal(gws[0], sa.conv3d_backward_weight_batch(good)[0])
    items[1].desc.sd = 2                                            # a strided problem in the list
    assert int(L.sfh_conv3d_wgrad_batch_workspace_bytes(items, 2, code, 0)) == 0
    assert L.sfh_conv3d_wgrad_batch(items, 2, code, _lib.ptr(ws), need, 0, stream) == _lib.SFH_ERR_UNSUPPORTED


def _tiny_net(device, defer, layers=2):
    torch.manual_seed(7)
    net = sa.UNet(1, 3, layers=layers, base_width=32).to(device).to(memory_format=CL).set_shard_halo(True)
    if defer == "early":
        return net.defer_weight_gradients(early=True)
    return net.defer_weight_gradients() if defer else net


@pytest.mark.parametrize("master", [True, False], ids=["fp32-masters", "bf16-weights"])
def test_backward_pass_with_deferred_weight_gradients(device, master):
    """The U-Net's backward pass with every batchable weight gradient left to the end of the pass: all gradients are
    there when ``backward()`` returns, those of the deferred convolutions within summation-order rounding of the ordinary
    pass's, every other gradient the same bits; a second pass accumulates; nothing stays queued."""
    x = torch.randn(1, 1, 8, 32, 64, device=device).contiguous(memory_format=CL)
    target = torch.randint(0, 3, (1, 8, 32, 64), device=device)
    grads = {}
    for defer in (False, True):
        net = _tiny_net(device, defer)
        if not master:
            net = net.to(torch.bfloat16)
        else:
            # the optimizer keeps the bf16 copies the convolutions read under autocast: their nodes then take the fp32
            # parameter itself and return (or defer) an fp32 gradient
            opt = sa.FusedClipAdam(net.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
        for rep in range(2):
            if master:
                with torch.autocast("cuda", dtype=torch.bfloat16):
                    logits = net(x)
            else:
                logits = net(x.to(torch.bfloat16))
            sa.ce_dice_loss(logits, target).backward()
            assert not modules._WEIGHT_GRAD_QUEUE
            if rep == 0:
                grads[defer, 0] = {n: p.grad.detach().clone() for n, p in net.named_parameters()}
        grads[defer, 1] = {n: p.grad.detach().clone() for n, p in net.named_parameters()}
        for n, p in net.named_parameters():
            assert p.grad.dtype is p.dtype and p.grad.stride() == p.stride(), n
    deferred = 0
    for rep in (0, 1):
        for n, g in grads[False, rep].items():
            d = grads[True, rep][n]
            if torch.equal(g, d):
                continue
            deferred += 1
            assert n.endswith("weight") and g.dim() == 5 and tuple(g.shape[2:]) == (3, 3, 3), n
            tol = 2e-5 if master else 2.0 ** -7          # fp32 sums in another order / one bf16 rounding of each
            assert (g.float() - d.float()).abs().max().item() <= tol * (rep + 1) * g.float().abs().max().item(), n
    assert deferred > 0                                   # the mode was taken up
    # the accumulated gradients are twice the first pass's (same inputs), up to the rounding of the addition
    for n, g in grads[True, 1].items():
        first = grads[True, 0][n].float()
        assert (g.float() - 2 * first).abs().max().item() <= 2.0 ** -6 * max(first.abs().max().item(), 1e-30), n


def test_flush_by_hand_and_unbatchable_weights_are_computed_in_place(device):
    """A convolution the batch does not serve (rows of 16 voxels, 160 tiles) computes its gradient in its own node although
    the flag is set; a queue left by a pass that raised is emptied by ``flush_weight_gradients()``."""
    torch.manual_seed(1)
    conv = sa.FastConv3d(32, 32, 3, padding=1, bias=False).to(device).to(torch.bfloat16).to(memory_format=CL)
    conv.defer_weight_grad = True
    x = torch.randn(1, 32, 40, 64, 16, device=device, dtype=torch.bfloat16).contiguous(memory_format=CL).requires_grad_()
    conv(x).sum().backward()
    assert conv.weight.grad is not None and not modules._WEIGHT_GRAD_QUEUE
    ref = sa.conv3d_backward_weight(x.detach(), conv.weight.shape, torch.ones(1, 32, 40, 64, 16, device=device, dtype=torch.bfloat16), 1, 1, 1)
    assert torch.equal(conv.weight.grad, ref)
    # a queued entry that no callback took: flush by hand
    conv.weight.grad = None
    x2 = torch.randn(1, 32, 4, 8, 32, device=device, dtype=torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn(1, 32, 4, 8, 32, device=device, dtype=torch.bfloat16).contiguous(memory_format=CL)
    modules._WEIGHT_GRAD_QUEUE.append(modules._QueuedWeightGrad(conv.weight, x2, conv.weight.shape, gy, (1, 1, 1), torch.bfloat16))
    modules.flush_weight_gradients()
    assert not modules._WEIGHT_GRAD_QUEUE
    assert torch.equal(conv.weight.grad, sa.conv3d_backward_weight_batch([(x2, conv.weight.shape, gy, (1, 1, 1))])[0])


def test_deferred_step_as_a_hip_graph_and_under_checkpointing(device):
    """The step with deferred weight gradients (fused clip + Adam keeping the bf16 copies) captured once and replayed gives
    the eager step's losses from the same state, replay after replay; and with activation checkpointing the nested backward
    passes flush their own queues: same gradients as without."""
    x = torch.randn(1, 1, 8, 32, 64, device=device).contiguous(memory_format=CL)
    target = torch.randint(0, 3, (1, 8, 32, 64), device=device)

    def make():
        net = _tiny_net(device, defer=True)
        opt = sa.FusedClipAdam(net.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)

        def step():
            with torch.autocast("cuda", dtype=torch.bfloat16):
                logits = net(x)
            loss = sa.ce_dice_loss(logits, target)
            loss.backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
            return loss.detach()
        return net, opt, step

    _, _, eager = make()
    want = [eager().item() for _ in range(4)]
    net2, opt2, step2 = make()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        warm = step2().item()  # the first step eagerly (libraries initialise, the optimizer state appears), the second captured
    torch.cuda.current_stream().wait_stream(side)
    assert warm == want[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_loss = step2()
    got = []
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        got.append(static_loss.item())
        torch.randn(1 << 16, device=device).sum().item()
    assert got == want[1:]
    assert not modules._WEIGHT_GRAD_QUEUE

    grads = {}
    for ckpt in (False, True):
        net = _tiny_net(device, defer=True)
        opt = sa.FusedClipAdam(net.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
        if ckpt:
            net.use_checkpointing()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = net(x.clone().requires_grad_(True) if ckpt else x)
        sa.ce_dice_loss(logits, target).backward()
        assert not modules._WEIGHT_GRAD_QUEUE
        grads[ckpt] = {n: p.grad.detach().clone() for n, p in net.named_parameters()}
    for n, g in grads[False].items():
        d = grads[True][n].float()
        assert (g.float() - d).abs().max().item() <= 2e-2 * max(g.float().abs().max().item(), 1e-30), n


def test_early_weight_gradients_on_a_stream_of_their_own(device, monkeypatch):
    """With ``defer_weight_gradients(early=True)`` the large-row gradients queued when the backward pass reaches its first
    small volume leave on a side stream (half of the compute units) and are joined at the end of the pass: every gradient
    is there when ``backward()`` returns, within summation-order rounding of the ordinary pass's; the captured step replays
    to the eager step's losses."""
    x = torch.randn(1, 1, 8, 32, 64, device=device).contiguous(memory_format=CL)
    target = torch.randint(0, 3, (1, 8, 32, 64), device=device)
    sent = []
    real = modules._send_early
    monkeypatch.setattr(modules, "_send_early", lambda items: (sent.append(len(items)), real(items))[1])
    grads = {}
    for defer in (False, "early"):
        net = _tiny_net(device, defer, layers=3)
        opt = sa.FusedClipAdam(net.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
        for rep in range(2):
            with torch.autocast("cuda", dtype=torch.bfloat16):
                logits = net(x)
            sa.ce_dice_loss(logits, target).backward()
            assert not modules._WEIGHT_GRAD_QUEUE and not modules._EARLY_DONE
        grads[defer] = {n: p.grad.detach().clone() for n, p in net.named_parameters()}
    assert sent and all(n >= 2 for n in sent)                 # the side stream was used, once per pass
    for n, g in grads[False].items():
        d = grads["early"][n]
        assert d.dtype is g.dtype and d.stride() == g.stride(), n
        assert (g.float() - d.float()).abs().max().item() <= 2 * 2e-5 * max(g.float().abs().max().item(), 1e-30), n

    def make():
        net = _tiny_net(device, "early", layers=3)
        opt = sa.FusedClipAdam(net.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)

        def step():
            with torch.autocast("cuda", dtype=torch.bfloat16):
                logits = net(x)
            loss = sa.ce_dice_loss(logits, target)
            loss.backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
            return loss.detach()
        return step

    eager = make()
    want = [eager().item() for _ in range(4)]
    step2 = make()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        warm = step2().item()
    torch.cuda.current_stream().wait_stream(side)
    assert warm == want[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_loss = step2()
    got = []
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        got.append(static_loss.item())
        torch.randn(1 << 16, device=device).sum().item()
    assert got == want[1:]
    assert not modules._WEIGHT_GRAD_QUEUE and not modules._EARLY_DONE
