#!/usr/bin/env python3
"""Throughput of the ScaFFold U-Net hot path on one MI355X.

``python bench.py [--steps K] [--warmup W]`` prints ONE JSON line.

The workload (``config.workload``) is BASELINE.json's headline convolution: the 3x3x3, 32->32 channel,
stride-1 convolution of the first encoder level on a 128^3 volume, bf16 NDHWC, N=1 (config 3 of
BASELINE.json).  One *step* is one pass of the hot path over that batch: forward + data gradient +
weight gradient, operands resident in HBM.  ``value`` is the algorithmic FLOPs of the three directions
(3 x 2*M*N*K) divided by the measured step time.

Also on the line:
* ``roofline``: the dominant kernel (the MFMA implicit-GEMM kernel, forward direction), its launches inside the
  step timed with HIP events on the launch stream, against the dense bf16 MFMA peak of 2.5 PFLOP/s;
* ``cpu_baseline``: the reference's CPU path for the same op (stock torch ``conv3d`` + autograd on
  channels_last_3d bf16 tensors, which is what the reference's ladders fall to off-GPU), timed on the
  host cores of this box on a bounded sample of the workload;
* ``details``: per-direction TFLOP/s, GroupNorm (config 2) GB/s against the 8 TB/s HBM peak, and the
  U-Net train step of one depth shard (config 5) in ms.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the forward kernel on the bench workload, from rocprofv3 FETCH_SIZE and WRITE_SIZE
# counter runs of this script scaled by the same counters on the 256 MiB copy kernel (profiles/ holds the runs).
CONV_FWD_HBM_TRAFFIC_BYTES = int((115560.0 * 2.000 + 131163.9) * 1024)
CL = torch.channels_last_3d


def event_time_ms(fn, iters: int, warmup: int = 2) -> float:
    """Average GPU time of ``fn`` over ``iters`` back-to-back calls, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def conv_operands(cin, cout, spatial, device, seed=3000):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((1, cin, *spatial), generator=g, dtype=torch.float32).to(torch.bfloat16).contiguous(memory_format=CL)
    bound = 1.0 / math.sqrt(cin * 27)
    w = ((torch.rand((cout, cin, 3, 3, 3), generator=g) * 2 - 1) * bound).to(torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn((1, cout, *spatial), generator=g, dtype=torch.float32).to(torch.bfloat16).contiguous(memory_format=CL)
    return x.to(device), w.to(device), gy.to(device)


def bench_conv(args, device):
    import scaffold_amd as sa

    cin = cout = 32
    spatial = (128, 128, 128)
    x, w, gy = conv_operands(cin, cout, spatial, device)
    flops = 2 * math.prod(spatial) * cin * cout * 27
    y = torch.empty_like(gy)
    gx = torch.empty_like(x)
    gw = sa.grad_weight_empty(cout, cin, (3, 3, 3), dtype=x.dtype, device=device)

    def fwd():
        sa.conv3d_forward(x, w, None, 1, 1, 1, out=y)

    def dgrad():
        sa.conv3d_backward_data(gy, w, x.shape, 1, 1, 1, out=gx)

    def wgrad():
        sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, 1, out=gw)

    def step():
        # as in a train step: the weight is packed once (one launch, inside the timed region) for both the forward
        # and the data gradient; the per-direction timings below use the default entry points, which pack per call
        pf, pd = sa.pack_weights(w, x.shape, 1, 1, 1)
        sa.conv3d_forward(x, w, None, 1, 1, 1, out=y, packed_weight=pf)
        sa.conv3d_backward_data(gy, w, x.shape, 1, 1, 1, out=gx, packed_weight=pd)
        wgrad()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = max(e0.elapsed_time(e1) / args.steps, 1e-9)
    # A second pass over the same steps with an event between the launches: the duration of each kernel INSIDE the
    # step, where the three directions evict one another's tensors from the memory-side cache and share the power
    # budget. The forward figure of this pass is the launch duration the roofline object is computed from.
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    for m in marks:
        pf, pd = sa.pack_weights(w, x.shape, 1, 1, 1)
        m[0].record()
        sa.conv3d_forward(x, w, None, 1, 1, 1, out=y, packed_weight=pf)
        m[1].record()
        sa.conv3d_backward_data(gy, w, x.shape, 1, 1, 1, out=gx, packed_weight=pd)
        m[2].record()
        wgrad()
        m[3].record()
    torch.cuda.synchronize()
    in_step = {name: sum(m[i].elapsed_time(m[i + 1]) for m in marks) / len(marks)
               for i, name in enumerate(("fwd", "dgrad", "wgrad"))}
    # each direction in a loop of its own (default entry points: forward and data gradient pack per call), and the
    # forward kernel alone in such a loop (weight packed beforehand): with 128 MB of operands per launch these loops
    # run out of the 256 MB memory-side cache and are faster than the same kernels inside the step
    per_dir = {name: event_time_ms(fn, max(args.steps, 5)) for name, fn in (("fwd", fwd), ("dgrad", dgrad), ("wgrad", wgrad))}
    pf, _ = sa.pack_weights(w, x.shape, 1, 1, 1, backward_data=False)
    fwd_kernel_ms = event_time_ms(lambda: sa.conv3d_forward(x, w, None, 1, 1, 1, out=y, packed_weight=pf), max(args.steps, 5))
    return {
        "flops_per_direction": flops,
        "ms_per_step": ms_per_step,
        "wall_ms_per_step": wall_ms,
        "in_step_ms": in_step,
        "per_direction_ms": per_dir,
        "fwd_kernel_alone_ms": fwd_kernel_ms,
        "per_direction_tflops": {k: flops / (v * 1e-3) / 1e12 for k, v in per_dir.items()},
        "bytes_compulsory": 2 * (x.numel() + w.numel() + y.numel()),
    }


def bench_groupnorm(args, device):
    """Config 2: N=2, C=64, 64^3, 8 groups, bf16, fused ReLU; algorithmic bytes 3B forward / 5B backward.

    Timed twice: through the C ABI directly (what a compiled caller sees; the launch chain keeps the GPU busy)
    and through the registered torch operator (adds the Python dispatcher and output allocation per call)."""
    import ctypes

    import scaffold_amd.groupnorm  # noqa: F401  (registers torch.ops.scaffold_gn.*)
    from scaffold_amd import _lib

    g = torch.Generator().manual_seed(2000)
    shape = (2, 64, 64, 64, 64)
    x = (torch.randn(shape, generator=g) * 3 + 0.5).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    gamma = (1 + 0.1 * torch.randn(64, generator=g)).to(device)
    beta = (0.1 * torch.randn(64, generator=g)).to(device)
    dy = torch.randn(shape, generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    B = x.numel() * x.element_size()
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(x, 8, gamma, beta, 1e-5, "relu", None)
    op_fwd_ms = event_time_ms(lambda: torch.ops.scaffold_gn.group_norm(x, 8, gamma, beta, 1e-5, "relu", None), 10)
    op_bwd_ms = event_time_ms(lambda: torch.ops.scaffold_gn.group_norm_backward(dy, x, gamma, beta, mean, rstd, 8, "relu"), 10)

    BF16, FP32 = _lib.dtype_code(torch.bfloat16), _lib.dtype_code(torch.float32)
    L = _lib.lib()
    desc = _lib.GroupNormDesc(2, 64, 8, 1, 64 ** 3, 1e-5)
    dref = ctypes.byref(desc)
    ws_f = torch.empty(max(1, L.sfh_groupnorm_fwd_workspace_bytes(dref, BF16)), dtype=torch.uint8, device=device)
    ws_b = torch.empty(max(1, L.sfh_groupnorm_bwd_workspace_bytes(dref, BF16)), dtype=torch.uint8, device=device)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    dgamma, dbeta = torch.empty_like(gamma), torch.empty_like(beta)
    stream = torch.cuda.current_stream().cuda_stream
    P = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731

    def abi_fwd():
        _lib.check(L.sfh_groupnorm_fwd(dref, BF16, BF16, FP32, P(x), P(gamma), P(beta), P(y),
                                       P(mean), P(rstd), P(ws_f), ws_f.numel(), stream), "sfh_groupnorm_fwd")

    def abi_bwd():
        _lib.check(L.sfh_groupnorm_bwd(dref, BF16, BF16, FP32, P(dy), P(x), P(gamma), P(beta),
                                       P(mean), P(rstd), P(dx), P(dgamma), P(dbeta), P(ws_b), ws_b.numel(), stream), "sfh_groupnorm_bwd")

    fwd_ms = event_time_ms(abi_fwd, 20)
    bwd_ms = event_time_ms(abi_bwd, 20)
    return {
        "tensor_bytes": B,
        "fwd_ms": fwd_ms, "fwd_gbs": 3 * B / (fwd_ms * 1e-3) / 1e9, "fwd_frac_of_hbm_peak": 3 * B / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "bwd_ms": bwd_ms, "bwd_gbs": 5 * B / (bwd_ms * 1e-3) / 1e9, "bwd_frac_of_hbm_peak": 5 * B / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "torch_op_fwd_ms": op_fwd_ms, "torch_op_bwd_ms": op_bwd_ms,
    }


def bench_ingest(args, device, iters=20):
    """One rank's share of a 128-cube sample as the dataset stores it (float32 (3, 64, 128, 128) + 16-bit mask) into the
    bf16 channels-last slab of the first convolution and int64 labels, through the C ABI with outputs allocated once.
    Algorithmic bytes per voxel: 4 C read + 2 C written + 2 + 8 for the label; beside it the three torch passes the
    trainer runs (ScaFFold/utils/trainer.py:572-589 and autocast's cast)."""
    import ctypes

    from scaffold_amd import _lib

    n, c, d, h, w, halo = 1, 3, 64, 128, 128, 1
    g = torch.Generator().manual_seed(5002)
    volume = torch.rand((n, c, d, h, w), generator=g).to(device)
    mask = torch.randint(0, 11, (n, d, h, w), generator=g, dtype=torch.int16).to(device)
    slab = torch.empty((n, c, d + 2 * halo, h, w), dtype=torch.bfloat16, device=device, memory_format=CL)
    labels = torch.empty((n, d, h, w), dtype=torch.long, device=device)
    L = _lib.lib()
    desc = _lib.IngestDesc(n, c, 1, d * h * w, halo * h * w)
    P = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731

    def abi():
        _lib.check(L.sfh_shard_ingest(ctypes.byref(desc), _lib.dtype_code(torch.bfloat16), P(volume), P(mask), P(slab), P(labels),
                                      torch.cuda.current_stream().cuda_stream), "sfh_shard_ingest")

    def torch_passes():
        x = volume.to(dtype=torch.float32, memory_format=CL).to(torch.bfloat16)
        return x, mask.to(torch.long)

    # a 7 us kernel: replayed from a graph of `chunk` launches so that the figure is kernel time, not the launcher's
    chunk = 20
    abi()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(chunk):
            abi()
    ms = event_time_ms(graph.replay, max(1, iters // chunk) * 2) / chunk
    nbytes = n * d * h * w * (4 * c + 2 * c + 2 + 8)
    return {"input": "1x3x64x128x128 float32 + int16 mask -> bf16 slab (halo 1) + int64 labels", "ms": ms, "algorithmic_bytes": nbytes,
            "gbs": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "launched_from_python_ms": event_time_ms(abi, iters), "torch_three_passes_ms": event_time_ms(torch_passes, iters)}


def gemm_reference(device):
    """What the vendor's tuned dense GEMM (hipBLASLt through torch.matmul, 8192^3 bf16) reaches on this box in this
    run: the practical ceiling of the matrix pipe under real data and the chip's power management, next to the
    nominal 2.5 PFLOP/s the roofline fraction is quoted against."""
    n = 8192
    g = torch.Generator(device=device).manual_seed(4000)
    a = torch.randn((n, n), generator=g, device=device, dtype=torch.bfloat16)
    b = torch.randn((n, n), generator=g, device=device, dtype=torch.bfloat16)
    ms = event_time_ms(lambda: torch.matmul(a, b), 20, warmup=5)
    tflops = 2 * n ** 3 / (ms * 1e-3) / 1e12
    return {"workload": "torch.matmul 8192x8192x8192 bf16", "ms": ms, "tflops": tflops, "frac_of_mfma_peak": tflops / MFMA_PEAK_TFLOPS}


def copy_calibration(device, mib=256, reps=4):
    """Runs the library's plain copy kernel on a buffer of known size, so that a counter run of this script
    also holds FETCH_SIZE / WRITE_SIZE for a launch whose HBM traffic is known exactly."""
    import ctypes

    from scaffold_amd import _lib

    L = _lib.lib()
    src = torch.empty(mib << 20, dtype=torch.uint8, device=device).fill_(1)
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(reps):
        _lib.check(L.sfh_stream_copy(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), src.numel(), stream), "sfh_stream_copy")
    torch.cuda.synchronize()
    return {"bytes_read": src.numel(), "bytes_written": src.numel(), "launches": reps}


def bench_unet_step(args, device, eager_only=False):
    """Config 5: one Adam step of the base-32, 5-level U-Net on a 64x128x128 depth shard (zero halo),
    bf16 autocast, fp32 master weights, fused CE + Dice loss head, gradient clipping at 1.0 fused with the Adam update.

    Timed eagerly (how the reference's trainer runs) and, when the replay check passes, as a captured HIP graph
    of the whole step: the eager step is bound by ~600 Python-side launches, not by the GPU."""
    import scaffold_amd as sa

    g = torch.Generator().manual_seed(5000)
    occ = (torch.rand((1, 1, 64, 128, 128), generator=g) < 0.05).float().contiguous(memory_format=CL).to(device)
    lab = torch.randint(0, 11, (1, 64, 128, 128), generator=g).to(device)

    def make(shard_halo=True):
        torch.manual_seed(5001)
        model = sa.UNet(1, 11, layers=4, base_width=32).to(device).to(memory_format=CL).set_shard_halo(shard_halo)
        # clip_grad_norm_(1.0) + Adam (trainer.py:678-694); the update kernel also keeps the bf16 copies of the weights
        # the convolutions read under autocast, and they return fp32 weight gradients: no per-step casts either way
        opt = sa.FusedClipAdam(model.parameters(), lr=1e-3, max_norm=1.0, shadow_dtype=torch.bfloat16)
        return model, opt

    def step_fn(model, opt):
        def step():
            with torch.autocast("cuda", dtype=torch.bfloat16):
                logits = model(occ)
            loss = sa.ce_dice_loss(logits, lab)
            loss.backward()
            opt.step()
            opt.zero_grad(set_to_none=True)  # ScaFFold/utils/trainer.py:694
            return loss
        return step

    model, opt = make()
    step = step_fn(model, opt)
    ms = event_time_ms(step, 10, warmup=3)
    out = {"ms_per_step": ms, "input": "1x1x64x128x128 occupancy (5% ones), zero depth halo, padding (0,1,1)"}
    if eager_only:
        return out
    # The same arithmetic without the halo emulation's copies (depth padding 1 inside the kernels; bitwise the same
    # result): what remains is the cost of the step itself, the difference is the bench's stand-in for DistConv's
    # halo exchange.
    model_p, opt_p = make(shard_halo=False)
    out["ms_per_step_padded_form"] = event_time_ms(step_fn(model_p, opt_p), 10, warmup=3)
    del model_p, opt_p

    # The same step as one HIP graph. Checked before it is reported: from identical initial state, the losses of
    # four graph replays (with eager work and synchronisations between them) must equal those of four eager steps.
    try:
        model_e, opt_e = make()
        eager = step_fn(model_e, opt_e)
        eager_losses = [float(eager()) for _ in range(4)]
        model_g, opt_g = make()
        gstep = step_fn(model_g, opt_g)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                gstep()
        torch.cuda.current_stream().wait_stream(side)
        # back to the initial state before capture
        ref_model, _ = make()
        model_g.load_state_dict(ref_model.state_dict())
        for st in opt_g.state.values():
            for k, v in st.items():
                if torch.is_tensor(v):
                    v.zero_()
        opt_g.refresh_shadows()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_loss = gstep()
        graph_losses = []
        for _ in range(4):
            graph.replay()
            torch.cuda.synchronize()
            graph_losses.append(float(static_loss))
            _ = (occ * 2).sum().item()  # unrelated eager work between replays
        ok = all(abs(a - b) <= 1e-5 * max(1.0, abs(a)) for a, b in zip(eager_losses, graph_losses))
        out["graph_replay_matches_eager"] = ok
        out["graph_check_losses"] = {"eager": eager_losses, "graph": graph_losses}
        if ok:
            out["graph_ms_per_step"] = event_time_ms(graph.replay, 10, warmup=2)
    except Exception as exc:  # report, do not hide
        out["graph_error"] = repr(exc)
    return out


#: every 3x3x3 convolution of the config-5 step (base width 32, 5 levels) on the 64 x 128 x 128 depth shard, as
#: (Cin, Cout, interior extents); each runs on the (D + 2) x H x W slab at padding (0, 1, 1)
CFG5_CONVS = [
    (32, 32, (64, 128, 128)), (64, 32, (64, 128, 128)),
    (32, 64, (32, 64, 64)), (64, 64, (32, 64, 64)), (128, 64, (32, 64, 64)),
    (64, 128, (16, 32, 32)), (128, 128, (16, 32, 32)), (256, 128, (16, 32, 32)),
    (128, 256, (8, 16, 16)), (256, 256, (8, 16, 16)), (512, 256, (8, 16, 16)),
    (256, 512, (4, 8, 8)), (512, 512, (4, 8, 8)),
]
#: config 3 / config 4 shapes on full cubes at padding 1
CUBE_CONVS = [(32, 32, (128, 128, 128)), (32, 64, (64, 64, 64)), (64, 64, (64, 64, 64)), (128, 64, (64, 64, 64))]


def conv_table(device, iters=20):
    """Per-shape table of the MFMA convolution launches: every direction of every shape in a loop of its own
    (weights packed beforehand, outputs and workspaces allocated once), time per launch from HIP events, algorithmic
    FLOPs 2 * voxels * Cin * Cout * 27 and the fraction of the dense bf16 MFMA peak."""
    import scaffold_amd as sa

    rows = []
    for form, shapes in (("slab pad (0,1,1)", CFG5_CONVS), ("cube pad 1", CUBE_CONVS)):
        for cin, cout, sp in shapes:
            slab = form.startswith("slab")
            in_sp = (sp[0] + 2, sp[1], sp[2]) if slab else sp
            pad = (0, 1, 1) if slab else (1, 1, 1)
            g = torch.Generator().manual_seed(3000 + cin + cout)
            x = torch.randn((1, cin, *in_sp), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
            w = ((torch.rand((cout, cin, 3, 3, 3), generator=g) * 2 - 1) / math.sqrt(cin * 27)).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
            gy = torch.randn((1, cout, *sp), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
            flops = 2 * math.prod(sp) * cin * cout * 27
            pf, pd = sa.pack_weights(w, x.shape, 1, pad, 1)
            y, gx = torch.empty_like(gy), torch.empty_like(x)
            gw = torch.empty((cout, cin, 3, 3, 3), dtype=torch.float32, device=device).contiguous(memory_format=CL)
            fns = {
                "fwd": lambda: sa.conv3d_forward(x, w, None, 1, pad, 1, out=y, packed_weight=pf),
                "dgrad": lambda: sa.conv3d_backward_data(gy, w, x.shape, 1, pad, 1, out=gx, packed_weight=pd),
                "wgrad": lambda: sa.conv3d_backward_weight(x, w.shape, gy, 1, pad, 1, out=gw, grad_dtype=torch.float32),
            }
            for direction, fn in fns.items():
                fn()
                torch.cuda.synchronize()
                chunk = 10
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for _ in range(chunk):
                        fn()
                ms = event_time_ms(graph.replay, max(2, iters // chunk), warmup=1) / chunk
                rows.append({"form": form, "cin": cin, "cout": cout, "spatial": list(sp), "direction": direction, "us": ms * 1e3,
                             "gflop": flops / 1e9, "tflops": flops / (ms * 1e-3) / 1e12, "frac": flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS})
            del x, w, gy, y, gx, gw, pf, pd
    return rows


def cpu_baseline():
    """The reference's CPU path (torch conv3d + autograd, channels_last_3d bf16) on the bench workload itself,
    repeated for about 12 s of host time."""
    import torch.nn.functional as F

    cin = cout = 32
    spatial = (128, 128, 128)
    g = torch.Generator().manual_seed(3000)
    x = torch.randn((1, cin, *spatial), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).requires_grad_(True)
    w = (torch.randn((cout, cin, 3, 3, 3), generator=g) / math.sqrt(cin * 27)).to(torch.bfloat16).contiguous(memory_format=CL).requires_grad_(True)
    gy = torch.randn((1, cout, *spatial), generator=g).to(torch.bfloat16).contiguous(memory_format=CL)
    flops = 3 * 2 * math.prod(spatial) * cin * cout * 27

    def once():
        y = F.conv3d(x, w, None, 1, 1)
        torch.autograd.grad(y, (x, w), gy)

    once()
    times = []
    budget = time.perf_counter() + 12.0
    while len(times) < 5 or (time.perf_counter() < budget and len(times) < 500):
        t0 = time.perf_counter()
        once()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    return {
        "value": flops / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"torch CPU conv3d fwd+dgrad+wgrad, bf16 channels_last_3d, 32->32 3x3x3 on 128^3 (the whole workload), "
                  f"median of {len(times)} runs over {sum(times):.1f} s, {t * 1e3:.1f} ms each",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The chip's power management settles only after ~10 ms of sustained MFMA load (the first steps run at boost
    # clocks, the next ones well below the steady state): the default warm-up covers that transient.
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline leg")
    ap.add_argument("--skip-unet", action="store_true", help="omit the U-Net train step")
    ap.add_argument("--unet-profile", action="store_true",
                    help="run only 13 eager U-Net train steps (3 warm-up + 10) and print their time: the command to trace "
                         "when a per-kernel breakdown of the step is wanted")
    ap.add_argument("--ingest-profile", action="store_true",
                    help="run only the shard ingest kernel (200 launches) and print its time: the command to trace for it")
    ap.add_argument("--conv-table", action="store_true",
                    help="run only the per-shape table of the MFMA convolution launches (config 3 / 4 / 5 shapes, all directions)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch the plain copy kernel on 256 MiB (reference point for HBM counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (one process, one MI355X); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the hot path)", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    if args.ingest_profile:
        print(json.dumps({"shard_ingest": bench_ingest(args, device, iters=200)}))
        return
    if args.conv_table:
        rows = conv_table(device)
        for r in rows:
            print(f"{r['form']:17s} {r['cin']:4d}->{r['cout']:<4d} {'x'.join(str(v) for v in r['spatial']):>11s} {r['direction']:6s} "
                  f"{r['us']:8.1f} us {r['gflop']:8.2f} GFLOP {r['tflops']:7.1f} TFLOP/s {r['frac']:.3f}", file=sys.stderr)
        print(json.dumps({"conv_table": rows}))
        return
    if args.unet_profile:
        print(json.dumps({"unet_step_cfg5": bench_unet_step(args, device, eager_only=True)}))
        return
    conv = bench_conv(args, device)
    details = {"conv": conv}
    try:
        details["vendor_gemm_reference"] = gemm_reference(device)
    except Exception as exc:  # report, do not hide
        details["vendor_gemm_reference"] = {"error": repr(exc)}
    if args.copy_calibration:
        details["copy_calibration"] = copy_calibration(device)
    try:
        details["groupnorm_cfg2"] = bench_groupnorm(args, device)
    except Exception as exc:  # report, do not hide
        details["groupnorm_cfg2"] = {"error": repr(exc)}
    try:
        details["shard_ingest"] = bench_ingest(args, device)
    except Exception as exc:  # report, do not hide
        details["shard_ingest"] = {"error": repr(exc)}
    if not args.skip_unet:
        try:
            details["unet_step_cfg5"] = bench_unet_step(args, device)
        except Exception as exc:
            details["unet_step_cfg5"] = {"error": repr(exc)}
    flops = conv["flops_per_direction"]
    fwd_ms = conv["in_step_ms"]["fwd"]
    achieved = flops / (fwd_ms * 1e-3) / 1e12
    line = {
        "metric": "conv3d fwd+dgrad+wgrad TFLOP/s @128^3 bf16 (U-Net level-0 conv 32->32, 1 GPU)",
        "value": 3 * flops / (conv["ms_per_step"] * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": conv["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "conv3d 3x3x3 stride 1 pad 1, Cin=Cout=32, 128^3, N=1, NDHWC bf16: fwd + dgrad + wgrad "
                               "(BASELINE.json config 3, first encoder level)"},
        "roofline": {
            "bound": "mfma", "kernel": "conv_persist_kernel (forward)", "achieved": achieved, "peak": MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS, "traffic": CONV_FWD_HBM_TRAFFIC_BYTES,
            "flops_per_launch": flops, "avg_launch_ms": fwd_ms,
        },
        "cpu_baseline": None if args.skip_cpu else cpu_baseline(),
        "details": details,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
