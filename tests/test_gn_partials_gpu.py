"""GroupNorm statistics left by the producing convolution (``conv3d_forward(gn_groups=)``), through the C ABI.

What is held to what:
* the convolution's output is the same bits with and without the statistics;
* the Welford records (count, mean, M2 per producer workgroup and group), merged in fp64, are the count, mean and
  centred sum of squares of that output: the counts exactly (every voxel counted once, none past a ragged edge), mean
  and M2 to fp32 round-off, on integer-valued and on Gaussian draws;
* ``group_norm`` fed by them agrees with the stand-alone statistics pass to the last bit or so of the 16-bit output, and
  with the fp64 ``F.group_norm`` oracle within the tolerance of the GroupNorm parity tests;
* the records depend on the output alone: the FIRST call on a tensor whose mean is a thousand times its spread
  normalises correctly, eagerly and inside a captured graph, and a call gives the same bits whatever ran before it;
* a tensor changed in place after the convolution is not normalised with stale statistics.
"""

import pytest
import torch
import torch.nn.functional as F

import scaffold_amd as sa
from oracle import oracle as orc
from scaffold_amd import conv3d as c3
from scaffold_amd.unet import DoubleConv

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d

# (n, cin, cout, spatial, padding, groups, kernel that serves the forward)
CASES = [
    (1, 1, 32, (8, 16, 64), (1, 1, 1), 8, "direct"),           # the one-channel stem (thin-channel kernel on the matrix cores)
    (2, 1, 64, (5, 6, 70), (0, 1, 1), 4, "direct"),            # two samples, ragged, 64 channels
    (1, 32, 32, (8, 8, 32), (1, 1, 1), 8, "persist"),          # 4 channels per group: two groups per lane run pair
    (1, 32, 32, (5, 7, 33), (1, 1, 1), 4, "persist"),          # ragged tiles on every axis
    (1, 32, 64, (6, 9, 40), (0, 1, 1), 8, "persist"),          # shard form, two output blocks
    (1, 32, 128, (4, 8, 16), (1, 1, 1), 2, "persist"),         # a group wider than a workgroup's 32 channels
    (1, 32, 32, (10, 8, 8), (1, 1, 1), 8, "persist"),          # rows of 8
    (2, 64, 64, (16, 32, 64), (1, 1, 1), 8, "brick"),          # two samples, no slices
    (1, 64, 128, (32, 64, 32), (1, 1, 1), 8, "brick"),         # two output blocks per workgroup
    (1, 64, 96, (16, 32, 33), (1, 1, 1), 1, "brick"),          # a group wider than the workgroup's span, ragged rows
    (1, 64, 128, (16, 32, 31), (1, 1, 1), 2, "split"),         # small volume, reduction cut over the wavefronts: a group = the workgroup's 64 channels
    (1, 128, 256, (10, 16, 16), (0, 1, 1), 8, "split"),        # two groups per workgroup, shard form
    (1, 128, 256, (8, 16, 16), (1, 1, 1), 1, "split"),         # one group of all channels: four workgroups of a brick leave a record each
    (2, 256, 128, (5, 9, 21), (1, 1, 1), 32, "split"),         # 4 channels per group, two samples, ragged bricks
    (2, 64, 64, (9, 10, 16), (1, 1, 1), 16, "brick"),          # small volume: the reduction is sliced, the slice sum counts
    (1, 256, 512, (4, 8, 8), (1, 1, 1), 8, "brick"),           # deep level, sliced
    (1, 128, 256, (4, 8, 8), (1, 1, 1), 1, "brick"),           # sliced, one group of all channels (256 pieces merged per record)
    (1, 256, 256, (4, 8, 8), (1, 1, 1), 64, "brick"),          # sliced, 4 channels per group (a piece per row of the workgroup's 1024 elements)
    (1, 128, 64, (32, 64, 64), (0, 1, 1), 8, "wide"),          # 4 x 4 x 32 tiles
    (1, 128, 64, (63, 61, 65), (1, 1, 1), 16, "wide"),         # 8 x 4 x 32 tiles, ragged on every axis
    (1, 192, 64, (30, 62, 34), (1, 1, 1), 1, "wide"),          # one group of all 64 channels
]


def merged_records(partials, n, records, groups):
    """Count, mean and M2 per (sample, group) from the fp32 records, merged in fp64 with the k-way rule of Chan et al."""
    rec = partials.view(n, records, groups, 4).double()
    cnt, mean_r, m2_r = rec[..., 0], rec[..., 1], rec[..., 2]
    assert (rec[..., 3] == 0).all() and (cnt >= 0).all() and (m2_r >= 0).all()
    total = cnt.sum(1)
    mean = (cnt * mean_r).sum(1) / total
    m2 = (m2_r + cnt * (mean_r - mean[:, None]) ** 2).sum(1)
    return total, mean, m2


def group_moments(y, groups):
    n = y.shape[0]
    v = y.double().reshape(n, groups, -1)
    mean = v.mean(-1)
    return v.shape[-1], mean, ((v - mean[:, :, None]) ** 2).sum(-1), v.abs().amax(-1)


def check_records(y, groups, handoff):
    partials, records, g, version = handoff
    n = y.shape[0]
    assert g == groups and version == y._version and partials.numel() == n * records * groups * 4
    total, mean, m2 = merged_records(partials, n, records, groups)
    m, want_mean, want_m2, peak = group_moments(y, groups)
    assert (total == m).all(), "every voxel inside the tensor is counted exactly once"
    rms = (want_m2 / m).sqrt()
    assert ((mean - want_mean).abs() <= 2e-6 * (rms + 1e-3 * peak) + 1e-7).all(), (mean - want_mean).abs().max()
    assert ((m2 - want_m2).abs() <= 2e-5 * want_m2 + 1e-6 * m).all(), ((m2 - want_m2).abs() / want_m2).max()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,cin,cout,spatial,padding,groups,kernel", CASES)
def test_records_are_the_moments_of_the_output(device, dtype, n, cin, cout, spatial, padding, groups, kernel):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    geom = c3.launch_geometry(prob.input_shape, prob.weight_shape, 1, padding, 1, dtype, "fwd")
    assert geom["kernel"] == kernel, geom
    for exact in (True, False):
        ops = orc.make_inputs(prob, seed=3, exact=True, density=0.02) if exact else orc.make_inputs(prob, seed=3)
        x, w = ops["input"].to(device), ops["weight"].to(device)
        b = (torch.arange(cout) % 5 - 2).to(dtype).to(device)  # small integers: the outputs stay integer-valued
        plain = sa.conv3d_forward(x, w, b, 1, padding, 1)
        y = sa.conv3d_forward(x, w, b, 1, padding, 1, gn_groups=groups)
        assert torch.equal(plain, y), "the statistics must not change the convolution's result"
        assert not hasattr(plain, "_sfh_gn_partials")
        check_records(y, groups, y._sfh_gn_partials)


def _random_cases(count, seed):
    """Seeded random problems across the kernels that leave statistics: channel counts, group widths from 4 channels to
    the whole tensor, ragged extents around the tile sizes (8 / 16 / 32 voxel rows), one to three samples."""
    import random
    rng = random.Random(seed)
    cases = []
    while len(cases) < count:
        cin = rng.choice([1, 32, 32, 64, 64, 96, 128, 256])
        cout = rng.choice([32, 64, 96, 128, 256]) if cin != 1 else rng.choice([32, 64])
        cg = rng.choice([c for c in (4, 8, 16, 32, 64, 96, 128, 256) if cout % c == 0])
        w = rng.choice([rng.randint(3, 8), rng.randint(9, 16), rng.randint(17, 70)])
        d, h = rng.randint(1, 12), rng.randint(2, 20)
        n = rng.choice([1, 1, 2, 3])
        pad = rng.choice([(1, 1, 1), (0, 1, 1), (1, 1, 1), (2, 1, 0)])
        if d + 2 * pad[0] < 3 or h + 2 * pad[1] < 3 or w + 2 * pad[2] < 3 or n * cin * d * h * w > 6_000_000:
            continue
        cases.append((n, cin, cout, (d, h, w), pad, cout // cg))
    return cases


@pytest.mark.parametrize("n,cin,cout,spatial,padding,groups", _random_cases(48, seed=20240607))
def test_random_problems(device, n, cin, cout, spatial, padding, groups):
    """Whatever kernel serves the problem: the result is unchanged, and where statistics are left they are the moments of
    the (integer-valued) output; where they are not, nothing is attached."""
    dtype = torch.bfloat16
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    ops = orc.make_inputs(prob, seed=n + cin + cout, exact=True, density=0.05)
    x, w = ops["input"].to(device), ops["weight"].to(device)
    plain = sa.conv3d_forward(x, w, None, 1, padding, 1)
    y = sa.conv3d_forward(x, w, None, 1, padding, 1, gn_groups=groups)
    assert torch.equal(plain, y)
    geom = c3.launch_geometry(prob.input_shape, prob.weight_shape, 1, padding, 1, dtype, "fwd")
    handoff = getattr(y, "_sfh_gn_partials", None)
    if handoff is None:
        # not offered: several samples on the persistent kernel; a sliced reduction whose slice sum cannot keep a thread on
        # one group (1024 is not a multiple of the channel count); a thin-channel kernel other than the 32 / 64 channel stem
        assert (geom["kernel"] == "persist" and n > 1) or (geom["kernel"] == "brick" and geom["slices"] > 1 and 1024 % cout != 0) \
            or (geom["kernel"] == "direct" and cin != 1), (geom, n, cout)
        return
    check_records(y, groups, handoff)
    fused = sa.group_norm(y, groups, None, None, 1e-5, "relu", out_dtype=None)
    ref = F.relu(F.group_norm(y.double(), groups, None, None, 1e-5))
    assert orc.gn_rel_error(fused, ref) < 2e-2


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("n,cin,cout,spatial,padding,groups,kernel", CASES)
def test_group_norm_from_partials_matches_the_statistics_pass(device, n, cin, cout, spatial, padding, groups, kernel, relu):
    dtype = torch.bfloat16
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    ops = orc.make_inputs(prob, seed=11)
    x, w = ops["input"].to(device), ops["weight"].to(device)
    gamma = torch.linspace(0.5, 1.5, cout, device=device)
    beta = torch.linspace(-0.3, 0.3, cout, device=device)
    act = "relu" if relu else None
    y = sa.conv3d_forward(x, w, None, 1, padding, 1, gn_groups=groups)
    assert hasattr(y, "_sfh_gn_partials")
    fused = sa.group_norm(y, groups, gamma.to(dtype), beta.to(dtype), 1e-5, act, out_dtype=None)
    plain_y = y.clone(memory_format=torch.preserve_format)  # same bits, no statistics attached
    assert not hasattr(plain_y, "_sfh_gn_partials")
    separate = sa.group_norm(plain_y, groups, gamma.to(dtype), beta.to(dtype), 1e-5, act, out_dtype=None)
    # two routes to mean and rstd in fp32 (shifted and unshifted sums): the 16-bit outputs may differ in the last bit
    diff = (fused.float() - separate.float()).abs()
    assert (diff <= 2.0 ** -7 * separate.float().abs() + 1e-6).all(), diff.max()
    assert (diff > 0).float().mean() < 0.02, "more than a rounding's worth of elements differ"
    ref = F.group_norm(y.double(), groups, gamma.double(), beta.double(), 1e-5)
    ref = F.relu(ref) if relu else ref
    assert orc.gn_rel_error(fused, ref) < 2e-2


@pytest.mark.parametrize("n,cin,cout,spatial,padding,groups,kernel", [CASES[2], CASES[7], CASES[11], CASES[14], CASES[18], CASES[19]])
def test_large_mean_small_std_on_the_first_call(device, n, cin, cout, spatial, padding, groups, kernel):
    """A mean a thousand times the spread (fp16 resolves it; bf16 does not), the case of the reference's
    ``test_large_mean_small_std`` (tests/test_triton_group_norm.py:502-547): plain fp32 sums of y and y^2 lose the variance
    altogether there. The records must carry it on the FIRST call -- there is no earlier call to learn a shift from --
    and two calls in a row, with another tensor normalised in between, must give the same bits."""
    dtype = torch.float16
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    big = torch.full((cout,), 1000.0, dtype=dtype, device=device)
    ops = orc.make_inputs(prob, seed=6)
    x, w = ops["input"].to(device), (ops["weight"] * (1.0 / (cin * 27) ** 0.5)).to(dtype).to(device)
    y = sa.conv3d_forward(x, w, big, 1, padding, 1, gn_groups=groups)
    assert hasattr(y, "_sfh_gn_partials")
    check_records(y, groups, y._sfh_gn_partials)
    ref = F.group_norm(y.double(), groups, None, None, 1e-5)
    first = sa.group_norm(y, groups, None, None, 1e-5, None, out_dtype=torch.float32)
    assert orc.gn_rel_error(first, ref) < 2e-3
    # something else in between (an ordinary tensor through the same kernels), then the same call again
    other = sa.conv3d_forward(torch.randn_like(x), w, None, 1, padding, 1, gn_groups=groups)
    sa.group_norm(other, groups, None, None, 1e-5, None, out_dtype=torch.float32)
    y2 = sa.conv3d_forward(x, w, big, 1, padding, 1, gn_groups=groups)
    assert torch.equal(y2._sfh_gn_partials[0], y._sfh_gn_partials[0]), "the records are a function of the output alone"
    assert torch.equal(sa.group_norm(y2, groups, None, None, 1e-5, None, out_dtype=torch.float32), first)


def _runaway_block(device):
    """A DoubleConv in fp16 whose second convolution has a bias of 1000 on outputs of spread ~1."""
    torch.manual_seed(3)
    block = DoubleConv(32, 32, 8).to(device).to(memory_format=CL).half()
    conv = block.double_conv[3]
    with torch.no_grad():
        conv.weight.mul_(0.5)
    conv.bias = torch.nn.Parameter(torch.full((32,), 1000.0, dtype=torch.float16, device=device))
    seen = {}
    conv.register_forward_hook(lambda mod, args, out: seen.__setitem__("y", out.detach().clone()))
    return block, seen


def test_large_mean_small_std_through_double_conv(device):
    """The U-Net block as wired (each convolution leaves its GroupNorm's records): first call, eager."""
    block, seen = _runaway_block(device)
    x = torch.randn(1, 32, 8, 16, 32, device=device).half().contiguous(memory_format=CL)
    with torch.no_grad():
        out = block(x)
    y = seen["y"]
    spread = y.double().reshape(8, -1).std(-1)
    assert (y.double().mean() / spread.max()) > 300, "the draw must put the mean far above the spread"
    ref = F.relu(F.group_norm(y.double(), 8, block.double_conv[4].weight.double(), block.double_conv[4].bias.double(), 1e-5))
    assert orc.gn_rel_error(out, ref) < 3e-3  # fp16 output


def test_large_mean_small_std_inside_a_captured_graph(device):
    """The same block captured as a HIP graph: the captured launches take the same numeric route as eager ones, so
    every replay reproduces the eager bits (replayed three times with eager work and synchronisations between)."""
    block, seen = _runaway_block(device)
    x = torch.randn(1, 32, 8, 16, 32, device=device).half().contiguous(memory_format=CL)
    with torch.no_grad():
        eager = block(x).clone()
        y = seen["y"]  # the second convolution's output of this very call
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            block(x)  # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = block(x)
        for _ in range(3):
            captured.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(captured, eager)
            block(torch.randn_like(x))  # eager work between the replays
            torch.cuda.synchronize()
    ref = F.relu(F.group_norm(y.double(), 8, block.double_conv[4].weight.double(), block.double_conv[4].bias.double(), 1e-5))
    assert orc.gn_rel_error(eager, ref) < 3e-3


def test_statistics_follow_the_tensor_not_the_name(device):
    prob = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(8, 8, 32), padding=(1, 1, 1), dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=5)
    x, w = ops["input"].to(device), ops["weight"].to(device)
    y = sa.conv3d_forward(x, w, None, 1, 1, 1, gn_groups=8)
    y.add_(3.0)  # in place: the statistics on the tensor are stale now and must not be used
    got = sa.group_norm(y, 8, None, None, 1e-5, None, out_dtype=None)
    want = sa.group_norm(y.clone(memory_format=torch.preserve_format), 8, None, None, 1e-5, None, out_dtype=None)
    assert torch.equal(got, want)
    # another group count than announced: the ordinary pass as well
    y2 = sa.conv3d_forward(x, w, None, 1, 1, 1, gn_groups=8)
    assert torch.equal(sa.group_norm(y2, 4, None, None, 1e-5, None, out_dtype=None),
                       sa.group_norm(y2.clone(memory_format=torch.preserve_format), 4, None, None, 1e-5, None, out_dtype=None))


def test_where_the_statistics_are_not_offered(device):
    bf = torch.bfloat16
    # two samples on the persistent kernel, groups of two channels, fp32 tiles, direct kernels: plain forward, no attribute
    for n, cin, cout, groups, dtype in [(2, 32, 32, 8, bf), (1, 32, 32, 16, bf), (1, 32, 32, 8, torch.float32), (1, 3, 6, 2, bf)]:
        x = torch.randn(n, cin, 8, 8, 32, device=device).to(dtype).contiguous(memory_format=CL)
        w = torch.randn(cout, cin, 3, 3, 3, device=device).to(dtype)
        y = sa.conv3d_forward(x, w, None, 1, 1, 1, gn_groups=groups)
        assert not hasattr(y, "_sfh_gn_partials")
        assert torch.equal(y, sa.conv3d_forward(x, w, None, 1, 1, 1))


def test_double_conv_with_and_without_the_handoff(device):
    """The U-Net block: convolutions that announce their GroupNorm against the same block with the announcement off."""
    torch.manual_seed(0)
    block = DoubleConv(32, 64, 8).to(device).to(memory_format=CL)
    x = torch.randn(1, 32, 8, 16, 32, device=device).contiguous(memory_format=CL)
    assert block.double_conv[0].gn_groups == 8 and block.double_conv[3].gn_groups == 8
    assert set(block.state_dict()) == {f"double_conv.{i}.weight" for i in (0, 1, 3, 4)} | {f"double_conv.{i}.bias" for i in (1, 4)}

    def run():
        for p in block.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block(xi)
        out.float().square().mean().backward()
        return out.detach(), xi.grad, [p.grad.clone() for p in block.parameters()]

    fused = run()
    again = run()  # nothing is carried from call to call
    assert torch.equal(again[0], fused[0]) and torch.equal(again[1], fused[1])
    for conv in (block.double_conv[0], block.double_conv[3]):
        conv.gn_groups = 0
    separate = run()
    assert orc.gn_rel_error(fused[0], separate[0].double()) < 1e-2
    assert orc.gn_rel_error(fused[1], separate[1].double()) < 2e-2
    for a, b in zip(fused[2], separate[2]):
        assert orc.gn_rel_error(a, b.double()) < 2e-2
