"""GroupNorm statistics left by the producing convolution (``conv3d_forward(gn_groups=)``), through the C ABI.

What is held to what:
* the convolution's output is the same bits with and without the statistics;
* the partial sums, added up, equal the per-group sum and sum of squares of that output -- bit for bit on integer-valued
  draws (every voxel counted exactly once, none past a ragged edge), to fp32 round-off on Gaussian ones;
* ``group_norm`` fed by them agrees with the stand-alone statistics pass to the last bit or so of the 16-bit output, and
  with the fp64 ``F.group_norm`` oracle within the tolerance of the GroupNorm parity tests;
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
    (1, 64, 128, (16, 32, 33), (1, 1, 1), 2, "brick"),         # a group wider than the workgroup's span, ragged rows
    (2, 64, 64, (9, 10, 16), (1, 1, 1), 16, "brick"),          # small volume: the reduction is sliced, the slice sum counts
    (1, 256, 512, (4, 8, 8), (1, 1, 1), 8, "brick"),           # deep level, sliced
    (1, 128, 64, (32, 64, 64), (0, 1, 1), 8, "wide"),          # 4 x 4 x 32 tiles
    (1, 128, 64, (63, 61, 65), (1, 1, 1), 16, "wide"),         # 8 x 4 x 32 tiles, ragged on every axis
    (1, 192, 64, (30, 62, 34), (1, 1, 1), 1, "wide"),          # one group of all 64 channels
]


def group_sums(y, groups):
    n, c = y.shape[:2]
    v = y.double().reshape(n, groups, -1)
    return v.sum(-1), (v * v).sum(-1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,cin,cout,spatial,padding,groups,kernel", CASES)
def test_partials_are_the_sums_of_the_output(device, dtype, n, cin, cout, spatial, padding, groups, kernel):
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
        partials, records, g, version, _shift = y._sfh_gn_partials
        assert g == groups and version == y._version and not hasattr(plain, "_sfh_gn_partials")
        assert partials.numel() == n * records * 2 * groups
        got = partials.view(n, records, 2, groups).double().sum(1)  # fp64 sum of the fp32 records
        s1, s2 = group_sums(y, groups)
        if exact:
            # integer-valued outputs: every partial sum is exact in fp32, so the totals must be, too
            assert partials.max() < 2 ** 24 and s2.min() > 0, "the draw must keep every record inside the fp32 mantissa"
            assert torch.equal(got[:, 0], s1) and torch.equal(got[:, 1], s2), (got[:, 0] - s1, got[:, 1] - s2)
        else:
            scale = s2.sqrt() * (y[0].numel() / groups) ** 0.5  # |sum| <= sqrt(m * sum of squares)
            assert ((got[:, 0] - s1).abs() <= 1e-6 * scale + 1e-3).all()
            assert ((got[:, 1] - s2).abs() <= 1e-5 * s2 + 1e-3).all()


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
    """Whatever kernel serves the problem: the result is unchanged, and where statistics are left they are exactly the sums of
    the (integer-valued) output; where they are not, nothing is attached."""
    dtype = torch.bfloat16
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    ops = orc.make_inputs(prob, seed=n + cin + cout, exact=True, density=0.05)
    x, w = ops["input"].to(device), ops["weight"].to(device)
    shift = (torch.arange(n * groups, dtype=torch.float32, device=device).reshape(n, groups) % 3) - 1.0
    plain = sa.conv3d_forward(x, w, None, 1, padding, 1)
    y = sa.conv3d_forward(x, w, None, 1, padding, 1, gn_groups=groups, gn_shift=shift)
    assert torch.equal(plain, y)
    geom = c3.launch_geometry(prob.input_shape, prob.weight_shape, 1, padding, 1, dtype, "fwd")
    handoff = getattr(y, "_sfh_gn_partials", None)
    if handoff is None:
        # not offered: several samples on the persistent kernel; a sliced reduction whose slice sum cannot keep a thread on
        # one group (1024 is not a multiple of the channel count); a thin-channel kernel other than the 32 / 64 channel stem
        assert (geom["kernel"] == "persist" and n > 1) or (geom["kernel"] == "brick" and geom["slices"] > 1 and 1024 % cout != 0) \
            or (geom["kernel"] == "direct" and cin != 1), (geom, n, cout)
        return
    partials, records, g, _, kept = handoff
    assert g == groups and kept is shift and partials.numel() == n * records * 2 * groups
    got = partials.view(n, records, 2, groups).double().sum(1)
    v = y.double().reshape(n, groups, -1) - shift.double()[:, :, None]
    assert partials.abs().max() < 2 ** 24
    assert torch.equal(got[:, 0], v.sum(-1)) and torch.equal(got[:, 1], (v * v).sum(-1)), (geom, records)
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,cin,cout,spatial,padding,groups,kernel", [CASES[0], CASES[2], CASES[7], CASES[10], CASES[12], CASES[13]])
def test_sums_about_a_shift(device, dtype, n, cin, cout, spatial, padding, groups, kernel):
    """With a shift K per (sample, group) the records hold sums of (y - K) and (y - K)^2: exact on integer draws, and the
    normalisation then survives a mean a thousand times the spread, where plain fp32 sums have lost the variance."""
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    ops = orc.make_inputs(prob, seed=4, exact=True, density=0.02)
    x, w = ops["input"].to(device), ops["weight"].to(device)
    b = (torch.arange(cout) % 5 - 2).to(dtype).to(device)
    shift = (torch.arange(n * groups, dtype=torch.float32, device=device).reshape(n, groups) % 7) - 3.0  # integers
    y = sa.conv3d_forward(x, w, b, 1, padding, 1, gn_groups=groups, gn_shift=shift)
    assert torch.equal(y, sa.conv3d_forward(x, w, b, 1, padding, 1))
    partials, records, g, version, kept = y._sfh_gn_partials
    assert kept is shift
    got = partials.view(n, records, 2, groups).double().sum(1)
    v = y.double().reshape(n, groups, -1) - shift.double()[:, :, None]
    assert torch.equal(got[:, 0], v.sum(-1)) and torch.equal(got[:, 1], (v * v).sum(-1))
    # group_norm takes the shift from the tensor: same result as the statistics pass
    fused = sa.group_norm(y, groups, None, None, 1e-5, None, out_dtype=None)
    plain = sa.group_norm(y.clone(memory_format=torch.preserve_format), groups, None, None, 1e-5, None, out_dtype=None)
    diff = (fused.float() - plain.float()).abs()
    assert (diff <= 2.0 ** -7 * plain.float().abs() + 1e-6).all()

    if dtype is torch.float16 and kernel != "direct":
        # mean = 1000 x spread (fp16 resolves it; bf16 does not): a bias of 1000 on outputs of spread ~1
        big = torch.full((cout,), 1000.0, dtype=dtype, device=device)
        ops = orc.make_inputs(prob, seed=6)
        x, w = ops["input"].to(device), (ops["weight"] * (1.0 / (cin * 27) ** 0.5)).to(dtype).to(device)
        y0 = sa.conv3d_forward(x, w, big, 1, padding, 1)
        ref = F.group_norm(y0.double(), groups, None, None, 1e-5)
        near = y0.double().reshape(n, groups, -1).mean(-1).float() + 0.5   # "last call's means": close, not equal
        y1 = sa.conv3d_forward(x, w, big, 1, padding, 1, gn_groups=groups, gn_shift=near)
        good = sa.group_norm(y1, groups, None, None, 1e-5, None, out_dtype=torch.float32)
        assert orc.gn_rel_error(good, ref) < 2e-3
        y2 = sa.conv3d_forward(x, w, big, 1, padding, 1, gn_groups=groups)  # no shift: plain sums, the variance is noise
        poor = sa.group_norm(y2, groups, None, None, 1e-5, None, out_dtype=torch.float32)
        assert orc.gn_rel_error(poor, ref) > 10 * orc.gn_rel_error(good, ref)
        # ... but that call reports the means as the shift for the next one (they exceed 16 spreads), and the next is right
        nxt = poor._sfh_gn_shift
        assert nxt is not None and (nxt - 1000.0).abs().max() < 5.0
        y3 = sa.conv3d_forward(x, w, big, 1, padding, 1, gn_groups=groups, gn_shift=nxt)
        assert orc.gn_rel_error(sa.group_norm(y3, groups, None, None, 1e-5, None, out_dtype=torch.float32), ref) < 2e-3


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

    fused = run()       # first call: plain sums
    nxt = block.double_conv[1]._next_shift
    assert nxt is not None and nxt.shape == (1, 8) and not nxt.any(), "ordinary activations: no shift, so call after call gives the same bits"
    again = run()
    assert torch.equal(again[0], fused[0]) and torch.equal(again[1], fused[1])
    for conv in (block.double_conv[0], block.double_conv[3]):
        conv.gn_groups = 0
    separate = run()
    assert orc.gn_rel_error(fused[0], separate[0].double()) < 1e-2
    assert orc.gn_rel_error(fused[1], separate[1].double()) < 2e-2
    for a, b in zip(fused[2], separate[2]):
        assert orc.gn_rel_error(a, b.double()) < 2e-2
