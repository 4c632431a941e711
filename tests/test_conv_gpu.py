"""GPU parity of the conv3d family against the fp64 oracle, through the C ABI.

Standards, as in the reference's kernel suite (``triton_conv3d/reference.py:4-18``):
1. bitwise on {-1,0,1} operands whose sums are exactly representable (catches a wrong voxel / tap /
   channel, which a tolerance hides), each with the shapes that exercise partial tiles and padding forms;
2. the K/dtype-derived ``error_bound`` on Gaussian operands, plus the stated tolerance
   (fp32 1e-5 relative, bf16 2e-2 relative + 1e-2 absolute);
3. fp32 must really accumulate in fp32 (``max_abs < 1e-4 * peak``).
"""

import pytest
import torch
import torch.nn.functional as F

import scaffold_amd as sa
from oracle import oracle as orc
from scaffold_amd import conv3d as c3

pytestmark = pytest.mark.gpu

DIRS = ("fwd", "bwd-data", "bwd-weight")


def run(problem, ops, direction, device, **kw):
    x, w, gy = (ops[k].to(device) for k in ("input", "weight", "grad_output"))
    b = ops["bias"].to(device) if ops["bias"] is not None else None
    s, p = problem.stride, problem.padding
    if problem.transposed:
        if direction == "fwd":
            return sa.conv_transpose3d_forward(x, w, b, s, 0, 0, 1, 1, **kw)
        if direction == "bwd-data":
            return sa.conv_transpose3d_backward_data(gy, w, x.shape, s, 0, 0, 1, 1, **kw)
        return sa.conv_transpose3d_backward_weight(x, w.shape, gy, s, 0, 0, 1, 1, **kw)
    if direction == "fwd":
        return sa.conv3d_forward(x, w, b, s, p, 1, 1, **kw)
    if direction == "bwd-data":
        return sa.conv3d_backward_data(gy, w, x.shape, s, p, 1, 1, **kw)
    return sa.conv3d_backward_weight(x, w.shape, gy, s, p, 1, 1, **kw)


def check_exact(problem, direction, device, seed=0, **kw):
    """Bitwise standard; thins the activations until the fp64 result is exactly representable."""
    density = orc.exact_density(problem, direction)
    for _ in range(6):
        ops = orc.make_inputs(problem, seed=seed, exact=True, density=density)
        ref = orc.conv_reference(problem, ops, direction)
        if orc.is_exactly_representable(ref, problem.dtype):
            break
        density *= 0.5
    else:
        pytest.skip("no exactly representable draw")
    assert ref.abs().max() > 0, "degenerate draw"
    got = run(problem, ops, direction, device, **kw)
    rep = orc.compare(got, ref)
    assert rep.bitwise, f"{problem} [{direction}] {kw}: {rep}"
    return got


# --- shapes -------------------------------------------------------------------------------------
# MFMA-tiled: 3x3x3, stride 1, channels multiples of 32; spatial extents chosen to hit all three
# brick shapes (W > 16, 9..16, <= 8), partial tiles, and the three padding forms of a depth shard.
MFMA_SHAPES = [
    # (cin, cout, spatial, padding)
    (32, 32, (8, 8, 32), (1, 1, 1)),
    (32, 32, (5, 7, 33), (1, 1, 1)),
    (32, 64, (6, 9, 40), (0, 1, 1)),
    (64, 32, (6, 6, 18), (0, 0, 0)),
    (64, 64, (9, 10, 16), (1, 1, 1)),
    (32, 96, (4, 13, 13), (1, 1, 1)),
    (96, 32, (10, 8, 8), (1, 1, 1)),
    (32, 32, (3, 5, 7), (1, 1, 1)),
    (128, 64, (4, 4, 4), (1, 1, 1)),
    (32, 32, (2, 2, 2), (1, 1, 1)),
    (32, 32, (4, 6, 20), (2, 2, 2)),
    # deep, small-volume levels: the forward / data gradient cut the reduction channels into summed slices
    (256, 512, (4, 8, 8), (1, 1, 1)),
    (512, 256, (6, 8, 8), (0, 1, 1)),
    (128, 256, (8, 16, 16), (1, 1, 1)),
]


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("cin,cout,spatial,padding", MFMA_SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mfma_exact(device, dtype, cin, cout, spatial, padding, direction):
    if direction == "bwd-data" and any(p > 2 for p in padding):
        pytest.skip("p > k-1")
    prob = orc.ConvProblem(n=2 if spatial[2] < 30 else 1, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
    assert c3.uses_mfma(prob.input_shape, prob.weight_shape, 1, padding, 1, dtype, direction)
    got = check_exact(prob, direction, device)
    # the direct kernels must agree bit for bit on the same exact draw
    check_exact(prob, direction, device, force_generic=True)
    if direction == "bwd-weight":
        assert got.is_contiguous(memory_format=torch.channels_last_3d) or got.shape[2:] == (1, 1, 1)


# The brick-per-workgroup kernel's launch geometry is picked by a cost rule (512- or 256-voxel tiles of the row class,
# one or two 32-channel output blocks per workgroup, slices of the reduction channels on small volumes). One case per
# tile shape and block count, with the geometry the rule must give for it, so that no instantiation goes untested and a
# change of the rule shows up here.
GEOMETRY_CASES = [
    # (n, cin, cout, spatial, direction, voxels, blocks); planes of more than 32 x 32 voxels, or 96 channels: small
    # planes with blocks of 64 channels belong to the kernel that cuts the reduction inside the workgroup (SPLIT_CASES)
    (1, 64, 128, (32, 33, 32), "bwd-data", 512, 1),   # rows of 32: 4 x 4 x 32
    (1, 64, 128, (32, 64, 32), "fwd", 512, 2),
    (1, 64, 128, (32, 33, 32), "fwd", 256, 1),        # 2 x 4 x 32
    (1, 64, 128, (2, 128, 128), "fwd", 256, 2),
    (1, 64, 96, (16, 128, 16), "fwd", 512, 1),        # rows of 16: 4 x 8 x 16
    (1, 64, 64, (32, 256, 16), "fwd", 512, 2),
    (1, 64, 64, (4, 8, 16), "fwd", 256, 1),           # 2 x 8 x 16
    (1, 64, 128, (9, 192, 16), "fwd", 256, 2),
    (1, 64, 96, (24, 128, 8), "fwd", 512, 1),         # rows of 8: 8 x 8 x 8
    (1, 64, 128, (32, 256, 8), "fwd", 512, 2),
    (1, 128, 64, (4, 8, 8), "fwd", 256, 1),           # 4 x 8 x 8
    (1, 64, 128, (17, 192, 8), "fwd", 256, 2),
]


# Small volumes with 64 or more reduction channels and output channels in blocks of 64 go to the kernel that cuts the
# reduction over the wavefronts of a workgroup (64-voxel bricks, two output blocks): both round sizes (four chunks, two
# chunks), several rounds, ragged bricks on every axis, several samples, the padding forms of a depth shard -- and the
# edges of its launch rule (the plane bound, the workgroup bound, channel counts it does not take).
SPLIT_CASES = [
    # (n, cin, cout, spatial, padding, direction, kernel)
    (1, 128, 128, (16, 32, 32), (1, 1, 1), "fwd", "split"),       # a 16 x 32 x 32 level: one round of four chunks
    (1, 128, 128, (18, 32, 32), (0, 1, 1), "fwd", "split"),       # ... on a depth shard's slab
    (1, 128, 128, (18, 32, 32), (0, 1, 1), "bwd-data", "split"),  # ... and the data gradient onto the slab (18 planes)
    (1, 64, 128, (16, 32, 32), (1, 1, 1), "fwd", "split"),        # two chunks: the wavefront pairs share a chunk's k-steps
    (1, 128, 64, (7, 13, 35), (1, 1, 1), "bwd-data", "split"),    # two chunks, ragged on every axis
    (1, 256, 128, (9, 18, 27), (1, 1, 1), "fwd", "split"),        # two rounds of four chunks, ragged
    (1, 192, 128, (8, 16, 40), (1, 1, 1), "fwd", "split"),        # six chunks: three rounds of two
    (2, 512, 256, (4, 16, 16), (1, 1, 1), "fwd", "split"),        # four rounds, two samples
    (1, 512, 256, (8, 16, 16), (1, 1, 1), "fwd", "brick"),        # 512 channels to reduce for 32 workgroups per two planes: slices
    (3, 128, 192, (3, 9, 11), (2, 2, 2), "fwd", "split"),         # padding 2, three samples, three block pairs
    (1, 256, 256, (8, 16, 16), (1, 1, 1), "bwd-data", "split"),   # an 8 x 16 x 16 level
    (1, 128, 128, (40, 32, 32), (1, 1, 1), "fwd", "split"),       # whatever the depth: several rounds of workgroups
    (1, 128, 128, (6, 32, 33), (1, 1, 1), "fwd", "brick"),        # a plane of more than 32 x 32 voxels
    (1, 256, 192, (8, 16, 16), (1, 1, 1), "fwd", "split"),        # 24 workgroups per two planes: the fewest it takes
    (1, 256, 128, (8, 16, 16), (1, 1, 1), "fwd", "brick"),        # 16
    (1, 256, 512, (4, 8, 8), (1, 1, 1), "fwd", "brick"),          # 16 per two planes: too few, the brick kernel slices
    (1, 128, 96, (16, 32, 32), (1, 1, 1), "fwd", "brick"),        # 96 output channels are not blocks of 64
    (1, 96, 128, (16, 32, 32), (1, 1, 1), "fwd", "brick"),        # three chunks are not an even number
]


@pytest.mark.parametrize("n,cin,cout,spatial,padding,direction,kernel", SPLIT_CASES)
def test_small_volume_kernel_exact(device, n, cin, cout, spatial, padding, direction, kernel):
    for dtype in (torch.bfloat16, torch.float16):
        prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=dtype)
        geom = c3.launch_geometry(prob.input_shape, prob.weight_shape, 1, padding, 1, dtype, direction)
        assert geom["kernel"] == kernel, geom
        if kernel == "split":
            assert (geom["voxels"], geom["blocks"], geom["slices"]) == (64, 2, 1), geom
        check_exact(prob, direction, device)


def _small_volume_cases(count, seed):
    """Seeded random problems inside the small-volume kernel's launch rule: channel counts, one to three samples, extents
    around the 2 x 4 x 8 brick (ragged on any axis), the padding forms of a depth shard, both directions."""
    import random
    rng = random.Random(seed)
    cases = []
    while len(cases) < count:
        cin, cout = rng.choice([64, 128, 192, 256, 320]), rng.choice([64, 128, 192, 256])
        n = rng.choice([1, 1, 2, 3])
        d, h, w = rng.randint(1, 9), rng.randint(3, 32), rng.randint(3, 32)
        pad = rng.choice([(1, 1, 1), (0, 1, 1), (2, 1, 1), (1, 0, 2)])
        direction = rng.choice(["fwd", "bwd-data"])
        if min(d + 2 * pad[0], h + 2 * pad[1], w + 2 * pad[2]) < 3 or n * max(cin, cout) * (d + 2) * h * w > 3_000_000:
            continue
        geom = c3.launch_geometry((n, cin, d, h, w), (cout, cin, 3, 3, 3), 1, pad, 1, torch.bfloat16, direction)
        if geom["kernel"] == "split":
            cases.append((n, cin, cout, (d, h, w), pad, direction))
    return cases


@pytest.mark.parametrize("n,cin,cout,spatial,padding,direction", _small_volume_cases(32, seed=20250311))
def test_small_volume_kernel_random_problems_exact(device, n, cin, cout, spatial, padding, direction):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=torch.bfloat16)
    check_exact(prob, direction, device, seed=cin + cout + n)


@pytest.mark.parametrize("n,cin,cout,spatial,direction,voxels,blocks", GEOMETRY_CASES)
def test_brick_geometries_exact(device, n, cin, cout, spatial, direction, voxels, blocks):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=(1, 1, 1), dtype=torch.bfloat16)
    geom = c3.launch_geometry(prob.input_shape, prob.weight_shape, 1, (1, 1, 1), 1, torch.bfloat16, direction)
    assert (geom["kernel"], geom["voxels"], geom["blocks"]) == ("brick", voxels, blocks), geom
    check_exact(prob, direction, device)


# The column-walking kernels (32 reduction channels / any weight gradient at rows of more than 16 voxels) on volumes that
# make a workgroup take several columns one after the other (more columns than workgroups), long columns in several
# segments, and columns cut by every edge.
RING_WALKS = [
    # (n, cin, cout, spatial, padding)
    (2, 32, 32, (5, 130, 259), (1, 1, 1)),     # 2 x 17 x 9 = 306 columns of 8 rows for 256 workgroups
    (1, 32, 64, (3, 200, 170), (0, 1, 1)),     # two output blocks of 128 workgroups each, 150 columns, shard form
    (1, 32, 32, (45, 9, 33), (1, 1, 1)),       # 4 columns of 23 steps: cut into segments, ragged in every direction
    (3, 32, 96, (7, 17, 40), (2, 2, 2)),       # three blocks, padding 2
]


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("n,cin,cout,spatial,padding", RING_WALKS)
def test_column_walks_exact(device, n, cin, cout, spatial, padding, direction):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=torch.bfloat16)
    check_exact(prob, direction, device)
    # the data gradient of the mirrored problem runs the same kernel with the roles of the channel counts swapped
    if direction == "bwd-data" and cout != cin:
        check_exact(orc.ConvProblem(n=n, cin=cout, cout=cin, spatial=spatial, padding=padding, dtype=torch.bfloat16), direction, device)


def _random_tiled_problems(count, seed):
    """Seeded random 3x3x3 stride-1 problems with channel counts in multiples of 32: extents around the tile sizes, the
    three padding forms, one to three samples -- whatever geometry the launch rules pick for them."""
    import random
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        cin, cout = rng.choice([32, 64, 96, 128, 256]), rng.choice([32, 64, 96, 128, 256])
        w = rng.choice([rng.randint(3, 8), rng.randint(9, 16), rng.randint(17, 48)])
        d, h = rng.randint(2, 14), rng.randint(3, 24)
        n = rng.choice([1, 1, 2, 3])
        pad = rng.choice([(1, 1, 1), (0, 1, 1), (2, 2, 2), (1, 0, 2)])
        if min(d + 2 * pad[0], h + 2 * pad[1], w + 2 * pad[2]) < 3 or n * max(cin, cout) * d * h * w > 3_000_000:
            continue
        out.append((n, cin, cout, (d, h, w), pad))
    return out


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("n,cin,cout,spatial,padding", _random_tiled_problems(24, seed=77))
def test_random_tiled_problems_exact(device, n, cin, cout, spatial, padding, direction):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=torch.bfloat16)
    assert c3.uses_mfma(prob.input_shape, prob.weight_shape, 1, padding, 1, torch.bfloat16, direction)
    check_exact(prob, direction, device)


# Shapes only the direct kernels serve: odd channel counts, strides, dilation, other kernel sizes,
# fp32 (``triton_conv3d/shapes.py:611-684`` edge list).
DIRECT_SHAPES = [
    # (n, cin, cout, spatial, kernel, stride, padding, bias)
    (1, 3, 6, (13, 13, 13), (3, 3, 3), (1, 1, 1), (1, 1, 1), False),
    (2, 5, 7, (1, 8, 8), (1, 3, 3), (1, 1, 1), (0, 1, 1), True),
    (1, 17, 6, (2, 31, 3), (3, 3, 3), (1, 1, 1), (1, 1, 1), False),
    (3, 8, 8, (5, 6, 7), (3, 3, 3), (2, 2, 2), (1, 1, 1), True),
    (1, 16, 11, (6, 6, 6), (1, 1, 1), (1, 1, 1), (0, 0, 0), True),
    (1, 1, 32, (6, 7, 9), (3, 3, 3), (1, 1, 1), (1, 1, 1), False),
    (1, 4, 4, (2, 2, 2), (3, 3, 3), (1, 1, 1), (1, 1, 1), False),
    (1, 8, 4, (8, 8, 8), (2, 2, 2), (2, 2, 2), (0, 0, 0), False),
]


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("n,cin,cout,spatial,kernel,stride,padding,bias", DIRECT_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_direct_exact(device, dtype, n, cin, cout, spatial, kernel, stride, padding, bias, direction):
    if direction == "bwd-data" and stride != (1, 1, 1):
        pytest.skip("the data gradient is served at stride 1 only")
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, kernel=kernel, stride=stride, padding=padding,
                           bias=bias, dtype=dtype)
    check_exact(prob, direction, device)


# Thin-channel problems: the one-channel 3x3x3 / 2x2x2 stem forms and the 1x1x1 head forms (thin input,
# thin output), each also checked bit for bit against the direct kernels on the same draw.
THIN_SHAPES = [
    # (n, cin, cout, spatial, kernel, stride, padding, bias)
    (1, 1, 32, (9, 10, 21), (3, 3, 3), (1, 1, 1), (1, 1, 1), True),     # U-Net stem
    (2, 1, 32, (6, 12, 12), (3, 3, 3), (1, 1, 1), (0, 1, 1), False),    # stem of a depth shard
    (1, 1, 32, (5, 9, 70), (3, 3, 3), (1, 1, 1), (1, 1, 1), True),      # several LDS bricks, ragged in every axis
    (1, 1, 8, (3, 5, 130), (3, 3, 3), (1, 1, 1), (2, 0, 1), False),
    (1, 1, 64, (9, 9, 9), (3, 3, 3), (2, 2, 2), (1, 1, 1), False),
    (1, 1, 16, (8, 8, 8), (2, 2, 2), (2, 2, 2), (0, 0, 0), True),
    (1, 32, 11, (7, 9, 13), (1, 1, 1), (1, 1, 1), (0, 0, 0), True),     # U-Net head
    (2, 64, 3, (4, 5, 6), (1, 1, 1), (1, 1, 1), (0, 0, 0), False),
    (1, 11, 32, (5, 6, 7), (1, 1, 1), (1, 1, 1), (0, 0, 0), True),      # thin input, wide output
    (1, 32, 32, (4, 4, 9), (1, 1, 1), (1, 1, 1), (0, 0, 0), False),
    (1, 2, 8, (30, 30, 30), (1, 1, 1), (1, 1, 1), (0, 0, 0), False),    # several splits in the weight gradient
    (1, 128, 20, (3, 7, 11), (1, 1, 1), (1, 1, 1), (0, 0, 0), True),    # two 16-channel steps on the thin side
    (2, 20, 64, (6, 5, 9), (1, 1, 1), (1, 1, 1), (0, 0, 0), True),
    (1, 32, 11, (3, 43, 1), (1, 1, 1), (1, 1, 1), (0, 0, 0), False),    # 129 voxels: a round of one voxel
]


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("n,cin,cout,spatial,kernel,stride,padding,bias", THIN_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_thin_exact(device, dtype, n, cin, cout, spatial, kernel, stride, padding, bias, direction):
    if direction == "bwd-data" and stride != (1, 1, 1):
        pytest.skip("the data gradient is served at stride 1 only")
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, kernel=kernel, stride=stride, padding=padding,
                           bias=bias, dtype=dtype)
    got = check_exact(prob, direction, device)
    ref = check_exact(prob, direction, device, force_generic=True)
    assert torch.equal(got, ref)


def test_thin_gaussian_within_tolerance(device):
    """Head and stem at Gaussian operands: fp32 within 1e-5 relative, bf16 within 2e-2 relative + 1e-2 absolute."""
    for dtype in (torch.float32, torch.bfloat16):
        for cin, cout, k, pad in ((1, 32, 3, 1), (32, 11, 1, 0)):
            prob = orc.ConvProblem(n=1, cin=cin, cout=cout, spatial=(12, 16, 20), kernel=(k, k, k), padding=(pad, pad, pad),
                                   bias=True, dtype=dtype)
            ops = orc.make_inputs(prob, seed=21)
            for direction in DIRS:
                got = run(prob, ops, direction, device)
                orc.assert_baseline_tolerance(got, orc.conv_reference(prob, ops, direction), dtype)


def test_dilation_and_anisotropic_stride(device):
    x = torch.randint(-1, 2, (1, 4, 9, 10, 11), dtype=torch.float32)
    w = torch.randint(-1, 2, (5, 4, 3, 2, 3), dtype=torch.float32)
    ref = torch.nn.functional.conv3d(x.double(), w.double(), None, (1, 2, 1), (2, 0, 1), (2, 1, 1))
    got = sa.conv3d_forward(x.to(device).contiguous(memory_format=torch.channels_last_3d), w.to(device), None, (1, 2, 1),
                            (2, 0, 1), (2, 1, 1))
    assert torch.equal(got.cpu().double(), ref)


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mfma_gaussian_tolerance(device, dtype, direction):
    prob = orc.ConvProblem(n=1, cin=64, cout=64, spatial=(12, 20, 36), dtype=dtype)
    ops = orc.make_inputs(prob, seed=3)
    ops["weight"] = (ops["weight"].float() / (prob.cin * 27) ** 0.5).to(dtype)
    ref = orc.conv_reference(prob, ops, direction)
    got = run(prob, ops, direction, device)
    orc.assert_close(got, ref, prob, direction)
    if dtype is torch.bfloat16:
        orc.assert_baseline_tolerance(got, ref, dtype, f"{direction}")


@pytest.mark.parametrize("direction", DIRS)
def test_fp32_is_true_fp32(device, direction):
    """Benchmark configuration 1: 32->32 at 32^3 in fp32, fwd + dgrad + wgrad."""
    prob = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(32, 32, 32), dtype=torch.float32)
    g = torch.Generator().manual_seed(1000)
    x = torch.randn(prob.input_shape, generator=g).contiguous(memory_format=torch.channels_last_3d)
    bound = 1.0 / (prob.cin * 27) ** 0.5
    w = ((torch.rand(prob.weight_shape, generator=torch.Generator().manual_seed(1001)) * 2 - 1) * bound).contiguous(
        memory_format=torch.channels_last_3d)
    gy = torch.randn(prob.output_shape, generator=torch.Generator().manual_seed(1002)).contiguous(
        memory_format=torch.channels_last_3d)
    ops = {"input": x, "weight": w, "grad_output": gy, "bias": None}
    ref = orc.conv_reference(prob, ops, direction)
    got = run(prob, ops, direction, device)
    rep = orc.compare(got, ref)
    assert rep.max_abs < 1e-4 * ref.abs().max().item(), rep
    orc.assert_baseline_tolerance(got, ref, torch.float32, direction)


# fp32 problems of the tiled shape run on the fp32 matrix pipe (forward and data gradient); the reference runs them through
# its tiled kernel at input_precision="ieee" (`triton_conv3d/gather_gemm.py:1334`).
F32_TILE_SHAPES = [
    # (n, cin, cout, spatial, padding, direction): both brick shapes (4 x 4 x 32 when such workgroups fill the chip, else
    # 2 x 2 x 32), ragged extents, reductions of 1 / 2 / 3 / 4 chunks of 16 channels (the forward reduces over cin, the data
    # gradient over cout), the three padding forms of a depth shard
    (1, 32, 32, (8, 8, 32), (1, 1, 1), "fwd"),
    (1, 32, 32, (8, 8, 32), (1, 1, 1), "bwd-data"),
    (2, 16, 32, (5, 7, 33), (1, 1, 1), "fwd"),
    (2, 32, 16, (5, 7, 33), (1, 1, 1), "bwd-data"),
    (1, 48, 64, (6, 9, 40), (0, 1, 1), "fwd"),
    (1, 64, 48, (6, 9, 40), (0, 1, 1), "bwd-data"),
    (1, 32, 96, (4, 6, 20), (2, 2, 2), "fwd"),
    (1, 96, 32, (4, 6, 20), (2, 2, 2), "bwd-data"),
    (1, 64, 32, (3, 3, 5), (0, 0, 0), "fwd"),
    (1, 32, 64, (33, 34, 70), (1, 1, 1), "fwd"),
    (1, 32, 64, (33, 34, 70), (1, 1, 1), "bwd-data"),
    # weight gradient (both channel counts multiples of 32): split over output rows, odd row lengths, batch > 1
    (1, 32, 32, (8, 8, 32), (1, 1, 1), "bwd-weight"),
    (2, 32, 64, (5, 7, 33), (1, 1, 1), "bwd-weight"),
    (1, 64, 32, (6, 9, 40), (0, 1, 1), "bwd-weight"),
    (1, 32, 96, (4, 6, 21), (2, 2, 2), "bwd-weight"),
    (3, 64, 64, (3, 3, 5), (0, 0, 0), "bwd-weight"),
    (1, 32, 32, (1, 1, 1), (1, 1, 1), "bwd-weight"),
]


@pytest.mark.parametrize("n,cin,cout,spatial,padding,direction", F32_TILE_SHAPES)
def test_fp32_tiles_exact(device, n, cin, cout, spatial, padding, direction):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, padding=padding, dtype=torch.float32, bias=direction == "fwd")
    assert c3.uses_mfma(prob.input_shape, prob.weight_shape, 1, padding, 1, torch.float32, direction)
    check_exact(prob, direction, device)
    check_exact(prob, direction, device, force_generic=True)


@pytest.mark.parametrize("direction", DIRS)
def test_fp32_tiles_gaussian_is_true_fp32(device, direction):
    """Gaussian operands through the fp32 matrix pipe: 1e-5 relative to the fp64 oracle, i.e. no 16-bit or tf32-like rounding
    of operands or products anywhere (a bf16 product alone would be off by 4e-3)."""
    prob = orc.ConvProblem(n=1, cin=64, cout=64, spatial=(9, 13, 35), padding=(1, 1, 1), dtype=torch.float32, bias=direction == "fwd")
    ops = orc.make_inputs(prob, seed=21)
    ref = orc.conv_reference(prob, ops, direction)
    got = run(prob, ops, direction, device)
    orc.assert_baseline_tolerance(got, ref, torch.float32, f"fp32 tiles {direction}")


def test_fp32_tiles_step_aside_for_operands_off_the_16_byte_grid(device):
    """The fp32 tiles move 16-byte pieces of x, bias and y. A bias that is a view 4 bytes into its storage must not go
    down that path: the call is served (by the direct kernel) with the same result as the aligned call."""
    prob = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(6, 9, 33), padding=(1, 1, 1), dtype=torch.float32, bias=True)
    ops = orc.make_inputs(prob, seed=23, exact=True, density=0.05)
    x, w, b = (ops[k].to(device) for k in ("input", "weight", "bias"))
    aligned = sa.conv3d_forward(x, w, b, 1, 1, 1)
    store = torch.zeros(33, device=device)
    store[1:] = b
    off = store[1:]
    assert off.data_ptr() % 16 == 4
    assert torch.equal(sa.conv3d_forward(x, w, off, 1, 1, 1), aligned)
    ref = orc.conv_reference(prob, ops, "fwd")
    assert torch.equal(aligned.cpu().double(), ref.double())


# --- transposed convolution ---------------------------------------------------------------------
CONVT_SHAPES = [
    (1, 128, 64, (4, 4, 4), (2, 2, 2), True),
    (2, 64, 32, (3, 5, 6), (2, 2, 2), True),
    (1, 5, 7, (2, 3, 4), (2, 2, 2), False),
    (1, 8, 8, (2, 2, 3), (1, 2, 3), True),
    # the MFMA 2x2x2 family: every U-Net up-convolution channel pair, ragged voxel counts
    (1, 512, 256, (2, 3, 4), (2, 2, 2), True),
    (1, 256, 128, (3, 5, 7), (2, 2, 2), False),
    (1, 64, 32, (9, 6, 11), (2, 2, 2), True),
    (2, 64, 96, (4, 4, 5), (2, 2, 2), False),
    (1, 32, 32, (1, 1, 1), (2, 2, 2), True),
    # launches of a few workgroups take the one-tap-per-workgroup / unrolled forms: chunk counts that are not a multiple of the unroll
    (1, 160, 96, (2, 2, 3), (2, 2, 2), True),
    (1, 96, 160, (2, 3, 2), (2, 2, 2), False),
]


@pytest.mark.parametrize("direction", DIRS)
@pytest.mark.parametrize("n,cin,cout,spatial,kernel,bias", CONVT_SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_transposed_exact(device, dtype, n, cin, cout, spatial, kernel, bias, direction):
    prob = orc.ConvProblem(n=n, cin=cin, cout=cout, spatial=spatial, kernel=kernel, stride=kernel, padding=(0, 0, 0),
                           transposed=True, bias=bias, dtype=dtype)
    got = check_exact(prob, direction, device)
    assert tuple(got.shape) == {"fwd": prob.output_shape, "bwd-data": prob.input_shape, "bwd-weight": prob.weight_shape}[direction]
    # the direct kernels must give the same bits on the same exact draw
    assert torch.equal(got, check_exact(prob, direction, device, force_generic=True))


@pytest.mark.parametrize("direction", DIRS)
def test_transposed_gaussian_tolerance(device, direction):
    """cfg4's up-convolution (128 -> 64) at Gaussian operands, bf16: 2e-2 relative + 1e-2 absolute."""
    prob = orc.ConvProblem(n=1, cin=128, cout=64, spatial=(8, 8, 8), kernel=(2, 2, 2), stride=(2, 2, 2), padding=(0, 0, 0),
                           transposed=True, bias=True, dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=40)
    ops["weight"] = (ops["weight"].float() / (prob.cin * 8) ** 0.5).to(torch.bfloat16)
    got = run(prob, ops, direction, device)
    orc.assert_baseline_tolerance(got, orc.conv_reference(prob, ops, direction), torch.bfloat16, direction)


def test_transposed_bias_is_per_channel_not_per_tap(device):
    x = torch.zeros((1, 4, 2, 2, 2), dtype=torch.float32, device=device).contiguous(memory_format=torch.channels_last_3d)
    w = torch.zeros((4, 3, 2, 2, 2), dtype=torch.float32, device=device)
    b = torch.tensor([1.0, 2.0, 3.0], device=device)
    y = sa.conv_transpose3d_forward(x, w, b, 2)
    assert torch.equal(y, b.view(1, 3, 1, 1, 1).expand_as(y))


# --- layouts, out=, determinism -----------------------------------------------------------------
def test_weight_layouts_give_identical_bits(device):
    prob = orc.ConvProblem(n=1, cin=32, cout=64, spatial=(6, 8, 20), dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=5)
    x = ops["input"].to(device)
    w_cl = ops["weight"].to(device)                       # channels_last_3d
    w_std = w_cl.contiguous()                              # PyTorch default
    w_rsck = w_cl.permute(2, 3, 4, 1, 0).contiguous()      # (kd, kh, kw, Cin, Cout)
    y0 = sa.conv3d_forward(x, w_cl, None, 1, 1)
    y1 = sa.conv3d_forward(x, w_std, None, 1, 1)
    y2 = sa.conv3d_forward(x, w_cl, None, 1, 1, weight_rsck=w_rsck)
    assert torch.equal(y0, y1) and torch.equal(y0, y2)
    gy = ops["grad_output"].to(device)
    g0 = sa.conv3d_backward_data(gy, w_cl, x.shape, 1, 1)
    g1 = sa.conv3d_backward_data(gy, w_std, x.shape, 1, 1)
    g2 = sa.conv3d_backward_data(gy, w_cl, x.shape, 1, 1, weight_rsck=w_rsck)
    assert torch.equal(g0, g1) and torch.equal(g0, g2)


def test_ncdhw_input_is_converted_not_misread(device):
    prob = orc.ConvProblem(n=2, cin=32, cout=32, spatial=(4, 6, 10), dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=9, exact=True, density=0.3)
    ref = orc.conv_reference(prob, ops, "fwd")
    x_ncdhw = ops["input"].contiguous().to(device)
    assert not x_ncdhw.is_contiguous(memory_format=torch.channels_last_3d)
    y = sa.conv3d_forward(x_ncdhw, ops["weight"].to(device), None, 1, 1)
    assert y.is_contiguous(memory_format=torch.channels_last_3d)
    assert orc.compare(y, ref).bitwise


def test_weight_flip_matches_flipped_weight(device):
    prob = orc.ConvProblem(n=1, cin=8, cout=8, spatial=(5, 5, 5), dtype=torch.float32)
    ops = orc.make_inputs(prob, seed=2, exact=True)
    x, w = ops["input"].to(device), ops["weight"].to(device)
    y = sa.conv3d_forward(x, w, None, 1, 1, weight_flip=True)
    ref = torch.nn.functional.conv3d(ops["input"].double(), ops["weight"].double().flip(2, 3, 4), None, 1, 1)
    assert torch.equal(y.cpu().double(), ref)


def test_out_and_workspace_are_validated(device):
    prob = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(4, 4, 8), dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=1)
    x, w, gy = (ops[k].to(device) for k in ("input", "weight", "grad_output"))
    good = torch.empty(prob.output_shape, dtype=x.dtype, device=device, memory_format=torch.channels_last_3d)
    assert sa.conv3d_forward(x, w, None, 1, 1, out=good) is good
    with pytest.raises(ValueError):
        sa.conv3d_forward(x, w, None, 1, 1, out=torch.empty(prob.output_shape, dtype=x.dtype, device=device))  # NCDHW
    with pytest.raises(ValueError):
        sa.conv3d_forward(x, w, None, 1, 1, out=good[:, :16])
    with pytest.raises(ValueError):
        sa.conv3d_forward(x, w, None, 1, 1, out=good.float())
    with pytest.raises(ValueError):
        sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, workspace=torch.empty(8, dtype=torch.float32, device=device))
    with pytest.raises(ValueError):
        sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, out=torch.empty(w.shape, dtype=x.dtype, device=device).contiguous())
    splits = c3.split_count(x.shape, w.shape, 1, 1, 1, x.dtype)
    ws = torch.empty(c3.workspace_elements(splits, 32, 32, (3, 3, 3)), dtype=torch.float32, device=device)
    gw = sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, workspace=ws)
    assert torch.equal(gw, sa.conv3d_backward_weight(x, w.shape, gy, 1, 1))
    with pytest.raises(NotImplementedError):
        sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, deterministic=False)
    with pytest.raises(NotImplementedError):
        sa.conv3d_backward_data(gy, w, x.shape, 2, 1)
    with pytest.raises(NotImplementedError):
        sa.conv3d_forward(x.cpu(), w.cpu(), None, 1, 1)


def test_same_call_same_bits(device):
    prob = orc.ConvProblem(n=1, cin=64, cout=64, spatial=(8, 16, 40), dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=4)
    outs = []
    for _ in range(3):
        # scratch comes from torch.empty: poison the allocator's free blocks between calls
        junk = torch.full((1 << 22,), float("nan"), device=device)
        del junk
        outs.append(tuple(run(prob, ops, d, device).clone() for d in DIRS))
    for o in outs[1:]:
        for a, b in zip(outs[0], o):
            assert torch.equal(a, b)


def test_empty_batch_forward(device):
    x = torch.empty((0, 32, 4, 4, 4), dtype=torch.bfloat16, device=device).contiguous(memory_format=torch.channels_last_3d)
    w = torch.empty((32, 32, 3, 3, 3), dtype=torch.bfloat16, device=device)
    assert sa.conv3d_forward(x, w, None, 1, 1).shape == (0, 32, 4, 4, 4)


# --- shard boundary -----------------------------------------------------------------------------
def test_depth_shard_with_halo_equals_slice_of_full_volume(device):
    """A (D_loc + 2) x H x W slab convolved at padding (0,1,1) is the D-slice of the full-volume
    convolution (``tests/helpers/rank_scripts/conv3d_shards_2rank.py:96-98`` without the second rank)."""
    prob = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(16, 12, 20), dtype=torch.bfloat16)
    ops = orc.make_inputs(prob, seed=8, exact=True, density=0.25)
    full = orc.conv_reference(prob, ops, "fwd")
    if not orc.is_exactly_representable(full, torch.bfloat16):
        pytest.skip("draw not exact")
    x, w = ops["input"], ops["weight"].to(device)
    lo = torch.cat([torch.zeros_like(x[:, :, :1]), x[:, :, :9]], dim=2).contiguous(memory_format=torch.channels_last_3d)
    hi = torch.cat([x[:, :, 7:], torch.zeros_like(x[:, :, :1])], dim=2).contiguous(memory_format=torch.channels_last_3d)
    y_lo = sa.conv3d_forward(lo.to(device), w, None, 1, (0, 1, 1))
    y_hi = sa.conv3d_forward(hi.to(device), w, None, 1, (0, 1, 1))
    assert torch.equal(torch.cat([y_lo, y_hi], dim=2).cpu().double(), full)


# --- full size: properties that do not need the CPU oracle --------------------------------------
def test_full_size_128cube_properties(device):
    """The headline conv (32 -> 32, 3x3x3, 128^3, bf16) on the exact standard: the fp64 oracle would
    take minutes on the host, so the full-size launch is pinned by size-independent properties.  Operands are
    in {-1,0,1}, thinned so every partial sum is an integer below 2^8 and the results are exact in bf16:
    (1) the tiled MFMA kernels agree bitwise with the untiled direct kernels (two independent index paths,
        the direct ones pinned against the oracle at small sizes above);
    (2) the three directions are adjoint to one another exactly: <fwd(x), g> = <x, dgrad(g)> = <w, wgrad(x, g)>;
    (3) the top-left corner equals the oracle on that corner's receptive field."""
    prob = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(128, 128, 128), dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(128)
    shape = (1, 32, 128, 128, 128)
    cl = torch.channels_last_3d

    def draw(shp, density):
        keep = torch.rand(shp, generator=g) < density
        sign = torch.randint(0, 2, shp, generator=g) * 2 - 1
        return (keep * sign).to(torch.bfloat16)

    x = draw(shape, 0.02).contiguous(memory_format=cl).to(device)
    gy = draw(shape, 0.02).contiguous(memory_format=cl).to(device)
    w = draw((32, 32, 3, 3, 3), 0.5).contiguous(memory_format=cl).to(device)

    y = sa.conv3d_forward(x, w, None, 1, 1)
    gx = sa.conv3d_backward_data(gy, w, x.shape, 1, 1)
    gw = sa.conv3d_backward_weight(x, w.shape, gy, 1, 1)
    assert c3.uses_mfma(x.shape, w.shape, 1, 1, 1, torch.bfloat16, "fwd")
    assert y.abs().max() > 0 and y.abs().max() < 256 and gx.abs().max() < 256
    # the weight gradient sums over 2M voxels: exact only while it stays below 2^8 in bf16
    assert gw.abs().max() <= 256, "draw too dense for an exact bf16 weight gradient"

    y_d = sa.conv3d_forward(x, w, None, 1, 1, force_generic=True)
    gx_d = sa.conv3d_backward_data(gy, w, x.shape, 1, 1, force_generic=True)
    assert torch.equal(y, y_d)
    assert torch.equal(gx, gx_d)

    # The weight gradient the same way: every product is in {-1, 0, 1} and a sum over the 2M voxels stays far below 2^24,
    # so fp32 accumulation is exact in ANY order -- the split-K MFMA kernel + ordered slice sum and the untiled kernel
    # (a workgroup per (output channel, tap), LDS tree) must round the same integer and agree in all 27,648 elements.
    gw_d = sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, force_generic=True)
    assert torch.equal(gw, gw_d)
    # ... and the unrounded fp32 form (what an fp32 master weight receives) is that integer itself
    gw32 = sa.conv3d_backward_weight(x, w.shape, gy, 1, 1, grad_dtype=torch.float32)
    assert gw32.dtype is torch.float32 and torch.equal(gw32, gw32.round()) and torch.equal(gw32.to(torch.bfloat16), gw)
    # a sub-volume against the fp64 oracle: the gradient of the first 8 x 16 x 128 output rows alone (gy zero elsewhere)
    gy_sub = torch.zeros_like(gy)
    gy_sub[:, :, :8, :16, :] = gy[:, :, :8, :16, :]
    gw_sub = sa.conv3d_backward_weight(x, w.shape, gy_sub, 1, 1, grad_dtype=torch.float32)
    sub = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(10, 18, 128), padding=(0, 0, 1), dtype=torch.bfloat16)
    xs = F.pad(x[:, :, :9, :17, :].cpu().float(), (0, 0, 1, 0, 1, 0)).contiguous(memory_format=cl)   # the volume's zero padding at d = h = -1
    ref = orc.conv_reference(sub, {"input": xs, "weight": w.cpu(), "bias": None,
                                   "grad_output": gy[:, :, :8, :16, :].cpu().contiguous(memory_format=cl)}, "bwd-weight")
    assert torch.equal(gw_sub.cpu().double(), ref)

    lhs = (y.double() * gy.double()).sum().item()
    mid = (x.double() * gx.double()).sum().item()
    rhs = (w.double() * gw32.double()).sum().item()
    assert lhs == mid == rhs

    corner = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(10, 10, 40), dtype=torch.bfloat16)
    xc = x[:, :, :10, :10, :40].cpu().contiguous(memory_format=cl)
    ref = orc.conv_reference(corner, {"input": xc, "weight": w.cpu(), "bias": None, "grad_output": None}, "fwd")
    assert torch.equal(y[:, :, :9, :9, :39].cpu().double(), ref[:, :, :9, :9, :39])


# --- wide-tile kernel (a 64-channel output from 128 or more reduction channels, rows of more than 16 voxels) ---------
# (cin, cout, spatial, padding, direction): the forward reduces over cin and produces cout, the data gradient the
# reverse. Both accumulator grids of the kernel (8 sub-tiles x 2 channel blocks when such workgroups fill the chip, else
# 4 x 2), ragged edges in all three extents, a reduction of 12 chunks, and the depth-slab padding form.
WIDE_SHAPES = [
    (128, 64, (63, 61, 65), (1, 1, 1), "fwd"),
    (64, 128, (63, 61, 65), (1, 1, 1), "bwd-data"),
    (128, 64, (32, 64, 64), (0, 1, 1), "fwd"),
    (64, 128, (30, 62, 34), (1, 1, 1), "bwd-data"),
    (192, 64, (30, 62, 34), (1, 1, 1), "fwd"),
]


@pytest.mark.parametrize("cin,cout,spatial,padding,direction", WIDE_SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_wide_tile_exact(device, dtype, cin, cout, spatial, padding, direction):
    """Exact standard at sizes the fp64 oracle does not finish in seconds: operands in {-1, 0, 1}, thinned so every
    partial sum is a small integer. The tiled kernel must agree bit for bit with the untiled direct kernel (an
    independent index path, itself held to the oracle at small sizes), with the oracle on the corner block of the
    volume, and the two directions must be exactly adjoint."""
    cl = torch.channels_last_3d
    g = torch.Generator().manual_seed(cin * 1000 + cout)
    out_sp = tuple(spatial[i] + 2 * padding[i] - 2 for i in range(3))

    def draw(shp, density):
        keep = torch.rand(shp, generator=g) < density
        sign = torch.randint(0, 2, shp, generator=g) * 2 - 1
        return (keep * sign).to(dtype)

    x = draw((1, cin, *spatial), 0.05).contiguous(memory_format=cl).to(device)
    gy = draw((1, cout, *out_sp), 0.05).contiguous(memory_format=cl).to(device)
    w = draw((cout, cin, 3, 3, 3), 0.5).contiguous(memory_format=cl).to(device)
    assert c3.uses_mfma(x.shape, w.shape, 1, padding, 1, dtype, direction)
    if direction == "fwd":
        got = sa.conv3d_forward(x, w, None, 1, padding, 1)
        ref_direct = sa.conv3d_forward(x, w, None, 1, padding, 1, force_generic=True)
    else:
        got = sa.conv3d_backward_data(gy, w, x.shape, 1, padding, 1)
        ref_direct = sa.conv3d_backward_data(gy, w, x.shape, 1, padding, 1, force_generic=True)
    assert got.abs().max() > 0 and got.abs().max() < 256
    assert torch.equal(got, ref_direct)
    # corner block against the oracle: outputs that depend on the first 10 x 10 x 40 input voxels only
    if direction == "fwd":
        corner = orc.ConvProblem(n=1, cin=cin, cout=cout, spatial=(10, 10, 40), padding=padding, dtype=dtype)
        xc = x[:, :, :10, :10, :40].cpu().contiguous(memory_format=cl)
        ref = orc.conv_reference(corner, {"input": xc, "weight": w.cpu(), "bias": None, "grad_output": None}, "fwd")
        d, h, wd = (ref.shape[2] - 1, ref.shape[3] - 1, ref.shape[4] - 1)
        assert torch.equal(got[:, :, :d, :h, :wd].cpu().double(), ref[:, :, :d, :h, :wd])
        # adjointness with the data gradient: <fwd(x), g> = <x, dgrad(g)>, exactly (small integers)
        gx = sa.conv3d_backward_data(gy, w, x.shape, 1, padding, 1)
        assert (got.double() * gy.double()).sum().item() == (x.double() * gx.double()).sum().item()
    else:
        # gradient of the corner outputs alone, against the oracle on that corner's receptive field
        gy_c = torch.zeros_like(gy)
        gy_c[:, :, :6, :6, :30] = gy[:, :, :6, :6, :30]
        got_c = sa.conv3d_backward_data(gy_c, w, x.shape, 1, padding, 1)
        in_c = tuple(6 + 2 - 2 * padding[i] if i < 2 else 30 + 2 - 2 * padding[i] for i in range(3))
        corner = orc.ConvProblem(n=1, cin=cin, cout=cout, spatial=in_c, padding=padding, dtype=dtype)
        ops = {"input": torch.zeros((1, cin, *in_c), dtype=dtype).contiguous(memory_format=cl), "weight": w.cpu(), "bias": None,
               "grad_output": gy[:, :, :6, :6, :30].cpu().contiguous(memory_format=cl)}
        ref = orc.conv_reference(corner, ops, "bwd-data")
        # away from the cut faces of the corner problem its data gradient is the full problem's
        d, h, wd = in_c[0] - 2, in_c[1] - 2, in_c[2] - 2
        assert torch.equal(got_c[:, :, :d, :h, :wd].cpu().double(), ref[:, :, :d, :h, :wd])
        assert got_c[:, :, in_c[0] + 1:].abs().max() == 0


@pytest.mark.parametrize("direction", ["fwd", "bwd-data"])
def test_wide_tile_bias_and_gaussian_tolerance(device, direction):
    """Gaussian operands (and a bias in the forward) through the wide-tile kernel at a size that selects it; held to
    the bf16 tolerance of the fp64 oracle on the corner block of the volume (the oracle on the whole volume takes minutes)."""
    cl = torch.channels_last_3d
    cin, cout = (128, 64) if direction == "fwd" else (64, 128)
    full = orc.ConvProblem(n=1, cin=cin, cout=cout, spatial=(32, 64, 64), padding=(1, 1, 1), dtype=torch.bfloat16, bias=direction == "fwd")
    ops = orc.make_inputs(full, seed=11)
    x, w, gy = (ops[k].to(device) for k in ("input", "weight", "grad_output"))
    corner = orc.ConvProblem(n=1, cin=cin, cout=cout, spatial=(10, 10, 40), padding=(1, 1, 1), dtype=torch.bfloat16, bias=full.bias)
    if direction == "fwd":
        got = sa.conv3d_forward(x, w, ops["bias"].to(device), 1, 1, 1)
        ref = orc.conv_reference(corner, {"input": ops["input"][:, :, :10, :10, :40].contiguous(memory_format=cl), "weight": ops["weight"],
                                          "bias": ops["bias"], "grad_output": None}, "fwd")
        orc.assert_baseline_tolerance(got[:, :, :9, :9, :39], ref[:, :, :9, :9, :39], torch.bfloat16, "wide fwd")
    else:
        gy_c = torch.zeros_like(gy)
        gy_c[:, :, :10, :10, :40] = gy[:, :, :10, :10, :40]
        got = sa.conv3d_backward_data(gy_c, w, x.shape, 1, 1, 1)
        ref = orc.conv_reference(corner, {"input": ops["input"][:, :, :10, :10, :40].contiguous(memory_format=cl), "weight": ops["weight"], "bias": None,
                                          "grad_output": ops["grad_output"][:, :, :10, :10, :40].contiguous(memory_format=cl)}, "bwd-data")
        orc.assert_baseline_tolerance(got[:, :, :10, :10, :40], ref, torch.bfloat16, "wide bwd-data")


# --- bias gradient --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 11, 7, 9, 13), (2, 32, 4, 5, 6), (1, 300, 2, 3, 3), (1, 1, 5, 5, 5), (1, 64, 33, 32, 31)])
def test_bias_grad_matches_sum(device, dtype, shape):
    """``grad_output.sum((0, 2, 3, 4))`` (``ScaFFold/unet/conv3d.py:1231``): bitwise on integer-valued gradients whose
    sums are exactly representable, within the dtype's rounding of an fp64 sum on Gaussian ones."""
    g = torch.Generator().manual_seed(7)
    exact = torch.randint(-1, 2, shape, generator=g).to(dtype)
    keep = torch.rand(shape, generator=g) < min(1.0, 100.0 / (shape[2] * shape[3] * shape[4]))
    exact = (exact * keep).contiguous(memory_format=torch.channels_last_3d)
    ref = exact.double().sum((0, 2, 3, 4))
    got = sa.bias_grad(exact.to(device), torch.float32)
    assert got.dtype is torch.float32 and torch.equal(got.cpu().double(), ref)
    if orc.is_exactly_representable(ref, dtype):
        assert torch.equal(sa.bias_grad(exact.to(device)).cpu().double(), ref)
    gauss = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=torch.channels_last_3d)
    ref = gauss.double().sum((0, 2, 3, 4))
    got = sa.bias_grad(gauss.to(device), torch.float32).cpu().double()
    assert (got - ref).abs().max() <= 1e-5 * gauss.double().abs().sum((0, 2, 3, 4)).max()
    # an NCDHW-contiguous gradient is converted, not misread
    assert torch.equal(sa.bias_grad(gauss.contiguous().to(device), torch.float32).cpu().double(), got)
    # same call, same bits
    assert torch.equal(sa.bias_grad(gauss.to(device), torch.float32).cpu().double(), got)


# ---- packing a weight once for both directions -------------------------------------------------------------------
CL = torch.channels_last_3d

@pytest.mark.parametrize("cin,cout,sp,pad", [
    (32, 32, (8, 16, 32), (1, 1, 1)),      # persistent kernel
    (32, 64, (6, 16, 32), (0, 1, 1)),      # shard form
    (64, 32, (8, 16, 32), (1, 1, 1)),      # brick-per-workgroup kernel
    (256, 256, (4, 8, 8), (1, 1, 1)),      # reduction channels cut into slices (partial workspace beside the weight)
])
def test_prepacked_weight_gives_the_same_bits(device, cin, cout, sp, pad):
    g = torch.Generator().manual_seed(61)
    x = torch.randn((1, cin, *sp), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    w = (torch.randn((cout, cin, 3, 3, 3), generator=g) * 0.05).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    y = sa.conv3d_forward(x, w, None, 1, pad, 1)
    gy = torch.randn(y.shape, generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    gx = sa.conv3d_backward_data(gy, w, x.shape, 1, pad, 1)
    pf, pd = sa.pack_weights(w, x.shape, 1, pad, 1)
    assert pf is not None and pd is not None
    assert (pf.numel(), pd.numel()) == sa.packed_weight_bytes(x.shape, w.shape, 1, pad, 1, w.dtype)
    assert torch.equal(sa.conv3d_forward(x, w, None, 1, pad, 1, packed_weight=pf), y)
    assert torch.equal(sa.conv3d_backward_data(gy, w, x.shape, 1, pad, 1, packed_weight=pd), gx)
    only_f, none_d = sa.pack_weights(w, x.shape, 1, pad, 1, backward_data=False)
    assert none_d is None and torch.equal(only_f, pf)


@pytest.mark.parametrize("cin_t,cout_t,sp", [(64, 32, (4, 6, 8)), (128, 64, (3, 4, 5)), (32, 32, (2, 2, 16))])
def test_prepacked_weight_of_the_up_convolution_gives_the_same_bits(device, cin_t, cout_t, sp):
    """The 2x2x2 stride-2 pair: the transposed convolution reads the data-gradient form, its own data gradient (a
    stride-2 convolution) the forward form, of ``pack_weights`` for the stride-2 problem over the up-convolution's output."""
    g = torch.Generator().manual_seed(71)
    x = torch.randn((1, cin_t, *sp), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    w = (torch.randn((cin_t, cout_t, 2, 2, 2), generator=g) * 0.1).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    b = torch.randn(cout_t, generator=g).to(torch.bfloat16).to(device)
    y = sa.conv_transpose3d_forward(x, w, b, 2)
    gy = torch.randn(y.shape, generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    gx = sa.conv_transpose3d_backward_data(gy, w, x.shape, 2)
    pf, pd = sa.pack_weights(w, y.shape, 2, 0, 1)
    assert pf is not None and pd is not None
    assert torch.equal(sa.conv_transpose3d_forward(x, w, b, 2, packed_weight=pd), y)
    assert torch.equal(sa.conv_transpose3d_backward_data(gy, w, x.shape, 2, packed_weight=pf), gx)
    assert torch.equal(sa.conv3d_forward(gy, w, None, 2, 0, 1, packed_weight=pf), gx)


def test_batch_packing_gives_the_same_bits(device):
    """Many weights packed in a few launches (more jobs than one launch's table holds), also on a second run of the
    same plan after the weights changed in place, and with layouts and dtypes mixed."""
    from scaffold_amd import conv3d as C
    g = torch.Generator().manual_seed(67)
    packs = []
    for i in range(11):
        cin, cout = (32, 64, 96)[i % 3], (64, 32, 128)[i % 3]
        dtype = torch.float16 if i % 4 == 3 else torch.bfloat16
        w = (torch.randn((cout, cin, 3, 3, 3), generator=g) * 0.05).to(dtype).to(device)
        if i % 2 == 0:
            w = w.contiguous(memory_format=CL)
        packs.append(C.PackedWeights(w, (1, cin, 4 + i, 8, 16), 1, 1, 1))
    packs.append(C.PackedWeights(torch.randn((7, 5, 3, 3, 3), device=device).to(torch.bfloat16), (1, 5, 8, 8, 8), 1, 1, 1))
    assert not packs[-1] and all(packs[:-1])
    plan = None
    for round_ in range(2):
        want = [sa.pack_weights(e.source, e.problem[0], 1, 1, 1) for e in packs[:-1]]
        for e in packs[:-1]:
            e.fwd.zero_(), e.dgrad.zero_()
        plan = C.pack_weights_batch(packs if plan is None else plan)
        for e, (pf, pd) in zip(packs, want):
            assert torch.equal(e.fwd, pf) and torch.equal(e.dgrad, pd)
        for e in packs[:-1]:
            e.source.mul_(-0.5)


def test_pack_weights_declines_problems_that_read_the_weight_where_it_lies(device):
    w5 = torch.randn((7, 5, 3, 3, 3), device=device).to(torch.bfloat16)
    assert sa.pack_weights(w5, (1, 5, 8, 8, 8), 1, 1, 1) == (None, None)
    w32 = torch.randn((32, 32, 3, 3, 3), device=device)           # fp32: true fp32 kernels, no MFMA packing
    assert sa.pack_weights(w32, (1, 32, 8, 8, 8), 1, 1, 1) == (None, None)
    wb = w32.to(torch.bfloat16).contiguous(memory_format=CL)
    x = torch.randn((1, 32, 8, 8, 8), device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    pf, _ = sa.pack_weights(wb, x.shape, 1, 1, 1)
    with pytest.raises(ValueError):
        sa.conv3d_forward(x, wb, None, 1, 1, 1, packed_weight=pf, force_generic=True)


# --- allocation contract ------------------------------------------------------------------------
def test_outputs_are_allocated_once_in_their_final_layout(device):
    """The forward output is allocated once, directly channels-last: peak memory of the call stays below 1.5 x the output
    (triton_conv3d/tests/test_gather_gemm.py:796-822); the weight gradient comes back channels-last, [Cout][tap][Cin] in
    memory (tests/test_bwd_weight.py:1276-1296); results of no_grad / inference_mode calls carry no graph."""
    x = torch.randn((1, 32, 32, 32, 64), device=device).to(torch.bfloat16).contiguous(memory_format=CL)
    w = (torch.randn((32, 32, 3, 3, 3), device=device) * 0.05).to(torch.bfloat16).contiguous(memory_format=CL)
    gy = torch.randn_like(x)
    sa.conv3d_forward(x, w, None, 1, 1)                         # first call: library load, workspace cache
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    y = sa.conv3d_forward(x, w, None, 1, 1)
    torch.cuda.synchronize()
    grown = torch.cuda.max_memory_allocated() - before
    assert y.is_contiguous(memory_format=CL)
    assert grown < 1.5 * y.numel() * y.element_size(), (grown, y.numel() * y.element_size())
    gw = sa.conv3d_backward_weight(x, w.shape, gy, 1, 1)
    assert gw.shape == w.shape and gw.stride(1) == 1 and gw.is_contiguous(memory_format=CL)
    gx = sa.conv3d_backward_data(gy, w, x.shape, 1, 1)
    assert gx.shape == x.shape and gx.is_contiguous(memory_format=CL)
    conv = sa.FastConv3d(32, 32, 3, padding=1).to(device).to(torch.bfloat16)
    with torch.no_grad():
        assert not conv(x).requires_grad
    with torch.inference_mode():
        assert conv(x).is_inference()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,cin,cout,spatial", [(1, 64, 32, (8, 16, 32)), (2, 128, 64, (3, 5, 7)), (1, 256, 128, (4, 8, 8)), (1, 64, 96, (5, 4, 6)),
                                                 (1, 64, 32, (32, 64, 64))])  # the last: the U-Net's level 0, thousands of bias slices
def test_transposed_weight_and_bias_gradient_in_one_pass(device, dtype, n, cin, cout, spatial):
    """``conv_transpose3d_backward_weight_bias``: the weight gradient is the bits of ``conv_transpose3d_backward_weight``; the
    bias gradient is ``grad_output.sum((0, 2, 3, 4))`` -- exactly on integer-valued gradients (fp32 sums of small integers in
    any order), within the bias-gradient tolerance of the Gaussian case on Gaussian ones -- in the operands' dtype and in fp32."""
    from scaffold_amd import transposed as ct

    g = torch.Generator().manual_seed(77)
    x = torch.randn((n, cin, *spatial), generator=g).to(dtype).contiguous(memory_format=torch.channels_last_3d).to(device)
    big = tuple(2 * v for v in spatial)
    wshape = (cin, cout, 2, 2, 2)
    for exact in (True, False):
        if exact:
            gy = torch.randint(-2, 3, (n, cout, *big), generator=g).to(dtype)
        else:
            gy = torch.randn((n, cout, *big), generator=g).to(dtype)
        gy = gy.contiguous(memory_format=torch.channels_last_3d).to(device)
        for grad_dtype in (None, torch.float32):
            both = ct.conv_transpose3d_backward_weight_bias(x, wshape, gy, 2, 0, 0, 1, 1, grad_dtype=grad_dtype)
            assert both is not None
            gw, gb = both
            want_w = ct.conv_transpose3d_backward_weight(x, wshape, gy, 2, 0, 0, 1, 1, grad_dtype=grad_dtype)
            assert gw.dtype is want_w.dtype and torch.equal(gw, want_w) and gw.stride() == want_w.stride()
            ref = gy.double().sum((0, 2, 3, 4))
            assert gb.dtype is gw.dtype and gb.shape == (cout,)
            if exact:
                assert ref.abs().max() < 2 ** 24
                if grad_dtype is torch.float32 or ref.abs().max() < 256:
                    assert torch.equal(gb.double(), ref if grad_dtype is torch.float32 else ref.to(dtype).double())
            else:
                scale = (gy.double() ** 2).sum((0, 2, 3, 4)).sqrt()  # |sum| of m terms is of the order sqrt(sum of squares)
                tol = 2e-6 * scale + 1e-3 + (0 if grad_dtype is torch.float32 else 2.0 ** -8 * ref.abs())  # fp32 sum, one rounding
                assert ((gb.double() - ref).abs() <= tol).all(), ((gb.double() - ref).abs().max(), tol.min())
    # what is not a 2x2x2 matrix-core problem is not offered: the caller computes the two apart
    x3 = torch.randn(1, 8, 4, 4, 4, device=device).to(dtype).contiguous(memory_format=torch.channels_last_3d)
    gy3 = torch.randn(1, 8, 8, 8, 8, device=device).to(dtype).contiguous(memory_format=torch.channels_last_3d)
    assert ct.conv_transpose3d_backward_weight_bias(x3, (8, 8, 2, 2, 2), gy3, 2, 0, 0, 1, 1) is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,cin,cout,spatial", [(1, 32, 11, (8, 16, 32)), (2, 64, 5, (3, 5, 7)), (1, 128, 32, (4, 8, 9)), (1, 32, 1, (5, 6, 7))])
def test_pointwise_weight_and_bias_gradient_in_one_pass(device, dtype, n, cin, cout, spatial):
    """``conv3d_backward_weight_bias`` on the head's kind of problem (1x1x1, few output channels): the weight gradient is the
    bits of ``conv3d_backward_weight``; the bias gradient is ``grad_output.sum((0, 2, 3, 4))``, exact on integer-valued
    gradients and within an fp32 sum's round-off (plus one rounding to the output type) on Gaussian ones."""
    from scaffold_amd import conv3d as c3

    g = torch.Generator().manual_seed(78)
    x = torch.randn((n, cin, *spatial), generator=g).to(dtype).contiguous(memory_format=torch.channels_last_3d).to(device)
    wshape = (cout, cin, 1, 1, 1)
    for exact in (True, False):
        gy = (torch.randint(-2, 3, (n, cout, *spatial), generator=g) if exact else torch.randn((n, cout, *spatial), generator=g)).to(dtype)
        gy = gy.contiguous(memory_format=torch.channels_last_3d).to(device)
        for grad_dtype in (None, torch.float32):
            both = c3.conv3d_backward_weight_bias(x, wshape, gy, 1, 0, 1, grad_dtype=grad_dtype)
            assert both is not None
            gw, gb = both
            want_w = sa.conv3d_backward_weight(x, wshape, gy, 1, 0, 1, grad_dtype=grad_dtype)
            assert gw.dtype is want_w.dtype and torch.equal(gw, want_w) and gw.stride() == want_w.stride()
            ref = gy.double().sum((0, 2, 3, 4))
            assert gb.dtype is gw.dtype and gb.shape == (cout,)
            if exact:
                if grad_dtype is torch.float32 or ref.abs().max() < 256:
                    assert torch.equal(gb.double(), ref if grad_dtype is torch.float32 else ref.to(dtype).double())
            else:
                scale = (gy.double() ** 2).sum((0, 2, 3, 4)).sqrt()
                tol = 2e-6 * scale + 1e-3 + (0 if grad_dtype is torch.float32 else 2.0 ** -8 * ref.abs())
                assert ((gb.double() - ref).abs() <= tol).all()
    # not offered: a 3x3x3 convolution, fp32 operands
    x3 = torch.randn(1, 32, 4, 4, 8, device=device).to(dtype).contiguous(memory_format=torch.channels_last_3d)
    gy3 = torch.randn(1, 32, 4, 4, 8, device=device).to(dtype).contiguous(memory_format=torch.channels_last_3d)
    assert c3.conv3d_backward_weight_bias(x3, (32, 32, 3, 3, 3), gy3, 1, 1, 1) is None
    assert c3.conv3d_backward_weight_bias(x3.float(), (11, 32, 1, 1, 1), gy3[:, :11].float().contiguous(memory_format=torch.channels_last_3d), 1, 0, 1) is None
