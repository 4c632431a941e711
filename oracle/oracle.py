"""CPU oracle for the ScaFFold U-Net hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product (``scaffold_amd/``) may import this module: it is the checker, used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``.

What it restates, and what pins each function (so a dropped term, a wrong sign or a transposed
operand fails a test in ``tests/test_oracle.py``):

======================  =========================================================  =====================================
function                reference it follows                                        pinned by
======================  =========================================================  =====================================
``conv_reference``      ``triton_conv3d/reference.py:201-238`` (fp64 ``F.conv3d`` /   brute-force C loops (``conv_ref.c``),
                        ``F.conv_transpose3d`` + ``torch.autograd.grad``)            delta-input closed form, adjoint
                                                                                     identities <conv x, g> = <x, dgrad g>
``make_inputs``         ``reference.py:63-138`` (seeded operands, ``{-1,0,1}`` exact   value-set / density / determinism checks
                        draw with activation thinning)
``exact_density``       ``reference.py:141-174`` closed form                         hand-computed values
``is_exactly_repr...``  ``reference.py:177-193``                                     integers at / beyond the mantissa limit
``compare``,            ``reference.py:289-361`` (RMS-normalised error; bound =        hand-computed report / bound
``error_bound``         8 u32 sqrt(K) rms + 2 r u_dtype peak)
``group_norm_reference``  ``tests/test_triton_group_norm.py:114-129`` (fp64             independent from-scratch formula
                        ``F.group_norm`` + ``F.relu`` + autograd)                     (``group_norm_manual``), C loops,
                                                                                     zero-variance / one-element-group cases
``train_step_loss``     ``ScaFFold/utils/trainer.py:640-663`` (fp32 log-softmax,      closed form on a two-voxel example
                        CE + 1 - mean foreground Dice, eps 1e-6)
``assert_baseline_...``  the parity bar itself: fp32 1e-5 relative, 16-bit          hand-computed tensors just inside and just
                        2e-2 relative + 1e-2 absolute, elementwise                    outside each limit, NaN, one bad element
``gn_rel_error``        ``tests/test_triton_group_norm.py:57-78`` (max error over     hand-computed three-element case
                        max |reference|)
``chaos_game``          ``ScaFFold/datagen/generate_fractal_points.py:62-104``        fixed point (I - M)^-1 o of one map; dyadic
                                                                                     orbit of x/2, x/2 + 1/2 by hand
``points_to_voxel_...``  ``ScaFFold/datagen/volumegen.py:103-160``                    hand-computed indices (scale, centring, clip)
``ifs_volume``          ``volumegen.py:259-292`` (mask = class id + 1, painted in     one contraction -> one centre voxel; the
                        turn)                                                         segment and Sierpinski attractors' voxel sets
``shard_ingest``        ``ScaFFold/utils/trainer.py:572-589`` (``.to(float32,          the calls are the reference's own library
                        channels_last_3d)``, ``.to(long)``) + autocast's cast;        routines; index-by-index loops on a small
                        file layout ``ScaFFold/datagen/volumegen.py:259-292``         case and the round trip through ``.npy``
======================  =========================================================  =====================================

The reference's own oracle *is* a library routine (torch in fp64), so this file calls the same
routine; the reference's Python is read, never imported.
"""

from __future__ import annotations

import dataclasses
import math
from typing import Optional, Sequence

import torch
import torch.nn.functional as F

MANTISSA_BITS = {torch.float64: 53, torch.float32: 24, torch.bfloat16: 8, torch.float16: 11}


def unit_roundoff(dtype: torch.dtype) -> float:
    return 2.0 ** -MANTISSA_BITS[dtype]


def _triple(v):
    return (v, v, v) if isinstance(v, int) else tuple(int(a) for a in v)


@dataclasses.dataclass(frozen=True)
class ConvProblem:
    """One convolution: logical NCDHW shapes, FLOPs and compulsory bytes (``triton_conv3d/shapes.py:288-340``)."""

    n: int
    cin: int
    cout: int
    spatial: tuple  # input (D, H, W)
    kernel: tuple = (3, 3, 3)
    stride: tuple = (1, 1, 1)
    padding: tuple = (1, 1, 1)
    transposed: bool = False
    bias: bool = False
    dtype: torch.dtype = torch.bfloat16

    @property
    def input_shape(self):
        return (self.n, self.cin, *self.spatial)

    @property
    def weight_shape(self):
        return ((self.cin, self.cout) if self.transposed else (self.cout, self.cin)) + tuple(self.kernel)

    @property
    def output_spatial(self):
        if self.transposed:
            return tuple((i - 1) * s - 2 * p + k for i, s, p, k in zip(self.spatial, self.stride, self.padding, self.kernel))
        return tuple((i + 2 * p - k) // s + 1 for i, s, p, k in zip(self.spatial, self.stride, self.padding, self.kernel))

    @property
    def output_shape(self):
        return (self.n, self.cout, *self.output_spatial)

    @property
    def taps(self):
        return self.kernel[0] * self.kernel[1] * self.kernel[2]

    def flops(self) -> int:
        """2*N*vol*Cin*Cout*taps; for a k == s transposed conv ``vol`` is the INPUT volume."""
        vol = math.prod(self.spatial if self.transposed else self.output_spatial)
        return 2 * self.n * vol * self.cin * self.cout * self.taps

    def bytes(self) -> int:
        """x + w + y once each."""
        item = torch.empty((), dtype=self.dtype).element_size()
        return item * (math.prod(self.input_shape) + math.prod(self.weight_shape) + math.prod(self.output_shape))

    def gemm_shape(self, direction: str = "fwd"):
        """(M, N, K) of the GEMM each direction runs."""
        vox_out = self.n * math.prod(self.output_spatial)
        vox_in = self.n * math.prod(self.spatial)
        if self.transposed:
            if direction == "fwd":
                return (vox_in, self.cout * self.taps, self.cin)
            if direction == "bwd-data":
                return (vox_in, self.cin, self.cout * self.taps)
            return (self.cin, self.cout * self.taps, vox_in)
        if direction == "fwd":
            return (vox_out, self.cout, self.cin * self.taps)
        if direction == "bwd-data":
            return (vox_in, self.cin, self.cout * self.taps)
        return (self.cout, self.cin * self.taps, vox_out)


# ---------------------------------------------------------------------------------------------
# operands
# ---------------------------------------------------------------------------------------------
def make_inputs(problem: ConvProblem, *, seed: int = 0, exact: bool = False, density: Optional[float] = None,
                channels_last: bool = True, dtype: Optional[torch.dtype] = None) -> dict:
    """Input, weight, bias and upstream gradient, drawn on the CPU generator (identical bits on
    every machine).  ``exact=True`` draws from {-1, 0, 1}; ``density`` then thins the two
    activations (never the weight) so realised sums stay inside the mantissa."""
    dtype = dtype or problem.dtype
    thin = exact and density is not None and density < 1.0

    def draw(shape, offset, activation=False):
        g = torch.Generator().manual_seed(seed + offset)
        if exact:
            t = torch.randint(-1, 2, shape, generator=g, dtype=torch.int8).to(dtype)
            if thin and activation:
                gm = torch.Generator().manual_seed(seed + offset + (1 << 20))
                t = t * (torch.rand(shape, generator=gm) < density).to(dtype)
            return t
        return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)

    fmt = torch.channels_last_3d if channels_last else torch.contiguous_format
    out = {
        "input": draw(problem.input_shape, 0, True).contiguous(memory_format=fmt),
        "weight": draw(problem.weight_shape, 1).contiguous(memory_format=fmt),
        "grad_output": draw(problem.output_shape, 2, True).contiguous(memory_format=fmt),
        "bias": draw((problem.cout,), 3) if problem.bias else None,
    }
    return out


def exact_density(problem: ConvProblem, direction: str = "fwd", *, dtype=None, headroom: float = 4.0) -> float:
    """q = min(1, (1.5 * 2^mant / headroom / sqrt(2 ln(MN)))^2 / K)."""
    dtype = dtype or problem.dtype
    m, n, k = problem.gemm_shape(direction)
    if k <= 0 or m * n <= 0:
        return 1.0
    limit = 2 ** MANTISSA_BITS[dtype] / headroom
    spread = math.sqrt(2.0 * math.log(max(m * n, 2)))
    return min(1.0, (1.5 * limit / spread) ** 2 / k)


def is_exactly_representable(result: torch.Tensor, dtype: torch.dtype) -> bool:
    finite = result[torch.isfinite(result)]
    if finite.numel() == 0:
        return True
    return bool(torch.equal(finite, finite.round()) and finite.abs().max().item() < 2 ** MANTISSA_BITS[dtype])


# ---------------------------------------------------------------------------------------------
# convolution references
# ---------------------------------------------------------------------------------------------
def _conv(problem: ConvProblem, x, w, b):
    op = F.conv_transpose3d if problem.transposed else F.conv3d
    return op(x, w, b, stride=problem.stride, padding=problem.padding)


def conv_reference(problem: ConvProblem, operands: dict, direction: str = "fwd", *, dtype=torch.float64) -> torch.Tensor:
    """The trusted answer in ``dtype`` (fp64): forward value, or the requested gradient via autograd."""
    x = operands["input"].to(device="cpu", dtype=dtype)
    w = operands["weight"].to(device="cpu", dtype=dtype)
    b = operands.get("bias")
    b = b.to(device="cpu", dtype=dtype) if b is not None else None
    if direction == "fwd":
        return _conv(problem, x, w, b)
    gy = operands["grad_output"].to(device="cpu", dtype=dtype)
    x = x.detach().requires_grad_(direction == "bwd-data")
    w = w.detach().requires_grad_(direction != "bwd-data")
    y = _conv(problem, x, w, b)
    (grad,) = torch.autograd.grad(y, (x if direction == "bwd-data" else w,), gy)
    return grad


# ---------------------------------------------------------------------------------------------
# comparison / tolerance policy
# ---------------------------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class ErrorReport:
    max_abs: float
    max_rel: float  # max_abs / rms(expected)
    rms_rel: float
    n_diff: int
    n_total: int

    @property
    def bitwise(self) -> bool:
        return self.n_diff == 0

    def __str__(self) -> str:
        return (f"max_abs={self.max_abs:.3e} max_rel={self.max_rel:.3e} rms_rel={self.rms_rel:.3e} "
                f"diff={self.n_diff}/{self.n_total}")


def compare(actual: torch.Tensor, expected: torch.Tensor) -> ErrorReport:
    a = actual.detach().to(device="cpu", dtype=torch.float64)
    e = expected.detach().to(device="cpu", dtype=torch.float64)
    if a.shape != e.shape:
        raise ValueError(f"shape mismatch: {tuple(a.shape)} vs {tuple(e.shape)}")
    if a.numel() == 0:
        return ErrorReport(0.0, 0.0, 0.0, 0, 0)
    diff = (a - e).abs()
    scale = e.pow(2).mean().sqrt().item()
    scale = scale if scale > 0 else 1.0
    return ErrorReport(diff.max().item(), diff.max().item() / scale, diff.pow(2).mean().sqrt().item() / scale,
                       int((a != e).sum().item()), a.numel())


def error_bound(problem: ConvProblem, expected: torch.Tensor, direction: str = "fwd", *, roundings: float = 1.0) -> float:
    """8 * u_fp32 * sqrt(K) * rms  +  2 * roundings * u_dtype * peak."""
    k = problem.gemm_shape(direction)[2]
    e = expected.detach().to(torch.float64)
    rms = e.pow(2).mean().sqrt().item()
    peak = e.abs().max().item()
    return 8.0 * unit_roundoff(torch.float32) * math.sqrt(k) * rms + 2.0 * roundings * unit_roundoff(problem.dtype) * peak


def assert_close(actual, expected, problem: ConvProblem, direction: str = "fwd", *, incumbent_error: Optional[ErrorReport] = None,
                 margin: float = 4.0, roundings: float = 1.0) -> ErrorReport:
    report = compare(actual, expected)
    bound = error_bound(problem, expected, direction, roundings=roundings)
    if incumbent_error is not None:
        bound = max(bound, margin * incumbent_error.max_abs)
    if not (report.max_abs <= bound):
        raise AssertionError(f"{problem} [{direction}]: {report}, bound max_abs <= {bound:.3e}")
    return report


def assert_baseline_tolerance(actual, expected, dtype: torch.dtype, what: str = "") -> ErrorReport:
    """The parity bar of the hot path: fp32 within 1e-5 relative (to the RMS of the expected tensor);
    bf16/fp16 within 2e-2 relative + 1e-2 absolute, elementwise."""
    report = compare(actual, expected)
    a = actual.detach().to(device="cpu", dtype=torch.float64)
    e = expected.detach().to(device="cpu", dtype=torch.float64)
    if dtype is torch.float32:
        ok = report.max_rel <= 1e-5
    else:
        ok = bool(((a - e).abs() <= 1e-2 + 2e-2 * e.abs()).all())
    if not ok:
        raise AssertionError(f"{what}: outside the parity tolerance for {dtype}: {report}")
    return report


# ---------------------------------------------------------------------------------------------
# GroupNorm references
# ---------------------------------------------------------------------------------------------
def group_norm_reference(x, num_groups, weight=None, bias=None, eps=1e-5, relu=False, grad_output=None, *, dtype=torch.float64):
    """fp64 ``F.group_norm`` (+``F.relu``); with ``grad_output`` also returns (dx, dweight, dbias)."""
    xd = x.detach().to(device="cpu", dtype=dtype).requires_grad_(grad_output is not None)
    wd = None if weight is None else weight.detach().to(device="cpu", dtype=dtype).requires_grad_(grad_output is not None)
    bd = None if bias is None else bias.detach().to(device="cpu", dtype=dtype).requires_grad_(grad_output is not None)
    # torch's CPU group_norm backward cannot differentiate a bias without a weight; unit weights are the same function
    w_arg = wd if (wd is not None or bd is None) else torch.ones(xd.shape[1], dtype=dtype)
    y = F.group_norm(xd, num_groups, w_arg, bd, eps)
    if relu:
        y = F.relu(y)
    if grad_output is None:
        return y.detach()
    wanted = [t for t in (xd, wd, bd) if t is not None]
    grads = list(torch.autograd.grad(y, wanted, grad_output.detach().to(device="cpu", dtype=dtype)))
    dx = grads.pop(0)
    dw = grads.pop(0) if wd is not None else None
    db = grads.pop(0) if bd is not None else None
    return y.detach(), dx, dw, db


def group_norm_manual(x, num_groups, weight=None, bias=None, eps=1e-5, relu=False, grad_output=None):
    """The same quantities from the textbook formulas, no autograd and no ``F.group_norm``:
    mean/var per (n, g), y = (x - mu) rstd gamma + beta, and
    dx = rstd (g gamma - mean_g(g gamma) - xhat mean_g(g gamma xhat)), dgamma = sum g xhat, dbeta = sum g,
    where g is the upstream gradient gated by the sign of the pre-activation when ``relu``."""
    xd = x.detach().to(device="cpu", dtype=torch.float64)
    n, c = xd.shape[:2]
    sp = xd.shape[2:]
    cg = c // num_groups
    xg = xd.reshape(n, num_groups, cg, -1)
    mu = xg.mean(dim=(2, 3), keepdim=True)
    var = ((xg - mu) ** 2).mean(dim=(2, 3), keepdim=True)
    rstd = 1.0 / torch.sqrt(var + eps)
    xhat = ((xg - mu) * rstd).reshape(n, c, *sp)
    shape = (1, c) + (1,) * len(sp)
    gamma = torch.ones(c, dtype=torch.float64) if weight is None else weight.detach().to(device="cpu", dtype=torch.float64)
    beta = torch.zeros(c, dtype=torch.float64) if bias is None else bias.detach().to(device="cpu", dtype=torch.float64)
    pre = xhat * gamma.reshape(shape) + beta.reshape(shape)
    y = torch.where(pre <= 0, torch.zeros_like(pre), pre) if relu else pre
    stats = (mu.reshape(n, num_groups), rstd.reshape(n, num_groups))
    if grad_output is None:
        return y, stats
    g = grad_output.detach().to(device="cpu", dtype=torch.float64)
    if relu:
        g = torch.where(pre <= 0, torch.zeros_like(g), g)
    gg = (g * gamma.reshape(shape)).reshape(n, num_groups, cg, -1)
    xh = xhat.reshape(n, num_groups, cg, -1)
    c1 = gg.mean(dim=(2, 3), keepdim=True)
    c2 = (gg * xh).mean(dim=(2, 3), keepdim=True)
    dx = (rstd * (gg - c1 - xh * c2)).reshape(n, c, *sp)
    red = (0,) + tuple(range(2, 2 + len(sp)))
    dw = (g * xhat).sum(dim=red)
    db = g.sum(dim=red)
    return y, stats, dx, dw, db


#: GroupNorm tolerances relative to max|reference| (``tests/test_triton_group_norm.py:57-78``)
GN_TOLERANCE = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 3e-3}


def gn_rel_error(actual: torch.Tensor, expected: torch.Tensor) -> float:
    a = actual.detach().to(device="cpu", dtype=torch.float64)
    e = expected.detach().to(device="cpu", dtype=torch.float64)
    denom = max(e.abs().max().item(), 1e-30)
    return (a - e).abs().max().item() / denom


# ---------------------------------------------------------------------------------------------
# train step recipe (config 5)
# ---------------------------------------------------------------------------------------------
def train_step_loss(logits: torch.Tensor, labels: torch.Tensor, n_classes: int, eps: float = 1e-6, class_weight=None,
                    dtype=torch.float32) -> torch.Tensor:
    """log-softmax in ``dtype`` -> (weighted) mean cross entropy + (1 - mean foreground soft Dice)
    (``ScaFFold/utils/trainer.py:640-663``, ``ScaFFold/utils/losses.py:119-214``,
    ``ScaFFold/utils/dice_score.py:101-136``)."""
    logp = F.log_softmax(logits.to(dtype), dim=1)
    ce = F.nll_loss(logp, labels, weight=None if class_weight is None else class_weight.to(dtype))
    prob = logp.exp()
    onehot = F.one_hot(labels, n_classes).movedim(-1, 1).to(prob.dtype)
    dims = (2, 3, 4)
    inter = (prob * onehot).sum(dims)
    sets = prob.sum(dims) + onehot.sum(dims)
    dice = (2 * inter + eps) / (sets + eps)  # (N, C)
    return ce + (1.0 - dice[:, 1:].mean())


def chaos_game(mats, offs, choice):
    """Orbit of an iterated function system: p_0 = origin, p_n = mats[choice[n]] @ p_{n-1} + offs[choice[n]] for
    n = 1 .. len(choice) - 1 (``ScaFFold/datagen/generate_fractal_points.py:62-104``: the first point is the origin and
    every later one is the chosen affine map of its predecessor).  Returns the (len(choice), 3) float64 points."""
    import numpy as np

    mats = np.asarray(mats, dtype=np.float64)
    offs = np.asarray(offs, dtype=np.float64)
    pts = np.zeros((len(choice), 3))
    p = np.zeros(3)
    for i in range(1, len(choice)):
        t = choice[i]
        p = mats[t] @ p + offs[t]
        pts[i] = p
    return pts


def points_to_voxel_indices(points, grid_size: int, eps: float = 1e-6):
    """The voxels a point cloud occupies on a ``grid_size``-cube (``ScaFFold/datagen/volumegen.py:103-160``): one
    isotropic voxel size ``(largest extent + eps) / grid_size`` for all axes, the cloud's bounding box centred in the
    grid (offset ``(grid_size - span) / 2`` per axis, span in voxels), floor, clip to the grid, duplicates removed.
    Non-finite coordinates are refused.  Returns a (K, 3) int64 array sorted lexicographically."""
    import numpy as np

    points = np.asarray(points, dtype=np.float64)
    if not np.isfinite(points).all():
        raise ValueError("non-finite coordinates in the point cloud")
    mins = points.min(axis=0)
    voxel = (float((points.max(axis=0) - mins).max()) + eps) / grid_size
    scaled = (points - mins) / voxel
    offset = (grid_size - scaled.max(axis=0)) / 2.0
    idx = np.clip(np.floor(scaled + offset).astype(np.int64), 0, grid_size - 1)
    return np.unique(idx, axis=0)


def ifs_volume(grid_size: int, *, n_fractals: int = 3, n_classes: int = 10, n_maps: int = 4, iterations: int = 200_000,
               seed: int = 5000, systems=None, burn_in: int = 100):
    """Config 5's synthetic sample on a ``grid_size``-cube: the voxelised orbits of ``n_fractals`` random 3-D iterated
    function systems (``n_maps`` affine maps each: a random rotation scaled by a contraction factor U(0.3, 0.7), offset
    U(-1, 1)^3, maps chosen uniformly), painted in turn with mask value ``class id + 1`` as the generator does
    (``ScaFFold/datagen/volumegen.py:259-292``: later fractals overwrite earlier ones; background stays 0).
    ``systems`` replaces the random draw by explicit ``(class_id, mats, offs)`` triples (orbit choices still come from
    ``seed``).  The first ``burn_in`` points of an orbit are dropped (they are not yet on the attractor).
    Returns (occupancy float32 (1, 1, G, G, G), labels int64 (1, G, G, G)); a depth shard is a slice of both."""
    import numpy as np

    rng = np.random.default_rng(seed)
    g = int(grid_size)
    labels = np.zeros((g, g, g), dtype=np.int64)
    if systems is None:
        systems = []
        for _ in range(n_fractals):
            cls = int(rng.integers(0, n_classes))
            mats, offs = [], []
            for _ in range(n_maps):
                q, _r = np.linalg.qr(rng.standard_normal((3, 3)))
                mats.append(q * rng.uniform(0.3, 0.7))
                offs.append(rng.uniform(-1.0, 1.0, size=3))
            systems.append((cls, np.stack(mats), np.stack(offs)))
    for cls, mats, offs in systems:
        choice = rng.integers(0, len(mats), size=iterations)
        idx = points_to_voxel_indices(chaos_game(mats, offs, choice)[burn_in:], g)
        labels[idx[:, 0], idx[:, 1], idx[:, 2]] = cls + 1
    lab = torch.from_numpy(labels)[None]
    occ = (lab > 0).to(torch.float32)[:, None]
    return occ, lab


# ---------------------------------------------------------------------------------------------
# dataset shard -> step inputs
# ---------------------------------------------------------------------------------------------
def shard_ingest(volume: torch.Tensor, mask: Optional[torch.Tensor] = None, *, dtype=torch.float32, halo: int = 0):
    """What the trainer does with a batch before the first convolution, on the CPU with the library calls it uses:
    ``volume (N, C, D, H, W)`` float32 -> channels-last ``dtype`` (``ScaFFold/utils/trainer.py:575-580``; the rounding to
    a 16-bit ``dtype`` is autocast's cast of the convolution input), ``mask (N, D, H, W)`` 16-bit -> int64
    (``trainer.py:581-583``).  ``halo`` > 0 returns the depth slab instead: ``halo`` zero planes on each face, the
    zero-filled form of the halo exchange (``ScaFFold/unet/conv3d.py:769-776``).  Returns ``(x, labels)``."""
    x = volume.to(dtype=torch.float32, memory_format=torch.channels_last_3d).to(dtype)
    if halo:
        x = F.pad(x, (0, 0, 0, 0, halo, halo)).contiguous(memory_format=torch.channels_last_3d)
    labels = None
    if mask is not None:
        if mask.dtype is torch.uint16:   # the file's type: widen through numpy, which has the conversion on every build
            labels = torch.from_numpy(mask.numpy().astype("int64"))
        else:
            labels = mask.to(torch.long)
    return x, labels
