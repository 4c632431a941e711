"""Pins the oracle (no GPU): every function of oracle/oracle.py and oracle/conv_ref.c is checked against
something it was not derived from -- the committed golden vectors (brute-force C loops), closed forms,
adjoint identities and special cases -- so that a dropped term, a wrong sign or a transposed operand fails."""

import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cref
from oracle import oracle as orc

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "hotpath_small.npz"))


def g(name):
    return torch.from_numpy(GOLD[name])


def cl(t):
    return t.contiguous(memory_format=torch.channels_last_3d)


# ---- convolution: torch fp64 oracle vs the committed brute-force answers ---------------------------------
def test_conv_reference_matches_golden_vectors():
    prob = orc.ConvProblem(n=2, cin=4, cout=3, spatial=(5, 6, 7), padding=(0, 1, 1), bias=True, dtype=torch.float32)
    ops = {"input": g("conv_x"), "weight": g("conv_w"), "bias": g("conv_b"), "grad_output": g("conv_gy")}
    assert torch.equal(orc.conv_reference(prob, ops, "fwd"), g("conv_y"))
    assert torch.equal(orc.conv_reference(prob, ops, "bwd-data"), g("conv_gx"))
    assert torch.equal(orc.conv_reference(prob, ops, "bwd-weight"), g("conv_gw"))


def test_strided_dilated_conv_matches_golden_vectors():
    x, w, gy = g("sconv_x"), g("sconv_w"), g("sconv_gy")
    y = F.conv3d(x, w, None, (2, 1, 3), (1, 0, 2), (1, 2, 1))
    assert torch.equal(y, g("sconv_y"))
    wr = w.clone().requires_grad_(True)
    (gw,) = torch.autograd.grad(F.conv3d(x, wr, None, (2, 1, 3), (1, 0, 2), (1, 2, 1)), wr, gy)
    assert torch.equal(gw, g("sconv_gw"))


def test_transposed_reference_matches_golden_vectors():
    prob = orc.ConvProblem(n=1, cin=3, cout=4, spatial=(2, 3, 2), kernel=(2, 2, 2), stride=(2, 2, 2), padding=(0, 0, 0),
                           transposed=True, bias=True, dtype=torch.float32)
    ops = {"input": g("convt_x"), "weight": g("convt_w"), "bias": g("convt_b"), "grad_output": None}
    assert torch.equal(orc.conv_reference(prob, ops, "fwd"), g("convt_y"))


def test_c_loops_reproduce_their_own_golden_vectors():
    assert torch.equal(cref.conv3d_fwd(g("conv_x"), g("conv_w"), g("conv_b"), (1, 1, 1), (0, 1, 1)), g("conv_y"))
    assert torch.equal(cref.convT3d_fwd(g("convt_x"), g("convt_w"), g("convt_b")), g("convt_y"))


# ---- closed forms and identities --------------------------------------------------------------------------
def test_delta_input_reads_back_the_flipped_kernel():
    """x = delta at voxel c, one channel: y[co, c + p - t] = w[co, 0, t]  (cross-correlation)."""
    prob = orc.ConvProblem(n=1, cin=1, cout=2, spatial=(5, 5, 5), dtype=torch.float32)
    w = torch.arange(2 * 27, dtype=torch.float64).reshape(2, 1, 3, 3, 3) + 1
    x = torch.zeros(prob.input_shape, dtype=torch.float64)
    x[0, 0, 2, 2, 2] = 1.0
    for impl in (lambda: orc.conv_reference(prob, {"input": x, "weight": w, "bias": None}, "fwd"),
                 lambda: cref.conv3d_fwd(x, w, None, (1, 1, 1), (1, 1, 1))):
        y = impl()
        assert torch.equal(y[0, :, 1:4, 1:4, 1:4], w[:, 0].flip(1, 2, 3))
        assert y.abs().sum() == w.abs().sum()


@pytest.mark.parametrize("stride,padding", [((1, 1, 1), (1, 1, 1)), ((1, 1, 1), (0, 1, 1)), ((2, 2, 2), (0, 0, 0))])
def test_adjoint_identities(stride, padding):
    """<conv(x, w), g> == <x, dgrad(g)> == <w, wgrad(x, g)> for both oracles."""
    k = (3, 3, 3) if stride == (1, 1, 1) else (2, 2, 2)
    prob = orc.ConvProblem(n=2, cin=3, cout=4, spatial=(6, 6, 6), kernel=k, stride=stride, padding=padding, dtype=torch.float32)
    ops = orc.make_inputs(prob, seed=3, dtype=torch.float64)
    x, w, gy = ops["input"], ops["weight"], ops["grad_output"]
    y = orc.conv_reference(prob, ops, "fwd")
    lhs = (y * gy).sum()
    assert torch.allclose(lhs, (x * orc.conv_reference(prob, ops, "bwd-data")).sum(), rtol=1e-12)
    assert torch.allclose(lhs, (w * orc.conv_reference(prob, ops, "bwd-weight")).sum(), rtol=1e-12)
    assert torch.allclose(lhs, (x * cref.conv3d_dgrad(gy, w, x.shape, stride, padding)).sum(), rtol=1e-12)
    assert torch.allclose(lhs, (w * cref.conv3d_wgrad(x, w.shape, gy, stride, padding)).sum(), rtol=1e-12)
    assert torch.allclose(y, cref.conv3d_fwd(x, w, None, stride, padding), rtol=1e-12, atol=1e-12)


def test_data_gradient_is_flipped_gather_with_complement_padding():
    """The identity the data-gradient kernels rely on: gx = conv(gy, swap(w) flipped, padding k-1-p)."""
    prob = orc.ConvProblem(n=1, cin=3, cout=5, spatial=(4, 5, 6), padding=(0, 1, 1), dtype=torch.float32)
    ops = orc.make_inputs(prob, seed=1, dtype=torch.float64)
    gx = orc.conv_reference(prob, ops, "bwd-data")
    wt = ops["weight"].permute(1, 0, 2, 3, 4).flip(2, 3, 4)
    assert torch.allclose(gx, F.conv3d(ops["grad_output"], wt, None, 1, (2, 1, 1)), rtol=1e-12, atol=1e-12)
    # the fused tap index complement is the three-axis flip
    for t in range(27):
        kd, kh, kw = t // 9, (t // 3) % 3, t % 3
        assert 26 - t == ((2 - kd) * 3 + (2 - kh)) * 3 + (2 - kw)


def test_transposed_windows_tile_exactly_once():
    """k == s, p == 0: every output voxel has exactly one (input voxel, tap) contribution."""
    prob = orc.ConvProblem(n=1, cin=1, cout=1, spatial=(2, 3, 4), kernel=(2, 2, 2), stride=(2, 2, 2), padding=(0, 0, 0),
                           transposed=True, dtype=torch.float32)
    ones = {"input": torch.ones(prob.input_shape, dtype=torch.float64),
            "weight": torch.ones(prob.weight_shape, dtype=torch.float64), "bias": None}
    y = orc.conv_reference(prob, ones, "fwd")
    assert y.shape == (1, 1, 4, 6, 8) and torch.equal(y, torch.ones_like(y))
    assert torch.equal(cref.convT3d_fwd(ones["input"], ones["weight"]), y)
    assert prob.flops() == 2 * 24 * 8  # no phantom tap factor beyond the 8 taps per INPUT voxel


def test_shard_with_zero_halo_equals_padded_convolution():
    prob = orc.ConvProblem(n=1, cin=2, cout=3, spatial=(5, 4, 4), dtype=torch.float32)
    ops = orc.make_inputs(prob, seed=5, dtype=torch.float64)
    x = ops["input"]
    halo = torch.cat([torch.zeros_like(x[:, :, :1]), x, torch.zeros_like(x[:, :, :1])], dim=2)
    assert torch.equal(F.conv3d(halo, ops["weight"], None, 1, (0, 1, 1)), F.conv3d(x, ops["weight"], None, 1, 1))


# ---- cost model -------------------------------------------------------------------------------------------
def test_cost_model_matches_the_published_figures():
    head = orc.ConvProblem(n=1, cin=32, cout=32, spatial=(128, 128, 128), dtype=torch.bfloat16)
    assert head.flops() == 115_964_116_992            # 115.96 GFLOP
    assert abs(head.bytes() / 2**20 - 256.05) < 0.01   # 256.05 MiB
    m, n, k = head.gemm_shape("fwd")
    assert (m, n, k) == (128**3, 32, 864) and 2 * m * n * k == head.flops()
    assert head.gemm_shape("bwd-weight") == (32, 864, 128**3)
    up = orc.ConvProblem(n=1, cin=128, cout=64, spatial=(32, 32, 32), kernel=(2, 2, 2), stride=(2, 2, 2), padding=(0, 0, 0),
                         transposed=True, dtype=torch.bfloat16)
    assert up.output_shape == (1, 64, 64, 64, 64)
    assert abs(up.flops() / 1e9 - 4.29) < 0.01 and abs(up.bytes() / 2**20 - 40.1) < 0.1
    x = torch.empty(head.input_shape, device="meta")
    w = torch.empty(head.weight_shape, device="meta")
    assert tuple(F.conv3d(x, w, None, 1, 1).shape) == head.output_shape


# ---- operand generator and tolerance policy ----------------------------------------------------------------
def test_make_inputs_is_seeded_exact_and_thins_only_activations():
    prob = orc.ConvProblem(n=1, cin=8, cout=8, spatial=(6, 6, 6), dtype=torch.bfloat16)
    a = orc.make_inputs(prob, seed=4, exact=True, density=0.25)
    b = orc.make_inputs(prob, seed=4, exact=True, density=0.25)
    assert all(torch.equal(a[k], b[k]) for k in ("input", "weight", "grad_output"))
    for k in ("input", "weight", "grad_output"):
        assert set(a[k].float().unique().tolist()) <= {-1.0, 0.0, 1.0}
        assert a[k].is_contiguous(memory_format=torch.channels_last_3d)
    dense_w = (a["weight"] != 0).float().mean().item()
    thin_x = (a["input"] != 0).float().mean().item()
    assert 0.55 < dense_w < 0.78 and 0.08 < thin_x < 0.26   # 2/3 dense; 2/3 * 0.25 thinned
    assert not torch.equal(a["input"], orc.make_inputs(prob, seed=5, exact=True, density=0.25)["input"])


def test_exact_density_closed_form():
    prob = orc.ConvProblem(n=1, cin=1024, cout=1024, spatial=(8, 8, 8), dtype=torch.bfloat16)
    m, n, k = prob.gemm_shape("fwd")
    want = (1.5 * (256 / 4.0) / math.sqrt(2 * math.log(m * n))) ** 2 / k
    assert math.isclose(orc.exact_density(prob, "fwd"), want, rel_tol=1e-12) and want < 1
    small = orc.ConvProblem(n=1, cin=2, cout=2, spatial=(4, 4, 4), dtype=torch.float32)
    assert orc.exact_density(small) == 1.0


def test_exact_representability_boundary():
    assert orc.is_exactly_representable(torch.tensor([255.0, -3.0, 0.0]), torch.bfloat16)
    assert not orc.is_exactly_representable(torch.tensor([256.0]), torch.bfloat16)
    assert not orc.is_exactly_representable(torch.tensor([1.5]), torch.float32)
    assert orc.is_exactly_representable(torch.tensor([2047.0]), torch.float16)


def test_compare_and_error_bound_by_hand():
    e = torch.tensor([3.0, -4.0, 0.0, 0.0])
    a = torch.tensor([3.0, -4.5, 0.0, 0.0])
    rep = orc.compare(a, e)
    rms = math.sqrt(25 / 4)
    assert rep.max_abs == 0.5 and math.isclose(rep.max_rel, 0.5 / rms) and rep.n_diff == 1 and not rep.bitwise
    prob = orc.ConvProblem(n=1, cin=4, cout=1, spatial=(1, 1, 4), kernel=(1, 1, 1), padding=(0, 0, 0), dtype=torch.bfloat16)
    bound = orc.error_bound(prob, e, "fwd")
    assert math.isclose(bound, 8 * 2**-24 * math.sqrt(4) * rms + 2 * 2**-8 * 4.0)
    with pytest.raises(AssertionError):
        orc.assert_close(a, e, prob, "fwd")


# ---- GroupNorm ---------------------------------------------------------------------------------------------
def test_groupnorm_oracles_agree_and_match_golden_vectors():
    x, gamma, beta, dy = g("gn_x"), g("gn_gamma"), g("gn_beta"), g("gn_dy")
    y, dx, dw, db = orc.group_norm_reference(x, 4, gamma, beta, 1e-5, True, dy)
    ym, (mean, rstd), dxm, dwm, dbm = orc.group_norm_manual(x, 4, gamma, beta, 1e-5, True, dy)
    for got, ref in ((y, g("gn_y")), (dx, g("gn_dx")), (dw, g("gn_dgamma")), (db, g("gn_dbeta")), (ym, g("gn_y")),
                     (dxm, g("gn_dx")), (dwm, g("gn_dgamma")), (dbm, g("gn_dbeta")), (mean, g("gn_mean")), (rstd, g("gn_rstd"))):
        assert torch.allclose(got, ref, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("affine", [(True, True), (True, False), (False, True), (False, False)])
def test_groupnorm_manual_formula_equals_autograd(relu, affine):
    gen = torch.Generator().manual_seed(2)
    x = torch.randn((3, 6, 2, 3, 4), generator=gen, dtype=torch.float64)
    w = torch.randn(6, generator=gen, dtype=torch.float64) if affine[0] else None
    b = torch.randn(6, generator=gen, dtype=torch.float64) if affine[1] else None
    dy = torch.randn(x.shape, generator=gen, dtype=torch.float64)
    y, dx, dw, db = orc.group_norm_reference(x, 3, w, b, 1e-5, relu, dy)
    ym, _, dxm, dwm, dbm = orc.group_norm_manual(x, 3, w, b, 1e-5, relu, dy)
    assert torch.allclose(y, ym, rtol=1e-10, atol=1e-12) and torch.allclose(dx, dxm, rtol=1e-9, atol=1e-11)
    if w is not None:
        assert torch.allclose(dw, dwm, rtol=1e-9, atol=1e-11)
    if b is not None:
        assert torch.allclose(db, dbm, rtol=1e-9, atol=1e-11)


def test_groupnorm_special_cases():
    x = torch.full((2, 4, 2, 2, 2), 7.5, dtype=torch.float64)
    y, (mean, rstd) = orc.group_norm_manual(x, 2, None, None, 1e-5)
    assert torch.equal(y, torch.zeros_like(y)) and torch.allclose(rstd, torch.full_like(rstd, 1e-5 ** -0.5))
    # dx sums to zero over a group and is orthogonal to xhat (the two projections the formula removes)
    gen = torch.Generator().manual_seed(9)
    x = torch.randn((1, 4, 3, 3, 3), generator=gen, dtype=torch.float64)
    dy = torch.randn(x.shape, generator=gen, dtype=torch.float64)
    _, (mean, rstd), dx, _, _ = orc.group_norm_manual(x, 2, None, None, 1e-14, False, dy)  # eps ~ 0: exact projections
    dxg = dx.reshape(1, 2, -1)
    xh = ((x.reshape(1, 2, -1) - mean.unsqueeze(-1)) * rstd.unsqueeze(-1))
    assert dxg.sum(-1).abs().max() < 1e-12 and (dxg * xh).sum(-1).abs().max() < 1e-9
    # one element per group: dx is exactly zero
    x1 = torch.randn((4, 8, 1, 1, 1), generator=gen, dtype=torch.float64)
    _, _, dx1, _, _ = orc.group_norm_manual(x1, 8, torch.randn(8, dtype=torch.float64), None, 1e-5, False, torch.randn(x1.shape, dtype=torch.float64))
    assert torch.equal(dx1, torch.zeros_like(dx1))


def test_train_step_loss_closed_form():
    """Two voxels, two classes, logits chosen so softmax = (0.75, 0.25) at both."""
    l = math.log(3.0)
    logits = torch.tensor([l, 0.0]).view(1, 2, 1, 1, 1).expand(1, 2, 1, 1, 2).contiguous()
    labels = torch.tensor([0, 1]).view(1, 1, 1, 2)
    ce = -(math.log(0.75) + math.log(0.25)) / 2
    inter, sets = 0.25, (0.25 + 0.25) + 1.0       # class 1: p = .25 at both voxels, one voxel labelled 1
    dice1 = (2 * inter + 1e-6) / (sets + 1e-6)
    want = ce + (1 - dice1)
    assert math.isclose(orc.train_step_loss(logits, labels, 2).item(), want, rel_tol=1e-6)


def test_chaos_game_by_hand_and_fixed_point():
    # x -> x/2 and x -> x/2 + 1/2 on the first axis, choices (., 1, 0, 1): 0 -> 1/2 -> 1/4 -> 5/8
    half = np.diag([0.5, 0.0, 0.0])
    pts = orc.chaos_game([half, half], [[0, 0, 0], [0.5, 0, 0]], [0, 1, 0, 1])
    assert np.array_equal(pts, [[0, 0, 0], [0.5, 0, 0], [0.25, 0, 0], [0.625, 0, 0]])
    # one non-symmetric contraction: the orbit converges to (I - M)^-1 o; applying the transposed map would not
    m = np.array([[0.3, 0.2, 0.0], [-0.1, 0.4, 0.1], [0.25, 0.0, -0.35]])
    o = np.array([0.5, -1.0, 2.0])
    pts = orc.chaos_game([m], [o], np.zeros(200, dtype=int))
    want = np.linalg.solve(np.eye(3) - m, o)
    assert np.allclose(pts[-1], want, rtol=0, atol=1e-13) and not np.allclose(want, np.linalg.solve(np.eye(3) - m.T, o), atol=1e-3)


def test_voxelisation_rule_by_hand():
    """grid 4, extents (1, 0.25, 0): voxel size (1 + 1e-6) / 4 for ALL axes; scaled spans (3.999996, 0.999999, 0) are centred
    with offsets (2e-6, 1.5000005, 2); then floor."""
    idx = orc.points_to_voxel_indices([[0, 0, 0], [1, 0, 0], [0.6, 0.25, 0], [0.6, 0.25, 0]], 4)
    assert idx.tolist() == [[0, 1, 2], [2, 2, 2], [3, 1, 2]]
    # a shifted and uniformly scaled cloud occupies the same voxels
    idx2 = orc.points_to_voxel_indices(np.array([[0, 0, 0], [1, 0, 0], [0.6, 0.25, 0]]) * 7.0 + [3.0, -2.0, 11.0], 4)
    assert idx2.tolist() == idx.tolist()
    with pytest.raises(ValueError):
        orc.points_to_voxel_indices([[0, 0, 0], [np.nan, 0, 0]], 4)


def test_ifs_volume_closed_forms():
    # one contraction map: every point past the burn-in is its fixed point -> one voxel, the centre of the grid
    m = np.array([[0.3, 0.2, 0.0], [-0.1, 0.4, 0.1], [0.25, 0.0, -0.35]])
    occ, lab = orc.ifs_volume(8, systems=[(6, [m], [[0.5, -1.0, 2.0]])], iterations=400, seed=1)
    assert occ.shape == (1, 1, 8, 8, 8) and lab.shape == (1, 8, 8, 8) and lab.dtype == torch.int64
    assert int(occ.sum()) == 1 and lab[0, 4, 4, 4] == 7 and torch.equal(occ[0, 0] > 0, lab[0] > 0)
    # x/2, x/2 + 1/2: the attractor is the unit segment of the first axis -> the whole centre line, nothing else
    half = np.diag([0.5, 0.0, 0.0])
    occ, lab = orc.ifs_volume(8, systems=[(0, [half, half], [[0, 0, 0], [0.5, 0, 0]])], iterations=4000, seed=2)
    want = torch.zeros(8, 8, 8, dtype=torch.int64)
    want[:, 4, 4] = 1
    assert torch.equal(lab[0], want)
    # Cantor dust of ratio 1/5 (8 maps p/5 + 4c/5, c a cube corner): coordinates lie in [0,.04] [.16,.2] [.8,.84] [.96,1], i.e.
    # voxels {0, 1, 6, 7} of 8 per axis with margins of a quarter voxel; a second system painted later overwrites the first
    corners = np.array([[i, j, k] for i in (0, 1) for j in (0, 1) for k in (0, 1)], dtype=float)
    dust = (3, [np.eye(3) / 5] * 8, corners * 0.8)
    occ, lab = orc.ifs_volume(8, systems=[dust, (8, [m], [[0.5, -1.0, 2.0]])], iterations=20000, seed=3)
    want = torch.zeros(8, 8, 8, dtype=torch.int64)
    on = torch.tensor([0, 1, 6, 7])
    want[on[:, None, None], on[None, :, None], on[None, None, :]] = 4
    want[4, 4, 4] = 9
    assert torch.equal(lab[0], want)
    occ, lab = orc.ifs_volume(8, systems=[(8, [m], [[4.0, 4.0, 4.0]]), (3, [np.eye(3) / 5] * 8, corners * 0.8 + 7.0)], iterations=20000, seed=3)
    assert lab[0, 4, 4, 4] == 9 and int((lab == 4).sum()) == 64      # the dust does not reach the centre voxel


def test_ifs_volume_random_systems_are_seeded_and_labelled():
    occ, lab = orc.ifs_volume(16, iterations=4000, seed=1)
    occ2, lab2 = orc.ifs_volume(16, iterations=4000, seed=1)
    assert torch.equal(lab, lab2) and not torch.equal(lab, orc.ifs_volume(16, iterations=4000, seed=2)[1])
    assert 0 < occ.mean() < 0.5 and 1 <= lab.max() <= 10 and torch.equal(occ[0, 0] > 0, lab[0] > 0)


# ---- the tolerance gates themselves ---------------------------------------------------------------------------
def test_parity_gate_fp32_is_1e5_of_the_rms():
    e = torch.tensor([3.0, -4.0, 0.0, 0.0], dtype=torch.float64)           # rms 2.5
    inside = e.clone(); inside[2] += 0.9e-5 * 2.5
    outside = e.clone(); outside[2] -= 2e-5 * 2.5
    rep = orc.assert_baseline_tolerance(inside, e, torch.float32)
    assert math.isclose(rep.max_rel, 0.9e-5, rel_tol=1e-9)
    with pytest.raises(AssertionError):
        orc.assert_baseline_tolerance(outside, e, torch.float32)
    barely = e.clone(); barely[0] += 1.01e-5 * 2.5
    with pytest.raises(AssertionError):
        orc.assert_baseline_tolerance(barely, e, torch.float32)
    with pytest.raises(AssertionError):
        orc.assert_baseline_tolerance(torch.tensor([3.0, float("nan"), 0.0, 0.0], dtype=torch.float64), e, torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_parity_gate_16bit_is_elementwise_2e2_relative_plus_1e2_absolute(dtype):
    e = torch.tensor([2.0, -10.0, 0.0, 100.0], dtype=torch.float64)        # limits 0.05, 0.21, 0.01, 2.01
    limit = torch.tensor([0.05, 0.21, 0.01, 2.01], dtype=torch.float64)
    sign = torch.tensor([1.0, -1.0, -1.0, 1.0], dtype=torch.float64)
    orc.assert_baseline_tolerance(e + sign * limit * 0.999, e, dtype)      # every element just inside
    for k in range(4):                                                     # ONE element just outside must fail
        a = e + sign * limit * 0.999
        a[k] = e[k] + sign[k] * limit[k] * 1.001
        with pytest.raises(AssertionError):
            orc.assert_baseline_tolerance(a, e, dtype)
    # the bar is per element, not relative to the tensor's scale: 0.02 off at an exact zero fails beside a value of 100
    with pytest.raises(AssertionError):
        orc.assert_baseline_tolerance(torch.tensor([2.0, -10.0, 0.02, 100.0], dtype=torch.float64), e, dtype)
    with pytest.raises(AssertionError):
        orc.assert_baseline_tolerance(torch.tensor([2.0, float("nan"), 0.0, 100.0], dtype=torch.float64), e, dtype)
    with pytest.raises(ValueError):
        orc.assert_baseline_tolerance(e[:3], e, dtype)


def test_groupnorm_error_measure_by_hand():
    e = torch.tensor([1.0, -4.0, 2.0])
    assert orc.gn_rel_error(torch.tensor([1.5, -4.0, 2.0]), e) == 0.125          # 0.5 / max|e| = 0.5 / 4
    assert orc.gn_rel_error(torch.tensor([1.0, -4.0, 1.0]), e) == 0.25
    assert orc.gn_rel_error(e, e) == 0.0
    poisoned = orc.gn_rel_error(torch.tensor([1.0, float("nan"), 2.0]), e)
    assert math.isnan(poisoned) and not poisoned <= 1.0                          # a NaN fails every `<= tol` check
    assert orc.GN_TOLERANCE == {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 3e-3}


def test_train_step_loss_weighted_ce_closed_form():
    """Two voxels, two classes, uniform logits: p = 1/2 everywhere, CE = log 2 whatever the weights (weighted mean of
    equal terms); with logits (a, 0) on the class-0 voxel only that voxel's term changes, weighted by w0 / (w0 + w1)."""
    import math
    labels = torch.tensor([[[[0, 1]]]])
    w = torch.tensor([3.0, 1.0], dtype=torch.float64)
    logits = torch.zeros((1, 2, 1, 1, 2), dtype=torch.float64)
    base = orc.train_step_loss(logits, labels, 2, class_weight=w, dtype=torch.float64)
    dice1 = (2 * 0.5 + 1e-6) / (1.0 + 1.0 + 1e-6)
    assert abs(base.item() - (math.log(2) + 1 - dice1)) < 1e-12
    a = 1.3
    logits[0, 0, 0, 0, 0] = a
    p0 = math.exp(a) / (math.exp(a) + 1)
    ce = (3.0 * -math.log(p0) + 1.0 * math.log(2)) / 4.0
    i1, p1 = 0.5, (1 - p0) + 0.5
    dice1 = (2 * i1 + 1e-6) / (p1 + 1.0 + 1e-6)
    got = orc.train_step_loss(logits, labels, 2, class_weight=w, dtype=torch.float64)
    assert abs(got.item() - (ce + 1 - dice1)) < 1e-12


def test_committed_ifs_shard_is_the_pinned_generators_output():
    """bench.py and the full-size checks read config 5's input from tests/golden/ifs_cfg5_shard.npz; it must be exactly
    what ``ifs_volume`` (pinned above by its closed forms) produces for 128^3, 2e5 iterations, seed 5000, planes 0..63."""
    import os

    import numpy as np

    path = os.path.join(os.path.dirname(__file__), "golden", "ifs_cfg5_shard.npz")
    with np.load(path) as f:
        labels, grid, depth, iterations, seed = f["labels"], int(f["grid"]), int(f["depth"]), int(f["iterations"]), int(f["seed"])
    assert (grid, depth, iterations, seed) == (128, 64, 200_000, 5000) and labels.dtype == np.uint8 and labels.shape == (64, 128, 128)
    occ, lab = orc.ifs_volume(grid, iterations=iterations, seed=seed)
    assert np.array_equal(lab[0, :depth].numpy(), labels.astype(np.int64))
    assert 0.01 < float((labels > 0).mean()) < 0.2 and labels.max() <= 10
