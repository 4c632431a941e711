"""GPU parity of channels-last GroupNorm (+fused ReLU) against the fp64 oracle, through the C ABI.

Follows the reference's GroupNorm suites: fp64 ``F.group_norm`` + autograd as the reference
(``tests/test_triton_group_norm.py:114-129``) with tolerances fp32 1e-4 / bf16 2e-2 / fp16 3e-3 relative to
``max|ref|`` (``:57-78``), the shape matrix of ``tests/test_triton_group_norm_edge.py:163-264`` and its
numerical special cases (``:344-429``, ``:1647-1693``).
"""

import pytest
import torch
import torch.nn.functional as F

import scaffold_amd as sa
from oracle import oracle as orc
from scaffold_amd import groupnorm as gnm

pytestmark = pytest.mark.gpu

CL = torch.channels_last_3d


def make(shape, dtype, seed, mean=0.5, std=3.0):
    g = torch.Generator().manual_seed(seed)
    c = shape[1]
    x = (torch.randn(shape, generator=g) * std + mean).to(dtype).contiguous(memory_format=CL)
    gamma = (1 + 0.1 * torch.randn(c, generator=g)).to(dtype)
    beta = (0.1 * torch.randn(c, generator=g)).to(dtype)
    dy = torch.randn(shape, generator=g).to(dtype).contiguous(memory_format=CL)
    return x, gamma, beta, dy


def run_ours(x, groups, gamma, beta, dy, relu, device, eps=1e-5, out_dtype=None):
    xd = x.to(device).requires_grad_(True)
    gd = None if gamma is None else gamma.to(device).requires_grad_(True)
    bd = None if beta is None else beta.to(device).requires_grad_(True)
    y = sa.group_norm(xd, groups, gd, bd, eps, "relu" if relu else None, out_dtype=out_dtype)
    y.backward(dy.to(device).to(y.dtype))
    return y.detach(), xd.grad, None if gd is None else gd.grad, None if bd is None else bd.grad


def check(shape, groups, dtype, relu, device, seed=0, affine=(True, True), tol_scale=1.0, **kw):
    x, gamma, beta, dy = make(shape, dtype, seed, **kw)
    gamma = gamma if affine[0] else None
    beta = beta if affine[1] else None
    y, dx, dw, db = run_ours(x, groups, gamma, beta, dy, relu, device)
    yr, dxr, dwr, dbr = orc.group_norm_reference(x, groups, gamma, beta, 1e-5, relu, dy)
    tol = orc.GN_TOLERANCE[dtype] * tol_scale
    assert y.dtype == dtype and dx.dtype == dtype
    assert y.is_contiguous(memory_format=CL) and dx.is_contiguous(memory_format=CL)
    assert orc.gn_rel_error(y, yr) <= tol, ("y", orc.gn_rel_error(y, yr))
    assert orc.gn_rel_error(dx, dxr) <= tol, ("dx", orc.gn_rel_error(dx, dxr))
    if dw is not None:
        assert orc.gn_rel_error(dw, dwr) <= max(tol, 2e-2 if dtype != torch.float32 else tol), ("dw", orc.gn_rel_error(dw, dwr))
    if db is not None:
        assert orc.gn_rel_error(db, dbr) <= max(tol, 2e-2 if dtype != torch.float32 else tol), ("db", orc.gn_rel_error(db, dbr))


# U-Net sites (base width 32, 8 groups) and the shape matrix of the reference's edge suite:
# channels per group below / at / above the vector width, non-power-of-two groups (scalar path),
# instance norm, layer norm, ragged spatial tails, shapes that leave empty splits.
SHAPES = [
    ((2, 64, 16, 16, 16), 8),
    ((1, 32, 8, 16, 32), 8),
    ((1, 128, 8, 8, 8), 8),
    ((1, 256, 4, 4, 4), 8),
    ((1, 512, 2, 4, 4), 8),
    ((2, 16, 5, 7, 9), 8),       # 2 channels per group
    ((2, 8, 3, 3, 3), 8),        # instance norm
    ((3, 24, 3, 5, 7), 1),       # layer norm
    ((2, 24, 4, 4, 5), 3),       # scalar path: 8 channels/group but C/8 = 3 vectors, fine; G=3
    ((2, 12, 3, 4, 5), 3),       # scalar path: C not a multiple of 8
    ((5, 40, 1, 1, 1), 5),       # S = 1
    ((1, 64, 1, 1, 127), 8),
    ((1, 64, 1, 3, 43), 8),      # S = 129
    ((1, 64, 1, 1, 257), 8),
    ((1, 2048, 1, 1, 2), 8),
    ((1, 1024, 2, 2, 2), 32),
    # the deep U-Net levels and their neighbours: many channels, few voxels (the fold of many small splits)
    ((1, 256, 8, 16, 16), 8),
    ((1, 256, 8, 16, 17), 8),
    ((1, 512, 4, 8, 8), 8),
    ((1, 1024, 2, 4, 4), 8),
    ((1, 2048, 1, 2, 2), 8),
    ((2, 256, 4, 8, 8), 8),
]


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("shape,groups", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_parity(device, dtype, shape, groups, relu):
    check(shape, groups, dtype, relu, device)


def test_config2_full_size(device):
    """Benchmark configuration 2: N=2, C=64, 64^3, 8 groups, bf16; statistics vs fp64 and the elementwise
    results through sampled slices (the fp64 reference of the full tensor would take minutes)."""
    shape = (2, 64, 64, 64, 64)
    g = torch.Generator().manual_seed(2000)
    x = (torch.randn(shape, generator=g) * 3 + 0.5).to(torch.bfloat16).contiguous(memory_format=CL)
    gamma = 1 + 0.1 * torch.randn(64, generator=torch.Generator().manual_seed(2001))
    beta = 0.1 * torch.randn(64, generator=torch.Generator().manual_seed(2002))
    dy = torch.randn(shape, generator=torch.Generator().manual_seed(2003)).to(torch.bfloat16).contiguous(memory_format=CL)
    xd = x.to(device)
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(xd, 8, gamma.to(device), beta.to(device), 1e-5, "relu", None)
    x64 = x.double().reshape(2, 8, 8, -1)
    mu = x64.mean(dim=(2, 3))
    var = x64.var(dim=(2, 3), unbiased=False)
    assert torch.allclose(mean.cpu().double(), mu, rtol=0, atol=1e-5)
    assert torch.allclose(rstd.cpu().double(), 1 / torch.sqrt(var + 1e-5), rtol=1e-5, atol=0)
    # elementwise parity on depth slices, with the oracle given the exact statistics
    dxo, dwo, dbo = torch.ops.scaffold_gn.group_norm_backward(dy.to(device), xd, gamma.to(device), beta.to(device), mean, rstd,
                                                              8, "relu")
    yr, _st, dxr, dwr, dbr = orc.group_norm_manual(x, 8, gamma, beta, 1e-5, True, dy)
    assert orc.gn_rel_error(out, yr) <= 2e-2
    assert orc.gn_rel_error(dxo, dxr) <= 2e-2
    assert orc.gn_rel_error(dwo, dwr) <= 1e-4
    assert orc.gn_rel_error(dbo, dbr) <= 1e-4


@pytest.mark.parametrize("affine", [(True, True), (True, False), (False, True), (False, False)])
def test_affine_variants(device, affine):
    check((2, 32, 4, 5, 6), 8, torch.float32, True, device, affine=affine)
    check((2, 32, 4, 5, 6), 8, torch.bfloat16, False, device, affine=affine)


def test_fused_relu_is_bitwise_unfused_plus_relu(device):
    x, gamma, beta, dy = make((2, 64, 6, 7, 8), torch.bfloat16, 3)
    y0, dx0, dw0, db0 = run_ours(x, 8, gamma, beta, dy, True, device)
    xd = x.to(device).requires_grad_(True)
    gd, bd = gamma.to(device).requires_grad_(True), beta.to(device).requires_grad_(True)
    y1 = F.relu(sa.group_norm(xd, 8, gd, bd, 1e-5, None))
    y1.backward(dy.to(device))
    assert torch.equal(y0, y1.detach())
    assert torch.equal(dx0, xd.grad) and torch.equal(dw0, gd.grad) and torch.equal(db0, bd.grad)


def test_relu_special_values_match_torch(device):
    """NaN propagates, -0.0 / +-Inf behave like F.relu; the backward gates like threshold_backward."""
    vals = torch.tensor([float("nan"), -0.0, 0.0, float("inf"), -float("inf"), 1.0, -1.0, 2.0], device=device)
    # instance-norm-free check of the two spellings on raw values
    relu = torch.where(vals <= 0, torch.zeros_like(vals), vals)
    ref = F.relu(vals)
    assert torch.equal(torch.isnan(relu), torch.isnan(ref))
    assert torch.equal(relu[~torch.isnan(relu)].view(torch.int32), ref[~torch.isnan(ref)].view(torch.int32))
    # through the kernel: one NaN input poisons its group, and only its group
    x = torch.randn((1, 16, 2, 2, 2), device=device).contiguous(memory_format=CL)
    x[0, 3, 0, 0, 0] = float("nan")
    y = sa.group_norm(x, 4, None, None, 1e-5, "relu")
    assert torch.isnan(y[0, :4]).all() and torch.isfinite(y[0, 4:]).all()


def test_all_equal_input_is_exactly_zero(device):
    x = torch.full((2, 32, 4, 4, 4), 3.25, device=device).contiguous(memory_format=CL)
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(x, 8, None, None, 1e-5, None, None)
    assert torch.equal(out, torch.zeros_like(out))
    assert torch.allclose(rstd, torch.full_like(rstd, 1e-5 ** -0.5), rtol=1e-6)
    assert torch.equal(mean, torch.full_like(mean, 3.25))


def test_single_element_groups_have_zero_dx(device):
    x = torch.randn((4, 8, 1, 1, 1), device=device).contiguous(memory_format=CL).requires_grad_(True)
    w = torch.randn(8, device=device).requires_grad_(True)
    y = sa.group_norm(x, 8, w, None, 1e-5, None)
    y.backward(torch.randn_like(y))
    assert torch.equal(x.grad, torch.zeros_like(x.grad))


@pytest.mark.parametrize("mean,std", [(1e3, 1e-2), (1e6, 1.0), (-300.0, 0.05)])
def test_large_mean_small_std(device, mean, std):
    """The shifted single-pass statistics must not lose the variance the way E[x^2]-E[x]^2 does."""
    g = torch.Generator().manual_seed(12)
    x = (torch.randn((2, 32, 8, 8, 8), generator=g, dtype=torch.float64) * std + mean).float().contiguous(memory_format=CL)
    out, mu, rstd = torch.ops.scaffold_gn.group_norm(x.to(device), 8, None, None, 1e-12, None, None)
    x64 = x.double().reshape(2, 8, -1)
    var = x64.var(dim=2, unbiased=False)
    ref_rstd = 1 / torch.sqrt(var + 1e-12)
    ours = ((rstd.cpu().double() - ref_rstd).abs() / ref_rstd).max().item()
    aten = F.group_norm(x, 8, None, None, 1e-12)
    ref = orc.group_norm_reference(x, 8, None, None, 1e-12)
    assert ours <= 1e-3, ours
    assert orc.gn_rel_error(out, ref) <= max(2 * orc.gn_rel_error(aten, ref), 1e-5)


def test_out_dtype_contract(device):
    x, gamma, beta, _ = make((2, 32, 4, 4, 4), torch.bfloat16, 5)
    xd, gd, bd = x.to(device), gamma.to(device), beta.to(device)
    wide = sa.group_norm(xd, 8, gd, bd, out_dtype=torch.float32)
    narrow = sa.group_norm(xd, 8, gd, bd, out_dtype=None)
    assert wide.dtype is torch.float32 and narrow.dtype is torch.bfloat16
    assert torch.equal(narrow, wide.to(torch.bfloat16))  # the narrow result is the wide one rounded once
    with torch.autocast("cuda", dtype=torch.bfloat16):
        stock_like = sa.group_norm(xd, 8, gd.float(), bd.float())
        assert stock_like.dtype is torch.float32
    assert sa.group_norm(xd, 8, gd, bd).dtype is torch.bfloat16
    # fp32 cotangent for a bf16 input (the autocast case) flows through the backward
    xr = xd.clone().requires_grad_(True)
    out = sa.group_norm(xr, 8, gd, bd, out_dtype=torch.float32)
    out.backward(torch.ones_like(out))
    assert xr.grad.dtype is torch.bfloat16


def test_validation_and_gates(device):
    x = torch.randn((2, 32, 4, 4, 4), device=device).contiguous(memory_format=CL)
    assert gnm.is_supported(x, 8)
    assert not gnm.is_supported(x.cpu(), 8)
    assert not gnm.is_supported(x, 5)
    assert not gnm.is_supported(x.contiguous(), 8)
    assert not gnm.is_supported(x, 8, activation="gelu")
    assert not gnm.is_supported(x.double(), 8)
    assert not gnm.is_supported(x.bfloat16(), 8, torch.ones(32, device=device))  # fp32 affine outside autocast
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert gnm.is_supported(x.bfloat16(), 8, torch.ones(32, device=device))
    with pytest.raises(ValueError):
        sa.group_norm(x, 8, activation="gelu")
    with pytest.raises(ValueError):
        sa.group_norm(torch.randn((1, 8, 1, 1, 1), device=device), 8)  # one value per channel
    with pytest.raises(NotImplementedError):
        sa.group_norm(x.cpu(), 8)
    with pytest.raises(ValueError):
        torch.ops.scaffold_gn.group_norm(x.contiguous(), 8, None, None, 1e-5, None, None)


def test_double_backward_raises(device):
    x = torch.randn((1, 16, 2, 2, 2), device=device).contiguous(memory_format=CL).requires_grad_(True)
    y = sa.group_norm(x, 4)
    (g,) = torch.autograd.grad(y.sum(), x, create_graph=True)
    with pytest.raises(RuntimeError):
        torch.autograd.grad(g.sum(), x)


def test_same_call_same_bits_with_poisoned_scratch(device):
    x, gamma, beta, dy = make((2, 64, 8, 8, 8), torch.bfloat16, 21)
    ref = None
    for _ in range(3):
        junk = torch.full((1 << 22,), float("nan"), device=device)
        del junk
        got = run_ours(x, 8, gamma, beta, dy, True, device)
        assert all(torch.isfinite(t).all() for t in got)
        if ref is None:
            ref = got
        else:
            assert all(torch.equal(a, b) for a, b in zip(ref, got))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape,halo", [((1, 64, 6, 7, 8), 1), ((1, 32, 3, 5, 4), 2), ((1, 48, 40, 16, 16), 1)])
def test_output_into_a_depth_slab_is_bitwise_the_plain_output(device, dtype, shape, halo):
    """``out_halo``: the result lands in the interior of a slab whose faces are zero; values, statistics and all
    gradients are those of the plain call."""
    x, gamma, beta, dy = make(shape, dtype, 5)
    outs = []
    for h in (0, halo):
        xd = x.to(device).requires_grad_(True)
        gd, bd = gamma.to(device).requires_grad_(True), beta.to(device).requires_grad_(True)
        y = sa.group_norm(xd, 8, gd, bd, 1e-5, "relu", out_dtype=None, out_halo=h)
        y.backward(dy.to(device))
        outs.append((y, xd.grad, gd.grad, bd.grad))
    (y0, *g0), (y1, *g1) = outs
    assert not hasattr(y0, "_sfh_slab")
    if shape[1] == 48:   # 6 sixteen-byte pieces per row do not divide the workgroup: plain form, same values
        assert not hasattr(y1, "_sfh_slab") and torch.equal(y0, y1)
        return
    slab, h = y1._sfh_slab
    assert h == halo and slab.shape == (1, shape[1], shape[2] + 2 * halo, shape[3], shape[4])
    assert slab.is_contiguous(memory_format=CL) and y1.is_contiguous(memory_format=CL)
    assert y1.data_ptr() == slab[:, :, halo:].data_ptr()
    assert torch.equal(y0, y1) and all(torch.equal(a, b) for a, b in zip(g0, g1))
    assert not slab[:, :, :halo].any() and not slab[:, :, -halo:].any()
    # batches and outputs of another width keep the plain form
    xb = torch.cat([x, x]).contiguous(memory_format=CL).to(device)
    assert not hasattr(sa.group_norm(xb, 8, None, None, 1e-5, None, out_dtype=None, out_halo=halo), "_sfh_slab")
    if dtype is torch.bfloat16:
        assert not hasattr(sa.group_norm(x.to(device), 8, None, None, 1e-5, None, out_dtype=torch.float32, out_halo=halo), "_sfh_slab")


# ---- argument layouts and partial gradients (the reference's edge suite: tests/test_triton_group_norm.py:402-425,661-684,
# ---- tests/test_triton_group_norm_edge.py:437-535) -------------------------------------------------------------------
def test_gradient_dtypes_under_autocast(device):
    x, gamma, beta, dy = make((2, 32, 4, 5, 6), torch.bfloat16, seed=31)
    xd = x.to(device).requires_grad_(True)
    gd, bd = gamma.float().to(device).requires_grad_(True), beta.float().to(device).requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = sa.group_norm(xd, 8, gd, bd, 1e-5, "relu")
    assert y.dtype is torch.float32                   # the stock operator's dtype under autocast
    y.backward(dy.to(device).float())
    assert xd.grad.dtype is torch.bfloat16 and gd.grad.dtype is torch.float32 and bd.grad.dtype is torch.float32
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y2 = sa.group_norm(xd, 8, gd, bd, 1e-5, "relu", out_dtype=None)
    assert y2.dtype is torch.bfloat16 and torch.equal(y2, y.to(torch.bfloat16))   # the narrow result is the wide one rounded once


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_partial_requires_grad_changes_no_other_gradient(device, dtype):
    x, gamma, beta, dy = make((2, 32, 4, 5, 6), dtype, seed=32)
    full = run_ours(x, 8, gamma, beta, dy, True, device)
    for need in [(True, False, False), (False, True, False), (False, False, True), (True, True, False), (False, True, True)]:
        xd = x.to(device).requires_grad_(need[0])
        gd, bd = gamma.to(device).requires_grad_(need[1]), beta.to(device).requires_grad_(need[2])
        y = sa.group_norm(xd, 8, gd, bd, 1e-5, "relu")
        y.backward(dy.to(device))
        assert torch.equal(y.detach(), full[0])
        for got, want, needed in ((xd.grad, full[1], need[0]), (gd.grad, full[2], need[1]), (bd.grad, full[3], need[2])):
            assert (got is None) == (not needed)
            if needed:
                assert torch.equal(got, want)


def test_parameter_views_and_offset_inputs_are_accepted(device):
    x, gamma, beta, dy = make((2, 16, 3, 5, 7), torch.float32, seed=33)
    want = run_ours(x, 4, gamma, beta, dy, False, device)
    # gamma / beta as every second element of a longer vector; x as a channels-last view with a storage offset
    wide_g, wide_b = torch.zeros(32, device=device), torch.zeros(32, device=device)
    wide_g[::2], wide_b[::2] = gamma.to(device), beta.to(device)
    gv, bv = wide_g[::2].requires_grad_(True), wide_b[::2].requires_grad_(True)
    assert not gv.is_contiguous()
    big = torch.zeros((3, 16, 3, 5, 7), device=device).contiguous(memory_format=CL)
    big[1:] = x.to(device)
    xv = big[1:].requires_grad_(True)
    assert xv.storage_offset() > 0 and xv.is_contiguous(memory_format=CL)
    y = sa.group_norm(xv, 4, gv, bv, 1e-5, None)
    y.backward(dy.to(device))
    for got, ref in zip((y.detach(), xv.grad, gv.grad, bv.grad), want):
        assert torch.equal(got, ref)


@pytest.mark.parametrize("layout", ["ncdhw", "sliced", "expanded", "transposed"])
def test_cotangent_layouts_are_relaid_out_not_misread(device, layout):
    x, gamma, beta, dy = make((2, 16, 4, 6, 6), torch.float32, seed=34)
    if layout == "ncdhw":
        cot = dy.to(device).contiguous()                                  # plain contiguous instead of channels-last
    elif layout == "sliced":
        wide = torch.randn((2, 16, 4, 6, 12), device=device)
        wide[..., ::2] = dy.to(device)
        cot = wide[..., ::2]
    elif layout == "expanded":
        dy = dy[:, :, :1].expand(-1, -1, 4, -1, -1)                      # stride 0 along depth
        cot = dy.to(device)[:, :, :1].expand(-1, -1, 4, -1, -1)
    else:
        dy = dy.transpose(3, 4).contiguous().transpose(3, 4)             # H and W swapped in memory
        cot = dy.to(device)
        assert not cot.is_contiguous() and not cot.is_contiguous(memory_format=CL)
    want = orc.group_norm_reference(x, 4, gamma, beta, 1e-5, True, dy.contiguous())
    xd = x.to(device).requires_grad_(True)
    gd, bd = gamma.to(device).requires_grad_(True), beta.to(device).requires_grad_(True)
    y = sa.group_norm(xd, 4, gd, bd, 1e-5, "relu")
    y.backward(cot)
    for got, ref in zip((y.detach(), xd.grad, gd.grad, bd.grad), want):
        assert orc.gn_rel_error(got, ref) <= orc.GN_TOLERANCE[torch.float32]
