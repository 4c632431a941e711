"""Host-side mirror of the reference interface, without a GPU: gates are total, unsupported calls raise the
reference's exception types, modules keep stock state dicts, the U-Net has the reference's census."""

import pytest
import torch
import torch.nn as nn

import scaffold_amd as sa
from scaffold_amd import conv3d as c3
from scaffold_amd import groupnorm as gnm
from scaffold_amd import transposed as ct
from scaffold_amd.modules import FastConv3d, FastConvTranspose3d, FastGroupNorm, cast_operand
from scaffold_amd.unet import UNet, skip_concat


def test_gates_are_total():
    x = torch.randn(1, 4, 5, 5, 5)
    w = torch.randn(6, 4, 3, 3, 3)
    junk = [None, 1.5, "1", (1, 2), (1, 2, 3, 4), (1.0, 1, 1), [1, "a", 1], object()]
    for bad in junk:
        assert c3.is_supported(x, w, None, bad, 0, 1) is False
        assert c3.is_supported(x, w, None, 1, bad, 1) is False
        assert c3.is_supported(x, w, None, 1, 0, bad) is False
        assert c3.is_supported_all(x, w, None, bad, bad, bad) is False
        assert c3.is_supported_bwd_data(x, w, (1, 4, 5, 5, 5), bad, 0, 1) is False
        assert c3.is_supported_bwd_weight(x, (6, 4, 3, 3, 3), x, bad) is False
        assert ct.is_supported_transposed(x, w, None, bad) is False
    for notatensor in (None, 3, "x", [1, 2]):
        assert c3.is_supported(notatensor, w) is False and c3.is_supported(x, notatensor) is False
        assert gnm.is_supported(notatensor, 2) is False
    assert c3.is_supported_bwd_data(x, w, None) is False and c3.is_supported_bwd_data(x, w, (1, 2)) is False
    assert gnm.is_supported(x, "8") is False and gnm.is_supported(x, True) is False


def test_cpu_tensors_are_not_served_and_entry_points_raise():
    x = torch.randn(1, 32, 4, 4, 4, dtype=torch.bfloat16)
    w = torch.randn(32, 32, 3, 3, 3, dtype=torch.bfloat16)
    assert not c3.is_supported(x, w, None, 1, 1) and not gnm.is_supported(x, 8)
    with pytest.raises(NotImplementedError):
        sa.conv3d_forward(x, w, None, 1, 1)
    with pytest.raises(NotImplementedError):
        sa.conv3d_backward_data(x, w, x.shape, 1, 1)
    with pytest.raises(NotImplementedError):
        sa.conv3d_backward_weight(x, w.shape, x, 1, 1)
    with pytest.raises(NotImplementedError):
        sa.conv_transpose3d_forward(x, torch.randn(32, 16, 2, 2, 2, dtype=torch.bfloat16), None, 2)
    with pytest.raises(NotImplementedError):
        sa.group_norm(x, 8)
    with pytest.raises(ValueError):
        sa.group_norm(x, 8, activation="gelu")
    with pytest.raises(ValueError):
        sa.group_norm(x, 8, out_dtype=torch.int8)
    with pytest.raises(NotImplementedError):
        FastConv3d(32, 32, 3, padding=1)(x.float())
    with pytest.raises(NotImplementedError):
        FastGroupNorm(8, 32)(x.float())


def test_shape_helpers():
    assert c3._triple(2, "s") == (2, 2, 2) and c3._triple([1, 2, 3], "s") == (1, 2, 3)
    for bad, exc in ((None, TypeError), (1.5, TypeError), ((1, 2), ValueError), (True, TypeError)):
        with pytest.raises(exc):
            c3._triple(bad, "s")
    assert c3.bwd_data_padding((0, 1, 1), 1, 3) == (2, 1, 1) and c3.bwd_data_padding(1, 2, 3) == (3, 3, 3)
    for k, p, d in [(3, 1, 1), (3, 0, 1), (1, 0, 1), (3, 2, 2), (2, 0, 1)]:
        # with padding dil*(k-1)-p the gather over grad_output recovers the input extent exactly
        pin = d * (k - 1) - p
        for n in (5, 8):
            out = n + 2 * p - d * (k - 1)
            assert out + 2 * pin - d * (k - 1) == n
    assert c3.output_shape((2, 4, 7, 8, 9), (5, 4, 2, 3, 1), (2, 1, 3), (1, 0, 2), (1, 2, 1)) == tuple(
        torch.nn.functional.conv3d(torch.empty((2, 4, 7, 8, 9), device="meta"), torch.empty((5, 4, 2, 3, 1), device="meta"),
                                   None, (2, 1, 3), (1, 0, 2), (1, 2, 1)).shape)
    assert c3.workspace_elements(7, 32, 16, (3, 3, 3)) == 7 * 32 * 16 * 27
    gw = c3.grad_weight_empty(6, 4, (3, 3, 3), dtype=torch.float32, device="cpu")
    assert gw.stride() == (108, 1, 36, 12, 4)
    gt = ct.grad_transposed_weight_empty(6, 4, (2, 2, 2), dtype=torch.float32, device="cpu")
    assert gt.shape == (6, 4, 2, 2, 2) and gt.stride(1) == 1


def test_modules_keep_stock_state_dicts():
    pairs = [(FastConv3d(3, 5, 3, padding=1, bias=False), nn.Conv3d(3, 5, 3, padding=1, bias=False)),
             (FastConv3d(3, 5, 1), nn.Conv3d(3, 5, 1)),
             (FastConvTranspose3d(4, 2, 2, stride=2), nn.ConvTranspose3d(4, 2, 2, stride=2)),
             (FastGroupNorm(2, 4, activation="relu"), nn.GroupNorm(2, 4))]
    for fast, stock in pairs:
        a, b = fast.state_dict(), stock.state_dict()
        assert list(a) == list(b) and all(a[k].shape == b[k].shape for k in a)
        assert list(fast.buffers()) == []
        stock.load_state_dict(a)
        fast.load_state_dict(b)
    assert FastConv3d.__init__ is nn.Conv3d.__init__ and FastConvTranspose3d.__init__ is nn.ConvTranspose3d.__init__
    assert FastGroupNorm(2, 4).activation is None and "relu" in repr(FastGroupNorm(2, 4, activation="relu"))
    with pytest.raises(ValueError):
        FastGroupNorm(2, 4, activation="gelu")


def test_unet_census_and_state_dict_identity():
    ours, stock = UNet(1, 11, layers=4, base_width=32), UNet(1, 11, layers=4, base_width=32, stock=True)
    count = lambda m, t: sum(isinstance(x, t) for x in m.modules())
    assert count(ours, FastConv3d) == 19 and count(ours, FastConvTranspose3d) == 4 and count(ours, FastGroupNorm) == 18
    assert all(m.bias is not None for m in ours.modules() if isinstance(m, FastConvTranspose3d))
    a, b = ours.state_dict(), stock.state_dict()
    assert list(a) == list(b) and all(a[k].shape == b[k].shape for k in a)
    stock.load_state_dict(a)
    assert sum(p.numel() for p in ours.parameters()) == 22_578_603
    assert "down_list.0.double_conv.0.weight" in a and "up_list.0.up.bias" in a and "up_list.4.conv.bias" in a
    widths = [m.out_channels for m in ours.modules() if isinstance(m, FastConv3d)]
    assert widths[:2] == [32, 32] and max(widths) == 512 and widths[-1] == 11
    ours.set_shard_halo(True)
    assert all(m.shard_halo for m in ours.modules() if isinstance(m, FastConv3d))
    with pytest.raises(ValueError):
        UNet(1, 11, layers=0)


def test_stock_unet_runs_on_cpu_with_checkpointing_identity():
    torch.manual_seed(0)
    m = UNet(1, 3, layers=2, base_width=8, group_norm_groups=4, stock=True)
    x = torch.randn(1, 1, 8, 8, 8)
    y0 = m(x)
    m.use_checkpointing()
    y1 = m(x.requires_grad_(True))
    assert y0.shape == (1, 3, 8, 8, 8) and torch.equal(y0, y1)


def test_skip_concat_and_autocast_cast_rule():
    a, b = torch.randn(1, 2, 2, 2, 2), torch.randn(1, 3, 2, 2, 2, dtype=torch.bfloat16)
    out = skip_concat(a, b)
    assert out.dtype is torch.float32 and out.shape[1] == 5 and torch.equal(out[:, :2], a)
    with torch.autocast("cpu", dtype=torch.bfloat16):
        assert skip_concat(a, b).dtype is torch.bfloat16
    assert cast_operand(a, torch.bfloat16).dtype is torch.bfloat16
    assert cast_operand(a.double(), torch.bfloat16).dtype is torch.float64   # only exactly-fp32 tensors are narrowed
    assert cast_operand(b, torch.float16) is b and cast_operand(None, torch.bfloat16) is None


def test_lazy_package_exports():
    for name in sa.__all__:
        assert getattr(sa, name) is not None
    assert sa.triton_group_norm is sa.group_norm
    with pytest.raises(AttributeError):
        sa.no_such_symbol


# ---- optimizer state as the kernels read it (host logic; the kernels themselves need the GPU) ------------------
def _stock_adam_checkpoint(params, steps=2):
    """A checkpoint as a non-fused torch.optim.Adam writes it: one host `step` tensor per parameter."""
    opt = torch.optim.Adam(params, lr=1e-2, foreach=False, fused=False)
    gen = torch.Generator().manual_seed(7)
    for _ in range(steps):
        for p in params:
            p.grad = torch.randn(p.shape, generator=gen).contiguous(memory_format=torch.channels_last_3d if p.dim() == 5 else torch.contiguous_format)
        opt.step()
    return opt.state_dict()


def test_loaded_optimizer_state_is_brought_to_the_parameters_device_dtype_and_strides():
    from scaffold_amd.optim import FusedClipAdam
    CL = torch.channels_last_3d
    src = [torch.randn(4, 3, 2, 2, 2).requires_grad_(True), torch.randn(5).requires_grad_(True)]   # contiguous weight
    sd = _stock_adam_checkpoint(src)
    assert sd["state"][0]["step"].device.type == "cpu" and sd["state"][0]["exp_avg"].is_contiguous()
    sd["state"][1]["step"] = sd["state"][1]["step"].double()          # a foreign dtype
    mine = [src[0].detach().clone().contiguous(memory_format=CL).requires_grad_(True), src[1].detach().clone().requires_grad_(True)]
    opt = FusedClipAdam(mine, lr=1e-2, max_norm=1.0)
    opt.load_state_dict(sd)
    for i, p in enumerate(mine):
        st = opt.state[p]
        assert st["step"].device == p.device and st["step"].dtype is torch.float32 and st["step"].shape == () and st["step"].item() == 2.0
        for k in ("exp_avg", "exp_avg_sq"):
            assert st[k].dtype is torch.float32 and st[k].device == p.device and st[k].stride() == p.stride()
            assert torch.equal(st[k], sd["state"][i][k])              # same values at the same logical index
        opt._check_state(p, st)                                       # what step() verifies before the first launch
    # python-number steps (old checkpoints) are accepted too
    sd2 = _stock_adam_checkpoint([torch.randn(5).requires_grad_(True)])
    sd2["state"][0]["step"] = 2
    o2 = FusedClipAdam([torch.zeros(5, requires_grad=True)])
    o2.load_state_dict(sd2)
    assert o2.state[o2.param_groups[0]["params"][0]]["step"].item() == 2.0


def test_optimizer_state_the_kernels_cannot_read_raises_before_any_launch():
    from scaffold_amd.optim import FusedClipAdam
    a, b = torch.zeros(5, requires_grad=True), torch.zeros(3, requires_grad=True)
    sd = _stock_adam_checkpoint([torch.randn(5).requires_grad_(True), torch.randn(3).requires_grad_(True)])
    sd["state"][1]["step"] = sd["state"][1]["step"] + 1                # torch allows per-parameter counters; the kernels keep one
    with pytest.raises(NotImplementedError, match="one step counter"):
        FusedClipAdam([a, b]).load_state_dict(sd)
    sd = _stock_adam_checkpoint([torch.randn(5).requires_grad_(True), torch.randn(3).requires_grad_(True)])
    del sd["state"][0]["exp_avg_sq"]
    with pytest.raises(NotImplementedError, match="lacks"):
        FusedClipAdam([a, b]).load_state_dict(sd)
    # state put there behind load_state_dict's back: a step counter on another device, a moment with other strides
    opt = FusedClipAdam([a])
    good = {"step": torch.zeros(()), "exp_avg": torch.zeros(5), "exp_avg_sq": torch.zeros(5)}
    opt._check_state(a, good)
    for key, bad in (("step", torch.zeros((), device="meta")), ("step", torch.zeros((), dtype=torch.float64)), ("step", 3.0),
                     ("exp_avg", torch.zeros(10)[::2]), ("exp_avg_sq", torch.zeros(5, dtype=torch.bfloat16))):
        with pytest.raises(NotImplementedError):
            opt._check_state(a, {**good, key: bad})


def test_a_callers_packed_weight_is_validated_not_trusted(monkeypatch):
    """`packed_weight=` must be the uint8 buffer of exactly this problem's and direction's packed size, on the operands'
    device: anything else raises before the library is called (the MFMA kernels would index it out of bounds)."""
    prob = c3._Problem((1, 32, 8, 8, 8), (64, 32, 3, 3, 3), 1, 1, 1, torch.bfloat16)
    prob.packed = (4096, 8192)                     # what the library would report (forward, data gradient)
    like = torch.empty(1)
    assert prob.check_packed(torch.empty(4096, dtype=torch.uint8), False, like) == 4096
    assert prob.check_packed(torch.empty(8192, dtype=torch.uint8), True, like) == 8192
    for bad in (torch.empty(8192, dtype=torch.uint8),             # the other direction's form
                torch.empty(4095, dtype=torch.uint8), torch.empty(2048, dtype=torch.bfloat16),
                torch.empty(8192, dtype=torch.uint8)[::2], torch.empty(64, 64, dtype=torch.uint8),
                torch.empty(4096, dtype=torch.uint8, device="meta"), None, 4096):
        with pytest.raises(ValueError):
            prob.check_packed(bad, False, like)
    prob.packed = (0, 0)                            # a problem whose kernels read the weight where it lies
    with pytest.raises(ValueError, match="does not read a packed weight"):
        prob.check_packed(torch.empty(0, dtype=torch.uint8), False, like)
