"""The allocation-free GroupNorm forward (`sfh_groupnorm_fwd_noalloc`) against the workspace form (`sfh_groupnorm_fwd`),
through the C ABI: bitwise the same output and statistics on two calls in a row, the second on a smaller input (the
built-in scratch keeps the first call's contents), and a clear refusal beyond the built-in buffer's size."""

import ctypes

import pytest
import torch

from scaffold_amd import _lib
from scaffold_amd._lib import GroupNormDesc

pytestmark = pytest.mark.gpu
CL = torch.channels_last_3d


def _both_ways(device, shape, groups, relu, dtype, seed):
    L = _lib.lib()
    g = torch.Generator().manual_seed(seed)
    n, c, d, h, w = shape
    x = (torch.randn(shape, generator=g) * 3 + 0.5).to(dtype).contiguous(memory_format=CL).to(device)
    gamma = (1 + 0.1 * torch.randn(c, generator=g)).to(device)
    beta = (0.1 * torch.randn(c, generator=g)).to(device)
    desc = GroupNormDesc(n, c, groups, int(relu), d * h * w, 1e-5)
    code = _lib.dtype_code(dtype)
    stream = _lib.stream_ptr(x.device)
    outs = []
    for noalloc in (False, True):
        y = torch.full_like(x, float("nan"))
        mean = torch.full((n, groups), float("nan"), device=device)
        rstd = torch.full((n, groups), float("nan"), device=device)
        if noalloc:
            rc = L.sfh_groupnorm_fwd_noalloc(ctypes.byref(desc), code, code, 2, _lib.ptr(x), _lib.ptr(gamma), _lib.ptr(beta), _lib.ptr(y),
                                             _lib.ptr(mean), _lib.ptr(rstd), stream)
        else:
            need = int(L.sfh_groupnorm_fwd_workspace_bytes(ctypes.byref(desc), code))
            assert 0 < need <= int(L.sfh_groupnorm_fwd_noalloc_max_bytes())
            ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=device)
            rc = L.sfh_groupnorm_fwd(ctypes.byref(desc), code, code, 2, _lib.ptr(x), _lib.ptr(gamma), _lib.ptr(beta), _lib.ptr(y),
                                     _lib.ptr(mean), _lib.ptr(rstd), _lib.ptr(ws), need, stream)
        _lib.check(rc, "groupnorm forward")
        torch.cuda.synchronize()
        outs.append((y, mean, rstd))
    return outs


def test_two_calls_in_a_row_match_the_workspace_form_bitwise(device):
    torch.cuda.set_device(device)
    # config 2's tensor halved along depth first (the larger problem), then a small ragged one that reuses a corner of the scratch
    for shape, groups, relu, dtype, seed in (((2, 64, 32, 64, 64), 8, True, torch.bfloat16, 1), ((1, 32, 5, 7, 9), 8, False, torch.bfloat16, 2),
                                             ((2, 64, 32, 64, 64), 8, False, torch.float32, 3), ((3, 16, 3, 4, 5), 4, True, torch.float16, 4)):
        (y0, m0, r0), (y1, m1, r1) = _both_ways(device, shape, groups, relu, dtype, seed)
        assert torch.isfinite(y1.float()).all() and torch.isfinite(m1).all() and torch.isfinite(r1).all()
        assert torch.equal(y0, y1) and torch.equal(m0, m1) and torch.equal(r0, r1), shape


def test_a_problem_beyond_the_built_in_scratch_is_refused_before_any_launch(device):
    torch.cuda.set_device(device)
    L = _lib.lib()
    n, c, s, groups = 64, 512, 4096, 32            # 64 samples x many splits x 2 x 32 groups of partials
    desc = GroupNormDesc(n, c, groups, 0, s, 1e-5)
    need = int(L.sfh_groupnorm_fwd_workspace_bytes(ctypes.byref(desc), 0))
    if need <= int(L.sfh_groupnorm_fwd_noalloc_max_bytes()):
        pytest.skip(f"this plan needs only {need} bytes")
    x = torch.zeros((n, s, c), dtype=torch.bfloat16, device=device)
    y = torch.full_like(x, 7.0)
    mean = torch.zeros((n, groups), device=device)
    rc = L.sfh_groupnorm_fwd_noalloc(ctypes.byref(desc), 0, 0, 2, _lib.ptr(x), None, None, _lib.ptr(y), _lib.ptr(mean), _lib.ptr(mean),
                                     _lib.stream_ptr(x.device))
    assert rc == _lib.SFH_ERR_WORKSPACE and b"built-in buffer" in L.sfh_last_error()
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())                   # nothing ran


def test_captured_into_a_graph_after_prepare_replays_to_the_workspace_forms_bits(device):
    """The caller this entry point is for: the call recorded into a HIP graph. The scratch address is looked up ahead of
    the capture (``sfh_groupnorm_fwd_noalloc_prepare``); the graph is replayed three times with eager work and
    synchronisations between, and every replay must give the workspace form's bits."""
    torch.cuda.set_device(device)
    L = _lib.lib()
    assert L.sfh_groupnorm_fwd_noalloc_prepare() == 0 and L.sfh_groupnorm_fwd_noalloc_prepare() == 0  # idempotent
    shape, groups = (2, 32, 6, 10, 12), 8
    (want_y, want_mean, want_rstd), _ = _both_ways(device, shape, groups, True, torch.bfloat16, seed=9)
    g = torch.Generator().manual_seed(9)
    n, c, d, h, w = shape
    x = (torch.randn(shape, generator=g) * 3 + 0.5).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    gamma = (1 + 0.1 * torch.randn(c, generator=g)).to(device)
    beta = (0.1 * torch.randn(c, generator=g)).to(device)
    desc = GroupNormDesc(n, c, groups, 1, d * h * w, 1e-5)
    y = torch.empty_like(x)
    mean = torch.empty((n, groups), device=device)
    rstd = torch.empty((n, groups), device=device)

    def call():
        _lib.check(L.sfh_groupnorm_fwd_noalloc(ctypes.byref(desc), 0, 0, 2, _lib.ptr(x), _lib.ptr(gamma), _lib.ptr(beta), _lib.ptr(y),
                                               _lib.ptr(mean), _lib.ptr(rstd), _lib.stream_ptr(x.device)), "no-alloc forward")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for _ in range(3):
        y.fill_(float("nan"))
        mean.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want_y) and torch.equal(mean, want_mean) and torch.equal(rstd, want_rstd)
        _both_ways(device, (1, 32, 5, 7, 9), 8, False, torch.bfloat16, seed=2)  # eager calls that overwrite the shared scratch
        torch.cuda.synchronize()
