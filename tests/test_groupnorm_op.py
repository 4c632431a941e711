"""The registered GroupNorm operators as the dispatcher sees them: the fake (shape-only) kernels on meta tensors here,
and on the GPU torch's own operator checks plus a traced run (`torch.compile`, fullgraph, the `aot_eager` backend: tracing
and functionalisation without any generated kernels) that must equal the eager result bit for bit -- the reference's
contract for its operators (ScaFFold/unet/triton_group_norm.py:1339-1479; tests/test_triton_group_norm.py:791-845)."""

import pytest
import torch

import scaffold_amd.groupnorm  # noqa: F401  (registers torch.ops.scaffold_gn.*)

CL = torch.channels_last_3d


@pytest.mark.parametrize("dtype, out_dtype", [(torch.bfloat16, None), (torch.bfloat16, torch.float32), (torch.float32, None)])
def test_fake_kernels_promise_the_real_layouts(dtype, out_dtype):
    x = torch.empty((2, 16, 3, 5, 7), dtype=dtype, device="meta").contiguous(memory_format=CL)
    gamma = torch.empty(16, device="meta")
    beta = torch.empty(16, device="meta")
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(x, 4, gamma, beta, 1e-5, "relu", out_dtype)
    assert out.shape == x.shape and out.dtype == (out_dtype or dtype) and out.is_contiguous(memory_format=CL)
    assert mean.shape == rstd.shape == (2, 4) and mean.dtype == rstd.dtype == torch.float32
    dy = torch.empty_like(x)
    dx, dw, db = torch.ops.scaffold_gn.group_norm_backward(dy, x, gamma, beta, mean, rstd, 4, "relu")
    assert dx.shape == x.shape and dx.dtype == dtype and dx.is_contiguous(memory_format=CL)
    assert dw.shape == db.shape == (16,) and dw.dtype == db.dtype == torch.float32
    dx, dw, db = torch.ops.scaffold_gn.group_norm_backward(dy, x, None, None, mean, rstd, 4, None)
    assert dw.numel() == 0 and db.numel() == 0


@pytest.mark.gpu
def test_operator_checks(device):
    g = torch.Generator().manual_seed(5)
    x = torch.randn((2, 16, 3, 5, 7), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device).requires_grad_(True)
    gamma = torch.randn(16, generator=g).to(device).requires_grad_(True)
    beta = torch.randn(16, generator=g).to(device).requires_grad_(True)
    checks = ("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_static")
    torch.library.opcheck(torch.ops.scaffold_gn.group_norm.default, (x, 4, gamma, beta, 1e-5, "relu", None), test_utils=checks)
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(x, 4, gamma, beta, 1e-5, "relu", None)
    dy = torch.randn(x.shape, generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    torch.library.opcheck(torch.ops.scaffold_gn.group_norm_backward.default,
                          (dy, x.detach(), gamma.detach(), beta.detach(), mean, rstd, 4, "relu"),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.gpu
def test_traced_whole_graph_equals_eager_bitwise(device):
    g = torch.Generator().manual_seed(6)
    x0 = torch.randn((1, 32, 4, 6, 8), generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)
    gamma0 = torch.randn(32, generator=g).to(device)
    beta0 = torch.randn(32, generator=g).to(device)
    dy = torch.randn(x0.shape, generator=g).to(torch.bfloat16).contiguous(memory_format=CL).to(device)

    def fn(x, gamma, beta):
        out, mean, rstd = torch.ops.scaffold_gn.group_norm(x, 8, gamma, beta, 1e-5, "relu", None)
        return out * 2, mean, rstd

    def run(f):
        x, gamma, beta = x0.clone().requires_grad_(True), gamma0.clone().requires_grad_(True), beta0.clone().requires_grad_(True)
        out, mean, rstd = f(x, gamma, beta)
        out.backward(dy)
        return out.detach(), mean, rstd, x.grad, gamma.grad, beta.grad

    eager = run(fn)
    traced = run(torch.compile(fn, backend="aot_eager", fullgraph=True))
    for a, b in zip(eager, traced):
        assert a.dtype == b.dtype and torch.equal(a, b)
    # mean / rstd carry no gradient, and differentiating twice is refused rather than answered with zeros
    x = x0.clone().requires_grad_(True)
    out, mean, rstd = torch.ops.scaffold_gn.group_norm(x, 8, gamma0, beta0, 1e-5, None, None)
    assert not mean.requires_grad and not rstd.requires_grad
    (gx,) = torch.autograd.grad(out, x, dy, create_graph=True)
    with pytest.raises(RuntimeError):
        gx.sum().backward()
