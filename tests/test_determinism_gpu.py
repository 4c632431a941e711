"""Same call, same bits -- in one process and across processes (the launch geometry is a pure function of the
problem; no float atomics anywhere): the property the reference pins in test_gather_gemm.py:983-995 and
test_bwd_weight.py:1146-1267."""

import hashlib
import json
import os
import subprocess
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def digests():
    """SHA-256 of the bytes of every output of a fixed set of calls on seeded operands (CPU generator, so that
    two processes see the same inputs)."""
    import scaffold_amd as sa

    dev = torch.device("cuda:0")
    cl = torch.channels_last_3d
    g = torch.Generator().manual_seed(777)
    out = {}

    def put(name, t):
        out[name] = hashlib.sha256(t.detach().float().cpu().contiguous().numpy().tobytes()).hexdigest()

    for tag, cin, cout, sp, dtype in [("mfma32", 32, 32, (10, 12, 40), torch.bfloat16), ("mfma64", 64, 64, (6, 9, 17), torch.bfloat16),
                                      ("split", 256, 128, (4, 8, 8), torch.bfloat16), ("thin", 1, 32, (6, 8, 33), torch.bfloat16),
                                      ("fp32", 5, 7, (5, 6, 7), torch.float32)]:
        x = torch.randn((1, cin) + sp, generator=g).to(dtype).contiguous(memory_format=cl).to(dev)
        w = (torch.randn((cout, cin, 3, 3, 3), generator=g) / (27 * cin) ** 0.5).to(dtype).contiguous(memory_format=cl).to(dev)
        b = torch.randn(cout, generator=g).to(dtype).to(dev)
        gy = torch.randn((1, cout) + sp, generator=g).to(dtype).contiguous(memory_format=cl).to(dev)
        put(tag + ".fwd", sa.conv3d_forward(x, w, b, 1, 1))
        put(tag + ".dgrad", sa.conv3d_backward_data(gy, w, x.shape, 1, 1))
        put(tag + ".wgrad", sa.conv3d_backward_weight(x, w.shape, gy, 1, 1))
    x = torch.randn((1, 64, 4, 6, 10), generator=g).to(torch.bfloat16).contiguous(memory_format=cl).to(dev)
    w = (torch.randn((64, 32, 2, 2, 2), generator=g) / 8).to(torch.bfloat16).contiguous(memory_format=cl).to(dev)
    put("convT.fwd", sa.conv_transpose3d_forward(x, w, None, 2))
    x = (torch.randn((2, 48, 7, 9, 11), generator=g) * 3 + 1).to(torch.bfloat16).contiguous(memory_format=cl).to(dev).requires_grad_(True)
    gamma = torch.randn(48, generator=g).to(dev).requires_grad_(True)
    beta = torch.randn(48, generator=g).to(dev).requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):         # fp32 parameters beside a bf16 input, as in the U-Net
        y = sa.group_norm(x, 8, gamma, beta, 1e-5, "relu", out_dtype=None)
    y.backward(torch.randn(y.shape, generator=g).to(torch.bfloat16).contiguous(memory_format=cl).to(dev))
    for name, t in (("gn.y", y), ("gn.dx", x.grad), ("gn.dgamma", gamma.grad), ("gn.dbeta", beta.grad)):
        put(name, t)
    logits = torch.randn((1, 11, 6, 8, 10), generator=g).to(torch.bfloat16).contiguous(memory_format=cl).to(dev).requires_grad_(True)
    labels = torch.randint(0, 11, (1, 6, 8, 10), generator=g).to(dev)
    loss = sa.ce_dice_loss(logits, labels)
    loss.backward()
    put("loss", loss)
    put("loss.dlogits", logits.grad)
    return out


def test_same_bits_in_process_and_across_processes():
    first = digests()
    assert digests() == first                                  # again in this process
    code = ("import json, sys; sys.path.insert(0, %r); sys.path.insert(0, %r); import test_determinism_gpu as t; "
            "print('DIGESTS ' + json.dumps(t.digests()))") % (ROOT, os.path.join(ROOT, "tests"))
    try:
        child = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=240, cwd=ROOT)
    except (OSError, subprocess.TimeoutExpired) as exc:        # a sandbox that forbids child processes: say so, do not guess
        pytest.skip(f"could not run a second process here: {exc!r}")
    lines = [ln for ln in child.stdout.splitlines() if ln.startswith("DIGESTS ")]
    if child.returncode != 0 or not lines:
        if "Operation not permitted" in child.stderr or "Permission denied" in child.stderr:
            pytest.skip("child processes may not use the GPU here: " + child.stderr[-300:])
        raise AssertionError(f"second process failed (rc={child.returncode}): {child.stderr[-2000:]}")
    other = json.loads(lines[-1][len("DIGESTS "):])
    assert other.keys() == first.keys()
    assert {k for k in first if first[k] != other[k]} == set()
