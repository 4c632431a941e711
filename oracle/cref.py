"""ctypes wrapper of ``oracle/conv_ref.c`` (plain-C brute-force loops).  TEST INFRASTRUCTURE ONLY.

Tensors go in and come out as torch tensors in PyTorch's NCDHW convention; the wrapper converts
to the dense channels-last double arrays the C code works on.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libconv_ref.so")
_lib = None


class _Desc(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int) for k in (
        "n", "cin", "id", "ih", "iw", "cout", "kd", "kh", "kw", "sd", "sh", "sw", "pd", "ph", "pw", "dd", "dh", "dw")]


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "conv_ref.c")):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _cl(t: torch.Tensor) -> np.ndarray:
    """NCDHW tensor -> contiguous double array in N D H W C order."""
    return np.ascontiguousarray(t.detach().to(device="cpu", dtype=torch.float64).permute(0, 2, 3, 4, 1).numpy())


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _vec(t):
    return None if t is None else np.ascontiguousarray(t.detach().to(device="cpu", dtype=torch.float64).numpy())


def _desc(x_shape, w_shape, stride, padding, dilation) -> _Desc:
    n, cin, d, h, w = (int(v) for v in x_shape)
    cout, _, kd, kh, kw = (int(v) for v in w_shape)
    return _Desc(n, cin, d, h, w, cout, kd, kh, kw, *stride, *padding, *dilation)


def _out_sp(desc):
    f = lambda i, k, s, p, d: (i + 2 * p - d * (k - 1) - 1) // s + 1
    return (f(desc.id, desc.kd, desc.sd, desc.pd, desc.dd), f(desc.ih, desc.kh, desc.sh, desc.ph, desc.dh),
            f(desc.iw, desc.kw, desc.sw, desc.pw, desc.dw))


def conv3d_fwd(x, w, bias=None, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1)) -> torch.Tensor:
    desc = _desc(x.shape, w.shape, stride, padding, dilation)
    od, oh, ow = _out_sp(desc)
    y = np.empty((desc.n, od, oh, ow, desc.cout), dtype=np.float64)
    lib().ref_conv3d_fwd(ctypes.byref(desc), _p(_cl(x)), _p(_cl(w)), _p(_vec(bias)), _p(y))
    return torch.from_numpy(y).permute(0, 4, 1, 2, 3)


def conv3d_dgrad(gy, w, x_shape, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1)) -> torch.Tensor:
    desc = _desc(x_shape, w.shape, stride, padding, dilation)
    gx = np.empty((desc.n, desc.id, desc.ih, desc.iw, desc.cin), dtype=np.float64)
    lib().ref_conv3d_dgrad(ctypes.byref(desc), _p(_cl(gy)), _p(_cl(w)), _p(gx))
    return torch.from_numpy(gx).permute(0, 4, 1, 2, 3)


def conv3d_wgrad(x, w_shape, gy, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1)) -> torch.Tensor:
    desc = _desc(x.shape, w_shape, stride, padding, dilation)
    gw = np.empty((desc.cout, desc.kd, desc.kh, desc.kw, desc.cin), dtype=np.float64)
    lib().ref_conv3d_wgrad(ctypes.byref(desc), _p(_cl(x)), _p(_cl(gy)), _p(gw))
    return torch.from_numpy(gw).permute(0, 4, 1, 2, 3)


def convT3d_fwd(x, w, bias=None) -> torch.Tensor:
    """``w`` is (Cin, Cout, kd, kh, kw); stride == kernel, padding 0."""
    n, cin, d, h, ww = (int(v) for v in x.shape)
    _, cout, kd, kh, kw = (int(v) for v in w.shape)
    y = np.empty((n, d * kd, h * kh, ww * kw, cout), dtype=np.float64)
    fn = lib().ref_convT3d_fwd
    fn.argtypes = [ctypes.c_int] * 9 + [ctypes.POINTER(ctypes.c_double)] * 4
    fn(n, cin, d, h, ww, cout, kd, kh, kw, _p(_cl(x)), _p(_cl(w)), _p(_vec(bias)), _p(y))
    return torch.from_numpy(y).permute(0, 4, 1, 2, 3)


def groupnorm_fwd(x, groups, gamma=None, beta=None, eps=1e-5, relu=False):
    n, c = int(x.shape[0]), int(x.shape[1])
    s = int(np.prod(x.shape[2:]))
    xa = _cl(x)
    y = np.empty_like(xa)
    mean = np.empty((n, groups), dtype=np.float64)
    rstd = np.empty((n, groups), dtype=np.float64)
    fn = lib().ref_groupnorm_fwd
    fn.argtypes = [ctypes.c_int, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_int] + \
        [ctypes.POINTER(ctypes.c_double)] * 6
    fn(n, s, c, groups, float(eps), int(relu), _p(xa), _p(_vec(gamma)), _p(_vec(beta)), _p(y), _p(mean), _p(rstd))
    return torch.from_numpy(y).permute(0, 4, 1, 2, 3), torch.from_numpy(mean), torch.from_numpy(rstd)


def groupnorm_bwd(dy, x, groups, gamma, beta, mean, rstd, relu=False):
    n, c = int(x.shape[0]), int(x.shape[1])
    s = int(np.prod(x.shape[2:]))
    xa, ga = _cl(x), _cl(dy)
    dx = np.empty_like(xa)
    dgamma = np.empty(c, dtype=np.float64)
    dbeta = np.empty(c, dtype=np.float64)
    fn = lib().ref_groupnorm_bwd
    fn.argtypes = [ctypes.c_int, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_int] + [ctypes.POINTER(ctypes.c_double)] * 9
    fn(n, s, c, groups, int(relu), _p(ga), _p(xa), _p(_vec(gamma)), _p(_vec(beta)), _p(_vec(mean.reshape(-1))),
       _p(_vec(rstd.reshape(-1))), _p(dx), _p(dgamma), _p(dbeta))
    return torch.from_numpy(dx).permute(0, 4, 1, 2, 3), torch.from_numpy(dgamma), torch.from_numpy(dbeta)
