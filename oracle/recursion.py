"""ctypes front end of the plain-C recursion oracle (TEST INFRASTRUCTURE ONLY).

``mi_forward`` / ``mi_backward`` follow the operator pair of
fast_rnnt/python/csrc/mutual_information.cu:27-67 on CPU tensors, and
``mutual_information_recursion`` follows
fast_rnnt/python/fast_rnnt/mutual_information.py:24-298, including the eager
backward inside forward and the in-place scaling of the saved gradients;
``joint_mutual_information_recursion`` follows :314-425 of the same file.
"""
import ctypes
import os
import subprocess
from typing import List, Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_mi.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile liboracle_mi.so with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        for sfx in ("f32", "f64"):
            f = getattr(lib, f"frnnt_oracle_mi_forward_{sfx}")
            f.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci]
            f.restype = ci
            g = getattr(lib, f"frnnt_oracle_mi_backward_{sfx}")
            g.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci]
            g.restype = ci
        _lib = lib
    return _lib


def _suffix(dtype: torch.dtype) -> str:
    if dtype == torch.float32:
        return "f32"
    if dtype == torch.float64:
        return "f64"
    raise RuntimeError(f"oracle supports float32/float64 only, got {dtype}")


def _check_shapes(px, py, boundary, p=None):
    if px.dim() != 3 or py.dim() != 3:
        raise RuntimeError("px and py must be 3-dimensional")
    B, S, T1 = px.shape
    T = py.shape[2]
    if T1 not in (T, T + 1) or tuple(py.shape) != (B, S + 1, T):
        raise RuntimeError("px/py shapes disagree")
    if p is not None and tuple(p.shape) != (B, S + 1, T + 1):
        raise RuntimeError("p has the wrong shape")
    if boundary is not None:
        if boundary.dtype != torch.int64 or tuple(boundary.shape) != (B, 4):
            raise RuntimeError("boundary must be int64 [B,4]")
    return B, S, T, int(T1 == T)


def mi_forward(px: torch.Tensor, py: torch.Tensor,
               boundary: Optional[torch.Tensor], p: torch.Tensor) -> torch.Tensor:
    """Fill the boundary window of ``p`` in place and return ``ans`` [B]."""
    lib = _load()
    B, S, T, modified = _check_shapes(px, py, boundary, p)
    assert p.is_contiguous() and p.dtype == px.dtype == py.dtype
    pxc, pyc = px.contiguous(), py.contiguous()
    bnd = boundary.contiguous() if boundary is not None else None
    ans = torch.empty(B, dtype=px.dtype)
    fn = getattr(lib, "frnnt_oracle_mi_forward_" + _suffix(px.dtype))
    rc = fn(pxc.data_ptr(), pyc.data_ptr(), bnd.data_ptr() if bnd is not None else None,
            p.data_ptr(), ans.data_ptr(), B, S, T, modified)
    assert rc == 0
    return ans


def mi_backward(px: torch.Tensor, py: torch.Tensor, boundary: Optional[torch.Tensor],
                p: torch.Tensor, ans_grad: torch.Tensor) -> List[torch.Tensor]:
    """Return ``[px_grad, py_grad]`` for the given ``p`` and ``ans_grad``."""
    lib = _load()
    B, S, T, modified = _check_shapes(px, py, boundary, p)
    if ans_grad.dim() != 1 or ans_grad.shape[0] != B:
        raise RuntimeError("ans_grad must be 1-dimensional of size B")
    pxc, pyc, pc = px.contiguous(), py.contiguous(), p.contiguous()
    agc = ans_grad.contiguous()
    bnd = boundary.contiguous() if boundary is not None else None
    px_grad = torch.empty_like(pxc)
    py_grad = torch.empty_like(pyc)
    fn = getattr(lib, "frnnt_oracle_mi_backward_" + _suffix(px.dtype))
    rc = fn(pxc.data_ptr(), pyc.data_ptr(), bnd.data_ptr() if bnd is not None else None,
            pc.data_ptr(), agc.data_ptr(), px_grad.data_ptr(), py_grad.data_ptr(),
            B, S, T, modified)
    assert rc >= 0
    return [px_grad, py_grad]


class _Recursion(torch.autograd.Function):
    """Mirrors fast_rnnt/python/fast_rnnt/mutual_information.py:24-181."""

    @staticmethod
    def forward(ctx, px, py, sink, boundary, return_grad):
        B, S, _ = px.shape
        T = py.shape[-1]
        p = torch.empty(B, S + 1, T + 1, dtype=px.dtype)
        ans = mi_forward(px, py, boundary, p)
        gx = gy = None
        if return_grad or px.requires_grad or py.requires_grad:
            seed = torch.ones(B, dtype=px.dtype)
            gx, gy = mi_backward(px, py, boundary, p, seed)
            ctx.save_for_backward(gx, gy)
        sink[0], sink[1] = gx, gy
        return ans

    @staticmethod
    def backward(ctx, ans_grad):
        gx, gy = ctx.saved_tensors
        scale = ans_grad.reshape(-1, 1, 1)
        gx *= scale  # in place: the caller's return_grad tensors change too
        gy *= scale
        return gx, gy, None, None, None


def mutual_information_recursion(px, py, boundary=None, return_grad=False):
    """Mirrors fast_rnnt/python/fast_rnnt/mutual_information.py:184-298."""
    assert px.ndim == 3
    B, S, T1 = px.shape
    T = py.shape[-1]
    assert T1 in (T, T + 1)
    assert py.shape == (B, S + 1, T)
    assert px.dtype == py.dtype
    if boundary is not None:
        assert boundary.dtype == torch.int64
        assert boundary.shape == (B, 4)
        for s0, t0, s1, t1 in boundary.tolist():
            assert 0 <= s0 <= s1 <= S
            assert 0 <= t0 <= t1 <= T
    sink = [None, None]
    scores = _Recursion.apply(px.contiguous(), py.contiguous(), sink, boundary, return_grad)
    return (scores, (sink[0], sink[1])) if return_grad else scores


def joint_mutual_information_recursion(px, py, boundary=None):
    """Mirrors fast_rnnt/python/fast_rnnt/mutual_information.py:314-425: the recursion
    on the summed terms, with the total score split over the summands by occupation-
    weighted sums (term n gets sum(px_grad * px[n]) + sum(py_grad * py[n])); what is
    left over -- log-of-sum minus sum-of-log -- is credited to term 0 (:420-424).
    -inf entries are raised to the most negative finite number first (:411-412), so a
    blocked cell contributes 0 * finite = 0.  Returns a tensor of shape (len(px), B).
    """
    n_terms = len(px)
    assert len(py) == n_terms and n_terms > 0
    B, S, T1 = px[0].shape
    T = py[0].shape[2]
    assert T1 in (T, T + 1)
    assert py[0].shape == (B, S + 1, T)
    assert px[0].dtype == py[0].dtype
    if boundary is not None:
        assert boundary.dtype == torch.int64
        assert boundary.shape == (B, 4)
        for s0, t0, s1, t1 in boundary.tolist():
            assert 0 <= s0 <= s1 <= S
            assert 0 <= t0 <= t1 <= T
    with torch.no_grad():
        x_total = torch.stack(list(px), dim=0).sum(dim=0).contiguous()
        y_total = torch.stack(list(py), dim=0).sum(dim=0).contiguous()
        p = torch.empty(B, S + 1, T + 1, dtype=x_total.dtype)
        total = mi_forward(x_total, y_total, boundary, p)
        occ_x, occ_y = mi_backward(x_total, y_total, boundary, p,
                                   torch.ones(B, dtype=x_total.dtype))
    floor = torch.finfo(x_total.dtype).min
    shares = []
    for x, y in zip(px, py):
        shares.append((occ_x * x.clamp(min=floor)).sum(dim=(1, 2))
                      + (occ_y * y.clamp(min=floor)).sum(dim=(1, 2)))
    shares = torch.stack(shares, dim=0)  # (N, B)
    with torch.no_grad():
        leftover = total - shares.sum(dim=0)
    first = shares[0] + leftover
    return torch.cat((first.unsqueeze(0), shares[1:]), dim=0)
