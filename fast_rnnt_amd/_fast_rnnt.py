"""Operator boundary: the three functions of the reference's ``_fast_rnnt``
extension module (fast_rnnt/python/csrc/mutual_information.cu:27-75), with the
same keyword names, shapes, ownership rules and error types, backed by the
gfx950 library instead of the reference's C++/CUDA.

Differences a caller can observe: tensors must live on a GPU (the library has no
CPU path; a CPU tensor raises RuntimeError, like a CUDA tensor does on the
reference's CPU-only build), and every cell of the returned gradients is written
(zeros outside the boundary window) whether or not a boundary is given.
"""
from typing import List, Optional

import torch

from . import _lib


def with_cuda() -> bool:
    """True: PyTorch-ROCm exposes the MI355X as device type "cuda"."""
    return True


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _common_checks(px, py, boundary, p):
    _check(px.dim() == 3, "px must be 3-dimensional")
    _check(py.dim() == 3, "py must be 3-dimensional.")
    _check(p.dim() == 3, "p must be 3-dimensional.")
    _check(px.is_cuda and py.is_cuda and p.is_cuda,
           "inputs must be GPU tensors: fast_rnnt_amd has no CPU path")
    _check(px.device == py.device == p.device, "px, py and p must share one device")
    _check(px.dtype == py.dtype == p.dtype, "px, py and p must share one dtype")
    B, S, T1 = px.shape
    T = py.shape[2]
    modified = T1 == T
    _check(T1 == (T if modified else T + 1), "px.size(2) must be T or T + 1")
    _check(tuple(py.shape) == (B, S + 1, T), "py must have shape [B][S+1][T]")
    _check(tuple(p.shape) == (B, S + 1, T + 1), "p must have shape [B][S+1][T+1]")
    if boundary is not None:
        _check(boundary.dim() == 2, "boundary must be 2-dimensional.")
        _check(tuple(boundary.shape) == (B, 4), "boundary must have shape [B][4]")
        _check(boundary.device == px.device and boundary.dtype == torch.int64,
               "boundary must be an int64 tensor on the same device")
    return B, S, T, int(modified)


def mutual_information_forward(px: torch.Tensor, py: torch.Tensor,
                               boundary: Optional[torch.Tensor], p: torch.Tensor) -> torch.Tensor:
    """Fill the boundary window of ``p`` (in place) and return ``ans`` of shape [B]."""
    B, S, T, modified = _common_checks(px, py, boundary, p)
    sfx = _lib.suffix(px.dtype)
    with torch.cuda.device(px.device):
        pxc, pyc = px.contiguous(), py.contiguous()
        bnd = boundary.contiguous() if boundary is not None else None
        pc = p if p.is_contiguous() else torch.empty_like(p, memory_format=torch.contiguous_format)
        ans = torch.empty(B, dtype=px.dtype, device=px.device)
        _lib.call("frnnt_mi_forward_" + sfx, pxc.data_ptr(), pyc.data_ptr(), _lib.ptr(bnd),
                  pc.data_ptr(), ans.data_ptr(), B, S, T, modified, _lib.stream_of(px))
        if pc is not p:
            p.copy_(pc)
    return ans


def mutual_information_backward(px: torch.Tensor, py: torch.Tensor,
                                boundary: Optional[torch.Tensor], p: torch.Tensor,
                                ans_grad: torch.Tensor) -> List[torch.Tensor]:
    """Return ``[px_grad, py_grad]``.  Like the reference's GPU path
    (fast_rnnt/python/csrc/mutual_information.cu:57-58) ``ans_grad`` is
    overwritten with the gradient that reaches the start of each lattice."""
    B, S, T, modified = _common_checks(px, py, boundary, p)
    _check(ans_grad.dim() == 1, "ans_grad must be 1-dimensional.")
    _check(ans_grad.shape[0] == B, "ans_grad must have B elements")
    _check(ans_grad.device == px.device and ans_grad.dtype == px.dtype,
           "ans_grad must match px in device and dtype")
    sfx = _lib.suffix(px.dtype)
    with torch.cuda.device(px.device):
        pxc, pyc, pc = px.contiguous(), py.contiguous(), p.contiguous()
        bnd = boundary.contiguous() if boundary is not None else None
        agc = ans_grad if ans_grad.is_contiguous() else ans_grad.contiguous()
        px_grad = torch.empty_like(pxc)
        py_grad = torch.empty_like(pyc)
        _lib.call("frnnt_mi_backward_" + sfx, pxc.data_ptr(), pyc.data_ptr(), _lib.ptr(bnd),
                  pc.data_ptr(), agc.data_ptr(), px_grad.data_ptr(), py_grad.data_ptr(),
                  B, S, T, modified, 1, _lib.stream_of(px))
        if agc is not ans_grad:
            ans_grad.copy_(agc)
    return [px_grad, py_grad]
