"""Operator boundary: the three functions of the reference's ``_fast_rnnt``
extension module (fast_rnnt/python/csrc/mutual_information.cu:27-75), with the
same keyword names, shapes, ownership rules and error types (RuntimeError from a
failed check), backed by the gfx950 library instead of the reference's C++/CUDA.
Like the reference's they are compiled functions (fast_rnnt_amd/csrc/torch_ops.cpp,
built as ``fast_rnnt_amd._C``): tensors in, stream and device guard from c10::hip,
outputs allocated by torch, the library called through its C ABI.  The same
functions are registered as ``torch.ops.fast_rnnt_amd.mutual_information_forward``
/ ``_backward``.

Differences a caller can observe: tensors must live on a GPU (the library has no
CPU path; a CPU tensor raises RuntimeError, like a CUDA tensor does on the
reference's CPU-only build), and every cell of the returned gradients is written
(zeros outside the boundary window) whether or not a boundary is given.
"""
from typing import List, Optional

import torch

from . import _lib

_C = _lib.ops()


def with_cuda() -> bool:
    """True: PyTorch-ROCm exposes the MI355X as device type "cuda"."""
    return _C.with_cuda()


def mutual_information_forward(px: torch.Tensor, py: torch.Tensor,
                               boundary: Optional[torch.Tensor], p: torch.Tensor) -> torch.Tensor:
    """Fill the boundary window of ``p`` (in place) and return ``ans`` of shape [B]."""
    return _C.mutual_information_forward(px, py, boundary, p)


def mutual_information_backward(px: torch.Tensor, py: torch.Tensor,
                                boundary: Optional[torch.Tensor], p: torch.Tensor,
                                ans_grad: torch.Tensor) -> List[torch.Tensor]:
    """Return ``[px_grad, py_grad]``.  Like the reference's GPU path
    (fast_rnnt/python/csrc/mutual_information.cu:57-58) ``ans_grad`` is
    overwritten with the gradient that reaches the start of each lattice."""
    return _C.mutual_information_backward(px, py, boundary, p, ans_grad)
