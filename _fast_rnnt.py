"""Top-level ``_fast_rnnt``: the name under which the reference installs its native
operator module (fast_rnnt/python/csrc/fast_rnnt.cu:24, imported by
fast_rnnt/python/fast_rnnt/__init__.py:1 and mutual_information.py:18).  Here it is
the operator boundary of the MI355X build: ``mutual_information_forward(px, py,
boundary, p)``, ``mutual_information_backward(px, py, boundary, p, ans_grad)`` and
``with_cuda()``, positional or by keyword, backed by libfast_rnnt_amd.so.
"""
from fast_rnnt_amd._fast_rnnt import (mutual_information_backward,  # noqa: F401
                                      mutual_information_forward, with_cuda)

__all__ = ["mutual_information_forward", "mutual_information_backward", "with_cuda"]
