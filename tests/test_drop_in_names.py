"""The reference's import names resolve to this build (CPU only).

fast_rnnt/python/fast_rnnt/__init__.py:1 imports a top-level ``_fast_rnnt``; user code
imports ``fast_rnnt`` and its submodules ``fast_rnnt.rnnt_loss`` /
``fast_rnnt.mutual_information``; setup.py:100-103 gives the package a ``__version__``.
"""
import inspect

import pytest
import torch

import _fast_rnnt
import fast_rnnt
import fast_rnnt_amd

REFERENCE_EXPORTS = [
    "with_cuda", "mutual_information_recursion", "joint_mutual_information_recursion",
    "do_rnnt_pruning", "get_rnnt_logprobs", "get_rnnt_logprobs_joint",
    "get_rnnt_logprobs_pruned", "get_rnnt_logprobs_smoothed", "get_rnnt_prune_ranges",
    "rnnt_loss", "rnnt_loss_pruned", "rnnt_loss_simple", "rnnt_loss_smoothed",
]


def test_package_exports_and_version():
    for name in REFERENCE_EXPORTS:
        assert getattr(fast_rnnt, name) is getattr(fast_rnnt_amd, name), name
    assert fast_rnnt.__version__.startswith("1.2")
    assert fast_rnnt.with_cuda() is True


def test_submodules_are_the_implementation():
    import sys
    from fast_rnnt.mutual_information import mutual_information_recursion
    from fast_rnnt.rnnt_loss import rnnt_loss_pruned
    assert sys.modules["fast_rnnt.rnnt_loss"] is sys.modules["fast_rnnt_amd.rnnt_loss"]
    assert sys.modules["fast_rnnt.mutual_information"] is \
        sys.modules["fast_rnnt_amd.mutual_information"]
    assert mutual_information_recursion is fast_rnnt_amd.mutual_information_recursion
    assert rnnt_loss_pruned is fast_rnnt_amd.rnnt_loss_pruned


def test_operator_module_signatures():
    # python/csrc/mutual_information.cu:27-67: keyword names are part of the interface
    assert list(inspect.signature(_fast_rnnt.mutual_information_forward).parameters) == \
        ["px", "py", "boundary", "p"]
    assert list(inspect.signature(_fast_rnnt.mutual_information_backward).parameters) == \
        ["px", "py", "boundary", "p", "ans_grad"]
    assert _fast_rnnt.with_cuda() is True
    # the reference's call pattern, positionally (mutual_information.py:157): argument
    # checks run, and the missing GPU is reported as the reference reports a device
    # mismatch -- with a RuntimeError
    px, py, p = torch.zeros(1, 2, 4), torch.zeros(1, 3, 3), torch.empty(1, 3, 4)
    with pytest.raises(RuntimeError, match="GPU"):
        _fast_rnnt.mutual_information_forward(px, py, None, p)
    with pytest.raises(RuntimeError, match="3-dimensional"):
        _fast_rnnt.mutual_information_forward(px[0], py, None, p)


def test_k2_names():
    # README.md:4 -- k2 ships the same functions; recipes written against `k2.*` can import
    # this module under that name (never a top-level `k2`)
    import importlib.util

    import fast_rnnt_amd.k2_compat as k2
    for name in REFERENCE_EXPORTS:
        if name != "with_cuda":
            assert getattr(k2, name) is getattr(fast_rnnt_amd, name), name
    assert sorted(k2.__all__) == sorted(n for n in REFERENCE_EXPORTS if n != "with_cuda")
    spec = importlib.util.find_spec("k2")
    assert spec is None or "fast_rnnt" not in (spec.origin or "")
