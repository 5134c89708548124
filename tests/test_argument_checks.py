"""Argument checks that run before any pointer reaches the library (CPU only: every
call here must raise before a kernel could be launched)."""
import pytest
import torch

import fast_rnnt_amd
from fast_rnnt_amd import mutual_information as MI


def _inputs(B=2, S=3, T=5, C=6):
    g = torch.Generator().manual_seed(0)
    am = torch.randn(B, T, C, generator=g)
    lm = torch.randn(B, S + 1, C, generator=g)
    sym = torch.randint(0, C, (B, S), generator=g)
    bnd = torch.tensor([[0, 0, S, T]] * B)
    return am, lm, sym, bnd


def test_index_tensors_must_be_int64():
    # the kernels read symbols / ranges / boundary as 64-bit words: an int32 tensor would
    # be read past its end, so it must raise like the reference's torch.gather does
    am, lm, sym, bnd = _inputs()
    B, T, C = am.shape
    S = sym.shape[1]
    for fn in (fast_rnnt_amd.get_rnnt_logprobs, fast_rnnt_amd.get_rnnt_logprobs_smoothed):
        with pytest.raises(RuntimeError, match="symbols must be an int64"):
            fn(lm, am, sym.int(), 0)
    with pytest.raises(RuntimeError, match="symbols must be an int64"):
        fast_rnnt_amd.rnnt_loss_simple(lm, am, sym.int(), 0)
    with pytest.raises(RuntimeError, match="boundary must be an int64"):
        fast_rnnt_amd.rnnt_loss_simple(lm, am, sym, 0, boundary=bnd.int())
    logits = torch.randn(B, T, S + 1, C)
    ranges = torch.arange(S + 1).reshape(1, 1, S + 1).expand(B, T, S + 1)
    with pytest.raises(RuntimeError, match="symbols must be an int64"):
        fast_rnnt_amd.rnnt_loss(logits, sym.int(), 0)
    with pytest.raises(RuntimeError, match="ranges must be an int64"):
        fast_rnnt_amd.rnnt_loss_pruned(logits, sym, ranges.int(), 0)
    with pytest.raises(RuntimeError, match="ranges must be an int64"):
        fast_rnnt_amd.do_rnnt_pruning(am, lm, ranges.int())
    gx, gy = torch.rand(B, S, T + 1), torch.rand(B, S + 1, T)
    with pytest.raises(RuntimeError, match="boundary must be an int64"):
        fast_rnnt_amd.get_rnnt_prune_ranges(gx, gy, bnd.int(), 2)


def test_floating_point_tensors_must_share_a_dtype():
    am, lm, sym, bnd = _inputs()
    with pytest.raises(RuntimeError, match="share one dtype"):
        fast_rnnt_amd.get_rnnt_logprobs_smoothed(lm, am.double(), sym, 0)
    with pytest.raises(RuntimeError, match="share one dtype"):
        fast_rnnt_amd.rnnt_loss_simple(lm.double(), am, sym, 0)
    with pytest.raises(RuntimeError, match="share one dtype"):
        fast_rnnt_amd.do_rnnt_pruning(am, lm.double(), bnd.reshape(2, 1, 4).expand(2, 5, 4))
    B, T, _ = am.shape
    S = sym.shape[1]
    with pytest.raises(RuntimeError, match="share one dtype"):
        fast_rnnt_amd.get_rnnt_prune_ranges(torch.rand(B, S, T + 1),
                                            torch.rand(B, S + 1, T).double(), bnd, 2)


def test_well_formed_cpu_tensors_are_refused_not_computed():
    am, lm, sym, bnd = _inputs()
    with pytest.raises(RuntimeError, match="no CPU path"):
        fast_rnnt_amd.rnnt_loss_simple(lm, am, sym, 0, boundary=bnd)


def test_boundary_rows_cache_follows_versions_and_rereads_on_request():
    bnd = torch.tensor([[0, 0, 3, 5], [0, 0, 2, 4]])
    MI.forget_boundary_rows()
    assert MI.boundary_rows(bnd) == [[0, 0, 3, 5], [0, 0, 2, 4]]
    bnd[1, 2] = 1                       # an in-place torch write bumps the version
    assert MI.boundary_rows(bnd)[1] == [0, 0, 1, 4]
    bnd.data[1, 3] = 3                  # a write the version counter does not see
    assert MI.boundary_rows(bnd, reread=True)[1] == [0, 0, 1, 3]
    assert MI.boundary_rows(bnd)[1] == [0, 0, 1, 3]
