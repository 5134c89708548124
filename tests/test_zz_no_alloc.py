"""frnnt_simple_logprobs_bwd_noalloc_f32 (scratch in the library's own per-GPU array)
against frnnt_simple_logprobs_bwd_f32 (scratch from the caller), through the C ABI:
the same kernels on the same inputs, so lm.grad, am.grad and the in-place scaled
px_grad / py_grad must agree bit for bit -- on two calls in a row, the second one
smaller (the array then still holds the first call's contents), and a size beyond the
array must be refused."""
import sys

import pytest
import torch

from fast_rnnt_amd import _lib

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _both_ways(dev, seed, B, S, T, C, rnnt_type, with_boundary, with_score_grad):
    g = torch.Generator().manual_seed(seed)
    f32 = dict(dtype=torch.float32, device=dev)
    lm = torch.randn(B, S + 1, C, generator=g).to(dev)
    am = torch.randn(B, T, C, generator=g).to(dev)
    sym = torch.randint(0, C, (B, S), generator=g).to(dev)
    bnd = None
    if with_boundary:
        Sb = torch.randint(1, S + 1, (B,), generator=g)
        Tb = torch.randint(S if rnnt_type else 1, T + 1, (B,), generator=g)
        z = torch.zeros(B, dtype=torch.int64)
        bnd = torch.stack([z, z, Sb, Tb], 1).to(dev)
    T1 = T + 1 if rnnt_type == 0 else T
    px, py = torch.empty(B, S, T1, **f32), torch.empty(B, S + 1, T, **f32)
    lm_max, am_max = torch.empty(B, S + 1, **f32), torch.empty(B, T, **f32)
    norm_raw = torch.empty(B, S + 1, T, **f32)
    stream = torch.cuda.current_stream().cuda_stream
    _lib.call("frnnt_simple_logprobs_fwd_f32", lm.data_ptr(), am.data_ptr(), sym.data_ptr(),
              _lib.ptr(bnd), px.data_ptr(), py.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(),
              norm_raw.data_ptr(), B, S, T, C, 0, rnnt_type, 0, stream)
    gpx = torch.rand(B, S, T1, generator=g).to(dev)
    gpy = torch.rand(B, S + 1, T, generator=g).to(dev)
    score_grad = torch.randn(B, generator=g).to(dev) if with_score_grad else None
    out = []
    for own_scratch in (False, True):
        gx, gy = gpx.clone(), gpy.clone()
        lm_grad, am_grad = torch.full_like(lm, float("nan")), torch.full_like(am, float("nan"))
        head = [lm.data_ptr(), am.data_ptr(), sym.data_ptr(), _lib.ptr(bnd), lm_max.data_ptr(),
                am_max.data_ptr(), norm_raw.data_ptr(), _lib.ptr(score_grad), 1, -0.5,
                gx.data_ptr(), gy.data_ptr()]
        tail = [lm_grad.data_ptr(), am_grad.data_ptr(), B, S, T, C, 0, rnnt_type, 0, stream]
        if own_scratch:
            _lib.call("frnnt_simple_logprobs_bwd_noalloc_f32", *head, *tail)
        else:
            dmat = torch.empty(B, S + 1, (T + 3) // 4 * 4, **f32)
            row_x, row_y = torch.empty(B, S + 1, **f32), torch.empty(B, S + 1, **f32)
            col_y = torch.empty(B, T, **f32)
            _lib.call("frnnt_simple_logprobs_bwd_f32", *head, dmat.data_ptr(), row_x.data_ptr(),
                      row_y.data_ptr(), col_y.data_ptr(), *tail)
        torch.cuda.synchronize()
        out.append((lm_grad, am_grad, gx, gy))
    return out


def test_own_scratch_matches_caller_scratch(gpu_device):
    dev = gpu_device
    # two calls in a row, the second smaller; then other lattice types and no boundary
    cases = [(1, 6, 80, 250, 500, 0, True, True), (2, 3, 33, 61, 47, 0, True, False),
             (3, 2, 20, 45, 30, 1, False, True), (4, 2, 9, 30, 12, 2, True, True),
             (5, 4, 100, 130, 96, 0, False, False)]
    for seed, B, S, T, C, kind, with_boundary, with_score_grad in cases:
        _say(f"no-alloc backward: B={B} S={S} T={T} C={C} rnnt_type={kind} "
             f"boundary={with_boundary} score_grad={with_score_grad}")
        want, got = _both_ways(dev, seed, B, S, T, C, kind, with_boundary, with_score_grad)
        for name, a, b in zip(("lm_grad", "am_grad", "px_grad", "py_grad"), want, got):
            assert not torch.isnan(b).any(), name
            assert torch.equal(a, b), name


def test_sizes_beyond_the_array_are_refused(gpu_device):
    # B (S+1) T beyond 4 Mi floats: refused with FRNNT_ELIMIT before anything is read
    B, S, T = 64, 255, 512
    with pytest.raises(RuntimeError, match="scratch"):
        _lib.call("frnnt_simple_logprobs_bwd_noalloc_f32", *([None] * 8), 1, 1.0, *([None] * 4),
                  B, S, T, 16, 0, 0, 0, None)
