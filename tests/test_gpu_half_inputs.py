"""float16 / bfloat16 inputs with float32 accumulation.

The reference's recursion has float32 and float64 forms only
(fast_rnnt/csrc/mutual_information_cuda.cu:37-38 notes the missing half LogAdd), so its
callers cast half-precision logits to float32 first.  Here the 2-byte tensors are read as
they are and everything after the load is float32, so the expected values are the CPU
oracle's on the SAME values widened to float32:

  loss, px, py           float32 results, the float32 tolerances (1e-5 relative / 2e-5);
  gradients of inputs    come back in the inputs' type: the oracle's float32 gradient,
                         within 1e-4 + one unit in the last place of the 2-byte type
                         (2^-10 relative for float16, 2^-7 for bfloat16);
  do_rnnt_pruning        bit patterns copied: exact.
"""
import sys

import pytest
import torch

import fast_rnnt_amd
from oracle import losses as O

pytestmark = pytest.mark.gpu
NARROW = [torch.float16, torch.bfloat16]
ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _close(a, b, atol, rtol=0.0):
    a, b = a.detach().float().cpu(), b.detach().float().cpu()
    same_inf = torch.isinf(a) & (a == b)
    return bool((same_inf | ((a - b).abs() <= atol + rtol * b.abs())).all())


def _boundary(g, B, S, T, kind):
    Sb = torch.randint(max(1, S // 2), S + 1, (B,), generator=g)
    lo = max(1, T // 2) if kind == "regular" else S
    Tb = torch.randint(lo, T + 1, (B,), generator=g)
    z = torch.zeros(B, dtype=torch.int64)
    return torch.stack([z, z, Sb, Tb], 1)


@pytest.mark.parametrize("kind", ["regular", "modified", "constrained"])
@pytest.mark.parametrize("dtype", NARROW)
def test_joint_loss_on_half_logits(gpu_device, dtype, kind):
    # rows of 8 k entries go through the register kernels, the others (37, 4104) through
    # the strided ones
    dev = gpu_device
    for n, (B, S, T, C) in enumerate([(2, 3, 6, 8), (3, 9, 20, 37), (2, 20, 30, 1000),
                                      (1, 4, 6, 4104)]):
        g = torch.Generator().manual_seed(400 + n)
        logits = (2 * torch.randn(B, T, S + 1, C, generator=g)).to(dtype)
        sym = torch.randint(0, C, (B, S), generator=g)
        for bnd in (None, _boundary(g, B, S, T, kind)):
            _say(f"half joint {kind} {dtype} shape{n} boundary={bnd is not None}")
            a = logits.float().requires_grad_(True)
            wx, wy = O.lattice_logprobs_joint(a, sym, C - 1, boundary=bnd, rnnt_type=kind)
            want = O.loss_joint(a, sym, C - 1, boundary=bnd, rnnt_type=kind, reduction="sum")
            want.backward()
            d = logits.to(dev).requires_grad_(True)
            dbnd = bnd.to(dev) if bnd is not None else None
            gx, gy = fast_rnnt_amd.get_rnnt_logprobs_joint(d, sym.to(dev), C - 1, boundary=dbnd,
                                                          rnnt_type=kind)
            assert gx.dtype == torch.float32 and gy.dtype == torch.float32
            assert _close(gx, wx, 2e-5, 1e-6) and _close(gy, wy, 2e-5, 1e-6)
            got = fast_rnnt_amd.rnnt_loss(d, sym.to(dev), C - 1, boundary=dbnd, rnnt_type=kind,
                                          reduction="sum")
            assert got.dtype == torch.float32
            got.backward()
            assert _close(got, want, 0.0, 1e-5)
            assert d.grad.dtype == dtype
            assert _close(d.grad, a.grad, 1e-4, ULP[dtype])
            if bnd is not None:
                # rows outside the window: exact zeros
                t_out = torch.arange(T).reshape(1, T) >= bnd[:, 3].reshape(B, 1)
                assert (d.grad.cpu()[t_out] == 0).all()


@pytest.mark.parametrize("dtype", NARROW)
def test_pruned_loss_on_half_logits(gpu_device, dtype):
    dev = gpu_device
    for n, (B, S, T, R, C) in enumerate([(2, 6, 9, 3, 16), (3, 20, 41, 5, 504), (2, 12, 16, 4, 30)]):
        g = torch.Generator().manual_seed(500 + n)
        logits = (2 * torch.randn(B, T, R, C, generator=g)).to(dtype)
        sym = torch.randint(0, C, (B, S), generator=g)
        bnd = _boundary(g, B, S, T, "regular")
        # any monotone ranges with steps below R will do here
        start = torch.cumsum(torch.randint(0, 2, (B, T), generator=g), 1).clamp(max=S + 1 - R)
        ranges = (start.unsqueeze(2) + torch.arange(R).reshape(1, 1, R)).contiguous()
        _say(f"half pruned {dtype} shape{n}")
        a = logits.float().requires_grad_(True)
        want = O.loss_pruned(a, sym, ranges, 0, boundary=bnd, reduction="sum")
        want.backward()
        d = logits.to(dev).requires_grad_(True)
        got = fast_rnnt_amd.rnnt_loss_pruned(d, sym.to(dev), ranges.to(dev), 0,
                                             boundary=bnd.to(dev), reduction="sum")
        got.backward()
        assert got.dtype == torch.float32 and d.grad.dtype == dtype
        assert _close(got, want, 0.0, 1e-5)
        assert _close(d.grad, a.grad, 1e-4, ULP[dtype])


@pytest.mark.parametrize("smoothed", [False, True])
@pytest.mark.parametrize("dtype", NARROW)
def test_simple_and_smoothed_loss_on_half_inputs(gpu_device, dtype, smoothed):
    dev = gpu_device
    B, S, T, C = 3, 11, 23, 40
    g = torch.Generator().manual_seed(600)
    am = torch.randn(B, T, C, generator=g).to(dtype)
    lm = torch.randn(B, S + 1, C, generator=g).to(dtype)
    sym = torch.randint(1, C, (B, S), generator=g)
    bnd = _boundary(g, B, S, T, "regular")
    a = am.float().requires_grad_(True)
    l = lm.float().requires_grad_(True)
    da = am.to(dev).requires_grad_(True)
    dl = lm.to(dev).requires_grad_(True)
    _say(f"half simple smoothed={smoothed} {dtype}")
    if smoothed:
        want, (wx, wy) = O.loss_smoothed(l, a, sym, 0, 0.25, 0.1, boundary=bnd, reduction="sum",
                                         return_grad=True)
        got, (gx, gy) = fast_rnnt_amd.rnnt_loss_smoothed(
            dl, da, sym.to(dev), 0, 0.25, 0.1, boundary=bnd.to(dev), reduction="sum",
            return_grad=True)
    else:
        want, (wx, wy) = O.loss_simple(l, a, sym, 0, boundary=bnd, reduction="sum",
                                       return_grad=True)
        got, (gx, gy) = fast_rnnt_amd.rnnt_loss_simple(
            dl, da, sym.to(dev), 0, boundary=bnd.to(dev), reduction="sum", return_grad=True)
    assert got.dtype == torch.float32 and gx.dtype == torch.float32
    assert _close(got, want, 0.0, 1e-5)
    assert _close(gx, wx, 1e-4) and _close(gy, wy, 1e-4)
    want.backward()
    got.backward()
    assert da.grad.dtype == dtype and dl.grad.dtype == dtype
    assert _close(da.grad, a.grad, 1e-4, ULP[dtype])
    assert _close(dl.grad, l.grad, 1e-4, ULP[dtype])


@pytest.mark.parametrize("dtype", NARROW)
def test_pruning_gather_on_half_inputs(gpu_device, dtype):
    # do_rnnt_pruning (rnnt_loss.py:780-818) is plain indexing in the reference: the gather
    # copies bit patterns (exact); its adjoint is a float32 sum rounded once
    dev = gpu_device
    for n, (B, S, T, R, C) in enumerate([(2, 5, 9, 3, 16), (3, 20, 41, 5, 500), (2, 12, 16, 4, 37)]):
        g = torch.Generator().manual_seed(650 + n)
        am = torch.randn(B, T, C, generator=g).to(dtype)
        lm = torch.randn(B, S + 1, C, generator=g).to(dtype)
        start = torch.randint(0, S + 2 - R, (B, T), generator=g)
        ranges = (start.unsqueeze(2) + torch.arange(R).reshape(1, 1, R)).contiguous()
        weight = torch.randn(B, T, R, C, generator=g).to(dtype)
        _say(f"half gather {dtype} shape{n}")
        dl = lm.to(dev).requires_grad_(True)
        am_p, lm_p = fast_rnnt_amd.do_rnnt_pruning(am.to(dev), dl, ranges.to(dev))
        _, want = O.prune(am, lm, ranges)
        assert lm_p.dtype == dtype and am_p.shape == lm_p.shape
        assert torch.equal(lm_p.cpu(), want)
        lm_p.backward(weight.to(dev))
        l32 = lm.float().requires_grad_(True)
        _, p32 = O.prune(am.float(), l32, ranges)
        p32.backward(weight.float())
        assert dl.grad.dtype == dtype
        assert _close(dl.grad, l32.grad, 1e-6, ULP[dtype])
    bad = ranges.clone()
    bad[0, 0, 0] = S + 1
    _, out = fast_rnnt_amd.do_rnnt_pruning(am.to(dev), lm.to(dev), bad.to(dev))
    assert torch.isnan(out[0, 0, 0]).all() and torch.isfinite(out[0, 0, 1]).all()
