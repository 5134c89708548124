"""Seeded random configurations of the whole pipeline and of the public (px, py)
builders against the CPU oracle, in float64 so that every difference is a difference of
meaning, not of rounding: loss type, lattice type, reduction, delay penalty, boundary or
none, boundary rows with offsets and with empty ranges, window sizes on either side of
16, vocabulary sizes on either side of the kernels' vector widths, arbitrary upstream
gradients (also into the cells that hold -inf).
"""
import random
import sys

import pytest
import torch

import fast_rnnt_amd as F
from oracle import losses as O

pytestmark = pytest.mark.gpu


def _close(x, y, tol):
    x, y = x.detach().cpu(), y.detach()
    if x.shape != y.shape:
        return False
    ok = ((x - y).abs() <= tol + tol * y.abs()) | (torch.isinf(x) & (x == y)) | \
        (torch.isnan(x) & torch.isnan(y))
    return bool(ok.all())


def _draw(rng, it, min_t_is_s):
    kind = rng.choice(["regular", "modified", "constrained"])
    B, S = rng.randint(1, 4), rng.randint(1, 90)
    C = rng.choice([1, 2, 3, 5, 8, 17, 40, 64, 100, 260, 513])
    T = rng.randint(max(S, 2) if (min_t_is_s or kind != "regular") else 1, 150)
    g = torch.Generator().manual_seed(31000 + it)
    am = torch.randn(B, T, C, generator=g, dtype=torch.float64) * 2
    lm = torch.randn(B, S + 1, C, generator=g, dtype=torch.float64) * 2
    sym = torch.randint(0, C, (B, S), generator=g)
    bnd = None
    if rng.random() < 0.75:
        Sb = torch.randint(1, S + 1, (B,), generator=g)
        Tb = torch.randint(1 if kind == "regular" else S, T + 1, (B,), generator=g)
        z = torch.zeros(B, dtype=torch.int64)
        bnd = torch.stack([z, z, Sb, Tb], 1)
        if rng.random() < 0.3:  # offsets, sometimes leaving an empty range
            bnd[:, 0] = torch.minimum(torch.randint(0, 3, (B,), generator=g), Sb)
            bnd[:, 1] = torch.minimum(torch.randint(0, 3, (B,), generator=g), Tb)
    return kind, B, S, T, C, g, am, lm, sym, bnd, rng.randint(0, C - 1)


def test_random_pipelines(gpu_device):
    """smoothed loss -> prune ranges -> pruning (or the fused joiner input) -> joiner ->
    pruned loss, both losses in the objective."""
    dev = gpu_device
    rng = random.Random(5)
    ran = 0
    for it in range(120):
        kind, B, S, T, C, g, am, lm, sym, bnd, term = _draw(rng, it, True)
        R = rng.choice([2, 3, 4, 5, 7, 9, 16, 17, 20, 33])
        lm_s, am_s = rng.choice([(0.25, 0.0), (0.1, 0.2), (0.0, 0.0)])
        red = rng.choice(["none", "mean", "sum"])
        dp = rng.choice([0.0, 0.0, 0.02])
        fused = rng.random() < 0.5
        W = torch.randn(C, C, generator=g, dtype=torch.float64) / C ** 0.5
        w8 = torch.randn(B, generator=g, dtype=torch.float64)
        print(f"pipeline {it}: {kind} B={B} S={S} T={T} C={C} R={R} scales={lm_s},{am_s} {red} "
              f"penalty={dp} fused={fused} boundary={None if bnd is None else bnd.tolist()}",
              flush=True)
        sys.stdout.flush()
        full = torch.tensor([[0, 0, S, T]] * B)

        def run(gpu, ranges_in=None):
            to = (lambda x: x.to(dev)) if gpu else (lambda x: x.clone())
            a, l = to(am).requires_grad_(True), to(lm).requires_grad_(True)
            b_ = None if bnd is None else to(bnd)
            smoothed = F.rnnt_loss_smoothed if gpu else O.loss_smoothed
            pruned = F.rnnt_loss_pruned if gpu else O.loss_pruned
            simple, (gx, gy) = smoothed(l, a, to(sym), term, lm_s, am_s, boundary=b_,
                                        rnnt_type=kind, reduction=red, delay_penalty=dp,
                                        return_grad=True)
            occ = gx.detach().clone(), gy.detach().clone()
            ranges = ranges_in
            if ranges is None:
                ranges = O.prune_ranges(gx, gy, full if bnd is None else bnd, R,
                                        window_sum="cascade")
            if gpu and fused:
                hidden = F.pruned_joiner_input(a, l, ranges, activation="tanh")
            else:
                am_p, lm_p = (F.do_rnnt_pruning if gpu else O.prune)(a, l, ranges)
                hidden = torch.tanh(am_p + lm_p)
            loss = pruned(hidden @ to(W), to(sym), ranges, term, boundary=b_, rnnt_type=kind,
                          reduction=red, delay_penalty=dp)
            total = simple * 0.5 + loss  # (an utterance without a path: +inf, gradients flow)
            ((total * to(w8)).sum() if red == "none" else total).backward()
            return simple.detach(), loss.detach(), occ, a.grad, l.grad, ranges

        try:
            want = run(False)
        except (AssertionError, RuntimeError) as err:  # e.g. a boundary the reference refuses
            print("   refused by the oracle:", type(err).__name__, flush=True)
            continue
        got = run(True, want[5].to(dev))
        ran += 1
        # the GPU's ranges from the oracle's gradients: bit for bit
        mine = F.get_rnnt_prune_ranges(want[2][0].to(dev), want[2][1].to(dev),
                                       (full if bnd is None else bnd).to(dev), R)
        assert torch.equal(mine.cpu(), want[5]), it
        assert _close(got[0], want[0], 1e-9) and _close(got[1], want[1], 1e-9), it
        assert _close(got[2][0], want[2][0], 1e-9) and _close(got[2][1], want[2][1], 1e-9), it
        assert _close(got[3], want[3], 1e-8) and _close(got[4], want[4], 1e-8), it
    assert ran >= 80


def test_random_logprob_builders_with_arbitrary_gradients(gpu_device):
    dev = gpu_device
    rng = random.Random(6)
    ran = 0
    for it in range(160):
        kind, B, S, T, C, g, am, lm, sym, bnd, term = _draw(rng, 1000 + it, False)
        which = rng.choice(["simple", "smoothed", "joint", "pruned"])
        R = min(S + 1, rng.choice([2, 3, 5, 8]))
        start = torch.clamp(torch.arange(T) * max(S + 1 - R, 0) // max(T - 1, 1), 0, S + 1 - R)
        ranges = (start.reshape(1, T, 1) + torch.arange(R).reshape(1, 1, R)).expand(B, T, R)
        ranges = ranges.contiguous()
        T1 = T + 1 if kind == "regular" else T
        wx = torch.randn(B, S, T1, generator=g, dtype=torch.float64)
        wy = torch.randn(B, S + 1, T, generator=g, dtype=torch.float64)
        print(f"builder {it}: {which} {kind} B={B} S={S} T={T} C={C} R={R} "
              f"boundary={None if bnd is None else bnd.tolist()}", flush=True)
        sys.stdout.flush()

        def run(gpu):
            to = (lambda x: x.to(dev)) if gpu else (lambda x: x.clone())
            a, l = to(am).requires_grad_(True), to(lm).requires_grad_(True)
            b_ = None if bnd is None else to(bnd)
            if which == "simple":
                f = F.get_rnnt_logprobs if gpu else O.lattice_logprobs_simple
                px, py = f(l, a, to(sym), term, boundary=b_, rnnt_type=kind)
            elif which == "smoothed":
                f = F.get_rnnt_logprobs_smoothed if gpu else O.lattice_logprobs_smoothed
                px, py = f(l, a, to(sym), term, 0.2, 0.15, boundary=b_, rnnt_type=kind)
            elif which == "joint":
                f = F.get_rnnt_logprobs_joint if gpu else O.lattice_logprobs_joint
                px, py = f(torch.tanh(a.unsqueeze(2) + l.unsqueeze(1)) * 3, to(sym), term,
                           boundary=b_, rnnt_type=kind)
            else:
                f = F.get_rnnt_logprobs_pruned if gpu else O.lattice_logprobs_pruned
                rg = to(ranges)
                lp = torch.gather(l.unsqueeze(1).expand(B, T, S + 1, C), 2,
                                  rg.unsqueeze(3).expand(B, T, R, C))
                px, py = f(torch.tanh(a.unsqueeze(2) + lp) * 3, to(sym), rg, term, boundary=b_,
                           rnnt_type=kind)

            def finite(v):
                return torch.where(torch.isfinite(v), v, torch.zeros_like(v))
            ((finite(px) * to(wx)).sum() + (finite(py) * to(wy)).sum()).backward()
            return px.detach(), py.detach(), a.grad, l.grad

        try:
            want = run(False)
        except (AssertionError, RuntimeError) as err:
            print("   refused by the oracle:", type(err).__name__, flush=True)
            continue
        got = run(True)
        ran += 1
        for x, y in zip(got, want):
            assert _close(x, y, 1e-9), it
    assert ran >= 100


def test_random_simple_losses_float32(gpu_device):
    """The float32 kernels of rnnt_loss_simple (the benchmarked path) on seeded random shapes:
    every output is judged against the float64 oracle and may be off by what the reference's
    own float32 arithmetic (the oracle in float32) is off, times three, plus a floor of a few
    ulps -- the occupation gradients are ill-conditioned in px / py
    (tests/test_oracle_conditioning.py), so a fixed bound would say nothing."""
    dev = gpu_device
    rng = random.Random(7)
    ran = 0
    for it in range(60):
        kind = rng.choice(["regular", "modified", "constrained"])
        B = rng.randint(1, 6)
        S = rng.choice([rng.randint(1, 40), rng.randint(60, 100), rng.randint(120, 140)])
        C = rng.choice([3, 17, 64, 100, 257, 500, 515, 1030])
        T = rng.randint(max(S, 2) if kind != "regular" else 1, 260)
        red = rng.choice(["none", "mean", "sum"])
        dp = rng.choice([0.0, 0.0, 0.01])
        g = torch.Generator().manual_seed(41000 + it)
        spread = rng.choice([1.0, 1.0, 3.0])
        am = torch.randn(B, T, C, generator=g) * spread
        lm = torch.randn(B, S + 1, C, generator=g) * spread
        sym = torch.randint(0, C, (B, S), generator=g)
        term = rng.randint(0, C - 1)
        bnd = None
        if rng.random() < 0.8:
            Sb = torch.randint(1, S + 1, (B,), generator=g)
            Tb = torch.randint(1 if kind == "regular" else S, T + 1, (B,), generator=g)
            z = torch.zeros(B, dtype=torch.int64)
            bnd = torch.stack([z, z, Sb, Tb], 1)
            if rng.random() < 0.3:
                bnd[:, 0] = torch.minimum(torch.randint(0, 3, (B,), generator=g), Sb)
                bnd[:, 1] = torch.minimum(torch.randint(0, 3, (B,), generator=g), Tb)
        w8 = torch.randn(B, generator=g)
        print(f"float32 case {it}: {kind} B={B} S={S} T={T} C={C} {red} penalty={dp} "
              f"spread={spread} boundary={None if bnd is None else bnd.tolist()}", flush=True)
        sys.stdout.flush()

        def run(fn, lm_, am_, to):
            a, l = to(am_).requires_grad_(True), to(lm_).requires_grad_(True)
            loss, (gx, gy) = fn(l, a, to(sym), term, boundary=None if bnd is None else to(bnd),
                                rnnt_type=kind, reduction=red, delay_penalty=dp,
                                return_grad=True)
            occ = gx.detach().clone(), gy.detach().clone()
            ((loss * to(w8.to(loss.dtype))).sum() if red == "none" else loss).backward()
            return [loss.detach(), occ[0], occ[1], a.grad, l.grad]

        try:
            truth = run(O.loss_simple, lm.double(), am.double(), lambda x: x.clone())
            ref32 = run(O.loss_simple, lm, am, lambda x: x.clone())
        except (AssertionError, RuntimeError) as err:
            print("   refused by the oracle:", type(err).__name__, flush=True)
            continue
        got = run(F.rnnt_loss_simple, lm, am, lambda x: x.to(dev))
        if not bool(torch.isfinite(truth[0]).all()):
            continue  # an utterance without a path: nothing to compare gradients on
        ran += 1
        for name, x, r, t in zip(("loss", "px_grad", "py_grad", "am.grad", "lm.grad"), got, ref32,
                                 truth):
            x = x.cpu().double()
            scale = max(1.0, t.abs().max().item())
            err = (x - t).abs().max().item()
            allowed = 3 * (r.double() - t).abs().max().item() + 8 * 1.2e-7 * scale
            assert err <= allowed, (it, name, err, allowed)
    assert ran >= 45
