"""Joint (unpruned), pruned and smoothed losses, prune ranges and the pruning
gather on the GPU against the CPU oracle and the golden vectors.

Tolerances (float32): loss 1e-5 relative, px/py and their gradients 1e-4
absolute, input gradients 1e-4 absolute + 1e-4 relative; ranges bit-exact.
"""
import os
import sys

import pytest
import torch

import fast_rnnt_amd
from fast_rnnt_amd import workloads
from oracle import losses as O

import ulp_sensitivity as U

pytestmark = pytest.mark.gpu
KINDS = ["regular", "modified", "constrained"]
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _close(a, b, atol, rtol=0.0):
    a, b = a.detach().cpu(), b.detach().cpu()
    same_inf = torch.isinf(a) & (a == b)
    return bool((same_inf | ((a - b).abs() <= atol + rtol * b.abs())).all())


def _case(seed, B, S, T, C, dtype, kind):
    g = torch.Generator().manual_seed(seed)
    am = torch.randn(B, T, C, generator=g, dtype=dtype)
    lm = torch.randn(B, S + 1, C, generator=g, dtype=dtype)
    sym = torch.randint(0, C, (B, S), generator=g)
    Sb = torch.randint(max(1, S // 2), S + 1, (B,), generator=g)
    lo = max(1, T // 2) if kind == "regular" else S
    Tb = torch.randint(lo, T + 1, (B,), generator=g)
    z = torch.zeros(B, dtype=torch.int64)
    return am, lm, sym, torch.stack([z, z, Sb, Tb], 1)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_joint_loss_and_gradient(gpu_device, dtype, kind):
    dev = gpu_device
    f32 = dtype == torch.float32
    for n, (B, S, T, C) in enumerate([(2, 3, 5, 4), (3, 9, 20, 33), (2, 66, 70, 17)]):
        for with_boundary in (False, True):
            _say(f"joint {kind} {dtype} shape{n} boundary={with_boundary}")
            am, lm, sym, bnd = _case(90 + n, B, S, T, C, dtype, kind)
            if not with_boundary:
                bnd = None
            logits = torch.tanh(am.unsqueeze(2) + lm.unsqueeze(1)) * 3
            a = logits.clone().requires_grad_(True)
            wx, wy = O.lattice_logprobs_joint(a, sym, C - 1, boundary=bnd, rnnt_type=kind)
            want = O.loss_joint(a, sym, C - 1, boundary=bnd, rnnt_type=kind, reduction="sum")
            want.backward()
            d = logits.to(dev).requires_grad_(True)
            dbnd = bnd.to(dev) if bnd is not None else None
            gx, gy = fast_rnnt_amd.get_rnnt_logprobs_joint(d, sym.to(dev), C - 1, boundary=dbnd,
                                                          rnnt_type=kind)
            assert _close(gx, wx, 2e-5 if f32 else 1e-11, 1e-6 if f32 else 0)
            assert _close(gy, wy, 2e-5 if f32 else 1e-11, 1e-6 if f32 else 0)
            got = fast_rnnt_amd.rnnt_loss(d, sym.to(dev), C - 1, boundary=dbnd, rnnt_type=kind,
                                          reduction="sum")
            got.backward()
            assert _close(got, want, 0.0, 1e-5 if f32 else 1e-12)
            assert _close(d.grad, a.grad, 1e-4 if f32 else 1e-9, 1e-4 if f32 else 1e-9)


def test_joint_equals_simple_on_additive_joiner(gpu_device):
    # fast_rnnt/python/tests/rnnt_loss_test.py:242-272
    dev = gpu_device
    am, lm, sym, bnd = _case(5, 3, 7, 25, 11, torch.float32, "regular")
    am, lm, sym, bnd = am.to(dev), lm.to(dev), sym.to(dev), bnd.to(dev)
    a = fast_rnnt_amd.rnnt_loss_simple(lm, am, sym, 0, boundary=bnd, reduction="none")
    b = fast_rnnt_amd.rnnt_loss(am.unsqueeze(2) + lm.unsqueeze(1), sym, 0, boundary=bnd,
                                reduction="none")
    c = fast_rnnt_amd.rnnt_loss_smoothed(lm, am, sym, 0, 0.0, 0.0, boundary=bnd, reduction="none")
    assert torch.allclose(a, b, rtol=1e-5) and torch.allclose(a, c, rtol=1e-5)
    # invariance to per-frame constants (rnnt_loss_test.py:287-321)
    g = torch.Generator().manual_seed(1)
    lm2 = lm + torch.randn(3, 8, 1, generator=g).to(dev)
    am2 = am + torch.randn(3, 25, 1, generator=g).to(dev)
    d = fast_rnnt_amd.rnnt_loss_smoothed(lm2, am2, sym, 0, 0.2, 0.333, boundary=bnd, reduction="none")
    e = fast_rnnt_amd.rnnt_loss_smoothed(lm, am, sym, 0, 0.2, 0.333, boundary=bnd, reduction="none")
    assert torch.allclose(d, e, rtol=2e-5)


def test_prune_ranges_golden_bit_exact(gpu_device, capsys):
    dev = gpu_device
    data = torch.load(os.path.join(GOLDEN, "prune_ranges.pt"), weights_only=True)
    for name, c in data.items():
        _say(f"golden ranges {name}")
        got = fast_rnnt_amd.get_rnnt_prune_ranges(c["px_grad"].to(dev), c["py_grad"].to(dev),
                                                  c["boundary"].to(dev), c["s_range"])
        assert got.dtype == torch.int64
        assert torch.equal(got.cpu(), c["ranges"]), name
        if "logits" in c:
            px, py = fast_rnnt_amd.get_rnnt_logprobs_pruned(
                c["logits"].to(dev), c["symbols"].to(dev), got, 0,
                boundary=c["boundary"].to(dev), rnnt_type=c["kind"])
            assert _close(px, c["px"], 2e-6, 1e-6) and _close(py, c["py"], 2e-6, 1e-6)
    assert "Adjusting to 4" in capsys.readouterr().out


@pytest.mark.parametrize("kind", ["regular", "modified"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_prune_ranges_random_bit_exact(gpu_device, dtype, kind):
    dev = gpu_device
    for n, (B, S, T, C) in enumerate([(3, 12, 40, 9), (4, 30, 100, 20), (2, 5, 300, 7)]):
        am, lm, sym, bnd = _case(120 + n, B, S, T, C, dtype, kind)
        _, (gx, gy) = O.loss_simple(lm, am, sym, 0, boundary=bnd, rnnt_type=kind,
                                    reduction="sum", return_grad=True)
        for R in (1, 2, 3, 5, 8, S + 1, S + 7):
            if kind == "regular" and R < 2:
                continue
            _say(f"ranges {kind} {dtype} shape{n} R={R}")
            want = O.prune_ranges(gx, gy, bnd, R)
            got = fast_rnnt_amd.get_rnnt_prune_ranges(gx.to(dev), gy.to(dev), bnd.to(dev), R)
            assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_prune_ranges_wide_windows_bit_exact(gpu_device, dtype):
    """s_range above 16, where the reference's torch.sum no longer adds the window left to
    right (ATen's CPU loop sums in stretches of 16), on occupancies of short targets in a
    tall lattice: the window covers the whole band that holds the alignment's mass, so
    neighbouring window starts tie up to rounding and the summation order picks the
    winner.  Against the oracle's torch.sum (frame counts that fill whole SIMD vectors,
    where it has no differently summed tail) and against its host-independent
    restatement of that order."""
    dev = gpu_device
    for seed, (B, S, T) in enumerate([(3, 69, 128), (2, 100, 64), (2, 150, 64)]):
        g = torch.Generator().manual_seed(40 + seed)
        am = torch.randn(B, T, 12, generator=g, dtype=dtype)
        lm = torch.randn(B, S + 1, 12, generator=g, dtype=dtype)
        sym = torch.randint(1, 12, (B, S), generator=g)
        Sb = torch.randint(S // 4, S // 2, (B,), generator=g)
        Tb = torch.randint(T // 2, T + 1, (B,), generator=g)
        z = torch.zeros(B, dtype=torch.int64)
        bnd = torch.stack([z, z, Sb, Tb], 1)
        _, (gx, gy) = O.loss_simple(lm, am, sym, 0, boundary=bnd, reduction="sum",
                                    return_grad=True)
        for R in (16, 17, 19, 33, 40, 64):
            _say(f"wide windows {dtype} B={B} S={S} T={T} R={R}")
            got = fast_rnnt_amd.get_rnnt_prune_ranges(gx.to(dev), gy.to(dev), bnd.to(dev), R).cpu()
            assert torch.equal(got, O.prune_ranges(gx, gy, bnd, R, window_sum="cascade"))
            assert torch.equal(got, O.prune_ranges(gx, gy, bnd, R))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_prune_ranges_ties_nans_and_long_targets(gpu_device, dtype):
    """Window scores with exact ties and NaNs (first maximum wins, NaN counts as the maximum,
    as torch.argmax in rnnt_loss.py:735-741), on targets short enough for the kernel that
    stages a frame tile in LDS and long enough (S = 300, and 160 in float64) for the one
    that does not.  Bit-exact against the oracle."""
    dev = gpu_device
    for n, (B, S, T) in enumerate([(2, 37, 90), (1, 160, 170), (1, 300, 330)]):
        g = torch.Generator().manual_seed(900 + n)
        # few distinct values: many windows tie
        gx = torch.randint(0, 3, (B, S, T + 1), generator=g).to(dtype) * 0.25
        gy = torch.randint(0, 3, (B, S + 1, T), generator=g).to(dtype) * 0.25
        gy[0, S // 2, 5::7] = float("nan")
        gx[0, S // 3, 3::11] = float("nan")
        Sb = torch.randint(S // 2, S + 1, (B,), generator=g)
        Tb = torch.randint(T // 2, T + 1, (B,), generator=g)
        z = torch.zeros(B, dtype=torch.int64)
        bnd = torch.stack([z, z, Sb, Tb], 1)
        for R in (2, 5, 9):
            _say(f"ranges ties/NaN {dtype} B={B} S={S} T={T} R={R}")
            want = O.prune_ranges(gx, gy, bnd, R)
            got = fast_rnnt_amd.get_rnnt_prune_ranges(gx.to(dev), gy.to(dev), bnd.to(dev), R)
            assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_pruned_pipeline(gpu_device, dtype, kind):
    """smoothed loss -> ranges -> pruning -> joiner -> pruned loss, with gradients."""
    dev = gpu_device
    f32 = dtype == torch.float32
    for n, (B, S, T, C, R) in enumerate([(2, 6, 14, 9, 3), (3, 20, 60, 30, 5), (2, 4, 30, 8, 9)]):
        _say(f"pipeline {kind} {dtype} shape{n}")
        am, lm, sym, bnd = _case(150 + n, B, S, T, C, dtype, kind)
        g = torch.Generator().manual_seed(n)
        W = (torch.randn(C, C, generator=g, dtype=dtype) / C ** 0.5)

        def run(mod, am_, lm_, sym_, bnd_, W_, prune_ranges, prune, smoothed, pruned):
            simple, (gx, gy) = smoothed(lm_, am_, sym_, 0, 0.25, 0.0, boundary=bnd_,
                                        rnnt_type=kind, reduction="sum", return_grad=True)
            gx0, gy0 = gx.detach().clone(), gy.detach().clone()  # backward scales gx, gy in place
            ranges = prune_ranges(gx, gy, bnd_, R)
            am_p, lm_p = prune(am_, lm_, ranges)
            logits = torch.tanh(am_p + lm_p) @ W_
            loss = pruned(logits, sym_, ranges, 0, boundary=bnd_, rnnt_type=kind, reduction="sum")
            (simple * 0.5 + loss).backward()
            return simple, loss, ranges, gx0, gy0

        a = am.clone().requires_grad_(True)
        l = lm.clone().requires_grad_(True)
        ws, wl, wr, wgx, wgy = run(O, a, l, sym, bnd, W, O.prune_ranges, O.prune,
                                   O.loss_smoothed, O.loss_pruned)
        da = am.to(dev).requires_grad_(True)
        dl = lm.to(dev).requires_grad_(True)
        gs, gl, gr, ggx, ggy = run(fast_rnnt_amd, da, dl, sym.to(dev), bnd.to(dev), W.to(dev),
                                   fast_rnnt_amd.get_rnnt_prune_ranges,
                                   fast_rnnt_amd.do_rnnt_pruning,
                                   fast_rnnt_amd.rnnt_loss_smoothed,
                                   fast_rnnt_amd.rnnt_loss_pruned)
        assert _close(gs, ws, 0.0, 1e-5 if f32 else 1e-11)
        # identical gradients in, identical ranges out
        assert torch.equal(fast_rnnt_amd.get_rnnt_prune_ranges(
            wgx.to(dev), wgy.to(dev), bnd.to(dev), R).cpu(), wr)
        if torch.equal(gr.cpu(), wr):
            assert _close(gl, wl, 0.0, 1e-5 if f32 else 1e-11)
            assert _close(da.grad, a.grad, 2e-4 if f32 else 1e-9, 1e-4 if f32 else 1e-9)
            assert _close(dl.grad, l.grad, 2e-4 if f32 else 1e-9, 1e-4 if f32 else 1e-9)
        else:  # a near-tie resolved differently because the gradients differ in the last bits
            assert f32, "float64 ranges must agree"
            _say("  note: ranges differ from the CPU run at a near-tie of the fp32 scores")


def test_pruning_gather_and_its_gradient(gpu_device):
    dev = gpu_device
    g = torch.Generator().manual_seed(2)
    B, S, T, C, R = 3, 9, 17, 21, 4
    am = torch.randn(B, T, C, generator=g)
    lm = torch.randn(B, S + 1, C, generator=g)
    r0 = torch.randint(0, S + 2 - R, (B, T), generator=g)
    ranges = r0.unsqueeze(2) + torch.arange(R)
    w = torch.randn(B, T, R, C, generator=g)
    a = am.clone().requires_grad_(True)
    l = lm.clone().requires_grad_(True)
    ap, lp = O.prune(a, l, ranges)
    ((ap + lp) * w).sum().backward()
    da = am.to(dev).requires_grad_(True)
    dl = lm.to(dev).requires_grad_(True)
    gap, glp = fast_rnnt_amd.do_rnnt_pruning(da, dl, ranges.to(dev))
    assert gap.shape == (B, T, R, C) and gap.stride(2) == 0  # zero-copy view, like the reference
    assert torch.equal(glp.cpu(), lp.detach())
    ((gap + glp) * w.to(dev)).sum().backward()
    assert _close(dl.grad, l.grad, 1e-5, 1e-5) and _close(da.grad, a.grad, 1e-5, 1e-5)


@pytest.mark.parametrize("C", [516, 1000, 1001, 2048, 4100])
def test_pruning_gather_wide_rows(gpu_device, C):
    # rows of several 16-byte pieces per lane, rows longer than the vector kernels take,
    # and a row length that is no multiple of 4 (the element-wise kernels)
    dev = gpu_device
    g = torch.Generator().manual_seed(400 + C)
    B, S, T, R = 2, 9, 14, 4
    lm = torch.randn(B, S + 1, C, generator=g)
    am = torch.randn(B, T, C, generator=g)
    ranges = torch.randint(0, S + 2 - R, (B, T), generator=g).unsqueeze(-1) + torch.arange(R)
    dl = lm.to(dev).requires_grad_(True)
    _say(f"pruning gather and adjoint, C={C}")
    _, lm_p = fast_rnnt_amd.do_rnnt_pruning(am.to(dev), dl, ranges.to(dev))
    want = torch.gather(lm.unsqueeze(1).expand(B, T, S + 1, C), 2,
                        ranges.unsqueeze(-1).expand(B, T, R, C))
    assert torch.equal(lm_p.detach().cpu(), want)
    w = torch.randn(B, T, R, C, generator=g)
    (lm_p * w.to(dev)).sum().backward()
    ref = torch.zeros(B, S + 1, C, dtype=torch.float64)
    ref.scatter_add_(1, ranges.reshape(B, T * R, 1).expand(B, T * R, C),
                     w.double().reshape(B, T * R, C))
    assert (dl.grad.cpu().double() - ref).abs().max().item() <= 1e-5


@pytest.mark.parametrize("C", [1500, 4096, 4100])
def test_joint_loss_wide_rows(gpu_device, C):
    # logits rows held in registers with 8 and 16 pieces per lane, and rows too long for that
    dev = gpu_device
    g = torch.Generator().manual_seed(500 + C)
    B, S, T = 2, 5, 7
    logits = torch.randn(B, T, S + 1, C, generator=g) * 2
    sym = torch.randint(1, C, (B, S), generator=g)
    bnd = torch.tensor([[0, 0, S, T], [0, 0, S - 1, T - 1]], dtype=torch.int64)
    a = logits.clone().requires_grad_(True)
    want = O.loss_joint(a, sym, 0, boundary=bnd, reduction="sum")
    want.backward()
    d = logits.to(dev).requires_grad_(True)
    _say(f"joint loss, C={C}")
    got = fast_rnnt_amd.rnnt_loss(d, sym.to(dev), 0, boundary=bnd.to(dev), reduction="sum")
    got.backward()
    assert abs(got.item() - want.item()) <= 1e-5 * abs(want.item())
    assert (d.grad.cpu() - a.grad).abs().max().item() <= 1e-5


def test_pruning_gradient_when_most_frames_share_a_row(gpu_device):
    """do_rnnt_pruning's lm gradient (the adjoint of the gather, rnnt_loss.py:797-802)
    when thousands of (frame, j) entries point at the same lm row: more than the adjoint
    kernel lists per round (4096), in several scan chunks, plus rows nobody points at."""
    dev = gpu_device
    g = torch.Generator().manual_seed(5)
    B, S, T, C, R = 2, 6, 2300, 5, 2
    am = torch.randn(B, T, C, generator=g)
    lm = torch.randn(B, S + 1, C, generator=g)
    r0 = torch.full((B, T), 2, dtype=torch.int64)
    r0[0, 2000:] = 4                     # rows 2, 3 get 2000 + 2000 entries, rows 4, 5 get 300
    r0[1, ::3] = 0
    ranges = r0.unsqueeze(2) + torch.arange(R)
    w = torch.randn(B, T, R, C, generator=g)
    l = lm.clone().requires_grad_(True)
    _, lp = O.prune(am, l, ranges)
    (lp * w).sum().backward()
    dl = lm.to(dev).requires_grad_(True)
    _, glp = fast_rnnt_amd.do_rnnt_pruning(am.to(dev), dl, ranges.to(dev))
    (glp * w.to(dev)).sum().backward()
    assert (l.grad[0, 6] == 0).all() and (dl.grad[0, 6].cpu() == 0).all()
    # sums of up to 2300 terms: the order of the float32 additions may differ
    assert _close(dl.grad, l.grad, 2e-4, 1e-5), (dl.grad.cpu() - l.grad).abs().max()
    # ... all entries on one row
    ranges = torch.ones(1, T, 2, dtype=torch.int64) * torch.tensor([3, 3])
    w = torch.randn(1, T, 2, C, generator=g)
    l = lm[:1].clone().requires_grad_(True)
    _, lp = O.prune(am[:1], l, ranges)
    (lp * w).sum().backward()
    dl = lm[:1].to(dev).requires_grad_(True)
    _, glp = fast_rnnt_amd.do_rnnt_pruning(am[:1].to(dev), dl, ranges.to(dev))
    (glp * w.to(dev)).sum().backward()
    assert _close(dl.grad, l.grad, 4e-4, 1e-5), (dl.grad.cpu() - l.grad).abs().max()


def test_smoothed_golden(gpu_device):
    dev = gpu_device
    data = torch.load(os.path.join(GOLDEN, "smoothed_logprobs.pt"), weights_only=True)
    for name, c in data.items():
        _say(f"golden smoothed {name}")
        args = (c["lm"].to(dev), c["am"].to(dev), c["symbols"].to(dev), 0, c["lm_only_scale"],
                c["am_only_scale"])
        px, py = fast_rnnt_amd.get_rnnt_logprobs_smoothed(
            *args, boundary=c["boundary"].to(dev), rnnt_type=c["kind"])
        assert _close(px, c["px"], 1e-5, 1e-5) and _close(py, c["py"], 1e-5, 1e-5)
        loss = fast_rnnt_amd.rnnt_loss_smoothed(*args, boundary=c["boundary"].to(dev),
                                                rnnt_type=c["kind"], reduction="none")
        assert _close(loss, c["loss"], 0.0, 1e-5)


@pytest.mark.parametrize("kind", KINDS)
def test_smoothed_gradients(gpu_device, kind):
    dev = gpu_device
    am, lm, sym, bnd = _case(200, 3, 11, 31, 19, torch.float64, kind)
    a = am.clone().requires_grad_(True)
    l = lm.clone().requires_grad_(True)
    want = O.loss_smoothed(l, a, sym, 3, 0.2, 0.15, boundary=bnd, rnnt_type=kind, reduction="mean",
                           delay_penalty=0.01)
    want.backward()
    da = am.to(dev).requires_grad_(True)
    dl = lm.to(dev).requires_grad_(True)
    got = fast_rnnt_amd.rnnt_loss_smoothed(dl, da, sym.to(dev), 3, 0.2, 0.15, boundary=bnd.to(dev),
                                           rnnt_type=kind, reduction="mean", delay_penalty=0.01)
    got.backward()
    assert _close(got, want, 0.0, 1e-6)  # the delay penalty is formed in float32
    assert _close(da.grad, a.grad, 1e-6, 1e-6) and _close(dl.grad, l.grad, 1e-6, 1e-6)


@pytest.mark.parametrize("S", [70, 130, 300])
def test_smoothed_gradients_long_targets(gpu_device, S):
    # more lattice rows than one wave holds (and, at 300, more than the fused am-gradient
    # kernel takes), few symbols, so that most of them occur many times
    dev = gpu_device
    am, lm, sym, bnd = _case(210 + S, 2, S, S + 20, 13, torch.float64, "regular")
    a = am.clone().requires_grad_(True)
    l = lm.clone().requires_grad_(True)
    want = O.loss_smoothed(l, a, sym, 3, 0.1, 0.3, boundary=bnd, rnnt_type="regular", reduction="sum")
    want.backward()
    da = am.to(dev).requires_grad_(True)
    dl = lm.to(dev).requires_grad_(True)
    got = fast_rnnt_amd.rnnt_loss_smoothed(dl, da, sym.to(dev), 3, 0.1, 0.3, boundary=bnd.to(dev),
                                           rnnt_type="regular", reduction="sum")
    got.backward()
    assert _close(got, want, 0.0, 1e-9)
    assert _close(da.grad, a.grad, 1e-8, 1e-8) and _close(dl.grad, l.grad, 1e-8, 1e-8)


def test_small_s_range_never_gives_inf(gpu_device):
    # fast_rnnt/python/tests/rnnt_loss_test.py:615-705: T = 1, s_range raised to its minimum
    dev = gpu_device
    g = torch.Generator().manual_seed(3)
    B, T, C = 2, 1, 10
    for S in range(1, 10):
        am = torch.randn(B, T, C, generator=g).to(dev)
        lm = torch.randn(B, S + 1, C, generator=g).to(dev)
        sym = torch.randint(0, C - 1, (B, S), generator=g).to(dev)
        bnd = torch.tensor([[0, 0, S, T]] * B).to(dev)
        _, (gx, gy) = fast_rnnt_amd.rnnt_loss_simple(lm, am, sym, C - 1, boundary=bnd,
                                                     reduction="none", return_grad=True)
        ranges = fast_rnnt_amd.get_rnnt_prune_ranges(gx, gy, bnd, 2)
        ap, lp = fast_rnnt_amd.do_rnnt_pruning(am, lm, ranges)
        loss = fast_rnnt_amd.rnnt_loss_pruned(torch.sigmoid(ap + lp), sym, ranges, C - 1,
                                              boundary=bnd, reduction="none")
        assert torch.isfinite(loss).all(), (S, loss)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_ranges_that_are_not_consecutive(gpu_device, dtype):
    # The reference takes any `ranges`: row j of frame t scores the symbol of lattice row
    # ranges[b,t,j] and is rolled to lattice row ranges[b,t,0] + j (rnnt_loss.py:955-984).  The
    # loss (which skips logits rows outside the boundary window) must place and skip by that
    # same rule: equal to the (px, py) builder followed by the recursion, and to the oracle.
    dev = gpu_device
    B, S, T, C, R = 3, 12, 20, 15, 4
    g = torch.Generator().manual_seed(811)
    logits = torch.randn(B, T, R, C, generator=g, dtype=dtype)
    sym = torch.randint(1, C, (B, S), generator=g)
    bnd = torch.tensor([[0, 0, S, T], [0, 0, 7, 13], [2, 3, 10, 18]])
    # first entries that follow each window's diagonal (so that every lattice has paths) ...
    t = torch.arange(T).reshape(1, T)
    s0, t0, s1, t1 = (bnd[:, k].reshape(B, 1) for k in range(4))
    along = s0 + ((t - t0).clamp(min=0) * (s1 - s0)) // (t1 - t0) - 1
    first = along.clamp(min=0, max=S + 1 - R).reshape(B, T, 1)
    ranges = first + torch.arange(R).reshape(1, 1, R)
    # ... and later entries shuffled or repeated, within [0, S]
    ranges[:, ::2, 1:] = ranges[:, ::2, 1:].flip(-1)
    ranges[:, 1::3, 2] = ranges[:, 1::3, 1]
    ranges[0, ::5, 3] = S
    a = logits.clone().requires_grad_(True)
    want = O.loss_pruned(a, sym, ranges, 0, boundary=bnd, reduction="none")
    finite = torch.isfinite(want)
    assert finite.all()
    want[finite].sum().backward()

    d1 = logits.to(dev).requires_grad_(True)
    loss = fast_rnnt_amd.rnnt_loss_pruned(d1, sym.to(dev), ranges.to(dev), 0, boundary=bnd.to(dev),
                                          reduction="none")
    loss[finite.to(dev)].sum().backward()
    d2 = logits.to(dev).requires_grad_(True)
    px, py = fast_rnnt_amd.get_rnnt_logprobs_pruned(d2, sym.to(dev), ranges.to(dev), 0,
                                                    boundary=bnd.to(dev))
    scores = fast_rnnt_amd.mutual_information_recursion(px, py, bnd.to(dev))
    (-scores)[finite.to(dev)].sum().backward()
    tol = 1e-4 if dtype == torch.float32 else 1e-9
    assert _close(loss, -scores, 0.0, 1e-6 if dtype == torch.float32 else 1e-12)
    assert _close(loss, want, 0.0, 1e-5 if dtype == torch.float32 else 1e-10)
    assert _close(d1.grad, d2.grad, tol * 0.1, tol * 0.1)
    assert _close(d1.grad, a.grad, tol, tol)


@pytest.mark.parametrize("kind", KINDS)
def test_pruned_with_every_row_kept_equals_unpruned(gpu_device, kind):
    # ranges that keep all S + 1 rows of every frame: rnnt_loss_pruned must give what
    # rnnt_loss gives on the same logits, loss and gradient (the identity the reference's
    # pruned tests print side by side, rnnt_loss_test.py:435-515), and both the oracle's
    dev = gpu_device
    for n, (B, S, T, C) in enumerate([(2, 5, 9, 8), (3, 20, 41, 30), (2, 66, 80, 17)]):
        am, lm, sym, bnd = _case(300 + n, B, S, T, C, torch.float32, kind)
        g = torch.Generator().manual_seed(300 + n)
        logits = torch.randn(B, T, S + 1, C, generator=g)
        ranges = torch.arange(S + 1).reshape(1, 1, S + 1).expand(B, T, S + 1).contiguous()
        _say(f"pruned(S+1) == joint, {kind} shape{n}")
        a = logits.clone().requires_grad_(True)
        want = O.loss_joint(a, sym, 0, boundary=bnd, rnnt_type=kind, reduction="none")
        want.sum().backward()
        full = logits.to(dev).requires_grad_(True)
        joint = fast_rnnt_amd.rnnt_loss(full, sym.to(dev), 0, boundary=bnd.to(dev),
                                        rnnt_type=kind, reduction="none")
        joint.sum().backward()
        kept = logits.to(dev).requires_grad_(True)
        pruned = fast_rnnt_amd.rnnt_loss_pruned(kept, sym.to(dev), ranges.to(dev), 0,
                                                boundary=bnd.to(dev), rnnt_type=kind,
                                                reduction="none")
        pruned.sum().backward()
        assert torch.equal(pruned, joint)
        assert torch.equal(kept.grad, full.grad)
        assert _close(joint, want, 0.0, 1e-5)
        assert _close(full.grad, a.grad, 1e-4, 1e-4)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_losses_do_not_read_logits_outside_the_window(gpu_device, dtype, kind):
    # rnnt_loss / rnnt_loss_pruned skip the logits rows of cells outside an utterance's
    # boundary window: NaN planted there (on the GPU side only) must change nothing -- loss
    # and in-window gradients as the oracle computes them on clean logits, exact zeros outside
    dev = gpu_device
    f32 = dtype == torch.float32
    for n, (B, S, T, C) in enumerate([(3, 9, 20, 12), (2, 40, 70, 1000), (2, 66, 50, 37)]):
        if kind != "regular" and T < S:
            continue
        am, lm, sym, bnd = _case(400 + n, B, S, T, C, dtype, kind)
        g = torch.Generator().manual_seed(400 + n)
        logits = torch.randn(B, T, S + 1, C, generator=g, dtype=dtype)
        s_idx = torch.arange(S + 1).reshape(1, 1, S + 1)
        t_idx = torch.arange(T).reshape(1, T, 1)
        inside = (s_idx <= bnd[:, 2].reshape(B, 1, 1)) & (t_idx < bnd[:, 3].reshape(B, 1, 1))
        poisoned = torch.where(inside.unsqueeze(3), logits, torch.full_like(logits, float("nan")))
        _say(f"window-only joint {kind} {dtype} shape{n}: {int((~inside).sum())} of "
             f"{inside.numel()} rows outside")
        a = logits.clone().requires_grad_(True)
        want = O.loss_joint(a, sym, 0, boundary=bnd, rnnt_type=kind, reduction="sum")
        want.backward()
        d = poisoned.to(dev).requires_grad_(True)
        got = fast_rnnt_amd.rnnt_loss(d, sym.to(dev), 0, boundary=bnd.to(dev), rnnt_type=kind,
                                      reduction="sum")
        got.backward()
        assert _close(got, want, 0.0, 1e-5 if f32 else 1e-12)
        grad = d.grad.cpu()
        assert bool((grad[~inside] == 0).all())
        assert _close(grad[inside], a.grad[inside], 1e-4 if f32 else 1e-9, 1e-4 if f32 else 1e-9)

        # pruned: ranges of width 4 following the diagonal, rows past S_b / frames past T_b out
        R = min(4, S + 1)
        start = (torch.arange(T).reshape(1, T) * (S + 1 - R) // max(T - 1, 1)).expand(B, T)
        ranges = (start.unsqueeze(2) + torch.arange(R).reshape(1, 1, R)).contiguous()
        kept = torch.randn(B, T, R, C, generator=g, dtype=dtype)
        in_p = (ranges <= bnd[:, 2].reshape(B, 1, 1)) & (t_idx < bnd[:, 3].reshape(B, 1, 1))
        poisoned = torch.where(in_p.unsqueeze(3), kept, torch.full_like(kept, float("nan")))
        a = kept.clone().requires_grad_(True)
        want = O.loss_pruned(a, sym, ranges, 0, boundary=bnd, rnnt_type=kind, reduction="none")
        live = torch.isfinite(want.detach())   # an arbitrary diagonal band may lose every path
        want[live].sum().backward()
        d = poisoned.to(dev).requires_grad_(True)
        got = fast_rnnt_amd.rnnt_loss_pruned(d, sym.to(dev), ranges.to(dev), 0,
                                             boundary=bnd.to(dev), rnnt_type=kind,
                                             reduction="none")
        got[live.to(dev)].sum().backward()
        assert torch.equal(torch.isfinite(got.detach().cpu()), live)
        assert _close(got.detach()[live.to(dev)], want.detach()[live], 0.0, 1e-5 if f32 else 1e-12)
        grad = d.grad.cpu()
        assert bool((grad[~in_p] == 0).all())
        assert _close(grad[in_p], a.grad[in_p], 1e-4 if f32 else 1e-9, 1e-4 if f32 else 1e-9)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_pruned_joiner_input_matches_gather_then_tanh(gpu_device, dtype):
    # pruned_joiner_input(am, lm, ranges) == tanh(am_pruned + lm_pruned) on the oracle's
    # do_rnnt_pruning (rnnt_loss.py:780-818), values and both gradients; also the plain sum,
    # rows that are not multiples of 16 bytes, and range entries outside [0, S] (NaN rows)
    dev = gpu_device
    f32 = dtype == torch.float32
    for n, (B, S, T, R, C) in enumerate([(2, 5, 9, 3, 8), (3, 20, 41, 5, 500), (2, 30, 25, 7, 37),
                                         (2, 12, 16, 13, 260)]):
        g = torch.Generator().manual_seed(700 + n)
        am = torch.randn(B, T, C, generator=g, dtype=dtype)
        lm = torch.randn(B, S + 1, C, generator=g, dtype=dtype)
        start = torch.randint(0, S + 2 - R, (B, T), generator=g)
        ranges = (start.unsqueeze(2) + torch.arange(R).reshape(1, 1, R)).contiguous()
        weight = torch.randn(B, T, R, C, generator=g, dtype=dtype)
        for act in ("tanh", None):
            _say(f"pruned joiner input {dtype} shape{n} activation={act}")
            a = am.clone().requires_grad_(True)
            l = lm.clone().requires_grad_(True)
            am_p, lm_p = O.prune(a, l, ranges)
            want = torch.tanh(am_p + lm_p) if act else am_p + lm_p
            (want * weight).sum().backward()
            da = am.to(dev).requires_grad_(True)
            dl = lm.to(dev).requires_grad_(True)
            got = fast_rnnt_amd.pruned_joiner_input(da, dl, ranges.to(dev), activation=act)
            (got * weight.to(dev)).sum().backward()
            tol = 2e-6 if f32 else 1e-12
            assert _close(got, want, tol, tol)
            assert _close(da.grad, a.grad, 1e-5 if f32 else 1e-11, 1e-5 if f32 else 1e-11)
            assert _close(dl.grad, l.grad, 2e-5 if f32 else 1e-11, 1e-5 if f32 else 1e-11)
            # the same numbers as the two-step route through do_rnnt_pruning on the GPU
            ea = am.to(dev).requires_grad_(True)
            el = lm.to(dev).requires_grad_(True)
            p_am, p_lm = fast_rnnt_amd.do_rnnt_pruning(ea, el, ranges.to(dev))
            two = torch.tanh(p_am + p_lm) if act else p_am + p_lm
            assert _close(got, two, tol, tol)
    bad = ranges.clone()
    bad[0, 0, 0] = S + 1
    out = fast_rnnt_amd.pruned_joiner_input(am.to(dev), lm.to(dev), bad.to(dev))
    assert torch.isnan(out[0, 0, 0]).all() and torch.isfinite(out[0, 0, 1]).all()


@pytest.mark.parametrize("reduction", ["none", "mean", "sum"])
@pytest.mark.parametrize("which", ["joint", "pruned", "smoothed"])
def test_loss_tail_reductions_weights_and_returned_gradients(gpu_device, which, reduction):
    """The part the three losses share after px, py: delay penalty, recursion, reduction.

    The loss is weighted per utterance before backward() (for "none"), so that the
    gradient of the scores is not a constant; px_grad / py_grad are compared as returned
    (the occupation counts) and after backward(), which scales them in place as the
    reference's recursion does (mutual_information.py:162-178).
    """
    dev = gpu_device
    kind = "regular"
    B, S, T, C, R = 4, 7, 19, 11, 4
    am, lm, sym, bnd = _case(300, B, S, T, C, torch.float64, kind)
    w = torch.tensor([0.5, -1.25, 2.0, 0.0], dtype=torch.float64)

    def run(mod_losses, to):
        a = to(am).requires_grad_(True)
        l = to(lm).requires_grad_(True)
        kw = dict(boundary=to(bnd), rnnt_type=kind, delay_penalty=0.02, reduction=reduction,
                  return_grad=True)
        if which == "smoothed":
            loss, (gx, gy) = mod_losses["smoothed"](l, a, to(sym), 2, 0.3, 0.1, **kw)
        elif which == "joint":
            logits = torch.tanh(a.unsqueeze(2) + l.unsqueeze(1)) * 2
            loss, (gx, gy) = mod_losses["joint"](logits, to(sym), 2, **kw)
        else:
            start = torch.clamp(torch.arange(T) * (S + 1 - R) // T, 0, S + 1 - R)
            ranges = to((start.reshape(1, T, 1) + torch.arange(R).reshape(1, 1, R))
                        .expand(B, T, R).contiguous())
            lp = torch.gather(l.unsqueeze(1).expand(B, T, S + 1, C), 2,
                              ranges.unsqueeze(3).expand(B, T, R, C))
            logits = torch.tanh(a.unsqueeze(2) + lp) * 2
            loss, (gx, gy) = mod_losses["pruned"](logits, to(sym), ranges, 2, **kw)
        before = gx.detach().clone(), gy.detach().clone()
        total = (loss * to(w)).sum() if reduction == "none" else loss * 1.5
        total.backward()
        return loss, before, (gx.detach(), gy.detach()), a.grad, l.grad

    want = run({"smoothed": O.loss_smoothed, "joint": O.loss_joint, "pruned": O.loss_pruned},
               lambda x: x.clone())
    got = run({"smoothed": fast_rnnt_amd.rnnt_loss_smoothed, "joint": fast_rnnt_amd.rnnt_loss,
               "pruned": fast_rnnt_amd.rnnt_loss_pruned}, lambda x: x.to(dev))
    _say(f"loss tail {which} {reduction}")
    assert got[0].shape == want[0].shape and _close(got[0], want[0], 0.0, 1e-6)
    for i in (0, 1):
        assert _close(got[1][i], want[1][i], 1e-7), "occupation counts as returned"
        assert _close(got[2][i], want[2][i], 1e-7), "the same tensors after backward()"
    # backward() did rescale them: by -w[b], -1.5/B or -1.5
    scale = {"none": -w, "mean": torch.full((B,), -1.5 / B, dtype=torch.float64),
             "sum": torch.full((B,), -1.5, dtype=torch.float64)}[reduction]
    assert _close(got[2][0], got[1][0].cpu() * scale.reshape(B, 1, 1), 1e-12)
    assert _close(got[3], want[3], 1e-7, 1e-7) and _close(got[4], want[4], 1e-7, 1e-7)


@pytest.mark.parametrize("kind", KINDS)
def test_smoothed_loss_equals_helper_then_recursion(gpu_device, kind):
    """rnnt_loss_smoothed writes the -inf beyond the last frame inside its kernel; the public
    get_rnnt_logprobs_smoothed followed by the recursion (rnnt_loss.py:1364-1365, 1480-1494)
    must give the same loss and gradients."""
    dev = gpu_device
    am, lm, sym, bnd = _case(310, 3, 9, 26, 15, torch.float64, kind)
    res = []
    for direct in (True, False):
        a = am.to(dev).requires_grad_(True)
        l = lm.to(dev).requires_grad_(True)
        if direct:
            loss = fast_rnnt_amd.rnnt_loss_smoothed(l, a, sym.to(dev), 1, 0.2, 0.1,
                                                    boundary=bnd.to(dev), rnnt_type=kind,
                                                    reduction="none")
        else:
            px, py = fast_rnnt_amd.get_rnnt_logprobs_smoothed(l, a, sym.to(dev), 1, 0.2, 0.1,
                                                              boundary=bnd.to(dev), rnnt_type=kind)
            loss = -fast_rnnt_amd.mutual_information_recursion(px, py, bnd.to(dev))
        loss.sum().backward()
        res.append((loss.detach(), a.grad, l.grad))
    for x, y in zip(*res):
        assert _close(x, y, 1e-12, 1e-12)


@pytest.mark.parametrize("which", ["simple", "smoothed", "joint", "pruned"])
def test_windows_without_a_path(gpu_device, which):
    """Boundary rows that leave no alignment: an empty range of frames behind a symbol range
    that is not (regular lattice: the -inf column is all there is to emit on), or none of
    either.  The loss is +inf or finite as in the reference, and the gradients that reach
    the inputs are the reference's -- the recursion leaves 1, not 0, in px_grad at the
    masked cells of a lattice without a path, which the -inf masking must not let through
    (rnnt_loss.py:45-63: scatter_ cuts the gradient)."""
    dev = gpu_device
    B, S, T, C, R = 4, 12, 20, 9, 4
    g = torch.Generator().manual_seed(77)
    am = torch.randn(B, T, C, generator=g, dtype=torch.float64)
    lm = torch.randn(B, S + 1, C, generator=g, dtype=torch.float64)
    sym = torch.randint(0, C, (B, S), generator=g)
    bnd = torch.tensor([[2, 1, 9, 1], [0, 0, 12, 20], [3, 5, 3, 5], [0, 7, 6, 7]])
    start = torch.clamp(torch.arange(T) * (S + 1 - R) // (T - 1), 0, S + 1 - R)
    ranges = (start.reshape(1, T, 1) + torch.arange(R).reshape(1, 1, R)).expand(B, T, R).contiguous()
    w = torch.tensor([1.0, 0.5, -2.0, 0.25], dtype=torch.float64)

    def run(fns, to):
        a = to(am).requires_grad_(True)
        l = to(lm).requires_grad_(True)
        kw = dict(boundary=to(bnd), reduction="none", return_grad=True)
        if which == "simple":
            loss, (gx, gy) = fns[0](l, a, to(sym), 0, **kw)
        elif which == "smoothed":
            loss, (gx, gy) = fns[1](l, a, to(sym), 0, 0.2, 0.1, **kw)
        elif which == "joint":
            loss, (gx, gy) = fns[2](torch.tanh(a.unsqueeze(2) + l.unsqueeze(1)), to(sym), 0, **kw)
        else:
            rg = to(ranges)
            lp = torch.gather(l.unsqueeze(1).expand(B, T, S + 1, C), 2,
                              rg.unsqueeze(3).expand(B, T, R, C))
            loss, (gx, gy) = fns[3](torch.tanh(a.unsqueeze(2) + lp), to(sym), rg, 0, **kw)
        occ = gx.detach().clone(), gy.detach().clone()
        # (utterances without a path have an infinite loss; their gradients still flow)
        (torch.where(torch.isfinite(loss), loss, torch.zeros_like(loss)) * to(w)).sum().backward()
        return loss.detach(), occ, a.grad, l.grad

    want = run((O.loss_simple, O.loss_smoothed, O.loss_joint, O.loss_pruned), lambda x: x.clone())
    got = run((fast_rnnt_amd.rnnt_loss_simple, fast_rnnt_amd.rnnt_loss_smoothed,
               fast_rnnt_amd.rnnt_loss, fast_rnnt_amd.rnnt_loss_pruned), lambda x: x.to(dev))
    _say(f"no path {which}: losses {want[0].tolist()}")
    assert torch.isinf(want[0][0]) and torch.isfinite(want[0][1])
    assert _close(got[0], want[0], 0.0, 1e-9)
    assert _close(got[1][0], want[1][0], 1e-9) and _close(got[1][1], want[1][1], 1e-9)
    assert _close(got[2], want[2], 1e-9, 1e-9) and _close(got[3], want[3], 1e-9, 1e-9)


@pytest.mark.parametrize("which", ["simple", "smoothed", "joint"])
def test_gradient_of_a_loss_without_a_path(gpu_device, which):
    """The same with the infinite losses left in the sum: their utterances' occupation
    gradients (1 at the masked cells) are scaled and passed back like any others, and must
    stop where the reference's scatter_ stops them."""
    dev = gpu_device
    B, S, T, C = 2, 10, 16, 7
    g = torch.Generator().manual_seed(78)
    am = torch.randn(B, T, C, generator=g, dtype=torch.float64)
    lm = torch.randn(B, S + 1, C, generator=g, dtype=torch.float64)
    sym = torch.randint(0, C, (B, S), generator=g)
    bnd = torch.tensor([[2, 1, 9, 1], [0, 0, 10, 16]])
    res = []
    for gpu_side in (False, True):
        to = (lambda x: x.to(dev)) if gpu_side else (lambda x: x.clone())
        a = to(am).requires_grad_(True)
        l = to(lm).requires_grad_(True)
        kw = dict(boundary=to(bnd), reduction="none")
        if which == "simple":
            f = fast_rnnt_amd.rnnt_loss_simple if gpu_side else O.loss_simple
            loss = f(l, a, to(sym), 0, **kw)
        elif which == "smoothed":
            f = fast_rnnt_amd.rnnt_loss_smoothed if gpu_side else O.loss_smoothed
            loss = f(l, a, to(sym), 0, 0.2, 0.1, **kw)
        else:
            f = fast_rnnt_amd.rnnt_loss if gpu_side else O.loss_joint
            loss = f(a.unsqueeze(2) + l.unsqueeze(1), to(sym), 0, **kw)
        loss.backward(torch.ones_like(loss))
        res.append((loss.detach(), a.grad, l.grad))
    _say(f"infinite loss {which}: {res[0][0].tolist()}")
    assert torch.isinf(res[0][0][0])
    for x, y in zip(res[1], res[0]):
        assert _close(x, y, 1e-9, 1e-9)


def test_c5_unpruned_full_size(gpu_device):
    dev = gpu_device
    w = workloads.make("c5")
    _say(f"workload c5: logits {tuple(w.logits.shape)}")
    a = w.logits.clone().requires_grad_(True)
    want = O.loss_joint(a, w.symbols, 0, boundary=w.boundary, reduction="sum")
    want.backward()
    d = w.logits.to(dev).requires_grad_(True)
    got = fast_rnnt_amd.rnnt_loss(d, w.symbols.to(dev), 0, boundary=w.boundary.to(dev),
                                  reduction="sum")
    got.backward()
    rel = abs(got.item() - want.item()) / abs(want.item())
    diff = (d.grad.cpu() - a.grad).abs().max().item()
    _say(f"  loss rel diff {rel:.2e}, logits.grad max diff {diff:.2e}")
    assert rel <= 1e-5 and diff <= 1e-4


def test_c3_pruned_full_size(gpu_device):
    dev = gpu_device
    w = workloads.make("c3")
    _say("workload c3: smoothed -> ranges -> pruning -> joiner -> pruned loss")

    def run(am_, lm_, sym_, bnd_, W_, F, feed=None):
        simple, (gx, gy) = F["smoothed"](lm_, am_, sym_, 0, 0.25, 0.0, boundary=bnd_,
                                         reduction="sum", return_grad=True)
        gx0, gy0 = gx.detach().clone(), gy.detach().clone()
        ranges = F["ranges"](*(feed if feed is not None else (gx, gy)), bnd_, w.s_range)
        am_p, lm_p = F["prune"](am_, lm_, ranges)
        loss = F["pruned"](torch.tanh(am_p + lm_p) @ W_, sym_, ranges, 0, boundary=bnd_,
                           reduction="sum")
        (simple + loss).backward()
        return simple, loss, ranges, gx0, gy0

    cpu = dict(smoothed=O.loss_smoothed, ranges=O.prune_ranges, prune=O.prune, pruned=O.loss_pruned)
    gpu = dict(smoothed=fast_rnnt_amd.rnnt_loss_smoothed,
               ranges=fast_rnnt_amd.get_rnnt_prune_ranges,
               prune=fast_rnnt_amd.do_rnnt_pruning, pruned=fast_rnnt_amd.rnnt_loss_pruned)
    a = w.am.clone().requires_grad_(True)
    l = w.lm.clone().requires_grad_(True)
    ws, wl, wr, wgx, wgy = run(a, l, w.symbols, w.boundary, w.joiner, cpu)
    da = w.am.to(dev).requires_grad_(True)
    dl = w.lm.to(dev).requires_grad_(True)
    # the GPU run is fed the CPU path's gradients for the ranges, so that both
    # pipelines prune identically (the acceptance criterion for bit-exact ranges)
    gs, gl, gr, ggx, ggy = run(da, dl, w.symbols.to(dev), w.boundary.to(dev), w.joiner.to(dev),
                               gpu, feed=(wgx.to(dev), wgy.to(dev)))
    assert torch.equal(gr.cpu(), wr)
    own = fast_rnnt_amd.get_rnnt_prune_ranges(ggx, ggy, w.boundary.to(dev), w.s_range)
    frames = (own.cpu()[:, :, 0] != wr[:, :, 0]).sum().item()
    _say(f"  smoothed loss rel {abs(gs.item() - ws.item()) / abs(ws.item()):.2e}, pruned loss rel "
         f"{abs(gl.item() - wl.item()) / abs(wl.item()):.2e}, px_grad diff "
         f"{(ggx.cpu() - wgx).abs().max().item():.2e}, py_grad diff "
         f"{(ggy.cpu() - wgy).abs().max().item():.2e}, frames whose range differs when each "
         f"side uses its own gradients: {frames} of {wr.shape[0] * wr.shape[1]}")
    assert abs(gs.item() - ws.item()) <= 1e-5 * abs(ws.item())
    assert abs(gl.item() - wl.item()) <= 1e-5 * abs(wl.item())
    # Scores reach |p| ~ 3000 here, where one float32 ulp of p is 2.4e-4, and the two
    # pipelines' px / py agree only to rounding (two GEMM summation orders).  The bound is
    # what such rounding does to the float32 CPU reference ITSELF: 1.25 x the movement of
    # its gradients under a one-ulp nudge of px / py (tests/ulp_sensitivity.py; 1.0e-4 at
    # this workload, so 1.25e-4), not less than the acceptance criterion's 1e-4.  The
    # recursion kernels alone, on identical px / py, stay below 1e-4
    # (tests/test_gpu_recursion_fidelity.py).
    opx, opy = O.lattice_logprobs_smoothed(w.lm, w.am, w.symbols, 0, 0.25, 0.0,
                                           boundary=w.boundary)
    bound = U.grad_bound(opx, opy, w.boundary)
    _say(f"  px_grad / py_grad bound from the reference's one-ulp sensitivity: {bound:.2e}")
    assert bound <= 2e-4
    assert _close(ggx, wgx, bound) and _close(ggy, wgy, bound)
    # am.grad / lm.grad add such cells up over lattice rows / frames
    assert _close(da.grad, a.grad, 2 * bound, 1e-3) and _close(dl.grad, l.grad, 2 * bound, 1e-3)
