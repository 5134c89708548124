"""Parity of the gfx950 lattice recursion with the CPU oracle (needs the GPU).

Tolerances: float32 scores 1e-5 relative, float32 gradients 1e-4 absolute,
float64 1e-10 -- the operators are called through the C-ABI library.
"""
import math
import sys

import pytest
import torch

import fast_rnnt_amd
from fast_rnnt_amd import _fast_rnnt
from oracle import recursion as oracle

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _windows(g, B, S, T, modified):
    rows = []
    for b in range(B):
        kind = b % 5
        if kind == 0:
            rows.append([0, 0, S, T])
        elif kind == 1:  # empty symbol range
            s = int(torch.randint(0, S + 1, (1,), generator=g))
            rows.append([s, 0, s, T])
        elif kind == 2:  # empty frame range
            t = int(torch.randint(0, T + 1, (1,), generator=g))
            rows.append([0, t, S, t])
        else:
            s0 = int(torch.randint(0, S + 1, (1,), generator=g))
            s1 = int(torch.randint(s0, S + 1, (1,), generator=g))
            t0 = int(torch.randint(0, T + 1, (1,), generator=g))
            t1 = int(torch.randint(t0, T + 1, (1,), generator=g))
            rows.append([s0, t0, s1, t1])
    return torch.tensor(rows, dtype=torch.int64)


def _compare(px, py, bnd, w, dev, tag):
    dtype = px.dtype
    B, S, _ = px.shape
    T = py.shape[2]
    _say(f"case {tag}: B={B} S={S} T={T} modified={px.shape[2] == T} dtype={dtype} "
         f"boundary={'yes' if bnd is not None else 'no'}")
    p_cpu = torch.full((B, S + 1, T + 1), float("nan"), dtype=dtype)
    a_cpu = oracle.mi_forward(px, py, bnd, p_cpu)
    gx_cpu, gy_cpu = oracle.mi_backward(px, py, bnd, p_cpu, w)

    dpx, dpy = px.to(dev), py.to(dev)
    dbnd = bnd.to(dev) if bnd is not None else None
    p_gpu = torch.full((B, S + 1, T + 1), float("nan"), dtype=dtype, device=dev)
    a_gpu = _fast_rnnt.mutual_information_forward(dpx, dpy, dbnd, p_gpu)
    dw = w.to(dev)
    gx_gpu, gy_gpu = _fast_rnnt.mutual_information_backward(dpx, dpy, dbnd, p_gpu, dw)
    torch.cuda.synchronize()

    rtol, gtol = (1e-5, 1e-4) if dtype == torch.float32 else (1e-12, 1e-10)
    a_gpu, p_gpu = a_gpu.cpu(), p_gpu.cpu()
    both_inf = torch.isinf(a_cpu) & (a_cpu == a_gpu)
    scale = a_cpu.abs().clamp(min=1.0)
    assert bool((both_inf | ((a_cpu - a_gpu).abs() <= rtol * scale)).all()), (a_cpu, a_gpu)
    # the window of p agrees, and nothing outside it is written
    written = ~torch.isnan(p_cpu)
    assert torch.equal(written, ~torch.isnan(p_gpu))
    pc, pg = p_cpu[written], p_gpu[written]
    same_inf = torch.isinf(pc) & (pc == pg)
    # A cell of p is a running sum along lattice paths: its absolute error is set by the
    # largest magnitude met on the way, not by its own.  Scores that climb to hundreds and
    # come back through zero keep errors of a few ulps of that maximum (the float32 CPU
    # reference itself is then 6e-5 off the float64 one at cells with |p| < 1, see
    # tests/test_oracle_conditioning.py), so the relative bound gets that much slack.
    finite = torch.isfinite(pc)
    top = pc[finite].abs().max().item() if bool(finite.any()) else 0.0
    slack = 4 * torch.finfo(dtype).eps * top
    assert bool((same_inf | ((pc - pg).abs() <= rtol * pc.abs().clamp(min=1.0) + slack)).all())
    assert (gx_cpu - gx_gpu.cpu()).abs().max().item() <= gtol if gx_cpu.numel() else True
    assert (gy_cpu - gy_gpu.cpu()).abs().max().item() <= gtol if gy_cpu.numel() else True
    # the gradient reaching the lattice origin is written back into ans_grad
    reach = dw.cpu()
    live = torch.isfinite(a_cpu)
    assert torch.allclose(reach[live], w[live], rtol=1e-3, atol=1e-6)


SHAPES = [
    # B, S, T
    (1, 1, 1), (3, 3, 4), (5, 7, 33), (5, 16, 250), (4, 63, 70), (4, 64, 40), (3, 65, 130),
    (2, 130, 97), (5, 200, 19), (2, 1, 500), (2, 300, 5),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_random_lattices_match_oracle(gpu_device, dtype, modified):
    g = torch.Generator().manual_seed(100 + int(modified))
    for n, (B, S, T) in enumerate(SHAPES):
        px = torch.randn(B, S, T + (0 if modified else 1), generator=g, dtype=dtype)
        py = torch.randn(B, S + 1, T, generator=g, dtype=dtype)
        if not modified and n % 2 == 0:
            px[:, :, T] = -math.inf  # as the loss layer produces it
        w = torch.randn(B, generator=g, dtype=dtype)
        _compare(px, py, None, w, gpu_device, f"plain{n}")
        _compare(px, py, _windows(g, B, S, T, modified), w, gpu_device, f"windows{n}")


@pytest.mark.parametrize("modified", [False, True])
def test_tile_and_seam_borders(gpu_device, modified):
    # The sweep waves treat a 32-step tile as "plain" (no tests inside) when all its steps
    # exist, the result's step is not among them and every seam column it looks at exists;
    # a wave feeds the seam only when rows lie below it.  Frame counts around the multiples
    # of 32 and row counts around one, two and three waves of 64 rows put every one of
    # those borders on either side.
    g = torch.Generator().manual_seed(300 + int(modified))
    n = 0
    for S in (62, 63, 64, 65, 126, 127, 128, 129, 191, 192):
        for T in (31, 32, 33, 63, 64, 65, 71, 72, 95, 96, 97, 100):
            if modified and T < S:
                continue
            B = 2
            px = -0.7 + 0.3 * torch.randn(B, S, T + (0 if modified else 1), generator=g)
            py = -0.7 + 0.3 * torch.randn(B, S + 1, T, generator=g)
            if not modified:
                px[:, :, T] = -math.inf
            # second utterance: a window that ends a few rows / frames early
            bnd = torch.tensor([[0, 0, S, T], [0, 0, S - n % 3, T - n % 5]], dtype=torch.int64)
            if not modified:
                px[1, :, T - n % 5] = -math.inf
            _compare(px, py, bnd, torch.ones(B), gpu_device, f"border{n}")
            n += 1


def test_large_magnitudes_and_neg_inf(gpu_device):
    # fast_rnnt/python/tests/mutual_information_test.py:113-130 ("big" inputs)
    g = torch.Generator().manual_seed(7)
    B, S, T = 4, 20, 90
    for offset in (15.0, -40.0):
        px = torch.randn(B, S, T + 1, generator=g) + offset
        py = torch.randn(B, S + 1, T, generator=g) + offset
        px[:, :, T] = -math.inf
        _compare(px, py, None, torch.ones(B), gpu_device, f"offset{offset}")
    px = torch.full((B, S, T + 1), -math.inf)
    py = torch.randn(B, S + 1, T, generator=g)
    _compare(px, py, None, torch.ones(B), gpu_device, "blocked-x")


def test_taller_than_one_workgroup(gpu_device):
    # more rows than 16 waves hold: the band loop and the wrap-around seam
    g = torch.Generator().manual_seed(8)
    B, S, T = 2, 1100, 9
    px = 0.1 * torch.randn(B, S, T + 1, generator=g, dtype=torch.float64)
    py = 0.1 * torch.randn(B, S + 1, T, generator=g, dtype=torch.float64)
    _compare(px, py, None, torch.ones(B, dtype=torch.float64), gpu_device, "tall")
    px32, py32 = px.float(), py.float()
    _compare(px32, py32, None, torch.ones(B), gpu_device, "tall32")


def test_long_utterance_two_tile_buffers(gpu_device):
    # T beyond what three LDS tile buffers per sweep wave leave room for (about 6100 frames
    # with two sweep waves): the float kernels fall back to two buffers and fewer staging
    # waves.  Inputs centred at -log 2 keep |p| small, so the float32 bounds stay meaningful.
    g = torch.Generator().manual_seed(9)
    B, S, T = 2, 70, 6300
    px = -math.log(2.0) + 0.05 * torch.randn(B, S, T + 1, generator=g)
    py = -math.log(2.0) + 0.05 * torch.randn(B, S + 1, T, generator=g)
    bnd = torch.tensor([[0, 0, S, T], [3, 40, 66, 6290]], dtype=torch.int64)
    _compare(px, py, bnd, torch.ones(B), gpu_device, "long")


def test_north_star_shape(gpu_device):
    g = torch.Generator().manual_seed(1002)
    B, S, T = 32, 80, 250
    px = -8 + 2.8 * torch.randn(B, S, T + 1, generator=g)
    py = -8 + 2.8 * torch.randn(B, S + 1, T, generator=g)
    Tb = torch.round(T * (0.6 + 0.4 * torch.rand(B, generator=g))).long()
    Sb = torch.minimum(torch.round(S * (0.6 + 0.4 * torch.rand(B, generator=g))).long(), Tb)
    z = torch.zeros(B, dtype=torch.int64)
    bnd = torch.stack([z, z, Sb, Tb], 1)
    px[torch.arange(B), :, Tb] = -math.inf
    _compare(px, py, bnd, torch.ones(B), gpu_device, "c2-shaped")


def test_invalid_window_is_skipped_not_read(gpu_device):
    px = torch.zeros(2, 3, 5, device=gpu_device)
    py = torch.zeros(2, 4, 4, device=gpu_device)
    p = torch.zeros(2, 4, 5, device=gpu_device)
    bnd = torch.tensor([[0, 0, 3, 4], [0, 0, 9, 4]], device=gpu_device)
    ans = _fast_rnnt.mutual_information_forward(px, py, bnd, p)
    gx, gy = _fast_rnnt.mutual_information_backward(px, py, bnd, p, torch.ones(2, device=gpu_device))
    assert math.isnan(ans[1].item()) and math.isfinite(ans[0].item())
    assert (gx[1] == 0).all() and (gy[1] == 0).all()
    # the operator also reports the row to the host, which raises it when it next looks
    with pytest.raises(AssertionError, match="boundary row 1"):
        fast_rnnt_amd.check_boundaries()


def test_autograd_front_end(gpu_device):
    g = torch.Generator().manual_seed(3)
    px = torch.randn(3, 6, 12, generator=g)
    py = torch.randn(3, 7, 11, generator=g)
    bnd = torch.tensor([[0, 0, 6, 11], [0, 0, 4, 9], [1, 2, 5, 10]])
    a = px.clone().requires_grad_(True)
    c = py.clone().requires_grad_(True)
    want, (wx, wy) = oracle.mutual_information_recursion(a, c, bnd, return_grad=True)
    wx0 = wx.clone()
    (want * torch.tensor([1.0, 2.0, -3.0])).sum().backward()

    da = px.to(gpu_device).requires_grad_(True)
    dc = py.to(gpu_device).requires_grad_(True)
    got, (gx, gy) = fast_rnnt_amd.mutual_information_recursion(da, dc, bnd.to(gpu_device), return_grad=True)
    assert torch.allclose(gx.cpu(), wx0, atol=1e-5)
    (got * torch.tensor([1.0, 2.0, -3.0], device=gpu_device)).sum().backward()
    assert torch.allclose(got.detach().cpu(), want.detach(), rtol=1e-5)
    assert torch.allclose(da.grad.cpu(), a.grad, atol=1e-4)
    assert torch.allclose(dc.grad.cpu(), c.grad, atol=1e-4)
    assert torch.allclose(gx.cpu(), wx, atol=1e-4)  # scaled in place by backward, like the reference
    # a boundary row out of range: the kernel skips the row (nan) and the reference's
    # AssertionError (mutual_information.py:277-288) is raised once the host looks
    bad = torch.tensor([[0, 0, 7, 11]] * 3, device=gpu_device)
    scores = fast_rnnt_amd.mutual_information_recursion(da, dc, bad)
    with pytest.raises(AssertionError):
        fast_rnnt_amd.check_boundaries()
    assert torch.isnan(scores).all()
    fast_rnnt_amd.set_boundary_checks("host")
    try:
        with pytest.raises(AssertionError):
            fast_rnnt_amd.mutual_information_recursion(da, dc, bad)
    finally:
        fast_rnnt_amd.set_boundary_checks("device")


def test_joint_recursion_splits_the_total(gpu_device):
    # fast_rnnt/python/tests/mutual_information_test.py:138-154
    g = torch.Generator().manual_seed(4)
    px = torch.randn(2, 5, 9, generator=g, dtype=torch.float64).to(gpu_device)
    py = torch.randn(2, 6, 8, generator=g, dtype=torch.float64).to(gpu_device)
    m = fast_rnnt_amd.mutual_information_recursion(px, py)
    m1 = fast_rnnt_amd.joint_mutual_information_recursion((px,), (py,))
    m2 = fast_rnnt_amd.joint_mutual_information_recursion((px * 0.5, px * 0.5), (py * 0.5, py * 0.5))
    assert torch.allclose(m, m1[0], atol=1e-9)
    assert torch.allclose(m, m2.sum(0), atol=1e-9)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_joint_recursion_matches_oracle(gpu_device, dtype, modified):
    # shares per term and their gradients against the CPU restatement of
    # mutual_information.py:314-425, with windows and blocked cells
    dev = gpu_device
    g = torch.Generator().manual_seed(31 + int(modified))
    for B, S, T, N in [(3, 6, 9, 1), (4, 70, 40, 3), (2, 33, 150, 2)]:
        if modified and S > T:
            S, T = T, S   # the modified lattice has no path with more symbols than frames
        _say(f"joint recursion {dtype} modified={modified} B={B} S={S} T={T} N={N}")
        xs = [torch.randn(B, S, T + (0 if modified else 1), generator=g, dtype=dtype) / N
              for _ in range(N)]
        ys = [torch.randn(B, S + 1, T, generator=g, dtype=dtype) / N for _ in range(N)]
        xs[0][:, 1, 2] = -math.inf
        if not modified:
            xs[0][:, :, T] = -math.inf
        for bnd in (None, _windows(g, B, S, T, modified)):
            cx = [x.clone().requires_grad_(True) for x in xs]
            cy = [y.clone().requires_grad_(True) for y in ys]
            want = oracle.joint_mutual_information_recursion(cx, cy, bnd)
            weights = torch.randn(N, B, generator=g, dtype=dtype)
            live = torch.isfinite(want.detach().sum(0))  # utterances with a path
            assert bool(live.any())
            (want[:, live] * weights[:, live]).sum().backward()
            dx = [x.to(dev).requires_grad_(True) for x in xs]
            dy = [y.to(dev).requires_grad_(True) for y in ys]
            got = fast_rnnt_amd.joint_mutual_information_recursion(
                dx, dy, bnd.to(dev) if bnd is not None else None)
            (got[:, live.to(dev)] * weights.to(dev)[:, live.to(dev)]).sum().backward()
            assert got.shape == (N, B)
            tol = 2e-5 if dtype == torch.float32 else 1e-10
            w_, g_ = want.detach()[:, live], got.detach().cpu()[:, live]
            assert torch.allclose(g_, w_, rtol=tol, atol=tol * max(1.0, float(w_.abs().max())))
            # the total is the plain recursion's score
            plain = fast_rnnt_amd.mutual_information_recursion(
                sum(x.to(dev) for x in xs), sum(y.to(dev) for y in ys),
                bnd.to(dev) if bnd is not None else None)
            assert torch.allclose(got.detach().sum(0)[live.to(dev)], plain[live.to(dev)],
                                  rtol=tol, atol=tol * 10)
            gtol = 1e-4 if dtype == torch.float32 else 1e-9
            for n in range(N):
                assert (dx[n].grad.cpu() - cx[n].grad).abs().max().item() <= gtol * 3
                assert (dy[n].grad.cpu() - cy[n].grad).abs().max().item() <= gtol * 3


def test_a_wait_that_runs_out_shows_as_nan(gpu_device):
    # The kernels' waves meet through bounded waits.  With the bound set to one poll from the
    # host every first wait fails (the staged tiles need a memory round trip to arrive): the
    # kernels must still exit, and mark what they could not finish -- NaN scores from the
    # forward kernel, NaN at the window's first cell of px_grad / py_grad and in the
    # written-back ans_grad from the backward kernel.  Afterwards everything is normal again.
    from fast_rnnt_amd import _lib
    dev = gpu_device
    g = torch.Generator().manual_seed(12)
    B, S, T = 6, 80, 250
    px = torch.randn(B, S, T + 1, generator=g).to(dev)
    py = torch.randn(B, S + 1, T, generator=g).to(dev)
    bnd = torch.tensor([[0, 0, S, T], [2, 3, 70, 200]] * 3).to(dev)
    p = torch.empty(B, S + 1, T + 1, device=dev)
    good = _fast_rnnt.mutual_information_forward(px, py, bnd, p)
    lib = _lib.load()
    lib.frnnt_set_spin_limit(1)
    try:
        _say("forward with a one-poll bound")
        q = torch.empty_like(p)
        ans = _fast_rnnt.mutual_information_forward(px, py, bnd, q)
        torch.cuda.synchronize()
        assert torch.isnan(ans).all()
        _say("backward with a one-poll bound")
        seed = torch.ones(B, device=dev)
        gx, gy = _fast_rnnt.mutual_information_backward(px, py, bnd, p, seed)
        torch.cuda.synchronize()
        rows = bnd.cpu().tolist()
        for b, (s0, t0, _, _) in enumerate(rows):
            assert math.isnan(gx[b, s0, t0].item()) and math.isnan(gy[b, s0, t0].item())
        assert torch.isnan(seed).all()
    finally:
        lib.frnnt_set_spin_limit(0)
    again = _fast_rnnt.mutual_information_forward(px, py, bnd, torch.empty_like(p))
    gx, gy = _fast_rnnt.mutual_information_backward(px, py, bnd, p, torch.ones(B, device=dev))
    assert torch.equal(again, good) and torch.isfinite(gx).all() and torch.isfinite(gy).all()
