"""Pins the plain-C recursion oracle (oracle/mi_oracle.c) without the reference:
closed forms, brute force, invariants, finite differences -- and, when
oracle/_ref has been built, bit-equality with the reference's own C++.
"""
import math

import numpy as np
import pytest
import torch

import lattice_truth as truth
from oracle import recursion, ref_build

DTYPES = [torch.float32, torch.float64]


def _run(px, py, boundary=None, ans_grad=None):
    B, S, _ = px.shape
    T = py.shape[2]
    p = torch.full((B, S + 1, T + 1), float("nan"), dtype=px.dtype)
    ans = recursion.mi_forward(px, py, boundary, p)
    if ans_grad is None:
        ans_grad = torch.ones(B, dtype=px.dtype)
    gx, gy = recursion.mi_backward(px, py, boundary, p, ans_grad)
    return p, ans, gx, gy


@pytest.mark.parametrize("dtype", DTYPES)
def test_zero_inputs_give_binomials(dtype):
    S, T = 7, 9
    px = torch.zeros(2, S, T + 1, dtype=dtype)
    py = torch.zeros(2, S + 1, T, dtype=dtype)
    p, ans, gx, gy = _run(px, py)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    for s in range(S + 1):
        for t in range(T + 1):
            assert abs(p[0, s, t].item() - truth.log_binom(s + t, s)) < tol * max(1, s + t)
    assert abs(ans[1].item() - truth.log_binom(S + T, S)) < tol * 20
    # occupancy of the edge (s,t)->(s+1,t): paths through it / all paths
    Z = math.comb(S + T, S)
    for s in range(S):
        for t in range(T + 1):
            want = math.comb(s + t, s) * math.comb(S - s - 1 + T - t, T - t) / Z
            assert abs(gx[0, s, t].item() - want) < 2e-5
    for s in range(S + 1):
        for t in range(T):
            want = math.comb(s + t, s) * math.comb(S - s + T - t - 1, S - s) / Z
            assert abs(gy[0, s, t].item() - want) < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_zero_inputs_modified(dtype):
    S, T = 5, 9
    px = torch.zeros(1, S, T, dtype=dtype)
    py = torch.zeros(1, S + 1, T, dtype=dtype)
    p, ans, gx, gy = _run(px, py)
    for s in range(S + 1):
        for t in range(T + 1):
            want = truth.log_binom(t, s)
            got = p[0, s, t].item()
            if math.isinf(want):
                assert got == -math.inf
            else:
                assert abs(got - want) < 1e-5 * max(1, t)
    # every frame advance is exactly one edge: the flows crossing frame t sum to 1
    total = gx[0].sum(0) + gy[0].sum(0)
    assert torch.allclose(total, torch.ones(T, dtype=dtype), atol=1e-5)


@pytest.mark.parametrize("modified", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_bruteforce_windows(dtype, modified):
    g = torch.Generator().manual_seed(5)
    B, S, T = 6, 4, 6
    px = torch.randn(B, S, T + (0 if modified else 1), generator=g, dtype=dtype)
    py = torch.randn(B, S + 1, T, generator=g, dtype=dtype)
    # offsets, empty symbol / frame sequences, full window, single cell
    boundary = torch.tensor(
        [[0, 0, 4, 6], [1, 2, 3, 6], [2, 1, 2, 5], [0, 3, 3, 3], [4, 6, 4, 6], [1, 0, 4, 4]])
    p, ans, gx, gy = _run(px, py, boundary)
    tol = 2e-5 if dtype == torch.float32 else 1e-12
    for b in range(B):
        s0, t0, s1, t1 = boundary[b].tolist()
        want = truth.enumerate_paths(px[b], py[b], s0, t0, s1, t1, modified)
        got = ans[b].item()
        if math.isinf(want):
            assert got == want
        else:
            assert abs(got - want) < tol
        ref = truth.dp_numpy(px[b].numpy(), py[b].numpy(), s0, t0, s1, t1, modified)
        win = p[b, s0:s1 + 1, t0:t1 + 1].double().numpy()
        refw = ref[s0:s1 + 1, t0:t1 + 1]
        both_inf = np.isinf(win) & np.isinf(refw)
        with np.errstate(invalid="ignore"):
            assert np.all(both_inf | (np.abs(win - refw) < tol))
        # cells outside the window are never written by forward
        mask = torch.ones(S + 1, T + 1, dtype=torch.bool)
        mask[s0:s1 + 1, t0:t1 + 1] = False
        assert torch.isnan(p[b][mask]).all()
        # gradients vanish outside the window
        gmask = torch.ones_like(gy[b], dtype=torch.bool)
        gmask[s0:s1 + 1, t0:t1] = False
        assert (gy[b][gmask] == 0).all()


@pytest.mark.parametrize("modified", [False, True])
def test_gradients_match_autograd_of_independent_dp(modified):
    g = torch.Generator().manual_seed(9)
    B, S, T = 3, 5, 7
    px = torch.randn(B, S, T + (0 if modified else 1), generator=g, dtype=torch.float64)
    py = torch.randn(B, S + 1, T, generator=g, dtype=torch.float64)
    boundary = torch.tensor([[0, 0, 5, 7], [1, 1, 4, 6], [0, 2, 3, 7]])
    w = torch.tensor([0.7, -1.3, 2.0], dtype=torch.float64)
    for bnd in (None, boundary):
        a = px.clone().requires_grad_(True)
        c = py.clone().requires_grad_(True)
        (truth.dp_torch(a, c, bnd, modified) * w).sum().backward()
        _, ans, gx, gy = _run(px, py, bnd, ans_grad=w)
        assert torch.allclose(gx, a.grad, atol=1e-10)
        assert torch.allclose(gy, c.grad, atol=1e-10)
        assert torch.allclose(ans, truth.dp_torch(px, py, bnd, modified), atol=1e-10)


@pytest.mark.parametrize("dtype", DTYPES)
def test_flow_conservation_regular(dtype):
    g = torch.Generator().manual_seed(11)
    B, S, T = 4, 9, 30
    px = torch.randn(B, S, T + 1, generator=g, dtype=dtype)
    py = torch.randn(B, S + 1, T, generator=g, dtype=dtype)
    boundary = torch.tensor([[0, 0, 9, 30], [2, 3, 8, 25], [0, 0, 1, 30], [3, 0, 9, 2]])
    _, _, gx, gy = _run(px, py, boundary)
    for b in range(B):
        s0, t0, s1, t1 = boundary[b].tolist()
        # every path crosses each frame boundary / symbol boundary exactly once
        assert torch.allclose(gy[b, :, t0:t1].sum(0), torch.ones(t1 - t0, dtype=dtype), atol=2e-5)
        assert torch.allclose(gx[b, s0:s1, :].sum(1), torch.ones(s1 - s0, dtype=dtype), atol=2e-5)


def test_finite_differences():
    # the scheme of fast_rnnt/python/tests/mutual_information_test.py:275-305
    g = torch.Generator().manual_seed(13)
    B, S, T = 4, 12, 17
    px = torch.randn(B, S, T + 1, generator=g, dtype=torch.float64)
    py = torch.randn(B, S + 1, T, generator=g, dtype=torch.float64)
    w = torch.randn(B, generator=g, dtype=torch.float64)
    _, ans, gx, gy = _run(px, py, None, ans_grad=w)
    dx = 1e-5 * torch.randn(px.shape, generator=g, dtype=torch.float64)
    dy = 1e-5 * torch.randn(py.shape, generator=g, dtype=torch.float64)
    _, ans2, _, _ = _run(px + dx, py + dy)
    observed = ((ans2 - ans) * w).sum().item()
    predicted = ((dx * gx).sum() + (dy * gy).sum()).item()
    assert abs(observed - predicted) < 1e-3 * abs(predicted) + 1e-9


def test_neg_inf_inputs_do_not_poison():
    # -inf in px blocks that edge; -inf everywhere gives -inf, never nan
    S, T = 3, 4
    px = torch.zeros(1, S, T + 1)
    py = torch.zeros(1, S + 1, T)
    px[0, :, T] = -math.inf
    p, ans, gx, gy = _run(px, py)
    assert torch.isfinite(ans).all()
    assert (gx[0, :, T] == 0).all() and torch.isfinite(gx).all() and torch.isfinite(gy).all()
    px[:] = -math.inf
    py[:] = -math.inf
    p, ans, gx, gy = _run(px, py)
    assert ans[0].item() == -math.inf
    assert not torch.isnan(p).any()
    assert torch.isfinite(gx).all() and torch.isfinite(gy).all()


def test_autograd_wrapper_mutates_returned_grads():
    # fast_rnnt/python/fast_rnnt/mutual_information.py:173-181 scales the saved
    # gradients in place, and those are the tensors handed out by return_grad.
    g = torch.Generator().manual_seed(17)
    px = torch.randn(2, 3, 6, generator=g).requires_grad_(True)
    py = torch.randn(2, 4, 5, generator=g).requires_grad_(True)
    scores, (gx, gy) = recursion.mutual_information_recursion(px, py, None, return_grad=True)
    before = gx.clone()
    (-scores.sum()).backward()
    assert torch.equal(gx, -before)
    assert torch.equal(px.grad, gx)


@pytest.mark.parametrize("modified", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_bit_equal_to_reference_build(dtype, modified):
    ref = ref_build.load()
    if ref is None:
        pytest.skip("oracle/_ref not built (make -C oracle ref)")
    g = torch.Generator().manual_seed(23)
    B, S, T = 7, 19, 45
    px = 3 * torch.randn(B, S, T + (0 if modified else 1), generator=g, dtype=dtype)
    py = 3 * torch.randn(B, S + 1, T, generator=g, dtype=dtype)
    if not modified:
        px[:, :, T] = -math.inf
    boundary = torch.tensor([[0, 0, 19, 45], [1, 2, 10, 30], [3, 3, 3, 3], [0, 5, 19, 5],
                             [2, 0, 2, 45], [0, 0, 19, 44], [5, 7, 19, 45]])
    w = torch.randn(B, generator=g, dtype=dtype)
    for bnd in (None, boundary):
        p1 = torch.zeros(B, S + 1, T + 1, dtype=dtype)
        p2 = torch.zeros(B, S + 1, T + 1, dtype=dtype)
        a1 = recursion.mi_forward(px, py, bnd, p1)
        a2 = ref.mutual_information_forward(px, py, bnd, p2)
        assert torch.equal(a1, a2) and torch.equal(p1, p2)
        g1 = recursion.mi_backward(px, py, bnd, p1, w)
        g2 = ref.mutual_information_backward(px, py, bnd, p2, w.clone())
        assert torch.equal(g1[0], g2[0]) and torch.equal(g1[1], g2[1])


# ---- joint_mutual_information_recursion (mutual_information.py:314-425) ---------------

@pytest.mark.parametrize("modified", [False, True])
def test_joint_recursion_constant_terms_closed_form(modified):
    # term n is a_n on every x-step and b_n on every y-step.  A path of the regular lattice
    # takes S x-steps and T y-steps, so term n's share is S a_n + T b_n and what is left of
    # the total, log C(S+T, S), goes to term 0; a path of the modified lattice takes S
    # diagonal steps and T - S y-steps, and there are C(T, S) of them.
    S, T = 4, 7
    a, b = [0.3, -1.1, 0.25], [-0.7, 0.4, -0.05]
    px = [torch.full((2, S, T if modified else T + 1), v, dtype=torch.float64) for v in a]
    py = [torch.full((2, S + 1, T), v, dtype=torch.float64) for v in b]
    got = recursion.joint_mutual_information_recursion(px, py)
    assert got.shape == (3, 2)
    ny = T - S if modified else T
    paths = truth.log_binom(T, S) if modified else truth.log_binom(S + T, S)
    for n in range(3):
        want = S * a[n] + ny * b[n] + (paths if n == 0 else 0.0)
        assert abs(got[n, 0].item() - want) < 1e-10 and abs(got[n, 1].item() - want) < 1e-10


@pytest.mark.parametrize("dtype", DTYPES)
def test_joint_recursion_one_term_and_halves(dtype):
    # mutual_information_test.py:138-154: one term gives the plain recursion, and the
    # shares of two halves add up to it; with windows, and with blocked cells in px
    g = torch.Generator().manual_seed(21)
    B, S, T = 3, 6, 9
    px = torch.randn(B, S, T + 1, generator=g, dtype=dtype)
    py = torch.randn(B, S + 1, T, generator=g, dtype=dtype)
    px[:, :, T] = -math.inf
    px[1, 2, 3] = -math.inf
    bnd = torch.tensor([[0, 0, S, T], [1, 2, 5, 8], [0, 0, 3, 9]])
    for boundary in (None, bnd):
        plain = recursion.mutual_information_recursion(px, py, boundary)
        one = recursion.joint_mutual_information_recursion((px,), (py,), boundary)
        two = recursion.joint_mutual_information_recursion((px * 0.5, px * 0.5),
                                                           (py * 0.5, py * 0.5), boundary)
        tol = 1e-5 if dtype == torch.float32 else 1e-12
        assert one.shape == (1, B) and two.shape == (2, B)
        assert torch.allclose(one[0], plain, rtol=tol, atol=tol)
        assert torch.allclose(two.sum(0), plain, rtol=tol, atol=tol)
        assert torch.isfinite(two).all()  # -inf * 0 was kept out


def test_joint_recursion_gradients_are_the_occupations():
    # d(sum of shares)/d px[n] is the occupation of the summed lattice for every n:
    # compare with autograd through an independent logaddexp programme on the sums
    g = torch.Generator().manual_seed(22)
    B, S, T = 2, 4, 5
    bnd = torch.tensor([[0, 0, 4, 5], [1, 0, 3, 4]])
    xs = [torch.randn(B, S, T + 1, generator=g, dtype=torch.float64).requires_grad_(True)
          for _ in range(2)]
    ys = [torch.randn(B, S + 1, T, generator=g, dtype=torch.float64).requires_grad_(True)
          for _ in range(2)]
    shares = recursion.joint_mutual_information_recursion(xs, ys, bnd)
    shares.sum().backward()
    ax = (xs[0] + xs[1]).detach().requires_grad_(True)
    ay = (ys[0] + ys[1]).detach().requires_grad_(True)
    total = truth.dp_torch(ax, ay, bnd, modified=False)
    total.sum().backward()
    assert torch.allclose(shares.sum(0).detach(), total.detach(), atol=1e-10)
    for n in range(2):
        assert torch.allclose(xs[n].grad, ax.grad, atol=1e-10)
        assert torch.allclose(ys[n].grad, ay.grad, atol=1e-10)
    # and a single share: weights another term's occupation-weighted sum does not see
    for t in xs + ys:
        t.grad = None
    shares = recursion.joint_mutual_information_recursion(xs, ys, bnd)
    shares[1].sum().backward()
    assert torch.allclose(xs[1].grad, ax.grad, atol=1e-10)
    assert xs[0].grad is None or float(xs[0].grad.abs().max()) == 0.0
