"""Pins the torch-CPU restatement of the loss layer (oracle/losses.py).

Sources of truth: brute-force alignment enumeration, log_softmax + an
independent dynamic programme, the docstring vectors the reference holds
(rnnt_loss.py:557-570, :829-840), cross-formulation identities and invariances
(the reference's own test strategy, fast_rnnt/python/tests/rnnt_loss_test.py),
and the golden vectors under tests/golden/ for the two functions nothing else
pins (smoothed log-probs with non-zero scales, prune ranges).
"""
import math
import os

import pytest
import torch

import lattice_truth as truth
from oracle import losses

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KINDS = ["regular", "modified", "constrained"]


def _tiny_fixture():
    # fast_rnnt/python/tests/rnnt_loss_test.py:70-82
    lm = torch.tensor([[[0, 0, 1], [0, 1, 1], [1, 0, 1], [2, 2, 0]]], dtype=torch.float)
    am = torch.tensor([[[0, 1, 2], [0, 0, 0], [0, 2, 4], [0, 3, 3]]], dtype=torch.float)
    sym = torch.tensor([[0, 1, 0]])
    return lm, am, sym, 2


def test_tiny_fixture_against_bruteforce():
    lm, am, sym, blank = _tiny_fixture()
    logits = am.unsqueeze(2) + lm.unsqueeze(1)  # [B,T,S+1,C]
    lsm = torch.log_softmax(logits.double(), dim=3)[0]
    want = truth.transducer_nll_bruteforce(lsm.numpy(), sym[0].tolist(), blank)
    assert abs(want - 7.5040133560) < 1e-8
    for got in (
        losses.loss_simple(lm, am, sym, blank, reduction="none"),
        losses.loss_smoothed(lm, am, sym, blank, 0.0, 0.0, reduction="none"),
        losses.loss_joint(logits, sym, blank, reduction="none"),
    ):
        assert abs(got.item() - want) < 2e-6


def _random_case(seed, B, S, T, C, dtype=torch.float64, with_boundary=True, modified=False):
    g = torch.Generator().manual_seed(seed)
    am = torch.randn(B, T, C, generator=g, dtype=dtype)
    lm = torch.randn(B, S + 1, C, generator=g, dtype=dtype)
    sym = torch.randint(0, C - 1, (B, S), generator=g)
    bnd = None
    if with_boundary:
        Sb = torch.randint(1, S + 1, (B,), generator=g)
        lo = S if modified else 1
        Tb = torch.randint(lo, T + 1, (B,), generator=g)
        z = torch.zeros(B, dtype=torch.int64)
        bnd = torch.stack([z, z, Sb, Tb], 1)
    return am, lm, sym, bnd


def _textbook_nll(am, lm, sym, blank, bnd, kind):
    """log_softmax of the additive joiner + the independent numpy lattice DP."""
    B, T, C = am.shape
    S = lm.shape[1] - 1
    lsm = torch.log_softmax((am.unsqueeze(2) + lm.unsqueeze(1)).double(), dim=3)
    out = []
    for b in range(B):
        Sb, Tb = (S, T) if bnd is None else (int(bnd[b, 2]), int(bnd[b, 3]))
        modified = kind != "regular"
        px = torch.full((S, T + (0 if modified else 1)), -math.inf, dtype=torch.float64)
        py = lsm[b, :, :, blank].t().clone()  # [S+1,T]
        for s in range(S):
            px[s, :T] = lsm[b, :, s, sym[b, s]]
            if kind == "constrained":
                px[s, :T] += py[s + 1, :]
        if not modified:
            px[:, Tb] = -math.inf
        p = truth.dp_numpy(px.numpy(), py.numpy(), 0, 0, Sb, Tb, modified)
        out.append(-p[Sb, Tb])
    return torch.tensor(out, dtype=torch.float64)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("with_boundary", [False, True])
def test_simple_and_joint_match_textbook(kind, with_boundary):
    am, lm, sym, bnd = _random_case(3, 4, 6, 11, 7, with_boundary=with_boundary,
                                    modified=kind != "regular")
    want = _textbook_nll(am, lm, sym, 6, bnd, kind)
    got_simple = losses.loss_simple(lm, am, sym, 6, boundary=bnd, rnnt_type=kind, reduction="none")
    logits = am.unsqueeze(2) + lm.unsqueeze(1)
    got_joint = losses.loss_joint(logits, sym, 6, boundary=bnd, rnnt_type=kind, reduction="none")
    got_smooth = losses.loss_smoothed(lm, am, sym, 6, 0.0, 0.0, boundary=bnd, rnnt_type=kind,
                                      reduction="none")
    assert torch.allclose(got_simple, want, atol=1e-9)
    assert torch.allclose(got_joint, want, atol=1e-9)
    assert torch.allclose(got_smooth, want, atol=1e-9)


@pytest.mark.parametrize("kind", KINDS)
def test_invariance_to_per_frame_constants(kind):
    # fast_rnnt/python/tests/rnnt_loss_test.py:155-189, :287-321
    am, lm, sym, bnd = _random_case(4, 3, 5, 9, 8, modified=kind != "regular")
    g = torch.Generator().manual_seed(99)
    a = losses.loss_smoothed(lm, am, sym, 7, 0.2, 0.333, boundary=bnd, rnnt_type=kind,
                             reduction="none")
    lm2 = lm + torch.randn(3, 6, 1, generator=g, dtype=lm.dtype)
    am2 = am + torch.randn(3, 9, 1, generator=g, dtype=am.dtype)
    b = losses.loss_smoothed(lm2, am2, sym, 7, 0.2, 0.333, boundary=bnd, rnnt_type=kind,
                             reduction="none")
    assert torch.allclose(a, b, atol=1e-9)
    c = losses.loss_simple(lm, am, sym, 7, boundary=bnd, rnnt_type=kind, reduction="none")
    d = losses.loss_simple(lm2, am2, sym, 7, boundary=bnd, rnnt_type=kind, reduction="none")
    assert torch.allclose(c, d, atol=1e-9)


def test_reductions_and_errors():
    am, lm, sym, bnd = _random_case(5, 3, 4, 8, 6)
    none = losses.loss_simple(lm, am, sym, 5, boundary=bnd, reduction="none")
    assert torch.allclose(losses.loss_simple(lm, am, sym, 5, boundary=bnd, reduction="sum"), none.sum())
    assert torch.allclose(losses.loss_simple(lm, am, sym, 5, boundary=bnd, reduction="mean"), none.mean())
    with pytest.raises(ValueError):
        losses.loss_simple(lm, am, sym, 5, boundary=bnd, reduction="bogus")


def test_delay_penalty_definition():
    am, lm, sym, bnd = _random_case(6, 2, 4, 9, 6)
    lam = 0.01
    px, py = losses.lattice_logprobs_simple(lm, am, sym, 5, boundary=bnd)
    t = torch.arange(px.shape[2], dtype=torch.float64).reshape(1, 1, -1)
    px2 = px + ((bnd[:, 3].double() - 1) / 2).reshape(-1, 1, 1) * lam - t * lam
    want = -losses.mutual_information_recursion(px2, py, bnd)
    got = losses.loss_simple(lm, am, sym, 5, boundary=bnd, delay_penalty=lam, reduction="none")
    assert torch.allclose(got, want, atol=1e-5)  # the penalty itself is formed in float32


def test_docstring_vectors():
    x = torch.tensor([0, 2, 1, 3, 6, 5, 8], dtype=torch.int32)
    assert losses.monotonic_lower_bound(x).tolist() == [0, 1, 1, 3, 5, 5, 8]
    x = torch.tensor([[12, 18, 5, 4, 18, 17], [11, 14, 14, 3, 10, 4], [19, 3, 8, 13, 7, 19]],
                     dtype=torch.int32)
    assert losses.monotonic_lower_bound(x).tolist() == [
        [4, 4, 4, 4, 17, 17], [3, 3, 3, 3, 4, 4], [3, 3, 7, 7, 7, 19]]
    src = torch.arange(15).reshape(1, 3, 5)
    got = losses.roll_rows(src, torch.tensor([[1, 2, 3]]))
    assert got.tolist() == [[[4, 0, 1, 2, 3], [8, 9, 5, 6, 7], [12, 13, 14, 10, 11]]]


@pytest.mark.parametrize("kind", KINDS)
def test_pruned_with_full_range_equals_joint(kind):
    am, lm, sym, bnd = _random_case(7, 3, 5, 9, 6, modified=kind != "regular")
    B, T, C = am.shape
    S = sym.shape[1]
    logits = torch.tanh(am.unsqueeze(2) + lm.unsqueeze(1))
    ranges = torch.arange(S + 1).reshape(1, 1, S + 1).expand(B, T, S + 1).contiguous()
    a = losses.loss_pruned(logits, sym, ranges, 5, boundary=bnd, rnnt_type=kind, reduction="none")
    b = losses.loss_joint(logits, sym, 5, boundary=bnd, rnnt_type=kind, reduction="none")
    assert torch.allclose(a, b, atol=1e-10)


def test_pruned_logprobs_dense_mask_definition():
    am, lm, sym, bnd = _random_case(8, 2, 7, 10, 6)
    B, T, C = am.shape
    S, R = 7, 3
    g = torch.Generator().manual_seed(1)
    r0 = torch.randint(0, S + 2 - R, (B, T), generator=g)
    ranges = r0.unsqueeze(2) + torch.arange(R)
    am_p, lm_p = losses.prune(am, lm, ranges)
    for b in range(B):
        for t in range(T):
            for j in range(R):
                assert torch.equal(lm_p[b, t, j], lm[b, ranges[b, t, j]])
                assert torch.equal(am_p[b, t, j], am[b, t])
    logits = am_p + lm_p
    px, py = losses.lattice_logprobs_pruned(logits, sym, ranges, 5, boundary=None)
    lsm = torch.log_softmax(logits, dim=3)
    for b in range(B):
        for t in range(T):
            for s in range(S + 1):
                j = s - int(r0[b, t])
                inside = 0 <= j < R
                want_y = lsm[b, t, j, 5].item() if inside else -math.inf
                assert abs(py[b, s, t].item() - want_y) < 1e-12 or py[b, s, t].item() == want_y
                if s < S:
                    want_x = lsm[b, t, j, sym[b, s]].item() if inside else -math.inf
                    assert abs(px[b, s, t].item() - want_x) < 1e-12 or px[b, s, t].item() == want_x
    assert (px[:, :, T] == -math.inf).all()


@pytest.mark.parametrize("kind", ["regular", "modified"])
def test_prune_ranges_invariants(kind):
    am, lm, sym, bnd = _random_case(10, 4, 12, 30, 9, dtype=torch.float32, modified=kind != "regular")
    _, (gx, gy) = losses.loss_simple(lm, am, sym, 8, boundary=bnd, rnnt_type=kind,
                                     reduction="sum", return_grad=True)
    for R in (2, 3, 5, 13, 40):
        ranges = losses.prune_ranges(gx, gy, bnd, R)
        B, T, RR = ranges.shape
        r0 = ranges[:, :, 0]
        assert (r0[:, 0] == 0).all()
        step = r0[:, 1:] - r0[:, :-1]
        assert (step >= 0).all()
        assert (step < (RR if kind == "regular" else 2)).all() or RR == 13
        assert (ranges >= 0).all() and (ranges <= 12).all()
        assert torch.equal(ranges, r0.unsqueeze(2) + torch.arange(RR))
        # the last real frame keeps the final symbol position inside the window
        for b in range(B):
            Sb, Tb = int(bnd[b, 2]), int(bnd[b, 3])
            assert r0[b, Tb - 1] <= Sb <= r0[b, Tb - 1] + RR - 1


def test_golden_smoothed_logprobs():
    data = torch.load(os.path.join(GOLDEN, "smoothed_logprobs.pt"), weights_only=True)
    assert len(data) == 4
    for name, c in data.items():
        px, py = losses.lattice_logprobs_smoothed(
            c["lm"], c["am"], c["symbols"], 0, c["lm_only_scale"], c["am_only_scale"],
            boundary=c["boundary"], rnnt_type=c["kind"])
        # (bit for bit on the host that wrote the vectors; torch's matmul and logsumexp add in
        # an order that depends on the host's thread count, hence the last-bit tolerance)
        assert torch.allclose(px, c["px"], rtol=2e-6, atol=2e-6), name
        assert torch.allclose(py, c["py"], rtol=2e-6, atol=2e-6), name
        loss = losses.loss_smoothed(
            c["lm"], c["am"], c["symbols"], 0, c["lm_only_scale"], c["am_only_scale"],
            boundary=c["boundary"], rnnt_type=c["kind"], reduction="none")
        assert torch.allclose(loss, c["loss"], rtol=2e-6, atol=0), name


def test_golden_prune_ranges(capsys):
    data = torch.load(os.path.join(GOLDEN, "prune_ranges.pt"), weights_only=True)
    assert len(data) == 7
    for name, c in data.items():
        got = losses.prune_ranges(c["px_grad"], c["py_grad"], c["boundary"], c["s_range"])
        assert got.dtype == torch.int64
        assert torch.equal(got, c["ranges"]), name
        ltr = losses.prune_ranges(c["px_grad"], c["py_grad"], c["boundary"], c["s_range"],
                                  window_sum="ltr")
        assert torch.equal(ltr, c["ranges"]), name
        if "logits" in c:
            px, py = losses.lattice_logprobs_pruned(
                c["logits"], c["symbols"], c["ranges"], 0, boundary=c["boundary"],
                rnnt_type=c["kind"])
            # (last-bit tolerance: logsumexp's summation order follows the host's threads)
            assert torch.allclose(px, c["px"], rtol=2e-6, atol=2e-6), name
            assert torch.allclose(py, c["py"], rtol=2e-6, atol=2e-6), name
    assert "Adjusting to 4" in capsys.readouterr().out
    assert data["ties"]["ranges"][0, :, 0].tolist()[0] == 0


def _occupancies(seed, B, S, T, C, dtype):
    g = torch.Generator().manual_seed(seed)
    am = torch.randn(B, T, C, generator=g, dtype=dtype)
    lm = torch.randn(B, S + 1, C, generator=g, dtype=dtype)
    sym = torch.randint(1, C, (B, S), generator=g)
    # short targets in a tall lattice: a wide window covers the whole band that holds the
    # alignment's mass, so neighbouring window starts tie up to rounding
    Sb = torch.randint(S // 4, S // 2, (B,), generator=g)
    Tb = torch.randint(T // 2, T + 1, (B,), generator=g)
    z = torch.zeros(B, dtype=torch.int64)
    bnd = torch.stack([z, z, Sb, Tb], 1)
    _, (gx, gy) = losses.loss_simple(lm, am, sym, 0, boundary=bnd, reduction="sum",
                                     return_grad=True)
    return gx, gy, bnd


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_window_sums_follow_torch_cpu_order(dtype):
    """The restatement of torch.sum's order over the window axis (what decides near-ties
    between window starts once s_range exceeds 16) against torch.sum itself, on one thread
    and with frame counts that fill whole SIMD vectors, where torch.sum has no differently
    summed tail; and the prune ranges that follow from either."""
    threads = torch.get_num_threads()
    torch.set_num_threads(1)
    try:
        for n_case, (B, S, T, R) in enumerate([(2, 30, 64, 5), (2, 30, 64, 16), (2, 30, 64, 17),
                                               (3, 69, 128, 19), (2, 80, 64, 33), (1, 300, 64, 70),
                                               (1, 700, 64, 300), (1, 600, 64, 513),
                                               (1, 5000, 64, 4500)]):
            g = torch.Generator().manual_seed(n_case)
            py = torch.rand(B, S + 1, T, generator=g, dtype=dtype) ** 3
            n = S + 2 - R
            sb, ss, st = py.stride()
            want = torch.sum(torch.as_strided(py, (B, n, R, T), (sb, ss, ss, st)), axis=2)
            got = losses.window_sums_in_torch_cpu_order(py, n, R)
            assert torch.equal(got, want), (B, S, T, R)
            if R <= 16:
                ltr = py[:, 0:n, :].clone()
                for j in range(1, R):
                    ltr = ltr + py[:, j:j + n, :]
                assert torch.equal(got, ltr)
        for seed, (B, S, T) in enumerate([(3, 69, 128), (2, 100, 64)]):
            gx, gy, bnd = _occupancies(40 + seed, B, S, T, 12, dtype)
            for R in (17, 19, 33, 40):
                a = losses.prune_ranges(gx, gy, bnd, R)
                b = losses.prune_ranges(gx, gy, bnd, R, window_sum="cascade")
                assert torch.equal(a, b), (B, S, T, R)
    finally:
        torch.set_num_threads(threads)
