"""The compiled operator module (fast_rnnt_amd._C, csrc/torch_ops.cpp) on the GPU: the
reference's ``_fast_rnnt`` call patterns, the dispatcher registration, and where a bad
boundary row is reported.  Oracle: oracle/ (CPU restatement of the reference)."""
import pytest
import torch

import _fast_rnnt
import fast_rnnt_amd
from oracle import losses as O
from oracle import recursion as oracle_rec

pytestmark = pytest.mark.gpu


def _lattice(seed, B, S, T, modified=False, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    px = torch.randn(B, S, T if modified else T + 1, generator=g, dtype=dtype)
    py = torch.randn(B, S + 1, T, generator=g, dtype=dtype)
    return px, py


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_strided_inputs_and_expanded_boundary(gpu_device, dtype):
    # fast_rnnt/python/tests/mutual_information_test.py:91-96: one boundary row expanded over
    # the batch (stride 0); the operator honours arbitrary strides
    # (mutual_information_cpu.cu:81-88 use accessors).  px / py / p here are transposed or
    # sliced views of larger tensors.
    B, S, T = 3, 7, 12
    px, py = _lattice(11, B, S, T, dtype=dtype)
    row = torch.tensor([1, 2, 6, 11])
    bnd_cpu = row.unsqueeze(0).expand(B, 4)
    want_p = torch.zeros(B, S + 1, T + 1, dtype=dtype)
    want = oracle_rec.mi_forward(px, py, bnd_cpu.contiguous(), want_p)
    ones = torch.ones(B, dtype=dtype)
    wx, wy = oracle_rec.mi_backward(px, py, bnd_cpu.contiguous(), want_p, ones)

    dev = gpu_device
    # px: a transposed view ([B][T+1][S] storage); py: every second row of a taller tensor
    px_store = px.transpose(1, 2).contiguous().to(dev)
    dpx = px_store.transpose(1, 2)
    py_store = torch.zeros(B, 2 * (S + 1), T, dtype=dtype)
    py_store[:, ::2] = py
    dpy = py_store.to(dev)[:, ::2]
    assert not dpx.is_contiguous() and not dpy.is_contiguous()
    bnd = row.to(dev).unsqueeze(0).expand(B, 4)
    assert bnd.stride(0) == 0
    # p: a slice of a wider tensor (row pitch T + 4)
    p_store = torch.full((B, S + 1, T + 4), float("nan"), dtype=dtype, device=dev)
    dp = p_store[:, :, : T + 1]
    assert not dp.is_contiguous()

    ans = _fast_rnnt.mutual_information_forward(dpx, dpy, bnd, dp)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    assert torch.allclose(ans.cpu(), want, rtol=tol, atol=tol)
    window = (slice(None), slice(1, 7), slice(2, 12))
    assert torch.allclose(dp.cpu()[window], want_p[window], rtol=tol, atol=10 * tol)
    # what lies past the slice is untouched
    assert torch.isnan(p_store[:, :, T + 1:]).all()

    ans_grad = torch.ones(B, dtype=dtype, device=dev)
    gx, gy = _fast_rnnt.mutual_information_backward(px=dpx, py=dpy, boundary=bnd, p=dp,
                                                    ans_grad=ans_grad)
    assert torch.allclose(gx.cpu(), wx, atol=1e-5 if dtype == torch.float32 else 1e-12)
    assert torch.allclose(gy.cpu(), wy, atol=1e-5 if dtype == torch.float32 else 1e-12)
    # the gradient that reaches the start of each lattice equals the one fed in
    assert torch.allclose(ans_grad.cpu(), ones, atol=1e-4)


def test_dispatcher_ops_are_the_same_functions(gpu_device):
    B, S, T = 2, 5, 9
    px, py = _lattice(12, B, S, T)
    dpx, dpy = px.to(gpu_device), py.to(gpu_device)
    p1 = torch.empty(B, S + 1, T + 1, device=gpu_device)
    p2 = torch.empty_like(p1)
    a1 = _fast_rnnt.mutual_information_forward(dpx, dpy, None, p1)
    a2 = torch.ops.fast_rnnt_amd.mutual_information_forward(dpx, dpy, None, p2)
    assert torch.equal(a1, a2) and torch.equal(p1, p2)
    g1 = _fast_rnnt.mutual_information_backward(dpx, dpy, None, p1, torch.ones(B, device=gpu_device))
    g2 = torch.ops.fast_rnnt_amd.mutual_information_backward(dpx, dpy, None, p2,
                                                             torch.ones(B, device=gpu_device))
    assert torch.equal(g1[0], g2[0]) and torch.equal(g1[1], g2[1])

    # the loss op through the dispatcher, with autograd, against the package function
    g = torch.Generator().manual_seed(13)
    C = 17
    am = torch.randn(B, T, C, generator=g)
    lm = torch.randn(B, S + 1, C, generator=g)
    sym = torch.randint(1, C, (B, S), generator=g).to(gpu_device)
    bnd = torch.tensor([[0, 0, S, T], [0, 0, S - 2, T - 3]]).to(gpu_device)
    a1_, l1_ = am.to(gpu_device).requires_grad_(True), lm.to(gpu_device).requires_grad_(True)
    a2_, l2_ = am.to(gpu_device).requires_grad_(True), lm.to(gpu_device).requires_grad_(True)
    loss1, (x1, y1) = fast_rnnt_amd.rnnt_loss_simple(l1_, a1_, sym, 0, boundary=bnd,
                                                    reduction="sum", return_grad=True)
    loss2, x2, y2 = torch.ops.fast_rnnt_amd.simple_loss(l2_, a2_, sym, bnd, 0, 0, 0.0, True, 2, 1)
    assert torch.equal(loss1, loss2) and torch.equal(x1, x2) and torch.equal(y1, y2)
    loss1.backward()
    loss2.backward()
    assert torch.equal(a1_.grad, a2_.grad) and torch.equal(l1_.grad, l2_.grad)
    # under no_grad nothing is saved and no gradient tensors are made unless asked for
    with torch.no_grad():
        loss3, x3, y3 = torch.ops.fast_rnnt_amd.simple_loss(l2_, a2_, sym, bnd, 0, 0, 0.0, False,
                                                            2, 1)
    assert torch.equal(loss3, loss2.detach()) and x3 is None and y3 is None


def _simple_inputs(dev, B=4, S=6, T=10, C=13, seed=21):
    g = torch.Generator().manual_seed(seed)
    am = torch.randn(B, T, C, generator=g)
    lm = torch.randn(B, S + 1, C, generator=g)
    sym = torch.randint(1, C, (B, S), generator=g)
    return am, lm, sym


@pytest.mark.parametrize("case", ["window", "no_symbols", "few_frames"])
def test_bad_boundary_rows_found_on_the_device(gpu_device, case):
    # rnnt_loss.py:25-42 and mutual_information.py:277-288 assert the rows on the host; here
    # the kernel tests them, the bad row's loss is nan, the others are what they are without
    # the bad row, and the AssertionError comes when the host next looks
    dev = gpu_device
    B, S, T = 4, 6, 10
    am, lm, sym = _simple_inputs(dev, B, S, T)
    good = torch.tensor([[0, 0, S, T], [0, 0, 4, 8], [0, 0, 5, 9], [0, 0, 3, 10]])
    bad = good.clone()
    kind = "regular"
    if case == "window":
        bad[2] = torch.tensor([0, 0, S + 1, T])
    elif case == "no_symbols":
        bad[2] = torch.tensor([0, 0, 0, 9])
    else:
        kind = "modified"
        bad[2] = torch.tensor([0, 0, 5, 4])
    want = O.loss_simple(lm, am, sym, 0, boundary=good, rnnt_type=kind, reduction="none")
    fast_rnnt_amd.check_boundaries()          # nothing pending from earlier tests
    a = am.to(dev).requires_grad_(True)
    l = lm.to(dev).requires_grad_(True)
    got = fast_rnnt_amd.rnnt_loss_simple(l, a, sym.to(dev), 0, boundary=bad.to(dev),
                                         rnnt_type=kind, reduction="none")
    got.nan_to_num(0.0).sum().backward()
    with pytest.raises(AssertionError, match="boundary row 2"):
        fast_rnnt_amd.check_boundaries()
    fast_rnnt_amd.check_boundaries()          # raised once, then cleared
    keep = [0, 1, 3]
    assert torch.isnan(got[2])
    assert torch.allclose(got[keep].detach().cpu(), want[keep], rtol=1e-5)
    assert torch.isfinite(a.grad).all() and torch.isfinite(l.grad).all()

    # without an explicit look, the next call on the GPU raises it
    fast_rnnt_amd.rnnt_loss_simple(l, a, sym.to(dev), 0, boundary=bad.to(dev), rnnt_type=kind)
    torch.cuda.synchronize()
    with pytest.raises(AssertionError, match="earlier call"):
        fast_rnnt_amd.rnnt_loss_simple(l, a, sym.to(dev), 0, boundary=good.to(dev), rnnt_type=kind)
    fast_rnnt_amd.check_boundaries()

    # "host": the reference's timing -- raised before anything runs
    fast_rnnt_amd.set_boundary_checks("host")
    try:
        with pytest.raises(AssertionError):
            fast_rnnt_amd.rnnt_loss_simple(l, a, sym.to(dev), 0, boundary=bad.to(dev),
                                           rnnt_type=kind)
    finally:
        fast_rnnt_amd.set_boundary_checks("device")
    fast_rnnt_amd.check_boundaries()


def test_other_losses_report_bad_rows_too(gpu_device):
    dev = gpu_device
    B, S, T, C = 3, 5, 8, 11
    g = torch.Generator().manual_seed(31)
    logits = torch.randn(B, T, S + 1, C, generator=g).to(dev)
    sym = torch.randint(1, C, (B, S), generator=g).to(dev)
    bad = torch.tensor([[0, 0, S, T], [0, 3, 4, 2], [0, 0, 5, 8]]).to(dev)   # t_begin > t_end
    fast_rnnt_amd.check_boundaries()
    loss = fast_rnnt_amd.rnnt_loss(logits, sym, 0, boundary=bad, reduction="none")
    with pytest.raises(AssertionError, match="boundary row 1"):
        fast_rnnt_amd.check_boundaries()
    assert torch.isnan(loss[1]) and torch.isfinite(loss[[0, 2]]).all()
    am, lm, sym2 = _simple_inputs(dev, B, S, T, C)
    loss = fast_rnnt_amd.rnnt_loss_smoothed(lm.to(dev), am.to(dev), sym2.to(dev), 0, boundary=bad,
                                            reduction="none")
    with pytest.raises(AssertionError, match="boundary row 1"):
        fast_rnnt_amd.check_boundaries()
    assert torch.isnan(loss[1]) and torch.isfinite(loss[[0, 2]]).all()
