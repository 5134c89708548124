"""Writes the golden vectors under tests/golden/ (run once, in the build container).

Two functions of the reference's Python layer are pinned by nothing but their
own source: ``get_rnnt_prune_ranges`` on real gradients (tie behaviour of the
fp32 window sum + argmax + the double suffix-minimum transform,
fast_rnnt/python/fast_rnnt/rnnt_loss.py:638-777) and
``get_rnnt_logprobs_smoothed`` with non-zero scales (unigram mean over padding
rows, ``tiny`` placement, the 1e-20 substitution, :1135-1369).  For these two
only, this script imports the reference package from /root/reference together
with the reference operator built into oracle/_ref, evaluates them on small
seeded inputs and stores inputs + outputs as ``.pt`` tensors dictionaries
(loaded later with ``torch.load(weights_only=True)``).

Usage:  python tests/golden/make_golden.py
"""
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF_PY = "/root/reference/fast_rnnt/python"


def _import_reference():
    sys.path.insert(0, ROOT)
    from oracle import ref_build

    ref_build.build()
    op = ref_build.load()
    if op is None:
        raise SystemExit("oracle/_ref is not built; run `make -C oracle ref`")
    sys.modules["_fast_rnnt"] = op
    sys.path.insert(0, REF_PY)
    import fast_rnnt  # the reference package

    return fast_rnnt


def _lengths(g, B, S, T, s_lo, t_lo):
    Sb = torch.randint(s_lo, S + 1, (B,), generator=g)
    Tb = torch.randint(t_lo, T + 1, (B,), generator=g)
    z = torch.zeros(B, dtype=torch.int64)
    return torch.stack([z, z, Sb, Tb], dim=1)


def smoothed_cases(ref):
    out = {}
    specs = [
        ("regular", 0.25, 0.0, 4, 50, 10, 50, 1001),
        ("regular", 0.1, 0.1, 3, 17, 6, 11, 11),
        ("modified", 0.2, 0.3, 3, 19, 7, 13, 12),
        ("constrained", 0.0, 0.333, 2, 15, 5, 9, 13),
    ]
    for i, (kind, ls, as_, B, T, S, C, seed) in enumerate(specs):
        g = torch.Generator().manual_seed(seed)
        am = torch.randn(B, T, C, generator=g)
        lm = torch.randn(B, S + 1, C, generator=g)
        sym = torch.randint(1, C, (B, S), generator=g)
        bnd = _lengths(g, B, S, T, max(1, S // 2), S if kind != "regular" else T // 2)
        px, py = ref.get_rnnt_logprobs_smoothed(
            lm=lm, am=am, symbols=sym, termination_symbol=0, lm_only_scale=ls,
            am_only_scale=as_, boundary=bnd, rnnt_type=kind)
        loss = ref.rnnt_loss_smoothed(
            lm=lm, am=am, symbols=sym, termination_symbol=0, lm_only_scale=ls,
            am_only_scale=as_, boundary=bnd, rnnt_type=kind, reduction="none")
        out[f"case{i}"] = dict(
            kind=kind, lm_only_scale=ls, am_only_scale=as_, am=am, lm=lm, symbols=sym,
            boundary=bnd, px=px, py=py, loss=loss)
    return out


def prune_cases(ref):
    out = {}
    specs = [
        ("regular", 5, 4, 50, 10, 50, 1001),
        ("regular", 3, 3, 40, 12, 20, 21),
        ("regular", 2, 2, 9, 20, 8, 22),   # s_range raised to s_range_min
        ("regular", 30, 2, 12, 4, 8, 23),  # s_range > S  ->  S + 1
        ("modified", 3, 3, 30, 9, 16, 24),
        ("constrained", 4, 2, 25, 8, 12, 25),
    ]
    for i, (kind, R, B, T, S, C, seed) in enumerate(specs):
        g = torch.Generator().manual_seed(seed)
        am = torch.randn(B, T, C, generator=g)
        lm = torch.randn(B, S + 1, C, generator=g)
        sym = torch.randint(1, C, (B, S), generator=g)
        bnd = _lengths(g, B, S, T, max(1, S // 2), S if kind != "regular" else max(1, T // 2))
        _, (gx, gy) = ref.rnnt_loss_simple(
            lm=lm, am=am, symbols=sym, termination_symbol=0, boundary=bnd,
            rnnt_type=kind, reduction="sum", return_grad=True)
        ranges = ref.get_rnnt_prune_ranges(px_grad=gx, py_grad=gy, boundary=bnd, s_range=R)
        am_p, lm_p = ref.do_rnnt_pruning(am=am, lm=lm, ranges=ranges)
        logits = torch.tanh(am_p + lm_p)
        px, py = ref.get_rnnt_logprobs_pruned(
            logits=logits, symbols=sym, ranges=ranges, termination_symbol=0,
            boundary=bnd, rnnt_type=kind)
        out[f"case{i}"] = dict(
            kind=kind, s_range=R, px_grad=gx.detach().clone(), py_grad=gy.detach().clone(),
            boundary=bnd, ranges=ranges, symbols=sym)
        if i > 0:  # the pruned log-probs of the larger case 0 would be 200 KB
            out[f"case{i}"].update(logits=logits, px=px, py=py)
    # a hand-made tie case: equal scores must resolve to the first maximum
    B, S, T = 1, 4, 6
    gy = torch.full((B, S + 1, T), 0.25)
    gx = torch.zeros(B, S, T + 1)
    bnd = torch.tensor([[0, 0, S, T]])
    out["ties"] = dict(kind="regular", s_range=2, px_grad=gx, py_grad=gy, boundary=bnd,
                       ranges=ref.get_rnnt_prune_ranges(gx, gy, bnd, 2))
    return out


def main():
    ref = _import_reference()
    torch.save(smoothed_cases(ref), os.path.join(HERE, "smoothed_logprobs.pt"))
    torch.save(prune_cases(ref), os.path.join(HERE, "prune_ranges.pt"))
    for name in ("smoothed_logprobs.pt", "prune_ranges.pt"):
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
