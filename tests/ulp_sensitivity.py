"""How far the float32 CPU reference's own occupation gradients move when its inputs
change in their last bit.

The lattice scores ``p`` grow to thousands (|p| ~ 3000 at the 250-frame workloads, ~4500 at
the 400-frame one), where one float32 ulp is 2.4e-4 .. 4.9e-4, and the gradients are
``exp`` of differences of ``p``.  Two pipelines that agree on px / py only to rounding (any
two GEMM summation orders do) therefore cannot agree on the gradients better than what this
module measures ON THE ORACLE ALONE: px / py are nudged by -1, 0 or +1 ulp per element and
the float32 oracle recursion (mutual_information_cpu.cu:89-121, :179-252 restated in C) is
run again.  The GPU tests take their px_grad / py_grad bound from this number where it
exceeds the 1e-4 of the acceptance criterion.
"""
import torch

from oracle import recursion as oracle


def nudge(x: torch.Tensor, g: torch.Generator) -> torch.Tensor:
    """Every finite float32 element moved by -1, 0 or +1 ulp (uniformly)."""
    assert x.dtype == torch.float32
    step = torch.randint(-1, 2, x.shape, generator=g, dtype=torch.int32)
    sign = torch.where(x < 0, -1, 1).to(torch.int32)
    out = (x.contiguous().view(torch.int32) + step * sign).view(torch.float32)
    return torch.where(torch.isfinite(x) & torch.isfinite(out), out, x)


def occupation_grads(px, py, boundary):
    B, S, _ = px.shape
    T = py.shape[2]
    p = torch.empty(B, S + 1, T + 1, dtype=px.dtype)
    oracle.mi_forward(px, py, boundary, p)
    return oracle.mi_backward(px, py, boundary, p, torch.ones(B, dtype=px.dtype))


def reference_sensitivity(px, py, boundary, trials: int = 4, seed: int = 5) -> float:
    """max |px_grad' - px_grad|, |py_grad' - py_grad| of the float32 oracle over `trials`
    random one-ulp nudges of (px, py)."""
    gx, gy = occupation_grads(px, py, boundary)
    g = torch.Generator().manual_seed(seed)
    worst = 0.0
    for _ in range(trials):
        gx2, gy2 = occupation_grads(nudge(px, g), nudge(py, g), boundary)
        worst = max(worst, (gx2 - gx).abs().max().item(), (gy2 - gy).abs().max().item())
    return worst


def grad_bound(px, py, boundary, floor: float = 1e-4, slack: float = 1.25) -> float:
    """The px_grad / py_grad bound a float32 parity test may use on these inputs: the
    acceptance criterion's 1e-4 while one ulp moves the reference by no more than that,
    `slack` times the movement otherwise."""
    moved = reference_sensitivity(px, py, boundary)
    return floor if moved <= floor else slack * moved
