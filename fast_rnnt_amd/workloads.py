"""Seeded synthetic workloads c1..c5 used by the benchmark and the parity tests.

Inputs are generated on the CPU with ``torch.Generator().manual_seed(seed)`` so
that the CPU baseline and the GPU path see identical bits; the caller moves them
to the device.
"""
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class Workload:
    name: str
    kind: str            # "simple" | "pruned" | "joint"
    B: int
    T: int
    S: int
    C: int
    seed: int
    am: Optional[torch.Tensor] = None       # [B,T,C]
    lm: Optional[torch.Tensor] = None       # [B,S+1,C]
    logits: Optional[torch.Tensor] = None   # [B,T,S+1,C] (joint only)
    symbols: Optional[torch.Tensor] = None  # [B,S] int64 in [1,C)
    boundary: Optional[torch.Tensor] = None  # [B,4] int64
    joiner: Optional[torch.Tensor] = None   # [C,C] (pruned only)
    s_range: int = 0
    termination_symbol: int = 0


def _ragged_boundary(g, B, S, T):
    """T_b, S_b uniform in [0.6, 1.0] x max, S_b <= T_b, both >= 1."""
    Tb = torch.round(T * (0.6 + 0.4 * torch.rand(B, generator=g))).long().clamp(min=1)
    Sb = torch.round(S * (0.6 + 0.4 * torch.rand(B, generator=g))).long()
    Sb = torch.minimum(Sb, Tb).clamp(min=1)
    z = torch.zeros(B, dtype=torch.int64)
    return torch.stack([z, z, Sb, Tb], dim=1)


def make(name: str) -> Workload:
    if name == "c1":
        w = Workload("c1", "simple", B=4, T=50, S=10, C=50, seed=1001)
        g = torch.Generator().manual_seed(w.seed)
        w.am = torch.randn(w.B, w.T, w.C, generator=g)
        w.lm = torch.randn(w.B, w.S + 1, w.C, generator=g)
        w.symbols = torch.randint(1, w.C, (w.B, w.S), generator=g)
        Sb = torch.randint(5, 11, (w.B,), generator=g)
        Tb = torch.randint(30, 51, (w.B,), generator=g)
        z = torch.zeros(w.B, dtype=torch.int64)
        w.boundary = torch.stack([z, z, Sb, Tb], dim=1)
        return w
    if name in ("c2", "c3"):
        w = Workload(name, "simple" if name == "c2" else "pruned", B=32, T=250, S=80, C=500,
                     seed=1002 if name == "c2" else 1003)
        g = torch.Generator().manual_seed(w.seed)
        w.am = 2.0 * torch.randn(w.B, w.T, w.C, generator=g)
        w.lm = 2.0 * torch.randn(w.B, w.S + 1, w.C, generator=g)
        w.symbols = torch.randint(1, w.C, (w.B, w.S), generator=g)
        w.boundary = _ragged_boundary(g, w.B, w.S, w.T)
        if name == "c3":
            w.s_range = 5
            w.joiner = torch.randn(w.C, w.C, generator=g) / (w.C ** 0.5)
        return w
    if name == "c4":
        w = Workload("c4", "simple", B=16, T=400, S=120, C=5000, seed=1004)
        g = torch.Generator().manual_seed(w.seed)
        w.am = torch.randn(w.B, w.T, w.C, generator=g)
        w.lm = torch.randn(w.B, w.S + 1, w.C, generator=g)
        w.symbols = torch.randint(1, w.C, (w.B, w.S), generator=g)
        w.boundary = _ragged_boundary(g, w.B, w.S, w.T)
        return w
    if name == "c5":
        w = Workload("c5", "joint", B=8, T=200, S=60, C=1000, seed=1005)
        g = torch.Generator().manual_seed(w.seed)
        w.logits = torch.randn(w.B, w.T, w.S + 1, w.C, generator=g)
        w.symbols = torch.randint(1, w.C, (w.B, w.S), generator=g)
        w.boundary = _ragged_boundary(g, w.B, w.S, w.T)
        return w
    raise ValueError(f"unknown workload {name!r}")


def simple_call_bytes(w: Workload) -> int:
    """Compulsory HBM bytes of one rnnt_loss_simple fwd+bwd call: read am, lm,
    symbols, boundary; write px_grad, py_grad, am.grad, lm.grad, loss."""
    B, T, S, C = w.B, w.T, w.S, w.C
    f = 4
    return (f * (B * T * C + B * (S + 1) * C) * 2 + 8 * B * S + 32 * B
            + f * (B * S * (T + 1) + B * (S + 1) * T) + f)
