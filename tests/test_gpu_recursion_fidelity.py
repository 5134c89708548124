"""The recursion kernels alone, at the lattice sizes of the benchmark workloads, fed the
ORACLE's own px / py bits -- so that what is compared is mi_forward / mi_backward and
nothing else (no GEMM summation order in between) -- and on inputs with -inf scattered
through px inside partial boundary windows.

Bounds: float32 scores 1e-5 relative; px_grad / py_grad 1e-4 absolute at every workload
(measured: 7e-6 .. 1.4e-5 -- on identical inputs the kernels follow the CPU reference far
more closely than one ulp of px / py moves the reference itself, which is 2.1e-4 at the
400-frame workload, tests/ulp_sensitivity.py), and never further from the float64 oracle
than 1.5 x the float32 CPU reference is.
"""
import math
import sys

import pytest
import torch

from fast_rnnt_amd import _fast_rnnt
from fast_rnnt_amd import workloads
from oracle import losses as O
from oracle import recursion as oracle

import test_gpu_recursion as base
import ulp_sensitivity as U

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _oracle_lattice(name):
    w = workloads.make(name)
    if name == "c3":
        px, py = O.lattice_logprobs_smoothed(w.lm, w.am, w.symbols, 0, 0.25, 0.0,
                                             boundary=w.boundary)
    elif name == "c5":
        px, py = O.lattice_logprobs_joint(w.logits, w.symbols, 0, boundary=w.boundary)
    else:
        px, py = O.lattice_logprobs_simple(w.lm, w.am, w.symbols, 0, boundary=w.boundary)
    return w, px.contiguous(), py.contiguous()


@pytest.mark.parametrize("name", ["c2", "c3", "c4", "c5"])
def test_recursion_alone_on_the_oracles_lattice(gpu_device, name):
    dev = gpu_device
    w, px, py = _oracle_lattice(name)
    B, S, T = w.B, w.S, w.T
    _say(f"recursion only, {name}: B={B} S={S} T={T}")
    ones = torch.ones(B)
    p_cpu = torch.empty(B, S + 1, T + 1)
    a_cpu = oracle.mi_forward(px, py, w.boundary, p_cpu)
    gx_cpu, gy_cpu = oracle.mi_backward(px, py, w.boundary, p_cpu, ones)
    gx64, gy64 = U.occupation_grads(px.double(), py.double(), w.boundary)

    dpx, dpy, dbnd = px.to(dev), py.to(dev), w.boundary.to(dev)
    p_gpu = torch.empty(B, S + 1, T + 1, device=dev)
    a_gpu = _fast_rnnt.mutual_information_forward(dpx, dpy, dbnd, p_gpu)
    gx, gy = _fast_rnnt.mutual_information_backward(dpx, dpy, dbnd, p_gpu, ones.to(dev))
    torch.cuda.synchronize()
    gx, gy = gx.cpu(), gy.cpu()

    rel = ((a_gpu.cpu() - a_cpu).abs() / a_cpu.abs()).max().item()
    off = max((gx - gx_cpu).abs().max().item(), (gy - gy_cpu).abs().max().item())
    bound = 1e-4
    gpu64 = max((gx.double() - gx64).abs().max().item(), (gy.double() - gy64).abs().max().item())
    cpu64 = max((gx_cpu.double() - gx64).abs().max().item(),
                (gy_cpu.double() - gy64).abs().max().item())
    _say(f"  scores rel {rel:.2e}; px/py_grad vs float32 oracle {off:.2e} (bound {bound:.2e}); "
         f"vs float64: gpu {gpu64:.2e}, cpu float32 {cpu64:.2e}")
    assert rel <= 1e-5
    assert off <= bound
    assert gpu64 <= 1.5 * cpu64 + 2e-5


def _sprinkled(seed, B, S, T, modified, dtype, scale):
    g = torch.Generator().manual_seed(seed)
    px = scale * torch.randn(B, S, T + (0 if modified else 1), generator=g, dtype=dtype)
    py = scale * torch.randn(B, S + 1, T, generator=g, dtype=dtype) - 2
    px[torch.rand(px.shape, generator=g) < 0.05] = -math.inf
    w = torch.randn(B, generator=g, dtype=dtype)
    return g, px, py, w


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_neg_inf_scattered_through_px_with_windows(gpu_device, dtype, modified):
    # 5 % of px blocked, partial / empty windows (some utterances lose every path: -inf
    # score, zero gradients), one and several sweep waves, inputs of scale 1 and 3
    for n, (B, S, T, scale) in enumerate([(5, 12, 40, 1.0), (5, 84, 165, 3.0), (5, 107, 342, 3.0),
                                          (5, 150, 90, 1.0), (10, 70, 33, 0.3)]):
        g, px, py, w = _sprinkled(500 + n, B, S, T, modified, dtype, scale)
        base._compare(px, py, base._windows(g, B, S, T, modified), w, gpu_device, f"sprinkled{n}")
        base._compare(px, py, None, w, gpu_device, f"sprinkled{n}-whole")


def test_scores_that_pass_through_zero(gpu_device):
    # inputs of scale 3: p climbs to several hundred and comes back through zero, where a
    # bound relative to the cell itself would ask for more than float32 holds (the float32
    # CPU reference is then 6e-5 from the float64 one at such cells)
    for n, (B, S, T, modified) in enumerate([(1, 84, 165, False), (3, 107, 342, True)]):
        g = torch.Generator().manual_seed(1036 + n)
        px = 3.0 * torch.randn(B, S, T + (0 if modified else 1), generator=g)
        py = 3.0 * torch.randn(B, S + 1, T, generator=g) - 2
        w = torch.randn(B, generator=g)
        base._compare(px, py, base._windows(g, B, S, T, modified), w, gpu_device, f"zero-crossing{n}")
        base._compare(px, py, None, w, gpu_device, f"zero-crossing{n}-whole")
