#!/usr/bin/env python3
"""Benchmark of the fast_rnnt loss hot path on one MI355X.

One step = one ``rnnt_loss_simple(..., reduction="sum", return_grad=True)`` call
plus ``loss.backward()`` on the synthetic ASR-shaped batch c2
(B=32, T=250, S=80, C=500, fp32; inputs already resident in HBM).  Prints ONE
JSON line: whole-call throughput (the faster of an eager loop and of the step
replayed as a HIP graph, which is checked bit-equal against eager steps; both
figures are in the line, and so is an eager loop that hands the call a NEW boundary
tensor every step), the roofline figure of the dominant kernel (timed live with
events on the launch stream, priced with the algorithmic work of the boundary
windows) and the CPU baseline (the oracle restatement of the reference path, timed
on this host's cores).

    python bench.py [--gpus 1] [--steps 1000] [--warmup 100] [--workload c2]

Other workloads (--workload c3 | c4 | c5) print the same kind of line for the
pruned pipeline, the large-vocabulary simple loss and the unpruned loss on logits.
"""
import argparse
import json
import os
import re
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3

# hardware-counter summaries (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, calibrated with a
# copy of known size) that `traffic` is read from, one file per workload
TRAFFIC_FILES = {
    "c2": "rnnt_loss_simple_c2_hbm_traffic.txt",
    "c3": "rnnt_pruned_pipeline_c3_hbm_traffic.txt",
    "c4": "rnnt_loss_simple_c4_hbm_traffic.txt",
    "c5": "rnnt_loss_c5_hbm_traffic.txt",
}


def _parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="budget of the CPU-baseline leg (0 disables it)")
    ap.add_argument("--kernel-reps", type=int, default=50)
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="skip the graph-replay leg")
    ap.add_argument("--logits-dtype", default="f32", choices=["f32", "f16", "bf16"],
                    help="c3 / c5: element type of the logits handed to the loss (the 2-byte "
                         "types are read as they are and accumulated in float32)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run device-to-device copies of this size (a reference of known "
                         "traffic for hardware-counter runs)")
    return ap.parse_args()


# ---- small helpers ------------------------------------------------------------------------

def _event_time_ms(fn, reps):
    """Average duration of fn() over `reps` back-to-back launches, measured with
    events recorded on the stream the kernels are enqueued on."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def _wall_loop(step, steps, warmup):
    """`steps` whole steps between two synchronisations; returns seconds."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def _rate(steps, elapsed):
    return {"value": round(steps / elapsed, 2), "unit": "calls/sec",
            "ms_per_step": round(1e3 * elapsed / steps, 4), "steps": steps}


def _measured_traffic(workload):
    """{kernel name: HBM bytes per launch} from the committed counter summary of this
    workload: the table rows `kernel  FETCH_SIZE  WRITE_SIZE  fetch MB  write MB  total MB`."""
    path = os.path.join(ROOT, "profiles", TRAFFIC_FILES.get(workload, ""))
    table = {}
    if not os.path.isfile(path):
        return table, None
    row = re.compile(r"^(\S.*?)\s+([0-9.]+)\s+([0-9.]+)\s+([0-9.]+)\s+([0-9.]+)\s+([0-9.]+)(\s|$)")
    with open(path) as f:
        for text in f:
            m = row.match(text)
            if m:
                table[m.group(1).strip()] = int(round(float(m.group(6)) * 1e6))
    return table, os.path.relpath(path, ROOT)


def _traffic_of(table, kernel):
    """The table's entry for this kernel: exact name first, else the only row of the same
    kernel function (template arguments aside)."""
    if kernel in table:
        return table[kernel]
    base = kernel.split("<")[0].split(" ")[0]
    same = [v for k, v in table.items() if k.split("<")[0] == base]
    return same[0] if len(same) == 1 else None


def _host_info():
    model = None
    try:
        with open("/proc/cpuinfo") as f:
            for text in f:
                if text.lower().startswith("model name"):
                    model = text.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(),
            "cpu_model": model}


def _cpu_baseline(cpu_step, seconds, what, gpu_loss_fn):
    """Times the oracle's restatement of the same call on the host cores for about `seconds`."""
    if seconds <= 0:
        return None
    torch.set_num_threads(os.cpu_count() or 1)
    cpu_step()
    n, t_start = 0, time.perf_counter()
    while True:
        cpu_loss = cpu_step()
        n += 1
        spent = time.perf_counter() - t_start
        if spent > seconds or n >= 5000:
            break
    gpu_loss = gpu_loss_fn()
    info = _host_info()
    return {
        "value": round(n / spent, 3),
        "unit": "fwd+bwd loss calls/sec",
        "cores": info["torch_threads"],
        "kind": "port",
        "sample": f"{n} full {what} calls in {spent:.1f} s (torch-CPU tensor algebra on "
                  f"{info['torch_threads']} threads + single-thread C recursion, serial over the "
                  "batch as in the reference's CPU operator)",
        "host": info,
        "loss_rel_diff_vs_gpu": abs(gpu_loss - cpu_loss.item()) / abs(cpu_loss.item()),
    }


def _hbm_line(table, kernel, nbytes, t_ms, **extra):
    achieved = nbytes / (t_ms * 1e-3) / 1e9
    line = {"kernel": kernel, "bound": "hbm", "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
            "traffic": _traffic_of(table, kernel), "algorithmic_bytes": int(nbytes),
            "avg_launch_us": round(1e3 * t_ms, 2)}
    line.update(extra)
    return line


def _mfma_line(table, kernel, flops, padded_flops, t_ms):
    tflops = flops / (t_ms * 1e-3) / 1e12
    return {"kernel": kernel, "bound": "mfma", "achieved": round(tflops, 3),
            "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tflops / FP32_MFMA_PEAK_TFLOPS, 5),
            "traffic": _traffic_of(table, kernel), "algorithmic_flops": flops,
            "padded_flops": padded_flops,
            "frac_padded": round(padded_flops / (t_ms * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS, 5),
            "avg_launch_us": round(1e3 * t_ms, 2)}


def _graph_replay(step, grads, args):
    """Captures one step (forward and backward through autograd) in a HIP graph and times
    `args.steps` replays; every replay recomputes the loss and the gradients in place.
    Checked against an eager step before and after the timed replays.  `grads()` returns
    the gradient tensors of the step's inputs."""
    try:
        # the gradient-accumulation nodes of the inputs were made on the default stream
        # by the eager steps; autograd's note about that is not an error
        quiet = getattr(torch.autograd.graph, "set_warn_on_accumulate_grad_stream_mismatch", None)
        if quiet is not None:
            quiet(False)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            loss = step()
        held = grads()   # the graph's own output tensors

        def differs():
            graph.replay()
            torch.cuda.synchronize()
            got = [loss.clone()] + [g.clone() for g in held]
            want_loss = step()          # eager work between replays
            torch.cuda.synchronize()
            want = [want_loss] + list(grads())
            return not all(torch.equal(a, b) for a, b in zip(got, want))

        if differs():
            return {"error": "replay differs from the eager step"}
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        if differs():
            return {"error": "replay differs from the eager step after the timed replays"}
        out = _rate(args.steps, elapsed)
        out["checked"] = "loss and gradients bit-equal to an eager step, before and after"
        return out
    except Exception as err:  # the eager figure stands on its own
        return {"error": f"{type(err).__name__}: {err}"}


def _windows(boundary):
    Sb = (boundary[:, 2] - boundary[:, 0]).double()
    Tb = (boundary[:, 3] - boundary[:, 1]).double()
    return Sb, Tb


def _recursion_bytes(boundary, S, T, B, backward):
    """Algorithmic HBM bytes of one recursion launch (fp32): every input cell of
    the boundary window read once, every output cell written once."""
    Sb, Tb = _windows(boundary)
    win = (Sb * (Tb + 1) + (Sb + 1) * Tb + (Sb + 1) * (Tb + 1)).sum().item()
    if not backward:
        return 4 * win + 4 * B + 32 * B
    # backward reads the px/py/p windows, writes the full gradient arrays
    return 4 * win + 4 * (B * S * (T + 1) + B * (S + 1) * T) + 4 * B + 32 * B


def _copy_probe(args, dev):
    """Device-to-device copies of a known size: the reference against which a hardware-counter
    run of this script calibrates FETCH_SIZE / WRITE_SIZE."""
    if args.copy_probe_mib <= 0:
        return
    src = torch.empty(args.copy_probe_mib << 20, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()


def _bmm_yardstick(w, dev, reps):
    """Context only, never on the product path: the vendor library's batched fp32 product of
    the normalizer's shape -- [B, S+1, C] x [B, C, T] on operands that are ALREADY
    exponentiated and resident -- and of the two gradient products' shapes.  It says what
    fraction of the fp32 MFMA peak this shape reaches with no exp, no maxima, no px / py
    assembly and every padded cell computed; the kernels of this library are priced against
    the same peak with the work of the boundary windows only."""
    B, S1, T, C = w.B, w.S + 1, w.T, w.C
    f32 = dict(dtype=torch.float32, device=dev)
    elm, eam = torch.rand(B, S1, C, **f32), torch.rand(B, T, C, **f32)
    d = torch.rand(B, S1, T, **f32)
    out = {}
    flops = 2.0 * B * S1 * T * C
    for name, fn in (("normalizer [B,S+1,C]x[B,C,T]", lambda: torch.bmm(elm, eam.transpose(1, 2))),
                     ("lm_grad [B,S+1,T]x[B,T,C]", lambda: torch.bmm(d, eam)),
                     ("am_grad [B,T,S+1]x[B,S+1,C]", lambda: torch.bmm(d.transpose(1, 2), elm))):
        t_ms = _event_time_ms(fn, reps)
        out[name] = {"us": round(1e3 * t_ms, 2),
                     "TFLOPs_padded": round(flops / (t_ms * 1e-3) / 1e12, 2),
                     "frac_of_fp32_mfma_peak_padded": round(flops / (t_ms * 1e-3) / 157.3e12, 4)}
    return out


def _emit(out):
    print(json.dumps(out))


# ---- c3 / c5: the losses on logits --------------------------------------------------------

def _bench_lattice(args, w, dev):
    """c3 (pruned pipeline) and c5 (unpruned loss on full logits): HBM-streaming
    workloads whose dominant kernel is the logits-gradient kernel."""
    import fast_rnnt_amd
    from fast_rnnt_amd import _lib
    from oracle import losses as O

    table, traffic_file = _measured_traffic(w.name)
    _copy_probe(args, dev)
    sym, bnd = w.symbols.to(dev), w.boundary.to(dev)
    extra = {}
    ldt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[args.logits_dtype]
    esize = 4 if args.logits_dtype == "f32" else 2
    sfx = args.logits_dtype
    if w.name == "c5":
        logits = w.logits.to(dev).to(ldt).requires_grad_(True)

        def step():
            logits.grad = None
            loss = fast_rnnt_amd.rnnt_loss(logits, sym, 0, boundary=bnd, reduction="sum")
            loss.backward()
            return loss

        def grads():
            return (logits.grad,)

        cl = w.logits.to(ldt).float().requires_grad_(True)

        def cpu_step():
            cl.grad = None
            loss = O.loss_joint(cl, w.symbols, 0, boundary=w.boundary, reduction="sum")
            loss.backward()
            return loss

        ranges, R = None, w.S + 1
        lg = logits.detach()
        what = (f"c5: rnnt_loss fwd+bwd on logits [B,T,S+1,C], B={w.B} T={w.T} S={w.S} C={w.C}, "
                "ragged boundary, reduction=sum")
        elapsed = _wall_loop(step, args.steps, args.warmup)
    else:
        am = w.am.to(dev).requires_grad_(True)
        lm = w.lm.to(dev).requires_grad_(True)
        W = w.joiner.to(dev)

        def pipeline(fused):
            am.grad = None
            lm.grad = None
            simple, (gx, gy) = fast_rnnt_amd.rnnt_loss_smoothed(
                lm, am, sym, 0, 0.25, 0.0, boundary=bnd, reduction="sum", return_grad=True)
            rg = fast_rnnt_amd.get_rnnt_prune_ranges(gx, gy, bnd, w.s_range)
            if fused:
                hidden = fast_rnnt_amd.pruned_joiner_input(am, lm, rg, activation="tanh")
            else:
                am_p, lm_p = fast_rnnt_amd.do_rnnt_pruning(am, lm, rg)
                hidden = torch.tanh(am_p + lm_p)
            loss = fast_rnnt_amd.rnnt_loss_pruned((hidden @ W).to(ldt), sym, rg, 0, boundary=bnd,
                                                  reduction="sum")
            (simple + loss).backward()
            return loss

        def step():
            return pipeline(False)

        def grads():
            return (am.grad, lm.grad)

        ca = w.am.clone().requires_grad_(True)
        cl = w.lm.clone().requires_grad_(True)

        def cpu_step():
            ca.grad = None
            cl.grad = None
            simple, (gx, gy) = O.loss_smoothed(cl, ca, w.symbols, 0, 0.25, 0.0,
                                               boundary=w.boundary, reduction="sum",
                                               return_grad=True)
            rg = O.prune_ranges(gx, gy, w.boundary, w.s_range)
            am_p, lm_p = O.prune(ca, cl, rg)
            loss = O.loss_pruned((torch.tanh(am_p + lm_p) @ w.joiner).to(ldt).float(), w.symbols,
                                 rg, 0, boundary=w.boundary, reduction="sum")
            (simple + loss).backward()
            return loss

        with torch.no_grad():
            _, (gx, gy) = fast_rnnt_amd.rnnt_loss_smoothed(
                lm, am, sym, 0, 0.25, 0.0, boundary=bnd, reduction="sum", return_grad=True)
            ranges = fast_rnnt_amd.get_rnnt_prune_ranges(gx, gy, bnd, w.s_range)
            hidden = fast_rnnt_amd.pruned_joiner_input(am, lm, ranges, activation="tanh")
            lg = (hidden @ W).to(ldt).contiguous()
        R = w.s_range
        what = (f"c3: rnnt_loss_smoothed -> get_rnnt_prune_ranges -> do_rnnt_pruning -> joiner "
                f"(tanh of the sum, [C,C] projection) -> rnnt_loss_pruned fwd+bwd, B={w.B} T={w.T} "
                f"S={w.S} C={w.C} s_range={w.s_range}")
        elapsed = _wall_loop(step, args.steps, args.warmup)
        # the same step with pruned_joiner_input in the place of do_rnnt_pruning and the
        # caller's add + tanh: lm_pruned is never written or read back
        fused = _rate(args.steps, _wall_loop(lambda: pipeline(True), args.steps, args.warmup))
        # the caller's joiner (not part of the library): the [B*T*R, C] x [C, C] product and
        # the product that takes the gradient back to the joiner's input (the projection is a
        # constant of the workload, so the step forms no gradient for it)
        g_out = torch.empty_like(lg, dtype=torch.float32)
        h2 = hidden.reshape(-1, w.C)

        def joiner_products():
            torch.matmul(h2, W)
            torch.matmul(g_out.reshape(-1, w.C), W.t())

        t_join = _event_time_ms(joiner_products, max(5, args.kernel_reps // 5))
        extra = {"with_pruned_joiner_input": fused,
                 "callers_joiner_matmuls_ms": round(t_join, 4),
                 "ms_per_step_without_callers_matmuls": round(1e3 * elapsed / args.steps - t_join,
                                                              4)}

    replay = None
    if args.graph:
        replay = _graph_replay(step, grads, args)

    # the two logits kernels alone, through the C ABI, with events on the launch stream; as
    # the losses run them: rows outside an utterance's boundary window are neither read nor
    # (their gradient being zero) computed
    B, S, T, C = w.B, w.S, w.T, w.C
    T1 = T + 1
    f32 = dict(dtype=torch.float32, device=dev)
    px, py = torch.empty(B, S, T1, **f32), torch.empty(B, S + 1, T, **f32)
    norm, xr, yr = (torch.empty(B, T, R, **f32) for _ in range(3))
    gpx, gpy = torch.rand(B, S, T1, **f32), torch.rand(B, S + 1, T, **f32)
    grad = torch.empty_like(lg)
    stream = torch.cuda.current_stream().cuda_stream
    rp = _lib.ptr(ranges)

    def fwd():
        _lib.call("frnnt_lattice_logprobs_fwd_" + sfx, lg.data_ptr(), sym.data_ptr(), rp,
                  bnd.data_ptr(), px.data_ptr(), py.data_ptr(), norm.data_ptr(), xr.data_ptr(),
                  yr.data_ptr(), B, S, T, R, C, 0, 0, 1, stream)

    def bwd():
        _lib.call("frnnt_lattice_logprobs_bwd_" + sfx, lg.data_ptr(), sym.data_ptr(), rp,
                  bnd.data_ptr(), norm.data_ptr(), gpx.data_ptr(), gpy.data_ptr(), grad.data_ptr(),
                  B, S, T, R, C, 0, 0, 1, stream)

    t_f = _event_time_ms(fwd, args.kernel_reps)
    t_b = _event_time_ms(bwd, args.kernel_reps)
    nbytes = lg.numel() * esize
    # rows of the logits inside the windows: frames < T_b and (c5) lattice rows <= S_b;
    # for c3 the range rows of a frame that fall on lattice rows <= S_b
    if ranges is None:
        Sb, Tb = _windows(w.boundary)
        rows_in = ((Sb + 1) * Tb).sum().item()
    else:
        rg = ranges.cpu()
        t_ok = torch.arange(T).reshape(1, T, 1) < w.boundary[:, 3].reshape(B, 1, 1)
        s_ok = rg <= w.boundary[:, 2].reshape(B, 1, 1)
        rows_in = int((t_ok & s_ok).sum().item())
    in_bytes = rows_in * C * esize
    # gradient kernel: reads the rows inside the windows, writes every row (zeros outside);
    # normalizer kernel: reads the rows inside the windows
    lines = [
        _hbm_line(table, "row_grad_regs_kernel" if esize == 4 else "row_grad_narrow_kernel",
                  in_bytes + nbytes, t_b, padded_bytes=2 * nbytes),
        _hbm_line(table, "row_norm_regs_kernel" if esize == 4 else "row_norm_narrow_kernel",
                  in_bytes, t_f, padded_bytes=nbytes,
                  note="launch time includes the small assemble_kernel of the same entry point"),
    ]
    lines.sort(key=lambda r: -r["avg_launch_us"])
    eager = _rate(args.steps, elapsed)
    # the headline is the eager loop (what a training loop runs); the replay is beside it
    best = eager
    cpu = _cpu_baseline(cpu_step, args.cpu_seconds, w.name, lambda: step().item())
    out = {
        "metric": f"fwd+bwd loss calls/sec (B={w.B},T={w.T},S={w.S},C={w.C}) + achieved HBM GB/s",
        "value": best["value"], "unit": "calls/sec", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": best["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if esize == 4 else f"f32 arithmetic on {sfx} logits", "data": "synthetic",
        "config": {"workload": what, "logits_bytes": nbytes,
                   "logits_bytes_inside_windows": in_bytes,
                   "mode": "eager calls"},
        "roofline": lines[0],
        "roofline_other_kernels": lines[1:],
        "traffic_source": traffic_file,
        "cpu_baseline": cpu,
        "eager": eager,
        "graph_replay": replay,
    }
    out.update(extra)
    _emit(out)


# ---- c1 / c2 / c4: the simple loss --------------------------------------------------------

def main():
    args = _parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: the loss path has no multi-GPU part "
              "(each rank would run this same kernel on its own shard); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    import fast_rnnt_amd
    from fast_rnnt_amd import _lib, workloads

    _lib.load()
    dev = torch.device("cuda", 0)
    w = workloads.make(args.workload)
    if w.name in ("c3", "c5"):
        _bench_lattice(args, w, dev)
        return
    table, traffic_file = _measured_traffic(w.name)
    am = w.am.to(dev).requires_grad_(True)
    lm = w.lm.to(dev).requires_grad_(True)
    sym = w.symbols.to(dev)
    bnd = w.boundary.to(dev)

    _copy_probe(args, dev)

    def step(boundary=bnd):
        am.grad = None
        lm.grad = None
        loss, (gx, gy) = fast_rnnt_amd.rnnt_loss_simple(
            lm, am, sym, w.termination_symbol, boundary=boundary, reduction="sum",
            return_grad=True)
        loss.backward()
        return loss

    eager = _rate(args.steps, _wall_loop(step, args.steps, args.warmup))
    # the same loop with a boundary tensor the call has not seen before, as a training loop
    # over ragged batches has: the reference's validity checks (rnnt_loss.py:25-42,
    # mutual_information.py:277-288) would copy its rows to the host and wait for the device;
    # here the recursion's forward kernel tests them (fast_rnnt_amd.set_boundary_checks)
    # (the tensors are made beforehand: the loop times the call, not torch's copy)
    unseen = [bnd.clone() for _ in range(args.steps + args.warmup)]
    torch.cuda.synchronize()
    fresh = _rate(args.steps, _wall_loop(lambda: step(unseen.pop()), args.steps, args.warmup))
    del unseen

    # ---- the same step captured once in a HIP graph and replayed: what the device
    # sustains when the host's launch cost (a handful of short kernels per step) is out of the way
    replay = _graph_replay(step, lambda: (am.grad, lm.grad), args) if args.graph else None

    # ---- per-kernel timings (events on the launch stream), through the entry points the
    # loss call chains and with its flags: with a boundary nothing outside the windows is
    # computed (window_only) ----------------------------------------------------------
    B, S, T, C = w.B, w.S, w.T, w.C
    f32 = dict(dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    with torch.no_grad():
        lm_c, am_c = lm.detach().contiguous(), am.detach().contiguous()
        px, py = torch.empty(B, S, T + 1, **f32), torch.empty(B, S + 1, T, **f32)
        lm_max, am_max = torch.empty(B, S + 1, **f32), torch.empty(B, T, **f32)
        norm_raw = torch.empty(B, S + 1, T, **f32)
        p, scores = torch.empty(B, S + 1, T + 1, **f32), torch.empty(B, **f32)
        gpx, gpy = torch.empty_like(px), torch.empty_like(py)
        dmat = torch.empty(B, S + 1, (T + 3) // 4 * 4, **f32)
        row_x, row_y = torch.empty(B, S + 1, **f32), torch.empty(B, S + 1, **f32)
        col_y = torch.empty(B, T, **f32)
        lm_grad, am_grad = torch.empty_like(lm_c), torch.empty_like(am_c)

        def logprobs():
            _lib.call("frnnt_simple_logprobs_fwd_f32", lm_c.data_ptr(), am_c.data_ptr(),
                      sym.data_ptr(), bnd.data_ptr(), px.data_ptr(), py.data_ptr(),
                      lm_max.data_ptr(), am_max.data_ptr(), norm_raw.data_ptr(), B, S, T, C, 0, 0,
                      1, stream)

        def rec_fwd():
            _lib.call("frnnt_mi_forward_f32", px.data_ptr(), py.data_ptr(), bnd.data_ptr(),
                      p.data_ptr(), scores.data_ptr(), B, S, T, 0, stream)

        def rec_bwd():
            _lib.call("frnnt_mi_backward_f32", px.data_ptr(), py.data_ptr(), bnd.data_ptr(),
                      p.data_ptr(), None, gpx.data_ptr(), gpy.data_ptr(), B, S, T, 0, 0, stream)

        def grads(want_lm, want_am):
            # (no score gradient: the occupation gradients are used as they are)
            _lib.call("frnnt_simple_logprobs_bwd_f32", lm_c.data_ptr(), am_c.data_ptr(),
                      sym.data_ptr(), bnd.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(),
                      norm_raw.data_ptr(), None, 0, 1.0, gpx.data_ptr(), gpy.data_ptr(),
                      dmat.data_ptr(), row_x.data_ptr(), row_y.data_ptr(), col_y.data_ptr(),
                      lm_grad.data_ptr() if want_lm else None,
                      am_grad.data_ptr() if want_am else None, B, S, T, C, 0, 0, 1, stream)

        t_logp = _event_time_ms(logprobs, args.kernel_reps)
        t_fwd = _event_time_ms(rec_fwd, args.kernel_reps)
        t_bwd = _event_time_ms(rec_bwd, args.kernel_reps)
        # The two gradient products (lm.grad, am.grad) through the backward entry point of
        # the logprobs: it also launches the small prep kernel, which the same call without
        # outputs runs alone; the difference of the two event timings is the product kernel(s).
        t_prep = _event_time_ms(lambda: grads(False, False), args.kernel_reps)
        one_launch = float(B) * (S + 1) * T * C < 1e9  # the library's rule for a single launch
        if one_launch:
            t_grads = {"both": _event_time_ms(lambda: grads(True, True), args.kernel_reps) - t_prep}
        else:
            t_grads = {"lm": _event_time_ms(lambda: grads(True, False), args.kernel_reps) - t_prep,
                       "am": _event_time_ms(lambda: grads(False, True), args.kernel_reps) - t_prep}
    stages = {"logprobs_fwd_ms": t_logp, "mi_forward_ms": t_fwd, "mi_backward_ms": t_bwd,
              "bwd_prep_ms": t_prep}
    stages.update({"bwd_grad_%s_ms" % k: v for k, v in t_grads.items()})

    # Algorithmic work of the normalizer contraction exp(lm - max) . exp(am - max)^T and of
    # each of its two gradient products: 2 C sum_b (S_b + 1) T_b flop -- the cells of the
    # boundary windows; outside them the loss uses nothing and the gradients are zero.
    # The padded figure 2 C B (S+1) T is printed beside it.
    Sb, Tb = _windows(w.boundary)
    gemm_flops = 2.0 * C * ((Sb + 1) * Tb).sum().item()
    gemm_padded = 2.0 * B * (S + 1) * T * C
    rows96 = (S + 1 + 95) // 96 * 96 < (S + 1 + 127) // 128 * 128
    fwd_name = "simple_fwd_panel_kernel<%s>" % ("96, 16" if rows96 else "128, 16")
    lm_shape = "96, 32" if rows96 else "128, 16"     # the lm.grad kernel on its own
    both_shape = "96, 16" if rows96 else "128, 16"   # inside the common launch
    # each gradient product is one GEMM of the forward's size (the one-hot product that
    # scatters px_grad into am.grad is not counted)
    if "both" in t_grads:
        lines = [_mfma_line(table, "simple_bwd_am_lm_kernel<%s>" % both_shape, 2 * gemm_flops,
                            2 * gemm_padded, t_grads["both"])]
    else:
        lines = [_mfma_line(table, "simple_bwd_am_panel_kernel", gemm_flops, gemm_padded,
                            t_grads["am"]),
                 _mfma_line(table, "simple_bwd_lm_slab_kernel<%s>" % lm_shape, gemm_flops,
                            gemm_padded, t_grads["lm"])]
    steps_chain = int((Sb + Tb).max().item())
    lines += [
        # the same kernel finds the row maxima on the way and assembles px / py at the end
        _mfma_line(table, fwd_name, gemm_flops, gemm_padded, t_logp),
        # the recursion kernels are bound by their dependent chain (S_b + T_b steps), not by
        # bytes: cycles per step at 2.4 GHz are given beside the bandwidth figure
        _hbm_line(table, "mi_forward_kernel", _recursion_bytes(w.boundary, S, T, B, False), t_fwd,
                  chain_steps=steps_chain,
                  cycles_per_step=round(t_fwd * 1e-3 * 2.4e9 / steps_chain, 1)),
        _hbm_line(table, "mi_backward_kernel", _recursion_bytes(w.boundary, S, T, B, True), t_bwd,
                  chain_steps=steps_chain,
                  cycles_per_step=round(t_bwd * 1e-3 * 2.4e9 / steps_chain, 1)),
    ]
    # the dominant kernel of the step is the one with the longest launch
    lines.sort(key=lambda r: -r["avg_launch_us"])

    # ---- CPU baseline: the oracle restatement of the reference path ------------------
    from oracle import losses as O

    a = w.am.clone().requires_grad_(True)
    l = w.lm.clone().requires_grad_(True)

    def cpu_step():
        a.grad = None
        l.grad = None
        loss, _ = O.loss_simple(l, a, w.symbols, 0, boundary=w.boundary, reduction="sum",
                                return_grad=True)
        loss.backward()
        return loss

    cpu = _cpu_baseline(cpu_step, args.cpu_seconds, w.name, lambda: step().item())

    # The headline is the eager loop: one API call and one backward per step, what a training
    # loop runs.  The step is a handful of kernels of 4-30 us, so the host's launch work per
    # step matters; the replayed HIP graph of the same step -- same kernels, outputs checked
    # bit-equal against eager steps -- shows what the device sustains without it and is
    # reported beside the headline, like the eager loop with a new boundary tensor per step.
    # All loops time exactly args.steps whole steps.
    best = eager
    mode = "eager calls"
    call_bytes = workloads.simple_call_bytes(w)
    out = {
        "metric": f"fwd+bwd loss calls/sec (B={w.B},T={w.T},S={w.S},C={w.C}) + achieved HBM GB/s",
        "value": best["value"],
        "unit": "calls/sec",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": best["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: rnnt_loss_simple fwd+bwd, B={w.B} T={w.T} S={w.S} "
                               f"C={w.C}, ragged boundary, reduction=sum, return_grad=True",
                   "mode": mode,
                   "call_bytes": call_bytes},
        "roofline": lines[0],
        "roofline_other_kernels": lines[1:],
        "traffic_source": traffic_file,
        "cpu_baseline": cpu,
        "eager": eager,
        "eager_fresh_boundary": fresh,
        "graph_replay": replay,
        "stages": {k: round(v, 4) for k, v in stages.items()},
        "whole_call_hbm_GBs": round(call_bytes / (best["ms_per_step"] * 1e-3) / 1e9, 2),
        "vendor_bmm_yardstick": _bmm_yardstick(w, dev, args.kernel_reps),
    }
    _emit(out)


if __name__ == "__main__":
    main()
