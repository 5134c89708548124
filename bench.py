#!/usr/bin/env python3
"""Benchmark of the fast_rnnt loss hot path on one MI355X.

One step = one ``rnnt_loss_simple(..., reduction="sum", return_grad=True)`` call
plus ``loss.backward()`` on the synthetic ASR-shaped batch c2
(B=32, T=250, S=80, C=500, fp32; inputs already resident in HBM).  Prints ONE
JSON line: whole-call throughput (the faster of an eager loop and of the step
replayed as a HIP graph, which is checked bit-equal against eager steps; both
figures are in the line), the roofline
figure of the dominant kernel (timed live with events on the launch stream) and
the CPU baseline (the oracle restatement of the reference path, timed on this
host's cores).

    python bench.py [--gpus 1] [--steps 1000] [--warmup 100] [--workload c2]
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3
# HBM bytes per launch (fetch + write) from the rocprofv3 --pmc runs summarised under
# profiles/ (FETCH_SIZE and WRITE_SIZE, scaled by what the same counters read for a
# copy of known size); filled in for the workloads that were profiled
MEASURED_TRAFFIC = {
    ("c2", "simple_fwd_panel_kernel<96, 16>"): 29256563,
    ("c2", "mi_forward_kernel<float, false, 2, 2, 3>"): 6732768,
    ("c2", "mi_backward_kernel<float, false, 2, 6, 3>"): 9667956,
    ("c2", "simple_bwd_am_lm_kernel<96, 16>"): 50092198,
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
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run device-to-device copies of this size (a reference of known "
                         "traffic for hardware-counter runs)")
    return ap.parse_args()


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


def _graph_replay(step, am, lm, args):
    """Captures one step (forward and backward through autograd) in a HIP graph and times
    `args.steps` replays; every replay recomputes the loss and both gradients in place.
    Checked against an eager step before and after the timed replays."""
    try:
        # the gradient-accumulation nodes of am / lm were made on the default stream
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
        g_am, g_lm = am.grad, lm.grad   # the graph's own output tensors

        def differs():
            graph.replay()
            torch.cuda.synchronize()
            got = (loss.clone(), g_am.clone(), g_lm.clone())
            want_loss = step()          # eager work between replays
            torch.cuda.synchronize()
            same = (torch.equal(got[0], want_loss) and torch.equal(got[1], am.grad)
                    and torch.equal(got[2], lm.grad))
            return not same

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
        return {"value": round(args.steps / elapsed, 2), "unit": "calls/sec",
                "ms_per_step": round(1e3 * elapsed / args.steps, 4), "steps": args.steps,
                "checked": "loss and both gradients bit-equal to an eager step, before and after"}
    except Exception as err:  # the eager figure stands on its own
        return {"error": f"{type(err).__name__}: {err}"}


def _recursion_bytes(boundary, S, T, B, backward):
    """Algorithmic HBM bytes of one recursion launch (fp32): every input cell of
    the boundary window read once, every output cell written once."""
    Sb = boundary[:, 2] - boundary[:, 0]
    Tb = boundary[:, 3] - boundary[:, 1]
    win = (Sb * (Tb + 1) + (Sb + 1) * Tb + (Sb + 1) * (Tb + 1)).sum().item()
    if not backward:
        return 4 * win + 4 * B + 32 * B
    # backward reads the px/py/p windows, writes the full gradient arrays
    return 4 * win + 4 * (B * S * (T + 1) + B * (S + 1) * T) + 4 * B + 32 * B


def _bench_lattice(args, w, dev):
    """c3 (pruned pipeline) and c5 (unpruned loss on full logits): HBM-streaming
    workloads whose dominant kernel is the logits-gradient kernel."""
    import fast_rnnt_amd
    from fast_rnnt_amd import _lib

    sym, bnd = w.symbols.to(dev), w.boundary.to(dev)
    if w.name == "c5":
        logits = w.logits.to(dev).requires_grad_(True)

        def step():
            logits.grad = None
            loss = fast_rnnt_amd.rnnt_loss(logits, sym, 0, boundary=bnd, reduction="sum")
            loss.backward()
            return loss

        ranges, R = None, w.S + 1
        lg = logits.detach()
        what = (f"c5: rnnt_loss fwd+bwd on logits [B,T,S+1,C], B={w.B} T={w.T} S={w.S} C={w.C}, "
                "ragged boundary, reduction=sum")
    else:
        am = w.am.to(dev).requires_grad_(True)
        lm = w.lm.to(dev).requires_grad_(True)
        W = w.joiner.to(dev)

        def step():
            am.grad = None
            lm.grad = None
            simple, (gx, gy) = fast_rnnt_amd.rnnt_loss_smoothed(
                lm, am, sym, 0, 0.25, 0.0, boundary=bnd, reduction="sum", return_grad=True)
            rg = fast_rnnt_amd.get_rnnt_prune_ranges(gx, gy, bnd, w.s_range)
            am_p, lm_p = fast_rnnt_amd.do_rnnt_pruning(am, lm, rg)
            loss = fast_rnnt_amd.rnnt_loss_pruned(torch.tanh(am_p + lm_p) @ W, sym, rg, 0,
                                                  boundary=bnd, reduction="sum")
            (simple + loss).backward()
            return loss

        with torch.no_grad():
            _, (gx, gy) = fast_rnnt_amd.rnnt_loss_smoothed(
                lm, am, sym, 0, 0.25, 0.0, boundary=bnd, reduction="sum", return_grad=True)
            ranges = fast_rnnt_amd.get_rnnt_prune_ranges(gx, gy, bnd, w.s_range)
            am_p, lm_p = fast_rnnt_amd.do_rnnt_pruning(am, lm, ranges)
            lg = (torch.tanh(am_p + lm_p) @ W).contiguous()
        R = w.s_range
        what = (f"c3: rnnt_loss_smoothed -> get_rnnt_prune_ranges -> do_rnnt_pruning -> joiner -> "
                f"rnnt_loss_pruned fwd+bwd, B={w.B} T={w.T} S={w.S} C={w.C} s_range={w.s_range}")

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # the two logits kernels alone, through the C ABI, with events on the launch stream
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
        _lib.call("frnnt_lattice_logprobs_fwd_f32", lg.data_ptr(), sym.data_ptr(), rp,
                  bnd.data_ptr(), px.data_ptr(), py.data_ptr(), norm.data_ptr(), xr.data_ptr(),
                  yr.data_ptr(), B, S, T, R, C, 0, 0, 1, stream)

    def bwd():
        _lib.call("frnnt_lattice_logprobs_bwd_f32", lg.data_ptr(), sym.data_ptr(), rp,
                  bnd.data_ptr(), norm.data_ptr(), gpx.data_ptr(), gpy.data_ptr(), grad.data_ptr(),
                  B, S, T, R, C, 0, 0, 1, stream)

    t_f = _event_time_ms(fwd, args.kernel_reps)
    t_b = _event_time_ms(bwd, args.kernel_reps)
    nbytes = lg.numel() * 4

    def line(kernel, b, t_ms):
        a = b / (t_ms * 1e-3) / 1e9
        return {"kernel": kernel, "bound": "hbm", "achieved": round(a, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(a / HBM_PEAK_GBS, 4), "traffic": None,
                "algorithmic_bytes": b, "avg_launch_us": round(1e3 * t_ms, 2)}

    out = {
        "metric": "fwd+bwd loss calls/sec + achieved HBM GB/s",
        "value": round(args.steps / elapsed, 2), "unit": "calls/sec", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(1e3 * elapsed / args.steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": what, "logits_bytes": nbytes},
        # one read and one write of the logits (gradient kernel); one read (normalizer kernel,
        # whose entry point also runs the small px/py assembly kernel)
        "roofline": line("row_grad_regs_kernel", 2 * nbytes, t_b),
        "roofline_other_kernels": [line("row_norm_regs_kernel (+ assemble_kernel)", nbytes, t_f)],
        "cpu_baseline": None,
    }
    print(json.dumps(out))


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
    from fast_rnnt_amd import _fast_rnnt, _lib, workloads
    from fast_rnnt_amd.rnnt_loss import _SimpleLogprobs

    _lib.load()
    dev = torch.device("cuda", 0)
    w = workloads.make(args.workload)
    if w.name in ("c3", "c5"):
        _bench_lattice(args, w, dev)
        return
    am = w.am.to(dev).requires_grad_(True)
    lm = w.lm.to(dev).requires_grad_(True)
    sym = w.symbols.to(dev)
    bnd = w.boundary.to(dev)

    if args.copy_probe_mib > 0:
        src = torch.empty(args.copy_probe_mib << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    def step():
        am.grad = None
        lm.grad = None
        loss, (gx, gy) = fast_rnnt_amd.rnnt_loss_simple(
            lm, am, sym, w.termination_symbol, boundary=bnd, reduction="sum", return_grad=True)
        loss.backward()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    calls_per_sec = args.steps / elapsed

    # ---- the same step captured once in a HIP graph and replayed: what the device
    # sustains when the host's launch cost (nine short kernels per step) is out of the way
    replay = _graph_replay(step, am, lm, args) if args.graph else None

    # ---- per-stage kernel timings (events on the launch stream) -------------------
    with torch.no_grad():
        px, py = fast_rnnt_amd.get_rnnt_logprobs(lm, am, sym, 0, boundary=bnd)
        B, S, T = w.B, w.S, w.T
        p = torch.empty(B, S + 1, T + 1, device=dev)
        ones = torch.ones(B, device=dev)
        t_fwd = _event_time_ms(lambda: _fast_rnnt.mutual_information_forward(px, py, bnd, p),
                               args.kernel_reps)
        t_bwd = _event_time_ms(
            lambda: _fast_rnnt.mutual_information_backward(px, py, bnd, p, ones),
            args.kernel_reps)
        t_logp = _event_time_ms(
            lambda: fast_rnnt_amd.get_rnnt_logprobs(lm, am, sym, 0, boundary=bnd),
            args.kernel_reps)
        # The two gradient products (lm.grad, am.grad) through the backward entry point of
        # the logprobs: it also launches the small prep kernel, which the same call without
        # outputs runs alone; the difference of the two event timings is the product kernel(s).
        C = w.C
        f32 = dict(dtype=torch.float32, device=dev)
        lm_c, am_c = lm.detach().contiguous(), am.detach().contiguous()
        lm_max, am_max = torch.empty(B, S + 1, **f32), torch.empty(B, T, **f32)
        norm_raw = torch.empty(B, S + 1, T, **f32)
        stream = torch.cuda.current_stream().cuda_stream
        _lib.call("frnnt_simple_logprobs_fwd_f32", lm_c.data_ptr(), am_c.data_ptr(), sym.data_ptr(),
                  bnd.data_ptr(), px.data_ptr(), py.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(),
                  norm_raw.data_ptr(), B, S, T, C, 0, 0, 1, stream)
        gpx, gpy = torch.rand_like(px), torch.rand_like(py)
        dmat = torch.empty(B, S + 1, (T + 3) // 4 * 4, **f32)
        row_x, row_y = torch.empty(B, S + 1, **f32), torch.empty(B, S + 1, **f32)
        col_y = torch.empty(B, T, **f32)
        lm_grad, am_grad = torch.empty_like(lm_c), torch.empty_like(am_c)

        def grads(want_lm, want_am):
            _lib.call("frnnt_simple_logprobs_bwd_f32", lm_c.data_ptr(), am_c.data_ptr(),
                      sym.data_ptr(), bnd.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(),
                      norm_raw.data_ptr(), None, 0, 1.0, gpx.data_ptr(), gpy.data_ptr(),
                      dmat.data_ptr(), row_x.data_ptr(), row_y.data_ptr(), col_y.data_ptr(),
                      lm_grad.data_ptr() if want_lm else None,
                      am_grad.data_ptr() if want_am else None, B, S, T, C, 0, 0, 1, stream)

        t_prep = _event_time_ms(lambda: grads(False, False), args.kernel_reps)
        one_launch = float(B) * (S + 1) * T * C < 1e9  # the library's rule for a single launch
        if one_launch:
            t_grads = {"both": _event_time_ms(lambda: grads(True, True), args.kernel_reps) - t_prep}
        else:
            t_grads = {"lm": _event_time_ms(lambda: grads(True, False), args.kernel_reps) - t_prep,
                       "am": _event_time_ms(lambda: grads(False, True), args.kernel_reps) - t_prep}
    stages = {"mi_forward_ms": t_fwd, "mi_backward_ms": t_bwd, "logprobs_fwd_ms": t_logp,
              "bwd_prep_ms": t_prep}
    stages.update({"bwd_grad_%s_ms" % k: v for k, v in t_grads.items()})

    def hbm_line(kernel, nbytes, t_ms):
        achieved = nbytes / (t_ms * 1e-3) / 1e9
        return {"kernel": kernel, "bound": "hbm", "achieved": round(achieved, 2),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                "traffic": MEASURED_TRAFFIC.get((w.name, kernel)), "algorithmic_bytes": nbytes,
                "avg_launch_us": round(1e3 * t_ms, 2)}

    # normalizer contraction exp(lm - max) . exp(am - max)^T on the fp32 matrix cores;
    # the same kernel finds the row maxima on the way and assembles px/py at the end,
    # so this figure is a lower bound on the rate of its MFMA loop
    gemm_name = "simple_fwd_panel_kernel<96, 16>" if (S + 1 + 95) // 96 * 96 < (S + 1 + 127) // 128 * 128 \
        else "simple_fwd_panel_kernel<128, 16>"
    gemm_flops = 2.0 * B * (S + 1) * T * w.C
    gemm_tflops = gemm_flops / (t_logp * 1e-3) / 1e12
    rows96 = (S + 1 + 95) // 96 * 96 < (S + 1 + 127) // 128 * 128
    lm_shape = "96, 32" if rows96 else "128, 16"     # the lm.grad kernel on its own
    both_shape = "96, 16" if rows96 else "128, 16"   # inside the common launch

    def mfma_line(kernel, flops, t_ms):
        tflops = flops / (t_ms * 1e-3) / 1e12
        return {"kernel": kernel, "bound": "mfma", "achieved": round(tflops, 3),
                "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tflops / FP32_MFMA_PEAK_TFLOPS, 5),
                "traffic": MEASURED_TRAFFIC.get((w.name, kernel)), "algorithmic_flops": flops,
                "avg_launch_us": round(1e3 * t_ms, 2)}

    # each gradient product is one GEMM of the forward's size (the one-hot product that
    # scatters px_grad into am.grad is not counted)
    if "both" in t_grads:
        grad_lines = [mfma_line("simple_bwd_am_lm_kernel<%s>" % both_shape, 2 * gemm_flops,
                                t_grads["both"])]
    else:
        grad_lines = [mfma_line("simple_bwd_am_panel_kernel", gemm_flops, t_grads["am"]),
                      mfma_line("simple_bwd_lm_slab_kernel<%s>" % lm_shape, gemm_flops,
                                t_grads["lm"])]
    lines = grad_lines + [
        hbm_line("mi_forward_kernel<float, false, 2, 2, 3>",
                 _recursion_bytes(w.boundary, S, T, B, backward=False), t_fwd),
        hbm_line("mi_backward_kernel<float, false, 2, 6, 3>",
                 _recursion_bytes(w.boundary, S, T, B, backward=True), t_bwd),
        {"kernel": gemm_name, "bound": "mfma", "achieved": round(gemm_tflops, 3),
         "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
         "frac": round(gemm_tflops / FP32_MFMA_PEAK_TFLOPS, 5),
         "traffic": MEASURED_TRAFFIC.get((w.name, gemm_name)), "algorithmic_flops": gemm_flops,
         "avg_launch_us": round(1e3 * t_logp, 2)},
    ]
    # the dominant kernel of the step is the one with the longest launch
    lines.sort(key=lambda r: -r["avg_launch_us"])
    roofline = lines[0]
    other = lines[1:]

    # ---- CPU baseline: the oracle restatement of the reference path ------------------
    cpu = None
    if args.cpu_seconds > 0:
        from oracle import losses as O

        cores = os.cpu_count() or 1
        torch.set_num_threads(min(cores, 16))
        a = w.am.clone().requires_grad_(True)
        l = w.lm.clone().requires_grad_(True)

        def cpu_step():
            a.grad = None
            l.grad = None
            loss, _ = O.loss_simple(l, a, w.symbols, 0, boundary=w.boundary, reduction="sum",
                                    return_grad=True)
            loss.backward()
            return loss

        cpu_step()
        cpu_step()
        n, t_start = 0, time.perf_counter()
        while True:
            cpu_loss = cpu_step()
            n += 1
            spent = time.perf_counter() - t_start
            if spent > args.cpu_seconds or n >= 5000:
                break
        gpu_loss = step().item()
        cpu = {
            "value": round(n / spent, 3),
            "unit": "fwd+bwd loss calls/sec",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{n} full {w.name} calls in {spent:.1f} s (torch-CPU tensor algebra on "
                      f"{torch.get_num_threads()} threads + single-thread C recursion)",
            "loss_rel_diff_vs_gpu": abs(gpu_loss - cpu_loss.item()) / abs(cpu_loss.item()),
        }

    # The step is seven kernels of 4-36 us.  An eager loop of nothing but this call is bound by
    # the host's launch work on slow hosts (in training that work hides behind the model's own
    # kernels); the replayed graph of the same step -- same kernels, outputs checked bit-equal
    # against eager steps -- does not depend on the host, but its nodes start a little further
    # apart than kernels a fast host has queued ahead.  Both loops time exactly args.steps whole
    # steps; the headline is the faster of the two and config.mode says which, and both are
    # reported beside it.  Without a graph (capture refused, --no-graph) eager is the headline.
    eager = {"value": round(calls_per_sec, 2), "unit": "calls/sec",
             "ms_per_step": round(ms_per_step, 4), "steps": args.steps}
    graphed = replay is not None and "value" in replay and replay["value"] > calls_per_sec
    mode = ("HIP-graph replay of one captured rnnt_loss_simple + backward step" if graphed
            else "eager calls")
    if graphed:
        calls_per_sec, ms_per_step = replay["value"], replay["ms_per_step"]
        elapsed = args.steps * ms_per_step * 1e-3
    out = {
        "metric": "fwd+bwd loss calls/sec (B=32,T=250,S=80,C=500) + achieved HBM GB/s",
        "value": round(calls_per_sec, 2),
        "unit": "calls/sec",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: rnnt_loss_simple fwd+bwd, B={w.B} T={w.T} S={w.S} "
                               f"C={w.C}, ragged boundary, reduction=sum, return_grad=True",
                   "mode": mode,
                   "call_bytes": workloads.simple_call_bytes(w)},
        "roofline": roofline,
        "roofline_other_kernels": other,
        "cpu_baseline": cpu,
        "eager": eager,
        "graph_replay": replay,
        "stages": {k: round(v, 4) for k, v in stages.items()},
        "whole_call_hbm_GBs": round(workloads.simple_call_bytes(w) / elapsed * args.steps / 1e9, 2),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
