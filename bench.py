"""Benchmark of the block-local grid update on one MI355X.

One "step" = one pass of the network body over one synthetic batch: ``outer`` x (stencil step,
LayerNorm) forward and, for training workloads, the same chain backward, called through the C
ABI on preallocated device buffers (inputs resident in HBM before the clock starts).
Prints ONE JSON line with the headline metric, the roofline of the dominant kernel and the
CPU baseline (the reference-style torch path, timed on this machine's host cores).
"""

import argparse
import dataclasses
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, vendor peak
FP32_PEAK_TFLOPS = 157.3  # MI355X vector fp32, vendor peak (with packed fp32 instructions)
# This build compiles with packed fp32 arithmetic switched off: one FMA per lane and clock,
# 256 CUs x 4 SIMDs x 16 lanes x 2 flop x 2.4 GHz = half the vendor figure.
FP32_UNPACKED_PEAK_TFLOPS = FP32_PEAK_TFLOPS / 2
LDS_BYTES_PER_CLOCK_PER_CU = 128
CUS = 256


def gpu_run(wl, steps, warmup, fused, graph_replay=True, chain_all=None, chain=None, outer_residual=False):
    import torch

    from gridnet_amd.configs import make_inputs
    from gridnet_amd.runner import BodyRunner

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    t = {k: v.to(dev) for k, v in make_inputs(wl, seed=0).items()}
    run = BodyRunner(t["weight"], t["bias"], t["scale"], t["gamma"], t["beta"], wl.batch, wl.inner,
                     wl.outer, wl.block_size, wl.activation, wl.normalize, backward=wl.backward,
                     fused=fused, chain_all=chain_all, chain=chain, outer_residual=outer_residual)

    def one_step():
        run.forward(t["x0"])
        if wl.backward:
            run.backward(t["grad_out"])

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    # the one-launch chain backward reports through a status word whether its bounded waits held;
    # a timing with invalid results is no timing
    if run.chain_all_status() != 0:
        sys.exit("bench.py: gridnet_hip_chain_backward_all gave up (status word set): results invalid; "
                 "re-run with --chain-all off")

    # The same step as one captured HIP graph, replayed: what is left when the host side (Python,
    # ctypes, launch calls) is taken out.  Reported beside the eager figure, which stays the headline.
    graph_s = None
    try:
        if not graph_replay:
            raise RuntimeError("switched off (--no-graph)")
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            one_step()  # this stream's first use, outside the capture
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                one_step()
            for _ in range(max(1, warmup)):
                graph.replay()
            side.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                graph.replay()
            side.synchronize()
            graph_s = (time.perf_counter() - t0) / steps
        torch.cuda.current_stream(dev).wait_stream(side)
        del graph
    except RuntimeError as exc:  # reported, not fatal: the headline does not depend on it
        print(f"bench.py: HIP graph replay skipped: {exc}", file=sys.stderr, flush=True)
    torch.cuda.synchronize()

    # per-entry-point device time: events recorded on the stream the kernels are launched on
    # (torch's current stream is the one handed to the C ABI), in a separate instrumented pass
    spans = {}
    pending = []

    def hook(name, phase):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(torch.cuda.current_stream(dev))
        pending.append((name, phase, ev))

    run.on_launch = hook
    reps = max(2, min(steps, 5))
    for _ in range(reps):
        one_step()
    torch.cuda.synchronize()
    run.on_launch = None
    for (name, p0, e0), (_, p1, e1) in zip(pending[0::2], pending[1::2]):
        assert p0 == 0 and p1 == 1
        spans.setdefault(name, []).append(e0.elapsed_time(e1) * 1e-3)
    kernel_s = {k: sum(v) / len(v) for k, v in spans.items()}
    return wall, graph_s, kernel_s, bool(getattr(run, "chain_all", False))


def what_binds(hbm_frac, valu_busy_pct, lds_busy_frac):
    """One sentence from the figures of this line: which of HBM, vector ALU and LDS pipe the
    dominant kernel keeps busiest, and whether that one is saturated."""
    util = {"HBM bandwidth": hbm_frac,
            "vector ALU": None if valu_busy_pct is None else valu_busy_pct / 100.0,
            "LDS pipe": lds_busy_frac}
    known = {k: v for k, v in util.items() if v is not None}
    if not known:
        return None
    shown = ", ".join(f"{k} {100 * v:.0f} %" for k, v in known.items())
    top = max(known, key=known.get)
    if known[top] >= 0.8:
        return f"{top} ({shown}; HBM against the vendor peak, the pipes as busy cycles from the profile)"
    return (f"none of the three is saturated ({shown}; HBM against the vendor peak, the pipes as busy cycles "
            f"from the profile): the busiest is the {top}, and the waves wait on LDS and ALU latency at the "
            "occupancy the register file allows")


def cpu_baseline(wl, budget_s=25.0):
    """The reference-style pure-torch path (block loop + gather; oracle.ref_style) composed with
    F.layer_norm, forward + autograd backward, on a bounded sample of the workload."""
    import torch

    from gridnet_amd.configs import make_inputs
    from oracle.network import network_forward
    from oracle.ref_style import gridnet_step_ref

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    grid, batch = min(wl.grid, 64), min(wl.batch, 32)
    t = make_inputs(wl, seed=0, batch=batch, grid=grid)
    params = [t[k].requires_grad_(wl.backward) for k in ("weight", "bias", "scale", "gamma", "beta")]
    x0 = t["x0"].requires_grad_(wl.backward)

    def once():
        y = network_forward(*params, x0, wl.inner, 1, wl.block_size, wl.activation, wl.normalize,
                            step_fn=gridnet_step_ref)
        if wl.backward:
            torch.autograd.grad(y, params + [x0], t["grad_out"])

    tiny = make_inputs(wl, seed=0, batch=2, grid=16)  # warm-up: thread pool, allocator
    network_forward(*[tiny[k] for k in ("weight", "bias", "scale", "gamma", "beta")], tiny["x0"],
                    wl.inner, 1, wl.block_size, wl.activation, wl.normalize, step_fn=gridnet_step_ref)
    times = []
    start = time.perf_counter()
    while len(times) < 3 and (time.perf_counter() - start < budget_s or not times):
        t0 = time.perf_counter()
        once()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    cu = batch * grid ** 3 * wl.inner
    return {
        "value": cu / med,
        "unit": "cell-updates/s",
        "cores": cores,
        "kind": "port",
        "sample": f"one outer step {'fwd+bwd' if wl.backward else 'fwd'} of a {grid}^3 grid, "
                  f"batch {batch}, bs {wl.block_size}, inner {wl.inner} "
                  f"(median of {len(times)}, {med:.2f} s each)",
    }


def reference_benchmark_shape(steps, warmup):
    """The reference's own benchmark (gridnet/backend_cuda_test.py:155-206; it stores no result):
    32^3 grid, batch 2, 10 inner iterations, 8^3 blocks, normalize=True, silu, all parameters
    N(0, 1), ONE op call through the autograd wrapper with a synchronisation after every call, as
    its harness does -- forward alone, forward + backward, and the gated twin (leaky_relu)."""
    import torch

    from gridnet_amd.backend_cuda import GatedGridnetCudaOp, GridnetCudaOp

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    shape = (32, 32, 32)
    x = torch.randn(2, *shape, device=dev, requires_grad=True)
    w = torch.randn(27, *shape, device=dev, requires_grad=True)
    b = torch.randn(*shape, device=dev, requires_grad=True)
    r = torch.randn(*shape, device=dev, requires_grad=True)
    wg = torch.randn(27, 2, *shape, device=dev, requires_grad=True)
    bg = torch.randn(2, *shape, device=dev, requires_grad=True)
    gy = torch.randn_like(x)

    def fwd():
        with torch.no_grad():
            GridnetCudaOp.apply(w, b, r, x, 10, 8, 1e-5, True, "silu")
        torch.cuda.synchronize()

    def fwd_bwd():
        out = GridnetCudaOp.apply(w, b, r, x, 10, 8, 1e-5, True, "silu")
        torch.autograd.grad(out, (x, w, b, r), gy)
        torch.cuda.synchronize()

    def gated_fwd_bwd():
        out = GatedGridnetCudaOp.apply(wg, bg, x, 10, 8, "leaky_relu")
        torch.autograd.grad(out, (x, wg, bg), gy)
        torch.cuda.synchronize()

    def clock(fn):
        for _ in range(warmup):
            fn()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        return (time.perf_counter() - t0) / steps

    t_f, t_fb, t_g = clock(fwd), clock(fwd_bwd), clock(gated_fwd_bwd)
    cu = 2 * 32 ** 3 * 10
    a, p = 2 * 32 ** 3 * 4, 32 ** 3 * 4
    algo = (2 * a + 29 * p) + (3 * a + 58 * p)  # one step forward, one step backward
    print(json.dumps({
        "metric": "cell-updates/s fwd+bwd, reference benchmark shape 32^3 grid 8^3 blocks batch 2 inner 10 normalize",
        "value": cu / t_fb, "unit": "cell-updates/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": t_fb * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "R 32^3 bs8 B2 inner10 normalize silu: the reference's own benchmark "
                               "shape and harness (one op call, synchronised, through autograd)",
                   "pass": "fwd+bwd"},
        "forward_only_ms": t_f * 1e3, "gated_fwd_bwd_ms": t_g * 1e3,
        "hbm_roofline_frac_whole_step": algo / t_fb / (HBM_PEAK_GBS * 1e9),
        "note": "a 64-block grid and two samples: host- and latency-bound, not a throughput shape",
    }), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C3")
    ap.add_argument("--path", choices=("steps", "fused"), default="fused",
                    help="fused: the entry points with the LayerNorm folded into the step kernels "
                         "(the faster of the two on MI355X as measured); steps: one call per step "
                         "and per LayerNorm, as the reference's callers do")
    ap.add_argument("--normalize", action="store_true",
                    help="the workload with normalize=True (the reference's default, which its "
                         "training scripts switch off); op-by-op path")
    ap.add_argument("--chain-all", choices=("auto", "on", "off"), default="auto",
                    help="the backward of the whole chain in one launch of resident workgroups "
                         "(gridnet_hip_chain_backward_all): where it applies and fills the chip, "
                         "wherever it applies, never")
    ap.add_argument("--chain", choices=("auto", "on", "off"), default="auto",
                    help="the backward inside a chain as one kernel per step that hands the cross-block "
                         "values on (gridnet_hip_chain_backward) instead of two kernels per step: where the "
                         "library's row-wise cross-block kernel does not apply, wherever supported, never "
                         "(off also rules out --chain-all)")
    ap.add_argument("--outer-residual", action="store_true",
                    help="the other shape of the loop, n = norm(h); h = h + (net(n) - n) "
                         "(the reference's --outer_residual); fused entry points only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the HIP graph replay (for runs under a counter-collecting profiler)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no collectives, no sharding); "
                 "use --gpus 1")
    from gridnet_amd.configs import WORKLOADS

    if args.workload == "R":
        return reference_benchmark_shape(args.steps, args.warmup)
    wl = WORKLOADS[args.workload]
    if args.normalize:
        wl = dataclasses.replace(wl, normalize=True, name=wl.name + " normalize")
    if args.outer_residual:
        if args.path != "fused" or wl.normalize:
            sys.exit("bench.py: --outer-residual runs through the fused entry points (no --path steps, no --normalize)")
        wl = dataclasses.replace(wl, name=wl.name + " outer_residual")
    fused = args.path == "fused" and not wl.normalize and wl.inner >= 1
    wall, graph_s, kernel_s, one_launch = gpu_run(wl, args.steps, args.warmup, fused, not args.no_graph,
                                      {"auto": None, "on": True, "off": False}[args.chain_all],
                                      {"auto": None, "on": True, "off": False}[args.chain], args.outer_residual)
    bytes_ = wl.algorithmic_bytes()
    if fused:  # a fused entry point does the work of the step AND of the LayerNorm beside it
        bytes_["step_fwd"] += bytes_["ln_fwd"]
        bytes_["step_bwd"] += bytes_["ln_bwd"]
    # the one-launch chain backward takes all outer steps in ONE call
    steps_per_call = {"step_bwd": wl.outer} if one_launch else {}
    for k, n_steps in steps_per_call.items():
        bytes_[k] *= n_steps
    dominant = max(kernel_s, key=lambda k: kernel_s[k])
    # HBM bytes per call of that entry point and the counters of its main kernel, from the
    # committed rocprofv3 --pmc summaries (FETCH_SIZE and WRITE_SIZE scaled by a copy kernel of
    # known size); null if absent
    traffic, counters, counted_kernel, profile_source = None, {}, None, None
    try:
        with open(os.path.join(ROOT, "profiles", "counters.json")) as fh:
            variant = "normalize" if args.normalize else "fused" if fused else "steps"
            prof = json.load(fh).get(args.workload, {}).get(variant, {})
            traffic = prof.get("traffic_bytes_per_call", {}).get(dominant)
            counted_kernel = prof.get("dominant_kernel", {}).get(dominant)
            counters = prof.get("kernels", {}).get(counted_kernel, {})
            profile_source = prof.get("source")
    except OSError:
        pass
    # ceilings of this machine, measured now by the probe library (bench-only; a failure there
    # must not cost the headline, so a figure that cannot be measured is reported as null)
    import gc

    import torch
    gc.collect()
    torch.cuda.empty_cache()  # the copy probe wants 2 GiB of its own
    ceil, lds_widths = {}, {}
    try:
        from gridnet_amd import probe
        for k in probe.PROBES:
            try:
                ceil[k] = probe.probe(k)
            except RuntimeError as exc:
                print(f"bench.py: probe {k} failed: {exc}", file=sys.stderr, flush=True)
        for k in probe.LDS_WIDTH_PROBES:
            try:
                lds_widths[k] = probe.probe(k)
            except RuntimeError as exc:
                print(f"bench.py: probe {k} failed: {exc}", file=sys.stderr, flush=True)
    except (ImportError, OSError) as exc:
        print(f"bench.py: probe library unavailable: {exc}", file=sys.stderr, flush=True)
    clock = ceil.get("clock_ghz")
    lds_peak = None if clock is None else LDS_BYTES_PER_CLOCK_PER_CU * CUS * clock
    dom_s = kernel_s[dominant]
    achieved = bytes_[dominant] / dom_s / 1e9
    # the same entry point against the vector ALU: algorithmic fp32 FMAs per cell-update (27 for
    # the update itself; 81 in the backward: recompute, weight gradient, input gradient)
    fma = {"step_fwd": 27, "step_bwd": 81}.get(dominant)
    per_launch = wl.cell_updates / wl.outer * steps_per_call.get(dominant, 1)
    tflops = None if fma is None else 2 * fma * per_launch / dom_s / 1e12
    out = {
        "metric": "cell-updates/s fwd+bwd, 64^3 grid 8^3 blocks batch 32; % of HBM roofline",
        "value": wl.cell_updates / wall,
        "unit": "cell-updates/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": wl.name, "activation": wl.activation, "normalize": wl.normalize,
                   "pass": "fwd+bwd" if wl.backward else "fwd",
                   "path": ("fused step+LayerNorm entry points" + (", backward of the chain in one launch"
                                                                   if one_launch else ""))
                           if fused else "step and LayerNorm calls"},
        "timing": {"headline": "eager wall clock over the timed steps, synchronised on both sides",
                   "eager_ms_per_step": wall * 1e3,
                   "hip_graph_replay_ms_per_step": None if graph_s is None else graph_s * 1e3},
        "hbm_roofline_frac_whole_step": bytes_["total"] / wall / (HBM_PEAK_GBS * 1e9),
        "entry_point_ms": {k: v * 1e3 for k, v in kernel_s.items()},
        "roofline": {
            "bound": "hbm",
            "kernel": dominant,
            "outer_steps_per_call": steps_per_call.get(dominant, 1),
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_from_profile": profile_source,
        },
        # the same entry point against the vector ALU (fp32 FMAs without packed instructions) and
        # against the LDS pipes; the counter figures are those of the committed profile summary
        "vector_alu": {"kernel": dominant, "achieved": tflops, "unit": "TFLOP/s",
                       "peak": FP32_UNPACKED_PEAK_TFLOPS,
                       "frac": None if tflops is None else tflops / FP32_UNPACKED_PEAK_TFLOPS,
                       "measured_fma_ceiling": None if "fma_tfma_per_s" not in ceil else 2 * ceil["fma_tfma_per_s"],
                       "frac_of_measured_ceiling": None if tflops is None or "fma_tfma_per_s" not in ceil
                       else tflops / (2 * ceil["fma_tfma_per_s"]),
                       "valu_busy_pct": counters.get("valu_busy_pct"),
                       "from_profile": profile_source,
                       "peak_with_packed_fp32": FP32_PEAK_TFLOPS},
        "lds": {"kernel": counted_kernel, "unit": "GB/s", "from_profile": profile_source,
                "achieved": counters.get("lds_gb_per_s_estimate"),
                "peak": lds_peak,
                "frac": None if not counters or not lds_peak else counters["lds_gb_per_s_estimate"] / lds_peak,
                "busy_frac": counters.get("lds_busy_frac"),
                "bank_conflict_frac_of_busy": counters.get("lds_conflict_frac_of_busy"),
                "measured_read_ceiling": ceil.get("lds_gb_per_s"),
                "pipe_cycles_per_wave_read": lds_widths,
                "peak_is": "128 B per clock and CU x 256 CUs x the measured core clock; 16-byte reads go "
                           "beyond it on this part, see measured_read_ceiling"},
        "machine": {"core_clock_ghz_under_load": clock,
                    "hbm_copy_gb_per_s": ceil.get("copy_gb_per_s"),
                    "hbm_read_gb_per_s": ceil.get("read_gb_per_s")},
        "binds": what_binds(achieved / HBM_PEAK_GBS, counters.get("valu_busy_pct"), counters.get("lds_busy_frac")),
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
