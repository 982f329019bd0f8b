#!/usr/bin/env python3
"""Throughput of the permutohedral encoding hot path on one MI355X.

A step is one pass of the hot path over one batch of seeded synthetic points: forward plus backward
w.r.t. the table for the headline workload "c2" (3-D, 24 levels, capacity 2^18, 2^20 points), with
every input already resident in HBM.  Prints ONE JSON line:

  value        point-levels/s of the whole step (points * levels / step time)
  roofline     the dominant kernel against the HBM peak: algorithmic bytes per launch / its average
               duration, measured with events on the launch stream inside the timed loop
  cpu_baseline the CPU oracle (a scalar-code OpenMP port of the reference kernels) timed on this
               machine's host cores on a bounded sample of the same workload
  probes       measured streaming / random-gather / random-atomic rates of this GPU, which are what
               the table traffic is really bounded by; hbm_traffic_rate relates the measured HBM
               bytes of each phase to them

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth


def algorithmic_bytes(w):
    """Bytes per point-level each phase must move (fp32, 2 features); positions counted once per point."""
    d, l, c, n = w.pos_dim, w.nr_levels, w.capacity, w.nr_points
    pos = 4.0 * d / l
    return {
        "forward": 8 * (d + 1) + 8 + pos,
        "backward_table": 8 + pos + 8 * (d + 1) + 8.0 * c / n,
        "backward_pos": 8 + 8 * (d + 1) + 2 * pos,
        "double_backward": 8 + 2 * pos + 8 * (d + 1) + 8 * (d + 1) + 8 + 8.0 * c / n,
    }


def cpu_baseline(w, inputs, sample_points, reps=5):
    """Oracle forward + table backward (fp32, omp atomic) on the first `sample_points` points."""
    from oracle import api as orc
    n = min(sample_points, w.nr_points)
    pos = np.ascontiguousarray(inputs["pos"][:n])
    grad = np.ascontiguousarray(inputs["grad"][:, :, :n])
    sf = orc.scale_factors(w.pos_dim, inputs["sigmas"])
    times = []
    for rep in range(reps + 1):
        t0 = time.perf_counter()
        orc.forward(pos, inputs["table"], sf, inputs["shift"], inputs["window"])
        if "backward_table" in w.phases:
            orc.backward_table(pos, sf, inputs["shift"], inputs["window"], grad, w.capacity, want32=True, want64=False)
        dt = time.perf_counter() - t0
        if rep:  # first pass is the warm-up
            times.append(dt)
    med = float(np.median(times))
    return {
        "value": n * w.nr_levels / med,
        "unit": "point-levels/s",
        "cores": orc.num_threads(),
        "kind": "port",
        "sample": f"first {n} of {w.nr_points} points of workload {w.name}, all {w.nr_levels} levels, forward + table "
                  f"backward, median of {reps} after 1 warm-up ({med * 1e3:.1f} ms per pass)",
    }


def module_level(torch, w, inputs, steps, warmup):
    """The same step through the PyTorch module and autograd, as a user of the package pays it: output
    allocation, the (N, 2L) view, a row-major upstream gradient of shape (N, 2L) and, if the workload
    has them, position gradients.  Not part of `value`."""
    import permutohedral_encoding_amd as pe
    enc = pe.PermutoEncoding(w.pos_dim, w.capacity, w.nr_levels, 2, inputs["sigmas"])
    with torch.no_grad():
        enc.lattice_values.copy_(torch.from_numpy(inputs["table"]))
        enc.random_shift_per_level.copy_(torch.from_numpy(inputs["shift"]))
    pos = torch.from_numpy(inputs["pos"]).cuda()
    if "backward_pos" in w.phases:
        pos.requires_grad_(True)
    window = torch.from_numpy(inputs["window"]).cuda()
    upstream = torch.from_numpy(np.ascontiguousarray(inputs["grad"].transpose(2, 0, 1).reshape(w.nr_points, -1))).cuda()
    backward = any(p.startswith("backward") for p in w.phases)

    def step():
        if backward:
            enc(pos, window).backward(upstream)
            enc.lattice_values.grad = None
            pos.grad = None
        else:
            with torch.no_grad():
                enc(pos, window)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    return {"ms_per_step": ms, "point_levels_per_s": w.point_levels / (ms * 1e-3),
            "what": "PermutoEncoding forward" + (" + autograd backward from a row-major (N, 2L) upstream gradient" if backward else "")}


def run_probes(torch, native, capacity, n_threads, per_thread):
    """Streaming copy, random 8-byte gathers and random fp32 atomic pairs over one level-sized slice."""
    lib = native.lib()
    st = lambda: torch.cuda.current_stream().cuda_stream
    dev = "cuda"
    res = {}

    def timed(fn, iters=20):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e-3

    n4 = 1 << 26  # 1 GiB each way
    src = torch.empty(n4 * 4, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    t = timed(lambda: lib.penc_probe_copy(src.data_ptr(), dst.data_ptr(), n4, st()))
    res["copy_GBps"] = 2 * n4 * 16 / t / 1e9
    del src, dst

    g = torch.Generator(device=dev)
    g.manual_seed(0)
    idx = torch.randint(0, capacity, (per_thread, n_threads), dtype=torch.int32, device=dev, generator=g)
    table = torch.zeros(capacity * 2, dtype=torch.float32, device=dev)
    out = torch.empty(n_threads * 2, dtype=torch.float32, device=dev)
    t = timed(lambda: lib.penc_probe_gather(table.data_ptr(), idx.data_ptr(), n_threads, per_thread, out.data_ptr(), st()))
    res["gather_Gacc_per_s"] = n_threads * per_thread / t / 1e9
    t = timed(lambda: lib.penc_probe_scatter(table.data_ptr(), idx.data_ptr(), n_threads, per_thread, st()))
    res["scatter_Gatomic_per_s"] = 2 * n_threads * per_thread / t / 1e9
    res["slice_bytes"] = capacity * 8
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-probes", action="store_true", help="skip the memory-system probes")
    ap.add_argument("--no-module", action="store_true", help="skip the module-level (autograd) timing")
    ap.add_argument("--levels-per-pass", type=int, default=0,
                    help="levels binned per scatter pass (0: library default, -1: no workspace, direct atomics)")
    ap.add_argument("--cpu-sample", type=int, default=1 << 20, help="points in the CPU baseline sample")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on one GPU only; --gpus N with N > 1 is not supported", file=sys.stderr)
        sys.exit(2)

    import torch
    from permutohedral_encoding_amd import _native, workloads
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the encoding has no CPU path", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    w = workloads.WORKLOADS[args.workload]
    inputs = workloads.make_inputs(w)
    t = lambda a: torch.from_numpy(a).to(dev)
    fp = _native.EncodingFixedParams(w.pos_dim, w.capacity, w.nr_levels, 2, inputs["sigmas"], t(inputs["shift"]), False, 1.0)
    enc = _native.EncodingWrapper.create(w.pos_dim, 2, fp)
    want_table = "backward_table" in w.phases
    want_pos = "backward_pos" in w.phases
    want_double = "double_backward" in w.phases
    inp = _native.EncodingInput(t(inputs["table"]), t(inputs["pos"]), t(inputs["window"]), want_table, want_pos)
    grad = t(inputs["grad"])
    dpos = t(inputs["dpos"])

    # Output buffers are allocated once; the timed region calls the C ABI directly.
    lib = _native.lib()
    n, levels, cap, d = w.nr_points, w.nr_levels, w.capacity, w.pos_dim
    out = torch.empty((levels, 2, n), dtype=torch.float32, device=dev)
    tgrad = torch.empty((levels, cap, 2), dtype=torch.float32, device=dev) if (want_table or want_double) else None
    pgrad = torch.empty((n, d), dtype=torch.float32, device=dev) if want_pos else None
    ggs = torch.empty((levels, 2, n), dtype=torch.float32, device=dev) if want_double else None
    P = lambda x: None if x is None else x.data_ptr()
    sf, shift, win = fp.m_scale_factor, fp.m_random_shift_per_level, inp.m_anneal_window
    stream = torch.cuda.current_stream().cuda_stream

    def forward():
        rc = lib.penc_forward(d, 2, n, levels, cap, P(inp.m_positions_raw), P(inp.m_lattice_values), P(sf), P(shift),
                              P(win), P(out), 0, 1.0, stream)
        assert rc == 0, rc

    ws_bytes = 0
    if args.levels_per_pass >= 0:
        ws_bytes = max(int(lib.penc_scatter_workspace_bytes(d, n, levels, cap, args.levels_per_pass)),
                       int(lib.penc_positions_workspace_bytes(d, n, levels)))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None

    def backward():
        rc = lib.penc_backward(d, 2, n, levels, cap, P(inp.m_positions_raw), P(inp.m_lattice_values), P(sf), P(shift),
                               P(win), P(grad), P(tgrad) if want_table else None, P(pgrad), P(ws), ws_bytes, stream)
        assert rc == 0, rc

    def double_backward():
        rc = lib.penc_double_backward_from_positions(d, 2, n, levels, cap, P(inp.m_positions_raw),
                                                     P(inp.m_lattice_values), P(sf), P(shift), P(win), P(dpos), P(grad),
                                                     P(tgrad), P(ggs), 0, P(ws), ws_bytes, stream)
        assert rc == 0, rc

    phases = [("forward", forward)]
    if want_table or want_pos:
        phases.append(("backward", backward))
    if want_double:
        phases.append(("double_backward", double_backward))

    for _ in range(args.warmup):
        for _, fn in phases:
            fn()
    torch.cuda.synchronize()

    events = [[torch.cuda.Event(enable_timing=True) for _ in range(len(phases) + 1)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        events[k][0].record()
        for j, (_, fn) in enumerate(phases):
            fn()
            events[k][j + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    ms_per_step = elapsed / args.steps * 1e3
    phase_ms, phase_median, phase_min = {}, {}, {}
    for j, (name, _) in enumerate(phases):
        samples = [events[k][j].elapsed_time(events[k][j + 1]) for k in range(args.steps)]
        phase_ms[name] = float(np.mean(samples))
        phase_median[name] = float(np.median(samples))
        phase_min[name] = float(np.min(samples))

    ab = algorithmic_bytes(w)
    phase_bytes = {"forward": ab["forward"]}
    phase_bytes["backward"] = (ab["backward_table"] if want_table else 0.0) + (ab["backward_pos"] if want_pos else 0.0)
    phase_bytes["double_backward"] = ab["double_backward"]
    kernel_names = {"forward": "forward_kernel",
                    "backward": "+".join((["fill_zero_kernel", "backward_table_kernel", "bin_reduce_kernel"] if want_table else [])
                                         + (["backward_pos_kernel", "reduce_level_groups_kernel"] if want_pos else [])),
                    "double_backward": "grad_grad_kernel+fill_zero_kernel+backward_table_kernel<second order>+bin_reduce_kernel"}
    dominant = max(phase_ms, key=phase_ms.get)
    achieved = phase_bytes[dominant] * w.point_levels / (phase_ms[dominant] * 1e-3) / 1e9
    traffic = None
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            traffic = json.load(f).get(w.name, {}).get(dominant)
    roofline = {"bound": "hbm", "kernel": kernel_names[dominant], "achieved": achieved, "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic,
                "algorithmic_bytes_per_launch": phase_bytes[dominant] * w.point_levels,
                "avg_launch_ms": phase_ms[dominant]}

    result = {
        "metric": "encoded point-levels/sec fwd and fwd+bwd, 3D 24 lvl 2^20 pts; % of BW roofline",
        "value": w.point_levels / (ms_per_step * 1e-3),
        "unit": "point-levels/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: pos_dim={d} levels={levels} capacity=2^{cap.bit_length() - 1} feat=2 "
                               f"points=2^{n.bit_length() - 1} phases={'+'.join(p for p, _ in phases)}"},
        "phases_ms": phase_ms,
        "phases_ms_median": phase_median,
        "phases_ms_min": phase_min,
        "phases_point_levels_per_s": {k: w.point_levels / (v * 1e-3) for k, v in phase_ms.items()},
        "phases_algorithmic_GBps": {k: phase_bytes[k] * w.point_levels / (v * 1e-3) / 1e9 for k, v in phase_ms.items()},
        "roofline": roofline,
    }
    if not args.no_probes:
        result["probes"] = run_probes(torch, _native, cap, n, d + 1)
        pr = result["probes"]
        # The measured L2/MALL gather roofline: what the step would take if every one of the
        # N*L*(D+1) slot accesses of each table-touching phase (gather or scatter alike) ran at the
        # measured random 8-byte gather rate, plus the streaming traffic at the measured copy rate.
        # frac can exceed 1: the coarse levels hit caches better than the probe's uniform indices, and
        # the binned table backward replaces random slot accesses by streamed records.
        table_phases = sum(1 for name, _ in phases if name == "forward" or (name == "backward" and (want_table or want_pos))
                           or name == "double_backward") + (1 if ("backward", backward) in phases and want_table and want_pos else 0)
        bound_s = table_phases * w.point_levels * (d + 1) / (pr["gather_Gacc_per_s"] * 1e9)
        stream_bytes = sum(phase_bytes[name] - 8 * (d + 1) * (2 if name == "double_backward" else 1) for name, _ in phases) * w.point_levels
        bound_s += max(stream_bytes, 0.0) / (pr["copy_GBps"] * 1e9)
        result["measured_roofline"] = {"bound_ms": bound_s * 1e3, "frac": bound_s * 1e3 / ms_per_step,
                                       "note": "every table slot access at the probe's random-gather rate + streaming at "
                                               "the probe's copy rate; frac = bound / measured step"}
        # How fast the HBM traffic each phase really makes (hardware byte counters, scaled by the copy
        # probe, from profiles/) is moved, next to the rate the copy probe reaches for pure streaming.
        if os.path.exists(traffic_file):
            with open(traffic_file) as f:
                per_phase = json.load(f).get(w.name, {})
            result["hbm_traffic_rate"] = {
                "GBps": {k: per_phase[k] / (phase_ms[k] * 1e-3) / 1e9 for k in phase_ms if k in per_phase},
                "copy_probe_GBps": result["probes"]["copy_GBps"],
                "note": "measured HBM bytes per launch / measured phase time; the forward is bound by random 8-byte "
                        "gathers (see probes.gather_Gacc_per_s), the table backward by streaming its slot-range records",
            }
    if not args.no_module:
        result["module_level"] = module_level(torch, w, inputs, args.steps, args.warmup)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(w, inputs, args.cpu_sample)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
