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
  probes       measured streaming / random-gather / random-atomic rates of this GPU; the gather probe is
               swept over loads in flight per lane, workgroup size and load flavour, and the fastest
               setting found is the rate the gathers are priced at
  measured_roofline
               per phase, a lower bound of the phase's time built from measurements of this GPU in
               this run, with no term that depends on how the kernels are written: the slots every
               level really touches are replayed through the gather-only probe (its default and its
               fastest setting, whichever is quicker at that level, minus the same probe with all
               slots equal, which keeps its streaming but takes the gathers out), next to the time to
               stream the phase's compulsory bytes at the copy probe's rate; frac = bound / measured,
               at most 1.  `with_vector_issue` repeats it with the time to issue the kernels' own
               vector instructions as a third term: a diagnostic, not a bound of the problem
  hbm_traffic_rate
               HBM bytes per launch from hardware counters (profiles/hbm_traffic.json) / phase time

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-cpu]
"""
import argparse
import itertools
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth


def kernel_source_digest():
    """Identifies the kernel sources a counter summary was taken with (a summary of other sources is stale)."""
    import hashlib
    h = hashlib.sha1()
    csrc = os.path.join(ROOT, "permutohedral_encoding_amd", "csrc")
    for name in ("penc_kernels.hip", "penc_scatter.hpp", "penc_lattice.hpp"):
        with open(os.path.join(csrc, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def traffic_entry_matches(entry, kernels, second_order):
    """Whether a phase's entry of profiles/hbm_traffic.json was summed over exactly the kernels the phase
    launches (by name, the scattering kernel also by its second-order template argument) and its totals
    are the sums of its per-kernel rows."""
    rows = entry.get("per_kernel")
    if not isinstance(rows, dict) or sorted(rows) != sorted(entry.get("kernels", [])):
        return False
    if sorted(k.split("<")[0] for k in rows) != sorted(kernels):
        return False
    for k in rows:
        if k.startswith("backward_table_kernel<"):
            args = [a.strip() for a in k[k.index("<") + 1:k.rindex(">")].split(",")]
            if len(args) < 3 or (args[2] == "true") != second_order:
                return False
    total = sum(r["hbm_bytes"] for r in rows.values())
    return abs(total - entry["hbm_bytes"]) <= 1e-6 * max(total, 1.0)


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
    has them, position gradients and the double backward of an eikonal-style loss.  Not part of `value`."""
    import permutohedral_encoding_amd as pe
    enc = pe.PermutoEncoding(w.pos_dim, w.capacity, w.nr_levels, 2, inputs["sigmas"])
    with torch.no_grad():
        enc.lattice_values.copy_(torch.from_numpy(inputs["table"]))
        enc.random_shift_per_level.copy_(torch.from_numpy(inputs["shift"]))
    pos = torch.from_numpy(inputs["pos"]).cuda()
    sdf_like = "double_backward" in w.phases
    if sdf_like or "backward_pos" in w.phases:
        pos.requires_grad_(True)
    window = torch.from_numpy(inputs["window"]).cuda()
    upstream = torch.from_numpy(np.ascontiguousarray(inputs["grad"].transpose(2, 0, 1).reshape(w.nr_points, -1))).cuda()
    q = torch.from_numpy(inputs["dpos"]).cuda()
    backward = any(p.startswith("backward") for p in w.phases)

    def step():
        if sdf_like:
            out = enc(pos, window)
            grad_pos, = torch.autograd.grad(out, pos, upstream, create_graph=True)
            (grad_pos * q).sum().backward()
        elif backward:
            enc(pos, window).backward(upstream)
        else:
            with torch.no_grad():
                enc(pos, window)
        enc.lattice_values.grad = None
        pos.grad = None

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    what = "PermutoEncoding forward"
    if sdf_like:
        what += " + autograd.grad w.r.t. positions (create_graph) from a row-major (N, 2L) upstream gradient + backward of <grad_pos, q>"
    elif backward:
        what += " + autograd backward from a row-major (N, 2L) upstream gradient"
    return {"ms_per_step": ms, "point_levels_per_s": w.point_levels / (ms * 1e-3), "what": what}


def optimizer_leg(torch, lib, w, table, tgrad, touched, run_gradients, clear_touched):
    """The optimizer step on the workload's table after its gradient calls: torch.optim.AdamW (every entry of
    the table, several kernels), penc_adamw_step with skip_zero_gradients (one kernel that reads the whole
    gradient) and penc_adamw_step_sparse (the slot ranges the gradient calls marked, nothing else).  Each is
    timed alone, on the gradient one step leaves; the sparse one is re-armed by repeating the gradient calls
    outside its timing.  Not part of `value`."""
    from permutohedral_encoding_amd.optim import AdamW
    st = torch.cuda.current_stream().cuda_stream
    kw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    res = {}
    run_gradients()
    dense_grad = tgrad.clone()
    for name, make in (("torch_adamw_ms", lambda p: torch.optim.AdamW([p], **kw)),
                       ("fused_adamw_skip_zero_ms", lambda p: AdamW([p], skip_zero_gradients=True, **kw))):
        p = torch.nn.Parameter(table.clone())
        p.grad = dense_grad
        opt = make(p)
        res[name] = _timed(torch, opt.step, iters=5, warm=2) * 1e3
        del opt, p
    p, m, v = table.clone(), torch.zeros_like(table), torch.zeros_like(table)
    times = []
    for k in range(6):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc = lib.penc_adamw_step_sparse(p.data_ptr(), tgrad.data_ptr(), m.data_ptr(), v.data_ptr(), 2, w.nr_levels, w.capacity,
                                        touched.data_ptr(), 1e-3, 0.9, 0.999, 1e-8, 0.0, k + 1, 1, st)
        e1.record()
        assert rc == 0, rc
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
        run_gradients()
    clear_touched()
    res["sparse_adamw_ms"] = float(np.median(times[1:]))
    res["touched_fraction_of_slot_ranges"] = None
    return res


def _timed(torch, fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def run_probes(torch, capacity, n_threads, per_thread):
    """Streaming copy, random 8-byte gathers and random fp32 atomic pairs over one level-sized slice."""
    from permutohedral_encoding_amd import probes
    lib = probes.lib()
    st = lambda: torch.cuda.current_stream().cuda_stream
    dev = "cuda"
    res = {}
    n4 = 1 << 26  # 1 GiB each way
    src = torch.empty(n4 * 4, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    t = _timed(torch, lambda: lib.penc_probe_copy(src.data_ptr(), dst.data_ptr(), n4, st()))
    res["copy_GBps"] = 2 * n4 * 16 / t / 1e9
    sink = torch.zeros(16384, dtype=torch.float32, device=dev)
    t = _timed(torch, lambda: lib.penc_probe_read(src.data_ptr(), n4, sink.data_ptr(), st()))
    res["read_GBps"] = n4 * 16 / t / 1e9
    del src, dst

    g = torch.Generator(device=dev)
    g.manual_seed(0)
    idx = torch.randint(0, capacity, (per_thread, n_threads), dtype=torch.int32, device=dev, generator=g)
    table = torch.zeros(capacity * 2, dtype=torch.float32, device=dev)
    out = torch.empty(n_threads * 2, dtype=torch.float32, device=dev)
    t = _timed(torch, lambda: lib.penc_probe_gather(table.data_ptr(), idx.data_ptr(), n_threads, per_thread, out.data_ptr(), st()))
    res["gather_Gacc_per_s"] = n_threads * per_thread / t / 1e9
    # Is that probe a ceiling?  The same gathers with 1, 2 or 4 points per lane (K, 2K, 4K loads in flight),
    # workgroups of 64 to 1024 threads, and ordinary, non-temporal and raw-buffer loads with each cache policy.
    sweep = []
    if per_thread in GATHER_VARIANT_K and n_threads % 4 == 0:
        for points, block, kind in itertools.product((1, 2, 4), (64, 256, 1024), sorted(GATHER_LOAD_KINDS)):
            call = lambda: lib.penc_probe_gather_variant(table.data_ptr(), capacity, idx.data_ptr(), n_threads, per_thread, points,
                                                         block, kind, out.data_ptr(), st())
            assert call() == 0
            sweep.append((_timed(torch, call, iters=10, warm=2), points, block, kind))
        sweep.sort()
        best = sweep[0]
        res["gather_sweep"] = {
            "best_Gacc_per_s": n_threads * per_thread / best[0] / 1e9,
            "best": {"points_per_lane": best[1], "block_threads": best[2], "load": GATHER_LOAD_KINDS[best[3]]},
            "worst_Gacc_per_s": n_threads * per_thread / sweep[-1][0] / 1e9,
            "best_per_load_Gacc_per_s": {GATHER_LOAD_KINDS[k]: n_threads * per_thread / min(t for t, _, _, kk in sweep if kk == k) / 1e9
                                          for k in sorted(GATHER_LOAD_KINDS)},
            "settings_tried": len(sweep),
        }
        res["gather_best_variant"] = list(best[1:])
    t = _timed(torch, lambda: lib.penc_probe_scatter(table.data_ptr(), idx.data_ptr(), n_threads, per_thread, st()))
    res["scatter_Gatomic_per_s"] = 2 * n_threads * per_thread / t / 1e9
    res["slice_bytes"] = capacity * 8
    return res


GATHER_VARIANT_K = (4, 5, 9)  # gathers per point the variant probe is built for (pos_dim 3, 4 and 8)
GATHER_LOAD_KINDS = {0: "global_load", 1: "global_load nt (compiler's non-temporal)", 2: "buffer_load", 3: "buffer_load sc0",
                     4: "buffer_load nt", 18: "buffer_load sc1", 19: "buffer_load sc0 sc1"}


def gather_pattern_seconds(torch, native, w, fp, table, pos, variant=None):
    """Per level: what the D+1 gathers per point cost on this memory system for the slots the workload
    really touches.  The slots (penc_simplex_debug, the forward's own device routine) are replayed
    through the gather-only probe; the same probe with every slot equal to 0 has the same streaming
    traffic (index reads, one store per point) but cache-resident gathers, and is subtracted.  With
    `variant` (points per lane, workgroup size, load flavour: the fastest setting of the sweep) every
    level is replayed through that setting as well and the quicker of the two counts."""
    from permutohedral_encoding_amd import probes
    lib, plib = native.lib(), probes.lib()
    st = torch.cuda.current_stream().cuda_stream
    n, d, levels, cap = w.nr_points, w.pos_dim, w.nr_levels, w.capacity
    out = torch.empty(n * 2, dtype=torch.float32, device="cuda")
    zeros = torch.zeros((d + 1, n), dtype=torch.int32, device="cuda")
    level_table = table[0]
    run_default = lambda idx_: plib.penc_probe_gather(level_table.data_ptr(), idx_.data_ptr(), n, d + 1, out.data_ptr(), st)
    run_variant = None
    if variant is not None:
        run_variant = lambda idx_: plib.penc_probe_gather_variant(level_table.data_ptr(), cap, idx_.data_ptr(), n, d + 1, variant[0],
                                                                  variant[1], variant[2], out.data_ptr(), st)
    slot = torch.empty((1, n, d + 1), dtype=torch.int32, device="cuda")
    real, real_variant, zero, zero_variant = [], [], [], []
    for l in range(levels):
        rc = lib.penc_simplex_debug(d, n, 1, cap, pos.data_ptr(), fp.m_scale_factor[l:l + 1].contiguous().data_ptr(),
                                    fp.m_random_shift_per_level[l:l + 1].contiguous().data_ptr(), 1, None, None,
                                    slot.data_ptr(), None, st)
        assert rc == 0, rc
        idx = slot[0].t().contiguous()
        level_table = table[l]
        real.append(_timed(torch, lambda: run_default(idx), iters=10))
        # the all-hit run is repeated beside every level and its median is what is subtracted: taken once, its
        # half-microsecond scatter would shift every level of the bound the same way
        zero.append(_timed(torch, lambda: run_default(zeros), iters=10))
        if run_variant is not None:
            real_variant.append(_timed(torch, lambda: run_variant(idx), iters=10))
            zero_variant.append(_timed(torch, lambda: run_variant(zeros), iters=10))
    t_zero = float(np.median(zero))
    result = [max(t - t_zero, 0.0) for t in real]
    if run_variant is not None:
        t_zero_variant = float(np.median(zero_variant))
        result = [min(c, max(t - t_zero_variant, 0.0)) for c, t in zip(result, real_variant)]
    return result, t_zero


VALU_WAVE_INSTR_PER_S = 256 * 4 * 2.4e9 / 4  # 256 CUs x 4 SIMDs, one wave64 vector instruction per 4 clocks at 2.4 GHz


def measured_roofline(w, phases, window, gather_s, copy_GBps, valu_per_point_level):
    """Lower bound per phase = sum over levels of max(gather pattern, compulsory streaming).  Both terms
    are properties of the problem on this memory system, so the sum is a bound for any implementation.
    With `valu_per_point_level` (the shipped kernels' own instruction counts) the time to issue those
    instructions is a third term: that figure describes the kernels, not the problem."""
    d, l, c, n = w.pos_dim, w.nr_levels, w.capacity, w.nr_points
    copy = copy_GBps * 1e9
    pos_bytes = 4.0 * d * n / l
    out = {}
    for name, _ in phases:
        if name == "clear_touched":  # bookkeeping of the sparse table gradient: no bound of its own
            out[name] = 0.0
            continue
        # (slot-access passes over the table, streamed bytes per level) of the phase
        if name == "forward":
            passes, stream = 1, 8.0 * n + pos_bytes
        elif name == "backward":
            has_table, has_pos = "backward_table" in w.phases, "backward_pos" in w.phases
            passes = int(has_table) + int(has_pos)
            stream = (8.0 * n + pos_bytes) * passes + (8.0 * c if has_table else 0.0) + (4.0 * d * n / l if has_pos else 0.0)
        else:
            passes, stream = 2, 2 * (8.0 * n + 2 * pos_bytes) + 8.0 * n + 8.0 * c
        valu = valu_per_point_level.get(name)
        total = 0.0
        for level in range(l):
            if window[level] == 0.0:
                total += (8.0 * n / copy) if name == "forward" else 0.0   # masked levels still store their zeros
                continue
            terms = [passes * gather_s[level], stream / copy]
            if valu:
                terms.append(valu * n / 64.0 / VALU_WAVE_INSTR_PER_S)
            total += max(terms)
        out[name] = total * 1e3
    return out


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
    ap.add_argument("--sparse-table-grad", action="store_true",
                    help="table gradients through the sparse entry points: both gradient calls add into one array kept across "
                         "steps and mark the slot ranges they touch, and the step ends by clearing what was touched "
                         "(penc_clear_touched) instead of each call clearing a dense gradient first")
    ap.add_argument("--optimizer", action="store_true",
                    help="with --sparse-table-grad: also time the optimizer step on the table (torch AdamW, fused, sparse)")
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

    sparse = args.sparse_table_grad and (want_table or want_double)
    touched = None
    if sparse:
        tgrad.zero_()
        touched = torch.zeros(int(lib.penc_touched_map_entries(2, levels, cap)), dtype=torch.int32, device=dev)

    def backward():
        if sparse and want_table:
            rc = lib.penc_backward_sparse(d, 2, n, levels, cap, P(inp.m_positions_raw), P(inp.m_lattice_values), P(sf), P(shift),
                                          P(win), P(grad), 0, P(tgrad), P(touched), P(pgrad), P(ws), ws_bytes, stream)
        else:
            rc = lib.penc_backward(d, 2, n, levels, cap, P(inp.m_positions_raw), P(inp.m_lattice_values), P(sf), P(shift),
                                   P(win), P(grad), P(tgrad) if want_table else None, P(pgrad), P(ws), ws_bytes, stream)
        assert rc == 0, rc

    def double_backward():
        if sparse:
            rc = lib.penc_double_backward_from_positions_sparse(d, 2, n, levels, cap, P(inp.m_positions_raw),
                                                                P(inp.m_lattice_values), P(sf), P(shift), P(win), P(dpos),
                                                                P(grad), 0, P(tgrad), P(touched), P(ggs), 0, P(ws), ws_bytes, stream)
        else:
            rc = lib.penc_double_backward_from_positions(d, 2, n, levels, cap, P(inp.m_positions_raw),
                                                         P(inp.m_lattice_values), P(sf), P(shift), P(win), P(dpos), P(grad),
                                                         P(tgrad), P(ggs), 0, P(ws), ws_bytes, stream)
        assert rc == 0, rc

    def clear_touched():
        rc = lib.penc_clear_touched(P(tgrad), 2, levels, cap, P(touched), stream)
        assert rc == 0, rc

    phases = [("forward", forward)]
    if want_table or want_pos:
        phases.append(("backward", backward))
    if want_double:
        phases.append(("double_backward", double_backward))
    if sparse:
        phases.append(("clear_touched", clear_touched))

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
    phase_bytes["clear_touched"] = 0.0  # bookkeeping of the sparse table gradient: no algorithmic bytes of its own
    # tables with more than 64 slot ranges of 8192 slots are reduced by workgroups that walk several levels
    reducer = "bin_reduce_levels_kernel" if w.capacity > 64 * 8192 else "bin_reduce_kernel"
    phase_kernels = {"forward": ["forward_kernel"],
                     "backward": (["fill_zero_kernel", "backward_table_kernel", reducer] if want_table else [])
                                 + (["backward_pos_kernel", "reduce_level_groups_kernel"] if want_pos else []),
                     "double_backward": ["grad_grad_kernel", "fill_zero_kernel", "backward_table_kernel", reducer]}
    phase_kernels["clear_touched"] = ["touched_ranges_kernel"]
    if sparse:  # nothing is cleared before the scatter
        for name in ("backward", "double_backward"):
            phase_kernels[name] = [k for k in phase_kernels[name] if k != "fill_zero_kernel"]
    kernel_names = {k: "+".join(v) for k, v in phase_kernels.items()}
    kernel_names["double_backward"] = kernel_names["double_backward"].replace("backward_table_kernel", "backward_table_kernel<second order>")
    dominant = max(phase_ms, key=phase_ms.get)
    achieved = phase_bytes[dominant] * w.point_levels / (phase_ms[dominant] * 1e-3) / 1e9
    # HBM bytes per launch and vector instructions per point-level come from the committed counter
    # summaries (profiles/hbm_traffic.json, written from rocprofv3 --pmc runs of this script); an entry
    # taken with other kernels than the ones this phase launches now is stale and is not used.
    per_phase, valu_per_point_level = {}, {}
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    traffic_note = "no counter summary for this workload under profiles/"
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            recorded = json.load(f)
        if recorded.get("source_digest") != kernel_source_digest():
            traffic_note = "profiles/hbm_traffic.json was taken with other kernel sources (stale): not used"
            recorded = {}
        elif w.name in recorded:
            traffic_note = f"profiles/hbm_traffic.json, commit {recorded.get('commit', '?')}"
        recorded = recorded.get(w.name, {})
        for name in phase_ms:
            entry = recorded.get(name)
            if entry and traffic_entry_matches(entry, phase_kernels[name], second_order=name == "double_backward"):
                per_phase[name] = entry["hbm_bytes"]
                if entry.get("valu_wave_instr"):
                    valu_per_point_level[name] = entry["valu_wave_instr"] * 64.0 / w.point_levels
            elif entry:
                traffic_note += f"; the entry for {name} does not cover the kernels this phase launches: not used"
    roofline = {"bound": "hbm", "kernel": kernel_names[dominant], "achieved": achieved, "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": per_phase.get(dominant),
                "traffic_source": traffic_note,
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
                               f"points=2^{n.bit_length() - 1} phases={'+'.join(p for p, _ in phases)}"
                               + (" (sparse table gradient)" if sparse else "")},
        "phases_ms": phase_ms,
        "phases_ms_median": phase_median,
        "phases_ms_min": phase_min,
        "phases_point_levels_per_s": {k: w.point_levels / (v * 1e-3) for k, v in phase_ms.items()},
        "phases_algorithmic_GBps": {k: phase_bytes[k] * w.point_levels / (v * 1e-3) / 1e9 for k, v in phase_ms.items()},
        "roofline": roofline,
    }
    if not args.no_probes:
        result["probes"] = run_probes(torch, cap, n, d + 1)
        pr = result["probes"]
        gather_s, t_zero = gather_pattern_seconds(torch, _native, w, fp, inp.m_lattice_values, inp.m_positions_raw,
                                                  pr.pop("gather_best_variant", None))
        bound_ms = measured_roofline(w, phases, inputs["window"], gather_s, pr["copy_GBps"], {})
        result["measured_roofline"] = {
            "bound_ms": bound_ms,
            "frac": {k: bound_ms[k] / phase_ms[k] for k in bound_ms},
            "step_bound_ms": sum(bound_ms.values()),
            "step_frac": sum(bound_ms.values()) / sum(phase_ms.values()),
            "gather_pattern_us_per_level": [round(x * 1e6, 2) for x in gather_s],
            "note": "per level max(replay of the level's own slots through the gather-only probe, at its default or at the "
                    "fastest setting of the sweep, minus the same probe with all slots equal; compulsory bytes at the copy "
                    "probe's rate), summed over the levels; a table gradient or second table pass counts its slot accesses "
                    "like gathers; frac = bound / measured phase time",
        }
        if valu_per_point_level:
            with_valu = measured_roofline(w, phases, inputs["window"], gather_s, pr["copy_GBps"], valu_per_point_level)
            result["measured_roofline"]["with_vector_issue"] = {
                "bound_ms": with_valu,
                "frac": {k: with_valu[k] / phase_ms[k] for k in with_valu},
                "step_frac": sum(with_valu.values()) / sum(phase_ms.values()),
                "note": "the same with a third term per level: the shipped kernels' own vector instructions (hardware counter) at "
                        "one per 4 clocks per SIMD.  It describes the kernels, not the problem: a kernel that issues more "
                        "instructions raises it.  Diagnostic only.",
            }
        if per_phase:
            result["hbm_traffic_rate"] = {
                "GBps": {k: per_phase[k] / (phase_ms[k] * 1e-3) / 1e9 for k in phase_ms if k in per_phase},
                "copy_probe_GBps": pr["copy_GBps"],
                "read_probe_GBps": pr["read_GBps"],
                "note": "bytes through the L2's memory-side port per launch from hardware counters (profiles/) / measured phase "
                        "time; a phase that mostly reads is bounded by the read probe, one that reads and writes alike by the "
                        "copy probe; part of the traffic of a table larger than the L2 is served by the memory-side cache",
            }
    if sparse and args.optimizer:
        def run_gradients():
            for name, fn in phases:
                if name in ("backward", "double_backward"):
                    fn()
        run_gradients()
        marked = float((touched != 0).float().mean().item())
        clear_touched()
        result["optimizer_step"] = optimizer_leg(torch, lib, w, inp.m_lattice_values, tgrad, touched, run_gradients, clear_touched)
        result["optimizer_step"]["touched_fraction_of_slot_ranges"] = marked
    if not args.no_module:
        result["module_level"] = module_level(torch, w, inputs, args.steps, args.warmup)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(w, inputs, args.cpu_sample)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
