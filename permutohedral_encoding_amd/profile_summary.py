"""Turns raw rocprofv3 output of ``bench.py`` runs into the short summaries kept under ``profiles/``.

For a workload ``<wl>`` the raw files are expected under ``gpurun_out/prof_<wl>/`` as written by the
commands the summaries quote (one ``--kernel-trace --stats`` run into ``trace/`` with bench.py's
output in ``trace.log``, and one ``--pmc`` run per counter set into ``fetch/``, ``write/``, ``tcc/``,
``tcp/``, ``sq/`` and, optionally, ``ea/``).  Written from them:

  profiles/<wl>_kernel_trace.md   per-kernel durations
  profiles/<wl>_counters.md       per phase of bench.py and kernel: bytes that crossed the L2's
                                  memory-side port (FETCH_SIZE / WRITE_SIZE), L2 requests and hit rate,
                                  L1->L2 requests, vector and LDS instructions, LDS bank conflicts
  profiles/hbm_traffic.json       per workload and phase the sums of those rows, with the rows
                                  themselves, which is what bench.py reads

A dispatch belongs to a phase by what it is, not by its position in a name list: the scattering
kernel by its second-order template argument, the kernels that serve both gradient calls (the
fill that clears the gradient, the bin reducers) by the scattering kernel they precede or follow
in the dispatch order.

Usage: python -m permutohedral_encoding_amd.profile_summary c2 [c3 ...]   (from the repository root)
"""
import collections
import csv
import glob
import json
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROFILES = os.path.join(ROOT, "profiles")

DESCRIPTION = {
    "c2": "forward + table backward",
    "c3": "forward + position backward + double backward",
    "c4": "forward + table backward (pos_dim 8)",
    "c5": "forward + table and position backward + double backward (2^22-slot table, top 8 levels masked)",
}
COUNTER_SETS = (
    ("fetch", "", "FETCH_SIZE"),
    ("write", "", "WRITE_SIZE"),
    ("tcc", " --no-probes", "TCC_HIT_sum TCC_MISS_sum TCC_REQ_sum TCC_ATOMIC_sum"),
    ("tcp", " --no-probes", "TCP_TCC_READ_REQ_sum TCP_TCC_WRITE_REQ_sum TCP_TCC_ATOMIC_WITHOUT_RET_REQ_sum TCP_TOTAL_CACHE_ACCESSES_sum"),
    ("sq", " --no-probes", "SQ_WAVES SQ_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_LDS SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT"),
    ("ea", " --no-probes", "TCC_EA0_RDREQ_sum TCC_EA0_RDREQ_32B_sum TCC_EA0_WRREQ_sum TCC_EA0_WRREQ_64B_sum"),
)
L2_LINE_BYTES = 128        # gfx950: an L2 request from the first-level cache moves at most one 128-byte line
SHARED = ("fill_zero_kernel", "bin_reduce_kernel", "bin_reduce_levels_kernel", "touched_")


def short(name):
    """Kernel name without namespaces, return type and argument list."""
    name = name.replace("(anonymous namespace)::", "").replace("void ", "").replace("penc::", "")
    depth = 0
    for i, ch in enumerate(name):  # cut at the argument list's parenthesis, not at one inside the template arguments
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            return name[:i]
    return name


def base_name(kernel):
    return kernel.split("<")[0]


def template_args(kernel):
    m = re.search(r"<(.*)>", kernel)
    return [a.strip() for a in m.group(1).split(",")] if m else []


def is_ours(kernel):
    return not ("at::" in kernel or "rocclr" in kernel or "copy_kernel" in kernel or "gather_" in kernel
                or "scatter_kernel" in kernel or "simplex_debug" in kernel)


def phase_of_dispatches(kernels):
    """Phase ("forward", "backward", "double_backward" or None) of every dispatch of a run, in order."""
    own = []
    for k in kernels:
        b = base_name(k)
        if not is_ours(k):
            own.append(None)
        elif b == "forward_kernel":
            own.append("forward")
        elif b in ("backward_pos_kernel", "reduce_level_groups_kernel", "transpose_kernel"):
            own.append("backward")
        elif b == "grad_grad_kernel":
            own.append("double_backward")
        elif b == "touched_ranges_kernel":
            own.append("clear_touched")
        elif b == "backward_table_kernel":
            args = template_args(k)  # <D, kRowMajor, kSecondOrder, kWideBins>
            own.append("double_backward" if len(args) >= 3 and args[2] == "true" else "backward")
        else:
            own.append("?")  # serves whichever gradient call launched it
    scatter_at = [i for i, k in enumerate(kernels) if base_name(k) == "backward_table_kernel"]
    for i, k in enumerate(kernels):
        if own[i] != "?":
            continue
        if base_name(k) == "fill_zero_kernel":   # clears the gradient before the scatter
            after = [j for j in scatter_at if j > i]
            own[i] = own[after[0]] if after else None
        else:                                     # reduces what the scatter left
            before = [j for j in scatter_at if j < i]
            own[i] = own[before[-1]] if before else None
    return own


def read_counters(base, name):
    """{(phase, kernel): {counter: average per dispatch}} of one counter run, or {} if the run is absent."""
    files = glob.glob(os.path.join(base, name, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        return {}
    per_dispatch = collections.OrderedDict()
    for r in csv.DictReader(open(files[0])):
        key = int(r["Dispatch_Id"])
        per_dispatch.setdefault(key, {"kernel": short(r["Kernel_Name"]), "values": {}})
        per_dispatch[key]["values"][r["Counter_Name"]] = per_dispatch[key]["values"].get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    order = sorted(per_dispatch)
    kernels = [per_dispatch[i]["kernel"] for i in order]
    phases = phase_of_dispatches(kernels)
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    copy = collections.defaultdict(list)
    for i, ph, k in zip(order, phases, kernels):
        for c, v in per_dispatch[i]["values"].items():
            if k.startswith("copy_kernel"):  # the probe library's own, not torch's copy kernels
                copy[c].append(v)
            if ph is not None:
                agg[(ph, k)][c].append(v)
    out = {key: {c: sum(v) / len(v) for c, v in d.items()} for key, d in agg.items()}
    out["__copy__"] = {c: sum(v) / len(v) for c, v in copy.items()}
    return out


def read_trace(base):
    """{(phase, kernel): average microseconds} from the kernel trace, and bench.py's own line of that run."""
    files = glob.glob(os.path.join(base, "trace", "**", "*kernel_trace.csv"), recursive=True)
    rows = sorted(csv.DictReader(open(files[0])), key=lambda r: int(r["Start_Timestamp"]))
    kernels = [short(r["Kernel_Name"]) for r in rows]
    phases = phase_of_dispatches(kernels)
    agg = collections.defaultdict(list)
    for r, ph, k in zip(rows, phases, kernels):
        if ph is not None:
            agg[(ph, k)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    bench = json.loads([l for l in open(os.path.join(base, "trace.log")) if l.startswith("{")][-1])
    return {k: (sum(v) / len(v), min(v), max(v), len(v)) for k, v in agg.items()}, bench


def summarise(wl, digest, commit):
    """`wl` is a workload of bench.py, or `<workload>_sparse` for its run with --sparse-table-grad (kernel trace only)."""
    base = os.path.join(ROOT, "gpurun_out", f"prof_{wl}")
    trace, bench = read_trace(base)
    wl_name, _, variant = wl.partition("_")
    flag = " --sparse-table-grad" if variant == "sparse" else ""
    with open(os.path.join(PROFILES, f"{wl}_kernel_trace.md"), "w") as f:
        f.write(f"# Kernel trace: bench.py, workload {wl_name}{' with the sparse table gradient' if flag else ''} ({DESCRIPTION[wl_name]}), one MI355X\n\n")
        f.write("Command (from the repository root on the GPU box, after `cd /tmp && export TMPDIR=/tmp && cd -`):\n\n")
        f.write(f"    rocprofv3 --kernel-trace --stats -f csv -d gpurun_out/prof_{wl}/trace -o run -- python3 bench.py --workload {wl_name}{flag} --no-cpu --no-probes --no-module --steps 20 --warmup 5\n\n")
        f.write(f"Per phase of bench.py and kernel, over the run's dispatches (5 warm-up + 20 timed steps); kernel sources {digest} (commit {commit}):\n\n")
        f.write("| phase | kernel | calls | average (us) | min (us) | max (us) |\n|---|---|---|---|---|---|\n")
        for (ph, k), (avg, lo, hi, n) in sorted(trace.items(), key=lambda kv: (kv[0][0], -kv[1][0])):
            f.write(f"| {ph} | `{k}` | {n} | {avg:.1f} | {lo:.1f} | {hi:.1f} |\n")
        f.write(f"\nbench.py's own event timing in the same run: phases_ms = {json.dumps({k: round(v, 4) for k, v in bench['phases_ms'].items()})}, ms_per_step = {bench['ms_per_step']:.4f}.\n")

    if variant:
        return None  # a variant run has a kernel trace only
    sets = {name: read_counters(base, name) for name, _, _ in COUNTER_SETS}
    fetch, write, tcc, tcp, sq, ea = (sets[n] for n in ("fetch", "write", "tcc", "tcp", "sq", "ea"))
    known_kib = (1 << 30) / 1024.0  # the copy probe moves 1 GiB each way
    fs = known_kib / fetch["__copy__"]["FETCH_SIZE"] if fetch.get("__copy__", {}).get("FETCH_SIZE") else 2.0
    ws = known_kib / write["__copy__"]["WRITE_SIZE"] if write.get("__copy__", {}).get("WRITE_SIZE") else 1.0
    rows = {}
    for key in fetch:
        if key == "__copy__" or key not in tcc:
            continue
        rd = fetch[key]["FETCH_SIZE"] * fs * 1024.0
        wr = write.get(key, {}).get("WRITE_SIZE", 0.0) * ws * 1024.0
        t, p, q, e = tcc[key], tcp.get(key, {}), sq.get(key, {}), ea.get(key, {})
        us = trace.get(key, (float("nan"),))[0]
        rows[key] = {
            "us": us, "read_bytes": rd, "written_bytes": wr, "hbm_bytes": rd + wr,
            "l2_requests": t["TCC_REQ_sum"], "l2_hit_rate": t["TCC_HIT_sum"] / max(t["TCC_HIT_sum"] + t["TCC_MISS_sum"], 1.0),
            "l2_atomics": t["TCC_ATOMIC_sum"],
            "l1_l2_reads": p.get("TCP_TCC_READ_REQ_sum", 0.0), "l1_l2_writes": p.get("TCP_TCC_WRITE_REQ_sum", 0.0),
            "l1_l2_atomics": p.get("TCP_TCC_ATOMIC_WITHOUT_RET_REQ_sum", 0.0),
            "valu_wave_instr": q.get("SQ_INSTS_VALU", 0.0), "lds_wave_instr": q.get("SQ_INSTS_LDS", 0.0),
            "lds_bank_conflict_cycles": q.get("SQ_LDS_BANK_CONFLICT", 0.0),
            "ea_read_requests": e.get("TCC_EA0_RDREQ_sum"), "ea_read_requests_32B": e.get("TCC_EA0_RDREQ_32B_sum"),
            "ea_write_requests": e.get("TCC_EA0_WRREQ_sum"), "ea_write_requests_64B": e.get("TCC_EA0_WRREQ_64B_sum"),
        }
    with open(os.path.join(PROFILES, f"{wl}_counters.md"), "w") as f:
        f.write(f"# Hardware counters per dispatch: bench.py, workload {wl} ({DESCRIPTION[wl]}), one MI355X\n\n")
        f.write("One rocprofv3 run per counter set (from the repository root on the GPU box):\n\n")
        for name, extra, ctrs in COUNTER_SETS:
            if sets[name]:
                f.write(f"    rocprofv3 --pmc {ctrs} -f csv -d gpurun_out/prof_{wl}/{name} -o run -- python3 bench.py --workload {wl} --no-cpu --no-module{extra} --steps 3 --warmup 1\n")
        f.write(f"\nKernel sources {digest} (commit {commit}). Averages over the dispatches of each kernel within each phase of bench.py "
                "(a kernel that serves two gradient calls has a row per phase). FETCH_SIZE and WRITE_SIZE count what crosses the L2's "
                "memory-side port, in units the 1 GiB copy probe (`copy_kernel`) of the same run calibrates: "
                f"x{fs:.3f} KiB (fetch) and x{ws:.3f} KiB (write). That port leads to the memory-side cache (256 MB) and through it to "
                "the HBM; the memory-side cache has no counter rocprofv3 exposes on this GPU, so \"memory-side\" bytes below are an upper "
                "bound of the HBM bytes, and its hit rate is not observable here. L2 bytes/s = L2 requests x 128 bytes (one line at most "
                "per request) / duration: an upper bound of what the L2 delivered.\n\n")
        f.write("| phase | kernel | avg us | memory-side read MiB | memory-side written MiB | memory-side TB/s | L2 requests | L2 TB/s (<=) | L2 hit rate | L2 atomics | L1->L2 reads | L1->L2 writes | L1->L2 atomics | atomic requests/s | VALU instr (wave) | LDS instr (wave) | LDS bank-conflict cycles |\n")
        f.write("|" + "---|" * 17 + "\n")
        for (ph, k), r in sorted(rows.items(), key=lambda kv: (kv[0][0], -kv[1]["us"])):
            sec = r["us"] * 1e-6
            f.write(f"| {ph} | `{k}` | {r['us']:.1f} | {r['read_bytes'] / 2**20:.1f} | {r['written_bytes'] / 2**20:.1f} | {r['hbm_bytes'] / sec / 1e12:.2f} | "
                    f"{r['l2_requests']:.3g} | {r['l2_requests'] * L2_LINE_BYTES / sec / 1e12:.1f} | {r['l2_hit_rate']:.2f} | {r['l2_atomics']:.3g} | "
                    f"{r['l1_l2_reads']:.3g} | {r['l1_l2_writes']:.3g} | {r['l1_l2_atomics']:.3g} | {r['l1_l2_atomics'] / sec:.3g} | "
                    f"{r['valu_wave_instr']:.3g} | {r['lds_wave_instr']:.3g} | {r['lds_bank_conflict_cycles']:.3g} |\n")
        if any(r["ea_read_requests"] is not None for r in rows.values()):
            f.write("\nRequests at the L2's memory-side port (TCC_EA0_*): reads are 64 bytes unless counted as 32-byte, writes 32 bytes unless counted as 64-byte.\n\n")
            f.write("| phase | kernel | read requests | of them 32 B | write requests | of them 64 B |\n|---|---|---|---|---|---|\n")
            for (ph, k), r in sorted(rows.items(), key=lambda kv: (kv[0][0], -kv[1]["us"])):
                if r["ea_read_requests"] is not None:
                    f.write(f"| {ph} | `{k}` | {r['ea_read_requests']:.3g} | {r['ea_read_requests_32B']:.3g} | {r['ea_write_requests']:.3g} | {r['ea_write_requests_64B']:.3g} |\n")
    entry = {}
    for ph in bench["phases_ms"]:
        mine = {k: r for (p, k), r in rows.items() if p == ph}
        entry[ph] = {
            "kernels": sorted(mine),
            "per_kernel": {k: {"hbm_bytes": r["hbm_bytes"], "valu_wave_instr": r["valu_wave_instr"], "us": r["us"]} for k, r in sorted(mine.items())},
            "hbm_bytes": sum(r["hbm_bytes"] for r in mine.values()),
            "valu_wave_instr": sum(r["valu_wave_instr"] for r in mine.values()),
        }
    return entry


def main(workloads):
    sys.path.insert(0, ROOT)
    from bench import kernel_source_digest
    os.makedirs(PROFILES, exist_ok=True)
    digest = kernel_source_digest()
    commit = subprocess.run(["git", "rev-parse", "--short", "HEAD"], capture_output=True, text=True, cwd=ROOT).stdout.strip()
    path = os.path.join(PROFILES, "hbm_traffic.json")
    cur = json.load(open(path)) if os.path.exists(path) else {}
    if cur.get("source_digest") != digest:
        cur = {}
    cur["source_digest"], cur["commit"] = digest, commit
    cur["note"] = ("bytes through the L2's memory-side port per launch (FETCH_SIZE and WRITE_SIZE, scaled by what the 1 GiB copy probe reads "
                   "back in the same run) and wave-level vector instructions per launch (SQ_INSTS_VALU), per bench.py phase; every phase "
                   "lists the kernels it was summed over, and the rows of profiles/<workload>_counters.md hold the same figures")
    for wl in workloads:
        entry = summarise(wl, digest, commit)
        if entry is not None:
            cur[wl] = entry
    json.dump(cur, open(path, "w"), indent=1)
    print(json.dumps(cur, indent=1))


if __name__ == "__main__":
    main(sys.argv[1:])
