"""Module-level throughput sweep over the input dimension, in points per second.

Follows the measurement protocol of the reference's performance script
(``examples/performance.py:59-183``): 2^19 points uniform in [-0.5, 0.5]^d, 24 levels, 2 features
per level, capacity 2^18, scales geomspace(1, 1e-4); every iteration is bracketed by a device
synchronisation and timed with ``perf_counter``; 300 iterations of which the first 10 are discarded;
throughput = points / second, averaged over the kept iterations.  Three modes:

  inference        module forward under no_grad
  train_table      forward, loss ((pred-10)^2).mean(), zero_grad, backward, AdamW step on the table
  train_table_pos  the same with points that require a gradient

Unlike the kernel benchmark (``bench.py``) these figures include everything a user of the module
pays: output allocation, the loss, the gradient layout change and the optimiser walking the whole
table.

    python -m permutohedral_encoding_amd.perf_sweep [--dims 2 3 4 5 6] [--points 524288] [--iters 300] [--fused-optimizer] [--contiguous-output]

``--consumers`` instead runs what the layer after the encoding does with the (N, 48) result of 2^20 points,
a few times each and meant to be run under a kernel trace: ``torch.nn.Linear``, ``torch.cat`` with
another (N, 3) array and an element-wise ``relu``, first on the module's default result (the strided
view of the reference's permute + reshape, modules.py:87), then with ``contiguous_output=True``.  The
trace shows which consumers copy the view and what the contiguous rows cost instead.

``--point-orders`` times the forward and the table backward (C ABI, events, config 2's geometry: 3-D, 24
levels, 2^18 slots, 2^20 points) on the same number of points in different orders: uniform and unordered
(the benchmark), consecutive samples along rays (64, 128 and 512 per ray), and the uniform points sorted
along a Z-order curve; then the table backward of every level on its own (all other levels masked by the
window) for three of them.  A renderer delivers the second kind, a caller who sorts for locality the third.
"""
import argparse
import json
import time

import numpy as np
import torch

from .modules import PermutoEncoding


def _timed(step, nr_points, iters, warmup):
    kept = []
    for it in range(iters):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if it > warmup:
            kept.append(nr_points / dt)
    return float(np.mean(kept))


def measure(pos_dim, nr_points, iters, warmup, levels=24, log2_capacity=18, fused_optimizer=False, contiguous_output=False):
    torch.manual_seed(0)
    enc = PermutoEncoding(pos_dim, 1 << log2_capacity, levels, 2, np.geomspace(1.0, 1e-4, num=levels),
                          contiguous_output=contiguous_output)
    if fused_optimizer:  # the library's one-kernel AdamW instead of torch's (same update)
        from .optim import AdamW
        opt = AdamW(enc.parameters(), betas=(0.9, 0.99), eps=1e-15, weight_decay=0.0, lr=1e-3)
    else:
        opt = torch.optim.AdamW(enc.parameters(), amsgrad=False, betas=(0.9, 0.99), eps=1e-15, weight_decay=0.0, lr=1e-3)
    pts = torch.rand(nr_points, pos_dim, device="cuda") - 0.5
    pts_grad = pts.clone().requires_grad_(True)

    def inference():
        with torch.no_grad():
            enc(pts)

    def train(points):
        pred = enc(points)
        loss = ((pred - 10) ** 2).mean()
        opt.zero_grad()
        loss.backward()
        opt.step()

    enc.eval()
    res = {"pos_dim": pos_dim, "points": nr_points, "inference": _timed(inference, nr_points, iters, warmup)}
    enc.train()
    res["train_table"] = _timed(lambda: train(pts), nr_points, iters, warmup)
    res["train_table_pos"] = _timed(lambda: train(pts_grad), nr_points, iters, warmup)
    return res


def consumers(nr_points=1 << 20, repeats=4):
    lin = torch.nn.Linear(48, 32).cuda()
    x = torch.rand(nr_points, 3, device="cuda")
    other = torch.rand(nr_points, 3, device="cuda")
    for contiguous in (False, True):
        enc = PermutoEncoding(3, 1 << 18, 24, 2, np.geomspace(1.0, 1e-4, num=24), contiguous_output=contiguous)
        with torch.no_grad():
            for _ in range(repeats):
                y = lin(enc(x))
                z = torch.cat([enc(x), other], dim=1)
                r = torch.relu(enc(x))
        torch.cuda.synchronize()
        print(f"contiguous_output={contiguous}: linear -> {tuple(y.shape)}, cat -> {tuple(z.shape)}, relu -> strides {r.stride()}")


def point_orders(repeats=25):
    from . import _native, workloads
    w = workloads.WORKLOADS["c2"]
    inputs = workloads.make_inputs(w)
    n, levels, cap, d = w.nr_points, w.nr_levels, w.capacity, w.pos_dim
    gpu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    lib = _native.lib()
    fixed = _native.EncodingFixedParams(d, cap, levels, 2, inputs["sigmas"], gpu(inputs["shift"]), False, 1.0)
    table, grad = gpu(inputs["table"]), gpu(inputs["grad"])
    out = torch.empty((levels, 2, n), device="cuda")
    table_grad = torch.empty((levels, cap, 2), device="cuda")
    ws_bytes = int(lib.penc_scatter_workspace_bytes(d, n, levels, cap, 0))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    sf, shift = fixed.m_scale_factor.data_ptr(), fixed.m_random_shift_per_level.data_ptr()

    def rays(samples):
        rng = np.random.default_rng(7)
        n_rays = (n + samples - 1) // samples
        origin = rng.uniform(0.25, 0.75, (n_rays, d))
        direction = rng.standard_normal((n_rays, d))
        direction /= np.linalg.norm(direction, axis=1, keepdims=True)
        along = (np.arange(samples) + rng.uniform(0, 1, (n_rays, samples))) / samples - 0.5
        pos = origin[:, None, :] + 0.8 * along[:, :, None] * direction[:, None, :]
        return np.clip(pos.reshape(-1, d)[:n], 0.0, 1.0).astype(np.float32)

    def z_order(p, bits=8):
        q = np.clip((p * (1 << bits)).astype(np.int64), 0, (1 << bits) - 1)
        key = np.zeros(len(p), np.int64)
        for b in range(bits):
            for k in range(p.shape[1]):
                key |= ((q[:, k] >> b) & 1) << (b * p.shape[1] + k)
        return p[np.argsort(key, kind="stable")]

    def median_us(call):
        for _ in range(3):
            call()
        times = []
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            call()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e3)
        return float(np.median(times))

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.penc_status_string(rc).decode())

    orders = {"uniform, unordered": inputs["pos"], "rays x 64 samples": rays(64), "rays x 128 samples": rays(128),
              "rays x 512 samples": rays(512), "uniform, Z-order": z_order(inputs["pos"])}
    ones = gpu(np.ones(levels, np.float32))
    print("| points | forward (us) | table backward (us) |")
    print("|---|---|---|")
    for name, pts in [("warm-up", inputs["pos"])] + list(orders.items()):
        pos = gpu(pts)
        fwd = median_us(lambda: check(lib.penc_forward(d, 2, n, levels, cap, pos.data_ptr(), table.data_ptr(), sf, shift,
                                                       ones.data_ptr(), out.data_ptr(), 0, 1.0, stream)))
        bwd = median_us(lambda: check(lib.penc_backward(d, 2, n, levels, cap, pos.data_ptr(), None, sf, shift, ones.data_ptr(),
                                                        grad.data_ptr(), table_grad.data_ptr(), None, ws.data_ptr(), ws_bytes, stream)))
        if name != "warm-up":  # the first measurements after start-up run at clocks that are still rising
            print(f"| {name} | {fwd:.0f} | {bwd:.0f} |", flush=True)
    print()
    print("Table backward with one level enabled (us, launch overheads included: 128 workgroups on 256 compute units):")
    print()
    print("| points | " + " | ".join(str(l) for l in range(levels)) + " |")
    print("|---|" + "---|" * levels)
    for name in ("uniform, unordered", "rays x 128 samples", "uniform, Z-order"):
        pos = gpu(orders[name])
        row = []
        for level in range(levels):
            window = gpu(np.eye(levels, dtype=np.float32)[level])
            row.append(median_us(lambda: check(lib.penc_backward(d, 2, n, levels, cap, pos.data_ptr(), None, sf, shift, window.data_ptr(),
                                                                 grad.data_ptr(), table_grad.data_ptr(), None, ws.data_ptr(), ws_bytes, stream))))
        print(f"| {name} | " + " | ".join(f"{x:.0f}" for x in row) + " |", flush=True)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--dims", type=int, nargs="+", default=[2, 3, 4, 5, 6])
    ap.add_argument("--points", type=int, default=1 << 19)
    ap.add_argument("--iters", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--fused-optimizer", action="store_true",
                    help="step the table with permutohedral_encoding_amd.optim.AdamW instead of torch.optim.AdamW")
    ap.add_argument("--contiguous-output", action="store_true",
                    help="build the module with contiguous_output=True: dense (N, F*L) rows instead of the strided view")
    ap.add_argument("--consumers", action="store_true", help="run the consumers of the forward result instead (for a kernel trace)")
    ap.add_argument("--point-orders", action="store_true", help="time forward and table backward on unordered, ray-ordered and Z-ordered points instead")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("perf_sweep: no GPU visible; the encoding has no CPU path")
    if args.consumers:
        consumers()
        return
    if args.point_orders:
        point_orders()
        return
    print("| pos_dim | inference (points/s) | training, table grad (points/s) | training, table + position grad (points/s) |")
    print("|---|---|---|---|")
    rows = []
    for d in args.dims:
        r = measure(d, args.points, args.iters, args.warmup, fused_optimizer=args.fused_optimizer,
                    contiguous_output=args.contiguous_output)
        rows.append(r)
        print(f"| {d} | {r['inference']:.3g} | {r['train_table']:.3g} | {r['train_table_pos']:.3g} |", flush=True)
    print(json.dumps(rows))


if __name__ == "__main__":
    main()
