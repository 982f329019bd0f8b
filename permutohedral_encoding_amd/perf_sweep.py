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

    python -m permutohedral_encoding_amd.perf_sweep [--dims 2 3 4 5 6] [--points 524288] [--iters 300] [--fused-optimizer]

``--consumers`` instead runs what the layer after the encoding does with the (N, 48) result of 2^20 points,
a few times each and meant to be run under a kernel trace: ``torch.nn.Linear``, ``torch.cat`` with
another (N, 3) array and an element-wise ``relu``, first on the module's default result (the strided
view of the reference's permute + reshape, modules.py:87), then with ``contiguous_output=True``.  The
trace shows which consumers copy the view and what the contiguous rows cost instead.
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


def measure(pos_dim, nr_points, iters, warmup, levels=24, log2_capacity=18, fused_optimizer=False):
    torch.manual_seed(0)
    enc = PermutoEncoding(pos_dim, 1 << log2_capacity, levels, 2, np.geomspace(1.0, 1e-4, num=levels))
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


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--dims", type=int, nargs="+", default=[2, 3, 4, 5, 6])
    ap.add_argument("--points", type=int, default=1 << 19)
    ap.add_argument("--iters", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--fused-optimizer", action="store_true",
                    help="step the table with permutohedral_encoding_amd.optim.AdamW instead of torch.optim.AdamW")
    ap.add_argument("--consumers", action="store_true", help="run the consumers of the forward result instead (for a kernel trace)")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("perf_sweep: no GPU visible; the encoding has no CPU path")
    if args.consumers:
        consumers()
        return
    print("| pos_dim | inference (points/s) | training, table grad (points/s) | training, table + position grad (points/s) |")
    print("|---|---|---|---|")
    rows = []
    for d in args.dims:
        r = measure(d, args.points, args.iters, args.warmup, fused_optimizer=args.fused_optimizer)
        rows.append(r)
        print(f"| {d} | {r['inference']:.3g} | {r['train_table']:.3g} | {r['train_table_pos']:.3g} |", flush=True)
    print(json.dumps(rows))


if __name__ == "__main__":
    main()
