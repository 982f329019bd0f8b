"""Seeded synthetic inputs for the five benchmark / parity configurations.

Everything is generated on the host with ``numpy.random.default_rng(seed)`` and uploaded
afterwards, so the CPU checker and the GPU kernels see identical bits.  Distributions follow the
reference's module (``src/pytorch_modules/modules.py:25-32``: table ~ small, shift ~ N(0,1)*10)
and its performance script (``examples/performance.py:41-43,152-154``: 24 levels, 2 features,
capacity 2^18, scales geomspace(1, 1e-4)).
"""
from dataclasses import dataclass, field
from typing import Optional, Tuple

import numpy as np


@dataclass(frozen=True)
class Workload:
    name: str
    pos_dim: int
    capacity: int
    nr_levels: int
    nr_points: int
    scale_range: Tuple[float, float]
    points: str = "uniform"  # "uniform" in [0,1]^D, "sphere" (shell of radius 0.5 around 0.5) or "rays" (samples along chords, in order)
    masked_top_levels: int = 0  # anneal window = 1 for the coarse levels, 0 for this many fine ones
    phases: Tuple[str, ...] = field(default=("forward",))

    @property
    def point_levels(self):
        return self.nr_points * self.nr_levels

    def scaled(self, nr_points):
        """Same encoding, fewer points (for checks the CPU checker finishes in seconds)."""
        return Workload(self.name, self.pos_dim, self.capacity, self.nr_levels, int(nr_points), self.scale_range,
                        self.points, self.masked_top_levels, self.phases)


WORKLOADS = {
    "c1": Workload("c1", 3, 1 << 18, 24, 1 << 16, (1.0, 1e-4), phases=("forward",)),
    "c2": Workload("c2", 3, 1 << 18, 24, 1 << 20, (1.0, 1e-4), phases=("forward", "backward_table")),
    "c3": Workload("c3", 4, 1 << 18, 24, 1 << 20, (1.0, 1e-4), phases=("forward", "backward_pos", "double_backward")),
    "c4": Workload("c4", 8, 1 << 19, 16, 1 << 19, (1.0, 1e-3), phases=("forward", "backward_table")),
    "c5": Workload("c5", 3, 1 << 22, 24, 1 << 20, (1.0, 1e-4), points="sphere", masked_top_levels=8,
                   phases=("forward", "backward_table", "backward_pos", "double_backward")),
    # not a BASELINE configuration: c2 with the points a renderer hands over, 128 consecutive samples along each of
    # 8192 rays, so that neighbouring points are neighbours in space (the benchmark's uniform points never are)
    "c2_rays": Workload("c2_rays", 3, 1 << 18, 24, 1 << 20, (1.0, 1e-4), points="rays", phases=("forward", "backward_table")),
}

RAY_SAMPLES = 128


def scale_list(w: Workload):
    return np.geomspace(w.scale_range[0], w.scale_range[1], num=w.nr_levels).astype(np.float32)


def anneal_window(w: Workload):
    win = np.ones(w.nr_levels, np.float32)
    if w.masked_top_levels:
        win[w.nr_levels - w.masked_top_levels:] = 0.0
    return win


def make_inputs(w: Workload, need=("table", "shift", "pos", "grad", "dpos"), nr_points: Optional[int] = None):
    """Dict of float32 arrays: table (L,C,2), shift (L,D), pos (N,D), grad (L,2,N), dpos (N,D), sigmas, window.

    ``grad`` is drawn as the module-level upstream gradient of shape (N, 2L) ~ N(0,1) and handed
    over in the kernel's (L, 2, N) layout, the way autograd delivers it through the module's
    permute (``src/pytorch_modules/modules.py:87``).
    """
    n = w.nr_points if nr_points is None else int(nr_points)
    d, l, c = w.pos_dim, w.nr_levels, w.capacity
    out = {"sigmas": scale_list(w), "window": anneal_window(w)}
    if "table" in need:
        out["table"] = np.random.default_rng(1).uniform(-1e-4, 1e-4, size=(l, c, 2)).astype(np.float32)
    if "shift" in need:
        out["shift"] = (np.random.default_rng(2).standard_normal((l, d)) * 10.0).astype(np.float32)
    if "pos" in need:
        if w.points == "uniform":
            out["pos"] = np.random.default_rng(3).uniform(0.0, 1.0, size=(n, d)).astype(np.float32)
        elif w.points == "sphere":
            rng = np.random.default_rng(6)
            u = rng.standard_normal((n, d))
            u /= np.linalg.norm(u, axis=1, keepdims=True)
            r = 0.5 + rng.standard_normal((n, 1)) * 0.02
            out["pos"] = (0.5 + r * u).astype(np.float32)
        elif w.points == "rays":
            rng = np.random.default_rng(7)
            n_rays = (n + RAY_SAMPLES - 1) // RAY_SAMPLES
            origin = rng.uniform(0.25, 0.75, (n_rays, d))
            direction = rng.standard_normal((n_rays, d))
            direction /= np.linalg.norm(direction, axis=1, keepdims=True)
            along = (np.arange(RAY_SAMPLES) + rng.uniform(0, 1, (n_rays, RAY_SAMPLES))) / RAY_SAMPLES - 0.5  # stratified
            pos = origin[:, None, :] + 0.8 * along[:, :, None] * direction[:, None, :]
            out["pos"] = np.clip(pos.reshape(-1, d)[:n], 0.0, 1.0).astype(np.float32)
        else:
            raise ValueError(w.points)
    if "grad" in need:
        g = np.random.default_rng(4).standard_normal((n, 2 * l), dtype=np.float32)
        out["grad"] = np.ascontiguousarray(g.reshape(n, l, 2).transpose(1, 2, 0))
    if "dpos" in need:
        out["dpos"] = np.random.default_rng(5).standard_normal((n, d), dtype=np.float32)
    return out
