"""Small shared helpers for the tests: random problems and tolerance checks."""
import numpy as np

HASH_MUL = 2531011


def random_problem(d, n, levels, capacity, seed=0, sigma_range=(1.0, 1e-2), dtype=np.float32, shift_scale=10.0, nr_feat=2):
    """A seeded problem with the reference module's distributions, at any size."""
    rng = np.random.default_rng(seed)
    sigmas = np.geomspace(sigma_range[0], sigma_range[1], levels).astype(np.float32)
    return dict(
        sigmas=sigmas,
        pos=rng.uniform(0, 1, (n, d)).astype(dtype),
        shift=(rng.standard_normal((levels, d)) * shift_scale).astype(dtype),
        table=rng.uniform(-1, 1, (levels, capacity, nr_feat)).astype(dtype),
        window=rng.uniform(0.2, 1.0, levels).astype(dtype),
        grad=rng.standard_normal((levels, nr_feat, n)).astype(dtype),
        dpos=rng.standard_normal((n, d)).astype(dtype),
    )


def assert_sum_close(got, want64, abs64, rel=1e-4, what=""):
    """Check an fp32 atomically-accumulated sum against its fp64 value.

    The error of summing terms t_k in fp32 in arbitrary order is bounded in terms of sum|t_k|, not
    of |sum t_k| (which can be arbitrarily smaller through cancellation), so the stated relative
    tolerance is applied to the sum of magnitudes.
    """
    err = np.abs(got.astype(np.float64) - want64)
    bound = rel * abs64 + 1e-30
    worst = np.max(err / bound)
    assert worst <= 1.0, f"{what}: max err/bound = {worst:.3g} (rel {rel} of sum|terms|)"


# ----------------------------------------------------------------------------- GPU side

def make_encoding(pos_dim, sigmas, shift, concat_points=False, points_scaling=1.0, device="cuda", nr_feat=2):
    """The native encoding handle (C ABI via ctypes) for a given geometry, plus its fixed parameters."""
    import torch
    from permutohedral_encoding_amd import _native
    shift_t = torch.from_numpy(np.ascontiguousarray(shift, dtype=np.float32)).to(device)
    fp = _native.EncodingFixedParams(pos_dim, 0, len(sigmas), nr_feat, sigmas, shift_t, concat_points, points_scaling)
    return _native.EncodingWrapper.create(pos_dim, nr_feat, fp), fp


def to_gpu(a, device="cuda"):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def gpu_input(p, need_table_grad=True, need_pos_grad=True, device="cuda"):
    from permutohedral_encoding_amd import _native
    return _native.EncodingInput(to_gpu(p["table"], device), to_gpu(p["pos"], device), to_gpu(p["window"], device),
                                 need_table_grad, need_pos_grad)
