"""Small shared helpers for the tests: random problems and tolerance checks."""
import numpy as np

HASH_MUL = 2531011


def random_problem(d, n, levels, capacity, seed=0, sigma_range=(1.0, 1e-2), dtype=np.float32, shift_scale=10.0):
    """A seeded problem with the reference module's distributions, at any size."""
    rng = np.random.default_rng(seed)
    sigmas = np.geomspace(sigma_range[0], sigma_range[1], levels).astype(np.float32)
    return dict(
        sigmas=sigmas,
        pos=rng.uniform(0, 1, (n, d)).astype(dtype),
        shift=(rng.standard_normal((levels, d)) * shift_scale).astype(dtype),
        table=rng.uniform(-1, 1, (levels, capacity, 2)).astype(dtype),
        window=rng.uniform(0.2, 1.0, levels).astype(dtype),
        grad=rng.standard_normal((levels, 2, n)).astype(dtype),
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
