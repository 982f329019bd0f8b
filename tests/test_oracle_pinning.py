"""Pins the CPU oracle to what the mathematics fixes.

The reference ships no tests, no golden vectors and no CPU path, so every function of the oracle
is pinned by a closed form, an invariant or a brute-force property chosen so that a plausible
mistake (a dropped term, a wrong sign or index, a transposed operand) fails:

  hash                  known answers evaluated as a polynomial in Python integers
  scale factors         closed form within 2 ulp (three fp32 roundings); division rule by a GPU test against torch
  elevation             sum = 0 and |E| = |pos+shift|/sigma (scaled isometry)
  simplex / rank / keys vertices are A_d* lattice points forming a canonical simplex that
                        contains the point: sum_r b_r * vertex_r = E, b >= 0, sum b = 1
  forward               reproduces affine functions on a collision-free table; constant table;
                        one-hot table entry
  table backward        adjoint of the forward (which is linear in the table)
  position backward     finite differences of the fp64 forward inside a simplex (exact there)
  double backward       the position gradient is bilinear in (table, grad): two adjoint identities
"""
import numpy as np
import pytest

from oracle import api as orc
from helpers import HASH_MUL, random_problem

DIMS = [2, 3, 4, 5, 6, 7, 8]
FEATS = [2, 4, 8]  # features per level: the reference's value and the two generalisations its text anticipates


# ----------------------------------------------------------------------------- hash

def poly_hash(key):
    d = len(key)
    return sum(int(k) * pow(HASH_MUL, d - i, 1 << 32) for i, k in enumerate(key)) % (1 << 32)


HASH_KATS = [  # (key, raw hash) -- literals worked out by hand with Python integers
    ((0, 0, 0), 0),
    ((0, 0, 1), 2531011),
    ((1, 0, 0), 2937900635),
    ((1, 2, 3), 3091413942),
    ((-1, -1, -1), 3429059161),
    ((4, -4, 0), 2869827400),
    ((100000, -200000, 300000), 2781112128),
    ((1, 2, 3, 4), 3081718446),
    ((3, -5, 7, -9, 11, -13, 15, -17), 2672460032),
]


@pytest.mark.parametrize("key,want", HASH_KATS)
def test_hash_known_answers(key, want):
    assert poly_hash(key) == want  # the literal and the polynomial form agree
    assert orc.hash_key(key) == want


def test_hash_slots():
    assert orc.slot((1, 0, 0), 1 << 18) == 52827
    assert orc.slot((0, 0, 1), 1 << 18) == 171715
    assert orc.slot((1, 2, 3), 1 << 18) == 211894
    assert orc.slot((-1, -1, -1), 1 << 18) == 215641
    assert orc.slot((-1, -1, -1), 1 << 22) == 2312793
    assert orc.slot((1, 2, 3, 4), 1 << 19) == 477870
    assert orc.slot((3, -5, 7, -9, 11, -13, 15, -17), 1 << 19) == 164096
    assert orc.slot((1, 2, 3), 100003) == 21203  # capacity need not be a power of two


@pytest.mark.parametrize("d", DIMS)
def test_hash_random_keys_match_polynomial(d):
    rng = np.random.default_rng(d)
    for _ in range(200):
        key = rng.integers(-2_000_000, 2_000_000, d)
        assert orc.hash_key(key) == poly_hash(key)
        cap = int(rng.integers(1, 1 << 23))
        assert orc.slot(key, cap) == poly_hash(key) % cap


# ----------------------------------------------------------------------------- scale factors

@pytest.mark.parametrize("d", DIMS)
def test_scale_factors_closed_form(d):
    sig = np.geomspace(1.0, 1e-4, 24).astype(np.float32)
    sf = orc.scale_factors(d, sig)
    i = np.arange(d, dtype=np.float64)
    want = 1.0 / (np.sqrt((i + 1) * (i + 2))[None, :] * sig.astype(np.float64)[:, None])
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    # three fp32 roundings (the numerator, the reciprocal of sigma, their product): at most 2 ulp from the exact value
    assert np.all(np.abs(sf.astype(np.float64) - want) <= 2.0 * ulp)
    # and exactly the rule fp32(numerator) * fp32(1 / sigma)
    num = (1.0 / np.sqrt((i + 1) * (i + 2))).astype(np.float32)
    assert np.array_equal(sf, num[None, :] * (np.float32(1.0) / sig)[:, None])


# ----------------------------------------------------------------------------- elevation + simplex

def _simplex_case(d, dtype, n=4096, levels=6, seed=0, capacity=1 << 20):
    p = random_problem(d, n, levels, 8, seed=seed, sigma_range=(1.0, 1e-2), dtype=dtype)
    sf = orc.scale_factors(d, p["sigmas"]).astype(dtype)
    s = orc.simplex(p["pos"], sf, p["shift"], capacity, dtype=dtype, with_keys=True)
    return p, sf, s


@pytest.mark.parametrize("d", DIMS)
def test_elevation_is_a_scaled_isometry_onto_the_zero_sum_hyperplane(d):
    p, sf, s = _simplex_case(d, np.float64)
    e = s["elevated"]  # (L,N,D+1)
    assert np.max(np.abs(e.sum(-1))) < 1e-9 * (1 + np.max(np.abs(e)))
    x = (p["pos"][None] + p["shift"][:, None])  # (L,N,D)
    # |E|^2 = sum_k ((x_k * sf_k)^2 * (k+1)(k+2)): each axis maps to an orthogonal direction
    k = np.arange(d)
    want = np.sqrt((((x * sf[:, None]) ** 2) * ((k + 1) * (k + 2))).sum(-1))
    assert np.allclose(np.linalg.norm(e, axis=-1), want, rtol=1e-12, atol=1e-12)
    # ... and since sf_k = 1/(sqrt((k+1)(k+2)) sigma) that is |x|/sigma
    sf64 = 1.0 / (np.sqrt((k + 1) * (k + 2))[None] * p["sigmas"].astype(np.float64)[:, None])
    s2 = orc.simplex(p["pos"], sf64, p["shift"], 1 << 20, dtype=np.float64)
    want2 = np.linalg.norm(x, axis=-1) / p["sigmas"].astype(np.float64)[:, None]
    assert np.allclose(np.linalg.norm(s2["elevated"], axis=-1), want2, rtol=1e-12)


@pytest.mark.parametrize("d", DIMS)
def test_elevation_matches_explicit_basis(d):
    """E = B (x * sf) with the triangular basis B[0,k]=1, B[i,k]=1 for k>=i, B[i,i-1]=-i."""
    p, sf, s = _simplex_case(d, np.float64, n=64, levels=3)
    b = np.zeros((d + 1, d))
    for i in range(d + 1):
        for k in range(d):
            if k >= i:
                b[i, k] = 1.0
            elif k == i - 1:
                b[i, k] = -float(i)
    x = (p["pos"][None] + p["shift"][:, None]) * sf[:, None]
    want = np.einsum("ik,lnk->lni", b, x)
    assert np.allclose(s["elevated"], want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("d", DIMS)
def test_simplex_is_the_enclosing_lattice_simplex(d, dtype):
    p, sf, s = _simplex_case(d, dtype)
    d1 = d + 1
    rem0, rank, keys, bary, e = s["rem0"], s["rank"], s["keys"], s["bary"].astype(np.float64), s["elevated"].astype(np.float64)
    # post-conditions of the wrap
    assert np.all(rem0.sum(-1) == 0)
    assert np.all(np.sort(rank, -1) == np.arange(d1))
    assert np.all(rem0 % d1 == 0)
    # vertex r is a lattice point of A_d*: coordinates sum to 0 and are all congruent to r mod d+1
    assert np.all(keys.sum(-1) == 0)
    for r in range(d1):
        assert np.all((keys[..., r, :] - r) % d1 == 0)
    assert np.all(keys[..., 0, :] == rem0)
    # canonical simplex: going from vertex r to r+1 adds 1 everywhere except -d on the coordinate of rank d-r
    for r in range(d):
        step = keys[..., r + 1, :] - keys[..., r, :]
        want = np.where(rank == d - r, -d, 1)
        assert np.all(step == want)
    # barycentric weights: non-negative, sum to one, and reproduce the point
    tol = 1e-9 if dtype == np.float64 else 2e-6 * (1 + np.abs(e).max(-1, keepdims=True))
    assert np.all(bary >= -np.max(tol))
    assert np.all(np.abs(bary.sum(-1) - 1.0) <= (1e-9 if dtype == np.float64 else 1e-5))
    recon = np.einsum("lnr,lnri->lni", bary, keys.astype(np.float64))
    assert np.all(np.abs(recon - e) <= tol * 4)


@pytest.mark.parametrize("d", [2, 3, 4, 8])
def test_rank_orders_the_residuals(d):
    p, sf, s = _simplex_case(d, np.float64, n=2048)
    resid = s["elevated"] - s["rem0"]
    # rank 0 = largest residual ... rank d = smallest (ties are measure-zero for random fp64 input)
    order = np.argsort(-resid, axis=-1, kind="stable")
    want = np.empty_like(order)
    np.put_along_axis(want, order, np.broadcast_to(np.arange(d + 1), order.shape), axis=-1)
    assert np.all(want == s["rank"])
    assert np.all(resid.max(-1) - resid.min(-1) <= d + 1 + 1e-9)


def test_simplex_hand_case_origin():
    """pos + shift = 0: E = 0, every residual ties, so rank = (0..d), weight 1 on the origin vertex (slot 0)."""
    for d in DIMS:
        pos = np.zeros((1, d), np.float32)
        shift = np.zeros((1, d), np.float32)
        sf = orc.scale_factors(d, [1.0])
        s = orc.simplex(pos, sf, shift, 1 << 10, with_keys=True)
        assert np.all(s["rem0"] == 0) and np.all(s["rank"][0, 0] == np.arange(d + 1))
        assert np.allclose(s["bary"][0, 0], [1.0] + [0.0] * d)
        assert s["slot"][0, 0, 0] == 0


def test_simplex_hand_case_2d():
    """d=2, sigma=1, shift=0, pos=(sqrt(2)*0.9, 0): cf=(0.9, 0) so E=(0.9,-0.9,0).

    Nearest multiples of 3 are (0,0,0); residuals (0.9,-0.9,0) give rank (0,2,1); weights
    b[2-rank_i] += e_i/3, b[3-rank_i] -= e_i/3, b0 += 1 + b3  ->  b = (0.4, 0.3, 0.3).
    Vertices: (0,0,0), (1,-2,1)->key(1,-2), (2,-1,-1)->key(2,-1).
    """
    pos = np.array([[np.sqrt(2.0) * 0.9, 0.0]], np.float64)
    sf = np.array([[1 / np.sqrt(2.0), 1 / np.sqrt(6.0)]])
    s = orc.simplex(pos, sf, np.zeros((1, 2)), 1 << 16, dtype=np.float64, with_keys=True)
    assert np.allclose(s["elevated"][0, 0], [0.9, -0.9, 0.0])
    assert list(s["rem0"][0, 0]) == [0, 0, 0]
    assert list(s["rank"][0, 0]) == [0, 2, 1]
    assert np.allclose(s["bary"][0, 0], [0.4, 0.3, 0.3])
    assert s["keys"][0, 0].tolist() == [[0, 0, 0], [1, -2, 1], [2, -1, -1]]
    assert s["slot"][0, 0].tolist() == [0, poly_hash((1, -2)) % (1 << 16), poly_hash((2, -1)) % (1 << 16)]


# Rounding ties.  A coordinate of the elevated point exactly halfway between two multiples of D+1
# takes the lower one (the comparison `up - e < e - down` is strict, EncodingGPU.cuh:153-157).
# Worked by hand, D = 3, pos = (2, 0, 0), unit scale factors, no shift:
#   elevated = (2, -2, 0, 0); both 2 and -2 are ties: rounded down to 0 and -4; sum/4 = -1
#   residuals (2, 2, 0, 0) -> ranks (0, 1, 2, 3) (equal residuals: the lower index ranks first), plus
#   the sum: (-1, 0, 1, 2); rank 0 wraps to 3 and its rem0 to 4  =>  rem0 (4, -4, 0, 0), rank (3, 0, 1, 2)
#   delta = (elevated - rem0)/4 = (-1/2, 1/2, 0, 0)  =>  weights (0, 1/2, 0, 1/2)
# and D = 2, pos = (1.5, 0): elevated (1.5, -1.5, 0) -> rem0 (3, -3, 0), rank (2, 0, 1), weights (0, 1/2, 1/2).
# (Taking the upper multiple at a tie instead ends in the same rem0, rank and weights: the tied
# coordinates then have the smallest residuals instead of the largest, the sum is larger by their
# number, and the wrap puts them back in front in index order.  So the direction of the tie is
# not observable, which the mutation check of these tests confirms; the values below are.)
TIE_CASES = [
    (3, [2.0, 0.0, 0.0], [2.0, -2.0, 0.0, 0.0], [4, -4, 0, 0], [3, 0, 1, 2], [0.0, 0.5, 0.0, 0.5]),
    (2, [1.5, 0.0], [1.5, -1.5, 0.0], [3, -3, 0], [2, 0, 1], [0.0, 0.5, 0.5]),
]


@pytest.mark.parametrize("d,pos,elevated,rem0,rank,bary", TIE_CASES)
def test_rounding_tie_hand_worked(d, pos, elevated, rem0, rank, bary):
    s = orc.simplex(np.array([pos], np.float32), np.ones((1, d), np.float32), np.zeros((1, d), np.float32), 1 << 16,
                    with_keys=True)
    assert s["elevated"][0, 0].tolist() == elevated
    assert s["rem0"][0, 0].tolist() == rem0
    assert s["rank"][0, 0].tolist() == rank
    assert s["bary"][0, 0].tolist() == bary
    keys = [[rem0[i] + r - (d + 1) * (rank[i] > d - r) for i in range(d + 1)] for r in range(d + 1)]
    assert s["keys"][0, 0].tolist() == keys
    assert s["slot"][0, 0].tolist() == [poly_hash(k[:d]) % (1 << 16) for k in keys]


# ----------------------------------------------------------------------------- forward

def _collision_free(d, dtype, n=512, levels=4, seed=1, capacity=1 << 22):
    """A problem plus, per level, a dict vertex-key -> slot that is injective on the touched vertices."""
    for attempt in range(20):
        p = random_problem(d, n, levels, 8, seed=seed + 100 * attempt, sigma_range=(1.0, 0.05), dtype=dtype)
        sf = orc.scale_factors(d, p["sigmas"]).astype(dtype)
        s = orc.simplex(p["pos"], sf, p["shift"], capacity, dtype=dtype, with_keys=True)
        ok = True
        for l in range(levels):
            k = s["keys"][l].reshape(-1, d + 1)
            sl = s["slot"][l].reshape(-1)
            uk = np.unique(k, axis=0)
            us = np.unique(sl)
            if len(uk) != len(us):
                ok = False
                break
        if ok:
            return p, sf, s, capacity
    raise AssertionError("no collision-free sample found")


@pytest.mark.parametrize("feat", FEATS)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("d", DIMS)
def test_forward_reproduces_affine_functions(d, dtype, feat):
    """Simplex interpolation has linear precision: a table holding a.v + c at every touched vertex v
    must give window * (a.E + c) at the point, whatever the simplex."""
    p, sf, s, cap = _collision_free(d, dtype)
    levels, n = s["slot"].shape[:2]
    rng = np.random.default_rng(7)
    a = rng.standard_normal((feat, d + 1))
    c = rng.standard_normal(feat)
    table = np.zeros((levels, cap, feat), dtype)
    for l in range(levels):
        k = s["keys"][l].reshape(-1, d + 1).astype(np.float64)
        table[l, s["slot"][l].reshape(-1)] = (k @ a.T + c).astype(dtype)
    out = orc.forward(p["pos"], table, sf, p["shift"], p["window"], dtype=dtype).astype(np.float64)
    want = (np.einsum("fi,lni->lfn", a, s["elevated"].astype(np.float64)) + c[None, :, None]) * p["window"].astype(np.float64)[:, None, None]
    scale = 1 + np.abs(want).max()
    tol = 1e-9 if dtype == np.float64 else 3e-5
    assert np.max(np.abs(out - want)) <= tol * scale


@pytest.mark.parametrize("feat", FEATS)
@pytest.mark.parametrize("d", [2, 3, 4, 8])
def test_forward_constant_table_and_one_hot(d, feat):
    p, sf, s, cap = _collision_free(d, np.float32, n=256, levels=3)
    levels, n = s["slot"].shape[:2]
    table = np.empty((levels, cap, feat), np.float32)
    consts = np.array([2.0, -3.0, 0.5, 7.0, -1.5, 4.0, 0.25, -8.0][:feat], np.float32)
    table[...] = consts
    out = orc.forward(p["pos"], table, sf, p["shift"], p["window"])
    for f in range(feat):
        assert np.allclose(out[:, f], consts[f] * p["window"][:, None], rtol=1e-5)
    # one-hot: only feature f of vertex r of point 0 at level 1 is set -> that output of point 0 is the vertex weight
    for r in range(d + 1):
        f = r % feat
        table[:] = 0
        table[1, s["slot"][1, 0, r], f] = 1.0
        out = orc.forward(p["pos"], table, sf, p["shift"], np.ones(levels, np.float32))
        assert np.isclose(out[1, f, 0], s["bary"][1, 0, r], rtol=1e-6, atol=1e-7)
        assert np.all(out[[0, 2]] == 0) and np.all(np.delete(out, f, axis=1) == 0)


def test_forward_window_zero_gives_exact_zero_and_is_linear():
    d = 3
    p = random_problem(d, 1000, 5, 1 << 10, seed=3)
    sf = orc.scale_factors(d, p["sigmas"])
    win = np.array([1, 0, 0.5, 0, 1], np.float32)
    out = orc.forward(p["pos"], p["table"], sf, p["shift"], win)
    ones = orc.forward(p["pos"], p["table"], sf, p["shift"], np.ones(5, np.float32))
    assert np.all(out[[1, 3]] == 0.0)
    assert np.array_equal(out[[0, 4]], ones[[0, 4]])
    assert np.allclose(out[2], 0.5 * ones[2], rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("feat", FEATS)
@pytest.mark.parametrize("d", [2, 3, 4, 5])
def test_forward_concat_points_extra_levels(d, feat):
    p = random_problem(d, 100, 3, 64, seed=4, nr_feat=feat)
    sf = orc.scale_factors(d, p["sigmas"])
    out = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"], concat_points=True, points_scaling=0.25)
    extra = -(-d // feat)
    assert out.shape == (3 + extra, feat, 100)
    flat = out[3:].reshape(extra * feat, 100)
    for k in range(extra * feat):
        want = p["pos"][:, k] * np.float32(0.25) if k < d else np.zeros(100, np.float32)
        assert np.array_equal(flat[k], want)
    base = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"])
    assert np.array_equal(out[:3], base)


# ----------------------------------------------------------------------------- gradients

@pytest.mark.parametrize("feat", FEATS)
@pytest.mark.parametrize("d", DIMS)
def test_table_backward_is_the_adjoint_of_forward(d, feat):
    p = random_problem(d, 700, 4, 1 << 9, seed=5, dtype=np.float64, nr_feat=feat)  # small capacity: many collisions
    sf = orc.scale_factors(d, p["sigmas"]).astype(np.float64)
    out = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"], dtype=np.float64)
    tg = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], 1 << 9, dtype=np.float64)["grad64"]
    lhs = np.sum(out * p["grad"])
    rhs = np.sum(tg * p["table"])
    assert np.isclose(lhs, rhs, rtol=1e-11)
    # the fp32 instantiation satisfies the same identity with its own (fp32) weights: forward and
    # backward share the preamble bit for bit, so only the rounding of the products differs
    p32 = {k: v.astype(np.float32) for k, v in p.items()}
    sf32 = sf.astype(np.float32)
    out32 = orc.forward(p32["pos"], p32["table"], sf32, p32["shift"], p32["window"]).astype(np.float64)
    r = orc.backward_table(p32["pos"], sf32, p32["shift"], p32["window"], p32["grad"], 1 << 9, want_abs=True)
    lhs32 = np.sum(out32 * p32["grad"])
    rhs32 = np.sum(r["grad64"] * p32["table"])
    assert abs(lhs32 - rhs32) <= 1e-6 * np.sum(r["abs64"] * np.abs(p32["table"]))
    assert np.all(np.abs(r["grad32"] - r["grad64"]) <= 1e-5 * r["abs64"] + 1e-12)


def _interior_points(d, levels, n, seed, margin=0.02, feat=2):
    """fp64 problem restricted to points whose barycentric weights are all > margin at every level."""
    p = random_problem(d, n, levels, 1 << 12, seed=seed, sigma_range=(1.0, 0.1), dtype=np.float64, nr_feat=feat)
    sf = orc.scale_factors(d, p["sigmas"]).astype(np.float64)
    s = orc.simplex(p["pos"], sf, p["shift"], 1 << 12, dtype=np.float64)
    keep = np.all(s["bary"].min(-1) > margin, axis=0)
    assert keep.sum() >= 8
    for k in ("pos", "dpos"):
        p[k] = np.ascontiguousarray(p[k][keep])
    p["grad"] = np.ascontiguousarray(p["grad"][:, :, keep])
    return p, sf


@pytest.mark.parametrize("feat", FEATS)
@pytest.mark.parametrize("d", DIMS)
def test_position_backward_matches_finite_differences(d, feat):
    levels = 3
    p, sf = _interior_points(d, levels, 4000 if d < 7 else 60000, seed=6, margin=0.02 if d < 6 else 0.005, feat=feat)
    n = p["pos"].shape[0]
    got = orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"], dtype=np.float64)["grad64"]
    h = 1e-6
    for i in range(d):
        dp = np.zeros((1, d))
        dp[0, i] = h
        fp = orc.forward(p["pos"] + dp, p["table"], sf, p["shift"], p["window"], dtype=np.float64)
        fm = orc.forward(p["pos"] - dp, p["table"], sf, p["shift"], p["window"], dtype=np.float64)
        fd = ((fp - fm) / (2 * h) * p["grad"]).sum((0, 1))
        assert np.allclose(got[:, i], fd, rtol=1e-6, atol=1e-6), f"axis {i}"
    # fp32 instantiation agrees with the fp64 one on the same (interior) points
    g32 = orc.backward_pos(*(p[k].astype(np.float32) for k in ("pos", "table")), sf.astype(np.float32),
                           *(p[k].astype(np.float32) for k in ("shift", "window", "grad")))
    scale = np.abs(got).max()
    assert np.max(np.abs(g32["grad32"] - got)) <= 2e-3 * scale  # fp32 positions move the point slightly
    assert np.max(np.abs(g32["grad32"] - g32["grad64"])) <= 1e-5 * scale
    assert n > 0


@pytest.mark.parametrize("feat", FEATS)
@pytest.mark.parametrize("d", DIMS)
def test_double_backward_adjoint_identities(d, feat):
    p = random_problem(d, 500, 4, 1 << 9, seed=8, dtype=np.float64, nr_feat=feat)
    sf = orc.scale_factors(d, p["sigmas"]).astype(np.float64)
    args = (p["pos"], p["table"], sf, p["shift"], p["window"])
    pg = orc.backward_pos(*args, p["grad"], dtype=np.float64)["grad64"]
    r = orc.double_backward(*args, p["dpos"], p["grad"], dtype=np.float64)
    lhs = np.sum(p["dpos"] * pg)
    assert np.isclose(lhs, np.sum(r["ggs"] * p["grad"]), rtol=1e-10)
    assert np.isclose(lhs, np.sum(r["grad64"] * p["table"]), rtol=1e-10)
    # fp32 instantiation: same identities with its own weights
    p32 = {k: v.astype(np.float32) for k, v in p.items()}
    a32 = (p32["pos"], p32["table"], sf.astype(np.float32), p32["shift"], p32["window"])
    pg32 = orc.backward_pos(*a32, p32["grad"])["grad64"]
    r32 = orc.double_backward(*a32, p32["dpos"], p32["grad"], want_abs=True)
    lhs32 = np.sum(p32["dpos"].astype(np.float64) * pg32)
    scale = np.sum(r32["abs64"] * np.abs(p32["table"]))
    assert abs(lhs32 - np.sum(r32["ggs"].astype(np.float64) * p32["grad"])) <= 1e-5 * scale
    assert abs(lhs32 - np.sum(r32["grad64"] * p32["table"])) <= 1e-5 * scale
    assert np.all(np.abs(r32["grad32"] - r32["grad64"]) <= 1e-5 * r32["abs64"] + 1e-9)


@pytest.mark.parametrize("feat", FEATS)
def test_double_backward_concat_levels_are_zero(feat):
    d = 3
    p = random_problem(d, 64, 2, 64, seed=9, nr_feat=feat)
    sf = orc.scale_factors(d, p["sigmas"])
    extra = -(-d // feat)
    grad = np.concatenate([p["grad"], np.ones((extra, feat, 64), np.float32)])
    r = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], grad, concat_points=True)
    assert r["ggs"].shape == (2 + extra, feat, 64) and np.all(r["ggs"][2:] == 0)
    r0 = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"])
    assert np.array_equal(r["ggs"][:2], r0["ggs"]) and np.array_equal(r["grad64"], r0["grad64"])


def test_fp32_and_fp64_instantiations_pick_the_same_simplex_away_from_faces():
    for d in (3, 4, 8):
        p = random_problem(d, 4000, 4, 1 << 12, seed=10, sigma_range=(1.0, 0.1), dtype=np.float64)
        sf = orc.scale_factors(d, p["sigmas"])
        s64 = orc.simplex(p["pos"], sf.astype(np.float64), p["shift"], 1 << 12, dtype=np.float64)
        s32 = orc.simplex(p["pos"].astype(np.float32), sf, p["shift"].astype(np.float32), 1 << 12)
        safe = s64["bary"].min(-1) > 1e-3
        assert safe.mean() > 0.5
        assert np.all(s32["rank"][safe] == s64["rank"][safe])
        assert np.all(s32["slot"][safe] == s64["slot"][safe])
