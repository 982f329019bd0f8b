"""Checks that the pinning tests of the CPU oracle discriminate: seeded single-token mistakes in
``oracle/penc_oracle.cpp`` (a wrong sign, index, comparison, constant or dropped term: the slips a
restatement of the reference's kernels is most likely to contain) must each make
``tests/test_oracle_pinning.py`` fail.

Every mutant is the oracle's source with one substitution, compiled into a temporary directory and
handed to a fresh pytest process through ``PENC_ORACLE_LIB``.  Three substitutions are known not to be
detectable and are listed separately with the reason; for those the test asserts what can be
asserted (the outputs are identical, or differ only for points within rounding distance of a simplex
face).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE = os.path.join(ROOT, "oracle", "penc_oracle.cpp")
CXXFLAGS = ["-O1", "-std=c++17", "-fopenmp", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-march=x86-64-v3", "-shared"]

# (name, text in the oracle, replacement)
KILLED = [
    ("hash multiplier", "k *= kHashMul;", "k *= kHashMul + 2;"),
    ("hash adds after multiplying", "k += static_cast<uint32_t>(key[i]);\n        k *= kHashMul;",
     "k *= kHashMul;\n        k += static_cast<uint32_t>(key[i]);"),
    ("elevation sign", "s.elevated[i] = fused_mul_add<R>(-static_cast<R>(i), cf, sm);",
     "s.elevated[i] = fused_mul_add<R>(static_cast<R>(i), cf, sm);"),
    ("elevation drops the running sum", "sm += cf;\n    }\n    s.elevated[0] = sm;", "sm = cf;\n    }\n    s.elevated[0] = sm;"),
    ("rounds to the farther multiple", "s.rem0[i] = (up - s.elevated[i] < s.elevated[i] - down)",
     "s.rem0[i] = (up - s.elevated[i] > s.elevated[i] - down)"),
    ("rank order reversed", "if (di < dj) s.rank[i]++; else s.rank[j]++;", "if (di > dj) s.rank[i]++; else s.rank[j]++;"),
    ("rank without the coordinate sum", "s.rank[i] += sum;", "s.rank[i] += 0;"),
    ("wrap moves rem0 the wrong way", "s.rank[i] += D1;\n            s.rem0[i] += D1;", "s.rank[i] += D1;\n            s.rem0[i] -= D1;"),
    ("barycentric sign", "s.bary[D1 - s.rank[i]] -= delta;", "s.bary[D1 - s.rank[i]] += delta;"),
    ("barycentric index", "s.bary[D - s.rank[i]] += delta;", "s.bary[D1 - s.rank[i]] += delta;"),
    ("barycentric without the wrap-around term", "s.bary[0] += static_cast<R>(1) + s.bary[D1];", "s.bary[0] += static_cast<R>(1);"),
    ("vertex key off by one rank", "if (s.rank[i] > D - r) key[i] -= (D + 1);", "if (s.rank[i] >= D - r) key[i] -= (D + 1);"),
    ("forward weights reversed", "const R w = s.bary[r] * w_lvl;\n                for (int f = 0; f < F; ++f) acc[f]",
     "const R w = s.bary[D - r] * w_lvl;\n                for (int f = 0; f < F; ++f) acc[f]"),
    ("forward feature stride", "const int64_t h = static_cast<int64_t>(F) * lattice_slot<D>(key, C);\n                const R w = s.bary[r]",
     "const int64_t h = static_cast<int64_t>(2) * lattice_slot<D>(key, C);\n                const R w = s.bary[r]"),
    ("table backward weights reversed", "const R w = s.bary[r] * w_lvl;\n                for (int f = 0; f < F; ++f) {\n                    const R t = g[f] * w;",
     "const R w = s.bary[D - r] * w_lvl;\n                for (int f = 0; f < F; ++f) {\n                    const R t = g[f] * w;"),
    ("table backward swaps the features", "const R t = g[f] * w;", "const R t = g[F - 1 - f] * w;"),
    ("position backward drops the wrap-around term", "dB[D1] += dB[0];  //", "dB[D1] += 0;  //"),
    ("position backward second index", "dE[i] -= dB[D1 - s.rank[i]] * inv;", "dE[i] -= dB[D - s.rank[i]] * inv;"),
    ("position backward factor", "dP -= dE[i + 1] * sfl[i] * static_cast<R>(i + 1);", "dP -= dE[i + 1] * sfl[i] * static_cast<R>(i);"),
    ("position backward loop bound", "for (int j = 0; j <= i; ++j) dP += dE[j] * sfl[i];", "for (int j = 0; j < i; ++j) dP += dE[j] * sfl[i];"),
    ("double backward sign of the folded term", "dB[0] += dB[D1];\n}", "dB[0] -= dB[D1];\n}"),
    ("double backward factor", "for (int i = 0; i < D; ++i) dE[i + 1] -= q[i] * sf[i] * static_cast<R>(i + 1);",
     "for (int i = 0; i < D; ++i) dE[i + 1] -= q[i] * sf[i] * static_cast<R>(i);"),
    ("double backward prefix sums", "for (int j = 0; j <= i; ++j) dE[j] += g;", "for (int j = 0; j < i; ++j) dE[j] += g;"),
    ("grad-grad uses the other feature", "if (ggs) gg[f] += dB[r] * w_lvl * table[h + f];", "if (ggs) gg[f] += dB[r] * w_lvl * table[h + F - 1 - f];"),
    ("position backward drops a feature", "for (int f = 0; f < F; ++f) {\n                    dB[r] += tl[h + f] * w_lvl * g[f];",
     "for (int f = 1; f < F; ++f) {\n                    dB[r] += tl[h + f] * w_lvl * g[f];"),
    ("scale factor numerator", "std::sqrt(static_cast<double>((i + 1) * (i + 2)))", "std::sqrt(static_cast<double>((i + 1) * (i + 1)))"),
]

# The direction of an exact rounding tie (strict `<`, reference EncodingGPU.cuh:153-157).  With `<=` the
# tied coordinates get the smallest residuals instead of the largest and the coordinate sum grows by
# their number; after the rank wrap they are back in front, in index order: same rem0, rank,
# weights and slots.  The mutant is equivalent, so nothing can detect it.
TIE_DIRECTION = ("tie direction", "s.rem0[i] = (up - s.elevated[i] < s.elevated[i] - down)",
                 "s.rem0[i] = (up - s.elevated[i] <= s.elevated[i] - down)")
# Rounding every coordinate down instead of to the nearer multiple: the rank wrap then moves exactly the
# coordinates back up that nearest rounding would have rounded up (the enclosing simplex of a generic
# point has one representation with sum(rem0) = 0), so this is not observable either, except that
# residuals of the form e - down are no longer exact in fp32 and two nearly equal ones may swap ranks.
ALWAYS_DOWN = ("always rounds down", "s.rem0[i] = (up - s.elevated[i] < s.elevated[i] - down) ? static_cast<int>(up)",
               "s.rem0[i] = (false) ? static_cast<int>(up)")
# The one fused multiply-add of the elevation (`sm - i*cf` with one rounding, which the reference's
# compiler forms by default).  Unfused, the elevated coordinate moves by at most one unit in the
# last place: no invariant or closed form sees that; only a build of the reference could.
UNFUSED_ELEVATION = ("unfused elevation", "s.elevated[i] = fused_mul_add<R>(-static_cast<R>(i), cf, sm);",
                     "s.elevated[i] = sm - static_cast<R>(i) * cf;")


def build_mutant(tmp_dir, index, old, new):
    text = open(SOURCE).read()
    assert text.count(old) >= 1, f"the oracle no longer contains: {old}"
    src = os.path.join(tmp_dir, f"mutant_{index}.cpp")
    lib = os.path.join(tmp_dir, f"mutant_{index}.so")
    with open(src, "w") as f:
        f.write(text.replace(old, new, 1))
    subprocess.run(["g++"] + CXXFLAGS + ["-o", lib, src], check=True, capture_output=True)
    return lib


def pinning_suite_passes(lib):
    env = dict(os.environ, PENC_ORACLE_LIB=lib, OMP_NUM_THREADS="2")
    res = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_oracle_pinning.py"), "-x", "-q",
                          "-p", "no:cacheprovider"], cwd=ROOT, env=env, capture_output=True, text=True)
    return res.returncode == 0, res.stdout[-400:]


def test_every_seeded_mistake_fails_the_pinning_suite(tmp_path):
    def run(job):
        index, (name, old, new) = job
        passed, tail = pinning_suite_passes(build_mutant(str(tmp_path), index, old, new))
        return name, passed, tail

    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(run, enumerate(KILLED)))
    survivors = [name for name, passed, _ in results if passed]
    assert not survivors, f"mutants the pinning tests do not catch: {survivors}"


def _simplex_of(lib_path, pos, sf, shift, capacity):
    """Runs one oracle build in a child process (the library path is fixed when oracle.api is imported)."""
    code = (
        "import sys, numpy as np\n"
        "from oracle import api as orc\n"
        "a = np.load(sys.argv[1])\n"
        "o = orc.simplex(a['pos'], a['sf'], a['shift'], int(a['cap']))\n"
        "np.savez(sys.argv[2], **o)\n")
    work = os.path.dirname(lib_path)
    tag = os.path.basename(lib_path)
    np.savez(os.path.join(work, tag + "_in.npz"), pos=pos, sf=sf, shift=shift, cap=capacity)
    env = dict(os.environ, PENC_ORACLE_LIB=lib_path)
    subprocess.run([sys.executable, "-c", code, os.path.join(work, tag + "_in.npz"), os.path.join(work, tag + "_out.npz")],
                   cwd=ROOT, env=env, check=True, capture_output=True)
    return dict(np.load(os.path.join(work, tag + "_out.npz")))


@pytest.mark.parametrize("d", [2, 3, 4, 7])
def test_tie_direction_is_not_observable(tmp_path, d):
    """The `<=` mutant gives the oracle's rem0, rank, weights and slots on every point of a grid of
    exact ties, lattice points and face points (unit scale factors: coordinates in quarters)."""
    mutant = build_mutant(str(tmp_path), 0, TIE_DIRECTION[1], TIE_DIRECTION[2])
    original = build_mutant(str(tmp_path), 1, "kHashMul = 2531011u", "kHashMul = 2531011u")
    rng = np.random.default_rng(d)
    pos = (rng.integers(-40, 41, size=(50000, d)) * 0.25).astype(np.float32)
    pos[:400, 1:] = 0.0
    pos[:400, 0] = (np.arange(400) - 200) * 0.125 * (d + 1)
    sf, shift = np.ones((1, d), np.float32), np.zeros((1, d), np.float32)
    a = _simplex_of(original, pos, sf, shift, 1 << 16)
    b = _simplex_of(mutant, pos, sf, shift, 1 << 16)
    e = a["elevated"][0]
    v = e / (d + 1)
    assert np.sum(np.abs(v - np.floor(v) - 0.5) == 0) > 1000  # the grid does contain exact ties
    for k in ("rem0", "rank", "bary", "slot"):
        assert np.array_equal(a[k], b[k]), k


def test_rounding_direction_is_absorbed_by_the_rank_wrap(tmp_path):
    mutant = build_mutant(str(tmp_path), 0, ALWAYS_DOWN[1], ALWAYS_DOWN[2])
    original = build_mutant(str(tmp_path), 1, "kHashMul = 2531011u", "kHashMul = 2531011u")
    rng = np.random.default_rng(4)
    d = 4
    pos = rng.uniform(0, 1, (100000, d)).astype(np.float32)
    from oracle import api as orc
    sf = orc.scale_factors(d, np.geomspace(1.0, 1e-3, 6).astype(np.float32))
    shift = (rng.standard_normal((6, d)) * 10).astype(np.float32)
    a = _simplex_of(original, pos, sf, shift, 1 << 18)
    b = _simplex_of(mutant, pos, sf, shift, 1 << 18)
    assert np.array_equal(a["rem0"], b["rem0"])
    assert np.any(a["rank"] != b["rank"], axis=2).mean() < 1e-5


def test_unfused_elevation_only_moves_points_within_rounding_of_a_face(tmp_path):
    """Without the fused multiply-add the elevated coordinates move by at most one unit in the last
    place, which changes the simplex only for points that close to a face; the pinning suite cannot
    see it (stated in the oracle's header), and this test records how small the effect is."""
    mutant = build_mutant(str(tmp_path), 0, UNFUSED_ELEVATION[1], UNFUSED_ELEVATION[2])
    original = build_mutant(str(tmp_path), 1, "kHashMul = 2531011u", "kHashMul = 2531011u")
    passed, _ = pinning_suite_passes(mutant)
    assert passed, "the pinning suite now separates fused from unfused elevation: move this mutant to KILLED"
    rng = np.random.default_rng(9)
    d = 3
    pos = rng.uniform(0, 1, (200000, d)).astype(np.float32)
    sig = np.geomspace(1.0, 1e-4, 8).astype(np.float32)
    from oracle import api as orc
    sf = orc.scale_factors(d, sig)
    shift = (rng.standard_normal((8, d)) * 10).astype(np.float32)
    a = _simplex_of(original, pos, sf, shift, 1 << 18)
    b = _simplex_of(mutant, pos, sf, shift, 1 << 18)
    scale = np.maximum(np.abs(a["elevated"]).max(axis=2, keepdims=True), 1.0)
    assert np.all(np.abs(a["elevated"] - b["elevated"]) <= 4 * np.spacing(scale.astype(np.float32)))
    moved = np.any(a["rank"] != b["rank"], axis=2)
    assert moved.mean() < 1e-4
    # where the simplex is the same the weights agree to rounding; where it moved, the point sits on the shared face
    assert np.all(np.abs(a["bary"] - b["bary"])[~moved] <= 1e-5 * np.maximum(1.0, scale[..., 0][~moved])[:, None] + 1e-6)
