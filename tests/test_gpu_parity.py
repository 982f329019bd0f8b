"""Parity of the HIP kernels (called through the C ABI) with the CPU oracle, on the same seeded inputs.

Bars (stated by the task): simplex rank, remainder-0 point and hashed slots bit-exact; forward
features within 1e-5 relative / 1e-6 absolute; atomically accumulated gradients within 1e-4
relative (of the sum of the magnitudes of the accumulated terms, see helpers.assert_sum_close).
"""
import numpy as np
import pytest

from helpers import random_problem, assert_sum_close, make_encoding, gpu_input, to_gpu
from permutohedral_encoding_amd import workloads as wl

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
orc = pytest.importorskip("oracle.api")

DIMS = [2, 3, 4, 5, 6, 7, 8]
FWD_RTOL, FWD_ATOL = 1e-5, 1e-6
SUM_RTOL = 1e-4
POS_RTOL = 1e-6  # sums of at most a few dozen levels, no atomics: far inside the 1e-4 bar


def workload_problem(name, n):
    w = wl.WORKLOADS[name]
    p = wl.make_inputs(w, nr_points=n)
    p["sf"] = orc.scale_factors(w.pos_dim, p["sigmas"])
    return w, p


def check_forward(got, want):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = FWD_ATOL + FWD_RTOL * np.abs(want.astype(np.float64))
    assert np.all(err <= bound), f"forward: max err {err.max():.3g}, worst err/bound {np.max(err / bound):.3g}"


def check_pos_grad(got, want):
    """Position gradient against the oracle's fp64 sum of the same fp32 terms, per element, relative to
    the chain of magnitudes behind that element (what its rounding error scales with).  The levels
    are summed in a different but fixed order (pairs, then groups): observed worst case 8e-8."""
    err = np.abs(got.astype(np.float64) - want["grad64"])
    bound = POS_RTOL * want["abs64"] + 1e-30
    assert np.all(err <= bound), f"position gradient: worst err/bound {np.max(err / bound):.3g} at rel {POS_RTOL}"


def check_grad_grad(got, want):
    """Gradient w.r.t. grad_sliced_values: the kernel performs the oracle's fp32 operations in the
    oracle's order (no atomics are involved), so beyond the 1e-4 bar relative to the chain of
    magnitudes it must be the same bits."""
    err = np.abs(got.astype(np.float64) - want["ggs"].astype(np.float64))
    bound = SUM_RTOL * want["ggs_abs64"] + 1e-30
    assert np.all(err <= bound), f"grad-grad: worst err/bound {np.max(err / bound):.3g}"
    assert np.array_equal(got, want["ggs"]), f"grad-grad: {np.mean(got != want['ggs']):.3g} of the values differ in the last bits"


# ----------------------------------------------------------------------------- simplex, slots

@pytest.mark.parametrize("name", ["c2", "c3", "c4"])
def test_scale_factors_follow_torch_division_by_a_host_scalar(name):
    """The reference fills its scale-factor tensor with `t[l][i] = 1/sqrt((i+1)(i+2))` followed by
    `t[l][i] = t[l][i] / sigma_l` on a float32 GPU tensor (Encoding.cuh:62-63).  Those two statements,
    evaluated by torch itself on this GPU, must give the bits penc_scale_factors computes on the host
    (torch multiplies by the rounded reciprocal of a host scalar; a true division differs by one
    unit in the last place for about a quarter of the entries)."""
    from permutohedral_encoding_amd import _native
    w = wl.WORKLOADS[name]
    sig = wl.scale_list(w)
    t = torch.zeros((w.nr_levels, w.pos_dim), dtype=torch.float32, device="cuda")
    for l in range(w.nr_levels):
        for i in range(w.pos_dim):
            t[l][i] = 1.0 / np.sqrt(float((i + 1) * (i + 2)))
            t[l][i] = t[l][i] / float(sig[l])
    got = _native.scale_factors(w.pos_dim, sig)
    assert np.array_equal(got, t.cpu().numpy())
    assert np.array_equal(got, orc.scale_factors(w.pos_dim, sig))


def check_simplex_bit_exact(enc, pos, want, capacity):
    """rem0, rank, slots and weights of both device routines (select chains: scatter / position
    kernels; LDS rank sort: forward / grad-of-grad kernels) against the oracle, bit for bit."""
    pos_t = to_gpu(pos)
    for gather_path in (False, True):
        got = enc.simplex_debug(pos_t, capacity, gather_path=gather_path)
        for k in ("rem0", "rank", "slot"):
            assert np.array_equal(got[k].cpu().numpy(), want[k]), (k, gather_path)
        # the weights are computed with the same operations in the same order
        assert np.array_equal(got["barycentric"].cpu().numpy(), want["bary"]), gather_path
        del got


@pytest.mark.parametrize("d", DIMS)
def test_simplex_rank_and_slots_bit_exact_all_dims(d):
    cap = (1 << 19) if d != 5 else 100003  # one non-power-of-two capacity
    p = random_problem(d, 5000, 12, 4, seed=20 + d, sigma_range=(1.0, 1e-4))
    sf = orc.scale_factors(d, p["sigmas"])
    want = orc.simplex(p["pos"], sf, p["shift"], cap)
    enc, fp = make_encoding(d, p["sigmas"], p["shift"])
    assert np.array_equal(fp.m_scale_factor.cpu().numpy(), sf)
    check_simplex_bit_exact(enc, p["pos"], want, cap)


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_simplex_bit_exact_on_benchmark_configs(name):
    w, p = workload_problem(name, 1 << 14)
    want = orc.simplex(p["pos"], p["sf"], p["shift"], w.capacity)
    enc, _ = make_encoding(w.pos_dim, p["sigmas"], p["shift"])
    check_simplex_bit_exact(enc, p["pos"], want, w.capacity)


@pytest.mark.parametrize("d", DIMS)
def test_rounding_ties_and_lattice_points_bit_exact(d):
    """Points whose elevated coordinates sit exactly on rounding ties, on lattice points and on
    simplex faces (unit scale factors, no shift, coordinates that are multiples of 1/4): the two
    hand-worked tie cases of the oracle's pinning tests, then a grid of them against the oracle."""
    from test_oracle_pinning import TIE_CASES
    enc, fp = make_encoding(d, np.ones(1, np.float32), np.zeros((1, d), np.float32))
    fp.m_scale_factor = torch.ones((1, d), device="cuda")
    for dd, pos, _, rem0, rank, bary in TIE_CASES:
        if dd == d:
            for gather_path in (False, True):
                got = enc.simplex_debug(to_gpu(np.array([pos], np.float32)), 1 << 16, gather_path=gather_path)
                assert got["rem0"][0, 0].tolist() == rem0 and got["rank"][0, 0].tolist() == rank
                assert got["barycentric"][0, 0].tolist() == bary
    rng = np.random.default_rng(d)
    pos = (rng.integers(-40, 41, size=(20000, d)) * 0.25).astype(np.float32)
    pos[:200, 1:] = 0.0
    pos[:200, 0] = (np.arange(200) - 100) * 0.25 * (d + 1)  # walks through every tie of the first two coordinates
    want = orc.simplex(pos, np.ones((1, d), np.float32), np.zeros((1, d), np.float32), 1 << 16)
    check_simplex_bit_exact(enc, pos, want, 1 << 16)


# ----------------------------------------------------------------------------- the five configs, reduced N

@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_config_all_phases_match_oracle(name):
    w, p = workload_problem(name, 1 << 14)
    enc, _ = make_encoding(w.pos_dim, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    grad_t, dpos_t = to_gpu(p["grad"]), to_gpu(p["dpos"])

    out = enc.forward(inp).cpu().numpy()
    check_forward(out, orc.forward(p["pos"], p["table"], p["sf"], p["shift"], p["window"]))
    if w.masked_top_levels:
        assert np.all(out[w.nr_levels - w.masked_top_levels:] == 0.0)

    tg, pg = enc.backward(inp, grad_t)
    want = orc.backward_table(p["pos"], p["sf"], p["shift"], p["window"], p["grad"], w.capacity, want32=False, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient")
    del want
    check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], p["sf"], p["shift"], p["window"], p["grad"]))

    tg2, ggs = enc.double_backward_from_positions(inp, dpos_t, grad_t)
    want = orc.double_backward(p["pos"], p["table"], p["sf"], p["shift"], p["window"], p["dpos"], p["grad"],
                               want32=False, want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "double-backward table gradient")
    check_grad_grad(ggs.cpu().numpy(), want)


@pytest.mark.parametrize("d", DIMS)
def test_all_dims_all_phases_match_oracle(d):
    cap = 1 << 12  # small table: heavy slot sharing
    p = random_problem(d, 3000, 8, cap, seed=40 + d, sigma_range=(1.0, 1e-3))
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    check_forward(enc.forward(inp).cpu().numpy(), orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"]))
    tg, pg = enc.backward(inp, to_gpu(p["grad"]))
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient")
    check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"]))
    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "double-backward table gradient")
    check_grad_grad(ggs.cpu().numpy(), want)


# ----------------------------------------------------------------------------- four and eight features per level

@pytest.mark.parametrize("feat", [4, 8])
@pytest.mark.parametrize("d", DIMS)
def test_more_features_per_level_all_phases_match_oracle(d, feat):
    """nr_feat_per_level = 4 and 8 (the reference stops at 2): same algorithm, 16- and 32-byte slots; the
    table gradient scatters the feature pairs (0,1), (2,3), ... like levels.  All phases against the oracle."""
    cap = (1 << 12) if d != 4 else 5000  # one capacity that is not a power of two
    n, levels = 6000, 5
    p = random_problem(d, n, levels, cap, seed=60 + d + feat, sigma_range=(1.0, 1e-3), nr_feat=feat)
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    inp = gpu_input(p)
    out = enc.forward(inp).cpu().numpy()
    want = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"])
    assert out.shape == (levels, feat, n)
    check_forward(out, want)
    assert np.array_equal(out, want)
    tg, pg = enc.backward(inp, to_gpu(p["grad"]))
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert tg.shape == (levels, cap, feat)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient, %d features" % feat)
    check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"]))
    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "double-backward table gradient, %d features" % feat)
    check_grad_grad(ggs.cpu().numpy(), want)


@pytest.mark.parametrize("feat,n", [(4, 1 << 18), (8, 1 << 17)])
def test_more_features_at_benchmark_size_with_rows_and_concat_points(feat, n):
    """The headline geometry (3-D, 24 levels, 2^18 slots) with four and eight features per level: binned
    scatter over 48 and 96 feature pairs, the upstream gradient given as rows of F * (24 + 1) columns."""
    from permutohedral_encoding_amd import _native
    d, levels, cap = 3, 24, 1 << 18
    p = random_problem(d, n, levels, cap, seed=71, sigma_range=(1.0, 1e-4), nr_feat=feat)
    p["table"] *= 1e-2
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], concat_points=True, points_scaling=0.5, nr_feat=feat)
    inp = gpu_input(p)
    out = enc.forward(inp).cpu().numpy()
    want = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"], concat_points=True, points_scaling=0.5)
    assert out.shape == (levels + 1, feat, n) and np.array_equal(out, want)
    rows = torch.randn(n, feat * (levels + 1), device="cuda")
    view = rows.reshape(n, levels + 1, feat).permute(1, 2, 0)
    assert _native.is_row_major_view(view)
    level_major = np.ascontiguousarray(view[:levels].cpu().numpy())
    tg, pg = enc.backward(inp, view)
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], level_major, cap, want32=False, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient from rows, %d features" % feat)
    check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], level_major))
    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), view)
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], level_major,
                               concat_points=True, want32=False, want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "second-order table gradient from rows")
    check_grad_grad(ggs.cpu().numpy(), want)


# ----------------------------------------------------------------------------- table in half precision

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("feat", [2, 4, 8])
@pytest.mark.parametrize("d", [2, 3, 4, 8])
def test_half_precision_table_equals_the_widened_table(d, feat, dtype):
    """A float16 or bfloat16 table through the *_half entry points: the kernels widen on load and compute in fp32, so
    every result is that of the fp32 path on the widened table: forward and grad-of-grad bit-equal to the
    oracle run on it, position gradient within its bound, table gradients (which never read the table)
    fp32 as before.  Level-major and row-major upstream gradients."""
    from permutohedral_encoding_amd import _native
    cap = (1 << 12) if d != 3 else 5001  # odd capacity: slots of 2F bytes at odd offsets
    n, levels = 5000, 4
    p = random_problem(d, n, levels, cap, seed=130 + d + feat, sigma_range=(1.0, 1e-3), nr_feat=feat)
    half = torch.from_numpy(p["table"]).to(dtype)  # rounded by torch: the conversion a caller would use
    p["table"] = half.to(torch.float32).numpy()
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    inp = gpu_input(p)
    inp.m_lattice_values = half.cuda()
    out = enc.forward(inp).cpu().numpy()
    assert np.array_equal(out, orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"]))
    rows = to_gpu(np.ascontiguousarray(p["grad"].transpose(2, 0, 1).reshape(n, levels * feat)))
    view = rows.reshape(n, levels, feat).permute(1, 2, 0)
    assert _native.is_row_major_view(view)
    want_t = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    want_p = orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"])
    want_d = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    for grad in (to_gpu(p["grad"]), view):
        tg, pg = enc.backward(inp, grad)
        assert tg.dtype == torch.float32 and tg.shape == (levels, cap, feat)
        assert_sum_close(tg.cpu().numpy(), want_t["grad64"], want_t["abs64"], SUM_RTOL, "table gradient, half table")
        check_pos_grad(pg.cpu().numpy(), want_p)
        tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), grad)
        assert tg2.dtype == torch.float32
        assert_sum_close(tg2.cpu().numpy(), want_d["grad64"], want_d["abs64"], SUM_RTOL, "second-order table gradient, half table")
        check_grad_grad(ggs.cpu().numpy(), want_d)


# ----------------------------------------------------------------------------- edge cases

@pytest.mark.parametrize("n", [1, 63, 64, 65, 255, 256, 257, 4095, 4097, 10001])
def test_ragged_point_counts(n):
    d, cap = 3, 1 << 10
    p = random_problem(d, n, 5, cap, seed=n, sigma_range=(1.0, 1e-2))
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    check_forward(enc.forward(inp).cpu().numpy(), orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"]))
    tg, pg = enc.backward(inp, to_gpu(p["grad"]))
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient")
    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "double-backward table gradient")
    assert ggs.shape == (5, 2, n)


@pytest.mark.parametrize("cap", [1, 2, 7, 1000, 100003])
def test_unusual_capacities_and_total_collision(cap):
    d = 4
    p = random_problem(d, 2000, 6, cap, seed=cap, sigma_range=(1.0, 1e-3))
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    check_forward(enc.forward(inp).cpu().numpy(), orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"]))
    tg, _ = enc.backward(inp, to_gpu(p["grad"]))
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient")


def test_concat_points_extra_levels():
    for d in (2, 3, 4, 5):
        p = random_problem(d, 777, 3, 256, seed=d)
        sf = orc.scale_factors(d, p["sigmas"])
        enc, _ = make_encoding(d, p["sigmas"], p["shift"], concat_points=True, points_scaling=0.5)
        inp = gpu_input(p)
        out = enc.forward(inp).cpu().numpy()
        want = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"], concat_points=True, points_scaling=0.5)
        assert out.shape == want.shape
        check_forward(out, want)
        assert np.array_equal(out[3:], want[3:])
        extra = want.shape[0] - 3
        grad = np.concatenate([p["grad"], np.ones((extra, 2, 777), np.float32)])
        tg, pg = enc.backward(inp, to_gpu(grad))
        w = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], 256, want_abs=True)
        assert_sum_close(tg.cpu().numpy(), w["grad64"], w["abs64"], SUM_RTOL, "table gradient")
        tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(grad))
        assert ggs.shape == grad.shape and torch.all(ggs[3:] == 0)


def test_masked_levels_are_exact_zeros_and_noops():
    d, cap = 3, 1 << 12
    p = random_problem(d, 5000, 6, cap, seed=77)
    p["window"] = np.array([1, 1, 0.5, 0, 0, 0], np.float32)
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    out = enc.forward(inp)
    assert torch.all(out[3:] == 0)
    tg, pg = enc.backward(inp, to_gpu(p["grad"]))
    assert torch.all(tg[3:] == 0) and not torch.all(tg[:3] == 0)
    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    assert torch.all(tg2[3:] == 0) and torch.all(ggs[3:] == 0)
    check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"]))


def test_only_one_gradient_requested():
    d, cap = 3, 1 << 10
    p = random_problem(d, 1000, 4, cap, seed=5)
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    both = enc.backward(gpu_input(p), to_gpu(p["grad"]))
    tg, none = enc.backward(gpu_input(p, True, False), to_gpu(p["grad"]))
    assert none is None and torch.allclose(tg, both[0], rtol=1e-4, atol=1e-6)
    none, pg = enc.backward(gpu_input(p, False, True), to_gpu(p["grad"]))
    assert none is None and torch.equal(pg, both[1])
    assert enc.backward(gpu_input(p, False, False), to_gpu(p["grad"])) == (None, None)


def test_error_paths():
    d, cap = 3, 64
    p = random_problem(d, 10, 2, cap, seed=1)
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    from permutohedral_encoding_amd import _native
    good = gpu_input(p)
    with pytest.raises(ValueError, match="0 points"):
        enc.forward(_native.EncodingInput(good.m_lattice_values, good.m_positions_raw[:0], good.m_anneal_window, True, True))
    with pytest.raises(ValueError, match="Pos dim"):
        enc.forward(_native.EncodingInput(good.m_lattice_values, to_gpu(np.zeros((4, 2), np.float32)), good.m_anneal_window, True, True))
    with pytest.raises(ValueError, match="GPU memory"):
        enc.forward(_native.EncodingInput(good.m_lattice_values, good.m_positions_raw.cpu(), good.m_anneal_window, True, True))
    with pytest.raises(ValueError, match="type float"):
        enc.forward(_native.EncodingInput(good.m_lattice_values, good.m_positions_raw.double(), good.m_anneal_window, True, True))
    with pytest.raises(ValueError, match="anneal_window"):
        enc.forward(_native.EncodingInput(good.m_lattice_values, good.m_positions_raw, good.m_anneal_window[:1], True, True))
    with pytest.raises(ValueError, match="contiguous"):
        enc.backward(good, to_gpu(p["grad"]).transpose(0, 1).contiguous().transpose(0, 1))
    with pytest.raises(ValueError, match="contiguous"):
        enc.forward(_native.EncodingInput(good.m_lattice_values.transpose(0, 1), good.m_positions_raw, good.m_anneal_window, True, True))
    with pytest.raises(RuntimeError, match="pos_dim"):
        _native.EncodingWrapper.create(9, 2, None)
    with pytest.raises(RuntimeError, match="nr_feat_per_level"):
        _native.EncodingWrapper.create(3, 16, None)
    # strided positions are accepted (the reference indexes through accessors)
    pos2 = to_gpu(np.concatenate([p["pos"], p["pos"]], axis=1))[:, :3]
    out = enc.forward(_native.EncodingInput(good.m_lattice_values, pos2, good.m_anneal_window, True, True))
    assert torch.equal(out, enc.forward(good))


# ----------------------------------------------------------------------------- the five configs at their stated sizes

FULL_SIZE_PHASES = [(name, phase) for name in ("c1", "c2", "c3", "c4", "c5")
                    for phase in ("simplex",) + wl.WORKLOADS[name].phases]


@pytest.mark.parametrize("name,phase", FULL_SIZE_PHASES, ids=[f"{n}-{ph}" for n, ph in FULL_SIZE_PHASES])
def test_full_size_config_matches_oracle(name, phase):
    """Every phase a benchmark configuration names, at the configuration's own size (2^16 points for
    c1, 2^19 for c4, 2^20 otherwise), against the oracle on all points, levels and slots: the large
    point groups, the level interleave over the dies, the bins of a 2^22-slot table and the
    multi-workgroup bin reducer are only in use at these sizes."""
    w = wl.WORKLOADS[name]
    need = {"simplex": ("shift", "pos"), "forward": ("table", "shift", "pos"),
            "backward_table": ("shift", "pos", "grad"), "backward_pos": ("table", "shift", "pos", "grad"),
            "double_backward": ("table", "shift", "pos", "grad", "dpos")}[phase]
    p = wl.make_inputs(w, need=need)
    sf = orc.scale_factors(w.pos_dim, p["sigmas"])
    enc, _ = make_encoding(w.pos_dim, p["sigmas"], p["shift"])
    from permutohedral_encoding_amd import _native

    if phase == "simplex":  # in slabs of points: (L, N, D+1) int32 arrays of the oracle and of both device routines
        slab = 1 << 17
        for first in range(0, w.nr_points, slab):
            pos = p["pos"][first:first + slab]
            check_simplex_bit_exact(enc, pos, orc.simplex(pos, sf, p["shift"], w.capacity), w.capacity)
        return

    pos_t, win_t = to_gpu(p["pos"]), to_gpu(p["window"])
    table_t = to_gpu(p["table"]) if "table" in p else torch.zeros((w.nr_levels, 1, 2), device="cuda")
    if phase == "forward":
        out = enc.forward(_native.EncodingInput(table_t, pos_t, win_t, False, False)).cpu().numpy()
        want = orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"])
        check_forward(out, want)
        assert np.array_equal(out, want), "same fp32 operations in the same order: the bits must agree"
        if w.masked_top_levels:
            assert np.all(out[w.nr_levels - w.masked_top_levels:] == 0.0)
    elif phase == "backward_table":
        table_t = torch.zeros((w.nr_levels, w.capacity, 2), device="cuda")  # never read by the table gradient
        tg, _ = enc.backward(_native.EncodingInput(table_t, pos_t, win_t, True, False), to_gpu(p["grad"]))
        want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], w.capacity, want32=False, want_abs=True)
        assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient")
        if w.masked_top_levels:
            assert torch.all(tg[w.nr_levels - w.masked_top_levels:] == 0.0)
    elif phase == "backward_pos":
        _, pg = enc.backward(_native.EncodingInput(table_t, pos_t, win_t, False, True), to_gpu(p["grad"]))
        check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"]))
    else:
        tg2, ggs = enc.double_backward_from_positions(_native.EncodingInput(table_t, pos_t, win_t, True, True),
                                                      to_gpu(p["dpos"]), to_gpu(p["grad"]))
        want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"],
                                   want32=False, want_abs=True)
        assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "double-backward table gradient")
        check_grad_grad(ggs.cpu().numpy(), want)


# ----------------------------------------------------------------------------- size-independent properties at full size

@pytest.mark.parametrize("name", ["c2", "c3", "c4", "c5"])
def test_full_size_adjoint_identities(name):
    """forward is linear in the table and the position gradient bilinear in (table, grad), so at any size
        <forward(T), g> = <T, table_grad(g)>
        <q, pos_grad(T, g)> = <ggs(q, T), g> = <table_grad2(q, g), T>
    must hold (fp64 dot products of the fp32 results)."""
    w = wl.WORKLOADS[name]
    p = wl.make_inputs(w)
    enc, _ = make_encoding(w.pos_dim, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    grad_t, dpos_t = to_gpu(p["grad"]), to_gpu(p["dpos"])
    table = inp.m_lattice_values.double()

    out = enc.forward(inp)
    tg, pg = enc.backward(inp, grad_t)
    lhs = torch.sum(out.double() * grad_t.double()).item()
    rhs = torch.sum(tg.double() * table).item()
    scale = torch.sum(torch.abs(out.double() * grad_t.double())).item()
    assert abs(lhs - rhs) <= 1e-5 * scale, (lhs, rhs, scale)

    tg2, ggs = enc.double_backward_from_positions(inp, dpos_t, grad_t)
    a = torch.sum(dpos_t.double() * pg.double()).item()
    b = torch.sum(ggs.double() * grad_t.double()).item()
    c = torch.sum(tg2.double() * table).item()
    scale2 = torch.sum(torch.abs(ggs.double() * grad_t.double())).item()
    assert abs(a - b) <= 1e-4 * scale2 and abs(a - c) <= 1e-4 * scale2, (a, b, c, scale2)

    # atomics make the summation order vary between runs; the result must not vary beyond rounding
    tg_again, _ = enc.backward(inp, grad_t)
    assert torch.allclose(tg, tg_again, rtol=1e-3, atol=1e-6 * tg.abs().max().item())
    assert torch.equal(out, enc.forward(inp))

    # every slot: the binned scatter (workspace, large point groups at this size) against the
    # independent direct-atomics path (no workspace)
    from permutohedral_encoding_amd import _native
    saved = _native.LEVELS_PER_PASS
    _native.LEVELS_PER_PASS = -1
    try:
        tg_direct, _ = enc.backward(inp, grad_t)
        tg2_direct, _ = enc.double_backward_from_positions(inp, dpos_t, grad_t)
    finally:
        _native.LEVELS_PER_PASS = saved
    assert torch.allclose(tg, tg_direct, rtol=1e-3, atol=1e-5 * tg.abs().max().item())
    assert torch.allclose(tg2, tg2_direct, rtol=1e-3, atol=1e-5 * tg2.abs().max().item())


@pytest.mark.parametrize("name", ["c2", "c3"])
def test_full_size_table_gradients_do_not_depend_on_the_order_of_the_points(name):
    """A permutation of the batch permutes nothing in the table gradient.  The scatter treats an ordered batch
    differently at every level (folded runs of neighbouring lanes, columns sized from the second tile, the
    accumulate cache where unordered points stream), so equal sums for the benchmark's unordered points, the same
    points along a Z-order curve and the same points sorted by their first coordinate check those paths at the
    full size.  Bound per slot: 1e-5 of the sum of the magnitudes of its terms (first order: that sum is the
    gradient of |g|, since the barycentric weights are not negative), and 2e-5 of the level's largest entry
    for the second order, whose weights have both signs."""
    from permutohedral_encoding_amd import _native
    w = wl.WORKLOADS[name]
    p = wl.make_inputs(w)
    enc, _ = make_encoding(w.pos_dim, p["sigmas"], p["shift"])
    table_t = torch.zeros((w.nr_levels, w.capacity, 2), device="cuda")
    win_t = to_gpu(p["window"])
    second = "double_backward" in w.phases

    def gradients(order, grad):
        pos_t = to_gpu(np.ascontiguousarray(p["pos"][order]))
        grad_t = to_gpu(np.ascontiguousarray(grad[:, :, order]))
        inp = _native.EncodingInput(table_t, pos_t, win_t, True, False)
        tg, _ = enc.backward(inp, grad_t)
        tg2 = None
        if second:
            tg2, _ = enc.double_backward_from_positions(_native.EncodingInput(table_t, pos_t, win_t, True, True),
                                                        to_gpu(np.ascontiguousarray(p["dpos"][order])), grad_t)
        return tg.double(), None if tg2 is None else tg2.double()

    n, d = w.nr_points, w.pos_dim
    cells = np.clip((p["pos"] * 256).astype(np.int64), 0, 255)
    key = np.zeros(n, np.int64)
    for bit in range(8):
        for k in range(d):
            key |= ((cells[:, k] >> bit) & 1) << (bit * d + k)
    orders = {"Z-order": np.argsort(key, kind="stable"), "sorted by x": np.argsort(p["pos"][:, 0], kind="stable"),
              "reversed": np.arange(n)[::-1].copy()}
    identity = np.arange(n)
    base, base2 = gradients(identity, p["grad"])
    magnitude, _ = gradients(identity, np.abs(p["grad"]))
    for what, order in orders.items():
        got, got2 = gradients(order, p["grad"])
        excess = (torch.abs(got - base) - (1e-5 * magnitude + 1e-30)).max().item()
        assert excess <= 0.0, f"{name}, {what}: first-order table gradient differs by {excess:.3g} beyond the bound"
        if second:
            level_scale = base2.abs().amax(dim=(1, 2), keepdim=True)
            excess2 = (torch.abs(got2 - base2) - (2e-5 * level_scale + 1e-30)).max().item()
            assert excess2 <= 0.0, f"{name}, {what}: second-order table gradient differs by {excess2:.3g} beyond the bound"


def test_full_size_constant_table_gives_window():
    w = wl.WORKLOADS["c2"]
    p = wl.make_inputs(w, need=("shift", "pos"))
    enc, _ = make_encoding(w.pos_dim, p["sigmas"], p["shift"])
    from permutohedral_encoding_amd import _native
    table = torch.empty((w.nr_levels, w.capacity, 2), device="cuda")
    table[..., 0] = 2.0
    table[..., 1] = -3.0
    win = torch.linspace(0.1, 1.0, w.nr_levels, device="cuda")
    out = enc.forward(_native.EncodingInput(table, to_gpu(p["pos"]), win, False, False))
    assert torch.allclose(out[:, 0], (2.0 * win)[:, None].expand(-1, w.nr_points), rtol=1e-5)
    assert torch.allclose(out[:, 1], (-3.0 * win)[:, None].expand(-1, w.nr_points), rtol=1e-5)


# ----------------------------------------------------------------------------- scatter workspace

def _table_grads_with_workspace(enc, p, ws_bytes, d, cap, dpos=None):
    """Calls the C ABI directly with a workspace of the given size (None: no workspace)."""
    from permutohedral_encoding_amd import _native
    lib = _native.lib()
    fp = enc.fixed_params
    pos, table, win, grad = to_gpu(p["pos"]), to_gpu(p["table"]), to_gpu(p["window"]), to_gpu(p["grad"])
    n, levels = pos.shape[0], table.shape[0]
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda") if ws_bytes else None
    wp, wb = (ws.data_ptr(), ws_bytes) if ws is not None else (None, 0)
    tg = torch.full_like(table, float("nan"))  # the library must clear it itself
    st = torch.cuda.current_stream().cuda_stream
    if dpos is None:
        rc = lib.penc_backward(d, 2, n, levels, cap, pos.data_ptr(), table.data_ptr(), fp.m_scale_factor.data_ptr(),
                               fp.m_random_shift_per_level.data_ptr(), win.data_ptr(), grad.data_ptr(), tg.data_ptr(),
                               None, wp, wb, st)
    else:
        q = to_gpu(dpos)
        rc = lib.penc_double_backward_from_positions(d, 2, n, levels, cap, pos.data_ptr(), table.data_ptr(),
                                                     fp.m_scale_factor.data_ptr(), fp.m_random_shift_per_level.data_ptr(),
                                                     win.data_ptr(), q.data_ptr(), grad.data_ptr(), tg.data_ptr(), None,
                                                     0, wp, wb, st)
    assert rc == 0
    torch.cuda.synchronize()
    return tg.cpu().numpy()


@pytest.mark.parametrize("ws_bytes", [0, 4096, 40_000, 300_000, 3_000_000, 64_000_000])
def test_table_gradient_does_not_depend_on_the_workspace(ws_bytes):
    """No workspace (direct atomics), one too small to use, ones that force many passes and full
    bins (spill to atomics), and a roomy one must all give the same sums."""
    d, cap = 3, 1 << 15
    p = random_problem(d, 30000, 9, cap, seed=3, sigma_range=(1.0, 1e-3))
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    got = _table_grads_with_workspace(enc, p, ws_bytes, d, cap)
    assert_sum_close(got, want["grad64"], want["abs64"], SUM_RTOL, f"table gradient, workspace {ws_bytes}")
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    got = _table_grads_with_workspace(enc, p, ws_bytes, d, cap, dpos=p["dpos"])
    assert_sum_close(got, want["grad64"], want["abs64"], SUM_RTOL, f"double-backward table gradient, workspace {ws_bytes}")


def test_capped_workspace_takes_more_passes_and_gives_the_same_sums():
    from permutohedral_encoding_amd import _native
    d, cap, n, levels = 3, 1 << 16, 1 << 17, 10
    p = random_problem(d, n, levels, cap, seed=17, sigma_range=(1.0, 1e-3))
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    full = _native.lib().penc_scatter_workspace_bytes(d, n, levels, cap, 0)
    for limit in (None, full // 3, 1 << 16):   # one pass, several passes, too small to bin anything
        _native.MAX_WORKSPACE_BYTES = limit
        try:
            tg, pg = enc.backward(gpu_input(p), to_gpu(p["grad"]))
        finally:
            _native.MAX_WORKSPACE_BYTES = None
        assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, f"table gradient, workspace cap {limit}")
        check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"]))


def test_misaligned_workspace_and_odd_capacity():
    d, cap = 4, 50000  # not a multiple of the bin size: the last bin is partial
    p = random_problem(d, 20000, 6, cap, seed=8, sigma_range=(1.0, 1e-3))
    sf = orc.scale_factors(d, p["sigmas"])
    enc, fp = make_encoding(d, p["sigmas"], p["shift"])
    from permutohedral_encoding_amd import _native
    lib = _native.lib()
    pos, table, win, grad = to_gpu(p["pos"]), to_gpu(p["table"]), to_gpu(p["window"]), to_gpu(p["grad"])
    ws = torch.empty(8_000_000 + 64, dtype=torch.uint8, device="cuda")
    tg = torch.empty_like(table)
    rc = lib.penc_backward(d, 2, 20000, 6, cap, pos.data_ptr(), table.data_ptr(), fp.m_scale_factor.data_ptr(),
                           fp.m_random_shift_per_level.data_ptr(), win.data_ptr(), grad.data_ptr(), tg.data_ptr(), None,
                           ws.data_ptr() + 13, 8_000_000, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient")


def test_position_gradient_with_and_without_workspace():
    """Level groups with partial sums (workspace) and one thread walking all levels (no workspace)
    must agree with the oracle; the grouped result is deterministic."""
    from permutohedral_encoding_amd import _native
    d, cap = 4, 1 << 12
    p = random_problem(d, 5000, 7, cap, seed=12, sigma_range=(1.0, 1e-3))  # 7 levels: a ragged last group
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    want = orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"])
    results = []
    for lpp in (0, -1, 0):
        _native.LEVELS_PER_PASS = lpp
        try:
            _, pg = enc.backward(gpu_input(p, False, True), to_gpu(p["grad"]))
        finally:
            _native.LEVELS_PER_PASS = 0
        got = pg.cpu().numpy()
        check_pos_grad(got, want)
        results.append(got)
    assert np.array_equal(results[0], results[2])


def test_non_finite_points_do_not_disturb_their_neighbours():
    """A point with NaN, infinite or overflowing coordinates gets garbage (as in the reference), but
    the other points of its workgroup must come out exactly as without it, and nothing may fault."""
    d, cap, n = 3, 1 << 14, 4096
    p = random_problem(d, n, 8, cap, seed=31, sigma_range=(1.0, 1e-3))
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    clean = gpu_input(p)
    grad, dpos = to_gpu(p["grad"]), to_gpu(p["dpos"])
    out_clean = enc.forward(clean)
    _, pg_clean = enc.backward(clean, grad)
    _, ggs_clean = enc.double_backward_from_positions(clean, dpos, grad)

    bad_rows = [5, 64, 65, 1000, 4095]
    dirty_pos = p["pos"].copy()
    for row, value in zip(bad_rows, [np.nan, np.inf, -np.inf, 3e38, -1e30]):
        dirty_pos[row, row % d] = value
    q = dict(p)
    q["pos"] = dirty_pos
    dirty = gpu_input(q)
    out = enc.forward(dirty)
    tg, pg = enc.backward(dirty, grad)
    tg2, ggs = enc.double_backward_from_positions(dirty, dpos, grad)
    torch.cuda.synchronize()
    keep = torch.ones(n, dtype=torch.bool, device="cuda")
    keep[bad_rows] = False
    assert torch.equal(out[:, :, keep], out_clean[:, :, keep])
    assert torch.equal(pg[keep], pg_clean[keep])
    assert torch.equal(ggs[:, :, keep], ggs_clean[:, :, keep])
    assert tg.shape == tg2.shape == (8, cap, 2)


def test_many_bins_and_few_contributions_per_slot():
    """A 2^22-slot table: with enough points the scatter bins into 512 slot ranges (the records are
    appended one by one, not sorted by wave), with few points it goes straight to atomics (less than
    one contribution per eight slots).  Both against the oracle."""
    d, cap, levels = 3, 1 << 22, 3
    for n in (140000, 3000):
        p = random_problem(d, n, levels, cap, seed=12, sigma_range=(3e-2, 1e-3))
        sf = orc.scale_factors(d, p["sigmas"])
        enc, _ = make_encoding(d, p["sigmas"], p["shift"])
        inp = gpu_input(p, need_pos_grad=False)
        tg, _ = enc.backward(inp, to_gpu(p["grad"]))
        want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
        assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, f"table gradient, {n} points")


def test_table_gradient_plain_relative_tolerance_without_cancellation():
    """The table gradient is checked against 1e-4 of the sum of the magnitudes of its terms, because a sum
    with cancellation has no meaningful relative error.  Without cancellation the two readings
    coincide: with a non-negative upstream gradient every term (barycentric weight x window x gradient)
    is non-negative, and every element must be within 1e-4 of its own value.  The headline geometry
    at 2^18 points, every path of the scatter in use."""
    d, n, levels, cap = 3, 1 << 18, 24, 1 << 18
    p = random_problem(d, n, levels, cap, seed=77, sigma_range=(1.0, 1e-4))
    p["grad"] = np.abs(p["grad"])
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    tg, _ = enc.backward(gpu_input(p, need_pos_grad=False), to_gpu(p["grad"]))
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want32=False, want_abs=True)
    # no cancellation: the sum of the magnitudes is the sum itself (the oracle's threads add the two
    # in whatever order they arrive, so the fp64 sums agree to rounding, not bit for bit)
    np.testing.assert_allclose(want["abs64"], np.abs(want["grad64"]), rtol=1e-12, atol=0)
    got = tg.cpu().numpy().astype(np.float64)
    rel = np.abs(got - want["grad64"]) / np.maximum(np.abs(want["grad64"]), 1e-300)
    assert np.all((rel <= 1e-4) | (want["grad64"] == 0)), rel.max()
    assert np.all(got[want["grad64"] == 0] == 0)
    assert rel[want["grad64"] != 0].max() < 1e-5  # observed: a few units in the last place of fp32


def _table_gradients_match(p, d, cap, what):
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p, need_pos_grad=False)
    tg, _ = enc.backward(inp, to_gpu(p["grad"]))
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, what + ", table gradient")
    tg2, _ = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, what + ", second-order table gradient")


@pytest.mark.parametrize("d", [3, 4, 6])
def test_first_tile_misleads_the_scatter_about_the_level(d):
    """A scattering workgroup chooses how it accumulates a level (a column of cells per slot, the
    accumulate cache, or records sorted by bin) from the first 512 of its 4096 or 8192 points.  Points
    laid out so that the choice is wrong for the rest of the group: (a) the first 512 points of every
    group sit in one simplex at every level and the others are spread out, so the few columns overflow
    and the rest goes to bins or atomics contribution by contribution; (b) the first 512 are spread out
    and all the others sit in one simplex, so the sorted stream sends thousands of records to the
    same few bins and their segments overflow into direct atomics."""
    n, levels, cap = 3 * 8192 + 777, 6, 1 << 15
    rng = np.random.default_rng(90 + d)
    first_tile = (np.arange(n) % 4096) < 512
    cluster = (0.37 + 1e-7 * rng.standard_normal((n, d))).astype(np.float32)
    for what, clustered in (("columns overflow", first_tile), ("segments overflow", ~first_tile)):
        p = random_problem(d, n, levels, cap, seed=91 + d, sigma_range=(1.0, 1e-3))
        p["pos"] = np.where(clustered[:, None], cluster, p["pos"]).astype(np.float32)
        _table_gradients_match(p, d, cap, what)


@pytest.mark.parametrize("seed", range(12))
def test_table_gradients_on_mixed_point_distributions(seed):
    """Clusters of random size and spread mixed with uniform points, random dimension, capacity, level
    range and point count: levels land on either side of every threshold the scatter decides by
    (distinct slots of the first tile, its hit rate, bins or no bins), some workgroups of a level on
    one side and some on the other."""
    rng = np.random.default_rng(1000 + seed)
    d = int(rng.choice([2, 3, 4, 5]))
    cap = int(rng.choice([1 << 12, 1 << 15, 1 << 18, 30011]))
    n = int(rng.integers(3000, 40000))
    levels = 6
    fine = float(10.0 ** rng.uniform(-4, -1.5))
    p = random_problem(d, n, levels, cap, seed=2000 + seed, sigma_range=(1.0, fine))
    n_clusters = int(rng.integers(1, 40))
    centres = rng.uniform(0, 1, (n_clusters, d))
    spread = 10.0 ** rng.uniform(-6, -1, n_clusters)
    member = rng.integers(0, n_clusters, n)
    clustered = centres[member] + spread[member, None] * rng.standard_normal((n, d))
    uniform = rng.uniform(0, 1, (n, d))
    # runs of points alternate between the two kinds, so that the first tile of a group of points need not
    # look like the rest of it
    run = int(rng.choice([64, 512, 3000]))
    pick = ((np.arange(n) // run) % 2 == 0) if rng.random() < 0.7 else (rng.random(n) < rng.uniform(0.1, 0.9))
    p["pos"] = np.where(pick[:, None], clustered, uniform).astype(np.float32)
    _table_gradients_match(p, d, cap, f"seed {seed}: D={d} cap={cap} n={n} clusters={n_clusters}")


@pytest.mark.parametrize("d,samples,n,cap", [(3, 512, 70000, 1 << 18), (3, 128, 50000, 1 << 16), (4, 64, 40000, 1 << 18),
                                             (2, 1024, 60000, 1 << 14), (6, 256, 30000, 1 << 18), (3, 7, 30000, 30011)])
def test_table_gradients_on_points_in_spatial_order(d, samples, n, cap):
    """Batches whose consecutive points are neighbours in space: samples along rays (a tile of 512 points is one
    ray, a few rays, or many short ones) and points sorted along a space-filling curve.  Neighbouring lanes then add
    to the same slots (the fold of adjacent runs), every tile brings slots of its own (column mode must not be
    chosen from the first tile alone), and the first and second order table gradients must still be the oracle's."""
    levels = 7
    rng = np.random.default_rng(500 + d + samples)
    p = random_problem(d, n, levels, cap, seed=600 + d, sigma_range=(1.0, 3e-3))
    n_rays = (n + samples - 1) // samples
    origin = rng.uniform(0.2, 0.8, (n_rays, d))
    direction = rng.standard_normal((n_rays, d))
    direction /= np.linalg.norm(direction, axis=1, keepdims=True)
    along = (np.arange(samples) + rng.uniform(0, 1, (n_rays, samples))) / samples - 0.5
    rays = (origin[:, None, :] + 0.6 * along[:, :, None] * direction[:, None, :]).reshape(-1, d)[:n]
    p["pos"] = rays.astype(np.float32)
    _table_gradients_match(p, d, cap, f"rays of {samples} samples, D={d}")
    # the same points along a Z-order curve: neighbours in space without being runs along a line
    q = np.clip((rays * 256).astype(np.int64), 0, 255)
    key = np.zeros(n, np.int64)
    for bit in range(8):
        for k in range(d):
            key |= ((q[:, k] >> bit) & 1) << (bit * d + k)
    p["pos"] = rays[np.argsort(key, kind="stable")].astype(np.float32)
    _table_gradients_match(p, d, cap, f"Z-order, D={d}")


def test_segments_overflow_with_more_bins_than_lanes():
    """The same deception on a 2^20-slot table (128 slot ranges: the tile is sorted with one counter and
    one thread per bin): the first 512 points of every group are spread out, all the others sit in one
    simplex, so thousands of records head for a few segments sized for a few hundred."""
    d, n, levels, cap = 3, 6 * 8192 + 777, 5, 1 << 20
    rng = np.random.default_rng(123)
    p = random_problem(d, n, levels, cap, seed=124, sigma_range=(1.0, 1e-3))
    clustered = (np.arange(n) % 4096) >= 512
    cluster = (0.61 + 1e-7 * rng.standard_normal((n, d))).astype(np.float32)
    p["pos"] = np.where(clustered[:, None], cluster, p["pos"]).astype(np.float32)
    _table_gradients_match(p, d, cap, "segments overflow, 128 bins")


@pytest.mark.parametrize("feat,cap,levels,n", [(4, 1 << 21, 13, 90000), (2, (1 << 21) + 1, 7, 90000), (2, 1 << 22, 16, 140000)])
def test_many_bins_levels_shared_by_a_reducer_workgroup(feat, cap, levels, n):
    """Tables with hundreds of slot ranges, whose segments hold a few dozen records, are reduced by
    workgroups that keep their range and walk several levels: level lists that divide unevenly among
    them (26 pairs of features over 2 workgroups, 7 levels over 2, 16 in one), masked levels in
    between, coarse levels whose scattering workgroups add straight into the gradient (so the
    reducer must add to what is there), and one slot range past a power of two.  First- and
    second-order table gradients against the oracle."""
    from permutohedral_encoding_amd import _native
    d = 3
    p = random_problem(d, n, levels, cap, seed=300 + levels, sigma_range=(1.0, 2e-3), nr_feat=feat)
    p["window"][[1, levels - 2]] = 0.0
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    inp = gpu_input(p, need_pos_grad=False)
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    full = _native.lib().penc_scatter_workspace_bytes(d, n, levels * feat // 2, cap, 0)
    for limit in (None, full // 3):  # all levels in one pass; several passes, each with its own share of the flags
        _native.MAX_WORKSPACE_BYTES = limit
        try:
            tg, _ = enc.backward(inp, to_gpu(p["grad"]))
        finally:
            _native.MAX_WORKSPACE_BYTES = None
        assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, f"table gradient, workspace cap {limit}")
        assert not tg[1].any() and not tg[levels - 2].any()
    tg2, _ = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "second-order table gradient")


@pytest.mark.parametrize("cap,n,feat", [(1 << 23, 300000, 2), (5_000_011, 200000, 2), (1 << 25, 1 << 20, 2), (1 << 23, 300000, 4)])
def test_tables_above_2_22_slots_get_wider_bins(cap, n, feat):
    """Above 2^22 slots a bin spans 2^14 to 2^16 slots and its reducer workgroup sums it one range of 2^13
    slots after the other (up to 2^25 slots: 512 bins of 2^16).  Coarse levels that add straight
    into the gradient, a masked level, a capacity that is no power of two, four features; first- and
    second-order table gradients against the oracle.  (The oracle's sums are compared level by level:
    at 2^25 slots one level's fp64 sums are 1 GiB.)"""
    from permutohedral_encoding_amd import _native
    d, levels = 3, 5
    assert _native.lib().penc_scatter_workspace_bytes(d, n, levels * feat // 2, cap, 0) > 0
    p = random_problem(d, n, levels, 1, seed=41 + feat, sigma_range=(0.3, 2e-3), nr_feat=feat)
    p["window"][1] = 0.0
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    table = torch.zeros(levels, cap, feat, device="cuda")  # the table gradient does not read the table
    inp = _native.EncodingInput(table, to_gpu(p["pos"]), to_gpu(p["window"]), True, False)
    tg, _ = enc.backward(inp, to_gpu(p["grad"]))
    tg2, _ = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    assert not tg[1].any() and not tg2[1].any()
    for level in range(levels):
        one = slice(level, level + 1)
        args = (p["pos"], sf[one], p["shift"][one], p["window"][one])
        want = orc.backward_table(*args, p["grad"][one], cap, want_abs=True)
        assert_sum_close(tg[level].cpu().numpy()[None], want["grad64"], want["abs64"], SUM_RTOL, f"table gradient, level {level}")
        want = orc.double_backward(p["pos"], np.zeros((1, cap, feat), np.float32), sf[one], p["shift"][one], p["window"][one], p["dpos"], p["grad"][one], want_abs=True)
        assert_sum_close(tg2[level].cpu().numpy()[None], want["grad64"], want["abs64"], SUM_RTOL, f"second-order table gradient, level {level}")


@pytest.mark.parametrize("n", [(1 << 15) + 5, (1 << 16) + 77, (1 << 17) + 1])
def test_small_batches_take_smaller_groups(n):
    """Below 2^17 points (24 levels) the scattering workgroups take groups of two or four tiles instead of
    eight, so that the launch still fills the chip; the headline geometry at those sizes, first- and
    second-order table gradients against the oracle."""
    d, levels, cap = 3, 24, 1 << 18
    p = random_problem(d, n, levels, cap, seed=n % 1000, sigma_range=(1.0, 1e-4))
    _table_gradients_match(p, d, cap, f"{n} points")


def test_records_crowd_one_bin():
    """Points chosen so that, at the finest level, at least three of their four vertices fall into the
    first of four slot ranges: the tile's records are all distinct (the workgroup streams them sorted
    by bin) but one bin receives three quarters of them where its segments are sized for a quarter plus
    three standard deviations, so most chunks take the path that checks every record against the room
    left and spills the excess."""
    d, levels, cap = 3, 3, 1 << 15
    p = random_problem(d, 600000, levels, cap, seed=97, sigma_range=(1e-2, 1e-3))
    sf = orc.scale_factors(d, p["sigmas"])
    slots = orc.simplex(p["pos"], sf, p["shift"], cap)["slot"][levels - 1]  # (N, D+1)
    crowded = np.sum(slots < (1 << 13), axis=1) >= 3
    keep = np.flatnonzero(crowded)[:20000]
    assert len(keep) >= 18000
    p["pos"], p["dpos"], p["grad"] = p["pos"][keep], p["dpos"][keep], np.ascontiguousarray(p["grad"][:, :, keep])
    _table_gradients_match(p, d, cap, "one crowded bin")


@pytest.mark.parametrize("d", [2, 5, 6, 7])
def test_large_size_identities_in_the_other_dimensions(d):
    """The benchmark configurations cover D = 3, 4, 8 at full size; the same size-independent checks for
    the remaining dimensions, at sizes where the large point groups and interleaved levels are in use:
    adjoint identities, and every slot of the binned table gradients against the direct-atomics path."""
    from permutohedral_encoding_amd import _native
    n, levels, cap = 1 << 19, 16, 1 << 18
    p = random_problem(d, n, levels, cap, seed=50 + d, sigma_range=(1.0, 1e-3))
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    grad_t, dpos_t = to_gpu(p["grad"]), to_gpu(p["dpos"])
    table = inp.m_lattice_values.double()
    out = enc.forward(inp)
    tg, pg = enc.backward(inp, grad_t)
    tg2, ggs = enc.double_backward_from_positions(inp, dpos_t, grad_t)
    lhs = torch.sum(out.double() * grad_t.double()).item()
    rhs = torch.sum(tg.double() * table).item()
    scale = torch.sum(torch.abs(out.double() * grad_t.double())).item()
    assert abs(lhs - rhs) <= 1e-5 * scale, (lhs, rhs, scale)
    a = torch.sum(dpos_t.double() * pg.double()).item()
    b = torch.sum(ggs.double() * grad_t.double()).item()
    c = torch.sum(tg2.double() * table).item()
    scale2 = torch.sum(torch.abs(ggs.double() * grad_t.double())).item()
    assert abs(a - b) <= 1e-4 * scale2 and abs(a - c) <= 1e-4 * scale2, (a, b, c, scale2)
    saved = _native.LEVELS_PER_PASS
    _native.LEVELS_PER_PASS = -1
    try:
        tg_direct, _ = enc.backward(inp, grad_t)
        tg2_direct, _ = enc.double_backward_from_positions(inp, dpos_t, grad_t)
    finally:
        _native.LEVELS_PER_PASS = saved
    assert torch.allclose(tg, tg_direct, rtol=1e-3, atol=1e-5 * tg.abs().max().item())
    assert torch.allclose(tg2, tg2_direct, rtol=1e-3, atol=1e-5 * tg2.abs().max().item())


# ----------------------------------------------------------------------------- randomized geometries

def _random_geometry(seed):
    """Input dimension, features, capacity (powers of two and not, from a thousand slots to beyond 2^22),
    number of points and levels, scale range, masked level and workspace size, all drawn from `seed`."""
    rng = np.random.default_rng(1000 + seed)
    d = int(rng.integers(2, 9))
    feat = int(rng.choice([2, 2, 4, 8]))
    kind = int(rng.integers(0, 4))
    if kind == 0:
        cap = int(rng.integers(1 << 10, 1 << 19))
    elif kind == 1:
        cap = int(rng.integers(1 << 19, 1 << 22))
    elif kind == 2:
        cap = int(rng.integers(1 << 22, 1 << 23))
    else:
        cap = 1 << int(rng.integers(12, 24))
    cap = min(cap, ((1 << 31) - 1) // (feat * 6))
    n = int(rng.integers(1000, 200000))
    levels = int(rng.integers(1, 6))
    while levels > 1 and cap * feat * levels > 1 << 27:  # keeps the oracle's fp64 sums of the table gradient within a few GB
        levels -= 1
    sigma_lo = float(10 ** rng.uniform(-3.5, -1.0))
    masked = int(rng.integers(levels)) if levels > 2 and rng.random() < 0.4 else None
    workspace = ["full", "full", "third", "none"][int(rng.integers(0, 4))]
    return dict(d=d, feat=feat, cap=cap, n=n, levels=levels, sigma_lo=sigma_lo, masked=masked, workspace=workspace,
                problem_seed=int(rng.integers(1 << 30)))


@pytest.mark.parametrize("seed", range(20))
def test_random_geometry_all_phases_match_oracle(seed, monkeypatch):
    """Twenty seeded random problems through every phase against the oracle, the points unordered or in one of three
    orders.  Run under -x the suite stops at the first geometry that disagrees; the assertion message names it."""
    from permutohedral_encoding_amd import _native
    g = _random_geometry(seed)
    d, feat, cap, n, levels = g["d"], g["feat"], g["cap"], g["n"], g["levels"]
    what = f"seed {seed}: {g}"
    p = random_problem(d, n, levels, 1, seed=g["problem_seed"], sigma_range=(1.0, g["sigma_lo"]), nr_feat=feat)
    # three seeds in four hand the points over in an order: along a Z-order curve, sorted by their first coordinate,
    # or in runs of identical points (the scatter folds neighbouring lanes and sizes its column tables from the second tile)
    order = seed % 4
    if order == 1:
        cells = np.clip((p["pos"] * 256).astype(np.int64), 0, 255)
        key = np.zeros(n, np.int64)
        for bit in range(7):
            for k in range(d):
                key |= ((cells[:, k] >> bit) & 1) << (bit * d + k)
        p["pos"] = np.ascontiguousarray(p["pos"][np.argsort(key, kind="stable")])
    elif order == 2:
        p["pos"] = np.ascontiguousarray(p["pos"][np.argsort(p["pos"][:, 0], kind="stable")])
    elif order == 3:
        run = int(np.random.default_rng(seed).choice([2, 7, 64, 700]))
        p["pos"] = np.ascontiguousarray(np.repeat(p["pos"][: (n + run - 1) // run], run, axis=0)[:n])
    what += f", point order {order}"
    if g["masked"] is not None:
        p["window"][g["masked"]] = 0.0
    p["table"] = np.random.default_rng(g["problem_seed"] + 1).uniform(-1, 1, (levels, cap, feat)).astype(np.float32)
    sf = orc.scale_factors(d, p["sigmas"])
    if g["workspace"] == "none":
        monkeypatch.setattr(_native, "MAX_WORKSPACE_BYTES", 0)
    elif g["workspace"] == "third":
        full = int(_native.lib().penc_scatter_workspace_bytes(d, n, levels * feat // 2, cap, 0))
        monkeypatch.setattr(_native, "MAX_WORKSPACE_BYTES", max(full // 3, 1 << 16))
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    inp = gpu_input(p)

    want = orc.simplex(p["pos"], sf, p["shift"], cap)
    for gather_path in (False, True):
        dbg = enc.simplex_debug(to_gpu(p["pos"]), cap, gather_path=gather_path)
        assert np.array_equal(dbg["slot"].cpu().numpy(), want["slot"]), what
        assert np.array_equal(dbg["rank"].cpu().numpy(), want["rank"]), what
        del dbg
    out = enc.forward(inp).cpu().numpy()
    assert np.array_equal(out, orc.forward(p["pos"], p["table"], sf, p["shift"], p["window"])), what

    tg, pg = enc.backward(inp, to_gpu(p["grad"]))
    wt = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), wt["grad64"], wt["abs64"], SUM_RTOL, f"table gradient, {what}")
    check_pos_grad(pg.cpu().numpy(), orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"]))
    del tg, pg, wt

    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(p["dpos"]), to_gpu(p["grad"]))
    wd = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], p["grad"], want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), wd["grad64"], wd["abs64"], SUM_RTOL, f"second-order table gradient, {what}")
    check_grad_grad(ggs.cpu().numpy(), wd)


# ----------------------------------------------------------------------------- sparse table gradient

def _touched_slots(sparse, level, pair):
    """Boolean (capacity,) array: slots whose range the map marks, for one level and pair of features."""
    m = sparse.touched_map()[level, pair].cpu().numpy() != 0
    return np.repeat(m, sparse.range_slots)[:sparse.capacity]


@pytest.mark.parametrize("d,feat,cap,n,levels,rows", [
    (3, 2, 1 << 18, 150000, 5, False),     # binned, slot ranges of 8192
    (4, 4, 100003, 60000, 3, True),        # not a power of two, two pairs of features, row-major upstream gradient
    (3, 2, 1 << 23, 120000, 3, False),     # ranges wider than a reducer's LDS
    (5, 2, 1 << 20, 3000, 4, False),       # too few contributions for binning: every add goes straight into the gradient
    (2, 8, 5000, 20000, 6, True),          # a single slot range per level
])
def test_sparse_table_gradient_accumulates_and_is_cleared(d, feat, cap, n, levels, rows):
    """penc_backward_sparse and penc_double_backward_from_positions_sparse add into one gradient kept
    across calls and mark the slot ranges they reach; penc_clear_touched restores the all-zero state.
    Twice in a row, the second time with fewer points, against the oracle's sums."""
    from permutohedral_encoding_amd import _native
    p = random_problem(d, n, levels, 1, seed=77 + d, sigma_range=(1.0, 2e-3), nr_feat=feat)
    if levels > 3:
        p["window"][2] = 0.0  # a masked level touches nothing
    p["table"] = np.random.default_rng(3).uniform(-1, 1, (levels, cap, feat)).astype(np.float32)
    sf = orc.scale_factors(d, p["sigmas"])
    enc, _ = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    enc.sparse_table_grad = True
    table = to_gpu(p["table"])
    for count in (n, n // 3):
        pos, dpos = p["pos"][:count], p["dpos"][:count]
        grad = np.ascontiguousarray(p["grad"][:, :, :count])
        inp = _native.EncodingInput(table, to_gpu(pos), to_gpu(p["window"]), True, True)
        g_dev = to_gpu(grad)
        if rows:  # the (L, F, N) view of rows (N, F*L) autograd hands over
            g_dev = to_gpu(np.ascontiguousarray(grad.transpose(2, 0, 1).reshape(count, -1))).view(count, levels, feat).permute(1, 2, 0)
        tg, pg = enc.backward(inp, g_dev)
        assert tg is None
        sparse = enc.sparse_grad
        first = orc.backward_table(pos, sf, p["shift"], p["window"], grad, cap, want_abs=True)
        assert_sum_close(sparse.grad.cpu().numpy(), first["grad64"], first["abs64"], SUM_RTOL, "sparse table gradient")
        check_pos_grad(pg.cpu().numpy(), orc.backward_pos(pos, p["table"], sf, p["shift"], p["window"], grad))
        tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(dpos), g_dev)
        assert tg2 is None and enc.sparse_grad is sparse
        second = orc.double_backward(pos, p["table"], sf, p["shift"], p["window"], dpos, grad, want_abs=True)
        check_grad_grad(ggs.cpu().numpy(), second)
        got = sparse.grad.cpu().numpy()
        assert_sum_close(got, first["grad64"] + second["grad64"], first["abs64"] + second["abs64"], SUM_RTOL,
                         "sum of the two sparse table gradients")
        # the map covers every slot that holds anything, and a masked level is not marked at all
        for level in range(levels):
            for pair in range(feat // 2):
                marked = _touched_slots(sparse, level, pair)
                held = np.any(got[level][:, 2 * pair:2 * pair + 2] != 0, axis=1)
                assert not np.any(held & ~marked), (level, pair)
                if p["window"][level] == 0.0:
                    assert not marked.any()
        sparse.clear()
        assert not sparse.touched.any().item() and not sparse.grad.any().item()
    enc.sparse_table_grad = False
    tg, _ = enc.backward(_native.EncodingInput(table, to_gpu(p["pos"]), to_gpu(p["window"]), True, False), to_gpu(p["grad"]))
    assert tg is not None  # the dense path is untouched by the switch
