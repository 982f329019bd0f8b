"""penc_backward_static (the entry point that allocates nothing) against penc_backward, through the C ABI.

Two calls in a row on the same GPU, the second with a smaller input: the static scratch keeps the
first call's records, and the second call must not see them.  Bars: the position gradient is computed
by the same deterministic kernels, so it is bit-equal whenever both calls can use level groups;
the table gradient is an atomically accumulated sum, held to 1e-4 of the sum of magnitudes of its
terms (the oracle supplies that sum) against both the existing entry point and the oracle.
"""
import numpy as np
import pytest

from helpers import random_problem, assert_sum_close, make_encoding, to_gpu

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
orc = pytest.importorskip("oracle.api")

SUM_RTOL = 1e-4


def _both_entry_points(d, n, levels, cap, seed, feat=2):
    from permutohedral_encoding_amd import _native
    lib = _native.lib()
    p = random_problem(d, n, levels, cap, seed=seed, sigma_range=(1.0, 1e-3), nr_feat=feat)
    sf = orc.scale_factors(d, p["sigmas"])
    enc, fp = make_encoding(d, p["sigmas"], p["shift"], nr_feat=feat)
    pos, table, win, grad = to_gpu(p["pos"]), to_gpu(p["table"]), to_gpu(p["window"]), to_gpu(p["grad"])
    st = torch.cuda.current_stream().cuda_stream
    common = (d, feat, n, levels, cap, pos.data_ptr(), table.data_ptr(), fp.m_scale_factor.data_ptr(),
              fp.m_random_shift_per_level.data_ptr(), win.data_ptr(), grad.data_ptr())

    ws_bytes = max(int(lib.penc_scatter_workspace_bytes(d, n, levels * feat // 2, cap, 0)),
                   int(lib.penc_positions_workspace_bytes(d, n, levels)))
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda")
    tg_ref = torch.full_like(table, float("nan"))
    pg_ref = torch.full_like(pos, float("nan"))
    assert lib.penc_backward(*common, tg_ref.data_ptr(), pg_ref.data_ptr(), ws.data_ptr(), ws_bytes, st) == 0

    tg = torch.full_like(table, float("nan"))
    pg = torch.full_like(pos, float("nan"))
    # The entry point allocates nothing: neither through torch's caching allocator nor from the device
    # directly.  The first call on a GPU looks up the scratch's address; the calls compared are later ones.
    assert lib.penc_backward_static(*common, tg.data_ptr(), pg.data_ptr(), st) == 0
    torch.cuda.synchronize()
    tg.fill_(float("nan"))
    pg.fill_(float("nan"))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    assert lib.penc_backward_static(*common, tg.data_ptr(), pg.data_ptr(), st) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed across penc_backward_static"

    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], p["grad"], cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "static-scratch table gradient vs oracle")
    diff = (tg.double() - tg_ref.double()).abs().cpu().numpy()
    assert np.all(diff <= 2 * SUM_RTOL * want["abs64"] + 1e-30), "static-scratch table gradient vs penc_backward"
    wantp = orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], p["grad"])["grad64"]
    scale = np.abs(wantp).max(axis=1, keepdims=True)
    assert np.all(np.abs(pg.cpu().numpy() - wantp) <= SUM_RTOL * (np.abs(wantp) + scale) + 1e-30)
    return pg, pg_ref


def test_static_scratch_backward_matches_the_workspace_entry_point_twice():
    lib = __import__("permutohedral_encoding_amd")._native.lib()
    assert lib.penc_static_scratch_bytes() == 64 << 20
    # first call: several passes over the levels (one level's records take about a third of the scratch)
    pg, pg_ref = _both_entry_points(3, 400_000, 10, 1 << 16, seed=101)
    # second call, smaller, straight after: groups, bins and segment sizes all differ from the first call's
    pg, pg_ref = _both_entry_points(3, 30_000, 6, 1 << 15, seed=102)
    assert torch.equal(pg, pg_ref)  # the partial sums fit the scratch here: same kernels, same order
    # and once more with another dimension and a capacity that is not a power of two
    _both_entry_points(5, 9_000, 5, 50_000, seed=103)
    # four features per level: every pair of features is scattered like a level of its own
    _both_entry_points(3, 120_000, 4, 1 << 16, seed=104, feat=4)


def test_static_scratch_rejects_what_does_not_fit_and_enqueues_nothing():
    from permutohedral_encoding_amd import _native
    lib = _native.lib()
    d, n, levels, cap = 3, 1 << 22, 2, 1 << 18  # one level's records need about 220 MiB
    assert lib.penc_scatter_workspace_bytes(d, n, levels, cap, 1) > lib.penc_static_scratch_bytes()
    sentinel = torch.full((levels, cap, 2), 7.0, device="cuda")
    some = torch.zeros(16, device="cuda")  # never dereferenced: the size check comes first
    rc = lib.penc_backward_static(d, 2, n, levels, cap, some.data_ptr(), some.data_ptr(), some.data_ptr(),
                                  some.data_ptr(), some.data_ptr(), some.data_ptr(), sentinel.data_ptr(), None,
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 7 and b"static scratch" in lib.penc_status_string(rc)
    torch.cuda.synchronize()
    assert torch.all(sentinel == 7.0)
