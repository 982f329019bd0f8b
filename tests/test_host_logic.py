"""CPU-side checks: the C-ABI library loads and exports what include/penc.h declares, the host
functions match their closed forms / the oracle, and the Python surface mirrors the reference's."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

import permutohedral_encoding_amd as pe
from permutohedral_encoding_amd import _native, workloads
from oracle import api as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header="penc.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(penc_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 9
    handle = ctypes.CDLL(_native.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f"{n} is declared in include/penc.h but not exported"
    assert set(names) == set(_native.EXPORTED_SYMBOLS)
    assert not [n for n in names if "probe" in n]  # measurement aids live in their own library
    from permutohedral_encoding_amd import probes
    probe_names = declared_functions("penc_probes.h")
    handle = ctypes.CDLL(probes.LIB_PATH)
    for n in probe_names:
        assert hasattr(handle, n), f"{n} is declared in include/penc_probes.h but not exported"
    assert set(probe_names) == set(probes.EXPORTED_SYMBOLS) and len(probe_names) == 5


def test_status_strings_and_extra_levels():
    lib = _native.lib()
    assert lib.penc_status_string(0) == b"ok"
    assert b"pos_dim" in lib.penc_status_string(3)
    assert b"nr_feat_per_level must be 2, 4 or 8" in lib.penc_status_string(4)
    for d in range(2, 9):
        assert _native.extra_levels(d, 2, False) == 0
        assert _native.extra_levels(d, 2, True) == math.ceil(d / 2) == orc.extra_levels(d, True)


def test_argument_validation_without_a_gpu():
    """The entry points validate before they launch, so the error codes can be checked on a CPU-only host."""
    lib = _native.lib()
    z = ctypes.c_void_p(0)
    buf = np.zeros(64, np.float32)
    p = buf.ctypes.data
    assert lib.penc_forward(9, 2, 10, 2, 16, p, p, p, p, p, p, 0, 1.0, None) == 3
    assert lib.penc_forward(1, 2, 10, 2, 16, p, p, p, p, p, p, 0, 1.0, None) == 3
    assert lib.penc_forward(3, 16, 10, 2, 16, p, p, p, p, p, p, 0, 1.0, None) == 4
    assert lib.penc_forward(3, 3, 10, 2, 16, p, p, p, p, p, p, 0, 1.0, None) == 4
    assert lib.penc_forward(3, 4, 10, 2, 16, p, p + 8, p, p, p, p, 0, 1.0, None) == 5  # four features: 16-byte slots
    assert lib.penc_forward(3, 2, 0, 2, 16, p, p, p, p, p, p, 0, 1.0, None) == 2
    assert lib.penc_forward(3, 2, 10, 0, 16, p, p, p, p, p, p, 0, 1.0, None) == 2
    assert lib.penc_forward(3, 2, 10, 2, 0, p, p, p, p, p, p, 0, 1.0, None) == 2
    assert lib.penc_forward(3, 2, 1 << 30, 24, 16, p, p, p, p, p, p, 0, 1.0, None) == 2
    assert lib.penc_forward(3, 2, 10, 2, 16, z, p, p, p, p, p, 0, 1.0, None) == 1
    assert lib.penc_forward(3, 2, 10, 2, 16, p, p + 4, p, p, p, p, 0, 1.0, None) == 5
    assert lib.penc_backward(3, 2, 10, 2, 16, p, p, p, p, p, p, z, z, None, 0, None) == 1
    assert lib.penc_backward(3, 2, 10, 2, 16, p, z, p, p, p, p, z, p, None, 0, None) == 1
    assert lib.penc_double_backward_from_positions(3, 2, 10, 2, 16, p, p, p, p, p, p, p, z, z, 0, None, 0, None) == 1
    assert lib.penc_simplex_debug(3, 0, 2, 16, p, p, p, 0, z, z, z, z, None) == 2
    # the sparse table gradient: gradient and map are both required; the map's size follows the slot ranges
    assert lib.penc_backward_sparse(3, 2, 10, 2, 16, p, p, p, p, p, p, 0, p, z, z, None, 0, None) == 1
    assert lib.penc_backward_sparse(3, 2, 10, 2, 16, p, p, p, p, p, p, 0, z, p, z, None, 0, None) == 1
    assert lib.penc_backward_sparse(9, 2, 10, 2, 16, p, p, p, p, p, p, 0, p, p, z, None, 0, None) == 3
    assert lib.penc_double_backward_from_positions_sparse(3, 2, 10, 2, 16, p, p, p, p, p, p, p, 0, p, z, p, 0, None, 0, None) == 1
    assert lib.penc_double_backward_from_positions_sparse(3, 2, 10, 2, 16, p, p, p, p, p, p, p, 3, p, p, p, 0, None, 0, None) == 2  # odd row stride
    assert lib.penc_touched_map_entries(2, 24, 1 << 18) == 24 * 32 and lib.penc_touched_range_slots(1 << 18) == 8192
    assert lib.penc_touched_map_entries(8, 3, 1 << 22) == 3 * 4 * 512 and lib.penc_touched_range_slots(1 << 22) == 8192
    assert lib.penc_touched_map_entries(2, 1, 1 << 24) == 512 and lib.penc_touched_range_slots(1 << 24) == 1 << 15
    assert lib.penc_touched_map_entries(2, 5, 100003) == 5 * 13 and lib.penc_touched_map_entries(3, 5, 100) == 0
    assert lib.penc_adamw_step_sparse(p, p, p, p, 2, 2, 16, z, 1e-3, 0.9, 0.99, 1e-8, 0.0, 1, 1, None) == 1
    assert lib.penc_adamw_step_sparse(p, p, p, p, 2, 2, 16, p, 1e-3, 0.9, 0.99, 1e-8, 0.0, 0, 1, None) == 2  # steps count from 1
    assert lib.penc_adamw_step_sparse(p, p, p, p, 3, 2, 16, p, 1e-3, 0.9, 0.99, 1e-8, 0.0, 1, 1, None) == 4
    assert lib.penc_adamw_step_sparse(p, p + 4, p, p, 2, 2, 16, p, 1e-3, 0.9, 0.99, 1e-8, 0.0, 1, 1, None) == 5
    assert lib.penc_clear_touched(z, 2, 2, 16, p, None) == 1 and lib.penc_clear_touched(p, 2, 0, 16, p, None) == 2
    # dense rows from the forward: the workspace must hold the level-major array
    assert lib.penc_forward_rowmajor(3, 2, 10, 2, 16, p, p, p, p, p, z, 4, 0, 1.0, p, 1 << 20, None) == 1
    assert lib.penc_forward_rowmajor(3, 2, 10, 2, 16, p, p, p, p, p, p, 3, 0, 1.0, p, 1 << 20, None) == 2  # rows shorter than F * L
    assert lib.penc_forward_rowmajor(3, 2, 10, 2, 16, p, p, p, p, p, p, 4, 0, 1.0, p, 16, None) == 8
    assert lib.penc_forward_rowmajor(3, 2, 10, 2, 16, p, p, p, p, p, p, 4, 0, 1.0, None, 0, None) == 8
    assert lib.penc_forward_rowmajor_workspace_bytes(3, 2, 10, 2, 0) == 4 * 2 * 2 * 10 + 256
    assert lib.penc_forward_rowmajor_workspace_bytes(3, 2, 10, 2, 1) == 4 * 2 * 4 * 10 + 256
    # a table in half precision: slots of 2F bytes (4 for two features, 16 for eight)
    assert lib.penc_forward_half(3, 2, 10, 2, 16, p, p + 2, 1, p, p, p, p, 0, 1.0, None) == 5
    assert lib.penc_forward_half(3, 8, 10, 2, 16, p, p + 8, 2, p, p, p, p, 0, 1.0, None) == 5
    assert lib.penc_forward_half(3, 2, 10, 2, 16, p, z, 1, p, p, p, p, 0, 1.0, None) == 1
    assert lib.penc_forward_half(3, 2, 10, 2, 16, p, p, 0, p, p, p, p, 0, 1.0, None) == 9  # neither binary16 nor bfloat16
    assert lib.penc_forward_half(3, 2, 10, 2, 16, p, p, 3, p, p, p, p, 0, 1.0, None) == 9
    assert lib.penc_backward_half(3, 2, 10, 2, 16, p, z, 1, p, p, p, p, 0, z, p, None, 0, None) == 1  # position gradient needs the table
    assert lib.penc_backward_half(3, 2, 10, 2, 16, p, p, 2, p, p, p, p, 3, p, z, None, 0, None) == 2  # odd row stride
    assert lib.penc_backward_half(3, 2, 10, 2, 16, p, p, 7, p, p, p, p, 0, p, z, None, 0, None) == 9
    assert lib.penc_double_backward_from_positions_half(3, 2, 10, 2, 16, p, p, 1, p, p, p, p, p, 0, z, z, 0, None, 0, None) == 1
    assert lib.penc_double_backward_from_positions_half(3, 2, 10, 2, 16, p, p, 0, p, p, p, p, p, 0, p, p, 0, None, 0, None) == 9
    # the optimizer step
    assert lib.penc_adamw_step(z, p, p, p, 16, 1e-3, 0.9, 0.99, 1e-8, 0.0, 1, 0, None) == 1
    assert lib.penc_adamw_step(p, p, p, p, 0, 1e-3, 0.9, 0.99, 1e-8, 0.0, 1, 0, None) == 2
    assert lib.penc_adamw_step(p, p, p, p, 16, 1e-3, 0.9, 0.99, 1e-8, 0.0, 0, 0, None) == 2  # steps count from 1
    assert lib.penc_backward_static(3, 2, 0, 2, 16, p, p, p, p, p, p, p, z, None) == 2
    assert lib.penc_backward_static(3, 2, 1 << 24, 2, 1 << 18, p, p, p, p, p, p, p, z, None) == 7  # before any pointer is read
    assert lib.penc_scale_factors(3, 2, z, p) == 1
    # workspace sizing: grows with the levels per pass, 0 when the capacity cannot be binned
    w1 = lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 18, 1)
    w4 = lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 18, 4)
    assert 0 < w1 < w4 <= 4 * w1 and lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 18, 100) <= 24 * w1
    assert lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 22, 4) > 0
    assert lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, (1 << 22) + 1, 4) > 0  # wider slot ranges up to 2^25 slots
    assert lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 25, 4) > 0
    assert lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, (1 << 25) + 1, 4) == 0
    assert lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 18, 0) == lib.penc_scatter_workspace_bytes(3, 1 << 20, 24, 1 << 18, 24)


@pytest.mark.parametrize("d", range(2, 9))
def test_scale_factors_match_oracle_and_closed_form(d):
    sig = np.geomspace(1.0, 1e-4, 24).astype(np.float32)
    sf = _native.scale_factors(d, sig)
    assert np.array_equal(sf, orc.scale_factors(d, sig))
    i = np.arange(d, dtype=np.float64)
    want = 1.0 / (np.sqrt((i + 1) * (i + 2))[None, :] * sig.astype(np.float64)[:, None])
    assert np.all(np.abs(sf - want) <= 2.0 * np.spacing(want.astype(np.float32)))


def test_cosine_window_and_coarse2fine():
    c2f = pe.Coarse2Fine(24)
    win = c2f(16 / 24)
    assert win.dtype == torch.float32 and win.shape == (24,)
    assert torch.equal(win, torch.tensor([1.0] * 16 + [0.0] * 8))  # exactly, not approximately
    assert c2f.get_last_t() == 16 / 24
    assert torch.equal(c2f(1.0), torch.ones(24))
    assert torch.equal(c2f(0.0), torch.zeros(24))
    w = c2f(0.3)  # alpha = 7.2: levels 0..6 on, level 7 at 0.5*(1+cos(pi*0.2+pi)), rest off
    assert torch.all(w[:7] == 1) and torch.all(w[8:] == 0)
    assert abs(w[7].item() - 0.5 * (1 + math.cos(math.pi * 0.2 + math.pi))) < 1e-6
    with pytest.raises(AssertionError):
        c2f(1.5)
    assert torch.equal(win, torch.from_numpy(workloads.anneal_window(workloads.WORKLOADS["c5"])))


def test_map_range_val():
    assert pe.map_range_val(5, 0, 10, 0.0, 1.0) == 0.5
    assert pe.map_range_val(-3, 0, 10, 2.0, 4.0) == 2.0
    assert pe.map_range_val(30, 0, 10, 2.0, 4.0) == 4.0
    assert pe.map_range_val(2.5, 0, 10, 1.0, -1.0) == 0.5


def test_module_surface_on_cpu():
    torch.manual_seed(0)
    m = pe.PermutoEncoding(3, 1 << 10, 6, 2, np.geomspace(1.0, 1e-2, 6), device="cpu")
    sd = m.state_dict()
    assert list(sd) == ["lattice_values", "random_shift_per_level"]
    assert sd["lattice_values"].shape == (6, 1 << 10, 2) and sd["lattice_values"].is_contiguous()
    assert sd["random_shift_per_level"].shape == (6, 3)
    assert torch.equal(m.anneal_window, torch.ones(6))
    assert m.output_dims() == 12
    assert 0.5e-5 < m.lattice_values.std().item() < 2e-5 and abs(m.lattice_values.mean().item()) < 1e-6
    assert 5 < m.random_shift_per_level.std().item() < 15
    assert np.array_equal(m.fixed_params.m_scale_factor.numpy(), orc.scale_factors(3, np.geomspace(1.0, 1e-2, 6)))
    m2 = pe.PermutoEncoding(5, 64, 2, 2, [1.0, 0.5], concat_points=True, device="cpu")
    assert m2.output_dims() == 2 * (2 + 3)
    # same RNG stream as the reference: values are drawn as (capacity, levels, feat) and permuted
    torch.manual_seed(0)
    want = (torch.randn(1 << 10, 6, 2) * 1e-5).permute(1, 0, 2).contiguous()
    assert torch.equal(sd["lattice_values"], want)
    # no CPU path: the forward refuses loudly instead of falling back
    with pytest.raises(ValueError, match="GPU memory"):
        m(torch.rand(4, 3))
    with pytest.raises(RuntimeError, match="nr_feat_per_level"):
        pe.PermutoEncoding(3, 64, 2, 6, [1.0, 0.5], device="cpu")
    m4 = pe.PermutoEncoding(3, 64, 2, 4, [1.0, 0.5], concat_points=True, device="cpu")   # four features per level
    assert m4.lattice_values.shape == (2, 64, 4) and m4.output_dims() == 4 * (2 + 1)
    with pytest.raises(RuntimeError, match="pos_dim"):
        pe.PermutoEncoding(9, 64, 2, 2, [1.0, 0.5], device="cpu")
    with pytest.raises(ValueError, match="one entry per level"):
        pe.PermutoEncoding(3, 64, 3, 2, [1.0, 0.5], device="cpu")
    import permutohedral_encoding
    assert permutohedral_encoding.PermutoEncoding is pe.PermutoEncoding


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "permutohedral_encoding_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("oracle of", ""), f"{f} mentions the oracle"


def test_workloads_are_seeded_and_shaped():
    w = workloads.WORKLOADS["c3"].scaled(1000)
    a, b = workloads.make_inputs(w), workloads.make_inputs(w)
    for k in a:
        assert np.array_equal(a[k], b[k])
    assert a["pos"].shape == (1000, 4) and a["grad"].shape == (24, 2, 1000) and a["table"].shape == (24, 1 << 18, 2)
    assert np.allclose(workloads.scale_list(w)[[0, -1]], [1.0, 1e-4])
    s = workloads.make_inputs(workloads.WORKLOADS["c5"].scaled(4000), need=("pos",))["pos"]
    r = np.linalg.norm(s - 0.5, axis=1)
    assert abs(r.mean() - 0.5) < 5e-3 and 0.015 < r.std() < 0.025
    assert workloads.WORKLOADS["c2"].point_levels == 25165824
    # the ray-ordered variant of c2: consecutive points are consecutive samples of one ray
    rays = workloads.make_inputs(workloads.WORKLOADS["c2_rays"].scaled(1024), need=("pos",))["pos"]
    step = np.linalg.norm(np.diff(rays.reshape(8, 128, 3), axis=1), axis=2)
    assert rays.shape == (1024, 3) and rays.min() >= 0 and rays.max() <= 1 and step.max() < 0.02


def test_workspace_request_is_capped_and_shrinks_when_memory_runs_out(monkeypatch):
    """The scatter workspace grows with points x levels; the binding caps it and, when the allocator
    refuses, asks again for fewer levels per pass, then for none (the library then adds directly)."""
    import torch
    d, n, levels, cap = 3, 1 << 20, 24, 1 << 18
    lib = _native.lib()
    full = lib.penc_scatter_workspace_bytes(d, n, levels, cap, 0)
    one = lib.penc_scatter_workspace_bytes(d, n, levels, cap, 1)
    assert full > 20 * one > 0
    requests = []
    limit = [None]

    def fake_empty(nbytes, dtype=None, device=None):
        requests.append(nbytes)
        if limit[0] is not None and nbytes > limit[0]:
            raise torch.cuda.OutOfMemoryError("simulated")
        return torch.zeros(1, dtype=torch.uint8)  # stands for the buffer

    monkeypatch.setattr(_native.torch, "empty", fake_empty)
    assert _native.scatter_workspace(d, n, levels, cap, "cpu") is not None and requests == [full]
    # capped: the largest power-of-two fraction of the levels whose records fit
    requests.clear()
    monkeypatch.setattr(_native, "MAX_WORKSPACE_BYTES", 400 << 20)
    _native.scatter_workspace(d, n, levels, cap, "cpu")
    assert len(requests) == 1 and one <= requests[0] <= 400 << 20
    monkeypatch.setattr(_native, "MAX_WORKSPACE_BYTES", None)
    # out of memory: 24 -> 12 -> 6 -> 3 -> 1 levels per pass, then nothing
    requests.clear()
    limit[0] = 2 * one
    assert _native.scatter_workspace(d, n, levels, cap, "cpu") is not None
    assert requests[0] == full and requests[-1] <= 2 * one and requests == sorted(requests, reverse=True)
    requests.clear()
    limit[0] = 0
    assert _native.scatter_workspace(d, n, levels, cap, "cpu") is None
    # the level-major copy of a row-major gradient is not optional: that request is repeated and may raise
    requests.clear()
    with pytest.raises(torch.cuda.OutOfMemoryError):
        _native.scatter_workspace(d, n, levels, cap, "cpu", positions_grad=True, fixed_bytes=1000, required_bytes=1000)
    assert requests[-1] == 1000


def _counter_rows(workload):
    """(phase, kernel) -> (memory-side bytes, vector instructions) from the table of profiles/<workload>_counters.md."""
    rows = {}
    header = None
    for line in open(os.path.join(ROOT, "profiles", f"{workload}_counters.md")):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if line.startswith("| phase | kernel | avg us"):
            header = cells
        elif header and line.startswith("|") and not line.startswith("|---") and len(cells) == len(header):
            r = dict(zip(header, cells))
            mib = float(r["memory-side read MiB"]) + float(r["memory-side written MiB"])
            rows[(r["phase"], r["kernel"].strip("`"))] = (mib * 2 ** 20, float(r["VALU instr (wave)"]))
        elif header and not line.startswith("|"):
            header = None
    return rows


@pytest.mark.parametrize("workload", ["c2", "c3", "c4", "c5"])
def test_traffic_summary_is_the_sum_of_the_counter_rows_it_names(workload):
    """profiles/hbm_traffic.json (what bench.py reads) against the per-kernel tables beside it: every
    phase's bytes and vector instructions are the sums of the rows of the kernels the phase names, every
    kernel the phase launches is named, and the scattering kernel of each phase is the right instance."""
    import json
    import bench
    recorded = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json")))
    assert workload in recorded
    w = workloads.WORKLOADS[workload]
    want_table, want_pos = "backward_table" in w.phases, "backward_pos" in w.phases
    reducer = "bin_reduce_levels_kernel" if w.capacity > 64 * 8192 else "bin_reduce_kernel"
    expected = {"forward": ["forward_kernel"]}
    if want_table or want_pos:
        expected["backward"] = ((["fill_zero_kernel", "backward_table_kernel", reducer] if want_table else [])
                                + (["backward_pos_kernel", "reduce_level_groups_kernel"] if want_pos else []))
    if "double_backward" in w.phases:
        expected["double_backward"] = ["grad_grad_kernel", "fill_zero_kernel", "backward_table_kernel", reducer]
    rows = _counter_rows(workload)
    assert sorted(recorded[workload]) == sorted(expected)
    for phase, kernels in expected.items():
        entry = recorded[workload][phase]
        assert bench.traffic_entry_matches(entry, kernels, second_order=phase == "double_backward"), (phase, entry["kernels"])
        table_bytes = sum(rows[(phase, k)][0] for k in entry["kernels"])
        table_valu = sum(rows[(phase, k)][1] for k in entry["kernels"])
        # the tables are rounded to 0.1 MiB and three significant digits per row
        assert abs(entry["hbm_bytes"] - table_bytes) <= 0.11 * 2 ** 20 * len(entry["kernels"]), phase
        assert abs(entry["valu_wave_instr"] - table_valu) <= 0.006 * table_valu + 1, phase
    # a wrongly attributed entry is refused: the first-order scatter does not serve the double backward
    if "double_backward" in expected and "backward_table_kernel" in expected.get("backward", []):
        assert not bench.traffic_entry_matches(recorded[workload]["backward"], expected["double_backward"], second_order=True)


def test_profile_summary_attributes_shared_kernels_by_dispatch_order():
    from permutohedral_encoding_amd import profile_summary as ps
    k = ["forward_kernel<4, 2, float>", "backward_pos_kernel<4, 2, float>", "reduce_level_groups_kernel",
         "grad_grad_kernel<4, 2, float>", "fill_zero_kernel", "backward_table_kernel<4, false, true, false>", "bin_reduce_kernel<true>",
         "fill_zero_kernel", "backward_table_kernel<4, false, false, false>", "bin_reduce_kernel<true>", "at::native::copy_kernel", "copy_kernel"]
    assert ps.phase_of_dispatches(k) == ["forward", "backward", "backward", "double_backward", "double_backward", "double_backward",
                                         "double_backward", "backward", "backward", "backward", None, None]
    assert ps.short("void penc::backward_table_kernel<3, false, true, false>(int, int)") == "backward_table_kernel<3, false, true, false>"
