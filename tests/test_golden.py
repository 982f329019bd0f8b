"""Golden vectors (tests/golden/penc_golden.npz, written by tests/golden/make_golden.py from the
CPU oracle): the oracle must keep reproducing them, and the HIP path must match them."""
import os

import numpy as np
import pytest

from helpers import make_encoding, to_gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "penc_golden.npz")
DIMS = [2, 3, 4, 5, 6, 7, 8]


def load_case(d):
    z = np.load(GOLDEN)  # allow_pickle stays False
    pre = f"d{d}_"
    return {k[len(pre):]: z[k] for k in z.files if k.startswith(pre)}


@pytest.mark.parametrize("d", DIMS)
def test_oracle_reproduces_golden(d):
    from oracle import api as orc
    c = load_case(d)
    cap = c["table"].shape[1]
    sf = orc.scale_factors(d, c["sigmas"])
    assert np.array_equal(sf, c["sf"])
    s = orc.simplex(c["pos"], sf, c["shift"], cap)
    for k in ("rem0", "rank", "slot"):
        assert np.array_equal(s[k], c[k]), k
    assert np.array_equal(s["bary"], c["bary"])
    assert np.array_equal(orc.forward(c["pos"], c["table"], sf, c["shift"], c["window"]), c["out"])
    tg = orc.backward_table(c["pos"], sf, c["shift"], c["window"], c["grad"], cap)["grad64"]
    assert np.allclose(tg, c["table_grad"], rtol=1e-12, atol=1e-12)
    pg = orc.backward_pos(c["pos"], c["table"], sf, c["shift"], c["window"], c["grad"])["grad64"]
    assert np.allclose(pg, c["pos_grad"], rtol=1e-12, atol=1e-12)
    r = orc.double_backward(c["pos"], c["table"], sf, c["shift"], c["window"], c["dpos"], c["grad"])
    assert np.allclose(r["grad64"], c["table_grad2"], rtol=1e-12, atol=1e-12)
    assert np.array_equal(r["ggs"], c["ggs"])


@pytest.mark.gpu
@pytest.mark.parametrize("d", DIMS)
def test_hip_matches_golden(d):
    import torch
    from permutohedral_encoding_amd import _native
    c = load_case(d)
    cap = c["table"].shape[1]
    enc, fp = make_encoding(d, c["sigmas"], c["shift"])
    assert np.array_equal(fp.m_scale_factor.cpu().numpy(), c["sf"])
    # both device routines that produce slots and weights: the select chains of the scattering and
    # position-gradient kernels, and the LDS rank sort of the forward and grad-of-grad kernels
    for gather_path in (False, True):
        dbg = enc.simplex_debug(to_gpu(c["pos"]), cap, gather_path=gather_path)
        for k in ("rem0", "rank", "slot"):
            assert np.array_equal(dbg[k].cpu().numpy(), c[k]), (k, gather_path)
        assert np.array_equal(dbg["barycentric"].cpu().numpy(), c["bary"]), gather_path
    inp = _native.EncodingInput(to_gpu(c["table"]), to_gpu(c["pos"]), to_gpu(c["window"]), True, True)
    out = enc.forward(inp).cpu().numpy()
    assert np.all(np.abs(out - c["out"]) <= 1e-6 + 1e-5 * np.abs(c["out"]))
    tg, pg = enc.backward(inp, to_gpu(c["grad"]))
    scale = np.abs(c["table_grad"]).max()
    assert np.all(np.abs(tg.cpu().numpy() - c["table_grad"]) <= 1e-4 * np.abs(c["table_grad"]) + 1e-5 * scale)
    assert np.allclose(pg.cpu().numpy(), c["pos_grad"], rtol=1e-4, atol=1e-4 * np.abs(c["pos_grad"]).max())
    tg2, ggs = enc.double_backward_from_positions(inp, to_gpu(c["dpos"]), to_gpu(c["grad"]))
    scale = np.abs(c["table_grad2"]).max()
    assert np.all(np.abs(tg2.cpu().numpy() - c["table_grad2"]) <= 1e-4 * np.abs(c["table_grad2"]) + 1e-5 * scale)
    assert np.allclose(ggs.cpu().numpy(), c["ggs"], rtol=1e-4, atol=1e-4 * np.abs(c["ggs"]).max())
    assert torch.all(out_is_zero := torch.from_numpy(out[3]) == 0)  # masked level
