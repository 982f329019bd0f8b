"""The PyTorch surface on the GPU: module forward layout, autograd backward and double backward
(eikonal-style), checked against the oracle through the chain rule."""
import numpy as np
import pytest

from helpers import to_gpu

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
orc = pytest.importorskip("oracle.api")


def make_module(d=3, cap=1 << 12, levels=6, **kw):
    import permutohedral_encoding_amd as pe
    torch.manual_seed(0)
    m = pe.PermutoEncoding(d, cap, levels, 2, np.geomspace(1.0, 1e-2, levels), **kw)
    with torch.no_grad():
        m.lattice_values.uniform_(-1, 1)
    return m


def oracle_args(m, pos):
    sf = orc.scale_factors(m.pos_dim, m.scale_per_level)
    return (pos.detach().cpu().numpy(), m.lattice_values.detach().cpu().numpy(), sf,
            m.random_shift_per_level.detach().cpu().numpy())


def test_forward_layout_and_no_grad():
    m = make_module()
    pos = torch.rand(1000, 3, device="cuda")
    with torch.no_grad():
        out = m(pos)
    assert out.shape == (1000, m.output_dims())
    # like the reference's permute+reshape, the result is a strided view of the kernel's (L, 2, N) output
    assert out.stride() == (1, 1000)
    p, t, sf, sh = oracle_args(m, pos)
    want = orc.forward(p, t, sf, sh, np.ones(6, np.float32))  # (L,2,N)
    want = want.transpose(2, 0, 1).reshape(1000, -1)  # column = level*2 + feat
    assert np.allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-6)
    with pytest.raises(RuntimeError):
        out.sum().backward()


def test_backward_through_autograd():
    m = make_module()
    pos = torch.rand(2000, 3, device="cuda", requires_grad=True)
    win = torch.tensor([1, 1, 1, 0.5, 0, 0], dtype=torch.float32)
    out = m(pos, win)
    up = torch.randn_like(out)
    (out * up).sum().backward()
    p, t, sf, sh = oracle_args(m, pos)
    g = up.cpu().numpy().reshape(2000, 6, 2).transpose(1, 2, 0)
    w = win.numpy()
    wt = orc.backward_table(p, sf, sh, w, g, m.capacity, want_abs=True)
    assert m.lattice_values.grad.shape == m.lattice_values.shape
    err = np.abs(m.lattice_values.grad.cpu().numpy() - wt["grad64"])
    assert np.all(err <= 1e-4 * wt["abs64"] + 1e-30)
    wp = orc.backward_pos(p, t, sf, sh, w, g)["grad64"]
    assert np.allclose(pos.grad.cpu().numpy(), wp, rtol=1e-4, atol=1e-4 * np.abs(wp).max())


def test_double_backward_eikonal_style():
    """loss = sum_n (|d(sum_c out[n,c]*a[c]) / d pos_n| - 1)^2 ; its gradient w.r.t. the table goes
    through the double-backward kernels."""
    m = make_module(levels=4)
    n = 1500
    pos = torch.rand(n, 3, device="cuda", requires_grad=True)
    a = torch.randn(m.output_dims(), device="cuda")
    out = m(pos)
    sdf = (out * a).sum(dim=1)
    grad_pos, = torch.autograd.grad(sdf.sum(), pos, create_graph=True)
    loss = ((grad_pos.norm(dim=1) - 1.0) ** 2).sum()
    loss.backward()
    # chain rule by hand with the oracle: q = dloss/dgrad_pos, then table gradient of <q, posgrad(T, g)>
    p, t, sf, sh = oracle_args(m, pos)
    g = np.broadcast_to(a.cpu().numpy()[None], (n, m.output_dims())).reshape(n, 4, 2).transpose(1, 2, 0).copy()
    w = np.ones(4, np.float32)
    gp = orc.backward_pos(p, t, sf, sh, w, g)["grad64"]
    assert np.allclose(grad_pos.detach().cpu().numpy(), gp, rtol=1e-4, atol=1e-4 * np.abs(gp).max())
    nrm = np.linalg.norm(gp, axis=1, keepdims=True)
    q = (2.0 * (nrm - 1.0) * gp / nrm).astype(np.float32)
    r = orc.double_backward(p, t, sf, sh, w, q, g, want_abs=True)
    err = np.abs(m.lattice_values.grad.cpu().numpy() - r["grad64"])
    assert np.all(err <= 1e-3 * r["abs64"] + 1e-6 * np.abs(r["grad64"]).max())
    # positions get no second-order gradient: the interpolant is piecewise linear
    assert pos.grad is None or torch.all(pos.grad == 0)


def test_state_dict_round_trip_and_pickle():
    import pickle
    m = make_module()
    sd = m.state_dict()
    assert set(sd) == {"lattice_values", "random_shift_per_level"}
    m2 = make_module()
    with torch.no_grad():
        m2.random_shift_per_level.add_(1.0)
    m2.load_state_dict(sd)
    pos = torch.rand(500, 3, device="cuda")
    with torch.no_grad():
        assert torch.equal(m(pos), m2(pos))  # the native side sees the in-place update of the shift
        m3 = pickle.loads(pickle.dumps(m))
        assert torch.equal(m(pos), m3(pos))


def test_concat_points_module():
    m = make_module(concat_points=True, concat_points_scaling=0.1)
    pos = torch.rand(300, 3, device="cuda", requires_grad=True)
    out = m(pos)
    assert out.shape == (300, 2 * (6 + 2)) == (300, m.output_dims())
    assert torch.allclose(out[:, 12:15], pos.detach() * 0.1)
    assert torch.all(out[:, 15] == 0)
    out.sum().backward()  # gradient does not flow to positions through the copied columns (as in the reference)
    assert m.lattice_values.grad is not None


def test_toy_sdf_training_with_eikonal_term():
    """End to end through autograd, like the reference's toy example plus an eikonal term:
    encoding -> small MLP -> SDF of a sphere; the loss uses the SDF value (first backward into the
    table), its gradient w.r.t. positions (position backward) and the norm of that gradient (double
    backward), with a coarse-to-fine window.  The loss must go down by a large factor."""
    import permutohedral_encoding_amd as pe
    torch.manual_seed(0)
    levels = 8
    enc = pe.PermutoEncoding(3, 1 << 14, levels, 2, np.geomspace(1.0, 0.05, levels))
    mlp = torch.nn.Sequential(torch.nn.Linear(enc.output_dims(), 32), torch.nn.Softplus(beta=20),
                              torch.nn.Linear(32, 1)).cuda()
    c2f = pe.Coarse2Fine(levels)
    opt = torch.optim.Adam(list(enc.parameters()) + list(mlp.parameters()), lr=1e-2)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    losses = []
    for it in range(150):
        pos = torch.rand(4096, 3, device="cuda", generator=gen).requires_grad_(True)
        target = (pos.detach() - 0.5).norm(dim=1, keepdim=True) - 0.3
        window = c2f(pe.map_range_val(it, 0, 100, 0.3, 1.0))
        sdf = mlp(enc(pos, window))
        grad, = torch.autograd.grad(sdf.sum(), pos, create_graph=True)
        loss = ((sdf - target) ** 2).mean() + 0.05 * ((grad.norm(dim=1) - 1.0) ** 2).mean()
        opt.zero_grad(set_to_none=True)
        loss.backward()
        assert enc.lattice_values.grad is not None and torch.isfinite(enc.lattice_values.grad).all()
        assert enc.random_shift_per_level.grad is None  # the shift is a parameter only to be checkpointed
        opt.step()
        losses.append(loss.item())
    assert np.mean(losses[-10:]) < 0.2 * np.mean(losses[:5]), (losses[:5], losses[-10:])


def test_forward_and_backward_replay_in_a_hip_graph():
    """The entry points only enqueue kernels on the given stream (the gradient is cleared by a fill
    kernel, not a memset), so a captured step must replay to the eager results, every time."""
    from permutohedral_encoding_amd import _native
    from helpers import random_problem, make_encoding, gpu_input
    d, cap = 3, 1 << 14
    p = random_problem(d, 20000, 8, cap, seed=21, sigma_range=(1.0, 1e-3))
    enc, _ = make_encoding(d, p["sigmas"], p["shift"])
    inp = gpu_input(p)
    grad = to_gpu(p["grad"])
    out_eager = enc.forward(inp)
    tg_eager, pg_eager = enc.backward(inp, grad)
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream, as torch asks for
        enc.forward(inp)
        enc.backward(inp, grad)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = enc.forward(inp)
        tg_g, pg_g = enc.backward(inp, grad)
    for replay in range(3):
        out_g.zero_()
        tg_g.fill_(float("nan"))
        pg_g.zero_()
        (grad * 2).sum().item()  # unrelated eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_eager), replay
        assert torch.equal(pg_g, pg_eager), replay
        assert torch.allclose(tg_g, tg_eager, rtol=1e-4, atol=1e-6 * tg_eager.abs().max().item()), replay


def test_sparse_training_step_replays_in_a_hip_graph():
    """A whole sparse step (gradient call that adds and marks, optimizer step that updates, zeroes and
    unmarks) is kernels on the given stream and nothing else: captured once and replayed, every replay
    moves the table exactly like the same step run eagerly."""
    from permutohedral_encoding_amd import _native
    from helpers import random_problem, make_encoding
    lib = _native.lib()
    d, cap, levels, n = 3, 1 << 16, 6, 40000
    p = random_problem(d, n, levels, cap, seed=33, sigma_range=(1.0, 2e-3))
    enc, fp = make_encoding(d, p["sigmas"], p["shift"])
    pos, win, grad = to_gpu(p["pos"]), to_gpu(p["window"]), to_gpu(p["grad"])
    entries = int(lib.penc_touched_map_entries(2, levels, cap))
    ws_bytes = int(lib.penc_scatter_workspace_bytes(d, n, levels, cap, 0))

    def fresh():
        return dict(table=to_gpu(p["table"]), m=torch.zeros(levels, cap, 2, device="cuda"), v=torch.zeros(levels, cap, 2, device="cuda"),
                    g=torch.zeros(levels, cap, 2, device="cuda"), touched=torch.zeros(entries, dtype=torch.int32, device="cuda"),
                    ws=torch.empty(ws_bytes, dtype=torch.uint8, device="cuda"))

    def step(s, k):
        st = torch.cuda.current_stream().cuda_stream
        assert lib.penc_backward_sparse(d, 2, n, levels, cap, pos.data_ptr(), s["table"].data_ptr(), fp.m_scale_factor.data_ptr(),
                                        fp.m_random_shift_per_level.data_ptr(), win.data_ptr(), grad.data_ptr(), 0, s["g"].data_ptr(),
                                        s["touched"].data_ptr(), None, s["ws"].data_ptr(), ws_bytes, st) == 0
        assert lib.penc_adamw_step_sparse(s["table"].data_ptr(), s["g"].data_ptr(), s["m"].data_ptr(), s["v"].data_ptr(), 2, levels, cap,
                                          s["touched"].data_ptr(), 1e-2, 0.9, 0.99, 1e-8, 0.01, k, 1, st) == 0

    eager = fresh()
    snapshots = []
    for k in range(3):  # the captured step keeps its step count: compare with eager steps that all use step 1
        step(eager, 1)
        torch.cuda.synchronize()
        snapshots.append(eager["table"].clone())
        assert not eager["g"].any().item() and not eager["touched"].any().item()

    captured = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        warm = fresh()
        step(warm, 1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(captured, 1)
    for k in range(3):
        (grad * 2).sum().item()  # unrelated eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        scale = snapshots[k].abs().max().item()
        assert torch.allclose(captured["table"], snapshots[k], rtol=1e-5, atol=1e-6 * scale), k
        assert not captured["g"].any().item() and not captured["touched"].any().item()
    assert free_before - torch.cuda.mem_get_info()[0] < (8 << 20)  # the capture itself allocated next to nothing


@pytest.mark.parametrize("rows,cols", [(1, 2), (255, 48), (256, 48), (257, 48), (100000, 32), (5000, 63), (7, 1), (1000, 255)])
def test_streaming_transpose(rows, cols):
    from permutohedral_encoding_amd import _native
    src = torch.randn(rows, cols, device="cuda")
    dst = torch.empty(cols, rows, device="cuda")
    rc = _native.lib().penc_transpose(src.data_ptr(), dst.data_ptr(), rows, cols, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(dst, src.t().contiguous())


def test_level_major_gradient_paths():
    from permutohedral_encoding_amd import _native
    up = torch.randn(3000, 12, device="cuda")                       # row-major (N, 2L) as a linear layer delivers it
    view = up.reshape(3000, 6, 2).permute(1, 2, 0)                   # what autograd hands to the Function
    assert not view.is_contiguous()
    got = _native.level_major_gradient(view)
    assert got.is_contiguous() and torch.equal(got, view.contiguous())
    odd = torch.randn(6, 2, 6000, device="cuda")[:, :, ::2]          # some other strided view: generic copy
    assert torch.equal(_native.level_major_gradient(odd), odd.contiguous())
    c = torch.randn(6, 2, 100, device="cuda")
    assert _native.level_major_gradient(c) is c


@pytest.mark.parametrize("d,n,levels,cap,concat", [(3, 20000, 8, 1 << 14, False), (4, 5001, 6, 50000, True), (2, 70000, 24, 1 << 15, False)])
def test_table_gradient_from_row_major_upstream_gradient(d, n, levels, cap, concat):
    """The table gradient read straight from rows grad[n][2*level+feature] must equal the oracle's on
    the level-major copy (same terms, same tolerance as any atomic sum), also with the extra
    columns of concatenated points and a padded row stride."""
    from permutohedral_encoding_amd import _native
    from helpers import random_problem, make_encoding, gpu_input, assert_sum_close
    SUM_RTOL = 1e-4  # atomically accumulated gradients, relative to the sum of magnitudes of their terms
    from oracle import api as orc
    p = random_problem(d, n, levels, cap, seed=41, sigma_range=(1.0, 1e-3))
    enc, fp = make_encoding(d, p["sigmas"], p["shift"], concat_points=concat)
    extra = _native.extra_levels(d, 2, concat)
    cols = 2 * (levels + extra)
    rng = np.random.default_rng(5)
    rows = torch.from_numpy(rng.standard_normal((n, cols + 2)).astype(np.float32)).cuda()   # padded rows
    view = rows[:, :cols].reshape(n, levels + extra, 2).permute(1, 2, 0)
    assert _native.is_row_major_view(view)
    inp = gpu_input(p, need_pos_grad=False)   # table gradient only
    tg, pg = enc.backward(inp, view)
    assert pg is None
    sf = orc.scale_factors(d, p["sigmas"])
    level_major = np.ascontiguousarray(view[:levels].cpu().numpy())
    want = orc.backward_table(p["pos"], sf, p["shift"], p["window"], level_major, cap, want_abs=True)
    assert_sum_close(tg.cpu().numpy(), want["grad64"], want["abs64"], SUM_RTOL, "table gradient from rows")
    tg_copy, _ = enc.backward(inp, view.contiguous())
    assert torch.allclose(tg, tg_copy, rtol=1e-3, atol=1e-6 * tg_copy.abs().max().item())


def test_row_major_entry_point_rejects_bad_strides():
    from permutohedral_encoding_amd import _native
    lib = _native.lib()
    t = torch.zeros(64, device="cuda")
    args = lambda stride, grad: (3, 2, 4, 2, 8, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), grad, stride,
                                 t.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
    assert lib.penc_backward_table_rowmajor(*args(3, t.data_ptr())) == 2      # stride < 2 * levels
    assert lib.penc_backward_table_rowmajor(*args(5, t.data_ptr())) == 2      # odd stride
    assert lib.penc_backward_table_rowmajor(*args(4, t.data_ptr() + 4)) == 5  # rows not 8-byte aligned
    assert lib.penc_backward_table_rowmajor(*args(4, None)) == 1


def test_module_backward_reads_the_upstream_gradient_in_place():
    """A row-major upstream gradient reaches the library as it is: neither table-only training nor the
    path with position gradients and a double backward (the SDF path) makes a layout copy first."""
    import permutohedral_encoding_amd as pe
    from permutohedral_encoding_amd import _native
    torch.manual_seed(3)
    enc = pe.PermutoEncoding(3, 1 << 14, 8, 2, np.geomspace(1.0, 1e-3, 8))
    pts = torch.rand(5000, 3, device="cuda")
    up = torch.randn(5000, 16, device="cuda")  # a row-major upstream gradient, as a consumer that copies would send
    calls = []
    real = _native.level_major_gradient
    _native_funcs = __import__("permutohedral_encoding_amd.funcs", fromlist=["x"])
    _native_funcs.level_major_gradient = lambda g: (calls.append(1), real(g))[1]
    try:
        enc(pts).backward(up)
        g_table_only = enc.lattice_values.grad.clone()
        enc.lattice_values.grad = None
        pts_g = pts.clone().requires_grad_(True)
        out = enc(pts_g)
        grad_pos, = torch.autograd.grad(out, pts_g, up, create_graph=True)
        g_table = enc.lattice_values.grad
        assert g_table is None  # autograd.grad with inputs=[pts_g] leaves the parameter alone
        (grad_pos ** 2).sum().backward()   # double backward from the row-major gradient saved by the first backward
        assert calls == []
    finally:
        _native_funcs.level_major_gradient = real
    # the same through the level-major copy the reference would make
    pts_c = pts.clone().requires_grad_(True)
    enc2 = pe.PermutoEncoding(3, 1 << 14, 8, 2, np.geomspace(1.0, 1e-3, 8))
    enc2.load_state_dict(enc.state_dict())
    sliced = pe.funcs.PermutoEncodingFunc.apply(enc2.lattice, enc2.lattice_values, pts_c, enc2.anneal_window, True, True)
    up_lm = up.reshape(5000, 8, 2).permute(1, 2, 0).contiguous()
    grad_pos_c, = torch.autograd.grad(sliced, pts_c, up_lm, create_graph=True)
    assert torch.equal(grad_pos.detach(), grad_pos_c.detach())  # same kernel, same level-major values
    (grad_pos_c ** 2).sum().backward()
    a, b = enc.lattice_values.grad, enc2.lattice_values.grad
    assert torch.allclose(a, b, rtol=1e-3, atol=1e-6 * b.abs().max().item())
    enc2.lattice_values.grad = None
    enc2(pts).backward(up)
    assert torch.allclose(g_table_only, enc2.lattice_values.grad, rtol=1e-3, atol=1e-6 * g_table_only.abs().max().item())


@pytest.mark.parametrize("d,n,levels,cap,concat", [(3, 20000, 7, 1 << 15, False), (4, 9000, 5, 50000, True), (8, 3000, 3, 1 << 12, False)])
def test_all_gradients_from_row_major_upstream_gradient(d, n, levels, cap, concat):
    """penc_backward_rowmajor and penc_double_backward_from_positions_rowmajor against the oracle: table
    gradient, position gradient (from the level-major copy the scattering kernel leaves behind, or from
    the transposed rows when the table gradient is not wanted), second-order table gradient, grad-grad."""
    from permutohedral_encoding_amd import _native
    from helpers import random_problem, assert_sum_close, make_encoding, gpu_input
    p = random_problem(d, n, levels, cap, seed=43, sigma_range=(1.0, 1e-3))
    enc, fp = make_encoding(d, p["sigmas"], p["shift"], concat_points=concat)
    extra = _native.extra_levels(d, 2, concat)
    cols = 2 * (levels + extra)
    rng = np.random.default_rng(6)
    rows = torch.from_numpy(rng.standard_normal((n, cols + 4)).astype(np.float32)).cuda()   # padded rows
    view = rows[:, :cols].reshape(n, levels + extra, 2).permute(1, 2, 0)
    assert _native.is_row_major_view(view)
    sf = orc.scale_factors(d, p["sigmas"])
    level_major = np.ascontiguousarray(view[:levels].cpu().numpy())
    want_t = orc.backward_table(p["pos"], sf, p["shift"], p["window"], level_major, cap, want_abs=True)
    want_p = orc.backward_pos(p["pos"], p["table"], sf, p["shift"], p["window"], level_major)
    for need_table in (True, False):
        tg, pg = enc.backward(gpu_input(p, need_table, True), view)
        if need_table:
            assert_sum_close(tg.cpu().numpy(), want_t["grad64"], want_t["abs64"], 1e-4, "table gradient from rows")
        else:
            assert tg is None
        err = np.abs(pg.cpu().numpy() - want_p["grad64"])
        assert np.all(err <= 1e-6 * want_p["abs64"] + 1e-30), "position gradient from rows"
    tg2, ggs = enc.double_backward_from_positions(gpu_input(p), to_gpu(p["dpos"]), view)
    want = orc.double_backward(p["pos"], p["table"], sf, p["shift"], p["window"], p["dpos"], level_major,
                               concat_points=concat, want_abs=True)
    assert_sum_close(tg2.cpu().numpy(), want["grad64"], want["abs64"], 1e-4, "second-order table gradient from rows")
    assert ggs.is_contiguous() and np.array_equal(ggs.cpu().numpy(), want["ggs"])


def test_row_major_backward_needs_room_for_the_copy():
    from permutohedral_encoding_amd import _native
    lib = _native.lib()
    n, levels, cap, d = 1000, 4, 256, 3
    t = torch.zeros(n * 8, device="cuda")
    ws = torch.empty(4096, dtype=torch.uint8, device="cuda")
    need = lib.penc_backward_rowmajor_workspace_bytes(d, 2, n, levels, cap, 1, 1)
    assert need >= 8 * levels * n
    assert lib.penc_backward_rowmajor_workspace_bytes(d, 2, n, levels, cap, 1, 0) == lib.penc_scatter_workspace_bytes(d, n, levels, cap, 0)
    assert lib.penc_backward_rowmajor_workspace_bytes(d, 4, n, levels, cap, 1, 0) == lib.penc_scatter_workspace_bytes(d, n, 2 * levels, cap, 0)
    rc = lib.penc_backward_rowmajor(d, 2, n, levels, cap, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(),
                                    t.data_ptr(), 8, t.data_ptr(), t.data_ptr(), ws.data_ptr(), 4096,
                                    torch.cuda.current_stream().cuda_stream)
    assert rc == 8 and b"level-major array" in lib.penc_status_string(rc)


@pytest.mark.parametrize("feat", [4, 8])
def test_module_with_more_features_per_level(feat):
    """PermutoEncoding(..., nr_feat_per_level=4 or 8): output layout (column = level * F + feature),
    training step and eikonal-style double backward through autograd, against the oracle."""
    import permutohedral_encoding_amd as pe
    torch.manual_seed(1)
    levels, n = 5, 3000
    m = pe.PermutoEncoding(3, 1 << 12, levels, feat, np.geomspace(1.0, 1e-2, levels))
    with torch.no_grad():
        m.lattice_values.uniform_(-1, 1)
    pos = torch.rand(n, 3, device="cuda", requires_grad=True)
    out = m(pos)
    assert out.shape == (n, levels * feat) == (n, m.output_dims())
    p, t, sf, sh = oracle_args(m, pos)
    w = np.ones(levels, np.float32)
    want = orc.forward(p, t, sf, sh, w).transpose(2, 0, 1).reshape(n, -1)
    assert np.array_equal(out.detach().cpu().numpy(), want)
    up = torch.randn(n, levels * feat, device="cuda")
    grad_pos, = torch.autograd.grad(out, pos, up, create_graph=True)
    g = up.cpu().numpy().reshape(n, levels, feat).transpose(1, 2, 0).copy()
    wp = orc.backward_pos(p, t, sf, sh, w, g)
    assert np.all(np.abs(grad_pos.detach().cpu().numpy() - wp["grad64"]) <= 1e-6 * wp["abs64"] + 1e-30)
    q = torch.randn(n, 3, device="cuda")
    (grad_pos * q).sum().backward()
    r = orc.double_backward(p, t, sf, sh, w, q.cpu().numpy(), g, want_abs=True)
    err = np.abs(m.lattice_values.grad.cpu().numpy() - r["grad64"])
    assert np.all(err <= 1e-4 * r["abs64"] + 1e-30)


@pytest.mark.parametrize("switch,dtype", [(True, torch.float16), (torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16)])
def test_module_gathers_from_a_half_precision_copy(switch, dtype):
    """PermutoEncoding(..., lattice_half_precision=True or a 16-bit dtype): the kernels gather from a 16-bit
    copy of the fp32 parameter; the output is that of the rounded table, gradients reach the fp32 parameter
    in fp32 (first and second order), and the copy follows in-place updates of the parameter."""
    import permutohedral_encoding_amd as pe
    torch.manual_seed(3)
    levels, n = 5, 2000
    m = pe.PermutoEncoding(3, 1 << 12, levels, 2, np.geomspace(1.0, 1e-2, levels), lattice_half_precision=switch)
    narrow = lambda a: torch.from_numpy(a).to(dtype).to(torch.float32).numpy()
    with torch.no_grad():
        m.lattice_values.uniform_(-1, 1)
    pos = torch.rand(n, 3, device="cuda", requires_grad=True)
    out = m(pos)
    p, t, sf, sh = oracle_args(m, pos)
    rounded = narrow(t)
    assert not np.array_equal(rounded, t)
    w = np.ones(levels, np.float32)
    want = orc.forward(p, rounded, sf, sh, w).transpose(2, 0, 1).reshape(n, -1)
    assert np.array_equal(out.detach().cpu().numpy(), want)
    up = torch.randn(n, 2 * levels, device="cuda")
    grad_pos, = torch.autograd.grad(out, pos, up, create_graph=True)
    g = up.cpu().numpy().reshape(n, levels, 2).transpose(1, 2, 0).copy()
    wp = orc.backward_pos(p, rounded, sf, sh, w, g)
    assert np.all(np.abs(grad_pos.detach().cpu().numpy() - wp["grad64"]) <= 1e-6 * wp["abs64"] + 1e-30)
    q = torch.randn(n, 3, device="cuda")
    (grad_pos * q).sum().backward()
    assert m.lattice_values.grad.dtype == torch.float32 and m.lattice_values.dtype == torch.float32
    r = orc.double_backward(p, rounded, sf, sh, w, q.cpu().numpy(), g, want_abs=True)
    assert np.all(np.abs(m.lattice_values.grad.cpu().numpy() - r["grad64"]) <= 1e-4 * r["abs64"] + 1e-30)
    # an optimizer step modifies the parameter in place: the next forward reads a fresh copy
    with torch.no_grad():
        m.lattice_values.mul_(0.5)
    out2 = m(pos.detach())
    want2 = orc.forward(p, narrow(0.5 * t), sf, sh, w).transpose(2, 0, 1).reshape(n, -1)
    assert np.array_equal(out2.detach().cpu().numpy(), want2)
    # pickling keeps the switch
    import pickle
    m2 = pickle.loads(pickle.dumps(m))
    assert m2.lattice_half_precision == dtype and torch.equal(m2(pos.detach()), out2)
    # a write the version counter does not see leaves the copy stale until it is invalidated
    m.lattice_values.data.mul_(2.0)
    assert torch.equal(m(pos.detach()), out2)
    m.invalidate_half_table()
    want3 = orc.forward(p, narrow(t), sf, sh, w).transpose(2, 0, 1).reshape(n, -1)
    assert np.array_equal(m(pos.detach()).detach().cpu().numpy(), want3)


@pytest.mark.parametrize("n", [4096, 4099, 3])
def test_fused_adamw_follows_torch_adamw(n):
    """penc_adamw_step through permutohedral_encoding_amd.optim.AdamW against torch.optim.AdamW on the same
    parameter and gradients, several steps, with weight decay; sizes that do and do not split into
    16-byte accesses."""
    from permutohedral_encoding_amd.optim import AdamW
    torch.manual_seed(n)
    start = torch.randn(n, device="cuda")
    a = torch.nn.Parameter(start.clone())
    b = torch.nn.Parameter(start.clone())
    kw = dict(lr=3e-3, betas=(0.9, 0.99), eps=1e-8, weight_decay=0.05)
    ours, theirs = AdamW([a], **kw), torch.optim.AdamW([b], **kw)
    for step in range(6):
        g = torch.randn(n, device="cuda") * (10.0 ** (step - 3))
        a.grad, b.grad = g.clone(), g.clone()
        version = a._version
        ours.step()
        theirs.step()
        assert a._version > version  # in-place change recorded
        assert torch.allclose(a, b, rtol=2e-6, atol=1e-7), (step, (a - b).abs().max().item())
    sa, sb = ours.state[a], theirs.state[b]
    # the moments are sums with cancellation: a few units in the last place of their largest terms
    for key in ("exp_avg", "exp_avg_sq"):
        assert torch.allclose(sa[key], sb[key], rtol=2e-6, atol=2e-6 * sb[key].abs().max().item()), key


def test_fused_adamw_leaves_entries_without_gradient_alone():
    """skip_zero_gradients: an entry with a zero gradient keeps its value and its moments (no decay of
    either, no weight decay); the others are updated as by torch.optim.AdamW with the same step count."""
    from permutohedral_encoding_amd.optim import AdamW
    torch.manual_seed(5)
    n = 10007
    start = torch.randn(n, device="cuda")
    a = torch.nn.Parameter(start.clone())
    b = torch.nn.Parameter(start.clone())
    kw = dict(lr=1e-2, betas=(0.9, 0.99), eps=1e-15, weight_decay=0.01)
    ours, theirs = AdamW([a], skip_zero_gradients=True, **kw), torch.optim.AdamW([b], **kw)
    touched = torch.rand(n, device="cuda") < 0.3
    for step in range(4):
        g = torch.randn(n, device="cuda") * touched
        a.grad, b.grad = g.clone(), g.clone()
        ours.step()
        theirs.step()
    assert torch.equal(a[~touched], start[~touched])
    assert torch.all(ours.state[a]["exp_avg"][~touched] == 0) and torch.all(ours.state[a]["exp_avg_sq"][~touched] == 0)
    assert torch.allclose(a[touched], b[touched], rtol=2e-6, atol=1e-7)


def test_training_with_the_fused_optimizer_and_a_half_precision_table():
    """A few steps of the reference's training protocol (loss ((pred-10)^2).mean(), zero_grad, backward,
    step) with the fused optimizer on a module that gathers from a half-precision copy: the loss goes
    down and the copy follows the optimizer's in-place updates."""
    import permutohedral_encoding_amd as pe
    from permutohedral_encoding_amd.optim import AdamW
    torch.manual_seed(0)
    m = pe.PermutoEncoding(3, 1 << 14, 8, 2, np.geomspace(1.0, 1e-2, 8), lattice_half_precision=True)
    opt = AdamW(m.parameters(), lr=1e-1, betas=(0.9, 0.99), eps=1e-15, weight_decay=0.0, skip_zero_gradients=True)
    pts = torch.rand(20000, 3, device="cuda") - 0.5
    losses = []
    for _ in range(8):
        loss = ((m(pts) - 10) ** 2).mean()
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < 0.9 * losses[0], losses
    assert all(later < earlier for earlier, later in zip(losses, losses[1:])), losses


def test_sparse_table_grad_module_and_optimizer_follow_the_dense_path():
    """PermutoEncoding(sparse_table_grad=True) with SparseTableAdamW against the same module with dense
    gradients: an eikonal-style step (backward and double backward both reach the table) leaves
    lattice_values.grad None and the sum of the two gradients in table_grad; the sparse step equals
    torch.optim.AdamW on every slot that received a gradient and leaves every other slot, its moments
    included, alone; gradient and map are zero again afterwards."""
    import permutohedral_encoding_amd as pe
    from permutohedral_encoding_amd.optim import SparseTableAdamW
    cap, levels, n = 1 << 16, 5, 3000
    sig = np.geomspace(1.0, 5e-3, levels)
    torch.manual_seed(1)
    dense = pe.PermutoEncoding(3, cap, levels, 2, sig)
    sparse = pe.PermutoEncoding(3, cap, levels, 2, sig, sparse_table_grad=True)
    with torch.no_grad():
        dense.lattice_values.uniform_(-1, 1)
        sparse.lattice_values.copy_(dense.lattice_values)
        sparse.random_shift_per_level.copy_(dense.random_shift_per_level)
    start = dense.lattice_values.detach().clone()
    kw = dict(lr=1e-2, betas=(0.9, 0.99), eps=1e-12, weight_decay=0.01)
    opt_dense, opt_sparse = torch.optim.AdamW([dense.lattice_values], **kw), SparseTableAdamW(sparse, **kw)
    pts = torch.rand(n, 3, device="cuda")
    a = torch.randn(dense.output_dims(), device="cuda")

    def loss_of(m):
        pos = pts.clone().requires_grad_(True)
        sdf = (m(pos) * a).sum(dim=1)
        grad_pos, = torch.autograd.grad(sdf.sum(), pos, create_graph=True)
        return ((grad_pos.norm(dim=1) - 1.0) ** 2).mean() + 1e-3 * (sdf ** 2).mean()

    for step in range(3):  # the same points every step: the same slots are touched, so the two optimizers agree on them
        opt_dense.zero_grad()
        loss_of(dense).backward()
        loss_of(sparse).backward()
        assert sparse.lattice_values.grad is None
        g_dense, g_sparse = dense.lattice_values.grad, sparse.table_grad.grad
        scale = g_dense.abs().max().item()
        assert torch.allclose(g_sparse, g_dense, rtol=1e-4, atol=1e-5 * scale), (step, (g_sparse - g_dense).abs().max().item())
        touched = g_dense != 0
        assert torch.equal(g_sparse != 0, touched) or (g_sparse != 0)[~touched].sum() == 0
        opt_dense.step()
        opt_sparse.step()
        assert not sparse.table_grad.grad.any().item() and not sparse.table_grad.touched.any().item()
        got, want = sparse.lattice_values.detach(), dense.lattice_values.detach()
        assert torch.allclose(got[touched], want[touched], rtol=1e-4, atol=1e-6), (step, (got - want)[touched].abs().max().item())
        assert torch.equal(got[~touched], start[~touched])
    state = opt_sparse.state[sparse.lattice_values]
    assert state["step"] == 3 and torch.all(state["exp_avg"][~touched] == 0) and torch.all(state["exp_avg_sq"][~touched] == 0)
    with pytest.raises(ValueError):
        SparseTableAdamW(dense)


def test_gradients_no_pass_consumes_are_not_computed():
    """autograd.grad(sdf, positions, create_graph=True) runs the first-order backward of the slicing, but
    nothing in that pass uses the table gradient: the library is then asked for the position gradient
    alone (the reference launches its table scatter regardless, src/Encoding.cu:167).  The later
    loss.backward() does ask for it, and a frozen table is never given a second-order gradient."""
    m = make_module(levels=4)
    calls, doubles = [], []
    backward, double = m.lattice.backward, m.lattice.double_backward_from_positions

    def spy_backward(inp, grad):
        calls.append((inp.m_require_lattice_values_grad, inp.m_require_positions_grad))
        return backward(inp, grad)

    def spy_double(inp, dpos, grad, want_lattice_values_grad=True):
        doubles.append(want_lattice_values_grad)
        return double(inp, dpos, grad, want_lattice_values_grad=want_lattice_values_grad)

    m.lattice.backward, m.lattice.double_backward_from_positions = spy_backward, spy_double
    pos = torch.rand(800, 3, device="cuda", requires_grad=True)
    a = torch.randn(m.output_dims(), device="cuda")
    sdf = (m(pos) * a).sum(dim=1)
    grad_pos, = torch.autograd.grad(sdf.sum(), pos, create_graph=True)
    assert calls == [(False, True)]
    (((grad_pos.norm(dim=1) - 1.0) ** 2).sum() + (sdf ** 2).sum()).backward()
    assert calls == [(False, True), (True, True)] and doubles == [True]
    assert m.lattice_values.grad is not None and pos.grad is not None
    # a frozen table: the double backward runs its gathering half only
    m.lattice_values.requires_grad_(False)
    calls.clear(), doubles.clear()
    sdf = (m(pos) * a).sum(dim=1)
    grad_pos, = torch.autograd.grad(sdf.sum(), pos, create_graph=True)
    ((grad_pos.norm(dim=1) - 1.0) ** 2).sum().backward()
    assert calls == [(False, True)] and doubles == [False]


@pytest.mark.parametrize("d,feat,concat,n", [(3, 2, False, 5000), (4, 4, True, 777), (8, 2, True, 64), (2, 8, False, 10001)])
def test_contiguous_output_equals_the_strided_view(d, feat, concat, n):
    """penc_forward_rowmajor through PermutoEncoding(contiguous_output=True): the same bits as the default
    (a strided view of the level-major result) in a contiguous (N, F(L+E)) array, gradients included."""
    import permutohedral_encoding_amd as pe
    levels = 6
    sig = np.geomspace(1.0, 1e-2, levels)
    torch.manual_seed(d)
    plain = pe.PermutoEncoding(d, 1 << 12, levels, feat, sig, concat_points=concat, concat_points_scaling=0.5)
    rows = pe.PermutoEncoding(d, 1 << 12, levels, feat, sig, concat_points=concat, concat_points_scaling=0.5, contiguous_output=True)
    with torch.no_grad():
        plain.lattice_values.uniform_(-1, 1)
    rows.load_state_dict(plain.state_dict())
    pos = torch.rand(n, d, device="cuda")
    win = torch.tensor([1, 1, 0.5, 0, 1, 1], dtype=torch.float32)
    pa, pb = pos.clone().requires_grad_(True), pos.clone().requires_grad_(True)
    a, b = plain(pa, win), rows(pb, win)
    assert b.is_contiguous() and not a.is_contiguous() and b.shape == a.shape == (n, plain.output_dims())
    assert torch.equal(a, b)
    up = torch.randn_like(b)
    (a * up).sum().backward()
    (b * up).sum().backward()
    assert torch.allclose(pa.grad, pb.grad, rtol=1e-6, atol=1e-7 * pa.grad.abs().max().item())
    assert torch.allclose(plain.lattice_values.grad, rows.lattice_values.grad, rtol=1e-5, atol=1e-6 * plain.lattice_values.grad.abs().max().item())
