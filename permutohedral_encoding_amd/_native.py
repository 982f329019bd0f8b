"""ctypes binding over ``libpenc_hip.so`` (the C ABI declared in ``include/penc.h``).

This is the only way the package computes anything: there is no CPU or pure-PyTorch fallback.
If the library is missing or a tensor is not on a GPU the call raises.

The classes ``EncodingInput``, ``EncodingFixedParams`` and ``EncodingWrapper`` mirror the three
classes the reference exposes through pybind11 (``src/PyBridge.cxx:20-42``) so that the autograd
functions and the module read like the reference's.
"""
import ctypes
import os

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# PENC_HIP_LIB names another build of the same library (kernel experiments, a debug build)
LIB_PATH = os.environ.get("PENC_HIP_LIB", os.path.join(_HERE, "libpenc_hip.so"))
_lib = None

_c_f32p = ctypes.c_void_p
_SIGNATURES = {
    "penc_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "penc_extra_levels": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "penc_scale_factors": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, _c_f32p, _c_f32p]),
    "penc_forward": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                    _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                    ctypes.c_int, ctypes.c_float, ctypes.c_void_p]),
    "penc_forward_rowmajor_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int]),
    "penc_forward_rowmajor": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                             _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64,
                                             ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "penc_scatter_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                                       ctypes.c_int]),
    "penc_positions_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int64, ctypes.c_int]),
    "penc_backward": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                     _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                     ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "penc_static_scratch_bytes": (ctypes.c_size_t, []),
    "penc_backward_static": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                            _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                            ctypes.c_void_p]),
    "penc_backward_rowmajor_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                                                 ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "penc_backward_rowmajor": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                              _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64,
                                              _c_f32p, _c_f32p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "penc_double_backward_from_positions_rowmajor": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                                                    ctypes.c_int, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                                                    _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64, _c_f32p,
                                                                    _c_f32p, ctypes.c_int, ctypes.c_void_p,
                                                                    ctypes.c_size_t, ctypes.c_void_p]),
    "penc_backward_table_rowmajor": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                                    _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64, _c_f32p,
                                                    ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "penc_double_backward_from_positions": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                                           ctypes.c_int, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                                           _c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int,
                                                           ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "penc_forward_half": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                         _c_f32p, ctypes.c_void_p, ctypes.c_int, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                         ctypes.c_int, ctypes.c_float, ctypes.c_void_p]),
    "penc_backward_half": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                          _c_f32p, ctypes.c_void_p, ctypes.c_int, _c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64,
                                          _c_f32p, _c_f32p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "penc_double_backward_from_positions_half": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                                                ctypes.c_int, _c_f32p, ctypes.c_void_p, ctypes.c_int, _c_f32p, _c_f32p,
                                                                _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64, _c_f32p,
                                                                _c_f32p, ctypes.c_int, ctypes.c_void_p,
                                                                ctypes.c_size_t, ctypes.c_void_p]),
    "penc_adamw_step": (ctypes.c_int, [_c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64, ctypes.c_double, ctypes.c_double,
                                       ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_int64, ctypes.c_int,
                                       ctypes.c_void_p]),
    "penc_touched_map_entries": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "penc_touched_range_slots": (ctypes.c_int, [ctypes.c_int]),
    "penc_backward_sparse": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                            _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int64,
                                            _c_f32p, ctypes.c_void_p, _c_f32p, ctypes.c_void_p, ctypes.c_size_t,
                                            ctypes.c_void_p]),
    "penc_double_backward_from_positions_sparse": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                                                  ctypes.c_int, _c_f32p, _c_f32p, _c_f32p, _c_f32p, _c_f32p,
                                                                  _c_f32p, _c_f32p, ctypes.c_int64, _c_f32p, ctypes.c_void_p,
                                                                  _c_f32p, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                                                  ctypes.c_void_p]),
    "penc_adamw_step_sparse": (ctypes.c_int, [_c_f32p, _c_f32p, _c_f32p, _c_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_double, ctypes.c_double, ctypes.c_double,
                                              ctypes.c_double, ctypes.c_double, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "penc_clear_touched": (ctypes.c_int, [_c_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "penc_transpose": (ctypes.c_int, [_c_f32p, _c_f32p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "penc_simplex_debug": (ctypes.c_int, [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, _c_f32p, _c_f32p,
                                          _c_f32p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                          _c_f32p, ctypes.c_void_p]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib():
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m permutohedral_encoding_amd.build` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def _check(status, what):
    if status != 0:
        msg = lib().penc_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (status {status})")


def extra_levels(pos_dim, nr_feat, concat_points):
    return int(lib().penc_extra_levels(int(pos_dim), int(nr_feat), int(bool(concat_points))))


def scale_factors(pos_dim, sigmas):
    """Host computation of the (L, D) scale-factor table (reference: Encoding.cuh:55-69)."""
    sig = np.ascontiguousarray(np.asarray(sigmas, dtype=np.float32).reshape(-1))
    out = np.empty((sig.size, int(pos_dim)), np.float32)
    _check(lib().penc_scale_factors(int(pos_dim), int(sig.size), sig.ctypes.data, out.ctypes.data), "scale_factors")
    return out


# Levels binned per pass by the table-gradient scatter (0: the library's default, all levels in one pass;
# < 0: no workspace, i.e. direct atomics).  The workspace is taken from torch's caching allocator for
# the duration of a call.  Its size grows with points x levels (about 1.4 GiB for 2^20 points, 24
# levels, pos_dim 3): MAX_WORKSPACE_BYTES caps the request, and a request the allocator cannot serve
# is retried with fewer levels per pass and finally without a workspace; the library computes the
# same sums either way (more passes over the levels, or direct atomics).
LEVELS_PER_PASS = 0
MAX_WORKSPACE_BYTES = None


def _scatter_bytes(pos_dim, nr_positions, nr_levels, capacity, levels_per_pass):
    return int(lib().penc_scatter_workspace_bytes(int(pos_dim), int(nr_positions), int(nr_levels), int(capacity),
                                                  int(levels_per_pass)))


def scatter_workspace(pos_dim, nr_positions, nr_levels, capacity, device, table_grad=True, positions_grad=False,
                      fixed_bytes=0, required_bytes=0, nr_feat=2):
    """Scratch memory for one gradient call (None when the library would not use any).

    The scatter counts every pair of features as a level (``nr_levels * nr_feat / 2`` of them).
    ``fixed_bytes`` is added to every request (the level-major copy of a row-major upstream gradient);
    ``required_bytes`` is the part of it the call cannot do without."""
    if LEVELS_PER_PASS < 0 and not required_bytes:
        return None
    pos_bytes = 0
    if positions_grad:
        pos_bytes = int(lib().penc_positions_workspace_bytes(int(pos_dim), int(nr_positions), int(nr_levels)))
    pair_levels = nr_levels * (nr_feat // 2)
    per_pass = pair_levels if LEVELS_PER_PASS <= 0 else min(LEVELS_PER_PASS, pair_levels)
    if not table_grad or LEVELS_PER_PASS < 0:
        per_pass = 0
    while True:
        nbytes = _scatter_bytes(pos_dim, nr_positions, pair_levels, capacity, per_pass) if per_pass else 0
        nbytes = max(nbytes, pos_bytes) + fixed_bytes
        over_cap = MAX_WORKSPACE_BYTES is not None and nbytes > MAX_WORKSPACE_BYTES
        if not over_cap:
            if nbytes == 0:
                return None
            try:
                return torch.empty(nbytes, dtype=torch.uint8, device=device)
            except torch.cuda.OutOfMemoryError:
                pass
        if per_pass > 1:
            per_pass //= 2      # fewer levels per pass: a smaller workspace, more passes
        elif per_pass == 1 or pos_bytes:
            per_pass, pos_bytes = 0, 0   # no binning and no partial sums: direct atomics, one thread per point
        elif required_bytes and fixed_bytes:
            return torch.empty(required_bytes, dtype=torch.uint8, device=device)   # raises if even that fails
        else:
            return None


def _ptr(t):
    return None if t is None else t.data_ptr()


TABLE_FORMATS = {torch.float16: 1, torch.bfloat16: 2}  # PENC_TABLE_FP16, PENC_TABLE_BF16 (include/penc.h)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _require(cond, msg):
    if not cond:
        raise ValueError(msg)


def _check_f32_gpu(t, name, ndim):
    _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
    _require(t.is_cuda, f"{name} should be in GPU memory. Please call .cuda() on the tensor")
    _require(t.dtype == torch.float32, f"{name} should be of type float")
    _require(t.dim() == ndim, f"{name} should have {ndim} dimensions, however it has sizes {tuple(t.shape)}")


def is_row_major_view(grad):
    """True for a (L, F, N) *view* of rows grad_rows[n][F*level + feature] (the upstream gradient of the
    module's (N, F*L) output seen through its permute+reshape): the library reads that as it is."""
    if grad.dim() != 3 or not grad.is_cuda or grad.dtype != torch.float32 or grad.is_contiguous():
        return False
    levels, feat, n = grad.shape
    s_level, s_feat, s_point = grad.stride()
    return (feat in (2, 4, 8) and n > 0 and s_level == feat and s_feat == 1 and s_point >= feat * levels and s_point % 2 == 0
            and grad.data_ptr() % 8 == 0 and s_point * n < 2 ** 31)


def level_major_gradient(grad):
    """The contiguous (L, 2, N) tensor the gradient kernels read, from whatever autograd hands over.

    The usual case is a (L, F, N) *view* of a row-major (N, F*L) gradient (what the layer after the
    encoding produces, seen through the module's permute+reshape): that is transposed by the
    library at streaming speed.  Anything else takes torch's generic copy (reference: funcs.py:47).
    """
    if grad.is_contiguous():
        return grad
    levels, feat, n = grad.shape
    cols = levels * feat
    if (grad.is_cuda and grad.dtype == torch.float32 and grad.stride() == (feat, 1, cols) and cols <= 255 and n > 0):
        out = torch.empty((levels, feat, n), dtype=torch.float32, device=grad.device)
        with torch.cuda.device(grad.device):
            _check(lib().penc_transpose(grad.data_ptr(), out.data_ptr(), n, cols, _stream()), "transpose")
        return out
    return grad.contiguous()


class SparseTableGrad:
    """A table gradient kept across calls together with the map of the slot ranges that hold anything
    (``penc_backward_sparse`` and friends): gradient calls add into ``grad`` and mark ``touched``;
    ``clear()`` or the sparse optimizer step zero what was touched and nothing else.  No call costs
    more than the batch touched, whatever the size of the table."""

    def __init__(self, lattice_values):
        levels, capacity, feat = lattice_values.shape
        self.nr_levels, self.capacity, self.nr_feat = int(levels), int(capacity), int(feat)
        self.grad = torch.zeros(lattice_values.shape, dtype=torch.float32, device=lattice_values.device)
        self.range_slots = int(lib().penc_touched_range_slots(self.capacity))
        entries = int(lib().penc_touched_map_entries(self.nr_feat, self.nr_levels, self.capacity))
        self.touched = torch.zeros(entries, dtype=torch.int32, device=lattice_values.device)

    def matches(self, lattice_values):
        return tuple(self.grad.shape) == tuple(lattice_values.shape) and self.grad.device == lattice_values.device

    def touched_map(self):
        """(L, F/2, ranges) view of the map: nonzero where a range of ``range_slots`` slots may hold a gradient."""
        return self.touched.view(self.nr_levels, self.nr_feat // 2, -1)

    def clear(self):
        with torch.cuda.device(self.grad.device):
            _check(lib().penc_clear_touched(self.grad.data_ptr(), self.nr_feat, self.nr_levels, self.capacity,
                                            self.touched.data_ptr(), _stream()), "clear_touched")


class EncodingInput:
    """Per-call inputs (reference: ``EncodingInput``, include/permutohedral_encoding/Encoding.cuh:14-29)."""

    def __init__(self, lattice_values, positions_raw, anneal_window, require_lattice_values_grad, require_positions_grad):
        self.m_lattice_values = lattice_values
        self.m_positions_raw = positions_raw
        self.m_anneal_window = anneal_window
        self.m_require_lattice_values_grad = bool(require_lattice_values_grad)
        self.m_require_positions_grad = bool(require_positions_grad)


class EncodingFixedParams:
    """Parameters fixed for the lifetime of an encoding (reference: ``EncodingFixedParams``, Encoding.cuh:31-70).

    Holds the random-shift tensor by handle, so an in-place update of the parameter (``load_state_dict``)
    is seen by later calls, and owns the scale-factor table.
    """

    def __init__(self, pos_dim, capacity, nr_levels, nr_feat_per_level, sigmas_list, random_shift_per_level,
                 concat_points, points_scaling):
        self.m_pos_dim = int(pos_dim)
        self.m_capacity = int(capacity)
        self.m_nr_levels = int(nr_levels)
        self.m_nr_feat_per_level = int(nr_feat_per_level)
        self.m_sigmas_list = [float(s) for s in np.asarray(sigmas_list, dtype=np.float32).reshape(-1)]
        self.m_random_shift_per_level = random_shift_per_level
        self.m_concat_points = bool(concat_points)
        self.m_points_scaling = float(points_scaling)
        sf = scale_factors(self.m_pos_dim, self.m_sigmas_list)
        self.m_scale_factor = torch.from_numpy(sf).to(random_shift_per_level.device)


class EncodingWrapper:
    """The native encoding object (reference: ``EncodingWrapper``, Encoding.cuh:162-188)."""

    def __init__(self, pos_dim, nr_feat_per_level, fixed_params):
        if nr_feat_per_level not in (2, 4, 8):
            raise RuntimeError("Encoding: nr_feat_per_level must be 2, 4 or 8")
        if pos_dim not in (2, 3, 4, 5, 6, 7, 8):
            raise RuntimeError("Encoding: pos_dim must be 2,3,4,5,6,7 or 8")
        self.pos_dim = int(pos_dim)
        self.nr_feat = int(nr_feat_per_level)
        self.fixed_params = fixed_params

    @staticmethod
    def create(pos_dim, nr_feat_per_level, fixed_params):
        return EncodingWrapper(pos_dim, nr_feat_per_level, fixed_params)

    # -- checks shared by the three calls (reference: src/Encoding.cu:38-45, 57-66, 119-125)
    half_table = None  # set by the module: torch.float16 or torch.bfloat16 to gather from such a copy of the fp32 table
    _half_copy = None
    _half_copy_of = None
    # set by the module (sparse_table_grad=True): table gradients are added into `sparse_grad`, a SparseTableGrad the
    # wrapper keeps across calls, and the gradient calls return None for them
    sparse_table_grad = False
    sparse_grad = None
    # set by the module (contiguous_output=True): the forward writes rows (N, F(L+E)) and returns a (L+E, F, N) view of them
    rows_output = False

    def sparse_grad_for(self, lattice_values):
        if self.sparse_grad is None or not self.sparse_grad.matches(lattice_values):
            self.sparse_grad = SparseTableGrad(lattice_values)
        return self.sparse_grad

    def gather_table(self, lattice_values):
        """The tensor the gathering kernels read for ``lattice_values``: the tensor itself, or, with
        ``half_table``, its 16-bit copy, made again whenever the tensor has been modified in place."""
        if self.half_table is None or lattice_values.dtype != torch.float32:
            return lattice_values
        key = (lattice_values.data_ptr(), lattice_values._version, lattice_values.device, tuple(lattice_values.shape),
               self.half_table)
        if self._half_copy_of != key:
            self._half_copy = lattice_values.detach().to(self.half_table)
            self._half_copy_of = key
        return self._half_copy

    def invalidate_half_table(self):
        """Forgets the 16-bit copy, so that the next call converts the table again.  The copy follows the
        tensor's version counter, which in-place operations under autograd's eyes and the bundled optimizers
        advance; a write that bypasses it (``p.data.add_(...)``, a kernel given the raw pointer) does not,
        and must be followed by this call."""
        self._half_copy = None
        self._half_copy_of = None

    def _check_common(self, inp):
        fp = self.fixed_params
        pos, lv, win = inp.m_positions_raw, inp.m_lattice_values, inp.m_anneal_window
        _check_f32_gpu(pos, "positions", 2)
        _require(pos.shape[0] != 0, "Why do we have 0 points")
        _require(pos.shape[1] == fp.m_pos_dim,
                 f"Pos dim for the lattice doesn't correspond with the position of the points. Lattice was initialized "
                 f"with {fp.m_pos_dim} and points have pos dim {pos.shape[1]}")
        if isinstance(lv, torch.Tensor) and lv.dtype in TABLE_FORMATS:  # a table kept in 16 bits per value: the *_half entry points
            _require(lv.is_cuda, "lattice_values should be in GPU memory. Please call .cuda() on the tensor")
            _require(lv.dim() == 3, f"lattice_values should have 3 dimensions, however it has sizes {tuple(lv.shape)}")
        else:
            _check_f32_gpu(lv, "lattice_values", 3)
        _require(lv.is_contiguous(), "lattice_values must be contiguous (a slot is loaded at a time)")
        _require(lv.shape[2] == self.nr_feat, f"lattice_values should be nr_levels x capacity x {self.nr_feat}")
        levels = lv.shape[0]
        shift = fp.m_random_shift_per_level
        _check_f32_gpu(shift, "random_shift_per_level", 2)
        _require(shift.shape[0] == levels,
                 "Random shift should have the first dimension the same as the nr of resolutions")
        _require(shift.shape[1] == fp.m_pos_dim, "Random shift should have the second dimension the same as the pos dim")
        _check_f32_gpu(win, "anneal_window", 1)
        _require(win.shape[0] == levels, "anneal_window should have the first dimension the same as the nr of resolutions")
        _require(fp.m_scale_factor.shape == (levels, fp.m_pos_dim), "scale list should have one entry per level")
        dev = pos.device
        for t, name in ((lv, "lattice_values"), (shift, "random_shift_per_level"), (win, "anneal_window")):
            _require(t.device == dev, f"{name} must be on the same device as positions")
        if fp.m_scale_factor.device != dev:
            fp.m_scale_factor = fp.m_scale_factor.to(dev)
        return pos.contiguous(), lv, shift.contiguous(), win.contiguous(), levels, lv.shape[1]

    def _check_grad(self, grad, levels, extra, n, allow_rows=False):
        _check_f32_gpu(grad, "grad_sliced_values_monolithic", 3)
        _require(grad.is_contiguous() or (allow_rows and is_row_major_view(grad)),
                 "Grad sliced values needs to be contiguous. Please call .contiguous() on it")
        _require(grad.shape == (levels + extra, self.nr_feat, n),
                 "grad_sliced_values_monolithic should be nr_resolutions x val_dim x nr_positions")

    def forward(self, inp):
        """-> sliced values (L+E, 2, N)  (reference: Encoding<D,2>::forward, src/Encoding.cu:55-108)."""
        fp = self.fixed_params
        pos, lv, shift, win, levels, cap = self._check_common(inp)
        n = pos.shape[0]
        extra = extra_levels(self.pos_dim, self.nr_feat, fp.m_concat_points)
        if self.rows_output and lv.dtype not in TABLE_FORMATS and self.nr_feat * (levels + extra) <= 255:
            # rows[n][F*level + feature], handed back as the (L+E, F, N) view of them: the module's
            # permute + reshape of that view is the contiguous (N, F(L+E)) array itself
            cols = self.nr_feat * (levels + extra)
            rows = torch.empty((n, cols), dtype=torch.float32, device=pos.device)
            with torch.cuda.device(pos.device):
                nbytes = int(lib().penc_forward_rowmajor_workspace_bytes(self.pos_dim, self.nr_feat, n, levels, int(fp.m_concat_points)))
                ws = torch.empty(nbytes, dtype=torch.uint8, device=pos.device)
                _check(lib().penc_forward_rowmajor(self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv),
                                                   _ptr(fp.m_scale_factor), _ptr(shift), _ptr(win), _ptr(rows), cols,
                                                   int(fp.m_concat_points), fp.m_points_scaling, _ptr(ws), nbytes, _stream()),
                       "forward_rowmajor")
            return rows.view(n, levels + extra, self.nr_feat).permute(1, 2, 0)
        out = torch.empty((levels + extra, self.nr_feat, n), dtype=torch.float32, device=pos.device)
        with torch.cuda.device(pos.device):
            if lv.dtype in TABLE_FORMATS:
                _check(lib().penc_forward_half(self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv),
                                               TABLE_FORMATS[lv.dtype], _ptr(fp.m_scale_factor), _ptr(shift), _ptr(win),
                                               _ptr(out), int(fp.m_concat_points), fp.m_points_scaling, _stream()), "forward")
            else:
                _check(lib().penc_forward(self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv),
                                          _ptr(fp.m_scale_factor), _ptr(shift), _ptr(win), _ptr(out),
                                          int(fp.m_concat_points), fp.m_points_scaling, _stream()), "forward")
        return out

    def backward(self, inp, grad_sliced_values_monolithic):
        """-> (lattice_values_grad (L,C,2) or None, positions_grad (N,D) or None)
        (reference: Encoding<D,2>::backward, src/Encoding.cu:112-215).

        The upstream gradient may be the contiguous (L+E, 2, N) tensor the reference asks for, or a
        (L+E, 2, N) view of row-major rows (what autograd hands over for the module's (N, 2(L+E))
        output, see ``is_row_major_view``): that is read as it is, with no layout copy by the caller."""
        fp = self.fixed_params
        pos, lv, shift, win, levels, cap = self._check_common(inp)
        n = pos.shape[0]
        extra = extra_levels(self.pos_dim, self.nr_feat, fp.m_concat_points)
        grad = grad_sliced_values_monolithic
        self._check_grad(grad, levels, extra, n, allow_rows=True)
        half = lv.dtype in TABLE_FORMATS  # the gradient w.r.t. the table is fp32 either way
        pos_grad = torch.empty_like(pos) if inp.m_require_positions_grad else None
        if self.sparse_table_grad and inp.m_require_lattice_values_grad:
            _require(not half, "sparse_table_grad needs an fp32 table")
            sparse = self.sparse_grad_for(lv)
            rows = not grad.is_contiguous()
            copy_bytes = 4 * self.nr_feat * levels * n + 512 if rows and pos_grad is not None else 0
            with torch.cuda.device(pos.device):
                ws = scatter_workspace(self.pos_dim, n, levels, cap, pos.device, True, pos_grad is not None,
                                       fixed_bytes=copy_bytes, required_bytes=copy_bytes, nr_feat=self.nr_feat)
                _check(lib().penc_backward_sparse(
                    self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), _ptr(fp.m_scale_factor), _ptr(shift),
                    _ptr(win), _ptr(grad), grad.stride(2) if rows else 0, _ptr(sparse.grad), _ptr(sparse.touched), _ptr(pos_grad),
                    _ptr(ws), 0 if ws is None else ws.numel(), _stream()), "backward_sparse")
            return None, pos_grad
        lv_grad = torch.empty(lv.shape, dtype=torch.float32, device=lv.device) if inp.m_require_lattice_values_grad else None
        if lv_grad is None and pos_grad is None:
            return None, None
        with torch.cuda.device(pos.device):
            if not grad.is_contiguous():  # rows (N, 2(L+E))
                copy_bytes = 4 * self.nr_feat * levels * n + 512 if pos_grad is not None else 0
                ws = scatter_workspace(self.pos_dim, n, levels, cap, pos.device, lv_grad is not None, pos_grad is not None,
                                       fixed_bytes=copy_bytes, required_bytes=copy_bytes, nr_feat=self.nr_feat)
                table = (_ptr(lv), TABLE_FORMATS[lv.dtype]) if half else (_ptr(lv),)
                _check((lib().penc_backward_half if half else lib().penc_backward_rowmajor)(
                    self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), *table, _ptr(fp.m_scale_factor), _ptr(shift),
                    _ptr(win), _ptr(grad), grad.stride(2), _ptr(lv_grad), _ptr(pos_grad), _ptr(ws),
                    0 if ws is None else ws.numel(), _stream()), "backward")
                return lv_grad, pos_grad
            ws = scatter_workspace(self.pos_dim, n, levels, cap, pos.device, lv_grad is not None, pos_grad is not None,
                                   nr_feat=self.nr_feat)
            if half:
                _check(lib().penc_backward_half(self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv),
                                                TABLE_FORMATS[lv.dtype], _ptr(fp.m_scale_factor), _ptr(shift), _ptr(win),
                                                _ptr(grad), 0, _ptr(lv_grad),
                                                _ptr(pos_grad), _ptr(ws), 0 if ws is None else ws.numel(), _stream()),
                       "backward")
                return lv_grad, pos_grad
            _check(lib().penc_backward(self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv),
                                       _ptr(fp.m_scale_factor), _ptr(shift), _ptr(win), _ptr(grad), _ptr(lv_grad),
                                       _ptr(pos_grad), _ptr(ws), 0 if ws is None else ws.numel(), _stream()), "backward")
        return lv_grad, pos_grad

    def double_backward_from_positions(self, inp, double_positions_grad, grad_sliced_values_monolithic,
                                       want_lattice_values_grad=True):
        """-> (lattice_values_grad (L,C,2), grad_grad_sliced_values (L+E,2,N))
        (reference: Encoding<D,2>::double_backward_from_positions, src/Encoding.cu:219-334).
        The upstream gradient of the first backward may again be a view of row-major rows.
        Without ``want_lattice_values_grad`` only the gathering half runs and the first result is None."""
        fp = self.fixed_params
        pos, lv, shift, win, levels, cap = self._check_common(inp)
        n = pos.shape[0]
        extra = extra_levels(self.pos_dim, self.nr_feat, fp.m_concat_points)
        grad = grad_sliced_values_monolithic
        self._check_grad(grad, levels, extra, n, allow_rows=True)
        _check_f32_gpu(double_positions_grad, "double_positions_grad", 2)
        _require(double_positions_grad.shape == pos.shape, "double_positions_grad should be nr_positions x pos_dim")
        dpos = double_positions_grad.contiguous()
        ggs = torch.empty((levels + extra, self.nr_feat, n), dtype=torch.float32, device=pos.device)
        if not want_lattice_values_grad:
            with torch.cuda.device(pos.device):
                if lv.dtype in TABLE_FORMATS:
                    _check(lib().penc_double_backward_from_positions_half(
                        self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), TABLE_FORMATS[lv.dtype],
                        _ptr(fp.m_scale_factor), _ptr(shift), _ptr(win), _ptr(dpos), _ptr(grad),
                        0 if grad.is_contiguous() else grad.stride(2), None, _ptr(ggs), int(fp.m_concat_points), None, 0,
                        _stream()), "double_backward_from_positions")
                else:
                    _check(lib().penc_double_backward_from_positions_rowmajor(
                        self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), _ptr(fp.m_scale_factor), _ptr(shift),
                        _ptr(win), _ptr(dpos), _ptr(grad), grad.stride(2), None, _ptr(ggs), int(fp.m_concat_points),
                        None, 0, _stream()) if not grad.is_contiguous() else lib().penc_double_backward_from_positions(
                        self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), _ptr(fp.m_scale_factor), _ptr(shift),
                        _ptr(win), _ptr(dpos), _ptr(grad), None, _ptr(ggs), int(fp.m_concat_points), None, 0, _stream()),
                        "double_backward_from_positions")
            return None, ggs
        if self.sparse_table_grad:
            _require(lv.dtype not in TABLE_FORMATS, "sparse_table_grad needs an fp32 table")
            sparse = self.sparse_grad_for(lv)
            with torch.cuda.device(pos.device):
                ws = scatter_workspace(self.pos_dim, n, levels, cap, pos.device, nr_feat=self.nr_feat)
                _check(lib().penc_double_backward_from_positions_sparse(
                    self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), _ptr(fp.m_scale_factor), _ptr(shift),
                    _ptr(win), _ptr(dpos), _ptr(grad), 0 if grad.is_contiguous() else grad.stride(2), _ptr(sparse.grad),
                    _ptr(sparse.touched), _ptr(ggs), int(fp.m_concat_points), _ptr(ws), 0 if ws is None else ws.numel(),
                    _stream()), "double_backward_from_positions_sparse")
            return None, ggs
        lv_grad = torch.empty(lv.shape, dtype=torch.float32, device=lv.device)
        with torch.cuda.device(pos.device):
            ws = scatter_workspace(self.pos_dim, n, levels, cap, pos.device, nr_feat=self.nr_feat)
            if lv.dtype in TABLE_FORMATS:
                _check(lib().penc_double_backward_from_positions_half(
                    self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), TABLE_FORMATS[lv.dtype],
                    _ptr(fp.m_scale_factor), _ptr(shift),
                    _ptr(win), _ptr(dpos), _ptr(grad), 0 if grad.is_contiguous() else grad.stride(2), _ptr(lv_grad), _ptr(ggs),
                    int(fp.m_concat_points), _ptr(ws), 0 if ws is None else ws.numel(), _stream()),
                    "double_backward_from_positions")
                return lv_grad, ggs
            if not grad.is_contiguous():
                _check(lib().penc_double_backward_from_positions_rowmajor(
                    self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), _ptr(fp.m_scale_factor), _ptr(shift),
                    _ptr(win), _ptr(dpos), _ptr(grad), grad.stride(2), _ptr(lv_grad), _ptr(ggs), int(fp.m_concat_points),
                    _ptr(ws), 0 if ws is None else ws.numel(), _stream()), "double_backward_from_positions")
                return lv_grad, ggs
            _check(lib().penc_double_backward_from_positions(
                self.pos_dim, self.nr_feat, n, levels, cap, _ptr(pos), _ptr(lv), _ptr(fp.m_scale_factor), _ptr(shift),
                _ptr(win), _ptr(dpos), _ptr(grad), _ptr(lv_grad), _ptr(ggs),
                int(fp.m_concat_points), _ptr(ws), 0 if ws is None else ws.numel(), _stream()),
                "double_backward_from_positions")
        return lv_grad, ggs

    def simplex_debug(self, positions, capacity, gather_path=False):
        """Introspection: dict(rem0, rank, slot (int32), barycentric) each of shape (L, N, D+1).

        ``gather_path`` picks the device routine whose slots and weights are reported: False for the
        select chains of the scattering and position-gradient kernels, True for the LDS rank sort of
        the forward and grad-of-grad kernels."""
        fp = self.fixed_params
        _check_f32_gpu(positions, "positions", 2)
        pos = positions.contiguous()
        n, levels = pos.shape[0], fp.m_scale_factor.shape[0]
        shape = (levels, n, self.pos_dim + 1)
        out = {k: torch.empty(shape, dtype=torch.int32, device=pos.device) for k in ("rem0", "rank", "slot")}
        out["barycentric"] = torch.empty(shape, dtype=torch.float32, device=pos.device)
        shift = fp.m_random_shift_per_level.contiguous()
        with torch.cuda.device(pos.device):
            _check(lib().penc_simplex_debug(self.pos_dim, n, levels, int(capacity), _ptr(pos),
                                            _ptr(fp.m_scale_factor.to(pos.device)), _ptr(shift), int(bool(gather_path)),
                                            _ptr(out["rem0"]),
                                            _ptr(out["rank"]), _ptr(out["slot"]), _ptr(out["barycentric"]), _stream()),
                   "simplex_debug")
        return out
