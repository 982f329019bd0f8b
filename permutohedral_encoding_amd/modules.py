"""``PermutoEncoding`` and ``Coarse2Fine`` (reference: src/pytorch_modules/modules.py)."""
import math

import numpy as np
import torch

from . import _native
from .funcs import PermutoEncodingFunc
from .utils import cosine_easing_window


class PermutoEncoding(torch.nn.Module):
    """Multi-resolution permutohedral-lattice hash encoding.

    Same constructor, parameters (``lattice_values`` (L, C, F), ``random_shift_per_level`` (L, D)) and
    forward as the reference module (modules.py:10-103).  Two additions: ``device`` defaults to the
    current GPU (a CPU device is accepted for construction only: the forward has no CPU path), and
    ``lattice_half_precision`` (``True`` or ``torch.float16``, or ``torch.bfloat16``) makes the
    kernels gather from a 16-bit copy of ``lattice_values`` (the switch the reference carries
    disabled, EncodingGPU.cuh:12).  The parameter itself and every gradient stay fp32; the copy is
    refreshed whenever the parameter has been modified in place (optimizer steps), so it pays for
    large tables and for inference.  float16 resolves the reference's initial values (about 1e-5)
    only to 6e-8; bfloat16 keeps three significant digits at any magnitude.

    ``contiguous_output=True`` returns the (N, F(L+E)) result as a contiguous array instead of the strided
    view the reference's permute + reshape produces (modules.py:87): for consumers that would otherwise
    copy it (``torch.cat``, element-wise layers); a matrix multiplication takes the view as it is.

    ``sparse_table_grad=True`` is for tables that dwarf the batch: the gradient w.r.t. ``lattice_values``
    is not handed to autograd (``lattice_values.grad`` stays None) but added into ``table_grad``, a
    gradient array the module keeps across steps together with a map of the slot ranges that hold
    anything; ``permutohedral_encoding_amd.optim.SparseTableAdamW`` steps the table from it and zeroes
    what was touched.  Neither the gradient calls nor the optimizer then walk the whole table (the
    reference clears a dense gradient in every call, src/Encoding.cu:141, 246, and its training
    protocol steps the whole table, examples/performance.py:99-101).
    """

    def __init__(self, pos_dim, capacity, nr_levels, nr_feat_per_level, scale_per_level,
                 appply_random_shift_per_level=True, concat_points=False, concat_points_scaling=1.0, device=None,
                 lattice_half_precision=False, sparse_table_grad=False, contiguous_output=False):
        super().__init__()
        self.sparse_table_grad = bool(sparse_table_grad)
        self.contiguous_output = bool(contiguous_output)
        if lattice_half_precision in (None, False):
            self.lattice_half_precision = None
        elif lattice_half_precision is True or lattice_half_precision == torch.float16:
            self.lattice_half_precision = torch.float16
        elif lattice_half_precision == torch.bfloat16:
            self.lattice_half_precision = torch.bfloat16
        else:
            raise ValueError("lattice_half_precision must be False, True, torch.float16 or torch.bfloat16")
        self.pos_dim = pos_dim
        self.capacity = capacity
        self.nr_levels = nr_levels
        self.nr_feat_per_level = nr_feat_per_level
        self.scale_per_level = np.asarray(scale_per_level, dtype=np.float32).reshape(-1)
        self.appply_random_shift_per_level = appply_random_shift_per_level
        self.concat_points = concat_points
        self.concat_points_scaling = concat_points_scaling
        if len(self.scale_per_level) != nr_levels:
            raise ValueError("scale_per_level should have one entry per level")
        if device is None:
            if not torch.cuda.is_available():
                raise RuntimeError("PermutoEncoding needs a GPU (no CPU implementation exists)")
            device = torch.device("cuda", torch.cuda.current_device())
        device = torch.device(device)

        # hash-table values: drawn as (capacity, levels, feat) and permuted, like the reference (modules.py:25-27)
        lattice_values = torch.randn(capacity, nr_levels, nr_feat_per_level) * 1e-5
        lattice_values = lattice_values.permute(1, 0, 2).contiguous()
        self.lattice_values = torch.nn.Parameter(lattice_values.to(device))

        # per-level random shift against collisions; a Parameter only so that it is checkpointed (modules.py:30-32).
        # Without the shift the reference builds a size-1 placeholder that its own launcher then rejects
        # (modules.py:34, src/Encoding.cu:63); here "no shift" is an all-zero shift.
        if appply_random_shift_per_level:
            random_shift_per_level = torch.randn(nr_levels, pos_dim) * 10
        else:
            random_shift_per_level = torch.zeros(nr_levels, pos_dim)
        self.random_shift_per_level = torch.nn.Parameter(random_shift_per_level.to(device))

        self.anneal_window = torch.ones((nr_levels), device=device)
        self.fixed_params, self.lattice = self._make_lattice_wrapper()

    def _make_lattice_wrapper(self):
        fixed_params = _native.EncodingFixedParams(self.pos_dim, self.capacity, self.nr_levels, self.nr_feat_per_level,
                                                   self.scale_per_level, self.random_shift_per_level,
                                                   self.concat_points, self.concat_points_scaling)
        lattice = _native.EncodingWrapper.create(self.pos_dim, self.nr_feat_per_level, fixed_params)
        lattice.half_table = getattr(self, "lattice_half_precision", None)
        lattice.sparse_table_grad = getattr(self, "sparse_table_grad", False)
        lattice.rows_output = getattr(self, "contiguous_output", False)
        return fixed_params, lattice

    def invalidate_half_table(self):
        """With ``lattice_half_precision``: makes the next forward convert ``lattice_values`` again.  Needed only
        after a write autograd's version counter does not see (``lattice_values.data.add_(...)``, a kernel
        given the raw pointer); optimizer steps, ``load_state_dict``, ``.to()`` and ``train()``/``eval()``
        are followed automatically."""
        self.lattice.invalidate_half_table()

    def train(self, mode=True):
        self.lattice.invalidate_half_table()  # a cheap point at which a stale copy cannot survive
        return super().train(mode)

    def load_state_dict(self, *args, **kwargs):
        out = super().load_state_dict(*args, **kwargs)
        self.lattice.invalidate_half_table()
        return out

    @property
    def table_grad(self):
        """With ``sparse_table_grad``: the ``SparseTableGrad`` the gradient calls add into (None before the first one)."""
        return self.lattice.sparse_grad

    def __getstate__(self):
        state = self.__dict__.copy()
        del state["fixed_params"]  # native handles are rebuilt on load (modules.py:51-62)
        del state["lattice"]
        return state

    def __setstate__(self, state):
        self.__dict__.update(state)
        self.fixed_params, self.lattice = self._make_lattice_wrapper()

    def _apply(self, fn, *args, **kwargs):
        # .to()/.cuda() replace the parameter tensors; the native handle must follow them
        out = super()._apply(fn, *args, **kwargs)
        self.lattice.invalidate_half_table()
        self.anneal_window = fn(self.anneal_window)
        self.fixed_params.m_random_shift_per_level = self.random_shift_per_level
        return out

    def forward(self, positions, anneal_window=None):
        nr_positions = positions.shape[0]
        if anneal_window is None:
            anneal_window = self.anneal_window
        else:
            anneal_window = anneal_window.to(device=positions.device, dtype=torch.float32)
        require_lattice_values_grad = self.lattice_values.requires_grad and torch.is_grad_enabled()
        require_positions_grad = positions.requires_grad and torch.is_grad_enabled()
        sliced_values = PermutoEncodingFunc.apply(self.lattice, self.lattice_values, positions, anneal_window,
                                                  require_lattice_values_grad, require_positions_grad)
        # (levels, feat, points) -> (points, levels*feat): column = level*feat_per_level + feat (modules.py:87)
        return sliced_values.permute(2, 0, 1).reshape(nr_positions, -1)

    def output_dims(self):
        nr_resolutions_extra = 0
        if self.concat_points:
            nr_resolutions_extra = math.ceil(float(self.pos_dim) / self.nr_feat_per_level)
        return self.nr_feat_per_level * (self.nr_levels + nr_resolutions_extra)


class Coarse2Fine(torch.nn.Module):
    """Anneal window over ``nr_values`` levels for ``t`` in [0, 1] (reference: modules.py:109-127)."""

    def __init__(self, nr_values):
        super().__init__()
        self.nr_values = nr_values
        self.last_t = 0

    def forward(self, t):
        alpha = t * self.nr_values
        window = cosine_easing_window(self.nr_values, alpha)
        self.last_t = t
        assert t <= 1.0, "t cannot be larger than 1.0"
        return window

    def get_last_t(self):
        return self.last_t
