"""A fused AdamW for the encoding's table (``penc_adamw_step``).

The reference library has no optimiser; its scripts step the table with ``torch.optim.AdamW``
(examples/performance.py:161), which walks the whole table with several elementwise kernels per
step.  ``AdamW`` here applies the same update (same formulas and order of operations, no amsgrad) in
one kernel per parameter, and can leave entries whose gradient is exactly zero untouched
(``skip_zero_gradients``), the usual way to train hash tables most of whose slots see no point in a
step.
"""
import torch

from . import _native


class AdamW(torch.optim.Optimizer):
    """``torch.optim.AdamW`` semantics (decoupled weight decay, no amsgrad) for fp32 GPU parameters.

    ``skip_zero_gradients=True`` leaves an entry with a zero gradient as it is: value, both moments
    and weight decay.  With ``False`` (default) the result follows ``torch.optim.AdamW`` step by step.
    """

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, skip_zero_gradients=False):
        if lr < 0.0 or eps < 0.0 or weight_decay < 0.0 or not 0.0 <= betas[0] < 1.0 or not 0.0 <= betas[1] < 1.0:
            raise ValueError("AdamW: lr, eps and weight_decay must be non-negative and the betas in [0, 1)")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
                                      skip_zero_gradients=bool(skip_zero_gradients)))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            for p in group["params"]:
                if p.grad is None:
                    continue
                if not (p.is_cuda and p.dtype == torch.float32 and p.is_contiguous()):
                    raise RuntimeError("AdamW: parameters must be contiguous float32 tensors in GPU memory")
                grad = p.grad
                if grad.is_sparse or grad.dtype != torch.float32:
                    raise RuntimeError("AdamW: gradients must be dense float32 tensors")
                grad = grad.contiguous()
                state = self.state[p]
                if not state:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                state["step"] += 1
                with torch.cuda.device(p.device):
                    _native._check(_native.lib().penc_adamw_step(
                        p.data_ptr(), grad.data_ptr(), state["exp_avg"].data_ptr(), state["exp_avg_sq"].data_ptr(), p.numel(),
                        float(group["lr"]), float(beta1), float(beta2), float(group["eps"]), float(group["weight_decay"]),
                        int(state["step"]), int(group["skip_zero_gradients"]), _native._stream()), "adamw_step")
                # the kernel wrote through a raw pointer: record the in-place change for autograd's version
                # checks and for the half-precision copy the module keeps of its table
                torch.autograd.graph.increment_version(p)
        return loss


class SparseTableAdamW(torch.optim.Optimizer):
    """AdamW on the tables of ``PermutoEncoding(..., sparse_table_grad=True)`` modules (``penc_adamw_step_sparse``).

    Takes the gradient from each module's ``table_grad`` and visits only the slot ranges its map names:
    an entry whose gradient is exactly zero keeps its value and both moments (``AdamW`` with
    ``skip_zero_gradients``), and the gradients used and the map are zeroed for the next step.  Other
    parameters (the MLP after the encoding) take any other optimizer.
    """

    def __init__(self, encodings, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2):
        encodings = list(encodings) if isinstance(encodings, (list, tuple)) else [encodings]
        if not encodings or not all(getattr(e, "sparse_table_grad", False) for e in encodings):
            raise ValueError("SparseTableAdamW: pass PermutoEncoding modules built with sparse_table_grad=True")
        if lr < 0.0 or eps < 0.0 or weight_decay < 0.0 or not 0.0 <= betas[0] < 1.0 or not 0.0 <= betas[1] < 1.0:
            raise ValueError("SparseTableAdamW: lr, eps and weight_decay must be non-negative and the betas in [0, 1)")
        self._encoding_of = {id(e.lattice_values): e for e in encodings}
        super().__init__([e.lattice_values for e in encodings], dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))

    def zero_grad(self, set_to_none=True):
        """Zeroes what the gradient calls have touched since the last step (``step`` does so itself)."""
        for enc in self._encoding_of.values():
            if enc.table_grad is not None:
                enc.table_grad.clear()

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            for p in group["params"]:
                sparse = self._encoding_of[id(p)].table_grad
                if sparse is None:
                    continue  # no gradient call yet
                if not (p.is_cuda and p.dtype == torch.float32 and p.is_contiguous() and sparse.matches(p)):
                    raise RuntimeError("SparseTableAdamW: the table must be a contiguous float32 GPU tensor of the gradient's shape")
                state = self.state[p]
                if not state:
                    state["step"] = 0
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                state["step"] += 1
                with torch.cuda.device(p.device):
                    _native._check(_native.lib().penc_adamw_step_sparse(
                        p.data_ptr(), sparse.grad.data_ptr(), state["exp_avg"].data_ptr(), state["exp_avg_sq"].data_ptr(),
                        sparse.nr_feat, sparse.nr_levels, sparse.capacity, sparse.touched.data_ptr(), float(group["lr"]),
                        float(beta1), float(beta2), float(group["eps"]), float(group["weight_decay"]), int(state["step"]), 1,
                        _native._stream()), "adamw_step_sparse")
                torch.autograd.graph.increment_version(p)
        return loss
