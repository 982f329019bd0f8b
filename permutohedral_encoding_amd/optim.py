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
