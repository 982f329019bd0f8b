"""Anneal-window helpers (reference: src/pytorch_modules/utils.py)."""
import math

import torch


def cosine_easing_window(num_freqs, alpha):
    """Eases the levels in one by one with a cosine as ``alpha`` goes from 0 to ``num_freqs``.

    ``win[k] = 0.5 * (1 + cos(pi * clip(alpha - k, 0, 1) + pi))``: exactly 1 for fully eased-in
    levels, exactly 0 for levels not yet started (reference: utils.py:5-16).
    """
    x = torch.clip(alpha - torch.arange(num_freqs, dtype=torch.float32), 0.0, 1.0)
    return 0.5 * (1 + torch.cos(math.pi * x + math.pi))


def map_range_val(input_val, input_start, input_end, output_start, output_end):
    """Clamps ``input_val`` to [input_start, input_end] and maps it linearly (reference: utils.py:19-23)."""
    input_clamped = max(input_start, min(input_end, input_val))
    return output_start + ((output_end - output_start) / (input_end - input_start)) * (input_clamped - input_start)
