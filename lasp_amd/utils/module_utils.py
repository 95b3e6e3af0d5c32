"""Slope and memory helpers (counterparts of lasp/utils/module_utils.py)."""
import math

import torch

__all__ = ["build_slope_tensor", "get_memory"]


def _geometric(m: int):
    # m a power of two: 2^(-8/m), 2^(-16/m), ...
    base = 2.0 ** (-8.0 / m)
    return [base ** (i + 1) for i in range(m)]


def build_slope_tensor(n_attention_heads: int) -> torch.Tensor:
    """Per-head decay slopes, shape (h, 1, 1), float32.

    Same values as lasp/utils/module_utils.py:6-31: for a power-of-two head count
    s_i = 2^(-8 (i+1) / h); otherwise the slopes of the largest power of two p <= h
    followed by the first h - p odd-indexed members (1st, 3rd, ...) of the 2p series.
    """
    h = int(n_attention_heads)
    if h <= 0:
        raise ValueError("n_attention_heads must be positive")
    p = 1 << (h.bit_length() - 1)
    values = _geometric(p)
    if p != h:
        values += _geometric(2 * p)[0::2][: h - p]
    return torch.tensor(values, dtype=torch.float32).reshape(h, 1, 1)


def get_memory(device):
    """Peak allocated MiB on `device` since the last call (lasp/utils/module_utils.py:34-38)."""
    mb_used = torch.cuda.max_memory_allocated(device) / 1024 / 1024
    torch.cuda.reset_peak_memory_stats(device)
    return mb_used
