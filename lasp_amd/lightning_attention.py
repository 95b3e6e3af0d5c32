"""Single-device causal decayed linear attention (lasp/lightning_attention.py)."""
import torch

from ._chain import ChunkFunction, run_sliced

__all__ = ["LightningAttention", "lightning_attn_", "lightning_attn"]


class LightningAttention(torch.autograd.Function):
    """O = ((Q K^T) (.) M) V with M_ij = exp(-s_h (i - j)) for j <= i.

    Same signature as lasp/lightning_attention.py:396-504: forward(q, k, v, s),
    gradients for q, k, v only.
    """

    @staticmethod
    def forward(ctx, q, k, v, s):
        # the per-segment states (64 KiB per (b, h, segment)) are kept for backward:
        # cheaper than re-reading K and V to rebuild them
        return ChunkFunction.forward(ctx, q, k, v, s, None, None, True, False)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:4]


lightning_attn_ = LightningAttention.apply


def lightning_attn(q, k, v, ed):
    """q, k (b, h, n, d); v (b, h, n, e); ed: h slopes.  Returns (b, h, n, e) in q.dtype."""
    d = q.shape[-1]
    if d <= 128:
        return lightning_attn_(q, k, v, ed)
    return run_sliced(q, k, v, ed, None, None, True, False)
