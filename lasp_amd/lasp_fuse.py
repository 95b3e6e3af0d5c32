"""lasp_fuse: per-rank chunk with KV in/out, states recomputed in backward (lasp/lasp_fuse.py)."""
import torch

from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspFuse", "lasp_fuse_", "lasp_fuse"]


class LaspFuse(torch.autograd.Function):
    """forward(q, k, v, s, KV, DKV) as lasp/lasp_fuse.py:478-532."""

    @staticmethod
    def forward(ctx, q, k, v, s, KV, DKV):
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, False, False)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:6]


lasp_fuse_ = LaspFuse.apply


def lasp_fuse(q, k, v, ed, KV, DKV):
    """KV, DKV: float32 (b, h, d, e) scratch owned by the caller; KV is left holding KV_out."""
    if q.shape[-1] <= 128:
        return lasp_fuse_(q, k, v, ed, KV, DKV)
    return run_sliced(q, k, v, ed, KV, DKV, False, False)
