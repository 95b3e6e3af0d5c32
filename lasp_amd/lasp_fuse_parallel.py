"""lasp_fuse_parallel: as lasp_fuse, but the chunk is cut into segments processed in
parallel and the per-segment states are kept for backward (lasp/lasp_fuse_parallel.py)."""
import torch

from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspFuseParallel", "lasp_fuse_parallel_", "lasp_fuse_parallel"]


class LaspFuseParallel(torch.autograd.Function):
    """forward(q, k, v, s, KV, DKV) as lasp/lasp_fuse_parallel.py:1073-1137 (incl. the barrier)."""

    @staticmethod
    def forward(ctx, q, k, v, s, KV, DKV):
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, True, True)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:6]


lasp_fuse_parallel_ = LaspFuseParallel.apply


def lasp_fuse_parallel(q, k, v, ed, KV, DKV):
    if q.shape[-1] <= 128:
        return lasp_fuse_parallel_(q, k, v, ed, KV, DKV)
    return run_sliced(q, k, v, ed, KV, DKV, True, True)
