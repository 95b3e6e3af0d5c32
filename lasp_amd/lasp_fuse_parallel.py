"""lasp_fuse_parallel: as lasp_fuse, but the chunk is cut into segments processed in
parallel and the per-segment states are kept for backward (lasp/lasp_fuse_parallel.py)."""
import torch

from . import _abi
from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspFuseParallel", "lasp_fuse_parallel_", "lasp_fuse_parallel"]


def lasp_forward(q, k, v, s, KV, BLOCK=128, CBLOCK=64):
    """Launch shim with the signature of lasp/lasp_fuse_parallel.py:833-944.

    Returns (o, kv, KV_out): kv is the float32 cache of the states entering each
    segment, to be handed to lasp_backward; KV_out is a new tensor and the caller's
    KV keeps the incoming state, as in the reference (:941-942).  BLOCK and CBLOCK
    are accepted for signature compatibility; the segment length is the library's.
    """
    KV_out = torch.empty_like(KV)
    o, kv, _ = _abi.chunk_fwd(q, k, v, s, kv_in=KV, kv_out=KV_out)
    return o, kv, KV_out


def lasp_backward(q, k, v, s, do, kv, KV, DKV, BLOCK=128, CBLOCK=64):
    """Launch shim with the signature of lasp/lasp_fuse_parallel.py:947-1070.

    kv is the cache lasp_forward returned for the same chunk, KV the state that
    entered it, DKV the incoming dKV.  Returns (dq, dk, dv, DKV_out) with DKV_out a
    new tensor (:1067-1070).
    """
    DKV_out = torch.empty_like(DKV)
    dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, kv_in=KV, dkv_in=DKV, dkv_out=DKV_out, kv_seg_states=kv)
    return dq, dk, dv, DKV_out


class LaspFuseParallel(torch.autograd.Function):
    """forward(q, k, v, s, KV, DKV) as lasp/lasp_fuse_parallel.py:1073-1137 (incl. the barrier)."""

    @staticmethod
    def forward(ctx, q, k, v, s, KV, DKV):
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, True, True, True)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:6]


lasp_fuse_parallel_ = LaspFuseParallel.apply


def lasp_fuse_parallel(q, k, v, ed, KV, DKV):
    if q.shape[-1] <= 128:
        return lasp_fuse_parallel_(q, k, v, ed, KV, DKV)
    return run_sliced(q, k, v, ed, KV, DKV, True, True, True)
