"""lasp_fuse: per-rank chunk with KV state in and out (lasp/lasp_fuse.py).

The reference's backward re-runs the kv recurrence (lasp/lasp_fuse.py:237-260).  Here the forward
leaves the state entering each segment in a workspace anyway, so the operator keeps it for backward
(64 KiB per (b, h, segment)) instead of re-reading K and V to rebuild it; the launch shims below
recompute, as they have no place to keep it."""
import torch

from . import _abi
from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspFuse", "lasp_fuse_", "lasp_fuse"]


def lasp_forward(q, k, v, s, KV):
    """Launch shim with the signature of lasp/lasp_fuse.py:356-406.

    Returns o for one chunk.  KV, float32 (b, h, d, e), holds the incoming state and
    is overwritten with the outgoing one, as the reference kernel does (:126-127).
    """
    o, _, _ = _abi.chunk_fwd(q, k, v, s, kv_in=KV, kv_out=KV)
    return o


def lasp_backward(q, k, v, s, do, KV, DKV):
    """Launch shim with the signature of lasp/lasp_fuse.py:409-475.

    KV is the state that entered the forward (the copy saved at :496); DKV holds the
    incoming dKV and is overwritten with the outgoing one.  Returns (dq, dk, dv).
    """
    return _abi.chunk_bwd(q, k, v, s, do, kv_in=KV, dkv_in=DKV, dkv_out=DKV)


class LaspFuse(torch.autograd.Function):
    """forward(q, k, v, s, KV, DKV) as lasp/lasp_fuse.py:478-532."""

    @staticmethod
    def forward(ctx, q, k, v, s, KV, DKV):
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, True, False)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:6]


lasp_fuse_ = LaspFuse.apply


def lasp_fuse(q, k, v, ed, KV, DKV):
    """KV, DKV: float32 (b, h, d, e) scratch owned by the caller; KV is left holding KV_out."""
    if q.shape[-1] <= 128:
        return lasp_fuse_(q, k, v, ed, KV, DKV)
    return run_sliced(q, k, v, ed, KV, DKV, True, False)
