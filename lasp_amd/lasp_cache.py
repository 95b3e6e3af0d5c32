"""lasp_cache: lasp_naive with caller-provided buffers (lasp/lasp_cache.py).

The reference re-uses the caller's `array` (positions 0..n-1, from which it builds decay factors in
torch), KV and DKV tensors instead of allocating them per call (lasp/lasp_cache.py:539-617).  Here
the decays are derived from the slopes inside the kernels, so `array` is accepted and ignored."""
import torch

from . import _abi
from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspCache", "lasp_cache_", "lasp_cache"]


def lasp_forward(q, k, v, s):
    """Launch shim with the signature of lasp/lasp_cache.py:427-465: (o, kv).

    o of the chunk with no incoming state, and the chunk's own state sum_j l^(n-j) k_j^T v_j in
    q.dtype (:438).  (The reference kernel adds its result to whatever the freshly allocated
    buffer holds, :104-106; the state is returned as computed here.)"""
    b, h, _, d = q.shape
    kv = torch.empty((b, h, d, v.shape[-1]), dtype=torch.float32, device=q.device)
    o, _, _ = _abi.chunk_fwd(q, k, v, s, kv_in=None, kv_out=kv)
    return o, kv.to(q.dtype)


def lasp_backward(q, k, v, s, do):
    """Launch shim with the signature of lasp/lasp_cache.py:468-536: (dq, dk, dv, None, dkv)."""
    b, h, _, d = q.shape
    dkv = torch.empty((b, h, d, v.shape[-1]), dtype=torch.float32, device=q.device)
    dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, dkv_out=dkv)
    return dq, dk, dv, None, dkv.to(q.dtype)


class LaspCache(torch.autograd.Function):
    """forward(q, k, v, s, array, KV, DKV) as lasp/lasp_cache.py:539-617.

    The reference receives into the caller's KV / DKV and then rebinds the name to a new tensor
    (`KV = block_decay * KV + kv`, :562; `DKV = ...`, :609), so after a call the caller's buffers hold
    the INCOMING states; the same here."""

    @staticmethod
    def forward(ctx, q, k, v, s, array, KV, DKV):
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, True, False, True)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:4] + (None, None, None)


lasp_cache_ = LaspCache.apply


def lasp_cache(q, k, v, ed, array, KV, DKV):
    if q.shape[-1] <= 128:
        return lasp_cache_(q, k, v, ed, array, KV, DKV)
    return run_sliced(q, k, v, ed, KV, DKV, True, False, True)
