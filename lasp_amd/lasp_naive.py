"""lasp_naive / lasp_cache: the two remaining public operators of the reference
(lasp/lasp_naive.py:541-648, lasp/lasp_cache.py:539-652).  Same mathematics as
lasp_fuse; the reference computes their incoming-state terms with torch matmuls and
(lasp_naive) allocates the KV / DKV buffers per call.  Here they run the same fused
kernels; lasp_naive owns its buffers, lasp_cache uses the caller's."""
import torch

from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspNaive", "lasp_naive_", "lasp_naive", "LaspCache", "lasp_cache_", "lasp_cache"]


def _state_buffers(q, v):
    b, h, _, d = q.shape
    e = v.shape[-1]
    KV = torch.zeros((b, h, d, e), dtype=torch.float32, device=q.device)
    return KV, torch.zeros_like(KV)


class LaspNaive(torch.autograd.Function):
    """forward(q, k, v, s) as lasp/lasp_naive.py:541-622."""

    @staticmethod
    def forward(ctx, q, k, v, s):
        KV, DKV = _state_buffers(q, v)
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, False, False)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:4]


lasp_naive_ = LaspNaive.apply


def lasp_naive(q, k, v, ed):
    if q.shape[-1] <= 128:
        return lasp_naive_(q, k, v, ed)
    KV, DKV = _state_buffers(q, v)
    return run_sliced(q, k, v, ed, KV, DKV, False, False)


class LaspCache(torch.autograd.Function):
    """forward(q, k, v, s, array, KV, DKV) as lasp/lasp_cache.py:539-617.

    `array` (positions 0..n-1, which the reference uses to build decay factors in
    torch) is accepted for signature compatibility; the kernels derive the decays
    from the slopes themselves.
    """

    @staticmethod
    def forward(ctx, q, k, v, s, array, KV, DKV):
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, False, False)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:4] + (None, None, None)


lasp_cache_ = LaspCache.apply


def lasp_cache(q, k, v, ed, array, KV, DKV):
    if q.shape[-1] <= 128:
        return lasp_cache_(q, k, v, ed, array, KV, DKV)
    return run_sliced(q, k, v, ed, KV, DKV, False, False)
