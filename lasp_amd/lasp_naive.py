"""lasp_naive: the chunk operator that owns its KV / DKV buffers (lasp/lasp_naive.py).

Same mathematics as lasp_fuse.  The reference runs Triton kernels for the chunk alone and adds the
incoming-state terms with torch matmuls (lasp/lasp_naive.py:560-565,604-614); here the operator
runs the fused kernels, and the module-level launch shims keep the reference's split: they compute
the chunk WITHOUT incoming state and hand back the chunk's own state contribution."""
import torch

from . import _abi
from ._chain import ChunkFunction, run_sliced

__all__ = ["LaspNaive", "lasp_naive_", "lasp_naive"]


def lasp_forward(q, k, v, s, kv):
    """Launch shim with the signature of lasp/lasp_naive.py:429-467.

    Returns o of the chunk with no incoming state and fills `kv`, (b, h, d, e) in any float
    dtype (the reference allocates it in q.dtype, :563), with the chunk's own state
    sum_j l^(n-j) k_j^T v_j, which the caller combines as KV <- l^n KV + kv (:565)."""
    kv32 = kv if kv.dtype == torch.float32 and kv.is_contiguous() else torch.empty(kv.shape, dtype=torch.float32,
                                                                                   device=kv.device)
    o, _, _ = _abi.chunk_fwd(q, k, v, s, kv_in=None, kv_out=kv32)
    if kv32 is not kv:
        kv.copy_(kv32)
    return o


def lasp_backward(q, k, v, s, do):
    """Launch shim with the signature of lasp/lasp_naive.py:470-538: (dq, dk, dv, None, dkv).

    Gradients of the chunk with no incoming KV / DKV, and dkv = sum_i l^i q_i^T do_i in q.dtype
    (:489), which the caller combines as DKV <- l^n DKV + dkv (:614)."""
    b, h, _, d = q.shape
    dkv = torch.empty((b, h, d, v.shape[-1]), dtype=torch.float32, device=q.device)
    dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, dkv_out=dkv)
    return dq, dk, dv, None, dkv.to(q.dtype)


def _state_buffers(q, v):
    b, h, _, d = q.shape
    e = v.shape[-1]
    KV = torch.empty((b, h, d, e), dtype=torch.float32, device=q.device)
    return KV, torch.empty_like(KV)


class LaspNaive(torch.autograd.Function):
    """forward(q, k, v, s) as lasp/lasp_naive.py:541-622."""

    @staticmethod
    def forward(ctx, q, k, v, s):
        KV, DKV = _state_buffers(q, v)
        return ChunkFunction.forward(ctx, q, k, v, s, KV, DKV, True, False)

    @staticmethod
    def backward(ctx, do):
        return ChunkFunction.backward(ctx, do)[:4]


lasp_naive_ = LaspNaive.apply


def lasp_naive(q, k, v, ed):
    if q.shape[-1] <= 128:
        return lasp_naive_(q, k, v, ed)
    KV, DKV = _state_buffers(q, v)
    return run_sliced(q, k, v, ed, KV, DKV, True, False)
