"""Shared machinery of the lasp_* operators: one autograd Function that runs a chunk
through the C ABI and passes the d x e state along the sequence-parallel chain.

Choreography (forward: rank r-1 -> r -> r+1, backward reversed) follows
lasp/lasp_fuse.py:478-532 and lasp/lasp_fuse_parallel.py:1073-1137:
zero the caller's KV buffer, receive the incoming state unless first in the chain,
keep a copy of it for backward, run the chunk (which overwrites KV with the
outgoing state), send it on unless last; backward mirrors this with DKV.
KV and DKV receive no gradient.
"""
from __future__ import annotations

import torch

from . import _abi
from .utils import seq_parallel_manager as spm


def feature_slices(d: int):
    """Column ranges the public wrappers cut q and k into.

    One kernel launch takes d <= 128, so wider heads are processed as 128-wide
    slices whose outputs add up (Q K^T is a sum over feature slices), as
    lasp/lightning_attention.py:513-529 does.
    """
    width = 128
    return [(lo, min(lo + width, d)) for lo in range(0, d, width)]


class ChunkFunction(torch.autograd.Function):
    """forward(q, k, v, s, KV, DKV, cache_states, barrier) -> o

    KV / DKV: caller-owned float32 (b, h, d, e) buffers, or None for the stateless
    single-device operator (then nothing is sent or received).
    cache_states: keep the per-segment incoming states for backward (the
    lasp_fuse_parallel trade, lasp/lasp_fuse_parallel.py:1103) instead of
    recomputing them (lasp_fuse, whose backward re-runs the kv recurrence,
    lasp/lasp_fuse.py:237-260).
    """

    @staticmethod
    def forward(ctx, q, k, v, s, KV, DKV, cache_states, barrier):
        chained = KV is not None
        ctx.chained = chained
        if not chained:
            o, states, seg_len = _abi.chunk_fwd(q, k, v, s)
            ctx.save_for_backward(q, k, v, s, states if cache_states else None)
            ctx.seg_len = seg_len
            return o

        KV.zero_()
        group = spm.get_sequence_parallel_group()
        rank = spm.get_sequence_parallel_rank()
        world = spm.get_sequence_parallel_world_size()
        prev_rank = spm.get_seq_parallel_send_rank()
        next_rank = spm.get_seq_parallel_receive_rank()
        if barrier and not isinstance(group, spm.LoopbackGroup):
            torch.distributed.barrier()
        if rank > 0:
            spm.state_recv(KV, prev_rank, group)
        kv_in = KV.clone()
        o, states, seg_len = _abi.chunk_fwd(q, k, v, s, kv_in=kv_in, kv_out=KV)
        # DKV is a scratch buffer that later backward calls overwrite in place, so it is
        # kept by reference rather than as a version-checked saved tensor.
        ctx.save_for_backward(q, k, v, s, states if cache_states else None, kv_in)
        ctx.dkv_buffer = DKV
        ctx.seg_len = seg_len
        if rank < world - 1:
            spm.state_send(KV, next_rank, group)
        ctx.group, ctx.rank, ctx.world = group, rank, world
        ctx.prev_rank, ctx.next_rank = prev_rank, next_rank
        return o

    @staticmethod
    def backward(ctx, do):
        if not ctx.chained:
            q, k, v, s, states = ctx.saved_tensors
            dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, kv_seg_states=states, seg_len=ctx.seg_len)
            return dq, dk, dv, None, None, None, None, None

        q, k, v, s, states, kv_in = ctx.saved_tensors
        DKV = ctx.dkv_buffer
        DKV.zero_()
        if ctx.rank < ctx.world - 1:
            spm.state_recv(DKV, ctx.next_rank, ctx.group, dst=ctx.rank)
        dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, kv_in=kv_in, dkv_in=DKV, dkv_out=DKV,
                                    kv_seg_states=states, seg_len=ctx.seg_len)
        if ctx.rank > 0:
            spm.state_send(DKV, ctx.prev_rank, ctx.group, src=ctx.rank)
        return dq, dk, dv, None, None, None, None, None


def run_sliced(q, k, v, ed, KV, DKV, cache_states, barrier):
    """Applies ChunkFunction per feature slice of q/k and adds the outputs."""
    d = q.shape[-1]
    parts = feature_slices(d)
    if len(parts) == 1:
        return ChunkFunction.apply(q, k, v, ed, KV, DKV, cache_states, barrier)
    out = None
    for lo, hi in parts:
        q1, k1 = q[..., lo:hi], k[..., lo:hi]
        if KV is None:
            o = ChunkFunction.apply(q1, k1, v, ed, None, None, cache_states, barrier)
        else:
            kv1 = KV[:, :, lo:hi].contiguous()
            dkv1 = DKV[:, :, lo:hi].contiguous()
            o = ChunkFunction.apply(q1, k1, v, ed, kv1, dkv1, cache_states, barrier)
            KV[:, :, lo:hi].copy_(kv1)
        out = o if out is None else out + o
    return out
