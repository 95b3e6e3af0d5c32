"""Shared machinery of the lasp_* operators: one autograd Function that runs a chunk
through the C ABI and passes the d x e state along the sequence-parallel chain.

Choreography (forward: rank r-1 -> r -> r+1, backward reversed) follows
lasp/lasp_fuse.py:478-532 and lasp/lasp_fuse_parallel.py:1073-1137: receive the
incoming state unless first in the chain, keep it for backward, run the chunk
(which leaves the outgoing state in the caller's KV buffer), send that on unless
last; backward mirrors this with DKV.  KV and DKV receive no gradient.

The reference zeroes KV, receives into it and clones it (lasp/lasp_fuse.py:485-496).
Here the received state lands in a tensor of its own (`state_take`), which is both the
kernel's input and the copy kept for backward, and the first rank passes "no incoming
state" instead of a zeroed buffer: the caller's KV is only ever written, with KV_out,
so what it holds on entry does not matter and no zero / copy / clone kernels run per chunk.
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
    """forward(q, k, v, s, KV, DKV, cache_states, barrier, rebind=False, tag=0) -> o

    KV / DKV: caller-owned float32 (b, h, d, e) buffers, or None for the stateless
    single-device operator (then nothing is sent or received).
    cache_states: keep the per-segment incoming states for backward (the
    lasp_fuse_parallel trade, lasp/lasp_fuse_parallel.py:1103) instead of
    recomputing them (lasp_fuse, whose backward re-runs the kv recurrence,
    lasp/lasp_fuse.py:237-260).
    rebind: the outgoing state goes to a new tensor and the caller's KV / DKV buffer is left
    holding the INCOMING state, which is what lasp_fuse_parallel's `KV = ...` rebinding does
    (lasp/lasp_fuse_parallel.py:941-942,1099-1106); otherwise the buffer receives the outgoing
    state in place (lasp/lasp_fuse.py:126-127,352-353).
    tag: feature-slice index, keeps the loopback messages of different slices apart.
    """

    @staticmethod
    def forward(ctx, q, k, v, s, KV, DKV, cache_states, barrier, rebind=False, tag=0):
        chained = KV is not None
        ctx.chained = chained
        if not chained:
            o, states, seg_len = _abi.chunk_fwd(q, k, v, s)
            ctx.save_for_backward(q, k, v, s, states if cache_states else None)
            ctx.seg_len = seg_len
            return o

        group = spm.get_sequence_parallel_group()
        rank = spm.get_sequence_parallel_rank()
        world = spm.get_sequence_parallel_world_size()
        prev_rank = spm.get_seq_parallel_send_rank()
        next_rank = spm.get_seq_parallel_receive_rank()
        if barrier and not isinstance(group, spm.LoopbackGroup):
            torch.distributed.barrier()
        kv_in = spm.state_take(KV, prev_rank, group, tag=tag) if rank > 0 else None
        kv_out = KV
        if rebind:  # the caller's buffer is left holding the incoming state
            if kv_in is None:
                KV.zero_()
            else:
                KV.copy_(kv_in)
            kv_out = torch.empty_like(KV) if rank < world - 1 else None  # the last rank's KV_out goes nowhere
        o, states, seg_len = _abi.chunk_fwd(q, k, v, s, kv_in=kv_in, kv_out=kv_out)
        # DKV is a scratch buffer that later backward calls overwrite in place, so it is
        # kept by reference rather than as a version-checked saved tensor.
        ctx.save_for_backward(q, k, v, s, states if cache_states else None, kv_in)
        ctx.dkv_buffer = DKV
        ctx.seg_len = seg_len
        if rank < world - 1:
            spm.state_send(kv_out, next_rank, group, tag=tag, give=rebind)
        ctx.group, ctx.rank, ctx.world, ctx.tag, ctx.rebind = group, rank, world, tag, rebind
        ctx.prev_rank, ctx.next_rank = prev_rank, next_rank
        return o

    @staticmethod
    def backward(ctx, do):
        none = (None,) * 7
        if not ctx.chained:
            q, k, v, s, states = ctx.saved_tensors
            dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, kv_seg_states=states, seg_len=ctx.seg_len)
            return (dq, dk, dv) + none

        q, k, v, s, states, kv_in = ctx.saved_tensors
        DKV = ctx.dkv_buffer
        dkv_in = None
        if ctx.rank < ctx.world - 1:
            dkv_in = spm.state_take(DKV, ctx.next_rank, ctx.group, dst=ctx.rank, tag=ctx.tag)
        dkv_out = DKV
        if ctx.rebind:
            if dkv_in is None:
                DKV.zero_()
            else:
                DKV.copy_(dkv_in)
            dkv_out = torch.empty_like(DKV) if ctx.rank > 0 else None
        dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, kv_in=kv_in, dkv_in=dkv_in, dkv_out=dkv_out,
                                    kv_seg_states=states, seg_len=ctx.seg_len)
        if ctx.rank > 0:
            spm.state_send(dkv_out, ctx.prev_rank, ctx.group, src=ctx.rank, tag=ctx.tag, give=ctx.rebind)
        return (dq, dk, dv) + none


def run_sliced(q, k, v, ed, KV, DKV, cache_states, barrier, rebind=False):
    """Applies ChunkFunction per feature slice of q/k and adds the outputs."""
    d = q.shape[-1]
    parts = feature_slices(d)
    if len(parts) == 1:
        return ChunkFunction.apply(q, k, v, ed, KV, DKV, cache_states, barrier, rebind, 0)
    out = None
    for tag, (lo, hi) in enumerate(parts):
        q1, k1 = q[..., lo:hi], k[..., lo:hi]
        if KV is None:
            o = ChunkFunction.apply(q1, k1, v, ed, None, None, cache_states, barrier, rebind, tag)
        else:
            kv1 = KV[:, :, lo:hi].contiguous()
            dkv1 = DKV[:, :, lo:hi].contiguous()
            o = ChunkFunction.apply(q1, k1, v, ed, kv1, dkv1, cache_states, barrier, rebind, tag)
            KV[:, :, lo:hi].copy_(kv1)
        out = o if out is None else out + o
    return out
