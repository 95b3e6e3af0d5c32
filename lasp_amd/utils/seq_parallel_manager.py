"""Sequence/data-parallel bookkeeping for the lasp_* operators.

Counterpart of lasp/utils/seq_parallel_manager.py: the same public names, so the
autograd Functions and user code written against the reference keep working.

Two modes:

* ``torch.distributed`` initialised: ``initialize_lasp(dp, sp)`` builds strided
  data-parallel groups and contiguous sequence-parallel groups
  (lasp/utils/seq_parallel_manager.py:37-106) and state passing uses
  ``dist.send/recv``.

* not initialised (one process, one GPU): ``initialize_lasp(1, C)`` -- or just
  ``set_sequence_parallel_world_size(C)`` -- opens an in-process LOOPBACK: the
  caller plays ranks 0..C-1 in turn with ``set_sequence_parallel_rank(c)``, and the
  d x e states the Functions "send" are parked in a mailbox until the neighbouring
  rank "receives" them.  A receive from an empty mailbox raises instead of
  blocking, which is the failure a dead peer would otherwise turn into a hang.
"""
from __future__ import annotations

import operator
from collections import deque
from functools import reduce
from typing import Dict, Optional, Tuple

import torch
import torch.distributed as dist

__all__ = [
    "initialize_lasp", "is_unitialized", "sequence_parallel_is_initialized",
    "get_sequence_parallel_group", "get_data_parallel_group",
    "set_sequence_parallel_world_size", "get_sequence_parallel_world_size",
    "set_sequence_parallel_rank", "get_sequence_parallel_rank",
    "get_sequence_parallel_src_rank", "get_data_parallel_src_rank",
    "get_data_parallel_world_size", "get_data_parallel_rank",
    "get_seq_parallel_send_rank", "get_seq_parallel_receive_rank",
    "get_global_memory_buffer", "destroy_global_memory_buffer", "destroy_parallel_groups",
    "get_rank", "GlobalMemoryBuffer", "LoopbackGroup", "state_send", "state_recv", "state_take", "loopback_pending",
]


class LoopbackGroup:
    """Stands in for a process group when one process plays every SP rank."""

    def __init__(self, size: int):
        self.size = int(size)
        # (src, dst, tag) -> states in the order they were sent; an emptied queue is removed
        self.mailbox: Dict[Tuple[int, int, int], deque] = {}

    def __repr__(self):
        return f"LoopbackGroup(size={self.size}, pending={sorted(self.mailbox)})"


class _State:
    def __init__(self):
        self.reset()

    def reset(self):
        self.dp_group = None
        self.sp_group = None
        self.sp_world_override: Optional[int] = None
        self.sp_rank_override: Optional[int] = None
        self.dp_global_ranks = None
        self.buffer: Optional["GlobalMemoryBuffer"] = None


_st = _State()


def _distributed() -> bool:
    return dist.is_available() and dist.is_initialized()


def _loopback() -> LoopbackGroup:
    if not isinstance(_st.sp_group, LoopbackGroup):
        _st.sp_group = LoopbackGroup(_st.sp_world_override or 1)
        if _st.dp_group is None:
            _st.dp_group = LoopbackGroup(1)
    return _st.sp_group


def initialize_lasp(data_parallel_size: int = 1, sequence_parallel_size: int = 1) -> None:
    """Creates the DP and SP groups (or the loopback when torch.distributed is down)."""
    if _st.dp_group is not None or _st.sp_group is not None:
        raise AssertionError("parallel groups are already initialized")
    if not _distributed():
        if data_parallel_size != 1:
            raise RuntimeError("the in-process loopback emulates sequence parallelism only (data_parallel_size must be 1)")
        _st.sp_group = LoopbackGroup(sequence_parallel_size)
        _st.dp_group = LoopbackGroup(1)
        _st.sp_world_override = sequence_parallel_size
        if _st.sp_rank_override is None:
            _st.sp_rank_override = 0
        _st.buffer = GlobalMemoryBuffer()
        return

    world = dist.get_world_size()
    me = dist.get_rank()
    sp, dp = int(sequence_parallel_size), int(data_parallel_size)
    if sp > 1 and world % sp != 0:
        raise RuntimeError(f"world_size ({world}) is not divisible by sequence_parallel_size {sp})")
    # data-parallel groups: ranks with the same position inside their SP group
    for offset in range(sp):
        members = list(range(offset, world, sp))
        grp = dist.new_group(members)
        if me in members:
            _st.dp_group = grp
            _st.dp_global_ranks = members
    # sequence-parallel groups: contiguous runs of sp ranks
    for first in range(0, dp * sp, sp):
        members = list(range(first, first + sp))
        grp = dist.new_group(members)
        if me in members:
            _st.sp_group = grp
    _st.buffer = GlobalMemoryBuffer()


def is_unitialized():
    return _st.dp_group is None


def sequence_parallel_is_initialized():
    return _st.sp_group is not None and _st.dp_group is not None


def get_sequence_parallel_group():
    if _st.sp_group is None and not _distributed():
        return _loopback()
    assert _st.sp_group is not None, "sequence parallel group is not initialized"
    return _st.sp_group


def get_data_parallel_group(with_sequence_parallel=False):
    assert _st.dp_group is not None, "data parallel group is not initialized"
    return _st.dp_group


def set_sequence_parallel_world_size(world_size):
    _st.sp_world_override = world_size
    if isinstance(_st.sp_group, LoopbackGroup) and world_size is not None:
        _st.sp_group.size = int(world_size)


def get_sequence_parallel_world_size():
    if _st.sp_world_override is not None:
        return _st.sp_world_override
    grp = get_sequence_parallel_group()
    if isinstance(grp, LoopbackGroup):
        return grp.size
    return dist.get_world_size(group=grp)


def set_sequence_parallel_rank(rank):
    _st.sp_rank_override = rank


def get_sequence_parallel_rank():
    if _st.sp_rank_override is not None:
        return _st.sp_rank_override
    grp = get_sequence_parallel_group()
    if isinstance(grp, LoopbackGroup):
        return 0
    return dist.get_rank(group=grp)


def _global_rank_and_world():
    if _distributed():
        return dist.get_rank(), dist.get_world_size()
    return get_sequence_parallel_rank(), get_sequence_parallel_world_size()


def get_seq_parallel_send_rank():
    """Global rank of the previous chunk's owner (lasp/utils/seq_parallel_manager.py:25-28)."""
    rank, world = _global_rank_and_world()
    return (rank - 1 + world) % world


def get_seq_parallel_receive_rank():
    """Global rank of the next chunk's owner (lasp/utils/seq_parallel_manager.py:31-34)."""
    rank, world = _global_rank_and_world()
    return (rank + 1 + world) % world


def get_sequence_parallel_src_rank():
    rank, _ = _global_rank_and_world()
    size = get_sequence_parallel_world_size()
    return (rank // size) * size


def get_data_parallel_src_rank():
    assert _st.dp_global_ranks is not None, "Data parallel group is not initialized"
    return _st.dp_global_ranks[0]


def get_data_parallel_world_size(with_sequence_parallel=False):
    grp = get_data_parallel_group()
    return grp.size if isinstance(grp, LoopbackGroup) else dist.get_world_size(group=grp)


def get_data_parallel_rank(with_sequence_parallel=False):
    grp = get_data_parallel_group()
    return 0 if isinstance(grp, LoopbackGroup) else dist.get_rank(group=grp)


def get_rank(group):
    if isinstance(group, LoopbackGroup):
        return get_sequence_parallel_rank()
    return dist.get_rank(group=group)


# ---------------------------------------------------------------- state passing
# The loopback mailbox is first-in first-out per (sender, receiver, tag), as dist.send / dist.recv
# are per pair of ranks: an operator on wide heads sends one state per feature slice to the same
# neighbour before that neighbour receives any of them.  `tag` (the feature-slice index) only
# exists in the loopback; over torch.distributed the order of the calls pairs the messages.
def state_send(tensor: torch.Tensor, dst: int, group, src: Optional[int] = None, tag: int = 0,
               give: bool = False) -> None:
    """Hands a d x e state to rank `dst` (dist.send, or the loopback mailbox).

    The mailbox keeps a copy, unless the sender gives the tensor away (`give`: it will not touch
    it again)."""
    if isinstance(group, LoopbackGroup):
        me = get_sequence_parallel_rank() if src is None else src
        t = tensor.detach()
        group.mailbox.setdefault((me, dst, tag), deque()).append(t if give else t.clone())
        return
    if _stage_through_host(tensor, group):
        dist.send(tensor.detach().cpu(), dst=dst, group=group)  # .cpu() waits for the producing kernels
        return
    dist.send(tensor, dst=dst, group=group)


def _stage_through_host(tensor: torch.Tensor, group) -> bool:
    """Device tensors only go to backends that move device memory themselves (nccl, i.e. RCCL).
    Over gloo a state is copied to host memory first and back after: gloo's own handling of device
    tensors can stall when several ranks share one GPU."""
    return tensor.is_cuda and dist.get_backend(group) == "gloo"


def _recv_into(tensor: torch.Tensor, src: int, group) -> None:
    if _stage_through_host(tensor, group):
        host = torch.empty(tensor.shape, dtype=tensor.dtype)
        dist.recv(host, src=src, group=group)
        tensor.copy_(host)
        return
    dist.recv(tensor, src=src, group=group)


def _loopback_pop(group: LoopbackGroup, src: int, me: int, tag: int) -> torch.Tensor:
    key = (src, me, tag)
    queue = group.mailbox.get(key)
    if not queue:
        raise RuntimeError(
            f"loopback recv on rank {me}: nothing was sent by rank {src} "
            f"(pending: {loopback_pending()}); chunks must run in chain order"
        )
    t = queue.popleft()
    if not queue:
        del group.mailbox[key]
    return t


def state_recv(tensor: torch.Tensor, src: int, group, dst: Optional[int] = None, tag: int = 0) -> None:
    """Fills `tensor` with the state rank `src` sent (dist.recv, or the mailbox)."""
    if isinstance(group, LoopbackGroup):
        me = get_sequence_parallel_rank() if dst is None else dst
        tensor.copy_(_loopback_pop(group, src, me, tag))
        return
    _recv_into(tensor, src, group)


def state_take(like: torch.Tensor, src: int, group, dst: Optional[int] = None, tag: int = 0) -> torch.Tensor:
    """The state rank `src` sent, as a tensor the caller owns (shaped like `like`).

    In the loopback the parked copy itself changes hands, so a chunk's incoming state costs no
    device copy beyond the one made when it was sent; over torch.distributed it is received into
    a fresh buffer.  Either way the result can be kept for backward while `like` (the caller's KV
    or DKV buffer) is overwritten with the outgoing state.
    """
    if isinstance(group, LoopbackGroup):
        me = get_sequence_parallel_rank() if dst is None else dst
        return _loopback_pop(group, src, me, tag)
    t = torch.empty_like(like)
    _recv_into(t, src, group)
    return t


def loopback_pending():
    """(src, dst) pairs with states sent but not yet received (loopback mode only)."""
    grp = _st.sp_group
    if not isinstance(grp, LoopbackGroup):
        return []
    return sorted({(src, dst) for (src, dst, _tag), q in grp.mailbox.items() if q})


# ---------------------------------------------------------------- memory buffer
class GlobalMemoryBuffer:
    """Named, growing scratch tensors (lasp/utils/seq_parallel_manager.py:235-256)."""

    def __init__(self):
        self.buffer = {}

    def get_tensor(self, tensor_shape, dtype, name):
        need = reduce(operator.mul, tensor_shape, 1)
        cur = self.buffer.get((name, dtype))
        if cur is None or cur.numel() < need:
            cur = torch.empty(need, dtype=dtype, device=torch.cuda.current_device(), requires_grad=False)
            self.buffer[(name, dtype)] = cur
        return cur[:need].view(*tensor_shape)


def get_global_memory_buffer():
    assert _st.buffer is not None, "global memory buffer is not initialized"
    return _st.buffer


def destroy_global_memory_buffer():
    _st.buffer = None


def destroy_parallel_groups():
    """Forgets groups, overrides and any parked loopback states."""
    _st.reset()
