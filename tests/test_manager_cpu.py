"""Host logic: slopes, feature slicing, the loopback state mailbox, and the
torch.distributed (gloo, world size 2) path of the sequence-parallel manager."""
import os
import socket

import pytest
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

import lasp_amd
from lasp_amd import _chain
from lasp_amd.utils import seq_parallel_manager as spm
from oracle import lasp_oracle as O


@pytest.fixture(autouse=True)
def _clean():
    lasp_amd.destroy_parallel_groups()
    yield
    lasp_amd.destroy_parallel_groups()


@pytest.mark.parametrize("h", [1, 2, 3, 8, 12, 16, 20, 32, 40, 64])
def test_build_slope_tensor_matches_oracle(h):
    got = lasp_amd.build_slope_tensor(h)
    assert got.shape == (h, 1, 1) and got.dtype == torch.float32
    assert torch.allclose(got, O.slopes_alibi(h), rtol=1e-6, atol=0)


def test_feature_slices():
    assert _chain.feature_slices(64) == [(0, 64)]
    assert _chain.feature_slices(128) == [(0, 128)]
    assert _chain.feature_slices(192) == [(0, 128), (128, 192)]
    assert _chain.feature_slices(256) == [(0, 128), (128, 256)]


def test_loopback_chain_bookkeeping():
    lasp_amd.initialize_lasp(1, 4)
    assert lasp_amd.sequence_parallel_is_initialized()
    assert lasp_amd.get_sequence_parallel_world_size() == 4
    grp = lasp_amd.get_sequence_parallel_group()
    assert isinstance(grp, spm.LoopbackGroup)
    lasp_amd.set_sequence_parallel_rank(2)
    assert lasp_amd.get_sequence_parallel_rank() == 2
    assert lasp_amd.get_seq_parallel_send_rank() == 1       # previous chunk's owner
    assert lasp_amd.get_seq_parallel_receive_rank() == 3    # next chunk's owner
    lasp_amd.set_sequence_parallel_rank(0)
    assert lasp_amd.get_seq_parallel_send_rank() == 3       # wraps like the reference, never used by rank 0
    with pytest.raises(AssertionError):
        lasp_amd.initialize_lasp(1, 2)


def test_loopback_mailbox_send_recv():
    lasp_amd.initialize_lasp(1, 2)
    grp = lasp_amd.get_sequence_parallel_group()
    a = torch.arange(6.0).reshape(2, 3)
    lasp_amd.set_sequence_parallel_rank(0)
    spm.state_send(a, 1, grp)
    a.zero_()  # the mailbox holds a copy
    assert lasp_amd.loopback_pending() == [(0, 1)]
    lasp_amd.set_sequence_parallel_rank(1)
    out = torch.empty(2, 3)
    spm.state_recv(out, 0, grp)
    assert torch.equal(out, torch.arange(6.0).reshape(2, 3))
    assert lasp_amd.loopback_pending() == []
    with pytest.raises(RuntimeError, match="nothing was sent"):
        spm.state_recv(out, 0, grp)



def test_loopback_mailbox_is_first_in_first_out_per_pair_and_tag():
    lasp_amd.initialize_lasp(1, 2)
    grp = lasp_amd.get_sequence_parallel_group()
    lasp_amd.set_sequence_parallel_rank(0)
    first, second, tagged = torch.full((2,), 1.0), torch.full((2,), 2.0), torch.full((2,), 9.0)
    spm.state_send(first, 1, grp)
    spm.state_send(second, 1, grp)      # a second message to the same neighbour queues behind the first
    spm.state_send(tagged, 1, grp, tag=1)
    given = torch.full((2,), 5.0)
    spm.state_send(given, 1, grp, tag=2, give=True)
    assert lasp_amd.loopback_pending() == [(0, 1)]
    lasp_amd.set_sequence_parallel_rank(1)
    out = torch.empty(2)
    spm.state_recv(out, 0, grp, tag=1)
    assert torch.equal(out, tagged)
    assert torch.equal(spm.state_take(out, 0, grp), first)
    spm.state_recv(out, 0, grp)
    assert torch.equal(out, second)
    assert spm.state_take(out, 0, grp, tag=2).data_ptr() == given.data_ptr()   # handed over, not copied
    assert lasp_amd.loopback_pending() == []
    with pytest.raises(RuntimeError, match="nothing was sent"):
        spm.state_take(out, 0, grp)

def test_loopback_rejects_data_parallel():
    with pytest.raises(RuntimeError, match="sequence parallelism only"):
        lasp_amd.initialize_lasp(2, 2)


def _free_port():
    with socket.socket() as s_:
        s_.bind(("127.0.0.1", 0))
        return s_.getsockname()[1]


def _worker(rank, world, port, dp, sp, ret):
    os.environ["MASTER_ADDR"] = "127.0.0.1"
    os.environ["MASTER_PORT"] = str(port)
    dist.init_process_group("gloo", rank=rank, world_size=world)
    try:
        lasp_amd.initialize_lasp(dp, sp)
        info = dict(
            sp_rank=lasp_amd.get_sequence_parallel_rank(),
            sp_world=lasp_amd.get_sequence_parallel_world_size(),
            dp_rank=lasp_amd.get_data_parallel_rank(),
            dp_world=lasp_amd.get_data_parallel_world_size(),
            prev=lasp_amd.get_seq_parallel_send_rank(),
            next=lasp_amd.get_seq_parallel_receive_rank(),
            src=lasp_amd.get_sequence_parallel_src_rank(),
        )
        if sp == 2:  # pass a state down the chain and back (CPU tensors over gloo)
            grp = lasp_amd.get_sequence_parallel_group()
            t = torch.full((2, 2), float(rank + 1))
            if info["sp_rank"] == 0:
                spm.state_send(t, info["next"], grp)
                spm.state_recv(t, info["next"], grp)
            else:
                got = spm.state_take(torch.empty(2, 2), info["prev"], grp)  # a fresh tensor, received into
                spm.state_send(got * 10, info["prev"], grp)
            info["t"] = t.tolist()
        ret[rank] = info
    finally:
        dist.destroy_process_group()


@pytest.mark.parametrize("dp,sp", [(1, 2), (2, 1)])
def test_distributed_groups_gloo(dp, sp):
    world = 2
    ctx = mp.get_context("spawn")
    with ctx.Manager() as m:
        ret = m.dict()
        mp.spawn(_worker, args=(world, _free_port(), dp, sp, ret), nprocs=world, join=True)
        r = dict(ret)
    assert set(r) == {0, 1}
    if sp == 2:
        assert [r[i]["sp_rank"] for i in (0, 1)] == [0, 1]
        assert r[0]["sp_world"] == 2 and r[0]["dp_world"] == 1
        assert r[0]["next"] == 1 and r[1]["prev"] == 0 and r[1]["src"] == 0
        assert r[0]["t"] == [[10.0, 10.0], [10.0, 10.0]]  # rank 1 got 1s, sent back 10s
    else:
        assert [r[i]["sp_rank"] for i in (0, 1)] == [0, 0]
        assert [r[i]["dp_rank"] for i in (0, 1)] == [0, 1]
        assert r[0]["dp_world"] == 2 and r[0]["sp_world"] == 1
