"""Host logic of the operators without a GPU: the autograd Functions, the loopback state
passing and the feature-slicing wrapper run here on CPU tensors with the two library calls
(`_abi.chunk_fwd`, `_abi.chunk_bwd`) replaced by the oracle.  What is under test is the
choreography around the calls -- zeroing KV, receive / clone / run / send, the reversed DKV
chain, in-place state updates, slicing wide heads -- not the kernels."""
import pytest
import torch

import lasp_amd
from lasp_amd import _abi
from oracle import lasp_oracle as O


def _fake_fwd(q, k, v, s, kv_in=None, kv_out=None, seg_len=0):
    o, kvo = O.ref_chunked_fwd(q, k, v, s, kv_in, 64, torch.float64)
    if kv_out is not None:
        kv_out.copy_(kvo.to(kv_out.dtype))
    states = torch.zeros(1)  # stands for the segment-state cache
    return o.to(q.dtype), states, 64


def _fake_bwd(q, k, v, s, do, kv_in=None, dkv_in=None, dkv_out=None, kv_seg_states=None, seg_len=0):
    dq, dk, dv, dkvo = O.ref_chunked_bwd(q, k, v, s, do, kv_in, dkv_in, 64, torch.float64)
    if dkv_out is not None:
        dkv_out.copy_(dkvo.to(dkv_out.dtype))
    return dq.to(q.dtype), dk.to(q.dtype), dv.to(q.dtype)


@pytest.fixture(autouse=True)
def _oracle_behind_the_abi(monkeypatch):
    monkeypatch.setattr(_abi, "chunk_fwd", _fake_fwd)
    monkeypatch.setattr(_abi, "chunk_bwd", _fake_bwd)
    lasp_amd.destroy_parallel_groups()
    yield
    lasp_amd.destroy_parallel_groups()


def _inputs(b, h, n, d, e, seed):
    g = torch.Generator().manual_seed(seed)
    q, k = [torch.randn(b, h, n, d, generator=g, dtype=torch.float64) for _ in range(2)]
    v, do = [torch.randn(b, h, n, e, generator=g, dtype=torch.float64) for _ in range(2)]
    return q, k, v, do


def _chain(op_name, q, k, v, do, s, chunks):
    op = getattr(lasp_amd, op_name)
    b, h, n, d = q.shape
    e = v.shape[-1]
    step = n // chunks
    lasp_amd.initialize_lasp(1, chunks)
    KV = torch.full((b, h, d, e), 7.0, dtype=torch.float64)   # garbage on entry: the operator never reads it
    DKV = torch.full((b, h, d, e), -3.0, dtype=torch.float64)
    outs, leaves, kv_after = [], [], []
    for c in range(chunks):
        lasp_amd.set_sequence_parallel_rank(c)
        sl = slice(c * step, (c + 1) * step)
        qc, kc, vc = [t[:, :, sl].clone().requires_grad_(True) for t in (q, k, v)]
        if op_name == "lasp_naive":
            o = op(qc, kc, vc, s)
        elif op_name == "lasp_cache":
            o = op(qc, kc, vc, s, torch.arange(step), KV, DKV)
        else:
            o = op(qc, kc, vc, s, KV, DKV)
        outs.append(o)
        leaves.append((qc, kc, vc))
        kv_after.append(KV.clone())
    dkv_after = [None] * chunks
    for c in reversed(range(chunks)):
        outs[c].backward(do[:, :, c * step:(c + 1) * step])
        dkv_after[c] = DKV.clone()
    assert lasp_amd.loopback_pending() == []
    cat = lambda i: torch.cat([l[i].grad for l in leaves], 2)
    return torch.cat([o.detach() for o in outs], 2), cat(0), cat(1), cat(2), kv_after, dkv_after


@pytest.mark.parametrize("op_name", ["lasp_fuse", "lasp_fuse_parallel", "lasp_cache", "lasp_naive"])
def test_chain_choreography_equals_single_pass(op_name):
    q, k, v, do = _inputs(2, 3, 256, 16, 8, seed=1)
    s = O.slopes_alibi(3)
    ref = O.ref_chunked(q, k, v, s, do, dtype=torch.float64)
    o, dq, dk, dv, kv_after, dkv_after = _chain(op_name, q, k, v, do, s, chunks=4)
    tol = 1e-6 if op_name == "lasp_naive" else 1e-12  # lasp_naive allocates its own float32 state buffers
    for got, name in ((o, "o"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert O.rel_err(got, ref[name]) < tol, (op_name, name)
    _, kv1 = O.ref_chunked_fwd(q[:, :, :64], k[:, :, :64], v[:, :, :64], s, None, 64, torch.float64)
    _, kv3 = O.ref_chunked_fwd(q[:, :, :192], k[:, :, :192], v[:, :, :192], s, None, 64, torch.float64)
    if op_name == "lasp_fuse":
        # the caller's KV holds KV_out of the chunk just run; after the last chunk, of the whole sequence
        # (in-place update, lasp/lasp_fuse.py:126-127)
        assert O.rel_err(kv_after[-1], ref["kv_out"]) < 1e-12
        assert O.rel_err(kv_after[0], kv1) < 1e-12
        # after the reversed chain the caller's DKV holds dL/dKV_in of the first chunk
        assert O.rel_err(dkv_after[0], ref["dkv_out"]) < 1e-12
    elif op_name in ("lasp_fuse_parallel", "lasp_cache"):
        # the caller's buffers are left holding the INCOMING states (lasp/lasp_fuse_parallel.py:1091-1101,
        # lasp/lasp_cache.py:549-562,597-609: KV is zeroed, received into, and the outgoing state is bound
        # to a new tensor)
        assert torch.count_nonzero(kv_after[0]) == 0
        assert O.rel_err(kv_after[1], kv1) < 1e-12
        assert O.rel_err(kv_after[-1], kv3) < 1e-12
        assert torch.count_nonzero(dkv_after[-1]) == 0
        # DKV entering chunk 0 = dL/dKV_out of chunk 0 = DKV_out of the chain over chunks 1..3
        tail = O.ref_chunked(q[:, :, 64:], k[:, :, 64:], v[:, :, 64:], s, do[:, :, 64:], kv1, None,
                             dtype=torch.float64)
        assert O.rel_err(dkv_after[0], tail["dkv_out"]) < 1e-12


@pytest.mark.parametrize("d", [192, 256])
@pytest.mark.parametrize("op_name", ["lasp_fuse", "lasp_fuse_parallel", "lasp_cache", "lasp_naive"])
def test_wide_heads_through_a_two_chunk_chain(op_name, d):
    """d > 128 runs one chunk call per 128-wide feature slice, and every slice sends its own state to
    the same neighbour: the loopback has to deliver them first-in first-out per slice."""
    q, k, v, do = _inputs(1, 2, 128, d, 8, seed=7)
    s = O.slopes_alibi(2)
    ref = O.ref_chunked(q, k, v, s, do, dtype=torch.float64)
    o, dq, dk, dv, _, _ = _chain(op_name, q, k, v, do, s, chunks=2)
    tol = 1e-6 if op_name == "lasp_naive" else 1e-12
    for got, name in ((o, "o"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert O.rel_err(got, ref[name]) < tol, (op_name, d, name)


def test_lightning_attn_and_wide_heads_are_sliced_and_summed():
    # d = 320 -> feature slices [0,128) [128,256) [256,320): three calls whose outputs add up
    q, k, v, do = _inputs(1, 2, 128, 320, 8, seed=2)
    s = O.slopes_alibi(2)
    ref = O.ref_chunked(q, k, v, s, do, dtype=torch.float64)
    qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
    o = lasp_amd.lightning_attn(qg, kg, vg, s)
    o.backward(do)
    assert O.rel_err(o, ref["o"]) < 1e-12
    assert O.rel_err(qg.grad, ref["dq"]) < 1e-12
    assert O.rel_err(kg.grad, ref["dk"]) < 1e-12
    assert O.rel_err(vg.grad, ref["dv"]) < 1e-12


def test_wide_heads_with_state_copy_back():
    q, k, v, do = _inputs(1, 2, 128, 192, 8, seed=3)
    s = O.slopes_alibi(2)
    lasp_amd.initialize_lasp(1, 1)
    KV = torch.empty(1, 2, 192, 8, dtype=torch.float64)
    DKV = torch.empty_like(KV)
    o = lasp_amd.lasp_fuse(q, k, v, s, KV, DKV)
    ref_o, ref_kv = O.ref_chunked_fwd(q, k, v, s, None, 64, torch.float64)
    assert O.rel_err(o, ref_o) < 1e-12
    assert O.rel_err(KV, ref_kv) < 1e-12  # every feature slice of the state was written back


def test_no_gradient_for_states_and_slopes():
    q, k, v, do = _inputs(1, 2, 64, 8, 8, seed=4)
    s = O.slopes_alibi(2).requires_grad_(True)
    lasp_amd.initialize_lasp(1, 1)
    KV = torch.zeros(1, 2, 8, 8, dtype=torch.float64)
    DKV = torch.zeros_like(KV)
    qg = q.clone().requires_grad_(True)
    o = lasp_amd.lasp_fuse(qg, k, v, s, KV, DKV)
    o.backward(do)
    assert qg.grad is not None and s.grad is None


def test_launch_shims_keep_the_reference_signatures_and_aliasing():
    """lasp_fuse.lasp_forward / lasp_backward update KV / DKV in place; the lasp_fuse_parallel
    pair returns new state tensors and leaves the caller's buffers alone
    (lasp/lasp_fuse.py:356-475, lasp/lasp_fuse_parallel.py:833-1070)."""
    import importlib

    # the package attributes of these names are the operators (as in the reference), so go through sys.modules
    LF = importlib.import_module("lasp_amd.lasp_fuse")
    LP = importlib.import_module("lasp_amd.lasp_fuse_parallel")

    q, k, v, do = _inputs(1, 2, 128, 16, 8, seed=5)
    s = O.slopes_alibi(2)
    g = torch.Generator().manual_seed(6)
    kv0 = torch.randn(1, 2, 16, 8, generator=g, dtype=torch.float64)
    dkv0 = torch.randn(1, 2, 16, 8, generator=g, dtype=torch.float64)
    ref = O.ref_chunked(q, k, v, s, do, kv0, dkv0, dtype=torch.float64)

    KV, DKV = kv0.clone(), dkv0.clone()
    o = LF.lasp_forward(q, k, v, s, KV)
    assert O.rel_err(o, ref["o"]) < 1e-12 and O.rel_err(KV, ref["kv_out"]) < 1e-12
    dq, dk, dv = LF.lasp_backward(q, k, v, s, do, kv0, DKV)
    assert max(O.rel_err(dq, ref["dq"]), O.rel_err(dk, ref["dk"]), O.rel_err(dv, ref["dv"])) < 1e-12
    assert O.rel_err(DKV, ref["dkv_out"]) < 1e-12

    KV, DKV = kv0.clone(), dkv0.clone()
    o, cache, KV_out = LP.lasp_forward(q, k, v, s, KV, 128, 64)
    assert torch.equal(KV, kv0) and O.rel_err(KV_out, ref["kv_out"]) < 1e-12 and O.rel_err(o, ref["o"]) < 1e-12
    dq, dk, dv, DKV_out = LP.lasp_backward(q, k, v, s, do, cache, kv0, DKV, 128, 64)
    assert torch.equal(DKV, dkv0) and O.rel_err(DKV_out, ref["dkv_out"]) < 1e-12
    assert max(O.rel_err(dq, ref["dq"]), O.rel_err(dk, ref["dk"]), O.rel_err(dv, ref["dv"])) < 1e-12


def test_lasp_cache_module_path():
    from lasp_amd.lasp_cache import LaspCache, lasp_cache  # noqa: F401

    assert lasp_cache is lasp_amd.lasp_cache and callable(lasp_amd.lasp_cache)
