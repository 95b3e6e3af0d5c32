"""The large benchmark configurations (2: TNL-1B head shape, 3: TNL-7B chunk, 4: 1M tokens) at full size.

Where the fp64/fp32 oracle on every head would take too long on the host, the
oracle is run on a subset of heads (stated per test) and the rest is covered by
size-independent properties: chunk chain == single pass, linearity in V, and
per-head independence."""
import pytest
import torch

from oracle import lasp_oracle as O

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _rel(x, ref):
    """Worst (batch, head) slice of max|x - ref| / max|ref|, evaluated on the device (full-size tensors)."""
    x, ref = x.float(), ref.float()
    if x.dim() == 3:  # one head of a (b, h, n, f) tensor
        x, ref = x[:, None], ref[:, None]
    err = (x - ref).abs().amax(dim=(2, 3))
    return (err / ref.abs().amax(dim=(2, 3)).clamp_min(1e-30)).max().item()


def _randn(shape, dev, seed, scale):
    g = torch.Generator(device=dev).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=dev) * scale).to(torch.bfloat16)


def _fwd_bwd(q, k, v, do, s, kv=None, dkv=None, seg_len=0, cache=True):
    from lasp_amd import _abi

    kv_out = torch.empty_like(kv) if kv is not None else None
    dkv_out = torch.empty_like(dkv) if dkv is not None else None
    o, states, sl = _abi.chunk_fwd(q, k, v, s, kv_in=kv, kv_out=kv_out, seg_len=seg_len)
    dq, dk, dv = _abi.chunk_bwd(q, k, v, s, do, kv_in=kv, dkv_in=dkv, dkv_out=dkv_out,
                                kv_seg_states=states if cache else None, seg_len=sl)
    return dict(o=o, dq=dq, dk=dk, dv=dv, kv_out=kv_out, dkv_out=dkv_out)


def _oracle_heads(q, k, v, do, s, heads, kv=None, dkv=None):
    idx = torch.tensor(heads)
    c = lambda t: None if t is None else t[:, heads].cpu()
    return O.ref_chunked(c(q), c(k), c(v), s.reshape(-1)[idx].cpu(), c(do), c(kv), c(dkv), dtype=torch.float32)


def _check_heads(got, ref, heads, names):
    errs = {n_: O.rel_err(got[n_][:, heads], ref[n_]) for n_ in names if got.get(n_) is not None}
    assert max(errs.values()) <= TOL, errs
    return errs


def test_config2_headline_shape(gpu_device):
    """b=1 h=16 n=65536 d=128 bf16 single pass; oracle on heads {0, 7, 15}."""
    dev = gpu_device
    b, h, n, d = 1, 16, 65536, 128
    q, k, v, do = [_randn((b, h, n, d), dev, 200 + i, d ** -0.5) for i in range(4)]
    s = O.slopes_baseline(h).to(dev)
    got = _fwd_bwd(q, k, v, do, s)
    torch.cuda.synchronize()
    heads = [0, 7, 15]
    _check_heads(got, _oracle_heads(q, k, v, do, s, heads), heads, ("o", "dq", "dk", "dv"))
    # no atomics, fixed reduction order: a second run gives the same bits
    again = _fwd_bwd(q, k, v, do, s)
    for name in ("o", "dq", "dk", "dv"):
        assert torch.equal(again[name], got[name]), name
    del again
    # chunk chain (4 x 16384, states carried) == single pass
    kv = torch.zeros(b, h, d, d, device=dev)
    outs = []
    states = [kv]
    for c in range(4):
        sl = slice(c * 16384, (c + 1) * 16384)
        from lasp_amd import _abi
        kvo = torch.empty_like(kv)
        o, _, _ = _abi.chunk_fwd(q[:, :, sl], k[:, :, sl], v[:, :, sl], s, kv_in=states[-1], kv_out=kvo)
        outs.append(o)
        states.append(kvo)
    assert _rel(torch.cat(outs, 2), got["o"]) <= TOL
    # linearity in V, head permutation
    o2 = _fwd_bwd(q, k, (2 * v.float()).to(torch.bfloat16), do, s)["o"]
    assert _rel(o2, 2 * got["o"].float()) <= 1e-6
    perm = torch.randperm(h, device=dev)
    o3 = _fwd_bwd(q[:, perm], k[:, perm], v[:, perm], do[:, perm], s[perm])["o"]
    assert torch.equal(o3, got["o"][:, perm])


def test_config3_chunk_with_incoming_state(gpu_device):
    """b=1 h=32 n=16384 d=128 bf16 with KV_in ~ N(0, 0.02); DKV_in = 0 and ~ N(0, 0.02)."""
    dev = gpu_device
    b, h, n, d = 1, 32, 16384, 128
    q, k, v, do = [_randn((b, h, n, d), dev, 300 + i, d ** -0.5) for i in range(4)]
    g = torch.Generator(device=dev).manual_seed(305)
    kv = torch.randn(b, h, d, d, generator=g, device=dev) * 0.02
    dkv = torch.randn(b, h, d, d, generator=g, device=dev) * 0.02
    s = O.slopes_baseline(h).to(dev)
    heads = [0, 13, 31]
    for dkv_in in (torch.zeros_like(dkv), dkv):
        got = _fwd_bwd(q, k, v, do, s, kv=kv, dkv=dkv_in)
        torch.cuda.synchronize()
        ref = _oracle_heads(q, k, v, do, s, heads, kv, dkv_in)
        _check_heads(got, ref, heads, ("o", "dq", "dk", "dv", "kv_out", "dkv_out"))
        # recomputing the segment states in backward gives the same gradients
        got2 = _fwd_bwd(q, k, v, do, s, kv=kv, dkv=dkv_in, cache=False)
        for name in ("dq", "dk", "dv", "dkv_out"):
            assert torch.equal(got[name], got2[name]), name


@pytest.mark.parametrize("variant", ["decay", "no_decay_elu"])
def test_config4_million_tokens_chunk_chain(gpu_device, variant):
    """b=1 h=16 n=1048576 d=128 bf16 as 64 chunks of 16384 with KV / DKV carry.

    Oracle (fp32 recurrence over the whole sequence) on heads {0, 15}; the chain is
    also compared with one single-pass launch over all 1M tokens for every head, and run a second time
    through the lasp_fuse operator with the loopback."""
    from lasp_amd import _abi

    dev = gpu_device
    b, h, n, d, chunks = 1, 16, 1 << 20, 128, 64
    step = n // chunks
    if variant == "decay":
        q, k, v, do = [_randn((b, h, n, d), dev, 400 + i, d ** -0.5) for i in range(4)]
        s = O.slopes_baseline(h).to(dev)
    else:
        elu1 = lambda t: (torch.nn.functional.elu(t.float()) + 1).to(torch.bfloat16)
        q, k = [elu1(_randn((b, h, n, d), dev, 410 + i, 1.0)) for i in range(2)]
        v, do = [_randn((b, h, n, d), dev, 412 + i, 1.0) for i in range(2)]
        s = torch.zeros(h, 1, 1, device=dev)

    kv_states = [torch.zeros(b, h, d, d, device=dev)]
    outs, caches = [], []
    for c in range(chunks):
        sl = slice(c * step, (c + 1) * step)
        kvo = torch.empty_like(kv_states[0])
        o, st, seg = _abi.chunk_fwd(q[:, :, sl], k[:, :, sl], v[:, :, sl], s, kv_in=kv_states[-1], kv_out=kvo)
        outs.append(o)
        caches.append(st)
        kv_states.append(kvo)
    dkv = torch.zeros(b, h, d, d, device=dev)
    dqs, dks, dvs = [None] * chunks, [None] * chunks, [None] * chunks
    for c in reversed(range(chunks)):
        sl = slice(c * step, (c + 1) * step)
        dkvo = torch.empty_like(dkv)
        dqs[c], dks[c], dvs[c] = _abi.chunk_bwd(q[:, :, sl], k[:, :, sl], v[:, :, sl], s, do[:, :, sl],
                                                kv_in=kv_states[c], dkv_in=dkv, dkv_out=dkvo,
                                                kv_seg_states=caches[c])
        dkv = dkvo
    torch.cuda.synchronize()
    got = dict(o=torch.cat(outs, 2), dq=torch.cat(dqs, 2), dk=torch.cat(dks, 2), dv=torch.cat(dvs, 2))
    del outs, dqs, dks, dvs, caches

    heads = [0, 15]
    ref = _oracle_heads(q, k, v, do, s, heads)
    _check_heads(got, ref, heads, ("o", "dq", "dk", "dv"))

    single = _fwd_bwd(q, k, v, do, s)
    torch.cuda.synchronize()
    for name in ("o", "dq", "dk", "dv"):
        for hd in range(h):  # per head: the scale of the outputs differs by orders of magnitude across slopes
            assert _rel(got[name][:, hd], single[name][:, hd]) <= TOL, (name, hd)
    del single

    # the same 64-chunk chain through the public operator (autograd + loopback state passing, one process
    # playing every rank): heads {0, 15} against the oracle, every head against the raw-ABI chain above
    via_op = _operator_chain(q, k, v, do, s, chunks)
    _check_heads(via_op, ref, heads, ("o", "dq", "dk", "dv"))
    for name in ("o", "dq", "dk", "dv"):
        for hd in range(h):
            assert _rel(via_op[name][:, hd], got[name][:, hd]) <= TOL, (name, hd)


def _operator_chain(q, k, v, do, s, chunks):
    import lasp_amd

    b, h, n, d = q.shape
    step = n // chunks
    KV = torch.empty(b, h, d, d, device=q.device)
    DKV = torch.empty_like(KV)
    lasp_amd.destroy_parallel_groups()
    lasp_amd.initialize_lasp(1, chunks)
    outs, leaves = [], []
    try:
        for c in range(chunks):
            lasp_amd.set_sequence_parallel_rank(c)
            sl = slice(c * step, (c + 1) * step)
            qc, kc, vc = [t[:, :, sl].clone().requires_grad_(True) for t in (q, k, v)]
            outs.append(lasp_amd.lasp_fuse(qc, kc, vc, s, KV, DKV))
            leaves.append((qc, kc, vc))
        for c in reversed(range(chunks)):
            outs[c].backward(do[:, :, c * step:(c + 1) * step])
        torch.cuda.synchronize()
        assert lasp_amd.loopback_pending() == []
    finally:
        lasp_amd.destroy_parallel_groups()
    return dict(o=torch.cat([o.detach() for o in outs], 2), dq=torch.cat([l[0].grad for l in leaves], 2),
                dk=torch.cat([l[1].grad for l in leaves], 2), dv=torch.cat([l[2].grad for l in leaves], 2))


def test_headline_shape_ragged_and_narrow_instantiations(gpu_device):
    """The ragged-length and narrow-row instantiations of the sweeps at the headline size (16 sweep segments of
    4096 tokens over 2048-token pieces of the pre-pass), every head, against the aligned full-width kernels:
    * a chunk of n - 8 tokens equals the first n - 8 tokens of the n-token chunk whose last 8 dO rows are zero
      (O and dQ are causal; with a zero tail in dO nothing flows back from the cut-off tokens into dK and dV);
    * rows of 64 features equal the full-width kernels on the same rows zero-extended to 128 (zero columns add
      nothing to any product)."""
    from lasp_amd import _abi

    dev = gpu_device
    b, h, n, d = 1, 16, 65536, 128
    q, k, v, do = [_randn((b, h, n, d), dev, 230 + i, d ** -0.5) for i in range(4)]
    s = O.slopes_baseline(h).to(dev)
    kv = torch.randn(b, h, d, d, device=dev, generator=torch.Generator(device=dev).manual_seed(240))
    do[:, :, n - 8:] = 0
    full = _fwd_bwd(q, k, v, do, s, kv=kv)
    cut = n - 8
    assert _abi.plan(b, h, cut, d, d, torch.bfloat16)[0] == _abi.plan(b, h, n, d, d, torch.bfloat16)[0] == 4096
    c = lambda t: t[:, :, :cut].contiguous()
    ragged = _fwd_bwd(c(q), c(k), c(v), c(do), s, kv=kv)
    torch.cuda.synchronize()
    for name in ("o", "dq", "dk", "dv"):
        assert _rel(ragged[name], full[name][:, :, :cut]) <= 1e-3, name
    del ragged, full

    half = lambda t: t[..., :64].contiguous()
    pad = lambda t: torch.nn.functional.pad(t, (0, 64))
    qn, kn, vn, don = half(q), half(k), half(v), half(do)
    kvn = kv[:, :, :64, :64].contiguous()
    narrow = _fwd_bwd(qn, kn, vn, don, s, kv=kvn)
    kvw = torch.zeros_like(kv)
    kvw[:, :, :64, :64] = kvn
    wide = _fwd_bwd(pad(qn), pad(kn), pad(vn), pad(don), s, kv=kvw)
    torch.cuda.synchronize()
    for name in ("o", "dq", "dk", "dv"):
        assert _rel(narrow[name], wide[name][..., :64]) <= 1e-3, name
    assert _rel(narrow["kv_out"], wide["kv_out"][:, :, :64, :64]) <= 1e-3
