"""Pins the CPU oracle: every function of oracle/lasp_oracle.py is checked against
something other than its own formula (closed form vs recurrence vs scalar loops vs
autograd vs textbook special cases)."""
import math

import pytest
import torch

from oracle import lasp_oracle as O

torch.manual_seed(0)


def _inputs(b, h, n, d, e, seed=0, dtype=torch.float64, state=True):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, n, d, generator=g, dtype=dtype)
    k = torch.randn(b, h, n, d, generator=g, dtype=dtype)
    v = torch.randn(b, h, n, e, generator=g, dtype=dtype)
    do = torch.randn(b, h, n, e, generator=g, dtype=dtype)
    kv = torch.randn(b, h, d, e, generator=g, dtype=dtype) if state else None
    dkv = torch.randn(b, h, d, e, generator=g, dtype=dtype) if state else None
    return q, k, v, do, kv, dkv


def test_slopes_known_answers():
    # hand-derived from lasp/utils/module_utils.py:8-24
    s8 = O.slopes_alibi(8).flatten()
    assert torch.allclose(s8, torch.tensor([2.0 ** -(i + 1) for i in range(8)]))
    s16 = O.slopes_alibi(16).flatten()
    assert torch.allclose(s16, torch.tensor([2.0 ** (-(i + 1) / 2) for i in range(16)]))
    s12 = O.slopes_alibi(12).flatten()
    want = [2.0 ** -(i + 1) for i in range(8)] + [2.0**-0.5, 2.0**-1.5, 2.0**-2.5, 2.0**-3.5]
    assert torch.allclose(s12, torch.tensor(want))
    assert O.slopes_alibi(12).shape == (12, 1, 1)
    assert O.slopes_alibi(12).dtype == torch.float32
    sb = O.slopes_baseline(12).flatten()
    assert torch.allclose(sb, torch.tensor([2.0 ** (-8 * (i + 1) / 12) for i in range(12)]))


def test_mask_definition():
    s = torch.tensor([0.5, 0.0])
    M = O.decay_mask(s, 5)
    for i in range(5):
        for j in range(5):
            want = math.exp(-0.5 * (i - j)) if j <= i else 0.0
            assert abs(M[0, i, j].item() - want) < 1e-15
            assert M[1, i, j].item() == (1.0 if j <= i else 0.0)


@pytest.mark.parametrize("state", [False, True])
def test_quadratic_matches_scalar_loops(state):
    q, k, v, do, kv, dkv = _inputs(1, 2, 9, 3, 4, seed=1, state=state)
    s = torch.tensor([0.3, 0.05])
    o1, kv1 = O.ref_quadratic_fwd(q, k, v, s, kv)
    o2, kv2 = O.ref_loops_fwd(q, k, v, s, kv)
    assert torch.allclose(o1, o2, atol=1e-12)
    assert torch.allclose(kv1, kv2, atol=1e-12)


@pytest.mark.parametrize("n,block", [(64, 64), (192, 64), (200, 64), (96, 32), (7, 64)])
def test_chunked_matches_quadratic(n, block):
    q, k, v, do, kv, dkv = _inputs(2, 3, n, 16, 8, seed=2)
    s = O.slopes_baseline(3)
    a = O.ref_quadratic(q, k, v, s, do, kv, dkv)
    c = O.ref_chunked(q, k, v, s, do, kv, dkv, block=block, dtype=torch.float64)
    for name in ("o", "kv_out", "dq", "dk", "dv", "dkv_out"):
        assert O.rel_err(c[name], a[name]) < 1e-11, name


def test_chunked_matches_quadratic_no_state():
    q, k, v, do, _, _ = _inputs(1, 2, 130, 8, 8, seed=3, state=False)
    s = torch.tensor([0.7, 0.01])
    a = O.ref_quadratic(q, k, v, s, do)
    c = O.ref_chunked(q, k, v, s, do, block=64, dtype=torch.float64)
    for name in ("o", "kv_out", "dq", "dk", "dv", "dkv_out"):
        assert O.rel_err(c[name], a[name]) < 1e-11, name


def test_gradcheck_closed_form():
    q, k, v, do, kv, dkv = _inputs(1, 2, 6, 3, 2, seed=4)
    s = torch.tensor([0.4, 0.1])

    def f(q_, k_, v_, kv_):
        o, kvo = O.ref_quadratic_fwd(q_, k_, v_, s, kv_)
        return o, kvo

    args = [t.clone().requires_grad_(True) for t in (q, k, v, kv)]
    assert torch.autograd.gradcheck(f, args, eps=1e-6, atol=1e-6)


def test_zero_slope_is_cumsum_linear_attention():
    # s = 0: O_i = q_i . sum_{j<=i} k_j^T v_j  (causal linear attention)
    q, k, v, do, _, _ = _inputs(1, 2, 100, 8, 6, seed=5, state=False)
    s = torch.zeros(2)
    outer = torch.einsum("bhnd,bhne->bhnde", k, v).cumsum(2)
    want = torch.einsum("bhnd,bhnde->bhne", q, outer)
    o, kvo = O.ref_chunked_fwd(q, k, v, s, block=32, dtype=torch.float64)
    assert O.rel_err(o, want) < 1e-12
    assert O.rel_err(kvo, outer[:, :, -1]) < 1e-12
    oq, kvq = O.ref_quadratic_fwd(q, k, v, s)
    assert O.rel_err(oq, want) < 1e-12


def test_large_slope_is_diagonal():
    q, k, v, do, _, _ = _inputs(1, 1, 40, 8, 6, seed=6, state=False)
    s = torch.tensor([60.0])
    want = (q * k).sum(-1, keepdim=True) * v
    o, kvo = O.ref_chunked_fwd(q, k, v, s, block=16, dtype=torch.float64)
    assert O.rel_err(o, want) < 1e-12
    # only the last token survives in KV_out, with one decay step
    last = math.exp(-60.0) * torch.einsum("bhd,bhe->bhde", k[:, :, -1], v[:, :, -1])
    assert O.rel_err(kvo, last) < 1e-9


def test_inter_path_in_isolation():
    # K = V = 0: O = diag(l^i) Q KV_in, KV_out = l^n KV_in
    q, k, v, do, kv, dkv = _inputs(1, 2, 70, 8, 8, seed=7)
    s = torch.tensor([0.2, 0.03])
    z = torch.zeros_like(k)
    o, kvo = O.ref_chunked_fwd(q, z, torch.zeros_like(v), s, kv, block=32, dtype=torch.float64)
    pos = torch.arange(70, dtype=torch.float64)
    lam = torch.exp(-s.double()[:, None] * pos)  # h n
    want = lam[None, :, :, None] * torch.matmul(q, kv)
    assert O.rel_err(o, want) < 1e-12
    assert O.rel_err(kvo, torch.exp(-s.double() * 70)[None, :, None, None] * kv) < 1e-12


@pytest.mark.parametrize("cuts", [[64, 64, 64], [50, 100, 42], [1, 191]])
def test_chunk_composition(cuts):
    n = sum(cuts)
    q, k, v, do, kv, dkv = _inputs(1, 2, n, 8, 8, seed=8)
    s = torch.tensor([0.25, 0.02])
    full = O.ref_chunked(q, k, v, s, do, kv, dkv, block=64, dtype=torch.float64)
    # forward chain
    outs, states = [], [kv]
    p = 0
    for c in cuts:
        sl = slice(p, p + c)
        o, kvn = O.ref_chunked_fwd(q[:, :, sl], k[:, :, sl], v[:, :, sl], s, states[-1], 64, torch.float64)
        outs.append(o)
        states.append(kvn)
        p += c
    assert O.rel_err(torch.cat(outs, 2), full["o"]) < 1e-12
    assert O.rel_err(states[-1], full["kv_out"]) < 1e-12
    # reverse chain
    dqs, dks, dvs = [], [], []
    d_state = dkv
    p = n
    for ci in reversed(range(len(cuts))):
        c = cuts[ci]
        sl = slice(p - c, p)
        dq, dk, dv, d_state = O.ref_chunked_bwd(
            q[:, :, sl], k[:, :, sl], v[:, :, sl], s, do[:, :, sl], states[ci], d_state, 64, torch.float64
        )
        dqs.insert(0, dq)
        dks.insert(0, dk)
        dvs.insert(0, dv)
        p -= c
    assert O.rel_err(torch.cat(dqs, 2), full["dq"]) < 1e-12
    assert O.rel_err(torch.cat(dks, 2), full["dk"]) < 1e-12
    assert O.rel_err(torch.cat(dvs, 2), full["dv"]) < 1e-12
    assert O.rel_err(d_state, full["dkv_out"]) < 1e-12


def test_head_independence_and_linearity():
    q, k, v, do, kv, dkv = _inputs(1, 3, 40, 4, 4, seed=9)
    s = torch.tensor([0.5, 0.1, 0.01])
    o, kvo = O.ref_chunked_fwd(q, k, v, s, kv, 16, torch.float64)
    perm = [2, 0, 1]
    o2, kvo2 = O.ref_chunked_fwd(q[:, perm], k[:, perm], v[:, perm], s[perm], kv[:, perm], 16, torch.float64)
    assert torch.allclose(o[:, perm], o2)
    assert torch.allclose(kvo[:, perm], kvo2)
    # linear in (V, KV_in)
    o3, _ = O.ref_chunked_fwd(q, k, 2 * v, s, 2 * kv, 16, torch.float64)
    assert torch.allclose(o3, 2 * o)


def test_fp32_oracle_close_to_fp64():
    q, k, v, do, kv, dkv = _inputs(1, 2, 256, 32, 32, seed=10)
    s = O.slopes_baseline(2)
    a = O.ref_quadratic(q, k, v, s, do, kv, dkv)
    c = O.ref_chunked(q.float(), k.float(), v.float(), s, do.float(), kv.float(), dkv.float(), 64, torch.float32)
    for name in ("o", "kv_out", "dq", "dk", "dv", "dkv_out"):
        assert O.rel_err(c[name], a[name]) < 2e-6, name
