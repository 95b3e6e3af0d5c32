"""CPU oracle for causal decayed linear attention with KV-state passing.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this module;
it is used by the tests, by the smoke check and by the CPU-baseline leg of the
benchmark, as the checker.

Two independent statements of the same operator are held here so that each can
pin the other:

* ``ref_quadratic``  -- the closed form  O = ((Q K^T) * M) V + diag(l^i) Q KV_in
  evaluated literally (an n x n mask), with the backward obtained from
  ``torch.autograd`` on  L = <O, dO> + <KV_out, DKV_in>.  It mirrors nothing in
  the reference but the definition of the mask
  (lasp/lightning_attention.py:49-52, lasp/lasp_fuse.py:95-98) and of the state
  update (lasp/lasp_fuse.py:126-127).

* ``ref_chunked``    -- the O(n) block recurrence with explicit backward
  formulas, following lasp/lasp_fuse.py:88-127 (forward sweep with the incoming
  state) and lasp/lasp_fuse.py:174-353 (forward-direction dq sweep, then the
  reverse dk/dv sweep with the DKV chain); the torch matmul spelling of the
  incoming-state terms follows lasp/lasp_naive.py:560-565,604-614.

What pins them (tests/test_oracle.py): the two agree with each other; the
explicit backward agrees with autograd of the closed form and with
``torch.autograd.gradcheck``; a scalar triple loop in pure Python agrees on tiny
shapes; s = 0 reduces to cumulative-sum causal linear attention; a very large
slope reduces to the diagonal  (q_i . k_i) v_i ; K = V = 0 isolates the
incoming-state GEMM; chunked evaluation composes to the single pass; heads are
independent.  The reference holds no golden vectors for this path (its test
prints unseeded statistics only), so bit-level agreement with the reference's
Triton arithmetic is "parity unpinned"; the mathematics is pinned.

Shapes: q, k (b, h, n, d); v, dO (b, h, n, e); s any tensor with h elements;
KV_in, DKV_in (b, h, d, e).  Positions are 0-based inside the chunk.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

__all__ = [
    "slopes_alibi",
    "slopes_baseline",
    "decay_mask",
    "ref_quadratic_fwd",
    "ref_quadratic",
    "ref_chunked_fwd",
    "ref_chunked_bwd",
    "ref_chunked",
    "ref_loops_fwd",
    "rel_err",
    "rel_err_slices",
    "rel_err_whole",
]


# --------------------------------------------------------------------------
# slopes
# --------------------------------------------------------------------------
def slopes_alibi(h: int) -> torch.Tensor:
    """Slopes as lasp/utils/module_utils.py:6-31 produces them, shape (h, 1, 1).

    Power-of-two h: s_i = 2^(-8 (i+1) / h).  Otherwise the slopes of the
    largest power of two below h, followed by every other slope of twice that
    power of two.
    """

    def pow2(m: int):
        return [2.0 ** (-8.0 * (i + 1) / m) for i in range(m)]

    def rec(m: int):
        lg = math.log2(m)
        if lg == int(lg):
            return pow2(m)
        p = 2 ** int(math.floor(lg))
        return pow2(p) + rec(2 * p)[0::2][: m - p]

    return torch.tensor(rec(h), dtype=torch.float32).reshape(h, 1, 1)


def slopes_baseline(h: int) -> torch.Tensor:
    """s_i = 2^(-8 (i+1) / h) for every h (the benchmark configurations)."""
    return torch.tensor(
        [2.0 ** (-8.0 * (i + 1) / h) for i in range(h)], dtype=torch.float32
    ).reshape(h, 1, 1)


def _flat_s(s: torch.Tensor, h: int, dtype) -> torch.Tensor:
    s = s.reshape(-1).to(dtype)
    assert s.numel() == h, f"need {h} slopes, got {s.numel()}"
    return s


def decay_mask(s: torch.Tensor, n: int, dtype=torch.float64) -> torch.Tensor:
    """M[h, i, j] = exp(-s_h (i - j)) for j <= i, else 0."""
    s = s.reshape(-1).to(dtype)
    idx = torch.arange(n, dtype=dtype)
    diff = idx[:, None] - idx[None, :]
    expo = torch.where(diff >= 0, -s[:, None, None] * diff, torch.full_like(diff, -float("inf")))
    return torch.exp(expo)


# --------------------------------------------------------------------------
# closed form (quadratic in n)
# --------------------------------------------------------------------------
def ref_quadratic_fwd(q, k, v, s, kv_in=None, dtype=torch.float64):
    """Returns (O, KV_out) from the closed form, in ``dtype``."""
    b, h, n, d = q.shape
    e = v.shape[-1]
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    sv = _flat_s(s, h, dtype)
    M = decay_mask(sv, n, dtype)  # h n n
    scores = torch.einsum("bhid,bhjd->bhij", q, k) * M[None]
    o = torch.einsum("bhij,bhje->bhie", scores, v)
    pos = torch.arange(n, dtype=dtype)
    if kv_in is not None:
        kv_in = kv_in.to(dtype)
        lam_i = torch.exp(-sv[:, None] * pos[None, :])  # h n
        o = o + lam_i[None, :, :, None] * torch.einsum("bhid,bhde->bhie", q, kv_in)
    lam_rev = torch.exp(-sv[:, None] * (n - pos)[None, :])  # h n : l^(n-j)
    kv_out = torch.einsum("bhjd,bhje->bhde", k * lam_rev[None, :, :, None], v)
    if kv_in is not None:
        kv_out = kv_out + torch.exp(-sv * n)[None, :, None, None] * kv_in
    return o, kv_out


def ref_quadratic(q, k, v, s, do, kv_in=None, dkv_in=None, dtype=torch.float64):
    """Closed-form forward plus autograd backward.

    Returns dict with o, kv_out, dq, dk, dv, dkv_out (dkv_out = dL/dKV_in).
    """
    b, h, n, d = q.shape
    e = v.shape[-1]
    qq = q.detach().to(dtype).clone().requires_grad_(True)
    kk = k.detach().to(dtype).clone().requires_grad_(True)
    vv = v.detach().to(dtype).clone().requires_grad_(True)
    kvi = (
        torch.zeros(b, h, d, e, dtype=dtype)
        if kv_in is None
        else kv_in.detach().to(dtype).clone()
    ).requires_grad_(True)
    o, kv_out = ref_quadratic_fwd(qq, kk, vv, s, kvi, dtype)
    loss = (o * do.to(dtype)).sum()
    if dkv_in is not None:
        loss = loss + (kv_out * dkv_in.to(dtype)).sum()
    dq, dk, dv, dkv_out = torch.autograd.grad(loss, [qq, kk, vv, kvi])
    return dict(
        o=o.detach(), kv_out=kv_out.detach(), dq=dq, dk=dk, dv=dv, dkv_out=dkv_out
    )


# --------------------------------------------------------------------------
# block recurrence (linear in n) with explicit backward
# --------------------------------------------------------------------------
def _block_consts(sv, B, dtype):
    """Per-head decay vectors for a block of B rows (all exponents <= 0)."""
    idx = torch.arange(B, dtype=dtype)
    lam_q = torch.exp(-sv[:, None] * idx[None, :])  # l^i          (h, B)
    lam_k = torch.exp(-sv[:, None] * (B - idx)[None, :])  # l^(B-j)  (h, B)
    lam_blk = torch.exp(-sv * B)  # l^B                              (h,)
    M = decay_mask(sv, B, dtype)  # (h, B, B)
    return lam_q, lam_k, lam_blk, M


def ref_chunked_fwd(q, k, v, s, kv_in=None, block=64, dtype=torch.float32):
    """Forward sweep of lasp/lasp_fuse.py:104-127.  Returns (O, KV_out).

    A tail shorter than ``block`` is handled by a final shorter block (the
    reference's lightning kernel masks the tail, lasp/lightning_attention.py:58-68).
    """
    b, h, n, d = q.shape
    e = v.shape[-1]
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    sv = _flat_s(s, h, dtype)
    kv = (
        torch.zeros(b, h, d, e, dtype=dtype) if kv_in is None else kv_in.to(dtype).clone()
    )
    o = torch.empty(b, h, n, e, dtype=dtype)
    for t0 in range(0, n, block):
        B = min(block, n - t0)
        lam_q, lam_k, lam_blk, M = _block_consts(sv, B, dtype)
        qt, kt, vt = q[:, :, t0 : t0 + B], k[:, :, t0 : t0 + B], v[:, :, t0 : t0 + B]
        intra = torch.matmul(torch.matmul(qt, kt.transpose(-1, -2)) * M[None], vt)
        inter = torch.matmul(qt, kv) * lam_q[None, :, :, None]
        o[:, :, t0 : t0 + B] = intra + inter
        kv = lam_blk[None, :, None, None] * kv + torch.matmul(
            (kt * lam_k[None, :, :, None]).transpose(-1, -2), vt
        )
    return o, kv


def ref_chunked_bwd(q, k, v, s, do, kv_in=None, dkv_in=None, block=64, dtype=torch.float32):
    """dq sweep (lasp/lasp_fuse.py:237-260) then reverse dk/dv sweep (:316-353).

    Returns (dq, dk, dv, dkv_out).
    """
    b, h, n, d = q.shape
    e = v.shape[-1]
    q, k, v, do = q.to(dtype), k.to(dtype), v.to(dtype), do.to(dtype)
    sv = _flat_s(s, h, dtype)
    dq = torch.empty(b, h, n, d, dtype=dtype)
    dk = torch.empty(b, h, n, d, dtype=dtype)
    dv = torch.empty(b, h, n, e, dtype=dtype)
    starts = list(range(0, n, block))

    kv = (
        torch.zeros(b, h, d, e, dtype=dtype) if kv_in is None else kv_in.to(dtype).clone()
    )
    for t0 in starts:
        B = min(block, n - t0)
        lam_q, lam_k, lam_blk, M = _block_consts(sv, B, dtype)
        dot, kt, vt = do[:, :, t0 : t0 + B], k[:, :, t0 : t0 + B], v[:, :, t0 : t0 + B]
        dp = torch.matmul(dot, vt.transpose(-1, -2)) * M[None]
        dq[:, :, t0 : t0 + B] = torch.matmul(dp, kt) + lam_q[None, :, :, None] * torch.matmul(
            dot, kv.transpose(-1, -2)
        )
        kv = lam_blk[None, :, None, None] * kv + torch.matmul(
            (kt * lam_k[None, :, :, None]).transpose(-1, -2), vt
        )

    dkv = (
        torch.zeros(b, h, d, e, dtype=dtype)
        if dkv_in is None
        else dkv_in.to(dtype).clone()
    )
    for t0 in reversed(starts):
        B = min(block, n - t0)
        lam_q, lam_k, lam_blk, M = _block_consts(sv, B, dtype)
        qt, kt, vt, dot = (
            q[:, :, t0 : t0 + B],
            k[:, :, t0 : t0 + B],
            v[:, :, t0 : t0 + B],
            do[:, :, t0 : t0 + B],
        )
        dp = torch.matmul(dot, vt.transpose(-1, -2)) * M[None]
        sc = torch.matmul(qt, kt.transpose(-1, -2)) * M[None]
        dk[:, :, t0 : t0 + B] = torch.matmul(dp.transpose(-1, -2), qt) + lam_k[
            None, :, :, None
        ] * torch.matmul(vt, dkv.transpose(-1, -2))
        dv[:, :, t0 : t0 + B] = torch.matmul(sc.transpose(-1, -2), dot) + lam_k[
            None, :, :, None
        ] * torch.matmul(kt, dkv)
        dkv = lam_blk[None, :, None, None] * dkv + torch.matmul(
            (qt * lam_q[None, :, :, None]).transpose(-1, -2), dot
        )
    return dq, dk, dv, dkv


def ref_chunked(q, k, v, s, do, kv_in=None, dkv_in=None, block=64, dtype=torch.float32):
    o, kv_out = ref_chunked_fwd(q, k, v, s, kv_in, block, dtype)
    dq, dk, dv, dkv_out = ref_chunked_bwd(q, k, v, s, do, kv_in, dkv_in, block, dtype)
    return dict(o=o, kv_out=kv_out, dq=dq, dk=dk, dv=dv, dkv_out=dkv_out)


# --------------------------------------------------------------------------
# scalar loops (tiny shapes only): an independent brute-force statement
# --------------------------------------------------------------------------
def ref_loops_fwd(q, k, v, s, kv_in=None):
    """Pure-Python triple loop over (i, j); returns (O, KV_out) as float64 tensors."""
    b, h, n, d = q.shape
    e = v.shape[-1]
    q, k, v = q.double(), k.double(), v.double()
    sv = s.reshape(-1).double()
    o = torch.zeros(b, h, n, e, dtype=torch.float64)
    kv_out = torch.zeros(b, h, d, e, dtype=torch.float64)
    for bi in range(b):
        for hi in range(h):
            lam = math.exp(-float(sv[hi]))
            for i in range(n):
                for j in range(i + 1):
                    w = lam ** (i - j) * float(torch.dot(q[bi, hi, i], k[bi, hi, j]))
                    o[bi, hi, i] += w * v[bi, hi, j]
                if kv_in is not None:
                    o[bi, hi, i] += lam**i * (q[bi, hi, i] @ kv_in[bi, hi].double())
            for j in range(n):
                kv_out[bi, hi] += lam ** (n - j) * torch.outer(k[bi, hi, j], v[bi, hi, j])
            if kv_in is not None:
                kv_out[bi, hi] += lam**n * kv_in[bi, hi].double()
    return o, kv_out


def rel_err_whole(x: torch.Tensor, ref: torch.Tensor) -> float:
    """max|x - ref| / max|ref| over the whole tensor (reported next to the per-head figure)."""
    x = x.detach().double().cpu()
    ref = ref.detach().double().cpu()
    denom = ref.abs().max().item()
    if denom == 0.0:
        return (x - ref).abs().max().item()
    return ((x - ref).abs().max() / denom).item()


def rel_err_slices(x: torch.Tensor, ref: torch.Tensor) -> torch.Tensor:
    """max|x - ref| / max|ref| of every (batch, head) slice of a (b, h, ., .) tensor, shape (b, h).

    Heads differ by orders of magnitude in output scale (slopes from 0.7 down to 0.004 make the
    slow-decay heads sum thousands of terms, the fast ones a handful), so a bound over the whole
    tensor would let the large heads vouch for the small ones.  A slice whose reference is all
    zero reports its absolute error.
    """
    x = x.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert x.shape == ref.shape and x.dim() == 4, (tuple(x.shape), tuple(ref.shape))
    err = (x - ref).abs().amax(dim=(2, 3))
    denom = ref.abs().amax(dim=(2, 3))
    return torch.where(denom > 0, err / denom.clamp_min(1e-300), err)


def rel_err(x: torch.Tensor, ref: torch.Tensor) -> float:
    """The parity metric: the worst (batch, head) slice of max|x - ref| / max|ref|.

    Tensors that are not (b, h, ., .) are measured as a whole."""
    if x.dim() != 4 or x.numel() == 0:
        return rel_err_whole(x, ref)
    return rel_err_slices(x, ref).max().item()
