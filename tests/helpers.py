"""Shared helpers for the parity tests (inputs by seed, oracle calls, error metric)."""
import torch

from oracle import lasp_oracle as O

TOL = {torch.float32: 1e-3, torch.bfloat16: 2e-2, torch.float16: 2e-2}
NAMES = ("o", "kv_out", "dq", "dk", "dv", "dkv_out")


def make_inputs(b, h, n, d, e, dtype, seed, scale=1.0, state=True, state_std=0.02, device="cpu"):
    """Seeded N(0, scale^2) q, k, v, do rounded to `dtype`; fp32 states N(0, state_std^2)."""
    g = torch.Generator().manual_seed(seed)
    mk = lambda *shape: (torch.randn(*shape, generator=g) * scale).to(dtype)
    q, k, v, do = mk(b, h, n, d), mk(b, h, n, d), mk(b, h, n, e), mk(b, h, n, e)
    kv = dkv = None
    if state:
        kv = torch.randn(b, h, d, e, generator=g) * state_std
        dkv = torch.randn(b, h, d, e, generator=g) * state_std
    out = dict(q=q, k=k, v=v, do=do, kv=kv, dkv=dkv)
    return {k_: (t.to(device) if t is not None else None) for k_, t in out.items()}


def oracle(inp, s, block=64, dtype=torch.float64):
    """Oracle on the SAME (already rounded) inputs, in fp64 unless told otherwise."""
    c = {k_: (t.detach().cpu() if t is not None else None) for k_, t in inp.items()}
    return O.ref_chunked(c["q"], c["k"], c["v"], s.cpu(), c["do"], c["kv"], c["dkv"], block=block, dtype=dtype)


def check(got: dict, ref: dict, tol: float, names=NAMES, what=""):
    """Asserts the parity bound on every (batch, head) slice of every output: the worst slice's
    max|x - ref| / max|ref| must not exceed `tol`.  The whole-tensor figure goes into the message."""
    errs, whole = {}, {}
    for name in names:
        if name in got and got[name] is not None:
            errs[name] = O.rel_err(got[name], ref[name])
            whole[name] = O.rel_err_whole(got[name], ref[name])
    bad = {k_: v_ for k_, v_ in errs.items() if not (v_ <= tol)}
    assert not bad, f"{what}: worst (b,h) slice over {tol}: {bad} (per-head: {errs}; whole tensor: {whole})"
    return errs
