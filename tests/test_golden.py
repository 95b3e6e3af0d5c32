"""Committed fixtures (tests/golden/*.npz): the oracle's recurrence on CPU, and the HIP
path on the GPU, both against the stored float64 closed-form results."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import lasp_oracle as O

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))
NAMES = ("o", "kv_out", "dq", "dk", "dv", "dkv_out")


def _load(path):
    z = np.load(path, allow_pickle=False)
    dtype = {"torch.float32": torch.float32, "torch.bfloat16": torch.bfloat16}[str(z["io_dtype"])]

    def io(name):
        t = torch.from_numpy(z[name].copy())
        return t.view(torch.bfloat16) if dtype == torch.bfloat16 else t

    inp = dict(q=io("q"), k=io("k"), v=io("v"), do=io("do"), kv=torch.from_numpy(z["kv"].copy()),
               dkv=torch.from_numpy(z["dkv"].copy()), s=torch.from_numpy(z["s"].copy()))
    ref = {n_: torch.from_numpy(z["ref_" + n_].copy()) for n_ in NAMES}
    return dtype, inp, ref


def test_fixtures_exist():
    assert len(GOLDEN) >= 2


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_oracle_recurrence_matches_fixture(path):
    dtype, inp, ref = _load(path)
    got = O.ref_chunked(inp["q"], inp["k"], inp["v"], inp["s"], inp["do"], inp["kv"], inp["dkv"], block=64,
                        dtype=torch.float64)
    for n_ in NAMES:
        assert O.rel_err(got[n_], ref[n_]) < 1e-6, n_  # fixtures are stored in float32


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_hip_path_matches_fixture(gpu_device, path):
    from lasp_amd import _abi

    dtype, inp, ref = _load(path)
    t = {k_: v_.to(gpu_device) for k_, v_ in inp.items()}
    kv_out, dkv_out = torch.empty_like(t["kv"]), torch.empty_like(t["dkv"])
    o, states, sl = _abi.chunk_fwd(t["q"], t["k"], t["v"], t["s"], kv_in=t["kv"], kv_out=kv_out, seg_len=64)
    dq, dk, dv = _abi.chunk_bwd(t["q"], t["k"], t["v"], t["s"], t["do"], kv_in=t["kv"], dkv_in=t["dkv"],
                                dkv_out=dkv_out, kv_seg_states=states, seg_len=sl)
    torch.cuda.synchronize()
    got = dict(o=o, kv_out=kv_out, dq=dq, dk=dk, dv=dv, dkv_out=dkv_out)
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    errs = {n_: O.rel_err(got[n_], ref[n_]) for n_ in NAMES}
    assert max(errs.values()) <= tol, errs
