"""Every head against the oracle where the decay-dependent shortcuts of the 16-bit kernels bite.

The pre-pass skips blocks whose weights lie below 2^-24, the scan leaves out heads whose state dies
within one segment, and both only take effect on long segments.  Here every (batch, head) slice of every
output is held to the oracle (fp32 block recurrence on the same rounded inputs) under the 2e-2 bound, on
the pre-pass / scan / sweep path (6 segments of 2048 tokens, the planned segment length, and 6 sweep segments
of 4096 tokens over a pre-pass on halves of them) and on the scan-less path (4 segments of 2048), with incoming KV and dKV states, with the forward's segment states
kept for the backward and with the backward recomputing them.  Slope sets: the benchmark's schedule,
and one built around the shortcuts' thresholds (no decay, the pre-pass reaching exactly one block, the
scan's cut-off at the segment length just met and just missed)."""
import math

import pytest
import torch

from oracle import lasp_oracle as O
from tests.helpers import NAMES, check

pytestmark = pytest.mark.gpu
TOL = 2e-2
H, D = 16, 128
SKIP_LOG2 = 24.0  # the kernels treat decay weights below 2^-24 as zero


def _inputs(n, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    mk = lambda: (torch.randn(1, H, n, D, generator=g, device=dev) * D ** -0.5).to(torch.bfloat16)
    q, k, v, do = mk(), mk(), mk(), mk()
    kv = torch.randn(1, H, D, D, generator=g, device=dev) * 0.02
    dkv = torch.randn(1, H, D, D, generator=g, device=dev) * 0.02
    return dict(q=q, k=k, v=v, do=do, kv=kv, dkv=dkv)


def _threshold_slopes(seg_len):
    """Heads 0-1: no decay (nothing may be skipped).  Heads 2-4: weights reach 2^-24 after exactly 64
    tokens, and a hair to either side.  Heads 5-7: the decay over one segment is 2^-24 exactly (the scan's
    cut-off) and a hair to either side.  The rest: the benchmark's schedule."""
    s = [2.0 ** (-8.0 * (i + 1) / H) for i in range(H)]
    one_block = SKIP_LOG2 * math.log(2.0) / 64  # SKIP_LOG2 / (s log2 e) = 64 tokens
    per_seg = SKIP_LOG2 * math.log(2.0) / seg_len
    s[0] = s[1] = 0.0
    s[2], s[3], s[4] = one_block, one_block * (1 + 1e-6), one_block * (1 - 1e-6)
    s[5], s[6], s[7] = per_seg, per_seg * (1 + 1e-6), per_seg * (1 - 1e-6)
    return torch.tensor(s, dtype=torch.float32).reshape(H, 1, 1)


def _run(inp, s, seg_len, cache):
    from lasp_amd import _abi

    kv_out, dkv_out = torch.empty_like(inp["kv"]), torch.empty_like(inp["dkv"])
    o, states, sl = _abi.chunk_fwd(inp["q"], inp["k"], inp["v"], s, kv_in=inp["kv"], kv_out=kv_out, seg_len=seg_len)
    dq, dk, dv = _abi.chunk_bwd(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=inp["dkv"],
                                dkv_out=dkv_out, kv_seg_states=states if cache else None, seg_len=sl)
    torch.cuda.synchronize()
    return {k_: t.cpu() for k_, t in dict(o=o, kv_out=kv_out, dq=dq, dk=dk, dv=dv, dkv_out=dkv_out).items()}


@pytest.mark.parametrize("slope_set", ["baseline", "thresholds"])
@pytest.mark.parametrize("n,seg_len", [(12288, 2048), (12288, 0), (8192, 2048), (8192, 0), (24576, 4096)],
                         ids=["scan_6x2048", "scan_planned", "combine_4x2048", "planned_8192", "scan_6x4096_prepass_2048"])
def test_every_head_with_states(gpu_device, slope_set, n, seg_len):
    from lasp_amd import _abi

    dev = gpu_device
    planned = _abi.plan(1, H, n, D, D, torch.bfloat16, seg_len)[0]
    # the scan's cut-off works on the pre-pass's segments, which are at most 2048 tokens long
    s = O.slopes_baseline(H) if slope_set == "baseline" else _threshold_slopes(min(planned, 2048))
    inp = _inputs(n, dev, seed=500 + n // 1024 + seg_len)
    cpu = {k_: t.cpu() for k_, t in inp.items()}
    ref = O.ref_chunked(cpu["q"], cpu["k"], cpu["v"], s, cpu["do"], cpu["kv"], cpu["dkv"], dtype=torch.float32)
    kept = _run(inp, s.to(dev), seg_len, cache=True)
    check(kept, ref, TOL, what=f"{slope_set} n={n} seg_len={planned} states kept")
    redone = _run(inp, s.to(dev), seg_len, cache=False)
    check(redone, ref, TOL, what=f"{slope_set} n={n} seg_len={planned} states recomputed")
    for name in NAMES:  # the same kernels on the same numbers either way
        assert torch.equal(kept[name], redone[name]), name
