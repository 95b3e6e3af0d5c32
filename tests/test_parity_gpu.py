"""Parity of the HIP path (through the C ABI) against the CPU oracle.

Error metric: max|x - ref| / max|ref| of every (batch, head) slice of every output tensor
(the worst slice is held to the tolerance), ref = fp64 oracle on the
same rounded inputs.  Tolerances: 1e-3 for fp32 I/O, 2e-2 for bf16 / fp16 I/O.
"""
import pytest
import torch

from oracle import lasp_oracle as O
from tests.helpers import TOL, check, make_inputs, oracle

pytestmark = pytest.mark.gpu


def run_abi(inp, s, dev, seg_len=0, cache=False, exact=False):
    """One chunk forward + backward through lasp_amd._abi (ctypes -> liblasp_hip.so).

    exact=True hands the shape to the library as is (narrow heads then run on the generic
    kernels); otherwise the Python layer zero-pads narrow heads onto the MFMA kernels."""
    from lasp_amd import _abi

    fwd = _abi._chunk_fwd_exact if exact else _abi.chunk_fwd
    bwd = _abi._chunk_bwd_exact if exact else _abi.chunk_bwd

    t = {k_: (x.to(dev) if x is not None else None) for k_, x in inp.items()}
    kv_out = torch.empty_like(t["kv"]) if t["kv"] is not None else None
    dkv_out = torch.empty_like(t["dkv"]) if t["dkv"] is not None else None
    o, states, sl = fwd(t["q"], t["k"], t["v"], s, kv_in=t["kv"], kv_out=kv_out, seg_len=seg_len)
    dq, dk, dv = bwd(t["q"], t["k"], t["v"], s, t["do"], kv_in=t["kv"], dkv_in=t["dkv"],
                     dkv_out=dkv_out, kv_seg_states=states if cache else None, seg_len=sl)
    torch.cuda.synchronize()
    return dict(o=o, kv_out=kv_out, dq=dq, dk=dk, dv=dv, dkv_out=dkv_out)


def mfma_path(b, h, n, dtype, d=128, e=128):
    """The path id of an MFMA-eligible shape under the default plan.  Short 16-bit chunks whose segments
    are few (longest walk over preceding blocks within 16 blocks) run as one launch per direction; an explicit seg_len,
    as most tests below pass, always selects the pre-pass / scan / sweep kernels."""
    from lasp_amd import _abi

    if dtype == torch.float32 or n > 2048:
        return _abi.PATH_MFMA
    seg_len, n_seg, _ = _abi.plan(b, h, n, d, e, dtype)
    per_seg = seg_len // 64
    return _abi.PATH_MFMA_FUSED if (n_seg - 1) * per_seg <= 16 else _abi.PATH_MFMA


def test_library_loaded_and_path_selection(gpu_device):
    from lasp_amd import _abi

    lib = _abi.load()
    assert lib.lasp_abi_version() == 1
    assert _abi.kernel_path(1, 16, 65536, 128, 128, torch.bfloat16) == _abi.PATH_MFMA
    assert _abi.kernel_path(2, 12, 2048, 128, 128, torch.float32) == _abi.PATH_MFMA
    assert _abi.kernel_path(2, 12, 2048, 128, 96, torch.float32) == _abi.PATH_GENERIC
    assert _abi.kernel_path(2, 12, 2047, 128, 128, torch.bfloat16) == _abi.PATH_MFMA       # 8 segments: too long a walk
    assert _abi.kernel_path(2, 12, 512, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED  # 2 segments
    assert _abi.kernel_path(1, 3, 768, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED   # 3 segments, 8-block walk
    assert _abi.kernel_path(4, 32, 2048, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED  # 2 segments of 1024: a 16-block walk
    assert _abi.kernel_path(4, 32, 2048, 128, 64, torch.bfloat16) == _abi.PATH_MFMA_FUSED  # narrow rows alike
    assert _abi.kernel_path(2, 12, 2048, 128, 64, torch.bfloat16) == _abi.PATH_MFMA
    assert _abi.kernel_path(2, 12, 2048, 128, 60, torch.bfloat16) == _abi.PATH_GENERIC


@pytest.mark.parametrize("state", [False, True])
@pytest.mark.parametrize("shape", [
    (1, 2, 64, 32, 32, 0), (2, 3, 200, 64, 32, 0), (1, 2, 7, 16, 48, 0),
    (1, 2, 1024, 128, 96, 256), (1, 3, 777, 128, 64, 256), (1, 1, 33, 8, 8, 0), (1, 2, 40, 96, 128, 0),
    (1, 2, 300, 24, 30, 64), (2, 1, 700, 17, 5, 128),   # widths that are no multiples of 4: the scan goes element by element
])
def test_generic_fp32_small(gpu_device, shape, state):
    b, h, n, d, e, seg = shape
    inp = make_inputs(b, h, n, d, e, torch.float32, seed=n + d, state=state, state_std=1.0)
    s = O.slopes_baseline(h)
    got = run_abi(inp, s, gpu_device, seg_len=seg, exact=True)
    check(got, oracle(inp, s), 1e-3 if n > 64 else 2e-4, what=f"fp32 {shape} state={state}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_generic_low_precision_io(gpu_device, dtype):
    # e not a multiple of 8, handed to the library as is: generic kernels with 16-bit I/O
    inp = make_inputs(2, 12, 500, 128, 60, dtype, seed=3, state=True, state_std=1.0)
    s = O.slopes_alibi(12)
    got = run_abi(inp, s, gpu_device, exact=True)
    check(got, oracle(inp, s), TOL[dtype], what=str(dtype))


def test_special_slopes_zero_and_huge(gpu_device):
    inp = make_inputs(1, 2, 300, 32, 32, torch.float32, seed=5, state=True, state_std=1.0)
    s = torch.tensor([0.0, 50.0])
    got = run_abi(inp, s, gpu_device, exact=True)
    assert all(torch.isfinite(v_).all() for v_ in got.values())
    check(got, oracle(inp, s), 1e-3, what="s in {0, 50}")


def test_cached_states_equal_recompute(gpu_device):
    inp = make_inputs(1, 4, 1024, 128, 96, torch.float32, seed=6, state=True, state_std=1.0)
    s = O.slopes_baseline(4)
    a = run_abi(inp, s, gpu_device, seg_len=256, cache=False, exact=True)
    c = run_abi(inp, s, gpu_device, seg_len=256, cache=True, exact=True)
    for name in ("dq", "dk", "dv", "dkv_out"):
        assert torch.equal(a[name], c[name]), name


def test_segment_length_does_not_change_result(gpu_device):
    inp = make_inputs(1, 2, 1536, 64, 64, torch.float32, seed=7, state=True, state_std=1.0)
    s = O.slopes_baseline(2)
    ref = oracle(inp, s)
    for seg in (64, 512, 2048):
        check(run_abi(inp, s, gpu_device, seg_len=seg, exact=True), ref, 1e-3, what=f"seg_len={seg}")


def test_config0_fp32_full(gpu_device):
    """Configuration 0 (the CPU-runnable case): b=2 n=2048 h=12 d=128 fp32, no incoming state."""
    inp = make_inputs(2, 12, 2048, 128, 128, torch.float32, seed=0, state=False)
    s = O.slopes_baseline(12)
    got = run_abi(inp, s, gpu_device)
    check(got, oracle(inp, s), 1e-3, what="config 0")


def test_argument_errors(gpu_device):
    from lasp_amd import _abi

    q = torch.zeros(1, 1, 64, 256, device=gpu_device)
    with pytest.raises(_abi.LaspError, match="unsupported shape"):
        _abi.chunk_fwd(q, q, q, torch.ones(1))
    q = torch.zeros(1, 1, 64, 64, device=gpu_device)
    with pytest.raises(_abi.LaspError, match="seg_len"):
        _abi.chunk_fwd(q, q, q, torch.ones(1), seg_len=100)
    with pytest.raises(_abi.LaspError, match="slopes"):
        _abi.chunk_fwd(q, q, q, torch.ones(3))
    with pytest.raises(_abi.LaspError, match="ROCm"):
        _abi.chunk_fwd(q.cpu(), q.cpu(), q.cpu(), torch.ones(1))


# ---------------------------------------------------------------- bf16 MFMA kernels (d = e = 128)
@pytest.mark.parametrize("state", [False, True])
@pytest.mark.parametrize("b,h,n,seg", [
    (1, 1, 64, 0), (1, 2, 128, 64), (1, 2, 256, 0), (2, 3, 512, 128), (1, 4, 1024, 256), (1, 2, 2048, 2048),
    (2, 2, 320, 256),   # last segment shorter than the others
    (3, 5, 192, 128),   # b*h*n_seg not a multiple of 8 (partial group of backward workgroup triples)
])
def test_mfma_bf16(gpu_device, b, h, n, seg, state):
    from lasp_amd import _abi

    assert _abi.kernel_path(b, h, n, 128, 128, torch.bfloat16) == mfma_path(b, h, n, torch.bfloat16)
    inp = make_inputs(b, h, n, 128, 128, torch.bfloat16, seed=n + h, state=state, state_std=1.0)
    s = O.slopes_baseline(h) if h > 1 else torch.tensor([0.05])
    got = run_abi(inp, s, gpu_device, seg_len=seg)
    check(got, oracle(inp, s), 2e-2, what=f"mfma b={b} h={h} n={n} seg={seg} state={state}")


def test_mfma_special_slopes(gpu_device):
    inp = make_inputs(1, 3, 512, 128, 128, torch.bfloat16, seed=11, state=True, state_std=1.0)
    s = torch.tensor([0.0, 1.0, 30.0])
    got = run_abi(inp, s, gpu_device, seg_len=128)
    assert all(torch.isfinite(v_.float()).all() for v_ in got.values())
    check(got, oracle(inp, s), 2e-2, what="mfma s in {0, 1, 30}")


def test_mfma_inter_path_in_isolation(gpu_device):
    # K = V = 0 leaves O = diag(l^i) Q KV_in and dQ = diag(l^i) dO KV_in^T: the state operand alone
    inp = make_inputs(1, 2, 256, 128, 128, torch.bfloat16, seed=12, state=True, state_std=1.0)
    inp["k"].zero_()
    inp["v"].zero_()
    s = torch.tensor([0.02, 0.3])
    got = run_abi(inp, s, gpu_device, seg_len=128)
    check(got, oracle(inp, s), 2e-2, what="mfma inter only")


def test_mfma_cached_states_equal_recompute(gpu_device):
    inp = make_inputs(1, 4, 1024, 128, 128, torch.bfloat16, seed=13, state=True, state_std=1.0)
    s = O.slopes_baseline(4)
    a = run_abi(inp, s, gpu_device, seg_len=256, cache=False)
    c = run_abi(inp, s, gpu_device, seg_len=256, cache=True)
    for name in ("dq", "dk", "dv", "dkv_out"):
        assert torch.equal(a[name], c[name]), name


@pytest.mark.parametrize("d,e", [(128, 64), (64, 128), (64, 64), (96, 32), (8, 120), (100, 36)])
def test_narrow_bf16_heads_on_mfma(gpu_device, d, e):
    """Narrow heads: the kernels read rows zero-extended when d and e are multiples of 8 (the reference's
    own test shape has e = 64, tests/test.py:95); otherwise the Python layer zero-pads.  Exact either way."""
    from lasp_amd import _abi

    native = d % 8 == 0 and e % 8 == 0
    assert _abi.kernel_path(2, 3, 512, d, e, torch.bfloat16) == (_abi.PATH_MFMA_FUSED if native else _abi.PATH_GENERIC)
    inp = make_inputs(2, 3, 512, d, e, torch.bfloat16, seed=d + e, state=True, state_std=1.0)
    assert _abi._pad_to_mfma(inp["q"], inp["v"]) == (not native)
    s = O.slopes_alibi(3)
    for cache in (False, True):
        got = run_abi(inp, s, gpu_device, seg_len=128, cache=cache)
        assert got["o"].shape[-1] == e and got["dq"].shape[-1] == d and got["kv_out"].shape[-2:] == (d, e)
        check(got, oracle(inp, s), 2e-2, what=f"narrow d={d} e={e} cache={cache}")


@pytest.mark.parametrize("seg", [0, 64])
def test_narrow_rows_leave_neighbouring_memory_alone(gpu_device, seg):
    """Outputs narrower than 128 features are written at their own width: a guard band after
    each output tensor keeps its bits (seg 0: the single-launch kernels, 64: pre-pass / scan / sweep)."""
    from lasp_amd import _abi

    b, h, n, d, e = 1, 2, 200, 64, 32
    inp = make_inputs(b, h, n, d, e, torch.bfloat16, seed=77, state=True, state_std=1.0, device=gpu_device)
    s = O.slopes_alibi(h).to(gpu_device)
    o, states, sl = _abi.chunk_fwd(inp["q"], inp["k"], inp["v"], s, kv_in=inp["kv"], kv_out=torch.empty_like(inp["kv"]),
                                   seg_len=seg)
    torch.cuda.synchronize()
    assert (states is None) == (seg == 0)
    # re-run into views of guarded buffers through the raw entry point
    lib = _abi.load()
    guard = 4096
    buf = torch.full((b * h * n * e + guard,), 1.5, dtype=torch.bfloat16, device=gpu_device)
    kvo = torch.full((b * h * d * e + guard,), -2.5, dtype=torch.float32, device=gpu_device)
    rc = lib.lasp_chunk_fwd(inp["q"].data_ptr(), inp["k"].data_ptr(), inp["v"].data_ptr(), s.data_ptr(),
                            inp["kv"].data_ptr(), kvo.data_ptr(), buf.data_ptr(),
                            None if states is None else states.data_ptr(),
                            b, h, n, d, e, _abi.DTYPE_CODE[torch.bfloat16], sl,
                            torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    assert torch.equal(buf[:b * h * n * e].view(b, h, n, e), o)
    assert (buf[b * h * n * e:] == 1.5).all() and (kvo[b * h * d * e:] == -2.5).all()
    # the gradients as well
    dkvo = torch.full((b * h * d * e + guard,), -2.5, dtype=torch.float32, device=gpu_device)
    outs = [torch.full((b * h * n * w_ + guard,), 1.5, dtype=torch.bfloat16, device=gpu_device) for w_ in (d, d, e)]
    ws = torch.empty(2 * b * h * 8 * 128 * 128, dtype=torch.float32, device=gpu_device)
    rc = lib.lasp_chunk_bwd(inp["q"].data_ptr(), inp["k"].data_ptr(), inp["v"].data_ptr(), s.data_ptr(),
                            inp["do"].data_ptr(), inp["kv"].data_ptr(), inp["dkv"].data_ptr(), outs[0].data_ptr(),
                            outs[1].data_ptr(), outs[2].data_ptr(), dkvo.data_ptr(), None, ws.data_ptr(),
                            ws.numel() * 4, b, h, n, d, e, _abi.DTYPE_CODE[torch.bfloat16], sl,
                            torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0, lib.lasp_last_error()
    for t, w_ in zip(outs, (d, d, e)):
        assert (t[b * h * n * w_:] == 1.5).all() and torch.isfinite(t[:b * h * n * w_].float()).all()
    assert (dkvo[b * h * d * e:] == -2.5).all()


@pytest.mark.parametrize("n,d,e", [(2047, 128, 128), (65, 128, 128), (700, 128, 64), (63, 128, 128), (1, 128, 128)])
def test_ragged_bf16_length(gpu_device, n, d, e):
    inp = make_inputs(1, 3, n, d, e, torch.bfloat16, seed=n, state=True, state_std=1.0)
    s = O.slopes_alibi(3)
    ref = oracle(inp, s)
    for cache in (False, True):
        got = run_abi(inp, s, gpu_device, cache=cache)
        assert got["o"].shape == inp["v"].shape and got["dq"].shape == inp["q"].shape
        check(got, ref, 2e-2, what=f"ragged n={n} d={d} e={e} cache={cache}")


@pytest.mark.parametrize("b,h,n,seg,state", [(1, 2, 256, 64, True), (2, 3, 1024, 256, True), (1, 4, 512, 0, False),
                                             (1, 2, 4096, 2048, True)])  # the last: the pre-pass's deep pipeline
def test_mfma_fp16(gpu_device, b, h, n, seg, state):
    from lasp_amd import _abi

    assert _abi.kernel_path(b, h, n, 128, 128, torch.float16) == mfma_path(b, h, n, torch.float16)
    inp = make_inputs(b, h, n, 128, 128, torch.float16, seed=n + 7, state=state, state_std=1.0)
    s = O.slopes_baseline(h)
    got = run_abi(inp, s, gpu_device, seg_len=seg)
    check(got, oracle(inp, s), 2e-2, what=f"fp16 mfma b={b} h={h} n={n}")


def test_fp16_narrow_and_ragged(gpu_device):
    inp = make_inputs(1, 3, 333, 64, 96, torch.float16, seed=17, state=True, state_std=1.0)
    s = O.slopes_alibi(3)
    check(run_abi(inp, s, gpu_device), oracle(inp, s), 2e-2, what="fp16 ragged narrow")
    # segments long enough for the pre-pass's deep pipeline, the last one partial
    inp = make_inputs(1, 2, 2100, 64, 96, torch.float16, seed=18, state=True, state_std=1.0)
    s = O.slopes_baseline(2)
    check(run_abi(inp, s, gpu_device, seg_len=1024), oracle(inp, s), 2e-2, what="fp16 ragged narrow, seg_len=1024")


# ---------------------------------------------------------------- fp32 MFMA kernels (d = e = 128)
@pytest.mark.parametrize("state", [False, True])
@pytest.mark.parametrize("b,h,n,seg", [
    (1, 1, 32, 0), (1, 2, 96, 64), (1, 2, 256, 64), (2, 3, 512, 128), (1, 4, 1024, 256), (1, 2, 2048, 2048),
    (2, 2, 320, 256), (3, 5, 192, 128),
])
def test_mfma_fp32(gpu_device, b, h, n, seg, state):
    from lasp_amd import _abi

    assert _abi.kernel_path(b, h, n, 128, 128, torch.float32) == _abi.PATH_MFMA
    inp = make_inputs(b, h, n, 128, 128, torch.float32, seed=n + h + 1, state=state, state_std=1.0)
    s = O.slopes_baseline(h) if h > 1 else torch.tensor([0.05])
    got = run_abi(inp, s, gpu_device, seg_len=seg)
    check(got, oracle(inp, s), 1e-4, what=f"fp32 mfma b={b} h={h} n={n} seg={seg} state={state}")


def test_mfma_fp32_special_slopes_and_padding(gpu_device):
    inp = make_inputs(1, 3, 512, 128, 128, torch.float32, seed=31, state=True, state_std=1.0)
    s = torch.tensor([0.0, 1.0, 30.0])
    got = run_abi(inp, s, gpu_device, seg_len=128)
    assert all(torch.isfinite(v_).all() for v_ in got.values())
    check(got, oracle(inp, s), 1e-4, what="fp32 mfma s in {0, 1, 30}")
    # narrow heads (zero-padded) with a ragged length (masked last block)
    inp = make_inputs(1, 2, 300, 64, 96, torch.float32, seed=32, state=True, state_std=1.0)
    s = O.slopes_baseline(2)
    check(run_abi(inp, s, gpu_device), oracle(inp, s), 1e-4, what="fp32 narrow ragged")


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2), (torch.float32, 1e-4)])
@pytest.mark.parametrize("b,h,n,seg", [(1, 2, 100, 0), (2, 3, 333, 128), (1, 2, 1000, 256), (1, 1, 31, 0)])
def test_mfma_ragged_lengths_in_kernel(gpu_device, dtype, tol, b, h, n, seg):
    """A chunk length that is not a multiple of the block: the last block is masked inside the kernels."""
    from lasp_amd import _abi

    assert _abi.kernel_path(b, h, n, 128, 128, dtype) == mfma_path(b, h, n, dtype)
    inp = make_inputs(b, h, n, 128, 128, dtype, seed=n + 3, state=True, state_std=1.0)
    s = torch.tensor([0.3, 0.01, 2.0][:h])
    ref = oracle(inp, s)
    for cache in (False, True):
        got = run_abi(inp, s, gpu_device, seg_len=seg, cache=cache)
        assert all(torch.isfinite(v_.float()).all() for v_ in got.values())
        check(got, ref, tol, what=f"ragged {dtype} n={n} seg={seg} cache={cache}")


def test_seeded_random_shapes(gpu_device):
    """24 shapes drawn from a fixed seed: any n (ragged against blocks and against segments), narrow and
    full heads, the three dtypes, forced and planned segment lengths, with and without incoming states."""
    import random

    rng = random.Random(20240607)
    dtypes = [torch.bfloat16, torch.float16, torch.float32]
    for case in range(24):
        b, h = rng.choice([1, 2]), rng.randint(1, 5)
        n = rng.choice([rng.randint(1, 130), rng.randint(131, 1500)])
        d, e = rng.choice([128, 128, 64, 48]), rng.choice([128, 128, 64, 16])
        dtype = rng.choice(dtypes)
        seg = rng.choice([0, 0, 64, 128, 256, 512])
        state = rng.random() < 0.6
        s = rng.choice([O.slopes_baseline(h), O.slopes_alibi(h), torch.zeros(h, 1, 1)])
        inp = make_inputs(b, h, n, d, e, dtype, seed=1000 + case, scale=0.3, state=state, state_std=0.5)
        what = f"case {case}: b={b} h={h} n={n} d={d} e={e} {dtype} seg={seg} state={state}"
        print(what, flush=True)
        got = run_abi(inp, s, gpu_device, seg_len=seg, cache=bool(case & 1))
        check(got, oracle(inp, s), 1e-4 if dtype == torch.float32 else 2e-2, what=what)


def test_seeded_random_shapes_of_whole_blocks(gpu_device):
    """40 shapes drawn from a fixed seed among the full-width 16-bit shapes of whole blocks (d = e = 128): 1 to 80 blocks, planned and forced segment lengths from one block upwards -- single-launch,
    scan-less (up to 4 segments) and scan paths, sweep segments longer than the pre-pass's 2048-token pieces,
    one-block segments, a short last segment -- with and without incoming states, states kept or recomputed."""
    import random

    rng = random.Random(20260925)
    for case in range(40):
        b, h = rng.choice([1, 2]), rng.randint(1, 6)
        n = 64 * rng.choice([rng.randint(1, 8), rng.randint(9, 40), rng.randint(41, 80)])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        seg = rng.choice([0, 0, 0, 64, 128, 192, 320, 512, 1024, 2048, 4096])
        state = rng.random() < 0.6
        s = rng.choice([O.slopes_baseline(h), O.slopes_alibi(h), torch.zeros(h, 1, 1), torch.full((h, 1, 1), 0.02),
                        torch.full((h, 1, 1), 5.0)])
        inp = make_inputs(b, h, n, 128, 128, dtype, seed=3000 + case, scale=0.3, state=state, state_std=0.5)
        what = f"case {case}: b={b} h={h} n={n} {dtype} seg={seg} state={state} slopes={s.flatten().tolist()[:3]}"
        print(what, flush=True)
        got = run_abi(inp, s, gpu_device, seg_len=seg, cache=bool(case & 1))
        assert all(torch.isfinite(v_.float()).all() for v_ in got.values() if v_ is not None)
        check(got, oracle(inp, s), 2e-2, what=what)


# ---------------------------------------------------------------- single-launch path for short chunks
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("state", [False, True])
@pytest.mark.parametrize("b,h,n,d,e", [
    (2, 12, 512, 128, 128),    # two segments of 256 tokens
    (2, 4, 640, 128, 128),     # three segments, the last one short
    (1, 3, 768, 128, 128),     # three segments
    (1, 2, 64, 128, 128), (1, 1, 192, 128, 128),
    (2, 12, 1024, 128, 128),   # six segments of 192 tokens, walks of up to 15 blocks
    (4, 32, 2048, 128, 128),   # two segments of 1024 tokens, a walk of 16 blocks; 3 * 128 * 2 workgroups backwards
    (2, 3, 700, 128, 128), (1, 4, 513, 128, 128), (1, 2, 333, 128, 128), (1, 2, 1, 128, 128),   # ragged lengths
    (2, 12, 512, 128, 64), (1, 3, 700, 64, 96), (2, 2, 321, 48, 16),                              # narrow rows
])
def test_fused_short_chunks_match_oracle_and_three_kernel_path(gpu_device, b, h, n, d, e, state, dtype):
    """Default plan, short chunk, few segments: one launch per direction, states rebuilt inside each workgroup.  Checked
    against the oracle and against the pre-pass / scan / sweep kernels on the same segment length."""
    from lasp_amd import _abi

    assert _abi.kernel_path(b, h, n, d, e, dtype) == _abi.PATH_MFMA_FUSED
    inp = make_inputs(b, h, n, d, e, dtype, seed=n + d + e, scale=0.5, state=state, state_std=1.0)
    s = O.slopes_baseline(h) if h > 1 else torch.tensor([0.004])
    got = run_abi(inp, s, gpu_device)                      # seg_len 0: the single-launch kernels
    check(got, oracle(inp, s), 2e-2, what=f"fused b={b} h={h} n={n} d={d} e={e} state={state}")
    planned = _abi.plan(b, h, n, d, e, dtype)[0]
    other = run_abi(inp, s, gpu_device, seg_len=planned)   # explicit seg_len: the three-kernel path
    for name in ("o", "dq", "dk", "dv", "kv_out", "dkv_out"):
        if got[name] is not None:
            assert O.rel_err(got[name], other[name].float()) <= 2e-2, name


def test_fused_special_slopes(gpu_device):
    # no decay (nothing may be skipped, the walk always reaches the chunk's start and the incoming state),
    # moderate and very fast decay (the walk is cut to a block or two)
    inp = make_inputs(1, 3, 768, 128, 128, torch.bfloat16, seed=19, scale=0.3, state=True, state_std=1.0)
    s = torch.tensor([0.0, 1.0, 30.0])
    from lasp_amd import _abi

    assert _abi.kernel_path(1, 3, 768, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED
    got = run_abi(inp, s, gpu_device)
    assert all(torch.isfinite(v_.float()).all() for v_ in got.values())
    check(got, oracle(inp, s), 2e-2, what="fused s in {0, 1, 30}")


def test_fused_needs_no_workspace_through_the_raw_abi(gpu_device):
    from lasp_amd import _abi

    lib = _abi.load()
    dev = gpu_device
    b, h, n, d = 1, 4, 512, 128
    assert _abi.kernel_path(b, h, n, d, d, torch.bfloat16) == _abi.PATH_MFMA_FUSED
    inp = make_inputs(b, h, n, d, d, torch.bfloat16, seed=23, scale=d ** -0.5, state=True, device=dev)
    s = O.slopes_baseline(h).reshape(-1).to(dev)
    o = torch.empty_like(inp["v"])
    kvo, dkvo = torch.empty_like(inp["kv"]), torch.empty_like(inp["dkv"])
    dq, dk, dv = torch.empty_like(inp["q"]), torch.empty_like(inp["k"]), torch.empty_like(inp["v"])
    stream = torch.cuda.current_stream(dev).cuda_stream
    code = _abi.DTYPE_CODE[torch.bfloat16]
    rc = lib.lasp_chunk_fwd(inp["q"].data_ptr(), inp["k"].data_ptr(), inp["v"].data_ptr(), s.data_ptr(),
                            inp["kv"].data_ptr(), kvo.data_ptr(), o.data_ptr(), None, b, h, n, d, d, code, 0, stream)
    assert rc == 0, lib.lasp_last_error()
    rc = lib.lasp_chunk_bwd(inp["q"].data_ptr(), inp["k"].data_ptr(), inp["v"].data_ptr(), s.data_ptr(),
                            inp["do"].data_ptr(), inp["kv"].data_ptr(), inp["dkv"].data_ptr(), dq.data_ptr(),
                            dk.data_ptr(), dv.data_ptr(), dkvo.data_ptr(), None, None, 0, b, h, n, d, d, code, 0, stream)
    assert rc == 0, lib.lasp_last_error()
    torch.cuda.synchronize()
    check(dict(o=o, kv_out=kvo, dq=dq, dk=dk, dv=dv, dkv_out=dkvo), oracle(inp, s), 2e-2, what="raw fused calls")


def test_fp16_large_incoming_state_stays_finite(gpu_device):
    """fp16 I/O rounds the fp32 state to fp16 before each matrix product: an incoming state three orders of
    magnitude above the activations is well inside the fp16 range and must come through with the usual bound
    (the range limit itself, |state| or |q.k| beyond 65504, is part of the contract in include/lasp_hip.h)."""
    inp = make_inputs(1, 3, 1024, 128, 128, torch.float16, seed=91, scale=128 ** -0.5, state=True, state_std=1e3)
    s = O.slopes_baseline(3)
    for seg in (0, 256):
        got = run_abi(inp, s, gpu_device, seg_len=seg)
        assert all(torch.isfinite(v_.float()).all() for v_ in got.values())
        check(got, oracle(inp, s), 2e-2, what=f"fp16 with kv_in of std 1e3, seg={seg}")


def test_odd_number_of_pre_pass_pieces(gpu_device):
    """A long sweep segment is cut in two for the pre-pass, and a chunk may end within the first half of its last
    segment: the workspace then holds an odd number of states per (b, h), which is not a multiple of the number
    of sweep segments (the workspace is sized by lasp_plan's state_bytes alone).  Forward + backward with the
    forward's states kept, against the oracle and against recomputed states."""
    from lasp_amd import _abi

    dev = gpu_device
    b, h, n, d = 1, 4, 4096 * 5 - 2048 - 8, 128
    seg_len, n_seg, state_bytes = _abi.plan(b, h, n, d, d, torch.bfloat16, 4096)
    assert (seg_len, n_seg) == (4096, 5) and state_bytes == b * h * 9 * d * d * 4
    inp = make_inputs(b, h, n, d, d, torch.bfloat16, seed=91, scale=d ** -0.5, state=True, device=dev)
    s = O.slopes_baseline(16).reshape(-1)[[0, 9, 14, 15]].contiguous().to(dev)
    kv_out, dkv_out = torch.empty_like(inp["kv"]), torch.empty_like(inp["dkv"])
    o, states, sl = _abi.chunk_fwd(inp["q"], inp["k"], inp["v"], s, kv_in=inp["kv"], kv_out=kv_out, seg_len=4096)
    assert states.numel() * 4 == state_bytes
    kept = _abi.chunk_bwd(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=inp["dkv"],
                          dkv_out=dkv_out, kv_seg_states=states, seg_len=sl)
    redone = _abi.chunk_bwd(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=inp["dkv"],
                            dkv_out=None, kv_seg_states=None, seg_len=sl)
    torch.cuda.synchronize()
    for a, r in zip(kept, redone):
        assert torch.equal(a, r)
    cpu = {k_: t.cpu() for k_, t in inp.items()}
    ref = O.ref_chunked(cpu["q"], cpu["k"], cpu["v"], s.cpu(), cpu["do"], cpu["kv"], cpu["dkv"], dtype=torch.float32)
    got = dict(o=o, dq=kept[0], dk=kept[1], dv=kept[2], kv_out=kv_out, dkv_out=dkv_out)
    for name, t in got.items():
        assert O.rel_err(t.cpu(), ref[name]) <= 2e-2, name


@pytest.mark.parametrize("n,seg_len", [(4096, 256), (4096 * 5 - 2048 - 8, 4096)])
def test_in_place_state_update_with_heads_outside_the_scan(gpu_device, n, seg_len):
    """kv_out = kv_in (and dkv_out = dkv_in) on the pre-pass / scan / sweep path.  The scan writes the outgoing
    state before the sweeps run; a head that takes no part in the scan needs the INCOMING state in the sweep of
    its first segment, which therefore must not come from the caller's buffer any more.  In place and out of
    place have to agree bit for bit, for heads in the scan and outside it, with the forward's states kept or not."""
    from lasp_amd import _abi

    dev = gpu_device
    b, h, d = 1, 4, 128
    inp = make_inputs(b, h, n, d, d, torch.bfloat16, seed=93, scale=d ** -0.5, state=True, device=dev)
    s = O.slopes_baseline(16).reshape(-1)[[0, 9, 14, 15]].contiguous().to(dev)
    assert _abi.inplace_ok(b, h, n, d, d, torch.bfloat16, seg_len, False)
    assert _abi.inplace_ok(b, h, n, d, d, torch.bfloat16, seg_len, True)

    def run(in_place):
        kv, dkv = inp["kv"].clone(), inp["dkv"].clone()
        kv_out = kv if in_place else torch.empty_like(kv)
        dkv_out = dkv if in_place else torch.empty_like(dkv)
        o, states, sl = _abi._chunk_fwd_exact(inp["q"], inp["k"], inp["v"], s, kv_in=kv, kv_out=kv_out, seg_len=seg_len)
        kept = _abi._chunk_bwd_exact(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=dkv,
                                     dkv_out=dkv_out, kv_seg_states=states, seg_len=sl)
        dkv2 = inp["dkv"].clone()
        redone = _abi._chunk_bwd_exact(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=dkv2,
                                       dkv_out=dkv2 if in_place else torch.empty_like(dkv2), kv_seg_states=None,
                                       seg_len=sl)
        torch.cuda.synchronize()
        return [o, kv_out, *kept, dkv_out, *redone]

    for a, r in zip(run(False), run(True)):
        assert torch.equal(a, r)
    cpu = {k_: t.cpu() for k_, t in inp.items()}
    ref = O.ref_chunked(cpu["q"], cpu["k"], cpu["v"], s.cpu(), cpu["do"], cpu["kv"], cpu["dkv"], dtype=torch.float32)
    got = run(True)
    for name, t in zip(("o", "kv_out", "dq", "dk", "dv", "dkv_out"), got):
        assert O.rel_err(t.cpu(), ref[name]) <= 2e-2, name


def test_unwritten_workspace_slots_are_never_read(gpu_device, monkeypatch):
    """Heads that take no part in the scan get only the piece states that something reads (one per sweep
    segment, and the two visited last for the outgoing state); the other slots of the workspace stay as they
    were allocated.  With every fresh allocation of the binding poisoned with NaN (workspaces and outputs alike)
    the results must be finite and bit-identical to those of a run on zeroed allocations."""
    from lasp_amd import _abi

    dev = gpu_device
    b, h, n, d = 1, 4, 4096 * 5 - 2048 - 8, 128
    inp = make_inputs(b, h, n, d, d, torch.bfloat16, seed=92, scale=d ** -0.5, state=True, device=dev)
    s = O.slopes_baseline(16).reshape(-1)[[0, 9, 14, 15]].contiguous().to(dev)  # two heads outside the scan, two in it
    real_empty, real_empty_like = torch.empty, torch.empty_like

    def run(fill, carry):
        def filled(t):
            return t.fill_(fill) if t.is_floating_point() else t
        monkeypatch.setattr(torch, "empty", lambda *a, **k: filled(real_empty(*a, **k)))
        monkeypatch.setattr(torch, "empty_like", lambda *a, **k: filled(real_empty_like(*a, **k)))
        try:
            kv_out = torch.empty_like(inp["kv"]) if carry else None
            dkv_out = torch.empty_like(inp["dkv"]) if carry else None
            o, states, sl = _abi.chunk_fwd(inp["q"], inp["k"], inp["v"], s, kv_in=inp["kv"], kv_out=kv_out, seg_len=4096)
            kept = _abi.chunk_bwd(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=inp["dkv"],
                                  dkv_out=dkv_out, kv_seg_states=states, seg_len=sl)
            redone = _abi.chunk_bwd(inp["q"], inp["k"], inp["v"], s, inp["do"], kv_in=inp["kv"], dkv_in=inp["dkv"],
                                    dkv_out=None, kv_seg_states=None, seg_len=sl)
            torch.cuda.synchronize()
        finally:
            monkeypatch.undo()
        out = [o, *kept, *redone] + ([kv_out, dkv_out] if carry else [])
        return out, states

    for carry in (True, False):
        clean, _ = run(0.0, carry)
        poisoned, states = run(float("nan"), carry)
        assert torch.isnan(states).any(), "the plan of this shape leaves pieces out: some slots stay unwritten"
        for a, r in zip(clean, poisoned):
            assert torch.isfinite(r.float()).all()
            assert torch.equal(a, r)


@pytest.mark.parametrize("shape", [
    (1, 28, 40000, 128, 128),   # two rounds of stretched segments, the pre-pass on whole segments
    (1, 24, 32768 - 8, 128, 128),  # one round of 10 stretched segments cut in two for the pre-pass, ragged
    (1, 56, 2048, 128, 128),    # many heads: 4 segments swept without a scan
    (2, 12, 4096, 128, 64),     # one round of short stretched segments, narrow rows
])
def test_default_plans_where_heads_do_not_divide_the_chip(gpu_device, shape):
    """The default plan stretches segments until the forward sweep fills whole rounds of workgroups, which
    gives segment lengths, piece counts and paths no other test picks: forward + backward with states, the
    default plan against an explicit seg_len = 1024 (the pre-pass / scan / sweep path on plain segments), states
    kept against states rebuilt (bit-equal), and -- where the host can afford it -- against the oracle."""
    from lasp_amd import _abi

    dev = gpu_device
    b, h, n, d, e = shape
    g = torch.Generator(device=dev).manual_seed(n + h)
    mk = lambda *s_: torch.randn(*s_, generator=g, device=dev)
    q, k = [(mk(b, h, n, d) * d ** -0.5).to(torch.bfloat16) for _ in range(2)]
    v, do = [mk(b, h, n, e).to(torch.bfloat16) for _ in range(2)]
    kv, dkv = mk(b, h, d, e) * 0.1, mk(b, h, d, e) * 0.1
    s = O.slopes_baseline(h).reshape(-1).to(dev)
    s[::5] = 0.0
    seg_len, n_seg, _ = _abi.plan(b, h, n, d, e, torch.bfloat16)
    assert seg_len != 1024 and seg_len % 64 == 0
    runs = []
    for seg in (0, 1024):
        kv_out, dkv_out = torch.empty_like(kv), torch.empty_like(dkv)
        print(f"b={b} h={h} n={n} d={d} e={e} seg_len={seg} (plan {seg_len} x {n_seg})", flush=True)
        o, states, sl = _abi.chunk_fwd(q, k, v, s, kv_in=kv, kv_out=kv_out, seg_len=seg)
        kept = _abi.chunk_bwd(q, k, v, s, do, kv_in=kv, dkv_in=dkv, dkv_out=dkv_out, kv_seg_states=states, seg_len=sl)
        redone = _abi.chunk_bwd(q, k, v, s, do, kv_in=kv, dkv_in=dkv, dkv_out=None, kv_seg_states=None, seg_len=sl)
        torch.cuda.synchronize()
        for a, r in zip(kept, redone):
            assert torch.equal(a, r)
        runs.append(dict(o=o, dq=kept[0], dk=kept[1], dv=kept[2], kv_out=kv_out, dkv_out=dkv_out))
    for name in runs[0]:
        assert O.rel_err(runs[0][name].cpu(), runs[1][name].float().cpu()) <= 1.2e-2, name
    if b * h * n <= 200000:
        c = lambda t: t.cpu()
        ref = O.ref_chunked(c(q), c(k), c(v), c(s), c(do), c(kv), c(dkv), dtype=torch.float32)
        for name in runs[0]:
            assert O.rel_err(runs[0][name].cpu(), ref[name]) <= 2e-2, name
