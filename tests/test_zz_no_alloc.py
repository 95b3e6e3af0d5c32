"""lasp_chunk_fwd_static -- the entry point that allocates nothing -- against lasp_chunk_fwd.

Both are called through the C ABI (ctypes) on the same inputs; the static variant keeps its segment
states in a scratch array inside the library, so it is called twice in a row, the second time on a
smaller input, and must reproduce the workspace variant's output and outgoing state bit for bit
(same kernels, same launch shapes) as well as meet the oracle bound.
"""
import pytest
import torch

from oracle import lasp_oracle as O
from tests.helpers import make_inputs

pytestmark = pytest.mark.gpu


def _both(lib, inp, s, dev, dtype_code, seg_len=0):
    from lasp_amd import _abi

    q, k, v, kv = inp["q"], inp["k"], inp["v"], inp["kv"]
    b, h, n, d = q.shape
    e = v.shape[-1]
    seg_len, n_seg, state_bytes = _abi.plan(b, h, n, d, e, q.dtype, seg_len)
    assert state_bytes <= _abi.STATIC_SCRATCH_BYTES
    stream = torch.cuda.current_stream(dev).cuda_stream
    o_ws, o_st = torch.empty_like(v), torch.empty_like(v)
    kv_ws, kv_st = torch.empty_like(kv), torch.empty_like(kv)
    ws = torch.empty(state_bytes // 4, dtype=torch.float32, device=dev)
    print(f"lasp_chunk_fwd b={b} h={h} n={n} d={d} e={e} seg_len={seg_len} n_seg={n_seg}", flush=True)
    rc = lib.lasp_chunk_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), kv.data_ptr(), kv_ws.data_ptr(),
                            o_ws.data_ptr(), ws.data_ptr(), b, h, n, d, e, dtype_code, seg_len, stream)
    assert rc == 0, lib.lasp_last_error()
    print("lasp_chunk_fwd_static, same shape", flush=True)
    rc = lib.lasp_chunk_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), kv.data_ptr(),
                                   kv_st.data_ptr(), o_st.data_ptr(), b, h, n, d, e, dtype_code, seg_len, stream)
    assert rc == 0, lib.lasp_last_error()
    torch.cuda.synchronize()
    return o_ws, kv_ws, o_st, kv_st


def test_static_scratch_forward_matches_workspace_forward_twice(gpu_device):
    from lasp_amd import _abi

    lib = _abi.load()
    dev = gpu_device
    # first call: 4 heads x 8 segments; second call, smaller: 2 heads, a ragged length, 3 segments.
    # The second call finds the first one's states in the scratch and must not be affected by them.
    for (b, h, n, d, e, seg), seed in (((1, 4, 2048, 128, 128, 256), 71), ((1, 2, 700, 128, 64, 256), 72)):
        inp = make_inputs(b, h, n, d, e, torch.bfloat16, seed=seed, scale=d ** -0.5, state=True, device=dev)
        s = O.slopes_baseline(h).reshape(-1).to(dev)
        o_ws, kv_ws, o_st, kv_st = _both(lib, inp, s, dev, _abi.DTYPE_CODE[torch.bfloat16], seg)
        assert torch.equal(o_st, o_ws) and torch.equal(kv_st, kv_ws)
        cpu = {k_: (t.cpu() if t is not None else None) for k_, t in inp.items()}
        ref_o, ref_kv = O.ref_chunked_fwd(cpu["q"], cpu["k"], cpu["v"], s.cpu(), cpu["kv"], 64, torch.float64)
        assert O.rel_err(o_st, ref_o) <= 2e-2 and O.rel_err(kv_st, ref_kv) <= 2e-2


@pytest.mark.parametrize("shape,seg", [((1, 4, 2048, 128, 128), 256),    # pre-pass / scan / sweep: 8 segments
                                       ((2, 3, 1536, 128, 128), 512),    # scan-less: 3 segments gathered by the sweeps
                                       ((1, 2, 320, 128, 128), 0),       # default plan: a single launch, no states
                                       ((1, 2, 700, 128, 64), 256)])     # narrow rows, ragged length
def test_static_scratch_forward_allocates_nothing(gpu_device, shape, seg):
    """After a first (warm) call -- which looks the scratch's address up and loads the kernels -- a second
    call must leave the device's free memory and torch's allocation count where they were, and give the
    workspace variant's bits."""
    from lasp_amd import _abi

    lib = _abi.load()
    dev = gpu_device
    b, h, n, d, e = shape
    inp = make_inputs(b, h, n, d, e, torch.bfloat16, seed=74, scale=d ** -0.5, state=True, device=dev)
    s = O.slopes_baseline(h).reshape(-1).to(dev)
    want, _, _ = _abi.chunk_fwd(inp["q"], inp["k"], inp["v"], s, kv_in=inp["kv"], kv_out=torch.empty_like(inp["kv"]),
                                seg_len=seg)
    o, kv_out = torch.empty_like(inp["v"]), torch.empty_like(inp["kv"])
    stream = torch.cuda.current_stream(dev).cuda_stream
    args = (inp["q"].data_ptr(), inp["k"].data_ptr(), inp["v"].data_ptr(), s.data_ptr(), inp["kv"].data_ptr(),
            kv_out.data_ptr(), o.data_ptr(), b, h, n, d, e, _abi.DTYPE_CODE[torch.bfloat16], seg, stream)
    print(f"lasp_chunk_fwd_static warm call b={b} h={h} n={n} d={d} e={e} seg_len={seg}", flush=True)
    assert lib.lasp_chunk_fwd_static(*args) == 0, lib.lasp_last_error()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    allocs_before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    o.zero_()  # in place: no allocation
    print("lasp_chunk_fwd_static second call", flush=True)
    assert lib.lasp_chunk_fwd_static(*args) == 0, lib.lasp_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == allocs_before
    assert torch.equal(o, want)


def test_static_scratch_python_wrapper_and_size_limit(gpu_device):
    from lasp_amd import _abi

    dev = gpu_device
    inp = make_inputs(1, 2, 512, 128, 128, torch.bfloat16, seed=73, scale=128 ** -0.5, state=False, device=dev)
    s = O.slopes_baseline(2).reshape(-1).to(dev)
    o = torch.empty_like(inp["v"])
    _abi.chunk_fwd_static(inp["q"], inp["k"], inp["v"], s, o)
    want, _, _ = _abi.chunk_fwd(inp["q"], inp["k"], inp["v"], s)
    torch.cuda.synchronize()
    assert torch.equal(o, want)
    # 1024 states of 64 KiB do not fit the 32 MiB scratch: refused before anything is launched
    big = torch.empty(1, 16, 65536, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(_abi.LaspError, match="scratch holds"):
        _abi.chunk_fwd_static(big, big, big, O.slopes_baseline(16).reshape(-1).to(dev), torch.empty_like(big),
                              seg_len=1024)
