"""CPU-side checks of the C ABI: the library loads, exports every function that
include/lasp_hip.h declares, and its host-only entry points (planning, argument
validation) behave.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lasp_hip.h")


@pytest.fixture(scope="module")
def lib():
    from lasp_amd import _abi

    if not os.path.exists(_abi.lib_path()):
        from lasp_amd import build

        build.build(verbose=False)
    return _abi.load()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(lasp_[a-z_0-9]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for must in ("lasp_abi_version", "lasp_last_error", "lasp_plan", "lasp_kernel_path", "lasp_chunk_fwd",
                 "lasp_chunk_fwd_static", "lasp_chunk_bwd", "lasp_profile_begin", "lasp_profile_end"):
        assert must in names


def test_library_exports_every_declared_symbol(lib):
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} is declared in lasp_hip.h but not exported"
    assert lib.lasp_abi_version() == 1


def test_plan_defaults_and_overrides(lib):
    from lasp_amd import _abi

    # headline shape: 16 (b,h) pairs -> 16 sweep segments of 4096 tokens = 256 workgroups of the
    # sweeps, one per CU; the pre-pass and the scan work on halves of them, so the workspace holds 32 states per (b,h)
    assert _abi.plan(1, 16, 65536, 128, 128, torch.bfloat16) == (4096, 16, 16 * 32 * 128 * 128 * 4)
    # an explicit seg_len gets the same treatment (the backward is handed the forward's seg_len)
    assert _abi.plan(1, 16, 65536, 128, 128, torch.bfloat16, 4096) == (4096, 16, 16 * 32 * 128 * 128 * 4)
    assert _abi.plan(1, 16, 65536, 128, 128, torch.bfloat16, 2048) == (2048, 32, 16 * 32 * 128 * 128 * 4)
    assert _abi.plan(1, 16, 65536, 128, 128, torch.bfloat16, 8192) == (8192, 8, 16 * 32 * 128 * 128 * 4)
    # ragged lengths and narrow rows are planned like the full-width shapes: 8 tokens more than 16 x 4096 still
    # make 16 segments (of 4224 tokens, pre-pass on halves of them), not 29 shorter ones in two rounds
    assert _abi.plan(1, 16, 65536 + 8, 128, 128, torch.bfloat16) == (4224, 16, 16 * 32 * 128 * 128 * 4)
    # where b*h does not divide the chip the segments are stretched until the forward sweep fits one round of 256
    assert _abi.plan(2, 12, 16384, 128, 128, torch.bfloat16)[:2] == (1664, 10)
    assert _abi.plan(1, 24, 32768, 128, 128, torch.bfloat16) == (3328, 10, 24 * 20 * 128 * 128 * 4)
    assert _abi.plan(1, 40, 4096, 128, 128, torch.bfloat16)[:2] == (704, 6)       # shorter chunks alike
    # ... and where the segments are short, a few longer ones that save the backward sweep (three workgroups per
    # segment) a round are taken instead: 7 x 3 x 24 = 504 workgroups are two rounds, 10 x 3 x 24 three
    assert _abi.plan(2, 12, 4096, 128, 128, torch.bfloat16)[:2] == (640, 7)
    assert _abi.plan(1, 12, 8192, 128, 128, torch.bfloat16)[:2] == (640, 13)
    assert _abi.plan(2, 12, 8192, 128, 128, torch.bfloat16)[:2] == (832, 10)      # not beyond about 10 blocks
    # many heads: one round means 2 to 4 segments, swept without a scan launch while they stay within 1024 tokens
    assert _abi.plan(1, 64, 2048, 128, 128, torch.bfloat16)[:2] == (512, 4)
    assert _abi.plan(1, 80, 2048, 128, 128, torch.bfloat16)[:2] == (704, 3)
    assert _abi.plan(1, 52, 8192, 128, 128, torch.bfloat16)[:2] == (1024, 8)       # 4 x 2048 would not pay
    # several rounds where one would need segments beyond ~4096 tokens; the pre-pass then takes whole segments
    assert _abi.plan(1, 48, 65536, 128, 128, torch.bfloat16) == (4096, 16, 48 * 16 * 128 * 128 * 4)
    assert _abi.plan(1, 28, 65536, 128, 128, torch.bfloat16)[:2] == (3648, 18)
    assert _abi.plan(1, 16, 65536, 128, 64, torch.bfloat16) == (4096, 16, 16 * 32 * 128 * 128 * 4)
    # short chunk: 256 tokens per segment at least ...
    assert _abi.plan(1, 16, 2048, 128, 128, torch.bfloat16)[:2] == (256, 8)
    # ... or 192 where even the backward's 3 workgroups per segment leave the chip under-filled
    assert _abi.plan(1, 12, 2048, 128, 128, torch.bfloat16)[:2] == (192, 11)
    assert _abi.plan(1, 2, 8192, 128, 128, torch.bfloat16)[:2] == (256, 32)   # not for one or two (b, h) pairs
    assert _abi.plan(1, 12, 768, 128, 128, torch.bfloat16)[:2] == (256, 3)    # nor where one launch does the chunk
    # 8 segments of 256 would give the backward 3 * 24 * 8 = 576 workgroups, a few more than fit at once:
    # 7 segments of 320 (the last one 128) keep it to one round
    assert _abi.plan(2, 12, 2048, 128, 128, torch.bfloat16)[:2] == (320, 7)
    # ... and only where the shorter segments do not cost the backward sweep's 3 workgroups per segment another round
    assert _abi.plan(1, 4, 4096, 128, 128, torch.bfloat16)[:2] == (256, 16)   # 22 x 192 would be 264 workgroups
    assert _abi.plan(1, 8, 2048, 128, 128, torch.bfloat16)[:2] == (256, 8)
    assert _abi.plan(1, 6, 4096, 128, 128, torch.bfloat16)[:2] == (192, 22)   # two rounds either way
    # one or two (b, h) pairs and a long chunk: about 2 sqrt(n) tokens per segment (sweeps against scan)
    assert _abi.plan(1, 1, 32768, 128, 128, torch.bfloat16)[:2] == (512, 64)
    assert _abi.plan(1, 1, 131072, 128, 128, torch.bfloat16)[:2] == (1024, 128)
    assert _abi.plan(1, 2, 32768, 128, 128, torch.bfloat16)[:2] == (512, 64)
    assert _abi.plan(1, 1, 16384, 128, 128, torch.bfloat16)[:2] == (256, 64)
    # few segments that fill the chip (to 7/8 and more) are taken up to 2048 tokens, and over two rounds
    assert _abi.plan(1, 64, 8192, 128, 128, torch.bfloat16)[:2] == (2048, 4)
    assert _abi.plan(1, 128, 4096, 128, 128, torch.bfloat16)[:2] == (2048, 2)
    assert _abi.plan(1, 128, 8192, 128, 128, torch.bfloat16)[:2] == (2048, 4)
    assert _abi.plan(1, 52, 8192, 128, 128, torch.bfloat16)[:2] == (1024, 8)   # 208 of 256 CUs: not worth the long walks
    # ragged n: last segment shorter
    assert _abi.plan(1, 1, 300, 64, 32, torch.float32, 64)[:2] == (64, 5)
    assert _abi.plan(1, 1, 300, 64, 32, torch.float32, 64)[2] == 5 * 64 * 32 * 4
    # many heads: one segment covers the chunk
    sl, ns, _ = _abi.plan(8, 128, 4096, 128, 128, torch.bfloat16)
    assert ns == 1 and sl >= 4096


def test_default_plan_of_the_kernels_that_run_two_workgroups_per_cu(lib):
    """fp32 and the generic kernels are bound by arithmetic and share a CU: the default plan gives every CU the
    same number of workgroups (a power-of-two segment length; the expectations are the fastest lengths measured)."""
    from lasp_amd import _abi

    f32 = lambda b, h, n: _abi.plan(b, h, n, 128, 128, torch.float32)[:2]
    assert f32(2, 12, 2048) == (128, 16)       # configuration 0: 384 workgroups
    assert f32(2, 12, 16384) == (512, 32)      # 768 = three per CU; 1024 tokens would leave half the CUs with two
    assert f32(1, 16, 65536) == (2048, 32)     # 512: a one-per-CU plan of 1024 tokens and more is cut in two
    assert f32(1, 32, 16384) == (1024, 16)
    assert f32(1, 4, 8192) == (128, 64)        # exactly one per CU
    assert f32(1, 1, 65536) == (256, 256)
    assert f32(1, 1, 8192) == (64, 128)        # never fills the chip: the shortest segments
    assert f32(1, 16, 1024) == (64, 16)
    assert f32(8, 32, 1024) == (1024, 1)       # one segment per (b, h) already fills it: no pre-pass, no scan
    assert f32(1, 1, 100) == (64, 2)
    # 16-bit shapes that the MFMA kernels do not take (e not a multiple of 8) are planned the same way
    assert _abi.plan(2, 12, 2048, 128, 60, torch.bfloat16)[:2] == (128, 16)
    # an explicit seg_len is taken as given
    assert _abi.plan(2, 12, 2048, 128, 128, torch.float32, 320)[:2] == (320, 7)


def test_plan_rejects_bad_arguments(lib):
    from lasp_amd import _abi

    with pytest.raises(_abi.LaspError, match="unsupported shape"):
        _abi.plan(1, 1, 64, 129, 64, torch.float32)
    with pytest.raises(_abi.LaspError, match="unsupported shape"):
        _abi.plan(1, 1, 0, 64, 64, torch.float32)
    with pytest.raises(_abi.LaspError, match="seg_len"):
        _abi.plan(1, 1, 640, 64, 64, torch.float32, 96)
    rc = lib.lasp_plan(1, 1, 64, 64, 64, 7, 0, None, None, None)
    assert rc == -3 and b"dtype" in lib.lasp_last_error()


def test_kernel_path_selection(lib):
    from lasp_amd import _abi

    assert _abi.kernel_path(1, 16, 65536, 128, 128, torch.bfloat16) == _abi.PATH_MFMA
    assert _abi.kernel_path(1, 16, 65536, 128, 128, torch.float16) == _abi.PATH_MFMA
    assert _abi.kernel_path(1, 16, 65536, 128, 128, torch.float32) == _abi.PATH_MFMA
    assert _abi.kernel_path(1, 16, 65520, 128, 128, torch.float32) == _abi.PATH_MFMA   # ragged: masked tail
    assert _abi.kernel_path(1, 16, 65536, 128, 64, torch.float32) == _abi.PATH_GENERIC
    assert _abi.kernel_path(1, 16, 65500, 128, 128, torch.bfloat16) == _abi.PATH_MFMA
    assert _abi.kernel_path(1, 16, 65536, 64, 128, torch.bfloat16) == _abi.PATH_MFMA    # rows read zero-extended
    assert _abi.kernel_path(1, 16, 65536, 128, 60, torch.bfloat16) == _abi.PATH_GENERIC  # not a multiple of 8
    # short 16-bit chunks under the default plan: one launch per direction, no workspace
    # (few segments: the longest walk over preceding blocks stays within 16 blocks)
    assert _abi.kernel_path(2, 12, 512, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED    # 2 x 256 tokens
    assert _abi.kernel_path(2, 12, 512, 128, 64, torch.float16) == _abi.PATH_MFMA_FUSED
    assert _abi.kernel_path(1, 3, 768, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED     # 3 x 256 tokens
    assert _abi.kernel_path(2, 12, 1024, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED   # 6 x 192 tokens: walks of 15 blocks
    assert _abi.kernel_path(2, 12, 1024, 128, 64, torch.bfloat16) == _abi.PATH_MFMA_FUSED    # narrow rows alike
    assert _abi.kernel_path(4, 32, 2048, 128, 128, torch.bfloat16) == _abi.PATH_MFMA_FUSED   # 2 x 1024 tokens: 16 blocks
    assert _abi.kernel_path(4, 32, 2048 + 8, 128, 128, torch.bfloat16) == _abi.PATH_MFMA     # ragged: 3 segments, 32 blocks
    assert _abi.kernel_path(2, 12, 1536, 128, 128, torch.bfloat16) == _abi.PATH_MFMA         # 6 x 256 tokens: 20 blocks
    assert _abi.kernel_path(2, 12, 2048, 128, 128, torch.bfloat16) == _abi.PATH_MFMA         # 7 x 320 tokens
    assert _abi.kernel_path(2, 12, 512, 128, 128, torch.float32) == _abi.PATH_MFMA
    # a state is stored zero-extended to 128 x 128 on the MFMA path, d x e on the generic one
    assert _abi.plan(1, 2, 256, 64, 128, torch.bfloat16, 256)[2] == 2 * 128 * 128 * 4
    assert _abi.plan(1, 2, 256, 64, 128, torch.float32, 256)[2] == 2 * 64 * 128 * 4


def test_null_and_workspace_errors_need_no_gpu(lib):
    # argument validation happens before any HIP call
    rc = lib.lasp_chunk_fwd(None, None, None, None, None, None, None, None, 1, 1, 64, 64, 64, 0, 0, None)
    assert rc == -1
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    rc = lib.lasp_chunk_fwd(one, one, one, one, None, None, one, None, 1, 1, 1024, 64, 64, 0, 256, None)
    assert rc == -5 and b"seg_states" in lib.lasp_last_error()
    rc = lib.lasp_chunk_bwd(one, one, one, one, one, None, None, one, one, one, None, None, None, 0,
                            1, 1, 1024, 64, 64, 0, 256, None)
    assert rc == -5 and b"workspace" in lib.lasp_last_error()


def test_in_place_state_update_rules(lib):
    """Out == in is taken where one thread (the scan) or one workgroup (a single segment, forward)
    reads the incoming state and writes the outgoing one; elsewhere, and for buffers that merely
    overlap, the call is refused before anything is launched."""
    from lasp_amd import _abi

    bf, f32 = torch.bfloat16, torch.float32
    assert _abi.inplace_ok(2, 12, 2048, 128, 128, bf, 0, False) and _abi.inplace_ok(2, 12, 2048, 128, 128, bf, 0, True)
    assert _abi.kernel_path(1, 2, 512, 128, 128, bf) == _abi.PATH_MFMA_FUSED      # two segments, one launch
    assert not _abi.inplace_ok(1, 2, 512, 128, 128, bf, 0, False) and not _abi.inplace_ok(1, 2, 512, 128, 128, bf, 0, True)
    assert _abi.inplace_ok(1, 2, 512, 128, 128, bf, 64, False)                    # explicit seg_len: 8 segments, scan
    assert not _abi.inplace_ok(2, 12, 1024, 128, 128, bf, 256, False)             # 4 segments: the sweeps gather
    assert _abi.inplace_ok(8, 128, 4096, 128, 128, bf, 0, False)                  # one segment, one workgroup
    assert not _abi.inplace_ok(8, 128, 4096, 128, 128, bf, 0, True)               # dV writes what dK reads
    assert _abi.inplace_ok(1, 2, 512, 128, 128, f32, 0, False) and _abi.inplace_ok(1, 2, 512, 128, 128, f32, 0, True)

    ok, kv = ctypes.c_void_p(4096), ctypes.c_void_p(1 << 20)
    fwd = lambda n, seg, kv_in, kv_out: lib.lasp_chunk_fwd(ok, ok, ok, ok, kv_in, kv_out, ok, ok, 1, 2, n, 128, 128,
                                                           1, seg, None)
    assert fwd(512, 0, kv, kv) == -8 and b"lasp_inplace_ok" in lib.lasp_last_error()
    assert fwd(512, 64, kv, ctypes.c_void_p((1 << 20) + 64)) == -8 and b"overlaps" in lib.lasp_last_error()
    assert fwd(512, 64, kv, kv) == -7   # accepted as far as aliasing goes: the next check (device) is what stops it here
    bwd = lambda n, seg: lib.lasp_chunk_bwd(ok, ok, ok, ok, ok, None, kv, ok, ok, ok, kv, None, ok, 1 << 30, 1, 2, n,
                                            128, 128, 1, seg, None)
    assert bwd(512, 0) == -8 and b"dkv_out is dkv_in" in lib.lasp_last_error()
    assert bwd(512, 64) == -7


def test_documented_launch_shims_run_as_written(lib, monkeypatch):
    """The reference-side binding that the integration notes at the repository root show (their python blocks,
    executed as they stand) must get past the library's argument checks on the reference's own per-rank test shape, n = 512, where the kernels
    cannot update a state in place: with host tensors the call that stops it is the device check, not
    LASP_E_ALIAS."""
    import contextlib
    import types

    from lasp_amd import _abi

    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = [b for b in re.findall(r"```python\n(.*?)```", text, flags=re.S) if "_lib" in b or "_plan(" in b]
    assert len(blocks) == 3, "expected the binding, lasp_forward and lasp_backward blocks"
    code = "\n".join(blocks).replace("/path/to/lasp_amd/liblasp_hip.so", _abi.lib_path())
    monkeypatch.setattr(torch.cuda, "device", lambda idx: contextlib.nullcontext())
    monkeypatch.setattr(torch.cuda, "current_stream", lambda *a: types.SimpleNamespace(cuda_stream=0))
    ns = {}
    exec(compile(code, "INTEGRATION.md", "exec"), ns)

    b, h, n, d = 2, 12, 512, 128
    assert not _abi.inplace_ok(b, h, n, d, d, torch.bfloat16, ns["_plan"](torch.empty(b, h, n, d, dtype=torch.bfloat16),
                                                                          torch.empty(b, h, n, d))[0], False)
    q, k, v, do = [torch.zeros(b, h, n, d, dtype=torch.bfloat16) for _ in range(4)]
    s = torch.ones(h)
    KV, DKV = torch.zeros(b, h, d, d), torch.zeros(b, h, d, d)
    with pytest.raises(RuntimeError, match="not a device pointer|current device"):
        ns["lasp_forward"](q, k, v, s, KV)
    with pytest.raises(RuntimeError, match="not a device pointer|current device"):
        ns["lasp_backward"](q, k, v, s, do, KV.clone(), DKV)
    # the same calls with the state buffer on both sides are what the library refuses
    seg, _ = ns["_plan"](q, v)
    rc = ns["_lib"].lasp_chunk_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), KV.data_ptr(), KV.data_ptr(),
                                   q.data_ptr(), k.data_ptr(), b, h, n, d, d, 1, seg, None)
    assert rc == -8


def test_alignment_and_device_errors_need_no_gpu(lib):
    """A misaligned tensor or state pointer is LASP_E_ALIGN; a pointer HIP does not know as memory of
    the current device is LASP_E_DEVICE.  Both are reported before anything is launched."""
    ok, odd16, odd4 = ctypes.c_void_p(4096), ctypes.c_void_p(4096 + 8), ctypes.c_void_p(4096 + 2)
    fwd = lambda q=ok, o=ok, kv=None, ws=ok: lib.lasp_chunk_fwd(q, ok, ok, ok, kv, None, o, ws, 1, 1, 1024, 128,
                                                                 128, 1, 256, None)
    assert fwd(q=odd16) == -6 and b"q" in lib.lasp_last_error() and b"16" in lib.lasp_last_error()
    assert fwd(o=odd16) == -6 and b" o " in lib.lasp_last_error()
    assert fwd(kv=odd4) == -6 and b"kv_in" in lib.lasp_last_error()
    bwd = lambda dq=ok, dkv=None: lib.lasp_chunk_bwd(ok, ok, ok, ok, ok, None, dkv, dq, ok, ok, None, None, ok,
                                                     1 << 30, 1, 1, 1024, 128, 128, 1, 256, None)
    assert bwd(dq=odd16) == -6 and b"dq" in lib.lasp_last_error()
    assert bwd(dkv=odd4) == -6 and b"dkv_in" in lib.lasp_last_error()
    # well-aligned but not device memory (no GPU here, or a made-up address on a GPU box)
    assert fwd() == -7 and b"q" in lib.lasp_last_error()
    assert bwd() == -7


def test_static_scratch_entry_rejects_oversized_calls_without_a_gpu(lib):
    ok = ctypes.c_void_p(4096)
    # b*h*n_seg = 16 * 64 states of 64 KiB = 64 MiB > the 32 MiB scratch
    rc = lib.lasp_chunk_fwd_static(ok, ok, ok, ok, None, None, ok, 1, 16, 65536, 128, 128, 1, 1024, None)
    assert rc == -5 and b"scratch holds" in lib.lasp_last_error()
    assert lib.lasp_chunk_fwd_static(None, ok, ok, ok, None, None, ok, 1, 1, 64, 128, 128, 1, 0, None) == -1


def test_product_path_refuses_cpu_tensors(lib):
    import lasp_amd
    from lasp_amd import _abi

    x = torch.zeros(1, 1, 64, 64)
    with pytest.raises(_abi.LaspError, match="ROCm devices only"):
        lasp_amd.lightning_attn(x, x, x, torch.ones(1))


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "lasp_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


def test_bench_reads_its_traffic_figures_from_the_committed_profile():
    """bench.py's roofline.traffic comes from profiles/pmc_hbm_bytes_config2.txt, not from constants in the
    script: the file parses, names the segment plan the library still chooses for the headline shape, and its
    figures are at least the algorithmic bytes of each kernel."""
    import sys

    sys.path.insert(0, ROOT)
    import bench
    from lasp_amd import _abi

    prof = bench.read_traffic_profile()
    assert prof is not None, "profiles/pmc_hbm_bytes_config2.txt is missing or has no plan/scale/traffic lines"
    assert (prof["seg_len"], prof["n_seg"]) == _abi.plan(bench.B, bench.H, bench.N, bench.D, bench.D, torch.bfloat16)[:2]
    th = bench.B * bench.H * bench.N
    assert prof["kernels"]["la_bwd3"] >= bench.BYTES_BWD_PER_TH * th
    assert prof["kernels"]["la_apply"] >= bench.BYTES_FWD_PER_TH * th
    assert prof["kernels"]["la_bwd3"] < 2 * bench.BYTES_BWD_PER_TH * th


def test_plan_invariants_on_random_shapes(lib):
    """The plan is what forward and backward agree on: for any shape the default plan must be reproduced by
    asking for its seg_len explicitly (the binding hands the planned seg_len to both calls), segments are
    whole blocks that cover the chunk, and the workspace holds a whole number of states, at least one per
    segment."""
    import random

    from lasp_amd import _abi

    rng = random.Random(7)
    for _ in range(3000):
        b = rng.choice([1, 1, 2, 3, 4, 8])
        h = rng.choice([1, 2, 3, 7, 8, 12, 16, 20, 24, 28, 32, 40, 48, 52, 64, 96, 100, 128, 200])
        n = rng.choice([1, 63, 64, 65, 500, 512, 1000, 2048, 2049, 4096, 5000, 8192, 16384, 20000, 32768, 65536,
                        65544, 100000, 1 << 20]) + rng.choice([0, 0, 0, -8, 8, 72])
        n = max(n, 1)
        dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        d, e = rng.choice([(128, 128), (128, 128), (128, 64), (64, 128), (96, 40), (64, 64)])
        seg_len, n_seg, state_bytes = _abi.plan(b, h, n, d, e, dtype)
        assert seg_len > 0 and seg_len % 64 == 0 and n_seg == -(-n // seg_len), (b, h, n, d, e, dtype, seg_len, n_seg)
        padded = (dtype != torch.float32 and d % 8 == 0 and e % 8 == 0) or (dtype == torch.float32 and d == e == 128)
        one = (128 * 128 if padded else d * e) * 4
        states, rest = divmod(state_bytes, b * h * one)
        assert rest == 0 and n_seg <= states <= 64 * n_seg, (b, h, n, d, e, dtype, seg_len, n_seg, state_bytes)
        if _abi.kernel_path(b, h, n, d, e, dtype) != _abi.PATH_MFMA_FUSED:
            assert _abi.plan(b, h, n, d, e, dtype, seg_len) == (seg_len, n_seg, state_bytes), (b, h, n, d, e, dtype)
