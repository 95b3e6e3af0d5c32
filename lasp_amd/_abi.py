"""ctypes binding of liblasp_hip.so (the C ABI declared in include/lasp_hip.h).

The library is the only compute path of this package: if it is missing, or a
tensor is not on a ROCm device, the calls raise -- there is no CPU or eager
fallback.  Tensors are borrowed as raw device pointers; outputs and workspaces
come from torch's caching allocator, and work is enqueued on torch's current
stream, like the Triton launches it replaces
(lasp/lightning_attention.py:414-429, lasp/lasp_fuse.py:380-399,438-461).
"""
from __future__ import annotations

import ctypes
import functools
import os
from typing import Optional, Tuple

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "liblasp_hip.so")
_lib = None

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
PATH_GENERIC, PATH_MFMA, PATH_MFMA_FUSED = 0, 1, 2

_c_void_p = ctypes.c_void_p
_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64
_c_size = ctypes.c_size_t


class LaspError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise LaspError(
            f"{_LIB_PATH} is missing: build it with `python -m lasp_amd.build` "
            "(hipcc --offload-arch=gfx950); lasp_amd has no fallback path"
        )
    lib = ctypes.CDLL(_LIB_PATH)
    lib.lasp_abi_version.restype = _c_int
    lib.lasp_abi_version.argtypes = []
    lib.lasp_last_error.restype = ctypes.c_char_p
    lib.lasp_last_error.argtypes = []
    lib.lasp_plan.restype = _c_int
    lib.lasp_plan.argtypes = [_c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int,
                              ctypes.POINTER(_c_int), ctypes.POINTER(_c_int), ctypes.POINTER(_c_size)]
    lib.lasp_kernel_path.restype = _c_int
    lib.lasp_kernel_path.argtypes = [_c_int, _c_int, _c_i64, _c_int, _c_int, _c_int]
    lib.lasp_inplace_ok.restype = _c_int
    lib.lasp_inplace_ok.argtypes = [_c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int]
    lib.lasp_chunk_fwd.restype = _c_int
    lib.lasp_chunk_fwd.argtypes = [_c_void_p] * 8 + [_c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_void_p]
    lib.lasp_chunk_fwd_static.restype = _c_int
    lib.lasp_chunk_fwd_static.argtypes = [_c_void_p] * 7 + [_c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_void_p]
    lib.lasp_chunk_bwd.restype = _c_int
    lib.lasp_chunk_bwd.argtypes = [_c_void_p] * 13 + [_c_size, _c_int, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_void_p]
    lib.lasp_profile_begin.restype = _c_int
    lib.lasp_profile_begin.argtypes = [_c_int]
    lib.lasp_profile_end.restype = _c_int
    lib.lasp_profile_end.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_c_int)]
    lib.lasp_stream_probe.restype = _c_int
    lib.lasp_stream_probe.argtypes = [ctypes.POINTER(_c_void_p), _c_int, ctypes.POINTER(_c_void_p), _c_int, _c_size,
                                      _c_int, _c_void_p]
    if lib.lasp_abi_version() != 1:
        raise LaspError(f"ABI version mismatch: library reports {lib.lasp_abi_version()}, binding expects 1")
    _lib = lib
    return lib


def _raise(rc: int, what: str):
    msg = load().lasp_last_error().decode("utf-8", "replace")
    raise LaspError(f"{what} failed (code {rc}): {msg}")


def _raw_stream(dev) -> int:
    """hipStream_t of torch's current stream on `dev`, as an integer (no Stream object is built on the way)."""
    return torch._C._cuda_getCurrentRawStream(dev.index)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _check_dev(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise LaspError("lasp_amd runs on ROCm devices only; got a tensor on " + str(t.device))
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise LaspError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _check_state(name, t, b, h, d, e):
    if t is None:
        return
    if t.dtype != torch.float32 or tuple(t.shape) != (b, h, d, e) or not t.is_contiguous():
        raise LaspError(f"{name} must be a contiguous float32 tensor of shape {(b, h, d, e)}, "
                        f"got {t.dtype} {tuple(t.shape)}")


@functools.lru_cache(maxsize=256)
def plan(b: int, h: int, n: int, d: int, e: int, dtype: torch.dtype, seg_len: int = 0) -> Tuple[int, int, int]:
    """(seg_len, n_seg, bytes of one segment-state array) for a shape (a pure function of its arguments)."""
    lib = load()
    sl, ns, sb = _c_int(0), _c_int(0), _c_size(0)
    rc = lib.lasp_plan(b, h, n, d, e, DTYPE_CODE[dtype], seg_len, ctypes.byref(sl), ctypes.byref(ns), ctypes.byref(sb))
    if rc:
        _raise(rc, "lasp_plan")
    return sl.value, ns.value, sb.value


@functools.lru_cache(maxsize=256)
def kernel_path(b, h, n, d, e, dtype) -> int:
    """PATH_* a shape runs on when it is given to the library with the default plan (seg_len = 0)."""
    rc = load().lasp_kernel_path(b, h, n, d, e, DTYPE_CODE[dtype])
    if rc < 0:
        _raise(rc, "lasp_kernel_path")
    return rc


@functools.lru_cache(maxsize=256)
def inplace_ok(b, h, n, d, e, dtype, seg_len: int, backward: bool) -> bool:
    """Whether this call may write its outgoing state over the incoming one (lasp_inplace_ok)."""
    rc = load().lasp_inplace_ok(b, h, n, d, e, DTYPE_CODE[dtype], seg_len, int(backward))
    if rc < 0:
        _raise(rc, "lasp_inplace_ok")
    return bool(rc)


def _private_incoming(state_in, state_out, shape_key, seg_len, backward):
    """`state_in`, or a copy of it when `state_out` is the same memory and the kernels this shape runs
    on cannot update a state in place (the copy then plays the reference's in-place update)."""
    if state_in is None or state_out is None or state_in.data_ptr() != state_out.data_ptr():
        return state_in
    return state_in if inplace_ok(*shape_key, seg_len, backward) else state_in.clone()


KERNEL_CLASSES = ("apply", "state", "scan", "generic", "bwd3", "fused")


def profile_begin(max_launches: int = 4096) -> None:
    """Starts bracketing every kernel launch of the library with HIP events."""
    rc = load().lasp_profile_begin(max_launches)
    if rc:
        _raise(rc, "lasp_profile_begin")


def profile_end() -> dict:
    """Waits for the bracketed launches; {class: (total_ms, launches)}."""
    ms = (ctypes.c_double * len(KERNEL_CLASSES))()
    cnt = (_c_int * len(KERNEL_CLASSES))()
    rc = load().lasp_profile_end(ms, cnt)
    if rc:
        _raise(rc, "lasp_profile_end")
    return {name: (ms[i], cnt[i]) for i, name in enumerate(KERNEL_CLASSES)}


def stream_probe(reads, writes, grid: int) -> None:
    """Enqueues one launch of the streaming probe (lasp_stream_probe) on torch's current stream: every tensor
    of `reads` is read once and every tensor of `writes` written once; all must have the same byte size."""
    lib = load()
    sizes = {t.numel() * t.element_size() for t in (*reads, *writes)}
    if len(sizes) != 1:
        raise LaspError(f"the probe's streams must all have the same size, got {sorted(sizes)}")
    dev = _check_dev(*reads, *writes)
    rd = (_c_void_p * max(len(reads), 1))(*[t.data_ptr() for t in reads])
    wr = (_c_void_p * max(len(writes), 1))(*[t.data_ptr() for t in writes])
    rc = lib.lasp_stream_probe(rd, len(reads), wr, len(writes), sizes.pop(), grid,
                               _raw_stream(dev))
    if rc:
        _raise(rc, "lasp_stream_probe")


def _shapes(q, k, v):
    if q.dim() != 4 or k.shape != q.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise LaspError(f"expected q,k (b,h,n,d) and v (b,h,n,e); got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    if q.dtype not in DTYPE_CODE or k.dtype != q.dtype or v.dtype != q.dtype:
        raise LaspError(f"q, k, v must share one of float32/bfloat16/float16; got {q.dtype}, {k.dtype}, {v.dtype}")
    b, h, n, d = q.shape
    return b, h, n, d, v.shape[-1]


def _slopes(s: torch.Tensor, h: int, dev) -> torch.Tensor:
    if s.numel() != h:
        raise LaspError(f"need {h} slopes, got a tensor with {s.numel()} elements")
    if s.dtype == torch.float32 and s.device == dev and s.is_contiguous():
        return s  # the usual case costs nothing; data_ptr() does not care about autograd
    return s.detach().to(device=dev, dtype=torch.float32).contiguous()


class _on_device:
    """`with torch.cuda.device(dev)` only when dev is not already current (backward runs on autograd's
    thread, which PyTorch has already switched to the right device)."""

    __slots__ = ("guard",)

    def __init__(self, dev):
        self.guard = None if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _chunk_fwd_exact(q, k, v, s, kv_in=None, kv_out=None, seg_len: int = 0):
    """Enqueues the forward of one chunk.  Returns (o, seg_states, seg_len).

    seg_states is the float32 array of states entering each segment, sized by
    lasp_plan (None when the call needed none); pass it to chunk_bwd to skip the
    recompute.
    """
    lib = load()
    dev = _check_dev(q, k, v, kv_in, kv_out)
    b, h, n, d, e = _shapes(q, k, v)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    s = _slopes(s, h, dev)
    _check_state("kv_in", kv_in, b, h, d, e)
    _check_state("kv_out", kv_out, b, h, d, e)
    # short chunks under the default plan run as one launch that needs no workspace and leaves no
    # segment states; seg_len stays 0 so that the backward makes the same choice
    fused = seg_len == 0 and kernel_path(b, h, n, d, e, q.dtype) == PATH_MFMA_FUSED
    if not fused:
        seg_len, n_seg, state_bytes = plan(b, h, n, d, e, q.dtype, seg_len)
    with _on_device(dev):
        kv_in = _private_incoming(kv_in, kv_out, (b, h, n, d, e, q.dtype), seg_len, False)
        o = torch.empty((b, h, n, e), dtype=q.dtype, device=dev)
        states = None
        if not fused and (n_seg > 1 or kv_in is not None or kv_out is not None):
            # the library decides how many states it keeps (one per segment, or per piece of a long segment)
            # and how each is stored (d x e, or zero-extended to 128 x 128): the array is opaque here
            states = torch.empty((state_bytes // 4,), dtype=torch.float32, device=dev)
        rc = lib.lasp_chunk_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), _ptr(kv_in), _ptr(kv_out),
                                o.data_ptr(), _ptr(states), b, h, n, d, e, DTYPE_CODE[q.dtype], seg_len,
                                _raw_stream(dev))
    if rc:
        _raise(rc, "lasp_chunk_fwd")
    return o, states, seg_len


STATIC_SCRATCH_BYTES = 32 << 20


def chunk_fwd_static(q, k, v, s, o, kv_in=None, kv_out=None, seg_len: int = 0) -> None:
    """Forward of one chunk into the caller's `o`, allocating nothing (lasp_chunk_fwd_static).

    For code that must not allocate device memory around the call (graph capture, serving loops):
    the segment states live in a scratch array inside the library, which limits the call to
    STATIC_SCRATCH_BYTES of states (see `plan`) and means calls that overlap in time on one GPU
    race.  Every tensor must already be contiguous and on the current device; s must be float32.
    """
    lib = load()
    dev = _check_dev(q, k, v, o, s, kv_in, kv_out)
    b, h, n, d, e = _shapes(q, k, v)
    if o.shape != v.shape or o.dtype != q.dtype:
        raise LaspError(f"o must match v: {tuple(o.shape)} {o.dtype} vs {tuple(v.shape)} {q.dtype}")
    if s.dtype != torch.float32 or s.numel() != h:
        raise LaspError(f"s must hold {h} float32 slopes, got {s.dtype} with {s.numel()} elements")
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o), ("s", s)):
        if not t.is_contiguous():
            raise LaspError(f"{name} must be contiguous (this call makes no copies)")
    _check_state("kv_in", kv_in, b, h, d, e)
    _check_state("kv_out", kv_out, b, h, d, e)
    rc = lib.lasp_chunk_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), _ptr(kv_in), _ptr(kv_out),
                                   o.data_ptr(), b, h, n, d, e, DTYPE_CODE[q.dtype], seg_len,
                                   _raw_stream(dev))
    if rc:
        _raise(rc, "lasp_chunk_fwd_static")


def _chunk_bwd_exact(q, k, v, s, do, kv_in=None, dkv_in=None, dkv_out=None, kv_seg_states=None, seg_len: int = 0):
    """Enqueues the backward of one chunk.  Returns (dq, dk, dv)."""
    lib = load()
    dev = _check_dev(q, k, v, do, kv_in, dkv_in, dkv_out, kv_seg_states)
    b, h, n, d, e = _shapes(q, k, v)
    if do.shape != v.shape or do.dtype != q.dtype:
        raise LaspError(f"do must match v: {tuple(do.shape)} {do.dtype} vs {tuple(v.shape)} {q.dtype}")
    q, k, v, do = q.contiguous(), k.contiguous(), v.contiguous(), do.contiguous()
    s = _slopes(s, h, dev)
    _check_state("kv_in", kv_in, b, h, d, e)
    _check_state("dkv_in", dkv_in, b, h, d, e)
    _check_state("dkv_out", dkv_out, b, h, d, e)
    fused = seg_len == 0 and kernel_path(b, h, n, d, e, q.dtype) == PATH_MFMA_FUSED
    if fused:
        n_seg, state_bytes, kv_seg_states = 1, 0, None  # one launch, no workspace, no use for cached states
    else:
        seg_len, n_seg, state_bytes = plan(b, h, n, d, e, q.dtype, seg_len)
    if kv_seg_states is not None:
        if (kv_seg_states.dtype != torch.float32 or kv_seg_states.numel() * 4 != state_bytes
                or not kv_seg_states.is_contiguous()):
            raise LaspError(f"kv_seg_states must be the contiguous float32 array of {state_bytes} bytes that "
                            f"chunk_fwd returned for this shape, got {kv_seg_states.dtype} "
                            f"{tuple(kv_seg_states.shape)}")
    with _on_device(dev):
        dkv_in = _private_incoming(dkv_in, dkv_out, (b, h, n, d, e, q.dtype), 0 if fused else seg_len, True)
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        # one state array for the dKV scan, one more when the KV states have to be rebuilt
        need_dkv = not fused and (n_seg > 1 or dkv_in is not None or dkv_out is not None)
        need_kv = not fused and kv_seg_states is None and (n_seg > 1 or kv_in is not None)
        n_arrays = int(need_dkv) + int(need_kv)
        ws = torch.empty((n_arrays * state_bytes // 4,), dtype=torch.float32, device=dev) if n_arrays else None
        rc = lib.lasp_chunk_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr(), do.data_ptr(), _ptr(kv_in),
                                _ptr(dkv_in), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), _ptr(dkv_out),
                                _ptr(kv_seg_states), _ptr(ws), n_arrays * state_bytes, b, h, n, d, e,
                                DTYPE_CODE[q.dtype], seg_len, _raw_stream(dev))
    if rc:
        _raise(rc, "lasp_chunk_bwd")
    return dq, dk, dv


# ---------------------------------------------------------------------------------------
# Narrow heads on the MFMA kernels.  The 16-bit MFMA kernels read rows of d, e <= 128 features
# zero-extended when d and e are multiples of 8 (the reference's own test uses e = 64,
# tests/test.py:95); the fp32 MFMA kernels take d = e = 128 only.  Any other narrow shape is
# zero-padded to 128 here: zero feature columns add nothing to q.k, to the outputs or to the
# states, so the results are exact, and the call runs an order of magnitude faster than on
# the generic fp32-FMA kernels.  Everything else goes to the library unchanged.
_MFMA_F = 128


def _pad_to_mfma(q, v) -> bool:
    d, e = q.shape[3], v.shape[3]
    if q.dtype not in DTYPE_CODE or d > _MFMA_F or e > _MFMA_F or (d == _MFMA_F and e == _MFMA_F):
        return False
    return q.dtype == torch.float32 or d % 8 != 0 or e % 8 != 0


def _pad_last(t, size):
    return t if t.shape[-1] == size else torch.nn.functional.pad(t, (0, size - t.shape[-1]))


def _pad_state(t, d, e):
    if t is None:
        return None
    out = torch.zeros(t.shape[0], t.shape[1], _MFMA_F, _MFMA_F, dtype=torch.float32, device=t.device)
    out[:, :, :d, :e] = t
    return out


def chunk_fwd(q, k, v, s, kv_in=None, kv_out=None, seg_len: int = 0):
    """Forward of one chunk: (o, seg_states, seg_len).  See _chunk_fwd_exact; narrow heads are padded."""
    if q.dim() != 4 or v.dim() != 4 or not _pad_to_mfma(q, v):
        return _chunk_fwd_exact(q, k, v, s, kv_in, kv_out, seg_len)
    b, h, n, d, e = _shapes(q, k, v)
    _check_state("kv_in", kv_in, b, h, d, e)
    _check_state("kv_out", kv_out, b, h, d, e)
    kv_out_p = None if kv_out is None else torch.empty(b, h, _MFMA_F, _MFMA_F, dtype=torch.float32, device=q.device)
    o, states, seg_len = _chunk_fwd_exact(_pad_last(q, _MFMA_F), _pad_last(k, _MFMA_F), _pad_last(v, _MFMA_F), s,
                                          _pad_state(kv_in, d, e), kv_out_p, seg_len)
    if kv_out is not None:
        kv_out.copy_(kv_out_p[:, :, :d, :e])
    return o[..., :e].contiguous(), states, seg_len


def chunk_bwd(q, k, v, s, do, kv_in=None, dkv_in=None, dkv_out=None, kv_seg_states=None, seg_len: int = 0):
    """Backward of one chunk: (dq, dk, dv).  See _chunk_bwd_exact; narrow heads are padded
    (kv_seg_states must then be what chunk_fwd returned for the same call)."""
    if q.dim() != 4 or v.dim() != 4 or not _pad_to_mfma(q, v):
        return _chunk_bwd_exact(q, k, v, s, do, kv_in, dkv_in, dkv_out, kv_seg_states, seg_len)
    b, h, n, d, e = _shapes(q, k, v)
    _check_state("kv_in", kv_in, b, h, d, e)
    _check_state("dkv_in", dkv_in, b, h, d, e)
    _check_state("dkv_out", dkv_out, b, h, d, e)
    dkv_out_p = None if dkv_out is None else torch.empty(b, h, _MFMA_F, _MFMA_F, dtype=torch.float32, device=q.device)
    dq, dk, dv = _chunk_bwd_exact(_pad_last(q, _MFMA_F), _pad_last(k, _MFMA_F), _pad_last(v, _MFMA_F), s,
                                  _pad_last(do, _MFMA_F), _pad_state(kv_in, d, e), _pad_state(dkv_in, d, e),
                                  dkv_out_p, kv_seg_states, seg_len)
    if dkv_out is not None:
        dkv_out.copy_(dkv_out_p[:, :, :d, :e])
    return dq[..., :d].contiguous(), dk[..., :d].contiguous(), dv[..., :e].contiguous()
