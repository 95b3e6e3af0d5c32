#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

One step = forward + backward of causal decayed linear attention through the
public operator (lightning_attn + autograd) on the headline workload (TNL-1B head shape):
b=1, h=16, n=65536, d=e=128, bf16, Q/K/V/dO ~ N(0,1)/sqrt(d), slopes
2^(-8(i+1)/16); inputs are resident in HBM before the timed region.
Prints ONE JSON line (metric = fwd+bwd tokens/s) that also carries
  roofline     -- la_bwd3, the dominant kernel, against the HBM roof: algorithmic
                  bytes per launch / its mean launch duration (HIP events around
                  every launch, on the launch stream); roofline_fwd: the same for la_apply
  cpu_baseline -- the CPU oracle (fp32 torch port of the same recurrence) timed on
                  the host cores on one pass of the same workload.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

B, H, N, D = 1, 16, 65536, 128
FLOP_FWD_PER_TH = 98304        # 2Bd + 2Be + 4de at B=64, d=e=128
FLOP_BWD_PER_TH = 245760       # 6Bd + 4Be + 10de
BYTES_FWD_PER_TH = 1024        # read Q,K,V + write O, bf16
BYTES_BWD_PER_TH = 1792        # read Q,K,V,dO + write dQ,dK,dV
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this workload
# (profiles/pmc_hbm_bytes_config2.txt); FETCH_SIZE is scaled by 2.0 and WRITE_SIZE by 1.0, the
# factors a plain 1 GiB device copy shows for the same counters.
TRAFFIC_BWD3_BYTES = 2708338 * 1024   # 2 x 960 953 KiB fetched + 786 432 KiB written
TRAFFIC_APPLY_BYTES = 1081509 * 1024  # 2 x 409 683 KiB fetched + 262 144 KiB written
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def slopes(h):
    return torch.tensor([2.0 ** (-8.0 * (i + 1) / h) for i in range(h)], dtype=torch.float32).reshape(h, 1, 1)


def make_inputs(device, n=N, seed=2):
    g = torch.Generator().manual_seed(seed)
    mk = lambda: (torch.randn(B, H, n, D, generator=g) / D ** 0.5).to(torch.bfloat16)
    q, k, v, do = mk(), mk(), mk(), mk()
    return [t.to(device) for t in (q, k, v, do)]


def cpu_baseline():
    """Oracle port (oracle/lasp_oracle.py: ref_chunked, fp32, block 64) on all host cores."""
    from oracle import lasp_oracle as O

    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    cores = min(cores, os.cpu_count() or cores)
    torch.set_num_threads(cores)
    q, k, v, do = [t.float() for t in make_inputs("cpu")]
    s = slopes(H)
    O.ref_chunked(q[:, :, :1024], k[:, :, :1024], v[:, :, :1024], s, do[:, :, :1024])  # warm the thread pool
    passes, t0 = 0, time.perf_counter()
    while True:  # about 10 s of CPU work
        O.ref_chunked(q, k, v, s, do, block=64, dtype=torch.float32)
        passes += 1
        if time.perf_counter() - t0 >= 10.0 or passes >= 16:
            break
    dt = (time.perf_counter() - t0) / passes
    return {
        "value": B * N / dt,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{passes} fwd+bwd passes of the full workload (b={B} h={H} n={N} d={D}), fp32 torch, {dt:.2f} s each",
        "gflops": (FLOP_FWD_PER_TH + FLOP_BWD_PER_TH) * B * H * N / dt / 1e9,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (reference point for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    import lasp_amd
    from lasp_amd import _abi

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    q, k, v, do = make_inputs(dev)
    q.requires_grad_(True)
    k.requires_grad_(True)
    v.requires_grad_(True)
    s = slopes(H).to(dev)
    assert _abi.kernel_path(B, H, N, D, D, torch.bfloat16) == _abi.PATH_MFMA
    seg_len, n_seg, _ = _abi.plan(B, H, N, D, D, torch.bfloat16)

    if args.copy_calibration:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).fill_(1.0)  # 1 GiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def step():
        q.grad = k.grad = v.grad = None
        o = lasp_amd.lightning_attn(q, k, v, s)
        o.backward(do)

    def fwd_only():
        with torch.no_grad():
            lasp_amd.lightning_attn(q, k, v, s)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt / args.steps * 1e3

    # forward alone
    fwd_only()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fwd_only()
    torch.cuda.synchronize()
    ms_fwd = (time.perf_counter() - t0) / args.steps * 1e3

    # per-kernel durations: the same K steps again with every launch bracketed by events
    _abi.profile_begin(16 * args.steps + 16)
    for _ in range(args.steps):
        step()
    prof = _abi.profile_end()
    th = B * H * N

    def roof(kernel, cls, alg_bytes, traffic):
        ms, cnt = prof[cls]
        avg_ms = ms / max(cnt, 1)
        achieved = alg_bytes / (avg_ms * 1e-3) / 1e9
        return {
            "kernel": kernel, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
            "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_ms": avg_ms, "launches": cnt,
        }

    flop_step = (FLOP_FWD_PER_TH + FLOP_BWD_PER_TH) * th
    tflops = flop_step / (ms_step * 1e-3) / 1e12

    out = {
        "metric": "fwd+bwd tokens/s, causal decayed linear attention, h=16 d=128 n=64K, 1 MI355X",
        "value": B * N / (ms_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "TNL-1B attention head shape: lightning_attn fwd+bwd, b=1 h=16 n=65536 d=e=128, single pass, no KV state",
            "seg_len": seg_len,
            "n_seg": n_seg,
        },
        "fwd_ms": ms_fwd,
        "fwd_tokens_per_s": B * N / (ms_fwd * 1e-3),
        "fwd_tflops": FLOP_FWD_PER_TH * th / (ms_fwd * 1e-3) / 1e12,
        "fwd_bwd_tflops": tflops,
        "frac_bf16_mfma_peak": tflops / MFMA_BF16_PEAK_TFLOPS,
        "step_algorithmic_gbs": (BYTES_FWD_PER_TH + BYTES_BWD_PER_TH) * th / (ms_step * 1e-3) / 1e9,
        "kernel_ms": {name: {"total_ms": ms, "launches": cnt} for name, (ms, cnt) in prof.items() if cnt},
        # dominant kernel: la_bwd3 (one launch = the whole backward sweep: reads Q,K,V,dO, writes dQ,dK,dV)
        "roofline": roof("la_bwd3", "bwd3", BYTES_BWD_PER_TH * th, TRAFFIC_BWD3_BYTES),
        # second kernel: la_apply (one launch = the forward sweep: reads Q,K,V, writes O)
        "roofline_fwd": roof("la_apply", "apply", BYTES_FWD_PER_TH * th, TRAFFIC_APPLY_BYTES),
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
