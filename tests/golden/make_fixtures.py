"""Writes the committed parity fixtures (inputs and expected outputs) from the CPU oracle.

    python tests/golden/make_fixtures.py

The reference holds no golden vectors for this path (its test prints unseeded
statistics), so these come from the oracle's closed form in float64
(oracle/lasp_oracle.py: ref_quadratic), which tests/test_oracle.py pins against
independent statements of the same mathematics.  Files are plain .npz arrays.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import lasp_oracle as O  # noqa: E402


def make(name, b, h, n, d, e, dtype, seed, slopes):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = [torch.randn(b, h, n, x, generator=g).to(dtype) for x in (d, d, e, e)]
    kv = torch.randn(b, h, d, e, generator=g) * 0.5
    dkv = torch.randn(b, h, d, e, generator=g) * 0.5
    s = torch.tensor(slopes, dtype=torch.float32)
    ref = O.ref_quadratic(q, k, v, s, do, kv, dkv)

    def store(t):
        if t.dtype == torch.bfloat16:
            return t.view(torch.int16).numpy()  # raw bf16 bits
        return t.numpy()

    arrays = dict(q=store(q), k=store(k), v=store(v), do=store(do), kv=kv.numpy(), dkv=dkv.numpy(), s=s.numpy(),
                  io_dtype=np.array(str(dtype)))
    for key, val in ref.items():
        arrays["ref_" + key] = val.to(torch.float32).numpy()
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **arrays)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    # fp32 I/O, ragged n (not a multiple of any block size), e != d
    make("generic_f32_b1_h2_n150_d32_e16", 1, 2, 150, 32, 16, torch.float32, 101, [0.25, 0.02])
    # bf16 I/O on the MFMA shape, two blocks
    make("mfma_bf16_b1_h1_n128_d128_e128", 1, 1, 128, 128, 128, torch.bfloat16, 102, [0.0625])
    # bf16 I/O with narrow value rows (the reference's own test has e = 64) and a ragged length
    make("mfma_bf16_b1_h2_n100_d128_e64", 1, 2, 100, 128, 64, torch.bfloat16, 103, [0.5, 0.0039])
    # fp32 I/O on the fp32 MFMA shape, ragged length
    make("mfma_f32_b1_h1_n80_d128_e128", 1, 1, 80, 128, 128, torch.float32, 104, [0.125])
