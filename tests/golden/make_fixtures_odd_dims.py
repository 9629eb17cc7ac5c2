#!/usr/bin/env python3
"""Write tests/golden/odd_dims.npz: MSECompressor round trips of the upstream Python reference at head dimensions that
are not a multiple of 32, among them ones whose codes do not fill a whole number of bytes (idx_pad != 0,
compressors_v3.py:64-68 and :101-102), which no other fixture reaches.

Run once, in the build container, where the reference checkout is mounted read-only at /root/reference (override
with TQ_REFERENCE_ROOT):

    python tests/golden/make_fixtures_odd_dims.py

Inputs and outputs are stored as plain numpy arrays (no pickles); bf16 / fp16 tensors as their uint16 bit patterns.
Nothing of the reference's text is stored.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF_ROOT = os.environ.get("TQ_REFERENCE_ROOT", "/root/reference")
sys.path.insert(0, HERE)
from make_fixtures import bits16, outlier_kv  # noqa: E402

# (head_dim, bits): 45 is odd (2-byte aligned bf16 vectors, idx_pad 3 / 1 / 1), 100 at 1 bit leaves idx_pad 4,
# 80 / 112 / 200 are the multiples of 8 that models use
CASES = ((45, 2), (45, 3), (45, 4), (80, 2), (80, 4), (100, 1), (100, 3), (112, 4), (200, 2))


def main():
    sys.path.insert(0, REF_ROOT)
    from turboquant.compressors_v3 import MSECompressor

    torch.set_num_threads(1)
    out = {}
    dts = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    for d, b in CASES:
        comp = MSECompressor(d, b, seed=7 * d + b)
        out[f"Pi_d{d}_b{b}"] = comp.Pi.numpy()
        out[f"centroids_d{d}_b{b}"] = comp.centroids.numpy()
        for dn, dt in dts.items():
            x = outlier_kv((1, 2, 40, d), seed=100 * d + 10 * b + len(dn), dtype=dt)
            x[0, 0, 0, :] = 0            # exact zero
            x[0, 0, 1, :] = 0
            x[0, 0, 1, d - 1] = 1.0      # one-hot in the last element
            x[0, 0, 2, :] = 9000.0 if dt is not torch.float16 else 6500.0 * (128.0 / d) ** 0.5   # norm beyond fp16
            c = comp.compress(x)
            rec = comp.decompress(c)
            key = f"d{d}_b{b}_{dn}"
            out[f"{key}_x"] = x.numpy() if dt is torch.float32 else bits16(x)
            out[f"{key}_idx_bytes"] = c["idx_bytes"].numpy()
            out[f"{key}_vec_norms"] = bits16(c["vec_norms"])
            out[f"{key}_recon"] = rec.numpy()
            out[f"{key}_idx_pad"] = np.array([int(c["idx_pad"])], dtype=np.int64)
        print(f"d={d} b={b} done", flush=True)
    np.savez_compressed(os.path.join(HERE, "odd_dims.npz"), **out)


if __name__ == "__main__":
    main()
