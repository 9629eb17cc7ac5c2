#!/usr/bin/env python3
"""Write tests/golden/v2_qjl.npz from the upstream Python reference: inputs and outputs of the V2 key path
(MSE codes + 1-bit QJL signs of the residual, turboquant/compressors.py:84-158) and of its value compressor
(compressors.py:200-221), on seeded inputs.

Run once, in the build container, where the reference checkout is mounted read-only at /root/reference
(override with TQ_REFERENCE_ROOT):

    python tests/golden/make_fixtures_v2.py

Data only (numpy arrays, no pickles); fp16 / bf16 tensors are stored as uint16 bit patterns.  What these vectors
pin and mathematics alone does not: the last bits of the QR rotation and of the 200-step codebook iterate as this
class computes them, the order of its float32 operations (residual in the original space, projection by S), and
its sign convention for a projection of exactly zero.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF_ROOT = os.environ.get("TQ_REFERENCE_ROOT", "/root/reference")


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def outlier_kv(shape, seed, dtype):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    x = torch.randn(*shape, generator=g)
    ch = torch.exp(torch.randn(shape[-1], generator=g))
    tok = 0.5 + 1.5 * torch.rand(*shape[:-1], 1, generator=g)
    return (x * ch * tok).to(dtype)


def main():
    sys.path.insert(0, REF_ROOT)
    from turboquant.compressors import TurboQuantCompressorV2, TurboQuantCompressorMSE
    torch.set_num_threads(1)
    out = {}
    D = 128
    for bits in (2, 3, 4, 5):
        seed = 1000 * bits
        kc = TurboQuantCompressorV2(D, bits, seed=seed, device="cpu")
        vc = TurboQuantCompressorMSE(D, bits, seed=seed + 500, device="cpu")
        out[f"b{bits}_Pi"] = kc.Pi.numpy()
        out[f"b{bits}_S"] = kc.S.numpy()
        out[f"b{bits}_centroids"] = kc.centroids.numpy()
        out[f"b{bits}_v_Pi"] = vc.Pi.numpy()
        out[f"b{bits}_v_centroids"] = vc.centroids.numpy()
        for dn, dt in (("f16", torch.float16), ("bf16", torch.bfloat16), ("f32", torch.float32)):
            x = outlier_kv((1, 2, 80, D), seed=7000 + bits, dtype=dt)
            x[0, 0, 0] = 0                      # an all-zero vector: residual 0, every projection exactly 0
            x[0, 1, 5] = 0
            x[0, 1, 5, 17] = 3.0                # a one-hot vector
            x[0, 0, 7] *= 1e-3
            c = kc.compress(x)
            tag = f"b{bits}_{dn}"
            out[tag + "_x"] = x.numpy() if dt == torch.float32 else bits16(x)
            out[tag + "_k_mse"] = bits16(c["k_mse"])
            out[tag + "_qjl_signs"] = c["qjl_signs"].numpy()
            out[tag + "_residual_norm"] = bits16(c["residual_norm"])
            g = torch.Generator(device="cpu")
            g.manual_seed(8000 + bits)
            q = torch.randn(1, 2, 5, D, generator=g)
            out[tag + "_q"] = q.numpy()
            out[tag + "_scores"] = kc.asymmetric_attention_scores(q, c).numpy()
            if dn == "f16":
                cv = vc.compress(x)
                out[tag + "_v_indices"] = cv["indices"].numpy()
                out[tag + "_v_vec_norms"] = bits16(cv["vec_norms"])
                out[tag + "_v_recon"] = vc.decompress(cv).numpy()
    np.savez_compressed(os.path.join(HERE, "v2_qjl.npz"), **out)
    print("wrote", os.path.join(HERE, "v2_qjl.npz"), len(out), "arrays")


if __name__ == "__main__":
    main()
