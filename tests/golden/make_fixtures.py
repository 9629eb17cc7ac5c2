#!/usr/bin/env python3
"""Write the golden input/output vectors under tests/golden/ from the upstream
Python reference.

Run once, in the build container, where the reference checkout is mounted
read-only at /root/reference (override with TQ_REFERENCE_ROOT):

    python tests/golden/make_fixtures.py

It imports the reference package, calls the functions on the KV compress /
decompress path with seeded inputs and stores inputs + outputs as plain numpy
arrays (.npz, no pickles) and JSON.  Nothing of the reference's text is stored:
the fixtures are data only.  The functions pinned here are the ones whose last
bits cannot be derived from mathematics alone:

  * solve_lloyd_max(d, bits)            lloyd_max.py:32-86   (200-step iterate, QUADPACK tails)
  * generate_rotation_matrix(d, seed)   turboquant.py:18-33  (LAPACK QR bits)
  * MSECompressor.compress/decompress   compressors_v3.py:46-105
  * TurboQuantV3.compress_kv/decompress_kv/memory_bytes  compressors_v3.py:171-265

bf16 / fp16 tensors are stored as their uint16 bit patterns.
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF_ROOT = os.environ.get("TQ_REFERENCE_ROOT", "/root/reference")


def bits16(t: torch.Tensor) -> np.ndarray:
    """fp16/bf16 tensor -> uint16 bit pattern array."""
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def outlier_kv(shape, seed, dtype):
    """N(0,1) x per-channel log-normal(sigma=1) scale x per-token U[0.5,2] spread."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    x = torch.randn(*shape, generator=g)
    ch = torch.exp(torch.randn(shape[-1], generator=g))
    tok = 0.5 + 1.5 * torch.rand(*shape[:-1], 1, generator=g)
    return (x * ch * tok).to(dtype)


def main():
    sys.path.insert(0, REF_ROOT)
    import turboquant  # noqa: F401  (the reference package)
    from turboquant.lloyd_max import solve_lloyd_max
    from turboquant.turboquant import generate_rotation_matrix
    from turboquant.compressors_v3 import MSECompressor, TurboQuantV3

    torch.set_num_threads(1)
    meta = {"torch": torch.__version__, "numpy": np.__version__}
    try:
        import scipy
        meta["scipy"] = scipy.__version__
    except Exception:  # pragma: no cover
        pass

    # ---- 1. codebooks -------------------------------------------------
    books = {}
    for d, bit_list in ((128, range(1, 9)), (64, (2, 4)), (256, (2, 4))):
        for b in bit_list:
            c, bnd = solve_lloyd_max(d, b)
            books[f"centroids_d{d}_b{b}"] = c.numpy().astype(np.float32)
            books[f"boundaries_d{d}_b{b}"] = bnd.numpy().astype(np.float32)
            print(f"codebook d={d} b={b}: {c.numel()} levels", flush=True)
    np.savez_compressed(os.path.join(HERE, "codebooks.npz"), **books)

    # ---- 2. rotations -------------------------------------------------
    rots = {}
    for seed in (0, 42, 542, 1042, 1542, 31042, 31542):
        rots[f"Pi_d128_s{seed}"] = generate_rotation_matrix(128, seed=seed).numpy().astype(np.float32)
    rots["Pi_d64_s42"] = generate_rotation_matrix(64, seed=42).numpy().astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "rotations.npz"), **rots)

    # ---- 3. MSECompressor round trips ----------------------------------
    cases = {}
    summary = {}
    dts = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    for b in (1, 2, 3, 4, 5, 6, 7, 8):
        comp = MSECompressor(128, b, seed=42 + b)
        cases[f"Pi_b{b}"] = comp.Pi.numpy()
        cases[f"centroids_b{b}"] = comp.centroids.numpy()
        for dn, dt in dts.items():
            if b in (5, 7) and dn != "f16":
                continue
            x = outlier_kv((1, 2, 48, 128), seed=1000 * b + len(dn), dtype=dt)
            # edge vectors: exact zero, a one-hot, a norm that overflows fp16, a tiny one
            x[0, 0, 0, :] = 0
            x[0, 0, 1, :] = 0
            x[0, 0, 1, 5] = 1.0
            if dt is not torch.float16:
                x[0, 0, 2, :] = 7000.0  # norm ~ 79196 -> fp16 inf
            else:
                x[0, 0, 2, :] = 6000.0  # norm ~ 67882 -> fp16 inf
            x[0, 0, 3, :] = x[0, 0, 4, :] * 1e-3
            out = comp.compress(x)
            rec = comp.decompress(out)
            key = f"b{b}_{dn}"
            cases[f"{key}_x"] = x.numpy() if dt is torch.float32 else bits16(x)
            cases[f"{key}_idx_bytes"] = out["idx_bytes"].numpy()
            cases[f"{key}_vec_norms"] = bits16(out["vec_norms"])
            cases[f"{key}_recon"] = rec.numpy()
            summary[key] = {
                "shape": list(out["shape"]), "idx_pad": int(out["idx_pad"]),
                "idx_bytes_shape": list(out["idx_bytes"].shape),
                "recon_dtype": str(rec.dtype),
                "memory_bytes": comp.memory_bytes(1, 2, 48),
            }
        print(f"round trips b={b} done", flush=True)
    np.savez_compressed(os.path.join(HERE, "mse_roundtrip.npz"), **cases)

    # ---- 4. the CPU-runnable benchmark configuration --------------------
    # K [1,8,1024,128] fp32 N(0,1) from seed 0, 4-bit, rotation seed 42.
    torch.manual_seed(0)
    k = torch.randn(1, 8, 1024, 128)
    comp = MSECompressor(128, 4, seed=42)
    out = comp.compress(k)
    rec = comp.decompress(out)
    err = (k - rec).reshape(-1, 128)
    cos = torch.nn.functional.cosine_similarity(k.reshape(-1, 128), rec.reshape(-1, 128), dim=-1)
    cfg1 = {
        "input_sha256": sha(k.numpy()),
        "idx_bytes_sha256": sha(out["idx_bytes"].numpy()),
        "vec_norms_sha256": sha(bits16(out["vec_norms"])),
        "recon_sha256": sha(rec.numpy()),
        "packed_bytes": int(out["idx_bytes"].numel() + 2 * out["vec_norms"].numel()),
        "mse_per_element": float((err ** 2).mean()),
        "rel_mse": float(((err ** 2).sum(-1) / (k.reshape(-1, 128) ** 2).sum(-1)).mean()),
        "cosine_mean": float(cos.mean()),
        "cosine_min": float(cos.min()),
        "memory_bytes": comp.memory_bytes(1, 8, 1024),
    }
    np.savez_compressed(
        os.path.join(HERE, "config1.npz"),
        idx_bytes=out["idx_bytes"].numpy(),
        vec_norms=bits16(out["vec_norms"]),
        x_head=k[0, 0, :64].numpy(),
        recon_head=rec[0, 0, :64].numpy(),
    )

    # ---- 5. TurboQuantV3 orchestration ----------------------------------
    v3 = {}
    v3_np = {}
    # bit selection per layer (only layers whose effective widths are <= 4 bits: the
    # constructor solves both codebooks, and the 8-bit ones are covered just below)
    sel = []
    for (kb, vb, pl, nl, pb) in ((4, 2, 4, 36, 8), (4, 2, 0, 36, 8), (3, 4, 2, 32, 4), (2, 1, 1, 4, 3), (4, 4, 2, 6, 2)):
        for li in sorted({0, max(pl - 1, 0), pl, nl // 2, nl - pl - 1, max(nl - pl, 0), nl - 1}):
            if not 0 <= li < nl:
                continue
            is_prot = li < pl or li >= nl - pl
            if is_prot and pb > 4:
                continue
            t = TurboQuantV3(128, key_bits=kb, value_bits=vb, layer_idx=li, n_layers=nl,
                             protected_layers=pl, protected_bits=pb)
            sel.append({"args": [kb, vb, pl, nl, pb, li], "key_bits": t.key_bits, "value_bits": t.value_bits})
    v3["bit_selection_cheap"] = sel

    # full constructor on protected layers (8-bit codebooks): a few, they are slow
    prot = []
    for li in (0, 3, 4, 31, 32, 35):
        t = TurboQuantV3(128, key_bits=4, value_bits=2, layer_idx=li, n_layers=36, protected_layers=4)
        prot.append({"layer_idx": li, "key_bits": t.key_bits, "value_bits": t.value_bits,
                     "memory_bytes_1_2_8192": t.memory_bytes(1, 2, 8192)})
        print(f"protected probe layer {li} done", flush=True)
    v3["protected_default"] = prot

    # residual-window split, K4/V2, layer 5 of 36 (unprotected), fp16, non-trivial batch/heads
    tq = TurboQuantV3(128, key_bits=4, value_bits=2, residual_window=16, layer_idx=5, n_layers=36, protected_layers=4)
    keys = outlier_kv((2, 2, 40, 128), seed=77, dtype=torch.float16)
    vals = outlier_kv((2, 2, 40, 128), seed=78, dtype=torch.float16)
    ck, cv = tq.compress_kv(keys, vals)
    rk, rv = tq.decompress_kv(ck, cv)
    v3_np.update(
        rw_keys=bits16(keys), rw_values=bits16(vals),
        rw_Pi_k=tq.key_compressor.Pi.numpy(), rw_Pi_v=tq.val_compressor.Pi.numpy(),
        rw_cent_k=tq.key_compressor.centroids.numpy(), rw_cent_v=tq.val_compressor.centroids.numpy(),
        rw_k_idx=ck["compressed"]["idx_bytes"].numpy(), rw_k_norms=bits16(ck["compressed"]["vec_norms"]),
        rw_v_idx=cv["compressed"]["idx_bytes"].numpy(), rw_v_norms=bits16(cv["compressed"]["vec_norms"]),
        rw_k_out=bits16(rk), rw_v_out=bits16(rv),
    )
    v3["rw_case"] = {
        "split_at": ck["split_at"], "shape": list(ck["shape"]),
        "compressed_shape": list(ck["compressed"]["shape"]),
        "fp16_shape": list(ck["fp16"].shape), "out_dtype": str(rk.dtype),
        "fp16_is_view_of_input": bool(ck["fp16"].data_ptr() == keys[:, :, ck["split_at"]:, :].data_ptr()),
        "memory_bytes": tq.memory_bytes(2, 2, 40),
        "seed_k": 42 + 5 * 1000, "seed_v": 42 + 5 * 1000 + 500,
    }
    # passthrough: S <= rw
    ck2, cv2 = tq.compress_kv(keys[:, :, :16], vals[:, :, :16])
    rk2, rv2 = tq.decompress_kv(ck2, cv2)
    v3["passthrough"] = {
        "compressed_is_none": ck2["compressed"] is None, "split_at": ck2["split_at"],
        "shape": list(ck2["shape"]),
        "returns_same_object": bool(rk2 is ck2["fp16"]) and bool(rv2 is cv2["fp16"]),
        "memory_bytes": tq.memory_bytes(2, 2, 16),
    }
    # rw = 0 compresses everything
    tq0 = TurboQuantV3(128, key_bits=4, value_bits=2, residual_window=0, layer_idx=5, n_layers=36, protected_layers=0)
    ck3, cv3 = tq0.compress_kv(keys, vals)
    rk3, rv3 = tq0.decompress_kv(ck3, cv3)
    v3["rw0"] = {"split_at": ck3["split_at"], "fp16_shape": list(ck3["fp16"].shape),
                 "memory_bytes": tq0.memory_bytes(2, 2, 40), "out_dtype": str(rk3.dtype)}
    v3_np.update(rw0_k_idx=ck3["compressed"]["idx_bytes"].numpy(), rw0_k_out=bits16(rk3),
                 rw0_v_idx=cv3["compressed"]["idx_bytes"].numpy(), rw0_v_out=bits16(rv3))
    # memory_bytes closed-form table
    mem = []
    for (kb, vb, rw, pl, li, nl, B, H, S) in ((4, 2, 0, 0, 0, 36, 1, 2, 8192), (4, 2, 128, 4, 0, 36, 1, 2, 8192),
                                                (4, 2, 128, 4, 10, 36, 1, 2, 8192), (3, 3, 128, 0, 3, 36, 8, 2, 4096),
                                                (4, 2, 128, 0, 3, 36, 1, 2, 100), (4, 2, 0, 0, 3, 36, 1, 2, 0)):
        t = TurboQuantV3(128, key_bits=kb, value_bits=vb, residual_window=rw, layer_idx=li, n_layers=nl, protected_layers=pl)
        mem.append({"args": [kb, vb, rw, pl, li, nl, B, H, S], "memory_bytes": t.memory_bytes(B, H, S)})
    v3["memory_bytes_table"] = mem
    np.savez_compressed(os.path.join(HERE, "v3.npz"), **v3_np)

    with open(os.path.join(HERE, "fixtures.json"), "w") as f:
        json.dump({"meta": meta, "mse_roundtrip": summary, "config1": cfg1, "v3": v3}, f, indent=1, sort_keys=True)
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
