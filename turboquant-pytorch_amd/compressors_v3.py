"""
TurboQuant V3 KV-cache compressors on MI355X.

Same classes, constructor arguments, method names, dictionary schemas and byte accounting as
the reference's turboquant/compressors_v3.py (MSECompressor :28-120, TurboQuantV3 :123-265);
the arithmetic runs in two fused gfx950 kernels (csrc/tq_compress.hip, csrc/tq_decompress.hip)
reached through the C ABI in include/tqamd.h.  There is no CPU path: tensors must live on a
HIP device.

Differences a caller can observe, all deliberate:
  * `device` (default "cpu", as in the reference) says where `Pi` and `centroids` live; the kernels
    run on the device of the tensors they are given, with their tables uploaded there on first use.
  * Codebooks and rotations are cached per (head_dim, bits) / (head_dim, seed); the reference
    re-solves them for every instance.  Values are identical.
  * `TurboQuantV3.decompress_kv` writes the de-quantised tokens straight into the
    full-length output in the window's dtype (one rounding from the fp32 accumulator) instead
    of materialising an fp32 tensor, casting and concatenating.
"""
from __future__ import annotations

import functools
import math
from typing import Tuple

import torch

from . import _native
from .lloyd_max import LloydMaxCodebook
from .rotation import generate_rotation_matrix


@functools.lru_cache(maxsize=None)
def _cached_rotation(head_dim: int, seed: int) -> torch.Tensor:
    return generate_rotation_matrix(head_dim, seed=seed, device="cpu")


@functools.lru_cache(maxsize=None)
def _cached_centroids(head_dim: int, bits: int) -> torch.Tensor:
    return LloydMaxCodebook(head_dim, bits).centroids


class MSECompressor:
    """
    Single-stage MSE-optimal compressor for keys or values: unit-normalise, rotate, pick the
    nearest Lloyd-Max centroid per coordinate, store bit-packed codes and fp16 norms.
    Interface of compressors_v3.py:28-120.
    """

    def __init__(self, head_dim: int, bits: int, seed: int, device: str = "cpu"):
        self.head_dim = head_dim
        self.bits = bits
        self.device = device      # where Pi and centroids live (the reference's default: "cpu"); the kernels follow the tensors

        pi_host = _cached_rotation(head_dim, seed)
        cent_host = _cached_centroids(head_dim, bits)
        self.Pi = pi_host.to(device).contiguous()      # row-major in memory: the kernels take its address
        self.centroids = cent_host.to(device)
        # Everything the kernels read, baked once: split rotation tiles, quantiser grid, decode tables.
        # (above 8 bits the reference constructs fine and fails in compress(); keep that order)
        self._table_host = _native.build_table(pi_host, cent_host, bits) if 1 <= bits <= 8 else None
        self._tables = {}
        self._pi_on = {}

    @classmethod
    def from_tensors(cls, Pi: torch.Tensor, centroids: torch.Tensor, bits: int, device: str = "cpu"):
        """Build a compressor from an explicit rotation and codebook (parity tests pass the
        reference's own matrices through here)."""
        self = cls.__new__(cls)
        self.head_dim = Pi.shape[0]
        self.bits = bits
        self.device = device
        self.Pi = Pi.to(device=device, dtype=torch.float32).contiguous()
        self.centroids = centroids.to(device=device, dtype=torch.float32)
        self._table_host = _native.build_table(Pi, centroids, bits)
        self._tables = {}
        self._pi_on = {}
        return self

    def pi(self, device=None) -> torch.Tensor:
        """Pi on `device` (default: the compressor's own): the compressor may sit on the CPU, as the reference's does
        by default, while the tensors it is given are on a HIP device; copies are made once per device."""
        dev = torch.device(self.device if device is None else device)
        if dev == self.Pi.device:
            return self.Pi
        t = self._pi_on.get(dev)
        if t is None:
            t = self._pi_on[dev] = self.Pi.to(dev).contiguous()
        return t

    def pi_transposed(self, device=None) -> torch.Tensor:
        """Pi^T as its own contiguous tensor (made on first use): the decode-step kernels read it row by row."""
        dev = torch.device(self.device if device is None else device)
        t = self._pi_on.get(("t", dev))
        if t is None:
            t = self._pi_on[("t", dev)] = self.pi(dev).t().contiguous()
        return t

    def table(self, device=None) -> torch.Tensor:
        """Copy of the codec table on `device` (default: the compressor's own), uploaded on first use."""
        dev = torch.device(self.device if device is None else device)
        if dev.type == "cuda" and dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        t = self._tables.get(dev)
        if t is None:
            if dev.type != "cuda":
                raise _native.TqError(f"MSECompressor: the codec runs on HIP devices only (asked for a table on {dev}); "
                                      "pass tensors that live on the GPU")
            t = self._tables[dev] = _native.upload_table(self._table_host, self.head_dim, self.bits, dev)
        return t

    @torch.no_grad()
    def compress(self, states: torch.Tensor) -> dict:
        """(B, H, S, D) -> {"idx_bytes" u8 [B,H,S,G], "vec_norms" f16 [B,H,S], "shape", "idx_pad"}."""
        B, H, S, D = states.shape
        indices_per_byte = 8 // self.bits
        idx_pad = (indices_per_byte - D % indices_per_byte) % indices_per_byte
        idx_bytes, vec_norms = _native.call("compress", states, self.table(states.device), self.bits)
        return {
            "idx_bytes": idx_bytes,
            "vec_norms": vec_norms,
            "shape": (B, H, S, D),
            "idx_pad": idx_pad,
        }

    @torch.no_grad()
    def compress_into(self, states: torch.Tensor, idx_bytes: torch.Tensor, vec_norms: torch.Tensor) -> None:
        """Compress (B, H, S, D) states into caller-owned packed buffers u8 [B,H,S,G] / f16 [B,H,S]:
        contiguous tensors, or token-axis slices of a preallocated [B,H,capacity,..] store (appending
        to a cache without reallocating it)."""
        B, H, S, D = states.shape
        width = math.ceil(D / (8 // self.bits))
        if tuple(idx_bytes.shape) != (B, H, S, width) or tuple(vec_norms.shape) != (B, H, S):
            raise ValueError(f"packed buffers {tuple(idx_bytes.shape)} / {tuple(vec_norms.shape)} do not match "
                             f"states {tuple(states.shape)} at {self.bits} bits")
        if idx_bytes.dtype != torch.uint8 or vec_norms.dtype != torch.float16:
            raise ValueError("packed buffers must be uint8 codes and float16 norms")
        if S * B * H:
            _native.call("compress_into", states, self.table(states.device), self.bits, idx_bytes, vec_norms)

    @torch.no_grad()
    def decompress_packed(self, idx_bytes: torch.Tensor, vec_norms: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """De-quantise packed buffers (as accepted by compress_into) into `out` [B,H,S,D]."""
        B, H, S, D = out.shape
        if tuple(idx_bytes.shape[:3]) != (B, H, S) or tuple(vec_norms.shape) != (B, H, S):
            raise ValueError(f"packed buffers {tuple(idx_bytes.shape)} / {tuple(vec_norms.shape)} do not match "
                             f"output {tuple(out.shape)}")
        if S * B * H:
            _native.call("decompress_into", idx_bytes, vec_norms, self.table(out.device), self.bits, out)
        return out

    @torch.no_grad()
    def packed_scores(self, idx_bytes: torch.Tensor, vec_norms: torch.Tensor, queries: torch.Tensor,
                      scale: float = 1.0, out: torch.Tensor = None) -> torch.Tensor:
        """scale * q . k_hat for every packed key, without de-quantising: queries [B,Hq,1,D] or [B,Hq,D]
        (Hq a multiple of the packed H: query head j reads kv head j // (Hq/H)), packed keys as accepted
        by decompress_packed -> float32 scores [B,Hq,S] (written into `out` when given).  Equals
        attention_scores(queries, decompress(...)) * scale (validate_v3.py:87) up to rounding."""
        B, H, S, _ = idx_bytes.shape
        q = queries.reshape(B, -1, self.head_dim)
        Hq = q.shape[1]
        if Hq % H:
            raise ValueError(f"{Hq} query heads do not divide over {H} kv heads")
        q_rot = torch.matmul(q.to(torch.float32), self.pi(q.device).T) * scale        # (Pi q): rotate once per step
        if out is None:
            out = torch.empty((B, Hq, S), dtype=torch.float32, device=idx_bytes.device)
        if B * Hq * S:
            _native.call("scores_into", idx_bytes, vec_norms, self.table(idx_bytes.device), self.bits, q_rot, out)
        return out

    @torch.no_grad()
    def packed_weighted_values(self, idx_bytes: torch.Tensor, vec_norms: torch.Tensor,
                               weights: torch.Tensor) -> torch.Tensor:
        """sum_t weights[b, hq, t] * v_hat[b, hq // group, t] over the packed values -> float32 [B,Hq,D],
        accumulated in the rotated space and rotated back once."""
        B, H, S, _ = idx_bytes.shape
        if S == 0:
            return torch.zeros((B, weights.shape[1], self.head_dim), dtype=torch.float32, device=idx_bytes.device)
        out_rot = _native.call("weighted_values", idx_bytes, vec_norms, self.table(idx_bytes.device), self.bits, weights, self.head_dim)
        return torch.matmul(out_rot, self.pi(out_rot.device))

    @torch.no_grad()
    def decompress(self, compressed: dict) -> torch.Tensor:
        """Back to a float32 (B, H, S, D) tensor."""
        B, H, S, D = compressed["shape"]
        width = math.ceil(D / (8 // self.bits))
        idx_bytes = compressed["idx_bytes"].reshape(B, H, S, width)
        vec_norms = compressed["vec_norms"].reshape(B, H, S)
        return _native.call("decompress", idx_bytes, vec_norms, self.table(idx_bytes.device), self.bits, D, torch.float32)

    @torch.no_grad()
    def decompress_into(self, compressed: dict, out: torch.Tensor) -> torch.Tensor:
        """De-quantise into `out` (a [B,H,S,D] tensor or strided view of any supported float type)."""
        B, H, S, D = compressed["shape"]
        if tuple(out.shape) != (B, H, S, D):
            raise ValueError(f"output shape {tuple(out.shape)} does not match compressed shape {(B, H, S, D)}")
        width = math.ceil(D / (8 // self.bits))
        _native.call("decompress_into", compressed["idx_bytes"].reshape(B, H, S, width),
                                        compressed["vec_norms"].reshape(B, H, S), self.table(out.device), self.bits, out)
        return out

    def memory_bytes(self, B: int, H: int, S: int) -> dict:
        """Bytes actually stored for B*H*S vectors (compressors_v3.py:107-120)."""
        n_vec = B * H * S
        indices_per_byte = 8 // self.bits
        compressed = n_vec * math.ceil(self.head_dim / indices_per_byte) + n_vec * 2
        fp16 = n_vec * self.head_dim * 2
        return {
            "compressed_bytes": compressed,
            "fp16_bytes": fp16,
            "compression_ratio": fp16 / compressed if compressed > 0 else 0,
        }


class TurboQuantV3:
    """
    KV-cache compressor: asymmetric key/value widths, an uncompressed window of recent tokens,
    wider codes for the first and last `protected_layers` layers.  Interface of
    compressors_v3.py:123-265.
    """

    def __init__(
        self,
        head_dim: int,
        key_bits: int = 4,
        value_bits: int = 2,
        residual_window: int = 128,
        layer_idx: int = 0,
        n_layers: int = 36,
        protected_layers: int = 4,
        protected_bits: int = 8,
        seed: int = 42,
        device: str = "cpu",
    ):
        self.head_dim = head_dim
        self.residual_window = residual_window
        self.device = device

        protected = layer_idx < protected_layers or layer_idx >= (n_layers - protected_layers)
        self.key_bits = min(protected_bits if protected else key_bits, 8)
        self.value_bits = min(protected_bits if protected else value_bits, 8)

        seed_base = seed + layer_idx * 1000
        self.key_compressor = MSECompressor(head_dim, self.key_bits, seed=seed_base, device=device)
        self.val_compressor = MSECompressor(head_dim, self.value_bits, seed=seed_base + 500, device=device)

    @torch.no_grad()
    def compress_kv(self, keys: torch.Tensor, values: torch.Tensor) -> Tuple[dict, dict]:
        """keys, values (B, H, S, D) -> two dicts with "compressed", "fp16", "shape", "split_at"."""
        B, H, S, D = keys.shape
        rw = self.residual_window
        if S <= rw:
            return (
                {"fp16": keys, "compressed": None, "shape": (B, H, S, D), "split_at": S},
                {"fp16": values, "compressed": None, "shape": (B, H, S, D), "split_at": S},
            )
        split_at = S - rw
        out = []
        for tensor, comp in ((keys, self.key_compressor), (values, self.val_compressor)):
            out.append({
                # the kernel reads the strided slice in place: no contiguous copy of the old tokens
                "compressed": comp.compress(tensor[:, :, :split_at, :]),
                "fp16": tensor[:, :, split_at:, :],
                "shape": (B, H, S, D),
                "split_at": split_at,
            })
        return out[0], out[1]

    @torch.no_grad()
    def decompress_kv(self, compressed_k: dict, compressed_v: dict) -> Tuple[torch.Tensor, torch.Tensor]:
        """-> keys, values (B, H, S, D) in the dtype of the uncompressed window."""
        if compressed_k["compressed"] is None:
            return compressed_k["fp16"], compressed_v["fp16"]
        out = []
        for c, comp in ((compressed_k, self.key_compressor), (compressed_v, self.val_compressor)):
            B, H, S, D = c["shape"]
            split_at = c["split_at"]
            window = c["fp16"]
            full = torch.empty((B, H, S, D), dtype=window.dtype, device=window.device)
            comp.decompress_into(c["compressed"], full[:, :, :split_at, :])
            if S > split_at:
                full[:, :, split_at:, :].copy_(window)
            out.append(full)
        return out[0], out[1]

    def memory_bytes(self, B: int, H: int, S: int) -> dict:
        """Bytes stored including the uncompressed window (compressors_v3.py:235-265)."""
        fp16_tokens = min(self.residual_window, S)
        compressed_tokens = max(S - fp16_tokens, 0)
        compressed_bytes = 0
        if compressed_tokens > 0:
            compressed_bytes = (self.key_compressor.memory_bytes(B, H, compressed_tokens)["compressed_bytes"]
                                + self.val_compressor.memory_bytes(B, H, compressed_tokens)["compressed_bytes"])
        window_bytes = B * H * fp16_tokens * self.head_dim * 2 * 2
        total = compressed_bytes + window_bytes
        baseline = B * H * S * self.head_dim * 2 * 2
        return {
            "compressed_bytes": total,
            "fp16_bytes": baseline,
            "compression_ratio": baseline / total if total > 0 else 0,
            "compressed_tokens": compressed_tokens,
            "fp16_tokens": fp16_tokens,
            "key_bits": self.key_bits,
            "value_bits": self.value_bits,
        }
