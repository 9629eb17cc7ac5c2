"""
On-disk form of compressed KV data.

The reference keeps compressed data as plain dicts of tensors and Python ints
(compressors_v3.py:76-81, :220-233) and the streaming cache as Python lists of such dicts
(generation_test_v2.py:58-63); neither has a wire format.  This module writes both as one
safetensors file: tensors under stable names, everything else as JSON in the file's metadata.
Loading executes nothing from the file.

File layout (metadata key "tqamd" holds the JSON header):

  kind "kv-cache"   a V3Cache: per layer  L{i}.k_idx u8 [B,H,n_c,Gk], L{i}.k_nrm f16 [B,H,n_c],
                    L{i}.v_idx, L{i}.v_nrm, L{i}.k_win / L{i}.v_win [B,H,n_w,D] (the uncompressed
                    window, oldest token first), and optionally the codec itself
                    (L{i}.k_pi, L{i}.k_centroids, L{i}.v_pi, L{i}.v_centroids);
  kind "kv-pair"    the two dicts TurboQuantV3.compress_kv returns: k.* / v.* tensors
                    (idx_bytes, vec_norms, fp16).

The header carries a SHA-256 of every layer's rotation and codebook.  A loader that regenerates the
codec from its seeds compares them, so a file is never decoded with a different rotation silently.
"""
from __future__ import annotations

import hashlib
import json
from typing import Dict, Optional, Tuple

import torch

from .compressors_v3 import MSECompressor, TurboQuantV3

FORMAT_VERSION = 1
_META_KEY = "tqamd"
_DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}


class FormatError(ValueError):
    """The file is not one this module wrote, or it does not match the codec it is loaded into."""


def codec_digest(comp: MSECompressor) -> str:
    """SHA-256 over bits, rotation and codebook of one MSECompressor (float32 bytes, row-major)."""
    h = hashlib.sha256()
    h.update(bytes([comp.bits]))
    h.update(comp.Pi.detach().to("cpu", torch.float32).contiguous().numpy().tobytes())
    h.update(comp.centroids.detach().to("cpu", torch.float32).contiguous().numpy().tobytes())
    return h.hexdigest()


def _write(path: str, tensors: Dict[str, torch.Tensor], header: dict) -> None:
    from safetensors.torch import save_file
    header = dict(header, version=FORMAT_VERSION)
    flat = {}
    for name, t in tensors.items():
        x = t.detach().contiguous().cpu()
        flat[name] = x.clone() if x.data_ptr() == t.data_ptr() else x      # entries never share memory (cached codebooks do)
    save_file(flat, path, metadata={_META_KEY: json.dumps(header)})


def _open(path: str, kind: str, device):
    from safetensors import safe_open
    f = safe_open(path, framework="pt", device=str(device))
    meta = f.metadata() or {}
    if _META_KEY not in meta:
        raise FormatError(f"{path}: no '{_META_KEY}' header; not a file written by this module")
    header = json.loads(meta[_META_KEY])
    if header.get("version") != FORMAT_VERSION:
        raise FormatError(f"{path}: format version {header.get('version')!r}, this build reads {FORMAT_VERSION}")
    if header.get("kind") != kind:
        raise FormatError(f"{path}: holds a {header.get('kind')!r}, expected a {kind!r}")
    return f, header


# ------------------------------------------------------------------------------------
# the dict pair of TurboQuantV3.compress_kv
# ------------------------------------------------------------------------------------
def save_compressed(path: str, compressed_k: dict, compressed_v: dict, codec: Optional[TurboQuantV3] = None) -> None:
    """Write the two dicts `TurboQuantV3.compress_kv` returned.  With `codec` the header also records the
    digests of its key and value compressors, which `load_compressed(..., codec=)` checks."""
    tensors: Dict[str, torch.Tensor] = {}
    header = {"kind": "kv-pair", "sides": {}}
    for side, c in (("k", compressed_k), ("v", compressed_v)):
        info = {"shape": list(c["shape"]), "split_at": int(c["split_at"]), "compressed": None}
        if c["fp16"] is not None:
            tensors[f"{side}.fp16"] = c["fp16"]
        inner = c["compressed"]
        if inner is not None:
            extra = {}
            for name, val in inner.items():
                if isinstance(val, torch.Tensor):
                    tensors[f"{side}.{name}"] = val
                else:
                    extra[name] = list(val) if isinstance(val, (tuple, list)) else val
            info["compressed"] = extra
        header["sides"][side] = info
    if codec is not None:
        header["digests"] = {"k": codec_digest(codec.key_compressor), "v": codec_digest(codec.val_compressor)}
    _write(path, tensors, header)


def load_compressed(path: str, device="cuda", codec: Optional[TurboQuantV3] = None) -> Tuple[dict, dict]:
    """Read a file written by `save_compressed` back into the dict pair `decompress_kv` takes."""
    f, header = _open(path, "kv-pair", device)
    if codec is not None and "digests" in header:
        got = {"k": codec_digest(codec.key_compressor), "v": codec_digest(codec.val_compressor)}
        if got != header["digests"]:
            raise FormatError(f"{path}: written with a different rotation / codebook than the codec it is loaded for")
    names = set(f.keys())
    out = []
    for side in ("k", "v"):
        info = header["sides"][side]
        c = {"shape": tuple(info["shape"]), "split_at": info["split_at"], "compressed": None,
             "fp16": f.get_tensor(f"{side}.fp16") if f"{side}.fp16" in names else None}
        if info["compressed"] is not None:
            inner = {k: (tuple(v) if isinstance(v, list) else v) for k, v in info["compressed"].items()}
            for name in names:
                if name.startswith(side + ".") and name != f"{side}.fp16":
                    inner[name[len(side) + 1:]] = f.get_tensor(name)
            c["compressed"] = inner
        out.append(c)
    return out[0], out[1]


# ------------------------------------------------------------------------------------
# the streaming cache
# ------------------------------------------------------------------------------------
def save_cache(cache, path: str, include_codec: bool = True) -> None:
    """Write a V3Cache: configuration, per layer the packed history and the uncompressed window.
    include_codec also stores every layer's rotations and codebooks (64 KiB per rotation), which makes the
    file readable where the seeded generator would produce different matrices."""
    header = {
        "kind": "kv-cache",
        "config": {"key_bits": cache.key_bits, "value_bits": cache.value_bits,
                   "residual_window": cache.residual_window, "protected_layers": cache.protected_layers,
                   "n_layers": cache.n_layers},
        "layers": {},
    }
    tensors: Dict[str, torch.Tensor] = {}
    for idx, st in sorted(cache._stores.items()):
        kc, vc = st.comp.key_compressor, st.comp.val_compressor
        n_c = st.n_compressed
        header["layers"][str(idx)] = {
            "batch": st.B, "heads": st.H, "head_dim": st.D, "dtype": str(st.dtype).replace("torch.", ""),
            "n_compressed": n_c, "n_recent": st.n_recent, "total_seq": st.total_seq,
            "key_bits": kc.bits, "value_bits": vc.bits,
            "digests": {"k": codec_digest(kc), "v": codec_digest(vc)},
        }
        p = f"L{idx}."
        if n_c:
            tensors[p + "k_idx"], tensors[p + "k_nrm"] = st.k_idx[:, :, :n_c], st.k_nrm[:, :, :n_c]
            tensors[p + "v_idx"], tensors[p + "v_nrm"] = st.v_idx[:, :, :n_c], st.v_nrm[:, :, :n_c]
        if st.n_recent:
            tensors[p + "k_win"], tensors[p + "v_win"] = st.window()
        if include_codec:
            tensors[p + "k_pi"], tensors[p + "k_centroids"] = kc.Pi, kc.centroids
            tensors[p + "v_pi"], tensors[p + "v_centroids"] = vc.Pi, vc.centroids
    _write(path, tensors, header)


def load_cache(path: str, device="cuda", cls=None):
    """Read a file written by `save_cache` into a new V3Cache (or `cls`, a subclass) on `device`.
    Each layer's codec is regenerated from its seeds and compared with the digests in the file; where they
    differ the stored codec is used if the file has one, otherwise FormatError."""
    from .kv_cache import V3Cache, _LayerStore
    f, header = _open(path, "kv-cache", device)
    cache = (cls or V3Cache)(**header["config"])
    names = set(f.keys())
    device = torch.device(device)
    for key, info in sorted(header["layers"].items(), key=lambda kv: int(kv[0])):
        idx = int(key)
        p = f"L{idx}."
        if info["dtype"] not in _DTYPES:
            raise FormatError(f"{path}: layer {idx} has element type {info['dtype']!r}")
        comp = cache._get_compressor(idx, info["head_dim"], device)
        for side, attr, bits in (("k", "key_compressor", info["key_bits"]), ("v", "val_compressor", info["value_bits"])):
            c = getattr(comp, attr)
            if c.bits == bits and codec_digest(c) == info["digests"][side]:
                continue
            if p + side + "_pi" not in names:
                raise FormatError(f"{path}: layer {idx} was written with a different rotation / codebook than this "
                                  f"build generates for its seed, and the file does not carry the codec")
            stored = MSECompressor.from_tensors(f.get_tensor(p + side + "_pi").cpu(), f.get_tensor(p + side + "_centroids").cpu(),
                                                bits, device=str(device))
            if codec_digest(stored) != info["digests"][side]:
                raise FormatError(f"{path}: layer {idx}: stored codec does not match its digest")
            setattr(comp, attr, stored)
            if side == "k":
                comp.key_bits = bits
            else:
                comp.value_bits = bits
        n_c, n_w = info["n_compressed"], info["n_recent"]
        st = _LayerStore(comp, info["batch"], info["heads"], info["head_dim"], _DTYPES[info["dtype"]], device,
                         n_c, cache.residual_window)
        if n_c:
            for name in ("k_idx", "k_nrm", "v_idx", "v_nrm"):
                src = f.get_tensor(p + name)
                dst = getattr(st, name)[:, :, :n_c]
                if src.shape != dst.shape or src.dtype != dst.dtype:
                    raise FormatError(f"{path}: {p + name} is {tuple(src.shape)} {src.dtype}, expected {tuple(dst.shape)} {dst.dtype}")
                dst.copy_(src)
            st.n_compressed = n_c
        if n_w:
            kw, vw = f.get_tensor(p + "k_win"), f.get_tensor(p + "v_win")
            want = (info["batch"], info["heads"], n_w, info["head_dim"])
            if tuple(kw.shape) != want or tuple(vw.shape) != want:
                raise FormatError(f"{path}: window of layer {idx} is {tuple(kw.shape)}, expected {want}")
            if n_w > st.win_cap:                       # a file whose window outgrew 2 x residual_window cannot come from save_cache
                raise FormatError(f"{path}: window of layer {idx} holds {n_w} tokens, more than the cache keeps")
            st.extend_window(kw, vw)
        st.total_seq = info["total_seq"]
        cache._stores[idx] = st
    return cache
