"""
TEST INFRASTRUCTURE ONLY -- not part of the product.

CPU oracle for the TurboQuant V3 KV codec.  Two independent restatements of the
upstream algorithm live here and check each other:

  * `NumpyOracle`  -- the reference's op sequence in numpy float32, vectorised
    the same way (norm, divide, [N,D]x[D,D] product, [N,D,L] |diff| argmin,
    integer pack; unpack, gather, product, scale), chunked over N.
    Follows turboquant/compressors_v3.py:46-81 (compress) and :84-105 (decompress).
  * `COracle`      -- ctypes front end of oracle/tq_oracle.c (scalar loops, OpenMP
    over vectors): fast enough for the large parity tests; the benchmark times it as a second CPU figure.
  * `TorchCpuOracle` -- the same op sequence issued as torch CPU operators (the reference's own
    library calls: fp32 cast, torch.norm, divide, sgemm, [n,D,L] broadcast / abs / argmin, int64
    pack; unpack, gather, sgemm, scale), chunked over N so that the [n,D,L] temporary stays under
    1 GiB.  This is what the benchmark times as "the reference's CPU path" on the host cores.

Only tests/, the repository's smoke check and the benchmark's cpu_baseline leg
may import this module; the shipped package never does.

  * `attention_decode` -- one-query attention over explicit K / V in float64: the score definition of
    turboquant/validate_v3.py:87 followed by the textbook softmax-weighted sum the model applies to the
    tensors generation_test_v2.py:131-153 returns.  Pinned in tests/test_oracle.py against
    torch.nn.functional.scaled_dot_product_attention and against a brute-force loop.

What pins it: tests/golden/*.npz hold outputs of the real reference on seeded
inputs (tests/golden/make_fixtures.py wrote them); tests/test_oracle.py checks
both restatements against those, against each other, against exhaustive
pack/unpack enumeration and brute-force nearest-centroid search.  Open at the
last-bit level ("parity unpinned"): the summation order inside torch.norm and
the BLAS sgemm the reference calls -- compared through the 1e-5 decision-boundary
window, never bit for bit.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")
_LIB = os.path.join(_BUILD, "libtq_oracle.so")


# --------------------------------------------------------------------------
# dtype helpers: fp16 / bf16 travel as uint16 bit patterns
# --------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16 bit pattern (NaN kept quiet)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), rounded)
    return rounded


def widen(x: np.ndarray, dtype: str) -> np.ndarray:
    """Exact conversion of a tensor given as 'f32' array or 'f16'/'bf16' bit patterns to float32."""
    if dtype == "f32":
        return np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "f16":
        return np.ascontiguousarray(x).view(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(np.ascontiguousarray(x))
    raise ValueError(dtype)


def indices_per_byte(bits: int) -> int:
    return 8 // bits  # compressors_v3.py:64 (ZeroDivisionError above 8 bits, like the reference)


def bytes_per_vector(D: int, bits: int) -> int:
    ipb = indices_per_byte(bits)
    return -(-D // ipb)


# --------------------------------------------------------------------------
# numpy restatement
# --------------------------------------------------------------------------
class NumpyOracle:
    """The reference op sequence in float32 numpy.  `chunk` bounds the [n,D,L] temporary."""

    def __init__(self, Pi: np.ndarray, centroids: np.ndarray, bits: int, chunk: int = 2048):
        self.Pi = np.ascontiguousarray(Pi, dtype=np.float32)
        self.centroids = np.ascontiguousarray(centroids, dtype=np.float32)
        self.bits = int(bits)
        self.D = self.Pi.shape[0]
        self.chunk = chunk

    def rotate(self, x: np.ndarray):
        """-> (norms fp32 [N], rotated unit coordinates fp32 [N,D])   (:52-59)"""
        flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.D)
        norms = np.sqrt(np.sum(flat * flat, axis=-1, dtype=np.float32)).astype(np.float32)
        unit = flat / (norms[:, None] + np.float32(1e-8))
        return norms, unit @ self.Pi.T

    def nearest(self, rotated: np.ndarray) -> np.ndarray:
        """argmin_j |r - c_j|, first minimum wins  (:60-61)"""
        out = np.empty(rotated.shape, dtype=np.uint8)
        flat_r = rotated.reshape(-1)
        flat_o = out.reshape(-1)
        step = max(1, (self.chunk * self.D))
        for s in range(0, flat_r.size, step):
            d = np.abs(flat_r[s:s + step, None] - self.centroids[None, :])
            flat_o[s:s + step] = np.argmin(d, axis=-1).astype(np.uint8)
        return out

    def pack(self, idx: np.ndarray) -> np.ndarray:
        """[N,D] codes -> [N,G] bytes, MSB first, zero padded  (:64-74)"""
        ipb = indices_per_byte(self.bits)
        N, D = idx.shape
        pad = (ipb - D % ipb) % ipb
        wide = idx.astype(np.int64)
        if pad:
            wide = np.pad(wide, ((0, 0), (0, pad)))
        weights = np.array([2 ** (self.bits * i) for i in range(ipb - 1, -1, -1)], dtype=np.int64)
        return (wide.reshape(N, -1, ipb) * weights).sum(-1).astype(np.uint8)

    def unpack(self, idx_bytes: np.ndarray) -> np.ndarray:
        """[N,G] bytes -> [N,D] codes  (:93-101)"""
        ipb = indices_per_byte(self.bits)
        mask = (1 << self.bits) - 1
        shifts = np.array([self.bits * i for i in range(ipb - 1, -1, -1)], dtype=np.int64)
        idx = (idx_bytes.astype(np.int64)[:, :, None] >> shifts) & mask
        return idx.reshape(idx_bytes.shape[0], -1)[:, :self.D].astype(np.uint8)

    def compress(self, x: np.ndarray):
        """x [..., D] float32 -> dict(idx_bytes [N,G] u8, vec_norms [N] fp16 bits, rotated [N,D])"""
        norms, rotated = self.rotate(x)
        idx = self.nearest(rotated)
        return {
            "idx_bytes": self.pack(idx),
            "vec_norms": norms.astype(np.float16).view(np.uint16),
            "rotated": rotated,
            "norms_f32": norms,
        }

    def decompress(self, idx_bytes: np.ndarray, vec_norms_bits: np.ndarray) -> np.ndarray:
        idx = self.unpack(idx_bytes.reshape(-1, idx_bytes.shape[-1]))
        y = self.centroids[idx]
        n = vec_norms_bits.reshape(-1, 1).view(np.float16).astype(np.float32)
        with np.errstate(invalid="ignore", over="ignore"):
            return (y @ self.Pi) * n


# --------------------------------------------------------------------------
# V2 key path: MSE codes plus 1-bit QJL signs of the residual
# --------------------------------------------------------------------------
class QjlOracle:
    """TurboQuantCompressorV2 of turboquant/compressors.py:84-158 in float32 numpy: `bits` is the total budget, the
    codebook `centroids` has 2^max(bits-1, 1) levels (:33), S is the [D, D] Gaussian projection (:49-52).
    Pinned by tests/golden/v2_qjl.npz (outputs of the reference class on seeded inputs)."""

    def __init__(self, Pi: np.ndarray, S: np.ndarray, centroids: np.ndarray):
        self.Pi = np.ascontiguousarray(Pi, dtype=np.float32)
        self.S = np.ascontiguousarray(S, dtype=np.float32)
        self.centroids = np.ascontiguousarray(centroids, dtype=np.float32)
        self.D = self.Pi.shape[0]
        self.mse = NumpyOracle(self.Pi, self.centroids, int(np.log2(self.centroids.size)))

    def compress(self, x: np.ndarray) -> dict:
        """x [..., D] float32 -> codes [N,D], norms fp32 [N], k_mse fp32 [N,D] (and its fp16 bits), residual norm fp32
        (and fp16 bits), projected residual fp32 [N,D], signs int8 [N,D] in {-1,+1}"""
        flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.D)
        norms, rotated = self.mse.rotate(flat)                                   # :96-103
        codes = self.mse.nearest(rotated)                                        # :104-105
        with np.errstate(invalid="ignore", over="ignore"):
            k_mse = (self.centroids[codes] @ self.Pi) * norms[:, None]           # :108-109, fp32 norms
            residual = flat - k_mse                                              # :112
            rnorm = np.sqrt(np.sum(residual * residual, axis=-1, dtype=np.float32)).astype(np.float32)   # :113
            projected = residual @ self.S.T                                      # :116
        signs = np.where(projected >= 0, 1, -1).astype(np.int8)                  # :117 (a projection of 0 counts as +1)
        return {"codes": codes, "norms_f32": norms, "rotated": rotated, "k_mse": k_mse,
                "k_mse_f16": k_mse.astype(np.float16).view(np.uint16), "residual_norm_f32": rnorm,
                "residual_norm": rnorm.astype(np.float16).view(np.uint16), "projected": projected, "signs": signs}

    def scores(self, q: np.ndarray, k_mse_f16: np.ndarray, signs: np.ndarray, residual_norm_f16: np.ndarray) -> np.ndarray:
        """asymmetric_attention_scores (:124-158): q [R, Sq, D]; stored fp16 k_mse [R, Sk, D], signs [R, Sk, D],
        fp16 residual norms [R, Sk] -> float32 [R, Sq, Sk]"""
        k = k_mse_f16.view(np.float16).astype(np.float32)
        rn = residual_norm_f16.view(np.float16).astype(np.float32)
        q = np.ascontiguousarray(q, dtype=np.float32)
        term1 = q @ np.swapaxes(k, -1, -2)                                       # :144
        ip = (q @ self.S.T) @ np.swapaxes(signs.astype(np.float32), -1, -2)      # :149-152
        scale = np.float32(np.sqrt(np.pi / 2) / self.S.shape[0])                 # :155-156
        return term1 + scale * ip * rn[..., None, :]                             # :158


def pack_signs(signs: np.ndarray) -> np.ndarray:
    """{-1,+1} [N, D] -> [N, D/8] bytes, coordinate 8b+k in bit 7-k of byte b (the 1-bit code packing of
    compressors_v3.py:64-74 applied to the bit (sign >= 0))."""
    bits = (np.asarray(signs) > 0).astype(np.uint8)
    return np.packbits(bits.reshape(bits.shape[0], -1, 8), axis=-1, bitorder="big").reshape(bits.shape[0], -1)


# --------------------------------------------------------------------------
# torch CPU restatement (the timed "reference CPU path")
# --------------------------------------------------------------------------
class TorchCpuOracle:
    """MSECompressor.compress / decompress of turboquant/compressors_v3.py as torch CPU operators, on chunks of
    `chunk` vectors (default: the largest power of two that keeps the [chunk, D, 2^bits] float32 intermediate of
    :60-61 under 1 GiB; unchunked, one 8-bit layer of 262 144 vectors would need 34 GB)."""

    def __init__(self, Pi: np.ndarray, centroids: np.ndarray, bits: int, chunk: int = 0):
        import torch
        self.torch = torch
        self.Pi = torch.from_numpy(np.ascontiguousarray(Pi, dtype=np.float32))
        self.centroids = torch.from_numpy(np.ascontiguousarray(centroids, dtype=np.float32))
        self.bits = int(bits)
        self.D = self.Pi.shape[0]
        if not chunk:
            chunk = 1
            while chunk * 2 * self.D * (1 << self.bits) * 4 < (1 << 30):
                chunk *= 2
        self.chunk = chunk
        ipb = indices_per_byte(self.bits)
        self.ipb = ipb
        self.pad = (ipb - self.D % ipb) % ipb                                                    # :65
        self.weights = torch.tensor([2 ** (self.bits * i) for i in range(ipb - 1, -1, -1)], dtype=torch.long)   # :70-73
        self.shifts = torch.tensor([self.bits * i for i in range(ipb - 1, -1, -1)], dtype=torch.long)           # :95-98

    def compress(self, x):
        """x: torch CPU tensor or array [..., D], any float type -> (idx_bytes u8 [N,G], vec_norms fp16 [N]) as torch tensors"""
        torch = self.torch
        x = torch.as_tensor(x).reshape(-1, self.D)
        out_b, out_n = [], []
        with torch.no_grad():
            for s in range(0, x.shape[0], self.chunk):
                flat = x[s:s + self.chunk].float()                                        # :52
                norms = torch.norm(flat, dim=-1)                                           # :55
                unit = flat / (norms.unsqueeze(-1) + 1e-8)                                 # :56
                rotated = unit @ self.Pi.T                                                 # :59
                codes = (rotated.unsqueeze(-1) - self.centroids).abs().argmin(dim=-1).to(torch.uint8)   # :60-61
                wide = codes.long()                                                        # :66
                if self.pad:
                    wide = torch.nn.functional.pad(wide, (0, self.pad))                    # :67-68
                groups = wide.shape[-1] // self.ipb
                out_b.append((wide.reshape(-1, groups, self.ipb) * self.weights).sum(-1).to(torch.uint8))  # :74
                out_n.append(norms.to(torch.float16))                                      # :78
        return torch.cat(out_b), torch.cat(out_n)

    def decompress(self, idx_bytes, vec_norms):
        """-> float32 [N, D] torch tensor (:84-105)"""
        torch = self.torch
        idx_bytes = torch.as_tensor(idx_bytes).reshape(-1, bytes_per_vector(self.D, self.bits))
        vec_norms = torch.as_tensor(vec_norms).reshape(-1, 1)
        mask = (1 << self.bits) - 1
        out = []
        with torch.no_grad():
            for s in range(0, idx_bytes.shape[0], self.chunk):
                b = idx_bytes[s:s + self.chunk]
                codes = ((b.long().unsqueeze(-1) >> self.shifts) & mask).reshape(b.shape[0], -1)   # :99
                if self.pad:
                    codes = codes[:, :self.D]                                                     # :100-101
                out.append((self.centroids[codes] @ self.Pi) * vec_norms[s:s + self.chunk].float())   # :104
        return torch.cat(out)


# --------------------------------------------------------------------------
# C restatement
# --------------------------------------------------------------------------
def build_c_oracle(force: bool = False) -> str:
    """Compile oracle/tq_oracle.c with gcc into oracle/_build/ and return the library path."""
    src = os.path.join(_HERE, "tq_oracle.c")
    if (not force and os.path.exists(_LIB)
            and os.path.getmtime(_LIB) >= os.path.getmtime(src)):
        return _LIB
    os.makedirs(_BUILD, exist_ok=True)
    cmd = ["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-shared", "-fPIC", src, "-o", _LIB, "-lm"]
    subprocess.run(cmd, check=True)
    return _LIB


_lib = None


def _load():
    global _lib
    if _lib is None:
        path = _LIB if os.path.exists(_LIB) else build_c_oracle()
        lib = ctypes.CDLL(path)
        f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
        u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
        u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
        lib.tqo_compress.argtypes = [f32p, ctypes.c_longlong, ctypes.c_int, f32p, f32p, ctypes.c_int,
                                     ctypes.c_int, u8p, u16p, ctypes.c_void_p]
        lib.tqo_compress.restype = ctypes.c_int
        lib.tqo_decompress.argtypes = [u8p, u16p, ctypes.c_longlong, ctypes.c_int, f32p, f32p,
                                       ctypes.c_int, ctypes.c_int, f32p]
        lib.tqo_decompress.restype = ctypes.c_int
        lib.tqo_nearest.argtypes = [f32p, ctypes.c_longlong, f32p, ctypes.c_int, u8p]
        lib.tqo_pack.argtypes = [u8p, ctypes.c_int, ctypes.c_int, u8p]
        lib.tqo_unpack.argtypes = [u8p, ctypes.c_int, ctypes.c_int, u8p]
        lib.tqo_f32_to_f16.argtypes = [f32p, u16p, ctypes.c_longlong]
        lib.tqo_f16_to_f32.argtypes = [u16p, f32p, ctypes.c_longlong]
        lib.tqo_max_threads.restype = ctypes.c_int
        lib.tqo_set_threads.argtypes = [ctypes.c_int]
        _lib = lib
    return _lib


class COracle:
    """ctypes front end of tq_oracle.c."""

    def __init__(self, Pi: np.ndarray, centroids: np.ndarray, bits: int, accum_double: bool = False):
        self.lib = _load()
        self.Pi = np.ascontiguousarray(Pi, dtype=np.float32)
        self.centroids = np.ascontiguousarray(centroids, dtype=np.float32)
        self.bits = int(bits)
        self.D = self.Pi.shape[0]
        self.accum_double = int(bool(accum_double))
        assert self.centroids.size == 1 << self.bits

    def compress(self, x: np.ndarray, want_rotated: bool = True):
        flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.D)
        N = flat.shape[0]
        G = bytes_per_vector(self.D, self.bits)
        idx_bytes = np.empty((N, G), dtype=np.uint8)
        norms = np.empty(N, dtype=np.uint16)
        rotated = np.empty((N, self.D), dtype=np.float32) if want_rotated else None
        rc = self.lib.tqo_compress(flat, N, self.D, self.Pi, self.centroids, self.bits, self.accum_double,
                                   idx_bytes, norms,
                                   rotated.ctypes.data_as(ctypes.c_void_p) if want_rotated else None)
        if rc:
            raise RuntimeError(f"tqo_compress failed: {rc}")
        return {"idx_bytes": idx_bytes, "vec_norms": norms, "rotated": rotated}

    def decompress(self, idx_bytes: np.ndarray, vec_norms_bits: np.ndarray) -> np.ndarray:
        G = bytes_per_vector(self.D, self.bits)
        b = np.ascontiguousarray(idx_bytes, dtype=np.uint8).reshape(-1, G)
        n = np.ascontiguousarray(vec_norms_bits, dtype=np.uint16).reshape(-1)
        out = np.empty((b.shape[0], self.D), dtype=np.float32)
        rc = self.lib.tqo_decompress(b, n, b.shape[0], self.D, self.Pi, self.centroids, self.bits,
                                     self.accum_double, out)
        if rc:
            raise RuntimeError(f"tqo_decompress failed: {rc}")
        return out

    @staticmethod
    def threads() -> int:
        return _load().tqo_max_threads()

    @staticmethod
    def set_threads(n: int) -> None:
        _load().tqo_set_threads(n)


# --------------------------------------------------------------------------
# comparison helpers shared by the parity tests
# --------------------------------------------------------------------------
def unpack_codes(idx_bytes: np.ndarray, D: int, bits: int) -> np.ndarray:
    ipb = indices_per_byte(bits)
    mask = (1 << bits) - 1
    shifts = np.array([bits * i for i in range(ipb - 1, -1, -1)], dtype=np.int64)
    flat = idx_bytes.reshape(-1, idx_bytes.shape[-1]).astype(np.int64)
    return ((flat[:, :, None] >> shifts) & mask).reshape(flat.shape[0], -1)[:, :D].astype(np.int16)


def code_mismatch_report(test_bytes: np.ndarray, oracle_bytes: np.ndarray, rotated: np.ndarray,
                         centroids: np.ndarray, bits: int, window: float = 1e-5) -> dict:
    """Compare packed codes.  A differing coordinate is excused only if the oracle's rotated
    coordinate lies within `window` of the decision boundary (midpoint) between the two codes
    and the codes are neighbours.  Returns counts; `outside` must be zero for parity."""
    D = rotated.shape[-1]
    a = unpack_codes(test_bytes, D, bits)
    b = unpack_codes(oracle_bytes, D, bits)
    diff = a != b
    n_diff = int(diff.sum())
    outside = 0
    worst = 0.0
    if n_diff:
        r = rotated.reshape(-1, D)[diff].astype(np.float64)
        ia = a[diff].astype(np.int64)
        ib = b[diff].astype(np.int64)
        c = centroids.astype(np.float64)
        neighbours = np.abs(ia - ib) == 1
        lo = np.minimum(ia, ib)
        hi = np.minimum(lo + 1, len(c) - 1)
        boundary = 0.5 * (c[lo] + c[hi])
        dist = np.abs(r - boundary)
        ok = neighbours & (dist <= window)
        outside = int((~ok).sum())
        worst = float(dist.max())
    return {"coords": int(a.size), "differ": n_diff, "outside_window": outside,
            "worst_boundary_distance": worst,
            "padding_equal": bool(np.array_equal(test_bytes.shape, oracle_bytes.shape))}


def fp16_ulp_distance(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in fp16 units-in-the-last-place between two bit-pattern arrays (same sign assumed ok)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


# --------------------------------------------------------------------------
# one-query attention (checker for the packed-cache attention kernels)
# --------------------------------------------------------------------------
def attention_decode(q: np.ndarray, K: np.ndarray, V: np.ndarray, scale: float):
    """q [B,Hq,D], K and V [B,H,S,D] (query head j reads kv head j // (Hq/H)) ->
    (scores [B,Hq,S] = scale * q.k as in validate_v3.py:87, out [B,Hq,D] = softmax(scores) @ V), float64."""
    B, Hq, D = q.shape
    H = K.shape[1]
    G = Hq // H
    q4 = q.astype(np.float64).reshape(B, H, G, D)
    scores = np.einsum("bhgd,bhsd->bhgs", q4, K.astype(np.float64)) * scale
    m = scores.max(-1, keepdims=True) if scores.shape[-1] else scores
    p = np.exp(scores - m)
    p /= p.sum(-1, keepdims=True)
    out = np.einsum("bhgs,bhsd->bhgd", p, V.astype(np.float64))
    return scores.reshape(B, Hq, -1), out.reshape(B, Hq, D)
