"""
The V2 compressors of the reference (turboquant/compressors.py) on the MI355X kernels: `TurboQuantCompressorV2`
(keys: MSE codes of bits-1 bits plus one QJL sign bit per coordinate of the residual, scores straight from the
compressed form, compressors.py:25-158) and `TurboQuantCompressorMSE` (values, compressors.py:161-221).

Same constructor arguments, method names and score definition.  What `compress` returns for keys is the packed form
the reference's own memory accounting describes (validate.py:121-127: indices, sign bits, residual norm, vector
norm): packed MSE codes, fp16 norms, 16 bytes of sign bits and an fp16 residual norm per vector, 4.5x to 9x smaller than
the fp16 reconstruction plus int8 signs the reference materialises.  `asymmetric_attention_scores` takes that dict;
`reference_format` expands it into the reference's keys ("k_mse", "qjl_signs") for callers that look inside.
"""
from __future__ import annotations

import math

import torch

from . import _native
from .compressors_v3 import MSECompressor, _cached_centroids, _cached_rotation


def _qjl_matrix(head_dim: int, seed: int) -> torch.Tensor:
    """The Gaussian projection of compressors.py:49-52 (CPU generator, seed + 10000)."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed + 10000)
    return torch.randn(head_dim, head_dim, generator=gen)


def _check_v2_bits(bits: int) -> None:
    """The kernels of the key path take MSE codes of 1 ... 7 bits (bits - 1 of them: the packings of the V3 codec,
    decoded through a 128-entry-per-half table), so `bits` is 1 ... 8.  The reference also constructs with bits = 9
    (256 levels in a uint8 index, compressors.py:38-47); here that is a clear error at construction."""
    if not 1 <= int(bits) <= 8:
        raise ValueError(f"TurboQuantCompressorV2: bits must be 1 ... 8 on this implementation (got {bits}); "
                         "the reference's bits = 9 (8-bit MSE codes plus the sign bit) is not supported")


class TurboQuantCompressorV2:
    """Keys for asymmetric attention: interface of compressors.py:25-158."""

    def __init__(self, head_dim: int, bits: int, seed: int, device: str = "cpu"):
        _check_v2_bits(bits)
        self.head_dim = head_dim
        self.bits = bits
        self.mse_bits = max(bits - 1, 1)
        self.device = device
        pi_host = _cached_rotation(head_dim, seed)
        cent_host = _cached_centroids(head_dim, self.mse_bits)
        self._setup(pi_host, _qjl_matrix(head_dim, seed), cent_host)

    @classmethod
    def from_tensors(cls, Pi: torch.Tensor, S: torch.Tensor, centroids: torch.Tensor, bits: int, device: str = "cpu"):
        """A compressor over explicit matrices and codebook (parity tests pass the reference's own through here)."""
        _check_v2_bits(bits)
        self = cls.__new__(cls)
        self.head_dim = Pi.shape[0]
        self.bits = bits
        self.mse_bits = max(bits - 1, 1)
        self.device = device
        self._setup(Pi.detach().cpu().float(), S.detach().cpu().float(), centroids.detach().cpu().float())
        return self

    def _setup(self, pi_host: torch.Tensor, s_host: torch.Tensor, cent_host: torch.Tensor) -> None:
        import numpy as np
        dev = self.device
        self.Pi = pi_host.to(dev).contiguous()
        self.PiT = self.Pi.T.contiguous()
        self.S = s_host.to(dev).contiguous()
        self.centroids = cent_host.to(dev)
        self._mse = MSECompressor.from_tensors(pi_host, cent_host, self.mse_bits, device=dev)
        self._qjl_host = None
        self._qjl_tables = {}
        self._s_on = {}
        if self.head_dim != _native.HEAD_DIM:
            # The residual kernels are built for 128-wide heads.  Other head dimensions (8 to 256, what
            # the MSE stage takes) get their codes and norms from the same kernels and the residual part (reconstruction,
            # projection by S, signs, norm) from float32 tensor operations on the device: the reference's own arithmetic.
            return
        L = _native.lib()
        n = L.tq_qjl_table_bytes(self.head_dim, self.mse_bits)
        if n < 0:
            _native.check(int(n), "tq_qjl_table_bytes")
        blob = np.zeros(n, dtype=np.uint8)
        pi = np.ascontiguousarray(pi_host.numpy(), dtype=np.float32)
        s = np.ascontiguousarray(s_host.numpy(), dtype=np.float32)
        c = np.ascontiguousarray(cent_host.numpy(), dtype=np.float32)
        _native.check(L.tq_qjl_table_build(pi.ctypes.data, s.ctypes.data, c.ctypes.data, self.head_dim, self.mse_bits,
                                           blob.ctypes.data, blob.size), "tq_qjl_table_build")
        self._qjl_host = blob

    def _table(self, device) -> torch.Tensor:
        """The QJL table on `device` (the compressor itself may sit on the CPU, the reference's default)."""
        dev = torch.device(device)
        t = self._qjl_tables.get(dev)
        if t is None:
            if dev.type != "cuda":
                raise _native.TqError(f"TurboQuantCompressorV2: the codec runs on HIP devices only (asked for a table on {dev})")
            t = self._qjl_tables[dev] = torch.from_numpy(self._qjl_host).to(dev)
        return t

    def _s(self, device) -> torch.Tensor:
        dev = torch.device(device)
        if dev == self.S.device:
            return self.S
        t = self._s_on.get(dev)
        if t is None:
            t = self._s_on[dev] = self.S.to(dev)
        return t

    @torch.no_grad()
    def compress(self, states: torch.Tensor) -> dict:
        """(B, H, S, D) -> {"idx_bytes" u8 [B,H,S,G], "vec_norms" f16 [B,H,S], "sign_bytes" u8 [B,H,S,D/8],
        "residual_norm" f16 [B,H,S], "shape"}.  One call (tq_qjl_compress): a single pass over the input for 16-bit
        elements and MSE codes of up to 4 bits, MSE codes and norms followed by residual signs and norms otherwise."""
        B, H, S, D = states.shape
        _native._require_gpu(states, "states")
        if not states.is_contiguous():
            states = states.contiguous()
        if states.data_ptr() % 16:       # a contiguous view into the middle of a buffer: contiguous() would hand it back as it is
            states = states.clone(memory_format=torch.contiguous_format)
        if D != _native.HEAD_DIM:
            return self._compress_by_tensor_ops(states)
        out = self.empty_packed(B, H, S, states.device)
        n_vec = B * H * S
        if n_vec:
            with _native._on(states.device):
                rc = _native.lib().tq_qjl_compress(states.data_ptr(), _native.dtype_code(states.dtype), n_vec, D,
                                                   self._mse.table(states.device).data_ptr(), self._table(states.device).data_ptr(),
                                                   D, self.mse_bits, out["idx_bytes"].data_ptr(), out["vec_norms"].data_ptr(),
                                                   out["sign_bytes"].data_ptr(), out["residual_norm"].data_ptr(),
                                                   _native._stream_handle(states.device))
            _native.check(rc, "tq_qjl_compress")
        return out

    def _unpacked_codes(self, idx_bytes: torch.Tensor) -> torch.Tensor:
        """[.., G] packed bytes -> [.., D] codes (most significant code of a byte first)."""
        ipb = 8 // self.mse_bits
        shifts = torch.arange(ipb - 1, -1, -1, device=idx_bytes.device, dtype=torch.uint8) * self.mse_bits
        codes = (idx_bytes.unsqueeze(-1) >> shifts) & ((1 << self.mse_bits) - 1)
        return codes.reshape(*idx_bytes.shape[:-1], -1)[..., :self.head_dim].long()

    def _compress_by_tensor_ops(self, states: torch.Tensor) -> dict:
        """compress for head dimensions other than 128: codes and norms from the MSE kernels, then compressors.py:107-121
        as float32 tensor operations (reconstruction with the float32 norm, residual, its norm, projection, signs)."""
        B, H, S, D = states.shape
        dev = states.device
        first = self._mse.compress(states)
        x = states.reshape(-1, D).float()
        norms = torch.norm(x, dim=-1, keepdim=True)
        k_mse = (self._mse.centroids.to(dev)[self._unpacked_codes(first["idx_bytes"]).reshape(-1, D)] @ self._mse.pi(dev)) * norms
        residual = x - k_mse
        signs = (residual @ self._s(dev).T) >= 0
        weights = torch.tensor([128, 64, 32, 16, 8, 4, 2, 1], device=dev, dtype=torch.int32)      # coordinate 8b + k in bit 7 - k
        if D % 8:       # the bits of the last byte a vector does not fill stay clear
            signs = torch.nn.functional.pad(signs, (0, 8 - D % 8))
        sign_bytes = (signs.reshape(-1, -(-D // 8), 8).to(torch.int32) * weights).sum(-1).to(torch.uint8)
        return {"idx_bytes": first["idx_bytes"], "vec_norms": first["vec_norms"], "sign_bytes": sign_bytes.reshape(B, H, S, -(-D // 8)),
                "residual_norm": torch.norm(residual, dim=-1).to(torch.float16).reshape(B, H, S), "shape": (B, H, S, D)}

    def empty_packed(self, B: int, H: int, S: int, device) -> dict:
        """The packed dictionary `compress` fills, with uninitialised buffers."""
        D = self.head_dim
        G = -(-D // (8 // self.mse_bits))
        return {"idx_bytes": torch.empty((B, H, S, G), dtype=torch.uint8, device=device),
                "vec_norms": torch.empty((B, H, S), dtype=torch.float16, device=device),
                "sign_bytes": torch.empty((B, H, S, -(-D // 8)), dtype=torch.uint8, device=device),
                "residual_norm": torch.empty((B, H, S), dtype=torch.float16, device=device), "shape": (B, H, S, D)}

    def job(self, states: torch.Tensor, packed: dict) -> dict:
        """A record for `_native.QjlJobList` (one launch for the keys of many layers): `states` compressed into `packed`."""
        return {"states": states, "idx_bytes": packed["idx_bytes"], "vec_norms": packed["vec_norms"], "sign_bytes": packed["sign_bytes"],
                "residual_norm": packed["residual_norm"], "table": self._mse.table(states.device), "qjl_table": self._table(states.device),
                "mse_bits": self.mse_bits}

    @torch.no_grad()
    def reference_format(self, compressed: dict) -> dict:
        """The dictionary the reference's compress returns (:119-124): "k_mse" fp16 [B,H,S,D], "qjl_signs" int8 in
        {-1,+1} [B,H,S,D], "residual_norm", "shape", expanded from the packed form."""
        B, H, S, D = compressed["shape"]
        k_mse = self._mse.decompress({"idx_bytes": compressed["idx_bytes"], "vec_norms": compressed["vec_norms"],
                                      "shape": (B, H, S, D), "idx_pad": -D % (8 // self.mse_bits)}).to(torch.float16)
        shifts = torch.arange(7, -1, -1, device=compressed["sign_bytes"].device, dtype=torch.uint8)
        bits = (compressed["sign_bytes"].unsqueeze(-1) >> shifts) & 1
        signs = (bits.to(torch.int8) * 2 - 1).reshape(B, H, S, -1)[..., :D]
        return {"k_mse": k_mse, "qjl_signs": signs, "residual_norm": compressed["residual_norm"], "shape": (B, H, S, D)}

    @torch.no_grad()
    def asymmetric_attention_scores(self, queries: torch.Tensor, compressed: dict) -> torch.Tensor:
        """<q, k> ~ <q, k_mse> + ||r|| sqrt(pi/2)/m <S q, sign(S r)>  (:124-158): queries (B, H, S_q, D) against a dict
        from compress -> float32 (B, H, S_q, S_k).  Both terms are computed from the packed bytes (the query is
        rotated by Pi for the first and projected by S for the second; neither the reconstruction nor the signs are
        expanded).  A dict in the reference's format (`reference_format`) is accepted too and takes plain matrix
        products."""
        m = self.S.shape[0]
        corr = math.sqrt(math.pi / 2) / m
        if "idx_bytes" not in compressed:
            k_mse = compressed["k_mse"].float()
            term1 = torch.matmul(queries.float(), k_mse.transpose(-2, -1))
            ip = torch.matmul(torch.matmul(queries.float(), self._s(queries.device).T), compressed["qjl_signs"].float().transpose(-2, -1))
            return term1 + corr * ip * compressed["residual_norm"].float().unsqueeze(-2)
        B, H, S_k, D = compressed["shape"]
        S_q = queries.shape[2]
        out = torch.empty((B, H, S_q, S_k), dtype=torch.float32, device=queries.device)
        if out.numel() == 0:
            return out
        _native._require_gpu(queries, "queries")
        q = queries.float()
        dev = q.device
        if D != _native.HEAD_DIM:       # other head dimensions: the reconstruction from the MSE kernels, the rest as tensor operations
            exp = self.reference_format(compressed)
            term1 = torch.matmul(q, exp["k_mse"].float().transpose(-2, -1))
            ip = torch.matmul(torch.matmul(q, self._s(dev).T), exp["qjl_signs"].float().transpose(-2, -1))
            return term1 + corr * ip * compressed["residual_norm"].float().unsqueeze(-2)
        q_rot = torch.matmul(q, self._mse.pi_transposed(dev)).contiguous()          # Pi q for every query token
        st = self._s_on.get(("t", dev))
        if st is None:
            st = self._s_on[("t", dev)] = (self._s(dev).T * corr).contiguous()      # sqrt(pi/2)/m S^T, made once per device
        q_sign = torch.matmul(q, st).contiguous()
        packed = [compressed[k] if compressed[k].is_contiguous() else compressed[k].contiguous()
                  for k in ("idx_bytes", "vec_norms", "sign_bytes", "residual_norm")]
        with _native._on(dev):
            rc = _native.lib().tq_qjl_scores(packed[0].data_ptr(), packed[1].data_ptr(), packed[2].data_ptr(), packed[3].data_ptr(),
                                             B * H, S_k, self._mse.table(dev).data_ptr(), D, self.mse_bits,
                                             q_rot.data_ptr(), q_sign.data_ptr(), S_q, out.data_ptr(), _native._stream_handle(dev))
        _native.check(rc, "tq_qjl_scores")
        return out


class TurboQuantCompressorMSE:
    """Values: MSE codes only, interface of compressors.py:161-221.  `compress` returns the reference's keys
    ("indices" one code per byte [N, D], "vec_norms" fp16 [N], "shape") next to the packed bytes the kernels wrote;
    `decompress` reads the packed bytes when they are there and packs the indices otherwise."""

    def __init__(self, head_dim: int, bits: int, seed: int, device: str = "cpu"):
        self.head_dim = head_dim
        self.bits = bits
        self.device = device
        self._mse = MSECompressor(head_dim, bits, seed, device=device)
        self.Pi = self._mse.Pi
        self.centroids = self._mse.centroids

    @torch.no_grad()
    def compress(self, states: torch.Tensor) -> dict:
        B, H, S, D = states.shape
        packed = self._mse.compress(states)
        ipb = 8 // self.bits
        shifts = torch.arange(ipb - 1, -1, -1, device=states.device, dtype=torch.uint8) * self.bits
        codes = (packed["idx_bytes"].reshape(B * H * S, -1, 1) >> shifts) & ((1 << self.bits) - 1)
        return {"indices": codes.reshape(B * H * S, -1)[:, :D].contiguous(), "vec_norms": packed["vec_norms"].reshape(-1),
                "shape": (B, H, S, D), "idx_bytes": packed["idx_bytes"]}

    @torch.no_grad()
    def decompress(self, compressed: dict) -> torch.Tensor:
        B, H, S, D = compressed["shape"]
        idx_bytes = compressed.get("idx_bytes")
        if idx_bytes is None:
            ipb = 8 // self.bits
            codes = compressed["indices"].reshape(B * H * S, D).to(torch.int32)
            if D % ipb:     # compressors_v3.py:64-68: zero codes up to a whole byte
                codes = torch.nn.functional.pad(codes, (0, ipb - D % ipb))
            codes = codes.reshape(B * H * S, -1, ipb)
            weights = torch.tensor([1 << (self.bits * i) for i in range(ipb - 1, -1, -1)], device=codes.device, dtype=torch.int32)
            idx_bytes = (codes * weights).sum(-1).to(torch.uint8).reshape(B, H, S, -1)
        return self._mse.decompress({"idx_bytes": idx_bytes, "vec_norms": compressed["vec_norms"].reshape(B, H, S),
                                     "shape": (B, H, S, D), "idx_pad": -D % (8 // self.bits)})
