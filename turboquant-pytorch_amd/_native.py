"""
Loader, builder and Python bindings of the C-ABI library `csrc/libtqamd.so`
(declared in include/tqamd.h), plus the `torch.library` custom ops that put the
HIP kernels behind ordinary tensor calls.

There is no CPU implementation and no fallback: if the library is missing, or a
tensor is not on a HIP device, the calls raise.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(CSRC, "libtqamd.so")
SOURCES = ("tq_host.cpp", "tq_compress.hip", "tq_decompress.hip", "tq_anydim.hip", "tq_wide.hip", "tq_attend.hip", "tq_qjl.hip")
HEADERS = ("tq_table.h", "tq_device.h", "tq_anydim.h", "tq_wide.h", os.path.join("..", "..", "include", "tqamd.h"))
GPU_ARCH = "gfx950"

TQ_F32, TQ_F16, TQ_BF16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: TQ_F32, torch.float16: TQ_F16, torch.bfloat16: TQ_BF16}
HEAD_DIM = 128


class TqError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


# ------------------------------------------------------------------------------------
# build
# ------------------------------------------------------------------------------------
OBJ_DIR = os.path.join(CSRC, "build")
# The "memory skeleton" build of the two codec kernels: same loads, LDS traffic, barriers and stores, with the matrix
# instructions and the code search (compress) or the decode, matrix instructions and operand reads (decompress) left
# out.  Its output is garbage; it exists to time what the memory pattern alone costs (bench.py --skeleton).
SKELETON_LIB_PATH = os.path.join(CSRC, "libtqamd_skeleton.so")
SKELETON_SOURCES = ("tq_compress.hip", "tq_decompress.hip")
SKELETON_DEFINES = ("-DTQ_SKELETON=1",)


def hipcc_flags() -> List[str]:
    return ["-fPIC", "-O3", "-std=c++17", f"--offload-arch={GPU_ARCH}",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Wno-unused-command-line-argument",
            # The ticket draws are single-lane atomics whose result is needed a tile's work later.  The atomic optimizer
            # would turn each into a wave-wide scan with a read-first-lane of the result, i.e. a wait for every memory
            # operation of the wave right behind the atomic.
            "-mllvm", "-amdgpu-atomic-optimizer-strategy=None",
            "-Wno-inline-asm"]      # the direct-to-LDS loads name m0 as clobbered, which clang reports as a reserved register


def _hipcc() -> str:
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _run(cmd: List[str]) -> str:
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    return res.stderr


def _compile_objects(tag: str, defines: Sequence[str], only: Optional[Sequence[str]], force: bool, verbose: bool) -> Dict[str, str]:
    """One object per source under csrc/build, compiled side by side; `only`: the sources that take `defines`
    (their objects carry `tag` in the name), the others are the plain objects.  Up-to-date objects are kept unless `force`."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OBJ_DIR, exist_ok=True)
    newest_header = max(os.path.getmtime(os.path.join(CSRC, h)) for h in HEADERS)
    jobs, objs = [], {}
    for src in SOURCES:
        special = bool(defines) and (only is None or src in only)
        obj = os.path.join(OBJ_DIR, src + ("." + tag if special else "") + ".o")
        objs[src] = obj
        path = os.path.join(CSRC, src)
        if not force and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(path), newest_header):
            continue
        jobs.append([_hipcc(), *hipcc_flags(), *(defines if special else ()), "-c", path, "-o", obj])
    if jobs:
        with ThreadPoolExecutor(max_workers=min(len(jobs), max(1, (os.cpu_count() or 2) - 1))) as pool:
            for err in pool.map(_run, jobs):
                if verbose and err:
                    print(err)
    return objs


def _link(objs: Dict[str, str], out_path: str) -> None:
    tmp = out_path + ".tmp"
    _run([_hipcc(), "-shared", "-fPIC", f"--offload-arch={GPU_ARCH}", *objs.values(), "-o", tmp])
    os.replace(tmp, out_path)


def build(force: bool = True, verbose: bool = False) -> str:
    """Compile the HIP/C++ sources into csrc/libtqamd.so (cross-compiles without a GPU): one object per source,
    compiled in parallel, then linked."""
    if not force and os.path.exists(LIB_PATH):
        newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in SOURCES + HEADERS)
        if os.path.getmtime(LIB_PATH) >= newest:
            return LIB_PATH
    _link(_compile_objects("", (), None, force, verbose), LIB_PATH)
    return LIB_PATH


def build_skeleton(force: bool = True, verbose: bool = False) -> str:
    """csrc/libtqamd_skeleton.so: the library with the memory-skeleton form of the compress and decompress kernels
    (a measurement aid, never loaded by the package itself)."""
    _compile_objects("", (), None, False, verbose)                       # the plain objects, if a build has not left them
    _link(_compile_objects("skeleton", SKELETON_DEFINES, SKELETON_SOURCES, force, verbose), SKELETON_LIB_PATH)
    return SKELETON_LIB_PATH


# ------------------------------------------------------------------------------------
# ctypes view of include/tqamd.h
# ------------------------------------------------------------------------------------
class TqJob(ctypes.Structure):
    _fields_ = [
        ("states", ctypes.c_void_p),
        ("idx_bytes", ctypes.c_void_p),
        ("vec_norms", ctypes.c_void_p),
        ("table_dev", ctypes.c_void_p),
        ("rows", ctypes.c_longlong),
        ("tokens", ctypes.c_longlong),
        ("row_stride", ctypes.c_longlong),
        ("token_stride", ctypes.c_longlong),
        ("bits", ctypes.c_int),
        ("dtype", ctypes.c_int),
        ("packed_row_stride", ctypes.c_longlong),
    ]


class TqQjlJob(ctypes.Structure):
    _fields_ = [
        ("states", ctypes.c_void_p),
        ("idx_bytes", ctypes.c_void_p),
        ("vec_norms", ctypes.c_void_p),
        ("sign_bytes", ctypes.c_void_p),
        ("residual_norm", ctypes.c_void_p),
        ("table_dev", ctypes.c_void_p),
        ("qjl_table_dev", ctypes.c_void_p),
        ("n_vec", ctypes.c_longlong),
        ("token_stride", ctypes.c_longlong),
        ("mse_bits", ctypes.c_int),
        ("dtype", ctypes.c_int),
    ]


EXPORTS = (
    "tq_abi_version", "tq_status_string", "tq_device_count", "tq_bytes_per_vector",
    "tq_decision_thresholds", "tq_table_bytes", "tq_table_build", "tq_table_check", "tq_table_quantize_host",
    "tq_compress", "tq_decompress", "tq_compress_batched", "tq_decompress_batched", "tq_workspace_bytes",
    "tq_decompress_batched_noalloc", "tq_qjl_table_bytes", "tq_qjl_table_build", "tq_qjl_signs",
    "tq_qjl_compress", "tq_qjl_compress_batched", "tq_qjl_scores",
    "tq_scores", "tq_weighted_values", "tq_weighted_values_splits", "tq_attend_partials", "tq_attend_splits",
    "tq_attend_prepare", "tq_attend_merge", "tq_append_token", "tq_attend_step",
)

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise TqError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation.")
    L = ctypes.CDLL(LIB_PATH)
    vp, ll, ci = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int
    L.tq_abi_version.restype = ci
    L.tq_status_string.restype = ctypes.c_char_p
    L.tq_status_string.argtypes = [ci]
    L.tq_device_count.restype = ci
    L.tq_bytes_per_vector.argtypes = [ci, ci]
    L.tq_decision_thresholds.argtypes = [vp, ci, vp]
    L.tq_table_bytes.restype = ll
    L.tq_table_bytes.argtypes = [ci, ci]
    L.tq_table_build.argtypes = [vp, vp, ci, ci, vp, ctypes.c_size_t]
    L.tq_table_check.argtypes = [vp, ctypes.c_size_t, ci, ci]
    L.tq_table_quantize_host.argtypes = [vp, vp, ll, vp]
    L.tq_compress.argtypes = [vp, ci, ll, ll, ll, ll, vp, ci, ci, vp, vp, ll, vp, vp]
    L.tq_decompress.argtypes = [vp, vp, ll, ll, ll, vp, ci, ci, vp, ci, ll, ll, vp, vp]
    L.tq_workspace_bytes.restype = ll
    L.tq_workspace_bytes.argtypes = [ci]
    L.tq_compress_batched.argtypes = [vp, vp, ci, ci, vp, vp]
    L.tq_scores.argtypes = [vp, vp, ll, ll, ll, vp, ci, ci, vp, ci, vp, ll, vp]
    L.tq_weighted_values_splits.argtypes = [ll, ll]
    L.tq_attend_splits.argtypes = [ll, ll]
    L.tq_attend_prepare.argtypes = [vp, ci, ll, ci, ctypes.c_float, vp, vp, vp, ci, ll, ll, vp, vp, vp]
    L.tq_attend_merge.argtypes = [vp, ci, vp, vp, ll, ci, vp, ci, vp]
    L.tq_attend_partials.argtypes = [vp, vp, vp, vp, ll, ll, ll, vp, vp, ci, ci, ci, vp, ci, ci, vp, vp]
    L.tq_weighted_values.argtypes = [vp, vp, ll, ll, ll, vp, ci, ci, vp, ll, ci, vp, ci, vp, vp]
    L.tq_decompress_batched.argtypes = [vp, vp, ci, ci, vp, vp]
    L.tq_decompress_batched_noalloc.argtypes = [vp, vp, ci, ci, vp]
    L.tq_qjl_table_bytes.restype = ll
    L.tq_qjl_table_bytes.argtypes = [ci, ci]
    L.tq_qjl_table_build.argtypes = [vp, vp, vp, ci, ci, vp, ctypes.c_size_t]
    L.tq_qjl_signs.argtypes = [vp, ci, ll, ll, vp, vp, ci, ci, vp, vp, vp]
    L.tq_qjl_compress.argtypes = [vp, ci, ll, ll, vp, vp, ci, ci, vp, vp, vp, vp, vp]
    L.tq_qjl_compress_batched.argtypes = [vp, vp, ci, ci, vp]
    L.tq_qjl_scores.argtypes = [vp, vp, vp, vp, ll, ll, vp, ci, ci, vp, vp, ll, vp, vp]
    L.tq_append_token.argtypes = [vp, vp, ci, ll, ll, vp, vp, ll, ll, ll, vp, vp, ci, ci, ci, vp, vp, vp, vp, ll, ll, ll, vp]
    L.tq_attend_step.argtypes = [vp, ci, ll, ci, ctypes.c_float, vp, vp, vp, vp, ci, ll, ll, vp, vp, vp, vp, ll, ll,
                                 vp, vp, ci, ci, ci, vp, vp, vp, ci, vp, ci, vp]
    for name in EXPORTS:
        if name not in ("tq_status_string", "tq_table_bytes", "tq_workspace_bytes", "tq_qjl_table_bytes"):
            getattr(L, name).restype = ci
    _lib = L
    return L


def check(status: int, what: str) -> None:
    if status != 0:
        msg = lib().tq_status_string(status).decode()
        raise TqError(f"{what}: {msg} (status {status})")


# ------------------------------------------------------------------------------------
# host-side table construction
# ------------------------------------------------------------------------------------
def decision_thresholds(centroids: np.ndarray) -> np.ndarray:
    c = np.ascontiguousarray(centroids, dtype=np.float32)
    out = np.empty(max(c.size - 1, 0), dtype=np.float32)
    check(lib().tq_decision_thresholds(c.ctypes.data, c.size, out.ctypes.data), "tq_decision_thresholds")
    return out


def build_table(Pi: torch.Tensor, centroids: torch.Tensor, bits: int) -> np.ndarray:
    """Bake rotation + codebook into the codec-table blob (host, uint8 array)."""
    pi = np.ascontiguousarray(Pi.detach().cpu().to(torch.float32).numpy())
    cent = np.ascontiguousarray(centroids.detach().cpu().to(torch.float32).numpy())
    d = pi.shape[0]
    if pi.shape != (d, d):
        raise ValueError("Pi must be square")
    if cent.size != 1 << bits:
        raise ValueError(f"expected {1 << bits} centroids, got {cent.size}")
    nbytes = lib().tq_table_bytes(d, bits)
    if nbytes < 0:
        check(int(nbytes), "tq_table_bytes")
    blob = np.zeros(nbytes, dtype=np.uint8)
    check(lib().tq_table_build(pi.ctypes.data, cent.ctypes.data, d, bits, blob.ctypes.data, blob.size), "tq_table_build")
    return blob


# The launch entry points take a table in device memory and a bit width that selects the kernel; nothing on the
# device side can tell them apart when they disagree (the codes would be garbage, silently).  Every table this
# module uploads therefore carries the width it was built for as an attribute of the tensor object, and every launch
# checks its pair.  (The tag lives and dies with the tensor: a map keyed by device address would keep entries of
# freed tables, and a later upload that the allocator places at the same address would meet a stale one.)
_TABLE_TAG = "_tq_table_width"


def upload_table(blob: np.ndarray, head_dim: int, bits: int, device: torch.device) -> torch.Tensor:
    """Device copy of a blob from build_table, after tq_table_check(blob, head_dim, bits)."""
    check(lib().tq_table_check(blob.ctypes.data, blob.size, head_dim, bits), "tq_table_check")
    t = torch.from_numpy(blob).to(device)
    setattr(t, _TABLE_TAG, (head_dim, bits))
    return t


def check_table(table: torch.Tensor, head_dim: int, bits: int) -> None:
    """Raises if `table` was uploaded for another (head_dim, bits).  Tables this module never saw (a caller's own
    upload) pass: their owner has to make the check, with tq_table_check on the host copy."""
    known = getattr(table, _TABLE_TAG, None)
    if known is not None and known != (head_dim, 8 if bits > 8 else bits):
        raise TqError(f"codec table built for head_dim {known[0]}, {known[1]} bits used with head_dim {head_dim}, {bits} bits")


def quantize_host(table: np.ndarray, r: np.ndarray) -> np.ndarray:
    """Table self-check used by the tests: the kernels' code search, emulated on the host."""
    rr = np.ascontiguousarray(r, dtype=np.float32).reshape(-1)
    out = np.empty(rr.size, dtype=np.uint8)
    check(lib().tq_table_quantize_host(table.ctypes.data, rr.ctypes.data, rr.size, out.ctypes.data), "tq_table_quantize_host")
    return out.reshape(np.shape(r))


# ------------------------------------------------------------------------------------
# tensor plumbing
# ------------------------------------------------------------------------------------
def _require_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise TqError(f"{what} must live on a HIP device (got {t.device}); this package has no CPU path")


ERR_ALIGN = -8      # TQ_ERR_ALIGN of include/tqamd.h


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise TqError(f"unsupported element type {dt}; float32, float16 and bfloat16 are supported") from None


def _vector_alignment(head_dim: int, elem_bytes: int) -> int:
    """Bytes the vectors' address and strides must be a multiple of: 16, except for head dimensions that are not a
    multiple of 32, which the kernels move element by element."""
    return elem_bytes if head_dim % 32 else 16


def vector_layout(t: torch.Tensor) -> Optional[Tuple[int, int, int, int]]:
    """(rows, tokens, row_stride, token_stride) in elements for a [B,H,S,D] tensor whose last
    dimension is dense, or None if its strides do not reduce to the two-level form."""
    B, H, S, D = t.shape
    sb, sh, ss, sd = t.stride()
    if D != 1 and sd != 1:
        return None
    esz = t.element_size()
    align = _vector_alignment(D, esz)
    if (t.data_ptr() % align) or any((s * esz) % align for s in (sb, sh, ss)):
        return None
    n = B * H * S
    if n == 0:
        return (0, 0, 0, D)
    # drop dimensions of extent 1, then try to merge (b,h,s) left to right
    dims = [(e, s) for e, s in ((B, sb), (H, sh), (S, ss)) if e != 1]
    if not dims:
        return (1, 1, 0, D)
    merged = [dims[0]]
    for e, s in dims[1:]:
        pe, ps = merged[-1]
        if ps == e * s:
            merged[-1] = (pe * e, s)
        else:
            merged.append((e, s))
    if len(merged) == 1:
        return (1, merged[0][0], 0, merged[0][1])
    if len(merged) == 2:
        return (merged[0][0], merged[1][0], merged[0][1], merged[1][1])
    return None


def row_layout(t: torch.Tensor) -> Optional[Tuple[int, int, int, int]]:
    """Like vector_layout, but always rows = B*H and tokens = S (the form a per-row packed store
    needs); None if the batch and head dimensions do not merge."""
    B, H, S, D = t.shape
    sb, sh, ss, sd = t.stride()
    if D != 1 and sd != 1:
        return None
    esz = t.element_size()
    align = _vector_alignment(D, esz)
    if (t.data_ptr() % align) or any((st * esz) % align for st in (sb, sh, ss)):
        return None
    if B != 1 and H != 1 and sb != H * sh:
        return None
    row_stride = sh if H != 1 else sb
    return (B * H, S, row_stride if B * H > 1 else 0, ss if S > 1 else D)


def packed_row_stride(idx_bytes: torch.Tensor, vec_norms: torch.Tensor) -> Optional[int]:
    """Packed slots per (batch, head) row of a [B,H,S,G] / [B,H,S] pair of packed buffers: 0 when
    both are contiguous, the row capacity when they are token-axis slices of a [B,H,capacity,..]
    store, None when they are neither."""
    if idx_bytes.is_contiguous() and vec_norms.is_contiguous():
        return 0
    B, H, S, G = idx_bytes.shape
    if tuple(vec_norms.shape) != (B, H, S):
        return None
    sb, sh, ss, sg = idx_bytes.stride()
    nb, nh, ns = vec_norms.stride()
    if sg != 1 or ss != G or ns != 1 or sh % G or sh // G != nh or sh // G < S:
        return None
    if B != 1 and (sb != H * sh or nb != H * nh):
        return None
    return sh // G


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)     # what torch's own launchers use: no Stream object


def _stream_handle(device: torch.device) -> int:
    """The current HIP stream of `device` as an integer handle."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _NoScope:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SCOPE = _NoScope()


def _on(device: torch.device):
    """Context that makes `device` current for a launch; free when it already is (the usual case)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SCOPE
    return torch.cuda.device(device)


_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, stream: int) -> int:
    """Address of the ticket counters tq_compress / tq_decompress draw their tiles from, or 0 (fixed assignment of tiles).
    One zero-filled buffer per (device, stream): launches on one stream run one after the other and each
    leaves the counters at zero, launches on different streams never share.  While a graph is being
    captured the answer is 0: the graph may be replayed on any stream, next to eager launches on this one."""
    if torch.cuda.is_current_stream_capturing():
        return 0
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.zeros(int(lib().tq_workspace_bytes(1)), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws.data_ptr()


def _drop_workspace(device: torch.device, stream: int) -> None:
    """Forget the counters kept for (device, stream) after a call that reported an error: the contract "zero before,
    zero after" only holds for launches that complete, so the next call gets fresh zeroed counters."""
    _workspaces.pop((device.index if device.index is not None else torch.cuda.current_device(), stream), None)


_step_scratch: Dict[Tuple[int, int], torch.Tensor] = {}


def step_scratch(device: torch.device, stream: int, floats: int) -> Optional[torch.Tensor]:
    """float32 scratch of a decode step (rotated queries, window record, split records), one buffer per
    (device, stream), grown on demand: the steps of all layers on a stream run one after the other.  One entry per
    stream that ever ran a decode step, kept for the life of the process (a few hundred KiB each).
    None while a graph is being captured: the caller then takes the general path, whose scratch comes from the
    graph's own memory pool."""
    if torch.cuda.is_current_stream_capturing():
        return None      # a captured step may be replayed on any stream, next to eager steps that use this buffer
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    buf = _step_scratch.get(key)
    if buf is None or buf.numel() < floats:
        buf = _step_scratch[key] = torch.empty(max(floats, 1 << 16), dtype=torch.float32, device=device)
    return buf


def compress_into(states: torch.Tensor, table: torch.Tensor, bits: int,
                  idx_bytes: torch.Tensor, vec_norms: torch.Tensor) -> None:
    """Launch tq_compress on `states` ([B,H,S,128], any supported float type, last dim dense).
    The packed buffers are contiguous, or token-axis slices of a [B,H,capacity,..] store."""
    _require_gpu(states, "states")
    _require_gpu(table, "codec table")
    prs = packed_row_stride(idx_bytes, vec_norms)
    if prs is None:
        raise TqError("packed buffers must be contiguous or token-axis slices of one [B,H,capacity,..] store")
    lay = row_layout(states) if prs else vector_layout(states)
    if lay is None:
        states = states.contiguous()
        lay = row_layout(states) if prs else vector_layout(states)
    rows, tokens, row_stride, token_stride = lay
    check_table(table, states.shape[-1], bits)
    with _on(states.device):
        stream = _stream_handle(states.device)
        # counters only where the kernel can use them (a large single-row job): a one-token append needs no look-up
        ws = _workspace(states.device, stream) if rows == 1 and tokens >= 65536 else 0
        rc = lib().tq_compress(states.data_ptr(), dtype_code(states.dtype), rows, tokens, row_stride, token_stride,
                               table.data_ptr(), states.shape[-1], bits,
                               idx_bytes.data_ptr(), vec_norms.data_ptr(), prs, ws, stream)
    if rc and ws:
        _drop_workspace(states.device, stream)
    check(rc, "tq_compress")


def decompress_into(idx_bytes: torch.Tensor, vec_norms: torch.Tensor, table: torch.Tensor, bits: int,
                    out: torch.Tensor) -> None:
    """Launch tq_decompress, writing vector n of the packed stream to `out` ([B,H,S,128] view).
    The packed buffers are contiguous, or token-axis slices of a [B,H,capacity,..] store."""
    _require_gpu(idx_bytes, "idx_bytes")
    _require_gpu(out, "output")
    prs = packed_row_stride(idx_bytes, vec_norms)
    if prs is None:
        idx_bytes, vec_norms, prs = idx_bytes.contiguous(), vec_norms.contiguous(), 0
    lay = row_layout(out) if prs else vector_layout(out)
    if lay is None:
        raise TqError("decompress output must have a dense last dimension, 16-byte aligned rows and at most "
                      "two stride levels")
    rows, tokens, row_stride, token_stride = lay
    check_table(table, out.shape[-1], bits)
    with _on(out.device):
        stream = _stream_handle(out.device)
        rc = lib().tq_decompress(idx_bytes.data_ptr(), vec_norms.data_ptr(), prs, rows, tokens, table.data_ptr(),
                                 out.shape[-1], bits, out.data_ptr(), dtype_code(out.dtype), row_stride,
                                 token_stride, _workspace(out.device, stream), stream)
    if rc:
        _drop_workspace(out.device, stream)
    check(rc, "tq_decompress")


# ------------------------------------------------------------------------------------
# torch.library custom ops (so the kernels compose with the dispatcher, autocast guards,
# fake tensors and graph capture like any other operator)
# ------------------------------------------------------------------------------------
def _packed_width(head_dim: int, bits: int) -> int:
    ipb = 8 // bits
    return -(-head_dim // ipb)


def _compress_impl(states: torch.Tensor, table: torch.Tensor, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    B, H, S, D = states.shape
    idx_bytes = torch.empty((B, H, S, _packed_width(D, bits)), dtype=torch.uint8, device=states.device)
    vec_norms = torch.empty((B, H, S), dtype=torch.float16, device=states.device)
    compress_into(states, table, bits, idx_bytes, vec_norms)
    return idx_bytes, vec_norms


compress_op = torch.library.custom_op("tqamd::compress", _compress_impl,
                                      mutates_args=(), device_types="cuda")


@compress_op.register_fake
def _(states, table, bits):
    B, H, S, D = states.shape
    return (states.new_empty((B, H, S, _packed_width(D, bits)), dtype=torch.uint8),
            states.new_empty((B, H, S), dtype=torch.float16))


def _compress_into_impl(states: torch.Tensor, table: torch.Tensor, bits: int,
                        idx_bytes: torch.Tensor, vec_norms: torch.Tensor) -> None:
    compress_into(states, table, bits, idx_bytes, vec_norms)


compress_into_op = torch.library.custom_op("tqamd::compress_into", _compress_into_impl,
                                           mutates_args=("idx_bytes", "vec_norms"), device_types="cuda")


def _decompress_impl(idx_bytes: torch.Tensor, vec_norms: torch.Tensor, table: torch.Tensor, bits: int,
                     head_dim: int, out_dtype: torch.dtype) -> torch.Tensor:
    B, H, S, _ = idx_bytes.shape
    out = torch.empty((B, H, S, head_dim), dtype=out_dtype, device=idx_bytes.device)
    decompress_into(idx_bytes, vec_norms, table, bits, out)
    return out


decompress_op = torch.library.custom_op("tqamd::decompress", _decompress_impl,
                                        mutates_args=(), device_types="cuda")


@decompress_op.register_fake
def _(idx_bytes, vec_norms, table, bits, head_dim, out_dtype):
    B, H, S, _ = idx_bytes.shape
    return idx_bytes.new_empty((B, H, S, head_dim), dtype=out_dtype)


def _decompress_into_impl(idx_bytes: torch.Tensor, vec_norms: torch.Tensor, table: torch.Tensor, bits: int,
                          out: torch.Tensor) -> None:
    decompress_into(idx_bytes, vec_norms, table, bits, out)


decompress_into_op = torch.library.custom_op("tqamd::decompress_into", _decompress_into_impl,
                                             mutates_args=("out",), device_types="cuda")


def _packed_rows(idx_bytes: torch.Tensor, vec_norms: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, int, int, int]:
    """(idx_bytes, vec_norms, packed_row_stride, rows, tokens) of a [B,H,S,G] / [B,H,S] packed pair for
    the row-wise entry points (copies only if the pair is not a slice of one per-row store)."""
    prs = packed_row_stride(idx_bytes, vec_norms)
    if prs is None:
        idx_bytes, vec_norms, prs = idx_bytes.contiguous(), vec_norms.contiguous(), 0
    B, H, S, _ = idx_bytes.shape
    return idx_bytes, vec_norms, prs, B * H, S


def _scores_into_impl(idx_bytes: torch.Tensor, vec_norms: torch.Tensor, table: torch.Tensor, bits: int,
                      q_rot: torch.Tensor, scores: torch.Tensor) -> None:
    """scores[b, h*G + g, t] = q_rot[b, h*G + g] . centroids[codes(b, h, t)] * norm(b, h, t), written into
    `scores` ([B, Hq, S] float32 view whose last dimension is dense and whose heads are equally spaced)."""
    _require_gpu(idx_bytes, "idx_bytes")
    idx_bytes, vec_norms, prs, rows, tokens = _packed_rows(idx_bytes, vec_norms)
    B, Hq, D = q_rot.shape
    group = Hq // idx_bytes.shape[1]
    if scores.dtype != torch.float32 or tuple(scores.shape) != (B, Hq, tokens) or (tokens > 1 and scores.stride(2) != 1) \
            or (Hq > 1 and B > 1 and scores.stride(0) != Hq * scores.stride(1)):
        raise TqError("scores must be a float32 [B, Hq, S] view with a dense last dimension and evenly spaced heads")
    q_rot = q_rot.to(torch.float32).contiguous()
    stride = scores.stride(1) if Hq > 1 else (scores.stride(0) if B > 1 else max(tokens, 1))
    with _on(idx_bytes.device):
        rc = lib().tq_scores(idx_bytes.data_ptr(), vec_norms.data_ptr(), prs, rows, tokens, table.data_ptr(), D, bits,
                             q_rot.data_ptr(), group, scores.data_ptr(), stride, _stream_handle(idx_bytes.device))
    check(rc, "tq_scores")


scores_into_op = torch.library.custom_op("tqamd::scores_into", _scores_into_impl,
                                         mutates_args=("scores",), device_types="cuda")


def _weighted_values_impl(idx_bytes: torch.Tensor, vec_norms: torch.Tensor, table: torch.Tensor, bits: int,
                          weights: torch.Tensor, head_dim: int) -> torch.Tensor:
    """out[b, h*G + g] = sum_t weights[b, h*G + g, t] * norm(b, h, t) * centroids[codes(b, h, t)]  (rotated space)."""
    _require_gpu(idx_bytes, "idx_bytes")
    idx_bytes, vec_norms, prs, rows, tokens = _packed_rows(idx_bytes, vec_norms)
    B, Hq, S = weights.shape
    Hkv = idx_bytes.shape[1]
    group = Hq // Hkv
    if weights.dtype != torch.float32 or S != tokens or (S > 1 and weights.stride(2) != 1) \
            or (Hq > 1 and B > 1 and weights.stride(0) != Hq * weights.stride(1)):
        weights = weights.to(torch.float32).contiguous()
    stride = weights.stride(1) if Hq > 1 else (weights.stride(0) if B > 1 else max(tokens, 1))
    out = torch.empty((B, Hq, head_dim), dtype=torch.float32, device=idx_bytes.device)
    L = lib()
    splits = L.tq_weighted_values_splits(rows, tokens)
    step = 8                                             # query heads per kv head and launch
    with _on(idx_bytes.device):
        if group <= step:
            partial = torch.empty((rows, splits, group, head_dim), dtype=torch.float32, device=idx_bytes.device)
            rc = L.tq_weighted_values(idx_bytes.data_ptr(), vec_norms.data_ptr(), prs, rows, tokens, table.data_ptr(),
                                      head_dim, bits, weights.data_ptr(), stride, group, partial.data_ptr(), splits,
                                      out.data_ptr(), _stream_handle(idx_bytes.device))
            check(rc, "tq_weighted_values")
        else:
            # wide groups: one launch per slice of 8 query heads, gathered through a [rows, g, D] buffer
            w4 = weights.reshape(B, Hkv, group, S) if weights.is_contiguous() else weights.contiguous().reshape(B, Hkv, group, S)
            o4 = out.view(B, Hkv, group, head_dim)
            for g0 in range(0, group, step):
                g1 = min(group, g0 + step)
                wpart = w4[:, :, g0:g1].contiguous()
                opart = torch.empty((rows, g1 - g0, head_dim), dtype=torch.float32, device=idx_bytes.device)
                partial = torch.empty((rows, splits, g1 - g0, head_dim), dtype=torch.float32, device=idx_bytes.device)
                rc = L.tq_weighted_values(idx_bytes.data_ptr(), vec_norms.data_ptr(), prs, rows, tokens, table.data_ptr(),
                                          head_dim, bits, wpart.data_ptr(), S, g1 - g0, partial.data_ptr(), splits,
                                          opart.data_ptr(), _stream_handle(idx_bytes.device))
                check(rc, "tq_weighted_values")
                o4[:, :, g0:g1].copy_(opart.view(B, Hkv, g1 - g0, head_dim))
    return out


weighted_values_op = torch.library.custom_op("tqamd::weighted_values", _weighted_values_impl,
                                             mutates_args=(), device_types="cuda")


@weighted_values_op.register_fake
def _(idx_bytes, vec_norms, table, bits, weights, head_dim):
    return weights.new_empty((weights.shape[0], weights.shape[1], head_dim), dtype=torch.float32)


def _attend_partials_impl(k_idx: torch.Tensor, k_norms: torch.Tensor, v_idx: torch.Tensor, v_norms: torch.Tensor,
                          table_k: torch.Tensor, table_v: torch.Tensor, bits_k: int, bits_v: int,
                          q_rot: torch.Tensor) -> torch.Tensor:
    """One pass over packed keys and values of a [B,H,S,..] store pair: per (batch, query head, split)
    [largest score, sum of exp, 128 weighted sums in the value codec's rotated space] -> [B, Hq, splits, 130]."""
    _require_gpu(k_idx, "k_idx")
    prs_k = packed_row_stride(k_idx, k_norms)
    prs_v = packed_row_stride(v_idx, v_norms)
    if prs_k is None or prs_v is None or prs_k != prs_v:
        k_idx, k_norms, v_idx, v_norms = k_idx.contiguous(), k_norms.contiguous(), v_idx.contiguous(), v_norms.contiguous()
        prs_k = 0
    B, H, S, _ = k_idx.shape
    Bq, Hq, D = q_rot.shape
    group = Hq // H
    q_rot = q_rot.to(torch.float32).contiguous()
    L = lib()
    splits = L.tq_attend_splits(B * H, S)
    part = torch.empty((B, H, splits, group, D + 2), dtype=torch.float32, device=k_idx.device)
    with _on(k_idx.device):
        rc = L.tq_attend_partials(k_idx.data_ptr(), k_norms.data_ptr(), v_idx.data_ptr(), v_norms.data_ptr(), prs_k,
                                  B * H, S, table_k.data_ptr(), table_v.data_ptr(), D, bits_k, bits_v,
                                  q_rot.data_ptr(), group, splits, part.data_ptr(), _stream_handle(k_idx.device))
    check(rc, "tq_attend_partials")
    return part.permute(0, 1, 3, 2, 4).reshape(B, Hq, splits, D + 2)


attend_partials_op = torch.library.custom_op("tqamd::attend_partials", _attend_partials_impl,
                                             mutates_args=(), device_types="cuda")


@attend_partials_op.register_fake
def _(k_idx, k_norms, v_idx, v_norms, table_k, table_v, bits_k, bits_v, q_rot):
    # the split count depends on shapes and on the device's compute-unit count only: ask the library, as the real op does
    B, H, S, _ = k_idx.shape
    splits = int(lib().tq_attend_splits(int(B) * int(H), int(S)))
    return q_rot.new_empty((q_rot.shape[0], q_rot.shape[1], max(splits, 1), q_rot.shape[2] + 2), dtype=torch.float32)


def _attend_packed_impl(queries: torch.Tensor, k_idx: torch.Tensor, k_norms: torch.Tensor, v_idx: torch.Tensor,
                        v_norms: torch.Tensor, table_k: torch.Tensor, table_v: torch.Tensor, bits_k: int, bits_v: int,
                        pi_k_t: torch.Tensor, pi_v: torch.Tensor, k_win: torch.Tensor, v_win: torch.Tensor,
                        scale: float) -> torch.Tensor:
    """Decode-step attention of queries [B,Hq,1,D] over a packed history ([B,H,S,..] store slices, S may be 0)
    plus uncompressed window tokens [B,H,n_w,D] (n_w may be 0, not both): three launches."""
    _require_gpu(queries, "queries")
    B, Hq, _, D = queries.shape
    H = k_idx.shape[1]
    S = k_idx.shape[2]
    n_w = k_win.shape[2]
    group = Hq // H
    rows = B * H
    dev = queries.device
    q = queries.contiguous()
    pi_k_t, pi_v = pi_k_t.contiguous(), pi_v.contiguous()       # copies only if the caller kept a strided view
    L = lib()
    stream = _stream_handle(dev)
    q_rot = torch.empty((B, Hq, D), dtype=torch.float32, device=dev)
    part_w = torch.empty((rows, group, D + 2), dtype=torch.float32, device=dev) if n_w else None
    win_stride = 0
    if n_w:
        lay_k, lay_v = row_layout(k_win), row_layout(v_win)
        if (lay_k is None or lay_v is None or lay_k != lay_v or lay_k[3] != D or k_win.dtype != v_win.dtype
                or lay_k[2] % 8 or k_win.data_ptr() % 16 or v_win.data_ptr() % 16):
            k_win, v_win = k_win.contiguous(), v_win.contiguous()
            lay_k = row_layout(k_win)
        win_stride = lay_k[2] if rows > 1 else n_w * D
    out = torch.empty((B, Hq, 1, D), dtype=queries.dtype, device=dev)
    with _on(dev):
        rc = L.tq_attend_prepare(q.data_ptr(), dtype_code(q.dtype), rows, group, scale, pi_k_t.data_ptr(),
                                 k_win.data_ptr() if n_w else None, v_win.data_ptr() if n_w else None,
                                 dtype_code(k_win.dtype) if n_w else 0, n_w, win_stride, q_rot.data_ptr(),
                                 part_w.data_ptr() if n_w else None, stream)
        check(rc, "tq_attend_prepare")
        splits = 0
        part = None
        if S:
            prs_k, prs_v = packed_row_stride(k_idx, k_norms), packed_row_stride(v_idx, v_norms)
            if prs_k is None or prs_v is None or prs_k != prs_v:
                k_idx, k_norms, v_idx, v_norms = k_idx.contiguous(), k_norms.contiguous(), v_idx.contiguous(), v_norms.contiguous()
                prs_k = 0
            splits = L.tq_attend_splits(rows, S)
            part = torch.empty((rows, splits, group, D + 2), dtype=torch.float32, device=dev)
            rc = L.tq_attend_partials(k_idx.data_ptr(), k_norms.data_ptr(), v_idx.data_ptr(), v_norms.data_ptr(), prs_k,
                                      rows, S, table_k.data_ptr(), table_v.data_ptr(), D, bits_k, bits_v,
                                      q_rot.data_ptr(), group, splits, part.data_ptr(), stream)
            check(rc, "tq_attend_partials")
        rc = L.tq_attend_merge(part.data_ptr() if S else None, splits, part_w.data_ptr() if n_w else None, pi_v.data_ptr(),
                               rows, group, out.data_ptr(), dtype_code(out.dtype), stream)
        check(rc, "tq_attend_merge")
    return out


attend_packed_op = torch.library.custom_op("tqamd::attend_packed", _attend_packed_impl,
                                           mutates_args=(), device_types="cuda")


@attend_packed_op.register_fake
def _(queries, k_idx, k_norms, v_idx, v_norms, table_k, table_v, bits_k, bits_v, pi_k_t, pi_v, k_win, v_win, scale):
    return torch.empty_like(queries)


# ------------------------------------------------------------------------------------
# batched jobs
# ------------------------------------------------------------------------------------
class JobList:
    """A fixed list of (tensor, packed buffers, table) jobs of one bit width and element type,
    uploaded once and launched as a single kernel per direction."""

    def __init__(self, jobs: Sequence[dict], device: torch.device):
        if not jobs:
            raise ValueError("empty job list")
        self.n = len(jobs)
        self.device = torch.device(device)
        self.host = (TqJob * self.n)()
        self._keep = []
        self.head_dim = int(jobs[0]["states"].shape[-1])
        for i, j in enumerate(jobs):
            t = j["states"]
            _require_gpu(t, "states")
            if t.shape[-1] != self.head_dim:
                raise TqError(f"the jobs of one list share a head dimension: {t.shape[-1]} after {self.head_dim}")
            prs = packed_row_stride(j["idx_bytes"], j["vec_norms"])
            lay = None if prs is None else (row_layout(t) if prs else vector_layout(t))
            if lay is None:
                raise TqError("batched jobs need tensors with a dense last dimension and at most two stride "
                              "levels, and packed buffers that are contiguous or slices of a per-row store")
            rows, tokens, row_stride, token_stride = lay
            check_table(j["table"], t.shape[-1], int(j["bits"]))
            self.host[i] = TqJob(t.data_ptr(), j["idx_bytes"].data_ptr(), j["vec_norms"].data_ptr(),
                                 j["table"].data_ptr(), rows, tokens, row_stride, token_stride,
                                 int(j["bits"]), dtype_code(t.dtype), prs)
            self._keep.append((t, j["idx_bytes"], j["vec_norms"], j["table"]))
        raw = np.frombuffer(bytes(self.host), dtype=np.uint8).copy()
        self.dev = torch.from_numpy(raw).to(self.device)
        # ticket counters of the launches, one record per job; zero now, and every launch leaves them zero.
        # Launches of one list read or write the same buffers, so they never overlap and can share the counters.
        self.workspace = torch.zeros(int(lib().tq_workspace_bytes(self.n)), dtype=torch.uint8, device=self.device)

    def compress(self) -> None:
        with _on(self.device):
            rc = lib().tq_compress_batched(ctypes.addressof(self.host), self.dev.data_ptr(), self.n, self.head_dim,
                                           self.workspace.data_ptr(), _stream_handle(self.device))
        if rc:
            self.workspace.zero_()      # counters of a launch that did not complete are not trusted
        check(rc, "tq_compress_batched")

    def decompress(self) -> None:
        with _on(self.device):
            rc = lib().tq_decompress_batched(ctypes.addressof(self.host), self.dev.data_ptr(), self.n, self.head_dim,
                                             self.workspace.data_ptr(), _stream_handle(self.device))
        if rc:
            self.workspace.zero_()      # counters of a launch that did not complete are not trusted
        check(rc, "tq_decompress_batched")


class QjlJobList:
    """A fixed list of V2 key jobs (one per layer) of one width and element type, uploaded once and compressed by a
    single tq_qjl_compress_batched call.  Every job: {"states" [.., 128] dense vectors, "idx_bytes", "vec_norms",
    "sign_bytes", "residual_norm" (dense outputs), "table" (codec table of the MSE stage), "qjl_table", "mse_bits"}."""

    def __init__(self, jobs: Sequence[dict], device: torch.device):
        if not jobs:
            raise ValueError("empty job list")
        self.n = len(jobs)
        self.device = torch.device(device)
        self.host = (TqQjlJob * self.n)()
        self._keep = []
        for i, j in enumerate(jobs):
            t = j["states"]
            _require_gpu(t, "states")
            if not t.is_contiguous() or t.data_ptr() % 16:
                raise TqError("batched V2 jobs need contiguous, 16-byte aligned inputs")
            for name in ("idx_bytes", "vec_norms", "sign_bytes", "residual_norm"):
                if not j[name].is_contiguous():
                    raise TqError(f"batched V2 jobs need dense outputs ({name})")
            D = t.shape[-1]
            check_table(j["table"], D, int(j["mse_bits"]))
            self.host[i] = TqQjlJob(t.data_ptr(), j["idx_bytes"].data_ptr(), j["vec_norms"].data_ptr(), j["sign_bytes"].data_ptr(),
                                    j["residual_norm"].data_ptr(), j["table"].data_ptr(), j["qjl_table"].data_ptr(),
                                    t.numel() // D, D, int(j["mse_bits"]), dtype_code(t.dtype))
            self._keep.append(tuple(j[k] for k in ("states", "idx_bytes", "vec_norms", "sign_bytes", "residual_norm", "table", "qjl_table")))
        self.head_dim = int(jobs[0]["states"].shape[-1])
        raw = np.frombuffer(bytes(self.host), dtype=np.uint8).copy()
        self.dev = torch.from_numpy(raw).to(self.device)

    def compress(self) -> None:
        with _on(self.device):
            rc = lib().tq_qjl_compress_batched(ctypes.addressof(self.host), self.dev.data_ptr(), self.n, self.head_dim,
                                               _stream_handle(self.device))
        check(rc, "tq_qjl_compress_batched")


# ------------------------------------------------------------------------------------
# eager fast path
# ------------------------------------------------------------------------------------
_IMPL = {
    "compress": _compress_impl,
    "compress_into": _compress_into_impl,
    "decompress": _decompress_impl,
    "decompress_into": _decompress_into_impl,
    "scores_into": _scores_into_impl,
    "weighted_values": _weighted_values_impl,
    "attend_partials": _attend_partials_impl,
    "attend_packed": _attend_packed_impl,
}


def call(name: str, *args):
    """tqamd::<name>(*args).  In eager mode the Python implementation is called directly (the operator
    dispatcher costs 20-30 us per call, more than the small launches of a decode step); while a compiler is
    tracing, the registered operator is used so that the call stays one node of the graph."""
    if torch.compiler.is_compiling():
        return getattr(torch.ops.tqamd, name)(*args)
    return _IMPL[name](*args)
