"""The C ABI bound by hand, the way a maintainer of the reference would bind it (ctypes, raw device pointers, no
helper of this package between the test and the library): table build, compress, decompress against the oracle."""
import ctypes
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


@pytest.fixture(scope="module")
def tq():
    if not torch.cuda.is_available():
        pytest.skip("needs a HIP device")
    pkg = importlib.import_module("turboquant-pytorch_amd")
    lib = ctypes.CDLL(pkg._native.LIB_PATH)
    lib.tq_table_bytes.restype = ctypes.c_longlong
    lib.tq_status_string.restype = ctypes.c_char_p
    return pkg, lib


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("bits,dtype", [(4, torch.bfloat16), (2, torch.float16), (8, torch.float32), (3, torch.bfloat16)])
def test_raw_binding_round_trip(tq, oracle, bits, dtype):
    pkg, lib = tq
    D, B, H, S = 128, 2, 3, 101
    pi = np.ascontiguousarray(pkg.generate_rotation_matrix(D, seed=1234 + bits).numpy(), np.float32)
    cent = np.ascontiguousarray(pkg.LloydMaxCodebook(D, bits).centroids.numpy(), np.float32)
    n = lib.tq_table_bytes(D, bits)
    blob = np.zeros(n, np.uint8)
    assert lib.tq_table_build(pi.ctypes.data_as(ctypes.c_void_p), cent.ctypes.data_as(ctypes.c_void_p), D, bits,
                              blob.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(n)) == 0
    table = torch.from_numpy(blob).to(DEV)
    g = torch.Generator().manual_seed(bits)
    x = (torch.randn(B, H, S, D, generator=g) * torch.exp(torch.randn(D, generator=g))).to(dtype).to(DEV)
    G = lib.tq_bytes_per_vector(D, bits)
    idx = torch.empty(B, H, S, G, dtype=torch.uint8, device=DEV)
    nrm = torch.empty(B, H, S, dtype=torch.float16, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ll = ctypes.c_longlong
    rc = lib.tq_compress(_p(x), DT[dtype], ll(1), ll(B * H * S), ll(0), ll(D), _p(table), D, bits, _p(idx), _p(nrm), ll(0), None, stream)
    assert rc == 0, lib.tq_status_string(rc)
    out = torch.empty(B, H, S, D, dtype=torch.float32, device=DEV)
    rc = lib.tq_decompress(_p(idx), _p(nrm), ll(0), ll(1), ll(B * H * S), _p(table), D, bits, _p(out), 0, ll(0), ll(D), None, stream)
    assert rc == 0, lib.tq_status_string(rc)
    # with a workspace (zero before, zero after) the same bytes come out
    lib.tq_workspace_bytes.restype = ctypes.c_longlong
    ws = torch.zeros(lib.tq_workspace_bytes(1), dtype=torch.uint8, device=DEV)
    out_ws = torch.empty_like(out)
    rc = lib.tq_decompress(_p(idx), _p(nrm), ll(0), ll(1), ll(B * H * S), _p(table), D, bits, _p(out_ws), 0, ll(0), ll(D), _p(ws), stream)
    assert rc == 0, lib.tq_status_string(rc)
    torch.cuda.synchronize()
    assert torch.equal(out, out_ws) and int(ws.sum()) == 0
    orc = oracle.COracle(pi, cent, bits, accum_double=True)
    ref = orc.compress(x.float().cpu().numpy().reshape(-1, D))
    got = idx.cpu().numpy().reshape(-1, G)
    rep = oracle.code_mismatch_report(got, ref["idx_bytes"], ref["rotated"], cent, bits, 1e-5)
    assert rep["outside_window"] == 0 and rep["differ"] <= max(8, 5e-4 * rep["coords"]), rep
    ulp = oracle.fp16_ulp_distance(nrm.cpu().view(torch.int16).numpy().view(np.uint16).reshape(-1), ref["vec_norms"].reshape(-1))
    assert ulp.max() <= 1
    rec = orc.decompress(got, nrm.cpu().view(torch.int16).numpy().view(np.uint16).reshape(-1))
    err = np.linalg.norm(out.cpu().numpy().reshape(-1, D) - rec) / np.linalg.norm(rec)
    assert err < 1e-3, err
    # the wrong call is refused before any launch: misaligned packed buffer, unknown element type
    assert lib.tq_compress(_p(x), DT[dtype], ll(1), ll(4), ll(0), ll(D), _p(table), D, bits,
                           ctypes.c_void_p(idx.data_ptr() + 1), _p(nrm), ll(0), None, stream) < 0
    assert lib.tq_compress(_p(x), 9, ll(1), ll(4), ll(0), ll(D), _p(table), D, bits, _p(idx), _p(nrm), ll(0), None, stream) < 0


class _Job(ctypes.Structure):   # struct tq_job of include/tqamd.h
    _fields_ = [("states", ctypes.c_void_p), ("idx_bytes", ctypes.c_void_p), ("vec_norms", ctypes.c_void_p),
                ("table_dev", ctypes.c_void_p), ("rows", ctypes.c_longlong), ("tokens", ctypes.c_longlong),
                ("row_stride", ctypes.c_longlong), ("token_stride", ctypes.c_longlong),
                ("bits", ctypes.c_int), ("dtype", ctypes.c_int), ("packed_row_stride", ctypes.c_longlong)]


@pytest.mark.parametrize("bits,dtype", [(4, torch.bfloat16), (2, torch.float16), (8, torch.bfloat16)])
def test_compress_tiles_drawn_from_counters_equal_the_fixed_assignment(tq, oracle, bits, dtype):
    """tq_compress / tq_compress_batched with a workspace (blocks draw runs of tiles from a counter) write the bytes
    they write without one, the counters are zero again after every launch, and the bytes are the oracle's: jobs large
    enough for the counters to be used, with a ragged end (a partial last tile inside a partial last run), next to a
    job too small for them and an empty one."""
    pkg, lib = tq
    D = 128
    ll = ctypes.c_longlong
    lib.tq_workspace_bytes.restype = ll
    G = lib.tq_bytes_per_vector(D, bits)
    pi = np.ascontiguousarray(pkg.generate_rotation_matrix(D, seed=4321 + bits).numpy(), np.float32)
    cent = np.ascontiguousarray(pkg.LloydMaxCodebook(D, bits).centroids.numpy(), np.float32)
    n = lib.tq_table_bytes(D, bits)
    blob = np.zeros(n, np.uint8)
    assert lib.tq_table_build(pi.ctypes.data_as(ctypes.c_void_p), cent.ctypes.data_as(ctypes.c_void_p), D, bits,
                              blob.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(n)) == 0
    table = torch.from_numpy(blob).to(DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    counts = [262144 + 8 * 32 * 5 + 3 * 32 + 17, 0, 1000, 300000]
    g = torch.Generator(device=DEV).manual_seed(bits)
    xs = [(torch.randn(c, D, generator=g, device=DEV) * torch.exp(torch.randn(D, generator=g, device=DEV))).to(dtype) for c in counts]

    def buffers():
        return ([torch.full((c, G), 0xA5, dtype=torch.uint8, device=DEV) for c in counts],
                [torch.full((c,), 7.0, dtype=torch.float16, device=DEV) for c in counts])

    def batched(ws):
        idx, nrm = buffers()
        host = (_Job * len(counts))(*[_Job(x.data_ptr(), i.data_ptr(), m.data_ptr(), table.data_ptr(), 1, c, 0, D, bits, DT[dtype], 0)
                                      for x, i, m, c in zip(xs, idx, nrm, counts)])
        dev = torch.from_numpy(np.frombuffer(bytes(host), dtype=np.uint8).copy()).to(DEV)
        rc = lib.tq_compress_batched(host, _p(dev), len(counts), D, _p(ws) if ws is not None else None, stream)
        assert rc == 0, lib.tq_status_string(rc)
        torch.cuda.synchronize()
        return idx, nrm

    ws = torch.zeros(lib.tq_workspace_bytes(len(counts)), dtype=torch.uint8, device=DEV)
    fixed_idx, fixed_nrm = batched(None)
    for trip in range(2):                       # the second launch finds the counters as the first left them
        drawn_idx, drawn_nrm = batched(ws)
        assert int(ws.sum()) == 0
        for a, b in zip(fixed_idx, drawn_idx):
            assert torch.equal(a, b)
        for a, b in zip(fixed_nrm, drawn_nrm):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # the single-job entry point, same vectors
    c = counts[0]
    idx1 = torch.empty((c, G), dtype=torch.uint8, device=DEV)
    nrm1 = torch.empty((c,), dtype=torch.float16, device=DEV)
    rc = lib.tq_compress(_p(xs[0]), DT[dtype], ll(1), ll(c), ll(0), ll(D), _p(table), D, bits, _p(idx1), _p(nrm1), ll(0), _p(ws), stream)
    assert rc == 0, lib.tq_status_string(rc)
    torch.cuda.synchronize()
    assert int(ws.sum()) == 0 and torch.equal(idx1, fixed_idx[0]) and torch.equal(nrm1.view(torch.int16), fixed_nrm[0].view(torch.int16))
    # and they are the oracle's bytes: the ragged end of the large job
    tail = 4096 + 17
    orc = oracle.COracle(pi, cent, bits, accum_double=True)
    ref = orc.compress(xs[0][-tail:].float().cpu().numpy())
    rep = oracle.code_mismatch_report(idx1[-tail:].cpu().numpy(), ref["idx_bytes"], ref["rotated"], cent, bits, 1e-5)
    assert rep["outside_window"] == 0 and rep["differ"] <= max(8, 5e-4 * rep["coords"]), rep
    ulp = oracle.fp16_ulp_distance(nrm1[-tail:].cpu().view(torch.int16).numpy().view(np.uint16), ref["vec_norms"].reshape(-1))
    assert ulp.max() <= 1
