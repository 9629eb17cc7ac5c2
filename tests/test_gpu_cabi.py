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
    rc = lib.tq_compress(_p(x), DT[dtype], ll(1), ll(B * H * S), ll(0), ll(D), _p(table), D, bits, _p(idx), _p(nrm), ll(0), stream)
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
                           ctypes.c_void_p(idx.data_ptr() + 1), _p(nrm), ll(0), stream) < 0
    assert lib.tq_compress(_p(x), 9, ll(1), ll(4), ll(0), ll(D), _p(table), D, bits, _p(idx), _p(nrm), ll(0), stream) < 0
