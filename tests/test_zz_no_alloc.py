"""tq_decompress_batched_noalloc, the entry point that allocates nothing, called through the C ABI by hand (ctypes, raw
device pointers): its output must be the bytes that tq_decompress_batched writes for the same jobs, on two calls in a
row of which the second is smaller, and the library's counters must be usable again after each call."""
import ctypes
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128
ll = ctypes.c_longlong


class Job(ctypes.Structure):   # struct tq_job of include/tqamd.h
    _fields_ = [("states", ctypes.c_void_p), ("idx_bytes", ctypes.c_void_p), ("vec_norms", ctypes.c_void_p),
                ("table_dev", ctypes.c_void_p), ("rows", ll), ("tokens", ll), ("row_stride", ll), ("token_stride", ll),
                ("bits", ctypes.c_int), ("dtype", ctypes.c_int), ("packed_row_stride", ll)]


@pytest.fixture(scope="module")
def tq():
    if not torch.cuda.is_available():
        pytest.skip("needs a HIP device")
    pkg = importlib.import_module("turboquant-pytorch_amd")
    lib = ctypes.CDLL(pkg._native.LIB_PATH)
    lib.tq_table_bytes.restype = ll
    lib.tq_workspace_bytes.restype = ll
    lib.tq_status_string.restype = ctypes.c_char_p
    return pkg, lib


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _table(pkg, lib, bits, seed):
    pi = np.ascontiguousarray(pkg.generate_rotation_matrix(D, seed=seed).numpy(), np.float32)
    cent = np.ascontiguousarray(pkg.LloydMaxCodebook(D, bits).centroids.numpy(), np.float32)
    n = lib.tq_table_bytes(D, bits)
    blob = np.zeros(n, np.uint8)
    assert lib.tq_table_build(pi.ctypes.data_as(ctypes.c_void_p), cent.ctypes.data_as(ctypes.c_void_p), D, bits,
                              blob.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(n)) == 0
    return torch.from_numpy(blob).to(DEV), pi, cent


def _run_case(pkg, lib, oracle, bits, counts, seed):
    """Compress len(counts) jobs of counts[i] vectors, then decompress them with the workspace form and with the
    form that allocates nothing; returns after checking that both wrote the same bytes (and the oracle's values)."""
    G = lib.tq_bytes_per_vector(D, bits)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(seed)
    keep, jobs_c, jobs_a, jobs_b, outs_a, outs_b, packed = [], [], [], [], [], [], []
    for i, n in enumerate(counts):
        table, pi, cent = _table(pkg, lib, bits, seed=100 * seed + i)
        x = (torch.randn(n, D, generator=g) * torch.exp(0.5 * torch.randn(D, generator=g))).to(torch.bfloat16).to(DEV)
        idx = torch.empty(n, G, dtype=torch.uint8, device=DEV)
        nrm = torch.empty(n, dtype=torch.float16, device=DEV)
        out_a = torch.full((n, D), 7.0, dtype=torch.bfloat16, device=DEV)
        out_b = torch.full((n, D), -7.0, dtype=torch.bfloat16, device=DEV)
        keep += [table, x, idx, nrm]
        jobs_c.append(Job(x.data_ptr(), idx.data_ptr(), nrm.data_ptr(), table.data_ptr(), 1, n, 0, D, bits, 2, 0))
        jobs_a.append(Job(out_a.data_ptr(), idx.data_ptr(), nrm.data_ptr(), table.data_ptr(), 1, n, 0, D, bits, 2, 0))
        jobs_b.append(Job(out_b.data_ptr(), idx.data_ptr(), nrm.data_ptr(), table.data_ptr(), 1, n, 0, D, bits, 2, 0))
        outs_a.append(out_a)
        outs_b.append(out_b)
        packed.append((idx, nrm, pi, cent))

    def upload(jobs):
        host = (Job * len(jobs))(*jobs)
        dev = torch.from_numpy(np.frombuffer(bytes(host), dtype=np.uint8).copy()).to(DEV)
        return host, dev

    hc, dc = upload(jobs_c)
    ha, da = upload(jobs_a)
    hb, db = upload(jobs_b)
    nj = len(counts)
    rc = lib.tq_compress_batched(hc, _p(dc), nj, D, None, stream)
    assert rc == 0, lib.tq_status_string(rc)
    ws = torch.zeros(lib.tq_workspace_bytes(nj), dtype=torch.uint8, device=DEV)
    rc = lib.tq_decompress_batched(ha, _p(da), nj, D, _p(ws), stream)
    assert rc == 0, lib.tq_status_string(rc)
    torch.cuda.synchronize()
    # "allocates nothing" is a statement about the driver, not about torch's caching allocator (which a hipMalloc
    # inside the library would never touch): the device's free memory is read before and after the call
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.tq_decompress_batched_noalloc(hb, _p(db), nj, D, stream)
    assert rc == 0, lib.tq_status_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    for a, b in zip(outs_a, outs_b):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # and the bytes are the right ones: the first job against the oracle's decode of the same packed bytes
    idx, nrm, pi, cent = packed[0]
    m = min(counts[0], 4096)
    orc = oracle.COracle(pi, cent, bits, accum_double=True)
    rec = orc.decompress(idx[:m].cpu().numpy(), nrm[:m].cpu().view(torch.int16).numpy().view(np.uint16))
    got = outs_b[0][:m].float().cpu().numpy()
    err = np.linalg.norm(got - rec) / np.linalg.norm(rec)
    assert err < 4e-3, err      # bf16 output rounding (2^-9 per element) on top of the kernel's 1e-3
    del keep


def test_noalloc_equals_workspace_form_twice_second_smaller(tq, oracle):
    pkg, lib = tq
    # first call: three jobs large enough for the ticket counters to be used (>= 4 tickets per block)
    _run_case(pkg, lib, oracle, 4, [262144, 262144, 200000 + 17], seed=1)
    # second call, smaller: fewer jobs, fewer vectors, another width; reuses the counters the first call left
    _run_case(pkg, lib, oracle, 2, [131072 + 5, 131072], seed=2)
    # third: tiny jobs (fixed assignment of tiles inside the kernel), ragged sizes, an empty job in the list
    _run_case(pkg, lib, oracle, 8, [33, 0, 1000], seed=3)


def test_noalloc_call_can_be_captured_into_a_graph(tq):
    """Stream capture fails on any allocation or synchronising call: a call recorded into a HIP graph, after an eager
    call has looked up the library's counters, replays to the bytes of the workspace form, three times over with the
    program's own work and synchronisations in between."""
    pkg, lib = tq
    bits, n = 4, 131072 + 40
    G = lib.tq_bytes_per_vector(D, bits)
    table, pi, cent = _table(pkg, lib, bits, seed=77)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(n, D, generator=g).to(torch.bfloat16).to(DEV)
    idx = torch.empty(n, G, dtype=torch.uint8, device=DEV)
    nrm = torch.empty(n, dtype=torch.float16, device=DEV)
    ref = torch.empty(n, D, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(n, D, dtype=torch.bfloat16, device=DEV)
    mk = lambda t: (Job * 1)(Job(t.data_ptr(), idx.data_ptr(), nrm.data_ptr(), table.data_ptr(), 1, n, 0, D, bits, 2, 0))
    up = lambda h: torch.from_numpy(np.frombuffer(bytes(h), dtype=np.uint8).copy()).to(DEV)
    hc, hr, ho = mk(x), mk(ref), mk(out)
    dc, dr, do = up(hc), up(hr), up(ho)
    cur = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.tq_compress_batched(hc, _p(dc), 1, D, None, cur()) == 0
    ws = torch.zeros(lib.tq_workspace_bytes(1), dtype=torch.uint8, device=DEV)
    assert lib.tq_decompress_batched(hr, _p(dr), 1, D, _p(ws), cur()) == 0
    assert lib.tq_decompress_batched_noalloc(ho, _p(do), 1, D, cur()) == 0       # eager: looks the counters up
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):           # captures on a side stream, which is the current one inside the block
        rc = lib.tq_decompress_batched_noalloc(ho, _p(do), 1, D, cur())
    assert rc == 0, lib.tq_status_string(rc)
    for _ in range(3):
        out.fill_(3.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_noalloc_rejects_what_it_cannot_hold(tq):
    pkg, lib = tq
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = 513
    host = (Job * n)()
    dev = torch.zeros(ctypes.sizeof(host), dtype=torch.uint8, device=DEV)
    rc = lib.tq_decompress_batched_noalloc(host, _p(dev), n, D, stream)
    assert rc == -10 and b"capacity" in lib.tq_status_string(rc)
    assert lib.tq_decompress_batched_noalloc(None, _p(dev), 1, D, stream) == -1
    assert lib.tq_decompress_batched_noalloc(host, _p(dev), 0, D, stream) == 0
