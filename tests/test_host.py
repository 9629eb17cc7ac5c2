"""Host logic of the package and the C ABI surface -- no GPU needed.

Codebook and rotation against tables written by the reference, the quantiser tables against
brute force, byte accounting and layer-bit selection against the reference's outputs, error
behaviour of the C entry points, and that the library exports what include/tqamd.h declares.
"""
import ctypes
import os
import re
import shutil
import subprocess

import numpy as np
import pytest
import torch

from conftest import ROOT


def test_library_exports_every_declared_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "tqamd.h")).read()
    declared = sorted(set(re.findall(r"\b(tq_[a-z_0-9]+)\s*\(", header)))
    assert len(declared) >= 12
    lib = pkg._native.lib()
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(pkg._native.EXPORTS) == declared
    assert lib.tq_abi_version() == 5
    assert lib.tq_status_string(0) == b"ok"
    assert b"bits" in lib.tq_status_string(-2)


def test_job_struct_layout_matches_header(pkg, tmp_path):
    # 4 pointers + 4 int64 + 2 int32 + 1 int64 = 80 bytes
    J = pkg._native.TqJob
    assert ctypes.sizeof(J) == 80
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler to read the header with")
    fields = [f[0] for f in J._fields_]
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "tqamd.h"\nint main(void) {\n'
                   '  printf("%zu", sizeof(tq_job));\n'
                   + "".join(f'  printf(" %zu", offsetof(tq_job, {f}));\n' for f in fields)
                   + '  printf(" %d\\n", TQ_ABI_VERSION);\n  return 0;\n}\n')
    exe = tmp_path / "layout"
    subprocess.run([gcc, "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert int(out[0]) == ctypes.sizeof(J)
    assert [int(x) for x in out[1:-1]] == [getattr(J, f).offset for f in fields]
    assert int(out[-1]) == pkg._native.lib().tq_abi_version()


def test_codebooks_match_reference_bits(pkg, golden):
    """Closed-form replay of the reference's 200-step Lloyd iteration == its quadrature result,
    float32 bit for bit, for every (d, bits) the fixtures hold."""
    cb = golden["codebooks"]
    n = 0
    for key in cb.files:
        m = re.fullmatch(r"centroids_d(\d+)_b(\d+)", key)
        if not m:
            continue
        d, b = int(m.group(1)), int(m.group(2))
        cent, bounds = pkg.solve_lloyd_max(d, b)
        assert np.array_equal(cent.numpy().view(np.uint32), cb[key].view(np.uint32)), key
        assert np.abs(bounds.numpy() - cb[f"boundaries_d{d}_b{b}"]).max() < 1e-12
        assert cent.dtype == torch.float32 and cent.numel() == 2 ** b
        n += 1
    assert n == 12


def test_codebook_textbook_values(pkg):
    """Where the iteration converges (bits <= 3) the table is Max's Gaussian quantiser times sigma."""
    s = 1 / np.sqrt(128)
    c1, _ = pkg.solve_lloyd_max(128, 1)
    assert np.allclose(c1.numpy() / s, [-0.7978846, 0.7978846], atol=1e-6)
    c2, _ = pkg.solve_lloyd_max(128, 2)
    assert np.allclose(c2.numpy() / s, [-1.5104, -0.4528, 0.4528, 1.5104], atol=1e-4)
    c3, _ = pkg.solve_lloyd_max(128, 3)
    assert np.allclose(c3.numpy()[[0, 3, 4, 7]] / s, [-2.1520, -0.2451, 0.2451, 2.1520], atol=1e-4)
    for b in range(1, 9):
        c, _ = pkg.solve_lloyd_max(128, b)
        assert abs(float(c.sum())) < 1e-5 and bool((c[1:] > c[:-1]).all())
    cb = pkg.LloydMaxCodebook(128, 3)   # the one assert of the reference's own test script
    assert cb.centroids.sum().abs().item() < 0.01 and cb.n_levels == 8


def test_rotation_matches_reference(pkg, golden):
    rots = golden["rotations"]
    threads = torch.get_num_threads()
    try:
        for key in rots.files:
            m = re.fullmatch(r"Pi_d(\d+)_s(\d+)", key)
            d, seed = int(m.group(1)), int(m.group(2))
            torch.set_num_threads(1)    # the fixtures were written single-threaded (LAPACK order)
            one = pkg.generate_rotation_matrix(d, seed=seed).numpy()
            torch.set_num_threads(threads)
            many = pkg.generate_rotation_matrix(d, seed=seed).numpy()
            # same recipe -> same matrix up to LAPACK rounding; bit-exact on the build container
            assert np.abs(one - rots[key]).max() < 1e-5
            assert np.abs(many - rots[key]).max() < 1e-5
            eye = one.astype(np.float64) @ one.astype(np.float64).T
            assert np.abs(eye - np.eye(d)).max() < 1e-5
    finally:
        torch.set_num_threads(threads)
    a = pkg.generate_rotation_matrix(128, seed=7)
    b = pkg.generate_rotation_matrix(128, seed=7)
    c = pkg.generate_rotation_matrix(128, seed=8)
    assert torch.equal(a, b) and not torch.equal(a, c)


@pytest.mark.parametrize("bits", range(1, 9))
def test_thresholds_and_grid_equal_argmin(pkg, golden, oracle, bits):
    """Both forms of the code search the kernels rely on -- counting thresholds, and the
    fused-multiply-add grid lookup -- equal the reference's argmin for every probed float,
    including the floats adjacent to every threshold."""
    cent = golden["codebooks"][f"centroids_d128_b{bits}"]
    Pi = golden["rotations"]["Pi_d128_s42"]
    thr = pkg._native.decision_thresholds(cent)
    assert thr.size == cent.size - 1 and np.all(np.diff(thr) > 0)
    mids = (cent[:-1].astype(np.float64) + cent[1:]) / 2
    assert np.abs(thr - mids).max() < 1e-7
    table = pkg._native.build_table(torch.from_numpy(Pi), torch.from_numpy(cent), bits)
    rng = np.random.default_rng(bits)
    probes = [rng.normal(0, 1 / np.sqrt(128), 200000).astype(np.float32),
              rng.uniform(-1.03, 1.03, 100000).astype(np.float32),
              np.array([0.0, -0.0, 1.0, -1.0, 1.03, -1.03], np.float32)]
    near = []
    for t in thr:
        lo = hi = np.float32(t)
        near.append(lo)
        for _ in range(4):
            lo = np.nextafter(lo, np.float32(-np.inf))
            hi = np.nextafter(hi, np.float32(np.inf))
            near += [lo, hi]
    probes.append(np.array(near, np.float32))
    # the first float of every grid cell and its predecessor
    hdr = table[:256].view(np.uint32)
    cells = int(hdr[7])
    scale = float(table[32:36].view(np.float32)[0])
    edges = ((np.arange(cells + 1) - cells // 2) / scale).astype(np.float32)
    edges = edges[np.abs(edges) <= 1.03]   # the grid covers |r| <= 1.05; unit coordinates stay below 1
    probes += [edges, np.nextafter(edges, np.float32(-np.inf)), np.nextafter(edges, np.float32(np.inf))]
    r = np.concatenate(probes)
    ref = np.empty(r.size, np.uint8)
    oracle._load().tqo_nearest(r, r.size, cent, cent.size, ref)
    counted = (r[:, None] >= thr[None, :]).sum(-1) if thr.size else np.zeros(r.size, np.int64)
    assert np.array_equal(counted.astype(np.uint8), ref)
    assert np.array_equal(pkg._native.quantize_host(table, r), ref)


@pytest.mark.parametrize("D,bits", [(8, 8), (8, 6), (12, 7), (16, 8), (10, 5)])
def test_codebooks_that_reach_beyond_the_unit_interval(pkg, oracle, D, bits):
    """Very small head dimensions at many bits: the outer levels of N(0, 1/d) codebooks lie beyond +-1, where no coordinate
    of a unit vector can fall.  The table builds (thresholds outside the grid's span are counted for every coordinate or
    for none) and the search agrees with the nearest-centroid definition on everything a coordinate can be."""
    cent = pkg.LloydMaxCodebook(D, bits).centroids.numpy()
    g = torch.Generator().manual_seed(D)
    Pi, _ = torch.linalg.qr(torch.randn(D, D, generator=g))
    table = pkg._native.build_table(Pi, torch.from_numpy(cent), bits)
    thr = pkg._native.decision_thresholds(cent)
    rng = np.random.default_rng(D * bits)
    near = []
    for t in thr[np.abs(thr) <= 1.0]:
        lo = hi = np.float32(t)
        near.append(lo)
        for _ in range(3):
            lo = np.nextafter(lo, np.float32(-np.inf))
            hi = np.nextafter(hi, np.float32(np.inf))
            near += [lo, hi]
    r = np.concatenate([rng.uniform(-1.0, 1.0, 200000).astype(np.float32), np.array(near + [1.0, -1.0, 0.0], np.float32)])
    r = r[np.abs(r) <= 1.0]
    ref = np.empty(r.size, np.uint8)
    oracle._load().tqo_nearest(r, r.size, cent, cent.size, ref)
    assert np.array_equal(pkg._native.quantize_host(table, r), ref)


def test_table_rotation_split_reconstructs_pi(pkg, golden):
    """The 16-bit operand tiles in the table sum back to Pi: fp16 hi+lo to ~2^-21 relative,
    bf16 three terms exactly, and the tiling puts element (out, k) where the kernels read it."""
    Pi = golden["rotations"]["Pi_d128_s42"]
    cent = golden["codebooks"]["centroids_d128_b4"]
    table = pkg._native.build_table(torch.from_numpy(Pi), torch.from_numpy(cent), 4)
    hdr = table[:256].view(np.uint32)
    off_a_f16, off_a_bf16, off_grid, off_at = (int(x) for x in hdr[11:15])
    op = 32768

    def tiles(raw16, transpose):
        a = raw16.reshape(4, 8, 64, 8)    # t, s, lane, i
        out = np.zeros((128, 128), raw16.dtype)
        for t in range(4):
            for s in range(8):
                for lane in range(64):
                    m, hk = lane % 32, lane // 32
                    h, r = (m // 4) % 2, 4 * (m // 8) + (m % 4)
                    o = 64 * h + 16 * t + r if transpose else 32 * t + 16 * h + r
                    for i in range(8):
                        if transpose:
                            out[64 * hk + 8 * s + i, o] = a[t, s, lane, i]
                        else:
                            out[o, 16 * s + 8 * hk + i] = a[t, s, lane, i]
        return out

    f16 = table[off_a_f16:off_a_f16 + 2 * op].view(np.float16).reshape(2, -1)
    hi, lo = tiles(f16[0], False).astype(np.float64), tiles(f16[1], False).astype(np.float64)
    assert np.abs((hi + lo) / 1024 - Pi).max() < 2.0 ** -21 * np.abs(Pi).max()
    bf = table[off_a_bf16:off_a_bf16 + 3 * op].view(np.uint16).reshape(3, -1)
    terms = [(tiles(bf[i], False).astype(np.uint32) << 16).view(np.float32).astype(np.float64) for i in range(3)]
    assert np.array_equal((terms[0] + terms[1] + terms[2]).astype(np.float32), Pi)
    assert np.abs(terms[0] + terms[1] - Pi).max() < 2.0 ** -16 * np.abs(Pi).max()
    at = table[off_at:off_at + 2 * op].view(np.float16).reshape(2, -1)
    assert np.abs(tiles(at[0], True).astype(np.float64) + tiles(at[1], True).astype(np.float64) - Pi).max() < 1e-6


def test_memory_bytes_match_reference(pkg, golden):
    j = golden["json"]
    for key, meta in j["mse_roundtrip"].items():
        bits = int(key.split("_")[0][1:])
        comp = pkg.MSECompressor(128, bits, seed=42 + bits, device="cpu")
        assert comp.memory_bytes(1, 2, 48) == meta["memory_bytes"]
        assert meta["idx_pad"] == 0 and meta["idx_bytes_shape"][-1] == -(-128 // (8 // bits))
    assert pkg.MSECompressor(128, 4, seed=42, device="cpu").memory_bytes(1, 8, 1024) == j["config1"]["memory_bytes"]
    for row in j["v3"]["memory_bytes_table"]:
        kb, vb, rw, pl, li, nl, B, H, S = row["args"]
        t = pkg.TurboQuantV3(128, key_bits=kb, value_bits=vb, residual_window=rw, layer_idx=li, n_layers=nl,
                             protected_layers=pl, device="cpu")
        assert t.memory_bytes(B, H, S) == row["memory_bytes"], row
    # README closed forms: K4/V2 = 100 B per 512 B pair; rw128 + protected-4 at 8K over 36 layers = 3.62x
    total = sum(pkg.TurboQuantV3(128, 4, 2, 128, li, 36, 4, device="cpu").memory_bytes(1, 2, 8192)["compressed_bytes"]
                for li in range(36))
    assert total == 2 * 41711616 and abs(36 * 8388608 / total - 3.62) < 0.005     # README: 3.6x
    assert pkg.TurboQuantV3(128, 4, 2, 0, 10, 36, 4, device="cpu").memory_bytes(1, 1, 1)["compressed_bytes"] == 100


def test_layer_bit_selection_matches_reference(pkg, golden):
    v3 = golden["json"]["v3"]
    for row in v3["bit_selection_cheap"]:
        kb, vb, pl, nl, pb, li = row["args"]
        t = pkg.TurboQuantV3(128, key_bits=kb, value_bits=vb, layer_idx=li, n_layers=nl, protected_layers=pl,
                             protected_bits=pb, device="cpu")
        assert (t.key_bits, t.value_bits) == (row["key_bits"], row["value_bits"]), row
    for row in v3["protected_default"]:
        t = pkg.TurboQuantV3(128, key_bits=4, value_bits=2, layer_idx=row["layer_idx"], n_layers=36,
                             protected_layers=4, device="cpu")
        assert (t.key_bits, t.value_bits) == (row["key_bits"], row["value_bits"])
        assert t.memory_bytes(1, 2, 8192) == row["memory_bytes_1_2_8192"]
    # protected_bits above 8 is capped at 8; seeds follow seed + 1000*layer (+500 for values)
    t = pkg.TurboQuantV3(128, 4, 2, layer_idx=0, n_layers=8, protected_layers=1, protected_bits=16, device="cpu")
    assert (t.key_bits, t.value_bits) == (8, 8)
    t = pkg.TurboQuantV3(128, 4, 2, layer_idx=5, n_layers=36, protected_layers=4, device="cpu")
    assert torch.equal(t.key_compressor.Pi, pkg.generate_rotation_matrix(128, seed=5042))
    assert torch.equal(t.val_compressor.Pi, pkg.generate_rotation_matrix(128, seed=5542))


def test_passthrough_and_errors_without_gpu(pkg):
    t = pkg.TurboQuantV3(128, 4, 2, residual_window=16, layer_idx=5, n_layers=36, device="cpu")
    k = torch.randn(1, 2, 16, 128)
    v = torch.randn(1, 2, 16, 128)
    ck, cv = t.compress_kv(k, v)               # S <= window: nothing is compressed, same objects back
    assert ck["compressed"] is None and ck["fp16"] is k and cv["fp16"] is v and ck["split_at"] == 16
    rk, rv = t.decompress_kv(ck, cv)
    assert rk is k and rv is v
    with pytest.raises(RuntimeError):          # no CPU fallback
        t.compress_kv(torch.randn(1, 2, 17, 128), torch.randn(1, 2, 17, 128))
    with pytest.raises(ValueError):            # non-4-D input, like the reference's tuple unpack
        t.key_compressor.compress(torch.randn(4, 128))
    wide = pkg.MSECompressor(128, 9, seed=1, device="cpu")   # constructs, like the reference ...
    with pytest.raises(ZeroDivisionError):                     # ... and fails at 8 // bits in compress
        wide.compress(torch.randn(1, 1, 4, 128))


def test_table_and_width_must_agree(pkg):
    """A table blob is checked against the (head_dim, bits) it is used with before anything is launched: by
    tq_table_check on the host copy, and by the registry of uploaded tables at every launch of this package."""
    native = pkg._native
    lib = native.lib()
    pi = pkg.generate_rotation_matrix(128, seed=3)
    blob = native.build_table(pi, pkg.LloydMaxCodebook(128, 4).centroids, 4)
    assert lib.tq_table_check(blob.ctypes.data, blob.size, 128, 4) == 0
    assert lib.tq_table_check(blob.ctypes.data, blob.size, 128, 2) == -7          # built for another width
    assert lib.tq_table_check(blob.ctypes.data, blob.size, 64, 4) == -7
    assert lib.tq_table_check(blob.ctypes.data, blob.size - 1, 128, 4) == -7      # truncated
    assert lib.tq_table_check(blob.ctypes.data, blob.size, 128, 9) == -2
    broken = blob.copy()
    broken[0] ^= 0xFF
    assert lib.tq_table_check(broken.ctypes.data, broken.size, 128, 4) == -7
    assert lib.tq_table_check(None, 0, 128, 4) == -1
    # the launch-side check: a tensor tagged as a 4-bit table cannot be launched as a 2-bit one
    fake = torch.zeros(16, dtype=torch.uint8)
    setattr(fake, native._TABLE_TAG, (128, 4))
    native.check_table(fake, 128, 4)
    with pytest.raises(native.TqError, match="4 bits used with head_dim 128, 2 bits"):
        native.check_table(fake, 128, 2)
    native.check_table(torch.zeros(16, dtype=torch.uint8), 128, 2)             # unknown tables pass


def test_table_tag_does_not_outlive_its_tensor(pkg):
    """The width a table was uploaded for is a property of the tensor object, not of its address: when a table is
    freed and a caller's own, untagged upload lands on the same storage, no stale width is found for it."""
    native = pkg._native
    storage = torch.zeros(64, dtype=torch.uint8)
    tagged = storage[:16]
    setattr(tagged, native._TABLE_TAG, (128, 4))
    address = tagged.data_ptr()
    with pytest.raises(native.TqError):
        native.check_table(tagged, 128, 2)
    del tagged
    reused = storage[:16]                       # same address, another tensor object: a caller's own table
    assert reused.data_ptr() == address
    native.check_table(reused, 128, 2)          # passes: nothing is known about it
    native.check_table(reused, 64, 8)


def test_workspace_is_dropped_after_a_failed_call(pkg):
    """The ticket counters kept per (device, stream) are only trusted while every call on them succeeded."""
    native = pkg._native
    dev = torch.device("cuda:0")
    native._workspaces[(0, 12345)] = torch.zeros(1)
    native._workspaces[(0, 777)] = torch.zeros(1)
    native._drop_workspace(dev, 12345)
    assert (0, 12345) not in native._workspaces and (0, 777) in native._workspaces
    native._drop_workspace(dev, 12345)                                             # nothing to drop: fine
    del native._workspaces[(0, 777)]


def test_c_abi_argument_errors(pkg):
    lib = pkg._native.lib()
    E = {k: v for k, v in (("NULL", -1), ("BITS", -2), ("HEAD_DIM", -3), ("DTYPE", -4), ("SIZE", -5),
                           ("CODEBOOK", -6), ("TABLE", -7), ("ALIGN", -8))}
    assert lib.tq_bytes_per_vector(128, 4) == 64 and lib.tq_bytes_per_vector(128, 3) == 64
    assert lib.tq_bytes_per_vector(128, 6) == 128 and lib.tq_bytes_per_vector(128, 1) == 16
    assert lib.tq_bytes_per_vector(6, 2) == 2
    assert lib.tq_bytes_per_vector(128, 0) == E["BITS"] and lib.tq_bytes_per_vector(128, 9) == E["BITS"]
    # compress / decompress take every head dimension from 8 to 256; one that is not a multiple of 32 has the table of the next multiple
    assert lib.tq_table_bytes(7, 4) == E["HEAD_DIM"] and lib.tq_table_bytes(257, 4) == E["HEAD_DIM"] and lib.tq_table_bytes(288, 4) == E["HEAD_DIM"]
    assert lib.tq_table_bytes(0, 4) == E["HEAD_DIM"] and lib.tq_table_bytes(128, 9) == E["BITS"]
    assert lib.tq_table_bytes(80, 4) == lib.tq_table_bytes(96, 4) == lib.tq_table_bytes(65, 4) and lib.tq_table_bytes(8, 2) == lib.tq_table_bytes(32, 2)
    assert 0 < lib.tq_table_bytes(32, 4) < lib.tq_table_bytes(128, 4) < lib.tq_table_bytes(256, 4)
    assert lib.tq_table_bytes(64, 4) > lib.tq_table_bytes(96, 4)      # 64: also the operands of diag(Pi, Pi) for the 128-wide kernels
    cent = np.array([0.1, -0.1], np.float32)
    thr = np.zeros(1, np.float32)
    assert lib.tq_decision_thresholds(cent.ctypes.data, 2, thr.ctypes.data) == E["CODEBOOK"]
    assert lib.tq_decision_thresholds(None, 2, thr.ctypes.data) == E["NULL"]
    pi = np.eye(128, dtype=np.float32)
    good = np.array([-0.1, 0.1], np.float32)
    blob = np.zeros(lib.tq_table_bytes(128, 1), np.uint8)
    assert lib.tq_table_build(pi.ctypes.data, good.ctypes.data, 128, 1, blob.ctypes.data, 16) == E["SIZE"]
    assert lib.tq_table_build(pi.ctypes.data, cent.ctypes.data, 128, 1, blob.ctypes.data, blob.size) == E["CODEBOOK"]
    assert lib.tq_table_build(pi.ctypes.data, good.ctypes.data, 128, 1, blob.ctypes.data, blob.size) == 0
    bad = np.zeros(256, np.uint8)
    out = np.zeros(1, np.uint8)
    assert lib.tq_table_quantize_host(bad.ctypes.data, thr.ctypes.data, 1, out.ctypes.data) == E["TABLE"]
    # launch entry points validate before touching the device
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data + (-buf.ctypes.data) % 16
    args = dict(rows=1, tokens=4, rs=0, ts=128)
    call = lambda states, dtype, bits, hd, idx=p, norms=p, table=p, **kw: lib.tq_compress(
        states, dtype, kw.get("rows", 1), kw.get("tokens", 4), kw.get("rs", 0), kw.get("ts", 128), table, hd, bits,
        idx, norms, kw.get("prs", 0), kw.get("ws", None), None)
    assert call(p, 1, 0, 128) == E["BITS"]
    assert call(p, 1, 4, 300) == E["HEAD_DIM"] and call(p, 1, 4, 4) == E["HEAD_DIM"]
    assert call(p, 1, 4, 80, ts=64) == E["SIZE"]
    assert call(p + 1, 1, 4, 80, ts=80) == E["ALIGN"]      # fp16 vectors of 80 elements may start on any even address, not on an odd one
    assert call(p, 1, 4, 64, ts=48) == E["SIZE"]
    assert call(p, 7, 4, 128) == E["DTYPE"]
    assert call(None, 1, 4, 128) == E["NULL"]
    assert call(p + 2, 1, 4, 128) == E["ALIGN"]
    assert call(p, 1, 4, 128, ts=100) == E["SIZE"]
    assert call(p, 1, 4, 128, tokens=-1) == E["SIZE"]
    assert call(p, 1, 4, 128, ts=132) == E["ALIGN"]
    assert call(None, 1, 4, 128, tokens=0) == 0          # empty input: nothing to do, not an error
    assert call(p, 1, 4, 128, rows=2, rs=1024, prs=3) == E["SIZE"]   # packed rows shorter than the token count
    assert call(p, 1, 4, 128, rows=2, rs=1024, prs=1 << 31) == E["SIZE"]
    assert lib.tq_decompress(p, p, 0, 1, 4, p, 128, 9, p, 0, 0, 128, None, None) == E["BITS"]
    assert lib.tq_decompress(p, p, 0, 1, 4, p, 128, 4, None, 0, 0, 128, None, None) == E["NULL"]
    assert lib.tq_decompress(p, p, 0, 1, 0, p, 128, 4, None, 0, 0, 128, None, None) == 0
    assert lib.tq_decompress(p, p, 2, 2, 4, p, 128, 4, p, 1, 1024, 128, None, None) == E["SIZE"]
    p64 = buf.ctypes.data + (-buf.ctypes.data) % 64
    assert lib.tq_decompress(p, p, 0, 1, 4, p, 128, 4, p, 0, 0, 128, p64 + 16, None) == E["ALIGN"]   # workspace: 64-byte aligned
    assert lib.tq_decompress(p, p, 0, 1, 0, p, 128, 4, None, 0, 0, 128, p64, None) == 0
    assert lib.tq_workspace_bytes(0) == 256 and lib.tq_workspace_bytes(1) == 256 and lib.tq_workspace_bytes(24) == 24 * 256
    assert lib.tq_workspace_bytes(-1) == E["SIZE"] and lib.tq_workspace_bytes(4097) == E["SIZE"]
    assert lib.tq_decompress_batched(None, None, 0, 128, None, None) == 0
    assert lib.tq_decompress_batched(None, None, 3, 128, None, None) == E["NULL"]
    assert lib.tq_decompress_batched(p, p, 3, 128, p64 + 32, None) == E["ALIGN"]
    assert call(p, 1, 4, 128, ws=p64 + 16) == E["ALIGN"]              # workspace: 64-byte aligned
    assert lib.tq_compress_batched(None, None, 0, 128, None, None) == 0
    assert lib.tq_compress_batched(None, None, 3, 128, None, None) == E["NULL"]
    assert lib.tq_compress_batched(p, p, 3, 128, p64 + 32, None) == E["ALIGN"]
    # the decode-step ends: (queries, q_dtype, rows, group, scale, pi_k_t, k_win, v_win, win_dtype, n_win, win_stride, q_rot, part_w)
    prep = lambda q=p, g=4, pit=p, kw=p, vw=p, wd=2, nw=8, ws=1024, qr=p, pw=p, rows=1, qd=2: lib.tq_attend_prepare(
        q, qd, rows, g, 0.5, pit, kw, vw, wd, nw, ws, qr, pw, None)
    assert prep(g=0) == E["SIZE"] and prep(g=17) == E["SIZE"] and prep(nw=513) == E["SIZE"] and prep(nw=-1) == E["SIZE"]
    assert prep(qd=5) == E["DTYPE"] and prep(wd=3) == E["DTYPE"]
    assert prep(rows=0) == 0
    assert prep(q=None) == E["NULL"] and prep(pit=None) == E["NULL"] and prep(qr=None) == E["NULL"]
    assert prep(kw=None) == E["NULL"] and prep(pw=None) == E["NULL"]
    assert prep(ws=512) == E["SIZE"]                       # rows of the window overlap
    assert prep(kw=p + 2) == E["ALIGN"] and prep(ws=1028) == E["ALIGN"]
    # the per-step calls: (k_new, v_new, dtype, strides, windows, win_stride, evict, put, tables, head_dim, bits, stores, prs, slot, rows)
    app = lambda kn=p, vn=p, dt=2, ks=128, vs=128, kw=p, vw=p, ws=4096, ev=0, put=16, tk=p, tv=p, hd=128, bk=4, bv=2, ki=p, kr=p, vi=p, vr=p, prs=64, slot=3, rows=2: \
        lib.tq_append_token(kn, vn, dt, ks, vs, kw, vw, ws, ev, put, tk, tv, hd, bk, bv, ki, kr, vi, vr, prs, slot, rows, None)
    assert app(dt=7) == E["DTYPE"] and app(hd=64) == E["HEAD_DIM"] and app(put=-1) == E["SIZE"] and app(ev=16) == E["SIZE"]
    assert app(put=32) == E["SIZE"] and app(slot=64) == E["SIZE"] and app(ks=64) == E["SIZE"] and app(rows=0) == 0
    assert app(kn=None) == E["NULL"] and app(ki=None) == E["NULL"] and app(bk=9) == E["BITS"]
    assert app(kw=p + 4) == E["ALIGN"] and app(ws=4100) == E["ALIGN"] and app(vs=132) == E["ALIGN"]
    att = lambda q=p, tokens=8, nw=4, splits=1, part=p, out=p, od=2, piv=p: lib.tq_attend_step(
        q, 2, 1, 4, 0.5, p, piv, p, p, 2, nw, 1024, p, p, p, p, 0, tokens, p, p, 128, 4, 2, p, p, part, splits, out, od, None)
    assert att(tokens=0, nw=0) == E["SIZE"] and att(tokens=-1) == E["SIZE"] and att(od=5) == E["DTYPE"]
    assert att(out=None) == E["NULL"] and att(piv=None) == E["NULL"] and att(splits=0) == E["SIZE"] and att(part=None) == E["NULL"]
    assert att(q=None) == E["NULL"]
    merge = lambda part=p, s=1, pw=p, piv=p, rows=1, g=4, out=p, od=2: lib.tq_attend_merge(part, s, pw, piv, rows, g, out, od, None)
    assert merge(g=17) == E["SIZE"] and merge(s=-1) == E["SIZE"] and merge(od=4) == E["DTYPE"] and merge(rows=0) == 0
    assert merge(piv=None) == E["NULL"] and merge(out=None) == E["NULL"] and merge(part=None) == E["NULL"]
    assert merge(part=None, s=0, pw=None) == E["NULL"]      # nothing to merge at all


def test_vector_layout_reduction(pkg):
    vl = pkg._native.vector_layout
    x = torch.zeros(2, 3, 40, 128, dtype=torch.float16)
    assert vl(x) == (1, 240, 0, 128)
    assert vl(x[:, :, :24]) == (6, 24, 40 * 128, 128)
    assert vl(x[:, :, 24:]) == (6, 16, 40 * 128, 128)
    assert vl(x[:1, :, :24]) == (3, 24, 40 * 128, 128)
    hf = torch.zeros(1, 40, 3, 128, dtype=torch.float16).transpose(1, 2)      # [B,S,H,D] storage, B = 1
    assert vl(hf) == (3, 40, 128, 384)
    assert vl(torch.zeros(2, 40, 3, 128).transpose(1, 2)) is None            # three stride levels
    assert vl(torch.zeros(1, 1, 0, 128)) == (0, 0, 0, 128)
    assert vl(torch.zeros(2, 3, 40, 130, dtype=torch.float16)[..., :128]) is None   # rows not 16-byte aligned


def test_row_layout_and_packed_row_stride(pkg):
    nat = pkg._native
    store = torch.zeros(2, 3, 64, 32, dtype=torch.uint8)
    norms = torch.zeros(2, 3, 64, dtype=torch.float16)
    assert nat.packed_row_stride(store, norms) == 0
    assert nat.packed_row_stride(store[:, :, 8:24], norms[:, :, 8:24]) == 64
    assert nat.packed_row_stride(store[:, :, :64], norms[:, :, :64]) == 0
    assert nat.packed_row_stride(store[:, :, 8:24], norms[:, :, 8:25]) is None       # shapes differ
    assert nat.packed_row_stride(store[:, :, ::2], norms[:, :, ::2]) is None         # not a slice
    assert nat.packed_row_stride(store[:, :, 8:24], torch.zeros(2, 3, 32, dtype=torch.float16)[:, :, 8:24]) is None
    x = torch.zeros(2, 3, 40, 128, dtype=torch.float16)
    assert nat.row_layout(x) == (6, 40, 40 * 128, 128)
    assert nat.row_layout(x[:, :, 5:6]) == (6, 1, 40 * 128, 128)
    assert nat.row_layout(x[:1, :1]) == (1, 40, 0, 128)
    assert nat.row_layout(torch.zeros(2, 40, 3, 128).transpose(1, 2)) is None        # batch and head do not merge
    assert nat.row_layout(torch.zeros(1, 40, 3, 128, dtype=torch.float16).transpose(1, 2)) == (3, 40, 128, 384)


def test_compute_metrics_definition(pkg):
    """The batched metric equals the per-head loop it replaces, on batch element 0 only."""
    g = torch.Generator().manual_seed(3)
    real = torch.randn(2, 6, 50, generator=g)
    tq = real + 0.3 * torch.randn(2, 6, 50, generator=g)
    tq[0, 2] = -real[0, 2]                                  # one head that disagrees completely
    m = pkg.compute_metrics(real, tq, 6)
    cos, t1, t5 = [], 0, 0
    for h in range(6):
        rs, ts = real[0, h], tq[0, h]
        cos.append(torch.nn.functional.cosine_similarity(rs.unsqueeze(0), ts.unsqueeze(0)).item())
        t1 += int(rs.argmax().item() == ts.argmax().item())
        t5 += int(rs.argmax().item() in ts.topk(5).indices.tolist())
    assert abs(m["cosine_sim"] - sum(cos) / 6) < 1e-6
    assert (m["top1_matches"], m["top5_matches"], m["n_checks"]) == (t1, t5, 6)
    assert m["top1_pct"] == 100 * t1 / 6 and m["top5_pct"] == 100 * t5 / 6 and t1 < 6
    same = pkg.compute_metrics(real, real.clone(), 6)
    assert abs(same["cosine_sim"] - 1) < 1e-6 and same["top1_pct"] == 100 and same["top5_pct"] == 100
    q = torch.randn(1, 2, 1, 8, generator=g)
    k = torch.randn(1, 2, 5, 8, generator=g)
    assert torch.allclose(pkg.attention_scores(q, k), torch.einsum("bhqd,bhsd->bhs", q, k), atol=1e-6)


def test_v3cache_refuses_cpu_tensors_and_reports_state(pkg):
    cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=4, n_layers=2)
    assert cache.get_seq_length() == 0 and cache.get_compression_info() == "no compression"
    with pytest.raises(Exception):                          # no CPU path: the codec tables live on HIP devices
        cache.update(torch.zeros(1, 1, 8, 128), torch.zeros(1, 1, 8, 128), 0)
    with pytest.raises(ValueError, match="nothing is cached"):
        pkg.V3Cache(key_bits=4, value_bits=2).attend(torch.zeros(1, 4, 1, 128), 0)


def test_tables_for_other_head_dimensions(pkg):
    """Tables for head dimensions other than 128: section sizes follow d (d/32 row tiles x d/16 steps of 1 KiB per
    operand term), the operands hold Pi in the compress tiling for both directions, and the quantiser grid may use
    all of its LDS budget (no shifted copies), which is what makes the dense 8-bit codebook of d = 256 fit."""
    native = pkg._native
    import ctypes

    class Header(ctypes.Structure):
        _fields_ = [(n, ctypes.c_uint32) for n in ("magic", "version", "head_dim", "bits", "levels", "ipb", "bytes_per_vec", "grid_cells")] + \
                   [("grid_scale", ctypes.c_float), ("grid_bias", ctypes.c_float)] + \
                   [(n, ctypes.c_uint32) for n in ("total_bytes", "off_a_f16", "off_a_bf16", "off_grid", "off_at_f16", "off_lut")]

    for D, bits in ((64, 4), (256, 8), (96, 3), (80, 4), (45, 2)):
        g = torch.Generator().manual_seed(D)
        Pi, _ = torch.linalg.qr(torch.randn(D, D, generator=g))
        cent = pkg.LloydMaxCodebook(D, bits).centroids
        blob = native.build_table(Pi, cent, bits)
        hd = Header.from_buffer_copy(blob[:ctypes.sizeof(Header)].tobytes())
        logical, D = D, -(-D // 32) * 32          # the operand sets are those of the rotation extended by zeros to a multiple of 32
        operand = (D // 32) * (D // 16) * 1024
        if logical != D:
            assert (hd.head_dim, hd.bits, hd.total_bytes) == (logical, bits, blob.size) and hd.bytes_per_vec == -(-logical // (8 // bits))
            a = blob[hd.off_a_bf16:hd.off_a_bf16 + operand].view(np.uint16).reshape(D // 32, D // 16, 64, 8)
            pi = np.zeros((D, D), np.float32)
            pi[:logical, :logical] = Pi.numpy()
            for (t, s, l, i) in ((0, 0, 0, 0), (D // 32 - 1, D // 16 - 1, 63, 7), (1, 2, 37, 3), (D // 32 - 1, 0, 5, 1), (0, D // 16 - 1, 33, 6)):
                m, hk = l % 32, l // 32
                row = 32 * t + 16 * ((m // 4) % 2) + 4 * (m // 8) + m % 4
                want = torch.tensor(pi[row, 16 * s + 8 * hk + i]).to(torch.bfloat16).view(torch.int16).item() & 0xffff
                assert a[t, s, l, i] == want, (logical, t, s, l, i)
            at = blob[hd.off_at_f16:hd.off_at_f16 + operand].view(np.float16).reshape(D // 32, D // 16, 64, 8)
            for (t, s, l, i) in ((1, 1, 40, 5), (D // 32 - 1, D // 16 - 1, 63, 7)):
                m, hk = l % 32, l // 32
                col = 32 * t + 16 * ((m // 4) % 2) + 4 * (m // 8) + m % 4
                assert at[t, s, l, i] == np.float16(pi[16 * s + 8 * hk + i, col])
            assert native.lib().tq_table_check(blob.ctypes.data, blob.size, logical, bits) == 0
            assert native.lib().tq_table_check(blob.ctypes.data, blob.size, D, bits) != 0
            continue
        assert (hd.head_dim, hd.bits, hd.total_bytes) == (D, bits, blob.size)
        assert hd.off_a_bf16 - hd.off_a_f16 == 2 * operand and hd.off_at_f16 - hd.off_a_bf16 == 3 * operand
        assert hd.bytes_per_vec == D // (8 // bits) and hd.grid_cells * 8 <= 18432
        # element (tile t, step s, lane l, i) of the leading bf16 term: Pi[32t + 16h + 4a + b][16s + 8hk + i], MFMA row m = 8a + 4h + b
        a = blob[hd.off_a_bf16:hd.off_a_bf16 + operand].view(np.uint16).reshape(D // 32, D // 16, 64, 8)
        pi = Pi.numpy()
        for (t, s, l, i) in ((0, 0, 0, 0), (D // 32 - 1, D // 16 - 1, 63, 7), (1, 2, 37, 3)):
            m, hk = l % 32, l // 32
            row = 32 * t + 16 * ((m // 4) % 2) + 4 * (m // 8) + m % 4
            want = torch.tensor(pi[row, 16 * s + 8 * hk + i]).to(torch.bfloat16).view(torch.int16).item() & 0xffff
            assert a[t, s, l, i] == want, (D, t, s, l, i)
        # decompress operand: Pi^T in the same tiling (out = column of Pi), leading fp16 term
        at = blob[hd.off_at_f16:hd.off_at_f16 + operand].view(np.float16).reshape(D // 32, D // 16, 64, 8)
        t, s, l, i = 1, 1, 40, 5
        m, hk = l % 32, l // 32
        col = 32 * t + 16 * ((m // 4) % 2) + 4 * (m // 8) + m % 4
        assert at[t, s, l, i] == np.float16(pi[16 * s + 8 * hk + i, col])
        assert native.lib().tq_table_check(blob.ctypes.data, blob.size, D, bits) == 0
        assert native.lib().tq_table_check(blob.ctypes.data, blob.size, 128, bits) != 0


def test_device_default_is_the_references(pkg):
    """compressors_v3.py:37,151 and compressors.py default to device="cpu": so do these classes; Pi and centroids then
    live on the CPU, and asking for a codec table there (there is no CPU codec) raises."""
    import inspect
    for cls in (pkg.MSECompressor, pkg.TurboQuantV3, pkg.TurboQuantCompressorV2, pkg.TurboQuantCompressorMSE):
        assert inspect.signature(cls.__init__).parameters["device"].default == "cpu", cls
    comp = pkg.MSECompressor(128, 4, seed=1)
    assert comp.Pi.device.type == "cpu" and comp.centroids.device.type == "cpu"
    with pytest.raises(pkg._native.TqError, match="HIP devices only"):
        comp.table()
    tq = pkg.TurboQuantV3(128)
    assert tq.key_compressor.Pi.device.type == "cpu"


def test_host_side_of_the_abi_under_sanitizers(tmp_path):
    """csrc/tq_host.cpp (table builders, thresholds, host quantiser) compiled with AddressSanitizer and
    UndefinedBehaviorSanitizer and driven by tests/native/host_sanitize.cpp over head dimensions 8 ... 256 (multiples of 32 and others) and every
    width, with table buffers of exactly the size tq_table_bytes reports; the driver also checks the host quantiser
    against the nearest-centroid definition."""
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    if gxx is None or not os.path.exists(os.path.join(rocm, "lib", "libamdhip64.so")):
        pytest.skip("needs g++ and the HIP runtime library to link tq_status_string")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = str(tmp_path / "host_sanitize")
    cmd = [gxx, "-O1", "-g", "-std=c++17", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-static-libasan", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include"),
           os.path.join(root, "tests", "native", "host_sanitize.cpp"),
           os.path.join(root, "turboquant-pytorch_amd", "csrc", "tq_host.cpp"), "-o", exe,
           "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")      # (the HIP runtime keeps its own allocations until exit)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr[-3000:]
