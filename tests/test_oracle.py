"""The CPU oracle against the reference's own outputs and against what the mathematics fixes.

Nothing here needs a GPU.  Two independent restatements (numpy op-sequence, scalar C) are checked
against tests/golden/*.npz (written by the real reference), against each other, against exhaustive
enumeration of the packing and brute-force nearest-centroid search.
"""
import hashlib

import numpy as np
import pytest
import torch

BITS = (1, 2, 3, 4, 5, 6, 7, 8)


def _cases(golden):
    fx = golden["mse_roundtrip"]
    for b in BITS:
        for dn in ("f32", "f16", "bf16"):
            if f"b{b}_{dn}_x" in fx:
                yield b, dn


def test_roundtrip_fixtures_numpy_bit_exact(golden, oracle):
    """The numpy op-sequence restatement reproduces the reference's bytes, norms and fp32
    reconstruction bit for bit on every fixture (same BLAS, same op order)."""
    fx = golden["mse_roundtrip"]
    n = 0
    for b, dn in _cases(golden):
        orc = oracle.NumpyOracle(fx[f"Pi_b{b}"], fx[f"centroids_b{b}"], b)
        x = oracle.widen(fx[f"b{b}_{dn}_x"], dn)
        with np.errstate(over="ignore", invalid="ignore"):
            out = orc.compress(x)
        ref_bytes = fx[f"b{b}_{dn}_idx_bytes"]
        assert np.array_equal(out["idx_bytes"], ref_bytes.reshape(-1, ref_bytes.shape[-1])), (b, dn)
        assert np.array_equal(out["vec_norms"], fx[f"b{b}_{dn}_vec_norms"].reshape(-1)), (b, dn)
        rec = orc.decompress(ref_bytes, fx[f"b{b}_{dn}_vec_norms"])
        assert np.array_equal(rec.view(np.uint32), fx[f"b{b}_{dn}_recon"].reshape(-1, 128).view(np.uint32)), (b, dn)
        n += 1
    assert n == 20


ODD_DIM_CASES = ((45, 2), (45, 3), (45, 4), (80, 2), (80, 4), (100, 1), (100, 3), (112, 4), (200, 2))


def test_odd_head_dimensions_numpy(golden, oracle):
    """Head dimensions that are not a multiple of 32, some with codes that do not fill their last byte (the zero padding
    of the codes, compressors_v3.py:64-68, and its removal, :101-102): the numpy restatement reproduces the reference's
    bytes and norms bit for bit and its fp32 reconstruction to rounding."""
    fx = golden["odd_dims"]
    pads = set()
    for d, b in ODD_DIM_CASES:
        orc = oracle.NumpyOracle(fx[f"Pi_d{d}_b{b}"], fx[f"centroids_d{d}_b{b}"], b)
        for dn in ("f32", "f16", "bf16"):
            key = f"d{d}_b{b}_{dn}"
            x = oracle.widen(fx[key + "_x"], dn)
            with np.errstate(over="ignore", invalid="ignore"):
                out = orc.compress(x)
            ref_bytes = fx[key + "_idx_bytes"]
            ipb = 8 // b
            assert ref_bytes.shape[-1] == -(-d // ipb) == oracle.bytes_per_vector(d, b)
            assert int(fx[key + "_idx_pad"][0]) == (ipb - d % ipb) % ipb
            pads.add(int(fx[key + "_idx_pad"][0]))
            assert np.array_equal(out["idx_bytes"], ref_bytes.reshape(-1, ref_bytes.shape[-1])), key
            assert np.array_equal(out["vec_norms"], fx[key + "_vec_norms"].reshape(-1)), key
            # the reconstruction's last bits depend on how the BLAS at hand blocks a contraction of this length (bit for bit
            # at 45 and 80, a few units in the last place at 100 and beyond)
            rec = orc.decompress(ref_bytes, fx[key + "_vec_norms"])
            ref = fx[key + "_recon"].reshape(-1, d)
            fin = np.isfinite(ref).all(-1)
            assert np.array_equal(np.isfinite(rec).all(-1), fin), key
            assert np.abs(rec[fin] - ref[fin]).max() <= 2e-6 * max(1.0, np.abs(ref[fin]).max()), key
    assert pads == {0, 1, 3, 4}


def test_odd_head_dimensions_c(golden, oracle):
    """The scalar C restatement on the same fixtures: the reference's codes except on a decision boundary, its norms
    to one fp16 step, its reconstruction to rounding."""
    fx = golden["odd_dims"]
    for d, b in ODD_DIM_CASES:
        cent = fx[f"centroids_d{d}_b{b}"]
        orc = oracle.COracle(fx[f"Pi_d{d}_b{b}"], cent, b)
        for dn in ("f32", "f16", "bf16"):
            key = f"d{d}_b{b}_{dn}"
            x = oracle.widen(fx[key + "_x"], dn)
            out = orc.compress(x)
            ref_bytes = fx[key + "_idx_bytes"]
            ref_bytes = ref_bytes.reshape(-1, ref_bytes.shape[-1])
            if not np.array_equal(out["idx_bytes"], ref_bytes):
                rot = oracle.NumpyOracle(fx[f"Pi_d{d}_b{b}"], cent, b).rotate(x)[1]
                rep = oracle.code_mismatch_report(out["idx_bytes"], ref_bytes, rot, cent, b)
                assert rep["outside_window"] == 0 and rep["differ"] <= 2, (key, rep)
            assert oracle.fp16_ulp_distance(out["vec_norms"], fx[key + "_vec_norms"].reshape(-1)).max() <= 1
            rec = orc.decompress(ref_bytes, fx[key + "_vec_norms"].reshape(-1))
            ref = fx[key + "_recon"].reshape(-1, d)
            fin = np.isfinite(ref).all(-1)
            assert np.abs(rec[fin] - ref[fin]).max() <= 1e-5 * max(1.0, np.abs(ref[fin]).max()), key


def test_roundtrip_fixtures_torch_cpu_op_sequence(golden, oracle):
    """The torch CPU op sequence that the benchmark times as the reference's CPU path: the reference's bytes and
    norms on every fixture (a tiny chunk size, so that the chunk loop is what is tested), fp32 reconstruction to
    rounding (sgemm blocks its sums by the row count, so the last bits move with the chunk size)."""
    fx = golden["mse_roundtrip"]
    for b, dn in _cases(golden):
        cent = fx[f"centroids_b{b}"]
        x = torch.from_numpy(oracle.widen(fx[f"b{b}_{dn}_x"], dn))
        ref_bytes = fx[f"b{b}_{dn}_idx_bytes"]
        ref_bytes = ref_bytes.reshape(-1, ref_bytes.shape[-1])
        ref_norms = fx[f"b{b}_{dn}_vec_norms"].reshape(-1)
        for chunk in (0, 7):
            orc = oracle.TorchCpuOracle(fx[f"Pi_b{b}"], cent, b, chunk=chunk)
            with np.errstate(over="ignore", invalid="ignore"):
                got_b, got_n = orc.compress(x)
            got_b = got_b.numpy()
            if not np.array_equal(got_b, ref_bytes):      # only a coordinate on a decision boundary may move
                rot = oracle.NumpyOracle(fx[f"Pi_b{b}"], cent, b).rotate(x.numpy())[1]
                rep = oracle.code_mismatch_report(got_b, ref_bytes, rot, cent, b)
                assert rep["outside_window"] == 0 and rep["differ"] <= 2, (b, dn, chunk, rep)
            assert oracle.fp16_ulp_distance(got_n.view(torch.int16).numpy().view(np.uint16), ref_norms).max() <= 1
            rec = orc.decompress(torch.from_numpy(ref_bytes), torch.from_numpy(ref_norms.view(np.float16))).numpy()
            ref = fx[f"b{b}_{dn}_recon"].reshape(-1, 128)
            fin = np.isfinite(ref).all(-1)
            assert np.array_equal(np.isfinite(rec).all(-1), fin)
            assert np.abs(rec[fin] - ref[fin]).max() <= 1e-5 * max(1.0, np.abs(ref[fin]).max())
    assert oracle.TorchCpuOracle(fx["Pi_b8"], fx["centroids_b8"], 8).chunk == 4096       # 4096 x 128 x 256 x 4 B = 512 MiB
    assert oracle.TorchCpuOracle(fx["Pi_b2"], fx["centroids_b2"], 2).chunk == 262144


@pytest.mark.parametrize("accum_double", [False, True])
def test_roundtrip_fixtures_c(golden, oracle, accum_double):
    """The scalar C restatement: same codes except inside the 1e-5 boundary window (none seen),
    norms within one fp16 ulp, reconstruction to fp32 rounding."""
    fx = golden["mse_roundtrip"]
    for b, dn in _cases(golden):
        cent = fx[f"centroids_b{b}"]
        orc = oracle.COracle(fx[f"Pi_b{b}"], cent, b, accum_double)
        x = oracle.widen(fx[f"b{b}_{dn}_x"], dn)
        out = orc.compress(x)
        ref_bytes = fx[f"b{b}_{dn}_idx_bytes"]
        ref_bytes = ref_bytes.reshape(-1, ref_bytes.shape[-1])
        rep = oracle.code_mismatch_report(out["idx_bytes"], ref_bytes, out["rotated"], cent, b)
        assert rep["outside_window"] == 0, (b, dn, rep)
        assert rep["differ"] <= 2, (b, dn, rep)
        ulp = oracle.fp16_ulp_distance(out["vec_norms"], fx[f"b{b}_{dn}_vec_norms"].reshape(-1))
        assert ulp.max() <= 1
        rec = orc.decompress(ref_bytes, fx[f"b{b}_{dn}_vec_norms"].reshape(-1))
        ref = fx[f"b{b}_{dn}_recon"].reshape(-1, 128)
        finite = np.isfinite(ref).all(-1)
        assert np.array_equal(np.isfinite(rec).all(-1), finite)
        rel = np.linalg.norm(rec[finite] - ref[finite]) / np.linalg.norm(ref[finite])
        assert rel < 1e-6, (b, dn, rel)


def test_config1_known_answer(golden, oracle):
    """The reference's CPU-runnable case (K [1,8,1024,128] fp32 N(0,1) seed 0, 4-bit, rotation seed 42): the
    reference's SHA-256 of packed bytes, norms and reconstruction, its MSE and cosine."""
    meta = golden["json"]["config1"]
    torch.manual_seed(0)
    k = torch.randn(1, 8, 1024, 128).numpy()
    assert hashlib.sha256(k.tobytes()).hexdigest() == meta["input_sha256"]
    Pi = golden["rotations"]["Pi_d128_s42"]
    cent = golden["codebooks"]["centroids_d128_b4"]
    ref_bytes = golden["config1"]["idx_bytes"].reshape(-1, 64)
    ref_norms = golden["config1"]["vec_norms"].reshape(-1)
    assert meta["packed_bytes"] == ref_bytes.size + 2 * ref_norms.size == 540672

    out = oracle.NumpyOracle(Pi, cent, 4).compress(k)
    assert hashlib.sha256(out["idx_bytes"].tobytes()).hexdigest() == meta["idx_bytes_sha256"]
    assert hashlib.sha256(out["vec_norms"].tobytes()).hexdigest() == meta["vec_norms_sha256"]
    rec = oracle.NumpyOracle(Pi, cent, 4).decompress(ref_bytes, ref_norms)
    assert hashlib.sha256(rec.tobytes()).hexdigest() == meta["recon_sha256"]
    flat = k.reshape(-1, 128)
    mse = float(((flat - rec) ** 2).mean())
    cos = (flat * rec).sum(-1) / (np.linalg.norm(flat, axis=-1) * np.linalg.norm(rec, axis=-1))
    assert abs(mse - meta["mse_per_element"]) < 1e-7
    assert abs(float(cos.mean()) - meta["cosine_mean"]) < 1e-6
    # textbook 4-bit Gaussian Lloyd-Max distortion is 0.009497 per unit variance
    assert 0.0090 < meta["rel_mse"] < 0.0098

    for dbl in (False, True):
        c = oracle.COracle(Pi, cent, 4, dbl).compress(k)
        rep = oracle.code_mismatch_report(c["idx_bytes"], ref_bytes, c["rotated"], cent, 4)
        assert rep["outside_window"] == 0 and rep["differ"] <= 8, rep
        assert oracle.fp16_ulp_distance(c["vec_norms"], ref_norms).max() <= 1


@pytest.mark.parametrize("bits", BITS)
def test_pack_unpack_exhaustive(oracle, bits):
    """Closed form of the packing: byte = sum code_k << bits*(ipb-1-k), MSB first; every byte value
    decodes and re-encodes to itself (masked to the used bits); C and numpy agree."""
    ipb = 8 // bits
    used = (1 << (bits * ipb)) - 1
    D = 128
    G = -(-D // ipb)
    assert oracle.bytes_per_vector(D, bits) == G == {1: 16, 2: 32, 3: 64, 4: 64}.get(bits, 128)
    npo = oracle.NumpyOracle(np.eye(D, dtype=np.float32), np.zeros(1 << bits, np.float32), bits)
    lib = oracle._load()
    # all 256 byte values in every byte position class
    allbytes = ((np.arange(256)[:, None] + 37 * np.arange(G)[None, :]) % 256).astype(np.uint8)
    codes = npo.unpack(allbytes)
    assert codes.shape == (256, D) and codes.max() <= (1 << bits) - 1
    assert np.array_equal(npo.pack(codes), allbytes & used)
    for row in range(0, 256, 17):
        c_codes = np.empty(D, np.uint8)
        lib.tqo_unpack(np.ascontiguousarray(allbytes[row]), D, bits, c_codes)
        assert np.array_equal(c_codes, codes[row])
        c_bytes = np.empty(G, np.uint8)
        lib.tqo_pack(c_codes, D, bits, c_bytes)
        assert np.array_equal(c_bytes, allbytes[row] & used)
    # hand-computed example: codes 1,2,3,... -> first byte
    seq = (np.arange(D) % (1 << bits)).astype(np.uint8)
    first = 0
    for k in range(ipb):
        first |= int(seq[k]) << (bits * (ipb - 1 - k))
    assert npo.pack(seq[None])[0, 0] == first


def test_pack_with_padding(oracle):
    """head_dim not a multiple of ipb: zero padding at the end (compressors_v3.py:65-68)."""
    npo = oracle.NumpyOracle(np.eye(6, dtype=np.float32), np.zeros(4, np.float32), 2)
    codes = np.array([[3, 2, 1, 0, 1, 2]], dtype=np.uint8)
    packed = npo.pack(codes)
    assert packed.tolist() == [[0b11100100, 0b01100000]]
    assert np.array_equal(npo.unpack(packed), codes)
    c = np.empty(2, np.uint8)
    oracle._load().tqo_pack(np.ascontiguousarray(codes[0]), 6, 2, c)
    assert c.tolist() == [0b11100100, 0b01100000]


@pytest.mark.parametrize("bits", (1, 2, 4, 8))
def test_nearest_bruteforce(golden, oracle, bits):
    """argmin with first-minimum ties: C loop == numpy argmin == literal Python on tiny inputs."""
    cent = golden["codebooks"][f"centroids_d128_b{bits}"]
    rng = np.random.default_rng(bits)
    r = rng.normal(0, 0.1, 4000).astype(np.float32)
    mids = ((cent[:-1].astype(np.float64) + cent[1:]) / 2).astype(np.float32)
    r = np.concatenate([r, cent, mids, np.nextafter(mids, np.float32(1)), np.nextafter(mids, np.float32(-1)),
                        np.array([0.0, -0.0, 1.0, -1.0], np.float32)])
    got = np.empty(r.size, np.uint8)
    oracle._load().tqo_nearest(r, r.size, cent, cent.size, got)
    ref = np.abs(r[:, None] - cent[None, :]).argmin(-1)
    assert np.array_equal(got, ref)
    for i in range(0, r.size, 97):
        best, bd = 0, abs(np.float32(r[i] - cent[0]))
        for j in range(1, cent.size):
            d = abs(np.float32(r[i] - cent[j]))
            if d < bd:
                best, bd = j, d
        assert best == got[i]
    # exact ties go to the lower index
    two = np.array([-0.5, 0.5], np.float32)
    t = np.empty(1, np.uint8)
    oracle._load().tqo_nearest(np.zeros(1, np.float32), 1, two, 2, t)
    assert t[0] == 0


def test_fp16_conversion_matches_numpy(oracle):
    """The C oracle's fp16 rounding == numpy's (round to nearest even, overflow to inf, subnormals)."""
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.normal(0, 1, 20000).astype(np.float32) * np.float32(10) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0, -0.0, 65504, 65519.99, 65520, 70000, 1e-8, 5.96e-8, 2.98e-8, 2.9802325e-8, 6.1e-5, np.inf, -np.inf],
                 np.float32)])
    out = np.empty(x.size, np.uint16)
    oracle._load().tqo_f32_to_f16(x, out, x.size)
    with np.errstate(over="ignore"):
        assert np.array_equal(out, x.astype(np.float16).view(np.uint16))
    allh = np.arange(65536, dtype=np.uint16)
    back = np.empty(65536, np.float32)
    oracle._load().tqo_f16_to_f32(allh, back, 65536)
    ref = allh.view(np.float16).astype(np.float32)
    ok = np.isnan(ref) | (back.view(np.uint32) == ref.view(np.uint32))
    assert ok.all()


def test_norm_has_no_epsilon_and_unit_scale(golden, oracle):
    """The stored norm is the plain L2 norm in fp16 (eps only in the divisor); scaling a vector by
    a power of two leaves its codes unchanged and scales the norm (linearity / invariance)."""
    Pi = golden["rotations"]["Pi_d128_s42"]
    cent = golden["codebooks"]["centroids_d128_b4"]
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, (64, 128)).astype(np.float32)
    for orc in (oracle.NumpyOracle(Pi, cent, 4), oracle.COracle(Pi, cent, 4)):
        a = orc.compress(x)
        b = orc.compress(x * np.float32(4))
        assert np.array_equal(a["idx_bytes"], b["idx_bytes"])
        na = a["vec_norms"].view(np.float16).astype(np.float32)
        nb = b["vec_norms"].view(np.float16).astype(np.float32)
        assert np.array_equal(na * 4, nb)
        assert np.abs(na - np.linalg.norm(x, axis=-1)).max() < 0.01
        # identity rotation + one-hot input: the hot coordinate gets the top code, the rest the
        # code nearest to zero
    eye = np.eye(128, dtype=np.float32)
    onehot = np.zeros((1, 128), np.float32)
    onehot[0, 5] = 2.0
    out = oracle.COracle(eye, cent, 4).compress(onehot)
    codes = oracle.unpack_codes(out["idx_bytes"], 128, 4)[0]
    assert codes[5] == 15 and set(np.delete(codes, 5)) == {7}
    assert out["vec_norms"].view(np.float16)[0] == np.float16(2.0)


def test_decompress_inverts_rotation(golden, oracle):
    """Orthogonality: decompress(codes) = (centroids[codes] @ Pi) * norm, so rotating it back
    returns the centroids; checked against a float64 evaluation."""
    Pi = golden["rotations"]["Pi_d128_s542"]
    cent = golden["codebooks"]["centroids_d128_b2"]
    rng = np.random.default_rng(9)
    codes = rng.integers(0, 4, (32, 128)).astype(np.uint8)
    npo = oracle.NumpyOracle(Pi, cent, 2)
    packed = npo.pack(codes)
    norms = np.full(32, np.float16(3.0)).view(np.uint16)
    ref = (cent[codes].astype(np.float64) @ Pi.astype(np.float64)) * 3.0
    for orc in (npo, oracle.COracle(Pi, cent, 2), oracle.COracle(Pi, cent, 2, True)):
        rec = orc.decompress(packed, norms)
        assert np.abs(rec - ref).max() < 2e-6
        back = (rec.astype(np.float64) / 3.0) @ Pi.astype(np.float64).T
        assert np.abs(back - cent[codes]).max() < 2e-6


def test_attention_decode_oracle_is_textbook_attention(oracle):
    """The float64 checker equals torch's scaled_dot_product_attention (grouped heads expanded) and a
    brute-force loop over heads and tokens."""
    rng = np.random.default_rng(5)
    B, H, G, S, D = 2, 3, 4, 37, 16
    q = rng.standard_normal((B, H * G, D)).astype(np.float32)
    K = rng.standard_normal((B, H, S, D)).astype(np.float32)
    V = rng.standard_normal((B, H, S, D)).astype(np.float32)
    scale = 0.3
    scores, out = oracle.attention_decode(q, K, V, scale)
    tq, tK, tV = (torch.from_numpy(a).double() for a in (q, K, V))
    ref = torch.nn.functional.scaled_dot_product_attention(
        tq.unsqueeze(2), tK.repeat_interleave(G, dim=1), tV.repeat_interleave(G, dim=1), scale=scale).squeeze(2)
    assert np.abs(out - ref.numpy()).max() < 1e-12
    for b, hq in ((0, 0), (1, 5), (1, 11)):
        h = hq // G
        s = np.array([scale * float(np.dot(q[b, hq].astype(np.float64), K[b, h, t].astype(np.float64))) for t in range(S)])
        assert np.abs(scores[b, hq] - s).max() < 1e-12
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.abs(out[b, hq] - (p[:, None] * V[b, h].astype(np.float64)).sum(0)).max() < 1e-12


def test_v2_qjl_oracle_against_reference_vectors(oracle):
    """The numpy restatement of the V2 key path against outputs of the reference class (tests/golden/v2_qjl.npz):
    stored fp16 reconstruction and residual norms to one fp16 unit, signs identical except where the projection is
    within 1e-5 * |S row| * |residual| of zero (none, or a handful), scores to float32 rounding."""
    import os
    fx = np.load(os.path.join(os.path.dirname(__file__), "golden", "v2_qjl.npz"))
    seen = 0
    for bits in (2, 3, 4, 5):
        orc = oracle.QjlOracle(fx[f"b{bits}_Pi"], fx[f"b{bits}_S"], fx[f"b{bits}_centroids"])
        assert orc.centroids.size == 1 << max(bits - 1, 1)
        srow = np.linalg.norm(orc.S, axis=1)
        for dn in ("f16", "bf16", "f32"):
            tag = f"b{bits}_{dn}"
            x = oracle.widen(fx[tag + "_x"], dn).reshape(-1, 128)
            out = orc.compress(x)
            assert oracle.fp16_ulp_distance(out["k_mse_f16"].reshape(-1), fx[tag + "_k_mse"].reshape(-1)).max() <= 1
            assert oracle.fp16_ulp_distance(out["residual_norm"], fx[tag + "_residual_norm"].reshape(-1)).max() <= 1
            ref_signs = fx[tag + "_qjl_signs"].reshape(-1, 128)
            diff = out["signs"] != ref_signs
            margin = np.abs(out["projected"]) / (srow[None, :] * np.maximum(out["residual_norm_f32"][:, None], 1e-30))
            assert diff.sum() <= 4 and (margin[diff] < 1e-5).all(), (tag, int(diff.sum()))
            assert (out["signs"][0] == 1).all()                       # the all-zero vector: projection 0 -> +1
            q = fx[tag + "_q"].reshape(2, 5, 128)
            sc = orc.scores(q, fx[tag + "_k_mse"].reshape(2, 80, 128), ref_signs.reshape(2, 80, 128),
                            fx[tag + "_residual_norm"].reshape(2, 80))
            ref = fx[tag + "_scores"].reshape(2, 5, 80)
            assert np.abs(sc - ref).max() <= 2e-5 * np.abs(ref).max(), tag
            seen += 1
    assert seen == 12
    s = np.array([[1, -1, -1, -1, -1, -1, -1, 1] + [1] * 8])
    assert oracle.pack_signs(s).tolist() == [[0x81, 0xFF]]


def test_c_oracle_under_sanitizers(tmp_path):
    """tq_oracle.c built with AddressSanitizer and UndefinedBehaviorSanitizer (host code only) and driven over ragged
    sizes, every bit width, both accumulation modes and every fp16 bit pattern: no out-of-bounds access, no overflowed
    shift, no misaligned read in the checker itself."""
    import os
    import shutil
    import subprocess
    ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc on this machine")
    src = os.path.join(ROOT, "oracle", "tq_oracle_sanitize.c")
    exe = str(tmp_path / "tq_oracle_sanitize")
    build = subprocess.run([gcc, "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=all", "-static-libasan", "-o", exe, src, "-lm"],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr
