"""GPU tests of the V2 key path (MSE codes + 1-bit QJL signs of the residual, scores from the packed form) and of the V2
value compressor, against outputs of the reference classes (tests/golden/v2_qjl.npz, written by
tests/golden/make_fixtures_v2.py) and against the numpy oracle (oracle.QjlOracle) on larger seeded inputs."""
import os

import numpy as np
import pytest
import torch

from test_gpu_parity import DEV, bits16, outlier_kv, to_torch

pytestmark = pytest.mark.gpu
FX = os.path.join(os.path.dirname(__file__), "golden", "v2_qjl.npz")
SIGN_WINDOW = 1e-4      # |projection| / (|S row| * |residual|) below which a sign may differ from the float32 reference


@pytest.fixture(scope="module")
def fx():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a HIP device; there is no CPU fallback to test")
    return np.load(FX)


def _check_key_path(oracle, comp, x_f32, packed, label, ref_signs=None, ref_rnorm=None):
    """Packed output of TurboQuantCompressorV2.compress against the oracle on the same float32 inputs (and, when given,
    against the reference's own signs and residual norms).  Vectors in which a code moved (a coordinate within 1e-5
    of a decision boundary) have another residual and are left out of the sign comparison."""
    D = x_f32.shape[-1]
    orc = oracle.QjlOracle(comp.Pi.cpu().numpy(), comp.S.cpu().numpy(), comp.centroids.cpu().numpy())
    ref = orc.compress(x_f32)
    G = packed["idx_bytes"].shape[-1]
    got_codes = packed["idx_bytes"].cpu().numpy().reshape(-1, G)
    rep = oracle.code_mismatch_report(got_codes, orc.mse.pack(ref["codes"]), ref["rotated"], orc.centroids, comp.mse_bits, 1e-5)
    assert rep["outside_window"] == 0 and rep["differ"] <= max(3, 3e-4 * rep["coords"]), (label, rep)
    same = (oracle.unpack_codes(got_codes, D, comp.mse_bits) == ref["codes"]).all(-1)
    ulp = oracle.fp16_ulp_distance(bits16(packed["vec_norms"]).reshape(-1), ref["norms_f32"].astype(np.float16).view(np.uint16))
    assert ulp.max() <= 1, label
    want_signs = ref["signs"] if ref_signs is None else ref_signs
    got_bytes = packed["sign_bytes"].cpu().numpy().reshape(-1, -(-D // 8))
    if D % 8:       # the bits a vector does not fill stay clear
        assert not (got_bytes[:, -1] & ((1 << (8 - D % 8)) - 1)).any(), label
    got_signs = np.unpackbits(got_bytes, axis=-1, bitorder="big")[:, :D].astype(np.int8) * 2 - 1
    diff = (got_signs != want_signs) & same[:, None]
    srow = np.linalg.norm(orc.S, axis=1)
    margin = np.abs(ref["projected"]) / (srow[None, :] * np.maximum(ref["residual_norm_f32"][:, None], 1e-30))
    print(f"[v2] {label}: {int(diff.sum())} of {int(same.sum()) * D} sign bits differ (largest margin "
          f"{float(margin[diff].max()) if diff.any() else 0:.1e}), {int((~same).sum())} vectors with a moved code")
    assert (margin[diff] < SIGN_WINDOW).all() and diff.sum() <= max(4, 2e-4 * diff.size), label
    want_rn = ref["residual_norm"] if ref_rnorm is None else ref_rnorm
    rn_ulp = oracle.fp16_ulp_distance(bits16(packed["residual_norm"]).reshape(-1)[same], want_rn.reshape(-1)[same])
    assert rn_ulp.max() <= 1 and (rn_ulp > 0).mean() < 0.02, (label, int(rn_ulp.max()))
    # a vector with a sign that moved (a projection within the window of zero) has other scores: one sign changes the
    # second term by 2 * sqrt(pi/2)/D * |residual| * |(S q)_j|; such vectors are left out of the score comparisons too
    return orc, ref, same & ~diff.any(-1)


def test_v2_keys_against_reference_vectors(pkg, oracle, fx):
    """Every width x input type of the fixture file: codes, norms, sign bits and residual norms against the reference's
    outputs; the expanded form (`reference_format`) against its fp16 reconstruction; scores from the packed bytes
    against its asymmetric_attention_scores on its own compressed dict."""
    for bits in (2, 3, 4, 5):
        comp = pkg.TurboQuantCompressorV2.from_tensors(torch.from_numpy(fx[f"b{bits}_Pi"]), torch.from_numpy(fx[f"b{bits}_S"]),
                                                       torch.from_numpy(fx[f"b{bits}_centroids"]), bits, device=DEV)
        assert comp.mse_bits == max(bits - 1, 1)
        for dn in ("f16", "bf16", "f32"):
            tag = f"b{bits}_{dn}"
            x = to_torch(fx[tag + "_x"], dn).reshape(1, 2, 80, 128)
            packed = comp.compress(x.to(DEV))
            assert packed["shape"] == (1, 2, 80, 128) and packed["sign_bytes"].shape == (1, 2, 80, 16)
            assert packed["sign_bytes"].dtype == torch.uint8 and packed["residual_norm"].dtype == torch.float16
            orc, ref, same = _check_key_path(oracle, comp, x.float().numpy().reshape(-1, 128), packed, tag,
                                             fx[tag + "_qjl_signs"].reshape(-1, 128), fx[tag + "_residual_norm"].reshape(-1))
            assert bool((packed["sign_bytes"][0, 0, 0] == 0xFF).all())      # the all-zero vector: every projection is 0 -> +1
            exp = comp.reference_format(packed)
            assert exp["k_mse"].dtype == torch.float16 and exp["qjl_signs"].dtype == torch.int8
            k_ref = fx[tag + "_k_mse"].view(np.float16).astype(np.float32).reshape(-1, 128)
            k_got = exp["k_mse"].float().cpu().numpy().reshape(-1, 128)
            err = np.linalg.norm(k_got[same] - k_ref[same]) / np.linalg.norm(k_ref[same])
            assert err < 1.5e-3, (tag, err)                                  # fp16 norm and fp16 output rounding
            q = torch.from_numpy(fx[tag + "_q"]).to(DEV)
            got = comp.asymmetric_attention_scores(q, packed).cpu().numpy()
            want = fx[tag + "_scores"]
            assert got.shape == want.shape == (1, 2, 5, 80)
            keep = same.reshape(1, 2, 1, 80).repeat(5, axis=2)
            scale = np.linalg.norm(fx[tag + "_q"], axis=-1)[..., None] * np.linalg.norm(x.float().numpy(), axis=-1)[:, :, None, :]
            bad = np.abs(got - want)[keep] / np.maximum(scale[keep], 1e-30)
            print(f"[v2] {tag}: scores from packed bytes vs the reference, largest error / (|q| |k|) = {bad.max():.2e}")
            assert bad.max() < 1e-3, tag
            # the same dict expanded into the reference's format takes the plain-product path and agrees
            alt = comp.asymmetric_attention_scores(q, exp).cpu().numpy()
            assert (np.abs(alt - got)[keep] / np.maximum(scale[keep], 1e-30)).max() < 1e-3


@pytest.mark.parametrize("bits,dtype,n_tok", [(3, torch.bfloat16, 3001), (4, torch.float16, 517), (2, torch.float32, 1000), (8, torch.bfloat16, 700)])
def test_v2_keys_against_oracle_at_scale(pkg, oracle, bits, dtype, n_tok):
    """Ragged sizes, several rows, more than 32 queries (several launches per term), every packing class; the estimate is
    checked for what it is for as well: unbiased against the true inner products."""
    comp = pkg.TurboQuantCompressorV2(128, bits, seed=1000 * bits + 7, device=DEV)
    x = outlier_kv((2, 3, n_tok, 128), seed=90 + bits, dtype=dtype)
    packed = comp.compress(x.to(DEV))
    orc, ref, same = _check_key_path(oracle, comp, x.float().numpy().reshape(-1, 128), packed, f"b{bits} {dtype} {n_tok}")
    g = torch.Generator().manual_seed(bits)
    q = torch.randn(2, 3, 37, 128, generator=g)
    got = comp.asymmetric_attention_scores(q.to(DEV), packed).cpu().numpy()
    k16 = ref["k_mse_f16"].reshape(6, n_tok, 128)
    want = orc.scores(q.numpy().reshape(6, 37, 128), k16, ref["signs"].reshape(6, n_tok, 128), ref["residual_norm"].reshape(6, n_tok))
    scale = np.linalg.norm(q.numpy().reshape(6, 37, 1, 128), axis=-1) * np.linalg.norm(x.float().numpy().reshape(6, 1, n_tok, 128), axis=-1)
    keep = same.reshape(6, 1, n_tok).repeat(37, axis=1)
    err = (np.abs(got.reshape(6, 37, n_tok) - want) / scale)[keep]
    print(f"[v2] b{bits}: scores vs oracle, largest error / (|q| |k|) = {err.max():.2e}")
    assert err.max() < 1e-3
    true = np.einsum("rqd,rtd->rqt", q.numpy().reshape(6, 37, 128).astype(np.float64), x.float().numpy().reshape(6, n_tok, 128).astype(np.float64))
    bias = ((got.reshape(6, 37, n_tok) - true) / scale).mean()
    spread = ((got.reshape(6, 37, n_tok) - true) / scale).std()
    print(f"[v2] b{bits}: estimate - true inner product, in units of |q| |k|: mean {bias:.2e}, std {spread:.2e}")
    assert abs(bias) < 4 * spread / np.sqrt(true.size) + 1e-4


def test_v2_value_compressor_against_reference_vectors(pkg, oracle, fx):
    """TurboQuantCompressorMSE: one code per byte as the reference returns them, norms, reconstruction."""
    for bits in (2, 3, 4, 5):
        tag = f"b{bits}_f16"
        comp = pkg.TurboQuantCompressorMSE(128, bits, seed=1000 * bits + 500, device=DEV)
        assert np.array_equal(comp.centroids.cpu().numpy(), fx[f"b{bits}_v_centroids"])
        assert np.abs(comp.Pi.cpu().numpy() - fx[f"b{bits}_v_Pi"]).max() < 1e-5
        comp = pkg.TurboQuantCompressorMSE(128, bits, seed=1000 * bits + 500, device=DEV)
        comp._mse = pkg.MSECompressor.from_tensors(torch.from_numpy(fx[f"b{bits}_v_Pi"]), torch.from_numpy(fx[f"b{bits}_v_centroids"]), bits, device=DEV)
        x = to_torch(fx[tag + "_x"], "f16").reshape(1, 2, 80, 128)
        c = comp.compress(x.to(DEV))
        assert c["indices"].shape == (160, 128) and c["indices"].dtype == torch.uint8 and c["vec_norms"].shape == (160,)
        got, want = c["indices"].cpu().numpy(), fx[tag + "_v_indices"]
        rot = oracle.NumpyOracle(fx[f"b{bits}_v_Pi"], fx[f"b{bits}_v_centroids"], bits).rotate(x.float().numpy().reshape(-1, 128))[1]
        moved = got != want
        assert moved.sum() <= 3
        if moved.any():
            cent = fx[f"b{bits}_v_centroids"].astype(np.float64)
            lo = np.minimum(got, want)[moved].astype(int)
            assert (np.abs(rot[moved] - 0.5 * (cent[lo] + cent[lo + 1])) < 1e-5).all()
        assert oracle.fp16_ulp_distance(bits16(c["vec_norms"]), fx[tag + "_v_vec_norms"].reshape(-1)).max() <= 1
        rec = comp.decompress({"indices": torch.from_numpy(want).to(DEV), "vec_norms": to_torch(fx[tag + "_v_vec_norms"], "f16").to(DEV),
                               "shape": (1, 2, 80, 128)})
        ref = fx[tag + "_v_recon"]
        assert rec.dtype == torch.float32 and rec.shape == ref.shape
        err = np.linalg.norm(rec.cpu().numpy() - ref) / np.linalg.norm(ref)
        assert err < 1e-3, (bits, err)


@pytest.mark.parametrize("bits,dtype", [(3, torch.bfloat16), (5, torch.float16), (2, torch.bfloat16)])
def test_v2_one_pass_form_against_the_two_kernel_form(pkg, oracle, bits, dtype):
    """The one-pass kernel (residual in rotated coordinates, projection by S Pi^T) against tq_compress followed by
    tq_qjl_signs on the same vectors: identical codes and norms, sign bits that differ only where a projection lies
    within 1e-5 of |S row| |residual| of zero, residual norms within one fp16 unit; single call and batched list."""
    import ctypes
    native = pkg._native
    L, n = 3, 4096 + 32 * 7 + 11                 # full tiles for the one-pass kernel, a ragged end for the other form
    comps = [pkg.TurboQuantCompressorV2(128, bits, seed=31 * l + bits, device=DEV) for l in range(L)]
    xs = [outlier_kv((1, 1, n, 128), seed=300 + l, dtype=dtype).to(DEV) for l in range(L)]
    packed = [c.empty_packed(1, 1, n, DEV) for c in comps]
    for p in packed:
        for k in ("idx_bytes", "vec_norms", "sign_bytes", "residual_norm"):
            p[k].fill_(0x55 if p[k].dtype == torch.uint8 else 3.0)
    native.QjlJobList([c.job(x, p) for c, x, p in zip(comps, xs, packed)], torch.device(DEV)).compress()
    torch.cuda.synchronize()
    for c, x, p in zip(comps, xs, packed):
        single = c.compress(x)
        for k in ("idx_bytes", "vec_norms", "sign_bytes", "residual_norm"):
            assert torch.equal(single[k].view(torch.uint8), p[k].view(torch.uint8)), k       # the list and the single call agree
        # the two-kernel form through the C entry points
        first = c._mse.compress(x)
        sb = torch.empty_like(p["sign_bytes"])
        rn = torch.empty_like(p["residual_norm"])
        rc = native.lib().tq_qjl_signs(x.data_ptr(), native.dtype_code(x.dtype), n, 128, first["idx_bytes"].data_ptr(),
                                       c._table(DEV).data_ptr(), 128, c.mse_bits, sb.data_ptr(), rn.data_ptr(),
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(first["idx_bytes"], p["idx_bytes"]) and torch.equal(first["vec_norms"].view(torch.int16), p["vec_norms"].view(torch.int16))
        a = np.unpackbits(p["sign_bytes"].cpu().numpy().reshape(-1, 16), axis=-1, bitorder="big")
        b = np.unpackbits(sb.cpu().numpy().reshape(-1, 16), axis=-1, bitorder="big")
        diff = a != b
        orc = oracle.QjlOracle(c.Pi.cpu().numpy(), c.S.cpu().numpy(), c.centroids.cpu().numpy())
        ref = orc.compress(x.float().cpu().numpy().reshape(-1, 128))
        srow = np.linalg.norm(orc.S, axis=1)
        margin = np.abs(ref["projected"]) / (srow[None, :] * np.maximum(ref["residual_norm_f32"][:, None], 1e-30))
        print(f"[v2] one pass vs two kernels, {bits} bits {dtype}: {int(diff.sum())} of {diff.size} sign bits differ, "
              f"largest margin {float(margin[diff].max()) if diff.any() else 0:.1e}")
        assert diff.sum() <= max(4, 5e-5 * diff.size) and (margin[diff] < 1e-5).all()
        ulp = oracle.fp16_ulp_distance(bits16(p["residual_norm"]).reshape(-1), bits16(rn).reshape(-1))
        assert ulp.max() <= 1 and (ulp > 0).mean() < 0.02


@pytest.mark.parametrize("D,bits,dtype", [(64, 3, torch.bfloat16), (256, 4, torch.float16), (96, 2, torch.float32),
                                          (80, 3, torch.float16), (45, 3, torch.bfloat16)])
def test_v2_keys_at_other_head_dimensions(pkg, oracle, D, bits, dtype):
    """Head dimensions other than 128: codes and norms from the MSE kernels, the residual part as float32 tensor
    operations on the device.  Same checks as for 128-wide heads."""
    n_tok = 333
    comp = pkg.TurboQuantCompressorV2(D, bits, seed=17 * bits + D, device=DEV)
    x = outlier_kv((2, 2, n_tok, D), seed=70 + bits, dtype=dtype)
    packed = comp.compress(x.to(DEV))
    assert packed["sign_bytes"].shape == (2, 2, n_tok, -(-D // 8)) and packed["idx_bytes"].shape[-1] == -(-D // (8 // comp.mse_bits))
    orc, ref, same = _check_key_path(oracle, comp, x.float().numpy().reshape(-1, D), packed, f"d{D} b{bits} {dtype}")
    g = torch.Generator().manual_seed(bits)
    q = torch.randn(2, 2, 9, D, generator=g)
    got = comp.asymmetric_attention_scores(q.to(DEV), packed).cpu().numpy()
    k16 = ref["k_mse_f16"].reshape(4, n_tok, D)
    want = orc.scores(q.numpy().reshape(4, 9, D), k16, ref["signs"].reshape(4, n_tok, D), ref["residual_norm"].reshape(4, n_tok))
    scale = np.linalg.norm(q.numpy().reshape(4, 9, 1, D), axis=-1) * np.linalg.norm(x.float().numpy().reshape(4, 1, n_tok, D), axis=-1)
    keep = same.reshape(4, 1, n_tok).repeat(9, axis=1)
    err = (np.abs(got.reshape(4, 9, n_tok) - want) / scale)[keep]
    assert err.max() < 1e-3
