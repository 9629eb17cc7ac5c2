"""GPU parity for head dimensions other than 128 (compress / decompress take every head dimension from 8 to 256;
upstream turboquant/compressors_v3.py:37-43 builds rotation and codebook for any head_dim, :64-68 pads the codes of a
vector to a whole byte).  Same bars as the
128-wide tests: codes bit-exact outside a 1e-5 window around a decision boundary, fp16 norms within one ulp,
reconstruction within 1e-3 relative L2 of the oracle's.
"""
import numpy as np
import pytest
import torch

from test_gpu_parity import DEV, REL_L2, TORCH_DT, bits16, check_codes, check_norms, outlier_kv, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a HIP device; there is no CPU fallback to test")


def _orthogonal(d, seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    q, r = torch.linalg.qr(torch.randn(d, d, generator=g))
    return (q * torch.sign(torch.diagonal(r))).contiguous()


def _roundtrip_against_oracle(pkg, oracle, comp, Pi, cent, bits, x, label, max_frac=None):
    dn = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}[x.dtype]
    D = x.shape[-1]
    out = comp.compress(x.to(DEV))
    ipb = 8 // bits
    assert out["idx_bytes"].shape[-1] == -(-D // ipb) and out["idx_pad"] == (ipb - D % ipb) % ipb
    ref, _ = check_codes(oracle, out["idx_bytes"].cpu().numpy(), x.float().numpy().reshape(-1, D), Pi, cent, bits, label, max_frac)
    check_norms(oracle, bits16(out["vec_norms"]), ref["vec_norms"], label)
    # de-quantise the ORACLE's packed form, so that a code on the other side of a boundary does not enter
    packed = {"idx_bytes": torch.from_numpy(ref["idx_bytes"].reshape(out["idx_bytes"].shape)).to(DEV),
              "vec_norms": torch.from_numpy(ref["vec_norms"].view(np.int16).reshape(out["vec_norms"].shape)).view(torch.float16).to(DEV),
              "shape": tuple(x.shape), "idx_pad": out["idx_pad"]}
    want = oracle.NumpyOracle(Pi, cent, bits).decompress(ref["idx_bytes"], ref["vec_norms"])
    rec = comp.decompress(packed)
    assert rec.dtype == torch.float32 and rec.shape == x.shape
    err, _ = rel_l2(rec.cpu().numpy(), want)
    print(f"[recon] {label}: relative L2 {err:.2e}")
    assert err <= REL_L2, label
    # 16-bit outputs: the fp32 result's own error plus roundings that fall the other way (one ulp: 2^-11 resp. 2^-8)
    for odt, tol in ((torch.float16, 1.5e-3), (torch.bfloat16, 4e-3)):
        o = torch.empty(x.shape, dtype=odt, device=DEV)
        comp.decompress_into(packed, o)
        want_t = torch.from_numpy(want).to(odt).float().numpy()
        err, _ = rel_l2(o.float().cpu().numpy(), want_t)
        assert err <= tol, (label, odt, err)
    return out


@pytest.mark.parametrize("D,bits", [(64, 2), (64, 4), (256, 2), (256, 4)])
def test_reference_codebooks_and_rotation(pkg, oracle, golden, D, bits):
    """The head dimensions the reference's own fixtures cover: its d=64 / d=256 codebooks, its d=64 rotation
    (seed 42); the d=256 rotation comes from this package's generator, which the CPU suite pins to the reference's."""
    cent = golden["codebooks"][f"centroids_d{D}_b{bits}"]
    comp = pkg.MSECompressor(D, bits, seed=42, device=DEV)
    Pi = comp.Pi.cpu().numpy()
    if D == 64:      # (QR on another host's LAPACK differs in the last bits: compare loosely, then use the reference's matrix)
        np.testing.assert_allclose(Pi, golden["rotations"]["Pi_d64_s42"], rtol=0, atol=2e-6)
        Pi = golden["rotations"]["Pi_d64_s42"]
    np.testing.assert_allclose(comp.centroids.cpu().numpy(), cent, rtol=0, atol=2e-6)
    comp = pkg.MSECompressor.from_tensors(torch.from_numpy(Pi), torch.from_numpy(cent), bits, device=DEV)
    for dn in ("f32", "f16", "bf16"):
        x = outlier_kv((2, 3, 173, D), seed=100 + D + bits, dtype=TORCH_DT[dn])
        _roundtrip_against_oracle(pkg, oracle, comp, Pi, cent, bits, x, f"d{D} b{bits} {dn}")


@pytest.mark.parametrize("D,bits", [(32, 1), (32, 8), (96, 3), (160, 5), (192, 6), (224, 4), (256, 8), (64, 7)])
def test_other_dimensions_and_widths(pkg, oracle, D, bits):
    """Every multiple of 32 up to 256, every packing (8, 4, 2 codes per byte, one code per byte), random orthogonal
    rotation, this package's Lloyd-Max codebook for the dimension."""
    Pi_t = _orthogonal(D, seed=7 * D + bits)
    cent_t = pkg.LloydMaxCodebook(D, bits).centroids
    comp = pkg.MSECompressor.from_tensors(Pi_t, cent_t, bits, device=DEV)
    Pi, cent = Pi_t.numpy(), cent_t.numpy()
    for dn, shape in (("f32", (1, 2, 211, D)), ("bf16", (3, 1, 129, D)), ("f16", (1, 1, 31, D))):
        x = outlier_kv(shape, seed=D + bits, dtype=TORCH_DT[dn])
        _roundtrip_against_oracle(pkg, oracle, comp, Pi, cent, bits, x, f"d{D} b{bits} {dn}", max_frac=2.5e-4 if bits > 4 else None)


ODD_DIM_CASES = ((45, 2), (45, 3), (45, 4), (80, 2), (80, 4), (100, 1), (100, 3), (112, 4), (200, 2))


@pytest.mark.parametrize("D,bits", ODD_DIM_CASES)
def test_reference_fixtures_at_head_dimensions_that_are_not_multiples_of_32(pkg, oracle, golden, D, bits):
    """The reference's own outputs at head dimensions 45, 80, 100, 112 and 200 (tests/golden/odd_dims.npz), among them
    ones whose codes do not fill the last byte of a vector: the reference's bytes except on a decision boundary (the
    padding bits among them: zero), its norms to one fp16 step, its reconstruction from its own packed form."""
    fx = golden["odd_dims"]
    Pi, cent = fx[f"Pi_d{D}_b{bits}"], fx[f"centroids_d{D}_b{bits}"]
    comp = pkg.MSECompressor.from_tensors(torch.from_numpy(Pi), torch.from_numpy(cent), bits, device=DEV)
    ipb = 8 // bits
    for dn in ("f32", "f16", "bf16"):
        key = f"d{D}_b{bits}_{dn}"
        raw = fx[key + "_x"]
        x = torch.from_numpy(raw) if dn == "f32" else torch.from_numpy(raw.view(np.int16)).view(TORCH_DT[dn])
        out = comp.compress(x.to(DEV))
        ref_bytes = fx[key + "_idx_bytes"]
        assert tuple(out["idx_bytes"].shape) == ref_bytes.shape and out["idx_pad"] == int(fx[key + "_idx_pad"][0])
        got = out["idx_bytes"].cpu().numpy().reshape(-1, ref_bytes.shape[-1])
        ref2 = ref_bytes.reshape(got.shape)
        if not np.array_equal(got, ref2):
            rot = oracle.NumpyOracle(Pi, cent, bits).rotate(oracle.widen(raw, dn))[1]
            rep = oracle.code_mismatch_report(got, ref2, rot, cent, bits)
            assert rep["outside_window"] == 0 and rep["differ"] <= 3, (key, rep)
        pad = out["idx_pad"]
        if pad:      # the bits of the codes a vector does not have
            assert not (got[:, -1] & ((1 << (bits * pad)) - 1)).any(), key
        check_norms(oracle, bits16(out["vec_norms"]), fx[key + "_vec_norms"], key)
        packed = {"idx_bytes": torch.from_numpy(ref_bytes).to(DEV),
                  "vec_norms": torch.from_numpy(fx[key + "_vec_norms"].view(np.int16)).view(torch.float16).to(DEV),
                  "shape": tuple(x.shape), "idx_pad": pad}
        rec = comp.decompress(packed).cpu().numpy()
        want = fx[key + "_recon"]
        err, fin = rel_l2(rec, want)
        assert err <= REL_L2, (key, err)
        assert np.array_equal(np.isfinite(rec).all(-1).reshape(-1), np.isfinite(want).all(-1).reshape(-1)), key
        assert not rec.reshape(-1, D)[0].any()       # the zero vector comes back as zeros


@pytest.mark.parametrize("D,bits", [(8, 4), (17, 2), (40, 8), (72, 5), (120, 3), (136, 4), (250, 1), (255, 2)])
def test_any_head_dimension_from_8_to_256(pkg, oracle, D, bits):
    """Dimensions on both sides of every multiple of 32, every packing, against the oracle; also as token-axis slices
    of a preallocated store (vectors and packed rows at addresses with no particular alignment) and as a job list."""
    Pi_t = _orthogonal(D, seed=3 * D + bits)
    cent_t = pkg.LloydMaxCodebook(D, bits).centroids
    comp = pkg.MSECompressor.from_tensors(Pi_t, cent_t, bits, device=DEV)
    Pi, cent = Pi_t.numpy(), cent_t.numpy()
    for dn, shape in (("f32", (1, 2, 77, D)), ("bf16", (2, 1, 129, D)), ("f16", (1, 1, 33, D))):
        x = outlier_kv(shape, seed=D + bits, dtype=TORCH_DT[dn])
        _roundtrip_against_oracle(pkg, oracle, comp, Pi, cent, bits, x, f"d{D} b{bits} {dn}", max_frac=2.5e-4 if bits > 4 else None)
    # a store with room for 50 tokens per row, filled from token 3 on
    B, H, S, cap = 2, 2, 21, 50
    G = -(-D // (8 // bits))
    x = outlier_kv((B, H, S, D), seed=9, dtype=torch.bfloat16).to(DEV)
    plain = comp.compress(x)
    idx = torch.zeros((B, H, cap, G), dtype=torch.uint8, device=DEV)
    nrm = torch.zeros((B, H, cap), dtype=torch.float16, device=DEV)
    comp.compress_into(x, idx[:, :, 3:3 + S], nrm[:, :, 3:3 + S])
    assert torch.equal(idx[:, :, 3:3 + S], plain["idx_bytes"]) and torch.equal(nrm[:, :, 3:3 + S], plain["vec_norms"])
    assert not idx[:, :, :3].any() and not idx[:, :, 3 + S:].any()
    big = torch.full((B, H, cap, D), 7.0, dtype=torch.bfloat16, device=DEV)
    comp.decompress_into({"idx_bytes": idx[:, :, 3:3 + S], "vec_norms": nrm[:, :, 3:3 + S], "shape": (B, H, S, D), "idx_pad": plain["idx_pad"]},
                         big[:, :, 5:5 + S])
    direct = torch.empty((B, H, S, D), dtype=torch.bfloat16, device=DEV)
    comp.decompress_into(plain, direct)
    assert torch.equal(big[:, :, 5:5 + S], direct)
    assert (big[:, :, :5] == 7.0).all() and (big[:, :, 5 + S:] == 7.0).all()       # nothing written past a vector's end
    # several tensors in one launch
    native = pkg._native
    xs = [outlier_kv((1, 2, 40 + 3 * i, D), seed=20 + i, dtype=torch.float16).to(DEV) for i in range(3)]
    jobs = [{"states": t, "idx_bytes": torch.zeros((1, 2, t.shape[2], G), dtype=torch.uint8, device=DEV),
             "vec_norms": torch.zeros((1, 2, t.shape[2]), dtype=torch.float16, device=DEV), "table": comp.table(DEV), "bits": bits} for t in xs]
    native.JobList(jobs, torch.device(DEV)).compress()
    for t, j in zip(xs, jobs):
        one = comp.compress(t)
        assert torch.equal(j["idx_bytes"], one["idx_bytes"]) and torch.equal(j["vec_norms"], one["vec_norms"])


def test_edge_inputs(pkg, oracle):
    """Empty input, a single vector, the all-zero vector, a one-hot vector, a norm that overflows fp16."""
    D, bits = 64, 4
    comp = pkg.MSECompressor(D, bits, seed=42, device=DEV)
    empty = comp.compress(torch.empty((1, 2, 0, D), device=DEV))
    assert empty["idx_bytes"].shape == (1, 2, 0, D // 2) and empty["vec_norms"].shape == (1, 2, 0)
    assert comp.decompress(empty).shape == (1, 2, 0, D)
    x = torch.zeros((1, 1, 4, D))
    x[0, 0, 1, 5] = 3.0
    x[0, 0, 2] = torch.randn(D) * 3e4      # norm about 2.4e5: infinite in fp16
    x[0, 0, 3] = torch.randn(D) * 1e-3
    out = comp.compress(x.to(DEV))
    ref = oracle.COracle(comp.Pi.cpu().numpy(), comp.centroids.cpu().numpy(), bits, accum_double=True).compress(x.numpy().reshape(-1, D))
    check_norms(oracle, bits16(out["vec_norms"]), ref["vec_norms"], "edge")
    rec = comp.decompress(out).cpu().numpy().reshape(-1, D)
    assert not rec[0].any()                                   # zero vector -> exact zeros
    assert np.isinf(out["vec_norms"].float().cpu().numpy().reshape(-1)[2]) and not np.isfinite(rec[2]).any()
    want = oracle.NumpyOracle(comp.Pi.cpu().numpy(), comp.centroids.cpu().numpy(), bits).decompress(
        out["idx_bytes"].cpu().numpy().reshape(-1, D // 2), bits16(out["vec_norms"]).reshape(-1))
    for i in (1, 3):
        assert np.linalg.norm(rec[i] - want[i]) <= REL_L2 * np.linalg.norm(want[i]), i
    one = comp.compress(x[:, :, 1:2].to(DEV))
    assert torch.equal(one["idx_bytes"], out["idx_bytes"][:, :, 1:2])


@pytest.mark.parametrize("D", [256, 96, 192, 32])
def test_strided_store_and_batched_jobs(pkg, oracle, D):
    """Token-axis slices of a preallocated [B,H,capacity,..] store, and a job list of several tensors in one launch,
    give the bytes of plain calls (256: the kernels of that width; 96, 192: the kernels templated on the dimension; 32:
    the run-time-dimension kernels)."""
    native = pkg._native
    bits = 2
    comp = pkg.MSECompressor(D, bits, seed=3, device=DEV)
    B, H, cap = 2, 2, 300
    x = outlier_kv((B, H, 140, D), seed=5, dtype=torch.bfloat16).to(DEV)
    plain = comp.compress(x)
    idx = torch.zeros((B, H, cap, D // 4), dtype=torch.uint8, device=DEV)
    nrm = torch.zeros((B, H, cap), dtype=torch.float16, device=DEV)
    comp.compress_into(x[:, :, :100], idx[:, :, 7:107], nrm[:, :, 7:107])
    comp.compress_into(x[:, :, 100:], idx[:, :, 107:147], nrm[:, :, 107:147])
    assert torch.equal(idx[:, :, 7:147], plain["idx_bytes"]) and torch.equal(nrm[:, :, 7:147], plain["vec_norms"])
    assert not idx[:, :, :7].any() and not idx[:, :, 147:].any()
    full = torch.zeros((B, H, 200, D), dtype=torch.bfloat16, device=DEV)
    comp.decompress_packed(idx[:, :, 7:147], nrm[:, :, 7:147], full[:, :, 20:160])
    assert torch.equal(full[:, :, 20:160], comp.decompress_into(plain, torch.empty_like(x)))
    assert not full[:, :, :20].any() and not full[:, :, 160:].any()

    jobs = []
    for k, tokens in enumerate((64, 1, 257)):
        t = outlier_kv((1, 2, tokens, D), seed=20 + k, dtype=torch.bfloat16).to(DEV)
        jobs.append({"states": t, "idx_bytes": torch.empty((1, 2, tokens, D // 4), dtype=torch.uint8, device=DEV),
                     "vec_norms": torch.empty((1, 2, tokens), dtype=torch.float16, device=DEV), "table": comp.table(),
                     "bits": bits, "out": torch.empty_like(t)})
    native.JobList(jobs, torch.device(DEV)).compress()
    native.JobList([dict(j, states=j["out"]) for j in jobs], torch.device(DEV)).decompress()
    for j in jobs:
        single = comp.compress(j["states"])
        assert torch.equal(j["idx_bytes"], single["idx_bytes"]) and torch.equal(j["vec_norms"], single["vec_norms"])
        assert torch.equal(j["out"], comp.decompress_into(single, torch.empty_like(j["states"])))
    with pytest.raises(native.TqError):
        native.JobList([jobs[0], dict(jobs[0], states=torch.empty((1, 2, 64, 128), dtype=torch.bfloat16, device=DEV))], torch.device(DEV))


def test_v3_orchestration_and_cache_at_head_dim_64(pkg, oracle):
    """TurboQuantV3 and the streaming cache at head_dim 64 (compress_kv / decompress_kv / update / attend)."""
    D = 64
    tq = pkg.TurboQuantV3(D, key_bits=4, value_bits=2, residual_window=0, layer_idx=5, n_layers=12, protected_layers=2, device=DEV)
    k = outlier_kv((1, 2, 200, D), seed=1, dtype=torch.float16).to(DEV)
    v = outlier_kv((1, 2, 200, D), seed=2, dtype=torch.float16).to(DEV)
    ck, cv = tq.compress_kv(k, v)
    dk, dv = tq.decompress_kv(ck, cv)
    assert dk.shape == k.shape and dv.shape == v.shape
    cos = torch.nn.functional.cosine_similarity(dk.float().flatten(), k.float().flatten(), dim=0)
    assert cos > 0.99
    cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=16, n_layers=12)
    fk, fv = cache.update(k[:, :, :150], v[:, :, :150], 5)
    for t in range(150, 160):
        fk, fv = cache.update(k[:, :, t:t + 1], v[:, :, t:t + 1], 5)
    assert fk.shape == (1, 2, 160, D)
    assert torch.equal(fk[:, :, -16:], k[:, :, 144:160]) and torch.equal(fv[:, :, -16:], v[:, :, 144:160])
    want = tq.key_compressor.decompress_into(tq.key_compressor.compress(k[:, :, :144]), torch.empty_like(k[:, :, :144]))
    assert torch.equal(fk[:, :, :144], want)
    q = torch.randn((1, 4, 1, D), device=DEV, dtype=torch.float16)
    got = cache.attend(q, 5)                    # other head dimensions: de-quantised history, then plain attention
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), fk.float().repeat_interleave(2, dim=1), fv.float().repeat_interleave(2, dim=1))
    assert got.shape == q.shape and float((got.float() - want).norm() / want.norm()) < 5e-3


@pytest.mark.parametrize("bits,dtype", [(4, torch.bfloat16), (2, torch.float16), (8, torch.float32), (3, torch.bfloat16)])
def test_head_dim_64_in_pairs_equals_the_one_by_one_form(pkg, oracle, bits, dtype):
    """64-wide vectors go through the 128-wide kernels two at a time (as rows rotated by diag(Pi, Pi)) whenever every
    row of the job holds an even number of tokens that lie 64 elements apart; otherwise one by one through the
    run-time-dimension kernels.  Both forms against the oracle, and against each other: the same codes (outside the
    boundary window), norms within one fp16 unit, the same de-quantised values; dense tensors, token slices of a
    preallocated store at even and odd offsets, job lists that mix both kinds."""
    native = pkg._native
    D = 64
    comp = pkg.MSECompressor(D, bits, seed=11 + bits, device=DEV)
    Pi, cent = comp.Pi.cpu().numpy(), comp.centroids.cpu().numpy()
    G = D // (8 // bits)
    B, H, S = 2, 3, 347                          # odd token count: slices decide which form runs
    x = outlier_kv((B, H, S, D), seed=40 + bits, dtype=dtype).to(DEV)
    orc = oracle.COracle(Pi, cent, bits, accum_double=True)
    ref = orc.compress(x.float().cpu().numpy().reshape(-1, D))
    ref_idx = ref["idx_bytes"].reshape(B, H, S, G)
    ref_nrm = ref["vec_norms"].reshape(B, H, S)
    ref_rot = ref["rotated"].reshape(B, H, S, D)

    def check(out_idx, out_nrm, sl, label):
        rep = oracle.code_mismatch_report(out_idx.cpu().numpy().reshape(-1, G), np.ascontiguousarray(ref_idx[:, :, sl]).reshape(-1, G),
                                          np.ascontiguousarray(ref_rot[:, :, sl]).reshape(-1, D), cent, bits, 1e-5)
        assert rep["outside_window"] == 0 and rep["differ"] <= max(4, 3e-4 * rep["coords"]), (label, rep)
        ulp = oracle.fp16_ulp_distance(bits16(out_nrm).reshape(-1), np.ascontiguousarray(ref_nrm[:, :, sl]).reshape(-1))
        assert ulp.max() <= 1, label

    even = comp.compress(x[:, :, :346])          # rows of 346 tokens, 64 apart: pairs
    odd = comp.compress(x[:, :, :345])           # 345 tokens per row: one by one
    check(even["idx_bytes"], even["vec_norms"], slice(0, 346), "pairs")
    check(odd["idx_bytes"], odd["vec_norms"], slice(0, 345), "one by one")
    whole = comp.compress(x)                     # contiguous: 2 * 3 * 347 = 2082 vectors in one row: pairs across the rows' ends
    check(whole["idx_bytes"], whole["vec_norms"], slice(0, S), "contiguous")
    same_codes = (even["idx_bytes"][:, :, :345] == odd["idx_bytes"]).all(-1)
    assert same_codes.float().mean() > 0.995
    # a preallocated store: even and odd slot offsets and capacities
    for cap, t0, n_tok in ((400, 6, 346), (401, 6, 346), (400, 7, 346), (400, 6, 345)):
        idx = torch.zeros((B, H, cap, G), dtype=torch.uint8, device=DEV)
        nrm = torch.zeros((B, H, cap), dtype=torch.float16, device=DEV)
        comp.compress_into(x[:, :, :n_tok], idx[:, :, t0:t0 + n_tok], nrm[:, :, t0:t0 + n_tok])
        check(idx[:, :, t0:t0 + n_tok], nrm[:, :, t0:t0 + n_tok], slice(0, n_tok), f"store cap {cap} at {t0}, {n_tok} tokens")
        assert not idx[:, :, :t0].any() and not idx[:, :, t0 + n_tok:].any() and not nrm[:, :, t0 + n_tok:].any()
        out = torch.zeros((B, H, cap + 3, D), dtype=torch.bfloat16 if dtype == torch.float32 else dtype, device=DEV)
        comp.decompress_packed(idx[:, :, t0:t0 + n_tok], nrm[:, :, t0:t0 + n_tok], out[:, :, t0:t0 + n_tok])
        want = oracle.NumpyOracle(Pi, cent, bits).decompress(idx[:, :, t0:t0 + n_tok].cpu().numpy().reshape(-1, G),
                                                             bits16(nrm[:, :, t0:t0 + n_tok]).reshape(-1))
        err, _ = rel_l2(out[:, :, t0:t0 + n_tok].float().cpu().numpy().reshape(-1, D), torch.from_numpy(want).to(out.dtype).float().numpy())
        assert err <= 4e-3, (cap, t0, n_tok, err)
        assert not out[:, :, :t0].any() and not out[:, :, t0 + n_tok:].any()
    # job lists: all jobs in pairs; one job that cannot be paired sends the whole launch through the one-by-one kernels
    for counts in ((64, 2, 258), (64, 1, 257)):
        jobs = []
        for k, tokens in enumerate(counts):
            t = outlier_kv((1, 2, tokens, D), seed=60 + k, dtype=dtype).to(DEV)
            jobs.append({"states": t, "idx_bytes": torch.empty((1, 2, tokens, G), dtype=torch.uint8, device=DEV),
                         "vec_norms": torch.empty((1, 2, tokens), dtype=torch.float16, device=DEV), "table": comp.table(),
                         "bits": bits, "out": torch.empty_like(t)})
        native.JobList(jobs, torch.device(DEV)).compress()
        native.JobList([dict(j, states=j["out"]) for j in jobs], torch.device(DEV)).decompress()
        for j in jobs:
            r = orc.compress(j["states"].float().cpu().numpy().reshape(-1, D))
            rep = oracle.code_mismatch_report(j["idx_bytes"].cpu().numpy().reshape(-1, G), r["idx_bytes"], r["rotated"], cent, bits, 1e-5)
            assert rep["outside_window"] == 0 and rep["differ"] <= max(4, 3e-4 * rep["coords"]), (counts, rep)
            want = oracle.NumpyOracle(Pi, cent, bits).decompress(j["idx_bytes"].cpu().numpy().reshape(-1, G), bits16(j["vec_norms"]).reshape(-1))
            err, _ = rel_l2(j["out"].float().cpu().numpy().reshape(-1, D), torch.from_numpy(want).to(j["out"].dtype).float().numpy())
            assert err <= 4e-3, (counts, err)
