"""GPU tests of the append-in-place packed store (packed_row_stride of the C ABI) and of the
streaming cache built on it, against the dense kernels, the CPU oracle and the bookkeeping of
the reference's generation-time cache (generation_test_v2.py:80-165)."""
import numpy as np
import pytest
import torch

from test_gpu_parity import DEV, bits16, outlier_kv, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a HIP device; there is no CPU fallback to test")


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_append_to_packed_store_equals_dense(pkg, bits):
    """Chunks compressed into consecutive token slots of a [B,H,capacity,G] store give the bytes of
    one dense call over the concatenated tokens; de-quantising a slice of the store gives the dense
    result; slots outside the written range stay untouched."""
    B, H, cap, D = 2, 3, 192, 128
    comp = pkg.MSECompressor(D, bits, seed=5, device=DEV)
    G = D // (8 // bits)
    x = outlier_kv((B, H, 150, D), seed=bits, dtype=torch.bfloat16).to(DEV)
    store = torch.full((B, H, cap, G), 0xEE, dtype=torch.uint8, device=DEV)
    norms = torch.full((B, H, cap), -7.0, dtype=torch.float16, device=DEV)
    pos = 3                                   # start away from slot 0: pointers are advanced, not rows
    for lo, hi in ((0, 70), (70, 71), (71, 150)):          # many tokens, a single one, a ragged rest
        n = hi - lo
        comp.compress_into(x[:, :, lo:hi], store[:, :, pos:pos + n], norms[:, :, pos:pos + n])
        pos += n
    dense = comp.compress(x)
    assert torch.equal(store[:, :, 3:153], dense["idx_bytes"])
    assert torch.equal(norms[:, :, 3:153], dense["vec_norms"])
    assert bool((store[:, :, :3] == 0xEE).all()) and bool((store[:, :, 153:] == 0xEE).all())
    assert bool((norms[:, :, :3] == -7).all()) and bool((norms[:, :, 153:] == -7).all())
    want = torch.empty(B, H, 150, D, dtype=torch.bfloat16, device=DEV)
    comp.decompress_into(dense, want)
    out = torch.zeros(B, H, 160, D, dtype=torch.bfloat16, device=DEV)
    comp.decompress_packed(store[:, :, 3:153], norms[:, :, 3:153], out[:, :, :150])
    assert torch.equal(out[:, :, :150], want) and not bool(out[:, :, 150:].any())
    # one row, one token: the smallest append
    one = torch.zeros(1, 1, 8, G, dtype=torch.uint8, device=DEV)
    onen = torch.zeros(1, 1, 8, dtype=torch.float16, device=DEV)
    comp.compress_into(x[:1, :1, 4:5], one[:, :, 6:7], onen[:, :, 6:7])
    assert torch.equal(one[0, 0, 6], dense["idx_bytes"][0, 0, 4]) and not bool(one[0, 0, :6].any())


def test_batched_jobs_with_packed_row_stride(pkg):
    native = pkg._native
    comps = [pkg.MSECompressor(128, 4, seed=100 + l, device=DEV) for l in range(3)]
    xs = [outlier_kv((2, 2, 90 + l, 128), seed=40 + l, dtype=torch.float16).to(DEV) for l in range(3)]
    stores = [torch.zeros(2, 2, 128, 64, dtype=torch.uint8, device=DEV) for _ in range(3)]
    norms = [torch.zeros(2, 2, 128, dtype=torch.float16, device=DEV) for _ in range(3)]
    jobs = [{"states": x, "idx_bytes": s[:, :, 10:10 + x.shape[2]], "vec_norms": n[:, :, 10:10 + x.shape[2]],
             "table": c.table(), "bits": 4} for x, s, n, c in zip(xs, stores, norms, comps)]
    native.JobList(jobs, DEV).compress()
    torch.cuda.synchronize()
    for x, s, n, c in zip(xs, stores, norms, comps):
        d = c.compress(x)
        assert torch.equal(s[:, :, 10:10 + x.shape[2]], d["idx_bytes"]) and torch.equal(n[:, :, 10:10 + x.shape[2]], d["vec_norms"])
        assert not bool(s[:, :, :10].any()) and not bool(s[:, :, 10 + x.shape[2]:].any())
    outs = [torch.zeros_like(x) for x in xs]
    native.JobList([dict(j, states=o) for j, o in zip(jobs, outs)], DEV).decompress()
    torch.cuda.synchronize()
    for x, o, c in zip(xs, outs, comps):
        want = torch.empty_like(x)
        c.decompress_into(c.compress(x), want)
        assert torch.equal(o, want)


@pytest.mark.parametrize("rw", [0, 16, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_v3cache_stream_equals_one_shot_codec(pkg, oracle, rw, dtype):
    """Prefill, single-token decode steps and a multi-token step through V3Cache.update.  After every
    call: length and bookkeeping as the reference's cache computes them, the uncompressed tail
    bit-identical to the incoming tokens, the de-quantised part bit-identical to one dense
    compress + decompress over the same tokens (codes do not depend on the chunking), and within
    tolerance of the CPU oracle's decode of the stored bytes."""
    B, H, D, L = 2, 2, 128, 2
    cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=rw, protected_layers=0, n_layers=L)
    steps = [150, 1, 1, 1, 7, 1, 40, 1]
    keys = [outlier_kv((B, H, sum(steps), D), seed=300 + l, dtype=dtype).to(DEV) for l in range(L)]
    vals = [outlier_kv((B, H, sum(steps), D), seed=400 + l, dtype=dtype).to(DEV) for l in range(L)]
    seen = 0
    for n_new in steps:
        for l in range(L):
            fk, fv = cache.update(keys[l][:, :, seen:seen + n_new], vals[l][:, :, seen:seen + n_new], l)
            total = seen + n_new
            n_c = total if rw == 0 else max(total - rw, 0)
            assert fk.shape == (B, H, total, D) and fv.shape == fk.shape and fk.dtype == dtype
            assert cache.get_seq_length(l) == total
            assert torch.equal(fk[:, :, n_c:], keys[l][:, :, n_c:total]), (rw, total)
            assert torch.equal(fv[:, :, n_c:], vals[l][:, :, n_c:total])
            if n_c:
                tq = cache._get_compressor(l, D, DEV)
                assert tq.residual_window == 0
                ck, cv = tq.compress_kv(keys[l][:, :, :n_c], vals[l][:, :, :n_c])
                dk, dv = tq.decompress_kv(ck, cv)
                assert torch.equal(fk[:, :, :n_c], dk) and torch.equal(fv[:, :, :n_c], dv), (rw, total)
        seen += n_new
    total = sum(steps)
    n_c = total if rw == 0 else total - rw
    assert cache.get_compression_info() == f"{n_c} compressed, {total - n_c} fp16, {total} total"
    # stored bytes decoded by the oracle
    st = cache._stores[1]
    tq = cache._get_compressor(1, D, DEV)
    for comp, idx, nrm, full in ((tq.key_compressor, st.k_idx, st.k_nrm, fk), (tq.val_compressor, st.v_idx, st.v_nrm, fv)):
        orc = oracle.COracle(comp.Pi.cpu().numpy(), comp.centroids.cpu().numpy(), comp.bits, True)
        packed = idx[:, :, :n_c].contiguous().cpu().numpy().reshape(-1, idx.shape[-1])
        ref = orc.decompress(packed, bits16(nrm[:, :, :n_c].contiguous()).reshape(-1))
        err, _ = rel_l2(full[:, :, :n_c].float().cpu().numpy().reshape(-1, D), ref)
        assert err < 5e-3, err               # bf16 / fp16 rounding of the output on top of the 1e-3 bar
    assert cache.stored_bytes() == L * B * H * (n_c * (64 + 32 + 4) + 2 * (total - n_c) * D * 2)


def test_config5_shape_decode_streaming(pkg, oracle):
    """The decode-streaming workload at its real shape, one layer: 64 sequences x 8 KV heads, 16 384 compressed +
    128 window tokens prefilled (bf16, K4/V2, residual_window=128), then three single-token decode steps.
    Everything is checked on all 512 rows against the one-shot codec on the device (bit for bit), and on a sample
    of rows (first and last sequence) against the CPU oracle: stored codes and norms, the de-quantised history
    `update` returns, and `attend` against float64 attention over the oracle-decoded cache."""
    B, H, D, S0, rw, G = 64, 8, 128, 16384, 128, 4
    from test_gpu_parity import _device_kv, check_codes, check_norms
    cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=rw, protected_layers=0, n_layers=32, capacity=S0 + 16)
    total = S0 + rw + 3
    keys = _device_kv((B, H, total, D), 5_000_000, torch.bfloat16)
    vals = _device_kv((B, H, total, D), 5_000_001, torch.bfloat16)
    layer = 0
    fk, fv = cache.update(keys[:, :, :S0 + rw], vals[:, :, :S0 + rw], layer)
    assert fk.shape == (B, H, S0 + rw, D) and cache.get_compression_info() == f"{S0} compressed, {rw} fp16, {S0 + rw} total"
    del fk, fv
    for t in range(S0 + rw, total):
        fk, fv = cache.update(keys[:, :, t:t + 1], vals[:, :, t:t + 1], layer)
        if t + 1 < total:
            del fk, fv
    n_c = total - rw
    st = cache._stores[layer]
    assert cache.get_seq_length(layer) == total and st.n_compressed == n_c == S0 + 3
    assert fk.shape == (B, H, total, D) and fk.dtype == torch.bfloat16
    # all rows: the window verbatim, the history equal to the one-shot codec over the same tokens
    assert torch.equal(fk[:, :, n_c:], keys[:, :, n_c:]) and torch.equal(fv[:, :, n_c:], vals[:, :, n_c:])
    tq = cache._get_compressor(layer, D, DEV)
    ck, cv = tq.compress_kv(keys[:, :, :n_c], vals[:, :, :n_c])
    assert torch.equal(st.k_idx[:, :, :n_c], ck["compressed"]["idx_bytes"]) and torch.equal(st.k_nrm[:, :, :n_c], ck["compressed"]["vec_norms"])
    assert torch.equal(st.v_idx[:, :, :n_c], cv["compressed"]["idx_bytes"]) and torch.equal(st.v_nrm[:, :, :n_c], cv["compressed"]["vec_norms"])
    dk, dv = tq.decompress_kv(ck, cv)
    assert torch.equal(fk[:, :, :n_c], dk) and torch.equal(fv[:, :, :n_c], dv)
    del dk, dv, ck, cv
    # the query step on all rows; sampled sequences against the oracle
    q = _device_kv((B, H * G, 1, D), 5_000_003, torch.bfloat16) * 0.05
    out = cache.attend(q, layer)
    assert out.shape == q.shape and bool(torch.isfinite(out.float()).all())
    for b in (0, B - 1):
        dec = {}
        for comp, idx, nrm, x, full, name in ((tq.key_compressor, st.k_idx, st.k_nrm, keys, fk, "K4"),
                                              (tq.val_compressor, st.v_idx, st.v_nrm, vals, fv, "V2")):
            Pi, cent = comp.Pi.cpu().numpy(), comp.centroids.cpu().numpy()
            flat = x[b, :, :n_c].float().cpu().numpy().reshape(-1, D)
            ref, _ = check_codes(oracle, idx[b, :, :n_c].contiguous().cpu().numpy(), flat, Pi, cent, comp.bits, f"config 5 seq {b} {name}")
            check_norms(oracle, bits16(nrm[b, :, :n_c].contiguous()), ref["vec_norms"], f"config 5 seq {b} {name}")
            orc = oracle.COracle(Pi, cent, comp.bits, True)
            stored = orc.decompress(idx[b, :, :n_c].contiguous().cpu().numpy().reshape(-1, idx.shape[-1]),
                                    bits16(nrm[b, :, :n_c].contiguous()).reshape(-1))
            err, _ = rel_l2(full[b, :, :n_c].float().cpu().numpy().reshape(-1, D), stored)
            assert err < 4e-3, (name, err)                 # bf16 output rounding on top of the 1e-3 bar
            dec[name] = np.concatenate([stored.reshape(H, n_c, D), x[b, :, n_c:].float().cpu().numpy()], axis=1)
        _, want = oracle.attention_decode(q[b:b + 1, :, 0].float().cpu().numpy(), dec["K4"][None], dec["V2"][None], D ** -0.5)
        got = out[b, :, 0].float().cpu().numpy()
        err = float(np.linalg.norm(got - want[0]) / np.linalg.norm(want[0]))
        print(f"[config 5] seq {b}: attend vs float64 attention over the oracle-decoded cache: {err:.2e}")
        assert err < 6e-3, err                             # bf16 output rounding of `attend`
    assert cache.stored_bytes() == B * H * (n_c * (64 + 32 + 4) + 2 * rw * D * 2)


def test_v3cache_grows_and_protects_layers(pkg):
    """Capacity doubles without losing history; protected layers store 8-bit codes for K and V."""
    cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=8, protected_layers=1, n_layers=3)
    x = outlier_kv((1, 2, 700, 128), seed=9, dtype=torch.bfloat16).to(DEV)
    out = None
    for lo in range(0, 700, 100):
        for l in range(3):
            out = cache.update(x[:, :, lo:lo + 100], x[:, :, lo:lo + 100], l)
    assert cache._stores[0].k_idx.shape[-1] == 128 and cache._stores[0].v_idx.shape[-1] == 128
    assert cache._stores[1].k_idx.shape[-1] == 64 and cache._stores[1].v_idx.shape[-1] == 32
    assert cache._stores[2].k_idx.shape[-1] == 128
    assert cache._stores[1].capacity >= 692 and cache._stores[1].n_compressed == 692
    tq = cache._get_compressor(2, 128, DEV)
    ck, cv = tq.compress_kv(x[:, :, :692], x[:, :, :692])
    dk, _ = tq.decompress_kv(ck, cv)
    assert torch.equal(out[0][:, :, :692], dk) and torch.equal(out[0][:, :, 692:], x[:, :, 692:])
    with pytest.raises(ValueError):
        cache.update(x[:, :1, :1], x[:, :1, :1], 0)          # head count changed


def test_hf_dynamic_cache_subclass(pkg):
    """The transformers-facing subclass keeps DynamicCache's interface alive around update()."""
    transformers = pytest.importorskip("transformers")
    cls = pkg.hf_cache_class()
    cache = cls(key_bits=4, value_bits=2, residual_window=4, n_layers=2)
    assert isinstance(cache, transformers.DynamicCache) and isinstance(cache, pkg.V3Cache)
    x = outlier_kv((1, 2, 12, 128), seed=1, dtype=torch.float16).to(DEV)
    for l in range(2):
        k, v = cache.update(x, x, l)
        assert k.shape == (1, 2, 12, 128)
    assert cache.get_seq_length() == 12 and cache.get_seq_length(1) == 12
    assert cache.get_compression_info() == "8 compressed, 4 fp16, 12 total"


# ---------------------------------------------------------------------------------------------
# attention straight from the packed store
# ---------------------------------------------------------------------------------------------
def _oracle_decode(oracle, comp, idx, nrm, shape):
    orc = oracle.COracle(comp.Pi.cpu().numpy(), comp.centroids.cpu().numpy(), comp.bits, True)
    flat = orc.decompress(idx.contiguous().cpu().numpy().reshape(-1, idx.shape[-1]), bits16(nrm.contiguous()).reshape(-1))
    return flat.reshape(shape)


@pytest.mark.parametrize("bits,group,S", [(4, 4, 1000), (2, 8, 333), (8, 1, 64), (3, 2, 31), (1, 16, 257), (6, 32, 96)])
def test_packed_scores_against_oracle(pkg, oracle, bits, group, S):
    """scale * q . k_hat from packed keys (query rotated once, codes never expanded to vectors) equals the
    float64 scores over the oracle's de-quantised keys; tolerance: the fp16 rounding of the centroid
    table the decode kernels share (2^-11 relative per coordinate), i.e. 1e-3 of scale*|q|*|k|."""
    B, H, D = 2, 3, 128
    comp = pkg.MSECompressor(D, bits, seed=77 + bits, device=DEV)
    keys = outlier_kv((B, H, S, D), seed=bits * 10 + group, dtype=torch.bfloat16).to(DEV)
    store = torch.zeros(B, H, S + 40, D // (8 // bits), dtype=torch.uint8, device=DEV)
    norms = torch.zeros(B, H, S + 40, dtype=torch.float16, device=DEV)
    comp.compress_into(keys, store[:, :, 7:7 + S], norms[:, :, 7:7 + S])
    g = torch.Generator(device="cpu")
    g.manual_seed(group)
    q = (torch.randn(B, H * group, 1, D, generator=g) * torch.exp(torch.randn(B, H * group, 1, 1, generator=g))).to(DEV)
    scale = D ** -0.5
    out = torch.full((B, H * group, S + 5), 123.0, dtype=torch.float32, device=DEV)
    got = comp.packed_scores(store[:, :, 7:7 + S], norms[:, :, 7:7 + S], q, scale, out=out[:, :, :S])
    assert got.data_ptr() == out.data_ptr() and bool((out[:, :, S:] == 123.0).all())
    k_hat = _oracle_decode(oracle, comp, store[:, :, 7:7 + S], norms[:, :, 7:7 + S], (B, H, S, D))
    ref, _ = oracle.attention_decode(q.squeeze(2).cpu().numpy(), k_hat, k_hat, scale)
    bound = scale * np.linalg.norm(q.squeeze(2).cpu().numpy().astype(np.float64), axis=-1)[:, :, None] \
        * np.repeat(np.linalg.norm(k_hat.astype(np.float64), axis=-1), group, axis=1)
    err = np.abs(got.cpu().numpy() - ref) / np.maximum(bound, 1e-30)
    print(f"[scores] b{bits} G{group} S{S}: max error {err.max():.2e} of scale*|q|*|k|")
    assert err.max() < 1e-3
    # and the definition the reference uses: scores over the product's own de-quantised keys
    deq = torch.empty(B, H, S, D, dtype=torch.float32, device=DEV)
    comp.decompress_packed(store[:, :, 7:7 + S], norms[:, :, 7:7 + S], deq)
    same = pkg.attention_scores(q, deq.repeat_interleave(group, dim=1)) * scale
    assert float((got - same).abs().max()) < 1e-3 * float(bound.max())
    dense = comp.packed_scores(store[:, :, 7:7 + S].contiguous(), norms[:, :, 7:7 + S].contiguous(), q.squeeze(2), scale)
    assert torch.equal(dense, got)


@pytest.mark.parametrize("bits,group,S", [(2, 4, 1000), (4, 8, 333), (8, 1, 64), (3, 2, 31), (1, 16, 257)])
def test_packed_weighted_values_against_oracle(pkg, oracle, bits, group, S):
    B, H, D = 2, 3, 128
    comp = pkg.MSECompressor(D, bits, seed=177 + bits, device=DEV)
    vals = outlier_kv((B, H, S, D), seed=bits * 10 + group + 1, dtype=torch.float16).to(DEV)
    store = torch.zeros(B, H, S + 9, D // (8 // bits), dtype=torch.uint8, device=DEV)
    norms = torch.zeros(B, H, S + 9, dtype=torch.float16, device=DEV)
    comp.compress_into(vals, store[:, :, 2:2 + S], norms[:, :, 2:2 + S])
    g = torch.Generator(device="cpu")
    g.manual_seed(S)
    w_full = torch.softmax(3 * torch.randn(B, H * group, S + 16, generator=g), dim=-1).to(DEV)
    w = w_full[:, :, :S]                                         # a strided slice, as the cache passes it
    got = comp.packed_weighted_values(store[:, :, 2:2 + S], norms[:, :, 2:2 + S], w)
    v_hat = _oracle_decode(oracle, comp, store[:, :, 2:2 + S], norms[:, :, 2:2 + S], (B, H, S, D)).astype(np.float64)
    ref = np.einsum("bhgs,bhsd->bhgd", w.cpu().numpy().astype(np.float64).reshape(B, H, group, S), v_hat).reshape(B, H * group, D)
    err = np.linalg.norm(got.cpu().numpy() - ref) / np.linalg.norm(ref)
    print(f"[weighted values] b{bits} G{group} S{S}: relative L2 error {err:.2e}")
    assert got.shape == (B, H * group, D) and err < 1e-3
    again = comp.packed_weighted_values(store[:, :, 2:2 + S], norms[:, :, 2:2 + S], w)
    assert torch.equal(again, got)                               # fixed summation order


@pytest.mark.parametrize("rw,dtype,D", [(128, torch.bfloat16, 128), (0, torch.float16, 128), (16, torch.bfloat16, 128),
                                         (16, torch.bfloat16, 64), (128, torch.float16, 256), (0, torch.bfloat16, 96),
                                         (16, torch.float16, 80), (8, torch.bfloat16, 45)])
def test_v3cache_attend_equals_attention_over_the_cache(pkg, oracle, rw, dtype, D):
    """append() leaves the cache in the state update() leaves it in, and attend() equals one-query
    attention over (oracle-decoded packed tokens ++ window) in float64; it also agrees with attention
    over the bf16 / fp16 tensors update() hands to the model within their rounding.  128-wide heads are read
    straight from the packed codes; other head dimensions are de-quantised by the codec kernels first."""
    B, H, G, L = 2, 2, 4, 2
    a = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=rw, n_layers=L)
    b = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=rw, n_layers=L)
    steps = [300, 1, 1, 5, 1] + [1] * 20
    total = sum(steps)
    keys = [outlier_kv((B, H, total, D), seed=600 + l, dtype=dtype).to(DEV) for l in range(L)]
    vals = [outlier_kv((B, H, total, D), seed=700 + l, dtype=dtype).to(DEV) for l in range(L)]
    g = torch.Generator(device="cpu")
    g.manual_seed(9)
    seen = 0
    for i, n_new in enumerate(steps):
        for l in range(L):
            fk, fv = a.update(keys[l][:, :, seen:seen + n_new], vals[l][:, :, seen:seen + n_new], l)
            b.append(keys[l][:, :, seen:seen + n_new], vals[l][:, :, seen:seen + n_new], l)
            sa, sb = a._stores[l], b._stores[l]
            assert (sa.n_compressed, sa.n_recent, sa.total_seq) == (sb.n_compressed, sb.n_recent, sb.total_seq)
            if i in (0, 3, len(steps) - 1):
                n_c = sb.n_compressed
                assert torch.equal(sa.k_idx[:, :, :n_c], sb.k_idx[:, :, :n_c]) and torch.equal(sa.v_nrm[:, :, :n_c], sb.v_nrm[:, :, :n_c])
                assert all(torch.equal(x, y) for x, y in zip(sa.window(), sb.window()))
                q = (4 * torch.randn(B, H * G, 1, D, generator=g)).to(dtype).to(DEV)
                out = b.attend(q, l)
                assert out.shape == (B, H * G, 1, D) and out.dtype == dtype
                three = b.attend(q, l, fused=False)              # scores / softmax / weighted values as separate steps
                assert float((out.float() - three.float()).norm() / three.float().norm()) < 4e-3
                tq = b._get_compressor(l, D, DEV)
                kw, vw = sb.window()
                parts_k, parts_v = [], []
                if n_c:
                    parts_k.append(_oracle_decode(oracle, tq.key_compressor, sb.k_idx[:, :, :n_c], sb.k_nrm[:, :, :n_c], (B, H, n_c, D)))
                    parts_v.append(_oracle_decode(oracle, tq.val_compressor, sb.v_idx[:, :, :n_c], sb.v_nrm[:, :, :n_c], (B, H, n_c, D)))
                parts_k.append(kw.float().cpu().numpy())
                parts_v.append(vw.float().cpu().numpy())
                _, ref = oracle.attention_decode(q.squeeze(2).float().cpu().numpy(), np.concatenate(parts_k, 2),
                                                 np.concatenate(parts_v, 2), D ** -0.5)
                got = out.squeeze(2).float().cpu().numpy()
                err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
                # what the model would compute from update()'s tensors
                model = torch.nn.functional.scaled_dot_product_attention(
                    q.float(), fk.float().repeat_interleave(G, dim=1), fv.float().repeat_interleave(G, dim=1)).squeeze(2)
                err_model = float((out.squeeze(2).float() - model).norm() / model.norm())
                print(f"[attend] rw={rw} step {i} layer {l}: vs oracle {err:.2e}, vs attention over update() tensors {err_model:.2e}")
                # output rounded to bf16 / fp16: 2^-9 / 2^-11.  (The tensors update() returns are rounded to 16 bits; with 64-wide
                # heads the softmax scale is 1/8 and the same rounding of a key moves a weight further.)
                assert err < 6e-3 and err_model < (2e-2 if D >= 128 else 4e-2)
        seen += n_new
    with pytest.raises(ValueError):
        b.attend(torch.zeros(B, H * G, 2, D, device=DEV), 0)


@pytest.mark.parametrize("kb,vb,G,S", [(4, 2, 4, 1500), (8, 8, 8, 200), (2, 4, 1, 77), (3, 1, 2, 640), (6, 2, 8, 33), (4, 2, 16, 900), (8, 4, 13, 150)])
def test_fused_attention_partials_against_oracle(pkg, oracle, kb, vb, G, S):
    """The one-pass kernel (scores, online softmax, weighted values per split) merged by the log-sum-exp rule
    equals float64 attention over the oracle-decoded packed keys and values; its records are consistent
    (reference score within the documented distance of the largest score, sums taken against it)."""
    B, H, D = 2, 3, 128
    kc = pkg.MSECompressor(D, kb, seed=11 + kb, device=DEV)
    vc = pkg.MSECompressor(D, vb, seed=511 + vb, device=DEV)
    keys = outlier_kv((B, H, S, D), seed=kb * 100 + S, dtype=torch.bfloat16).to(DEV)
    vals = outlier_kv((B, H, S, D), seed=vb * 100 + S + 1, dtype=torch.bfloat16).to(DEV)
    cap = S + 24
    k_idx = torch.zeros(B, H, cap, D // (8 // kb), dtype=torch.uint8, device=DEV)
    v_idx = torch.zeros(B, H, cap, D // (8 // vb), dtype=torch.uint8, device=DEV)
    k_nrm = torch.zeros(B, H, cap, dtype=torch.float16, device=DEV)
    v_nrm = torch.zeros(B, H, cap, dtype=torch.float16, device=DEV)
    kc.compress_into(keys, k_idx[:, :, :S], k_nrm[:, :, :S])
    vc.compress_into(vals, v_idx[:, :, :S], v_nrm[:, :, :S])
    g = torch.Generator(device="cpu")
    g.manual_seed(S)
    q = (3 * torch.randn(B, H * G, D, generator=g) * torch.exp(0.5 * torch.randn(B, H * G, 1, generator=g))).to(DEV)
    q[0, 0] = 0                                              # a zero query: uniform attention
    scale = D ** -0.5
    q_rot = torch.matmul(q, kc.Pi.T) * scale
    part = torch.ops.tqamd.attend_partials(k_idx[:, :, :S], k_nrm[:, :, :S], v_idx[:, :, :S], v_nrm[:, :, :S],
                                           kc.table(), vc.table(), kb, vb, q_rot)
    assert part.shape[:2] == (B, H * G) and part.shape[3] == D + 2
    m_s, l_s, a_s = part[..., 0], part[..., 1], part[..., 2:]
    m_all = m_s.amax(dim=-1, keepdim=True)
    f = torch.exp(m_s - m_all)
    got = (torch.matmul((f.unsqueeze(-1) * a_s).sum(2), vc.Pi) / (f * l_s).sum(-1, keepdim=True)).cpu().numpy()
    k_hat = _oracle_decode(oracle, kc, k_idx[:, :, :S], k_nrm[:, :, :S], (B, H, S, D))
    v_hat = _oracle_decode(oracle, vc, v_idx[:, :, :S], v_nrm[:, :, :S], (B, H, S, D))
    ref_scores, ref = oracle.attention_decode(q.cpu().numpy(), k_hat, v_hat, scale)
    err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
    # the record's reference score is at most the largest score and at most 8 binary orders below it ...
    gap = ref_scores.max(-1) - m_all.squeeze(-1).cpu().numpy()
    tol = 1e-3 * np.abs(ref_scores).max() + 1e-6
    assert gap.min() > -tol and gap.max() < 8 * np.log(2.0) + tol
    # ... and the sum of exponentials is taken against exactly that reference
    l_got = (f * l_s).sum(-1).cpu().numpy()
    l_ref = np.exp(ref_scores - m_all.cpu().numpy().astype(np.float64)).sum(-1)
    # (a score error ds changes exp(score) by the factor e^ds: fp16 keys and queries put ds near 1e-4 of the largest |score|)
    assert np.abs(l_got / l_ref - 1).max() < 3e-3 + 4e-4 * np.abs(ref_scores).max()
    print(f"[fused attention] K{kb} V{vb} G{G} S{S}: relative L2 error {err:.2e}")
    # queries and decoded keys enter the score product as fp16 (2^-12 relative per coordinate), probabilities times
    # value norms as fp16 as well; the queries here are scaled up to logits beyond 100, where that shows most
    assert err < 3e-3


def test_attend_with_window_only_and_without_window(pkg, oracle):
    """Decode-step attention when nothing is compressed yet (window tokens only) and when there is no window."""
    B, H, G, D = 2, 2, 4, 128
    for rw, n in ((128, 50), (0, 90)):
        cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=rw, n_layers=1)
        k = outlier_kv((B, H, n, D), seed=800 + rw, dtype=torch.bfloat16).to(DEV)
        v = outlier_kv((B, H, n, D), seed=801 + rw, dtype=torch.bfloat16).to(DEV)
        fk, fv = cache.update(k, v, 0)
        g = torch.Generator(device="cpu")
        g.manual_seed(rw)
        q = (2 * torch.randn(B, H * G, 1, D, generator=g)).to(torch.bfloat16).to(DEV)
        out = cache.attend(q, 0)
        ref = torch.nn.functional.scaled_dot_product_attention(
            q.float(), fk.float().repeat_interleave(G, dim=1), fv.float().repeat_interleave(G, dim=1))
        err = float((out.float() - ref).norm() / ref.norm())
        print(f"[attend] rw={rw}, {n} tokens: vs attention over update() tensors {err:.2e}")
        assert out.shape == q.shape and err < (4e-3 if rw else 2e-2)
        assert float((out.float() - cache.attend(q, 0, fused=False).float()).norm() / ref.norm()) < 4e-3


@pytest.mark.parametrize("wdtype,qdtype,G,W,splits", [(torch.bfloat16, torch.bfloat16, 4, 128, 3), (torch.float16, torch.float16, 8, 512, 1),
                                                      (torch.float32, torch.float32, 1, 37, 2), (torch.bfloat16, torch.float32, 7, 1, 0),
                                                      (torch.float16, torch.bfloat16, 3, 0, 4), (torch.bfloat16, torch.bfloat16, 16, 300, 2), (torch.float32, torch.float16, 11, 70, 1)])
@pytest.mark.parametrize("B", [2, 50])       # 6 rows: one merge block per (row, head); 150 rows: one per row, all heads
def test_attend_prepare_and_merge_against_float64(pkg, wdtype, qdtype, G, W, splits, B):
    """tq_attend_prepare / tq_attend_merge through the C-ABI against the same arithmetic in float64:
    rotated queries to 1e-5, window records to 1e-5, merged output to the output type's rounding."""
    nat = pkg._native
    L = nat.lib()
    H, D, cap = 3, 128, 520
    rows = B * H
    g = torch.Generator(device="cpu")
    g.manual_seed(1000 + G * 7 + W + B)
    q = (3 * torch.randn(B, H * G, 1, D, generator=g)).to(qdtype).to(DEV)
    kbuf = torch.randn(B, H, cap, D, generator=g).to(wdtype).to(DEV)
    vbuf = torch.randn(B, H, cap, D, generator=g).to(wdtype).to(DEV)
    kw, vw = kbuf[:, :, 8:8 + W], vbuf[:, :, 8:8 + W]                # token-axis slices of a larger buffer
    pi_k = pkg.generate_rotation_matrix(D, seed=11).contiguous().to(DEV)
    pi_v = pkg.generate_rotation_matrix(D, seed=12).contiguous().to(DEV)
    scale = 0.11
    q_rot = torch.empty(B, H * G, D, dtype=torch.float32, device=DEV)
    part_w = torch.full((rows, G, D + 2), float("nan"), dtype=torch.float32, device=DEV)
    rc = L.tq_attend_prepare(q.data_ptr(), nat.dtype_code(q.dtype), rows, G, scale, pi_k.t().contiguous().data_ptr(),
                             kw.data_ptr() if W else None, vw.data_ptr() if W else None, nat.dtype_code(wdtype), W, cap * D,
                             q_rot.data_ptr(), part_w.data_ptr() if W else None, None)
    assert rc == 0
    torch.cuda.synchronize()
    q64 = q.double().reshape(B, H, G, D) * scale
    ref_rot = torch.matmul(q64, pi_k.double().T).reshape(B, H * G, D)
    assert float((q_rot.double() - ref_rot).norm() / ref_rot.norm()) < 1e-5
    if W:
        s = torch.matmul(q64, kw.double().transpose(-2, -1))
        m = s.amax(-1)
        p = torch.exp(s - m.unsqueeze(-1))
        l = p.sum(-1)
        a = torch.matmul(p, vw.double())
        pw = part_w.double().reshape(B, H, G, D + 2)
        assert float((pw[..., 0] - m).abs().max()) < 1e-4 and float(((pw[..., 1] - l) / l).abs().max()) < 1e-5
        assert float(((pw[..., 2:] - a).norm(dim=-1) / a.norm(dim=-1)).max()) < 1e-5
    # split records as the one-pass kernel would leave them: random maxima, sums, rotated value sums
    part = None
    if splits:
        part = torch.randn(rows, splits, G, D + 2, generator=g).to(DEV)
        part[..., 0] = part[..., 0] * 3 + (float(m.mean()) if W else 0.0)
        part[..., 1] = part[..., 1].abs() + 0.5
    for odtype in (torch.float32, qdtype):
        out = torch.empty(B, H * G, 1, D, dtype=odtype, device=DEV)
        rc = L.tq_attend_merge(part.data_ptr() if splits else None, splits, part_w.data_ptr() if W else None, pi_v.data_ptr(),
                               rows, G, out.data_ptr(), nat.dtype_code(odtype), None)
        assert rc == 0
        torch.cuda.synchronize()
        m_all = torch.full((rows, G), -float("inf"), dtype=torch.float64, device=DEV)
        if splits:
            p64 = part.double()
            m_all = torch.maximum(m_all, p64[..., 0].amax(dim=1))
        if W:
            w64 = part_w.double()
            m_all = torch.maximum(m_all, w64[..., 0])
        num = torch.zeros(rows, G, D, dtype=torch.float64, device=DEV)
        den = torch.zeros(rows, G, dtype=torch.float64, device=DEV)
        if splits:
            f = torch.exp(p64[..., 0] - m_all.unsqueeze(1))
            num = torch.matmul((f.unsqueeze(-1) * p64[..., 2:]).sum(1), pi_v.double())
            den = (f * p64[..., 1]).sum(1)
        if W:
            f = torch.exp(w64[..., 0] - m_all)
            num = num + f.unsqueeze(-1) * w64[..., 2:]
            den = den + f * w64[..., 1]
        ref = (num / den.unsqueeze(-1)).reshape(B, H * G, 1, D)
        err = float((out.double() - ref).norm() / ref.norm())
        tol = {torch.float32: 1e-5, torch.float16: 1e-3, torch.bfloat16: 6e-3}[odtype]
        print(f"[prepare/merge] window {W} x {wdtype}, {G} heads, {splits} splits -> {odtype}: {err:.2e}")
        assert err < tol


def test_hf_model_runs_on_the_cache(pkg):
    """A small randomly initialised Llama (transformers, no download) runs prefill + decode and `generate` with the
    cache as `past_key_values`, the way generation_test_v2.py:178-201 drives the reference's cache.  With 8-bit keys
    and values the logits stay close to those of the stock DynamicCache; with K4/V2 the run completes and the cache
    holds what the model fed it."""
    transformers = pytest.importorskip("transformers")
    from transformers import DynamicCache, LlamaConfig, LlamaForCausalLM
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=256, hidden_size=512, intermediate_size=1024, num_hidden_layers=3, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=128, max_position_embeddings=512)
    model = LlamaForCausalLM(cfg).to(DEV, dtype=torch.bfloat16).eval()
    cls = pkg.hf_cache_class()
    ids = torch.randint(0, 256, (2, 40), device=DEV)
    mask = torch.ones_like(ids)
    with torch.no_grad():
        cache = cls(key_bits=8, value_bits=8, residual_window=8, n_layers=3)
        ref_cache = DynamicCache()
        out = model(ids, attention_mask=mask, past_key_values=cache, use_cache=True)
        ref = model(ids, attention_mask=mask, past_key_values=ref_cache, use_cache=True)
        # prefill attends over what update() returned: the de-quantised prompt (all but the window)
        rel = float((out.logits.float() - ref.logits.float()).norm() / ref.logits.float().norm())
        print(f"[hf] prefill logits, 8-bit cache vs DynamicCache: {rel:.2e}")
        assert rel < 3e-2
        for step in range(6):
            nxt = torch.randint(0, 256, (2, 1), device=DEV)
            mask = torch.cat([mask, torch.ones_like(nxt)], dim=1)
            out = model(nxt, attention_mask=mask, past_key_values=cache, use_cache=True)
            ref = model(nxt, attention_mask=mask, past_key_values=ref_cache, use_cache=True)
            rel = float((out.logits.float() - ref.logits.float()).norm() / ref.logits.float().norm())
            assert rel < 3e-2, (step, rel)
        print(f"[hf] decode step logits, 8-bit cache vs DynamicCache: {rel:.2e}")
        assert cache.get_seq_length() == 46 and ref_cache.get_seq_length() == 46
        assert cache.get_compression_info() == "38 compressed, 8 fp16, 46 total"
        small = cls(key_bits=4, value_bits=2, residual_window=16, n_layers=3)
        gen = model.generate(ids, attention_mask=torch.ones_like(ids), past_key_values=small, max_new_tokens=12, do_sample=False)
        assert gen.shape == (2, 52) and torch.equal(gen[:, :40], ids)
        assert small.get_seq_length() == 51            # the last generated token has not been fed back
        assert small.get_compression_info() == "35 compressed, 16 fp16, 51 total"
        assert sorted(small._stores) == [0, 1, 2]


def test_hf_model_decodes_through_packed_attention(pkg):
    """The same small Llama with the registered attention function: decode steps are answered from the packed
    store (`attend`) and never de-quantise the history.  Same tokens fed to both, the logits equal those of the
    ordinary `update` path of an identically configured cache up to rounding; `generate` runs on it."""
    transformers = pytest.importorskip("transformers")
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=256, hidden_size=512, intermediate_size=1024, num_hidden_layers=3, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=128, max_position_embeddings=512)
    model = LlamaForCausalLM(cfg).to(DEV, dtype=torch.bfloat16).eval()
    name = pkg.register_packed_attention()
    cls = pkg.hf_cache_class()
    ids = torch.randint(0, 256, (2, 70), device=DEV)
    steps = [torch.randint(0, 256, (2, 1), device=DEV) for _ in range(8)]
    logits = {}
    with torch.no_grad():
        for packed in (False, True):
            model.config._attn_implementation = name if packed else "sdpa"
            cache = cls(key_bits=4, value_bits=2, residual_window=16, n_layers=3, packed_attention=packed)
            mask = torch.ones_like(ids)
            out = [model(ids, attention_mask=mask, past_key_values=cache, use_cache=True).logits[:, -1:].float()]
            for nxt in steps:
                mask = torch.cat([mask, torch.ones_like(nxt)], dim=1)
                out.append(model(nxt, attention_mask=mask, past_key_values=cache, use_cache=True).logits.float())
            logits[packed] = torch.cat(out, dim=1)
            assert cache.get_seq_length() == 78 and cache.get_compression_info() == "62 compressed, 16 fp16, 78 total"
        a, b = logits[False], logits[True]
        assert torch.equal(a[:, 0], b[:, 0])                       # prefill takes the same path in both
        rel = float((a[:, 1:] - b[:, 1:]).norm() / a[:, 1:].norm())
        print(f"[hf] decode logits, packed attention vs update path (K4/V2): {rel:.2e}")
        assert rel < 2e-2
        model.config._attn_implementation = name
        cache = cls(key_bits=4, value_bits=2, residual_window=16, n_layers=3, packed_attention=True)
        gen = model.generate(ids, attention_mask=torch.ones_like(ids), past_key_values=cache, max_new_tokens=10, do_sample=False)
        assert gen.shape == (2, 80) and cache.get_seq_length() == 79
        # a padded batch is refused in that mode: attention from the packed store counts every cached token
        cache = cls(key_bits=4, value_bits=2, residual_window=16, n_layers=3, packed_attention=True)
        mask = torch.ones_like(ids)
        model(ids, attention_mask=mask, past_key_values=cache, use_cache=True)
        mask = torch.cat([mask, torch.ones_like(steps[0])], dim=1)
        mask[1, :3] = 0
        with pytest.raises(RuntimeError, match="hides cached tokens"):
            model(steps[0], attention_mask=mask, past_key_values=cache, use_cache=True)
        # a cache in packed mode under a model whose attention is not the registered function: the step of layer 0
        # would be attention over one token; the next call on the cache says so instead
        model.config._attn_implementation = "sdpa"
        cache = cls(key_bits=4, value_bits=2, residual_window=16, n_layers=3, packed_attention=True)
        mask = torch.ones_like(ids)
        model(ids, attention_mask=mask, past_key_values=cache, use_cache=True)
        mask = torch.cat([mask, torch.ones_like(steps[0])], dim=1)
        with pytest.raises(RuntimeError, match="never answered"):
            model(steps[0], attention_mask=mask, past_key_values=cache, use_cache=True)


def test_fused_attention_over_extreme_value_norms(pkg, oracle):
    """Value norms spanning twelve decimal orders inside one history (tiny, ordinary, huge, exactly zero) and keys
    with zero vectors: the kernel scales value norms relative to the largest one it has seen, so the result follows
    float64 attention over the oracle-decoded cache wherever the huge-norm tokens carry weight, and rows whose
    values are all tiny or all zero come out tiny or zero, never NaN."""
    B, H, G, S, D = 1, 4, 4, 700, 128
    kc = pkg.MSECompressor(D, 4, seed=21, device=DEV)
    vc = pkg.MSECompressor(D, 2, seed=521, device=DEV)
    g = torch.Generator(device="cpu")
    g.manual_seed(77)
    keys = torch.randn(B, H, S, D, generator=g)
    vals = torch.randn(B, H, S, D, generator=g)
    vals[:, 0] *= 1e-6                                   # a row of tiny values
    vals[:, 1, :300] *= 1e-6                             # tiny first, then huge: the reference exponent has to move
    vals[:, 1, 300:] *= 3e3
    vals[:, 2] = 0                                       # all zero
    vals[:, 3, ::7] *= 3e3                               # mixed within every run (norms stay below the fp16 limit of 65504)
    keys[:, 3, 100:140] = 0                              # zero keys score 0
    keys, vals = keys.to(torch.bfloat16).to(DEV), vals.to(torch.bfloat16).to(DEV)
    ck, cv = kc.compress(keys), vc.compress(vals)
    k_idx, k_nrm = ck["idx_bytes"].reshape(B, H, S, -1), ck["vec_norms"].reshape(B, H, S)
    v_idx, v_nrm = cv["idx_bytes"].reshape(B, H, S, -1), cv["vec_norms"].reshape(B, H, S)
    q = torch.randn(B, H * G, D, generator=g).to(DEV)
    scale = D ** -0.5
    q_rot = torch.matmul(q, kc.Pi.T) * scale
    part = torch.ops.tqamd.attend_partials(k_idx, k_nrm, v_idx, v_nrm, kc.table(), vc.table(), 4, 2, q_rot)
    assert bool(torch.isfinite(part).all())
    m_s, l_s, a_s = part[..., 0], part[..., 1], part[..., 2:]
    f = torch.exp(m_s - m_s.amax(dim=-1, keepdim=True))
    got = (torch.matmul((f.unsqueeze(-1) * a_s).sum(2), vc.Pi) / (f * l_s).sum(-1, keepdim=True)).cpu().numpy()
    k_hat = _oracle_decode(oracle, kc, k_idx, k_nrm, (B, H, S, D))
    v_hat = _oracle_decode(oracle, vc, v_idx, v_nrm, (B, H, S, D))
    _, ref = oracle.attention_decode(q.cpu().numpy(), k_hat, v_hat, scale)
    got, ref = got.reshape(H, G, D), ref.reshape(H, G, D)
    for h in (0, 1, 3):
        err = np.linalg.norm(got[h] - ref[h]) / np.linalg.norm(ref[h])
        print(f"[fused attention] value-norm case {h}: relative L2 error {err:.2e}, |out| = {np.linalg.norm(ref[h]):.2e}")
        assert err < 3e-3
    assert np.all(got[2] == 0) and np.all(ref[2] == 0)


def test_attend_with_sixteen_query_heads_per_kv_head(pkg, oracle):
    """The widest group the one-pass path takes (128 query heads over 8 kv heads): same result as the three-step
    form and as attention over the tensors update() returns."""
    B, H, G, D = 1, 2, 16, 128
    a = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=32, n_layers=1)
    b = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=32, n_layers=1)
    k = outlier_kv((B, H, 700, D), seed=900, dtype=torch.bfloat16).to(DEV)
    v = outlier_kv((B, H, 700, D), seed=901, dtype=torch.bfloat16).to(DEV)
    fk, fv = a.update(k, v, 0)
    b.append(k, v, 0)
    g = torch.Generator(device="cpu")
    g.manual_seed(16)
    q = (2 * torch.randn(B, H * G, 1, D, generator=g)).to(torch.bfloat16).to(DEV)
    out = b.attend(q, 0)
    three = b.attend(q, 0, fused=False)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.float(), fk.float().repeat_interleave(G, dim=1), fv.float().repeat_interleave(G, dim=1))
    e1 = float((out.float() - three.float()).norm() / three.float().norm())
    e2 = float((out.float() - ref).norm() / ref.norm())
    print(f"[attend] 16 heads per kv head: vs three-step {e1:.2e}, vs attention over update() tensors {e2:.2e}")
    assert e1 < 4e-3 and e2 < 1.5e-2


@pytest.mark.parametrize("dtype,layout", [(torch.bfloat16, "bhsd"), (torch.float16, "bshd"), (torch.float32, "bhsd")])
def test_single_call_decode_step_equals_the_general_path(pkg, dtype, layout):
    """Steady-state decode steps go through tq_append_token / tq_attend_step (one library call each).  Two
    caches fed the same tokens, one of them forced onto the general path, must hold the same bytes after every
    step and give the same attention output; the run crosses several compactions of the window buffer and a
    growth of the packed store."""
    kvc = pkg.kv_cache
    B, H, G, D, rw = 2, 3, 4, 128, 16
    fast = pkg.V3Cache(4, 2, residual_window=rw, n_layers=4)
    slow = pkg.V3Cache(4, 2, residual_window=rw, n_layers=4)
    g = torch.Generator().manual_seed(5)

    def tokens(n):
        if layout == "bshd":                      # what a model's projections give: [B,S,H,D] storage
            return (torch.randn(B, n, H, D, generator=g) * 1.5).to(dtype).to(DEV).transpose(1, 2)
        return (torch.randn(B, H, n, D, generator=g) * 1.5).to(dtype).to(DEV)

    calls = {"append": 0, "attend": 0}
    real_append, real_attend = kvc._LayerStore.append_one, kvc.V3Cache._attend_step

    def counted_append(self, k, v):
        done = real_append(self, k, v)
        calls["append"] += bool(done)
        return done

    def counted_attend(st, q, G_, scale):
        out = real_attend(st, q, G_, scale)
        calls["attend"] += out is not None
        return out

    k0, v0 = tokens(40), tokens(40)
    for c in (fast, slow):
        c.append(k0, v0, 1)
    steps = 300
    for i in range(steps):
        k, v = tokens(1), tokens(1)
        q = (torch.randn(B, H * G, 1, D, generator=g)).to(dtype).to(DEV)
        kvc._LayerStore.append_one, kvc.V3Cache._attend_step = counted_append, staticmethod(counted_attend)
        try:
            fast.append(k, v, 1)
            a = fast.attend(q, 1)
        finally:
            kvc._LayerStore.append_one, kvc.V3Cache._attend_step = real_append, staticmethod(real_attend)
        kvc._LayerStore.append_one = lambda self, k_, v_: False
        kvc.V3Cache._attend_step = staticmethod(lambda st, q_, G_, s_: None)
        try:
            slow.append(k, v, 1)
            b = slow.attend(q, 1)
        finally:
            kvc._LayerStore.append_one, kvc.V3Cache._attend_step = real_append, staticmethod(real_attend)
        assert torch.equal(a, b), i
    sf, ss = fast._stores[1], slow._stores[1]
    assert (sf.n_compressed, sf.n_recent, sf.total_seq) == (ss.n_compressed, ss.n_recent, ss.total_seq) == (40 + steps - rw, rw, 40 + steps)
    n = sf.n_compressed
    for name in ("k_idx", "k_nrm", "v_idx", "v_nrm"):
        assert torch.equal(getattr(sf, name)[:, :, :n], getattr(ss, name)[:, :, :n]), name
    for x, y in zip(sf.window(), ss.window()):
        assert torch.equal(x, y)
    # the single-call path really ran: every step attends through it, and every append except those that
    # first have to move the window back to the front of its buffer or to grow the packed store
    assert calls["attend"] == steps and calls["append"] >= steps - steps // rw - 6, calls


def test_append_token_and_attend_step_through_the_c_abi(pkg, oracle):
    """The two per-step entry points called by hand: the evicted window token lands in the packed slot with the
    bytes tq_compress gives, the new token in the window slot, and tq_attend_step returns what the three
    separate calls return."""
    nat = pkg._native
    L = nat.lib()
    rows, D, G, win_cap, cap = 6, 128, 4, 32, 64
    kc, vc = pkg.MSECompressor(D, 4, seed=1, device=DEV), pkg.MSECompressor(D, 2, seed=2, device=DEV)
    g = torch.Generator().manual_seed(9)
    k_win = torch.randn(rows, win_cap, D, generator=g).to(torch.bfloat16).to(DEV)
    v_win = torch.randn(rows, win_cap, D, generator=g).to(torch.bfloat16).to(DEV)
    k_new = torch.randn(rows, 2, D, generator=g).to(torch.bfloat16).to(DEV)[:, 1]      # rows 2*D elements apart
    v_new = torch.randn(rows, D, generator=g).to(torch.bfloat16).to(DEV)
    k_idx = torch.full((rows, cap, 64), 0xEE, dtype=torch.uint8, device=DEV)
    v_idx = torch.full((rows, cap, 32), 0xEE, dtype=torch.uint8, device=DEV)
    k_nrm = torch.full((rows, cap), -3.0, dtype=torch.float16, device=DEV)
    v_nrm = torch.full((rows, cap), -3.0, dtype=torch.float16, device=DEV)
    want_k, want_v = k_win.clone(), v_win.clone()
    stream = torch.cuda.current_stream().cuda_stream
    evict, put, slot = 5, 21, 7
    rc = L.tq_append_token(k_new.data_ptr(), v_new.data_ptr(), 2, 2 * D, D, k_win.data_ptr(), v_win.data_ptr(), win_cap * D,
                           evict, put, kc.table().data_ptr(), vc.table().data_ptr(), D, 4, 2,
                           k_idx.data_ptr(), k_nrm.data_ptr(), v_idx.data_ptr(), v_nrm.data_ptr(), cap, slot, rows, stream)
    assert rc == 0, L.tq_status_string(rc)
    torch.cuda.synchronize()
    want_k[:, put], want_v[:, put] = k_new, v_new
    assert torch.equal(k_win, want_k) and torch.equal(v_win, want_v)
    ck = kc.compress(want_k[:, evict].reshape(1, rows, 1, D))
    cv = vc.compress(want_v[:, evict].reshape(1, rows, 1, D))
    assert torch.equal(k_idx[:, slot], ck["idx_bytes"].reshape(rows, 64)) and torch.equal(k_nrm[:, slot], ck["vec_norms"].reshape(rows))
    assert torch.equal(v_idx[:, slot], cv["idx_bytes"].reshape(rows, 32)) and torch.equal(v_nrm[:, slot], cv["vec_norms"].reshape(rows))
    untouched = torch.ones(cap, dtype=torch.bool)
    untouched[slot] = False
    assert bool((k_idx[:, untouched] == 0xEE).all()) and bool((v_nrm[:, untouched] == -3).all())
    # evict = -1: only the window is written
    rc = L.tq_append_token(k_new.data_ptr(), v_new.data_ptr(), 2, 2 * D, D, k_win.data_ptr(), v_win.data_ptr(), win_cap * D,
                           -1, 0, None, None, D, 4, 2, None, None, None, None, cap, 0, rows, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(k_win[:, 0], k_new) and bool((k_idx[:, untouched] == 0xEE).all())
    # attend over 40 packed tokens + 9 window tokens: one call against three
    x = outlier_kv((1, rows, 40, D), seed=3, dtype=torch.bfloat16).to(DEV)
    pk, pv = kc.compress(x), vc.compress(x * 0.7)
    q = torch.randn(rows, G, D, generator=g).to(torch.bfloat16).to(DEV)
    n_w, splits, scale = 9, 2, D ** -0.5
    outs = []
    for single in (True, False):
        q_rot = torch.empty(rows, G, D, device=DEV)
        part_w = torch.empty(rows, G, D + 2, device=DEV)
        part = torch.empty(rows, splits, G, D + 2, device=DEV)
        out = torch.empty(rows, G, D, dtype=torch.bfloat16, device=DEV)
        kw, vw = k_win[:, 3:], v_win[:, 3:]
        packed = (pk["idx_bytes"].data_ptr(), pk["vec_norms"].data_ptr(), pv["idx_bytes"].data_ptr(), pv["vec_norms"].data_ptr())
        if single:
            rc = L.tq_attend_step(q.data_ptr(), 2, rows, G, scale, kc.pi_transposed().data_ptr(), vc.Pi.data_ptr(),
                                  kw.data_ptr(), vw.data_ptr(), 2, n_w, win_cap * D, *packed, 0, 40,
                                  kc.table().data_ptr(), vc.table().data_ptr(), D, 4, 2,
                                  q_rot.data_ptr(), part_w.data_ptr(), part.data_ptr(), splits, out.data_ptr(), 2, stream)
            assert rc == 0, L.tq_status_string(rc)
        else:
            assert L.tq_attend_prepare(q.data_ptr(), 2, rows, G, scale, kc.pi_transposed().data_ptr(), kw.data_ptr(), vw.data_ptr(),
                                       2, n_w, win_cap * D, q_rot.data_ptr(), part_w.data_ptr(), stream) == 0
            assert L.tq_attend_partials(*packed, 0, rows, 40, kc.table().data_ptr(), vc.table().data_ptr(), D, 4, 2,
                                        q_rot.data_ptr(), G, splits, part.data_ptr(), stream) == 0
            assert L.tq_attend_merge(part.data_ptr(), splits, part_w.data_ptr(), vc.Pi.data_ptr(), rows, G, out.data_ptr(), 2, stream) == 0
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    # and against float64 attention over the de-quantised history and the window
    kd = kc.decompress(pk).double().reshape(rows, 40, D)
    vd = vc.decompress(pv).double().reshape(rows, 40, D)
    K = torch.cat([kd, k_win[:, 3:3 + n_w].double()], 1)
    V = torch.cat([vd, v_win[:, 3:3 + n_w].double()], 1)
    ref = torch.softmax(torch.einsum("rgd,rtd->rgt", q.double(), K) * scale, -1) @ V
    err = float((outs[0].double() - ref).norm() / ref.norm())
    assert err < 6e-3, err
