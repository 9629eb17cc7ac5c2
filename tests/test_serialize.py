"""On-disk form of compressed KV data: round trips, header checks, and that a reloaded cache continues
exactly where the saved one stopped.  The reference has no wire format (compressors_v3.py:76-81 keeps
plain dicts); what is checked here is that writing and reading change no byte."""
import importlib
import json

import pytest
import torch

DEV = "cuda:0"


@pytest.fixture(scope="module")
def pkg():
    return importlib.import_module("turboquant-pytorch_amd")


def _filled_cpu_cache(pkg, n_c=300, n_w=5):
    """A V3Cache whose stores are filled by hand on the CPU (the codec itself only runs on the GPU)."""
    kvc = importlib.import_module("turboquant-pytorch_amd.kv_cache")
    B, H, D = 1, 2, 128
    g = torch.Generator().manual_seed(5)
    cache = pkg.V3Cache(4, 2, residual_window=8, protected_layers=1, n_layers=4)
    for layer in (0, 2):
        comp = cache._get_compressor(layer, D, torch.device("cpu"))
        st = kvc._LayerStore(comp, B, H, D, torch.bfloat16, torch.device("cpu"), n_c, 8)
        if n_c:
            for name in ("k_idx", "v_idx"):
                buf = getattr(st, name)
                buf[:, :, :n_c] = torch.randint(0, 256, buf[:, :, :n_c].shape, generator=g).to(torch.uint8)
            for name in ("k_nrm", "v_nrm"):
                getattr(st, name)[:, :, :n_c] = torch.rand(B, H, n_c, generator=g).half()
        st.n_compressed = n_c
        st.extend_window(torch.randn(B, H, n_w, D, generator=g).bfloat16(), torch.randn(B, H, n_w, D, generator=g).bfloat16())
        st.total_seq = n_c + n_w
        cache._stores[layer] = st
    return cache


def _same_state(a, b):
    assert sorted(a._stores) == sorted(b._stores)
    for idx in a._stores:
        x, y = a._stores[idx], b._stores[idx]
        assert (x.n_compressed, x.n_recent, x.total_seq, x.B, x.H, x.D, x.dtype) == (y.n_compressed, y.n_recent, y.total_seq, y.B, y.H, y.D, y.dtype)
        assert (x.comp.key_bits, x.comp.value_bits) == (y.comp.key_bits, y.comp.value_bits)
        n = x.n_compressed
        for name in ("k_idx", "k_nrm", "v_idx", "v_nrm"):
            if n:
                assert torch.equal(getattr(x, name)[:, :, :n].cpu(), getattr(y, name)[:, :, :n].cpu()), name
        assert all(torch.equal(p.cpu(), q.cpu()) for p, q in zip(x.window(), y.window()))
        assert torch.equal(x.comp.key_compressor.Pi.cpu(), y.comp.key_compressor.Pi.cpu())
        assert torch.equal(x.comp.val_compressor.centroids.cpu(), y.comp.val_compressor.centroids.cpu())


def test_cache_file_round_trip_on_host(pkg, tmp_path):
    cache = _filled_cpu_cache(pkg)
    for include_codec in (True, False):
        path = str(tmp_path / f"cache{int(include_codec)}.safetensors")
        cache.save(path, include_codec=include_codec)
        back = pkg.V3Cache.load(path, device="cpu")
        assert (back.key_bits, back.value_bits, back.residual_window, back.protected_layers, back.n_layers) == (4, 2, 8, 1, 4)
        _same_state(cache, back)
        assert back._stores[0].comp.key_bits == 8 and back._stores[2].comp.key_bits == 4      # layer 0 is protected
        assert back.get_compression_info() == cache.get_compression_info()
    # header is plain JSON in the safetensors metadata; tensors carry the documented names
    from safetensors import safe_open
    f = safe_open(path, framework="pt", device="cpu")
    header = json.loads(f.metadata()["tqamd"])
    assert header["kind"] == "kv-cache" and header["version"] == 1 and sorted(header["layers"]) == ["0", "2"]
    assert header["layers"]["2"]["n_compressed"] == 300 and header["layers"]["2"]["dtype"] == "bfloat16"
    assert set(f.keys()) == {f"L{i}.{n}" for i in (0, 2) for n in ("k_idx", "k_nrm", "v_idx", "v_nrm", "k_win", "v_win")}
    assert f.get_tensor("L2.k_idx").shape == (1, 2, 300, 64) and f.get_tensor("L2.v_idx").shape == (1, 2, 300, 32)


def test_empty_cache_and_empty_window(pkg, tmp_path):
    path = str(tmp_path / "empty.safetensors")
    pkg.V3Cache(3, 3, residual_window=0, n_layers=2).save(path)
    back = pkg.V3Cache.load(path, device="cpu")
    assert back._stores == {} and back.key_bits == 3 and back.residual_window == 0
    cache = _filled_cpu_cache(pkg, n_c=64, n_w=0)
    cache.save(path)
    _same_state(cache, pkg.V3Cache.load(path, device="cpu"))
    cache = _filled_cpu_cache(pkg, n_c=0, n_w=7)
    cache.save(path)
    _same_state(cache, pkg.V3Cache.load(path, device="cpu"))


def test_codec_mismatch_is_detected(pkg, tmp_path):
    """A file written with other rotations is refused unless it carries its codec, in which case that codec is used."""
    cache = _filled_cpu_cache(pkg)
    other = pkg.MSECompressor(128, 4, seed=987654, device="cpu")        # not the seed layer 2 would get
    cache._stores[2].comp.key_compressor = other
    bare, full = str(tmp_path / "bare.safetensors"), str(tmp_path / "full.safetensors")
    cache.save(bare, include_codec=False)
    cache.save(full, include_codec=True)
    with pytest.raises(pkg.FormatError, match="different rotation"):
        pkg.V3Cache.load(bare, device="cpu")
    back = pkg.V3Cache.load(full, device="cpu")
    assert torch.equal(back._stores[2].comp.key_compressor.Pi, other.Pi)
    assert pkg.codec_digest(back._stores[2].comp.key_compressor) == pkg.codec_digest(other)
    assert pkg.codec_digest(other) != pkg.codec_digest(pkg.MSECompressor(128, 4, seed=987655, device="cpu"))
    assert pkg.codec_digest(other) != pkg.codec_digest(pkg.MSECompressor(128, 3, seed=987654, device="cpu"))


def test_dict_pair_round_trip_and_header_checks(pkg, tmp_path):
    B, H, S, D = 1, 2, 10, 128
    g = torch.Generator().manual_seed(3)
    t = pkg.TurboQuantV3(128, 4, 2, residual_window=4, layer_idx=5, n_layers=36, device="cpu")
    ck = {"compressed": {"idx_bytes": torch.randint(0, 256, (B, H, 6, 64), generator=g).to(torch.uint8),
                         "vec_norms": torch.rand(B, H, 6, generator=g).half(), "shape": (B, H, 6, D), "idx_pad": 0},
          "fp16": torch.randn(B, H, 4, D, generator=g).half(), "shape": (B, H, S, D), "split_at": 6}
    cv = {"compressed": None, "fp16": torch.randn(B, H, S, D, generator=g).half(), "shape": (B, H, S, D), "split_at": S}
    path = str(tmp_path / "pair.safetensors")
    pkg.save_compressed(path, ck, cv, codec=t)
    a, b = pkg.load_compressed(path, device="cpu", codec=t)
    assert a["shape"] == (B, H, S, D) and a["split_at"] == 6 and b["compressed"] is None and b["split_at"] == S
    assert a["compressed"]["shape"] == (B, H, 6, D) and a["compressed"]["idx_pad"] == 0
    assert torch.equal(a["compressed"]["idx_bytes"], ck["compressed"]["idx_bytes"])
    assert torch.equal(a["compressed"]["vec_norms"], ck["compressed"]["vec_norms"])
    assert torch.equal(a["fp16"], ck["fp16"]) and torch.equal(b["fp16"], cv["fp16"])
    wrong = pkg.TurboQuantV3(128, 4, 2, residual_window=4, layer_idx=6, n_layers=36, device="cpu")
    with pytest.raises(pkg.FormatError, match="different rotation"):
        pkg.load_compressed(path, device="cpu", codec=wrong)
    with pytest.raises(pkg.FormatError, match="expected a 'kv-cache'"):
        pkg.V3Cache.load(path, device="cpu")
    from safetensors.torch import save_file
    alien = str(tmp_path / "alien.safetensors")
    save_file({"x": torch.zeros(1)}, alien)
    with pytest.raises(pkg.FormatError, match="not a file written"):
        pkg.load_compressed(alien, device="cpu")
    save_file({"x": torch.zeros(1)}, alien, metadata={"tqamd": json.dumps({"kind": "kv-pair", "version": 99})})
    with pytest.raises(pkg.FormatError, match="format version 99"):
        pkg.load_compressed(alien, device="cpu")


@pytest.mark.gpu
def test_reloaded_cache_continues_bit_exactly(pkg, tmp_path):
    """Prefill + a few decode steps, save, load: identical state, identical attend() output, and both caches
    stay identical through further appends (one of which makes the reloaded store grow)."""
    from test_gpu_parity import outlier_kv
    B, H, G, D, L = 2, 2, 4, 128, 3
    cache = pkg.V3Cache(key_bits=4, value_bits=2, residual_window=16, protected_layers=1, n_layers=L)
    total = 300 + 6 + 400
    keys = [outlier_kv((B, H, total, D), seed=40 + l, dtype=torch.bfloat16).to(DEV) for l in range(L)]
    vals = [outlier_kv((B, H, total, D), seed=50 + l, dtype=torch.bfloat16).to(DEV) for l in range(L)]
    seen = 0
    for n in (300, 1, 1, 4):
        for l in range(L):
            cache.append(keys[l][:, :, seen:seen + n], vals[l][:, :, seen:seen + n], l)
        seen += n
    path = str(tmp_path / "cache.safetensors")
    cache.save(path)
    back = pkg.V3Cache.load(path, device=DEV)
    _same_state(cache, back)
    g = torch.Generator().manual_seed(1)
    q = (3 * torch.randn(B, H * G, 1, D, generator=g)).to(torch.bfloat16).to(DEV)
    for l in range(L):
        assert torch.equal(cache.attend(q, l), back.attend(q, l))
    for n in (1, 399):
        for l in range(L):
            cache.append(keys[l][:, :, seen:seen + n], vals[l][:, :, seen:seen + n], l)
            back.append(keys[l][:, :, seen:seen + n], vals[l][:, :, seen:seen + n], l)
        seen += n
    _same_state(cache, back)
    for l in range(L):
        assert torch.equal(cache.attend(q, l), back.attend(q, l))


@pytest.mark.gpu
def test_compress_kv_pair_survives_the_file(pkg, tmp_path):
    from test_gpu_parity import outlier_kv
    t = pkg.TurboQuantV3(128, 4, 2, residual_window=32, layer_idx=7, n_layers=36, device=DEV)
    k = outlier_kv((1, 4, 200, 128), seed=60, dtype=torch.float16).to(DEV)
    v = outlier_kv((1, 4, 200, 128), seed=61, dtype=torch.float16).to(DEV)
    ck, cv = t.compress_kv(k, v)
    path = str(tmp_path / "pair.safetensors")
    pkg.save_compressed(path, ck, cv, codec=t)
    ck2, cv2 = pkg.load_compressed(path, device=DEV, codec=t)
    rk, rv = t.decompress_kv(ck, cv)
    rk2, rv2 = t.decompress_kv(ck2, cv2)
    assert torch.equal(rk, rk2) and torch.equal(rv, rv2)
