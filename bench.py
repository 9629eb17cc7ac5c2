#!/usr/bin/env python3
"""Benchmark of the KV-cache compress + decompress hot path on one MI355X.

A "step" is one pass over the whole synthetic cache: every layer's K and V tensor is compressed
(packed codes + fp16 norms) and then de-quantised again, through the batched C-ABI entry points
(one launch per bit-width group and direction).  Inputs, packed buffers and outputs are
resident in HBM before the timed region starts.

Default workload (the headline configuration): Llama-3-8B-shaped cache,
32 layers x [1, 8, 32768, 128] bf16, K4/V2, protected_layers=4 with the reference's semantics
(the first and last 4 layers use 8-bit keys AND values, compressors_v3.py:158-160), no residual
window.  `--workload llama3-8b-32k-k4v2` runs the same shape with every layer at K4/V2;
`--workload qwen2.5-3b-8k` is the small Qwen2.5-3B-shaped cache (36 layers x [1, 2, 8192, 128] fp16); `--workload decode-64x16k` is the streaming
decode case (config 5): a step is one generated token through `V3Cache.update` on every layer.

Order of a run: W warm-up steps (and, for workloads with very short steps, more untimed steps until 60 ms of work have
gone by: the clocks come up from idle that slowly); an untimed pass with every launch between its own HIP events (the
per-kernel table, and which launch is the slowest); then the timed region of exactly K steps, with events around that slowest launch only (its
duration in `roofline` is the one measured there).

Prints ONE JSON line: metric, value (vectors/s), ms_per_step, config.workload, roofline (dominant kernel) and cpu_baseline.
"""
import argparse
import importlib
import json
import os
import platform
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X published HBM3E bandwidth, GB/s
MFMA_PEAK_PFLOPS = 2.5    # MI355X published dense bf16 / fp16 matrix rate, PFLOP/s
# Matrix-core work per vector: the rotation is a 128 x 128 contraction (32 768 flop).  compress runs it over the two
# 16-bit terms of the split rotation (fp32-grade result from 16-bit operands), decompress over one.
ROTATION_FLOP = 2 * 128 * 128
MFMA_PASSES = {"compress": 2, "decompress": 1}

WORKLOADS = {
    # name: layers, batch, kv heads, tokens, dtype, key_bits, value_bits, protected_layers
    "llama3-8b-32k": dict(layers=32, batch=1, heads=8, tokens=32768, dtype="bf16", key_bits=4, value_bits=2, protected=4),
    "llama3-8b-32k-k4v2": dict(layers=32, batch=1, heads=8, tokens=32768, dtype="bf16", key_bits=4, value_bits=2, protected=0),
    "qwen2.5-3b-8k": dict(layers=36, batch=1, heads=2, tokens=8192, dtype="f16", key_bits=4, value_bits=2, protected=0),
    # the same amount of data as one third of the headline cache, in heads of 64 and of 256 elements (K4/V2, bf16):
    # 64-wide vectors go through the 128-wide kernels two at a time, 256-wide ones through kernels of their own
    "d64-k4v2-64k": dict(layers=8, batch=1, heads=8, tokens=65536, dtype="bf16", key_bits=4, value_bits=2, protected=0, head_dim=64),
    "d256-k4v2-16k": dict(layers=8, batch=1, heads=8, tokens=16384, dtype="bf16", key_bits=4, value_bits=2, protected=0, head_dim=256),
    # 96 (with 160, 192 and 224: the 256-wide kernels' structure with the dimension as a template argument), and 80, which the
    # same kernels work on as 96 (zero elements in, zero codes out, whole 16-byte pieces moved as such)
    "d96-k4v2-43k": dict(layers=8, batch=1, heads=8, tokens=43648, dtype="bf16", key_bits=4, value_bits=2, protected=0, head_dim=96),
    "d80-k4v2-52k": dict(layers=8, batch=1, heads=8, tokens=52416, dtype="bf16", key_bits=4, value_bits=2, protected=0, head_dim=80),
    # streaming decode: 64 sequences with 16384 compressed + 128 window tokens; a step is
    # one new token through V3Cache.update on all 32 layers (compress what leaves the window, de-quantise all)
    "decode-64x16k": dict(layers=32, batch=64, heads=8, tokens=16384, dtype="bf16", key_bits=4, value_bits=2,
                          protected=0, window=128, decode=True),
    # the same cache read through V3Cache.append + V3Cache.attend: attention of one query token per sequence
    # (32 query heads over 8 kv heads) computed from the packed store, nothing de-quantised to memory
    "decode-attend-64x16k": dict(layers=32, batch=64, heads=8, tokens=16384, dtype="bf16", key_bits=4, value_bits=2,
                                 protected=0, window=128, decode=True, attend=True, q_heads=32),
    # the V2 key path (MSE codes + 1-bit QJL signs of the residual): a step compresses every layer's keys (two launches
    # per layer) and scores one query per head against them from the packed bytes
    "v2-keys-32k": dict(layers=8, batch=1, heads=8, tokens=32768, dtype="bf16", key_bits=3, value_bits=0, protected=0, v2=True),
    # one sequence with a long context: the latency-bound end of the same path
    "decode-attend-1x32k": dict(layers=32, batch=1, heads=8, tokens=32768, dtype="bf16", key_bits=4, value_bits=2,
                                protected=0, window=128, decode=True, attend=True, q_heads=32),
}


def packed_bytes(bits: int, head_dim: int = 128) -> int:
    return -(-head_dim // (8 // bits))


def algorithmic_bytes(bits: int, elem: int, direction: str, head_dim: int = 128) -> int:
    """Bytes per vector that must cross HBM: the vector itself plus packed codes plus the fp16 norm.
    Rotation tiles and codebook tables stay in L2/LDS and are not counted."""
    return head_dim * elem + packed_bytes(bits, head_dim) + 2


def synth_kv(torch, shape, seed, dtype, device):
    """N(0,1) x per-channel log-normal(sigma=1) x per-token U[0.5, 2], generated on the device."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    x = torch.randn(shape, generator=g, device=device, dtype=torch.float32)
    ch = torch.exp(torch.randn(shape[-1], generator=g, device=device))
    tok = 0.5 + 1.5 * torch.rand(shape[:-1] + (1,), generator=g, device=device)
    return (x * ch * tok).to(dtype)


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or platform.machine()


def stream_rates(torch, dev, gib=1.0, reps=7):
    """What this part's memory system delivers to plain streaming kernels (torch operators only, untimed leg of the
    bench): copy (1 GiB read + 1 GiB written), read-only (a sum over 1 GiB) and write-only (a fill of 1 GiB), in GB/s of
    bytes moved, median of `reps` runs after two warm-up runs.  The buffers are four times the last-level cache."""
    n = int(gib * (1 << 30)) // 4
    a = torch.zeros(n, dtype=torch.float32, device=dev)
    b = torch.empty_like(a)

    def rate(fn, nbytes):
        times = []
        for k in range(reps + 2):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            if k >= 2:
                times.append(e0.elapsed_time(e1))
        times.sort()
        return nbytes / times[len(times) // 2] / 1e6

    out = {"copy": rate(lambda: b.copy_(a), 8 * n), "read": rate(lambda: a.sum(), 4 * n), "write": rate(lambda: b.fill_(1.0), 4 * n),
           "buffer_GiB": gib, "how": "torch copy_ / sum / fill_ on float32, HIP events, median of %d" % reps}
    del a, b
    return out


def _timed_sample(run, make_input, share, budget_s, probe_n=2048, cap=4_000_000):
    """Times run(x) on a sample sized so that it takes about share * budget_s seconds; returns (vectors/s, n)."""
    x = make_input(probe_n)
    run(x)                                   # first call: thread pools, page faults
    t0 = time.perf_counter()
    run(x)
    probe = time.perf_counter() - t0
    n = int(min(max(probe_n * budget_s * share / max(probe, 1e-6), 2 * probe_n), cap))
    x = make_input(n)
    t0 = time.perf_counter()
    run(x)
    return n / (time.perf_counter() - t0), n


def cpu_baseline(pkg, widths, budget_s=20.0, head_dim=128):
    """The reference's CPU path on this machine's host cores, on a bounded sample: `widths` = {bits: share of
    vectors}.  Primary figure: the reference's op sequence issued as torch CPU operators on all cores
    (oracle.TorchCpuOracle: fp32 cast, norm, divide, sgemm, [n,D,L] broadcast / abs / argmin, int64 pack; unpack,
    gather, sgemm, scale; chunks that keep the [n,D,L] temporary under 1 GiB).  Second figure ("port"): the scalar C
    restatement of the same algorithm (oracle/tq_oracle.c, OpenMP over vectors)."""
    import numpy as np
    import torch
    from oracle import tq_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    rng = np.random.default_rng(0)
    make = lambda n: rng.standard_normal((n, head_dim), dtype=np.float32)
    seq, port, seq_desc, port_desc = {}, {}, [], []
    for bits, share in sorted(widths.items()):
        comp = pkg.MSECompressor(head_dim, bits, seed=42, device="cpu")
        pi, cent = comp.Pi.numpy(), comp.centroids.numpy()
        tor = O.TorchCpuOracle(pi, cent, bits)

        def run_seq(x):
            b, n = tor.compress(torch.from_numpy(x))
            tor.decompress(b, n)
        seq[bits], n = _timed_sample(run_seq, make, share, 0.65 * budget_s, probe_n=min(2048, tor.chunk))
        seq_desc.append(f"{n} x {bits}-bit (chunks of {tor.chunk})")
        orc = O.COracle(pi, cent, bits, accum_double=False)

        def run_port(x):
            out = orc.compress(x, want_rotated=False)
            orc.decompress(out["idx_bytes"], out["vec_norms"])
        port[bits], n = _timed_sample(run_port, make, share, 0.35 * budget_s, probe_n=4096)
        port_desc.append(f"{n} x {bits}-bit")
    # harmonic mix: time per vector of the workload = sum share_b / rate_b
    mix = lambda rates: 1.0 / sum(share / rates[b] for b, share in widths.items())
    return {
        "value": mix(seq), "unit": "vectors/s", "cores": cores, "kind": "op-sequence",
        "sample": "compress+decompress of " + ", ".join(seq_desc) + " random fp32 vectors through torch CPU operators "
                  "(the reference's op sequence, compressors_v3.py:46-105), mixed in the workload's width shares",
        "per_width_vectors_per_s": {str(b): r for b, r in seq.items()},
        "cpu": cpu_model(), "torch": torch.__version__, "torch_threads": torch.get_num_threads(),
        "port": {"value": mix(port), "unit": "vectors/s", "cores": O.COracle.threads(), "kind": "port",
                 "sample": "the same on " + ", ".join(port_desc) + " vectors through the scalar C restatement (oracle/tq_oracle.c, OpenMP)",
                 "per_width_vectors_per_s": {str(b): r for b, r in port.items()}},
    }


def power_probe(torch, step, seconds):
    """Socket power and clocks while the step runs back to back: `amd-smi metric -p -c` is called every half second from a
    thread while this thread keeps the device busy (batches of steps with a synchronisation in between, so the queue stays
    short).  Returns what amd-smi printed, reduced to the figures; untimed, and not part of any other number."""
    import re
    import shutil
    import subprocess
    import threading
    exe = shutil.which("amd-smi") or "/opt/rocm/bin/amd-smi"
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                out = subprocess.run([exe, "metric", "-p", "-c"], capture_output=True, text=True, timeout=10).stdout
            except Exception as e:      # the tool is missing or hangs: say so in the result
                samples.append({"error": repr(e)})
                return
            power = re.search(r"SOCKET_POWER:\s*(\d+)", out)
            gfx = [int(v) for v in re.findall(r"GFX_\d+:\s*\n\s*CLK:\s*(\d+)\s*MHz", out)]
            mem = re.search(r"MEM_0:\s*\n\s*CLK:\s*(\d+)\s*MHz", out)
            samples.append({"t": time.perf_counter(), "socket_W": int(power.group(1)) if power else None,
                            "gfx_clk_MHz": gfx, "mem_clk_MHz": int(mem.group(1)) if mem else None, "raw_chars": len(out)})
            stop.wait(0.5)

    th = threading.Thread(target=sampler, daemon=True)
    t0 = time.perf_counter()
    th.start()
    n = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
        n += 20
    elapsed = time.perf_counter() - t0
    stop.set()
    th.join(timeout=15)
    good = [x for x in samples if x.get("socket_W") is not None and x["t"] - t0 > 1.0]       # skip the first second
    res = {"seconds": elapsed, "steps": n, "ms_per_step": elapsed * 1e3 / max(n, 1), "samples": len(good),
           "how": "amd-smi metric -p -c every 0.5 s while the step runs back to back (samples of the first second left out)"}
    if good:
        res["socket_W"] = sorted(x["socket_W"] for x in good)[len(good) // 2]
        clocks = sorted(c for x in good for c in x["gfx_clk_MHz"])
        if clocks:
            res["gfx_clk_MHz"] = {"min": clocks[0], "median": clocks[len(clocks) // 2], "max": clocks[-1]}
        mems = [x["mem_clk_MHz"] for x in good if x["mem_clk_MHz"]]
        if mems:
            res["mem_clk_MHz"] = sorted(mems)[len(mems) // 2]
    else:
        res["note"] = "amd-smi gave no usable sample: " + json.dumps(samples[:2])
    return res


def run_v2(args, torch, pkg, w, dev):
    """TurboQuantCompressorV2 on synthetic keys: a step compresses the keys of every layer (one launch for all layers
    through the batched entry point: codes, norms, residual signs and residual norms from one pass over the input) and
    computes asymmetric_attention_scores for one query token per head, every layer with its own rotation and projection."""
    L, B, H, S, bits = w["layers"], w["batch"], w["heads"], w["tokens"], w["key_bits"]
    native = pkg._native
    comps = [pkg.TurboQuantCompressorV2(128, bits, seed=1000 * l, device=str(dev)) for l in range(L)]
    keys = [synth_kv(torch, (B, H, S, 128), seed=6_000_000 + l, dtype=torch.bfloat16, device=dev) for l in range(L)]
    packed = [comps[l].empty_packed(B, H, S, dev) for l in range(L)]
    jobs = native.QjlJobList([comps[l].job(keys[l], packed[l]) for l in range(L)], dev)
    q = synth_kv(torch, (B, H, 1, 128), seed=6_000_100, dtype=torch.float32, device=dev)
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def step(marks=None):
        out = None
        if marks:
            marks[0].record()
        jobs.compress()
        if marks:
            marks[1].record()
        for l in range(L):
            out = comps[l].asymmetric_attention_scores(q, packed[l])
        if marks:
            marks[2].record()
        return out

    for _ in range(args.warmup):
        step()
    # per-phase times from an untimed pass of its own (an event record between two kernels keeps the second from
    # starting under the tail of the first); the timed region below runs bare steps
    phase_steps = max(args.steps, 10)
    marks = [(ev(), ev(), ev()) for _ in range(phase_steps)]
    torch.cuda.synchronize()
    for k in range(phase_steps):
        step(marks[k])
    torch.cuda.synchronize()
    c_ms = sum(m[0].elapsed_time(m[1]) for m in marks) / phase_steps
    s_ms = sum(m[1].elapsed_time(m[2]) for m in marks) / phase_steps
    t0 = time.perf_counter()
    for k in range(args.steps):
        scores = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    sec = wall / args.steps
    # sanity: the estimate tracks the true inner products of the last layer
    true = torch.matmul(q.float(), keys[-1].float().transpose(-2, -1))
    cos = float(torch.nn.functional.cosine_similarity(scores.flatten(), true.flatten(), dim=0))
    if not cos > 0.8:       # (3 bits, random query: noise of the estimate ~0.04 |q||k| against signals ~0.09 |q||k|)
        sys.exit(f"bench.py: V2 scores do not follow the true inner products (cosine {cos})")
    n_vec = L * B * H * S
    mse_bits = max(bits - 1, 1)
    stored = packed_bytes(mse_bits) + 2 + 16 + 2
    comp_bytes = n_vec * (256 + stored)                 # one pass over the keys, the packed form written once
    score_bytes = n_vec * (stored + 4)                  # the packed form read once, one float32 score per key written
    # matrix work of the one-pass kernel: the rotation over two 16-bit terms, the projection by S Pi^T over three
    one_pass = mse_bits <= 4
    flop = n_vec * ROTATION_FLOP * (5 if one_pass else 8)
    result = {
        "metric": "KV vectors/sec (V2 keys: compress + scores from the packed form)", "value": n_vec / sec, "unit": "vectors/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "warmup_total": args.warmup + phase_steps, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "layers": L, "batch": B, "kv_heads": H, "tokens": S, "head_dim": 128,
                   "bits": bits, "mse_bits": mse_bits, "stored_bytes_per_vector": stored, "queries_per_head": 1},
        "compress_ms_per_step": c_ms, "scores_ms_per_step": s_ms,
        "step_algorithmic_GB": (comp_bytes + score_bytes) / 1e9, "step_GBps": (comp_bytes + score_bytes) / sec / 1e9,
        "roofline": {"bound": "mfma", "kernel": "compress (tq_qjl_compress_batched: one launch for all layers)",
                     "achieved": flop / c_ms / 1e12 * 1e3, "peak": MFMA_PEAK_PFLOPS * 1e3, "unit": "TFLOP/s",
                     "frac": flop / c_ms / 1e12 / MFMA_PEAK_PFLOPS, "traffic": None,
                     "flop_per_vector": flop // n_vec,
                     "hbm": {"achieved": comp_bytes / c_ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": comp_bytes / c_ms / 1e6 / HBM_PEAK_GBS, "algorithmic_bytes_per_vector": 256 + stored}},
        "score_cosine_vs_true": cos,
    }
    print(json.dumps(result))


def run_decode(args, torch, pkg, w, dev):
    """One decode token per step through the streaming cache: per layer, the token leaving the window
    is compressed and appended, the whole history is de-quantised into fresh K / V tensors."""
    L, B, H, S0, rw = w["layers"], w["batch"], w["heads"], w["tokens"], w["window"]
    dtype = torch.bfloat16
    cache = pkg.V3Cache(key_bits=w["key_bits"], value_bits=w["value_bits"], residual_window=rw,
                        protected_layers=w["protected"], n_layers=L, capacity=S0 + args.steps + args.warmup + 8)
    # prefill: the same synthetic K / V tensors for every layer (each layer has its own rotation)
    k0 = synth_kv(torch, (B, H, S0 + rw, 128), seed=5_000_000, dtype=dtype, device=dev)
    v0 = synth_kv(torch, (B, H, S0 + rw, 128), seed=5_000_001, dtype=dtype, device=dev)
    for l in range(L):
        cache.update(k0, v0, l)
    del k0, v0
    torch.cuda.synchronize()
    kn = synth_kv(torch, (B, H, 1, 128), seed=5_000_002, dtype=dtype, device=dev)
    vn = synth_kv(torch, (B, H, 1, 128), seed=5_000_003, dtype=dtype, device=dev)

    attend = bool(w.get("attend"))
    qn = synth_kv(torch, (B, w.get("q_heads", H), 1, 128), seed=5_000_004, dtype=dtype, device=dev) if attend else None

    def step():
        out = None
        for l in range(L):
            if attend:
                cache.append(kn, vn, l)
                out = cache.attend(qn, l)
            else:
                out = cache.update(kn, vn, l)
        return out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        res = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    total = cache.get_seq_length(0)
    n_c = total - rw
    if attend:
        if res.shape != qn.shape or not bool(torch.isfinite(res.float()).all()):
            sys.exit("bench.py: attend returned the wrong tensor")
        # what was timed equals the three-step form (scores, softmax, weighted values as separate kernels)
        ref = cache.attend(qn, L - 1, fused=False).float()
        rel = float((res.float() - ref).norm() / ref.norm())
        if not rel < 1e-2:
            sys.exit(f"bench.py: one-pass attention differs from the three-step form ({rel:.3e})")
    elif res[0].shape != (B, H, total, 128) or not torch.equal(res[0][:, :, -1:], kn):
        sys.exit("bench.py: decode step returned the wrong tensors")
    # per step and layer: K and V de-quantise ~n_c tokens per row, compress one, copy the window
    rows = B * H
    deq_vec = 2 * L * rows * (n_c - (args.steps - 1) / 2.0)
    cmp_vec = 2 * L * rows
    step_bytes = L * rows * ((n_c - (args.steps - 1) / 2.0) * (algorithmic_bytes(w["key_bits"], 2, "d") + algorithmic_bytes(w["value_bits"], 2, "d"))
                             + (algorithmic_bytes(w["key_bits"], 2, "c") + algorithmic_bytes(w["value_bits"], 2, "c"))
                             + 2 * rw * 512)
    sec = wall / args.steps
    if attend:
        # packed codes and norms are read once; nothing de-quantised is written
        step_bytes = L * rows * ((n_c - (args.steps - 1) / 2.0) * (packed_bytes(w["key_bits"]) + packed_bytes(w["value_bits"]) + 4)
                                 + (algorithmic_bytes(w["key_bits"], 2, "c") + algorithmic_bytes(w["value_bits"], 2, "c"))
                                 + 2 * rw * 256)
    result = {
        "metric": ("KV vectors/sec (compressed on append + attended from packed codes)" if attend
                   else "KV vectors/sec (compress+decompress)"),
        "value": (deq_vec + cmp_vec) / sec, "unit": "vectors/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "layers": L, "batch": B, "kv_heads": H, "compressed_tokens": n_c,
                   "window_tokens": rw, "head_dim": 128, "key_bits": w["key_bits"], "value_bits": w["value_bits"],
                   "new_tokens_per_step": 1},
        "decode_steps_per_s": 1.0 / sec,
        "step_algorithmic_GB": step_bytes / 1e9, "step_GBps": step_bytes / sec / 1e9,
        "roofline": {"bound": "hbm", "kernel": "whole step (query rotation + window, one-pass attention over packed codes, merge)" if attend else "whole step (decompress dominates)", "achieved": step_bytes / sec / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": step_bytes / sec / 1e9 / HBM_PEAK_GBS, "traffic": None},
        "stored_GB": cache.stored_bytes() / 1e9,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(pkg, {w["key_bits"]: 0.5, w["value_bits"]: 0.5}, args.cpu_seconds)
    print(json.dumps(result))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3-8b-32k", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=20.0)
    ap.add_argument("--skeleton", action="store_true",
                    help="time the memory-skeleton build of the two codec kernels (csrc/libtqamd_skeleton.so from "
                         "_native.build_skeleton(): loads, LDS traffic and stores only; the output is garbage)")
    ap.add_argument("--no-stream-rates", action="store_true", help="skip the plain-stream leg (copy / read / write rates of the part)")
    ap.add_argument("--power-probe", type=float, default=0.0, metavar="SECONDS",
                    help="after the timed region keep the step running for this long and sample socket power and clocks with amd-smi "
                         "(reported as `power_probe`; untimed)")
    ap.add_argument("--probe-launches", default="all", choices=("all", "compress", "decompress"),
                    help="which launches of the step the power probe repeats (default: the whole step)")
    ap.add_argument("--launch-order", default="",
                    help="sequence of the step's launches, e.g. c2,c4,c8,d8,d4,d2 (default: compress by width, then decompress by width)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; the codec shards without communication "
                 "(by layer / KV head / token range), so run one process per GPU instead of --gpus N>1")

    import torch
    pkg = importlib.import_module("turboquant-pytorch_amd")
    native = pkg._native
    if args.skeleton:
        if not os.path.exists(native.SKELETON_LIB_PATH):
            sys.exit(f"bench.py --skeleton: {native.SKELETON_LIB_PATH} is missing; build it first (on the CPU): "
                     "python -c 'import importlib; importlib.import_module(\"turboquant-pytorch_amd._native\").build_skeleton()'")
        native.LIB_PATH = native.SKELETON_LIB_PATH          # before the first call loads the library
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    w = WORKLOADS[args.workload]
    if w.get("decode"):
        return run_decode(args, torch, pkg, w, dev)
    if w.get("v2"):
        return run_v2(args, torch, pkg, w, dev)
    L, B, H, S = w["layers"], w["batch"], w["heads"], w["tokens"]
    D = w.get("head_dim", 128)
    rotation_flop = 2 * D * D                 # the rotation is a D x D contraction
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16}[w["dtype"]]
    n_vec = B * H * S

    # ---- compressors (reference constructor semantics) and resident buffers -------------------
    groups = {}   # bits -> list of job dicts
    layers = []
    for l in range(L):
        tq = pkg.TurboQuantV3(D, key_bits=w["key_bits"], value_bits=w["value_bits"], residual_window=0,
                              layer_idx=l, n_layers=L, protected_layers=w["protected"], device=str(dev))
        layers.append(tq)
        for which, comp in (("k", tq.key_compressor), ("v", tq.val_compressor)):
            x = synth_kv(torch, (B, H, S, D), seed=4_000_000 + 10 * l + (0 if which == "k" else 1), dtype=dtype, device=dev)
            job = {
                "states": x,
                "idx_bytes": torch.empty((B, H, S, packed_bytes(comp.bits, D)), dtype=torch.uint8, device=dev),
                "vec_norms": torch.empty((B, H, S), dtype=torch.float16, device=dev),
                "table": comp.table(), "bits": comp.bits,
                "out": torch.empty((B, H, S, D), dtype=dtype, device=dev),
            }
            groups.setdefault(comp.bits, []).append(job)
    comp_lists = {b: native.JobList(jobs, dev) for b, jobs in groups.items()}
    deco_lists = {b: native.JobList([dict(j, states=j["out"]) for j in jobs], dev) for b, jobs in groups.items()}
    order = sorted(groups)
    torch.cuda.synchronize()

    launches = [("compress", b) for b in order] + [("decompress", b) for b in order]
    if args.launch_order:     # e.g. "c2,c4,c8,d8,d4,d2": the same six launches in another sequence
        launches = [("compress" if t[0] == "c" else "decompress", int(t[1:])) for t in args.launch_order.split(",")]
        if sorted(launches) != sorted([("compress", b) for b in order] + [("decompress", b) for b in order]):
            raise SystemExit(f"--launch-order must name every launch of the workload once: {order}")
        if any(launches.index(("compress", b)) > launches.index(("decompress", b)) for b in order):
            raise SystemExit("--launch-order: a width group is de-quantised before it is compressed")

    def step(evs=None, only=None):
        """One pass over the cache.  `evs`: pre-created (start, stop) event pairs, one per launch; `only`: the
        index of the single launch that is bracketed (all of them when None)."""
        for i, (direction, b) in enumerate(launches):
            timed = evs is not None and (only is None or only == i)
            if timed:
                evs[i][0].record()
            (comp_lists[b].compress if direction == "compress" else deco_lists[b].decompress)()
            if timed:
                evs[i][1].record()

    def make_events(n_steps):
        # HIP events are created and recorded once (which is what allocates them) outside any timed region
        evs = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in launches]
               for _ in range(n_steps)]
        for row in evs:
            for e0, e1 in row:
                e0.record()
                e1.record()
        return evs

    for _ in range(args.warmup):
        step()
    # A workload whose step takes a fraction of a millisecond would otherwise be timed while the clocks are still on
    # their way up from idle (the first tens of milliseconds of work after a pause run slower): untimed steps until
    # about 60 ms of work have gone by since the start of the warm-up.
    torch.cuda.synchronize()
    t_probe = time.perf_counter()
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    per_step = max((time.perf_counter() - t_probe) / 3, 1e-6)
    conditioning_steps = min(1000, max(0, int(0.06 / per_step) - args.warmup - 3))
    for _ in range(conditioning_steps):
        step()
    # ---- per-kernel pass (untimed): every launch between its own pair of events.  An event record between two
    # kernels keeps the second from starting under the tail of the first (about 3 us each, 12 of them a step), so the
    # timed region below brackets one launch only, the slowest one of this pass.  The pass also brings the clocks to
    # the state of a running job: the first tens of milliseconds after an idle period run slower.
    table_steps = max(args.steps, 10)
    table_events = make_events(table_steps)
    torch.cuda.synchronize()
    for evs in table_events:
        step(evs)
    torch.cuda.synchronize()
    table_ms = {}
    for li, launch in enumerate(launches):
        table_ms[launch] = sum(evs[li][0].elapsed_time(evs[li][1]) for evs in table_events) / table_steps
    dominant_launch = max(table_ms, key=table_ms.get)
    dominant_index = launches.index(dominant_launch)
    step_events = make_events(args.steps)
    torch.cuda.synchronize()

    # ---- timed region: exactly `steps` steps ----------------------------------------------------
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for k in range(args.steps):
        step(step_events[k], only=dominant_index)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = start.elapsed_time(stop)
    ms_per_step = wall * 1000.0 / args.steps
    live_ms = sum(evs[dominant_index][0].elapsed_time(evs[dominant_index][1]) for evs in step_events) / args.steps

    # ---- sanity: what was timed is a real round trip ----------------------------------------------
    j = groups[order[0]][0]
    rel = float((j["out"].float() - j["states"].float()).norm() / j["states"].float().norm())
    if not (0.0 < rel < 0.6) and not args.skeleton:
        sys.exit(f"bench.py: round trip looks wrong (relative error {rel})")

    # ---- accounting ------------------------------------------------------------------------------------
    elem = 2
    total_vec = 2 * L * n_vec                       # K and V counted separately
    kernels = {}
    step_bytes = 0
    for (direction, b), table_avg in table_ms.items():
        jobs = len(groups[b])
        bytes_per_launch = jobs * n_vec * algorithmic_bytes(b, elem, direction, D)
        live = (direction, b) == dominant_launch
        avg_ms = live_ms if live else table_avg          # the dominant launch: measured inside the timed region
        step_bytes += bytes_per_launch
        flop = jobs * n_vec * rotation_flop * MFMA_PASSES[direction]
        kernels[f"{direction}_b{b}"] = {
            "launches_per_step": 1, "jobs": jobs, "vectors_per_launch": jobs * n_vec,
            "algorithmic_bytes_per_launch": bytes_per_launch, "avg_ms": avg_ms,
            "timed": "events inside the timed region" if live else f"events in the {table_steps} untimed steps before it",
            "avg_ms_untimed_pass": table_avg,
            "achieved_GBps": bytes_per_launch / avg_ms / 1e6,
            "frac_of_hbm_peak": bytes_per_launch / avg_ms / 1e6 / HBM_PEAK_GBS,
            "mfma_flop_per_launch": flop, "mfma_PFLOPs": flop / avg_ms / 1e12,
            "frac_of_mfma_peak": flop / avg_ms / 1e12 / MFMA_PEAK_PFLOPS,
        }
    dominant = f"{dominant_launch[0]}_b{dominant_launch[1]}"
    dk = kernels[dominant]
    # HBM bytes per launch of the dominant kernel as the counters saw them (FETCH_SIZE + WRITE_SIZE, calibrated against
    # a copy kernel): a number from the committed profile run of this workload, not measured by this process
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        try:
            traffic = json.load(open(tpath)).get(args.workload, {}).get(dominant)
            traffic_source = "profiles/hbm_traffic.json (rocprofv3 --pmc run of this workload, committed)" if traffic else None
        except Exception:
            traffic = None

    def mfma_of(direction):
        """the rotation's matrix-core rate in the slowest launch of one direction"""
        name = max((k for k in kernels if k.startswith(direction)), key=lambda k: kernels[k]["avg_ms"])
        k = kernels[name]
        return {"kernel": name, "flop_per_vector": rotation_flop * MFMA_PASSES[direction],
                "flop_per_launch": k["mfma_flop_per_launch"], "achieved": k["mfma_PFLOPs"], "peak": MFMA_PEAK_PFLOPS,
                "unit": "PFLOP/s", "frac": k["frac_of_mfma_peak"]}

    # The bound is the one the dominant launch is nearer to.  At 128 elements a vector it is the memory system (about 6
    # matrix flop per byte); at 256 the rotation does four times the flop per vector on twice the bytes and the
    # two-pass split-precision product makes compress matrix-bound.
    if dk["frac_of_mfma_peak"] > dk["frac_of_hbm_peak"]:
        roofline = {"bound": "mfma", "kernel": dominant, "achieved": dk["mfma_PFLOPs"] * 1e3, "peak": MFMA_PEAK_PFLOPS * 1e3,
                    "unit": "TFLOP/s", "frac": dk["frac_of_mfma_peak"], "traffic": traffic, "traffic_source": traffic_source,
                    "hbm": {"achieved": dk["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dk["frac_of_hbm_peak"]}}
    else:
        roofline = {"bound": "hbm", "kernel": dominant, "achieved": dk["achieved_GBps"], "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": dk["frac_of_hbm_peak"], "traffic": traffic, "traffic_source": traffic_source}
    roofline["mfma"] = {"compress": mfma_of("compress"), "decompress": mfma_of("decompress")}

    widths = {}
    for b, jobs in groups.items():
        widths[b] = len(jobs) / (2 * L)
    result = {
        "metric": "KV vectors/sec (compress+decompress)",
        "value": total_vec * args.steps / wall,
        "unit": "vectors/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "untimed_steps_after_warmup": 3 + conditioning_steps + table_steps,
        "warmup_total": args.warmup + 3 + conditioning_steps + table_steps,      # every untimed step before the timed region
        "config": {"workload": args.workload, "layers": L, "batch": B, "kv_heads": H, "tokens": S, "head_dim": D,
                   "key_bits": w["key_bits"], "value_bits": w["value_bits"], "protected_layers": w["protected"],
                   "residual_window": 0, "width_groups": {str(b): len(groups[b]) for b in order},
                   "vectors_per_step": total_vec},
        "gpu_ms_per_step": gpu_ms / args.steps,
        "step_algorithmic_GB": step_bytes / 1e9,
        "step_GBps": step_bytes / (wall / args.steps) / 1e9,
        "step_frac_of_hbm_peak": step_bytes / (wall / args.steps) / 1e9 / HBM_PEAK_GBS,
        "roofline": roofline,
        "kernels": kernels,
        "round_trip_rel_error": rel,
    }
    if args.skeleton:
        result["skeleton"] = ("memory-skeleton build: no matrix instructions, no code search, no decode; the output is "
                              "garbage and `value` is not a measurement of the codec")
    if not args.no_stream_rates:
        # the part's plain-stream rates beside the codec's: what a copy, a read and a write kernel reach on this box
        result["roofline"]["stream_GBps"] = stream_rates(torch, dev)
        result["roofline"]["step_frac_of_copy_rate"] = result["step_GBps"] / result["roofline"]["stream_GBps"]["copy"]
    if args.power_probe > 0:
        def probe_step():
            for direction, b in launches:
                if args.probe_launches in ("all", direction):
                    (comp_lists[b].compress if direction == "compress" else deco_lists[b].decompress)()
        result["power_probe"] = power_probe(torch, probe_step, args.power_probe)
        result["power_probe"]["launches"] = args.probe_launches
    if not args.no_cpu_baseline and not args.skeleton:
        result["cpu_baseline"] = cpu_baseline(pkg, widths, args.cpu_seconds, head_dim=D)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
