#!/usr/bin/env python3
"""Decode-step benchmark of the KV-cache hot path on one MI355X.

A step = one new token for every sequence: for each layer, append K and V to the
cache and run GQA decode attention over the whole context, then positions += 1.
The step is captured once in a hipGraph and replayed.  Inputs (caches, q, k, v)
are resident in HBM before the timed region; every layer has its own cache, so
nothing is re-read from a cache level between layers or steps.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--kv-bits 0|2|4]

Prints one JSON line: decode-attention tokens/s (sequences advanced per second),
the HBM roofline of the context-scanning attention kernel, and the CPU oracle
timed on this machine's host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

# name -> shape.  "target" is the case the headline metric is quoted on.
WORKLOADS = {
    "target":  dict(desc="TQ decode attention, Qwen3-0.6B KV shape, 28 layers, batch 64, context 8192",
                    L=28, H=16, Hk=8, G=64, ctx=8192, ragged=None, kv_bits=4),
    "config1": dict(desc="fp16 cache, 1 layer, batch 4, context 612+1", L=1, H=16, Hk=8, G=4, ctx=613, ragged=None, kv_bits=0),
    "config2": dict(desc="TQ4, 28 layers, batch 4, context 612+1", L=28, H=16, Hk=8, G=4, ctx=613, ragged=None, kv_bits=4),
    "config3": dict(desc="TQ4, 28 layers, batch 64 ragged contexts U[512,8192]", L=28, H=16, Hk=8, G=64, ctx=8192,
                    ragged=(512, 8192), kv_bits=4),
    "config5": dict(desc="GRPO rollout: 16 prompts x group 8 = 128 sequences, shared 256-token prefix, decode from context 257 "
                         "(run with --steps 512)", L=28, H=16, Hk=8, G=128, ctx=257, ragged=None, kv_bits=4, prefix=(256, 8)),
    "config4": dict(desc="TQ2, Qwen3-8B-like KV shape, 36 layers, batch 16, context 4096+1", L=36, H=32, Hk=8, G=16,
                    ctx=4097, ragged=None, kv_bits=2),
}
BYTES_HEAD = {0: 256, 4: 66, 2: 34}  # per (token, kv head): fp16 row | codes + fp16 norm

# HBM bytes per launch (read + write) of the context-scanning kernel, from rocprofv3 --pmc FETCH_SIZE
# and WRITE_SIZE on this file's own run, each counter scaled by what `--copy-calibration` reads for a
# copy of known size (2.0 and 1.0); summary and commands in profiles/scan_target_hbm_traffic_pmc.txt.
# Keyed by (workload, kv_bits, kernel that ran).  Counters are not read in this run: the figures belong to
# the kernel sources whose digest is recorded with them (`python bench.py --csrc-digest` prints the current
# one) and are only reported while the sources are still those; otherwise `traffic` is null.
MEASURED_TRAFFIC_CSRC_DIGEST = "b9f7671537eaf017"
MEASURED_TRAFFIC_BYTES = {("target", 4, "one-launch"): 555.1e6, ("target", 4, "scan"): 560.8e6,
                          ("target", 2, "one-launch"): 286.8e6, ("target", 2, "scan"): 292.3e6,
                          ("target", 0, "scan"): 2154.7e6}
TRAFFIC_SOURCE = "profiles/scan_target_hbm_traffic_pmc.txt"


def csrc_digest() -> str:
    """Digest of the sources of the decode kernels (triebwerk_amd/csrc without the prompt kernels' own files,
    kv_prefill_*, which no decode kernel includes), file names and contents in sorted order."""
    import hashlib
    h = hashlib.sha256()
    for f in sorted((ROOT / "triebwerk_amd" / "csrc").iterdir()):
        if f.suffix in (".hip", ".hpp") and not f.name.startswith("kv_prefill"):
            h.update(f.name.encode()); h.update(b"\0"); h.update(f.read_bytes())
    return h.hexdigest()[:16]


def measured_traffic(workload: str, kv_bits: int, one_launch: bool):
    """(bytes or None, where the figure comes from)."""
    if csrc_digest() != MEASURED_TRAFFIC_CSRC_DIGEST:
        return None, f"none: kernel sources changed since {TRAFFIC_SOURCE} was measured"
    val = MEASURED_TRAFFIC_BYTES.get((workload, kv_bits, "one-launch" if one_launch else "scan"))
    return val, (f"{TRAFFIC_SOURCE} (rocprofv3 --pmc, not read in this run; kernel sources {MEASURED_TRAFFIC_CSRC_DIGEST})"
                 if val is not None else "none: not measured for this workload")


DTYPE = {0: "f16 cache, f32 accumulate (vector ALU)",
         4: "u8 codes (4 bit) + f16 norms -> f16-operand MFMA (centroids as f16, q and p as f16 hi+lo pairs), f32 accumulate",
         2: "u8 codes (2 bit) + f16 norms -> f16-operand MFMA (centroids as f16, q and p as f16 hi+lo pairs), f32 accumulate"}


def algorithmic_bytes(n_tokens_total: int, G: int, L: int, H: int, Hk: int, kv_bits: int, with_append: bool) -> int:
    """Bytes one step must move, each cache byte counted once per step (not once per query head)."""
    D = 128
    per_layer = n_tokens_total * Hk * 2 * BYTES_HEAD[kv_bits] + G * H * D * 2 * 2
    if with_append:
        per_layer += G * (Hk * 2 * BYTES_HEAD[kv_bits] + Hk * D * 2 * 2)
    return per_layer * L


def fill_caches(eng, L, kv_bits, seed):
    """Random cache contents: uniform code bytes, norms around sqrt(128)."""
    import torch
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    for l in range(L):
        ck, cv, kn, vn = eng.cache(l)
        if kv_bits == 0:
            for t in (ck, cv):
                flat = t.view(-1)
                step = 1 << 28
                for i in range(0, flat.numel(), step):
                    part = flat[i:i + step]
                    part.copy_(torch.randn(part.numel(), generator=gen, device="cuda", dtype=torch.float16))
        else:
            for t in (ck, cv):
                flat = t.view(-1).view(torch.int32)
                flat.copy_(torch.randint(-2 ** 31, 2 ** 31 - 1, (flat.numel(),), generator=gen, device="cuda",
                                         dtype=torch.int32))
            for t in (kn, vn):
                t.copy_((11.3 + 0.7 * torch.randn(t.shape, generator=gen, device="cuda")).to(torch.float16))


def cpu_baseline(w, kv_bits, seconds_budget=15.0):
    """The CPU oracle (a restatement of the reference kernels, oracle/kv_oracle.cpp) on a
    bounded sample of the workload: one layer, as many sequences as fit the time budget."""
    import gen
    import oracle_lib
    o = oracle_lib.load_o3()          # the oracle's source built -O3 for x86-64-v3 (oracle/Makefile)
    threads = o.num_threads()
    H, Hk, D = w["H"], w["Hk"], 128
    kv_dim, q_dim = Hk * D, H * D
    ctx = w["ctx"]
    r = gen.rng(9)
    rot, _ = o.make_rotation(128, 42)

    def run(S):
        msl = ctx
        pos = np.full(S, ctx - 1, np.int32)
        q = gen.normal_f16(r, (S, q_dim)); k = gen.normal_f16(r, (S, kv_dim)); v = gen.normal_f16(r, (S, kv_dim))
        out = np.zeros((S, q_dim), np.float16)
        if kv_bits == 0:
            ck = gen.normal_f16(r, (S, msl, kv_dim)); cv = gen.normal_f16(r, (S, msl, kv_dim))
            t0 = time.perf_counter()
            o.kv_cache_write_batch(ck, cv, k, v, pos, msl, S, kv_dim)
            o.gqa_attention_batch(out, q, ck, cv, pos, msl, S, H, Hk, D, q_dim, kv_dim)
            return time.perf_counter() - t0
        kvp = kv_dim * kv_bits // 8
        ck = r.integers(0, 256, (S, msl, kvp), dtype=np.uint8); cv = r.integers(0, 256, (S, msl, kvp), dtype=np.uint8)
        kn = np.full((S, msl, Hk), 11.3, np.float16); vn = np.full((S, msl, Hk), 11.3, np.float16)
        t0 = time.perf_counter()
        o.turbo_kv_quantize_batch(ck, kn, k, rot, pos, msl, S, Hk, D, kv_dim, kv_bits)
        o.turbo_kv_quantize_batch(cv, vn, v, rot, pos, msl, S, Hk, D, kv_dim, kv_bits)
        o.turbo_gqa_attention_batch(out, q, ck, cv, kn, vn, rot, pos, msl, S, H, Hk, D, q_dim, kv_dim, kv_bits)
        return time.perf_counter() - t0

    S = max(1, min(w["G"], (threads + H - 1) // H))     # one pass that occupies every thread
    t = run(S)
    per_seq = t / S
    S2 = int(max(S, min(w["G"], seconds_budget / max(per_seq, 1e-9))))
    if S2 > S:
        t, S = run(S2), S2
    # more layers of the same sample until the budget is used (never more than the workload has)
    layers = 1
    while layers < w["L"] and t + t / layers < seconds_budget:
        t += run(S)
        layers += 1
    tokens_per_s = S * layers / (t * w["L"])   # `layers` layers measured; a step needs L of them
    return dict(value=tokens_per_s, unit="tokens/s", cores=threads, kind="port",
                sample=f"{layers} of {w['L']} layers x {S} of {w['G']} sequences at context {ctx}, "
                       f"{t:.2f} s of CPU time, scaled linearly; oracle/kv_oracle.cpp built -O3 -march=x86-64-v3, OpenMP over (sequence, head), "
                       f"{os.cpu_count()} logical CPUs visible")


def prefill_bench(args, quiet=False):
    """Causal prefill attention of one sequence, one layer: ms per launch and the matrix-core rate.
    FLOPs counted: 4 * head_dim per (query head, query token, attended token), causal half only."""
    import torch
    from triebwerk_amd import kvcache
    w = WORKLOADS[args.workload]
    kv_bits = w["kv_bits"] if args.kv_bits is None else args.kv_bits
    H, Hk, D, T = w["H"], w["Hk"], 128, args.prefill
    kvcache.set_attention_variant(args.variant)
    kvcache.set_prefill_form(args.prefill_form)
    g = torch.Generator(device="cuda"); g.manual_seed(11)
    q = torch.randn((T, H * D), generator=g, device="cuda", dtype=torch.float16)
    out = torch.zeros_like(q)
    ws = torch.zeros(H * T * min(T, 4096), dtype=torch.float32, device="cuda")
    if kv_bits:
        kvp = Hk * D * kv_bits // 8
        ck = torch.randint(0, 256, (T, kvp), generator=g, device="cuda", dtype=torch.uint8)
        cv = torch.randint(0, 256, (T, kvp), generator=g, device="cuda", dtype=torch.uint8)
        kn = (11.3 + 0.7 * torch.randn((T, Hk), generator=g, device="cuda")).to(torch.float16)
        vn = (11.3 + 0.7 * torch.randn((T, Hk), generator=g, device="cuda")).to(torch.float16)
        rot = kvcache.make_rotation().cuda()

        def launch():
            kvcache.launch_turbo_gqa_prefill_attention(out, q, ck, cv, kn, vn, rot, ws, T, T, H, Hk, D, H * D, Hk * D, kv_bits)
    else:
        ck = torch.randn((T, Hk * D), generator=g, device="cuda", dtype=torch.float16)
        cv = torch.randn((T, Hk * D), generator=g, device="cuda", dtype=torch.float16)

        def launch():
            kvcache.launch_gqa_prefill_attention(out, q, ck, cv, ws, T, T, H, Hk, D, H * D, Hk * D)
    if args.prompt_step:
        # the whole layer over the prompt: producers of q and k, T-token append, attention (prefill_chunked,
        # engine.cpp:2097-2146), as one call (1) or as the reference's sequence of launchers (2)
        k = torch.randn((T, Hk * D), generator=g, device="cuda", dtype=torch.float16)
        v = torch.randn((T, Hk * D), generator=g, device="cuda", dtype=torch.float16)
        qw = (1 + 0.1 * torch.randn(D, generator=g, device="cuda")).to(torch.float16)
        kw = (1 + 0.1 * torch.randn(D, generator=g, device="cuda")).to(torch.float16)
        ang = torch.arange(T, device="cuda", dtype=torch.float64)[:, None] * 1e6 ** (-2.0 * torch.arange(D // 2, device="cuda", dtype=torch.float64) / D)[None, :]
        ct, st = torch.cos(ang).to(torch.float16), torch.sin(ang).to(torch.float16)
        pos = torch.arange(T, device="cuda", dtype=torch.int32)
        q0, k0 = q.clone(), k.clone()
        attention_only = launch

        def launch():
            q.copy_(q0); k.copy_(k0)                     # the producers work in place (two copies: 50 MB at 8192 tokens)
            if args.prompt_step == 1:
                kvcache.tw_layer_prompt_step(out, q, k, v, pos, T, T, H, Hk, D, H * D, Hk * D, ck, cv, ws, kv_bits=kv_bits,
                                             k_norms=kn if kv_bits else None, v_norms=vn if kv_bits else None,
                                             rotation=rot if kv_bits else None, q_weight=qw, k_weight=kw, eps=1e-6,
                                             cos_table=ct, sin_table=st, rope_dim=D)
                return
            kvcache.launch_qk_norm_batch(q, k, qw, kw, H, Hk, D, T, 1e-6, H * D, Hk * D)
            kvcache.launch_rope_batch(q, k, ct, st, pos, T, T, H, Hk, D, H * D, Hk * D, D)
            if kv_bits:
                kvcache.launch_turbo_kv_quantize(ck, kn, k, rot, pos, T, T, Hk, D, Hk * D, kv_bits)
                kvcache.launch_turbo_kv_quantize(cv, vn, v, rot, pos, T, T, Hk, D, Hk * D, kv_bits)
            else:
                ck.copy_(k); cv.copy_(v)
            attention_only()
    for _ in range(max(args.warmup, 1)):
        launch()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        launch()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    flop = 4.0 * D * H * T * (T + 1) / 2
    tflops = flop / (ms * 1e-3) * 1e-12
    result = {
        "metric": "prefill-attn prompt tokens/s (one layer)", "value": T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": max(args.warmup, 1), "ms_per_step": ms, "higher_is_better": True,
        "dtype": "f16-operand MFMA, f32 accumulate" if not kv_bits else DTYPE[kv_bits], "data": "synthetic",
        "config": {"workload": f"causal prefill attention, one sequence, {T} tokens, {H} heads over {Hk} KV heads",
                   "kv_bits": kv_bits if kv_bits else 16, "variant": args.variant, "form": args.prefill_form,
                   "timed": ["the attention launch", "tw_layer_prompt_step: producers + T-token append + attention (+ 2 copies restoring q and k)",
                             "launch_qk_norm_batch, launch_rope_batch, 2 appends, the attention launch (+ 2 copies restoring q and k)"][args.prompt_step]},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": 2500.0, "unit": "TFLOP/s", "frac": tflops / 2500.0,
                     "flops_per_launch": flop, "traffic": None},
    }
    kvcache.set_prefill_form(0)
    if quiet:
        return result
    print(json.dumps(result))
    return result


def paged_bench(args):
    """The decode step over a paged cache: 16-token pages in one pool per layer, a per-sequence block table in
    random page order (shared by the layers), every layer = paged append of K and V + paged decode attention, then
    positions += 1; the step is captured in a graph and replayed.  Same metric and byte count as the contiguous
    run of the same workload; the roofline object is the context-scanning kernel's."""
    import torch
    from triebwerk_amd import _lib, kvcache
    w = dict(WORKLOADS[args.workload])
    kv_bits = w["kv_bits"] if args.kv_bits is None else args.kv_bits
    if kv_bits == 0:
        sys.exit("bench.py: --paged measures the compressed caches (--kv-bits 4 or 2)")
    for key, val in (("ctx", args.ctx), ("G", args.batch), ("L", args.layers)):
        if val is not None:
            w[key] = val
    L, H, Hk, G, D = w["L"], w["H"], w["Hk"], w["G"], 128
    K, W = args.steps, args.warmup
    kv_dim, q_dim, kvp = Hk * D, H * D, Hk * D * kv_bits // 8
    total_steps = W + K + max(1, min(K, 4096 // L, args.profile_steps or K)) + 2
    msl = (w["ctx"] + total_steps + 255) // 256 * 256
    pages_per_seq, n_pages = msl // 16, G * msl // 16
    lib = _lib.load()
    torch.cuda.set_device(0)
    kvcache.set_attention_variant(args.variant)
    kvcache.set_num_splits(args.nsplit)

    rng = np.random.Generator(np.random.Philox(3))            # the same lengths as the contiguous run
    if w["ragged"]:
        ctx0 = rng.integers(w["ragged"][0], w["ragged"][1] + 1, size=G).astype(np.int64)
    else:
        ctx0 = np.full(G, w["ctx"], np.int64)
    start_pos = np.maximum(ctx0 - 1 - W, 0).astype(np.int32)
    bt = np.random.Generator(np.random.Philox(4)).permutation(n_pages).astype(np.int32).reshape(G, pages_per_seq)
    g = torch.Generator(device="cuda"); g.manual_seed(1)
    pools = []
    for _ in range(L):
        pools.append((torch.randint(0, 256, (n_pages, 16, kvp), generator=g, device="cuda", dtype=torch.uint8),
                      torch.randint(0, 256, (n_pages, 16, kvp), generator=g, device="cuda", dtype=torch.uint8),
                      (11.3 + 0.7 * torch.randn((n_pages, 16, Hk), generator=g, device="cuda")).to(torch.float16),
                      (11.3 + 0.7 * torch.randn((n_pages, 16, Hk), generator=g, device="cuda")).to(torch.float16)))
    q = torch.randn((L, G, q_dim), generator=g, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, kv_dim), generator=g, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, kv_dim), generator=g, device="cuda", dtype=torch.float16)
    out = torch.zeros((L, G, q_dim), device="cuda", dtype=torch.float16)
    rot = kvcache.make_rotation().cuda()
    ws = torch.zeros(kvcache.attention_workspace_floats(G, H, msl), dtype=torch.float32, device="cuda")
    pos = torch.from_numpy(start_pos).cuda()
    d_bt = torch.from_numpy(bt).cuda()
    stream = torch.cuda.Stream()

    def layers():
        for l in range(L):
            ck, cv, kn, vn = pools[l]
            if args.launchers == "reference":      # the two calls: append, then attention (four launches)
                kvcache.tw_paged_turbo_kv_append_batch(ck, kn, cv, vn, k[l], v[l], rot, pos, d_bt, pages_per_seq, G, Hk, D,
                                                       kv_dim, kv_bits)
                kvcache.tw_paged_turbo_gqa_attention_batch(out[l], q[l], ck, cv, kn, vn, rot, ws, pos, d_bt, pages_per_seq,
                                                           msl, G, H, Hk, D, q_dim, kv_dim, kv_bits)
            else:                                  # the layer step in one call (three launches)
                kvcache.tw_paged_turbo_append_attention_batch(out[l], q[l], k[l], v[l], ck, cv, kn, vn, rot, ws, pos, d_bt,
                                                              pages_per_seq, msl, G, H, Hk, D, q_dim, kv_dim, kv_bits)
        pos.add_(1)

    use_graph = not args.no_graph
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        layers()                                             # warm-up step 1, eager
        if use_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                layers()
        step = graph.replay if use_graph else layers
        for _ in range(W - 1):
            step()
    torch.cuda.synchronize()
    pos_now = start_pos.astype(np.int64) + max(W, 1)
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        for _ in range(K):
            step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    n_tokens_timed = int(sum(int((pos_now + i + 1).sum()) for i in range(K)))
    pos_now = pos_now + K
    assert np.array_equal(pos.cpu().numpy().astype(np.int64), pos_now), "positions drifted"
    assert torch.isfinite(out.float()).all(), "non-finite attention output"
    step_bytes = algorithmic_bytes(n_tokens_timed, G * K, L, H, Hk, kv_bits, with_append=True) / K
    step_gbs = step_bytes / (elapsed / K) * 1e-9

    Kp = max(1, min(K, 4096 // L, args.profile_steps or K))
    lib.tw_kv_debug_profile_attention(1)
    with torch.cuda.stream(stream):
        for _ in range(Kp):
            layers()
    torch.cuda.synchronize()
    total_ms, launches = C.c_double(0), C.c_int(0)
    rc = lib.tw_kv_debug_profile_read(C.byref(total_ms), C.byref(launches))
    lib.tw_kv_debug_profile_attention(0)
    assert rc == 0 and launches.value == Kp * L, (rc, launches.value)
    scan_kernel_name = lib.tw_kv_debug_last_scan_kernel().decode()       # what those launches ran
    n_tokens_prof = int(sum(int((pos_now + i + 1).sum()) for i in range(Kp)))
    kern_ms = total_ms.value / launches.value
    launch_bytes = algorithmic_bytes(n_tokens_prof, G * Kp, L, H, Hk, kv_bits, with_append=False) / (Kp * L)
    achieved = launch_bytes / (kern_ms * 1e-3) * 1e-9
    del pools, q, k, v, ws
    torch.cuda.empty_cache()
    return {
        "metric": "decode-attn tokens/s", "value": G * K / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": elapsed / K * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DTYPE[kv_bits], "data": "synthetic",
        "config": {"workload": f"{args.workload}: {w['desc']}, paged cache: 16-token pages, block table in random page order",
                   "kv_bits": kv_bits, "layers": L, "num_heads": H, "num_kv_heads": Hk, "head_dim": D, "batch": G,
                   "pages": n_pages, "context_first_timed_step": [int(ctx0.min()), int(ctx0.max())],
                   "tokens_attended_per_step": n_tokens_timed / K, "hipgraph": use_graph,
                   "launches_per_layer": 4 if args.launchers == "reference" else 3,
                   "step": ("paged append K,V + paged decode attention for every layer (two calls, four launches), positions += 1"
                            if args.launchers == "reference" else
                            "tw_paged_turbo_append_attention_batch for every layer (three launches), positions += 1")},
        "step_algorithmic_GB": step_bytes * 1e-9, "step_achieved_GBps": step_gbs,
        "step_frac_of_hbm_peak": step_gbs / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "kernel": "paged decode attention (context scan), one launch per layer",
                     "kernel_name": scan_kernel_name,
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "launch_ms": kern_ms, "launch_algorithmic_MB": launch_bytes * 1e-6, "traffic": None},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 20; with --prefill, launches for about 0.4 s)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 3; with --prefill, a quarter of the steps)")
    ap.add_argument("--workload", default="target", choices=sorted(WORKLOADS))
    ap.add_argument("--kv-bits", type=int, default=None, choices=[0, 2, 4])
    ap.add_argument("--variant", type=int, default=0, help="0 auto, 1 vector-ALU kernel, 2 MFMA kernel")
    ap.add_argument("--nsplit", type=int, default=0)
    ap.add_argument("--one-launch", type=int, default=None, choices=[0, 1, 2, 3],
                    help="decode step of a compressed layer as one kernel: 0 by max_seq_len, 1 whenever possible, 2 never "
                         "(default: what the engine picks from the spread of the context lengths)")
    ap.add_argument("--fused-shape", default=None, metavar="HKW,SHARES",
                    help="force the one-launch step's KV heads per workgroup and workgroups per (sequence, head group); "
                         "0 = the library's choice")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--producers", default="none", choices=["none", "fused", "separate"],
                    help="also run QK RMSNorm + RoPE each layer: fused into the append, or as the reference's two "
                         "launches (not part of the metric's definition; off by default)")
    ap.add_argument("--ctx", type=int, default=None, help="override the workload's context length")
    ap.add_argument("--batch", type=int, default=None, help="override the workload's batch size")
    ap.add_argument("--layers", type=int, default=None, help="override the workload's layer count")
    ap.add_argument("--launchers", default="engine", choices=["engine", "reference"],
                    help="engine: one tw_layer_attention_step per layer (default); reference: only the launchers the "
                         "reference's forward_layer_batch calls (two appends + attention per layer), captured in a graph")
    ap.add_argument("--headline-only", action="store_true",
                    help="default run: skip the other two cache widths (per_kv_bits)")
    ap.add_argument("--csrc-digest", action="store_true", help="print the digest of the kernel sources and exit")
    ap.add_argument("--paged", action="store_true",
                    help="the same step over a paged cache (16-token pages, block table in random page order) through "
                         "the tw_paged_* entry points; compressed caches only")
    ap.add_argument("--max-seq-len", type=int, default=None,
                    help="the engine's max_seq_len (rows per sequence in every cache array); default: context + steps, rounded up to 256")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="only run a plain device-to-device copy of this many MiB five times (reference for the "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    ap.add_argument("--prompt-step", type=int, default=0, choices=[0, 1, 2],
                    help="with --prefill: 0 time the attention launch alone, 1 the whole layer over the prompt through "
                         "tw_layer_prompt_step (QK norm, RoPE, T-token append, attention), 2 the same as the reference's "
                         "sequence of launchers")
    ap.add_argument("--profile-steps", type=int, default=None,
                    help="eager steps after the timed region whose scan launches are timed one by one with HIP events "
                         "(default: as many as --steps, at most 4096 launches)")
    ap.add_argument("--per-config", action="store_true",
                    help="also measure the BASELINE configs 1-5 (and the reference's launchers at the target shape) with "
                         "few steps each and report them under per_config; the default run does this")
    ap.add_argument("--prefill-form", type=int, default=0,
                    help="with --prefill: force a form of the prompt kernel (tw_kv_debug_set_prefill_form; 0 = automatic)")
    ap.add_argument("--prefill", type=int, default=0, metavar="T",
                    help="instead of the decode step, time causal prefill attention over a T-token prompt of one "
                         "sequence (one layer's launch, the workload's head counts, --kv-bits cache) and exit")
    args = ap.parse_args()
    if args.prefill and args.steps is None:
        # The prompt kernels keep the matrix cores busy, and the GPU raises its clock only under sustained load of
        # that kind: 2 launches of the 8192-token fp16 kernel measure 0.32 ms each, 1000 launches 0.285 ms (MI355X).
        # The default burst is long enough to time the sustained rate, as a prompt of 28 layers would see it.
        args.steps = max(20, 4_000_000 // args.prefill)
        if args.warmup is None:
            args.warmup = args.steps // 4
    if args.steps is None:
        args.steps = 20
    if args.warmup is None:
        args.warmup = 3
    if args.csrc_digest:
        print(csrc_digest())
        return
    if args.prefill:
        prefill_bench(args)
        return
    if args.copy_calibration:
        import torch
        n = args.copy_calibration << 20
        src = torch.full((n,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": n, "copies": 5, "reads_bytes_each": n, "writes_bytes_each": n}))
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; sharding is by sequence or KV head with no exchange "
              "inside the path, and is not implemented. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if args.paged:
        print(json.dumps(paged_bench(args)))
        return

    headline_bits = WORKLOADS[args.workload]["kv_bits"] if args.kv_bits is None else args.kv_bits
    result = decode_bench(args, headline_bits, with_probe=True)
    # The metric is quoted at kv_bits = 16 / 4 / 2: the default run measures the other two widths of the same
    # workload as well (same shapes and steps; no CPU leg, no read probe) and reports them beside the headline.
    default_run = (args.workload == "target" and args.kv_bits is None and args.ctx is None and args.batch is None and
                   args.layers is None and args.producers == "none" and args.launchers == "engine" and
                   not args.headline_only)
    if default_run:
        per = {str(headline_bits if headline_bits else 16): compact(result)}
        for bits in (2, 0):
            if bits != headline_bits:
                per[str(bits if bits else 16)] = compact(decode_bench(args, bits, with_probe=False))
        result["per_kv_bits"] = {k: per[k] for k in ("16", "4", "2") if k in per}
    if default_run or args.per_config:
        result["per_config"] = per_config(args)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(workload_of(args), headline_bits)
    print(json.dumps(result))


def compact(r):
    """The figures of one cache width for the per_kv_bits table."""
    return {"tokens_per_s": r["value"], "ms_per_step": r["ms_per_step"], "step_achieved_GBps": r["step_achieved_GBps"],
            "step_frac_of_hbm_peak": r["step_frac_of_hbm_peak"], "dtype": r["dtype"], "launches_per_layer": r["config"]["launches_per_layer"],
            "roofline": {k: r["roofline"][k] for k in ("kernel", "kernel_name", "achieved", "frac", "frac_timed_region", "frac_eager_kernel_events",
                                                       "launch_ms", "launch_ms_timed", "launch_algorithmic_MB", "traffic", "traffic_source")}}


# The BASELINE configs beside the headline: (key, workload, cache width or None for the workload's own, steps, warm-up,
# paged, launchers).  Few steps each -- config 5 runs its whole rollout of 512 decode steps, which is what it is --, no
# CPU leg, no read probe; the scan's launches are timed with events in at most 8 further eager steps.
PER_CONFIG_LEGS = (
    ("config1_fp16", "config1", None, 50, 5, False, "engine"),
    ("config2_tq4", "config2", None, 30, 5, False, "engine"),
    ("config3_tq4_contiguous", "config3", None, 10, 3, False, "engine"),
    ("config3_tq4_paged", "config3", None, 10, 3, True, "engine"),
    ("config3_tq2_paged", "config3", 2, 10, 3, True, "engine"),
    ("config4_tq2", "config4", None, 20, 3, False, "engine"),
    ("config5_rollout_tq4", "config5", 4, 512, 3, False, "engine"),
    ("config5_rollout_fp16", "config5", 0, 512, 3, False, "engine"),
    ("target_tq4_reference_launchers", "target", 4, 10, 3, False, "reference"),
)


def per_config(args):
    """Every leg of PER_CONFIG_LEGS as {ms_per_step, tokens_per_s, step_frac_of_hbm_peak, kernel_name, launch_ms, ...}."""
    import copy
    out = {}
    for key, workload, bits, steps, warmup, paged, launchers in PER_CONFIG_LEGS:
        a = copy.copy(args)
        a.workload, a.kv_bits, a.steps, a.warmup, a.paged, a.launchers = workload, bits, steps, warmup, paged, launchers
        a.ctx = a.batch = a.layers = a.max_seq_len = None
        a.profile_steps = 8
        kv_bits = WORKLOADS[workload]["kv_bits"] if bits is None else bits
        r = paged_bench(a) if paged else decode_bench(a, kv_bits, with_probe=False)
        out[key] = {"workload": r["config"]["workload"], "kv_bits": kv_bits if kv_bits else 16, "steps": r["steps"],
                    "ms_per_step": r["ms_per_step"], "tokens_per_s": r["value"],
                    "step_algorithmic_GB": r["step_algorithmic_GB"], "step_frac_of_hbm_peak": r["step_frac_of_hbm_peak"],
                    "launches_per_layer": r["config"]["launches_per_layer"],
                    "kernel_name": r["roofline"]["kernel_name"], "launch_ms": r["roofline"]["launch_ms"],
                    "launch_algorithmic_MB": r["roofline"]["launch_algorithmic_MB"], "launch_frac_of_hbm_peak": r["roofline"]["frac"]}
    # the prompt side of the cache (not a BASELINE config; bound by the matrix cores, not by HBM): causal attention over
    # an 8192-token prompt, one layer, the target workload's head counts, a sustained burst of launches
    for key, bits in (("prefill_8192_fp16", 0), ("prefill_8192_tq4", 4)):
        a = copy.copy(args)
        a.workload, a.kv_bits, a.prefill, a.prompt_step, a.prefill_form = "target", bits, 8192, 0, 0
        a.steps, a.warmup = 300, 100
        r = prefill_bench(a, quiet=True)
        out[key] = {"workload": r["config"]["workload"], "kv_bits": bits if bits else 16, "steps": r["steps"],
                    "ms_per_launch": r["ms_per_step"], "prompt_tokens_per_s": r["value"], "bound": "mfma",
                    "tflops": r["roofline"]["achieved"], "frac_of_dense_fp16_mfma_peak": r["roofline"]["frac"]}
    return out


def workload_of(args):
    w = dict(WORKLOADS[args.workload])
    overridden = []
    for key, val in (("ctx", args.ctx), ("G", args.batch), ("L", args.layers)):
        if val is not None:
            w[key] = val
            overridden.append(f"{key}={val}")
    if overridden:
        w["desc"] += " [override " + ",".join(overridden) + "]"
    w["overridden"] = bool(overridden)
    return w


def decode_bench(args, kv_bits, with_probe):
    """W warm-up steps, K timed steps (one hipGraph replay each), then the dominant kernel's launches timed
    one by one, for one cache width.  Returns the result dictionary (without the CPU leg)."""
    import torch
    from triebwerk_amd import Engine, _lib, kvcache

    w = workload_of(args)
    L, H, Hk, G, D = w["L"], w["H"], w["Hk"], w["G"], 128
    K, W = args.steps, args.warmup
    kv_dim, q_dim = Hk * D, H * D
    Kp = max(1, min(K, 4096 // L, args.profile_steps or K))   # eager steps whose scan launches are timed one by one
    total_steps = W + K + Kp + 2         # warm-up, graph-timed, kernel-timed (eager), slack
    msl = (w["ctx"] + total_steps + 255) // 256 * 256   # the engine's max_seq_len: context + room for the steps, rounded up
    if args.max_seq_len is not None:
        if args.max_seq_len < w["ctx"] + total_steps:
            sys.exit(f"bench.py: --max-seq-len {args.max_seq_len} leaves no room for context {w['ctx']} + {total_steps} steps")
        msl = args.max_seq_len
        w["desc"] += f" [max_seq_len={msl}]"

    lib = _lib.load()
    torch.cuda.set_device(0)
    kvcache.set_attention_variant(args.variant)
    if args.one_launch is not None:
        kvcache.set_decode_fused(args.one_launch)
    kvcache.set_num_splits(args.nsplit)
    if args.fused_shape:
        kvcache.set_fused_shape(*[int(x) for x in args.fused_shape.split(",")])
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    fill_caches(eng, L, kv_bits, seed=1)

    prefix_ms = None
    if w.get("prefix"):
        # The shared prompt: each group's first sequence gets the T prefix rows through the T-token
        # append (fp16: a row copy), the others get them by the engine's row broadcast
        # (the reference's prefill-once-then-broadcast, engine.cpp:2173-2214).
        T, group = w["prefix"]
        gp = torch.Generator(device="cuda"); gp.manual_seed(5)
        tok = torch.arange(T, dtype=torch.int32, device="cuda")
        rot = eng.rotation()
        # the prompts' K and V rows of every layer and group (what the projections would hand over), made before
        # the clock starts
        rows = [[(torch.randn((T, kv_dim), generator=gp, device="cuda", dtype=torch.float16),
                  torch.randn((T, kv_dim), generator=gp, device="cuda", dtype=torch.float16))
                 for _ in range(0, G, group)] for _ in range(L)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for l in range(L):
            ck, cv, kn, vn = eng.cache(l)
            for i, g0 in enumerate(range(0, G, group)):
                rk, rv = rows[l][i]
                if kv_bits == 0:
                    ck[g0, :T].copy_(rk); cv[g0, :T].copy_(rv)
                else:
                    kvcache.tw_turbo_kv_append_tokens(ck[g0], kn[g0], cv[g0], vn[g0], rk, rv, rot, tok, msl, T, Hk, D,
                                                      kv_dim, kv_bits)
        for g0 in range(0, G, group):
            eng.broadcast_prefix(g0, g0 + 1, min(g0 + group, G), T)
        torch.cuda.synchronize()
        prefix_ms = (time.perf_counter() - t0) * 1e3
        del rows

    rng = np.random.Generator(np.random.Philox(3))
    if w["ragged"]:
        ctx0 = rng.integers(w["ragged"][0], w["ragged"][1] + 1, size=G).astype(np.int64)
    else:
        ctx0 = np.full(G, w["ctx"], np.int64)
    # ctx0 = tokens attended by the first timed step (the appended one included)
    start_pos = (ctx0 - 1 - W).astype(np.int32)
    start_pos = np.maximum(start_pos, 0)
    eng.set_positions(start_pos)

    g = torch.Generator(device="cuda"); g.manual_seed(2)
    q = torch.randn((L, G, q_dim), generator=g, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, kv_dim), generator=g, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, kv_dim), generator=g, device="cuda", dtype=torch.float16)
    out = torch.zeros((L, G, q_dim), device="cuda", dtype=torch.float16)
    stream = torch.cuda.Stream()
    use_graph = not args.no_graph
    if args.producers != "none":
        gw = torch.Generator(device="cuda"); gw.manual_seed(7)
        q_norm = (1.0 + 0.1 * torch.randn((L, D), generator=gw, device="cuda")).to(torch.float16)
        k_norm = (1.0 + 0.1 * torch.randn((L, D), generator=gw, device="cuda")).to(torch.float16)
        inv = 1e6 ** (-torch.arange(0, D, 2, device="cuda", dtype=torch.float64) / D)
        ang = torch.arange(msl, device="cuda", dtype=torch.float64)[:, None] * inv[None, :]
        rope_cos, rope_sin = torch.cos(ang).to(torch.float16).contiguous(), torch.sin(ang).to(torch.float16).contiguous()
        eng.set_producers(1 if args.producers == "fused" else 2, q_norm, k_norm, 1e-6, False, rope_cos, rope_sin, D)

    if args.launchers == "reference":
        # forward_layer_batch's own calls and nothing else (engine.cpp:1979-2006, 2394): what an engine whose
        # source is left as it is gets from this library
        if args.producers != "none":
            sys.exit("bench.py: --launchers reference runs the append and attention launchers only")
        caches = [eng.cache(l) for l in range(L)]
        rot = eng.rotation()
        pos = eng.positions()
        scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")

        def layers():
            for l in range(L):
                ck, cv, kn, vn = caches[l]
                if kv_bits == 0:
                    kvcache.launch_kv_cache_write_batch(ck, cv, k[l], v[l], pos, msl, G, kv_dim)
                    kvcache.launch_gqa_attention_batch(out[l], q[l], ck, cv, scratch, pos, msl, G, H, Hk, D, q_dim, kv_dim)
                else:
                    kvcache.launch_turbo_kv_quantize_batch(ck, kn, k[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                    kvcache.launch_turbo_kv_quantize_batch(cv, vn, v[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                    kvcache.launch_turbo_gqa_attention_batch(out[l], q[l], ck, cv, kn, vn, rot, scratch, pos, msl, G, H, Hk, D,
                                                             q_dim, kv_dim, kv_bits)
            kvcache.launch_increment_positions(pos, G)

        eager_step = layers
        with torch.cuda.stream(stream):
            layers()                                         # first warm-up step, eager (loads the kernels)
            if use_graph:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    layers()
                graph.replay()                               # the captured step was recorded, not run
        torch.cuda.synchronize()
        step = graph.replay if use_graph else layers
        warm_done = 2 if use_graph else 1
    else:
        def step():
            eng.decode_step(q, k, v, out, use_graph=use_graph, stream=stream)

        def eager_step():
            eng.decode_step(q, k, v, out, use_graph=False, stream=stream)
        warm_done = 0

    with torch.cuda.stream(stream):
        for _ in range(max(W - warm_done, 0)):
            step()
    torch.cuda.synchronize()
    W_run = max(W, warm_done)
    pos_now = start_pos.astype(np.int64) + W_run
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fused_before = lib.tw_kv_decode_fused_launches()
    t0 = time.perf_counter()
    with torch.cuda.stream(stream):
        e0.record(stream)
        for _ in range(K):
            step()
        e1.record(stream)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    events_ms = e0.elapsed_time(e1)      # the same K steps as seen by events on the launch stream
    n_tokens_timed = int(sum(int((pos_now + i + 1).sum()) for i in range(K)))   # attended tokens, all steps
    pos_now = pos_now + K
    assert np.array_equal(eng.positions().cpu().numpy().astype(np.int64), pos_now), "positions drifted"
    assert torch.isfinite(out.float()).all(), "non-finite attention output"

    ms_per_step = elapsed / K * 1e3
    tokens_per_s = G * K / elapsed
    step_bytes = algorithmic_bytes(n_tokens_timed, G * K, L, H, Hk, kv_bits, with_append=True) / K
    step_gbs = step_bytes / (elapsed / K) * 1e-9

    # ---- dominant kernel alone: a pair of HIP events attached to every launch of the context-scanning
    # kernel on its stream (hipExtLaunchKernelGGL: start = the kernel begins, stop = it ends), in eager
    # steps that continue the same decode; the library holds 4096 event pairs
    fused_before = lib.tw_kv_decode_fused_launches()
    lib.tw_kv_debug_profile_attention(1)
    with torch.cuda.stream(stream):
        for _ in range(Kp):
            eager_step()
    torch.cuda.synchronize()
    total_ms, launches = C.c_double(0), C.c_int(0)
    rc = lib.tw_kv_debug_profile_read(C.byref(total_ms), C.byref(launches))
    lib.tw_kv_debug_profile_attention(0)
    assert rc == 0 and launches.value == Kp * L, (rc, launches.value)
    scan_kernel_name = lib.tw_kv_debug_last_scan_kernel().decode()       # what those launches ran
    n_tokens_prof = int(sum(int((pos_now + i + 1).sum()) for i in range(Kp)))
    eager_kern_ms = total_ms.value / launches.value
    # which kernel those launches were: the whole layer step in one launch (append included), or the scan of the
    # three-kernel path
    one_launch = lib.tw_kv_decode_fused_launches() - fused_before == Kp * L
    launch_bytes = algorithmic_bytes(n_tokens_prof, G * Kp, L, H, Hk, kv_bits, with_append=one_launch) / (Kp * L)
    frac_eager = launch_bytes / (eager_kern_ms * 1e-3) * 1e-9 / HBM_PEAK_GBS     # per-launch events, eager steps
    if one_launch and use_graph:
        # The layer step is this one kernel, so the timed region itself is K * L launches of it (plus K one-block
        # position increments): its average duration there, the launches `value` is made of, is the events' time
        # over the region divided by the launches.  (Launched one by one with events attached the same kernel
        # reads 1-2 % longer: a replayed graph overlaps one kernel's drain with the next one's start.)
        kern_ms = events_ms / (K * L)
        launch_bytes = algorithmic_bytes(n_tokens_timed, G * K, L, H, Hk, kv_bits, with_append=True) / (K * L)
        timed = (f"HIP events on the launch stream around the {K} graph-replayed steps of the timed region / ({K} x {L}) launches; "
                 "includes 1/L of a one-block positions += 1 kernel per launch")
    else:
        kern_ms = eager_kern_ms
        timed = (f"a pair of HIP events attached to each of {Kp * L} eager launches of the kernel on its stream, in steps that "
                 "continue the timed decode")
    achieved = launch_bytes / (kern_ms * 1e-3) * 1e-9
    if args.launchers == "reference":
        launches_per_layer = 3 if kv_bits == 0 else 5     # write + scan + merge | 2 appends + query rotation + scan + merge
    else:
        launches_per_layer = 1 if one_launch else (2 if kv_bits == 0 else 3)

    read_big = read_same = None
    if with_probe:
        # ---- what a plain contiguous read kernel reaches on this GPU: over 4 GiB, and over exactly the
        # scan's bytes per launch on memory not touched since (launch overheads included, as for the scan)
        probe = torch.empty(int(4 << 30), dtype=torch.uint8, device="cuda")
        probe.fill_(1)
        torch.cuda.synchronize()
        lib.tw_kv_measure_read_bandwidth.restype = C.c_double
        read_big = lib.tw_kv_measure_read_bandwidth(C.c_void_p(probe.data_ptr()), C.c_size_t(probe.numel()), 3,
                                                    C.c_void_p(stream.cuda_stream))
        nb = int(launch_bytes) // 16 * 16
        same, reps = 0.0, 0
        for off in range(0, probe.numel() - nb + 1, max(nb, 1) + (1 << 20)):
            same += lib.tw_kv_measure_read_bandwidth(C.c_void_p(probe.data_ptr() + off // 16 * 16), C.c_size_t(nb), 1,
                                                     C.c_void_p(stream.cuda_stream))
            reps += 1
            if reps == 6:
                break
        read_same = same / max(reps, 1)
        del probe

    traffic, traffic_source = (measured_traffic(args.workload, kv_bits, one_launch)
                               if not w["overridden"] and args.producers == "none" and args.launchers == "engine"
                               else (None, "none: not measured for this variation of the workload"))
    result = {
        "metric": "decode-attn tokens/s",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W_run,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": DTYPE[kv_bits],
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: {w['desc']}" + (f" [kv_bits={kv_bits}]" if kv_bits != WORKLOADS[args.workload]["kv_bits"] else ""),
            "kv_bits": kv_bits if kv_bits else 16,
            "layers": L, "num_heads": H, "num_kv_heads": Hk, "head_dim": D, "batch": G,
            "context_first_timed_step": [int(ctx0.min()), int(ctx0.max())],
            "tokens_attended_per_step": n_tokens_timed / K,
            "hipgraph": use_graph,
            "launchers": ("tw_layer_attention_step per layer (engine object)" if args.launchers == "engine" else
                          "the reference's own launchers only: " +
                          ("launch_kv_cache_write_batch + launch_gqa_attention_batch" if kv_bits == 0 else
                           "launch_turbo_kv_quantize_batch x2 + launch_turbo_gqa_attention_batch") + " per layer, launch_increment_positions"),
            "launches_per_layer": launches_per_layer,
            "step": ("append K,V + decode attention for every layer, positions += 1" if args.producers == "none" else
                     f"QK RMSNorm + RoPE ({args.producers}) + append K,V + decode attention for every layer, positions += 1"),
            **({"shared_prefix_tokens": w["prefix"][0], "prefix_append_and_broadcast_ms": prefix_ms} if w.get("prefix") else {}),
        },
        "step_algorithmic_GB": step_bytes * 1e-9,
        "step_achieved_GBps": step_gbs,
        "step_frac_of_hbm_peak": step_gbs / HBM_PEAK_GBS,
        "roofline": {
            "bound": "hbm",
            "kernel": ("decode step of a layer in one launch (append, query rotation, context scan, merge, rotate-back)"
                       if one_launch else "decode attention (context scan), one launch per layer"),
            "kernel_name": scan_kernel_name,
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            # the two readings of the same kernel, side by side: `frac` above is frac_timed_region where the layer is one
            # launch and the step is graph-replayed (the launches `value` is made of, back to back), else
            # frac_eager_kernel_events (a pair of events on each launch of eager steps)
            "frac_timed_region": (achieved / HBM_PEAK_GBS) if (one_launch and use_graph) else None,
            "frac_eager_kernel_events": frac_eager,
            "launch_ms": kern_ms,
            "launch_ms_timed": timed,
            "launch_ms_eager_events": eager_kern_ms,
            "launch_algorithmic_MB": launch_bytes * 1e-6,
            "plain_read_GBps_4GiB": read_big,
            "plain_read_GBps_same_bytes_per_launch": read_same,
            "traffic": traffic,
            "traffic_source": traffic_source,
        },
    }
    if args.producers != "none":
        eng.set_producers(0)
    del eng, q, k, v, out
    torch.cuda.empty_cache()
    return result


if __name__ == "__main__":
    main()
