#!/usr/bin/env python3
"""Benchmark of the routed, compressed KV-cache data path on one MI355X.

A step is one pass of the hot path over one prefill batch of the
"prefill compress-write" workload (hidden 4096, 8 experts top-2, capacity
factor 1.25, 32 heads x 128, bf16, batch 16 x seq 2048 = 32768 tokens, 1 % outlier
channels x20, int8 symmetric per token per head, 8 caches x 8192 slots):

    reset fill -> K1 fused router (+capacity slots)
               -> K2 fused quantise + scatter of K and V into the routed caches
               -> K3 gather + dequantise + QK^T scores over the 8 caches
               -> softmax-normalised H2O importance accumulation

Inputs are synthetic, seeded, and resident in HBM before the timed region.
Prints ONE JSON line.  `value` = tokens routed and cached per second over the
whole step; `roofline` is for the dominant kernel (K2), from HIP events recorded
around that kernel inside the timed steps (the other kernels' figures come from a
second pass, so that the timed steps carry two event records, not five); `cpu_baseline` times the C restatement
of the same step (oracle/pikv_oracle.c) on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "routed KV tokens/s (quant+scatter+gather+dequant), 1 MI355X; % HBM peak"
HBM_PEAK_GBPS = 8000.0


def profiled_traffic(kernel_prefixes, summary="prefill.md"):
    """HBM bytes per launch (fetched + written) of the named kernel(s), summed, as the rocprofv3
    --pmc runs of the builder recorded them - NOT measured in this run: read from the
    machine-readable block at the end of profiles/<summary> (written by bench_profile.py,
    counters scaled by a streaming probe of known traffic in the same run).  None when the
    summary is missing or lacks one of the kernels."""
    import re
    if isinstance(kernel_prefixes, str):
        kernel_prefixes = [kernel_prefixes]
    try:
        text = open(os.path.join(ROOT, "profiles", summary)).read()
        blob = json.loads(re.search(r"<!-- machine-readable: (.*) -->", text).group(1))
    except (OSError, AttributeError, ValueError):
        return None
    total = 0.0
    for prefix in kernel_prefixes:
        best = None
        for name, rec in blob.get("kernels", {}).items():
            if name.startswith(prefix) and rec.get("fetch_bytes") is not None and rec.get("write_bytes") is not None:
                if best is None or rec["calls"] > best["calls"]:
                    best = rec
        if best is None:
            return None
        total += float(best["fetch_bytes"] + best["write_bytes"])
    return total

WORKLOAD = dict(name="prefill compress-write", batch=16, seq=2048, hidden=4096, experts=8, top_k=2,
                capacity_factor=1.25, heads=32, head_dim=128, cache_slots=8192,
                quant="int8 symmetric per token per head", outlier_frac=0.01, outlier_scale=20.0,
                seed=1)


def make_inputs(torch, dev, w):
    g = torch.Generator(device="cpu").manual_seed(w["seed"])
    T, H, E = w["batch"] * w["seq"], w["hidden"], w["experts"]
    D = w["heads"] * w["head_dim"]
    gd = torch.Generator(device=dev).manual_seed(w["seed"])
    hidden = torch.randn(T, H, generator=gd, device=dev, dtype=torch.float32).to(torch.bfloat16)
    gate_w = (0.02 * torch.randn(E, H, generator=g)).to(dev).to(torch.bfloat16)
    n_out = max(1, int(D * w["outlier_frac"]))
    ch = torch.randperm(D, generator=g)[:n_out].to(dev)
    kv = []
    for _ in range(2):
        t = torch.randn(T, D, generator=gd, device=dev, dtype=torch.float32)
        t[:, ch] *= w["outlier_scale"]
        kv.append(t.to(torch.bfloat16))
    q = torch.randn(E, w["heads"], w["head_dim"], generator=gd, device=dev).to(torch.bfloat16)
    return hidden, gate_w, kv[0], kv[1], q


def cpu_baseline(torch, w, hidden, gate_w, k_src, v_src, q, reps=5):
    """Time the C restatement of the same step on the host (all of the batch)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import c_oracle as CO
    import pikv_oracle as O

    def bits(t):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)

    T = hidden.shape[0]
    E, k = w["experts"], w["top_k"]
    D = w["heads"] * w["head_dim"]
    xh, wh, kh, vh, qh = bits(hidden), bits(gate_w), bits(k_src), bits(v_src), bits(q)
    cap = O.compute_capacity(w["batch"], w["seq"], w["capacity_factor"], k, E)
    times = []
    for _ in range(reps):
        pool = CO.CPool([w["cache_slots"]] * E, D, w["head_dim"], O.Q_I8_SYM)
        t0 = time.perf_counter()
        _, _, idx, _ = CO.router(xh, wh, None, k)
        slot, count = CO.capacity_slots(idx, E, cap)
        pool.quant_scatter(kh, vh, idx, slot, k, now=1.0)
        pool.advance(count, cap)
        pool.scores_h2o(qh, w["heads"], w["heads"], w["head_dim"], 1.0 / w["head_dim"] ** 0.5,
                        now=1.0, want_scores=False)
        times.append(time.perf_counter() - t0)
    best = min(times)
    return {"value": T / best, "unit": "tokens/s", "cores": CO.threads(), "kind": "port",
            "sample": f"whole batch of {T} tokens, best of {reps} runs of oracle/pikv_oracle.c "
                      f"(OpenMP, {CO.threads()} threads), {best:.2f} s per step"}


def _median_ms(torch, fn, iters, warm=3, setup=None):
    """Median time of fn over `iters` calls; `setup` (state restoring, not part of the measured
    work) runs before every call, ahead of the opening event."""
    import time
    t_start = time.perf_counter()
    n_warm = 0
    # at least `warm` calls, and at least 30 ms of them: after a stretch of short launches the first
    # heavy kernels run measurably slower (the clocks come up over some milliseconds of load)
    while n_warm < warm or time.perf_counter() - t_start < 0.03:
        if setup:
            setup()
        fn()
        n_warm += 1
        if n_warm % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
           for _ in range(iters)]
    for a, b in evs:
        if setup:
            setup()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return ts[len(ts) // 2]


def _entry(ms, nbytes, traffic_bytes=None, **extra):
    """nbytes: the ALGORITHMIC bytes of the step (what the cache format and the step's inputs and
    outputs make unavoidable) - `GBps` and `hbm_frac` are on those alone.  traffic_bytes: what the
    implementation moves on top of them or instead (score matrices, exchange rows, re-reads),
    algorithmic bytes included; reported beside, never counted into hbm_frac."""
    d = {"ms": ms, "algorithmic_bytes": nbytes, "GBps": nbytes / (ms * 1e-3) / 1e9,
         "hbm_frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
    if traffic_bytes is not None:
        d["traffic_bytes"] = traffic_bytes
        d["traffic_GBps"] = traffic_bytes / (ms * 1e-3) / 1e9
    d.update(extra)
    return d


def hbm_ceiling(torch, dev, iters, nbytes=2 << 30):
    """Practical HBM rates of this machine with the library's own access pattern (16 bytes per
    lane, 1 KiB per wavefront, 8 accesses in flight per lane; bench_probe.hip, a library of its
    own beside this file): read only, write only, copy;
    plain and non-temporal stores; and a read stream in a tile loop without and with small stores.  Median of `iters` launches over `nbytes` (2 GiB: eight times
    the last-level cache), HIP events on the launch stream."""
    import bench_probe
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def run(mode, nt):
        st = torch.cuda.current_stream().cuda_stream
        return lambda: bench_probe.stream_probe(mode, src.data_ptr(), dst.data_ptr(), nbytes, nt, sink.data_ptr(), st)
    gb = nbytes / 1e9
    ms = {name: _median_ms(torch, run(mode, nt), iters)
          for name, mode, nt in (("read", 0, 0), ("write", 1, 0), ("write_nt", 1, 1), ("copy", 2, 0), ("copy_nt", 2, 1),
                                 ("tile_loop_read", 3, 0), ("tile_loop_read_with_stores", 4, 0))}
    del src, dst
    torch.cuda.empty_cache()
    return {"buffer_bytes": nbytes, "pattern": "16 B per lane, 1 KiB per wavefront, 8 in flight per lane",
            "read_GBps": gb / (ms["read"] * 1e-3), "write_GBps": gb / (ms["write"] * 1e-3),
            "write_nontemporal_GBps": gb / (ms["write_nt"] * 1e-3),
            "copy_GBps": 2 * gb / (ms["copy"] * 1e-3), "copy_nontemporal_GBps": 2 * gb / (ms["copy_nt"] * 1e-3),
            "tile_loop_read_GBps": gb / (ms["tile_loop_read"] * 1e-3),
            "tile_loop_read_with_6pct_stores_GBps": gb / (ms["tile_loop_read_with_stores"] * 1e-3),
            "ms": ms, "note": "copy rates count bytes read + bytes written; tile_loop_*: persistent blocks of eight "
                              "wavefronts reading 64 KiB tiles, two in flight per block (the loop shape of the one-pass "
                              "decode kernels), without and with 8 bytes stored per lane and tile (1/16 of the bytes read); "
                              "both rates count the bytes read only"}


def decode_read_workload(torch, ops, dev, iters):
    """Decode read path: 64 sequences x 32768 cached tokens, 8 KV heads (GQA from 32
    q heads) x 128, int4 asymmetric, group 32, fp16 scale/zero; H2O keeps 2048 heavy
    + 256 recent."""
    B, N, hkv, hq, dh = 64, 32768, 8, 32, 128
    D = hkv * dh
    g = torch.Generator(device=dev).manual_seed(2)
    pool = ops.CachePool([N] * B, hkv, dh, 32, ops.Q_I4_ASYM, dev, with_v=True)
    chunk = 4
    slot = torch.arange(N, device=dev, dtype=torch.int32).repeat(chunk)
    t_write = None
    for b0 in range(0, B, chunk):
        ks = torch.randn(chunk * N, D, generator=g, device=dev).to(torch.bfloat16)
        vs = torch.randn(chunk * N, D, generator=g, device=dev).to(torch.bfloat16)
        cid = torch.arange(b0, b0 + chunk, device=dev, dtype=torch.int32).repeat_interleave(N)
        if b0 == 0:
            t_write = _median_ms(torch, lambda: pool.quant_scatter(ks, vs, cid, slot, 1), iters)
        pool.quant_scatter(ks, vs, cid, slot, 1)
    pool.fill.fill_(N)
    q = torch.randn(B, hq, dh, generator=g, device=dev).to(torch.bfloat16)
    t_scores = _median_ms(torch, lambda: pool.scores(q, hq), iters)
    sc, tm, tsu = pool.scores(q, hq)
    t_h2o = _median_ms(torch, lambda: pool.h2o_accumulate(sc, tm, tsu, now=1.0), iters)
    t_att = _median_ms(torch, lambda: pool.attend_values(sc, pool.head_stats), iters)
    # one whole decode step: append the new token of every sequence, read the cache
    pool.fill.fill_(N - 1)
    new_k = torch.randn(B, D, generator=g, device=dev).to(torch.bfloat16)
    new_v = torch.randn(B, D, generator=g, device=dev).to(torch.bfloat16)
    seq_id = torch.arange(B, device=dev, dtype=torch.int32)
    zero_slot = torch.zeros(B, device=dev, dtype=torch.int32)
    one = torch.ones(B, device=dev, dtype=torch.int32)

    def decode_step():
        pool.quant_scatter(new_k, new_v, seq_id, zero_slot, 1, now=2.0)
        pool.advance(one)
        return pool.decode_attend(q, hq, now=2.0)     # scores + softmax + attention output + H2O accumulate
    # every step starts from caches of N - 1 rows: the reset is the bench's, not the step's
    t_step = _median_ms(torch, decode_step, iters, setup=lambda: pool.fill.fill_(N - 1))
    t_fused = _median_ms(torch, lambda: pool.decode_attend(q, hq, now=2.0), iters)
    t_fused_nb = _median_ms(torch, lambda: pool.decode_attend(q, hq, now=2.0, accumulate=False), iters)
    qf = q.float()
    t_fused_f32 = _median_ms(torch, lambda: pool.decode_attend(qf, hq, now=2.0), iters)
    t_fused_f32_nb = _median_ms(torch, lambda: pool.decode_attend(qf, hq, now=2.0, accumulate=False), iters)
    t_att_acc = _median_ms(torch, lambda: pool.attend_values(sc, pool.head_stats, accumulate=True, now=1.0), iters)
    pool.fill.fill_(N)
    # the plain gather + dequantise of the metric's name over this cache format: the K rows of 8 of the 64 sequences
    gd_rows = 8 * N
    t_gd32 = _median_ms(torch, lambda: pool.gather_dequant("k", row0=0, n=gd_rows), iters)
    t_gd16 = _median_ms(torch, lambda: pool.gather_dequant("k", row0=0, n=gd_rows, out_dtype=torch.bfloat16), iters)

    # Eviction with a realistic state every time: importance as accumulated above, timestamps =
    # token positions (the recent rows are the tail).  Without the restore the second call would
    # find its survivors already compacted at the front and move nothing.
    acc0 = pool.acc.clone()
    ts0 = torch.arange(N, device=dev, dtype=torch.float32).repeat(B)

    def restore():
        pool.fill.fill_(N)
        pool.acc.copy_(acc0)
        pool.ts.copy_(ts0)

    def evict():
        restore()
        pool.evict(0, heavy_ratio=1 / 16, recent_ratio=1 / 128)
    t_restore = _median_ms(torch, restore, iters)
    restore()
    t_sel = _median_ms(torch, lambda: pool.evict_select(0, heavy_ratio=1 / 16, recent_ratio=1 / 128), iters)
    t_evict = _median_ms(torch, evict, iters) - t_restore
    kept_rows = int(pool.fill.sum())
    rows = B * N
    k_bytes = rows * (D // 2 + (D // 32) * 4)          # codes + half scale / zero point of one of K, V
    q_bytes = B * hq * dh * 2
    acc_rw = rows * 8                                   # H2O accumulator read + written
    # algorithmic bytes of a decode step: K (1.36 GB with queries and accumulators) / K + V (2.70 GB)
    alg_k, alg_kv = k_bytes + q_bytes + acc_rw, 2 * k_bytes + q_bytes + acc_rw
    score_bytes = rows * hq * 4                         # the float score matrix of the public three-step form
    half_bytes = rows * hq * 2                          # the half-precision importance exchange of the one-pass form
    return {
        "workload": "decode read: 64 seq x 32768 cached tokens, 8 KV heads x 128 (32 q heads), int4 asym g32",
        "algorithmic_bytes_K": alg_k, "algorithmic_bytes_KV": alg_kv,
        "quant_scatter_i4": _entry(t_write, chunk * N * (2 * (D * 2 + D // 2 + (D // 32) * 4) + 8),
                                   rows=chunk * N),
        "gather_dequant_scores": _entry(t_scores, k_bytes + q_bytes, traffic_bytes=k_bytes + q_bytes + score_bytes,
                                        cached_tokens_per_s=rows / (t_scores * 1e-3),
                                        what="public float score matrix [cache, head, token] + tile statistics"),
        "gather_dequant_f32": _entry(t_gd32, gd_rows * (D // 2 + (D // 32) * 4) + gd_rows * D * 4, rows=gd_rows,
                                     what="pikv_gather_dequant, K rows of 8 sequences (262144 rows) -> float32: "
                                          "640 B read and 4096 B written per row"),
        "gather_dequant_bf16": _entry(t_gd16, gd_rows * (D // 2 + (D // 32) * 4) + gd_rows * D * 2, rows=gd_rows),
        "h2o_accumulate": _entry(t_h2o, acc_rw, traffic_bytes=score_bytes + acc_rw + rows * 4,
                                 what="reads the float score matrix; only the accumulators are algorithmic"),
        "attend_values": _entry(t_att, k_bytes, traffic_bytes=k_bytes + score_bytes),
        "attend_values_with_h2o": _entry(t_att_acc, k_bytes + acc_rw, traffic_bytes=k_bytes + score_bytes + acc_rw + rows * 4),
        "decode_attend": _entry(t_fused, alg_kv, traffic_bytes=alg_kv + 2 * half_bytes + rows * 4,
                                what="pikv_decode_attend: scores + softmax + attention output + H2O accumulate in "
                                     "one call (one pass over K and V; halves written and read back for the importance)"),
        "decode_attend_without_h2o": _entry(t_fused_nb, 2 * k_bytes + q_bytes,
                                            what="pikv_decode_attend with row_acc = row_ts = NULL: attention output only"),
        "decode_attend_f32_queries": _entry(t_fused_f32, alg_kv + q_bytes, traffic_bytes=alg_kv + q_bytes + 2 * half_bytes + rows * 4,
                                            what="the same call with float32 queries (the reference modules' own dtype): two bf16 limbs "
                                                 "per query element, decode_fused_i4w_kernel"),
        "decode_attend_f32_queries_without_h2o": _entry(t_fused_f32_nb, 2 * k_bytes + 2 * q_bytes),
        "decode_step": _entry(t_step, alg_kv, traffic_bytes=alg_kv + 2 * half_bytes + rows * 4,
                              what="append 1 token per sequence + pikv_decode_attend",
                              cached_tokens_per_s=rows / (t_step * 1e-3)),
        "roofline": {"bound": "hbm", "kernel": "decode_fused_i4_kernel<I4_ASYM, bookkeeping> + decode_finish_kernel + "
                                               "decode_importance_kernel (one pikv_decode_attend call)",
                     "achieved": alg_kv / (t_fused * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": alg_kv / (t_fused * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "traffic": profiled_traffic(["decode_fused_i4_kernel<2, true>", "decode_finish_kernel",
                                                  "decode_importance_kernel"], "decode_read.md"),
                     "traffic_source": "profiles/decode_read.md (builder's rocprofv3 --pmc runs, not this run)",
                     "algorithmic_bytes": alg_kv, "avg_launch_ms": t_fused,
                     "note": "time of the whole call (three launches) by HIP events on its stream"},
        "evict_select": _entry(t_sel, rows * 8 + rows * 5,
                               what="exact top-k selection, six dependent launches over 17 MB of keys: latency-bound, "
                                    "hbm_frac is not its measure"),
        "evict_select_plus_compact": {"ms": t_evict, "kept_rows": kept_rows,
                                      "moved_bytes": 2 * kept_rows * (2 * (D // 2 + (D // 32) * 4) + 8)},
    }


def decode_read_int8_workload(torch, ops, dev, iters):
    """Not one of the listed configurations: the decode read of the same 64 x 32768 cached
    tokens with the int8 per-token-per-head format of the write-side workloads, read by 8
    query heads per kv head (8 kv heads, 64 query heads) - the shape that takes the 8-bit
    matrix-core kernels."""
    B, N, hkv, hq, dh = 64, 32768, 8, 64, 128
    D = hkv * dh
    g = torch.Generator(device=dev).manual_seed(5)
    pool = ops.CachePool([N] * B, hkv, dh, dh, ops.Q_I8_SYM, dev, with_v=True)
    chunk = 4
    slot = torch.arange(N, device=dev, dtype=torch.int32).repeat(chunk)
    for b0 in range(0, B, chunk):
        ks = torch.randn(chunk * N, D, generator=g, device=dev).to(torch.bfloat16)
        vs = torch.randn(chunk * N, D, generator=g, device=dev).to(torch.bfloat16)
        cid = torch.arange(b0, b0 + chunk, device=dev, dtype=torch.int32).repeat_interleave(N)
        pool.quant_scatter(ks, vs, cid, slot, 1)
    pool.fill.fill_(N)
    q = torch.randn(B, hq, dh, generator=g, device=dev).to(torch.bfloat16)
    t_scores = _median_ms(torch, lambda: pool.scores(q, hq), iters)
    sc, tm, tsu = pool.scores(q, hq)
    pool.h2o_accumulate(sc, tm, tsu, now=1.0, stats_only=True)
    t_att = _median_ms(torch, lambda: pool.attend_values(sc, pool.head_stats, accumulate=True, now=1.0), iters)
    t_call = _median_ms(torch, lambda: pool.decode_attend(q, hq, now=2.0), iters)
    t_call_nb = _median_ms(torch, lambda: pool.decode_attend(q, hq, now=2.0, accumulate=False), iters)
    rows = B * N
    k_bytes = rows * (D + hkv * 4)
    q_bytes = B * hq * dh * 2
    half_bytes = rows * hq * 2                          # the half-precision importance exchange of the one-pass form
    return {
        "workload": "decode read, int8 per token per head: 64 seq x 32768 cached tokens, 8 KV heads x 128 (64 q heads)",
        "algorithmic_bytes_KV": 2 * k_bytes + q_bytes + rows * 8,
        "gather_dequant_scores": _entry(t_scores, k_bytes + q_bytes,
                                        traffic_bytes=k_bytes + q_bytes + rows * hq * 4),
        "attend_values_with_h2o": _entry(t_att, k_bytes + rows * 8, traffic_bytes=k_bytes + rows * hq * 4 + rows * 12),
        "decode_attend": _entry(t_call, 2 * k_bytes + q_bytes + rows * 8,
                                traffic_bytes=2 * k_bytes + q_bytes + 2 * half_bytes + rows * 12,
                                what="pikv_decode_attend: one pass over K and V (decode_fused_i8_kernel), halves written "
                                     "and read back for the H2O importance"),
        "decode_attend_without_h2o": _entry(t_call_nb, 2 * k_bytes + q_bytes,
                                            what="pikv_decode_attend with row_acc = row_ts = NULL: attention output only"),
    }


GEOMETRIES = [  # (model whose cache has this shape, kv heads, query heads, head_dim)
    ("llama-3-8b", 8, 32, 128), ("llama-3-70b", 8, 64, 128), ("llama-2-7b", 32, 32, 128), ("llama-2-13b", 40, 40, 128),
    ("qwen2.5-7b", 4, 28, 128), ("qwen2.5-3b", 2, 16, 128), ("qwen2.5-1.5b", 2, 12, 128), ("qwen2.5-0.5b", 2, 14, 64),
    ("qwen2.5-14b", 8, 40, 128), ("chatglm3-6b", 2, 32, 128), ("gpt2", 12, 12, 64), ("gpt2-medium", 16, 16, 64),
    ("gpt2-xl", 25, 25, 64), ("llama-3.2-1b", 8, 32, 64), ("llama-3.2-3b", 8, 24, 128), ("gemma-7b", 16, 16, 256),
    ("gemma-2-9b", 8, 16, 256), ("falcon-7b", 1, 71, 64), ("starcoder2-7b", 4, 36, 128), ("starcoder-15b", 1, 48, 128),
]


def geometries_workload(torch, ops, dev, iters):
    """pikv_decode_attend (the whole read of a decode step) over the cache geometries of published models:
    64 sequences, about 0.6 GB of K + V codes each way, 4-bit group-32 and 8-bit per-head caches, bf16
    queries.  Not part of the default run (`--workload geometries`); reported rates count the K and V bytes
    only, the score traffic of many query heads comes on top."""
    out, B = {}, 64
    for eight in (False, True):
        for name, hkv, hq, dh in GEOMETRIES:
            row = hkv * dh * (1.0 if eight else 0.5) + (hkv * 4 if eight else hkv * dh // 32 * 4)
            n_tok = int(min(32768, max(2048, (6e8 / B / row) // 512 * 512)))
            pool = ops.CachePool([n_tok] * B, hkv, dh, dh if eight else 32, ops.Q_I8_SYM if eight else ops.Q_I4_ASYM,
                                 dev, with_v=True)
            if eight:
                pool.k_codes.random_(-127, 127), pool.v_codes.random_(-127, 127)
            else:
                pool.k_codes.random_(0, 255), pool.v_codes.random_(0, 255)
                pool.k_zero.fill_(7.0), pool.v_zero.fill_(7.0)
            pool.k_scale.fill_(0.05), pool.v_scale.fill_(0.05)
            pool.fill.fill_(n_tok)
            q = torch.randn(B, hq, dh, device=dev).to(torch.bfloat16)
            t = _median_ms(torch, lambda: pool.decode_attend(q, hq, now=3.0), iters)
            kv_bytes = 2 * row * n_tok * B
            out[("int8 " if eight else "int4 ") + name] = {"kv_heads": hkv, "q_heads": hq, "head_dim": dh, "tokens": n_tok,
                                                         "ms": t, "kv_GBps": kv_bytes / t / 1e6}
            del pool
            torch.cuda.empty_cache()
    return out


def wide_routing_workload(torch, ops, dev, iters):
    """Wide MoE routing: 65536 tokens, hidden 7168, 64 experts top-8, Zipf(1.2) expert
    popularity, EPLB-style per-expert logit scale; int8 KV of 8 heads x 128 scattered
    to per-expert caches sized by the observed load."""
    T, H, E, k, heads, dh = 65536, 7168, 64, 8, 8, 128
    D = heads * dh
    gc = torch.Generator().manual_seed(3)
    g = torch.Generator(device=dev).manual_seed(3)
    hidden = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    gw = (0.02 * torch.randn(E, H, generator=gc)).to(dev).to(torch.bfloat16)
    rank = torch.randperm(E, generator=gc).float() + 1
    pop = rank ** -1.2
    bias = (pop / pop.sum()).log().to(dev)
    ks = torch.randn(T, D, generator=g, device=dev).to(torch.bfloat16)
    vs = torch.randn(T, D, generator=g, device=dev).to(torch.bfloat16)
    warm = ops.router_fused(hidden, gw, bias, top_k=k, capacity=T)
    load = warm.count.float() / warm.count.float().mean()
    ew = (1.0 / load.clamp_min(0.1)).clamp(0.5, 2.0)
    r = ops.router_fused(hidden, gw, bias, top_k=k, capacity=T, expert_scale=ew)
    counts = r.count.cpu().tolist()
    t_router = _median_ms(torch, lambda: ops.router_fused(hidden, gw, bias, top_k=k, capacity=T,
                                                          expert_scale=ew), iters)
    pool = ops.CachePool(counts, heads, dh, dh, ops.Q_I8_SYM, dev)
    t_q = _median_ms(torch, lambda: pool.quant_scatter(ks, vs, r.topk_idx, r.slot, k), iters)
    A = T * k
    return {
        "workload": "wide MoE routing: T=65536, hidden 7168, 64 experts top-8, Zipf 1.2, int8 KV 8x128",
        "router": _entry(t_router, T * H * 2 + T * E * 4 + A * 12, tflops=2.0 * T * H * E / (t_router * 1e-3) / 1e12,
                         tokens_per_s=T / (t_router * 1e-3)),
        "quant_scatter": _entry(t_q, T * 2 * D * 2 + A * (2 * D + 2 * heads * 4) + A * 8,
                                assignments_per_s=A / (t_q * 1e-3)),
        "expert_load_max_over_mean": max(counts) / (sum(counts) / E),
    }


def pyramid_workload(torch, ops, dev, iters):
    """Long-context pyramid compression: 131072 tokens, 32 layers, 8 KV heads x 128
    bf16; layer l keeps int(N*(1-0.75*l/31)) rows by score, then int8 per token per
    head."""
    from pikv_amd import pyramid
    L, N, heads, dh = 32, 131072, 8, 128
    D = heads * dh
    g = torch.Generator(device=dev).manual_seed(4)
    keep = pyramid.linear_keep_budget(N, L)
    ks = torch.empty(L, N, D, dtype=torch.bfloat16, device=dev)
    vs = torch.empty(L, N, D, dtype=torch.bfloat16, device=dev)
    for l in range(L):
        ks[l] = torch.randn(N, D, generator=g, device=dev).to(torch.bfloat16)
        vs[l] = torch.randn(N, D, generator=g, device=dev).to(torch.bfloat16)
    z = torch.randn(L, N, generator=g, device=dev)
    heavy = torch.rand(L, N, generator=g, device=dev) < 0.05
    sc = torch.softmax(z + 4.0 * heavy, dim=-1).contiguous()
    pc = pyramid.PyramidCache(keep, heads, dh, scheme=ops.Q_I8_SYM, device=dev)
    seg_base = torch.arange(L, dtype=torch.int64, device=dev) * N
    seg_len = torch.full((L,), N, dtype=torch.int32, device=dev)
    nk = torch.tensor(keep, dtype=torch.int32, device=dev)
    flat = sc.reshape(-1)
    t_sel = _median_ms(torch, lambda: ops.select_top_rows(flat, seg_base, seg_len, nk), iters)
    _, index, kept = ops.select_top_rows(flat, seg_base, seg_len, nk)
    pc.pool.fill.zero_()
    t_g = _median_ms(torch, lambda: pc.pool.quant_gather(ks, vs, seg_base, index, kept, max(keep),
                                                         src_score=flat), iters)
    rows = sum(keep)
    return {
        "workload": "pyramid compression: 32 layers x 131072 tokens, 8 heads x 128 bf16, budget 100% -> 25%, int8",
        "select_top_rows": _entry(t_sel, L * N * 4 + L * N * 5,
                                  what="exact top-k selection over small key arrays: latency-bound, hbm_frac is not its measure"),
        "quant_gather": _entry(t_g, rows * (2 * D * 2 + 2 * D + 2 * heads * 4), rows=rows,
                               rows_per_s=rows / (t_g * 1e-3)),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only-headline", action="store_true",
                    help="skip the per-kernel figures of the decode, wide-routing and pyramid workloads")
    ap.add_argument("--workload", default="all",
                    choices=["all", "prefill", "decode_read", "decode_read_int8_gqa8", "wide_routing", "pyramid", "geometries"],
                    help="run one workload only (for profiling; the bench line proper is the default, all)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only the streaming probes over 1 GiB (kernels of known traffic, to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from pikv_amd import ops
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        # five launches each of the read, write and copy probes over 1 GiB: kernels of exactly
        # known traffic for scaling FETCH_SIZE / WRITE_SIZE, and the ceilings as a JSON line
        import bench_probe
        n = 1 << 30
        src = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        st = torch.cuda.current_stream().cuda_stream
        for mode in (0, 1, 2):
            for _ in range(5):
                bench_probe.stream_probe(mode, src.data_ptr(), dst.data_ptr(), n, 0, None, st)
        torch.cuda.synchronize()
        del src, dst
        print(json.dumps({"calibrate_bytes_per_launch": n,
                          "kernels": {"stream_probe_kernel<0,false>": "reads n", "stream_probe_kernel<1,false>": "writes n",
                                      "stream_probe_kernel<2,false>": "reads n and writes n"},
                          "hbm_ceiling": hbm_ceiling(torch, dev, 10)}))
        return
    others = {"decode_read": decode_read_workload, "decode_read_int8_gqa8": decode_read_int8_workload,
              "wide_routing": wide_routing_workload, "pyramid": pyramid_workload}
    if args.workload in others or args.workload == "geometries":
        it = max(5, min(args.steps, 20))
        fn = geometries_workload if args.workload == "geometries" else others[args.workload]
        print(json.dumps({"workload_only": args.workload, "hbm_ceiling": hbm_ceiling(torch, dev, 10),
                          args.workload: fn(torch, ops, dev, it)}))
        return
    w = WORKLOAD
    T, E, k = w["batch"] * w["seq"], w["experts"], w["top_k"]
    heads, dh = w["heads"], w["head_dim"]
    D = heads * dh
    hidden, gate_w, k_src, v_src, q = make_inputs(torch, dev, w)
    cap = int(w["batch"] * w["seq"] * w["capacity_factor"] * k / E)
    pool = ops.CachePool([w["cache_slots"]] * E, heads, dh, dh, ops.Q_I8_SYM, dev)

    def step(ev=None, now=1.0, all_events=False):
        """ev: 5 events.  In the timed steps only the pair around the quantise+scatter
        launch is recorded (the roofline kernel); the separate per-kernel pass records all."""
        pool.fill.zero_()
        if ev and all_events: ev[0].record()
        r = ops.router_fused(hidden, gate_w, top_k=k, capacity=cap)
        if ev: ev[1].record()
        pool.quant_scatter(k_src, v_src, r.topk_idx, r.slot, k, now=now)
        if ev: ev[2].record()
        pool.advance(r.count, cap)
        scores, tmax, tsum = pool.scores(q, heads)
        if ev and all_events: ev[3].record()
        pool.h2o_accumulate(scores, tmax, tsum, now=now)
        if ev and all_events: ev[4].record()
        return r

    # The streaming probes run first: their figures belong to the same line, and the timed steps then
    # start on a machine that has been under load for some tens of milliseconds - as it is in a
    # serving loop - instead of on clocks that are still coming up after start-up.
    ceiling = hbm_ceiling(torch, dev, 10)
    for i in range(args.warmup):
        r = step()
    torch.cuda.synchronize()
    kept = int(pool.fill.sum().item())
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(events[i], now=float(i + 2))
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    t_quant = sum(ev[1].elapsed_time(ev[2]) for ev in events) / len(events)
    # per-kernel figures of the other launches: a second, untimed pass with all events
    for i in range(args.steps):
        step(events[i], now=float(i + 2), all_events=True)
    torch.cuda.synchronize()

    def avg(a, b):
        return sum(ev[a].elapsed_time(ev[b]) for ev in events) / len(events)

    t_router, t_scores, t_h2o = avg(0, 1), avg(2, 3), avg(3, 4)
    # the plain gather + dequantise of the metric's name (pikv_gather_dequant): every K row the step cached,
    # to float32 and to bf16
    n_rows = pool.rows
    t_gd32 = _median_ms(torch, lambda: pool.gather_dequant("k"), max(5, min(args.steps, 20)))
    t_gd16 = _median_ms(torch, lambda: pool.gather_dequant("k", out_dtype=torch.bfloat16), max(5, min(args.steps, 20)))
    A = T * k
    # algorithmic bytes of one launch
    b_quant = T * 2 * D * 2 + kept * (2 * D + 2 * heads * 4) + A * 8
    b_router = T * w["hidden"] * 2 + T * E * 4 + A * 12
    b_scores = kept * (D + heads * 4) + kept * heads * 4
    b_h2o = kept * heads * 4 + kept * 8
    gbps = lambda b, ms: b / (ms * 1e-3) / 1e9
    out = {
        "metric": METRIC, "value": T / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "prefill compress-write: T=32768 (16x2048), hidden 4096, 8 experts top-2 "
                               "cf 1.25, 32 heads x 128 bf16, int8 sym per token per head, 8 caches x 8192 slots",
                   "kept_assignments": kept, "assignments": A},
        "roofline": {"bound": "hbm", "kernel": "quant_scatter_kernel<I8_SYM,bf16>",
                     "achieved": gbps(b_quant, t_quant), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": gbps(b_quant, t_quant) / HBM_PEAK_GBPS,
                     "traffic": profiled_traffic("quant_scatter_kernel<0, 1, 2, true>"),
                     "traffic_source": "profiles/prefill.md (builder's rocprofv3 --pmc runs, not this run)",
                     "algorithmic_bytes": b_quant, "avg_launch_ms": t_quant},
        "kernels": {
            "router": {"ms": t_router, "GBps": gbps(b_router, t_router)},
            "quant_scatter": {"ms": t_quant, "GBps": gbps(b_quant, t_quant),
                              "tokens_per_s": T / (t_quant * 1e-3)},
            "scores": {"ms": t_scores, "GBps": gbps(b_scores, t_scores),
                       "cached_token_reads_per_s": kept / (t_scores * 1e-3)},
            "h2o_accumulate": {"ms": t_h2o, "GBps": gbps(b_h2o, t_h2o)},
            "gather_dequant_f32": _entry(t_gd32, n_rows * (D + heads * 4) + n_rows * D * 4, rows=n_rows,
                                         cached_tokens_per_s=n_rows / (t_gd32 * 1e-3),
                                         what="pikv_gather_dequant over all 65536 slots of the 8 caches, K plane -> float32"),
            "gather_dequant_bf16": _entry(t_gd16, n_rows * (D + heads * 4) + n_rows * D * 2, rows=n_rows,
                                          cached_tokens_per_s=n_rows / (t_gd16 * 1e-3)),
        },
    }
    out["hbm_ceiling"] = ceiling
    if not args.only_headline and args.workload == "all":
        it = max(5, min(args.steps, 20))
        out["other_workloads"] = {}
        for name, fn in others.items():
            out["other_workloads"][name] = fn(torch, ops, dev, it)
            torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, w, hidden, gate_w, k_src, v_src, q)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
