"""GPU: seeded sweep over small random shapes of the whole chain - scatter two
batches, scores, attention output, H2O accumulate, evict, compact - against the numpy
restatement.  The shapes are drawn from everything the entry points accept (all four
schemes, 1-8 kv heads, 1-8 query heads per kv head, head sizes 64/128, every legal
group, fp32 and bf16 sources and queries, ragged and empty caches), so that indexing
that only holds for the benchmark shapes shows up here."""
import os

import numpy as np
import pytest

import pikv_oracle as O
from test_gpu_read_evict import _check_compacted
from util import codes_np, kv_like, np_of, rng, to_dev

pytestmark = pytest.mark.gpu

# number of seeds of the widest sweep (the others scale with it); raise it for a longer soak
SEEDS = int(os.environ.get("PIKV_SWEEP_SEEDS", "64"))


def _draw(r, big):
    scheme = int(r.integers(0, 4))
    four = scheme in (O.Q_I4_ASYM, O.Q_I4_SYM)
    heads = int(r.choice([1, 2, 4, 8]))
    dh = int(r.choice([64, 128]))
    rep = int(r.choice([1, 2, 4, 8]))
    D = heads * dh
    groups = [g for g in (32, 64, 128, 256, 512, 1024) if (g >= (32 if four else 16)) and
              ((g <= dh and dh % g == 0) or g == D)]
    if not four:
        groups += [16] if dh % 16 == 0 else []
    group = int(r.choice(sorted(set(groups))))
    n_caches = int(r.integers(1, 6))
    caps = [int(r.integers(1, 6000 if big else 260)) for _ in range(n_caches)]
    return scheme, heads, dh, rep, group, caps


@pytest.mark.parametrize("seed", range(SEEDS))
def test_random_shape_chain(dev, seed):
    from pikv_amd import ops
    r = rng(1000 + seed)
    big = seed % 4 == 3     # caches that span several score tiles and attention token ranges
    scheme, heads, dh, rep, group, caps = _draw(r, big)
    hq, D, E = heads * rep, heads * dh, len(caps)
    src_dt = "bf16" if seed % 2 else "f32"
    q_dt = "bf16" if (seed // 2) % 2 else "f32"
    print(f"seed {seed}: scheme {scheme} heads {heads} dh {dh} rep {rep} group {group} caps {caps} "
          f"src {src_dt} q {q_dt}", flush=True)
    pool = ops.CachePool(caps, heads, dh, group, scheme, dev, with_v=True)
    ref = O.CachePool(caps, D, group, scheme)
    k = min(2, E)
    for step in range(2):
        T = int(r.integers(1, 5000 if big else 200))
        capacity = int(r.integers(1, 2 * T))
        idx = np.stack([r.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        slot, count = O.capacity_slots(idx, E, capacity)
        ks, vs = kv_like(r, T, D, dtype=src_dt), kv_like(r, T, D, dtype=src_dt)
        pool.quant_scatter(to_dev(ks, dev, src_dt), to_dev(vs, dev, src_dt), to_dev(idx, dev), to_dev(slot, dev),
                           k, now=float(step))
        pool.advance(to_dev(count, dev), capacity)
        ref.quant_scatter(ks, vs, idx, slot, k, now=float(step))
        ref.advance(count, capacity)
    assert np.array_equal(np_of(pool.fill), ref.fill)
    lens = [int(x) for x in ref.fill]
    for c in range(E):
        rows = ref.valid_rows(c)
        assert np.array_equal(codes_np(pool.k_codes, scheme)[rows], ref.k_codes[rows]), c
        assert np.array_equal(codes_np(pool.v_codes, scheme)[rows], ref.v_codes[rows]), c
        assert np.array_equal(np_of(pool.k_scale)[rows].astype(np.float32), ref.k_scale[rows]), c
        if pool.k_zero is not None:
            assert np.array_equal(np_of(pool.v_zero)[rows].astype(np.float32), ref.v_zero[rows]), c

    # read: scores, attention output, importance
    q = r.standard_normal((E, hq, dh)).astype(np.float32)
    if q_dt == "bf16":
        q = O.bf16_round(q)
    scale_qk = 1.0 / np.sqrt(dh)
    scores, tmax, tsum = pool.scores(to_dev(q, dev, q_dt), hq, scale_qk)
    pool.h2o_accumulate(scores, tmax, tsum, now=9.0, stats_only=True)
    out = np_of(pool.attend_values(scores, pool.head_stats, accumulate=True, now=9.0))
    sc = np_of(scores)
    for c, L in enumerate(lens):
        if L == 0:
            assert not out[c].any()
            continue
        rows = ref.valid_rows(c)
        k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
        s_ref = O.attention_scores(q[c], k_hat, heads, scale_qk)
        rms = np.sqrt((s_ref.astype(np.float64) ** 2).mean()) + 1e-12
        assert np.abs(sc[c, :, :L] - s_ref).max() <= 1e-3 * rms, c
        p_ref, imp_ref = O.h2o_importance(s_ref)
        want = O.attend_values(p_ref, v_hat, heads)
        orms = np.sqrt((want.astype(np.float64) ** 2).mean()) + 1e-12
        assert np.abs(out[c] - want).max() <= 2e-3 * orms, (c, np.abs(out[c] - want).max(), orms)
        O.h2o_accumulate(ref.acc, ref.ts, rows, imp_ref, 9.0)
    assert np.allclose(np_of(pool.acc), ref.acc, rtol=1e-3, atol=1e-6)
    assert np.array_equal(np_of(pool.ts), ref.ts)

    # evict on exact-tie-rich state, compact
    acc = (np.round(r.random(pool.rows) * 8) / 8).astype(np.float32)
    ts = r.integers(0, 6, pool.rows).astype(np.float32)
    ref.acc[:], ref.ts[:] = acc, ts
    pool.acc.copy_(to_dev(acc, dev))
    pool.ts.copy_(to_dev(ts, dev))
    if seed % 3 == 0:
        ne = np.array([int(r.integers(0, L + 2)) for L in lens], dtype=np.int32)
        pool.evict(ops.EVICT_LRU, n_evict=to_dev(ne, dev))
        keeps = [O.lru_keep(ref.ts[ref.valid_rows(c)], int(ne[c])) if L else np.zeros(0, dtype=bool)
                 for c, L in enumerate(lens)]
    else:
        nh = np.array([int(r.integers(0, L + 2)) for L in lens], dtype=np.int32)
        nr = np.array([int(r.integers(0, L + 2)) for L in lens], dtype=np.int32)
        pool.evict(ops.EVICT_H2O, n_heavy=to_dev(nh, dev), n_recent=to_dev(nr, dev))
        keeps = [O.h2o_keep(ref.acc[ref.valid_rows(c)], ref.ts[ref.valid_rows(c)], int(nh[c]), int(nr[c]))
                 if L else np.zeros(0, dtype=bool) for c, L in enumerate(lens)]
    _check_compacted(pool, ref, scheme, keeps)


@pytest.mark.parametrize("seed", range(SEEDS // 2))
def test_random_shape_router(dev, seed):
    """Fused gate projection + tail over random T, H (multiples of 8), E <= 64, k <= 8, both
    dtypes, with and without bias / scaling / mask / capacity."""
    from pikv_amd import ops
    r = rng(2000 + seed)
    T = int(r.integers(1, 700))
    H = 8 * int(r.integers(1, 200))
    E = int(r.integers(1, 65))
    k = int(r.integers(1, min(E, 8) + 1))
    dtype = "bf16" if seed % 2 else "f32"
    print(f"seed {seed}: T {T} H {H} E {E} k {k} {dtype}", flush=True)
    x = r.standard_normal((T, H)).astype(np.float32)
    w = (r.standard_normal((E, H)) / np.sqrt(H)).astype(np.float32)
    if dtype == "bf16":
        x, w = O.bf16_round(x), O.bf16_round(w)
    b = (0.1 * r.standard_normal(E)).astype(np.float32) if seed % 3 else None
    kw, okw = {}, {}
    if seed % 4 == 1:
        scale = (0.5 + r.random(E)).astype(np.float32)
        kw.update(temperature=0.8, expert_scale=to_dev(scale, dev))
        okw.update(temperature=0.8, expert_scale=scale)
    if seed % 4 == 2:
        mask = (r.random(E) > 0.3).astype(np.float32)
        if mask.sum() < k:
            mask[:] = 1
        kw.update(expert_mask=to_dev(mask, dev))
        okw.update(expert_mask=mask)
    cap = int(r.integers(1, 2 * T + 2)) if seed % 5 else None
    out = ops.router_fused(to_dev(x, dev, dtype), to_dev(w, dev, dtype), None if b is None else to_dev(b, dev),
                           top_k=k, capacity=cap, return_logits=True, **kw)
    lg = (x.astype(np.float64) @ w.astype(np.float64).T + (0 if b is None else b)).astype(np.float32)
    # the returned logits are the scaled / masked ones (what the softmax sees)
    if "temperature" in okw:
        lg = lg / np.float32(okw["temperature"]) * okw["expert_scale"]
    if "expert_mask" in okw:
        lg = lg + (np.float32(1) - okw["expert_mask"]) * np.float32(-1e9)
    assert np.allclose(np_of(out.logits), lg, atol=4e-5 * np.sqrt(H), rtol=1e-5)
    # everything after the projection is exact arithmetic on the logits the GPU produced
    probs, idx, wts, _ = O.router_tail(np_of(out.logits), k)
    assert np.array_equal(np_of(out.topk_idx), idx)
    assert np.allclose(np_of(out.probs), probs, atol=2e-6, rtol=1e-5)
    assert np.allclose(np_of(out.topk_w), wts, atol=2e-6, rtol=1e-5)
    if cap is not None:
        slot, count = O.capacity_slots(idx, E, cap)
        assert np.array_equal(np_of(out.slot), slot)
        assert np.array_equal(np_of(out.count), count)


@pytest.mark.parametrize("seed", range(SEEDS // 2))
def test_random_shape_quantize_dequantize(dev, seed):
    """quantize_rows / dequantize_rows (plain and through a row list) for random widths and groups."""
    import torch
    from pikv_amd import ops
    r = rng(3000 + seed)
    scheme = int(r.integers(0, 4))
    four = scheme in (O.Q_I4_ASYM, O.Q_I4_SYM)
    group = int(r.choice([32, 64, 128, 256, 512, 1024, 2048] if four else [16, 32, 64, 128, 256, 512, 1024]))
    D = group * int(r.integers(1, 9))
    n = int(r.integers(1, 400))
    dtype = "bf16" if seed % 2 else "f32"
    print(f"seed {seed}: scheme {scheme} D {D} group {group} n {n} {dtype}", flush=True)
    x = kv_like(r, n, D, dtype=dtype)
    try:
        codes, scale, zero = ops.quantize_rows(to_dev(x, dev, dtype), group, scheme)
    except ValueError as e:      # widths the entry point states it does not take
        pytest.skip(str(e))
    q_ref, s_ref, z_ref = O.quantize_groups(x, group, scheme)
    assert np.array_equal(codes_np(codes, scheme), q_ref)
    assert np.array_equal(np_of(scale).astype(np.float32), s_ref)
    if zero is not None:
        assert np.array_equal(np_of(zero).astype(np.float32), z_ref)
    dq_ref = O.dequantize_groups(q_ref, s_ref, z_ref, group)
    assert np.array_equal(np_of(ops.dequantize_rows(codes, scale, zero, group, scheme)), dq_ref, equal_nan=True)
    rows = r.integers(0, n, size=int(r.integers(1, 50))).astype(np.int64)
    got = ops.dequantize_rows(codes, scale, zero, group, scheme, out_dtype=torch.bfloat16, rows=to_dev(rows, dev))
    assert np.array_equal(np_of(got), O.bf16_round(dq_ref[rows]), equal_nan=True)


@pytest.mark.parametrize("seed", range(SEEDS // 4))
def test_random_shape_select_and_gather(dev, seed):
    """select_top_rows + quant_gather (the pyramid path) over random segment lengths and budgets."""
    from pikv_amd import ops
    r = rng(4000 + seed)
    L = int(r.integers(1, 7))
    n = int(r.integers(1, 9000 if seed % 4 == 3 else 300))
    heads, dh = int(r.choice([1, 2, 4])), int(r.choice([64, 128]))
    D = heads * dh
    scheme = int(r.integers(0, 4))
    group = dh if scheme in (O.Q_I8_SYM, O.Q_I8_ASYM) else 32
    lens = np.array([int(r.integers(0, n + 1)) for _ in range(L)], dtype=np.int32)
    keep = np.array([int(r.integers(0, l + 2)) for l in lens], dtype=np.int32)
    print(f"seed {seed}: L {L} n {n} D {D} scheme {scheme} lens {lens} keep {keep}", flush=True)
    sc = (np.round(r.random((L, n)) * 16) / 16).astype(np.float32)
    seg_base = np.arange(L, dtype=np.int64) * n
    flag, index, kept = ops.select_top_rows(to_dev(sc.reshape(-1), dev), to_dev(seg_base, dev), to_dev(lens, dev),
                                            to_dev(keep, dev), max_len=n)
    want_kept = np.minimum(keep, lens)
    assert np.array_equal(np_of(kept), want_kept)
    ks, vs = kv_like(r, L * n, D, dtype="bf16"), kv_like(r, L * n, D, dtype="bf16")
    caps = [int(max(1, k_ - (1 if seed % 2 else 0))) for k_ in want_kept]     # some caches one row short
    pool = ops.CachePool(caps, heads, dh, group, scheme, dev, with_v=True)
    pool.quant_gather(to_dev(ks, dev, "bf16"), to_dev(vs, dev, "bf16"), to_dev(seg_base, dev), index, kept,
                      int(n), src_score=to_dev(sc.reshape(-1), dev), now=2.0)
    base = np_of(pool.row_base)
    for l in range(L):
        want = np.nonzero(O.h2o_keep(sc[l, :lens[l]], sc[l, :lens[l]], int(keep[l]), 0))[0]
        assert np.array_equal(np_of(index)[l * n:l * n + want.size], want), l
        m = min(want.size, caps[l])
        rows = slice(int(base[l]), int(base[l]) + m)
        for src, codes, scale in ((ks, pool.k_codes, pool.k_scale), (vs, pool.v_codes, pool.v_scale)):
            q, s, _ = O.quantize_groups(src[l * n + want[:m]], group, scheme)
            assert np.array_equal(codes_np(codes, scheme)[rows], q), l
            assert np.array_equal(np_of(scale)[rows].astype(np.float32), s), l
        assert np.array_equal(np_of(pool.acc)[rows], sc[l, want[:m]])
