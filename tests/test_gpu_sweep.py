"""GPU: seeded sweep over small random shapes of the whole chain - scatter two
batches, scores, attention output, H2O accumulate, evict, compact - against the numpy
restatement.  The shapes are drawn from everything the entry points accept (all four
schemes, 1-8 kv heads, 1-4 query heads per kv head, head sizes 64/128, every legal
group, fp32 and bf16 sources and queries, ragged and empty caches), so that indexing
that only holds for the benchmark shapes shows up here."""
import numpy as np
import pytest

import pikv_oracle as O
from test_gpu_read_evict import _check_compacted
from util import codes_np, kv_like, np_of, rng, to_dev

pytestmark = pytest.mark.gpu


def _draw(r, big):
    scheme = int(r.integers(0, 4))
    four = scheme in (O.Q_I4_ASYM, O.Q_I4_SYM)
    heads = int(r.choice([1, 2, 4, 8]))
    dh = int(r.choice([64, 128]))
    rep = int(r.choice([1, 2, 4]))
    D = heads * dh
    groups = [g for g in (32, 64, 128, 256, 512, 1024) if (g >= (32 if four else 16)) and
              ((g <= dh and dh % g == 0) or g == D)]
    if not four:
        groups += [16] if dh % 16 == 0 else []
    group = int(r.choice(sorted(set(groups))))
    n_caches = int(r.integers(1, 6))
    caps = [int(r.integers(1, 6000 if big else 260)) for _ in range(n_caches)]
    return scheme, heads, dh, rep, group, caps


@pytest.mark.parametrize("seed", range(64))
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
