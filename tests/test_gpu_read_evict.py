"""GPU parity: K3 (scores over the compressed cache, softmax statistics, H2O
accumulation) and K4 (eviction top-k, stable in-place compaction) through the
C ABI against the numpy restatement.

Scores and importance are float results: tolerance 1e-3 relative to the
root-mean-square score of the row (float32 path; the bound stated for this
path), checked against a float64 evaluation of the same formula on the same
dequantised codes.  Eviction sets, survivor order, compacted bytes and fill
counts are bit-exact, ties broken towards the lower index."""
import numpy as np
import pytest

import pikv_oracle as O
from util import codes_np, kv_like, np_of, rng, to_dev

pytestmark = pytest.mark.gpu


def _fill_pool(dev, r, caps, lens, heads, dh, group, scheme, dtype="bf16"):
    """Build a device pool and its numpy mirror with lens[c] rows in cache c."""
    import torch
    from pikv_amd import ops
    D = heads * dh
    pool = ops.CachePool(caps, heads, dh, group, scheme, dev)
    ref = O.CachePool(caps, D, group, scheme)
    n = int(sum(lens))
    ks, vs = kv_like(r, n, D, dtype=dtype), kv_like(r, n, D, dtype=dtype)
    cid = np.concatenate([np.full(l, c, dtype=np.int32) for c, l in enumerate(lens)])
    slot = np.concatenate([np.arange(l, dtype=np.int32) for l in lens])
    pool.quant_scatter(to_dev(ks, dev, dtype), to_dev(vs, dev, dtype), to_dev(cid, dev),
                       to_dev(slot, dev), 1, now=0.0)
    cnt = np.array(lens, dtype=np.int32)
    pool.advance(to_dev(cnt, dev))
    ref.quant_scatter(ks, vs, cid, slot, 1, now=0.0)
    ref.advance(cnt)
    assert np.array_equal(np_of(pool.fill), ref.fill)
    return pool, ref


@pytest.mark.parametrize("scheme,group,heads,hq,dh", [
    (O.Q_I4_ASYM, 32, 8, 32, 128),     # decode read path shape (GQA 4:1)
    (O.Q_I8_SYM, 128, 4, 4, 128),      # int8 per token per head, MHA
    (O.Q_I8_SYM, 256, 4, 8, 64),       # per-token scale
    (O.Q_I8_ASYM, 64, 2, 16, 64),
    (O.Q_I4_SYM, 64, 4, 4, 64),
    (O.Q_I4_SYM, 32, 2, 4, 128),       # matrix-core kernel, symmetric codes, 2 q heads per kv head
    (O.Q_I4_ASYM, 32, 1, 16, 128),     # matrix-core kernel, all 16 rows of the tile in use
    (O.Q_I4_ASYM, 32, 8, 64, 128),     # 8 q heads per kv head: two sets of A rows against the same codes
    (O.Q_I4_SYM, 32, 2, 12, 128),      # 6 q heads per kv head: the second set half empty
    (O.Q_I4_ASYM, 32, 4, 28, 128),     # 7 q heads per kv head
    (O.Q_I4_SYM, 32, 8, 40, 128),      # 5 q heads per kv head, 8 kv heads
    (O.Q_I4_ASYM, 32, 16, 128, 128),   # 16 kv heads x 8: too much LDS for two sets, generic kernel
    (O.Q_I4_ASYM, 32, 16, 16, 128),    # more kv heads than wavefronts, one q head each
    (O.Q_I4_ASYM, 32, 8, 24, 128),     # 3 q heads per kv head: one of the four staged head slots stays empty
    (O.Q_I4_SYM, 32, 4, 4, 128),       # one q head per kv head on the GQA kernel
    (O.Q_I4_ASYM, 32, 16, 48, 128),    # 16 kv heads x 3
    (O.Q_I8_SYM, 128, 8, 32, 128),     # 8-bit matrix-core kernel: 4 q heads per kv head, scale per head
    (O.Q_I8_ASYM, 128, 2, 16, 128),    # ... 8 q heads per kv head, zero points
    (O.Q_I8_SYM, 256, 4, 64, 128),     # ... 16 q heads per kv head, one scale per two heads
    (O.Q_I8_ASYM, 128, 16, 32, 128),   # ... 16 kv heads (four per wavefront)
    (O.Q_I8_SYM, 1024, 8, 16, 128),    # ... one scale per token
    (O.Q_I4_ASYM, 32, 4, 8, 64),       # heads of 64: two kv heads share a 128-dimension slab of the matrix-core kernel
    (O.Q_I4_SYM, 32, 12, 12, 64),      # ... 12 x 64, one q head each (six slabs)
    (O.Q_I4_ASYM, 32, 2, 8, 64),       # ... 4 q heads per kv head: two sets of A rows
    (O.Q_I4_SYM, 32, 4, 12, 64),       # ... 3 per kv head
    (O.Q_I4_ASYM, 32, 8, 16, 32),      # heads of 32: four kv heads per slab
    (O.Q_I4_ASYM, 32, 3, 3, 64),       # an odd number of narrow heads fills no slab: vector form
    (O.Q_I4_ASYM, 32, 2, 10, 64),      # 5 q heads per narrow kv head: vector form
    (O.Q_I8_SYM, 64, 8, 16, 64),       # 8-bit heads of 64 on the matrix-core kernel: a scale per kv head, two per slab
    (O.Q_I8_ASYM, 64, 4, 16, 64),      # ... 4 q heads per kv head, zero points
    (O.Q_I8_SYM, 128, 4, 8, 64),       # ... one scale per slab
    (O.Q_I8_ASYM, 32, 8, 16, 32),      # ... heads of 32
    (O.Q_I8_SYM, 64, 32, 64, 64),      # ... 16 slabs (four per wavefront)
    (O.Q_I4_ASYM, 32, 32, 32, 128),    # 32 kv heads of 128: four groups of 8 slabs as independent blocks of the matrix-core kernel
    (O.Q_I4_SYM, 32, 24, 48, 128),     # ... three groups, 2 q heads per kv head
    (O.Q_I4_ASYM, 32, 24, 120, 128),   # ... 5 q heads per kv head: two sets
    (O.Q_I8_SYM, 64, 12, 12, 64),      # 12 kv heads: three blocks of four heads per tile
    (O.Q_I4_ASYM, 32, 3, 6, 128),      # 3 kv heads
    (O.Q_I8_ASYM, 128, 5, 10, 128),    # 5 kv heads: one block per head
    (O.Q_I4_ASYM, 32, 2, 32, 128),     # 16 q heads per kv head: two launches of eight heads over the same codes
    (O.Q_I4_SYM, 32, 1, 12, 128),      # ... 12: the second launch with four heads
    (O.Q_I4_ASYM, 32, 4, 36, 128),     # ... 9: the second launch with one head
    (O.Q_I4_ASYM, 32, 2, 14, 64),      # heads of 64, 14 q heads on the one slab (Qwen2.5-0.5B): two launches
    (O.Q_I4_SYM, 32, 4, 20, 64),       # ... two slabs x 10
    (O.Q_I4_ASYM, 32, 4, 12, 32),      # heads of 32: 12 q heads on the one slab
    (O.Q_I4_ASYM, 32, 1, 48, 128),     # multi-query: 48 q heads on one kv head, six launches
    (O.Q_I4_SYM, 32, 2, 40, 64),       # ... 40 on one slab of two narrow heads
    (O.Q_I8_SYM, 128, 1, 48, 128),     # 8-bit multi-query: three launches of 16 heads
    (O.Q_I8_SYM, 128, 1, 128, 128),    # ... 128 heads: beyond the matrix-core kernel's staging, the vector form
    (O.Q_I8_ASYM, 128, 2, 122, 128),   # ... 2 kv x 61 q heads
    (O.Q_I8_ASYM, 128, 2, 40, 128),    # ... 20 per kv head: launches of 16 and 4
])
@pytest.mark.parametrize("qdtype", ["f32", "bf16"])
def test_scores_and_h2o(dev, scheme, group, heads, hq, dh, qdtype):
    r = rng(scheme * 7 + heads)
    caps = [300, 64, 130, 10]
    lens = [257, 64, 1, 0]            # ragged: partial tile, full tile, single row, empty
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    q = r.standard_normal((len(caps), hq, dh)).astype(np.float32)
    if qdtype == "bf16":
        q = O.bf16_round(q)
    scale_qk = 1.0 / np.sqrt(dh)
    scores, tmax, tsum = pool.scores(to_dev(q, dev, qdtype), hq)
    sc = np_of(scores)
    imp_ref_all = []
    for c, L in enumerate(lens):
        if L == 0:
            continue
        rows = ref.valid_rows(c)
        k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        s_ref = O.attention_scores(q[c], k_hat, heads, scale_qk)
        rms = np.sqrt((s_ref.astype(np.float64) ** 2).mean()) + 1e-12
        assert np.abs(sc[c, :, :L] - s_ref).max() <= 1e-3 * rms, (c, np.abs(sc[c, :, :L] - s_ref).max(), rms)
        imp_ref_all.append((c, rows, O.h2o_importance(s_ref)))
    # accumulate twice (second time with decay) and compare the running state
    acc_ref, ts_ref = ref.acc.copy(), ref.ts.copy()
    imp = pool.h2o_accumulate(scores, tmax, tsum, now=5.0, return_importance=True)
    for c, rows, (p_ref, i_ref) in imp_ref_all:
        O.h2o_accumulate(acc_ref, ts_ref, rows, i_ref, 5.0)
        assert np.allclose(np_of(imp)[c, :len(rows)], i_ref, rtol=1e-3, atol=1e-6)
        assert abs(np_of(imp)[c, :len(rows)].sum() - hq) < 1e-3 * hq
    assert np.allclose(np_of(pool.acc), acc_ref, rtol=1e-3, atol=1e-6)
    assert np.array_equal(np_of(pool.ts), ts_ref)
    scores2, tmax2, tsum2 = pool.scores(to_dev(q, dev, qdtype), hq)
    pool.h2o_accumulate(scores2, tmax2, tsum2, now=6.0, decay=0.95, write_probs=True)
    for c, rows, (p_ref, i_ref) in imp_ref_all:
        O.h2o_accumulate(acc_ref, ts_ref, rows, i_ref, 6.0, decay=0.95)
        assert np.allclose(np_of(scores2)[c, :, :len(rows)], p_ref, rtol=1e-3, atol=1e-7)
    assert np.allclose(np_of(pool.acc), acc_ref, rtol=1e-3, atol=1e-6)
    assert np.array_equal(np_of(pool.ts), ts_ref)


@pytest.mark.parametrize("scheme,group,heads,hq,dh", [
    (O.Q_I4_ASYM, 32, 8, 32, 128),     # decode shape
    (O.Q_I4_SYM, 32, 2, 2, 128),
    (O.Q_I4_ASYM, 32, 4, 8, 64),       # two heads of 64 per slab, 2 query heads each
    (O.Q_I4_ASYM, 32, 3, 12, 128),     # 3 kv heads x 4
    (O.Q_I4_ASYM, 32, 4, 28, 128),     # 7 query heads per kv head: two sets of heads, two limbs each
    (O.Q_I4_SYM, 32, 1, 8, 128),
    (O.Q_I8_SYM, 128, 8, 32, 128),     # 8-bit kernel: two operand rows per head
    (O.Q_I8_ASYM, 128, 2, 16, 128),    # ... all 16 rows in use
    (O.Q_I8_ASYM, 64, 4, 16, 64),      # ... heads of 64
])
def test_scores_float32_queries_as_two_limbs(dev, scheme, group, heads, hq, dh):
    """float32 queries on the matrix-core score kernels: every query element goes in as two bf16 limbs,
    q = hi + lo + (at most 2^-17 |q|).  The scores against float64 on the dequantised rows: within
    2^-14 of sum |q k| - the limbs' 2^-17 plus the float32 rounding of accumulators that carry the
    codes with an offset of 128 (the same for bf16 queries) - far inside the 1e-3 of the row RMS
    that the float path is held to; and queries that ARE bf16 numbers give the scores of the bf16
    call bit for bit (their low limbs are zero)."""
    r = rng(90 + heads)
    caps, lens = [200, 70], [193, 64]
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    q = (r.standard_normal((2, hq, dh)) * (1.0 + 1e-3 * r.standard_normal((2, hq, dh)))).astype(np.float32)
    assert not np.array_equal(q, O.bf16_round(q))
    scale_qk = 1.0 / np.sqrt(dh)
    sc = np_of(pool.scores(to_dev(q, dev, "f32"), hq)[0])
    rep = hq // heads
    for c, L in enumerate(lens):
        rows = ref.valid_rows(c)
        k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group).astype(np.float64)
        k_hat = k_hat.reshape(L, heads, dh)
        for h in range(hq):
            want = k_hat[:, h // rep, :] @ q[c, h].astype(np.float64) * scale_qk
            bound = (np.abs(k_hat[:, h // rep, :]) @ np.abs(q[c, h]).astype(np.float64)) * scale_qk
            err = np.abs(sc[c, h, :L] - want)
            assert (err <= 2.0 ** -14 * bound + 1e-7).all(), (c, h, (err / bound).max())
    qb = O.bf16_round(q)
    s_f = np_of(pool.scores(to_dev(qb, dev, "f32"), hq)[0])
    s_b = np_of(pool.scores(to_dev(qb, dev, "bf16"), hq)[0])
    for c, L in enumerate(lens):
        assert np.array_equal(s_f[c, :, :L], s_b[c, :, :L])


@pytest.mark.parametrize("scheme,group,heads,hq,dh,qdtype", [
    (O.Q_I4_ASYM, 32, 8, 32, 128, "bf16"),    # matrix-core 4-bit kernels
    (O.Q_I4_ASYM, 32, 8, 64, 128, "bf16"),    # ... two sets of query heads
    (O.Q_I8_SYM, 128, 8, 32, 128, "bf16"),    # matrix-core 8-bit kernels
    (O.Q_I8_SYM, 128, 4, 4, 64, "f32"),       # vector forms
    (O.Q_I4_SYM, 64, 2, 6, 64, "f32"),
])
def test_cache_longer_than_max_len(dev, scheme, group, heads, hq, dh, qdtype):
    """A cache may hold more rows than the caller covers: with max_len = 200 (not a multiple of
    the 64-token tile) only the first 200 rows of a longer cache are read, nothing is written
    beyond column 200 of a score row or outside the covered rows' accumulators, and the
    statistics, importance and attention output are those of the first 200 rows."""
    import torch
    from pikv_amd import _native as N
    r = rng(scheme * 13 + hq)
    caps = [300, 100, 260]
    lens = [300, 100, 257]
    cover = 200
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    nc = len(caps)
    q = r.standard_normal((nc, hq, dh)).astype(np.float32)
    if qdtype == "bf16":
        q = O.bf16_round(q)
    qd = to_dev(q, dev, qdtype)
    guard = 1024
    flat = torch.full((nc * hq * cover + guard,), 777.0, dtype=torch.float32, device=dev)
    n_tiles = (cover + 63) // 64
    tmax = torch.empty(nc, n_tiles, hq, dtype=torch.float32, device=dev)
    tsum = torch.empty_like(tmax)
    stats = torch.empty(nc, hq, 2, dtype=torch.float32, device=dev)
    imp = torch.full((nc, cover), -5.0, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    zero = None if pool.k_zero is None else pool.k_zero.data_ptr()
    N.call("pikv_gather_dequant_scores", pool.k_codes.data_ptr(), pool.k_scale.data_ptr(), zero, scheme, group,
           heads, hq, dh, qd.data_ptr(), 0 if qdtype == "f32" else 1, float(1.0 / np.sqrt(dh)),
           pool.row_base.data_ptr(), pool.fill.data_ptr(), nc, cover, cover, flat.data_ptr(),
           tmax.data_ptr(), tsum.data_ptr(), st)
    pool.acc.fill_(0.25)
    pool.ts.fill_(-1.0)
    N.call("pikv_h2o_accumulate", flat.data_ptr(), tmax.data_ptr(), tsum.data_ptr(), hq, pool.row_base.data_ptr(),
           pool.fill.data_ptr(), nc, cover, cover, 1.0, 9.0, 0, pool.acc.data_ptr(), pool.ts.data_ptr(),
           imp.data_ptr(), stats.data_ptr(), st)
    scores = flat[:nc * hq * cover].view(nc, hq, cover)
    out = np_of(pool.attend_values(scores, stats))
    torch.cuda.synchronize()
    assert bool((flat[nc * hq * cover:] == 777.0).all()), "score rows were written past the covered columns"
    sc = np_of(scores)
    acc, ts = np_of(pool.acc), np_of(pool.ts)
    for c, L in enumerate(lens):
        n = min(L, cover)
        rows = ref.valid_rows(c)[:n]
        k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
        s_ref = O.attention_scores(q[c], k_hat, heads, 1.0 / np.sqrt(dh))
        rms = np.sqrt((s_ref.astype(np.float64) ** 2).mean())
        assert np.abs(sc[c, :, :n] - s_ref).max() <= 1e-3 * rms
        if n < cover:
            assert (sc[c, :, n:] == 777.0).all()
        p_ref, i_ref = O.h2o_importance(s_ref)
        assert np.allclose(np_of(imp)[c, :n], i_ref, rtol=1e-3, atol=1e-6)
        assert np.allclose(acc[rows], 0.25 + i_ref, rtol=1e-3, atol=1e-6)
        assert (ts[rows] == 9.0).all()
        rest = ref.valid_rows(c)[n:]                      # rows of the cache that were not covered
        assert (acc[rest] == 0.25).all() and (ts[rest] == -1.0).all()
        want = O.attend_values(p_ref, v_hat, heads)
        assert np.abs(out[c] - want).max() <= 2e-3 * np.sqrt((want.astype(np.float64) ** 2).mean())


def _set_state(pool, ref, r, ties):
    """Random accumulators / timestamps (with many exact ties when asked)."""
    acc = r.random(pool.rows).astype(np.float32)
    ts = r.integers(0, 50, pool.rows).astype(np.float32)
    if ties:
        acc = np.round(acc * 8) / 8
        acc[::7] = 0.0
        acc[3::11] = -0.0
    ref.acc[:], ref.ts[:] = acc, ts
    pool.acc.copy_(to_dev(acc, pool.device))
    pool.ts.copy_(to_dev(ts, pool.device))


def _check_compacted(pool, ref, scheme, keep_masks):
    for c, keep in enumerate(keep_masks):
        rows = ref.valid_rows(c)
        if len(rows) == 0:
            continue
        planes = [ref.k_codes, ref.k_scale, ref.k_zero, ref.v_codes, ref.v_scale, ref.v_zero,
                  ref.acc, ref.ts]
        views = [p[rows[0]:rows[0] + len(rows)] for p in planes]
        m = O.compact(keep, *views)
        ref.fill[c] = m
    assert np.array_equal(np_of(pool.fill), ref.fill)
    for c in range(len(keep_masks)):
        rows = ref.valid_rows(c)
        assert np.array_equal(codes_np(pool.k_codes, scheme)[rows], ref.k_codes[rows])
        assert np.array_equal(codes_np(pool.v_codes, scheme)[rows], ref.v_codes[rows])
        assert np.array_equal(np_of(pool.k_scale)[rows].astype(np.float32), ref.k_scale[rows])
        if pool.k_zero is not None:
            assert np.array_equal(np_of(pool.v_zero)[rows].astype(np.float32), ref.v_zero[rows])
        assert np.array_equal(np_of(pool.acc)[rows], ref.acc[rows])
        assert np.array_equal(np_of(pool.ts)[rows], ref.ts[rows])


@pytest.mark.parametrize("ties", [False, True])
@pytest.mark.parametrize("scheme,group,heads,dh", [(O.Q_I4_ASYM, 32, 8, 128), (O.Q_I8_SYM, 64, 4, 64)])
def test_h2o_evict_and_compact(dev, ties, scheme, group, heads, dh):
    r = rng(31 + ties)
    caps = [3000, 1024, 40, 5, 16]
    lens = [2999, 1024, 33, 1, 0]
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    _set_state(pool, ref, r, ties)
    heavy, recent = 0.0625, 0.03
    pool.evict_select(0, heavy_ratio=heavy, recent_ratio=recent)
    keeps = []
    for c, L in enumerate(lens):
        rows = ref.valid_rows(c)
        if L == 0:
            keeps.append(np.zeros(0, dtype=bool))
            continue
        nh, nr = O.h2o_budget(L, heavy, recent)
        keep = O.h2o_keep(ref.acc[rows], ref.ts[rows], nh, nr)
        keeps.append(keep)
        got = np_of(pool.keep_flag)[rows].astype(bool)
        assert np.array_equal(got, keep), (c, np.argwhere(got != keep)[:5])
        m = int(np_of(pool.new_len)[c])
        assert m == keep.sum()
        assert np.array_equal(np_of(pool.keep_index)[rows[0]:rows[0] + m], np.nonzero(keep)[0])
    assert int(np_of(pool.new_len)[4]) == 0
    pool.compact()
    _check_compacted(pool, ref, scheme, keeps)


@pytest.mark.parametrize("ties", [False, True])
def test_lru_evict_and_compact(dev, ties):
    scheme, group, heads, dh = O.Q_I8_SYM, 256, 4, 64   # config-0 layout: one scale per token
    r = rng(41 + ties)
    caps = [128, 128, 128, 128]
    lens = [128, 100, 128, 7]
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme, dtype="f32")
    _set_state(pool, ref, r, ties)
    n_evict = np.array([32, 0, 128, 3], dtype=np.int32)
    pool.evict_select(1, n_evict=to_dev(n_evict, dev))
    keeps = []
    for c, L in enumerate(lens):
        rows = ref.valid_rows(c)
        keep = O.lru_keep(ref.ts[rows], int(n_evict[c]))
        keeps.append(keep)
        assert np.array_equal(np_of(pool.keep_flag)[rows].astype(bool), keep), c
    pool.compact()
    _check_compacted(pool, ref, scheme, keeps)


def test_select_brute_force_small(dev):
    """Tiny caches against an O(n^2) ranking: element i is kept iff fewer than
    m elements precede it in (value desc, index asc) order."""
    r = rng(5)
    caps = [16] * 32
    lens = [int(v) for v in r.integers(1, 17, 32)]
    pool, ref = _fill_pool(dev, r, caps, lens, 1, 64, 64, O.Q_I8_SYM, dtype="f32")
    _set_state(pool, ref, r, True)
    nh = np.array([int(v) for v in r.integers(0, 6, 32)], dtype=np.int32)
    nr = np.array([int(v) for v in r.integers(0, 4, 32)], dtype=np.int32)
    pool.evict_select(0, n_heavy=to_dev(nh, dev), n_recent=to_dev(nr, dev))
    flags = np_of(pool.keep_flag)
    for c, L in enumerate(lens):
        rows = ref.valid_rows(c)
        a, t = ref.acc[rows] + 0.0, ref.ts[rows]
        for i in range(L):
            before_a = sum((a[j] > a[i]) or (a[j] == a[i] and j < i) for j in range(L))
            before_t = sum((t[j] > t[i]) or (t[j] == t[i] and j < i) for j in range(L))
            want = before_a < nh[c] or before_t < nr[c]
            assert bool(flags[rows[i]]) == want, (c, i)


@pytest.mark.parametrize("multi_block", [False, True])
@pytest.mark.parametrize("ties", [False, True])
def test_h2o_select_long_cache(dev, ties, multi_block):
    """Long caches.  One block per cache (no workspace): caches longer than 32768 rows
    take the selection path that re-reads its keys from memory in every pass, a shorter
    one rides along on the register path.  With the workspace every cache is cut into
    4096-row chunks; budgets of 1, of everything and lengths one off a chunk edge."""
    r = rng(77 + ties)
    caps = [70000, 33000, 32768]
    lens = [69999, 32769, 32768]
    pool, ref = _fill_pool(dev, r, caps, lens, 1, 32, 32, O.Q_I8_SYM, dtype="f32")
    _set_state(pool, ref, r, ties)
    nh = np.array([4375, 1, 2048], dtype=np.int32)
    nr = np.array([546, 32769, 256], dtype=np.int32)
    pool.evict_select(0, n_heavy=to_dev(nh, dev), n_recent=to_dev(nr, dev), multi_block=multi_block)
    keeps = []
    for c, L in enumerate(lens):
        rows = ref.valid_rows(c)
        keep = O.h2o_keep(ref.acc[rows], ref.ts[rows], int(nh[c]), int(nr[c]))
        keeps.append(keep)
        got = np_of(pool.keep_flag)[rows].astype(bool)
        assert np.array_equal(got, keep), (c, np.argwhere(got != keep)[:5])
        m = int(np_of(pool.new_len)[c])
        assert m == keep.sum()
        assert np.array_equal(np_of(pool.keep_index)[rows[0]:rows[0] + m], np.nonzero(keep)[0])
    pool.compact()
    _check_compacted(pool, ref, O.Q_I8_SYM, keeps)


@pytest.mark.parametrize("ties", [False, True])
def test_select_chunked_edges(dev, ties):
    """Several blocks per cache: empty cache, lengths around the 4096-row chunk edge,
    zero and full budgets, both policies; twice in a row on the same workspace."""
    r = rng(91 + ties)
    caps = [20000] * 6
    lens = [0, 1, 4095, 4096, 4097, 20000]
    pool, ref = _fill_pool(dev, r, caps, lens, 1, 32, 32, O.Q_I8_SYM, dtype="f32")
    _set_state(pool, ref, r, ties)
    for rep in range(2):
        nh = np.array([3, 1, 0, 4096, 17, 1250 + rep], dtype=np.int32)
        nr = np.array([2, 0, 100, 0, 4097, 156], dtype=np.int32)
        pool.evict_select(0, n_heavy=to_dev(nh, dev), n_recent=to_dev(nr, dev))
        for c, L in enumerate(lens):
            rows = ref.valid_rows(c)
            keep = O.h2o_keep(ref.acc[rows], ref.ts[rows], int(nh[c]), int(nr[c]))
            m = int(np_of(pool.new_len)[c])
            assert m == keep.sum(), (c, m, keep.sum())
            if L:
                assert np.array_equal(np_of(pool.keep_flag)[rows].astype(bool), keep), c
                assert np.array_equal(np_of(pool.keep_index)[rows[0]:rows[0] + m], np.nonzero(keep)[0])
        ne = np.array([1, 1, 4000, 0, 4097, 9999 - rep], dtype=np.int32)
        pool.evict_select(1, n_evict=to_dev(ne, dev))
        for c, L in enumerate(lens):
            rows = ref.valid_rows(c)
            keep = O.lru_keep(ref.ts[rows], int(ne[c]))
            m = int(np_of(pool.new_len)[c])
            assert m == keep.sum(), (c, m, keep.sum())
            if L:
                assert np.array_equal(np_of(pool.keep_flag)[rows].astype(bool), keep), c
                assert np.array_equal(np_of(pool.keep_index)[rows[0]:rows[0] + m], np.nonzero(keep)[0])
