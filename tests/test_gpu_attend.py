"""GPU parity: attention output over the compressed V cache (probabilities times
dequantised V rows) through the C ABI against a float64 evaluation on the numpy
restatement's dequantised rows.  Tolerance 1e-3 of the output's root-mean-square
(float32 path).  Both input forms are covered: raw scores + per-head softmax
statistics, and ready probabilities."""
import numpy as np
import pytest

import pikv_oracle as O
from util import np_of, rng, to_dev
from test_gpu_read_evict import _fill_pool

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("scheme,group,heads,hq,dh", [
    (O.Q_I4_ASYM, 32, 8, 32, 128),     # decode shape: matrix-core form, 4 q heads per kv head
    (O.Q_I4_SYM, 32, 2, 4, 128),       # matrix-core form, symmetric codes
    (O.Q_I4_ASYM, 32, 1, 8, 128),      # matrix-core form, all 16 operand rows in use
    (O.Q_I4_ASYM, 32, 4, 4, 128),      # matrix-core form, one row pair per kv head
    (O.Q_I4_ASYM, 32, 16, 16, 128),    # 16 kv heads: two groups of 8 as neighbouring blocks of the matrix-core form
    (O.Q_I4_ASYM, 32, 32, 32, 128),    # ... 32 kv heads, four groups
    (O.Q_I4_SYM, 32, 24, 120, 128),    # ... 5 q heads per kv head: six groups of 4, two sets
    (O.Q_I4_ASYM, 32, 12, 12, 128),    # 12 kv heads are no whole groups of 8: vector form
    (O.Q_I4_ASYM, 32, 8, 24, 128),     # 3 q heads per kv head: a row pair of every kv head stays empty
    (O.Q_I4_ASYM, 32, 8, 64, 128),     # 8 q heads per kv head: two groups of 4 kv heads side by side, two sets of four heads each
    (O.Q_I4_SYM, 32, 2, 12, 128),      # 6 q heads per kv head: the second launch half empty
    (O.Q_I8_SYM, 128, 4, 4, 128),      # int8 per token per head
    (O.Q_I8_SYM, 256, 4, 8, 64),       # one scale per token
    (O.Q_I8_ASYM, 64, 2, 16, 64),      # 8 q heads per kv head in one pass
    (O.Q_I8_SYM, 128, 2, 24, 128),     # 12 q heads per kv head: passes of 8 and 4
    (O.Q_I8_SYM, 128, 8, 32, 128),     # 8-bit matrix-core form: 4 q heads per kv head
    (O.Q_I8_ASYM, 128, 2, 16, 128),    # ... 8 q heads per kv head, zero points
    (O.Q_I8_SYM, 256, 4, 8, 128),      # ... one scale per two heads
    (O.Q_I8_ASYM, 128, 1, 6, 128),     # ... one kv head, 6 q heads
    (O.Q_I4_SYM, 64, 4, 4, 64),
    (O.Q_I4_ASYM, 32, 4, 8, 64),       # heads of 64: two kv heads share a 128-dimension slab of the matrix-core form
    (O.Q_I4_SYM, 32, 2, 8, 64),        # ... 4 q heads per kv head: two launches over the one slab
    (O.Q_I4_ASYM, 32, 16, 16, 64),     # ... eight slabs
    (O.Q_I4_SYM, 32, 4, 12, 64),       # ... 3 q heads per kv head: the second launch half empty
    (O.Q_I4_ASYM, 32, 8, 16, 32),      # heads of 32: four kv heads per slab
    (O.Q_I4_ASYM, 32, 12, 12, 64),     # ... six slabs
    (O.Q_I4_ASYM, 32, 20, 20, 64),     # ten slabs: vector form
    (O.Q_I8_SYM, 64, 8, 16, 64),       # 8-bit heads of 64 on the matrix-core form: a scale per kv head, two per slab
    (O.Q_I8_ASYM, 64, 4, 16, 64),      # ... 4 q heads per kv head: all 16 operand rows, zero points per kv head
    (O.Q_I8_SYM, 128, 4, 8, 64),       # ... one scale per slab
    (O.Q_I8_ASYM, 32, 8, 16, 32),      # ... heads of 32
    (O.Q_I8_ASYM, 64, 16, 32, 64),     # ... eight slabs
    (O.Q_I8_SYM, 64, 12, 12, 64),      # 12 kv heads, vector form: five whole rows per pass of a block
    (O.Q_I4_SYM, 32, 3, 6, 128),       # 3 kv heads: matrix-core form with a kv head count that is no power of two
    (O.Q_I4_ASYM, 32, 6, 12, 128),     # ... 6
    (O.Q_I4_ASYM, 32, 5, 5, 128),      # ... 5, one q head each
    (O.Q_I4_SYM, 32, 7, 42, 128),      # ... 7 x 6: two launches
    (O.Q_I8_SYM, 128, 3, 6, 128),      # 8-bit matrix-core form, 3 kv heads
    (O.Q_I8_ASYM, 128, 6, 12, 128),    # ... 6
    (O.Q_I8_SYM, 128, 5, 40, 128),     # ... 5 x 8
    (O.Q_I8_ASYM, 128, 7, 14, 128),    # ... 7
    (O.Q_I8_SYM, 64, 12, 24, 64),      # ... 12 heads of 64: six slabs
    (O.Q_I4_ASYM, 32, 2, 32, 128),     # 16 q heads per kv head: two launches of two sets each
    (O.Q_I4_SYM, 32, 1, 12, 128),      # ... 12: the second launch with one set
    (O.Q_I4_ASYM, 32, 4, 36, 128),     # ... 9 on 4 kv heads
    (O.Q_I8_SYM, 128, 40, 40, 128),    # 40 kv heads of 128, 8-bit: rows of 320 lanes, the vector form in windows of 8 kv heads
    (O.Q_I4_SYM, 64, 72, 72, 128),     # ... 4-bit, 288 lanes: windows of 8
    (O.Q_I4_ASYM, 32, 2, 14, 64),      # heads of 64, 14 q heads on the one slab: two launches
    (O.Q_I4_SYM, 32, 4, 12, 32),       # heads of 32, 12 q heads on the one slab
    (O.Q_I4_ASYM, 32, 1, 48, 128),     # multi-query: 48 q heads on one kv head, six launches
    (O.Q_I8_SYM, 128, 1, 48, 128),     # ... 8-bit
    (O.Q_I8_ASYM, 128, 4, 80, 128),    # ... 8-bit, 20 per kv head on 4 kv heads
    (O.Q_I8_SYM, 128, 2, 32, 128),     # 8-bit, 16 q heads per kv head: two launches of eight heads
    (O.Q_I8_ASYM, 128, 1, 12, 128),    # ... 12: the second launch with four
    (O.Q_I8_SYM, 128, 4, 40, 128),     # ... 10 on 4 kv heads (single rows)
])
@pytest.mark.parametrize("form", ["stats", "probs"])
def test_attend_values(dev, scheme, group, heads, hq, dh, form):
    import torch
    r = rng(scheme * 11 + heads + hq)
    caps = [4200, 64, 130, 10]
    lens = [4100, 64, 1, 0]           # spans three token ranges, full tile, single row, empty
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    q = O.bf16_round(r.standard_normal((len(caps), hq, dh)).astype(np.float32) * 3)
    scores, tmax, tsum = pool.scores(to_dev(q, dev, "bf16"), hq)
    pool.h2o_accumulate(scores, tmax, tsum, now=1.0, write_probs=(form == "probs"))
    out = pool.attend_values(scores, None if form == "probs" else pool.head_stats)
    got = np_of(out)
    assert got.shape == (len(caps), hq, dh)
    sc = np_of(scores)
    for c, L in enumerate(lens):
        if L == 0:
            assert not got[c].any()
            continue
        rows = ref.valid_rows(c)
        v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
        if form == "probs":
            p = sc[c, :, :L]
        else:
            p, _ = O.h2o_importance(sc[c, :, :L])
        want = O.attend_values(p, v_hat, heads)
        rms = np.sqrt((want.astype(np.float64) ** 2).mean()) + 1e-12
        err = np.abs(got[c] - want).max()
        assert err <= 1e-3 * rms, (c, err, rms)


@pytest.mark.parametrize("scheme,group,heads,hq,dh", [
    (O.Q_I4_ASYM, 32, 8, 32, 128),     # matrix-core form: importance summed from the staged tile
    (O.Q_I4_ASYM, 32, 2, 4, 128),
    (O.Q_I4_ASYM, 32, 4, 32, 128),     # two launches: the second adds to what the first decayed
    (O.Q_I4_ASYM, 32, 8, 24, 128),     # 3 q heads per kv head
    (O.Q_I4_SYM, 32, 8, 40, 128),      # 5 per kv head: two groups of 4 kv heads, the second set with a single head
    (O.Q_I8_SYM, 128, 4, 8, 128),      # 8-bit matrix-core form
    (O.Q_I8_ASYM, 128, 8, 64, 128),    # ... 64 query heads
    (O.Q_I8_SYM, 64, 4, 8, 64),        # vector form: importance in a kernel of its own
    (O.Q_I4_ASYM, 32, 4, 8, 64),       # heads of 64 on the matrix-core form
    (O.Q_I4_SYM, 32, 2, 8, 64),        # ... two launches
    (O.Q_I4_ASYM, 32, 8, 8, 32),       # heads of 32
    (O.Q_I8_ASYM, 64, 8, 16, 64),      # 8-bit heads of 64 on the matrix-core form
    (O.Q_I4_ASYM, 32, 6, 36, 128),     # 6 kv heads x 6: two groups of 3
    (O.Q_I8_SYM, 128, 3, 12, 128),     # 8-bit, 3 kv heads
    (O.Q_I4_ASYM, 32, 16, 32, 128),    # 16 kv heads in two groups: the importance comes from a kernel of its own
    (O.Q_I4_SYM, 32, 24, 24, 128),
    (O.Q_I4_ASYM, 32, 1, 4, 128),      # one kv head: four neighbouring rows as one row of four slabs
    (O.Q_I4_SYM, 32, 1, 8, 128),       # ... 8 q heads: two sets
    (O.Q_I4_ASYM, 32, 2, 12, 128),     # two kv heads x 6: pairs of rows, two sets
    (O.Q_I4_ASYM, 32, 3, 9, 128),      # three kv heads: pairs of rows, six slabs
    (O.Q_I4_ASYM, 32, 2, 24, 128),     # 12 q heads per kv head: two launches, the second adds to what the first decayed
    (O.Q_I4_SYM, 32, 2, 14, 64),       # ... heads of 64, 14 on the one slab
    (O.Q_I4_ASYM, 32, 1, 20, 128),     # ... multi-query, 20 heads: three launches
    (O.Q_I8_SYM, 128, 2, 24, 128),     # 8-bit, 12 q heads per kv head: two launches
    (O.Q_I8_ASYM, 128, 1, 8, 128),     # 8-bit, one kv head: eight neighbouring rows as one row
    (O.Q_I8_SYM, 128, 2, 4, 128),      # ... two kv heads: four rows
])
@pytest.mark.parametrize("decay", [1.0, 0.95])
def test_attend_accumulates_importance(dev, scheme, group, heads, hq, dh, decay):
    """attend_values(accumulate=True) after a statistics-only h2o_accumulate leaves the
    same accumulators and timestamps as the separate h2o_accumulate pass, and the same
    output as without the bookkeeping."""
    import torch
    r = rng(scheme * 7 + hq)
    caps = [4200, 64, 130, 10]
    lens = [4100, 64, 1, 0]
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    pool.acc.copy_(to_dev(r.random(pool.rows).astype(np.float32), dev))
    pool.ts.fill_(-3.0)
    acc0 = pool.acc.clone()
    q = O.bf16_round(r.standard_normal((len(caps), hq, dh)).astype(np.float32) * 3)
    scores, tmax, tsum = pool.scores(to_dev(q, dev, "bf16"), hq)
    pool.h2o_accumulate(scores, tmax, tsum, now=9.0, decay=decay)
    acc_sep, ts_sep = np_of(pool.acc), np_of(pool.ts)
    out_sep = np_of(pool.attend_values(scores, pool.head_stats))
    pool.acc.copy_(acc0)
    pool.ts.fill_(-3.0)
    pool.h2o_accumulate(scores, tmax, tsum, now=9.0, stats_only=True)
    assert torch.equal(pool.acc, acc0) and bool((pool.ts == -3.0).all())
    out = np_of(pool.attend_values(scores, pool.head_stats, accumulate=True, now=9.0, decay=decay))
    assert np.array_equal(out, out_sep)
    assert np.array_equal(np_of(pool.ts), ts_sep)
    np.testing.assert_allclose(np_of(pool.acc), acc_sep, rtol=1e-5, atol=1e-6)
    # against the numpy restatement as well
    for c, L in enumerate(lens):
        if L:
            rows = ref.valid_rows(c)
            _, imp = O.h2o_importance(np_of(scores)[c, :, :L])
            want = np_of(acc0)[rows] * np.float32(decay) + imp
            np.testing.assert_allclose(np_of(pool.acc)[rows], want, rtol=1e-3, atol=1e-5)
            assert (np_of(pool.ts)[rows] == 9.0).all()


def test_attend_peaked_distribution(dev):
    """One token carries almost all the weight: the output must equal that row of V to
    float32 accuracy, which a bf16-only weight operand would miss by 2^-9."""
    import torch
    r = rng(5)
    heads, hq, dh, L = 8, 32, 128, 300
    pool, ref = _fill_pool(dev, r, [320], [L], heads, dh, 32, O.Q_I4_ASYM)
    probs = np.full((1, hq, 320), 1e-7, dtype=np.float32)
    hot = r.integers(0, L, hq)
    probs[0, np.arange(hq), hot] = 0.77777
    out = np_of(pool.attend_values(to_dev(probs, dev)))
    rows = ref.valid_rows(0)
    v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], 32)
    want = O.attend_values(probs[0, :, :L], v_hat, heads)
    assert np.abs(out[0] - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("scheme,group,heads,hq,dh,qdtype", [
    (O.Q_I4_ASYM, 32, 8, 32, 128, "bf16"),   # decode shape: exchange format between the matrix-core kernels
    (O.Q_I4_SYM, 32, 2, 4, 128, "bf16"),     # ... symmetric codes
    (O.Q_I4_ASYM, 32, 1, 8, 128, "bf16"),    # ... 8 q heads per kv head: two sets, two attention launches
    (O.Q_I4_ASYM, 32, 8, 24, 128, "bf16"),   # ... 3 q heads per kv head
    (O.Q_I4_SYM, 32, 4, 28, 128, "bf16"),    # ... 7 q heads per kv head
    (O.Q_I4_ASYM, 32, 16, 16, 128, "bf16"),  # 16 kv heads: exchange format, the attention kernel in two groups of 8
    (O.Q_I4_SYM, 32, 32, 32, 128, "bf16"),   # ... 32 kv heads: both kernels in four groups
    (O.Q_I4_ASYM, 32, 24, 48, 128, "f32"),   # ... three groups, float32 queries
    (O.Q_I4_ASYM, 32, 12, 12, 128, "bf16"),  # 12 kv heads: no whole groups, the three public steps inside the call
    (O.Q_I4_ASYM, 32, 8, 32, 128, "f32"),    # float32 queries: same
    (O.Q_I8_SYM, 128, 8, 32, 128, "bf16"),   # 8-bit matrix-core kernels
    (O.Q_I8_ASYM, 64, 2, 16, 64, "f32"),     # vector forms
    (O.Q_I4_SYM, 64, 4, 12, 64, "bf16"),
    (O.Q_I4_ASYM, 32, 4, 8, 64, "bf16"),     # heads of 64: exchange format, two kv heads per 128-dimension slab
    (O.Q_I4_SYM, 32, 2, 8, 64, "bf16"),      # ... 4 q heads per kv head
    (O.Q_I4_ASYM, 32, 16, 16, 64, "bf16"),   # ... eight slabs
    (O.Q_I4_ASYM, 32, 8, 16, 32, "bf16"),    # heads of 32
    (O.Q_I4_SYM, 32, 12, 12, 64, "bf16"),    # ... six slabs
    (O.Q_I4_ASYM, 32, 6, 24, 128, "bf16"),   # kv head counts that are no power of two: 6
    (O.Q_I4_SYM, 32, 5, 10, 128, "bf16"),    # ... 5
    (O.Q_I4_ASYM, 32, 7, 7, 128, "bf16"),    # ... 7
    (O.Q_I4_ASYM, 32, 20, 20, 64, "bf16"),   # ten slabs: the three public steps inside the call
    (O.Q_I4_ASYM, 32, 2, 6, 64, "f32"),
    (O.Q_I8_ASYM, 64, 8, 16, 64, "bf16"),    # 8-bit heads of 64 on the matrix-core kernels
    (O.Q_I8_SYM, 64, 12, 12, 64, "f32"),     # 12 kv heads of 64, 8-bit
    (O.Q_I4_ASYM, 32, 3, 6, 128, "bf16"),    # 3 kv heads
    (O.Q_I4_ASYM, 32, 8, 64, 128, "bf16"),   # 8 q heads per kv head of 8: two groups of 4 kv heads, two sets each
    (O.Q_I4_SYM, 32, 6, 36, 128, "f32"),     # ... 6 x 6: two groups of 3
    (O.Q_I4_ASYM, 32, 16, 80, 128, "bf16"),  # ... 16 x 5: four groups of 4, the second set with one head
    (O.Q_I4_SYM, 32, 7, 35, 128, "bf16"),    # 7 kv heads cannot be halved: two launches over all of them
    (O.Q_I4_ASYM, 32, 4, 16, 128, "bf16"),   # 4 kv heads: pairs of neighbouring rows as one row of eight slabs
    (O.Q_I4_SYM, 32, 2, 8, 128, "f32"),      # 2 kv heads: four rows as one
    (O.Q_I4_ASYM, 32, 1, 3, 128, "bf16"),    # 1 kv head, 3 q heads
    (O.Q_I4_ASYM, 32, 2, 32, 128, "bf16"),   # 16 q heads per kv head: both kernels in two launches of eight heads
    (O.Q_I4_SYM, 32, 1, 12, 128, "f32"),     # ... 12, float32 queries
    (O.Q_I4_ASYM, 32, 4, 40, 128, "bf16"),   # ... 10 on 4 kv heads
    (O.Q_I8_ASYM, 128, 40, 40, 128, "bf16"), # 40 kv heads of 128, 8-bit: the vector forms in windows of kv heads
    (O.Q_I4_ASYM, 32, 2, 14, 64, "bf16"),    # ... heads of 64: 14 q heads on the one slab
    (O.Q_I4_SYM, 32, 4, 20, 64, "bf16"),     # ... two slabs x 10
    (O.Q_I4_ASYM, 32, 1, 48, 128, "bf16"),   # multi-query: 48 q heads on one kv head
    (O.Q_I8_SYM, 128, 1, 48, 128, "bf16"),   # ... 8-bit
    (O.Q_I8_SYM, 128, 1, 128, 128, "bf16"),  # ... 128 q heads on one 8-bit kv head: the staged rows exceed the matrix-core kernel's LDS, vector scores
    (O.Q_I8_ASYM, 128, 2, 128, 128, "bf16"), # ... 2 kv x 64 q heads each, same limit
    (O.Q_I8_ASYM, 128, 2, 8, 128, "bf16"),   # 8-bit, 2 kv heads: four neighbouring rows as one row of eight slabs
    (O.Q_I8_ASYM, 128, 2, 20, 128, "bf16"),  # ... 10 q heads per kv head: the attention output in two launches
    (O.Q_I8_SYM, 128, 1, 4, 128, "f32"),     # ... 1 kv head: eight rows as one
    (O.Q_I8_SYM, 128, 3, 12, 128, "bf16"),   # ... 3 kv heads x 4: pairs of rows, 24 staged probability rows
    (O.Q_I8_SYM, 128, 3, 24, 128, "bf16"),   # ... 3 kv heads x 8; scores up to 36 in this draw: needs the 8-bit scores' part-wise offsets
    (O.Q_I8_SYM, 128, 8, 64, 128, "bf16"),   # 8-bit one-pass form: 8 q heads per kv head, every lane of a record
    (O.Q_I8_ASYM, 128, 6, 42, 128, "bf16"),  # ... 7 q heads per kv head, zero points
    (O.Q_I8_ASYM, 256, 4, 20, 128, "bf16"),  # ... a scale per pair of kv heads, 5 q heads per kv head
    (O.Q_I8_SYM, 512, 4, 8, 128, "bf16"),    # ... a scale per token, 2 q heads per kv head: records of 32 lanes
    (O.Q_I8_ASYM, 128, 7, 14, 128, "bf16"),  # ... 7 kv heads x 2
    (O.Q_I8_SYM, 128, 5, 5, 128, "bf16"),    # ... one q head per kv head: one pass only without the bookkeeping
    (O.Q_I4_ASYM, 32, 8, 40, 128, "bf16"),   # 4-bit one-pass form with two operand sets: 5 q heads per kv head
    (O.Q_I4_SYM, 32, 5, 40, 128, "bf16"),    # ... 8 on 5 kv heads, symmetric codes
    (O.Q_I4_SYM, 32, 4, 16, 128, "f32"),     # ... float32 queries: the sets are the limbs
    (O.Q_I4_ASYM, 32, 6, 18, 128, "f32"),    # ... 3 q heads per kv head
    (O.Q_I4_ASYM, 32, 3, 3, 128, "f32"),     # ... one
    (O.Q_I8_SYM, 128, 8, 32, 128, "f32"),    # ... float32 queries as two bf16 limbs
    (O.Q_I8_ASYM, 128, 4, 32, 128, "f32"),   # ... 8 q heads per kv head, zero points
    (O.Q_I8_ASYM, 256, 6, 18, 128, "f32"),   # ... 6 kv heads x 3: two blocks of three wavefronts, a scale per pair of heads
])
@pytest.mark.parametrize("decay", [1.0, 0.9])
def test_decode_attend_one_call(dev, scheme, group, heads, hq, dh, qdtype, decay):
    """pikv_decode_attend against core/single/pikv_attention.py:123,163,188 and
    cache_scheduling.py:69-73 evaluated in float64 on the restatement's dequantised K and V
    rows: attention output within 1e-3 of its root-mean-square, accumulators within 1e-3
    relative, timestamps exact; rows outside the caches' fill untouched.  Two calls in a row
    (the second after an append) reuse the pool's workspace."""
    import torch
    r = rng(scheme * 5 + heads + hq)
    caps = [4300, 64, 130, 10]
    lens = [4100, 64, 1, 0]           # spans three token ranges, full tile, single row, empty
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    acc0 = r.random(pool.rows).astype(np.float32)
    pool.acc.copy_(to_dev(acc0, dev))
    pool.ts.fill_(-3.0)
    scale_qk = 1.0 / np.sqrt(dh)

    def reference(q, lens_now, acc_before):
        outs, accs = [], acc_before.copy()
        for c, L in enumerate(lens_now):
            if L == 0:
                outs.append(np.zeros((hq, dh), np.float32))
                continue
            rows = ref.valid_rows(c)[:L]
            k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
            v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
            s = O.attention_scores(q[c], k_hat, heads, scale_qk)
            p, imp = O.h2o_importance(s)
            outs.append(O.attend_values(p, v_hat, heads))
            accs[rows] = accs[rows] * np.float32(decay) + imp
        return np.stack(outs), accs

    q = r.standard_normal((len(caps), hq, dh)).astype(np.float32) * 2
    if qdtype == "bf16":
        q = O.bf16_round(q)
    out = np_of(pool.decode_attend(to_dev(q, dev, qdtype), hq, now=7.0, decay=decay))
    want, acc_ref = reference(q, lens, acc0)
    for c, L in enumerate(lens):
        if L == 0:
            assert not out[c].any()
            continue
        rms = np.sqrt((want[c].astype(np.float64) ** 2).mean()) + 1e-12
        assert np.abs(out[c] - want[c]).max() <= 1e-3 * rms, (c, np.abs(out[c] - want[c]).max(), rms)
    np.testing.assert_allclose(np_of(pool.acc), acc_ref, rtol=1e-3, atol=1e-5)
    ts = np_of(pool.ts)
    for c, L in enumerate(lens):
        rows = ref.valid_rows(c)
        assert (ts[rows[:L]] == 7.0).all()
    touched = np.zeros(pool.rows, bool)
    for c, L in enumerate(lens):
        touched[ref.valid_rows(c)[:L]] = True
    assert (ts[~touched] == -3.0).all() and np.array_equal(np_of(pool.acc)[~touched], acc0[~touched])
    # same result as the three public steps
    scores, tmax, tsum = pool.scores(to_dev(q, dev, qdtype), hq)
    pool.h2o_accumulate(scores, tmax, tsum, now=7.0, stats_only=True)
    out3 = np_of(pool.attend_values(scores, pool.head_stats))
    assert np.abs(out - out3).max() <= 1e-3 * (np.sqrt((out3.astype(np.float64) ** 2).mean()) + 1e-12)
    # second call on the same workspace, without the bookkeeping, covering fewer rows than cached
    acc_now = np_of(pool.acc).copy()
    q2 = O.bf16_round(r.standard_normal((len(caps), hq, dh)).astype(np.float32))
    out2 = np_of(pool.decode_attend(to_dev(q2, dev, qdtype), hq, now=8.0, accumulate=False, max_len=4300))
    want2, _ = reference(q2, lens, acc_now)
    for c, L in enumerate(lens):
        if L:
            rms = np.sqrt((want2[c].astype(np.float64) ** 2).mean()) + 1e-12
            assert np.abs(out2[c] - want2[c]).max() <= 1e-3 * rms
    assert np.array_equal(np_of(pool.acc), acc_now)
    out_short = np_of(pool.decode_attend(to_dev(q2, dev, qdtype), hq, accumulate=False, max_len=200))
    want_s, _ = reference(q2, [min(L, 200) for L in lens], acc_now)
    for c, L in enumerate(lens):
        if L:
            rms = np.sqrt((want_s[c].astype(np.float64) ** 2).mean()) + 1e-12
            assert np.abs(out_short[c] - want_s[c]).max() <= 1e-3 * rms


@pytest.mark.parametrize("n_caches,length,scheme,heads,hq", [
    (64, 4096, O.Q_I4_ASYM, 1, 4),     # 512 blocks of 512 cached tokens: eight neighbouring rows of the one kv head as one row
    (64, 7168, O.Q_I4_SYM, 1, 2),      # 448 blocks of 1024
    (56, 16384, O.Q_I4_ASYM, 1, 1),    # 448 blocks of 2048
    (40, 2500, O.Q_I8_SYM, 1, 2),      # 8-bit matrix-core form, 400 blocks of 256, ragged lengths
])
def test_attend_block_lengths(dev, n_caches, length, scheme, heads, hq):
    """The number of cached tokens a block walks is chosen per call from the batch (256 ... 4096, so that
    the blocks fill the chip); batches that select the longer walks, attention output and H2O
    accumulators of three caches against float64 on the restatement's dequantised rows, for the
    separate steps and for the one call."""
    dh, group = 128, (32 if scheme in (O.Q_I4_ASYM, O.Q_I4_SYM) else 128)
    r = rng(n_caches + length)
    lens = [length - (17 * c) % 300 for c in range(n_caches)]
    lens[0] = length
    pool, ref = _fill_pool(dev, r, [length] * n_caches, lens, heads, dh, group, scheme)
    q = O.bf16_round(r.standard_normal((n_caches, hq, dh)).astype(np.float32) * 2)
    qd = to_dev(q, dev, "bf16")
    scale_qk = 1.0 / np.sqrt(dh)
    pool.acc.zero_()
    out1 = np_of(pool.decode_attend(qd, hq, now=5.0))
    acc1 = np_of(pool.acc).copy()
    pool.acc.zero_()
    scores, tmax, tsum = pool.scores(qd, hq)
    pool.h2o_accumulate(scores, tmax, tsum, now=5.0, stats_only=True)
    out3 = np_of(pool.attend_values(scores, pool.head_stats, accumulate=True, now=5.0))
    acc3 = np_of(pool.acc)
    for c in (0, n_caches // 2, n_caches - 1):
        rows = ref.valid_rows(c)[:lens[c]]
        k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
        s = O.attention_scores(q[c], k_hat, heads, scale_qk)
        p, imp = O.h2o_importance(s)
        want = O.attend_values(p, v_hat, heads)
        rms = np.sqrt((want.astype(np.float64) ** 2).mean()) + 1e-12
        v_rms = np.sqrt((v_hat.astype(np.float64) ** 2).mean())
        tol = max(1e-3 * rms, 1e-4 * v_rms)       # a long, nearly uniform sum is what cancellation leaves of its terms
        assert np.abs(out1[c] - want).max() <= tol, (c, "one call")
        assert np.abs(out3[c] - want).max() <= tol, (c, "three steps")
        np.testing.assert_allclose(acc1[rows], imp, rtol=1e-3, atol=1e-6)
        np.testing.assert_allclose(acc3[rows], imp, rtol=1e-3, atol=1e-6)


def _decode_reference(ref, q, lens_now, acc_before, heads, group, scale_qk, decay):
    """softmax(q k^T) v and the H2O sums of every cache in float64 on the restatement's dequantised rows."""
    outs, accs = [], acc_before.copy()
    hq, dh = q.shape[1], q.shape[2]
    for c, L in enumerate(lens_now):
        if L == 0:
            outs.append(np.zeros((hq, dh), np.float32))
            continue
        rows = ref.valid_rows(c)[:L]
        k_hat = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        v_hat = O.dequantize_groups(ref.v_codes[rows], ref.v_scale[rows], ref.v_zero[rows], group)
        s = O.attention_scores(q[c], k_hat, heads, scale_qk)
        p, imp = O.h2o_importance(s)
        outs.append(O.attend_values(p, v_hat, heads))
        accs[rows] = accs[rows] * np.float32(decay) + imp
    return np.stack(outs), accs


@pytest.mark.parametrize("draw", range(20))
def test_decode_attend_one_pass_sweep(dev, draw):
    """Seeded random draws over the shapes the one-pass decode kernels take (2 to 8 kv heads of 128
    dimensions; 4-bit: 1 to 8 bf16 or 1 to 4 float32 query heads per kv head; 8-bit: 1 to 8 of either):
    ragged cache lengths around the 64-token tile and the token-range boundaries, empty caches, reads cut
    by max_len, queries scaled up to peaked distributions (scores of +-80: the running maximum moves, most
    halves of the bookkeeping underflow), with and without the bookkeeping.  Same bars as
    test_decode_attend_one_call."""
    r = rng(1000 + draw)
    eight = bool(draw % 2)
    sym = bool((draw // 2) % 2)
    scheme = (O.Q_I8_SYM if sym else O.Q_I8_ASYM) if eight else (O.Q_I4_SYM if sym else O.Q_I4_ASYM)
    heads = int(r.integers(2, 9))
    qdtype = "f32" if r.random() < 0.4 else "bf16"
    max_rep = 8 if (eight or qdtype == "bf16") else 4
    rep = int(r.integers(1, max_rep + 1))
    if draw % 5 == 0:
        rep = 4          # the shape the 4-bit bookkeeping path takes
    hq, dh = heads * rep, 128
    group = 32 if not eight else int(r.choice([128, 128, heads * 128 if (heads & (heads - 1)) == 0 else 128]))
    n_caches = int(r.integers(1, 6))
    edge = [0, 1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 513]
    lens = [int(r.choice(edge)) if r.random() < 0.5 else int(r.integers(1, 2600)) for _ in range(n_caches)]
    caps = [max(L + int(r.integers(0, 70)), 1) for L in lens]
    pool, ref = _fill_pool(dev, r, caps, lens, heads, dh, group, scheme)
    acc0 = r.random(pool.rows).astype(np.float32)
    pool.acc.copy_(to_dev(acc0, dev))
    pool.ts.fill_(-3.0)
    scale_qk = 1.0 / np.sqrt(dh)
    qscale = float(r.choice([1.0, 2.0, 6.0]))
    q = r.standard_normal((n_caches, hq, dh)).astype(np.float32) * qscale
    if qdtype == "bf16":
        q = O.bf16_round(q)
    decay = float(r.choice([1.0, 0.9]))
    cut = int(r.integers(1, max(caps) + 1)) if r.random() < 0.3 else None
    lens_now = [min(L, cut) for L in lens] if cut else lens
    out = np_of(pool.decode_attend(to_dev(q, dev, qdtype), hq, now=7.0, decay=decay, max_len=cut))
    want, acc_ref = _decode_reference(ref, q, lens_now, acc0, heads, group, scale_qk, decay)
    for c, L in enumerate(lens_now):
        if L == 0:
            assert not out[c].any()
            continue
        rms = np.sqrt((want[c].astype(np.float64) ** 2).mean()) + 1e-12
        assert np.abs(out[c] - want[c]).max() <= 1e-3 * rms, (c, L, np.abs(out[c] - want[c]).max(), rms)
    np.testing.assert_allclose(np_of(pool.acc), acc_ref, rtol=1e-3, atol=1e-5)
    ts = np_of(pool.ts)
    touched = np.zeros(pool.rows, bool)
    for c, L in enumerate(lens_now):
        touched[ref.valid_rows(c)[:L]] = True
    assert (ts[touched] == 7.0).all() and (ts[~touched] == -3.0).all()
    # without the bookkeeping: same output path, accumulators untouched
    acc_now = np_of(pool.acc).copy()
    out_nb = np_of(pool.decode_attend(to_dev(q, dev, qdtype), hq, now=8.0, accumulate=False, max_len=cut))
    for c, L in enumerate(lens_now):
        if L:
            rms = np.sqrt((want[c].astype(np.float64) ** 2).mean()) + 1e-12
            assert np.abs(out_nb[c] - want[c]).max() <= 1e-3 * rms, (c, L)
    assert np.array_equal(np_of(pool.acc), acc_now)
