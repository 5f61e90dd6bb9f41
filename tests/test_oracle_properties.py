"""CPU: property tests (hypothesis) of the numpy restatement and its C twin.  They pin
what the mathematics fixes - ranges, error bounds, total orders, conservation laws,
invariances - on inputs a hand-written case would not think of."""
import numpy as np
import pytest
from hypothesis import assume, given, settings, strategies as st
from hypothesis.extra import numpy as hnp

import c_oracle as C
import pikv_oracle as O

F32 = np.float32
# magnitudes below 1e-6 are drawn as exact zeros: scales of 1e-9 and less run into float32 / float16
# underflow, which the formula inherits from the reference and which is pinned by known answers instead
finite = st.floats(min_value=-1e4, max_value=1e4, allow_nan=False, allow_infinity=False, width=32).map(
    lambda v: 0.0 if abs(v) < 1e-6 else v)
SET = settings(max_examples=80, deadline=None, derandomize=True)


@SET
@given(hnp.arrays(F32, st.tuples(st.integers(1, 5), st.sampled_from([32, 64, 128])), elements=finite),
       st.sampled_from([O.Q_I8_SYM, O.Q_I8_ASYM, O.Q_I4_ASYM, O.Q_I4_SYM]), st.sampled_from([32, 64]))
def test_quantise_range_and_error_bound(x, scheme, group):
    if x.shape[1] % group:
        group = 32
    bits, sym, qmin, qmax = O.scheme_info(scheme)
    # Left out: a constant group of magnitude >= 128, whose range of 1e-5 (the reference's rule for
    # max == min) vanishes in float32, so that the scale is 0 and the formula yields NaN.
    g3 = x.reshape(x.shape[0], -1, group)
    assume(((g3.max(-1) > g3.min(-1)) | (np.abs(g3).max(-1) < 100)).all())
    q, s, z = O.quantize_groups(x, group, scheme)
    assert q.min() >= qmin and q.max() <= qmax
    assert (s > 0).all()
    dq = O.dequantize_groups(q, s, z, group).astype(np.float64)
    step = np.repeat(s.astype(np.float64), group, axis=-1)
    err = np.abs(dq - x.astype(np.float64)) / step
    if not sym:
        # the range [min, max] maps onto [qmin, qmax]: rounding, plus the rounding of the zero point -
        # to an integer, and where the offset dwarfs the spread to what float32 (8-bit: integers beyond
        # 2^24 are even) or the widened 4-bit scale can hold
        assert err.max() <= (2.0 if bits == 8 else 1.6), err.max()
        assert np.abs(dq - x).max() <= 2.0 * s.max() + 1e-3 * np.abs(x).max()
    else:
        # +absmax lands one step past qmax and is clamped: at most one step there, half a step elsewhere
        assert err.max() <= 1.0 + 1e-3, err.max()
        inside = np.abs(x.astype(np.float64)) <= np.repeat(np.abs(x).reshape(x.shape[0], -1, group).max(-1), group,
                                                         axis=-1).astype(np.float64) * (1 - 1.0 / qmax)
        assert err[inside].max(initial=0.0) <= (0.5 + 1e-3 if bits == 8 else 0.51)


@SET
@given(hnp.arrays(F32, st.tuples(st.integers(1, 4), st.just(64)), elements=finite), st.sampled_from([0, 1, 2, 3]),
       st.floats(min_value=0.25, max_value=4.0))
def test_quantise_symmetric_codes_scale_with_input(x, scheme, factor):
    """Scaling the input by a power of two scales the float32 scale and leaves the 8-bit codes alone."""
    f = F32(2.0 ** round(np.log2(factor)))
    q1, s1, z1 = O.quantize_groups(x, 64, scheme)
    q2, s2, z2 = O.quantize_groups(x * f, 64, scheme)
    const = (x.max(axis=1) == x.min(axis=1))          # the max = min + 1e-5 rule is not scale-free
    if scheme in (O.Q_I8_SYM, O.Q_I8_ASYM):
        assert np.array_equal(q1[~const], q2[~const])
        assert np.array_equal((s1 * f)[~const], s2[~const])


@SET
@given(st.integers(1, 300), st.integers(1, 9), st.integers(0, 80), st.randoms(use_true_random=False))
def test_capacity_slots_conservation(A, E, cap, rnd):
    idx = np.array([rnd.randrange(E) for _ in range(A)], dtype=np.int32).reshape(-1, 1)
    slot, count = O.capacity_slots(idx, E, cap)
    s2, c2 = O.capacity_slots_loop(idx, E, cap)
    assert np.array_equal(slot, s2) and np.array_equal(count, c2)
    assert count.sum() == A
    for e in range(E):
        mine = slot.reshape(-1)[idx.reshape(-1) == e]
        kept = mine[mine >= 0]
        assert np.array_equal(kept, np.arange(min(count[e], cap)))       # dense, in token order
        assert (mine[len(kept):] == -1).all()                            # the surplus is the tail


@SET
@given(hnp.arrays(F32, st.tuples(st.integers(1, 6), st.integers(1, 40)),
                  elements=st.sampled_from([F32(v) for v in (-2, -0.0, 0.0, 0.5, 1, 1, 3, 7.25)])), st.integers(1, 8))
def test_topk_is_the_total_order(v, k):
    k = min(k, v.shape[1])
    got = O.topk_desc(v, k)
    for r in range(v.shape[0]):
        order = sorted(range(v.shape[1]), key=lambda i: (-float(v[r, i]), i))
        assert list(got[r]) == order[:k]
    small = O.topk_asc(v, k)
    for r in range(v.shape[0]):
        order = sorted(range(v.shape[1]), key=lambda i: (float(v[r, i]), i))
        assert list(small[r]) == order[:k]


@SET
@given(hnp.arrays(F32, st.tuples(st.integers(1, 8), st.integers(1, 12)), elements=st.floats(-30, 30, width=32)),
       st.integers(1, 4), st.floats(-5, 5, width=32))
def test_router_tail_invariants(lg, k, shift):
    k = min(k, lg.shape[1])
    probs, idx, w, _ = O.router_tail(lg, k)
    assert np.allclose(probs.sum(1), 1.0, atol=1e-5)
    assert np.allclose(w.sum(1), 1.0, atol=1e-5)
    assert all(len(set(r)) == k for r in idx)
    sel = np.take_along_axis(probs, idx, 1)
    assert (np.diff(sel, axis=1) <= 0).all()                                  # descending probabilities
    rest = probs.copy()
    np.put_along_axis(rest, idx.astype(np.int64), -1.0, 1)
    assert (rest.max(1) <= sel[:, -1]).all()                                  # nothing larger was left out
    assert (np.diff(np.take_along_axis(lg, idx, 1), axis=1) <= 0).all() or \
        (np.diff(sel, axis=1) == 0).any()                # logits descend too, except inside a run of equal probabilities
    # the C twin: the stable top-k of ITS probabilities (libm's expf and numpy's exp may round
    # differently), the same selection wherever numpy's probabilities are not within a rounding
    E = lg.shape[1]
    p2, _, i2, w2 = C.router(lg, np.eye(E, dtype=F32), None, k)    # identity gate: logits pass through
    from util import assert_topk_of_probs
    assert_topk_of_probs(i2, p2, k)
    same = (i2 == idx).all(axis=1)
    a = np.take_along_axis(probs, i2.astype(np.int64), 1)[~same]
    assert (np.abs(a - sel[~same]) <= 4 * np.spacing(sel[~same])).all()
    assert np.allclose(w2[same], w[same], atol=2e-6)
    # softmax is shift-invariant; a shift by a representable amount keeps the order
    lg2 = (lg.astype(np.float64) + np.float64(shift)).astype(F32)
    if np.array_equal((lg2.astype(np.float64) - np.float64(shift)).astype(F32), lg):
        p_s, idx_s, _, _ = O.router_tail(lg2, k)
        moved = (idx_s != idx).any(axis=1)               # only where probabilities sit within a rounding of each other
        a = np.take_along_axis(probs, idx_s.astype(np.int64), 1)[moved]
        assert (np.abs(a - sel[moved]) <= 4 * np.spacing(sel[moved])).all()


@SET
@given(st.integers(1, 60), st.integers(0, 70), st.integers(0, 70), st.randoms(use_true_random=False))
def test_h2o_keep_set_algebra(L, nh, nr, rnd):
    acc = np.array([rnd.randrange(6) / 4 for _ in range(L)], dtype=F32)
    ts = np.array([rnd.randrange(5) for _ in range(L)], dtype=F32)
    keep = O.h2o_keep(acc, ts, nh, nr)
    heavy = np.zeros(L, bool); heavy[O.topk_desc(acc[None], min(nh, L))[0]] = True
    recent = np.zeros(L, bool); recent[O.topk_desc(ts[None], min(nr, L))[0]] = True
    assert np.array_equal(keep, heavy | recent)
    assert max(min(nh, L), min(nr, L)) <= keep.sum() <= min(L, nh + nr)
    # budgets are monotone: a larger budget never drops a row
    assert (O.h2o_keep(acc, ts, nh + 1, nr) | ~keep).all()
    assert (O.h2o_keep(acc, ts, nh, nr + 1) | ~keep).all()
    # LRU: evicting n leaves L - min(n, L) rows, and every evicted row is no younger than every kept row
    k2 = O.lru_keep(ts, nr)
    assert k2.sum() == L - min(nr, L)
    if k2.any() and (~k2).any():
        assert ts[~k2].max() <= ts[k2].min()
    # C twin
    pool = C.CPool([L], 32, 32, O.Q_I8_SYM, with_v=False)
    pool.fill[:] = L
    pool.acc[:], pool.ts[:] = acc, ts
    flag, kidx, newlen = pool.evict(0, [nh], [nr], compact=False)
    assert np.array_equal(flag[:L].astype(bool), keep) and newlen[0] == keep.sum()
    assert np.array_equal(kidx[:keep.sum()], np.nonzero(keep)[0])


@SET
@given(st.integers(0, 50), st.randoms(use_true_random=False))
def test_compaction_is_stable_selection(L, rnd):
    keep = np.array([rnd.random() < 0.5 for _ in range(L)], dtype=bool)
    a = np.arange(L, dtype=np.int32).copy()
    b = (np.arange(L * 3, dtype=F32).reshape(L, 3) * 0.5).copy()
    a0, b0 = a.copy(), b.copy()
    m = O.compact(keep, a, b)
    assert m == keep.sum()
    assert np.array_equal(a[:m], a0[keep]) and np.array_equal(b[:m], b0[keep])


@SET
@given(hnp.arrays(F32, st.tuples(st.integers(1, 4), st.integers(1, 30)), elements=st.floats(-20, 20, width=32)))
def test_importance_is_a_distribution_per_head(s):
    p, imp = O.h2o_importance(s)
    assert np.allclose(p.sum(1), 1.0, atol=1e-5)
    assert abs(imp.sum() - s.shape[0]) < 1e-4 * s.shape[0]
    assert (imp >= 0).all()


def test_four_bit_zero_point_always_fits_half():
    """Constant and nearly constant groups (4-bit asymmetric): the zero point stays an exact half-precision
    integer and the values come back to within |x| / 2048 + half a step."""
    rows = np.stack([np.full(32, 1.0), np.full(32, -3.5), np.full(32, 1000.0), np.zeros(32),
                     1.0 + 1e-4 * np.arange(32) / 31, np.full(32, 0.04), -200.0 - 1e-3 * np.arange(32)]).astype(F32)
    q, s, z = O.quantize_groups(rows, 32, O.Q_I4_ASYM)
    assert (np.abs(z) <= 1025).all() and np.array_equal(z, np.rint(z))
    assert np.array_equal(z.astype(np.float16).astype(F32), z)
    dq = O.dequantize_groups(q, s, z, 32)
    bound = np.abs(rows).max(1, keepdims=True) / 2048 * 1.01 + 0.5 * s + 1e-7
    assert (np.abs(dq - rows) <= bound).all(), np.abs(dq - rows).max(1)
    assert not dq[3].any()
    # ordinary data is untouched by the rule: the zero point of a spread-out group is small
    r = np.random.default_rng(0).standard_normal((50, 32)).astype(F32)
    _, s2, z2 = O.quantize_groups(r, 32, O.Q_I4_ASYM)
    assert (np.abs(z2) <= 15).all()
    assert np.array_equal(s2, ((r.max(1) - r.min(1)) / F32(15)).astype(np.float16).astype(F32)[:, None])
