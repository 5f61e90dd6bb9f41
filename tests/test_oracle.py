"""Pins the CPU oracle (oracle/pikv_oracle.py and its independent C twin
oracle/pikv_oracle.c) without running the reference: hand-derived known-answer
vectors, closed forms, invariants that a dropped term / wrong sign / wrong index
would break, brute force on tiny inputs, and agreement of the two restatements
with each other.  The reference's own tests hold no golden vectors for this
path, so these checks are what fixes the oracle."""
import math

import numpy as np
import pytest

import c_oracle as CO
import pikv_oracle as O
from util import kv_like, rng

SCHEMES = [O.Q_I8_SYM, O.Q_I8_ASYM, O.Q_I4_ASYM, O.Q_I4_SYM]


# ---------------------------------------------------------------- known answers
def test_quant_known_answers():
    # asymmetric 8-bit on [-1,0,1]: scale = 2/255 (float32), -1/scale = -127.49999 -> zp 127
    q, s, z = O.quantize_groups(np.array([[-1, 0, 1]], np.float32), 3, O.Q_I8_ASYM)
    assert s[0, 0] == np.float32(2.0) / np.float32(255.0) == np.float32(0.007843137718737125)
    assert z[0, 0] == 127 and q.tolist() == [[0, 127, 254]]
    dq = O.dequantize_groups(q, s, z, 3)
    assert np.allclose(dq, [[-0.99607849, 0, 0.99607849]], atol=1e-8)
    # symmetric: scale = 2*absmax/255, NOT absmax/127
    q, s, z = O.quantize_groups(np.array([[-1, 0, 1]], np.float32), 3, O.Q_I8_SYM)
    assert s[0, 0] == np.float32(2.0) / np.float32(255.0) and z[0, 0] == 0
    assert q.tolist() == [[-127, 0, 127]]          # +-127.5 rounds to even = +-128 -> only +128 clamps
    q, _, _ = O.quantize_groups(np.array([[0.3, -0.7, 0.05, 0.7]], np.float32), 4, O.Q_I8_SYM)
    assert q.tolist() == [[55, -128, 9, 127]]
    # 4-bit asymmetric, metadata stored as float16: scale = half(0.2)
    q, s, z = O.quantize_groups(np.array([[0, 1, 2, 3]], np.float32), 4, O.Q_I4_ASYM)
    assert s[0, 0] == np.float32(np.float16(0.2)) and z[0, 0] == 0 and q.tolist() == [[0, 5, 10, 15]]
    # degenerate constant block: max := min + 1e-5
    q, s, z = O.quantize_groups(np.full((1, 8), 0.5, np.float32), 8, O.Q_I8_ASYM)
    assert s[0, 0] == (np.float32(0.5) + np.float32(1e-5) - np.float32(0.5)) / np.float32(255)
    # round half to even
    assert np.rint(np.float32(0.5)) == 0 and np.rint(np.float32(1.5)) == 2 and np.rint(np.float32(-127.5)) == -128


def test_budget_and_capacity_known_answers():
    assert O.h2o_budget(32768, 0.0625, 0.0078125) == (2048, 256)
    assert O.h2o_budget(5, 0.1, 0.1) == (1, 1)                  # max(1, int(0.5))
    assert O.compute_capacity(2, 64, 1.5, 2, 4) == 96
    assert O.compute_capacity(16, 2048, 1.25, 2, 8) == 10240
    assert O.pyramid_cache_sizes(128, 10, 5) == [128, 118, 108, 98, 88]
    kc = O.pyramid_keep_counts(131072, 32)
    assert kc[0] == 131072 and kc[-1] == 32768 and all(a >= b for a, b in zip(kc, kc[1:]))


# ---------------------------------------------------------------- quantisation invariants
@pytest.mark.parametrize("scheme", SCHEMES)
@pytest.mark.parametrize("group", [32, 128])
def test_quant_invariants(scheme, group):
    bits, sym, qmin, qmax = O.scheme_info(scheme)
    r = rng(scheme)
    x = kv_like(r, 200, 256, dtype="bf16")
    q, s, z = O.quantize_groups(x, group, scheme)
    assert q.min() >= qmin and q.max() <= qmax
    xg = x.reshape(200, -1, group)
    qg = q.reshape(200, -1, group)
    dq = O.dequantize_groups(q, s, z, group).reshape(xg.shape)
    # reconstruction error <= scale/2 wherever the code did not clamp (+ float32 slack)
    inner = (qg > qmin) & (qg < qmax)
    err = np.abs(xg - dq)
    assert (err[inner] <= (0.5 * s[..., None] * (1 + 1e-5) + 1e-6).repeat(group, -1)[inner]).all()
    if not sym:
        # the minimum maps to qmin (zero point definition) and the maximum to qmax (+-1 for half scales)
        amin = xg.argmin(-1)
        assert (np.take_along_axis(qg, amin[..., None], -1)[..., 0] <= qmin + (1 if bits == 4 else 0)).all()
        amax = xg.argmax(-1)
        assert (np.take_along_axis(qg, amax[..., None], -1)[..., 0] >= qmax - 1).all()
    else:
        # symmetric: codes are an odd function of the input
        q2, s2, _ = O.quantize_groups(-x, group, scheme)
        assert np.array_equal(s, s2)
        flip = (q2 == -q) | (np.abs(q) == -qmin) | (np.abs(q2) == -qmin)
        assert flip.all()
    # monotone: a larger input never gets a smaller code inside one group
    order = np.argsort(xg, axis=-1)
    assert (np.diff(np.take_along_axis(qg, order, -1), axis=-1) >= 0).all()
    # scaling the input by 2 doubles the scale and keeps the codes (exact in float32);
    # not for half metadata, where the zero point may round differently
    if bits == 8:
        qd, sd, zd = O.quantize_groups(2 * x, group, scheme)
        assert np.array_equal(qd, q) and np.array_equal(sd, 2 * s)


def test_int4_pack_roundtrip_and_layout():
    c = np.arange(-8, 8, dtype=np.int16)[None, :]
    p = O.pack_int4(c)
    assert p.shape == (1, 8)
    assert p[0, 0] == ((-8 & 0xF) | ((-7 & 0xF) << 4))           # low nibble = even element
    assert np.array_equal(O.unpack_int4(p, signed=True), c)
    u = np.arange(16, dtype=np.int16)[None, :]
    assert np.array_equal(O.unpack_int4(O.pack_int4(u), signed=False), u)


def test_half_conversion_matches_numpy():
    r = rng(3)
    v = np.concatenate([r.standard_normal(2000) * 10.0 ** r.integers(-9, 6, 2000),
                        [0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25, 3e-8, 6.1e-5]]).astype(np.float32)
    for f in v:
        h = CO.lib().pko_f32_to_half(float(f))
        want = O._to_half_sat(np.array([f], np.float32))[0]
        assert h == want.view(np.uint16), f
        assert CO.lib().pko_half_to_f32(h) == np.float32(want)


def test_fakequant_reference_domain_is_blockwise():
    """min/max over ALL rows of a 128-column block: changing one row's outlier
    changes every row's codes in that block and no other block."""
    r = rng(9)
    x = r.standard_normal((64, 256)).astype(np.float32)
    dq, st, mse = O.fakequant_colblocks(x, 128)
    y = x.copy(); y[5, 3] = 50.0
    dq2, st2, _ = O.fakequant_colblocks(y, 128)
    assert st2[0, 1] == 50.0 and np.array_equal(st[1], st2[1])
    assert np.array_equal(dq[:, 128:], dq2[:, 128:]) and not np.array_equal(dq[0, :128], dq2[0, :128])
    assert np.allclose(mse, ((x - dq) ** 2).reshape(64, 2, 128).mean((0, 2)), rtol=1e-6)
    # per-row stored-code algebra of the kernel facade: dq = q*s + min
    q, dq3, s, mn = O.quant8_minshift(x)
    assert q.min() == 0 and q.max() == 255 and np.abs(dq3 - x).max() <= s.max() * 0.5001


# ---------------------------------------------------------------- router
def test_softmax_and_topk_closed_forms():
    lg = np.log(np.array([[1, 2, 3, 4]], np.float32))
    probs, idx, w, _ = O.router_tail(lg, 2)
    assert np.allclose(probs, [[0.1, 0.2, 0.3, 0.4]], atol=1e-6)
    assert idx.tolist() == [[3, 2]] and np.allclose(w, [[4 / 7, 3 / 7]], atol=1e-6)
    # ties -> lowest index; all-equal logits give uniform probs
    probs, idx, w, _ = O.router_tail(np.zeros((1, 4), np.float32), 2)
    assert idx.tolist() == [[0, 1]] and np.allclose(probs, 0.25) and np.allclose(w, 0.5)
    # mask: masked experts never win, probs are exactly 0
    probs, idx, _, _ = O.router_tail(np.array([[5, 1, 0, 3]], np.float32), 2,
                                     expert_mask=np.array([0, 1, 1, 1], np.float32))
    assert idx.tolist() == [[3, 1]] and probs[0, 0] == 0
    # EPLB order: divide by temperature first, then multiply by the expert weight
    lg = np.array([[1.0, 2.0]], np.float32)
    out = O.scale_logits(lg, temperature=0.5, expert_scale=np.array([3.0, 1.0], np.float32))
    assert out.tolist() == [[6.0, 4.0]]
    # two-gate select (PiKV router)
    out = O.scale_logits(np.array([[1.0], [1.0]], np.float32), logits_b=np.array([[9.0], [9.0]], np.float32),
                         select=np.array([1, 0]))
    assert out.tolist() == [[1.0], [9.0]]
    # renorm epsilon variant
    _, _, w, _ = O.router_tail(np.log(np.array([[1, 1]], np.float32)), 2, renorm_eps=1.0)
    assert np.allclose(w, 0.25)


def test_topk_is_taken_on_probabilities():
    """core/single/pikv_routing.py:73-76: torch.topk(softmax(logits)).  Distinct logits whose
    float32 probabilities coincide tie, the lower expert wins (the build's tie rule), although
    its logit is the smaller one; without the softmax (core/single/pikv_kernels.py:97) the
    logits decide.  Both restatements."""
    hi = np.float32(2.0 ** -10)
    lo = np.nextafter(hi, np.float32(0), dtype=np.float32)
    lg = np.array([[lo, hi, -3.0, -4.0], [-3.0, hi, -4.0, lo]], np.float32)
    probs, idx, w, _ = O.router_tail(lg, 2)
    assert probs[0, 0] == probs[0, 1] and probs[1, 1] == probs[1, 3]
    assert idx.tolist() == [[0, 1], [1, 3]]
    assert O.router_tail(lg, 1)[1].tolist() == [[0], [1]]
    assert O.router_tail(lg, 1, use_softmax=False)[1].tolist() == [[1], [1]]
    p2, _, i2, _ = CO.router(lg, np.eye(4, dtype=np.float32), None, 2)
    assert p2[0, 0] == p2[0, 1] and i2.tolist() == [[0, 1], [1, 3]]
    # rows whose probabilities are NaN (a NaN or +inf logit) select experts 0..k-1
    bad = np.array([[0.0, np.nan, 1.0, 2.0], [0.0, 1.0, np.inf, 2.0]], np.float32)
    with np.errstate(invalid="ignore"):
        assert O.router_tail(bad, 2)[1].tolist() == [[0, 1], [0, 1]]
    assert CO.router(bad, np.eye(4, dtype=np.float32), None, 2)[2].tolist() == [[0, 1], [0, 1]]


def test_capacity_slots_vs_literal_loop_and_invariants():
    r = rng(12)
    for (T, k, E, cap) in [(50, 2, 4, 10), (64, 8, 64, 3), (31, 1, 3, 100), (40, 2, 4, 0)]:
        idx = np.stack([r.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        s1, c1 = O.capacity_slots(idx, E, cap)
        s2, c2 = O.capacity_slots_loop(idx, E, cap)
        s3, c3 = CO.capacity_slots(idx, E, cap)
        assert np.array_equal(s1, s2) and np.array_equal(c1, c2)
        assert np.array_equal(s1, s3) and np.array_equal(c1, c3)
        flat, fs = idx.reshape(-1), s1.reshape(-1)
        for e in range(E):
            got = fs[flat == e]
            kept = got[got >= 0]
            assert kept.size == min(c1[e], cap)
            assert np.array_equal(kept, np.arange(kept.size))       # 0..kept-1 in token order
            assert (got[kept.size:] == -1).all()                    # overflow only after the expert is full
    disp, comb = O.dense_dispatch_combine(idx, np.full(idx.shape, 0.5, np.float32), s1, E, max(cap, 1))
    assert disp.sum() == (s1 >= 0).sum()


def test_router_c_and_numpy_agree():
    r = rng(21)
    T, H, E, k = 300, 128, 8, 2
    x = O.bf16_round(r.standard_normal((T, H)).astype(np.float32))
    w = O.bf16_round((0.02 * r.standard_normal((E, H))).astype(np.float32))
    b = (0.1 * r.standard_normal(E)).astype(np.float32)
    sc = (0.5 + r.random(E)).astype(np.float32)
    probs_c, logits_c, idx_c, w_c = CO.router(O.f32_to_bf16_bits(x), O.f32_to_bf16_bits(w), b, k,
                                               temperature=0.7, expert_scale=sc)
    lg = O.gate_logits(x, w, b)
    probs, idx, wts, lgs = O.router_tail(lg, k, temperature=0.7, expert_scale=sc)
    assert np.array_equal(logits_c, lgs)
    assert np.array_equal(idx_c, idx)
    assert np.allclose(probs_c, probs, atol=1e-6) and np.allclose(w_c, wts, atol=1e-6)
    assert np.allclose(wts.sum(1), 1, atol=1e-6)


# ---------------------------------------------------------------- caches
@pytest.mark.parametrize("scheme,group", [(O.Q_I8_SYM, 64), (O.Q_I4_ASYM, 32), (O.Q_I8_ASYM, 128), (O.Q_I4_SYM, 64)])
def test_scatter_c_and_numpy_agree(scheme, group):
    r = rng(scheme + 40)
    E, k, D = 4, 2, 256
    caps = [30, 64, 5, 40]
    ref = O.CachePool(caps, D, group, scheme)
    cp = CO.CPool(caps, D, group, scheme)
    for step, T in enumerate([48, 30]):
        cap = O.compute_capacity(1, T, 1.5, k, E)
        idx = np.stack([r.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        slot, count = O.capacity_slots(idx, E, cap)
        ks = kv_like(r, T, D, dtype="bf16")
        vs = kv_like(r, T, D, dtype="bf16")
        ref.quant_scatter(ks, vs, idx, slot, k, now=step + 1.0)
        cp.quant_scatter(O.f32_to_bf16_bits(ks), O.f32_to_bf16_bits(vs), idx, slot, k, now=step + 1.0)
        ref.advance(count, cap); cp.advance(count, cap)
    assert np.array_equal(ref.fill, cp.fill)
    bits = O.scheme_info(scheme)[0]
    for c in range(E):
        rows = ref.valid_rows(c)
        cc = cp.k_codes[rows]
        cc = O.unpack_int4(cc, signed=(scheme == O.Q_I4_SYM)) if bits == 4 else cc.astype(np.int16)
        assert np.array_equal(cc, ref.k_codes[rows])
        sc = cp.k_scale[rows].view(np.float16).astype(np.float32) if bits == 4 else cp.k_scale[rows]
        assert np.array_equal(sc, ref.k_scale[rows])
        assert np.array_equal(cp.ts[rows], ref.ts[rows])
        # a row holds the codes of the token that was routed there: dequantise and compare with the source
    dq = cp.gather_dequant("k")
    for c in range(E):
        rows = ref.valid_rows(c)
        want = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        assert np.array_equal(dq[rows], want)


def test_cache_append_brute_force():
    """List-based model of core/single/cache_scheduling.py:429-436 on a tiny
    pool: per expert, kept assignments in token order, truncated at the cache."""
    r = rng(77)
    E, k, D, group = 3, 2, 32, 32
    caps = [4, 9, 2]
    ref = O.CachePool(caps, D, group, O.Q_I8_SYM, with_v=False)
    lists = [[] for _ in range(E)]
    src_all = []
    for step in range(3):
        T = 5
        idx = np.stack([r.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        cap = O.compute_capacity(1, T, 1.0, k, E)
        slot, count = O.capacity_slots_loop(idx, E, cap)
        ks = r.standard_normal((T, D)).astype(np.float32)
        ref.quant_scatter(ks, None, idx, slot, k)
        ref.advance(count, cap)
        used = [0] * E
        for t in range(T):
            for j in range(k):
                e = int(idx[t, j])
                if used[e] < cap:
                    used[e] += 1
                    if len(lists[e]) < caps[e]:
                        lists[e].append(ks[t])
    for e in range(E):
        assert ref.fill[e] == len(lists[e])
        rows = ref.valid_rows(e)
        want = O.quantize_groups(np.stack(lists[e]), group, O.Q_I8_SYM)[0] if lists[e] else np.zeros((0, D))
        assert np.array_equal(ref.k_codes[rows], want)


# ---------------------------------------------------------------- read path
def test_scores_importance_closed_forms():
    r = rng(5)
    n_kv, n_q, dh, N = 2, 4, 16, 37
    k_hat = r.standard_normal((N, n_kv * dh)).astype(np.float32)
    q = r.standard_normal((n_q, dh)).astype(np.float32)
    s = O.attention_scores(q, k_hat, n_kv, 1 / math.sqrt(dh))
    # GQA mapping: head h reads kv head h // rep; check one entry by hand
    h, n = 3, 11
    want = float(np.dot(q[h].astype(np.float64), k_hat[n, 16:32].astype(np.float64)) / math.sqrt(dh))
    assert abs(s[h, n] - want) < 1e-6
    probs, imp = O.h2o_importance(s)
    assert np.allclose(probs.sum(1), 1, atol=1e-6) and abs(imp.sum() - n_q) < 1e-5
    # a key equal to a scaled query dominates its head
    k_hat[7, :16] = 10 * q[0]
    s = O.attention_scores(q, k_hat, n_kv, 1 / math.sqrt(dh))
    assert s[0].argmax() == 7
    # accumulate: acc += imp, ts = now; decay multiplies first
    acc, ts = np.ones(N, np.float32), np.zeros(N, np.float32)
    O.h2o_accumulate(acc, ts, np.arange(N), imp, 3.0, decay=0.5)
    assert np.allclose(acc, 0.5 + imp) and (ts == 3).all()


def test_read_path_c_and_numpy_agree():
    r = rng(8)
    n_kv, n_q, dh, group, scheme = 2, 8, 64, 32, O.Q_I4_ASYM
    D = n_kv * dh
    caps, lens = [70, 20], [65, 3]
    cp = CO.CPool(caps, D, group, scheme, with_v=False)
    ref = O.CachePool(caps, D, group, scheme, with_v=False)
    ks = kv_like(r, sum(lens), D, dtype="bf16")
    cid = np.repeat(np.arange(2, dtype=np.int32), lens)
    slot = np.concatenate([np.arange(l, dtype=np.int32) for l in lens])
    cp.quant_scatter(O.f32_to_bf16_bits(ks), None, cid, slot, 1); cp.advance(lens)
    ref.quant_scatter(ks, None, cid, slot, 1); ref.advance(lens)
    q = r.standard_normal((2, n_q, dh)).astype(np.float32)
    sc, imp = cp.scores_h2o(q, n_kv, n_q, dh, 1 / math.sqrt(dh), now=2.0)
    for c in range(2):
        rows = ref.valid_rows(c)
        kh = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], group)
        s = O.attention_scores(q[c], kh, n_kv, 1 / math.sqrt(dh))
        assert np.allclose(sc[c, :, :lens[c]], s, atol=1e-6)
        _, i_ref = O.h2o_importance(s)
        assert np.allclose(imp[c, :lens[c]], i_ref, atol=1e-6)
        assert np.allclose(cp.acc[rows], i_ref, atol=1e-6) and (cp.ts[rows] == 2).all()


# ---------------------------------------------------------------- eviction
def test_select_brute_force_and_c_twin():
    r = rng(14)
    for L in [1, 2, 9, 40]:
        acc = (np.round(r.random(L) * 4) / 4).astype(np.float32)     # many ties
        ts = r.integers(0, 5, L).astype(np.float32)
        for nh, nr in [(1, 1), (3, 2), (L, 0), (0, 0)]:
            keep = O.h2o_keep(acc, ts, nh, nr)
            for i in range(L):
                ba = sum((acc[j] > acc[i]) or (acc[j] == acc[i] and j < i) for j in range(L))
                bt = sum((ts[j] > ts[i]) or (ts[j] == ts[i] and j < i) for j in range(L))
                assert keep[i] == (ba < nh or bt < nr)
            assert keep.sum() <= min(L, nh + nr) and (nh == 0 or keep.sum() >= min(nh, L))
        ne = L // 3
        keep = O.lru_keep(ts, ne)
        assert keep.sum() == L - ne
        for i in range(L):
            b = sum((ts[j] < ts[i]) or (ts[j] == ts[i] and j < i) for j in range(L))
            assert keep[i] == (b >= ne)
    # C twin on a pool
    caps, lens = [40, 16], [40, 9]
    cp = CO.CPool(caps, 32, 32, O.Q_I8_SYM, with_v=False)
    ks = r.standard_normal((sum(lens), 32)).astype(np.float32)
    cid = np.repeat(np.arange(2, dtype=np.int32), lens)
    slot = np.concatenate([np.arange(l, dtype=np.int32) for l in lens])
    cp.quant_scatter(ks, None, cid, slot, 1); cp.advance(lens)
    cp.acc[:] = np.round(r.random(cp.rows) * 4) / 4
    cp.ts[:] = r.integers(0, 5, cp.rows)
    before = (cp.k_codes.copy(), cp.acc.copy(), cp.ts.copy())
    flag, kidx, new_len = cp.evict(0, [5, 2], [3, 1])
    for c in range(2):
        b, L = int(cp.base[c]), lens[c]
        keep = O.h2o_keep(before[1][b:b + L], before[2][b:b + L], [5, 2][c], [3, 1][c])
        assert np.array_equal(flag[b:b + L].astype(bool), keep)
        assert new_len[c] == keep.sum()
        assert np.array_equal(kidx[b:b + new_len[c]], np.nonzero(keep)[0])
    # compaction is stable and in place: survivors keep their relative order
    assert (np.diff(kidx[:new_len[0]]) > 0).all()
    assert np.array_equal(cp.k_codes[:new_len[0]], before[0][kidx[:new_len[0]]])
    assert np.array_equal(cp.acc[:new_len[0]], before[1][kidx[:new_len[0]]])
    assert np.array_equal(cp.fill, new_len)


def test_compact_is_stable_and_in_place():
    keep = np.array([0, 1, 1, 0, 1, 0, 0, 1], bool)
    a = np.arange(8, dtype=np.float32)
    b = np.arange(16, dtype=np.int16).reshape(8, 2)
    m = O.compact(keep, a, b)
    assert m == 4 and a[:4].tolist() == [1, 2, 4, 7] and b[:4, 0].tolist() == [2, 4, 8, 14]


def test_other_policies_known_answers():
    """StreamingLLM / QUEST / FlexGen / LRU+ restatements against hand-computed values
    and a brute-force ranking."""
    # StreamingLLM: 10 rows, 2 start + 3 recent -> rows 0,1 and 7,8,9
    assert O.streaming_keep(10, 2, 3).tolist() == [True, True] + [False] * 5 + [True] * 3
    # window larger than the cache: everything stays
    assert O.streaming_keep(5, 4, 124).all()
    # QUEST: quality .5, used twice, last touched 2 ticks ago, decay .5 -> .5*2*.25 = .25
    u = O.quest_utility([0.5, 1.0, 0.0], [2, 1, 5], [3, 5, 5], 5, 0.5)
    assert np.allclose(u, [0.25, 1.0, 0.0])
    assert O.quest_evict(u, 0.3, 1).tolist() == [True, False, True]     # two below the threshold
    assert O.quest_evict(u, 0.1, 2).tolist() == [True, False, True]     # too few below: the two lowest
    # FlexGen: freq/cost
    b = O.flexgen_benefit([4, 1, 9, 0], [2, 1, 3, 1])
    assert b.tolist() == [2.0, 1.0, 3.0, 0.0]
    assert O.evict_lowest(b, 2).tolist() == [False, True, False, True]
    # LRU+: weights .3/.3/.4, times [0,5,10], freq [1,2,4], importance [1,0,.5]
    p = O.lruplus_priority([0, 5, 10], [1, 2, 4], [1.0, 0.0, 0.5])
    assert np.allclose(p, [0.3 * 0.25 + 0.4, 0.3 * 0.5 + 0.3 * 0.5, 0.3 + 0.3 + 0.2], atol=1e-6)
    # lowest-n against an O(n^2) ranking with ties (lower index goes first)
    r = np.random.default_rng(11)
    s = (np.round(r.random(40) * 6) / 6).astype(np.float32)
    for n in (0, 1, 7, 40):
        ev = O.evict_lowest(s, n)
        for i in range(40):
            before = sum((s[j] < s[i]) or (s[j] == s[i] and j < i) for j in range(40))
            assert ev[i] == (before < n)


def test_adakv_duo_known_answers():
    s = np.array([0.1, 0.9, 0.5, 0.9, -1.0, 0.3, 0.2, 0.8, 0.0, 0.4], dtype=np.float32)
    # keep 5 of 10; safeguard 1 (the first 0.9), then the next four: 0.9(idx 3), 0.8, 0.5, 0.4
    k = O.adakv_keep(s, 0.5, 0.2)
    assert np.nonzero(k)[0].tolist() == [1, 2, 3, 7, 9]
    # the two-stage pick equals the plain top-num_keep under the tie rule
    r = np.random.default_rng(2)
    for _ in range(20):
        x = (np.round(r.standard_normal(37) * 3) / 3).astype(np.float32)
        kk = O.adakv_keep(x, 0.4, 0.3)
        want = np.zeros(37, dtype=bool)
        want[O.topk_desc(x[None, :], int(37 * 0.6))[0]] = True
        assert np.array_equal(kk, want)
    assert O.duo_keep(10, 2, 3).tolist() == [True, True] + [False] * 5 + [True] * 3
    assert O.duo_keep(4, 3, 3).all()


def test_fakequant_preset_known_answers():
    """Pre-calibrated fake quantisation (core/single/pikv_compression.py:455-472): hand-computed
    values, clamping at both ends, and the identity with the block form when it is handed the
    block's own parameters."""
    x = np.array([[1.3, -2.0, 200.0, 0.26, 0.24]], dtype=np.float32)
    dq, mse = O.fakequant_preset(x, 0.5, 3.0, 5)
    # 1.3/0.5+3 = 5.6 -> 6 -> 1.5 ; -2/0.5+3 = -1 -> 0 -> -1.5 ; 403 -> 255 -> 126 ;
    # 0.52+3 -> 4 -> 0.5 ; 0.48+3 -> 3 -> 0
    assert dq.tolist() == [[1.5, -1.5, 126.0, 0.5, 0.0]]
    want = np.mean((x.astype(np.float64) - dq.astype(np.float64)) ** 2)
    assert abs(mse[0] - want) < 1e-12
    dq, _ = O.fakequant_preset(np.array([[-3.0, 0.26, 9.0]], np.float32), 0.5, 0.0, 3, bits=4, symmetric=True)
    assert dq.tolist() == [[-3.0, 0.5, 3.5]]          # 18 -> 7 -> 3.5; -6 stays
    r = np.random.default_rng(5)
    y = r.standard_normal((50, 96)).astype(np.float32)
    ref, st, mse_ref = O.fakequant_colblocks(y, 96)
    dq, mse = O.fakequant_preset(y, st[0, 2], st[0, 3], 96)
    assert np.array_equal(dq, ref) and np.allclose(mse, mse_ref, rtol=0, atol=0)


def _rn32(fr):
    """Round an exact rational to the nearest float32, ties to even, without using any
    float32 arithmetic: the independent arbiter of what one IEEE operation returns."""
    from fractions import Fraction
    fr = Fraction(fr)
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)
    q = a / Fraction(2) ** (e - 23)                 # significand in units of the last place
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return np.float32(sign * float(Fraction(n) * Fraction(2) ** (e - 23)))


def test_fakequant_colblocks_scale_and_zero_known_answers():
    """core/single/pikv_compression.py:396-429 on a block: the block-wide scale and zero point
    by hand.  [-1, 0, 1] (one row, then spread over three rows of one column block):
    scale = RN(2/255) = 0.007843137718737125; -1/scale = -127.49999 in float32 (the real quotient
    is -127.5 only for the unrounded scale), so round() gives -127 and zero = 0 - (-127) = 127
    (floor would give 128; a range of 256 instead of 255 gives scale 0.0078125 and zero 128).
    codes 0, 127, 254 -> dq = (q - 127) * scale."""
    from fractions import Fraction as Fr
    s_lit = np.float32(0.007843137718737125)
    assert _rn32(Fr(2, 255)) == s_lit
    assert _rn32(Fr(-1) / Fr(float(s_lit))) == np.float32(-127.49999237060547)   # not -127.5
    for x in (np.array([[-1.0, 0.0, 1.0]], np.float32),
              np.array([[-1.0], [0.0], [1.0]], np.float32)):
        dq, st, mse = O.fakequant_colblocks(x, x.shape[1])
        assert st.shape == (1, 4)
        assert st[0, 0] == -1.0 and st[0, 1] == 1.0
        assert st[0, 2] == s_lit, st
        assert st[0, 3] == 127.0, st
        want = np.array([-127, 0, 127], np.float32) * s_lit
        assert want[2] == np.float32(0.9960784912109375)
        assert np.array_equal(dq.reshape(-1), want)
        assert abs(mse[0] - 2 * (1 - 0.9960784912109375) ** 2 / 3) < 1e-15
    # min and max in different rows AND interior values: [[-1, 0.25], [0.5, 1]] as one block.
    # 0.25/scale = 31.874998 -> +127 = 158.875 -> 159 -> 32*scale; 0.5/scale = 63.749996 -> 190.75 -> 191
    dq, st, _ = O.fakequant_colblocks(np.array([[-1.0, 0.25], [0.5, 1.0]], np.float32), 2)
    assert st[0, 2] == s_lit and st[0, 3] == 127.0
    assert np.array_equal(dq, np.array([[-127, 32], [64, 127]], np.float32) * s_lit)
    # two column blocks with different parameters: block 0 = {0, 51} -> scale 0.2, zero 0;
    # block 1 = {10, 265} -> scale 1, zero = 0 - 10 = -10, codes round(x - 10), dq = code + 10
    x = np.array([[0.0, 10.0], [51.0, 265.0], [25.5, 137.5]], np.float32)
    dq, st, _ = O.fakequant_colblocks(x, 1)
    assert st[0, 2] == _rn32(Fr(51, 255)) == np.float32(0.2) and st[0, 3] == 0.0
    assert st[1, 2] == 1.0 and st[1, 3] == -10.0
    # 25.5/0.2f: the real quotient 127.4999981 rounds to the float32 127.5 -> half to even -> 128
    assert _rn32(Fr(51, 2) / Fr(float(np.float32(0.2)))) == np.float32(127.5)
    assert dq[2, 0] == np.float32(128.0) * np.float32(0.2) and dq[1, 0] == np.float32(255.0) * np.float32(0.2)
    assert dq[:, 1].tolist() == [10.0, 265.0, 138.0]                    # 137.5 - 10 = 127.5 -> 128 (even) -> 138
    # 4-bit asymmetric and the symmetric variants (core/single/module/pikv_compression.py:945-1012)
    dq, st, _ = O.fakequant_colblocks(np.array([[0.0, 1.0, 2.0, 3.75]], np.float32), 4, bits=4)
    assert st[0, 2] == 0.25 and st[0, 3] == 0.0 and dq.tolist() == [[0.0, 1.0, 2.0, 3.75]]
    dq, st, _ = O.fakequant_colblocks(np.array([[0.3, -0.7, 0.05, 0.7]], np.float32), 4, symmetric=True)
    assert st[0, 2] == _rn32(Fr(float(np.float32(2.0) * np.float32(0.7))) / 255) and st[0, 3] == 0.0
    assert np.array_equal(dq, np.array([[55, -128, 9, 127]], np.float32) * st[0, 2])
    dq, st, _ = O.fakequant_colblocks(np.array([[-3.75, 1.0, 0.26, 3.0]], np.float32), 4, bits=4, symmetric=True)
    assert st[0, 2] == 0.5 and dq.tolist() == [[-4.0, 1.0, 0.5, 3.0]]   # -7.5 -> -8 (even, in range) -> -4; 0.52 -> 1


@pytest.mark.parametrize("bits,symmetric", [(8, False), (8, True), (4, False), (4, True)])
def test_fakequant_one_row_block_equals_group_quantisation(bits, symmetric):
    """With one row, the block domain of QuantizedCompressor.forward IS a per-row group: the result
    must be quantize_groups + dequantize_groups (pinned by the known answers above) bit for bit.
    The 4-bit group format rounds its metadata to float16, so those rows are built with extremes
    whose scale and zero point are float16 numbers (range 15 * 2^-k)."""
    scheme = {(8, False): O.Q_I8_ASYM, (8, True): O.Q_I8_SYM,
              (4, False): O.Q_I4_ASYM, (4, True): O.Q_I4_SYM}[(bits, symmetric)]
    r = rng(100 + bits + symmetric)
    for trial in range(40):
        G = [16, 32, 128][trial % 3]
        if bits == 8:
            x = (r.standard_normal((1, 3 * G)) * r.choice([1e-3, 1.0, 30.0])).astype(np.float32)
            if trial % 5 == 0:
                x += np.float32(r.uniform(-4, 4))
        else:
            step = np.float32(2.0 ** -r.integers(0, 6))
            lo = np.float32(-r.integers(0, 16)) * step if not symmetric else np.float32(-7.5) * step
            x = (lo + r.uniform(0, 15, (1, 3 * G)).astype(np.float32) * step).astype(np.float32)
            for b in range(3):
                x[0, b * G] = lo
                x[0, b * G + 1] = lo + np.float32(15) * step
        dq, st, _ = O.fakequant_colblocks(x, G, bits=bits, symmetric=symmetric)
        q, s, z = O.quantize_groups(x, G, scheme)
        want = O.dequantize_groups(q, s, z, G)
        assert np.array_equal(st[:, 2], s[0]) and np.array_equal(st[:, 3], z[0]), (trial, st, s, z)
        assert np.array_equal(dq, want), trial


def test_scale_logits_order_and_penalty_known_answers():
    """The two reference copies scale logits in different orders and mask with different
    penalties; in float32 the orders differ in the last bit.  lg = 2.1f, T = 0.7f, w = 1.1f:
      core/single/pikv_routing.py:653-656         (lg / T) * w = 3.3000001907348633
      core/single/module/pikv_routing.py:596-600  (lg * w) / T = 3.299999952316284
    (both literals re-derived below with exact rational arithmetic, one rounding per operation).
    Penalties: single adds (1 - m) * -1e9 (:68-70), module adds (1 - m) * finfo(float32).min
    (:133-134)."""
    from fractions import Fraction as Fr
    lg, T, w = np.float32(2.1), np.float32(0.7), np.float32(1.1)
    single = _rn32(Fr(float(_rn32(Fr(float(lg)) / Fr(float(T))))) * Fr(float(w)))
    module = _rn32(Fr(float(_rn32(Fr(float(lg)) * Fr(float(w))))) / Fr(float(T)))
    assert single == np.float32(3.3000001907348633) and module == np.float32(3.299999952316284)
    assert single != module
    es = np.array([w, 1.0], np.float32)
    row = np.array([[lg, lg]], np.float32)
    out = O.scale_logits(row, temperature=float(T), expert_scale=es)
    assert out[0, 0] == single and out[0, 1] == _rn32(Fr(float(lg)) / Fr(float(T)))
    out = O.scale_logits(row, temperature=float(T), expert_scale=es, module_arithmetic=True)
    assert out[0, 0] == module and out[0, 1] == _rn32(Fr(float(lg)) / Fr(float(T)))
    # the C twin (single/ order only) through an identity gate
    got = CO.router(row, np.eye(2, dtype=np.float32), None, 1, temperature=float(T), expert_scale=es)[1]
    assert got[0, 0] == single
    # penalties: 5 - 1e9 rounds to -1e9 (spacing 64 there); 5 + finfo.min rounds to finfo.min
    m = np.array([0.0, 1.0], np.float32)
    out = O.scale_logits(np.array([[5.0, -5.0]], np.float32), expert_mask=m)
    assert out.tolist() == [[-1e9, -5.0]]
    out = O.scale_logits(np.array([[5.0, -5.0]], np.float32), expert_mask=m, module_arithmetic=True)
    assert out.tolist() == [[-3.4028234663852886e+38, -5.0]]
    # a NEGATIVE masked logit overflows past finfo.min only when it is huge; an ordinary one stays finite
    out = O.scale_logits(np.array([[-5.0, 1.0]], np.float32), expert_mask=m, module_arithmetic=True)
    assert out[0, 0] == np.float32(-3.4028234663852886e+38) and np.isfinite(out[0, 0])
    # the penalty is added after scaling in both copies: (lg / T) * w - 1e9, not (lg - 1e9) / T * w
    out = O.scale_logits(np.array([[5.0, 1.0]], np.float32), temperature=0.5,
                         expert_scale=np.array([2.0, 1.0], np.float32), expert_mask=m)
    assert out.tolist() == [[-1e9, 2.0]]


# ---------------------------------------------------------------- hand-computed pins of the facade / caller helpers
def test_quant8_minshift_known_answers():
    """core/single/pikv_kernels.py:215-232 by hand.  Row 0: min 0, max 255, s = 1, so the
    code is the value rounded half to even.  Row 1 is row 0 shifted by +10: same codes,
    dq = code + 10 (a dropped '- min' or '+ min' fails here).  Row 2: min 1, max 128.5,
    s = 0.5; (1.75-1)/0.5 = 1.5 -> 2, (2.25-1)/0.5 = 2.5 -> 2, dq = 2*0.5 + 1 = 2.  Row 3 is
    constant: s = 0, 0/0 = NaN -> code 0, dq = min."""
    x = np.array([[0.0, 255.0, 127.4, 127.5, 128.5, 3.0],
                  [10.0, 265.0, 137.4, 137.5, 138.5, 13.0],
                  [1.0, 128.5, 1.75, 2.25, 64.75, 1.0],
                  [3.0, 3.0, 3.0, 3.0, 3.0, 3.0]], np.float32)
    q, dq, s, mn = O.quant8_minshift(x)
    assert q.dtype == np.uint8 and s.shape == (4, 1) and mn.shape == (4, 1)
    assert s[:, 0].tolist() == [1.0, 1.0, 0.5, 0.0] and mn[:, 0].tolist() == [0.0, 10.0, 1.0, 3.0]
    assert q[0].tolist() == [0, 255, 127, 128, 128, 3]
    assert q[1].tolist() == [0, 255, 127, 128, 128, 3]
    assert q[2].tolist() == [0, 255, 2, 2, 128, 0]          # (64.75-1)/0.5 = 127.5 -> 128
    assert q[3].tolist() == [0] * 6
    assert dq[0].tolist() == [0.0, 255.0, 127.0, 128.0, 128.0, 3.0]
    assert dq[1].tolist() == [10.0, 265.0, 137.0, 138.0, 138.0, 13.0]
    assert dq[2].tolist() == [1.0, 128.5, 2.0, 2.0, 65.0, 1.0]
    assert dq[3].tolist() == [3.0] * 6


def test_attend_values_known_answer():
    """matmul(attention_probs, v) (core/single/pikv_attention.py:188) with grouped heads:
    4 query heads over 2 kv heads (heads 0,1 read kv head 0; heads 2,3 read kv head 1),
    3 cached tokens, head_dim 2.  V[n] = [kv0: (n+1, 10(n+1)) | kv1: (-(n+1), 100(n+1))]."""
    v = np.array([[1, 10, -1, 100],
                  [2, 20, -2, 200],
                  [3, 30, -3, 300]], np.float32)
    p = np.array([[1.0, 0.0, 0.0],          # picks token 0 of kv head 0
                  [0.5, 0.25, 0.25],        # 0.5*1 + 0.25*2 + 0.25*3 = 1.75
                  [0.0, 0.0, 1.0],          # token 2 of kv head 1
                  [0.25, 0.5, 0.25]], np.float32)   # -(0.25 + 1 + 0.75) = -2
    out = O.attend_values(p, v, 2)
    assert out.tolist() == [[1.0, 10.0], [1.75, 17.5], [-3.0, 300.0], [-2.0, 200.0]]
    # one kv head per query head (no grouping): head h reads columns [2h, 2h+2)
    out = O.attend_values(p[:2], v, 2)
    assert out.tolist() == [[1.0, 10.0], [-1.75, 175.0]]


def test_pyramid_keep_counts_interior_values():
    """keep_l = int(N * (1 - 0.75 * l / 31)) = floor(32768 * (124 - 3 l) / 31) for N = 131072,
    evaluated in integers: l = 1 -> 3964928 // 31, l = 16 -> 2490368 // 31, l = 30 -> 1114112 // 31."""
    kc = O.pyramid_keep_counts(131072, 32)
    assert (kc[1], kc[16], kc[30]) == (127900, 80334, 35939)
    assert kc == [(32768 * (124 - 3 * l)) // 31 for l in range(32)]
    assert O.pyramid_keep_counts(100, 1) == [100]
    assert O.pyramid_keep_counts(1000, 5, 0.5) == [1000, 875, 750, 625, 500]


def test_dense_dispatch_combine_known_answer():
    """core/single/module/pikv_routing.py:77-104 on two tokens, 3 experts, capacity 1:
    token 0 -> experts (2, 0) in slots (0, 0); token 1 -> expert 2 is full (slot -1, dropped),
    expert 1 slot 0."""
    idx = np.array([[2, 0], [2, 1]], np.int32)
    w = np.array([[0.75, 0.25], [0.5, 0.125]], np.float32)
    slot, count = O.capacity_slots(idx, 3, 1)
    assert slot.tolist() == [[0, 0], [-1, 0]] and count.tolist() == [1, 1, 2]
    disp, comb = O.dense_dispatch_combine(idx, w, slot, 3, 1)
    assert disp[:, :, 0].tolist() == [[1.0, 0.0, 1.0], [0.0, 1.0, 0.0]]
    assert comb[:, :, 0].tolist() == [[0.25, 0.0, 0.75], [0.0, 0.125, 0.0]]
