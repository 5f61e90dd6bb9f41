"""GPU parity: layer-wise pyramid compression (top-keep_l rows by score, original
order, then quantise) through the C ABI against the numpy restatement.  Kept sets,
codes, scales and fill counts are bit-exact."""
import numpy as np
import pytest

import pikv_oracle as O
from util import codes_np, kv_like, np_of, rng, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("scheme,group,dtype", [(O.Q_I8_SYM, 64, "bf16"), (O.Q_I4_ASYM, 32, "bf16"),
                                                (O.Q_I8_ASYM, 128, "f32")])
@pytest.mark.parametrize("ties", [False, True])
def test_pyramid_compress(dev, scheme, group, dtype, ties):
    from pikv_amd import pyramid
    r = rng(90 + scheme + ties)
    L, n, heads, dh = 5, 3001, 2, 64
    D = heads * dh
    keep = pyramid.linear_keep_budget(n, L)
    assert keep == O.pyramid_keep_counts(n, L)
    ks = kv_like(r, L * n, D, dtype=dtype).reshape(L, n, D)
    vs = kv_like(r, L * n, D, dtype=dtype).reshape(L, n, D)
    sc = r.random((L, n)).astype(np.float32)
    if ties:
        sc = np.round(sc * 16) / 16
    pc = pyramid.PyramidCache(keep, heads, dh, group=group, scheme=scheme, device=dev)
    index, kept = pc.compress(to_dev(ks, dev, dtype), to_dev(vs, dev, dtype), to_dev(sc, dev), now=3.0)
    pool = pc.pool
    assert np.array_equal(np_of(kept), np.array(keep, dtype=np.int32))
    assert np.array_equal(np_of(pool.fill), np.array(keep, dtype=np.int32))
    base = np_of(pool.row_base)
    for l in range(L):
        want = np.nonzero(O.h2o_keep(sc[l], sc[l], keep[l], 0))[0]
        assert want.size == keep[l]
        got = np_of(index)[l * n:l * n + keep[l]]
        assert np.array_equal(got, want), l
        rows = slice(int(base[l]), int(base[l]) + keep[l])
        for src, codes, scale, zero in ((ks, pool.k_codes, pool.k_scale, pool.k_zero),
                                        (vs, pool.v_codes, pool.v_scale, pool.v_zero)):
            q, s, z = O.quantize_groups(src[l][want], group, scheme)
            assert np.array_equal(codes_np(codes, scheme)[rows], q)
            assert np.array_equal(np_of(scale)[rows].astype(np.float32), s)
            if zero is not None:
                assert np.array_equal(np_of(zero)[rows].astype(np.float32), z)
        assert np.array_equal(np_of(pool.acc)[rows], sc[l][want])
        assert np.all(np_of(pool.ts)[rows] == 3.0)


def test_pyramid_small_brute_force(dev):
    """Kept set against an O(n^2) ranking: row i survives iff fewer than keep rows
    precede it in (score desc, index asc) order."""
    from pikv_amd import ops
    r = rng(3)
    n, L = 37, 6
    sc = (np.round(r.random((L, n)) * 8) / 8).astype(np.float32)
    keep = np.array([37, 20, 9, 1, 0, 36], dtype=np.int32)
    seg_base = np.arange(L, dtype=np.int64) * n
    flag, index, kept = ops.select_top_rows(to_dev(sc.reshape(-1), dev), to_dev(seg_base, dev),
                                            to_dev(np.full(L, n, dtype=np.int32), dev), to_dev(keep, dev))
    f = np_of(flag).reshape(L, n)
    assert np.array_equal(np_of(kept), keep)
    for l in range(L):
        for i in range(n):
            before = sum((sc[l, j] > sc[l, i]) or (sc[l, j] == sc[l, i] and j < i) for j in range(n))
            assert bool(f[l, i]) == (before < keep[l]), (l, i)
