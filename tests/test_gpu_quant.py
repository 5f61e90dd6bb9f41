"""GPU parity: K2 quantise (+ scatter) and the dequantising gather, through the
C ABI, against the numpy restatement.  Integer codes, scales and zero points
must be bit-exact; dequantised float32 values are produced by the same two
float32 operations on both sides and must be bit-exact too; bf16 outputs must
equal the round-to-nearest-even of the float32 value."""
import numpy as np
import pytest

import pikv_oracle as O
from util import codes_np, kv_like, np_of, rng, to_dev

pytestmark = pytest.mark.gpu

SCHEMES = [O.Q_I8_SYM, O.Q_I8_ASYM, O.Q_I4_ASYM, O.Q_I4_SYM]


def _edge_rows(D):
    """Rows that exercise the formula's corners: all zero, constant, a single
    spike, exact .5 ties, tiny and huge magnitudes, negative-only."""
    rows = [np.zeros(D), np.full(D, 3.25), np.full(D, -7.5)]
    spike = np.zeros(D); spike[5] = 100.0
    rows.append(spike)
    ramp = np.linspace(-1.0, 1.0, D)
    rows.append(ramp)
    rows.append(np.arange(D) % 16 * 0.5)            # many rounding ties
    rows.append(np.full(D, 1e-30)); rows[-1][0] = -1e-30
    rows.append(np.linspace(1e4, 3e4, D))
    rows.append(-np.abs(np.linspace(0.1, 5.0, D)))
    # spread tiny next to the offset: the 4-bit zero point would not fit half precision
    rows += [np.full(D, 1.0), np.full(D, 1000.0), 1.0 + 1e-4 * np.linspace(0, 1, D), -200.0 - 1e-3 * np.arange(D) / D,
             np.full(D, 0.04)]
    return np.stack(rows).astype(np.float32)


@pytest.mark.parametrize("scheme", SCHEMES)
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("D,group", [(256, 256), (512, 128), (1024, 32), (128, 64)])
def test_quantize_rows_bit_exact(dev, scheme, dtype, D, group):
    from pikv_amd import ops
    bits = O.scheme_info(scheme)[0]
    if bits == 8 and group < 16 or bits == 4 and group < 32:
        pytest.skip("group below one lane")
    r = rng(100 + scheme)
    x = np.concatenate([kv_like(r, 300, D, dtype=dtype), _edge_rows(D)])
    if dtype == "bf16":
        x = O.bf16_round(x)
    codes, scale, zero = ops.quantize_rows(to_dev(x, dev, dtype), group, scheme)
    q_ref, s_ref, z_ref = O.quantize_groups(x, group, scheme)
    assert np.array_equal(np_of(scale).astype(np.float32), s_ref), "scale"
    if zero is not None:
        assert np.array_equal(np_of(zero).astype(np.float32), z_ref), "zero"
    got = codes_np(codes, scheme)
    assert np.array_equal(got, q_ref), f"codes differ at {np.argwhere(got != q_ref)[:5]}"

    # read side: same (q - z) * s in float32 -> bit-exact; bf16 = RNE of that
    dq = ops.dequantize_rows(codes, scale, zero, group, scheme)
    dq_ref = O.dequantize_groups(q_ref, s_ref, z_ref, group)
    # (rows whose float32 range collapses to a zero scale give NaN on both sides,
    # as the reference's formula does)
    assert np.array_equal(np_of(dq), dq_ref, equal_nan=True)
    import torch
    dqb = ops.dequantize_rows(codes, scale, zero, group, scheme, out_dtype=torch.bfloat16)
    assert np.array_equal(np_of(dqb), O.bf16_round(dq_ref), equal_nan=True)


def test_known_answers(dev):
    """Hand-derived vectors: asym8 [-1,0,1] -> zp 127, q [0,127,254];
    sym8 [0.3,-0.7,0.05,0.7] -> [55,-128,9,127]; asym4 [0,1,2,3] -> [0,5,10,15]."""
    from pikv_amd import ops
    def run(vals, scheme, group):
        x = np.zeros((1, group), dtype=np.float32)
        reps = group // len(vals)
        x[0] = np.tile(np.array(vals, dtype=np.float32), reps)
        c, s, z = ops.quantize_rows(to_dev(x, dev), group, scheme)
        return codes_np(c, scheme)[0, :len(vals)], np_of(s)[0, 0], None if z is None else np_of(z)[0, 0]
    q, s, z = run([-1, 0, 1, 0], O.Q_I8_ASYM, 16)
    assert list(q) == [0, 127, 254, 127] and z == 127 and s == np.float32(2.0) / np.float32(255)
    q, s, _ = run([-1, 0, 1, 0], O.Q_I8_SYM, 16)
    assert list(q) == [-127, 0, 127, 0]
    q, s, _ = run([0.3, -0.7, 0.05, 0.7], O.Q_I8_SYM, 16)
    assert list(q) == [55, -128, 9, 127]
    q, s, z = run([0, 1, 2, 3], O.Q_I4_ASYM, 32)
    assert list(q) == [0, 5, 10, 15] and z == 0 and s == np.float32(np.float16(0.2))


def _route(r, T, E, k, capacity):
    idx = np.stack([r.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    slot, count = O.capacity_slots(idx, E, capacity)
    return idx, slot, count


@pytest.mark.parametrize("scheme,group", [(O.Q_I8_SYM, 64), (O.Q_I8_SYM, 256), (O.Q_I4_ASYM, 32),
                                          (O.Q_I8_ASYM, 64), (O.Q_I4_SYM, 64)])
@pytest.mark.parametrize("shared", [True, False])
def test_quant_scatter_matches_cache_model(dev, scheme, group, shared):
    """Config-0-like shape (4 experts, top-2, 4 heads x 64) plus skew so that the
    router capacity AND the cache capacity both drop rows; two successive
    batches so the second appends at a non-zero fill."""
    import torch
    from pikv_amd import ops
    E, k, heads, dh = 4, 2, 4, 64
    D = heads * dh
    caps = [40, 128, 7, 64]
    pool = ops.CachePool(caps, heads, dh, group, scheme, dev)
    ref = O.CachePool(caps, D, group, scheme)
    r = rng(7)
    for step, T in enumerate([96, 50]):
        capacity = O.compute_capacity(1, T, 1.5, k, E)
        idx, slot, count = _route(r, T, E, k, capacity)
        n_src = T if shared else T * k
        fan = k if shared else 1
        ks, vs = kv_like(r, n_src, D, dtype="f32"), kv_like(r, n_src, D, dtype="f32")
        pool.quant_scatter(to_dev(ks, dev), to_dev(vs, dev), to_dev(idx, dev), to_dev(slot, dev),
                           fan, now=float(step + 1))
        pool.advance(to_dev(count, dev), capacity)
        ref.quant_scatter(ks, vs, idx, slot, fan, now=float(step + 1))
        ref.advance(count, capacity)
        assert np.array_equal(np_of(pool.fill), ref.fill)
        for c in range(E):
            rows = ref.valid_rows(c)
            assert np.array_equal(codes_np(pool.k_codes, scheme)[rows], ref.k_codes[rows])
            assert np.array_equal(codes_np(pool.v_codes, scheme)[rows], ref.v_codes[rows])
            assert np.array_equal(np_of(pool.k_scale)[rows].astype(np.float32), ref.k_scale[rows])
            assert np.array_equal(np_of(pool.v_scale)[rows].astype(np.float32), ref.v_scale[rows])
            if pool.k_zero is not None:
                assert np.array_equal(np_of(pool.k_zero)[rows].astype(np.float32), ref.k_zero[rows])
            assert np.array_equal(np_of(pool.ts)[rows], ref.ts[rows])
            assert np.array_equal(np_of(pool.acc)[rows], ref.acc[rows])
    # rows never written stay zero (no stray stores outside the valid region)
    untouched = np.ones(pool.rows, dtype=bool)
    for c in range(E):
        untouched[ref.valid_rows(c)] = False
    assert not np_of(pool.k_codes)[untouched].any()
    torch.cuda.synchronize()


def test_empty_and_error_paths(dev):
    import torch
    from pikv_amd import ops
    from pikv_amd._native import PiKVNativeError
    pool = ops.CachePool([8, 8], 2, 64, 64, O.Q_I8_SYM, dev)
    empty = torch.zeros(0, 128, device=dev)
    e32 = torch.zeros(0, dtype=torch.int32, device=dev)
    pool.quant_scatter(empty, empty, e32, e32, 2)          # no rows: a no-op
    assert int(pool.fill.sum()) == 0
    with pytest.raises(ValueError):
        ops.quantize_rows(torch.zeros(4, 96, device=dev), 96, O.Q_I8_SYM)   # not a power of two
    with pytest.raises(ValueError):
        ops.quantize_rows(torch.zeros(4, 128), 128, O.Q_I8_SYM)             # CPU tensor
    with pytest.raises(ValueError):
        ops.quantize_rows(torch.zeros(4, 128, device=dev).double(), 128, O.Q_I8_SYM)
    with pytest.raises(ValueError):
        pool.quant_scatter(torch.zeros(3, 128, device=dev), torch.zeros(3, 128, device=dev),
                           torch.zeros(5, dtype=torch.int32, device=dev),
                           torch.zeros(5, dtype=torch.int32, device=dev), 2)
    # the C ABI itself reports bad arguments with a status, not a crash
    from pikv_amd import _native as N
    assert N.lib().pikv_quantize_rows(None, 0, 1, 128, 128, 0, 0, None, None, None, None) == -1
    with pytest.raises(PiKVNativeError):
        N.call("pikv_quantize_rows", 1, 0, 1, 100, 100, 0, 0, 1, 1, None, None)


def test_fakequant_reference_domain(dev):
    """QuantizedCompressor.forward's domain: min/max over all rows of each
    128-column block (ragged last block)."""
    from pikv_amd import ops
    r = rng(11)
    for (n, H, g, bits, sym) in [(128, 256, 128, 8, False), (777, 200, 128, 4, False),
                                 (64, 256, 128, 8, True)]:
        x = r.standard_normal((n, H)).astype(np.float32)
        dq, stats, mse = ops.fakequant_colblocks(to_dev(x, dev), g, bits, sym)
        dq_ref, st_ref, mse_ref = O.fakequant_colblocks(x, g, bits, sym)
        assert np.array_equal(np_of(stats), st_ref)
        assert np.array_equal(np_of(dq), dq_ref)
        assert np.allclose(np_of(mse), mse_ref, rtol=1e-5)


@pytest.mark.parametrize("scheme,group", [(O.Q_I8_SYM, 128), (O.Q_I8_ASYM, 128), (O.Q_I4_ASYM, 32), (O.Q_I4_SYM, 32)])
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_quantize_many_values_bit_exact(dev, scheme, group, dtype):
    """8.4 M values per case: the kernel replaces the per-element division by a
    per-group reciprocal with an exactness check, so the codes are compared on
    enough data that thousands of elements fall next to a rounding tie, plus rows
    that leave the fast path's range (large offsets, huge and tiny magnitudes)."""
    from pikv_amd import ops
    r = rng(900 + scheme)
    n, D = 2048, 4096
    x = kv_like(r, n, D, dtype="f32")
    x[100:140] += 1000.0                       # large zero points -> exact path
    x[200:220] *= 1e-20
    x[300:320] *= 1e20
    x[400:420] = np.round(x[400:420] * 4) / 4  # coarse grid: exact ties in many groups
    if dtype == "bf16":
        x = O.bf16_round(x)
    codes, scale, zero = ops.quantize_rows(to_dev(x, dev, dtype), group, scheme)
    q_ref, s_ref, z_ref = O.quantize_groups(x, group, scheme)
    assert np.array_equal(np_of(scale).astype(np.float32), s_ref)
    if zero is not None:
        assert np.array_equal(np_of(zero).astype(np.float32), z_ref, equal_nan=True)
    got = codes_np(codes, scheme)
    bad = np.argwhere(got != q_ref)
    assert bad.size == 0, f"{len(bad)} codes differ, first {bad[:5]}"
