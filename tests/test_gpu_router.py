"""GPU parity: K1 router (gate projection, softmax, top-k, renormalise, capacity
slots) through the C ABI against the numpy restatement.

Expert indices: on every row the stable top-k (value descending, lower expert first
among equal float32 values) of the probabilities the kernel returned - the tensor the
reference hands to torch.topk - and equal to the restatement's selection except where
the two sides' exp() round a near-tie differently (util.assert_topk_of_probs); slots
bit-exact for the indices chosen; masks, scaling and the two-gate select included.  For the fused gate projection the float32 summation order differs
from any CPU order, so indices are compared exactly wherever the float64 gap
between the k-th and (k+1)-th logit exceeds 1e-4 (relative to the logit range)
and the capacity slots are checked for exact consistency with the indices the
GPU produced.  Probabilities and weights: |diff| <= 1e-5 (float32) /
1e-3 relative of the logit scale for bf16 inputs."""
import numpy as np
import pytest

import pikv_oracle as O
from util import assert_topk_of_probs, np_of, rng, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("E,k", [(4, 2), (8, 2), (6, 3), (16, 4), (64, 8), (33, 1), (1, 1), (48, 5), (40, 8), (64, 2), (64, 5), (33, 6)])
def test_router_tail_bit_exact(dev, E, k):
    from pikv_amd import ops
    r = rng(E * 10 + k)
    T = 1000
    lg = r.standard_normal((T, E)).astype(np.float32)
    # force ties: duplicate columns and quantise some rows coarsely
    lg[::3] = np.round(lg[::3] * 2) / 2
    if E > 2:
        lg[::5, 1] = lg[::5, 0]
    lg_b = r.standard_normal((T, E)).astype(np.float32)
    sel = (r.random(T) > 0.5)
    scale = (0.5 + r.random(E)).astype(np.float32)
    mask = (r.random(E) > 0.3).astype(np.float32)
    if mask.sum() < k:
        mask[:] = 1
    cap = O.compute_capacity(1, T, 1.25, k, E)
    for kw in [dict(), dict(temperature=0.7, expert_scale=scale),
               dict(expert_mask=mask), dict(logits_b=lg_b, select=sel, expert_scale=scale),
               dict(renorm_eps=1e-8)]:
        okw = dict(kw)
        dkw = {key: (to_dev(v, dev) if isinstance(v, np.ndarray) and v.dtype != bool else v)
               for key, v in kw.items()}
        if "select" in dkw:
            dkw["select"] = to_dev(sel.astype(np.uint8), dev)
        out = ops.router_tail(to_dev(lg, dev), top_k=k, capacity=cap, **dkw)
        probs, idx, w, _ = O.router_tail(lg, k, **okw)
        got = np_of(out.topk_idx)
        assert_topk_of_probs(got, np_of(out.probs), k, idx, probs)
        same = (got == idx).all(axis=1)
        assert np.allclose(np_of(out.probs), probs, atol=2e-6, rtol=1e-5)
        assert np.allclose(np_of(out.topk_w)[same], w[same], atol=2e-6, rtol=1e-5)
        slot, count = O.capacity_slots(got, E, cap)
        assert np.array_equal(np_of(out.slot), slot)
        assert np.array_equal(np_of(out.count), count)
    # raw top-k of logits (the facade's top_k_routing): values are the logits
    out = ops.router_tail(to_dev(lg, dev), top_k=k, use_softmax=False)
    _, idx, vals, _ = O.router_tail(lg, k, use_softmax=False)
    assert np.array_equal(np_of(out.topk_idx), idx)
    assert np.array_equal(np_of(out.topk_w), vals)


def _collapse_logits(E):
    """Distinct logits whose float32 probabilities coincide: 2^-10 and its two predecessors
    differ by 2^-34 - exp() of that difference is 1 to 2^-35, far inside one rounding - with
    the LOWER logits at the LOWER expert indices (and, from 40 experts on, in the other half
    of the row), everything else far below."""
    hi = np.float32(2.0 ** -10)
    lo = np.nextafter(hi, np.float32(0), dtype=np.float32)
    lo2 = np.nextafter(lo, np.float32(0), dtype=np.float32)
    row = np.linspace(-3.0, -6.0, E).astype(np.float32)
    a, b, c = (3, 17, 40) if E > 40 else (0, 1, 2)
    row[a], row[b], row[c] = lo2, lo, hi
    return row, (a, b, c)


@pytest.mark.parametrize("E,k", [(4, 1), (4, 2), (8, 2), (16, 3), (32, 2), (40, 1), (40, 2), (64, 1), (64, 2), (64, 8)])
def test_topk_ties_on_probabilities_not_logits(dev, E, k):
    """The reference takes torch.topk of the float32 PROBABILITIES (core/single/pikv_routing.py:
    73-76).  Where exp() maps distinct logits to one float32 the experts tie and the lower index
    wins, although its logit is the smaller one - in the restatement and in every form of the
    kernel tail (standalone tail on given logits; the gate kernels fed the same logits through
    the bias, for short, medium and long token streams, bf16 and float32 inputs)."""
    import torch
    from pikv_amd import ops
    row, (a, b, c) = _collapse_logits(E)
    want = [a, b, c][:k] + list(np.argsort(-row, kind="stable")[3:])[:max(0, k - 3)]
    lg = np.tile(row, (300, 1))
    probs, idx, w, _ = O.router_tail(lg, k)
    assert probs[0, a] == probs[0, b] == probs[0, c] and row[a] < row[b] < row[c]
    assert idx[0].tolist() == want
    out = ops.router_tail(to_dev(lg, dev), top_k=k)
    p = np_of(out.probs)
    assert p[0, a] == p[0, b] == p[0, c]
    assert (np_of(out.topk_idx) == np.array(want)).all()
    raw = ops.router_tail(to_dev(lg, dev), top_k=k, use_softmax=False)      # without the softmax the key is the logit
    assert np_of(raw.topk_idx)[0].tolist() == list(np.argsort(-row, kind="stable")[:k])
    H = 256
    for T, dt in [(300, torch.bfloat16), (300, torch.float32), (20480 + 64, torch.bfloat16), (32768 + 128, torch.bfloat16),
                  (65536, torch.bfloat16)]:
        if T == 65536 and E > 16:
            continue
        x = torch.randn(T, H, device=dev).to(dt)
        out = ops.router_fused(x, torch.zeros(E, H, device=dev, dtype=dt), to_dev(row, dev), top_k=k, return_logits=True)
        assert torch.equal(out.logits, to_dev(row, dev).expand(T, E))
        got = np_of(out.topk_idx)
        assert (got == np.array(want)).all(), (T, dt, got[0], want)
        assert_topk_of_probs(got, np_of(out.probs), k)


@pytest.mark.parametrize("E", [40, 64])
def test_router_tail_special_values_both_forms(dev, E):
    """33-64 experts are served by arg-max rounds at k = 1 and by the lanes-per-token sort from
    k = 2 on: on rows with NaN, +-inf, signed zeros and many ties the two must agree on the
    first choice and give bit-identical probabilities, shorter lists must be prefixes of longer
    ones, and NaN is picked last, lowest index first."""
    from pikv_amd import ops
    r = rng(E)
    T = 512
    lg = r.standard_normal((T, E)).astype(np.float32)
    lg[0] = 0.0
    lg[1, ::2] = -0.0
    lg[1, 1::2] = 0.0
    lg[2] = np.nan
    lg[3, : E - 3] = np.nan                      # three numbers, the rest NaN
    lg[4] = -np.inf
    lg[4, 7] = 1.0
    lg[5, ::3] = np.inf
    lg[6, 5] = np.nan
    lg[7] = np.round(lg[7])
    lg[8:64] = np.round(lg[8:64] * 2) / 2
    lg[64:80, 3] = np.nan
    lg[64:80, 9] = -np.inf
    d = to_dev(lg, dev)
    a = np_of(ops.router_tail(d, top_k=1, use_softmax=False).topk_idx)    # arg-max form
    a4 = np_of(ops.router_tail(d, top_k=4, use_softmax=False).topk_idx)
    b = np_of(ops.router_tail(d, top_k=8, use_softmax=False).topk_idx)
    assert np.array_equal(a[:, 0], b[:, 0]) and np.array_equal(a4, b[:, :4])
    assert ((b >= 0) & (b < E)).all()
    assert all(len(set(row)) == 8 for row in b)
    assert list(b[0]) == list(range(8)) and list(b[1]) == list(range(8)) and list(b[2]) == list(range(8))
    assert sorted(b[3][:3]) == [E - 3, E - 2, E - 1] and list(b[3][3:]) == [0, 1, 2, 3, 4]
    assert b[4][0] == 7 and list(b[4][1:]) == [0, 1, 2, 3, 4, 5, 6]
    assert list(b[5]) == [0, 3, 6, 9, 12, 15, 18, 21]
    assert 5 not in b[6]
    # with the softmax: same selection, probabilities of the two forms bit-identical on finite rows
    fin = np.isfinite(lg).all(axis=1)
    oa = ops.router_tail(d, top_k=1)
    ob = ops.router_tail(d, top_k=8)
    assert np.array_equal(np_of(oa.topk_idx)[fin][:, 0], np_of(ob.topk_idx)[fin][:, 0])
    assert np.array_equal(np_of(oa.probs)[fin], np_of(ob.probs)[fin])


@pytest.mark.parametrize("A,E,cap", [(1, 4, 1), (2047, 8, 100), (2049, 8, 3), (100000, 64, 1500),
                                      (65536, 8, 10240), (5000, 3, 0),
                                      # 8192 (chunk, expert) words is where the rank blocks stop summing the
                                      # earlier chunks themselves: both sides of it, and an odd expert count
                                      (65536, 64, 900), (66000, 64, 1100), (40000, 5, 7000), (513, 64, 4)])
def test_capacity_slots_exact(dev, A, E, cap):
    from pikv_amd import ops
    r = rng(A + E)
    # Zipf-like skew so that some experts overflow
    p = 1.0 / np.arange(1, E + 1) ** 1.2
    idx = r.choice(E, size=A, p=p / p.sum()).astype(np.int32)
    slot, count = ops.capacity_slots(to_dev(idx, dev), E, cap)
    s_ref, c_ref = O.capacity_slots(idx, E, cap)
    assert np.array_equal(np_of(slot), s_ref)
    assert np.array_equal(np_of(count), c_ref)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("T,H,E,k", [(128, 256, 4, 2), (1000, 512, 8, 2), (257, 1024, 16, 4),
                                      (130, 7168, 64, 8), (64, 264, 5, 2),
                                      (300, 272, 24, 4),       # float32: matrix cores, 17 k-steps of 16, two expert tiles
                                      (1000, 512, 64, 8),      # ... four expert tiles, weights re-laid
                                      (32768 + 37, 256, 64, 8)])  # ... 128-token blocks, ragged last one
def test_router_fused(dev, dtype, T, H, E, k):
    from pikv_amd import ops
    r = rng(T + H + E)
    x = r.standard_normal((T, H)).astype(np.float32)
    w = (0.02 * r.standard_normal((E, H))).astype(np.float32)
    b = (0.1 * r.standard_normal(E)).astype(np.float32)
    if dtype == "bf16":
        x, w = O.bf16_round(x), O.bf16_round(w)
    cap = O.compute_capacity(1, T, 1.25, k, E)
    out = ops.router_fused(to_dev(x, dev, dtype), to_dev(w, dev, dtype), to_dev(b, dev),
                           top_k=k, capacity=cap, return_logits=True)
    lg64 = x.astype(np.float64) @ w.astype(np.float64).T + b
    lg = lg64.astype(np.float32)
    probs, idx, wts, _ = O.router_tail(lg, k)
    assert np.allclose(np_of(out.logits), lg, atol=1e-5 * np.sqrt(H), rtol=1e-5)
    assert np.allclose(np_of(out.probs), probs, atol=1e-5)
    got = np_of(out.topk_idx)
    # EVERY row: the selection is exactly the top-k (ties to the lower index) of the
    # probabilities the kernel itself returned
    klg = np_of(out.logits)
    p_own, idx_own, w_own, _ = O.router_tail(klg, k)
    assert_topk_of_probs(got, np_of(out.probs), k, idx_own, p_own)
    same = (got == idx_own).all(axis=1)
    assert np.allclose(np_of(out.topk_w)[same], w_own[same], atol=1e-6)
    # and it is the float64 selection wherever the gap between neighbouring logits exceeds twice
    # the largest error the kernel's logits show against float64
    err = float(np.abs(klg.astype(np.float64) - lg64).max())
    srt = -np.sort(-lg64, axis=1)
    gaps = np.abs(np.diff(srt, axis=1))[:, :k].min(axis=1) if E > 1 else np.ones(T)
    clear = gaps > 2.0 * err + 1e-12
    assert err <= 1e-5 * np.sqrt(H)
    assert clear.mean() > 0.98
    assert np.array_equal(got[clear], idx[clear])
    # rows with a near-tie must still select valid, distinct experts
    assert ((got >= 0) & (got < E)).all()
    assert all(len(set(row)) == k for row in got)
    assert np.allclose(np_of(out.topk_w)[clear], wts[clear], atol=1e-5)
    assert np.allclose(np_of(out.topk_w).sum(1), 1.0, atol=1e-5)
    # slots are exactly the token-major rule applied to the indices the GPU chose
    slot, count = O.capacity_slots(got, E, cap)
    assert np.array_equal(np_of(out.slot), slot)
    assert np.array_equal(np_of(out.count), count)


def test_router_float32_without_workspace(dev):
    """float32 inputs, no slots requested, no workspace passed: the call is valid (only bf16 inputs
    need one), more than 16 experts are then read from the weight matrix where it lies - same results
    as with a workspace, where the weights are re-laid first."""
    import torch
    from pikv_amd import _native as N
    from pikv_amd import ops
    r = rng(77)
    T, H, E, k = 700, 320, 40, 3
    x = to_dev(r.standard_normal((T, H)).astype(np.float32), dev)
    w = to_dev((0.05 * r.standard_normal((E, H))).astype(np.float32), dev)
    ref = ops.router_fused(x, w, top_k=k, return_logits=True)
    probs = torch.empty(T, E, device=dev)
    logits = torch.empty(T, E, device=dev)
    idx = torch.empty(T, k, dtype=torch.int32, device=dev)
    wts = torch.empty(T, k, device=dev)
    N.call("pikv_router_fused", x.data_ptr(), w.data_ptr(), N.F32, None, None, None, 1.0, 0.0, 0, T, H, E, k, 0,
           probs.data_ptr(), logits.data_ptr(), idx.data_ptr(), wts.data_ptr(), None, None, None, 0,
           torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(idx, ref.topk_idx)
    assert torch.equal(logits, ref.logits)      # the same products in the same order, whichever way the weights come
    assert torch.equal(wts, ref.topk_w)


@pytest.mark.parametrize("T,H,E,k", [(32768 + 37, 256, 64, 8), (32768, 128, 40, 3), (32768 + 5, 416, 64, 8),
                                      (40000, 1152, 33, 1), (32768 + 70, 512, 8, 2), (32768 + 3, 256, 16, 4),
                                      (33000, 384, 20, 4), (32768, 768, 5, 1), (32768 + 1, 1024, 32, 8),
                                      (32768, 384, 8, 2), (65536 + 3, 256, 8, 2), (65536, 512, 16, 8)])
def test_router_long_stream(dev, T, H, E, k):
    """At least 32768 tokens take the tiled, LDS-staged kernels (H % 128 == 0, or % 256 up to 16
    experts; otherwise the generic ones): ragged last block, one and several stages, padded
    expert columns, every tile split over the wavefronts."""
    import torch
    from pikv_amd import ops
    g = torch.Generator(device=dev).manual_seed(T + H + E)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    w = (0.05 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    b = 0.1 * torch.randn(E, generator=g, device=dev)
    if E >= 40:  # three experts with identical rows: exact ties in every token, lowest index first
        w[5], w[17], w[31] = w[2], w[2], w[2]
        b[5], b[17], b[31] = b[2], b[2], b[2]
    cap = int(T * 1.25 * k / E)
    out = ops.router_fused(x, w, b, top_k=k, capacity=cap, return_logits=True)
    if E >= 40:
        assert torch.equal(out.logits[:, 2], out.logits[:, 17]) and torch.equal(out.logits[:, 2], out.logits[:, 31])
    lg = x.double() @ w.double().T + b.double()
    assert torch.allclose(out.logits.double(), lg, atol=1e-5 * H ** 0.5, rtol=1e-5)
    assert torch.allclose(out.probs, torch.softmax(out.logits, dim=1), atol=1e-6)
    order = torch.sort(out.probs, dim=1, descending=True, stable=True).indices[:, :k]
    assert torch.equal(out.topk_idx.long(), order)
    sel = torch.gather(out.probs, 1, order)
    assert torch.allclose(out.topk_w, sel / sel.sum(1, keepdim=True), atol=1e-6)
    slot, count = O.capacity_slots(np_of(out.topk_idx), E, cap)
    assert np.array_equal(np_of(out.slot), slot)
    assert np.array_equal(np_of(out.count), count)


@pytest.mark.parametrize("T,H,E,k", [(64, 7168, 64, 8), (1, 4096, 8, 2), (700, 2048, 20, 4), (4096 + 9, 1024, 64, 6),
                                      (8192, 512, 8, 1), (16383, 1536, 33, 2), (20479, 512, 64, 8),
                                      (20480 + 5, 512, 64, 8), (24000, 256, 8, 2), (30000, 768, 24, 3)])
def test_router_short_stream_split(dev, T, H, E, k):
    """Short token streams split the gate projection over the hidden dimension (partial logits
    per slice, summed in slice order by the tail): single token, ragged blocks, slices that do
    not divide the k-steps, every padded expert width."""
    import torch
    from pikv_amd import ops
    g = torch.Generator(device=dev).manual_seed(T + H + E)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    w = (0.05 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    b = 0.1 * torch.randn(E, generator=g, device=dev)
    if E >= 20:
        w[5], w[17] = w[2], w[2]
        b[5], b[17] = b[2], b[2]
    cap = max(1, int(T * 1.25 * k / E))
    out = ops.router_fused(x, w, b, top_k=k, capacity=cap, return_logits=True)
    lg = x.double() @ w.double().T + b.double()
    assert torch.allclose(out.logits.double(), lg, atol=1e-5 * H ** 0.5, rtol=1e-5)
    if E >= 20:
        assert torch.equal(out.logits[:, 2], out.logits[:, 17])
    assert torch.allclose(out.probs, torch.softmax(out.logits, dim=1), atol=1e-6)
    order = torch.sort(out.probs, dim=1, descending=True, stable=True).indices[:, :k]
    assert torch.equal(out.topk_idx.long(), order)
    slot, count = O.capacity_slots(np_of(out.topk_idx), E, cap)
    assert np.array_equal(np_of(out.slot), slot)
    assert np.array_equal(np_of(out.count), count)
    # the same call twice gives the same bits (fixed order of the partial sums)
    again = ops.router_fused(x, w, b, top_k=k, capacity=cap, return_logits=True)
    assert torch.equal(out.logits, again.logits) and torch.equal(out.topk_w, again.topk_w)


@pytest.mark.parametrize("module", [False, True])
def test_router_tiled_and_rows_forms_logit_arithmetic(dev, module):
    """Temperature, per-expert scale, mask and bias through the branch-free per-row arithmetic of
    the token-per-lane forms, in both orders of the reference's two router copies: the
    standalone tail (bit-exact against the restatement) and the tiled gate kernel (final logits
    against float64, top-k exact on the kernel's own logits, masked experts never chosen)."""
    import torch
    from pikv_amd import ops
    r = rng(170 + module)
    T, E, k = 3000, 64, 8
    lg = (r.standard_normal((T, E)) * 3).astype(np.float32)
    lg[::4, 2] = lg[::4, 7]
    scale = (0.5 + r.random(E)).astype(np.float32)
    mask = np.ones(E, dtype=np.float32)
    mask[[1, 9, 33]] = 0
    kw = dict(temperature=0.7, expert_scale=scale, expert_mask=mask, renorm_eps=1e-8 if module else 0.0)
    out = ops.router_tail(to_dev(lg, dev), top_k=k, temperature=0.7, expert_scale=to_dev(scale, dev),
                          expert_mask=to_dev(mask, dev), renorm_eps=kw["renorm_eps"], module_arithmetic=module)
    probs, idx, w, final = O.router_tail(lg, k, module_arithmetic=module, **kw)
    assert_topk_of_probs(np_of(out.topk_idx), np_of(out.probs), k, idx, probs)
    same = (np_of(out.topk_idx) == idx).all(axis=1)
    assert np.allclose(np_of(out.probs), probs, atol=2e-6, rtol=1e-5)
    assert np.allclose(np_of(out.topk_w)[same], w[same], atol=2e-6, rtol=1e-5)
    assert not np.isin(np_of(out.topk_idx), [1, 9, 33]).any()
    # tiled gate kernel (more than 20480 tokens)
    T2, H = 20480 + 77, 256
    g = torch.Generator(device=dev).manual_seed(5 + module)
    x = torch.randn(T2, H, generator=g, device=dev).to(torch.bfloat16)
    wg = (0.05 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    b = 0.1 * torch.randn(E, generator=g, device=dev)
    o2 = ops.router_fused(x, wg, b, top_k=k, temperature=0.7, expert_scale=to_dev(scale, dev),
                          expert_mask=to_dev(mask, dev), renorm_eps=kw["renorm_eps"], module_arithmetic=module,
                          return_logits=True)
    raw = (x.double() @ wg.double().T + b.double()).float().cpu().numpy()
    want = O.scale_logits(raw, 0.7, scale, mask, module_arithmetic=module)
    fin = np_of(o2.logits)
    live = mask > 0
    assert np.allclose(fin[:, live], want[:, live], atol=2e-5 * H ** 0.5, rtol=2e-5)
    assert (fin[:, ~live] < (-1e38 if module else -1e8)).all()
    order = torch.sort(o2.probs, dim=1, descending=True, stable=True).indices[:, :k]
    assert torch.equal(o2.topk_idx.long(), order)
    assert not np.isin(np_of(o2.topk_idx), [1, 9, 33]).any()
    p2, idx2, w2, _ = O.router_tail(fin, k, renorm_eps=kw["renorm_eps"])
    assert_topk_of_probs(np_of(o2.topk_idx), np_of(o2.probs), k, idx2, p2)
    same = (np_of(o2.topk_idx) == idx2).all(axis=1)
    assert np.allclose(np_of(o2.topk_w)[same], w2[same], atol=2e-6, rtol=1e-5)


def test_router_module_arithmetic(dev):
    """The arithmetic of the reference's module/ copy (core/single/module/pikv_routing.py:596-600,
    :133-134, :143): scale before temperature, finfo.min penalty, + 1e-8 in the renormalisation -
    bit-exact indices against the restatement, on logits chosen so that the order of the two
    roundings matters for some rows."""
    from pikv_amd import ops
    r = rng(77)
    T, E, k = 3000, 12, 3
    lg = (r.standard_normal((T, E)) * 3).astype(np.float32)
    lg[::4, 2] = lg[::4, 7]
    scale = (0.5 + r.random(E)).astype(np.float32)
    mask = np.ones(E, dtype=np.float32)
    mask[[1, 9]] = 0
    kw = dict(temperature=0.7, expert_scale=scale, expert_mask=mask, renorm_eps=1e-8)
    out = ops.router_tail(to_dev(lg, dev), top_k=k, capacity=900, temperature=0.7, expert_scale=to_dev(scale, dev),
                          expert_mask=to_dev(mask, dev), renorm_eps=1e-8, module_arithmetic=True)
    probs, idx, w, final = O.router_tail(lg, k, module_arithmetic=True, **kw)
    assert_topk_of_probs(np_of(out.topk_idx), np_of(out.probs), k, idx, probs)
    same = (np_of(out.topk_idx) == idx).all(axis=1)
    assert np.allclose(np_of(out.probs), probs, atol=2e-6, rtol=1e-5)
    assert np.allclose(np_of(out.topk_w)[same], w[same], atol=2e-6, rtol=1e-5)
    assert not np.isin(np_of(out.topk_idx), [1, 9]).any()
    # the two orders really differ in the last bit for some logits
    other = O.scale_logits(lg, 0.7, scale, None)
    assert (other != O.scale_logits(lg, 0.7, scale, None, module_arithmetic=True)).any()
    # fused projection: same flag
    x = O.bf16_round(r.standard_normal((500, 256)).astype(np.float32))
    wg = O.bf16_round((0.05 * r.standard_normal((E, 256))).astype(np.float32))
    out = ops.router_fused(to_dev(x, dev, "bf16"), to_dev(wg, dev, "bf16"), top_k=k, temperature=0.7,
                           expert_scale=to_dev(scale, dev), expert_mask=to_dev(mask, dev), renorm_eps=1e-8,
                           module_arithmetic=True, return_logits=True)
    fin = np_of(out.logits)
    assert (fin[:, [1, 9]] < -1e38).all()
    p2, idx2, w2, _ = O.router_tail(fin, k, renorm_eps=1e-8)
    assert_topk_of_probs(np_of(out.topk_idx), np_of(out.probs), k, idx2, p2)
    same = (np_of(out.topk_idx) == idx2).all(axis=1)
    assert np.allclose(np_of(out.topk_w)[same], w2[same], atol=2e-6, rtol=1e-5)


def test_router_empty_and_errors(dev):
    import torch
    from pikv_amd import ops
    out = ops.router_fused(torch.zeros(0, 64, device=dev), torch.zeros(4, 64, device=dev),
                           top_k=2, capacity=4)
    assert out.topk_idx.shape == (0, 2) and int(out.count.sum()) == 0
    with pytest.raises(ValueError):
        ops.router_fused(torch.zeros(4, 63, device=dev), torch.zeros(4, 63, device=dev))
    with pytest.raises(ValueError):
        ops.router_fused(torch.zeros(4, 64, device=dev), torch.zeros(80, 64, device=dev))
    with pytest.raises(ValueError):
        ops.router_fused(torch.zeros(4, 64, device=dev), torch.zeros(4, 64, device=dev), top_k=5)
    with pytest.raises(ValueError):
        ops.router_fused(torch.zeros(4, 64), torch.zeros(4, 64))


@pytest.mark.parametrize("T", [4096, 40000])
def test_router_logits_of_identical_rows_across_the_batch(dev, T):
    """The gate kernels walk a token row's k-steps from an offset that depends on the block, so the
    float32 summation order - and the last bits of a token's logits - depend on where the token
    stands in the batch.  Pinned here: identical rows give logits within 1e-5 * sqrt(H) of the float64
    value at every position (the bound every router test uses), so their spread is at most twice
    that; the selection may differ between positions only on rows whose float64 gap is inside that
    band (none in this draw)."""
    import torch
    from pikv_amd import ops
    g = torch.Generator(device=dev).manual_seed(7)
    H, E, k = 4096, 8, 2
    row = torch.randn(1, H, generator=g, device=dev).to(torch.bfloat16)
    w = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(torch.bfloat16)
    out = ops.router_fused(row.expand(T, H).contiguous(), w, top_k=k, return_logits=True)
    want = (row.double() @ w.double().T)[0]
    err = (out.logits.double() - want).abs().max().item()
    assert err <= 1e-5 * H ** 0.5
    spread = (out.logits.max(0).values - out.logits.min(0).values).max().item()
    assert spread <= 2e-5 * H ** 0.5
    gap = torch.sort(want, descending=True).values
    assert float(gap[k - 1] - gap[k]) > 4e-5 * H ** 0.5
    assert bool((out.topk_idx == out.topk_idx[0]).all())
