"""GPU tests of the host-side mirror of the reference's Python interface: same
constructors, argument meaning, return arity / shapes / dtypes and error
behaviour, with results checked against the oracle."""
import numpy as np
import pytest

import pikv_oracle as O
from util import np_of, rng, to_dev

pytestmark = pytest.mark.gpu


def _mlp_hidden(seq, x2d):
    import torch
    h = x2d
    with torch.no_grad():
        for layer in list(seq)[:-1]:
            h = layer(h)
    return h


def test_base_and_balanced_router_dense_outputs(dev):
    """Config-0 shape: batch 2 x seq 64, hidden 256, 4 experts top-2, cf 1.5."""
    import torch
    from pikv_amd.routing import BaseRouter, TopKBalancedRouter
    torch.manual_seed(0)
    for cls in (BaseRouter, TopKBalancedRouter):
        r = cls(256, 4, top_k=2, capacity_factor=1.5).to(dev)
        for lin in (r.router[0], r.router[2]):
            torch.nn.init.normal_(lin.weight, std=0.02)
        x = torch.randn(2, 64, 256, device=dev)
        disp, comb, probs, aux = r(x)
        cap = O.compute_capacity(2, 64, 1.5, 2, 4)
        assert cap == 96
        assert disp.shape == (2, 64, 4, cap) and comb.shape == disp.shape and probs.shape == (2, 64, 4)
        h = _mlp_hidden(r.router, x.reshape(128, 256)).cpu().numpy()
        w = r.router[2].weight.detach().cpu().numpy()
        b = r.router[2].bias.detach().cpu().numpy()
        p_ref, idx, wts, _ = O.router_tail(O.gate_logits(h, w, b), 2)
        slot, count = O.capacity_slots(idx, 4, cap)
        d_ref, c_ref = O.dense_dispatch_combine(idx, wts, slot, 4, cap)
        assert np.allclose(np_of(probs).reshape(128, 4), p_ref, atol=1e-5)
        assert np.array_equal(np_of(disp).reshape(128, 4, cap), d_ref)
        assert np.allclose(np_of(comb).reshape(128, 4, cap), c_ref, atol=1e-5)
        pm = p_ref.reshape(128, 4).mean(0)
        base = float(np.sum(pm * np.log(pm * 4 + 1e-9)))
        if cls is TopKBalancedRouter:
            ent = -np.sum(pm * np.log(pm + 1e-9)) / np.log(4)
            base += -0.01 * ent
        assert abs(float(aux) - base) < 1e-4
        # compact form
        out, probs2, _ = r(x, return_compact=True)
        assert np.array_equal(np_of(out.topk_idx), idx) and np.array_equal(np_of(out.slot), slot)
        # expert mask: masked experts get no tokens
        mask = torch.tensor([1.0, 0.0, 1.0, 1.0], device=dev)
        out, _, _ = r(x, expert_mask=mask, return_compact=True)
        assert (np_of(out.topk_idx) != 1).all()


def test_eplb_and_pikv_router(dev):
    import torch
    from pikv_amd.routing import EPLBRouter, PiKVRouter
    torch.manual_seed(1)
    r = EPLBRouter(128, 8, top_k=2, temperature=0.7).to(dev).eval()
    x = torch.randn(2, 32, 128, device=dev)
    r.expert_weights = torch.linspace(0.5, 1.5, 8, device=dev)
    ew = r.expert_weights.clone()
    disp, comb, probs, aux = r(x)
    h = _mlp_hidden(r.router, x.reshape(64, 128)).cpu().numpy()
    lg = O.gate_logits(h, r.router[-1].weight.detach().cpu().numpy(), r.router[-1].bias.detach().cpu().numpy())
    p_ref, idx, wts, _ = O.router_tail(lg, 2, temperature=0.7, expert_scale=ew.cpu().numpy())
    assert np.allclose(np_of(probs).reshape(64, 8), p_ref, atol=1e-5)
    cap = O.compute_capacity(2, 32, 1.5, 2, 8)
    slot, count = O.capacity_slots(idx, 8, cap)
    d_ref, _ = O.dense_dispatch_combine(idx, wts, slot, 8, cap)
    assert np.array_equal(np_of(disp).reshape(64, 8, cap), d_ref)
    # expert_weights updated from usage: mean / (usage + 1e-8)
    usage = count.astype(np.float32)
    assert np.allclose(np_of(r.expert_weights), usage.mean() / (usage + 1e-8), rtol=1e-5)
    assert r.global_step == 1 and float(aux) == float(aux)

    p = PiKVRouter(128, 4, top_k=2).to(dev).eval()
    with torch.no_grad():
        p.cache_correction_factor.copy_(torch.tensor([1.0, 0.5, 2.0, 1.0]))
    x = torch.randn(2, 16, 128, device=dev)
    disp, comb, probs, aux, imp = p(x, kv_states=torch.randn(2, 16, 128, device=dev))
    assert imp.shape == (2, 16, 1) and disp.shape[:3] == (2, 16, 4)
    x2 = x.reshape(32, 128)
    with torch.no_grad():
        la = p.router_important(x2).cpu().numpy()
        lb = p.router_unimportant(x2).cpu().numpy()
    sel = (np_of(imp).reshape(-1) > 0.5)
    p_ref, idx, _, _ = O.router_tail(la, 2, logits_b=lb, select=sel,
                                     expert_scale=np.array([1.0, 0.5, 2.0, 1.0], np.float32))
    assert np.allclose(np_of(probs).reshape(32, 4), p_ref, atol=1e-5)
    assert int(p.update_counter) == 1


def test_router_legacy_dense_layouts(dev):
    """legacy_fairscale: the round-wise fill of core/single/pikv_routing.py:102-128 (every token of
    a round that picked expert e shares position used[e]; used[e] += 1 per round), against a literal
    loop; expert_backend='basic': [B,S,E,1] tensors (:133-153)."""
    import torch
    from pikv_amd.routing import BaseRouter
    torch.manual_seed(5)
    B, S, H, E, k = 2, 16, 64, 4, 2
    r = BaseRouter(H, E, top_k=k, capacity_factor=1.5).to(dev)
    x = torch.randn(B, S, H, device=dev)
    out, _, _ = r(x, return_compact=True)
    idx, w = np_of(out.topk_idx), np_of(out.topk_w)
    r.legacy_fairscale = True
    disp, comb, _, _ = r(x)
    cap = O.compute_capacity(B, S, 1.5, k, E)
    want_d = np.zeros((B * S, E, cap), np.float32)
    want_c = np.zeros_like(want_d)
    used = np.zeros(E, np.int64)
    for j in range(k):
        snapshot = used.copy()
        for t in range(B * S):
            e = idx[t, j]
            if snapshot[e] < cap:
                want_d[t, e, snapshot[e]] = 1.0
                want_c[t, e, snapshot[e]] = w[t, j]
        for e in set(idx[:, j][snapshot[idx[:, j]] < cap]):
            used[e] += 1
    assert np.array_equal(np_of(disp).reshape(B * S, E, cap), want_d)
    assert np.array_equal(np_of(comb).reshape(B * S, E, cap), want_c)
    assert want_d[:, :, 2:].sum() == 0          # two rounds: only positions 0 and 1 are ever used
    basic = BaseRouter(H, E, top_k=k, expert_backend="basic").to(dev)
    basic.load_state_dict(r.state_dict())
    d1, c1, _, _ = basic(x)
    assert d1.shape == (B, S, E, 1)
    assert np.array_equal(np_of(d1).reshape(B * S, E).sum(1), np.full(B * S, k, np.float32))
    assert np.allclose(np_of(c1).reshape(B * S, E).sum(1), 1.0, atol=1e-5)


def test_hierarchical_router(dev):
    """core/single/pikv_routing.py:737-860: probabilities as the reference forms them (torch
    float64 evaluation of the same graph), top-k of the products with ties to the lower index,
    renormalised weights, token-major capacity slots, dense tensors of the reference's shape."""
    import torch
    from pikv_amd.routing import HierarchicalRouter
    torch.manual_seed(3)
    B, S, H, E, k = 2, 48, 128, 16, 2
    r = HierarchicalRouter(H, E, top_k=k, capacity_factor=1.5, num_groups=4).to(dev)
    x = torch.randn(B, S, H, device=dev)
    mask = torch.ones(E, device=dev)
    mask[5] = 0
    disp, comb, probs, aux = r(x, expert_mask=mask)
    cap = O.compute_capacity(B, S, 1.5, k, E)
    assert disp.shape == (B, S, E, cap) and comb.shape == disp.shape and probs.shape == (B, S, E)
    r64 = HierarchicalRouter(H, E, top_k=k, num_groups=4).double()
    r64.load_state_dict({n: v.double().cpu() for n, v in r.state_dict().items()})
    want = r64.router_probs(x.double().cpu(), mask.double().cpu()).detach().numpy()
    assert np.allclose(np_of(probs), want, atol=1e-6)
    assert (np_of(probs)[..., 5] == 0).all()
    out, _, _ = r(x, expert_mask=mask, return_compact=True)
    p = np_of(out.probs)
    idx = O.topk_desc(p, k)
    assert np.array_equal(np_of(out.topk_idx), idx)
    vals = np.take_along_axis(p, idx.astype(np.int64), 1)
    assert np.allclose(np_of(out.topk_w), vals / vals.sum(1, keepdims=True), rtol=1e-6)
    slot, count = O.capacity_slots(idx, E, cap)
    assert np.array_equal(np_of(out.slot), slot) and np.array_equal(np_of(out.count), count)
    # the dense tensors carry exactly the kept assignments
    assert int(disp.sum().item()) == int((slot >= 0).sum())
    assert np.isclose(float(comb.sum().item()), float(np_of(out.topk_w)[slot >= 0].sum()), rtol=1e-5)
    p_mean = want.mean(axis=(0, 1))
    assert np.isclose(float(aux.detach()), float((p_mean * np.log(p_mean * E + 1e-9)).sum()), atol=1e-5)


def test_quantized_compressor_static_mode(dev):
    """dynamic_quantization=False (core/single/pikv_compression.py:430-472): the first column
    block of the first keys calibrates one (scale, zero_point); values, later blocks and later
    calls reuse it."""
    import torch
    from pikv_amd import ops
    from pikv_amd.compression import QuantizedCompressor
    r = rng(4)
    c = QuantizedCompressor(256, bits=8, group_size=128, dynamic_quantization=False).to(dev)
    k = torch.from_numpy(r.standard_normal((3, 20, 256)).astype(np.float32)).to(dev)
    v = torch.from_numpy((3 * r.standard_normal((3, 20, 256))).astype(np.float32)).to(dev)
    dk, dv = c(k, v)
    kn, vn = np_of(k).reshape(-1, 256), np_of(v).reshape(-1, 256)
    _, st, _ = O.fakequant_colblocks(kn[:, :128], 128)
    assert float(c.scale) == st[0, 2] and float(c.zero_point) == st[0, 3] and c.calibrated
    ref_k, _ = O.fakequant_preset(kn, st[0, 2], st[0, 3], 128)
    ref_v, mse_v = O.fakequant_preset(vn, st[0, 2], st[0, 3], 128)
    assert np.array_equal(np_of(dk).reshape(-1, 256), ref_k)
    assert np.array_equal(np_of(dv).reshape(-1, 256), ref_v)
    assert (np.abs(np_of(dv)) <= np.abs(ref_v).max()).all()      # the wider values are clamped
    st_ = c.get_compression_stats()
    assert abs(st_["quantization_error"] - mse_v[-1]) < 1e-6 * max(1.0, mse_v[-1]) and st_["num_samples"] == 4
    # a second call keeps the parameters
    k2 = 5 * k
    dk2, _ = c(k2, v)
    ref_k2, _ = O.fakequant_preset(5 * kn, st[0, 2], st[0, 3], 128)
    assert np.array_equal(np_of(dk2).reshape(-1, 256), ref_k2) and float(c.scale) == st[0, 2]
    q, dq, scale = c._quantize(k[0])
    assert np.array_equal(np_of(dq), O.fakequant_preset(np_of(k[0]), st[0, 2], st[0, 3], 256)[0])
    assert float(q.min()) >= 0 and float(q.max()) <= 255 and float(scale) == st[0, 2]
    # the raw op: ragged last block, 4-bit symmetric, errors
    x = r.standard_normal((77, 200)).astype(np.float32)
    preset = torch.tensor([0.0, 0.0, 0.37, 0.0], device=dev)
    dq, mse = ops.fakequant_preset(to_dev(x, dev), preset, 128, 4, True)
    ref, mse_ref = O.fakequant_preset(x, 0.37, 0.0, 128, 4, True)
    assert np.array_equal(np_of(dq), ref) and np.allclose(np_of(mse), mse_ref, rtol=1e-5)
    with pytest.raises(ValueError):
        ops.fakequant_preset(to_dev(x, dev), preset[:3], 128)


def test_quantized_compressor(dev):
    import torch
    from pikv_amd.compression import QuantizedCompressor
    r = rng(3)
    c = QuantizedCompressor(256, bits=8, group_size=128).to(dev)
    k = torch.from_numpy(r.standard_normal((4, 32, 256)).astype(np.float32)).to(dev)
    v = torch.from_numpy(r.standard_normal((4, 32, 256)).astype(np.float32)).to(dev)
    dk, dv = c(k, v)
    assert dk.shape == k.shape and dk.dtype == k.dtype
    ref_k, _, mse_k = O.fakequant_colblocks(np_of(k).reshape(-1, 256), 128)
    ref_v, _, mse_v = O.fakequant_colblocks(np_of(v).reshape(-1, 256), 128)
    assert np.array_equal(np_of(dk).reshape(-1, 256), ref_k)
    assert np.array_equal(np_of(dv).reshape(-1, 256), ref_v)
    st = c.get_compression_stats()
    assert set(st) == {"compression_ratio", "memory_reduction", "bits", "quantization_error",
                       "group_size", "num_samples"}
    assert st["compression_ratio"] == 0.25 and abs(st["quantization_error"] - mse_v[-1]) < 1e-8
    assert st["num_samples"] == 4            # two column blocks for keys, two for values
    q, dq, scale = c._quantize(k[0])
    ref, stats, _ = O.fakequant_colblocks(np_of(k[0]).reshape(1, -1), k[0].numel())
    assert np.array_equal(np_of(dq).reshape(1, -1), ref) and float(scale) == stats[0, 2]
    assert float(q.min()) >= 0 and float(q.max()) <= 255
    # integer-code interface
    codes, s, z = c.quantize(k, granularity="token_head", head_dim=64)
    q_ref, s_ref, z_ref = O.quantize_groups(np_of(k).reshape(-1, 256), 64, O.Q_I8_ASYM)
    assert np.array_equal(np_of(codes).astype(np.int16), q_ref) and np.array_equal(np_of(s), s_ref)
    back = c.dequantize(codes, s, z, granularity="token_head", head_dim=64)
    assert np.array_equal(np_of(back), O.dequantize_groups(q_ref, s_ref, z_ref, 64))
    with pytest.raises(ValueError):
        QuantizedCompressor(256, bits=3)


def test_schedulers_select(dev):
    import torch
    from pikv_amd.scheduling import H2OScheduler, LRUScheduler
    r = rng(4)
    h = H2OScheduler(64, 32, heavy_ratio=0.25, recent_ratio=0.1).to(dev)
    idx = torch.arange(50, device=dev)
    w = torch.from_numpy((np.round(r.random(50) * 4) / 4).astype(np.float32)).to(dev)
    h.update_attention_scores(idx, w)
    h.update_attention_scores(idx[:10], w[:10])
    keys = torch.zeros(50, 32, device=dev)
    mask = h.select_eviction_candidates(keys, keys, {})
    nh, nr = O.h2o_budget(50, 0.25, 0.1)
    keep = O.h2o_keep(np_of(h.attention_accumulator)[:50], np_of(h.access_timestamps)[:50], nh, nr)
    assert mask.dtype == torch.bool and np.array_equal(np_of(mask), ~keep)
    l = LRUScheduler(40, 32).to(dev)
    for t in range(5):
        l.update_access_time(torch.from_numpy(r.permutation(40)[:20]).to(dev))   # indices inside the 40-entry table
    m = l.select_eviction_candidates(keys, keys, {})
    # 50 rows shown to a 40-row scheduler: rows beyond its table count as never accessed
    times = np.concatenate([np_of(l.access_times), np.zeros(10, np.float32)])
    assert np.array_equal(np_of(m), ~O.lru_keep(times, 10))
    assert not np_of(l.select_eviction_candidates(keys[:40], keys[:40], {})).any()


@pytest.mark.parametrize("policy_name", ["LRU", "H2O"])
def test_cache_scheduling_manager(dev, policy_name):
    """Cache of 128 rows x 256, int8 symmetric per token (the config-0 cache)."""
    import torch
    from pikv_amd.scheduling import CacheSchedulingManager, SchedulingPolicy
    r = rng(6)
    policy = SchedulingPolicy[policy_name]
    m = CacheSchedulingManager(128, 256, policy, heavy_ratio=0.25, recent_ratio=0.125)
    ref = O.CachePool([128], 256, 256, O.Q_I8_SYM)
    t = 0
    evicted = 0
    for step in range(5):
        k = r.standard_normal((2, 24, 256)).astype(np.float32)
        v = r.standard_normal((2, 24, 256)).astype(np.float32)
        m.update_cache(torch.from_numpy(k).to(dev), torch.from_numpy(v).to(dev))
        n, cur = 48, int(ref.fill[0])
        if cur + n > 128:
            rows = ref.valid_rows(0)
            if policy_name == "H2O":
                nh, nr = O.h2o_budget(cur, 0.25, 0.125)
                keep = O.h2o_keep(ref.acc[rows], ref.ts[rows], nh, nr)
            else:
                keep = O.lru_keep(ref.ts[rows], cur + n - 128)
            planes = [ref.k_codes, ref.k_scale, ref.k_zero, ref.v_codes, ref.v_scale, ref.v_zero, ref.acc, ref.ts]
            new = O.compact(keep, *[p[:cur] for p in planes])
            evicted += cur - new
            ref.fill[0] = new
        t += 1
        ref.quant_scatter(k.reshape(-1, 256), v.reshape(-1, 256), np.zeros(n, np.int32),
                          np.arange(n, dtype=np.int32), 1, now=float(t))
        ref.advance([n])
        st = m.get_cache_stats()
        assert st["cache_size"] == int(ref.fill[0]) and st["policy"] == policy.value
        assert st["eviction_count"] == evicted
        rows = ref.valid_rows(0)
        want = O.dequantize_groups(ref.k_codes[rows], ref.k_scale[rows], ref.k_zero[rows], 256)
        assert np.array_equal(np_of(m.cache_keys)[:len(rows)], want)
    assert set(st) == {"cache_size", "cache_utilization", "policy", "hit_rate", "eviction_count"}
    m.reset_cache()
    assert m.get_cache_stats()["cache_size"] == 0
    m.change_policy(SchedulingPolicy.NONE)
    m.update_cache(torch.zeros(1, 1, 256, device=dev), torch.zeros(1, 1, 256, device=dev))
    assert m.get_cache_stats()["cache_size"] == 0     # no policy: update is a no-op, as in the reference
    with pytest.raises(ValueError):
        CacheSchedulingManager(8, 256, "bogus")


def test_kernels_facade(dev):
    import torch
    from pikv_amd.kernels import CompressionMode, EvictionPolicy, PiKVKernels
    r = rng(8)
    K = PiKVKernels()
    lg = r.standard_normal((32, 64)).astype(np.float32)
    idx, val = K.top_k_routing(torch.from_numpy(lg).to(dev), 8)
    _, i_ref, v_ref, _ = O.router_tail(lg, 8, use_softmax=False)
    assert np.array_equal(np_of(idx), i_ref) and np.array_equal(np_of(val), v_ref)
    keys = r.standard_normal((32, 512)).astype(np.float32)
    vals = r.standard_normal((32, 512)).astype(np.float32)
    ck, cv, meta = K.compress_kv(torch.from_numpy(keys).to(dev), torch.from_numpy(vals).to(dev),
                                 CompressionMode.QUANT8)
    assert meta["compression_type"] == "quant8"
    for got, codes, sc, mn, src in ((ck, "k_codes", "k_scale", "k_min", keys), (cv, "v_codes", "v_scale", "v_min", vals)):
        q_ref, dq_ref, s_ref, mn_ref = O.quant8_minshift(src)      # the facade's own algebra, :215-232
        assert meta[sc].shape == (32, 1) and meta[mn].shape == (32, 1)
        assert np.array_equal(np_of(meta[codes]), q_ref)
        assert np.array_equal(np_of(meta[sc]), s_ref) and np.array_equal(np_of(meta[mn]), mn_ref)
        assert np.array_equal(np_of(got), dq_ref)
    # eviction: sliding window, stable compaction
    n = 2048
    keys = r.standard_normal((n, 512)).astype(np.float32)
    vals = r.standard_normal((n, 512)).astype(np.float32)
    ts = r.integers(0, 1000, n).astype(np.float32)
    use = r.integers(1, 10, n).astype(np.float32)
    out = K.evict_cache(*[torch.from_numpy(a).to(dev) for a in (keys, vals, ts, use)], 1000,
                        EvictionPolicy.SLIDING, window_threshold=600)
    valid = (1000 - ts) <= 600
    assert out[4] == valid.sum()
    assert np.array_equal(np_of(out[0]), keys[valid]) and np.array_equal(np_of(out[1]), vals[valid])
    assert np.array_equal(np_of(out[2]), ts[valid]) and np.array_equal(np_of(out[3]), use[valid])
    score = np.linalg.norm(keys.astype(np.float64), axis=1) * use
    srt = np.sort(score)
    gap = np.argmax(np.diff(srt[900:1100])) + 900          # threshold inside the widest nearby gap
    thr = float((srt[gap] + srt[gap + 1]) / 2)
    out = K.evict_cache(*[torch.from_numpy(a).to(dev) for a in (keys, vals, ts, use)], 1000,
                        EvictionPolicy.QUEST, quest_threshold=thr)
    valid = score >= thr
    assert out[4] == valid.sum() and np.array_equal(np_of(out[0]), keys[valid])
    # inputs are left alone by default; inplace=True moves the survivors inside the caller's tensors
    tens = [torch.from_numpy(a).to(dev) for a in (keys, vals, ts, use)]
    out = K.evict_cache(*tens, 1000, EvictionPolicy.SLIDING, window_threshold=600)
    assert np.array_equal(np_of(tens[0]), keys) and np.array_equal(np_of(tens[2]), ts)
    out = K.evict_cache(*tens, 1000, EvictionPolicy.SLIDING, window_threshold=600, inplace=True)
    valid = (1000 - ts) <= 600
    m = int(valid.sum())
    assert out[4] == m and out[0].data_ptr() == tens[0].data_ptr()
    assert np.array_equal(np_of(tens[0][:m]), keys[valid]) and np.array_equal(np_of(tens[1][:m]), vals[valid])
    assert np.array_equal(np_of(tens[2][:m]), ts[valid]) and np.array_equal(np_of(tens[3][:m]), use[valid])
    # LORA and MASK (core/single/pikv_kernels.py:185-204, 248-275): hand-checkable cases
    kk = torch.tensor([[1.0, -2.0, 0.0625, 4.0], [0.0, 0.0, 0.0, 3.0]], device=dev)
    a = torch.tensor([[1.0], [0.0], [0.0], [1.0]], device=dev)            # rank 1: K A = k0 + k3
    b = torch.tensor([[0.0, 1.0, 0.0, 2.0]], device=dev)
    ck, cv, meta = K.compress_kv(kk, kk * 2, CompressionMode.LORA,
                                 dict(lora_a_k=a, lora_b_k=b, lora_a_v=a, lora_b_v=b.t().contiguous()))
    assert meta == {"compression_type": "lora", "lora_rank": 1, "lora_ratio": 0.25}
    assert ck.tolist() == [[1.0, -2.0 + 5 * 0.25, 0.0625, 4.0 + 10 * 0.25], [0.0, 3 * 0.25, 0.0, 3.0 + 6 * 0.25]]
    assert torch.equal(cv, 2 * ck)                                         # B given as [hidden, rank] for the values
    ck, cv, meta = K.compress_kv(kk, kk, CompressionMode.LORA)             # default: zero B, the identity
    assert torch.equal(ck, kk) and meta["lora_rank"] == 1
    ck, cv, meta = K.compress_kv(kk, -kk, CompressionMode.MASK)
    # row 0: mean |k| = 1.765625, threshold 0.1765625 -> 0.0625 goes; row 1: mean 0.75 -> the zeros stay zero
    assert ck.tolist() == [[1.0, -2.0, 0.0, 4.0], [0.0, 0.0, 0.0, 3.0]] and torch.equal(cv, -ck)
    assert meta["compression_type"] == "mask" and abs(meta["k_sparsity"] - 0.5) < 1e-6
    with pytest.raises(ValueError):
        K.compress_kv(torch.zeros(4, 64), torch.zeros(4, 64), CompressionMode.MASK)


@pytest.mark.parametrize("trim", [True, False])
def test_cache_pool_checkpoint_round_trip(dev, trim, tmp_path):
    """state_dict -> torch.save -> torch.load(weights_only=True) -> load_state_dict restores
    codes, metadata, accumulators and fill exactly, and reads give identical scores."""
    import torch
    from pikv_amd import ops
    from test_gpu_read_evict import _fill_pool
    r = rng(12)
    caps, lens = [70, 40, 16], [65, 0, 16]
    pool, ref = _fill_pool(dev, r, caps, lens, 2, 64, 32, O.Q_I4_ASYM)
    pool.acc.copy_(torch.rand(pool.rows, device=dev))
    q = torch.randn(3, 4, 64, device=dev)
    s0, _, _ = pool.scores(q, 4)
    path = tmp_path / "pool.pt"
    torch.save(pool.state_dict(trim=trim), path)
    sd = torch.load(path, weights_only=True)
    fresh = ops.CachePool(caps, 2, 64, 32, ops.Q_I4_ASYM, dev)
    fresh.load_state_dict(sd)
    assert torch.equal(fresh.fill, pool.fill)
    for c in range(3):
        rows = ref.valid_rows(c)
        for name in ("k_codes", "k_scale", "k_zero", "v_codes", "v_scale", "v_zero", "acc", "ts"):
            assert torch.equal(getattr(fresh, name)[rows], getattr(pool, name)[rows]), name
    s1, _, _ = fresh.scores(q, 4)
    assert torch.equal(s0[0, :, :65], s1[0, :, :65]) and torch.equal(s0[2, :, :16], s1[2, :, :16])
    other = ops.CachePool(caps, 2, 64, 64, ops.Q_I4_ASYM, dev)
    with pytest.raises(ValueError):
        other.load_state_dict(sd)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("n,D", [(1, 16), (37, 512), (5, 100), (3, 7), (64, 4096), (9, 8200)])
def test_quant8_minshift_matches_facade_algebra(dev, dtype, n, D):
    """pikv_quant8_minshift against core/single/pikv_kernels.py:215-232: codes, scale, row
    minimum and dequantised floats bit for bit, for row widths on and off the 16-element
    vector path, rows with rounding ties, a constant row (scale 0 -> codes 0, dq = min),
    a two-valued row and a row with a huge outlier."""
    from pikv_amd import ops
    r = rng(n * 31 + D)
    x = r.standard_normal((n, D)).astype(np.float32)
    x[0] = np.round(x[0] * 4) / 4                       # many exact .5 ties after the shift
    if n > 2:
        x[1] = 3.0                                      # constant row
        x[2] = np.where(np.arange(D) % 2 == 0, -1.5, 2.0)
    if n > 4:
        x[4, D // 2] = 1e30
    if dtype == "bf16":
        x = O.bf16_round(x)
    dq, codes, s, mn = ops.quant8_minshift(to_dev(x, dev, dtype))
    q_ref, dq_ref, s_ref, mn_ref = O.quant8_minshift(x)
    assert np.array_equal(np_of(codes), q_ref)
    assert np.array_equal(np_of(s), s_ref) and np.array_equal(np_of(mn), mn_ref)
    assert np.array_equal(np_of(dq), dq_ref)
    _, codes2, _, _ = ops.quant8_minshift(to_dev(x, dev, dtype), want_dq=False)
    assert np.array_equal(np_of(codes2), q_ref)


def test_router_outputs_carry_gradients(dev):
    """The gate MLPs must be trainable as in the reference (ordinary nn.Module outputs,
    core/single/pikv_routing.py:44-161): values come from the native kernel, gradients from
    the same formula in torch.  Checked against a pure-torch evaluation of the formula on the
    experts the kernel selected."""
    import torch
    import torch.nn.functional as F
    from pikv_amd.routing import EPLBRouter, HierarchicalRouter, PiKVRouter, TopKBalancedRouter
    torch.manual_seed(2)
    B, S, H, E, k = 2, 24, 64, 8, 2
    x = torch.randn(B, S, H, device=dev, requires_grad=True)
    router = TopKBalancedRouter(H, E, top_k=k).to(dev)
    r, probs, aux = router(x, return_compact=True)
    assert probs.requires_grad and r.topk_w.requires_grad and aux.requires_grad
    loss = (r.topk_w * torch.arange(1, k + 1, device=dev)).sum() + 3.0 * aux + (probs ** 2).sum()
    loss.backward()
    got = {n: p.grad.clone() for n, p in router.named_parameters()}
    got_x = x.grad.clone()
    # the same loss in torch only, on the kernel's indices
    router.zero_grad()
    x2 = x.detach().clone().requires_grad_(True)
    lg = router.router(x2.reshape(B * S, H))
    p_t = F.softmax(lg, dim=-1)
    w_t = p_t.gather(-1, r.topk_idx.long())
    w_t = w_t / w_t.sum(-1, keepdim=True)
    pm = p_t.view(B, S, E).mean(dim=[0, 1])
    aux_t = torch.sum(pm * torch.log(pm * E + 1e-9))
    p3 = p_t.view(B, S, E)
    aux_t = aux_t + router._balance(p3)
    loss_t = (w_t * torch.arange(1, k + 1, device=dev)).sum() + 3.0 * aux_t + (p_t ** 2).sum()
    loss_t.backward()
    for n, p in router.named_parameters():
        assert p.grad is not None and torch.allclose(got[n], p.grad, rtol=1e-4, atol=1e-6), n
    assert torch.allclose(got_x, x2.grad, rtol=1e-4, atol=1e-6)
    # values are still the kernel's: identical to a no-grad call
    with torch.no_grad():
        r0, probs0, aux0 = router(x.detach(), return_compact=True)
    assert torch.equal(r0.topk_idx, r.topk_idx) and torch.equal(r0.slot, r.slot)
    assert torch.allclose(probs0, probs.detach(), rtol=0, atol=1e-7)
    assert not probs0.requires_grad
    # every router class: the auxiliary loss reaches the gate parameters
    for make in (lambda: EPLBRouter(H, E, top_k=k), lambda: PiKVRouter(H, E, top_k=k),
                 lambda: HierarchicalRouter(H, E, top_k=k, num_groups=2)):
        rt = make().to(dev).eval()
        res = rt(x.detach(), return_compact=True)
        rr, aux = res[0], res[2]
        (aux + rr.topk_w.sum() * 0.5 + (rr.topk_w ** 2).sum()).backward()
        grads = [p.grad for p in rt.parameters() if p.grad is not None]
        assert grads and any(float(g.abs().sum()) > 0 for g in grads), type(rt).__name__


def test_moe_load_balance_loss_backpropagates(dev):
    import torch
    from pikv_amd.moe import PiKVMoE
    torch.manual_seed(0)
    model = PiKVMoE().to(dev)
    from pikv_amd.config import config
    x = torch.randn(2, 16, config['hidden_size'], device=dev)
    logits, lb = model(x, return_loss=True)
    (logits.float().pow(2).mean() + lb).backward()
    # (expert_capacity takes no part in the forward, here as in core/single/routing_strategy.py:22)
    g = [p.grad for n, p in model.router.named_parameters() if not n.endswith('expert_capacity')]
    assert all(t is not None for t in g) and any(float(t.abs().sum()) > 0 for t in g)


def test_eplb_router_training_with_dropout_uses_one_mask(dev):
    """EPLBRouter's gate has dropout layers (core/single/pikv_routing.py:596-610).  In training the
    values of the native tail and the gradients of the torch tail must belong to ONE draw of the
    dropout masks: the returned logits (kernel values) equal the torch tail applied to the very
    activation that carries the gradient, which a second pass through the gate would not give."""
    import torch
    from pikv_amd.routing import EPLBRouter
    torch.manual_seed(11)
    r = EPLBRouter(64, 8, top_k=2).to(dev).train()
    x = torch.randn(2, 40, 64, device=dev, requires_grad=True)
    seen = {}
    hook = r.router[-1].register_forward_hook(lambda m, inp, out: seen.setdefault("calls", []).append(out))
    out, probs, aux = r(x, return_compact=True)
    hook.remove()
    assert len(seen["calls"]) == 1                       # the gate's last layer ran once, on the one activation
    lg_t = seen["calls"][0].float() / r.temperature      # expert_weights are ones on the first call
    assert torch.allclose(probs.reshape(-1, 8), torch.softmax(lg_t, -1), atol=2e-6)
    (probs.square().sum() + out.topk_w.sum()).backward()
    assert x.grad is not None and float(x.grad.abs().sum()) > 0
    dropped = [m for m in r.router if isinstance(m, torch.nn.Dropout)]
    assert dropped and all(m.p > 0 for m in dropped)
