"""GPU parity of the StreamingLLM / QUEST / FlexGen / LRU+ schedulers and of the
manager running them: scores against the numpy restatement (float tolerance), the
eviction set exactly (native selection, ties to the lower index) for the scores the
GPU produced, and the manager's cache contents exactly after evict + compact +
append over several updates."""
import numpy as np
import pytest

import pikv_oracle as O
from util import np_of, rng

pytestmark = pytest.mark.gpu


def test_streaming_llm_scheduler(dev):
    import torch
    from pikv_amd.scheduling import StreamingLLMScheduler
    s = StreamingLLMScheduler(48, 32, start_size=4, recent_size=20).to(dev)
    keys = torch.zeros(60, 32, device=dev)
    assert not np_of(s.select_eviction_candidates(keys[:48], keys[:48], {})).any()
    ev = np_of(s.select_eviction_candidates(keys, keys, {}))
    assert np.array_equal(ev, ~O.streaming_keep(60, 4, 20))
    d = StreamingLLMScheduler(16, 32).to(dev)       # default window = cache_size - start
    ev = np_of(d.select_eviction_candidates(keys[:30], keys[:30], {}))
    assert np.array_equal(ev, ~O.streaming_keep(30, 4, 12))


def test_quest_flexgen_lruplus_schedulers(dev):
    import torch
    from pikv_amd.scheduling import FlexGenScheduler, LRUPlusScheduler, QUESTScheduler
    r = rng(21)
    C, L = 40, 52
    keys = torch.zeros(L, 16, device=dev)
    # QUEST
    q = QUESTScheduler(C, 16, quality_threshold=0.1, decay_factor=0.9).to(dev)
    for step in range(6):
        idx = torch.from_numpy(r.permutation(C)[:15]).to(dev)
        q.update_quality_scores(idx, torch.from_numpy(r.random(15).astype(np.float32) * 3).to(dev))
    u = np_of(q.compute_utility_scores(L))
    u_ref = O.quest_utility(np.pad(np_of(q.quality_scores), (0, L - C)), np.pad(np_of(q.usage_frequency), (0, L - C)),
                            np.pad(np_of(q.last_access_time), (0, L - C)), int(q.global_time), 0.9)
    assert np.allclose(u, u_ref, rtol=1e-5, atol=1e-7)
    ev = np_of(q.select_eviction_candidates(keys, keys, {}))
    assert np.array_equal(ev, O.quest_evict(u, 0.1, L - C))
    q.quality_threshold = -1.0                       # nothing below the threshold: the lowest L-C go
    ev = np_of(q.select_eviction_candidates(keys, keys, {}))
    assert ev.sum() == L - C and np.array_equal(ev, O.evict_lowest(u, L - C))
    assert not np_of(q.select_eviction_candidates(keys[:C], keys[:C], {})).any()
    # FlexGen
    f = FlexGenScheduler(C, 16).to(dev)
    assert (f.gpu_cache_size, f.cpu_cache_size, f.disk_cache_size) == (12, 20, 8)
    for step in range(5):
        idx = torch.from_numpy(r.permutation(C)[:20]).to(dev)
        f.update_access_patterns(idx, torch.from_numpy(1 + r.integers(0, 3, 20).astype(np.float32)).to(dev))
    b = np_of(f.compute_benefit_scores(L))
    assert np.array_equal(b, O.flexgen_benefit(np.pad(np_of(f.access_frequency), (0, L - C)),
                                               np.pad(np_of(f.access_cost), (0, L - C), constant_values=1)))
    ev = np_of(f.select_eviction_candidates(keys, keys, {}))
    assert np.array_equal(ev, O.evict_lowest(b, L - C))   # many exact ties: lower index goes first
    # LRU+
    p = LRUPlusScheduler(C, 16, frequency_weight=0.3, importance_weight=0.4).to(dev)
    for step in range(7):
        idx = torch.from_numpy(r.permutation(C)[:12]).to(dev)
        p.update_access_info(idx, torch.from_numpy(r.random(12).astype(np.float32)).to(dev))
    pr = np_of(p.compute_priority_scores(L))
    pr_ref = O.lruplus_priority(np.pad(np_of(p.access_times), (0, L - C)), np.pad(np_of(p.access_frequency), (0, L - C)),
                                np.pad(np_of(p.importance_scores), (0, L - C)))
    assert np.allclose(pr, pr_ref, rtol=1e-5, atol=1e-7)
    ev = np_of(p.select_eviction_candidates(keys, keys, {}))
    assert np.array_equal(ev, O.evict_lowest(pr, L - C))


@pytest.mark.parametrize("policy_name", ["STREAMING_LLM", "QUEST", "FLEXGEN", "LRU_PLUS"])
def test_manager_other_policies(dev, policy_name):
    import torch
    from pikv_amd.scheduling import CacheSchedulingManager, SchedulingPolicy
    r = rng(33)
    C, H, n = 64, 128, 20
    m = CacheSchedulingManager(C, H, SchedulingPolicy[policy_name])
    ref = O.CachePool([C], H, H, O.Q_I8_SYM)
    planes = [ref.k_codes, ref.k_scale, ref.k_zero, ref.v_codes, ref.v_scale, ref.v_zero, ref.acc, ref.ts]
    for step in range(1, 7):
        k = r.standard_normal((1, n, H)).astype(np.float32)
        v = r.standard_normal((1, n, H)).astype(np.float32)
        cur = int(ref.fill[0])
        sch = m.scheduler
        # feed the scheduler some access statistics about the rows it currently holds
        if cur and policy_name != "STREAMING_LLM":
            sch.to(dev)
            idx = torch.from_numpy(r.permutation(cur)[:max(1, cur // 2)]).to(dev)
            val = torch.from_numpy((1 + r.integers(0, 4, idx.numel())).astype(np.float32)).to(dev)
            if policy_name == "QUEST":
                sch.update_quality_scores(idx, val)
            elif policy_name == "FLEXGEN":
                sch.update_access_patterns(idx, val)
            else:
                sch.update_access_info(idx, val / 8)
        n_ev = max(0, min(cur, cur + n - C))
        if cur + n > C:
            if policy_name == "STREAMING_LLM":
                keep = O.streaming_keep(cur, 4, cur - n_ev - 4)
            elif policy_name == "QUEST":
                keep = ~O.quest_evict(np_of(sch.compute_utility_scores(cur)), sch.quality_threshold, n_ev)
            elif policy_name == "FLEXGEN":
                keep = ~O.evict_lowest(np_of(sch.compute_benefit_scores(cur)), n_ev)
            else:
                keep = ~O.evict_lowest(np_of(sch.compute_priority_scores(cur)), n_ev)
            side = [np_of(b).copy() for b in (sch.row_buffers() if hasattr(sch, "row_buffers") else [])]
            ref.fill[0] = O.compact(keep, *[p[:cur] for p in planes])
        m.update_cache(torch.from_numpy(k).to(dev), torch.from_numpy(v).to(dev))
        if cur + n > C and hasattr(sch, "row_buffers"):   # per-slot statistics moved with their rows
            kept = np.nonzero(keep)[0]
            for b, old in zip(sch.row_buffers(), side):
                assert np.array_equal(np_of(b)[:kept.size], old[kept])
        ref.quant_scatter(k.reshape(-1, H), v.reshape(-1, H), np.zeros(n, np.int32), np.arange(n, dtype=np.int32),
                          1, now=float(step))
        ref.advance([n])
        rows = ref.valid_rows(0)
        assert m.get_cache_stats()["cache_size"] == len(rows)
        assert np.array_equal(np_of(m.pool.k_codes)[rows], ref.k_codes[rows]), step
        assert np.array_equal(np_of(m.pool.v_codes)[rows], ref.v_codes[rows]), step
        assert np.array_equal(np_of(m.pool.ts)[rows], ref.ts[rows])
    assert m.get_cache_stats()["policy"] == SchedulingPolicy[policy_name].value
    assert m.get_cache_stats()["eviction_count"] > 0


def test_adakv_and_duoattention_schedulers(dev):
    import torch
    from pikv_amd.scheduling import AdaKVScheduler, CacheSchedulingManager, DuoAttentionScheduler, SchedulingPolicy
    r = rng(44)
    C, L = 40, 60
    a = AdaKVScheduler(C, 16, compression_ratio=0.5, safeguard_ratio=0.2).to(dev)
    keys = torch.from_numpy(np.round(r.standard_normal((C, 16)) * 2).astype(np.float32) / 2).to(dev)
    a.update_importance(torch.arange(C, device=dev), keys)
    sc = np.pad(np_of(a.importance_scores), (0, L - C))
    big = torch.zeros(L, 16, device=dev)
    ev = np_of(a.select_eviction_candidates(big, big, {}))
    assert np.array_equal(ev, ~O.adakv_keep(sc, 0.5, 0.2))
    assert (~ev).sum() == int(L * 0.5)
    assert not np_of(a.select_eviction_candidates(big[:C], big[:C], {})).any()
    d = DuoAttentionScheduler(32, 16, sink_size=4, recent_size=10).to(dev)
    ev = np_of(d.select_eviction_candidates(big, big, {}))
    assert np.array_equal(ev, ~O.duo_keep(L, 4, 10))
    for name in ("ADAKV", "DUOATTENTION"):
        m = CacheSchedulingManager(32, 64, SchedulingPolicy[name])
        for step in range(4):
            m.update_cache(torch.randn(1, 12, 64, device=dev), torch.randn(1, 12, 64, device=dev))
            assert 0 < m.get_cache_stats()["cache_size"] <= 32
        assert m.get_cache_stats()["eviction_count"] > 0
