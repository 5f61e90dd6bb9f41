"""PiKVMoE and KVCache with the reference's interface (core/single/pikv_moe.py),
their cache traffic routed through the HIP library.

What stays in torch: the embedding, the dense experts (LoRAExpert,
core/single/lora.py:31-52), the query/key projections and the vocabulary
projection - dense GEMMs of the caller, not part of the cache data path.

The router is the reference's routing_strategy.AdaptiveRouter (routing_strategy.py in this
package: same parameter names, a reference state_dict loads), and the expert outputs are
combined with its DENSE routing weights, as core/single/pikv_moe.py:281,312 does; on a model
whose caches are empty the logits are the reference's up to the term its learned pyramid
compressor adds for an all-zero cache (tests/test_gpu_moe_golden.py holds them to the output of
the reference's own module).

What runs natively, once per forward and for all experts together:
  * every softmax + top-k + renormalise of the router, and the capacity slots of its top-k;
  * eviction of the rows that have to make room (LRU by default, H2O on request)
    and in-place compaction of every per-expert cache;
  * quantisation of the routed tokens' K/V rows and their scatter into the
    per-expert caches;
  * with H2O scheduling, the scores of a per-expert query over the compressed
    cache and the importance accumulation that H2O selects on.

Differences from the reference that are deliberate:
  * a cache holds the routed TOKENS' rows (quantised), not one mean vector per
    forward (pikv_moe.py:53-78 averages the whole batch into one row);
  * `KVCache.get_all()` returns the mean of the dequantised cached values (plus
    the value LoRA); the reference first sends the cache through a learned
    pyramid MLP (kv_cache_compression.py), which is not on the data path;
  * `cache_sizes` has one entry per expert (the reference allocates `num_layers`
    caches and uses the first `num_experts`, pikv_moe.py:170-177).
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .config import config
from .routing_strategy import AdaptiveRouter
from .scheduling import SchedulingPolicy

_SCHEMES = {"int8": ops.Q_I8_SYM, "int8_asym": ops.Q_I8_ASYM, "int4": ops.Q_I4_ASYM,
            "int4_sym": ops.Q_I4_SYM}


class LoRALayer(nn.Module):
    """core/single/lora.py:8-29."""

    def __init__(self, in_features, out_features, rank=4, alpha=1.0, dropout=0.0):
        super().__init__()
        self.rank, self.alpha, self.scaling = rank, alpha, alpha / rank
        self.lora_A = nn.Parameter(torch.zeros(in_features, rank))
        self.lora_B = nn.Parameter(torch.zeros(rank, out_features))
        self.dropout = nn.Dropout(p=dropout)
        nn.init.kaiming_uniform_(self.lora_A, a=math.sqrt(5))
        nn.init.zeros_(self.lora_B)

    def forward(self, x):
        return self.dropout(x @ self.lora_A @ self.lora_B) * self.scaling


class LoRAExpert(nn.Module):
    """core/single/lora.py:31-52."""

    def __init__(self, hidden_size, rank=4, alpha=1.0):
        super().__init__()
        self.hidden_size = hidden_size
        self.dense = nn.Linear(hidden_size, hidden_size)
        self.lora = LoRALayer(hidden_size, hidden_size, rank=rank, alpha=alpha)

    def forward(self, x):
        return F.relu(self.dense(x) + self.lora(x))


def _make_pool(sizes, hidden_size, device):
    heads = int(config.get('kv_heads', 1))
    if hidden_size % heads:
        raise ValueError(f"hidden_size {hidden_size} is not divisible by kv_heads {heads}")
    group = config.get('kv_group') or hidden_size
    return ops.CachePool(list(sizes), heads, hidden_size // heads, int(group),
                         _SCHEMES[config.get('kv_quant', 'int8')], device)


class KVCache(nn.Module):
    """One expert's cache: cache `index` of a shared quantised pool
    (core/single/pikv_moe.py:13-137).  Standalone instances own a one-cache pool."""

    def __init__(self, size, use_scheduling=False, scheduling_policy=SchedulingPolicy.NONE):
        super().__init__()
        self.size = size
        self.hidden_size = config['hidden_size']
        self.use_scheduling = use_scheduling
        self.scheduling_policy = scheduling_policy
        self.value_lora = LoRALayer(self.hidden_size, self.hidden_size, rank=4, alpha=1.0)
        self.pool: Optional[ops.CachePool] = None
        self.index = 0
        self._time = 0

    def _bind(self, pool: ops.CachePool, index: int):
        self.pool, self.index = pool, index

    def _own_pool(self, device):
        if self.pool is None:
            self.pool, self.index = _make_pool([self.size], self.hidden_size, device), 0
        return self.pool

    def _policy(self):
        if self.use_scheduling and self.scheduling_policy == SchedulingPolicy.H2O:
            return ops.EVICT_H2O
        return ops.EVICT_LRU  # also the ring of the unscheduled cache: the oldest rows go first

    def update(self, idx, key, value, importance=None):
        """Append the rows of key/value ([n,H] or [B,S,H]); `idx` is the write
        clock (the reference's ring pointer / timestamp)."""
        k2 = key.reshape(-1, self.hidden_size).float().contiguous()
        v2 = value.reshape(-1, self.hidden_size).float().contiguous()
        pool = self._own_pool(k2.device)
        n = k2.shape[0]
        dev = pool.device
        # this cache takes n rows, the other caches of a shared pool none: they keep every row
        n_new = torch.zeros(pool.n_caches, dtype=torch.int32, device=dev)
        n_new[self.index] = min(n, self.size)
        _evict_for(pool, n_new, self._policy())
        self._time = max(self._time + 1, int(idx) + 1)
        pool.quant_scatter(k2, v2, torch.full((n,), self.index, dtype=torch.int32, device=dev),
                           torch.arange(n, dtype=torch.int32, device=dev), 1, now=float(self._time))
        pool.advance(n_new)

    def _mean_value(self):
        pool = self.pool
        base = int(pool.row_base[self.index].item())
        fill = int(pool.fill[self.index].item())
        if fill == 0:
            return torch.zeros(self.hidden_size, device=pool.device)
        return pool.gather_dequant("v", row0=base, n=fill).mean(dim=0)

    def get_all(self):
        if self.pool is None:
            return torch.zeros(self.hidden_size, device=self.value_lora.lora_A.device)
        m = self._mean_value()
        return m + self.value_lora(m)

    def set_all(self, data):
        if data is not None and self.pool is not None:
            self.pool.fill[self.index] = 0

    def get_cache_stats(self):
        fill = 0 if self.pool is None else int(self.pool.fill[self.index].item())
        policy = self.scheduling_policy.value if self.use_scheduling else 'none'
        return {'cache_size': fill, 'cache_utilization': fill / max(self.size, 1), 'policy': policy}

    def change_scheduling_policy(self, new_policy: SchedulingPolicy):
        self.scheduling_policy = new_policy


def _evict_for(pool: ops.CachePool, n_new: torch.Tensor, policy: int, heavy_ratio=0.1,
               recent_ratio=0.1):
    """Make room for n_new[c] rows in every cache (core/single/cache_scheduling.py:
    404-427): caches that would overflow evict first - the fill+n_new-cap least
    recently used rows, or everything outside H2O's heavy and recent sets - and are
    compacted in place; the others keep all their rows.  No host synchronisation."""
    over = (pool.fill + n_new - pool.cap).clamp_min(0)
    if policy == ops.EVICT_LRU:
        pool.evict(ops.EVICT_LRU, n_evict=torch.minimum(over, pool.fill).to(torch.int32))
        return
    f = pool.fill.double()
    nh = (f * heavy_ratio).floor().clamp_min(1).to(torch.int32)
    nr = (f * recent_ratio).floor().clamp_min(1).to(torch.int32)
    keep_all = over == 0
    pool.evict(ops.EVICT_H2O, n_heavy=torch.where(keep_all, pool.fill, nh).contiguous(),
               n_recent=torch.where(keep_all, torch.zeros_like(nr), nr).contiguous())


class PiKVMoE(nn.Module):
    """core/single/pikv_moe.py:139-505 (distillation and the external memory cache
    are outside the data path and not provided)."""

    def __init__(self, rank=4, alpha=1.0, use_distillation=False, teacher_hidden_size=None,
                 use_cache_scheduling=False, cache_scheduling_policy=SchedulingPolicy.NONE):
        super().__init__()
        if use_distillation:
            raise NotImplementedError("knowledge distillation is not part of the cache data path")
        self.use_distillation = False
        self.use_cache_scheduling = use_cache_scheduling
        self.cache_scheduling_policy = cache_scheduling_policy
        H, E = config['hidden_size'], config['num_experts']
        self.embedding = nn.Embedding(config['vocab_size'], H)
        self.experts = nn.ModuleList([LoRAExpert(H, rank=rank, alpha=alpha) for _ in range(E)])
        self.router = AdaptiveRouter(hidden_size=H, num_experts=E, top_k=2, temperature=1.0)
        self.query_proj = nn.Linear(H, H)
        self.key_proj = nn.Linear(H, H)
        self.query_lora = LoRALayer(H, H, rank=rank, alpha=alpha)
        self.key_lora = LoRALayer(H, H, rank=rank, alpha=alpha)
        self.cache_sizes = self.pyramidal_cache_allocation()
        self.kv_caches = nn.ModuleList([
            KVCache(size, use_scheduling=use_cache_scheduling, scheduling_policy=cache_scheduling_policy)
            for size in self.cache_sizes])
        self.register_buffer('cache_ptrs', torch.zeros(E, dtype=torch.long))
        self.vocab_proj = nn.Linear(H, config['vocab_size'])
        self.pool: Optional[ops.CachePool] = None
        self.clock = 0
        self.debug_capture = False   # keep the routed rows of the last forward in self.captured
        self.captured = None

    def pyramidal_cache_allocation(self):
        """C_i = C_1 - (i-1)*d, one cache per expert (core/single/pikv_moe.py:218-224)."""
        C1, d = config['kv_cache_size'], config['cache_decrement']
        return [C1 - (i - 1) * d for i in range(1, config['num_experts'] + 1)]

    def _ensure_pool(self, device):
        if self.pool is None:
            self.pool = _make_pool(self.cache_sizes, config['hidden_size'], device)
            for i, c in enumerate(self.kv_caches):
                c._bind(self.pool, i)
        return self.pool

    def compute_token_importance(self, query, key):
        """core/single/pikv_moe.py:226-247."""
        q = self.query_proj(query) + self.query_lora(query)
        k = self.key_proj(key) + self.key_lora(key)
        scores = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(config['hidden_size'])
        return F.softmax(scores, dim=-1).sum(dim=1)

    def _cached_means(self, pool):
        """Mean dequantised cached value of every expert, [E, H] (zeros when empty).  Plain
        masked sums per cache: the result does not depend on scheduling."""
        v = pool.gather_dequant("v")                                   # [rows, H]
        means = []
        for c, (b, cap) in enumerate(zip(pool.base_host, pool.caps_host)):
            live = (torch.arange(cap, device=pool.device) < pool.fill[c]).unsqueeze(1)
            means.append((v[b:b + cap] * live).sum(dim=0))
        return torch.stack(means) / pool.fill.clamp_min(1).unsqueeze(1).float()

    def update_cache(self, expert_idx, key, value, importance):
        """Update one expert's cache with new key / value rows (core/single/pikv_moe.py:249-261).
        The reference averages key and value over batch and sequence into ONE row and writes it at
        the expert's ring pointer; here every given row ([n,H] or [B,S,H]) is quantised and appended,
        the expert's policy (LRU, or H2O when scheduled so) evicting first when the cache is full.
        `importance` has no part in either policy (the reference stores its mean and, with
        scheduling, never reads it).  forward() updates all experts together instead."""
        if not 0 <= int(expert_idx) < len(self.kv_caches):
            raise IndexError(f"expert_idx {expert_idx} out of range")
        self._ensure_pool(key.device)
        self.clock += 1
        self.kv_caches[int(expert_idx)].update(self.clock - 1, key, value, importance)
        self.cache_ptrs = self.pool.fill.long()

    def forward(self, x, query=None, return_loss=False, targets=None, use_teacher=False):
        if x.dim() == 2:
            x = self.embedding(x)
        elif x.dim() != 3:
            raise ValueError(f"Input must be 2D (token IDs) or 3D (embeddings), got shape: {x.shape}")
        if x.dtype != torch.float32:
            x = x.to(torch.float32)
        B, S, H = x.shape
        T, E = B * S, config['num_experts']
        pool = self._ensure_pool(x.device)

        routing_weights, expert_indices, top_k_weights, lb_loss, importance = self.router(x)
        k = expert_indices.shape[-1]
        if query is not None:
            importance = self.compute_token_importance(query.to(torch.float32), x)

        cached = self._cached_means(pool)                              # [E, H]
        expert_output = torch.zeros(B, S, H, device=x.device)
        outs = []
        for i, expert in enumerate(self.experts):
            c = cached[i] + self.kv_caches[i].value_lora(cached[i])
            out_i = expert(x) + c.view(1, 1, H)
            outs.append(out_i)
            expert_output = expert_output + out_i * routing_weights[:, :, i].unsqueeze(-1)

        # cache update: K = projected token, V = its expert's output, one row per assignment
        with torch.no_grad():
            x2 = x.reshape(T, H)
            keys = (self.key_proj(x2) + self.key_lora(x2)).repeat_interleave(k, dim=0).contiguous()
            stacked = torch.stack([o.reshape(T, H) for o in outs])     # [E, T, H]
            tok = torch.arange(T, device=x.device).repeat_interleave(k)
            # which token rows go to which expert's cache: the router's top-k, at most `capacity` per
            # expert and forward in token order (core/single/pikv_routing.py:40-42,
            # core/single/module/pikv_routing.py:93-104)
            idx32 = expert_indices.reshape(T * k).to(torch.int32).contiguous()
            capacity = int(B * S * config.get('capacity_factor', 1.5) * k / E)
            slot, count = ops.capacity_slots(idx32, E, capacity)
            values = stacked[idx32.long(), tok].contiguous()
            n_new = torch.minimum(torch.minimum(count, torch.full_like(count, capacity)), pool.cap)
            policy = (ops.EVICT_H2O if self.use_cache_scheduling and
                      self.cache_scheduling_policy == SchedulingPolicy.H2O else ops.EVICT_LRU)
            _evict_for(pool, n_new, policy)
            self.clock += 1
            if self.debug_capture:
                self.captured = dict(keys=keys, values=values, idx=idx32.view(T, k), slot=slot.view(T, k),
                                     count=count, capacity=capacity, n_new=n_new, cached=cached,
                                     fill_before=pool.fill.clone(), routing_weights=routing_weights,
                                     top_k_weights=top_k_weights, importance=importance)
            pool.quant_scatter(keys, values, idx32, slot, 1, now=float(self.clock))
            pool.advance(count, capacity)
            self.cache_ptrs = pool.fill.long()
            if policy == ops.EVICT_H2O:
                self._accumulate_h2o(pool, x2 if query is None else query.reshape(-1, H).float())

        logits = self.vocab_proj(expert_output)
        if return_loss:
            return logits, lb_loss
        return logits

    def _accumulate_h2o(self, pool, q_tokens):
        """Scores of one query per expert (the mean projected query of the batch) over
        that expert's compressed cache feed the H2O accumulators."""
        H = config['hidden_size']
        q = (self.query_proj(q_tokens) + self.query_lora(q_tokens)).mean(dim=0)
        q = q.view(1, pool.n_heads, pool.head_dim).expand(pool.n_caches, -1, -1).contiguous()
        scores, tmax, tsum = pool.scores(q, pool.n_heads)
        pool.h2o_accumulate(scores, tmax, tsum, now=float(self.clock))

    # ---- scheduling controls (core/single/pikv_moe.py:338-395) ------------------
    def enable_cache_scheduling(self, policy: SchedulingPolicy = SchedulingPolicy.LRU):
        self.use_cache_scheduling = True
        self.cache_scheduling_policy = policy
        for cache in self.kv_caches:
            cache.use_scheduling = True
            cache.scheduling_policy = policy

    def disable_cache_scheduling(self):
        self.use_cache_scheduling = False
        for cache in self.kv_caches:
            cache.use_scheduling = False
        if self.pool is not None:
            self.pool.fill.zero_()

    def change_cache_scheduling_policy(self, new_policy: SchedulingPolicy):
        if self.use_cache_scheduling:
            self.cache_scheduling_policy = new_policy
            for cache in self.kv_caches:
                cache.change_scheduling_policy(new_policy)

    def get_cache_stats(self):
        return {f'expert_{i}': cache.get_cache_stats() for i, cache in enumerate(self.kv_caches)}

    def print_cache_stats(self):
        """core/single/pikv_moe.py:388-402."""
        if not self.use_cache_scheduling:
            print("Cache scheduling is not enabled.")
            return
        print("\n===== Cache Scheduling Statistics =====")
        for expert_name, expert_stats in self.get_cache_stats().items():
            print(f"\n{expert_name.upper()}:")
            for stat_name, value in expert_stats.items():
                print(f"  {stat_name}: {value:.4f}" if isinstance(value, float) else f"  {stat_name}: {value}")
        print("\n======================================")

    # ---- distillation (core/single/pikv_moe.py:404-454): outside the cache data path ----
    def enable_distillation(self, teacher_model_path=None):
        raise NotImplementedError("knowledge distillation is not part of the cache data path")

    def disable_distillation(self):
        self.use_distillation = False

    def load_teacher_model(self, model_path):
        raise NotImplementedError("knowledge distillation is not part of the cache data path")

    def distillation_step(self, input_data, targets=None, optimizer=None):
        raise NotImplementedError("knowledge distillation is not part of the cache data path")

    # ---- checkpoint (core/single/pikv_moe.py:456-505) -----------------------------------
    def save_checkpoint(self, path):
        """The reference stores the module weights, the write pointers and one MEAN vector
        per expert cache (get_all).  Here 'kv_pool' holds the caches themselves - codes,
        scales, zero points, accumulators, timestamps and fill of the shared pool - so a
        resumed model continues with the very rows it had; 'kv_caches' keeps the
        reference's mean vectors for readers of that key.  Tensors and plain values only:
        the file loads with torch.load(weights_only=True)."""
        checkpoint = {
            'model_state_dict': self.state_dict(),
            'cache_ptrs': self.cache_ptrs,
            'kv_caches': [cache.get_all() for cache in self.kv_caches],
            'kv_pool': None if self.pool is None else self.pool.state_dict(),
            'clock': self.clock,
            'use_distillation': False,
            'use_cache_scheduling': self.use_cache_scheduling,
            'cache_scheduling_policy': self.cache_scheduling_policy.value if self.use_cache_scheduling else None,
        }
        if self.use_cache_scheduling:
            checkpoint['cache_stats'] = self.get_cache_stats()
        torch.save(checkpoint, path)

    def load_checkpoint(self, path):
        checkpoint = torch.load(path, weights_only=True)
        self.load_state_dict(checkpoint['model_state_dict'])
        self.cache_ptrs.copy_(checkpoint['cache_ptrs'])
        self.clock = int(checkpoint.get('clock', 0))
        if checkpoint.get('kv_pool') is not None:
            device = self.cache_ptrs.device
            self._ensure_pool(device).load_state_dict(checkpoint['kv_pool'])
        if checkpoint.get('use_cache_scheduling', False):
            policy_name = checkpoint.get('cache_scheduling_policy', 'none')
            try:
                self.enable_cache_scheduling(SchedulingPolicy(policy_name))
            except ValueError:
                print(f"Unknown scheduling policy in checkpoint: {policy_name}")
