"""Cache schedulers and the scheduling manager with the reference's interface
(core/single/cache_scheduling.py), backed by the HIP kernels.

  SchedulingPolicy ................ :9-17
  BaseScheduler ................... :19-51   (hit/miss/eviction counters)
  H2OScheduler .................... :53-99   (accumulator, timestamps, heavy/recent keep set)
  StreamingLLMScheduler ........... :101-134 (first tokens + recent window)
  QUESTScheduler .................. :136-203 (quality x frequency x time decay, threshold)
  FlexGenScheduler ................ :205-251 (access frequency / access cost)
  LRUScheduler .................... :253-285
  LRUPlusScheduler ................ :287-349 (recency + frequency + importance)
  AdaKVScheduler .................. core/single/module/pikv_scheduling.py:624-673
  DuoAttentionScheduler ........... core/single/module/pikv_scheduling.py:675-710
  CacheSchedulingManager .......... :351-467 (append / evict / compact / stats)

Every policy is "a score per row, then keep the top / drop the bottom": the score
is a handful of elementwise operations on [cache_size] buffers (left to torch),
the selection - exact top-k with ties to the lower index - runs in
pikv_evict_select, as does everything that moves rows.

Selection and compaction run in pikv_evict_select / pikv_compact_rows; the
manager stores its rows as integer codes in a one-cache CachePool (quantise +
append in pikv_quant_scatter) and exposes dequantised `cache_keys` /
`cache_values` views.  Two deliberate differences from the reference, both
switchable:
  * after a compaction the accumulator / timestamp entries move with their rows
    (the reference leaves them in place, detaching scores from rows);
  * LRU evicts the `cur + n - C` least recently used rows before appending (the
    reference's LRU never evicts because it is only ever shown `cur <= C` rows
    and then silently drops the new ones); `legacy_no_evict=True` restores that.
Ties in every selection go to the lower index.  GPU tensors only.
"""
from __future__ import annotations

from enum import Enum
from typing import Dict, Optional

import torch
import torch.nn as nn

from . import ops


class SchedulingPolicy(Enum):
    NONE = "none"
    H2O = "h2o"
    STREAMING_LLM = "streaming_llm"
    QUEST = "quest"
    FLEXGEN = "flexgen"
    LRU = "lru"
    LRU_PLUS = "lru_plus"
    ADAKV = "adakv"                 # core/single/module/pikv_scheduling.py:23-33
    DUOATTENTION = "duoattention"


class BaseScheduler(nn.Module):
    def __init__(self, cache_size: int, hidden_size: int):
        super().__init__()
        self.cache_size = cache_size
        self.hidden_size = hidden_size
        self.register_buffer("hit_count", torch.tensor(0))
        self.register_buffer("miss_count", torch.tensor(0))
        self.register_buffer("eviction_count", torch.tensor(0))

    def get_hit_rate(self) -> float:
        total = self.hit_count + self.miss_count
        return float(self.hit_count.float() / total.float()) if total > 0 else 0.0

    def reset_stats(self):
        self.hit_count.zero_()
        self.miss_count.zero_()
        self.eviction_count.zero_()

    def should_evict(self, cache_usage, new_importance):
        raise NotImplementedError

    def select_eviction_candidates(self, keys, values, metadata):
        raise NotImplementedError


def _one_cache_select(policy: int, acc: Optional[torch.Tensor], ts: torch.Tensor, length: int,
                      *, heavy_ratio=0.1, recent_ratio=0.1, n_evict=0, budgets=None) -> torch.Tensor:
    """Run the native selection on a single cache of `length` rows whose state is
    acc/ts (float32, >= length entries).  Returns the bool EVICT mask [length]."""
    from . import _native as N
    dev = ts.device
    if dev.type != "cuda":
        raise ValueError("schedulers need GPU tensors; there is no CPU path")
    if length == 0:
        return torch.zeros(0, dtype=torch.bool, device=dev)
    i32 = dict(dtype=torch.int32, device=dev)
    row_base = torch.zeros(1, dtype=torch.int64, device=dev)
    fill = torch.tensor([length], **i32)
    nh, nr = torch.zeros(1, **i32), torch.zeros(1, **i32)
    flag = torch.empty(length, dtype=torch.uint8, device=dev)
    kidx = torch.empty(length, **i32)
    new_len = torch.empty(1, **i32)
    st = torch.cuda.current_stream().cuda_stream
    if policy == ops.EVICT_H2O and budgets is not None:   # explicit (n_heavy, n_recent)
        nh.fill_(int(budgets[0]))
        nr.fill_(int(budgets[1]))
    elif policy == ops.EVICT_H2O:
        N.call("pikv_h2o_budget", fill.data_ptr(), 1, float(heavy_ratio), float(recent_ratio),
               nh.data_ptr(), nr.data_ptr(), st)
    else:
        nh.fill_(int(n_evict))
    N.call("pikv_evict_select", policy, None if acc is None else acc.data_ptr(), ts.data_ptr(),
           row_base.data_ptr(), fill.data_ptr(), nh.data_ptr(), nr.data_ptr(), 1, length, flag.data_ptr(),
           kidx.data_ptr(), new_len.data_ptr(), None, 0, st)
    return flag == 0


class H2OScheduler(BaseScheduler):
    def __init__(self, cache_size: int, hidden_size: int, heavy_ratio: float = 0.1,
                 recent_ratio: float = 0.1):
        super().__init__(cache_size, hidden_size)
        self.heavy_ratio = heavy_ratio
        self.recent_ratio = recent_ratio
        self.register_buffer("attention_accumulator", torch.zeros(cache_size))
        self.register_buffer("access_timestamps", torch.zeros(cache_size))
        self.register_buffer("current_time", torch.tensor(0))

    def update_attention_scores(self, indices: torch.Tensor, attention_weights: torch.Tensor):
        """acc[idx] += w; ts[idx] = t; t += 1 (:69-73).  The bulk form of this
        update - scores of a whole cache folded in by one kernel - is
        CachePool.h2o_accumulate; this method is the reference's indexed form."""
        self.attention_accumulator[indices] += attention_weights
        self.access_timestamps[indices] = self.current_time.float()
        self.current_time += 1

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len > self.attention_accumulator.numel():
            raise ValueError(f"{cache_len} rows shown to a scheduler that tracks {self.attention_accumulator.numel()}")
        return _one_cache_select(ops.EVICT_H2O, self.attention_accumulator.contiguous(),
                                 self.access_timestamps.contiguous(), cache_len,
                                 heavy_ratio=self.heavy_ratio, recent_ratio=self.recent_ratio)


class LRUScheduler(BaseScheduler):
    def __init__(self, cache_size: int, hidden_size: int):
        super().__init__(cache_size, hidden_size)
        self.register_buffer("access_times", torch.zeros(cache_size))
        self.register_buffer("global_time", torch.tensor(0))

    def update_access_time(self, indices: torch.Tensor):
        self.access_times[indices] = self.global_time.float()
        self.global_time += 1

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len <= self.cache_size:
            return torch.zeros(cache_len, dtype=torch.bool, device=keys.device)
        times = self.access_times
        if times.numel() < cache_len:   # rows beyond the tracked range count as never accessed
            times = torch.cat([times, torch.zeros(cache_len - times.numel(), device=times.device)])
        return _one_cache_select(ops.EVICT_LRU, None, times.contiguous(), cache_len,
                                 n_evict=cache_len - self.cache_size)


def _evict_lowest(score: torch.Tensor, cache_len: int, n_evict: int) -> torch.Tensor:
    """EVICT mask of the n_evict lowest scores among the first cache_len (ties: the
    lower index goes first), through the native smallest-n selection."""
    if n_evict <= 0:
        return torch.zeros(cache_len, dtype=torch.bool, device=score.device)
    return _one_cache_select(ops.EVICT_LRU, None, score[:cache_len].float().contiguous(), cache_len,
                             n_evict=min(n_evict, cache_len))


def _padded(buf: torch.Tensor, n: int, fill: float = 0.0) -> torch.Tensor:
    """First n entries of a per-slot buffer; slots beyond the tracked range read `fill`."""
    if buf.numel() >= n:
        return buf[:n]
    return torch.cat([buf, torch.full((n - buf.numel(),), fill, dtype=buf.dtype, device=buf.device)])


class StreamingLLMScheduler(BaseScheduler):
    """Keep the first start_size rows and the last recent_size rows (:101-134)."""

    def __init__(self, cache_size: int, hidden_size: int, start_size: int = 4,
                 recent_size: Optional[int] = None):
        super().__init__(cache_size, hidden_size)
        self.start_size = start_size
        self.recent_size = recent_size if recent_size is not None else (cache_size - start_size)
        self.register_buffer("position_counter", torch.tensor(0))

    def keep_budgets(self, cache_len: int):
        """(rows kept at the front, rows kept at the back) of a cache_len-row cache."""
        n_start = min(self.start_size, cache_len)
        recent_start = max(self.start_size, cache_len - self.recent_size)
        return n_start, max(0, cache_len - recent_start)

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len <= self.cache_size:
            return torch.zeros(cache_len, dtype=torch.bool, device=keys.device)
        return self.evict_mask(cache_len, keys.device)

    def evict_mask(self, cache_len: int, device) -> torch.Tensor:
        # position is the score: the "heavy" set takes the lowest positions, the
        # "recent" set the highest
        pos = torch.arange(cache_len, dtype=torch.float32, device=device)
        n_start, n_recent = self.keep_budgets(cache_len)
        return _one_cache_select(ops.EVICT_H2O, (-pos).contiguous(), pos, cache_len,
                                 budgets=(n_start, n_recent))


class QUESTScheduler(BaseScheduler):
    """utility = quality * usage frequency * decay^(now - last access); rows below
    the threshold go, or the lowest cache_len - cache_size when those are too few
    (:136-203)."""

    def __init__(self, cache_size: int, hidden_size: int, quality_threshold: float = 0.1,
                 decay_factor: float = 0.95):
        super().__init__(cache_size, hidden_size)
        self.quality_threshold = quality_threshold
        self.decay_factor = decay_factor
        self.register_buffer("quality_scores", torch.zeros(cache_size))
        self.register_buffer("usage_frequency", torch.zeros(cache_size))
        self.register_buffer("last_access_time", torch.zeros(cache_size))
        self.register_buffer("global_time", torch.tensor(0))

    def update_quality_scores(self, indices: torch.Tensor, reconstruction_errors: torch.Tensor):
        self.quality_scores[indices] = 1.0 / (1.0 + reconstruction_errors)
        self.usage_frequency[indices] += 1
        self.last_access_time[indices] = self.global_time.float()
        self.global_time += 1

    def compute_utility_scores(self, cache_len: int) -> torch.Tensor:
        last = _padded(self.last_access_time, cache_len)
        decay = torch.pow(torch.tensor(self.decay_factor, device=last.device),
                          self.global_time.float() - last)
        return _padded(self.quality_scores, cache_len) * _padded(self.usage_frequency, cache_len) * decay

    def row_buffers(self):
        return [self.quality_scores, self.usage_frequency, self.last_access_time]

    def evict_mask(self, cache_len: int, n_evict: int) -> torch.Tensor:
        utility = self.compute_utility_scores(cache_len)
        below = utility < self.quality_threshold
        if int(below.sum()) < n_evict:
            return _evict_lowest(utility, cache_len, n_evict)
        return below

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len <= self.cache_size:
            return torch.zeros(cache_len, dtype=torch.bool, device=keys.device)
        return self.evict_mask(cache_len, cache_len - self.cache_size)


class FlexGenScheduler(BaseScheduler):
    """benefit = access frequency / access cost; the lowest go (:205-251)."""

    def __init__(self, cache_size: int, hidden_size: int, gpu_ratio: float = 0.3,
                 cpu_ratio: float = 0.5):
        super().__init__(cache_size, hidden_size)
        self.gpu_ratio, self.cpu_ratio = gpu_ratio, cpu_ratio
        self.gpu_cache_size = int(cache_size * gpu_ratio)
        self.cpu_cache_size = int(cache_size * cpu_ratio)
        self.disk_cache_size = cache_size - self.gpu_cache_size - self.cpu_cache_size
        self.register_buffer("access_frequency", torch.zeros(cache_size))
        self.register_buffer("access_cost", torch.ones(cache_size))
        self.register_buffer("cache_level", torch.zeros(cache_size, dtype=torch.long))

    def update_access_patterns(self, indices: torch.Tensor, access_costs: torch.Tensor):
        self.access_frequency[indices] += 1
        self.access_cost[indices] = access_costs

    def compute_benefit_scores(self, cache_len: int) -> torch.Tensor:
        return _padded(self.access_frequency, cache_len) / _padded(self.access_cost, cache_len, 1.0)

    def row_buffers(self):
        return [self.access_frequency, self.access_cost]

    def evict_mask(self, cache_len: int, n_evict: int) -> torch.Tensor:
        return _evict_lowest(self.compute_benefit_scores(cache_len), cache_len, n_evict)

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len <= self.cache_size:
            return torch.zeros(cache_len, dtype=torch.bool, device=keys.device)
        return self.evict_mask(cache_len, cache_len - self.cache_size)


class LRUPlusScheduler(BaseScheduler):
    """priority = w_r * recency + w_f * frequency + w_i * importance, recency and
    frequency normalised by their maxima; the lowest go (:287-349)."""

    def __init__(self, cache_size: int, hidden_size: int, frequency_weight: float = 0.3,
                 importance_weight: float = 0.4):
        super().__init__(cache_size, hidden_size)
        self.frequency_weight = frequency_weight
        self.importance_weight = importance_weight
        self.recency_weight = 1.0 - frequency_weight - importance_weight
        self.register_buffer("access_times", torch.zeros(cache_size))
        self.register_buffer("access_frequency", torch.zeros(cache_size))
        self.register_buffer("importance_scores", torch.zeros(cache_size))
        self.register_buffer("global_time", torch.tensor(0))

    def update_access_info(self, indices: torch.Tensor, importance: torch.Tensor):
        self.access_times[indices] = self.global_time.float()
        self.access_frequency[indices] += 1
        self.importance_scores[indices] = importance
        self.global_time += 1

    def compute_priority_scores(self, cache_len: int) -> torch.Tensor:
        times = _padded(self.access_times, cache_len)
        freq = _padded(self.access_frequency, cache_len)
        recency = times / (times.max() + 1e-8)
        frequency = freq / (freq.max() + 1e-8)
        return (self.recency_weight * recency + self.frequency_weight * frequency +
                self.importance_weight * _padded(self.importance_scores, cache_len))

    def row_buffers(self):
        return [self.access_times, self.access_frequency, self.importance_scores]

    def evict_mask(self, cache_len: int, n_evict: int) -> torch.Tensor:
        return _evict_lowest(self.compute_priority_scores(cache_len), cache_len, n_evict)

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len <= self.cache_size:
            return torch.zeros(cache_len, dtype=torch.bool, device=keys.device)
        return self.evict_mask(cache_len, cache_len - self.cache_size)



class AdaKVScheduler(BaseScheduler):
    """Keep the int(len*(1-compression_ratio)) rows with the highest linear importance
    score (core/single/module/pikv_scheduling.py:624-673).  The reference picks a
    safeguarded top slice first and fills up from the rest; both slices together are the
    plain top-num_keep of one score, which is what the native selection returns."""

    def __init__(self, cache_size: int, hidden_size: int, compression_ratio: float = 0.5,
                 safeguard_ratio: float = 0.2):
        super().__init__(cache_size, hidden_size)
        self.compression_ratio = compression_ratio
        self.safeguard_ratio = safeguard_ratio
        self.register_buffer("importance_scores", torch.zeros(cache_size))
        self.linear_proj = nn.Linear(hidden_size, 1)

    def update_importance(self, indices: torch.Tensor, keys: torch.Tensor):
        with torch.no_grad():
            self.importance_scores[indices] = self.linear_proj(keys).squeeze(-1)

    def row_buffers(self):
        return [self.importance_scores]

    def num_keep(self, cache_len: int) -> int:
        return int(cache_len * (1 - self.compression_ratio))

    def evict_mask(self, cache_len: int, n_evict: int = 0) -> torch.Tensor:
        """n_evict > 0 (the manager making room) lowers the kept count when needed."""
        scores = _padded(self.importance_scores, cache_len).float().contiguous()
        keep = max(0, min(self.num_keep(cache_len), cache_len - n_evict))
        return _one_cache_select(ops.EVICT_H2O, scores, scores, cache_len, budgets=(keep, 0))

    def select_eviction_candidates(self, keys, values, metadata) -> torch.Tensor:
        cache_len = keys.size(0)
        if cache_len <= self.cache_size:
            return torch.zeros(cache_len, dtype=torch.bool, device=keys.device)
        return self.evict_mask(cache_len)


class DuoAttentionScheduler(StreamingLLMScheduler):
    """Keep sink_size rows at the front and recent_size rows at the back
    (core/single/module/pikv_scheduling.py:675-710)."""

    def __init__(self, cache_size: int, hidden_size: int, sink_size: int = 64, recent_size: int = 512):
        super().__init__(cache_size, hidden_size, start_size=sink_size, recent_size=recent_size)
        self.sink_size = sink_size

    def keep_budgets(self, cache_len: int):
        # the reference keeps [:sink] and [-recent:] independently (they may overlap)
        n_start = min(self.sink_size, cache_len)
        return n_start, min(self.recent_size, cache_len)


_NATIVE = {SchedulingPolicy.H2O: ops.EVICT_H2O, SchedulingPolicy.LRU: ops.EVICT_LRU}


class CacheSchedulingManager(nn.Module):
    """Quantised, natively scheduled replacement of the reference manager.

    cache_size rows of hidden_size values; rows are stored as codes
    (`quant`: 'int8' symmetric per token by default, 'int8_asym', 'int4',
    'int4_sym'; `group` = elements per scale, default the whole row when that
    is a power of two, else 128/64/32)."""

    def __init__(self, cache_size: int, hidden_size: int,
                 policy: SchedulingPolicy = SchedulingPolicy.NONE, *, device=None,
                 quant: str = "int8", group: Optional[int] = None, n_heads: int = 1,
                 heavy_ratio: float = 0.1, recent_ratio: float = 0.1,
                 legacy_no_evict: bool = False):
        super().__init__()
        self.cache_size = cache_size
        self.hidden_size = hidden_size
        self.policy = policy
        self.legacy_no_evict = legacy_no_evict
        self.heavy_ratio, self.recent_ratio = heavy_ratio, recent_ratio
        self.scheme = {"int8": ops.Q_I8_SYM, "int8_asym": ops.Q_I8_ASYM, "int4": ops.Q_I4_ASYM,
                       "int4_sym": ops.Q_I4_SYM}[quant]
        if group is None:
            eight = ops.scheme_bits(self.scheme) == 8
            lo, hi = (16, 1024) if eight else (32, 2048)
            cands = [hidden_size] + [g for g in (2048, 1024, 512, 256, 128, 64, 32, 16)]
            group = next((g for g in cands
                          if lo <= g <= hi and g & (g - 1) == 0 and hidden_size % g == 0), None)
            if group is None:
                raise ValueError(f"hidden_size {hidden_size} has no power-of-two quantisation group")
        self.group = group
        self.n_heads = n_heads
        self.scheduler = self._create_scheduler(policy)
        self._device = torch.device(device) if device is not None else None
        self.pool: Optional[ops.CachePool] = None
        self.time = 0
        self.register_buffer("cache_valid", torch.zeros(cache_size, dtype=torch.bool))
        self._fill_host = 0

    # ---- construction --------------------------------------------------------
    def _create_scheduler(self, policy):
        if policy == SchedulingPolicy.NONE:
            return None
        if policy == SchedulingPolicy.H2O:
            return H2OScheduler(self.cache_size, self.hidden_size, self.heavy_ratio, self.recent_ratio)
        if policy == SchedulingPolicy.LRU:
            return LRUScheduler(self.cache_size, self.hidden_size)
        if policy == SchedulingPolicy.STREAMING_LLM:
            return StreamingLLMScheduler(self.cache_size, self.hidden_size)
        if policy == SchedulingPolicy.QUEST:
            return QUESTScheduler(self.cache_size, self.hidden_size)
        if policy == SchedulingPolicy.FLEXGEN:
            return FlexGenScheduler(self.cache_size, self.hidden_size)
        if policy == SchedulingPolicy.LRU_PLUS:
            return LRUPlusScheduler(self.cache_size, self.hidden_size)
        if policy == SchedulingPolicy.ADAKV:
            return AdaKVScheduler(self.cache_size, self.hidden_size)
        if policy == SchedulingPolicy.DUOATTENTION:
            return DuoAttentionScheduler(self.cache_size, self.hidden_size,
                                         sink_size=max(1, self.cache_size // 16),
                                         recent_size=max(1, self.cache_size // 2))
        raise ValueError(f"Unknown scheduling policy: {policy}")

    def _ensure_pool(self, device):
        if self.pool is None:
            dev = self._device or device
            self.pool = ops.CachePool([self.cache_size], self.n_heads, self.hidden_size // self.n_heads,
                                      self.group, self.scheme, dev)
        return self.pool

    # ---- reference surface ----------------------------------------------------
    @property
    def cache_size_current(self) -> torch.Tensor:
        return torch.tensor(self._fill_host)

    @property
    def cache_keys(self) -> torch.Tensor:
        """Dequantised [cache_size, hidden_size] view (rows beyond the fill are zero)."""
        return self._dequant("k")

    @property
    def cache_values(self) -> torch.Tensor:
        return self._dequant("v")

    def _dequant(self, which):
        if self.pool is None:
            raise RuntimeError("cache is empty: nothing has been written yet")
        out = torch.zeros(self.cache_size, self.hidden_size, device=self.pool.device)
        if self._fill_host:
            out[:self._fill_host] = self.pool.gather_dequant(which, row0=0, n=self._fill_host)
        return out

    def update_cache(self, keys: torch.Tensor, values: torch.Tensor,
                     metadata: Optional[Dict[str, torch.Tensor]] = None):
        """core/single/cache_scheduling.py:391-436: flatten, evict + compact when the
        new rows do not fit, append, truncate silently at the cache size."""
        if self.scheduler is None:
            return
        if keys.dim() != 3:
            raise ValueError("keys must be [batch, seq, hidden]")
        hidden = keys.shape[-1]
        if hidden != self.hidden_size:
            raise ValueError(f"hidden size {hidden} != {self.hidden_size}")
        k2 = keys.reshape(-1, hidden).contiguous()
        v2 = values.reshape(-1, hidden).contiguous()
        if k2.dtype not in (torch.float32, torch.bfloat16):
            k2, v2 = k2.float(), v2.float()
        pool = self._ensure_pool(k2.device)
        n = k2.shape[0]
        cur = self._fill_host
        if cur + n > self.cache_size and cur > 0:
            n_ev = min(cur, cur + n - self.cache_size)
            if self.policy == SchedulingPolicy.H2O:
                pool.evict(ops.EVICT_H2O, heavy_ratio=self.scheduler.heavy_ratio,
                           recent_ratio=self.scheduler.recent_ratio)
            elif self.legacy_no_evict:
                pass
            elif self.policy == SchedulingPolicy.LRU:
                pool.evict(ops.EVICT_LRU, n_evict=torch.tensor([n_ev], dtype=torch.int32, device=pool.device))
            else:
                self._evict_by_scheduler(pool, cur, n_ev)
            new_cur = int(pool.fill.item())
            self.scheduler.eviction_count += cur - new_cur
            cur = new_cur
        self.time += 1
        dev = pool.device
        cid = torch.zeros(n, dtype=torch.int32, device=dev)
        slot = torch.arange(n, dtype=torch.int32, device=dev)
        pool.quant_scatter(k2, v2, cid, slot, 1, now=float(self.time))
        pool.advance(torch.tensor([n], dtype=torch.int32, device=dev))
        self._fill_host = min(cur + n, self.cache_size)
        self.cache_valid = torch.arange(self.cache_size) < self._fill_host

    def _evict_by_scheduler(self, pool, cur: int, n_ev: int):
        """StreamingLLM / DuoAttention / QUEST / FlexGen / LRU+ / AdaKV: the scheduler scores its slots, the
        native selection turns the score into a keep list, and the compaction moves
        the scheduler's per-slot buffers together with the rows."""
        sch = self.scheduler.to(pool.device)
        if isinstance(sch, StreamingLLMScheduler):
            # room for the new rows: the window shrinks to what fits beside the start tokens
            n_start = min(sch.start_size, cur)
            n_recent = max(0, min(cur - n_start, cur - n_ev - n_start))
            pos = torch.arange(pool.rows, dtype=torch.float32, device=pool.device)
            evict = _one_cache_select(ops.EVICT_H2O, (-pos).contiguous(), pos, cur,
                                      budgets=(n_start, n_recent))
            extra = []
        else:
            evict = sch.evict_mask(cur, n_ev)
            extra = sch.row_buffers()
        keep = ~evict
        m = int(keep.sum())
        pool.keep_flag[:cur] = keep.to(torch.uint8)
        pool.keep_index[:m] = torch.nonzero(keep).reshape(-1).to(torch.int32)
        pool.new_len.fill_(m)
        pool.compact(extra_planes=extra)
        for b in extra:   # slots behind the survivors start fresh
            b[m:] = 1.0 if b is getattr(sch, "access_cost", None) else 0.0

    def get_cache_stats(self) -> Dict[str, float]:
        stats = {"cache_size": self._fill_host,
                 "cache_utilization": self._fill_host / self.cache_size,
                 "policy": self.policy.value}
        if self.scheduler is not None:
            stats.update({"hit_rate": self.scheduler.get_hit_rate(),
                          "eviction_count": int(self.scheduler.eviction_count.item())})
        return stats

    def reset_cache(self):
        if self.pool is not None:
            self.pool.fill.zero_()
            for p in self.pool.planes():
                p.zero_()
        self._fill_host = 0
        self.cache_valid = torch.zeros(self.cache_size, dtype=torch.bool)
        if self.scheduler is not None:
            self.scheduler.reset_stats()

    def change_policy(self, new_policy: SchedulingPolicy):
        self.policy = new_policy
        self.scheduler = self._create_scheduler(new_policy)
