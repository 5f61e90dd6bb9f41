"""Pyramid cache budgets and layer-wise top-k compression.

Mirrors ``PiKVMoE.pyramidal_cache_allocation`` (core/single/pikv_moe.py:218-224:
``C_l = C_1 - (l-1)*d``) and replaces the importance-descending partition of
``PyramidCompressor.forward`` (core/single/pikv_compression.py:145-160) by an
exact selection: layer l keeps its ``keep_l`` highest-scoring tokens (ties to the
lower index) in their original order and stores them quantised.  Selection and
quantisation run in the HIP library; nothing here touches the rows on the host.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from . import ops


def pyramidal_cache_allocation(kv_cache_size: int, cache_decrement: int, num_layers: int) -> List[int]:
    """core/single/pikv_moe.py:218-224."""
    return [kv_cache_size - (i - 1) * cache_decrement for i in range(1, num_layers + 1)]


def linear_keep_budget(n_tokens: int, num_layers: int, last_fraction: float = 0.25) -> List[int]:
    """Budget decaying linearly from 100 % (layer 0) to last_fraction (last layer):
    keep_l = int(N * (1 - (1 - last_fraction) * l / (L - 1))), evaluated in
    double precision like the reference's Python arithmetic."""
    if num_layers < 1:
        raise ValueError("num_layers must be >= 1")
    if num_layers == 1:
        return [int(n_tokens)]
    return [int(n_tokens * (1.0 - (1.0 - last_fraction) * l / (num_layers - 1)))
            for l in range(num_layers)]


class PyramidCache:
    """One quantised cache per layer, layer l sized keep[l]."""

    def __init__(self, keep: Sequence[int], n_heads: int, head_dim: int, *, group: int = None,
                 scheme: int = ops.Q_I8_SYM, device="cuda", with_v: bool = True):
        self.keep = [int(k) for k in keep]
        self.pool = ops.CachePool(self.keep, n_heads, head_dim, group or head_dim, scheme, device,
                                  with_v=with_v)
        self.n_layers = len(self.keep)
        self._n_keep = torch.tensor(self.keep, dtype=torch.int32, device=self.pool.device)

    def compress(self, keys, values, scores, now: float = 0.0):
        """keys/values [L, N, heads*head_dim] (or [L, N, heads, head_dim]), scores
        [L, N] float32.  Resets the caches, then fills layer l with its keep[l]
        best rows.  Returns (keep_index int32 [L*N], n_kept int32 [L])."""
        L = self.n_layers
        scores = scores.reshape(L, -1)
        n = scores.shape[1]
        if keys.shape[0] != L or keys.numel() != L * n * self.pool.D:
            raise ValueError("keys must be [layers, tokens, heads*head_dim]")
        if max(self.keep) > n:
            raise ValueError("a layer cannot keep more rows than it has")
        dev = self.pool.device
        seg_base = torch.arange(L, dtype=torch.int64, device=dev) * n
        seg_len = torch.full((L,), n, dtype=torch.int32, device=dev)
        flat = scores.contiguous().reshape(-1)
        _, index, kept = ops.select_top_rows(flat, seg_base, seg_len, self._n_keep, max_len=n)
        self.pool.fill.zero_()
        self.pool.quant_gather(keys, values if self.pool.with_v else None, seg_base, index, kept,
                               max(self.keep), src_score=flat, now=now)
        self.pool.advance(kept)
        return index, kept
