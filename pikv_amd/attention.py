"""PiKVAttention with the reference's interface (core/single/pikv_attention.py:7-283)
on a quantised, natively read KV cache.

The reference keeps `k_cache` / `v_cache` as float buffers `[cache_size, heads, head_dim]`
that `forward` only ever writes (`_update_cache`, :74-102) and attends over the K/V of
the current call.  Here every sequence of the batch owns one cache of a shared
`CachePool` (rows = tokens, quantised on the way in by the fused quantise + scatter
kernel), and a single-token call - the decode step - attends over the WHOLE cached
context natively:

    scores   = pikv_gather_dequant_scores   (QK^T over the compressed K rows, :123)
    softmax  = pikv_h2o_accumulate          (:163; here only the per-head max and sum)
    context  = pikv_attend_values           (probabilities x compressed V rows, :188; the same
                                             pass adds the probabilities to the H2O importance)

Multi-token or masked calls compute their attention in torch as the reference does, over
the dequantised cached rows followed by their own K/V (the reference concatenates
`past_key_values` and the current K/V, :240-244), and write their K/V rows into the cache.  When a cache would overflow, the
reference wipes it (:85-90); here H2O eviction keeps the heavy and the recent rows
(`on_overflow="reset"` restores the wipe).

`load_past_key_values` accepts `(k, v)` in the Hugging Face layout `[batch, heads, seq,
head_dim]` or the reference's `[batch, seq, heads, head_dim]`, tuples of per-layer pairs and
cache objects (transformers' DynamicCache); `past_key_values` returns the Hugging Face layout.
"""
from __future__ import annotations

import math
import warnings
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

_SCHEMES = {"int8": ops.Q_I8_SYM, "int8_asym": ops.Q_I8_ASYM, "int4": ops.Q_I4_ASYM,
            "int4_sym": ops.Q_I4_SYM}


class RotaryEmbedding(nn.Module):
    """core/single/pikv_attention.py:285-363 (rotate-half form on [B,S,heads,dim])."""

    def __init__(self, dim: int, max_position_embeddings: int = 2048):
        super().__init__()
        self.dim = dim
        self.max_position_embeddings = max_position_embeddings
        position = torch.arange(max_position_embeddings, dtype=torch.float).unsqueeze(1)
        freq = 1.0 / (10000 ** (torch.arange(0, dim, step=2, dtype=torch.float) / dim))
        self.register_buffer("cos_cached", torch.cos(position * freq), persistent=False)
        self.register_buffer("sin_cached", torch.sin(position * freq), persistent=False)

    def forward(self, q, k, position_ids):
        cos = self.cos_cached[position_ids].unsqueeze(2)   # [B,S,1,dim/2]
        sin = self.sin_cached[position_ids].unsqueeze(2)

        def rot(x):
            x1, x2 = x[..., 0::2], x[..., 1::2]
            out = torch.empty_like(x)
            out[..., 0::2] = x1 * cos - x2 * sin
            out[..., 1::2] = x1 * sin + x2 * cos
            return out
        return rot(q), rot(k)


class PiKVAttention(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: Optional[int] = None,
                 dropout: float = 0.1, use_rotary: bool = False,
                 max_position_embeddings: int = 2048, cache_size: int = 4096, *,
                 num_kv_heads: Optional[int] = None, kv_quant: str = "int4", kv_group: int = 32,
                 heavy_ratio: float = 0.0625, recent_ratio: float = 0.0078125,
                 on_overflow: str = "h2o", layer_idx: int = 0, past_layout: str = "reference"):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.head_dim = head_dim if head_dim is not None else hidden_size // num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        if num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if on_overflow not in ("h2o", "reset"):
            raise ValueError("on_overflow must be 'h2o' or 'reset'")
        self.dropout = dropout
        self.use_rotary = use_rotary
        self.cache_size = cache_size
        self.scheme = _SCHEMES[kv_quant]
        self.kv_group = kv_group
        self.heavy_ratio, self.recent_ratio = heavy_ratio, recent_ratio
        self.on_overflow = on_overflow
        if past_layout not in ("hf", "reference"):
            raise ValueError("past_layout must be 'hf' or 'reference'")
        self.layer_idx, self.past_layout = layer_idx, past_layout
        self.q_proj = nn.Linear(hidden_size, num_heads * self.head_dim)
        self.k_proj = nn.Linear(hidden_size, self.num_kv_heads * self.head_dim)
        self.v_proj = nn.Linear(hidden_size, self.num_kv_heads * self.head_dim)
        self.o_proj = nn.Linear(num_heads * self.head_dim, hidden_size)
        self.attn_dropout = nn.Dropout(dropout)
        if use_rotary:
            self.rotary_emb = RotaryEmbedding(self.head_dim, max_position_embeddings)
        for m in (self.q_proj, self.k_proj, self.v_proj, self.o_proj):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
            nn.init.zeros_(m.bias)
        self.pool: Optional[ops.CachePool] = None
        self.clock = 0

    # ---- cache ---------------------------------------------------------------------
    def _ensure_pool(self, batch_size: int, device) -> ops.CachePool:
        if self.pool is None or self.pool.n_caches != batch_size:
            self.pool = ops.CachePool([self.cache_size] * batch_size, self.num_kv_heads, self.head_dim,
                                      self.kv_group, self.scheme, device)
            self.clock = 0
        return self.pool

    @property
    def cache_ptr(self) -> torch.Tensor:
        """Rows cached per sequence (the reference's single write pointer, per sequence)."""
        if self.pool is None:
            return torch.zeros(1, dtype=torch.long)
        return self.pool.fill.long()

    def reset_cache(self):
        if self.pool is not None:
            self.pool.fill.zero_()

    def _update_cache(self, k: torch.Tensor, v: torch.Tensor):
        """Append k, v [B,S,kv_heads,head_dim] to the B caches (core/single/
        pikv_attention.py:74-102), making room first when a cache would overflow."""
        B, S = k.shape[0], k.shape[1]
        pool = self._ensure_pool(B, k.device)
        dev = pool.device
        n_new = torch.full((B,), min(S, self.cache_size), dtype=torch.int32, device=dev)
        over = (pool.fill + n_new - pool.cap).clamp_min(0)
        if self.on_overflow == "reset":
            pool.fill.copy_(torch.where(over > 0, torch.zeros_like(pool.fill), pool.fill))
        else:
            f = pool.fill.double()
            nh = (f * self.heavy_ratio).floor().clamp_min(1).to(torch.int32)
            nr = (f * self.recent_ratio).floor().clamp_min(1).to(torch.int32)
            # never keep more than what leaves room for the new rows
            room = (pool.cap - n_new).clamp_min(0)
            nh = torch.minimum(nh, room)
            nr = torch.minimum(nr, (room - nh).clamp_min(0))
            keep_all = over == 0
            pool.evict(ops.EVICT_H2O, n_heavy=torch.where(keep_all, pool.fill, nh).contiguous(),
                       n_recent=torch.where(keep_all, torch.zeros_like(nr), nr).contiguous())
        self.clock += 1
        D = self.num_kv_heads * self.head_dim
        dt = k.dtype if k.dtype in (torch.float32, torch.bfloat16) else torch.float32
        cid = torch.arange(B, dtype=torch.int32, device=dev).repeat_interleave(S)
        slot = torch.arange(S, dtype=torch.int32, device=dev).repeat(B)
        pool.quant_scatter(k.reshape(B * S, D).to(dt).contiguous(), v.reshape(B * S, D).to(dt).contiguous(),
                           cid, slot, 1, now=float(self.clock))
        pool.advance(n_new)

    def _split_past(self, past_key_values, layer_idx: Optional[int]):
        """(k, v) tensors of one layer out of what callers carry: a (k, v) pair, a tuple of
        per-layer pairs (downstream_tasks/llm/next_tok_pred/s_transformers.py:85-98), or a
        cache object with per-layer `.layers[i].keys / .values` (transformers' DynamicCache)
        or `.key_cache[i] / .value_cache[i]` lists."""
        li = self.layer_idx if layer_idx is None else layer_idx
        pkv = past_key_values
        if hasattr(pkv, "layers"):
            layer = pkv.layers[li]
            return layer.keys, layer.values
        if hasattr(pkv, "key_cache") and hasattr(pkv, "value_cache"):
            return pkv.key_cache[li], pkv.value_cache[li]
        if isinstance(pkv, (tuple, list)) and len(pkv) > 0 and isinstance(pkv[0], (tuple, list)):
            pkv = pkv[li]
        if not (isinstance(pkv, (tuple, list)) and len(pkv) == 2 and all(isinstance(t, torch.Tensor) for t in pkv)):
            raise ValueError("past_key_values must be (k, v), a tuple of per-layer (k, v), or a cache object "
                             "with .layers[i].keys/.values")
        return pkv[0], pkv[1]

    def _to_rows(self, t: torch.Tensor, name: str, layout: str) -> torch.Tensor:
        """[B, rows, kv_heads, head_dim] from either layout, with the shape checked."""
        if t.dim() != 4 or t.shape[3] != self.head_dim:
            raise ValueError(f"{name}: expected 4 dimensions ending in head_dim={self.head_dim}, got {tuple(t.shape)}")
        hf = t.shape[1] == self.num_kv_heads          # [B, kv_heads, S, head_dim]
        ref = t.shape[2] == self.num_kv_heads         # [B, S, kv_heads, head_dim]
        if layout == "auto":
            if hf and ref:
                # S == kv_heads: the shape cannot tell.  past_layout decides - it is also the layout
                # forward() returns `present` in, so the module's own output always reads back right
                warnings.warn(f"{name} {tuple(t.shape)} fits both layouts; read as '{self.past_layout}' "
                              "(the module's past_layout) - pass layout= to say which", stacklevel=3)
                layout = self.past_layout
            elif hf or ref:
                layout = "hf" if hf else "reference"
            else:
                raise ValueError(f"{name}: neither [B, {self.num_kv_heads}, S, {self.head_dim}] nor "
                                 f"[B, S, {self.num_kv_heads}, {self.head_dim}]: got {tuple(t.shape)}")
        if layout == "hf":
            if not hf:
                raise ValueError(f"{name}: expected [B, {self.num_kv_heads}, S, {self.head_dim}], got {tuple(t.shape)}")
            return t.transpose(1, 2).contiguous()
        if layout == "reference":
            if not ref:
                raise ValueError(f"{name}: expected [B, S, {self.num_kv_heads}, {self.head_dim}], got {tuple(t.shape)}")
            return t.contiguous()
        raise ValueError("layout must be 'auto', 'hf' or 'reference'")

    def load_past_key_values(self, past_key_values, layout: str = "auto", layer_idx: Optional[int] = None):
        """Replace the caches' contents by a past context.  Accepted: (k, v) as
        [batch, kv_heads, seq, head_dim] (Hugging Face; layout "hf") or
        [batch, seq, kv_heads, head_dim] (the layout core/single/pikv_attention.py:240-244
        concatenates along dim 1; layout "reference"); a tuple of such pairs per layer; or a
        cache object (see _split_past).  "auto" tells the two layouts apart by which axis has
        kv_heads entries and falls back to `past_layout` when both do."""
        past_k, past_v = self._split_past(past_key_values, layer_idx)
        if past_k.shape != past_v.shape:
            raise ValueError(f"past k {tuple(past_k.shape)} and v {tuple(past_v.shape)} differ in shape")
        k_rows, v_rows = self._to_rows(past_k, "past k", layout), self._to_rows(past_v, "past v", layout)
        if k_rows.shape[1] > self.cache_size:
            raise ValueError(f"past context of {k_rows.shape[1]} rows exceeds cache_size={self.cache_size}")
        self.reset_cache()
        if k_rows.shape[1] > 0:
            self._update_cache(k_rows, v_rows)

    def _cached_rows(self):
        """Dequantised caches as rows: (k, v) [batch, L, kv_heads, head_dim] with L the longest
        fill, and valid [batch, L] (False past a sequence's fill).  None when nothing is cached."""
        pool = self.pool
        if pool is None:
            return None
        L = int(pool.fill.max().item())
        if L == 0:
            return None
        B = pool.n_caches
        valid = torch.arange(L, device=pool.device).unsqueeze(0) < pool.fill.unsqueeze(1)
        out = []
        for which in ("k", "v"):
            full = pool.gather_dequant(which).view(B, self.cache_size, self.num_kv_heads, self.head_dim)[:, :L]
            out.append(full * valid[:, :, None, None])
        return out[0], out[1], valid

    def past_key_values(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """Dequantised caches as (k, v) [batch, kv_heads, max cached rows, head_dim]; rows past
        a sequence's fill are zero."""
        if self.pool is None:
            raise RuntimeError("nothing cached yet")
        rows = self._cached_rows()
        if rows is None:
            B = self.pool.n_caches
            z = torch.zeros(B, self.num_kv_heads, 0, self.head_dim, device=self.pool.device)
            return z, z.clone()
        return rows[0].transpose(1, 2).contiguous(), rows[1].transpose(1, 2).contiguous()

    # ---- attention --------------------------------------------------------------------
    def _decode_attention(self, q: torch.Tensor) -> torch.Tensor:
        """q [B, heads, head_dim] against the whole compressed cache of each sequence."""
        pool = self.pool
        qq = q.to(torch.bfloat16) if q.dtype == torch.bfloat16 else q.float()
        # scores, softmax, probabilities x V rows and the H2O importance of the same probabilities: one call
        return pool.decode_attend(qq.contiguous(), self.num_heads, now=float(self.clock),
                                  scale_qk=1.0 / math.sqrt(self.head_dim))

    def _dense_attention(self, q, k, v, attention_mask, causal_mask, past=None):
        """core/single/pikv_attention.py:104-191 over [cached rows ; rows of this call]
        (:240-244 concatenates past and current K/V along the sequence axis)."""
        rep = self.num_heads // self.num_kv_heads
        B, S = q.shape[0], q.shape[1]
        key_valid = None
        if past is not None:
            past_k, past_v, past_valid = past
            k = torch.cat([past_k.to(k.dtype), k], dim=1)
            v = torch.cat([past_v.to(v.dtype), v], dim=1)
            key_valid = torch.cat([past_valid, torch.ones(B, S, dtype=torch.bool, device=q.device)], dim=1)
        m = k.shape[1]
        q = q.transpose(1, 2)
        k = k.transpose(1, 2).repeat_interleave(rep, dim=1)
        v = v.transpose(1, 2).repeat_interleave(rep, dim=1)
        s = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(self.head_dim)
        if attention_mask is not None:
            if attention_mask.dim() != 4:
                if attention_mask.dim() != 2 or attention_mask.shape[0] != B:
                    raise ValueError(f"attention_mask must be [batch, keys] or 4-D, got {tuple(attention_mask.shape)}")
                if attention_mask.shape[1] == S and m != S:
                    # a mask over this call's tokens only: the cached context stays visible
                    attention_mask = torch.cat([torch.ones(B, m - S, dtype=attention_mask.dtype,
                                                           device=attention_mask.device), attention_mask], dim=1)
                attention_mask = attention_mask.unsqueeze(1).unsqueeze(2)
            if attention_mask.shape[-1] != m:
                raise ValueError(f"attention_mask covers {attention_mask.shape[-1]} keys, the context has {m} "
                                 f"({m - S} cached + {S} new)")
            s = s.masked_fill(attention_mask == 0, float("-inf"))
        if key_valid is not None:
            s = s.masked_fill(~key_valid[:, None, None, :], float("-inf"))
        if causal_mask:
            n = s.shape[-2]
            tri = torch.triu(torch.ones(n, m, device=q.device), diagonal=1 + m - n).bool()
            s = s.masked_fill(tri, float("-inf"))
        p = self.attn_dropout(F.softmax(s, dim=-1))
        return torch.matmul(p, v).transpose(1, 2)                   # [B,S,heads,head_dim]

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_values=None,
                position_ids: Optional[torch.Tensor] = None, use_cache: bool = False,
                causal_mask: bool = True, stream_mode: bool = False,
                stream_position: Optional[int] = None):
        """The context of a call is everything cached (after `past_key_values`, if given, has
        replaced the caches' contents) followed by the call's own tokens.  A single new token
        without a mask takes the native read path over the compressed rows; any other call
        attends in torch over the dequantised cached rows plus its own exact K/V.  Call
        reset_cache() to start a new sequence."""
        B, S, _ = hidden_states.shape
        q = self.q_proj(hidden_states).view(B, S, self.num_heads, self.head_dim)
        k = self.k_proj(hidden_states).view(B, S, self.num_kv_heads, self.head_dim)
        v = self.v_proj(hidden_states).view(B, S, self.num_kv_heads, self.head_dim)
        if self.use_rotary and position_ids is not None:
            q, k = self.rotary_emb(q, k, position_ids)
        if past_key_values is not None:
            self.load_past_key_values(past_key_values)
        if self.pool is not None and self.pool.n_caches != B and int(self.pool.fill.max().item()) > 0:
            raise ValueError(f"batch of {B} sequences, but {self.pool.n_caches} caches hold a context: "
                             "reset_cache() first")
        if S == 1 and attention_mask is None:
            with torch.no_grad():
                self._update_cache(k.detach(), v.detach())
            context = self._decode_attention(q[:, 0]).unsqueeze(1)  # over everything cached
        else:
            with torch.no_grad():
                past = self._cached_rows()                          # before this call's rows go in
                self._update_cache(k.detach(), v.detach())
            context = self._dense_attention(q, k, v, attention_mask, causal_mask, past)
        output = self.o_proj(context.reshape(B, S, self.num_heads * self.head_dim).to(hidden_states.dtype))
        # `present` in the module's past_layout: [B,S,kv_heads,head_dim] as the reference returns it
        # (core/single/pikv_attention.py:240-247), or [B,kv_heads,S,head_dim] for past_layout="hf"
        present = None
        if use_cache:
            present = (k, v) if self.past_layout == "reference" else (k.transpose(1, 2), v.transpose(1, 2))
        return output, present
