"""PiKVKernels facade: the reference's kernel-binding class
(core/single/pikv_kernels.py:20-422) with the same enums, method names, argument
order and return tuples, dispatching into libpikv_hip.so.

  top_k_routing(routing_logits, k) -> (indices, values)              :54-99
      the fallback there is torch.topk on the raw logits; ties go to the lower
      index here (torch's tie order is unspecified).
  compress_kv(keys, values, mode, lora_params) -> (k', v', meta)       :101-287
      QUANT8: the facade's own algebra (s = (max-min)/255, q = round((x-min)/s)
      clamped to 0..255, dq = q*s+min, :215-232) in pikv_quant8_minshift; meta holds
      k_scale, k_min, v_scale, v_min as [N,1] like the reference, plus the uint8
      codes (k_codes, v_codes), which the reference computes and throws away.
      NONE returns the inputs.  LORA (K + (K A) B * rank/hidden, :185-204) and MASK
      (entries below 0.1 x the row's mean magnitude set to zero, :248-275) are a dense
      product and an elementwise pass, done by torch on the GPU as the reference's own
      fallback does them - no kernel of this library is involved; they exist so that a
      caller of the facade finds every mode.  (The reference's LORA fallback multiplies
      by B through F.linear, which only accepts B as [hidden, rank]; both that layout and
      the [rank, hidden] one its own default allocates are taken here.)
  evict_cache(keys, values, timestamps, usage, now, policy, window, thr)
      -> (keys, values, timestamps, usage, new_size)                   :289-422
      SLIDING keeps rows with now - ts <= window; QUEST keeps rows with
      ||k|| * usage >= threshold; survivors are compacted in order by
      pikv_compact_rows.
Where the reference silently falls back to torch when its library is missing
(:44-52), this class raises.
"""
from __future__ import annotations

import ctypes as C
from enum import IntEnum
from typing import Dict, Optional, Tuple

import torch

from . import _native as N
from . import ops


class CompressionMode(IntEnum):
    NONE = 0
    LORA = 1
    QUANT8 = 2
    MASK = 3


class EvictionPolicy(IntEnum):
    SLIDING = 0
    QUEST = 1


class PiKVKernels:
    def __init__(self, lib_path: Optional[str] = None):
        if lib_path is not None:
            N.LIB_PATH = lib_path
        self.lib = N.lib()          # raises if the library is not built
        self.hip_enabled = True

    # ---- routing ---------------------------------------------------------------
    def top_k_routing(self, routing_logits: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
        out = ops.router_tail(routing_logits.float().contiguous(), top_k=k, use_softmax=False)
        return out.topk_idx, out.topk_w

    # ---- compression -------------------------------------------------------------
    def compress_kv(self, keys: torch.Tensor, values: torch.Tensor,
                    compression_mode: CompressionMode = CompressionMode.QUANT8,
                    lora_params: Optional[Dict[str, torch.Tensor]] = None):
        mode = CompressionMode(compression_mode)
        if mode == CompressionMode.NONE:
            return keys, values, {"compression_type": "none"}
        if keys.dim() != 2 or values.shape != keys.shape:
            raise ValueError("keys and values must be [batch, hidden] of one shape")
        if keys.device.type != "cuda":
            raise ValueError("compress_kv needs GPU tensors; there is no CPU path")
        hidden = keys.shape[1]
        if mode == CompressionMode.LORA:
            rank = max(int(hidden * 0.1), 1)
            if lora_params is None:      # the reference's default: random A, zero B - the identity
                a_k = torch.randn(hidden, rank, device=keys.device) * 0.1
                a_v = torch.randn(hidden, rank, device=keys.device) * 0.1
                b_k = torch.zeros(rank, hidden, device=keys.device)
                b_v = torch.zeros(rank, hidden, device=keys.device)
            else:
                a_k, b_k = lora_params.get('lora_a_k'), lora_params.get('lora_b_k')
                a_v, b_v = lora_params.get('lora_a_v'), lora_params.get('lora_b_v')
                rank = a_k.shape[1]

            def adapt(x, a, b):
                if b.shape == (hidden, rank) and hidden != rank:
                    b = b.t()
                return x + ((x.float() @ a.float()) @ b.float()).to(x.dtype) * (rank / hidden)
            return adapt(keys, a_k, b_k), adapt(values, a_v, b_v), {
                "compression_type": "lora", "lora_rank": rank, "lora_ratio": rank / hidden}
        if mode == CompressionMode.MASK:
            threshold = 0.1
            k_mask = keys.abs() >= threshold * keys.abs().mean(dim=1, keepdim=True)
            v_mask = values.abs() >= threshold * values.abs().mean(dim=1, keepdim=True)
            return keys * k_mask.to(keys.dtype), values * v_mask.to(values.dtype), {
                "compression_type": "mask", "threshold": threshold,
                "k_sparsity": 1.0 - k_mask.float().mean().item(),
                "v_sparsity": 1.0 - v_mask.float().mean().item()}
        ck, kc, ks, kmin = ops.quant8_minshift(keys)
        cv, vc, vs, vmin = ops.quant8_minshift(values)
        meta = {"compression_type": "quant8", "k_scale": ks, "k_min": kmin, "v_scale": vs, "v_min": vmin,
                "k_codes": kc, "v_codes": vc}
        return ck.to(keys.dtype), cv.to(values.dtype), meta

    # ---- eviction ------------------------------------------------------------------
    def evict_cache(self, keys, values, timestamps, usage_counts, current_time: int,
                    policy: EvictionPolicy, window_threshold: int = 1024,
                    quest_threshold: float = 0.1, inplace: bool = False):
        """Returns (keys, values, timestamps, usage_counts, new_size) of the surviving rows, in order.
        inplace=False (the reference's behaviour, core/single/pikv_kernels.py:386-420): the inputs are
        left as they are and the survivors are moved inside copies.  inplace=True: the survivors are
        moved to the front of the caller's own (contiguous) tensors, no copy is made, and the returned
        tensors are views of their first new_size rows."""
        n, hidden = keys.shape
        dev = keys.device
        if dev.type != "cuda":
            raise ValueError("evict_cache needs GPU tensors; there is no CPU path")
        if EvictionPolicy(policy) == EvictionPolicy.SLIDING:
            valid = (current_time - timestamps) <= window_threshold
        else:
            valid = torch.linalg.vector_norm(keys.float(), dim=1) * usage_counts >= quest_threshold
        keep_index = torch.nonzero(valid, as_tuple=False).reshape(-1).to(torch.int32).contiguous()
        new_size = int(keep_index.numel())
        if new_size == 0:
            return keys[:0], values[:0], timestamps[:0], usage_counts[:0], 0
        if inplace:
            planes = [keys, values, timestamps, usage_counts]
            if not all(p.is_contiguous() for p in planes):
                raise ValueError("inplace=True needs contiguous tensors")
        else:
            planes = [keys.clone().contiguous(), values.clone().contiguous(),
                      timestamps.clone().contiguous(), usage_counts.clone().contiguous()]
        if any((p[0].numel() * p.element_size()) % 4 for p in planes):
            raise ValueError("rows must be a multiple of 4 bytes")
        # one cache spanning all rows: keep_index is already the ascending survivor list
        kidx = torch.zeros(n, dtype=torch.int32, device=dev)
        kidx[:new_size] = keep_index
        row_base = torch.zeros(1, dtype=torch.int64, device=dev)
        new_len = torch.tensor([new_size], dtype=torch.int32, device=dev)
        ptrs = (C.c_void_p * 4)(*[p.data_ptr() for p in planes])
        rbs = (C.c_int64 * 4)(*[(p[0].numel() if p.dim() > 1 else 1) * p.element_size() for p in planes])
        N.call("pikv_compact_rows", ptrs, rbs, 4, row_base.data_ptr(), kidx.data_ptr(),
               new_len.data_ptr(), None, 1, torch.cuda.current_stream().cuda_stream)
        return (planes[0][:new_size], planes[1][:new_size], planes[2][:new_size],
                planes[3][:new_size], new_size)
