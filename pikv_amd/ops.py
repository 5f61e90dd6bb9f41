"""Tensor-level operators over the C ABI of libpikv_hip.so.

Every function validates device / dtype / contiguity / shape in Python, raises
ValueError on a bad argument, allocates the outputs with torch (device memory
and streams are the only things torch is used for here) and enqueues the HIP
kernels on torch's current stream.  There is no CPU path: a CPU tensor is an
error, and a missing library raises PiKVNativeError.

The operator set follows the reference's PiKVKernels facade
(core/single/pikv_kernels.py: top_k_routing :54-99, compress_kv :101-287,
evict_cache :289-422) and the module functions it would have served:
router tail (core/single/pikv_routing.py:65-82), quantise formula
(core/single/module/pikv_compression.py:945-1012), manager append / evict /
compact (core/single/cache_scheduling.py:391-436), H2O bookkeeping (:69-99).
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional, Sequence

import torch

from . import _native as N
from ._native import (BF16, EVICT_H2O, EVICT_LRU, F32, Q_I4_ASYM, Q_I4_SYM,
                      Q_I8_ASYM, Q_I8_SYM, SCORE_TILE)

__all__ = [
    "router_fused", "router_tail", "capacity_slots", "quantize_rows", "quant8_minshift",
    "dequantize_rows", "fakequant_colblocks", "fakequant_preset", "CachePool", "scheme_bits",
    "Q_I8_SYM", "Q_I8_ASYM", "Q_I4_ASYM", "Q_I4_SYM", "EVICT_H2O", "EVICT_LRU",
]


# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------

def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dt(t: torch.Tensor, name: str) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise ValueError(f"{name}: dtype must be float32 or bfloat16, got {t.dtype}")


def _need(t, name, *, dtype=None, ndim=None, optional=False):
    if t is None:
        if optional:
            return None
        raise ValueError(f"{name} is required")
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name}: dtype must be {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name}: expected {ndim} dimensions, got {tuple(t.shape)}")
    return t


def _vecf(t, name, n, device):
    """Optional float32 [n] vector on `device`."""
    if t is None:
        return None
    t = torch.as_tensor(t, dtype=torch.float32, device=device).contiguous()
    if t.numel() != n:
        raise ValueError(f"{name} must have {n} elements, got {t.numel()}")
    return t


def scheme_bits(scheme: int) -> int:
    return 8 if scheme in (Q_I8_SYM, Q_I8_ASYM) else 4


def _scheme_asym(scheme: int) -> bool:
    return scheme in (Q_I8_ASYM, Q_I4_ASYM)


def _check_scheme(scheme, D, group):
    if scheme not in (Q_I8_SYM, Q_I8_ASYM, Q_I4_ASYM, Q_I4_SYM):
        raise ValueError(f"unknown quantisation scheme {scheme}")
    epl = 16 if scheme_bits(scheme) == 8 else 32
    if D <= 0 or group <= 0 or D % group:
        raise ValueError(f"group {group} must divide the row width {D}")
    if group & (group - 1) or group < epl or group > 64 * epl:
        raise ValueError(
            f"group must be a power of two in [{epl}, {64 * epl}] for {scheme_bits(scheme)}-bit codes, got {group}")


def _meta_dtype(scheme):
    return torch.float32 if scheme_bits(scheme) == 8 else torch.float16


def _code_plane(rows, D, scheme, device):
    if scheme_bits(scheme) == 8:
        dt = torch.int8 if scheme == Q_I8_SYM else torch.uint8
        return torch.zeros(rows, D, dtype=dt, device=device)
    return torch.zeros(rows, D // 2, dtype=torch.uint8, device=device)


# --------------------------------------------------------------------------
# K1 router
# --------------------------------------------------------------------------

class RouterOut:
    """Compact routing result.  probs [T,E] f32, topk_idx [T,k] i32,
    topk_w [T,k] f32, slot [T,k] i32 (-1 = dropped by capacity) or None,
    count [E] i32 or None, logits [T,E] f32 or None."""
    __slots__ = ("probs", "topk_idx", "topk_w", "slot", "count", "logits", "capacity")

    def __init__(self, probs, topk_idx, topk_w, slot, count, logits, capacity):
        self.probs, self.topk_idx, self.topk_w = probs, topk_idx, topk_w
        self.slot, self.count, self.logits, self.capacity = slot, count, logits, capacity

    @property
    def keep(self):
        return None if self.slot is None else self.slot >= 0


def _router_common(T, E, k, capacity, device, want_probs=True, want_logits=False):
    if not (1 <= E <= 64):
        raise ValueError(f"num_experts must be in [1,64], got {E}")
    if not (1 <= k <= min(E, 8)):
        raise ValueError(f"top_k must be in [1,min(E,8)], got {k}")
    probs = torch.empty(T, E, dtype=torch.float32, device=device) if want_probs else None
    logits = torch.empty(T, E, dtype=torch.float32, device=device) if want_logits else None
    idx = torch.empty(T, k, dtype=torch.int32, device=device)
    w = torch.empty(T, k, dtype=torch.float32, device=device)
    slot = count = ws = None
    ws_bytes = 0
    if capacity is not None:
        if capacity < 0:
            raise ValueError("capacity must be >= 0")
        slot = torch.empty(T, k, dtype=torch.int32, device=device)
        count = torch.empty(E, dtype=torch.int32, device=device)
        ws_bytes = int(N.lib().pikv_router_workspace_bytes(T, E, k))
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=device)
    return probs, logits, idx, w, slot, count, ws, ws_bytes


ROUTER_SINGLE, ROUTER_MODULE = 0, 1


def _arith(module_arithmetic: bool) -> int:
    return ROUTER_MODULE if module_arithmetic else ROUTER_SINGLE


def router_fused(x, weight, bias=None, *, top_k=2, capacity=None, expert_scale=None,
                 expert_mask=None, temperature=1.0, renorm_eps=0.0,
                 return_logits=False, module_arithmetic=False) -> RouterOut:
    """Gate projection + softmax + top-k + renormalise (+ capacity slots).
    x [T,H] f32|bf16, weight [E,H] same dtype (nn.Linear layout).
    module_arithmetic=True: the operation order and mask penalty of the reference's
    module/ copy (* expert_scale before / temperature, finfo.min instead of -1e9;
    core/single/module/pikv_routing.py:596-600, :133-134)."""
    x = _need(x, "x", ndim=2)
    weight = _need(weight, "weight", ndim=2)
    if x.dtype != weight.dtype:
        raise ValueError(f"x and weight must share a dtype ({x.dtype} vs {weight.dtype})")
    dt = _dt(x, "x")
    T, H = x.shape
    E = weight.shape[0]
    if weight.shape[1] != H:
        raise ValueError(f"weight must be [E,{H}], got {tuple(weight.shape)}")
    if H % 8:
        raise ValueError(f"hidden size must be a multiple of 8, got {H}")
    dev = x.device
    bias = _vecf(bias, "bias", E, dev)
    expert_scale = _vecf(expert_scale, "expert_scale", E, dev)
    expert_mask = _vecf(expert_mask, "expert_mask", E, dev)
    probs, logits, idx, w, slot, count, ws, ws_bytes = _router_common(
        T, E, top_k, capacity, dev, True, return_logits)
    ws_bytes = int(N.lib().pikv_router_fused_workspace_bytes(T, H, E, top_k))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    if T == 0:  # nothing to route (empty tensors have no device address)
        if count is not None:
            count.zero_()
        return RouterOut(probs, idx, w, slot, count, logits, capacity)
    N.call("pikv_router_fused", _ptr(x), _ptr(weight), dt, _ptr(bias), _ptr(expert_scale),
           _ptr(expert_mask), float(temperature), float(renorm_eps), _arith(module_arithmetic),
           T, H, E, top_k,
           int(capacity or 0), _ptr(probs), _ptr(logits), _ptr(idx), _ptr(w), _ptr(slot),
           _ptr(count), _ptr(ws), ws_bytes, _stream())
    return RouterOut(probs, idx, w, slot, count, logits, capacity)


def router_tail(logits, *, top_k=2, capacity=None, logits_b=None, select=None,
                expert_scale=None, expert_mask=None, temperature=1.0, renorm_eps=0.0,
                use_softmax=True, module_arithmetic=False) -> RouterOut:
    """Router tail on precomputed float32 logits [T,E]."""
    logits = _need(logits, "logits", dtype=torch.float32, ndim=2)
    T, E = logits.shape
    dev = logits.device
    if (logits_b is None) != (select is None):
        raise ValueError("logits_b and select must be given together")
    if logits_b is not None:
        logits_b = _need(logits_b, "logits_b", dtype=torch.float32, ndim=2)
        if logits_b.shape != logits.shape:
            raise ValueError("logits_b must match logits")
        select = _need(select.reshape(-1).to(torch.uint8).contiguous(), "select")
        if select.numel() != T:
            raise ValueError(f"select must have {T} elements")
    expert_scale = _vecf(expert_scale, "expert_scale", E, dev)
    expert_mask = _vecf(expert_mask, "expert_mask", E, dev)
    probs, _, idx, w, slot, count, ws, ws_bytes = _router_common(
        T, E, top_k, capacity, dev, bool(use_softmax), False)
    if T == 0:
        if count is not None:
            count.zero_()
        return RouterOut(probs, idx, w, slot, count, None, capacity)
    N.call("pikv_router_tail", _ptr(logits), _ptr(logits_b), _ptr(select), _ptr(expert_scale),
           _ptr(expert_mask), float(temperature), float(renorm_eps), int(bool(use_softmax)),
           _arith(module_arithmetic), T, E, top_k, int(capacity or 0), _ptr(probs), _ptr(idx), _ptr(w), _ptr(slot),
           _ptr(count), _ptr(ws), ws_bytes, _stream())
    return RouterOut(probs, idx, w, slot, count, None, capacity)


def capacity_slots(expert_idx, num_experts: int, capacity: int):
    """slot / count for expert indices in token-major order."""
    expert_idx = _need(expert_idx, "expert_idx", dtype=torch.int32)
    if not (1 <= num_experts <= 64):
        raise ValueError("num_experts must be in [1,64]")
    if capacity < 0:
        raise ValueError("capacity must be >= 0")
    A = expert_idx.numel()
    dev = expert_idx.device
    slot = torch.empty_like(expert_idx)
    count = torch.empty(num_experts, dtype=torch.int32, device=dev)
    ws_bytes = int(N.lib().pikv_router_workspace_bytes(A, num_experts, 1))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    if A == 0:
        return slot, count.zero_()
    N.call("pikv_capacity_slots", _ptr(expert_idx), A, num_experts, int(capacity), _ptr(slot),
           _ptr(count), _ptr(ws), ws_bytes, _stream())
    return slot, count


# --------------------------------------------------------------------------
# K2 / K3 on plain rows
# --------------------------------------------------------------------------

def quantize_rows(x, group: int, scheme: int):
    """Quantise x [n,D] per `group` contiguous elements.  Returns
    (codes, scale, zero|None); 4-bit codes are packed two per byte."""
    x = _need(x, "x", ndim=2)
    dt = _dt(x, "x")
    n, D = x.shape
    _check_scheme(scheme, D, group)
    dev = x.device
    codes = _code_plane(n, D, scheme, dev)
    scale = torch.empty(n, D // group, dtype=_meta_dtype(scheme), device=dev)
    zero = torch.empty_like(scale) if _scheme_asym(scheme) else None
    if n == 0:
        return codes, scale, zero
    N.call("pikv_quantize_rows", _ptr(x), dt, n, D, group, scheme, 0, _ptr(codes), _ptr(scale),
           _ptr(zero), _stream())
    return codes, scale, zero


def quant8_minshift(x, want_dq: bool = True):
    """Min-shift 8-bit quantisation of whole rows (core/single/pikv_kernels.py:215-232).
    x [n, D] float32 or bfloat16.  Returns (dq float32 [n,D] or None, codes uint8 [n,D],
    scale [n,1], row_min [n,1])."""
    x = _need(x, "x", ndim=2)
    dt = _dt(x, "x")
    n, D = x.shape
    if D < 1:
        raise ValueError("rows must not be empty")
    dev = x.device
    codes = torch.empty(n, D, dtype=torch.uint8, device=dev)
    dq = torch.empty(n, D, dtype=torch.float32, device=dev) if want_dq else None
    scale = torch.empty(n, 1, dtype=torch.float32, device=dev)
    mn = torch.empty(n, 1, dtype=torch.float32, device=dev)
    if n:
        N.call("pikv_quant8_minshift", _ptr(x), dt, n, D, _ptr(codes), _ptr(dq), _ptr(scale), _ptr(mn), _stream())
    return dq, codes, scale, mn


def dequantize_rows(codes, scale, zero, group: int, scheme: int, out_dtype=torch.float32,
                    rows: Optional[torch.Tensor] = None, row0: int = 0, n: Optional[int] = None):
    """(q - zero) * scale for rows `rows` (int64 indices) or [row0, row0+n)."""
    codes = _need(codes, "codes", ndim=2)
    scale = _need(scale, "scale", ndim=2)
    bits = scheme_bits(scheme)
    D = codes.shape[1] * (1 if bits == 8 else 2)
    _check_scheme(scheme, D, group)
    if _scheme_asym(scheme):
        zero = _need(zero, "zero", ndim=2)
    if scale.dtype != _meta_dtype(scheme) or scale.shape != (codes.shape[0], D // group):
        raise ValueError("scale plane has the wrong dtype or shape")
    total = codes.shape[0]
    if rows is not None:
        rows = _need(rows, "rows", dtype=torch.int64, ndim=1)
        cnt = rows.numel()
    else:
        cnt = total - row0 if n is None else n
        if row0 < 0 or cnt < 0 or row0 + cnt > total:
            raise ValueError("row range outside the plane")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("out_dtype must be float32 or bfloat16")
    out = torch.empty(cnt, D, dtype=out_dtype, device=codes.device)
    if cnt == 0:
        return out
    N.call("pikv_gather_dequant", _ptr(codes), _ptr(scale), _ptr(zero), D, group, scheme,
           _ptr(rows), row0, cnt, _ptr(out), F32 if out_dtype == torch.float32 else BF16,
           _stream())
    return out


def fakequant_colblocks(x, group: int, bits: int = 8, symmetric: bool = False):
    """Reference-domain fake quantisation (min/max over all rows x `group`
    columns).  x [N,H] f32 -> (dq [N,H] f32, stats [nblk,4], mse [nblk])."""
    x = _need(x, "x", dtype=torch.float32, ndim=2)
    Nr, H = x.shape
    if group < 1:
        raise ValueError("group must be >= 1")
    nblk = (H + group - 1) // group
    dev = x.device
    out = torch.empty_like(x)
    stats = torch.zeros(nblk, 4, dtype=torch.float32, device=dev)
    mse = torch.zeros(nblk, dtype=torch.float32, device=dev)
    ws_bytes = int(N.lib().pikv_fakequant_workspace_bytes(Nr, H, group))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    N.call("pikv_fakequant_colblocks", _ptr(x), Nr, H, group, bits, int(bool(symmetric)),
           _ptr(out), _ptr(stats), _ptr(mse), _ptr(ws), ws_bytes, _stream())
    return out, stats, mse


def fakequant_preset(x, preset, group: int, bits: int = 8, symmetric: bool = False):
    """Fake quantisation with parameters fixed beforehand: `preset` is a (min, max, scale,
    zero) row of a fakequant_colblocks `stats` output; one (scale, zero) serves every
    element.  x [N,H] f32 -> (dq [N,H] f32, mse [nblk] per block of `group` columns)."""
    x = _need(x, "x", dtype=torch.float32, ndim=2)
    preset = _need(preset, "preset", dtype=torch.float32)
    if preset.numel() != 4:
        raise ValueError("preset must hold (min, max, scale, zero)")
    Nr, H = x.shape
    if group < 1:
        raise ValueError("group must be >= 1")
    nblk = (H + group - 1) // group
    dev = x.device
    out = torch.empty_like(x)
    mse = torch.zeros(nblk, dtype=torch.float32, device=dev)
    ws_bytes = int(N.lib().pikv_fakequant_workspace_bytes(Nr, H, group))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    N.call("pikv_fakequant_preset", _ptr(x), Nr, H, group, bits, int(bool(symmetric)),
           _ptr(preset), _ptr(out), _ptr(mse), _ptr(ws), ws_bytes, _stream())
    return out, mse


# --------------------------------------------------------------------------
# cache pool
# --------------------------------------------------------------------------

def _evict_workspace(n_caches: int, max_len: int, device):
    nbytes = int(N.lib().pikv_evict_workspace_bytes(n_caches, max_len))
    return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device), nbytes


def select_top_rows(score, seg_base, seg_len, n_keep, max_len: Optional[int] = None):
    """Per segment c of a flat score array (rows seg_base[c] .. +seg_len[c]): keep
    the n_keep[c] largest scores, ties to the lower index.  Returns (keep_flag
    uint8 [rows], keep_index int32 [rows], n_kept int32 [segments]); segment c's
    ascending survivor list sits at keep_index[seg_base[c] : +n_kept[c]]."""
    score = _need(score, "score", dtype=torch.float32, ndim=1)
    seg_base = _need(seg_base, "seg_base", dtype=torch.int64, ndim=1)
    seg_len = _need(seg_len, "seg_len", dtype=torch.int32, ndim=1)
    n_keep = _need(n_keep, "n_keep", dtype=torch.int32, ndim=1)
    n = seg_base.numel()
    if seg_len.numel() != n or n_keep.numel() != n:
        raise ValueError("seg_base, seg_len and n_keep must have the same length")
    dev = score.device
    flag = torch.zeros(score.numel(), dtype=torch.uint8, device=dev)
    index = torch.zeros(score.numel(), dtype=torch.int32, device=dev)
    kept = torch.zeros(n, dtype=torch.int32, device=dev)
    if n == 0 or score.numel() == 0:
        return flag, index, kept
    zero = torch.zeros(n, dtype=torch.int32, device=dev)
    if max_len is None:   # an upper bound of every segment length that needs no device read
        max_len = score.numel()
    ws, ws_bytes = _evict_workspace(n, int(max_len), dev)
    # H2O selection with an empty "recent" budget; the score doubles as the (unused) timestamp
    N.call("pikv_evict_select", EVICT_H2O, _ptr(score), _ptr(score), _ptr(seg_base), _ptr(seg_len),
           _ptr(n_keep), _ptr(zero), n, int(max_len), _ptr(flag), _ptr(index), _ptr(kept), _ptr(ws),
           ws_bytes, _stream())
    return flag, index, kept


class CachePool:
    """n_caches quantised KV caches (one per expert or per sequence) sharing a
    row space in HBM; see include/pikv_hip.h for the plane layout.  State
    (planes, fill) lives on the GPU; no method reads it back to the host."""

    def __init__(self, caps: Sequence[int], n_heads: int, head_dim: int, group: int,
                 scheme: int, device, with_v: bool = True):
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise ValueError("CachePool needs a GPU device; there is no CPU path")
        self.n_heads, self.head_dim = int(n_heads), int(head_dim)
        self.D = self.n_heads * self.head_dim
        self.group, self.scheme, self.with_v = int(group), int(scheme), bool(with_v)
        _check_scheme(scheme, self.D, group)
        caps = [int(c) for c in caps]
        if not caps or min(caps) < 0:
            raise ValueError("caps must be a non-empty list of non-negative sizes")
        self.n_caches = len(caps)
        self.max_cap = max(caps)
        base, run = [], 0
        for c in caps:
            base.append(run)
            run += c
        self.rows = run
        self.caps_host, self.base_host = caps, base     # the geometry, for host-side slicing
        dev = self.device
        self.cap = torch.tensor(caps, dtype=torch.int32, device=dev)
        self.row_base = torch.tensor(base, dtype=torch.int64, device=dev)
        self.fill = torch.zeros(self.n_caches, dtype=torch.int32, device=dev)
        ng = self.D // group
        md = _meta_dtype(scheme)
        asym = _scheme_asym(scheme)
        self.k_codes = _code_plane(self.rows, self.D, scheme, dev)
        self.k_scale = torch.zeros(self.rows, ng, dtype=md, device=dev)
        self.k_zero = torch.zeros(self.rows, ng, dtype=md, device=dev) if asym else None
        self.v_codes = self.v_scale = self.v_zero = None
        if with_v:
            self.v_codes = _code_plane(self.rows, self.D, scheme, dev)
            self.v_scale = torch.zeros(self.rows, ng, dtype=md, device=dev)
            self.v_zero = torch.zeros(self.rows, ng, dtype=md, device=dev) if asym else None
        self.acc = torch.zeros(self.rows, dtype=torch.float32, device=dev)
        self.ts = torch.zeros(self.rows, dtype=torch.float32, device=dev)
        # eviction scratch
        self.keep_flag = torch.zeros(self.rows, dtype=torch.uint8, device=dev)
        self.keep_index = torch.zeros(self.rows, dtype=torch.int32, device=dev)
        self.new_len = torch.zeros(self.n_caches, dtype=torch.int32, device=dev)
        self.n_heavy = torch.zeros(self.n_caches, dtype=torch.int32, device=dev)
        self.n_recent = torch.zeros(self.n_caches, dtype=torch.int32, device=dev)

    # ---- checkpoint ----
    _STATE_PLANES = ("k_codes", "k_scale", "k_zero", "v_codes", "v_scale", "v_zero", "acc", "ts")

    def state_dict(self, trim: bool = True):
        """Everything needed to restore the caches: geometry, fill counts and the
        quantised planes (codes, scales, zero points, accumulators, timestamps) as
        CPU tensors.  With trim=True only the valid rows of every cache are kept
        (rows [row_base[c], row_base[c]+fill[c]), concatenated in cache order)."""
        fill = self.fill.cpu()
        sd = {"layout": torch.tensor([self.n_heads, self.head_dim, self.group, self.scheme,
                                      int(self.with_v), int(trim)], dtype=torch.int64),
              "cap": self.cap.cpu(), "fill": fill}
        rows = None
        if trim:
            base = self.row_base.cpu()
            rows = torch.cat([torch.arange(int(base[c]), int(base[c]) + int(fill[c]))
                              for c in range(self.n_caches)]) if self.n_caches else torch.zeros(0, dtype=torch.int64)
            rows = rows.to(self.device)
        for name in self._STATE_PLANES:
            t = getattr(self, name)
            if t is not None:
                sd[name] = (t.index_select(0, rows) if rows is not None else t).cpu()
        return sd

    def load_state_dict(self, sd):
        """Restore what state_dict() saved into a pool of the same geometry."""
        layout = [int(v) for v in sd["layout"]]
        mine = [self.n_heads, self.head_dim, self.group, self.scheme, int(self.with_v)]
        if layout[:5] != mine:
            raise ValueError(f"checkpoint layout {layout[:5]} does not match this pool {mine}")
        if not torch.equal(sd["cap"].to(torch.int32).cpu(), self.cap.cpu()):
            raise ValueError("checkpoint cache capacities do not match this pool")
        fill = sd["fill"].to(torch.int32)
        if bool((fill > self.cap.cpu()).any()) or bool((fill < 0).any()):
            raise ValueError("checkpoint fill counts exceed the capacities")
        trim = bool(layout[5])
        rows = None
        if trim:
            base = self.row_base.cpu()
            rows = torch.cat([torch.arange(int(base[c]), int(base[c]) + int(fill[c]))
                              for c in range(self.n_caches)]).to(self.device)
        for name in self._STATE_PLANES:
            t = getattr(self, name)
            if t is None:
                continue
            src = sd[name].to(self.device)
            if src.dtype != t.dtype or src.shape[1:] != t.shape[1:]:
                raise ValueError(f"checkpoint plane {name} has the wrong dtype or row shape")
            if rows is not None:
                if src.shape[0] != rows.numel():
                    raise ValueError(f"checkpoint plane {name} does not hold the saved rows")
                t.index_copy_(0, rows, src)
            else:
                if src.shape != t.shape:
                    raise ValueError(f"checkpoint plane {name} has the wrong number of rows")
                t.copy_(src)
        self.fill.copy_(fill.to(self.device))

    # ---- write path ----
    def quant_scatter(self, k_src, v_src, cache_id, slot, fanout: int, now: float = 0.0):
        """Quantise source rows once and append them to their routed caches.
        k_src/v_src [n_src, D] (or [n_src, heads, head_dim]); cache_id/slot
        int32 [n_src*fanout] (any shape).  fill is not advanced."""
        k_src = _need(k_src, "k_src")
        dt = _dt(k_src, "k_src")
        k2 = k_src.reshape(-1, self.D)
        n_src = k2.shape[0]
        v2 = None
        if self.with_v:
            v_src = _need(v_src, "v_src", dtype=k_src.dtype)
            v2 = v_src.reshape(-1, self.D)
            if v2.shape != k2.shape:
                raise ValueError("v_src must match k_src")
        cache_id = _need(cache_id, "cache_id", dtype=torch.int32)
        slot = _need(slot, "slot", dtype=torch.int32)
        if not (1 <= fanout <= 8):
            raise ValueError("fanout must be in [1,8]")
        if cache_id.numel() != n_src * fanout or slot.numel() != n_src * fanout:
            raise ValueError(f"cache_id/slot must have n_src*fanout = {n_src * fanout} elements")
        if n_src == 0:
            return
        N.call("pikv_quant_scatter", _ptr(k2), _ptr(v2), dt, n_src, fanout, self.D, self.group,
               self.scheme, _ptr(cache_id), _ptr(slot), _ptr(self.row_base), _ptr(self.fill),
               _ptr(self.cap), self.n_caches, _ptr(self.k_codes), _ptr(self.v_codes),
               _ptr(self.k_scale), _ptr(self.v_scale), _ptr(self.k_zero), _ptr(self.v_zero),
               _ptr(self.acc), _ptr(self.ts), float(now), _stream())

    def quant_gather(self, k_src, v_src, src_row_base, src_index, n_take, max_take: int,
                     src_score=None, now: float = 0.0):
        """Quantise the listed source rows into the caches in list order: for
        cache c and j < n_take[c], source row src_row_base[c] +
        src_index[src_row_base[c] + j] goes to cache row fill[c] + j.  fill is
        not advanced."""
        k_src = _need(k_src, "k_src")
        dt = _dt(k_src, "k_src")
        k2 = k_src.reshape(-1, self.D)
        v2 = None
        if self.with_v:
            v_src = _need(v_src, "v_src", dtype=k_src.dtype)
            v2 = v_src.reshape(-1, self.D)
            if v2.shape != k2.shape:
                raise ValueError("v_src must match k_src")
        src_row_base = _need(src_row_base, "src_row_base", dtype=torch.int64, ndim=1)
        src_index = _need(src_index, "src_index", dtype=torch.int32, ndim=1)
        n_take = _need(n_take, "n_take", dtype=torch.int32, ndim=1)
        if src_row_base.numel() != self.n_caches or n_take.numel() != self.n_caches:
            raise ValueError("src_row_base / n_take must have one entry per cache")
        if src_index.numel() < k2.shape[0]:
            raise ValueError("src_index must cover the source row space")
        if src_score is not None:
            src_score = _need(src_score, "src_score", dtype=torch.float32)
            if src_score.numel() != k2.shape[0]:
                raise ValueError("src_score must have one entry per source row")
        if max_take <= 0 or k2.shape[0] == 0:
            return
        N.call("pikv_quant_gather", _ptr(k2), _ptr(v2), dt, self.D, self.group, self.scheme,
               _ptr(src_row_base), _ptr(src_index), _ptr(n_take), int(max_take), _ptr(src_score),
               _ptr(self.row_base), _ptr(self.fill), _ptr(self.cap), self.n_caches,
               _ptr(self.k_codes), _ptr(self.v_codes), _ptr(self.k_scale), _ptr(self.v_scale),
               _ptr(self.k_zero), _ptr(self.v_zero), _ptr(self.acc), _ptr(self.ts), float(now),
               _stream())

    def advance(self, count, per_call_limit: int = -1):
        """fill[c] = min(fill[c] + min(count[c], limit), cap[c])."""
        count = _need(count, "count", dtype=torch.int32, ndim=1)
        if count.numel() != self.n_caches:
            raise ValueError("count must have one entry per cache")
        N.call("pikv_cache_advance", _ptr(self.fill), _ptr(count), _ptr(self.cap), self.n_caches,
               int(per_call_limit), _stream())

    # ---- read path ----
    def _planes(self, which):
        if which == "k":
            return self.k_codes, self.k_scale, self.k_zero
        if which == "v" and self.with_v:
            return self.v_codes, self.v_scale, self.v_zero
        raise ValueError("which must be 'k' or 'v' (and the pool must hold V)")

    def gather_dequant(self, which="k", rows=None, row0=0, n=None, out_dtype=torch.float32):
        codes, scale, zero = self._planes(which)
        return dequantize_rows(codes, scale, zero, self.group, self.scheme, out_dtype,
                               rows=rows, row0=row0, n=n)

    def scores(self, q, n_q_heads: int, scale_qk: Optional[float] = None,
               max_len: Optional[int] = None):
        """scores[c,h,n] = q[c,h,:] . dequant(K[c,n,h//rep,:]) * scale_qk for
        n < fill[c].  q [n_caches, n_q_heads, head_dim] f32|bf16.  Returns
        (scores [n_caches,n_q_heads,stride] f32, tile_max, tile_sum)."""
        q = _need(q, "q", ndim=3)
        qdt = _dt(q, "q")
        if q.shape != (self.n_caches, n_q_heads, self.head_dim):
            raise ValueError(f"q must be [{self.n_caches},{n_q_heads},{self.head_dim}]")
        if n_q_heads % self.n_heads:
            raise ValueError("n_q_heads must be a multiple of the kv heads")
        max_len = self.max_cap if max_len is None else int(max_len)
        stride = max_len
        n_tiles = (max_len + SCORE_TILE - 1) // SCORE_TILE
        dev = self.device
        scores = torch.empty(self.n_caches, n_q_heads, stride, dtype=torch.float32, device=dev)
        tmax = torch.empty(self.n_caches, max(n_tiles, 1), n_q_heads, dtype=torch.float32, device=dev)
        tsum = torch.empty_like(tmax)
        if scale_qk is None:
            scale_qk = 1.0 / (self.head_dim ** 0.5)
        N.call("pikv_gather_dequant_scores", _ptr(self.k_codes), _ptr(self.k_scale),
               _ptr(self.k_zero), self.scheme, self.group, self.n_heads, n_q_heads, self.head_dim,
               _ptr(q), qdt, float(scale_qk), _ptr(self.row_base), _ptr(self.fill), self.n_caches,
               max_len, stride, _ptr(scores), _ptr(tmax), _ptr(tsum), _stream())
        return scores, tmax, tsum

    def h2o_accumulate(self, scores, tile_max, tile_sum, now: float, decay: float = 1.0,
                       write_probs: bool = False, return_importance: bool = False,
                       stats_only: bool = False):
        """Normalise, sum over heads, acc += importance, ts = now.  stats_only=True
        leaves acc and ts alone and only fills self.head_stats (for an attend_values
        call that accumulates itself)."""
        scores = _need(scores, "scores", dtype=torch.float32, ndim=3)
        tile_max = _need(tile_max, "tile_max", dtype=torch.float32, ndim=3)
        tile_sum = _need(tile_sum, "tile_sum", dtype=torch.float32, ndim=3)
        nc, hq, stride = scores.shape
        if nc != self.n_caches:
            raise ValueError("scores must have one slab per cache")
        n_tiles = (stride + SCORE_TILE - 1) // SCORE_TILE
        if tile_max.shape != (nc, max(n_tiles, 1), hq) or tile_sum.shape != tile_max.shape:
            raise ValueError("tile statistics do not match scores")
        dev = self.device
        imp = torch.zeros(nc, stride, dtype=torch.float32, device=dev) if return_importance else None
        head_stats = torch.empty(nc, hq, 2, dtype=torch.float32, device=dev)
        N.call("pikv_h2o_accumulate", _ptr(scores), _ptr(tile_max), _ptr(tile_sum), hq,
               _ptr(self.row_base), _ptr(self.fill), nc, stride, stride, float(decay), float(now),
               int(bool(write_probs)), None if stats_only else _ptr(self.acc),
               None if stats_only else _ptr(self.ts), _ptr(imp), _ptr(head_stats), _stream())
        self.head_stats = head_stats   # (max, sum) per (cache, head): what attend_values normalises with
        return imp

    def attend_values(self, scores, head_stats=None, accumulate: bool = False, now: float = 0.0,
                      decay: float = 1.0):
        """out[c,h,:] = sum_n p[c,h,n] * dequant(V[c,n,h/rep,:]) over the valid rows.
        scores [n_caches, n_q_heads, stride] float32: raw scores together with
        head_stats [n_caches, n_q_heads, 2] (as left in self.head_stats by
        h2o_accumulate), or probabilities when head_stats is None.
        accumulate=True also does h2o_accumulate's bookkeeping (acc = acc*decay + sum of
        the probabilities over the heads, ts = now) in the same pass."""
        if not self.with_v:
            raise ValueError("this pool stores no V rows")
        scores = _need(scores, "scores", dtype=torch.float32, ndim=3)
        nc, hq, stride = scores.shape
        if nc != self.n_caches or hq % self.n_heads:
            raise ValueError("scores must be [n_caches, n_q_heads, stride] with n_q_heads a multiple of the kv heads")
        if head_stats is not None:
            head_stats = _need(head_stats, "head_stats", dtype=torch.float32, ndim=3)
            if head_stats.shape != (nc, hq, 2):
                raise ValueError("head_stats must be [n_caches, n_q_heads, 2]")
        dev = self.device
        out = torch.zeros(nc, hq, self.head_dim, dtype=torch.float32, device=dev)
        if stride == 0:
            return out
        ws_bytes = int(N.lib().pikv_attend_workspace_bytes(nc, hq, self.head_dim, stride))
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
        N.call("pikv_attend_values", _ptr(scores), _ptr(head_stats), stride, _ptr(self.v_codes),
               _ptr(self.v_scale), _ptr(self.v_zero), self.scheme, self.group, self.n_heads, hq,
               self.head_dim, _ptr(self.row_base), _ptr(self.fill), nc, stride, float(decay), float(now),
               _ptr(self.acc) if accumulate else None, _ptr(self.ts) if accumulate else None,
               _ptr(out), _ptr(ws), ws_bytes, _stream())
        return out

    def decode_attend(self, q, n_q_heads: int, now: float = 0.0, scale_qk: Optional[float] = None,
                      max_len: Optional[int] = None, accumulate: bool = True, decay: float = 1.0):
        """The whole decode read in one native call (pikv_decode_attend): scores of q
        [n_caches, n_q_heads, head_dim] against the compressed K rows, softmax over each cache's
        rows, attention output over the compressed V rows -> out [n_caches, n_q_heads, head_dim]
        float32; accumulate=True adds the probabilities to the H2O accumulators (acc = acc*decay +
        sum over the heads, ts = now).  The score matrix stays inside the library's workspace."""
        if not self.with_v:
            raise ValueError("this pool stores no V rows")
        q = _need(q, "q", ndim=3)
        dt = _dt(q, "q")
        if q.shape != (self.n_caches, n_q_heads, self.head_dim):
            raise ValueError(f"q must be [{self.n_caches},{n_q_heads},{self.head_dim}], got {tuple(q.shape)}")
        if n_q_heads % self.n_heads:
            raise ValueError("n_q_heads must be a multiple of the kv heads")
        if scale_qk is None:
            scale_qk = 1.0 / math.sqrt(self.head_dim)
        max_len = self.max_cap if max_len is None else int(max_len)
        dev = self.device
        out = torch.empty(self.n_caches, n_q_heads, self.head_dim, dtype=torch.float32, device=dev)
        key = (n_q_heads, max_len)
        if getattr(self, "_decode_ws_key", None) != key:
            nb = int(N.lib().pikv_decode_attend_workspace_bytes(self.n_caches, n_q_heads, self.head_dim, max_len))
            self._decode_ws = torch.empty(max(nb, 256), dtype=torch.uint8, device=dev)
            self._decode_ws_key = key
        ws = self._decode_ws
        N.call("pikv_decode_attend", _ptr(self.k_codes), _ptr(self.k_scale), _ptr(self.k_zero),
               _ptr(self.v_codes), _ptr(self.v_scale), _ptr(self.v_zero), self.scheme, self.group,
               self.n_heads, n_q_heads, self.head_dim, _ptr(q), dt, float(scale_qk), _ptr(self.row_base),
               _ptr(self.fill), self.n_caches, max_len, float(decay), float(now),
               _ptr(self.acc) if accumulate else None, _ptr(self.ts) if accumulate else None,
               _ptr(out), _ptr(ws), ws.numel(), _stream())
        return out

    # ---- eviction ----
    def evict_select(self, policy: int, *, heavy_ratio=0.1, recent_ratio=0.1,
                     n_heavy=None, n_recent=None, n_evict=None, multi_block: bool = True):
        """Fill keep_flag / keep_index / new_len.  H2O: budgets from the
        ratios (per cache, from its current fill) or explicit int32 tensors;
        LRU: n_evict int32 [n_caches].  multi_block=False withholds the workspace, so
        that one block selects each cache whatever its length (same result)."""
        if policy == EVICT_H2O:
            if n_heavy is None:
                N.call("pikv_h2o_budget", _ptr(self.fill), self.n_caches, float(heavy_ratio),
                       float(recent_ratio), _ptr(self.n_heavy), _ptr(self.n_recent), _stream())
                nh, nr = self.n_heavy, self.n_recent
            else:
                nh = _need(n_heavy, "n_heavy", dtype=torch.int32, ndim=1)
                nr = _need(n_recent, "n_recent", dtype=torch.int32, ndim=1)
        elif policy == EVICT_LRU:
            nh = _need(n_evict, "n_evict", dtype=torch.int32, ndim=1)
            nr = None
        else:
            raise ValueError(f"unknown eviction policy {policy}")
        if nh.numel() != self.n_caches or (nr is not None and nr.numel() != self.n_caches):
            raise ValueError("budgets must have one entry per cache")
        ws, ws_bytes = None, 0
        if multi_block:
            if getattr(self, "_evict_ws", None) is None:
                self._evict_ws = _evict_workspace(self.n_caches, self.max_cap, self.device)
            ws, ws_bytes = self._evict_ws
        N.call("pikv_evict_select", policy, _ptr(self.acc), _ptr(self.ts), _ptr(self.row_base),
               _ptr(self.fill), _ptr(nh), _ptr(nr), self.n_caches, self.max_cap, _ptr(self.keep_flag),
               _ptr(self.keep_index), _ptr(self.new_len), _ptr(ws), ws_bytes, _stream())

    def planes(self):
        ps = [self.k_codes, self.k_scale, self.k_zero, self.v_codes, self.v_scale, self.v_zero,
              self.acc, self.ts]
        return [p for p in ps if p is not None]

    def compact(self, extra_planes: Sequence[torch.Tensor] = ()):
        """Move survivors (keep_index/new_len) to the front of every plane and
        set fill = new_len."""
        ps = self.planes() + [_need(p, "extra plane") for p in extra_planes]
        if len(ps) > N.MAX_PLANES:
            raise ValueError(f"at most {N.MAX_PLANES} planes")
        ptrs = (C.c_void_p * len(ps))(*[p.data_ptr() for p in ps])
        rbs = (C.c_int64 * len(ps))(*[math.prod(p.shape[1:]) * p.element_size() for p in ps])
        N.call("pikv_compact_rows", ptrs, rbs, len(ps), _ptr(self.row_base), _ptr(self.keep_index),
               _ptr(self.new_len), _ptr(self.fill), self.n_caches, _stream())

    def evict(self, policy: int, **kw):
        self.evict_select(policy, **kw)
        self.compact()
