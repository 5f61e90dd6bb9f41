"""CPU restatement (numpy) of PiKV's routed, compressed KV-cache data path.

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP kernels are
compared against; nothing in the product package imports it.  Every function
restates, in plain numpy float32/integer arithmetic, what the reference's
PyTorch path computes, and cites the reference lines it follows
(paths relative to the reference repository root).

Where the reference leaves a result implementation-defined the rule used here
is stated in the docstring:
  * every top-k orders by (value, index) with the LOWER index first among
    equal values (torch.topk's tie order on CPU is unspecified);
  * expert top-k is taken on what the reference hands to torch.topk, the float32
    probabilities (core/single/pikv_routing.py:73-76): two distinct logits whose
    probabilities round to the same float32 tie, and the lower expert wins; rows
    whose probabilities are NaN (a NaN or +inf logit) select experts 0..k-1.
    Without the softmax (PiKVKernels.top_k_routing) the key is the logit.

Pinning status (what, besides this file, fixes each function's output):
  router_tail / capacity_slots ....... brute-force loops + invariants + the C
                                       restatement in pikv_oracle.c
  quant_params / quantize_groups ..... hand-derived known-answer vectors,
                                       error-bound and range invariants, C
                                       restatement
  scores / h2o ....................... float64 closed forms, C restatement
  select / compact ................... brute force on tiny inputs, invariants
  streaming / quest / flexgen / lru+ . hand-computed known answers, brute-force
                                       ranking on tiny inputs
  adakv / duo / attend_values ........ hand-computed known answers (attend_values: a
                                       2-kv-head, 4-query-head, 3-token case), float64
                                       closed forms
  quant8_minshift / pyramid_keep_counts / dense_dispatch_combine
                                       hand-computed known answers (tie rounding, a shifted
                                       and a constant row; interior budgets from the integer
                                       formula; a literal 2-token dispatch)
  scale_logits ....................... literals of a float32 case where (lg/T)*w and
                                       (lg*w)/T differ in the last bit (one per reference
                                       copy, re-derived with exact rationals), both mask
                                       penalties as literals
  fakequant_colblocks / _preset ...... hand-computed block scale / zero point / codes
                                       ([-1,0,1] -> 2/255, 127; extremes in different rows;
                                       two blocks; 4-bit; symmetric), identity with
                                       quantize_groups on one-row inputs for all four
                                       (bits, symmetric) pairs; the preset form given a
                                       block's own parameters must repeat the block form
                                       bit for bit
  all of the above ................... property tests (ranges, error bounds, total
                                       orders, conservation, monotone budgets) and the
                                       frozen digests of tests/golden
The reference's own tests hold no golden vectors for any of these.  Parity
unpinned: none of the functions here.  The end-to-end outputs of the reference's
PiKVMoE module graph are not restated in this file: they are held as a fixture written
by the reference's own module (tests/golden/make_ref_moe_golden.py ->
tests/golden/ref_moe_forward.npz).
"""
from __future__ import annotations

import math
import numpy as np

F32 = np.float32

# --------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------

def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bfloat16 (ties to even) and return
    them as float32.  Used to make synthetic bf16 inputs and to model bf16
    output rounding."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounding = ((u >> 16) & 1) + 0x7FFF
    r = ((u + rounding) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32)
    nan = np.isnan(x)
    if nan.any():
        out = out.copy()
        out[nan] = np.nan
    return out


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of bf16_round(x)."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


# --------------------------------------------------------------------------
# R1-R4  router
# --------------------------------------------------------------------------

def gate_logits(x: np.ndarray, w: np.ndarray, bias=None) -> np.ndarray:
    """logits[t,e] = sum_h x[t,h]*w[e,h] + b[e]; nn.Linear weight layout [E,H]
    (core/single/pikv_routing.py:34-38,65).  Accumulated in float64 and
    rounded once to float32: the best estimate of what any float32 summation
    order returns; compare with a tolerance."""
    acc = x.astype(np.float64) @ w.astype(np.float64).T
    if bias is not None:
        acc = acc + bias.astype(np.float64)
    return acc.astype(np.float32)


def scale_logits(logits, temperature=1.0, expert_scale=None, expert_mask=None,
                 logits_b=None, select=None, module_arithmetic=False) -> np.ndarray:
    """Logit post-processing in float32, in the order of
    core/single/pikv_routing.py:
      PiKV  (:450-460)  row-wise choice between two gates by the importance
                        mask, then * cache_correction_factor[e];
      EPLB  (:653-656)  / temperature, then * expert_weights[e];
      mask  (:68-70)    + (1 - mask[e]) * -1e9.
    module_arithmetic=True follows core/single/module/pikv_routing.py instead:
    * expert_weights before / temperature (:596-600), penalty finfo(float32).min (:133-134).
    """
    lg = np.asarray(logits, dtype=F32)
    if logits_b is not None and select is not None:
        sel = np.asarray(select).astype(bool)[:, None]
        lg = np.where(sel, lg, np.asarray(logits_b, dtype=F32))
    if module_arithmetic:
        if expert_scale is not None:
            lg = lg * np.asarray(expert_scale, dtype=F32)[None, :]
        if temperature != 1.0:
            lg = lg / F32(temperature)
        if expert_mask is not None:
            m = np.asarray(expert_mask, dtype=F32)[None, :]
            with np.errstate(over="ignore"):
                lg = (lg + (F32(1.0) - m) * np.finfo(F32).min).astype(F32)
        return lg.astype(F32)
    if temperature != 1.0:
        lg = lg / F32(temperature)
    if expert_scale is not None:
        lg = lg * np.asarray(expert_scale, dtype=F32)[None, :]
    if expert_mask is not None:
        m = np.asarray(expert_mask, dtype=F32)[None, :]
        lg = lg + (F32(1.0) - m) * F32(-1e9)
    return lg.astype(F32)


def softmax_rows(lg: np.ndarray) -> np.ndarray:
    """F.softmax(router_logits, dim=-1) in float32
    (core/single/pikv_routing.py:73): subtract the row max, exp, divide."""
    lg = np.asarray(lg, dtype=F32)
    m = lg.max(axis=-1, keepdims=True)
    e = np.exp((lg - m).astype(F32)).astype(F32)
    s = e.sum(axis=-1, keepdims=True, dtype=F32)
    return (e / s).astype(F32)


def topk_desc(v: np.ndarray, k: int) -> np.ndarray:
    """Indices of the k largest entries of each row, largest first, lower
    index first among equals (stable sort); NaN sorts after every number."""
    order = np.argsort(-v.astype(np.float64), axis=-1, kind="stable")
    return order[..., :k].astype(np.int32)


def topk_asc(v: np.ndarray, k: int) -> np.ndarray:
    """Indices of the k smallest entries, smallest first, lower index first
    among equals."""
    order = np.argsort(v.astype(np.float64), axis=-1, kind="stable")
    return order[..., :k].astype(np.int32)


def router_tail(logits, top_k, temperature=1.0, expert_scale=None,
                expert_mask=None, logits_b=None, select=None,
                renorm_eps=0.0, use_softmax=True, module_arithmetic=False):
    """softmax -> top-k -> renormalise (core/single/pikv_routing.py:73-79;
    the +1e-8 variant is core/single/module/pikv_routing.py:143).
    Returns (probs [T,E] f32, idx [T,k] i32, w [T,k] f32, final logits).
    With use_softmax=False this is PiKVKernels.top_k_routing's fallback,
    torch.topk on the raw logits (core/single/pikv_kernels.py:97): w holds
    the selected logits."""
    lg = scale_logits(logits, temperature, expert_scale, expert_mask,
                      logits_b, select, module_arithmetic)
    k = min(int(top_k), lg.shape[-1])
    if not use_softmax:
        idx = topk_desc(lg, k)
        vals = np.take_along_axis(lg, idx.astype(np.int64), axis=-1)
        return None, idx, vals.astype(F32), lg
    probs = softmax_rows(lg)
    idx = topk_desc(probs, k)
    vals = np.take_along_axis(probs, idx.astype(np.int64), axis=-1)
    s = np.zeros(vals.shape[:-1] + (1,), dtype=F32)
    for j in range(k):                       # left-to-right float32 sum
        s = (s + vals[..., j:j + 1]).astype(F32)
    w = (vals / (s + F32(renorm_eps))).astype(F32) if renorm_eps else (vals / s).astype(F32)
    return probs, idx, w, lg


# --------------------------------------------------------------------------
# R5  capacity and slots
# --------------------------------------------------------------------------

def compute_capacity(batch_size: int, seq_len: int, capacity_factor: float,
                     top_k: int, num_experts: int) -> int:
    """int(B*S*cf*k/E), evaluated left to right in Python floats
    (core/single/pikv_routing.py:40-42)."""
    return int(batch_size * seq_len * capacity_factor * top_k / num_experts)


def capacity_slots(expert_idx: np.ndarray, num_experts: int, capacity: int):
    """Token-major sequential fill of core/single/module/pikv_routing.py:93-104
    in compact form.  expert_idx [T,k] (or flat [A]).  Returns
    (slot int32, same shape, -1 where the expert was full; count [E] int32 of
    all assignments, kept or not)."""
    flat = np.asarray(expert_idx).reshape(-1).astype(np.int64)
    slot = np.full(flat.shape, -1, dtype=np.int32)
    count = np.zeros(num_experts, dtype=np.int32)
    for e in range(num_experts):
        pos = np.nonzero(flat == e)[0]
        count[e] = pos.size
        rank = np.arange(pos.size, dtype=np.int64)
        kept = rank < capacity
        slot[pos[kept]] = rank[kept].astype(np.int32)
    return slot.reshape(np.asarray(expert_idx).shape), count


def capacity_slots_loop(expert_idx, num_experts, capacity):
    """The same rule as a literal loop (small inputs only); pins
    capacity_slots."""
    flat = [int(v) for v in np.asarray(expert_idx).reshape(-1)]
    used = [0] * num_experts
    total = [0] * num_experts
    slot = []
    for e in flat:
        total[e] += 1
        if used[e] < capacity:
            slot.append(used[e])
            used[e] += 1
        else:
            slot.append(-1)
    return (np.array(slot, dtype=np.int32).reshape(np.asarray(expert_idx).shape),
            np.array(total, dtype=np.int32))


def dense_dispatch_combine(idx, w, slot, num_experts, capacity):
    """dispatch[t,e,slot]=1, combine[t,e,slot]=w for kept assignments
    (core/single/module/pikv_routing.py:77-104).  idx,w,slot: [T,k]."""
    T, k = idx.shape
    disp = np.zeros((T, num_experts, capacity), dtype=F32)
    comb = np.zeros((T, num_experts, capacity), dtype=F32)
    for t in range(T):
        for j in range(k):
            s = int(slot[t, j])
            if s >= 0:
                disp[t, idx[t, j], s] = 1.0
                comb[t, idx[t, j], s] = w[t, j]
    return disp, comb


# --------------------------------------------------------------------------
# R6/R10  quantisation
# --------------------------------------------------------------------------
Q_I8_SYM, Q_I8_ASYM, Q_I4_ASYM, Q_I4_SYM = 0, 1, 2, 3


def scheme_info(scheme: int):
    """(bits, symmetric, qmin, qmax) - core/single/module/pikv_compression.py:947-963."""
    return {Q_I8_SYM: (8, True, -128, 127), Q_I8_ASYM: (8, False, 0, 255),
            Q_I4_ASYM: (4, False, 0, 15), Q_I4_SYM: (4, True, -8, 7)}[scheme]


def _to_half_sat(v: np.ndarray) -> np.ndarray:
    """float32 -> float16 round-to-nearest-even, saturating finite values to
    +-65504 instead of overflowing to infinity."""
    with np.errstate(over="ignore"):
        h = v.astype(np.float16)
    big = np.isinf(h) & np.isfinite(v)
    if big.any():
        h = h.copy()
        h[big] = np.where(v[big] > 0, np.float16(65504.0), np.float16(-65504.0))
    return h


def quant_params(x_min: np.ndarray, x_max: np.ndarray, scheme: int):
    """scale and zero point of a reduction domain, float32 arithmetic in the
    reference's operation order (core/single/module/pikv_compression.py:966-979):
        if x_max == x_min: x_max = x_min + 1e-5
        sym : scale = 2*max(|x_min|,|x_max|)/(qmax-qmin); zero = 0
        asym: scale = (x_max-x_min)/(qmax-qmin); zero = qmin - round(x_min/scale)
    For the 4-bit schemes the stored metadata is float16: the scale is rounded
    to float16 first, and the zero point is computed from that rounded scale
    and itself rounded (saturating) to float16, so that the encoder and every
    decoder use the same two numbers.  4-bit asymmetric only: when |x_min| > 1024*scale
    the scale becomes float16(|x_min|/1024), which keeps the zero point an integer that
    float16 represents exactly (a build rule; the reference keeps float32 metadata)."""
    bits, sym, qmin, qmax = scheme_info(scheme)
    x_min = np.asarray(x_min, dtype=F32)
    x_max = np.asarray(x_max, dtype=F32)
    x_max = np.where(x_max == x_min, (x_min + F32(1e-5)).astype(F32), x_max)
    qr = F32(qmax - qmin)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        if sym:
            amax = np.maximum(np.abs(x_min), np.abs(x_max))
            scale = ((F32(2.0) * amax).astype(F32) / qr).astype(F32)
        else:
            scale = ((x_max - x_min).astype(F32) / qr).astype(F32)
        if bits == 4:
            # a scale that underflows to zero in float16 becomes 2**-24, the
            # smallest positive float16, so nothing divides by zero
            scale = _to_half_sat(scale).astype(F32)
            scale = np.where(scale == 0, F32(2.0 ** -24), scale).astype(F32)
            if not sym:
                # the zero point is float16 too and must stay an integer float16 holds
                # exactly (here |zero| <= 1025): a group whose spread is tiny next to its offset
                # (a constant non-zero group and its 1e-5 range) gets a wider scale
                wide = _to_half_sat((np.abs(x_min) * F32(2.0 ** -10)).astype(F32)).astype(F32)
                wide = np.where(wide == 0, F32(2.0 ** -24), wide).astype(F32)
                scale = np.where(np.abs(x_min) > (F32(1024.0) * scale).astype(F32), wide, scale).astype(F32)
        if sym:
            zero = np.zeros_like(scale)
        else:
            zero = (F32(qmin) - np.rint((x_min / scale).astype(F32))).astype(F32)
            if bits == 4:
                zero = _to_half_sat(zero).astype(F32)
    return scale.astype(F32), zero.astype(F32)


def quantize_groups(x: np.ndarray, group: int, scheme: int):
    """Quantise every run of `group` contiguous elements of the last axis.
        q = clamp(round(x/scale + zero), qmin, qmax)   (round half to even)
    (core/single/module/pikv_compression.py:1003).  x is float32 (bf16 inputs
    are upcast first).  Returns (codes int16 [..., D], scale f32 [..., D/group],
    zero f32 [..., D/group])."""
    bits, sym, qmin, qmax = scheme_info(scheme)
    x = np.asarray(x, dtype=F32)
    D = x.shape[-1]
    assert D % group == 0
    xg = x.reshape(x.shape[:-1] + (D // group, group))
    scale, zero = quant_params(xg.min(axis=-1), xg.max(axis=-1), scheme)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        y = (xg / scale[..., None]).astype(F32)
        y = (y + zero[..., None]).astype(F32)
        q = np.clip(np.rint(y), qmin, qmax)
    q = np.nan_to_num(q, nan=float(qmin)).astype(np.int16)
    return q.reshape(x.shape), scale, zero


def dequantize_groups(codes, scale, zero, group: int) -> np.ndarray:
    """dq = (q - zero) * scale in float32
    (core/single/module/pikv_compression.py:1006)."""
    codes = np.asarray(codes)
    D = codes.shape[-1]
    qg = codes.reshape(codes.shape[:-1] + (D // group, group)).astype(F32)
    dq = ((qg - np.asarray(zero, F32)[..., None]).astype(F32)
          * np.asarray(scale, F32)[..., None]).astype(F32)
    return dq.reshape(codes.shape)


def pack_int4(codes: np.ndarray) -> np.ndarray:
    """Two 4-bit codes per byte, low nibble = even element.  Signed codes are
    stored as two's-complement nibbles."""
    c = (np.asarray(codes).astype(np.int16) & 0xF).astype(np.uint8)
    return (c[..., 0::2] | (c[..., 1::2] << 4)).astype(np.uint8)


def unpack_int4(packed: np.ndarray, signed: bool) -> np.ndarray:
    p = np.asarray(packed, dtype=np.uint8)
    lo = (p & 0xF).astype(np.int16)
    hi = (p >> 4).astype(np.int16)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.int16)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    if signed:
        out = np.where(out >= 8, out - 16, out)
    return out.astype(np.int16)


def fakequant_colblocks(x: np.ndarray, group: int, bits: int = 8,
                        symmetric: bool = False):
    """QuantizedCompressor.forward's domain (core/single/pikv_compression.py:
    474-506): rows flattened to [N,H]; for each block of `group` columns the
    min/max are taken over ALL rows of the block; output is the dequantised
    float tensor.  Returns (dq [N,H] f32, stats [nblk,4] = (min,max,scale,zero),
    mse [nblk])."""
    x = np.asarray(x, dtype=F32)
    N, H = x.shape
    scheme = {(8, False): Q_I8_ASYM, (8, True): Q_I8_SYM,
              (4, False): Q_I4_ASYM, (4, True): Q_I4_SYM}[(bits, symmetric)]
    _, sym, qmin, qmax = scheme_info(scheme)
    out = np.empty_like(x)
    stats, mse = [], []
    for c0 in range(0, H, group):
        blk = x[:, c0:c0 + group]
        mn, mx = F32(blk.min()), F32(blk.max())
        if mx == mn:
            mx = F32(mn + F32(1e-5))
        qr = F32(qmax - qmin)
        if sym:
            scale = F32(F32(2.0) * max(abs(mn), abs(mx))) / qr
            zero = F32(0.0)
        else:
            scale = F32(mx - mn) / qr
            zero = F32(qmin) - F32(np.rint(F32(mn / scale)))
        scale = F32(scale)
        q = np.clip(np.rint(((blk / scale).astype(F32) + zero).astype(F32)), qmin, qmax).astype(F32)
        dq = ((q - zero).astype(F32) * scale).astype(F32)
        out[:, c0:c0 + group] = dq
        stats.append((mn, mx, scale, zero))
        mse.append(np.mean((blk.astype(np.float64) - dq.astype(np.float64)) ** 2))
    return out, np.array(stats, dtype=F32), np.array(mse, dtype=np.float64)


def fakequant_preset(x: np.ndarray, scale, zero, group: int, bits: int = 8,
                     symmetric: bool = False):
    """QuantizedCompressor._quantize with dynamic_quantization=False once calibrated
    (core/single/pikv_compression.py:455-472): q = clamp(round(x/scale + zero_point)),
    dq = (q - zero_point)*scale with the stored scalars.  Returns (dq [N,H] f32,
    mse per block of `group` columns)."""
    x = np.asarray(x, dtype=F32)
    scale, zero = F32(scale), F32(zero)
    qmin = -(1 << (bits - 1)) if symmetric else 0
    qmax = (1 << (bits - 1)) - 1 if symmetric else (1 << bits) - 1
    q = np.clip(np.rint(((x / scale).astype(F32) + zero).astype(F32)), qmin, qmax).astype(F32)
    dq = ((q - zero).astype(F32) * scale).astype(F32)
    mse = [np.mean((x[:, c0:c0 + group].astype(np.float64) - dq[:, c0:c0 + group].astype(np.float64)) ** 2)
           for c0 in range(0, x.shape[1], group)]
    return dq, np.array(mse, dtype=np.float64)


def quant8_minshift(x: np.ndarray):
    """PiKVKernels.compress_kv QUANT8 fallback (core/single/pikv_kernels.py:
    215-232): per row, s=(max-min)/255; q=round((x-min)/s).clamp(0,255);
    dq=q*s+min.  Returns (q uint8, dq f32, s [N,1], min [N,1])."""
    x = np.asarray(x, dtype=F32)
    mn = x.min(axis=1, keepdims=True)
    mx = x.max(axis=1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        s = ((mx - mn).astype(F32) / F32(255.0)).astype(F32)
        q = np.clip(np.rint(((x - mn).astype(F32) / s).astype(F32)), 0, 255)
    q = np.nan_to_num(q, nan=0.0).astype(np.uint8)
    dq = ((q.astype(F32) * s).astype(F32) + mn).astype(F32)
    return q, dq, s, mn


# --------------------------------------------------------------------------
# R9  cache pool: scatter / append
# --------------------------------------------------------------------------

class CachePool:
    """n_caches caches sharing one row space; cache c owns rows
    [base[c], base[c]+cap[c]), the first fill[c] of them valid.  Layout
    precedent: k_cache[slot, head, head_dim] (core/single/pikv_attention.py:
    41-48); append semantics: core/single/cache_scheduling.py:429-436."""

    def __init__(self, caps, D, group, scheme, with_v=True):
        self.cap = np.asarray(caps, dtype=np.int32)
        self.base = np.concatenate([[0], np.cumsum(self.cap.astype(np.int64))[:-1]]).astype(np.int64)
        self.rows = int(self.cap.astype(np.int64).sum())
        self.fill = np.zeros(len(self.cap), dtype=np.int32)
        self.D, self.group, self.scheme = D, group, scheme
        bits, sym, _, _ = scheme_info(scheme)
        self.bits, self.sym = bits, sym
        ng = D // group
        self.k_codes = np.zeros((self.rows, D), dtype=np.int16)
        self.k_scale = np.zeros((self.rows, ng), dtype=F32)
        self.k_zero = np.zeros((self.rows, ng), dtype=F32)
        self.with_v = with_v
        if with_v:
            self.v_codes = np.zeros((self.rows, D), dtype=np.int16)
            self.v_scale = np.zeros((self.rows, ng), dtype=F32)
            self.v_zero = np.zeros((self.rows, ng), dtype=F32)
        self.acc = np.zeros(self.rows, dtype=F32)
        self.ts = np.zeros(self.rows, dtype=F32)

    def quant_scatter(self, k_src, v_src, cache_id, slot, fanout, now=0.0):
        """Quantise source row s once and write it to the rows of its
        assignments a = s*fanout + j: row = fill[c] + slot[a]; dropped when
        slot[a] < 0 or row >= cap[c].  fill is not advanced."""
        kq, ks, kz = quantize_groups(k_src, self.group, self.scheme)
        if self.with_v:
            vq, vs, vz = quantize_groups(v_src, self.group, self.scheme)
        cache_id = np.asarray(cache_id).reshape(-1)
        slot = np.asarray(slot).reshape(-1)
        a = np.arange(cache_id.size)
        src = a // fanout
        r = self.fill[cache_id].astype(np.int64) + slot
        ok = (slot >= 0) & (r < self.cap[cache_id])
        rows = (self.base[cache_id] + r)[ok]
        s_ok = src[ok]
        self.k_codes[rows] = kq[s_ok]
        self.k_scale[rows] = ks[s_ok]
        self.k_zero[rows] = kz[s_ok]
        if self.with_v:
            self.v_codes[rows] = vq[s_ok]
            self.v_scale[rows] = vs[s_ok]
            self.v_zero[rows] = vz[s_ok]
        self.acc[rows] = 0.0
        self.ts[rows] = F32(now)
        return rows

    def advance(self, count, per_call_limit=-1):
        """fill[c] = min(fill[c] + min(count[c], limit), cap[c])
        (core/single/cache_scheduling.py:430-436)."""
        add = np.asarray(count, dtype=np.int64)
        if per_call_limit >= 0:
            add = np.minimum(add, per_call_limit)
        self.fill = np.minimum(self.fill.astype(np.int64) + add, self.cap).astype(np.int32)

    def valid_rows(self, c):
        return np.arange(self.base[c], self.base[c] + self.fill[c])


# --------------------------------------------------------------------------
# R11-R12  scores and H2O accumulation
# --------------------------------------------------------------------------

def attention_scores(q: np.ndarray, k_hat: np.ndarray, n_kv_heads: int,
                     scale_qk: float) -> np.ndarray:
    """scores[h,n] = dot(q[h,:], K^[n, h//rep, :]) * scale_qk
    (core/single/pikv_attention.py:123: matmul(q,k^T)/sqrt(head_dim)).
    q [Hq,dh]; k_hat [N, Hkv*dh] dequantised float32.  float64 accumulate,
    rounded once to float32."""
    Hq, dh = q.shape
    N = k_hat.shape[0]
    rep = Hq // n_kv_heads
    kh = k_hat.reshape(N, n_kv_heads, dh).astype(np.float64)
    out = np.empty((Hq, N), dtype=np.float64)
    for h in range(Hq):
        out[h] = kh[:, h // rep, :] @ q[h].astype(np.float64)
    return (out * np.float64(F32(scale_qk))).astype(F32)


def h2o_importance(scores: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """probs = softmax over cached tokens (core/single/pikv_attention.py:163);
    importance[n] = sum of probs over the query heads
    (core/single/pikv_moe.py:241-245).  scores [Hq,N] -> (probs, imp [N])."""
    s = scores.astype(np.float64)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    p = e / e.sum(axis=-1, keepdims=True)
    return p.astype(F32), p.sum(axis=0).astype(F32)


def attend_values(probs: np.ndarray, v_hat: np.ndarray, n_kv_heads: int) -> np.ndarray:
    """context[h,:] = sum_n probs[h,n] * V^[n, h//rep, :]
    (core/single/pikv_attention.py:188: matmul(attention_probs, v)).
    probs [Hq,N]; v_hat [N, Hkv*dh] dequantised float32.  float64 accumulate."""
    Hq, N = probs.shape
    rep = Hq // n_kv_heads
    vh = v_hat.reshape(N, n_kv_heads, -1).astype(np.float64)
    out = np.empty((Hq, vh.shape[2]), dtype=np.float64)
    for h in range(Hq):
        out[h] = probs[h].astype(np.float64) @ vh[:, h // rep, :]
    return out.astype(F32)


def h2o_accumulate(acc, ts, rows, imp, now, decay=1.0):
    """acc[idx] += w; ts[idx] = t (core/single/cache_scheduling.py:69-73);
    decay-first variant core/single/module/pikv_scheduling.py:119-130."""
    if decay != 1.0:
        acc[rows] = (acc[rows] * F32(decay)).astype(F32)
    acc[rows] = (acc[rows] + imp.astype(F32)).astype(F32)
    ts[rows] = F32(now)


# --------------------------------------------------------------------------
# R13-R16  eviction selection and compaction
# --------------------------------------------------------------------------

def h2o_budget(length: int, heavy_ratio: float, recent_ratio: float):
    """num_heavy = max(1,int(len*ratio)), num_recent likewise
    (core/single/cache_scheduling.py:83-84)."""
    return max(1, int(length * heavy_ratio)), max(1, int(length * recent_ratio))


def h2o_keep(acc: np.ndarray, ts: np.ndarray, n_heavy: int, n_recent: int) -> np.ndarray:
    """keep = top-n_heavy of the accumulator UNION top-n_recent of the
    timestamps (core/single/cache_scheduling.py:86-97); returns bool [len]."""
    L = acc.shape[0]
    keep = np.zeros(L, dtype=bool)
    keep[topk_desc(acc[None, :], min(n_heavy, L))[0]] = True
    keep[topk_desc(ts[None, :], min(n_recent, L))[0]] = True
    return keep


def lru_keep(access_times: np.ndarray, n_evict: int) -> np.ndarray:
    """Evict the n_evict least recently used rows
    (core/single/cache_scheduling.py:278-283, topk largest=False)."""
    L = access_times.shape[0]
    keep = np.ones(L, dtype=bool)
    if n_evict > 0:
        keep[topk_asc(access_times[None, :], min(n_evict, L))[0]] = False
    return keep


def streaming_keep(cache_len: int, start_size: int, recent_size: int) -> np.ndarray:
    """Keep the first start_size rows and the rows from
    max(start_size, cache_len - recent_size) on (core/single/cache_scheduling.py:125-132)."""
    keep = np.zeros(cache_len, dtype=bool)
    keep[:start_size] = True
    keep[max(start_size, cache_len - recent_size):] = True
    return keep


def duo_keep(cache_len: int, sink_size: int, recent_size: int) -> np.ndarray:
    """Keep rows [:sink_size] and [-recent_size:]
    (core/single/module/pikv_scheduling.py:695-700)."""
    keep = np.zeros(cache_len, dtype=bool)
    keep[:sink_size] = True
    if recent_size > 0:
        keep[-recent_size:] = True
    return keep


def adakv_keep(scores: np.ndarray, compression_ratio: float, safeguard_ratio: float) -> np.ndarray:
    """num_keep = int(len*(1-ratio)); the top int(num_keep*safeguard) scores are kept
    first, then the top (num_keep - safeguarded) of the remaining ones
    (core/single/module/pikv_scheduling.py:648-661).  Ties to the lower index."""
    s = np.asarray(scores, F32)
    L = s.shape[0]
    num_keep = int(L * (1 - compression_ratio))
    num_safe = int(num_keep * safeguard_ratio)
    keep = np.zeros(L, dtype=bool)
    safe = topk_desc(s[None, :], num_safe)[0] if num_safe > 0 else np.zeros(0, dtype=np.int64)
    keep[safe] = True
    rest = s.copy()
    rest[safe] = -np.inf
    if num_keep - num_safe > 0:
        keep[topk_desc(rest[None, :], num_keep - num_safe)[0]] = True
    return keep


def quest_utility(quality, frequency, last_access, now, decay_factor) -> np.ndarray:
    """utility = quality * frequency * decay^(now - last access)
    (core/single/cache_scheduling.py:166-176), float32."""
    decay = np.power(F32(decay_factor), (F32(now) - np.asarray(last_access, F32))).astype(F32)
    return (np.asarray(quality, F32) * np.asarray(frequency, F32) * decay).astype(F32)


def evict_lowest(score: np.ndarray, n_evict: int) -> np.ndarray:
    """EVICT mask of the n_evict lowest scores (topk largest=False,
    core/single/cache_scheduling.py:197,245,343), ties to the lower index."""
    L = score.shape[0]
    ev = np.zeros(L, dtype=bool)
    if n_evict > 0:
        ev[topk_asc(np.asarray(score, F32)[None, :], min(n_evict, L))[0]] = True
    return ev


def quest_evict(utility: np.ndarray, threshold: float, n_evict: int) -> np.ndarray:
    """Rows below the threshold go; when they are fewer than n_evict, the n_evict
    lowest go instead (core/single/cache_scheduling.py:190-201)."""
    below = np.asarray(utility, F32) < F32(threshold)
    if below.sum() < n_evict:
        return evict_lowest(utility, n_evict)
    return below


def flexgen_benefit(frequency, cost) -> np.ndarray:
    """benefit = access frequency / access cost (core/single/cache_scheduling.py:241)."""
    return (np.asarray(frequency, F32) / np.asarray(cost, F32)).astype(F32)


def lruplus_priority(times, frequency, importance, frequency_weight=0.3,
                     importance_weight=0.4) -> np.ndarray:
    """priority = w_r*t/(max t + 1e-8) + w_f*f/(max f + 1e-8) + w_i*importance with
    w_r = 1 - w_f - w_i (core/single/cache_scheduling.py:296,311-327), float32."""
    t, f = np.asarray(times, F32), np.asarray(frequency, F32)
    w_r = 1.0 - frequency_weight - importance_weight
    rec = (t / (t.max() + F32(1e-8))).astype(F32)
    frq = (f / (f.max() + F32(1e-8))).astype(F32)
    return (F32(w_r) * rec + F32(frequency_weight) * frq
            + F32(importance_weight) * np.asarray(importance, F32)).astype(F32)


def compact(keep: np.ndarray, *planes):
    """keep_indices = where(keep)[0]; cache[:m] = cur[keep_indices]
    (core/single/cache_scheduling.py:418-424): survivors move to the front in
    ascending order, in place.  Returns m."""
    idx = np.nonzero(keep)[0]
    for p in planes:
        p[:idx.size] = p[idx]
    return int(idx.size)


def pyramid_cache_sizes(c1: int, decrement: int, num_layers: int):
    """C_l = C_1 - (l-1)*d (core/single/pikv_moe.py:218-224)."""
    return [c1 - (i - 1) * decrement for i in range(1, num_layers + 1)]


def pyramid_keep_counts(n_tokens: int, num_layers: int, final_fraction: float = 0.25):
    """Per-layer kept-token budget decaying linearly from 100% at layer 0 to
    final_fraction at the last layer: keep_l = int(N*(1-(1-f)*l/(L-1)))."""
    L = num_layers
    return [int(n_tokens * (1.0 - (1.0 - final_fraction) * l / (L - 1))) if L > 1 else n_tokens
            for l in range(L)]
