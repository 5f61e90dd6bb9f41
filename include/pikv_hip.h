/*
 * pikv_hip.h - C ABI of libpikv_hip.so: the routed, compressed KV-cache data
 * path of PiKV as hand-written gfx950 (MI355X) HIP kernels.
 *
 * Conventions (shared by every entry point)
 *   - Every pointer is a DEVICE pointer unless the name ends in _host.
 *   - Tensors are row-major and contiguous; shapes are given in the comments.
 *   - The caller allocates every output and every workspace; no entry point
 *     allocates, frees or synchronises.  Work is enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the default stream).
 *   - Return value: PIKV_OK (0) or a negative PIKV_ERR_* code.  Nothing is
 *     enqueued when an error is returned.  pikv_status_string() names a code.
 *   - Deterministic: no floating-point atomics; integer outputs (expert
 *     indices, slots, codes, eviction sets) do not depend on launch geometry.
 *   - Every top-k in this library orders by (value, index): larger value first
 *     (or smaller first where stated), LOWER INDEX FIRST among equal values.
 *
 * The reference keeps its native surface in core/cuda/ as
 *   extern "C" void launch_<name>(ptrs..., ints..., floats..., cudaStream_t)
 * (core/cuda/pikv_routing_kernel.cu:404-511, pikv_compression_kernel.cu:463-623,
 * pikv_scheduling_kernel.cu:504-676) and binds it from
 * core/single/pikv_kernels.py:36-52.  Each entry point below names the
 * reference interface it replaces.
 *
 * "Cache pool" layout used by the scatter / read / evict entry points
 *   A pool holds n_caches independent caches (one per expert, or one per
 *   sequence) in one row space.  Cache c owns rows
 *   [cache_row_base[c], cache_row_base[c] + cache_cap[c]) of which the first
 *   cache_fill[c] are valid.  Per row the pool stores, in separate planes,
 *     codes  : int8  [rows, D]        (8-bit)   or uint8 [rows, D/2] (4-bit,
 *              two codes per byte, low nibble = even element)
 *     scale  : float [rows, D/group]  (8-bit)   or __half [rows, D/group] (4-bit)
 *     zero   : same shape/type as scale; only for asymmetric schemes
 *     acc,ts : float [rows]           H2O accumulator and access timestamp
 *   with D = n_heads * head_dim, and `group` the quantisation domain
 *   (D = per token, head_dim = per token per head, 32 = per group of 32).
 *   Row layout inside a plane is [head][head_dim], as the reference's
 *   k_cache[slot, head, head_dim] (core/single/pikv_attention.py:41-48).
 */
#ifndef PIKV_HIP_H
#define PIKV_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes ------------------------------------------------------ */
#define PIKV_OK                 0
#define PIKV_ERR_NULL          -1   /* a required pointer is NULL            */
#define PIKV_ERR_SHAPE         -2   /* a dimension is out of range           */
#define PIKV_ERR_UNSUPPORTED   -3   /* valid request this build cannot serve */
#define PIKV_ERR_WORKSPACE     -4   /* workspace too small                   */
#define PIKV_ERR_LAUNCH        -5   /* the HIP runtime refused the launch    */

/* ---- element types ------------------------------------------------------ */
#define PIKV_F32   0
#define PIKV_BF16  1

/* ---- quantisation schemes (reference formula:
 *      core/single/module/pikv_compression.py:945-1012) -------------------- */
#define PIKV_Q_I8_SYM    0   /* codes -128..127, float scale                 */
#define PIKV_Q_I8_ASYM   1   /* codes 0..255,    float scale + float zero    */
#define PIKV_Q_I4_ASYM   2   /* codes 0..15,     half scale + half zero      */
#define PIKV_Q_I4_SYM    3   /* codes -8..7,     half scale                  */
/* 4-bit metadata is rounded to half BEFORE the codes are computed, so encoder and
 * decoders share the same two numbers.  PIKV_Q_I4_ASYM only: when |min| > 1024*scale
 * (a spread that is tiny next to the offset, e.g. a constant group) the scale becomes
 * half(|min|/1024), which keeps the zero point an integer that half represents exactly. */

/* ---- router arithmetic: the reference holds two copies of its routers --------
 * SINGLE (core/single/pikv_routing.py:653-656, :68-70):  logits / temperature, then
 *        * expert_scale, mask penalty (1-mask)*-1e9.
 * MODULE (core/single/module/pikv_routing.py:596-600, :133-134): * expert_scale, then
 *        / temperature, mask penalty (1-mask)*finfo(float32).min; its renormalisation
 *        adds 1e-8 to the sum (:143) - pass renorm_eps = 1e-8. */
#define PIKV_ROUTER_SINGLE 0
#define PIKV_ROUTER_MODULE 1

/* ---- eviction policies (core/single/cache_scheduling.py:9-17) ----------- */
#define PIKV_EVICT_H2O   0
#define PIKV_EVICT_LRU   1

const char* pikv_status_string(int status);

/* Library/ABI version: major*1000 + minor. */
int pikv_abi_version(void);

/* ------------------------------------------------------------------------
 * K1  fused router
 * Replaces: BaseRouter.forward's tail - last nn.Linear of the gate, mask,
 *   softmax, top-k, renormalise, capacity slots
 *   (core/single/pikv_routing.py:65-82; capacity rule
 *   core/single/module/pikv_routing.py:62-106); EPLBRouter's temperature and
 *   expert_weights scaling (core/single/pikv_routing.py:653-660); native
 *   precedents launch_adaptive_routing_kernel / launch_topk_routing_kernel /
 *   launch_expert_capacity_kernel (core/cuda/pikv_routing_kernel.cu:404-511).
 *
 *   logits[t,e] = sum_h x[t,h]*w[e,h] + bias[e]          (fp32 accumulate)
 *   logits     /= temperature            (if temperature != 1; true division)
 *   logits     *= expert_scale[e]        (if expert_scale != NULL)
 *   logits     += (1-expert_mask[e])*-1e9 (if expert_mask != NULL)
 *                 (order and penalty of arithmetic = PIKV_ROUTER_SINGLE; see above)
 *   probs       = softmax_e(logits)
 *   topk_idx    = k largest PROBABILITIES (the float32 values of `probs`, what the
 *                 reference hands to torch.topk), (value desc, index asc, NaN last):
 *                 distinct logits whose probabilities round to one float32 tie, and
 *                 the lower expert wins
 *   topk_w      = probs[topk_idx] / (sum_j probs[topk_idx[j]] + renorm_eps)
 *   slot[t,j]   = number of assignments (t',j') < (t,j) in token-major order
 *                 with the same expert; -1 when that count >= capacity
 *   count[e]    = number of assignments to e (kept or not)
 *
 *   The float32 summation order of the projection depends on T (short, medium and long
 *   token streams take different kernels) and on the token's position in the batch (a
 *   block starts its walk along H at a block-dependent offset): the same token row gives
 *   logits that agree to within 1e-5 * sqrt(H) of the exact value, not bit for bit, and a
 *   near-tie can resolve differently.  For one (T, position) the result is deterministic.
 *
 *   x        [T,H]  x_dtype (PIKV_F32|PIKV_BF16)   w [E,H] same dtype
 *   bias     [E] float or NULL        expert_scale, expert_mask [E] float|NULL
 *   probs    [T,E] float or NULL      logits_out [T,E] float or NULL
 *   topk_idx [T,k] int32              topk_w [T,k] float
 *   slot     [T,k] int32 or NULL (then capacity/count/workspace are unused)
 *   count    [E] int32 or NULL
 *   1 <= E <= 64, 1 <= k <= min(E,8), H % 8 == 0
 *   workspace: pikv_router_fused_workspace_bytes(T,H,E,k) bytes, 256-byte aligned
 *              (slot scan counters, the gate weights re-laid per 32-wide k-step
 *              for the bf16 matrix-core projection and, for short token streams,
 *              partial logits per slice of H); required whenever slot != NULL
 *              or x_dtype == PIKV_BF16.
 * ---------------------------------------------------------------------- */
int pikv_router_fused(const void* x, const void* w, int x_dtype,
                      const float* bias, const float* expert_scale,
                      const float* expert_mask, float temperature,
                      float renorm_eps, int arithmetic,
                      int64_t T, int H, int E, int k, int64_t capacity,
                      float* probs, float* logits_out,
                      int32_t* topk_idx, float* topk_w,
                      int32_t* slot, int32_t* count,
                      void* workspace, int64_t workspace_bytes, void* stream);

/* Router tail on precomputed logits.
 * Replaces: PiKVRouter.forward's importance-gated blend of two gates,
 *   cache_correction_factor and everything after
 *   (core/single/pikv_routing.py:450-470), and PiKVKernels.top_k_routing
 *   (core/single/pikv_kernels.py:54-99; use_softmax = 0 gives the raw top-k
 *   of the logits that its fallback computes).
 *   logits_b and select are optional: row t uses logits_a when
 *   select[t] != 0 (or select == NULL) else logits_b.
 *   With use_softmax = 0, probs is not written and topk_w holds the selected
 *   logits themselves (no renormalisation).
 *   Other arguments as in pikv_router_fused.
 * ---------------------------------------------------------------------- */
int pikv_router_tail(const float* logits_a, const float* logits_b,
                     const uint8_t* select,
                     const float* expert_scale, const float* expert_mask,
                     float temperature, float renorm_eps, int use_softmax,
                     int arithmetic,
                     int64_t T, int E, int k, int64_t capacity,
                     float* probs, int32_t* topk_idx, float* topk_w,
                     int32_t* slot, int32_t* count,
                     void* workspace, int64_t workspace_bytes, void* stream);

/* Capacity slots alone, from expert indices in token-major order.
 * Replaces: _create_dispatch_combine_tensors' sequential fill
 *   (core/single/module/pikv_routing.py:93-104) in its compact form.
 *   expert_idx [A] int32 in [0,E); slot [A]; count [E]. */
int pikv_capacity_slots(const int32_t* expert_idx, int64_t A, int E,
                        int64_t capacity, int32_t* slot, int32_t* count,
                        void* workspace, int64_t workspace_bytes, void* stream);

/* pikv_capacity_slots for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference: there every intermediate is a fresh torch tensor.
 * Same arguments, same kernels and bit-identical results as pikv_capacity_slots,
 * but the per-chunk counters live in a 512 KiB device array that is part of the
 * library image (one copy per GPU, held until the process ends) instead of a
 * caller workspace; the call allocates and frees nothing.
 *   A <= pikv_capacity_slots_static_max() (= 1048576 assignments), E <= 64;
 *   a larger A returns PIKV_ERR_WORKSPACE and enqueues nothing.
 *   All calls on one GPU share the array: calls that overlap on one GPU (two
 *   streams, two threads) race; calls on one stream are ordered and safe.
 *   The device that is current at the call must be the one that owns the pointers.
 *   Set-up: the first use on a device looks up the array's address there, which can
 *   make the HIP runtime load the library's code object - not something to do inside an
 *   open graph capture.  pikv_capacity_slots_static_max() performs that look-up for the
 *   current device (and returns the limit): call it, or make one eager call, on every
 *   device before capturing. */
int pikv_capacity_slots_static(const int32_t* expert_idx, int64_t A, int E,
                               int64_t capacity, int32_t* slot, int32_t* count,
                               void* stream);
int64_t pikv_capacity_slots_static_max(void);

/* Workspace of pikv_router_tail / pikv_capacity_slots, and of pikv_router_fused. */
int64_t pikv_router_workspace_bytes(int64_t T, int E, int k);
int64_t pikv_router_fused_workspace_bytes(int64_t T, int H, int E, int k);

/* ------------------------------------------------------------------------
 * K2  fused KV quantise + per-cache scatter (append)
 * Replaces: QuantizedCompressor._quantize_tensor's formula
 *   (core/single/module/pikv_compression.py:945-1012; asymmetric form also
 *   core/single/pikv_compression.py:396-429) applied per `group` contiguous
 *   elements of a token row, with the integer codes KEPT, followed by
 *   CacheSchedulingManager.update_cache's append
 *   (core/single/cache_scheduling.py:429-436) into each routed expert's cache;
 *   native precedents launch_quantization_compression_kernel
 *   (core/cuda/pikv_compression_kernel.cu:490-508) and
 *   launch_lru_cache_management_kernel (pikv_scheduling_kernel.cu:506-529).
 *
 *   Source row s (0 <= s < n_src) is quantised once and written to the rows
 *   of its `fanout` assignments a = s*fanout + j:
 *     c = cache_id[a]; if slot[a] < 0 the assignment is dropped;
 *     r = cache_fill[c] + slot[a]; dropped when r >= cache_cap[c]
 *     (core/single/cache_scheduling.py:431-432: rows beyond the cache are
 *     silently truncated); pool row = cache_row_base[c] + r.
 *   n_src = T, fanout = k      : K/V shared by a token's k experts
 *   n_src = T*k, fanout = 1    : K/V projected per assignment
 *   cache_fill is NOT modified here (see pikv_cache_advance).
 *
 *   k_src, v_src [n_src, D] src_dtype; v_src and its outputs may be NULL.
 *   scheme       PIKV_Q_*; group: power of two, 16 <= group <= 1024 for
 *                8-bit, 32 <= group <= 2048 for 4-bit, D % group == 0.
 *   k_codes/v_codes, k_scale/v_scale, k_zero/v_zero: pool planes (see top);
 *                zero planes are required for asymmetric schemes only.
 *   row_acc,row_ts [rows] float or NULL: set to 0 and `now` for written rows.
 * ---------------------------------------------------------------------- */
int pikv_quant_scatter(const void* k_src, const void* v_src, int src_dtype,
                       int64_t n_src, int fanout, int D, int group, int scheme,
                       const int32_t* cache_id, const int32_t* slot,
                       const int64_t* cache_row_base, const int32_t* cache_fill,
                       const int32_t* cache_cap, int n_caches,
                       void* k_codes, void* v_codes,
                       void* k_scale, void* v_scale,
                       void* k_zero, void* v_zero,
                       float* row_acc, float* row_ts, float now,
                       void* stream);

/* cache_fill[c] = min(cache_fill[c] + min(count[c], per_call_limit), cache_cap[c])
 * Replaces: cache_size_current.fill_(end_idx)
 *   (core/single/cache_scheduling.py:436).  per_call_limit is the router
 *   capacity (rows with slot >= capacity were dropped); pass a negative value
 *   for "no limit". */
int pikv_cache_advance(int32_t* cache_fill, const int32_t* count,
                       const int32_t* cache_cap, int n_caches,
                       int64_t per_call_limit, void* stream);

/* Pyramid compression: quantise a SELECTED subset of source rows into the caches,
 * in list order.  For cache c and j < n_take[c], the source row
 *     src_row_base[c] + src_index[src_row_base[c] + j]
 * is quantised (same formula as pikv_quant_scatter) and appended at cache row
 * cache_fill[c] + j; rows past cache_cap[c] are dropped; cache_fill is not advanced.
 * src_index is an ascending survivor list in the SOURCE row space, as
 * pikv_evict_select writes it when it is handed the source geometry
 * (cache_row_base = src_row_base, cache_fill = rows per layer, n_heavy = keep_l,
 * n_recent = 0): top-keep_l by score, ties to the lower index, original order kept.
 * A gathered row starts with accumulator src_score[source row] (0 when src_score
 * is NULL) and timestamp `now`.
 * Replaces: the importance-descending partition of PyramidCompressor.forward
 *   (core/single/pikv_compression.py:145-160) followed by per-level compression,
 *   with the per-layer budgets of PiKVMoE.pyramidal_cache_allocation
 *   (core/single/pikv_moe.py:218-224); max_take >= max_c n_take[c] sizes the grid. */
int pikv_quant_gather(const void* k_src, const void* v_src, int src_dtype,
                      int D, int group, int scheme,
                      const int64_t* src_row_base, const int32_t* src_index,
                      const int32_t* n_take, int64_t max_take, const float* src_score,
                      const int64_t* cache_row_base, const int32_t* cache_fill,
                      const int32_t* cache_cap, int n_caches,
                      void* k_codes, void* v_codes,
                      void* k_scale, void* v_scale,
                      void* k_zero, void* v_zero,
                      float* row_acc, float* row_ts, float now,
                      void* stream);

/* Quantise rows in place order (no routing): row i of the source goes to row
 * dst_row0 + i of the planes. Same formula as pikv_quant_scatter; used for
 * QuantizedCompressor.quantize() and for bulk cache prefill. */
int pikv_quantize_rows(const void* src, int src_dtype, int64_t n_rows, int D,
                       int group, int scheme, int64_t dst_row0,
                       void* codes, void* scale, void* zero, void* stream);

/* Min-shift 8-bit quantisation of whole rows, the algebra of the kernel facade.
 * Replaces: PiKVKernels.compress_kv, CompressionMode.QUANT8
 *   (core/single/pikv_kernels.py:215-246):
 *     mn = min(row); s = (max(row) - mn) / 255
 *     codes = clamp(round((x - mn) / s), 0, 255); dq = codes * s + mn
 *   float32 arithmetic in that order (bf16 sources are widened first).  A constant
 *   row has s = 0, codes 0 and dq = mn.
 *   src [n_rows, D] src_dtype; codes uint8 [n_rows, D]; dq float [n_rows, D] or NULL;
 *   scale, row_min float [n_rows] (the reference's k_scale / k_min as [N,1]). */
int pikv_quant8_minshift(const void* src, int src_dtype, int64_t n_rows, int D,
                         uint8_t* codes, float* dq, float* scale, float* row_min,
                         void* stream);

/* ------------------------------------------------------------------------
 * K3  gather + dequantise read path, attention scores, H2O accumulation
 * Replaces: dq = (q - zero_point) * scale
 *   (core/single/module/pikv_compression.py:1006), attention_scores =
 *   matmul(q, k^T)/sqrt(head_dim) and softmax(dim=-1)
 *   (core/single/pikv_attention.py:123,163), importance = probs.sum over
 *   queries (core/single/pikv_moe.py:241-245) and
 *   H2OScheduler.update_attention_scores
 *   (core/single/cache_scheduling.py:69-73); native precedent
 *   launch_cache_access_update_kernel (pikv_scheduling_kernel.cu:616-631).
 * ---------------------------------------------------------------------- */

/* out[i,:] = dequant(row rows[i]) (rows == NULL: row row0 + i).
 * out [n, D] out_dtype (PIKV_F32 | PIKV_BF16, round-to-nearest-even). */
int pikv_gather_dequant(const void* codes, const void* scale, const void* zero,
                        int D, int group, int scheme,
                        const int64_t* rows, int64_t row0, int64_t n,
                        void* out, int out_dtype, void* stream);

/* For every cache c and query head h (kv head g = h / (n_q_heads/n_kv_heads)):
 *   scores[c,h,n] = dot(q[c,h,:], dequant(K[row_base[c]+n, g, :])) * scale_qk
 *   for n < min(cache_fill[c], max_len); other entries are not written.  A cache
 *   that holds more than max_len rows is read as its first max_len rows, here and
 *   in pikv_h2o_accumulate / pikv_attend_values (same max_len in all three).
 *   q       [n_caches, n_q_heads, head_dim] q_dtype
 *   scores  [n_caches, n_q_heads, score_stride] float
 *   tile_max, tile_sum [n_caches, n_tiles, n_q_heads] float: per tile of
 *   PIKV_SCORE_TILE cached tokens, max score and sum of exp(score - max);
 *   n_tiles = ceil(max_len / PIKV_SCORE_TILE) with max_len <= score_stride
 *   the number of rows per cache the caller wants covered.
 *   D = n_kv_heads*head_dim; head_dim a power of two >= 16 (8-bit) / 32 (4-bit);
 *   any number of kv heads, any n_q_heads <= 128 that is a multiple of n_kv_heads, for
 *   either q_dtype (more query heads: PIKV_ERR_UNSUPPORTED).  float32 queries against 4-bit group-32 caches, or 8-bit caches
 *   with a scale per kv head or coarser, with up to 8 query heads per 128 dimensions
 *   of kv heads are multiplied on the matrix cores as two bf16 limbs (q = hi + lo to
 *   2^-18 |q|; float32 accumulation). */
#define PIKV_SCORE_TILE 64
int pikv_gather_dequant_scores(const void* k_codes, const void* k_scale,
                               const void* k_zero, int scheme, int group,
                               int n_kv_heads, int n_q_heads, int head_dim,
                               const void* q, int q_dtype, float scale_qk,
                               const int64_t* cache_row_base,
                               const int32_t* cache_fill, int n_caches,
                               int64_t max_len, int64_t score_stride,
                               float* scores, float* tile_max, float* tile_sum,
                               void* stream);

/* Softmax-normalise the scores over each cache's valid tokens, sum the
 * probabilities over the n_q_heads heads and fold them into the H2O state:
 *   acc[row] = acc[row]*decay + sum_h softmax_n(scores[c,h,:])[n]
 *   ts[row]  = now                                  (row = row_base[c]+n)
 *   decay = 1 reproduces core/single/cache_scheduling.py:69-73; decay = 0.95
 *   the decay-first variant (core/single/module/pikv_scheduling.py:119-130).
 *   If write_probs != 0 scores is overwritten with the probabilities.
 *   importance_out [n_caches, score_stride] float or NULL receives the summed
 *   probabilities.  head_stats [n_caches, n_q_heads, 2] float receives the final
 *   (max, sum of exp(score - max)) of every head; pikv_attend_values takes it.
 *   With write_probs == 0 and row_acc, row_ts, importance_out all NULL only the
 *   statistics are computed (for a pikv_attend_values call that accumulates itself). */
int pikv_h2o_accumulate(float* scores, const float* tile_max,
                        const float* tile_sum, int n_q_heads,
                        const int64_t* cache_row_base,
                        const int32_t* cache_fill, int n_caches,
                        int64_t max_len, int64_t score_stride,
                        float decay, float now, int write_probs,
                        float* row_acc, float* row_ts, float* importance_out,
                        float* head_stats, void* stream);

/* Attention output over the compressed V cache:
 *   out[c,h,:] = sum_{n < cache_fill[c]} p[c,h,n] * dequant(V[c,n,h/rep,:])
 *   p = exp(scores - head_stats[c,h,0]) / head_stats[c,h,1]   (head_stats != NULL:
 *       raw scores of pikv_gather_dequant_scores + the statistics that
 *       pikv_h2o_accumulate leaves in its head_stats argument), or
 *   p = scores                                              (head_stats == NULL:
 *       scores already hold probabilities, e.g. after write_probs = 1).
 * Replaces: context = torch.matmul(attention_probs, v)
 *   (core/single/pikv_attention.py:188) on a dequantised copy of the cache.
 *   out [n_caches, n_q_heads, head_dim] float; V planes as in the pool layout;
 *   workspace: pikv_attend_workspace_bytes(...) bytes (partial sums of token
 *   ranges, added in a fixed order), 256-byte aligned.  Shape limits as for
 *   pikv_gather_dequant_scores.
 *   row_acc / row_ts (each may be NULL): the H2O bookkeeping of pikv_h2o_accumulate
 *   on the same probabilities, done in the same pass over the scores:
 *   acc[row] = acc[row]*decay + sum_h p[c,h,n], ts[row] = now
 *   (core/single/cache_scheduling.py:69-73). */
int pikv_attend_values(const float* scores, const float* head_stats,
                       int64_t score_stride,
                       const void* v_codes, const void* v_scale, const void* v_zero,
                       int scheme, int group,
                       int n_kv_heads, int n_q_heads, int head_dim,
                       const int64_t* cache_row_base, const int32_t* cache_fill,
                       int n_caches, int64_t max_len,
                       float decay, float now, float* row_acc, float* row_ts,
                       float* out, void* workspace, int64_t workspace_bytes,
                       void* stream);
int64_t pikv_attend_workspace_bytes(int n_caches, int n_q_heads, int head_dim,
                                    int64_t max_len);

/* The whole decode read in one call: scores of one query per cache against the
 * compressed K rows, softmax over each cache's tokens, attention output over the
 * compressed V rows, and the H2O bookkeeping of the same probabilities:
 *   s[c,h,n]  = dot(q[c,h,:], dequant(K[c,n,h/rep,:])) * scale_qk        n < min(cache_fill[c], max_len)
 *   p[c,h,:]  = softmax_n(s[c,h,:])
 *   out[c,h,:] = sum_n p[c,h,n] * dequant(V[c,n,h/rep,:])
 *   acc[row] = acc[row]*decay + sum_h p[c,h,n];  ts[row] = now          (row_acc / row_ts may be NULL)
 * Replaces: matmul(q, k^T)/sqrt(head_dim), softmax(dim=-1), matmul(probs, v)
 *   (core/single/pikv_attention.py:123,163,188) on dequantised copies of the cache, and
 *   H2OScheduler.update_attention_scores (core/single/cache_scheduling.py:69-73).
 * Same results as pikv_gather_dequant_scores + pikv_h2o_accumulate + pikv_attend_values
 * (to the float tolerance of those), but the score matrix never leaves the library.
 * Caches of 2 to 8 kv heads of 128 dimensions take ONE pass over K and V (scores, running
 * softmax and attention output per 64-token tile, no score matrix at all; exp(score - running
 * maximum) leaves the pass as a half per head and token for the accumulators only): 4-bit
 * codes in groups of 32 with up to 4 bf16 or float32 query heads per kv head (with row_acc:
 * exactly 4, on 3 or more kv heads) or 5 to 8 bf16 ones (3 or more kv heads), 8-bit codes
 * with a scale per kv head or coarser and up to 8 bf16 or float32 ones (with row_acc: 2 to 8);
 * float32 queries go in as two bf16 limbs.  Otherwise, for
 * 4-bit caches with group 32, rows that are 1 to 8 slabs of 128 dimensions, or whole groups
 * of 8 kv heads of 128 dimensions (a slab is one kv
 * head of 128 dimensions, two of 64 or four of 32) and up to 8 query heads per slab (5 to 8
 * heads with float32 queries: up to 7 slabs; more than 8 bf16 query heads per slab on rows of up to
 * 4 slabs, in launches of eight heads of each kernel) the two matrix-core kernels exchange exp(score - tile max)
 * with a tile's heads side by side, so that both sides stream contiguous 8 KB runs instead
 * of the 256-byte pieces of a [head][token] score matrix; every other format runs the three
 * steps with float scores in the workspace.
 *   q [n_caches, n_q_heads, head_dim] q_dtype; out [n_caches, n_q_heads, head_dim] float;
 *   planes and shape limits as for the three entry points above;
 *   workspace: pikv_decode_attend_workspace_bytes(...) bytes, 256-byte aligned. */
int pikv_decode_attend(const void* k_codes, const void* k_scale, const void* k_zero,
                       const void* v_codes, const void* v_scale, const void* v_zero,
                       int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim,
                       const void* q, int q_dtype, float scale_qk,
                       const int64_t* cache_row_base, const int32_t* cache_fill,
                       int n_caches, int64_t max_len, float decay, float now,
                       float* row_acc, float* row_ts, float* out,
                       void* workspace, int64_t workspace_bytes, void* stream);
int64_t pikv_decode_attend_workspace_bytes(int n_caches, int n_q_heads, int head_dim,
                                           int64_t max_len);

/* ------------------------------------------------------------------------
 * K4  eviction top-k + stable in-place compaction
 * Replaces: H2OScheduler.select_eviction_candidates
 *   (core/single/cache_scheduling.py:75-99), LRUScheduler's
 *   (core/single/cache_scheduling.py:262-285), and the manager's compaction
 *   keep = where(~mask); cache[:m] = cur[keep]
 *   (core/single/cache_scheduling.py:418-424); native precedent
 *   launch_cache_compaction_kernel (pikv_scheduling_kernel.cu:633-654).
 *
 *   For each cache c with len = cache_fill[c]:
 *     H2O: keep = top-n_heavy[c] of row_acc  UNION  top-n_recent[c] of row_ts
 *     LRU: evict the n_evict[c] rows with the smallest row_ts
 *          (n_heavy is read as n_evict; n_recent is ignored)
 *   keep_flag  [rows_total] uint8  : 1 for survivors (written for n < len)
 *   keep_index [rows_total] int32  : ascending cache-local indices of the
 *                                    survivors, at [row_base[c] .. +new_len)
 *   new_len    [n_caches]  int32   : number of survivors
 *   n_heavy/n_recent are per-cache DEVICE arrays so that no host read of
 *   cache_fill is needed; pikv_h2o_budget fills them from the ratios.
 *   max_len >= max_c cache_fill[c] sizes the launch.  workspace (optional,
 *   pikv_evict_workspace_bytes(n_caches, max_len) bytes, 256-byte aligned) lets long
 *   caches be selected by several blocks each; with workspace == NULL one block
 *   serves a cache whatever its length.  Both forms give identical results.
 * ---------------------------------------------------------------------- */
int pikv_evict_select(int policy, const float* row_acc, const float* row_ts,
                      const int64_t* cache_row_base, const int32_t* cache_fill,
                      const int32_t* n_heavy, const int32_t* n_recent,
                      int n_caches, int64_t max_len,
                      uint8_t* keep_flag, int32_t* keep_index, int32_t* new_len,
                      void* workspace, int64_t workspace_bytes, void* stream);
int64_t pikv_evict_workspace_bytes(int n_caches, int64_t max_len);

/* n_heavy[c] = max(1,int(len*heavy_ratio)); n_recent[c] = max(1,int(len*recent_ratio))
 * with len = cache_fill[c] and the product evaluated in double precision as
 * Python does (core/single/cache_scheduling.py:83-84). */
int pikv_h2o_budget(const int32_t* cache_fill, int n_caches,
                    double heavy_ratio, double recent_ratio,
                    int32_t* n_heavy, int32_t* n_recent, void* stream);

/* Move surviving rows to the front of every cache, in place and in ascending
 * order, for up to PIKV_MAX_PLANES planes (codes, scales, zeros, acc, ts ...),
 * then set cache_fill[c] = new_len[c].
 *   plane_ptrs_host  [n_planes] device pointers (the ARRAY itself is on the
 *                    host); plane_row_bytes_host [n_planes] bytes per row
 *                    (any positive width; rows are moved in the widest units
 *                    their width is a multiple of, up to 16 bytes). */
#define PIKV_MAX_PLANES 10
int pikv_compact_rows(void* const* plane_ptrs_host,
                      const int64_t* plane_row_bytes_host, int n_planes,
                      const int64_t* cache_row_base, const int32_t* keep_index,
                      const int32_t* new_len, int32_t* cache_fill,
                      int n_caches, void* stream);

/* ------------------------------------------------------------------------
 * API-compatible fake quantisation of QuantizedCompressor.forward
 * Replaces: core/single/pikv_compression.py:474-506 - min/max over ALL rows
 *   of each block of `group` columns, asymmetric, output = dequantised floats.
 *   x, out [N,H] float; stats [H/group (rounded up), 4] float workspace/out:
 *   (min, max, scale, zero) per column block; sq_err [ceil(H/group)] float:
 *   mean squared error per block (the reference's quantization_error is the
 *   value of the LAST block processed).
 * ---------------------------------------------------------------------- */
int pikv_fakequant_colblocks(const float* x, int64_t N, int H, int group,
                             int bits, int symmetric, float* out,
                             float* stats, float* sq_err,
                             void* workspace, int64_t workspace_bytes,
                             void* stream);
int64_t pikv_fakequant_workspace_bytes(int64_t N, int H, int group);

/* The same with parameters fixed beforehand: out = (clamp(round(x/scale + zero)) - zero)*scale
 * with ONE (scale, zero) for every element.
 * Replaces: QuantizedCompressor._quantize with dynamic_quantization=False
 *   (core/single/pikv_compression.py:430-472): the first tensor the module sees fixes scale
 *   and zero_point, every later one is quantised with them.
 *   preset [4] float (device): a (min, max, scale, zero) row as pikv_fakequant_colblocks
 *   writes it; only scale and zero are read.  sq_err, workspace as above (group only
 *   sets the column blocks that the errors are reported for). */
int pikv_fakequant_preset(const float* x, int64_t N, int H, int group,
                          int bits, int symmetric, const float* preset,
                          float* out, float* sq_err,
                          void* workspace, int64_t workspace_bytes,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PIKV_HIP_H */
