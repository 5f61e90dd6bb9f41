// K1: fused router - gate projection, logit scaling/mask, softmax, top-k,
// renormalisation - and the capacity-slot pass.
//
// Three forms of the gate projection (skinny: E <= 64 outputs per token):
//   bf16, >= 32768 tokens ... router_gate_lds_kernel: token rows staged through LDS in whole
//                             256/512-byte pieces, matrix cores, one token per lane in the tail
//   bf16, fewer tokens ...... router_gate_mfma_kernel: matrix cores, k-steps dealt to the
//                             wavefronts, operands straight from global memory
//   fp32, or H % 32 != 0 .... router_gate_kernel, vector ALU:
// a wavefront owns a tile of TPW = 64/EPAD tokens (EPAD = E rounded up to
// 8/16/32/64).  Lanes stride the hidden dimension with 128-bit loads; every lane
// keeps TPW*EPAD = 64 partial sums, so a slice of W fetched once (from L2) is
// used for all TPW tokens.  The 64 partial-sum vectors are then reduced with a
// 63-shuffle transpose-reduction that leaves lane l holding the finished logit of
// (token l / EPAD, expert l % EPAD): each token's experts sit in EPAD adjacent
// lanes and the whole tail (softmax, k rounds of arg-max with lowest-index
// tie-break via ballot, renormalisation) runs on those lane groups without LDS.
//
// Capacity slots: deterministic three-step histogram / scan / rank over the
// assignments in token-major order (integer LDS atomics only feed counts, whose
// value does not depend on arrival order).
#include <atomic>

#include "common.hpp"

namespace pikv {

constexpr int kSlotChunk = 512;  // assignments per block in the slot pass
constexpr int64_t kSlotSelfPrefixWords = 8192;  // chunks x experts up to which a rank block sums the earlier chunks itself
constexpr int kRowsTailMinK = 2;  // standalone tail, 33-64 experts: lanes per token instead of per expert from this k on

struct TailParams {
  const float* bias;
  const float* expert_scale;
  const float* expert_mask;
  float temperature;
  float renorm_eps;
  int use_softmax;
  int arithmetic;  // PIKV_ROUTER_SINGLE | PIKV_ROUTER_MODULE
  int E;
  int k;
  int64_t T;
  float* probs;
  float* logits_out;
  int32_t* topk_idx;
  float* topk_w;
};

// 64 values per lane -> lane l ends with the wave-wide sum of v[l].  Each step
// halves the live values: a lane keeps the half selected by one bit of its lane
// id and receives the partner's partial sums for that half.
template <int HALF>
__device__ __forceinline__ void transpose_reduce_step(float (&v)[64], int lane) {
  const bool up = (lane & HALF) != 0;
#pragma unroll
  for (int i = 0; i < HALF; ++i) {
    const float keep = up ? v[i + HALF] : v[i];
    const float send = up ? v[i] : v[i + HALF];
    v[i] = keep + __shfl_xor(send, HALF, PIKV_WAVE);
  }
}
__device__ __forceinline__ float wave_transpose_reduce(float (&v)[64], int lane) {
  transpose_reduce_step<32>(v, lane);
  transpose_reduce_step<16>(v, lane);
  transpose_reduce_step<8>(v, lane);
  transpose_reduce_step<4>(v, lane);
  transpose_reduce_step<2>(v, lane);
  transpose_reduce_step<1>(v, lane);
  return v[0];
}

// Bias, temperature, per-expert scale and mask penalty of expert e, in the order of the
// chosen copy of the reference's routers.  The per-expert numbers are loaded once per lane.
struct ExpertConsts {
  float bias, scale, penalty;
};
// Absent vectors load as the neutral elements -0 (x + -0 == x bit for bit), 1 and -0.
__device__ __forceinline__ ExpertConsts load_expert_consts(int e, const TailParams& p) {
  ExpertConsts c{-0.f, 1.f, -0.f};
  if (e < p.E) {
    if (p.bias) c.bias = p.bias[e];
    if (p.expert_scale) c.scale = p.expert_scale[e];
    if (p.expert_mask)
      c.penalty = (1.0f - p.expert_mask[e]) * (p.arithmetic == PIKV_ROUTER_MODULE
                                                    ? -3.4028234663852886e38f  // finfo(float32).min
                                                    : -1e9f);
  }
  return c;
}
__device__ __forceinline__ float final_logit(float lg, const ExpertConsts& c, const TailParams& p) {
  if (p.bias) lg = lg + c.bias;
  if (p.arithmetic == PIKV_ROUTER_MODULE) {
    // core/single/module/pikv_routing.py:596-600, :133-134
    if (p.expert_scale) lg = lg * c.scale;
    if (p.temperature != 1.0f) lg = lg / p.temperature;
    if (p.expert_mask) lg = lg + c.penalty;
  } else {
    // core/single/pikv_routing.py:653-656, :68-70
    if (p.temperature != 1.0f) lg = lg / p.temperature;
    if (p.expert_scale) lg = lg * c.scale;
    if (p.expert_mask) lg = lg + c.penalty;
  }
  return lg;
}
// The same without branches, for loops over many rows: MODE 0 = temperature 1 (both orders
// coincide), 1 = divide then scale (single/), 2 = scale then divide (module/).
template <int MODE>
__device__ __forceinline__ float final_logit_rows(float lg, const ExpertConsts& c, float temperature) {
  lg = lg + c.bias;
  if (MODE == 1) lg = lg / temperature;
  lg = lg * c.scale;
  if (MODE == 2) lg = lg / temperature;
  return lg + c.penalty;
}
__device__ __forceinline__ int final_logit_mode(const TailParams& p) {
  return p.temperature == 1.0f ? 0 : (p.arithmetic == PIKV_ROUTER_MODULE ? 2 : 1);
}
__device__ __forceinline__ float final_logit(float lg, int e, const TailParams& p) {
  return final_logit(lg, load_expert_consts(e, p), p);
}

// Lane holds the raw logit of (token t, expert e); groups of EPAD adjacent lanes
// form one token.  Writes probs / top-k for the token.
// The top-k is taken on what the reference hands to torch.topk - the float32 probabilities
// (core/single/pikv_routing.py:73-76), or the final logits without the softmax
// (core/single/pikv_kernels.py:97) - in the total order (value descending, expert index
// ascending, NaN last): two distinct logits whose probabilities round to the same float32
// are a tie, and the lower expert wins it.
// NTOK independent token groups go through the steps side by side: every step is a
// chain of dependent cross-lane operations, and the chains of different tokens fill each
// other's wait states.
template <int EPAD, int NTOK>
__device__ __forceinline__ void router_tail_multi(float (&lg)[NTOK], const int64_t (&t)[NTOK], int e, int lane,
                                                  const TailParams& p) {
  bool valid[NTOK];
#pragma unroll
  for (int n = 0; n < NTOK; ++n) {
    valid[n] = (t[n] < p.T) && (e < p.E);
    if (valid[n]) {
      lg[n] = final_logit(lg[n], e, p);
      if (p.logits_out) p.logits_out[t[n] * p.E + e] = lg[n];
    } else {
      lg[n] = -__builtin_inff();
    }
  }
  float carried[NTOK];
#pragma unroll
  for (int n = 0; n < NTOK; ++n) carried[n] = lg[n];
  if (p.use_softmax) {
    float m[NTOK], ex[NTOK], sum[NTOK];
#pragma unroll
    for (int n = 0; n < NTOK; ++n) m[n] = group_max_dpp(lg[n], EPAD);
#pragma unroll
    for (int n = 0; n < NTOK; ++n) ex[n] = valid[n] ? expf(lg[n] - m[n]) : 0.f;
#pragma unroll
    for (int n = 0; n < NTOK; ++n) sum[n] = group_sum_dpp(ex[n], EPAD);
#pragma unroll
    for (int n = 0; n < NTOK; ++n) {
      carried[n] = ex[n] / sum[n];
      if (valid[n] && p.probs) p.probs[t[n] * p.E + e] = carried[n];
    }
  }

  const int gstart = lane & ~(EPAD - 1);
  const uint64_t gmask = (EPAD == 64) ? ~0ull : (((1ull << EPAD) - 1ull) << gstart);
  bool remaining[NTOK];
  int my_idx[NTOK];
  float my_val[NTOK], wsum[NTOK];  // wsum: sum of the selected values, in selection order
#pragma unroll
  for (int n = 0; n < NTOK; ++n) {
    remaining[n] = valid[n];
    my_idx[n] = 0;
    my_val[n] = 0.f;
    wsum[n] = 0.f;
  }
  for (int j = 0; j < p.k; ++j) {
    float key[NTOK], mx[NTOK];
#pragma unroll
    for (int n = 0; n < NTOK; ++n) key[n] = remaining[n] ? carried[n] : -__builtin_inff();
#pragma unroll
    for (int n = 0; n < NTOK; ++n) mx[n] = group_max_dpp(key[n], EPAD);
#pragma unroll
    for (int n = 0; n < NTOK; ++n) {
      uint64_t cand = __ballot(remaining[n] && key[n] == mx[n]) & gmask;
      if (cand == 0) cand = __ballot(remaining[n]) & gmask;  // only NaNs left
      int win = e;  // padding tokens (no candidates at all) stay harmless
      if (cand != 0) win = (int)__builtin_ctzll(cand) - gstart;
      float wv;
      if constexpr (EPAD == 64) {
        // one token per wavefront: the winner is wave-uniform
        wv = read_lane_f(carried[n], __builtin_amdgcn_readfirstlane(win));
      } else {
        wv = __shfl(carried[n], gstart + win, PIKV_WAVE);
      }
      wsum[n] = wsum[n] + wv;
      if (e == j) {
        my_idx[n] = win;
        my_val[n] = wv;
      }
      if (e == win) remaining[n] = false;
    }
  }
#pragma unroll
  for (int n = 0; n < NTOK; ++n) {
    if (p.use_softmax) {
      float sden = wsum[n];
      if (p.renorm_eps != 0.f) sden = sden + p.renorm_eps;
      my_val[n] = my_val[n] / sden;
    }
    if (t[n] < p.T && e < p.k) {
      p.topk_idx[t[n] * p.k + e] = my_idx[n];
      p.topk_w[t[n] * p.k + e] = my_val[n];
    }
  }
}

template <int EPAD>
__device__ __forceinline__ void router_tail_lanes(float lg, int64_t t, int e, int lane,
                                                  const TailParams& p) {
  float lgs[1] = {lg};
  const int64_t ts[1] = {t};
  router_tail_multi<EPAD, 1>(lgs, ts, e, lane, p);
}

template <int EPAD, int DT>
__global__ __launch_bounds__(256) void router_gate_kernel(const void* __restrict__ x,
                                                          const void* __restrict__ w, int H,
                                                          TailParams p) {
  constexpr int TPW = 64 / EPAD;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t tile = (int64_t)blockIdx.x * 4 + wave;
  const int64_t tok0 = tile * TPW;
  if (tok0 >= p.T) return;  // whole wavefront leaves together

  float acc[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) acc[i] = 0.f;

  for (int h0 = 0; h0 < H; h0 += 512) {
    const int h = h0 + lane * 8;
    if (h < H) {
      float xs[TPW][8];
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        if (tok0 + t < p.T) {
          load_as_float<DT, 8>(x, (tok0 + t) * H + h, xs[t]);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) xs[t][i] = 0.f;
        }
      }
#pragma unroll
      for (int e = 0; e < EPAD; ++e) {
        if (e < p.E) {
          float we[8];
          load_as_float<DT, 8>(w, (int64_t)e * H + h, we);
#pragma unroll
          for (int t = 0; t < TPW; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[t * EPAD + e] = fmaf(xs[t][i], we[i], acc[t * EPAD + e]);
        }
      }
    }
  }
  const float lg = wave_transpose_reduce(acc, lane);
  router_tail_lanes<EPAD>(lg, tok0 + lane / EPAD, lane % EPAD, lane, p);
}

// n_parts > 1: logits_a holds n_parts slabs [T,E] of partial sums (the split gate
// projection), added in slab order.
template <int EPAD>
__global__ __launch_bounds__(256) void router_tail_kernel(const float* __restrict__ la,
                                                          const float* __restrict__ lb,
                                                          const uint8_t* __restrict__ select,
                                                          TailParams p, int n_parts = 1) {
  constexpr int TPW = 64 / EPAD;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t tile = (int64_t)blockIdx.x * 4 + wave;
  const int64_t t = tile * TPW + lane / EPAD;
  const int e = lane % EPAD;
  if (tile * TPW >= p.T) return;
  float lg = 0.f;
  if (t < p.T && e < p.E) {
    const bool use_a = (lb == nullptr) || (select == nullptr) || (select[t] != 0);
    lg = use_a ? la[t * p.E + e] : lb[t * p.E + e];
    for (int s = 1; s < n_parts; ++s) lg = lg + la[((int64_t)s * p.T + t) * p.E + e];
  }
  router_tail_lanes<EPAD>(lg, t, e, lane, p);
}

// ---- bf16 gate projection on the matrix cores ------------------------------------
// Measured on the prefill workload (T=32768, H=4096, E=8) the VALU kernel above
// issues 25.8 M wavefront instructions - 42 us of pure issue time against 34 us of
// HBM time - and has too few wavefronts to hide latency.  For bf16 inputs the
// contraction over H therefore runs as v_mfma_f32_16x16x32_bf16: a block owns 16 MT
// tokens, its wavefronts interleave over 32-wide slices of H (so the block
// reads 64 WAVES contiguous bytes of each token row per sweep), every wavefront keeps
// one 16x16 fp32 tile per token tile and group of 16 experts, and the partial tiles meet in LDS.
// The kernel stays HBM-bound up to E = 64 (the MFMA work is ~1/7 of the HBM time
// there), which the VALU formulation cannot be.
typedef __bf16 pikv_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pikv_f32x4 __attribute__((ext_vector_type(4)));


// Gate weights re-laid for the matrix-core kernel: wb[step][expert (padded to EP)][32 k]
// so that the B operands of one k-step are EP*64 contiguous bytes.  Rows of the
// original [E,H] layout are a multiple of 2 KB apart for the usual hidden sizes and
// would all fall into the same L2 channel.
// (row_bytes = bytes of a row of w: a k-step is 64 bytes of it, 32 bf16 or 16 float32 values)
__global__ __launch_bounds__(256) void gate_weight_relayout_kernel(const void* __restrict__ w, int64_t row_bytes,
                                                                  int E, int EP, uint4* __restrict__ wb) {
  const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;  // 16-byte chunk of wb
  const int64_t total = (row_bytes / 64) * EP * 4;
  if (chunk >= total) return;
  const int kg = (int)(chunk & 3);
  const int e = (int)((chunk >> 2) % EP);
  const int64_t st = (chunk >> 2) / EP;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (e < E) v = ld16(reinterpret_cast<const char*>(w) + (int64_t)e * row_bytes + st * 64 + kg * 16);
  wb[chunk] = v;
}

// NT 16-expert tiles (1, 2 or 4) x MT 16-token tiles per block; WAVES wavefronts share the k-steps
// PARTIAL (short token streams): blockIdx.y picks a slice of the k-steps, and the block
// writes its partial logits to part[slice][T][E] instead of running the tail - with a few
// dozen tokens a single block would walk all of H alone, one load latency per k-step.
// DIRECT (up to 16 experts): wb is the caller's [E, H] weight matrix itself, lane (expert m, kg)
// reads its 16 bytes of a k-step from row m.  Every block starts its walk at another k-step (below),
// so the rows - a multiple of 2 KB apart - no longer meet in one L2 channel at the same time, and the
// launch that re-lays the weights is saved (config[1], router call: 65.2 -> 63.0 us).
// F32IN: float32 activations and weights, multiplied exactly by v_mfma_f32_16x16x4_f32.  A k-step is
// 16 values - the same 64 bytes of a row as 32 bf16 - and a lane's four floats feed four instructions:
// lane (m, kg) holds k = k0 + 4 kg + j for instruction j on both operands, so the four cover all 16.
template <int NT, int MT, int WAVES, bool PARTIAL = false, bool DIRECT = false, bool F32IN = false>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(2))) void router_gate_mfma_kernel(
    const void* __restrict__ x, const void* __restrict__ wb, int H, TailParams p, float* __restrict__ part = nullptr,
    int steps_per_slice = 0) {
  static_assert(!DIRECT || !PARTIAL, "direct weights: whole rows per block");
  constexpr int ES = F32IN ? 4 : 2;        // bytes per element
  constexpr int KL = 16 / ES;              // elements of a lane's 16 bytes
  constexpr int EP = 16 * NT;
  constexpr int TB = 16 * MT;  // tokens per block
  // Partial sums of the wavefronts: one slab each, or - when those would not leave room
  // for two blocks per compute unit - a single slab that the wavefronts add to in turn
  // (same order of additions either way).
  constexpr bool SEQ = WAVES * TB * EP * 4 > 32 * 1024;
  __shared__ float red[SEQ ? 1 : WAVES][TB][EP];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t tok0 = (int64_t)blockIdx.x * TB;
  const int m = lane & 15;    // token row of the A operand / expert column of B and C
  const int kg = lane >> 4;   // which 8 of the 32 k-values this lane feeds
  const char* xrow[MT];
  bool tok_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    tok_ok[mt] = tok0 + mt * 16 + m < p.T;
    xrow[mt] = reinterpret_cast<const char*>(x) +
               ((tok_ok[mt] ? tok0 + mt * 16 + m : 0) * (int64_t)H + kg * KL) * ES;
  }
  const char* wlane = DIRECT ? reinterpret_cast<const char*>(wb) + ((int64_t)(m < p.E ? m : 0) * H + kg * KL) * ES
                             : reinterpret_cast<const char*>(wb) + (m * 32 + kg * 8) * 2;
  pikv_f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};

  // the k-steps are dealt round-robin to the wavefronts; each keeps UN steps in flight
  int steps = H / (4 * KL), step0 = 0;
  if constexpr (PARTIAL) {
    step0 = blockIdx.y * steps_per_slice;
    steps = step0 + steps_per_slice < steps ? step0 + steps_per_slice : steps;
  }
  constexpr int UN = (MT >= 8) ? 1 : (MT + NT > 4) ? 2 : 4;  // registers: 2 wavefronts per SIMD must fit
  // Every block starts its walk along the rows at another offset (a hash of the block index, in
  // whole iterations, wrapping around): with all blocks walking front to back together the whole
  // chip reads the same 1 KB window of its 8 KB rows at any time, which loads the memory channels
  // unevenly (config[1]: router call 73.5 -> 70 us).  The pattern matters: offsets that are small
  // multiples of the block index moved the time both ways (73 ... 90 us), a scattered assignment or
  // one that changes every 64 blocks gained.  The order of a wavefront's additions, and so the last
  // bits of a logit, depend on the block a token falls into.
  const int n_it = (steps - step0 + WAVES * UN - 1) / (WAVES * UN);
  const int rot = PARTIAL ? 0 : (int)(((blockIdx.x * 0x9E3779B1u) >> 16) % (unsigned)n_it);
  struct Ops {
    uint4 av[UN][MT], bv[UN][NT];
  };
  auto load_ops = [&](int it, Ops& o) {
    int itr = it + rot;
    if (itr >= n_it) itr -= n_it;
    const int st0 = step0 + wave + itr * (WAVES * UN);
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int st = st0 + u * WAVES;
      const bool ok = st < steps;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        o.av[u][mt] = (ok && tok_ok[mt]) ? ld16(xrow[mt] + (int64_t)st * 64) : make_uint4(0, 0, 0, 0);
      // (columns of experts that do not exist are zero in the re-laid weights: not loaded at all)
#pragma unroll
      for (int t = 0; t < NT; ++t)
        o.bv[u][t] = (ok && t * 16 + m < p.E)
                         ? ld16(DIRECT ? wlane + (int64_t)st * 64 + (int64_t)t * 16 * H * ES
                                       : wlane + ((int64_t)st * EP + t * 16) * 64)
                         : make_uint4(0, 0, 0, 0);
    }
  };
  if constexpr (F32IN) {
    // The float32 form is bound by the matrix instruction (32 cycles each): the operands of the next
    // trip are asked for before this trip's instructions, or the two wavefronts of a SIMD spend half
    // their time waiting for loads (64 experts: 923 us without).  The four instructions of a lane's
    // 16 bytes are outermost: neighbours in the issue order write different accumulators.
    Ops cur, nxt;
    load_ops(0, cur);
    for (int it = 0; it < n_it; ++it) {
      if (it + 1 < n_it) load_ops(it + 1, nxt);
#pragma unroll
      for (int u = 0; u < UN; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              const uint4 a4 = cur.av[u][mt], b4 = cur.bv[u][t];
              const uint32_t af = j == 0 ? a4.x : j == 1 ? a4.y : j == 2 ? a4.z : a4.w;
              const uint32_t bf = j == 0 ? b4.x : j == 1 ? b4.y : j == 2 ? b4.z : b4.w;
              acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(af), __uint_as_float(bf), acc[mt][t], 0, 0, 0);
            }
      if (it + 1 < n_it) cur = nxt;
    }
  } else {
    for (int it = 0; it < n_it; ++it) {
      Ops o;
      load_ops(it, o);
#pragma unroll
      for (int u = 0; u < UN; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(pikv_bf16x8, o.av[u][mt]), __builtin_bit_cast(pikv_bf16x8, o.bv[u][t]),
                acc[mt][t], 0, 0, 0);
    }
  }
  // C layout: lane holds rows 4*(lane/16)+i, column lane%16 of each tile.
  if constexpr (SEQ) {
    for (int w2 = 0; w2 < WAVES; ++w2) {
      if (wave == w2) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float* cell = &red[0][mt * 16 + 4 * kg + i][t * 16 + m];
              *cell = (w2 == 0 ? 0.f : *cell) + acc[mt][t][i];
            }
      }
      __syncthreads();
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][mt * 16 + 4 * kg + i][t * 16 + m] = acc[mt][t][i];
    __syncthreads();
  }
  if constexpr (PARTIAL) {
    float* dst = part + (int64_t)blockIdx.y * p.T * p.E;
    for (int i = threadIdx.x; i < TB * EP; i += WAVES * 64) {
      const int tl = i / EP, e = i % EP;
      const int64_t t = tok0 + tl;
      if (t < p.T && e < p.E) {
        float v = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < (SEQ ? 1 : WAVES); ++w2) v += red[w2][tl][e];
        dst[t * p.E + e] = v;
      }
    }
    return;
  }
  // Wavefront w finishes tokens TW*w .. TW*w+TW-1: lane -> (token, expert) with the
  // experts of a token in EP adjacent lanes, as the tail expects.
  constexpr int TW = TB / WAVES;  // tokens finished by one wavefront
  constexpr int TPC = 64 / EP;         // tokens per tail call
  constexpr int CALLS = (TW + TPC - 1) / TPC;
  constexpr int NTOK = CALLS >= 4 ? 4 : CALLS >= 2 ? 2 : 1;  // token groups finished side by side
  static_assert(CALLS % NTOK == 0, "calls come in whole bundles");
#pragma unroll
  for (int c0 = 0; c0 < CALLS; c0 += NTOK) {
    float lg[NTOK];
    int64_t tt[NTOK];
    const int e = lane % EP;
#pragma unroll
    for (int n = 0; n < NTOK; ++n) {
      const int tw = (c0 + n) * TPC + lane / EP;
      const int tl = TW * wave + tw;
      const bool in_range = tw < TW;
      lg[n] = 0.f;
      if (in_range) {
#pragma unroll
        for (int w2 = 0; w2 < (SEQ ? 1 : WAVES); ++w2) lg[n] += red[w2][tl][e];
      }
      // lanes beyond this wavefront's tokens present an out-of-range token
      tt[n] = in_range ? tok0 + tl : p.T;
    }
    router_tail_multi<EP, NTOK>(lg, tt, e, lane, p);
  }
}

// ---- one token per LANE: softmax and top-k of 64 logits held in LDS ------------------
// A cross-lane arg-max round costs ~27 instructions per token and round; with a token per
// lane the same work is compare-exchanges on registers, 64 tokens per instruction.
// Order key: (float order with -0 = +0 and NaN below -inf, then the LOWER expert first)
// packed as one 64-bit integer, larger = earlier.  0 marks a padding column (below NaN).
__device__ __forceinline__ uint64_t lane_topk_key(float v, int e) {
  uint32_t k;
  if (v != v) {
    k = 1u;
  } else {
    const uint32_t u = __float_as_uint(v + 0.0f);  // -0 + 0 = +0
    k = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // >= 0x007fffff (-inf)
  }
  return ((uint64_t)k << 32) | (uint32_t)(63 - e);
}
__device__ __forceinline__ void ce_desc(uint64_t& a, uint64_t& b) {
  const bool sw = b > a;
  const uint64_t hi = sw ? b : a;
  b = sw ? a : b;
  a = hi;
}
// 19-comparator network for eight keys, descending
__device__ __forceinline__ void sort8_desc(uint64_t (&v)[8]) {
  ce_desc(v[0], v[2]); ce_desc(v[1], v[3]); ce_desc(v[4], v[6]); ce_desc(v[5], v[7]);
  ce_desc(v[0], v[4]); ce_desc(v[1], v[5]); ce_desc(v[2], v[6]); ce_desc(v[3], v[7]);
  ce_desc(v[0], v[1]); ce_desc(v[2], v[3]); ce_desc(v[4], v[5]); ce_desc(v[6], v[7]);
  ce_desc(v[2], v[4]); ce_desc(v[3], v[5]);
  ce_desc(v[1], v[4]); ce_desc(v[3], v[6]);
  ce_desc(v[1], v[2]); ce_desc(v[3], v[4]); ce_desc(v[5], v[6]);
}
// top = the eight largest of two descending lists: max(top[i], other[7-i]) is that set as a
// bitonic sequence, three half-cleaner stages sort it
__device__ __forceinline__ void merge_top8(uint64_t (&top)[8], const uint64_t (&other)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) top[i] = top[i] > other[7 - i] ? top[i] : other[7 - i];
  ce_desc(top[0], top[4]); ce_desc(top[1], top[5]); ce_desc(top[2], top[6]); ce_desc(top[3], top[7]);
  ce_desc(top[0], top[2]); ce_desc(top[1], top[3]); ce_desc(top[4], top[6]); ce_desc(top[5], top[7]);
  ce_desc(top[0], top[1]); ce_desc(top[2], top[3]); ce_desc(top[4], top[5]); ce_desc(top[6], top[7]);
}
// Sum of 16 values in the order of the DPP row reduction (pairs, quads, halves, row)
__device__ __forceinline__ float tree16(const float* a) {
  const float q0 = (a[0] + a[1]) + (a[2] + a[3]), q1 = (a[4] + a[5]) + (a[6] + a[7]);
  const float q2 = (a[8] + a[9]) + (a[10] + a[11]), q3 = (a[12] + a[13]) + (a[14] + a[15]);
  return (q0 + q1) + (q2 + q3);
}

// Largest of 16 values, NaN ignored unless all are NaN (fmaxf), as a balanced tree
__device__ __forceinline__ float max16(const float* a) {
  const float q0 = fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])), q1 = fmaxf(fmaxf(a[4], a[5]), fmaxf(a[6], a[7]));
  const float q2 = fmaxf(fmaxf(a[8], a[9]), fmaxf(a[10], a[11])), q3 = fmaxf(fmaxf(a[12], a[13]), fmaxf(a[14], a[15]));
  return fmaxf(fmaxf(q0, q1), fmaxf(q2, q3));
}
// The value a key was made from (keys of values >= +0 or NaN only: probabilities)
__device__ __forceinline__ float prob_of_key(uint64_t key) {
  const uint32_t k = (uint32_t)(key >> 32);
  return k == 1u ? __builtin_nanf("") : __uint_as_float(k & 0x7fffffffu);
}
// The eight largest of row[e0 .. e0 + 8*G) by (value desc, expert asc), sorted
template <int G>
__device__ __forceinline__ void top8_of_row(const float* row, int e0, int E, uint64_t (&top)[8]) {
#pragma unroll
  for (int g = 0; g < G; ++g) {
    uint64_t cur[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = e0 + 8 * g + i;
      cur[i] = e < E ? lane_topk_key(row[e], e) : 0ull;
    }
    sort8_desc(cur);
    if (g == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) top[i] = cur[i];
    } else {
      merge_top8(top, cur);
    }
  }
}

// Row `row` (stride RS floats) holds the final logits of one token, -inf in the padding
// columns e >= E.  Leaves the probabilities in the row and writes the token's top-k
// (without the softmax: the top-k of the logits, nothing else).
// Same arithmetic, in the same order, as the lane-per-expert tail: max, expf(l - max), the
// balanced sum, one division per expert; the top-k is then taken on the PROBABILITIES (what
// the reference passes to torch.topk, core/single/pikv_routing.py:73-76; value descending,
// lower expert first among equal float32 values, NaN last); weights = p / (sum of the
// selected p, largest first).
template <int EP, int RS>
__device__ __forceinline__ void lane_token_tail(float* row, int64_t t, const TailParams& p) {
  static_assert(EP == 16 || EP == 32 || EP == 64, "rows of 16, 32 or 64 columns");
  if (p.use_softmax) {
    float ex[EP];
#pragma unroll
    for (int e = 0; e < EP; ++e) ex[e] = row[e];
    float m = max16(ex);
    if constexpr (EP >= 32) m = fmaxf(m, max16(ex + 16));
    if constexpr (EP == 64) m = fmaxf(m, fmaxf(max16(ex + 32), max16(ex + 48)));
#pragma unroll
    for (int e = 0; e < EP; ++e) ex[e] = expf(ex[e] - m);  // padding: expf(-inf) = 0
    float sum = tree16(ex);
    if constexpr (EP == 32) sum = sum + tree16(ex + 16);
    if constexpr (EP == 64) sum = (sum + tree16(ex + 16)) + (tree16(ex + 32) + tree16(ex + 48));
#pragma unroll
    for (int e = 0; e < EP; ++e) row[e] = ex[e] / sum;
  }
  uint64_t top[8];
  top8_of_row<EP / 8>(row, 0, p.E, top);
  int idx[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) idx[j] = 63 - (int)(uint32_t)top[j];
  float pv[8], wsum = 0.f;
  if (p.use_softmax) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      pv[j] = j < p.k ? prob_of_key(top[j]) : 0.f;
      if (j < p.k) wsum = wsum + pv[j];
    }
    if (p.renorm_eps != 0.f) wsum = wsum + p.renorm_eps;
#pragma unroll
    for (int j = 0; j < 8; ++j) pv[j] = pv[j] / wsum;
  } else {  // raw top-k: the selected logits themselves
#pragma unroll
    for (int j = 0; j < 8; ++j) pv[j] = j < p.k ? row[idx[j]] : 0.f;
  }
  if (t >= p.T) return;
  // k values per token, contiguous over the lanes
  if (p.k == 8) {
    int4* oi = reinterpret_cast<int4*>(p.topk_idx + t * 8);
    float4* ow = reinterpret_cast<float4*>(p.topk_w + t * 8);
    oi[0] = make_int4(idx[0], idx[1], idx[2], idx[3]);
    oi[1] = make_int4(idx[4], idx[5], idx[6], idx[7]);
    ow[0] = make_float4(pv[0], pv[1], pv[2], pv[3]);
    ow[1] = make_float4(pv[4], pv[5], pv[6], pv[7]);
  } else if (p.k == 4) {
    *reinterpret_cast<int4*>(p.topk_idx + t * 4) = make_int4(idx[0], idx[1], idx[2], idx[3]);
    *reinterpret_cast<float4*>(p.topk_w + t * 4) = make_float4(pv[0], pv[1], pv[2], pv[3]);
  } else if (p.k == 2) {
    *reinterpret_cast<int2*>(p.topk_idx + t * 2) = make_int2(idx[0], idx[1]);
    *reinterpret_cast<float2*>(p.topk_w + t * 2) = make_float2(pv[0], pv[1]);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < p.k) {
        p.topk_idx[t * p.k + j] = idx[j];
        p.topk_w[t * p.k + j] = pv[j];
      }
  }
}

// The same for 64 columns with TWO lanes per token: `half` 0 takes experts 0..31, half 1 the
// rest.  The two maxima, then the two partial sums (two 16-trees each; the total is still
// (R0 + R1) + (R2 + R3)) meet in LDS; each lane divides its half, sorts its 32 probabilities,
// the two top-8 lists meet in LDS and half 0 merges them and writes the token's top-k.  Every
// thread of the block has to call this (three block barriers, one without the softmax);
// `active` says whether it holds a token.  xkeys: [8][2][TB] 64-bit keys (its first 2*TB
// words also carry the two maxima), xsum: [2][TB] floats.
template <int RS, int TB>
__device__ __forceinline__ void pair_token_tail(float* row, int half, int tl, bool active, int64_t t,
                                                const TailParams& p, uint64_t* xkeys, float* xsum) {
  uint64_t top[8];
  if (p.use_softmax) {  // uniform for the block
    float ex[32];
    float* xmax = reinterpret_cast<float*>(xkeys);
    if (active) {
#pragma unroll
      for (int e = 0; e < 32; ++e) ex[e] = row[32 * half + e];
      xmax[half * TB + tl] = fmaxf(max16(ex), max16(ex + 16));
    }
    __syncthreads();
    if (active) {
      const float m = fmaxf(xmax[tl], xmax[TB + tl]);
#pragma unroll
      for (int e = 0; e < 32; ++e) ex[e] = expf(ex[e] - m);  // padding: expf(-inf) = 0
      xsum[half * TB + tl] = tree16(ex) + tree16(ex + 16);
    }
    __syncthreads();  // also: every maximum has been read, xkeys may take the keys
    if (active) {
      const float sum = xsum[tl] + xsum[TB + tl];
#pragma unroll
      for (int e = 0; e < 32; ++e) row[32 * half + e] = ex[e] / sum;
    }
  }
  if (active) {
    top8_of_row<4>(row, 32 * half, p.E, top);
    if (half == 1) {
#pragma unroll
      for (int j = 0; j < 8; ++j) xkeys[j * TB + tl] = top[j];
    }
  }
  __syncthreads();
  if (!active || half != 0 || t >= p.T) return;
  {
    uint64_t other[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) other[j] = xkeys[j * TB + tl];
    merge_top8(top, other);
  }
  int idx[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) idx[j] = 63 - (int)(uint32_t)top[j];
  if (!p.use_softmax) {  // raw top-k: the selected logits themselves
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < p.k) {
        p.topk_idx[t * p.k + j] = idx[j];
        p.topk_w[t * p.k + j] = row[idx[j]];
      }
    return;
  }
  float pv[8], wsum = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    pv[j] = j < p.k ? prob_of_key(top[j]) : 0.f;
    if (j < p.k) wsum = wsum + pv[j];
  }
  if (p.renorm_eps != 0.f) wsum = wsum + p.renorm_eps;
#pragma unroll
  for (int j = 0; j < 8; ++j) pv[j] = pv[j] / wsum;
  if (p.k == 8) {
    int4* oi = reinterpret_cast<int4*>(p.topk_idx + t * 8);
    float4* ow = reinterpret_cast<float4*>(p.topk_w + t * 8);
    oi[0] = make_int4(idx[0], idx[1], idx[2], idx[3]);
    oi[1] = make_int4(idx[4], idx[5], idx[6], idx[7]);
    ow[0] = make_float4(pv[0], pv[1], pv[2], pv[3]);
    ow[1] = make_float4(pv[4], pv[5], pv[6], pv[7]);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < p.k) {
        p.topk_idx[t * p.k + j] = idx[j];
        p.topk_w[t * p.k + j] = pv[j];
      }
  }
}

// Long token streams: the classic tiled form.  A block owns TB tokens x EP (padded)
// experts; its 256 threads bring KS k-values of every token row (256 or 512 contiguous
// bytes per row, whole rows per load instruction) through registers into one of two LDS
// buffers while the matrix cores work on the other, one barrier per stage.  The 16 x 16
// output tiles are dealt to the four wavefronts along the experts first (64 experts:
// wavefront w owns expert tile w for all eight token tiles), so a wavefront's B operands
// (the re-laid weights, L2 hits) are at most 4 KB per stage and no partial sums have to
// meet at the end.  Rows are padded by 16 bytes: the 16 rows that one ds_read_b128 phase
// touches then start 4 banks apart.  Two blocks per compute unit (2 x 68 KB of LDS).
// Requires H % KS == 0 and the softmax form of the tail.  128 tokens x 64-wide stages (four
// blocks of 36 KB per compute unit) measured slower at 65536 tokens x 64 experts: 512 blocks
// are two per compute unit either way, and the narrower stage only halves the bytes each
// has in flight.
template <int EP, int TB, int KS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void router_gate_lds_kernel(
    const void* __restrict__ x, const void* __restrict__ wb, int H, TailParams p) {
  constexpr int WAVES = 4;
  constexpr int NT = EP / 16, MT = TB / 16;  // expert and token tiles of the block
  constexpr int WE = NT < WAVES ? NT : WAVES;  // wavefronts along the experts
  constexpr int WT = WAVES / WE;               // ... and along the tokens
  constexpr int MTW = MT / WT;                 // token tiles per wavefront (one expert tile each)
  static_assert(NT <= WAVES && MT % WT == 0, "one expert tile per wavefront");
  constexpr int ROW = KS * 2 + 16;  // bytes of one staged token row
  constexpr int BUF = TB * ROW;
  constexpr int CPR = KS / 8;        // 16-byte chunks per row
  constexpr int RPP = 256 / CPR;     // rows per staging pass
  constexpr int NP = TB / RPP;       // staging passes
  constexpr int NK = KS / 32;        // k-steps per stage
  constexpr int RS = EP + 1;         // floats per token row of the block's logits
  constexpr int LDS_BYTES = 2 * BUF > TB * RS * 4 ? 2 * BUF : TB * RS * 4;
  __shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];  // staging, then the block's logits
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform
  const int we = wave % WE, wt = wave / WE;
  const int m = lane & 15, kg = lane >> 4;
  const int64_t tok0 = (int64_t)blockIdx.x * TB;
  // staging: thread -> 16-byte chunk (tid % CPR) of rows tid/CPR + RPP i
  const int srow = tid / CPR, schunk = tid % CPR;
  const char* xsrc[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    int64_t t = tok0 + srow + RPP * i;
    if (t >= p.T) t = p.T - 1;  // rows past the end repeat the last token; the tail drops them
    xsrc[i] = reinterpret_cast<const char*>(x) + (t * (int64_t)H) * 2 + schunk * 16;
  }
  char* swrite = lds + srow * ROW + schunk * 16;
  const char* aread = lds + (wt * MTW * 16 + m) * ROW + kg * 16;
  const char* wlane = reinterpret_cast<const char*>(wb) + ((we * 16 + m) * 32 + kg * 8) * 2;
  pikv_f32x4 acc[MTW];
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt) acc[mt] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
  uint4 areg[NP], bcur[NK], bnext[NK];
  const int stages = H / KS;
#pragma unroll
  for (int i = 0; i < NP; ++i) areg[i] = ld16(xsrc[i]);
#pragma unroll
  for (int ks = 0; ks < NK; ++ks) bcur[ks] = ld16(wlane + (int64_t)ks * EP * 64);
#pragma unroll
  for (int i = 0; i < NP; ++i) *reinterpret_cast<uint4*>(swrite + i * RPP * ROW) = areg[i];
  __syncthreads();
  for (int s = 0; s < stages; ++s) {
    const int buf = (s & 1) * BUF;
    const bool more = s + 1 < stages;
    if (more) {
#pragma unroll
      for (int i = 0; i < NP; ++i) areg[i] = ld16(xsrc[i] + (int64_t)(s + 1) * (KS * 2));
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) bnext[ks] = ld16(wlane + (int64_t)(NK * (s + 1) + ks) * EP * 64);
    }
#pragma unroll
    for (int ks = 0; ks < NK; ++ks)
#pragma unroll
      for (int mt = 0; mt < MTW; ++mt) {
        const uint4 a = *reinterpret_cast<const uint4*>(aread + buf + mt * 16 * ROW + ks * 64);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, a),
                                                          __builtin_bit_cast(pikv_bf16x8, bcur[ks]),
                                                          acc[mt], 0, 0, 0);
      }
    if (more) {
      // the other buffer was last read before the barrier that ended the previous stage
#pragma unroll
      for (int i = 0; i < NP; ++i) *reinterpret_cast<uint4*>(swrite + (BUF - buf) + i * RPP * ROW) = areg[i];
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) bcur[ks] = bnext[ks];
    }
    __syncthreads();
  }
  // The block's logits, one row of RS floats per token (RS odd: a lane per token and a lane
  // per expert both walk the banks without conflicts).
  float* red = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[((wt * MTW + mt) * 16 + 4 * kg + i) * RS + we * 16 + m] = acc[mt][i];
  __syncthreads();
  // lanes = (token, expert), 64 / EP tokens side by side: bias / temperature / scale / mask,
  // the logits output
  constexpr int TW = TB / WAVES;  // tokens finished by one wavefront
  constexpr int TPP = 64 / EP;    // tokens per pass
  const int e = lane % EP, sub = lane / EP;
  {
    const ExpertConsts ec = load_expert_consts(e, p);
    const int mode = final_logit_mode(p);
    const bool col = e < p.E;
    for (int i = 0; i < TW; i += TPP) {
      const int tl = TW * wave + i + sub;
      const int64_t t = tok0 + tl;
      const float raw = red[tl * RS + e];
      float lg = mode == 0 ? final_logit_rows<0>(raw, ec, p.temperature)
                 : mode == 1 ? final_logit_rows<1>(raw, ec, p.temperature)
                             : final_logit_rows<2>(raw, ec, p.temperature);
      if (!col) lg = -__builtin_inff();
      if (p.logits_out && col && t < p.T) p.logits_out[t * p.E + e] = lg;
      red[tl * RS + e] = lg;
    }
  }
  __syncthreads();
  // lane = token: softmax and top-k of a whole row on registers
  if constexpr (EP == 64) {
    // two lanes per token; the exchange area lies behind the logits
    static_assert(TB * RS * 4 + 8 * 2 * TB * 8 + 2 * TB * 4 <= LDS_BYTES, "exchange area fits behind the logits");
    uint64_t* xkeys = reinterpret_cast<uint64_t*>(lds + ((TB * RS * 4 + 7) & ~7));
    float* xsum = reinterpret_cast<float*>(xkeys + 8 * 2 * TB);
    const int half = tid / TB, tl = tid % TB;
    pair_token_tail<RS, TB>(red + tl * RS, half, tl, tid < 2 * TB, tok0 + tl, p, xkeys, xsum);
  } else {
    if (tid < TB) lane_token_tail<EP, RS>(red + tid * RS, tok0 + tid, p);
  }
  __syncthreads();
  if (p.probs) {
    for (int i = 0; i < TW; i += TPP) {
      const int tl = TW * wave + i + sub;
      const int64_t t = tok0 + tl;
      if (e < p.E && t < p.T) p.probs[t * p.E + e] = red[tl * RS + e];
    }
  }
}

// Router tail on precomputed logits, 33-64 experts: 128 tokens per block go through LDS as
// [token][65] - read and written with a lane per expert (coalesced), finished with a lane
// per token.
template <int MODE>
__device__ __forceinline__ void tail_rows_stage(const float* __restrict__ la, const float* __restrict__ lb,
                                                uint32_t from_a, int64_t tbase, int wave, int lane,
                                                float* red, const TailParams& p) {
  constexpr int RS = 65;
  const ExpertConsts ec = load_expert_consts(lane, p);
  const bool col = lane < p.E;
  for (int i0 = 0; i0 < 32; i0 += 16) {
    float v[16];  // sixteen rows in flight per wavefront
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int64_t t = tbase + i0 + u;
      const float* src = ((from_a >> (i0 + u)) & 1u) ? la : lb;
      v[u] = (t < p.T && col) ? src[t * p.E + lane] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int tl = 32 * wave + i0 + u;
      const float lg = final_logit_rows<MODE>(v[u], ec, p.temperature);
      red[tl * RS + lane] = (tbase + i0 + u < p.T && col) ? lg : -__builtin_inff();
    }
  }
}

__global__ __launch_bounds__(256) void router_tail_rows_kernel(const float* __restrict__ la,
                                                               const float* __restrict__ lb,
                                                               const uint8_t* __restrict__ select,
                                                               TailParams p) {
  constexpr int TB = 128, RS = 65;
  __shared__ float red[TB * RS];
  __shared__ uint64_t xkeys[8 * 2 * TB];
  __shared__ float xsum[2 * TB];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: row addresses stay scalar
  const int64_t tok0 = (int64_t)blockIdx.x * TB;
  const int64_t tbase = tok0 + 32 * wave;  // first of the 32 tokens this wavefront stages
  uint32_t from_a = ~0u;                   // bit i: token tbase + i reads logits_a
  if (lb != nullptr && select != nullptr) {
    const int64_t t = tbase + (lane & 31);
    from_a = (uint32_t)__ballot(t < p.T ? select[t] != 0 : true);
  }
  const int mode = final_logit_mode(p);
  if (mode == 0) tail_rows_stage<0>(la, lb, from_a, tbase, wave, lane, red, p);
  else if (mode == 1) tail_rows_stage<1>(la, lb, from_a, tbase, wave, lane, red, p);
  else tail_rows_stage<2>(la, lb, from_a, tbase, wave, lane, red, p);
  __syncthreads();
  // two lanes per token: threads 0..127 take experts 0..31, threads 128..255 the rest
  const int half = tid / TB, tl = tid % TB;
  pair_token_tail<RS, TB>(red + tl * RS, half, tl, true, tok0 + tl, p, xkeys, xsum);
  if (p.probs) {  // (not with the raw top-k, which has returned without the last barrier)
    for (int i = 0; i < 32; ++i) {
      const int64_t t = tbase + i;
      if (t < p.T && lane < p.E) p.probs[t * p.E + lane] = red[(32 * wave + i) * RS + lane];
    }
  }
}

// ---- capacity slots -------------------------------------------------------------
__global__ __launch_bounds__(256) void slot_hist_kernel(const int32_t* __restrict__ idx, int64_t A,
                                                        int E, int32_t* __restrict__ ws) {
  __shared__ int hist[64];
  if (threadIdx.x < 64) hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSlotChunk;
  for (int i = threadIdx.x; i < kSlotChunk; i += 256) {
    const int64_t a = base + i;
    if (a < A) {
      const int e = idx[a];
      if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1);
    }
  }
  __syncthreads();
  if ((int)threadIdx.x < E) ws[(int64_t)blockIdx.x * E + threadIdx.x] = hist[threadIdx.x];
}

// One wavefront per expert: exclusive scan of the per-chunk histograms, in place.
// Lane l owns a contiguous run of chunks; the lane totals are scanned across the
// wavefront with shuffles, so the chain of dependent global loads is n_chunks/64
// long instead of n_chunks.
__global__ __launch_bounds__(64) void slot_scan_kernel(int32_t* __restrict__ ws, int64_t n_chunks,
                                                       int E, int32_t* __restrict__ count) {
  const int e = blockIdx.x;
  const int lane = threadIdx.x;
  const int64_t per = (n_chunks + 63) / 64;
  const int64_t b0 = lane * per;
  const int64_t b1 = (b0 + per < n_chunks) ? b0 + per : n_chunks;
  // (eight loads in flight per lane: the chunks of a lane are a chain of dependent round trips
  // to L2 otherwise)
  int total = 0;
  for (int64_t b = b0; b < b1; b += 8) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = (b + u < b1) ? ws[(b + u) * E + e] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) total += v[u];
  }
  int incl = total;
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(incl, d, PIKV_WAVE);
    if (lane >= d) incl += up;
  }
  int run = incl - total;
  for (int64_t b = b0; b < b1; b += 8) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = (b + u < b1) ? ws[(b + u) * E + e] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (b + u < b1) ws[(b + u) * E + e] = run;
      run += v[u];
    }
  }
  if (count && lane == 63) count[e] = incl;
}

// SELF_PREFIX: ws holds the raw per-chunk histograms and every block adds up the chunks before
// its own by itself (integer sums: the order does not matter); the last block also writes the
// totals.  For short assignment streams this saves the scan launch, which is all latency there.
template <bool SELF_PREFIX>
__global__ __launch_bounds__(256) void slot_rank_kernel(const int32_t* __restrict__ idx, int64_t A,
                                                        int E, int64_t capacity,
                                                        const int32_t* __restrict__ ws,
                                                        int32_t* __restrict__ slot,
                                                        int32_t* __restrict__ count) {
  __shared__ int running[64];
  __shared__ int wcnt[4][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if constexpr (SELF_PREFIX) {
    if (threadIdx.x < 64) running[threadIdx.x] = 0;
    __syncthreads();
    const int n = (int)blockIdx.x * E;  // words of the earlier chunks, [chunk][expert]
    for (int p0 = threadIdx.x; p0 < n; p0 += 256 * 8) {
      int v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = (p0 + u * 256 < n) ? ws[p0 + u * 256] : 0;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (v[u]) atomicAdd(&running[(p0 + u * 256) % E], v[u]);
    }
    __syncthreads();
    if (count && blockIdx.x == gridDim.x - 1 && (int)threadIdx.x < E)
      count[threadIdx.x] = running[threadIdx.x] + ws[n + threadIdx.x];
  } else {
    if ((int)threadIdx.x < 64)
      running[threadIdx.x] = ((int)threadIdx.x < E) ? ws[(int64_t)blockIdx.x * E + threadIdx.x] : 0;
  }
  const int64_t base = (int64_t)blockIdx.x * kSlotChunk;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int step = 0; step < kSlotChunk / 256; ++step) {
    wcnt[wave][lane] = 0;
    __syncthreads();
    const int64_t a = base + step * 256 + threadIdx.x;
    int e = -1;
    if (a < A) {
      e = idx[a];
      if ((unsigned)e >= (unsigned)E) e = -1;  // out-of-range ids get slot -1
    }
    const bool valid = e >= 0;
    // lanes with the same expert: one ballot per bit of the expert id, and every lane keeps
    // the side of each ballot it is on (six ballots instead of one round per distinct expert)
    uint64_t same = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 6; ++bit) {
      const uint64_t ones = __ballot(valid && ((e >> bit) & 1));
      same &= ((e >> bit) & 1) ? ones : ~ones;
    }
    const int rank = __popcll(same & lt_mask);
    if (valid && rank == 0) wcnt[wave][e] = __popcll(same);
    __syncthreads();
    if (valid) {
      int pos = running[e] + rank;
      for (int w2 = 0; w2 < wave; ++w2) pos += wcnt[w2][e];
      slot[a] = ((int64_t)pos < capacity) ? pos : -1;
    } else if (a < A) {
      slot[a] = -1;
    }
    __syncthreads();
    if (threadIdx.x < 64)
      running[threadIdx.x] += wcnt[0][threadIdx.x] + wcnt[1][threadIdx.x] + wcnt[2][threadIdx.x] +
                              wcnt[3][threadIdx.x];
    __syncthreads();
  }
}

static int64_t slot_chunks(int64_t A) { return (A + kSlotChunk - 1) / kSlotChunk; }

static int64_t slot_workspace_bytes(int64_t A, int E) {
  int64_t b = slot_chunks(A) * E * (int64_t)sizeof(int32_t);
  return (b + 255) / 256 * 256;
}

static int launch_slots(const int32_t* idx, int64_t A, int E, int64_t capacity, int32_t* slot,
                        int32_t* count, void* ws, int64_t ws_bytes, hipStream_t st) {
  if (A == 0) {
    if (count) {
      // count must still be defined: scan over zero chunks writes zeros.
      hipLaunchKernelGGL(slot_scan_kernel, dim3((unsigned)E), dim3(64), 0, st, (int32_t*)ws, (int64_t)0, E, count);
      PIKV_CHECK_LAUNCH();
    }
    return PIKV_OK;
  }
  if (!ws) return PIKV_ERR_NULL;
  if (ws_bytes < slot_workspace_bytes(A, E)) return PIKV_ERR_WORKSPACE;
  const int64_t nb = slot_chunks(A);
  if (nb > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  hipLaunchKernelGGL(slot_hist_kernel, dim3((unsigned)nb), dim3(256), 0, st, idx, A, E, (int32_t*)ws);
  if (nb * E <= kSlotSelfPrefixWords) {
    hipLaunchKernelGGL((slot_rank_kernel<true>), dim3((unsigned)nb), dim3(256), 0, st, idx, A, E, capacity,
                       (const int32_t*)ws, slot, count);
  } else {
    hipLaunchKernelGGL(slot_scan_kernel, dim3((unsigned)E), dim3(64), 0, st, (int32_t*)ws, nb, E, count);
    hipLaunchKernelGGL((slot_rank_kernel<false>), dim3((unsigned)nb), dim3(256), 0, st, idx, A, E, capacity,
                       (const int32_t*)ws, slot, count);
  }
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

static int epad_of(int E) { return E <= 8 ? 8 : E <= 16 ? 16 : E <= 32 ? 32 : 64; }

template <int DT>
static void launch_gate(int epad, unsigned blocks, hipStream_t st, const void* x, const void* w,
                        int H, const TailParams& p) {
  switch (epad) {
    case 8: hipLaunchKernelGGL((router_gate_kernel<8, DT>), dim3(blocks), dim3(256), 0, st, x, w, H, p); break;
    case 16: hipLaunchKernelGGL((router_gate_kernel<16, DT>), dim3(blocks), dim3(256), 0, st, x, w, H, p); break;
    case 32: hipLaunchKernelGGL((router_gate_kernel<32, DT>), dim3(blocks), dim3(256), 0, st, x, w, H, p); break;
    default: hipLaunchKernelGGL((router_gate_kernel<64, DT>), dim3(blocks), dim3(256), 0, st, x, w, H, p); break;
  }
}

}  // namespace pikv

using namespace pikv;

extern "C" int64_t pikv_router_workspace_bytes(int64_t T, int E, int k) {
  if (T < 0 || E < 1 || k < 1) return 0;
  return slot_workspace_bytes(T * k, E);
}

static int gate_epad(int E) { return E <= 16 ? 16 : E <= 32 ? 32 : 64; }
static int64_t gate_weight_bytes(int H, int E) { return (int64_t)H * gate_epad(E) * 4; }  // re-laid weights, float32 at most
static int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

// Short token streams split the gate projection over the hidden dimension: slices of at
// least 16 k-steps, as many as it takes to put about a thousand blocks on the chip.
// Measured at H = 7168, 64 experts: 71 -> 25 us (64..1024 tokens), 74 -> 35 us (4096),
// 77 -> 67 us (16384); with 8 experts (H = 4096) nothing is gained from 16384 tokens on.
constexpr int64_t kTiled64MinTokens = 20480;
static int gate_slices(int64_t T, int H, int E) {
  const int64_t max_tokens = E > 16 ? kTiled64MinTokens - 1 : 16383;
  if (T <= 0 || T > max_tokens || H % 32 != 0) return 1;
  const int64_t steps = H / 32, token_blocks = (T + 63) / 64;
  int64_t s = (steps + 15) / 16;
  const int64_t want = (1024 + token_blocks - 1) / token_blocks;
  if (s > want) s = want;
  return s < 1 ? 1 : (int)s;
}
static int64_t gate_partial_bytes(int64_t T, int H, int E) {
  const int s = gate_slices(T, H, E);
  return s > 1 ? align256((int64_t)s * T * E * 4) : 0;
}

extern "C" int64_t pikv_router_fused_workspace_bytes(int64_t T, int H, int E, int k) {
  if (T < 0 || H < 1 || E < 1 || k < 1) return 0;
  return align256(slot_workspace_bytes(T * k, E)) + align256(gate_weight_bytes(H, E)) + gate_partial_bytes(T, H, E);
}

extern "C" int pikv_capacity_slots(const int32_t* expert_idx, int64_t A, int E, int64_t capacity,
                                   int32_t* slot, int32_t* count, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  if (A != 0 && (!expert_idx || !slot)) return PIKV_ERR_NULL;  // an empty stream needs no buffers
  if (A < 0 || A > 0x7fffffffLL || E < 1 || E > 64 || capacity < 0) return PIKV_ERR_SHAPE;
  return launch_slots(expert_idx, A, E, capacity, slot, count, workspace, workspace_bytes,
                      (hipStream_t)stream);
}

// ---- capacity slots for callers that cannot allocate ------------------------------
// The per-chunk histograms of the slot pass live in a file-scope device array instead of a
// caller workspace.  Every GPU holds its own copy of the array at its own address; the host
// learns that address once per device and passes it to the kernels like any workspace.
constexpr int64_t kSlotStaticMaxAssignments = 1 << 20;
constexpr int kSlotStaticMaxExperts = 64;
constexpr int64_t kSlotStaticWords = (kSlotStaticMaxAssignments / kSlotChunk) * kSlotStaticMaxExperts;
static __device__ __align__(256) int32_t scratch[kSlotStaticWords];  // 512 KiB per GPU

constexpr int kMaxDevices = 64;
static std::atomic<int32_t*> g_scratch_ptr[kMaxDevices];

// Address of this device's copy of `scratch` (looked up on the first call on the device).
static int scratch_of_current_device(int32_t** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return PIKV_ERR_LAUNCH;
  int32_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) return PIKV_ERR_LAUNCH;
    p = static_cast<int32_t*>(sym);
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // every thread finds the same address
  }
  *out = p;
  return PIKV_OK;
}

// The limit of the static form - and its set-up call: asking for the limit also looks up the array's
// address on the current device (which may make the runtime load the code object, a host-side step that
// does not belong inside an open graph capture).  A caller that captures asks here first, per device.
extern "C" int64_t pikv_capacity_slots_static_max(void) {
  int32_t* p = nullptr;
  (void)scratch_of_current_device(&p);   // no device current / no GPU: the limit is still the answer
  return kSlotStaticMaxAssignments;
}

extern "C" int pikv_capacity_slots_static(const int32_t* expert_idx, int64_t A, int E, int64_t capacity,
                                          int32_t* slot, int32_t* count, void* stream) {
  if (A != 0 && (!expert_idx || !slot)) return PIKV_ERR_NULL;  // an empty stream needs no buffers
  if (A < 0 || E < 1 || E > kSlotStaticMaxExperts || capacity < 0) return PIKV_ERR_SHAPE;
  if (A > kSlotStaticMaxAssignments) return PIKV_ERR_WORKSPACE;
  int32_t* ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc != PIKV_OK) return rc;
  // Nothing has to start at zero: the histogram pass writes every word the later passes read.
  return launch_slots(expert_idx, A, E, capacity, slot, count, ws, kSlotStaticWords * (int64_t)sizeof(int32_t),
                      (hipStream_t)stream);
}

static int check_router_dims(int64_t T, int E, int k, int64_t capacity) {
  if (T < 0 || E < 1 || E > 64 || k < 1 || k > 8 || k > E || capacity < 0) return PIKV_ERR_SHAPE;
  if (T * k > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  return PIKV_OK;
}

extern "C" int pikv_router_fused(const void* x, const void* w, int x_dtype, const float* bias,
                                 const float* expert_scale, const float* expert_mask,
                                 float temperature, float renorm_eps, int arithmetic, int64_t T,
                                 int H, int E, int k, int64_t capacity, float* probs, float* logits_out,
                                 int32_t* topk_idx, float* topk_w, int32_t* slot, int32_t* count,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
  if (!x || !w || !topk_idx || !topk_w) return PIKV_ERR_NULL;
  if (x_dtype != PIKV_F32 && x_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  if (arithmetic != PIKV_ROUTER_SINGLE && arithmetic != PIKV_ROUTER_MODULE) return PIKV_ERR_UNSUPPORTED;
  int rc = check_router_dims(T, E, k, capacity);
  if (rc != PIKV_OK) return rc;
  if (H < 8) return PIKV_ERR_SHAPE;
  if (H % 8 != 0) return PIKV_ERR_UNSUPPORTED;
  const bool mfma = x_dtype == PIKV_BF16 && H % 32 == 0;
  // float32 inputs on the matrix cores (exact products, float32 accumulation): 256 tokens and more
  const bool mfma32 = x_dtype == PIKV_F32 && H % 16 == 0 && T >= 256;
  const int64_t slot_ws = align256(slot_workspace_bytes(T * k, E));
  if ((slot || mfma) && T > 0) {
    if (!workspace) return PIKV_ERR_NULL;
    if (workspace_bytes < (slot ? slot_ws : 0) +
                              (mfma ? align256(gate_weight_bytes(H, E)) + gate_partial_bytes(T, H, E) : 0))
      return PIKV_ERR_WORKSPACE;
  }
  // the re-laid gate weights sit behind the slot area when both are in use
  char* wb = reinterpret_cast<char*>(workspace) + (slot ? slot_ws : 0);
  hipStream_t st = (hipStream_t)stream;
  if (T > 0) {
    TailParams p{bias, expert_scale, expert_mask, temperature, renorm_eps, 1, arithmetic, E, k, T,
                 probs, logits_out, topk_idx, topk_w};
    const int epad = epad_of(E);
    const int64_t tiles = (T + (64 / epad) - 1) / (64 / epad);
    const int64_t blocks = (tiles + 3) / 4;
    if (blocks > 0x7fffffffLL) return PIKV_ERR_SHAPE;
    if (mfma) {
      const int ep = gate_epad(E);
      const int64_t chunks = (int64_t)(H / 32) * ep * 4;
      // 64 tokens per block.  Few experts: 8 wavefronts share the k-steps; many
      // experts: 4 (the accumulators of 4 x 4 tiles and the partial sums in LDS
      // leave room for two such blocks per compute unit)
      const int64_t mb = (T + 63) / 64;
      if (mb > 0x7fffffffLL) return PIKV_ERR_SHAPE;
      const dim3 grid((unsigned)mb);
      const int slices = gate_slices(T, H, E);
      // 20480 tokens and more: the tiled kernel.  Its blocks hold 68 KB of LDS, two per compute
      // unit = 512 on the chip: 64-token blocks while they fit in one round (<= 32768 tokens;
      // 32768 x 7168 x 64 experts: 129 us against 155 us with half as many 128-token blocks),
      // 128-token blocks beyond (40960 tokens: 167 us against 185 us in two uneven rounds).
      // Up to 16 experts the untiled kernel streams as fast (8 experts, H = 4096: 81 vs 88 us
      // at 40960 tokens) until about 65536 tokens (117 vs 110 us; H = 7168: 195 vs 178 us),
      // always on 64-token blocks (128-token blocks: 129 us).
      const bool tiled = T >= (ep == 16 ? 65536 : kTiled64MinTokens);
      const bool t128 = tiled && ep != 16 && H % 128 == 0 && (T > 32768 || H % 256 != 0);
      const bool t64 = tiled && !t128 && H % 256 == 0;
      const dim3 g64((unsigned)((T + 63) / 64)), g128((unsigned)((T + 127) / 128));
      // up to 16 experts on the untiled kernel: the weights are read where they lie
      const bool direct = slices <= 1 && !t64 && !t128 && ep == 16;
      if (!direct)
        hipLaunchKernelGGL(gate_weight_relayout_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256),
                           0, st, w, (int64_t)H * 2, E, ep, (uint4*)wb);
      if (slices > 1) {
        // short token streams: partial logits per slice of H, then the tail on their sum
        float* part = reinterpret_cast<float*>(wb + align256(gate_weight_bytes(H, E)));
        const int sps = (int)((H / 32 + slices - 1) / slices);
        const dim3 g2((unsigned)mb, (unsigned)slices);
        if (ep == 16)
          hipLaunchKernelGGL((router_gate_mfma_kernel<1, 4, 8, true>), g2, dim3(512), 0, st, x, wb, H, p, part, sps);
        else if (ep == 32)
          hipLaunchKernelGGL((router_gate_mfma_kernel<2, 4, 4, true>), g2, dim3(256), 0, st, x, wb, H, p, part, sps);
        else
          hipLaunchKernelGGL((router_gate_mfma_kernel<4, 4, 4, true>), g2, dim3(256), 0, st, x, wb, H, p, part, sps);
        switch (epad) {
          case 8: hipLaunchKernelGGL((router_tail_kernel<8>), dim3((unsigned)blocks), dim3(256), 0, st, part, nullptr, nullptr, p, slices); break;
          case 16: hipLaunchKernelGGL((router_tail_kernel<16>), dim3((unsigned)blocks), dim3(256), 0, st, part, nullptr, nullptr, p, slices); break;
          case 32: hipLaunchKernelGGL((router_tail_kernel<32>), dim3((unsigned)blocks), dim3(256), 0, st, part, nullptr, nullptr, p, slices); break;
          default: hipLaunchKernelGGL((router_tail_kernel<64>), dim3((unsigned)blocks), dim3(256), 0, st, part, nullptr, nullptr, p, slices); break;
        }
      } else if (t64 && ep == 64)
        hipLaunchKernelGGL((router_gate_lds_kernel<64, 64, 256>), g64, dim3(256), 0, st, x, wb, H, p);
      else if (t64 && ep == 32)
        hipLaunchKernelGGL((router_gate_lds_kernel<32, 64, 256>), g64, dim3(256), 0, st, x, wb, H, p);
      else if (t64)
        hipLaunchKernelGGL((router_gate_lds_kernel<16, 64, 256>), g64, dim3(256), 0, st, x, wb, H, p);
      else if (t128 && ep == 64)
        hipLaunchKernelGGL((router_gate_lds_kernel<64, 128, 128>), g128, dim3(256), 0, st, x, wb, H, p);
      else if (t128 && ep == 32)
        hipLaunchKernelGGL((router_gate_lds_kernel<32, 128, 128>), g128, dim3(256), 0, st, x, wb, H, p);
      else if (ep == 64 && T >= 32768)
        // 128-token blocks: the weights are re-read from L2 once per block, so twice the
        // tokens per block halves that traffic
        hipLaunchKernelGGL((router_gate_mfma_kernel<4, 8, 4>), dim3((unsigned)((T + 127) / 128)), dim3(256), 0, st,
                           x, wb, H, p);
      else if (ep == 16)
        hipLaunchKernelGGL((router_gate_mfma_kernel<1, 4, 8, false, true>), grid, dim3(512), 0, st, x, w, H, p);
      else if (ep == 32)
        hipLaunchKernelGGL((router_gate_mfma_kernel<2, 4, 4>), grid, dim3(256), 0, st, x, wb, H, p);
      else
        hipLaunchKernelGGL((router_gate_mfma_kernel<4, 4, 4>), grid, dim3(256), 0, st, x, wb, H, p);
    } else if (x_dtype == PIKV_BF16) {
      launch_gate<PIKV_BF16>(epad, (unsigned)blocks, st, x, w, H, p);
    } else if (mfma32) {
      const int ep = gate_epad(E);
      const int64_t mb = (T + 63) / 64;
      if (mb > 0x7fffffffLL) return PIKV_ERR_SHAPE;
      // more than 16 experts: the weights re-laid per k-step like the bf16 ones, when the caller's
      // workspace has room for them; read in place otherwise
      const bool relaid = ep > 16 && workspace &&
                          workspace_bytes >= (slot ? slot_ws : 0) + align256(gate_weight_bytes(H, E));
      if (relaid) {
        const int64_t chunks = (int64_t)(H / 16) * ep * 4;
        hipLaunchKernelGGL(gate_weight_relayout_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256),
                           0, st, w, (int64_t)H * 4, E, ep, (uint4*)wb);
      }
      if (ep == 16)
        hipLaunchKernelGGL((router_gate_mfma_kernel<1, 4, 8, false, true, true>), dim3((unsigned)mb), dim3(512), 0, st, x, w, H, p);
      else if (ep == 32 && relaid)
        hipLaunchKernelGGL((router_gate_mfma_kernel<2, 4, 4, false, false, true>), dim3((unsigned)mb), dim3(256), 0, st, x, wb, H, p);
      else if (ep == 32)
        hipLaunchKernelGGL((router_gate_mfma_kernel<2, 4, 4, false, true, true>), dim3((unsigned)mb), dim3(256), 0, st, x, w, H, p);
      else if (relaid && T >= 32768)   // 128 tokens per block: every weight operand serves eight token tiles
        hipLaunchKernelGGL((router_gate_mfma_kernel<4, 8, 4, false, false, true>), dim3((unsigned)((T + 127) / 128)), dim3(256), 0, st, x, wb, H, p);
      else if (relaid)
        hipLaunchKernelGGL((router_gate_mfma_kernel<4, 4, 4, false, false, true>), dim3((unsigned)mb), dim3(256), 0, st, x, wb, H, p);
      else
        hipLaunchKernelGGL((router_gate_mfma_kernel<4, 4, 4, false, true, true>), dim3((unsigned)mb), dim3(256), 0, st, x, w, H, p);
    } else {
      launch_gate<PIKV_F32>(epad, (unsigned)blocks, st, x, w, H, p);
    }
    PIKV_CHECK_LAUNCH();
  }
  if (slot) return launch_slots(topk_idx, T * k, E, capacity, slot, count, workspace, workspace_bytes, st);
  return PIKV_OK;
}

extern "C" int pikv_router_tail(const float* logits_a, const float* logits_b, const uint8_t* select,
                                const float* expert_scale, const float* expert_mask,
                                float temperature, float renorm_eps, int use_softmax,
                                int arithmetic, int64_t T, int E, int k, int64_t capacity,
                                float* probs, int32_t* topk_idx,
                                float* topk_w, int32_t* slot, int32_t* count, void* workspace,
                                int64_t workspace_bytes, void* stream) {
  if (!logits_a || !topk_idx || !topk_w) return PIKV_ERR_NULL;
  if (arithmetic != PIKV_ROUTER_SINGLE && arithmetic != PIKV_ROUTER_MODULE) return PIKV_ERR_UNSUPPORTED;
  int rc = check_router_dims(T, E, k, capacity);
  if (rc != PIKV_OK) return rc;
  if (slot) {
    if (!workspace && T > 0) return PIKV_ERR_NULL;
    if (workspace_bytes < slot_workspace_bytes(T * k, E)) return PIKV_ERR_WORKSPACE;
  }
  hipStream_t st = (hipStream_t)stream;
  if (T > 0) {
    TailParams p{nullptr, expert_scale, expert_mask, temperature, renorm_eps, use_softmax ? 1 : 0,
                 arithmetic, E, k, T, use_softmax ? probs : nullptr, nullptr, topk_idx, topk_w};
    const int epad = epad_of(E);
    const int64_t tiles = (T + (64 / epad) - 1) / (64 / epad);
    const int64_t blocks = (tiles + 3) / 4;
    if (blocks > 0x7fffffffLL) return PIKV_ERR_SHAPE;
    switch (epad) {
      case 8: hipLaunchKernelGGL((router_tail_kernel<8>), dim3((unsigned)blocks), dim3(256), 0, st, logits_a, logits_b, select, p); break;
      case 16: hipLaunchKernelGGL((router_tail_kernel<16>), dim3((unsigned)blocks), dim3(256), 0, st, logits_a, logits_b, select, p); break;
      case 32: hipLaunchKernelGGL((router_tail_kernel<32>), dim3((unsigned)blocks), dim3(256), 0, st, logits_a, logits_b, select, p); break;
      default:
        // 33-64 experts: an arg-max round over 64 lanes costs ~2.9 us per round at 65536 tokens
        // (21 us at k = 1, 24 at k = 2), two lanes per token 20.6 us whatever k
        if (k >= kRowsTailMinK)
          hipLaunchKernelGGL(router_tail_rows_kernel, dim3((unsigned)((T + 127) / 128)), dim3(256), 0, st, logits_a, logits_b, select, p);
        else
          hipLaunchKernelGGL((router_tail_kernel<64>), dim3((unsigned)blocks), dim3(256), 0, st, logits_a, logits_b, select, p);
        break;
    }
    PIKV_CHECK_LAUNCH();
  }
  if (slot) return launch_slots(topk_idx, T * k, E, capacity, slot, count, workspace, workspace_bytes, st);
  return PIKV_OK;
}
