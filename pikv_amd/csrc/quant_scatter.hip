// K2: fused KV quantise + per-cache scatter (append), and plain row quantise.
//
// One lane owns 16 code bytes of one row: 16 source elements for the 8-bit
// schemes, 32 for the 4-bit ones.  A quantisation group spans
// group/elements-per-lane adjacent lanes (a power of two <= 64, so a group never
// straddles a wavefront) and its min/max is reduced across exactly those lanes.
// A source row is read once, quantised once, and its 16-byte code vectors are
// stored to each of the row's `fanout` destination rows, so HBM sees the
// algorithmic traffic only: D*sizeof(src) bytes in, fanout*(D*bits/8 + metadata)
// bytes out per source row, all as 128-bit accesses contiguous across lanes.
// The per-element division of the reference formula is replaced by one division per
// group and three multiply-adds per element that reproduce the correctly rounded
// quotient (see quantize_lane), which is what takes the kernel from VALU-bound to
// HBM-bound.
#include "common.hpp"

namespace pikv {

constexpr int kMaxFanout = 8;

struct QuantScatterArgs {
  const void* src[2];   // K, V source [n_src, D]
  void* codes[2];       // pool code planes
  void* scale[2];       // pool scale planes
  void* zero[2];        // pool zero planes (asymmetric only)
  const int32_t* cache_id;
  const int32_t* slot;
  const int64_t* row_base;
  const int32_t* fill;
  const int32_t* cap;
  float* row_acc;
  float* row_ts;
  float now;
  // gather mode (seg_index != nullptr): grid row y = cache c; logical source j of
  // cache c is source row seg_src_base[c] + seg_index[seg_src_base[c] + j],
  // j < seg_count[c], appended at cache row fill[c] + j
  const int64_t* seg_src_base;
  const int32_t* seg_index;
  const int32_t* seg_count;
  const float* seg_score;  // optional: initial accumulator of a gathered row, by source row
  int64_t n_src;
  int64_t dst_row0;     // used when cache_id == nullptr
  int fanout;
  int D;
  int group;
  int n_tensors;        // 1 (K only) or 2 (K and V)
  int n_caches;
  int lpr_shift;        // log2(lanes per row) or -1 when it is not a power of two
  int lpg_shift;        // log2(lanes per group)
};

template <int DT, int EPL>
struct RawRow {
  static constexpr int kVec = (DT == PIKV_BF16) ? EPL / 8 : EPL / 4;
  uint4 v[kVec];
  __device__ __forceinline__ void load(const void* base, int64_t elem_off) {
    const char* p = reinterpret_cast<const char*>(base) + elem_off * (DT == PIKV_BF16 ? 2 : 4);
#pragma unroll
    for (int i = 0; i < kVec; ++i) v[i] = ld16(p + 16 * i);
  }
  __device__ __forceinline__ void zero_fill() {
#pragma unroll
    for (int i = 0; i < kVec; ++i) v[i] = make_uint4(0, 0, 0, 0);
  }
  __device__ __forceinline__ void to_float(float (&x)[EPL]) const {
    if constexpr (DT == PIKV_BF16) {
#pragma unroll
      for (int i = 0; i < kVec; ++i) {
        const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[8 * i + 2 * j] = __uint_as_float(w[j] << 16);
          x[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kVec; ++i) {
        x[4 * i] = __uint_as_float(v[i].x);
        x[4 * i + 1] = __uint_as_float(v[i].y);
        x[4 * i + 2] = __uint_as_float(v[i].z);
        x[4 * i + 3] = __uint_as_float(v[i].w);
      }
    }
  }
};

// ROW_UNIFORM: lanes_per_row is a power of two >= 64, so a wavefront never spans two
// source rows; the row index, its destinations and every address base are then
// wave-uniform and live in scalar registers.
template <int SCHEME, int SRC_DT, int FANOUT, bool ROW_UNIFORM>
__global__ __launch_bounds__(256) void quant_scatter_kernel(QuantScatterArgs a) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  const int lanes_per_row = a.D / EPL;
  const int lanes_per_group = a.group / EPL;
  const int groups_per_row = a.D / a.group;

  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t s;
  int part;
  if constexpr (ROW_UNIFORM) {
    const int64_t g0 = (int64_t)blockIdx.x * 256 + (threadIdx.x & ~63u);
    const uint32_t g0lo = __builtin_amdgcn_readfirstlane((uint32_t)g0);
    const uint32_t g0hi = __builtin_amdgcn_readfirstlane((uint32_t)(g0 >> 32));
    const int64_t gu = (int64_t)(((uint64_t)g0hi << 32) | g0lo);
    s = gu >> a.lpr_shift;
    part = (int)(gu & (lanes_per_row - 1)) + (int)(threadIdx.x & 63u);
  } else if (a.lpr_shift >= 0) {
    s = g >> a.lpr_shift;
    part = (int)(g & (lanes_per_row - 1));
  } else {
    s = g / lanes_per_row;
    part = (int)(g - s * lanes_per_row);
  }
  bool valid = s < a.n_src;
  int64_t srow = s;  // row of src[] this lane reads
  int64_t gather_dst = -1;
  if (a.seg_index != nullptr) {
    const int c = blockIdx.y;
    valid = valid && s < a.seg_count[c];
    if (valid) {
      const int64_t sb = a.seg_src_base[c];
      srow = sb + a.seg_index[sb + s];
      const int64_t r = (int64_t)a.fill[c] + s;
      if (r < a.cap[c]) gather_dst = a.row_base[c] + r;
    }
  }

  // Destination rows of this source row (-1 = dropped).
  int64_t dst[FANOUT];
  bool any = false;
#pragma unroll
  for (int j = 0; j < FANOUT; ++j) {
    dst[j] = -1;
    if (valid && j < a.fanout) {
      if (a.seg_index != nullptr) {
        dst[j] = gather_dst;
      } else if (a.cache_id == nullptr) {
        dst[j] = a.dst_row0 + s;
      } else {
        const int64_t as = s * a.fanout + j;
        const int sl = a.slot[as];
        if (sl >= 0) {
          const int c = a.cache_id[as];
          if ((unsigned)c < (unsigned)a.n_caches) {  // ids outside the pool are dropped
            const int64_t r = (int64_t)a.fill[c] + sl;
            if (r < a.cap[c]) dst[j] = a.row_base[c] + r;
          }
        }
      }
      any |= dst[j] >= 0;
    }
  }
  // Lanes of one group share s, hence the same destinations: the whole group
  // takes the same branch below, and cross-lane traffic stays inside the group.
  const bool live = valid && any;
  // A group never straddles a wavefront, so a wavefront without live lanes has
  // nothing to reduce or store.
  if (__ballot(live) == 0) return;

  RawRow<SRC_DT, EPL> raw[2];
  raw[0].zero_fill();
  raw[1].zero_fill();
  if (live) {
    const int64_t off = srow * a.D + (int64_t)part * EPL;
    raw[0].load(a.src[0], off);
  }
  const bool meta_lane = (part & (lanes_per_group - 1)) == 0;
  const int grp = part >> a.lpg_shift;

#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (t >= a.n_tensors) break;
    // The V row is fetched only now: holding both raw rows across the K arithmetic cost
    // the registers of one to two resident wavefronts per SIMD (4-bit: 86 -> 68 registers,
    // 150 -> 125 us at 131072 rows x 1024), and the other wavefronts cover the wait.
    if (t == 1 && live) raw[1].load(a.src[1], srow * a.D + (int64_t)part * EPL);
    float x[EPL];
    raw[t].to_float(x);
    float mn = x[0], mx = x[0];
#pragma unroll
    for (int i = 1; i < EPL; ++i) {
      mn = fminf(mn, x[i]);
      mx = fmaxf(mx, x[i]);
    }
    group_minmax_dpp(mn, mx, lanes_per_group);
    const GroupQuant gq = make_group_quant<SCHEME>(mn, mx);
    const uint4 packed = quantize_lane<SCHEME>(x, gq);
    if (live) {
#pragma unroll
      for (int j = 0; j < FANOUT; ++j) {
        const int64_t row = dst[j];
        if (row < 0) continue;
        char* cp = reinterpret_cast<char*>(a.codes[t]) + (row * lanes_per_row + part) * 16;
        st16_stream(cp, packed);
        if (meta_lane) {
          store_meta<SCHEME>(a.scale[t], row * groups_per_row + grp, gq.scale);
          if constexpr (!Q::sym) store_meta<SCHEME>(a.zero[t], row * groups_per_row + grp, gq.zero);
        }
      }
    }
  }
  if (live && part == 0) {
#pragma unroll
    for (int j = 0; j < FANOUT; ++j) {
      if (dst[j] < 0) continue;
      if (a.row_acc) a.row_acc[dst[j]] = a.seg_score ? a.seg_score[srow] : 0.f;
      if (a.row_ts) a.row_ts[dst[j]] = a.now;
    }
  }
}

template <int SCHEME, int SRC_DT, bool RU>
static void launch_quant_f(int fanout, unsigned blocks, hipStream_t st, const QuantScatterArgs& a) {
  const dim3 grid(blocks, a.seg_index ? (unsigned)a.n_caches : 1u);
  if (fanout <= 1)
    hipLaunchKernelGGL((quant_scatter_kernel<SCHEME, SRC_DT, 1, RU>), grid, dim3(256), 0, st, a);
  else if (fanout <= 2)
    hipLaunchKernelGGL((quant_scatter_kernel<SCHEME, SRC_DT, 2, RU>), grid, dim3(256), 0, st, a);
  else if (fanout <= 4)
    hipLaunchKernelGGL((quant_scatter_kernel<SCHEME, SRC_DT, 4, RU>), grid, dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((quant_scatter_kernel<SCHEME, SRC_DT, 8, RU>), grid, dim3(256), 0, st, a);
}

template <int SCHEME>
static int launch_quant(QuantScatterArgs a, int src_dtype, hipStream_t st) {
  using Q = QScheme<SCHEME>;
  const int lanes_per_row = a.D / Q::epl;
  a.lpr_shift = -1;
  if (is_pow2(lanes_per_row)) {
    a.lpr_shift = 0;
    while ((1 << a.lpr_shift) < lanes_per_row) ++a.lpr_shift;
  }
  a.lpg_shift = 0;
  while ((Q::epl << a.lpg_shift) < a.group) ++a.lpg_shift;
  const int64_t lanes = a.n_src * lanes_per_row;
  if (lanes == 0) return PIKV_OK;
  const int64_t blocks = (lanes + 255) / 256;
  if (blocks > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  const bool ru = a.lpr_shift >= 6;
  if (src_dtype == PIKV_BF16) {
    if (ru) launch_quant_f<SCHEME, PIKV_BF16, true>(a.fanout, (unsigned)blocks, st, a);
    else launch_quant_f<SCHEME, PIKV_BF16, false>(a.fanout, (unsigned)blocks, st, a);
  } else {
    if (ru) launch_quant_f<SCHEME, PIKV_F32, true>(a.fanout, (unsigned)blocks, st, a);
    else launch_quant_f<SCHEME, PIKV_F32, false>(a.fanout, (unsigned)blocks, st, a);
  }
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

static int check_quant_shape(int D, int group, int scheme) {
  if (scheme < 0 || scheme > 3) return PIKV_ERR_UNSUPPORTED;
  const bool eight = (scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM);
  const int epl = eight ? 16 : 32;
  if (D <= 0 || group <= 0 || D % group != 0) return PIKV_ERR_SHAPE;
  if (!is_pow2(group) || group < epl || group > epl * 64) return PIKV_ERR_UNSUPPORTED;
  return PIKV_OK;
}

static int dispatch_quant(const QuantScatterArgs& a, int scheme, int src_dtype, hipStream_t st) {
  switch (scheme) {
    case PIKV_Q_I8_SYM: return launch_quant<PIKV_Q_I8_SYM>(a, src_dtype, st);
    case PIKV_Q_I8_ASYM: return launch_quant<PIKV_Q_I8_ASYM>(a, src_dtype, st);
    case PIKV_Q_I4_ASYM: return launch_quant<PIKV_Q_I4_ASYM>(a, src_dtype, st);
    case PIKV_Q_I4_SYM: return launch_quant<PIKV_Q_I4_SYM>(a, src_dtype, st);
  }
  return PIKV_ERR_UNSUPPORTED;
}

__global__ void cache_advance_kernel(int32_t* fill, const int32_t* count, const int32_t* cap,
                                     int n, int64_t limit) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n) return;
  int64_t add = count[c];
  if (limit >= 0 && add > limit) add = limit;
  int64_t f = (int64_t)fill[c] + add;
  if (f > cap[c]) f = cap[c];
  fill[c] = (int32_t)f;
}

}  // namespace pikv

using namespace pikv;

extern "C" int pikv_quant_scatter(const void* k_src, const void* v_src, int src_dtype,
                                  int64_t n_src, int fanout, int D, int group, int scheme,
                                  const int32_t* cache_id, const int32_t* slot,
                                  const int64_t* cache_row_base, const int32_t* cache_fill,
                                  const int32_t* cache_cap, int n_caches,
                                  void* k_codes, void* v_codes, void* k_scale, void* v_scale,
                                  void* k_zero, void* v_zero, float* row_acc, float* row_ts,
                                  float now, void* stream) {
  if (!k_src || !k_codes || !k_scale || !cache_id || !slot || !cache_row_base || !cache_fill ||
      !cache_cap)
    return PIKV_ERR_NULL;
  if (src_dtype != PIKV_F32 && src_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  if (n_src < 0 || fanout < 1 || fanout > kMaxFanout || n_caches < 1) return PIKV_ERR_SHAPE;
  int rc = check_quant_shape(D, group, scheme);
  if (rc != PIKV_OK) return rc;
  const bool asym = (scheme == PIKV_Q_I8_ASYM || scheme == PIKV_Q_I4_ASYM);
  if (asym && !k_zero) return PIKV_ERR_NULL;
  if (v_src && (!v_codes || !v_scale || (asym && !v_zero))) return PIKV_ERR_NULL;
  QuantScatterArgs a{};
  a.src[0] = k_src; a.src[1] = v_src;
  a.codes[0] = k_codes; a.codes[1] = v_codes;
  a.scale[0] = k_scale; a.scale[1] = v_scale;
  a.zero[0] = k_zero; a.zero[1] = v_zero;
  a.cache_id = cache_id; a.slot = slot; a.row_base = cache_row_base;
  a.fill = cache_fill; a.cap = cache_cap;
  a.row_acc = row_acc; a.row_ts = row_ts; a.now = now;
  a.n_src = n_src; a.dst_row0 = 0; a.fanout = fanout; a.D = D; a.group = group;
  a.n_tensors = v_src ? 2 : 1;
  a.n_caches = n_caches;
  return dispatch_quant(a, scheme, src_dtype, (hipStream_t)stream);
}

extern "C" int pikv_quant_gather(const void* k_src, const void* v_src, int src_dtype, int D,
                                 int group, int scheme, const int64_t* src_row_base,
                                 const int32_t* src_index, const int32_t* n_take, int64_t max_take,
                                 const float* src_score, const int64_t* cache_row_base,
                                 const int32_t* cache_fill, const int32_t* cache_cap, int n_caches,
                                 void* k_codes, void* v_codes, void* k_scale, void* v_scale,
                                 void* k_zero, void* v_zero, float* row_acc, float* row_ts,
                                 float now, void* stream) {
  if (!k_src || !k_codes || !k_scale || !src_row_base || !src_index || !n_take || !cache_row_base ||
      !cache_fill || !cache_cap)
    return PIKV_ERR_NULL;
  if (src_dtype != PIKV_F32 && src_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  if (max_take < 0 || n_caches < 1 || n_caches > 65535) return PIKV_ERR_SHAPE;
  int rc = check_quant_shape(D, group, scheme);
  if (rc != PIKV_OK) return rc;
  const bool asym = (scheme == PIKV_Q_I8_ASYM || scheme == PIKV_Q_I4_ASYM);
  if (asym && !k_zero) return PIKV_ERR_NULL;
  if (v_src && (!v_codes || !v_scale || (asym && !v_zero))) return PIKV_ERR_NULL;
  QuantScatterArgs a{};
  a.src[0] = k_src; a.src[1] = v_src;
  a.codes[0] = k_codes; a.codes[1] = v_codes;
  a.scale[0] = k_scale; a.scale[1] = v_scale;
  a.zero[0] = k_zero; a.zero[1] = v_zero;
  a.row_base = cache_row_base; a.fill = cache_fill; a.cap = cache_cap;
  a.seg_src_base = src_row_base; a.seg_index = src_index; a.seg_count = n_take;
  a.seg_score = src_score;
  a.row_acc = row_acc; a.row_ts = row_ts; a.now = now;
  a.n_src = max_take; a.dst_row0 = 0; a.fanout = 1; a.D = D; a.group = group;
  a.n_tensors = v_src ? 2 : 1;
  a.n_caches = n_caches;
  return dispatch_quant(a, scheme, src_dtype, (hipStream_t)stream);
}

extern "C" int pikv_quantize_rows(const void* src, int src_dtype, int64_t n_rows, int D, int group,
                                  int scheme, int64_t dst_row0, void* codes, void* scale,
                                  void* zero, void* stream) {
  if (!src || !codes || !scale) return PIKV_ERR_NULL;
  if (src_dtype != PIKV_F32 && src_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  if (n_rows < 0 || dst_row0 < 0) return PIKV_ERR_SHAPE;
  int rc = check_quant_shape(D, group, scheme);
  if (rc != PIKV_OK) return rc;
  const bool asym = (scheme == PIKV_Q_I8_ASYM || scheme == PIKV_Q_I4_ASYM);
  if (asym && !zero) return PIKV_ERR_NULL;
  QuantScatterArgs a{};
  a.src[0] = src; a.codes[0] = codes; a.scale[0] = scale; a.zero[0] = zero;
  a.cache_id = nullptr; a.n_src = n_rows; a.dst_row0 = dst_row0; a.fanout = 1;
  a.D = D; a.group = group; a.n_tensors = 1; a.n_caches = 1;
  return dispatch_quant(a, scheme, src_dtype, (hipStream_t)stream);
}

extern "C" int pikv_cache_advance(int32_t* cache_fill, const int32_t* count,
                                  const int32_t* cache_cap, int n_caches, int64_t per_call_limit,
                                  void* stream) {
  if (!cache_fill || !count || !cache_cap) return PIKV_ERR_NULL;
  if (n_caches < 1) return PIKV_ERR_SHAPE;
  hipLaunchKernelGGL(cache_advance_kernel, dim3((n_caches + 63) / 64), dim3(64), 0,
                     (hipStream_t)stream, cache_fill, count, cache_cap, n_caches, per_call_limit);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
