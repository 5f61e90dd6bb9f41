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
  int64_t n_src;
  int64_t dst_row0;     // used when cache_id == nullptr
  int fanout;
  int D;
  int group;
  int n_tensors;        // 1 (K only) or 2 (K and V)
  int n_caches;
};

template <int SCHEME, int SRC_DT>
__global__ __launch_bounds__(256) void quant_scatter_kernel(QuantScatterArgs a) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  const int lanes_per_row = a.D / EPL;
  const int lanes_per_group = a.group / EPL;
  const int groups_per_row = a.D / a.group;

  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t s = g / lanes_per_row;
  const int part = (int)(g - s * lanes_per_row);
  const bool valid = s < a.n_src;

  // Destination rows of this source row (-1 = dropped).  Fixed-trip unrolled
  // loops keep the array in registers.
  int64_t dst[kMaxFanout];
  bool any = false;
#pragma unroll
  for (int j = 0; j < kMaxFanout; ++j) {
    dst[j] = -1;
    if (valid && j < a.fanout) {
      if (a.cache_id == nullptr) {
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

  for (int t = 0; t < a.n_tensors; ++t) {
    float x[EPL];
    if (live) {
      load_as_float<SRC_DT, EPL>(a.src[t], s * a.D + (int64_t)part * EPL, x);
    } else {
#pragma unroll
      for (int i = 0; i < EPL; ++i) x[i] = 0.f;
    }
    float mn = x[0], mx = x[0];
#pragma unroll
    for (int i = 1; i < EPL; ++i) {
      mn = fminf(mn, x[i]);
      mx = fmaxf(mx, x[i]);
    }
    mn = group_min_rt(mn, lanes_per_group);
    mx = group_max_rt(mx, lanes_per_group);
    float scale, zero;
    quant_params<SCHEME>(mn, mx, scale, zero);
    int c[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) c[i] = quant_code<SCHEME>(x[i], scale, zero);
    const uint4 packed = pack_codes<SCHEME>(c);
    if (live) {
      const bool meta_lane = (part % lanes_per_group) == 0;
      const int grp = part / lanes_per_group;
#pragma unroll
      for (int j = 0; j < kMaxFanout; ++j) {
        const int64_t row = dst[j];
        if (row < 0) continue;
        char* cp = reinterpret_cast<char*>(a.codes[t]) + (row * lanes_per_row + part) * 16;
        st16(cp, packed);
        if (meta_lane) {
          store_meta<SCHEME>(a.scale[t], row * groups_per_row + grp, scale);
          if constexpr (!Q::sym) store_meta<SCHEME>(a.zero[t], row * groups_per_row + grp, zero);
        }
      }
    }
  }
  if (live && part == 0) {
#pragma unroll
    for (int j = 0; j < kMaxFanout; ++j) {
      if (dst[j] < 0) continue;
      if (a.row_acc) a.row_acc[dst[j]] = 0.f;
      if (a.row_ts) a.row_ts[dst[j]] = a.now;
    }
  }
}

template <int SCHEME>
static int launch_quant(const QuantScatterArgs& a, int src_dtype, hipStream_t st) {
  using Q = QScheme<SCHEME>;
  const int64_t lanes = a.n_src * (a.D / Q::epl);
  if (lanes == 0) return PIKV_OK;
  const int64_t blocks = (lanes + 255) / 256;
  if (blocks > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  if (src_dtype == PIKV_BF16)
    hipLaunchKernelGGL((quant_scatter_kernel<SCHEME, PIKV_BF16>), dim3((unsigned)blocks), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((quant_scatter_kernel<SCHEME, PIKV_F32>), dim3((unsigned)blocks), dim3(256), 0, st, a);
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
  a.D = D; a.group = group; a.n_tensors = 1;
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
