// K4: eviction top-k selection and stable in-place compaction.
//
// Selection: one 1024-thread block per cache.  A float is mapped to a 32-bit key
// whose unsigned order is the float order; an MSB-first radix select (4 passes of
// 8 bits, LDS histogram) finds the key of the m-th largest element, and an
// ordered marking pass takes every larger element plus the first (lowest-index)
// elements equal to it.  Total order = (value desc, index asc); the "smallest m"
// variant runs the same code on the complemented key.
//
// Compaction: survivors move to the front in ascending order.  A block owns one
// (cache, plane, column slab) and walks the survivor list in steps: all source
// rows of a step are read into registers, the block synchronises, then the
// destinations are written.  Because destination j <= source keep_index[j] and
// the list is ascending, a later step never reads what an earlier one wrote, and
// blocks never share bytes - so the move is in place, race-free and needs no
// staging buffer.
#include "common.hpp"

namespace pikv {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / 64;

__device__ __forceinline__ uint32_t order_key(float v, bool smallest) {
  v = v + 0.0f;  // -0 -> +0 so that they tie
  uint32_t u = __float_as_uint(v);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return smallest ? ~u : u;
}

// Exclusive prefix count of a per-thread flag over the block, in thread order.
// sh must hold kSelWaves ints.  Returns the prefix; total gets the block sum.
__device__ __forceinline__ int block_flag_scan(bool f, int* sh, int& total) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const uint64_t b = __ballot(f);
  const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  const int in_wave = __popcll(b & lt);
  __syncthreads();  // previous use of sh is over
  if (lane == 0) sh[wave] = __popcll(b);
  __syncthreads();
  int pre = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kSelWaves; ++w) {
    const int v = sh[w];
    if (w < wave) pre += v;
    tot += v;
  }
  total = tot;
  return pre + in_wave;
}

// Mark the m top elements of v[0..len): flag[i] = mark.  All threads must call.
__device__ void block_select_mark(const float* __restrict__ v, int len, int m, bool smallest,
                                  uint8_t* __restrict__ flag, uint8_t mark, int* hist /*256*/,
                                  int* sh /*kSelWaves + 2*/) {
  if (m <= 0 || len <= 0) return;  // uniform
  if (m >= len) {
    for (int i = threadIdx.x; i < len; i += kSelThreads) flag[i] = mark;
    return;
  }
  uint32_t prefix = 0, pmask = 0;
  int remaining = m;
  for (int shift = 24; shift >= 0; shift -= 8) {
    __syncthreads();
    if (threadIdx.x < 256) hist[threadIdx.x] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < len; i += kSelThreads) {
      const uint32_t key = order_key(v[i], smallest);
      if ((key & pmask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int cum = 0, d = 255;
      for (; d > 0; --d) {
        if (cum + hist[d] >= remaining) break;
        cum += hist[d];
      }
      sh[kSelWaves] = d;
      sh[kSelWaves + 1] = remaining - cum;
    }
    __syncthreads();
    prefix |= (uint32_t)sh[kSelWaves] << shift;
    pmask |= 255u << shift;
    remaining = sh[kSelWaves + 1];
  }
  // prefix = key of the m-th element; `remaining` of the elements equal to it are taken.
  int taken_eq = 0;
  for (int i0 = 0; i0 < len; i0 += kSelThreads) {
    const int i = i0 + threadIdx.x;
    uint32_t key = 0;
    bool eq = false, gt = false;
    if (i < len) {
      key = order_key(v[i], smallest);
      eq = key == prefix;
      gt = key > prefix;
    }
    int tot;
    const int r = block_flag_scan(eq, sh, tot);
    if (gt || (eq && taken_eq + r < remaining)) flag[i] = mark;
    taken_eq += tot;
  }
}

__global__ __launch_bounds__(kSelThreads) void evict_select_kernel(
    int policy, const float* __restrict__ row_acc, const float* __restrict__ row_ts,
    const int64_t* __restrict__ row_base, const int32_t* __restrict__ fill,
    const int32_t* __restrict__ n_heavy, const int32_t* __restrict__ n_recent,
    uint8_t* __restrict__ keep_flag, int32_t* __restrict__ keep_index, int32_t* __restrict__ new_len) {
  __shared__ int hist[256];
  __shared__ int sh[kSelWaves + 2];
  const int c = blockIdx.x;
  const int len = fill[c];
  const int64_t base = row_base[c];
  uint8_t* flag = keep_flag + base;
  if (len <= 0) {
    if (threadIdx.x == 0) new_len[c] = 0;
    return;
  }
  if (policy == PIKV_EVICT_H2O) {
    for (int i = threadIdx.x; i < len; i += kSelThreads) flag[i] = 0;
    __syncthreads();
    block_select_mark(row_acc + base, len, n_heavy[c], false, flag, 1, hist, sh);
    __syncthreads();
    block_select_mark(row_ts + base, len, n_recent[c], false, flag, 1, hist, sh);
  } else {
    for (int i = threadIdx.x; i < len; i += kSelThreads) flag[i] = 1;
    __syncthreads();
    block_select_mark(row_ts + base, len, n_heavy[c], true, flag, 0, hist, sh);
  }
  __syncthreads();
  // Ascending list of survivors.
  int32_t* out = keep_index + base;
  int kept = 0;
  for (int i0 = 0; i0 < len; i0 += kSelThreads) {
    const int i = i0 + threadIdx.x;
    const bool k = (i < len) && flag[i] != 0;
    int tot;
    const int r = block_flag_scan(k, sh, tot);
    if (k) out[kept + r] = i;
    kept += tot;
  }
  if (threadIdx.x == 0) new_len[c] = kept;
}

__global__ void h2o_budget_kernel(const int32_t* __restrict__ fill, int n, double heavy_ratio,
                                  double recent_ratio, int32_t* __restrict__ n_heavy,
                                  int32_t* __restrict__ n_recent) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const double len = (double)fill[c];
  int h = (int)(len * heavy_ratio);
  int r = (int)(len * recent_ratio);
  n_heavy[c] = h < 1 ? 1 : h;
  n_recent[c] = r < 1 ? 1 : r;
}

// ---- compaction -------------------------------------------------------------------
struct CompactPlanes {
  void* ptr[PIKV_MAX_PLANES];
  int64_t row_bytes[PIKV_MAX_PLANES];
  int slab_begin[PIKV_MAX_PLANES + 1];  // prefix of slabs per plane
  int n_planes;
};

constexpr int kSlabBytes = 256;
constexpr int kRowsUnroll = 4;

template <typename V>
__device__ __forceinline__ void compact_slab(char* plane, int64_t row_bytes, int64_t base_row,
                                             int64_t col0, int slab_bytes,
                                             const int32_t* __restrict__ keep, int m) {
  const int lanes_per_row = slab_bytes / (int)sizeof(V);
  const int rows_per_pass = 256 / lanes_per_row;
  const int lane_in_row = threadIdx.x % lanes_per_row;
  const int row_in_pass = threadIdx.x / lanes_per_row;
  const bool active = row_in_pass < rows_per_pass;  // 256 % lanes_per_row may be non-zero
  const int step_rows = rows_per_pass * kRowsUnroll;
  const int64_t col = col0 + (int64_t)lane_in_row * sizeof(V);
  for (int j0 = 0; j0 < m; j0 += step_rows) {
    V val[kRowsUnroll];
    int src[kRowsUnroll];
#pragma unroll
    for (int u = 0; u < kRowsUnroll; ++u) {
      const int j = j0 + u * rows_per_pass + row_in_pass;
      src[u] = -1;
      val[u] = V{};
      if (active && j < m) {
        const int s = keep[j];
        if (s != j) src[u] = s;
      }
      if (src[u] >= 0)
        val[u] = *reinterpret_cast<const V*>(plane + (base_row + src[u]) * row_bytes + col);
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kRowsUnroll; ++u) {
      const int j = j0 + u * rows_per_pass + row_in_pass;
      if (src[u] >= 0) *reinterpret_cast<V*>(plane + (base_row + j) * row_bytes + col) = val[u];
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(256) void compact_rows_kernel(CompactPlanes pl,
                                                           const int64_t* __restrict__ row_base,
                                                           const int32_t* __restrict__ keep_index,
                                                           const int32_t* __restrict__ new_len) {
  const int c = blockIdx.y;
  const int slab = blockIdx.x;
  int p = 0;
  while (p + 1 < pl.n_planes && slab >= pl.slab_begin[p + 1]) ++p;
  const int64_t rb = pl.row_bytes[p];
  const int64_t col0 = (int64_t)(slab - pl.slab_begin[p]) * kSlabBytes;
  const int64_t left = rb - col0;
  const int slab_bytes = left < kSlabBytes ? (int)left : kSlabBytes;
  const int64_t base = row_base[c];
  const int m = new_len[c];
  const int32_t* keep = keep_index + base;
  char* plane = reinterpret_cast<char*>(pl.ptr[p]);
  if (rb % 16 == 0)
    compact_slab<uint4>(plane, rb, base, col0, slab_bytes, keep, m);
  else
    compact_slab<uint32_t>(plane, rb, base, col0, slab_bytes, keep, m);
}

__global__ void set_fill_kernel(int32_t* __restrict__ fill, const int32_t* __restrict__ new_len, int n) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c < n) fill[c] = new_len[c];
}

}  // namespace pikv

using namespace pikv;

extern "C" int pikv_evict_select(int policy, const float* row_acc, const float* row_ts,
                                 const int64_t* cache_row_base, const int32_t* cache_fill,
                                 const int32_t* n_heavy, const int32_t* n_recent, int n_caches,
                                 uint8_t* keep_flag, int32_t* keep_index, int32_t* new_len,
                                 void* stream) {
  if (!row_ts || !cache_row_base || !cache_fill || !n_heavy || !keep_flag || !keep_index || !new_len)
    return PIKV_ERR_NULL;
  if (policy != PIKV_EVICT_H2O && policy != PIKV_EVICT_LRU) return PIKV_ERR_UNSUPPORTED;
  if (policy == PIKV_EVICT_H2O && (!row_acc || !n_recent)) return PIKV_ERR_NULL;
  if (n_caches < 1) return PIKV_ERR_SHAPE;
  hipLaunchKernelGGL(evict_select_kernel, dim3((unsigned)n_caches), dim3(kSelThreads), 0,
                     (hipStream_t)stream, policy, row_acc, row_ts, cache_row_base, cache_fill,
                     n_heavy, n_recent, keep_flag, keep_index, new_len);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

extern "C" int pikv_h2o_budget(const int32_t* cache_fill, int n_caches, double heavy_ratio,
                               double recent_ratio, int32_t* n_heavy, int32_t* n_recent,
                               void* stream) {
  if (!cache_fill || !n_heavy || !n_recent) return PIKV_ERR_NULL;
  if (n_caches < 1) return PIKV_ERR_SHAPE;
  hipLaunchKernelGGL(h2o_budget_kernel, dim3((n_caches + 63) / 64), dim3(64), 0, (hipStream_t)stream,
                     cache_fill, n_caches, heavy_ratio, recent_ratio, n_heavy, n_recent);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

extern "C" int pikv_compact_rows(void* const* plane_ptrs_host, const int64_t* plane_row_bytes_host,
                                 int n_planes, const int64_t* cache_row_base,
                                 const int32_t* keep_index, const int32_t* new_len,
                                 int32_t* cache_fill, int n_caches, void* stream) {
  if (!plane_ptrs_host || !plane_row_bytes_host || !cache_row_base || !keep_index || !new_len)
    return PIKV_ERR_NULL;
  if (n_planes < 0 || n_planes > PIKV_MAX_PLANES || n_caches < 1 || n_caches > 65535)
    return PIKV_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  if (n_planes > 0) {
    CompactPlanes pl{};
    pl.n_planes = n_planes;
    int slabs = 0;
    for (int p = 0; p < n_planes; ++p) {
      if (!plane_ptrs_host[p]) return PIKV_ERR_NULL;
      const int64_t rb = plane_row_bytes_host[p];
      if (rb <= 0 || rb % 4 != 0 || rb > (1 << 24)) return PIKV_ERR_SHAPE;
      pl.ptr[p] = plane_ptrs_host[p];
      pl.row_bytes[p] = rb;
      pl.slab_begin[p] = slabs;
      slabs += (int)((rb + kSlabBytes - 1) / kSlabBytes);
    }
    pl.slab_begin[n_planes] = slabs;
    hipLaunchKernelGGL(compact_rows_kernel, dim3((unsigned)slabs, (unsigned)n_caches), dim3(256), 0,
                       st, pl, cache_row_base, keep_index, new_len);
  }
  if (cache_fill)
    hipLaunchKernelGGL(set_fill_kernel, dim3((n_caches + 63) / 64), dim3(64), 0, st, cache_fill,
                       new_len, n_caches);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
