// K4: eviction top-k selection and stable in-place compaction.
//
// Selection: one 1024-thread block per cache.  A float is mapped to a 32-bit key
// whose unsigned order is the float order; an MSB-first radix select (4 passes of
// 8 bits, one LDS histogram per wavefront) finds the key of the m-th largest
// element, and an ordered marking pass takes every larger element plus the first
// (lowest-index) elements equal to it.  Caches of up to 32768 rows keep their keys
// in registers between the passes.  Total order = (value desc, index asc); the "smallest m"
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
constexpr int kSelItems = 32;  // keys a thread keeps in registers (caches of <= 32768 rows)

__device__ __forceinline__ uint32_t order_key(float v, bool smallest) {
  v = v + 0.0f;  // -0 -> +0 so that they tie
  uint32_t u = __float_as_uint(v);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return smallest ? ~u : u;
}

struct SelShared {
  int whist[kSelWaves][256];  // one digit histogram per wavefront
  int hist[256];
  int wtot[kSelWaves];
  int pick_digit, pick_rem;
};

// Element order inside the block: wavefront w owns the contiguous segment
// [w*items*64, (w+1)*items*64); its round j covers 64 consecutive elements, one
// per lane.  Prefix counts in index order are then ballots inside a round, a
// running count over the rounds of a wavefront, and one 16-entry scan across
// wavefronts.
struct SelGeom {
  int len, items, lane, wave, seg0;
  __device__ __forceinline__ int index(int j) const { return seg0 + j * 64 + lane; }
};

// Exclusive prefix over the wavefronts of a per-wavefront total (uniform in the
// wavefront).  All threads call.
__device__ __forceinline__ int wave_base(int total, const SelGeom& g, SelShared& s) {
  __syncthreads();  // previous use of wtot is over
  if (g.lane == 0) s.wtot[g.wave] = total;
  __syncthreads();
  int pre = 0;
#pragma unroll
  for (int w = 0; w < kSelWaves; ++w)
    if (w < g.wave) pre += s.wtot[w];
  return pre;
}

// Run f(j) for every round of this thread; fully unrolled when the keys sit in
// registers so that the register array is indexed by constants only.
template <bool CACHED, typename F>
__device__ __forceinline__ void for_rounds(const SelGeom& g, F&& f) {
  if constexpr (CACHED) {
#pragma unroll
    for (int j = 0; j < kSelItems; ++j) {
      if (j < g.items) f(j);  // uniform
    }
  } else {
    for (int j = 0; j < g.items; ++j) f(j);
  }
}

// Mark the m top elements of v[0..len): flag[i] = mark.  All threads must call.
// CACHED: every thread holds its <= kSelItems keys in registers across the passes.
template <bool CACHED>
__device__ void block_select_mark(const float* __restrict__ v, int m, bool smallest,
                                  uint8_t* __restrict__ flag, uint8_t mark, const SelGeom& g,
                                  SelShared& s) {
  const int len = g.len;
  if (m <= 0 || len <= 0) return;  // uniform
  if (m >= len) {  // every thread marks its own elements
    for (int j = 0; j < g.items; ++j)
      if (g.index(j) < len) flag[g.index(j)] = mark;
    return;
  }
  uint32_t kreg[CACHED ? kSelItems : 1];
  uint32_t vbits = 0;  // CACHED: bit j = round j holds an element
  if (CACHED) {
#pragma unroll
    for (int j = 0; j < kSelItems; ++j) {
      const int i = g.index(j);
      kreg[j] = 0;
      if (j < g.items && i < len) {
        kreg[j] = order_key(v[i], smallest);
        vbits |= 1u << j;
      }
    }
  }
  auto fetch = [&](int j, uint32_t& key) -> bool {
    if (CACHED) {
      key = kreg[j];
      return (vbits >> j) & 1u;
    }
    const int i = g.index(j);
    if (i >= len) return false;
    key = order_key(v[i], smallest);
    return true;
  };
  const uint64_t lt = (g.lane == 0) ? 0ull : (~0ull >> (64 - g.lane));

  uint32_t prefix = 0, pmask = 0;
  int remaining = m;
  for (int shift = 24; shift >= 0; shift -= 8) {
    __syncthreads();  // the histograms of the previous pass have been read
    *reinterpret_cast<int4*>(&s.whist[g.wave][g.lane * 4]) = make_int4(0, 0, 0, 0);
    for_rounds<CACHED>(g, [&](int j) {
      uint32_t key = 0;
      bool act = fetch(j, key);
      act = act && ((key & pmask) == prefix);
      const uint64_t am = __ballot(act);
      if (am == 0) return;  // uniform
      const int d = (key >> shift) & 255u;
      // floats of similar magnitude share their leading digit: count the first
      // active lane's digit with one ballot, the rest with LDS atomics
      const int lead = __builtin_ctzll(am);
      const int ld = __builtin_amdgcn_readlane(d, lead);
      const uint64_t mm = __ballot(act && d == ld);
      if (g.lane == lead) atomicAdd(&s.whist[g.wave][ld], __popcll(mm));
      if (act && d != ld) atomicAdd(&s.whist[g.wave][d], 1);
    });
    __syncthreads();
    if (threadIdx.x < 256) {
      int h = 0;
#pragma unroll
      for (int w = 0; w < kSelWaves; ++w) h += s.whist[w][threadIdx.x];
      s.hist[threadIdx.x] = h;
    }
    __syncthreads();
    if (g.wave == 0) {
      // lane l owns digits 255-4l .. 252-4l (descending); find the digit where the
      // running count from the top first reaches `remaining`
      int cnt[4], tot = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        cnt[k] = s.hist[255 - 4 * g.lane - k];
        tot += cnt[k];
      }
      int incl = tot;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int o = __shfl_up(incl, off, 64);
        if (g.lane >= off) incl += o;
      }
      int before = incl - tot;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (before < remaining && remaining <= before + cnt[k]) {
          s.pick_digit = 255 - 4 * g.lane - k;
          s.pick_rem = remaining - before;
        }
        before += cnt[k];
      }
    }
    __syncthreads();
    prefix |= (uint32_t)s.pick_digit << shift;
    pmask |= 255u << shift;
    remaining = s.pick_rem;
  }
  // prefix = key of the m-th element; `remaining` of the elements equal to it are
  // taken, lowest index first.
  int weq = 0;
  for_rounds<CACHED>(g, [&](int j) {
    uint32_t key = 0;
    const bool ok = fetch(j, key);
    weq += __popcll(__ballot(ok && key == prefix));
  });
  int rank = wave_base(weq, g, s);
  for_rounds<CACHED>(g, [&](int j) {
    uint32_t key = 0;
    const bool ok = fetch(j, key);
    const bool eq = ok && key == prefix;
    const bool gt = ok && key > prefix;
    const uint64_t eb = __ballot(eq);
    if (gt || (eq && rank + __popcll(eb & lt) < remaining)) flag[g.index(j)] = mark;
    rank += __popcll(eb);
  });
}

template <bool CACHED>
__device__ void evict_select_body(int policy, const float* __restrict__ acc,
                                  const float* __restrict__ ts, int n_heavy, int n_recent,
                                  uint8_t* __restrict__ flag, int32_t* __restrict__ out,
                                  int32_t* __restrict__ new_len_c, const SelGeom& g, SelShared& s) {
  const int rounds = g.items;
  // a thread initialises, marks and later reads only its own flags: no barrier needed for them
  const uint8_t init = (policy == PIKV_EVICT_H2O) ? 0 : 1;
  for (int j = 0; j < rounds; ++j) {
    const int i = g.index(j);
    if (i < g.len) flag[i] = init;
  }
  if (policy == PIKV_EVICT_H2O) {
    block_select_mark<CACHED>(acc, n_heavy, false, flag, 1, g, s);
    block_select_mark<CACHED>(ts, n_recent, false, flag, 1, g, s);
  } else {
    block_select_mark<CACHED>(ts, n_heavy, true, flag, 0, g, s);
  }
  // Ascending list of survivors.
  const uint64_t lt = (g.lane == 0) ? 0ull : (~0ull >> (64 - g.lane));
  int wk = 0;
  for (int j = 0; j < rounds; ++j) {
    const int i = g.index(j);
    wk += __popcll(__ballot(i < g.len && flag[i] != 0));
  }
  int pos = wave_base(wk, g, s);
  for (int j = 0; j < rounds; ++j) {
    const int i = g.index(j);
    const bool k = i < g.len && flag[i] != 0;
    const uint64_t kb = __ballot(k);
    if (k) out[pos + __popcll(kb & lt)] = i;
    pos += __popcll(kb);
  }
  if (threadIdx.x == kSelThreads - 1) *new_len_c = pos;  // the last wavefront ends at the total
}

__global__ __launch_bounds__(kSelThreads) void evict_select_kernel(
    int policy, const float* __restrict__ row_acc, const float* __restrict__ row_ts,
    const int64_t* __restrict__ row_base, const int32_t* __restrict__ fill,
    const int32_t* __restrict__ n_heavy, const int32_t* __restrict__ n_recent,
    uint8_t* __restrict__ keep_flag, int32_t* __restrict__ keep_index, int32_t* __restrict__ new_len) {
  __shared__ SelShared s;
  const int c = blockIdx.x;
  const int len = fill[c];
  const int64_t base = row_base[c];
  if (len <= 0) {
    if (threadIdx.x == 0) new_len[c] = 0;
    return;
  }
  SelGeom g;
  g.len = len;
  g.items = (len + kSelThreads - 1) / kSelThreads;
  g.lane = threadIdx.x & 63;
  g.wave = threadIdx.x >> 6;
  g.seg0 = g.wave * g.items * 64;
  const float* acc = row_acc ? row_acc + base : nullptr;
  const int nh = n_heavy[c];
  const int nr = (policy == PIKV_EVICT_H2O) ? n_recent[c] : 0;
  if (g.items <= kSelItems)
    evict_select_body<true>(policy, acc, row_ts + base, nh, nr, keep_flag + base, keep_index + base,
                            new_len + c, g, s);
  else
    evict_select_body<false>(policy, acc, row_ts + base, nh, nr, keep_flag + base, keep_index + base,
                             new_len + c, g, s);
}

// ---- multi-block selection ---------------------------------------------------------
// Long caches are cut into chunks of kMbChunk rows, one 256-thread block each.  The
// order-preserving key is split into three digits (11 + 11 + 10 bits); pass p builds
// the histogram of digit p over the keys that match the digits already chosen
// (integer atomics into a per-cache table, so the result does not depend on
// scheduling), and every later kernel re-derives the chosen digits from the tables.
// Kernels, in stream order: zero tables | hist 0 | hist 1 | hist 2 | mark | list.
// A thread owns 16 CONSECUTIVE rows, so ranks in index order are a thread-local count
// plus one block scan plus the per-chunk counts of the earlier chunks.
constexpr int kMbThreads = 256;
constexpr int kMbItems = 16;  // 8 measured the same, 32 slower (99 vs 75 us at 64 x 32768)
constexpr int kMbChunk = kMbThreads * kMbItems;
constexpr int kMbBins = 2048;

struct MbArgs {
  int policy;
  const float* acc;
  const float* ts;
  const int64_t* row_base;
  const int32_t* fill;
  const int32_t* n_heavy;
  const int32_t* n_recent;
  uint8_t* keep_flag;
  int32_t* keep_index;
  int32_t* new_len;
  int* hist;       // [cache][pass 0..2][slot 0..1][kMbBins]
  int* blk_hist2;  // [cache][chunk][slot][1024]: last-digit histogram of every chunk
  int* blk_kept;   // [cache][chunk]
  int n_chunks;
};

__device__ __forceinline__ int mb_digit(uint32_t key, int pass) {
  return pass == 0 ? (int)(key >> 21) : pass == 1 ? (int)((key >> 10) & 2047u) : (int)(key & 1023u);
}
__device__ __forceinline__ uint32_t mb_mask(int passes_done) {
  return passes_done == 0 ? 0u : passes_done == 1 ? 0xffe00000u : passes_done == 2 ? 0xfffffc00u : 0xffffffffu;
}

// Selection `slot` of cache c: H2O slot 0 = n_heavy largest of acc, slot 1 = n_recent
// largest of ts; LRU slot 0 = n_evict smallest of ts.  m is clamped to [0, len].
struct MbSel {
  const float* v;
  bool smallest;
  int m;
  bool used;     // the slot exists for this policy
  bool partial;  // 0 < m < len: a threshold has to be found
};
__device__ __forceinline__ MbSel mb_sel(const MbArgs& a, int c, int slot, int len) {
  MbSel s;
  const int64_t base = a.row_base[c];
  if (a.policy == PIKV_EVICT_H2O) {
    s.v = (slot == 0 ? a.acc : a.ts) + base;
    s.smallest = false;
    s.m = slot == 0 ? a.n_heavy[c] : a.n_recent[c];
    s.used = true;
  } else {
    s.v = a.ts + base;
    s.smallest = true;
    s.m = a.n_heavy[c];
    s.used = slot == 0;
  }
  s.m = s.m < 0 ? 0 : (s.m > len ? len : s.m);
  s.partial = s.used && s.m > 0 && s.m < len;
  return s;
}

// Exclusive prefix of v over the 256 threads (thread order); total to all.
__device__ __forceinline__ int mb_block_scan(int v, int* sh /*4*/, int& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(incl, off, 64);
    if (lane >= off) incl += o;
  }
  __syncthreads();
  if (lane == 63) sh[wave] = incl;
  __syncthreads();
  int pre = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int t = sh[w];
    if (w < wave) pre += t;
    tot += t;
  }
  total = tot;
  return pre + incl - v;
}

// Digit at which the running count from the top first reaches `remaining`; remaining
// becomes the count still to take inside that digit.  All threads call; nb is 2048 or 1024.
__device__ __forceinline__ int mb_pick(const int* __restrict__ hist, int nb, int& remaining, int* sh /*6*/) {
  const int per = nb / kMbThreads;  // 8 or 4
  int cnt[8], tot = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    cnt[k] = k < per ? hist[nb - 1 - (threadIdx.x * per + k)] : 0;
    tot += cnt[k];
  }
  int all;
  int before = mb_block_scan(tot, sh, all);
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    if (k < per && before < remaining && remaining <= before + cnt[k]) {
      sh[4] = nb - 1 - (threadIdx.x * per + k);
      sh[5] = remaining - before;
    }
    before += cnt[k];
  }
  __syncthreads();
  remaining = sh[5];
  return sh[4];
}

// Digits chosen by the first `passes` passes for one slot: key prefix and what remains.
__device__ __forceinline__ uint32_t mb_prefix(const MbArgs& a, int c, int slot, int passes, int& remaining,
                                              int* sh, int* last_digit) {
  uint32_t prefix = 0;
  for (int p = 0; p < passes; ++p) {
    const int* h = a.hist + (((int64_t)c * 3 + p) * 2 + slot) * kMbBins;
    const int d = mb_pick(h, p == 2 ? 1024 : kMbBins, remaining, sh);
    prefix |= (uint32_t)d << (p == 0 ? 21 : p == 1 ? 10 : 0);
    if (last_digit) *last_digit = d;
  }
  return prefix;
}

__global__ void mb_zero_kernel(int* __restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

template <int PASS>
__global__ __launch_bounds__(kMbThreads) void mb_hist_kernel(MbArgs a) {
  __shared__ int lh[kMbBins];
  __shared__ int sh[8];
  const int c = blockIdx.y, chunk = blockIdx.x;
  const int len = a.fill[c];
  const int64_t i0 = (int64_t)chunk * kMbChunk + threadIdx.x * kMbItems;
  constexpr int NB = PASS == 2 ? 1024 : kMbBins;
  // the two selections of a cache run in different blocks (grid z): half the serial work each
  for (int slot = blockIdx.z; slot <= (int)blockIdx.z; ++slot) {
    const MbSel s = mb_sel(a, c, slot, len);
    int* bh = PASS == 2 ? a.blk_hist2 + (((int64_t)c * a.n_chunks + chunk) * 2 + slot) * 1024 : nullptr;
    // (no table for such a chunk: the marking pass reads the tables of chunks before one that
    // lies inside the cache, for selections that need a threshold)
    if (!s.partial || (int64_t)chunk * kMbChunk >= len) continue;  // uniform
    int remaining = s.m;
    const uint32_t prefix = mb_prefix(a, c, slot, PASS, remaining, sh, nullptr);
    const uint32_t pmask = mb_mask(PASS);
    for (int b = threadIdx.x; b < NB; b += kMbThreads) lh[b] = 0;
    __syncthreads();
    // neighbouring rows often share a digit (timestamps grow along the cache, scores of a
    // region are of one magnitude): a run of equal digits costs one LDS atomic, not one per row
    int run_digit = -1, run = 0;
#pragma unroll
    for (int j = 0; j < kMbItems; ++j) {
      int d = -1;
      if (i0 + j < len) {
        const uint32_t key = order_key(s.v[i0 + j], s.smallest);
        if ((key & pmask) == prefix) d = mb_digit(key, PASS);
      }
      if (d != run_digit) {
        if (run_digit >= 0) atomicAdd(&lh[run_digit], run);
        run_digit = d;
        run = 0;
      }
      ++run;
    }
    if (run_digit >= 0) atomicAdd(&lh[run_digit], run);
    __syncthreads();
    int* gh = a.hist + (((int64_t)c * 3 + PASS) * 2 + slot) * kMbBins;
    for (int b = threadIdx.x; b < NB; b += kMbThreads) {
      const int n = lh[b];
      if (PASS == 2) bh[b] = n;
      if (n) atomicAdd(&gh[b], n);
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kMbThreads) void mb_mark_kernel(MbArgs a) {
  __shared__ int sh[8];
  const int c = blockIdx.y, chunk = blockIdx.x;
  const int len = a.fill[c];
  const int64_t i0 = (int64_t)chunk * kMbChunk + threadIdx.x * kMbItems;
  if ((int64_t)chunk * kMbChunk >= len) {  // uniform
    if (threadIdx.x == 0) a.blk_kept[(int64_t)c * a.n_chunks + chunk] = 0;
    return;
  }
  uint32_t selbits[2] = {0u, 0u};  // bit j: row i0+j is taken by the slot's selection
  for (int slot = 0; slot < 2; ++slot) {
    const MbSel s = mb_sel(a, c, slot, len);
    if (!s.used || s.m <= 0) continue;  // uniform
    if (s.m >= len) {
      selbits[slot] = (1u << kMbItems) - 1u;
      continue;
    }
    int remaining = s.m, d2 = 0;
    const uint32_t kstar = mb_prefix(a, c, slot, 3, remaining, sh, &d2);
    // rows equal to the threshold key in earlier chunks
    int part = 0;
    for (int b = threadIdx.x; b < chunk; b += kMbThreads)
      part += a.blk_hist2[(((int64_t)c * a.n_chunks + b) * 2 + slot) * 1024 + d2];
    int eq_before;
    mb_block_scan(part, sh, eq_before);
    uint32_t gt = 0, eq = 0;
#pragma unroll
    for (int j = 0; j < kMbItems; ++j) {
      if (i0 + j < len) {
        const uint32_t key = order_key(s.v[i0 + j], s.smallest);
        gt |= (key > kstar ? 1u : 0u) << j;
        eq |= (key == kstar ? 1u : 0u) << j;
      }
    }
    int tot;
    int rank = eq_before + mb_block_scan(__popc(eq), sh, tot);
    uint32_t take = gt;
#pragma unroll
    for (int j = 0; j < kMbItems; ++j) {
      if ((eq >> j) & 1u) {
        if (rank < remaining) take |= 1u << j;
        ++rank;
      }
    }
    selbits[slot] = take;
  }
  uint32_t valid = 0;
#pragma unroll
  for (int j = 0; j < kMbItems; ++j) valid |= (i0 + j < len ? 1u : 0u) << j;
  const uint32_t keep = (a.policy == PIKV_EVICT_H2O ? (selbits[0] | selbits[1]) : ~selbits[0]) & valid;
  uint8_t* flag = a.keep_flag + a.row_base[c];
  static_assert(kMbItems == 16, "sixteen flags = one 16-byte store");
  if (valid == 0xffffu && (reinterpret_cast<uintptr_t>(flag + i0) & 15) == 0) {
    // four bits -> four 0/1 bytes: the shifts 0, 7, 14, 21 put bit k at bit 8 k
    auto spread = [](uint32_t nib) { return ((nib & 0xfu) * 0x00204081u) & 0x01010101u; };
    *reinterpret_cast<uint4*>(flag + i0) =
        make_uint4(spread(keep), spread(keep >> 4), spread(keep >> 8), spread(keep >> 12));
  } else {
#pragma unroll
    for (int j = 0; j < kMbItems; ++j)
      if ((valid >> j) & 1u) flag[i0 + j] = (keep >> j) & 1u;
  }
  int kept;
  mb_block_scan(__popc(keep), sh, kept);
  if (threadIdx.x == 0) a.blk_kept[(int64_t)c * a.n_chunks + chunk] = kept;
}

__global__ __launch_bounds__(kMbThreads) void mb_list_kernel(MbArgs a) {
  __shared__ int sh[8];
  const int c = blockIdx.y, chunk = blockIdx.x;
  const int len = a.fill[c];
  // survivors in the earlier chunks, and (chunk 0) in all of them
  int before = 0, all = 0;
  const int lim = chunk == 0 ? a.n_chunks : chunk;
  for (int b = threadIdx.x; b < lim; b += kMbThreads) before += a.blk_kept[(int64_t)c * a.n_chunks + b];
  mb_block_scan(before, sh, all);
  if (chunk == 0) {
    if (threadIdx.x == 0) a.new_len[c] = len > 0 ? all : 0;
    all = 0;
  }
  if ((int64_t)chunk * kMbChunk >= len) return;  // uniform
  const int64_t i0 = (int64_t)chunk * kMbChunk + threadIdx.x * kMbItems;
  const uint8_t* flag = a.keep_flag + a.row_base[c];
  uint32_t keep = 0;
  if (i0 + kMbItems <= len && (reinterpret_cast<uintptr_t>(flag + i0) & 15) == 0) {
    // four 0/1 bytes -> four bits: the shifts 3, 10, 17, 24 collect them in bits 24..27
    const uint4 f = *reinterpret_cast<const uint4*>(flag + i0);
    auto gather = [](uint32_t w) { return (((w & 0x01010101u) * 0x01020408u) >> 24) & 0xfu; };
    keep = gather(f.x) | (gather(f.y) << 4) | (gather(f.z) << 8) | (gather(f.w) << 12);
  } else {
#pragma unroll
    for (int j = 0; j < kMbItems; ++j)
      if (i0 + j < len && flag[i0 + j]) keep |= 1u << j;
  }
  // the chunk's survivors are gathered in LDS and leave as one contiguous run
  __shared__ int32_t run[kMbChunk];
  int tot;
  int pos = mb_block_scan(__popc(keep), sh, tot);
#pragma unroll
  for (int j = 0; j < kMbItems; ++j)
    if ((keep >> j) & 1u) run[pos++] = (int32_t)(i0 + j);
  __syncthreads();
  int32_t* out = a.keep_index + a.row_base[c] + all;
  for (int i = threadIdx.x; i < tot; i += kMbThreads) out[i] = run[i];
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
constexpr int kRowsUnroll = 16;

// Survivor j of a cache moves from row keep[j] to row j (keep ascending, keep[j] >= j).
// The m survivors split at j* = first j with keep[j] >= m:
//   head (j < j*): sources lie inside the final region [0, m) and are themselves
//     destinations of other survivors, so the moves are ordered - one block walks them in
//     ascending passes, every pass reads all its rows before it writes any;
//   tail (j >= j*): sources lie beyond the final region, nobody writes them, and their
//     destinations [j*, m) are read by the head only - once the head is done they can move
//     in any order, by as many blocks as there are.
// After an eviction that keeps a small fraction nearly every survivor is in the tail.
template <typename V, bool TAIL>
__device__ __forceinline__ void compact_slab(char* plane, int64_t row_bytes, int64_t base_row,
                                             int64_t col0, int slab_bytes,
                                             const int32_t* __restrict__ keep, int j_begin, int j_end,
                                             int chunk, int n_chunks) {
  const int lanes_per_row = slab_bytes / (int)sizeof(V);
  const int rows_per_pass = 256 / lanes_per_row;
  const int lane_in_row = threadIdx.x % lanes_per_row;
  const int row_in_pass = threadIdx.x / lanes_per_row;
  const bool active = row_in_pass < rows_per_pass;  // 256 % lanes_per_row may be non-zero
  const int step_rows = rows_per_pass * kRowsUnroll;
  const int64_t col = col0 + (int64_t)lane_in_row * sizeof(V);
  for (int j0 = j_begin + chunk * step_rows; j0 < j_end; j0 += n_chunks * step_rows) {
    V val[kRowsUnroll];
    int src[kRowsUnroll];
#pragma unroll
    for (int u = 0; u < kRowsUnroll; ++u) {
      const int j = j0 + u * rows_per_pass + row_in_pass;
      src[u] = -1;
      val[u] = V{};
      if (active && j < j_end) {
        const int s = keep[j];
        if (s != j) src[u] = s;
      }
      if (src[u] >= 0)
        val[u] = *reinterpret_cast<const V*>(plane + (base_row + src[u]) * row_bytes + col);
    }
    if (!TAIL) __syncthreads();
#pragma unroll
    for (int u = 0; u < kRowsUnroll; ++u) {
      const int j = j0 + u * rows_per_pass + row_in_pass;
      if (src[u] >= 0) *reinterpret_cast<V*>(plane + (base_row + j) * row_bytes + col) = val[u];
    }
    if (!TAIL) __syncthreads();
  }
}

// grid (slabs of all planes, caches, chunks).  TAIL = false: chunks == 1.
template <bool TAIL>
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
  // j* = first survivor whose source lies beyond the final region (binary search, uniform)
  int lo = 0, hi = m;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (keep[mid] >= m) hi = mid; else lo = mid + 1;
  }
  const int j_begin = TAIL ? lo : 0;
  const int j_end = TAIL ? m : lo;
  if (j_begin >= j_end) return;  // uniform
  char* plane = reinterpret_cast<char*>(pl.ptr[p]);
  const int chunk = TAIL ? (int)blockIdx.z : 0;
  const int n_chunks = TAIL ? (int)gridDim.z : 1;
  // widest element that every row start is aligned to
  if (rb % 16 == 0)
    compact_slab<uint4, TAIL>(plane, rb, base, col0, slab_bytes, keep, j_begin, j_end, chunk, n_chunks);
  else if (rb % 4 == 0)
    compact_slab<uint32_t, TAIL>(plane, rb, base, col0, slab_bytes, keep, j_begin, j_end, chunk, n_chunks);
  else if (rb % 2 == 0)
    compact_slab<uint16_t, TAIL>(plane, rb, base, col0, slab_bytes, keep, j_begin, j_end, chunk, n_chunks);
  else
    compact_slab<uint8_t, TAIL>(plane, rb, base, col0, slab_bytes, keep, j_begin, j_end, chunk, n_chunks);
}

__global__ void set_fill_kernel(int32_t* __restrict__ fill, const int32_t* __restrict__ new_len, int n) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c < n) fill[c] = new_len[c];
}

}  // namespace pikv

using namespace pikv;

static int64_t mb_chunks(int64_t max_len) { return (max_len + kMbChunk - 1) / kMbChunk; }

extern "C" int64_t pikv_evict_workspace_bytes(int n_caches, int64_t max_len) {
  if (n_caches < 1 || max_len < 0) return 0;
  const int64_t nch = mb_chunks(max_len);
  return (int64_t)n_caches * (3 * 2 * kMbBins + nch * 2 * 1024 + nch) * (int64_t)sizeof(int);
}

extern "C" int pikv_evict_select(int policy, const float* row_acc, const float* row_ts,
                                 const int64_t* cache_row_base, const int32_t* cache_fill,
                                 const int32_t* n_heavy, const int32_t* n_recent, int n_caches,
                                 int64_t max_len, uint8_t* keep_flag, int32_t* keep_index,
                                 int32_t* new_len, void* workspace, int64_t workspace_bytes,
                                 void* stream) {
  if (!row_ts || !cache_row_base || !cache_fill || !n_heavy || !keep_flag || !keep_index || !new_len)
    return PIKV_ERR_NULL;
  if (policy != PIKV_EVICT_H2O && policy != PIKV_EVICT_LRU) return PIKV_ERR_UNSUPPORTED;
  if (policy == PIKV_EVICT_H2O && (!row_acc || !n_recent)) return PIKV_ERR_NULL;
  if (n_caches < 1 || max_len < 0) return PIKV_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  // caches of more than two chunks are worth several blocks each, when the caller
  // brought the tables
  if (workspace && max_len > 2 * kMbChunk) {
    if (n_caches > 65535) return PIKV_ERR_SHAPE;
    if (workspace_bytes < pikv_evict_workspace_bytes(n_caches, max_len)) return PIKV_ERR_WORKSPACE;
    const int64_t nch = mb_chunks(max_len);
    if (nch > 0x7fffffffLL) return PIKV_ERR_SHAPE;
    MbArgs a{policy, row_acc, row_ts, cache_row_base, cache_fill, n_heavy, n_recent, keep_flag,
             keep_index, new_len, nullptr, nullptr, nullptr, (int)nch};
    a.hist = reinterpret_cast<int*>(workspace);
    a.blk_hist2 = a.hist + (int64_t)n_caches * 3 * 2 * kMbBins;
    a.blk_kept = a.blk_hist2 + (int64_t)n_caches * nch * 2 * 1024;
    const int64_t nz = (int64_t)n_caches * 3 * 2 * kMbBins;
    hipLaunchKernelGGL(mb_zero_kernel, dim3((unsigned)((nz + 255) / 256)), dim3(256), 0, st, a.hist, nz);
    const dim3 grid((unsigned)nch, (unsigned)n_caches);
    const dim3 grid2((unsigned)nch, (unsigned)n_caches, 2);
    hipLaunchKernelGGL(mb_hist_kernel<0>, grid2, dim3(kMbThreads), 0, st, a);
    hipLaunchKernelGGL(mb_hist_kernel<1>, grid2, dim3(kMbThreads), 0, st, a);
    hipLaunchKernelGGL(mb_hist_kernel<2>, grid2, dim3(kMbThreads), 0, st, a);
    hipLaunchKernelGGL(mb_mark_kernel, grid, dim3(kMbThreads), 0, st, a);
    hipLaunchKernelGGL(mb_list_kernel, grid, dim3(kMbThreads), 0, st, a);
    PIKV_CHECK_LAUNCH();
    return PIKV_OK;
  }
  hipLaunchKernelGGL(evict_select_kernel, dim3((unsigned)n_caches), dim3(kSelThreads), 0, st, policy,
                     row_acc, row_ts, cache_row_base, cache_fill, n_heavy, n_recent, keep_flag,
                     keep_index, new_len);
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
      if (rb <= 0 || rb > (1 << 24)) return PIKV_ERR_SHAPE;
      pl.ptr[p] = plane_ptrs_host[p];
      pl.row_bytes[p] = rb;
      pl.slab_begin[p] = slabs;
      slabs += (int)((rb + kSlabBytes - 1) / kSlabBytes);
    }
    pl.slab_begin[n_planes] = slabs;
    // ordered head first, then the free-moving tail spread over enough blocks to fill the chip
    hipLaunchKernelGGL(compact_rows_kernel<false>, dim3((unsigned)slabs, (unsigned)n_caches), dim3(256), 0,
                       st, pl, cache_row_base, keep_index, new_len);
    int64_t chunks = 4096 / ((int64_t)slabs * n_caches);
    chunks = chunks < 1 ? 1 : (chunks > 64 ? 64 : chunks);
    hipLaunchKernelGGL(compact_rows_kernel<true>, dim3((unsigned)slabs, (unsigned)n_caches, (unsigned)chunks),
                       dim3(256), 0, st, pl, cache_row_base, keep_index, new_len);
  }
  if (cache_fill)
    hipLaunchKernelGGL(set_fill_kernel, dim3((n_caches + 63) / 64), dim3(64), 0, st, cache_fill,
                       new_len, n_caches);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
