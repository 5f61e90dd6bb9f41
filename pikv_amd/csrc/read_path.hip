// K3: gather + dequantise read path, QK^T scores over the compressed cache,
// softmax statistics and H2O importance accumulation.
//
// Data movement is the cost here: every cached row is 16-byte code vectors laid
// out [row][head][head_dim], so a 256-thread block reads 4 KiB of contiguous
// codes per step with one 128-bit load per lane.  A lane dequantises the 16 code
// bytes it loaded (16 or 32 elements of ONE kv head) and multiplies them with
// the matching slice of the query heads that share that kv head, held in
// registers for the whole tile; the partial dot products are reduced over the
// few lanes that make up a head.  Scores of a 64-token tile are staged in LDS so
// that they leave the CU as contiguous 256-byte rows, and the tile's softmax
// statistics (max, sum of exp) are produced from the same staging buffer, which
// lets the normalisation run as a second light pass over the scores instead of
// a second pass over the cache.
#include "common.hpp"

namespace pikv {

constexpr int kTile = PIKV_SCORE_TILE;  // cached tokens per block
static_assert(kTile == 64, "one wavefront writes one staged score row");
constexpr int kMaxQHeads = 128;  // LDS staging limit: kMaxQHeads * kTile floats

// ---- plain gather + dequantise ----------------------------------------------------
template <int SCHEME, int OUT_DT>
__global__ __launch_bounds__(256) void gather_dequant_kernel(
    const void* __restrict__ codes, const void* __restrict__ scale, const void* __restrict__ zero,
    int D, int group, const int64_t* __restrict__ rows, int64_t row0, int64_t n,
    void* __restrict__ out) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  const int lanes_per_row = D / EPL;
  const int groups_per_row = D / group;
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t i = g / lanes_per_row;
  if (i >= n) return;
  const int part = (int)(g - i * lanes_per_row);
  const int64_t row = rows ? rows[i] : row0 + i;
  const uint4 v = ld16(reinterpret_cast<const char*>(codes) + (row * lanes_per_row + part) * 16);
  int c[EPL];
  unpack_codes<SCHEME>(v, c);
  float f[EPL];
  if (group >= EPL) {
    const int64_t mi = row * groups_per_row + (part * EPL) / group;
    const float s = load_meta<SCHEME>(scale, mi);
    const float z = Q::sym ? 0.f : load_meta<SCHEME>(zero, mi);
#pragma unroll
    for (int j = 0; j < EPL; ++j) f[j] = ((float)c[j] - z) * s;
  } else {
    // several groups inside one lane (group = 16 with 4-bit codes is excluded by
    // the host check; kept for completeness of the formula)
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      const int64_t mi = row * groups_per_row + (part * EPL + j) / group;
      const float s = load_meta<SCHEME>(scale, mi);
      const float z = Q::sym ? 0.f : load_meta<SCHEME>(zero, mi);
      f[j] = ((float)c[j] - z) * s;
    }
  }
  if constexpr (OUT_DT == PIKV_F32) {
    char* o = reinterpret_cast<char*>(out) + (i * D + (int64_t)part * EPL) * 4;
#pragma unroll
    for (int j = 0; j < EPL / 4; ++j)
      st16(o + 16 * j, make_uint4(__float_as_uint(f[4 * j]), __float_as_uint(f[4 * j + 1]),
                                  __float_as_uint(f[4 * j + 2]), __float_as_uint(f[4 * j + 3])));
  } else {
    char* o = reinterpret_cast<char*>(out) + (i * D + (int64_t)part * EPL) * 2;
#pragma unroll
    for (int j = 0; j < EPL / 8; ++j) {
      uint32_t w[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        w[q] = float_to_bf16_bits(f[8 * j + 2 * q]) | (float_to_bf16_bits(f[8 * j + 2 * q + 1]) << 16);
      st16(o + 16 * j, make_uint4(w[0], w[1], w[2], w[3]));
    }
  }
}

// ---- scores ---------------------------------------------------------------------------
struct ScoreArgs {
  const void* codes;
  const void* scale;
  const void* zero;
  const void* q;
  const int64_t* row_base;
  const int32_t* fill;
  float* scores;
  float* tile_max;
  float* tile_sum;
  int64_t score_stride;
  int64_t n_tiles;
  float scale_qk;
  int group;
  int n_kv_heads;
  int n_q_heads;
  int head_dim;
};

template <int SCHEME, int REP, int Q_DT>
__global__ __launch_bounds__(256) void scores_kernel(ScoreArgs a) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  __shared__ float stage[kMaxQHeads * kTile];  // [q head][token in tile]

  const int c = blockIdx.y;
  const int64_t tile = blockIdx.x;
  const int len = a.fill[c];
  const int64_t n0 = tile * kTile;
  if (n0 >= len) return;  // uniform for the block
  const int D = a.n_kv_heads * a.head_dim;
  const int lanes_per_row = D / EPL;           // <= 256, divides 256
  const int lanes_per_head = a.head_dim / EPL; // power of two
  const int groups_per_row = D / a.group;
  const int tok_per_step = 256 / lanes_per_row;
  const int part = threadIdx.x % lanes_per_row;  // fixed (kv head, slice) of this lane
  const int tok_in_step = threadIdx.x / lanes_per_row;
  const int kvh = part / lanes_per_head;
  const int d0 = (part % lanes_per_head) * EPL;

  // Query slices of the REP heads that read this kv head, and their sums (for the
  // zero-point term: dot(q, (c - z) * s) = s * (dot(q, c) - z * sum(q))).
  float qv[REP][EPL];
  float qsum[REP];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    const int hq = kvh * REP + r;
    load_as_float<Q_DT, EPL>(a.q, ((int64_t)c * a.n_q_heads + hq) * a.head_dim + d0, qv[r]);
    float sacc = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) sacc += qv[r][j];
    qsum[r] = sacc;
  }
  const int64_t base_row = a.row_base[c];
  constexpr int UN = 4;  // token steps in flight per lane

  for (int s0 = 0; s0 < kTile; s0 += tok_per_step * UN) {
    uint4 v[UN];
    float sc[UN], zr[UN];
    bool ok[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int tl = s0 + u * tok_per_step + tok_in_step;
      const int64_t n = n0 + tl;
      ok[u] = tl < kTile && n < len;
      v[u] = make_uint4(0, 0, 0, 0);
      sc[u] = 0.f;
      zr[u] = 0.f;
      if (ok[u]) {
        const int64_t row = base_row + n;
        v[u] = ld16(reinterpret_cast<const char*>(a.codes) + (row * lanes_per_row + part) * 16);
        const int64_t mi = row * groups_per_row + (part * EPL) / a.group;
        sc[u] = load_meta<SCHEME>(a.scale, mi);
        if constexpr (!Q::sym) zr[u] = load_meta<SCHEME>(a.zero, mi);
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int tl = s0 + u * tok_per_step + tok_in_step;
      float cf[EPL];
      unpack_codes_unsigned<SCHEME>(v[u], cf);
      const float zu = zr[u] - (float)Q::qmin;  // zero point of the unsigned stored form
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) d = fmaf(qv[r][j], cf[j], d);
        d = (d - zu * qsum[r]) * sc[u];
        for (int m = 1; m < lanes_per_head; m <<= 1) d += __shfl_xor(d, m, PIKV_WAVE);
        if ((part % lanes_per_head) == 0 && tl < kTile)
          stage[(kvh * REP + r) * kTile + tl] = ok[u] ? d * a.scale_qk : -__builtin_inff();
      }
    }
  }
  __syncthreads();

  // One wavefront per query head: write the 64 scores as one 256-byte row and
  // reduce the tile's softmax statistics.
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  for (int hq = wave; hq < a.n_q_heads; hq += 4) {
    const float s = stage[hq * kTile + lane];
    const bool ok = n0 + lane < len;
    if (ok) a.scores[((int64_t)c * a.n_q_heads + hq) * a.score_stride + n0 + lane] = s;
    const float m = group_max<64>(ok ? s : -__builtin_inff());
    const float e = ok ? expf(s - m) : 0.f;
    const float sum = group_sum<64>(e);
    if (lane == 0) {
      const int64_t ti = ((int64_t)c * a.n_q_heads + hq) * a.n_tiles + tile;
      a.tile_max[ti] = m;
      a.tile_sum[ti] = sum;
    }
  }
}

// Final max and sum per (cache, q head) from the tile statistics.
__global__ __launch_bounds__(64) void head_stats_kernel(const float* __restrict__ tile_max,
                                                        const float* __restrict__ tile_sum,
                                                        const int32_t* __restrict__ fill,
                                                        int n_q_heads, int64_t n_tiles,
                                                        float* __restrict__ head_stats) {
  const int c = blockIdx.y;
  const int hq = blockIdx.x;
  const int lane = threadIdx.x;
  const int64_t used = ((int64_t)fill[c] + kTile - 1) / kTile;
  const int64_t lim = used < n_tiles ? used : n_tiles;
  const float* tm = tile_max + ((int64_t)c * n_q_heads + hq) * n_tiles;
  const float* tsum = tile_sum + ((int64_t)c * n_q_heads + hq) * n_tiles;
  float m = -__builtin_inff();
  for (int64_t t = lane; t < lim; t += 64) m = fmaxf(m, tm[t]);
  m = group_max<64>(m);
  float z = 0.f;
  for (int64_t t = lane; t < lim; t += 64) z += tsum[t] * expf(tm[t] - m);
  z = group_sum<64>(z);
  if (lane == 0) {
    head_stats[((int64_t)c * n_q_heads + hq) * 2] = m;
    head_stats[((int64_t)c * n_q_heads + hq) * 2 + 1] = z;
  }
}

__global__ __launch_bounds__(256) void h2o_accumulate_kernel(
    float* __restrict__ scores, const float* __restrict__ head_stats, int n_q_heads,
    const int64_t* __restrict__ row_base, const int32_t* __restrict__ fill, int64_t score_stride,
    float decay, float now, int write_probs, float* __restrict__ row_acc, float* __restrict__ row_ts,
    float* __restrict__ importance_out) {
  const int c = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n >= fill[c]) return;
  float imp = 0.f;
  for (int hq = 0; hq < n_q_heads; ++hq) {
    const int64_t si = ((int64_t)c * n_q_heads + hq) * score_stride + n;
    const float m = head_stats[((int64_t)c * n_q_heads + hq) * 2];
    const float z = head_stats[((int64_t)c * n_q_heads + hq) * 2 + 1];
    const float p = expf(scores[si] - m) / z;
    if (write_probs) scores[si] = p;
    imp = imp + p;
  }
  const int64_t row = row_base[c] + n;
  if (row_acc) {
    float acc = row_acc[row];
    if (decay != 1.0f) acc = acc * decay;
    row_acc[row] = acc + imp;
  }
  if (row_ts) row_ts[row] = now;
  if (importance_out) importance_out[(int64_t)c * score_stride + n] = imp;
}

template <int SCHEME, int OUT_DT>
static void launch_gather(unsigned blocks, hipStream_t st, const void* codes, const void* scale,
                          const void* zero, int D, int group, const int64_t* rows, int64_t row0,
                          int64_t n, void* out) {
  hipLaunchKernelGGL((gather_dequant_kernel<SCHEME, OUT_DT>), dim3(blocks), dim3(256), 0, st, codes,
                     scale, zero, D, group, rows, row0, n, out);
}

template <int SCHEME, int REP>
static void launch_scores_q(dim3 grid, hipStream_t st, int q_dtype, const ScoreArgs& a) {
  if (q_dtype == PIKV_BF16)
    hipLaunchKernelGGL((scores_kernel<SCHEME, REP, PIKV_BF16>), grid, dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((scores_kernel<SCHEME, REP, PIKV_F32>), grid, dim3(256), 0, st, a);
}

template <int SCHEME>
static int launch_scores(int rep, dim3 grid, hipStream_t st, int q_dtype, const ScoreArgs& a) {
  switch (rep) {
    case 1: launch_scores_q<SCHEME, 1>(grid, st, q_dtype, a); break;
    case 2: launch_scores_q<SCHEME, 2>(grid, st, q_dtype, a); break;
    case 4: launch_scores_q<SCHEME, 4>(grid, st, q_dtype, a); break;
    case 8: launch_scores_q<SCHEME, 8>(grid, st, q_dtype, a); break;
    default: return PIKV_ERR_UNSUPPORTED;
  }
  return PIKV_OK;
}

}  // namespace pikv

using namespace pikv;

extern "C" int pikv_gather_dequant(const void* codes, const void* scale, const void* zero, int D,
                                   int group, int scheme, const int64_t* rows, int64_t row0,
                                   int64_t n, void* out, int out_dtype, void* stream) {
  if (!codes || !scale || !out) return PIKV_ERR_NULL;
  if (scheme < 0 || scheme > 3) return PIKV_ERR_UNSUPPORTED;
  if (out_dtype != PIKV_F32 && out_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  const bool eight = (scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM);
  const bool asym = (scheme == PIKV_Q_I8_ASYM || scheme == PIKV_Q_I4_ASYM);
  const int epl = eight ? 16 : 32;
  if (asym && !zero) return PIKV_ERR_NULL;
  if (D <= 0 || group <= 0 || D % group != 0 || D % epl != 0 || n < 0 || row0 < 0) return PIKV_ERR_SHAPE;
  if (group % epl != 0) return PIKV_ERR_UNSUPPORTED;
  if (n == 0) return PIKV_OK;
  const int64_t lanes = n * (D / epl);
  const int64_t blocks = (lanes + 255) / 256;
  if (blocks > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const unsigned nb = (unsigned)blocks;
#define PIKV_GATHER_CASE(S)                                                                      \
  case S:                                                                                        \
    if (out_dtype == PIKV_F32)                                                                   \
      launch_gather<S, PIKV_F32>(nb, st, codes, scale, zero, D, group, rows, row0, n, out);     \
    else                                                                                         \
      launch_gather<S, PIKV_BF16>(nb, st, codes, scale, zero, D, group, rows, row0, n, out);    \
    break;
  switch (scheme) {
    PIKV_GATHER_CASE(PIKV_Q_I8_SYM)
    PIKV_GATHER_CASE(PIKV_Q_I8_ASYM)
    PIKV_GATHER_CASE(PIKV_Q_I4_ASYM)
    PIKV_GATHER_CASE(PIKV_Q_I4_SYM)
  }
#undef PIKV_GATHER_CASE
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

extern "C" int pikv_gather_dequant_scores(const void* k_codes, const void* k_scale,
                                          const void* k_zero, int scheme, int group, int n_kv_heads,
                                          int n_q_heads, int head_dim, const void* q, int q_dtype,
                                          float scale_qk, const int64_t* cache_row_base,
                                          const int32_t* cache_fill, int n_caches, int64_t max_len,
                                          int64_t score_stride, float* scores, float* tile_max,
                                          float* tile_sum, void* stream) {
  if (!k_codes || !k_scale || !q || !cache_row_base || !cache_fill || !scores || !tile_max || !tile_sum)
    return PIKV_ERR_NULL;
  if (scheme < 0 || scheme > 3) return PIKV_ERR_UNSUPPORTED;
  if (q_dtype != PIKV_F32 && q_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  const bool eight = (scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM);
  const bool asym = (scheme == PIKV_Q_I8_ASYM || scheme == PIKV_Q_I4_ASYM);
  const int epl = eight ? 16 : 32;
  if (asym && !k_zero) return PIKV_ERR_NULL;
  if (n_kv_heads < 1 || n_q_heads < 1 || head_dim < 1 || n_caches < 1 || n_caches > 65535 ||
      max_len < 0 || score_stride < max_len || group < 1)
    return PIKV_ERR_SHAPE;
  if (n_q_heads % n_kv_heads != 0) return PIKV_ERR_SHAPE;
  const int D = n_kv_heads * head_dim;
  if (D % group != 0) return PIKV_ERR_SHAPE;
  if (!is_pow2(head_dim) || head_dim < epl || group % epl != 0) return PIKV_ERR_UNSUPPORTED;
  const int lanes_per_row = D / epl;
  if (lanes_per_row > 256 || 256 % lanes_per_row != 0) return PIKV_ERR_UNSUPPORTED;
  if (kTile % (256 / lanes_per_row) != 0) return PIKV_ERR_UNSUPPORTED;
  if (n_q_heads > kMaxQHeads) return PIKV_ERR_UNSUPPORTED;
  if (max_len == 0) return PIKV_OK;
  const int64_t n_tiles = (max_len + kTile - 1) / kTile;
  if (n_tiles > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  ScoreArgs a{k_codes, k_scale, k_zero, q, cache_row_base, cache_fill, scores, tile_max, tile_sum,
              score_stride, n_tiles, scale_qk, group, n_kv_heads, n_q_heads, head_dim};
  const dim3 grid((unsigned)n_tiles, (unsigned)n_caches);
  hipStream_t st = (hipStream_t)stream;
  const int rep = n_q_heads / n_kv_heads;
  int rc = PIKV_ERR_UNSUPPORTED;
  switch (scheme) {
    case PIKV_Q_I8_SYM: rc = launch_scores<PIKV_Q_I8_SYM>(rep, grid, st, q_dtype, a); break;
    case PIKV_Q_I8_ASYM: rc = launch_scores<PIKV_Q_I8_ASYM>(rep, grid, st, q_dtype, a); break;
    case PIKV_Q_I4_ASYM: rc = launch_scores<PIKV_Q_I4_ASYM>(rep, grid, st, q_dtype, a); break;
    case PIKV_Q_I4_SYM: rc = launch_scores<PIKV_Q_I4_SYM>(rep, grid, st, q_dtype, a); break;
  }
  if (rc != PIKV_OK) return rc;
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

extern "C" int pikv_h2o_accumulate(float* scores, const float* tile_max, const float* tile_sum,
                                   int n_q_heads, const int64_t* cache_row_base,
                                   const int32_t* cache_fill, int n_caches, int64_t max_len,
                                   int64_t score_stride, float decay, float now, int write_probs,
                                   float* row_acc, float* row_ts, float* importance_out,
                                   float* head_stats, void* stream) {
  if (!scores || !tile_max || !tile_sum || !cache_row_base || !cache_fill || !head_stats)
    return PIKV_ERR_NULL;
  if (n_q_heads < 1 || n_q_heads > 65535 || n_caches < 1 || n_caches > 65535 || max_len < 0 ||
      score_stride < max_len)
    return PIKV_ERR_SHAPE;
  if (max_len == 0) return PIKV_OK;
  const int64_t n_tiles = (max_len + kTile - 1) / kTile;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(head_stats_kernel, dim3((unsigned)n_q_heads, (unsigned)n_caches), dim3(64), 0,
                     st, tile_max, tile_sum, cache_fill, n_q_heads, n_tiles, head_stats);
  const int64_t nb = (max_len + 255) / 256;
  if (nb > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  hipLaunchKernelGGL(h2o_accumulate_kernel, dim3((unsigned)nb, (unsigned)n_caches), dim3(256), 0, st,
                     scores, head_stats, n_q_heads, cache_row_base, cache_fill, score_stride, decay,
                     now, write_probs, row_acc, row_ts, importance_out);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
