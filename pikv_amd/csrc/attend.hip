// Attention output over the compressed V cache:
//   out[c, h, :] = sum_n p[c, h, n] * dequant(V[c, n, h / rep, :]),   n < fill[c]
// with p either given (scores already normalised) or formed on the fly from raw
// scores and the per-head softmax statistics (max, sum).
//
// Every block covers a run of cached tokens of one cache and writes a partial
// result; a second small kernel adds the partials in a fixed order, so the sum does
// not depend on scheduling.
//
// Two forms:
//  * attend_valu_kernel - any scheme / group / head size: one lane owns 16 code
//    bytes of a token (as in the score kernel), w = p * scale multiplies the codes
//    into float accumulators, the zero-point term is carried as one extra sum.
//  * attend_mfma_i4_kernel - 4-bit codes, groups of 32, head_dim 128 (64 and 32 as slabs of two / four heads), bf16-exact:
//    the contraction runs over TOKENS, so the matrix-core B operand needs, per lane,
//    the codes of 8 tokens for ONE dimension - the transpose of how rows are stored.
//    The codes of a 64-token tile are staged in LDS as they are and read back with
//    ds_read_b64_tr_b4, which hands lane i the i-th nibble of 16 lanes' words, i.e.
//    16 tokens of one dimension.  Nibbles become bf16 128+u exactly (0x4300 | u);
//    the A operand rows are the weights p*scale of up to 8 query heads, split into a
//    bf16 high part and a bf16 remainder (two rows per head) so that no precision is
//    lost against float32; the zero-point term is summed on the vector unit.
#include "common.hpp"

namespace pikv {

typedef __bf16 pikv_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pikv_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kAttTile = 64;          // cached tokens per step of the matrix-core form
constexpr int kAttMaxTokensPerBlock = 4096;  // cached tokens one block walks: chosen per call, see attend_tokens_per_block

struct AttendArgs {
  const float* scores;      // [n_caches, n_q_heads, score_stride]
  const float* head_stats;  // [n_caches, n_q_heads, 2] (max, sum) or nullptr: scores are probabilities
  const void* codes;
  const void* scale;
  const void* zero;
  const int64_t* row_base;
  const int32_t* fill;
  float* partial;           // [n_splits, n_caches, n_q_heads, head_dim]
  int64_t score_stride;
  int group;
  int n_kv_heads;
  int n_q_heads;
  int head_dim;
  int n_caches;
  // optional H2O bookkeeping of the same probabilities: acc = acc*decay + sum over heads, ts = now
  float* row_acc;
  float* row_ts;
  float decay;
  float now;
  int64_t max_len;  // rows of a cache beyond max_len are not read
  // exchange format of pikv_decode_attend (attend_mfma_i4_kernel only): when escores is set, `scores` is
  // not read; escores [cache][tile][q head][64] floats hold exp(score - tile max), tile_max [cache][tile][q head]
  const float* escores;
  const float* tile_max;
  int64_t n_tiles;
  int head_off;  // attend_mfma_i4_kernel: first query head of every kv group handled by this launch
  int tokens_per_block;  // cached tokens per block (a multiple of 64): block x covers tokens [x * tokens_per_block, ...)
  int kv_window;         // attend_valu_kernel: kv heads per block when a whole row has more than 256 lanes (0: all)
  int row_slabs;         // attend_mfma_i4_kernel<SPLIT>: 128-dimension slabs of a whole cached row (the block takes 8 of them)
};

__device__ __forceinline__ float prob_of(float s, float mx, float rz, bool normalise) {
  return normalise ? __builtin_amdgcn_exp2f((s - mx) * 1.4426950408889634f) * rz : s;
}

// ---- vector-unit form --------------------------------------------------------------
// RP query heads of every kv head per pass (blockIdx.z selects the pass).
// Rows of more than 256 lanes (e.g. 40 kv heads of 128, 8-bit): a block takes a window of a.kv_window kv heads -
// kv heads are independent here - and blockIdx.z = pass * windows + window.
template <int SCHEME, int RP>
__global__ __launch_bounds__(256) void attend_valu_kernel(AttendArgs a) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  __shared__ float red[256 * EPL];
  const int c = blockIdx.y;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  const int64_t t0 = (int64_t)blockIdx.x * a.tokens_per_block;
  const int64_t t1 = (t0 + a.tokens_per_block < len) ? t0 + a.tokens_per_block : len;
  const int rep = a.n_q_heads / a.n_kv_heads;
  const int wk = a.kv_window ? a.kv_window : a.n_kv_heads;   // kv heads of this block
  const int n_win = a.n_kv_heads / wk;
  const int r0 = (blockIdx.z / n_win) * RP;
  const int D = a.n_kv_heads * a.head_dim;
  const int lanes_full = D / EPL;                 // 16-byte pieces of a whole cached row
  const int lanes_per_head = a.head_dim / EPL;
  const int lanes_per_row = wk * lanes_per_head;  // ... of the block's window
  const int groups_per_row = D / a.group;
  const int tok_per_step = 256 / lanes_per_row;
  const int part = threadIdx.x % lanes_per_row;
  const int gpart = (blockIdx.z % n_win) * lanes_per_row + part;   // piece of the whole row
  const int tok_in_step = threadIdx.x / lanes_per_row;
  const int kvh = gpart / lanes_per_head;
  const int d0 = (part % lanes_per_head) * EPL;
  const bool normalise = a.head_stats != nullptr;

  float acc[RP][EPL];
  float zacc[RP], mx[RP], rz[RP];
  const float* srow[RP];
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    const int hq = kvh * rep + ((r0 + r < rep) ? r0 + r : 0);
    srow[r] = a.scores + ((int64_t)c * a.n_q_heads + hq) * a.score_stride;
    mx[r] = 0.f;
    rz[r] = 1.f;
    if (normalise) {
      mx[r] = a.head_stats[((int64_t)c * a.n_q_heads + hq) * 2];
      rz[r] = 1.0f / a.head_stats[((int64_t)c * a.n_q_heads + hq) * 2 + 1];
    }
    zacc[r] = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) acc[r][j] = 0.f;
  }
  const int64_t base_row = a.row_base[c];
  // (a row's lanes need not divide the block: the threads beyond the last whole row stay idle)
  // UN tokens per thread and trip: their codes, metadata and scores are asked for together, one
  // memory round trip instead of UN (a step past the end re-reads the trip's first token, weight 0)
  constexpr int UN = RP >= 8 ? 2 : 4;
  for (int64_t n = tok_in_step < tok_per_step ? t0 + tok_in_step : t1; n < t1; n += (int64_t)tok_per_step * UN) {
    uint4 v[UN];
    float sc[UN], zu[UN], sv[UN][RP];
    bool ok[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int64_t nn = n + (int64_t)u * tok_per_step;
      ok[u] = nn < t1;
      const int64_t nc = ok[u] ? nn : n;
      const int64_t row = base_row + nc;
      v[u] = ld16(reinterpret_cast<const char*>(a.codes) + (row * lanes_full + gpart) * 16);
      const int64_t mi = row * groups_per_row + (gpart * EPL) / a.group;
      sc[u] = load_meta<SCHEME>(a.scale, mi);
      zu[u] = (Q::sym ? 0.f : load_meta<SCHEME>(a.zero, mi)) - (float)Q::qmin;
#pragma unroll
      for (int r = 0; r < RP; ++r) sv[u][r] = srow[r][nc];
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      float cf[EPL];
      unpack_codes_unsigned<SCHEME>(v[u], cf);
#pragma unroll
      for (int r = 0; r < RP; ++r) {
        const float w = ok[u] ? prob_of(sv[u][r], mx[r], rz[r], normalise) * sc[u] : 0.f;
        zacc[r] = fmaf(w, zu[u], zacc[r]);
#pragma unroll
        for (int j = 0; j < EPL; ++j) acc[r][j] = fmaf(w, cf[j], acc[r][j]);
      }
    }
  }
  // add the token slots of the block (threads that share `part`), one head at a time
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < EPL; ++j) red[threadIdx.x * EPL + j] = acc[r][j] - zacc[r];
    __syncthreads();
    if (tok_in_step == 0 && r0 + r < rep) {
      float sum[EPL];
#pragma unroll
      for (int j = 0; j < EPL; ++j) sum[j] = 0.f;
      for (int s = 0; s < tok_per_step; ++s)
#pragma unroll
        for (int j = 0; j < EPL; ++j) sum[j] += red[(s * lanes_per_row + part) * EPL + j];
      const int hq = kvh * rep + r0 + r;
      float* o = a.partial + (((int64_t)blockIdx.x * a.n_caches + c) * a.n_q_heads + hq) * a.head_dim + d0;
#pragma unroll
      for (int j = 0; j < EPL; ++j) o[j] = sum[j];
    }
  }
}

// Importance of every cached token (sum of its probabilities over the query heads, in
// head order) for callers of the vector-unit form.
__global__ __launch_bounds__(256) void attend_importance_kernel(AttendArgs a) {
  const int c = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n >= a.fill[c] || n >= a.max_len) return;
  const bool normalise = a.head_stats != nullptr;
  float imp = 0.f;
  for (int h0 = 0; h0 < a.n_q_heads; h0 += 8) {   // eight heads in flight per thread
    float sv[8], mx[8], hz[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t hi = (int64_t)c * a.n_q_heads + (h0 + u < a.n_q_heads ? h0 + u : 0);
      sv[u] = a.scores[hi * a.score_stride + n];
      mx[u] = normalise ? a.head_stats[hi * 2] : 0.f;
      hz[u] = normalise ? a.head_stats[hi * 2 + 1] : 1.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (h0 + u < a.n_q_heads) imp = imp + prob_of(sv[u], mx[u], 1.0f / hz[u], normalise);
  }
  const int64_t row = a.row_base[c] + n;
  if (a.row_acc) {
    float acc = a.row_acc[row];
    if (a.decay != 1.0f) acc = acc * a.decay;
    a.row_acc[row] = acc + imp;
  }
  if (a.row_ts) a.row_ts[row] = a.now;
}

// H2O bookkeeping from the exchange format of pikv_decode_attend, for the attention kernels that
// cannot do it themselves (split rows: a block sees only some heads of a token):
//   p[h][n] = e[c][tile][h][n % 64] * exp(tile max[h] - head max[h]) / head sum[h],  imp[n] = sum_h p[h][n]
// One block per 64-token tile; four lanes per token add every fourth head, then the four partial sums.
__global__ __launch_bounds__(256) void exch_importance_kernel(AttendArgs a) {
  __shared__ float part[4][kAttTile];
  const int c = blockIdx.y;
  const int64_t tile = blockIdx.x;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  const int64_t n0 = tile * kAttTile;
  if (n0 >= len) return;  // uniform
  const int t = threadIdx.x & 63, hl = threadIdx.x >> 6;
  const int64_t trow = ((int64_t)c * a.n_tiles + tile) * a.n_q_heads;
  float imp = 0.f;
  for (int h0 = hl; h0 < a.n_q_heads; h0 += 4 * 8) {   // eight heads in flight per thread
    float e[8], tm[8], hm[8], hz[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int h = h0 + 4 * u < a.n_q_heads ? h0 + 4 * u : hl;
      const int64_t hi = (int64_t)c * a.n_q_heads + h;
      e[u] = a.escores[(trow + h) * kAttTile + t];
      tm[u] = a.tile_max[trow + h];
      hm[u] = a.head_stats[hi * 2];
      hz[u] = a.head_stats[hi * 2 + 1];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (h0 + 4 * u < a.n_q_heads)
        imp = imp + e[u] * (__builtin_amdgcn_exp2f((tm[u] - hm[u]) * 1.4426950408889634f) * (1.0f / hz[u]));
  }
  part[hl][t] = imp;
  __syncthreads();
  if (hl == 0 && n0 + t < len) {
    imp = (part[0][t] + part[1][t]) + (part[2][t] + part[3][t]);
    const int64_t row = a.row_base[c] + n0 + t;
    if (a.row_acc) {
      float acc = a.row_acc[row];
      if (a.decay != 1.0f) acc = acc * a.decay;
      a.row_acc[row] = acc + imp;
    }
    if (a.row_ts) a.row_ts[row] = a.now;
  }
}

// ---- matrix-core form -----------------------------------------------------------------
typedef int pikv_i32x2 __attribute__((ext_vector_type(2)));

constexpr int kAttARow = 144;  // bytes per staged A-operand row: 64 tokens x bf16 + 16 (bank spread)

// Metadata of token t, kv head g (one float4 = the 4 groups of the head) sits at byte
// t*(HK*16+16) + (t/16)*64 + g*16: the 16 tokens {k + 16w} that one pass of 16 lanes reads
// fall into 16 different banks quads, and consecutive (token, head) writers stay contiguous.
__host__ __device__ constexpr size_t att_meta_bytes(int hk) { return (size_t)kAttTile * (hk * 16 + 16) + 4 * 64; }
__device__ __forceinline__ int att_meta_off(int tok, int g, int hk) {
  return tok * (hk * 16 + 16) + (tok >> 4) * 64 + g * 16;
}

constexpr int kAttPRow = 68;  // floats per query head of staged probabilities: 64 tokens + 4 (bank spread)

static size_t attend_mfma_lds_bytes(int n_kv_heads, int n_q_heads, int nsets = 1) {
  // codes [64 tokens][n_kv_heads*64 + 8 bytes]; scale and zero + bias as float4 (4 groups)
  // [64 tokens][kv head] in padded token rows; A operands per wavefront [4 groups][8 rows][kAttARow];
  // probabilities [query head][kAttPRow]
  // + one all-zero piece of an A row (32 bytes) for the lanes whose row holds no head
  return (size_t)kAttTile * (n_kv_heads * 64 + 8) + 2 * att_meta_bytes(n_kv_heads) + 4 * (size_t)nsets * 4 * 8 * kAttARow +
         (size_t)4 * n_kv_heads * nsets * kAttPRow * 4 + 32;
}

// HK = n_kv_heads (1..8); at most 4 query heads per kv head.  EXCH: the scores come in the exchange
// format of pikv_decode_attend (a.escores, a.tile_max) instead of a.scores.
// Heads narrower than 128 (a.head_dim 64 or 32): the kernel's kv heads are 128-dimension slabs of
// the cached row, each the stored bytes of hps = 128 / head_dim neighbouring kv heads, and the query
// heads of a slab are the heads of those kv heads in order.  A query head is multiplied with the
// whole slab and only the dimensions of its own kv head are written out.
// NARROW selects that form at compile time: the kernel for heads of 128 carries none of it.
// NSETS = 2 (up to 4 kv heads): a launch covers up to 8 query heads of every kv head as two sets of
// four that are multiplied with the same staged tile and the same expanded codes - the V codes of a
// cache with 5 to 8 query heads per kv head are read from memory once instead of once per launch.
// SPLIT (rows of a.row_slabs = groups x HK slabs): neighbouring blocks take the groups of HK slabs of
// one token range, block index = range * groups + group; a group is a piece of HK x 64 bytes of every
// cached row.  Rows of more than 8 slabs (e.g. 32 kv heads of 128) go as groups of 8; rows of 6, 8 or
// more slabs with 5 to 8 query heads per kv head go as groups of 3 or 4 with two sets each, so that
// also their V codes are read once.  The H2O bookkeeping needs all heads of a token and is left to a
// kernel of its own (row_acc and row_ts are not touched here).
// TI > 1 (rows of few slabs: 1 to 4 kv heads of 128): TI neighbouring cached rows - they lie side by side in
// memory - are taken as ONE row of HK = TI x (real slabs) slabs, slab g' = (row parity) * slabs + g.  A tile
// is then 64 x TI tokens: TI times fewer trips of the tile loop (each pays a memory round trip and two block
// barriers, which is what bounds small rows) and every wavefront has a slab to multiply.  Slab g' sees the
// probabilities of its own tokens only; the TI partial outputs of a head are added at the end, in order.
template <int SCHEME, int HK, bool EXCH = false, bool NARROW = false, int NSETS = 1, bool SPLIT = false, int TI = 1>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void attend_mfma_i4_kernel(AttendArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 4, "4-bit schemes only");
  static_assert(HK >= 1 && HK <= 8, "1 to 8 kv heads");
  constexpr int NH = (HK + 3) / 4;        // kv heads per wavefront
  constexpr int NI = NH * NSETS;          // (kv head, set of four query heads) pairs per wavefront
  static_assert(NSETS == 1 || (NSETS == 2 && HK <= 4), "two sets: the staged rows of 8 x 4 heads, accumulators of one kv head");
  static_assert(TI == 1 || (!SPLIT && HK % TI == 0), "interleaved rows: whole rows");
  constexpr int HR = HK / TI;             // slabs of a cached row
  constexpr int TT = kAttTile * TI;       // cached tokens per tile
  constexpr int RS = HK * 64 + 8;         // bytes per token row of staged codes
  constexpr int LPR = HK * 4;             // 16-byte chunks per cached row
  constexpr int NCH = kAttTile * LPR / 256 > 0 ? kAttTile * LPR / 256 : 1;  // code chunks per thread
  constexpr int NMC = (kAttTile * HK + 255) / 256;                          // metadata chunks per thread
  extern __shared__ __align__(16) unsigned char att_lds[];
  unsigned char* lcodes = att_lds;
  unsigned char* lscale = att_lds + kAttTile * RS;
  unsigned char* lzterm = lscale + att_meta_bytes(HK);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  unsigned char* abuf = lzterm + att_meta_bytes(HK) + wave * (NSETS * 4 * 8 * kAttARow);   // [set][4 groups][8 rows]
  float* lprob = reinterpret_cast<float*>(lzterm + att_meta_bytes(HK) + 4 * (NSETS * 4 * 8 * kAttARow));
  unsigned char* azero = reinterpret_cast<unsigned char*>(lprob + 4 * HK * NSETS * kAttPRow);
  if (threadIdx.x < 8) reinterpret_cast<uint32_t*>(azero)[threadIdx.x] = 0u;  // visible after the loop's first barrier

  const int c = blockIdx.y;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  static_assert(!SPLIT || !NARROW, "split rows: groups of HK slabs, heads of 128 dimensions");
  const int n_groups = SPLIT ? a.row_slabs / HK : 1;
  const int xb = SPLIT ? blockIdx.x / n_groups : blockIdx.x;            // token range of this block
  const int kv_off = SPLIT ? (blockIdx.x % n_groups) * HK : 0;          // its first slab
  const int row_slabs = SPLIT ? a.row_slabs : HR;
  const int64_t t0 = (int64_t)xb * a.tokens_per_block;
  const int64_t t1 = (t0 + a.tokens_per_block < len) ? t0 + a.tokens_per_block : len;
  if (t0 >= t1) {  // nothing cached in this range: the partial (of this block's heads) is zero
    const int hd = NARROW ? a.head_dim : 128;
    const int nh = a.n_q_heads / n_groups;   // query heads of the block's slabs, a contiguous run
    for (int idx = threadIdx.x; idx < nh * hd; idx += 256)
      a.partial[(((int64_t)xb * a.n_caches + c) * a.n_q_heads + (SPLIT ? (blockIdx.x % n_groups) * nh : 0)) * hd + idx] = 0.f;
    return;
  }
  // A launch covers up to 4 query heads of every kv group: heads head_off .. head_off+nr-1.
  // More than 4 heads per kv head are served by a second launch over the same codes.
  const int rep_all = a.n_q_heads / row_slabs;   // query heads per slab
  const int rep = rep_all - a.head_off < 4 ? rep_all - a.head_off : 4;  // heads of a group in this launch (first set)
  const int rep_b = NSETS == 1 ? 0 : rep_all - a.head_off - 4 < 0 ? 0 : rep_all - a.head_off - 4 < 4 ? rep_all - a.head_off - 4 : 4;  // second set
  // matrix-core roles: A row / B,C column i, token group kg
  const int i = lane & 15;
  const int kg = lane >> 4;
  // weight-preparation roles: head r of the kv group, tokens {tk, tk+4, tk+8, tk+12} of group wkg
  const int r = lane >> 4;
  const int wkg = (lane >> 2) & 3;
  const int tk = wkg * 16 + (lane & 3);
  const bool normalise = a.head_stats != nullptr;
  const float zbias = 128.0f - (float)Q::qmin;
  const int64_t base_row = a.row_base[c];

  pikv_f32x4 C[NI][8];
  float zacc[NI][4];
#pragma unroll
  for (int hs = 0; hs < NI; ++hs) {
#pragma unroll
    for (int d = 0; d < 8; ++d) C[hs][d] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) zacc[hs][sg] = 0.f;
  }
  // score-staging role: staged row sh = 4 * (set * HK + kv head) + head of the set, tokens
  // st8..st8+7 of the tile (32 rows x 8 runs); rows without a head stage zeros.
  // Interleaved rows: sh = 4 * (set * HR + kv head) + head counts the heads of the REAL rows (32 / TI of
  // them, 8 TI runs each); a thread reads eight consecutive tokens of its head and deals them to the
  // staged rows of the TI slabs of that kv head.
  const int sh = TI == 1 ? threadIdx.x >> 3 : threadIdx.x / (8 * TI);
  const int st8 = TI == 1 ? (threadIdx.x & 7) * 8 : (threadIdx.x % (8 * TI)) * 8;
  const int s_set = NSETS == 1 && TI == 1 ? 0 : sh / (4 * HR);
  const int s_g = NSETS == 1 && TI == 1 ? sh >> 2 : (sh >> 2) % HR;
  const bool s_on = s_set < NSETS && s_g < HR && (sh & 3) < (s_set ? rep_b : rep);
  const int s_hq = s_on ? (kv_off + s_g) * rep_all + a.head_off + 4 * s_set + (sh & 3) : 0;
  const float* srow = a.scores + ((int64_t)c * a.n_q_heads + s_hq) * a.score_stride;
  float smx = 0.f, srz = 1.f;
  if (normalise) {
    smx = a.head_stats[((int64_t)c * a.n_q_heads + s_hq) * 2];
    srz = 1.0f / a.head_stats[((int64_t)c * a.n_q_heads + s_hq) * 2 + 1];
  }
  const bool s_vec = (a.score_stride & 3) == 0 && (reinterpret_cast<uintptr_t>(a.scores) & 15) == 0;
  const float s_off = normalise ? -INFINITY : 0.f;  // what a token past the end contributes: p = 0
  // exchange format: eight values exp(score - tile max) per thread and tile, and the tile's max of the head;
  // the rows of a tile lie side by side, [tile][q head][64], so a block reads one contiguous run
  constexpr bool exch = EXCH;
  const float* const ep = exch ? a.escores + ((int64_t)c * a.n_tiles * a.n_q_heads + s_hq) * kAttTile + st8 % kAttTile : nullptr;
  const float* const tmp = exch ? a.tile_max + (int64_t)c * a.n_tiles * a.n_q_heads + s_hq : nullptr;
  float ptm = 0.f;

  // registers that carry the next tile from HBM to LDS
  uint4 pc[NCH];
  uint2 ps[NMC], pz[NMC];
  float psc[8];
  // importance role: wavefront w owns tokens 16w..16w+15 of a tile, lanes 0..15 hold their accumulators
  const int it = wave * 16 + (lane & 15);
  const int igrp = lane >> 4;
  float pacc[TI];
#pragma unroll
  for (int k = 0; k < TI; ++k) pacc[k] = 0.f;
  // Every address below is a wave-uniform base plus a multiple of the thread index: chunk
  // ch = k * 256 + thread of the tile's code rows IS the (token, 16-byte piece) pair
  // (tok * LPR + off), and 4 * ch halves the (token, kv head) pair of the metadata rows; the
  // bounds are uniform thresholds on the thread index.  (Per-chunk 64-bit lane addresses and
  // token indices had cost the registers whose spill reloads waited, inside the loop, for
  // the whole prefetch.)
  const float* const sp = srow + st8;
  auto fetch = [&](int64_t n0) {
    const int64_t left = t1 - n0;
    const int rem = left < TT ? (int)left : TT;  // tokens of this tile
    const int64_t urow = base_row + n0;
#pragma unroll
    for (int k = 0; k < TI; ++k)
      if (a.row_acc && igrp == 0 && k * kAttTile + it < rem) pacc[k] = (a.row_acc + urow)[k * kAttTile + it];
    if (exch) {
      // staged rows without a head read head 0 (and are multiplied by zero): no branch around the loads
      // the 64-token tile of the exchange rows that holds this thread's tokens; with interleaved rows the
      // last tile of the loop may reach past the range, into exchange rows that were never written
      const int64_t tile = n0 / kAttTile + (TI == 1 ? 0 : st8 / kAttTile);
      const bool live = TI == 1 || tile * kAttTile < t1;
      float4 lo4 = make_float4(0.f, 0.f, 0.f, 0.f), hi4 = lo4;
      ptm = smx;
      if (live) {
        lo4 = *reinterpret_cast<const float4*>(ep + tile * a.n_q_heads * kAttTile);
        hi4 = *reinterpret_cast<const float4*>(ep + tile * a.n_q_heads * kAttTile + 4);
        ptm = tmp[tile * a.n_q_heads];
      }
      psc[0] = lo4.x, psc[1] = lo4.y, psc[2] = lo4.z, psc[3] = lo4.w;
      psc[4] = hi4.x, psc[5] = hi4.y, psc[6] = hi4.z, psc[7] = hi4.w;
    } else if (s_on) {
      const float* spn = sp + n0;
      if (s_vec && st8 + 8 <= rem) {
        const float4 lo4 = *reinterpret_cast<const float4*>(spn);
        const float4 hi4 = *reinterpret_cast<const float4*>(spn + 4);
        psc[0] = lo4.x, psc[1] = lo4.y, psc[2] = lo4.z, psc[3] = lo4.w;
        psc[4] = hi4.x, psc[5] = hi4.y, psc[6] = hi4.z, psc[7] = hi4.w;
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) psc[k] = st8 + k < rem ? spn[k] : s_off;
      }
    }
    // Every load is issued, from an offset clamped to the tile's last cached row: tokens past the
    // end of a short tile see a copy of that row, and their weight is zero (p = 0, finite scale).
    if constexpr (SPLIT) {
      // the block's slabs are a piece of every row: (token, piece) from the chunk index, the token clamped
      const char* cb = reinterpret_cast<const char*>(a.codes) + (urow * row_slabs + kv_off) * 64;
#pragma unroll
      for (int k = 0; k < NCH; ++k) {
        const int ch = k * 256 + threadIdx.x;
        const int tok = ch / LPR < rem ? ch / LPR : rem - 1;
        pc[k] = ld16(cb + (int64_t)tok * row_slabs * 64 + (ch % LPR) * 16);
      }
      const char* sb = reinterpret_cast<const char*>(a.scale) + (urow * row_slabs + kv_off) * 8;
      const char* zb = reinterpret_cast<const char*>(a.zero) + (urow * row_slabs + kv_off) * 8;
#pragma unroll
      for (int k = 0; k < NMC; ++k) {
        const int ch = k * 256 + threadIdx.x;
        const int tok = ch / HK < rem ? ch / HK : rem - 1;
        const int64_t mo = (int64_t)tok * row_slabs * 8 + (ch % HK) * 8;
        ps[k] = *reinterpret_cast<const uint2*>(sb + mo);
        pz[k] = make_uint2(0, 0);
        if constexpr (!Q::sym) pz[k] = *reinterpret_cast<const uint2*>(zb + mo);
      }
    } else {
    const char* cb = reinterpret_cast<const char*>(a.codes) + urow * (HR * 64);
    const unsigned c_last = (unsigned)(rem * (HR * 4) - 1) * 16u;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const unsigned off = k * 4096u + threadIdx.x * 16u;
      pc[k] = ld16(cb + (off < c_last ? off : c_last));
    }
    const char* sb = reinterpret_cast<const char*>(a.scale) + urow * (HR * 8);
    const char* zb = reinterpret_cast<const char*>(a.zero) + urow * (HR * 8);
    const unsigned m_last = (unsigned)(rem * HR - 1) * 8u;
#pragma unroll
    for (int k = 0; k < NMC; ++k) {
      const unsigned off = k * 2048u + threadIdx.x * 8u;
      const unsigned mo = off < m_last ? off : m_last;
      ps[k] = *reinterpret_cast<const uint2*>(sb + mo);
      pz[k] = make_uint2(0, 0);
      if constexpr (!Q::sym) pz[k] = *reinterpret_cast<const uint2*>(zb + mo);
    }
    }
  };
  auto h2f = [](uint32_t w, int hi) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> (16 * hi))); };
  auto stage = [&]() {
    {
      // tokens {l, l+4, l+8, l+12} of a 16-token group go side by side: one float4 per reader
      if (exch) {
        // p = exp(s - tile max) * exp(tile max - head max) / head sum: one exponential per thread and tile
        const float coef = s_on ? __builtin_amdgcn_exp2f((ptm - smx) * 1.4426950408889634f) * srz : 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) psc[k] = s_on ? psc[k] * coef : 0.f;
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        // token j of the tile is row j % TI of tile row t = j / TI: it belongs to slab (j % TI) * HR + kv head
        const int t = (st8 + k) / TI;
        const int row = TI == 1 ? sh : ((s_set * HK + ((st8 + k) % TI) * HR + s_g) * 4 + (sh & 3));
        if (TI == 1 || s_set < NSETS)
          lprob[row * kAttPRow + (t & ~15) + (t & 3) * 4 + ((t >> 2) & 3)] =
              exch ? psc[k] : (s_on ? prob_of(psc[k], smx, srz, normalise) : 0.f);
      }
    }
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int ch = k * 256 + threadIdx.x;
      const int tok = ch / LPR, off = ch % LPR;
      if (tok < kAttTile) {
        uint2* dst = reinterpret_cast<uint2*>(lcodes + tok * RS + off * 16);  // rows are 8-byte aligned only
        dst[0] = make_uint2(pc[k].x, pc[k].y);
        dst[1] = make_uint2(pc[k].z, pc[k].w);
      }
    }
#pragma unroll
    for (int k = 0; k < NMC; ++k) {
      const int ch = k * 256 + threadIdx.x;
      const int tok = ch / HK, hd = ch % HK;
      if (tok < kAttTile) {
        const int mo = att_meta_off(tok, hd, HK);
        *reinterpret_cast<float4*>(lscale + mo) =
            make_float4(h2f(ps[k].x, 0), h2f(ps[k].x, 1), h2f(ps[k].y, 0), h2f(ps[k].y, 1));
        *reinterpret_cast<float4*>(lzterm + mo) = make_float4(h2f(pz[k].x, 0) + zbias, h2f(pz[k].x, 1) + zbias,
                                                              h2f(pz[k].y, 0) + zbias, h2f(pz[k].y, 1) + zbias);
      }
    }
  };

  // A-operand piece of this lane: row i of group sg (8 rows of kAttARow bytes per group), or the zero piece
  const unsigned char* a_row[NSETS];
  int a_step[NSETS];
#pragma unroll
  for (int set = 0; set < NSETS; ++set) {
    const bool on = i < 2 * (set ? rep_b : rep);
    a_row[set] = on ? abuf + set * (4 * 8 * kAttARow) + i * kAttARow + kg * 32 : azero;
    a_step[set] = on ? 8 * kAttARow : 0;
  }
  // two nibbles -> two bf16 values 128 + code.  Both constants are kept in vector registers (the
  // empty statement hides their values from the compiler, it emits no instruction): with a literal
  // operand the three-operand and-or instruction cannot be encoded and every expansion falls apart
  // into an AND and an OR.
  uint32_t kNib = 0x000f000fu, kExp = 0x43004300u;
  asm volatile("" : "+v"(kNib), "+v"(kExp));

  fetch(t0);
  for (int64_t n0 = t0; n0 < t1; n0 += TT) {
    __syncthreads();  // the previous tile has been consumed
    stage();
    __syncthreads();
    if constexpr (TI > 1) {
      if (a.row_acc || a.row_ts) {  // uniform
        // token j = 64 k + it of the tile is row j % TI of tile row j / TI: its probabilities are the staged
        // rows of the slabs of that parity
        float* const acc_rows = a.row_acc ? a.row_acc + (base_row + n0) : nullptr;
        float* const ts_rows = a.row_ts ? a.row_ts + (base_row + n0) : nullptr;
#pragma unroll
        for (int k = 0; k < TI; ++k) {
          const int j = k * kAttTile + it;
          const int vt = j / TI, par = j % TI;
          const float* lp = lprob + igrp * kAttPRow + (vt & ~15) + (vt & 3) * 4 + ((vt >> 2) & 3);
          float imp = 0.f;
#pragma unroll
          for (int hs = 0; hs < NSETS * HR; ++hs)
            imp = imp + lp[((hs / HR) * HK + par * HR + hs % HR) * 4 * kAttPRow];
          imp = imp + __shfl_xor(imp, 16, 64);
          imp = imp + __shfl_xor(imp, 32, 64);
          if (igrp == 0 && n0 + j < t1) {
            if (acc_rows) {
              float acc = pacc[k];
              if (a.decay != 1.0f) acc = acc * a.decay;
              acc_rows[j] = acc + imp;
            }
            if (ts_rows) {
              float now = a.now;
              asm volatile("" : "+v"(now));
              ts_rows[j] = now;
            }
          }
        }
      }
    }
    float acc = pacc[0];
    if (TI == 1 && (a.row_acc || a.row_ts)) {  // uniform
      // importance of the tile's tokens: four lanes per token add every fourth head, and two
      // exchanges add the four partial sums
      const int t = it;
      const int grp = igrp;
      const bool mine = grp == 0 && n0 + t < t1;
      // wave-uniform row pointers + a 32-bit lane offset: the addresses cost no registers
      // across the loop (a per-lane 64-bit address pair per plane had been spilled, and its
      // reload waited for the whole prefetch of the next tile)
      float* const acc_rows = a.row_acc ? a.row_acc + (base_row + n0) : nullptr;
      float* const ts_rows = a.row_ts ? a.row_ts + (base_row + n0) : nullptr;
      const float* lp = lprob + (t & ~15) + (t & 3) * 4 + ((t >> 2) & 3);
      float imp = 0.f;
      for (int hq = grp; hq < 4 * HK * NSETS; hq += 4) imp = imp + lp[hq * kAttPRow];
      imp = imp + __shfl_xor(imp, 16, 64);
      imp = imp + __shfl_xor(imp, 32, 64);
      if (mine) {
        if (acc_rows) {
          if (a.decay != 1.0f) acc = acc * a.decay;
          acc_rows[t] = acc + imp;
        }
        if (ts_rows) {
          float now = a.now;
          asm volatile("" : "+v"(now));  // copied from its scalar register here, not kept live across the loop
          ts_rows[t] = now;
        }
      }
    }
    // The next tile's loads go out AFTER the bookkeeping stores: the wait at the top of the
    // loop covers everything outstanding, and stores issued behind the loads had been
    // adding their latency to it (366 vs 347 us).
    if (n0 + TT < t1) fetch(n0 + TT);  // in flight while this tile is multiplied

#pragma unroll
    for (int hk = 0; hk < NH; ++hk) {   // kv head slot of this wavefront
      const int g = wave + 4 * hk;
      if (g >= HK) continue;  // uniform
      // ---- weights: this lane prepares head r of every set for four tokens, all four groups ----
      float4 s4[4], z4[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s4[j] = *reinterpret_cast<const float4*>(lscale + att_meta_off(tk + 4 * j, g, HK));
        z4[j] = *reinterpret_cast<const float4*>(lzterm + att_meta_off(tk + 4 * j, g, HK));
      }
#pragma unroll
      for (int set = 0; set < NSETS; ++set) {
        const int hs = hk * NSETS + set;
        const bool row_on = r < (set ? rep_b : rep);
        unsigned char* const aset = abuf + set * (4 * 8 * kAttARow);
        const float4 pv = *reinterpret_cast<const float4*>(lprob + (row_on ? (set * HK + g) * 4 + r : 0) * kAttPRow +
                                                           wkg * 16 + (lane & 3) * 4);
        const float p4[4] = {row_on ? pv.x : 0.f, row_on ? pv.y : 0.f, row_on ? pv.z : 0.f, row_on ? pv.w : 0.f};
#pragma unroll
        for (int sg = 0; sg < 4; ++sg) {
          // w = p * scale cut into a bf16 high part and a bf16 remainder.  The zero-point
          // sum uses the SAME two-part value, so that what the matrix core multiplies with
          // 128 + u is taken off again exactly.
          float hi[4], lo[4];
          float zsum = 0.f;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float sc = sg == 0 ? s4[j].x : sg == 1 ? s4[j].y : sg == 2 ? s4[j].z : s4[j].w;
            const float zt = sg == 0 ? z4[j].x : sg == 1 ? z4[j].y : sg == 2 ? z4[j].z : z4[j].w;
            const float w = p4[j] * sc;
            hi[j] = __uint_as_float(__float_as_uint(w) & 0xffff0000u);
            lo[j] = __uint_as_float(__float_as_uint(w - hi[j]) & 0xffff0000u);
            zsum = fmaf(hi[j] + lo[j], zt, zsum);
          }
          zacc[hs][sg] += zsum;
          // operand order inside 8 tokens is {0,4,1,5,2,6,3,7}: tokens (k, k+4) share a dword
          if (row_on) {
            uint32_t* rowh = reinterpret_cast<uint32_t*>(aset + (sg * 8 + 2 * r) * kAttARow + wkg * 32) + (lane & 3);
            uint32_t* rowl = reinterpret_cast<uint32_t*>(aset + (sg * 8 + 2 * r + 1) * kAttARow + wkg * 32) + (lane & 3);
            rowh[0] = (__float_as_uint(hi[0]) >> 16) | __float_as_uint(hi[1]);
            rowh[4] = (__float_as_uint(hi[2]) >> 16) | __float_as_uint(hi[3]);
            rowl[0] = (__float_as_uint(lo[0]) >> 16) | __float_as_uint(lo[1]);
            rowl[4] = (__float_as_uint(lo[2]) >> 16) | __float_as_uint(lo[3]);
          }
        }
      }
      // the rows were written by other lanes of this wavefront
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      // ---- products: rows 2r / 2r+1 of A against 16 dimensions of 64 tokens; the expanded
      // codes of a 16-dimension block serve every set ----
#pragma unroll
      for (int sg = 0; sg < 4; ++sg) {
        // a lane whose A row holds no head reads the zero piece: no branch, no cleared registers
        uint4 a1[NSETS], a2[NSETS];
#pragma unroll
        for (int set = 0; set < NSETS; ++set) {
          const uint4* ap = reinterpret_cast<const uint4*>(a_row[set] + sg * a_step[set]);
          a1[set] = ap[0];
          a2[set] = ap[1];
        }
#pragma unroll
        for (int dbl = 0; dbl < 2; ++dbl) {
          const int db = 2 * sg + dbl;
          // lane i lends the 8 code bytes of token kg*16+i that cover dims db*16..+15 and
          // receives the nibbles of dimension db*16+i from its 16 neighbours
          const pikv_i32x2 tr = __builtin_amdgcn_ds_read_tr4_b64_v2i32(
              (pikv_i32x2 __attribute__((address_space(3)))*)(lcodes + (kg * 16 + i) * RS + g * 64 + db * 8));
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const uint32_t u = Q::sym ? ((uint32_t)tr[half] ^ 0x88888888u) : (uint32_t)tr[half];
            const uint4 bb = make_uint4(and_or(u, kNib, kExp), and_or(u >> 4, kNib, kExp), and_or(u >> 8, kNib, kExp),
                                        and_or(u >> 12, kNib, kExp));
#pragma unroll
            for (int set = 0; set < NSETS; ++set)
              C[hk * NSETS + set][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  __builtin_bit_cast(pikv_bf16x8, half ? a2[set] : a1[set]), __builtin_bit_cast(pikv_bf16x8, bb),
                  C[hk * NSETS + set][db], 0, 0, 0);
          }
        }
      }
      // the next head's rows go into the same buffer
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }

  // Epilogue.  C: lane (dimension i, rows 4*kg + q): rows 2r / 2r+1 are the two parts of
  // head r, so head 2*kg is q = 0,1 and head 2*kg+1 is q = 2,3.  The zero-point sums sit
  // spread over the 16 lanes that prepared head r.
  __syncthreads();
  float* zl = reinterpret_cast<float*>(att_lds);  // [wave][kv head slot, set][r][sg]
  const int hps = NARROW ? 128 / a.head_dim : 1;   // kv heads per slab
  const int rep1 = rep_all / hps;                  // query heads per kv head
#pragma unroll
  for (int hs = 0; hs < NI; ++hs)
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) {
      const float z = group_sum_dpp(zacc[hs][sg], 16);
      if ((lane & 15) == 0) zl[((wave * NI + hs) * 4 + r) * 4 + sg] = z;
    }
  __syncthreads();
  if constexpr (TI > 1) {
    // the TI slabs of a kv head hold partial outputs over different tokens: added in LDS, parity by parity
    float* ol = zl + 4 * NI * 4 * 4;   // [kv head][head of the launch: 4 * set + ro][128]
    for (int par = 0; par < TI; ++par) {
#pragma unroll
      for (int hs = 0; hs < NI; ++hs) {
        const int set = hs % NSETS;
        const int g = wave + 4 * (hs / NSETS);
        if (g >= HK || g / HR != par) continue;  // uniform
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          const int ro = 2 * kg + rr;
          if (ro >= (set ? rep_b : rep)) continue;
          float* o = ol + ((g % HR) * (4 * NSETS) + 4 * set + ro) * 128;
#pragma unroll
          for (int db = 0; db < 8; ++db) {
            const float v = (C[hs][db][2 * rr] + C[hs][db][2 * rr + 1]) - zl[((wave * NI + hs) * 4 + ro) * 4 + (db >> 1)];
            o[db * 16 + i] = par == 0 ? v : o[db * 16 + i] + v;
          }
        }
      }
      __syncthreads();
    }
    const int heads = rep + rep_b;   // heads of a slab in this launch
    for (int idx = threadIdx.x; idx < HR * 4 * NSETS * 128; idx += 256) {
      const int row = idx >> 7, g = row / (4 * NSETS), hl = row % (4 * NSETS), d = idx & 127;
      if (hl >= heads) continue;
      const int64_t ohead = ((int64_t)xb * a.n_caches + c) * a.n_q_heads + g * rep_all + a.head_off + hl;
      if constexpr (!NARROW) {
        a.partial[ohead * 128 + d] = ol[idx];
      } else {
        // a narrow head keeps the dimensions of its own kv head of the slab
        const int hh = (a.head_off + hl) / rep1;
        if (d / a.head_dim == hh) a.partial[ohead * a.head_dim + d - hh * a.head_dim] = ol[idx];
      }
    }
    return;
  }
#pragma unroll
  for (int hs = 0; hs < NI; ++hs) {
    const int set = hs % NSETS;
    const int g = wave + 4 * (hs / NSETS);
    if (g >= HK) continue;
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      const int ro = 2 * kg + rr;  // head (inside the set) held by this lane
      if (ro >= (set ? rep_b : rep)) continue;
      const int hro = a.head_off + 4 * set + ro;   // head inside the kv group
      const int64_t ohead = ((int64_t)xb * a.n_caches + c) * a.n_q_heads + (kv_off + g) * rep_all + hro;
      if constexpr (!NARROW) {
        float* o = a.partial + ohead * 128;
#pragma unroll
        for (int db = 0; db < 8; ++db)
          o[db * 16 + i] = (C[hs][db][2 * rr] + C[hs][db][2 * rr + 1]) - zl[((wave * NI + hs) * 4 + ro) * 4 + (db >> 1)];
      } else {
        // kv head hh of the slab owns the 16-dimension blocks db with db * hps / 8 == hh
        const int hh = hro / rep1;
        float* o = a.partial + ohead * a.head_dim - hh * a.head_dim;
#pragma unroll
        for (int db = 0; db < 8; ++db)
          if ((db * hps) >> 3 == hh)
            o[db * 16 + i] = (C[hs][db][2 * rr] + C[hs][db][2 * rr + 1]) - zl[((wave * NI + hs) * 4 + ro) * 4 + (db >> 1)];
      }
    }
  }
}

// ---- matrix-core form, 8-bit codes ------------------------------------------------------
// Per-head (or coarser) scales, head_dim 128 (64 and 32 as slabs of two / four heads), 2..8 query heads per
// slab.  Same plan as
// the 4-bit kernel - contraction over tokens, codes staged in LDS as stored and read back
// transposed - with two differences.  An 8-bit code is not exact as one bf16, so a stored
// byte u is fed as its nibbles, u = 16*hi + lo, each exact as 128 + nibble, against two
// copies of the weights, w and 16*w (a power of two: exact).  And ds_read_b64_tr_b8 hands
// result lane i byte q = byte i%8 of source lane 2q + i/8 (per 16 lanes): source lane j
// therefore points at token T[j/2], dims d0 + 8*(j%2) .. +7, which makes result lane i
// hold dimension d0 + i of tokens T[0..7] - the B operand layout, tokens in natural order.
// With nibbles fed as 16 + nibble (0x4180 | nibble << 3):
//   sum_n w_n*(16 + lo) + 16*w_n*(16 + hi) = sum_n w_n*u_n + 272*sum_n w_n
// and the value wanted is sum_n w_n*(u_n - zz_n), zz = 128 (symmetric) or the zero point.
// The offset term is many times the result, and taken off at the end it would cost the
// float32 sum its low bits over thousands of tokens; a third product per tile, the weights
// against the constant column -(272 + zz_n), removes it inside the accumulation instead.
constexpr int kAtt8Tile = 32;    // cached tokens per step
constexpr int kAtt8ARow = 80;    // bytes per staged A row: 32 tokens x bf16 + 16 (bank spread)
constexpr int kAtt8PRow = 36;    // floats per query head of staged probabilities: 32 tokens + 4

static size_t attend_mfma8_lds_bytes(int n_slabs, int n_q_heads, int hps) {
  // codes [32 tokens][n_slabs*128 + 8]; scale and zero term [32][n_slabs*hps] float; A rows per
  // wavefront [2 copies][16 rows][kAtt8ARow]; probabilities [query head][kAtt8PRow]
  return (size_t)kAtt8Tile * (n_slabs * 128 + 8) + 2 * (size_t)kAtt8Tile * n_slabs * hps * 4 +
         4 * (size_t)2 * 16 * kAtt8ARow + (size_t)n_q_heads * kAtt8PRow * 4;
}

// HK = n_kv_heads (1..8); 2..8 query heads per kv head, at most 64 query heads.
// Heads narrower than 128 (HPS = 128 / head_dim = 2 or 4): the kernel's kv heads are 128-dimension
// slabs of the cached row, each the stored bytes of HPS neighbouring kv heads with a scale (and
// zero point) each; the query heads of a slab are the heads of those kv heads in order.  A query
// head is weighted with its own kv head's scale, multiplied with the whole slab, and only the
// dimensions of its own kv head are written out.
// TI > 1 (rows of 1 to 4 kv heads of 128): TI neighbouring cached rows as ONE row of HK = TI x (real slabs)
// slabs, slab g' = (row parity) * slabs + kv head, exactly as in the 4-bit kernel: tiles of 32 x TI tokens,
// every wavefront with a slab to multiply, the TI partial outputs of a head added at the end.  The staged
// probabilities are [parity][query head] rows.
template <int SCHEME, int HK, int HPS = 1, int TI = 1>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void attend_mfma_i8_kernel(AttendArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 8, "8-bit schemes only");
  static_assert(HK >= 1 && HK <= 8, "1 to 8 kv heads");
  static_assert(TI == 1 || (HPS == 1 && HK % TI == 0), "interleaved rows: whole rows of 128-wide heads");
  constexpr int HKR = HK / TI;            // slabs of a cached row
  constexpr int TT = kAtt8Tile * TI;      // cached tokens per tile
  constexpr int NH = (HK + 3) / 4;   // kv heads per wavefront
  constexpr int RS = HK * 128 + 8;   // bytes per token row of staged codes
  constexpr int LPR = HK * 8;        // 16-byte chunks per cached row
  constexpr int NCH = kAtt8Tile * LPR / 256;  // code chunks per thread (= HK)
  constexpr int HR = HK * HPS;                // stored kv heads = (scale, zero) pairs per token
  constexpr int NMT = (kAtt8Tile * HR + 255) / 256;  // metadata pairs per thread
  extern __shared__ __align__(16) unsigned char att8_lds[];
  unsigned char* lcodes = att8_lds;
  float* lscale = reinterpret_cast<float*>(att8_lds + kAtt8Tile * RS);
  float* lzterm = lscale + kAtt8Tile * HR;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  unsigned char* abuf = reinterpret_cast<unsigned char*>(lzterm + kAtt8Tile * HR) + wave * (2 * 16 * kAtt8ARow);
  float* lprob = reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(lzterm + kAtt8Tile * HR) +
                                          4 * (2 * 16 * kAtt8ARow));

  const int c = blockIdx.y;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  const int64_t t0 = (int64_t)blockIdx.x * a.tokens_per_block;
  const int64_t t1 = (t0 + a.tokens_per_block < len) ? t0 + a.tokens_per_block : len;
  if (t0 >= t1) {  // nothing cached in this range: the partial is zero
    for (int idx = threadIdx.x; idx < a.n_q_heads * a.head_dim; idx += 256)
      a.partial[((int64_t)blockIdx.x * a.n_caches + c) * a.n_q_heads * a.head_dim + idx] = 0.f;
    return;
  }
  // a launch serves heads a.head_off .. a.head_off + rep - 1 of every kv head (more than 8 per kv head: two
  // launches; narrow heads are launched with head_off = 0 only); the staged rows count these heads alone
  const int rep_all = a.n_q_heads / HKR;
  const int rep = rep_all - a.head_off < 8 ? rep_all - a.head_off : 8;  // 1..8
  const int nql = HKR * rep;         // staged heads: row (kv head) * rep + head of the launch
  const int rep1 = rep / HPS;        // query heads per stored kv head
  const int groups_per_row = (HKR * 128) / a.group;
  // matrix-core roles: A row / B,C column i, token group kg (tokens 8*kg .. 8*kg+7 of the tile)
  const int i = lane & 15;
  const int kg = lane >> 4;
  // weight-preparation roles: head r of the kv group, tokens t4 .. t4+3 of the tile
  const int r = lane >> 3;
  const int t4 = (lane & 7) * 4;
  const bool row_on = r < rep;
  const int hh_w = (HPS > 1 && row_on) ? r / rep1 : 0;   // stored kv head, inside its slab, of the head this lane weights
  const bool normalise = a.head_stats != nullptr;
  const int64_t base_row = a.row_base[c];

  pikv_f32x4 C[NH][8];
#pragma unroll
  for (int hs = 0; hs < NH; ++hs)
#pragma unroll
    for (int d = 0; d < 8; ++d) C[hs][d] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
  // score-staging role: query head sh, tokens st8..st8+7 of the tile (64 heads x 4 runs; interleaved rows:
  // 64 / TI heads x 4 TI runs)
  const int sh = threadIdx.x / (4 * TI);
  const int st8 = (threadIdx.x % (4 * TI)) * 8;
  const bool s_on = sh < nql;
  const int s_hq = s_on ? (sh / rep) * rep_all + a.head_off + sh % rep : 0;   // the query head itself
  const float* srow = a.scores + ((int64_t)c * a.n_q_heads + s_hq) * a.score_stride;
  float smx = 0.f, srz = 1.f;
  if (normalise) {
    smx = a.head_stats[((int64_t)c * a.n_q_heads + s_hq) * 2];
    srz = 1.0f / a.head_stats[((int64_t)c * a.n_q_heads + s_hq) * 2 + 1];
  }
  const bool s_vec = (a.score_stride & 3) == 0 && (reinterpret_cast<uintptr_t>(a.scores) & 15) == 0;
  const float s_off = normalise ? -INFINITY : 0.f;  // what a token past the end contributes: p = 0
  // importance role: wavefront w owns tokens 8w..8w+7 of a tile, eight lanes per token
  const int it = wave * 8 + (lane & 7);
  const int igrp = lane >> 3;

  // registers that carry the next tile from HBM to LDS
  uint4 pc[NCH];
  float ps[NMT], pz[NMT], pacc[TI];
#pragma unroll
  for (int k = 0; k < TI; ++k) pacc[k] = 0.f;
  float psc[8];
  auto fetch = [&](int64_t n0) {
#pragma unroll
    for (int k = 0; k < TI; ++k)
      if (a.row_acc && igrp == 0 && n0 + k * kAtt8Tile + it < t1)
        pacc[k] = (a.row_acc + (base_row + n0))[k * kAtt8Tile + it];  // uniform base + lane
    if (s_on) {
      const int64_t n = n0 + st8;
      if (s_vec && n + 8 <= t1) {
        const float4 lo4 = *reinterpret_cast<const float4*>(srow + n);
        const float4 hi4 = *reinterpret_cast<const float4*>(srow + n + 4);
        psc[0] = lo4.x, psc[1] = lo4.y, psc[2] = lo4.z, psc[3] = lo4.w;
        psc[4] = hi4.x, psc[5] = hi4.y, psc[6] = hi4.z, psc[7] = hi4.w;
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) psc[k] = n + k < t1 ? srow[n + k] : s_off;
      }
    }
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int ch = k * 256 + threadIdx.x;   // 16-byte chunk of the tile's rows, which lie side by side
      pc[k] = make_uint4(0, 0, 0, 0);
      if (n0 + ch / (LPR / TI) < t1)
        pc[k] = ld16(reinterpret_cast<const char*>(a.codes) + ((base_row + n0) * (LPR / TI) + ch) * 16);
    }
#pragma unroll
    for (int k = 0; k < NMT; ++k) {  // (token, stored kv head) metadata pairs
      const int ch = k * 256 + threadIdx.x;
      const int tok = ch / HR, hd = ch % HR;
      ps[k] = 0.f;
      pz[k] = 0.f;
      // (interleaved rows: slab hd of tile row tok is kv head hd % HKR of cached row tok * TI + hd / HKR)
      const int64_t rtok = TI == 1 ? n0 + tok : n0 + tok * TI + hd / HKR;
      if (tok < kAtt8Tile && rtok < t1) {
        const int64_t mi = (base_row + rtok) * groups_per_row + ((TI == 1 ? hd : hd % HKR) * (128 / HPS)) / a.group;
        ps[k] = reinterpret_cast<const float*>(a.scale)[mi];
        if constexpr (!Q::sym) pz[k] = reinterpret_cast<const float*>(a.zero)[mi];
      }
    }
  };
  auto stage = [&]() {
    if (s_on) {
      float4 v0, v1;
      v0.x = prob_of(psc[0], smx, srz, normalise), v0.y = prob_of(psc[1], smx, srz, normalise);
      v0.z = prob_of(psc[2], smx, srz, normalise), v0.w = prob_of(psc[3], smx, srz, normalise);
      v1.x = prob_of(psc[4], smx, srz, normalise), v1.y = prob_of(psc[5], smx, srz, normalise);
      v1.z = prob_of(psc[6], smx, srz, normalise), v1.w = prob_of(psc[7], smx, srz, normalise);
      if constexpr (TI == 1) {
        *reinterpret_cast<float4*>(lprob + sh * kAtt8PRow + st8) = v0;
        *reinterpret_cast<float4*>(lprob + sh * kAtt8PRow + st8 + 4) = v1;
      } else {
        // token j of the tile is row j % TI of tile row j / TI
        const float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int k = 0; k < 8; ++k)
          lprob[(((st8 + k) % TI) * nql + sh) * kAtt8PRow + (st8 + k) / TI] = v[k];
      }
    }
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int ch = k * 256 + threadIdx.x;
      const int tok = ch / LPR, off = ch % LPR;
      uint2* dst = reinterpret_cast<uint2*>(lcodes + tok * RS + off * 16);  // rows are 8-byte aligned only
      dst[0] = make_uint2(pc[k].x, pc[k].y);
      dst[1] = make_uint2(pc[k].z, pc[k].w);
    }
#pragma unroll
    for (int k = 0; k < NMT; ++k) {
      const int ch = k * 256 + threadIdx.x;   // = tok * HR + stored kv head
      if (ch < kAtt8Tile * HR) {
        lscale[ch] = ps[k];
        lzterm[ch] = -(272.0f + (Q::sym ? 128.0f : pz[k]));
      }
    }
  };
  auto bf16_hi = [](float v) { return __float_as_uint(v) & 0xffff0000u; };

  fetch(t0);
  for (int64_t n0 = t0; n0 < t1; n0 += TT) {
    __syncthreads();  // the previous tile has been consumed
    stage();
    __syncthreads();
    float accs[TI];
#pragma unroll
    for (int k = 0; k < TI; ++k) accs[k] = pacc[k];
    float acc = accs[0];
    if (n0 + TT < t1) fetch(n0 + TT);  // in flight while this tile is multiplied
    if constexpr (TI > 1) {
      if (a.row_acc || a.row_ts) {  // uniform
        float* const acc_rows = a.row_acc ? a.row_acc + (base_row + n0) : nullptr;
        float* const ts_rows = a.row_ts ? a.row_ts + (base_row + n0) : nullptr;
#pragma unroll
        for (int k = 0; k < TI; ++k) {
          const int j = k * kAtt8Tile + it;   // token of the tile: row j % TI of tile row j / TI
          const float* lp = lprob + (j % TI) * nql * kAtt8PRow + j / TI;
          float imp = 0.f;
          for (int hq = igrp; hq < nql; hq += 8) imp = imp + lp[hq * kAtt8PRow];
          imp = imp + __shfl_xor(imp, 8, 64);
          imp = imp + __shfl_xor(imp, 16, 64);
          imp = imp + __shfl_xor(imp, 32, 64);
          if (igrp == 0 && n0 + j < t1) {
            if (acc_rows) {
              float av = accs[k];
              if (a.decay != 1.0f) av = av * a.decay;
              acc_rows[j] = av + imp;
            }
            if (ts_rows) {
              float now = a.now;
              asm volatile("" : "+v"(now));
              ts_rows[j] = now;
            }
          }
        }
      }
    }
    if (TI == 1 && (a.row_acc || a.row_ts)) {  // uniform
      const bool mine = igrp == 0 && n0 + it < t1;
      const int t = it;
      // wave-uniform row pointers + a 32-bit lane offset (no per-lane address registers live
      // across the loop)
      float* const acc_rows = a.row_acc ? a.row_acc + (base_row + n0) : nullptr;
      float* const ts_rows = a.row_ts ? a.row_ts + (base_row + n0) : nullptr;
      float imp = 0.f;
      for (int hq = igrp; hq < nql; hq += 8) imp = imp + lprob[hq * kAtt8PRow + it];
      imp = imp + __shfl_xor(imp, 8, 64);
      imp = imp + __shfl_xor(imp, 16, 64);
      imp = imp + __shfl_xor(imp, 32, 64);
      if (mine) {
        if (acc_rows) {
          if (a.decay != 1.0f) acc = acc * a.decay;
          acc_rows[t] = acc + imp;
        }
        if (ts_rows) {
          float now = a.now;
          asm volatile("" : "+v"(now));  // copied from its scalar register here, not kept live across the loop
          ts_rows[t] = now;
        }
      }
    }

#pragma unroll
    for (int hs = 0; hs < NH; ++hs) {
      const int g = wave + 4 * hs;
      if (g >= HK) continue;  // uniform
      // ---- weights: head r, tokens t4..t4+3: w = p * scale as bf16 high part + remainder,
      // both also times 16; the bias sum uses the same two-part value ----
      const float4 pv = *reinterpret_cast<const float4*>(lprob + (row_on ? g * rep + r : 0) * kAtt8PRow + t4);
      const float p4[4] = {row_on ? pv.x : 0.f, row_on ? pv.y : 0.f, row_on ? pv.z : 0.f, row_on ? pv.w : 0.f};
      uint32_t hi[4], lo[4], hi16[4], lo16[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float w = p4[j] * lscale[(t4 + j) * HR + g * HPS + hh_w];
        const float wh = __uint_as_float(bf16_hi(w));
        const float wl = __uint_as_float(bf16_hi(w - wh));
        hi[j] = __float_as_uint(wh) >> 16;
        lo[j] = __float_as_uint(wl) >> 16;
        hi16[j] = __float_as_uint(wh * 16.0f) >> 16;
        lo16[j] = __float_as_uint(wl * 16.0f) >> 16;
      }
      if (row_on) {
        unsigned char* rowp = abuf + (2 * r) * kAtt8ARow + t4 * 2;
        *reinterpret_cast<uint2*>(rowp) = make_uint2(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16));
        *reinterpret_cast<uint2*>(rowp + kAtt8ARow) = make_uint2(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16));
        *reinterpret_cast<uint2*>(rowp + 16 * kAtt8ARow) = make_uint2(hi16[0] | (hi16[1] << 16), hi16[2] | (hi16[3] << 16));
        *reinterpret_cast<uint2*>(rowp + 17 * kAtt8ARow) = make_uint2(lo16[0] | (lo16[1] << 16), lo16[2] | (lo16[3] << 16));
      }
      // the rows were written by other lanes of this wavefront
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      // ---- products: rows 2r / 2r+1 of A against 16 dimensions of 32 tokens ----
      uint4 a1 = make_uint4(0, 0, 0, 0), a16 = make_uint4(0, 0, 0, 0);
      if (i < 2 * rep) {
        a1 = *reinterpret_cast<const uint4*>(abuf + i * kAtt8ARow + kg * 16);
        a16 = *reinterpret_cast<const uint4*>(abuf + (16 + i) * kAtt8ARow + kg * 16);
      }
      // the offset column of tokens 8*kg .. 8*kg+7 (the same for every dimension), as a bf16
      // high part and - asymmetric schemes, whose zero points are arbitrary floats - a remainder
      // (narrow heads: the column of the stored kv head that owns the dimensions, rebuilt where the
      // 16-dimension blocks pass from one kv head to the next)
      uint4 bz = make_uint4(0, 0, 0, 0), bzl = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        if (db % (8 / HPS) == 0) {
          uint32_t zh[8], zlw[8];
#pragma unroll
          for (int q8 = 0; q8 < 8; ++q8) {
            const float zt = lzterm[(kg * 8 + q8) * HR + g * HPS + db / (8 / HPS)];
            const float zhf = __uint_as_float(bf16_hi(zt));
            zh[q8] = __float_as_uint(zhf) >> 16;
            zlw[q8] = bf16_hi(zt - zhf) >> 16;
          }
          bz = make_uint4(zh[0] | (zh[1] << 16), zh[2] | (zh[3] << 16), zh[4] | (zh[5] << 16), zh[6] | (zh[7] << 16));
          bzl = make_uint4(zlw[0] | (zlw[1] << 16), zlw[2] | (zlw[3] << 16), zlw[4] | (zlw[5] << 16), zlw[6] | (zlw[7] << 16));
        }
        // source lane i points at token 8*kg + i/2, dims 16*db + 8*(i%2) .. +7; result lane i
        // holds dimension 16*db + i of tokens 8*kg .. 8*kg+7
        const pikv_i32x2 tr = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (pikv_i32x2 __attribute__((address_space(3)))*)(lcodes + (kg * 8 + (i >> 1)) * RS + g * 128 + db * 16 +
                                                            8 * (i & 1)));
        const uint32_t x0 = Q::sym ? ((uint32_t)tr[0] ^ 0x80808080u) : (uint32_t)tr[0];
        const uint32_t x1 = Q::sym ? ((uint32_t)tr[1] ^ 0x80808080u) : (uint32_t)tr[1];
        // nibble n -> bf16 16 + n = 0x4180 | n << 3: bytes {0x80 | n << 3, 0x41}
        const uint32_t l0 = ((x0 << 3) & 0x78787878u) | 0x80808080u, l1 = ((x1 << 3) & 0x78787878u) | 0x80808080u;
        const uint32_t h0 = ((x0 >> 1) & 0x78787878u) | 0x80808080u, h1 = ((x1 >> 1) & 0x78787878u) | 0x80808080u;
        const uint32_t k43 = 0x41414141u;
        const uint4 blo = make_uint4(__builtin_amdgcn_perm(k43, l0, 0x05010400u), __builtin_amdgcn_perm(k43, l0, 0x05030402u),
                                     __builtin_amdgcn_perm(k43, l1, 0x05010400u), __builtin_amdgcn_perm(k43, l1, 0x05030402u));
        const uint4 bhi = make_uint4(__builtin_amdgcn_perm(k43, h0, 0x05010400u), __builtin_amdgcn_perm(k43, h0, 0x05030402u),
                                     __builtin_amdgcn_perm(k43, h1, 0x05010400u), __builtin_amdgcn_perm(k43, h1, 0x05030402u));
        C[hs][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, a1),
                                                            __builtin_bit_cast(pikv_bf16x8, blo), C[hs][db], 0, 0, 0);
        C[hs][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, a16),
                                                            __builtin_bit_cast(pikv_bf16x8, bhi), C[hs][db], 0, 0, 0);
        C[hs][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, a1),
                                                            __builtin_bit_cast(pikv_bf16x8, bz), C[hs][db], 0, 0, 0);
        if constexpr (!Q::sym)
          C[hs][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, a1),
                                                              __builtin_bit_cast(pikv_bf16x8, bzl), C[hs][db], 0, 0, 0);
      }
      // the next head's rows go into the same buffer
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }

  // Epilogue.  C: lane (dimension i, rows 4*kg + q): rows 2r / 2r+1 are the two parts of head r,
  // so head 2*kg is q = 0,1 and head 2*kg+1 is q = 2,3.
  if constexpr (TI > 1) {
    // the TI slabs of a kv head hold partial outputs over different tokens: added in LDS, parity by parity
    __syncthreads();
    float* ol = reinterpret_cast<float*>(att8_lds);   // [kv head][head of the kv group, 8 slots][128]
    for (int par = 0; par < TI; ++par) {
#pragma unroll
      for (int hs = 0; hs < NH; ++hs) {
        const int g = wave + 4 * hs;
        if (g >= HK || g / HKR != par) continue;  // uniform
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          const int ro = 2 * kg + rr;
          if (ro >= rep) continue;
          float* o = ol + ((g % HKR) * 8 + ro) * 128;
#pragma unroll
          for (int db = 0; db < 8; ++db) {
            const float v = C[hs][db][2 * rr] + C[hs][db][2 * rr + 1];
            o[db * 16 + i] = par == 0 ? v : o[db * 16 + i] + v;
          }
        }
      }
      __syncthreads();
    }
    for (int idx = threadIdx.x; idx < HKR * 8 * 128; idx += 256) {
      const int row = idx >> 7, g = row >> 3, ro = row & 7;
      if (ro < rep)
        a.partial[(((int64_t)blockIdx.x * a.n_caches + c) * a.n_q_heads + g * rep_all + a.head_off + ro) * 128 + (idx & 127)] = ol[idx];
    }
    return;
  }
#pragma unroll
  for (int hs = 0; hs < NH; ++hs) {
    const int g = wave + 4 * hs;
    if (g >= HK) continue;
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      const int ro = 2 * kg + rr;  // head (inside the kv group) held by this lane
      if (ro >= rep) continue;
      const int hh = HPS > 1 ? ro / rep1 : 0;   // stored kv head of the slab that owns this head: blocks db with db * HPS / 8 == hh
      float* o = a.partial + (((int64_t)blockIdx.x * a.n_caches + c) * a.n_q_heads + g * rep_all + a.head_off + ro) * (128 / HPS) -
                 hh * (128 / HPS);
#pragma unroll
      for (int db = 0; db < 8; ++db)
        if (HPS == 1 || db / (8 / HPS) == hh) o[db * 16 + i] = C[hs][db][2 * rr] + C[hs][db][2 * rr + 1];
    }
  }
}

template <int SCHEME, int HPS>
static void launch_attend_mfma8_slabs(int n_slabs, dim3 grid, hipStream_t st, const AttendArgs& a) {
  const size_t lds = attend_mfma8_lds_bytes(n_slabs, a.n_q_heads, HPS);
  switch (n_slabs) {
    case 1: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 1, HPS>), grid, dim3(256), lds, st, a); break;
    case 2: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 2, HPS>), grid, dim3(256), lds, st, a); break;
    case 3: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 3, HPS>), grid, dim3(256), lds, st, a); break;
    case 4: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 4, HPS>), grid, dim3(256), lds, st, a); break;
    case 5: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 5, HPS>), grid, dim3(256), lds, st, a); break;
    case 6: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 6, HPS>), grid, dim3(256), lds, st, a); break;
    case 7: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 7, HPS>), grid, dim3(256), lds, st, a); break;
    default: hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 8, HPS>), grid, dim3(256), lds, st, a); break;
  }
}
template <int SCHEME>
static void launch_attend_mfma8_heads(int n_slabs, int hps, dim3 grid, hipStream_t st, const AttendArgs& a);
// All query heads of every kv head: up to eight per launch; a later launch (same codes, next heads) adds its
// share of the importance to the accumulators that the first one has decayed.
template <int SCHEME>
static void launch_attend_mfma8(int n_slabs, int hps, dim3 grid, hipStream_t st, AttendArgs a) {
  const int rep = a.n_q_heads / n_slabs;
  for (int off = 0; off < rep; off += 8) {
    a.head_off = off;
    if (off > 0) a.decay = 1.0f;
    launch_attend_mfma8_heads<SCHEME>(n_slabs, hps, grid, st, a);
  }
}
template <int SCHEME>
static void launch_attend_mfma8_heads(int n_slabs, int hps, dim3 grid, hipStream_t st, const AttendArgs& a) {
  if (hps == 1 && n_slabs <= 3 && a.tokens_per_block % (kAtt8Tile * 8) == 0) {
    // rows of few slabs: 8, 4 or 2 neighbouring rows as one row of (up to) 8 slabs (pairs of rows of 4 slabs
    // measured the same as single rows: 322 vs 325 us at 64 caches x 32768 tokens x 16 query heads)
    const int ti = n_slabs == 1 ? 8 : n_slabs == 2 ? 4 : 2;
    const int staged = a.n_q_heads < n_slabs * 8 ? a.n_q_heads : n_slabs * 8;   // heads of one launch
    const size_t lds = attend_mfma8_lds_bytes(n_slabs * ti, staged * ti, 1);
    if (n_slabs == 1) hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 8, 1, 8>), grid, dim3(256), lds, st, a);
    else if (n_slabs == 2) hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 8, 1, 4>), grid, dim3(256), lds, st, a);
    else hipLaunchKernelGGL((attend_mfma_i8_kernel<SCHEME, 6, 1, 2>), grid, dim3(256), lds, st, a);
    return;
  }
  if (hps == 1) launch_attend_mfma8_slabs<SCHEME, 1>(n_slabs, grid, st, a);
  else if (hps == 2) launch_attend_mfma8_slabs<SCHEME, 2>(n_slabs, grid, st, a);
  else launch_attend_mfma8_slabs<SCHEME, 4>(n_slabs, grid, st, a);
}

template <int SCHEME, bool EXCH, bool NARROW>
static void launch_attend_mfma_slabs(int n_slabs, int nsets, dim3 grid, hipStream_t st, const AttendArgs& a) {
  const size_t lds = attend_mfma_lds_bytes(n_slabs, a.n_q_heads, nsets);
  if (nsets == 2) {
    switch (n_slabs) {
      case 1: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 1, EXCH, NARROW, 2>), grid, dim3(256), lds, st, a); break;
      case 2: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 2, EXCH, NARROW, 2>), grid, dim3(256), lds, st, a); break;
      case 3: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 3, EXCH, NARROW, 2>), grid, dim3(256), lds, st, a); break;
      default: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 4, EXCH, NARROW, 2>), grid, dim3(256), lds, st, a); break;
    }
    return;
  }
  switch (n_slabs) {
    case 1: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 1, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    case 2: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 2, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    case 3: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 3, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    case 4: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 4, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    case 5: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 5, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    case 6: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 6, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    case 7: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 7, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
    default: hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 8, EXCH, NARROW>), grid, dim3(256), lds, st, a); break;
  }
}
// All query heads of every slab: four per launch, or - up to 4 slabs - eight per launch in two sets.  A
// later launch (same codes, next heads) adds its share to the accumulators that the first one has decayed.
template <int SCHEME, bool EXCH = false>
static void launch_attend_mfma(int n_slabs, int heads_per_slab, dim3 grid, hipStream_t st, AttendArgs a) {
  // split rows (heads of 128; whole groups of 8 slabs for more than 8 are checked by the caller): slabs per group
  const bool wide = heads_per_slab > 4 && a.head_dim == 128;
  const int gs = wide && n_slabs >= 8 && n_slabs % 4 == 0 ? 4 : wide && n_slabs == 6 ? 3 : n_slabs > 8 ? 8 : 0;
  if (gs) {
    // the groups of a token range are neighbouring blocks; the H2O bookkeeping runs first, as a kernel of its own
    if (a.row_acc || a.row_ts) {
      const dim3 ig((unsigned)((a.max_len + kAttTile - 1) / kAttTile), (unsigned)a.n_caches);
      if (EXCH) hipLaunchKernelGGL(exch_importance_kernel, ig, dim3(256), 0, st, a);
      else hipLaunchKernelGGL(attend_importance_kernel, dim3((unsigned)((a.max_len + 255) / 256), (unsigned)a.n_caches), dim3(256), 0, st, a);
    }
    a.row_acc = nullptr;
    a.row_ts = nullptr;
    a.row_slabs = n_slabs;
    const dim3 sgrid(grid.x * (unsigned)(n_slabs / gs), grid.y);
    const int nsets = gs == 8 ? 1 : 2;
    const size_t lds = attend_mfma_lds_bytes(gs, a.n_q_heads, nsets);
    for (int off = 0; off < heads_per_slab; off += 4 * nsets) {
      a.head_off = off;
      if (gs == 8) hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 8, EXCH, false, 1, true>), sgrid, dim3(256), lds, st, a);
      else if (gs == 4) hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 4, EXCH, false, 2, true>), sgrid, dim3(256), lds, st, a);
      else hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, 3, EXCH, false, 2, true>), sgrid, dim3(256), lds, st, a);
    }
    return;
  }
  const int nsets = (n_slabs <= 4 && heads_per_slab > 4) ? 2 : 1;
  // rows of few slabs: 8, 4 or 2 neighbouring rows as one (a block's token range must hold whole tiles of them)
  int ti = 1;
  if (n_slabs <= 4) {
    const int room = (nsets == 2 ? 4 : 8) / n_slabs;
    ti = room >= 8 ? 8 : room >= 4 ? 4 : room >= 2 ? 2 : 1;
    while (ti > 1 && a.tokens_per_block % (kAttTile * ti) != 0) ti >>= 1;
    // 4 slabs already fill the wavefronts; pairs of rows gain 5 % on the exchange rows and lose 4 % on float scores
    if (n_slabs == 4 && !EXCH) ti = 1;
  }
  for (int off = 0; off < heads_per_slab; off += 4 * nsets) {
    a.head_off = off;
    if (off > 0) a.decay = 1.0f;
    if (ti > 1) {
      const int hk = n_slabs * ti;
      const size_t lds = attend_mfma_lds_bytes(hk, a.n_q_heads, nsets);
#define PIKV_ATT_ROWS(HKV, TIV, NS)                                                                              \
  if (hk == HKV && ti == TIV && nsets == NS) {                                                                   \
    if (a.head_dim == 128)                                                                                       \
      hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, HKV, EXCH, false, NS, false, TIV>), grid, dim3(256), lds, st, a); \
    else                                                                                                         \
      hipLaunchKernelGGL((attend_mfma_i4_kernel<SCHEME, HKV, EXCH, true, NS, false, TIV>), grid, dim3(256), lds, st, a);  \
  }
      PIKV_ATT_ROWS(8, 8, 1)   // 1 kv head
      PIKV_ATT_ROWS(4, 4, 1)   // ... token ranges of 256
      PIKV_ATT_ROWS(8, 4, 1)   // 2
      PIKV_ATT_ROWS(6, 2, 1)   // 3
      PIKV_ATT_ROWS(8, 2, 1)   // 4
      PIKV_ATT_ROWS(4, 4, 2)   // 1 kv head, 5-8 query heads
      PIKV_ATT_ROWS(4, 2, 2)   // 2 kv heads, 5-8 query heads each
#undef PIKV_ATT_ROWS
    } else if (a.head_dim == 128) launch_attend_mfma_slabs<SCHEME, EXCH, false>(n_slabs, nsets, grid, st, a);
    else launch_attend_mfma_slabs<SCHEME, EXCH, true>(n_slabs, nsets, grid, st, a);
  }
}

// out[c,h,d] = sum over the splits that hold tokens of cache c, in split order
__global__ __launch_bounds__(256) void attend_reduce_kernel(const float* __restrict__ partial,
                                                           const int32_t* __restrict__ fill, int n_caches,
                                                           int n_q_heads, int head_dim, int n_splits,
                                                           int tokens_per_block, float* __restrict__ out) {
  const int64_t per_cache = (int64_t)n_q_heads * head_dim;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_cache * n_caches) return;
  const int c = (int)(idx / per_cache);
  const int64_t used = ((int64_t)fill[c] + tokens_per_block - 1) / tokens_per_block;
  const int lim = used < n_splits ? (int)used : n_splits;
  float s = 0.f;
  for (int sp = 0; sp < lim; ++sp) s += partial[(int64_t)sp * per_cache * n_caches + idx];
  out[idx] = s;
}

}  // namespace pikv

using namespace pikv;

// Cached tokens per block.  Two blocks are resident per compute unit (512 on the chip): the longest
// walk that still fills the chip wins (64 caches x 32768 tokens: 4096 tokens per block, one round of
// 512 blocks, 342 us; 2048: 346 us; 1024: 361 us; 512: 380 us), a small batch is cut finer so that more
// compute units take part, and a count of blocks that would leave the last round mostly idle is avoided.
static int attend_tokens_per_block(int n_caches, int64_t max_len) {
  constexpr int64_t kResident = 512;
  int best = 256;
  double best_eff = -1.0;
  for (int tpb = kAttMaxTokensPerBlock; tpb >= 256; tpb >>= 1) {
    const int64_t blocks = (int64_t)n_caches * ((max_len + tpb - 1) / tpb);
    const int64_t rounds = (blocks + kResident - 1) / kResident;
    const double eff = rounds > 0 ? (double)blocks / (double)(rounds * kResident) : 0.0;
    if (eff >= 0.85) return tpb;
    if (eff > best_eff) {  // nothing fills the chip: the finest cut has the most blocks
      best_eff = eff;
      best = tpb;
    }
  }
  return best;
}
static int64_t attend_splits(int n_caches, int64_t max_len) {
  const int tpb = attend_tokens_per_block(n_caches, max_len);
  return (max_len + tpb - 1) / tpb;
}

extern "C" int64_t pikv_attend_workspace_bytes(int n_caches, int n_q_heads, int head_dim, int64_t max_len) {
  if (n_caches < 1 || n_q_heads < 1 || head_dim < 1 || max_len < 0) return 0;
  return attend_splits(n_caches, max_len) * n_caches * (int64_t)n_q_heads * head_dim * (int64_t)sizeof(float);
}

extern "C" int pikv_attend_values(const float* scores, const float* head_stats, int64_t score_stride,
                                  const void* v_codes, const void* v_scale, const void* v_zero,
                                  int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim,
                                  const int64_t* cache_row_base, const int32_t* cache_fill,
                                  int n_caches, int64_t max_len, float decay, float now,
                                  float* row_acc, float* row_ts, float* out, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  if (!scores || !v_codes || !v_scale || !cache_row_base || !cache_fill || !out) return PIKV_ERR_NULL;
  if (scheme < 0 || scheme > 3) return PIKV_ERR_UNSUPPORTED;
  const bool eight = (scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM);
  const bool asym = (scheme == PIKV_Q_I8_ASYM || scheme == PIKV_Q_I4_ASYM);
  const int epl = eight ? 16 : 32;
  if (asym && !v_zero) return PIKV_ERR_NULL;
  if (n_kv_heads < 1 || n_q_heads < 1 || head_dim < 1 || n_caches < 1 || n_caches > 65535 ||
      max_len < 0 || score_stride < max_len || group < 1)
    return PIKV_ERR_SHAPE;
  if (n_q_heads % n_kv_heads != 0) return PIKV_ERR_SHAPE;
  const int D = n_kv_heads * head_dim;
  if (D % group != 0) return PIKV_ERR_SHAPE;
  if (!is_pow2(head_dim) || head_dim < epl || group % epl != 0) return PIKV_ERR_UNSUPPORTED;
  const int lanes_per_row = D / epl;
  if (head_dim / epl > 256) return PIKV_ERR_UNSUPPORTED;   // one kv head must fit a block of the vector form
  hipStream_t st = (hipStream_t)stream;
  const int64_t total = (int64_t)n_caches * n_q_heads * head_dim;
  const int64_t splits = attend_splits(n_caches, max_len);
  if (splits > 65535) return PIKV_ERR_SHAPE;
  if (max_len > 0) {
    if (!workspace) return PIKV_ERR_NULL;
    if (workspace_bytes < pikv_attend_workspace_bytes(n_caches, n_q_heads, head_dim, max_len))
      return PIKV_ERR_WORKSPACE;
  }
  AttendArgs a{scores, head_stats, v_codes, v_scale, v_zero, cache_row_base, cache_fill,
               (float*)workspace, score_stride, group, n_kv_heads, n_q_heads, head_dim, n_caches,
               row_acc, row_ts, decay, now, max_len, nullptr, nullptr, 0, 0, attend_tokens_per_block(n_caches, max_len)};
  const int rep = n_q_heads / n_kv_heads;
  if (max_len > 0) {
    // the matrix-core kernels see 128-dimension slabs of the row: one kv head, or 2 / 4 narrow ones
    const int hps = mfma_heads_per_slab(head_dim, n_kv_heads);
    const int slabs = hps > 0 ? n_kv_heads / hps : 0;
    const bool slabs_ok = (slabs >= 1 && slabs <= 8) || (hps == 1 && slabs > 8 && slabs % 8 == 0 && splits * (slabs / 8) <= 0x7fffffffLL);
    if (!eight && group == 32 && slabs_ok && (rep * hps <= 8 || slabs <= 4)) {
      const dim3 grid((unsigned)splits, (unsigned)n_caches);
      if (scheme == PIKV_Q_I4_ASYM) launch_attend_mfma<PIKV_Q_I4_ASYM>(slabs, rep * hps, grid, st, a);
      else launch_attend_mfma<PIKV_Q_I4_SYM>(slabs, rep * hps, grid, st, a);
    } else if (eight && slabs >= 1 && slabs <= 8 && group % head_dim == 0 && rep * hps >= 2 &&
               (rep * hps <= 8 || (hps == 1 && (n_q_heads <= 64 || slabs <= 4)))) {
      const dim3 grid((unsigned)splits, (unsigned)n_caches);
      if (scheme == PIKV_Q_I8_SYM) launch_attend_mfma8<PIKV_Q_I8_SYM>(slabs, hps, grid, st, a);
      else launch_attend_mfma8<PIKV_Q_I8_ASYM>(slabs, hps, grid, st, a);
    } else {
      if (row_acc || row_ts)
        hipLaunchKernelGGL(attend_importance_kernel, dim3((unsigned)((max_len + 255) / 256), (unsigned)n_caches),
                           dim3(256), 0, st, a);
      // heads of a kv group per pass: the float accumulators of one lane must fit
      const int rp = eight ? (rep >= 8 ? 8 : rep >= 4 ? 4 : rep >= 2 ? 2 : 1) : (rep >= 2 ? 2 : 1);
      // rows of more than 256 lanes: windows of kv heads, preferably of a lane count that divides the block
      int n_win = 1;
      if (lanes_per_row > 256) {
        const int lph = head_dim / epl;
        int wk = 0;
        for (int w = n_kv_heads; w >= 1; --w)
          if (n_kv_heads % w == 0 && w * lph <= 256 && (wk == 0 || (256 % (w * lph) == 0 && 256 % (wk * lph) != 0))) wk = w;
        a.kv_window = wk;
        n_win = n_kv_heads / wk;
      }
      if ((int64_t)((rep + rp - 1) / rp) * n_win > 65535) return PIKV_ERR_SHAPE;
      const dim3 grid((unsigned)splits, (unsigned)n_caches, (unsigned)((rep + rp - 1) / rp * n_win));
#define PIKV_ATTEND_CASE(S)                                                                        \
  case S:                                                                                          \
    if (rp == 8) hipLaunchKernelGGL((attend_valu_kernel<S, 8>), grid, dim3(256), 0, st, a);        \
    else if (rp == 4) hipLaunchKernelGGL((attend_valu_kernel<S, 4>), grid, dim3(256), 0, st, a);   \
    else if (rp == 2) hipLaunchKernelGGL((attend_valu_kernel<S, 2>), grid, dim3(256), 0, st, a);   \
    else hipLaunchKernelGGL((attend_valu_kernel<S, 1>), grid, dim3(256), 0, st, a);                \
    break;
      switch (scheme) {
        PIKV_ATTEND_CASE(PIKV_Q_I8_SYM)
        PIKV_ATTEND_CASE(PIKV_Q_I8_ASYM)
        case PIKV_Q_I4_ASYM:
          if (rp == 2) hipLaunchKernelGGL((attend_valu_kernel<PIKV_Q_I4_ASYM, 2>), grid, dim3(256), 0, st, a);
          else hipLaunchKernelGGL((attend_valu_kernel<PIKV_Q_I4_ASYM, 1>), grid, dim3(256), 0, st, a);
          break;
        case PIKV_Q_I4_SYM:
          if (rp == 2) hipLaunchKernelGGL((attend_valu_kernel<PIKV_Q_I4_SYM, 2>), grid, dim3(256), 0, st, a);
          else hipLaunchKernelGGL((attend_valu_kernel<PIKV_Q_I4_SYM, 1>), grid, dim3(256), 0, st, a);
          break;
      }
#undef PIKV_ATTEND_CASE
    }
  }
  hipLaunchKernelGGL(attend_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     (const float*)workspace, cache_fill, n_caches, n_q_heads, head_dim, (int)splits,
                     a.tokens_per_block, out);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

// ---- one call for the decode read: scores, softmax, attention output, H2O bookkeeping ----
static int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

struct DecodeWs {
  int64_t n_tiles, stride, scores, tmax, tsum, stats, partial, total;
};
static DecodeWs decode_ws(int n_caches, int n_q_heads, int head_dim, int64_t max_len) {
  DecodeWs w;
  w.n_tiles = (max_len + PIKV_SCORE_TILE - 1) / PIKV_SCORE_TILE;
  w.stride = w.n_tiles * PIKV_SCORE_TILE;
  w.scores = 0;  // float scores [cache][head][stride], or the exchange rows [cache][tile][head][64] (same size)
  // (the two tile tables have room for one tile more than max_len holds: the one-pass form keeps a spare
  // record per cache there, and its ranges' statistics - 8 bytes per head and range of at least 128 tokens -
  // fit the second table)
  w.tmax = align256((int64_t)n_caches * n_q_heads * w.stride * 4);
  w.tsum = w.tmax + align256((int64_t)n_caches * (w.n_tiles + 1) * n_q_heads * 4);
  w.stats = w.tsum + align256((int64_t)n_caches * (w.n_tiles + 1) * n_q_heads * 4);
  w.partial = w.stats + align256((int64_t)n_caches * n_q_heads * 2 * 4);
  w.total = w.partial + align256(pikv_attend_workspace_bytes(n_caches, n_q_heads, head_dim, max_len));
  return w;
}

extern "C" int64_t pikv_decode_attend_workspace_bytes(int n_caches, int n_q_heads, int head_dim, int64_t max_len) {
  if (n_caches < 1 || n_q_heads < 1 || head_dim < 1 || max_len < 0) return 0;
  return decode_ws(n_caches, n_q_heads, head_dim, max_len).total;
}

extern "C" int pikv_decode_attend(const void* k_codes, const void* k_scale, const void* k_zero,
                                  const void* v_codes, const void* v_scale, const void* v_zero,
                                  int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim,
                                  const void* q, int q_dtype, float scale_qk,
                                  const int64_t* cache_row_base, const int32_t* cache_fill, int n_caches,
                                  int64_t max_len, float decay, float now, float* row_acc, float* row_ts,
                                  float* out, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!k_codes || !k_scale || !v_codes || !v_scale || !q || !cache_row_base || !cache_fill || !out)
    return PIKV_ERR_NULL;
  if (scheme < 0 || scheme > 3) return PIKV_ERR_UNSUPPORTED;
  if (n_caches < 1 || n_q_heads < 1 || n_kv_heads < 1 || head_dim < 1 || max_len < 0) return PIKV_ERR_SHAPE;
  const DecodeWs w = decode_ws(n_caches, n_q_heads, head_dim, max_len);
  if (max_len > 0) {
    if (!workspace) return PIKV_ERR_NULL;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return PIKV_ERR_SHAPE;
    if (workspace_bytes < w.total) return PIKV_ERR_WORKSPACE;
  }
  char* ws = reinterpret_cast<char*>(workspace);
  float* tmax = reinterpret_cast<float*>(ws + w.tmax);
  float* tsum = reinterpret_cast<float*>(ws + w.tsum);
  float* stats = reinterpret_cast<float*>(ws + w.stats);
  void* partial = ws + w.partial;
  const int64_t partial_bytes = w.total - w.partial;
  hipStream_t st = (hipStream_t)stream;
  if (max_len == 0)  // nothing cached anywhere: the output is zero (the reduction writes it)
    return pikv_attend_values(reinterpret_cast<const float*>(out), nullptr, 0, v_codes, v_scale, v_zero, scheme, group,
                              n_kv_heads, n_q_heads, head_dim, cache_row_base, cache_fill, n_caches, 0, decay, now,
                              row_acc, row_ts, out, nullptr, 0, stream);
  const bool asym = scheme == PIKV_Q_I4_ASYM;
  const bool any_asym = asym || scheme == PIKV_Q_I8_ASYM;
  // one pass over K and V (no score matrix): heads of 128, bf16 queries; 4-bit codes with up to 4 query heads per
  // kv head, 8-bit codes (scale per kv head or coarser) with up to 8.
  // Its halves (n_q_heads * 128 bytes per tile and one spare tile per cache) lie where the float scores would
  // (256 bytes per head and tile), the tiles' reference maxima in the tile-maximum table, the ranges' statistics
  // in the tile-sum table.
  if (decode_fused_serves(scheme, group, n_kv_heads, n_q_heads, head_dim, q_dtype, row_acc != nullptr) && (!any_asym || (k_zero && v_zero)) &&
      n_caches <= 65535) {
    const int tpb = fused_tokens_per_block(n_caches, n_kv_heads, max_len, attend_tokens_per_block(n_caches, max_len));
    return decode_fused_launch(k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, scheme, group, n_kv_heads, n_q_heads, q,
                               q_dtype, scale_qk, cache_row_base, cache_fill, n_caches, max_len, tpb, decay, now, row_acc, row_ts,
                               out, ws + w.scores, tmax, tsum, reinterpret_cast<float*>(partial), stats, st);
  }
  // the 4-bit matrix-core kernels meeting in the exchange format
  const int rep = n_q_heads % n_kv_heads == 0 ? n_q_heads / n_kv_heads : 0;
  const int hps = mfma_heads_per_slab(head_dim, n_kv_heads);   // 128-dimension slabs: one kv head, or 2 / 4 narrow ones
  const int slabs = hps > 0 ? n_kv_heads / hps : 0;
  const bool hk_ok = (slabs >= 1 && slabs <= 8) || (hps == 1 && slabs > 8 && slabs % 8 == 0);
  const int64_t splits = attend_splits(n_caches, max_len);
  if ((scheme == PIKV_Q_I4_ASYM || scheme == PIKV_Q_I4_SYM) && group == 32 && rep >= 1 &&
      (rep * hps <= 8 || slabs <= 4) && hk_ok && (q_dtype == PIKV_BF16 || q_dtype == PIKV_F32) && n_caches <= 65535 && splits <= 65535 && (!asym || (k_zero && v_zero))) {
    float* esc = reinterpret_cast<float*>(ws + w.scores);
    const int rc = scores_exchange_launch(k_codes, k_scale, k_zero, scheme, group, n_kv_heads, n_q_heads, head_dim, q,
                                          q_dtype, scale_qk, cache_row_base, cache_fill, n_caches, max_len, esc, tmax,
                                          tsum, stats, st);
    if (rc == PIKV_OK) {
      AttendArgs a{nullptr, stats, v_codes, v_scale, v_zero, cache_row_base, cache_fill,
                   (float*)partial, 0, group, n_kv_heads, n_q_heads, head_dim, n_caches,
                   row_acc, row_ts, decay, now, max_len, esc, tmax, w.n_tiles, 0, attend_tokens_per_block(n_caches, max_len)};
      const dim3 grid((unsigned)splits, (unsigned)n_caches);
      if (asym) launch_attend_mfma<PIKV_Q_I4_ASYM, true>(slabs, rep * hps, grid, st, a);
      else launch_attend_mfma<PIKV_Q_I4_SYM, true>(slabs, rep * hps, grid, st, a);
      const int64_t total = (int64_t)n_caches * n_q_heads * head_dim;
      hipLaunchKernelGGL(attend_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                         (const float*)partial, cache_fill, n_caches, n_q_heads, head_dim, (int)splits,
                         a.tokens_per_block, out);
      PIKV_CHECK_LAUNCH();
      return PIKV_OK;
    }
    if (rc != PIKV_ERR_UNSUPPORTED) return rc;
  }
  // every other cache format: the three public steps, with float scores in the workspace
  float* scores = reinterpret_cast<float*>(ws + w.scores);
  int rc = pikv_gather_dequant_scores(k_codes, k_scale, k_zero, scheme, group, n_kv_heads, n_q_heads, head_dim, q,
                                      q_dtype, scale_qk, cache_row_base, cache_fill, n_caches, max_len, w.stride,
                                      scores, tmax, tsum, stream);
  if (rc != PIKV_OK) return rc;
  rc = pikv_h2o_accumulate(scores, tmax, tsum, n_q_heads, cache_row_base, cache_fill, n_caches, max_len, w.stride,
                           1.0f, now, 0, nullptr, nullptr, nullptr, stats, stream);
  if (rc != PIKV_OK) return rc;
  return pikv_attend_values(scores, stats, w.stride, v_codes, v_scale, v_zero, scheme, group, n_kv_heads, n_q_heads,
                            head_dim, cache_row_base, cache_fill, n_caches, max_len, decay, now, row_acc, row_ts, out,
                            partial, partial_bytes, stream);
}
