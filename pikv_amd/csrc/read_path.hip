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
  // A lane holds EPL consecutive output elements, a wavefront 64 * EPL of them, contiguous in `out`
  // (whatever rows were gathered).  Stored from the lanes' registers, every store instruction would
  // write 16 bytes per lane at a stride of the lane's whole run; the values cross LDS instead, so
  // that each instruction writes one contiguous kilobyte (32768 x 4096 8-bit codes to float32:
  // 171 -> 119 us, the rate of a plain write stream).  A wavefront that is not full (the tail of the last row) stores directly.
  constexpr int OB = OUT_DT == PIKV_F32 ? 4 : 2;      // bytes per output element
  constexpr int NC = EPL * OB / 16;                   // 16-byte chunks per lane
  constexpr int LSTRIDE = EPL * OB + 16;              // bytes per lane in LDS (+16: bank spread)
  __shared__ __attribute__((aligned(16))) char xpose[4][64 * LSTRIDE];
  uint4 chunk[NC];
  if constexpr (OUT_DT == PIKV_F32) {
#pragma unroll
    for (int j = 0; j < NC; ++j)
      chunk[j] = make_uint4(__float_as_uint(f[4 * j]), __float_as_uint(f[4 * j + 1]), __float_as_uint(f[4 * j + 2]),
                            __float_as_uint(f[4 * j + 3]));
  } else {
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      uint32_t w[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        w[q] = float_to_bf16_bits(f[8 * j + 2 * q]) | (float_to_bf16_bits(f[8 * j + 2 * q + 1]) << 16);
      chunk[j] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t g0 = g - lane;                        // first lane of this wavefront
  const bool full = (g0 + 63) / lanes_per_row < n;    // uniform: every lane of the wavefront has a row
  if (full) {
    char* mine = xpose[wave] + lane * LSTRIDE;
#pragma unroll
    for (int j = 0; j < NC; ++j) *reinterpret_cast<uint4*>(mine + 16 * j) = chunk[j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    char* o = reinterpret_cast<char*>(out) + g0 * (EPL * OB);
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int e = k * 64 + lane;                    // 16-byte chunk of the wavefront's run
      const uint4 v16 = *reinterpret_cast<const uint4*>(xpose[wave] + (e / NC) * LSTRIDE + (e % NC) * 16);
      st16(o + (int64_t)e * 16, v16);
    }
  } else {
    char* o = reinterpret_cast<char*>(out) + (i * D + (int64_t)part * EPL) * OB;
#pragma unroll
    for (int j = 0; j < NC; ++j) st16(o + 16 * j, chunk[j]);
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
  float* escores;    // when set (4-bit GQA kernel only), written INSTEAD of scores: [cache][tile][q head][64] floats,
                     // exp(score - tile max) of every token - the exchange format of pikv_decode_attend
  int max_len;      // rows of a cache beyond max_len are not read (a cache may hold more than the caller covers)
  int rep;          // scores_kernel: query heads per kv head, and the first head of every kv group that
  int head_off;     //   this launch serves (it serves REP of them; other ratios take several launches)
  int head_split;   // scores_kernel: head_split blocks share a tile, each owns n_kv_heads/head_split heads
  int row_slabs;    // scores_mfma_i4_gqa_kernel<SPLIT>: 128-dimension slabs of a whole cached row (n_kv_heads of them per block)
};

template <int SCHEME, int REP, int Q_DT>
__global__ __launch_bounds__(256) void scores_kernel(ScoreArgs a) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  extern __shared__ float stage[];  // [q head of this block][token in tile]

  // blockIdx.x = tile * head_split + piece: the blocks that share a tile's rows are dispatched side
  // by side, so that whole rows are in flight at any time and not the same 512-byte piece of every
  // 4 KB row (which lands on a fraction of the memory channels)
  // ... and, inside a run of 8 tiles, block r serves piece r / 8 of tile r % 8: consecutive block
  // indices go round the 8 XCDs, so the pieces of one tile meet in one L2 and the scale rows and
  // queries they share are fetched from memory once, not once per piece.  (Any dispatch order gives
  // the same results; a ragged last run keeps the plain order.)
  const int c = blockIdx.y;
  const unsigned run = 8u * (unsigned)a.head_split;
  const unsigned run0 = blockIdx.x / run * run;
  int64_t tile;
  int piece;
  if (run0 + run <= gridDim.x) {
    const unsigned r = blockIdx.x - run0;
    tile = (int64_t)(run0 / (unsigned)a.head_split) + (r & 7u);
    piece = (int)(r >> 3);
  } else {
    tile = blockIdx.x / a.head_split;
    piece = blockIdx.x - (int)tile * a.head_split;
  }
  const int64_t base_row = a.row_base[c];  // asked for together with the fill: one round trip, not two
  const int len = a.fill[c] < a.max_len ? a.fill[c] : a.max_len;
  const int64_t n0 = tile * kTile;
  if (n0 >= len) return;  // uniform for the block
  // A block owns the kv heads [kv0, kv0 + kv_blk) of its tile: wide rows are split
  // over several blocks so that while one block reduces its tile, others still load.
  const int kv_blk = a.n_kv_heads / a.head_split;
  const int kv0 = piece * kv_blk;
  const int D = a.n_kv_heads * a.head_dim;
  const int lanes_per_row = D / EPL;                         // lanes of a whole cached row
  const int lanes_per_head = a.head_dim / EPL;               // power of two
  const int lanes_blk = kv_blk * lanes_per_head;             // <= 256, divides 256
  const int groups_per_row = D / a.group;
  const int tok_per_step = 256 / lanes_blk;
  const int part_blk = threadIdx.x % lanes_blk;
  const int part = kv0 * lanes_per_head + part_blk;          // fixed (kv head, slice) of this lane
  const int tok_in_step = threadIdx.x / lanes_blk;
  const int kvl = part_blk / lanes_per_head;                 // kv head inside the block
  const int kvh = kv0 + kvl;
  const int d0 = (part % lanes_per_head) * EPL;

  constexpr int UN = 4;  // token steps per batch of loads
  const int batch = tok_per_step * UN;  // tokens of the tile covered by one batch

  // Two register sets: the loads of the next batch are in flight while the current one is
  // multiplied.  Loads are issued unconditionally from clamped rows (a token past the end of
  // the cache or of the tile re-reads the last valid one and is masked when its score is
  // staged): loads under conditions would make the wait before the arithmetic cover the
  // prefetch as well.
  struct Batch {
    uint4 v[UN];
    float sc[UN], zr[UN];
  };
  const char* const code_base = reinterpret_cast<const char*>(a.codes) + ((base_row + n0) * lanes_per_row + part) * 16;
  const int64_t meta_base = (base_row + n0) * groups_per_row + (part * EPL) / a.group;
  const int last_tl = (len - n0 < kTile ? (int)(len - n0) : kTile) - 1;   // last token of the tile that exists
  auto load_batch = [&](int s0, Batch& t) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      int tl = s0 + u * tok_per_step + tok_in_step;
      tl = tl < last_tl ? tl : last_tl;
      t.v[u] = ld16(code_base + (int64_t)tl * lanes_per_row * 16);
      const int64_t mi = meta_base + (int64_t)tl * groups_per_row;
      t.sc[u] = load_meta<SCHEME>(a.scale, mi);
      if constexpr (!Q::sym) t.zr[u] = load_meta<SCHEME>(a.zero, mi);
      else t.zr[u] = 0.f;
    }
  };
  // The first batch goes out before the queries are fetched: the block's first rows and its
  // query slices then share one memory round trip.
  Batch ba, bb;
  load_batch(0, ba);

  // Query slices of the REP heads that read this kv head, and their sums (for the
  // zero-point term: dot(q, (c - z) * s) = s * (dot(q, c) - z * sum(q))).
  float qv[REP][EPL];
  float qsum[REP];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    const int hq = kvh * a.rep + a.head_off + r;
    load_as_float<Q_DT, EPL>(a.q, ((int64_t)c * a.n_q_heads + hq) * a.head_dim + d0, qv[r]);
    float sacc = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) sacc += qv[r][j];
    qsum[r] = sacc;
  }

  auto mul_batch = [&](int s0, const Batch& t) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int tl = s0 + u * tok_per_step + tok_in_step;
      const bool ok = tl < kTile && n0 + tl < len;
      float cf[EPL];
      unpack_codes_unsigned<SCHEME>(t.v[u], cf);
      const float zu = t.zr[u] - (float)Q::qmin;  // zero point of the unsigned stored form
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) d = fmaf(qv[r][j], cf[j], d);
        d = (d - zu * qsum[r]) * t.sc[u];
        d = group_sum_dpp(d, lanes_per_head);
        if ((part % lanes_per_head) == 0 && tl < kTile)
          stage[(kvl * REP + r) * kTile + tl] = ok ? d * a.scale_qk : -__builtin_inff();
      }
    }
  };
  for (int s0 = 0; s0 < kTile; s0 += 2 * batch) {
    if (s0 + batch < kTile) load_batch(s0 + batch, bb);
    mul_batch(s0, ba);
    if (s0 + batch >= kTile) break;
    if (s0 + 2 * batch < kTile) load_batch(s0 + 2 * batch, ba);
    mul_batch(s0 + batch, bb);
  }
  __syncthreads();

  // One wavefront per query head: write the 64 scores as one 256-byte row and
  // reduce the tile's softmax statistics.
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int hq_blk = kv_blk * REP;
  for (int hl = wave; hl < hq_blk; hl += 4) {
    const int hq = (kv0 + hl / REP) * a.rep + a.head_off + hl % REP;
    const float s = stage[hl * kTile + lane];
    const bool ok = n0 + lane < len;
    if (ok) a.scores[((int64_t)c * a.n_q_heads + hq) * a.score_stride + n0 + lane] = s;
    const float m = group_max_dpp(ok ? s : -__builtin_inff(), 64);
    const float e = ok ? __builtin_amdgcn_exp2f((s - m) * 1.4426950408889634f) : 0.f;
    const float sum = group_sum_dpp(e, 64);
    if (lane == 0) {
      const int64_t ti = ((int64_t)c * a.n_tiles + tile) * a.n_q_heads + hq;  // heads of a tile side by side
      a.tile_max[ti] = m;
      a.tile_sum[ti] = sum;
    }
  }
}

// ---- 4-bit scores on the matrix cores ------------------------------------------------
// The VALU kernel above is instruction-bound for grouped 4-bit caches read by
// several query heads per kv head (decode, GQA): 4 heads x 128 dims per cached
// token-head against a budget of ~4 instructions per element at the HBM rate
// (measured: 1.18 ms where HBM allows 0.24 ms).  Here the contraction over a
// 32-element quantisation group is one v_mfma_f32_16x16x32_bf16:
//   A (16 x 32) = the query heads of one kv head (rows >= rep are zero),
//   B (32 x 16) = the codes of one group for 16 cached tokens, expanded to bf16
//                 as 0x4300|u = 128 + u (exact), u = unsigned stored code,
//   C           = 128*Qs + sum q*u per (head, token); the group scale and zero
//                 point are applied in the epilogue:
//                 s * (C - (z + bias) * Qs),  Qs = sum of q over the group.
// Loads stay 16 bytes per lane and contiguous: lane (token n, j) fetches group j
// of its token, and a 4x4 transpose across the four 16-lane rows
// (v_permlane16_swap / v_permlane32_swap) hands lane (n, kg) the k-slice kg of
// every group, which is the operand layout the MFMA wants.
typedef __bf16 pikv_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pikv_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void transpose4x4_rows(uint32_t (&v)[4]) {
  auto a = __builtin_amdgcn_permlane16_swap(v[0], v[1], false, false);
  auto b = __builtin_amdgcn_permlane16_swap(v[2], v[3], false, false);
  auto c = __builtin_amdgcn_permlane32_swap(a[0], b[0], false, false);
  auto d = __builtin_amdgcn_permlane32_swap(a[1], b[1], false, false);
  v[0] = c[0]; v[2] = c[1]; v[1] = d[0]; v[3] = d[1];
}

template <int SCHEME>
__global__ __launch_bounds__(256) void scores_mfma_i4_kernel(ScoreArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 4, "4-bit schemes only");
  extern __shared__ float mfma_lds[];
  float* stage = mfma_lds;                      // [q head][token in tile]
  float* qs = mfma_lds + a.n_q_heads * kTile;   // sum of q over each 32-wide group

  const int c = blockIdx.y;
  const int64_t tile = blockIdx.x;
  const int len = a.fill[c] < a.max_len ? a.fill[c] : a.max_len;
  const int64_t n0 = tile * kTile;
  if (n0 >= len) return;  // uniform for the block
  const int rep = a.n_q_heads / a.n_kv_heads;
  const int lanes_per_row = a.n_kv_heads * 4;   // 16-byte groups per cached row
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nl = lane & 15;   // token column / query-head row
  const int rg = lane >> 4;   // group fetched by this lane; k-slice after the transpose
  const uint16_t* qbase = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)c * a.n_q_heads * 128;

  // Group sums of the query (float32), one (head, group) pair per thread.
  for (int i = threadIdx.x; i < a.n_q_heads * 4; i += 256) {
    const uint16_t* qp = qbase + (int64_t)(i >> 2) * 128 + (i & 3) * 32;
    float sacc = 0.f;
    for (int k = 0; k < 32; ++k) sacc += bf16_bits_to_float(qp[k]);
    qs[i] = sacc;
  }
  __syncthreads();

  const float zbias = 128.0f - (float)Q::qmin;  // 128 (asymmetric) or 136 (symmetric)
  const int64_t base_row = a.row_base[c];
  // two nibbles -> two bf16 values 128 + code; both constants held in vector registers so that the
  // three-operand and-or instruction can be encoded (the empty statement emits no instruction)
  uint32_t kNib = 0x000f000fu, kExp = 0x43004300u;
  asm volatile("" : "+v"(kNib), "+v"(kExp));

  for (int g = wave; g < a.n_kv_heads; g += 4) {
    // A operands of this kv head: lane (row m = nl, k-slice rg) of group gq holds
    // q[g*rep + m][32*gq + 8*rg + {0,4,1,5,2,6,3,7}] - the element order in which
    // the codes come out of the nibble expansion below.
    pikv_bf16x8 amat[4];
    float qsum[4][4];  // [gq][i] for C rows 4*rg + i
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      uint4 d = make_uint4(0, 0, 0, 0);
      if (nl < rep) d = ld16(qbase + (int64_t)(g * rep + nl) * 128 + gq * 32 + rg * 8);
      const uint4 p = make_uint4((d.x & 0xffffu) | (d.z << 16), (d.x >> 16) | (d.z & 0xffff0000u),
                                 (d.y & 0xffffu) | (d.w << 16), (d.y >> 16) | (d.w & 0xffff0000u));
      amat[gq] = __builtin_bit_cast(pikv_bf16x8, p);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * rg + i;
        qsum[gq][i] = (r < rep) ? qs[(g * rep + r) * 4 + gq] : 0.f;
      }
    }
    // All four 16-token slices of the tile are fetched before any of them is used:
    // four 16-byte loads (plus metadata) in flight per lane.
    constexpr int NTG = kTile / 16;
    uint32_t v[NTG][4], meta1[NTG];
    bool ok[NTG];
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
      const int64_t n = n0 + tg * 16 + nl;
      ok[tg] = n < len;
      v[tg][0] = v[tg][1] = v[tg][2] = v[tg][3] = 0;
      meta1[tg] = 0;
      if (ok[tg]) {
        const int64_t gi = (base_row + n) * lanes_per_row + g * 4 + rg;
        const uint4 cv = ld16(reinterpret_cast<const char*>(a.codes) + gi * 16);
        v[tg][0] = cv.x; v[tg][1] = cv.y; v[tg][2] = cv.z; v[tg][3] = cv.w;
        uint32_t m = reinterpret_cast<const uint16_t*>(a.scale)[gi];
        if constexpr (!Q::sym) m |= (uint32_t) reinterpret_cast<const uint16_t*>(a.zero)[gi] << 16;
        meta1[tg] = m;
      }
    }
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
      const int tl = tg * 16 + nl;
      uint32_t meta[4] = {meta1[tg], meta1[tg], meta1[tg], meta1[tg]};
      transpose4x4_rows(v[tg]);  // v[gq] = k-slice rg of group gq of token nl
      transpose4x4_rows(meta);   // meta[gq] = (scale, zero) of group gq of token nl
      pikv_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const uint32_t w = Q::sym ? (v[tg][gq] ^ 0x88888888u) : v[tg][gq];
        const uint4 b = make_uint4(and_or(w, kNib, kExp), and_or(w >> 4, kNib, kExp), and_or(w >> 8, kNib, kExp),
                                   and_or(w >> 12, kNib, kExp));
        const pikv_f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
        const pikv_f32x4 pc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            amat[gq], __builtin_bit_cast(pikv_bf16x8, b), zero4, 0, 0, 0);
        const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)(meta[gq] & 0xffffu));
        const _Float16 zh = __builtin_bit_cast(_Float16, (uint16_t)(meta[gq] >> 16));
        const float sc = (float)sh;
        const float zq = (Q::sym ? 0.f : (float)zh) + zbias;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(sc, fmaf(-zq, qsum[gq][i], pc[i]), acc[i]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 4 * rg + i;
        if (r < rep) stage[(g * rep + r) * kTile + tl] = ok[tg] ? acc[i] * a.scale_qk : -__builtin_inff();
      }
    }
  }
  __syncthreads();

  for (int hq = wave; hq < a.n_q_heads; hq += 4) {
    const float sv = stage[hq * kTile + lane];
    const bool ok = n0 + lane < len;
    if (ok) a.scores[((int64_t)c * a.n_q_heads + hq) * a.score_stride + n0 + lane] = sv;
    const float m = group_max<64>(ok ? sv : -__builtin_inff());
    const float e = ok ? expf(sv - m) : 0.f;
    const float sum = group_sum<64>(e);
    if (lane == 0) {
      const int64_t ti = ((int64_t)c * a.n_tiles + tile) * a.n_q_heads + hq;  // heads of a tile side by side
      a.tile_max[ti] = m;
      a.tile_sum[ti] = sum;
    }
  }
}

// Variant for at most 4 query heads per kv head (the usual GQA ratios), where the
// layout above leaves 12 of the 16 tile rows empty.  Here the 16 rows are
// (group gq, head r) and the A operand is block-diagonal in the k-slices: the
// k-slice kg of MFMA #b multiplies q[r][32*gq + 8*b ..] only in rows with gq == kg.
// Four MFMAs accumulate into one tile that holds, in row-group rg, the partial dot
// products of group rg for the lane's own token - so every lane uses the codes and
// the (scale, zero) it loaded itself: no transpose, one epilogue per 16 tokens
// instead of one per MFMA, and a 3-swap transpose-reduction over the four
// row-groups leaves row-group r with the finished score of head r.

// Tile statistics and score rows from the staged scores [q head][token in tile], four
// heads per wavefront pass: lane (rg, nl) owns tokens nl, nl+16, nl+32, nl+48 of head
// h4 + rg; the 16 lanes of a row reduce with DPP.
// GROUPED: the staged rows are [kv head][SLOTS] (row SLOTS g + r = head g * rep + r, rows
// r >= rep unused), so that the row of a kv head sits at a compile-time offset for the writers.
template <bool GROUPED, int SLOTS = 4>
__device__ __forceinline__ void tile_stats_store(const ScoreArgs& a, const float* stage, int c, int64_t tile,
                                                 int64_t n0, int len, int wave, int rg, int nl, int rep = 4,
                                                 int hq0 = 0,    // hq0: first query head of the block's kv heads
                                                 int rep_all = 0) {  // query heads per kv head when the launch serves only rep of them
  const int slots = SLOTS > 0 ? SLOTS : rep;                   // SLOTS = 0: compact rows, rep per kv head
  const int n_pass_rows = GROUPED ? a.n_kv_heads * slots : a.n_q_heads;
  for (int h4 = wave * 4; h4 < n_pass_rows; h4 += 16) {
    const int srow = h4 + rg;                                  // staged row = kv head * slots + slot
    const int slot = srow % slots;
    const int hq = hq0 + (GROUPED ? (srow / slots) * (rep_all ? rep_all : rep) + slot : srow);  // query head
    const bool hok = GROUPED ? (slot < rep && srow < n_pass_rows) : hq < a.n_q_heads;
    float x[4];
    bool okk[4];
    float m = -__builtin_inff();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      okk[k] = hok && (n0 + nl + 16 * k < len);
      x[k] = okk[k] ? stage[srow * kTile + nl + 16 * k] : -__builtin_inff();
      m = fmaxf(m, x[k]);
    }
    m = dpp_max<kDppXor1>(m);
    m = dpp_max<kDppXor2>(m);
    m = dpp_max<kDppHalfMirror>(m);
    m = dpp_max<kDppMirror>(m);
    float sum = 0.f;
    float* out = a.scores + ((int64_t)c * a.n_q_heads + (hok ? hq : 0)) * a.score_stride + n0 + nl;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (okk[k]) {
        sum += __builtin_amdgcn_exp2f((x[k] - m) * 1.4426950408889634f);
        out[16 * k] = x[k];
      }
    }
    sum = dpp_add<kDppXor1>(sum);
    sum = dpp_add<kDppXor2>(sum);
    sum = dpp_add<kDppHalfMirror>(sum);
    sum = dpp_add<kDppMirror>(sum);
    if (nl == 0 && hok) {
      const int64_t ti = ((int64_t)c * a.n_tiles + tile) * a.n_q_heads + hq;  // heads of a tile side by side
      a.tile_max[ti] = m;
      a.tile_sum[ti] = sum;
    }
  }
}

// The same for the exchange format of pikv_decode_attend (a.escores set): lane (rg, nl) owns the
// four consecutive tokens 4 nl .. 4 nl + 3 of head h4 + rg and stores exp(score - tile max) of
// them as one 16-byte vector into [cache][tile][q head][64]; the heads of a tile lie side by
// side, so a block's output is one contiguous run.  (For the public [head][token] score rows the
// same 16-byte stores were measured and changed nothing; they keep the token-strided map.)
// GROUPED: the staged rows are [kv head][SLOTS] (row SLOTS g + r = head g * rep + r, rows
// r >= rep unused), so that the row of a kv head sits at a compile-time offset for the writers.
template <bool GROUPED, int SLOTS = 4>
__device__ __forceinline__ void tile_stats_exchange(const ScoreArgs& a, const float* stage, int c, int64_t tile,
                                                 int64_t n0, int len, int wave, int rg, int nl, int rep = 4,
                                                 int hq0 = 0,    // hq0: first query head of the block's kv heads
                                                 int rep_all = 0) {  // query heads per kv head when the launch serves only rep of them
  const int n_pass_rows = GROUPED ? a.n_kv_heads * SLOTS : a.n_q_heads;
  const int left = len - (int)n0 - 4 * nl;                     // tokens of this lane's run that exist
  for (int h4 = wave * 4; h4 < n_pass_rows; h4 += 16) {
    const int srow = h4 + rg;                                  // staged row = kv head * SLOTS + slot
    const int slot = srow % SLOTS;
    const int hq = hq0 + (GROUPED ? (srow / SLOTS) * (rep_all ? rep_all : rep) + slot : srow);  // query head
    const bool hok = GROUPED ? slot < rep : hq < a.n_q_heads;
    const float4 sv = hok ? *reinterpret_cast<const float4*>(stage + srow * kTile + 4 * nl)
                          : make_float4(0.f, 0.f, 0.f, 0.f);
    const float ninf = -__builtin_inff();
    float x[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) x[k] = (hok && k < left) ? x[k] : ninf;
    float m = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
    m = dpp_max<kDppXor1>(m);
    m = dpp_max<kDppXor2>(m);
    m = dpp_max<kDppHalfMirror>(m);
    m = dpp_max<kDppMirror>(m);
    float e[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)   // exp2(-inf) = 0 for the tokens that do not exist
      e[k] = (m > ninf) ? __builtin_amdgcn_exp2f((x[k] - m) * 1.4426950408889634f) : 0.f;  // (a row without tokens: -inf - -inf)
    if (hok)   // whole tiles: tokens that do not exist are stored as zeros
      *reinterpret_cast<float4*>(a.escores + (((int64_t)c * a.n_tiles + tile) * a.n_q_heads + hq) * kTile + 4 * nl) =
          make_float4(e[0], e[1], e[2], e[3]);
    float sum = (e[0] + e[1]) + (e[2] + e[3]);
    sum = dpp_add<kDppXor1>(sum);
    sum = dpp_add<kDppXor2>(sum);
    sum = dpp_add<kDppHalfMirror>(sum);
    sum = dpp_add<kDppMirror>(sum);
    if (nl == 0 && hok) {
      const int64_t ti = ((int64_t)c * a.n_tiles + tile) * a.n_q_heads + hq;  // heads of a tile side by side
      a.tile_max[ti] = m;
      a.tile_sum[ti] = sum;
    }
  }
}

constexpr int kGqaTilesPerBlock = 2;   // consecutive 64-token tiles handled by one block (4: 1.6 % slower in the one-call decode read; 8 and 16 as 4)
constexpr int kGqaMaxKvHeads = 16;     // code vectors of one 16-token slice kept in registers

// LDS bytes of scores_mfma_i4_gqa_kernel: score staging, query sums, compact A
// operands plus an all-zero twin, and the (scale, zero) rows of one tile.
// (na = copies of the A operands: one per set, or the two limbs of float32 queries)
static size_t gqa_lds_bytes(int n_kv_heads, int nset, int na) {
  return (size_t)nset * n_kv_heads * 4 * kTile * sizeof(float) + (size_t)nset * n_kv_heads * 16 * sizeof(float) +
         (size_t)(na + 1) * n_kv_heads * 4 * 16 * 16 + 2 * (size_t)kTile * (n_kv_heads * 4 + 2) * sizeof(uint16_t);
}

// A wavefront owns one 16-token slice of the tile and walks over ALL kv heads, so
// its loads cover 16 whole cached rows (n_kv_heads * 64 contiguous bytes each),
// issued back to back - HBM sees complete rows instead of 64-byte pieces that are
// revisited later.  The next tile's rows are prefetched while the current ones are
// multiplied (two register sets, used alternately).
// NSET sets of four query heads per kv head (1: up to 4 heads, 2: up to 8): the unpacked codes
// of a kv head are multiplied with one block-diagonal A operand per set.
// NARROW: heads of 64 or 32 dimensions (below); the kernel for heads of 128 carries none of it.
// QF32: float32 queries.  A query element goes in as two bf16 limbs, q = hi + lo + (at most
// 2^-18 |q|), hi = the float rounded to bf16, lo = the rest rounded to bf16: two copies of a
// set's A operands, one per limb, are multiplied with the same unpacked codes into the same
// accumulators, and the group sums of q are those of hi + lo.
// SPLIT (rows of more than 16 slabs, e.g. 32 kv heads of 128): a block takes a group of a.n_kv_heads slabs
// out of the a.row_slabs of a cached row; the groups of a tile are independent blocks with neighbouring
// block indices, so that whole rows are in flight at any time and not one 512-byte window of every row.
template <int SCHEME, int NKV, int NSET = 1, bool EXCH = false, bool NARROW = false, bool QF32 = false, bool SPLIT = false>  // NKV = n_kv_heads rounded up to 2/4/8/16; EXCH: exchange format out
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NKV * NSET <= 8 ? 4 : 2))) void scores_mfma_i4_gqa_kernel(ScoreArgs a) {
  constexpr int SL = 4 * NSET;  // head slots per kv head
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 4, "4-bit schemes only");
  static_assert(kGqaTilesPerBlock % 2 == 0, "tiles are processed in pairs");
  constexpr int NL = QF32 ? 2 : 1;     // limbs of a query element
  constexpr int NA = NL * NSET;        // copies of the A operands: copy = set * NL + limb
  extern __shared__ float gqa_lds[];
  float* stage = gqa_lds;                            // [kv head][SL head slots][token in tile]
  float4* qs4 = reinterpret_cast<float4*>(stage + a.n_kv_heads * SL * kTile);  // [set][kv head][group]: q sums of the set's 4 heads
  uint4* alds = reinterpret_cast<uint4*>(qs4 + NSET * a.n_kv_heads * 4);  // [set][kv head][b][gq*4 + r]
  uint4* azero = alds + NA * a.n_kv_heads * 64;                           // [kv head][b][gq*4 + r], all zero
  const int meta_stride = a.n_kv_heads * 4 + 2;      // halves; +2 spreads the tokens over banks
  uint16_t* smeta = reinterpret_cast<uint16_t*>(azero + a.n_kv_heads * 64);
  uint16_t* zmeta = smeta + kTile * meta_stride;

  const int c = blockIdx.y;
  const int len = a.fill[c] < a.max_len ? a.fill[c] : a.max_len;
  const int n_groups = SPLIT ? a.row_slabs / a.n_kv_heads : 1;
  const int64_t tile0 = (int64_t)(SPLIT ? blockIdx.x / n_groups : blockIdx.x) * kGqaTilesPerBlock;
  const int64_t tok0 = tile0 * kTile;
  if (tok0 >= len) return;  // uniform for the block
  // query heads per slab; a launch serves heads a.head_off .. a.head_off + rep - 1 of every slab, rep <= 4 NSET
  // (more than 8 heads per slab: two launches; split rows are launched with head_off = 0 only)
  const int rep_all = a.n_q_heads / (SPLIT ? a.row_slabs : a.n_kv_heads);
  const int rep = rep_all - a.head_off < 4 * NSET ? rep_all - a.head_off : 4 * NSET;
  // Heads narrower than 128: a.n_kv_heads counts 128-dimension slabs of the cached row, each the
  // stored bytes of hps = 128 / head_dim neighbouring kv heads, and the rep query heads of a slab
  // are the heads of those kv heads, rep1 each, in order.  Query head r of a slab belongs to kv
  // head r / rep1 of it and its A rows are zero outside that head's groups - the products
  // with the neighbours' codes vanish exactly.
  // (hps is 1, 2 or 4: shifts and comparisons, no integer division in a prologue that every block of
  // two tiles runs)
  const int head_dim = NARROW ? a.head_dim : 128;
  const int gshift = head_dim == 64 ? 1 : 0;          // log2 of a narrow head's groups of 32
  const int rep1 = head_dim == 64 ? rep_all >> 1 : rep_all >> 2;
  auto owns = [&](int r, int gq) {                    // group gq of the slab belongs to the kv head of the launch's query head r
    const int ra = r + a.head_off;                    // ... which is head ra of the slab
    return !NARROW || (gq >> gshift) == (ra >= rep1) + (ra >= 2 * rep1) + (ra >= 3 * rep1);
  };
  auto group_in_head = [&](int gq) { return NARROW ? gq & ((1 << gshift) - 1) : gq; };
  const int lanes_per_row = SPLIT ? a.row_slabs * 4 : a.n_kv_heads * 4;   // 16-byte pieces of a whole cached row
  const int kv_off = SPLIT ? (blockIdx.x % n_groups) * a.n_kv_heads : 0;  // first slab of this block
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nl = lane & 15;
  const int rg = lane >> 4;
  // (the queries of this block's slabs: heads kv_off * rep ...)
  const uint16_t* qbase = reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)c * a.n_q_heads + kv_off * rep_all + a.head_off) * head_dim;
  const float* qfbase = reinterpret_cast<const float*>(a.q) + ((int64_t)c * a.n_q_heads + kv_off * rep_all + a.head_off) * head_dim;
  // bf16 bits of limb `set` of a float32 query element
  auto limb_bits = [](float v, int set) -> uint32_t { return bf16_limb_bits(v, set); };
  const int64_t base_row = a.row_base[c];

  // Code vectors of this wavefront's slice of tile tt (one 16-byte load per kv
  // head) and this thread's share of the tile's (scale, zero) rows: chunk
  // j*256 + thread = (token, kv head), 8 bytes each.
  constexpr int NM = (NKV + 3) / 4;   // 256 (token, kv head) chunks per pass
  struct TileRegs {
    uint4 cv[NKV];
    uint2 sv[NM], zv[NM];
  };
  // Addresses are a wave-uniform base plus a small lane offset: this wavefront's slice starts
  // (wave*16 + nl) rows into the tile, and chunk ch = j*256 + thread of the tile's metadata
  // rows is the (token, kv head) pair, 4*ch halves into the rows (lanes_per_row = 4 kv heads).
  // (64-bit lane addresses per chunk had cost the registers whose spill reloads waited,
  // inside the loop, for the code loads just issued.)
  const int code_lane_off = ((wave * 16 + nl) * lanes_per_row + kv_off * 4 + rg) * 16;
  auto issue = [&](int tt, TileRegs& t) {
    const int64_t t0 = tok0 + tt * kTile;
    const int64_t left = len - t0;
    const int rem = left < kTile ? (int)left : kTile;  // tokens of the tile that exist
    const bool okn = wave * 16 + nl < rem;
    const char* rowp = reinterpret_cast<const char*>(a.codes) + (base_row + t0) * lanes_per_row * 16 + code_lane_off;
#pragma unroll
    for (int g = 0; g < NKV; ++g) {
      t.cv[g] = make_uint4(0, 0, 0, 0);
      if (okn && g < a.n_kv_heads) t.cv[g] = ld16(rowp + g * 64);
    }
    const uint16_t* sb = reinterpret_cast<const uint16_t*>(a.scale) + (base_row + t0) * lanes_per_row;
    const uint16_t* zb = reinterpret_cast<const uint16_t*>(a.zero) + (base_row + t0) * lanes_per_row;
#pragma unroll
    for (int j = 0; j < NM; ++j) {
      t.sv[j] = make_uint2(0, 0);
      t.zv[j] = make_uint2(0, 0);
      if ((int)threadIdx.x < rem * a.n_kv_heads - j * 256) {
        int mo = j * 1024 + threadIdx.x * 4;   // halves into the tile's metadata rows
        if constexpr (SPLIT) {                 // the block's slabs are a piece of every row
          const int ch = j * 256 + threadIdx.x, tok = ch / a.n_kv_heads;
          mo = (tok * a.row_slabs + kv_off + (ch - tok * a.n_kv_heads)) * 4;
        }
        t.sv[j] = *reinterpret_cast<const uint2*>(sb + mo);
        if constexpr (!Q::sym) t.zv[j] = *reinterpret_cast<const uint2*>(zb + mo);
      }
    }
  };
  TileRegs ra, rb;
  issue(0, ra);  // in flight while the prologue runs

  // Prologue: group sums of q, and the non-zero part of the block-diagonal A
  // operands: entry (g, b, gq, r) = q[g*rep + r][32*gq + 8*b + {0,4,1,5,2,6,3,7}].
  // (set s holds heads g*rep + 4 s + r of kv head g; with narrow heads gq counts the groups of
  // the slab and the head's own dimensions start at group (r / rep1) * gph)
  for (int i = threadIdx.x; i < NSET * a.n_kv_heads * 16; i += 256) {
    const int set = i / (a.n_kv_heads * 16), ig = i - set * a.n_kv_heads * 16;
    const int g = ig >> 4, gq = (ig >> 2) & 3, r = (ig & 3) + 4 * set;
    float sacc = 0.f;
    if (r < rep && owns(r, gq)) {
      float h32[32];
      if constexpr (QF32) {
        load_as_float<PIKV_F32, 32>(qfbase, (int64_t)(g * rep_all + r) * head_dim + group_in_head(gq) * 32, h32);
#pragma unroll
        for (int k = 0; k < 32; ++k) h32[k] = bf16_bits_to_float(limb_bits(h32[k], 0)) + bf16_bits_to_float(limb_bits(h32[k], 1));
      } else {
        load_as_float<PIKV_BF16, 32>(qbase, (int64_t)(g * rep_all + r) * head_dim + group_in_head(gq) * 32, h32);
      }
#pragma unroll
      for (int k = 0; k < 32; ++k) sacc += h32[k];
    }
    reinterpret_cast<float*>(qs4)[i] = sacc;
  }
  for (int i = threadIdx.x; i < NA * a.n_kv_heads * 64; i += 256) {
    const int copy = i / (a.n_kv_heads * 64), ig = i - copy * a.n_kv_heads * 64;
    const int set = copy / NL, limb = copy % NL;
    const int g = ig >> 6, b2 = (ig >> 4) & 3, gq = (ig >> 2) & 3, r = (ig & 3) + 4 * set;
    uint4 d = make_uint4(0, 0, 0, 0);
    if (r < rep && owns(r, gq)) {
      if constexpr (QF32) {
        float f8[8];
        load_as_float<PIKV_F32, 8>(qfbase, (int64_t)(g * rep_all + r) * head_dim + group_in_head(gq) * 32 + b2 * 8, f8);
        d = make_uint4(limb_bits(f8[0], limb) | (limb_bits(f8[1], limb) << 16), limb_bits(f8[2], limb) | (limb_bits(f8[3], limb) << 16),
                       limb_bits(f8[4], limb) | (limb_bits(f8[5], limb) << 16), limb_bits(f8[6], limb) | (limb_bits(f8[7], limb) << 16));
      } else {
        d = ld16(qbase + (int64_t)(g * rep_all + r) * head_dim + group_in_head(gq) * 32 + b2 * 8);
      }
    }
    alds[i] = make_uint4((d.x & 0xffffu) | (d.z << 16), (d.x >> 16) | (d.z & 0xffff0000u),
                         (d.y & 0xffffu) | (d.w << 16), (d.y >> 16) | (d.w & 0xffff0000u));
    if (copy == 0) azero[ig] = make_uint4(0, 0, 0, 0);
  }

  const float zbias = 128.0f - (float)Q::qmin;  // 128 (asymmetric) or 136 (symmetric)
  // a lane whose k-slice does not meet its row's group reads zeros
  const bool a_on = (nl >> 2) == rg;
  const uint4* a_lane[NA];
#pragma unroll
  for (int set = 0; set < NA; ++set) a_lane[set] = (a_on ? alds + set * a.n_kv_heads * 64 : azero) + nl;
  // two nibbles -> two bf16 values 128 + code.  Both constants are kept in vector registers
  // (the empty statement hides their values from the compiler, it emits no instruction): with
  // a literal or scalar operand the three-operand and-or instruction cannot be encoded and
  // every expansion falls apart into an AND and an OR.
  uint32_t kNib = 0x000f000fu, kExp = 0x43004300u;
  asm volatile("" : "+v"(kNib), "+v"(kExp));

  // One tile: returns false when the block has run past the cache's fill.
  auto do_tile = [&](int tt, TileRegs& cur, TileRegs& nxt) -> bool {
    const int64_t tile = tile0 + tt;
    const int64_t n0 = tile * kTile;
    if (n0 >= len) return false;  // uniform
    // (scale, zero) rows of the tile into LDS, then start the next tile's loads
#pragma unroll
    for (int j = 0; j < NM; ++j) {
      const int ch = j * 256 + threadIdx.x;
      const int tok = ch / a.n_kv_heads, hd = ch - tok * a.n_kv_heads;
      if (tok < kTile) {
        uint32_t* sd = reinterpret_cast<uint32_t*>(smeta + tok * meta_stride + hd * 4);
        sd[0] = cur.sv[j].x; sd[1] = cur.sv[j].y;
        if constexpr (!Q::sym) {
          uint32_t* zd = reinterpret_cast<uint32_t*>(zmeta + tok * meta_stride + hd * 4);
          zd[0] = cur.zv[j].x; zd[1] = cur.zv[j].y;
        }
      }
    }
    if ((tt + 1 < kGqaTilesPerBlock) && (n0 + kTile < len)) issue(tt + 1, nxt);
    __syncthreads();  // metadata (and, first time, qs4 / alds) visible

    const int tl = wave * 16 + nl;
    const bool okt = n0 + tl < len;
#pragma unroll
    for (int g = 0; g < NKV; ++g) {
      if (g < a.n_kv_heads) {
        const uint32_t wv[4] = {cur.cv[g].x, cur.cv[g].y, cur.cv[g].z, cur.cv[g].w};
        pikv_f32x4 pc[NSET];
#pragma unroll
        for (int set = 0; set < NSET; ++set) pc[set] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int b2 = 0; b2 < 4; ++b2) {
          const uint32_t w = Q::sym ? (wv[b2] ^ 0x88888888u) : wv[b2];
          const uint4 bb = make_uint4(and_or(w, kNib, kExp), and_or(w >> 4, kNib, kExp),
                                      and_or(w >> 8, kNib, kExp), and_or(w >> 12, kNib, kExp));
#pragma unroll
          for (int copy = 0; copy < NA; ++copy) {   // the limbs of float32 queries meet in one accumulator
            const uint4 av = a_lane[copy][(g * 4 + b2) * 16];
            pc[copy / NL] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(pikv_bf16x8, av), __builtin_bit_cast(pikv_bf16x8, bb), pc[copy / NL], 0, 0, 0);
          }
        }
        const int mo = tl * meta_stride + g * 4 + rg;
        const float sc = (float)__builtin_bit_cast(_Float16, smeta[mo]);
        const float zq = (Q::sym ? 0.f : (float)__builtin_bit_cast(_Float16, zmeta[mo])) + zbias;
#pragma unroll
        for (int set = 0; set < NSET; ++set) {
          const float4 qv = qs4[(set * a.n_kv_heads + g) * 4 + rg];
          const float t0 = sc * fmaf(-zq, qv.x, pc[set][0]), t1 = sc * fmaf(-zq, qv.y, pc[set][1]);
          const float t2 = sc * fmaf(-zq, qv.z, pc[set][2]), t3 = sc * fmaf(-zq, qv.w, pc[set][3]);
          // sum over the four row-groups; row-group r ends with head r of the set
          auto s01 = __builtin_amdgcn_permlane16_swap(__float_as_uint(t0), __float_as_uint(t1), false, false);
          auto s23 = __builtin_amdgcn_permlane16_swap(__float_as_uint(t2), __float_as_uint(t3), false, false);
          const float u01 = __uint_as_float(s01[0]) + __uint_as_float(s01[1]);
          const float u23 = __uint_as_float(s23[0]) + __uint_as_float(s23[1]);
          auto sf = __builtin_amdgcn_permlane32_swap(__float_as_uint(u01), __float_as_uint(u23), false, false);
          const float score = (__uint_as_float(sf[0]) + __uint_as_float(sf[1])) * a.scale_qk;
          if (4 * set + rg < rep) stage[(g * SL + 4 * set + rg) * kTile + tl] = okt ? score : -__builtin_inff();
        }
      }
    }
    __syncthreads();

    if constexpr (EXCH) tile_stats_exchange<true, SL>(a, stage, c, tile, n0, len, wave, rg, nl, rep, kv_off * rep_all + a.head_off, rep_all);
    else tile_stats_store<true, SL>(a, stage, c, tile, n0, len, wave, rg, nl, rep, kv_off * rep_all + a.head_off, rep_all);
    __syncthreads();  // stage and the metadata rows are reused by the next tile
    return true;
  };

  for (int tt = 0; tt < kGqaTilesPerBlock; tt += 2) {
    if (!do_tile(tt, ra, rb)) break;
    if (!do_tile(tt + 1, rb, ra)) break;
  }
}

// ---- 8-bit scores on the matrix cores ------------------------------------------------
// Per-head (or coarser) scales, head_dim 128 (64 and 32 as slabs of two / four heads), bf16 queries, up to 16 query heads per kv
// head.  The vector form above is instruction-bound as soon as several query heads share
// a kv head (measured at 64 x 32768 cached tokens, 8 kv heads: 793 us for 4 heads per kv
// head, 2143 us for 8, where HBM allows about 440 us).  An 8-bit code does not fit one
// bf16 exactly, so a stored byte u (the code itself, or code + 128 for the symmetric
// scheme) is fed as its two nibbles: u = 16*hi + lo, both exact as bf16 16 + nibble,
// against A operands that hold q for the low nibble and 16*q (exact,
// a power of two) for the high one:
//   C[head][token] = sum_d q_d*(16 + lo_d) + 16*q_d*(16 + hi_d) = sum_d q_d*u_d + 272*Qs
// with Qs = sum_d q_d, which comes out of the same matrix cores from a constant B operand
// (1 at the low-nibble positions).  score = scale * (C - (272 + zz)*Qs), zz = 128
// (symmetric) or the zero point.  (16 + nibble = 0x4180 | nibble << 3 is the smallest
// offset a single OR can give; the smaller the offset, the less the subtraction costs in
// float32 accuracy.)
// A wavefront owns kv heads {w, w+4, ...} and keeps their A operands in registers (8
// k-steps of 16 dimensions per head); per 16-token slice a lane loads the two 16-byte
// halves of its token's head row, so one load instruction fetches whole 128-byte lines.
constexpr int kI8TilesPerBlock = 4;
constexpr int kI8QsFloats = 4 * 4 * 4 * 16;   // query sums in LDS: 4 wavefronts x up to 4 kv head slots x up to 4 parts x 16

// Heads narrower than 128 (HPS = 128 / head_dim = 2 or 4): a.n_kv_heads counts 128-dimension slabs of
// the cached row, each the stored bytes of HPS neighbouring kv heads; the rep query heads of a slab
// are the heads of those kv heads, rep / HPS each, in order.  A query head's A rows are zero outside
// its own kv head's dimensions, and its scores take that kv head's scale and zero point.
// QF32 (up to 8 query heads per slab): float32 queries as two bf16 limbs, q = hi + lo + (at most
// 2^-18 |q|): A rows 2r and 2r+1 hold the limbs of head r, and the two rows' scores - they sit in
// the same lane - are added before they are staged.
template <int SCHEME, int NHW, int HPS = 1, bool QF32 = false>  // NHW = kv heads per wavefront: ceil(n_kv_heads / 4), 1, 2 or 4
__global__ __launch_bounds__(256) void scores_mfma_i8_kernel(ScoreArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 8, "8-bit schemes only");
  extern __shared__ float i8_lds[];
  float* qs_lds = i8_lds;           // [wavefront][kv head slot][part][row group][4]: query sums (see NQ below)
  float* stage = i8_lds + kI8QsFloats;  // [q head][token in tile]

  const int c = blockIdx.y;
  const int len = a.fill[c] < a.max_len ? a.fill[c] : a.max_len;
  const int64_t tile0 = (int64_t)blockIdx.x * kI8TilesPerBlock;
  if (tile0 * kTile >= len) return;  // uniform for the block
  // a launch serves heads a.head_off .. a.head_off + rep - 1 of every kv head (more than 16 per kv head: several
  // launches, heads of 128 only); the staged rows are those heads, rep per kv head
  const int rep_all = a.n_q_heads / a.n_kv_heads;
  const int rep = rep_all - a.head_off < 16 ? rep_all - a.head_off : 16;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nl = lane & 15;   // token of a slice (B, C column) / query head (A row)
  const int rg = lane >> 4;   // k-slice: dimensions 16*rg .. 16*rg+15 of a 64-wide half
  const int64_t row_bytes = (int64_t)a.n_kv_heads * 128;
  const int groups_per_row = (a.n_kv_heads * 128) / a.group;
  const int64_t base_row = a.row_base[c];
  const uint16_t* qbase = reinterpret_cast<const uint16_t*>(a.q) + (int64_t)c * a.n_q_heads * (128 / HPS);
  const int rep1 = HPS == 1 ? rep : HPS == 2 ? rep >> 1 : rep >> 2;   // query heads per kv head
  // kv head (inside the slab) of query head r: comparisons, no integer division
  auto head_in_slab = [&](int r) { return HPS == 1 ? 0 : (r >= rep1) + (r >= 2 * rep1) + (r >= 3 * rep1); };
  constexpr int RSH = QF32 ? 1 : 0;   // A / C row -> query head of the kv group: row >> RSH (two limb rows per head)
  const int hh_a = head_in_slab(nl >> RSH);  // ... of the query head in A row nl (rows past the heads hold none)
  int hh_c[4];                               // ... of the query heads in this lane's four C rows
#pragma unroll
  for (int qq = 0; qq < 4; ++qq)
    hh_c[qq] = head_in_slab((4 * rg + qq) >> RSH) < HPS ? head_in_slab((4 * rg + qq) >> RSH) : HPS - 1;
  const float* qfbase = reinterpret_cast<const float*>(a.q) + (int64_t)c * a.n_q_heads * (128 / HPS);
  // two nibbles -> two bf16 values 16 + nibble; both constants held in vector registers so that the
  // three-operand and-or instruction can be encoded (the empty statement emits no instruction)
  uint32_t kNib = 0x00780078u, kExp = 0x41804180u;
  asm volatile("" : "+v"(kNib), "+v"(kExp));

  // A operands of this wavefront's kv heads: lane (row nl = query head, k-slice rg), k-step
  // (half, b2) covers dimensions d0 = 64*half + 16*rg + 4*b2 .. +3 in the slot order
  // {d0, d0+2, 16x d0, 16x d0+2, d0+1, d0+3, 16x d0+1, 16x d0+3} that the nibble unpack produces.
  // Rows of 1 or 2 slabs (spread): the wavefronts take (kv head, tile) pairs - item = wave + 4 * round is kv
  // head item % n_kv_heads of tile item / n_kv_heads - so that all four load and multiply and 4 / n_kv_heads
  // tiles of the block are in flight at a time; a wavefront's kv head is the same in every round.
  const int spread = (NHW == 1 && a.n_kv_heads <= 2) ? a.n_kv_heads : 0;
  // The accumulators carry the nibble offsets, 272 * (sum of q) - some 10^4 against scores of some 10 - and every
  // k-step rounds at that magnitude.  The 128 dimensions are therefore accumulated in NQ parts, each with the
  // offset of its own dimensions taken off before the parts are added (four parts: 1.4e-4 -> 4e-5 absolute at
  // |score| 36); fewer parts where the registers of more kv heads per wavefront leave no room.
  // The query sums of the parts live in LDS and are read where they are used: as registers they cost a resident
  // wavefront per SIMD (8-bit scores at 8 kv heads x 32 q heads: 699 vs 588 us).
  constexpr int NQ = NHW == 1 ? 4 : NHW == 2 ? 2 : 1;
  uint4 areg[NHW][8];
#pragma unroll
  for (int hs = 0; hs < NHW; ++hs) {
    const int g = spread ? wave % (spread ? spread : 1) : wave + 4 * hs;
    const bool on = g < a.n_kv_heads && (nl >> RSH) < rep;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      uint2 qd = make_uint2(0, 0);
      const int ds = 64 * (ks >> 2) + 16 * rg + 4 * (ks & 3);   // dimension inside the slab
      if (on && (HPS == 1 || ds / (128 / HPS) == hh_a)) {
        const int64_t qo = (int64_t)(g * rep_all + a.head_off + (nl >> RSH)) * (128 / HPS) + (ds - hh_a * (128 / HPS));
        if constexpr (QF32) {
          float f4[4];
          load_as_float<PIKV_F32, 4>(qfbase, qo, f4);
          uint32_t lb[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) lb[k] = bf16_limb_bits(f4[k], nl & 1);   // limb nl & 1: the float rounded to bf16, or the rest
          qd = make_uint2(lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16));
        } else {
          qd = *reinterpret_cast<const uint2*>(qbase + qo);
        }
      }
      // bf16 x 16: through float, exact (zero stays zero)
      auto x16 = [](uint32_t h) { return __float_as_uint(__uint_as_float(h << 16) * 16.0f) >> 16; };
      const uint32_t q0 = qd.x & 0xffffu, q1 = qd.x >> 16, q2 = qd.y & 0xffffu, q3 = qd.y >> 16;
      areg[hs][ks] = make_uint4(q0 | (q2 << 16), x16(q0) | (x16(q2) << 16), q1 | (q3 << 16), x16(q1) | (x16(q3) << 16));
    }
    // Qs of heads 4*rg .. 4*rg+3 (C rows) from a B operand that is 1 at the low-nibble slots
    const uint4 ones = make_uint4(0x3f803f80u, 0u, 0x3f803f80u, 0u);
#pragma unroll
    for (int part = 0; part < NQ; ++part) {
      pikv_f32x4 sumq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = part * (8 / NQ); ks < (part + 1) * (8 / NQ); ++ks)
        sumq = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, areg[hs][ks]),
                                                       __builtin_bit_cast(pikv_bf16x8, ones), sumq, 0, 0, 0);
      // lanes with the same row group hold the same four sums
      if (nl == 0) *reinterpret_cast<float4*>(qs_lds + (((wave * NHW + hs) * NQ + part) * 4 + rg) * 4) =
          make_float4(sumq[0], sumq[1], sumq[2], sumq[3]);
    }
  }

  // kv head g (A operands of slot hs) against the tile that starts at token n0, scores into st
  auto head_tile = [&](int hs, int g, int64_t n0, float* st) {
    {
      // the four 16-token slices of the tile: two 16-byte halves and the metadata of each
      uint4 cv[4][2];
      float sc[4][HPS], zr[4][HPS];
      bool ok[4];
#pragma unroll
      for (int sl = 0; sl < 4; ++sl) {
        const int64_t n = n0 + 16 * sl + nl;
        ok[sl] = n < len;
        cv[sl][0] = cv[sl][1] = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int k = 0; k < HPS; ++k) sc[sl][k] = zr[sl][k] = 0.f;
        if (ok[sl]) {
          const char* rowp = reinterpret_cast<const char*>(a.codes) + (base_row + n) * row_bytes + g * 128 + 16 * rg;
          cv[sl][0] = ld16(rowp);
          cv[sl][1] = ld16(rowp + 64);
#pragma unroll
          for (int k = 0; k < HPS; ++k) {   // one (scale, zero) per kv head of the slab
            const int64_t mi = (base_row + n) * groups_per_row + (g * 128 + k * (128 / HPS)) / a.group;
            sc[sl][k] = reinterpret_cast<const float*>(a.scale)[mi];
            if constexpr (!Q::sym) zr[sl][k] = reinterpret_cast<const float*>(a.zero)[mi];
          }
        }
      }
#pragma unroll
      for (int sl = 0; sl < 4; ++sl) {
        pikv_f32x4 pc[NQ];
#pragma unroll
        for (int part = 0; part < NQ; ++part) pc[part] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const uint32_t wv[4] = {cv[sl][half].x, cv[sl][half].y, cv[sl][half].z, cv[sl][half].w};
#pragma unroll
          for (int b2 = 0; b2 < 4; ++b2) {
            const uint32_t w = Q::sym ? (wv[b2] ^ 0x80808080u) : wv[b2];
            const uint4 bb = make_uint4(and_or(w << 3, kNib, kExp), and_or(w >> 1, kNib, kExp),
                                        and_or(w >> 5, kNib, kExp), and_or(w >> 9, kNib, kExp));
            constexpr int kPerPart = 8 / NQ;
            pikv_f32x4& pp = pc[(half * 4 + b2) / kPerPart];
            pp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, areg[hs][half * 4 + b2]),
                                                         __builtin_bit_cast(pikv_bf16x8, bb), pp, 0, 0, 0);
          }
        }
        // (the offset is hidden from the compiler, which would otherwise keep the sums in registers across the slices)
        int qoff = ((wave * NHW + hs) * NQ * 4 + rg) * 4;
        asm volatile("" : "+v"(qoff));
        float qsum[NQ][4];
#pragma unroll
        for (int part = 0; part < NQ; ++part) {
          const float4 v = *reinterpret_cast<const float4*>(qs_lds + qoff + part * 16);
          qsum[part][0] = v.x, qsum[part][1] = v.y, qsum[part][2] = v.z, qsum[part][3] = v.w;
        }
        float row_score[4];
#pragma unroll
        for (int qq = 0; qq < 4; ++qq) {
          float scl = sc[sl][0], zrl = zr[sl][0];
#pragma unroll
          for (int k = 1; k < HPS; ++k) {
            scl = hh_c[qq] == k ? sc[sl][k] : scl;
            zrl = hh_c[qq] == k ? zr[sl][k] : zrl;
          }
          const float zz = 272.0f + (Q::sym ? 128.0f : zrl);
          float dot = fmaf(-zz, qsum[0][qq], pc[0][qq]);
#pragma unroll
          for (int part = 1; part < NQ; ++part) dot = dot + fmaf(-zz, qsum[part][qq], pc[part][qq]);
          row_score[qq] = scl * dot * a.scale_qk;
        }
        if constexpr (QF32) {
#pragma unroll
          for (int hq2 = 0; hq2 < 2; ++hq2) {   // rows (2 hq2, 2 hq2 + 1) of this lane: the limbs of one head
            const int r = 2 * rg + hq2;
            if (r < rep)
              st[(g * rep + r) * kTile + 16 * sl + nl] =
                  ok[sl] ? row_score[2 * hq2] + row_score[2 * hq2 + 1] : -__builtin_inff();
          }
        } else {
#pragma unroll
          for (int qq = 0; qq < 4; ++qq) {
            const int r = 4 * rg + qq;
            if (r < rep) st[(g * rep + r) * kTile + 16 * sl + nl] = ok[sl] ? row_score[qq] : -__builtin_inff();
          }
        }
      }
    }
  };
  // the query sums were written by other lanes of this wavefront
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (spread) {
    const int tpr = kI8TilesPerBlock / spread;   // tiles per round, each with a staging area of its own
    for (int round = 0; round < spread; ++round) {
      const int item = wave + 4 * round;
      const int tt = item / spread;
      if ((tile0 + tt) * kTile < len) head_tile(0, item % spread, (tile0 + tt) * kTile, stage + (tt % tpr) * a.n_q_heads * kTile);
      __syncthreads();
      for (int k = 0; k < tpr; ++k) {
        const int64_t tile = tile0 + round * tpr + k;
        if (tile * kTile < len) {  // uniform
          if (rep == rep_all) tile_stats_store<false>(a, stage + k * a.n_q_heads * kTile, c, tile, tile * kTile, len, wave, rg, nl);
          else tile_stats_store<true, 0>(a, stage + k * a.n_q_heads * kTile, c, tile, tile * kTile, len, wave, rg, nl, rep, a.head_off, rep_all);
        }
      }
      __syncthreads();  // the staging areas are reused by the next round
    }
    return;
  }
  for (int tt = 0; tt < kI8TilesPerBlock; ++tt) {
    const int64_t tile = tile0 + tt;
    const int64_t n0 = tile * kTile;
    if (n0 >= len) break;  // uniform
#pragma unroll
    for (int hs = 0; hs < NHW; ++hs) {
      const int g = wave + 4 * hs;
      if (g >= a.n_kv_heads) continue;  // uniform
      head_tile(hs, g, n0, stage);
    }
    __syncthreads();
    if (rep == rep_all) tile_stats_store<false>(a, stage, c, tile, n0, len, wave, rg, nl);
    else tile_stats_store<true, 0>(a, stage, c, tile, n0, len, wave, rg, nl, rep, a.head_off, rep_all);
    __syncthreads();  // stage is reused by the next tile
  }
}

// LDS of scores_mfma_i8_kernel: the staged score rows of every query head of the cache, for 4 or 2 tiles at
// a time on rows of 1 or 2 slabs, plus the query sums.  (The kernel strides its staging areas by
// n_q_heads * 64 floats, whatever part of the heads a launch serves.)
static size_t i8_mfma_lds_bytes(int n_slabs, int n_q_heads) {
  return (size_t)n_q_heads * kTile * sizeof(float) * (n_slabs <= 2 ? kI8TilesPerBlock / n_slabs : 1) +
         kI8QsFloats * sizeof(float);
}
constexpr size_t kI8MfmaMaxLds = 64 * 1024;   // beyond it the vector form serves the cache (one block per compute unit otherwise)

template <int SCHEME, int HPS, bool QF32>
static void launch_i8_mfma_q(const ScoreArgs& a, int n_caches, int64_t n_tiles, hipStream_t st) {
  const size_t lds = i8_mfma_lds_bytes(a.n_kv_heads, a.n_q_heads);
  const dim3 grid((unsigned)((n_tiles + kI8TilesPerBlock - 1) / kI8TilesPerBlock), (unsigned)n_caches);
  if (a.n_kv_heads <= 4)
    hipLaunchKernelGGL((scores_mfma_i8_kernel<SCHEME, 1, HPS, QF32>), grid, dim3(256), lds, st, a);
  else if (a.n_kv_heads <= 8)
    hipLaunchKernelGGL((scores_mfma_i8_kernel<SCHEME, 2, HPS, QF32>), grid, dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((scores_mfma_i8_kernel<SCHEME, 4, HPS, QF32>), grid, dim3(256), lds, st, a);
}
template <int SCHEME, int HPS = 1>
static int launch_i8_mfma(const ScoreArgs& a, int n_caches, int64_t n_tiles, hipStream_t st, bool qf32) {
  if (qf32) launch_i8_mfma_q<SCHEME, HPS, true>(a, n_caches, n_tiles, st);
  else launch_i8_mfma_q<SCHEME, HPS, false>(a, n_caches, n_tiles, st);
  return PIKV_OK;
}

template <int SCHEME, bool EXCH, bool NARROW>
static int launch_gqa_slabs(const ScoreArgs& a0, int n_caches, int64_t n_tiles, hipStream_t st, bool qf32) {
  ScoreArgs a = a0;
  const int rep = a.n_q_heads / a.n_kv_heads;
  const int nset = rep <= 4 ? 1 : 2;
  const size_t lds = gqa_lds_bytes(a.n_kv_heads, nset, qf32 ? 2 * nset : nset);   // float32 queries: a copy of the A operands per limb
  // more than 8 query heads per slab (rows of up to 4 slabs): launches of eight heads each over the same codes
  if (rep > 8 && a.n_kv_heads > 4) return PIKV_ERR_UNSUPPORTED;
  if (lds > 64 * 1024 || a.n_kv_heads > (qf32 ? 8 : kGqaMaxKvHeads)) return PIKV_ERR_UNSUPPORTED;
  for (a.head_off = 0; a.head_off < rep; a.head_off += 4 * nset) {
  const dim3 grid((unsigned)((n_tiles + kGqaTilesPerBlock - 1) / kGqaTilesPerBlock), (unsigned)n_caches);
  // (rows of 1 or 2 slabs have a kernel of their own: fewer registers, 8 instead of 6 blocks per compute unit,
  // and with 5 KB tiles the bytes in flight are what bounds them - 1 kv head x 4 q heads 61.3 -> 52.1 us,
  // 2 x 8: 83.6 -> 76.8 us at 64 caches x 32768 tokens)
  if (qf32 && nset == 1) {
    if (a.n_kv_heads <= 2)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 2, 1, EXCH, NARROW, true>), grid, dim3(256), lds, st, a);
    else if (a.n_kv_heads <= 4)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 4, 1, EXCH, NARROW, true>), grid, dim3(256), lds, st, a);
    else
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 1, EXCH, NARROW, true>), grid, dim3(256), lds, st, a);
  } else if (qf32) {
    if (a.n_kv_heads <= 2)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 2, 2, EXCH, NARROW, true>), grid, dim3(256), lds, st, a);
    else if (a.n_kv_heads <= 4)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 4, 2, EXCH, NARROW, true>), grid, dim3(256), lds, st, a);
    else
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 2, EXCH, NARROW, true>), grid, dim3(256), lds, st, a);
  } else if (nset == 1) {
    if (a.n_kv_heads <= 2)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 2, 1, EXCH, NARROW>), grid, dim3(256), lds, st, a);
    else if (a.n_kv_heads <= 4)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 4, 1, EXCH, NARROW>), grid, dim3(256), lds, st, a);
    else if (a.n_kv_heads <= 8)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 1, EXCH, NARROW>), grid, dim3(256), lds, st, a);
    else
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 16, 1, EXCH, NARROW>), grid, dim3(256), lds, st, a);
  } else {
    // 5-8 query heads per kv head; 16 kv heads x 8 would need more than 64 KB of LDS
    if (a.n_kv_heads <= 2)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 2, 2, EXCH, NARROW>), grid, dim3(256), lds, st, a);
    else if (a.n_kv_heads <= 4)
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 4, 2, EXCH, NARROW>), grid, dim3(256), lds, st, a);
    else
      hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 2, EXCH, NARROW>), grid, dim3(256), lds, st, a);
  }
  }
  return PIKV_OK;
}
// Rows of more than 16 slabs (heads of 128 dimensions): groups of 8 slabs as independent blocks, grid z.
template <int SCHEME, bool EXCH>
static int launch_gqa_split(const ScoreArgs& a0, int n_caches, int64_t n_tiles, hipStream_t st, bool qf32) {
  if (a0.head_dim != 128 || a0.n_kv_heads % 8 != 0) return PIKV_ERR_UNSUPPORTED;
  ScoreArgs a = a0;
  a.row_slabs = a0.n_kv_heads;
  a.n_kv_heads = 8;
  const int rep = a.n_q_heads / a.row_slabs;
  const int nset = rep <= 4 ? 1 : 2;
  const size_t lds = gqa_lds_bytes(8, nset, qf32 ? 2 * nset : nset);
  if (rep > 8 || lds > 64 * 1024) return PIKV_ERR_UNSUPPORTED;
  const int64_t gx = (n_tiles + kGqaTilesPerBlock - 1) / kGqaTilesPerBlock * (a.row_slabs / 8);
  if (gx > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  const dim3 grid((unsigned)gx, (unsigned)n_caches);
  if (qf32 && nset == 1)
    hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 1, EXCH, false, true, true>), grid, dim3(256), lds, st, a);
  else if (qf32)
    hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 2, EXCH, false, true, true>), grid, dim3(256), lds, st, a);
  else if (nset == 1)
    hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 1, EXCH, false, false, true>), grid, dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((scores_mfma_i4_gqa_kernel<SCHEME, 8, 2, EXCH, false, false, true>), grid, dim3(256), lds, st, a);
  return PIKV_OK;
}
// a.n_kv_heads counts 128-dimension slabs, a.head_dim is the width of a stored kv head
template <int SCHEME, bool EXCH = false>
static int launch_gqa(const ScoreArgs& a, int n_caches, int64_t n_tiles, hipStream_t st, bool qf32 = false) {
  if (a.n_kv_heads > 16) return launch_gqa_split<SCHEME, EXCH>(a, n_caches, n_tiles, st, qf32);
  return a.head_dim == 128 ? launch_gqa_slabs<SCHEME, EXCH, false>(a, n_caches, n_tiles, st, qf32)
                           : launch_gqa_slabs<SCHEME, EXCH, true>(a, n_caches, n_tiles, st, qf32);
}

// Final max and sum per (cache, q head) from the tile statistics [cache][tile][head].
// A block takes 16 heads of one cache: thread (head hl, tile lane tl of TL) asks for tiles
// tl, tl+TL, ... eight at a time - neighbouring threads read neighbouring heads - and folds them
// into a running (max, sum) pair; the TL pairs of a head are merged over the 4 tile lanes of a
// wavefront and then over the TL/4 wavefronts, in a fixed order.  TL = 16 (256 threads) covers 128
// tiles in one round of loads, TL = 64 (1024 threads) 512 tiles = 32768 cached tokens
// (64 caches x 512 tiles x 32 heads: 14.1 -> 12.2 us; 8 caches x 128 tiles stay on TL = 16: 16.1 us
// for the whole H2O call against 18.0 us).
constexpr int kStatHeads = 16;   // heads per block of head_stats_kernel
__device__ __forceinline__ void stat_merge(float& m, float& z, float m2, float z2) {
  const float mm = fmaxf(m, m2);
  const float ninf = -__builtin_inff();
  // an empty side has max -inf and sum 0: its term is left out (exp(-inf - -inf) is NaN)
  const float a = m == ninf ? 0.f : z * expf(m - mm);
  const float b = m2 == ninf ? 0.f : z2 * expf(m2 - mm);
  m = mm;
  z = a + b;
}
template <int TL>
__global__ __launch_bounds__(16 * TL) void head_stats_kernel(const float* __restrict__ tile_max,
                                                         const float* __restrict__ tile_sum,
                                                         const int32_t* __restrict__ fill,
                                                         int n_q_heads, int64_t n_tiles,
                                                         float* __restrict__ head_stats) {
  __shared__ float sm[TL / 4][kStatHeads + 1], sz[TL / 4][kStatHeads + 1];
  const int c = blockIdx.y;
  const int hl = threadIdx.x & (kStatHeads - 1), tl = threadIdx.x >> 4;
  const int wave = threadIdx.x >> 6;
  const int hq = blockIdx.x * kStatHeads + hl;
  const int64_t used = ((int64_t)fill[c] + kTile - 1) / kTile;
  const int64_t lim = used < n_tiles ? used : n_tiles;
  const float ninf = -__builtin_inff();
  float m = ninf, z = 0.f;
  if (hq < n_q_heads) {
    const float* tm = tile_max + (int64_t)c * n_tiles * n_q_heads + hq;
    const float* ts = tile_sum + (int64_t)c * n_tiles * n_q_heads + hq;
    for (int64_t t0 = tl; t0 < lim; t0 += TL * 8) {
      float tmx[8], tsm[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {  // eight tiles in flight per thread
        const int64_t t = t0 + TL * u;
        tmx[u] = t < lim ? tm[t * n_q_heads] : ninf;
        tsm[u] = t < lim ? ts[t * n_q_heads] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) stat_merge(m, z, tmx[u], tsm[u]);
    }
  }
  // lanes of a wavefront: 4 tile lanes x 16 heads; lane bits 4..5 are the tile lane
#pragma unroll
  for (int b = 16; b < 64; b <<= 1) {
    const float m2 = __shfl_xor(m, b, 64), z2 = __shfl_xor(z, b, 64);
    // both partners must add in the same order: the lower lane's pair comes first
    if (threadIdx.x & b) { float mo = m2, zo = z2; stat_merge(mo, zo, m, z); m = mo; z = zo; }
    else stat_merge(m, z, m2, z2);
  }
  if ((threadIdx.x & 63) < kStatHeads) {
    sm[wave][hl] = m;
    sz[wave][hl] = z;
  }
  __syncthreads();
  if (threadIdx.x < kStatHeads && hq < n_q_heads) {
    float mm = sm[0][hl], zz = sz[0][hl];
    for (int k = 1; k < TL / 4; ++k) stat_merge(mm, zz, sm[k][hl], sz[k][hl]);
    head_stats[((int64_t)c * n_q_heads + hq) * 2] = mm;
    head_stats[((int64_t)c * n_q_heads + hq) * 2 + 1] = zz;
  }
}

static void launch_head_stats(const float* tile_max, const float* tile_sum, const int32_t* cache_fill, int n_q_heads,
                              int64_t n_tiles, int n_caches, float* head_stats, hipStream_t st) {
  const dim3 grid((unsigned)((n_q_heads + kStatHeads - 1) / kStatHeads), (unsigned)n_caches);
  if (n_tiles > 128)
    hipLaunchKernelGGL(head_stats_kernel<64>, grid, dim3(1024), 0, st, tile_max, tile_sum, cache_fill, n_q_heads, n_tiles,
                       head_stats);
  else
    hipLaunchKernelGGL(head_stats_kernel<16>, grid, dim3(256), 0, st, tile_max, tile_sum, cache_fill, n_q_heads, n_tiles,
                       head_stats);
}

// VEC consecutive tokens per thread (16-byte accesses when VEC = 4) and four q
// heads per round, their loads issued before any store of the round.
template <int VEC, bool WRITE_PROBS>
__global__ __launch_bounds__(256) void h2o_accumulate_kernel(
    float* __restrict__ scores, const float* __restrict__ head_stats, int n_q_heads,
    const int64_t* __restrict__ row_base, const int32_t* __restrict__ fill, int64_t max_len,
    int64_t score_stride, float decay, float now, float* __restrict__ row_acc, float* __restrict__ row_ts,
    float* __restrict__ importance_out) {
  constexpr int UN = VEC == 1 ? 8 : 4;  // heads in flight per thread
  const int c = blockIdx.y;
  const int64_t n0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  const int64_t len = fill[c] < max_len ? (int64_t)fill[c] : max_len;
  if (n0 >= len) return;
  const int cnt = (len - n0 < VEC) ? (int)(len - n0) : VEC;
  const float* hs = head_stats + (int64_t)c * n_q_heads * 2;
  float* sc = scores + (int64_t)c * n_q_heads * score_stride + n0;
  float imp[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) imp[j] = 0.f;
  for (int h0 = 0; h0 < n_q_heads; h0 += UN) {
    float x[UN][VEC];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int hq = h0 + u;
#pragma unroll
      for (int j = 0; j < VEC; ++j) x[u][j] = -__builtin_inff();
      if (hq < n_q_heads) {
        const float* p = sc + (int64_t)hq * score_stride;
        if (VEC == 4 && cnt == 4) {
          const float4 v = *reinterpret_cast<const float4*>(p);
          x[u][0] = v.x; x[u][1] = v.y; x[u][2] = v.z; x[u][3] = v.w;
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            if (j < cnt) x[u][j] = p[j];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int hq = h0 + u;
      if (hq < n_q_heads) {
        const float m = hs[hq * 2];
        const float rz = 1.0f / hs[hq * 2 + 1];
        float pr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          pr[j] = __builtin_amdgcn_exp2f((x[u][j] - m) * 1.4426950408889634f) * rz;
          imp[j] = imp[j] + pr[j];
        }
        if (WRITE_PROBS) {
          float* p = sc + (int64_t)hq * score_stride;
          if (VEC == 4 && cnt == 4) {
            *reinterpret_cast<float4*>(p) = make_float4(pr[0], pr[1], pr[2], pr[3]);
          } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
              if (j < cnt) p[j] = pr[j];
          }
        }
      }
    }
  }
  const int64_t row = row_base[c] + n0;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    if (j < cnt) {
      if (row_acc) {
        float acc = row_acc[row + j];
        if (decay != 1.0f) acc = acc * decay;
        row_acc[row + j] = acc + imp[j];
      }
      if (row_ts) row_ts[row + j] = now;
      if (importance_out) importance_out[(int64_t)c * score_stride + n0 + j] = imp[j];
    }
  }
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
  // staged scores of the block's query heads: the fewer, the more blocks share a compute unit
  const size_t lds = (size_t)(a.n_kv_heads / a.head_split) * REP * kTile * sizeof(float);
  if (q_dtype == PIKV_BF16)
    hipLaunchKernelGGL((scores_kernel<SCHEME, REP, PIKV_BF16>), grid, dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((scores_kernel<SCHEME, REP, PIKV_F32>), grid, dim3(256), lds, st, a);
}

template <int SCHEME>
static int launch_scores(int rep, dim3 grid, hipStream_t st, int q_dtype, ScoreArgs a) {
  // The kernel is compiled for 8, 4, 2 and 1 query heads per kv head; any other ratio is served
  // as the sum of those (7 = 4 + 2 + 1), one launch each over the same codes.
  a.rep = rep;
  for (int off = 0; off < rep;) {
    const int left = rep - off;
    a.head_off = off;
    if (left >= 8) { launch_scores_q<SCHEME, 8>(grid, st, q_dtype, a); off += 8; }
    else if (left >= 4) { launch_scores_q<SCHEME, 4>(grid, st, q_dtype, a); off += 4; }
    else if (left >= 2) { launch_scores_q<SCHEME, 2>(grid, st, q_dtype, a); off += 2; }
    else { launch_scores_q<SCHEME, 1>(grid, st, q_dtype, a); off += 1; }
  }
  return PIKV_OK;
}

int scores_exchange_launch(const void* k_codes, const void* k_scale, const void* k_zero, int scheme, int group,
                           int n_kv_heads, int n_q_heads, int head_dim, const void* q, int q_dtype, float scale_qk,
                           const int64_t* cache_row_base, const int32_t* cache_fill, int n_caches, int64_t max_len,
                           float* escores, float* tile_max, float* tile_sum, float* head_stats, hipStream_t st) {
  if (scheme != PIKV_Q_I4_ASYM && scheme != PIKV_Q_I4_SYM) return PIKV_ERR_UNSUPPORTED;
  if (group != 32 || (q_dtype != PIKV_BF16 && q_dtype != PIKV_F32) || n_q_heads % n_kv_heads != 0) return PIKV_ERR_UNSUPPORTED;
  const int hps = mfma_heads_per_slab(head_dim, n_kv_heads);
  if (hps == 0) return PIKV_ERR_UNSUPPORTED;
  const int slabs = n_kv_heads / hps;   // the kernel's kv heads are 128-dimension slabs of the row
  if ((n_q_heads / slabs > 8 && !(slabs <= 4 && q_dtype == PIKV_BF16)) ||
      n_q_heads > kMaxQHeads || max_len < 1)
    return PIKV_ERR_UNSUPPORTED;
  const int64_t n_tiles = (max_len + kTile - 1) / kTile;
  ScoreArgs a{k_codes, k_scale, k_zero, q, cache_row_base, cache_fill, nullptr, tile_max, tile_sum,
              0, n_tiles, scale_qk, group, slabs, n_q_heads, head_dim, escores,
              (int)(max_len < 0x7fffffffLL ? max_len : 0x7fffffffLL), n_q_heads / slabs, 0, 1};
  const bool qf32 = q_dtype == PIKV_F32;
  const int rc = (scheme == PIKV_Q_I4_ASYM) ? launch_gqa<PIKV_Q_I4_ASYM, true>(a, n_caches, n_tiles, st, qf32)
                                            : launch_gqa<PIKV_Q_I4_SYM, true>(a, n_caches, n_tiles, st, qf32);
  if (rc != PIKV_OK) return rc;
  launch_head_stats(tile_max, tile_sum, cache_fill, n_q_heads, n_tiles, n_caches, head_stats, st);
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
  if (n_q_heads > kMaxQHeads) return PIKV_ERR_UNSUPPORTED;
  if (max_len == 0) return PIKV_OK;
  const int64_t n_tiles = (max_len + kTile - 1) / kTile;
  if (n_tiles > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  ScoreArgs a{k_codes, k_scale, k_zero, q, cache_row_base, cache_fill, scores, tile_max, tile_sum,
              score_stride, n_tiles, scale_qk, group, n_kv_heads, n_q_heads, head_dim, nullptr,
              (int)(max_len < 0x7fffffffLL ? max_len : 0x7fffffffLL), n_q_heads / n_kv_heads, 0, 1};
  const dim3 grid((unsigned)n_tiles, (unsigned)n_caches);
  hipStream_t st = (hipStream_t)stream;
  const int rep = n_q_heads / n_kv_heads;
  // grouped 4-bit caches read with bf16 queries go to the matrix-core kernels; heads of 64 or 32
  // dimensions are served as 128-dimension slabs of two or four neighbouring kv heads
  const int hps = mfma_heads_per_slab(head_dim, n_kv_heads);
  // (float32 queries: as two bf16 limbs on the same kernel, where its operands fit)
  // (more than 8 bf16 query heads per slab on rows of up to 4 slabs: launches of eight heads each; float32
  // queries of such ratios stay on the vector form, which multiplies them exactly)
  const bool more_launches = hps > 0 && n_kv_heads / hps <= 4 && rep * hps > 8;
  if (!eight && group == 32 && hps > 0 && q_dtype == PIKV_F32 && rep * hps <= 8) {
    ScoreArgs as = a;
    as.n_kv_heads = n_kv_heads / hps;
    const int grc = (scheme == PIKV_Q_I4_ASYM) ? launch_gqa<PIKV_Q_I4_ASYM>(as, n_caches, n_tiles, st, true)
                                               : launch_gqa<PIKV_Q_I4_SYM>(as, n_caches, n_tiles, st, true);
    if (grc == PIKV_OK) {
      PIKV_CHECK_LAUNCH();
      return PIKV_OK;
    }
  }
  if (!eight && group == 32 && hps > 0 && q_dtype == PIKV_BF16 && (rep * hps <= (hps == 1 ? 16 : 8) || more_launches)) {
    int grc = PIKV_ERR_UNSUPPORTED;
    const size_t mlds = (size_t)n_q_heads * (kTile + 4) * sizeof(float);
    if (rep * hps <= 8 || more_launches) {
      ScoreArgs as = a;
      as.n_kv_heads = n_kv_heads / hps;
      grc = (scheme == PIKV_Q_I4_ASYM) ? launch_gqa<PIKV_Q_I4_ASYM>(as, n_caches, n_tiles, st)
                                       : launch_gqa<PIKV_Q_I4_SYM>(as, n_caches, n_tiles, st);
    }
    if (grc == PIKV_OK) {
      PIKV_CHECK_LAUNCH();
      return PIKV_OK;
    }
    if (hps == 1) {
      if (scheme == PIKV_Q_I4_ASYM)
        hipLaunchKernelGGL((scores_mfma_i4_kernel<PIKV_Q_I4_ASYM>), grid, dim3(256), mlds, st, a);
      else
        hipLaunchKernelGGL((scores_mfma_i4_kernel<PIKV_Q_I4_SYM>), grid, dim3(256), mlds, st, a);
      PIKV_CHECK_LAUNCH();
      return PIKV_OK;
    }
    // narrow heads that do not fit the slab kernel: the vector form below
  }
  // 8-bit caches with per-head (or coarser) scales, several bf16 query heads per kv head
  // (heads of 64 or 32 dimensions as 128-dimension slabs of two or four neighbouring kv heads)
  // (float32 queries as two bf16 limbs, two operand rows per head: up to 8 heads per slab)
  const bool qf32 = q_dtype == PIKV_F32;
  // (more than 16 bf16 query heads per kv head of 128 on rows of up to 4 kv heads: launches of 16 heads each)
  const bool many = hps == 1 && !qf32 && n_kv_heads <= 4 && rep > 16;
  if (eight && hps > 0 && group % head_dim == 0 && rep >= 2 && (rep * hps <= (qf32 ? 8 : 16) || many) && n_kv_heads / hps <= 16 &&
      i8_mfma_lds_bytes(n_kv_heads / hps, n_q_heads) <= kI8MfmaMaxLds) {
    ScoreArgs as = a;
    as.n_kv_heads = n_kv_heads / hps;
    const bool sym = scheme == PIKV_Q_I8_SYM;
    if (many) {
      for (as.head_off = 0; as.head_off < rep; as.head_off += 16)
        sym ? launch_i8_mfma<PIKV_Q_I8_SYM>(as, n_caches, n_tiles, st, false) : launch_i8_mfma<PIKV_Q_I8_ASYM>(as, n_caches, n_tiles, st, false);
    } else if (hps == 1) sym ? launch_i8_mfma<PIKV_Q_I8_SYM>(as, n_caches, n_tiles, st, qf32) : launch_i8_mfma<PIKV_Q_I8_ASYM>(as, n_caches, n_tiles, st, qf32);
    else if (hps == 2) sym ? launch_i8_mfma<PIKV_Q_I8_SYM, 2>(as, n_caches, n_tiles, st, qf32) : launch_i8_mfma<PIKV_Q_I8_ASYM, 2>(as, n_caches, n_tiles, st, qf32);
    else sym ? launch_i8_mfma<PIKV_Q_I8_SYM, 4>(as, n_caches, n_tiles, st, qf32) : launch_i8_mfma<PIKV_Q_I8_ASYM, 4>(as, n_caches, n_tiles, st, qf32);
    PIKV_CHECK_LAUNCH();
    return PIKV_OK;
  }
  // The blocks of a tile own a power-of-two number of kv heads each (a block's lanes per token must
  // divide 256): 12 kv heads are three blocks of four.  Rows wider than 512 bytes are split further:
  // short-lived blocks of 64 tokens x 512 bytes keep more loads in flight per compute unit than
  // fewer, longer ones.
  a.head_split = n_kv_heads / (n_kv_heads & -n_kv_heads);
  while (lanes_per_row / a.head_split > 32 && n_kv_heads % (a.head_split * 2) == 0) a.head_split *= 2;
  if (lanes_per_row / a.head_split > 256) return PIKV_ERR_UNSUPPORTED;
  if (n_tiles * a.head_split > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  const dim3 vgrid((unsigned)(n_tiles * a.head_split), (unsigned)n_caches);
  int rc = PIKV_ERR_UNSUPPORTED;
  switch (scheme) {
    case PIKV_Q_I8_SYM: rc = launch_scores<PIKV_Q_I8_SYM>(rep, vgrid, st, q_dtype, a); break;
    case PIKV_Q_I8_ASYM: rc = launch_scores<PIKV_Q_I8_ASYM>(rep, vgrid, st, q_dtype, a); break;
    case PIKV_Q_I4_ASYM: rc = launch_scores<PIKV_Q_I4_ASYM>(rep, vgrid, st, q_dtype, a); break;
    case PIKV_Q_I4_SYM: rc = launch_scores<PIKV_Q_I4_SYM>(rep, vgrid, st, q_dtype, a); break;
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
  launch_head_stats(tile_max, tile_sum, cache_fill, n_q_heads, n_tiles, n_caches, head_stats, st);
  // nothing to normalise or accumulate: the caller only wanted the statistics
  if (!write_probs && !row_acc && !row_ts && !importance_out) {
    PIKV_CHECK_LAUNCH();
    return PIKV_OK;
  }
  // 16-byte accesses need every score row to start on a 16-byte boundary - and enough rows to fill the
  // chip with blocks of 1024 tokens: a small problem is a chain of load latencies, and blocks of 256
  // tokens with eight heads in flight per thread put four times the compute units on it
  // (8 caches x 8192 tokens x 32 heads: 19.6 -> 15.6 us)
  const bool vec4 = (score_stride % 4 == 0) && ((reinterpret_cast<uintptr_t>(scores) & 15) == 0) &&
                    ((max_len + 1023) / 1024) * n_caches >= 1024;
  const int per_block = 256 * (vec4 ? 4 : 1);
  const int64_t nb = (max_len + per_block - 1) / per_block;
  if (nb > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  const dim3 grid((unsigned)nb, (unsigned)n_caches);
#define PIKV_H2O_LAUNCH(V, W)                                                                       \
  hipLaunchKernelGGL((h2o_accumulate_kernel<V, W>), grid, dim3(256), 0, st, scores, head_stats,     \
                     n_q_heads, cache_row_base, cache_fill, max_len, score_stride, decay, now, row_acc, \
                     row_ts, importance_out)
  if (vec4) {
    if (write_probs) PIKV_H2O_LAUNCH(4, true); else PIKV_H2O_LAUNCH(4, false);
  } else {
    if (write_probs) PIKV_H2O_LAUNCH(1, true); else PIKV_H2O_LAUNCH(1, false);
  }
#undef PIKV_H2O_LAUNCH
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
