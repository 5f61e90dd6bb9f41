// The decode read over a compressed cache as ONE pass: scores, running softmax and attention
// output in the same kernel, so that no score matrix ever exists in memory.
//
// Replaces, for one new token per sequence, the reference's
//   attention_scores = matmul(q, k^T) / sqrt(dh); probs = softmax(scores); out = matmul(probs, v)
// (core/single/pikv_attention.py:123,163,188) over the dequantised cache, and feeds
// H2OScheduler.update_attention_scores (core/single/cache_scheduling.py:69-73).
//
// Served here: heads of 128 dimensions, 2..8 kv heads; 4-bit codes in groups of 32 (half scale /
// zero point) with 1..4 bf16 query heads per kv head (decode_fused_i4_kernel), with 5..8, or with
// 1..4 float32 ones (decode_fused_i4w_kernel); 8-bit codes with a float scale per kv head or
// coarser and 1..8 bf16 or float32 ones (decode_fused_i8_kernel).  Everything else keeps the
// two-kernel forms of read_path.hip / attend.hip.
//
// Division of labour: a WAVEFRONT owns one kv head of one token range of one cache and walks it
// in tiles of 64 cached tokens - its K codes go straight from memory into matrix-core operands,
// its V codes through a wavefront-private piece of LDS (they are needed transposed), its scores
// never leave registers: the lane that receives the score of (head r, token t) from the
// matrix core is the lane that turns it into the weight rows of the second product.  The
// wavefronts of a block share no data, but they share cache lines (the pieces of a cached row,
// the metadata rows): one block barrier per tile keeps them on the same tile, and the
// metadata of a tile is loaded once for the whole block, a tile ahead.  The 4-bit kernel has two
// tiles on their way from memory per wavefront (two register sets), the 8-bit kernel one.
//
// Softmax over a token range that is still being read: the running maximum m of every head
// (flash-decoding).  When a tile raises it, the accumulators are scaled by exp(m_old - m_new)
// (skipped while no head's maximum moves).  A block leaves (m, sum, unnormalised output) per
// head; decode_finish_kernel merges the ranges.
//
// H2O importance needs every head's final probability of every token, which exists only when
// the last tile has been seen.  The pass therefore leaves e = exp(score - m_at_that_tile) as a
// HALF per (head, token), scaled by 2^15 so that values down to 2^-29 keep 11 significant bits,
// and m_at_that_tile per (tile, head); decode_importance_kernel turns them into probabilities
// (e * exp(m_tile - M) / Z) and adds them to the accumulators.  A sum of positive terms each
// within 2^-11 stays within 2^-11: inside the 1e-3 bar of the accumulators.  The attention
// output never sees the halves.  These stores are what the bookkeeping costs: a compute unit
// whose read stream is saturated takes about 17 cycles per 64-byte write request, during which
// it issues no load addresses (0.8 us per MB written, whatever the size, place or scope of the
// stores; the bare loop shape shows the same in bench_probe.hip).
#include "common.hpp"

namespace pikv {

typedef __bf16 pikv_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pikv_f32x4 __attribute__((ext_vector_type(4)));
typedef int pikv_i32x2 __attribute__((ext_vector_type(2)));

constexpr int kFTile = 64;        // cached tokens per step
constexpr int kFCodeRow = 80;     // bytes per staged V row of one kv head: 64 code bytes + 16 (bank spread, 16-byte aligned)
constexpr int kFARow = 144;       // bytes per staged weight row: 64 tokens x bf16 + 16 (bank spread)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kHalfScale = 32768.0f;   // e is stored as half(e * 2^15)

// wavefront-private LDS (bytes)
constexpr int kFVCodes = 0;                                   // [64 tokens][kFCodeRow]
constexpr int kFVScale = kFVCodes + kFTile * kFCodeRow;       // float4 (4 groups) per token, padded
constexpr int kFMetaBytes = kFTile * 16 + 4 * 64;
constexpr int kFVZterm = kFVScale + kFMetaBytes;
constexpr int kFKMeta = kFVZterm + kFMetaBytes;               // float2 (scale, zero + bias) per (token, group), padded
constexpr int kFKMetaBytes = kFTile * 32 + 4 * 16;
constexpr int kFMetaSet = 2 * kFMetaBytes + kFKMetaBytes;     // the three metadata pieces exist twice: this tile's and the next one's
constexpr int kFABuf = kFVScale + 2 * kFMetaSet;              // [4 groups][8 rows][kFARow]
constexpr int kFAZero = kFABuf + 4 * 8 * kFARow;              // 32 zero bytes: the A piece of rows without a head
constexpr int kFWaveLds = (kFAZero + 32 + 255) & ~255;
static_assert(kFWaveLds * 8 <= 160 * 1024, "eight wavefronts per block fit the LDS of a compute unit");

// V metadata of token t: the tokens {q, 16+q, 32+q, 48+q} one read instruction touches fall
// into different bank quads.
__device__ __forceinline__ int fused_vmeta_off(int tok) { return tok * 16 + (tok >> 4) * 64; }
__device__ __forceinline__ int fused_kmeta_off(int tok, int grp) { return tok * 32 + (tok >> 4) * 16 + grp * 8; }

struct FusedArgs {
  const void* k_codes;
  const void* k_scale;
  const void* k_zero;
  const void* v_codes;
  const void* v_scale;
  const void* v_zero;
  const void* q;            // bf16 [cache][n_q_heads][128]
  const int64_t* row_base;
  const int32_t* fill;
  float* partial;           // [range][cache][q head][128]: unnormalised output of the range
  float* pstats;            // [range][cache][q head][2]: running maximum, sum of exp(score - maximum)
  uint2* e16;               // [cache][tile][kv head][rep * 16 lanes]: 4 halves per lane
  float* tref;              // [cache][tile][q head]: the running maximum the tile's halves refer to
  int64_t n_tiles;          // records per cache in e16 / tref: the tiles of max_len and one spare
  int64_t max_len;
  int n_caches;
  int n_kv_heads;
  int n_q_heads;
  int tokens_per_block;     // a multiple of 128
  float scale_qk;
  int groups;               // blocks per token range: each takes n_kv_heads / groups neighbouring kv heads
};

// BOOK (four query heads per kv head only): the halves and reference maxima of the H2O bookkeeping are
// written, unconditionally - a tile past the end of a range writes zeros into a spare record behind the
// cache's last tile, all 16 lanes of a row-group store the head's reference maximum.
template <int SCHEME, bool BOOK>
__global__ __launch_bounds__(512) void decode_fused_i4_kernel(FusedArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 4, "4-bit schemes only");
  extern __shared__ __align__(16) unsigned char fused_lds[];
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  unsigned char* const lds = fused_lds + wv * kFWaveLds;
  unsigned char* const vcodes = lds + kFVCodes;
  unsigned char* const abuf = lds + kFABuf;
  unsigned char* const azero = lds + kFAZero;

  // grid: x = cache, y = (token range, group of kv heads).  Workgroups go round the eight XCDs in the order
  // of their linear index, so every block of a cache lands on XCD c % 8: the groups of a range share the
  // metadata lines of its rows in one L2.
  const int c = blockIdx.x;
  const int xr = blockIdx.y / a.groups;                                      // token range
  const int HK = a.n_kv_heads;
  const int g = (blockIdx.y % a.groups) * (HK / a.groups) + wv;              // this wavefront's kv head
  const int rep = a.n_q_heads / HK;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  const int64_t t0 = (int64_t)xr * a.tokens_per_block;
  if (t0 >= len) return;   // the merge skips ranges that hold no token
  const int span = (int)((t0 + a.tokens_per_block < len ? t0 + a.tokens_per_block : len) - t0);  // cached tokens of this range
  const int last = span - 1;

  // matrix-core roles.  Scores: lane = (column nl: a token, k-slice rg: a group of 32 dimensions);
  // the result lane (nl, rg) ends with head rg of that token.  Output: lane = (A row / dimension i,
  // k-slice kg: 16 tokens).  Weight preparation: head r, tokens {tk, tk+4, tk+8, tk+12}.
  const int nl = lane & 15, rg = lane >> 4;
  const int i = nl, kg = rg, r = rg;
  const int wkg = nl >> 2, qd = nl & 3;
  const int tk = wkg * 16 + qd;
  const bool row_on = r < rep;
  const float zbias = 128.0f - (float)Q::qmin;
  const int row_codes = HK * 64, row_meta = HK * 8;    // bytes per cached row in the code / metadata planes
  const int64_t urow = a.row_base[c] + t0;
  const char* const kc = reinterpret_cast<const char*>(a.k_codes) + urow * row_codes + g * 64;
  const char* const vc = reinterpret_cast<const char*>(a.v_codes) + urow * row_codes + g * 64;

  if (lane < 8) reinterpret_cast<uint32_t*>(azero)[lane] = 0u;

  // Metadata: the block's 64 x (kv heads) entries of a tile - 8 bytes per entry and plane - are
  // one contiguous run of memory.  Thread e loads entry e = (token e / heads, head e % heads) of every
  // plane, converts it and writes it into the LDS piece of THAT head's wavefront, one tile ahead:
  // the barrier at the top of the next tile publishes it.  (Every wavefront fetching its own head's 8
  // bytes of each row had cost 64 cache lines per load instruction: 140 us of 550.)
  const int nwb = blockDim.x >> 6;                       // wavefronts (kv heads) of this block
  const int g0 = g - wv;                                 // its first kv head
  const int m_tok = threadIdx.x / nwb, m_hd = threadIdx.x - m_tok * nwb;
  unsigned char* const m_lds = fused_lds + m_hd * kFWaveLds;
  const char* const ksb = reinterpret_cast<const char*>(a.k_scale) + urow * row_meta + (g0 + m_hd) * 8;
  const char* const kzb = reinterpret_cast<const char*>(a.k_zero) + urow * row_meta + (g0 + m_hd) * 8;
  const char* const vsb = reinterpret_cast<const char*>(a.v_scale) + urow * row_meta + (g0 + m_hd) * 8;
  const char* const vzb = reinterpret_cast<const char*>(a.v_zero) + urow * row_meta + (g0 + m_hd) * 8;

  // ---- queries: the block-diagonal A operands of the score product, in registers ----
  // A row nl = 4 * group + head; a lane's k-slice rg meets its row's group only when nl / 4 == rg.
  uint4 aq[4];
  float qsum = 0.f;
  {
    const bool a_on = (nl >> 2) == rg && (nl & 3) < rep;
    const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)c * a.n_q_heads + g * rep + (nl & 3)) * 128 + rg * 32;
#pragma unroll
    for (int b2 = 0; b2 < 4; ++b2) {
      uint4 d = make_uint4(0, 0, 0, 0);
      if (a_on) d = ld16(qp + b2 * 8);
      const uint32_t w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        qsum += __uint_as_float(w[k] << 16);
        qsum += __uint_as_float(w[k] & 0xffff0000u);
      }
      // element order inside a k-slice is {0,4,1,5,2,6,3,7}: what the nibble expansion yields
      aq[b2] = make_uint4((d.x & 0xffffu) | (d.z << 16), (d.x >> 16) | (d.z & 0xffff0000u),
                          (d.y & 0xffffu) | (d.w << 16), (d.y >> 16) | (d.w & 0xffff0000u));
    }
  }
  // group sums of the four heads' queries for this lane's group rg: held by lanes 20 * rg + head
  float4 qv;
  qv.x = __shfl(qsum, 20 * rg + 0, PIKV_WAVE);
  qv.y = __shfl(qsum, 20 * rg + 1, PIKV_WAVE);
  qv.z = __shfl(qsum, 20 * rg + 2, PIKV_WAVE);
  qv.w = __shfl(qsum, 20 * rg + 3, PIKV_WAVE);

  pikv_f32x4 C[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) C[d] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
  float zacc[4] = {0.f, 0.f, 0.f, 0.f};
  float lsum = 0.f;
  float m_run = -__builtin_inff();

  // A-operand piece of this lane in the output product: row i of a group's eight rows, or the zero piece
  const bool arow_on = i < 2 * rep;
  const unsigned char* const a_row = arow_on ? abuf + i * kFARow + kg * 32 : azero;
  const int a_step = arow_on ? 8 * kFARow : 0;
  uint32_t kNib = 0x000f000fu, kExp = 0x43004300u;
  asm volatile("" : "+v"(kNib), "+v"(kExp));   // both constants in vector registers: the and-or stays one instruction

  struct TileRegs {
    uint4 k[4], v[4];
    uint2 ks, kz, vs, vz;
  };
  // Every load is issued, from a row clamped to the range's last cached token: a token past the end
  // reads a copy of that row and gets the weight zero.
  auto clamp_row = [&](int tok) { return tok < last ? tok : last; };
  auto issue_meta = [&](int n0, TileRegs& t) {   // this thread's metadata entry of the tile that starts at n0
    const uint32_t mo = (uint32_t)(clamp_row(n0 + m_tok) * row_meta);
    t.ks = *reinterpret_cast<const uint2*>(ksb + mo);
    t.vs = *reinterpret_cast<const uint2*>(vsb + mo);
    t.kz = make_uint2(0, 0);
    t.vz = make_uint2(0, 0);
    if constexpr (!Q::sym) {
      t.kz = *reinterpret_cast<const uint2*>(kzb + mo);
      t.vz = *reinterpret_cast<const uint2*>(vzb + mo);
    }
  };
  auto issue_v = [&](int n0, TileRegs& t) {   // n0: first token of the tile, relative to the range
#pragma unroll
    for (int k = 0; k < 4; ++k)
      t.v[k] = ld16(vc + (uint32_t)(clamp_row(n0 + 16 * k + (lane >> 2)) * row_codes + (lane & 3) * 16));
    issue_meta(n0 + kFTile, t);   // the metadata of the tile AFTER these codes: it is staged a tile ahead
  };
  auto issue_k = [&](int n0, TileRegs& t) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
      t.k[s] = ld16(kc + (uint32_t)(clamp_row(n0 + tk + 4 * s) * row_codes + rg * 16));
  };
  auto h2f = [](uint32_t w, int hi) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> (16 * hi))); };
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  auto pin_order = [] { asm volatile("" ::: "memory"); };
  auto stage_meta = [&](const TileRegs& t, int set) {
    unsigned char* const mb = m_lds + set * kFMetaSet;
    const int mo = fused_vmeta_off(m_tok);
    *reinterpret_cast<float4*>(mb + kFVScale + mo) = make_float4(h2f(t.vs.x, 0), h2f(t.vs.x, 1), h2f(t.vs.y, 0), h2f(t.vs.y, 1));
    *reinterpret_cast<float4*>(mb + kFVZterm + mo) = make_float4(h2f(t.vz.x, 0) + zbias, h2f(t.vz.x, 1) + zbias,
                                                                 h2f(t.vz.y, 0) + zbias, h2f(t.vz.y, 1) + zbias);
    float4* km = reinterpret_cast<float4*>(mb + kFKMeta + fused_kmeta_off(m_tok, 0));
    km[0] = make_float4(h2f(t.ks.x, 0), h2f(t.kz.x, 0) + zbias, h2f(t.ks.x, 1), h2f(t.kz.x, 1) + zbias);
    km[1] = make_float4(h2f(t.ks.y, 0), h2f(t.kz.y, 0) + zbias, h2f(t.ks.y, 1), h2f(t.kz.y, 1) + zbias);
  };
  auto do_tile = [&](int n0, TileRegs& t, const int par) {   // par: parity of the tile = the metadata set it reads
    // ---- stage: V codes, V metadata (as floats, zero point + bias) and K metadata of the tile ----
    // The wavefronts of a block share nothing, but they share cache lines: the eight 64-byte pieces of a
    // cached row, the eight 8-byte pieces of a metadata row.  Left to drift apart they fetched every
    // line again and again (5.76 GB from memory for 2.68 GB of cache); one block barrier per tile keeps
    // their requests for a line inside the caches' reach.
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k)
      *reinterpret_cast<uint4*>(vcodes + (16 * k + (lane >> 2)) * kFCodeRow + (lane & 3) * 16) = t.v[k];
    stage_meta(t, par ^ 1);   // the NEXT tile's metadata, into the other set
    wave_sync();
    const unsigned char* const vscale = lds + kFVScale + par * kFMetaSet;
    const unsigned char* const vzterm = lds + kFVZterm + par * kFMetaSet;
    const unsigned char* const kmeta = lds + kFKMeta + par * kFMetaSet;
    pin_order();
    issue_v(n0 + 2 * kFTile, t);   // the tile after the next one, into the registers just emptied
    pin_order();

    // ---- scores of (head rg, tokens tk + 4 s) ----
    float sc4[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint32_t wv[4] = {t.k[s].x, t.k[s].y, t.k[s].z, t.k[s].w};
      pikv_f32x4 pc = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int b2 = 0; b2 < 4; ++b2) {
        const uint32_t w = Q::sym ? (wv[b2] ^ 0x88888888u) : wv[b2];
        const uint4 bb = make_uint4(and_or(w, kNib, kExp), and_or(w >> 4, kNib, kExp), and_or(w >> 8, kNib, kExp),
                                    and_or(w >> 12, kNib, kExp));
        pc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aq[b2]),
                                                     __builtin_bit_cast(pikv_bf16x8, bb), pc, 0, 0, 0);
      }
      const int tok = tk + 4 * s;
      const float2 km = *reinterpret_cast<const float2*>(kmeta + fused_kmeta_off(tok, rg));
      const float u0 = km.x * fmaf(-km.y, qv.x, pc[0]), u1 = km.x * fmaf(-km.y, qv.y, pc[1]);
      const float u2 = km.x * fmaf(-km.y, qv.z, pc[2]), u3 = km.x * fmaf(-km.y, qv.w, pc[3]);
      // sum over the four groups; row-group r ends with head r
      auto s01 = __builtin_amdgcn_permlane16_swap(__float_as_uint(u0), __float_as_uint(u1), false, false);
      auto s23 = __builtin_amdgcn_permlane16_swap(__float_as_uint(u2), __float_as_uint(u3), false, false);
      const float u01 = __uint_as_float(s01[0]) + __uint_as_float(s01[1]);
      const float u23 = __uint_as_float(s23[0]) + __uint_as_float(s23[1]);
      auto sf = __builtin_amdgcn_permlane32_swap(__float_as_uint(u01), __float_as_uint(u23), false, false);
      const float score = (__uint_as_float(sf[0]) + __uint_as_float(sf[1])) * a.scale_qk;
      sc4[s] = (n0 + tok <= last && row_on) ? score : -__builtin_inff();
    }
    pin_order();
    issue_k(n0 + 2 * kFTile, t);
    pin_order();

    // ---- running softmax of head r (all 16 lanes of a row-group hold the same statistics) ----
    const float m_tile = group_max_dpp(fmaxf(fmaxf(sc4[0], sc4[1]), fmaxf(sc4[2], sc4[3])), 16);
    const float m_new = fmaxf(m_run, m_tile);
    // rows without a head (and tiles past the end) keep -inf: their weights are zero whatever the reference
    const float m_ref = m_new == -__builtin_inff() ? 0.f : m_new;
    // (exp(-inf) = 0 the first time; a maximum that did not move - also the -inf of a row without a head - is 1)
    const float alpha = m_run == m_new ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_ref) * kLog2e);
    m_run = m_new;
    if (__ballot(alpha != 1.0f) != 0ull) {   // some head's maximum moved: scale what has been added so far
      lsum *= alpha;
#pragma unroll
      for (int sg = 0; sg < 4; ++sg) zacc[sg] *= alpha;
      const float a0 = __shfl(alpha, 32 * kg, PIKV_WAVE), a1 = __shfl(alpha, 32 * kg + 16, PIKV_WAVE);   // heads 2 kg, 2 kg + 1
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        C[d][0] *= a0; C[d][1] *= a0;
        C[d][2] *= a1; C[d][3] *= a1;
      }
    }
    float p4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p4[j] = __builtin_amdgcn_exp2f((sc4[j] - m_ref) * kLog2e);
      lsum += p4[j];
    }
    if constexpr (BOOK) {
      // a.n_tiles counts one spare record per cache: the tile index of a tile past the end is at most that
      const int64_t tile = (t0 + n0) / kFTile;
      const uint32_t h0 = __builtin_bit_cast(uint16_t, (_Float16)(p4[0] * kHalfScale));
      const uint32_t h1 = __builtin_bit_cast(uint16_t, (_Float16)(p4[1] * kHalfScale));
      const uint32_t h2 = __builtin_bit_cast(uint16_t, (_Float16)(p4[2] * kHalfScale));
      const uint32_t h3 = __builtin_bit_cast(uint16_t, (_Float16)(p4[3] * kHalfScale));
      uint2* const erec = a.e16 + (((int64_t)c * a.n_tiles + tile) * HK + g) * (rep * 16);
      float* const rrec = a.tref + ((int64_t)c * a.n_tiles + tile) * a.n_q_heads + g * rep;
      erec[lane] = make_uint2(h0 | (h1 << 16), h2 | (h3 << 16));
      rrec[r] = m_ref;
    }

    // ---- weights: p * scale of the V group as a bf16 high part and a bf16 remainder ----
    float4 s4[4], z4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s4[j] = *reinterpret_cast<const float4*>(vscale + fused_vmeta_off(tk + 4 * j));
      z4[j] = *reinterpret_cast<const float4*>(vzterm + fused_vmeta_off(tk + 4 * j));
    }
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) {
      float hi[4], lo[4];
      float zsum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sc = sg == 0 ? s4[j].x : sg == 1 ? s4[j].y : sg == 2 ? s4[j].z : s4[j].w;
        const float zt = sg == 0 ? z4[j].x : sg == 1 ? z4[j].y : sg == 2 ? z4[j].z : z4[j].w;
        const float w = p4[j] * sc;
        hi[j] = __uint_as_float(__float_as_uint(w) & 0xffff0000u);
        lo[j] = __uint_as_float(__float_as_uint(w - hi[j]) & 0xffff0000u);
        // the zero-point sum uses the SAME two-part value: what the matrix core multiplies with
        // 128 + code is taken off again exactly
        zsum = fmaf(hi[j] + lo[j], zt, zsum);
      }
      zacc[sg] += zsum;
      if (row_on) {
        // operand order inside 8 tokens is {0,4,1,5,2,6,3,7}: tokens (k, k+4) share a dword
        uint32_t* rowh = reinterpret_cast<uint32_t*>(abuf + (sg * 8 + 2 * r) * kFARow + wkg * 32) + qd;
        uint32_t* rowl = reinterpret_cast<uint32_t*>(abuf + (sg * 8 + 2 * r + 1) * kFARow + wkg * 32) + qd;
        rowh[0] = (__float_as_uint(hi[0]) >> 16) | __float_as_uint(hi[1]);
        rowh[4] = (__float_as_uint(hi[2]) >> 16) | __float_as_uint(hi[3]);
        rowl[0] = (__float_as_uint(lo[0]) >> 16) | __float_as_uint(lo[1]);
        rowl[4] = (__float_as_uint(lo[2]) >> 16) | __float_as_uint(lo[3]);
      }
    }
    wave_sync();   // the rows were written by other lanes of this wavefront

    // ---- output product: rows 2r / 2r+1 against 16 dimensions of 64 tokens ----
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) {
      const uint4* ap = reinterpret_cast<const uint4*>(a_row + sg * a_step);
      const uint4 a1 = ap[0], a2 = ap[1];
#pragma unroll
      for (int dbl = 0; dbl < 2; ++dbl) {
        const int db = 2 * sg + dbl;
        // lane i lends the 8 code bytes of token kg*16+i that cover dims db*16..+15 and receives
        // the nibbles of dimension db*16+i from its 16 neighbours
        const pikv_i32x2 tr = __builtin_amdgcn_ds_read_tr4_b64_v2i32(
            (pikv_i32x2 __attribute__((address_space(3)))*)(vcodes + (kg * 16 + i) * kFCodeRow + db * 8));
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const uint32_t u = Q::sym ? ((uint32_t)tr[half] ^ 0x88888888u) : (uint32_t)tr[half];
          const uint4 bb = make_uint4(and_or(u, kNib, kExp), and_or(u >> 4, kNib, kExp), and_or(u >> 8, kNib, kExp),
                                      and_or(u >> 12, kNib, kExp));
          C[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, half ? a2 : a1),
                                                          __builtin_bit_cast(pikv_bf16x8, bb), C[db], 0, 0, 0);
        }
      }
    }
  };

  // The loads of a register set must stay in program order against those of the other set: the wait in
  // front of a tile counts the loads issued AFTER the ones it needs, and one count serves the first trip
  // and every later one.  (Left to itself the scheduler had put the first tile's V loads last: the wait
  // became "everything", the second set's prefetch included.)
  auto pin = [] { asm volatile("" ::: "memory"); };
  TileRegs ra, rb;
  issue_meta(0, ra);
  stage_meta(ra, 0);
  pin();
  issue_v(0, ra);
  pin();
  issue_k(0, ra);
  pin();
  issue_v(kFTile, rb);
  pin();
  issue_k(kFTile, rb);
  pin();
  for (int n0 = 0; n0 < span; n0 += 2 * kFTile) {
    do_tile(n0, ra, 0);
    do_tile(n0 + kFTile, rb, 1);   // a tile past the end adds nothing (weights zero)
  }

  // ---- what the range leaves: (maximum, sum, unnormalised output) of each head ----
  const float ltot = group_sum_dpp(lsum, 16);
  wave_sync();
  float* const zl = reinterpret_cast<float*>(lds);   // [head r][group]
#pragma unroll
  for (int sg = 0; sg < 4; ++sg) {
    const float z = group_sum_dpp(zacc[sg], 16);
    if (nl == 0) zl[r * 4 + sg] = z;
  }
  wave_sync();
  const int64_t pbase = ((int64_t)xr * a.n_caches + c) * a.n_q_heads + g * rep;
  if (row_on && nl == 0) {
    a.pstats[(pbase + r) * 2] = m_run;
    a.pstats[(pbase + r) * 2 + 1] = ltot;
  }
  // C: lane (dimension i, rows 4 kg + q): rows 2r / 2r+1 are the two parts of head r
#pragma unroll
  for (int rr = 0; rr < 2; ++rr) {
    const int ro = 2 * kg + rr;
    if (ro >= rep) continue;
    float* o = a.partial + (pbase + ro) * 128;
#pragma unroll
    for (int db = 0; db < 8; ++db) o[db * 16 + i] = (C[db][2 * rr] + C[db][2 * rr + 1]) - zl[ro * 4 + (db >> 1)];
  }
}

// ---- the 4-bit pass with TWO sets of query operands ------------------------------------------------
// The block-diagonal A operand above holds four query heads (rows = 4 groups x 4 heads).  A second operand
// set, multiplied with the same expanded codes, serves either heads 4..7 of the kv head (5 to 8 bf16 query
// heads per kv head) or the low limbs of float32 queries (QF32: q = hi + lo to 2^-18 |q|, hi = the float rounded
// to bf16, lo = the rest rounded to bf16; the two sets' scores of a head are added, everything
// after that is the one-set kernel's).  What changes besides: a lane runs the softmax of TWO heads (rg and
// 4 + rg) x four tokens; the weight rows of eight heads x two parts fill all 16 A rows of the output product,
// which therefore runs in two passes of two groups each through the same 4.6 KB of LDS; and there is ONE
// register set for the codes on their way (the second operand set and the second head's state take the
// registers of the other one), refilled as in the 8-bit kernel: V as soon as the tile's codes are staged, K
// as soon as its scores are done.  Bookkeeping records: one per (kv head, operand set), each laid out as the
// one-set kernel's (QF32: that kernel's records exactly).
template <int SCHEME, bool BOOK, bool QF32>
__global__ __launch_bounds__(512) void decode_fused_i4w_kernel(FusedArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 4, "4-bit schemes only");
  constexpr int NH = QF32 ? 1 : 2;   // query heads per lane: rg (and 4 + rg)
  extern __shared__ __align__(16) unsigned char fused_lds[];
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  unsigned char* const lds = fused_lds + wv * kFWaveLds;
  unsigned char* const vcodes = lds + kFVCodes;
  unsigned char* const abuf = lds + kFABuf;     // [2 groups][16 rows][kFARow]
  unsigned char* const azero = lds + kFAZero;

  const int c = blockIdx.x;
  const int xr = blockIdx.y;
  const int HK = a.n_kv_heads;
  const int g = wv;
  const int rep = a.n_q_heads / HK;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  const int64_t t0 = (int64_t)xr * a.tokens_per_block;
  if (t0 >= len) return;   // the merge skips ranges that hold no token
  const int span = (int)((t0 + a.tokens_per_block < len ? t0 + a.tokens_per_block : len) - t0);
  const int last = span - 1;

  const int nl = lane & 15, rg = lane >> 4;
  const int i = nl, kg = rg;
  const int wkg = nl >> 2, qd = nl & 3;
  const int tk = wkg * 16 + qd;
  bool row_on[NH];
#pragma unroll
  for (int k = 0; k < NH; ++k) row_on[k] = rg + 4 * k < rep;
  const float zbias = 128.0f - (float)Q::qmin;
  const int row_codes = HK * 64, row_meta = HK * 8;
  const int64_t urow = a.row_base[c] + t0;
  const char* const kc = reinterpret_cast<const char*>(a.k_codes) + urow * row_codes + g * 64;
  const char* const vc = reinterpret_cast<const char*>(a.v_codes) + urow * row_codes + g * 64;

  if (lane < 8) reinterpret_cast<uint32_t*>(azero)[lane] = 0u;

  // metadata: thread e takes entry (token e / heads, head e % heads) of a tile's rows, one tile ahead
  const int m_tok = threadIdx.x / HK, m_hd = threadIdx.x - m_tok * HK;
  unsigned char* const m_lds = fused_lds + m_hd * kFWaveLds;
  const char* const ksb = reinterpret_cast<const char*>(a.k_scale) + urow * row_meta + m_hd * 8;
  const char* const kzb = reinterpret_cast<const char*>(a.k_zero) + urow * row_meta + m_hd * 8;
  const char* const vsb = reinterpret_cast<const char*>(a.v_scale) + urow * row_meta + m_hd * 8;
  const char* const vzb = reinterpret_cast<const char*>(a.v_zero) + urow * row_meta + m_hd * 8;

  // ---- queries: two block-diagonal A operand sets.  Row nl = 4 * group + head of the set; a lane's k-slice
  // rg meets its row's group only when nl / 4 == rg.  Set s holds heads 4 s .. 4 s + 3 (QF32: limb s of heads 0..3).
  uint4 aq[2][4];
  float4 qv[2];
#pragma unroll
  for (int st = 0; st < 2; ++st) {
    const int head = QF32 ? (nl & 3) : 4 * st + (nl & 3);
    const bool a_on = (nl >> 2) == rg && head < rep;
    const int64_t qo = ((int64_t)c * a.n_q_heads + g * rep + (head < rep ? head : 0)) * 128 + rg * 32;
    float qsum = 0.f;
#pragma unroll
    for (int b2 = 0; b2 < 4; ++b2) {
      uint4 d = make_uint4(0, 0, 0, 0);
      if constexpr (QF32) {
        if (a_on) {
          const float* qf = reinterpret_cast<const float*>(a.q) + qo + b2 * 8;
          uint32_t e[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            e[k] = bf16_limb_bits(qf[k], st);
          }
          d = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
        }
      } else {
        if (a_on) d = ld16(reinterpret_cast<const uint16_t*>(a.q) + qo + b2 * 8);
      }
      const uint32_t w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        qsum += __uint_as_float(w[k] << 16);
        qsum += __uint_as_float(w[k] & 0xffff0000u);
      }
      // element order inside a k-slice is {0,4,1,5,2,6,3,7}: what the nibble expansion yields
      aq[st][b2] = make_uint4((d.x & 0xffffu) | (d.z << 16), (d.x >> 16) | (d.z & 0xffff0000u),
                              (d.y & 0xffffu) | (d.w << 16), (d.y >> 16) | (d.w & 0xffff0000u));
    }
    // group sums of the set's four rows for this lane's group rg: held by lanes 20 * rg + row
    qv[st].x = __shfl(qsum, 20 * rg + 0, PIKV_WAVE);
    qv[st].y = __shfl(qsum, 20 * rg + 1, PIKV_WAVE);
    qv[st].z = __shfl(qsum, 20 * rg + 2, PIKV_WAVE);
    qv[st].w = __shfl(qsum, 20 * rg + 3, PIKV_WAVE);
  }

  pikv_f32x4 C[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) C[d] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
  float zacc[NH][4], lsum[NH], m_run[NH];
#pragma unroll
  for (int k = 0; k < NH; ++k) {
    lsum[k] = 0.f;
    m_run[k] = -__builtin_inff();
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) zacc[k][sg] = 0.f;
  }

  // A-operand piece of this lane in the output product: row i = (head i / 2, part i % 2) of a group's 16 rows
  const bool arow_on = i < 2 * rep;
  const unsigned char* const a_row = arow_on ? abuf + i * kFARow + kg * 32 : azero;
  const int a_gstep = arow_on ? 16 * kFARow : 0;
  uint32_t kNib = 0x000f000fu, kExp = 0x43004300u;
  asm volatile("" : "+v"(kNib), "+v"(kExp));   // both constants in vector registers: the and-or stays one instruction

  uint4 rk[4], rv[4];
  uint2 mks, mkz, mvs, mvz;
  auto clamp_row = [&](int tok) { return tok < last ? tok : last; };
  auto issue_meta = [&](int n0) {
    const uint32_t mo = (uint32_t)(clamp_row(n0 + m_tok) * row_meta);
    mks = *reinterpret_cast<const uint2*>(ksb + mo);
    mvs = *reinterpret_cast<const uint2*>(vsb + mo);
    mkz = make_uint2(0, 0);
    mvz = make_uint2(0, 0);
    if constexpr (!Q::sym) {
      mkz = *reinterpret_cast<const uint2*>(kzb + mo);
      mvz = *reinterpret_cast<const uint2*>(vzb + mo);
    }
  };
  auto issue_v = [&](int n0) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      rv[k] = ld16(vc + (uint32_t)(clamp_row(n0 + 16 * k + (lane >> 2)) * row_codes + (lane & 3) * 16));
  };
  auto issue_k = [&](int n0) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
      rk[s] = ld16(kc + (uint32_t)(clamp_row(n0 + tk + 4 * s) * row_codes + rg * 16));
  };
  auto h2f = [](uint32_t w, int hi) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> (16 * hi))); };
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  auto pin_order = [] { asm volatile("" ::: "memory"); };
  auto stage_meta = [&](int set) {
    unsigned char* const mb = m_lds + set * kFMetaSet;
    const int mo = fused_vmeta_off(m_tok);
    *reinterpret_cast<float4*>(mb + kFVScale + mo) = make_float4(h2f(mvs.x, 0), h2f(mvs.x, 1), h2f(mvs.y, 0), h2f(mvs.y, 1));
    *reinterpret_cast<float4*>(mb + kFVZterm + mo) = make_float4(h2f(mvz.x, 0) + zbias, h2f(mvz.x, 1) + zbias,
                                                                 h2f(mvz.y, 0) + zbias, h2f(mvz.y, 1) + zbias);
    float4* km = reinterpret_cast<float4*>(mb + kFKMeta + fused_kmeta_off(m_tok, 0));
    km[0] = make_float4(h2f(mks.x, 0), h2f(mkz.x, 0) + zbias, h2f(mks.x, 1), h2f(mkz.x, 1) + zbias);
    km[1] = make_float4(h2f(mks.y, 0), h2f(mkz.y, 0) + zbias, h2f(mks.y, 1), h2f(mkz.y, 1) + zbias);
  };

  issue_meta(0);
  stage_meta(0);
  pin_order();
  issue_meta(kFTile);
  issue_v(0);
  pin_order();
  issue_k(0);
  pin_order();

  for (int n0 = 0; n0 < span; n0 += kFTile) {
    const int par = (n0 / kFTile) & 1;
    __syncthreads();   // keeps the wavefronts on one tile, and publishes the metadata their threads wrote for each other
#pragma unroll
    for (int k = 0; k < 4; ++k)
      *reinterpret_cast<uint4*>(vcodes + (16 * k + (lane >> 2)) * kFCodeRow + (lane & 3) * 16) = rv[k];
    stage_meta(par ^ 1);   // the NEXT tile's metadata, into the other set
    wave_sync();
    const unsigned char* const vscale = lds + kFVScale + par * kFMetaSet;
    const unsigned char* const vzterm = lds + kFVZterm + par * kFMetaSet;
    const unsigned char* const kmeta = lds + kFKMeta + par * kFMetaSet;
    pin_order();
    issue_v(n0 + kFTile);
    issue_meta(n0 + 2 * kFTile);
    pin_order();

    // ---- scores of heads rg (and 4 + rg), tokens tk + 4 s ----
    float sc[NH][4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint32_t wv4[4] = {rk[s].x, rk[s].y, rk[s].z, rk[s].w};
      pikv_f32x4 pc0 = pikv_f32x4{0.f, 0.f, 0.f, 0.f}, pc1 = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int b2 = 0; b2 < 4; ++b2) {
        const uint32_t w = Q::sym ? (wv4[b2] ^ 0x88888888u) : wv4[b2];
        const uint4 bb = make_uint4(and_or(w, kNib, kExp), and_or(w >> 4, kNib, kExp), and_or(w >> 8, kNib, kExp),
                                    and_or(w >> 12, kNib, kExp));
        pc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aq[0][b2]),
                                                      __builtin_bit_cast(pikv_bf16x8, bb), pc0, 0, 0, 0);
        pc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aq[1][b2]),
                                                      __builtin_bit_cast(pikv_bf16x8, bb), pc1, 0, 0, 0);
      }
      const int tok = tk + 4 * s;
      const float2 km = *reinterpret_cast<const float2*>(kmeta + fused_kmeta_off(tok, rg));
      float set_score[2];
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const pikv_f32x4 pc = st ? pc1 : pc0;
        const float4 q4 = qv[st];
        const float u0 = km.x * fmaf(-km.y, q4.x, pc[0]), u1 = km.x * fmaf(-km.y, q4.y, pc[1]);
        const float u2 = km.x * fmaf(-km.y, q4.z, pc[2]), u3 = km.x * fmaf(-km.y, q4.w, pc[3]);
        // sum over the four groups; row-group r ends with row r of the set
        auto s01 = __builtin_amdgcn_permlane16_swap(__float_as_uint(u0), __float_as_uint(u1), false, false);
        auto s23 = __builtin_amdgcn_permlane16_swap(__float_as_uint(u2), __float_as_uint(u3), false, false);
        const float u01 = __uint_as_float(s01[0]) + __uint_as_float(s01[1]);
        const float u23 = __uint_as_float(s23[0]) + __uint_as_float(s23[1]);
        auto sf = __builtin_amdgcn_permlane32_swap(__float_as_uint(u01), __float_as_uint(u23), false, false);
        set_score[st] = __uint_as_float(sf[0]) + __uint_as_float(sf[1]);
      }
      const bool tok_on = n0 + tok <= last;
      if constexpr (QF32) {
        sc[0][s] = (tok_on && row_on[0]) ? (set_score[0] + set_score[1]) * a.scale_qk : -__builtin_inff();
      } else {
        sc[0][s] = (tok_on && row_on[0]) ? set_score[0] * a.scale_qk : -__builtin_inff();
        sc[NH - 1][s] = (tok_on && row_on[NH - 1]) ? set_score[1] * a.scale_qk : -__builtin_inff();
      }
    }
    pin_order();
    issue_k(n0 + kFTile);
    pin_order();

    // ---- running softmax of the lane's heads (all 16 lanes of a row-group hold the same statistics) ----
    float alpha[NH], m_ref[NH], p4[NH][4];
    bool moved = false;
#pragma unroll
    for (int k = 0; k < NH; ++k) {
      const float m_tile = group_max_dpp(fmaxf(fmaxf(sc[k][0], sc[k][1]), fmaxf(sc[k][2], sc[k][3])), 16);
      const float m_new = fmaxf(m_run[k], m_tile);
      m_ref[k] = m_new == -__builtin_inff() ? 0.f : m_new;
      alpha[k] = m_run[k] == m_new ? 1.0f : __builtin_amdgcn_exp2f((m_run[k] - m_ref[k]) * kLog2e);
      moved = moved || alpha[k] != 1.0f;
      m_run[k] = m_new;
    }
    if (__ballot(moved) != 0ull) {   // some head's maximum moved: scale what has been added so far
#pragma unroll
      for (int k = 0; k < NH; ++k) {
        lsum[k] *= alpha[k];
#pragma unroll
        for (int sg = 0; sg < 4; ++sg) zacc[k][sg] *= alpha[k];
      }
      // result rows 4 kg + q: heads 2 kg (q = 0, 1) and 2 kg + 1 (q = 2, 3); head h is slot h / 4 of the lanes with rg = h % 4
      const int src0 = 16 * ((2 * kg) & 3), src1 = 16 * ((2 * kg + 1) & 3);
      const float t00 = __shfl(alpha[0], src0, PIKV_WAVE), t01 = __shfl(alpha[NH - 1], src0, PIKV_WAVE);
      const float t10 = __shfl(alpha[0], src1, PIKV_WAVE), t11 = __shfl(alpha[NH - 1], src1, PIKV_WAVE);
      const float a0 = (kg >> 1) ? t01 : t00, a1 = (kg >> 1) ? t11 : t10;
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        C[d][0] *= a0; C[d][1] *= a0;
        C[d][2] *= a1; C[d][3] *= a1;
      }
    }
#pragma unroll
    for (int k = 0; k < NH; ++k)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        p4[k][j] = __builtin_amdgcn_exp2f((sc[k][j] - m_ref[k]) * kLog2e);
        lsum[k] += p4[k][j];
      }
    if constexpr (BOOK) {
      const int64_t tile = (t0 + n0) / kFTile;
      auto hb = [](float p) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)(p * kHalfScale)); };
#pragma unroll
      for (int k = 0; k < NH; ++k) {
        const uint2 ev = make_uint2(hb(p4[k][0]) | (hb(p4[k][1]) << 16), hb(p4[k][2]) | (hb(p4[k][3]) << 16));
        if constexpr (QF32) a.e16[(((int64_t)c * a.n_tiles + tile) * HK + g) * (rep * 16) + lane] = ev;
        else a.e16[((((int64_t)c * a.n_tiles + tile) * HK + g) * 2 + k) * 64 + lane] = ev;
        if (nl == 0 && row_on[k])
          a.tref[((int64_t)c * a.n_tiles + tile) * a.n_q_heads + g * rep + rg + 4 * k] = m_ref[k];
      }
    }

    // ---- weights and output product, two groups of 32 dimensions at a time ----
#pragma unroll
    for (int pp = 0; pp < 2; ++pp) {
      float2 s2[4], z2[4];   // scale and zero term of this pass's two groups, tokens tk + 4 j
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s2[j] = *reinterpret_cast<const float2*>(vscale + fused_vmeta_off(tk + 4 * j) + 8 * pp);
        z2[j] = *reinterpret_cast<const float2*>(vzterm + fused_vmeta_off(tk + 4 * j) + 8 * pp);
      }
#pragma unroll
      for (int sgl = 0; sgl < 2; ++sgl) {
        const int sg = 2 * pp + sgl;
#pragma unroll
        for (int k = 0; k < NH; ++k) {
          float hi[4], lo[4];
          float zsum = 0.f;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float scl = sgl == 0 ? s2[j].x : s2[j].y;
            const float zt = sgl == 0 ? z2[j].x : z2[j].y;
            const float w = p4[k][j] * scl;
            hi[j] = __uint_as_float(__float_as_uint(w) & 0xffff0000u);
            lo[j] = __uint_as_float(__float_as_uint(w - hi[j]) & 0xffff0000u);
            // the zero-point sum uses the SAME two-part value the matrix core multiplies with 128 + code
            zsum = fmaf(hi[j] + lo[j], zt, zsum);
          }
          zacc[k][sg] += zsum;
          if (row_on[k]) {
            const int h = rg + 4 * k;
            // operand order inside 8 tokens is {0,4,1,5,2,6,3,7}: tokens (k, k+4) share a dword
            uint32_t* rowh = reinterpret_cast<uint32_t*>(abuf + (sgl * 16 + 2 * h) * kFARow + wkg * 32) + qd;
            uint32_t* rowl = reinterpret_cast<uint32_t*>(abuf + (sgl * 16 + 2 * h + 1) * kFARow + wkg * 32) + qd;
            rowh[0] = (__float_as_uint(hi[0]) >> 16) | __float_as_uint(hi[1]);
            rowh[4] = (__float_as_uint(hi[2]) >> 16) | __float_as_uint(hi[3]);
            rowl[0] = (__float_as_uint(lo[0]) >> 16) | __float_as_uint(lo[1]);
            rowl[4] = (__float_as_uint(lo[2]) >> 16) | __float_as_uint(lo[3]);
          }
        }
      }
      wave_sync();   // the rows were written by other lanes of this wavefront
#pragma unroll
      for (int sgl = 0; sgl < 2; ++sgl) {
        const int sg = 2 * pp + sgl;
        const uint4* ap = reinterpret_cast<const uint4*>(a_row + sgl * a_gstep);
        const uint4 a1 = ap[0], a2 = ap[1];
#pragma unroll
        for (int dbl = 0; dbl < 2; ++dbl) {
          const int db = 2 * sg + dbl;
          const pikv_i32x2 tr = __builtin_amdgcn_ds_read_tr4_b64_v2i32(
              (pikv_i32x2 __attribute__((address_space(3)))*)(vcodes + (kg * 16 + i) * kFCodeRow + db * 8));
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const uint32_t u = Q::sym ? ((uint32_t)tr[half] ^ 0x88888888u) : (uint32_t)tr[half];
            const uint4 bb = make_uint4(and_or(u, kNib, kExp), and_or(u >> 4, kNib, kExp), and_or(u >> 8, kNib, kExp),
                                        and_or(u >> 12, kNib, kExp));
            C[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, half ? a2 : a1),
                                                            __builtin_bit_cast(pikv_bf16x8, bb), C[db], 0, 0, 0);
          }
        }
      }
      wave_sync();   // the rows are rewritten by the next pass / the next tile
    }
  }

  // ---- what the range leaves: (maximum, sum, unnormalised output) of each head ----
  wave_sync();
  float* const zl = reinterpret_cast<float*>(lds);   // [head][group]
  float ltot[NH];
#pragma unroll
  for (int k = 0; k < NH; ++k) {
    ltot[k] = group_sum_dpp(lsum[k], 16);
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) {
      const float z = group_sum_dpp(zacc[k][sg], 16);
      if (nl == 0) zl[(rg + 4 * k) * 4 + sg] = z;
    }
  }
  wave_sync();
  const int64_t pbase = ((int64_t)xr * a.n_caches + c) * a.n_q_heads + g * rep;
#pragma unroll
  for (int k = 0; k < NH; ++k)
    if (row_on[k] && nl == 0) {
      a.pstats[(pbase + rg + 4 * k) * 2] = m_run[k];
      a.pstats[(pbase + rg + 4 * k) * 2 + 1] = ltot[k];
    }
  // C: lane (dimension i, rows 4 kg + q): rows 2 h / 2 h + 1 are the two parts of head h
#pragma unroll
  for (int rr = 0; rr < 2; ++rr) {
    const int ho = 2 * kg + rr;
    if (ho >= rep) continue;
    float* o = a.partial + (pbase + ho) * 128;
#pragma unroll
    for (int db = 0; db < 8; ++db) o[db * 16 + i] = (C[db][2 * rr] + C[db][2 * rr + 1]) - zl[ho * 4 + (db >> 1)];
  }
}

// ---- the same pass over an 8-bit cache ----------------------------------------------------------
// Codes of one byte, a float scale (and zero point) per (token, kv head) or coarser, heads of 128
// dimensions, 2..8 kv heads, 1..8 bf16 query heads per kv head.  The plan is the 4-bit kernel's - a
// wavefront per kv head, 64-token tiles, K from memory into matrix-core operands, V through a private
// piece of LDS and ds_read_b64_tr_b8, running softmax, ranges merged by decode_finish_kernel - with
// these differences:
//  * A stored byte u (the code, or code + 128 for the symmetric scheme: one XOR per word) IS a bf16
//    number - integers up to 255 need eight significant bits - so it goes to the matrix cores as
//    itself (v_cvt_f32_ubyteN + v_cvt_pk_bf16_f32, three instructions per two codes): no nibble
//    split, no offset beyond the zero point.  score = s (sum q u - zz sum q), the two halves of the
//    head dimension accumulated apart, each with its own query sum taken off first.
//  * The A operand of the score product holds the query heads as rows (up to 8 of 16), so a result
//    lane holds FOUR heads of one token; lanes 32..63 (rows of no head) take over two of the four
//    16-token slices from lanes 0..31 (v_permlane32_swap), and every lane runs the softmax of four
//    heads x two neighbouring tokens.  Slice s of lane column n is token 4 n + s.
//  * One register set: the V codes of the next tile are asked for as soon as this tile's are staged,
//    the K codes as soon as this tile's scores are done (a tile is 16 KB per wavefront).
//  * Bookkeeping records: 16 bytes per lane - 2 tokens x 4 heads as halves - from every lane (5..8
//    query heads per kv head: 1 KB per tile and kv head) or from the lanes of heads 0..3 (512 B).
constexpr int k8CodeRow = 144;    // bytes per staged V row: 128 code bytes + 16 (bank spread, 16-byte aligned)
constexpr int k8VCodes = 0;                                    // [64 tokens][k8CodeRow]
constexpr int k8Meta = k8VCodes + kFTile * k8CodeRow;          // two sets of {K (scale, zz), V (scale, zz)} float2 per token
constexpr int k8MetaSet = 2 * kFTile * 8;
constexpr int k8ABuf = k8Meta + 2 * k8MetaSet;                 // [16 rows][kFARow]
constexpr int k8AZero = k8ABuf + 16 * kFARow;                  // 32 zero bytes
constexpr int k8WaveLds = (k8AZero + 32 + 255) & ~255;
static_assert(k8WaveLds * 8 <= 160 * 1024, "eight wavefronts per block fit the LDS of a compute unit");

struct Fused8Args {
  const void* k_codes;
  const void* k_scale;
  const void* k_zero;
  const void* v_codes;
  const void* v_scale;
  const void* v_zero;
  const void* q;            // bf16 (float32 for the QF32 kernels) [cache][n_q_heads][128]
  const int64_t* row_base;
  const int32_t* fill;
  float* partial;           // [range][cache][q head][128]
  float* pstats;            // [range][cache][q head][2]
  uint4* e16;               // [cache][tile][kv head][64 or 32 lanes]: 8 halves per lane
  float* tref;              // [cache][tile][q head]
  int64_t n_tiles;          // records per cache
  int64_t max_len;
  int n_caches;
  int n_kv_heads;
  int n_q_heads;
  int tokens_per_block;     // a multiple of 64
  float scale_qk;
  int group;                // elements per scale: a multiple of 128 that divides the row
  int blocks_per_range;     // each block takes n_kv_heads / blocks_per_range neighbouring kv heads
};

// four bytes of a word as bf16, in order: {b0, b1}, {b2, b3}
__device__ __forceinline__ uint2 bytes_to_bf16(uint32_t w) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 lo, hi;
  lo[0] = (float)(w & 0xffu);
  lo[1] = (float)((w >> 8) & 0xffu);
  hi[0] = (float)((w >> 16) & 0xffu);
  hi[1] = (float)(w >> 24);
  return make_uint2(__builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf2)),
                    __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf2)));
}

// QF32: float32 queries as two bf16 limbs, q = hi + lo to 2^-18 |q| (hi = the float rounded to bf16, lo = the
// rest rounded to bf16); both limbs are multiplied with the same converted codes into the same accumulators.
template <int SCHEME, bool BOOK, bool QF32 = false>
__global__ __launch_bounds__(512) void decode_fused_i8_kernel(Fused8Args a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 8, "8-bit schemes only");
  extern __shared__ __align__(16) unsigned char fused_lds[];
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  unsigned char* const lds = fused_lds + wv * k8WaveLds;
  unsigned char* const vcodes = lds + k8VCodes;
  unsigned char* const abuf = lds + k8ABuf;
  unsigned char* const azero = lds + k8AZero;

  const int c = blockIdx.x;
  const int xr = blockIdx.y / a.blocks_per_range;   // token range
  const int HK = a.n_kv_heads;
  const int nwb = blockDim.x >> 6;                  // wavefronts (kv heads) of this block
  const int g0 = (blockIdx.y % a.blocks_per_range) * nwb;
  const int g = g0 + wv;                            // this wavefront's kv head
  const int rep = a.n_q_heads / HK;
  const int64_t len = a.fill[c] < a.max_len ? (int64_t)a.fill[c] : a.max_len;
  const int64_t t0 = (int64_t)xr * a.tokens_per_block;
  if (t0 >= len) return;   // the merge skips ranges that hold no token
  const int span = (int)((t0 + a.tokens_per_block < len ? t0 + a.tokens_per_block : len) - t0);
  const int last = span - 1;

  // roles.  Score product: lane = (column nl: a token, k-slice rg: 16 dimensions of each half of the head);
  // result lane (nl, rg) holds heads 4 rg .. 4 rg + 3 of its token.  Softmax and weights: heads
  // hq0 .. hq0 + 3, tokens tp, tp + 1.  Output product: lane = (A row / dimension i, k-slice kg: 8 tokens).
  const int nl = lane & 15, rg = lane >> 4;
  const int i = nl, kg = rg;
  const int hq0 = 4 * (rg & 1);
  const int tp = 4 * nl + 2 * (rg >> 1);
  const int row_codes = HK * 128;                       // bytes per cached row in the code planes
  const int gpr = row_codes / a.group;                  // metadata entries per cached row
  const int64_t urow = a.row_base[c] + t0;
  const char* const kc = reinterpret_cast<const char*>(a.k_codes) + urow * row_codes + g * 128;
  const char* const vc = reinterpret_cast<const char*>(a.v_codes) + urow * row_codes + g * 128;

  if (lane < 8) reinterpret_cast<uint32_t*>(azero)[lane] = 0u;

  // metadata: thread e takes entry (token e / heads, head e % heads) of the next tile's rows and writes
  // it into the owning wavefront's piece of LDS; the barrier at the top of the next tile publishes it
  const int m_tok = threadIdx.x / nwb, m_hd = threadIdx.x - m_tok * nwb;
  unsigned char* const m_lds = fused_lds + m_hd * k8WaveLds + k8Meta;
  const int m_ent = ((g0 + m_hd) * 128) / a.group;
  const float* const ksb = reinterpret_cast<const float*>(a.k_scale) + urow * gpr + m_ent;
  const float* const kzb = reinterpret_cast<const float*>(a.k_zero) + urow * gpr + m_ent;
  const float* const vsb = reinterpret_cast<const float*>(a.v_scale) + urow * gpr + m_ent;
  const float* const vzb = reinterpret_cast<const float*>(a.v_zero) + urow * gpr + m_ent;

  // ---- queries: A rows = the kv head's query heads, k-step (half, o) = dimensions 64 half + 16 rg + 8 o .. + 7 ----
  uint4 aq[4], aql[QF32 ? 4 : 1];
  float qs0, qs1;   // sum of the head's query over the dimensions of half 0 / half 1 (lane's row nl)
  {
    const bool a_on = nl < rep;
    const int64_t qoff = ((int64_t)c * a.n_q_heads + g * rep + (a_on ? nl : 0)) * 128 + rg * 16;
    float part[2] = {0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t eo = qoff + (k >> 1) * 64 + (k & 1) * 8;
      if constexpr (QF32) {
        const float* qf = reinterpret_cast<const float*>(a.q) + eo;
        uint32_t hb[8], lb[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float f = a_on ? qf[e] : 0.f;
          hb[e] = bf16_limb_bits(f, 0);
          lb[e] = bf16_limb_bits(f, 1);
          part[k >> 1] += __uint_as_float(hb[e] << 16);
          part[k >> 1] += __uint_as_float(lb[e] << 16);
        }
        aq[k] = make_uint4(hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16), hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16));
        aql[k] = make_uint4(lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16), lb[4] | (lb[5] << 16), lb[6] | (lb[7] << 16));
      } else {
        uint4 d = make_uint4(0, 0, 0, 0);
        if (a_on) d = ld16(reinterpret_cast<const uint16_t*>(a.q) + eo);
        aq[k] = d;
        const uint32_t w[4] = {d.x, d.y, d.z, d.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          part[k >> 1] += __uint_as_float(w[e] << 16);
          part[k >> 1] += __uint_as_float(w[e] & 0xffff0000u);
        }
      }
    }
    part[0] += __shfl_xor(part[0], 16, PIKV_WAVE);
    part[0] += __shfl_xor(part[0], 32, PIKV_WAVE);
    part[1] += __shfl_xor(part[1], 16, PIKV_WAVE);
    part[1] += __shfl_xor(part[1], 32, PIKV_WAVE);
    qs0 = part[0];
    qs1 = part[1];
  }
  // ... of the four heads in this lane's result rows 4 rg .. 4 rg + 3 (rows past the heads: zero)
  float4 q0v, q1v;
  q0v.x = __shfl(qs0, 4 * rg + 0, PIKV_WAVE); q0v.y = __shfl(qs0, 4 * rg + 1, PIKV_WAVE);
  q0v.z = __shfl(qs0, 4 * rg + 2, PIKV_WAVE); q0v.w = __shfl(qs0, 4 * rg + 3, PIKV_WAVE);
  q1v.x = __shfl(qs1, 4 * rg + 0, PIKV_WAVE); q1v.y = __shfl(qs1, 4 * rg + 1, PIKV_WAVE);
  q1v.z = __shfl(qs1, 4 * rg + 2, PIKV_WAVE); q1v.w = __shfl(qs1, 4 * rg + 3, PIKV_WAVE);

  pikv_f32x4 C[8];
#pragma unroll
  for (int d = 0; d < 8; ++d) C[d] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
  float zacc[4] = {0.f, 0.f, 0.f, 0.f};
  float lsum[4] = {0.f, 0.f, 0.f, 0.f};
  float m_run[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) m_run[j] = -__builtin_inff();

  // A-operand piece of this lane in the output product: row i = (head i / 2, part i % 2), or the zero piece
  const bool arow_on = i < 2 * rep;
  const unsigned char* const a_row = arow_on ? abuf + i * kFARow + kg * 16 : azero;
  const int a_half = arow_on ? 64 : 0;   // bytes from the first 32 tokens of a row to the second

  uint4 rk[8], rv[8];
  float mks, mkz, mvs, mvz;
  auto clamp_row = [&](int tok) { return tok < last ? tok : last; };
  auto issue_meta = [&](int n0) {   // this thread's metadata entry of the tile that starts at n0
    const uint32_t mo = (uint32_t)(clamp_row(n0 + m_tok) * gpr);
    mks = ksb[mo];
    mvs = vsb[mo];
    mkz = 128.0f;
    mvz = 128.0f;
    if constexpr (!Q::sym) {
      mkz = kzb[mo];
      mvz = vzb[mo];
    }
  };
  auto stage_meta = [&](int set) {
    float2* const mb = reinterpret_cast<float2*>(m_lds + set * k8MetaSet);
    mb[m_tok] = make_float2(mks, mkz);
    mb[kFTile + m_tok] = make_float2(mvs, mvz);
  };
  auto issue_v = [&](int n0) {   // whole 128-byte rows: 8 tokens per instruction
#pragma unroll
    for (int k = 0; k < 8; ++k)
      rv[k] = ld16(vc + (uint32_t)(clamp_row(n0 + 8 * k + (lane >> 3)) * row_codes + (lane & 7) * 16));
  };
  auto issue_k = [&](int n0) {   // slice s: token 4 nl + s, the lane's 16 bytes of each half
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint32_t ro = (uint32_t)(clamp_row(n0 + 4 * nl + s) * row_codes + rg * 16);
      rk[2 * s] = ld16(kc + ro);
      rk[2 * s + 1] = ld16(kc + ro + 64);
    }
  };
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  auto pin_order = [] { asm volatile("" ::: "memory"); };
  auto both_halves_max = [](float v) {   // max over lanes l and l ^ 32
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
  };
  auto both_halves_sum = [](float v) {
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  };

  issue_meta(0);
  stage_meta(0);
  pin_order();
  issue_meta(kFTile);
  issue_v(0);
  pin_order();
  issue_k(0);
  pin_order();

  for (int n0 = 0; n0 < span; n0 += kFTile) {
    const int par = (n0 / kFTile) & 1;
    // one block barrier per tile: it publishes the metadata other wavefronts' threads wrote
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 8; ++k)
      *reinterpret_cast<uint4*>(vcodes + (8 * k + (lane >> 3)) * k8CodeRow + (lane & 7) * 16) = rv[k];
    stage_meta(par ^ 1);   // the NEXT tile's metadata, into the other set
    wave_sync();
    const float2* const kmeta = reinterpret_cast<const float2*>(lds + k8Meta + par * k8MetaSet);
    const float2* const vmeta = kmeta + kFTile;
    pin_order();
    issue_v(n0 + kFTile);
    issue_meta(n0 + 2 * kFTile);
    pin_order();

    // ---- scores: heads 4 rg .. 4 rg + 3 of tokens 4 nl + s ----
    float sc[4][4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      pikv_f32x4 pc0 = pikv_f32x4{0.f, 0.f, 0.f, 0.f}, pc1 = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const uint4 cw = rk[2 * s + half];
        const uint32_t w0 = Q::sym ? cw.x ^ 0x80808080u : cw.x, w1 = Q::sym ? cw.y ^ 0x80808080u : cw.y;
        const uint32_t w2 = Q::sym ? cw.z ^ 0x80808080u : cw.z, w3 = Q::sym ? cw.w ^ 0x80808080u : cw.w;
        const uint2 b0 = bytes_to_bf16(w0), b1 = bytes_to_bf16(w1), b2 = bytes_to_bf16(w2), b3 = bytes_to_bf16(w3);
        const uint4 bo0 = make_uint4(b0.x, b0.y, b1.x, b1.y), bo1 = make_uint4(b2.x, b2.y, b3.x, b3.y);
        pikv_f32x4& pc = half ? pc1 : pc0;
        pc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aq[2 * half]),
                                                     __builtin_bit_cast(pikv_bf16x8, bo0), pc, 0, 0, 0);
        pc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aq[2 * half + 1]),
                                                     __builtin_bit_cast(pikv_bf16x8, bo1), pc, 0, 0, 0);
        if constexpr (QF32) {
          pc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aql[2 * half]),
                                                       __builtin_bit_cast(pikv_bf16x8, bo0), pc, 0, 0, 0);
          pc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aql[2 * half + 1]),
                                                       __builtin_bit_cast(pikv_bf16x8, bo1), pc, 0, 0, 0);
        }
      }
      const float2 km = kmeta[4 * nl + s];
      const float f = km.x * a.scale_qk;
      sc[s][0] = f * (fmaf(-km.y, q0v.x, pc0[0]) + fmaf(-km.y, q1v.x, pc1[0]));
      sc[s][1] = f * (fmaf(-km.y, q0v.y, pc0[1]) + fmaf(-km.y, q1v.y, pc1[1]));
      sc[s][2] = f * (fmaf(-km.y, q0v.z, pc0[2]) + fmaf(-km.y, q1v.z, pc1[2]));
      sc[s][3] = f * (fmaf(-km.y, q0v.w, pc0[3]) + fmaf(-km.y, q1v.w, pc1[3]));
    }
    pin_order();
    issue_k(n0 + kFTile);
    pin_order();
    // lanes 32..63 take slices 2, 3 of lanes 0..31: afterwards every lane holds heads hq0 .. hq0 + 3 of
    // tokens tp (e0) and tp + 1 (e1)
    float e0[4], e1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      auto s02 = __builtin_amdgcn_permlane32_swap(__float_as_uint(sc[0][j]), __float_as_uint(sc[2][j]), false, false);
      auto s13 = __builtin_amdgcn_permlane32_swap(__float_as_uint(sc[1][j]), __float_as_uint(sc[3][j]), false, false);
      const bool head_on = hq0 + j < rep;
      e0[j] = (head_on && n0 + tp <= last) ? __uint_as_float(s02[0]) : -__builtin_inff();
      e1[j] = (head_on && n0 + tp + 1 <= last) ? __uint_as_float(s13[0]) : -__builtin_inff();
    }

    // ---- running softmax of the four heads ----
    float alpha[4], m_ref[4];
    bool moved = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float m_tile = both_halves_max(group_max_dpp(fmaxf(e0[j], e1[j]), 16));
      const float m_new = fmaxf(m_run[j], m_tile);
      m_ref[j] = m_new == -__builtin_inff() ? 0.f : m_new;
      alpha[j] = m_run[j] == m_new ? 1.0f : __builtin_amdgcn_exp2f((m_run[j] - m_ref[j]) * kLog2e);
      moved = moved || alpha[j] != 1.0f;
      m_run[j] = m_new;
    }
    if (__ballot(moved) != 0ull) {   // some head's maximum moved: scale what has been added so far
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        lsum[j] *= alpha[j];
        zacc[j] *= alpha[j];
      }
      // result rows 4 kg + q of the output product: heads 2 kg (q = 0, 1) and 2 kg + 1 (q = 2, 3); head h
      // is slot h % 4 of the lanes with rg % 2 == h / 4
      const int src = 16 * (kg >> 1);
      const float al0 = __shfl(alpha[0], src, PIKV_WAVE), al1 = __shfl(alpha[1], src, PIKV_WAVE);
      const float al2 = __shfl(alpha[2], src, PIKV_WAVE), al3 = __shfl(alpha[3], src, PIKV_WAVE);
      const float a0 = (kg & 1) ? al2 : al0, a1 = (kg & 1) ? al3 : al1;
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        C[d][0] *= a0; C[d][1] *= a0;
        C[d][2] *= a1; C[d][3] *= a1;
      }
    }
    float p0[4], p1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p0[j] = __builtin_amdgcn_exp2f((e0[j] - m_ref[j]) * kLog2e);
      p1[j] = __builtin_amdgcn_exp2f((e1[j] - m_ref[j]) * kLog2e);
      lsum[j] += p0[j] + p1[j];
    }
    if constexpr (BOOK) {
      const int64_t tile = (t0 + n0) / kFTile;
      auto hb = [](float p) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)(p * kHalfScale)); };
      const uint4 ev = make_uint4(hb(p0[0]) | (hb(p1[0]) << 16), hb(p0[1]) | (hb(p1[1]) << 16),
                                  hb(p0[2]) | (hb(p1[2]) << 16), hb(p0[3]) | (hb(p1[3]) << 16));
      float* const rrec = a.tref + ((int64_t)c * a.n_tiles + tile) * a.n_q_heads + g * rep;
      if (rep > 4) {
        a.e16[(((int64_t)c * a.n_tiles + tile) * HK + g) * 64 + lane] = ev;
      } else if (hq0 == 0) {
        a.e16[(((int64_t)c * a.n_tiles + tile) * HK + g) * 32 + 16 * (rg >> 1) + nl] = ev;
      }
      if (nl == 0 && rg < 2) {   // (one store of the eight maxima from lanes nl < 4 measured slower: 1053 vs 1040 us)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (hq0 + j < rep) rrec[hq0 + j] = m_ref[j];
      }
    }

    // ---- weights: p * scale of the token's V row as a bf16 high part and a bf16 remainder ----
    {
      const float2 vm0 = vmeta[tp], vm1 = vmeta[tp + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float w0 = p0[j] * vm0.x, w1 = p1[j] * vm1.x;
        const float h0 = __uint_as_float(__float_as_uint(w0) & 0xffff0000u);
        const float h1 = __uint_as_float(__float_as_uint(w1) & 0xffff0000u);
        const float l0 = __uint_as_float(__float_as_uint(w0 - h0) & 0xffff0000u);
        const float l1 = __uint_as_float(__float_as_uint(w1 - h1) & 0xffff0000u);
        // the zero-point sum uses the SAME two-part values the matrix core multiplies with the codes
        zacc[j] = fmaf(h0 + l0, vm0.y, zacc[j]);
        zacc[j] = fmaf(h1 + l1, vm1.y, zacc[j]);
        if (hq0 + j < rep) {
          unsigned char* const rowp = abuf + (2 * (hq0 + j)) * kFARow + tp * 2;
          *reinterpret_cast<uint32_t*>(rowp) = (__float_as_uint(h0) >> 16) | __float_as_uint(h1);
          *reinterpret_cast<uint32_t*>(rowp + kFARow) = (__float_as_uint(l0) >> 16) | __float_as_uint(l1);
        }
      }
    }
    wave_sync();   // the rows were written by other lanes of this wavefront

    // ---- output product: A rows (head, part) against 16 dimensions of 2 x 32 tokens ----
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const uint4 aw = *reinterpret_cast<const uint4*>(a_row + hf * a_half);
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        // source lane i points at token 32 hf + 8 kg + i / 2, dims 16 db + 8 (i % 2) .. + 7; result lane i
        // holds dimension 16 db + i of tokens 32 hf + 8 kg .. + 7
        const pikv_i32x2 tr = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (pikv_i32x2 __attribute__((address_space(3)))*)(vcodes + (32 * hf + 8 * kg + (i >> 1)) * k8CodeRow + db * 16 + 8 * (i & 1)));
        const uint32_t x0 = Q::sym ? ((uint32_t)tr[0] ^ 0x80808080u) : (uint32_t)tr[0];
        const uint32_t x1 = Q::sym ? ((uint32_t)tr[1] ^ 0x80808080u) : (uint32_t)tr[1];
        const uint2 b0 = bytes_to_bf16(x0), b1 = bytes_to_bf16(x1);
        C[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pikv_bf16x8, aw),
                                                        __builtin_bit_cast(pikv_bf16x8, make_uint4(b0.x, b0.y, b1.x, b1.y)),
                                                        C[db], 0, 0, 0);
      }
    }
  }

  // ---- what the range leaves: (maximum, sum, unnormalised output) of each head ----
  wave_sync();
  float* const zl = reinterpret_cast<float*>(lds);   // [head]: zero-point sums
  float ltot[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    ltot[j] = both_halves_sum(group_sum_dpp(lsum[j], 16));
    const float z = both_halves_sum(group_sum_dpp(zacc[j], 16));
    if (nl == 0 && rg < 2) zl[hq0 + j] = z;
  }
  wave_sync();
  const int64_t pbase = ((int64_t)xr * a.n_caches + c) * a.n_q_heads + g * rep;
  if (nl == 0 && rg < 2) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (hq0 + j < rep) {
        a.pstats[(pbase + hq0 + j) * 2] = m_run[j];
        a.pstats[(pbase + hq0 + j) * 2 + 1] = ltot[j];
      }
  }
  // C: lane (dimension i, rows 4 kg + q): rows 2 h / 2 h + 1 are the two parts of head h
#pragma unroll
  for (int rr = 0; rr < 2; ++rr) {
    const int ho = 2 * kg + rr;
    if (ho >= rep) continue;
    float* o = a.partial + (pbase + ho) * 128;
#pragma unroll
    for (int db = 0; db < 8; ++db) o[db * 16 + i] = (C[db][2 * rr] + C[db][2 * rr + 1]) - zl[ho];
  }
}

// out[c,h,:] = sum over ranges of partial * exp(m_range - M) / Z,  M = max of the ranges' maxima,
// Z = sum of their sums scaled alike.  One thread per output element; caches without a token give 0.
__global__ __launch_bounds__(256) void decode_finish_kernel(const float* __restrict__ partial,
                                                           const float* __restrict__ pstats,
                                                           const int32_t* __restrict__ fill, int64_t max_len,
                                                           int n_caches, int n_q_heads, int n_splits,
                                                           int tokens_per_block, float* __restrict__ out,
                                                           float* __restrict__ head_stats) {
  const int64_t per_cache = (int64_t)n_q_heads * 128;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_cache * n_caches) return;
  const int c = (int)(idx / per_cache);
  const int h = (int)((idx - (int64_t)c * per_cache) >> 7);
  const int64_t len = fill[c] < max_len ? (int64_t)fill[c] : max_len;
  const int64_t used = (len + tokens_per_block - 1) / tokens_per_block;
  const int lim = used < n_splits ? (int)used : n_splits;
  float M = -__builtin_inff();
  for (int sp = 0; sp < lim; ++sp) M = fmaxf(M, pstats[(((int64_t)sp * n_caches + c) * n_q_heads + h) * 2]);
  float Z = 0.f, s = 0.f;
  for (int sp = 0; sp < lim; ++sp) {
    const int64_t pi = ((int64_t)sp * n_caches + c) * n_q_heads + h;
    const float f = __builtin_amdgcn_exp2f((pstats[pi * 2] - M) * kLog2e);
    Z = fmaf(pstats[pi * 2 + 1], f, Z);
    s = fmaf(partial[(int64_t)sp * per_cache * n_caches + idx], f, s);
  }
  out[idx] = lim > 0 ? s / Z : 0.f;
  if (head_stats != nullptr && (idx & 127) == 0) {
    head_stats[((int64_t)c * n_q_heads + h) * 2] = M;
    head_stats[((int64_t)c * n_q_heads + h) * 2 + 1] = Z;
  }
}

// H2O bookkeeping from the halves the fused pass left: one wavefront per tile of 64 cached tokens.
//   acc[n] = acc[n] * decay + sum_h e[h,n] * exp(m_tile[h] - M[h]) / Z[h];  ts[n] = now
// with (M, Z) of every head as decode_finish_kernel merged them into head_stats [cache][q head][2].
__global__ __launch_bounds__(256) void decode_importance_kernel(const uint2* __restrict__ e16,
                                                               const float* __restrict__ tref,
                                                               const float* __restrict__ head_stats,
                                                               const int64_t* __restrict__ row_base,
                                                               const int32_t* __restrict__ fill, int64_t max_len,
                                                               int64_t n_tiles, int n_kv_heads, int n_q_heads,
                                                               float decay, float now, float* __restrict__ row_acc,
                                                               float* __restrict__ row_ts, int sets) {
  // sets = 1: one record of rep * 16 lanes per kv head (heads 0 .. rep - 1); sets = 2 (the two-set kernel with
  // 5 to 8 heads per kv head): two records of 64 lanes, heads 0..3 and 4..7
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.y;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t len = fill[c] < max_len ? (int64_t)fill[c] : max_len;
  if (tile * kFTile >= len) return;
  const int rep = n_q_heads / n_kv_heads;
  const int r = lane >> 4;
  // token of the tile this lane finishes: row-group j holds tokens 16 wkg + 4 j + q
  const int tok = 16 * ((lane >> 2) & 3) + 4 * r + (lane & 3);
  const int64_t n = tile * kFTile + tok;
  const int64_t row = row_base[c] + n;
  float val = 0.f;
  float acc0 = 0.f;
  if (row_acc != nullptr && n < len) acc0 = row_acc[row];
  if (row_acc != nullptr) {
    // everything the wavefront reads is asked for at once: the tile's halves, the heads' merged statistics
    // (decode_finish_kernel left them in head_stats), the tile's reference maxima, the accumulators
    uint2 hv[16];
    const int rec = sets == 2 ? 64 : rep * 16;        // lanes per record
    const uint2* ep = e16 + ((int64_t)c * n_tiles + tile) * n_kv_heads * sets * rec + lane;
#pragma unroll
    for (int gs = 0; gs < 16; ++gs) {
      hv[gs] = make_uint2(0, 0);
      if (gs < n_kv_heads * sets && (sets == 2 ? 4 * (gs & 1) + r : r) < rep) hv[gs] = ep[(int64_t)gs * rec];
    }
    float fac = 0.f;   // lane h: what turns a stored half of head h in this tile into a probability
    if (lane < n_q_heads) {
      const float2 mz = *reinterpret_cast<const float2*>(head_stats + ((int64_t)c * n_q_heads + lane) * 2);
      const float mt = tref[((int64_t)c * n_tiles + tile) * n_q_heads + lane];
      fac = __builtin_amdgcn_exp2f((mt - mz.x) * kLog2e) / (mz.y * kHalfScale);
    }
    float imp[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int gs = 0; gs < 16; ++gs) {   // (no early exit: the loop must unroll, or the records live in scratch memory)
      const int g = sets == 2 ? gs >> 1 : gs;
      const int hr = sets == 2 ? 4 * (gs & 1) + r : r;   // head of this lane's row group inside the kv head
      const float f = __shfl(fac, (gs < n_kv_heads * sets && hr < rep) ? g * rep + hr : 0, PIKV_WAVE);
      const uint2 v = hv[gs];   // zero beyond the last record
      imp[0] = fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(v.x & 0xffffu)), f, imp[0]);
      imp[1] = fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(v.x >> 16)), f, imp[1]);
      imp[2] = fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(v.y & 0xffffu)), f, imp[2]);
      imp[3] = fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(v.y >> 16)), f, imp[3]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      imp[j] += __shfl_xor(imp[j], 16, PIKV_WAVE);
      imp[j] += __shfl_xor(imp[j], 32, PIKV_WAVE);
    }
    val = r == 0 ? imp[0] : r == 1 ? imp[1] : r == 2 ? imp[2] : imp[3];
  }
  if (n < len) {
    if (row_acc != nullptr) {
      float acc = acc0;
      if (decay != 1.0f) acc = acc * decay;
      row_acc[row] = acc + val;
    }
    if (row_ts != nullptr) row_ts[row] = now;
  }
}

// The same for the records of the 8-bit pass: lane (nl, rg) of a record holds heads 4 (rg % 2) .. + 3 of
// tokens 4 nl + 2 (rg / 2) and the next one, two tokens x four heads as halves {token, token + 1} per
// head; with up to four query heads per kv head a record is the 32 lanes of heads 0..3 only.
__global__ __launch_bounds__(256) void decode_importance8_kernel(const uint4* __restrict__ e16,
                                                                const float* __restrict__ tref,
                                                                const float* __restrict__ head_stats,
                                                                const int64_t* __restrict__ row_base,
                                                                const int32_t* __restrict__ fill, int64_t max_len,
                                                                int64_t n_tiles, int n_kv_heads, int n_q_heads,
                                                                float decay, float now, float* __restrict__ row_acc,
                                                                float* __restrict__ row_ts) {
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.y;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t len = fill[c] < max_len ? (int64_t)fill[c] : max_len;
  if (tile * kFTile >= len) return;
  const int rep = n_q_heads / n_kv_heads;
  const int nl = lane & 15, rg = lane >> 4;
  const int hq0 = 4 * (rg & 1);
  const int64_t n = tile * kFTile + 4 * nl + 2 * (rg >> 1);   // first of this lane's two tokens
  const int64_t row = row_base[c] + n;
  const bool writer = hq0 == 0;
  float acc0 = 0.f, acc1 = 0.f;
  if (row_acc != nullptr && writer) {
    if (n < len) acc0 = row_acc[row];
    if (n + 1 < len) acc1 = row_acc[row + 1];
  }
  float i0 = 0.f, i1 = 0.f;
  if (row_acc != nullptr) {
    const int lanes = rep > 4 ? 64 : 32;
    const bool have = rep > 4 || hq0 == 0;
    const uint4* ep = e16 + ((int64_t)c * n_tiles + tile) * n_kv_heads * lanes + (rep > 4 ? lane : 16 * (rg >> 1) + nl);
    uint4 hv[8];
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      hv[g] = make_uint4(0, 0, 0, 0);
      if (g < n_kv_heads && have) hv[g] = ep[(int64_t)g * lanes];
    }
    float fac = 0.f;   // lane h: what turns a stored half of head h in this tile into a probability
    if (lane < n_q_heads) {
      const float2 mz = *reinterpret_cast<const float2*>(head_stats + ((int64_t)c * n_q_heads + lane) * 2);
      const float mt = tref[((int64_t)c * n_tiles + tile) * n_q_heads + lane];
      fac = __builtin_amdgcn_exp2f((mt - mz.x) * kLog2e) / (mz.y * kHalfScale);
    }
    auto lo = [](uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu)); };
    auto hi = [](uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); };
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      if (g >= n_kv_heads) break;
      const uint32_t w[4] = {hv[g].x, hv[g].y, hv[g].z, hv[g].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int h = g * rep + hq0 + j;
        const float f = __shfl(fac, hq0 + j < rep ? h : 0, PIKV_WAVE);
        const float ff = hq0 + j < rep ? f : 0.f;
        i0 = fmaf(lo(w[j]), ff, i0);
        i1 = fmaf(hi(w[j]), ff, i1);
      }
    }
    // heads 4..7 of the same tokens sit 16 lanes up
    i0 += __shfl_xor(i0, 16, PIKV_WAVE);
    i1 += __shfl_xor(i1, 16, PIKV_WAVE);
  }
  if (writer) {
    if (row_acc != nullptr) {
      if (decay != 1.0f) {
        acc0 = acc0 * decay;
        acc1 = acc1 * decay;
      }
      if (n < len) row_acc[row] = acc0 + i0;
      if (n + 1 < len) row_acc[row + 1] = acc1 + i1;
    }
    if (row_ts != nullptr) {
      if (n < len) row_ts[row] = now;
      if (n + 1 < len) row_ts[row + 1] = now;
    }
  }
}

}  // namespace pikv

using namespace pikv;

namespace pikv {

// Cached tokens per block of the fused pass: a block is n_kv_heads wavefronts and as many pieces of
// LDS, so a compute unit holds 8 / n_kv_heads of them (at most 8 wavefronts' pieces fit); the longest
// range that still fills the chip wins, and it is never shorter than `min_tpb` (the workspace is
// laid out for that many ranges).
// (4-bit rows as two blocks of half the kv heads per token range measured slower - 662 vs 632 us at 8 kv
// heads: the halves of a 128-byte line then belong to different blocks and the metadata is fetched 1.75 x.)
static int fused_groups(int n_kv_heads) { (void)n_kv_heads; return 1; }
// the 8-bit pass: its wavefronts share no code lines (a kv head's 128 bytes of a row are a line of their own)
static int fused8_blocks_per_range(int n_kv_heads) { return (n_kv_heads == 8 || n_kv_heads == 6) ? 2 : 1; }

int fused_tokens_per_block(int n_caches, int n_kv_heads, int64_t max_len, int min_tpb) {
  const int groups = fused_groups(n_kv_heads);
  int per_cu = 8 / (n_kv_heads / groups);
  if (per_cu < 1) per_cu = 1;
  const int64_t resident = 256 * (int64_t)per_cu / groups;
  int best = 0;
  double best_eff = -1.0;
  for (int tpb = 8192; tpb >= 128 && tpb >= min_tpb; tpb >>= 1) {
    const int64_t blocks = (int64_t)n_caches * ((max_len + tpb - 1) / tpb);
    const int64_t rounds = (blocks + resident - 1) / resident;
    const double eff = rounds > 0 ? (double)blocks / (double)(rounds * resident) : 0.0;
    if (eff >= 0.85) return tpb;
    if (eff > best_eff) {
      best_eff = eff;
      best = tpb;
    }
  }
  return best > 0 ? best : (min_tpb > 128 ? min_tpb : 128);
}

// Which calls take the one-pass form (measured against the two-kernel forms at 64 caches x 32768 tokens,
// one process, alternating).  4-bit: without bookkeeping every geometry from 2 kv heads on (8 kv x 32 q heads
// 625 -> 502 us, 4 x 16: 333 -> 266, 6 x 24: 499 -> 418, 2 x 8: 194 -> 177; 1 x 4: 122 vs 128, left alone);
// with bookkeeping only four query heads per kv head on at least 3 kv heads (3 x 12: 306 -> 297,
// 6 x 24: 552 -> 537, 8 x 32: 660-680 -> 643 - the halves cost the pass 0.1 ms, see the top of this file; with
// fewer query heads per kv head the float rows of the two-kernel form are the smaller exchange).
// 4-bit, two operand sets, with / without bookkeeping: float32 queries 8 kv x 32 q heads 919 -> 674 / 887 -> 537 us,
// 6 x 24: 738 -> 540 / 664 -> 446, 4 x 16: 470 -> 371 / 426 -> 281, 3 x 12: 399 -> 293 / 357 -> 236, 2 x 8 without
// bookkeeping 261 -> 210, 8 x 16 without bookkeeping 847 -> 554; bf16, 5 to 8 heads per kv head: 8 x 64
// 1040 -> 741 / 873 -> 608, 8 x 40: 970 -> 726 / 807 -> 592, 4 x 28: 481 -> 401 / 420 -> 312; 2 kv heads are left
// on the two-kernel form (2 x 16 bf16 without bookkeeping: 233 vs 241 us).
// 8-bit: everything it can hold, with / without bookkeeping - 8 kv x 64 q heads 1225 -> 1032 / 1148 -> 788 us,
// 8 x 32: 1107 -> 956 / 1031 -> 786, 8 x 16: 1053 -> 962 / 981 -> 779, 6 x 24: 972 -> 743 / 898 -> 580,
// 4 x 16: 619 -> 516 / 541 -> 391, 3 x 12: 519 -> 392 / 442 -> 304, 2 x 8: 361 -> 292 / 297 -> 244,
// 8 x 8 without bookkeeping 826 -> 777 (with it the records of one head per kv head do not fit the workspace
// piece the float scores would take: two-kernel form, 853 us).
bool decode_fused_serves(int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim, int q_dtype, bool bookkeeping) {
  const bool eight = scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM;
  if (head_dim != 128 || !(q_dtype == PIKV_BF16 || q_dtype == PIKV_F32)) return false;
  (void)eight;
  if (n_kv_heads < 2 || n_kv_heads > 8 || n_q_heads % n_kv_heads != 0) return false;
  const int rep = n_q_heads / n_kv_heads;
  if (scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM) {
    // a scale per (token, kv head) or coarser; with bookkeeping the records must fit where the float scores would
    if (group < 128 || group % 128 != 0 || (n_kv_heads * 128) % group != 0) return false;
    if (bookkeeping) return rep >= 2 && rep <= 8;
    return rep >= 1 && rep <= 8;
  }
  if (group != 32) return false;
  // two operand sets: the limbs of four float32 heads, or eight bf16 heads
  if (q_dtype == PIKV_F32) return bookkeeping ? (rep == 4 && n_kv_heads >= 3) : rep <= 4;
  if (rep >= 5 && rep <= 8) return n_kv_heads >= 3;
  if (bookkeeping) return rep == 4 && n_kv_heads >= 3;
  return rep >= 1 && rep <= 4;
}

// Enqueues the fused pass, the merge of the ranges and (when row_acc or row_ts is given) the H2O
// bookkeeping.  e16 / tref / pstats / partial are workspace pieces sized by the caller, with
// n_tiles = ceil(max_len / 64) + 1 (a spare record per cache) and splits = ceil(max_len / tokens_per_block):
//   e16     n_caches * n_tiles * n_q_heads * 128 bytes       tref   n_caches * n_tiles * n_q_heads floats
//   pstats  splits * n_caches * n_q_heads * 2 floats          partial splits * n_caches * n_q_heads * 128 floats
int decode_fused_launch(const void* k_codes, const void* k_scale, const void* k_zero, const void* v_codes,
                        const void* v_scale, const void* v_zero, int scheme, int group, int n_kv_heads, int n_q_heads,
                        const void* q, int q_dtype, float scale_qk, const int64_t* cache_row_base, const int32_t* cache_fill,
                        int n_caches, int64_t max_len, int tokens_per_block, float decay, float now, float* row_acc,
                        float* row_ts, float* out, void* e16, float* tref, float* pstats, float* partial,
                        float* head_stats, hipStream_t st) {
  // one spare record per cache for the one-set 4-bit kernel (it walks tiles in pairs); the others touch no tile past a range's end
  const int64_t n_tiles = (max_len + kFTile - 1) / kFTile + ((q_dtype == PIKV_F32 || n_q_heads > 4 * n_kv_heads) ? 0 : 1);
  const int64_t splits = (max_len + tokens_per_block - 1) / tokens_per_block;
  if (splits > 65535 || (tokens_per_block & 127) != 0) return PIKV_ERR_SHAPE;
  const bool book = row_acc != nullptr || row_ts != nullptr;
  if (q_dtype != PIKV_BF16 && q_dtype != PIKV_F32) return PIKV_ERR_UNSUPPORTED;
  if (scheme == PIKV_Q_I8_SYM || scheme == PIKV_Q_I8_ASYM) {
    const int64_t n_tiles8 = (max_len + kFTile - 1) / kFTile;   // this pass never touches a tile past a range's end
    Fused8Args a8{k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, q, cache_row_base, cache_fill, partial, pstats,
                  reinterpret_cast<uint4*>(e16), tref, n_tiles8, max_len, n_caches, n_kv_heads, n_q_heads,
                  tokens_per_block, scale_qk, group,
                  splits * fused8_blocks_per_range(n_kv_heads) <= 65535 ? fused8_blocks_per_range(n_kv_heads) : 1};
    const dim3 grid8((unsigned)n_caches, (unsigned)(splits * a8.blocks_per_range));
    const dim3 block8((unsigned)(n_kv_heads / a8.blocks_per_range * 64));
    const size_t lds8 = (size_t)(n_kv_heads / a8.blocks_per_range) * k8WaveLds;
    const bool wr8 = row_acc != nullptr;
#define PIKV_FUSED8(S, F)                                                                                   \
  do {                                                                                                      \
    if (wr8) hipLaunchKernelGGL((decode_fused_i8_kernel<S, true, F>), grid8, block8, lds8, st, a8);         \
    else hipLaunchKernelGGL((decode_fused_i8_kernel<S, false, F>), grid8, block8, lds8, st, a8);            \
  } while (0)
    const bool qf = q_dtype == PIKV_F32;
    if (scheme == PIKV_Q_I8_SYM) {
      if (qf) PIKV_FUSED8(PIKV_Q_I8_SYM, true);
      else PIKV_FUSED8(PIKV_Q_I8_SYM, false);
    } else {
      if (qf) PIKV_FUSED8(PIKV_Q_I8_ASYM, true);
      else PIKV_FUSED8(PIKV_Q_I8_ASYM, false);
    }
#undef PIKV_FUSED8
    PIKV_CHECK_LAUNCH();
    const int64_t total8 = (int64_t)n_caches * n_q_heads * 128;
    hipLaunchKernelGGL(decode_finish_kernel, dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0, st, partial, pstats,
                       cache_fill, max_len, n_caches, n_q_heads, (int)splits, tokens_per_block, out, head_stats);
    if (book)
      hipLaunchKernelGGL(decode_importance8_kernel, dim3((unsigned)((n_tiles8 + 3) / 4), (unsigned)n_caches), dim3(256), 0,
                         st, reinterpret_cast<const uint4*>(e16), tref, head_stats, cache_row_base, cache_fill, max_len,
                         n_tiles8, n_kv_heads, n_q_heads, decay, now, row_acc, row_ts);
    PIKV_CHECK_LAUNCH();
    return PIKV_OK;
  }
  FusedArgs a{k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, q, cache_row_base, cache_fill, partial, pstats,
              reinterpret_cast<uint2*>(e16), tref, n_tiles, max_len, n_caches, n_kv_heads, n_q_heads, tokens_per_block,
              scale_qk, fused_groups(n_kv_heads)};
  const dim3 grid((unsigned)n_caches, (unsigned)(splits * a.groups));
  const dim3 block((unsigned)(n_kv_heads / a.groups * 64));
  const size_t lds = (size_t)(n_kv_heads / a.groups) * kFWaveLds;
  const bool wr = row_acc != nullptr;
  const int rep4 = n_q_heads / n_kv_heads;
  const bool qf = q_dtype == PIKV_F32;
  const bool wide = qf || rep4 > 4;   // two operand sets: float32 limbs, or 5 to 8 heads per kv head
  if (wide ? (qf ? (rep4 > 4 || (wr && rep4 != 4)) : rep4 > 8) : (wr && rep4 != 4)) return PIKV_ERR_UNSUPPORTED;
#define PIKV_FUSED(S)                                                                                   \
  do {                                                                                                  \
    if (wide && qf && wr) hipLaunchKernelGGL((decode_fused_i4w_kernel<S, true, true>), grid, block, lds, st, a);        \
    else if (wide && qf) hipLaunchKernelGGL((decode_fused_i4w_kernel<S, false, true>), grid, block, lds, st, a);        \
    else if (wide && wr) hipLaunchKernelGGL((decode_fused_i4w_kernel<S, true, false>), grid, block, lds, st, a);        \
    else if (wide) hipLaunchKernelGGL((decode_fused_i4w_kernel<S, false, false>), grid, block, lds, st, a);             \
    else if (wr) hipLaunchKernelGGL((decode_fused_i4_kernel<S, true>), grid, block, lds, st, a);        \
    else hipLaunchKernelGGL((decode_fused_i4_kernel<S, false>), grid, block, lds, st, a);               \
  } while (0)
  if (scheme == PIKV_Q_I4_ASYM) PIKV_FUSED(PIKV_Q_I4_ASYM);
  else PIKV_FUSED(PIKV_Q_I4_SYM);
#undef PIKV_FUSED
  PIKV_CHECK_LAUNCH();
  const int64_t total = (int64_t)n_caches * n_q_heads * 128;
  hipLaunchKernelGGL(decode_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, partial, pstats,
                     cache_fill, max_len, n_caches, n_q_heads, (int)splits, tokens_per_block, out, head_stats);
  if (book)
    hipLaunchKernelGGL(decode_importance_kernel, dim3((unsigned)((n_tiles + 3) / 4), (unsigned)n_caches), dim3(256), 0,
                       st, reinterpret_cast<const uint2*>(e16), tref, head_stats, cache_row_base, cache_fill, max_len,
                       n_tiles, n_kv_heads, n_q_heads, decay, now, row_acc, row_ts, (wide && !qf) ? 2 : 1);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

}  // namespace pikv
