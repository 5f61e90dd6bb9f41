// The decode read over a 4-bit cache as ONE pass: scores, running softmax and attention
// output in the same kernel, so that no score matrix ever exists in memory.
//
// Replaces, for one new token per sequence, the reference's
//   attention_scores = matmul(q, k^T) / sqrt(dh); probs = softmax(scores); out = matmul(probs, v)
// (core/single/pikv_attention.py:123,163,188) over the dequantised cache, and feeds
// H2OScheduler.update_attention_scores (core/single/cache_scheduling.py:69-73).
//
// Served here: 4-bit codes in groups of 32 (half scale / zero point), heads of 128 dimensions,
// 1..8 kv heads, 1..4 query heads per kv head, bf16 queries.  Everything else keeps the
// two-kernel forms of read_path.hip / attend.hip.
//
// Division of labour: a WAVEFRONT owns one kv head of one token range of one cache and walks it
// in tiles of 64 cached tokens - its K codes go straight from memory into matrix-core operands,
// its V codes through a wavefront-private piece of LDS (they are needed transposed), its scores
// never leave registers: the lane that receives the score of (head r, token t) from the
// matrix core is the lane that turns it into the weight rows of the second product.  Nothing is
// shared between the wavefronts of a block, so the tile loop has no block barrier; a block is
// the kv heads of one token range only so that whole cached rows are in flight together.
// Two tiles are on their way from memory per wavefront (two register sets).
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
// output never sees the halves.
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
                                                               float* __restrict__ row_ts) {
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
    uint2 hv[8];
    const uint2* ep = e16 + ((int64_t)c * n_tiles + tile) * n_kv_heads * (rep * 16) + lane;
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      hv[g] = make_uint2(0, 0);
      if (g < n_kv_heads && r < rep) hv[g] = ep[(int64_t)g * (rep * 16)];
    }
    float fac = 0.f;   // lane h: what turns a stored half of head h in this tile into a probability
    if (lane < n_q_heads) {
      const float2 mz = *reinterpret_cast<const float2*>(head_stats + ((int64_t)c * n_q_heads + lane) * 2);
      const float mt = tref[((int64_t)c * n_tiles + tile) * n_q_heads + lane];
      fac = __builtin_amdgcn_exp2f((mt - mz.x) * kLog2e) / (mz.y * kHalfScale);
    }
    float imp[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      if (g >= n_kv_heads) break;
      const float f = __shfl(fac, r < rep ? g * rep + r : 0, PIKV_WAVE);
      const uint2 v = hv[g];
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

}  // namespace pikv

using namespace pikv;

namespace pikv {

// Cached tokens per block of the fused pass: a block is n_kv_heads wavefronts and as many pieces of
// LDS, so a compute unit holds 8 / n_kv_heads of them (at most 8 wavefronts' pieces fit); the longest
// range that still fills the chip wins, and it is never shorter than `min_tpb` (the workspace is
// laid out for that many ranges).
// Rows of 8 (6) kv heads go as two blocks of 4 (3) wavefronts per token range: two independent blocks per
// compute unit fill each other's waits, where one block of eight wavefronts meets at one barrier per tile.
static int fused_groups(int n_kv_heads) { (void)n_kv_heads; return 1; }

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
// one process, alternating): without bookkeeping every geometry from 2 kv heads on (8 kv x 32 q heads
// 625 -> 524 us, 4 x 16: 333 -> 266, 6 x 24: 499 -> 418, 2 x 8: 194 -> 177; 1 x 4: 122 vs 128, left alone);
// with bookkeeping only four query heads per kv head on at least 3 kv heads (3 x 12: 306 -> 297,
// 6 x 24: 552 -> 537, 8 x 32: 675 vs 677 - the halves cost the pass 0.1 ms, see the kernel's comment; with
// fewer query heads per kv head the float rows of the two-kernel form are the smaller exchange).
bool decode_fused_serves(int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim, int q_dtype, bool bookkeeping) {
  if (scheme != PIKV_Q_I4_ASYM && scheme != PIKV_Q_I4_SYM) return false;
  if (group != 32 || head_dim != 128 || q_dtype != PIKV_BF16) return false;
  if (n_kv_heads < 2 || n_kv_heads > 8 || n_q_heads % n_kv_heads != 0) return false;
  const int rep = n_q_heads / n_kv_heads;
  if (bookkeeping) return rep == 4 && n_kv_heads >= 3;
  return rep >= 1 && rep <= 4;
}

// Enqueues the fused pass, the merge of the ranges and (when row_acc or row_ts is given) the H2O
// bookkeeping.  e16 / tref / pstats / partial are workspace pieces sized by the caller, with
// n_tiles = ceil(max_len / 64) + 1 (a spare record per cache) and splits = ceil(max_len / tokens_per_block):
//   e16     n_caches * n_tiles * n_q_heads * 128 bytes       tref   n_caches * n_tiles * n_q_heads floats
//   pstats  splits * n_caches * n_q_heads * 2 floats          partial splits * n_caches * n_q_heads * 128 floats
int decode_fused_launch(const void* k_codes, const void* k_scale, const void* k_zero, const void* v_codes,
                        const void* v_scale, const void* v_zero, int scheme, int n_kv_heads, int n_q_heads,
                        const void* q, float scale_qk, const int64_t* cache_row_base, const int32_t* cache_fill,
                        int n_caches, int64_t max_len, int tokens_per_block, float decay, float now, float* row_acc,
                        float* row_ts, float* out, void* e16, float* tref, float* pstats, float* partial,
                        float* head_stats, hipStream_t st) {
  const int64_t n_tiles = (max_len + kFTile - 1) / kFTile + 1;   // one spare record per cache
  const int64_t splits = (max_len + tokens_per_block - 1) / tokens_per_block;
  if (splits > 65535 || (tokens_per_block & 127) != 0) return PIKV_ERR_SHAPE;
  const bool book = row_acc != nullptr || row_ts != nullptr;
  FusedArgs a{k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, q, cache_row_base, cache_fill, partial, pstats,
              reinterpret_cast<uint2*>(e16), tref, n_tiles, max_len, n_caches, n_kv_heads, n_q_heads, tokens_per_block,
              scale_qk, fused_groups(n_kv_heads)};
  const dim3 grid((unsigned)n_caches, (unsigned)(splits * a.groups));
  const dim3 block((unsigned)(n_kv_heads / a.groups * 64));
  const size_t lds = (size_t)(n_kv_heads / a.groups) * kFWaveLds;
  const bool wr = row_acc != nullptr;
  if (wr && n_q_heads != 4 * n_kv_heads) return PIKV_ERR_UNSUPPORTED;
#define PIKV_FUSED(S)                                                                                   \
  do {                                                                                                  \
    if (wr) hipLaunchKernelGGL((decode_fused_i4_kernel<S, true>), grid, block, lds, st, a);             \
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
                       n_tiles, n_kv_heads, n_q_heads, decay, now, row_acc, row_ts);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

}  // namespace pikv
