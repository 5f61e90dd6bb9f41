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
//  * attend_mfma_i4_kernel - 4-bit codes, groups of 32, head_dim 128, bf16-exact:
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
constexpr int kAttTokensPerBlock = 2048;

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
};

__device__ __forceinline__ float prob_of(float s, float mx, float rz, bool normalise) {
  return normalise ? __builtin_amdgcn_exp2f((s - mx) * 1.4426950408889634f) * rz : s;
}

// ---- vector-unit form --------------------------------------------------------------
// RP query heads of every kv head per pass (blockIdx.z selects the pass).
template <int SCHEME, int RP>
__global__ __launch_bounds__(256) void attend_valu_kernel(AttendArgs a) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  __shared__ float red[256 * EPL];
  const int c = blockIdx.y;
  const int64_t len = a.fill[c];
  const int64_t t0 = (int64_t)blockIdx.x * kAttTokensPerBlock;
  const int64_t t1 = (t0 + kAttTokensPerBlock < len) ? t0 + kAttTokensPerBlock : len;
  const int rep = a.n_q_heads / a.n_kv_heads;
  const int r0 = blockIdx.z * RP;
  const int D = a.n_kv_heads * a.head_dim;
  const int lanes_per_row = D / EPL;
  const int lanes_per_head = a.head_dim / EPL;
  const int groups_per_row = D / a.group;
  const int tok_per_step = 256 / lanes_per_row;
  const int part = threadIdx.x % lanes_per_row;
  const int tok_in_step = threadIdx.x / lanes_per_row;
  const int kvh = part / lanes_per_head;
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
  for (int64_t n = t0 + tok_in_step; n < t1; n += tok_per_step) {
    const int64_t row = base_row + n;
    const uint4 v = ld16(reinterpret_cast<const char*>(a.codes) + (row * lanes_per_row + part) * 16);
    const int64_t mi = row * groups_per_row + (part * EPL) / a.group;
    const float sc = load_meta<SCHEME>(a.scale, mi);
    const float zu = (Q::sym ? 0.f : load_meta<SCHEME>(a.zero, mi)) - (float)Q::qmin;
    float cf[EPL];
    unpack_codes_unsigned<SCHEME>(v, cf);
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      const float w = prob_of(srow[r][n], mx[r], rz[r], normalise) * sc;
      zacc[r] = fmaf(w, zu, zacc[r]);
#pragma unroll
      for (int j = 0; j < EPL; ++j) acc[r][j] = fmaf(w, cf[j], acc[r][j]);
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

// ---- matrix-core form -----------------------------------------------------------------
typedef int pikv_i32x2 __attribute__((ext_vector_type(2)));

static size_t attend_mfma_lds_bytes(int n_kv_heads) {
  // codes [64 tokens][n_kv_heads*64 + 8 bytes]; scale and zero + bias as float
  // [kv head][group of 32][64 tokens + 8]
  return (size_t)kAttTile * (n_kv_heads * 64 + 8) + 2 * (size_t)n_kv_heads * 4 * (kAttTile + 8) * sizeof(float);
}

template <int SCHEME>
__global__ __launch_bounds__(256) void attend_mfma_i4_kernel(AttendArgs a) {
  using Q = QScheme<SCHEME>;
  static_assert(Q::bits == 4, "4-bit schemes only");
  constexpr int kMaxHeadsPerWave = 2;  // n_kv_heads <= 8
  constexpr int MS = kAttTile + 8;     // floats per (kv head, group) row of the metadata
  extern __shared__ __align__(16) unsigned char att_lds[];
  const int HK = a.n_kv_heads;
  const int RS = HK * 64 + 8;          // bytes per token row of staged codes
  unsigned char* lcodes = att_lds;
  float* lscale = reinterpret_cast<float*>(att_lds + (size_t)kAttTile * RS);
  float* lzterm = lscale + HK * 4 * MS;

  const int c = blockIdx.y;
  const int64_t len = a.fill[c];
  const int64_t t0 = (int64_t)blockIdx.x * kAttTokensPerBlock;
  const int64_t t1 = (t0 + kAttTokensPerBlock < len) ? t0 + kAttTokensPerBlock : len;
  const int rep = a.n_q_heads / a.n_kv_heads;  // <= 8
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int i = lane & 15;   // A: row (head r = i/2, part h = i%2); B/C: dimension inside a block of 16
  const int kg = lane >> 4;  // 16 tokens of the tile
  const int r = i >> 1;
  const bool lo_row = (i & 1) != 0;
  const bool row_on = r < rep;
  const bool normalise = a.head_stats != nullptr;
  const float zbias = 128.0f - (float)Q::qmin;
  const int64_t base_row = a.row_base[c];
  const int lanes_per_row = HK * 4;

  pikv_f32x4 C[kMaxHeadsPerWave][8];
  float zacc[kMaxHeadsPerWave][4];
  float mx[kMaxHeadsPerWave], rz[kMaxHeadsPerWave];
  const float* srow[kMaxHeadsPerWave];
#pragma unroll
  for (int hs = 0; hs < kMaxHeadsPerWave; ++hs) {
    const int g = wave + 4 * hs;
    const int hq = (g < HK && row_on) ? g * rep + r : 0;
    srow[hs] = a.scores + ((int64_t)c * a.n_q_heads + hq) * a.score_stride;
    mx[hs] = 0.f;
    rz[hs] = 1.f;
    if (normalise) {
      mx[hs] = a.head_stats[((int64_t)c * a.n_q_heads + hq) * 2];
      rz[hs] = 1.0f / a.head_stats[((int64_t)c * a.n_q_heads + hq) * 2 + 1];
    }
#pragma unroll
    for (int d = 0; d < 8; ++d) C[hs][d] = pikv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sg = 0; sg < 4; ++sg) zacc[hs][sg] = 0.f;
  }

  for (int64_t n0 = t0; n0 < t1; n0 += kAttTile) {
    __syncthreads();  // the previous tile has been consumed
    // stage the codes of 64 tokens as they are (rows past the fill as zeros)
    for (int ch = threadIdx.x; ch < kAttTile * lanes_per_row; ch += 256) {
      const int tok = ch / lanes_per_row, off = ch - tok * lanes_per_row;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (n0 + tok < t1) v = ld16(reinterpret_cast<const char*>(a.codes) + ((base_row + n0 + tok) * lanes_per_row + off) * 16);
      uint2* dst = reinterpret_cast<uint2*>(lcodes + tok * RS + off * 16);  // 8-byte aligned only
      dst[0] = make_uint2(v.x, v.y);
      dst[1] = make_uint2(v.z, v.w);
    }
    // scale and zero + bias of every (token, kv head, group), token-minor
    for (int ch = threadIdx.x; ch < kAttTile * HK; ch += 256) {
      const int tok = ch / HK, hd = ch - tok * HK;
      uint2 sv = make_uint2(0, 0), zv = make_uint2(0, 0);
      if (n0 + tok < t1) {
        const int64_t mi = (base_row + n0 + tok) * lanes_per_row + hd * 4;
        sv = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(a.scale) + mi);
        if constexpr (!Q::sym) zv = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(a.zero) + mi);
      }
      const uint32_t sw[2] = {sv.x, sv.y}, zw[2] = {zv.x, zv.y};
#pragma unroll
      for (int sg = 0; sg < 4; ++sg) {
        const float s = (float)__builtin_bit_cast(_Float16, (uint16_t)(sw[sg >> 1] >> (16 * (sg & 1))));
        const float z = (float)__builtin_bit_cast(_Float16, (uint16_t)(zw[sg >> 1] >> (16 * (sg & 1))));
        lscale[(hd * 4 + sg) * MS + tok] = s;
        lzterm[(hd * 4 + sg) * MS + tok] = z + zbias;
      }
    }
    __syncthreads();

#pragma unroll
    for (int hs = 0; hs < kMaxHeadsPerWave; ++hs) {
      const int g = wave + 4 * hs;
      if (g < HK) {  // uniform
        // probabilities of this lane's head for its 16 tokens
        float p[16];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int64_t n = n0 + kg * 16 + q4 * 4;
          float4 sv = make_float4(0.f, 0.f, 0.f, 0.f);
          if (row_on && n < t1) sv = *reinterpret_cast<const float4*>(srow[hs] + n);  // t1 - t0 and n are multiples of 4 apart
          const float s4[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const float pv = prob_of(s4[k], mx[hs], rz[hs], normalise);
            p[q4 * 4 + k] = (row_on && n + k < t1) ? pv : 0.f;
          }
        }
#pragma unroll
        for (int sg = 0; sg < 4; ++sg) {
          const float4* sp = reinterpret_cast<const float4*>(lscale + (g * 4 + sg) * MS + kg * 16);
          const float4* zp = reinterpret_cast<const float4*>(lzterm + (g * 4 + sg) * MS + kg * 16);
          // w = p * scale, cut into a bf16 high part and a bf16 remainder.  The
          // zero-point sum uses the SAME two-part value, so that what the matrix core
          // multiplies with 128 + u is subtracted again exactly; only the product with
          // (u - zero) keeps the 2^-16 relative rounding of the split.
          float x[16];
          float zsum = 0.f;
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const float4 s4 = sp[q4], z4 = zp[q4];
            const float ss[4] = {s4.x, s4.y, s4.z, s4.w}, zz[4] = {z4.x, z4.y, z4.z, z4.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const float w = p[q4 * 4 + k] * ss[k];
              const float hi = __uint_as_float(__float_as_uint(w) & 0xffff0000u);
              const float lo = __uint_as_float(__float_as_uint(w - hi) & 0xffff0000u);
              zsum = fmaf(hi + lo, zz[k], zsum);
              x[q4 * 4 + k] = lo_row ? lo : hi;
            }
          }
          zacc[hs][sg] += zsum;
          // token order {0,4,1,5,2,6,3,7} inside each half of 8 to match the nibble
          // expansion below
          uint32_t ab[8];
#pragma unroll
          for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int k = 0; k < 4; ++k)
              ab[half * 4 + k] = (__float_as_uint(x[half * 8 + k]) >> 16) | __float_as_uint(x[half * 8 + k + 4]);
          const uint4 a1 = make_uint4(ab[0], ab[1], ab[2], ab[3]);
          const uint4 a2 = make_uint4(ab[4], ab[5], ab[6], ab[7]);
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
              const uint4 bb = make_uint4((u & 0x000f000fu) | 0x43004300u, ((u >> 4) & 0x000f000fu) | 0x43004300u,
                                          ((u >> 8) & 0x000f000fu) | 0x43004300u,
                                          ((u >> 12) & 0x000f000fu) | 0x43004300u);
              C[hs][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  __builtin_bit_cast(pikv_bf16x8, half ? a2 : a1), __builtin_bit_cast(pikv_bf16x8, bb), C[hs][db], 0, 0, 0);
            }
          }
        }
      }
    }
  }

  // Epilogue.  C: lane (dimension i, rows 4*kg + q): rows 2r / 2r+1 are the two parts of
  // head r, so head 2*kg is q = 0,1 and head 2*kg+1 is q = 2,3.  The zero-point sums sit
  // with the lanes of row 2r (all four token groups): they meet in LDS.
  __syncthreads();
  float* zl = reinterpret_cast<float*>(att_lds);  // [wave][head slot][kg][r][sg]
#pragma unroll
  for (int hs = 0; hs < kMaxHeadsPerWave; ++hs)
    if ((i & 1) == 0 && row_on)
#pragma unroll
      for (int sg = 0; sg < 4; ++sg)
        zl[((((wave * kMaxHeadsPerWave + hs) * 4 + kg) * 8) + r) * 4 + sg] = zacc[hs][sg];
  __syncthreads();
#pragma unroll
  for (int hs = 0; hs < kMaxHeadsPerWave; ++hs) {
    const int g = wave + 4 * hs;
    if (g >= HK) continue;
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      const int ro = 2 * kg + rr;  // head (inside the kv group) held by this lane
      if (ro >= rep) continue;
      float* o = a.partial + (((int64_t)blockIdx.x * a.n_caches + c) * a.n_q_heads + g * rep + ro) * a.head_dim;
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        float z = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < 4; ++k2)
          z += zl[((((wave * kMaxHeadsPerWave + hs) * 4 + k2) * 8) + ro) * 4 + (db >> 1)];
        o[db * 16 + i] = (C[hs][db][2 * rr] + C[hs][db][2 * rr + 1]) - z;
      }
    }
  }
}

// out[c,h,d] = sum over the splits that hold tokens of cache c, in split order
__global__ __launch_bounds__(256) void attend_reduce_kernel(const float* __restrict__ partial,
                                                           const int32_t* __restrict__ fill, int n_caches,
                                                           int n_q_heads, int head_dim, int n_splits,
                                                           float* __restrict__ out) {
  const int64_t per_cache = (int64_t)n_q_heads * head_dim;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_cache * n_caches) return;
  const int c = (int)(idx / per_cache);
  const int64_t used = ((int64_t)fill[c] + kAttTokensPerBlock - 1) / kAttTokensPerBlock;
  const int lim = used < n_splits ? (int)used : n_splits;
  float s = 0.f;
  for (int sp = 0; sp < lim; ++sp) s += partial[(int64_t)sp * per_cache * n_caches + idx];
  out[idx] = s;
}

}  // namespace pikv

using namespace pikv;

static int64_t attend_splits(int64_t max_len) {
  return (max_len + kAttTokensPerBlock - 1) / kAttTokensPerBlock;
}

extern "C" int64_t pikv_attend_workspace_bytes(int n_caches, int n_q_heads, int head_dim, int64_t max_len) {
  if (n_caches < 1 || n_q_heads < 1 || head_dim < 1 || max_len < 0) return 0;
  return attend_splits(max_len) * n_caches * (int64_t)n_q_heads * head_dim * (int64_t)sizeof(float);
}

extern "C" int pikv_attend_values(const float* scores, const float* head_stats, int64_t score_stride,
                                  const void* v_codes, const void* v_scale, const void* v_zero,
                                  int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim,
                                  const int64_t* cache_row_base, const int32_t* cache_fill,
                                  int n_caches, int64_t max_len, float* out, void* workspace,
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
  if (lanes_per_row > 256 || 256 % lanes_per_row != 0) return PIKV_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const int64_t total = (int64_t)n_caches * n_q_heads * head_dim;
  const int64_t splits = attend_splits(max_len);
  if (splits > 65535) return PIKV_ERR_SHAPE;
  if (max_len > 0) {
    if (!workspace) return PIKV_ERR_NULL;
    if (workspace_bytes < pikv_attend_workspace_bytes(n_caches, n_q_heads, head_dim, max_len))
      return PIKV_ERR_WORKSPACE;
  }
  AttendArgs a{scores, head_stats, v_codes, v_scale, v_zero, cache_row_base, cache_fill,
               (float*)workspace, score_stride, group, n_kv_heads, n_q_heads, head_dim, n_caches};
  const int rep = n_q_heads / n_kv_heads;
  if (max_len > 0) {
    const bool aligned = (score_stride % 4 == 0) && ((reinterpret_cast<uintptr_t>(scores) & 15) == 0);
    if (!eight && group == 32 && head_dim == 128 && rep <= 8 && n_kv_heads <= 8 && aligned) {
      const size_t lds = attend_mfma_lds_bytes(n_kv_heads);
      const dim3 grid((unsigned)splits, (unsigned)n_caches);
      if (scheme == PIKV_Q_I4_ASYM)
        hipLaunchKernelGGL((attend_mfma_i4_kernel<PIKV_Q_I4_ASYM>), grid, dim3(256), lds, st, a);
      else
        hipLaunchKernelGGL((attend_mfma_i4_kernel<PIKV_Q_I4_SYM>), grid, dim3(256), lds, st, a);
    } else {
      // heads of a kv group per pass: the float accumulators of one lane must fit
      const int rp = eight ? (rep >= 4 ? 4 : rep >= 2 ? 2 : 1) : (rep >= 2 ? 2 : 1);
      const dim3 grid((unsigned)splits, (unsigned)n_caches, (unsigned)((rep + rp - 1) / rp));
#define PIKV_ATTEND_CASE(S)                                                                        \
  case S:                                                                                          \
    if (rp == 4) hipLaunchKernelGGL((attend_valu_kernel<S, 4>), grid, dim3(256), 0, st, a);        \
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
                     (const float*)workspace, cache_fill, n_caches, n_q_heads, head_dim, (int)splits, out);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
