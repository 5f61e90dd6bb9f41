// Shared device/host helpers for the gfx950 kernels of libpikv_hip.so.
// Wavefront width is 64 everywhere; nothing here is written for 32-wide waves.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pikv_hip.h"

#define PIKV_WAVE 64

#define PIKV_CHECK_LAUNCH()                              \
  do {                                                   \
    if (hipGetLastError() != hipSuccess) return PIKV_ERR_LAUNCH; \
  } while (0)

namespace pikv {

// ---- scalar type conversion --------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) {
  return __uint_as_float(b << 16);
}

// float -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

// A float32 value as two bf16 limbs, f = hi + lo to 2^-18 |f|: hi = f rounded to bf16 (cut to its upper 16
// bits instead where rounding would carry a finite value to infinity), lo = the rest rounded to bf16.  A value
// that is a bf16 number gives (itself, 0).  Returns the bits of limb `which`.
__device__ __forceinline__ uint32_t bf16_limb_bits(float f, int which) {
  uint32_t h = float_to_bf16_bits(f);
  if ((h & 0x7f80u) == 0x7f80u && (__float_as_uint(f) & 0x7f800000u) != 0x7f800000u) h = __float_as_uint(f) >> 16;
  return which == 0 ? h : float_to_bf16_bits(f - __uint_as_float(h << 16));
}

// float -> half, round to nearest even, finite values saturate at +-65504.
__device__ __forceinline__ _Float16 float_to_half_sat(float f) {
  if (f > 65504.0f && f < __builtin_inff()) return (_Float16)65504.0f;
  if (f < -65504.0f && f > -__builtin_inff()) return (_Float16)(-65504.0f);
  _Float16 h = (_Float16)f;
  if (__builtin_isinf((float)h) && !__builtin_isinf(f))
    h = (_Float16)(f > 0.f ? 65504.0f : -65504.0f);
  return h;
}

// ---- 16-byte global access -----------------------------------------------------
__device__ __forceinline__ uint4 ld16(const void* p) {
  return *reinterpret_cast<const uint4*>(p);
}
__device__ __forceinline__ void st16(void* p, uint4 v) {
  *reinterpret_cast<uint4*>(p) = v;
}
// Streaming store: code rows are written once and not read again by the writer,
// so they should not displace L2 lines (measured: ~2 % faster scatter; the same
// hint on the loads was slower).
typedef uint32_t pikv_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st16_stream(void* p, uint4 v) {
  pikv_u32x4 t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<pikv_u32x4*>(p));
}

// Load N consecutive source elements (N % 8 == 0) as float.
template <int DT, int N>
__device__ __forceinline__ void load_as_float(const void* base, int64_t elem_off,
                                              float (&out)[N]) {
  if constexpr (DT == PIKV_BF16) {
    const char* p = reinterpret_cast<const char*>(base) + elem_off * 2;
#pragma unroll
    for (int i = 0; i < N / 8; ++i) {
      uint4 v = ld16(p + 16 * i);
      uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        out[8 * i + 2 * j] = __uint_as_float(w[j] << 16);
        out[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
    }
  } else {
    const char* p = reinterpret_cast<const char*>(base) + elem_off * 4;
#pragma unroll
    for (int i = 0; i < N / 4; ++i) {
      uint4 v = ld16(p + 16 * i);
      out[4 * i] = __uint_as_float(v.x);
      out[4 * i + 1] = __uint_as_float(v.y);
      out[4 * i + 2] = __uint_as_float(v.z);
      out[4 * i + 3] = __uint_as_float(v.w);
    }
  }
}

// ---- cross-lane reductions over aligned groups of LANES lanes (power of two) -----
template <int LANES>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int m = 1; m < LANES; m <<= 1) v = fmaxf(v, __shfl_xor(v, m, PIKV_WAVE));
  return v;
}
template <int LANES>
__device__ __forceinline__ float group_min(float v) {
#pragma unroll
  for (int m = 1; m < LANES; m <<= 1) v = fminf(v, __shfl_xor(v, m, PIKV_WAVE));
  return v;
}
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int m = 1; m < LANES; m <<= 1) v += __shfl_xor(v, m, PIKV_WAVE);
  return v;
}
// Runtime-width variants (width = power of two <= 64).
__device__ __forceinline__ float group_max_rt(float v, int width) {
  for (int m = 1; m < width; m <<= 1) v = fmaxf(v, __shfl_xor(v, m, PIKV_WAVE));
  return v;
}
__device__ __forceinline__ float group_min_rt(float v, int width) {
  for (int m = 1; m < width; m <<= 1) v = fminf(v, __shfl_xor(v, m, PIKV_WAVE));
  return v;
}

// ---- quantisation formula --------------------------------------------------------
// Float32 arithmetic in the operation order of the reference's
// QuantizedCompressor._quantize_tensor (core/single/module/pikv_compression.py:
// 945-1012): true division, round-half-even, no reciprocal, no contraction.
template <int SCHEME>
struct QScheme {
  static constexpr int bits = (SCHEME == PIKV_Q_I8_SYM || SCHEME == PIKV_Q_I8_ASYM) ? 8 : 4;
  static constexpr bool sym = (SCHEME == PIKV_Q_I8_SYM || SCHEME == PIKV_Q_I4_SYM);
  static constexpr int qmin = sym ? -(1 << (bits - 1)) : 0;
  static constexpr int qmax = sym ? (1 << (bits - 1)) - 1 : (1 << bits) - 1;
  static constexpr int epl = bits == 8 ? 16 : 32;  // elements per lane (16 code bytes)
  static constexpr int meta_bytes = bits == 8 ? 4 : 2;
};

template <int SCHEME>
__device__ __forceinline__ void quant_params(float mn, float mx, float& scale, float& zero) {
  using Q = QScheme<SCHEME>;
  if (mx == mn) mx = mn + 1e-5f;
  const float qr = (float)(Q::qmax - Q::qmin);
  if constexpr (Q::sym) {
    float amax = fmaxf(fabsf(mn), fabsf(mx));
    scale = (2.0f * amax) / qr;
  } else {
    scale = (mx - mn) / qr;
  }
  if constexpr (Q::bits == 4) {
    // stored as half: a scale that underflows to zero becomes the smallest
    // positive half (2^-24) so that encoder and decoder never divide by zero
    scale = (float)float_to_half_sat(scale);
    if (scale == 0.0f) scale = 5.9604644775390625e-08f;
    if constexpr (!Q::sym) {
      // The zero point is stored as half as well and must stay an integer that half
      // holds exactly.  A group whose spread is tiny next to its offset (a constant
      // non-zero group, with the 1e-5 range above) would need a far larger one: its
      // scale is widened to |min| / 1024 (|zero| <= 1025).  Error <= |min| / 2048.
      if (fabsf(mn) > 1024.0f * scale) {
        scale = (float)float_to_half_sat(fabsf(mn) * 0.0009765625f);
        if (scale == 0.0f) scale = 5.9604644775390625e-08f;
      }
    }
  }
  if constexpr (Q::sym) {
    zero = 0.0f;
  } else {
    zero = (float)Q::qmin - rintf(mn / scale);
    if constexpr (Q::bits == 4) zero = (float)float_to_half_sat(zero);
  }
}

template <int SCHEME>
__device__ __forceinline__ int quant_code(float x, float scale, float zero) {
  using Q = QScheme<SCHEME>;
  float y = x / scale;
  y = y + zero;
  y = rintf(y);
  // NaN (0/0 from a zero scale) maps to qmin, as the CPU restatement does.
  y = (y != y) ? (float)Q::qmin : y;
  y = fminf(fmaxf(y, (float)Q::qmin), (float)Q::qmax);
  return (int)y;
}

// ---- exact quantiser of one lane without a division per element ------------------
// The reference divides every element by the group's scale.  A float32 division is a
// dozen instructions; here the group pays for ONE, r = RN(1 / scale), and every element
// gets its correctly rounded quotient from three:
//     q0 = RN(x * r);  e = x - scale * q0 (exact, one fma);  q = RN(q0 + e * r)
// With r the correctly rounded reciprocal and q0 within one unit in the last place of
// x / scale, q IS RN(x / scale) (Markstein's theorem on fma-based division; checked
// against the division operator on 9e8 random and structured pairs, including scales
// with an all-ones significand, powers of two, and bf16 / half operands).  The rest is the
// reference's own arithmetic: t = RN(q + zero), round half to even, clamp.
// The construction needs no intermediate to overflow or vanish: a group takes it only when
// its scale lies in [1e-30, 1e30] and |x / scale| <= 768 for all of its elements (elements
// far below the scale are harmless: any quotient of magnitude < 1/4 yields the same code).
// Other groups - infinities, collapsed ranges - go through quant_code() element by element.
struct GroupQuant {
  float scale, zero, r;
  bool fast;
};

template <int SCHEME>
__device__ __forceinline__ GroupQuant make_group_quant(float mn, float mx) {
  GroupQuant g;
  quant_params<SCHEME>(mn, mx, g.scale, g.zero);
  g.r = 1.0f / g.scale;  // correctly rounded (-fhip-fp32-correctly-rounded-divide-sqrt)
  const float amax = fmaxf(fabsf(mn), fabsf(mx));
  g.fast = (g.scale >= 1e-30f) && (g.scale <= 1e30f) && (amax * g.r <= 768.0f);
  return g;
}

// Stored (unsigned) form of the code of t = x / scale + zero, as a float in [0, 2^bits - 1]
// that the byte conversion takes as is.  NaN ends as 0, the stored form of qmin.
template <int SCHEME>
__device__ __forceinline__ float stored_code_value(float t) {
  using Q = QScheme<SCHEME>;
  if constexpr (Q::sym) t = rintf(t) + (float)(-Q::qmin);   // exact: integers
  // the byte conversion itself rounds half to even and saturates at [0, 255]; four-bit
  // codes are cut to [0, 15] first (median of three: a NaN gives the smaller bound)
  if constexpr (Q::bits == 4) t = __builtin_amdgcn_fmed3f(t, 0.0f, 15.0f);
  return t;
}

// Quantise the EPL elements of a lane and pack them into 16 code bytes.
template <int SCHEME>
__device__ __forceinline__ uint4 quantize_lane(const float (&x)[QScheme<SCHEME>::epl],
                                               const GroupQuant& g) {
  using Q = QScheme<SCHEME>;
  constexpr int EPL = Q::epl;
  constexpr int NW = EPL / 4;                          // words of one byte per element
  uint32_t w[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) w[i] = 0;
  if (g.fast) {
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      // 8-bit: element i -> byte i%4 of word i/4.  4-bit: even elements of an octet
      // go to word 2*(i/8), odd ones to word 2*(i/8)+1, byte (i%8)/2.
      const int wi = Q::bits == 8 ? i / 4 : 2 * (i / 8) + (i & 1);
      const int bi = Q::bits == 8 ? i % 4 : (i % 8) / 2;
      const float q0 = x[i] * g.r;
      const float e = __builtin_fmaf(-g.scale, q0, x[i]);
      const float q = __builtin_fmaf(e, g.r, q0);
      float t = q;
      if constexpr (!Q::sym) t = q + g.zero;
      w[wi] = __builtin_amdgcn_cvt_pk_u8_f32(stored_code_value<SCHEME>(t), bi, w[wi]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int wi = Q::bits == 8 ? i / 4 : 2 * (i / 8) + (i & 1);
      const int bi = Q::bits == 8 ? i % 4 : (i % 8) / 2;
      const int c = quant_code<SCHEME>(x[i], g.scale, g.zero) - Q::qmin;  // unsigned stored form
      w[wi] |= (uint32_t)c << (8 * bi);
    }
  }
  uint32_t o[4];
  if constexpr (Q::bits == 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = Q::sym ? (w[i] ^ 0x80808080u) : w[i];
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = w[2 * i] | (w[2 * i + 1] << 4);
      if constexpr (Q::sym) o[i] ^= 0x88888888u;
    }
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// ---- DPP reductions over aligned groups of `lanes` lanes (runtime power of two) ----
// quad_perm xor-1 / xor-2, row_half_mirror and row_mirror combine disjoint halves
// inside a 16-lane row in one instruction each; wider groups finish with two
// cross-row shuffles.
// The partner's value comes from the data-parallel-primitive builtin, so the compiler sees
// an ordinary VALU definition: it folds the move into the min / max / add that consumes it
// (one VOP2-DPP instruction) and places every wait state itself, before and after.
constexpr int kDppXor1 = 0xB1;         // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // row_half_mirror
constexpr int kDppMirror = 0x140;      // row_mirror
template <int CTRL>
__device__ __forceinline__ float dpp_partner(float v) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL> __device__ __forceinline__ float dpp_min(float v) { return fminf(v, dpp_partner<CTRL>(v)); }
template <int CTRL> __device__ __forceinline__ float dpp_max(float v) { return fmaxf(v, dpp_partner<CTRL>(v)); }
template <int CTRL> __device__ __forceinline__ float dpp_add(float v) { return v + dpp_partner<CTRL>(v); }

__device__ __forceinline__ void group_minmax_dpp(float& mn, float& mx, int lanes) {
  if (lanes >= 2) {
    mn = dpp_min<kDppXor1>(mn);
    mx = dpp_max<kDppXor1>(mx);
  }
  if (lanes >= 4) {
    mn = dpp_min<kDppXor2>(mn);
    mx = dpp_max<kDppXor2>(mx);
  }
  if (lanes >= 8) {
    mn = dpp_min<kDppHalfMirror>(mn);
    mx = dpp_max<kDppHalfMirror>(mx);
  }
  if (lanes >= 16) {
    mn = dpp_min<kDppMirror>(mn);
    mx = dpp_max<kDppMirror>(mx);
  }
  if (lanes >= 32) { mn = fminf(mn, __shfl_xor(mn, 16, PIKV_WAVE)); mx = fmaxf(mx, __shfl_xor(mx, 16, PIKV_WAVE)); }
  if (lanes >= 64) { mn = fminf(mn, __shfl_xor(mn, 32, PIKV_WAVE)); mx = fmaxf(mx, __shfl_xor(mx, 32, PIKV_WAVE)); }
}

__device__ __forceinline__ float read_lane_f(float v, int l) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), l));
}

// Sum / max over aligned groups of `lanes` (a power of two <= 64) adjacent lanes;
// every lane of the group ends with the result.  Rows of 16 lanes reduce with DPP;
// a whole wavefront then combines its four rows through scalar registers.
__device__ __forceinline__ float group_sum_dpp(float v, int lanes) {
  if (lanes >= 2) v = dpp_add<kDppXor1>(v);
  if (lanes >= 4) v = dpp_add<kDppXor2>(v);
  if (lanes >= 8) v = dpp_add<kDppHalfMirror>(v);
  if (lanes >= 16) v = dpp_add<kDppMirror>(v);
  if (lanes >= 64)
    v = (read_lane_f(v, 0) + read_lane_f(v, 16)) + (read_lane_f(v, 32) + read_lane_f(v, 48));
  else if (lanes >= 32)
    v += __shfl_xor(v, 16, PIKV_WAVE);
  return v;
}
__device__ __forceinline__ float group_max_dpp(float v, int lanes) {
  if (lanes >= 2) v = dpp_max<kDppXor1>(v);
  if (lanes >= 4) v = dpp_max<kDppXor2>(v);
  if (lanes >= 8) v = dpp_max<kDppHalfMirror>(v);
  if (lanes >= 16) v = dpp_max<kDppMirror>(v);
  if (lanes >= 64)
    v = fmaxf(fmaxf(read_lane_f(v, 0), read_lane_f(v, 16)), fmaxf(read_lane_f(v, 32), read_lane_f(v, 48)));
  else if (lanes >= 32)
    v = fmaxf(v, __shfl_xor(v, 16, PIKV_WAVE));
  return v;
}

// Pack the codes of one lane (16 x 8-bit or 32 x 4-bit) into 16 bytes.
template <int SCHEME>
__device__ __forceinline__ uint4 pack_codes(const int* c) {
  using Q = QScheme<SCHEME>;
  uint32_t w[4];
  if constexpr (Q::bits == 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (uint32_t)(c[4 * i] & 0xff) | ((uint32_t)(c[4 * i + 1] & 0xff) << 8) |
             ((uint32_t)(c[4 * i + 2] & 0xff) << 16) | ((uint32_t)(c[4 * i + 3] & 0xff) << 24);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t v = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) v |= (uint32_t)(c[8 * i + j] & 0xf) << (4 * j);
      w[i] = v;
    }
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Unpack 16 bytes of codes into integers (sign-extended for symmetric schemes).
template <int SCHEME>
__device__ __forceinline__ void unpack_codes(uint4 v, int* c) {
  using Q = QScheme<SCHEME>;
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
  if constexpr (Q::bits == 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t b = (w[i] >> (8 * j)) & 0xff;
        c[4 * i + j] = Q::sym ? (int)(int8_t)b : (int)b;
      }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        int b = (int)((w[i] >> (4 * j)) & 0xf);
        c[8 * i + j] = Q::sym ? ((b ^ 8) - 8) : b;
      }
  }
}

// Codes of one lane as floats of (code - qmin), i.e. the unsigned stored form: the
// byte extractions below compile to v_cvt_f32_ubyteN (one instruction per code),
// and the caller folds qmin into the zero point.
template <int SCHEME>
__device__ __forceinline__ void unpack_codes_unsigned(uint4 v, float* f) {
  using Q = QScheme<SCHEME>;
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
  if constexpr (Q::bits == 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = Q::sym ? (w[i] ^ 0x80808080u) : w[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) f[4 * i + j] = (float)((u >> (8 * j)) & 0xffu);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = Q::sym ? (w[i] ^ 0x88888888u) : w[i];
      const uint32_t ev = u & 0x0f0f0f0fu, od = (u >> 4) & 0x0f0f0f0fu;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f[8 * i + 2 * j] = (float)((ev >> (8 * j)) & 0xffu);
        f[8 * i + 2 * j + 1] = (float)((od >> (8 * j)) & 0xffu);
      }
    }
  }
}

// Metadata (scale / zero) element access: float for 8-bit, half for 4-bit.
template <int SCHEME>
__device__ __forceinline__ void store_meta(void* plane, int64_t idx, float v) {
  if constexpr (QScheme<SCHEME>::bits == 8)
    reinterpret_cast<float*>(plane)[idx] = v;
  else
    reinterpret_cast<_Float16*>(plane)[idx] = (_Float16)v;  // exact: already half-valued
}
template <int SCHEME>
__device__ __forceinline__ float load_meta(const void* plane, int64_t idx) {
  if constexpr (QScheme<SCHEME>::bits == 8)
    return reinterpret_cast<const float*>(plane)[idx];
  else
    return (float)reinterpret_cast<const _Float16*>(plane)[idx];
}

__host__ __device__ inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

// The matrix-core read kernels work on 128-dimension slabs of a cached row: one kv head of 128
// dimensions, or the stored bytes of 2 / 4 neighbouring kv heads of 64 / 32.  Heads per slab, or 0
// when the head width is another one or the heads of a row do not fill whole slabs.
inline int mfma_heads_per_slab(int head_dim, int n_kv_heads) {
  if (head_dim != 128 && head_dim != 64 && head_dim != 32) return 0;
  const int hps = 128 / head_dim;
  return n_kv_heads % hps == 0 ? hps : 0;
}

// read_path.hip, for pikv_decode_attend in attend.hip: the 4-bit matrix-core score kernel writing the
// exchange format (escores [cache][tile][q head][64] floats = exp(score - tile max); tile_max, tile_sum
// [cache][tile][q head]) followed by the merge of the tile statistics into head_stats [cache][q head][2].
// Returns PIKV_ERR_UNSUPPORTED, with nothing enqueued, for cache formats that kernel does not serve.
int scores_exchange_launch(const void* k_codes, const void* k_scale, const void* k_zero, int scheme, int group,
                           int n_kv_heads, int n_q_heads, int head_dim, const void* q, int q_dtype, float scale_qk,
                           const int64_t* cache_row_base, const int32_t* cache_fill, int n_caches, int64_t max_len,
                           float* escores, float* tile_max, float* tile_sum, float* head_stats, hipStream_t st);

// decode_fused.hip, for pikv_decode_attend in attend.hip: the one-pass decode read (heads of 128, 2 to 8
// kv heads; 4-bit codes in groups of 32 with up to 4 bf16 or float32 query heads per kv head, or 5 to 8 bf16
// ones; 8-bit codes with a scale per kv head or coarser and up to 8 bf16 or float32 ones).
bool decode_fused_serves(int scheme, int group, int n_kv_heads, int n_q_heads, int head_dim, int q_dtype, bool bookkeeping);
int fused_tokens_per_block(int n_caches, int n_kv_heads, int64_t max_len, int min_tpb);
int decode_fused_launch(const void* k_codes, const void* k_scale, const void* k_zero, const void* v_codes,
                        const void* v_scale, const void* v_zero, int scheme, int group, int n_kv_heads, int n_q_heads,
                        const void* q, int q_dtype, float scale_qk, const int64_t* cache_row_base, const int32_t* cache_fill,
                        int n_caches, int64_t max_len, int tokens_per_block, float decay, float now, float* row_acc,
                        float* row_ts, float* out, void* e16, float* tref, float* pstats, float* partial,
                        float* head_stats, hipStream_t st);

// (x & m) | o.  Plain C on purpose: the value feeds a matrix-core operand, and a
// result produced inside an inline-asm block is invisible to the compiler's
// hazard handling between vector and matrix-core instructions.
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t m, uint32_t o) { return (x & m) | o; }

}  // namespace pikv
