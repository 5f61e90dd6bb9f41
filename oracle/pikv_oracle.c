/*
 * pikv_oracle.c - scalar C restatement of PiKV's routed, compressed KV-cache
 * data path.  TEST INFRASTRUCTURE ONLY: it is the checker the HIP kernels are
 * compared against and the timed CPU baseline of bench.py; the product library
 * never links or loads it.
 *
 * Written independently of pikv_oracle.py (loops instead of array algebra) so
 * that each pins the other; both follow the same reference lines:
 *   router tail ....... core/single/pikv_routing.py:65-82, :653-656
 *   capacity fill ..... core/single/module/pikv_routing.py:93-104
 *   quantise .......... core/single/module/pikv_compression.py:945-1012
 *   append ............ core/single/cache_scheduling.py:429-436
 *   scores / softmax .. core/single/pikv_attention.py:123,163
 *   importance ........ core/single/pikv_moe.py:241-245
 *   H2O state ......... core/single/cache_scheduling.py:69-99
 *   LRU ............... core/single/cache_scheduling.py:272-285
 *   compaction ........ core/single/cache_scheduling.py:418-424
 *
 * Build: see oracle/Makefile (-O2, no fast-math, no FP contraction; OpenMP only
 * spreads independent rows over threads and never changes a result).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define PKO_F32 0
#define PKO_BF16 1
#define Q_I8_SYM 0
#define Q_I8_ASYM 1
#define Q_I4_ASYM 2
#define Q_I4_SYM 3

int pko_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- scalar conversions ------------------------------------------------- */
static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline float load_elem(const void* p, int dtype, int64_t i) {
  return dtype == PKO_BF16 ? bf16_to_f32(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}

/* float -> IEEE half bits, round to nearest even, finite overflow saturates to 65504 */
static uint16_t f32_to_half_sat(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | (ax > 0x7f800000u ? 0x7e00u : 0x7c00u));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7bffu); /* >= 65520 rounds past max: saturate */
  if (ax < 0x33000001u) return (uint16_t)sign;             /* <= 2^-25: rounds to zero */
  int32_t exp = (int32_t)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u;
  if (exp < -14) { /* subnormal half */
    int shift = -14 - exp + 13;
    uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)(exp + 15) << 10) | ((man >> 13) & 0x3ffu);
  uint32_t rem = man & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
  return (uint16_t)(sign | q);
}

static float half_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff, u;
  if (e == 0) {
    if (m == 0) u = sign;
    else {
      int s = 0;
      while (!(m & 0x400u)) { m <<= 1; s++; }
      u = sign | ((uint32_t)(127 - 15 - s + 1) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (e == 31) u = sign | 0x7f800000u | (m << 13);
  else u = sign | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &u, 4);
  return f;
}

uint16_t pko_f32_to_half(float f) { return f32_to_half_sat(f); }
float pko_half_to_f32(uint16_t h) { return half_to_f32(h); }

/* ---- router --------------------------------------------------------------- */
/* logits (double accumulation, rounded once), scaling, softmax, top-k of the float32
 * probabilities by (value desc, index asc, NaN last) as core/single/pikv_routing.py:73-76
 * hands them to torch.topk, renormalise.  probs/logits_out may be NULL. */
void pko_router(const void* x, const void* w, int dtype, const float* bias, const float* escale,
                const float* emask, float temperature, float renorm_eps, int64_t T, int H, int E,
                int k, float* probs, float* logits_out, int32_t* idx, float* wts) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; ++t) {
    float lg[64], pr[64];
    for (int e = 0; e < E; ++e) {
      double acc = 0.0;
      for (int h = 0; h < H; ++h)
        acc += (double)load_elem(x, dtype, t * H + h) * (double)load_elem(w, dtype, (int64_t)e * H + h);
      if (bias) acc += (double)bias[e];
      float v = (float)acc;
      if (temperature != 1.0f) v = v / temperature;
      if (escale) v = v * escale[e];
      if (emask) {
        float pen = (1.0f - emask[e]) * -1e9f;
        v = v + pen;
      }
      lg[e] = v;
      if (logits_out) logits_out[t * E + e] = v;
    }
    float m = lg[0];
    for (int e = 1; e < E; ++e) m = lg[e] > m ? lg[e] : m;
    float sum = 0.f;
    for (int e = 0; e < E; ++e) { pr[e] = expf(lg[e] - m); sum += pr[e]; }
    for (int e = 0; e < E; ++e) { pr[e] = pr[e] / sum; if (probs) probs[t * E + e] = pr[e]; }
    char used[64] = {0};
    float s = 0.f;
    for (int j = 0; j < k; ++j) {
      int best = -1;
      for (int e = 0; e < E; ++e) { /* strict >: lowest index wins ties; a NaN never beats anything */
        if (used[e]) continue;
        if (best < 0 || pr[e] > pr[best] || (pr[best] != pr[best] && pr[e] == pr[e])) best = e;
      }
      used[best] = 1;
      idx[t * k + j] = best;
      wts[t * k + j] = pr[best];
      s = s + pr[best];
    }
    if (renorm_eps != 0.f) s = s + renorm_eps;
    for (int j = 0; j < k; ++j) wts[t * k + j] = wts[t * k + j] / s;
  }
}

/* The literal sequential fill: walk assignments in token-major order. */
void pko_capacity_slots(const int32_t* idx, int64_t A, int E, int64_t capacity, int32_t* slot,
                        int32_t* count) {
  int64_t used[64] = {0};
  for (int e = 0; e < E; ++e) count[e] = 0;
  for (int64_t a = 0; a < A; ++a) {
    int e = idx[a];
    count[e]++;
    if (used[e] < capacity) { slot[a] = (int32_t)used[e]; used[e]++; }
    else slot[a] = -1;
  }
}

/* ---- quantisation ----------------------------------------------------------- */
static void scheme_range(int scheme, int* bits, int* sym, int* qmin, int* qmax) {
  *bits = (scheme == Q_I8_SYM || scheme == Q_I8_ASYM) ? 8 : 4;
  *sym = (scheme == Q_I8_SYM || scheme == Q_I4_SYM);
  *qmin = *sym ? -(1 << (*bits - 1)) : 0;
  *qmax = *sym ? (1 << (*bits - 1)) - 1 : (1 << *bits) - 1;
}

/* One reduction domain of g elements -> codes (int), scale, zero. */
static void quant_domain(const float* x, int g, int scheme, int* q, float* scale_out, float* zero_out) {
  int bits, sym, qmin, qmax;
  scheme_range(scheme, &bits, &sym, &qmin, &qmax);
  float mn = x[0], mx = x[0];
  for (int i = 1; i < g; ++i) { if (x[i] < mn) mn = x[i]; if (x[i] > mx) mx = x[i]; }
  if (mx == mn) mx = mn + 1e-5f;
  float qr = (float)(qmax - qmin), scale, zero;
  if (sym) {
    float a = fabsf(mn), b = fabsf(mx);
    scale = (2.0f * (a > b ? a : b)) / qr;
  } else scale = (mx - mn) / qr;
  if (bits == 4) {
    scale = half_to_f32(f32_to_half_sat(scale));
    if (scale == 0.0f) scale = 5.9604644775390625e-08f; /* 2^-24 */
    if (!sym && fabsf(mn) > 1024.0f * scale) {
      /* the half-precision zero point must stay an exact integer: widen the scale */
      scale = half_to_f32(f32_to_half_sat(fabsf(mn) * 0.0009765625f));
      if (scale == 0.0f) scale = 5.9604644775390625e-08f;
    }
  }
  if (sym) zero = 0.f;
  else {
    zero = (float)qmin - rintf(mn / scale);
    if (bits == 4) zero = half_to_f32(f32_to_half_sat(zero));
  }
  for (int i = 0; i < g; ++i) {
    float y = x[i] / scale;
    y = y + zero;
    y = rintf(y);
    if (y != y) y = (float)qmin;
    if (y < (float)qmin) y = (float)qmin;
    if (y > (float)qmax) y = (float)qmax;
    q[i] = (int)y;
  }
  *scale_out = scale;
  *zero_out = zero;
}

static void store_row(const int* q, const float* sc, const float* zr, int D, int group, int scheme,
                      void* codes, void* scale, void* zero, int64_t row) {
  int bits, sym, qmin, qmax;
  scheme_range(scheme, &bits, &sym, &qmin, &qmax);
  int ng = D / group;
  if (bits == 8) {
    int8_t* c = (int8_t*)codes + row * D;
    for (int i = 0; i < D; ++i) c[i] = (int8_t)(q[i] & 0xff);
    for (int g = 0; g < ng; ++g) {
      ((float*)scale)[row * ng + g] = sc[g];
      if (!sym) ((float*)zero)[row * ng + g] = zr[g];
    }
  } else {
    uint8_t* c = (uint8_t*)codes + row * (D / 2);
    for (int i = 0; i < D / 2; ++i) c[i] = (uint8_t)((q[2 * i] & 0xf) | ((q[2 * i + 1] & 0xf) << 4));
    for (int g = 0; g < ng; ++g) {
      ((uint16_t*)scale)[row * ng + g] = f32_to_half_sat(sc[g]);
      if (!sym) ((uint16_t*)zero)[row * ng + g] = f32_to_half_sat(zr[g]);
    }
  }
}

/* Quantise source row s once, write it to the rows of its `fanout` assignments.
 * cache_id == NULL: plain rows, destination row = dst_row0 + s. */
void pko_quant_scatter(const void* k_src, const void* v_src, int dtype, int64_t n_src, int fanout,
                       int D, int group, int scheme, const int32_t* cache_id, const int32_t* slot,
                       const int64_t* row_base, const int32_t* fill, const int32_t* cap,
                       int64_t dst_row0, void* k_codes, void* v_codes, void* k_scale, void* v_scale,
                       void* k_zero, void* v_zero, float* acc, float* ts, float now) {
  int ng = D / group;
#pragma omp parallel
  {
    float* x = (float*)malloc(sizeof(float) * D);
    int* q = (int*)malloc(sizeof(int) * D);
    float* sc = (float*)malloc(sizeof(float) * ng);
    float* zr = (float*)malloc(sizeof(float) * ng);
#pragma omp for schedule(static)
    for (int64_t s = 0; s < n_src; ++s) {
      int64_t dst[8];
      int nd = 0;
      if (!cache_id) dst[nd++] = dst_row0 + s;
      else
        for (int j = 0; j < fanout; ++j) {
          int64_t a = s * fanout + j;
          if (slot[a] < 0) continue;
          int c = cache_id[a];
          int64_t r = (int64_t)fill[c] + slot[a];
          if (r >= cap[c]) continue;
          dst[nd++] = row_base[c] + r;
        }
      if (nd == 0) continue;
      for (int t = 0; t < 2; ++t) {
        const void* src = t ? v_src : k_src;
        if (!src) continue;
        for (int i = 0; i < D; ++i) x[i] = load_elem(src, dtype, s * D + i);
        for (int g = 0; g < ng; ++g) quant_domain(x + g * group, group, scheme, q + g * group, &sc[g], &zr[g]);
        for (int j = 0; j < nd; ++j)
          store_row(q, sc, zr, D, group, scheme, t ? v_codes : k_codes, t ? v_scale : k_scale,
                    t ? v_zero : k_zero, dst[j]);
      }
      for (int j = 0; j < nd; ++j) {
        if (acc) acc[dst[j]] = 0.f;
        if (ts) ts[dst[j]] = now;
      }
    }
    free(x); free(q); free(sc); free(zr);
  }
}

static inline float dequant_elem(const void* codes, const void* scale, const void* zero, int D,
                                 int group, int scheme, int64_t row, int i) {
  int bits, sym, qmin, qmax;
  scheme_range(scheme, &bits, &sym, &qmin, &qmax);
  int ng = D / group, g = i / group;
  float s, z = 0.f, qv;
  if (bits == 8) {
    s = ((const float*)scale)[row * ng + g];
    if (!sym) z = ((const float*)zero)[row * ng + g];
    qv = sym ? (float)((const int8_t*)codes)[row * D + i] : (float)((const uint8_t*)codes)[row * D + i];
  } else {
    s = half_to_f32(((const uint16_t*)scale)[row * ng + g]);
    if (!sym) z = half_to_f32(((const uint16_t*)zero)[row * ng + g]);
    uint8_t b = ((const uint8_t*)codes)[row * (D / 2) + i / 2];
    int n = (i & 1) ? (b >> 4) : (b & 0xf);
    if (sym && n >= 8) n -= 16;
    qv = (float)n;
  }
  return (qv - z) * s;
}

/* out[i,:] = (q - zero) * scale of row rows[i] (rows == NULL: row0 + i), float32. */
void pko_gather_dequant(const void* codes, const void* scale, const void* zero, int D, int group,
                        int scheme, const int64_t* rows, int64_t row0, int64_t n, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int64_t row = rows ? rows[i] : row0 + i;
    for (int d = 0; d < D; ++d) out[i * D + d] = dequant_elem(codes, scale, zero, D, group, scheme, row, d);
  }
}

/* Read path of one pool: for every cache c and q head h
 *   s[h,n] = dot(q[c,h,:], K^[n, h/rep, :]) * scale_qk   (double accumulation)
 *   p      = softmax_n(s);  imp[n] = sum_h p[h,n]
 *   acc[row] = acc[row]*decay + imp[n]; ts[row] = now
 * scores (may be NULL) [n_caches, n_q, stride] receives s. */
void pko_scores_h2o(const void* k_codes, const void* k_scale, const void* k_zero, int scheme,
                    int group, int n_kv, int n_q, int dh, const void* q, int q_dtype,
                    float scale_qk, const int64_t* row_base, const int32_t* fill, int n_caches,
                    int64_t stride, float decay, float now, float* scores, float* acc, float* ts,
                    float* importance) {
  int D = n_kv * dh, rep = n_q / n_kv;
  for (int c = 0; c < n_caches; ++c) {
    int64_t L = fill[c];
    if (L <= 0) continue;
    double* s = (double*)malloc(sizeof(double) * (size_t)n_q * (size_t)L);
#pragma omp parallel
    {
      float* kr = (float*)malloc(sizeof(float) * D);
#pragma omp for schedule(static)
      for (int64_t n = 0; n < L; ++n) {
        int64_t row = row_base[c] + n;
        for (int d = 0; d < D; ++d) kr[d] = dequant_elem(k_codes, k_scale, k_zero, D, group, scheme, row, d);
        for (int h = 0; h < n_q; ++h) {
          const float* kh = kr + (h / rep) * dh;
          double a = 0.0;
          for (int d = 0; d < dh; ++d) a += (double)load_elem(q, q_dtype, ((int64_t)c * n_q + h) * dh + d) * (double)kh[d];
          s[(size_t)h * L + n] = a * (double)scale_qk;
          if (scores) scores[((int64_t)c * n_q + h) * stride + n] = (float)s[(size_t)h * L + n];
        }
      }
      free(kr);
    }
    double* imp = (double*)calloc((size_t)L, sizeof(double));
    for (int h = 0; h < n_q; ++h) {
      double m = -INFINITY, z = 0.0;
      for (int64_t n = 0; n < L; ++n) if (s[(size_t)h * L + n] > m) m = s[(size_t)h * L + n];
      for (int64_t n = 0; n < L; ++n) z += exp(s[(size_t)h * L + n] - m);
      for (int64_t n = 0; n < L; ++n) imp[n] += exp(s[(size_t)h * L + n] - m) / z;
    }
    for (int64_t n = 0; n < L; ++n) {
      int64_t row = row_base[c] + n;
      float a = acc[row];
      if (decay != 1.0f) a = a * decay;
      acc[row] = a + (float)imp[n];
      ts[row] = now;
      if (importance) importance[(int64_t)c * stride + n] = (float)imp[n];
    }
    free(imp);
    free(s);
  }
}

/* ---- eviction ----------------------------------------------------------------- */
typedef struct { float v; int32_t i; } pko_item;
static int cmp_desc(const void* a, const void* b) {
  const pko_item *x = a, *y = b;
  if (x->v > y->v) return -1;
  if (x->v < y->v) return 1;
  return (x->i > y->i) - (x->i < y->i);
}
static int cmp_asc(const void* a, const void* b) {
  const pko_item *x = a, *y = b;
  if (x->v < y->v) return -1;
  if (x->v > y->v) return 1;
  return (x->i > y->i) - (x->i < y->i);
}
static void mark_top(const float* v, int len, int m, int smallest, uint8_t* flag, uint8_t mark) {
  if (m <= 0) return;
  if (m > len) m = len;
  pko_item* it = (pko_item*)malloc(sizeof(pko_item) * (size_t)len);
  for (int i = 0; i < len; ++i) { it[i].v = v[i] + 0.0f; it[i].i = i; }
  qsort(it, (size_t)len, sizeof(pko_item), smallest ? cmp_asc : cmp_desc);
  for (int j = 0; j < m; ++j) flag[it[j].i] = mark;
  free(it);
}

/* policy 0 = H2O: keep top n_heavy of acc UNION top n_recent of ts;
 * policy 1 = LRU: evict the n_heavy[c] smallest ts. */
void pko_evict_select(int policy, const float* acc, const float* ts, const int64_t* row_base,
                      const int32_t* fill, const int32_t* n_heavy, const int32_t* n_recent,
                      int n_caches, uint8_t* keep_flag, int32_t* keep_index, int32_t* new_len) {
  for (int c = 0; c < n_caches; ++c) {
    int len = fill[c];
    int64_t b = row_base[c];
    if (policy == 0) {
      memset(keep_flag + b, 0, (size_t)len);
      mark_top(acc + b, len, n_heavy[c], 0, keep_flag + b, 1);
      mark_top(ts + b, len, n_recent[c], 0, keep_flag + b, 1);
    } else {
      memset(keep_flag + b, 1, (size_t)len);
      mark_top(ts + b, len, n_heavy[c], 1, keep_flag + b, 0);
    }
    int m = 0;
    for (int i = 0; i < len; ++i) if (keep_flag[b + i]) keep_index[b + m++] = i;
    new_len[c] = m;
  }
}

/* cache[:m] = cur[keep] for one plane of row_bytes bytes per row. */
void pko_compact_plane(void* plane, int64_t row_bytes, const int64_t* row_base,
                       const int32_t* keep_index, const int32_t* new_len, int n_caches) {
  for (int c = 0; c < n_caches; ++c) {
    char* p = (char*)plane + row_base[c] * row_bytes;
    for (int j = 0; j < new_len[c]; ++j) {
      int s = keep_index[row_base[c] + j];
      if (s != j) memmove(p + (int64_t)j * row_bytes, p + (int64_t)s * row_bytes, (size_t)row_bytes);
    }
  }
}
