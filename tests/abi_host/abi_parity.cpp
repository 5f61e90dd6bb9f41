// A host program in plain C++ that uses libpikv_hip.so the way a native caller
// would: include/pikv_hip.h, hipMalloc'ed buffers, no Python, no torch.  It runs
// router tail -> capacity slots -> quantise + scatter -> advance -> gather +
// dequantise -> H2O budget -> eviction select -> compaction on one small workload
// and checks every result, bit for bit, against the scalar C restatement
// (oracle/pikv_oracle.c, linked as libpikv_oracle.so).  Test infrastructure only.
//
// Exit status 0 and a last line "abi_parity: ALL OK" on success.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "pikv_hip.h"

extern "C" {
void pko_router(const void* x, const void* w, int dtype, const float* bias, const float* escale,
                const float* emask, float temperature, float renorm_eps, int64_t T, int H, int E,
                int k, float* probs, float* logits_out, int32_t* idx, float* wts);
void pko_capacity_slots(const int32_t* idx, int64_t A, int E, int64_t capacity, int32_t* slot,
                        int32_t* count);
void pko_quant_scatter(const void* k_src, const void* v_src, int dtype, int64_t n_src, int fanout,
                       int D, int group, int scheme, const int32_t* cache_id, const int32_t* slot,
                       const int64_t* row_base, const int32_t* fill, const int32_t* cap,
                       int64_t dst_row0, void* k_codes, void* v_codes, void* k_scale, void* v_scale,
                       void* k_zero, void* v_zero, float* acc, float* ts, float now);
void pko_gather_dequant(const void* codes, const void* scale, const void* zero, int D, int group,
                        int scheme, const int64_t* rows, int64_t row0, int64_t n, float* out);
void pko_evict_select(int policy, const float* acc, const float* ts, const int64_t* row_base,
                      const int32_t* fill, const int32_t* n_heavy, const int32_t* n_recent,
                      int n_caches, uint8_t* keep_flag, int32_t* keep_index, int32_t* new_len);
void pko_compact_plane(void* plane, int64_t row_bytes, const int64_t* row_base,
                       const int32_t* keep_index, const int32_t* new_len, int n_caches);
}

#define HIP_OK(call)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) {                                                               \
      std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      std::exit(2);                                                                       \
    }                                                                                     \
  } while (0)

#define PIKV_CALL(call)                                                                   \
  do {                                                                                    \
    int rc_ = (call);                                                                     \
    if (rc_ != PIKV_OK) {                                                                 \
      std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #call, pikv_status_string(rc_)); \
      std::exit(3);                                                                       \
    }                                                                                     \
  } while (0)

static int failures = 0;
static void expect(bool ok, const char* what) {
  std::printf("%-58s %s\n", what, ok ? "ok" : "MISMATCH");
  std::fflush(stdout);
  if (!ok) ++failures;
}

// device buffer that mirrors a host vector
template <typename T>
struct Dev {
  T* p = nullptr;
  size_t n = 0;
  explicit Dev(size_t count) : n(count) { HIP_OK(hipMalloc((void**)&p, (count ? count : 1) * sizeof(T))); }
  explicit Dev(const std::vector<T>& h) : Dev(h.size()) { up(h); }
  ~Dev() { (void)hipFree(p); }
  void up(const std::vector<T>& h) { HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> down() const {
    std::vector<T> h(n);
    HIP_OK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
  void zero() { HIP_OK(hipMemset(p, 0, (n ? n : 1) * sizeof(T))); }
};

static uint32_t rng_state = 0x1234567u;
static float urand() {  // xorshift, uniform in [0, 1)
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 17;
  rng_state ^= rng_state << 5;
  return (float)(rng_state >> 8) * (1.0f / 16777216.0f);
}
static float nrand() {  // roughly normal
  float s = 0.f;
  for (int i = 0; i < 12; ++i) s += urand();
  return s - 6.0f;
}
static uint16_t to_bf16(float f) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

int main() {
  const int64_t T = 1536;
  const int E = 8, K = 2, heads = 4, dh = 64, D = heads * dh, group = dh;
  const int scheme = PIKV_Q_I8_SYM;
  const int64_t capacity = (int64_t)((double)T * 1.25 * K / E);  // 480
  const int64_t A = T * K;
  const int cap_rows = 400;  // smaller than the router capacity: the surplus is dropped
  std::printf("abi_parity: T=%lld E=%d k=%d D=%d capacity=%lld cache rows=%d, ABI %d\n", (long long)T, E, K, D,
              (long long)capacity, cap_rows, pikv_abi_version());

  // ---- router tail + capacity slots ------------------------------------------------
  std::vector<float> logits((size_t)T * E);
  for (auto& v : logits) v = 2.0f * nrand();
  for (int64_t t = 0; t < T; t += 7) logits[t * E + 3] = logits[t * E + 5];  // exact ties
  std::vector<float> eye((size_t)E * E, 0.f);
  for (int e = 0; e < E; ++e) eye[(size_t)e * E + e] = 1.0f;
  std::vector<float> probs_ref((size_t)T * E), w_ref((size_t)A);
  std::vector<int32_t> idx_ref((size_t)A), slot_ref((size_t)A), count_ref(E);
  pko_router(logits.data(), eye.data(), PIKV_F32, nullptr, nullptr, nullptr, 1.0f, 0.0f, T, E, E, K,
             probs_ref.data(), nullptr, idx_ref.data(), w_ref.data());
  pko_capacity_slots(idx_ref.data(), A, E, capacity, slot_ref.data(), count_ref.data());

  Dev<float> d_logits(logits), d_probs((size_t)T * E), d_w((size_t)A);
  Dev<int32_t> d_idx((size_t)A), d_slot((size_t)A), d_count(E);
  const int64_t ws_bytes = pikv_router_workspace_bytes(T, E, K);
  Dev<uint8_t> d_ws((size_t)ws_bytes);
  PIKV_CALL(pikv_router_tail(d_logits.p, nullptr, nullptr, nullptr, nullptr, 1.0f, 0.0f, 1, PIKV_ROUTER_SINGLE, T, E, K,
                             capacity,
                             d_probs.p, d_idx.p, d_w.p, d_slot.p, d_count.p, d_ws.p, ws_bytes, nullptr));
  HIP_OK(hipDeviceSynchronize());
  expect(d_idx.down() == idx_ref, "router: expert indices (ties to the lower index)");
  expect(d_slot.down() == slot_ref, "router: capacity slots");
  expect(d_count.down() == count_ref, "router: per-expert counts");
  {
    const std::vector<float> w = d_w.down();
    float worst = 0.f;
    for (size_t i = 0; i < w.size(); ++i) worst = std::fmax(worst, std::fabs(w[i] - w_ref[i]));
    expect(worst <= 1e-6f, "router: renormalised weights within 1e-6");
  }

  // ---- quantise + scatter, advance ----------------------------------------------------
  std::vector<uint16_t> k_src((size_t)T * D), v_src((size_t)T * D);
  for (auto& v : k_src) v = to_bf16(nrand());
  for (auto& v : v_src) v = to_bf16(3.0f * nrand());
  for (int i = 0; i < D; ++i) k_src[5 * D + i] = to_bf16(0.25f);  // a constant row: max == min
  std::vector<int64_t> row_base(E);
  std::vector<int32_t> fill(E, 0), cap(E, cap_rows);
  for (int c = 0; c < E; ++c) row_base[c] = (int64_t)c * cap_rows;
  fill[2] = 37;  // one cache already holds rows
  const int64_t rows = (int64_t)E * cap_rows;
  const int ng = D / group;
  std::vector<int8_t> kc_ref((size_t)rows * D, 0), vc_ref((size_t)rows * D, 0);
  std::vector<float> ks_ref((size_t)rows * ng, 0.f), vs_ref((size_t)rows * ng, 0.f), acc_ref((size_t)rows, -1.f),
      ts_ref((size_t)rows, -1.f);
  pko_quant_scatter(k_src.data(), v_src.data(), PIKV_BF16, T, K, D, group, scheme, idx_ref.data(), slot_ref.data(),
                    row_base.data(), fill.data(), cap.data(), 0, kc_ref.data(), vc_ref.data(), ks_ref.data(),
                    vs_ref.data(), nullptr, nullptr, acc_ref.data(), ts_ref.data(), 3.0f);

  Dev<uint16_t> d_ksrc(k_src), d_vsrc(v_src);
  Dev<int64_t> d_base(row_base);
  Dev<int32_t> d_fill(fill), d_cap(cap);
  Dev<int8_t> d_kc((size_t)rows * D), d_vc((size_t)rows * D);
  Dev<float> d_ks((size_t)rows * ng), d_vs((size_t)rows * ng);
  d_kc.zero(); d_vc.zero(); d_ks.zero(); d_vs.zero();
  Dev<float> d_acc(std::vector<float>((size_t)rows, -1.f)), d_ts(std::vector<float>((size_t)rows, -1.f));
  PIKV_CALL(pikv_quant_scatter(d_ksrc.p, d_vsrc.p, PIKV_BF16, T, K, D, group, scheme, d_idx.p, d_slot.p, d_base.p,
                               d_fill.p, d_cap.p, E, d_kc.p, d_vc.p, d_ks.p, d_vs.p, nullptr, nullptr, d_acc.p,
                               d_ts.p, 3.0f, nullptr));
  PIKV_CALL(pikv_cache_advance(d_fill.p, d_count.p, d_cap.p, E, capacity, nullptr));
  HIP_OK(hipDeviceSynchronize());
  expect(d_kc.down() == kc_ref, "quant_scatter: K codes");
  expect(d_vc.down() == vc_ref, "quant_scatter: V codes");
  expect(d_ks.down() == ks_ref, "quant_scatter: K scales");
  expect(d_vs.down() == vs_ref, "quant_scatter: V scales");
  expect(d_acc.down() == acc_ref, "quant_scatter: accumulators of written rows reset");
  expect(d_ts.down() == ts_ref, "quant_scatter: timestamps of written rows");
  std::vector<int32_t> fill_ref(E);
  for (int c = 0; c < E; ++c) {
    const int64_t add = count_ref[c] < capacity ? count_ref[c] : capacity;
    fill_ref[c] = (int32_t)(fill[c] + add < cap[c] ? fill[c] + add : cap[c]);
  }
  expect(d_fill.down() == fill_ref, "cache_advance: fill counts (clamped to the capacity)");

  // ---- gather + dequantise ---------------------------------------------------------------
  std::vector<float> dq_ref((size_t)rows * D);
  pko_gather_dequant(kc_ref.data(), ks_ref.data(), nullptr, D, group, scheme, nullptr, 0, rows, dq_ref.data());
  Dev<float> d_dq((size_t)rows * D);
  PIKV_CALL(pikv_gather_dequant(d_kc.p, d_ks.p, nullptr, D, group, scheme, nullptr, 0, rows, d_dq.p, PIKV_F32, nullptr));
  HIP_OK(hipDeviceSynchronize());
  {
    const std::vector<float> dq = d_dq.down();
    expect(std::memcmp(dq.data(), dq_ref.data(), dq.size() * sizeof(float)) == 0, "gather_dequant: float32 rows");
  }

  // ---- H2O budget, eviction select, compaction --------------------------------------------
  std::vector<float> acc((size_t)rows), ts((size_t)rows);
  for (auto& v : acc) v = std::floor(urand() * 16.0f) / 16.0f;  // many exact ties
  for (auto& v : ts) v = std::floor(urand() * 9.0f);
  d_acc.up(acc);
  d_ts.up(ts);
  const double heavy_ratio = 0.2, recent_ratio = 0.1;
  std::vector<int32_t> nh_ref(E), nr_ref(E);
  for (int c = 0; c < E; ++c) {
    nh_ref[c] = (int32_t)((double)fill_ref[c] * heavy_ratio);
    nr_ref[c] = (int32_t)((double)fill_ref[c] * recent_ratio);
    if (nh_ref[c] < 1) nh_ref[c] = 1;
    if (nr_ref[c] < 1) nr_ref[c] = 1;
  }
  std::vector<uint8_t> flag_ref((size_t)rows, 0);
  std::vector<int32_t> kidx_ref((size_t)rows, 0), newlen_ref(E);
  pko_evict_select(PIKV_EVICT_H2O, acc.data(), ts.data(), row_base.data(), fill_ref.data(), nh_ref.data(),
                   nr_ref.data(), E, flag_ref.data(), kidx_ref.data(), newlen_ref.data());

  Dev<int32_t> d_nh(E), d_nr(E), d_kidx((size_t)rows), d_newlen(E);
  Dev<uint8_t> d_flag((size_t)rows);
  PIKV_CALL(pikv_h2o_budget(d_fill.p, E, heavy_ratio, recent_ratio, d_nh.p, d_nr.p, nullptr));
  PIKV_CALL(pikv_evict_select(PIKV_EVICT_H2O, d_acc.p, d_ts.p, d_base.p, d_fill.p, d_nh.p, d_nr.p, E, cap_rows,
                              d_flag.p, d_kidx.p, d_newlen.p, nullptr, 0, nullptr));
  HIP_OK(hipDeviceSynchronize());
  expect(d_nh.down() == nh_ref && d_nr.down() == nr_ref, "h2o_budget: heavy / recent budgets");
  expect(d_newlen.down() == newlen_ref, "evict_select: survivors per cache");
  {
    const std::vector<uint8_t> flag = d_flag.down();
    const std::vector<int32_t> kidx = d_kidx.down();
    bool f_ok = true, i_ok = true;
    for (int c = 0; c < E; ++c) {
      for (int i = 0; i < fill_ref[c]; ++i) f_ok = f_ok && flag[row_base[c] + i] == flag_ref[row_base[c] + i];
      for (int j = 0; j < newlen_ref[c]; ++j) i_ok = i_ok && kidx[row_base[c] + j] == kidx_ref[row_base[c] + j];
    }
    expect(f_ok, "evict_select: keep flags (heavy UNION recent, ties by index)");
    expect(i_ok, "evict_select: ascending survivor lists");
  }

  void* planes[4] = {d_kc.p, d_ks.p, d_acc.p, d_ts.p};
  const int64_t plane_bytes[4] = {(int64_t)D, (int64_t)ng * 4, 4, 4};
  PIKV_CALL(pikv_compact_rows(planes, plane_bytes, 4, d_base.p, d_kidx.p, d_newlen.p, d_fill.p, E, nullptr));
  HIP_OK(hipDeviceSynchronize());
  pko_compact_plane(kc_ref.data(), D, row_base.data(), kidx_ref.data(), newlen_ref.data(), E);
  pko_compact_plane(ks_ref.data(), (int64_t)ng * 4, row_base.data(), kidx_ref.data(), newlen_ref.data(), E);
  pko_compact_plane(acc.data(), 4, row_base.data(), kidx_ref.data(), newlen_ref.data(), E);
  {
    const std::vector<int8_t> kc = d_kc.down();
    const std::vector<float> ks = d_ks.down(), ac = d_acc.down();
    bool ok = true;
    for (int c = 0; c < E; ++c)
      for (int j = 0; j < newlen_ref[c]; ++j) {
        const int64_t r = row_base[c] + j;
        ok = ok && std::memcmp(&kc[r * D], &kc_ref[r * D], D) == 0;
        ok = ok && std::memcmp(&ks[r * ng], &ks_ref[r * ng], ng * 4) == 0;
        ok = ok && std::memcmp(&ac[r], &acc[r], 4) == 0;
      }
    expect(ok, "compact_rows: codes, scales and accumulators of the survivors");
  }
  expect(d_fill.down() == newlen_ref, "compact_rows: fill = survivors");

  if (failures) {
    std::printf("abi_parity: %d check(s) FAILED\n", failures);
    return 1;
  }
  std::printf("abi_parity: ALL OK\n");
  return 0;
}
