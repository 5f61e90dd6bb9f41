// API-compatible fake quantisation: min/max over ALL rows of each block of
// `group` columns (the domain of QuantizedCompressor.forward in the reference,
// core/single/pikv_compression.py:474-506), output = dequantised floats, plus the
// mean squared error per column block.
//
// Four small launches: partial min/max per (column block, row chunk); reduce to
// (min, max, scale, zero) per column block; apply + partial squared error in
// double; fixed-order sum of the partials.  Everything is order-deterministic.
// The pre-calibrated mode of the same class (core/single/pikv_compression.py:430-472)
// skips the first two launches and applies one given (scale, zero) to every element.
#include "common.hpp"

namespace pikv {

constexpr int kFqRows = 256;  // rows per chunk

struct FqMeta {
  float mn, mx;
};

__device__ __forceinline__ float block_reduce_minmax(float v, bool is_max, float* sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v = is_max ? group_max<64>(v) : group_min<64>(v);
  __syncthreads();
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  float r = sh[0];
  for (int w = 1; w < 4; ++w) r = is_max ? fmaxf(r, sh[w]) : fminf(r, sh[w]);
  return r;
}

__global__ __launch_bounds__(256) void fq_minmax_kernel(const float* __restrict__ x, int64_t N, int H,
                                                        int group, int64_t n_chunks,
                                                        float* __restrict__ part) {
  __shared__ float sh[4];
  const int cb = blockIdx.x;
  const int64_t chunk = blockIdx.y;
  const int c0 = cb * group;
  const int gw = (H - c0) < group ? (H - c0) : group;
  const int64_t r0 = chunk * kFqRows;
  const int64_t rows = (N - r0) < kFqRows ? (N - r0) : kFqRows;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  // 16-byte accesses, four of them in flight per thread, where the block's columns and the rows allow
  // it (32768 x 4096 float32, fake-quantisation as a whole: 507 -> 341 us); else one element at a time
  const bool vec = (gw % 4 == 0) && (H % 4 == 0) && (c0 % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  if (vec) {
    const int q4 = gw / 4;
    const int64_t n4 = rows * q4;
    for (int64_t e0 = threadIdx.x; e0 < n4; e0 += 256 * 4) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t e = e0 + 256 * u < n4 ? e0 + 256 * u : e0;
        v[u] = ld16(reinterpret_cast<const char*>(x + (r0 + e / q4) * H + c0 + 4 * (int)(e % q4)));
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float f[4] = {__uint_as_float(v[u].x), __uint_as_float(v[u].y), __uint_as_float(v[u].z), __uint_as_float(v[u].w)};
#pragma unroll
        for (int q = 0; q < 4; ++q) { mn = fminf(mn, f[q]); mx = fmaxf(mx, f[q]); }
      }
    }
  } else {
    for (int64_t e = threadIdx.x; e < rows * gw; e += 256) {
      const float v = x[(r0 + e / gw) * H + c0 + (int)(e % gw)];
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
  }
  mn = block_reduce_minmax(mn, false, sh);
  mx = block_reduce_minmax(mx, true, sh);
  if (threadIdx.x == 0) {
    part[((int64_t)cb * n_chunks + chunk) * 2] = mn;
    part[((int64_t)cb * n_chunks + chunk) * 2 + 1] = mx;
  }
}

__global__ __launch_bounds__(256) void fq_params_kernel(const float* __restrict__ part,
                                                        int64_t n_chunks, int bits, int symmetric,
                                                        float* __restrict__ stats) {
  __shared__ float sh[4];
  const int cb = blockIdx.x;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t i = threadIdx.x; i < n_chunks; i += 256) {
    mn = fminf(mn, part[((int64_t)cb * n_chunks + i) * 2]);
    mx = fmaxf(mx, part[((int64_t)cb * n_chunks + i) * 2 + 1]);
  }
  mn = block_reduce_minmax(mn, false, sh);
  mx = block_reduce_minmax(mx, true, sh);
  if (threadIdx.x == 0) {
    float scale, zero;
    const float lo = mn;
    float hi = mx;
    if (hi == lo) hi = lo + 1e-5f;
    const int qmin = symmetric ? -(1 << (bits - 1)) : 0;
    const int qmax = symmetric ? (1 << (bits - 1)) - 1 : (1 << bits) - 1;
    const float qr = (float)(qmax - qmin);
    if (symmetric) {
      scale = (2.0f * fmaxf(fabsf(lo), fabsf(hi))) / qr;
      zero = 0.f;
    } else {
      scale = (hi - lo) / qr;
      zero = (float)qmin - rintf(lo / scale);
    }
    stats[cb * 4 + 0] = lo;
    stats[cb * 4 + 1] = hi;
    stats[cb * 4 + 2] = scale;
    stats[cb * 4 + 3] = zero;
  }
}

__global__ __launch_bounds__(256) void fq_apply_kernel(const float* __restrict__ x, int64_t N, int H,
                                                       int group, int64_t n_chunks, int bits,
                                                       int symmetric, const float* __restrict__ stats,
                                                       int stats_stride, float* __restrict__ out,
                                                       double* __restrict__ err_part) {
  __shared__ double shd[256];
  const int cb = blockIdx.x;
  const int64_t chunk = blockIdx.y;
  const int c0 = cb * group;
  const int gw = (H - c0) < group ? (H - c0) : group;
  const int64_t r0 = chunk * kFqRows;
  const int64_t rows = (N - r0) < kFqRows ? (N - r0) : kFqRows;
  // stats_stride 4: one (min, max, scale, zero) row per column block; 0: one row for all
  const float scale = stats[cb * stats_stride + 2];
  const float zero = stats[cb * stats_stride + 3];
  const float qmin = symmetric ? -(float)(1 << (bits - 1)) : 0.f;
  const float qmax = symmetric ? (float)((1 << (bits - 1)) - 1) : (float)((1 << bits) - 1);
  double err = 0.0;
  auto fq = [&](float v) {
    float y = v / scale;
    y = y + zero;
    y = rintf(y);
    y = fminf(fmaxf(y, qmin), qmax);
    const float dq = (y - zero) * scale;
    const double d = (double)v - (double)dq;
    err += d * d;
    return dq;
  };
  const bool vec = (gw % 4 == 0) && (H % 4 == 0) && (c0 % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                   ((reinterpret_cast<uintptr_t>(out) & 15) == 0);
  if (vec) {   // 16-byte accesses, four of them in flight per thread
    const int q4 = gw / 4;
    const int64_t n4 = rows * q4;
    for (int64_t e0 = threadIdx.x; e0 < n4; e0 += 256 * 4) {
      uint4 v[4];
      int64_t idx[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t e = e0 + 256 * u < n4 ? e0 + 256 * u : e0;
        idx[u] = (r0 + e / q4) * H + c0 + 4 * (int)(e % q4);
        v[u] = ld16(reinterpret_cast<const char*>(x + idx[u]));
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (e0 + 256 * u < n4) {
          const float o0 = fq(__uint_as_float(v[u].x)), o1 = fq(__uint_as_float(v[u].y));
          const float o2 = fq(__uint_as_float(v[u].z)), o3 = fq(__uint_as_float(v[u].w));
          st16(reinterpret_cast<char*>(out + idx[u]),
               make_uint4(__float_as_uint(o0), __float_as_uint(o1), __float_as_uint(o2), __float_as_uint(o3)));
        }
      }
    }
  } else {
    for (int64_t e = threadIdx.x; e < rows * gw; e += 256) {
      const int64_t i = (r0 + e / gw) * H + c0 + (int)(e % gw);
      out[i] = fq(x[i]);
    }
  }
  shd[threadIdx.x] = err;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) shd[threadIdx.x] += shd[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) err_part[(int64_t)cb * n_chunks + chunk] = shd[0];
}

__global__ void fq_err_kernel(const double* __restrict__ err_part, int64_t n_chunks, int64_t N, int H,
                              int group, float* __restrict__ sq_err) {
  const int cb = blockIdx.x;
  if (threadIdx.x != 0) return;
  const int c0 = cb * group;
  const int gw = (H - c0) < group ? (H - c0) : group;
  double s = 0.0;
  for (int64_t i = 0; i < n_chunks; ++i) s += err_part[(int64_t)cb * n_chunks + i];
  sq_err[cb] = (float)(s / ((double)N * (double)gw));
}

static int64_t fq_chunks(int64_t N) { return (N + kFqRows - 1) / kFqRows; }

}  // namespace pikv

using namespace pikv;

extern "C" int64_t pikv_fakequant_workspace_bytes(int64_t N, int H, int group) {
  if (N <= 0 || H <= 0 || group <= 0) return 0;
  const int64_t nblk = (H + group - 1) / group;
  // per (block, chunk): two floats (min, max) and one double (squared error)
  return (nblk * fq_chunks(N) * 16 + 255) / 256 * 256;
}

extern "C" int pikv_fakequant_colblocks(const float* x, int64_t N, int H, int group, int bits,
                                        int symmetric, float* out, float* stats, float* sq_err,
                                        void* workspace, int64_t workspace_bytes, void* stream) {
  if (!x || !out || !stats || !sq_err) return PIKV_ERR_NULL;
  if (N < 0 || H < 1 || group < 1) return PIKV_ERR_SHAPE;
  if (bits < 2 || bits > 16) return PIKV_ERR_UNSUPPORTED;
  if (N == 0) return PIKV_OK;
  if (!workspace) return PIKV_ERR_NULL;
  if (workspace_bytes < pikv_fakequant_workspace_bytes(N, H, group)) return PIKV_ERR_WORKSPACE;
  const int64_t nblk = (H + group - 1) / group;
  const int64_t nch = fq_chunks(N);
  if (nblk > 0x7fffffffLL || nch > 65535) return PIKV_ERR_SHAPE;
  // layout: doubles first (8-byte aligned), then the float pairs
  double* err_part = reinterpret_cast<double*>(workspace);
  float* part = reinterpret_cast<float*>(err_part + nblk * nch);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)nblk, (unsigned)nch);
  hipLaunchKernelGGL(fq_minmax_kernel, grid, dim3(256), 0, st, x, N, H, group, nch, part);
  hipLaunchKernelGGL(fq_params_kernel, dim3((unsigned)nblk), dim3(256), 0, st, part, nch, bits,
                     symmetric, stats);
  hipLaunchKernelGGL(fq_apply_kernel, grid, dim3(256), 0, st, x, N, H, group, nch, bits, symmetric,
                     stats, 4, out, err_part);
  hipLaunchKernelGGL(fq_err_kernel, dim3((unsigned)nblk), dim3(64), 0, st, err_part, nch, N, H, group,
                     sq_err);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}

extern "C" int pikv_fakequant_preset(const float* x, int64_t N, int H, int group, int bits,
                                     int symmetric, const float* preset, float* out, float* sq_err,
                                     void* workspace, int64_t workspace_bytes, void* stream) {
  if (!x || !out || !preset || !sq_err) return PIKV_ERR_NULL;
  if (N < 0 || H < 1 || group < 1) return PIKV_ERR_SHAPE;
  if (bits < 2 || bits > 16) return PIKV_ERR_UNSUPPORTED;
  if (N == 0) return PIKV_OK;
  if (!workspace) return PIKV_ERR_NULL;
  if (workspace_bytes < pikv_fakequant_workspace_bytes(N, H, group)) return PIKV_ERR_WORKSPACE;
  const int64_t nblk = (H + group - 1) / group;
  const int64_t nch = fq_chunks(N);
  if (nblk > 0x7fffffffLL || nch > 65535) return PIKV_ERR_SHAPE;
  double* err_part = reinterpret_cast<double*>(workspace);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)nblk, (unsigned)nch);
  hipLaunchKernelGGL(fq_apply_kernel, grid, dim3(256), 0, st, x, N, H, group, nch, bits, symmetric,
                     preset, 0, out, err_part);
  hipLaunchKernelGGL(fq_err_kernel, dim3((unsigned)nblk), dim3(64), 0, st, err_part, nch, N, H, group,
                     sq_err);
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
