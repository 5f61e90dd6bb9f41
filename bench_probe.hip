// Streaming probes for bench.py / bench_profile.py (libbench_probe.so; NOT part of libpikv_hip.so
// and not declared in include/pikv_hip.h): the access pattern every kernel of the library uses for
// its bulk data - 16 bytes per lane, 1 KiB contiguous per wavefront, several accesses in flight per
// lane - over a plain buffer.  They put the practical HBM rates of the machine at hand (read only,
// write only, read + write) on record next to the kernels' own figures, and give profiler counters a
// launch of exactly known traffic to be scaled by.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pikv {

typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st16_stream(void* p, uint4 v) {
  probe_u32x4 t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<probe_u32x4*>(p));
}

constexpr int kProbeUnroll = 8;                              // 16-byte accesses in flight per lane
constexpr int64_t kProbeBlockBytes = 256 * 16 * kProbeUnroll;  // 32 KiB per block

// mode 0: read src, keep a running xor; the (never true) comparison keeps the loads alive
// mode 1: write a constant pattern to dst
// mode 2: copy src to dst
template <int MODE, bool STREAM_STORE>
__global__ __launch_bounds__(256) void stream_probe_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                           int64_t n16, uint32_t* __restrict__ sink) {
  const int64_t base = (int64_t)blockIdx.x * (256 * kProbeUnroll) + threadIdx.x;
  uint4 v[kProbeUnroll];
#pragma unroll
  for (int u = 0; u < kProbeUnroll; ++u) {
    const int64_t i = base + (int64_t)u * 256;
    if constexpr (MODE != 1) v[u] = i < n16 ? src[i] : make_uint4(0, 0, 0, 0);
    else v[u] = make_uint4(0x01020304u, (uint32_t)i, 0x0badc0deu, (uint32_t)u);
  }
  if constexpr (MODE == 0) {
    uint32_t acc = 0;
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (acc == 0x9e3779b9u && sink) sink[0] = acc;  // practically never: the data would have to conspire
  } else {
#pragma unroll
    for (int u = 0; u < kProbeUnroll; ++u) {
      const int64_t i = base + (int64_t)u * 256;
      if (i < n16) {
        if constexpr (STREAM_STORE) st16_stream(dst + i, v[u]);
        else dst[i] = v[u];
      }
    }
  }
}

// modes 3 / 4: what small stores cost a saturated read stream.  Persistent blocks of eight wavefronts
// walk `tiles` tiles of 64 KiB each (16 bytes per lane and access, two tiles in flight per block: the
// shape of the one-pass decode kernels' tile loop); mode 4 additionally stores 8 bytes per lane and tile
// (4 KiB per block and tile, 6 % of what it reads) to dst, as those kernels do for the H2O bookkeeping.
constexpr int kMixTileBytes = 512 * 8 * 16;
template <bool STORES>
__global__ __launch_bounds__(512) void mixed_probe_kernel(const uint4* __restrict__ src, uint2* __restrict__ dst,
                                                          int tiles, uint32_t* __restrict__ sink) {
  const int tid = threadIdx.x;
  const uint4* s = src + (int64_t)blockIdx.x * tiles * (kMixTileBytes / 16);
  uint2* d = dst + (int64_t)blockIdx.x * tiles * 512;
  uint4 a[8], b[8];
  uint32_t acc = 0;
  auto issue = [&](int t, uint4* r) {   // a tile past the end repeats the last one
    const int tt = t < tiles ? t : tiles - 1;
#pragma unroll
    for (int u = 0; u < 8; ++u) r[u] = s[(int64_t)tt * (kMixTileBytes / 16) + u * 512 + tid];
  };
  auto use = [&](const uint4* r) {
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= r[u].x ^ r[u].y ^ r[u].z ^ r[u].w;
  };
  issue(0, a);
  asm volatile("" ::: "memory");
  issue(1, b);
  asm volatile("" ::: "memory");
  for (int t = 0; t < tiles; t += 2) {   // tiles is even
    use(a);
    asm volatile("" ::: "memory");
    issue(t + 2, a);
    asm volatile("" ::: "memory");
    if constexpr (STORES) d[(int64_t)t * 512 + tid] = make_uint2(acc, (uint32_t)t);
    use(b);
    asm volatile("" ::: "memory");
    issue(t + 3, b);
    asm volatile("" ::: "memory");
    if constexpr (STORES) d[(int64_t)(t + 1) * 512 + tid] = make_uint2(acc, (uint32_t)t);
  }
  if (acc == 0x9e3779b9u && sink) sink[0] = acc;
}

}  // namespace pikv

using namespace pikv;

// 0 on success, negative on a bad argument or a refused launch.  Modes 3 and 4: `bytes` (read from src) must be a
// multiple of 8 MiB; mode 4 writes bytes / 16 to the front of dst.
extern "C" int bench_stream_probe(int mode, const void* src, void* dst, int64_t bytes, int streaming_stores,
                                 void* sink, void* stream) {
  if (mode == 3 || mode == 4) {
    // 128 tiles per block; every address the kernel forms lies inside src[0, bytes) and dst[0, bytes / 16)
    constexpr int tiles = 128;
    if (!src || (mode == 4 && !dst) || bytes <= 0 || bytes % ((int64_t)tiles * kMixTileBytes) != 0) return -2;
    const int64_t nb = bytes / ((int64_t)tiles * kMixTileBytes);
    if (nb > 0x7fffffffLL) return -2;
    hipStream_t st3 = (hipStream_t)stream;
    if (mode == 3)
      hipLaunchKernelGGL((mixed_probe_kernel<false>), dim3((unsigned)nb), dim3(512), 0, st3,
                         reinterpret_cast<const uint4*>(src), reinterpret_cast<uint2*>(dst), tiles,
                         reinterpret_cast<uint32_t*>(sink));
    else
      hipLaunchKernelGGL((mixed_probe_kernel<true>), dim3((unsigned)nb), dim3(512), 0, st3,
                         reinterpret_cast<const uint4*>(src), reinterpret_cast<uint2*>(dst), tiles,
                         reinterpret_cast<uint32_t*>(sink));
    return hipGetLastError() == hipSuccess ? 0 : -5;
  }
  if (mode < 0 || mode > 2) return -3;
  if ((mode != 1 && !src) || (mode != 0 && !dst)) return -1;
  if (bytes < 0 || bytes % 16 != 0) return -2;
  if ((reinterpret_cast<uintptr_t>(src) & 15) || (reinterpret_cast<uintptr_t>(dst) & 15)) return -2;
  if (bytes == 0) return 0;
  const int64_t blocks = (bytes + kProbeBlockBytes - 1) / kProbeBlockBytes;
  if (blocks > 0x7fffffffLL) return -2;
  const int64_t n16 = bytes / 16;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks);
  const uint4* s = reinterpret_cast<const uint4*>(src);
  uint4* d = reinterpret_cast<uint4*>(dst);
  uint32_t* sk = reinterpret_cast<uint32_t*>(sink);
  if (mode == 0) hipLaunchKernelGGL((stream_probe_kernel<0, false>), grid, dim3(256), 0, st, s, d, n16, sk);
  else if (mode == 1 && streaming_stores) hipLaunchKernelGGL((stream_probe_kernel<1, true>), grid, dim3(256), 0, st, s, d, n16, sk);
  else if (mode == 1) hipLaunchKernelGGL((stream_probe_kernel<1, false>), grid, dim3(256), 0, st, s, d, n16, sk);
  else if (streaming_stores) hipLaunchKernelGGL((stream_probe_kernel<2, true>), grid, dim3(256), 0, st, s, d, n16, sk);
  else hipLaunchKernelGGL((stream_probe_kernel<2, false>), grid, dim3(256), 0, st, s, d, n16, sk);
  if (hipGetLastError() != hipSuccess) return -5;
  return 0;
}
