// Min-shift 8-bit quantisation of whole rows: the algebra of the reference's kernel
// facade, PiKVKernels.compress_kv(QUANT8) (core/single/pikv_kernels.py:215-246):
//   mn = min(row), mx = max(row), s = (mx - mn) / 255
//   q  = clamp(round((x - mn) / s), 0, 255)  as uint8
//   dq = q * s + mn
// It differs from the cache formula (integer zero point) in that the offset is the row
// minimum itself, so codes, metadata and dequantised floats are not interchangeable.
// float32 arithmetic in the reference's operation order: true division, round half to
// even, no reciprocal, no contraction.  A constant row has s = 0: 0/0 is NaN, which the
// uint8 conversion of the reference's CPU path turns into code 0, so dq = mn.
//
// One wavefront per row, four rows per block.  The row is read twice (minimum / maximum,
// then codes); the second read is served by the caches.  Rows whose width is a multiple of
// 16 move as 16-byte code stores and 16-byte float stores; other widths go element by element.
#include "common.hpp"

namespace pikv {

template <int DT>
__device__ __forceinline__ float load_elem(const void* p, int64_t i) {
  if constexpr (DT == PIKV_BF16) return bf16_bits_to_float(reinterpret_cast<const uint16_t*>(p)[i]);
  else return reinterpret_cast<const float*>(p)[i];
}

__device__ __forceinline__ uint32_t minshift_code(float x, float mn, float s) {
  float y = (x - mn) / s;
  y = rintf(y);
  y = (y != y) ? 0.0f : fminf(fmaxf(y, 0.0f), 255.0f);
  return (uint32_t)y;
}

// four consecutive source elements as floats (16 bytes of float32, 8 of bf16)
template <int DT>
__device__ __forceinline__ void load4_as_float(const void* base, int64_t elem_off, float (&out)[4]) {
  if constexpr (DT == PIKV_BF16) {
    const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(base) + elem_off * 2);
    out[0] = __uint_as_float(v.x << 16);
    out[1] = __uint_as_float(v.x & 0xffff0000u);
    out[2] = __uint_as_float(v.y << 16);
    out[3] = __uint_as_float(v.y & 0xffff0000u);
  } else {
    const uint4 v = ld16(reinterpret_cast<const char*>(base) + elem_off * 4);
    out[0] = __uint_as_float(v.x);
    out[1] = __uint_as_float(v.y);
    out[2] = __uint_as_float(v.z);
    out[3] = __uint_as_float(v.w);
  }
}

template <int DT, bool VEC>
__global__ __launch_bounds__(256) void minshift_rows_kernel(const void* __restrict__ src, int64_t n_rows, int D,
                                                            uint8_t* __restrict__ codes, float* __restrict__ dq,
                                                            float* __restrict__ scale, float* __restrict__ row_min) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= n_rows) return;  // uniform for the wavefront
  const int64_t e0 = row * D;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  // VEC: a wavefront walks its row in pieces of 1024 elements.  Float32 values (the source, the
  // dequantised output) move as four accesses of 16 bytes per lane, each of them one contiguous
  // kilobyte of the row: lane l, access j holds elements 256 j + 4 l .. + 3 of the piece.  (Sixteen
  // consecutive elements per lane make every access 16 bytes at a stride of 64, which stores at
  // a fraction of the rate: 341 us for 32768 x 4096 float32 against 293 us.)  The four code words of a lane cross LDS
  // so that the codes, too, leave as 16 bytes per lane.
  __shared__ uint32_t cx[4][256];
  constexpr int PIECE = 1024;
  if constexpr (VEC) {
    for (int p0 = 0; p0 < D; p0 += PIECE) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = p0 + 256 * j + 4 * lane;
        if (e < D) {
          float x[4];
          load4_as_float<DT>(src, e0 + e, x);
#pragma unroll
          for (int q = 0; q < 4; ++q) { mn = fminf(mn, x[q]); mx = fmaxf(mx, x[q]); }
        }
      }
    }
  } else {
    for (int i = lane; i < D; i += 64) {
      const float x = load_elem<DT>(src, e0 + i);
      mn = fminf(mn, x);
      mx = fmaxf(mx, x);
    }
  }
  group_minmax_dpp(mn, mx, 64);
  const float s = (mx - mn) / 255.0f;
  if (lane == 0) {
    scale[row] = s;
    row_min[row] = mn;
  }
  if constexpr (VEC) {
    for (int p0 = 0; p0 < D; p0 += PIECE) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = p0 + 256 * j + 4 * lane;
        uint32_t w = 0;
        if (e < D) {
          float x[4];
          load4_as_float<DT>(src, e0 + e, x);
          uint32_t c[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) c[q] = minshift_code(x[q], mn, s);
          w = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
          if (dq) {
            float o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float t = (float)c[q] * s;
              o[q] = t + mn;
            }
            st16(dq + e0 + e,
                 make_uint4(__float_as_uint(o[0]), __float_as_uint(o[1]), __float_as_uint(o[2]), __float_as_uint(o[3])));
          }
        }
        cx[wave][64 * j + lane] = w;   // code word of elements 256 j + 4 lane ..: word 64 j + lane of the piece
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if (p0 + 16 * lane < D)   // D is a multiple of 16: whole 16-byte runs
        st16(codes + e0 + p0 + 16 * lane, *reinterpret_cast<const uint4*>(&cx[wave][4 * lane]));
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  } else {
    for (int i = lane; i < D; i += 64) {
      const uint32_t c = minshift_code(load_elem<DT>(src, e0 + i), mn, s);
      codes[e0 + i] = (uint8_t)c;
      if (dq) {
        const float t = (float)c * s;
        dq[e0 + i] = t + mn;
      }
    }
  }
}

}  // namespace pikv

using namespace pikv;

extern "C" int pikv_quant8_minshift(const void* src, int src_dtype, int64_t n_rows, int D, uint8_t* codes,
                                    float* dq, float* scale, float* row_min, void* stream) {
  if (!src || !codes || !scale || !row_min) return PIKV_ERR_NULL;
  if (src_dtype != PIKV_F32 && src_dtype != PIKV_BF16) return PIKV_ERR_UNSUPPORTED;
  if (n_rows < 0 || D < 1) return PIKV_ERR_SHAPE;
  if (n_rows == 0) return PIKV_OK;
  const int64_t blocks = (n_rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return PIKV_ERR_SHAPE;
  const int esz = src_dtype == PIKV_BF16 ? 2 : 4;
  // 16-byte accesses need a row width of whole 16-element pieces and aligned planes
  const bool vec = D % 16 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(codes) & 15) == 0 && (reinterpret_cast<uintptr_t>(dq) & 15) == 0 &&
                   ((int64_t)D * esz) % 16 == 0;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks);
#define PIKV_MINSHIFT_LAUNCH(DT, V)                                                                   \
  hipLaunchKernelGGL((minshift_rows_kernel<DT, V>), grid, dim3(256), 0, st, src, n_rows, D, codes, dq, scale, row_min)
  if (src_dtype == PIKV_BF16) {
    if (vec) PIKV_MINSHIFT_LAUNCH(PIKV_BF16, true); else PIKV_MINSHIFT_LAUNCH(PIKV_BF16, false);
  } else {
    if (vec) PIKV_MINSHIFT_LAUNCH(PIKV_F32, true); else PIKV_MINSHIFT_LAUNCH(PIKV_F32, false);
  }
#undef PIKV_MINSHIFT_LAUNCH
  PIKV_CHECK_LAUNCH();
  return PIKV_OK;
}
