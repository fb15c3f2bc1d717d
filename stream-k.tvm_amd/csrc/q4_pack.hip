// Offline side of the Q4 path: nibble packing and group-wise quantisation of fp16 weights into the
// natural-order format the Q4 kernels read (element k of row n in nibble k&1 of byte Wq[n][k/2],
// streamk_fp16_ladder_block_reduce_q4.py:552).  The reference obtains its device layout by running
// LadderPermutate and LOP3Permutate over such an array on the CPU (:568-595); here the natural
// order is the device layout, so packing is all there is to do.
//
// Quantisation rule (the reference draws random nibbles and has none), per group of `group`
// K-values of one row:
//   levels = min(zero, 15 - zero), or 15 when that is 0 (zero point at an end: one-sided)
//   scale  = fp16_rn(max|w| / levels)                        (fp32 division)
//   q      = clamp(rint(w / scale) + zero, 0, 15)            (fp32 division, ties to even)
//   q      = zero when scale rounds to 0
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "../../include/streamk.h"
#include "sk_device.h"

namespace sk {
namespace {

__host__ __device__ inline int q4_levels(int zero) {
  const int m = zero < 15 - zero ? zero : 15 - zero;
  return m == 0 ? 15 : m;
}

__host__ __device__ inline uint32_t q4_quantize_one(float w, float scale, int zero) {
  if (scale == 0.f) return (uint32_t)zero;
  float q = rintf(w / scale) + (float)zero;
  q = q < 0.f ? 0.f : (q > 15.f ? 15.f : q);
  return (uint32_t)q;
}

// software binary16 <-> binary32 for the host path (round to nearest even)
inline float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31, man = h & 1023;
  float mag;
  if (exp == 0)
    mag = ldexpf((float)man, -24);
  else if (exp == 31)
    mag = man ? NAN : INFINITY;
  else
    mag = ldexpf((float)(man | 1024), (int)exp - 25);
  return sign ? -mag : mag;
}
inline uint16_t float_to_half_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000);
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return sign | (x > 0x7f800000u ? 0x7e00 : 0x7c00);
  if (x >= 0x477ff000u) return sign | 0x7c00;  // rounds to or beyond 65520: infinity
  if (x < 0x33000001u) return sign;            // at most half of the smallest subnormal: zero
  int e = (int)(x >> 23) - 127;
  uint32_t m = (x & 0x7fffffu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13;  // bits dropped
  uint32_t kept = m >> shift, rest = m & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rest > half || (rest == half && (kept & 1))) ++kept;
  if (e < -14) return sign | (uint16_t)kept;  // subnormal (a carry lands on the smallest normal)
  return sign | (uint16_t)(((uint32_t)(e + 15) << 10) + (kept - 1024));  // a carry bumps the exponent
}

// 16 lanes per group of 128: lane i quantises K-values [8i, 8i+8) of its group
__global__ __launch_bounds__(256) void quantize_q4_kernel(const half_t *W, uint32_t *wq, half_t *scales, int64_t chunks,
                                                          int chunks_per_row, int64_t ldw, int zero) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool live = i < chunks;  // chunks is a multiple of 16: a group is live or not as a whole
  const int64_t ic = live ? i : 0;
  const int64_t row = ic / chunks_per_row;
  const int c = (int)(ic % chunks_per_row);
  const half8v v = *reinterpret_cast<const half8v *>(W + row * ldw + (int64_t)c * 8);
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)v[e]));
#pragma unroll
  for (int m = 1; m < 16; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m));
  const half_t sh = (half_t)(amax / (float)q4_levels(zero));
  const float s = (float)sh;
  uint32_t word = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) word |= q4_quantize_one((float)v[e], s, zero) << (4 * e);
  if (live) {
    wq[i] = word;
    if ((c & 15) == 0) scales[row * (chunks_per_row / 16) + c / 16] = sh;
  }
}

// asymmetric rule: the group's range [lo, hi] (widened to contain 0) is mapped onto 0..15
__host__ __device__ inline float q4_zp_of(float lo, float scale) {
  if (scale == 0.f) return 0.f;
  float z = rintf(-lo / scale);
  return z < 0.f ? 0.f : (z > 15.f ? 15.f : z);
}

// 16 lanes per group of 128, as quantize_q4_kernel
__global__ __launch_bounds__(256) void quantize_q4_zp_kernel(const half_t *W, uint32_t *wq, half_t *scales, half_t *zeros,
                                                             int64_t chunks, int chunks_per_row, int64_t ldw) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool live = i < chunks;
  const int64_t ic = live ? i : 0;
  const int64_t row = ic / chunks_per_row;
  const int c = (int)(ic % chunks_per_row);
  const half8v v = *reinterpret_cast<const half8v *>(W + row * ldw + (int64_t)c * 8);
  float lo = 0.f, hi = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo = fminf(lo, (float)v[e]);
    hi = fmaxf(hi, (float)v[e]);
  }
#pragma unroll
  for (int m = 1; m < 16; m <<= 1) {
    lo = fminf(lo, __shfl_xor(lo, m));
    hi = fmaxf(hi, __shfl_xor(hi, m));
  }
  const half_t sh = (half_t)((hi - lo) / 15.f);
  const float s = (float)sh;
  const float z = q4_zp_of(lo, s);
  uint32_t word = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) word |= q4_quantize_one((float)v[e], s, (int)z) << (4 * e);
  if (live) {
    wq[i] = word;
    if ((c & 15) == 0) {
      scales[row * (chunks_per_row / 16) + c / 16] = sh;
      zeros[row * (chunks_per_row / 16) + c / 16] = (half_t)z;
    }
  }
}

// tiled position of byte b of row n (runs = K / 128 tiles per row block)
__host__ __device__ inline int64_t q4_tiled_offset(int64_t n, int64_t b, int64_t runs) {
  return ((n / 16) * runs + b / 64) * 1024 + (n % 16) * 64 + b % 64;
}

// one thread per 16 bytes of the tiled array (rows past N are written as zeros)
__global__ __launch_bounds__(256) void tile_q4_kernel(const uint4v *wq, uint4v *tiled, int64_t pieces, int64_t N,
                                                      int64_t runs) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= pieces) return;
  const int64_t tile = i / 64, in = i % 64;           // 64 pieces of 16 bytes per tile
  const int64_t n = (tile / runs) * 16 + in / 4, b = (tile % runs) * 64 + (in % 4) * 16;
  tiled[i] = n < N ? wq[(n * runs * 64 + b) / 16] : uint4v{0, 0, 0, 0};
}

}  // namespace
}  // namespace sk

using namespace sk;

extern "C" int sk_q4_tile_host(const uint8_t *Wq, int64_t N, int64_t K, uint8_t *tiled) {
  if (!Wq || !tiled) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || (K % 128)) return SK_ERR_SHAPE;
  const int64_t runs = K / 128, n16 = (N + 15) / 16 * 16;
  memset(tiled, 0, (size_t)(n16 * (K / 2)));
  for (int64_t n = 0; n < N; ++n)
    for (int64_t b = 0; b < K / 2; b += 64) memcpy(tiled + q4_tiled_offset(n, b, runs), Wq + n * (K / 2) + b, 64);
  return SK_OK;
}

extern "C" int sk_q4_untile_host(const uint8_t *tiled, int64_t N, int64_t K, uint8_t *Wq) {
  if (!Wq || !tiled) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || (K % 128)) return SK_ERR_SHAPE;
  const int64_t runs = K / 128;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t b = 0; b < K / 2; b += 64) memcpy(Wq + n * (K / 2) + b, tiled + q4_tiled_offset(n, b, runs), 64);
  return SK_OK;
}

extern "C" int sk_q4_tile(const void *Wq, int64_t N, int64_t K, void *tiled, void *stream) {
  if (!Wq || !tiled) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || (K % 128)) return SK_ERR_SHAPE;
  if ((reinterpret_cast<uintptr_t>(Wq) & 15) || (reinterpret_cast<uintptr_t>(tiled) & 15)) return SK_ERR_ALIGN;
  const int64_t runs = K / 128, pieces = (N + 15) / 16 * runs * 64;
  const int64_t blocks = (pieces + 255) / 256;
  if (blocks > 0x7fffffff) return SK_ERR_SHAPE;
  hipLaunchKernelGGL(tile_q4_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint4v *)Wq,
                     (uint4v *)tiled, pieces, N, runs);
  return hipGetLastError() == hipSuccess ? SK_OK : SK_ERR_LAUNCH;
}

extern "C" int sk_q4_pack_host(const uint8_t *q, int64_t N, int64_t K, uint8_t *Wq) {
  if (!q || !Wq) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || (K & 1)) return SK_ERR_SHAPE;
  for (int64_t i = 0; i < N * K; ++i)
    if (q[i] > 15) return SK_ERR_CONFIG;
  for (int64_t i = 0; i < N * K / 2; ++i) Wq[i] = (uint8_t)(q[2 * i] | (q[2 * i + 1] << 4));
  return SK_OK;
}

extern "C" int sk_q4_unpack_host(const uint8_t *Wq, int64_t N, int64_t K, uint8_t *q) {
  if (!q || !Wq) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || (K & 1)) return SK_ERR_SHAPE;
  for (int64_t i = 0; i < N * K / 2; ++i) {
    q[2 * i] = Wq[i] & 15;
    q[2 * i + 1] = Wq[i] >> 4;
  }
  return SK_OK;
}

extern "C" int sk_q4_quantize_host(const uint16_t *W, int64_t N, int64_t K, int64_t ldw, int group, int zero,
                                   uint8_t *Wq, uint16_t *scales) {
  if (!W || !Wq || !scales) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || ldw < K) return SK_ERR_SHAPE;
  if (group <= 0 || (group % 8) || (K % group) || zero < 0 || zero > 15) return SK_ERR_CONFIG;
  const int64_t groups = K / group;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t g = 0; g < groups; ++g) {
      const uint16_t *w = W + n * ldw + g * group;
      float amax = 0.f;
      for (int k = 0; k < group; ++k) {
        const float f = fabsf(half_bits_to_float(w[k]));
        if (!(f <= 65504.f)) return SK_ERR_CONFIG;  // NaN or infinity
        amax = f > amax ? f : amax;
      }
      const uint16_t sh = float_to_half_bits(amax / (float)q4_levels(zero));
      const float s = half_bits_to_float(sh);
      scales[n * groups + g] = sh;
      uint8_t *out = Wq + (n * K + g * group) / 2;
      for (int k = 0; k < group; k += 2)
        out[k / 2] = (uint8_t)(q4_quantize_one(half_bits_to_float(w[k]), s, zero) |
                               (q4_quantize_one(half_bits_to_float(w[k + 1]), s, zero) << 4));
    }
  return SK_OK;
}

extern "C" int sk_q4_quantize(const void *W, int64_t N, int64_t K, int64_t ldw, int group, int zero, void *Wq,
                              void *scales, void *stream) {
  if (!W || !Wq || !scales) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || ldw < K || (ldw % 8)) return SK_ERR_SHAPE;
  if (group != 128 || (K % group) || zero < 0 || zero > 15) return SK_ERR_CONFIG;
  if ((reinterpret_cast<uintptr_t>(W) & 15) || (reinterpret_cast<uintptr_t>(Wq) & 3) ||
      (reinterpret_cast<uintptr_t>(scales) & 1))
    return SK_ERR_ALIGN;
  const int64_t chunks = N * K / 8;
  const int64_t blocks = (chunks + 255) / 256;
  if (blocks > 0x7fffffff) return SK_ERR_SHAPE;
  hipLaunchKernelGGL(quantize_q4_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const half_t *)W,
                     (uint32_t *)Wq, (half_t *)scales, chunks, (int)(K / 8), ldw, zero);
  return hipGetLastError() == hipSuccess ? SK_OK : SK_ERR_LAUNCH;
}

extern "C" int sk_q4_quantize_zp_host(const uint16_t *W, int64_t N, int64_t K, int64_t ldw, int group, uint8_t *Wq,
                                      uint16_t *scales, uint16_t *zeros) {
  if (!W || !Wq || !scales || !zeros) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || ldw < K) return SK_ERR_SHAPE;
  if (group <= 0 || (group % 8) || (K % group)) return SK_ERR_CONFIG;
  const int64_t groups = K / group;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t g = 0; g < groups; ++g) {
      const uint16_t *w = W + n * ldw + g * group;
      float lo = 0.f, hi = 0.f;
      for (int k = 0; k < group; ++k) {
        const float f = half_bits_to_float(w[k]);
        if (!(fabsf(f) <= 65504.f)) return SK_ERR_CONFIG;  // NaN or infinity
        lo = f < lo ? f : lo;
        hi = f > hi ? f : hi;
      }
      const uint16_t sh = float_to_half_bits((hi - lo) / 15.f);
      const float s = half_bits_to_float(sh);
      const float z = q4_zp_of(lo, s);
      scales[n * groups + g] = sh;
      zeros[n * groups + g] = float_to_half_bits(z);
      uint8_t *out = Wq + (n * K + g * group) / 2;
      for (int k = 0; k < group; k += 2)
        out[k / 2] = (uint8_t)(q4_quantize_one(half_bits_to_float(w[k]), s, (int)z) |
                               (q4_quantize_one(half_bits_to_float(w[k + 1]), s, (int)z) << 4));
    }
  return SK_OK;
}

extern "C" int sk_q4_quantize_zp(const void *W, int64_t N, int64_t K, int64_t ldw, int group, void *Wq, void *scales,
                                 void *zeros, void *stream) {
  if (!W || !Wq || !scales || !zeros) return SK_ERR_NULL;
  if (N <= 0 || K <= 0 || ldw < K || (ldw % 8)) return SK_ERR_SHAPE;
  if (group != 128 || (K % group)) return SK_ERR_CONFIG;
  if ((reinterpret_cast<uintptr_t>(W) & 15) || (reinterpret_cast<uintptr_t>(Wq) & 3) ||
      (reinterpret_cast<uintptr_t>(scales) & 1) || (reinterpret_cast<uintptr_t>(zeros) & 1))
    return SK_ERR_ALIGN;
  const int64_t chunks = N * K / 8;
  const int64_t blocks = (chunks + 255) / 256;
  if (blocks > 0x7fffffff) return SK_ERR_SHAPE;
  hipLaunchKernelGGL(quantize_q4_zp_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const half_t *)W,
                     (uint32_t *)Wq, (half_t *)scales, (half_t *)zeros, chunks, (int)(K / 8), ldw);
  return hipGetLastError() == hipSuccess ? SK_OK : SK_ERR_LAUNCH;
}
