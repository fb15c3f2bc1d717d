// Measurement aid for bench.py (built into libstreamk_bench.so, not part of the library or its C ABI): what the
// matrix pipes of this part sustain with nothing else in flight.
// The published fp16 peak assumes the maximum clock; under its power limit the part clocks down as soon as the
// operands are not zero, by an amount that differs from box to box.  A benchmark that prices a GEMM against the
// peak can run this loop in the same process to say how much of the gap no GEMM kernel can close.
#include <hip/hip_runtime.h>


namespace sk {

typedef _Float16 half8d __attribute__((ext_vector_type(8)));
typedef float float4d __attribute__((ext_vector_type(4)));
typedef float float16d __attribute__((ext_vector_type(16)));

__device__ inline half8d diag_operand(unsigned &state, bool zeros) {
  half8d v;
  for (int e = 0; e < 8; ++e) {
    state = state * 1664525u + 1013904223u;
    v[e] = zeros ? (_Float16)0.f : (_Float16)((float)(state >> 8) * (2.0f / 16777216.0f) - 1.0f);
  }
  return v;
}

// every wave: 2^20 FLOP per iteration in the instruction pattern of the 256 x 256 tile kernels -- an 8 x 8 (4 x 4)
// grid of accumulator blocks, one A fragment held over a row of blocks while the B fragment changes, fragments
// U[-1,1) fp16 values that differ from lane to lane -- with no memory traffic at all.  (Operands that change
// on both sides with every MFMA draw more power per FLOP than any GEMM does and sustain less.)
template <bool WIDE>
__global__ __launch_bounds__(256) void mfma_only_kernel(float *out, int iters, int zeros) {
  unsigned state = (blockIdx.x * 256 + threadIdx.x) * 2654435761u + 12345u;
  half8d a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    a[i] = diag_operand(state, zeros != 0);
    b[i] = diag_operand(state, zeros != 0);
  }
  float s = 0.f;
  if (WIDE) {
    float16d acc[4][4];
    for (int i = 0; i < 4; ++i)
      for (int j = 0; j < 4; ++j)
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const int j = (i & 1) ? 3 - jj : jj;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[4 * kk + j], a[4 * kk + i], acc[i][j], 0, 0, 0);
          }
    }
    for (int i = 0; i < 4; ++i)
      for (int j = 0; j < 4; ++j)
        for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  } else {
    float4d acc[8][8];
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 8; ++j)
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          const int j = (i & 1) ? 7 - jj : jj;
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[j], a[i], acc[i][j], 0, 0, 0);
        }
    }
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 8; ++j)
        for (int r = 0; r < 4; ++r) s += acc[i][j][r];
  }
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace sk

extern "C" int skb_mfma_only(int shape, int iters, int zeros, void *scratch, size_t scratch_bytes, void *stream,
                                 double *flop) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return -1;
  if (!scratch || iters <= 0 || (shape != 0 && shape != 1)) return -2;
  if (scratch_bytes < (size_t)cus * 256 * sizeof(float)) return -3;
  if (shape == 0)
    hipLaunchKernelGGL(sk::mfma_only_kernel<true>, dim3(cus), dim3(256), 0, (hipStream_t)stream, (float *)scratch, iters, zeros);
  else
    hipLaunchKernelGGL(sk::mfma_only_kernel<false>, dim3(cus), dim3(256), 0, (hipStream_t)stream, (float *)scratch, iters, zeros);
  if (flop) *flop = (double)cus * 4.0 * (double)iters * 1048576.0;  // 32 x 32x32x16 = 64 x 16x16x32 = 2^20 FLOP per wave and iteration
  return hipGetLastError() == hipSuccess ? 0 : -1;
}
