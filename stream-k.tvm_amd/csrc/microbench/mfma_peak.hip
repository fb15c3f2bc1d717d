// Microbenchmark: sustained v_mfma_f32_32x32x16_f16 rate with nothing else in the loop, for operand
// registers holding zeros or non-zero data and for 4 or 8 waves per CU.  On the MI355X the result
// depends on the operand data (clocks drop under the power limit), which bounds what any fp16 GEMM
// can reach on that part.  Build: make -C stream-k.tvm_amd/csrc microbench
#include <hip/hip_runtime.h>
#include <cstdio>
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
template <int NACC>
__global__ __launch_bounds__(512) void mfma_only(float* out, int iters, _Float16 seed) {
  half8 a, b;
  for (int e = 0; e < 8; ++e) { a[e] = seed * (_Float16)(threadIdx.x % 7) ; b[e] = seed * (_Float16)(threadIdx.x % 5); }
  float16v acc[NACC];
  for (int i = 0; i < NACC; ++i) for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
  }
  float s = 0; for (int i = 0; i < NACC; ++i) for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}
// The same with operands that differ from lane to lane and from one MFMA to the next (eight random
// fp16 vectors in [-1, 1) per lane and operand), for the two dense fp16 shapes: 32x32x16 reads half
// as many operand registers per FLOP as 16x16x32.
typedef float float4v __attribute__((ext_vector_type(4)));
__device__ inline half8 random_operand(unsigned &state) {
  half8 v;
  for (int e = 0; e < 8; ++e) {
    state = state * 1664525u + 1013904223u;
    v[e] = (_Float16)((float)(state >> 8) * (2.0f / 16777216.0f) - 1.0f);
  }
  return v;
}
template <bool WIDE>
__global__ __launch_bounds__(512) void mfma_random(float* out, int iters) {
  unsigned state = (blockIdx.x * 512 + threadIdx.x) * 2654435761u + 12345u;
  half8 a[8], b[8];
  for (int i = 0; i < 8; ++i) { a[i] = random_operand(state); b[i] = random_operand(state); }
  float s = 0;
  if (WIDE) {
    float16v acc[8];
    for (int i = 0; i < 8; ++i) for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[(i + 3) & 7], acc[i], 0, 0, 0);
    }
    for (int i = 0; i < 8; ++i) for (int r = 0; r < 16; ++r) s += acc[i][r];
  } else {
    float4v acc[16];
    for (int i = 0; i < 16; ++i) for (int r = 0; r < 4; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i & 7], b[(i + 3 + (i >> 3)) & 7], acc[i], 0, 0, 0);
    }
    for (int i = 0; i < 16; ++i) for (int r = 0; r < 4; ++r) s += acc[i][r];
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}
int main() {
  float* out; hipMalloc(&out, 256 * 512 * 4 * 4);
  hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
  for (int rep = 0; rep < 3; ++rep) {
    int iters = 20000;
    hipEventRecord(e0); mfma_only<8><<<256, 512>>>(out, iters, (_Float16)0.0f); hipEventRecord(e1); hipDeviceSynchronize();
    float ms; hipEventElapsedTime(&ms, e0, e1);
    double fl = 256.0 * 8 * iters * 8 * 32768.0;
    printf("mfma only (zeros), 8 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, fl / ms / 1e9);
    hipEventRecord(e0); mfma_only<8><<<256, 512>>>(out, iters, (_Float16)0.37f); hipEventRecord(e1); hipDeviceSynchronize();
    hipEventElapsedTime(&ms, e0, e1);
    printf("mfma only (nonzero data), 8 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, fl / ms / 1e9);
    hipEventRecord(e0); mfma_only<8><<<256, 256>>>(out, iters, (_Float16)0.37f); hipEventRecord(e1); hipDeviceSynchronize();
    hipEventElapsedTime(&ms, e0, e1);
    printf("mfma only (nonzero data), 4 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, fl / 2 / ms / 1e9);
  }
  for (int rep = 0; rep < 3; ++rep) {
    int iters = 20000;
    float ms;
    hipEventRecord(e0); mfma_random<true><<<256, 512>>>(out, iters); hipEventRecord(e1); hipDeviceSynchronize();
    hipEventElapsedTime(&ms, e0, e1);
    printf("32x32x16, random operands, 8 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, 256.0 * 8 * iters * 8 * 32768.0 / ms / 1e9);
    hipEventRecord(e0); mfma_random<false><<<256, 512>>>(out, iters); hipEventRecord(e1); hipDeviceSynchronize();
    hipEventElapsedTime(&ms, e0, e1);
    printf("16x16x32, random operands, 8 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, 256.0 * 8 * iters * 16 * 16384.0 / ms / 1e9);
    hipEventRecord(e0); mfma_random<true><<<256, 256>>>(out, iters); hipEventRecord(e1); hipDeviceSynchronize();
    hipEventElapsedTime(&ms, e0, e1);
    printf("32x32x16, random operands, 4 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, 256.0 * 4 * iters * 8 * 32768.0 / ms / 1e9);
    hipEventRecord(e0); mfma_random<false><<<256, 256>>>(out, iters); hipEventRecord(e1); hipDeviceSynchronize();
    hipEventElapsedTime(&ms, e0, e1);
    printf("16x16x32, random operands, 4 waves/CU: %.3f ms %.0f TFLOP/s\n", ms, 256.0 * 4 * iters * 16 * 16384.0 / ms / 1e9);
  }
  return 0;
}
