// fp8 (OCP e4m3) MFMA probe for gfx950.  (1) One v_mfma_f32_32x32x64_f8f6f4 with zero scale arguments
// against a host product of the decoded bytes: the compiler emits the unscaled form of the
// instruction, whose scale is 1.  (2) Sustained rate of an MFMA-only loop for the two fp8 shapes,
// on all-zero and on random operands (the clock under the power limit depends on the data).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
#include <math.h>
#include <vector>
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

static float e4m3(uint8_t b) {
  int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) v = ldexpf((float)m, -9); else v = ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

// A [32][64] bytes, B [32][64] bytes, C [32][32] floats (C = A B^T)
__global__ void one_mfma(const uint8_t *A, const uint8_t *B, float *C) {
  const int lane = threadIdx.x, r = lane & 31, g = lane >> 5;
  intx8 a = *reinterpret_cast<const intx8 *>(A + r * 64 + g * 32);
  intx8 b = *reinterpret_cast<const intx8 *>(B + r * 64 + g * 32);
  floatx16 c = {0};
  c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
  // 32x32 layout: lane l holds column l%32, rows 8*q + 4*(l/32) + e at register 4*q + e
  for (int q = 0; q < 4; ++q)
    for (int e = 0; e < 4; ++e) C[(8 * q + 4 * g + e) * 32 + r] = c[4 * q + e];
}

template <int SHAPE>
__global__ __launch_bounds__(256) void rate(const intx8 *src, float *out, int iters) {
  intx8 a = src[threadIdx.x], b = src[256 + threadIdx.x];
  if (SHAPE == 32) {
    floatx16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; ++i) {
      c0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c0, 0, 0, 0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c1, 0, 0, 0, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c2, 0, 0, 0, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c3, 0, 0, 0, 0, 0, 0);
    }
    out[blockIdx.x * 256 + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3];
  } else {
    floatx4 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; ++i) {
      c0 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c0, 0, 0, 0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c1, 0, 0, 0, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c2, 0, 0, 0, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c3, 0, 0, 0, 0, 0, 0);
    }
    out[blockIdx.x * 256 + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3];
  }
}

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 1; } } while (0)
int main() {
  srand(1);
  std::vector<uint8_t> A(32 * 64), B(32 * 64);
  for (auto &x : A) { do x = rand() & 255; while ((x & 127) == 127); }
  for (auto &x : B) { do x = rand() & 255; while ((x & 127) == 127); }
  uint8_t *dA, *dB; float *dC;
  CK(hipMalloc(&dA, 2048)); CK(hipMalloc(&dB, 2048)); CK(hipMalloc(&dC, 4096));
  CK(hipMemcpy(dA, A.data(), 2048, hipMemcpyHostToDevice)); CK(hipMemcpy(dB, B.data(), 2048, hipMemcpyHostToDevice));
  one_mfma<<<1, 64>>>(dA, dB, dC);
  std::vector<float> C(1024);
  CK(hipMemcpy(C.data(), dC, 4096, hipMemcpyDeviceToHost));
  double maxrel = 0, sum_ratio = 0; int cnt = 0;
  for (int i = 0; i < 32; ++i) for (int j = 0; j < 32; ++j) {
    double ref = 0; for (int k = 0; k < 64; ++k) ref += (double)e4m3(A[i * 64 + k]) * e4m3(B[j * 64 + k]);
    double got = C[i * 32 + j];
    if (fabs(ref) > 1) { maxrel = fmax(maxrel, fabs(got - ref) / fabs(ref)); sum_ratio += got / ref; ++cnt; }
  }
  printf("one 32x32x64 e4m3 MFMA with zero scale arguments: max rel err %.3g, mean got/ref %.6g (%d entries)\n", maxrel, sum_ratio / cnt, cnt);

  const int iters = 20000, blocks = 256 * 8;
  std::vector<uint8_t> S(512 * 32);
  intx8 *dS; float *dO; CK(hipMalloc(&dS, S.size())); CK(hipMalloc(&dO, blocks * 256 * 4));
  for (int kind = 0; kind < 2; ++kind) {
    for (auto &x : S) { if (kind == 0) x = 0; else do x = rand() & 255; while ((x & 0x78) == 0x78); }
    CK(hipMemcpy(dS, S.data(), S.size(), hipMemcpyHostToDevice));
    for (int shape : {32, 16}) {
      hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
      for (int rep = 0; rep < 3; ++rep) {
        CK(hipEventRecord(e0));
        if (shape == 32) rate<32><<<blocks, 256>>>(dS, dO, iters); else rate<16><<<blocks, 256>>>(dS, dO, iters);
        CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        double flop = (double)blocks * 4 * iters * 4 * (shape == 32 ? 32.0 * 32 * 64 * 2 : 16.0 * 16 * 128 * 2);
        if (rep == 2) printf("%s operands, %s: %.1f ms, %.0f TFLOP/s\n", kind ? "random" : "zero", shape == 32 ? "32x32x64" : "16x16x128", ms, flop / ms * 1e-9);
      }
    }
  }
  return 0;
}
