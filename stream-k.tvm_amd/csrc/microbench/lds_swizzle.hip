// Microbenchmark: LDS read throughput of the fp16 tile kernels' fragment-read pattern (8 waves,
// ds_read_b128, 32-row blocks of 128-byte rows) under candidate XOR swizzles of the 16-byte chunk
// index.  Run it under `rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE` to see conflict
// cycles per variant; (row >> 1) & 7 (mode 1) is conflict free, row & 7 (mode 0) is 2-way.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
// Fragment-read pattern of the tile kernel: lane (r = lane%32, g = lane/32) reads row r of a 32-row block, chunk 2*kk+g.
// MODE selects the swizzle f(row): position = chunk ^ f(row).
template <int MODE> __device__ inline int swz(int row) {
  switch (MODE) {
    case 0: return row & 7;
    case 1: return (row >> 1) & 7;
    case 2: return (row >> 2) & 7;
    case 3: return ((row & 3) | ((row >> 1) & 4));      // bits 0,1,3
    case 4: return ((row & 1) | ((row >> 1) & 6));      // bits 0,2,3
    case 5: return (row ^ (row >> 3)) & 7;
    case 6: return ((row >> 1) ^ (row >> 4)) & 7;
    case 7: return 0;
    case 8: return (row & 7) ^ ((row >> 3) & 3);         // r&7 xor bits 3,4
    case 9: return ((row >> 1) & 7) ^ ((row & 1) << 2);
  }
  return 0;
}
template <int MODE>
__global__ __launch_bounds__(512) void lds_frag(uint32_t* out, int iters) {
  __shared__ __attribute__((aligned(16))) char lds[65536];
  int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 65536 / 4; i += 512) ((uint32_t*)lds)[i] = i;
  __syncthreads();
  uint4v acc = {0, 0, 0, 0};
  int wm = wave >> 2, wn = wave & 3;
  for (int it = 0; it < iters; ++it) {
    int rot = (it * 8) & 31;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {  // A frags: rows wm*128 + i*32 + r
        int row = wm * 128 + i * 32 + ((lane + rot) & 31);
        int pos = (2 * kk + (lane >> 5)) ^ swz<MODE>(row);
        acc += *(const uint4v*)(lds + row * 128 + pos * 16);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {  // B frags: rows 256 + wn*64 + j*32 + r
        int row = 256 + wn * 64 + j * 32 + ((lane + rot) & 31);
        int pos = (2 * kk + (lane >> 5)) ^ swz<MODE>(row);
        acc += *(const uint4v*)(lds + row * 128 + pos * 16);
      }
    }
  }
  out[blockIdx.x * 512 + tid] = acc[0] + acc[1] + acc[2] + acc[3];
}
template <int MODE> void run(uint32_t* out) {
  hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
  lds_frag<MODE><<<256, 512>>>(out, 200); hipDeviceSynchronize();
  hipEventRecord(a); lds_frag<MODE><<<256, 512>>>(out, 2000); hipEventRecord(b); hipDeviceSynchronize();
  float ms; hipEventElapsedTime(&ms, a, b);
  double bytes = 256.0 * 8 * 2000 * 24 * 1024;
  printf("mode %d: %.3f ms  %.1f TB/s aggregate LDS read (%.1f B/clk/CU at 2.4GHz)\n", MODE, ms, bytes / ms / 1e9, bytes / ms / 1e-3 / 256 / 2.4e9);
}
int main() {
  uint32_t* out; hipMalloc(&out, 256 * 512 * 4);
  run<0>(out); run<1>(out); run<2>(out); run<3>(out); run<4>(out); run<5>(out); run<6>(out); run<7>(out); run<8>(out); run<9>(out);
  return 0;
}
