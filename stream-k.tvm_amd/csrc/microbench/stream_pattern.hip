// Microbenchmark: time to stream 32 MB once with the small-M kernels' access pattern (a wave reads
// 64 contiguous bytes from each of 16 rows per load) against fully contiguous 1 KB-per-wave loads.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
// Pattern A ("rows"): wave handles 16 rows (pitch bytes apart); lane (r=l%16,g=l/16) reads 16B at row r, byte off it*128 + c*64 + g*16.
// Pattern B ("contig"): wave reads 1KB contiguous per load.
template <int PATTERN, int ROT>
__global__ __launch_bounds__(64) void stream(const char* base, uint32_t* out, int pitch, int iters_per_wave, int waves_per_rowblock) {
  int wave = blockIdx.x, lane = threadIdx.x;
  uint4v acc = {0, 0, 0, 0};
  if (PATTERN == 0) {
    int rb = wave / waves_per_rowblock, seg = wave % waves_per_rowblock;
    const char* p = base + (size_t)(rb * 16 + (lane & 15)) * pitch + (size_t)seg * iters_per_wave * 128 + (lane >> 4) * 16;
    int rot = ROT ? (wave * 5) % iters_per_wave : 0;
#pragma unroll 4
    for (int it = 0; it < iters_per_wave; ++it) {
      int i2 = it + rot; if (i2 >= iters_per_wave) i2 -= iters_per_wave;
      acc += *(const uint4v*)(p + i2 * 128);
      acc += *(const uint4v*)(p + i2 * 128 + 64);
    }
  } else if (PATTERN >= 2 && PATTERN <= 4) {
    // PATTERN 2: 4 rows x 256 contiguous bytes per load (lane l: row l/16, piece l%16)
    // PATTERN 3: 8 rows x 128 bytes (row l/8, piece l%8); PATTERN 4: 16 rows x 64 bytes with the four
    // lanes of a row adjacent (row l/4, piece l%4).  A wave still owns 16 rows x (iters*128) bytes.
    constexpr int LPR = PATTERN == 2 ? 16 : (PATTERN == 3 ? 8 : 4);   // lanes per row
    constexpr int RPL = 64 / LPR;                                     // rows per load
    constexpr int LOADS = 16 / RPL;                                   // loads to cover 16 rows
    int rb = wave / waves_per_rowblock, seg = wave % waves_per_rowblock;
    const char* p = base + (size_t)(rb * 16 + lane / LPR) * pitch + (size_t)seg * iters_per_wave * 128 + (lane % LPR) * 16;
    // per "iteration" the wave consumes 2 KB: LOADS row groups x (2048 / LOADS / RPL) bytes per row
    constexpr int BYTES_PER_ROW = LPR * 16;
    const int steps = iters_per_wave * 128 / BYTES_PER_ROW;  // steps along K
#pragma unroll(8 / LOADS)
    for (int st = 0; st < steps; ++st) {
#pragma unroll
      for (int g = 0; g < LOADS; ++g) acc += *(const uint4v*)(p + (size_t)g * RPL * pitch + st * BYTES_PER_ROW);
    }
  } else if (PATTERN == 5) {
    // 1 KB contiguous per load, but lane l reads the piece a 16x16 MFMA operand layout takes from
    // a 16-row x 64-byte tile stored row by row: offset (l%16)*64 + (l/16)*16
    const char* p = base + (size_t)wave * iters_per_wave * 2048 + (lane & 15) * 64 + (lane >> 4) * 16;
#pragma unroll 4
    for (int it = 0; it < iters_per_wave; ++it) {
      acc += *(const uint4v*)(p + it * 2048);
      acc += *(const uint4v*)(p + it * 2048 + 1024);
    }
  } else {
    const char* p = base + (size_t)wave * iters_per_wave * 2048 + lane * 16;
#pragma unroll 4
    for (int it = 0; it < iters_per_wave; ++it) {
      acc += *(const uint4v*)(p + it * 2048);
      acc += *(const uint4v*)(p + it * 2048 + 1024);
    }
  }
  out[blockIdx.x * 64 + lane] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
}
template <int PATTERN, int ROT> void run(const char* name, const char* buf, uint32_t* out, int waves, int iters, int wprb) {
  hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
  for (int i = 0; i < 3; ++i) stream<PATTERN, ROT><<<waves, 64>>>(buf, out, 4096, iters, wprb);
  hipDeviceSynchronize();
  hipEventRecord(a);
  for (int i = 0; i < 20; ++i) stream<PATTERN, ROT><<<waves, 64>>>(buf, out, 4096, iters, wprb);
  hipEventRecord(b); hipDeviceSynchronize();
  float ms; hipEventElapsedTime(&ms, a, b); ms /= 20;
  double bytes = (double)waves * iters * 2048;
  printf("%-28s waves=%5d iters=%3d  %.2f us  %.0f GB/s\n", name, waves, iters, ms * 1e3, bytes / ms / 1e6);
}
int main() {
  char* buf; uint32_t* out; hipMalloc(&buf, 64 << 20); hipMalloc(&out, 1 << 22); hipMemset(buf, 1, 64 << 20);
  // 32 MB = 8192 rows x 4096 B.  rowblocks = 512; each row = 32 iterations of 128B.
  for (int wprb : {1, 2, 4, 8}) {
    int waves = 512 * wprb, iters = 32 / wprb;
    run<0, 0>("rows", buf, out, waves, iters, wprb);
    run<0, 1>("rows+rot", buf, out, waves, iters, wprb);
    run<1, 0>("contig", buf, out, waves, iters, wprb);
    if (iters * 128 >= 256) run<2, 0>("4rows x 256B", buf, out, waves, iters, wprb);
    run<3, 0>("8rows x 128B", buf, out, waves, iters, wprb);
    run<4, 0>("16rows x 64B, quads", buf, out, waves, iters, wprb);
    run<5, 0>("1KB tile, MFMA16 lane order", buf, out, waves, iters, wprb);
  }
  return 0;
}
