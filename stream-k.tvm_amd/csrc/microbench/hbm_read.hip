// Microbenchmark: what one kernel launch can read from HBM, by size.  A grid of CTAs reads S bytes
// once with 16-byte loads, eight in flight per lane; consecutive launches read different regions of a
// 2 GiB buffer, so nothing is left in the 256 MB Infinity Cache from the launch before ("cold"),
// or the same region again ("warm").  The small-M kernels are priced against these figures: a
// launch of a few microseconds pays the launch itself and the latency of its first loads.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void read_once(const char *base, uint32_t *out, size_t bytes_per_cta) {
  const char *p = base + (size_t)blockIdx.x * bytes_per_cta + threadIdx.x * 16;
  uint4v acc = {0, 0, 0, 0};
  for (size_t off = 0; off < bytes_per_cta; off += 8 * 4096) {
    uint4v v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *(const uint4v *)(p + off + u * 4096);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[blockIdx.x * 256 + threadIdx.x] = acc[0];
}

int main() {
  const size_t total = (size_t)2 << 30;
  char *buf;
  uint32_t *out;
  if (hipMalloc(&buf, total) != hipSuccess || hipMalloc(&out, 1 << 24) != hipSuccess) return 1;
  hipMemset(buf, 1, total);
  hipEvent_t a, b;
  hipEventCreate(&a);
  hipEventCreate(&b);
  const size_t sizes[] = {(size_t)32 << 20, (size_t)64 << 20, (size_t)128 << 20, (size_t)448 << 20, (size_t)1 << 30};
  for (size_t S : sizes)
    for (int ctas_per_cu : {2, 4, 8})
      for (int cold = 0; cold < 2; ++cold) {
        const int grid = 256 * ctas_per_cu;
        const size_t per_cta = S / grid;
        if (per_cta % (8 * 4096) != 0) continue;  // the kernel reads whole 32 KB steps
        const int regions = (int)(total / S);
        const int reps = 24;
        for (int i = 0; i < 3; ++i) read_once<<<grid, 256>>>(buf, out, per_cta);
        hipDeviceSynchronize();
        hipEventRecord(a);
        for (int i = 0; i < reps; ++i)
          read_once<<<grid, 256>>>(buf + (cold ? (size_t)(i % regions) * S : 0), out, per_cta);
        hipEventRecord(b);
        hipDeviceSynchronize();
        float ms;
        hipEventElapsedTime(&ms, a, b);
        ms /= reps;
        printf("%5zu MB  grid %4d  %s  %8.2f us  %6.0f GB/s\n", S >> 20, grid,
               cold && regions > 1 ? "cold" : "warm", ms * 1e3, (double)S / ms / 1e6);
      }
  return 0;
}
