// Prints, for every lane, which (source lane, element) each of the four 16-bit results of
// ds_read_b64_tr_b16 comes from when lane l points at elements 4l..4l+3: within each 16-lane
// group, lane L receives element (L & 3) of lanes (L >> 2) + 4j, j = 0..3.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef short short4v __attribute__((ext_vector_type(4)));
__global__ void tr_probe(uint16_t* out) {
  __shared__ __attribute__((aligned(16))) uint16_t lds[1024];
  int l = threadIdx.x;
  for (int i = l; i < 1024; i += 64) lds[i] = (uint16_t)i;
  __syncthreads();
  // lane l points at elements 4l .. 4l+3
  short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v*)(lds + 4 * l));
  for (int j = 0; j < 4; ++j) out[l * 4 + j] = (uint16_t)v[j];
}
int main() {
  uint16_t* d; hipMalloc(&d, 64 * 4 * 2);
  tr_probe<<<1, 64>>>(d); hipDeviceSynchronize();
  uint16_t h[256]; hipMemcpy(h, d, 512, hipMemcpyDeviceToHost);
  for (int l = 0; l < 64; ++l) {
    printf("lane %2d:", l);
    for (int j = 0; j < 4; ++j) printf("  (src lane %2d, elem %d)", h[l * 4 + j] / 4, h[l * 4 + j] % 4);
    printf("\n");
  }
  return 0;
}
