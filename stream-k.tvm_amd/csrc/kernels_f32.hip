// fp32 Stream-K kernels (gfx950): 128x128x16 tiles on fp32 MFMA, B as [K,N] or [N,K].
#include "launch.h"
#include "sk_persistent.h"
#include "tile_f32.h"

namespace sk {

template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_f32_kernel(typename P::Args a, DevPlan plan, Workspace ws) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P>(a, plan, ws, smem);
}

int f32_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
  if (n < max) {
    typedef TileF32<true> P;
    out[n++] = KernelInfo{200, FAMILY_TILE, 1, 1, 0, P::BM, P::BN, P::BK, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU,
                          P::TILE_ELEMS, 0, 0, 4, "tile_f32_nn_128x128x16"};
  }
  if (n < max) {
    typedef TileF32<false> P;
    out[n++] = KernelInfo{201, FAMILY_TILE, 1, 0, 0, P::BM, P::BN, P::BK, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU,
                          P::TILE_ELEMS, 0, 0, 4, "tile_f32_nt_128x128x16"};
  }
  return n;
}

int launch_f32(int id, const GemmArgsF32 &a, const DevPlan &p, const Workspace &ws, hipStream_t s) {
  if (id == 200) {
    hipLaunchKernelGGL(sk_f32_kernel<TileF32<true>>, dim3(p.grid), dim3(256), 0, s, a, p, ws);
  } else if (id == 201) {
    hipLaunchKernelGGL(sk_f32_kernel<TileF32<false>>, dim3(p.grid), dim3(256), 0, s, a, p, ws);
  } else {
    return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

int occupancy_f32(int id) {
  int occ = 0;
  hipError_t e = id == 200 ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_f32_kernel<TileF32<true>>, 256, 0)
                           : hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_f32_kernel<TileF32<false>>, 256, 0);
  return e == hipSuccess ? occ : -1;
}

}  // namespace sk
