// fp32 Stream-K kernels (gfx950): fp32 MFMA tiles, B as [K,N] or [N,K].
#include "launch.h"
#include "sk_persistent.h"
#include "tile_f32.h"

namespace sk {

template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_f32_kernel(typename P::Args a, DevPlan plan, Workspace ws) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P>(a, plan, ws, smem);
}

// X(id, B is [K,N], BM, BN, WM, WN): 128 x 128 for large problems, 32 x 256 for M <= 32 (the reference's own
// fp32 run is 16 x 16384 x 8192, streamk_fp32.py:10-12 with the values of :24-28)
#define SK_F32_KERNELS(X)        \
  X(200, true, 128, 128, 2, 2)   \
  X(201, false, 128, 128, 2, 2)  \
  X(202, true, 32, 256, 1, 4)    \
  X(203, false, 32, 256, 1, 4)

int f32_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
#define X(id, KN, TBM, TBN, TWM, TWN)                                                                      \
  if (n < max) {                                                                                           \
    typedef TileF32<KN, TBM, TBN, TWM, TWN> P;                                                             \
    out[n++] = KernelInfo{id, FAMILY_TILE, 1, (KN) ? 1 : 0, 0, TBM, TBN, 16, P::NT, P::LDS_TOTAL,          \
                          P::CTAS_PER_CU, P::TILE_ELEMS, 0, 0, 4,                                          \
                          (KN) ? "tile_f32_nn_" #TBM "x" #TBN "x16" : "tile_f32_nt_" #TBM "x" #TBN "x16"}; \
  }
  SK_F32_KERNELS(X)
#undef X
  return n;
}

int launch_f32(int id, const GemmArgsF32 &a, const DevPlan &p, const Workspace &ws, hipStream_t s) {
  switch (id) {
#define X(id_, KN, TBM, TBN, TWM, TWN)                                                              \
  case id_:                                                                                         \
    hipLaunchKernelGGL((sk_f32_kernel<TileF32<KN, TBM, TBN, TWM, TWN>>), dim3(p.grid), dim3(256), 0, s, a, p, ws); \
    return (int)hipGetLastError();
    SK_F32_KERNELS(X)
#undef X
  }
  return (int)hipErrorInvalidValue;
}

int occupancy_f32(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, KN, TBM, TBN, TWM, TWN)                                                                          \
  case id_:                                                                                                     \
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_f32_kernel<TileF32<KN, TBM, TBN, TWM, TWN>>, 256, \
                                                        0) == hipSuccess                                        \
               ? occ                                                                                            \
               : -1;
    SK_F32_KERNELS(X)
#undef X
  }
  return -1;
}

}  // namespace sk
