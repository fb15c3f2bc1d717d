// Stream-K tile kernels for Q4 weights with more than 64 rows of A: the 16x16x32 fp16 tile kernel with B
// dequantised in registers on its way into the LDS stage (tile_f16_dma.h, Q4_).
#include "launch.h"
#include "sk_persistent.h"

namespace sk {

template <class P, bool FIXUP>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_tile_q4_kernel(typename P::Args a, DevPlan plan, Workspace ws,
                                                                           const void *bias) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P, FIXUP, true>(a, plan, ws, smem, bias);
}

#define SK_POLICY_Q4(BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 64, true, false, 0, true>

int tile_q4_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
#define X(id, BM, BN, WM, WN)                                                                                  \
  if (n < max) {                                                                                               \
    typedef SK_POLICY_Q4(BM, BN, WM, WN) P;                                                                    \
    out[n++] = KernelInfo{id, FAMILY_TILE, 2 /* SK_Q4 */, 0, 4, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 128, "tile_q4_nt_dma16_" #BM "x" #BN "x64"};                    \
  }
  SK_TILE_Q4_KERNELS(X)
#undef X
  return n;
}

int launch_tile_q4(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  switch (id) {
#define X(id_, BM, BN, WM, WN)                                                                               \
  case id_: {                                                                                                \
    typedef SK_POLICY_Q4(BM, BN, WM, WN) P;                                                                  \
    if (p.sk_tiles == 0)                                                                                     \
      hipLaunchKernelGGL((sk_tile_q4_kernel<P, false>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);    \
    else                                                                                                     \
      hipLaunchKernelGGL((sk_tile_q4_kernel<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);     \
    return (int)hipGetLastError();                                                                           \
  }
    SK_TILE_Q4_KERNELS(X)
#undef X
  }
  return launch_tile_8bit(id, a, p, ws, s, bias);
}

int occupancy_tile_q4(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, BM, BN, WM, WN)                                                                                         \
  case id_: {                                                                                                          \
    typedef SK_POLICY_Q4(BM, BN, WM, WN) P;                                                                            \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_q4_kernel<P, true>, P::NT, 0) != hipSuccess) return -1; \
    return occ;                                                                                                        \
  }
    SK_TILE_Q4_KERNELS(X)
#undef X
  }
  return occupancy_tile_8bit(id);
}

}  // namespace sk
