// fp16 LDS-tiled Stream-K kernels (gfx950).
#include "launch.h"
#include "sk_persistent.h"

namespace sk {

// bias: optional row added in the epilogue (null: none); one instance serves both cases, the epilogue branches
template <class P, bool FIXUP = true>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_tile_kernel(typename P::Args a, DevPlan plan, Workspace ws,
                                                                        const void *bias) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];  // policies with their own LDS arrays keep this at 16 bytes
  run_persistent<P, FIXUP, true>(a, plan, ws, smem, bias);
}

// data-parallel launches of the direct-to-LDS kernels use the instance without fix-up code
template <class P>
static int launch_dma(const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  if (p.sk_tiles == 0)
    hipLaunchKernelGGL((sk_tile_kernel<P, false>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);
  else
    hipLaunchKernelGGL((sk_tile_kernel<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);
  return (int)hipGetLastError();
}

#define SK_POLICY(id, BM, BN, BK, WM, WN) TileF16NT<BM, BN, BK, WM, WN>
#define SK_POLICY_DMA(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN>
#define SK_POLICY_NN(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, true>
#define SK_POLICY_DMA32(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 32>
#define SK_POLICY_DMA16(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 64, true>
#define SK_POLICY_DMA32_16(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 32, true>
#define SK_POLICY_NN16(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, true, 64, true>
#define SK_POLICY_BF16(id, BM, BN, WM, WN, BK, NN) TileF16NTDma<BM, BN, WM, WN, NN, BK, true, true>

int tile_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
#define X(id, BM, BN, BK, WM, WN)                                                                   \
  if (n < max) {                                                                                    \
    typedef SK_POLICY(id, BM, BN, BK, WM, WN) P;                                                    \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 0, 0, BM, BN, BK, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU,  \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nt_" #BM "x" #BN "x" #BK};                 \
  }
  SK_TILE_F16_NT_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_DMA(id, BM, BN, WM, WN) P;                                                    \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 0, (P::TM * P::TN > 8) ? 2 : 1, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nt_dma_" #BM "x" #BN "x64"};               \
  }
  SK_TILE_F16_NT_DMA_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_NN(id, BM, BN, WM, WN) P;                                                     \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 1, 1, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nn_dma_" #BM "x" #BN "x64"};            \
  }
  SK_TILE_F16_NN_DMA_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_DMA32(id, BM, BN, WM, WN) P;                                                  \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 0, 3, BM, BN, 32, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nt_dma_" #BM "x" #BN "x32"};            \
  }
  SK_TILE_F16_NT_DMA32_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_DMA16(id, BM, BN, WM, WN) P;                                                  \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 0, 4, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nt_dma16_" #BM "x" #BN "x64"};          \
  }
  SK_TILE_F16_NT_DMA16_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_DMA32_16(id, BM, BN, WM, WN) P;                                               \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 0, 5, BM, BN, 32, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nt_dma16_" #BM "x" #BN "x32"};          \
  }
  SK_TILE_F16_NT_DMA32_16_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_NN16(id, BM, BN, WM, WN) P;                                                   \
    out[n++] = KernelInfo{id, FAMILY_TILE, 0, 1, 4, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 8, "tile_f16_nn_dma16_" #BM "x" #BN "x64"};          \
  }
  SK_TILE_F16_NN_DMA16_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN, BK, NN)                                                               \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_BF16(id, BM, BN, WM, WN, BK, NN) P;                                           \
    out[n++] = KernelInfo{id, FAMILY_TILE, 3 /* SK_BF16 */, (NN) ? 1 : 0, (BK) == 32 ? 5 : 4, BM, BN, BK, P::NT, P::LDS_TOTAL, \
                          P::CTAS_PER_CU, P::TILE_ELEMS, 0, 0, 8,                                    \
                          (NN) ? "tile_bf16_nn_dma16_" #BM "x" #BN "x" #BK : "tile_bf16_nt_dma16_" #BM "x" #BN "x" #BK}; \
  }
  SK_TILE_BF16_KERNELS(X)
#undef X
  return n;
}

int launch_tile_f16(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  switch (id) {
#define X(id_, BM, BN, BK, WM, WN)                                                       \
  case id_: {                                                                            \
    typedef SK_POLICY(id_, BM, BN, BK, WM, WN) P;                                        \
    hipLaunchKernelGGL(sk_tile_kernel<P>, dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);    \
    return (int)hipGetLastError();                                                       \
  }
    SK_TILE_F16_NT_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_DMA(id_, BM, BN, WM, WN) P;                                      \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_F16_NT_DMA_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_NN(id_, BM, BN, WM, WN) P;                                      \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_F16_NN_DMA_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_DMA32(id_, BM, BN, WM, WN) P;                                      \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_F16_NT_DMA32_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_DMA16(id_, BM, BN, WM, WN) P;                                      \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_F16_NT_DMA16_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_DMA32_16(id_, BM, BN, WM, WN) P;                                   \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_F16_NT_DMA32_16_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_NN16(id_, BM, BN, WM, WN) P;                                       \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_F16_NN_DMA16_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN, BK, NN)                                                   \
  case id_: {                                                                            \
    typedef SK_POLICY_BF16(id_, BM, BN, WM, WN, BK, NN) P;                               \
    return launch_dma<P>(a, p, ws, s, bias);                                                       \
  }
    SK_TILE_BF16_KERNELS(X)
#undef X
  }
  return launch_tile_asm(id, a, p, ws, s, bias);
}

int occupancy_tile(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, BM, BN, BK, WM, WN)                                                                  \
  case id_: {                                                                                       \
    typedef SK_POLICY(id_, BM, BN, BK, WM, WN) P;                                                   \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NT_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_DMA(id_, BM, BN, WM, WN) P;                                                   \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NT_DMA_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_NN(id_, BM, BN, WM, WN) P;                                                    \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NN_DMA_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_DMA32(id_, BM, BN, WM, WN) P;                                                 \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NT_DMA32_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_DMA16(id_, BM, BN, WM, WN) P;                                                 \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NT_DMA16_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_DMA32_16(id_, BM, BN, WM, WN) P;                                              \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NT_DMA32_16_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_NN16(id_, BM, BN, WM, WN) P;                                                  \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F16_NN_DMA16_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN, BK, NN)                                                              \
  case id_: {                                                                                       \
    typedef SK_POLICY_BF16(id_, BM, BN, WM, WN, BK, NN) P;                                          \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_BF16_KERNELS(X)
#undef X
  }
  return occupancy_tile_asm(id);
}

}  // namespace sk
