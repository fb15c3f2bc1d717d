// Stream-K tile kernels for one-byte operands (fp8 e4m3 / e5m2 with fp16 C, int8 with int32 C): the F8_ instances of
// tile_f16_dma.h, in two stages of 128 K-values and in four stages of 64.  A translation unit of its own, so that
// it compiles beside the 16-bit tile kernels.
#include "launch.h"
#include "sk_persistent.h"

namespace sk {

// (the kernel template of kernels_tile.hip: bias is an optional row added in the epilogue)
template <class P, bool FIXUP = true>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_tile_kernel(typename P::Args a, DevPlan plan, Workspace ws,
                                                                        const void *bias) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P, FIXUP, true>(a, plan, ws, smem, bias);
}

// data-parallel launches use the instance without fix-up code
template <class P>
static int launch_dma(const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  if (p.sk_tiles == 0)
    hipLaunchKernelGGL((sk_tile_kernel<P, false>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);
  else
    hipLaunchKernelGGL((sk_tile_kernel<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);
  return (int)hipGetLastError();
}

#define SK_POLICY_F8(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 64, false, false, 1>
#define SK_POLICY_F8E5M2(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 64, false, false, 2>
#define SK_POLICY_I8(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 64, true, false, 3>
#define SK_POLICY_I8_BK64(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 32, true, false, 3>
#define SK_POLICY_F8_BK64(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 32, false, false, 1>
#define SK_POLICY_F8E5M2_BK64(id, BM, BN, WM, WN) TileF16NTDma<BM, BN, WM, WN, false, 32, false, false, 2>

int tile_8bit_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_F8(id, BM, BN, WM, WN) P;                                                     \
    out[n++] = KernelInfo{id, FAMILY_TILE, 5 /* SK_F8E4M3 */, 0, 6, BM, BN, 128, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 16, "tile_f8e4m3_nt_dma_" #BM "x" #BN "x128"};       \
  }
  SK_TILE_F8_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_F8E5M2(id, BM, BN, WM, WN) P;                                                 \
    out[n++] = KernelInfo{id, FAMILY_TILE, 8 /* SK_F8E5M2 */, 0, 6, BM, BN, 128, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 16, "tile_f8e5m2_nt_dma_" #BM "x" #BN "x128"};       \
  }
  SK_TILE_F8E5M2_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_I8(id, BM, BN, WM, WN) P;                                                     \
    out[n++] = KernelInfo{id, FAMILY_TILE, 6 /* SK_I8 */, 0, 4, BM, BN, 128, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 16, "tile_i8_nt_dma16_" #BM "x" #BN "x128"};         \
  }
  SK_TILE_I8_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_I8_BK64(id, BM, BN, WM, WN) P;                                                \
    out[n++] = KernelInfo{id, FAMILY_TILE, 6 /* SK_I8 */, 0, 5, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 16, "tile_i8_nt_dma16_" #BM "x" #BN "x64"};          \
  }
  SK_TILE_I8_BK64_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_F8_BK64(id, BM, BN, WM, WN) P;                                                \
    out[n++] = KernelInfo{id, FAMILY_TILE, 5 /* SK_F8E4M3 */, 0, 5, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 16, "tile_f8e4m3_nt_dma_" #BM "x" #BN "x64"};        \
  }
  SK_TILE_F8_BK64_KERNELS(X)
#undef X
#define X(id, BM, BN, WM, WN)                                                                       \
  if (n < max) {                                                                                    \
    typedef SK_POLICY_F8E5M2_BK64(id, BM, BN, WM, WN) P;                                            \
    out[n++] = KernelInfo{id, FAMILY_TILE, 8 /* SK_F8E5M2 */, 0, 5, BM, BN, 64, P::NT, P::LDS_TOTAL, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, 0, 16, "tile_f8e5m2_nt_dma_" #BM "x" #BN "x64"};        \
  }
  SK_TILE_F8E5M2_BK64_KERNELS(X)
#undef X
  return n;
}

int launch_tile_8bit(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  switch (id) {
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_F8(id_, BM, BN, WM, WN) P;                                         \
    return launch_dma<P>(a, p, ws, s, bias);                                                   \
  }
    SK_TILE_F8_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_F8E5M2(id_, BM, BN, WM, WN) P;                                     \
    return launch_dma<P>(a, p, ws, s, bias);                                             \
  }
    SK_TILE_F8E5M2_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_I8(id_, BM, BN, WM, WN) P;                                         \
    return launch_dma<P>(a, p, ws, s, bias);                                                   \
  }
    SK_TILE_I8_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_I8_BK64(id_, BM, BN, WM, WN) P;                                    \
    return launch_dma<P>(a, p, ws, s, bias);                                             \
  }
    SK_TILE_I8_BK64_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_F8_BK64(id_, BM, BN, WM, WN) P;                                    \
    return launch_dma<P>(a, p, ws, s, bias);                                             \
  }
    SK_TILE_F8_BK64_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                           \
  case id_: {                                                                            \
    typedef SK_POLICY_F8E5M2_BK64(id_, BM, BN, WM, WN) P;                                \
    return launch_dma<P>(a, p, ws, s, bias);                                             \
  }
    SK_TILE_F8E5M2_BK64_KERNELS(X)
#undef X
  }
  return (int)hipErrorInvalidValue;
}

int occupancy_tile_8bit(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_F8(id_, BM, BN, WM, WN) P;                                                    \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F8_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_F8E5M2(id_, BM, BN, WM, WN) P;                                                \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F8E5M2_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_I8(id_, BM, BN, WM, WN) P;                                                    \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_I8_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_I8_BK64(id_, BM, BN, WM, WN) P;                                               \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_I8_BK64_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_F8_BK64(id_, BM, BN, WM, WN) P;                                               \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F8_BK64_KERNELS(X)
#undef X
#define X(id_, BM, BN, WM, WN)                                                                      \
  case id_: {                                                                                       \
    typedef SK_POLICY_F8E5M2_BK64(id_, BM, BN, WM, WN) P;                                           \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                    \
    return occ;                                                                                     \
  }
    SK_TILE_F8E5M2_BK64_KERNELS(X)
#undef X
  }
  return -1;
}

}  // namespace sk
