// Small-M Stream-K kernels, fp16 and Q4 weights (gfx950).
#include "launch.h"
#include "sk_persistent.h"

namespace sk {
#ifdef SK_PHASE_TRACE
__device__ long long g_trace_buf[2048 * 16];
#endif

template <class P, bool FIXUP = true>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_kernel(typename P::Args a, DevPlan plan, Workspace ws) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P, FIXUP>(a, plan, ws, smem);
}
// the same with a bias row added in the epilogue (a second instance: see run_persistent)
template <class P, bool FIXUP = true>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_kernel_bias(typename P::Args a, DevPlan plan, Workspace ws,
                                                                               const void *bias) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P, FIXUP, true>(a, plan, ws, smem, bias);
}

// Launches without Stream-K tiles: every CTA owns whole tiles (tile = block index, then strides of the grid;
// one row of tiles, since these kernels take all of A's rows in one tile), so the kernel needs neither the plan
// nor the workspace.  These kernels run for a few microseconds, most of which is set-up executed from a cold
// instruction cache: without the plan's argument loads, the range and tile-coordinate arithmetic and the fix-up
// code the first loads go out earlier.
template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_dp_kernel(typename P::Args a, int total_tiles, int ipt) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  typename P::Acc acc;
  SK_TRACE(0);
  for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {
    SK_TRACE(11);
    P::mac(a, acc, 0, tile, 0, ipt, smem);
    SK_TRACE(8);
    P::store_c(a, acc, 0, tile, smem, nullptr);
    SK_TRACE(9);
  }
}
template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_dp_kernel_bias(typename P::Args a, int total_tiles, int ipt,
                                                                                  const void *bias_arg) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  const void *bias = bias_arg;
  asm volatile("" ::"s"(bias));  // fetched with the other arguments, not before the first store
  typename P::Acc acc;
  for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {
    P::mac(a, acc, 0, tile, 0, ipt, smem);
    P::store_c(a, acc, 0, tile, smem, bias);
  }
}

template <class P>
static int launch_policy(const SkinnyArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  if (p.sk_tiles == 0 && p.tiles_m != 1) return (int)hipErrorInvalidValue;  // (no plan of these kernels has two tile rows)
  if (bias != nullptr) {
    if (p.sk_tiles == 0)
      hipLaunchKernelGGL((sk_skinny_dp_kernel_bias<P>), dim3(p.grid), dim3(P::NT), 0, s, a, p.total_tiles, p.ipt, bias);
    else
      hipLaunchKernelGGL((sk_skinny_kernel_bias<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);
  } else if (p.sk_tiles == 0) {
    hipLaunchKernelGGL((sk_skinny_dp_kernel<P>), dim3(p.grid), dim3(P::NT), 0, s, a, p.total_tiles, p.ipt);
  } else {
    hipLaunchKernelGGL((sk_skinny_kernel<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws);
  }
  return (int)hipGetLastError();
}

#define SK_POLICY(MB, NB, WN, RK, Q4, DEPTH, ROW1) TileSkinny<MB, NB, WN, RK, (Q4) != 0, DEPTH, (ROW1) != 0>
#define SK_POLICY_BF16(MB, NB, WN, RK, DEPTH, ROW1) \
  TileSkinny<MB, NB, WN, RK, false, DEPTH, (ROW1) != 0, false, false, true>
#define SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, FMT) \
  TileSkinny<MB, NB, WN, RK, false, DEPTH, (ROW1) != 0, false, false, false, FMT>

int skinny_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
#define X(id, MB, NB, WN, RK, Q4, DEPTH, ROW1)                                                         \
  if (n < max) {                                                                                   \
    typedef SK_POLICY(MB, NB, WN, RK, Q4, DEPTH, ROW1) P;                                                \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, (Q4) ? 2 : 0, 0, (ROW1) ? 1 : 0, P::BM, P::BN, P::BKC, P::NT, \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, (Q4) ? P::SC_MAX_ITERS : 0, \
                          P::MAX_M, (Q4) ? 128 : 8,                                               \
                          (Q4) ? "skinny_q4_mb" #MB "_wn" #WN "_rk" #RK "_row1_" #ROW1             \
                               : "skinny_f16_mb" #MB "_wn" #WN "_rk" #RK "_row1_" #ROW1};          \
  }
  SK_SKINNY_KERNELS(X)
#undef X
#define X(id, MB, NB, WN, RK, DEPTH, ROW1)                                                                \
  if (n < max) {                                                                                      \
    typedef SK_POLICY_BF16(MB, NB, WN, RK, DEPTH, ROW1) P;                                              \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 3, 0, (ROW1) ? 1 : 0, P::BM, P::BN, P::BKC, P::NT,         \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, 0, P::MAX_M, 8,                \
                          "skinny_bf16_mb" #MB "_wn" #WN "_rk" #RK "_row1_" #ROW1};                      \
  }
  SK_SKINNY_BF16_KERNELS(X)
#undef X
#define X(id, MB, NB, WN, RK, DEPTH, ROW1)                                                                \
  if (n + 1 < max) {                                                                                  \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 1) P;                                             \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 5, 0, (ROW1) ? 1 : 0, P::BM, P::BN, 2 * P::BKC, P::NT,     \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, 0, P::MAX_M, 16,               \
                          "skinny_f8e4m3_mb" #MB "_wn" #WN "_rk" #RK "_row1_" #ROW1};                    \
    out[n++] = KernelInfo{id + 10, FAMILY_SKINNY, 8, 0, (ROW1) ? 1 : 0, P::BM, P::BN, 2 * P::BKC, P::NT, \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, 0, P::MAX_M, 16,               \
                          "skinny_f8e5m2_mb" #MB "_wn" #WN "_rk" #RK "_row1_" #ROW1};                    \
  }
  SK_SKINNY_F8_KERNELS(X)
#undef X
#define X(id, MB, NB, WN, RK, DEPTH, ROW1)                                                                \
  if (n < max) {                                                                                      \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 3) P;                                             \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 6, 0, (ROW1) ? 1 : 0, P::BM, P::BN, 2 * P::BKC, P::NT,     \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, 0, P::MAX_M, 16,               \
                          "skinny_i8_mb" #MB "_wn" #WN "_rk" #RK "_row1_" #ROW1};                        \
  }
  SK_SKINNY_I8_KERNELS(X)
#undef X
#define X(id, NB, WN, RK, DEPTH, KMAX)                                                                        \
  if (n < max) {                                                                                         \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX> P;                                                        \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 2, 0, 2, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES,         \
                          P::CTAS_PER_CU, P::TILE_ELEMS, P::MAX_ITERS, P::MAX_M, 128,                    \
                          "gemv_q4_nb" #NB "_wn" #WN "_rk" #RK "_k" #KMAX};                                     \
  }
  SK_GEMV_Q4_KERNELS(X)
#undef X
#define X(id, NB, WN, RK, DEPTH, KMAX)                                                                        \
  if (n < max) {                                                                                         \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, false, true> P;                                           \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 7 /* SK_Q4_ZP */, 0, 2, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, \
                          P::CTAS_PER_CU, P::TILE_ELEMS, P::MAX_ITERS, P::MAX_M, 128,                    \
                          "gemv_q4zp_nb" #NB "_wn" #WN "_rk" #RK "_k" #KMAX};                                   \
  }
  SK_GEMV_Q4ZP_KERNELS(X)
#undef X
#define X(id, NB, WN, RK, DEPTH, KMAX)                                                                        \
  if (n < max) {                                                                                         \
    typedef TileGemvF16<NB, WN, RK, DEPTH, KMAX> P;                                                       \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 0, 0, 2, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES,         \
                          P::CTAS_PER_CU, P::TILE_ELEMS, P::MAX_ITERS, P::MAX_M, 8,                      \
                          "gemv_f16_nb" #NB "_wn" #WN "_rk" #RK "_k" #KMAX};                                    \
  }
  SK_GEMV_F16_KERNELS(X)
#undef X
#define X(id, NB, WN, RK, DEPTH, KMAX)                                                                        \
  if (n < max) {                                                                                         \
    typedef TileGemvF16<NB, WN, RK, DEPTH, KMAX, true> P;                                                 \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 3, 0, 2, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES,         \
                          P::CTAS_PER_CU, P::TILE_ELEMS, P::MAX_ITERS, P::MAX_M, 8,                      \
                          "gemv_bf16_nb" #NB "_wn" #WN "_rk" #RK "_k" #KMAX};                                   \
  }
  SK_GEMV_BF16_KERNELS(X)
#undef X
#define X(id, MB, NB, WN, RK, DEPTH)                                                                     \
  if (n < max) {                                                                                     \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, true> P;                                  \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 4 /* SK_Q4_TILED */, 0, 0, P::BM, P::BN, P::BKC, P::NT, \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, P::SC_MAX_ITERS, P::MAX_M, 128, \
                          "skinny_q4t_mb" #MB "_wn" #WN "_rk" #RK};                                   \
  }
  SK_SKINNY_Q4T_KERNELS(X)
#undef X
#define X(id, MB, NB, WN, RK, DEPTH)                                                                     \
  if (n < max) {                                                                                     \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, false, true> P;                           \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 7 /* SK_Q4_ZP */, 0, 0, P::BM, P::BN, P::BKC, P::NT,    \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, P::SC_MAX_ITERS, P::MAX_M, 128, \
                          "skinny_q4zp_mb" #MB "_wn" #WN "_rk" #RK};                                  \
  }
  SK_SKINNY_Q4ZP_KERNELS(X)
#undef X
#define X(id, NB, WN, RK, DEPTH, KMAX)                                                                   \
  if (n < max) {                                                                                     \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, true> P;                                              \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 4 /* SK_Q4_TILED */, 0, 2, P::BM, P::BN, P::BKC, P::NT, \
                          P::LDS_BYTES, P::CTAS_PER_CU, P::TILE_ELEMS, P::MAX_ITERS, P::MAX_M, 128,   \
                          "gemv_q4t_nb" #NB "_wn" #WN "_rk" #RK "_k" #KMAX};                          \
  }
  SK_GEMV_Q4T_KERNELS(X)
#undef X
  return n;
}

int launch_skinny(int id, const SkinnyArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  switch (id) {
#define X(id_, MB, NB, WN, RK, Q4, DEPTH, ROW1)                                                \
  case id_: {                                                                              \
    typedef SK_POLICY(MB, NB, WN, RK, Q4, DEPTH, ROW1) P;                                        \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_SKINNY_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH, ROW1)                                                 \
  case id_: {                                                                              \
    typedef SK_POLICY_BF16(MB, NB, WN, RK, DEPTH, ROW1) P;                                   \
    return launch_policy<P>(a, p, ws, s, bias);                                            \
  }
    SK_SKINNY_BF16_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH, ROW1)                                                 \
  case id_: {                                                                              \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 1) P;                                  \
    return launch_policy<P>(a, p, ws, s, bias);                                            \
  }                                                                                        \
  case id_ + 10: {                                                                         \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 2) P;                                  \
    return launch_policy<P>(a, p, ws, s, bias);                                            \
  }
    SK_SKINNY_F8_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH, ROW1)                                                 \
  case id_: {                                                                              \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 3) P;                                  \
    return launch_policy<P>(a, p, ws, s, nullptr);                                         \
  }
    SK_SKINNY_I8_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                        \
  case id_: {                                                                              \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX> P;                                          \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_GEMV_Q4_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                        \
  case id_: {                                                                              \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, false, true> P;                             \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_GEMV_Q4ZP_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                        \
  case id_: {                                                                              \
    typedef TileGemvF16<NB, WN, RK, DEPTH, KMAX> P;                                         \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_GEMV_F16_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                     \
  case id_: {                                                                              \
    typedef TileGemvF16<NB, WN, RK, DEPTH, KMAX, true> P;                                   \
    return launch_policy<P>(a, p, ws, s, bias);                                            \
  }
    SK_GEMV_BF16_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH)                                                       \
  case id_: {                                                                              \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, true> P;                        \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_SKINNY_Q4T_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH)                                                       \
  case id_: {                                                                              \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, false, true> P;                 \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_SKINNY_Q4ZP_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                     \
  case id_: {                                                                              \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, true> P;                                    \
    return launch_policy<P>(a, p, ws, s, bias);                                                         \
  }
    SK_GEMV_Q4T_KERNELS(X)
#undef X
  }
  return (int)hipErrorInvalidValue;
}

int occupancy_skinny(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, MB, NB, WN, RK, Q4, DEPTH, ROW1)                                                           \
  case id_: {                                                                                         \
    typedef SK_POLICY(MB, NB, WN, RK, Q4, DEPTH, ROW1) P;                                                   \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                      \
    return occ;                                                                                       \
  }
    SK_SKINNY_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH, ROW1)                                                              \
  case id_: {                                                                                         \
    typedef SK_POLICY_BF16(MB, NB, WN, RK, DEPTH, ROW1) P;                                                \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                      \
    return occ;                                                                                       \
  }
    SK_SKINNY_BF16_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH, ROW1)                                                              \
  case id_:                                                                                           \
  case id_ + 10: {  /* the two formats differ in one instruction: one occupancy */                    \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 1) P;                                               \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                      \
    return occ;                                                                                       \
  }
    SK_SKINNY_F8_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH, ROW1)                                                              \
  case id_: {                                                                                         \
    typedef SK_POLICY_F8(MB, NB, WN, RK, DEPTH, ROW1, 3) P;                                               \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                      \
    return occ;                                                                                       \
  }
    SK_SKINNY_I8_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                                      \
  case id_: {                                                                                            \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX> P;                                                        \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_Q4_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                                      \
  case id_: {                                                                                            \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, false, true> P;                                           \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_Q4ZP_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                                      \
  case id_: {                                                                                            \
    typedef TileGemvF16<NB, WN, RK, DEPTH, KMAX> P;                                                       \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_F16_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                                      \
  case id_: {                                                                                            \
    typedef TileGemvF16<NB, WN, RK, DEPTH, KMAX, true> P;                                                 \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_BF16_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH)                                                                     \
  case id_: {                                                                                            \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, true> P;                                      \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_SKINNY_Q4T_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH)                                                                     \
  case id_: {                                                                                            \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, false, true> P;                               \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_SKINNY_Q4ZP_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                                   \
  case id_: {                                                                                            \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, true> P;                                                  \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_Q4T_KERNELS(X)
#undef X
  }
  return -1;
}

}  // namespace sk

#ifdef SK_PHASE_TRACE
extern "C" int sk_debug_trace_read(long long *out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(sk::g_trace_buf), sizeof(long long) * 2048 * 16);
}
#endif
