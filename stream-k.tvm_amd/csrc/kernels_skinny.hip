// Small-M Stream-K kernels, fp16 and Q4 weights (gfx950).
#include "skinny_launch.h"

namespace sk {
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
  n += gemv_rows_kernel_infos(out + n, max - n);
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
  return launch_gemv_rows(id, a, p, ws, s, bias);
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
  return occupancy_gemv_rows(id);
}

}  // namespace sk
