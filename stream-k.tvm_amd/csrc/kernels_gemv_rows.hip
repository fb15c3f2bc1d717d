// Small-M kernels in the matrix-vector kernels' form (tile_gemv_rows.h): 2 <= M <= 16, fp16 / bfloat16, NT;
// the Q4 kernels for per-group zero points with tiled weights (dtype 9, SK_Q4_ZP_TILED); and the kernels that stream
// fp16 / bfloat16 weights through LDS in contiguous loads (tile_stream_pairs.h).
#include "skinny_launch.h"

namespace sk {

int gemv_rows_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
#define X(id, MR, WN, RK, DEPTH)                                                                               \
  if (n < max) {                                                                                               \
    typedef TileGemvRows<MR, WN, RK, DEPTH, false> P;                                                          \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 0, 0, 3, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, P::MAX_M, 8, "gemv_rows_f16_m" #MR "_wn" #WN "_rk" #RK};            \
  }
  SK_GEMV_ROWS_F16_KERNELS(X)
#undef X
#define X(id, MR, WN, RK, DEPTH)                                                                               \
  if (n < max) {                                                                                               \
    typedef TileGemvRows<MR, WN, RK, DEPTH, true> P;                                                           \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 3, 0, 3, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, P::MAX_M, 8, "gemv_rows_bf16_m" #MR "_wn" #WN "_rk" #RK};           \
  }
  SK_GEMV_ROWS_BF16_KERNELS(X)
#undef X
#define X(id, NB, WN, RK, DEPTH, KMAX)                                                                         \
  if (n < max) {                                                                                               \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, true, true> P;                                                 \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 9, 0, 2, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, P::MAX_ITERS, P::MAX_M, 128,                                          \
                          "gemv_q4zpt_nb" #NB "_wn" #WN "_rk" #RK "_k" #KMAX};                                  \
  }
  SK_GEMV_Q4ZPT_KERNELS(X)
#undef X
#define X(id, MB, NB, WN, RK, DEPTH)                                                                           \
  if (n < max) {                                                                                               \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, true, true> P;                                      \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 9, 0, 0, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, P::SC_MAX_ITERS, P::MAX_M, 128, "skinny_q4zpt_mb" #MB "_wn" #WN "_rk" #RK}; \
  }
  SK_SKINNY_Q4ZPT_KERNELS(X)
#undef X
#define X(id, MB, WM, WN, RK, DEPTH)                                                                                       \
  if (n < max) {                                                                                               \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, false> P;                                                               \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 0, 0, 4, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, P::MAX_M, 8, "stream_f16_mb" #MB "_wm" #WM "_wn" #WN "_rk" #RK "_d" #DEPTH};                      \
  }
  SK_STREAM_PAIRS_F16_KERNELS(X)
#undef X
#define X(id, MB, WM, WN, RK, DEPTH)                                                                                       \
  if (n < max) {                                                                                               \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, true> P;                                                                \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 3, 0, 4, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, P::MAX_M, 8, "stream_bf16_mb" #MB "_wm" #WM "_wn" #WN "_rk" #RK "_d" #DEPTH};                     \
  }
  SK_STREAM_PAIRS_BF16_KERNELS(X)
#undef X
#define X(id, MB, WM, WN, RK, DEPTH, NB, AD, BF)                                                                 \
  if (n < max) {                                                                                                \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, BF, NB, AD, false, 2> P;                                        \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, (BF) ? 3 : 0, 0, 4, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, P::MAX_M, 8, (BF) ? "stream_bf16_mb" #MB "_nb" #NB "_wm" #WM "_wn" #WN "_rk" #RK "_d" #DEPTH \
                                                              : "stream_f16_mb" #MB "_nb" #NB "_wm" #WM "_wn" #WN "_rk" #RK "_d" #DEPTH}; \
  }
  SK_STREAM_BLOCKS_KERNELS(X)
#undef X
#define X(id, WN, RK, KH, WD, AD)                                                                                   \
  if (n < max) {                                                                                                \
    typedef TileStreamQ4<WN, RK, KH, WD, AD> P;                                                                     \
    out[n++] = KernelInfo{id, FAMILY_SKINNY, 2 /* SK_Q4 */, 0, 4, P::BM, P::BN, P::BKC, P::NT, P::LDS_BYTES, P::CTAS_PER_CU, \
                          P::TILE_ELEMS, 0, P::MAX_M, 256, "stream_q4_wn" #WN "_rk" #RK "_kh" #KH "_d" #WD};              \
  }
  SK_STREAM_Q4_KERNELS(X)
#undef X
  return n;
}

int launch_gemv_rows(int id, const SkinnyArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  switch (id) {
#define X(id_, MR, WN, RK, DEPTH)                        \
  case id_: {                                            \
    typedef TileGemvRows<MR, WN, RK, DEPTH, false> P;    \
    return launch_policy<P>(a, p, ws, s, bias);          \
  }
    SK_GEMV_ROWS_F16_KERNELS(X)
#undef X
#define X(id_, MR, WN, RK, DEPTH)                        \
  case id_: {                                            \
    typedef TileGemvRows<MR, WN, RK, DEPTH, true> P;     \
    return launch_policy<P>(a, p, ws, s, bias);          \
  }
    SK_GEMV_ROWS_BF16_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                        \
  case id_: {                                                  \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, true, true> P; \
    return launch_policy<P>(a, p, ws, s, bias);                \
  }
    SK_GEMV_Q4ZPT_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH)                                      \
  case id_: {                                                              \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, true, true> P;  \
    return launch_policy<P>(a, p, ws, s, bias);                            \
  }
    SK_SKINNY_Q4ZPT_KERNELS(X)
#undef X
#define X(id_, MB, WM, WN, RK, DEPTH)                              \
  case id_: {                                          \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, false> P;       \
    return launch_policy<P>(a, p, ws, s, bias);        \
  }
    SK_STREAM_PAIRS_F16_KERNELS(X)
#undef X
#define X(id_, MB, WM, WN, RK, DEPTH)                              \
  case id_: {                                          \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, true> P;        \
    return launch_policy<P>(a, p, ws, s, bias);        \
  }
    SK_STREAM_PAIRS_BF16_KERNELS(X)
#undef X
#define X(id_, MB, WM, WN, RK, DEPTH, NB, AD, BF)                         \
  case id_: {                                                             \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, BF, NB, AD, false, 2> P;  \
    return launch_policy<P>(a, p, ws, s, bias);                           \
  }
    SK_STREAM_BLOCKS_KERNELS(X)
#undef X
#define X(id_, WN, RK, KH, WD, AD)                   \
  case id_: {                                    \
    typedef TileStreamQ4<WN, RK, KH, WD, AD> P;      \
    return launch_policy<P>(a, p, ws, s, bias);  \
  }
    SK_STREAM_Q4_KERNELS(X)
#undef X
  }
  return (int)hipErrorInvalidValue;
}

int occupancy_gemv_rows(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, MR, WN, RK, DEPTH)                                                                        \
  case id_: {                                                                                            \
    typedef TileGemvRows<MR, WN, RK, DEPTH, false> P;                                                    \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_ROWS_F16_KERNELS(X)
#undef X
#define X(id_, MR, WN, RK, DEPTH)                                                                        \
  case id_: {                                                                                            \
    typedef TileGemvRows<MR, WN, RK, DEPTH, true> P;                                                     \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_ROWS_BF16_KERNELS(X)
#undef X
#define X(id_, NB, WN, RK, DEPTH, KMAX)                                                                  \
  case id_: {                                                                                            \
    typedef TileGemvQ4<NB, WN, RK, DEPTH, KMAX, true, true> P;                                           \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_GEMV_Q4ZPT_KERNELS(X)
#undef X
#define X(id_, MB, NB, WN, RK, DEPTH)                                                                    \
  case id_: {                                                                                            \
    typedef TileSkinny<MB, NB, WN, RK, true, DEPTH, false, true, true> P;                                \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_SKINNY_Q4ZPT_KERNELS(X)
#undef X
#define X(id_, MB, WM, WN, RK, DEPTH)                                                                                \
  case id_: {                                                                                            \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, false> P;                                                         \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_STREAM_PAIRS_F16_KERNELS(X)
#undef X
#define X(id_, MB, WM, WN, RK, DEPTH)                                                                                \
  case id_: {                                                                                            \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, true> P;                                                          \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_STREAM_PAIRS_BF16_KERNELS(X)
#undef X
#define X(id_, MB, WM, WN, RK, DEPTH, NB, AD, BF)                                                        \
  case id_: {                                                                                            \
    typedef TileStreamPairs<MB, WM, WN, RK, DEPTH, BF, NB, AD, false, 2> P;                                 \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_STREAM_BLOCKS_KERNELS(X)
#undef X
#define X(id_, WN, RK, KH, WD, AD)                                                                           \
  case id_: {                                                                                            \
    typedef TileStreamQ4<WN, RK, KH, WD, AD> P;                                                              \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_skinny_kernel<P>, P::NT, 0) != hipSuccess) \
      return -1;                                                                                         \
    return occ;                                                                                          \
  }
    SK_STREAM_Q4_KERNELS(X)
#undef X
  }
  return -1;
}

}  // namespace sk
