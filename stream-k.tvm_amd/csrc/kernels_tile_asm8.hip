// The one-byte instances (int8, fp8) of the four-wave assembly-loop tile kernels (tile_f16_asm.h).
#include "launch.h"
#include "sk_persistent.h"
#include "tile_f16_asm.h"

namespace sk {

template <class P, bool FIXUP>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_tile_asm_kernel(typename P::Args a, DevPlan plan, Workspace ws,
                                                                            const void *bias) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  run_persistent<P, FIXUP, true>(a, plan, ws, smem, bias);
}

int tile_asm8_kernel_infos(KernelInfo *out, int max) {
  int n = 0;
  // (the one-byte instances count bk and K in elements: 128 per iteration)
  static const int dtypes[5] = {0 /* SK_F16 */, 3 /* SK_BF16 */, 6 /* SK_I8 */, 5 /* SK_F8E4M3 */, 8 /* SK_F8E5M2 */};
  static const char *const names[2][5] = {
      {"tile_f16_nt_asm_256x256x64", "tile_bf16_nt_asm_256x256x64", "tile_i8_nt_asm_256x256x128",
       "tile_f8e4m3_nt_asm_256x256x128", "tile_f8e5m2_nt_asm_256x256x128"},
      {"tile_f16_nn_asm_256x256x64", "tile_bf16_nn_asm_256x256x64", "", "", ""}};
#define X(id, MODE, NN)                                                                                          \
  if (n < max) {                                                                                                 \
    typedef TileF16Asm<MODE, NN> P;                                                                              \
    const int kb = (MODE) >= 2 ? 2 : 1;                                                                          \
    out[n++] = KernelInfo{id, FAMILY_TILE, dtypes[MODE], (NN) ? 1 : 0, 7, P::BM, P::BN, P::BK * kb, P::NT,       \
                          P::LDS_TOTAL, P::CTAS_PER_CU, P::TILE_ELEMS, 0, 0, 64 * kb, names[(NN) ? 1 : 0][MODE]}; \
  }
  SK_TILE_ASM8_KERNELS(X)
#undef X
  return n;
}

// data-parallel launches use the instance without fix-up code
int launch_tile_asm8(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  switch (id) {
#define X(id_, MODE, NN)                                                                                              \
  case id_: {                                                                                                     \
    typedef TileF16Asm<MODE, NN> P;                                                                                   \
    if (p.sk_tiles == 0)                                                                                          \
      hipLaunchKernelGGL((sk_tile_asm_kernel<P, false>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);        \
    else                                                                                                          \
      hipLaunchKernelGGL((sk_tile_asm_kernel<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);         \
    return (int)hipGetLastError();                                                                                \
  }
    SK_TILE_ASM8_KERNELS(X)
#undef X
  }
  return launch_tile_q4(id, a, p, ws, s, bias);
}

int occupancy_tile_asm8(int id) {
  int occ = 0;
  switch (id) {
#define X(id_, MODE, NN)                                                                                                    \
  case id_: {                                                                                                           \
    typedef TileF16Asm<MODE, NN> P;                                                                                         \
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, sk_tile_asm_kernel<P, true>, P::NT, 0) != hipSuccess) return -1; \
    return occ;                                                                                                         \
  }
    SK_TILE_ASM8_KERNELS(X)
#undef X
  }
  return occupancy_tile_q4(id);
}

}  // namespace sk
