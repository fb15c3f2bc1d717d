// Kernel entry points and the launcher shared by the small-M translation units.
#pragma once
#include "launch.h"
#include "sk_persistent.h"

namespace sk {

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
// The hardware deals workgroups round-robin to the 8 XCDs.  Policies with XCD_CONTIGUOUS give XCD x a contiguous range
// of tiles, as the planned launches do (logical_pid), so that each XCD streams one contiguous eighth of the weights;
// the others take tile = block index (measured per kernel family).
template <class P, class = void>
struct xcd_contiguous { static constexpr bool value = false; };
template <class P>
struct xcd_contiguous<P, std::void_t<decltype(P::XCD_CONTIGUOUS)>> { static constexpr bool value = P::XCD_CONTIGUOUS; };
template <class P>
__device__ __forceinline__ int first_tile_of_block() {
  const int b = blockIdx.x, grid = gridDim.x, x = b & 7;
  if constexpr (xcd_contiguous<P>::value) return x * (grid >> 3) + min(x, grid & 7) + (b >> 3);
  return b;
}

// policies with mac_again: what a CTA's later tiles skip because its first tile left it in LDS (the row of A)
template <class P, class = void>
struct has_mac_again { static constexpr bool value = false; };
template <class P>
struct has_mac_again<P, std::void_t<decltype(&P::mac_again)>> { static constexpr bool value = true; };
template <class P>
__device__ __forceinline__ void mac_of_tile(const typename P::Args &a, typename P::Acc &acc, int tile, int ipt, char *smem, bool first) {
  if constexpr (has_mac_again<P>::value) {
    if (!first) {
      P::mac_again(a, acc, 0, tile, 0, ipt, smem);
      return;
    }
  }
  P::mac(a, acc, 0, tile, 0, ipt, smem);
}

// policies with mac_tiles: the whole data-parallel loop of a CTA, stores included (a tile's first loads are requested
// while the tile before is still being summed)
template <class P, class = void>
struct has_mac_tiles { static constexpr bool value = false; };
template <class P>
struct has_mac_tiles<P, std::void_t<decltype(&P::mac_tiles)>> { static constexpr bool value = true; };

template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_dp_kernel(typename P::Args a, int total_tiles, int ipt) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  const int tile0 = first_tile_of_block<P>();
  if constexpr (has_mac_tiles<P>::value) {
    P::mac_tiles(a, tile0, gridDim.x, total_tiles, ipt, smem, nullptr);
    return;
  }
  typename P::Acc acc;
  for (int tile = tile0; tile < total_tiles; tile += gridDim.x) {
    mac_of_tile<P>(a, acc, tile, ipt, smem, tile == tile0);
    P::store_c(a, acc, 0, tile, smem, nullptr);
  }
}
template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_dp_kernel_bias(typename P::Args a, int total_tiles, int ipt,
                                                                                  const void *bias_arg) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  const void *bias = bias_arg;
  asm volatile("" ::"s"(bias));  // fetched with the other arguments, not before the first store
  const int tile0 = first_tile_of_block<P>();
  if constexpr (has_mac_tiles<P>::value) {
    P::mac_tiles(a, tile0, gridDim.x, total_tiles, ipt, smem, bias);
    return;
  }
  typename P::Acc acc;
  for (int tile = tile0; tile < total_tiles; tile += gridDim.x) {
    mac_of_tile<P>(a, acc, tile, ipt, smem, tile == tile0);
    P::store_c(a, acc, 0, tile, smem, bias);
  }
}

// The same with the operands as 14 scalar kernel arguments instead of the argument structure, for the common call
// (rows of A and C packed, no per-group zero points, no bias).  Scalar arguments can be preloaded into scalar
// registers by the command processor before the first wave starts (this translation unit is compiled with a
// kernel-argument preload count; a structure passed by value cannot be), which takes the ~1 us "wait for the kernel
// arguments" off the front of launches that run for 6 to 40 us.  One tile per CTA; the iterations per tile follow from
// K.  (Where the firmware does not preload, the kernel starts at its ordinary entry, which loads the arguments.)
template <class P>
__global__ __launch_bounds__(P::NT, P::WAVES_PER_EU) void sk_skinny_flat_kernel(const half_t *A, const void *W, const half_t *scales,
                                                                              half_t *C, int M, int N, int K, int ldw, int zero,
                                                                              int groups) {
  __shared__ __attribute__((aligned(16))) char smem[P::LDS_BYTES];
  SkinnyArgs a;
  a.A = A; a.W = W; a.scales = scales; a.C = C;
  a.M = M; a.N = N; a.K = K;
  a.lda = K; a.ldw = ldw; a.ldc = N;
  a.zero = zero; a.groups = groups; a.zeros = nullptr;
  typename P::Acc acc;
  const int tile = first_tile_of_block<P>();
  P::mac(a, acc, 0, tile, 0, (K + P::BKC - 1) / P::BKC, smem);
  P::store_c(a, acc, 0, tile, smem, nullptr);
}

// NO_FLAT_ARGS: policies whose scalar-argument instance the compiler does not fit into the register budget
template <class P, class = void>
struct no_flat_args { static constexpr bool value = false; };
template <class P>
struct no_flat_args<P, std::void_t<decltype(P::NO_FLAT_ARGS)>> { static constexpr bool value = P::NO_FLAT_ARGS; };

template <class P>
static inline int launch_policy(const SkinnyArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias) {
  if (p.sk_tiles == 0 && p.tiles_m != 1) return (int)hipErrorInvalidValue;  // (no plan of these kernels has two tile rows)
  if (bias != nullptr) {
    if (p.sk_tiles == 0)
      hipLaunchKernelGGL((sk_skinny_dp_kernel_bias<P>), dim3(p.grid), dim3(P::NT), 0, s, a, p.total_tiles, p.ipt, bias);
    else
      hipLaunchKernelGGL((sk_skinny_kernel_bias<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws, bias);
  } else if (p.sk_tiles == 0) {
    if constexpr (!no_flat_args<P>::value) {
      if (p.grid == p.total_tiles && p.ipt == (a.K + P::BKC - 1) / P::BKC && a.zeros == nullptr && a.lda == a.K && a.ldc == a.N &&
          a.ldw <= 0x7fffffff) {
        hipLaunchKernelGGL((sk_skinny_flat_kernel<P>), dim3(p.grid), dim3(P::NT), 0, s, a.A, a.W, a.scales, a.C, a.M, a.N, a.K,
                           (int)a.ldw, a.zero, a.groups);
        return (int)hipGetLastError();
      }
    }
    hipLaunchKernelGGL((sk_skinny_dp_kernel<P>), dim3(p.grid), dim3(P::NT), 0, s, a, p.total_tiles, p.ipt);
  } else {
    hipLaunchKernelGGL((sk_skinny_kernel<P, true>), dim3(p.grid), dim3(P::NT), 0, s, a, p, ws);
  }
  return (int)hipGetLastError();
}

}  // namespace sk
