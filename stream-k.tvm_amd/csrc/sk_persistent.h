// The persistent Stream-K + data-parallel loop every kernel family shares.
//
// A policy class P supplies the tile arithmetic:
//   P::Args, P::Acc, P::TILE_ELEMS, P::NT
//   P::mac(args, acc, pm, pn, k0, n, smem)      accumulate K-iterations [k0, k0+n) of tile (pm,pn)
//   P::store_c(args, acc, pm, pn, smem, bias)   write the finished tile to C (+ optional bias row)
//   P::store_partial / add_partial / atomic_partial / take_partial   fp32 partials in workspace
//
// Control flow follows the reference's persistent kernel: every CTA first walks its share of the
// Stream-K iteration space (streamk_fp32.py:93-136), then its data-parallel tiles (:149-158).
#pragma once
#include <type_traits>

#include "sk_device.h"

namespace sk {

// policies that lend the persistent loop its one word of LDS (see run_persistent)
template <class P, class = void>
struct fixup_word_in_lds { static constexpr bool value = false; };
template <class P>
struct fixup_word_in_lds<P, std::void_t<decltype(P::FIXUP_WORD_IN_LDS)>> { static constexpr bool value = P::FIXUP_WORD_IN_LDS; };

// policies whose half tiles can travel rounded to 16 bits (store_partial_half16 / add_partial_half16)
template <class P, class = void>
struct has_halves16 { static constexpr bool value = false; };
template <class P>
struct has_halves16<P, std::void_t<decltype(P::HALVES16)>> { static constexpr bool value = P::HALVES16; };
template <class P>
__device__ __forceinline__ void park_half(const DevPlan &plan, const typename P::Acc &acc, float *dst, int h) {
  if constexpr (has_halves16<P>::value) {
    if (plan.partials16) {
      P::store_partial_half16(acc, dst, h);
      return;
    }
  }
  P::store_partial_half(acc, dst, h);
}
template <class P>
__device__ __forceinline__ void take_half(const DevPlan &plan, typename P::Acc &acc, const float *src, int h) {
  if constexpr (has_halves16<P>::value) {
    if (plan.partials16) {
      P::add_partial_half16(acc, src, h);
      return;
    }
  }
  P::add_partial_half(acc, src, h);
}

// optional members of a policy: COHERENT_REDUCE (partials of the REDUCE fix-up travel with device-scope
// accesses; default: as COHERENT_PARTIALS says), HALVES (the policy has store_partial_half /
// add_partial_half / store_c_half, see below) and ATOMIC_C (the policy has atomic_c: its accumulators added to C
// with packed 16-bit atomics)
template <class P, class = void>
struct reduce_is_coherent { static constexpr bool value = P::COHERENT_PARTIALS; };
template <class P>
struct reduce_is_coherent<P, std::void_t<decltype(P::COHERENT_REDUCE)>> { static constexpr bool value = P::COHERENT_REDUCE; };
template <class P, class = void>
struct has_atomic_c { static constexpr bool value = false; };
template <class P>
struct has_atomic_c<P, std::void_t<decltype(P::ATOMIC_C)>> { static constexpr bool value = P::ATOMIC_C; };
// CROSS_TILE_PREFETCH: the policy has prefetch_first_stage / epilogue_lds_free and mac takes a last argument that says
// the first stage of the segment has already been requested (see the loop below)
template <class P, class = void>
struct has_prefetch { static constexpr bool value = false; };
template <class P>
struct has_prefetch<P, std::void_t<decltype(P::CROSS_TILE_PREFETCH)>> { static constexpr bool value = P::CROSS_TILE_PREFETCH; };
template <class P, class = void>
struct has_halves { static constexpr bool value = false; };
template <class P>
struct has_halves<P, std::void_t<decltype(P::HALVES)>> { static constexpr bool value = P::HALVES; };

// FIXUP = false: an instance for launches without Stream-K tiles.  Every segment is a whole tile
// and the fix-up code is not compiled in -- its hundreds of partial-tile addresses otherwise
// shape the register allocation of the main loop (spills in the 256x256 kernels).
// BIAS: the kernel has the optional bias row among its arguments (bias_arg, may still be null); without it the
// epilogue's bias code is not compiled in.  The small-M kernels exist in both forms, because even an unused
// bias argument costs them 0.2-0.3 us of their 7-12 us (argument loads and waits at kernel entry move).
template <class P, bool FIXUP = true, bool BIAS = false>
__device__ __forceinline__ void run_persistent(const typename P::Args &a, const DevPlan &plan,
                                               const Workspace &ws, char *smem, const void *bias_arg = nullptr) {
  // one word through which thread 0 tells the CTA whether it arrived last at a tile.  Policies whose LDS is dead
  // between two calls of mac and who need all of it (FIXUP_WORD_IN_LDS) lend its first word
  int *s_word_p;
  if constexpr (fixup_word_in_lds<P>::value) {
    s_word_p = reinterpret_cast<int *>(smem);
  } else {
    __shared__ int s_word_own;
    s_word_p = &s_word_own;
  }
  int &s_word = *s_word_p;
  // Fetch the bias pointer with the other kernel arguments: left to the compiler it is read from the argument
  // buffer right before the first store, a dependent scalar load (~0.3 us) at the end of every CTA.
  const void *bias = nullptr;
  if constexpr (BIAS) {
    bias = bias_arg;
    asm volatile("" ::"s"(bias));
  }
  const int pid = logical_pid(plan);
  const int ipt = plan.ipt;
  typename P::Acc acc;

  // The instance without fix-up code is only launched for plans without Stream-K tiles, whose range is empty.
  // P::LEAN_ENTRY: leave its computation out there.  Worth 0.8 % to the 256x256 tile kernels at 8192^3; the
  // small-M kernels start 0.2-0.3 us later without it (their argument loads get ordered differently), so they
  // keep it.
  int start = 0, last = 0;
  if constexpr (FIXUP || !P::LEAN_ENTRY) sk_range(plan, pid, start, last);
  int dp_tile = (FIXUP || !P::LEAN_ENTRY) ? plan.sk_tiles + pid : pid;

  // One loop body serves both phases so that the MAC loop and the epilogue exist once in the
  // kernel: first the CTA's Stream-K segments, then its data-parallel tiles
  // (tile = streamk_tiles + pid + wave * grid, streamk_fp32.py:149-158).
  // Policies with CROSS_TILE_PREFETCH: once every wave has left the MAC loop the LDS stages are free, and where the
  // epilogue of this tile will not use them (stores straight from registers) the loads of the next segment's first
  // stage go out before the fix-up and the epilogue instead of after them: a tile costs the 256 x 256 kernels about
  // 13 000 cycles outside its loop, most of them the epilogue and the first loads' trip to memory, one after the other.
  bool first_stage_requested = false;
  for (;;) {
    int tile, k0, n;
    if (start < last) {
      tile = plan.by_ipt.div(start);
      k0 = start - tile * ipt;
      n = min(ipt - k0, last - start);
      start += n;
    } else if (dp_tile < plan.total_tiles) {
      tile = dp_tile;
      k0 = 0;
      n = ipt;
      dp_tile += plan.grid;
    } else {
      break;
    }
    int pm, pn;
    tile_coords(plan, tile, pm, pn);
    if constexpr (has_prefetch<P>::value) {
      P::mac(a, acc, pm, pn, k0, n, smem, first_stage_requested);
      first_stage_requested = false;
      // the segment after this one (start and dp_tile already point behind the current one)
      int next_tile = -1, next_k0 = 0, next_n = ipt;
      if (start < last) {
        next_tile = plan.by_ipt.div(start);
        next_k0 = start - next_tile * ipt;
        next_n = min(ipt - next_k0, last - start);
      } else if (dp_tile < plan.total_tiles) {
        next_tile = dp_tile;
      }
      if (next_tile >= 0 && P::epilogue_lds_free(a, pn, bias)) {
        int npm, npn;
        tile_coords(plan, next_tile, npm, npn);
        P::prefetch_first_stage(a, npm, npn, next_k0, next_n);
        first_stage_requested = true;
      }
    } else {
      P::mac(a, acc, pm, pn, k0, n, smem);
    }

    // a segment that is the whole tile is simply stored (streamk_fp32.py:128-129)
    bool store = (n == ipt) || !FIXUP;
    if (FIXUP && !store) {
      if (plan.fixup == FIXUP_ATOMIC_C) {
        // the reference's fix-up (streamk_fp16.py:248-255): every partial goes straight into C, which the
        // launcher has zero-filled; nobody finishes the tile
        if constexpr (has_atomic_c<P>::value) P::atomic_c(a, acc, pm, pn);
      } else if (plan.fixup == FIXUP_ATOMIC) {
        // fp32 atomicAdd into the tile's accumulation buffer; whoever completes the K range
        // converts and stores, then leaves buffer and counter zeroed for the next launch.
        float *part = ws.partials + (size_t)tile * P::TILE_ELEMS;
        P::atomic_partial(acc, part);
        wait_own_memory_ops();
        __syncthreads();
        if (threadIdx.x == 0) {
          int old = __hip_atomic_fetch_add(&ws.flags[tile], n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          s_word = (old + n == ipt);
          // the last arriver reads the sum with ordinary loads: drop stale L2 lines first
          if (!P::COHERENT_PARTIALS && s_word) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
        __syncthreads();
        store = s_word != 0;
        __syncthreads();
        if (store) {
          P::take_partial(acc, part);
          if (threadIdx.x == 0)
            __hip_atomic_store(&ws.flags[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else if (has_halves<P>::value && plan.halves) {
        // Every Stream-K tile of this plan is shared by exactly two CTAs, each with this one segment.
        // Instead of one of them finishing the whole tile while the other idles, each finishes half of
        // it: it parks the other half of its accumulators in its slot, raises its flag, waits for the
        // peer's, adds the peer's contribution to the half it kept and stores that half of C.  The
        // exchange moves the same bytes as the owner scheme, but over twice as many CTAs at once, and
        // the sum of two terms does not depend on their order.
        if constexpr (has_halves<P>::value) {
          if (plan.halves == 2) {
            // Four equal segments per tile, CTAs base .. base + 3.  First exchange: the pairs (0, 1) and (2, 3) swap
            // halves as above; CTAs 0 and 2 then hold the pair's sum of half 0, CTAs 1 and 3 that of half 1.
            // Second exchange: CTA 2 hands its half to CTA 0 and CTA 3 its half to CTA 1 (parked in the other half of
            // their slots, which nobody reads in the first; flags of their own, grid entries further on), and CTAs 0
            // and 1 finish half of C each.  Every flag has one reader, who clears it; the order of the sums is
            // fixed.  Two half-tile exchanges in a row instead of one CTA adding three partial tiles.
            const int q = plan.by_full.div(k0), base = pid - q;
            const int half = q & 1, peer1 = base + (q ^ 1);
            const int units = (int)(((size_t)(pid + 1) * P::TILE_ELEMS * 4 + 255) >> 8);
            bool ok = true;
            park_half<P>(plan, acc, ws.partials + (size_t)pid * P::TILE_ELEMS, 1 - half);
            signal_partial_ready<true>(&ws.flags[pid], ws.status + WS_DIRTY, units);
            if (wait_partials_ready<true>(&ws.flags[peer1], 1, plan.spin_limit)) {
              take_half<P>(plan, acc, ws.partials + (size_t)peer1 * P::TILE_ELEMS, half);
              clear_flags_after_use(&ws.flags[peer1], 1);
            } else {
              ok = false;
            }
            if (q >= 2) {
              park_half<P>(plan, acc, ws.partials + (size_t)pid * P::TILE_ELEMS, half);
              signal_partial_ready<true>(&ws.flags[plan.grid + pid], ws.status + WS_DIRTY, units);
            } else {
              const int peer2 = pid + 2;
              if (wait_partials_ready<true>(&ws.flags[plan.grid + peer2], 1, plan.spin_limit)) {
                take_half<P>(plan, acc, ws.partials + (size_t)peer2 * P::TILE_ELEMS, half);
                clear_flags_after_use(&ws.flags[plan.grid + peer2], 1);
              } else {
                ok = false;
              }
              P::store_c_half(a, acc, pm, pn, smem, bias, half);
            }
            if (!ok && threadIdx.x == 0) ws.status[WS_STATUS] = -8;  // SK_ERR_TIMEOUT
            continue;
          }
          const int half = k0 != 0 ? 1 : 0, peer = k0 != 0 ? pid - 1 : pid + 1;
          park_half<P>(plan, acc, ws.partials + (size_t)pid * P::TILE_ELEMS, 1 - half);
          signal_partial_ready<true>(&ws.flags[pid], ws.status + WS_DIRTY,
                                     (int)(((size_t)(pid + 1) * P::TILE_ELEMS * 4 + 255) >> 8));
          if (!wait_partials_ready<true>(&ws.flags[peer], 1, plan.spin_limit)) {
            if (threadIdx.x == 0) ws.status[WS_STATUS] = -8;  // SK_ERR_TIMEOUT
          } else {
            take_half<P>(plan, acc, ws.partials + (size_t)peer * P::TILE_ELEMS, half);
            clear_flags_after_use(&ws.flags[peer], 1);
          }
          P::store_c_half(a, acc, pm, pn, smem, bias, half);
        }
      } else if (k0 != 0) {
        // not the tile's first CTA: park the partial in this CTA's slot and raise its flag
        P::store_partial(acc, ws.partials + (size_t)pid * P::TILE_ELEMS);
        signal_partial_ready<reduce_is_coherent<P>::value>(
            &ws.flags[pid], ws.status + WS_DIRTY, (int)(((size_t)(pid + 1) * P::TILE_ELEMS * 4 + 255) >> 8));
      } else {
        // tile's first CTA: wait for all followers at once, then add their partials in ascending
        // CTA order and store
        const int npeers = sk_pid_of_iter(plan, (tile + 1) * ipt - 1) - pid;
        if (!wait_partials_ready<reduce_is_coherent<P>::value, fixup_word_in_lds<P>::value>(&ws.flags[pid + 1], npeers,
                                                                                            plan.spin_limit, s_word_p)) {
          if (threadIdx.x == 0) ws.status[WS_STATUS] = -8;  // SK_ERR_TIMEOUT
        } else {
          for (int p = 1; p <= npeers; ++p) P::add_partial(acc, ws.partials + (size_t)(pid + p) * P::TILE_ELEMS);
          clear_flags_after_use(&ws.flags[pid + 1], npeers);
        }
        store = true;
      }
    }
    if (store) P::store_c(a, acc, pm, pn, smem, bias);
  }
}

}  // namespace sk
