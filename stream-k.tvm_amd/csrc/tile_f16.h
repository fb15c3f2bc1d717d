// fp16 tile arithmetic for the LDS-tiled kernels: BM x BN x BK CTA tile, WM x WN waves, each wave
// a (TM*32) x (TN*32) block of v_mfma_f32_32x32x16_f16 accumulators.
//
// Replaces the reference's inner MAC (streamk_fp16.py:196-240: cp.async -> ldmatrix -> mma.sync)
// with: 16-byte global loads -> registers -> padded LDS rows -> ds_read_b128 fragments -> MFMA.
// LDS rows are padded by 8 halfs (the reference's pad_factor, streamk_fp16_block_reduce.py:158-165)
// which makes the 32-row fragment reads bank-conflict free.
#pragma once
#include "sk_device.h"

namespace sk {

struct GemmArgs {
  const half_t *A;
  const half_t *B;
  half_t *C;
  int M, N, K;
  int64_t lda, ldb, ldc;
  float alpha;  // fp8 kernels: C = fp16(alpha * A B^T); unused elsewhere
  // Q4 tile kernels: B points at the packed nibbles [N, K/2] (ldb = K/2 bytes per row); scales [N, groups] fp16,
  // one per 128 K-values; the scalar zero point
  const half_t *scales;
  int zero, groups;
};

template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct TileF16NT {
  typedef GemmArgs Args;
  static constexpr bool LEAN_ENTRY = true;  // see run_persistent
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int NT = WM * WN * 64;
  static constexpr int TM = BM / (WM * 32), TN = BN / (WN * 32);
  static constexpr int LDK = BK + 8;
  static constexpr int A_STAGE = BM * LDK, B_STAGE = BN * LDK, STAGE = A_STAGE + B_STAGE;
  static constexpr int CPR = BK / 8;  // 16-byte chunks per tile row
  static constexpr int A_LOADS = BM * CPR / NT, B_LOADS = BN * CPR / NT;
  static constexpr int ROWS_PER_PASS = NT / CPR;
  static constexpr int WTM = TM * 32, WTN = TN * 32;  // wave tile
  static constexpr int LDC = WTN + 8;                 // epilogue row (halfs)
  static constexpr int LDS_STAGING = 2 * STAGE * 2;
  static constexpr int LDS_EPILOGUE = WM * WN * WTM * LDC * 2;
  static constexpr int LDS_BYTES = LDS_STAGING > LDS_EPILOGUE ? LDS_STAGING : LDS_EPILOGUE;
  static constexpr int LDS_TOTAL = LDS_BYTES;
  static constexpr int TILE_ELEMS = BM * BN;
  static constexpr int NV4 = TM * TN * 4;  // float4 groups per thread
  // co-resident CTAs per CU the kernel is compiled for (register budget = 512 / waves per SIMD)
  static constexpr int CTAS_PER_CU_REGS = NT >= 512 ? 1 : (TM * TN <= 1 ? 4 : 2);
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_BYTES + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_REGS < CTAS_PER_CU_LDS ? CTAS_PER_CU_REGS : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % 16 == 0, "tile shape");
  static_assert((BM * CPR) % NT == 0 && (BN * CPR) % NT == 0, "loads must divide evenly");

  struct Acc {
    floatx16 c[TM][TN];
  };

  // Accumulates K-iterations [k0, k0+n) of tile (pm, pn).  acc[i][j][r] ends up holding
  // C[pm*BM + wm*WTM + i*32 + lane%32][pn*BN + wn*WTN + j*32 + 8*(r/4) + 4*(lane/32) + r%4].
  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n,
                                             char *smem) {
    half_t *lds = reinterpret_cast<half_t *>(smem);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc.c[i][j][r] = 0.f;

    // global addressing: one buffer descriptor per operand covering the tile's rows, so rows past
    // the matrix edge read as zero.  Per lane: one 32-bit offset per operand; per load: a uniform
    // (scalar) offset.
    const int ld_row = tid / CPR, ld_kc = tid % CPR;
    const int rows_a = min(BM, a.M - pm * BM), rows_b = min(BN, a.N - pn * BN);
    const BufferRsrc rsrc_a = make_rsrc(a.A + (int64_t)pm * BM * a.lda, (uint32_t)(rows_a * a.lda * 2));
    const BufferRsrc rsrc_b = make_rsrc(a.B + (int64_t)pn * BN * a.ldb, (uint32_t)(rows_b * a.ldb * 2));
    const uint32_t voff_a = (uint32_t)(ld_row * a.lda + ld_kc * 8) * 2;
    const uint32_t voff_b = (uint32_t)(ld_row * a.ldb + ld_kc * 8) * 2;
    const uint32_t pass_a = (uint32_t)(ROWS_PER_PASS * a.lda * 2), pass_b = (uint32_t)(ROWS_PER_PASS * a.ldb * 2);
    const int lds_st = ld_row * LDK + ld_kc * 8;
    const int a_rd = (wm * WTM + (lane & 31)) * LDK + (lane >> 5) * 8;
    const int b_rd = A_STAGE + (wn * WTN + (lane & 31)) * LDK + (lane >> 5) * 8;
    // only the last K-iteration of a tile can hang over K (K % 8 == 0: a 16-byte chunk is all in
    // or all out)
    const int tail_kt = (a.K % BK != 0) ? (a.K / BK) : -1;

    uint4v ra[A_LOADS], rb[B_LOADS];
    auto load_global = [&](int kt) {
      const uint32_t koff = (uint32_t)kt * (BK * 2);
      uint32_t va = voff_a, vb = voff_b;
      if (kt == tail_kt && kt * BK + ld_kc * 8 >= a.K) va = vb = OOB_OFFSET;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) ra[i] = buffer_load_16(rsrc_a, va, koff + i * pass_a);
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i) rb[i] = buffer_load_16(rsrc_b, vb, koff + i * pass_b);
    };

    load_global(k0);
    for (int it = 0; it < n; ++it) {
      half_t *st = lds + (it & 1) * STAGE;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i)
        *reinterpret_cast<uint4v *>(st + lds_st + i * ROWS_PER_PASS * LDK) = ra[i];
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i)
        *reinterpret_cast<uint4v *>(st + A_STAGE + lds_st + i * ROWS_PER_PASS * LDK) = rb[i];
      __syncthreads();
      if (it + 1 < n) load_global(k0 + it + 1);
      // fragments are double-buffered in registers: the ds_reads of K-step kk+1 are issued before
      // the MFMAs of step kk so that LDS latency hides behind the matrix pipe
      half8v fa[2][TM], fb[2][TN];
      auto read_frags = [&](int buf, int kk) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa[buf][i] = *reinterpret_cast<const half8v *>(st + a_rd + i * 32 * LDK + kk * 16);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          fb[buf][j] = *reinterpret_cast<const half8v *>(st + b_rd + j * 32 * LDK + kk * 16);
      };
      read_frags(0, 0);
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        if (kk + 1 < BK / 16) read_frags((kk + 1) & 1, kk + 1);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc.c[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk & 1][j], fa[kk & 1][i], acc.c[i][j], 0, 0, 0);
        // one DS read per MFMA keeps the order above through instruction scheduling
        if (kk + 1 < BK / 16) {
#pragma unroll
          for (int g = 0; g < TM + TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          }
        }
      }
    }
    __syncthreads();  // staging buffers are free again (next segment or the epilogue may write)
  }

  // fp32 -> fp16, through a per-wave LDS patch so that global stores are 16 bytes per lane and
  // 128 bytes contiguous per row.
  // (two copies behind one uniform branch, so that the epilogue without a bias carries none of its code)
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int pm, int pn, char *smem,
                                                 const void *bias) {
    if (bias == nullptr)
      store_c_impl<false>(a, acc, pm, pn, smem, nullptr);
    else
      store_c_impl<true>(a, acc, pm, pn, smem, bias);
  }
  template <bool BIAS>
  static __device__ __forceinline__ void store_c_impl(const Args &a, const Acc &acc, int pm, int pn, char *smem,
                                                      const void *epi) {
    const half_t *bias = BIAS ? epi_bias(epi) : nullptr;
    const int act = BIAS ? epi_act(epi) : 0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    half_t *patch = reinterpret_cast<half_t *>(smem) + wave * (WTM * LDC);
    const int bias_col0 = BIAS ? pn * BN + wn * WTN + pin_here(lane >> 5) * 4 : 0;  // not hoisted out of the persistent loop
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          half4v h;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = acc.c[i][j][q * 4 + e];
            if constexpr (BIAS) x = activate(x + bias_at(bias, bias_col0 + j * 32 + q * 8 + e, a.N), act);
            h[e] = (half_t)x;
          }
          *reinterpret_cast<half4v *>(patch + (i * 32 + (lane & 31)) * LDC + j * 32 + q * 8 +
                                      (lane >> 5) * 4) = h;
        }
    // the patch is private to the wave: no CTA barrier, only LDS ordering within the wave
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int row0 = pm * BM + wm * WTM, col0 = pn * BN + wn * WTN;
    constexpr int CPRC = WTN / 8;
    const bool vec_ok = (a.ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 15) == 0);
#pragma unroll
    for (int s = 0; s < WTM * CPRC / 64; ++s) {
      int idx = s * 64 + lane;
      int r = idx / CPRC, cc = idx % CPRC;
      int grow = row0 + r, gcol = col0 + cc * 8;
      if (grow < a.M && gcol < a.N) {
        const half_t *src = patch + r * LDC + cc * 8;
        half_t *dst = a.C + (int64_t)grow * a.ldc + gcol;
        if (vec_ok && gcol + 8 <= a.N) {
          *reinterpret_cast<uint4v *>(dst) = *reinterpret_cast<const uint4v *>(src);
        } else {
          for (int e = 0; e < 8 && gcol + e < a.N; ++e) dst[e] = src[e];
        }
      }
    }
    __syncthreads();  // patches overlap the staging buffers of the next tile
  }

  // Partial tiles are large (BM*BN*4 bytes) and few: they go through the L2 with ordinary 16-byte
  // accesses, and each CTA pays one L2 write-back (contributor) or invalidate (owner) per fix-up.
  static constexpr bool COHERENT_PARTIALS = false;

  // Partials live in the workspace in "fragment order": float4 group v of thread t sits at
  // (v * NT + t) * 4, so every access is a fully coalesced 16 bytes per lane.
  static __device__ __forceinline__ floatx4 grp(const Acc &acc, int v) {
    const floatx16 &c = acc.c[(v / 4) / TN][(v / 4) % TN];
    const int q = (v % 4) * 4;
    return floatx4{c[q], c[q + 1], c[q + 2], c[q + 3]};
  }
  static __device__ __forceinline__ void store_partial(const Acc &acc, float *dst) {
    dst = pin_here(dst);
#pragma unroll
    for (int v = 0; v < NV4; ++v)
      *reinterpret_cast<floatx4 *>(dst + ((size_t)v * NT + threadIdx.x) * 4) = grp(acc, v);
  }
  static __device__ __forceinline__ void add_partial(Acc &acc, const float *src) {
    src = pin_here(src);
#pragma unroll
    for (int v = 0; v < NV4; ++v) {
      floatx4 x = *reinterpret_cast<const floatx4 *>(src + ((size_t)v * NT + threadIdx.x) * 4);
      floatx16 &c = acc.c[(v / 4) / TN][(v / 4) % TN];
      const int q = (v % 4) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) c[q + e] += x[e];
      // keep at most 8 loads in flight: hoisting all of them would double the register need
      if (v % 8 == 7) asm volatile("" ::: "memory");
    }
  }
  // The accumulation buffer of the ATOMIC fix-up is element-major (element s of thread t at
  // s * NT + t) so that the 64 atomics of one instruction fall on consecutive addresses.
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst) {
    dst = pin_here(dst);
#pragma unroll
    for (int v = 0; v < NV4; ++v) {
      floatx4 x = grp(acc, v);
#pragma unroll
      for (int e = 0; e < 4; ++e) atomic_add_f32(dst + (size_t)(v * 4 + e) * NT + threadIdx.x, x[e]);
    }
  }
  // reads the completed sum and leaves zeros behind
  static __device__ __forceinline__ void take_partial(Acc &acc, float *src) {
    src = pin_here(src);
#pragma unroll
    for (int v = 0; v < NV4; ++v) {
      floatx16 &c = acc.c[(v / 4) / TN][(v / 4) % TN];
      const int q = (v % 4) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float *p = src + (size_t)(v * 4 + e) * NT + threadIdx.x;
        c[q + e] = *p;
        *p = 0.f;
      }
      if (v % 4 == 3) asm volatile("" ::: "memory");
    }
  }
};

}  // namespace sk
