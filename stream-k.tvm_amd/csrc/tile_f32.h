// fp32 tile arithmetic: BM x BN x 16 CTA tile (128 x 128 on 2 x 2 waves; 32 x 256 on 1 x 4 waves for small M),
// v_mfma_f32_32x32x2_f32.
//
// Replaces the T.gemm of the reference's fp32 kernel (streamk_fp32.py:109-125).  B may be [K,N]
// (the reference's layout, streamk_fp32.py:74) or [N,K].
//
// One MFMA multiplies a 32 x 2 slice: lane (r = lane%32, g = lane/32) supplies A[r][k_g].  A lane
// reads four consecutive K of its row in one 16-byte LDS access and feeds them to four MFMAs, so
// MFMA e of an 8-wide K step contracts K = {e, 4 + e}; the B operand follows the same rule.
#pragma once
#include "sk_device.h"

namespace sk {

struct GemmArgsF32 {
  const float *A;
  const float *B;
  float *C;
  int M, N, K;
  int64_t lda, ldb, ldc;
};

template <bool B_KN_, int BM_ = 128, int BN_ = 128, int WM_ = 2, int WN_ = 2>
struct TileF32 {
  typedef GemmArgsF32 Args;
  static constexpr bool LEAN_ENTRY = true;  // see run_persistent
  static constexpr bool B_KN = B_KN_;
  static constexpr int BM = BM_, BN = BN_, BK = 16, WM = WM_, WN = WN_;
  static constexpr int NT = 256, TM = BM / (WM * 32), TN = BN / (WN * 32), WTM = TM * 32, WTN = TN * 32;
  static_assert(WM * WN == 4 && BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BN % 64 == 0, "tile shape");
  static constexpr int LDA = BK + 4;                 // floats per LDS row of A (and of B when [N,K])
  static constexpr int LDB = B_KN ? BN + 8 : BK + 4; // floats per LDS row of B
  static constexpr int A_STAGE = BM * LDA, B_STAGE = B_KN ? BK * LDB : BN * LDB, STAGE = A_STAGE + B_STAGE;
  static constexpr int LDS_BYTES = 2 * STAGE * 4, LDS_TOTAL = LDS_BYTES;
  static constexpr int TILE_ELEMS = BM * BN, NV4 = TM * TN * 4;
  static constexpr int CTAS_PER_CU = 2, WAVES_PER_EU = 2;
  static constexpr bool COHERENT_PARTIALS = false;
  // 16-byte loads per thread: a pass of the 256 threads covers 64 rows of 16 K-values (A, and B as
  // [N,K]) or 1024 / BN K-rows of BN values (B as [K,N])
  static constexpr int A_LOADS = (BM + 63) / 64, B_LOADS = BN * BK / 4 / NT;
  static constexpr int B_CPR = BN / 4, B_RPP = NT / B_CPR;  // [K,N]: chunks per K-row, K-rows per pass

  struct Acc {
    floatx16 c[TM][TN];
  };

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n, char *smem) {
    float *lds = reinterpret_cast<float *>(smem);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc.c[i][j][r] = 0.f;

    // ---- global addressing (buffer descriptors: rows past the matrix read as zero) ----
    const int rows_a = min(BM, a.M - pm * BM), cols_b = min(BN, a.N - pn * BN);
    const BufferRsrc rsrc_a = make_rsrc(a.A + (int64_t)pm * BM * a.lda, (uint32_t)(rows_a * a.lda * 4));
    const int a_row = tid / 4, a_c = tid % 4;  // 4 chunks of 4 floats per K-row of 16
    const uint32_t voff_a = (BM % 64 == 0 || a_row < BM) ? (uint32_t)(a_row * a.lda + a_c * 4) * 4 : OOB_OFFSET;
    const uint32_t pass_a = (uint32_t)(64 * a.lda * 4);
    BufferRsrc rsrc_b;
    uint32_t voff_b, pass_b, kstep_b;
    int b_st;  // LDS float offset of this thread's first B chunk
    if (!B_KN) {
      rsrc_b = make_rsrc(a.B + (int64_t)pn * BN * a.ldb, (uint32_t)(cols_b * a.ldb * 4));
      voff_b = (uint32_t)(a_row * a.ldb + a_c * 4) * 4;
      pass_b = (uint32_t)(64 * a.ldb * 4);
      kstep_b = BK * 4;
      b_st = a_row * LDB + a_c * 4;
    } else {
      rsrc_b = make_rsrc(a.B + (int64_t)pn * BN, (uint32_t)(((int64_t)(a.K - 1) * a.ldb + cols_b) * 4));
      const int k_row = tid / B_CPR, c = tid % B_CPR;
      voff_b = (c * 4 < cols_b) ? (uint32_t)(k_row * a.ldb + c * 4) * 4 : OOB_OFFSET;
      pass_b = (uint32_t)(B_RPP * a.ldb * 4);
      kstep_b = (uint32_t)(BK * a.ldb * 4);
      b_st = k_row * LDB + c * 4;
    }
    const int a_st = a_row * LDA + a_c * 4;
    const int tail_kt = (a.K % BK != 0) ? (a.K / BK) : -1;

    uint4v ra[A_LOADS], rb[B_LOADS];
    auto load_global = [&](int kt) {
      uint32_t va = voff_a, vb = voff_b;
      if (kt == tail_kt && kt * BK + a_c * 4 >= a.K) {
        va = OOB_OFFSET;
        if (!B_KN) vb = OOB_OFFSET;
      }
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) ra[i] = buffer_load_16(rsrc_a, va, (uint32_t)kt * (BK * 4) + i * pass_a);
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i) rb[i] = buffer_load_16(rsrc_b, vb, (uint32_t)kt * kstep_b + i * pass_b);
    };

    const int a_rd = (wm * WTM + (lane & 31)) * LDA + (lane >> 5) * 4;
    const int b_rd = B_KN ? A_STAGE + (lane >> 5) * 4 * LDB + wn * WTN + (lane & 31)
                          : A_STAGE + (wn * WTN + (lane & 31)) * LDB + (lane >> 5) * 4;

    load_global(k0);
    for (int it = 0; it < n; ++it) {
      float *st = lds + (it & 1) * STAGE;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i)
        if (BM % 64 == 0 || a_row + i * 64 < BM) *reinterpret_cast<uint4v *>(st + a_st + i * 64 * LDA) = ra[i];
#pragma unroll
      for (int i = 0; i < B_LOADS; ++i)
        *reinterpret_cast<uint4v *>(st + A_STAGE + b_st + i * (B_KN ? B_RPP * LDB : 64 * LDB)) = rb[i];
      __syncthreads();
      if (it + 1 < n) load_global(k0 + it + 1);
#pragma unroll
      for (int kk = 0; kk < BK / 8; ++kk) {
        floatx4 fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const floatx4 *>(st + a_rd + i * 32 * LDA + kk * 8);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if (!B_KN) {
            fb[j] = *reinterpret_cast<const floatx4 *>(st + b_rd + j * 32 * LDB + kk * 8);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) fb[j][e] = st[b_rd + (kk * 8 + e) * LDB + j * 32];
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc.c[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][e], fb[j][e], acc.c[i][j], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // acc.c[i][j][r] = C[pm*BM + wm*WTM + i*32 + 8*(r/4) + 4*(lane/32) + r%4][pn*BN + wn*WTN + j*32 + lane%32]
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int pm, int pn, char *,
                                                 const void * /*bias: not offered for fp32*/) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = pn * BN + wn * WTN + j * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = pm * BM + wm * WTM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
          if (row < a.M && col < a.N) a.C[(int64_t)row * a.ldc + col] = acc.c[i][j][r];
        }
      }
  }

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
    }
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst) {
    dst = pin_here(dst);
#pragma unroll
    for (int v = 0; v < NV4; ++v) {
      floatx4 x = grp(acc, v);
#pragma unroll
      for (int e = 0; e < 4; ++e) atomic_add_f32(dst + (size_t)(v * 4 + e) * NT + threadIdx.x, x[e]);
    }
  }
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
    }
  }
};

}  // namespace sk
