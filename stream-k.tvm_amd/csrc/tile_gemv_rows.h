// A few rows of A (2 <= M <= MR, MR = 4 in the instances built) with fp16 / bfloat16 weights in the NT layout: the
// matrix-vector kernel of tile_gemv_f16.h with MR rows of A per weight fragment.
//
// The weights are loaded exactly as there -- the four lanes of a quad read four consecutive 16-byte pieces of
// one weight row, a wave 16 rows, the order the memory pipeline coalesces -- and enter v_mfma_f32_4x4x4_16b_f16
// as they arrive: block b of the instruction (lanes 4b .. 4b+3) multiplies piece p of weight row b with piece p
// of one row of A (the diagonal of the 4x4 block result).  For MR rows of A the same weight registers are
// multiplied with MR fragments of A, one accumulator per row: 2 MR matrix instructions and MR 16-byte LDS reads
// per 16-byte load.  The LDS reads are what limits MR: all lanes of a wave fetch the same four pieces, but the
// LDS returns a full KB per read all the same, MR KB per KB of weights.  (The 16x16x32 MFMA of tile_skinny.h
// wants one weight row per lane, an order that streams 1.8 x slower, and a tile of A through LDS with a barrier
// in every iteration; it takes over from MR + 1 rows.)
//
// A lives in LDS for a window of KW K-values at a time (MR rows of KW halfs = 64 KB), staged by all threads
// between two barriers; inside a window the loop has no barrier and every wave streams its weight rows on its
// own.  Waves are WN x RK: RK is the reference's intra-CTA K split (streamk_fp16_block_reduce.py:45,235-306).
#pragma once
#include "sk_device.h"
#include "tile_skinny.h"

namespace sk {

template <int MR_, int WN_, int RK_, int DEPTH_, bool BF16_ = false>
struct TileGemvRows {
  typedef SkinnyArgs Args;
  static constexpr bool LEAN_ENTRY = false;  // see run_persistent
  static constexpr int MR = MR_, WN = WN_, RK = RK_, DEPTH = DEPTH_;
  static constexpr int BM = 16, BN = 16 * WN;
  static constexpr int LOADS = 4;          // 16-byte loads per lane and iteration
  static constexpr int BK = 32 * LOADS;    // K per wave per iteration
  static constexpr int BKC = BK * RK;      // K per CTA iteration
  static constexpr int NT = WN * RK * 64;
  static constexpr int MAX_M = MR;
  static constexpr int LDS_A = 64 * 1024;
  static constexpr int KW = LDS_A / (2 * MR);  // K-values of A resident at a time
  static constexpr int WIN_ITERS = KW / BKC;   // iterations per window
  static_assert(KW % BKC == 0 && WIN_ITERS % DEPTH == 0, "a window holds whole rounds of the load ring");
  static constexpr int LDS_RED = RK > 1 ? (RK - 1) * WN * 64 * 4 * MR : 0;
  static constexpr int LDS_BYTES = LDS_A + LDS_RED;
  static constexpr int TILE_ELEMS = MR * BN;
  static constexpr int CTAS_PER_CU_WAVES = 16 / (NT / 64) > 0 ? 16 / (NT / 64) : 1;
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_BYTES + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_WAVES < CTAS_PER_CU_LDS ? CTAS_PER_CU_WAVES : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;
  static constexpr bool COHERENT_PARTIALS = true;

  // y[m]: row m of A against weight row wn*16 + lane/4 of the tile, valid in the lanes with lane%4 == 0 of the
  // rk == 0 waves
  struct Acc {
    float y[MR];
  };

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int /*pm*/, int pn, int k0, int n,
                                             char *smem) {
    char *ldsA = smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, rk = wave / WN;
    const int row = lane >> 2, piece = lane & 3;

    // ---- weights: lane (row, piece) reads K-values [32c + 8*piece, +8) of the wave's 128.  The buffer ends with
    // the last row of W the tile has, so rows past N read as zero ----
    const int rows_w = min(BN, a.N - pn * BN);
    const uint32_t ldw = (uint32_t)a.ldw * 2;  // bytes
    const BufferRsrc rsrc_w = make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * BN * ldw,
                                        (uint32_t)(rows_w - 1) * ldw + (uint32_t)a.K * 2);
    const int klane = rk * BK + piece * 8;
    const uint32_t voff_w = (uint32_t)(wn * 16 + row) * ldw + (uint32_t)klane * 2;
    uint4v wreg[DEPTH][LOADS];
    // loads of iterations past the segment or past K get an out-of-range offset: they return zero weights
    // without touching memory, and every round of the main loop has the same loads in flight
    auto issue_loads = [&](int slot, int rel_it) {
      const int kbase = (k0 + rel_it) * BKC;
      const int klimit = rel_it < n ? a.K - kbase : 0;
#pragma unroll
      for (int c = 0; c < LOADS; ++c)
        wreg[slot][c] = buffer_load_16(rsrc_w, klane + c * 32 < klimit ? voff_w : OOB_OFFSET, (uint32_t)kbase * 2 + c * 64);
    };
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue_loads(d, d);

    // ---- A: rows past M and K-values past K read as zero (a zero fragment times a weight is zero) ----
    const int a_rows = min(a.M, MR);
    const BufferRsrc rsrc_a = make_rsrc(a.A, (uint32_t)(((int64_t)(a_rows - 1) * a.lda + a.K) * 2));
    floatx4 c_acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) c_acc[m] = floatx4{0.f, 0.f, 0.f, 0.f};
    const char *a_rd = ldsA + klane * 2;

    for (int w0 = 0; w0 < n; w0 += WIN_ITERS) {
      const int wn_iters = min(n - w0, WIN_ITERS);
      // stage the window: 16-byte chunk kc of row m to ldsA + (m * KW + 8 kc) * 2
      const int chunks_per_row = wn_iters * (BKC / 8);
      const int kwin = (k0 + w0) * BKC;
#pragma unroll 4
      for (int b = tid; b < MR * chunks_per_row; b += NT) {
        const int m = b / chunks_per_row, kc = b - m * chunks_per_row;
        const bool live = m < a_rows && kwin + kc * 8 < a.K;
        const uint4v v = buffer_load_16(rsrc_a, live ? (uint32_t)(m * a.lda + kwin + kc * 8) * 2 : OOB_OFFSET, 0);
        *reinterpret_cast<uint4v *>(ldsA + (m * KW + kc * 8) * 2) = v;
      }
      __syncthreads();

      // ---- the window's iterations: rounds of DEPTH without an exit inside a round ----
      for (int it0 = w0; it0 < w0 + wn_iters; it0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
          const int it = it0 + d;
          // an iteration past the segment multiplies zero weights with the A of the window's last iteration
          const int its = min(it, w0 + wn_iters - 1) - w0;
#pragma unroll
          for (int c = 0; c < LOADS; ++c) {
            union {
              uint32_t u[2];
              half4v v;
            } w_lo, w_hi;
            const uint4v w = wreg[d][c];
            w_lo.u[0] = w[0], w_lo.u[1] = w[1], w_hi.u[0] = w[2], w_hi.u[1] = w[3];
#pragma unroll
            for (int m = 0; m < MR; ++m) {
              union {
                uint32_t u[2];
                half4v v;
              } a_lo, a_hi;
              const uint4v f = *reinterpret_cast<const uint4v *>(a_rd + (m * KW + its * BKC) * 2 + c * 64);
              a_lo.u[0] = f[0], a_lo.u[1] = f[1], a_hi.u[0] = f[2], a_hi.u[1] = f[3];
              if constexpr (BF16_) {
                typedef short shortx4 __attribute__((ext_vector_type(4)));
                c_acc[m] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(shortx4, w_lo.v),
                                                                  __builtin_bit_cast(shortx4, a_lo.v), c_acc[m], 0, 0, 0);
                c_acc[m] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(shortx4, w_hi.v),
                                                                  __builtin_bit_cast(shortx4, a_hi.v), c_acc[m], 0, 0, 0);
              } else {
                c_acc[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(w_lo.v, a_lo.v, c_acc[m], 0, 0, 0);
                c_acc[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(w_hi.v, a_hi.v, c_acc[m], 0, 0, 0);
              }
            }
          }
          issue_loads(d, it + DEPTH);
        }
      }
      __syncthreads();  // the next window (or the next segment) overwrites A
    }

    // ---- register `piece` of each block result is this lane's term; add up the four pieces of each weight
    // row (the lanes of a quad), then the RK partial results into the rk == 0 waves ----
    const bool p1 = piece & 1, p2 = piece & 2;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const floatx4 s = c_acc[m];
      float y = p2 ? (p1 ? s[3] : s[2]) : (p1 ? s[1] : s[0]);
      y += __shfl_xor(y, 1);
      y += __shfl_xor(y, 2);
      acc.y[m] = y;
    }
    if (RK > 1) {
      float *red = reinterpret_cast<float *>(smem + LDS_A);
      if (rk > 0) {
#pragma unroll
        for (int m = 0; m < MR; ++m) red[(((rk - 1) * WN + wn) * MR + m) * 64 + lane] = acc.y[m];
      }
      __syncthreads();
      if (rk == 0) {
#pragma unroll
        for (int r = 1; r < RK; ++r)
#pragma unroll
          for (int m = 0; m < MR; ++m) acc.y[m] += red[(((r - 1) * WN + wn) * MR + m) * 64 + lane];
      }
      __syncthreads();  // the next segment's reduction reuses the area
    }
  }

  // this thread's column of the tile (one weight row), if it holds results at all
  static __device__ __forceinline__ bool owns_output(int &col) {
    const int tid = threadIdx.x;
    col = (tid >> 6) * 16 + ((tid & 63) >> 2);
    return tid < WN * 64 && (tid & 3) == 0;
  }

  // fp32 -> C's 16-bit pattern
  static __device__ __forceinline__ half_t to_c(float x) {
    if constexpr (BF16_) {
      const __bf16 b = (__bf16)x;
      return __builtin_bit_cast(half_t, b);
    } else {
      return (half_t)x;
    }
  }
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int /*pm*/, int pn, char *,
                                                 const void *bias_) {
    int e;
    if (!owns_output(e)) return;
    const int col = pn * BN + e;
    if (col >= a.N) return;
    float bv = 0.f;
    int act = 0;
    if (bias_ != nullptr) {
      bv = bias_at<BF16_>(epi_bias(bias_), col, a.N);
      act = epi_act(bias_);
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
      if (m < a.M) a.C[(int64_t)m * a.ldc + col] = to_c(bias_ != nullptr ? activate(acc.y[m] + bv, act) : acc.y[m]);
  }
  // element m * BN + e of the tile's partial: row m of A, weight row e of the tile
  static __device__ __forceinline__ void store_partial(const Acc &acc, float *dst) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int m = 0; m < MR; ++m) st_coherent(dst + m * BN + e, acc.y[m]);
  }
  static __device__ __forceinline__ void add_partial(Acc &acc, const float *src) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int m = 0; m < MR; ++m) acc.y[m] += ld_coherent_scalar(src + m * BN + e);
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int m = 0; m < MR; ++m) atomic_add_f32(dst + m * BN + e, acc.y[m]);
  }
  static __device__ __forceinline__ void take_partial(Acc &acc, float *src) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      acc.y[m] = ld_coherent_scalar(src + m * BN + e);
      st_coherent(src + m * BN + e, 0.f);
    }
  }
};

}  // namespace sk
