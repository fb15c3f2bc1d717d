// M == 1 with fp16 weights in the NT layout: a matrix-vector product that streams W[N,K] from HBM
// once, in the order the memory pipeline coalesces.
//
// Same structure as the Q4 matrix-vector kernel (tile_gemv_q4.h): the four lanes of a quad read
// four consecutive 16-byte pieces of one weight row, a wave 16 rows; v_mfma_f32_4x4x4_16b_f16
// multiplies piece p of the weights with piece p of A inside each quad (the diagonal of the 4x4
// block result), and the quad is summed once at the end of the segment.  The K range of A that a
// segment needs is staged in LDS before the main loop, so the loop has no barrier.  Waves are
// WN x RK: RK is the reference's intra-CTA K split (streamk_fp16_block_reduce.py:45,235-306).
#pragma once
#include "sk_device.h"
#include "tile_skinny.h"

namespace sk {

// BF16_: the row of A, the weights, the bias and C are bfloat16 (v_mfma_f32_4x4x4_16b_bf16; C rounded to nearest even)
template <int NB_, int WN_, int RK_, int DEPTH_, int KMAX_ = 8192, bool BF16_ = false>
struct TileGemvF16 {
  typedef SkinnyArgs Args;
  static constexpr bool LEAN_ENTRY = false;  // see run_persistent
  static constexpr int NB = NB_, WN = WN_, RK = RK_, DEPTH = DEPTH_, KMAX = KMAX_;
  static constexpr int BM = 16, BN = 16 * NB * WN;
  static constexpr int LOADS = 4;          // 16-byte loads per lane, row block and iteration
  static constexpr int BK = 32 * LOADS;    // K per wave per iteration
  static constexpr int BKC = BK * RK;      // K per CTA iteration
  static constexpr int NT = WN * RK * 64;
  static constexpr int MAX_M = 1;
  static constexpr int MAX_ITERS = KMAX / BKC;
  static constexpr int LDS_A = KMAX * 2;
  static constexpr int LDS_RED = RK > 1 ? (RK - 1) * WN * NB * 64 * 4 : 0;
  static constexpr int LDS_BYTES = LDS_A + LDS_RED;
  static constexpr int TILE_ELEMS = BN;
  static constexpr int CTAS_PER_CU_WAVES = 12 / (NT / 64) > 0 ? 12 / (NT / 64) : 1;
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_BYTES + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_WAVES < CTAS_PER_CU_LDS ? CTAS_PER_CU_WAVES : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;
  static constexpr bool COHERENT_PARTIALS = true;

  // y[j]: result for weight row (wn*NB + j)*16 + lane/4 of the tile, valid in the lanes with
  // lane%4 == 0 of the rk == 0 waves
  struct Acc {
    float y[NB];
  };

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int /*pm*/, int pn, int k0, int n,
                                             char *smem) {
    char *ldsA = smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, rk = wave / WN;
    const int row = lane >> 2, piece = lane & 3;

    // ---- weights: lane (row, piece) reads K-values [32c + 8*piece, +8) of the wave's 128.  The
    // buffer ends with the last row of W the tile has, so rows past N read as zero ----
    const int rows_w = min(BN, a.N - pn * BN);
    const uint32_t ldw = (uint32_t)a.ldw * 2;  // bytes
    const BufferRsrc rsrc_w = make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * BN * ldw,
                                        (uint32_t)(rows_w - 1) * ldw + (uint32_t)a.K * 2);
    const int klane = rk * BK + piece * 8;
    uint32_t voff_w[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) voff_w[j] = (uint32_t)((wn * NB + j) * 16 + row) * ldw + (uint32_t)klane * 2;
    uint4v wreg[DEPTH][NB][LOADS];
    // loads of iterations past the segment or past K get an out-of-range offset: they return zero
    // weights without touching memory, and every round of the main loop has the same loads in flight
    auto issue_loads = [&](int slot, int rel_it) {
      const int kbase = (k0 + rel_it) * BKC;
      const int klimit = rel_it < n ? a.K - kbase : 0;
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int c = 0; c < LOADS; ++c)
          wreg[slot][j][c] = buffer_load_16(rsrc_w, klane + c * 32 < klimit ? voff_w[j] : OOB_OFFSET,
                                            (uint32_t)kbase * 2 + c * 64);
    };

    // ---- all global loads of the prologue go out back to back: A (first rounds of the CTA), then
    // DEPTH iterations of weights ----
    const BufferRsrc rsrc_a = make_rsrc(a.A, (uint32_t)a.K * 2);
    const int nchunk = n * (BKC / 8);
    constexpr int A_PRE = 2;
    uint4v a_pre[A_PRE];
#pragma unroll
    for (int t = 0; t < A_PRE; ++t) {
      const int b = t * NT + tid;
      a_pre[t] = buffer_load_16(rsrc_a, b < nchunk ? (uint32_t)(k0 * BKC + b * 8) * 2 : OOB_OFFSET, 0);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue_loads(d, d);
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int t = 0; t < A_PRE; ++t) {
      const int b = t * NT + tid;
      if (b < nchunk) *reinterpret_cast<uint4v *>(ldsA + b * 16) = a_pre[t];
    }
    for (int b = A_PRE * NT + tid; b < nchunk; b += NT)
      *reinterpret_cast<uint4v *>(ldsA + b * 16) = buffer_load_16(rsrc_a, (uint32_t)(k0 * BKC + b * 8) * 2, 0);
    __syncthreads();

    const char *a_rd = ldsA + klane * 2;
    floatx4 c_acc[NB][2];
#pragma unroll
    for (int j = 0; j < NB; ++j) c_acc[j][0] = c_acc[j][1] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- main loop: rounds of DEPTH iterations without an exit inside a round ----
    for (int it0 = 0; it0 < n; it0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int it = it0 + d;
        // an iteration past the segment multiplies zero weights with the A of the last iteration
        const int its = min(it, n - 1);
        uint4v fa[LOADS];
#pragma unroll
        for (int c = 0; c < LOADS; ++c) fa[c] = *reinterpret_cast<const uint4v *>(a_rd + its * (BKC * 2) + c * 64);
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int c = 0; c < LOADS; ++c) {
            union {
              uint32_t u[2];
              half4v v;
            } w0, w1, a0, a1;
            const uint4v w = wreg[d][j][c], f = fa[c];
            w0.u[0] = w[0], w0.u[1] = w[1], w1.u[0] = w[2], w1.u[1] = w[3];
            a0.u[0] = f[0], a0.u[1] = f[1], a1.u[0] = f[2], a1.u[1] = f[3];
            if constexpr (BF16_) {
              typedef short shortx4 __attribute__((ext_vector_type(4)));
              c_acc[j][0] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(shortx4, w0.v), __builtin_bit_cast(shortx4, a0.v),
                                                                   c_acc[j][0], 0, 0, 0);
              c_acc[j][1] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(shortx4, w1.v), __builtin_bit_cast(shortx4, a1.v),
                                                                   c_acc[j][1], 0, 0, 0);
            } else {
              c_acc[j][0] = __builtin_amdgcn_mfma_f32_4x4x4f16(w0.v, a0.v, c_acc[j][0], 0, 0, 0);
              c_acc[j][1] = __builtin_amdgcn_mfma_f32_4x4x4f16(w1.v, a1.v, c_acc[j][1], 0, 0, 0);
            }
          }
        issue_loads(d, it + DEPTH);
      }
    }

    // ---- register `piece` of each block result is this lane's term; add up the four pieces of
    // each row (the lanes of a quad), then the RK partial results into the rk == 0 waves.  Either
    // way the segment ends with a barrier: the next segment's prologue overwrites the LDS. ----
    const bool p1 = piece & 1, p2 = piece & 2;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const floatx4 s = c_acc[j][0] + c_acc[j][1];
      float y = p2 ? (p1 ? s[3] : s[2]) : (p1 ? s[1] : s[0]);
      y += __shfl_xor(y, 1);
      y += __shfl_xor(y, 2);
      acc.y[j] = y;
    }
    if (RK == 1) __syncthreads();
    if (RK > 1) {
      float *red = reinterpret_cast<float *>(smem + LDS_A);
      if (rk > 0) {
#pragma unroll
        for (int j = 0; j < NB; ++j) red[(((rk - 1) * WN + wn) * NB + j) * 64 + lane] = acc.y[j];
      }
      __syncthreads();
      if (rk == 0) {
#pragma unroll
        for (int r = 1; r < RK; ++r)
#pragma unroll
          for (int j = 0; j < NB; ++j) acc.y[j] += red[(((r - 1) * WN + wn) * NB + j) * 64 + lane];
      }
    }
  }

  // element e of the tile's partial vector: weight row e of the tile
  static __device__ __forceinline__ bool owns_output(int &first) {
    const int tid = threadIdx.x;
    first = (tid >> 6) * NB * 16 + ((tid & 63) >> 2);
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
    if (bias_ == nullptr) {  // the common case keeps the code it had before the epilogue operands existed
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = pn * BN + e + j * 16;
        if (col < a.N) a.C[col] = to_c(acc.y[j]);
      }
    } else {
      const half_t *bias = epi_bias(bias_);
      const int act = epi_act(bias_);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = pn * BN + e + j * 16;
        if (col < a.N) a.C[col] = to_c(activate(acc.y[j] + bias_at<BF16_>(bias, col, a.N), act));
      }
    }
  }
  static __device__ __forceinline__ void store_partial(const Acc &acc, float *dst) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int j = 0; j < NB; ++j) st_coherent(dst + e + j * 16, acc.y[j]);
  }
  static __device__ __forceinline__ void add_partial(Acc &acc, const float *src) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int j = 0; j < NB; ++j) acc.y[j] += ld_coherent_scalar(src + e + j * 16);
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int j = 0; j < NB; ++j) atomic_add_f32(dst + e + j * 16, acc.y[j]);
  }
  static __device__ __forceinline__ void take_partial(Acc &acc, float *src) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      acc.y[j] = ld_coherent_scalar(src + e + j * 16);
      st_coherent(src + e + j * 16, 0.f);
    }
  }
};

}  // namespace sk
