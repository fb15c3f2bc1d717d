// M == 1 with Q4 weights: a matrix-vector product whose only job is to stream the packed weights
// from HBM once while the instruction count per 32-bit word of weights stays small.
//
// CTA tile: BN = 16*NB*WN weight rows x BKC = RK*256 K-values per iteration; waves WN x RK as in
// the other small-M kernels (RK is the reference's intra-CTA K split, "block reduction",
// streamk_fp16_block_reduce.py:45,235-306).
//
// Differences from the general small-M kernel:
//  * the K range of A that a segment needs is staged in LDS once, before the main loop, so the
//    loop has no barrier: every wave streams its weight rows on its own;
//  * nibbles are not turned into finished fp16 weights.  OR-ing a nibble into the mantissa of
//    fp16 1024.0 (the decode trick of q4_dequant.h; the reference calls an external LOP3 decode at
//    streamk_fp16_ladder_block_reduce_q4.py:289-290) gives 1024 + q for the nibbles at bits 0..3 of
//    a 16-bit half and 1024 + 16 q for those at bits 4..7.  These go straight into the MFMA, the
//    low-position and the high-position nibbles into separate accumulators, over one scale group
//    (128 K-values, which is what one 16-byte load per lane of a wave covers):
//        c_lo = sum a_k (1024 + q_k)      k even
//        c_hi = sum a_k (1024 + 16 q_k)   k odd
//        sum a_k (q_k - zero) = c_lo + c_hi / 16 - [(1024 + zero) * sum_even a_k + (64 + zero) * sum_odd a_k]
//    The bracket depends on A and the group only; it is computed in fp32 while A is staged.  The
//    group's scale multiplies the fp32 group sum.  Per word of weights that leaves one shift and
//    four v_and_or_b32; per 16-byte load three more fp32 operations.  The products a_k * (1024 + q)
//    are exact in fp32 and the accumulation is fp32, so the result is at least as close to the
//    exact dot product as one computed from rounded fp16 weights.
//
// MFMA operand roles: D[m][n] = sum_k A[m][k] W[n][k] with v_mfma_f32_16x16x32_f16; all 16 rows m
// carry the same vector, so every register of the result holds y[n] for n = lane % 16 -- the
// lane's own weight row, whose scale the lane therefore applies without any exchange.
#pragma once
#include "q4_dequant.h"
#include "sk_device.h"
#include "tile_skinny.h"

namespace sk {

template <int NB_, int WN_, int RK_, int DEPTH_, int KMAX_ = 16384>
struct TileGemvQ4 {
  typedef SkinnyArgs Args;
  static constexpr int NB = NB_, WN = WN_, RK = RK_, DEPTH = DEPTH_, KMAX = KMAX_;
  static constexpr int BM = 16, BN = 16 * NB * WN;
  static constexpr int BK = 256;        // K per wave per iteration: two 16-byte loads per lane and block
  static constexpr int BKC = BK * RK;   // K per CTA iteration
  static constexpr int NT = WN * RK * 64;
  static constexpr int MAX_M = 1;
  static constexpr int QGROUP = 128;
  static constexpr int SC_PER_ITER = BKC / QGROUP;
  static constexpr int MAX_ITERS = KMAX / BKC;              // iterations one segment may span
  static constexpr int SC_ROW = KMAX / QGROUP + 8;          // halfs per LDS scale row
  static constexpr int LDS_A = KMAX * 2;
  static constexpr int LDS_CORR = KMAX / QGROUP * 4;
  static constexpr int LDS_SC = BN * SC_ROW * 2;
  static constexpr int LDS_RED = RK > 1 ? (RK - 1) * WN * NB * 64 * 4 : 0;
  static constexpr int LDS_BYTES = LDS_A + LDS_CORR + LDS_SC + LDS_RED;
  static constexpr int TILE_ELEMS = BN;
  static constexpr int CTAS_PER_CU_WAVES = 16 / (NT / 64);
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_BYTES + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_WAVES < CTAS_PER_CU_LDS ? CTAS_PER_CU_WAVES : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;
  static constexpr bool COHERENT_PARTIALS = true;

  // y[j]: result for weight row (wn*NB + j)*16 + lane%16 of the tile (valid in the rk == 0 waves)
  struct Acc {
    float y[NB];
  };

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int /*pm*/, int pn, int k0, int n,
                                             char *smem) {
    char *ldsA = smem;
    float *ldsCorr = reinterpret_cast<float *>(smem + LDS_A);
    half_t *ldsS = reinterpret_cast<half_t *>(smem + LDS_A + LDS_CORR);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, rk = wave / WN;
    const int lr = lane & 15, lg = lane >> 4;

#pragma unroll
    for (int j = 0; j < NB; ++j) acc.y[j] = 0.f;

    // ---- weights: lane (lr, lg) of a wave reads bytes [lg*16, lg*16+16) of each 64-byte piece of
    // row lr, i.e. K-values [lg*32, lg*32+32) of the piece's 128; rows past N read as zero ----
    const int rows_w = min(BN, a.N - pn * BN);
    const uint32_t ldw = (uint32_t)a.ldw;
    const BufferRsrc rsrc_w = make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * BN * ldw, rows_w * ldw);
    const int klane = rk * BK + lg * 32;
    uint32_t voff_w[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) voff_w[j] = (uint32_t)((wn * NB + j) * 16 + lr) * ldw + (uint32_t)(klane / 2);
    uint4v wreg[DEPTH][NB][2];
    // loads of iterations past the segment or past K get an out-of-range offset: they return
    // zeros without touching memory, and every round of the main loop has the same loads in flight
    auto issue_loads = [&](int slot, int rel_it) {
      const int kbase = (k0 + rel_it) * BKC;
      const int klimit = rel_it < n ? a.K - kbase : 0;
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int c = 0; c < 2; ++c)
          wreg[slot][j][c] =
              buffer_load_16(rsrc_w, klane + c * 128 < klimit ? voff_w[j] : OOB_OFFSET, (uint32_t)(kbase / 2) + c * 64);
    };
    __syncthreads();  // the previous segment's readers are done with the LDS
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue_loads(d, d);

    // ---- A: K-values [k0*BKC, (k0+n)*BKC) in blocks of 16.  Block b lands at byte 32 b as
    // [a0 a4 a2 a6 a8 a12 a10 a14 | a1 a5 a3 a7 a9 a13 a11 a15]: the even-k half multiplies the
    // nibbles at bits 0..3, the odd-k half those at bits 4..7 of two consecutive weight words.
    // Eight consecutive threads cover one scale group and reduce its two sums.
    {
      const BufferRsrc rsrc_a = make_rsrc(a.A, (uint32_t)a.K * 2);
      const int nblk = n * (BKC / 16);
      const float w_even = (float)(1024 + a.zero), w_odd = (float)(64 + a.zero);
      for (int b0 = 0; b0 < nblk; b0 += NT) {
        const int b = b0 + tid;
        const uint32_t off = (uint32_t)(k0 * BKC + b * 16) * 2;
        const uint4v v0 = buffer_load_16(rsrc_a, off, 0), v1 = buffer_load_16(rsrc_a, off, 16);
        uint4v even, odd;
        even[0] = __builtin_amdgcn_perm(v0[2], v0[0], 0x05040100u);
        even[1] = __builtin_amdgcn_perm(v0[3], v0[1], 0x05040100u);
        even[2] = __builtin_amdgcn_perm(v1[2], v1[0], 0x05040100u);
        even[3] = __builtin_amdgcn_perm(v1[3], v1[1], 0x05040100u);
        odd[0] = __builtin_amdgcn_perm(v0[2], v0[0], 0x07060302u);
        odd[1] = __builtin_amdgcn_perm(v0[3], v0[1], 0x07060302u);
        odd[2] = __builtin_amdgcn_perm(v1[2], v1[0], 0x07060302u);
        odd[3] = __builtin_amdgcn_perm(v1[3], v1[1], 0x07060302u);
        float se = 0.f, so = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // (bit-casting a vector element in place reads element 0: go through a scalar copy)
          const uint32_t ue = even[i], uo = odd[i];
          const half2v he = __builtin_bit_cast(half2v, ue), ho = __builtin_bit_cast(half2v, uo);
          se += (float)he[0] + (float)he[1];
          so += (float)ho[0] + (float)ho[1];
        }
        float corr = w_even * se + w_odd * so;
        corr += __shfl_xor(corr, 1);
        corr += __shfl_xor(corr, 2);
        corr += __shfl_xor(corr, 4);
        if (b < nblk) {
          *reinterpret_cast<uint4v *>(ldsA + b * 32) = even;
          *reinterpret_cast<uint4v *>(ldsA + b * 32 + 16) = odd;
          if ((tid & 7) == 0) ldsCorr[b >> 3] = corr;
        }
      }
    }
    // ---- scales of the segment, 16 bytes at a time: row r needs groups
    // [k0*SC_PER_ITER, (k0+n)*SC_PER_ITER); the copy starts at the 8-aligned group below and
    // ldsS[r][sc_shift + i] is group k0*SC_PER_ITER + i ----
    const int g_first = k0 * SC_PER_ITER, g0 = g_first & ~7;
    const int sc_shift = g_first - g0;
    stage_scales<BN, SC_ROW, NT>(ldsS, a.scales + (int64_t)pn * BN * a.groups, rows_w, a.groups, g0,
                                 (sc_shift + n * SC_PER_ITER + 7) >> 3);
    __syncthreads();

    Q4Consts qc;
    q4_pin_patterns(qc);
    const uint32_t magic = qc.magic, mlo = qc.mask_lo, mhi = qc.mask_hi;
    const char *a_rd = ldsA + klane * 2;
    const half_t *s_rd[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) s_rd[j] = ldsS + ((wn * NB + j) * 16 + lr) * SC_ROW + sc_shift + rk * 2;
    const float *c_rd = ldsCorr + rk * 2;

    // ---- main loop: rounds of DEPTH iterations without an exit inside a round ----
    for (int it0 = 0; it0 < n; it0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int it = it0 + d;
        // an iteration past the segment decodes zero nibbles, which are not zero weights: its
        // group sums are discarded by a zero scale
        const int its = min(it, n - 1);
        const float live = it < n ? 1.f : 0.f;
        const float corr0 = c_rd[its * SC_PER_ITER], corr1 = c_rd[its * SC_PER_ITER + 1];
        half8v fa[2][4];  // [load c][even01, odd01, even23, odd23]
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            fa[c][q] = *reinterpret_cast<const half8v *>(a_rd + its * (BKC * 2) + c * 256 + q * 16);
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const half2v s2 = *reinterpret_cast<const half2v *>(s_rd[j] + its * SC_PER_ITER);
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const uint4v w = wreg[d][j][c];
            union {
              uint32_t u[4];
              half8v v;
            } e01, o01, e23, o23;
            const uint32_t t0 = w[0] >> 8, t1 = w[1] >> 8, t2 = w[2] >> 8, t3 = w[3] >> 8;
            e01.u[0] = and_or(w[0], mlo, magic);
            e01.u[1] = and_or(t0, mlo, magic);
            e01.u[2] = and_or(w[1], mlo, magic);
            e01.u[3] = and_or(t1, mlo, magic);
            o01.u[0] = and_or(w[0], mhi, magic);
            o01.u[1] = and_or(t0, mhi, magic);
            o01.u[2] = and_or(w[1], mhi, magic);
            o01.u[3] = and_or(t1, mhi, magic);
            e23.u[0] = and_or(w[2], mlo, magic);
            e23.u[1] = and_or(t2, mlo, magic);
            e23.u[2] = and_or(w[3], mlo, magic);
            e23.u[3] = and_or(t3, mlo, magic);
            o23.u[0] = and_or(w[2], mhi, magic);
            o23.u[1] = and_or(t2, mhi, magic);
            o23.u[2] = and_or(w[3], mhi, magic);
            o23.u[3] = and_or(t3, mhi, magic);
            const floatx4 zero4 = floatx4{0.f, 0.f, 0.f, 0.f};
            floatx4 ce = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[c][0], e01.v, zero4, 0, 0, 0);
            floatx4 co = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[c][1], o01.v, zero4, 0, 0, 0);
            ce = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[c][2], e23.v, ce, 0, 0, 0);
            co = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[c][3], o23.v, co, 0, 0, 0);
            const float group_sum = __builtin_fmaf(co[0], 0.0625f, ce[0]) - (c == 0 ? corr0 : corr1);
            acc.y[j] = __builtin_fmaf(group_sum, (float)s2[c] * live, acc.y[j]);
          }
        }
        issue_loads(d, it + DEPTH);
      }
    }

    // ---- sum the RK partial results into the rk == 0 waves ----
    if (RK > 1) {
      float *red = reinterpret_cast<float *>(smem + LDS_A + LDS_CORR + LDS_SC);
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
    first = (tid >> 6) * NB * 16 + (tid & 15);
    return tid < WN * 64 && (tid & 63) < 16;
  }

  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int /*pm*/, int pn, char *) {
    int e;
    if (!owns_output(e)) return;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int col = pn * BN + e + j * 16;
      if (col < a.N) a.C[col] = (half_t)acc.y[j];
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
