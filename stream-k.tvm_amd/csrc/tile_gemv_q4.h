// M == 1 with Q4 weights: a matrix-vector product whose only job is to stream the packed weights
// from HBM once while the instruction count per 32-bit word of weights stays small.
//
// CTA tile: BN = 16*NB*WN weight rows x BKC = RK*256 K-values per iteration; waves WN x RK as in
// the other small-M kernels (RK is the reference's intra-CTA K split, "block reduction",
// streamk_fp16_block_reduce.py:45,235-306).
//
// Differences from the general small-M kernel:
//  * Loads are issued in the order the memory pipeline coalesces: the four lanes of a quad read
//    the four 16-byte pieces of one 64-byte run (one scale group of one weight row), a wave 16
//    rows.  (With one row per lane, the 16x16 MFMA's own layout, the same bytes stream 1.8x
//    slower.)  The arithmetic uses the layout as it is: v_mfma_f32_4x4x4_16b_f16 computes sixteen
//    independent 4x4x4 products, block b from lanes 4b..4b+3.  Lane (b, p) supplies row p of the
//    block's first operand -- piece p of weight row b, four K-values at a time -- and column p of
//    the second -- the same K-values of A.  D_b[i][j] pairs piece i of the weights with piece j
//    of A; the lane keeps the diagonal term j = i = p (register p of its result) and the quad is
//    summed once, when the segment ends.
//  * The K range of A that a segment needs is staged in LDS once, before the main loop, so the
//    loop has no barrier: every wave streams its weight rows on its own.
//  * Nibbles are not turned into finished fp16 weights.  OR-ing a nibble into the mantissa of
//    fp16 1024.0 (the decode trick of q4_dequant.h; the reference calls an external LOP3 decode at
//    streamk_fp16_ladder_block_reduce_q4.py:289-290) gives 1024 + q for the nibbles at bits 0..3 of
//    a 16-bit half and 1024 + 16 q for those at bits 4..7.  These go straight into the MFMA, the
//    low-position and the high-position nibbles into separate accumulators, over the 32 K-values
//    of one 16-byte load:
//        c_lo = sum a_k (1024 + q_k)      k even
//        c_hi = sum a_k (1024 + 16 q_k)   k odd
//        sum a_k (q_k - zero) = c_lo + c_hi / 16 - [(1024 + zero) * sum_even a_k + (64 + zero) * sum_odd a_k]
//    The bracket depends on A only; it is computed in fp32, per 32 K-values, while A is staged.
//    The group's scale multiplies the fp32 sum.  Per word of weights that leaves one shift and
//    four v_and_or_b32; per 16-byte load nine more fp32 operations.  The products a_k * (1024 + q)
//    are exact in fp32 and the accumulation is fp32, so the result is at least as close to the
//    exact dot product as one computed from rounded fp16 weights.
#pragma once
#include "q4_dequant.h"
#include "sk_device.h"
#include "tile_skinny.h"

namespace sk {

//
// TILED_: the weights come in 16-row x 64-byte tiles (see tile_skinny.h); the lane order of the
// loads, row = lane/4, piece = lane%4, is then the byte order of a tile: one contiguous KB per load.
//
// ZP_: one zero point per scale group and row (a.zeros, the shape of the scales; a.zero is ignored).  The
// bracket above splits into a part that depends on A only and one that is linear in the zero point:
//     sum a_k (q_k - z) = c_lo + c_hi / 16 - [1024 sum_even a_k + 64 sum_odd a_k] - z [sum_even a_k + sum_odd a_k]
// Both sums of A are kept per 32 K-values; the zero points are staged in LDS beside the scales.  (Scales and
// zero points are row-major [N, groups] also where the weights are tiled.)
template <int NB_, int WN_, int RK_, int DEPTH_, int KMAX_ = 16384, bool TILED_ = false, bool ZP_ = false>
struct TileGemvQ4 {
  // data-parallel launches give each XCD a contiguous eighth of the row blocks (skinny_launch.h): N = K = 8192 with
  // the weights in the Infinity Cache 6.08-6.14 -> 5.81 us, from HBM 8.6-8.8 -> 8.55 us; other shapes unchanged
  static constexpr bool XCD_CONTIGUOUS = true;
  typedef SkinnyArgs Args;
  static constexpr bool LEAN_ENTRY = false;  // see run_persistent
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
  static constexpr int LDS_CORR1 = KMAX / 32 * 4;           // one correction per 32 K-values
  static constexpr int LDS_CORR = ZP_ ? 2 * LDS_CORR1 : LDS_CORR1;  // ZP_: then the plain sums of A
  static constexpr int LDS_SC1 = BN * SC_ROW * 2;
  static constexpr int LDS_SC = ZP_ ? 2 * LDS_SC1 : LDS_SC1;        // scales, then zero points
  static constexpr int LDS_RED = RK > 1 ? (RK - 1) * WN * NB * 64 * 4 : 0;
  static constexpr int LDS_BYTES = LDS_A + LDS_CORR + LDS_SC + LDS_RED;
  static constexpr int TILE_ELEMS = BN;
  // at most three waves per SIMD: the loop wants ~140 VGPRs
  static constexpr int CTAS_PER_CU_WAVES = 12 / (NT / 64);
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_BYTES + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_WAVES < CTAS_PER_CU_LDS ? CTAS_PER_CU_WAVES : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;
  static constexpr bool COHERENT_PARTIALS = true;

  // y[j]: result for weight row (wn*NB + j)*16 + lane/4 of the tile, valid in the lanes with
  // lane%4 == 0 of the rk == 0 waves
  struct Acc {
    float y[NB];
  };

  // What one tile leaves in registers for the next tile of the same CTA: the weights of the next tile's first DEPTH
  // iterations and the first pieces of its scales (and zero points), requested during the last round of the tile
  // before, so that the memory round trip of a tile's start overlaps the end of the one before.
  struct Carry {
    uint4v wreg[DEPTH][NB][2];
    ScaleStager<BN, SC_ROW, NT> scales, zero_points;
  };

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n, char *smem) {
    Carry cy;
    mac_impl<false, false, false>(a, acc, pm, pn, k0, n, smem, cy, -1);
  }
  // The same for a CTA whose previous call had the same k0 and n (the tiles of a data-parallel launch that a CTA
  // takes one after the other): the row of A and its correction sums are in LDS already and are neither loaded
  // nor staged again -- a fifth of a tile's time at K = 8192.
  static __device__ __forceinline__ void mac_again(const Args &a, Acc &acc, int pm, int pn, int k0, int n, char *smem) {
    Carry cy;
    mac_impl<true, false, false>(a, acc, pm, pn, k0, n, smem, cy, -1);
  }
  // All tiles of a CTA in a data-parallel launch (tile0, tile0 + stride, ... below total), K from 0 over ipt
  // iterations each, C stored as store_c does: every tile but the first finds its first loads in flight.
  static __device__ __forceinline__ void mac_tiles(const Args &a, int tile0, int stride, int total, int ipt, char *smem,
                                                   const void *bias) {
    if (tile0 >= total) return;
    Carry cy;
    Acc acc;
    int next = tile0 + stride < total ? tile0 + stride : -1;
    mac_impl<false, false, true>(a, acc, 0, tile0, 0, ipt, smem, cy, next);
    store_c(a, acc, 0, tile0, smem, bias);
    while (next >= 0) {
      const int tile = next;
      next = tile + stride < total ? tile + stride : -1;
      mac_impl<true, true, true>(a, acc, 0, tile, 0, ipt, smem, cy, next);
      store_c(a, acc, 0, tile, smem, bias);
    }
  }
  // PRELOADED: cy holds this tile's first DEPTH iterations of weights and the first pieces of its scales (the
  // previous call was given this tile as next_pn, same k0 and n).  CHAIN with next_pn >= 0: the last round requests
  // those of tile next_pn instead of reading past the segment.
  template <bool A_RESIDENT, bool PRELOADED, bool CHAIN>
  static __device__ __forceinline__ void mac_impl(const Args &a, Acc &acc, int /*pm*/, int pn, int k0, int n,
                                                  char *smem, Carry &cy, int next_pn) {
    char *ldsA = smem;
    float *ldsCorr = reinterpret_cast<float *>(smem + LDS_A);
    half_t *ldsS = reinterpret_cast<half_t *>(smem + LDS_A + LDS_CORR);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, rk = wave / WN;
    const int row = lane >> 2, piece = lane & 3;

#pragma unroll
    for (int j = 0; j < NB; ++j) acc.y[j] = 0.f;

    // ---- weights: lane (row, piece) reads K-values [piece*32, piece*32+32) of each 128-wide
    // group of its row; rows past N read as zero ----
    const int rows_w = min(BN, a.N - pn * BN);
    const uint32_t ldw = (uint32_t)a.ldw;
    const uint32_t block_bytes = (uint32_t)a.groups * 1024;  // tiled: one 16-row block of W
    const BufferRsrc rsrc_w =
        TILED_ ? make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * (BN / 16) * block_bytes,
                           (uint32_t)((rows_w + 15) / 16) * block_bytes)
               : make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * BN * ldw, rows_w * ldw);
    const int klane = rk * BK + piece * 32;
    uint32_t voff_w[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j)
      voff_w[j] = TILED_ ? (uint32_t)(wn * NB + j) * block_bytes + (uint32_t)lane * 16
                         : (uint32_t)((wn * NB + j) * 16 + row) * ldw + (uint32_t)(klane / 2);
    auto &wreg = cy.wreg;
    // the next tile's rows (an empty range without one: its loads return zeros without touching memory)
    const int rows_next = next_pn >= 0 ? min(BN, a.N - next_pn * BN) : 0;
    const char *base_cur = reinterpret_cast<const char *>(a.W) + (int64_t)pn * (TILED_ ? (BN / 16) * block_bytes : BN * ldw);
    const char *base_next =
        reinterpret_cast<const char *>(a.W) + (int64_t)max(next_pn, 0) * (TILED_ ? (BN / 16) * block_bytes : BN * ldw);
    const uint32_t bytes_cur = TILED_ ? (uint32_t)((rows_w + 15) / 16) * block_bytes : rows_w * ldw;
    const uint32_t bytes_next = TILED_ ? (uint32_t)((rows_next + 15) / 16) * block_bytes : rows_next * ldw;
    // loads of iterations past the segment or past K get an out-of-range offset: they return
    // zeros without touching memory, and every round of the main loop has the same loads in flight
    auto issue_from = [&](const BufferRsrc &rsrc, int slot, int rel_it) {
      const int kbase = (k0 + rel_it) * BKC;
      const int klimit = rel_it < n ? a.K - kbase : 0;
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int c = 0; c < 2; ++c)
          wreg[slot][j][c] =
              TILED_ ? buffer_load_16(rsrc, rk * BK + c * 128 < klimit ? voff_w[j] : OOB_OFFSET,
                                      (uint32_t)((kbase + rk * BK) / QGROUP + c) * 1024)
                     : buffer_load_16(rsrc, klane + c * 128 < klimit ? voff_w[j] : OOB_OFFSET,
                                      (uint32_t)(kbase / 2) + c * 64);
    };
    auto issue_loads = [&](int slot, int rel_it) { issue_from(rsrc_w, slot, rel_it); };

    // ---- all global loads of the prologue go out back to back, in the order they are consumed:
    // A (first two rounds of the CTA), the first round of scale pieces, then DEPTH iterations of
    // weights.  One memory round trip covers all of them.
    // A: K-values [k0*BKC, (k0+n)*BKC) in blocks of 16, two 16-byte units per block.  The unit of
    // K-values 8u..8u+7 lands at byte 16 u as [a0 a4 a2 a6 | a1 a5 a3 a7]: the even-k half multiplies
    // the nibbles at bits 0..3, the odd-k half those at bits 4..7 of one weight word.  Two
    // consecutive threads cover 32 K-values and add up their correction.
    const BufferRsrc rsrc_a = make_rsrc(a.A, (uint32_t)a.K * 2);
    const int nblk = n * (BKC / 16);
    constexpr int A_PRE = 2;
    uint4v a_lo[A_PRE], a_hi[A_PRE];
    if constexpr (!A_RESIDENT) {
#pragma unroll
      for (int t = 0; t < A_PRE; ++t) {
        const int b = t * NT + tid;
        const uint32_t off = b < nblk ? (uint32_t)(k0 * BKC + b * 16) * 2 : OOB_OFFSET;
        a_lo[t] = buffer_load_16(rsrc_a, off, 0);
        a_hi[t] = buffer_load_16(rsrc_a, off, 16);
      }
    }
    // scales: row r needs groups [k0*SC_PER_ITER, (k0+n)*SC_PER_ITER); the copy starts at the
    // 8-aligned group below and ldsS[r][sc_shift + i] is group k0*SC_PER_ITER + i
    const int g_first = k0 * SC_PER_ITER, g0 = g_first & ~7;
    const int sc_shift = g_first - g0;
    auto &scales = cy.scales;
    auto &zero_points = cy.zero_points;
    const int sc_chunks = (sc_shift + n * SC_PER_ITER + 7) >> 3;
    if constexpr (!PRELOADED) {
      scales.begin(ldsS, a.scales + (int64_t)pn * BN * a.groups, rows_w, a.groups, g0, sc_chunks);
      if constexpr (ZP_)
        zero_points.begin(ldsS + BN * SC_ROW, a.zeros + (int64_t)pn * BN * a.groups, rows_w, a.groups, g0, sc_chunks);
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) issue_loads(d, d);
    }
    // nothing of what follows is to be scheduled ahead of these loads
    __builtin_amdgcn_sched_barrier(0);

    const float w_even = (float)(1024 + (ZP_ ? 0 : a.zero)), w_odd = (float)(64 + (ZP_ ? 0 : a.zero));
    float *ldsSumA = ldsCorr + KMAX / 32;  // ZP_: sum of the 32 K-values of A, beside their correction
    auto stage_a_block = [&](int b, uint4v v0, uint4v v1) {
      uint4v u0, u1;  // [even | odd] of K-values 0..7 and 8..15 of the block
      u0[0] = __builtin_amdgcn_perm(v0[2], v0[0], 0x05040100u);
      u0[1] = __builtin_amdgcn_perm(v0[3], v0[1], 0x05040100u);
      u0[2] = __builtin_amdgcn_perm(v0[2], v0[0], 0x07060302u);
      u0[3] = __builtin_amdgcn_perm(v0[3], v0[1], 0x07060302u);
      u1[0] = __builtin_amdgcn_perm(v1[2], v1[0], 0x05040100u);
      u1[1] = __builtin_amdgcn_perm(v1[3], v1[1], 0x05040100u);
      u1[2] = __builtin_amdgcn_perm(v1[2], v1[0], 0x07060302u);
      u1[3] = __builtin_amdgcn_perm(v1[3], v1[1], 0x07060302u);
      float se = 0.f, so = 0.f;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        // (bit-casting a vector element in place reads element 0: go through scalar copies)
        const uint32_t e0 = u0[i], e1 = u1[i], o0 = u0[2 + i], o1 = u1[2 + i];
        const half2v he0 = __builtin_bit_cast(half2v, e0), he1 = __builtin_bit_cast(half2v, e1);
        const half2v ho0 = __builtin_bit_cast(half2v, o0), ho1 = __builtin_bit_cast(half2v, o1);
        se += ((float)he0[0] + (float)he0[1]) + ((float)he1[0] + (float)he1[1]);
        so += ((float)ho0[0] + (float)ho0[1]) + ((float)ho1[0] + (float)ho1[1]);
      }
      float corr = w_even * se + w_odd * so;
      corr += __shfl_xor(corr, 1);
      float sum_a = se + so;
      if constexpr (ZP_) sum_a += __shfl_xor(sum_a, 1);
      if (b < nblk) {
        *reinterpret_cast<uint4v *>(ldsA + b * 32) = u0;
        *reinterpret_cast<uint4v *>(ldsA + b * 32 + 16) = u1;
        if ((tid & 1) == 0) {
          ldsCorr[b >> 1] = corr;
          if constexpr (ZP_) ldsSumA[b >> 1] = sum_a;
        }
      }
    };
    if constexpr (!A_RESIDENT) {
#pragma unroll
      for (int t = 0; t < A_PRE; ++t)
        if (t * NT < nblk) stage_a_block(t * NT + tid, a_lo[t], a_hi[t]);
      for (int b0 = A_PRE * NT; b0 < nblk; b0 += NT) {
        const uint32_t off = (uint32_t)(k0 * BKC + (b0 + tid) * 16) * 2;
        stage_a_block(b0 + tid, buffer_load_16(rsrc_a, off, 0), buffer_load_16(rsrc_a, off, 16));
      }
    }
    scales.finish();
    if constexpr (ZP_) zero_points.finish();
    __syncthreads();

    Q4Consts qc;
    q4_pin_patterns(qc);
    const uint32_t magic = qc.magic, mlo = qc.mask_lo, mhi = qc.mask_hi;
    const char *a_rd = ldsA + klane * 2;
    const half_t *s_rd[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) s_rd[j] = ldsS + ((wn * NB + j) * 16 + row) * SC_ROW + sc_shift + rk * 2;
    const float *c_rd = ldsCorr + rk * 8 + piece;
    const bool p1 = piece & 1, p2 = piece & 2;

    // ---- main loop: rounds of DEPTH iterations without an exit inside a round ----
    for (int it0 = 0; it0 < n; it0 += DEPTH) {
      // the last round asks for the next tile's start instead of iterations past the segment: its scales first,
      // then slot by slot the weights of its iterations 0 .. DEPTH-1
      const bool last_round = CHAIN && it0 + DEPTH >= n;
      // (one descriptor per round, chosen with scalar selects: the loop body has a single path)
      const BufferRsrc rsrc_it = CHAIN ? make_rsrc(last_round ? base_next : base_cur, last_round ? bytes_next : bytes_cur) : rsrc_w;
      if (last_round && next_pn >= 0) {
        scales.begin(ldsS, a.scales + (int64_t)next_pn * BN * a.groups, rows_next, a.groups, g0, sc_chunks);
        if constexpr (ZP_)
          zero_points.begin(ldsS + BN * SC_ROW, a.zeros + (int64_t)next_pn * BN * a.groups, rows_next, a.groups, g0,
                            sc_chunks);
      }
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int it = it0 + d;
        // an iteration past the segment decodes zero nibbles, which are not zero weights: its
        // sums are discarded by a zero scale
        const int its = min(it, n - 1);
        const float live = it < n ? 1.f : 0.f;
        const float corr0 = c_rd[its * (BKC / 32)], corr1 = c_rd[its * (BKC / 32) + 4];
        float suma0 = 0.f, suma1 = 0.f;
        if constexpr (ZP_) {
          suma0 = c_rd[KMAX / 32 + its * (BKC / 32)];
          suma1 = c_rd[KMAX / 32 + its * (BKC / 32) + 4];
        }
        uint4v fa[2][4];  // [load c][word]: {even half, odd half} of the word's eight K-values of A
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            fa[c][q] = *reinterpret_cast<const uint4v *>(a_rd + its * (BKC * 2) + c * 256 + q * 16);
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const half2v s2 = *reinterpret_cast<const half2v *>(s_rd[j] + its * SC_PER_ITER);
          half2v z2 = {(half_t)0.f, (half_t)0.f};
          if constexpr (ZP_) z2 = *reinterpret_cast<const half2v *>(s_rd[j] + BN * SC_ROW + its * SC_PER_ITER);
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const uint4v w = wreg[d][j][c];
            floatx4 ce = floatx4{0.f, 0.f, 0.f, 0.f}, co = ce;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              union {
                uint32_t u[2];
                half4v v;
              } we, wo, ae, ao;
              const uint32_t wq = w[q], t = wq >> 8;
              we.u[0] = and_or(wq, mlo, magic);
              we.u[1] = and_or(t, mlo, magic);
              wo.u[0] = and_or(wq, mhi, magic);
              wo.u[1] = and_or(t, mhi, magic);
              const uint4v f = fa[c][q];
              ae.u[0] = f[0];
              ae.u[1] = f[1];
              ao.u[0] = f[2];
              ao.u[1] = f[3];
              ce = __builtin_amdgcn_mfma_f32_4x4x4f16(we.v, ae.v, ce, 0, 0, 0);
              co = __builtin_amdgcn_mfma_f32_4x4x4f16(wo.v, ao.v, co, 0, 0, 0);
            }
            // register `piece` of each result is this lane's term
            const float se = p2 ? (p1 ? ce[3] : ce[2]) : (p1 ? ce[1] : ce[0]);
            const float so = p2 ? (p1 ? co[3] : co[2]) : (p1 ? co[1] : co[0]);
            float sum32 = __builtin_fmaf(so, 0.0625f, se) - (c == 0 ? corr0 : corr1);
            if constexpr (ZP_) sum32 = __builtin_fmaf(-(float)z2[c], c == 0 ? suma0 : suma1, sum32);
            acc.y[j] = __builtin_fmaf(sum32, (float)s2[c] * live, acc.y[j]);
          }
        }
        issue_from(rsrc_it, d, last_round ? d : it + DEPTH);
      }
    }

    // ---- add up the four pieces of each row (the lanes of a quad), then the RK partial results
    // into the rk == 0 waves.  Either way the segment ends with a barrier: the next segment's
    // prologue overwrites the LDS without waiting. ----
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      acc.y[j] += __shfl_xor(acc.y[j], 1);
      acc.y[j] += __shfl_xor(acc.y[j], 2);
    }
    if (RK == 1) __syncthreads();
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
    first = (tid >> 6) * NB * 16 + ((tid & 63) >> 2);
    return tid < WN * 64 && (tid & 3) == 0;
  }

  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int /*pm*/, int pn, char *,
                                                 const void *bias_) {
    int e;
    if (!owns_output(e)) return;
    if (bias_ == nullptr) {  // the common case keeps the code it had before the epilogue operands existed
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = pn * BN + e + j * 16;
        if (col < a.N) a.C[col] = (half_t)acc.y[j];
      }
    } else {
      const half_t *bias = epi_bias(bias_);
      const int act = epi_act(bias_);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = pn * BN + e + j * 16;
        if (col < a.N) a.C[col] = (half_t)activate(acc.y[j] + bias_at(bias, col, a.N), act);
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
