// Up to 16 rows of A against Q4 weights [N, K/2] (row-major nibbles, one scalar zero point): the packed weights stream
// through LDS in loads that read CONTIGUOUS bytes, as the fp16 weights do in tile_stream_pairs.h.
//
// The general small-M kernel (tile_skinny.h) loads 16 bytes of weight row l % 16 per lane: one load instruction
// touches 16 rows, 64 bytes of each.  Here a load instruction reads four rows of 256 contiguous bytes (512 K-values)
// directly into LDS, and lane (i, g) reads its 16 bytes of row i back out of LDS: the registers then hold what the
// general kernel's loads deliver, and the arithmetic is that kernel's for up to 16 rows (tile_skinny.h, UNDECODED):
// the nibbles enter the 16x16x32 MFMA as 1024 + q / 64 + q, every 128-wide scale group's sum starts from
// -sum a_k (offset_k + zero) (four MFMAs on a constant fragment) and is multiplied by the group's scale in fp32.
//
//  * CTA = WN_ along N x RK_ along K rings of weights, KH_ waves per ring, which share out the 512 K-values of an
//    iteration in steps of 128 (one scale group): four rings of four waves each in the instances built, sixteen waves,
//    four per SIMD (one wave's waits for LDS and for its MFMAs are covered by the three others: with two waves per
//    ring 16 x 8192 x 8192 took 10.7 us against 10.2 with the weights in the Infinity Cache, 16 x 4096 x 11008 13.3
//    against 12.2).  Per iteration and ring: four loads of weights (16 rows x 256 bytes) shared out between its
//    waves, one load of scales per wave (16 rows x the pair of groups its step is in, four bytes per lane), and the
//    16 RK_ loads of A (one row of 1024 bytes each) shared out among all waves, all direct to LDS.
//  * No padding: lane l of a load fetches the 16-byte piece (l % 16) ^ (row % 16) of its row for position l % 16
//    (A: piece l ^ row of the row's 64), so the sixteen lanes that read the same piece of sixteen rows find it on
//    sixteen different bank groups.
//  * A arrives in natural element order; the extraction delivers the eight values of a word in the order
//    0,4,1,5,2,6,3,7, so each 16-byte fragment of A is put into that order with four byte permutes after it is read.
//  * Rings of WD_ slots for weights and scales (per wave), AD_ slots for A; loads are issued in the order
//    A(t + AD_ - 1), W(t + WD_ - 1) and complete in that order, one wait and one barrier per iteration.
//  * Tiles walk K from different offsets (rotation_of, sk_device.h).
//
// Where the time goes (16 x 16384 x 16384, 134 MB of weights, one 64-row tile per CU): A is as many bytes per CTA as
// the weights (16 rows of fp16 against 64 rows of nibbles) and travels from the L2 into LDS beside them; with the
// bit-exact decode it had first (fp16((q - zero) * scale) per weight, 155 vector instructions per wave and iteration
// for 8 MFMAs) and the permutes taken out the kernel ran 24 us with the weights in the Infinity Cache and 32 us
// from HBM, with them 35 / 41 us; with the nibbles undecoded 31.7 / 37.8 us.
//
// Epilogue, partial tiles and fix-ups are those of tile_stream_pairs.h (one block of 16 rows of A per wave).
// Replaces the reference's decode-then-MMA step for its own run shape, 16 x 16384 x 16384
// (streamk_fp16_ladder_block_reduce_q4.py:73, :283-294).
#pragma once
#include "q4_dequant.h"
#include "tile_stream_pairs.h"

namespace sk {

template <int WN_, int RK_, int KH_, int WD_, int AD_>
struct TileStreamQ4 : TileStreamPairs<1, 1, WN_, RK_, 3, false> {
  typedef TileStreamPairs<1, 1, WN_, RK_, 3, false> Base;
  typedef typename Base::Args Args;
  typedef typename Base::Acc Acc;
  typedef typename Base::AccV AccV;
  static constexpr int KH = KH_;                       // waves that share the weights of an iteration, 512 / KH_ K-values each
  static constexpr int STEPS = 4 / KH;                 // steps of 128 K-values (one scale group) per wave and iteration
  static constexpr int RINGS = WN_ * RK_, NWAVES = RINGS * KH;
  static_assert(KH == 1 || KH == 2 || KH == 4, "one, two or four waves per ring");
  static constexpr int SG = STEPS < 2 ? 2 : STEPS;     // scale groups a wave's load of scales brings per row (a load moves four bytes per lane)
  static constexpr int WN = WN_, RK = RK_, WD = WD_, AD = AD_, NT = 64 * NWAVES, BM = 16, BN = 16 * WN, MAX_M = 16;
  static constexpr int BK = 512, BKC = 512 * RK;       // K-values per iteration: of a weight ring, of the CTA
  static constexpr int W_SLOT = 16 * 256;              // 16 weight rows x 256 bytes
  static constexpr int S_SLOT = 256;                   // a wave's scales: 16 rows x STEPS groups in the first lanes of one load
  static constexpr int A_CHUNK = 16 * 1024;            // 16 rows of A x 512 K-values
  static constexpr int A_SLOT = RK * A_CHUNK;
  static constexpr int LDS_W = RINGS * WD * W_SLOT, LDS_S = NWAVES * WD * S_SLOT;
  static constexpr int LDS_BYTES = LDS_W + LDS_S + AD * A_SLOT, LDS_TOTAL = LDS_BYTES;
  static_assert(LDS_BYTES <= 160 * 1024, "the rings must fit the LDS of a CU");
  static_assert(WD >= AD && AD >= 2, "weights are requested at least as far ahead as A");
  static_assert((NWAVES - WN) * 64 * 16 <= LDS_W, "the sums of the K-splitting waves pass through the weights' rings");
  static_assert((16 * RK) % NWAVES == 0, "the loads of A are shared out evenly");
  static constexpr int CTAS_PER_CU = 1, WAVES_PER_EU = KH;
  static constexpr int TILE_ELEMS = BM * BN;
  // direct-to-LDS loads per wave and iteration: half of the ring's four loads of weights, the wave's own scales,
  // its share of the iteration's 16 RK rows of A
  static constexpr int LOADS_W = 4 / KH + 1, LOADS_A = 16 * RK / NWAVES;
  // at the top of iteration t everything up to A(t) has to be there: what may still be on its way are the weights
  // issued behind A(t) (when they are requested further ahead than A) and the AD - 2 iterations of loads after them
  static constexpr int OUTSTANDING = (WD > AD ? LOADS_W : 0) + (AD - 2) * (LOADS_W + LOADS_A);

  template <int N>
  static __device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
  }
  static __device__ __forceinline__ void dma_load_4(uint4v rsrc, uint32_t lds_base, uint32_t lane_off, uint32_t uniform_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_base), "v"(lane_off), "s"(rsrc), "s"(uniform_off)
                 : "memory", "m0");
  }

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n, char *smem) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    // wave = (kh RK + rk) WN + wn: the waves that end up with the tile's sums come first
    const int wn = wave % WN, rk = (wave / WN) % RK, kh = wave / RINGS;
    const int ring = rk * WN + wn;
    AccV part[2] = {AccV{0, 0, 0, 0}, AccV{0, 0, 0, 0}};

    // ---- descriptors: the ring's 16 weight rows and their scales (rows past N read as zero), the rows of A ----
    const int row0 = pn * BN + wn * 16;
    const int rows_w = max(0, min(16, a.N - row0));
    const uint32_t ldw_bytes = (uint32_t)a.ldw, lda_bytes = (uint32_t)a.lda * 2, lds_bytes = (uint32_t)a.groups * 2;
    const uint4v rsrc_w = uniform_rsrc(
        make_rsrc_words(reinterpret_cast<const char *>(a.W) + (int64_t)row0 * ldw_bytes, (uint32_t)rows_w * ldw_bytes));
    const uint4v rsrc_s = uniform_rsrc(make_rsrc_words(a.scales + (int64_t)row0 * a.groups, (uint32_t)rows_w * lds_bytes));
    const int a_rows = max(0, min(a.M - pm * BM, BM));
    const uint4v rsrc_a = uniform_rsrc(make_rsrc_words(a.A + (int64_t)pm * BM * a.lda, (uint32_t)a_rows * lda_bytes));
    // weights: lane l of load j writes position l % 16 of row 4 j + l / 16, which holds piece (l % 16) ^ (row % 16);
    // wave kh issues the loads j = 2 kh, 2 kh + 1
    const int wr = lane >> 4, wp0 = (lane & 15) ^ wr;
    uint32_t voff_w[4 / KH];
    int piece_w[4 / KH];
#pragma unroll
    for (int jj = 0; jj < 4 / KH; ++jj) {
      piece_w[jj] = wp0 ^ (4 * (kh * (4 / KH) + jj));
      voff_w[jj] = (uint32_t)wr * ldw_bytes + (uint32_t)piece_w[jj] * 16;
    }
    // scales: STEPS / 2 lanes per row, four bytes each (the groups of the wave's 128 STEPS K-values)
    const uint32_t voff_s = lane < 8 * SG ? (uint32_t)(lane / (SG / 2)) * lds_bytes + (uint32_t)(lane % (SG / 2)) * 4 : OOB_OFFSET;
    // fragments: wave kh takes the steps s = 2 kh, 2 kh + 1 of the iteration; lane (i, g) reads piece 4 s + g of
    // weight row i, found at position (4 s + g) ^ i, and for word q of it the eight values of A row i from K offset
    // 32 (4 s + g) + 8 q: piece 16 s + 4 g + q, at position piece ^ i
    const int fi = lane & 15, fg = lane >> 4;
    const uint32_t base = lds_address(smem);
    const uint32_t w_ring = (uint32_t)__builtin_amdgcn_readfirstlane((int)(base + (uint32_t)ring * (WD * W_SLOT)));
    const uint32_t s_ring = (uint32_t)__builtin_amdgcn_readfirstlane((int)(base + (uint32_t)(LDS_W + wave * (WD * S_SLOT))));
    const uint32_t a_ring = (uint32_t)__builtin_amdgcn_readfirstlane((int)(base + (uint32_t)(LDS_W + LDS_S)));
    const char *w_rd[STEPS], *a_rd[4];
#pragma unroll
    for (int ss = 0; ss < STEPS; ++ss)
      w_rd[ss] = smem + ring * (WD * W_SLOT) + fi * 256 + 64 * ((STEPS * kh + ss) ^ (fi >> 2)) + 16 * (fg ^ (fi & 3));
#pragma unroll
    for (int q = 0; q < 4; ++q)
      a_rd[q] = smem + LDS_W + LDS_S + rk * A_CHUNK + fi * 1024 + 256 * STEPS * kh + 16 * ((4 * fg + q) ^ fi);
    const char *s_rd4 = smem + LDS_W + wave * (WD * S_SLOT) + fg * (4 * 2 * SG) + ((STEPS * kh) % SG) * 2;
    const Q4Consts qc = q4_consts(a.zero);
    // the magic of the nibbles at bits 4..7 of a half (fp16 64.0: 64 + q) and minus the offsets of a word's eight
    // elements in the order the extraction leaves them (0,4 | 1,5 | 2,6 | 3,7: bits 0..3, bits 4..7, 0..3, 4..7)
    uint32_t magic_hi = 0x54005400u;
    asm volatile("" : "+v"(magic_hi));
    const half_t off_lo = (half_t)(float)(-(1024 + a.zero)), off_hi = (half_t)(float)(-(64 + a.zero));
    const half8v neg_offsets = half8v{off_lo, off_lo, off_hi, off_hi, off_lo, off_lo, off_hi, off_hi};

    // iteration t of the segment (t = 0 .. n - 1) covers K-values k_of(t) 512 RK ..; iterations past the segment and
    // pieces past K fetch nothing (out-of-range offset: zeros arrive and the wait counts stay exact)
    const int rot = rotation_of(pn, n);
    auto k_of = [&](int t) { return k0 + rotated_iteration(t, rot, n); };
    auto issue_w = [&](int t, int slot) {
      const int kk = k_of(t) * BKC + rk * BK;
      const uint32_t kbytes = (uint32_t)__builtin_amdgcn_readfirstlane(kk / 2);
#pragma unroll
      for (int jj = 0; jj < 4 / KH; ++jj) {
        const int j = kh * (4 / KH) + jj;
        dma_load_16(rsrc_w, w_ring + (uint32_t)(slot * W_SLOT + j * 1024),
                    (t < n && kk + piece_w[jj] * 32 < a.K) ? voff_w[jj] : OOB_OFFSET, kbytes + (uint32_t)(4 * j) * ldw_bytes);
      }
      dma_load_4(rsrc_s, s_ring + (uint32_t)(slot * S_SLOT), t < n ? voff_s : OOB_OFFSET,
                 (uint32_t)__builtin_amdgcn_readfirstlane((kk / 128 + (STEPS * kh) / SG * SG) * 2));
    };
    auto issue_a = [&](int t, int slot) {
#pragma unroll
      for (int j = 0; j < LOADS_A; ++j) {
        const int q = wave * LOADS_A + j;   // this wave's share of the iteration's RK x 16 rows of A
        const int chunk = q >> 4, m = q & 15;
        const int kk = k_of(t) * BKC + chunk * BK;
        const int piece = lane ^ m;
        dma_load_16(rsrc_a, a_ring + (uint32_t)(slot * A_SLOT + chunk * A_CHUNK + m * 1024),
                    (t < n && kk + piece * 8 < a.K) ? (uint32_t)piece * 16 : OOB_OFFSET,
                    (uint32_t)__builtin_amdgcn_readfirstlane(kk * 2) + (uint32_t)m * lda_bytes);
      }
    };
    // what the iterations -(WD - 1) .. -1 would have issued
#pragma unroll
    for (int j = 1 - WD; j < 0; ++j) {
      if (j + AD - 1 >= 0) issue_a(j + AD - 1, j + AD - 1);
      issue_w(j + WD - 1, j + WD - 1);
    }

    int ws = 0, as = 0;   // slots of iteration t: t % WD, t % AD
    for (int t = 0; t < n; ++t) {   // (n is the same for every wave of the CTA: the barriers stay matched)
      wait_loads<OUTSTANDING>();
      __syncthreads();   // everybody's loads of the iteration have landed; everybody has read the slots refilled next
      issue_a(t + AD - 1, as == 0 ? AD - 1 : as - 1);
      issue_w(t + WD - 1, ws == 0 ? WD - 1 : ws - 1);
      const int wofs = ws * W_SLOT, aofs = as * A_SLOT;
      uint4v wf[STEPS];
#pragma unroll
      for (int ss = 0; ss < STEPS; ++ss) wf[ss] = *reinterpret_cast<const uint4v *>(w_rd[ss] + wofs);
      // the scales of the four weight rows this lane holds sums of (result register r: row 4 (lane / 16) + r)
      half_t sc[4][STEPS];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int ss = 0; ss < STEPS; ++ss) sc[r][ss] = *reinterpret_cast<const half_t *>(s_rd4 + ws * S_SLOT + (r * SG + ss) * 2);
#pragma unroll
      for (int ss = 0; ss < STEPS; ++ss) {
        // one step is one scale group: its sum starts from -sum a_k (offset_k + zero), four MFMAs on a constant
        // fragment; the nibbles follow undecoded (1024 + q, 64 + q); the scale multiplies the fp32 group sum
        half8v fa[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint4v v = *reinterpret_cast<const uint4v *>(a_rd[q] + aofs + 256 * ss);
          uint4v p;   // element order 0,4,1,5,2,6,3,7
          p[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
          p[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
          p[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
          p[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
          fa[q] = __builtin_bit_cast(half8v, p);
        }
        AccV sum = AccV{0, 0, 0, 0};   // (one chain: the other waves of the SIMD cover the wait between dependent MFMAs)
#pragma unroll
        for (int q = 0; q < 4; ++q) sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(neg_offsets, fa[q], sum, 0, 0, 0);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          union {
            uint32_t u[4];
            half8v v;
          } raw;
          const uint32_t w = wf[ss][q], t8 = w >> 8;
          raw.u[0] = and_or(w, qc.mask_lo, qc.magic);
          raw.u[1] = and_or(w, qc.mask_hi, magic_hi);
          raw.u[2] = and_or(t8, qc.mask_lo, qc.magic);
          raw.u[3] = and_or(t8, qc.mask_hi, magic_hi);
          sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(raw.v, fa[q], sum, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) part[0][r] = __builtin_fmaf(sum[r], (float)sc[r][ss], part[0][r]);
      }
      // the fragments are in registers before the next barrier hands the slots back to the loads
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      ws = ws + 1 == WD ? 0 : ws + 1;
      as = as + 1 == AD ? 0 : as + 1;
    }
    acc.c[0][0] = part[0] + part[1];
    // the loads still in flight (they fetch nothing) write LDS: let them land before the rings are reused
    wait_loads<0>();
    __syncthreads();

    // ---- sum the partial accumulators of the waves that split K into the first WN waves (through the weights'
    // rings, free by now) ----
    if constexpr (NWAVES > WN) {
      float *red = reinterpret_cast<float *>(smem);
      if (wave >= WN) *reinterpret_cast<AccV *>(red + ((wave - WN) * 64 + lane) * 4) = acc.c[0][0];
      __syncthreads();
      if (wave < WN) {
#pragma unroll
        for (int r = 1; r < KH * RK; ++r) acc.c[0][0] += *reinterpret_cast<const AccV *>(red + (((r - 1) * WN + wave) * 64 + lane) * 4);
      }
      __syncthreads();
    }
  }
};

}  // namespace sk
