// Up to 64 rows of A against fp16 / bfloat16 weights [N, K] (NT): the weights stream through LDS in loads that
// read CONTIGUOUS bytes.
//
// The general small-M kernel (tile_skinny.h) loads the 16x16x32 MFMA's operand layout straight from memory: lane l
// takes 16 bytes of weight row l % 16, so one load instruction touches 16 rows, 64 bytes of each.  Here a load
// instruction reads two rows of 512 contiguous bytes (the first 32 lanes one row, the others the next) directly into
// LDS, and the fragments come back out of LDS in the MFMA's order (16 x 16384 x 16384: 134 us -> 87 us, 6.2 TB/s):
//
//  * CTA = four waves (times KH_, below), WM_ along M x WN_ along N x RK_ along K: wave (wm, wn, rk) owns MB_ blocks of 16 rows of A,
//    16 weight rows and the K sub-block rk of every iteration; the RK_ sums are added through LDS when the segment
//    ends (the reference's "block reduction", streamk_fp16_block_reduce.py:45,235-306).  An iteration is 256
//    K-values per wave.  The 16 weight rows x 512 bytes of (wn, rk) are fetched once, by eight loads shared out
//    among its WM_ waves, and the CTA's 16 MB_ WM_ rows of A x 512 RK_ bytes once, shared out among all four: both
//    operands travel once per CTA, in the same contiguous order.
//    Tile shapes: 16 x 32 with K split in two (N = 8192 gives every CU a tile of its own and no fix-up between
//    CTAs), 16 x 64 and 32 x 64 without, 64 x 32 as two by two waves.
//  * A pair of rows occupies 1056 bytes of LDS (two rows of 512 bytes and 32 bytes of padding); the odd row of a pair
//    holds its 16-byte pieces with neighbours swapped (the lane fetches piece p ^ 1 for position p).  A fragment read
//    -- lane (i = l % 16, g = l / 16) wants piece 4 s + g of row i -- then has its 16 lanes of equal g on 16
//    different bank groups.
//  * A ring of DEPTH_ slots per (wn, rk) holds the weights, a ring of three slots A: DEPTH_ - 1 iterations of weights
//    and two of A are in flight.  Per iteration one wait for the wave's own loads (vmcnt, in order), one barrier
//    (everybody's loads of the iteration have landed, and the slots refilled next have been read by everybody), the
//    loads that refill them, 8 + 8 MB_ fragment reads and 8 MB_ MFMAs.
//  * KH_ = 2 (the 64 x 64 and the 16 x 16 instances): two waves share the eight 32-wide K-steps of every (wm, wn, rk)
//    and its loads, eight waves per CTA, their sums added through LDS with the RK_ ones (64 x 28672 x 8192 from HBM
//    90.8 -> 86.4 us, 16 x 4096 x 4096 9.7 -> 9.2; the other instances gain nothing or lose: 64 x 32 tiles at
//    64 x 8192 x 8192 28.8 -> 33.8 us).
//  * Tiles walk K from different offsets (rotation_of, sk_device.h).
//
// Replaces the reference's inner MAC for its own run shape, 16 x 16384 x 8192 (streamk_fp16_nt.py:15, :196-240).
#pragma once
#include "tile_skinny.h"

namespace sk {

template <int MB_, int WM_, int WN_, int RK_, int DEPTH_, bool BF16_ = false, int NB_ = 1, int AD_ = 3, bool PADDED_ = true,
          int KH_ = 1>
struct TileStreamPairs {
  typedef SkinnyArgs Args;
  typedef floatx4 AccV;
  static constexpr bool LEAN_ENTRY = false;  // see run_persistent
  static constexpr bool NO_FLAT_ARGS = false;
  static constexpr bool COHERENT_PARTIALS = true;
  // the rings are dead between two calls of mac (it ends with every load landed and a barrier), and the 64 x 64
  // instance fills the 160 KB of LDS: the persistent loop's one word of LDS is the first word of the rings
  static constexpr bool FIXUP_WORD_IN_LDS = true;
  // AD slots of A (three unless LDS is short): its loads are issued later than the weights' when DEPTH_ is larger
  // KH_ waves share the eight 32-wide K-steps of a (wm, wn, rk) wave's iteration (and its loads) between them
  static constexpr int MB = MB_, NB = NB_, WM = WM_, WN = WN_, RK = RK_, WD = DEPTH_, AD = AD_, KH = KH_, NT = 256 * KH_;
  static constexpr int NWAVES = 4 * KH, STEPS = 8 / KH;
  static_assert(KH == 1 || KH == 2 || KH == 4, "one, two or four waves per K sub-block");
  static constexpr bool PADDED = PADDED_;
  static_assert(WM == 1 || WM == 2, "the eight loads of a weight ring are shared out among WM_ waves");
  static constexpr int BM = 16 * MB * WM, BN = 16 * NB * WN, MAX_M = BM;
  static constexpr int BK = 256, BKC = 256 * RK;       // K-values per iteration: of a wave, of the CTA
  // a pair of rows: two rows of 512 bytes; PADDED_: + 32 bytes and neighbouring pieces swapped in the odd row;
  // else no padding and piece p of row r (of its block of 16) kept at position p ^ r
  static constexpr int PAIR = PADDED ? 1056 : 1024;
  static constexpr int W_SLOT = 8 * PAIR;              // 16 weight rows of one iteration
  static constexpr int A_PAIRS = 8 * MB * WM;          // pairs of rows of A in the tile
  static constexpr int A_CHUNK = A_PAIRS * PAIR;       // the tile's rows of A, 256 K-values
  static constexpr int A_SLOT = RK * A_CHUNK;          // the tile's rows of A of one iteration
  static constexpr int RINGS = WN * NB * RK;           // one ring per block of 16 weight rows and K sub-block
  static constexpr int LDS_W = RINGS * WD * W_SLOT, LDS_BYTES = LDS_W + AD * A_SLOT, LDS_TOTAL = LDS_BYTES;
  static_assert(WD >= AD && AD >= 2, "the barrier of an iteration frees the slots read an iteration earlier");
  static constexpr int CTAS_PER_CU = (160 * 1024) / (LDS_BYTES + 64) > 0 ? (160 * 1024) / (LDS_BYTES + 64) : 1;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * KH;
  static constexpr int TILE_ELEMS = BM * BN;
  static constexpr int NTP = WM * WN * 64;             // the rk == 0 waves hold the tile's sums
  static constexpr int NV4 = MB * NB;
  static constexpr int LOADS_W = NB * 8 / (WM * KH), LOADS_A = (A_PAIRS * RK) / NWAVES;  // direct-to-LDS loads per wave and iteration
  // Loads are issued in the order A(t + AD - 1), W(t + WD - 1) in iteration t, and complete in that order.  Iteration t
  // needs everything up to A(t) and W(t): with WD == AD that leaves the AD - 2 later iterations outstanding, with
  // WD > AD (W(t) is older than A(t)) the weights issued with A(t) and the AD - 2 iterations after them.
  static constexpr int OUTSTANDING = (WD > AD ? LOADS_W : 0) + (AD - 2) * (LOADS_W + LOADS_A);

  // c[i][j][r] = C[pm*BM + (wm*MB + i)*16 + lane%16][pn*BN + (wn*NB + j)*16 + 4*(lane/16) + r]
  struct Acc {
    AccV c[MB][NB];
  };

  template <int N>
  static __device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
  }

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n, char *smem) {
    // (checked here and not in the class: tile_stream_q4.h derives from instances it does not run this loop of)
    static_assert(WM * WN * RK == 4, "four waves");
    static_assert(LDS_BYTES <= 160 * 1024, "the rings must fit the LDS of a CU");
    static_assert((RK * KH - 1) * WN * WM * 64 * MB * NB * 16 <= LDS_W, "the sums of the K-splitting waves pass through the weights' rings");
    static_assert((A_PAIRS * RK) % NWAVES == 0 && 8 % (WM * KH) == 0, "the loads are shared out evenly");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    // wave = ((kh RK + rk) WN + wn) WM + wm: the waves that end up with the tile's sums come first
    const int wm = wave % WM, wn = (wave / WM) % WN, rk = (wave / (WM * WN)) % RK, kh = wave / (WM * WN * RK);
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc.c[i][j] = AccV{0, 0, 0, 0};

    // ---- descriptors: the NB blocks of 16 weight rows of (wn) (rows past N read as zero), the tile's rows of A ----
    const int row0 = pn * BN + wn * (16 * NB);
    const int rows_w = max(0, min(16 * NB, a.N - row0));
    const uint32_t ldw_bytes = (uint32_t)a.ldw * 2, lda_bytes = (uint32_t)a.lda * 2;
    const uint4v rsrc_w = uniform_rsrc(
        make_rsrc_words(reinterpret_cast<const char *>(a.W) + (int64_t)row0 * ldw_bytes, (uint32_t)rows_w * ldw_bytes));
    const int a_rows = max(0, min(a.M - pm * BM, BM));
    const uint4v rsrc_a = uniform_rsrc(make_rsrc_words(a.A + (int64_t)pm * BM * a.lda, (uint32_t)a_rows * lda_bytes));
    // a load: lane l writes position l % 32 of row 2 j + l / 32 of pair j (of a block of 16 rows).  PADDED: the
    // position holds piece (l % 32) ^ (l / 32); else piece (l % 32) ^ (row % 16)
    const int odd = lane >> 5, piece0 = (lane & 31) ^ odd;
    auto piece_of = [&](int j) { return PADDED ? piece0 : piece0 ^ ((2 * j) & 15); };
    // fragment of lane (i, g) for K-step s of the iteration: row i, piece 4 s + g
    const int fi = lane & 15, fg = lane >> 4;
    const int frag0 = PADDED ? (fi >> 1) * PAIR + (fi & 1) * 512 + ((fg ^ (fi & 1)) * 16)
                             : fi * 512 + 16 * ((fi & 12) | (fg ^ (fi & 3)));
    const uint32_t base = lds_address(smem);
    const int ring0 = (rk * WN + wn) * NB;   // this wave's first ring
    const uint32_t w_ring = (uint32_t)__builtin_amdgcn_readfirstlane((int)(base + (uint32_t)ring0 * (WD * W_SLOT)));
    const uint32_t a_ring = (uint32_t)__builtin_amdgcn_readfirstlane((int)(base + (uint32_t)LDS_W));
    const char *w_ptr = smem + ring0 * (WD * W_SLOT) + frag0;
    const char *a_ptr = smem + LDS_W + rk * A_CHUNK + wm * (8 * MB * PAIR) + frag0;

    // iteration t of the segment (t = 0 .. n - 1) covers K-values k_of(t) 256 RK ..; iterations past the segment and
    // pieces past K fetch nothing (out-of-range offset: zeros arrive and the wait counts stay exact)
    const int rot = rotation_of(pn, n);
    auto k_of = [&](int t) { return k0 + rotated_iteration(t, rot, n); };
    auto issue_w = [&](int t, int slot) {
      const int kk = k_of(t) * BKC + rk * BK;
      const uint32_t kbytes = (uint32_t)__builtin_amdgcn_readfirstlane(kk * 2);
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int jj = 0; jj < 8 / (WM * KH); ++jj) {
          const int j = (kh * WM + wm) * (8 / (WM * KH)) + jj;   // this wave's share of the ring's eight pairs of rows
          const int pc = piece_of(j);
          dma_load_16(rsrc_w, w_ring + (uint32_t)((b * WD + slot) * W_SLOT + j * PAIR),
                      (t < n && kk + pc * 8 < a.K) ? (uint32_t)odd * ldw_bytes + (uint32_t)pc * 16 : OOB_OFFSET,
                      kbytes + (uint32_t)(16 * b + 2 * j) * ldw_bytes);
        }
    };
    auto issue_a = [&](int t, int slot) {
#pragma unroll
      for (int j = 0; j < LOADS_A; ++j) {
        const int q = wave * LOADS_A + j;   // this wave's share of the iteration's RK x A_PAIRS pairs of A's rows
        const int chunk = q / A_PAIRS, pj = q % A_PAIRS;
        const int kk = k_of(t) * BKC + chunk * BK;
        const uint32_t kbytes = (uint32_t)__builtin_amdgcn_readfirstlane(kk * 2);
        const int pc = piece_of(pj);
        dma_load_16(rsrc_a, a_ring + (uint32_t)(slot * A_SLOT + chunk * A_CHUNK + pj * PAIR),
                    (t < n && kk + pc * 8 < a.K) ? (uint32_t)odd * lda_bytes + (uint32_t)pc * 16 : OOB_OFFSET,
                    kbytes + (uint32_t)(2 * pj) * lda_bytes);
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
      const char *wp = w_ptr + ws * W_SLOT, *ap = a_ptr + as * A_SLOT;
      half8v fw[NB][8], fa[MB][8];   // (this wave's steps kh STEPS .. kh STEPS + STEPS - 1 only)
#pragma unroll
      for (int s8 = 0; s8 < STEPS; ++s8) {
        const int s = KH == 1 ? s8 : kh * STEPS + s8;
        // PADDED: piece 4 s + g sits 64 s bytes further on; else its position is (4 s + g) ^ i: 64 s XORed in
        const int so = PADDED ? s * 64 : 0;
        const int sx = PADDED ? 0 : s * 64;
#pragma unroll
        for (int j = 0; j < NB; ++j)
          fw[j][s8] = *reinterpret_cast<const half8v *>(xor_offset(wp + j * (WD * W_SLOT), frag0, sx) + so);
#pragma unroll
        for (int i = 0; i < MB; ++i) fa[i][s8] = *reinterpret_cast<const half8v *>(xor_offset(ap + i * 8 * PAIR, frag0, sx) + so);
      }
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
          for (int j = 0; j < NB; ++j) {
            if constexpr (BF16_) {
              typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
              acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fw[j][s]), __builtin_bit_cast(bf16x8, fa[i][s]),
                                                                    acc.c[i][j], 0, 0, 0);
            } else {
              acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[j][s], fa[i][s], acc.c[i][j], 0, 0, 0);
            }
          }
      // the fragments are in registers before the next barrier hands the slots back to the loads
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      ws = ws + 1 == WD ? 0 : ws + 1;
      as = as + 1 == AD ? 0 : as + 1;
    }
    // the loads still in flight (they fetch nothing) write LDS: let them land before the rings are reused
    wait_loads<0>();
    __syncthreads();

    // ---- sum the RK partial accumulators into the rk == 0 waves (through the weights' rings, free by now) ----
    if constexpr (RK * KH > 1) {
      float *red = reinterpret_cast<float *>(smem);
      if (wave >= WM * WN) {
#pragma unroll
        for (int v = 0; v < NV4; ++v)
          *reinterpret_cast<AccV *>(red + (((wave - WM * WN) * NV4 + v) * 64 + lane) * 4) = acc.c[v / NB][v % NB];
      }
      __syncthreads();
      if (wave < WM * WN) {
#pragma unroll
        for (int r = 1; r < RK * KH; ++r)
#pragma unroll
          for (int v = 0; v < NV4; ++v)
            acc.c[v / NB][v % NB] += *reinterpret_cast<const AccV *>(red + ((((r - 1) * WM * WN + wave) * NV4 + v) * 64 + lane) * 4);
      }
      __syncthreads();
    }
  }
  // p + (x ^ frag-relative bits): the position of a piece inside its row is the low part of the lane's offset frag0
  // (bits 4..8), which the unpadded layout XORs with 64 s
  static __device__ __forceinline__ const char *xor_offset(const char *p, int frag0, int sx) {
    return p - frag0 + (frag0 ^ sx);
  }

  // (two copies behind one uniform branch: the epilogue without a bias carries none of its code)
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int pm, int pn, char *smem, const void *bias) {
    if (bias == nullptr)
      store_c_impl<false>(a, acc, pm, pn, nullptr);
    else
      store_c_impl<true>(a, acc, pm, pn, bias);
  }
  template <bool BIAS>
  static __device__ __forceinline__ void store_c_impl(const Args &a, const Acc &acc, int pm, int pn, const void *epi) {
    const half_t *bias = BIAS ? epi_bias(epi) : nullptr;
    const int act = BIAS ? epi_act(epi) : 0;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (wave >= WM * WN) return;
    const int wm = wave % WM, wn = wave / WM;
    const int lr = lane & 15, lg = lane >> 4;
    const bool vec_ok = (a.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 7) == 0);
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const int row = pm * BM + (wm * MB + i) * 16 + lr;
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = pn * BN + (wn * NB + j) * 16 + lg * 4;
        if (row < a.M && col < a.N) {
          half4v h;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = acc.c[i][j][e];
            if constexpr (BIAS) x = activate(x + bias_at<BF16_>(bias, col + e, a.N), act);
            if constexpr (BF16_) {
              const __bf16 b = (__bf16)x;
              h[e] = __builtin_bit_cast(half_t, b);  // C carries 16-bit patterns
            } else {
              h[e] = (half_t)x;
            }
          }
          half_t *dst = a.C + (int64_t)row * a.ldc + col;
          if (vec_ok && col + 4 <= a.N) {
            *reinterpret_cast<half4v *>(dst) = h;
          } else {
            for (int e = 0; e < 4 && col + e < a.N; ++e) dst[e] = h[e];
          }
        }
      }
    }
  }

  // Partial tiles are a few KB: every access is a coherent (write-through / L2-bypassing) one, as in tile_skinny.h.
  // Block v = i NB + j of thread t (one of the NTP threads of the rk == 0 waves) is kept at (v NTP + t) 4; the
  // accumulating form keeps element e of it at (v 4 + e) NTP + t.
  static __device__ __forceinline__ void store_partial(const Acc &acc, float *dst) {
    if (threadIdx.x >= NTP) return;
#pragma unroll
    for (int v = 0; v < NV4; ++v) st_coherent(dst + ((size_t)v * NTP + threadIdx.x) * 4, acc.c[v / NB][v % NB]);
  }
  static __device__ __forceinline__ void add_partial(Acc &acc, const float *src) {
    if (threadIdx.x >= NTP) return;
#pragma unroll
    for (int v = 0; v < NV4; ++v) acc.c[v / NB][v % NB] += ld_coherent(src + ((size_t)v * NTP + threadIdx.x) * 4);
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst) {
    if (threadIdx.x >= NTP) return;
#pragma unroll
    for (int v = 0; v < NV4; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) atomic_add_f32(dst + (size_t)(v * 4 + e) * NTP + threadIdx.x, acc.c[v / NB][v % NB][e]);
  }
  static __device__ __forceinline__ void take_partial(Acc &acc, float *src) {
    if (threadIdx.x >= NTP) return;
#pragma unroll
    for (int v = 0; v < NV4; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float *p = src + (size_t)(v * 4 + e) * NTP + threadIdx.x;
        acc.c[v / NB][v % NB][e] = ld_coherent_scalar(p);
        st_coherent(p, 0.f);
      }
  }
};

}  // namespace sk
