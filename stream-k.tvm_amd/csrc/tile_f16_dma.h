// fp16 NT tile arithmetic with direct global->LDS loads (buffer_load ... lds, 16 bytes per lane),
// XOR-swizzled LDS rows and a two-stage software pipeline.  BK is fixed at 64 (one LDS row = 128
// bytes = 8 chunks of 16 bytes).
//
// LDS layout of one stage: BM rows of A then BN rows of B, 128 bytes each; chunk c of row r lives
// at chunk position c ^ ((r >> 1) & 7) (XOR swizzle in the spirit of the reference's,
// streamk_fp16.py:72-80).  With 64 four-byte banks and 16 lanes served per cycle, rows r and r+1
// fall in different bank halves and (r >> 1) spreads the 8 row pairs over the 8 chunk positions:
// measured conflict-free for the 32-row fragment reads (r & 7 is 2-way conflicted).
// A wave-wide DMA instruction fills 1 KB = 8 consecutive rows: lane l writes position
// (row 8*G + l/8, chunk l%8) of row group G and therefore fetches global chunk
// (l%8) ^ (4*(G&1) + l/16).  A wave only ever loads groups of its own parity, so this is a
// per-lane constant and one VGPR offset per operand serves every load.
//
// Pipeline per K-iteration (stage `cur` holds the iteration's tiles, `nxt` the next one's):
//   K-steps 0..2:  wait fragments(kk) | issue ds_reads(kk+1) | 8 MFMAs(kk)
//   K-step 3:      wait fragments(3)  | wait own DMA(nxt), barrier
//                  | issue DMA(cur <- iteration+2), ds_reads(nxt, 0) | 8 MFMAs(3)
// so the barrier, the DMA issue and the first fragment reads of the next iteration all overlap
// with the last MFMA block.
#pragma once
#include <type_traits>

#include "q4_dequant.h"
#include "sk_device.h"
#include "tile_f16.h"

namespace sk {

// one LDS array per (size, id): distinct arrays let the compiler tell the stages apart when it
// orders LDS reads against in-flight DMA writes
template <int BYTES, int ID>
struct LdsArray {
  static __device__ __forceinline__ char *get() {
    __shared__ __attribute__((aligned(1024))) char buf[BYTES];
    return buf;
  }
};

// B_KN_: B is [K,N] row-major (NN GEMM).  Its stage is then 64 rows (K) of BN halfs.  Fragments
// are read with ds_read_b64_tr_b16, which hands lane L of each 16-lane group the element (L & 3) of
// the 8 bytes addressed by lane (L >> 2) + 4*j of that group, j = 0..3: a 16-lane group pointing at
// a 4 (K) x 16 (N) patch receives, per lane, 4 consecutive K of one column -- half an MFMA operand.
// 16-byte chunk c of K-row k is stored at position c ^ (4 * (k & 3)), which keeps the 32 lanes
// served in one cycle (2 groups x 4 rows x 32 bytes) on distinct banks.
//
// BK_ = 32: four stages of half the depth (LDS rows of 64 bytes, 4 chunks, chunk c of row r at
// position c ^ ((r >> 2) & 3); a wave-wide load fills 16 rows).  The tiles of iteration it+4 are
// requested when iteration it has been read, three iterations (about 1.5 iterations of the
// two-stage pipeline) before they are needed: a load that misses the L2 takes longer than one
// iteration of MFMAs, which the two-stage pipeline exposes as a stall at every barrier.
//
// MFMA16_: the arithmetic uses v_mfma_f32_16x16x32_f16 instead of v_mfma_f32_32x32x16_f16.  Both
// run at the same FLOP per cycle, but the 16x16x32 form reads and writes half as many accumulator
// registers per FLOP, and on random operands the part sustains a ~12 % higher clock with it under
// its power limit.  The accumulator is then kept as 16x16 blocks of four registers: lane l holds
// C[16*ii + l%16][16*jj + 4*(l/16) + e] of block (ii, jj).  A K-step covers 32 K-values: lane
// group g = l/16 takes 16-byte chunk 4*kk + g of its row.
//
// F8_ (1: e4m3, 2: e5m2, both OCP): A and B hold one byte per element and C is fp16.  The launcher
// passes K and the leading dimensions of A and B in 16-bit units (half the element counts), so the
// data movement is that of the fp16 kernel: an LDS row of 128 bytes is 128 K-values, one iteration.
// The arithmetic is v_mfma_f32_32x32x64_f8f6f4 (twice the FLOP of the 16-bit forms per byte of
// operand) into the 32x32 accumulator blocks of the fp16 kernel.  Lane (r = l%32, g = l/32) hands
// the instruction, for K-step s of 64 bytes, chunks 4s + g and 4s + 2 + g of row r as its 32-byte
// operand.  Which K-values a lane's bytes stand for does not matter as long as A and B agree: the
// instruction pairs byte b of lane group g of one operand with the same byte of the other.  With BK_ = 32
// an LDS row is 64 bytes, one K-step, and the loop is the four-stage one of the 16x16x32 form.
//
// F8_ = 3: int8 operands, int32 accumulators and C.  The 16x16x32 pipeline as it is, with
// v_mfma_i32_16x16x64_i8 on the same 16-byte fragments (64 K-values per K-step, same cycles as the fp16
// form); partial tiles travel through the workspace as int32 in the fp32 slots, so both fix-ups are
// exact and independent of the order of the additions.  C is stored from registers (a lane holds four
// consecutive int32 of a row).
//
// Q4_: B is not fp16 but packed nibbles with one fp16 scale per 128 K-values (the weight-only format of
// q4_dequant.h), for calls with more rows of A than the weight-streaming kernels take.  A travels as before.  B's
// nibbles of iteration it + 3 are loaded straight into one of two small LDS buffers (32 bytes per weight row);
// behind the barrier of iteration it, where the fp16 kernel requests B of iteration it + 2, every thread instead
// reads its share of the nibbles of iteration it + 2, dequantises them in registers with dequant_word_q4 -- the
// bit-exact decode (the reference dequantises in registers right before the MMA,
// streamk_fp16_ladder_block_reduce_q4.py:283-294) -- puts the eight weights of a word back into K order and stores
// them where the direct load would have put them.  The fragment reads and the MFMAs do not know the difference.
template <int BM_, int BN_, int WM_, int WN_, bool B_KN_ = false, int BK_ = 64, bool MFMA16_ = false, bool BF16_ = false,
          int F8_ = 0, bool Q4_ = false>
struct TileF16NTDma {
  static constexpr bool Q4 = Q4_;
  static_assert(!Q4_ || (MFMA16_ && !B_KN_ && BK_ == 64 && !BF16_ && F8_ == 0), "Q4: the two-stage 16x16x32 fp16 form");
  static constexpr bool B_KN = B_KN_, MFMA16 = MFMA16_;
  static constexpr bool I8 = F8_ == 3;
  static constexpr int F8 = I8 ? 0 : F8_;
  static_assert(F8 == 0 || (!MFMA16_ && !B_KN_ && !BF16_), "fp8: NT layout (two stages of 128 K-values or four of 64)");
  static_assert(!I8 || (MFMA16_ && !B_KN_ && !BF16_), "int8: NT layout, 16x16 accumulator blocks");
  // BF16_: operands and C are bfloat16 (same 16-bit data movement; v_mfma_f32_16x16x32_bf16; C rounded to
  // nearest even with v_cvt_pk_bf16_f32)
  static_assert(!BF16_ || MFMA16_, "bfloat16 exists in the 16x16x32 form");
  static constexpr int ROW_BYTES = BK_ * 2;                    // bytes of one LDS row of A (and of B, NT)
  static constexpr int ROWS_PER_DMA = 1024 / ROW_BYTES;        // rows one wave-wide load fills
  static constexpr int NSTAGE = 128 / BK_, KSTEPS = BK_ / (MFMA16_ ? 32 : 16);
  static_assert(BK_ == 64 || (BK_ == 32 && !B_KN_), "BK is 64, or 32 for the NT layout");
  static constexpr int B_ROW_BYTES = B_KN_ ? BN_ * 2 : ROW_BYTES;  // bytes of one LDS row of the B stage
  static constexpr int B_ROWS_PER_DMA = 1024 / B_ROW_BYTES;    // rows one wave-wide load fills
  static_assert(!B_KN_ || (BN_ >= 128 && BN_ <= 512), "NN layout: 16..64 chunks per LDS row");
  typedef GemmArgs Args;
  static constexpr bool LEAN_ENTRY = true;  // see run_persistent
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int NW = WM * WN, NT = NW * 64;
  static constexpr int TM = BM / (WM * 32), TN = BN / (WN * 32);
  static constexpr int WTM = TM * 32, WTN = TN * 32;
  static constexpr int FROWS = MFMA16_ ? 16 : 32;              // rows of one operand fragment
  static constexpr int FM = WTM / FROWS, FN = WTN / FROWS;     // fragments per K-step
  static constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES, STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int A_DMA = A_BYTES / 1024 / NW, B_DMA = Q4_ ? 0 : B_BYTES / 1024 / NW, DMA_PER_WAVE = A_DMA + B_DMA;
  // Q4: raw nibbles of one iteration: BN rows x 32 bytes; a wave-wide load covers 32 rows; a thread converts
  // Q4_WORDS 32-bit words (eight weights each)
  static constexpr int RAW_BYTES = BN * 32, RAW_DMA = RAW_BYTES / 1024, Q4_WORDS = BN * 8 / NT;
  static_assert(!Q4_ || (RAW_DMA <= NW && Q4_WORDS >= 1 && Q4_WORDS <= A_DMA && 8 % Q4_WORDS == 0), "Q4 tile shape");
  static constexpr int LDC = WTN + 8;
  // epilogue patches: the waves share out the stages evenly; split the wave tile's rows into
  // passes until the patches fit
  static constexpr int WAVES_PER_STAGE = NW / NSTAGE;
  static constexpr int patch_passes() {
    int p = 1;
    while (WAVES_PER_STAGE * (WTM / p) * LDC * 2 > STAGE_BYTES) p *= 2;
    return p;
  }
  static constexpr int PASSES = patch_passes();
  static constexpr int PATCH_ROWS = WTM / PASSES;
  static constexpr int LDS_BYTES = 16;  // the kernel's generic buffer is unused
  static constexpr int LDS_TOTAL = NSTAGE * STAGE_BYTES + (Q4_ ? 2 * RAW_BYTES : 0);
  static constexpr int TILE_ELEMS = BM * BN;
  static constexpr int NV4 = TM * TN * 4;
  static constexpr int CTAS_PER_CU_REGS = (NT >= 512 || TM * TN > 4) ? 1 : (TM * TN <= 2 ? 4 : 2);
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_TOTAL + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_REGS < CTAS_PER_CU_LDS ? CTAS_PER_CU_REGS : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile shape");
  static_assert((A_BYTES / 1024) % NW == 0 && (Q4_ || (B_BYTES / 1024) % NW == 0), "DMA groups must divide over the waves");
  static_assert(NW % NSTAGE == 0, "a wave must keep to row groups of one parity; patches per stage");
  static_assert(PATCH_ROWS % 32 == 0, "epilogue pass must hold whole 32-row blocks");
  static_assert(F8 == 0 || TM % 2 == 0, "fp8: the wave tile's rows are processed in two halves");

  typedef TileF16NT<BM_, BN_, 64, WM_, WN_> Base;  // shares the accumulator type and the partials
  // 16x16x32: the accumulator is kept as 16x16 blocks of four registers (block (ii, jj): lane l holds
  // C[16*ii + l%16][16*jj + 4*(l/16) + e]), each updated in place by its MFMA
  typedef int intx4 __attribute__((ext_vector_type(4)));
  typedef typename std::conditional<I8, intx4, floatx4>::type AccV;
  struct Acc16 {
    AccV v[FM][FN];
  };
  typedef typename std::conditional<MFMA16_, Acc16, typename Base::Acc>::type Acc;

  static __device__ __forceinline__ char *stage(int s) {
    if (NSTAGE == 2) return s == 0 ? LdsArray<STAGE_BYTES, 0>::get() : LdsArray<STAGE_BYTES, 1>::get();
    return s == 0 ? LdsArray<STAGE_BYTES, 0>::get()
                  : (s == 1 ? LdsArray<STAGE_BYTES, 1>::get()
                            : (s == 2 ? LdsArray<STAGE_BYTES, 2>::get() : LdsArray<STAGE_BYTES, 3>::get()));
  }

  template <int N>
  static __device__ __forceinline__ void wait_dma_then_barrier() {
    // own DMA writes of the awaited stage have landed (at most N younger loads still in flight),
    // then everybody's have.  "memory": nothing may be moved across by the compiler.
    if (N == 0)
      asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
  }

  // scheduling hint: one LDS read, then PER MFMAs, READS times
  template <int READS, int PER>
  static __device__ __forceinline__ void interleave16() {
#pragma unroll
    for (int g = 0; g < READS; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
    }
  }

  // scheduling hint for MFMAS matrix instructions with READS LDS reads spread over them
  template <int MFMAS, int READS>
  static __device__ __forceinline__ void interleave8() {
    if (READS % MFMAS) __builtin_amdgcn_sched_group_barrier(0x100, READS % MFMAS, 0);
#pragma unroll
    for (int g = 0; g < MFMAS; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x100, READS / MFMAS, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
  }

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n,
                                             char *) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;

    if constexpr (MFMA16) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc.v[i][j] = AccV{0, 0, 0, 0};
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc.c[i][j][r] = 0.f;
    }

    const int rows_a = min(BM, a.M - pm * BM), rows_b = min(BN, a.N - pn * BN);
    const uint4v rsrc_a = make_rsrc_words(a.A + (int64_t)pm * BM * a.lda, (uint32_t)(rows_a * a.lda * 2));
    // global chunk this lane fetches: its LDS position XOR the swizzle of its row
    const int my_chunk = BK == 64 ? (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4)) : (lane & 3) ^ (lane >> 4);
    const int my_row = BK == 64 ? lane >> 3 : lane >> 2;  // row within the load's group
    const uint32_t voff_a = (uint32_t)(my_row * a.lda + my_chunk * 8) * 2;
    const uint32_t grp_a = (uint32_t)(ROWS_PER_DMA * a.lda * 2);
    const int tail_kt = (a.K % BK != 0) ? (a.K / BK) : -1;
    // B operand.  NT: rows are N, same scheme as A.  NN: rows are K; the descriptor starts at the
    // tile's first column and ends with the last valid element of row K-1, so K-rows past the
    // matrix read as zero; columns past N are masked per lane (N % 8 == 0).
    uint4v rsrc_b;
    uint32_t voff_b, grp_b, kstep_b;
    if constexpr (Q4_) {
      // packed nibbles: ldb is the row pitch in bytes; a wave-wide load covers 32 rows x 32 bytes, lane l the
      // 16-byte half l % 2 of row l / 2
      rsrc_b = make_rsrc_words(reinterpret_cast<const char *>(a.B) + (int64_t)pn * BN * a.ldb, (uint32_t)(rows_b * a.ldb));
      voff_b = (uint32_t)((32 * wave + (lane >> 1)) * a.ldb + (lane & 1) * 16);
      grp_b = 0;
      kstep_b = 32;
    } else if (!B_KN) {
      rsrc_b = make_rsrc_words(a.B + (int64_t)pn * BN * a.ldb, (uint32_t)(rows_b * a.ldb * 2));
      voff_b = (uint32_t)(my_row * a.ldb + my_chunk * 8) * 2;
      grp_b = (uint32_t)(ROWS_PER_DMA * a.ldb * 2);
      kstep_b = BK * 2;
    } else {
      rsrc_b = make_rsrc_words(a.B + (int64_t)pn * BN, (uint32_t)(((int64_t)(a.K - 1) * a.ldb + rows_b) * 2));
      // this lane's K-row within the stage is B_ROWS_PER_DMA * (wave + x * NW) + row_in; its bits
      // 0..3 do not depend on x
      static_assert((B_ROWS_PER_DMA * NW) % 16 == 0, "swizzle bits of a lane's K-row must not depend on the load");
      const int row_in = (lane * 16) / B_ROW_BYTES, pos = ((lane * 16) % B_ROW_BYTES) / 16;
      const int k_bits = B_ROWS_PER_DMA * wave + row_in;
      const int chunk = pos ^ (4 * (k_bits & 3)) ^ (MFMA16 ? 2 * ((k_bits >> 3) & 1) : 0);
      voff_b = (chunk * 8 < rows_b) ? (uint32_t)(row_in * a.ldb + chunk * 8) * 2 : OOB_OFFSET;
      grp_b = (uint32_t)(B_ROWS_PER_DMA * a.ldb * 2);
      kstep_b = (uint32_t)(BK * a.ldb * 2);
    }

    // one wave-wide load of stage `st` for K-iteration kt: x < A_DMA loads rows of A, the rest B
    auto dma_one = [&](char *st, int kt, int x) {
      // the four-stage pipeline also issues the loads of iterations past the segment (the wait
      // counts stay uniform): they fetch nothing and fill a stage nobody reads with zeros
      const bool tail_oob = ((kt == tail_kt) && (kt * BK + my_chunk * 8 >= a.K)) || (NSTAGE == 4 && kt >= k0 + n);
      if (x < A_DMA) {
        const int g = wave + x * NW;
        dma_load_16(rsrc_a, lds_address(st) + g * 1024, tail_oob ? OOB_OFFSET : voff_a,
                    (uint32_t)kt * (BK * 2) + g * grp_a);
      } else {
        const int g = wave + (x - A_DMA) * NW;
        dma_load_16(rsrc_b, lds_address(st) + A_BYTES + g * 1024, (tail_oob && !B_KN) ? OOB_OFFSET : voff_b,
                    (uint32_t)kt * kstep_b + g * grp_b);
      }
    };
    auto issue_dma = [&](char *st, int kt) {
#pragma unroll
      for (int x = 0; x < DMA_PER_WAVE; ++x) dma_one(st, kt, x);
    };

    // fragment addressing: lane (r = lane%32, g = lane/32) reads row r of a 32-row block, logical
    // chunk 2*kk + g, stored at chunk position (2*kk + g) ^ ((r >> 1) & 7)
    // (BK = 32: swizzle (r >> 2) & 3)
    // (16x16x32: row lane%16, logical chunk 4*kk + lane/16, same swizzle)
    int rd_a[KSTEPS], rd_b[KSTEPS];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      const int chunk = MFMA16 ? 4 * kk + (lane >> 4) : 2 * kk + (lane >> 5);
      const int pos = (chunk ^ (BK == 64 ? (lane >> 1) & 7 : (lane >> 2) & 3)) * 16;
      rd_a[kk] = (wm * WTM + (lane & (FROWS - 1))) * ROW_BYTES + pos;
      rd_b[kk] = A_BYTES + (wn * WTN + (lane & (FROWS - 1))) * ROW_BYTES + pos;
    }
    // NN: per 32-column block j, the byte address of this lane's 8-byte piece in K-row
    // 8*(lane/32) + (lane%16)/4 of the stage; K-steps and the second half add row multiples
    // (16x16x32: lane group g = lane/16 reads K-rows 8g..8g+7 of a 16-column block.  Groups 0 and
    // 1 are served in the same cycle and read the same columns of K-rows 8 apart, so the swizzle
    // also flips chunk bit 1 with bit 3 of the K-row.)
    int rd_bt[FN];
    if (B_KN) {
      const int k_lane = MFMA16 ? 8 * (lane >> 4) + ((lane & 15) >> 2) : 8 * (lane >> 5) + ((lane & 15) >> 2);
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int col = MFMA16 ? wn * WTN + j * 16 + 4 * (lane & 3)
                               : wn * WTN + j * 32 + 16 * ((lane & 31) >> 4) + 4 * (lane & 3);
        const int chunk = (col >> 3) ^ (4 * (k_lane & 3)) ^ (MFMA16 ? 2 * ((k_lane >> 3) & 1) : 0);
        rd_bt[j] = A_BYTES + k_lane * B_ROW_BYTES + chunk * 16 + (col & 7) * 2;
      }
    }
    // 16x16x32: A fragments are double-buffered per half of the wave tile's rows (two half-steps per
    // K-step), which keeps accumulators + fragments + addresses within 256 registers
    constexpr int FA = MFMA16 ? FM / 2 : FM;
    half8v fa[2][FA], fb[2][FN];
    auto read_a16 = [&](const char *st, int buf, int kk, int mh) {
#pragma unroll
      for (int i = 0; i < FA; ++i)
        fa[buf][i] = *reinterpret_cast<const half8v *>(st + rd_a[kk] + (mh * FA + i) * FROWS * ROW_BYTES);
    };
    auto read_b16_one = [&](const char *st, int buf, int kk, int j) {
      if (!B_KN) {
        fb[buf][j] = *reinterpret_cast<const half8v *>(st + rd_b[kk] + j * FROWS * ROW_BYTES);
      } else {
        typedef short short4v __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) short4v *lds_s4;
        union { short4v s[2]; half8v h; } u;
        u.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(st + rd_bt[j] + (kk * 32) * B_ROW_BYTES));
        u.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(st + rd_bt[j] + (kk * 32 + 4) * B_ROW_BYTES));
        fb[buf][j] = u.h;
      }
    };
    auto read_b16 = [&](const char *st, int buf, int kk) {
#pragma unroll
      for (int j = 0; j < FN; ++j) read_b16_one(st, buf, kk, j);
    };
    auto mfma_one16 = [&](int abuf, int bbuf, int mh, int idx) {
      if constexpr (MFMA16) {
        const int i = idx / FN, j = idx % FN, ii = mh * FA + i;
        if constexpr (I8) {
          acc.v[ii][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, fb[bbuf][j]),
                                                               __builtin_bit_cast(intx4, fa[abuf][i]), acc.v[ii][j], 0, 0, 0);
        } else if constexpr (BF16_) {
          typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
          acc.v[ii][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fb[bbuf][j]),
                                                                 __builtin_bit_cast(bf16x8, fa[abuf][i]), acc.v[ii][j], 0, 0, 0);
        } else {
          acc.v[ii][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[bbuf][j], fa[abuf][i], acc.v[ii][j], 0, 0, 0);
        }
      }
    };
    auto mfma_half16 = [&](int abuf, int bbuf, int mh) {
#pragma unroll
      for (int idx = 0; idx < FA * FN; ++idx) mfma_one16(abuf, bbuf, mh, idx);
    };
    auto read_frags = [&](const char *st, int buf, int kk) {
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[buf][i] = *reinterpret_cast<const half8v *>(st + rd_a[kk] + i * FROWS * ROW_BYTES);
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if (!B_KN) {
          fb[buf][j] = *reinterpret_cast<const half8v *>(st + rd_b[kk] + j * FROWS * ROW_BYTES);
        } else {
          typedef short short4v __attribute__((ext_vector_type(4)));
          typedef __attribute__((address_space(3))) short4v *lds_s4;
          union { short4v s[2]; half8v h; } u;
          u.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(st + rd_bt[j] + (kk * 16) * B_ROW_BYTES));
          u.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(st + rd_bt[j] + (kk * 16 + 4) * B_ROW_BYTES));
          fb[buf][j] = u.h;
        }
      }
    };
    auto mfma_step = [&](int buf) {
      if constexpr (!MFMA16) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc.c[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[buf][j], fa[buf][i], acc.c[i][j], 0, 0, 0);
      }
    };
    // 16x16x32, the half-step behind the barrier, in DMA_PER_WAVE slices: each issues one load of
    // K-iteration kt_next into `cur`, its share of the first fragment reads of `nxt` (A into
    // fa[0], B into fb[bnext]) and its share of the MFMAs of the second half of the rows (fa[1],
    // fb[bcur]), so the matrix pipe does not run dry behind a block of load instructions.  No
    // branches: past the segment the loads get an out-of-range offset (they fetch nothing and zero
    // a stage nobody reads; drained after the loop) and the reads fetch fragments nobody uses.
    auto tail16 = [&](char *cur, const char *nxt, int kt_next, bool dead, int bcur, int bnext) {
      const bool oob = dead || (kt_next == tail_kt && kt_next * BK + my_chunk * 8 >= a.K);
      // (NN: the K tail of B is cut off by its descriptor, not per lane)
      const uint32_t va = oob ? OOB_OFFSET : voff_a, vb = (B_KN ? dead : oob) ? OOB_OFFSET : voff_b;
      constexpr int CH = DMA_PER_WAVE, NRD = FA + FN, NMF = FA * FN;
#pragma unroll
      for (int x = 0; x < CH; ++x) {
#pragma unroll
        for (int r = 0; r < NRD; ++r)
          if (r * CH / NRD == x) {
            if (r < FA)
              fa[0][r] = *reinterpret_cast<const half8v *>(nxt + rd_a[0] + r * FROWS * ROW_BYTES);
            else
              read_b16_one(nxt, bnext, 0, r - FA);
          }
        if (x < A_DMA) {
          const int g = wave + x * NW;
          dma_load_16(rsrc_a, lds_address(cur) + g * 1024, va, (uint32_t)kt_next * (BK * 2) + g * grp_a);
        } else {
          const int g = wave + (x - A_DMA) * NW;
          dma_load_16(rsrc_b, lds_address(cur) + A_BYTES + g * 1024, vb, (uint32_t)kt_next * kstep_b + g * grp_b);
        }
#pragma unroll
        for (int m = 0; m < NMF; ++m)
          if (m * CH / NMF == x) mfma_one16(1, bcur, 1, m);
      }
    };
    // fp8: 32-byte fragments, A double-buffered per half of the wave tile's rows, B per K-step
    typedef int intx8 __attribute__((ext_vector_type(8)));
    constexpr int FA8 = TM / 2 > 0 ? TM / 2 : 1;
    intx8 fa8[2][FA8], fb8[2][TN];
    auto read8 = [&](const char *p0, const char *p1) {
      union { uint4v q[2]; intx8 v; } u;
      u.q[0] = *reinterpret_cast<const uint4v *>(p0);
      u.q[1] = *reinterpret_cast<const uint4v *>(p1);
      return u.v;
    };
    auto read_a8_one = [&](const char *st, int buf, int s, int mh, int i) {
      const int off = (mh * FA8 + i) * 32 * ROW_BYTES;
      fa8[buf][i] = read8(st + rd_a[(2 * s) % KSTEPS] + off, st + rd_a[(2 * s + 1) % KSTEPS] + off);
    };
    auto read_b8_one = [&](const char *st, int buf, int s, int j) {
      const int off = j * 32 * ROW_BYTES;
      fb8[buf][j] = read8(st + rd_b[(2 * s) % KSTEPS] + off, st + rd_b[(2 * s + 1) % KSTEPS] + off);
    };
    auto read_a8 = [&](const char *st, int buf, int s, int mh) {
#pragma unroll
      for (int i = 0; i < FA8; ++i) read_a8_one(st, buf, s, mh, i);
    };
    auto read_b8 = [&](const char *st, int buf, int s) {
#pragma unroll
      for (int j = 0; j < TN; ++j) read_b8_one(st, buf, s, j);
    };
    auto mfma_one8 = [&](int abuf, int bbuf, int mh, int idx) {
      if constexpr (F8 != 0) {
        const int i = idx / TN, j = idx % TN, ii = mh * FA8 + i;
        acc.c[ii][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb8[bbuf][j], fa8[abuf][i], acc.c[ii][j], F8 - 1,
                                                                       F8 - 1, 0, 0, 0, 0);
      }
    };
    auto mfma_half8 = [&](int abuf, int bbuf, int mh) {
#pragma unroll
      for (int idx = 0; idx < FA8 * TN; ++idx) mfma_one8(abuf, bbuf, mh, idx);
    };
    // the half-step behind the barrier, sliced like tail16: loads of K-iteration kt_next into `cur`,
    // the first fragments of `nxt` (A into fa8[0], B into fb8[0]) and the MFMAs of (K-step 1, second
    // half of the rows)
    auto tail8 = [&](char *cur, const char *nxt, int kt_next, bool dead, int bcur = 1, int bnext = 0) {
      const bool oob = dead || (kt_next == tail_kt && kt_next * BK + my_chunk * 8 >= a.K);
      const uint32_t va = oob ? OOB_OFFSET : voff_a, vb = oob ? OOB_OFFSET : voff_b;
      constexpr int CH = DMA_PER_WAVE, NRD = FA8 + TN, NMF = FA8 * TN;
#pragma unroll
      for (int x = 0; x < CH; ++x) {
#pragma unroll
        for (int r = 0; r < NRD; ++r)
          if (r * CH / NRD == x) {
            if (r < FA8)
              read_a8_one(nxt, 0, 0, 0, r);
            else
              read_b8_one(nxt, bnext, 0, r - FA8);
          }
        if (x < A_DMA) {
          const int g = wave + x * NW;
          dma_load_16(rsrc_a, lds_address(cur) + g * 1024, va, (uint32_t)kt_next * (BK * 2) + g * grp_a);
        } else {
          const int g = wave + (x - A_DMA) * NW;
          dma_load_16(rsrc_b, lds_address(cur) + A_BYTES + g * 1024, vb, (uint32_t)kt_next * kstep_b + g * grp_b);
        }
#pragma unroll
        for (int m = 0; m < NMF; ++m)
          if (m * CH / NMF == x) mfma_one8(1, bcur, 1, m);
      }
    };
    if constexpr (F8 != 0 && NSTAGE == 4) {
      // BK = 32 (64 K-values) is one K-step: two half-steps per iteration, the four-stage schedule of the
      // 16x16x32 form below.  Entering, fa8[0] holds the first half of the A rows and fb8[par] the B
      // fragments of stage `cur` (par = iteration parity).
      auto iteration4 = [&](char *cur, char *nxt, int it, int par) {
        read_a8(cur, 1, 0, 1);
        mfma_half8(0, par, 0);
        interleave8<FA8 * TN, 2 * FA8>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<2 * DMA_PER_WAVE>();
        tail8(cur, nxt, k0 + it + 4, it + 4 >= n, par, par ^ 1);
      };
      char *s0 = stage(0), *s1 = stage(1), *s2 = stage(2), *s3 = stage(3);
      issue_dma(s0, k0);
      issue_dma(s1, k0 + 1);
      issue_dma(s2, k0 + 2);
      wait_dma_then_barrier<2 * DMA_PER_WAVE>();
      issue_dma(s3, k0 + 3);
      read_a8(s0, 0, 0, 0);
      read_b8(s0, 0, 0);
      int it = 0;
      for (; it + 3 < n; it += 4) {
        iteration4(s0, s1, it, 0);
        iteration4(s1, s2, it + 1, 1);
        iteration4(s2, s3, it + 2, 0);
        iteration4(s3, s0, it + 3, 1);
      }
      if (it < n) iteration4(s0, s1, it, 0);
      if (it + 1 < n) iteration4(s1, s2, it + 1, 1);
      if (it + 2 < n) iteration4(s2, s3, it + 2, 0);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if constexpr (F8 != 0) {
      // one K-iteration (128 K-values) on stage `cur`: two K-steps of 64, each in two halves of the
      // wave tile's rows.  Entering, fa8[0] / fb8[0] hold the fragments of (K-step 0, first half).
      auto iteration8 = [&](char *cur, char *nxt, int it) {
        read_a8(cur, 1, 0, 1);
        read_b8(cur, 1, 1);
        mfma_half8(0, 0, 0);
        interleave8<FA8 * TN, 2 * (FA8 + TN)>();
        read_a8(cur, 0, 1, 0);
        mfma_half8(1, 0, 1);
        interleave8<FA8 * TN, 2 * FA8>();
        read_a8(cur, 1, 1, 1);
        mfma_half8(0, 1, 0);
        interleave8<FA8 * TN, 2 * FA8>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<0>();
        tail8(cur, nxt, k0 + it + 2, it + 2 >= n);
      };
      char *s0 = stage(0), *s1 = stage(1);
      issue_dma(s0, k0);
      wait_dma_then_barrier<0>();
      if (n > 1) issue_dma(s1, k0 + 1);
      read_a8(s0, 0, 0, 0);
      read_b8(s0, 0, 0);
      int it = 0;
      for (; it + 1 < n; it += 2) {
        iteration8(s0, s1, it);
        iteration8(s1, s0, it + 1);
      }
      if (it < n) iteration8(s0, s1, it);
      // the empty loads of the last two iterations still write LDS
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if constexpr (NSTAGE == 4 && MFMA16) {
      // BK = 32 is one K-step: two half-steps per iteration.  Entering, fa[0] holds the first half
      // of the A rows and fb[par] the B fragments of stage `cur` (par = iteration parity).
      auto iteration4 = [&](char *cur, char *nxt, int it, int par) {
        read_a16(cur, 1, 0, 1);
        mfma_half16(0, par, 0);
        interleave16<FA, FN>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<2 * DMA_PER_WAVE>();
        tail16(cur, nxt, k0 + it + 4, it + 4 >= n, par, par ^ 1);
      };
      char *s0 = stage(0), *s1 = stage(1), *s2 = stage(2), *s3 = stage(3);
      issue_dma(s0, k0);
      issue_dma(s1, k0 + 1);
      issue_dma(s2, k0 + 2);
      wait_dma_then_barrier<2 * DMA_PER_WAVE>();
      issue_dma(s3, k0 + 3);
      read_a16(s0, 0, 0, 0);
      read_b16(s0, 0, 0);
      int it = 0;
      for (; it + 3 < n; it += 4) {
        iteration4(s0, s1, it, 0);
        iteration4(s1, s2, it + 1, 1);
        iteration4(s2, s3, it + 2, 0);
        iteration4(s3, s0, it + 3, 1);
      }
      if (it < n) iteration4(s0, s1, it, 0);
      if (it + 1 < n) iteration4(s1, s2, it + 1, 1);
      if (it + 2 < n) iteration4(s2, s3, it + 2, 0);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if constexpr (NSTAGE == 4) {
      // one K-iteration (two K-steps) on stage `cur`: the barrier in the middle retires the reads
      // of `cur` (it is refilled for iteration it+4 right away) and publishes stage `nxt`, whose
      // loads were issued three iterations ago -- two younger groups may still be in flight
      auto iteration4 = [&](char *cur, char *nxt, int it) {
        read_frags(cur, 1, 1);
        mfma_step(0);
#pragma unroll
        for (int g = 0; g < TM + TN; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<2 * DMA_PER_WAVE>();
        issue_dma(cur, k0 + it + 4);
        read_frags(nxt, 0, 0);
        mfma_step(1);
      };
      char *s0 = stage(0), *s1 = stage(1), *s2 = stage(2), *s3 = stage(3);
      issue_dma(s0, k0);
      issue_dma(s1, k0 + 1);
      issue_dma(s2, k0 + 2);
      wait_dma_then_barrier<2 * DMA_PER_WAVE>();
      issue_dma(s3, k0 + 3);
      read_frags(s0, 0, 0);
      int it = 0;
      for (; it + 3 < n; it += 4) {
        iteration4(s0, s1, it);
        iteration4(s1, s2, it + 1);
        iteration4(s2, s3, it + 2);
        iteration4(s3, s0, it + 3);
      }
      if (it < n) iteration4(s0, s1, it);
      if (it + 1 < n) iteration4(s1, s2, it + 1);
      if (it + 2 < n) iteration4(s2, s3, it + 2);
      // the (empty) loads of the iterations past the segment still write LDS: drain them before
      // the stages are handed to the epilogue / the next tile
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if constexpr (Q4_) {
      // ---- Q4 weights: the pipeline of the 16x16x32 fp16 kernel, B produced by a conversion step ----
      char *s0 = stage(0), *s1 = stage(1);
      char *raw0 = LdsArray<RAW_BYTES, 4>::get(), *raw1 = LdsArray<RAW_BYTES, 5>::get();
      const Q4Consts qc = q4_consts(a.zero);
      // this thread converts words [tid * Q4_WORDS, +Q4_WORDS) of the tile's BN x 8 words: one row's
      const int cv_row = (tid * Q4_WORDS) >> 3, cv_c0 = (tid * Q4_WORDS) & 7;
      const BufferRsrc rsrc_s = make_rsrc(a.scales + (int64_t)pn * BN * a.groups, (uint32_t)(rows_b * a.groups * 2));
      const uint32_t voff_s = (uint32_t)(cv_row * a.groups * 2);
      auto load_scale = [&](int kt) {  // the scale of this thread's row for K-iteration kt (zero past K or N)
        return __builtin_bit_cast(half_t, (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(
                                              rsrc_s, (kt * BK < a.K) ? voff_s : OOB_OFFSET, (uint32_t)(kt >> 1) * 2, 0));
      };
      auto raw_dma = [&](char *raw, int kt, bool dead) {
        if (wave < RAW_DMA)
          dma_load_16(rsrc_b, lds_address(raw) + wave * 1024, dead ? OOB_OFFSET : voff_b, (uint32_t)kt * kstep_b);
      };
      auto a_dma = [&](char *st, int kt, bool dead, int x) {
        const int g = wave + x * NW;
        dma_load_16(rsrc_a, lds_address(st) + g * 1024, dead ? OOB_OFFSET : voff_a, (uint32_t)kt * (BK * 2) + g * grp_a);
      };
      // word w of this thread: eight weights -> their 16-byte chunk of the B stage, in K order
      auto convert_word = [&](char *st, uint32_t word, int w, half_t scale) {
        union { half8v v; uint32_t u[4]; } d;
        d.v = dequant_word_q4(word, qc, half2v{scale, scale});
        uint4v o;  // (e0,e4)(e1,e5)(e2,e6)(e3,e7) -> (e0,e1)(e2,e3)(e4,e5)(e6,e7)
        o[0] = __builtin_amdgcn_perm(d.u[1], d.u[0], 0x05040100u);
        o[1] = __builtin_amdgcn_perm(d.u[3], d.u[2], 0x05040100u);
        o[2] = __builtin_amdgcn_perm(d.u[1], d.u[0], 0x07060302u);
        o[3] = __builtin_amdgcn_perm(d.u[3], d.u[2], 0x07060302u);
        *reinterpret_cast<uint4v *>(st + A_BYTES + cv_row * ROW_BYTES + (((cv_c0 + w) ^ ((cv_row >> 1) & 7)) * 16)) = o;
      };
      typedef uint32_t rawv __attribute__((ext_vector_type(Q4_WORDS)));
      auto read_raw = [&](const char *raw) {
        rawv r;
        if constexpr (Q4_WORDS == 1) r = rawv(*reinterpret_cast<const uint32_t *>(raw + tid * 4));
        else r = *reinterpret_cast<const rawv *>(raw + tid * (Q4_WORDS * 4));
        return r;
      };
      auto word_of = [&](const rawv &r, int w) {
        if constexpr (Q4_WORDS == 1) return (uint32_t)r;
        else return (uint32_t)r[w];
      };
      // the half-step behind the barrier: A loads of iteration kt_next into `cur`, nibble loads of iteration
      // kt_next + 1, conversion of iteration kt_next (raw_cv -> cur's B rows), first fragments of `nxt`, MFMAs
      auto tail_q4 = [&](char *cur, const char *nxt, const char *raw_cv, char *raw_ld, int kt_next, bool dead, bool dead1,
                         half_t scale) {
        constexpr int CH = A_DMA, NRD = FA + FN, NMF = FA * FN;
        const rawv words = read_raw(raw_cv);
#pragma unroll
        for (int x = 0; x < CH; ++x) {
#pragma unroll
          for (int r = 0; r < NRD; ++r)
            if (r * CH / NRD == x) {
              if (r < FA)
                fa[0][r] = *reinterpret_cast<const half8v *>(nxt + rd_a[0] + r * FROWS * ROW_BYTES);
              else
                read_b16_one(nxt, 0, 0, r - FA);
            }
          a_dma(cur, kt_next, dead, x);
          if (x == 0) raw_dma(raw_ld, kt_next + 1, dead1);
          if (x < Q4_WORDS) convert_word(cur, word_of(words, x), x, scale);
#pragma unroll
          for (int m = 0; m < NMF; ++m)
            if (m * CH / NMF == x) mfma_one16(1, 1, 1, m);
        }
      };
      half_t sc_next;  // scale for the conversion the next tail performs
      auto iteration_q4 = [&](char *cur, char *nxt, char *raw_cv, char *raw_ld, int it) {
        read_a16(cur, 1, 0, 1);
        read_b16(cur, 1, 1);
        mfma_half16(0, 0, 0);
        interleave16<FA + FN, FA * FN / (FA + FN)>();
        read_a16(cur, 0, 1, 0);
        mfma_half16(1, 0, 1);
        interleave16<FA, FN>();
        read_a16(cur, 1, 1, 1);
        mfma_half16(0, 1, 0);
        interleave16<FA, FN>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<0>();
        const half_t sc = sc_next;
        sc_next = load_scale(k0 + it + 3);
        tail_q4(cur, nxt, raw_cv, raw_ld, k0 + it + 2, it + 2 >= n, it + 3 >= n, sc);
      };
      // prologue: nibbles of the first two iterations and A of the first; convert both; then the loads that a
      // tail would have issued
      raw_dma(raw0, k0, false);
      raw_dma(raw1, k0 + 1, n < 2);
#pragma unroll
      for (int x = 0; x < A_DMA; ++x) a_dma(s0, k0, false, x);
      {
        const half_t sc0 = load_scale(k0), sc1 = load_scale(k0 + 1);
        sc_next = load_scale(k0 + 2);
        wait_dma_then_barrier<0>();
        const rawv w0 = read_raw(raw0), w1 = read_raw(raw1);
#pragma unroll
        for (int w = 0; w < Q4_WORDS; ++w) {
          convert_word(s0, word_of(w0, w), w, sc0);
          convert_word(s1, word_of(w1, w), w, sc1);
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      wait_dma_then_barrier<0>();
#pragma unroll
      for (int x = 0; x < A_DMA; ++x) a_dma(s1, k0 + 1, n < 2, x);
      raw_dma(raw0, k0 + 2, n < 3);
      read_a16(s0, 0, 0, 0);
      read_b16(s0, 0, 0);
      int it = 0;
      for (; it + 1 < n; it += 2) {
        iteration_q4(s0, s1, raw0, raw1, it);
        iteration_q4(s1, s0, raw1, raw0, it + 1);
      }
      if (it < n) iteration_q4(s0, s1, raw0, raw1, it);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if constexpr (MFMA16) {
      // one K-iteration on stage `cur`: two K-steps of 32, each in two halves of the wave tile's
      // rows.  Entering, fa[0] / fb[0] hold the fragments of (K-step 0, first half).
      auto iteration16 = [&](char *cur, char *nxt, int it) {
        // (hints: the reads are spread evenly over the MFMAs of a half-step.  Issuing them all at
        // its start is faster on all-zero operands and slower on random ones, where the power
        // limit sets the clock.)
        read_a16(cur, 1, 0, 1);
        read_b16(cur, 1, 1);
        mfma_half16(0, 0, 0);
        interleave16<FA + FN, FA * FN / (FA + FN)>();
        read_a16(cur, 0, 1, 0);
        mfma_half16(1, 0, 1);
        interleave16<FA, FN>();
        read_a16(cur, 1, 1, 1);
        mfma_half16(0, 1, 0);
        interleave16<FA, FN>();
        // every read of `cur` has been issued and has completed behind the MFMAs above
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<0>();
        tail16(cur, nxt, k0 + it + 2, it + 2 >= n, 1, 0);
      };
      char *s0 = stage(0), *s1 = stage(1);
      issue_dma(s0, k0);
      wait_dma_then_barrier<0>();
      if (n > 1) issue_dma(s1, k0 + 1);
      read_a16(s0, 0, 0, 0);
      read_b16(s0, 0, 0);
      int it = 0;
      for (; it + 1 < n; it += 2) {
        iteration16(s0, s1, it);
        iteration16(s1, s0, it + 1);
      }
      if (it < n) iteration16(s0, s1, it);
      // the empty loads of the last two iterations still write LDS
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
      // one K-iteration on stage `cur`; `more1`/`more2`: iterations it+1 / it+2 exist
      auto iteration = [&](char *cur, char *nxt, int it) {
#pragma unroll
        for (int kk = 0; kk < 3; ++kk) {
          read_frags(cur, (kk + 1) & 1, kk + 1);
          mfma_step(kk & 1);
#pragma unroll
          for (int g = 0; g < TM + TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          }
        }
        // every read of `cur` has been issued; they complete before the barrier below because the
        // MFMAs of step 3 (which need them) follow it -- make that explicit for the hardware:
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_dma_then_barrier<0>();
        if (it + 2 < n) issue_dma(cur, k0 + it + 2);
        if (it + 1 < n) read_frags(nxt, 0, 0);
        mfma_step(1);
      };

      char *s0 = stage(0), *s1 = stage(1);
      issue_dma(s0, k0);
      wait_dma_then_barrier<0>();
      if (n > 1) issue_dma(s1, k0 + 1);
      read_frags(s0, 0, 0);
      int it = 0;
      for (; it + 1 < n; it += 2) {
        iteration(s0, s1, it);
        iteration(s1, s0, it + 1);
      }
      if (it < n) iteration(s0, s1, it);
      // all LDS reads are complete and every wave has passed the last barrier only after finishing
      // its reads of the other stage; one more barrier frees both stages for the epilogue / next tile
    }
    __syncthreads();
  }

  // two copies of the epilogue behind one uniform branch: the one without a bias is the code the kernel had
  // before the bias existed (bias loads inside a single epilogue cost the 256x256 kernel 6 % at 8192^3)
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int pm, int pn, char *smem,
                                                 const void *bias) {
    if (bias == nullptr)
      store_c_impl<false, -1>(a, acc, pm, pn, smem, nullptr);
    else
      store_c_impl<true, -1>(a, acc, pm, pn, smem, bias);
  }
  // Half h of the tile, in the sense of the halves fix-up: the rows of every wave's block that live in the
  // first (h = 0) or second (h = 1) half of that wave's accumulators.
  static __device__ __forceinline__ void store_c_half(const Args &a, const Acc &acc, int pm, int pn, char *smem,
                                                      const void *bias, int h) {
    if constexpr (HALVES) {
      if (bias == nullptr) {
        if (h == 0) store_c_impl<false, 0>(a, acc, pm, pn, smem, nullptr);
        else store_c_impl<false, 1>(a, acc, pm, pn, smem, nullptr);
      } else {
        if (h == 0) store_c_impl<true, 0>(a, acc, pm, pn, smem, bias);
        else store_c_impl<true, 1>(a, acc, pm, pn, smem, bias);
      }
    }
  }
  // HALF < 0: the whole tile; 0 / 1: rows [HALF * WTM / 2, (HALF + 1) * WTM / 2) of every wave's block
  template <bool BIAS, int HALF>
  static __device__ __forceinline__ void store_c_impl(const Args &a, const Acc &acc, int pm, int pn, char *,
                                                      const void *epi) {
    constexpr int ROW_BEGIN = HALF < 0 ? 0 : HALF * (WTM / 2), NROWS = HALF < 0 ? WTM : WTM / 2;
    constexpr int PR = PATCH_ROWS < NROWS ? PATCH_ROWS : NROWS;  // rows of the wave's block per pass
    constexpr int NPASS = NROWS / PR;
    const half_t *bias = BIAS ? epi_bias(epi) : nullptr;
    const int act = BIAS ? epi_act(epi) : 0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    if constexpr (I8) {
      // int32 C straight from the accumulators: lane l of block (ii, jj) holds row 16*ii + l%16, columns
      // 16*jj + 4*(l/16) .. +3
      int *C = reinterpret_cast<int *>(a.C);
      const bool vec_ok = (a.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 15) == 0);
      const int row0 = pm * BM + wm * WTM + (lane & 15), col0 = pn * BN + wn * WTN + 4 * (lane >> 4);
#pragma unroll
      for (int ii = ROW_BEGIN / 16; ii < (ROW_BEGIN + NROWS) / 16; ++ii)
#pragma unroll
        for (int jj = 0; jj < FN; ++jj) {
          const int grow = row0 + 16 * ii, gcol = col0 + 16 * jj;
          if (grow < a.M && gcol < a.N) {
            int *dst = C + (int64_t)grow * a.ldc + gcol;
            if (vec_ok && gcol + 4 <= a.N) {
              *reinterpret_cast<intx4 *>(dst) = acc.v[ii][jj];
            } else {
              for (int e = 0; e < 4 && gcol + e < a.N; ++e) dst[e] = acc.v[ii][jj][e];
            }
          }
        }
      return;
    }
    // first column of this lane's accumulator groups, for the bias; computed here, from a value the compiler cannot
    // see through, so that it is not hoisted out of the persistent loop and kept in a register across the main loop
    const int bias_col0 = BIAS ? pn * BN + wn * WTN + pin_here(lane >> (MFMA16 ? 4 : 5)) * 4 : 0;
    half_t *patch = reinterpret_cast<half_t *>(stage(wave / WAVES_PER_STAGE)) +
                    (wave % WAVES_PER_STAGE) * (PATCH_ROWS * LDC);
    const bool vec_ok = (a.ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 15) == 0);
    constexpr int CPRC = WTN / 8;
    constexpr int BLK = PR / 32;  // 32-row blocks per pass
    static_assert(MFMA16 ? PR % 16 == 0 : PR % 32 == 0, "an epilogue pass holds whole accumulator blocks");
    static_for<0, NPASS>([&](auto pass) {
      constexpr int p = decltype(pass)::value;
      if constexpr (I8) {
      } else if constexpr (MFMA16) {
#pragma unroll
        for (int ib = 0; ib < PR / 16; ++ib)
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            half4v h;
            floatx4 bv = {0.f, 0.f, 0.f, 0.f};
            if constexpr (BIAS) bv = bias4_at<BF16_>(bias, bias_col0 + j * 16, a.N);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float x = acc.v[ROW_BEGIN / 16 + p * (PR / 16) + ib][j][e];
              if constexpr (BIAS) x = activate(x + bv[e], act);
              if constexpr (BF16_) {
                const __bf16 b = (__bf16)x;
                h[e] = __builtin_bit_cast(half_t, b);  // the patch only carries 16-bit patterns
              } else {
                h[e] = (half_t)x;
              }
            }
            *reinterpret_cast<half4v *>(patch + (ib * 16 + (lane & 15)) * LDC + j * 16 + (lane >> 4) * 4) = h;
          }
      } else {
#pragma unroll
        for (int ib = 0; ib < BLK; ++ib)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              half4v h;
              floatx4 bv = {0.f, 0.f, 0.f, 0.f};
              if constexpr (BIAS) bv = bias4_at(bias, bias_col0 + j * 32 + q * 8, a.N);
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float x = acc.c[ROW_BEGIN / 32 + p * BLK + ib][j][q * 4 + e];
                if constexpr (F8 != 0) x *= a.alpha;  // the product of fp8 operands is scaled before it is rounded to fp16
                if constexpr (BIAS) x = activate(x + bv[e], act);
                h[e] = (half_t)x;
              }
              *reinterpret_cast<half4v *>(patch + (ib * 32 + (lane & 31)) * LDC + j * 32 + q * 8 +
                                          (lane >> 5) * 4) = h;
            }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int row0 = pm * BM + wm * WTM + ROW_BEGIN + p * PR, col0 = pn * BN + wn * WTN;
#pragma unroll
      for (int s = 0; s < PR * CPRC / 64; ++s) {
        const int idx = s * 64 + lane;
        const int r = idx / CPRC, cc = idx % CPRC;
        const int grow = row0 + r, gcol = col0 + cc * 8;
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
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    });
    __syncthreads();  // patches overlap the stages of the next tile
  }

  static constexpr bool COHERENT_PARTIALS = false;
  // The 16x16x32 forms exchange the partial tiles of the REDUCE fix-up with 16-byte device-scope accesses:
  // stores write through, loads bypass stale lines, and no CTA pays a write-back or invalidate of its XCD's
  // whole L2 (which, with 16 CTAs per XCD finishing at the same moment, cost more than the exchange itself).
  static constexpr bool COHERENT_REDUCE = MFMA16_;
  // both CTAs of a tile cut in two finish half of it each (see run_persistent); needs accumulator blocks of
  // 16 rows and at least two of them per wave
  static constexpr bool HALVES = MFMA16_ && FM % 2 == 0;
  // the reference's fix-up: partial sums rounded to C's type and added into C (fp16 / bfloat16, 16x16 blocks)
  static constexpr bool ATOMIC_C = MFMA16_ && F8_ == 0 && !Q4_;
  static __device__ __forceinline__ void atomic_c(const Args &a, const Acc &acc, int pm, int pn) {
    if constexpr (ATOMIC_C) {
      // lane l of block (ii, jj) holds row 16 ii + l % 16, columns 16 jj + 4 (l / 16) .. + 3 of the wave tile
      const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      const int wm = wave / WN, wn = wave % WN;
      const int row0 = pm * BM + wm * WTM + (lane & 15), col0 = pn * BN + wn * WTN + 4 * (lane >> 4);
#pragma unroll
      for (int ii = 0; ii < FM; ++ii)
#pragma unroll
        for (int jj = 0; jj < FN; ++jj) {
          const int grow = row0 + 16 * ii, gcol = col0 + 16 * jj;
          if (grow < a.M && gcol < a.N) {  // (N is even: a pair never straddles the edge)
            half_t *p = a.C + (int64_t)grow * a.ldc + gcol;
            atomic_add_pair16<BF16_>(p, acc.v[ii][jj][0], acc.v[ii][jj][1]);
            if (gcol + 2 < a.N) atomic_add_pair16<BF16_>(p + 2, acc.v[ii][jj][2], acc.v[ii][jj][3]);
          }
        }
    }
  }
  // partials in the workspace: float4 group v of thread t at (v * NT + t) * 4 (ordered reduce),
  // element s of thread t at s * NT + t (atomic accumulation buffer); see tile_f16.h
  template <int V0, int V1>
  static __device__ __forceinline__ void store_groups(const Acc &acc, float *dst) {
    if constexpr (MFMA16) {
      const BufferRsrc r = make_rsrc(dst, TILE_ELEMS * 4);
      const uint32_t off = (uint32_t)pin_here((int)threadIdx.x) * 16;
#pragma unroll
      for (int v = V0; v < V1; ++v)
        st_coherent16(r, off, (uint32_t)v * NT * 16, __builtin_bit_cast(uint4v, acc.v[v / FN][v % FN]));
    }
  }
  template <int V0, int V1>
  static __device__ __forceinline__ void add_groups(Acc &acc, const float *src) {
    if constexpr (MFMA16) {
      const BufferRsrc r = make_rsrc(src, TILE_ELEMS * 4);
      const uint32_t off = (uint32_t)pin_here((int)threadIdx.x) * 16;
#pragma unroll
      for (int v = V0; v < V1; ++v) {
        acc.v[v / FN][v % FN] += __builtin_bit_cast(AccV, ld_coherent16(r, off, (uint32_t)v * NT * 16));
        if (v % 8 == 7) asm volatile("" ::: "memory");  // at most 8 loads in flight
      }
    }
  }
  static __device__ __forceinline__ void store_partial(const Acc &acc, float *dst) {
    if constexpr (MFMA16) {
      store_groups<0, NV4>(acc, dst);
    } else {
      Base::store_partial(acc, dst);
    }
  }
  static __device__ __forceinline__ void add_partial(Acc &acc, const float *src) {
    if constexpr (MFMA16) {
      add_groups<0, NV4>(acc, src);
    } else {
      Base::add_partial(acc, src);
    }
  }
  // half h of the accumulators: blocks [h * FM / 2, (h + 1) * FM / 2), i.e. groups [h * NV4 / 2, (h + 1) * NV4 / 2)
  static __device__ __forceinline__ void store_partial_half(const Acc &acc, float *dst, int h) {
    if (h == 0) store_groups<0, NV4 / 2>(acc, dst);
    else store_groups<NV4 / 2, NV4>(acc, dst);
  }
  static __device__ __forceinline__ void add_partial_half(Acc &acc, const float *src, int h) {
    if (h == 0) add_groups<0, NV4 / 2>(acc, src);
    else add_groups<NV4 / 2, NV4>(acc, src);
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst) {
    if constexpr (MFMA16) {
      dst = pin_here(dst);
#pragma unroll
      for (int v = 0; v < NV4; ++v)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (I8)
            atomic_add_i32(reinterpret_cast<int *>(dst) + (size_t)(v * 4 + e) * NT + threadIdx.x, acc.v[v / FN][v % FN][e]);
          else
            atomic_add_f32(dst + (size_t)(v * 4 + e) * NT + threadIdx.x, acc.v[v / FN][v % FN][e]);
        }
    } else {
      Base::atomic_partial(acc, dst);
    }
  }
  static __device__ __forceinline__ void take_partial(Acc &acc, float *src) {
    if constexpr (MFMA16) {
      src = pin_here(src);
#pragma unroll
      for (int v = 0; v < NV4; ++v) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float *p = src + (size_t)(v * 4 + e) * NT + threadIdx.x;
          if constexpr (I8)
            acc.v[v / FN][v % FN][e] = *reinterpret_cast<int *>(p);
          else
            acc.v[v / FN][v % FN][e] = *p;
          *p = 0.f;
        }
        if (v % 4 == 3) asm volatile("" ::: "memory");
      }
    } else {
      Base::take_partial(acc, src);
    }
  }
};

}  // namespace sk
