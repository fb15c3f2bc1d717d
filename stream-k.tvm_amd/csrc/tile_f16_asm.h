// fp16 / bfloat16 NT tile arithmetic, 256 x 256 x 64 CTA tile on FOUR waves (2 x 2), each owning a 128 x 128
// block of C: 256 fp32 accumulators per lane, kept in the accumulation registers a[0:255] from the first MFMA
// of a segment to the store of C.  A wave tile of 128 x 128 reads a third fewer LDS bytes per FLOP than the
// 128 x 64 blocks of the eight-wave kernel (tile_f16_dma.h), and on a part whose matrix clock is set by the
// power drawn, bytes moved are clock.
//
// The data movement is that of tile_f16_dma.h (direct global -> LDS loads of 16 bytes per lane, LDS rows of 128
// bytes with chunk c of row r at position c ^ ((r >> 1) & 7), two stages of 64 KB, fragments for
// v_mfma_f32_16x16x32_f16 read with ds_read_b128; replaces the reference's inner MAC, streamk_fp16.py:196-240).
// The K loop itself is one block of assembly with fixed registers (gen_tile_asm.py writes it, with the register
// plan and the schedule): the compiler does not keep 256 accumulators in one register file while it schedules
// the loop around them.  Everything else -- addressing, fix-up, epilogue -- is ordinary code that reaches the
// accumulators four at a time through v_accvgpr_read_b32 / v_accvgpr_write_b32.  The compiler itself must not
// touch the accumulation registers between those statements: the kernels of this policy contain no other MFMA
// and stay far below 256 architectural registers, so it has no reason to (the build checks the generated
// assembly for accumulation-register instructions outside the hand-written blocks).
//
// NN_ (B is [K, N] row-major): the B half of a stage holds 64 K-rows of 512 bytes, swizzled and read with
// transposing 8-byte LDS reads as in the NN form of tile_f16_dma.h; see gen_tile_asm.py for the loop's side.
//
// Restrictions: K a multiple of 64 (int8: NT only, K a multiple of 128 bytes).
#pragma once
#include "sk_device.h"
#include "tile_f16.h"
#include "tile_f16_asm_gen.h"

namespace sk {

// accumulators a[R .. R+3] <-> four floats
template <int R>
__device__ __forceinline__ floatx4 agpr_read4() {
  float x0, x1, x2, x3;
  asm volatile(
      "v_accvgpr_read_b32 %0, a[%4]\n\tv_accvgpr_read_b32 %1, a[%5]\n\t"
      "v_accvgpr_read_b32 %2, a[%6]\n\tv_accvgpr_read_b32 %3, a[%7]"
      : "=v"(x0), "=v"(x1), "=v"(x2), "=v"(x3)
      : "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
  return floatx4{x0, x1, x2, x3};
}
template <int R>
__device__ __forceinline__ void agpr_write4(floatx4 x) {
  asm volatile(
      "v_accvgpr_write_b32 a[%4], %0\n\tv_accvgpr_write_b32 a[%5], %1\n\t"
      "v_accvgpr_write_b32 a[%6], %2\n\tv_accvgpr_write_b32 a[%7], %3"
      :
      : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "n"(R), "n"(R + 1), "n"(R + 2), "n"(R + 3));
}

// MODE_: 0 fp16, 1 bfloat16, 2 int8 (int32 C; the bytes travel as pairs, so K and the leading dimensions of A
// and B arrive in 16-bit units and the loop is the fp16 one with v_mfma_i32_16x16x64_i8 on the same fragments),
// 3 / 4 fp8 e4m3 / e5m2 (fp16 C scaled by alpha; bytes as pairs again, one v_mfma_f32_16x16x128_f8f6f4 per block
// and iteration in a two-phase loop of its own, see gen_tile_asm.py)
template <int MODE_ = 0, bool NN_ = false>
struct TileF16Asm {
  static_assert(!(NN_ && MODE_ >= 2), "one-byte operands: NT layout only");
  typedef GemmArgs Args;
  static constexpr bool BF16_ = MODE_ == 1, I8 = MODE_ == 2;
  static constexpr int F8 = MODE_ >= 3 ? MODE_ - 2 : 0;  // 1: e4m3, 2: e5m2
  typedef int intx4 __attribute__((ext_vector_type(4)));
  static constexpr bool LEAN_ENTRY = true;  // see run_persistent
  static constexpr int BM = 256, BN = 256, BK = 64, WM = 2, WN = 2, NW = 4, NT = 256;
  static constexpr int WTM = 128, WTN = 128, FM = 8, FN = 8;  // wave tile; 16 x 16 accumulator blocks per wave
  static constexpr int ROW_BYTES = 128, A_BYTES = BM * ROW_BYTES, STAGE_BYTES = 2 * A_BYTES;
  // behind the two stages: one patch of 16 rows x 272 bytes per wave for the epilogue that leaves the stages alone
  static constexpr int PATCH_STRIDE = 272, FAST_PATCH_BYTES = 16 * PATCH_STRIDE;
  static constexpr int LDS_TOTAL = 2 * STAGE_BYTES + NW * FAST_PATCH_BYTES, LDS_BYTES = 16;
  static constexpr int TILE_ELEMS = BM * BN, NV4 = FM * FN;
  static constexpr int CTAS_PER_CU = 1, WAVES_PER_EU = 1;
  static constexpr int LDC = WTN + 8, PATCH_ROWS = 64;  // epilogue patch: 64 rows x 136 halfs per wave and pass
  static_assert(PATCH_ROWS * LDC * 2 <= 2 * STAGE_BYTES / NW, "epilogue patches must fit the stages");

  struct Acc {};  // the accumulators live in a[0:255]: block (i, j) in a[(8 i + j) 4 .. + 3]

  static __device__ __forceinline__ char *lds() {
    __shared__ __attribute__((aligned(1024))) char buf[LDS_TOTAL];
    return buf;
  }

  // Everything the loads and the loop of one segment need: descriptors, lane offsets, wave-uniform global offsets
  // (iteration k0 of tile (pm, pn)), LDS addresses.
  struct Ctx {
    uint4v rsrc_a, rsrc_b;
    uint32_t voff_a, voff_b, voff_b1;  // voff_b1: NN only (odd row groups of B)
    uint32_t goff_a, goff_b, gstep_a, gstep_b, kstep_b;  // kstep_b: bytes B advances per iteration
    uint32_t lds_wave;
    uint32_t ra0, ra1, rb0, rb1, rbt[8];  // fragment addresses (rbt: NN)
  };
  static __device__ __forceinline__ Ctx make_ctx(const Args &a, int pm, int pn, int k0) {
    Ctx c;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int rows_a = min(BM, a.M - pm * BM), rows_b = min(BN, a.N - pn * BN);
    // rows past the matrix edge lie beyond the descriptors' ranges and read as zero
    c.rsrc_a = make_rsrc_words(a.A + (int64_t)pm * BM * a.lda, (uint32_t)(rows_a * a.lda * 2));
    // a wave-wide load fills 8 LDS rows; lane l writes (row l / 8, position l % 8) and therefore fetches
    // chunk (l % 8) ^ swizzle(row); a wave only loads row groups of its own parity (see tile_f16_dma.h)
    const int my_chunk = (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4)), my_row = lane >> 3;
    c.voff_a = (uint32_t)(my_row * a.lda + my_chunk * 8) * 2;
    // row group g = wave + 4 x of a stage: rows 8 g .. 8 g + 7, at wave-uniform byte offset 16 g ld
    c.goff_a = (uint32_t)k0 * (BK * 2) + (uint32_t)(wave * 16 * a.lda);
    c.gstep_a = (uint32_t)(64 * a.lda);
    const uint32_t base = lds_address(lds());
    c.lds_wave = base + wave * 1024;
    // fragments: lane (r = l % 16, g = l / 16) reads row r of a 16-row block, chunk 4 kk + g at position
    // (4 kk + g) ^ ((r >> 1) & 7); K-step 1 is K-step 0 with address bit 6 flipped
    const uint32_t pos0 = (uint32_t)((lane >> 4) ^ ((lane >> 1) & 7)) * 16;
    c.ra0 = base + (uint32_t)(wm * WTM + (lane & 15)) * ROW_BYTES + pos0;
    c.ra1 = c.ra0 ^ 64;
    if constexpr (NN_) {
      // B: the descriptor starts at the tile's first column and ends with the last valid element of row K - 1;
      // columns past N are masked per lane (N is a multiple of 8).  A wave-wide load fills K-rows 2 g, 2 g + 1 of
      // the stage (g = wave + 4 x): lane l writes position l % 32 of row 2 g + l / 32 and therefore fetches chunk
      // (l % 32) ^ swizzle(row); bit 3 of the row is the parity of x, hence two offsets.
      c.rsrc_b = make_rsrc_words(a.B + (int64_t)pn * BN, (uint32_t)(((int64_t)(a.K - 1) * a.ldb + rows_b) * 2));
      const int row_in = lane >> 5, k_bits = 2 * wave + row_in;
      const int chunk0 = (lane & 31) ^ (4 * (k_bits & 3)), chunk1 = chunk0 ^ 2;
      c.voff_b = chunk0 * 8 < rows_b ? (uint32_t)(row_in * a.ldb + chunk0 * 8) * 2 : OOB_OFFSET;
      c.voff_b1 = chunk1 * 8 < rows_b ? (uint32_t)(row_in * a.ldb + chunk1 * 8) * 2 : OOB_OFFSET;
      c.kstep_b = (uint32_t)(128 * a.ldb);  // 64 K-rows
      c.goff_b = (uint32_t)k0 * c.kstep_b + (uint32_t)(wave * 4 * a.ldb);
      c.gstep_b = (uint32_t)(16 * a.ldb);
      // fragments of B: lane group g' = l / 16 reads K-rows 8 g' .. 8 g' + 7 of a 16-column block, four rows per
      // transposing read; block j's address differs from block 0's by an XOR (the swizzle), so each has its own
      const int k_lane = 8 * (lane >> 4) + ((lane & 15) >> 2);
      const int swz = (4 * (k_lane & 3)) ^ (2 * ((k_lane >> 3) & 1));
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int col = wn * WTN + j * 16 + 4 * (lane & 3);
        c.rbt[j] = base + A_BYTES + (uint32_t)(k_lane * 512 + (((col >> 3) ^ swz) * 16) + (col & 7) * 2);
      }
      c.rb0 = c.rb1 = 0;
    } else {
      c.rsrc_b = make_rsrc_words(a.B + (int64_t)pn * BN * a.ldb, (uint32_t)(rows_b * a.ldb * 2));
      c.voff_b = (uint32_t)(my_row * a.ldb + my_chunk * 8) * 2;
      c.voff_b1 = 0;
      c.kstep_b = 128;
      c.goff_b = (uint32_t)k0 * (BK * 2) + (uint32_t)(wave * 16 * a.ldb);
      c.gstep_b = (uint32_t)(64 * a.ldb);
      c.rb0 = base + A_BYTES + (uint32_t)(wn * WTN + (lane & 15)) * ROW_BYTES + pos0;
      c.rb1 = c.rb0 ^ 64;
    }
    return c;
  }

  // the 16 loads of stage `stage` (iteration k0 + stage of the segment; nothing is fetched if the segment is shorter),
  // or -- EARLY_ONLY -- just those the loop does not send itself: the row groups that hold blocks 0-3 of the wave tiles
  // (NN: and all of B); see gen_tile_asm.py
  template <bool EARLY_ONLY = false>
  static __device__ __forceinline__ void stage_loads(const Ctx &c, int stage, int n) {
    const uint32_t oob = stage < n ? 0u : OOB_OFFSET;
    const uint32_t voa = c.voff_a | oob, vob = c.voff_b | oob, vob1 = c.voff_b1 | oob;
    const uint32_t ga = c.goff_a + (uint32_t)stage * 128, gb = c.goff_b + (uint32_t)stage * c.kstep_b;
    const uint32_t lds_stage = c.lds_wave + (uint32_t)stage * STAGE_BYTES;
#define SK_ASM_LOAD_OPERANDS                                                                                             \
  : : [rsa] "s"(c.rsrc_a), [rsb] "s"(c.rsrc_b), [voa] "v"(voa), [vob] "v"(vob), [vob1] "v"(vob1), [ga] "s"(ga),            \
      [gb] "s"(gb), [gas] "s"(c.gstep_a), [gas2] "s"(2 * c.gstep_a), [gas3] "s"(3 * c.gstep_a), [gbs] "s"(c.gstep_b),     \
      [gbs2] "s"(2 * c.gstep_b), [gbs3] "s"(3 * c.gstep_b), [lds] "s"(lds_stage)                                          \
  : "memory", "m0", "scc", "s83"
    if constexpr (NN_ && EARLY_ONLY) {
      asm volatile(SK_TILE_ASM_LOADS_EARLY_NN SK_ASM_LOAD_OPERANDS);
    } else if constexpr (NN_) {
      asm volatile(SK_TILE_ASM_LOADS_NN SK_ASM_LOAD_OPERANDS);
    } else if constexpr (EARLY_ONLY) {
      asm volatile(SK_TILE_ASM_LOADS_EARLY SK_ASM_LOAD_OPERANDS);
    } else {
      asm volatile(SK_TILE_ASM_LOADS SK_ASM_LOAD_OPERANDS);
    }
#undef SK_ASM_LOAD_OPERANDS
  }

  // Cross-segment prefetch (see run_persistent): the first stage of the NEXT segment is requested as soon as every
  // wave has left the loop of the current one, ahead of an epilogue that does not use LDS, and mac() is then told
  // that the stage is on its way.
  static constexpr bool CROSS_TILE_PREFETCH = true;
  static __device__ __forceinline__ void prefetch_first_stage(const Args &a, int pm, int pn, int k0, int n) {
    const Ctx c = make_ctx(a, pm, pn, k0);
    stage_loads(c, 0, n);
  }

  static __device__ __forceinline__ void mac(const Args &a, Acc &, int pm, int pn, int k0, int n, char *,
                                             bool first_stage_requested = false) {
    Ctx c = make_ctx(a, pm, pn, k0);
    if (!first_stage_requested) stage_loads(c, 0, n);
    // (directly ahead of the loop, whose first wait counts on these being the youngest operations; the 16-bit loops
    // send the late row groups of the second stage themselves)
    stage_loads<F8 == 0>(c, 1, n);
    const uint32_t iters = (uint32_t)n;
    if constexpr (NN_) {
#define SK_ASM_NN_OPERANDS                                                                                            \
  : [ra0] "+v"(c.ra0), [ra1] "+v"(c.ra1), [rbt0] "+v"(c.rbt[0]), [rbt1] "+v"(c.rbt[1]), [rbt2] "+v"(c.rbt[2]),          \
    [rbt3] "+v"(c.rbt[3]), [rbt4] "+v"(c.rbt[4]), [rbt5] "+v"(c.rbt[5]), [rbt6] "+v"(c.rbt[6]), [rbt7] "+v"(c.rbt[7])  \
  : [rsa] "s"(c.rsrc_a), [rsb] "s"(c.rsrc_b), [voa] "v"(c.voff_a), [vob] "v"(c.voff_b), [vob1] "v"(c.voff_b1),          \
    [ga0] "s"(c.goff_a), [gb0] "s"(c.goff_b), [gas] "s"(c.gstep_a), [gas2] "s"(2 * c.gstep_a),                          \
    [gas3] "s"(3 * c.gstep_a), [gbs] "s"(c.gstep_b), [kbs] "s"(c.kstep_b), [n] "s"(iters), [lds] "s"(c.lds_wave)        \
  : "memory", "m0", "scc", SK_TILE_ASM_CLOBBERS
      if constexpr (BF16_) {
        asm volatile(SK_TILE_ASM_LOOP_NN("v_mfma_f32_16x16x32_bf16") SK_ASM_NN_OPERANDS);
      } else {
        asm volatile(SK_TILE_ASM_LOOP_NN("v_mfma_f32_16x16x32_f16") SK_ASM_NN_OPERANDS);
      }
#undef SK_ASM_NN_OPERANDS
    } else {
#define SK_ASM_NT_OPERANDS                                                                                          \
  : [ra0] "+v"(c.ra0), [ra1] "+v"(c.ra1), [rb0] "+v"(c.rb0), [rb1] "+v"(c.rb1)                                      \
  : [rsa] "s"(c.rsrc_a), [rsb] "s"(c.rsrc_b), [voa] "v"(c.voff_a), [vob] "v"(c.voff_b), [ga0] "s"(c.goff_a),          \
    [gb0] "s"(c.goff_b), [gas] "s"(c.gstep_a), [gas2] "s"(2 * c.gstep_a), [gas3] "s"(3 * c.gstep_a),                  \
    [gbs] "s"(c.gstep_b), [gbs2] "s"(2 * c.gstep_b), [gbs3] "s"(3 * c.gstep_b), [n] "s"(iters), [lds] "s"(c.lds_wave)  \
  : "memory", "m0", "scc", SK_TILE_ASM_CLOBBERS
      if constexpr (F8 == 1) {
        asm volatile(SK_TILE_ASM_LOOP_F8("v_mfma_f32_16x16x128_f8f6f4", "") SK_ASM_NT_OPERANDS);
      } else if constexpr (F8 == 2) {
        asm volatile(SK_TILE_ASM_LOOP_F8("v_mfma_f32_16x16x128_f8f6f4", "cbsz:1 blgp:1") SK_ASM_NT_OPERANDS);
      } else if constexpr (I8) {
        asm volatile(SK_TILE_ASM_LOOP("v_mfma_i32_16x16x64_i8") SK_ASM_NT_OPERANDS);
      } else if constexpr (BF16_) {
        asm volatile(SK_TILE_ASM_LOOP("v_mfma_f32_16x16x32_bf16") SK_ASM_NT_OPERANDS);
      } else {
        asm volatile(SK_TILE_ASM_LOOP("v_mfma_f32_16x16x32_f16") SK_ASM_NT_OPERANDS);
      }
#undef SK_ASM_NT_OPERANDS
    }
    // every wave has left the loop and its own loads have landed: both stages are free (for the epilogue's patches,
    // for the loads of the next segment)
    __syncthreads();
  }

  // ---- epilogue that leaves the stages alone (patches of their own behind them; gen_tile_asm.py: store_text) ----
  // Possible where the tile's 256 columns are inside the matrix and rows of C are 16-byte aligned; rows past M are
  // dropped by the descriptor's range.  The bias / activation epilogue and tiles on the right edge take the path below.
  static __device__ __forceinline__ bool direct_store_ok(const Args &a, int pn, const void *bias) {
    if constexpr (I8) return false;  // (its own register epilogue, below)
    return bias == nullptr && (pn + 1) * BN <= a.N && (a.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(a.C) & 15) == 0;
  }
  // true if the epilogue of this tile will not touch the stages (the int32 epilogue uses no LDS at all)
  static __device__ __forceinline__ bool epilogue_lds_free(const Args &a, int pn, const void *bias) {
    return I8 || direct_store_ok(a, pn, bias);
  }
  template <int HALF>
  static __device__ __forceinline__ void store_c_direct(const Args &a, int pm, int pn) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int row0 = pm * BM + wm * WTM, col0 = pn * BN + wn * WTN;
    const int rows = max(0, min(WTM, a.M - row0));
    const uint32_t bytes = rows > 0 ? (uint32_t)(((int64_t)(rows - 1) * a.ldc + WTN) * 2) : 0u;
    const uint4v words = make_rsrc_words(a.C + (int64_t)row0 * a.ldc + col0, bytes);
    const uint4v rsrc_c = uniform_rsrc(words);  // (it depends on the wave's index)
    const uint32_t patch = lds_address(lds()) + 2 * STAGE_BYTES + (uint32_t)wave * FAST_PATCH_BYTES;
    const uint32_t wr = patch + (uint32_t)((lane & 15) * PATCH_STRIDE + (lane >> 4) * 8);
    const uint32_t rd = patch + (uint32_t)((lane >> 4) * PATCH_STRIDE + (lane & 15) * 16);
    const uint32_t voff = (uint32_t)((lane >> 4) * a.ldc + (lane & 15) * 8) * 2;
    const uint32_t rowstep = (uint32_t)(16 * a.ldc * 2), q1 = (uint32_t)(4 * a.ldc * 2);
#define SK_ASM_STORE_OPERANDS                                                                                        \
  : : [rsc] "s"(rsrc_c), [voff] "v"(voff), [wr] "v"(wr), [rd] "v"(rd), [rowstep] "s"(rowstep), [q1] "s"(q1),         \
      [alpha] "s"(a.alpha) : "memory", "scc", SK_TILE_ASM_CLOBBERS
#define SK_ASM_STORE(WHICH)                                                                            \
  if constexpr (F8 != 0) {                                                                             \
    asm volatile(SK_TILE_ASM_STORE_##WHICH##_SCALED("v_cvt_pk_f16_f32") SK_ASM_STORE_OPERANDS);        \
  } else if constexpr (BF16_) {                                                                        \
    asm volatile(SK_TILE_ASM_STORE_##WHICH("v_cvt_pk_bf16_f32") SK_ASM_STORE_OPERANDS);                \
  } else {                                                                                             \
    asm volatile(SK_TILE_ASM_STORE_##WHICH("v_cvt_pk_f16_f32") SK_ASM_STORE_OPERANDS);                 \
  }
    if constexpr (HALF < 0) {
      SK_ASM_STORE(ALL)
    } else if constexpr (HALF == 0) {
      SK_ASM_STORE(HALF0)
    } else {
      SK_ASM_STORE(HALF1)
    }
#undef SK_ASM_STORE
#undef SK_ASM_STORE_OPERANDS
  }

  // ---- epilogue: fp32 -> C's type through a per-wave LDS patch, 16-byte stores of whole rows ----
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &, int pm, int pn, char *, const void *bias) {
    if (direct_store_ok(a, pn, bias))
      store_c_direct<-1>(a, pm, pn);
    else if (bias == nullptr)
      store_c_impl<false, -1>(a, pm, pn, nullptr);
    else
      store_c_impl<true, -1>(a, pm, pn, bias);
  }
  static __device__ __forceinline__ void store_c_half(const Args &a, const Acc &, int pm, int pn, char *,
                                                      const void *bias, int h) {
    if (direct_store_ok(a, pn, bias)) {
      if (h == 0) store_c_direct<0>(a, pm, pn);
      else store_c_direct<1>(a, pm, pn);
    } else if (bias == nullptr) {
      if (h == 0) store_c_impl<false, 0>(a, pm, pn, nullptr);
      else store_c_impl<false, 1>(a, pm, pn, nullptr);
    } else {
      if (h == 0) store_c_impl<true, 0>(a, pm, pn, bias);
      else store_c_impl<true, 1>(a, pm, pn, bias);
    }
  }
  // HALF < 0: the whole tile; 0 / 1: rows [HALF * 64, HALF * 64 + 64) of every wave's block
  template <bool BIAS, int HALF>
  static __device__ __forceinline__ void store_c_impl(const Args &a, int pm, int pn, const void *epi) {
    constexpr int ROW_BEGIN = HALF < 0 ? 0 : HALF * (WTM / 2), NPASS = HALF < 0 ? 2 : 1;
    const half_t *bias = BIAS ? epi_bias(epi) : nullptr;
    const int act = BIAS ? epi_act(epi) : 0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    if constexpr (I8) {
      // int32 C straight from the accumulators: lane l of block (ii, j) holds row 16 ii + l % 16, columns
      // 16 j + 4 (l / 16) .. + 3
      int *C = reinterpret_cast<int *>(a.C);
      const bool vec_ok = (a.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 15) == 0);
      const int row0 = pm * BM + wm * WTM + (lane & 15), col0 = pn * BN + wn * WTN + 4 * (lane >> 4);
      static_for<ROW_BEGIN / 16, ROW_BEGIN / 16 + NPASS * (PATCH_ROWS / 16)>([&](auto blk) {
        constexpr int ii = decltype(blk)::value;
        static_for<0, FN>([&](auto col) {
          constexpr int j = decltype(col)::value;
          const intx4 x = __builtin_bit_cast(intx4, agpr_read4<(ii * FN + j) * 4>());
          const int grow = row0 + 16 * ii, gcol = col0 + 16 * j;
          if (grow < a.M && gcol < a.N) {
            int *dst = C + (int64_t)grow * a.ldc + gcol;
            if (vec_ok && gcol + 4 <= a.N) {
              *reinterpret_cast<intx4 *>(dst) = x;
            } else {
              for (int e = 0; e < 4 && gcol + e < a.N; ++e) dst[e] = x[e];
            }
          }
        });
      });
      return;
    }
    const int bias_col0 = BIAS ? pn * BN + wn * WTN + pin_here(lane >> 4) * 4 : 0;
    half_t *patch = reinterpret_cast<half_t *>(lds() + wave * (2 * STAGE_BYTES / NW));
    const bool vec_ok = (a.ldc % 8 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 15) == 0);
    constexpr int CPRC = WTN / 8;
    static_for<0, NPASS>([&](auto pass) {
      constexpr int p = decltype(pass)::value;
      static_for<0, PATCH_ROWS / 16>([&](auto blk) {
        constexpr int ib = decltype(blk)::value;
        constexpr int ii = ROW_BEGIN / 16 + p * (PATCH_ROWS / 16) + ib;
        static_for<0, FN>([&](auto col) {
          constexpr int j = decltype(col)::value;
          const floatx4 x = agpr_read4<(ii * FN + j) * 4>();
          floatx4 bv = {0.f, 0.f, 0.f, 0.f};
          if constexpr (BIAS) bv = bias4_at<BF16_>(bias, bias_col0 + j * 16, a.N);
          half4v h;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float y = x[e];
            if constexpr (F8 != 0) y *= a.alpha;  // the product of fp8 operands is scaled before bias and rounding
            if constexpr (BIAS) y = activate(y + bv[e], act);
            if constexpr (BF16_) {
              const __bf16 b = (__bf16)y;
              h[e] = __builtin_bit_cast(half_t, b);  // the patch only carries 16-bit patterns
            } else {
              h[e] = (half_t)y;
            }
          }
          *reinterpret_cast<half4v *>(patch + (ib * 16 + (lane & 15)) * LDC + j * 16 + (lane >> 4) * 4) = h;
        });
      });
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int row0 = pm * BM + wm * WTM + ROW_BEGIN + p * PATCH_ROWS, col0 = pn * BN + wn * WTN;
      constexpr int NCH = PATCH_ROWS * CPRC / 64;  // 16-byte pieces per lane and pass
      // eight LDS reads go out before the first of their stores: inside the edge tests each read would wait out
      // its own LDS round trip
      constexpr int BATCH = 8;
      static_assert(NCH % BATCH == 0, "whole batches");
#pragma unroll
      for (int s0 = 0; s0 < NCH; s0 += BATCH) {
        uint4v v[BATCH];
#pragma unroll
        for (int s = 0; s < BATCH; ++s) {
          const int idx = (s0 + s) * 64 + lane;
          v[s] = *reinterpret_cast<const uint4v *>(patch + (idx / CPRC) * LDC + (idx % CPRC) * 8);
        }
#pragma unroll
        for (int s = 0; s < BATCH; ++s) {
          const int idx = (s0 + s) * 64 + lane;
          const int grow = row0 + idx / CPRC, gcol = col0 + (idx % CPRC) * 8;
          if (grow < a.M && gcol < a.N) {
            half_t *dst = a.C + (int64_t)grow * a.ldc + gcol;
            if (vec_ok && gcol + 8 <= a.N) {
              *reinterpret_cast<uint4v *>(dst) = v[s];
            } else {
              union { uint4v q; half_t h[8]; } u;
              u.q = v[s];
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (gcol + e < a.N) dst[e] = u.h[e];
            }
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    });
    __syncthreads();  // patches overlap the stages of the next tile
  }

  // ---- partial tiles (same workspace layouts as tile_f16_dma.h: float4 group v of thread t at
  // (v * NT + t) * 4 for the ordered reduce, element s of thread t at s * NT + t for the atomic buffer) ----
  static constexpr bool COHERENT_PARTIALS = false;
  static constexpr bool COHERENT_REDUCE = true;
  static constexpr bool HALVES = true;
  // the reference's fix-up: partial sums rounded to C's type and added into C (fp16 / bfloat16 only)
  static constexpr bool ATOMIC_C = MODE_ <= 1;
  static __device__ __forceinline__ void atomic_c(const Args &a, const Acc &, int pm, int pn) {
    if constexpr (ATOMIC_C) {
      const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      const int wm = wave >> 1, wn = wave & 1;
      const int row0 = pm * BM + wm * WTM + (lane & 15), col0 = pn * BN + wn * WTN + 4 * (lane >> 4);
      static_for<0, FM>([&](auto bi) {
        constexpr int ii = decltype(bi)::value;
        static_for<0, FN>([&](auto bj) {
          constexpr int j = decltype(bj)::value;
          const floatx4 x = agpr_read4<(ii * FN + j) * 4>();
          const int grow = row0 + 16 * ii, gcol = col0 + 16 * j;
          if (grow < a.M && gcol < a.N) {  // (N is even: a pair never straddles the edge)
            half_t *p = a.C + (int64_t)grow * a.ldc + gcol;
            atomic_add_pair16<BF16_>(p, x[0], x[1]);
            if (gcol + 2 < a.N) atomic_add_pair16<BF16_>(p + 2, x[2], x[3]);
          }
        });
      });
    }
  }
  template <int V0, int V1>
  static __device__ __forceinline__ void store_groups(float *dst) {
    const BufferRsrc r = make_rsrc(dst, TILE_ELEMS * 4);
    const uint32_t off = (uint32_t)pin_here((int)threadIdx.x) * 16;
    static_for<V0, V1>([&](auto g) {
      constexpr int v = decltype(g)::value;
      st_coherent16(r, off, (uint32_t)v * NT * 16, __builtin_bit_cast(uint4v, agpr_read4<v * 4>()));
    });
  }
  template <int V0, int V1>
  static __device__ __forceinline__ void add_groups(const float *src) {
    const BufferRsrc r = make_rsrc(src, TILE_ELEMS * 4);
    const uint32_t off = (uint32_t)pin_here((int)threadIdx.x) * 16;
    // sixteen loads in flight per lane, then the sixteen sums: the accumulator moves are assembly statements, which
    // the compiler keeps in order, so a loop of load-then-add leaves one load in flight and the exchange of a
    // 256 KB partial tile waits out 64 memory round trips
    constexpr int BATCH = 16;
    static_assert((V1 - V0) % BATCH == 0, "whole batches");
    static_for<0, (V1 - V0) / BATCH>([&](auto b) {
      constexpr int base = V0 + decltype(b)::value * BATCH;
      uint4v raw[BATCH];
      static_for<0, BATCH>([&](auto i) {
        constexpr int v = base + decltype(i)::value;
        raw[decltype(i)::value] = ld_coherent16(r, off, (uint32_t)v * NT * 16);
      });
      static_for<0, BATCH>([&](auto i) {
        constexpr int v = base + decltype(i)::value;
        if constexpr (I8) {
          const intx4 sum = __builtin_bit_cast(intx4, agpr_read4<v * 4>()) + __builtin_bit_cast(intx4, raw[decltype(i)::value]);
          agpr_write4<v * 4>(__builtin_bit_cast(floatx4, sum));
        } else {
          agpr_write4<v * 4>(agpr_read4<v * 4>() + __builtin_bit_cast(floatx4, raw[decltype(i)::value]));
        }
      });
    });
  }
  // The same exchange with the partial sums rounded to C's 16-bit type (SK_FIXUP_REDUCE16: half the bytes through
  // memory; fp16 / bfloat16 kernels).  Groups v and v + 1 of thread t travel as eight 16-bit values at
  // (v / 2 * NT + t) * 16; the receiver widens them and adds in fp32.
  static constexpr bool HALVES16 = MODE_ <= 1;
  static __device__ __forceinline__ uint32_t pack16(float lo, float hi) {
    uint32_t r;
    if constexpr (BF16_)
      asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    else
      asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
  }
  static __device__ __forceinline__ float widen16(uint32_t w, int hi) {
    if constexpr (BF16_) return __builtin_bit_cast(float, hi ? (w & 0xffff0000u) : (w << 16));
    const half2v h = __builtin_bit_cast(half2v, w);
    return (float)h[hi];
  }
  template <int V0, int V1>
  static __device__ __forceinline__ void store_groups16(float *dst) {
    static_assert((V0 | V1) % 2 == 0, "pairs of groups");
    const BufferRsrc r = make_rsrc(dst, TILE_ELEMS * 2);
    const uint32_t off = (uint32_t)pin_here((int)threadIdx.x) * 16;
    static_for<V0 / 2, V1 / 2>([&](auto g) {
      constexpr int v = decltype(g)::value;
      const floatx4 a0 = agpr_read4<(2 * v) * 4>(), a1 = agpr_read4<(2 * v + 1) * 4>();
      const uint4v w = {pack16(a0[0], a0[1]), pack16(a0[2], a0[3]), pack16(a1[0], a1[1]), pack16(a1[2], a1[3])};
      st_coherent16(r, off, (uint32_t)v * NT * 16, w);
    });
  }
  template <int V0, int V1>
  static __device__ __forceinline__ void add_groups16(const float *src) {
    const BufferRsrc r = make_rsrc(src, TILE_ELEMS * 2);
    const uint32_t off = (uint32_t)pin_here((int)threadIdx.x) * 16;
    constexpr int BATCH = 16;   // loads in flight per lane (see add_groups)
    static_assert((V1 - V0) / 2 % BATCH == 0 && V0 % 2 == 0, "whole batches of pairs of groups");
    static_for<0, (V1 - V0) / 2 / BATCH>([&](auto b) {
      constexpr int base = V0 / 2 + decltype(b)::value * BATCH;
      uint4v raw[BATCH];
      static_for<0, BATCH>([&](auto i) {
        constexpr int v = base + decltype(i)::value;
        raw[decltype(i)::value] = ld_coherent16(r, off, (uint32_t)v * NT * 16);
      });
      static_for<0, BATCH>([&](auto i) {
        constexpr int v = base + decltype(i)::value;
        const uint4v w = raw[decltype(i)::value];
        const floatx4 p0 = {widen16(w[0], 0), widen16(w[0], 1), widen16(w[1], 0), widen16(w[1], 1)};
        const floatx4 p1 = {widen16(w[2], 0), widen16(w[2], 1), widen16(w[3], 0), widen16(w[3], 1)};
        agpr_write4<(2 * v) * 4>(agpr_read4<(2 * v) * 4>() + p0);
        agpr_write4<(2 * v + 1) * 4>(agpr_read4<(2 * v + 1) * 4>() + p1);
      });
    });
  }
  static __device__ __forceinline__ void store_partial_half16(const Acc &, float *dst, int h) {
    if (h == 0) store_groups16<0, NV4 / 2>(dst);
    else store_groups16<NV4 / 2, NV4>(dst);
  }
  static __device__ __forceinline__ void add_partial_half16(Acc &, const float *src, int h) {
    if (h == 0) add_groups16<0, NV4 / 2>(src);
    else add_groups16<NV4 / 2, NV4>(src);
  }
  static __device__ __forceinline__ void store_partial(const Acc &, float *dst) { store_groups<0, NV4>(dst); }
  static __device__ __forceinline__ void add_partial(Acc &, const float *src) { add_groups<0, NV4>(src); }
  static __device__ __forceinline__ void store_partial_half(const Acc &, float *dst, int h) {
    if (h == 0) store_groups<0, NV4 / 2>(dst);
    else store_groups<NV4 / 2, NV4>(dst);
  }
  static __device__ __forceinline__ void add_partial_half(Acc &, const float *src, int h) {
    if (h == 0) add_groups<0, NV4 / 2>(src);
    else add_groups<NV4 / 2, NV4>(src);
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &, float *dst) {
    dst = pin_here(dst) + threadIdx.x;
    static_for<0, NV4>([&](auto g) {
      constexpr int v = decltype(g)::value;
      const floatx4 x = agpr_read4<v * 4>();
      const intx4 xi = __builtin_bit_cast(intx4, x);  // (the whole vector: a bit cast of one element reads element 0)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (I8)
          atomic_add_i32(reinterpret_cast<int *>(dst) + (size_t)(v * 4 + e) * NT, xi[e]);
        else
          atomic_add_f32(dst + (size_t)(v * 4 + e) * NT, x[e]);
      }
    });
  }
  // reads the completed sum and leaves zeros behind
  static __device__ __forceinline__ void take_partial(Acc &, float *src) {
    src = pin_here(src) + threadIdx.x;
    constexpr int BATCH = 8;  // (loads in flight per lane: see add_groups)
    static_for<0, NV4 / BATCH>([&](auto b) {
      constexpr int base = decltype(b)::value * BATCH;
      floatx4 x[BATCH];
      static_for<0, BATCH>([&](auto i) {
        constexpr int v = base + decltype(i)::value;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float *p = src + (size_t)(v * 4 + e) * NT;
          x[decltype(i)::value][e] = *p;
          *p = 0.f;
        }
      });
      static_for<0, BATCH>([&](auto i) { agpr_write4<(base + decltype(i)::value) * 4>(x[decltype(i)::value]); });
    });
  }
};

}  // namespace sk
