// Small-M ("skinny") tile arithmetic, fp16 and Q4 weights: M <= 64, the weight matrix streams from
// HBM exactly once and never touches LDS.
//
// CTA tile: BM = 16*MB rows of A  x  BN = 16*NB*WN rows of W  x  BKC = RK*BK of K per iteration.
// Waves are arranged WN (along N) x RK (along K): wave (wn, rk) multiplies its NB 16-row weight
// blocks with the K sub-block rk of the iteration; the RK partial accumulators are summed through
// LDS when the segment ends.  RK is the reference's intra-CTA K split ("block reduction",
// streamk_fp16_block_reduce.py:45,235-306).
//
// Per v_mfma_f32_16x16x32_f16 a lane (row = lane%16, g = lane/16) supplies 8 K-values.  Which 8 is
// free as long as both operands agree.  Weights are loaded straight from global memory, 16 bytes
// per lane: load c of an iteration covers E*4 consecutive K-values of each of the wave's 16 rows
// (E = K-values per 16 bytes: 8 for fp16, 32 for Q4), lane group g taking piece g -- so one load
// instruction reads 64 contiguous bytes from every row.  The A tile is read from LDS at the same
// K offsets.  For Q4, A is written to LDS in the element order the nibble decode produces
// (0,4,1,5,2,6,3,7).
#pragma once
#include <type_traits>
#include "q4_dequant.h"
#include "sk_device.h"

namespace sk {

struct SkinnyArgs {
  const half_t *A;
  const void *W;          // fp16 [N,K] or packed nibbles [N,K/2]
  const half_t *scales;   // Q4: [N, K/group]
  half_t *C;
  int M, N, K;
  int64_t lda, ldw, ldc;  // ldw in elements (fp16) or bytes (Q4)
  int zero;               // Q4: the scalar zero point; fp8: the bits of the fp32 scalar alpha
  int groups;             // Q4: scales per row
  const half_t *zeros;    // Q4 with per-group zero points: [N, K/group], integer values 0..15 (else unused)
};

// Copies the scales of groups [g0, g0 + 8*chunks) of the tile's BN weight rows to LDS rows of SC_ROW
// halfs, 16 bytes at a time.  A 16-byte piece that would run past the end of its row (K / group
// not a multiple of 8) is fetched half by half instead: on the tile's last row a vector load would
// cross the end of the buffer, and the hardware then zeroes the straddling dword.
// begin() issues the first piece of every thread and returns; finish() stores it and copies the
// rest, so a caller can put its other loads in flight between the two.
template <int BN, int SC_ROW, int NT>
struct ScaleStager {
  BufferRsrc rsrc;
  half_t *lds;
  int groups, g0, chunks;
  uint4v first;

  __device__ __forceinline__ bool whole_piece(int idx) const { return g0 + (idx / BN) * 8 + 8 <= groups; }
  __device__ __forceinline__ uint4v load_piece(int idx) const {
    const int r = idx % BN, g = g0 + (idx / BN) * 8;
    return buffer_load_16(rsrc, (uint32_t)(r * groups + g) * 2, 0);
  }
  __device__ __forceinline__ void store_piece(int idx, uint4v v) const {
    const int r = idx % BN, c = idx / BN, g = g0 + c * 8;
    half_t *dst = lds + r * SC_ROW + c * 8;
    if (whole_piece(idx)) {
      *reinterpret_cast<uint4v *>(dst) = v;
    } else {
      for (int e = 0; e < 8; ++e) {
        const uint16_t h =
            g + e < groups ? __builtin_amdgcn_raw_buffer_load_b16(rsrc, (uint32_t)(r * groups + g + e) * 2, 0, 0) : 0;
        dst[e] = __builtin_bit_cast(half_t, h);
      }
    }
  }
  __device__ __forceinline__ void begin(half_t *ldsS, const half_t *scales_tile, int rows, int groups_, int g0_,
                                        int chunks_) {
    rsrc = make_rsrc(scales_tile, (uint32_t)(rows * groups_ * 2));
    lds = ldsS;
    groups = groups_;
    g0 = g0_;
    chunks = chunks_;
    const int idx = threadIdx.x;
    // a piece that is out of range or not whole is loaded from an out-of-range offset (zeros)
    first = buffer_load_16(rsrc, idx < BN * chunks && whole_piece(idx) ? (uint32_t)((idx % BN) * groups + g0 + (idx / BN) * 8) * 2
                                                                       : OOB_OFFSET, 0);
  }
  __device__ __forceinline__ void finish() const {
    if ((int)threadIdx.x < BN * chunks) store_piece(threadIdx.x, first);
    for (int idx = threadIdx.x + NT; idx < BN * chunks; idx += NT) store_piece(idx, whole_piece(idx) ? load_piece(idx) : first);
  }
};
template <int BN, int SC_ROW, int NT>
__device__ __forceinline__ void stage_scales(half_t *ldsS, const half_t *scales_tile, int rows, int groups, int g0,
                                             int chunks) {
  ScaleStager<BN, SC_ROW, NT> st;
  st.begin(ldsS, scales_tile, rows, groups, g0, chunks);
  st.finish();
}

// ROW1_: M == 1 only.  A single row of A is staged and every lane reads it (an LDS broadcast);
// rows 1..15 of the MFMA result are then copies of row 0 and are never stored.
//
// TILED_ (Q4 only): the packed weights are stored in tiles of 16 rows x 64 bytes (one 128-wide scale
// group of 16 weight rows), row by row inside a tile, tiles ordered [row block][group]
// (sk_q4_tile_host / sk_q4_tile).  A wave's load instruction then reads one contiguous KB instead
// of 64 bytes from each of 16 rows 4 KB apart, which streams 1.5x faster (profiles/
// gemv_q4_M1_N8192_K8192.md, access pattern table); each lane receives the same bytes as from the
// row-major array.
//
// ZP_ (Q4 only): one zero point per scale group and row (a.zeros, same shape as the scales) instead of
// one for the whole matrix; staged in LDS beside the scales.
//
// BF16_ (not Q4): operands, bias and C are bfloat16 -- the same 16-bit data movement, the bfloat16 form of the
// MFMA, C rounded to nearest even.
template <int MB_, int NB_, int WN_, int RK_, bool Q4_, int DEPTH_, bool ROW1_ = false, bool TILED_ = false,
          bool ZP_ = false, bool BF16_ = false, int F8_ = 0>
struct TileSkinny {
  static_assert(!BF16_ || !Q4_, "the Q4 decode produces fp16");
  // F8_ (1: OCP e4m3, 2: OCP e5m2; not Q4, not BF16): A and the weights hold fp8 bytes and travel as pairs -- the
  // launcher passes K, lda and ldw halved, and all data movement is the 16-bit kernel's.  A lane's 16 bytes are 16
  // K-values, fed to two v_mfma_f32_16x16x32 fp8 instructions (8 bytes per lane each); A and the weights are cut up
  // the same way, so which K-values a lane holds does not matter.  C is fp16; a.zero carries the bits of the
  // scalar that multiplies the fp32 sums before the epilogue.
  // F8_ == 3: int8 operands the same way, one v_mfma_i32_16x16x64_i8 per 16 bytes; accumulators, the sums of the
  // K-splitting waves, partials and C are int32 and stay in integer registers throughout; no epilogue operands.
  static_assert(F8_ == 0 || (!Q4_ && !BF16_), "one-byte operands exclude the Q4 decode and bfloat16");
  static constexpr bool I8 = F8_ == 3;
  static constexpr int F8 = I8 ? 0 : F8_;
  typedef int intx4 __attribute__((ext_vector_type(4)));
  typedef typename std::conditional<I8, intx4, floatx4>::type AccV;
  typedef typename std::conditional<I8, int, float>::type AccT;
  static_assert(!TILED_ || Q4_, "tiled weights exist for Q4");
  static_assert(!ZP_ || Q4_, "zero points exist for Q4");
  typedef SkinnyArgs Args;
  static constexpr bool LEAN_ENTRY = false;  // see run_persistent
  static constexpr int MB = MB_, NB = NB_, WN = WN_, RK = RK_, DEPTH = DEPTH_;
  static constexpr bool Q4 = Q4_;
  // Up to 16 rows of A with a scalar zero point: the nibbles go into the MFMA undecoded (1024 + q from bits 0..3
  // of a half, 64 + q from bits 4..7: one shift and four v_and_or_b32 per word), the sum over each 128-wide scale
  // group starts from -sum a_k (offset_k + zero) -- four MFMAs per group on a constant fragment, shared by the
  // wave's row blocks -- and the group's scale multiplies the fp32 group sum.  (q - zero) * scale is then never
  // rounded to fp16: the result is at least as close to the exact product as the one from rounded weights, as in
  // the matrix-vector kernels (tile_gemv_q4.h).  8 vector instructions per MFMA instead of 15.
  // (not the instance of four waves along N without a K split, whose registers it does not fit)
  static constexpr bool UNDECODED = Q4_ && !ZP_ && !ROW1_ && MB_ == 1 && F8_ == 0 && !(NB_ == 1 && WN_ == 4 && RK_ == 1);
  // the Q4 instances of one row block per wave without K split: their scalar-argument form spills (skinny_launch.h)
  static constexpr bool NO_FLAT_ARGS = Q4_ && NB_ == 1 && WN_ == 4 && RK_ == 1 && !ROW1_;
  static constexpr int BM = 16 * MB, BN = 16 * NB * WN;
  static constexpr int BK = Q4 ? 256 : 128;  // K per wave per iteration
  static constexpr int BKC = BK * RK;        // K per CTA iteration
  static constexpr int KL = BK / 4;          // K per lane group
  static constexpr int NCH = KL / 8;         // MFMA K-chunks per iteration
  static constexpr int WLOADS = Q4 ? KL / 32 : KL / 8;  // 16-byte weight loads per lane, block, iter
  static constexpr int NT = WN * RK * 64;
  static constexpr int LDA = BKC + 8;        // LDS row of A (halfs)
  static constexpr bool ROW1 = ROW1_;
  static constexpr int A_ROWS = ROW1 ? 1 : BM;  // rows of A staged in LDS
  static constexpr int MAX_M = ROW1 ? 1 : BM;
  static constexpr int A_STAGE = A_ROWS * LDA;
  static constexpr int A_CHUNKS = A_ROWS * BKC / 8;
  static_assert(!ROW1 || MB_ == 1, "the single-row variant has one 16-row block");
  static constexpr int A_LOADS = (A_CHUNKS + NT - 1) / NT;
  static constexpr int QGROUP = 128;
  static constexpr int SC_PER_ITER = BKC / QGROUP;  // Q4 scale groups per CTA iteration
  static constexpr int SC_MAX_ITERS = 64;           // scale staging covers this many iterations
  static constexpr int LDS_A = 2 * A_STAGE * 2;
  static constexpr int SC_ROW = SC_MAX_ITERS * SC_PER_ITER + 8;  // halfs per LDS scale row
  static constexpr int LDS_SC1 = Q4 ? BN * SC_ROW * 2 : 0;       // scales
  static constexpr int LDS_SC = ZP_ ? 2 * LDS_SC1 : LDS_SC1;     // scales, then zero points
  static constexpr int LDS_RED = RK > 1 ? (RK - 1) * WN * 64 * MB * NB * 16 : 0;
  static constexpr int LDS_BYTES = LDS_A + LDS_SC + LDS_RED;
  static constexpr int LDS_TOTAL = LDS_BYTES;
  // partials are held by the rk == 0 waves only
  static constexpr int TILE_ELEMS = BM * BN;
  static constexpr int NTP = WN * 64;
  static constexpr int NV4 = MB * NB;
  // co-resident CTAs per CU the kernel is compiled for: 16 waves per CU unless LDS says less
  static constexpr int CTAS_PER_CU_WAVES = 16 / (NT / 64);
  static constexpr int CTAS_PER_CU_LDS = (160 * 1024) / (LDS_BYTES + 64);
  static constexpr int CTAS_PER_CU = CTAS_PER_CU_WAVES < CTAS_PER_CU_LDS ? CTAS_PER_CU_WAVES : CTAS_PER_CU_LDS;
  static constexpr int WAVES_PER_EU = CTAS_PER_CU * (NT / 64) / 4 > 0 ? CTAS_PER_CU * (NT / 64) / 4 : 1;

  struct Acc {
    AccV c[MB][NB];
  };

  static __device__ __forceinline__ void mac(const Args &a, Acc &acc, int pm, int pn, int k0, int n,
                                             char *smem) {
    half_t *ldsA = reinterpret_cast<half_t *>(smem);
    half_t *ldsS = reinterpret_cast<half_t *>(smem + LDS_A);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, rk = wave / WN;
    const int lr = lane & 15, lg = lane >> 4;

#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc.c[i][j] = AccV{0, 0, 0, 0};

    // ---- weights: one row per lane and block; the buffer descriptor covers the tile's rows, so
    // rows past N read as zero ----
    constexpr int WB = Q4 ? 1 : 4;  // bytes per 2 K-values... (Q4: 1 byte, fp16: 4 bytes)
    const int rows_w = min(BN, a.N - pn * BN);
    const uint32_t ldw_bytes = (uint32_t)a.ldw * (Q4 ? 1 : 2);
    // tiled: a 16-row block of the tile is a.groups consecutive KB; blocks past N are out of range
    const uint32_t block_bytes = (uint32_t)a.groups * 1024;
    const BufferRsrc rsrc_w =
        TILED_ ? make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * (BN / 16) * block_bytes,
                           (uint32_t)((rows_w + 15) / 16) * block_bytes)
               : make_rsrc(reinterpret_cast<const char *>(a.W) + (int64_t)pn * BN * ldw_bytes, rows_w * ldw_bytes);
    constexpr int E = Q4 ? 32 : 8;               // K-values in one 16-byte load
    const int klane = rk * BK + lg * E;          // K offset of this lane's piece of load 0
    uint32_t voff_w[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j)
      voff_w[j] = TILED_ ? (uint32_t)(wn * NB + j) * block_bytes + (uint32_t)(lr * 64 + lg * 16)
                         : (uint32_t)((wn * NB + j) * 16 + lr) * ldw_bytes + (uint32_t)(klane / 2) * WB;

    // ---- A tile: all BM rows are staged; rows past M read as zero ----
    const int a_rows = min(a.M - pm * BM, A_ROWS);
    const BufferRsrc rsrc_a = make_rsrc(a.A + (int64_t)pm * BM * a.lda, (uint32_t)(a_rows * a.lda * 2));
    int a_rd[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) a_rd[i] = (ROW1 ? 0 : (i * 16 + lr) * LDA) + klane;
    uint32_t voff_a[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int idx = i * NT + tid;
      const int row = idx / (BKC / 8), kc = idx % (BKC / 8);
      voff_a[i] = (A_CHUNKS % NT == 0 || idx < A_CHUNKS) ? (uint32_t)(row * a.lda + kc * 8) * 2 : OOB_OFFSET;
    }
    uint4v wreg[DEPTH][NB][WLOADS];
    uint4v areg[DEPTH][A_LOADS];

    // Loads for iterations past the segment (or past K) are still issued -- every trip through
    // the main loop then has the same loads in flight in the same order, which keeps the waits
    // exact -- but with an out-of-range offset, which returns zeros without touching memory.
    // klimit = K-values left in the tile row from this iteration's start (<= 0 past the segment).
    auto issue_loads = [&](int slot, int rel_it) {
      const int kbase = (k0 + rel_it) * BKC;
      const uint32_t koff_w = TILED_ ? (uint32_t)((kbase + rk * BK) / QGROUP) * 1024 : (uint32_t)(kbase / 2) * WB;
      const uint32_t koff_a = (uint32_t)kbase * 2;
      const int klimit = rel_it < n ? a.K - kbase : 0;
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int c = 0; c < WLOADS; ++c) {
          const bool inside = (TILED_ ? rk * BK : klane) + c * (4 * E) < klimit;
          wreg[slot][j][c] = buffer_load_16(rsrc_w, inside ? voff_w[j] : OOB_OFFSET, koff_w + c * (TILED_ ? 1024 : 64));
        }
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) {
        const bool inside = ((i * NT + tid) % (BKC / 8)) * 8 < klimit;
        areg[slot][i] = buffer_load_16(rsrc_a, inside ? voff_a[i] : OOB_OFFSET, koff_a);
      }
    };
    auto stage_a = [&](int slot, int buf) {
      half_t *dst = ldsA + buf * A_STAGE;
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) {
        const int idx = i * NT + tid;
        const int row = idx / (BKC / 8), kc = idx % (BKC / 8);
        if (A_CHUNKS % NT == 0 || idx < A_CHUNKS) {
          uint4v v = areg[slot][i];
          if (Q4) {
            // element order 0,4,1,5,2,6,3,7 == interleave the low and high 8 bytes by halfs
            uint4v p;
            p[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
            p[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
            p[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
            p[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
            v = p;
          }
          *reinterpret_cast<uint4v *>(dst + row * LDA + kc * 8) = v;
        }
      }
    };

    const Q4Consts qc = q4_consts(a.zero);
    // UNDECODED: the magic of the nibbles at bits 4..7 (fp16 64.0: 64 + q) and minus the offsets of a word's eight
    // elements in the order the decode leaves them (0,4 | 1,5 | 2,6 | 3,7: bits 0..3, bits 4..7, 0..3, 4..7)
    uint32_t magic_hi = 0x54005400u;
    asm volatile("" : "+v"(magic_hi));
    half8v neg_offsets;
    {
      const half_t lo = (half_t)(float)(-(1024 + a.zero)), hi = (half_t)(float)(-(64 + a.zero));
      neg_offsets = half8v{lo, lo, hi, hi, lo, lo, hi, hi};
    }

    // ---- prologue: DEPTH iterations of loads in flight ----
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue_loads(d, d);

    // ---- Q4: stage the scales of this segment, 16 bytes at a time.  Row r of the tile needs
    // groups [k0*SC_PER_ITER, (k0+n)*SC_PER_ITER); the copy starts at the 8-aligned group below
    // and ldsS[r][sc_shift + i] is group k0*SC_PER_ITER + i.
    int sc_shift = 0;
    if (Q4) {
      const int g_first = k0 * SC_PER_ITER, g0 = g_first & ~7;
      sc_shift = g_first - g0;
      const int chunks = (sc_shift + n * SC_PER_ITER + 7) >> 3;
      stage_scales<BN, SC_ROW, NT>(ldsS, a.scales + (int64_t)pn * BN * a.groups, rows_w, a.groups, g0, chunks);
      if (ZP_)
        stage_scales<BN, SC_ROW, NT>(ldsS + BN * SC_ROW, a.zeros + (int64_t)pn * BN * a.groups, rows_w, a.groups, g0, chunks);
    }
    stage_a(0, 0);
    __syncthreads();

    // ---- main loop: rounds of DEPTH iterations, no exit inside a round.  Iterations past the
    // segment multiply zeros (their loads were pushed out of range), so n need not be a multiple
    // of DEPTH. ----
    for (int it0 = 0; it0 < n; it0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int it = it0 + d;
        const half_t *abuf = ldsA + (it & 1) * A_STAGE;
        half2v sc[NB][WLOADS], zlo[NB][WLOADS], zhi[NB][WLOADS];
        if (Q4) {
#pragma unroll
          for (int j = 0; j < NB; ++j) {
            // iterations past the segment multiply zero weights; they must still see a finite scale
            // load c of a Q4 iteration spans exactly one 128-wide scale group: group rk*2 + c
            const half_t *sp = ldsS + ((wn * NB + j) * 16 + lr) * SC_ROW + sc_shift + min(it, n - 1) * SC_PER_ITER + rk * 2;
#pragma unroll
            for (int c = 0; c < WLOADS; ++c) {
              sc[j][c] = half2v{sp[c], sp[c]};
              if (ZP_) {
                const half_t z = sp[BN * SC_ROW + c];
                const half_t lo = (half_t)1024.f + z, hi = (half_t)-64.f - z;   // exact: integers below 2048
                zlo[j][c] = half2v{lo, lo};
                zhi[j][c] = half2v{hi, hi};
              }
            }
          }
        }
        if constexpr (UNDECODED) {
          // load c of the iteration is one scale group: chunks 4c .. 4c+3
#pragma unroll
          for (int c = 0; c < WLOADS; ++c) {
            half8v fa4[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) fa4[q] = *reinterpret_cast<const half8v *>(abuf + a_rd[0] + c * 128 + q * 8);
            floatx4 base = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < 4; ++q) base = __builtin_amdgcn_mfma_f32_16x16x32_f16(neg_offsets, fa4[q], base, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < NB; ++j) {
              floatx4 p = base;
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                union {
                  uint32_t u[4];
                  half8v v;
                } r;
                const uint32_t w = wreg[d][j][c][q], t = w >> 8;
                r.u[0] = and_or(w, qc.mask_lo, qc.magic);
                r.u[1] = and_or(w, qc.mask_hi, magic_hi);
                r.u[2] = and_or(t, qc.mask_lo, qc.magic);
                r.u[3] = and_or(t, qc.mask_hi, magic_hi);
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.v, fa4[q], p, 0, 0, 0);
              }
              // result register r of the lane is weight row 4 * (lane / 16) + r of the block
              const half_t *sp = ldsS + ((wn * NB + j) * 16 + lg * 4) * SC_ROW + sc_shift + min(it, n - 1) * SC_PER_ITER + rk * 2 + c;
#pragma unroll
              for (int r4 = 0; r4 < 4; ++r4)
                acc.c[0][j][r4] = __builtin_fmaf(p[r4], (float)sp[r4 * SC_ROW], acc.c[0][j][r4]);
            }
          }
        } else
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
          half8v fa[MB];
          // K offset of chunk ch relative to the lane's piece of load 0
          constexpr int CH_PER_LOAD = E / 8;
          const int koff_ch = (ch / CH_PER_LOAD) * (4 * E) + (ch % CH_PER_LOAD) * 8;
#pragma unroll
          for (int i = 0; i < MB; ++i) fa[i] = *reinterpret_cast<const half8v *>(abuf + a_rd[i] + koff_ch);
#pragma unroll
          for (int j = 0; j < NB; ++j) {
            half8v fw;
            if (Q4) {
              if (ZP_)
                fw = dequant_word_q4(wreg[d][j][ch / 4][ch % 4], qc, sc[j][ch / 4], zlo[j][ch / 4], zhi[j][ch / 4]);
              else
                fw = dequant_word_q4(wreg[d][j][ch / 4][ch % 4], qc, sc[j][ch / 4]);
            } else {
              fw = __builtin_bit_cast(half8v, wreg[d][j][ch]);
            }
#pragma unroll
            for (int i = 0; i < MB; ++i)
              if constexpr (I8) {
                acc.c[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, fw), __builtin_bit_cast(intx4, fa[i]),
                                                                    acc.c[i][j], 0, 0, 0);
              } else if constexpr (F8 != 0) {
                typedef long longx2 __attribute__((ext_vector_type(2)));
                const longx2 w2 = __builtin_bit_cast(longx2, fw), a2 = __builtin_bit_cast(longx2, fa[i]);
                if constexpr (F8 == 1) {
                  acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w2[0], a2[0], acc.c[i][j], 0, 0, 0);
                  acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w2[1], a2[1], acc.c[i][j], 0, 0, 0);
                } else {
                  acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(w2[0], a2[0], acc.c[i][j], 0, 0, 0);
                  acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(w2[1], a2[1], acc.c[i][j], 0, 0, 0);
                }
              } else if constexpr (BF16_) {
                typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
                acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fw),
                                                                      __builtin_bit_cast(bf16x8, fa[i]), acc.c[i][j], 0, 0, 0);
              } else {
                acc.c[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw, fa[i], acc.c[i][j], 0, 0, 0);
              }
          }
        }
        // A tile of the next iteration into the other LDS buffer, then refill this ring slot
        stage_a((d + 1) % DEPTH, (it + 1) & 1);
        issue_loads(d, it + DEPTH);
        __syncthreads();
      }
    }

    // ---- sum the RK partial accumulators into the rk == 0 waves ----
    if (RK > 1) {
      AccT *red = reinterpret_cast<AccT *>(smem + LDS_A + LDS_SC);
      if (rk > 0) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
          for (int j = 0; j < NB; ++j)
            *reinterpret_cast<AccV *>(red + ((((rk - 1) * WN + wn) * NV4 + i * NB + j) * 64 + lane) * 4) =
                acc.c[i][j];
      }
      __syncthreads();
      if (rk == 0) {
#pragma unroll
        for (int r = 1; r < RK; ++r)
#pragma unroll
          for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int j = 0; j < NB; ++j)
              acc.c[i][j] += *reinterpret_cast<const AccV *>(
                  red + ((((r - 1) * WN + wn) * NV4 + i * NB + j) * 64 + lane) * 4);
      }
      __syncthreads();
    }
  }

  // acc.c[i][j][r] = C[pm*BM + i*16 + lane%16][pn*BN + (wn*NB + j)*16 + 4*(lane/16) + r]
  // (two copies behind one uniform branch: the epilogue without a bias carries none of its code)
  static __device__ __forceinline__ void store_c(const Args &a, const Acc &acc, int pm, int pn, char *smem,
                                                 const void *bias) {
    if (bias == nullptr)
      store_c_impl<false>(a, acc, pm, pn, smem, nullptr);
    else
      store_c_impl<true>(a, acc, pm, pn, smem, bias);
  }
  template <bool BIAS>
  static __device__ __forceinline__ void store_c_impl(const Args &a, const Acc &acc, int pm, int pn, char *,
                                                      const void *epi) {
    const half_t *bias = BIAS ? epi_bias(epi) : nullptr;
    const int act = BIAS ? epi_act(epi) : 0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (wave >= WN) return;
    const int lr = lane & 15, lg = lane >> 4;
    if constexpr (I8) {  // int32 C straight from the accumulators (ldc counts int32 elements)
      int *C = reinterpret_cast<int *>(a.C);
      const bool vec_ok = (a.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 15) == 0);
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const int row = pm * BM + i * 16 + lr;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const int col = pn * BN + (wave * NB + j) * 16 + lg * 4;
          if (row < a.M && col < a.N) {
            int *dst = C + (int64_t)row * a.ldc + col;
            if (vec_ok && col + 4 <= a.N) {
              *reinterpret_cast<intx4 *>(dst) = acc.c[i][j];
            } else {
              for (int e = 0; e < 4 && col + e < a.N; ++e) dst[e] = acc.c[i][j][e];
            }
          }
        }
      }
      return;
    } else {
    const bool vec_ok = (a.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.C) & 7) == 0);
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const int row = pm * BM + i * 16 + lr;
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int col = pn * BN + (wave * NB + j) * 16 + lg * 4;
        if (row < a.M && col < a.N) {
          half4v h;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x = acc.c[i][j][e];
            if constexpr (F8 != 0) x *= __builtin_bit_cast(float, a.zero);
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
    }  // !I8
  }

  // Partial tiles are a few KB and there can be thousands of CTAs: every access is a coherent
  // (write-through / L2-bypassing) one, so no CTA ever flushes or invalidates a whole L2.
  static constexpr bool COHERENT_PARTIALS = true;

  // (int8: the partial buffer holds int32 sums; the fix-up code addresses it as float, 4 bytes either way)
  static __device__ __forceinline__ void store_partial(const Acc &acc, float *dst_) {
    if (threadIdx.x >= NTP) return;
    AccT *dst = reinterpret_cast<AccT *>(dst_);
#pragma unroll
    for (int v = 0; v < NV4; ++v)
      st_coherent(dst + ((size_t)v * NTP + threadIdx.x) * 4, acc.c[v / NB][v % NB]);
  }
  static __device__ __forceinline__ void add_partial(Acc &acc, const float *src_) {
    if (threadIdx.x >= NTP) return;
    const AccT *src = reinterpret_cast<const AccT *>(src_);
#pragma unroll
    for (int v = 0; v < NV4; ++v)
      acc.c[v / NB][v % NB] += ld_coherent(src + ((size_t)v * NTP + threadIdx.x) * 4);
  }
  static __device__ __forceinline__ void atomic_partial(const Acc &acc, float *dst_) {
    if (threadIdx.x >= NTP) return;
    AccT *dst = reinterpret_cast<AccT *>(dst_);
#pragma unroll
    for (int v = 0; v < NV4; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (I8)
          atomic_add_i32(dst + (size_t)(v * 4 + e) * NTP + threadIdx.x, acc.c[v / NB][v % NB][e]);
        else
          atomic_add_f32(dst + (size_t)(v * 4 + e) * NTP + threadIdx.x, acc.c[v / NB][v % NB][e]);
      }
  }
  static __device__ __forceinline__ void take_partial(Acc &acc, float *src_) {
    if (threadIdx.x >= NTP) return;
    AccT *src = reinterpret_cast<AccT *>(src_);
#pragma unroll
    for (int v = 0; v < NV4; ++v)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        AccT *p = src + (size_t)(v * 4 + e) * NTP + threadIdx.x;
        acc.c[v / NB][v % NB][e] = ld_coherent_scalar(p);
        st_coherent(p, (AccT)0);
      }
  }
};

}  // namespace sk
