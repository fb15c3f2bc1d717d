// Host-side Stream-K partitioner and kernel selection (pure integer code, no device access).
//
// The arithmetic restates streamk_fp32.py:30-54 of the reference for run-time shapes, with two
// changes: the persistent grid is a parameter instead of `total_sm = 108`, and the number of
// data-parallel waves is ceil(blocking_tiles / grid) with 0 allowed (the reference's
// max(blocking_tiles // total_sm, 1) walks out of range when there are no data-parallel tiles).
#include <string.h>

#include <mutex>

#include "kernel_table.h"
#include "streamk.h"

namespace sk {

static KernelInfo g_table[400];
static int g_count = 0;
static std::once_flag g_table_once;

int tile_kernel_infos(KernelInfo *out, int max);
int tile_asm_kernel_infos(KernelInfo *out, int max);
int tile_asm8_kernel_infos(KernelInfo *out, int max);
int tile_q4_kernel_infos(KernelInfo *out, int max);
int tile_8bit_kernel_infos(KernelInfo *out, int max);
int skinny_kernel_infos(KernelInfo *out, int max);
int f32_kernel_infos(KernelInfo *out, int max);

const KernelInfo *kernel_table(int *count) {
  std::call_once(g_table_once, [] {
    int n = tile_kernel_infos(g_table, 400);
    n += tile_8bit_kernel_infos(g_table + n, 400 - n);
    n += tile_asm_kernel_infos(g_table + n, 400 - n);
    n += tile_asm8_kernel_infos(g_table + n, 400 - n);
    n += tile_q4_kernel_infos(g_table + n, 400 - n);
    n += skinny_kernel_infos(g_table + n, 400 - n);
    n += f32_kernel_infos(g_table + n, 400 - n);
    g_count = n;
  });
  if (count) *count = g_count;
  return g_table;
}

const KernelInfo *kernel_by_id(int id) {
  int n;
  const KernelInfo *t = kernel_table(&n);
  for (int i = 0; i < n; ++i)
    if (t[i].id == id) return &t[i];
  return nullptr;
}

static int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// preference among kernel variants of one tile shape when the caller does not ask for one: the
// eight-wave direct-to-LDS tile kernels; the most specialised small-M kernel that accepts the shape
static int variant_rank(const KernelInfo &k) {
  // (small-M: general 0 < rows-of-A matrix-vector form 3 < single-row 1 < matrix-vector 2; the kernels that stream
  // the weights through LDS, variant 4, share tile shapes with general kernels and are taken when asked for by
  // variant, or by the default rule below)
  if (k.family == FAMILY_SKINNY)
    return k.variant == 4 ? -1 : (k.variant == 3 ? 1 : (k.variant == 0 ? 0 : k.variant + 1));
  return k.variant == 7 ? 4 : (k.variant == 4 ? 3 : (k.variant == 1 ? 2 : (k.variant == 2 ? 1 : 0)));
}
static bool accepts_shape(const KernelInfo &k, int64_t M, int64_t K) {
  // (the assembly-loop tile kernels have no K tail: other K go to the next-best variant of the tile)
  return (k.max_m == 0 || M <= k.max_m) && (k.max_ipt == 0 || (K + k.bk - 1) / k.bk <= k.max_ipt) &&
         (k.family != FAMILY_TILE || k.variant != 7 || K % k.k_align == 0);
}

// 65 to 96 rows of fp16 / bfloat16 (NT) whose 96 x 32 tiles fill the device in one round: see pick_kernel
static bool rows_65_to_96_stream(int64_t M, int64_t N, int dtype, int layout, int num_cus) {
  return (dtype == SK_F16 || dtype == SK_BF16) && layout == SK_LAYOUT_NT && M > 64 && M <= 96 && cdiv(N, 32) <= num_cus &&
         cdiv(N, 32) * 5 >= (int64_t)num_cus * 3;
}

static const KernelInfo *pick_kernel(int64_t M, int64_t N, int64_t K, int dtype, int layout,
                                     const sk_config *cfg, int num_cus) {
  int n;
  const KernelInfo *t = kernel_table(&n);
  const bool want_tile = cfg && cfg->bm > 0 && cfg->bn > 0;
  // cfg->reserved[0]: 0 = newest variant of the tile, v > 0 = variant v - 1
  const int want_variant = cfg ? cfg->reserved[0] - 1 : -1;
  if (want_tile) {
    const KernelInfo *found = nullptr;
    for (int i = 0; i < n; ++i)
      if (t[i].dtype == dtype && t[i].layout == layout && t[i].bm == cfg->bm && t[i].bn == cfg->bn &&
          (cfg->bk <= 0 || t[i].bk == cfg->bk) && (want_variant < 0 || t[i].variant == want_variant) &&
          accepts_shape(t[i], M, K) && (found == nullptr || variant_rank(t[i]) > variant_rank(*found)))
        found = &t[i];
    return found;
  }
  // heuristic: small M -> weight-streaming kernels; otherwise the largest tile that still gives
  // every CU something to do
  const KernelInfo *best = nullptr;
  // (for 32 < M <= 64 the 64x64 LDS tile below is faster than streaming the weights past 64 rows)
  const bool q4 = dtype == SK_Q4 || dtype == SK_Q4_TILED || dtype == SK_Q4_ZP || dtype == SK_Q4_ZP_TILED;
  // (one-byte operands: up to 64 rows -- their tile kernels start at 128 rows)
  const bool one_byte = dtype == SK_F8E4M3 || dtype == SK_F8E5M2 || dtype == SK_I8;
  if (dtype == SK_Q4 && M > 64 && want_variant < 0) {
    // more rows than the weight-streaming kernels take: the tile kernels that dequantise B on its way into LDS.
    // 256 rows of A per tile as soon as M has them: a CTA decodes its BN weight rows whatever BM is, and the
    // four-wave 128 x 128 kernel waits for its loads (one wave per SIMD, a short iteration), so a 256 x 128 tile
    // takes no longer than a 128 x 128 one; where that leaves CUs without a tile the Stream-K schedule splits K
    // (N = K = 8192, M = 512: 73 us against 109 us on 128 x 128 tiles).  There is no 256 x 256 instance: eight waves
    // that decode and hold 128 x 64 accumulators each do not fit the register file (it spilled); large M is better
    // served by dequantising once and running the fp16 kernels, which is what streamk_q4 does from 1024 rows on.
    const int want_bm = M > 128 ? 256 : 128;
    const int want_bn = 128;
    for (int i = 0; i < n; ++i)
      if (t[i].family == FAMILY_TILE && t[i].dtype == SK_Q4 && t[i].bm == want_bm && t[i].bn == want_bn) return &t[i];
    return nullptr;
  }
  // (2 <= M <= 4 as well: the matrix-vector form with four rows of A (variant 3) is behind at every size measured,
  // weights from HBM -- 2 x 4096 x 4096 11.3 us against 8.7 us on 16 x 16 tiles, 4 x 11008 x 4096 23.0 / 17.5,
  // 4 x 4096 x 11008 26.9 / 17.4, 4 x 8192 x 8192 32.0 / 24.8 -- and stays as an explicit choice)
  // (one row: from 40 MB on -- 1 x 8192 x 8192 24.4 us against 28.9 us for the matrix-vector kernel, 1 x 14336 x 4096
  // 22.3 / 27.3, 1 x 4096 x 11008 17.3 / 19.9, 1 x 5120 x 5120 11.7 / 13.8, 1 x 11008 x 4096 17.5 / 17.2; 1 x 4096 x 4096
  // 8.6 / 8.1 stays with the matrix-vector kernel)
  const bool stream_rows = M >= 2 || N * K >= (int64_t)20 << 20;
  if ((dtype == SK_F16 || dtype == SK_BF16) && layout == SK_LAYOUT_NT && stream_rows && M <= 64 && want_variant < 0) {
    // 5 <= M <= 64 (fewer rows on large weights, above) with fp16 / bfloat16 weights: the kernels that stream the weights through LDS in contiguous loads
    // (tile_stream_pairs.h).  Tiles of 32 weight rows while one wave of them fits the device (N = 8192: one tile per
    // CU and no fix-up), 64 rows beyond; 64 rows of A exist with 32 weight rows only.
    // (more than 32 rows: 64 weight rows where they give three fifths of the CUs a tile -- A is then as many bytes
    // per CTA as the weights instead of twice as many; 64 x 16384 x 8192: 49 us against 56 us)
    const bool narrow = M > 32 ? cdiv(N, 64) * 5 < (int64_t)num_cus * 3 : cdiv(N, 32) <= num_cus;
    int bm = M <= 16 ? 16 : (M <= 32 ? 32 : 64), bn = narrow ? 32 : 64, bk = (bm == 16 && narrow) ? 512 : 256;
    // (up to 16 rows and no more than a tile of 16 weight rows per CU: K split over all four waves -- N = 4096 then
    // has a tile per CU; 16 x 4096 x 11008: 18.6 us against 21.4 us on 32-row tiles with a fix-up)
    if (bm == 16 && cdiv(N, 16) <= num_cus) bn = 16, bk = 1024;
    for (int i = 0; i < n; ++i)
      if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].variant == 4 && t[i].bm == bm && t[i].bn == bn &&
          t[i].bk == bk && accepts_shape(t[i], M, K))
        return &t[i];
  }
  // 65 to 96 rows of fp16 / bfloat16 where 96 x 32 tiles fill the device in one round (N = 8192 on 256 CUs): the
  // streaming kernel with three blocks of rows per wave -- A is three times the bytes of the weights per CTA, but the
  // weights still arrive in contiguous loads; 80 x 8192 x 8192 from HBM 38.5 us against 44.1 us on the tile kernels.
  // From three fifths of the CUs on (80 x 6144 x 4096: 19.6 / 27.1, 80 x 5120 x 5120: 24.0 / 33.5); other widths lose
  // to the tile kernels (96 x 11008 x 4096: 38.8 / 32.2, 80 x 4096 x 11008: 44.7 / 37.9, 80 x 16384 x 8192: 74.7 / 67.7).
  if (want_variant < 0 && rows_65_to_96_stream(M, N, dtype, layout, num_cus))
    for (int i = 0; i < n; ++i)
      if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].variant == 4 && t[i].bm == 96 && accepts_shape(t[i], M, K))
        return &t[i];
  if ((M <= (one_byte ? 64 : 32) && layout == SK_LAYOUT_NT) || q4) {
    // M == 1 with Q4 weights: the matrix-vector kernel with four waves splitting K (data-parallel
    // over 16-row tiles), the fastest instance at LLM-sized N and K.  Weights from HBM: from K = 14336 on eight waves
    // (1 x 16384 x 16384: 25.9 us against 28.7 us, 1 x 4096 x 14336: 7.9 / 9.0; 1 x 4096 x 11008: 8.2 / 7.4).  With more
    // 16-row tiles than CTAs of four waves stay resident (three per CU): K up to 6144 split over two waves, four
    // CTAs per CU (1 x 14336 x 4096: 7.7 us in one round against 10.8 us in two; 1 x 32000 x 4096: 14.6 / 16.2,
    // 1 x 65536 x 4096: 25.7 / 27.9), K from 8192 on over eight (1 x 28672 x 8192: 25.5 / 27.1).
    if (q4 && M == 1 && want_variant < 0) {
      int bk = 1024;
      if (K >= 14336) bk = 2048;
      else if (cdiv(N, 16) > (int64_t)num_cus * 3) bk = K <= 6144 ? 512 : (K >= 8192 ? 2048 : 1024);
      for (int pass = 0; pass < 2; ++pass, bk = 1024)
        for (int i = 0; i < n; ++i)
          if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].variant == 2 && t[i].bn == 16 &&
              t[i].bk == bk && accepts_shape(t[i], M, K))
            return &t[i];
    }
    // 2 <= M <= 16 with row-major Q4 weights (scalar zero point), weights from HBM.  Where 64-row tiles give three
    // fifths of the CUs a tile the general kernel with 64 weight rows and K split over two waves, data-parallel
    // (16 x 28672 x 8192: 32.8 us; the 32-row kernel below: 48.5; 16 x 11008 x 4096: 10.7 / 14.8; 16 x 16384 x 16384:
    // 37.6 / 38.1).  Fewer rows and 16 MB of weights or more: the kernel that streams the packed weights through
    // LDS in contiguous loads, 32 weight rows per tile (tile_stream_q4.h; 16 x 8192 x 8192: 12.2 us against 14.2,
    // 16 x 4096 x 11008: 13.3 / 15.3; 16 x 4096 x 4096: 6.9 / 7.3).
    if (dtype == SK_Q4 && M > 1 && M <= 16 && want_variant < 0) {
      if (cdiv(N, 64) * 5 >= (int64_t)num_cus * 3) {
        for (int i = 0; i < n; ++i)
          if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].variant == 0 && t[i].bm == 16 &&
              t[i].bn == 64 && t[i].bk == 512 && accepts_shape(t[i], M, K))
            return &t[i];
      } else if (N * K >= ((int64_t)16 << 20) && K % 256 == 0) {
        for (int i = 0; i < n; ++i)
          if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].variant == 4 && t[i].bn == 32 &&
              accepts_shape(t[i], M, K))
            return &t[i];
      }
    }
    // 2 <= M <= 16 with Q4 weights: eight waves per CTA (two per SIMD cover each other's waits),
    // 32 weight rows, K split over four waves
    if (((dtype == SK_Q4 && M > 1) || dtype == SK_Q4_ZP || dtype == SK_Q4_ZP_TILED) && M <= 16 && want_variant < 0)
      for (int i = 0; i < n; ++i)
        if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].variant == 0 && t[i].bm == 16 &&
            t[i].bn == 32 && t[i].bk == 1024 && accepts_shape(t[i], M, K))
          return &t[i];
    // 2 <= M <= 4 with fp16 / bfloat16 weights: the matrix-vector form with four rows of A
    if ((dtype == SK_F16 || dtype == SK_BF16) && M >= 2 && M <= 4 && want_variant < 0)
      for (int i = 0; i < n; ++i)
        if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].layout == layout && t[i].variant == 3 &&
            t[i].bn == 16 && t[i].bk == 512 && accepts_shape(t[i], M, K))
          return &t[i];
    // M == 1 with fp16 / bfloat16 weights: the same structure, K split over four waves
    if ((dtype == SK_F16 || dtype == SK_BF16) && M == 1 && want_variant < 0)
      for (int i = 0; i < n; ++i)
        if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].layout == layout && t[i].variant == 2 &&
            t[i].bn == 16 && t[i].bk == 512 && accepts_shape(t[i], M, K))
          return &t[i];
    int mb = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
    for (int i = 0; i < n; ++i)
      if (t[i].family == FAMILY_SKINNY && t[i].dtype == dtype && t[i].bm == mb && t[i].bn == 64 &&
          accepts_shape(t[i], M, K) && (want_variant < 0 || t[i].variant == want_variant) &&
          t[i].variant <= 2 && (best == nullptr || t[i].variant > best->variant))
        best = &t[i];
    if (best) return best;
    if (q4) return nullptr;
  }
  if (dtype == SK_F32) {
    // 32 x 256 tiles for M <= 32 (a quarter of the wasted rows of a 128-row tile), else 128 x 128
    const int want_bm = M <= 32 ? 32 : 128;
    const KernelInfo *any = nullptr;
    for (int i = 0; i < n; ++i)
      if (t[i].dtype == SK_F32 && t[i].layout == layout) {
        if (t[i].bm == want_bm) return &t[i];
        if (!any) any = &t[i];
      }
    return any;
  }
  // 256x256 tiles when they fill the device; else 128x128, else 64x64.  The smaller tiles run one
  // or two waves per SIMD, where the four-stage (BK = 32) pipeline hides the load latency better;
  // it exists for the NT layout only.
  const int64_t tiles256 = cdiv(M, 256) * cdiv(N, 256), tiles128 = cdiv(M, 128) * cdiv(N, 128);
  // (256x256: the four-wave kernel with the K loop in assembly where it applies -- K a multiple of 64 --
  // else the eight-wave 16x16x32-MFMA form)
  int pref[3][4] = {{256, 256, 64, 4}, {128, 128, 32, 3}, {64, 64, 32, 3}};  // bm, bn, bk, variant
  if (K % 64 == 0 && (dtype == SK_F16 || dtype == SK_BF16)) pref[0][3] = 7;
  const int first = tiles256 * 4 >= (int64_t)num_cus * 3 ? 0 : (tiles128 * 2 >= num_cus ? 1 : 2);
  const int order[3][3] = {{0, 1, 2}, {1, 2, 0}, {2, 1, 0}};  // smaller tiles first, then larger ones
  for (int oi = 0; oi < 3 && !best; ++oi) {
    const int pi = order[first][oi];
    for (int pass = 0; pass < 2 && !best; ++pass) {  // pass 1: any variant / BK of the tile shape
      for (int i = 0; i < n; ++i) {
        if (t[i].family != FAMILY_TILE || t[i].dtype != dtype || t[i].layout != layout) continue;
        if (t[i].bm != pref[pi][0] || t[i].bn != pref[pi][1]) continue;
        if (want_variant >= 0 && t[i].variant != want_variant) continue;
        if (pass == 0 && want_variant < 0 && (t[i].bk != pref[pi][2] || t[i].variant != pref[pi][3])) continue;
        if (!accepts_shape(t[i], M, K)) continue;
        if (best == nullptr || variant_rank(t[i]) > variant_rank(*best)) best = &t[i];
      }
    }
  }
  return best;
}

// ---- which tile kernel and which split of K, when the caller leaves both open (M > 64) ----
// A cost model with four constants per kernel family, fitted to 80 shapes x 5 families x splits 1, 2, 4 timed on
// an MI355X (mean |log error| 5-10 %):
//     time = rounds * (n * tau * clock + o) + phi * log2(split)
//   n       K-iterations per CTA (iterations per tile / split)
//   clock   1 + 0.4 * (busy CUs / CUs)^2: the part is power-limited, busy CUs slow each other down
//   rounds  CTAs the busiest CU runs one after another; a family whose CTAs share a CU (occ > 1) is charged
//           1 + (rounds - 1) * gamma for them
//   o       prologue and epilogue of a CTA, phi one exchange of half tiles between the CTAs of a split tile (a
//           tile cut in two takes one, a tile cut in four two in a row: see run_persistent)
// Choosing by it is within 5 % of the fastest of the candidates on average (worst case 23 %) on those shapes, where
// the earlier rule (largest tile that fills the device, Stream-K for what is left) was 49 % behind on average.
static int gcd_int(int a, int b) {
  while (b) {
    const int r = a % b;
    a = b;
    b = r;
  }
  return a;
}

// The automatic schedule of a tile kernel with more tiles than CTAs; *sk_tiles: how many tiles it splits.
// Data-parallel when the last wave of tiles is at least 90 % full.  Else Stream-K over the remainder plus one
// wave of tiles (`sk2`, streamk_fp32.py:37-43; with fewer than two waves that is every tile, `basic` -- the
// reference's formula would split the remainder alone there, 2 tiles over 256 CTAs for 258 tiles, and the ordered
// fix-up has one CTA add up 63 partial tiles per tile: 1243 us against 130 us) -- but only where the CTAs of an
// XCD stay close to lock-step on K, which the L2 reuse of the tile kernels depends on: either every CTA range
// starts at the beginning or in the middle of a tile (grid / gcd(Stream-K tiles, grid) <= 2), or consecutive
// ranges start within ipt / 2 iterations of each other across the grid / 8 CTAs of an XCD.  Measured against
// data-parallel: 3-22 % faster where admitted; 4 or 8 distinct offsets between 8 % faster and 40 % slower;
// ranges that start anywhere up to 1.5x slower.  `interleave` (may be null: not offered) opens a third way for a
// one-CTA-per-CU kernel: with g = gcd(Stream-K tiles, grid) >= 8 the interleaved tile order puts the g CTAs that
// start at the same offset side by side on one XCD, which restores their lock-step (fp16 256 x 256 tiles, every
// tile split: 4096 x 5120 x 5120 172 us against 203 us in raster order, 3000 x 6144 x 4096 132 against 172,
// 2048 x 11008 x 4096 171 against 172; the best data-parallel plan of any tile: 215 / 160 / 178 us).
static int auto_tile_schedule(int64_t total, int grid, int ipt, int *sk_tiles, int *interleave = nullptr) {
  *sk_tiles = 0;
  if (interleave) *interleave = 0;
  const int64_t waves = (total + grid - 1) / grid;
  if (total < grid || total * 10 >= waves * grid * 9 || ipt < 64) return SK_SCHED_DP;  // (short K: the fix-up outweighs the tail)
  const int sched = total >= 2 * (int64_t)grid ? SK_SCHED_SK_TWO_TILE : SK_SCHED_SK_BASIC;
  const int skt = (int)(total % grid) + grid;
  const int64_t iters = (int64_t)skt * ipt;          // spread over `grid` CTAs
  const double per_cta = (double)iters / grid;       // in [ipt, 2 ipt)
  const double r = per_cta - ipt;                    // how far consecutive ranges drift apart, in iterations
  const double d = r < ipt - r ? r : ipt - r;
  const bool aligned = grid / gcd_int(skt, grid) <= 2;
  const bool close = d * (grid / 8 > 0 ? grid / 8 : 1) <= ipt / 2.0;
  if (!aligned && !close) {
    const int g = gcd_int(skt, grid);
    if (!interleave || g < 8 || skt / g < 2) return SK_SCHED_DP;
    *interleave = 1;
  }
  *sk_tiles = skt;
  return sched;
}

struct TileFamily {
  int bm, bn, bk, variant, occ, max_split;  // variant -1: the preferred variant of the tile
  float tau, gamma, o, phi;
};
static const TileFamily kFamilies16[] = {
    {256, 256, 64, 7, 1, 4, 0.919f, 0.20f, 6.4f, 6.9f},   // four waves, K loop in assembly (K % 64 == 0)
    {256, 256, 64, 4, 1, 2, 1.080f, 0.20f, 9.3f, 10.0f},  // eight waves, for the other K
    {128, 128, 64, 4, 2, 4, 0.497f, 0.47f, 4.9f, 5.1f},
    {128, 128, 32, 5, 2, 4, 0.218f, 0.89f, 3.8f, 4.5f},   // four stages of 32 (NT only)
    {64, 128, 32, 5, 3, 4, 0.154f, 0.89f, 3.5f, 3.2f},
    {128, 256, 64, 4, 1, 4, 0.689f, 1.00f, 6.0f, 5.9f},
    {256, 128, 64, 4, 1, 4, 0.685f, 0.20f, 5.3f, 5.8f},
};
// one-byte operands (BK = 128), fitted the same way to 36 shapes each (64 x 128: to 42 shapes with M <= 1024)
static const TileFamily kFamiliesF8[] = {
    {256, 256, 128, -1, 1, 4, 0.934f, 1.00f, 8.8f, 6.1f},
    {128, 128, 128, -1, 2, 2, 0.435f, 0.52f, 6.3f, 6.6f},
    {128, 256, 128, -1, 1, 2, 0.580f, 0.20f, 9.3f, 6.7f},
    {256, 128, 128, -1, 1, 2, 0.608f, 1.00f, 7.2f, 7.8f},
    {64, 128, 128, -1, 2, 2, 0.335f, 0.46f, 4.3f, 6.5f},
    {128, 128, 64, 5, 2, 4, 0.218f, 0.88f, 2.3f, 11.0f},  // four stages of 64 (fitted to 48 shapes with M <= 1024)
    {64, 128, 64, 5, 3, 4, 0.135f, 1.00f, 2.9f, 8.6f},
};
static const TileFamily kFamiliesI8[] = {
    {256, 256, 128, -1, 1, 4, 0.876f, 0.20f, 13.3f, 4.2f},
    {128, 128, 128, -1, 2, 2, 0.531f, 0.52f, 2.3f, 6.4f},
    {128, 256, 128, -1, 1, 2, 0.674f, 0.20f, 6.5f, 6.5f},
    {256, 128, 128, -1, 1, 2, 0.700f, 1.00f, 4.9f, 6.5f},
    {64, 128, 128, -1, 2, 2, 0.392f, 0.39f, 3.3f, 4.0f},
    {128, 128, 64, 5, 2, 4, 0.222f, 0.77f, 4.7f, 3.9f},   // four stages of 64 (fitted to 48 shapes with M <= 1024)
    {64, 128, 64, 5, 3, 4, 0.143f, 0.88f, 4.0f, 4.1f},
};

static const KernelInfo *model_pick(int64_t M, int64_t N, int64_t K, int dtype, int layout, int num_cus, int *split,
                                    int *sched) {
  const TileFamily *fams = kFamilies16;
  int nfams = (int)(sizeof(kFamilies16) / sizeof(kFamilies16[0]));
  if (dtype == SK_F8E4M3 || dtype == SK_F8E5M2) {
    fams = kFamiliesF8;
    nfams = (int)(sizeof(kFamiliesF8) / sizeof(kFamiliesF8[0]));
  } else if (dtype == SK_I8) {
    fams = kFamiliesI8;
    nfams = (int)(sizeof(kFamiliesI8) / sizeof(kFamiliesI8[0]));
  }
  const KernelInfo *best = nullptr;
  double best_time = 0;
  bool have_asm = false;
  for (int fi = 0; fi < nfams; ++fi) {
    const TileFamily &f = fams[fi];
    sk_config want;
    memset(&want, 0, sizeof(want));
    want.bm = f.bm; want.bn = f.bn; want.bk = f.bk;
    want.reserved[0] = f.variant + 1;
    const KernelInfo *k = pick_kernel(M, N, K, dtype, layout, &want, num_cus);
    if (!k || k->family != FAMILY_TILE || K % k->k_align != 0) continue;
    if (f.variant == 7) have_asm = true;
    if (f.variant == 4 && f.bm == 256 && f.bn == 256 && have_asm) continue;  // the assembly kernel applies
    const int64_t tiles = cdiv(M, f.bm) * cdiv(N, f.bn);
    const int64_t ipt = cdiv(K, f.bk);
    for (int s = 1; s <= f.max_split; s *= 2) {
      if (ipt % s != 0 || (s > 1 && ipt / s < 8)) continue;
      const int64_t ctas = tiles * s;
      if (s > 1 && ctas > (int64_t)num_cus * k->ctas_per_cu) continue;  // the CTAs of a split tile wait for each other
      const double busy = ctas < num_cus ? (double)ctas / num_cus : 1.0;
      const double clock = 1.0 + 0.4 * busy * busy;
      const int64_t rounds = ctas > num_cus ? cdiv(ctas, num_cus) : 1;
      const double eff = f.occ == 1 ? (double)rounds : 1.0 + (rounds - 1) * f.gamma;
      const double time = eff * ((double)(ipt / s) * f.tau * clock + f.o) + (s == 1 ? 0.0 : (s == 2 ? f.phi : 2.0 * f.phi));
      if (!best || time < best_time) {
        best = k;
        best_time = time;
        *split = s;
        *sched = s > 1 ? SK_SCHED_SPLIT_K : SK_SCHED_DP;
      }
    }
    // more tiles than CUs on a one-CTA-per-CU kernel, and a Stream-K schedule that the automatic rule admits: the
    // iterations spread evenly over the CUs, plus one exchange of partial tiles (the rule is applied again below,
    // to the same effect, when the plan is made)
    int skt = 0;
    int ilv = 0;
    int *offer = f.bm == 256 && f.bn == 256 ? &ilv : nullptr;  // (the interleaved order: measured on these tiles)
    if (f.occ == 1 && tiles > num_cus && auto_tile_schedule(tiles, num_cus, (int)ipt, &skt, offer) != SK_SCHED_DP) {
      const double time = (double)tiles * ipt / num_cus * f.tau * 1.4 + f.o * (double)cdiv(tiles, num_cus) + 2.0 * f.phi;
      if (!best || time < best_time) {
        best = k;
        best_time = time;
        *split = 1;
        *sched = SK_SCHED_AUTO;
      }
    }
  }
  return best;
}

}  // namespace sk

using namespace sk;

extern "C" int sk_selfcheck(void) {
  int n;
  const KernelInfo *t = kernel_table(&n);
  if (n <= 0 || n >= 400) return SK_ERR_CONFIG;  // (400: the table's capacity)
  for (int i = 0; i < n; ++i) {
    if (t[i].id < 0 || t[i].id >= 512 || !t[i].name || !t[i].name[0]) return SK_ERR_CONFIG;
    for (int j = 0; j < i; ++j)
      if (t[j].id == t[i].id) return SK_ERR_CONFIG;
  }
  return SK_OK;
}

extern "C" int sk_make_plan(int64_t M, int64_t N, int64_t K, int dtype, int layout, const sk_config *cfg,
                            int num_cus, sk_plan *out) {
  if (!out) return SK_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return SK_ERR_SHAPE;
  if (dtype != SK_F16 && dtype != SK_F32 && dtype != SK_Q4 && dtype != SK_BF16 && dtype != SK_Q4_TILED &&
      dtype != SK_F8E4M3 && dtype != SK_I8 && dtype != SK_Q4_ZP && dtype != SK_F8E5M2 && dtype != SK_Q4_ZP_TILED)
    return SK_ERR_CONFIG;
  if ((dtype == SK_F8E4M3 || dtype == SK_F8E5M2 || dtype == SK_I8) && layout != SK_LAYOUT_NT) return SK_ERR_CONFIG;
  if (layout != SK_LAYOUT_NT && layout != SK_LAYOUT_NN) return SK_ERR_CONFIG;
  if (num_cus <= 0) return SK_ERR_DEVICE;
  // tile, variant, schedule and grid all left open for a 16-bit or one-byte problem with more rows than the
  // weight-streaming kernels take: the cost model chooses kernel and split
  sk_config modelled;
  if ((dtype == SK_F16 || dtype == SK_BF16 || dtype == SK_F8E4M3 || dtype == SK_F8E5M2 || dtype == SK_I8) && M > 64 &&
      !rows_65_to_96_stream(M, N, dtype, layout, num_cus) &&
      (!cfg || (cfg->bm == 0 && cfg->bn == 0 && cfg->bk == 0 && cfg->reserved[0] == 0 &&
                cfg->schedule == SK_SCHED_AUTO && cfg->grid == 0))) {
    int split = 1, model_sched = SK_SCHED_AUTO;
    if (const KernelInfo *mk = model_pick(M, N, K, dtype, layout, num_cus, &split, &model_sched)) {
      if (cfg) modelled = *cfg; else memset(&modelled, 0, sizeof(modelled));
      modelled.bm = mk->bm; modelled.bn = mk->bn; modelled.bk = mk->bk;
      modelled.reserved[0] = mk->variant + 1;
      modelled.schedule = model_sched;
      if (split > 1) modelled.reserved[1] = split;
      cfg = &modelled;
    }
  }
  const KernelInfo *k = pick_kernel(M, N, K, dtype, layout, cfg, num_cus);
  if (!k) return SK_ERR_CONFIG;
  if (K % k->k_align != 0) return SK_ERR_ALIGN;

  memset(out, 0, sizeof(*out));
  out->M = M; out->N = N; out->K = K;
  out->dtype = dtype; out->layout = layout;
  out->bm = k->bm; out->bn = k->bn; out->bk = k->bk;
  out->kernel_id = k->id; out->threads = k->threads; out->lds_bytes = k->lds_bytes;
  out->num_block_m = (int32_t)cdiv(M, k->bm);
  out->num_block_n = (int32_t)cdiv(N, k->bn);
  out->iters_per_tile = (int32_t)cdiv(K, k->bk);
  if (k->max_ipt > 0 && out->iters_per_tile > k->max_ipt) return SK_ERR_CONFIG;
  const int64_t total64 = (int64_t)out->num_block_m * out->num_block_n;
  if (total64 * out->iters_per_tile > 0x7fffffff) return SK_ERR_SHAPE;
  const int total = (int)total64;
  out->total_tiles = total;

  // every CTA of the Stream-K wave may wait for another one, so the grid is capped at what the
  // device keeps resident
  const int occ = k->ctas_per_cu;
  const int max_grid = num_cus * occ;
  int grid = cfg && cfg->grid > 0 ? cfg->grid : max_grid;
  if (grid > max_grid) return SK_ERR_CONFIG;
  int sched = cfg ? cfg->schedule : SK_SCHED_AUTO;
  if (!(cfg && cfg->grid > 0)) {
    const int64_t iters = total64 * out->iters_per_tile;
    // (the kernels that stream the weights through LDS are bound by memory: with tiles for three fifths of the CUs --
    // fp16 / bfloat16: two fifths -- they run data-parallel rather than pay a fix-up; Q4 16 x 11008 x 4096: 11.5 us
    // against 14.3 us, fp16 16 x 2048 x 8192 on 128 tiles: 11.5 against 14.1, 32 x 11008 x 4096 on 172 tiles of 32 x 64:
    // 19.2 against 22.7; not the 64 x 32 tiles, where the split wins)
    const bool stream_dp = k->family == FAMILY_SKINNY && (k->variant == 4 || k->dtype == SK_Q4) && k->max_m >= 16 &&
                           (k->bm == 16 || (k->variant == 4 && k->dtype != SK_Q4 && !(k->bm == 64 && k->bn == 32))) &&
                           total64 * 5 >= (int64_t)num_cus * (k->variant == 4 && k->dtype != SK_Q4 ? 2 : 3);
    const bool q4_gemv = k->family == FAMILY_SKINNY && k->variant == 2 && k->max_m == 1 &&
                         (k->dtype == SK_Q4 || k->dtype == SK_Q4_ZP || k->dtype == SK_Q4_TILED || k->dtype == SK_Q4_ZP_TILED);
    if ((total64 >= num_cus || stream_dp) && total64 <= max_grid) {
      grid = (int)total64;  // one tile per CTA, all resident: a single data-parallel wave
    } else if (q4_gemv && total64 > max_grid) {
      // more tiles than resident CTAs: as few CTAs as finish in the same number of rounds, so that every CTA walks
      // (nearly) the same number of tiles -- a CTA's later tiles find their first loads in flight (mac_tiles)
      grid = (int)cdiv(total64, cdiv(total64, max_grid));
    } else if (total64 < num_cus) {
      // fewer tiles than CUs: one CTA per CU, but a split tile keeps at least 4 K-iterations per CTA
      // and there are never fewer CTAs than tiles
      int64_t want = iters / 4 < num_cus ? iters / 4 : num_cus;
      if (want < total64) want = total64;
      grid = (int)(want > 8 && want != total64 ? want / 8 * 8 : want);
      if (grid > max_grid) grid = max_grid;
    }
  }
  if (sched == SK_SCHED_SPLIT_K) {
    // fixed split: the grid follows from the split factor, a caller's grid is not consulted
    const int ipt = out->iters_per_tile;
    int split = cfg ? cfg->reserved[1] : 0;
    if (split < 0) return SK_ERR_CONFIG;
    if (split == 0) {
      split = 1;
      for (int s = 2; s <= ipt / 4 && total64 * s <= max_grid; ++s)
        if (ipt % s == 0) split = s;
    }
    if (ipt % split != 0 || total64 * split > max_grid) return SK_ERR_CONFIG;
    grid = (int)(total64 * split);
  }
  int auto_interleave = 0;  // the automatic schedule asks for the interleaved order of its Stream-K tiles
  if (sched == SK_SCHED_AUTO) {
    // data-parallel when the last wave of tiles is (nearly) full: Stream-K's fix-up and the L2
    // reuse it gives up cost more than a tail of under 10 %.  Otherwise Stream-K, splitting only
    // the remainder tiles when there are at least two full waves beside them.
    const int64_t waves = (total64 + grid - 1) / grid;
    if (total64 * 10 >= waves * grid * 9) sched = SK_SCHED_DP;
    else sched = total64 >= 2 * (int64_t)grid ? SK_SCHED_SK_ONE_TILE : SK_SCHED_SK_TWO_TILE;
    // (the kernels that stream the weights through LDS are bound by memory, not by the busiest CU: an uneven last
    // wave costs them less than the fix-up; 16 x 28672 x 8192: 77.8 us data-parallel against 83.6 us.  With 64 rows of
    // A on 64 x 32 tiles it is the other way round, 110 us against 103 us; on 64 x 64 tiles 91.5 against 92.6)
    if (k->family == FAMILY_SKINNY && k->variant == 4 && (k->bm == 16 || k->bn == 64) && total64 >= grid) sched = SK_SCHED_DP;
    // (the same for the Q4 matrix-vector kernels: 1 x 28672 x 8192 on 1792 tiles 28.0 us data-parallel against 31.2 us,
    // 1 x 14336 x 4096 with K split over four waves 10.8 against 16.1)
    if (k->family == FAMILY_SKINNY && k->variant == 2 && k->max_m == 1 && total64 >= grid &&
        (k->dtype == SK_Q4 || k->dtype == SK_Q4_ZP || k->dtype == SK_Q4_TILED || k->dtype == SK_Q4_ZP_TILED))
      sched = SK_SCHED_DP;
    if (k->family == FAMILY_TILE && sched != SK_SCHED_DP) {
      // Fewer tiles than CUs: the idle CUs are put to work by an aligned split in two or four, never by CTA ranges
      // that start anywhere.  More tiles than CTAs: see
      // auto_tile_schedule.
      if (total64 < num_cus && !(cfg && cfg->grid > 0)) {
        const int ipt = out->iters_per_tile, max_split = 4;
        int split = 1;
        for (int s = 2; s <= max_split && total64 * s <= max_grid; s *= 2)
          if (ipt % s == 0 && ipt / s >= 8) split = s;
        sched = split > 1 ? SK_SCHED_SPLIT_K : SK_SCHED_DP;
        grid = split > 1 ? (int)(total64 * split) : grid;
      } else {
        int skt;
        sched = auto_tile_schedule(total64, grid, out->iters_per_tile, &skt, occ == 1 && k->bm == 256 && k->bn == 256 ? &auto_interleave : nullptr);  // (measured on these)
      }
    }
  }
  // a data-parallel-only launch never has more CTAs than tiles (idle CTAs would also skew the
  // CTA -> XCD mapping: the low logical ids sit on the first XCDs)
  if (sched == SK_SCHED_DP && grid > total) grid = total;
  int sk_tiles;
  switch (sched) {
    case SK_SCHED_DP: sk_tiles = 0; break;
    case SK_SCHED_SK_TWO_TILE:  // streamk_fp32.py:37-43
      sk_tiles = total % grid;
      if (total - sk_tiles > grid) sk_tiles += grid;
      break;
    case SK_SCHED_SK_ONE_TILE: sk_tiles = total % grid; break;
    case SK_SCHED_SK_BASIC: sk_tiles = total; break;
    case SK_SCHED_SPLIT_K: sk_tiles = grid == total ? 0 : total; break;  // split 1 is data-parallel
    default: return SK_ERR_CONFIG;
  }
  out->schedule = sched;
  out->grid = grid;
  out->streamk_tiles = sk_tiles;
  out->blocking_tiles = total - sk_tiles;
  out->streamk_iters = sk_tiles * out->iters_per_tile;
  out->streamk_full_tiles = out->streamk_iters / grid;
  out->streamk_partial_tiles = out->streamk_iters % grid;
  out->dp_waves = (int32_t)cdiv(out->blocking_tiles, grid);
  int fixup = cfg ? cfg->fixup : SK_FIXUP_AUTO;
  if (fixup == SK_FIXUP_AUTO) fixup = SK_FIXUP_REDUCE;
  if (fixup != SK_FIXUP_ATOMIC && fixup != SK_FIXUP_REDUCE && fixup != SK_FIXUP_ATOMIC_C && fixup != SK_FIXUP_REDUCE16)
    return SK_ERR_CONFIG;
  // partial sums exchanged in 16 bits: the assembly-loop kernels for fp16 / bfloat16, every Stream-K tile cut into two
  // or four equal segments (what the device side's exchange of half tiles handles)
  if (fixup == SK_FIXUP_REDUCE16 &&
      !(k->family == FAMILY_TILE && k->variant == 7 && (dtype == SK_F16 || dtype == SK_BF16) && sk_tiles > 0 &&
        out->streamk_partial_tiles == 0 &&
        (2 * out->streamk_full_tiles == out->iters_per_tile || 4 * out->streamk_full_tiles == out->iters_per_tile)))
    return SK_ERR_CONFIG;
  // packed 16-bit atomics into C: the 16-bit tile kernels with 16x16 accumulator blocks
  if (fixup == SK_FIXUP_ATOMIC_C &&
      !(k->family == FAMILY_TILE && (k->variant == 4 || k->variant == 5 || k->variant == 7) &&
        (dtype == SK_F16 || dtype == SK_BF16) && N % 2 == 0))
    return SK_ERR_CONFIG;
  out->fixup = fixup;
  out->spin_limit = cfg && cfg->spin_limit > 0 ? cfg->spin_limit : (1 << 22);
  out->interleave = 0;
  if (cfg && cfg->reserved[2] != 0 && cfg->reserved[2] != 1) return SK_ERR_CONFIG;
  if ((cfg && cfg->reserved[2] == 1) || auto_interleave) {
    int g = sk_tiles, b = grid;  // gcd
    while (b) { const int t = g % b; g = b; b = t; }
    if (sk_tiles > 0 && g > 1 && sk_tiles / g > 1) out->interleave = sk_tiles / g;
  }
  out->raster = cfg ? cfg->raster : 0;
  if (out->raster < 0) return SK_ERR_CONFIG;
  // default tile order of the LDS-tiled 16-bit and fp8 kernels: groups of 8 tile rows.  Concurrent CTAs
  // then share B tiles as well as A tiles in the L2s: 0-20 % faster than row-major order on every shape
  // measured (no effect on the fp32 kernels, which keep the reference's order).
  if (out->raster == 0 && k->family == FAMILY_TILE && dtype != SK_F32 && out->num_block_m > 1) out->raster = 8;

  // workspace: status block, fixed-size flag area, fp32 partial tiles
  int64_t ws = 0;
  // (CTA ranges that are whole tiles -- e.g. `basic` on a tile count that is a multiple of the grid, which only
  // changes which tiles a CTA takes -- never reach the fix-up: no workspace)
  const bool whole_tiles = out->streamk_partial_tiles == 0 && out->streamk_full_tiles % out->iters_per_tile == 0;
  if (sk_tiles > 0 && fixup != SK_FIXUP_ATOMIC_C && !whole_tiles) {
    const int64_t nflags = (fixup == SK_FIXUP_REDUCE || fixup == SK_FIXUP_REDUCE16) ? grid : sk_tiles;
    if (nflags > WS_MAX_FLAGS) return SK_ERR_CONFIG;
    ws = WS_PART_OFF + nflags * (int64_t)k->partial_elems * 4;
  }
  out->workspace_bytes = ws;
  return SK_OK;
}

extern "C" int sk_plan_cta_range(const sk_plan *p, int pid, int32_t *start, int32_t *last) {
  if (!p || !start || !last) return SK_ERR_NULL;
  if (pid < 0 || pid >= p->grid) return SK_ERR_CONFIG;
  const int full = p->streamk_full_tiles, part = p->streamk_partial_tiles;
  *start = pid * full + (pid < part ? pid : part);              // streamk_fp32.py:93
  *last = (pid + 1) * full + (pid + 1 < part ? pid + 1 : part);  // streamk_fp32.py:94-96
  return SK_OK;
}

extern "C" int sk_plan_tile_coords(const sk_plan *p, int tile, int32_t *pid_m, int32_t *pid_n) {
  if (!p || !pid_m || !pid_n) return SK_ERR_NULL;
  if (tile < 0 || tile >= p->total_tiles) return SK_ERR_CONFIG;
  if (p->interleave > 1 && tile < p->streamk_tiles)
    tile = (tile % p->interleave) * (p->streamk_tiles / p->interleave) + tile / p->interleave;
  if (p->raster <= 0) {  // streamk_fp32.py:106-107
    *pid_m = tile / p->num_block_n;
    *pid_n = tile % p->num_block_n;
  } else {  // triton_impl.py:14-28
    const int width = p->raster * p->num_block_n;
    const int group = tile / width;
    const int first_m = group * p->raster;
    const int gsize = p->num_block_m - first_m < p->raster ? p->num_block_m - first_m : p->raster;
    const int r = tile - group * width;
    *pid_m = first_m + r % gsize;
    *pid_n = r / gsize;
  }
  return SK_OK;
}

extern "C" size_t sk_workspace_bytes(const sk_plan *p) { return p ? (size_t)p->workspace_bytes : 0; }
