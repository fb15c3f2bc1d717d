/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference Stream-K algorithm.
 *
 * Nothing in the shipped library or its Python host layer may call into this file; it exists so
 * that tests, the smoke check and the benchmark's cpu_baseline leg have an independent checker.
 *
 * Each function cites the reference lines (relative to the LeiWang1999/Stream-k.tvm checkout) it
 * follows.  The reference itself cannot run on a CPU (it is TVM-TL code generated for CUDA), so
 * these are plain-C restatements of its arithmetic:
 *
 *   ora_partition          streamk_fp32.py:33-54   (== streamk_fp16.py:92-113, triton_impl.py:205-219)
 *   ora_cta_range          streamk_fp32.py:93-96   (== triton_impl.py:117-119)
 *   ora_streamk_gemm_f32   streamk_fp32.py:80-158  (segment loop, fixup predicate, DP loop) with the
 *                          masked edges of triton_impl.py:45-92
 *   ora_dequant_q4         streamk.fp16.breakdown/streamk_fp16_ladder_block_reduce_q4.py:552
 *                          (element order) extended with zero-point / group scale as
 *                          w = fp16_rn((fp16(q) - zero) * scale[n][k / group])
 *
 * Pinning (see tests/test_oracle_*.py): partition numbers against the reference's own shapes worked
 * by hand, the 9-tile/4-CTA schematic of figures/image.png, coverage-exactly-once invariants and a
 * pure-Python twin; GEMM against numpy matmul; dequant against an independent numpy float16
 * evaluation over every nibble x every finite fp16 scale.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
  int num_block_m, num_block_n, iters_per_tile, total_tiles;
  int streamk_tiles, blocking_tiles, streamk_iters;
  int streamk_full_tiles;    /* iterations every CTA gets (the reference's misnomer is kept) */
  int streamk_partial_tiles; /* first this-many CTAs get one extra iteration */
  int sm_partition_factor;   /* DP tiles per CTA: blocking_tiles / P (0 allowed, see below) */
} ora_partition_t;

static int cdiv(int a, int b) { return (a + b - 1) / b; }

/* streamk_fp32.py:33-54.  One deliberate deviation: the reference computes
 * max(blocking_tiles // P, 1), which runs one out-of-range DP tile per CTA when blocking_tiles == 0
 * (its author notes the problem at streamk.fp32.breakdown/full_tiles.py:148-150); here it is
 * blocking_tiles // P. */
void ora_partition(int M, int N, int K, int BM, int BN, int BK, int P, ora_partition_t *o) {
  o->num_block_m = cdiv(M, BM);
  o->num_block_n = cdiv(N, BN);
  o->iters_per_tile = cdiv(K, BK);
  o->total_tiles = o->num_block_m * o->num_block_n;
  o->streamk_tiles = o->total_tiles % P;
  if (o->total_tiles - o->streamk_tiles > P) o->streamk_tiles += P;
  o->blocking_tiles = o->total_tiles - o->streamk_tiles;
  o->streamk_iters = o->streamk_tiles * o->iters_per_tile;
  o->streamk_full_tiles = o->streamk_iters / P;
  o->streamk_partial_tiles = o->streamk_iters % P;
  o->sm_partition_factor = o->blocking_tiles / P;
}

/* streamk_fp32.py:93-96 */
void ora_cta_range(const ora_partition_t *p, int pid, int *start, int *last) {
  int a = pid < p->streamk_partial_tiles ? pid : p->streamk_partial_tiles;
  int b = pid + 1 < p->streamk_partial_tiles ? pid + 1 : p->streamk_partial_tiles;
  *start = pid * p->streamk_full_tiles + a;
  *last = (pid + 1) * p->streamk_full_tiles + b;
}

/* One BMxBN accumulator over k-iterations [k0, k0+n) of tile (pm, pn); edges read as zero
 * (triton_impl.py:76-77 boundary_check).  trans_b: 0 -> B is [K,N] (streamk_fp32.py:74),
 * 1 -> B is [N,K] (streamk_fp16.py:132). */
static void mac_segment(const float *A, const float *B, float *acc, int M, int N, int K, int trans_b,
                        int BM, int BN, int BK, int pm, int pn, int k0, int n) {
  memset(acc, 0, sizeof(float) * (size_t)BM * BN);
  for (int it = 0; it < n; ++it) {
    int kb = (k0 + it) * BK;
    for (int i = 0; i < BM; ++i) {
      int gi = pm * BM + i;
      if (gi >= M) break;
      for (int j = 0; j < BN; ++j) {
        int gj = pn * BN + j;
        if (gj >= N) break;
        float s = acc[i * BN + j];
        int kend = kb + BK < K ? kb + BK : K;
        if (trans_b) {
          const float *a = A + (size_t)gi * K, *b = B + (size_t)gj * K;
          for (int k = kb; k < kend; ++k) s += a[k] * b[k];
        } else {
          const float *a = A + (size_t)gi * K;
          for (int k = kb; k < kend; ++k) s += a[k] * B[(size_t)k * N + gj];
        }
        acc[i * BN + j] = s;
      }
    }
  }
}

/*
 * Executes the persistent kernel of streamk_fp32.py:160-175 with P simulated CTAs on the CPU.
 *   cta_order  permutation of [0,P) giving the order CTAs are run in (NULL = ascending).  With
 *              fixup 0 this is the order "atomic" adds land in C.
 *   fixup 0    reference behaviour (streamk_fp32.py:127-134): whole-tile segment -> store, otherwise
 *              C += partial.  C must be zero on entry for the Stream-K tiles (streamk_fp32.py:200).
 *   fixup 1    ordered reduce: every partial of a tile is kept; the tile is written once as
 *              ((p_owner + p_next) + p_next2 ...) in ascending CTA id, whatever cta_order is.
 * Returns 0, or -1 on bad arguments.
 */
int ora_streamk_gemm_f32(const float *A, const float *B, float *C, int M, int N, int K, int trans_b,
                         int BM, int BN, int BK, int P, const int *cta_order, int fixup) {
  if (M <= 0 || N <= 0 || K <= 0 || BM <= 0 || BN <= 0 || BK <= 0 || P <= 0) return -1;
  ora_partition_t pt;
  ora_partition(M, N, K, BM, BN, BK, P, &pt);
  const int ipt = pt.iters_per_tile;
  float *acc = (float *)malloc(sizeof(float) * (size_t)BM * BN);
  /* fixup 1: one slot per (CTA, segment-is-partial); a CTA has at most 2 partial segments */
  float *slots = NULL;
  int *slot_tile = NULL;
  if (fixup == 1) {
    slots = (float *)calloc((size_t)2 * P * BM * BN, sizeof(float));
    slot_tile = (int *)malloc(sizeof(int) * 2 * P);
    for (int i = 0; i < 2 * P; ++i) slot_tile[i] = -1;
  }
  for (int oi = 0; oi < P; ++oi) {
    int pid = cta_order ? cta_order[oi] : oi;
    if (pid < 0 || pid >= P) { free(acc); free(slots); free(slot_tile); return -1; }
    int start, last;
    ora_cta_range(&pt, pid, &start, &last);
    int nseg = 0;
    while (start < last) { /* streamk_fp32.py:98-136 */
      int end = start + (ipt - start % ipt);
      if (end > last) end = last;
      int tile = start / ipt, k0 = start % ipt;
      int pm = tile / pt.num_block_n, pn = tile % pt.num_block_n;
      mac_segment(A, B, acc, M, N, K, trans_b, BM, BN, BK, pm, pn, k0, end - start);
      int whole = (k0 == 0) && (end % ipt == 0);
      if (fixup == 1 && !whole) {
        int s = 2 * pid + (nseg ? 1 : 0);
        memcpy(slots + (size_t)s * BM * BN, acc, sizeof(float) * (size_t)BM * BN);
        slot_tile[s] = tile;
      } else {
        for (int i = 0; i < BM && pm * BM + i < M; ++i)
          for (int j = 0; j < BN && pn * BN + j < N; ++j) {
            float *c = C + (size_t)(pm * BM + i) * N + pn * BN + j;
            if (whole) *c = acc[i * BN + j]; else *c += acc[i * BN + j];
          }
      }
      ++nseg;
      start = end;
    }
    for (int p = 0; p < pt.sm_partition_factor; ++p) { /* streamk_fp32.py:149-158 */
      int tile = pid + pt.streamk_tiles + p * P;
      int pm = tile / pt.num_block_n, pn = tile % pt.num_block_n;
      mac_segment(A, B, acc, M, N, K, trans_b, BM, BN, BK, pm, pn, 0, ipt);
      for (int i = 0; i < BM && pm * BM + i < M; ++i)
        for (int j = 0; j < BN && pn * BN + j < N; ++j)
          C[(size_t)(pm * BM + i) * N + pn * BN + j] = acc[i * BN + j];
    }
  }
  if (fixup == 1) {
    /* slots are visited in ascending (pid, segment) order == ascending k within each tile */
    for (int t = 0; t < pt.streamk_tiles; ++t) {
      int pm = t / pt.num_block_n, pn = t % pt.num_block_n, first = 1;
      for (int s = 0; s < 2 * P; ++s) {
        if (slot_tile[s] != t) continue;
        const float *sl = slots + (size_t)s * BM * BN;
        for (int i = 0; i < BM && pm * BM + i < M; ++i)
          for (int j = 0; j < BN && pn * BN + j < N; ++j) {
            float *c = C + (size_t)(pm * BM + i) * N + pn * BN + j;
            if (first) *c = sl[i * BN + j]; else *c += sl[i * BN + j];
          }
        first = 0;
      }
    }
    free(slots);
    free(slot_tile);
  }
  free(acc);
  return 0;
}

/* ---- IEEE binary16 helpers (software; round-to-nearest-even, subnormals kept) ---- */
static float half_bits_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu, f;
  if (e == 0) {
    if (m == 0) f = sign;
    else { int sh = 0; while (!(m & 0x400u)) { m <<= 1; ++sh; } m &= 0x3ffu; f = sign | ((uint32_t)(113 - sh) << 23) | (m << 13); }
  } else if (e == 31) f = sign | 0x7f800000u | (m << 13);
  else f = sign | ((e + 112) << 23) | (m << 13);
  float r; memcpy(&r, &f, 4); return r;
}
static uint16_t float_to_half_bits(float x) {
  uint32_t f; memcpy(&f, &x, 4);
  uint16_t sign = (uint16_t)((f >> 16) & 0x8000u);
  uint32_t a = f & 0x7fffffffu;
  if (a >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((a > 0x7f800000u) ? 0x200u : 0));
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (a < 0x33000001u) return sign;                         /* <= 2^-25 rounds to zero (tie to even) */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13; /* subnormal results lose extra bits */
  uint32_t q = m >> shift, rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1))) ++q;
  if (e < -14) return (uint16_t)(sign | q); /* q may carry into the smallest normal: still right */
  return (uint16_t)(sign | (uint16_t)(((uint32_t)(e + 15) << 10) + (q - 0x400u)));
}

/* streamk_fp16_ladder_block_reduce_q4.py:552: element k of row n is
 * (Wq[n][k/2] >> (4*(k%2))) & 0xF.  The reference stops there (value 0..15 as fp16); with
 * zero = 0 and all scales 1.0 this function reproduces it.  The product (q - zero) * scale is
 * exact in binary32 (|q - zero| < 16, scale has 11 significant bits), so one rounding to binary16
 * equals a single IEEE fp16 multiply. */
void ora_dequant_q4(const uint8_t *Wq, const uint16_t *scales, uint16_t *out, int N, int K, int group,
                    int zero) {
  int ngroups = cdiv(K, group);
  for (int n = 0; n < N; ++n)
    for (int k = 0; k < K; ++k) {
      int q = (Wq[(size_t)n * (K / 2) + k / 2] >> (4 * (k % 2))) & 0xF;
      float s = half_bits_to_float(scales[(size_t)n * ngroups + k / group]);
      out[(size_t)n * K + k] = float_to_half_bits((float)(q - zero) * s);
    }
}

/* conversion helpers exported for the tests that pin them against numpy */
float ora_half_to_float(uint16_t h) { return half_bits_to_float(h); }
uint16_t ora_float_to_half(float x) { return float_to_half_bits(x); }
