/*
 * streamk.h -- C ABI of the MI355X (gfx950) Stream-K GEMM library (libstreamk.so).
 *
 * Plain C: pointers, sizes and PODs only.  Device pointers are ordinary HIP device addresses, the
 * stream argument is a hipStream_t passed as void*.  Every function returns SK_OK (0) or a negative
 * sk_status; nothing throws, nothing allocates or frees caller memory, all device work is enqueued
 * on the caller's stream without a host synchronisation.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * LeiWang1999/Stream-k.tvm checkout).  In the reference the "operator" is a TVM-TL compiled callable
 * `tl_mod(A, B, C)` (streamk_fp32.py:197-202) whose shapes, tiles and partition are compile-time
 * constants; here they are run-time arguments.
 */
#ifndef STREAMK_H_
#define STREAMK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SK_VERSION 100

typedef enum sk_status {
  SK_OK = 0,
  SK_ERR_NULL = -1,        /* a required pointer is NULL */
  SK_ERR_SHAPE = -2,       /* M, N or K <= 0, or a leading dimension smaller than the row */
  SK_ERR_ALIGN = -3,       /* pointer / leading dimension / K not aligned as the kernel needs */
  SK_ERR_CONFIG = -4,      /* tile shape, grid, schedule or fix-up not supported */
  SK_ERR_WORKSPACE = -5,   /* workspace missing or smaller than sk_workspace_bytes() */
  SK_ERR_LAUNCH = -6,      /* HIP reported an error at launch */
  SK_ERR_DEVICE = -7,      /* not a gfx950 device / device query failed */
  SK_ERR_TIMEOUT = -8      /* a fix-up wait gave up (reported by sk_workspace_status) */
} sk_status;

/* B operand layout.  NT: B is [N,K] row-major, C = A * B^T (streamk_fp16.py:131-133).
 *                    NN: B is [K,N] row-major, C = A * B   (streamk_fp32.py:65-76). */
typedef enum sk_layout { SK_LAYOUT_NT = 0, SK_LAYOUT_NN = 1 } sk_layout;

/* How output tiles are split over the persistent grid. */
typedef enum sk_schedule {
  SK_SCHED_AUTO = 0,       /* library heuristic */
  SK_SCHED_DP = 1,         /* data-parallel only: one CTA per tile, ceil(tiles/grid) waves
                              (dataparallel.fp16.breakdown/block_level_gemm.py:36-53) */
  SK_SCHED_SK_TWO_TILE = 2,/* reference hybrid: (tiles % P) + P Stream-K tiles, rest data-parallel
                              (streamk_fp32.py:37-43) */
  SK_SCHED_SK_ONE_TILE = 3,/* tiles % P Stream-K tiles, rest data-parallel */
  SK_SCHED_SK_BASIC = 4,   /* every tile is a Stream-K tile (figures/image.png "basic Stream-K") */
  SK_SCHED_SPLIT_K = 5     /* fixed split: every tile is cut into `split` equal K ranges, one CTA each, grid =
                              tiles * split (the comparator of dataparallel.fp16.breakdown/
                              thread_level_gemm_with_macro_ladder_atomic_reduce.py:129-131,153-154).  split
                              comes from sk_config.reserved[1]; 0 picks the largest factor that divides the
                              K-iterations of a tile, leaves at least 4 of them per CTA and keeps the grid
                              resident.  Both fix-ups apply (the reference's atomicAdd into C is ATOMIC). */
} sk_schedule;

/* How partial tiles of the Stream-K wave are combined. */
typedef enum sk_fixup {
  SK_FIXUP_AUTO = 0,       /* SK_FIXUP_REDUCE */
  SK_FIXUP_ATOMIC = 1,     /* fp32 atomicAdd of partial accumulators (streamk_fp32.py:127-134);
                              summation order varies run to run */
  SK_FIXUP_REDUCE = 2,     /* per-CTA fp32 partial + flag; the tile's first CTA adds the others in
                              ascending CTA order: bitwise reproducible.  One CTA adds a tile's partials one after
                              the other, so a schedule that cuts a few tiles into dozens of segments (an explicit
                              sk1 / sk2 over a handful of remainder tiles) is better served by SK_FIXUP_ATOMIC;
                              the planner's own schedules for the tile kernels keep to at most four contributors per
                              tile (the small-M kernels' partials are a few KB) */
  SK_FIXUP_ATOMIC_C = 3    /* the reference's own fix-up (streamk_fp16.py:248-255, atomic_addx2 on half2): every
                              segment of a split tile rounds its partial sums to C's 16-bit type and adds them
                              into C with packed 16-bit atomic adds; no workspace.  The library zero-fills C
                              first (the reference leaves that to its caller).  Every partial is rounded, so it
                              is less accurate than the other two, and like ATOMIC not reproducible.  fp16 and
                              bfloat16 tile kernels with 16x16 accumulator blocks only (256x256, 128x128,
                              128x256, 256x128); N and ldc even, C 4-byte aligned; no bias / activation */
  ,
  SK_FIXUP_REDUCE16 = 4    /* SK_FIXUP_REDUCE with the exchanged partial sums rounded to C's 16-bit type, as the
                              reference's fix-up rounds them (streamk_fp16.py:248-255), and added in fp32 by the
                              CTA that finishes the tile: half the bytes through memory, which is what the
                              exchange costs (1024 x 8192 x 8192 on 256 x 256 tiles cut in two: 105 -> 97 us).
                              Still the same bits on every launch.  Only for plans whose every Stream-K tile
                              is cut into two or four equal segments on the fp16 / bfloat16 256 x 256 assembly-
                              loop kernel (the fixed split in two or four, `basic` with a grid of two or four
                              CTAs per tile); anything else is refused.  Never chosen by SK_FIXUP_AUTO */
} sk_fixup;

typedef enum sk_dtype {
  SK_F16 = 0,
  SK_F32 = 1,
  SK_Q4 = 2,       /* fp16 A, packed nibbles [N, K/2] row-major */
  SK_BF16 = 3,
  SK_Q4_TILED = 4, /* fp16 A, packed nibbles in 16-row x 64-byte tiles (sk_q4_tile_host / sk_q4_tile) */
  SK_F8E4M3 = 5,   /* A and B one byte per element, OCP e4m3 (bias 7, no infinities, NaN = S.1111.111); C fp16 */
  SK_I8 = 6,       /* A and B int8, C int32 */
  SK_Q4_ZP = 7,    /* as SK_Q4 with one zero point per scale group and row (sk_gemm_q4_zp) */
  SK_F8E5M2 = 8,   /* as SK_F8E4M3 for OCP e5m2 bytes (the upper byte of an fp16: bias 15, infinities and NaNs) */
  SK_Q4_ZP_TILED = 9 /* as SK_Q4_ZP with the nibbles in the tiled layout of SK_Q4_TILED (scales and zero points row-major) */
} sk_dtype;

/* Tunables; a zero field means "choose for me".  Replaces the module-level constants and
 * bitblas Hint of the reference (streamk_fp32.py:24-28, streamk_fp16.py:32-59) and is what the
 * autotuner enumerates (autotune/streamk_fp16_autotune.py:38-53). */
typedef struct sk_config {
  int32_t bm, bn, bk;     /* CTA tile */
  int32_t grid;           /* persistent CTAs; the reference's total_sm (streamk_fp32.py:17) */
  int32_t schedule;       /* sk_schedule */
  int32_t fixup;          /* sk_fixup */
  int32_t raster;         /* g>0: tiles walk g rows down before stepping one column (triton_impl.py:14-28);
                             1 is the reference's row-major order (streamk_fp32.py:106-107); 0: choose
                             (8 for the 16-bit and fp8 tile kernels, row-major otherwise) */
  int32_t spin_limit;     /* REDUCE fix-up: polls of a peer flag before giving up; 0 = default */
  int32_t reserved[4];    /* reserved[0]: 0 = preferred kernel variant of the tile, v > 0 = variant v - 1
                             (implementation alternatives of one tile shape, for the autotuner);
                             reserved[1]: split factor of SK_SCHED_SPLIT_K, 0 = choose;
                             reserved[2]: 1 = interleaved order of the Stream-K tiles (see sk_plan.interleave); with 0 the
                             automatic schedule still chooses it for 256 x 256 tiles whose CTA ranges would start
                             anywhere in their tiles */
} sk_config;

/* Result of the host partitioner: the integers of streamk_fp32.py:30-54 for the chosen tile/grid. */
typedef struct sk_plan {
  int32_t bm, bn, bk, grid, schedule, fixup, raster, dtype, layout;
  int32_t num_block_m, num_block_n, iters_per_tile, total_tiles;
  int32_t streamk_tiles;         /* tile ids [0, streamk_tiles) are split along K */
  int32_t blocking_tiles;        /* tile ids [streamk_tiles, total_tiles) are data-parallel */
  int32_t streamk_iters;         /* streamk_tiles * iters_per_tile */
  int32_t streamk_full_tiles;    /* K-iterations every CTA gets (reference's name kept) */
  int32_t streamk_partial_tiles; /* the first this-many CTAs get one more */
  int32_t dp_waves;              /* ceil(blocking_tiles / grid); the reference's
                                    sm_patition_factor without its max(...,1) */
  int32_t kernel_id;             /* which compiled kernel instance runs this plan */
  int32_t threads;               /* workgroup size of that kernel */
  int32_t lds_bytes;             /* static LDS of that kernel */
  int32_t spin_limit;            /* REDUCE fix-up: polls of a peer's flag before giving up */
  int32_t interleave;            /* 0 or 1: Stream-K tile ids are positions in the tile order; S > 1: tile id v stands
                                    at position (v % S) * (streamk_tiles / S) + v / S of it.  With g =
                                    gcd(streamk_tiles, grid) and S = streamk_tiles / g, the CTAs pid, pid + grid/g,
                                    pid + 2 grid/g, ... are at the same K offset of their tiles at the same time
                                    (their ranges start S tiles apart); the interleaved order puts the g tiles they
                                    work on next to each other in the tile order, so that with a grouped raster they
                                    share rows of A and columns of B while those are in the L2, as the tiles of a
                                    data-parallel wave do.  Those CTAs sit on one XCD when grid/g is a multiple of 8. */
  int64_t workspace_bytes;       /* what sk_gemm_* needs for this plan (0: data-parallel, ATOMIC_C, or CTA ranges that are whole tiles) */
  int64_t M, N, K;
} sk_plan;

int sk_version(void);
const char *sk_strerror(int status);
/* Name of the compiled kernel instance a plan runs (sk_plan.kernel_id), e.g. for reading profiler
 * output; NULL for an unknown id.  The reference names its generated kernel after the script. */
const char *sk_kernel_name(int kernel_id);
/* Consistency of the compiled-in kernel table (every instance has a name and an id of its own, below 512):
 * SK_OK, or SK_ERR_CONFIG for a library that was built wrong.  Needs no GPU. */
int sk_selfcheck(void);

/* Number of compute units and max co-resident CTAs per CU are read from the current HIP device.
 * Replaces `total_sm = 108` (streamk_fp32.py:17). */
int sk_device_info(int *num_cus, int *clock_khz, int *lds_bytes_per_cu);

/*
 * Host partitioner (pure integer arithmetic, no GPU needed when num_cus > 0 is given).
 * Replaces streamk_fp32.py:30-54 / streamk_fp16.py:92-113.
 *   dtype/layout select the kernel family; cfg may be NULL (all heuristic).
 */
int sk_make_plan(int64_t M, int64_t N, int64_t K, int dtype, int layout, const sk_config *cfg,
                 int num_cus, sk_plan *out);

/* K-iteration range [start, last) of CTA pid in the Stream-K wave (streamk_fp32.py:93-96). */
int sk_plan_cta_range(const sk_plan *plan, int pid, int32_t *start, int32_t *last);

/* Tile id -> (pid_m, pid_n) under the plan's raster (streamk_fp32.py:106-107). */
int sk_plan_tile_coords(const sk_plan *plan, int tile, int32_t *pid_m, int32_t *pid_n);

/* Workspace the plan needs (partials, flags / counters, status word).  0 is possible. */
size_t sk_workspace_bytes(const sk_plan *plan);

/* Must be run once on a freshly allocated workspace (and after an SK_ERR_TIMEOUT); kernels leave
 * flags and counters clean for the next launch, and the workspace itself records whether its partial
 * area holds leftovers (REDUCE launches leave partial tiles behind, ATOMIC launches need zeroed
 * accumulators: every ATOMIC launch is preceded by a small kernel that zero-fills the area if, and as
 * far as, it is marked dirty).  That record lives in device memory, so launches replayed from a HIP
 * graph see what really ran before them: one workspace may serve eager and captured launches of both
 * fix-ups, as long as they do not overlap in time.  Uses a fill kernel, so it may be graph-captured.
 * The library remembers which addresses were initialised (launches on any other workspace return
 * SK_ERR_WORKSPACE); sk_workspace_release forgets one -- call it before freeing the buffer, so that a
 * later allocation at the same address is not mistaken for it.  No counterpart in the reference, whose
 * kernels use no workspace (atomicAdd into a pre-zeroed C, streamk_fp16.py:248-255,385). */
int sk_workspace_init(void *ws, size_t ws_bytes, void *stream);
int sk_workspace_release(void *ws);

/* Reads the workspace status word (synchronises the stream): SK_OK or SK_ERR_TIMEOUT.  A fix-up wait
 * that timed out stored an incomplete tile to C and may have left flags raised: once this call has
 * reported it, every launch on the workspace returns SK_ERR_TIMEOUT until sk_workspace_init has run on
 * it again.  Callers that set a small spin_limit should poll this at their synchronisation points. */
int sk_workspace_status(void *ws, void *stream);

/*
 * fp16 GEMM, fp32 accumulate, fp16 out.  C[M,N] (ldc) = A[M,K] (lda) * op(B).
 * Replaces tl_mod(A, B, C) of streamk_fp16.py:382-387.  C need not be zeroed by the caller
 * (the reference requires it, streamk_fp16.py:385).
 * Requirements: K, lda, ldb multiples of 8 and 16-byte aligned A, B (vector loads).
 * Results are the same bits on every launch of a plan with the data-parallel, fixed-split or any schedule with
 * the REDUCE fix-up.  The order in which a tile's K-iterations are summed is the kernel's: the kernels that take
 * 5 to 64 rows of A (2 to 4 on large weights) start each tile at a different K offset and wrap around, so two
 * tiles of one launch do not add their products in the same order.
 */
int sk_gemm_f16(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws, size_t ws_bytes,
                void *stream);

/*
 * sk_gemm_f16 without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * The partial tiles and flags of the fix-up live in an array that is part of the library's code object: one
 * copy of SK_STATIC_WORKSPACE_BYTES per GPU, held until the process ends.  The call allocates and frees
 * nothing; every call is preceded by a small kernel that clears the flags the plan uses (and, for the ATOMIC
 * fix-up, zero-fills the accumulators if an earlier call left partial tiles there).  A plan whose
 * sk_workspace_bytes() exceeds SK_STATIC_WORKSPACE_BYTES is refused with SK_ERR_WORKSPACE (the limit covers
 * every fp16 plan up to 256 partial tiles of 256 x 256, e.g. M = N = K = 8192 with the two-tile Stream-K
 * schedule on 256 CUs).  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (two streams, two threads) race; serialise them.  There is no status word to poll: a fix-up wait that gives
 * up (spin_limit) leaves its tile incomplete as with sk_gemm_f16, but unreported -- callers that lower
 * spin_limit should use sk_gemm_f16 with their own workspace.
 *
 * sk_static_init() looks up the array's address on the current device (one symbol query per device and
 * process; later calls return at once).  sk_gemm_f16_static does the same on its first call on a device, so
 * the call is optional -- except for callers that record sk_gemm_f16_static into a HIP graph: they call
 * sk_static_init() on that device before the capture begins, so that the capture holds kernel launches only.
 * No counterpart in the reference.
 */
#define SK_STATIC_WORKSPACE_BYTES (64u * 1024u * 1024u + 262144u + 256u)
int sk_static_init(void);
int sk_gemm_f16_static(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                       int64_t ldb, int64_t ldc, const sk_plan *plan, void *stream);

/* Optional epilogue of the *_ex entry points (NULL = none): bias points at N device values of C's type
 * (fp16, or bfloat16 for sk_gemm_bf16_ex) that are added to every row of C in fp32 before the rounding --
 * the bias of a linear layer, which the reference leaves to a separate kernel -- or is NULL; activation
 * (an sk_activation, 0 = none) is applied after the bias, also in fp32 -- the nonlinearity of an MLP's
 * first projection.  Fix-ups are unaffected (partials stay linear; the CTA that stores a tile applies the
 * epilogue).  reserved must be zero. */
typedef enum sk_activation {
  SK_ACT_NONE = 0,
  SK_ACT_RELU = 1,      /* max(x, 0) */
  SK_ACT_GELU_TANH = 2, /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) */
  SK_ACT_SILU = 3       /* x / (1 + exp(-x)) */
} sk_activation;

typedef struct sk_epilogue {
  const void *bias;
  int64_t activation;
  int64_t reserved[2];
} sk_epilogue;

int sk_gemm_f16_ex(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                   int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws, size_t ws_bytes, void *stream,
                   const sk_epilogue *epi);
int sk_gemm_bf16_ex(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                    int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws, size_t ws_bytes, void *stream,
                    const sk_epilogue *epi);
/* Q4 with the epilogue: zeros == NULL is sk_gemm_q4 (plan dtype SK_Q4 or SK_Q4_TILED, scalar `zero`),
 * otherwise sk_gemm_q4_zp (plan dtype SK_Q4_ZP or SK_Q4_ZP_TILED, `zero` ignored). */
int sk_gemm_q4_ex(const void *A, const void *Wq, const void *scales, const void *zeros, void *C, int64_t M,
                  int64_t N, int64_t K, int64_t lda, int64_t ldc, int group, int zero, const sk_plan *plan,
                  void *ws, size_t ws_bytes, void *stream, const sk_epilogue *epi);

/* The same call for bfloat16 operands and output (fp32 accumulate, C rounded to nearest even); the
 * plan is made with dtype SK_BF16.  No counterpart in the reference, whose scripts are fp16 / fp32:
 * the tile kernels with the bfloat16 form of the MFMA.  Requirements as for sk_gemm_f16. */
int sk_gemm_bf16(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                 int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws, size_t ws_bytes, void *stream);

/* fp8 operands: A [M,K] and B [N,K] (NT only) hold OCP e4m3 bytes, C is fp16, accumulation fp32;
 * the plan is made with dtype SK_F8E4M3 (its bk counts fp8 elements), or SK_F8E5M2 for OCP e5m2 bytes (the
 * dtype of the plan tells sk_gemm_f8 which format both operands are in).  No counterpart in the
 * reference's scripts; its Triton comparator takes whatever dtype its inputs have
 * (triton.streamk/first_wave.py:123 picks the accumulator type from them).  Same partitioner,
 * fix-ups and workspace rules as sk_gemm_f16.  K, lda and ldb multiples of 16; A and B 16-byte
 * aligned.  C = fp16_rn(alpha * (A B^T)): alpha (finite; the product of the two per-tensor scales of
 * a scaled-fp8 caller, 1 for none) multiplies the fp32 sums before they are rounded, so sums beyond
 * fp16's range can be brought back into it. */
int sk_gemm_f8(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
               int64_t ldb, int64_t ldc, float alpha, const sk_plan *plan, void *ws, size_t ws_bytes,
               void *stream);
/* The same with the epilogue of the *_ex entry points: C = activation(alpha * A B^T + bias), bias in fp16
 * (C's type). */
int sk_gemm_f8_ex(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                  int64_t ldb, int64_t ldc, float alpha, const sk_plan *plan, void *ws, size_t ws_bytes,
                  void *stream, const sk_epilogue *epi);

/* int8 operands: A [M,K] and B [N,K] (NT only) int8, C int32 (ldc in int32 elements), exact int32
 * accumulation (wraps beyond 2^31, i.e. not below K = 133 000); the plan is made with dtype SK_I8.  The
 * reference's Triton comparator accumulates integer inputs in int32 (triton.streamk/first_wave.py:123).
 * Partial tiles are int32 too, so every schedule and both fix-ups give the same bits.  K, lda and ldb
 * multiples of 16; A and B 16-byte aligned; C 4-byte aligned (16 bytes and ldc a multiple of 4 for
 * vector stores). */
int sk_gemm_i8(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
               int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws, size_t ws_bytes, void *stream);

/* fp32 GEMM (fp32 MFMA, fp32 out).  Replaces tl_mod(A, B, C) of streamk_fp32.py:197-202. */
int sk_gemm_f32(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int64_t lda,
                int64_t ldb, int64_t ldc, const sk_plan *plan, void *ws, size_t ws_bytes,
                void *stream);

/*
 * Q4 weight-only GEMM: C[M,N] fp16 = A[M,K] fp16 * dequant(Wq)^T.
 *   Wq      [N, K/2] bytes, element k of row n = (Wq[n][k/2] >> 4*(k&1)) & 0xF
 *           (streamk.fp16.breakdown/streamk_fp16_ladder_block_reduce_q4.py:552)
 *   scales  [N, K/group] fp16, w = fp16_rn((fp16(q) - zero) * scale)
 * Replaces tl_mod(A, QLB, C) of streamk_fp16_ladder_block_reduce_q4.py:597-599; the weights stay in
 * the natural byte order above (no LadderPermutate / LOP3Permutate step, :568-595).
 * Requirements: K multiple of 128, group == 128, 0 <= zero <= 15.
 * Up to 16 rows of A (the matrix-vector kernels for M == 1; the 16-row kernels with a scalar zero point)
 * the nibbles are multiplied undecoded and zero point and scale are applied to fp32 group sums, i.e.
 * these kernels use the unrounded (q - zero) * scale: at least as close to the exact product as the
 * rounded-weight form (within 2^-11 relative per weight of it).
 * sk_dequant_q4, the kernels for more than 16 rows and the per-group zero-point kernels for M > 1
 * produce the rounded weights bit for bit.
 * Up to 64 rows of A the plan is a weight-streaming kernel; for more rows (plan dtype SK_Q4) it is a tile kernel
 * that moves the nibbles through LDS and dequantises them, bit for bit as above, on their way into the fp16
 * stage of the 16x16x32 MFMA loop (256x256, 256x128 or 128x128 tiles; every schedule and fix-up).
 * A plan made with dtype SK_Q4_TILED takes Wq in the tiled layout instead (see sk_q4_tile_host): same
 * results bit for bit, the weights stream faster; at most 64 rows of A per call.
 */
int sk_gemm_q4(const void *A, const void *Wq, const void *scales, void *C, int64_t M, int64_t N,
               int64_t K, int64_t lda, int64_t ldc, int group, int zero, const sk_plan *plan,
               void *ws, size_t ws_bytes, void *stream);

/* The same with one zero point per scale group and row: zeros [N, K/group] fp16 holding integers 0..15,
 * w = fp16_rn((fp16(q) - zeros[n][k/group]) * scales[n][k/group]) -- the asymmetric formats of weight-only
 * quantisers (min/max per group), which the reference's unsigned nibbles with one implied zero point do
 * not cover.  The plan is made with dtype SK_Q4_ZP; at most 64 rows per call.  M == 1 takes matrix-vector kernels
 * that, like sk_gemm_q4's, multiply the nibbles undecoded and apply zero point and scale to fp32 group sums (the
 * unrounded (q - zero) * scale); 2 <= M <= 64, and M == 1 with an explicit variant-0 plan, the general small-M
 * kernels, which form the rounded weights bit for bit.
 * A plan made with dtype SK_Q4_ZP_TILED takes Wq in the tiled layout (sk_q4_tile_host / sk_q4_tile; scales and
 * zeros stay row-major): the same kernels with the tiled loads, results bit for bit those of SK_Q4_ZP. */
int sk_gemm_q4_zp(const void *A, const void *Wq, const void *scales, const void *zeros, void *C, int64_t M,
                  int64_t N, int64_t K, int64_t lda, int64_t ldc, int group, const sk_plan *plan, void *ws,
                  size_t ws_bytes, void *stream);
int sk_dequant_q4_zp(const void *Wq, const void *scales, const void *zeros, void *W, int64_t N, int64_t K,
                     int group, void *stream);
/* Asymmetric group-wise quantiser producing that format (host memory / device memory, same bytes):
 *   lo = min(min w, 0), hi = max(max w, 0) over the group;  scale = fp16_rn((hi - lo) / 15)
 *   z = clamp(rint(-lo / scale), 0, 15);  q = clamp(rint(w / scale) + z, 0, 15);  scale 0: z = q = 0
 * (fp32 arithmetic, ties to even).  zeros is written as fp16 (uint16_t bit patterns on the host). */
int sk_q4_quantize_zp_host(const uint16_t *W, int64_t N, int64_t K, int64_t ldw, int group, uint8_t *Wq,
                           uint16_t *scales, uint16_t *zeros);
int sk_q4_quantize_zp(const void *W, int64_t N, int64_t K, int64_t ldw, int group, void *Wq, void *scales,
                      void *zeros, void *stream);

/* Device dequantisation of Wq into fp16 W[N,K] with the device function the M > 1 GEMM uses
 * (the closed form of streamk_fp16_ladder_block_reduce_q4.py:548-554 plus zero/scale). */
int sk_dequant_q4(const void *Wq, const void *scales, void *W, int64_t N, int64_t K, int group,
                  int zero, void *stream);

/*
 * Offline side of the Q4 path: what produces Wq and scales.  The reference packs two nibbles per
 * byte (streamk_fp16_ladder_block_reduce_q4.py:545,552) and then runs BitBLAS LadderPermutate and
 * LOP3Permutate over the array on the CPU (:568-595); this library reads the packed array as it is,
 * so these calls replace that whole step.
 *
 * sk_q4_pack_host / sk_q4_unpack_host: q[N,K] bytes with values 0..15 <-> Wq[N,K/2] (host memory).
 * sk_q4_quantize_host (host memory, W as fp16 bit patterns, row pitch ldw elements) and
 * sk_q4_quantize (device memory, stream-ordered; group must be 128, ldw a multiple of 8, W 16-byte
 * aligned) quantise fp16 weights group by group:
 *   levels = min(zero, 15 - zero), or 15 if that is 0;  scale = fp16_rn(max|w| / levels);
 *   q = clamp(rint(w / scale) + zero, 0, 15), divisions in fp32, ties to even; q = zero if scale is 0.
 * Both produce the same bytes.  Weights must be finite (the host call returns SK_ERR_CONFIG otherwise,
 * the device call does not look).
 */
int sk_q4_pack_host(const uint8_t *q, int64_t N, int64_t K, uint8_t *Wq);
/* Tiled layout of the packed weights, the MI355X-side counterpart of the reference's weight
 * pre-transformation (LadderPermutate, streamk_fp16_ladder_block_reduce_q4.py:568-580): byte b of row
 * n of Wq[N, K/2] moves to ((n/16) * (K/128) + b/64) * 1024 + (n%16) * 64 + b%64, i.e. tiles of 16 rows
 * x 64 bytes (one scale group), row by row inside a tile.  N is padded to a multiple of 16 with zero
 * rows: the tiled array has ceil(N/16)*16 * K/2 bytes.  K must be a multiple of 128.
 * sk_q4_tile_host / sk_q4_untile_host work on host memory, sk_q4_tile on device memory (stream-ordered). */
int sk_q4_tile_host(const uint8_t *Wq, int64_t N, int64_t K, uint8_t *tiled);
int sk_q4_untile_host(const uint8_t *tiled, int64_t N, int64_t K, uint8_t *Wq);
int sk_q4_tile(const void *Wq, int64_t N, int64_t K, void *tiled, void *stream);
int sk_q4_unpack_host(const uint8_t *Wq, int64_t N, int64_t K, uint8_t *q);
int sk_q4_quantize_host(const uint16_t *W, int64_t N, int64_t K, int64_t ldw, int group, int zero,
                        uint8_t *Wq, uint16_t *scales);
int sk_q4_quantize(const void *W, int64_t N, int64_t K, int64_t ldw, int group, int zero, void *Wq,
                   void *scales, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* STREAMK_H_ */
