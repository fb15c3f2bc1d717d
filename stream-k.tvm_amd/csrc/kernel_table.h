// Registry of compiled kernel instances.  The host partitioner picks one by (dtype, layout, tile);
// the launchers switch on its id.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace sk {

// Workspace layout (bytes): [0,256) status block; [256, 256+WS_FLAG_BYTES) flags (REDUCE: one per
// CTA) or arrival counters (ATOMIC: one per Stream-K tile); then the fp32 partial tiles.  The flag
// area has a fixed size so that partial tiles of one plan never land where another plan keeps
// its flags.  The words of the status block are named in sk_device.h (WS_STATUS, ...).
constexpr int64_t WS_FLAG_BYTES = 262144;
constexpr int64_t WS_PART_OFF = 256 + WS_FLAG_BYTES;
constexpr int64_t WS_MAX_FLAGS = WS_FLAG_BYTES / 4;

enum Family { FAMILY_TILE = 0, FAMILY_SKINNY = 1 };

struct KernelInfo {
  int id;
  int family;
  int dtype;    // sk_dtype
  int layout;   // sk_layout
  int variant;  // tile kernels -- 0: registers -> padded LDS rows; 1: direct global -> LDS loads,
                // swizzled rows; 2: as 1 with four waves per CTA (one per SIMD, accumulators in AGPRs);
                // 3: as 1 with BK = 32 and four LDS stages (loads three iterations ahead);
                // 4: as 1 with 16x16x32 MFMAs; 5: as 3 with 16x16x32 MFMAs; 6: as 1 for fp8 operands (32x32x64 MFMAs);
                // 7: as 4 with four waves per CTA, the K loop in assembly and the accumulators in a[0:255]
                // small-M kernels -- 0: up to 16*MB rows of A; 1: M == 1; 2: M == 1, matrix-vector on 4x4x4 MFMA;
                // 3: the matrix-vector form with up to four rows of A; 4: weights streamed through LDS in contiguous loads
  int bm, bn, bk;  // CTA tile; bk is the K extent of one CTA iteration
  int threads;
  int lds_bytes;
  int ctas_per_cu;    // co-resident CTAs per CU the kernel is compiled for
  int partial_elems;  // fp32 elements of one partial tile in the workspace
  int max_ipt;        // largest iterations-per-tile the kernel supports (0 = unlimited)
  int max_m;          // small-M kernels: largest M the kernel accepts (0 = unlimited)
  int k_align;        // K must be a multiple of this
  const char *name;
};

// fp16 LDS-tiled kernels, NT layout:  X(id, BM, BN, BK, WM, WN)
#define SK_TILE_F16_NT_KERNELS(X) \
  X(1, 128, 128, 64, 2, 2)        \
  X(2, 128, 256, 64, 2, 4)        \
  X(3, 256, 128, 64, 4, 2)        \
  X(4, 64, 64, 64, 2, 2)          \
  X(6, 128, 128, 32, 2, 2)

// fp16 LDS-tiled kernels with direct-to-LDS loads (BK = 64), NT layout:  X(id, BM, BN, WM, WN)
#define SK_TILE_F16_NT_DMA_KERNELS(X) \
  X(11, 128, 128, 2, 2)               \
  X(12, 128, 256, 2, 4)               \
  X(13, 256, 128, 4, 2)               \
  X(24, 64, 64, 2, 2)                 \
  X(25, 128, 64, 2, 2)                \
  X(26, 64, 128, 2, 2)

// direct-to-LDS loads, BK = 32, four stages (variant 3), NT layout:  X(id, BM, BN, WM, WN)
#define SK_TILE_F16_NT_DMA32_KERNELS(X) \
  X(16, 128, 128, 2, 2)                 \
  X(17, 128, 256, 2, 4)                 \
  X(18, 256, 128, 4, 2)                 \
  X(27, 64, 64, 2, 2)                   \
  X(28, 128, 64, 2, 2)                  \
  X(29, 64, 128, 2, 2)

// direct-to-LDS loads, BK = 64, arithmetic on v_mfma_f32_16x16x32_f16 (variant 4), NT layout:  X(id, BM, BN, WM, WN)
#define SK_TILE_F16_NT_DMA16_KERNELS(X) \
  X(30, 256, 256, 2, 4)                 \
  X(31, 128, 128, 2, 2)                 \
  X(32, 128, 256, 2, 4)                 \
  X(33, 256, 128, 4, 2)

// BK = 32, four stages, 16x16x32 MFMAs (variant 5), NT layout:  X(id, BM, BN, WM, WN)
#define SK_TILE_F16_NT_DMA32_16_KERNELS(X) \
  X(36, 128, 128, 2, 2)                    \
  X(37, 128, 256, 2, 4)                    \
  X(38, 256, 128, 4, 2)                    \
  X(39, 64, 64, 2, 2)                      \
  X(40, 128, 64, 2, 2)                     \
  X(41, 64, 128, 2, 2)

// the same for the NN layout (B is [K,N]), fragments through transposing LDS reads:  X(id, BM, BN, WM, WN)
#define SK_TILE_F16_NN_DMA_KERNELS(X) \
  X(21, 128, 128, 2, 2)               \
  X(22, 128, 256, 2, 4)               \
  X(23, 256, 128, 4, 2)

// small-M kernels:  X(id, MB, NB, WN, RK, Q4, DEPTH, ROW1)
#define SK_SKINNY_KERNELS(X)     \
  X(100, 1, 1, 4, 1, 0, 2, 0)    \
  X(101, 2, 1, 4, 1, 0, 2, 0)    \
  X(102, 4, 1, 4, 1, 0, 2, 0)    \
  X(103, 1, 1, 1, 4, 0, 2, 0)    \
  X(104, 1, 1, 2, 2, 0, 2, 0)    \
  X(105, 1, 1, 1, 1, 0, 4, 1)    \
  X(106, 1, 1, 4, 1, 0, 4, 1)    \
  X(107, 1, 1, 2, 4, 0, 2, 0)    \
  X(108, 1, 1, 4, 2, 0, 2, 0)    \
  X(109, 2, 1, 4, 2, 0, 2, 0)    \
  X(110, 4, 1, 4, 2, 0, 2, 0)    \
  X(120, 1, 1, 4, 1, 1, 4, 0)    \
  X(121, 2, 1, 4, 1, 1, 2, 0)    \
  X(122, 4, 1, 4, 1, 1, 2, 0)    \
  X(123, 1, 1, 1, 4, 1, 4, 0)    \
  X(124, 1, 1, 2, 2, 1, 4, 0)    \
  X(125, 1, 1, 1, 1, 1, 4, 1)    \
  X(126, 1, 1, 4, 1, 1, 4, 1)    \
  X(127, 1, 2, 1, 1, 1, 4, 1)    \
  X(128, 1, 2, 2, 1, 1, 4, 1)    \
  X(129, 1, 4, 1, 1, 1, 2, 1)    \
  X(130, 1, 2, 1, 2, 1, 4, 1)    \
  X(131, 1, 1, 2, 4, 1, 2, 0)    \
  X(132, 1, 1, 4, 2, 1, 2, 0)

// bfloat16 twins of the fp16 small-M kernels above (dtype SK_BF16):  X(id, MB, NB, WN, RK, DEPTH, ROW1)
#define SK_SKINNY_BF16_KERNELS(X) \
  X(230, 1, 1, 4, 1, 2, 0)        \
  X(231, 2, 1, 4, 1, 2, 0)        \
  X(232, 4, 1, 4, 1, 2, 0)        \
  X(233, 1, 1, 1, 4, 2, 0)        \
  X(234, 1, 1, 2, 2, 2, 0)        \
  X(235, 1, 1, 1, 1, 4, 1)        \
  X(236, 1, 1, 4, 1, 4, 1)        \
  X(237, 1, 1, 2, 4, 2, 0)        \
  X(238, 1, 1, 4, 2, 2, 0)        \
  X(239, 2, 1, 4, 2, 2, 0)        \
  X(240, 4, 1, 4, 2, 2, 0)

// M == 1 Q4 matrix-vector kernels (variant 2):  X(id, NB, WN, RK, DEPTH, KMAX)
// KMAX is the largest K range one segment may span (A is kept in LDS for the whole segment).
#define SK_GEMV_Q4_KERNELS(X)  \
  X(140, 1, 4, 1, 4, 16384)    \
  X(141, 1, 2, 2, 4, 16384)    \
  X(142, 1, 1, 4, 4, 16384)    \
  X(143, 2, 4, 1, 2, 16384)    \
  X(144, 1, 4, 2, 4, 16384)    \
  X(145, 1, 2, 1, 4, 16384)    \
  X(146, 1, 1, 2, 4, 16384)    \
  X(147, 1, 1, 1, 4, 16384)    \
  X(148, 1, 2, 4, 4, 16384)    \
  X(149, 1, 1, 8, 4, 16384)    \
  X(150, 1, 1, 4, 4, 32768)    \
  X(151, 1, 2, 4, 4, 32768)

// M == 1 with per-group zero points (dtype SK_Q4_ZP): the matrix-vector kernels with the zero points staged beside
// the scales:  X(id, NB, WN, RK, DEPTH, KMAX)
#define SK_GEMV_Q4ZP_KERNELS(X) \
  X(152, 1, 1, 4, 4, 16384)     \
  X(153, 1, 2, 2, 4, 16384)     \
  X(154, 1, 4, 1, 4, 16384)     \
  X(155, 1, 1, 4, 4, 32768)

// Q4 kernels reading tiled weights (dtype SK_Q4_TILED), same variants as their row-major twins.
// general small-M:  X(id, MB, NB, WN, RK, DEPTH);  matrix-vector:  X(id, NB, WN, RK, DEPTH, KMAX)
#define SK_SKINNY_Q4T_KERNELS(X) \
  X(180, 1, 1, 4, 1, 4)          \
  X(181, 2, 1, 4, 1, 2)          \
  X(182, 4, 1, 4, 1, 2)          \
  X(183, 1, 1, 1, 4, 4)          \
  X(184, 1, 1, 2, 2, 4)
#define SK_GEMV_Q4T_KERNELS(X) \
  X(190, 1, 4, 1, 4, 16384)    \
  X(191, 1, 2, 2, 4, 16384)    \
  X(192, 1, 1, 4, 4, 16384)    \
  X(193, 1, 2, 4, 4, 16384)    \
  X(194, 1, 1, 4, 4, 32768)

// Q4 with one zero point per group and row (dtype SK_Q4_ZP), general small-M kernels:  X(id, MB, NB, WN, RK, DEPTH)
#define SK_SKINNY_Q4ZP_KERNELS(X) \
  X(220, 1, 1, 4, 1, 4)           \
  X(221, 2, 1, 4, 1, 2)           \
  X(222, 4, 1, 4, 1, 2)           \
  X(223, 1, 1, 2, 4, 2)           \
  X(224, 1, 1, 4, 2, 2)           \
  X(225, 1, 1, 1, 4, 4)

// Per-group zero points with tiled weights (dtype SK_Q4_ZP_TILED): twins of SK_GEMV_Q4ZP_KERNELS and
// SK_SKINNY_Q4ZP_KERNELS (translation unit kernels_gemv_rows.hip)
#define SK_GEMV_Q4ZPT_KERNELS(X) \
  X(156, 1, 1, 4, 4, 16384)      \
  X(157, 1, 2, 2, 4, 16384)      \
  X(158, 1, 1, 4, 4, 32768)      \
  X(159, 1, 4, 1, 4, 16384)
#define SK_SKINNY_Q4ZPT_KERNELS(X) \
  X(300, 1, 1, 4, 1, 4)            \
  X(301, 2, 1, 4, 1, 2)            \
  X(302, 4, 1, 4, 1, 2)            \
  X(303, 1, 1, 2, 4, 2)            \
  X(304, 1, 1, 4, 2, 2)            \
  X(305, 1, 1, 1, 4, 4)

// M == 1 fp16 (NT) matrix-vector kernels (variant 2):  X(id, NB, WN, RK, DEPTH, KMAX)
#define SK_GEMV_F16_KERNELS(X) \
  X(160, 1, 1, 4, 4, 8192)     \
  X(161, 1, 1, 8, 4, 8192)     \
  X(162, 2, 1, 4, 2, 8192)     \
  X(163, 1, 4, 1, 4, 8192)     \
  X(164, 1, 2, 2, 4, 8192)     \
  X(165, 1, 1, 2, 4, 8192)     \
  X(166, 1, 1, 4, 4, 32768)    \
  X(167, 2, 1, 4, 2, 32768)

// fp8 small-M kernels (dtypes SK_F8E4M3 and SK_F8E5M2, one instance each; the second id is the first + 10);
// bk counts fp8 elements:  X(id, MB, NB, WN, RK, DEPTH, ROW1)
#define SK_SKINNY_F8_KERNELS(X) \
  X(250, 1, 1, 4, 1, 2, 0)      \
  X(251, 2, 1, 4, 1, 2, 0)      \
  X(252, 1, 1, 1, 4, 2, 0)      \
  X(253, 1, 1, 2, 2, 2, 0)      \
  X(254, 1, 1, 2, 4, 2, 0)      \
  X(255, 1, 1, 4, 2, 2, 0)      \
  X(256, 2, 1, 4, 2, 2, 0)      \
  X(257, 1, 1, 4, 1, 4, 1)      \
  X(258, 4, 1, 4, 1, 2, 0)      \
  X(259, 4, 1, 4, 2, 2, 0)

// int8 small-M kernels (dtype SK_I8, int32 C); bk counts int8 elements:  X(id, MB, NB, WN, RK, DEPTH, ROW1)
#define SK_SKINNY_I8_KERNELS(X) \
  X(270, 1, 1, 4, 1, 2, 0)      \
  X(271, 2, 1, 4, 1, 2, 0)      \
  X(272, 1, 1, 1, 4, 2, 0)      \
  X(273, 1, 1, 2, 2, 2, 0)      \
  X(274, 1, 1, 2, 4, 2, 0)      \
  X(275, 1, 1, 4, 2, 2, 0)      \
  X(276, 2, 1, 4, 2, 2, 0)      \
  X(277, 1, 1, 4, 1, 4, 1)      \
  X(278, 4, 1, 4, 1, 2, 0)      \
  X(279, 4, 1, 4, 2, 2, 0)

// 2 <= M <= 4, fp16 / bfloat16 weights (NT): the matrix-vector kernels' quad-coalesced weight stream against up to
// MR rows of A (variant 3):  X(id, MR, WN, RK, DEPTH).  (Instances with MR = 8 and 16 were measured and are not
// kept: every row of A costs a 16-byte LDS read per weight load and lane, and from 8 rows on that traffic, not
// the weight stream, sets the time -- 43 and 57 us at 8192 x 8192 against 33 us for the general kernel.)
#define SK_GEMV_ROWS_F16_KERNELS(X) \
  X(168, 4, 1, 4, 4)                \
  X(169, 4, 2, 4, 2)                \
  X(170, 4, 4, 2, 2)
#define SK_GEMV_ROWS_BF16_KERNELS(X) \
  X(210, 4, 1, 4, 4)                 \
  X(211, 4, 2, 4, 2)

// Up to 16 / 32 / 64 rows of A, fp16 / bfloat16 weights (NT), the weights streaming through LDS in contiguous loads
// (tile_stream_pairs.h; variant 4):  X(id, MB, WM, WN, RK, DEPTH)
#define SK_STREAM_PAIRS_F16_KERNELS(X) \
  X(280, 1, 1, 4, 1, 4)                \
  X(281, 2, 1, 4, 1, 3)                \
  X(284, 1, 1, 2, 2, 3)                \
  X(286, 2, 2, 2, 1, 3)                \
  X(288, 1, 2, 2, 1, 4)
#define SK_STREAM_PAIRS_BF16_KERNELS(X) \
  X(282, 1, 1, 4, 1, 4)                 \
  X(283, 2, 1, 4, 1, 3)                 \
  X(285, 1, 1, 2, 2, 3)                 \
  X(287, 2, 2, 2, 1, 3)                 \
  X(289, 1, 2, 2, 1, 4)

// the same with NB blocks of 16 weight rows per wave, AD slots of A and the unpadded rings (64 x 64 tiles: the 160 KB
// of LDS exactly; 16 x 16 tiles with K split over the four waves: the same), and two waves sharing the K-steps of each
// of those four (eight waves per CTA); 96 x 32 tiles (three blocks of rows per wave, four slots of weights and two of
// A: the 160 KB as well) for 65 to 96 rows where N gives every CU a tile:  X(id, MB, WM, WN, RK, DEPTH, NB, AD, BF16)
#define SK_STREAM_BLOCKS_KERNELS(X)  \
  X(292, 2, 2, 2, 1, 3, 2, 2, false) \
  X(293, 2, 2, 2, 1, 3, 2, 2, true)  \
  X(296, 1, 1, 1, 4, 3, 1, 2, false) \
  X(297, 1, 1, 1, 4, 3, 1, 2, true)  \
  X(298, 3, 2, 2, 1, 4, 1, 2, false) \
  X(299, 3, 2, 2, 1, 4, 1, 2, true)

// Up to 16 rows of A, Q4 weights (row-major, scalar zero point) streaming through LDS in contiguous loads
// (tile_stream_q4.h; dtype SK_Q4, variant 4):  X(id, WN, RK, KH, WD, AD)
#define SK_STREAM_Q4_KERNELS(X) \
  X(290, 4, 1, 4, 4, 4)         \
  X(291, 2, 2, 4, 3, 3)
// (the 32-row instance asks for A two iterations ahead, three slots of each ring: with five slots of weights and two
// of A -- A requested one iteration ahead -- 16 x 8192 x 8192 took 13.2 us from HBM against 12.2, 11.6 / 10.7 with the
// weights in the Infinity Cache; four waves per ring instead of two: 10.7 -> 10.2, the 64-row instance 31.7 -> 28.9 us
// at 16 x 16384 x 16384, 37.7 -> 36.2 from HBM)
// (an instance of 32 weight rows with 512 instead of 1024 K-values per iteration, eight waves and six slots of A
// -- X(294, 2, 1, 4, 4, 6), weights issued before A -- was measured and is not built: 16 x 8192 x 8192 13.6 us from HBM
// against 12.1, 12.6 / 10.2 with the weights in the Infinity Cache)
// (an instance with eight rings, 128 weight rows and one wave per ring -- X(294, 8, 1, 1, 3, 3): half the bytes of A per
// byte of weights -- was measured and is not built: 16 x 16384 x 16384 split in two over K 39.7 us against 39.4 for the
// 64-row instance and 37.5 for the general kernel, 16 x 8192 x 8192 17.8 against 13.8)

// bfloat16 twins of the fp16 matrix-vector kernels (dtype SK_BF16, variant 2)
#define SK_GEMV_BF16_KERNELS(X) \
  X(241, 1, 1, 4, 4, 8192)      \
  X(242, 1, 1, 8, 4, 8192)      \
  X(243, 2, 1, 4, 2, 8192)      \
  X(244, 1, 4, 1, 4, 8192)      \
  X(245, 1, 2, 2, 4, 8192)      \
  X(246, 1, 1, 2, 4, 8192)      \
  X(247, 1, 1, 4, 4, 32768)     \
  X(248, 2, 1, 4, 2, 32768)

// NN layout, 16x16x32 MFMAs (variant 4):  X(id, BM, BN, WM, WN)
#define SK_TILE_F16_NN_DMA16_KERNELS(X) \
  X(42, 256, 256, 2, 4)                 \
  X(43, 128, 128, 2, 2)                 \
  X(44, 128, 256, 2, 4)                 \
  X(45, 256, 128, 4, 2)

// bfloat16 instances of the direct-to-LDS tile kernels (16x16x32 MFMAs):  X(id, BM, BN, WM, WN, BK, NN)
#define SK_TILE_BF16_KERNELS(X)    \
  X(60, 256, 256, 2, 4, 64, false) \
  X(61, 128, 128, 2, 2, 64, false) \
  X(62, 128, 128, 2, 2, 32, false) \
  X(63, 64, 64, 2, 2, 32, false)   \
  X(64, 256, 256, 2, 4, 64, true)  \
  X(65, 128, 128, 2, 2, 64, true)  \
  X(50, 128, 256, 2, 4, 64, false) \
  X(51, 256, 128, 4, 2, 64, false) \
  X(52, 64, 128, 2, 2, 32, false)  \
  X(53, 128, 256, 2, 4, 64, true)  \
  X(54, 256, 128, 4, 2, 64, true)

// fp8 (OCP e4m3) operands, fp16 C, NT layout; bk counts fp8 elements (variant 6):  X(id, BM, BN, WM, WN)
#define SK_TILE_F8_KERNELS(X) \
  X(70, 256, 256, 2, 4)       \
  X(71, 128, 128, 2, 2)       \
  X(72, 128, 256, 2, 4)       \
  X(73, 256, 128, 4, 2)       \
  X(75, 64, 128, 1, 4)

// the same for OCP e5m2 operands (dtype SK_F8E5M2):  X(id, BM, BN, WM, WN)
#define SK_TILE_F8E5M2_KERNELS(X) \
  X(90, 256, 256, 2, 4)           \
  X(91, 128, 128, 2, 2)           \
  X(92, 128, 256, 2, 4)           \
  X(93, 256, 128, 4, 2)           \
  X(95, 64, 128, 1, 4)

// int8 operands, int32 C, NT layout; bk counts int8 elements (variant 4: 16x16 accumulator blocks):  X(id, BM, BN, WM, WN)
#define SK_TILE_I8_KERNELS(X) \
  X(80, 256, 256, 2, 4)       \
  X(81, 128, 128, 2, 2)       \
  X(82, 128, 256, 2, 4)       \
  X(83, 256, 128, 4, 2)       \
  X(85, 64, 128, 2, 2)

// the same in four stages of 64 int8 per row (variant 5), for short rows of CTAs:  X(id, BM, BN, WM, WN)
#define SK_TILE_I8_BK64_KERNELS(X) \
  X(86, 128, 128, 2, 2)            \
  X(87, 64, 128, 2, 2)

// fp8 in four stages of 64 K-values (variant 5; e5m2: ids + 20):  X(id, BM, BN, WM, WN)
#define SK_TILE_F8_BK64_KERNELS(X) \
  X(76, 128, 128, 2, 2)            \
  X(77, 64, 128, 1, 4)
#define SK_TILE_F8E5M2_BK64_KERNELS(X) \
  X(96, 128, 128, 2, 2)                \
  X(97, 64, 128, 1, 4)

// 256 x 256 x 64 on four waves, K loop in assembly (variant 7), K a multiple of 64 (int8: 128 bytes per
// iteration):  X(id, MODE, NN)  with MODE 0 fp16, 1 bfloat16, 2 int8, 3 fp8 e4m3, 4 fp8 e5m2; NN: B is [K,N]
#define SK_TILE_ASM_KERNELS(X) \
  X(34, 0, false)              \
  X(66, 1, false)              \
  X(49, 0, true)               \
  X(67, 1, true)
// (the one-byte instances, translation unit kernels_tile_asm8.hip)
#define SK_TILE_ASM8_KERNELS(X) \
  X(84, 2, false)               \
  X(74, 3, false)               \
  X(94, 4, false)

// Q4 weights (dtype SK_Q4) for more rows of A than the weight-streaming kernels take: the two-stage 16x16x32 tile
// kernel with B dequantised into its LDS stage (variant 4):  X(id, BM, BN, WM, WN)
#define SK_TILE_Q4_KERNELS(X) \
  X(46, 128, 128, 2, 2)       \
  X(47, 256, 128, 4, 2)

const KernelInfo *kernel_table(int *count);
const KernelInfo *kernel_by_id(int id);

}  // namespace sk
