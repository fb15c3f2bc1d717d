// Internal launch interface between the C ABI and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "kernel_table.h"
#include "sk_device.h"
#include "tile_f16.h"
#include "tile_f16_dma.h"
#include "tile_f32.h"
#include "tile_gemv_f16.h"
#include "tile_gemv_q4.h"
#include "tile_gemv_rows.h"
#include "tile_stream_pairs.h"
#include "tile_stream_q4.h"
#include "tile_skinny.h"

namespace sk {

int tile_kernel_infos(KernelInfo *out, int max);
int skinny_kernel_infos(KernelInfo *out, int max);

// return hipError_t as int; occupancy_* return co-resident CTAs per CU (<= 0 on error)
// bias: optional row of N values of C's type added in the epilogue (null: none)
int launch_tile_f16(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
int launch_skinny(int id, const SkinnyArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
// the four-wave kernels whose K loop is assembly live in a translation unit of their own
int tile_asm_kernel_infos(KernelInfo *out, int max);
int launch_tile_asm(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
int occupancy_tile_asm(int id);
int tile_asm8_kernel_infos(KernelInfo *out, int max);
int launch_tile_asm8(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
int occupancy_tile_asm8(int id);
// tile kernels for Q4 weights (translation unit kernels_tile_q4.hip)
int tile_q4_kernel_infos(KernelInfo *out, int max);
int launch_tile_q4(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
int occupancy_tile_q4(int id);
// tile kernels for one-byte operands (translation unit kernels_tile_8bit.hip)
int tile_8bit_kernel_infos(KernelInfo *out, int max);
int launch_tile_8bit(int id, const GemmArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
int occupancy_tile_8bit(int id);
// 2 <= M <= 16 kernels in the matrix-vector kernels' form, and the Q4 kernels for tiled weights with per-group zero
// points (translation unit kernels_gemv_rows.hip)
int gemv_rows_kernel_infos(KernelInfo *out, int max);
int launch_gemv_rows(int id, const SkinnyArgs &a, const DevPlan &p, const Workspace &ws, hipStream_t s, const void *bias);
int occupancy_gemv_rows(int id);
int f32_kernel_infos(KernelInfo *out, int max);
int launch_f32(int id, const GemmArgsF32 &a, const DevPlan &p, const Workspace &ws, hipStream_t s);
int occupancy_f32(int id);
int occupancy_tile(int id);
int occupancy_skinny(int id);

}  // namespace sk
