// uint4 -> fp16 dequantisation in registers.
//
// Value contract (bit exact): w = fp16_rn((fp16(q) - zero) * scale), q the nibble of element k of
// row n: (Wq[n][k/2] >> 4*(k&1)) & 0xF  (streamk_fp16_ladder_block_reduce_q4.py:552).
//
// Bit trick (replaces the external LOP3 decode the reference calls at :289-290): OR-ing a nibble
// into the mantissa of fp16 1024.0 (0x6400) gives the fp16 number 1024 + q exactly; subtracting
// 1024 + zero is exact as well, so the only rounding is the multiply by the scale.
#pragma once
#include "sk_device.h"

namespace sk {

// One 32-bit word holds nibbles n0..n7 of elements k..k+7.  The four half2 results are
// (n0,n4) (n1,n5) (n2,n6) (n3,n7): element order 0,4,1,5,2,6,3,7.  GEMM kernels feed the other
// operand in the same order, so the weights never need re-packing on the host.
__device__ __forceinline__ half8v dequant_word_q4(uint32_t w, half2v bias, half2v scale) {
  union {
    uint32_t u[4];
    half2v h[4];
    half8v v;
  } r;
  r.u[0] = (w & 0x000F000Fu) | 0x64006400u;
  r.u[1] = ((w >> 4) & 0x000F000Fu) | 0x64006400u;
  r.u[2] = ((w >> 8) & 0x000F000Fu) | 0x64006400u;
  r.u[3] = ((w >> 12) & 0x000F000Fu) | 0x64006400u;
#pragma unroll
  for (int i = 0; i < 4; ++i) r.h[i] = (r.h[i] - bias) * scale;
  return r.v;
}

// position of logical element e (0..7) inside the vector dequant_word_q4 returns
__device__ __forceinline__ constexpr int q4_slot_of_element(int e) { return (e & 3) * 2 + (e >> 2); }

__device__ __forceinline__ half2v q4_bias(int zero) {
  half_t b = (half_t)(float)(1024 + zero);
  return half2v{b, b};
}

}  // namespace sk
