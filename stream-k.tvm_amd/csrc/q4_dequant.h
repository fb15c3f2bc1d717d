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
//
// 13 VALU operations per word: one shift, four v_and_or_b32, two packed subtracts, two packed
// FMAs, four packed multiplies.  Nibbles sitting at bits 4..7 of a half are OR-ed in place, which
// yields 1024 + 16*q; fma(x, 1/16, -(64 + zero)) = q - zero exactly, saving the shift.
struct Q4Consts {
  uint32_t magic;    // 0x64006400 in a VGPR (v_and_or_b32 takes a single scalar operand)
  uint32_t mask_lo;  // 0x000F000F: nibbles at bits 0..3 of each half
  uint32_t mask_hi;  // 0x00F000F0: nibbles at bits 4..7 of each half
  half2v bias_lo;    // 1024 + zero
  half2v bias_hi;    // -(64 + zero)
  half2v sixteenth;
};
// The three bit patterns are made opaque to the optimiser (empty asm statements that only pin the
// register class), so that (x & mask) | magic is selected as one v_and_or_b32 with the mask in an
// SGPR and the magic in a VGPR instead of being split around literal constants.  The operation
// itself stays ordinary code: the compiler must see it to keep MFMA hazards covered.
__device__ __forceinline__ void q4_pin_patterns(Q4Consts &c) {
  c.magic = 0x64006400u;
  c.mask_lo = 0x000F000Fu;
  c.mask_hi = 0x00F000F0u;
  asm volatile("" : "+v"(c.magic));
  asm volatile("" : "+s"(c.mask_lo));
  asm volatile("" : "+s"(c.mask_hi));
}
__device__ __forceinline__ Q4Consts q4_consts(int zero) {
  Q4Consts c;
  q4_pin_patterns(c);
  const half_t lo = (half_t)(float)(1024 + zero), hi = (half_t)(float)(-(64 + zero));
  c.bias_lo = half2v{lo, lo};
  c.bias_hi = half2v{hi, hi};
  c.sixteenth = half2v{(half_t)0.0625f, (half_t)0.0625f};
  return c;
}
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits) { return (x & mask) | bits; }
__device__ __forceinline__ half8v dequant_word_q4(uint32_t w, const Q4Consts &c, half2v scale) {
  union {
    uint32_t u[4];
    half2v h[4];
    half8v v;
  } r;
  const uint32_t t = w >> 8;
  r.u[0] = and_or(w, c.mask_lo, c.magic);
  r.u[1] = and_or(w, c.mask_hi, c.magic);
  r.u[2] = and_or(t, c.mask_lo, c.magic);
  r.u[3] = and_or(t, c.mask_hi, c.magic);
  r.h[0] = (r.h[0] - c.bias_lo) * scale;
  r.h[1] = __builtin_elementwise_fma(r.h[1], c.sixteenth, c.bias_hi) * scale;
  r.h[2] = (r.h[2] - c.bias_lo) * scale;
  r.h[3] = __builtin_elementwise_fma(r.h[3], c.sixteenth, c.bias_hi) * scale;
  return r.v;
}

// the same with the zero point given per call: bias_lo = 1024 + z, bias_hi = -(64 + z), z an integer in
// 0..15 (both exact in fp16), for weights quantised with one zero point per group
__device__ __forceinline__ half8v dequant_word_q4(uint32_t w, const Q4Consts &c, half2v scale, half2v bias_lo, half2v bias_hi) {
  union {
    uint32_t u[4];
    half2v h[4];
    half8v v;
  } r;
  const uint32_t t = w >> 8;
  r.u[0] = and_or(w, c.mask_lo, c.magic);
  r.u[1] = and_or(w, c.mask_hi, c.magic);
  r.u[2] = and_or(t, c.mask_lo, c.magic);
  r.u[3] = and_or(t, c.mask_hi, c.magic);
  r.h[0] = (r.h[0] - bias_lo) * scale;
  r.h[1] = __builtin_elementwise_fma(r.h[1], c.sixteenth, bias_hi) * scale;
  r.h[2] = (r.h[2] - bias_lo) * scale;
  r.h[3] = __builtin_elementwise_fma(r.h[3], c.sixteenth, bias_hi) * scale;
  return r.v;
}

// position of logical element e (0..7) inside the vector dequant_word_q4 returns
__device__ __forceinline__ constexpr int q4_slot_of_element(int e) { return (e & 3) * 2 + (e >> 2); }

}  // namespace sk
