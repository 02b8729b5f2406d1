// Device helpers shared by the fused GEMV kernels: int4 -> fp16 expansion in "pair order".
#pragma once
#include "gq_common.h"

namespace gq {

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

// (w & mask) | magic in one VALU op; mask and magic live in VGPRs (one constant-bus operand is
// all a VOP3 instruction may take on this target).
__device__ __forceinline__ uint32_t and_or(uint32_t w, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "v"(mask), "v"(magic));
  return r;
}

// 8 codes of `w` -> 8 fp16 weights, order (0,4,1,5,2,6,3,7).  The nibble is or-ed into the
// mantissa of 1024.0 (ulp 1) or, for nibbles sitting at bits 7:4, read as 1024 + 16*code; both
// are brought back to the exact code with one packed op, then scaled with a packed fma:
// 13 VALU instructions per 8 weights.
__device__ __forceinline__ half8_t dequant_word(uint32_t w, half2_t s2, half2_t b2) {
  const half2_t kNeg1024 = {(half_t)-1024.0f, (half_t)-1024.0f};
  const half2_t kSixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  const half2_t kNeg64 = {(half_t)-64.0f, (half_t)-64.0f};
  const uint32_t kLo = 0x000F000Fu, kHi = 0x00F000F0u, kMagic = 0x64006400u;
  const uint32_t hi = w >> 8;
  const half2_t c0 = __builtin_elementwise_fma(as_half2(and_or(hi, kHi, kMagic)), kSixteenth, kNeg64);
  const half2_t c1 = as_half2(and_or(hi, kLo, kMagic)) + kNeg1024;
  const half2_t c2 = __builtin_elementwise_fma(as_half2(and_or(w, kHi, kMagic)), kSixteenth, kNeg64);
  const half2_t c3 = as_half2(and_or(w, kLo, kMagic)) + kNeg1024;
  const half2_t w0 = __builtin_elementwise_fma(c0, s2, b2);
  const half2_t w1 = __builtin_elementwise_fma(c1, s2, b2);
  const half2_t w2 = __builtin_elementwise_fma(c2, s2, b2);
  const half2_t w3 = __builtin_elementwise_fma(c3, s2, b2);
  return __builtin_shufflevector(__builtin_shufflevector(w0, w1, 0, 1, 2, 3),
                                 __builtin_shufflevector(w2, w3, 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
}

// 8 codes of a word as fp16 in the order (0,4,1,5,2,6,3,7) of their input features: (64 + c, 64 + c,
// 1024 + c, 1024 + c) twice.  Plain C with the masks in vector registers the compiler cannot see
// through (it then selects v_and_or_b32, and places the wait states a VALU write next to an MFMA needs).
__device__ __forceinline__ half8_t sums_raw_codes(uint32_t w, uint32_t mask_lo, uint32_t mask_hi, uint32_t magic_lo,
                                                  uint32_t magic_hi) {
  const uint32_t hi = w >> 8;
  uint4_t v;
  v.x = (hi & mask_hi) | magic_hi;  // nibbles 3, 7: features 0, 4
  v.y = (hi & mask_lo) | magic_lo;  // nibbles 2, 6: features 1, 5
  v.z = (w & mask_hi) | magic_hi;   // nibbles 1, 5: features 2, 6
  v.w = (w & mask_lo) | magic_lo;   // nibbles 0, 4: features 3, 7
  return __builtin_bit_cast(half8_t, v);
}

// 8 consecutive fp16 of x -> order (0,4,1,5,2,6,3,7)
__device__ __forceinline__ half8_t permute_x(uint4_t q) {
  uint4_t p;
  p.x = __builtin_amdgcn_perm(q.z, q.x, 0x05040100u);
  p.y = __builtin_amdgcn_perm(q.z, q.x, 0x07060302u);
  p.z = __builtin_amdgcn_perm(q.w, q.y, 0x05040100u);
  p.w = __builtin_amdgcn_perm(q.w, q.y, 0x07060302u);
  return __builtin_bit_cast(half8_t, p);
}

}  // namespace gq
