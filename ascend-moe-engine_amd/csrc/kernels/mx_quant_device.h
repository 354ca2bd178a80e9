// Device pieces of the block-32 MX quantisation (OCP Microscaling Formats v1.0, E4M3 elements with
// an E8M0 shared scale) used by the attention epilogues and by the standalone kernel. Device code
// only: include from .hip files.
//
//   shared_exp = floor(log2(max |v|)) - 8, clamped to [-127, 127];  scale code = shared_exp + 127
//   code_i     = e4m3(v_i * 2^-shared_exp), round to nearest even, saturating at +-448
//   a block of zeros: scale code 0, zero elements; a block with Inf/NaN: scale 0xff, NaN elements
#pragma once

#include <hip/hip_runtime.h>

namespace mlakv {

struct MxScale {
  unsigned code;  // E8M0
  float inverse;  // 2^-shared_exp, a normal fp32 for every bf16 input
  bool nan;
};

// The input is bf16, so the largest magnitude of a block is the largest 15-bit pattern, and its
// floor(log2) is the exponent field (a subnormal or zero maximum clamps to the smallest scale).
__device__ __forceinline__ MxScale MxScaleFromMaxBits(unsigned max_magnitude_bits) {
  const unsigned exponent = max_magnitude_bits >> 7;
  MxScale s;
  s.nan = exponent == 255u;
  s.code = s.nan ? 0xffu : (exponent > 8u ? exponent - 8u : 0u);
  s.inverse = __builtin_bit_cast(float, (254u - (s.nan ? 127u : s.code)) << 23);
  return s;
}

__device__ __forceinline__ unsigned MxMagnitudeMax(unsigned word, unsigned running) {
  const unsigned lo = word & 0x7fffu, hi = (word >> 16) & 0x7fffu;
  return max(running, max(lo, hi));
}

// Two bf16 values (one dword, low half first) -> their two codes in the low 16 bits.
// v_cvt_pk_fp8_f32 rounds to nearest even onto the E4M3 grid for |v| < 464 and returns NaN beyond,
// so the clamp supplies the saturation.
__device__ __forceinline__ unsigned MxEncodeWord(unsigned word, const MxScale& s) {
  if (s.nan) return ((word >> 8) & 0x80u) | ((word >> 16) & 0x8000u) | 0x7f7fu;
  float lo = __builtin_bit_cast(float, word << 16) * s.inverse;
  float hi = __builtin_bit_cast(float, word & 0xffff0000u) * s.inverse;
  lo = fminf(fmaxf(lo, -448.0f), 448.0f);
  hi = fminf(fmaxf(hi, -448.0f), 448.0f);
  return static_cast<unsigned>(__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, 0, false)) & 0xffffu;
}

}  // namespace mlakv
