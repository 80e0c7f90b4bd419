// Arithmetic of the row quantizer shared by the stand-alone quantizer and the kernels that quantize on the fly:
// per-dtype constants of the reference's torch branch (mslk/quantize/triton/fp8_quantize.py:360-378) and the step from
// a row's amax to the multiplier and the scale.
#pragma once
#include "common.h"

namespace mslk_amd {

typedef unsigned short us2 __attribute__((ext_vector_type(2)));

template <int DTYPE> struct Traits;

template <> struct Traits<0> {  // bf16
  using elem_t = uint16_t;
  MSLK_AMD_DEVINL static float to_f32(uint32_t bits) { return bf16_bits_to_f32(bits); }
  MSLK_AMD_DEVINL static float abs_bits_to_f32(uint32_t b) { return bf16_bits_to_f32(b); }
  MSLK_AMD_DEVINL static float eps() { return __uint_as_float(0x2B8D0000u); }  // bf16(1e-12)
  MSLK_AMD_DEVINL static float round_ub(float ub) { return bf16_bits_to_f32(f32_to_bf16_bits(ub)); }
};
template <> struct Traits<1> {  // fp16
  using elem_t = uint16_t;
  MSLK_AMD_DEVINL static float to_f32(uint32_t bits) {
    unsigned short s = (unsigned short)bits;
    return (float)__builtin_bit_cast(_Float16, s);
  }
  MSLK_AMD_DEVINL static float abs_bits_to_f32(uint32_t b) { return to_f32(b); }
  MSLK_AMD_DEVINL static float eps() { return 0.0f; }  // fp16(1e-12) == 0
  MSLK_AMD_DEVINL static float round_ub(float ub) { return (float)(_Float16)ub; }
};
template <> struct Traits<2> {  // fp32
  using elem_t = float;
  MSLK_AMD_DEVINL static float abs_bits_to_f32(uint32_t b) { return __uint_as_float(b); }
  MSLK_AMD_DEVINL static float eps() { return 1e-12f; }
  MSLK_AMD_DEVINL static float round_ub(float ub) { return ub; }
};

// amax (as fp32, NaN if the row holds a NaN) -> (inv, scale) of the reference formula.
template <int DTYPE, bool TRITON>
MSLK_AMD_DEVINL void scales_from_amax(float amax, const float* scale_ub, float triton_eps, float& inv, float& scale) {
  if constexpr (TRITON) {
    // tl.maximum / tl.clamp against fp32 constants, then div_rn(cur_max, MAX_FP8); `inv` carries the divisor
    float c = (amax < triton_eps) ? triton_eps : amax;
    if (scale_ub != nullptr) c = (c > *scale_ub) ? *scale_ub : c;
    scale = c / 448.0f;
    inv = scale;
    return;
  }
  const float eps = Traits<DTYPE>::eps();
  float c = (amax < eps) ? eps : amax;  // comparisons are false for NaN: NaN propagates
  if (scale_ub != nullptr) {
    const float ub = Traits<DTYPE>::round_ub(*scale_ub);
    c = (c > ub) ? ub : c;
  }
  const float recip = 1.0f / c;  // IEEE-correct division (no fast-math in this build)
  inv = recip * 448.0f;
  if (inv == __builtin_inff()) inv = 1.0f;
  scale = 1.0f / inv;
}

}  // namespace mslk_amd
