// Shared device/host helpers for the gfx950 FP8 rowwise kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mslk_amd {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round to nearest even (finite inputs; NaN stays NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}

// Two fp32 -> packed e4m3fn codes in the low 16 bits (lo = a, hi = b).
// The hardware conversion rounds to nearest even; what it does above the largest finite
// value depends on a mode bit, so magnitudes beyond 464 (the first value that does not round to
// 448) are forced to the NaN code 0x7F here, which is what a non-saturating cast produces.
__device__ __forceinline__ uint32_t cvt_pk_e4m3fn(float a, float b) {
  uint32_t r = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xFFFFu;
  uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
  if ((ua & 0x7FFFFFFFu) > 0x43E80000u) r = (r & 0xFF00u) | ((ua >> 24) & 0x80u) | 0x7Fu;
  if ((ub & 0x7FFFFFFFu) > 0x43E80000u) r = (r & 0x00FFu) | ((((ub >> 24) & 0x80u) | 0x7Fu) << 8);
  return r;
}

#define MSLK_AMD_DEVINL __device__ __forceinline__

// 8-byte store of quantized codes, written through to memory at system scope (sc1) instead of being left dirty in the
// L2 of the XCD that produced them or streamed past the caches (nt).  A write-through leaves nothing to flush when the
// kernel ends (plain stores cost the row quantizer 1.6 us at 4096 x 4096) and, unlike a streaming store, leaves the
// codes in the memory-side cache, where the GEMM that consumes them finds them: quantize -> GEMM at 4096^3 takes
// 60.6 us with nt stores, 58.9 with plain ones and 57.7 with these; the quantizer alone 12.4 / 14.0 / 12.5 us.
// Written as an instruction because the compiler offers no spelling for the scope bits of a plain store; an 8-byte store
// needs no wait states behind it, and the "memory" clobber keeps it ordered with the surrounding accesses.
__device__ __forceinline__ void store8_write_through(void* dst, v2i v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc1" : : "v"(dst), "v"(v) : "memory");
}

// Two fp32 -> packed bf16 (lo = a, hi = b), round to nearest even, by the hardware conversion.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// fp32 -> fp16, round to nearest even, overflow to infinity (v_cvt_f16_f32 in the default rounding mode).
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f);
}
__device__ __forceinline__ uint32_t pack_f16x2(float a, float b) { return f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16); }

// 16-bit output element of the GEMMs: bf16 (F16 = false) or fp16 (F16 = true).
template <bool F16>
__device__ __forceinline__ uint32_t pack_out_x2(float a, float b) {
  if constexpr (F16) return pack_f16x2(a, b);
  else return pack_bf16x2(a, b);
}
__device__ __forceinline__ uint32_t f32_to_out_bits(float v, int out_f16) {
  return out_f16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
}

}  // namespace mslk_amd
