// Row-wise FP8 (e4m3fn) quantizer for gfx950.
//
// Bit-exact to the torch branch of the reference's quantize_fp8_row
// (mslk/quantize/triton/fp8_quantize.py:360-378):
//   amax  = max|x| over the row, taken in the input dtype (exact for bf16/fp16/fp32)
//   amax  = clamp(amax, min = dtype(1e-12) [, max = dtype(*scale_ub)]), NaN propagates
//   inv   = fl32(fl32(1 / amax) * 448);  inv == +inf -> 1
//   code  = e4m3fn_rne(fl32(fl32(x) * inv))            (no saturation: > 464 becomes NaN)
//   scale = fl32(1 / inv)
//
// The pass is HBM-bound (2 B in + 1 B out per element for bf16), so the kernel is organised
// around 128-bit coalesced loads that stay in registers between the amax pass and the convert
// pass: a row is owned by a "team" of 64 lanes (one wavefront) or 256 lanes (one workgroup);
// each lane keeps up to NV vectors of 8 elements.  Rows longer than TEAM*8*NV are streamed twice
// (the second read hits L2 / Infinity Cache).
#include "common.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

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

// 8 consecutive elements of a row.
template <int DTYPE> struct Vec8 { uint4 w; };          // 8 x 16-bit
template <> struct Vec8<2> { uint4 lo, hi; };           // 8 x fp32

MSLK_AMD_DEVINL void store8_stream(uint2* dst, uint2 val) {
  __builtin_nontemporal_store(v2i{(int)val.x, (int)val.y}, reinterpret_cast<v2i*>(dst));
}

template <int DTYPE>
MSLK_AMD_DEVINL Vec8<DTYPE> load_vec8(const void* row_ptr, int vec_idx) {
  Vec8<DTYPE> v;
  // the input is read once (rows cached in registers) or twice in quick succession: stream it
  if constexpr (DTYPE == 2) {
    const v4i* p = reinterpret_cast<const v4i*>(row_ptr) + 2 * (int64_t)vec_idx;
    const v4i a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
    v.lo = make_uint4(a.x, a.y, a.z, a.w);
    v.hi = make_uint4(b.x, b.y, b.z, b.w);
  } else {
    const v4i a = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(row_ptr) + vec_idx);
    v.w = make_uint4(a.x, a.y, a.z, a.w);
  }
  return v;
}

// Running maximum of |x| kept as raw bits: for non-negative IEEE values unsigned integer order
// equals numeric order and every NaN pattern sorts above +inf, so a NaN in the row survives.
template <int DTYPE>
MSLK_AMD_DEVINL uint32_t absmax_bits(uint32_t m, const Vec8<DTYPE>& v) {
  if constexpr (DTYPE == 2) {
    const uint32_t w[8] = {v.lo.x, v.lo.y, v.lo.z, v.lo.w, v.hi.x, v.hi.y, v.hi.z, v.hi.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) m = max(m, w[i] & 0x7FFFFFFFu);
    return m;
  } else {
    const uint32_t w[4] = {v.w.x, v.w.y, v.w.z, v.w.w};
    us2 acc = __builtin_bit_cast(us2, m);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc = __builtin_elementwise_max(acc, __builtin_bit_cast(us2, w[i] & 0x7FFF7FFFu));
    return __builtin_bit_cast(uint32_t, acc);
  }
}

template <int DTYPE>
MSLK_AMD_DEVINL uint32_t finish_absmax_bits(uint32_t m) {
  if constexpr (DTYPE == 2) return m;
  return max(m & 0xFFFFu, m >> 16);
}

template <int DTYPE>
MSLK_AMD_DEVINL uint2 quantize_vec8(const Vec8<DTYPE>& v, float inv) {
  float f[8];
  if constexpr (DTYPE == 2) {
    const uint32_t w[8] = {v.lo.x, v.lo.y, v.lo.z, v.lo.w, v.hi.x, v.hi.y, v.hi.z, v.hi.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = __uint_as_float(w[i]);
  } else {
    const uint32_t w[4] = {v.w.x, v.w.y, v.w.z, v.w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = Traits<DTYPE>::to_f32(w[i] & 0xFFFFu);
      f[2 * i + 1] = Traits<DTYPE>::to_f32(w[i] >> 16);
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = f[i] * inv;
  uint2 r;
  r.x = cvt_pk_e4m3fn(f[0], f[1]) | (cvt_pk_e4m3fn(f[2], f[3]) << 16);
  r.y = cvt_pk_e4m3fn(f[4], f[5]) | (cvt_pk_e4m3fn(f[6], f[7]) << 16);
  return r;
}

// amax (as fp32, NaN if the row holds a NaN) -> (inv, scale) of the reference formula.
template <int DTYPE>
MSLK_AMD_DEVINL void scales_from_amax(float amax, const float* scale_ub, float& inv, float& scale) {
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

template <int TEAM>
MSLK_AMD_DEVINL uint32_t team_max(uint32_t m, uint32_t* smem, int team_in_block) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
  if constexpr (TEAM > kWave) {
    constexpr int WAVES = TEAM / kWave;
    const int wave = (threadIdx.x % TEAM) / kWave;
    uint32_t* s = smem + team_in_block * WAVES;
    if ((threadIdx.x & 63) == 0) s[wave] = m;
    __syncthreads();
    m = s[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) m = max(m, s[w]);
  }
  return m;
}

// Vector path: K % 8 == 0, row starts 16-byte aligned, output rows 8-byte aligned.
template <int DTYPE, int TEAM, int NV, bool CACHED>
__global__ __launch_bounds__(256) void quantize_rows_vec_kernel(
    const void* __restrict__ x, int64_t rows, int K, int64_t in_stride, uint8_t* __restrict__ out,
    int64_t out_stride, float* __restrict__ scale, const float* __restrict__ scale_ub) {
  constexpr int TEAMS = 256 / TEAM;
  constexpr int ELEM_BYTES = (DTYPE == 2) ? 4 : 2;
  __shared__ uint32_t smem[4];
  const int team_in_block = threadIdx.x / TEAM;
  const int lane = threadIdx.x % TEAM;
  const int64_t row = (int64_t)blockIdx.x * TEAMS + team_in_block;
  const bool valid = row < rows;
  const int nvec = K >> 3;
  const char* row_ptr = reinterpret_cast<const char*>(x) + (valid ? row : 0) * in_stride * ELEM_BYTES;

  Vec8<DTYPE> cache[NV];
  uint32_t m = 0;
  if constexpr (CACHED) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = i * TEAM + lane;
      if (valid && idx < nvec) {
        cache[i] = load_vec8<DTYPE>(row_ptr, idx);
        m = absmax_bits<DTYPE>(m, cache[i]);
      }
    }
  } else {
    if (valid)
      for (int idx = lane; idx < nvec; idx += TEAM) m = absmax_bits<DTYPE>(m, load_vec8<DTYPE>(row_ptr, idx));
  }
  m = team_max<TEAM>(finish_absmax_bits<DTYPE>(m), smem, team_in_block);
  if (!valid) return;

  float inv, sc;
  scales_from_amax<DTYPE>(Traits<DTYPE>::abs_bits_to_f32(m), scale_ub, inv, sc);
  if (lane == 0) scale[row] = sc;

  uint2* out_row = reinterpret_cast<uint2*>(out + row * out_stride);
  if constexpr (CACHED) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = i * TEAM + lane;
      if (idx < nvec) store8_stream(out_row + idx, quantize_vec8<DTYPE>(cache[i], inv));
    }
  } else {
    for (int idx = lane; idx < nvec; idx += TEAM)
      store8_stream(out_row + idx, quantize_vec8<DTYPE>(load_vec8<DTYPE>(row_ptr, idx), inv));
  }
  // zero padding columns [K, out_stride)
  for (int64_t k = K + lane; k < out_stride; k += TEAM) out[row * out_stride + k] = 0;
}

// Generic path: any K, any alignment; one workgroup per row, scalar accesses, two passes.
template <int DTYPE>
__global__ __launch_bounds__(256) void quantize_rows_generic_kernel(
    const void* __restrict__ x, int64_t rows, int64_t K, int64_t in_stride, uint8_t* __restrict__ out,
    int64_t out_stride, float* __restrict__ scale, const float* __restrict__ scale_ub) {
  using elem_t = typename Traits<DTYPE>::elem_t;
  __shared__ uint32_t smem[4];
  const int64_t row = blockIdx.x;
  const elem_t* xr = reinterpret_cast<const elem_t*>(x) + row * in_stride;
  uint32_t m = 0;
  for (int64_t k = threadIdx.x; k < K; k += 256) {
    if constexpr (DTYPE == 2) m = max(m, __float_as_uint(xr[k]) & 0x7FFFFFFFu);
    else m = max(m, (uint32_t)xr[k] & 0x7FFFu);
  }
  m = team_max<256>(m, smem, 0);
  float inv, sc;
  scales_from_amax<DTYPE>(Traits<DTYPE>::abs_bits_to_f32(m), scale_ub, inv, sc);
  if (threadIdx.x == 0) scale[row] = sc;
  for (int64_t k = threadIdx.x; k < out_stride; k += 256) {
    uint8_t code = 0;
    if (k < K) {
      float f;
      if constexpr (DTYPE == 2) f = xr[k];
      else f = Traits<DTYPE>::to_f32(xr[k]);
      code = (uint8_t)(cvt_pk_e4m3fn(f * inv, 0.0f) & 0xFFu);
    }
    out[row * out_stride + k] = code;
  }
}

__global__ void cast_e4m3fn_kernel(const float* __restrict__ in, int64_t n, uint8_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = (uint8_t)(cvt_pk_e4m3fn(in[i], 0.0f) & 0xFFu);
}

template <int DTYPE>
hipError_t launch_quantize_t(const void* x, int64_t rows, int64_t K, int64_t in_stride, uint8_t* out,
                             int64_t out_stride, float* scale, const float* scale_ub, hipStream_t s) {
  constexpr int ELEM_BYTES = (DTYPE == 2) ? 4 : 2;
  constexpr int NV = 16;
  const bool vec_ok = (K % 8 == 0) && (K < (int64_t(1) << 31)) && ((in_stride * ELEM_BYTES) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (out_stride % 8 == 0) &&
                      (reinterpret_cast<uintptr_t>(out) % 8 == 0);
  if (!vec_ok) {
    quantize_rows_generic_kernel<DTYPE><<<dim3((unsigned)rows), dim3(256), 0, s>>>(
        x, rows, K, in_stride, out, out_stride, scale, scale_ub);
    return hipGetLastError();
  }
  const int k = (int)K;
  // One wavefront per row once there are enough rows to fill the chip; otherwise a workgroup per row.
  if (K <= kWave * 8 * NV && rows >= 2048) {
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    if (K <= kWave * 8 * 4)
      quantize_rows_vec_kernel<DTYPE, 64, 4, true><<<blocks, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub);
    else if (K <= kWave * 8 * 8)
      quantize_rows_vec_kernel<DTYPE, 64, 8, true><<<blocks, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub);
    else
      quantize_rows_vec_kernel<DTYPE, 64, NV, true><<<blocks, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub);
  } else if (K <= 256 * 8 * 4) {
    quantize_rows_vec_kernel<DTYPE, 256, 4, true><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub);
  } else if (K <= 256 * 8 * NV) {
    quantize_rows_vec_kernel<DTYPE, 256, NV, true><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub);
  } else {
    quantize_rows_vec_kernel<DTYPE, 256, 1, false><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_quantize_fp8_row(const void* x, int dtype, int64_t rows, int64_t K, int64_t in_stride,
                                   void* xq, int64_t K_out, float* scale, const float* scale_ub,
                                   hipStream_t s) {
  uint8_t* out = reinterpret_cast<uint8_t*>(xq);
  switch (dtype) {
    case 0: return launch_quantize_t<0>(x, rows, K, in_stride, out, K_out, scale, scale_ub, s);
    case 1: return launch_quantize_t<1>(x, rows, K, in_stride, out, K_out, scale, scale_ub, s);
    default: return launch_quantize_t<2>(x, rows, K, in_stride, out, K_out, scale, scale_ub, s);
  }
}

hipError_t launch_cast_e4m3fn(const float* in, int64_t n, void* out, hipStream_t s) {
  const int64_t want = (n + 255) / 256;
  const unsigned blocks = (unsigned)(want < 1 ? 1 : (want > 65536 ? 65536 : want));
  cast_e4m3fn_kernel<<<blocks, 256, 0, s>>>(in, n, reinterpret_cast<uint8_t*>(out));
  return hipGetLastError();
}

}  // namespace mslk_amd
