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
// TRITON = true selects the arithmetic of the reference's GPU (Triton) kernel instead
// (mslk/quantize/triton/fp8_quantize.py:131-207): amax clamped at `eps` (default 1/512) [and *scale_ub],
//   scale = fl32(amax / 448);  code = e4m3fn_rne(clamp(fl32(fl32(x) / scale), -448, 448))
// with IEEE-correct divisions (div_rn) and saturation.
//
// The pass is HBM-bound (2 B in + 1 B out per element for bf16), so the kernel is organised
// around 128-bit coalesced loads that stay in registers between the amax pass and the convert
// pass: a row is owned by a "team" of 64 lanes (one wavefront) or 256 lanes (one workgroup);
// each lane keeps up to NV vectors of 8 elements.  Rows longer than TEAM*8*NV are streamed twice
// (the second read hits L2 / Infinity Cache).
#include "common.h"
#include "kernels.h"
#include "quant_math.h"

namespace mslk_amd {
namespace {

// 8 consecutive elements of a row.
template <int DTYPE> struct Vec8 { uint4 w; };          // 8 x 16-bit
template <> struct Vec8<2> { uint4 lo, hi; };           // 8 x fp32

MSLK_AMD_DEVINL void store8_stream(uint2* dst, uint2 val) { store8_write_through(dst, v2i{(int)val.x, (int)val.y}); }

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

// `factor` is the multiplier `inv` of the torch-branch formula, or the divisor `scale` of the Triton one.
// TRITON with rcp != 0: x / factor is formed as q0 = x * rcp, e = fma(-q0, factor, x), q = e == 0 ? q0 : fma(e, rcp, q0)
// with rcp = fl32(1 / factor) -- a handful of instructions instead of a division sequence.  The e4m3 codes are those of the
// IEEE division for every 16-bit element not above a 16-bit row maximum of at least 2^-64 (checked exhaustively on the
// CPU, tests/test_oracle.py); the caller passes rcp = 0 for every other row, which then divides.
// clamp(v, -448, 448) in one instruction (the median of the three; a NaN comes out as -448, like fmin(fmax(v, -448), 448))
MSLK_AMD_DEVINL float clamp448(float v) { return __builtin_amdgcn_fmed3f(v, -448.0f, 448.0f); }

// PLAIN (torch arithmetic only): the caller knows that no product of the row exceeds 448 (1 + 2^-22) and none is NaN -- a
// finite row maximum that scale_ub has not cut -- so the hardware conversion alone gives the codes.
template <int DTYPE, bool TRITON, bool PLAIN = false>
MSLK_AMD_DEVINL uint2 quantize_vec8(const Vec8<DTYPE>& v, float factor, float rcp = 0.f) {
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
  if constexpr (TRITON) {
    if (rcp != 0.f) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float q0 = f[i] * rcp;
        const float e = __builtin_fmaf(-q0, factor, f[i]);
        const float q = e == 0.f ? q0 : __builtin_fmaf(e, rcp, q0);
        f[i] = clamp448(q);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = clamp448(f[i] / factor);
    }
    // Everything is within +-448 now (a NaN quotient came out of the clamp as -448, as it did with a max / min pair), so
    // the plain hardware conversion gives the codes; the fix-up for magnitudes beyond 464 has nothing left to do.
    uint2 r;
    r.x = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false), true);
    r.y = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false), true);
    return r;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = f[i] * factor;
    if constexpr (PLAIN) {
      uint2 r;
      r.x = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false), true);
      r.y = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false), true);
      return r;
    }
  }
  uint2 r;
  r.x = cvt_pk_e4m3fn(f[0], f[1]) | (cvt_pk_e4m3fn(f[2], f[3]) << 16);
  r.y = cvt_pk_e4m3fn(f[4], f[5]) | (cvt_pk_e4m3fn(f[6], f[7]) << 16);
  return r;
}

// Jagged rows (reference: JAGGED branch of _kernel_quantize_fp8_row, fp8_quantize.py:123-129): rows are
// grouped in blocks of `rows_per_group`; inside block b only the first zero_start[b] rows hold data,
// the others are treated as all-zero rows and are never read.
struct JaggedRows {
  const void* zero_start;   // nullptr: every row is live
  int64_t rows_per_group;
  int index_is_i32;
  float triton_eps;         // lower bound of amax in the TRITON arithmetic
};

MSLK_AMD_DEVINL bool row_is_live(const JaggedRows& j, int64_t row) {
  if (j.zero_start == nullptr) return true;
  const int64_t b = row / j.rows_per_group, n = row - b * j.rows_per_group;
  const int64_t live = j.index_is_i32 ? (int64_t) static_cast<const int32_t*>(j.zero_start)[b]
                                      : static_cast<const int64_t*>(j.zero_start)[b];
  return n < live;
}

template <int TEAM>
MSLK_AMD_DEVINL uint32_t team_max(uint32_t m, uint32_t* smem, int team_in_block) {
  constexpr int SPAN = TEAM < kWave ? TEAM : kWave;   // teams narrower than a wavefront are aligned lane groups of it
#pragma unroll
  for (int off = SPAN / 2; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
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

// Reciprocal of the Triton-arithmetic divisor for rows that may use the multiply form of quantize_vec8, else 0: the row
// maximum is a finite 16-bit value of at least 2^-64 that neither the lower bound nor scale_ub replaced.
template <int DTYPE, bool TRITON>
MSLK_AMD_DEVINL float triton_fast_rcp(float amax, const float* scale_ub, float triton_eps, float divisor) {
  if constexpr (!TRITON || DTYPE == 2) return 0.f;
  const bool ok = scale_ub == nullptr && amax >= triton_eps && amax >= 0x1p-64f && amax < __builtin_inff();
  return ok ? 1.0f / divisor : 0.f;
}

// Vector path: K % 8 == 0, row starts 16-byte aligned, output rows 8-byte aligned.
template <int DTYPE, int TEAM, int NV, bool CACHED, bool TRITON>
__global__ __launch_bounds__(256) void quantize_rows_vec_kernel(
    const void* __restrict__ x, int64_t rows, int K, int64_t in_stride, uint8_t* __restrict__ out,
    int64_t out_stride, float* __restrict__ scale, const float* __restrict__ scale_ub, JaggedRows jag) {
  constexpr int TEAMS = 256 / TEAM;
  constexpr int ELEM_BYTES = (DTYPE == 2) ? 4 : 2;
  __shared__ uint32_t smem[4];
  const int team_in_block = threadIdx.x / TEAM;
  const int lane = threadIdx.x % TEAM;
  const int64_t row = (int64_t)blockIdx.x * TEAMS + team_in_block;
  const bool valid = row < rows;
  const bool live = valid && row_is_live(jag, row);   // uniform over the team
  const int nvec = K >> 3;
  const char* row_ptr = reinterpret_cast<const char*>(x) + (valid ? row : 0) * in_stride * ELEM_BYTES;

  Vec8<DTYPE> cache[NV];
  uint32_t m = 0;
  if constexpr (CACHED) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = i * TEAM + lane;
      if (live && idx < nvec) {
        cache[i] = load_vec8<DTYPE>(row_ptr, idx);
        m = absmax_bits<DTYPE>(m, cache[i]);
      }
    }
  } else {
    if (live)
      for (int idx = lane; idx < nvec; idx += TEAM) m = absmax_bits<DTYPE>(m, load_vec8<DTYPE>(row_ptr, idx));
  }
  m = team_max<TEAM>(finish_absmax_bits<DTYPE>(m), smem, team_in_block);
  if (!valid) return;

  float inv, sc;
  const float amax = Traits<DTYPE>::abs_bits_to_f32(m);
  scales_from_amax<DTYPE, TRITON>(amax, scale_ub, jag.triton_eps, inv, sc);
  if (lane == 0) scale[row] = sc;
  const float rcp = triton_fast_rcp<DTYPE, TRITON>(amax, scale_ub, jag.triton_eps, inv);

  uint2* out_row = reinterpret_cast<uint2*>(out + row * out_stride);
  if (!live) {   // an empty row quantizes to zero codes
    for (int idx = lane; idx < nvec; idx += TEAM) store8_stream(out_row + idx, make_uint2(0u, 0u));
  } else if constexpr (CACHED) {
    // torch arithmetic: a row with a finite maximum that scale_ub did not cut needs no NaN / overflow fix-up behind the
    // hardware conversion (uniform over the team)
    if (!TRITON && scale_ub == nullptr && amax < __builtin_inff()) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int idx = i * TEAM + lane;
        if (idx < nvec) store8_stream(out_row + idx, quantize_vec8<DTYPE, TRITON, !TRITON>(cache[i], inv, rcp));
      }
    } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int idx = i * TEAM + lane;
        if (idx < nvec) store8_stream(out_row + idx, quantize_vec8<DTYPE, TRITON>(cache[i], inv, rcp));
      }
    }
  } else {
    for (int idx = lane; idx < nvec; idx += TEAM)
      store8_stream(out_row + idx, quantize_vec8<DTYPE, TRITON>(load_vec8<DTYPE>(row_ptr, idx), inv, rcp));
  }
  // zero padding columns [K, out_stride)
  for (int64_t k = K + lane; k < out_stride; k += TEAM) out[row * out_stride + k] = 0;
}

// Generic path: any K, any alignment; one workgroup per row, two passes.  Full groups of eight elements move as 16- / 32-byte
// copies without an alignment promise (the compiler picks the access width the target allows), the K % 8 tail and the
// padding columns element by element.
template <int DTYPE, bool TRITON>
__global__ __launch_bounds__(256) void quantize_rows_generic_kernel(
    const void* __restrict__ x, int64_t rows, int64_t K, int64_t in_stride, uint8_t* __restrict__ out,
    int64_t out_stride, float* __restrict__ scale, const float* __restrict__ scale_ub, JaggedRows jag) {
  using elem_t = typename Traits<DTYPE>::elem_t;
  __shared__ uint32_t smem[4];
  const int64_t row = blockIdx.x;
  const elem_t* xr = reinterpret_cast<const elem_t*>(x) + row * in_stride;
  if (!row_is_live(jag, row)) K = 0;   // nothing of the row is read; all codes become zero
  const int64_t nvec = K >> 3;
  const char* xb = reinterpret_cast<const char*>(xr);
  uint32_t m = 0;
  for (int64_t idx = threadIdx.x; idx < nvec; idx += 256) {
    Vec8<DTYPE> v;
    __builtin_memcpy(&v, xb + idx * sizeof(Vec8<DTYPE>), sizeof(Vec8<DTYPE>));
    m = absmax_bits<DTYPE>(m, v);
  }
  m = finish_absmax_bits<DTYPE>(m);
  for (int64_t k = nvec * 8 + threadIdx.x; k < K; k += 256) {
    if constexpr (DTYPE == 2) m = max(m, __float_as_uint(xr[k]) & 0x7FFFFFFFu);
    else m = max(m, (uint32_t)xr[k] & 0x7FFFu);
  }
  m = team_max<256>(m, smem, 0);
  float inv, sc;
  scales_from_amax<DTYPE, TRITON>(Traits<DTYPE>::abs_bits_to_f32(m), scale_ub, jag.triton_eps, inv, sc);
  if (threadIdx.x == 0) scale[row] = sc;
  uint8_t* out_row = out + row * out_stride;
  for (int64_t idx = threadIdx.x; idx < nvec; idx += 256) {
    Vec8<DTYPE> v;
    __builtin_memcpy(&v, xb + idx * sizeof(Vec8<DTYPE>), sizeof(Vec8<DTYPE>));
    const uint2 q = quantize_vec8<DTYPE, TRITON>(v, inv);
    __builtin_memcpy(out_row + idx * 8, &q, 8);
  }
  for (int64_t k = nvec * 8 + threadIdx.x; k < out_stride; k += 256) {
    uint8_t code = 0;
    if (k < K) {
      float f;
      if constexpr (DTYPE == 2) f = xr[k];
      else f = Traits<DTYPE>::to_f32(xr[k]);
      if constexpr (TRITON) f = __builtin_fminf(__builtin_fmaxf(f / inv, -448.0f), 448.0f);
      else f = f * inv;
      code = (uint8_t)(cvt_pk_e4m3fn(f, 0.0f) & 0xFFu);
    }
    out_row[k] = code;
  }
}

// Row-wise dequantization (reference: _kernel_dequantize_fp8_row, fp8_quantize.py:1060-1113):
// out = bf16_rne(fl32(fp8 -> f32) * scale[row]).  1 byte in, 2 bytes out per element: HBM-bound.
// A lane converts 16 consecutive codes of one row (K % 16 == 0) per iteration.
__global__ __launch_bounds__(256) void dequantize_rows_vec_kernel(const uint8_t* __restrict__ xq,
                                                                  const float* __restrict__ scale, int64_t chunks,
                                                                  int chunks_per_row, uint16_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    const v4i q = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(xq) + c);
    const float sc = scale[c / chunks_per_row];
    const int w[4] = {q.x, q.y, q.z, q.w};
    uint32_t o[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[i], false);
      const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[i], true);
      o[2 * i] = pack_bf16x2(lo[0] * sc, lo[1] * sc);
      o[2 * i + 1] = pack_bf16x2(hi[0] * sc, hi[1] * sc);
    }
    v4i* dst = reinterpret_cast<v4i*>(out) + 2 * c;
    __builtin_nontemporal_store(v4i{(int)o[0], (int)o[1], (int)o[2], (int)o[3]}, dst);
    __builtin_nontemporal_store(v4i{(int)o[4], (int)o[5], (int)o[6], (int)o[7]}, dst + 1);
  }
}

// As above for K % 8 == 0 (rows of codes 8-byte aligned, rows of the output 16-byte aligned): 8 codes per lane.
__global__ __launch_bounds__(256) void dequantize_rows_vec8_kernel(const uint8_t* __restrict__ xq,
                                                                   const float* __restrict__ scale, int64_t chunks,
                                                                   int chunks_per_row, uint16_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    const v2i q = __builtin_nontemporal_load(reinterpret_cast<const v2i*>(xq) + c);
    const float sc = scale[c / chunks_per_row];
    const int w[2] = {q.x, q.y};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[i], false);
      const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[i], true);
      o[2 * i] = pack_bf16x2(lo[0] * sc, lo[1] * sc);
      o[2 * i + 1] = pack_bf16x2(hi[0] * sc, hi[1] * sc);
    }
    __builtin_nontemporal_store(v4i{(int)o[0], (int)o[1], (int)o[2], (int)o[3]}, reinterpret_cast<v4i*>(out) + c);
  }
}

// Any K, any alignment: a lane takes 8 consecutive codes of the flat tensor; when they lie in one row they move as an
// 8-byte and a 16-byte copy without an alignment promise, otherwise (row boundary, end of the tensor) one by one.
__global__ __launch_bounds__(256) void dequantize_rows_generic_kernel(const uint8_t* __restrict__ xq,
                                                                      const float* __restrict__ scale, int64_t total,
                                                                      int64_t K, uint16_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t chunks = (total + 7) / 8;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    const int64_t i0 = c * 8;
    const int n = total - i0 < 8 ? (int)(total - i0) : 8;
    const int64_t r0 = i0 / K;
    if (n == 8 && (i0 + 7) / K == r0) {
      uint32_t w[2];
      __builtin_memcpy(w, xq + i0, 8);
      const float sc = scale[r0];
      uint32_t o[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
        const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
        o[2 * i] = pack_bf16x2(lo[0] * sc, lo[1] * sc);
        o[2 * i + 1] = pack_bf16x2(hi[0] * sc, hi[1] * sc);
      }
      __builtin_memcpy(out + i0, o, 16);
    } else {
      for (int e = 0; e < n; ++e)
        out[i0 + e] = (uint16_t)f32_to_bf16_bits(__builtin_amdgcn_cvt_f32_fp8((int)xq[i0 + e], 0) * scale[(i0 + e) / K]);
    }
  }
}

__global__ void cast_e4m3fn_kernel(const float* __restrict__ in, int64_t n, uint8_t* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = (uint8_t)(cvt_pk_e4m3fn(in[i], 0.0f) & 0xFFu);
}

template <int DTYPE, bool TRITON>
hipError_t launch_quantize_t(const void* x, int64_t rows, int64_t K, int64_t in_stride, uint8_t* out,
                             int64_t out_stride, float* scale, const float* scale_ub, JaggedRows jag,
                             hipStream_t s) {
  constexpr int ELEM_BYTES = (DTYPE == 2) ? 4 : 2;
  constexpr int NV = 16;
  const bool vec_ok = (K % 8 == 0) && (K < (int64_t(1) << 31)) && ((in_stride * ELEM_BYTES) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (out_stride % 8 == 0) &&
                      (reinterpret_cast<uintptr_t>(out) % 8 == 0);
  if (!vec_ok) {
    quantize_rows_generic_kernel<DTYPE, TRITON><<<dim3((unsigned)rows), dim3(256), 0, s>>>(
        x, rows, K, in_stride, out, out_stride, scale, scale_ub, jag);
    return hipGetLastError();
  }
  const int k = (int)K;
  // Short rows (per-head quantization: K = 64 ... 256) in large numbers: 8 / 16 / 32 lanes per row, one 16-byte load each,
  // so that a wavefront covers 8 / 4 / 2 rows instead of idling three quarters of its lanes (131072 x 128 bf16: 37 -> 12 us).
  if (K <= 256 && rows >= 4096) {
    if (K <= 64)
      quantize_rows_vec_kernel<DTYPE, 8, 1, true, TRITON><<<(unsigned)((rows + 31) / 32), 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
    else if (K <= 128)
      quantize_rows_vec_kernel<DTYPE, 16, 1, true, TRITON><<<(unsigned)((rows + 15) / 16), 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
    else
      quantize_rows_vec_kernel<DTYPE, 32, 1, true, TRITON><<<(unsigned)((rows + 7) / 8), 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
    return hipGetLastError();
  }
  // One wavefront per row once there are enough rows to fill the chip; otherwise a workgroup per row.
  if (K <= kWave * 8 * NV && rows >= 2048) {
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    if (K <= kWave * 8 * 4)
      quantize_rows_vec_kernel<DTYPE, 64, 4, true, TRITON><<<blocks, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
    else if (K <= kWave * 8 * 8)
      quantize_rows_vec_kernel<DTYPE, 64, 8, true, TRITON><<<blocks, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
    else
      quantize_rows_vec_kernel<DTYPE, 64, NV, true, TRITON><<<blocks, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
  } else if (K <= 256 * 8 * 4) {
    quantize_rows_vec_kernel<DTYPE, 256, 4, true, TRITON><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
  } else if (K <= 256 * 8 * NV) {
    quantize_rows_vec_kernel<DTYPE, 256, NV, true, TRITON><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
  } else if (DTYPE != 2 && K <= 256 * 8 * 32) {
    // 16-bit rows up to 65536 elements still fit the registers of one workgroup (32 x 16 bytes per lane)
    quantize_rows_vec_kernel<DTYPE, 256, (DTYPE != 2 ? 32 : 1), true, TRITON><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
  } else {
    quantize_rows_vec_kernel<DTYPE, 256, 1, false, TRITON><<<(unsigned)rows, 256, 0, s>>>(x, rows, k, in_stride, out, out_stride, scale, scale_ub, jag);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_quantize_fp8_row(const void* x, int dtype, int64_t rows, int64_t K, int64_t in_stride,
                                   void* xq, int64_t K_out, float* scale, const float* scale_ub,
                                   const void* zero_start, int zero_start_is_i32, int64_t rows_per_group,
                                   int triton_arithmetic, float triton_eps, hipStream_t s) {
  uint8_t* out = reinterpret_cast<uint8_t*>(xq);
  const JaggedRows jag{zero_start, rows_per_group > 0 ? rows_per_group : 1, zero_start_is_i32, triton_eps};
  if (triton_arithmetic) {
    switch (dtype) {
      case 0: return launch_quantize_t<0, true>(x, rows, K, in_stride, out, K_out, scale, scale_ub, jag, s);
      case 1: return launch_quantize_t<1, true>(x, rows, K, in_stride, out, K_out, scale, scale_ub, jag, s);
      default: return launch_quantize_t<2, true>(x, rows, K, in_stride, out, K_out, scale, scale_ub, jag, s);
    }
  }
  switch (dtype) {
    case 0: return launch_quantize_t<0, false>(x, rows, K, in_stride, out, K_out, scale, scale_ub, jag, s);
    case 1: return launch_quantize_t<1, false>(x, rows, K, in_stride, out, K_out, scale, scale_ub, jag, s);
    default: return launch_quantize_t<2, false>(x, rows, K, in_stride, out, K_out, scale, scale_ub, jag, s);
  }
}

hipError_t launch_dequantize_fp8_row(const void* xq, const float* scale, int64_t rows, int64_t K, void* out,
                                     hipStream_t s) {
  const int64_t total = rows * K;
  if (total <= 0) return hipSuccess;
  const bool vec_ok = K % 16 == 0 && reinterpret_cast<uintptr_t>(xq) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (vec_ok) {
    const int64_t chunks = total / 16;
    const int64_t want = (chunks + 255) / 256;
    // enough resident waves to cover HBM latency; each lane then walks the tensor grid-stride
    const unsigned blocks = (unsigned)(want > 256 * 32 ? 256 * 32 : want);
    dequantize_rows_vec_kernel<<<blocks, 256, 0, s>>>(reinterpret_cast<const uint8_t*>(xq), scale, chunks, (int)(K / 16),
                                                     reinterpret_cast<uint16_t*>(out));
  } else if (K % 8 == 0 && reinterpret_cast<uintptr_t>(xq) % 8 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t chunks = total / 8;
    const int64_t want = (chunks + 255) / 256;
    const unsigned blocks = (unsigned)(want > 256 * 32 ? 256 * 32 : want);
    dequantize_rows_vec8_kernel<<<blocks, 256, 0, s>>>(reinterpret_cast<const uint8_t*>(xq), scale, chunks, (int)(K / 8),
                                                      reinterpret_cast<uint16_t*>(out));
  } else {
    const int64_t want = ((total + 7) / 8 + 255) / 256;
    const unsigned blocks = (unsigned)(want > 65536 ? 65536 : want);
    dequantize_rows_generic_kernel<<<blocks, 256, 0, s>>>(reinterpret_cast<const uint8_t*>(xq), scale, total, K,
                                                         reinterpret_cast<uint16_t*>(out));
  }
  return hipGetLastError();
}

hipError_t launch_cast_e4m3fn(const float* in, int64_t n, void* out, hipStream_t s) {
  const int64_t want = (n + 255) / 256;
  const unsigned blocks = (unsigned)(want < 1 ? 1 : (want > 65536 ? 65536 : want));
  cast_e4m3fn_kernel<<<blocks, 256, 0, s>>>(in, n, reinterpret_cast<uint8_t*>(out));
  return hipGetLastError();
}

}  // namespace mslk_amd
