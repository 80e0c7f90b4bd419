// Fused producers of the quantized MoE activations for gfx950: the row is produced in fp32
// (SiLU-gated product, or a gathered token times its routing score) and quantized to e4m3fn in the
// same pass, so the fp32 / bf16 intermediate never goes to HBM.
//
//   silu_mul_quant                  (reference: _mslk_silu_mul_quant, mslk/moe/activation.py:232-300)
//       y = x0 * sigmoid(x0) * x1                       fp32, evaluated left to right
//   gather_scale_quant_dense_tokens (reference: _mslk_gather_scale_fp8_rowwise_quant_dense_tokens,
//                                    mslk/moe/gather_scatter.py:545-640)
//       y = x[token[i]] * scores[token[i], expert[i]]   fp32
// followed in both by the quantization of those kernels:
//   row_max = clamp(max|y|, 1e-12 [, *scale_ub]);  s = 448 / row_max;  out_scale = 1 / s;
//   code = e4m3fn_rne(clamp(y * s, -448, 448))
// (saturating, unlike the stand-alone quantizer whose contract is the reference's torch branch).
// The two divisions of the scale are IEEE-correct; sigmoid is rcp(1 + exp(-x)) on the hardware
// transcendental units, accurate to a few fp32 ulp.
//
// HBM-bound (silu: 4 B in + 1 B out per element for 16-bit inputs; gather: 2 B in + 1 B out).  One
// workgroup of 256 lanes owns a row; the produced fp32 values stay in registers between the
// maximum pass and the convert pass for rows of up to 16384 elements.
#include "common.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

constexpr float kMaxFp8 = 448.0f;
constexpr float kEps = 1e-12f;

template <int DTYPE>
MSLK_AMD_DEVINL float elem_to_f32(uint32_t bits) {
  if constexpr (DTYPE == 0) return bf16_bits_to_f32(bits);
  else return (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
}

MSLK_AMD_DEVINL float load_scalar_f32(const void* p, int64_t idx, int dtype) {
  if (dtype == 2) return static_cast<const float*>(p)[idx];
  const uint32_t b = static_cast<const uint16_t*>(p)[idx];
  return dtype == 0 ? bf16_bits_to_f32(b) : (float)__builtin_bit_cast(_Float16, (unsigned short)b);
}

MSLK_AMD_DEVINL int64_t load_index(const void* p, int64_t i, int is_i64) {
  return is_i64 ? static_cast<const int64_t*>(p)[i] : (int64_t) static_cast<const int32_t*>(p)[i];
}

// exp(-a) through the hardware base-2 exponential (1 ulp); the rounding error of the product
// -a * log2(e) is carried separately and folded back in, so the result stays within about 2 ulp for
// every argument instead of growing with |a|.
MSLK_AMD_DEVINL float exp_neg(float a) {
  constexpr float kLog2eHi = 1.44269502162933349609375f, kLog2eLo = 1.925963033500011e-8f, kLn2 = 0.693147182464599609375f;
  const float na = -a;
  const float t = na * kLog2eHi;
  float e = __builtin_fmaf(na, kLog2eHi, -t);
  e = __builtin_fmaf(na, kLog2eLo, e);
  const float p = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(p, e * kLn2, p);
}

// sigmoid through the hardware reciprocal (1 ulp): the convert that follows keeps 3 mantissa bits.
MSLK_AMD_DEVINL float silu_mul(float a, float b) {
  const float sig = __builtin_amdgcn_rcpf(1.0f + exp_neg(a));
  return (a * sig) * b;
}

// 8 consecutive 16-bit elements -> fp32
template <int DTYPE>
MSLK_AMD_DEVINL void unpack8(const v4i& v, float (&f)[8]) {
  const uint32_t w[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = elem_to_f32<DTYPE>(w[i] & 0xFFFFu);
    f[2 * i + 1] = elem_to_f32<DTYPE>(w[i] >> 16);
  }
}

// The row a workgroup works on, resolved once per workgroup.
struct RowSource {
  const char* a;    // x0 row, or the gathered x row
  const char* b;    // x1 row (silu only)
  float score;      // gather only
  bool live;
};

template <int OP>
MSLK_AMD_DEVINL RowSource resolve_row(const FusedQuantArgs& p, int64_t row) {
  RowSource r{nullptr, nullptr, 1.0f, false};
  if (p.valid_count != nullptr && row >= load_index(p.valid_count, 0, p.valid_is_i64)) return r;
  if constexpr (OP == kFusedSiluMul) {
    r.a = static_cast<const char*>(p.x0) + row * p.stride0 * 2;
    r.b = static_cast<const char*>(p.x1) + row * p.stride1 * 2;
    r.live = true;
  } else {
    const int64_t t = load_index(p.token_idx, row, p.token_is_i64);
    const int64_t e = load_index(p.expert_idx, row, p.expert_is_i64);
    if (t < 0 || t >= p.T || e < 0 || e >= p.E) return r;   // an index outside the tensors: touch nothing
    r.a = static_cast<const char*>(p.x0) + t * p.stride0 * 2;
    r.score = load_scalar_f32(p.scores, t * p.stride_t + e * p.stride_e, p.score_dtype);
    r.live = true;
  }
  return r;
}

template <int OP, int DTYPE>
MSLK_AMD_DEVINL void produce8(const RowSource& r, int vec, float (&y)[8]) {
  float a[8];
  unpack8<DTYPE>(__builtin_nontemporal_load(reinterpret_cast<const v4i*>(r.a) + vec), a);
  if constexpr (OP == kFusedSiluMul) {
    float b[8];
    unpack8<DTYPE>(__builtin_nontemporal_load(reinterpret_cast<const v4i*>(r.b) + vec), b);
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = silu_mul(a[i], b[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = a[i] * r.score;
  }
}

template <int OP, int DTYPE>
MSLK_AMD_DEVINL float produce1(const FusedQuantArgs& p, const RowSource& r, int k) {
  const float a = elem_to_f32<DTYPE>(reinterpret_cast<const uint16_t*>(r.a)[k]);
  if constexpr (OP == kFusedSiluMul) return silu_mul(a, elem_to_f32<DTYPE>(reinterpret_cast<const uint16_t*>(r.b)[k]));
  else return a * r.score;
}

MSLK_AMD_DEVINL uint32_t block_max_bits(uint32_t m, uint32_t* smem) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = m;
  __syncthreads();
  return max(max(smem[0], smem[1]), max(smem[2], smem[3]));
}

// |y| as raw bits orders like the value for non-negative floats and puts every NaN above +inf.
MSLK_AMD_DEVINL void row_scales(uint32_t max_bits, const float* scale_ub, float& s, float& inv) {
  const float amax = __uint_as_float(max_bits);
  float c = (amax < kEps) ? kEps : amax;
  if (scale_ub != nullptr) c = (c > *scale_ub) ? *scale_ub : c;
  s = kMaxFp8 / c;
  inv = 1.0f / s;
}

MSLK_AMD_DEVINL uint2 quantize8_saturating(const float (&y)[8], float s) {
  float f[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = __builtin_amdgcn_fmed3f(y[i] * s, -kMaxFp8, kMaxFp8);   // clamp; a NaN comes out as -448, as from fmin(fmax())
  // within +-448 the hardware conversion alone gives the codes (no NaN / overflow fix-up to apply)
  uint2 r;
  r.x = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false), true);
  r.y = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false), true);
  return r;
}

// Vector path: D % 8 == 0, input rows 16-byte aligned, output rows 8-byte aligned.  NV > 0: the lane
// keeps NV x 8 produced values in registers; NV == 0: rows of any length, produced twice.
// TEAM = 256: one workgroup per row; TEAM = 64: one wavefront per row, four rows per workgroup (rows of MoE
// intermediate sizes, 768 ... 2048 elements, leave most of a 256-lane team idle).
template <int OP, int DTYPE, int NV, int TEAM = 256>
__global__ __launch_bounds__(256) void fused_quant_vec_kernel(FusedQuantArgs p) {
  __shared__ uint32_t smem[4];
  const int64_t row = TEAM == 256 ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (TEAM != 256 && row >= p.rows) return;      // uniform over the wavefront; this variant has no workgroup barrier
  const RowSource r = resolve_row<OP>(p, row);   // uniform over the team
  if (!r.live) return;
  const int nvec = p.D >> 3;
  const int lane = TEAM == 256 ? (int)threadIdx.x : (int)(threadIdx.x & 63);
  uint32_t m = 0;
  float cache[NV > 0 ? NV : 1][8];
  if constexpr (NV > 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int vec = i * TEAM + lane;
      if (vec < nvec) {
        produce8<OP, DTYPE>(r, vec, cache[i]);
#pragma unroll
        for (int e = 0; e < 8; ++e) m = max(m, __float_as_uint(cache[i][e]) & 0x7FFFFFFFu);
      }
    }
  } else {
    for (int vec = lane; vec < nvec; vec += TEAM) {
      float y[8];
      produce8<OP, DTYPE>(r, vec, y);
#pragma unroll
      for (int e = 0; e < 8; ++e) m = max(m, __float_as_uint(y[e]) & 0x7FFFFFFFu);
    }
  }
  if constexpr (TEAM == 256) {
    m = block_max_bits(m, smem);
  } else {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
  }
  float s, inv;
  row_scales(m, p.scale_ub, s, inv);
  if (lane == 0) p.out_scale[row] = inv;
  uint2* out_row = reinterpret_cast<uint2*>(p.out + row * (int64_t)p.D);
  if constexpr (NV > 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int vec = i * TEAM + lane;
      if (vec < nvec) {
        const uint2 q = quantize8_saturating(cache[i], s);
        store8_write_through(reinterpret_cast<v2i*>(out_row + vec), v2i{(int)q.x, (int)q.y});
      }
    }
  } else {
    for (int vec = lane; vec < nvec; vec += TEAM) {
      float y[8];
      produce8<OP, DTYPE>(r, vec, y);
      const uint2 q = quantize8_saturating(y, s);
      store8_write_through(reinterpret_cast<v2i*>(out_row + vec), v2i{(int)q.x, (int)q.y});
    }
  }
}

// Any D, any alignment: scalar accesses, the row is produced twice.
template <int OP, int DTYPE>
__global__ __launch_bounds__(256) void fused_quant_generic_kernel(FusedQuantArgs p) {
  __shared__ uint32_t smem[4];
  const int64_t row = blockIdx.x;
  const RowSource r = resolve_row<OP>(p, row);
  if (!r.live) return;
  uint32_t m = 0;
  for (int k = threadIdx.x; k < p.D; k += 256) m = max(m, __float_as_uint(produce1<OP, DTYPE>(p, r, k)) & 0x7FFFFFFFu);
  m = block_max_bits(m, smem);
  float s, inv;
  row_scales(m, p.scale_ub, s, inv);
  if (threadIdx.x == 0) p.out_scale[row] = inv;
  for (int k = threadIdx.x; k < p.D; k += 256) {
    const float f = __builtin_fminf(__builtin_fmaxf(produce1<OP, DTYPE>(p, r, k) * s, -kMaxFp8), kMaxFp8);
    p.out[row * (int64_t)p.D + k] = (uint8_t)(cvt_pk_e4m3fn(f, 0.0f) & 0xFFu);
  }
}

template <int OP, int DTYPE>
hipError_t launch_fused_t(const FusedQuantArgs& p, hipStream_t s) {
  const unsigned rows = (unsigned)p.rows;
  const bool vec_ok = p.D % 8 == 0 && reinterpret_cast<uintptr_t>(p.x0) % 16 == 0 && (p.stride0 * 2) % 16 == 0 &&
                      (OP != kFusedSiluMul || (reinterpret_cast<uintptr_t>(p.x1) % 16 == 0 && (p.stride1 * 2) % 16 == 0)) &&
                      reinterpret_cast<uintptr_t>(p.out) % 8 == 0;
  if (!vec_ok) {
    fused_quant_generic_kernel<OP, DTYPE><<<rows, 256, 0, s>>>(p);
  } else if (p.D <= 2048 && p.rows >= 2048) {
    // enough rows to fill the chip with one wavefront each
    const unsigned blocks = (unsigned)((p.rows + 3) / 4);
    if (p.D <= 512) fused_quant_vec_kernel<OP, DTYPE, 1, 64><<<blocks, 256, 0, s>>>(p);
    else if (p.D <= 1024) fused_quant_vec_kernel<OP, DTYPE, 2, 64><<<blocks, 256, 0, s>>>(p);
    else fused_quant_vec_kernel<OP, DTYPE, 4, 64><<<blocks, 256, 0, s>>>(p);
  } else if (p.D <= 2048) {
    fused_quant_vec_kernel<OP, DTYPE, 1><<<rows, 256, 0, s>>>(p);
  } else if (p.D <= 4096) {
    fused_quant_vec_kernel<OP, DTYPE, 2><<<rows, 256, 0, s>>>(p);
  } else if (p.D <= 8192) {
    fused_quant_vec_kernel<OP, DTYPE, 4><<<rows, 256, 0, s>>>(p);
  } else if (p.D <= 16384) {
    fused_quant_vec_kernel<OP, DTYPE, 8><<<rows, 256, 0, s>>>(p);
  } else {
    fused_quant_vec_kernel<OP, DTYPE, 0><<<rows, 256, 0, s>>>(p);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_fused_quant(const FusedQuantArgs& p, int op, hipStream_t s) {
  if (p.rows <= 0 || p.D <= 0) return hipSuccess;
  if (op == kFusedSiluMul) return p.dtype == 0 ? launch_fused_t<kFusedSiluMul, 0>(p, s) : launch_fused_t<kFusedSiluMul, 1>(p, s);
  if (op == kFusedGatherScale)
    return p.dtype == 0 ? launch_fused_t<kFusedGatherScale, 0>(p, s) : launch_fused_t<kFusedGatherScale, 1>(p, s);
  return hipErrorInvalidValue;
}

}  // namespace mslk_amd
