// Skinny-M (decode) f8f8bf16_rowwise for gfx950: M <= 64, the weight matrix is streamed once.
//
// The op is HBM-bound: N*K weight bytes dominate (reference shape class: Llama-70B o_proj,
// csrc/gemm/ck/fp8_rowwise/fp8fp8bf16_rowwise_gemm.hip:422-468 sends M < 64 to a tiny-tile kernel).
// Here every workgroup owns 16 weight rows (one MFMA n-fragment) and ALL of K:
//   * the 4 wavefronts of the workgroup take the 128-byte K steps round-robin, so the workgroup
//     reads 512 contiguous bytes of each of its rows per round;
//   * weight fragments go global -> VGPR directly (each byte is used once: LDS would add nothing);
//     lane (i = l & 15, g = l >> 4) loads bytes [16 g, 16 g + 16) and [64 + 16 g, 64 + 16 g + 16) of
//     row i of the step, so one load instruction covers 64 contiguous bytes per row; the activation
//     fragment uses the same k assignment (any shared permutation of k is a valid MFMA operand pair);
//   * activations (M x K, a few hundred KB at most) are re-read from L2 by every workgroup;
//   * the four per-wave partial sums meet in LDS; 256 lanes reduce, scale and store bf16.
// There is no split-K across workgroups, hence no workspace and no atomics.
#include "common.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

constexpr int kStep = 128;

MSLK_AMD_DEVINL v4i load16_or_zero(const uint8_t* p, bool ok) {
  v4i z = {0, 0, 0, 0};
  return ok ? *reinterpret_cast<const v4i*>(p) : z;
}

template <int MT, int BIAS>
__global__ __launch_bounds__(256) void skinny_kernel(GemmProblem p) {
  __shared__ float red[4][MT][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int K = p.K;
  const int w_row = (n0 + i < p.N) ? n0 + i : p.N - 1;
  const uint8_t* wp = p.wq + (int64_t)w_row * K + g * 16;
  const uint8_t* xp[MT];
  bool xok[MT];
#pragma unroll
  for (int tm = 0; tm < MT; ++tm) {
    const int m = tm * 16 + i;
    xok[tm] = m < p.M;
    xp[tm] = p.xq + (int64_t)(xok[tm] ? m : 0) * K + g * 16;
  }
  v4f acc[MT];
#pragma unroll
  for (int tm = 0; tm < MT; ++tm) acc[tm] = v4f{0.f, 0.f, 0.f, 0.f};

  const int KT = (K + kStep - 1) / kStep;
#pragma unroll 4
  for (int kt = wave; kt < KT; kt += 4) {
    const int k0 = kt * kStep;
    const bool ok0 = k0 + g * 16 < K, ok1 = k0 + 64 + g * 16 < K;
    const v4i wlo = load16_or_zero(wp + k0, ok0);
    const v4i whi = load16_or_zero(wp + k0 + 64, ok1);
    const v8i wf = __builtin_shufflevector(wlo, whi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
    for (int tm = 0; tm < MT; ++tm) {
      const v4i xlo = load16_or_zero(xp[tm] + k0, ok0 && xok[tm]);
      const v4i xhi = load16_or_zero(xp[tm] + k0 + 64, ok1 && xok[tm]);
      const v8i xf = __builtin_shufflevector(xlo, xhi, 0, 1, 2, 3, 4, 5, 6, 7);
      acc[tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf, acc[tm], 0, 0, 0, 0, 0, 0);
    }
  }

#pragma unroll
  for (int tm = 0; tm < MT; ++tm)
    *reinterpret_cast<v4f*>(&red[wave][tm][lane * 4]) = acc[tm];
  __syncthreads();

  // value index t = 4 * lane' + r holds D[n = 4 * (lane' >> 4) + r][m = lane' & 15]
  const int t = threadIdx.x;
  const int n = n0 + 4 * (t >> 6) + (t & 3);
  const int mj = (t >> 2) & 15;
  if (n >= p.N) return;
  const float wsn = p.ws[n];
  float bn = 0.f;
  if constexpr (BIAS == 1) bn = reinterpret_cast<const float*>(p.bias)[n];
  if constexpr (BIAS == 2) bn = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n]);
#pragma unroll
  for (int tm = 0; tm < MT; ++tm) {
    const int m = tm * 16 + mj;
    if (m >= p.M) continue;
    const float sum = (red[0][tm][t] + red[1][tm][t]) + (red[2][tm][t] + red[3][tm][t]);
    float v = (sum * p.xs[m]) * wsn;
    if constexpr (BIAS != 0) v += bn;
    p.y[(int64_t)m * p.N + n] = (uint16_t)f32_to_bf16_bits(v);
  }
}

template <int MT>
hipError_t launch_mt(const GemmProblem& p, hipStream_t s) {
  const unsigned grid = (unsigned)((p.N + 15) / 16);
  switch (p.bias_dtype) {
    case 0: skinny_kernel<MT, 0><<<grid, 256, 0, s>>>(p); break;
    case 1: skinny_kernel<MT, 1><<<grid, 256, 0, s>>>(p); break;
    default: skinny_kernel<MT, 2><<<grid, 256, 0, s>>>(p); break;
  }
  return hipGetLastError();
}

}  // namespace

bool skinny_supports(const GemmProblem& p) {
  return p.M >= 1 && p.M <= 64 && p.K % 16 == 0 && p.K >= 16 &&
         reinterpret_cast<uintptr_t>(p.xq) % 16 == 0 && reinterpret_cast<uintptr_t>(p.wq) % 16 == 0;
}

hipError_t launch_skinny(const GemmProblem& p, hipStream_t s) {
  if (!skinny_supports(p)) return hipErrorInvalidValue;
  if (p.M <= 16) return launch_mt<1>(p, s);
  if (p.M <= 32) return launch_mt<2>(p, s);
  if (p.M <= 48) return launch_mt<3>(p, s);
  return launch_mt<4>(p, s);
}

}  // namespace mslk_amd
