// Skinny-M (decode) f8f8bf16_rowwise for gfx950: M <= 64, the weight matrix is streamed once.
//
// The op is HBM-bound: the N*K weight bytes dominate (reference shape class: Llama-70B o_proj;
// csrc/gemm/ck/fp8_rowwise/fp8fp8bf16_rowwise_gemm.hip:422-468 sends M < 64 to a tiny-tile kernel).
// What matters is the number of bytes in flight per CU, so the kernel is organised around deep,
// batched, register-resident loads and never touches LDS for the operands:
//   * a workgroup of 8 wavefronts owns NT*16 weight rows and ALL of K; the wavefronts take the
//     128-byte K steps round-robin (wave w: steps w, w+8, ...), so the workgroup reads 1 KiB of each of
//     its rows per round and no cross-workgroup reduction (workspace, atomics) is needed;
//   * per batch a wave issues the loads of U of its K steps (U * NT KiB * 2 of weights per wave) before
//     the first MFMA consumes them;
//   * weight fragments go global -> VGPR directly (each byte is used once).  Lane (i = l & 15, g = l >> 4)
//     loads bytes [16 g, 16 g + 16) and [64 + 16 g, 64 + 16 g + 16) of row i of the step, so one load
//     instruction covers 64 contiguous bytes per row; the activation fragment uses the same k
//     assignment (any k permutation shared by both MFMA operands gives the same dot products);
//   * activations (M x K, at most 512 KiB) are re-read from L2; each activation fragment is reused by
//     the NT weight fragments of the step, which bounds the L2 traffic for M > 16;
//   * the eight per-wave partial sums meet in LDS; the lanes reduce, scale and store bf16.
#include "common.h"
#include "kernels.h"
#include "quant_math.h"

namespace mslk_amd {
namespace {

constexpr int kStep = 128;

MSLK_AMD_DEVINL v4i load16_or_zero(const uint8_t* p, bool ok) {
  v4i z = {0, 0, 0, 0};
  if (ok) z = *reinterpret_cast<const v4i*>(p);
  return z;
}

// Weights are read exactly once: stream them past the caches.
MSLK_AMD_DEVINL v4i load16_stream(const uint8_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
}
// Cache policy of a global -> LDS load of bytes that are read exactly once (the weights of these kernels): non-temporal,
// as load16_stream is for register loads (the `nt` bit of the instruction).  N = K = 8192: M = 1 14.2 -> 13.5 us, M = 8
// 14.7 -> 13.8 us; the configuration with one K step per batch (32 < M <= 64) keeps the default policy (N = K = 4096,
// M = 64: 8.3 us against 8.7 with streamed weights).
constexpr int kStreamOnce = 2;

// One batch: the loads of U K-steps of this wave (steps kt0, kt0 + 8, ...), then their MFMAs.
// CHECKED = false is the fast path: every step lies fully inside K, so no lane is predicated.
// PS: the weights are in the blocked layout [N/16][K/64][4][16][16 B]; wp[tn] then points at this
// lane's 16 bytes of the first block of its row group, and the two halves of a K step are the next
// two 1 KiB blocks, each read by the wave as one contiguous KiB.
template <int MT, int NT, int U, int kWaves, bool CHECKED, bool PS = false>
MSLK_AMD_DEVINL void skinny_batch(const uint8_t* const (&wp)[NT], const uint8_t* const (&xp)[MT], int kt0, int K, int g,
                                  v4f (&acc)[NT][MT]) {
  v8i wf[U][NT], xf[U][MT];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int k0 = (kt0 + u * kWaves) * kStep;
    const bool ok0 = !CHECKED || k0 + g * 16 < K, ok1 = !CHECKED || k0 + 64 + g * 16 < K;
#pragma unroll
    for (int tn = 0; tn < NT; ++tn) {
      v4i lo, hi;
      const int64_t w0 = PS ? (int64_t)k0 * 16 : k0, w1 = PS ? w0 + 1024 : w0 + 64;
      if constexpr (CHECKED) {
        lo = load16_or_zero(wp[tn] + w0, ok0);
        hi = load16_or_zero(wp[tn] + w1, ok1);
      } else {
        lo = load16_stream(wp[tn] + w0);
        hi = load16_stream(wp[tn] + w1);
      }
      wf[u][tn] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
#pragma unroll
    for (int tm = 0; tm < MT; ++tm) {
      v4i lo, hi;
      if constexpr (CHECKED) {
        lo = load16_or_zero(xp[tm] + k0, ok0);
        hi = load16_or_zero(xp[tm] + k0 + 64, ok1);
      } else {
        lo = *reinterpret_cast<const v4i*>(xp[tm] + k0);
        hi = *reinterpret_cast<const v4i*>(xp[tm] + k0 + 64);
      }
      xf[u][tm] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int tn = 0; tn < NT; ++tn)
#pragma unroll
      for (int tm = 0; tm < MT; ++tm)
        acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[u][tn], xf[u][tm], acc[tn][tm], 0, 0, 0, 0, 0, 0);
}

template <int MT, int NT, int U, int kWaves, int BIAS, bool PS>
__global__ __launch_bounds__(kWaves * 64) void skinny_kernel(GemmProblem p) {
  __shared__ float red[kWaves][NT][MT][256];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (NT * 16);
  const int K = p.K;

  // Rows beyond N / M are clamped to the last valid row: an MFMA output row or column depends only on
  // its own operand row, and the clamped ones are never stored.
  const uint8_t* wp[NT];
#pragma unroll
  for (int tn = 0; tn < NT; ++tn) {
    if constexpr (PS) {
      const int group = (n0 >> 4) + tn, groups = p.N >> 4;
      wp[tn] = p.wq + (int64_t)(group < groups ? group : groups - 1) * 16 * K + lane * 16;
    } else {
      const int row = n0 + tn * 16 + i;
      wp[tn] = p.wq + (int64_t)(row < p.N ? row : p.N - 1) * K + g * 16;
    }
  }
  const uint8_t* xp[MT];
#pragma unroll
  for (int tm = 0; tm < MT; ++tm) {
    const int m = tm * 16 + i;
    xp[tm] = p.xq + (int64_t)(m < p.M ? m : p.M - 1) * K + g * 16;
  }
  v4f acc[NT][MT];
#pragma unroll
  for (int tn = 0; tn < NT; ++tn)
#pragma unroll
    for (int tm = 0; tm < MT; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

  // Epilogue operands are fetched before the weight stream so that their (cold) latency is hidden:
  // value index t = 4 * l + r of a fragment holds D[n = 4 * (l >> 4) + r][m = l & 15]; the 512 lanes
  // cover the NT * MT * 256 values in ROUNDS rounds.
  constexpr int ROUNDS = (NT * MT * 256 + kWaves * 64 - 1) / (kWaves * 64);
  float e_xs[ROUNDS], e_ws[ROUNDS], e_b[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int v = threadIdx.x + r * kWaves * 64;
    const int frag = v >> 8, t = v & 255;
    const int tn = frag / MT, tm = frag % MT;
    const int n = n0 + tn * 16 + 4 * (t >> 6) + (t & 3);
    const int m = tm * 16 + ((t >> 2) & 15);
    const bool ok = frag < NT * MT && n < p.N && m < p.M;
    e_xs[r] = ok ? p.xs[m] : 0.f;
    e_ws[r] = ok ? p.ws[n] : 0.f;
    e_b[r] = 0.f;
    if constexpr (BIAS == 1) e_b[r] = ok ? reinterpret_cast<const float*>(p.bias)[n] : 0.f;
    if constexpr (BIAS == 2) e_b[r] = ok ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n]) : 0.f;
  }

  const int KT = (K + kStep - 1) / kStep;
  int kt0 = wave;
  if (K % (kWaves * kStep) == 0) {
    // every wave owns the same number of complete steps: unpredicated batches
    for (; kt0 + (U - 1) * kWaves < KT; kt0 += kWaves * U) skinny_batch<MT, NT, U, kWaves, false, PS>(wp, xp, kt0, K, g, acc);
    for (; kt0 < KT; kt0 += kWaves) skinny_batch<MT, NT, 1, kWaves, false, PS>(wp, xp, kt0, K, g, acc);
  } else {
    for (; kt0 < KT; kt0 += kWaves * 2) skinny_batch<MT, NT, 2, kWaves, true, PS>(wp, xp, kt0, K, g, acc);
  }

#pragma unroll
  for (int tn = 0; tn < NT; ++tn)
#pragma unroll
    for (int tm = 0; tm < MT; ++tm)
      *reinterpret_cast<v4f*>(&red[wave][tn][tm][lane * 4]) = acc[tn][tm];
  __syncthreads();

#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int v = threadIdx.x + r * kWaves * 64;
    const int frag = v >> 8, t = v & 255;
    const int tn = frag / MT, tm = frag % MT;
    const int n = n0 + tn * 16 + 4 * (t >> 6) + (t & 3);
    const int m = tm * 16 + ((t >> 2) & 15);
    if (frag >= NT * MT || n >= p.N || m >= p.M) continue;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum += red[w][tn][tm][t];
    float val = (sum * e_ws[r]) * e_xs[r];
    if constexpr (BIAS != 0) val += e_b[r];
    p.y[(int64_t)m * p.N + n] = (uint16_t)f32_to_out_bits(val, p.out_f16);
  }
}

template <int MT, int NT, int U, bool PS = false, int kWaves = 8>
hipError_t launch_cfg(const GemmProblem& p, hipStream_t s) {
  const unsigned grid = (unsigned)((p.N + NT * 16 - 1) / (NT * 16));
  if (dispatch_probe_record("skinny_registers<m_frags=%d,n_frags=%d,steps=%d>%s workgroups=%u", MT, NT, U, PS ? " preshuffled" : "", grid))
    return hipSuccess;
  switch (p.bias_dtype) {
    case 0: skinny_kernel<MT, NT, U, kWaves, 0, PS><<<grid, kWaves * 64, 0, s>>>(p); break;
    case 1: skinny_kernel<MT, NT, U, kWaves, 1, PS><<<grid, kWaves * 64, 0, s>>>(p); break;
    default: skinny_kernel<MT, NT, U, kWaves, 2, PS><<<grid, kWaves * 64, 0, s>>>(p); break;
  }
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Main variant (K % 1024 == 0): both operands staged through wave-private LDS.
//
// A register-direct fragment load touches 16 different 128-byte lines (64 bytes of each) per
// instruction, and the texture path handles such an instruction about four times slower than one that
// covers 8 full lines; with more than a few activation rows that path, not HBM, becomes the limit.
// Here every wave copies the weight rows AND the activation rows of its own K steps global -> LDS
// with DMA loads of 8 full lines each (the same XOR-swizzled 128-byte rows as the tiled kernel) and
// reads its MFMA fragments back from LDS.  The buffer is private to the wave, so no barrier is
// involved: a batch is "issue all DMA, wait for this wave's loads, multiply".
// ---------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

MSLK_AMD_DEVINL int row_swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

//
// PS (pre-shuffled weights, blocked layout [N/16][K/64][4][16][16 B]): a weight fragment is two
// contiguous KiB blocks, so the weights go global -> VGPR with full-line requests and only the
// activations are staged.
template <int MT, int NT, int U, int BIAS, bool PS = false>
__global__ __launch_bounds__(512) void skinny_lds_kernel(GemmProblem p) {
  constexpr int kWaves = 8;
  constexpr int WT = PS ? 0 : NT;                           // weight tiles staged in LDS per step
  constexpr int XBUF = (U * (MT + WT) * 2048 > NT * MT * 1024) ? U * (MT + WT) * 2048 : NT * MT * 1024;
  static_assert(XBUF >= NT * MT * 1024, "the reduction slot of a wave lives inside its staging buffer");
  __shared__ __attribute__((aligned(1024))) char lds[kWaves * XBUF];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (NT * 16);
  const int K = p.K;
  char* xbuf = lds + wave * XBUF;

  // weight rows of this workgroup, as DMA source offsets (same lane -> (row, chunk) map as the activations)
  uint32_t w_off[NT][2];
  const uint8_t* w_base = p.wq + (int64_t)n0 * K;
  const uint8_t* wps[NT];   // PS: this lane's 16 bytes of the first block of each row group
#pragma unroll
  for (int tn = 0; tn < NT; ++tn) {
    const int group = (n0 >> 4) + tn, groups = p.N >> 4;
    wps[tn] = p.wq + (int64_t)(group < groups ? group : groups - 1) * 16 * K + lane * 16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = 8 * h + (lane >> 3);
      const int row = tn * 16 + r;
      w_off[tn][h] = (uint32_t)(n0 + row < p.N ? row : p.N - 1 - n0) * (uint32_t)K + (((lane & 7) ^ row_swz(r)) << 4);
    }
  }
  // DMA source offsets: load h (0 / 1) of m-tile tm covers rows tm*16 + 8h + (lane >> 3); lane fetches the
  // logical 16-byte chunk that belongs at physical position (lane & 7) of its swizzled LDS row.
  uint32_t x_off[MT][2];
#pragma unroll
  for (int tm = 0; tm < MT; ++tm)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = 8 * h + (lane >> 3);
      const int m = tm * 16 + r;
      x_off[tm][h] = (uint32_t)(m < p.M ? m : p.M - 1) * (uint32_t)K + (((lane & 7) ^ row_swz(r)) << 4);
    }
  // Fragment read offsets: lane (i, g) reads logical chunks g and g + 4 of row i (the k assignment of the
  // weight fragments above).
  const int xr0 = i * 128 + ((g ^ row_swz(i)) << 4);
  const int xr1 = i * 128 + (((g + 4) ^ row_swz(i)) << 4);

  v4f acc[NT][MT];
#pragma unroll
  for (int tn = 0; tn < NT; ++tn)
#pragma unroll
    for (int tm = 0; tm < MT; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

  constexpr int ROUNDS = (NT * MT * 256 + kWaves * 64 - 1) / (kWaves * 64);
  float e_xs[ROUNDS], e_ws[ROUNDS], e_b[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int v = threadIdx.x + r * kWaves * 64;
    const int frag = v >> 8, t = v & 255;
    const int tn = frag / MT, tm = frag % MT;
    const int n = n0 + tn * 16 + 4 * (t >> 6) + (t & 3);
    const int m = tm * 16 + ((t >> 2) & 15);
    const bool ok = frag < NT * MT && n < p.N && m < p.M;
    e_xs[r] = ok ? p.xs[m] : 0.f;
    e_ws[r] = ok ? p.ws[n] : 0.f;
    e_b[r] = 0.f;
    if constexpr (BIAS == 1) e_b[r] = ok ? reinterpret_cast<const float*>(p.bias)[n] : 0.f;
    if constexpr (BIAS == 2) e_b[r] = ok ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n]) : 0.f;
  }

  const int KT = K / kStep;   // K % (8 * 128) == 0: every wave owns KT / 8 complete steps
  for (int kt0 = wave; kt0 < KT; kt0 += kWaves * U) {
    // Weights first: their HBM requests must not queue behind the (L2-resident) activation traffic.
    v8i wreg[U][NT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = kt0 + u * kWaves;
      if (kt < KT) {           // wave-uniform
        const int k0 = kt * kStep;
#pragma unroll
        for (int tn = 0; tn < NT; ++tn) {
          if constexpr (PS) {
            const v4i lo = load16_stream(wps[tn] + (int64_t)k0 * 16);
            const v4i hi = load16_stream(wps[tn] + (int64_t)k0 * 16 + 1024);
            wreg[u][tn] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          } else {
#pragma unroll
            for (int h = 0; h < 2; ++h)
              __builtin_amdgcn_global_load_lds((gbl_ptr_t)(w_base + k0 + w_off[tn][h]),
                                               (lds_ptr_t)(xbuf + ((u * (MT + WT) + MT + tn) * 2 + h) * 1024), 16, 0,
                                               U >= 2 ? kStreamOnce : 0);   // one step per batch: nothing overlaps the longer trip
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = kt0 + u * kWaves;
      if (kt < KT) {
        const int k0 = kt * kStep;
#pragma unroll
        for (int tm = 0; tm < MT; ++tm)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(p.xq + k0 + x_off[tm][h]),
                                             (lds_ptr_t)(xbuf + ((u * (MT + WT) + tm) * 2 + h) * 1024), 16, 0, 0);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's DMA has landed in its private buffer
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (kt0 + u * kWaves < KT) {
        v8i wf[NT];
#pragma unroll
        for (int tn = 0; tn < NT; ++tn) {
          if constexpr (PS) {
            wf[tn] = wreg[u][tn];
          } else {
            const char* wt = xbuf + (u * (MT + WT) + MT + tn) * 2048;
            const v4i lo = *reinterpret_cast<const v4i*>(wt + xr0);
            const v4i hi = *reinterpret_cast<const v4i*>(wt + xr1);
            wf[tn] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          }
        }
#pragma unroll
        for (int tm = 0; tm < MT; ++tm) {
          const char* xt = xbuf + (u * (MT + WT) + tm) * 2048;
          const v4i lo = *reinterpret_cast<const v4i*>(xt + xr0);
          const v4i hi = *reinterpret_cast<const v4i*>(xt + xr1);
          const v8i xf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
          for (int tn = 0; tn < NT; ++tn)
            acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[tn], xf, acc[tn][tm], 0, 0, 0, 0, 0, 0);
        }
      }
    }
    // the next batch re-uses the buffer: all LDS reads above have returned (their MFMAs were issued)
  }

  // Reduction across the 8 waves: each wave parks its partial tiles in its own (now dead) staging buffer.
  float* red = reinterpret_cast<float*>(xbuf);
#pragma unroll
  for (int tn = 0; tn < NT; ++tn)
#pragma unroll
    for (int tm = 0; tm < MT; ++tm)
      *reinterpret_cast<v4f*>(&red[(tn * MT + tm) * 256 + lane * 4]) = acc[tn][tm];
  __syncthreads();
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int v = threadIdx.x + r * kWaves * 64;
    const int frag = v >> 8, t = v & 255;
    const int tn = frag / MT, tm = frag % MT;
    const int n = n0 + tn * 16 + 4 * (t >> 6) + (t & 3);
    const int m = tm * 16 + ((t >> 2) & 15);
    if (frag >= NT * MT || n >= p.N || m >= p.M) continue;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum += reinterpret_cast<const float*>(lds + w * XBUF)[frag * 256 + t];
    float val = (sum * e_ws[r]) * e_xs[r];
    if constexpr (BIAS != 0) val += e_b[r];
    p.y[(int64_t)m * p.N + n] = (uint16_t)f32_to_out_bits(val, p.out_f16);
  }
}

template <int MT, int NT, int U, bool PS = false>
hipError_t launch_lds(const GemmProblem& p, hipStream_t s) {
  const unsigned grid = (unsigned)((p.N + NT * 16 - 1) / (NT * 16));
  if (dispatch_probe_record("skinny_lds<m_frags=%d,n_frags=%d,steps=%d>%s workgroups=%u", MT, NT, U, PS ? " preshuffled" : "", grid))
    return hipSuccess;
  switch (p.bias_dtype) {
    case 0: skinny_lds_kernel<MT, NT, U, 0, PS><<<grid, 512, 0, s>>>(p); break;
    case 1: skinny_lds_kernel<MT, NT, U, 1, PS><<<grid, 512, 0, s>>>(p); break;
    default: skinny_lds_kernel<MT, NT, U, 2, PS><<<grid, 512, 0, s>>>(p); break;
  }
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Decode with the activation quantizer fused in: bf16 activations in, M <= 4, K % 1024 == 0.
//
// The reference quantizes the activations with one launch and multiplies with a second
// (bench/gemm/gemm_ops.py:593-673); at decode sizes the first launch costs about a third of the pair.  Here every
// workgroup quantizes the (at most 4) activation rows itself, with the arithmetic of the stand-alone quantizer
// (mslk/quantize/triton/fp8_quantize.py:356-378; the codes and scales are the same bits):
//   1. row maxima: the 512 lanes sweep each row with 16-byte loads (the rows stay in L2: M * K * 2 bytes in all),
//      wave reduction, partial maxima meet in LDS, every lane picks up the multipliers of the M rows;
//   2. the weight stream as in skinny_lds_kernel (DMA into wave-private LDS).  A wave owns the K steps
//      wave, wave + 8, ...: next to their weight loads it fetches the bf16 activations of just these steps (M * 256 bytes
//      per step, 8 elements per lane and load), converts them in registers and parks the codes in its private LDS
//      buffer, from where the MFMA fragment is two 16-byte reads.  The conversion work of a workgroup is therefore M * K
//      elements split over its 512 lanes.  No scale_ub here, so in a row with a finite maximum no product exceeds
//      448 (1 + 2^-22) and the conversion needs no overflow fix-up; rows with a NaN or an infinity take the quantizer's
//      own conversion routine.
// Workgroup 0 also writes the codes and the scales out when the caller wants them.
// ---------------------------------------------------------------------------------------------
MSLK_AMD_DEVINL v2i quantize8_bf16(v4i raw, float inv) {
  const uint32_t w[4] = {(uint32_t)raw.x, (uint32_t)raw.y, (uint32_t)raw.z, (uint32_t)raw.w};
  float f[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = __uint_as_float(w[j] << 16) * inv;
    f[2 * j + 1] = __uint_as_float(w[j] & 0xFFFF0000u) * inv;
  }
  int lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
  int hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
  // A row whose maximum is NaN or infinite has inv = NaN or 0 and NaN products (NaN * x, inf * 0); only such a row can
  // hold anything the plain conversion does not settle.  It takes the stand-alone quantizer's conversion, which forces
  // sign | 0x7F, so that the codes written out are that kernel's bits for every input, NaN signs included.
  if (!(inv > 0.f && inv < __builtin_inff())) {
    lo = (int)(cvt_pk_e4m3fn(f[0], f[1]) | (cvt_pk_e4m3fn(f[2], f[3]) << 16));
    hi = (int)(cvt_pk_e4m3fn(f[4], f[5]) | (cvt_pk_e4m3fn(f[6], f[7]) << 16));
  }
  return v2i{lo, hi};
}

constexpr int kFusedMaxM = 4;

template <int U, int BIAS>
__global__ __launch_bounds__(512) void skinny_fused_quant_kernel(GemmProblem p, const uint16_t* __restrict__ x, int64_t x_stride,
                                                                 uint8_t* __restrict__ xq_out, float* __restrict__ xs_out) {
  constexpr int kWaves = 8;
  constexpr int WBYTES = U * 2048;                       // U weight tiles (16 rows x 128 B) of one K step each
  constexpr int CBYTES = U * kFusedMaxM * 128;           // codes of up to 4 activation rows for the same U steps
  constexpr int XBUF = WBYTES + CBYTES;                  // 10 KiB per wave at U = 4: two workgroups fill the LDS of a CU exactly
  constexpr int NCH = U * kFusedMaxM * 16 / 64;          // 16-byte bf16 chunks (8 elements) per lane and batch, at most
  __shared__ __attribute__((aligned(1024))) char lds[kWaves * XBUF];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int K = p.K, M = p.M;
  char* xbuf = lds + wave * XBUF;
  // small arrays of the set-up phase live in the staging area, which the weight stream only starts to fill after the
  // last barrier of the set-up
  uint32_t* amax_part = reinterpret_cast<uint32_t*>(lds);              // [4][8]
  float* row_inv = reinterpret_cast<float*>(lds + 256);                // [4]
  float* row_scale = reinterpret_cast<float*>(lds + 256 + 16);         // [4]

  // weight rows of this workgroup as DMA source offsets (see skinny_lds_kernel)
  uint32_t w_off[2];
  const uint8_t* w_base = p.wq + (int64_t)n0 * K;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = 8 * h + (lane >> 3);
    w_off[h] = (uint32_t)(n0 + r < p.N ? r : p.N - 1 - n0) * (uint32_t)K + (((lane & 7) ^ row_swz(r)) << 4);
  }
  const int xr0 = i * 128 + ((g ^ row_swz(i)) << 4);
  const int xr1 = i * 128 + (((g + 4) ^ row_swz(i)) << 4);

  // epilogue operands first: their latency hides behind the quantizer
  const int t = threadIdx.x & 255;
  const int e_n = n0 + 4 * (t >> 6) + (t & 3);
  const int e_m = (t >> 2) & 15;
  const bool e_ok = threadIdx.x < 256 && e_n < p.N && e_m < M;
  const float e_ws = e_ok ? p.ws[e_n] : 0.f;
  float e_b = 0.f;
  if constexpr (BIAS == 1) e_b = e_ok ? reinterpret_cast<const float*>(p.bias)[e_n] : 0.f;
  if constexpr (BIAS == 2) e_b = e_ok ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[e_n]) : 0.f;

  // 1. row maxima (as raw bf16 bits: unsigned order equals numeric order for non-negative values, NaN sorts last)
  const int chunks = K >> 3;
  for (int r = 0; r < M; ++r) {
    const v4i* xr = reinterpret_cast<const v4i*>(x + (int64_t)r * x_stride);
    us2 acc2 = {0, 0};
    for (int c = threadIdx.x; c < chunks; c += kWaves * 64) {
      const v4i v = xr[c];
      const uint32_t w4[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) acc2 = __builtin_elementwise_max(acc2, __builtin_bit_cast(us2, w4[j] & 0x7FFF7FFFu));
    }
    uint32_t m = __builtin_bit_cast(uint32_t, acc2);
    m = max(m & 0xFFFFu, m >> 16);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
    if (lane == 0) amax_part[r * kWaves + wave] = m;
  }
  __syncthreads();
  if (threadIdx.x < M) {
    uint32_t mb = amax_part[threadIdx.x * kWaves];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mb = max(mb, amax_part[threadIdx.x * kWaves + w]);
    float inv, sc;
    scales_from_amax<0, false>(bf16_bits_to_f32(mb), nullptr, 0.f, inv, sc);
    row_inv[threadIdx.x] = inv;
    row_scale[threadIdx.x] = sc;
    if (blockIdx.x == 0 && xs_out != nullptr) xs_out[threadIdx.x] = sc;
  }
  __syncthreads();
  float inv_r[kFusedMaxM];
#pragma unroll
  for (int r = 0; r < kFusedMaxM; ++r) inv_r[r] = row_inv[r < M ? r : 0];
  const float e_xs = row_scale[e_m < M ? e_m : 0];
  __syncthreads();   // the staging area is free for the weight stream from here on

  // This lane's chunks of a batch: chunk c = (step u of the batch, row, 8-element column block) -- the same for every batch.
  const bool write_codes = blockIdx.x == 0 && xq_out != nullptr;
  const int per_step = M * 16;                         // chunks per K step
  int64_t c_src[NCH];                                  // element offset into x, less the K offset of the batch
  int c_dst[NCH];                                      // byte offset into the wave's code area; -1: no chunk
  int64_t c_out[NCH];                                  // byte offset into xq_out, less the K offset of the batch
  float c_inv[NCH];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = lane + j * 64;
    const int u = c / per_step, rem = c - u * per_step;
    const int row = rem >> 4, col = rem & 15;
    const bool ok = u < U;
    c_src[j] = (int64_t)row * x_stride + u * kWaves * kStep + col * 8;
    c_out[j] = (int64_t)row * K + u * kWaves * kStep + col * 8;
    c_dst[j] = ok ? (u * kFusedMaxM + row) * 128 + col * 8 : -1;
    c_inv[j] = row == 0 ? inv_r[0] : row == 1 ? inv_r[1] : row == 2 ? inv_r[2] : inv_r[3];
  }
  char* cbuf = xbuf + WBYTES;
  const char* xfrag = cbuf + (i < M ? i : M - 1) * 128 + g * 16;   // fragment rows beyond M repeat the last row; never stored

  // 2. weight stream: whole K steps, dealt to the eight waves in batches of U (the last batch may be partly empty)
  v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
  const int KT = K / kStep;
  for (int kt0 = wave; kt0 < KT; kt0 += kWaves * U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = kt0 + u * kWaves;
      if (kt < KT) {           // wave-uniform
#pragma unroll
        for (int h = 0; h < 2; ++h)
          __builtin_amdgcn_global_load_lds((gbl_ptr_t)(w_base + kt * kStep + w_off[h]), (lds_ptr_t)(xbuf + (u * 2 + h) * 1024), 16, 0, kStreamOnce);
      }
    }
    const int steps_left = (KT - kt0 + kWaves - 1) / kWaves;       // K steps of this batch that exist (wave-uniform), >= 1
    v4i raw[NCH];
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const bool ok = c_dst[j] >= 0 && (c_dst[j] >> 9) < steps_left;   // 512 bytes of codes per step
      raw[j] = v4i{0, 0, 0, 0};
      if (ok) raw[j] = *reinterpret_cast<const v4i*>(x + c_src[j] + (int64_t)kt0 * kStep);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's loads have landed
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const bool ok = c_dst[j] >= 0 && (c_dst[j] >> 9) < steps_left;
      if (ok) {
        const v2i q = quantize8_bf16(raw[j], c_inv[j]);
        *reinterpret_cast<v2i*>(cbuf + c_dst[j]) = q;
        if (write_codes) *reinterpret_cast<v2i*>(xq_out + c_out[j] + (int64_t)kt0 * kStep) = q;
      }
    }
    // the codes were written by other lanes of this wave: LDS operations of a wave complete in order, no barrier needed
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = kt0 + u * kWaves;
      if (kt < KT) {
        const char* wt = xbuf + u * 2048;
        const v4i wlo = *reinterpret_cast<const v4i*>(wt + xr0);
        const v4i whi = *reinterpret_cast<const v4i*>(wt + xr1);
        const v4i xlo = *reinterpret_cast<const v4i*>(xfrag + u * kFusedMaxM * 128);
        const v4i xhi = *reinterpret_cast<const v4i*>(xfrag + u * kFusedMaxM * 128 + 64);
        const v8i wf = __builtin_shufflevector(wlo, whi, 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i xf = __builtin_shufflevector(xlo, xhi, 0, 1, 2, 3, 4, 5, 6, 7);
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf, acc, 0, 0, 0, 0, 0, 0);
      }
    }
  }

  // reduction across the 8 waves in their (now dead) staging buffers, then scale, bias and store
  *reinterpret_cast<v4f*>(reinterpret_cast<float*>(xbuf) + lane * 4) = acc;
  __syncthreads();
  if (e_ok) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum += reinterpret_cast<const float*>(lds + w * XBUF)[t];
    float val = (sum * e_ws) * e_xs;
    if constexpr (BIAS != 0) val += e_b;
    p.y[(int64_t)e_m * p.N + e_n] = (uint16_t)f32_to_out_bits(val, p.out_f16);
  }
}

}  // namespace

bool skinny_fused_quant_supports(const GemmProblem& p, const void* x, int64_t x_stride) {
  return p.M >= 1 && p.M <= kFusedMaxM && p.N >= 1 && p.K >= 1024 && p.K % kStep == 0 &&
         (int64_t)64 * p.K < (int64_t(1) << 32) && !p.w_preshuffled && x_stride >= p.K && x_stride % 8 == 0 &&
         reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(p.wq) % 16 == 0;
}

hipError_t launch_skinny_fused_quant(const GemmProblem& p, const void* x, int64_t x_stride, void* xq_out, float* xs_out,
                                     hipStream_t s) {
  if (!skinny_fused_quant_supports(p, x, x_stride)) return hipErrorInvalidValue;
  if (xq_out != nullptr && reinterpret_cast<uintptr_t>(xq_out) % 8 != 0) return hipErrorInvalidValue;
  constexpr int U = 4;
  const uint16_t* xb = static_cast<const uint16_t*>(x);
  uint8_t* q = static_cast<uint8_t*>(xq_out);
  const unsigned grid = (unsigned)((p.N + 15) / 16);
  switch (p.bias_dtype) {
    case 0: skinny_fused_quant_kernel<U, 0><<<grid, 512, 0, s>>>(p, xb, x_stride, q, xs_out); break;
    case 1: skinny_fused_quant_kernel<U, 1><<<grid, 512, 0, s>>>(p, xb, x_stride, q, xs_out); break;
    default: skinny_fused_quant_kernel<U, 2><<<grid, 512, 0, s>>>(p, xb, x_stride, q, xs_out); break;
  }
  return hipGetLastError();
}

bool skinny_supports(const GemmProblem& p) {
  if (p.w_preshuffled && (p.N % 16 != 0 || p.K % 64 != 0)) return false;
  // the kernels form 32-bit byte offsets of up to 64 rows x K
  return p.M >= 1 && p.M <= 64 && p.K % 16 == 0 && p.K >= 16 && (int64_t)64 * p.K < (int64_t(1) << 32) &&
         reinterpret_cast<uintptr_t>(p.xq) % 16 == 0 && reinterpret_cast<uintptr_t>(p.wq) % 16 == 0;
}

hipError_t launch_skinny(const GemmProblem& p, hipStream_t s) {
  if (!skinny_supports(p)) return hipErrorInvalidValue;
  // (K steps that do not divide among the eight waves, as below: from 40 steps on, except for at most 16 rows on at most
  // 4096 weight rows -- M = 64, N = 8192, K = 13824: 35.6 -> 28.0 us; M = 8, N = 4096, K = 11008: 9.3 against 12.2 us)
  if (p.w_preshuffled && p.K % kStep == 0 && p.M > 4 &&
      (p.K % (8 * kStep) == 0 || (p.K >= 40 * kStep && !(p.M <= 16 && p.N <= 4096)))) {
    // weights straight into registers (contiguous KiB blocks), activations through LDS; 16 weight rows per workgroup
    // instead of 32 on narrow weights, which 32 would leave with fewer workgroups than CUs
    if (p.N <= 4096) {
      if (p.M <= 16) return launch_lds<1, 1, 4, true>(p, s);
      if (p.M <= 32) return launch_lds<2, 1, 1, true>(p, s);
      if (p.M <= 48) return launch_lds<3, 1, 1, true>(p, s);
      return launch_lds<4, 1, 1, true>(p, s);
    }
    if (p.M <= 16) return launch_lds<1, 2, 2, true>(p, s);
    if (p.M <= 32) return launch_lds<2, 2, 1, true>(p, s);
    if (p.M <= 48) return launch_lds<3, 2, 1, true>(p, s);
    return launch_lds<4, 2, 1, true>(p, s);
  }
  if (p.w_preshuffled) {   // weight fragments are contiguous KiB blocks: straight into registers
    if (p.M <= 16) return launch_cfg<1, 1, 8, true>(p, s);
    if (p.M <= 32) return launch_cfg<2, 2, 4, true>(p, s);
    if (p.M <= 48) return launch_cfg<3, 2, 4, true>(p, s);
    return launch_cfg<4, 2, 4, true>(p, s);
  }
  // Both operands through LDS, all global traffic in full lines: whole K steps, and when they do not divide evenly among
  // the eight waves (K % 1024 != 0: 11008, 13824 ...) enough of them that the uneven last batch is a small part --
  // K = 2560 (20 steps, a batch of M <= 16 is 32) is 39 % slower this way, K = 11008 / 13824 10 - 60 % faster
  // (M = 48, N = 2560, K = 11008: 26.7 -> 10.6 us; M = 2, N = 22016, K = 11008: 52.0 -> 47.4) except for at most eight
  // rows on at most 4096 weight rows (M = 1, N = 4096, K = 11008: 10.3 against 11.1 us).
  const bool even = p.K % (8 * kStep) == 0;
  if (p.K % kStep == 0 && (even || (p.K >= 40 * kStep && !(p.M <= 8 && p.N <= 4096)))) {
    if (p.M <= 16) return launch_lds<1, 1, 4>(p, s);
    if (p.M <= 32) return launch_lds<2, 1, 1>(p, s);
    // 32 weight rows per workgroup halve the activation re-reads, but up to N = 4096 they leave half the CUs
    // without a workgroup: 16 rows there (N = 4096, K = 14336, M = 48 / 64: 25.6 -> 19.7 / 27.6 -> 22.4 us).
    if (p.N <= 4096) return p.M <= 48 ? launch_lds<3, 1, 1>(p, s) : launch_lds<4, 1, 1>(p, s);
    return p.M <= 48 ? launch_lds<3, 2, 1>(p, s) : launch_lds<4, 2, 1>(p, s);
  }
  if (p.M <= 16) return launch_cfg<1, 1, 8>(p, s);
  if (p.M <= 32) return launch_cfg<2, 2, 4>(p, s);
  if (p.M <= 48) return launch_cfg<3, 2, 4>(p, s);
  return launch_cfg<4, 2, 4>(p, s);
}

}  // namespace mslk_amd
