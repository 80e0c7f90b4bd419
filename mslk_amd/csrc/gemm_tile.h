// LDS-tiled FP8 x FP8 -> fp32 MFMA main loop and fused rowwise-scale epilogue for gfx950.
//
// One workgroup of 256 lanes (4 wavefronts in a 2 x 2 grid) produces a BM x BN tile of
//   Y[m, n] = bf16( (sum_k XQ[m, k] * WQ[n, k]) * x_scale[m] * w_scale[n] + bias[n] )
// (reference math: csrc/gemm/ck/fp8_rowwise/kernels/fp8_rowwise_common.h:54-82,168-204; bias:
//  csrc/gemm/cutlass/f8f8bf16_rowwise/f8f8bf16_rowwise_common.cuh:150-198).
//
// Data movement
//   * K is consumed in steps of 128 bytes.  Each step's XQ tile (BM rows x 128 B) and WQ tile
//     (BN rows x 128 B) are copied global -> LDS by the DMA form of the 128-bit global load
//     (no VGPR staging).  One wave-level load fills 1024 contiguous LDS bytes = 8 tile rows.
//   * Inside a 128-byte LDS row the eight 16-byte chunks are XOR-permuted with
//     swz(row) = (row & 7) ^ ((row >> 3) & 1), so that the 16 lanes of an MFMA operand read
//     (16 consecutive rows, same logical chunk) touch 16 different 16-byte bank groups.  The DMA
//     cannot scatter inside a wave, so the permutation is applied on the GLOBAL side: lane l of a
//     load fetches logical chunk (l & 7) ^ swz(row) of its row.
//   * Two LDS stages; the loads of step k+1 are in flight while step k is multiplied.
// Math
//   * v_mfma_f32_16x16x128_f8f6f4 (both operands e4m3, unit block scales).  WQ rows are the first
//     operand and XQ rows the second, so a lane ends up holding 4 consecutive n for one m and
//     stores them as one 8-byte bf16x4.
//   * Both operands give lane (i = l & 15, g = l >> 4) the 32 bytes k in [32 g, 32 g + 32) of
//     row i; any k permutation would do as long as both operands share it.
#pragma once
#include "common.h"

namespace mslk_amd {

constexpr int kBK = 128;  // bytes (= fp8 elements) of K per main-loop step

template <int BM, int BN>
struct TileShape {
  static constexpr int kBM = BM, kBN = BN;
  static constexpr int FM = BM / 32;            // 16-row m fragments per wave (wave covers BM/2 rows)
  static constexpr int FN = BN / 32;            // 16-row n fragments per wave
  static constexpr int A_BYTES = BM * kBK;
  static constexpr int B_BYTES = BN * kBK;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static constexpr int LA = BM / 32;            // wave-level loads of the A tile per wave per step
  static constexpr int LB = BN / 32;
};

MSLK_AMD_DEVINL int lds_swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

MSLK_AMD_DEVINL void wait_vmcnt0() { __builtin_amdgcn_s_waitcnt(0x0F70); }

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

MSLK_AMD_DEVINL void dma16(const uint8_t* g, char* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)g, (lds_ptr_t)lds_wave_base, 16, 0, 0);
}

template <typename TS, int BIAS>
struct GemmTile {
  // Per-lane state that is constant over the K loop.
  uint32_t a_off[TS::LA];   // byte offset of this lane's 16-byte chunk relative to a_base, k = 0
  uint32_t b_off[TS::LB];
  const uint8_t* a_base;    // XQ + m0 * K   (wave-uniform)
  const uint8_t* b_base;    // WQ + n0 * K

  // xq/wq point at row m0 / n0 of the operands; rows_a / rows_b = valid rows from there (>= 1).
  MSLK_AMD_DEVINL void init(const uint8_t* xq_tile, const uint8_t* wq_tile, int rows_a, int rows_b, int K) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    a_base = xq_tile;
    b_base = wq_tile;
#pragma unroll
    for (int i = 0; i < TS::LA; ++i) {
      const int row = (wave * TS::LA + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      const int rc = row < rows_a ? row : rows_a - 1;   // clamp: edge tiles re-read the last row
      a_off[i] = (uint32_t)rc * (uint32_t)K + chunk * 16;
    }
#pragma unroll
    for (int i = 0; i < TS::LB; ++i) {
      const int row = (wave * TS::LB + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      const int rc = row < rows_b ? row : rows_b - 1;
      b_off[i] = (uint32_t)rc * (uint32_t)K + chunk * 16;
    }
  }

  // Issue the DMA loads of a full K step (128 valid bytes per row) starting at byte k0 into `stage`.
  MSLK_AMD_DEVINL void issue_loads(char* stage, int k0) {
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < TS::LA; ++i)
      dma16(a_base + k0 + a_off[i], stage + (wave * TS::LA + i) * 1024);
#pragma unroll
    for (int i = 0; i < TS::LB; ++i)
      dma16(b_base + k0 + b_off[i], stage + TS::A_BYTES + (wave * TS::LB + i) * 1024);
  }

  // K tail (K % 128 != 0, K % 16 == 0): only `k_valid` bytes of each row remain.  Chunks at or
  // beyond K are zero-filled with a plain LDS store by the lane that would have fetched them.
  MSLK_AMD_DEVINL void issue_loads_tail(char* stage, int k0, int k_valid) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < TS::LA; ++i) {
      const int row = (wave * TS::LA + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      char* dst = stage + (wave * TS::LA + i) * 1024;
      if (chunk * 16 < k_valid) dma16(a_base + k0 + a_off[i], dst);
      else *reinterpret_cast<uint4*>(dst + lane * 16) = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < TS::LB; ++i) {
      const int row = (wave * TS::LB + i) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ lds_swz(row);
      char* dst = stage + TS::A_BYTES + (wave * TS::LB + i) * 1024;
      if (chunk * 16 < k_valid) dma16(b_base + k0 + b_off[i], dst);
      else *reinterpret_cast<uint4*>(dst + lane * 16) = make_uint4(0, 0, 0, 0);
    }
  }

  // One K step of MFMAs out of `stage`.
  MSLK_AMD_DEVINL void compute(const char* stage, v4f (&acc)[TS::FN][TS::FM]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int i = lane & 15, g = lane >> 4;
    const int s = lds_swz(i);
    const int off0 = i * kBK + (((2 * g) ^ s) << 4);
    const int off1 = i * kBK + (((2 * g + 1) ^ s) << 4);
    const char* a_tile = stage + wm * (TS::kBM / 2) * kBK;
    const char* b_tile = stage + TS::A_BYTES + wn * (TS::kBN / 2) * kBK;
    v8i xf[TS::FM];
#pragma unroll
    for (int tm = 0; tm < TS::FM; ++tm) {
      const v4i lo = *reinterpret_cast<const v4i*>(a_tile + tm * 16 * kBK + off0);
      const v4i hi = *reinterpret_cast<const v4i*>(a_tile + tm * 16 * kBK + off1);
      xf[tm] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
#pragma unroll
    for (int tn = 0; tn < TS::FN; ++tn) {
      const v4i lo = *reinterpret_cast<const v4i*>(b_tile + tn * 16 * kBK + off0);
      const v4i hi = *reinterpret_cast<const v4i*>(b_tile + tn * 16 * kBK + off1);
      const v8i wf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int tm = 0; tm < TS::FM; ++tm)
        acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, xf[tm], acc[tn][tm], 0, 0, 0, 0, 0, 0);
    }
  }

  // Whole tile: K loop + epilogue.  m_rem / n_rem = valid rows / columns of this tile (>= 1).
  // y, xs point at row m0; ws, bias, and the column offset of y at n0 are applied by the caller
  // through y (= Y + m0 * N + n0), ws (= w_scale + n0) and bias (+ n0).
  MSLK_AMD_DEVINL void run(char* lds, const uint8_t* xq_tile, const uint8_t* wq_tile, const float* xs,
                           const float* ws, const void* bias, uint16_t* y, int m_rem, int n_rem, int N, int K) {
    init(xq_tile, wq_tile, m_rem < TS::kBM ? m_rem : TS::kBM, n_rem < TS::kBN ? n_rem : TS::kBN, K);
    v4f acc[TS::FN][TS::FM];
#pragma unroll
    for (int tn = 0; tn < TS::FN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TS::FM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    const int KT = K / kBK;          // full steps
    const int k_tail = K - KT * kBK;  // 0 or a multiple of 16
    if (KT > 0) issue_loads(lds, 0);
    for (int kt = 0; kt < KT; ++kt) {
      // Every wave has waited for its own DMA before the barrier, so after it the whole stage
      // kt & 1 is in LDS and nobody still reads the other stage (it was consumed in step kt - 1).
      wait_vmcnt0();
      __syncthreads();
      if (kt + 1 < KT) issue_loads(lds + ((kt + 1) & 1) * TS::STAGE_BYTES, (kt + 1) * kBK);
      compute(lds + (kt & 1) * TS::STAGE_BYTES, acc);
    }
    if (k_tail > 0) {
      char* stage = lds + (KT & 1) * TS::STAGE_BYTES;
      __syncthreads();
      issue_loads_tail(stage, KT * kBK, k_tail);
      wait_vmcnt0();
      __syncthreads();
      compute(stage, acc);
    }
    epilogue(acc, xs, ws, bias, y, m_rem, n_rem, N);
  }

  MSLK_AMD_DEVINL void epilogue(v4f (&acc)[TS::FN][TS::FM], const float* xs, const float* ws, const void* bias,
                                uint16_t* y, int m_rem, int n_rem, int N) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int mi = wm * (TS::kBM / 2) + (lane & 15);
    const int ni = wn * (TS::kBN / 2) + 4 * (lane >> 4);
    const bool vec_store = (N & 3) == 0;
    float xsv[TS::FM];
#pragma unroll
    for (int tm = 0; tm < TS::FM; ++tm) {
      const int m = mi + tm * 16;
      xsv[tm] = m < m_rem ? xs[m] : 0.f;
    }
#pragma unroll
    for (int tn = 0; tn < TS::FN; ++tn) {
      const int n = ni + tn * 16;
      float wsv[4], bv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool ok = n + r < n_rem;
        wsv[r] = ok ? ws[n + r] : 0.f;
        if constexpr (BIAS == 1) bv[r] = ok ? reinterpret_cast<const float*>(bias)[n + r] : 0.f;
        else if constexpr (BIAS == 2) bv[r] = ok ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(bias)[n + r]) : 0.f;
        else bv[r] = 0.f;
      }
#pragma unroll
      for (int tm = 0; tm < TS::FM; ++tm) {
        const int m = mi + tm * 16;
        if (m >= m_rem) continue;
        uint32_t h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = (acc[tn][tm][r] * xsv[tm]) * wsv[r];
          if constexpr (BIAS != 0) v += bv[r];
          h[r] = f32_to_bf16_bits(v);
        }
        uint16_t* dst = y + (int64_t)m * N + n;
        if (vec_store && n + 3 < n_rem) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < n_rem) dst[r] = (uint16_t)h[r];
        }
      }
    }
  }
};

}  // namespace mslk_amd
