// Measured ceilings of the machine for the two resources the path is priced against: a pure streaming read of HBM and a
// register-only FP8 MFMA loop.  Neither is part of the product path; they exist so that the roofline fractions the
// benchmark prints can be set beside what this GPU actually sustains, from committed code (bench.py --only ceilings).
// No counterpart in the reference, whose bench divides by fixed denominators (bench/gemm/gemm_bench.py:61-68).
#include "common.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// Streaming read into registers: every lane keeps eight 16-byte non-temporal loads in flight; the values are folded into
// one word that is stored only under a condition no input meets, so the loads cannot be dropped.
__global__ __launch_bounds__(256) void stream_read_kernel(const v4i* __restrict__ src, int64_t chunks, int* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int acc = 0;
  for (; c + 7 * stride < chunks; c += 8 * stride) {
    v4i v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + c + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; c < chunks; c += stride) {
    const v4i v = __builtin_nontemporal_load(src + c);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x5EEDBEEF && sink != nullptr) sink[0] = acc;
}

// The same bytes through the global -> LDS DMA form of the load, the way the GEMM kernels fetch their operands: each
// wave moves 1 KiB per instruction into a private 16 KiB ring and never reads it back.  NT: with the non-temporal bit,
// as the kernels fetch weights that are read once.
template <bool NT>
__global__ __launch_bounds__(256) void stream_dma_kernel(const uint8_t* __restrict__ src, int64_t kib, int* __restrict__ sink) {
  __shared__ __attribute__((aligned(1024))) char lds[4 * 16 * 1024];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  char* ring = lds + wave * 16 * 1024;
  const int64_t waves = (int64_t)gridDim.x * 4;
  int slot = 0;
  for (int64_t b = (int64_t)blockIdx.x * 4 + wave; b < kib; b += waves) {
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)(src + b * 1024 + lane * 16), (lds_ptr_t)(ring + slot * 1024), 16, 0, NT ? 2 : 0);
    slot = (slot + 1) & 15;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the loads have landed before the wave ends
  (void)sink;
}

// The two operand streams of the 128 x 64 tile kernel's K loop without its LDS reads and multiplies: a workgroup fetches
// the 128 activation rows of its row tile (shared with every workgroup of that row tile: L2 hits) and its own 64 weight
// rows (read by the row tiles of one panel only: HBM), 128 bytes of K per step through a ring of six 24 KiB stages, five
// steps ahead, a wave-level wait and a workgroup barrier per step -- the access pattern, tile order and pipeline depth
// of dense_tiled<128, 64, ring 6>.  WHICH: 1 activations only, 2 weights only, 3 both.  What the launch takes is what
// the memory system allows that kernel on the same operands.
template <int WHICH>
__global__ __launch_bounds__(256) void tile_streams_kernel(const uint8_t* __restrict__ x, const uint8_t* __restrict__ w, int K,
                                                           int tiles_m, int tiles_n) {
  constexpr int NS = 6, STAGE = 24 * 1024, XL = 4, WL = 2;    // per wave and step: four activation loads, two weight loads
  constexpr int PER = ((WHICH & 1) ? XL : 0) + ((WHICH & 2) ? WL : 0);
  __shared__ __attribute__((aligned(1024))) char lds[NS * STAGE];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // tile order of the dense kernels: XCD x (workgroup id mod 8) takes a contiguous slice of the list of panels of up to
  // four row tiles, column-major inside a panel
  const int ntiles = tiles_m * tiles_n, per_xcd = (ntiles + 7) / 8;
  const int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (t >= ntiles || (int)(blockIdx.x / 8) >= per_xcd) return;
  const int panel = 4 * tiles_n, first_m = (t / panel) * 4;
  const int rows = tiles_m - first_m < 4 ? tiles_m - first_m : 4;
  const int tm = first_m + (t % panel) % rows, tn = (t % panel) / rows;
  const uint8_t* xb = x + (int64_t)tm * 128 * K + (lane >> 3) * (int64_t)K + (lane & 7) * 16;   // a load covers 8 rows x 128 bytes
  const uint8_t* wb = w + (int64_t)tn * 64 * K + (lane >> 3) * (int64_t)K + (lane & 7) * 16;
  const int KT = K / 128;
  auto issue = [&](int kt) {
    char* st = lds + (kt % NS) * STAGE + wave * (STAGE / 4);
    if constexpr ((WHICH & 1) != 0) {
#pragma unroll
      for (int q = 0; q < XL; ++q)
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)(xb + (int64_t)(wave * XL + q) * 8 * K + kt * 128), (lds_ptr_t)(st + q * 1024), 16, 0, 0);
    }
    if constexpr ((WHICH & 2) != 0) {
#pragma unroll
      for (int q = 0; q < WL; ++q)
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)(wb + (int64_t)(wave * WL + q) * 8 * K + kt * 128), (lds_ptr_t)(st + (XL + q) * 1024), 16, 0, 0);
    }
  };
  for (int i = 0; i < NS - 1 && i < KT; ++i) issue(i);
  for (int kt = 0; kt < KT; ++kt) {
    if (kt + NS - 1 < KT) {
      issue(kt + NS - 1);
      constexpr int PENDING = (NS - 1) * PER;   // the loads of the five steps ahead may still be in flight
      __builtin_amdgcn_s_waitcnt(0x0F70 | (PENDING & 15) | ((PENDING >> 4) << 14));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0)
    }
    __builtin_amdgcn_s_barrier();
  }
}

// Register-only MFMA loops on the operands at `src` (4096 fragments of 32 bytes per lane slot): 64 (16x16x128) or 32
// (32x32x64) independent accumulators per wave, the wave tile of the GEMM (128 x 128 x 128 per iteration), one wave per
// SIMD.  No memory traffic inside the loop: what it sustains is the matrix cores' rate at the clock the power limit grants
// for these operand values.
__global__ __launch_bounds__(256) void mfma_16x16x128_kernel(const v8i* __restrict__ src, int iters, float* __restrict__ sink) {
  v8i a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = src[(threadIdx.x + i * 256) & 4095];
    b[i] = src[(threadIdx.x + 2048 + i * 256) & 4095];
  }
  v4f acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) s += acc[i][j][0] + acc[i][j][3];
  if (s == 123.456f && sink != nullptr) sink[0] = s;
}

__global__ __launch_bounds__(256) void mfma_32x32x64_kernel(const v8i* __restrict__ src, int iters, float* __restrict__ sink) {
  v8i a[8], b[8];   // 4 blocks of 32 rows x 2 halves of the 128-byte K step
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = src[(threadIdx.x + i * 256) & 4095];
    b[i] = src[(threadIdx.x + 2048 + i * 256) & 4095];
  }
  v16f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i * 2 + h], b[j * 2 + h], acc[i][j], 0, 0, 0, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][15];
  if (s == 123.456f && sink != nullptr) sink[0] = s;
}

}  // namespace

hipError_t launch_debug_stream_read(const void* src, int64_t bytes, int mode, int workgroups, void* sink, hipStream_t s) {
  if (mode == 0) stream_read_kernel<<<workgroups, 256, 0, s>>>(static_cast<const v4i*>(src), bytes / 16, static_cast<int*>(sink));
  else if (mode == 1) stream_dma_kernel<false><<<workgroups, 256, 0, s>>>(static_cast<const uint8_t*>(src), bytes / 1024, static_cast<int*>(sink));
  else stream_dma_kernel<true><<<workgroups, 256, 0, s>>>(static_cast<const uint8_t*>(src), bytes / 1024, static_cast<int*>(sink));
  return hipGetLastError();
}

hipError_t launch_debug_tile_streams(const void* x, const void* w, int K, int tiles_m, int tiles_n, int which, hipStream_t s) {
  const int grid = (tiles_m * tiles_n + 7) / 8 * 8;
  const uint8_t* xp = static_cast<const uint8_t*>(x);
  const uint8_t* wp = static_cast<const uint8_t*>(w);
  if (which == 1) tile_streams_kernel<1><<<grid, 256, 0, s>>>(xp, wp, K, tiles_m, tiles_n);
  else if (which == 2) tile_streams_kernel<2><<<grid, 256, 0, s>>>(xp, wp, K, tiles_m, tiles_n);
  else tile_streams_kernel<3><<<grid, 256, 0, s>>>(xp, wp, K, tiles_m, tiles_n);
  return hipGetLastError();
}

hipError_t launch_debug_mfma_loop(const void* operands, int form, int iters, int workgroups, void* sink, hipStream_t s) {
  if (form == 0) mfma_16x16x128_kernel<<<workgroups, 256, 0, s>>>(static_cast<const v8i*>(operands), iters, static_cast<float*>(sink));
  else mfma_32x32x64_kernel<<<workgroups, 256, 0, s>>>(static_cast<const v8i*>(operands), iters, static_cast<float*>(sink));
  return hipGetLastError();
}

}  // namespace mslk_amd
