// Dense f8f8bf16_rowwise for gfx950: LDS-tiled MFMA kernel (large shapes), a generic
// any-shape kernel, and the zero-fill used for empty problems.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include "gemm_dense_shapes.h"

namespace mslk_amd {
namespace {

constexpr int kCus = 256;     // compute units of a whole MI355X (used when the device cannot be queried)

struct DispatchProbe {
  bool active = false;
  char text[512] = "";
};
thread_local DispatchProbe g_probe;

}  // namespace

void dispatch_probe_begin() {
  g_probe.active = true;
  g_probe.text[0] = 0;
}
const char* dispatch_probe_end() {
  g_probe.active = false;
  return g_probe.text;
}
bool dispatch_probe_record(const char* fmt, ...) {
  if (!g_probe.active) return false;
  const size_t used = strlen(g_probe.text);
  if (used > 0 && used + 4 < sizeof(g_probe.text)) strcat(g_probe.text, " + ");
  const size_t at = strlen(g_probe.text);
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_probe.text + at, sizeof(g_probe.text) - at, fmt, ap);
  va_end(ap);
  return true;
}

// Compute units of the current device (a partitioned MI355X shows fewer than 256), as a multiple of the XCD count:
// the number of persistent workgroups and the CU count of the tile-shape thresholds.  Queried once per device.
int device_compute_units() {
  static std::atomic<int> cached[64];   // zero-initialised; concurrent first calls store the same value
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return kCus;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = kCus;
    cus = cus / kXcds * kXcds;
    if (cus < kXcds) cus = kXcds;
    cached[dev].store(cus, std::memory_order_relaxed);
  }
  return cus;
}

namespace {
// Measuring build of dense_tiled_kernel<TileShape<256, 256>> for shapes made of interior tiles only: the same tile
// map, K loop and fused epilogue, and per wave four readings of the constant-rate counter (100 MHz): kernel entry,
// first operands behind the first barrier, the K loop's hand-over of its last step, the end of the fused epilogue.
__global__ __launch_bounds__(256) void dense_phases_kernel(GemmProblem p, int tiles_m, int tiles_n, uint64_t* __restrict__ stamps) {
  using TS = TileShape<256, 256>;
  using Tile = GemmTile<TS, 0, false, false, TS::LA / 2, true>;
  const uint64_t t_entry = __builtin_amdgcn_s_memrealtime();
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  int tm, tn;
  if (!map_tile(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  const int m0 = tm * TS::kBM, n0 = tn * TS::kBN;
  Tile tile;
  tile.out_f16 = p.out_f16;
  tile.run_interior(lds, p.xq + (int64_t)m0 * p.K, p.wq + (int64_t)n0 * p.K, p.xs + m0, p.ws + n0, nullptr,
                    p.y + (int64_t)m0 * p.N + n0, p.N, p.K);
  const uint64_t t_end = __builtin_amdgcn_s_memrealtime();
  if ((threadIdx.x & 63) == 0) {
    uint64_t* o = stamps + ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4;
    o[0] = t_entry;
    o[1] = tile.stamp_first_operands;
    o[2] = tile.stamp_k_loop_end;
    o[3] = t_end;
  }
}

// Any shape, no alignment requirement: one lane per output element, sequential K.
__global__ __launch_bounds__(256) void generic_kernel(GemmProblem p) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)p.M * p.N) return;
  const int m = (int)(idx / p.N), n = (int)(idx % p.N);
  const uint8_t* a = p.xq + (int64_t)m * p.K;
  float acc = 0.f;
  if (p.w_preshuffled) {
    // element (n, k) of the blocked layout [N/16][K/64][4][16][16]
    const uint8_t* b = p.wq + (int64_t)(n >> 4) * 16 * p.K + (n & 15) * 16;
    for (int k = 0; k < p.K; ++k)
      acc += __builtin_amdgcn_cvt_f32_fp8((int)a[k], 0) *
             __builtin_amdgcn_cvt_f32_fp8((int)b[(int64_t)(k >> 6) * 1024 + ((k >> 4) & 3) * 256 + (k & 15)], 0);
  } else {
    const uint8_t* b = p.wq + (int64_t)n * p.K;
    for (int k = 0; k < p.K; ++k)
      acc += __builtin_amdgcn_cvt_f32_fp8((int)a[k], 0) * __builtin_amdgcn_cvt_f32_fp8((int)b[k], 0);
  }
  float v = (acc * p.ws[n]) * p.xs[m];
  if (p.bias_dtype == 1) v += reinterpret_cast<const float*>(p.bias)[n];
  else if (p.bias_dtype == 2) v += bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n]);
  p.y[idx] = (uint16_t)f32_to_out_bits(v, p.out_f16);
}

// Row-major [G, N, K] -> blocked [G][N/16][K/64][4][16][16 B] (reference: ck_preshuffle / preshuffle_b_mfma,
// mslk/quantize/shuffle.py:182-246).  A pure permutation of 16-byte chunks; one lane moves one chunk, and
// the lanes of a wave write 1 KiB contiguous while reading 16 rows x 64 bytes.
__global__ __launch_bounds__(256) void preshuffle_b_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, int64_t chunks,
                                                           int K) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int kblocks = K >> 6;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    // destination chunk c = ((group * kblocks + kb) * 4 + klane) * 16 + nlane   (group counts 16-row groups over G * N / 16)
    const int nlane = (int)(c & 15), klane = (int)((c >> 4) & 3);
    const int64_t blk = c >> 6;
    const int64_t group = blk / kblocks;
    const int kb = (int)(blk - group * kblocks);
    const int64_t row = group * 16 + nlane;
    dst[c] = src[row * (K >> 4) + kb * 4 + klane];
  }
}

// Rows of K bytes copied into rows of Kp bytes with a zero tail: one lane per 16-byte chunk of the destination.
// The source rows start at any byte, so the reads carry no alignment promise.
__global__ __launch_bounds__(256) void pad_rows_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                       int64_t chunks, int chunks_per_row, int K) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += stride) {
    const int64_t row = c / chunks_per_row;
    const int k0 = (int)(c - row * chunks_per_row) * 16;
    const uint8_t* in = src + row * K + k0;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (k0 + 16 <= K) {
      __builtin_memcpy(w, in, 16);   // alignment 1: the compiler picks whatever access width the target allows
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (k0 + i < K) w[i >> 2] |= (uint32_t)in[i] << (8 * (i & 3));
    }
    reinterpret_cast<v4i*>(dst)[c] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  }
}

__global__ void fill_zero_kernel(uint16_t* y, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) y[i] = 0;
}

}  // namespace

bool dense_tiled_supports(const GemmProblem& p) {
  if (p.w_preshuffled && (p.N % 16 != 0 || p.K % 64 != 0)) return false;   // the blocked layout itself needs this
  return p.K % 16 == 0 && p.K >= 16 && (int64_t)256 * p.K < (int64_t(1) << 32) && p.N < (1 << 26) &&
         reinterpret_cast<uintptr_t>(p.xq) % 16 == 0 && reinterpret_cast<uintptr_t>(p.wq) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(p.y) % 16 == 0;
}

hipError_t launch_dense_tiled(const GemmProblem& p, hipStream_t s) {
  if (!dense_tiled_supports(p)) return hipErrorInvalidValue;
  // Tile-count quantisation: with more 256 x 256 tiles than CUs the persistent workgroups run whole passes, and a
  // last pass that is less than half full costs a full tile time.  The rows of that pass are then computed by a
  // second launch, which picks smaller tiles for them (N = K = 8192, M = 2304: 160 -> 125 us; N = K = 4096, M = 4608:
  // 82 -> 62 us).
  {
    const int wgs = device_compute_units();
    const int64_t tiles_n = (p.N + 255) / 256, tiles = (int64_t)((p.M + 255) / 256) * tiles_n;
    if (tiles > wgs) {
      const int64_t passes = (tiles + wgs - 1) / wgs;
      const int64_t last = tiles - (passes - 1) * wgs;           // tiles of the last pass
      const int64_t rows1 = ((passes - 1) * wgs / tiles_n) * 256;   // rows whose tiles fit the full passes
      // ... and up to three quarters full when the remaining rows fit one pass of 192 x 256 tiles: a quarter less work
      // per tile than the pass of 256 x 256 tiles they replace
      const int64_t rest192 = (p.M - rows1 + 191) / 192 * tiles_n;
      if ((last * 2 <= wgs || (last * 4 <= wgs * 3 && rest192 <= wgs && p.K >= 2048)) && rows1 > 0 && rows1 < p.M) {
        GemmProblem a = p, b = p;
        a.M = (int)rows1;
        b.M = p.M - (int)rows1;
        b.xq += rows1 * p.K;
        b.xs += rows1;
        b.y += rows1 * p.N;
        const hipError_t e = launch_dense_tiled(a, s);
        return e != hipSuccess ? e : launch_dense_tiled(b, s);
      }
    }
  }
  // 256 x 256 tiles once they give most CUs work (one persistent workgroup per CU when there are more tiles than
  // CUs); smaller tiles below that.  Every tile-count threshold below was measured on a whole MI355X (256 CUs: 64, 128,
  // 160, 192, 256 tiles) and is written as a fraction of the CU count of the device, so a partition scales them.
  const int cus = device_compute_units();   // 256 on a whole MI355X; the thresholds below scale with a partition's CU count
  const int64_t big_tiles = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256);
  // 128 x 128 tiles: with at most one tile per CU a workgroup gets the whole LDS for a five-deep ring (its step is
  // much shorter than a memory round trip); with more tiles two workgroups per CU hide each other's latency better.
  const int64_t small_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
  // At most 128 / 64 such tiles: narrower tiles (128 x 64, 128 x 32; four waves stacked along M, six / eight ring
  // buffers) put the weight stream on two / four times as many CUs, still one workgroup per CU; the activations they
  // re-read come from L2.  Going narrower than one workgroup per CU was measured and is slower.
  if (p.w_preshuffled) return launch_dense_tiled_preshuffled(p, cus, s);
  // M <= 64 on wide row-major weights (the caller sends M <= 8 to the weight-streaming kernel): the activation rows
  // are re-read by every workgroup, so the tile is only as tall as M needs -- 32 x 32 (two waves) or 64 x 32 tiles with
  // six to eight ring buffers, two workgroups per CU.  Measured against the 128-row tiles and the streaming kernel
  // at N = 5120 ... 57344.  Above N = 8192 the 64 x 32 tiles of 32 < M <= 64 no longer fit one per CU and the CUs that
  // hold two move twice the activation bytes; 64 x 64 tiles halve the tile count and the activation traffic
  // (N = 10240, K = 8192, M = 64: 33.3 -> 28.3 us; N = 57344, K = 4096, M = 64: 68.4 -> 55.5 us).
  // The same holds for fewer rows on wider weights (M = 32: N = 10240, K = 8192 21.4 -> 20.0 us, N = 32768, K = 7168
  // 46.4 -> 39.0 us; M = 12, N = 28672, K = 8192 45.3 -> 39.8 us), down to M <= 16, where the 32 x 32 tiles hold up to
  // N = 16384 (N = 14336, K = 8192: 22.8 against 23.4 us).
  if (p.M <= 64 && p.N >= kShortTileMinN) {
    if (p.M <= 32 && p.N <= (p.M <= 16 ? 16384 : 8192)) return launch_dense_small_tile(kTile32x32, p, s);
    if (p.M > 32 ? p.N <= 8192 : (p.N > 16384 && p.N < 24576))   // M = 9, N = 22016, K = 8192: 36.8 against 38.9 us on 64 x 64 tiles
      return launch_dense_small_tile(kTile64x32, p, s);
    return launch_dense_small_tile(kTile64x64, p, s);
  }
  if (big_tiles > cus) return launch_persistent_shape<TileShape<256, 256>, false>(p, cus, s);
  // 128 x 256 tiles (wave tile 64 x 128, three ring buffers, one workgroup per CU) when they cover 160 ... 256 CUs in
  // a single pass and the 256 x 256 tiles would cover fewer than 160, or would leave their last row of tiles at most
  // half full -- fewer LDS bytes per MFMA than 128 x 128 tiles and half the row granularity of 256 x 256
  // (N = K = 8192, M = 1024: 66.4 -> 59.7 us; N = K = 4096, M = 2048: 31.6 -> 29.0 us; N = 57344, K = 8192, M = 128:
  // 118.5 -> 108.6 us).
  // 192 x 128 tiles (wave tile 96 x 64, three ring buffers) when the 128 x 128 tiles no longer fit one per CU and these
  // do: with at most one tile per CU the launch takes what one tile takes, and a tile's K step costs what it moves
  // into the LDS -- 40 KiB here against 48 KiB for 128 x 256 (M = 768, N = 7168, K = 6144: 45.8 -> 36.7 us;
  // M = 768, N = 6144, K = 7168: 47.5 -> 40.6; M = 768, N = K = 8192: 54.6 -> 49.0).
  if (small_tiles > cus && big_tiles <= cus / 2) {
    const int64_t tiles19 = (int64_t)((p.M + 191) / 192) * ((p.N + 127) / 128);
    if (tiles19 <= cus) return launch_dense_small_tile(kTile192x128, p, s);
  }
  {
    const int64_t rows128 = (p.M + 127) / 128;
    const int64_t tiles12 = rows128 * ((p.N + 255) / 256);
    if (tiles12 >= cus * 5 / 8 && tiles12 <= cus && (big_tiles < cus * 5 / 8 || rows128 % 2 == 1))
      return launch_tiled_shape<TileShape<128, 256, 2, 2, 3>, false, 1>(p, s);
  }
  // Otherwise 256 x 256 tiles from 129 tiles on: the 128 x 256 tiles would then need two passes and the co-resident
  // 128 x 128 tiles more than two per CU (N = 6144, M = 1536: 144 tiles, K = 8192: 100.0 -> 87.1 us, K = 4096:
  // 48.9 -> 39.5 us).
  if (big_tiles > cus / 2) {
    // 192 x 256 tiles (wave tile 96 x 128, two-plus-three buffers) where they still fit one per CU: a quarter less work
    // per tile on a third more CUs (M = 1536, N = K = 8192: 80.0 -> 76.3 us; M = 768, N = 16384, K = 8192: 85.0 -> 76.3;
    // M = 1344, N = 8192, K = 4096: 41.5 -> 37.5)
    const int64_t tiles19 = (int64_t)((p.M + 191) / 192) * ((p.N + 255) / 256);
    if (tiles19 <= cus && p.K >= 2048) return launch_tiled_shape<TileShape<192, 256>, false>(p, s);
    return launch_tiled_shape<TileShape<256, 256>, false, 1>(p, s);
  }
  // M > 64 with at most one 64 x 64 tile per CU: such tiles (four waves stacked along M, five ring buffers, two
  // workgroups per CU) wherever they cover at least as many CUs as the 128-row tiles below would, in a single pass:
  // rows 65 ... 128 then do not cost a second, half-empty 128-row tile's worth of activation traffic (N = K = 8192,
  // M = 96: 23.8 -> 21.2 us; N = 4096, K = 14336, M = 96: 36.3 -> 30.4 us; 1024^3: 5.9 -> 5.5 us).
  if (p.M > 64 && p.N >= 1024) {
    const int64_t tiles64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64);
    const int64_t rows128 = (p.M + 127) / 128;
    const int64_t tiles128 = small_tiles <= cus / 4 ? rows128 * ((p.N + 31) / 32) : small_tiles <= cus / 2 ? rows128 * ((p.N + 63) / 64) : small_tiles;
    if (tiles64 <= cus && tiles64 >= tiles128) return launch_dense_small_tile(kTile64x64, p, s);
  }
  if (small_tiles <= cus / 4 && p.N >= 64) return launch_dense_small_tile(kTile128x32, p, s);
  if (small_tiles <= cus / 2 && p.N >= 128) return launch_dense_small_tile(kTile128x64, p, s);
  if (small_tiles <= cus) {
    // 96 x 128 tiles (wave tile 48 x 64, ring of five) where they fit one per CU as well: never more work per tile, and
    // more tiles wherever M is not close under a multiple of 128 (M = 384, N = K = 8192: 192 -> 256 tiles, 39.5 -> 35.6 us;
    // M = 320, N = 6144, K = 13824: 144 -> 192 tiles, 61.5 -> 53.3 us; M = 192, N = 14336: the same 224 tiles, 21.8 us both)
    if ((int64_t)((p.M + 95) / 96) * ((p.N + 127) / 128) <= cus) return launch_dense_small_tile(kTile96x128, p, s);
    return launch_dense_small_tile(kTile128x128Ring, p, s);
  }
  return launch_dense_small_tile(kTile128x128, p, s);
}

hipError_t launch_generic(const GemmProblem& p, hipStream_t s) {
  if (dispatch_probe_record("generic_scalar")) return hipSuccess;
  const int64_t total = (int64_t)p.M * p.N;
  generic_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(p);
  return hipGetLastError();
}

hipError_t launch_preshuffle_b(const void* src, void* dst, int64_t G, int64_t N, int64_t K, hipStream_t s) {
  const int64_t chunks = G * N * (K / 16);
  if (chunks <= 0) return hipSuccess;
  const int64_t want = (chunks + 255) / 256;
  preshuffle_b_kernel<<<(unsigned)(want > 65536 ? 65536 : want), 256, 0, s>>>(static_cast<const v4i*>(src), static_cast<v4i*>(dst),
                                                                              chunks, (int)K);
  return hipGetLastError();
}

hipError_t launch_pad_rows(const uint8_t* src, uint8_t* dst, int64_t rows, int64_t K, int64_t Kp, hipStream_t s) {
  const int64_t chunks = rows * (Kp / 16);
  if (chunks <= 0) return hipSuccess;
  if (dispatch_probe_record("pad_rows")) return hipSuccess;
  const int64_t want = (chunks + 255) / 256;
  pad_rows_kernel<<<(unsigned)(want > 65536 ? 65536 : want), 256, 0, s>>>(src, dst, chunks, (int)(Kp / 16), (int)K);
  return hipGetLastError();
}

hipError_t launch_debug_gemm_phases(const GemmProblem& p, uint64_t* stamps, hipStream_t s) {
  const int tiles_m = p.M / 256, tiles_n = p.N / 256;
  const int grid = (tiles_m * tiles_n + kXcds - 1) / kXcds * kXcds;
  dense_phases_kernel<<<(unsigned)grid, 256, 0, s>>>(p, tiles_m, tiles_n, stamps);
  return hipGetLastError();
}

hipError_t launch_fill_zero_bf16(uint16_t* y, int64_t n, hipStream_t s) {
  if (n <= 0) return hipSuccess;
  if (dispatch_probe_record("fill_zero")) return hipSuccess;
  const int64_t want = (n + 255) / 256;
  fill_zero_kernel<<<(unsigned)(want > 4096 ? 4096 : want), 256, 0, s>>>(y, n);
  return hipGetLastError();
}

}  // namespace mslk_amd
