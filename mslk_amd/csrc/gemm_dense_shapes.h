// Tile-shape kernels of the dense f8f8bf16_rowwise GEMM and their launchers: one tile per workgroup and the persistent
// form, each for row-major and for pre-shuffled weights.  Included by the translation units that instantiate them
// (gemm_dense.hip: the large shapes on row-major weights; gemm_dense_small.hip: the small ones; gemm_dense_preshuffled.hip:
// pre-shuffled weights), so that the sets compile side by side.
#pragma once
#include "gemm_tile.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

constexpr int kXcds = 8;      // MI355X: 8 accelerator dies, workgroups are dealt to them round-robin
constexpr int kGroupM = 4;    // tiles of one XCD form kGroupM-row panels (L2 reuse of the WQ panel)

// Workgroup id -> tile.  Consecutive workgroup ids land on different XCDs (each with a private
// L2), so XCD x is handed a contiguous range of the panel-ordered tile list.
// Entry t of the panel-ordered tile list.
MSLK_AMD_DEVINL void list_tile(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int panel = kGroupM * tiles_n;
  const int first_m = (t / panel) * kGroupM;
  const int rows = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  tm = first_m + (t % panel) % rows;
  tn = (t % panel) / rows;
}

MSLK_AMD_DEVINL bool map_tile(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int ntiles = tiles_m * tiles_n;
  const int per_xcd = (ntiles + kXcds - 1) / kXcds;
  const int t = (bid % kXcds) * per_xcd + bid / kXcds;
  if (t >= ntiles || bid / kXcds >= per_xcd) return false;
  list_tile(t, tiles_m, tiles_n, tm, tn);
  return true;
}

// WS: the weights are fetched with non-temporal loads (shapes of one or two row tiles: no other tile of the XCD asks for
// a weight line again).
template <typename TS, int BIAS, bool PS, bool WS = false>
__global__ __launch_bounds__(TS::NTHREADS) void dense_tiled_kernel(GemmProblem p, int tiles_m, int tiles_n) {
  constexpr int BM = TS::kBM, BN = TS::kBN;
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  int tm, tn;
  if (!map_tile(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  GemmTile<TS, BIAS, PS, false, TS::LA / 2, false, WS> tile;
  tile.out_f16 = p.out_f16;
  const void* bias = nullptr;
  if constexpr (BIAS == 1) bias = reinterpret_cast<const float*>(p.bias) + n0;
  if constexpr (BIAS == 2) bias = reinterpret_cast<const uint16_t*>(p.bias) + n0;
  if constexpr (BIAS == 0 && TS::RING == 0 && TS::NW == 4 && TS::FM * TS::FN * 4 >= 256) {
    // tiles with every row and column: the epilogue starts inside the last K step
    if (decltype(tile)::interior_ok(p.ws + n0, bias, p.y + (int64_t)m0 * p.N + n0, p.M - m0, p.N - n0, p.N, p.K)) {
      tile.run_interior(lds, p.xq + (int64_t)m0 * p.K, p.wq + (int64_t)n0 * p.K, p.xs + m0, p.ws + n0, bias,
                        p.y + (int64_t)m0 * p.N + n0, p.N, p.K);
      return;
    }
  }
  tile.run(lds, p.xq + (int64_t)m0 * p.K, p.wq + (int64_t)n0 * p.K, p.xs + m0, p.ws + n0, bias,
           p.y + (int64_t)m0 * p.N + n0, p.M - m0, p.N - n0, p.N, p.K);
}

// More tiles than CUs: one workgroup per CU walks its share of the tile list (XCD x keeps its contiguous slice,
// its workgroups take the entries round-robin, so at any time an XCD works on neighbouring tiles as it does with
// one workgroup per tile).  The first DMA loads of the next tile are issued before the epilogue of the current one
// and land while it runs, and no workgroup has to be started per tile.
template <typename TS, int BIAS, bool PS>
__global__ __launch_bounds__(TS::NTHREADS) void dense_persistent_kernel(GemmProblem p, int tiles_m, int tiles_n) {
  static_assert(TS::RING == 0 && TS::NTHREADS == 256, "two-plus-three buffer tiles with four waves");
  constexpr int BM = TS::kBM, BN = TS::kBN;
  using Tile = GemmTile<TS, BIAS, PS, false, 0>;   // many tiles per XCD share every XQ line: one step ahead is enough
  // The epilogue parks its transposes in the two buffers the next tile's prologue does not fill.
  static_assert(2 * Tile::EPI_WAVE_BYTES <= TS::A_BYTES && 2 * Tile::EPI_WAVE_BYTES <= TS::B_BYTES, "transpose buffers fit");
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  const int ntiles = tiles_m * tiles_n;
  const int per_xcd = (ntiles + kXcds - 1) / kXcds;
  const int xcd = blockIdx.x % kXcds, stride = gridDim.x / kXcds;
  int j = blockIdx.x / kXcds;
  if (j >= per_xcd || xcd * per_xcd + j >= ntiles) return;
  Tile tile;
  tile.out_f16 = p.out_f16;
  const int wave = Tile::wave_id();
  char* const epi_buf = lds + (wave < 2 ? TS::A_BYTES + wave * Tile::EPI_WAVE_BYTES
                                        : 2 * TS::A_BYTES + 2 * TS::B_BYTES + (wave - 2) * Tile::EPI_WAVE_BYTES);
  int tm, tn;
  list_tile(xcd * per_xcd + j, tiles_m, tiles_n, tm, tn);
  tm = __builtin_amdgcn_readfirstlane(tm);   // the divisions above ran on the vector unit; the results are uniform
  tn = __builtin_amdgcn_readfirstlane(tn);
  tile.prologue(lds, p.xq + (int64_t)tm * BM * p.K, p.wq + (int64_t)tn * BN * p.K, p.M - tm * BM, p.N - tn * BN, p.K,
                (uint32_t)p.K);
  for (;;) {
    v4f acc[TS::FN][TS::FM];
    tile.template accumulate_issued<true>(lds, p.K, acc);
    const int m0 = tm * BM, n0 = tn * BN;
    j += stride;
    const bool more = __builtin_amdgcn_readfirstlane((int)(j < per_xcd && xcd * per_xcd + j < ntiles)) != 0;
    if (more) {
      list_tile(xcd * per_xcd + j, tiles_m, tiles_n, tm, tn);
      tm = __builtin_amdgcn_readfirstlane(tm);
      tn = __builtin_amdgcn_readfirstlane(tn);
      tile.prologue(lds, p.xq + (int64_t)tm * BM * p.K, p.wq + (int64_t)tn * BN * p.K, p.M - tm * BM, p.N - tn * BN, p.K,
                    (uint32_t)p.K);
    }
    const void* bias = nullptr;
    if constexpr (BIAS == 1) bias = reinterpret_cast<const float*>(p.bias) + n0;
    if constexpr (BIAS == 2) bias = reinterpret_cast<const uint16_t*>(p.bias) + n0;
    tile.epilogue_at(epi_buf, acc, p.xs + m0, p.ws + n0, bias, p.y + (int64_t)m0 * p.N + n0, p.M - m0, p.N - n0, p.N);
    if (!more) break;
    // The per-lane load offsets of the next tile are formed again here rather than carried through the epilogue,
    // which needs the registers.
    tile.init(p.xq + (int64_t)tm * BM * p.K, p.wq + (int64_t)tn * BN * p.K, p.M - tm * BM < BM ? p.M - tm * BM : BM,
              p.N - tn * BN < BN ? p.N - tn * BN : BN, (uint32_t)p.K);
  }
}

template <typename TS, bool PS>
hipError_t launch_persistent_shape(const GemmProblem& p, int wgs, hipStream_t s) {
  constexpr int BM = TS::kBM, BN = TS::kBN;
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  if (dispatch_probe_record("dense_persistent<%d,%d>%s tiles=%d workgroups=%d", BM, BN, PS ? " preshuffled" : "", tiles_m * tiles_n, wgs))
    return hipSuccess;
  switch (p.bias_dtype) {
    case 0: dense_persistent_kernel<TS, 0, PS><<<wgs, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
    case 1: dense_persistent_kernel<TS, 1, PS><<<wgs, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
    default: dense_persistent_kernel<TS, 2, PS><<<wgs, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
  }
  return hipGetLastError();
}

// STREAM_W: 0 never; 1 when the shape is one row of tiles, so that every weight line is asked for exactly once (measured at
// M = 16 ... 128 on six weight shapes: 3 - 11 % faster, e.g. N = K = 8192, M = 16: 14.9 -> 13.3 us; with two row tiles it
// depends on whether the two land in one XCD at the same time: 9 % faster at N = 28672, 24 % slower at 4096 x 14336);
// 2 always (tile shapes that are only picked for a single row of tiles).
template <typename TS, bool PS, int STREAM_W = 0>
hipError_t launch_tiled_shape(const GemmProblem& p, hipStream_t s) {
  constexpr int BM = TS::kBM, BN = TS::kBN;
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int ntiles = tiles_m * tiles_n;
  const int grid = ((ntiles + kXcds - 1) / kXcds) * kXcds;
  const bool stream = STREAM_W == 2 || (STREAM_W == 1 && tiles_m == 1);
  if (dispatch_probe_record("dense_tiled<%d,%d,waves=%dx%d,ring=%d>%s%s tiles=%d", BM, BN, TS::WM, TS::WN, TS::RING,
                            PS ? " preshuffled" : "", stream ? " weights streamed" : "", ntiles))
    return hipSuccess;
  if constexpr (STREAM_W != 0) {
    if (stream || STREAM_W == 2) {
      switch (p.bias_dtype) {
        case 0: dense_tiled_kernel<TS, 0, PS, true><<<grid, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
        case 1: dense_tiled_kernel<TS, 1, PS, true><<<grid, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
        default: dense_tiled_kernel<TS, 2, PS, true><<<grid, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
      }
      return hipGetLastError();
    }
  }
  if constexpr (STREAM_W != 2) {
    switch (p.bias_dtype) {
      case 0: dense_tiled_kernel<TS, 0, PS><<<grid, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
      case 1: dense_tiled_kernel<TS, 1, PS><<<grid, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
      default: dense_tiled_kernel<TS, 2, PS><<<grid, TS::NTHREADS, 0, s>>>(p, tiles_m, tiles_n); break;
    }
  }
  return hipGetLastError();
}

}  // namespace
}  // namespace mslk_amd
