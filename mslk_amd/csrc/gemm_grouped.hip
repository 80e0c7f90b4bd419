// Grouped (MoE) f8f8bf16_rowwise for gfx950: the dense LDS-tiled MFMA tile driven by a
// per-launch tile list over all groups.
//
//   * TensorList API (reference csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:481-559):
//     shapes are host-known, so the group descriptors and their tile prefix sums travel in the
//     kernel-argument block (no device-side setup launches, no workspace, graph-safe).
//   * Stacked API (same file, 607-655): group sizes live in device memory; every workgroup walks the
//     G sizes (L2-resident) to find its tile, and the grid is sized for the worst case
//     ceil(total_M / BM) + G row tiles, so no host synchronisation is needed.
// Empty groups own no tiles and are never touched.
#include "gemm_tile.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

constexpr int kXcds = 8;
constexpr int kGroupM = 4;

// Tile order inside one group: panels of kGroupM row tiles, column-major inside a panel.
MSLK_AMD_DEVINL void local_tile(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int panel = kGroupM * tiles_n;
  const int first_m = (t / panel) * kGroupM;
  const int rows = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  tm = first_m + (t % panel) % rows;
  tn = (t % panel) / rows;
}

template <int BM, int BN>
__global__ __launch_bounds__(256) void grouped_tiled_kernel(GroupTable tab) {
  using TS = TileShape<BM, BN>;
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  // XCD x works on a contiguous slice of the tile list.
  const int per_xcd = (tab.total_tiles + kXcds - 1) / kXcds;
  const int t = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  if (t >= tab.total_tiles) return;
  int gi = 0;
  while (gi + 1 < tab.count && t >= tab.g[gi + 1].tile_begin) ++gi;
  const GroupDesc& d = tab.g[gi];
  const int tiles_m = (d.M + BM - 1) / BM, tiles_n = (d.N + BN - 1) / BN;
  int tm, tn;
  local_tile(t - d.tile_begin, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  GemmTile<TS, 0> tile;
  tile.run(lds, d.xq + (int64_t)m0 * d.K, d.wq + (int64_t)n0 * d.K, d.xs + m0, d.ws + n0, nullptr,
           d.y + (int64_t)m0 * d.N + n0, d.M - m0, d.N - n0, d.N, d.K);
}

template <int BM, int BN>
__global__ __launch_bounds__(256) void grouped_stacked_kernel(const uint8_t* xq, const uint8_t* wq, const float* xs,
                                                              const float* ws, const int64_t* m_sizes, int G,
                                                              int64_t total_M, int N, int K, uint16_t* y) {
  using TS = TileShape<BM, BN>;
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  const int tiles_n = (N + BN - 1) / BN;
  int t = blockIdx.x;
  int64_t row0 = 0;
  int gi = 0, Mg = 0;
  for (; gi < G; ++gi) {
    const int64_t mg = m_sizes[gi];
    const int tiles = (int)((mg + BM - 1) / BM) * tiles_n;
    if (t < tiles) { Mg = (int)mg; break; }
    t -= tiles;
    row0 += mg;
  }
  if (gi >= G || row0 + Mg > total_M) return;
  int tm, tn;
  local_tile(t, (Mg + BM - 1) / BM, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  GemmTile<TS, 0> tile;
  tile.run(lds, xq + (row0 + m0) * K, wq + ((int64_t)gi * N + n0) * K, xs + row0 + m0, ws + (int64_t)gi * N + n0,
           nullptr, y + (row0 + m0) * N + n0, Mg - m0, N - n0, N, K);
}

}  // namespace

bool grouped_tiled_supports(int N, int K) {
  return K % 16 == 0 && K >= 16 && (int64_t)256 * K < (int64_t(1) << 32) && N >= 1;
}

hipError_t launch_grouped_tiled(const GroupTable& t, hipStream_t s) {
  if (t.total_tiles <= 0) return hipSuccess;
  const int grid = ((t.total_tiles + kXcds - 1) / kXcds) * kXcds;
  grouped_tiled_kernel<256, 256><<<grid, 256, 0, s>>>(t);
  return hipGetLastError();
}

hipError_t launch_grouped_stacked(const uint8_t* xq, const uint8_t* wq, const float* xs, const float* ws,
                                  const int64_t* m_sizes, int G, int64_t total_M, int N, int K, uint16_t* y,
                                  hipStream_t s) {
  constexpr int BM = 256, BN = 256;
  const int64_t tiles = ((total_M + BM - 1) / BM + G) * ((N + BN - 1) / BN);
  if (tiles <= 0) return hipSuccess;
  grouped_stacked_kernel<BM, BN><<<(unsigned)tiles, 256, 0, s>>>(xq, wq, xs, ws, m_sizes, G, total_M, N, K, y);
  return hipGetLastError();
}

}  // namespace mslk_amd
