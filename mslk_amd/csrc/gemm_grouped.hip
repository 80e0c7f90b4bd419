// Grouped (MoE) f8f8bf16_rowwise for gfx950: the dense LDS-tiled MFMA tile driven by a
// per-launch tile list over all groups.
//
//   * TensorList API (reference csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:481-559):
//     shapes are host-known, so the group descriptors and their tile prefix sums travel in the
//     kernel-argument block (no device-side setup launches, no workspace, graph-safe).
//   * Stacked API (same file, 607-655) and the offsets API (f8f8bf16_rowwise_grouped_mm, same file
//     720-845; its device-side layouts are restated from set_kernel_args, 161-296): group extents live
//     in device memory; every workgroup walks the G entries (L2-resident) to find its tile, and the
//     grid is sized for the worst case (one partial tile per group), so no host synchronisation is
//     needed.  The batched op (csrc/gemm/ck/fp8_rowwise_batched/fp8_rowwise_batched_gemm.hip:199-254)
//     is the uniform layout.
// Empty groups own no tiles and are never touched.
#include <algorithm>

#include "gemm_grouped_device.h"

namespace mslk_amd {
namespace {

template <int BM, int BN>
__global__ __launch_bounds__(256) void grouped_tiled_kernel(GroupTable tab) {
  using TS = TileShape<BM, BN>;
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  // XCD x works on its own contiguous slice of the tile list (the launcher has cut the list by estimated cost).
  const int xcd = blockIdx.x % kXcds;
  const int t = tab.xcd_begin[xcd] + blockIdx.x / kXcds;
  if (t >= tab.xcd_begin[xcd + 1]) return;
  // group lookup in one step: lane i compares against the first tile of group i (count <= 64, begins ascend)
  const int lane = threadIdx.x & 63;
  const int begin = lane < tab.count ? tab.g[lane].tile_begin : 0x7FFFFFFF;
  const int gi = __builtin_amdgcn_readfirstlane(__popcll(__ballot(t >= begin)) - 1);
  const GroupDesc& d = tab.g[gi];
  const int tiles_m = (d.M + BM - 1) / BM, tiles_n = (d.N + BN - 1) / BN;
  int tm, tn;
  const int panel_rows = local_tile(t - d.tile_begin, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  // ROWSKIP: the ragged last row tile of a group costs what its rows cost.  A tile alone in its panel is the only reader
  // of its weight block at that time: it fetches the weights with non-temporal loads.
  if (panel_rows == 1) {
    GemmTile<TS, 0, false, true, TS::LA / 2, false, true> tile;
    tile.run(lds, d.xq + (int64_t)m0 * d.K, d.wq + (int64_t)n0 * d.K, d.xs + m0, d.ws + n0, nullptr,
             d.y + (int64_t)m0 * d.N + n0, d.M - m0, d.N - n0, d.N, d.K);
  } else {
    GemmTile<TS, 0, false, true> tile;
    tile.run(lds, d.xq + (int64_t)m0 * d.K, d.wq + (int64_t)n0 * d.K, d.xs + m0, d.ws + n0, nullptr,
             d.y + (int64_t)m0 * d.N + n0, d.M - m0, d.N - n0, d.N, d.K);
  }
}

}  // namespace

// Host-side schedule of a TensorList launch.  Workgroup ids go round the eight XCDs, and inside an XCD the hardware
// hands the next workgroup to the first CU that is free -- so an XCD finishes when its share of the WORK is done, and
// the launch when the slowest XCD is.  Equal tile COUNTS per XCD are not equal work: a tile of an expert with one row
// tile fetches its whole weight block from HBM alone (measured about 67 us at K = 5120), a tile out of a panel of four
// row tiles shares it (59 us), and a ragged tile with a quarter of the rows takes about three quarters of a full one.
// The groups are therefore cut into panels of up to kGroupM row tiles (all column tiles of those rows: the unit inside
// which operand tiles are shared through the L2), every panel gets a cost from that model, the panels are dealt to the
// XCDs longest first onto the least loaded one -- every XCD gets dear and cheap panels alike; all the weight-bound ones
// on two XCDs was measured and is 7 - 13 % slower --, and inside an XCD the panels with the cheapest tiles come last, so
// that the last pass over the CUs is a short one.  Where the deal leaves an XCD more than 3 % of an even share away from
// it (few panels: one or two big groups), the boundary between two XCDs moves into a panel instead: its tiles are
// ordered column by column, so the two XCDs get column ranges of it.  A panel is just another group descriptor (same
// weights, row range of the activations and of the output); when the panels would not fit the descriptor table, whole
// groups are dealt.
hipError_t launch_grouped_tiled(const GroupTable& in, hipStream_t s) {
  if (in.total_tiles <= 0 || in.count <= 0) return hipSuccess;
  constexpr int BM = 256, BN = 256;
  struct Chunk { int group, row0, rows, tiles; float cost, cheapest; };
  Chunk chunks[kMaxGroupsPerLaunch];
  auto tile_cost = [](int rows, int sharing) {   // relative time of one tile: rows valid, `sharing` row tiles use its weights
    const int q = (rows + BM / 4 - 1) / (BM / 4);
    static const float base[5] = {0.f, 42.4f, 48.3f, 55.0f, 56.7f};
    return base[q < 4 ? q : 4] + 9.3f / (float)sharing;
  };
  auto cut = [&](int rows_per_chunk) {   // number of chunks, or -1 if they do not fit
    int n = 0;
    for (int g = 0; g < in.count; ++g) {
      const GroupDesc& d = in.g[g];
      const int tiles_n = (d.N + BN - 1) / BN;
      for (int64_t r0 = 0; r0 < d.M; r0 += rows_per_chunk) {
        if (n == kMaxGroupsPerLaunch) return -1;
        const int rows = (int)(d.M - r0 < rows_per_chunk ? d.M - r0 : rows_per_chunk);
        const int tiles_m = (rows + BM - 1) / BM;
        Chunk& c = chunks[n++];
        c.group = g; c.row0 = (int)r0; c.rows = rows; c.tiles = tiles_m * tiles_n;
        const int last = rows - (tiles_m - 1) * BM;
        c.cheapest = tile_cost(last, tiles_m);
        c.cost = (float)tiles_n * ((float)(tiles_m - 1) * tile_cost(BM, tiles_m) + c.cheapest);
      }
    }
    return n;
  };
  int n = cut(kGroupM * BM);
  if (n < 0) n = cut(0x7FFFFF00);   // one chunk per group always fits
  // longest first onto the least loaded XCD
  int order[kMaxGroupsPerLaunch];
  for (int i = 0; i < n; ++i) order[i] = i;
  std::stable_sort(order, order + n, [&](int a, int b) { return chunks[a].cost > chunks[b].cost; });
  int bin_of[kMaxGroupsPerLaunch];
  float load[kXcds] = {};
  double total = 0.0;
  for (int i = 0; i < n; ++i) {
    int best = 0;
    for (int x = 1; x < kXcds; ++x)
      if (load[x] < load[best]) best = x;
    bin_of[order[i]] = best;
    load[best] += chunks[order[i]].cost;
    total += chunks[order[i]].cost;
  }
  // inside an XCD: panels whose cheapest tile is expensive first
  std::stable_sort(order, order + n, [&](int a, int b) {
    if (bin_of[a] != bin_of[b]) return bin_of[a] < bin_of[b];
    return chunks[a].cheapest > chunks[b].cheapest;
  });
  GroupTable t;
  t.count = n;
  int tiles = 0;
  for (int i = 0; i < n; ++i) {
    const Chunk& c = chunks[order[i]];
    const GroupDesc& d = in.g[c.group];
    GroupDesc& o = t.g[i];
    o = d;
    o.xq = d.xq + (int64_t)c.row0 * d.K;
    o.xs = d.xs + c.row0;
    o.y = d.y + (int64_t)c.row0 * d.N;
    o.M = c.rows;
    o.tile_begin = tiles;
    tiles += c.tiles;
  }
  t.total_tiles = tiles;
  // XCD x works on tiles [xcd_begin[x], xcd_begin[x + 1]).  Two plans: the deal (whole panels per XCD), and the same list
  // cut into eight runs of equal cost, a cut falling wherever the running cost reaches the next eighth.  Each is priced as
  // the slowest XCD's passes over its CUs (tiles / CUs of an XCD, rounded up) times the mean cost of its tiles; the deal
  // keeps every XCD at whole panels -- multiples of the column count, which full passes are made of -- and wins whenever
  // there are panels enough (measured: cutting cfg4 evenly by cost costs 7 %, because the cuts leave partial passes);
  // the even cut wins when the deal leaves XCDs idle (one group of 1024 rows: 189 -> 47 us).
  const int cus_per_xcd = device_compute_units() / kXcds;
  int plan_a[kXcds + 1], plan_b[kXcds + 1];
  plan_a[0] = plan_b[0] = 0;
  plan_a[kXcds] = plan_b[kXcds] = tiles;
  const double share = total / kXcds;
  for (int x = 0, i = 0; x + 1 < kXcds; ++x) {
    while (i < n && bin_of[order[i]] <= x) ++i;
    plan_a[x + 1] = i < n ? t.g[i].tile_begin : tiles;
    const double target = share * (x + 1);
    double done = 0.0;
    int j = 0;
    while (j + 1 < n && done + chunks[order[j]].cost < target) done += chunks[order[j++]].cost;
    const Chunk& c = chunks[order[j]];
    int in_chunk = (int)((target - done) / ((double)c.cost / c.tiles) + 0.5);   // a chunk's tiles are taken to cost the same
    in_chunk = in_chunk < 0 ? 0 : (in_chunk > c.tiles ? c.tiles : in_chunk);
    const int at = t.g[j].tile_begin + in_chunk;
    plan_b[x + 1] = at < plan_b[x] ? plan_b[x] : at;
  }
  auto price = [&](const int* begin) {
    double worst = 0.0;
    int j = 0;
    for (int x = 0; x < kXcds; ++x) {
      const int lo = begin[x], hi = begin[x + 1];
      if (hi <= lo) continue;
      double cost = 0.0;
      while (j < n && t.g[j].tile_begin + chunks[order[j]].tiles <= lo) ++j;
      for (int k = j; k < n && t.g[k].tile_begin < hi; ++k) {
        const Chunk& c = chunks[order[k]];
        const int from = t.g[k].tile_begin > lo ? t.g[k].tile_begin : lo;
        const int to = t.g[k].tile_begin + c.tiles < hi ? t.g[k].tile_begin + c.tiles : hi;
        cost += (double)c.cost / c.tiles * (to - from);
      }
      const int passes = (hi - lo + cus_per_xcd - 1) / cus_per_xcd;
      const double time = cost / (hi - lo) * passes;
      if (time > worst) worst = time;
    }
    return worst;
  };
  const bool even_cut = price(plan_b) < 0.9 * price(plan_a);
  for (int x = 0; x <= kXcds; ++x) t.xcd_begin[x] = even_cut ? plan_b[x] : plan_a[x];
  int longest = 0;
  for (int i = 0; i < kXcds; ++i)
    if (t.xcd_begin[i + 1] - t.xcd_begin[i] > longest) longest = t.xcd_begin[i + 1] - t.xcd_begin[i];
  grouped_tiled_kernel<256, 256><<<longest * kXcds, 256, 0, s>>>(t);
  return hipGetLastError();
}

// Whether every operand row of the problem can be fetched by the 16-byte DMA path.
static bool device_groups_aligned(const DeviceGroups& p) {
  return p.K % 16 == 0 && (int64_t)256 * p.K < (int64_t(1) << 32) && p.N < (1 << 26) &&
         reinterpret_cast<uintptr_t>(p.xq) % 16 == 0 && reinterpret_cast<uintptr_t>(p.wq) % 16 == 0;
}

hipError_t launch_device_groups(const DeviceGroups& in, int layout, hipStream_t s) {
  DeviceGroups p = in;
  p.unaligned = device_groups_aligned(p) ? 0 : 1;
  switch (layout) {
    case kGroupsSizesM: return launch_device_layout<kGroupsSizesM, 0>(p, s);
    case kGroupsOffsetsM: return launch_device_layout<kGroupsOffsetsM, 0>(p, s);
    case kGroupsOffsetsN:
    case kGroupsOffsetsK:
    case kGroupsPrepadM: return launch_device_groups_layouts(p, layout, s);
    case kGroupsUniform: return launch_device_groups_uniform(p, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace mslk_amd
