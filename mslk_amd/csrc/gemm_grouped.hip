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

#include "gemm_tile.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

constexpr int kXcds = 8;
constexpr int kGroupM = 4;

// Tile order inside one group: panels of kGroupM row tiles, column-major inside a panel.  Returns the number of row tiles
// of the tile's panel: the tiles that read one weight block at about the same time.
MSLK_AMD_DEVINL int local_tile(int t, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int panel = kGroupM * tiles_n;
  const int first_m = (t / panel) * kGroupM;
  const int rows = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  tm = first_m + (t % panel) % rows;
  tn = (t % panel) / rows;
  return rows;
}

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

// Groups whose extents live in device memory (or are uniform).  `layout` says which dimension varies
// per group and how it is encoded; the fixed dimensions come from p.M / p.N / p.K, where the varying
// one holds the total over all groups.
//   kGroupsSizesM    int64 sizes of the row blocks of XQ [sum M, K]; WQ [G, N, K]; Y [sum M, N]
//   kGroupsOffsetsM  int32 cumulative ends of the same row blocks
//   kGroupsOffsetsN  XQ [G, M, K]; int32 cumulative ends of row blocks of WQ [sum N, K]; Y [M, sum N]
//   kGroupsOffsetsK  XQ [M, sum K], WQ [N, sum K]; int32 cumulative ends of K slices; Y [G, M, N]
//   kGroupsUniform   XQ [G, M, K], WQ [G, N, K], Y [G, M, N]
//   kGroupsPrepadM   as uniform, but only the first layout[g] (int64) rows of group g are computed
// Scales follow the operand they belong to ([sum M] or [G, M]; [sum N] or [G, N]).
struct GroupSpan {
  int gi;        // group
  int64_t o0;    // first index of the group along the varying dimension
  int len;       // extent of the group along the varying dimension
  int t;         // tile index inside the group
};

MSLK_AMD_DEVINL int64_t uniform64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)v), hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

template <int LAYOUT, int BM, int BN>
MSLK_AMD_DEVINL bool find_group(const DeviceGroups& p, int t, GroupSpan& sp) {
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  if constexpr (LAYOUT == kGroupsUniform || LAYOUT == kGroupsOffsetsK || LAYOUT == kGroupsPrepadM) {
    const int per = tiles_m * tiles_n;
    sp.gi = t / per;
    sp.t = t - sp.gi * per;
    if (sp.gi >= p.G) return false;
    if constexpr (LAYOUT == kGroupsUniform) {
      sp.o0 = 0;
      sp.len = 0;
      return true;
    } else if constexpr (LAYOUT == kGroupsPrepadM) {
      const int64_t live = static_cast<const int64_t*>(p.layout)[sp.gi];
      sp.o0 = 0;
      sp.len = (int)(live < 0 ? 0 : (live > p.M ? p.M : live));
      return true;
    } else {
      const int32_t* off = static_cast<const int32_t*>(p.layout);
      const int64_t b = sp.gi ? off[sp.gi - 1] : 0, e = off[sp.gi];
      sp.o0 = b;
      sp.len = (int)(e - b);
      return b >= 0 && e >= b && e <= p.K;
    }
  } else {
    // The G extents are read 64 at a time, one per lane, and turned into tile ranges by a wave-level
    // prefix sum, so the lookup costs one memory round trip instead of G dependent ones.  The total tile count is formed
    // first: XCD x (workgroup id mod 8) then takes a contiguous slice of the tile list, so that the row tiles of a group
    // that share a weight panel run on one XCD and find it in its L2 (without the slices the device-extent layouts
    // fetched 1.6 times what the host-extent kernel fetches for the same 16 experts).
    const int fixed_tiles = LAYOUT == kGroupsOffsetsN ? tiles_m : tiles_n;
    const int blk = LAYOUT == kGroupsOffsetsN ? BN : BM;
    const int64_t total = LAYOUT == kGroupsOffsetsN ? p.N : p.M;
    const int lane = threadIdx.x & 63;
    // Every quantity fits 32 bits (the host checks the dimensions and the grid): sizes beyond the tensor mark the group bad.
    struct Chunk { int start, len, tiles, incl; bool bad; };
    // `seen_bad` carries "an earlier group was inconsistent" from chunk to chunk: such a group and every group after it
    // own no tiles, so the tile count, the XCD slices and the lookup all stop at the first bad group and every tile
    // of the groups in front of it gets a workgroup (the grid is sized for consistent extents).
    auto load_chunk = [&](int base, int& carry_len, bool& seen_bad) {
      Chunk c;
      const int gi = base + lane;
      const bool in = gi < p.G;
      c.start = 0;
      c.len = 0;
      c.bad = false;
      if constexpr (LAYOUT == kGroupsSizesM) {
        int64_t len64 = 0;
        if (in) len64 = static_cast<const int64_t*>(p.layout)[gi];
        c.bad = len64 < 0 || len64 > total;
        c.len = c.bad ? 0 : (int)len64;
        // running sum that saturates at 2^31 - 1 instead of wrapping (the terms are below 2^31, so one unsigned addition
        // cannot wrap): sizes that add up to more than the tensor holds always end beyond it and mark their group bad
        auto sat_add = [](int x, int y) {
          const uint32_t u = (uint32_t)x + (uint32_t)y;
          return (int)(u > 0x7FFFFFFFu ? 0x7FFFFFFFu : u);
        };
        int incl_len = c.len;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int v = __shfl_up(incl_len, d, 64);
          if (lane >= d) incl_len = sat_add(incl_len, v);
        }
        const int end = sat_add(carry_len, incl_len);
        c.start = end - c.len;
        carry_len = sat_add(carry_len, __shfl(incl_len, 63, 64));
        c.bad = c.bad || (in && (end > total || end == 0x7FFFFFFF));
      } else {
        const int32_t* off = static_cast<const int32_t*>(p.layout);
        if (in) {
          c.start = gi ? off[gi - 1] : 0;
          const int64_t len64 = (int64_t)off[gi] - c.start;
          c.bad = len64 < 0 || c.start < 0 || (int64_t)c.start + len64 > total;
          c.len = c.bad ? 0 : (int)len64;
        }
      }
      const unsigned long long bad_lanes = __ballot(c.bad);
      const bool after_bad = seen_bad || (bad_lanes != 0 && lane >= __ffsll((long long)bad_lanes) - 1);
      seen_bad = seen_bad || bad_lanes != 0;
      c.tiles = (in && !after_bad) ? ((c.len + blk - 1) / blk) * fixed_tiles : 0;
      c.incl = c.tiles;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(c.incl, d, 64);
        if (lane >= d) c.incl += v;
      }
      return c;
    };
    int64_t total_tiles = 0;
    int carry_len = 0;
    bool seen_bad = false;
    Chunk first = load_chunk(0, carry_len, seen_bad);
    const bool first_bad = seen_bad;
    total_tiles = __shfl(first.incl, 63, 64);
    for (int base = 64; base < p.G && !seen_bad; base += 64) total_tiles += __shfl(load_chunk(base, carry_len, seen_bad).incl, 63, 64);
    const int64_t per_xcd = (total_tiles + kXcds - 1) / kXcds;
    const int64_t slot = t / kXcds;                       // `t` arrives as the workgroup id
    const int64_t tile = (int64_t)(t % kXcds) * per_xcd + slot;
    if (slot >= per_xcd || tile >= total_tiles) return false;
    int64_t carry_tiles = 0;
    carry_len = 0;
    seen_bad = first_bad;
    for (int base = 0; base < p.G; base += 64) {
      Chunk c = first;
      if (base == 0) carry_len = __shfl(first.start + first.len, 63, 64);   // sizes: rows of the first 64 groups
      else c = load_chunk(base, carry_len, seen_bad);
      const int64_t excl = carry_tiles + c.incl - c.tiles;
      const bool hit = c.tiles > 0 && tile >= excl && tile < excl + c.tiles;
      const unsigned long long hit_mask = __ballot(hit), bad_mask = __ballot(c.bad);
      if (hit_mask != 0) {
        const int src = __ffsll((long long)hit_mask) - 1;
        if (bad_mask & ((1ull << src) - 1ull)) return false;   // a group before this one is inconsistent: touch nothing
        // the results are the same in every lane: say so, so that the tile's addresses live in scalar registers
        sp.gi = base + src;
        sp.o0 = __builtin_amdgcn_readfirstlane(__shfl(c.start, src, 64));
        sp.len = __builtin_amdgcn_readfirstlane(__shfl(c.len, src, 64));
        sp.t = (int)(tile - uniform64(__shfl(excl, src, 64)));
        return true;
      }
      if (bad_mask != 0) return false;
      carry_tiles += __shfl(c.incl, 63, 64);
    }
    return false;
  }
}

// Scalar tile for operands the DMA path cannot fetch (row starts or K extents that are not multiples
// of 16 bytes): one lane per output element, sequential K.
template <int BM, int BN, int BIAS>
MSLK_AMD_DEVINL void slow_tile(const uint8_t* a, const uint8_t* b, const float* xs, const float* ws,
                               const void* bias, uint16_t* y, int m_rem, int n_rem, int ldc, int K, int64_t ld) {
  const int mt = m_rem < BM ? m_rem : BM, nt = n_rem < BN ? n_rem : BN;
  for (int idx = threadIdx.x; idx < mt * nt; idx += 256) {
    const int m = idx / nt, n = idx - m * nt;
    const uint8_t* ar = a + m * ld;
    const uint8_t* br = b + n * ld;
    float acc = 0.f;
    for (int k = 0; k < K; ++k)
      acc += __builtin_amdgcn_cvt_f32_fp8((int)ar[k], 0) * __builtin_amdgcn_cvt_f32_fp8((int)br[k], 0);
    float v = (acc * ws[n]) * xs[m];
    if constexpr (BIAS == 1) v += static_cast<const float*>(bias)[n];
    if constexpr (BIAS == 2) v += bf16_bits_to_f32(static_cast<const uint16_t*>(bias)[n]);
    y[(int64_t)m * ldc + n] = (uint16_t)f32_to_bf16_bits(v);
  }
}

template <int LAYOUT, int BM, int BN, int BIAS>
__global__ __launch_bounds__(256) void grouped_device_kernel(DeviceGroups p) {
  using TS = TileShape<BM, BN>;
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  int t = blockIdx.x;
  if constexpr (LAYOUT == kGroupsUniform || LAYOUT == kGroupsOffsetsK || LAYOUT == kGroupsPrepadM) {
    // The tile count is known on the host: XCD x works on a contiguous slice of the tile list.
    const int total = p.G * ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    const int per_xcd = (total + kXcds - 1) / kXcds;
    t = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (t >= total) return;
  }
  GroupSpan sp;
  if (!find_group<LAYOUT, BM, BN>(p, t, sp)) return;
  const int64_t g = sp.gi, M = p.M, N = p.N, K = p.K;
  const int Mg = (LAYOUT == kGroupsSizesM || LAYOUT == kGroupsOffsetsM || LAYOUT == kGroupsPrepadM) ? sp.len : p.M;
  const int Ng = LAYOUT == kGroupsOffsetsN ? sp.len : p.N;
  const int Kg = LAYOUT == kGroupsOffsetsK ? sp.len : p.K;
  int tm, tn;
  local_tile(sp.t, ((LAYOUT == kGroupsPrepadM ? p.M : Mg) + BM - 1) / BM, (Ng + BN - 1) / BN, tm, tn);
  const int64_t m0 = tm * BM, n0 = tn * BN;
  if constexpr (LAYOUT == kGroupsPrepadM) {
    if (m0 >= sp.len) return;   // tile of padding rows only
  }
  const uint8_t *a, *b;
  const float *xs, *ws;
  uint16_t* y;
  if constexpr (LAYOUT == kGroupsSizesM || LAYOUT == kGroupsOffsetsM) {
    a = p.xq + (sp.o0 + m0) * K;      b = p.wq + (g * N + n0) * K;
    xs = p.xs + sp.o0 + m0;           ws = p.ws + g * N + n0;
    y = p.y + (sp.o0 + m0) * N + n0;
  } else if constexpr (LAYOUT == kGroupsOffsetsN) {
    a = p.xq + (g * M + m0) * K;      b = p.wq + (sp.o0 + n0) * K;
    xs = p.xs + g * M + m0;           ws = p.ws + sp.o0 + n0;
    y = p.y + m0 * N + sp.o0 + n0;
  } else if constexpr (LAYOUT == kGroupsOffsetsK) {
    a = p.xq + m0 * K + sp.o0;        b = p.wq + n0 * K + sp.o0;
    xs = p.xs + g * M + m0;           ws = p.ws + g * N + n0;
    y = p.y + (g * M + m0) * N + n0;
  } else {
    a = p.xq + (g * M + m0) * K;      b = p.wq + (g * N + n0) * K;
    xs = p.xs + g * M + m0;           ws = p.ws + g * N + n0;
    y = p.y + (g * M + m0) * N + n0;
  }
  const int m_rem = Mg - (int)m0, n_rem = Ng - (int)n0;
  const void* bias = nullptr;
  if constexpr (BIAS == 1) bias = static_cast<const float*>(p.bias) + g * N + n0;
  if constexpr (BIAS == 2) bias = static_cast<const uint16_t*>(p.bias) + g * N + n0;
  bool slow = p.unaligned != 0;
  if constexpr (LAYOUT == kGroupsOffsetsK) slow = slow || (sp.o0 & 15) != 0 || (Kg & 15) != 0;
  if (slow) {   // Kg == 0 needs no special case on either path: the sum is empty
    slow_tile<BM, BN, BIAS>(a, b, xs, ws, bias, y, m_rem, n_rem, p.N, Kg, K);
    return;
  }
  // A weight block that a single row tile reads at a time (the tile is the only one of its panel with rows to compute:
  // a group of at most BM rows, or the last panel of a group of 4 k + 1 row tiles) is fetched with non-temporal loads
  // (cfg4 307 -> 298 us, four big experts + eight of 256 rows 276 -> 253 us; with panels of two row tiles included:
  // cfg4 304 -> 315 us, a uniform batch of 512-row groups 268 -> 263 us -- not taken).
  const int live_tiles = (Mg + BM - 1) / BM, panel_first = tm / kGroupM * kGroupM;
  if (live_tiles - panel_first == 1) {
    GemmTile<TS, BIAS, false, true, TS::LA / 2, false, true> tile;
    tile.run(lds, a, b, xs, ws, bias, y, m_rem, n_rem, p.N, Kg, (uint32_t)p.K);
  } else {
    GemmTile<TS, BIAS, false, true> tile;
    tile.run(lds, a, b, xs, ws, bias, y, m_rem, n_rem, p.N, Kg, (uint32_t)p.K);
  }
}

template <int LAYOUT, int BM, int BN, int BIAS>
hipError_t launch_device_shape(const DeviceGroups& p, hipStream_t s) {
  const int64_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  int64_t grid;
  if (LAYOUT == kGroupsUniform || LAYOUT == kGroupsOffsetsK || LAYOUT == kGroupsPrepadM) {
    grid = (p.G * tiles_m * tiles_n + kXcds - 1) / kXcds * kXcds;
  } else if (LAYOUT == kGroupsOffsetsN) {
    grid = (tiles_m * (tiles_n + p.G) + kXcds - 1) / kXcds * kXcds;   // every group may end in a partial tile; 8 slices
  } else {
    grid = ((tiles_m + p.G) * tiles_n + kXcds - 1) / kXcds * kXcds;
  }
  if (grid <= 0) return hipSuccess;
  if (grid > 2147483647) return hipErrorInvalidValue;
  grouped_device_kernel<LAYOUT, BM, BN, BIAS><<<(unsigned)grid, 256, 0, s>>>(p);
  return hipGetLastError();
}

template <int LAYOUT, int BIAS>
hipError_t launch_device_layout(const DeviceGroups& p, hipStream_t s) {
  // Tile shape from the average group: 256 x 256 once such tiles give every CU work.
  const int64_t G = p.G > 0 ? p.G : 1;
  int64_t Mg = p.M, Ng = p.N;
  if (LAYOUT == kGroupsSizesM || LAYOUT == kGroupsOffsetsM) Mg = (p.M + G - 1) / G;
  if (LAYOUT == kGroupsOffsetsN) Ng = (p.N + G - 1) / G;
  const int64_t big = G * ((Mg + 255) / 256) * ((Ng + 255) / 256);
  const int64_t pad = ((Mg + 255) / 256 * 256) * ((Ng + 255) / 256 * 256);
  const bool use_big = big >= 192 && pad * 4 <= Mg * Ng * 5;   // at most 25 % padding
  if (use_big) return launch_device_shape<LAYOUT, 256, 256, BIAS>(p, s);
  return launch_device_shape<LAYOUT, 128, 128, BIAS>(p, s);
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
    case kGroupsOffsetsN: return launch_device_layout<kGroupsOffsetsN, 0>(p, s);
    case kGroupsOffsetsK: return launch_device_layout<kGroupsOffsetsK, 0>(p, s);
    case kGroupsPrepadM: return launch_device_layout<kGroupsPrepadM, 0>(p, s);
    case kGroupsUniform:
      if (p.bias_dtype == 1) return launch_device_layout<kGroupsUniform, 1>(p, s);
      if (p.bias_dtype == 2) return launch_device_layout<kGroupsUniform, 2>(p, s);
      return launch_device_layout<kGroupsUniform, 0>(p, s);
  }
  return hipErrorInvalidValue;
}

}  // namespace mslk_amd
