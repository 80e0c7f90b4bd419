// Kernels of the grouped GEMM whose group extents live in device memory (or are uniform), with the tile order they share
// with the TensorList kernel.  Included by the translation units that instantiate the layouts (gemm_grouped.hip: row blocks
// given by sizes or offsets, and the TensorList form; gemm_grouped_layouts.hip: offsets over N and K, padded rows;
// gemm_grouped_uniform.hip: the uniform batch with its bias variants), so that they compile side by side.
#pragma once
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
}  // namespace mslk_amd
