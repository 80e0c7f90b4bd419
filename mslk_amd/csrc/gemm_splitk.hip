// Dense f8f8bf16_rowwise on shapes with few output tiles and a long K: the K range is cut into slices, every (tile, slice)
// pair is a workgroup that writes raw fp32 sums into a workspace, and a second launch adds the slices, applies the row
// and column scales (and bias) and converts.  The launch boundary is what makes the sums of one launch visible to the
// next: no fences, no atomics.  The reference's CK instances for such shapes carry a K-batch count the same way
// (csrc/gemm/ck/fp8_rowwise/kernels/fp8_rowwise_common.h:168-204 passes it to the device op).
#include "gemm_tile.h"
#include "kernels.h"

namespace mslk_amd {
namespace {

constexpr int kXcds = 8;
constexpr int kGroupM = 4;

// One workgroup per (tile, slice).  The slices of a tile column sit side by side in the tile list (virtual column
// s * tiles_n + tn), and the list is dealt to the XCDs in contiguous runs of panels of up to kGroupM row tiles, so the
// row tiles that read one slice of one weight panel share an L2.
template <typename TS, bool PS>
__global__ __launch_bounds__(TS::NTHREADS) void splitk_partial_kernel(GemmProblem p, float* __restrict__ part, int tiles_m,
                                                                      int tiles_n, int slices) {
  constexpr int BM = TS::kBM, BN = TS::kBN;
  __shared__ __attribute__((aligned(1024))) char lds[TS::LDS_BYTES];
  const int cols = tiles_n * slices, ntiles = tiles_m * cols;
  const int per_xcd = (ntiles + kXcds - 1) / kXcds;
  const int t = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  if (t >= ntiles || (int)(blockIdx.x / kXcds) >= per_xcd) return;
  const int panel = kGroupM * cols, first_m = (t / panel) * kGroupM;
  const int rows = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  const int tm = first_m + (t % panel) % rows, vcol = (t % panel) / rows;
  const int sl = vcol / tiles_n, tn = vcol % tiles_n;
  // slice sl takes K steps [KT * sl / slices, KT * (sl + 1) / slices); the last one also takes the K tail
  const int KT = p.K / kBK;
  const int step0 = (int)((int64_t)KT * sl / slices), step1 = (int)((int64_t)KT * (sl + 1) / slices);
  const int k0 = step0 * kBK;
  const int klen = (sl == slices - 1 ? p.K : step1 * kBK) - k0;
  const int m0 = tm * BM, n0 = tn * BN;
  GemmTile<TS, 0, PS> tile;
  tile.out_f16 = 0;
  // pre-shuffled weights: a group of 16 rows is contiguous, K step by K step, so byte k0 of its rows lies 16 * k0 bytes in
  tile.run_partial(lds, p.xq + (int64_t)m0 * p.K + k0, p.wq + (int64_t)n0 * p.K + (PS ? (int64_t)k0 * 16 : (int64_t)k0),
                   part + ((int64_t)sl * p.M + m0) * p.N + n0, p.M - m0, p.N - n0, p.N, klen, (uint32_t)p.K);
}

// y[m][n] = convert((sum over slices of part[s][m][n]) * w_scale[n] * x_scale[m] + bias[n]): four columns per lane.
template <int BIAS, bool F16>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, GemmProblem p, int slices) {
  const int64_t quads_per_row = ((int64_t)p.N + 3) / 4;
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (q >= quads_per_row * p.M) return;
  const int m = (int)(q / quads_per_row), n = (int)(q % quads_per_row) * 4;
  const int64_t plane = (int64_t)p.M * p.N, at = (int64_t)m * p.N + n;
  const bool vec = (p.N & 3) == 0;
  float sum[4] = {0.f, 0.f, 0.f, 0.f};
  for (int sl = 0; sl < slices; ++sl) {
    const float* src = part + sl * plane + at;
    if (vec) {
      const float4 v = *reinterpret_cast<const float4*>(src);
      sum[0] += v.x; sum[1] += v.y; sum[2] += v.z; sum[3] += v.w;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < p.N) sum[r] += src[r];
    }
  }
  const float xsv = p.xs[m];
  uint16_t out[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (n + r >= p.N) { out[r] = 0; continue; }
    float v = (sum[r] * p.ws[n + r]) * xsv;   // w_scale first, then x_scale: the order of the tile kernels' epilogue
    if constexpr (BIAS == 1) v += static_cast<const float*>(p.bias)[n + r];
    if constexpr (BIAS == 2) v += bf16_bits_to_f32(static_cast<const uint16_t*>(p.bias)[n + r]);
    out[r] = (uint16_t)(pack_out_x2<F16>(v, 0.f) & 0xFFFFu);
  }
  uint16_t* dst = p.y + at;
  if (vec && (reinterpret_cast<uintptr_t>(p.y) & 7) == 0) {
    uint2 pk;
    pk.x = (uint32_t)out[0] | ((uint32_t)out[1] << 16);
    pk.y = (uint32_t)out[2] | ((uint32_t)out[3] << 16);
    *reinterpret_cast<uint2*>(dst) = pk;
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (n + r < p.N) dst[r] = out[r];
  }
}

template <typename TS>
hipError_t launch_partial(const GemmProblem& p, float* part, int slices, hipStream_t s) {
  const int tiles_m = (p.M + TS::kBM - 1) / TS::kBM, tiles_n = (p.N + TS::kBN - 1) / TS::kBN;
  const int grid = (tiles_m * tiles_n * slices + kXcds - 1) / kXcds * kXcds;
  if (p.w_preshuffled) splitk_partial_kernel<TS, true><<<grid, TS::NTHREADS, 0, s>>>(p, part, tiles_m, tiles_n, slices);
  else splitk_partial_kernel<TS, false><<<grid, TS::NTHREADS, 0, s>>>(p, part, tiles_m, tiles_n, slices);
  return hipGetLastError();
}

template <int BIAS>
hipError_t launch_reduce(const GemmProblem& p, const float* part, int slices, hipStream_t s) {
  const int64_t quads = (((int64_t)p.N + 3) / 4) * p.M;
  const unsigned grid = (unsigned)((quads + 255) / 256);
  if (p.out_f16) splitk_reduce_kernel<BIAS, true><<<grid, 256, 0, s>>>(part, p, slices);
  else splitk_reduce_kernel<BIAS, false><<<grid, 256, 0, s>>>(part, p, slices);
  return hipGetLastError();
}

}  // namespace

// The plan for a shape: number of K slices on 64 x 64 tiles; 1 means "do not split".  Measured on M = 16 ... 512,
// N = 512 ... 8192, K = 4096 / 8192 / 14336 against the unsplit dispatch: the two launches cost about 10 us, so a split
// pays only where the unsplit launch is a long K loop on few CUs -- more than 64 rows (below that the weight-streaming
// kernel and the short tiles already cover the CUs; 33 ... 64 rows gain only from K = 12288 on: M = 64, N = 4096, K = 14336
// 22.4 -> 19.1 us, but K = 8192 10.2 -> 12.7), at most half as many 64 x 64 tiles as CUs, K from 8192 on (6144
// when the tiles cover at most a quarter of the CUs); then as many slices as fill the CUs once, at most eight, each at
// least eight K steps long.  M = 128, N = 512, K = 14336: 37.8 -> 12.4 us; M = 96, N = 2048, K = 8192: 15.8 -> 11.9;
// M = 128, N = 4096, K = 14336: 34.2 -> 24.8; 128 x 128 tiles in slices were slower than these on every shape.
SplitKPlan splitk_plan(int64_t M, int64_t N, int64_t K, int cus) {
  SplitKPlan plan{64, 1};
  if (M <= 32 || (M <= 64 && K < 12288) || N < 64 || K < 6144 || K % 16 != 0) return plan;
  const int64_t steps = K / kBK;
  const int64_t tiles = ((M + 63) / 64) * ((N + 63) / 64);
  if (tiles > cus / 2 || (K < 8192 && tiles > cus / 4)) return plan;   // (two slices on up to 3/4 of the CUs at K >= 12288: 3 - 17 % slower)
  int64_t slices = cus / tiles;
  if (slices > steps / 8) slices = steps / 8;
  if (slices > 8) slices = 8;
  if (slices >= 2) plan.slices = (int)slices;
  return plan;
}

hipError_t launch_splitk(const GemmProblem& p, const SplitKPlan& plan, float* part, hipStream_t s) {
  if (dispatch_probe_record("splitk_partial<64,64,waves=4x1,ring=5>%s slices=%d + splitk_reduce", p.w_preshuffled ? " preshuffled" : "", plan.slices))
    return hipSuccess;
  const hipError_t e = launch_partial<TileShape<64, 64, 4, 1, 5>>(p, part, plan.slices, s);
  if (e != hipSuccess) return e;
  switch (p.bias_dtype) {
    case 0: return launch_reduce<0>(p, part, plan.slices, s);
    case 1: return launch_reduce<1>(p, part, plan.slices, s);
    default: return launch_reduce<2>(p, part, plan.slices, s);
  }
}

}  // namespace mslk_amd
