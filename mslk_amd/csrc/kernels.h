// Internal launcher declarations shared between the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mslk_amd {

// zero_start != nullptr: jagged rows (blocks of rows_per_group rows, the first zero_start[block] are live).
hipError_t launch_quantize_fp8_row(const void* x, int dtype, int64_t rows, int64_t K, int64_t in_stride,
                                   void* xq, int64_t K_out, float* scale, const float* scale_ub,
                                   const void* zero_start, int zero_start_is_i32, int64_t rows_per_group,
                                   int triton_arithmetic, float triton_eps, hipStream_t s);
hipError_t launch_dequantize_fp8_row(const void* xq, const float* scale, int64_t rows, int64_t K, void* out,
                                     hipStream_t s);
// WQ [G, N, K] row-major -> the blocked layout the *_preshuffle GEMMs read (N % 16 == 0, K % 64 == 0).
hipError_t launch_preshuffle_b(const void* src, void* dst, int64_t G, int64_t N, int64_t K, hipStream_t s);
hipError_t launch_cast_e4m3fn(const float* in, int64_t n, void* out, hipStream_t s);
// Ceiling probes (ceilings.hip): a pure read of `bytes` from src (mode 0: 16-byte loads into registers, bytes % 16 == 0;
// mode 1: global -> LDS DMA loads, mode 2: the same non-temporal, bytes % 1024 == 0), and a register-only MFMA loop
// (form 0: 16x16x128, form 1: 32x32x64) of `iters` 128 x 128 x 128 wave tiles per wave on the 128 KiB of operand bytes
// at `operands`.
hipError_t launch_debug_stream_read(const void* src, int64_t bytes, int mode, int workgroups, void* sink, hipStream_t s);
hipError_t launch_debug_mfma_loop(const void* operands, int form, int iters, int workgroups, void* sink, hipStream_t s);
// The operand streams of a 128 x 64 tile K loop alone (which: 1 activations, 2 weights, 3 both); x holds tiles_m * 128 rows
// of K bytes, w tiles_n * 64 rows; K a multiple of 128.
hipError_t launch_debug_tile_streams(const void* x, const void* w, int K, int tiles_m, int tiles_n, int which, hipStream_t s);

// Fused producers of quantized activations (fused_quant.hip).
enum FusedQuantOp : int { kFusedSiluMul = 0, kFusedGatherScale = 1 };
struct FusedQuantArgs {
  const void* x0;            // silu: gate input [rows, D]; gather: token matrix x [T, D]
  const void* x1;            // silu: up input [rows, D]
  int64_t stride0, stride1;  // row strides in elements
  int dtype;                 // element type of x0 / x1: 0 bf16, 1 fp16
  uint8_t* out;              // [rows, D] e4m3fn, contiguous
  float* out_scale;          // [rows]
  int64_t rows;
  int D;
  const float* scale_ub;     // optional
  const void* valid_count;   // optional device scalar: rows at or beyond it are left untouched
  int valid_is_i64;
  // gather only
  const void* token_idx;     // [rows]
  int token_is_i64;
  const void* expert_idx;    // [rows]
  int expert_is_i64;
  const void* scores;        // [T, E] with strides (stride_t, stride_e) in elements
  int score_dtype;           // 0 bf16, 1 fp16, 2 fp32
  int64_t stride_t, stride_e;
  int64_t T, E;
};
hipError_t launch_fused_quant(const FusedQuantArgs& p, int op, hipStream_t s);

// One GEMM problem: Y[M,N] = bf16(XQ[M,K] . WQ[N,K]^T * xs[:,None] * ws[None,:] + bias[None,:]).
struct GemmProblem {
  const uint8_t* xq;
  const uint8_t* wq;
  const float* xs;
  const float* ws;
  const void* bias;   // nullptr, fp32 or bf16 according to bias_dtype
  uint16_t* y;
  int M, N, K;
  int bias_dtype;     // 0 none, 1 fp32, 2 bf16
  int out_f16;        // 0: Y is bf16, 1: Y is fp16
  int w_preshuffled;  // 1: WQ is in the blocked layout [N/16][K/64][4][16][16 B] (N % 16 == 0, K % 64 == 0)
};
// The 256 x 256 tile kernel with four counter readings per wave (mslk_amd_debug_gemm_phases): M, N multiples of 256,
// K a multiple of 128 and at least 256, no bias, bf16 output.
hipError_t launch_debug_gemm_phases(const GemmProblem& p, uint64_t* stamps, hipStream_t s);

// Dry run of the shape dispatch (mslk_amd_debug_dispatch_name): between dispatch_probe_begin() and dispatch_probe_end()
// on the calling thread every GEMM launcher records the kernel it would launch (name, tile shape, grid) and launches
// nothing -- the recorded choice is made by the very code that makes the real one.
void dispatch_probe_begin();
const char* dispatch_probe_end();                       // "a + b" when the dispatch would issue several launches
bool dispatch_probe_record(const char* fmt, ...);       // false when no dry run is active on this thread
// Compute units of the current device, rounded down to a multiple of the XCD count (256 on a whole MI355X, also
// when no device can be queried); the tile-shape thresholds and the persistent grid both use it.
int device_compute_units();

// Shape classes; each returns hipErrorInvalidValue when the shape is outside what it supports.
bool dense_tiled_supports(const GemmProblem& p);
hipError_t launch_dense_tiled(const GemmProblem& p, hipStream_t s);
// The tile shapes below 128 x 256 on row-major weights (gemm_dense_small.hip), launched by name.
enum DenseSmallTile : int {
  kTile32x32, kTile64x32, kTile64x64, kTile128x32, kTile128x64, kTile96x128,
  kTile128x128Ring,   // five ring buffers, one workgroup per CU
  kTile128x128,       // two-plus-three buffers, two workgroups per CU
  kTile192x128,
};
hipError_t launch_dense_small_tile(int shape, const GemmProblem& p, hipStream_t s);
// Its branch for pre-shuffled weights (a translation unit of its own); cus: device_compute_units().
hipError_t launch_dense_tiled_preshuffled(const GemmProblem& p, int cus, hipStream_t s);
// K-split form for shapes with few output tiles and a long K (gemm_splitk.hip): `slices` workgroups per tile of edge
// `tile` write fp32 sums to a workspace of slices * M * N floats, a second launch reduces, scales and converts.
struct SplitKPlan {
  int tile;     // 64
  int slices;   // 1: the shape is not split
};
SplitKPlan splitk_plan(int64_t M, int64_t N, int64_t K, int cus);
hipError_t launch_splitk(const GemmProblem& p, const SplitKPlan& plan, float* part, hipStream_t s);
bool skinny_supports(const GemmProblem& p);
// Row-major weights at least this wide take the short LDS tiles instead of the weight-streaming kernel for 8 < M <= 64
// (measured crossover: streaming wins at N = 4096, tiles from N = 5120 on).
constexpr int kShortTileMinN = 5120;
hipError_t launch_skinny(const GemmProblem& p, hipStream_t s);
// Decode with the activation quantizer fused in: `x` holds p.M <= 4 rows of p.K bf16 (row stride x_stride elements);
// p.xq / p.xs are not read.  xq_out [M, K] / xs_out [M] (optional) receive the codes and scales the kernel multiplied with.
bool skinny_fused_quant_supports(const GemmProblem& p, const void* x, int64_t x_stride);
hipError_t launch_skinny_fused_quant(const GemmProblem& p, const void* x, int64_t x_stride, void* xq_out, float* xs_out,
                                     hipStream_t s);
hipError_t launch_generic(const GemmProblem& p, hipStream_t s);   // any shape, slow
hipError_t launch_fill_zero_bf16(uint16_t* y, int64_t n, hipStream_t s);
// dst[r, 0:K] = src[r, 0:K], dst[r, K:Kp] = 0 for `rows` rows of bytes (Kp a multiple of 16, dst 16-byte aligned)
hipError_t launch_pad_rows(const uint8_t* src, uint8_t* dst, int64_t rows, int64_t K, int64_t Kp, hipStream_t s);

// Grouped problems.  Up to kMaxGroupsPerLaunch descriptors travel in the kernel argument block.
constexpr int kMaxGroupsPerLaunch = 64;
struct GroupDesc {
  const uint8_t* xq;
  const uint8_t* wq;
  const float* xs;
  const float* ws;
  uint16_t* y;
  int M, N, K;
  int tile_begin;     // first tile index of this group inside the launch
};
struct GroupTable {
  GroupDesc g[kMaxGroupsPerLaunch];
  int count;
  int total_tiles;
  int xcd_begin[9];   // filled by the launcher: XCD x works on tiles [xcd_begin[x], xcd_begin[x + 1])
};
// Takes one descriptor per group (tile_begin ascending); re-cuts them into row chunks dealt to the XCDs by estimated cost.
hipError_t launch_grouped_tiled(const GroupTable& t, hipStream_t s);

// Groups described in device memory (or uniform); see gemm_grouped.hip for the layouts.
enum GroupLayout : int {
  kGroupsSizesM = 0,
  kGroupsOffsetsM = 1,
  kGroupsOffsetsN = 2,
  kGroupsOffsetsK = 3,
  kGroupsUniform = 4,
  kGroupsPrepadM = 5,
};
struct DeviceGroups {
  const uint8_t* xq;
  const uint8_t* wq;
  const float* xs;
  const float* ws;
  const void* bias;     // [G, N], uniform layout only
  uint16_t* y;
  const void* layout;   // int64 sizes / live-row counts, int32 cumulative ends, or nullptr
  int G;
  int M, N, K;          // the varying dimension holds the total over all groups
  int bias_dtype;       // 0 none, 1 fp32, 2 bf16
  int unaligned;        // set by the launcher: operands need the scalar tile path
};
hipError_t launch_device_groups(const DeviceGroups& p, int layout, hipStream_t s);
// Its layouts outside gemm_grouped.hip (translation units of their own); p.unaligned already set.
hipError_t launch_device_groups_layouts(const DeviceGroups& p, int layout, hipStream_t s);
hipError_t launch_device_groups_uniform(const DeviceGroups& p, hipStream_t s);

}  // namespace mslk_amd
