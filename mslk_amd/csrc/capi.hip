// C ABI of the library (declared in include/mslk_amd.h): argument validation, shape-class
// dispatch, error reporting.  No allocation, no synchronisation, no host reads of device memory.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "../../include/mslk_amd.h"
#include "kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  return fail("%s: %s", what, hipGetErrorString(e));
}

constexpr int64_t kIntMax = 2147483647;

// Device memory for the padded operand copies (or the fp32 sums of a K split) of mslk_amd_f8f8bf16_rowwise_static_scratch: part of the code object, so
// every GPU the library runs on holds its own copy from module load until the process ends.  In host code the name
// below is only a handle for hipGetSymbolAddress; kernels and copies get the per-device address it returns.
constexpr size_t kScratchBytes = MSLK_AMD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device; looked up once per device, with that device current.
int scratch_of_current_device(void** out) {
  int dev = 0;
  if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (dev < 0 || dev >= kMaxDevices) return fail("static scratch: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    if (int rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
    if (ptr == nullptr) return fail("static scratch: hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace

using namespace mslk_amd;

extern "C" {

const char* mslk_amd_version(void) { return "mslk_amd 0.1 (gfx950)"; }
const char* mslk_amd_last_error(void) { return g_err; }

int mslk_amd_quantize_fp8_row(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t x_row_stride,
                              void* xq, int64_t K_out, float* scale, const float* scale_ub, void* stream) {
  if (x_dtype < 0 || x_dtype > 2) return fail("quantize_fp8_row: unsupported input dtype code %d", x_dtype);
  if (rows < 0 || K <= 0) return fail("quantize_fp8_row: rows must be >= 0 and K > 0 (got %lld, %lld)", (long long)rows, (long long)K);
  if (K_out < K) return fail("quantize_fp8_row: K_out (%lld) < K (%lld)", (long long)K_out, (long long)K);
  if (rows == 0) return 0;
  if (rows > kIntMax) return fail("quantize_fp8_row: rows (%lld) exceeds 2^31-1", (long long)rows);
  if (!x || !xq || !scale) return fail("quantize_fp8_row: null pointer");
  return check_hip(launch_quantize_fp8_row(x, x_dtype, rows, K, x_row_stride, xq, K_out, scale, scale_ub, nullptr, 0, 1,
                                           0, 0.f, (hipStream_t)stream),
                   "quantize_fp8_row launch");
}

int mslk_amd_quantize_fp8_row_jagged(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t x_row_stride,
                                     void* xq, int64_t K_out, float* scale, const float* scale_ub,
                                     const void* zero_start_index, int index_dtype, int64_t rows_per_group,
                                     void* stream) {
  if (x_dtype < 0 || x_dtype > 2) return fail("quantize_fp8_row_jagged: unsupported input dtype code %d", x_dtype);
  if (index_dtype != MSLK_AMD_INDEX_I64 && index_dtype != MSLK_AMD_INDEX_I32)
    return fail("quantize_fp8_row_jagged: unsupported index dtype code %d", index_dtype);
  if (rows < 0 || K <= 0) return fail("quantize_fp8_row_jagged: rows must be >= 0 and K > 0 (got %lld, %lld)", (long long)rows, (long long)K);
  if (K_out < K) return fail("quantize_fp8_row_jagged: K_out (%lld) < K (%lld)", (long long)K_out, (long long)K);
  if (rows_per_group <= 0 || rows % rows_per_group != 0)
    return fail("quantize_fp8_row_jagged: rows (%lld) must be a multiple of rows_per_group (%lld)", (long long)rows,
                (long long)rows_per_group);
  if (rows == 0) return 0;
  if (rows > kIntMax) return fail("quantize_fp8_row_jagged: rows (%lld) exceeds 2^31-1", (long long)rows);
  if (!x || !xq || !scale || !zero_start_index) return fail("quantize_fp8_row_jagged: null pointer");
  return check_hip(launch_quantize_fp8_row(x, x_dtype, rows, K, x_row_stride, xq, K_out, scale, scale_ub,
                                           zero_start_index, index_dtype == MSLK_AMD_INDEX_I32, rows_per_group,
                                           0, 0.f, (hipStream_t)stream),
                   "quantize_fp8_row_jagged launch");
}

int mslk_amd_quantize_fp8_row_triton_arithmetic(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t x_row_stride,
                                                void* xq, int64_t K_out, float* scale, const float* scale_ub, float eps,
                                                const void* zero_start_index, int index_dtype, int64_t rows_per_group,
                                                void* stream) {
  const char* op = "quantize_fp8_row_triton_arithmetic";
  if (x_dtype < 0 || x_dtype > 2) return fail("%s: unsupported input dtype code %d", op, x_dtype);
  if (rows < 0 || K <= 0) return fail("%s: rows must be >= 0 and K > 0 (got %lld, %lld)", op, (long long)rows, (long long)K);
  if (K_out < K) return fail("%s: K_out (%lld) < K (%lld)", op, (long long)K_out, (long long)K);
  if (!(eps > 0.f)) return fail("%s: eps must be positive", op);
  if (zero_start_index != nullptr) {
    if (index_dtype != MSLK_AMD_INDEX_I64 && index_dtype != MSLK_AMD_INDEX_I32) return fail("%s: unsupported index dtype code %d", op, index_dtype);
    if (rows_per_group <= 0 || rows % rows_per_group != 0)
      return fail("%s: rows (%lld) must be a multiple of rows_per_group (%lld)", op, (long long)rows, (long long)rows_per_group);
  }
  if (rows == 0) return 0;
  if (rows > kIntMax) return fail("%s: rows (%lld) exceeds 2^31-1", op, (long long)rows);
  if (!x || !xq || !scale) return fail("%s: null pointer", op);
  return check_hip(launch_quantize_fp8_row(x, x_dtype, rows, K, x_row_stride, xq, K_out, scale, scale_ub, zero_start_index,
                                           index_dtype == MSLK_AMD_INDEX_I32, rows_per_group, 1, eps, (hipStream_t)stream),
                   "quantize_fp8_row_triton_arithmetic launch");
}

int mslk_amd_dequantize_fp8_row(const void* xq, const float* scale, int64_t rows, int64_t K, void* out, void* stream) {
  if (rows < 0 || K < 0) return fail("dequantize_fp8_row: negative dimension");
  if (rows == 0 || K == 0) return 0;
  if (!xq || !scale || !out) return fail("dequantize_fp8_row: null pointer");
  return check_hip(launch_dequantize_fp8_row(xq, scale, rows, K, out, (hipStream_t)stream), "dequantize_fp8_row launch");
}

int mslk_amd_silu_mul_quant(const void* x0, const void* x1, int x_dtype, int64_t T, int64_t D, int64_t x0_row_stride,
                            int64_t x1_row_stride, void* out, float* out_scale, const float* scale_ub,
                            const void* valid_token_count, int count_dtype, void* stream) {
  if (x_dtype != MSLK_AMD_DTYPE_BF16 && x_dtype != MSLK_AMD_DTYPE_F16)
    return fail("silu_mul_quant: inputs must be bf16 or fp16 (dtype code %d)", x_dtype);
  if (count_dtype != MSLK_AMD_INDEX_I64 && count_dtype != MSLK_AMD_INDEX_I32)
    return fail("silu_mul_quant: unsupported valid_token_count dtype code %d", count_dtype);
  if (T < 0 || D < 0) return fail("silu_mul_quant: negative dimension");
  if (T > kIntMax || D > kIntMax) return fail("silu_mul_quant: dimension exceeds 2^31-1");
  if (T == 0 || D == 0) return 0;
  if (!x0 || !x1 || !out || !out_scale) return fail("silu_mul_quant: null pointer");
  if (x0_row_stride < D || x1_row_stride < D) return fail("silu_mul_quant: row stride smaller than D");
  FusedQuantArgs p{};
  p.x0 = x0; p.x1 = x1; p.stride0 = x0_row_stride; p.stride1 = x1_row_stride; p.dtype = x_dtype;
  p.out = (uint8_t*)out; p.out_scale = out_scale; p.rows = T; p.D = (int)D; p.scale_ub = scale_ub;
  p.valid_count = valid_token_count; p.valid_is_i64 = count_dtype == MSLK_AMD_INDEX_I64;
  return check_hip(launch_fused_quant(p, kFusedSiluMul, (hipStream_t)stream), "silu_mul_quant launch");
}

int mslk_amd_gather_scale_quant_dense_tokens(const void* x, int x_dtype, int64_t T, int64_t D,
                                             const void* token_indices, int token_dtype,
                                             const void* expert_indices, int expert_dtype, int64_t a,
                                             const void* scores, int score_dtype, int64_t E, int64_t score_stride_t,
                                             int64_t score_stride_e, void* out, float* out_scale,
                                             const float* scale_ub, const void* valid_token_count, int count_dtype,
                                             void* stream) {
  const char* op = "gather_scale_quant_dense_tokens";
  if (x_dtype != MSLK_AMD_DTYPE_BF16 && x_dtype != MSLK_AMD_DTYPE_F16) return fail("%s: x must be bf16 or fp16 (dtype code %d)", op, x_dtype);
  if (score_dtype < 0 || score_dtype > 2) return fail("%s: unsupported scores dtype code %d", op, score_dtype);
  if ((token_dtype | expert_dtype | count_dtype) & ~1) return fail("%s: index dtype codes must be MSLK_AMD_INDEX_I64 or _I32", op);
  if (T < 0 || D < 0 || a < 0 || E < 0) return fail("%s: negative dimension", op);
  if (a > kIntMax || D > kIntMax) return fail("%s: dimension exceeds 2^31-1", op);
  if (a == 0 || D == 0) return 0;
  if (!x || !token_indices || !expert_indices || !scores || !out || !out_scale) return fail("%s: null pointer", op);
  FusedQuantArgs p{};
  p.x0 = x; p.stride0 = D; p.dtype = x_dtype;
  p.out = (uint8_t*)out; p.out_scale = out_scale; p.rows = a; p.D = (int)D; p.scale_ub = scale_ub;
  p.valid_count = valid_token_count; p.valid_is_i64 = count_dtype == MSLK_AMD_INDEX_I64;
  p.token_idx = token_indices; p.token_is_i64 = token_dtype == MSLK_AMD_INDEX_I64;
  p.expert_idx = expert_indices; p.expert_is_i64 = expert_dtype == MSLK_AMD_INDEX_I64;
  p.scores = scores; p.score_dtype = score_dtype; p.stride_t = score_stride_t; p.stride_e = score_stride_e;
  p.T = T; p.E = E;
  return check_hip(launch_fused_quant(p, kFusedGatherScale, (hipStream_t)stream), "gather_scale_quant launch");
}

// K that is not a multiple of 16: the operand rows cannot be fetched by the 16-byte loads of the MFMA kernels.  With a
// workspace the call copies both operands into rows of K rounded up to 16 (zero tail: code 0x00 is +0) and runs the
// ordinary kernels on the copies; without one it falls back to the scalar kernel, which is orders of magnitude slower.
// K a multiple of 16 on a shape with few output tiles and a long K: with a workspace of slices * M * N floats the call
// splits K (gemm_splitk.hip); without one it runs the ordinary kernels.
size_t mslk_amd_f8f8bf16_rowwise_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || M > kIntMax || N > kIntMax || K > kIntMax) return 0;
  if (K % 16 != 0) return (size_t)((M + N) * ((K + 15) / 16 * 16));
  const SplitKPlan plan = splitk_plan(M, N, K, device_compute_units());
  return plan.slices > 1 ? (size_t)plan.slices * (size_t)M * (size_t)N * sizeof(float) : 0;
}

static int rowwise_impl(const char* op, int out_f16, int preshuffled, const void* xq, const void* wq, const float* x_scale,
                        const float* w_scale, const void* bias, int bias_dtype, void* y, int64_t M, int64_t N,
                        int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  if (M < 0 || N < 0 || K < 0) return fail("%s: negative dimension", op);
  if (M > kIntMax || N > kIntMax || K > kIntMax) return fail("%s: dimension exceeds 2^31-1", op);
  if (bias_dtype < 0 || bias_dtype > 2) return fail("%s: bad bias dtype code %d", op, bias_dtype);
  if ((bias_dtype != 0) != (bias != nullptr)) return fail("%s: bias pointer and bias dtype disagree", op);
  hipStream_t s = (hipStream_t)stream;
  if (M == 0 || N == 0) return 0;
  if (!y) return fail("%s: null output", op);
  if (K == 0) return check_hip(launch_fill_zero_bf16((uint16_t*)y, M * N, s), "zero fill");
  if (!xq || !wq || !x_scale || !w_scale) return fail("%s: null pointer", op);
  if (preshuffled && (N % 16 != 0 || K % 64 != 0))
    return fail("%s: pre-shuffled weights need N %% 16 == 0 and K %% 64 == 0 (got N=%lld, K=%lld)", op, (long long)N, (long long)K);
  GemmProblem p{(const uint8_t*)xq, (const uint8_t*)wq, x_scale, w_scale, bias, (uint16_t*)y,
                (int)M, (int)N, (int)K, bias_dtype, out_f16, preshuffled};
  // Operand rows the 16-byte loads cannot fetch (K % 16 != 0, or a base pointer that is not 16-byte aligned) are copied
  // into the workspace when the caller gave one that holds both copies.
  const int64_t Kp = (K + 15) / 16 * 16;
  const bool unfetchable = K % 16 != 0 || reinterpret_cast<uintptr_t>(xq) % 16 != 0 || reinterpret_cast<uintptr_t>(wq) % 16 != 0;
  if (unfetchable && !preshuffled && workspace && workspace_bytes >= (size_t)((M + N) * Kp) &&
      reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
    if (Kp <= kIntMax) {
      uint8_t* xp = static_cast<uint8_t*>(workspace);
      uint8_t* wp = xp + M * Kp;
      if (int rc = check_hip(launch_pad_rows(p.xq, xp, M, K, Kp, s), "pad rows launch")) return rc;
      if (int rc = check_hip(launch_pad_rows(p.wq, wp, N, K, Kp, s), "pad rows launch")) return rc;
      p.xq = xp;
      p.wq = wp;
      p.K = (int)Kp;
    }
  }
  const bool tiled_ok = dense_tiled_supports(p);
  // Few output tiles and a long K: split K when the caller's workspace holds the fp32 sums of every slice.
  if (!unfetchable && tiled_ok && workspace && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
    const SplitKPlan plan = splitk_plan(M, N, K, device_compute_units());
    if (plan.slices > 1 && workspace_bytes >= (size_t)plan.slices * (size_t)M * (size_t)N * sizeof(float))
      return check_hip(launch_splitk(p, plan, static_cast<float*>(workspace), s), "split-K launch");
  }
  // M <= 64: the weight-streaming kernel, except on wide row-major weights, where short tiles that share their
  // activation rows through LDS win from M = 9 on.  Pre-shuffled weights
  // keep the streaming kernel, whose register-direct weight loads stay ahead up to M = 64.
  const bool wide = !p.w_preshuffled && p.M > 8 && p.N >= kShortTileMinN;
  if (skinny_supports(p) && !(tiled_ok && wide)) return check_hip(launch_skinny(p, s), "skinny launch");
  if (tiled_ok) return check_hip(launch_dense_tiled(p, s), "tiled launch");
  return check_hip(launch_generic(p, s), "generic launch");
}

int mslk_amd_f8f8bf16_rowwise(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                              const void* bias, int bias_dtype, void* y, int64_t M, int64_t N, int64_t K,
                              void* workspace, size_t workspace_bytes, void* stream) {
  return rowwise_impl("f8f8bf16_rowwise", 0, 0, xq, wq, x_scale, w_scale, bias, bias_dtype, y, M, N, K, workspace, workspace_bytes, stream);
}

size_t mslk_amd_static_scratch_bytes(void) { return kScratchBytes; }

int mslk_amd_f8f8bf16_rowwise_static_scratch(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                                             const void* bias, int bias_dtype, void* y, int64_t M, int64_t N, int64_t K,
                                             void* stream) {
  const char* op = "f8f8bf16_rowwise_static_scratch";
  void* ptr = nullptr;
  size_t bytes = 0;
  const bool unfetchable = K % 16 != 0 || reinterpret_cast<uintptr_t>(xq) % 16 != 0 || reinterpret_cast<uintptr_t>(wq) % 16 != 0;
  if (M > 0 && N > 0 && K > 0 && M <= kIntMax && N <= kIntMax && K <= kIntMax && unfetchable) {
    const int64_t Kp = (K + 15) / 16 * 16;
    const double need = ((double)M + (double)N) * (double)Kp;
    if (need > (double)kScratchBytes)
      return fail("%s: the padded operand copies need (M + N) * round_up(K, 16) = %.0f bytes, the static scratch array holds %zu; "
                  "use mslk_amd_f8f8bf16_rowwise with a workspace", op, need, kScratchBytes);
    if (int rc = scratch_of_current_device(&ptr)) return rc;
    bytes = kScratchBytes;
  } else {
    // a shape the library would split along K: the fp32 sums of the slices go into the array when they fit (otherwise
    // the unsplit kernels run, as without a workspace)
    const size_t need = mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K);
    if (need > 0 && need <= kScratchBytes) {
      if (int rc = scratch_of_current_device(&ptr)) return rc;
      bytes = kScratchBytes;
    }
  }
  return rowwise_impl(op, 0, 0, xq, wq, x_scale, w_scale, bias, bias_dtype, y, M, N, K, ptr, bytes, stream);
}

int mslk_amd_quantize_f8f8bf16_rowwise_supported(int64_t M, int64_t N, int64_t K) {
  return M >= 1 && M <= 4 && N >= 1 && N <= kIntMax && K >= 1024 && K % 128 == 0 && K <= (int64_t(1) << 25);
}

int mslk_amd_quantize_f8f8bf16_rowwise(const void* x, int x_dtype, int64_t x_row_stride, const void* wq, const float* w_scale,
                                       const void* bias, int bias_dtype, void* y, int64_t M, int64_t N, int64_t K,
                                       void* xq_out, float* x_scale_out, void* stream) {
  const char* op = "quantize_f8f8bf16_rowwise";
  if (x_dtype != MSLK_AMD_DTYPE_BF16) return fail("%s: activations must be bf16 (dtype code %d)", op, x_dtype);
  if (bias_dtype < 0 || bias_dtype > 2) return fail("%s: bad bias dtype code %d", op, bias_dtype);
  if ((bias_dtype != 0) != (bias != nullptr)) return fail("%s: bias pointer and bias dtype disagree", op);
  if (!mslk_amd_quantize_f8f8bf16_rowwise_supported(M, N, K))
    return fail("%s: the one-launch path needs 1 <= M <= 4 and K a multiple of 1024 (got M=%lld, N=%lld, K=%lld); "
                "use mslk_amd_quantize_fp8_row followed by mslk_amd_f8f8bf16_rowwise", op, (long long)M, (long long)N, (long long)K);
  if (!x || !wq || !w_scale || !y) return fail("%s: null pointer", op);
  GemmProblem p{nullptr, (const uint8_t*)wq, nullptr, w_scale, bias, (uint16_t*)y, (int)M, (int)N, (int)K, bias_dtype, 0, 0};
  if (!skinny_fused_quant_supports(p, x, x_row_stride) || (xq_out && reinterpret_cast<uintptr_t>(xq_out) % 16 != 0))
    return fail("%s: x, wq and xq_out must be 16-byte aligned and the row stride of x a multiple of 8 elements, at least K", op);
  return check_hip(launch_skinny_fused_quant(p, x, x_row_stride, xq_out, x_scale_out, (hipStream_t)stream), "fused decode launch");
}

int mslk_amd_f8f8f16_rowwise(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                             const void* bias, int bias_dtype, void* y, int64_t M, int64_t N, int64_t K,
                             void* workspace, size_t workspace_bytes, void* stream) {
  return rowwise_impl("f8f8f16_rowwise", 1, 0, xq, wq, x_scale, w_scale, bias, bias_dtype, y, M, N, K, workspace, workspace_bytes, stream);
}

int mslk_amd_f8f8_rowwise_preshuffle(const void* xq, const void* wq_shuffled, const float* x_scale, const float* w_scale,
                                     const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M, int64_t N,
                                     int64_t K, void* stream) {
  if (y_dtype != MSLK_AMD_DTYPE_BF16 && y_dtype != MSLK_AMD_DTYPE_F16)
    return fail("f8f8_rowwise_preshuffle: output dtype code %d is neither bf16 nor fp16", y_dtype);
  return rowwise_impl(y_dtype == MSLK_AMD_DTYPE_F16 ? "f8f8f16_rowwise_preshuffle" : "f8f8bf16_rowwise_preshuffle",
                      y_dtype == MSLK_AMD_DTYPE_F16, 1, xq, wq_shuffled, x_scale, w_scale, bias, bias_dtype, y, M, N, K, nullptr, 0, stream);
}

int mslk_amd_f8f8_rowwise_preshuffle_workspace(const void* xq, const void* wq_shuffled, const float* x_scale, const float* w_scale,
                                               const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M, int64_t N,
                                               int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  if (y_dtype != MSLK_AMD_DTYPE_BF16 && y_dtype != MSLK_AMD_DTYPE_F16)
    return fail("f8f8_rowwise_preshuffle: output dtype code %d is neither bf16 nor fp16", y_dtype);
  return rowwise_impl(y_dtype == MSLK_AMD_DTYPE_F16 ? "f8f8f16_rowwise_preshuffle" : "f8f8bf16_rowwise_preshuffle",
                      y_dtype == MSLK_AMD_DTYPE_F16, 1, xq, wq_shuffled, x_scale, w_scale, bias, bias_dtype, y, M, N, K, workspace,
                      workspace_bytes, stream);
}

int mslk_amd_preshuffle_b(const void* wq, void* wq_shuffled, int64_t G, int64_t N, int64_t K, void* stream) {
  if (G < 0 || N < 0 || K < 0) return fail("preshuffle_b: negative dimension");
  if (N % 16 != 0 || K % 64 != 0) return fail("preshuffle_b needs N %% 16 == 0 and K %% 64 == 0, got N=%lld K=%lld", (long long)N, (long long)K);
  if (G == 0 || N == 0 || K == 0) return 0;
  if (!wq || !wq_shuffled) return fail("preshuffle_b: null pointer");
  if (wq == wq_shuffled) return fail("preshuffle_b: the permutation cannot run in place");
  if (reinterpret_cast<uintptr_t>(wq) % 16 || reinterpret_cast<uintptr_t>(wq_shuffled) % 16) return fail("preshuffle_b: pointers must be 16-byte aligned");
  return check_hip(launch_preshuffle_b(wq, wq_shuffled, G, N, K, (hipStream_t)stream), "preshuffle_b launch");
}

int mslk_amd_f8f8bf16_rowwise_grouped(int G, const void* const* xq, const void* const* wq,
                                      const float* const* x_scale, const float* const* w_scale, void* const* y,
                                      const int64_t* M, const int64_t* N, const int64_t* K, void* stream) {
  if (G < 0) return fail("f8f8bf16_rowwise_grouped: negative group count");
  hipStream_t s = (hipStream_t)stream;
  GroupTable tab;
  tab.count = 0;
  tab.total_tiles = 0;
  auto flush = [&]() -> int {
    if (tab.count == 0) return 0;
    int rc = check_hip(launch_grouped_tiled(tab, s), "grouped launch");
    tab.count = 0;
    tab.total_tiles = 0;
    return rc;
  };
  for (int g = 0; g < G; ++g) {
    if (M[g] < 0 || N[g] < 0 || K[g] < 0 || M[g] > kIntMax || N[g] > kIntMax || K[g] > kIntMax)
      return fail("f8f8bf16_rowwise_grouped: bad dimensions in group %d", g);
    if (M[g] == 0 || N[g] == 0) continue;
    if (!y[g]) return fail("f8f8bf16_rowwise_grouped: null output in group %d", g);
    if (K[g] == 0) {
      if (int rc = check_hip(launch_fill_zero_bf16((uint16_t*)y[g], M[g] * N[g], s), "zero fill")) return rc;
      continue;
    }
    if (!xq[g] || !wq[g] || !x_scale[g] || !w_scale[g]) return fail("f8f8bf16_rowwise_grouped: null pointer in group %d", g);
    GemmProblem p{(const uint8_t*)xq[g], (const uint8_t*)wq[g], x_scale[g], w_scale[g], nullptr, (uint16_t*)y[g],
                  (int)M[g], (int)N[g], (int)K[g], 0, 0, 0};
    if (!dense_tiled_supports(p)) {  // odd K or alignment: per-group fallback
      if (int rc = check_hip(launch_generic(p, s), "generic launch")) return rc;
      continue;
    }
    GroupDesc& d = tab.g[tab.count];
    d.xq = p.xq; d.wq = p.wq; d.xs = p.xs; d.ws = p.ws; d.y = p.y;
    d.M = p.M; d.N = p.N; d.K = p.K;
    d.tile_begin = tab.total_tiles;
    const int64_t tiles = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256);
    if (tab.total_tiles + tiles > kIntMax) return fail("f8f8bf16_rowwise_grouped: too many tiles");
    tab.total_tiles += (int)tiles;
    if (++tab.count == kMaxGroupsPerLaunch)
      if (int rc = flush()) return rc;
  }
  return flush();
}

int mslk_amd_f8f8bf16_rowwise_grouped_stacked(const void* xq, const void* wq, const float* x_scale,
                                              const float* w_scale, const int64_t* m_sizes_dev, int G,
                                              int64_t total_M, int64_t N, int64_t K, void* y, void* stream) {
  if (G < 0 || total_M < 0 || N < 0 || K < 0) return fail("f8f8bf16_rowwise_grouped_stacked: negative dimension");
  if (total_M > kIntMax || N > kIntMax || K > kIntMax) return fail("f8f8bf16_rowwise_grouped_stacked: dimension exceeds 2^31-1");
  hipStream_t s = (hipStream_t)stream;
  if (G == 0 || total_M == 0 || N == 0) return 0;
  if (!y) return fail("f8f8bf16_rowwise_grouped_stacked: null output");
  if (K == 0) return check_hip(launch_fill_zero_bf16((uint16_t*)y, total_M * N, s), "zero fill");
  if (!xq || !wq || !x_scale || !w_scale || !m_sizes_dev) return fail("f8f8bf16_rowwise_grouped_stacked: null pointer");
  DeviceGroups p{(const uint8_t*)xq, (const uint8_t*)wq, x_scale, w_scale, nullptr, (uint16_t*)y, m_sizes_dev, G,
                 (int)total_M, (int)N, (int)K, 0, 0};
  return check_hip(launch_device_groups(p, kGroupsSizesM, s), "grouped stacked launch");
}

int mslk_amd_f8f8bf16_rowwise_grouped_mm(const void* xq, const void* wq, const float* x_scale,
                                         const float* w_scale, const int32_t* offsets_dev, int layout, int G,
                                         int64_t M, int64_t N, int64_t K, void* y, void* stream) {
  if (layout < MSLK_AMD_GROUPS_M_OFFSETS || layout > MSLK_AMD_GROUPS_UNIFORM)
    return fail("f8f8bf16_rowwise_grouped_mm: unknown group layout code %d", layout);
  if (G < 0 || M < 0 || N < 0 || K < 0) return fail("f8f8bf16_rowwise_grouped_mm: negative dimension");
  if (M > kIntMax || N > kIntMax || K > kIntMax) return fail("f8f8bf16_rowwise_grouped_mm: dimension exceeds 2^31-1");
  const bool uniform = layout == MSLK_AMD_GROUPS_UNIFORM;
  if (uniform != (offsets_dev == nullptr))
    return fail(uniform ? "f8f8bf16_rowwise_grouped_mm: offsets must be NULL for the uniform layout"
                        : "f8f8bf16_rowwise_grouped_mm: offsets are required for this layout");
  hipStream_t s = (hipStream_t)stream;
  if (G == 0 || M == 0 || N == 0) return 0;
  if (!y) return fail("f8f8bf16_rowwise_grouped_mm: null output");
  const bool stacked_out = layout == MSLK_AMD_GROUPS_K_OFFSETS || uniform;   // y is [G, M, N]
  if (stacked_out && (double)G * (double)M * (double)N > 9.0e18) return fail("f8f8bf16_rowwise_grouped_mm: output too large");
  // K == 0 needs no special case: every tile a group owns is written with the empty sum.
  if ((K > 0 && (!xq || !wq)) || !x_scale || !w_scale) return fail("f8f8bf16_rowwise_grouped_mm: null pointer");
  DeviceGroups p{(const uint8_t*)xq, (const uint8_t*)wq, x_scale, w_scale, nullptr, (uint16_t*)y, offsets_dev, G,
                 (int)M, (int)N, (int)K, 0, 0};
  return check_hip(launch_device_groups(p, layout, s), "grouped_mm launch");
}

int mslk_amd_f8f8bf16_rowwise_grouped_dynamic(const void* xq, const void* wq, const float* x_scale,
                                              const float* w_scale, const int64_t* zero_start_index_M_dev, int G,
                                              int64_t M, int64_t N, int64_t K, void* y, int zeroing_output,
                                              void* stream) {
  if (G < 0 || M < 0 || N < 0 || K < 0) return fail("f8f8bf16_rowwise_grouped_dynamic: negative dimension");
  if (M > kIntMax || N > kIntMax || K > kIntMax) return fail("f8f8bf16_rowwise_grouped_dynamic: dimension exceeds 2^31-1");
  hipStream_t s = (hipStream_t)stream;
  if (G == 0 || M == 0 || N == 0) return 0;
  if (!y) return fail("f8f8bf16_rowwise_grouped_dynamic: null output");
  if ((double)G * (double)M * (double)N > 9.0e18) return fail("f8f8bf16_rowwise_grouped_dynamic: output too large");
  if ((K > 0 && (!xq || !wq)) || !x_scale || !w_scale || !zero_start_index_M_dev)
    return fail("f8f8bf16_rowwise_grouped_dynamic: null pointer");
  if (zeroing_output)
    if (int rc = check_hip(launch_fill_zero_bf16((uint16_t*)y, (int64_t)G * M * N, s), "zero fill")) return rc;
  DeviceGroups p{(const uint8_t*)xq, (const uint8_t*)wq, x_scale, w_scale, nullptr, (uint16_t*)y, zero_start_index_M_dev,
                 G, (int)M, (int)N, (int)K, 0, 0};
  return check_hip(launch_device_groups(p, kGroupsPrepadM, s), "grouped dynamic launch");
}

int mslk_amd_f8f8bf16_rowwise_batched(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                                      const void* bias, int bias_dtype, int64_t B, int64_t M, int64_t N,
                                      int64_t K, void* y, void* stream) {
  if (B < 0 || M < 0 || N < 0 || K < 0) return fail("f8f8bf16_rowwise_batched: negative dimension");
  if (B > kIntMax || M > kIntMax || N > kIntMax || K > kIntMax) return fail("f8f8bf16_rowwise_batched: dimension exceeds 2^31-1");
  if (bias_dtype < 0 || bias_dtype > 2) return fail("f8f8bf16_rowwise_batched: bad bias dtype code %d", bias_dtype);
  if ((bias_dtype != 0) != (bias != nullptr)) return fail("f8f8bf16_rowwise_batched: bias pointer and bias dtype disagree");
  hipStream_t s = (hipStream_t)stream;
  if (B == 0 || M == 0 || N == 0) return 0;
  if (!y) return fail("f8f8bf16_rowwise_batched: null output");
  if ((double)B * (double)M * (double)N > 9.0e18) return fail("f8f8bf16_rowwise_batched: output too large");
  if ((K > 0 && (!xq || !wq)) || !x_scale || !w_scale) return fail("f8f8bf16_rowwise_batched: null pointer");
  DeviceGroups p{(const uint8_t*)xq, (const uint8_t*)wq, x_scale, w_scale, bias, (uint16_t*)y, nullptr, (int)B,
                 (int)M, (int)N, (int)K, bias_dtype, 0};
  return check_hip(launch_device_groups(p, kGroupsUniform, s), "batched launch");
}

int mslk_amd_debug_cast_e4m3fn(const float* in, int64_t n, void* out, void* stream) {
  if (n < 0) return fail("debug_cast_e4m3fn: negative count");
  if (n == 0) return 0;
  if (!in || !out) return fail("debug_cast_e4m3fn: null pointer");
  return check_hip(launch_cast_e4m3fn(in, n, out, (hipStream_t)stream), "cast launch");
}

const char* mslk_amd_debug_dispatch_name(int64_t M, int64_t N, int64_t K, int bias_dtype, int y_dtype, int preshuffled,
                                         int with_workspace) {
  // Aligned stand-in pointers: the dry run dereferences nothing and launches nothing.
  void* const fake = reinterpret_cast<void*>(uintptr_t(1) << 20);
  thread_local char result[600];
  const size_t wbytes = with_workspace ? mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K) : 0;
  dispatch_probe_begin();
  const int rc = rowwise_impl("debug_dispatch_name", y_dtype == MSLK_AMD_DTYPE_F16, preshuffled, fake, fake, (const float*)fake,
                              (const float*)fake, bias_dtype ? fake : nullptr, bias_dtype, fake, M, N, K, wbytes ? fake : nullptr,
                              wbytes, nullptr);
  const char* text = dispatch_probe_end();
  if (rc != 0) snprintf(result, sizeof(result), "error: %s", g_err);
  else snprintf(result, sizeof(result), "%s", text[0] ? text : "nothing to launch");
  return result;
}

int mslk_amd_debug_stream_read(const void* src, int64_t bytes, int mode, int workgroups, void* sink, void* stream) {
  if (mode < 0 || mode > 2) return fail("debug_stream_read: mode must be 0 (register loads), 1 (LDS DMA loads) or 2 (non-temporal LDS DMA loads)");
  if (bytes < 0 || bytes % (mode == 0 ? 16 : 1024) != 0) return fail("debug_stream_read: bytes must be a non-negative multiple of %d", mode == 0 ? 16 : 1024);
  if (workgroups <= 0 || workgroups > 65536) return fail("debug_stream_read: workgroups must be in 1 .. 65536");
  if (bytes == 0) return 0;
  if (!src || reinterpret_cast<uintptr_t>(src) % 16 != 0) return fail("debug_stream_read: src must be a 16-byte aligned device pointer");
  return check_hip(launch_debug_stream_read(src, bytes, mode, workgroups, sink, (hipStream_t)stream), "stream read launch");
}

int mslk_amd_debug_mfma_loop(const void* operands, int form, int iters, int workgroups, void* sink, void* stream) {
  if (form != 0 && form != 1) return fail("debug_mfma_loop: form must be 0 (16x16x128) or 1 (32x32x64)");
  if (iters < 0 || iters > (1 << 20)) return fail("debug_mfma_loop: iters must be in 0 .. 2^20");
  if (workgroups <= 0 || workgroups > 65536) return fail("debug_mfma_loop: workgroups must be in 1 .. 65536");
  if (!operands || reinterpret_cast<uintptr_t>(operands) % 32 != 0) return fail("debug_mfma_loop: operands must be a 32-byte aligned device pointer to 128 KiB");
  return check_hip(launch_debug_mfma_loop(operands, form, iters, workgroups, sink, (hipStream_t)stream), "mfma loop launch");
}

int mslk_amd_debug_tile_streams(const void* x, int64_t x_bytes, const void* w, int64_t w_bytes, int64_t K, int tiles_m, int tiles_n,
                                int which, void* stream) {
  if (which < 1 || which > 3) return fail("debug_tile_streams: which must be 1 (activations), 2 (weights) or 3 (both)");
  if (K < 128 || K % 128 != 0 || K > (1 << 20)) return fail("debug_tile_streams: K must be a multiple of 128 in 128 .. 2^20, got %lld", (long long)K);
  if (tiles_m <= 0 || tiles_n <= 0 || (int64_t)tiles_m * tiles_n > (1 << 20)) return fail("debug_tile_streams: tiles_m * tiles_n must be in 1 .. 2^20");
  if (x_bytes < (int64_t)tiles_m * 128 * K || w_bytes < (int64_t)tiles_n * 64 * K)
    return fail("debug_tile_streams: x must hold tiles_m * 128 rows of K bytes and w tiles_n * 64 rows");
  if (!x || !w || reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0)
    return fail("debug_tile_streams: x and w must be 16-byte aligned device pointers");
  return check_hip(launch_debug_tile_streams(x, w, (int)K, tiles_m, tiles_n, which, (hipStream_t)stream), "tile streams launch");
}

int mslk_amd_debug_gemm_phases(const void* xq, const void* wq, const float* x_scale, const float* w_scale, void* y, int64_t M,
                               int64_t N, int64_t K, uint64_t* stamps, void* stream) {
  if (M <= 0 || N <= 0 || M % 256 != 0 || N % 256 != 0 || M > (1 << 20) || N > (1 << 20))
    return fail("debug_gemm_phases: M and N must be positive multiples of 256 (interior tiles only), got M=%lld N=%lld", (long long)M, (long long)N);
  if (K < 256 || K % 128 != 0 || K > (1 << 24)) return fail("debug_gemm_phases: K must be a multiple of 128, at least 256, got %lld", (long long)K);
  if ((M / 256) * (N / 256) > (1 << 20)) return fail("debug_gemm_phases: more than 2^20 tiles");
  if (!xq || !wq || !x_scale || !w_scale || !y || !stamps) return fail("debug_gemm_phases: null pointer");
  if (reinterpret_cast<uintptr_t>(xq) % 16 || reinterpret_cast<uintptr_t>(wq) % 16 || reinterpret_cast<uintptr_t>(y) % 16 ||
      reinterpret_cast<uintptr_t>(w_scale) % 16 || reinterpret_cast<uintptr_t>(stamps) % 8)
    return fail("debug_gemm_phases: operands, output and w_scale must be 16-byte aligned, stamps 8-byte aligned");
  GemmProblem p{(const uint8_t*)xq, (const uint8_t*)wq, x_scale, w_scale, nullptr, (uint16_t*)y, (int)M, (int)N, (int)K, 0, 0, 0};
  return check_hip(launch_debug_gemm_phases(p, stamps, (hipStream_t)stream), "gemm phases launch");
}

}  // extern "C"
