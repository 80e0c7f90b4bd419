/*
 * mslk_amd -- C ABI of the MI355X (gfx950) FP8 rowwise quantized-linear path.
 *
 * Every entry point is plain C: device pointers, sizes, a HIP stream handle passed as void*.
 * Nothing is allocated, freed or synchronised inside a call; all pointers are borrowed for the
 * duration of the call; kernels are enqueued on `stream` (NULL = the default stream) and are
 * safe to record into a HIP graph.  Return value 0 = success; non-zero = argument or launch error,
 * with a human-readable message available from mslk_amd_last_error() (thread-local).
 *
 * Data conventions (unchanged from the reference operators):
 *   XQ  [M, K]  e4m3fn codes, row-major contiguous          (activations)
 *   WQ  [N, K]  e4m3fn codes, row-major contiguous          (weights; i.e. B is column-major, "TN")
 *   x_scale [M], w_scale [N]  fp32
 *   bias [N]  fp32 or bf16, optional
 *   Y   [M, N]  bf16, row-major contiguous:  Y = bf16( (acc_fp32 * w_scale[n]) * x_scale[m] + bias[n] )
 */
#ifndef MSLK_AMD_H_
#define MSLK_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of the high-precision quantizer input */
#define MSLK_AMD_DTYPE_BF16 0
#define MSLK_AMD_DTYPE_F16 1
#define MSLK_AMD_DTYPE_F32 2

/* bias element types */
#define MSLK_AMD_BIAS_NONE 0
#define MSLK_AMD_BIAS_F32 1
#define MSLK_AMD_BIAS_BF16 2

/* Library version string and the last error message of the calling thread. */
const char* mslk_amd_version(void);
const char* mslk_amd_last_error(void);

/*
 * Row-wise FP8 quantization.  Replaces quantize_fp8_row
 * (reference: mslk/quantize/triton/fp8_quantize.py:319-378; bit-exact to its torch branch 356-378,
 * whose arithmetic is: amax in the input dtype, clamp(min=1e-12[, max=*scale_ub]) in the input
 * dtype, inv = fl32(fl32(1/amax) * 448), inf -> 1, code = e4m3fn_rne(fl32(x) * inv), scale = fl32(1/inv)).
 *   x          [rows, K] elements of `x_dtype`, row stride `x_row_stride` elements, unit column stride
 *   xq         [rows, K_out] e4m3fn, contiguous; K_out >= K, columns [K, K_out) are zero-filled
 *              (K_out > K is the reference's align_rows_to padding, fp8_quantize.py:251-259)
 *   scale      [rows] fp32
 *   scale_ub   optional device pointer to ONE fp32 upper bound for amax (fp8_quantize.py:365-366)
 */
int mslk_amd_quantize_fp8_row(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t x_row_stride,
                              void* xq, int64_t K_out, float* scale, const float* scale_ub, void* stream);

/*
 * The same quantizer over jagged groups of rows.  Replaces quantize_fp8_row(..., zero_start_index_M=...)
 * (reference: mslk/quantize/triton/fp8_quantize.py:238-243 for the grouping, 123-129 for the row rule):
 * the rows form rows / rows_per_group consecutive blocks; in block b only the first
 * zero_start_index[b] rows hold data.  The remaining rows are never read and quantize exactly like
 * all-zero rows (zero codes, the scale of a zero row).
 *   zero_start_index  [rows / rows_per_group] int64 or int32 (index_dtype) in device memory
 */
#define MSLK_AMD_INDEX_I64 0
#define MSLK_AMD_INDEX_I32 1
int mslk_amd_quantize_fp8_row_jagged(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t x_row_stride,
                                     void* xq, int64_t K_out, float* scale, const float* scale_ub,
                                     const void* zero_start_index, int index_dtype, int64_t rows_per_group,
                                     void* stream);

/*
 * The quantizer with the arithmetic of the reference's GPU (Triton) branch instead of its torch branch
 * (reference: _kernel_quantize_fp8_row, mslk/quantize/triton/fp8_quantize.py:131-207; eps default 1/512,
 * same file 215,246-247):
 *   amax = clamp(max|x|, eps [, *scale_ub]);  scale = fl32(amax / 448);
 *   code = e4m3fn_rne(clamp(fl32(fl32(x) / scale), -448, 448))      (IEEE divisions, saturating)
 * Arguments as mslk_amd_quantize_fp8_row_jagged; zero_start_index may be NULL (then index_dtype and
 * rows_per_group are ignored).  The bits differ from mslk_amd_quantize_fp8_row in the last place of some
 * scales and codes, in the lower bound of amax, and in saturating where scale_ub cuts the maximum.
 */
int mslk_amd_quantize_fp8_row_triton_arithmetic(const void* x, int x_dtype, int64_t rows, int64_t K, int64_t x_row_stride,
                                                void* xq, int64_t K_out, float* scale, const float* scale_ub, float eps,
                                                const void* zero_start_index, int index_dtype, int64_t rows_per_group,
                                                void* stream);

/*
 * Row-wise dequantization to bf16.  Replaces dequantize_fp8_row
 * (reference: mslk/quantize/triton/fp8_quantize.py:1060-1113 kernel, 1140-1182 wrapper):
 *   out[r, k] = bf16_rne( fl32( f32(xq[r, k]) * scale[r] ) )
 *   xq [rows, K] e4m3fn contiguous, scale [rows] fp32, out [rows, K] bf16 contiguous.
 */
int mslk_amd_dequantize_fp8_row(const void* xq, const float* scale, int64_t rows, int64_t K, void* out, void* stream);

/*
 * Fused SiLU-gate, multiply and row-wise FP8 quantization: the producer of the second MoE GEMM's
 * activations.  Replaces mslk::silu_mul_quant (reference: mslk/moe/activation.py:72-135 wrapper,
 * 232-300 kernel):
 *   y = x0 * sigmoid(x0) * x1 in fp32;  row_max = clamp(max|y|, 1e-12 [, *scale_ub]);  s = 448 / row_max;
 *   out = e4m3fn_rne(clamp(y * s, -448, 448));  out_scale = 1 / s.
 *   x0, x1     [T, D] bf16 or fp16 (x_dtype), unit column stride, row strides in elements
 *   out        [T, D] e4m3fn contiguous;  out_scale [T] fp32
 *   valid_token_count  optional device scalar (int32 or int64 per count_dtype): rows at or beyond it
 *                      are neither read nor written
 */
int mslk_amd_silu_mul_quant(const void* x0, const void* x1, int x_dtype, int64_t T, int64_t D, int64_t x0_row_stride,
                            int64_t x1_row_stride, void* out, float* out_scale, const float* scale_ub,
                            const void* valid_token_count, int count_dtype, void* stream);

/*
 * Fused gather of routed tokens, multiplication by the routing score and row-wise FP8 quantization:
 * the producer of the first MoE GEMM's activations.  Replaces gather_scale_quant_dense_tokens
 * (reference: mslk/moe/gather_scatter.py:96-170 wrapper, 545-640 kernel):
 *   y[i] = x[token_indices[i]] * scores[token_indices[i], expert_indices[i]] in fp32, then quantized
 *   as in mslk_amd_silu_mul_quant.
 *   x [T, D] bf16/fp16 contiguous; token_indices, expert_indices [a] int32 or int64 (per *_dtype);
 *   scores [T, E] bf16/fp16/fp32 with element strides (score_stride_t, score_stride_e);
 *   out [a, D] e4m3fn; out_scale [a].  Rows at or beyond *valid_token_count, and rows whose indices fall
 *   outside [0, T) x [0, E), are neither read nor written.
 */
int mslk_amd_gather_scale_quant_dense_tokens(const void* x, int x_dtype, int64_t T, int64_t D,
                                             const void* token_indices, int token_dtype,
                                             const void* expert_indices, int expert_dtype, int64_t a,
                                             const void* scores, int score_dtype, int64_t E, int64_t score_stride_t,
                                             int64_t score_stride_e, void* out, float* out_scale,
                                             const float* scale_ub, const void* valid_token_count, int count_dtype,
                                             void* stream);

/*
 * Dense rowwise-scaled FP8 GEMM.  Replaces mslk::gemm::f8f8bf16_rowwise / f8f8bf16_rowwise_out
 * (reference: csrc/gemm/gemm_ops.cpp:31-34; host wrapper csrc/gemm/ck/fp8_rowwise/fp8fp8bf16_rowwise_gemm.hip:499-576;
 * math csrc/gemm/ck/fp8_rowwise/kernels/fp8_rowwise_common.h:54-82,168-204; bias semantics
 * csrc/gemm/cutlass/f8f8bf16_rowwise/f8f8bf16_rowwise_common.cuh:150-198).
 * M, N or K equal to 0 writes zeros to Y (fp8fp8bf16_rowwise_gemm.hip:531-534).
 * `workspace` (device memory, 16-byte aligned) is optional and only used when
 * mslk_amd_f8f8bf16_rowwise_workspace_bytes(M,N,K) > 0.  Two cases:
 *   - K is not a multiple of 16: the call copies both operands into workspace rows of K rounded up to 16 (zero tail) and
 *     runs the MFMA kernels on the copies (the CK instances of the reference pad K inside the kernel,
 *     fp8_rowwise_common.h:109-110 `GemmSpecialization::MNKPadding`).  An operand base pointer that is not 16-byte aligned
 *     is handled the same way if the workspace holds (M + N) * round_up(K, 16) bytes.  Without a workspace (null or too
 *     small) such operands still give the same results through a scalar kernel that is orders of magnitude slower.
 *   - few output tiles and a long K (64 < M, or 32 < M with K >= 12288; at most 128 tiles of 64 x 64 on a whole MI355X,
 *     K >= 6144 ... 8192; the
 *     reference's instances for such shapes split K as well, fp8_rowwise_common.h:168-204 `KBatch`): the call cuts K into
 *     2 ... 8 slices, whose fp32 sums go into the workspace (slices * M * N floats), and a second launch adds them and
 *     applies scales, bias and the conversion -- two to three times faster where the unsplit kernels would leave most
 *     CUs idle.  Without a workspace the unsplit kernels run; on operands whose products and sums are exact in fp32
 *     both give the same bits, otherwise they differ by the rounding of a different summation order.
 * The workspace needs no initialisation and holds nothing between calls; calls that share one workspace must not overlap.
 */
int mslk_amd_f8f8bf16_rowwise(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                              const void* bias, int bias_dtype, void* y,
                              int64_t M, int64_t N, int64_t K,
                              void* workspace, size_t workspace_bytes, void* stream);
size_t mslk_amd_f8f8bf16_rowwise_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * mslk_amd_f8f8bf16_rowwise for callers that cannot allocate a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation).  No counterpart in the reference.  Same arguments and results as
 * mslk_amd_f8f8bf16_rowwise, but the padded operand copies of the K % 16 != 0 / unaligned-operand case go into a
 * fixed array of MSLK_AMD_STATIC_SCRATCH_BYTES that is part of the library's device code (every GPU the library runs on
 * holds it until the process ends); the call allocates and frees nothing.  Shapes whose copies do not fit,
 * (M + N) * round_up(K, 16) > MSLK_AMD_STATIC_SCRATCH_BYTES, are rejected with an error.  The array needs no
 * initialisation (the copies overwrite every byte they later read), but all calls on one GPU share it: calls that
 * overlap on one GPU (different streams, or threads) race.  Shapes that the library splits along K (see above) put the
 * sums of their slices into the same array when they fit, and run unsplit when they do not.  Other shapes never touch it.
 * The first call on a device that needs the copies looks the array's address up (hipGetSymbolAddress; not a stream
 * operation) and is also the moment HIP commits the array's device memory; a caller that captures graphs or measures
 * memory makes that first call outside the capture / before the measurement.
 */
#define MSLK_AMD_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int mslk_amd_f8f8bf16_rowwise_static_scratch(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                                             const void* bias, int bias_dtype, void* y,
                                             int64_t M, int64_t N, int64_t K, void* stream);
size_t mslk_amd_static_scratch_bytes(void);

/*
 * Decode fast path: row-wise quantization of the activations AND the GEMM in one launch.  Replaces the pair
 * quantize_fp8_row(x) -> f8f8bf16_rowwise(xq, wq, x_scale, w_scale) that callers of the reference issue for every
 * decode step (reference: bench/gemm/gemm_ops.py:593-673; mslk/moe/layers.py:1096,1123), for the shapes where the first
 * launch costs about as much as the work: 1 <= M <= 4, K >= 1024, K % 128 == 0 (mslk_amd_quantize_f8f8bf16_rowwise_supported).
 *   x    [M, K] bf16 (x_dtype must be MSLK_AMD_DTYPE_BF16), row stride x_row_stride elements (a multiple of 8), 16-byte aligned
 *   wq, w_scale, bias, y   as mslk_amd_f8f8bf16_rowwise
 *   xq_out [M, K] e4m3fn, x_scale_out [M] fp32: optional (NULL to skip); they receive the codes and scales the kernel
 *          multiplied with -- the bits mslk_amd_quantize_fp8_row produces for x (no scale_ub).
 * Every workgroup quantizes the M rows itself (they stay in L2; each wave converts the K steps it multiplies), so nothing is exchanged between workgroups and the
 * call is one kernel: no workspace, graph-safe.  Other shapes return an error; use the two entry points then.
 */
int mslk_amd_quantize_f8f8bf16_rowwise(const void* x, int x_dtype, int64_t x_row_stride, const void* wq, const float* w_scale,
                                       const void* bias, int bias_dtype, void* y, int64_t M, int64_t N, int64_t K,
                                       void* xq_out, float* x_scale_out, void* stream);
int mslk_amd_quantize_f8f8bf16_rowwise_supported(int64_t M, int64_t N, int64_t K);

/*
 * The same GEMM with an fp16 (IEEE half, round to nearest even, overflow to infinity) output.
 * Replaces mslk::gemm::f8f8f16_rowwise (reference: csrc/gemm/gemm_ops.cpp:88-89,
 * csrc/gemm/ck/fp8_rowwise/fp8fp8fp16_rowwise_gemm.hip:66-133).  Arguments as above (the same workspace rule); y is fp16.
 */
int mslk_amd_f8f8f16_rowwise(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                             const void* bias, int bias_dtype, void* y, int64_t M, int64_t N, int64_t K,
                             void* workspace, size_t workspace_bytes, void* stream);

/*
 * The dense GEMM on PRE-SHUFFLED weights.  Replaces mslk::gemm::f8f8bf16_rowwise_preshuffle and
 * f8f8f16_rowwise_preshuffle (reference: csrc/gemm/gemm_ops.cpp:90-93,
 * csrc/gemm/ck/fp8_rowwise_preshuffle/fp8_rowwise_preshuffle_gemm.hip:93-171).  `wq_shuffled` holds the
 * [N, K] weights in the blocked order [N/16][K/64][4][16][16 bytes] that ck_preshuffle(wq, 16) /
 * preshuffle_b_mfma produce (reference: mslk/quantize/shuffle.py:182-246): every 16-row x 64-byte block is
 * stored as (16-byte k chunk, row, byte), i.e. in the order the 64 lanes of an MFMA operand read it.
 * Requires N % 16 == 0 and K % 64 == 0; everything else as mslk_amd_f8f8bf16_rowwise.
 * y_dtype: MSLK_AMD_DTYPE_BF16 or MSLK_AMD_DTYPE_F16.
 */
int mslk_amd_f8f8_rowwise_preshuffle(const void* xq, const void* wq_shuffled, const float* x_scale, const float* w_scale,
                                     const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M, int64_t N,
                                     int64_t K, void* stream);
/*
 * The same with the optional workspace of mslk_amd_f8f8bf16_rowwise (mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K)
 * bytes, 16-byte aligned): shapes with few output tiles and a long K are then split along K as on row-major weights.
 * Without a workspace it is the entry point above.
 */
int mslk_amd_f8f8_rowwise_preshuffle_workspace(const void* xq, const void* wq_shuffled, const float* x_scale,
                                               const float* w_scale, const void* bias, int bias_dtype, void* y, int y_dtype,
                                               int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                                               void* stream);

/*
 * Weight re-layout for the entry point above: wq [G, N, K] row-major -> wq_shuffled, the blocked
 * order applied to each of the G matrices (out of place).  Replaces ck_preshuffle / preshuffle_b_mfma
 * (reference: mslk/quantize/shuffle.py:182-246).  N % 16 == 0, K % 64 == 0, 16-byte aligned pointers.
 */
int mslk_amd_preshuffle_b(const void* wq, void* wq_shuffled, int64_t G, int64_t N, int64_t K, void* stream);

/*
 * Grouped (MoE) rowwise FP8 GEMM over G independent problems given as host arrays of device
 * pointers.  Replaces mslk::gemm::f8f8bf16_rowwise_grouped (TensorList API; reference:
 * csrc/gemm/gemm_ops.cpp:37-38, csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:481-559,586-593).
 * Group g computes Y_g[M_g, N_g] = bf16(XQ_g[M_g,K_g] . WQ_g[N_g,K_g]^T * x_scale_g[:,None] * w_scale_g[None,:]).
 * M/N/K and the pointer arrays live in HOST memory and are consumed before the call returns.
 * Groups with M_g == 0 are skipped; K_g == 0 writes zeros.
 */
int mslk_amd_f8f8bf16_rowwise_grouped(int G, const void* const* xq, const void* const* wq,
                                      const float* const* x_scale, const float* const* w_scale,
                                      void* const* y, const int64_t* M, const int64_t* N, const int64_t* K,
                                      void* stream);

/*
 * Grouped GEMM over stacked tensors with DEVICE-resident group sizes (no host sync; graph-safe).
 * Replaces mslk::gemm::f8f8bf16_rowwise_grouped_stacked (reference: csrc/gemm/gemm_ops.cpp:41-42,
 * csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:607-655).
 *   xq [total_M, K], wq [G, N, K], x_scale [total_M], w_scale [G, N], m_sizes int64 [G] on device,
 *   y [total_M, N].  Rows beyond sum(m_sizes) are left untouched.
 */
int mslk_amd_f8f8bf16_rowwise_grouped_stacked(const void* xq, const void* wq, const float* x_scale,
                                              const float* w_scale, const int64_t* m_sizes_dev, int G,
                                              int64_t total_M, int64_t N, int64_t K, void* y, void* stream);

/*
 * Grouped GEMM in the torch._grouped_mm calling convention: group boundaries are int32 cumulative
 * END offsets in DEVICE memory (no host sync; graph-safe).  Replaces
 * mslk::gemm::f8f8bf16_rowwise_grouped_mm (reference: csrc/gemm/gemm_ops.cpp:95-96,
 * csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:720-845; the per-group pointer
 * arithmetic restates set_kernel_args, same file 161-296).  `layout` selects the varying dimension;
 * M, N, K are the full tensor extents (the varying one is the total over groups):
 *   MSLK_AMD_GROUPS_M_OFFSETS  "2D-3D": xq [M, K], wq [G, N, K], x_scale [M], w_scale [G, N], y [M, N];
 *                              group g owns rows offsets[g-1] .. offsets[g] of xq / y.
 *   MSLK_AMD_GROUPS_N_OFFSETS  "3D-2D": xq [G, M, K], wq [N, K], x_scale [G, M], w_scale [N], y [M, N];
 *                              group g owns rows offsets[g-1] .. offsets[g] of wq = those columns of y.
 *   MSLK_AMD_GROUPS_K_OFFSETS  "2D-2D": xq [M, K], wq [N, K], x_scale [G*M], w_scale [G*N], y [G, M, N];
 *                              group g multiplies the K slice offsets[g-1] .. offsets[g] of both.
 *   MSLK_AMD_GROUPS_UNIFORM    "3D-3D": xq [G, M, K], wq [G, N, K], x_scale [G, M], w_scale [G, N],
 *                              y [G, M, N]; offsets must be NULL.
 * Rows / columns beyond offsets[G-1] are left untouched; an empty K slice writes zeros.  Offsets that
 * decrease or exceed the tensor extent make the affected workgroups write nothing.
 */
#define MSLK_AMD_GROUPS_M_OFFSETS 1
#define MSLK_AMD_GROUPS_N_OFFSETS 2
#define MSLK_AMD_GROUPS_K_OFFSETS 3
#define MSLK_AMD_GROUPS_UNIFORM 4
int mslk_amd_f8f8bf16_rowwise_grouped_mm(const void* xq, const void* wq, const float* x_scale,
                                         const float* w_scale, const int32_t* offsets_dev, int layout, int G,
                                         int64_t M, int64_t N, int64_t K, void* y, void* stream);

/*
 * Grouped GEMM over pre-padded groups: xq [G, M, K], wq [G, N, K], x_scale [G, M], w_scale [G, N],
 * y [G, M, N]; only the first zero_start_index_M[g] (int64, device memory) rows of group g are
 * multiplied.  With zeroing_output != 0 the whole of y is zero-filled first, so the padding rows read
 * as zero; otherwise they are left untouched.  Replaces mslk::gemm::f8f8bf16_rowwise_grouped_dynamic
 * (reference: csrc/gemm/gemm_ops.cpp:43-44, csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:656-714,
 * which marks the operator deprecated in favour of the stacked / offsets entry points above).
 */
int mslk_amd_f8f8bf16_rowwise_grouped_dynamic(const void* xq, const void* wq, const float* x_scale,
                                              const float* w_scale, const int64_t* zero_start_index_M_dev, int G,
                                              int64_t M, int64_t N, int64_t K, void* y, int zeroing_output,
                                              void* stream);

/*
 * Batched rowwise FP8 GEMM: Y[b] = bf16(XQ[b] . WQ[b]^T * x_scale[b][:,None] * w_scale[b][None,:] + bias[b]).
 * Replaces mslk::gemm::f8f8bf16_rowwise_batched (reference: csrc/gemm/gemm_ops.cpp:35-36,
 * csrc/gemm/ck/fp8_rowwise_batched/fp8_rowwise_batched_gemm.hip:199-254).
 *   xq [B, M, K], wq [B, N, K], x_scale [B, M], w_scale [B, N], bias NULL or [B, N] (layout of
 *   csrc/gemm/cutlass/f8f8bf16_rowwise_batched/f8f8bf16_rowwise_batched_common.cuh:272-275), y [B, M, N].
 */
int mslk_amd_f8f8bf16_rowwise_batched(const void* xq, const void* wq, const float* x_scale, const float* w_scale,
                                      const void* bias, int bias_dtype, int64_t B, int64_t M, int64_t N,
                                      int64_t K, void* y, void* stream);

/*
 * Self-test helper: converts n fp32 values to e4m3fn with the same device routine the quantizer
 * uses (hardware v_cvt_pk_fp8_f32 plus the NaN fix-up for |v| > 464).  Used by the parity tests to
 * sweep the conversion against the oracle; no counterpart in the reference.
 */
int mslk_amd_debug_cast_e4m3fn(const float* in, int64_t n, void* out, void* stream);

/*
 * Which kernel the dense entry points (mslk_amd_f8f8bf16_rowwise, mslk_amd_f8f8f16_rowwise, mslk_amd_f8f8_rowwise_preshuffle)
 * pick for a shape, as text ("dense_tiled<256,256,waves=2x2,ring=0> tiles=256", "skinny_lds<...>", "pad_rows + pad_rows +
 * dense_tiled<...>", ...), on aligned operands; with_workspace != 0 assumes the caller passes the workspace of
 * mslk_amd_f8f8bf16_rowwise_workspace_bytes.  A dry run of the real dispatch code on the current device (or, with no GPU,
 * for a whole MI355X): nothing is launched and no pointer is read.  Used by the tests to pin the shape classes of the
 * benchmark configurations; no counterpart in the reference, whose dispatch is a table of tuned instances
 * (csrc/gemm/ck/fp8_rowwise/fp8fp8bf16_rowwise_gemm.hip:158-468).  The returned string is thread-local and valid until
 * the next call on the same thread.
 */
const char* mslk_amd_debug_dispatch_name(int64_t M, int64_t N, int64_t K, int bias_dtype, int y_dtype, int preshuffled,
                                         int with_workspace);

/*
 * Ceiling probes for the benchmark's roofline columns; no counterpart in the reference (its bench divides by fixed
 * peak figures, bench/gemm/gemm_bench.py:61-68) and not part of the product path.
 *   mslk_amd_debug_stream_read: `workgroups` x 256 lanes read `bytes` from `src` once and write nothing.  mode 0: 16-byte
 *     non-temporal loads into registers (bytes % 16 == 0); mode 1: the global -> LDS DMA loads the GEMM kernels use
 *     (bytes % 1024 == 0); mode 2: the same with the non-temporal bit, as the kernels fetch weights that are read once.
 *     `sink` (device int, may be NULL) is never written for real inputs.
 *   mslk_amd_debug_mfma_loop: `workgroups` x 4 waves each run `iters` iterations of a 128 x 128 x 128 wave tile out of
 *     registers: 64 v_mfma_f32_16x16x128_f8f6f4 (form 0) or 32 v_mfma_f32_32x32x64_f8f6f4 (form 1) per iteration, i.e.
 *     iters * 2 * 128^3 FLOP per wave.  `operands` points at 128 KiB of e4m3 codes (32-byte aligned) that fill the operand
 *     registers once; the rate depends on these values through the power they draw.
 *   mslk_amd_debug_tile_streams: the global -> LDS loads of the 128 x 64 tile kernel's K loop and nothing else (no LDS
 *     reads, no multiplies, no output): tiles_m x tiles_n workgroups in the dense kernels' tile order, each fetching the
 *     128 rows of its row tile from x (tiles_m * 128 rows of K bytes, x_bytes in all) and / or its 64 weight rows from w
 *     (tiles_n * 64 rows, w_bytes), 128 bytes of K per step, five steps ahead.  which: 1 activations only, 2 weights
 *     only, 3 both.  K a multiple of 128.  The duration is what the memory system allows the tile kernel on operands of
 *     that shape.
 */
int mslk_amd_debug_stream_read(const void* src, int64_t bytes, int mode, int workgroups, void* sink, void* stream);
int mslk_amd_debug_mfma_loop(const void* operands, int form, int iters, int workgroups, void* sink, void* stream);
int mslk_amd_debug_tile_streams(const void* x, int64_t x_bytes, const void* w, int64_t w_bytes, int64_t K, int tiles_m, int tiles_n,
                                int which, void* stream);

/*
 * Where the time of one dense launch goes: the 256 x 256 tile kernel of mslk_amd_f8f8bf16_rowwise (one tile per
 * workgroup, last K step fused with the epilogue, bf16 output, no bias) built with four readings of the GPU's
 * constant-rate counter (100 MHz) per wave.  stamps[((workgroup * 4) + wave) * 4 + i], i = 0 kernel entry, 1 first
 * operands behind the first barrier, 2 the K loop hands its last step to the epilogue, 3 end of the epilogue (the wave's
 * stores may still be in flight).  Workgroup ids beyond the tile count (the grid is rounded up to a multiple of 8) write
 * nothing.  M, N multiples of 256, K a multiple of 128 and at least 256: every tile takes the interior path.  Y receives
 * the product.  `stamps` holds ceil(M/256 * N/256 / 8) * 8 * 16 values.  Not part of the product path; no counterpart in
 * the reference.
 */
int mslk_amd_debug_gemm_phases(const void* xq, const void* wq, const float* x_scale, const float* w_scale, void* y, int64_t M,
                               int64_t N, int64_t K, uint64_t* stamps, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MSLK_AMD_H_ */
