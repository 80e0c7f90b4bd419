/*
 * Scalar C twin of the FP8 rowwise oracle.  TEST INFRASTRUCTURE ONLY: nothing in the
 * product package links or loads this file; tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg are its only users.
 *
 * It restates, with integer/IEEE scalar arithmetic only (no torch, no libm beyond rintf),
 * what the reference's CPU torch branch computes:
 *
 *   oracle_quantize_rows   mslk/quantize/triton/fp8_quantize.py:360-378
 *                          row_max = max|a| in the input dtype (363); clamp(min=1e-12[,max=ub])
 *                          with both bounds rounded to the input dtype (365-369);
 *                          a_scale = 448 / row_max.f32, which PyTorch evaluates as
 *                          reciprocal(row_max) * 448 (371); inf -> 1.0 (372);
 *                          code = e4m3fn_rne(f32(a) * a_scale) (373-375); scale = 1 / a_scale (378).
 *   oracle_e4m3fn_from_f32 OCP FP8 E4M3 (fn variant: no inf, S.1111.111 = NaN), round to nearest
 *                          even, values that round beyond 448 become NaN (0x7F) -- the behaviour of
 *                          torch's float8_e4m3fn cast that line 375 relies on.
 *   oracle_dequant_gemm    test/gemm/triton/fp8_gemm_test.py:126-132 in float64, brute force.
 *
 * Pinned by tests/test_oracle.py: exhaustive comparison with torch's own cast and with the
 * torch restatement in fp8_rowwise_oracle.py, plus closed forms.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return u32_as_f32((uint32_t)h << 16); }

/* fp32 -> bf16 bits, round to nearest even, NaN kept quiet. */
static inline uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = f32_as_u32(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0) {
    /* zero / subnormal: man * 2^-24 is exact in fp32 */
    float v = (float)man * u32_as_f32(0x33800000u); /* 2^-24 */
    return u32_as_f32(f32_as_u32(v) | sign);
  }
  if (exp == 31) return u32_as_f32(sign | 0x7F800000u | (man << 13));
  return u32_as_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* double -> fp16 value (as float), round to nearest even; used only for the clamp bounds. */
static inline float f64_to_f16_value(double d) {
  if (d != d) return (float)d;
  double a = fabs(d);
  if (a >= 65520.0) return (float)(d < 0 ? -INFINITY : INFINITY);
  int e;
  (void)frexp(a, &e); /* a = m * 2^e, m in [0.5,1) */
  int q = e - 11;      /* 11 significant bits for normals */
  if (q < -24) q = -24; /* subnormal spacing 2^-24 */
  double r = ldexp(rint(ldexp(a, -q)), q);
  return (float)(d < 0 ? -r : r);
}

uint8_t oracle_e4m3fn_from_f32(float f) {
  uint32_t u = f32_as_u32(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t mag = u & 0x7FFFFFFFu;
  if (mag >= 0x43F00000u) return sign | 0x7Fu;          /* >= 480, inf, NaN */
  if (mag < 0x3C800000u) {                              /* < 2^-6: subnormal grid 2^-9 */
    float scaled = u32_as_f32(mag) * 512.0f;            /* exact */
    return sign | (uint8_t)rintf(scaled);               /* RNE; 8 -> 0x08 = 2^-6 */
  }
  /* normal: keep 3 mantissa bits, RNE on the 20 dropped bits, rebias 127 -> 7 */
  uint32_t r = mag + 0x7FFFFu + ((mag >> 20) & 1u);
  uint32_t code = (r >> 20) - ((127u - 7u) << 3);
  if (code > 0x7Fu) code = 0x7Fu;
  return sign | (uint8_t)code;                          /* (464,480) lands on 0x7F = NaN */
}

float oracle_e4m3fn_to_f32(uint8_t c) {
  uint32_t sign = (uint32_t)(c & 0x80u) << 24;
  uint32_t exp = (c >> 3) & 0xFu, man = c & 7u;
  float v;
  if (exp == 15 && man == 7) v = u32_as_f32(0x7FC00000u);
  else if (exp == 0) v = (float)man * 0.001953125f; /* 2^-9 */
  else v = u32_as_f32(((exp + 120u) << 23) | (man << 20));
  return u32_as_f32(f32_as_u32(v) | sign);
}

void oracle_e4m3fn_cast(const float* in, int64_t n, uint8_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_e4m3fn_from_f32(in[i]);
}

static inline float load_elem(const void* a, int dtype, int64_t i) {
  switch (dtype) {
    case 0: return bf16_to_f32(((const uint16_t*)a)[i]);
    case 1: return f16_to_f32(((const uint16_t*)a)[i]);
    default: return ((const float*)a)[i];
  }
}

/* dtype: 0 = bf16, 1 = fp16, 2 = fp32.  ub is read only when has_ub != 0.
 * out_stride >= K; columns [K, out_stride) are not touched. */
void oracle_quantize_rows(const void* a, int dtype, int64_t rows, int64_t K, int64_t in_stride,
                          int has_ub, double ub, uint8_t* out, int64_t out_stride, float* scale) {
  float eps, ubf = 0.0f;
  if (dtype == 0) {
    eps = bf16_to_f32(f32_to_bf16_rne((float)1e-12));
    if (has_ub) ubf = bf16_to_f32(f32_to_bf16_rne((float)ub));
  } else if (dtype == 1) {
    eps = f64_to_f16_value(1e-12);
    if (has_ub) ubf = f64_to_f16_value(ub);
  } else {
    eps = (float)1e-12;
    if (has_ub) ubf = (float)ub;
  }
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * in_stride;
    float amax = 0.0f;
    int has_nan = 0;
    for (int64_t k = 0; k < K; ++k) {
      float v = fabsf(load_elem(a, dtype, base + k));
      if (v != v) has_nan = 1;
      if (v > amax) amax = v;
    }
    if (has_nan) amax = NAN;
    if (amax == amax) {            /* clamp propagates NaN */
      if (amax < eps) amax = eps;
      if (has_ub && amax > ubf) amax = ubf;
    }
    float recip = 1.0f / amax;     /* correctly rounded */
    float inv = recip * 448.0f;
    if (inv == INFINITY) inv = 1.0f;
    for (int64_t k = 0; k < K; ++k) {
      float v = load_elem(a, dtype, base + k) * inv;
      out[r * out_stride + k] = oracle_e4m3fn_from_f32(v);
    }
    scale[r] = 1.0f / inv;
  }
}

/* y[m,n] = sum_k (xq[m,k]*xs[m]) * (wq[n,k]*ws[n]) + bias[n], float64 throughout. */
void oracle_dequant_gemm(const uint8_t* xq, const uint8_t* wq, const float* xs, const float* ws,
                         const float* bias, int64_t M, int64_t N, int64_t K, double* y) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += ((double)oracle_e4m3fn_to_f32(xq[m * K + k]) * (double)xs[m]) *
               ((double)oracle_e4m3fn_to_f32(wq[n * K + k]) * (double)ws[n]);
      y[m * N + n] = acc + (bias ? (double)bias[n] : 0.0);
    }
}

/*
 * Checker for a kernel optimisation, not a restatement of the reference: the quantizer's Triton-arithmetic mode needs
 * code = e4m3fn(clamp(x / s, -448, 448)) with an IEEE division (div_rn, mslk/quantize/triton/fp8_quantize.py:164-166),
 * s = fl32(c / 448), for every element x of a row whose maximum is c.  The kernel replaces the division by
 *     r = fl32(1 / s);  q0 = fl32(x * r);  e = fma(-q0, s, x);  q = e == 0 ? q0 : fma(e, r, q0)
 * (a handful of instructions per element instead of a division sequence; rows whose r is not finite keep the division).
 * This function walks EVERY pair (c, x) of 16-bit values of the given dtype (0 bf16, 1 fp16) with c finite and positive,
 * r finite and |x| <= c, and counts the pairs whose code differs between the two forms; `first_bad` / `last_bad`
 * receive the first and the last offending pair as (c bits << 16 | x bits); the walk covers c bits in
 * [first_c_bits, end_c_bits) (0 = from the smallest / to the largest finite value).
 */
uint64_t oracle_count_division_mismatches(int dtype, uint32_t first_c_bits, uint32_t end_c_bits, uint32_t* first_bad,
                                          uint32_t* last_bad) {
  uint64_t bad = 0;
  uint32_t top = dtype == 0 ? 0x7F80u : 0x7C00u;      /* first non-finite magnitude */
  if (end_c_bits > 0 && end_c_bits < top) top = end_c_bits;
  for (uint32_t cb = first_c_bits > 0 ? first_c_bits : 1; cb < top; ++cb) {
    const float c = dtype == 0 ? bf16_to_f32((uint16_t)cb) : f16_to_f32((uint16_t)cb);
    const float s = c / 448.0f;
    const float r = 1.0f / s;
    if (!(r <= 3.4028234663852886e38f)) continue;   /* r overflowed: the kernel divides in such rows */
    for (uint32_t xb = 0; xb <= cb; ++xb) {
      for (int sign = 0; sign < 2; ++sign) {
        const uint16_t bits = (uint16_t)(xb | (sign ? 0x8000u : 0u));
        const float x = dtype == 0 ? bf16_to_f32(bits) : f16_to_f32(bits);
        float want = x / s;
        const float q0 = x * r;
        const float e = fmaf(-q0, s, x);
        float got = e == 0.0f ? q0 : fmaf(e, r, q0);
        want = want < -448.0f ? -448.0f : (want > 448.0f ? 448.0f : want);
        got = got < -448.0f ? -448.0f : (got > 448.0f ? 448.0f : got);
        if (oracle_e4m3fn_from_f32(want) != oracle_e4m3fn_from_f32(got)) {
          if (bad == 0 && first_bad) *first_bad = (cb << 16) | bits;
          if (last_bad) *last_bad = (cb << 16) | bits;
          ++bad;
        }
      }
    }
  }
  return bad;
}
