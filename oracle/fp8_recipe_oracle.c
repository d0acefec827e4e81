/*
 * CPU oracle for the row-wise float8 linear recipe.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the parity tests,
 * the smoke test and the cpu_baseline leg of the benchmark compare the HIP
 * kernels against.  Nothing in the shipped package may call it, link it or
 * fall back to it.
 *
 * It restates, in plain C with integer bit arithmetic where rounding matters,
 * the algorithm of the reference file lingua/float8.py:
 *   - scale floor EPS                         lingua/float8.py:11
 *   - tile-broadcast multiply (row / tensor)  lingua/float8.py:24-30
 *   - scale(t, amax): s = max(f32(amax),EPS)/448 ; q = e4m3fn(t * (1/s))
 *                                             lingua/float8.py:43-47
 *     (the quotient as ATen's CPU kernel rounds it, or, under l8o_set_scale_rule(1), as ATen's GPU kernel does)
 *   - matmul(): NT product of the two quantised operands, fp32 accumulation,
 *     scales applied to the product, optional bias, bf16 result
 *                                             lingua/float8.py:50-79
 *   - row amax in bf16, NaN propagating       lingua/float8.py:86-87,112-114
 *   - tensor amax of the weight from its saved row amaxes
 *                                             lingua/float8.py:115-118
 *   - grad_bias = column sum of grad_out      lingua/float8.py:127
 * The fp32 -> float8_e4m3fn conversion itself lives in PyTorch
 * (aten::_to_copy, pinned torch==2.7.0 by setup/create_env.sh:35); its
 * published behaviour (OCP FP8 E4M3 "fn": no inf, 0x7F/0xFF = NaN, round to
 * nearest even, subnormals down to 2^-9, magnitudes >= 480 and NaN/inf give
 * NaN, 448 < |v| <= 464 rounds to 448) is restated below as integer code.
 *
 * Pinning (see tests/test_oracle_*.py): the cast against torch's CPU library
 * routine and against a brute-force nearest-value search over the 256 decoded
 * codes; the scale against numpy float32 division over every non-negative
 * bf16 amax; amax / transposed / tensor-wise variants by reduction to the
 * row-wise case; the product against an fp64 triple loop and exact integer
 * matmuls.  No function here is "parity unpinned" except the accumulation
 * order of the H100 _scaled_mm kernel, which nothing available can pin and
 * which the rel-L2 <= 1e-3 tolerance on bf16 outputs supersedes.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define L8O_EXPORT __attribute__((visibility("default")))

static inline float bits_to_f32(uint32_t w) { float f; memcpy(&f, &w, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t w; memcpy(&w, &f, 4); return w; }
static inline float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even, NaN kept quiet (what Tensor.bfloat16() does). */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t w = f32_to_bits(f);
  if ((w & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((w >> 16) | 0x0040u);
  uint32_t keep_odd = (w >> 16) & 1u;
  w += 0x7fffu + keep_odd;
  return (uint16_t)(w >> 16);
}

/* fp32 bits -> OCP e4m3fn byte.  Integer only.
 * e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; normal range 2^-6 .. 448;
 * subnormal step 2^-9; S.1111.111 is NaN; there is no infinity. */
L8O_EXPORT uint8_t l8o_e4m3fn_from_f32_bits(uint32_t w) {
  const uint8_t sign = (uint8_t)((w >> 24) & 0x80u);
  const uint32_t mag = w & 0x7fffffffu;
  /* 480.0f = 0x43F00000 is where rounding would land on the NaN code or beyond;
   * infinities and NaNs compare above it as integers. */
  if (mag >= 0x43F00000u) return (uint8_t)(sign | 0x7Fu);
  const int e = (int)(mag >> 23);            /* biased fp32 exponent */
  const uint32_t frac = mag & 0x7fffffu;
  if (e >= 121) {                             /* |v| >= 2^-6 : fp8 normal */
    /* drop 20 fraction bits with ties-to-even; a carry walks into the exponent
     * field, which is exactly the next binade. */
    uint32_t t = ((uint32_t)(e - 120) << 23) | frac;   /* fp8 exponent field = e-120 */
    uint32_t lsb = (t >> 20) & 1u;
    t += 0x7ffffu + lsb;
    return (uint8_t)(sign | (t >> 20));
  }
  /* subnormal target: count of 2^-9 units, 0..8 (8 is the code of 2^-6). */
  if (e < 127 - 11) return sign;              /* |v| < 2^-11 : below half a unit */
  /* significand with hidden bit, value = sig * 2^(e-150) ; units = value * 2^9
   * => shift right by (141 - e) bits, 21 <= shift <= 25. */
  const uint32_t sig = frac | 0x800000u;
  const int sh = 141 - e;
  uint32_t q = sig >> sh;
  const uint32_t rem = sig & ((1u << sh) - 1u);
  const uint32_t half = 1u << (sh - 1);
  if (rem > half || (rem == half && (q & 1u))) q += 1;
  return (uint8_t)(sign | q);
}

L8O_EXPORT float l8o_e4m3fn_to_f32(uint8_t b) {
  const int e = (b >> 3) & 0xF, m = b & 7;
  float v;
  if (e == 0xF && m == 7) v = NAN;
  else if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf((float)(8 + m), e - 10);
  return (b & 0x80) ? -v : v;
}

/* scale = clamp(f32(amax), min=EPS) / 448  -- lingua/float8.py:44-45.
 * torch.clamp keeps NaN.  Rule 0 (default): the division is a correctly rounded fp32 division, which is what
 * ATen's CPU kernel computes.  Rule 1: ATen's GPU kernel divides a tensor by a Python scalar by multiplying with
 * the scalar's fp32 reciprocal, so the reference run on a GPU computes amax * fp32(1/448); the product differs
 * from the quotient in the last bit for about half of all amaxes.  (Pinned on the GPU against PyTorch's own
 * kernel over every bf16 amax, and here against numpy float32 arithmetic.) */
static int g_scale_rule = 0;
L8O_EXPORT void l8o_set_scale_rule(int rule) { g_scale_rule = rule; }
L8O_EXPORT int l8o_get_scale_rule(void) { return g_scale_rule; }
L8O_EXPORT float l8o_scale_from_amax(uint16_t amax_bf16) {
  volatile float a = bf16_to_f32(amax_bf16);
  const float eps = 1e-12f;
  if (a < eps) a = eps;                       /* false for NaN: NaN passes through */
  if (g_scale_rule == 1) {
    volatile float one = 1.0f, max = 448.0f;
    volatile float inv = one / max;
    volatile float s = a * inv;
    return s;
  }
  volatile float s = a / 448.0f;
  return s;
}

/* |x| max in bf16, NaN propagating (Tensor.abs().amax()). Returns bf16 bits. */
static inline uint16_t amax_step(uint16_t acc, uint16_t x) {
  uint16_t m = x & 0x7fffu;
  int acc_nan = acc > 0x7f80u, m_nan = m > 0x7f80u;
  if (acc_nan) return acc;
  if (m_nan) return m;
  return m > acc ? m : acc;                   /* non-negative bf16 order == integer order */
}

L8O_EXPORT void l8o_row_amax(const uint16_t *x, int64_t R, int64_t C, int64_t ldx, uint16_t *amax) {
  for (int64_t r = 0; r < R; ++r) {
    uint16_t a = 0;
    for (int64_t c = 0; c < C; ++c) a = amax_step(a, x[r * ldx + c]);
    amax[r] = a;
  }
}

L8O_EXPORT void l8o_col_amax(const uint16_t *x, int64_t R, int64_t C, int64_t ldx, uint16_t *amax) {
  for (int64_t c = 0; c < C; ++c) amax[c] = 0;
  for (int64_t r = 0; r < R; ++r)
    for (int64_t c = 0; c < C; ++c) amax[c] = amax_step(amax[c], x[r * ldx + c]);
}

/* weight tensor amax from the saved per-row amaxes -- lingua/float8.py:115-118 */
L8O_EXPORT uint16_t l8o_amax_of_amaxes(const uint16_t *amax, int64_t n) {
  uint16_t a = 0;
  for (int64_t i = 0; i < n; ++i) a = amax_step(a, amax[i]);
  return a;
}

/* q = e4m3fn( f32(x) * (1/s) ): reciprocal and product each rounded to fp32
 * (lingua/float8.py:46; mul_tiled promotes bf16 x fp32 to fp32). */
static inline uint8_t quant1(uint16_t x, float recip) {
  volatile float p = bf16_to_f32(x) * recip;
  return l8o_e4m3fn_from_f32_bits(f32_to_bits(p));
}

static inline float recip_of(float s) { volatile float r = 1.0f / s; return r; }

/* Row-wise scale(): one amax per row.  q[R,C] row-major (ldq), scale[R], amax_out[R] bf16 (may be NULL). */
L8O_EXPORT void l8o_cast_rowwise(const uint16_t *x, int64_t R, int64_t C, int64_t ldx,
                                 uint8_t *q, int64_t ldq, float *scale, uint16_t *amax_out) {
  for (int64_t r = 0; r < R; ++r) {
    uint16_t a = 0;
    for (int64_t c = 0; c < C; ++c) a = amax_step(a, x[r * ldx + c]);
    const float s = l8o_scale_from_amax(a);
    const float rs = recip_of(s);
    for (int64_t c = 0; c < C; ++c) q[r * ldq + c] = quant1(x[r * ldx + c], rs);
    scale[r] = s;
    if (amax_out) amax_out[r] = a;
  }
}

/* Tensor-wise scale(): a (1,1) amax is one tile covering the whole tensor
 * (lingua/float8.py:24-30).  transpose!=0 writes q as [C,R] (the layout of
 * b = b_t.t().contiguous(), lingua/float8.py:111). */
L8O_EXPORT void l8o_cast_tensorwise(const uint16_t *x, int64_t R, int64_t C, int64_t ldx,
                                    uint16_t amax_bf16, int transpose,
                                    uint8_t *q, int64_t ldq, float *scale) {
  const float s = l8o_scale_from_amax(amax_bf16);
  const float rs = recip_of(s);
  for (int64_t r = 0; r < R; ++r)
    for (int64_t c = 0; c < C; ++c) {
      uint8_t b = quant1(x[r * ldx + c], rs);
      if (transpose) q[c * ldq + r] = b; else q[r * ldq + c] = b;
    }
  *scale = s;
}

/* scale(t.t().contiguous(), row amax of that): amax down each column of x,
 * output q[C,R] (ldq), scale[C].  amax_in (bf16[C]) may be NULL -> computed here. */
L8O_EXPORT void l8o_cast_colwise_transposed(const uint16_t *x, int64_t R, int64_t C, int64_t ldx,
                                            const uint16_t *amax_in,
                                            uint8_t *q, int64_t ldq, float *scale) {
  for (int64_t c = 0; c < C; ++c) {
    uint16_t a = 0;
    if (amax_in) a = amax_in[c];
    else for (int64_t r = 0; r < R; ++r) a = amax_step(a, x[r * ldx + c]);
    const float s = l8o_scale_from_amax(a);
    const float rs = recip_of(s);
    for (int64_t r = 0; r < R; ++r) q[c * ldq + r] = quant1(x[r * ldx + c], rs);
    scale[c] = s;
  }
}

/* out[M,N] = bf16( sum_k deq(A[m,k]) * deq(B[n,k]) * sa * sb + bias[n] ), fp32 accumulation.
 * sa_n / sb_n: number of scale entries (M or 1, N or 1).  bias: bf16[N] or NULL.
 * The product of the two e4m3 values is exact in fp32 (8 significant bits);
 * only the running sum rounds. */
L8O_EXPORT void l8o_gemm_nt(const uint8_t *A, const uint8_t *B, int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb,
                            const float *sa, int64_t sa_n, const float *sb, int64_t sb_n,
                            const uint16_t *bias, uint16_t *out, int64_t ldc) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = l8o_e4m3fn_to_f32((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float arow[4096];
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t k0 = 0; k0 < K; k0 += 4096) {
        int64_t kn = K - k0 < 4096 ? K - k0 : 4096;
        if (n == 0 || K > 4096) for (int64_t k = 0; k < kn; ++k) arow[k] = lut[A[m * lda + k0 + k]];
        const uint8_t *b = B + n * ldb + k0;
        float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int64_t k = 0;
        for (; k + 8 <= kn; k += 8)
          for (int j = 0; j < 8; ++j) part[j] += arow[k + j] * lut[b[k + j]];
        for (; k < kn; ++k) part[0] += arow[k] * lut[b[k]];
        acc += ((part[0] + part[4]) + (part[1] + part[5])) + ((part[2] + part[6]) + (part[3] + part[7]));
      }
      float v = acc * sa[sa_n == 1 ? 0 : m] * sb[sb_n == 1 ? 0 : n];
      if (bias) v += bf16_to_f32(bias[n]);
      out[m * ldc + n] = f32_to_bf16(v);
    }
  }
}

/* Same product accumulated in fp64, result left in fp64 (no bf16 rounding):
 * the brute-force triple loop the fp32 version is pinned against. */
L8O_EXPORT void l8o_gemm_nt_f64(const uint8_t *A, const uint8_t *B, int64_t M, int64_t N, int64_t K,
                                int64_t lda, int64_t ldb,
                                const float *sa, int64_t sa_n, const float *sb, int64_t sb_n,
                                const uint16_t *bias, double *out, int64_t ldc) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += (double)l8o_e4m3fn_to_f32(A[m * lda + k]) * (double)l8o_e4m3fn_to_f32(B[n * ldb + k]);
      acc *= (double)sa[sa_n == 1 ? 0 : m] * (double)sb[sb_n == 1 ? 0 : n];
      if (bias) acc += (double)bf16_to_f32(bias[n]);
      out[m * ldc + n] = acc;
    }
}

/* grad_bias = grad_out.sum(0) in fp32 then bf16 -- lingua/float8.py:127 */
L8O_EXPORT void l8o_col_sum(const uint16_t *g, int64_t R, int64_t C, int64_t ldg, uint16_t *out) {
  for (int64_t c = 0; c < C; ++c) {
    float acc = 0.0f;
    for (int64_t r = 0; r < R; ++r) acc += bf16_to_f32(g[r * ldg + c]);
    out[c] = f32_to_bf16(acc);
  }
}

L8O_EXPORT uint16_t l8o_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* array forms of the scalar routines, for exhaustive tests */
L8O_EXPORT void l8o_e4m3fn_from_f32_array(const uint32_t *w, int64_t n, uint8_t *out) {
  for (int64_t i = 0; i < n; ++i) out[i] = l8o_e4m3fn_from_f32_bits(w[i]);
}

L8O_EXPORT void l8o_scale_from_amax_array(const uint16_t *amax, int64_t n, float *out) {
  for (int64_t i = 0; i < n; ++i) out[i] = l8o_scale_from_amax(amax[i]);
}
