// RMSNorm fused with the row-wise fp8 cast of its output.
//
// The blocks of the model normalise the residual stream and hand the result to
// wq / wk / wv or w1 / w3 (lingua/transformer.py:283-289 for the norm,
// :357-359 and :469-471 for the consumers).  Eagerly that is seven elementwise
// / reduction kernels with fp32 temporaries for the norm, then one pass of the
// row-wise cast per consuming linear (lingua/float8.py:86-87, :43-47).  Here the
// row is read once, normalised, written as bf16 (autograd and the wgrad casts
// need it) and quantised from registers:
//
//   r  = rsqrt(mean(f32(x)^2) + eps)
//   y  = bf16( (f32(x) * r) * f32(w) )            (the reference's op order)
//   q, scale = row-wise cast of y, [rstd = r], [column amaxes of y]
//
// Everything after r is exact elementwise arithmetic; r itself depends on the
// order of the fp32 sum of squares, which differs from ATen's reduction, so y
// can differ from the eager result in the last bf16 bit of an element now and
// then (the tests bound it: at most one bf16 ulp, > 99.5 % identical).
// One 256-thread workgroup per row, as the long-row cast kernel.
#include "l8_common.h"

namespace l8 {

constexpr int kNormBlock = 256;
constexpr int kNormWaves = kNormBlock / 64;

// sum over the 64 lanes of a wave, result uniform
L8_DEV float wave_sum_f32(float v) {
  auto step = [&](int moved) { v += __int_as_float(moved); };
  step(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  step(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  step(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, true));  // row_ror:4
  step(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true));  // row_ror:8
  const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (a + b) + (c + d);
}

template <int NCHW, bool COLMAX, bool W_F32>
__global__ __launch_bounds__(kNormBlock, 2) void rmsnorm_cast_rowwise_kernel(
    const uint16_t *__restrict__ x, const void *__restrict__ w, int64_t R, int C, int64_t ldx, float eps,
    uint16_t *__restrict__ y, int64_t ldy, uint8_t *__restrict__ q, int64_t ldq, float *__restrict__ scale,
    float *__restrict__ rstd, uint16_t *__restrict__ col_partials, int scale_rule) {
  __shared__ float red_ss[2][kNormWaves];
  __shared__ uint32_t red_mx[2][kNormWaves];
  extern __shared__ __attribute__((aligned(16))) uint8_t dyn_lds[];
  constexpr bool CLDS = COLMAX && colmax_in_lds<NCHW, 1>();
  v4i *lds_cm = (v4i *)dyn_lds;  // [C / 8]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  auto col_of = [&](int j) { return (j * kNormWaves + wave) * 512 + lane * 8; };
  uint32_t cmax[(COLMAX && !CLDS) ? NCHW * 4 : 1];
  if (COLMAX) {
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      if (CLDS) {
        if (col_of(j) < C) lds_cm[col_of(j) / 8] = v4i{0, 0, 0, 0};
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) cmax[j * 4 + k] = 0;
      }
    }
  }
  // the weights of this thread's columns stay in registers for all its rows
  float wf[NCHW][8];
#pragma unroll
  for (int j = 0; j < NCHW; ++j) {
    const int c = col_of(j);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (c < C) wf[j][e] = W_F32 ? ((const float *)w)[c + e] : bf16_bits_to_f32(((const uint16_t *)w)[c + e]);
      else wf[j][e] = 0.0f;
    }
  }
  const float inv_c = 1.0f / (float)C;
  int it = 0;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x, ++it) {
    v4i xv[NCHW];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      xv[j] = c < C ? __builtin_nontemporal_load((const v4i *)(x + r * ldx + c)) : v4i{0, 0, 0, 0};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float lo = __uint_as_float((uint32_t)xv[j][k] << 16), hi = __uint_as_float((uint32_t)xv[j][k] & 0xffff0000u);
        ss += lo * lo;
        ss += hi * hi;
      }
    }
    ss = wave_sum_f32(ss);
    if (lane == 0) red_ss[it & 1][wave] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kNormWaves; ++wv) tot += red_ss[it & 1][wv];
    const float rinv = 1.0f / sqrtf(tot * inv_c + eps);
    if (threadIdx.x == 0 && rstd) rstd[r] = rinv;

    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      v4i yv;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float lo = __uint_as_float((uint32_t)xv[j][k] << 16), hi = __uint_as_float((uint32_t)xv[j][k] & 0xffff0000u);
        const uint32_t ylo = bf16_rne_bits((lo * rinv) * wf[j][2 * k]);
        const uint32_t yhi = bf16_rne_bits((hi * rinv) * wf[j][2 * k + 1]);
        yv[k] = (int)(ylo | (yhi << 16));
        m = pk_absmax_u16(m, (uint32_t)yv[k]);
        if (COLMAX && !CLDS) cmax[j * 4 + k] = pk_absmax_u16(cmax[j * 4 + k], (uint32_t)yv[k]);
      }
      const int c = col_of(j);
      if (CLDS && c < C) {
        v4i old = lds_cm[c / 8];
#pragma unroll
        for (int k = 0; k < 4; ++k) old[k] = (int)pk_absmax_u16((uint32_t)old[k], (uint32_t)yv[k]);
        lds_cm[c / 8] = old;
      }
      if (c < C) __builtin_nontemporal_store(yv, (v4i *)(y + r * ldy + c));
      xv[j] = yv;  // the row of y replaces the row of x in registers
    }
    m = wave_max_u32(max(m & 0xffffu, m >> 16));
    if (lane == 0) red_mx[it & 1][wave] = m;
    __syncthreads();
    uint32_t amax_bits = 0;
#pragma unroll
    for (int wv = 0; wv < kNormWaves; ++wv) amax_bits = max(amax_bits, red_mx[it & 1][wv]);
    const RowScale rs = row_scale(amax_bits, scale_rule);
    if (threadIdx.x == 0 && scale) scale[r] = rs.s;
    if (q) {
      uint8_t *qrow = q + r * ldq;
#pragma unroll
      for (int j = 0; j < NCHW; ++j) {
        const int c = col_of(j);
        if (c < C) {
          if (rs.finite) __builtin_nontemporal_store(cvt8(xv[j], rs.recip), (v2i *)(qrow + c));
          else *(v2i *)(qrow + c) = cvt8_slow(xv[j], rs.recip);
        }
      }
    }
  }
  if (COLMAX) {
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      if (c < C)
        *(v4i *)(col_partials + (int64_t)blockIdx.x * C + c) =
            CLDS ? lds_cm[c / 8] : v4i{(int)cmax[j * 4], (int)cmax[j * 4 + 1], (int)cmax[j * 4 + 2], (int)cmax[j * 4 + 3]};
    }
  }
}

// Backward of the norm: with xhat = x * r and gh = gy * w,
//   gx = (gh - xhat * mean(gh * xhat)) * r        (bf16)
//   gw = sum over rows of gy * xhat               (fp32)
// One workgroup per row again; the row products for gw are accumulated in
// registers over all rows a workgroup sees and leave as one row of fp32
// partial sums per workgroup, which rmsnorm_gw_fold_kernel adds up column by
// column in a fixed order (no atomics: the result does not depend on timing).
template <int NCHW, bool W_F32>
__global__ __launch_bounds__(kNormBlock, 2) void rmsnorm_bwd_kernel(
    const uint16_t *__restrict__ gy, const uint16_t *__restrict__ x, const void *__restrict__ w,
    const float *__restrict__ rstd, int64_t R, int C, int64_t ldg, int64_t ldx, uint16_t *__restrict__ gx, int64_t ldgx,
    float *__restrict__ gw_partials) {
  __shared__ float red[2][kNormWaves];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  auto col_of = [&](int j) { return (j * kNormWaves + wave) * 512 + lane * 8; };
  float wf[NCHW][8], gwacc[NCHW][8];
#pragma unroll
  for (int j = 0; j < NCHW; ++j) {
    const int c = col_of(j);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      gwacc[j][e] = 0.0f;
      if (c < C) wf[j][e] = W_F32 ? ((const float *)w)[c + e] : bf16_bits_to_f32(((const uint16_t *)w)[c + e]);
      else wf[j][e] = 0.0f;
    }
  }
  const float inv_c = 1.0f / (float)C;
  int it = 0;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x, ++it) {
    const float rinv = rstd[r];
    float xh[NCHW][8], gh[NCHW][8];
    float dot = 0.0f;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      v4i xv = {0, 0, 0, 0}, gv = {0, 0, 0, 0};
      if (c < C) {
        xv = __builtin_nontemporal_load((const v4i *)(x + r * ldx + c));
        gv = __builtin_nontemporal_load((const v4i *)(gy + r * ldg + c));
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int e = 2 * k + half;
          const float xe = __uint_as_float(half ? ((uint32_t)xv[k] & 0xffff0000u) : ((uint32_t)xv[k] << 16));
          const float ge = __uint_as_float(half ? ((uint32_t)gv[k] & 0xffff0000u) : ((uint32_t)gv[k] << 16));
          xh[j][e] = xe * rinv;
          gh[j][e] = ge * wf[j][e];
          gwacc[j][e] += ge * xh[j][e];
          dot += gh[j][e] * xh[j][e];
        }
      }
    }
    dot = wave_sum_f32(dot);
    if (lane == 0) red[it & 1][wave] = dot;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kNormWaves; ++wv) tot += red[it & 1][wv];
    const float c1 = tot * inv_c;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      if (c < C) {
        v4i out;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const uint32_t lo = bf16_rne_bits((gh[j][2 * k] - xh[j][2 * k] * c1) * rinv);
          const uint32_t hi = bf16_rne_bits((gh[j][2 * k + 1] - xh[j][2 * k + 1] * c1) * rinv);
          out[k] = (int)(lo | (hi << 16));
        }
        __builtin_nontemporal_store(out, (v4i *)(gx + r * ldgx + c));
      }
    }
  }
#pragma unroll
  for (int j = 0; j < NCHW; ++j) {
    const int c = col_of(j);
    if (c < C) {
      float *dst = gw_partials + (int64_t)blockIdx.x * C + c;
      *(v4f *)dst = v4f{gwacc[j][0], gwacc[j][1], gwacc[j][2], gwacc[j][3]};
      *(v4f *)(dst + 4) = v4f{gwacc[j][4], gwacc[j][5], gwacc[j][6], gwacc[j][7]};
    }
  }
}

// gw[c] = sum over the partial rows.  A workgroup owns 32 columns; thread (tx, ty)
// adds slots ty, ty+8, ... of column tx, then the eight sums are added in order of ty.
__global__ __launch_bounds__(256) void rmsnorm_gw_fold_kernel(const float *__restrict__ partials, int n_slots, int C,
                                                              float *__restrict__ gw) {
  __shared__ float part[8][32];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + tx;
  float s = 0.0f;
  if (c < C)
    for (int sl = ty; sl < n_slots; sl += 8) s += partials[(int64_t)sl * C + c];
  part[ty][tx] = s;
  __syncthreads();
  if (ty == 0 && c < C) {
    float t = part[0][tx];
#pragma unroll
    for (int k = 1; k < 8; ++k) t += part[k][tx];
    gw[c] = t;
  }
}

static int64_t norm_blocks(int64_t R) {
  const int64_t cap = (int64_t)num_cus() * 2;
  return R < cap ? R : cap;
}

constexpr int64_t kNormMaxC = 4 * kNormWaves * 512;  // 8192: the weights of a thread's columns live in registers

template <int NCHW, bool W_F32>
static int launch_norm(const void *x, const void *w, int64_t R, int64_t C, int64_t ldx, float eps, void *y, int64_t ldy,
                       void *q, int64_t ldq, float *scale, float *rstd, float *col_amax, void *ws, hipStream_t st) {
  const int64_t blocks = norm_blocks(R);
  if (col_amax) {
    const size_t lds = colmax_in_lds<NCHW, 1>() ? (size_t)C * 2 : 0;
    hipLaunchKernelGGL((rmsnorm_cast_rowwise_kernel<NCHW, true, W_F32>), dim3((unsigned)blocks), dim3(kNormBlock), lds, st,
                       (const uint16_t *)x, w, R, (int)C, ldx, eps, (uint16_t *)y, ldy, (uint8_t *)q, ldq, scale, rstd,
                       (uint16_t *)ws, l8::scale_rule());
    L8_HIP(hipGetLastError());
    return fold_colmax(ws, blocks, C, col_amax, st);
  }
  hipLaunchKernelGGL((rmsnorm_cast_rowwise_kernel<NCHW, false, W_F32>), dim3((unsigned)blocks), dim3(kNormBlock), 0, st,
                     (const uint16_t *)x, w, R, (int)C, ldx, eps, (uint16_t *)y, ldy, (uint8_t *)q, ldq, scale, rstd,
                     (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

template <int NCHW, bool W_F32>
static int launch_norm_bwd(const void *gy, const void *x, const void *w, const float *rstd, int64_t R, int64_t C,
                           int64_t ldg, int64_t ldx, void *gx, int64_t ldgx, float *gw, void *ws, hipStream_t st) {
  const int64_t blocks = norm_blocks(R);
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<NCHW, W_F32>), dim3((unsigned)blocks), dim3(kNormBlock), 0, st,
                     (const uint16_t *)gy, (const uint16_t *)x, w, rstd, R, (int)C, ldg, ldx, (uint16_t *)gx, ldgx,
                     (float *)ws);
  L8_HIP(hipGetLastError());
  hipLaunchKernelGGL(rmsnorm_gw_fold_kernel, dim3((unsigned)((C + 31) / 32)), dim3(256), 0, st, (const float *)ws,
                     (int)blocks, (int)C, gw);
  L8_HIP(hipGetLastError());
  return L8_OK;
}

}  // namespace l8

using namespace l8;

extern "C" int64_t l8_rmsnorm_bwd_workspace(int64_t R, int64_t C) {
  if (R <= 0 || C <= 0) return 0;
  return norm_blocks(R) * C * (int64_t)sizeof(float);
}

extern "C" int l8_rmsnorm_bwd(const void *gy, const void *x, const void *w, int w_is_f32, const float *rstd, int64_t R,
                              int64_t C, int64_t ldg, int64_t ldx, void *gx, int64_t ldgx, float *gw, void *workspace,
                              int64_t workspace_bytes, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_rmsnorm_bwd: negative shape R=%lld C=%lld", (long long)R, (long long)C);
  if (C == 0) return L8_OK;
  L8_REQUIRE(gw, "l8_rmsnorm_bwd: null pointer");
  if (R == 0) {  // no rows: gw = 0, written by the fold kernel over zero partial rows
    hipLaunchKernelGGL(rmsnorm_gw_fold_kernel, dim3((unsigned)((C + 31) / 32)), dim3(256), 0, (hipStream_t)stream,
                       (const float *)nullptr, 0, (int)C, gw);
    L8_HIP(hipGetLastError());
    return L8_OK;
  }
  L8_REQUIRE(gy && x && w && rstd && gx, "l8_rmsnorm_bwd: null pointer");
  L8_REQUIRE(C % 8 == 0 && ldg % 8 == 0 && ldx % 8 == 0 && ldgx % 8 == 0 && ldg >= C && ldx >= C && ldgx >= C,
             "l8_rmsnorm_bwd: C=%lld and the leading dimensions must be multiples of 8 with ld >= C", (long long)C);
  L8_REQUIRE(((uintptr_t)gy % 16) == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)gx % 16) == 0,
             "l8_rmsnorm_bwd: gy, x and gx must be 16-byte aligned");
  L8_REQUIRE(C <= kNormMaxC, "l8_rmsnorm_bwd: C=%lld exceeds %lld", (long long)C, (long long)kNormMaxC);
  const int64_t need = l8_rmsnorm_bwd_workspace(R, C);
  L8_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0,
             "l8_rmsnorm_bwd: needs a 16-byte aligned workspace of %lld bytes", (long long)need);
  hipStream_t st = (hipStream_t)stream;
  const int64_t nchw = ((C + 511) / 512 + kNormWaves - 1) / kNormWaves;
#define L8_NORM_BWD(N)                                                                                               \
  return w_is_f32 ? launch_norm_bwd<N, true>(gy, x, w, rstd, R, C, ldg, ldx, gx, ldgx, gw, workspace, st)             \
                  : launch_norm_bwd<N, false>(gy, x, w, rstd, R, C, ldg, ldx, gx, ldgx, gw, workspace, st)
  if (nchw <= 1) L8_NORM_BWD(1);
  if (nchw <= 2) L8_NORM_BWD(2);
  L8_NORM_BWD(4);
#undef L8_NORM_BWD
}

extern "C" int64_t l8_rmsnorm_workspace(int64_t R, int64_t C) {
  if (R <= 0 || C <= 0) return 0;
  return norm_blocks(R) * C * (int64_t)sizeof(uint16_t);
}

extern "C" int l8_rmsnorm_cast_rowwise(const void *x, const void *w, int w_is_f32, int64_t R, int64_t C, int64_t ldx, float eps,
                                       void *y, int64_t ldy, void *q, int64_t ldq, float *scale, float *rstd,
                                       float *col_amax, void *workspace, int64_t workspace_bytes, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_rmsnorm_cast_rowwise: negative shape R=%lld C=%lld", (long long)R, (long long)C);
  if (R == 0 || C == 0) return L8_OK;
  L8_REQUIRE(x && w && y, "l8_rmsnorm_cast_rowwise: null pointer");
  L8_REQUIRE((q == nullptr) == (scale == nullptr), "l8_rmsnorm_cast_rowwise: pass q and scale together");
  L8_REQUIRE(C % 8 == 0 && ldx % 8 == 0 && ldy % 8 == 0 && ldx >= C && ldy >= C && (!q || (ldq % 8 == 0 && ldq >= C)),
             "l8_rmsnorm_cast_rowwise: C=%lld and the leading dimensions must be multiples of 8 with ld >= C", (long long)C);
  L8_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)q % 8) == 0,
             "l8_rmsnorm_cast_rowwise: x and y must be 16-byte aligned and q 8-byte aligned");
  L8_REQUIRE(C <= kNormMaxC, "l8_rmsnorm_cast_rowwise: C=%lld exceeds %lld", (long long)C, (long long)kNormMaxC);
  L8_REQUIRE(!col_amax || q, "l8_rmsnorm_cast_rowwise: column amaxes come with the cast");
  if (col_amax) {
    const int64_t need = l8_rmsnorm_workspace(R, C);
    L8_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0,
               "l8_rmsnorm_cast_rowwise: col_amax needs a 16-byte aligned workspace of %lld bytes", (long long)need);
  }
  hipStream_t st = (hipStream_t)stream;
  const int64_t nchw = ((C + 511) / 512 + kNormWaves - 1) / kNormWaves;
#define L8_NORM(N)                                                                                                        \
  return w_is_f32 ? launch_norm<N, true>(x, w, R, C, ldx, eps, y, ldy, q, ldq, scale, rstd, col_amax, workspace, st)      \
                  : launch_norm<N, false>(x, w, R, C, ldx, eps, y, ldy, q, ldq, scale, rstd, col_amax, workspace, st)
  if (nchw <= 1) L8_NORM(1);
  if (nchw <= 2) L8_NORM(2);
  L8_NORM(4);
#undef L8_NORM
}
