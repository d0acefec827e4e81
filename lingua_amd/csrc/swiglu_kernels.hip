// SwiGLU gate fused with the row-wise fp8 cast, forward and backward.
//
// The MLP of lingua/transformer.py:430-471 computes w2(silu(w1(x)) * w3(x)).
// Between the GEMMs sit bf16 elementwise passes (silu, mul; in backward two
// muls and silu_backward) and, with the float8 recipe, the casts of the w2
// input and of the two gate gradients (lingua/float8.py:86-87, :43-47).  Each
// of those passes streams a [tokens, ffn] tensor through HBM.  The kernels
// below do the elementwise arithmetic while the row is in registers for its
// amax and cast anyway:
//
//   forward : h  = bf16(bf16(silu(h1)) * h3)          -> q(h), scale, [h], [col amax]
//   backward: g3 = bf16(dh * bf16(silu(h1)))
//             g1 = bf16(bf16(dh * h3) * sig * (1 + h1 * (1 - sig)))
//                                                      -> g1, g3, q(g1), q(g3), scales, [col amaxes]
//
// Every intermediate is rounded to bf16 where the unfused PyTorch chain
// materialises a bf16 tensor, so the results agree with that chain up to the
// last bits of the fp32 sigmoid: at most two bf16 ulps apart, identical for
// more than 99.5 % of the elements (the bound the tests state); amax, scale
// and e4m3 bytes are then exact functions of the bf16 values produced here.
// One 256-thread workgroup per row (wave
// w owns the 512-column chunks w, w+4, ...), the layout of the long-row kernel
// of cast_kernels.hip; the amax -> scale -> cast stage is shared with it.
#include "l8_common.h"

namespace l8 {

constexpr int kGateBlock = 256;
constexpr int kGateWaves = kGateBlock / 64;

// 1 / (1 + exp(-x)) with the hardware exp2 and reciprocal (about 1 ulp of fp32
// each).  The library exp and the IEEE division cost ~5x the instructions and
// made these kernels VALU-bound (302 us forward / 550 us backward on
// [16384, 11008] against ~230 / ~400 us of memory time); every result is
// rounded to bf16 right away, where an fp32 ulp decides one rounding in ~10^4.
L8_DEV float sigmoid_f32(float x) {
  const float e = __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
  return __builtin_amdgcn_rcpf(1.0f + e);
}
// silu(x) = x / (1 + exp(-x)), fp32
L8_DEV float silu_f32(float x) { return x * sigmoid_f32(x); }

// one element of the forward gate
L8_DEV uint32_t gate_fwd(float a, float b) { return bf16_rne_bits(bf16_round(silu_f32(a)) * b); }

// two packed bf16 of h1 and h3 -> two packed bf16 of h
L8_DEV uint32_t gate_fwd2(uint32_t a, uint32_t b) {
  const uint32_t lo = gate_fwd(__uint_as_float(a << 16), __uint_as_float(b << 16));
  const uint32_t hi = gate_fwd(__uint_as_float(a & 0xffff0000u), __uint_as_float(b & 0xffff0000u));
  return lo | (hi << 16);
}

// one element of the backward gate: d = dh, a = h1, b = h3
L8_DEV void gate_bwd(float d, float a, float b, uint32_t &g1, uint32_t &g3) {
  const float sig = sigmoid_f32(a);
  const float s = bf16_round(a * sig);          // what forward saved: bf16 silu(h1)
  const float gs = bf16_round(d * b);           // gradient of the silu output, a bf16 tensor in the unfused chain
  g3 = bf16_rne_bits(d * s);
  g1 = bf16_rne_bits((gs * sig) * (1.0f + a * (1.0f - sig)));
}
L8_DEV void gate_bwd2(uint32_t d, uint32_t a, uint32_t b, uint32_t &g1, uint32_t &g3) {
  uint32_t g1l, g3l, g1h, g3h;
  gate_bwd(__uint_as_float(d << 16), __uint_as_float(a << 16), __uint_as_float(b << 16), g1l, g3l);
  gate_bwd(__uint_as_float(d & 0xffff0000u), __uint_as_float(a & 0xffff0000u), __uint_as_float(b & 0xffff0000u), g1h, g3h);
  g1 = g1l | (g1h << 16);
  g3 = g3l | (g3h << 16);
}

template <int NCHW, bool COLMAX>
__global__ __launch_bounds__(kGateBlock, 2) void swiglu_cast_rowwise_kernel(
    const uint16_t *__restrict__ h1, const uint16_t *__restrict__ h3, int64_t R, int C, int64_t ld1, int64_t ld3,
    uint16_t *__restrict__ hout, int64_t ldh, uint8_t *__restrict__ q, int64_t ldq, float *__restrict__ scale,
    uint16_t *__restrict__ amax_out, uint16_t *__restrict__ col_partials, int scale_rule) {
  __shared__ uint32_t red[2][kGateWaves];
  extern __shared__ __attribute__((aligned(16))) uint8_t dyn_lds[];
  constexpr bool CLDS = COLMAX && colmax_in_lds<NCHW, 1>();
  v4i *lds_cm = (v4i *)dyn_lds;  // [C / 8]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  auto col_of = [&](int j) { return (j * kGateWaves + wave) * 512 + lane * 8; };
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
  int it = 0;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x, ++it) {
    v4i a[NCHW], b[NCHW], h[NCHW];
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      if (c < C) {
        a[j] = __builtin_nontemporal_load((const v4i *)(h1 + r * ld1 + c));
        b[j] = __builtin_nontemporal_load((const v4i *)(h3 + r * ld3 + c));
      } else {
        a[j] = v4i{0, 0, 0, 0};
        b[j] = v4i{0, 0, 0, 0};
      }
    }
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        h[j][k] = (int)gate_fwd2((uint32_t)a[j][k], (uint32_t)b[j][k]);
        m = pk_absmax_u16(m, (uint32_t)h[j][k]);
        if (COLMAX && !CLDS) cmax[j * 4 + k] = pk_absmax_u16(cmax[j * 4 + k], (uint32_t)h[j][k]);
      }
      const int c = col_of(j);
      if (CLDS && c < C) {
        v4i old = lds_cm[c / 8];
#pragma unroll
        for (int k = 0; k < 4; ++k) old[k] = (int)pk_absmax_u16((uint32_t)old[k], (uint32_t)h[j][k]);
        lds_cm[c / 8] = old;
      }
      if (hout && c < C) __builtin_nontemporal_store(h[j], (v4i *)(hout + r * ldh + c));
    }
    m = wave_max_u32(max(m & 0xffffu, m >> 16));
    if (lane == 0) red[it & 1][wave] = m;
    __syncthreads();
    uint32_t amax_bits = 0;
#pragma unroll
    for (int w = 0; w < kGateWaves; ++w) amax_bits = max(amax_bits, red[it & 1][w]);
    const RowScale rs = row_scale(amax_bits, scale_rule);
    if (threadIdx.x == 0) {
      if (scale) scale[r] = rs.s;
      if (amax_out) amax_out[r] = (uint16_t)amax_bits;
    }
    if (q) {
      uint8_t *qrow = q + r * ldq;
#pragma unroll
      for (int j = 0; j < NCHW; ++j) {
        const int c = col_of(j);
        if (c < C) {
          if (rs.finite) __builtin_nontemporal_store(cvt8(h[j], rs.recip), (v2i *)(qrow + c));
          else *(v2i *)(qrow + c) = cvt8_slow(h[j], rs.recip);
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

template <int NCHW, bool COLMAX>
__global__ __launch_bounds__(kGateBlock, 2) void swiglu_bwd_cast_rowwise_kernel(
    const uint16_t *__restrict__ dh, const uint16_t *__restrict__ h1, const uint16_t *__restrict__ h3, int64_t R, int C,
    int64_t lddh, int64_t ld1, int64_t ld3, uint16_t *__restrict__ g1out, uint16_t *__restrict__ g3out, int64_t ldg,
    uint8_t *__restrict__ q1, uint8_t *__restrict__ q3, int64_t ldq, float *__restrict__ scale1,
    float *__restrict__ scale3, uint16_t *__restrict__ col_partials1, uint16_t *__restrict__ col_partials3, int scale_rule) {
  __shared__ uint32_t red[2][2][kGateWaves];
  extern __shared__ __attribute__((aligned(16))) uint8_t dyn_lds[];
  constexpr bool CLDS = COLMAX && colmax_in_lds<NCHW, 2>();
  v4i *lds_cm1 = (v4i *)dyn_lds, *lds_cm3 = lds_cm1 + C / 8;  // [C / 8] each
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  auto col_of = [&](int j) { return (j * kGateWaves + wave) * 512 + lane * 8; };
  uint32_t cmax1[(COLMAX && !CLDS) ? NCHW * 4 : 1], cmax3[(COLMAX && !CLDS) ? NCHW * 4 : 1];
  if (COLMAX) {
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      if (CLDS) {
        if (col_of(j) < C) lds_cm1[col_of(j) / 8] = lds_cm3[col_of(j) / 8] = v4i{0, 0, 0, 0};
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) cmax1[j * 4 + k] = cmax3[j * 4 + k] = 0;
      }
    }
  }
  int it = 0;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x, ++it) {
    v4i g1[NCHW], g3[NCHW];
    uint32_t m1 = 0, m3 = 0;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      v4i d = {0, 0, 0, 0}, a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
      if (c < C) {
        d = __builtin_nontemporal_load((const v4i *)(dh + r * lddh + c));
        a = __builtin_nontemporal_load((const v4i *)(h1 + r * ld1 + c));
        b = __builtin_nontemporal_load((const v4i *)(h3 + r * ld3 + c));
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        uint32_t x1, x3;
        gate_bwd2((uint32_t)d[k], (uint32_t)a[k], (uint32_t)b[k], x1, x3);
        g1[j][k] = (int)x1;
        g3[j][k] = (int)x3;
        m1 = pk_absmax_u16(m1, x1);
        m3 = pk_absmax_u16(m3, x3);
        if (COLMAX && !CLDS) {
          cmax1[j * 4 + k] = pk_absmax_u16(cmax1[j * 4 + k], x1);
          cmax3[j * 4 + k] = pk_absmax_u16(cmax3[j * 4 + k], x3);
        }
      }
      if (CLDS && c < C) {
        v4i o1 = lds_cm1[c / 8], o3 = lds_cm3[c / 8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          o1[k] = (int)pk_absmax_u16((uint32_t)o1[k], (uint32_t)g1[j][k]);
          o3[k] = (int)pk_absmax_u16((uint32_t)o3[k], (uint32_t)g3[j][k]);
        }
        lds_cm1[c / 8] = o1;
        lds_cm3[c / 8] = o3;
      }
      if (c < C) {
        __builtin_nontemporal_store(g1[j], (v4i *)(g1out + r * ldg + c));
        __builtin_nontemporal_store(g3[j], (v4i *)(g3out + r * ldg + c));
      }
    }
    m1 = wave_max_u32(max(m1 & 0xffffu, m1 >> 16));
    m3 = wave_max_u32(max(m3 & 0xffffu, m3 >> 16));
    if (lane == 0) {
      red[it & 1][0][wave] = m1;
      red[it & 1][1][wave] = m3;
    }
    __syncthreads();
    uint32_t bits1 = 0, bits3 = 0;
#pragma unroll
    for (int w = 0; w < kGateWaves; ++w) {
      bits1 = max(bits1, red[it & 1][0][w]);
      bits3 = max(bits3, red[it & 1][1][w]);
    }
    const RowScale rs1 = row_scale(bits1, scale_rule), rs3 = row_scale(bits3, scale_rule);
    if (threadIdx.x == 0) {
      scale1[r] = rs1.s;
      scale3[r] = rs3.s;
    }
    uint8_t *q1row = q1 + r * ldq, *q3row = q3 + r * ldq;
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      if (c < C) {
        if (rs1.finite) __builtin_nontemporal_store(cvt8(g1[j], rs1.recip), (v2i *)(q1row + c));
        else *(v2i *)(q1row + c) = cvt8_slow(g1[j], rs1.recip);
        if (rs3.finite) __builtin_nontemporal_store(cvt8(g3[j], rs3.recip), (v2i *)(q3row + c));
        else *(v2i *)(q3row + c) = cvt8_slow(g3[j], rs3.recip);
      }
    }
  }
  if (COLMAX) {
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      if (c < C) {
        *(v4i *)(col_partials1 + (int64_t)blockIdx.x * C + c) =
            CLDS ? lds_cm1[c / 8] : v4i{(int)cmax1[j * 4], (int)cmax1[j * 4 + 1], (int)cmax1[j * 4 + 2], (int)cmax1[j * 4 + 3]};
        *(v4i *)(col_partials3 + (int64_t)blockIdx.x * C + c) =
            CLDS ? lds_cm3[c / 8] : v4i{(int)cmax3[j * 4], (int)cmax3[j * 4 + 1], (int)cmax3[j * 4 + 2], (int)cmax3[j * 4 + 3]};
      }
    }
  }
}

// Wide rows (ffn dimensions beyond what a 256-thread workgroup holds in
// registers without spilling): 1024 threads per row, two passes.  Pass 1
// computes the gate, stores the bf16 result and reduces the row amax; pass 2
// reads the thread's own bf16 values back (they are still in L2) and casts.
// Column maxima live in LDS (one bf16 per column and tensor, each owned by one
// thread).  Any C that is a multiple of 8.
constexpr int kWideBlock = 1024;
constexpr int kWideWaves = kWideBlock / 64;

template <bool COLMAX>
__global__ __launch_bounds__(kWideBlock) void swiglu_cast_rowwise_wide_kernel(
    const uint16_t *__restrict__ h1, const uint16_t *__restrict__ h3, int64_t R, int C, int64_t ld1, int64_t ld3,
    uint16_t *__restrict__ hout, int64_t ldh, uint8_t *__restrict__ q, int64_t ldq, float *__restrict__ scale,
    uint16_t *__restrict__ amax_out, uint16_t *__restrict__ col_partials, int scale_rule) {
  __shared__ uint32_t red[2][kWideWaves];
  extern __shared__ __attribute__((aligned(16))) uint8_t dyn_lds[];
  v4i *lds_cm = (v4i *)dyn_lds;  // [C / 8]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (COLMAX)
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) lds_cm[c / 8] = v4i{0, 0, 0, 0};
  int it = 0;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x, ++it) {
    uint32_t m = 0;
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) {
      const v4i a = __builtin_nontemporal_load((const v4i *)(h1 + r * ld1 + c));
      const v4i b = __builtin_nontemporal_load((const v4i *)(h3 + r * ld3 + c));
      v4i h;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        h[k] = (int)gate_fwd2((uint32_t)a[k], (uint32_t)b[k]);
        m = pk_absmax_u16(m, (uint32_t)h[k]);
      }
      if (COLMAX) {
        v4i old = lds_cm[c / 8];
#pragma unroll
        for (int k = 0; k < 4; ++k) old[k] = (int)pk_absmax_u16((uint32_t)old[k], (uint32_t)h[k]);
        lds_cm[c / 8] = old;
      }
      if (hout) *(v4i *)(hout + r * ldh + c) = h;
    }
    m = wave_max_u32(max(m & 0xffffu, m >> 16));
    if (lane == 0) red[it & 1][wave] = m;
    __syncthreads();
    uint32_t amax_bits = 0;
#pragma unroll
    for (int w = 0; w < kWideWaves; ++w) amax_bits = max(amax_bits, red[it & 1][w]);
    const RowScale rs = row_scale(amax_bits, scale_rule);
    if (threadIdx.x == 0) {
      if (scale) scale[r] = rs.s;
      if (amax_out) amax_out[r] = (uint16_t)amax_bits;
    }
    if (q) {
      uint8_t *qrow = q + r * ldq;
      for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) {
        v4i h;
        if (hout) {
          h = *(const v4i *)(hout + r * ldh + c);  // this thread's own store of pass 1
        } else {
          const v4i a = *(const v4i *)(h1 + r * ld1 + c);
          const v4i b = *(const v4i *)(h3 + r * ld3 + c);
#pragma unroll
          for (int k = 0; k < 4; ++k) h[k] = (int)gate_fwd2((uint32_t)a[k], (uint32_t)b[k]);
        }
        if (rs.finite) __builtin_nontemporal_store(cvt8(h, rs.recip), (v2i *)(qrow + c));
        else *(v2i *)(qrow + c) = cvt8_slow(h, rs.recip);
      }
    }
  }
  if (COLMAX)
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8)
      *(v4i *)(col_partials + (int64_t)blockIdx.x * C + c) = lds_cm[c / 8];
}

template <bool COLMAX>
__global__ __launch_bounds__(kWideBlock) void swiglu_bwd_cast_rowwise_wide_kernel(
    const uint16_t *__restrict__ dh, const uint16_t *__restrict__ h1, const uint16_t *__restrict__ h3, int64_t R, int C,
    int64_t lddh, int64_t ld1, int64_t ld3, uint16_t *__restrict__ g1out, uint16_t *__restrict__ g3out, int64_t ldg,
    uint8_t *__restrict__ q1, uint8_t *__restrict__ q3, int64_t ldq, float *__restrict__ scale1,
    float *__restrict__ scale3, uint16_t *__restrict__ col_partials1, uint16_t *__restrict__ col_partials3, int scale_rule) {
  __shared__ uint32_t red[2][2][kWideWaves];
  extern __shared__ __attribute__((aligned(16))) uint8_t dyn_lds[];
  v4i *lds_cm1 = (v4i *)dyn_lds, *lds_cm3 = lds_cm1 + C / 8;  // [C / 8] each
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (COLMAX)
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) lds_cm1[c / 8] = lds_cm3[c / 8] = v4i{0, 0, 0, 0};
  int it = 0;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x, ++it) {
    uint32_t m1 = 0, m3 = 0;
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) {
      const v4i d = __builtin_nontemporal_load((const v4i *)(dh + r * lddh + c));
      const v4i a = __builtin_nontemporal_load((const v4i *)(h1 + r * ld1 + c));
      const v4i b = __builtin_nontemporal_load((const v4i *)(h3 + r * ld3 + c));
      v4i g1, g3;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        uint32_t x1, x3;
        gate_bwd2((uint32_t)d[k], (uint32_t)a[k], (uint32_t)b[k], x1, x3);
        g1[k] = (int)x1;
        g3[k] = (int)x3;
        m1 = pk_absmax_u16(m1, x1);
        m3 = pk_absmax_u16(m3, x3);
      }
      if (COLMAX) {
        v4i o1 = lds_cm1[c / 8], o3 = lds_cm3[c / 8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          o1[k] = (int)pk_absmax_u16((uint32_t)o1[k], (uint32_t)g1[k]);
          o3[k] = (int)pk_absmax_u16((uint32_t)o3[k], (uint32_t)g3[k]);
        }
        lds_cm1[c / 8] = o1;
        lds_cm3[c / 8] = o3;
      }
      *(v4i *)(g1out + r * ldg + c) = g1;
      *(v4i *)(g3out + r * ldg + c) = g3;
    }
    m1 = wave_max_u32(max(m1 & 0xffffu, m1 >> 16));
    m3 = wave_max_u32(max(m3 & 0xffffu, m3 >> 16));
    if (lane == 0) {
      red[it & 1][0][wave] = m1;
      red[it & 1][1][wave] = m3;
    }
    __syncthreads();
    uint32_t bits1 = 0, bits3 = 0;
#pragma unroll
    for (int w = 0; w < kWideWaves; ++w) {
      bits1 = max(bits1, red[it & 1][0][w]);
      bits3 = max(bits3, red[it & 1][1][w]);
    }
    const RowScale rs1 = row_scale(bits1, scale_rule), rs3 = row_scale(bits3, scale_rule);
    if (threadIdx.x == 0) {
      scale1[r] = rs1.s;
      scale3[r] = rs3.s;
    }
    uint8_t *q1row = q1 + r * ldq, *q3row = q3 + r * ldq;
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) {
      const v4i g1 = *(const v4i *)(g1out + r * ldg + c);  // this thread's own stores of pass 1
      const v4i g3 = *(const v4i *)(g3out + r * ldg + c);
      if (rs1.finite) __builtin_nontemporal_store(cvt8(g1, rs1.recip), (v2i *)(q1row + c));
      else *(v2i *)(q1row + c) = cvt8_slow(g1, rs1.recip);
      if (rs3.finite) __builtin_nontemporal_store(cvt8(g3, rs3.recip), (v2i *)(q3row + c));
      else *(v2i *)(q3row + c) = cvt8_slow(g3, rs3.recip);
    }
  }
  if (COLMAX)
    for (int c = threadIdx.x * 8; c < C; c += kWideBlock * 8) {
      *(v4i *)(col_partials1 + (int64_t)blockIdx.x * C + c) = lds_cm1[c / 8];
      *(v4i *)(col_partials3 + (int64_t)blockIdx.x * C + c) = lds_cm3[c / 8];
    }
}

// workgroups (= rows of a partial-maxima array) for R rows
static int64_t gate_blocks(int64_t R) {
  const int64_t cap = (int64_t)num_cus() * 2;
  return R < cap ? R : cap;
}

// the column maxima of the wide kernels must fit LDS: 2 B (forward) or 4 B (backward) per column
constexpr int64_t kGateMaxC = 65536;
constexpr int64_t kGateBwdMaxC = 32768;

// dynamic LDS above the default limit needs the attribute once per device
template <typename K>
static int allow_lds(K kernel, size_t bytes, bool (&done)[kMaxDev]) {
  if (bytes <= 48 * 1024) return L8_OK;
  const int slot = device_slot();
  if (slot >= 0 && done[slot]) return L8_OK;
  L8_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 159 * 1024));
  if (slot >= 0) done[slot] = true;
  return L8_OK;
}

static int launch_fwd_wide(const void *h1, const void *h3, int64_t R, int64_t C, int64_t ld1, int64_t ld3, void *h,
                           int64_t ldh, void *q, int64_t ldq, float *scale, void *amax, float *col_amax, void *ws,
                           hipStream_t st) {
  const int64_t blocks = gate_blocks(R);
  if (col_amax) {
    static bool done[kMaxDev] = {};
    const size_t lds = (size_t)C * 2;
    const int rc = allow_lds(swiglu_cast_rowwise_wide_kernel<true>, lds, done);
    if (rc != L8_OK) return rc;
    hipLaunchKernelGGL((swiglu_cast_rowwise_wide_kernel<true>), dim3((unsigned)blocks), dim3(kWideBlock), lds, st,
                       (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, ld1, ld3, (uint16_t *)h, ldh, (uint8_t *)q, ldq,
                       scale, (uint16_t *)amax, (uint16_t *)ws, l8::scale_rule());
    L8_HIP(hipGetLastError());
    return fold_colmax(ws, blocks, C, col_amax, st);
  }
  hipLaunchKernelGGL((swiglu_cast_rowwise_wide_kernel<false>), dim3((unsigned)blocks), dim3(kWideBlock), 0, st,
                     (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, ld1, ld3, (uint16_t *)h, ldh, (uint8_t *)q, ldq,
                     scale, (uint16_t *)amax, (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

static int launch_bwd_wide(const void *dh, const void *h1, const void *h3, int64_t R, int64_t C, int64_t lddh, int64_t ld1,
                           int64_t ld3, void *g1, void *g3, int64_t ldg, void *q1, void *q3, int64_t ldq, float *s1,
                           float *s3, float *ca1, float *ca3, void *ws, hipStream_t st) {
  const int64_t blocks = gate_blocks(R);
  if (ca1) {
    static bool done[kMaxDev] = {};
    uint16_t *w1 = (uint16_t *)ws, *w3 = w1 + blocks * C;
    const size_t lds = (size_t)C * 4;
    int rc = allow_lds(swiglu_bwd_cast_rowwise_wide_kernel<true>, lds, done);
    if (rc != L8_OK) return rc;
    hipLaunchKernelGGL((swiglu_bwd_cast_rowwise_wide_kernel<true>), dim3((unsigned)blocks), dim3(kWideBlock), lds, st,
                       (const uint16_t *)dh, (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, lddh, ld1, ld3,
                       (uint16_t *)g1, (uint16_t *)g3, ldg, (uint8_t *)q1, (uint8_t *)q3, ldq, s1, s3, w1, w3, l8::scale_rule());
    L8_HIP(hipGetLastError());
    rc = fold_colmax(w1, blocks, C, ca1, st);
    if (rc != L8_OK) return rc;
    return fold_colmax(w3, blocks, C, ca3, st);
  }
  hipLaunchKernelGGL((swiglu_bwd_cast_rowwise_wide_kernel<false>), dim3((unsigned)blocks), dim3(kWideBlock), 0, st,
                     (const uint16_t *)dh, (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, lddh, ld1, ld3,
                     (uint16_t *)g1, (uint16_t *)g3, ldg, (uint8_t *)q1, (uint8_t *)q3, ldq, s1, s3, (uint16_t *)nullptr,
                     (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

template <int NCHW>
static int launch_fwd(const void *h1, const void *h3, int64_t R, int64_t C, int64_t ld1, int64_t ld3, void *h, int64_t ldh,
                      void *q, int64_t ldq, float *scale, void *amax, float *col_amax, void *ws, hipStream_t st) {
  const int64_t blocks = gate_blocks(R);
  if (col_amax) {
    const size_t lds = colmax_in_lds<NCHW, 1>() ? (size_t)C * 2 : 0;
    if (lds > 48 * 1024) {  // above the default limit for dynamic LDS; idempotent
      static bool raised[kMaxDev] = {};
      const int slot = device_slot();
      if (slot < 0 || !raised[slot])
        L8_HIP(hipFuncSetAttribute((const void *)swiglu_cast_rowwise_kernel<NCHW, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
      if (slot >= 0) raised[slot] = true;
    }
    hipLaunchKernelGGL((swiglu_cast_rowwise_kernel<NCHW, true>), dim3((unsigned)blocks), dim3(kGateBlock), lds, st,
                       (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, ld1, ld3, (uint16_t *)h, ldh, (uint8_t *)q, ldq,
                       scale, (uint16_t *)amax, (uint16_t *)ws, l8::scale_rule());
    L8_HIP(hipGetLastError());
    return fold_colmax(ws, blocks, C, col_amax, st);
  }
  hipLaunchKernelGGL((swiglu_cast_rowwise_kernel<NCHW, false>), dim3((unsigned)blocks), dim3(kGateBlock), 0, st,
                     (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, ld1, ld3, (uint16_t *)h, ldh, (uint8_t *)q, ldq,
                     scale, (uint16_t *)amax, (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

template <int NCHW>
static int launch_bwd(const void *dh, const void *h1, const void *h3, int64_t R, int64_t C, int64_t lddh, int64_t ld1,
                      int64_t ld3, void *g1, void *g3, int64_t ldg, void *q1, void *q3, int64_t ldq, float *s1, float *s3,
                      float *ca1, float *ca3, void *ws, hipStream_t st) {
  const int64_t blocks = gate_blocks(R);
  if (ca1) {
    uint16_t *w1 = (uint16_t *)ws, *w3 = w1 + blocks * C;
    const size_t lds = colmax_in_lds<NCHW, 2>() ? (size_t)C * 4 : 0;
    if (lds > 48 * 1024) {  // above the default limit for dynamic LDS; idempotent
      static bool raised[kMaxDev] = {};
      const int slot = device_slot();
      if (slot < 0 || !raised[slot])
        L8_HIP(hipFuncSetAttribute((const void *)swiglu_bwd_cast_rowwise_kernel<NCHW, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
      if (slot >= 0) raised[slot] = true;
    }
    hipLaunchKernelGGL((swiglu_bwd_cast_rowwise_kernel<NCHW, true>), dim3((unsigned)blocks), dim3(kGateBlock), lds, st,
                       (const uint16_t *)dh, (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, lddh, ld1, ld3,
                       (uint16_t *)g1, (uint16_t *)g3, ldg, (uint8_t *)q1, (uint8_t *)q3, ldq, s1, s3, w1, w3, l8::scale_rule());
    L8_HIP(hipGetLastError());
    const int rc = fold_colmax(w1, blocks, C, ca1, st);
    if (rc != L8_OK) return rc;
    return fold_colmax(w3, blocks, C, ca3, st);
  }
  hipLaunchKernelGGL((swiglu_bwd_cast_rowwise_kernel<NCHW, false>), dim3((unsigned)blocks), dim3(kGateBlock), 0, st,
                     (const uint16_t *)dh, (const uint16_t *)h1, (const uint16_t *)h3, R, (int)C, lddh, ld1, ld3,
                     (uint16_t *)g1, (uint16_t *)g3, ldg, (uint8_t *)q1, (uint8_t *)q3, ldq, s1, s3, (uint16_t *)nullptr,
                     (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

static bool aligned16(const void *p) { return ((uintptr_t)p % 16) == 0; }

}  // namespace l8

using namespace l8;

extern "C" int64_t l8_swiglu_workspace(int64_t R, int64_t C) {
  if (R <= 0 || C <= 0) return 0;
  return 2 * gate_blocks(R) * C * (int64_t)sizeof(uint16_t);
}

extern "C" int l8_swiglu_cast_rowwise(const void *h1, const void *h3, int64_t R, int64_t C, int64_t ld1, int64_t ld3, void *h,
                                      int64_t ldh, void *q, int64_t ldq, float *scale, void *amax, float *col_amax,
                                      void *workspace, int64_t workspace_bytes, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_swiglu_cast_rowwise: negative shape R=%lld C=%lld", (long long)R, (long long)C);
  if (R == 0 || C == 0) return L8_OK;
  L8_REQUIRE(h1 && h3 && q && scale, "l8_swiglu_cast_rowwise: null pointer");
  L8_REQUIRE(C % 8 == 0 && ld1 % 8 == 0 && ld3 % 8 == 0 && ld1 >= C && ld3 >= C,
             "l8_swiglu_cast_rowwise: C=%lld, ld1=%lld, ld3=%lld must be multiples of 8 and ld >= C", (long long)C,
             (long long)ld1, (long long)ld3);
  L8_REQUIRE(ldq % 8 == 0 && ldq >= C, "l8_swiglu_cast_rowwise: ldq=%lld must be a multiple of 8 and >= C", (long long)ldq);
  L8_REQUIRE(!h || (ldh % 8 == 0 && ldh >= C), "l8_swiglu_cast_rowwise: ldh=%lld must be a multiple of 8 and >= C", (long long)ldh);
  L8_REQUIRE(aligned16(h1) && aligned16(h3) && (!h || aligned16(h)) && ((uintptr_t)q % 8) == 0,
             "l8_swiglu_cast_rowwise: h1, h3, h must be 16-byte aligned and q 8-byte aligned");
  L8_REQUIRE(C <= kGateMaxC, "l8_swiglu_cast_rowwise: C=%lld exceeds %lld", (long long)C, (long long)kGateMaxC);
  if (col_amax) {
    const int64_t need = l8_swiglu_workspace(R, C) / 2;
    L8_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
               "l8_swiglu_cast_rowwise: col_amax needs a 16-byte aligned workspace of %lld bytes", (long long)need);
  }
  hipStream_t st = (hipStream_t)stream;
  const int64_t nchw = ((C + 511) / 512 + kGateWaves - 1) / kGateWaves;
#define L8_FWD(N) return launch_fwd<N>(h1, h3, R, C, ld1, ld3, h, ldh, q, ldq, scale, amax, col_amax, workspace, st)
  if (nchw <= 1) L8_FWD(1);
  if (nchw <= 2) L8_FWD(2);
  if (nchw <= 4) L8_FWD(4);
  if (nchw <= 6) L8_FWD(6);
  if (nchw <= 8) L8_FWD(8);
#undef L8_FWD
  return launch_fwd_wide(h1, h3, R, C, ld1, ld3, h, ldh, q, ldq, scale, amax, col_amax, workspace, st);
}

extern "C" int l8_swiglu_bwd_cast_rowwise(const void *dh, const void *h1, const void *h3, int64_t R, int64_t C, int64_t lddh,
                                          int64_t ld1, int64_t ld3, void *g1, void *g3, int64_t ldg, void *q1, void *q3,
                                          int64_t ldq, float *scale1, float *scale3, float *col_amax1, float *col_amax3,
                                          void *workspace, int64_t workspace_bytes, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_swiglu_bwd_cast_rowwise: negative shape R=%lld C=%lld", (long long)R, (long long)C);
  if (R == 0 || C == 0) return L8_OK;
  L8_REQUIRE(dh && h1 && h3 && g1 && g3 && q1 && q3 && scale1 && scale3, "l8_swiglu_bwd_cast_rowwise: null pointer");
  L8_REQUIRE((col_amax1 == nullptr) == (col_amax3 == nullptr), "l8_swiglu_bwd_cast_rowwise: pass both column amaxes or neither");
  L8_REQUIRE(C % 8 == 0 && lddh % 8 == 0 && ld1 % 8 == 0 && ld3 % 8 == 0 && ldg % 8 == 0 && ldq % 8 == 0,
             "l8_swiglu_bwd_cast_rowwise: C and every leading dimension must be multiples of 8");
  L8_REQUIRE(lddh >= C && ld1 >= C && ld3 >= C && ldg >= C && ldq >= C, "l8_swiglu_bwd_cast_rowwise: leading dimension < C");
  L8_REQUIRE(aligned16(dh) && aligned16(h1) && aligned16(h3) && aligned16(g1) && aligned16(g3) && ((uintptr_t)q1 % 8) == 0 &&
                 ((uintptr_t)q3 % 8) == 0,
             "l8_swiglu_bwd_cast_rowwise: bf16 operands must be 16-byte aligned and q1, q3 8-byte aligned");
  L8_REQUIRE(C <= kGateBwdMaxC, "l8_swiglu_bwd_cast_rowwise: C=%lld exceeds %lld", (long long)C, (long long)kGateBwdMaxC);
  if (col_amax1) {
    const int64_t need = l8_swiglu_workspace(R, C);
    L8_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
               "l8_swiglu_bwd_cast_rowwise: column amaxes need a 16-byte aligned workspace of %lld bytes", (long long)need);
  }
  hipStream_t st = (hipStream_t)stream;
  const int64_t nchw = ((C + 511) / 512 + kGateWaves - 1) / kGateWaves;
#define L8_BWD(N)                                                                                                  \
  return launch_bwd<N>(dh, h1, h3, R, C, lddh, ld1, ld3, g1, g3, ldg, q1, q3, ldq, scale1, scale3, col_amax1, col_amax3, \
                       workspace, st)
  if (nchw <= 1) L8_BWD(1);
  if (nchw <= 2) L8_BWD(2);
  if (nchw <= 4) L8_BWD(4);
  if (nchw <= 6) L8_BWD(6);
#undef L8_BWD
  return launch_bwd_wide(dh, h1, h3, R, C, lddh, ld1, ld3, g1, g3, ldg, q1, q3, ldq, scale1, scale3, col_amax1, col_amax3,
                         workspace, st);
}
