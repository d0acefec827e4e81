// Fused amax -> fp32 scale -> e4m3fn cast kernels for gfx950 (HBM-bound).
//
// Replaces the eager ATen chain of lingua/float8.py:43-47 (scale()), the row
// amax reductions at :86-87 / :112-114, the tensor amax at :115-118 and the
// weight transpose copy at :111.  Compulsory traffic per element is 2 bytes
// read + 1 byte written; every kernel here reads each input byte from HBM once.
#include <atomic>
#include <mutex>

#include "l8_common.h"

namespace l8 {

// ---------------------------------------------------------------------------
// Row-wise: one wavefront owns one row at a time and keeps it in registers
// between the amax reduction and the cast.  Lane l of chunk j holds columns
// [j*512 + l*8, +8) (one 16-byte load, 1 KiB per wave instruction).
// A workgroup is 4 waves; waves stride over rows so that the optional
// column-amax by-product is accumulated in registers over many rows, merged
// once per workgroup in LDS and written as one row of a partial-maxima array
// that a small second kernel folds into the caller's column amaxes (overwriting them).
// ---------------------------------------------------------------------------
constexpr int kRowBlock = 256;
constexpr int kRowWaves = kRowBlock / 64;

// Row r of x into NCH register quadruples per lane, through a descriptor over the row: a chunk at or beyond column C
// returns zeros, and so does every chunk of a row at or beyond R (a descriptor of no bytes), so there is no branch
// around a load and the compiler's count of outstanding loads stays exact -- which is what lets a wave wait for the
// current row while the next one is still in flight.
#if defined(__HIP_DEVICE_COMPILE__)
template <int NCH>
L8_DEV void load_row(v4i (&buf)[NCH], const uint16_t *x, int64_t r, int64_t R, int64_t ldx, int C, int lane) {
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(x + (r < R ? r : 0) * ldx, r < R ? (uint32_t)C * 2u : 0u);
#pragma unroll
  for (int j = 0; j < NCH; ++j) buf[j] = load16_nt(rs, (uint32_t)(j * 512 + lane * 8) * 2u, 0);
}
#endif

template <int NCH, bool COLMAX>
__global__ __launch_bounds__(kRowBlock, 2) void cast_rowwise_kernel(
    const uint16_t *__restrict__ x, int64_t R, int C, int64_t ldx, uint8_t *__restrict__ q, int64_t ldq,
    float *__restrict__ scale, uint16_t *__restrict__ amax_out, uint16_t *__restrict__ col_partials, int scale_rule) {
#if defined(__HIP_DEVICE_COMPILE__)  // buffer descriptors exist in the device pass only
  extern __shared__ uint32_t lds_colmax[];  // [C/2] packed bf16 pairs when COLMAX
  // the next row is prefetched into a second register set unless that would
  // push the wave beyond 256 VGPRs (two waves per SIMD are worth more)
  constexpr bool PREFETCH = COLMAX ? (NCH <= 8) : (NCH <= 24);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register: the row descriptors hang on it
  const int64_t wave_stride = (int64_t)gridDim.x * kRowWaves;
  int64_t r = (int64_t)blockIdx.x * kRowWaves + wave;

  uint32_t cmax[COLMAX ? NCH * 4 : 1];
  if (COLMAX) {
#pragma unroll
    for (int i = 0; i < NCH * 4; ++i) cmax[i] = 0;
  }

  v4i cur[NCH];
  load_row<NCH>(cur, x, r, R, ldx, C, lane);
  while (r < R) {
    const int64_t rn = r + wave_stride;
    v4i nxt[PREFETCH ? NCH : 1];
    if (PREFETCH) load_row<PREFETCH ? NCH : 1>(nxt, x, rn, R, ldx, C, lane);

    // row amax on packed pairs
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < NCH; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        m = pk_absmax_u16(m, (uint32_t)cur[j][k]);
        if (COLMAX) cmax[j * 4 + k] = pk_absmax_u16(cmax[j * 4 + k], (uint32_t)cur[j][k]);
      }
    m = max(m & 0xffffu, m >> 16);
    const uint32_t amax_bits = wave_max_u32(m);  // bf16 bits, uniform
    const bool finite = amax_bits < 0x7f80u;
    float s;
    if (finite) {
      s = scale_from_amax(bf16_bits_to_f32(amax_bits), scale_rule);
    } else if (amax_bits == 0x7f80u) {
      s = __uint_as_float(0x7f800000u);  // inf / 448
    } else {
      s = __uint_as_float(0x7fc00000u);  // NaN amax -> NaN scale
    }
    const float recip = recip_exact(s);
    if (lane == 0) {
      if (scale) scale[r] = s;
      if (amax_out) amax_out[r] = (uint16_t)amax_bits;
    }
    uint8_t *qrow = q ? q + r * ldq : nullptr;
    const __amdgpu_buffer_rsrc_t rsQ = make_rsrc(qrow, q ? (uint32_t)C : 0u);  // stores beyond column C, or without q, are dropped
#pragma unroll
    for (int j = 0; j < NCH; ++j) store8(rsQ, (uint32_t)(j * 512 + lane * 8), cvt8(cur[j], recip));
    if (q && !finite) {
      // a row with a non-finite amax: redone from memory with the integer conversion, replacing the bytes above (one
      // small loop beside the common path instead of NCH unrolled copies of that conversion inside it)
#pragma unroll 1
      for (int c = lane * 8; c < C; c += 512) *(v2i *)(qrow + c) = cvt8_slow(*(const v4i *)(x + r * ldx + c), recip);
    }
    if (PREFETCH) {
#pragma unroll
      for (int j = 0; j < NCH; ++j) cur[j] = nxt[PREFETCH ? j : 0];
    } else {
      __builtin_amdgcn_sched_barrier(0);  // the row registers are reused: do not start the loads early
      load_row<NCH>(cur, x, rn, R, ldx, C, lane);
    }
    r = rn;
  }

  if (COLMAX) {
    // merge the four waves' column maxima through LDS, one wave after the other
    // (packed pairs, plain reads and writes), then write this workgroup's row of
    // the partial-maxima array; a second small kernel folds the rows.  (Global
    // atomics from every workgroup cost more than the cast itself.)
    v4i *lds4 = (v4i *)lds_colmax;
    for (int w = 0; w < kRowWaves; ++w) {
      if (wave == w) {
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
          const int c = j * 512 + lane * 8;
          if (c < C) {
            v4i mine = {(int)cmax[j * 4], (int)cmax[j * 4 + 1], (int)cmax[j * 4 + 2], (int)cmax[j * 4 + 3]};
            if (w > 0) {
              const v4i old = lds4[c / 8];
#pragma unroll
              for (int k = 0; k < 4; ++k) mine[k] = (int)pk_absmax_u16((uint32_t)old[k], (uint32_t)mine[k]);
            }
            if (w == kRowWaves - 1) *(v4i *)(col_partials + (int64_t)blockIdx.x * C + c) = mine;
            else lds4[c / 8] = mine;
          }
        }
      }
      __syncthreads();
    }
  }
#endif
}

// Long rows: the four waves of a workgroup share one row (wave w owns chunks
// w, w+4, w+8, ... of 512 columns), so a lane holds at most NCHW chunks and
// many workgroups fit a CU.  The row amax crosses waves through LDS with one
// barrier per row (double-buffered).  Column maxima of different waves cover
// disjoint columns and are merged into the global array directly.
template <int NCHW, bool COLMAX>
__global__ __launch_bounds__(kRowBlock, (NCHW <= 4 ? 4 : (NCHW <= 8 ? 2 : 1))) void cast_rowwise_wg_kernel(
    const uint16_t *__restrict__ x, int64_t R, int C, int64_t ldx, uint8_t *__restrict__ q, int64_t ldq,
    float *__restrict__ scale, uint16_t *__restrict__ amax_out, uint16_t *__restrict__ col_partials, int scale_rule) {
#if defined(__HIP_DEVICE_COMPILE__)  // buffer descriptors exist in the device pass only
  __shared__ uint32_t red[2][kRowWaves];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  auto col_of = [&](int j) { return (j * kRowWaves + wave) * 512 + lane * 8; };
  auto load = [&](v4i (&buf)[NCHW], int64_t r) {  // zeros beyond column C and for a row beyond R, as in load_row
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(x + (r < R ? r : 0) * ldx, r < R ? (uint32_t)C * 2u : 0u);
#pragma unroll
    for (int j = 0; j < NCHW; ++j) buf[j] = load16_nt(rs, (uint32_t)col_of(j) * 2u, 0);
  };
  uint32_t cmax[COLMAX ? NCHW * 4 : 1];
  if (COLMAX) {
#pragma unroll
    for (int i = 0; i < NCHW * 4; ++i) cmax[i] = 0;
  }
  int64_t r = blockIdx.x;
  v4i cur[NCHW], nxt[NCHW];
  load(cur, r);
  for (int it = 0; r < R; ++it) {
    const int64_t rn = r + gridDim.x;
    load(nxt, rn);
    // Both rows are waited for here, the next one too.  Letting the next row's loads run on under the arithmetic and
    // the stores (the compiler's own wait would be vmcnt(NCHW)) measured 5 % slower on [16384,11008] when the input
    // had just been written by the kernel before (95.3 against 90.6 us), and no faster on a cold one.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < NCHW; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        m = pk_absmax_u16(m, (uint32_t)cur[j][k]);
        if (COLMAX) cmax[j * 4 + k] = pk_absmax_u16(cmax[j * 4 + k], (uint32_t)cur[j][k]);
      }
    m = wave_max_u32(max(m & 0xffffu, m >> 16));
    if (lane == 0) red[it & 1][wave] = m;
    __syncthreads();
    uint32_t amax_bits = 0;
#pragma unroll
    for (int w = 0; w < kRowWaves; ++w) amax_bits = max(amax_bits, red[it & 1][w]);
    const bool finite = amax_bits < 0x7f80u;
    float s;
    if (finite) s = scale_from_amax(bf16_bits_to_f32(amax_bits), scale_rule);
    else s = __uint_as_float(amax_bits == 0x7f80u ? 0x7f800000u : 0x7fc00000u);
    const float recip = recip_exact(s);
    if (threadIdx.x == 0) {
      if (scale) scale[r] = s;
      if (amax_out) amax_out[r] = (uint16_t)amax_bits;
    }
    uint8_t *qrow = q ? q + r * ldq : nullptr;
    const __amdgpu_buffer_rsrc_t rsQ = make_rsrc(qrow, q ? (uint32_t)C : 0u);  // stores beyond column C, or without q, are dropped
#pragma unroll
    for (int j = 0; j < NCHW; ++j) store8(rsQ, (uint32_t)col_of(j), cvt8(cur[j], recip));
    if (q && !finite) {  // non-finite amax: redone from memory with the integer conversion, as in cast_rowwise_kernel
#pragma unroll 1
      for (int c = threadIdx.x * 8; c < C; c += kRowBlock * 8)
        *(v2i *)(qrow + c) = cvt8_slow(*(const v4i *)(x + r * ldx + c), recip);
    }
#pragma unroll
    for (int j = 0; j < NCHW; ++j) cur[j] = nxt[j];
    r = rn;
  }
  if (COLMAX) {
    // the four waves own disjoint columns: together they write this workgroup's
    // row of the partial-maxima array
#pragma unroll
    for (int j = 0; j < NCHW; ++j) {
      const int c = col_of(j);
      if (c < C)
        *(v4i *)(col_partials + (int64_t)blockIdx.x * C + c) =
            v4i{(int)cmax[j * 4], (int)cmax[j * 4 + 1], (int)cmax[j * 4 + 2], (int)cmax[j * 4 + 3]};
    }
  }
#endif
}

// Folds the partial column maxima [n_slots, C] (bf16, one row per workgroup of a row-wise kernel) into
// col_amax[C] (fp32 bit patterns), which is overwritten.  A workgroup owns 64 columns -- one 128-byte line of
// every partial row -- and its 1024 threads read 16 bytes each from 128 rows at a time, so that a fold of a few
// hundred rows is two to four loads per thread, all in flight at once (the kernel is pure latency: a few MB
// read by a launch that lasts microseconds); the 128 row groups then meet in LDS.  One launch, no atomics,
// nothing to zero beforehand.
constexpr int kFoldCols = 64, kFoldThreads = 1024, kFoldRowGroups = kFoldThreads / 8;
__global__ __launch_bounds__(kFoldThreads) void colmax_fold_kernel(const uint16_t *__restrict__ partials,
                                                                   int n_slots, int C,
                                                                   uint32_t *__restrict__ col_amax) {
  __shared__ v4i red[kFoldRowGroups][8];
  __shared__ uint32_t red2[8][32];
  const int cc = threadIdx.x & 7;   // which 8 columns (16 bytes) of the 64
  const int sg = threadIdx.x >> 3;  // row group
  const int col = blockIdx.x * kFoldCols + cc * 8;
  v4i m = {0, 0, 0, 0};
  if (col < C) {
#pragma unroll 4
    for (int sl = sg; sl < n_slots; sl += kFoldRowGroups) {
      const v4i v = __builtin_nontemporal_load((const v4i *)(partials + (int64_t)sl * C + col));
#pragma unroll
      for (int k = 0; k < 4; ++k) m[k] = (int)pk_absmax_u16((uint32_t)m[k], (uint32_t)v[k]);
    }
  }
  red[sg][cc] = m;
  __syncthreads();
  if (threadIdx.x < 256) {
    const int pair = threadIdx.x & 31, part = threadIdx.x >> 5;  // 32 column pairs x 8 parts of 16 row groups
    uint32_t mm = 0;
#pragma unroll
    for (int g = 0; g < kFoldRowGroups / 8; ++g)
      mm = pk_absmax_u16(mm, reinterpret_cast<const uint32_t *>(&red[part * (kFoldRowGroups / 8) + g][0])[pair]);
    red2[part][pair] = mm;
  }
  __syncthreads();
  if (threadIdx.x < 32) {
    uint32_t mm = 0;
#pragma unroll
    for (int part = 0; part < 8; ++part) mm = pk_absmax_u16(mm, red2[part][threadIdx.x]);
    const int c = blockIdx.x * kFoldCols + threadIdx.x * 2;
    if (c < C) {
      col_amax[c] = (mm & 0xffffu) << 16;  // bf16 -> fp32 bit patterns
      col_amax[c + 1] = mm & 0xffff0000u;
    }
  }
}

// Zero fill for the two kernels that merge into col_amax with atomics (a kernel, not a memset, so that
// a caller may capture the sequence in a graph).
__global__ __launch_bounds__(256) void zero_u32_kernel(uint32_t *__restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

// Fallback for rows too long to keep in registers: two passes over the row by
// one workgroup (the second pass hits L2).
__global__ __launch_bounds__(kRowBlock) void cast_rowwise_long_kernel(
    const uint16_t *__restrict__ x, int64_t R, int C, int64_t ldx, uint8_t *__restrict__ q, int64_t ldq,
    float *__restrict__ scale, uint16_t *__restrict__ amax_out, uint32_t *__restrict__ col_amax, int scale_rule) {
  __shared__ uint32_t red[kRowWaves];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t r = blockIdx.x; r < R; r += gridDim.x) {
    const uint16_t *row = x + r * ldx;
    uint32_t m = 0;
    for (int c = threadIdx.x * 8; c < C; c += kRowBlock * 8) {
      const v4i v = *(const v4i *)(row + c);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        m = pk_absmax_u16(m, (uint32_t)v[k]);
        if (col_amax) {
          const uint32_t a = (uint32_t)v[k] & 0x7fff7fffu;
          if (a & 0xffffu) atomicMax(&col_amax[c + 2 * k], (a & 0xffffu) << 16);
          if (a >> 16) atomicMax(&col_amax[c + 2 * k + 1], a & 0xffff0000u);
        }
      }
    }
    m = wave_max_u32(max(m & 0xffffu, m >> 16));
    __syncthreads();
    if (lane == 0) red[wave] = m;
    __syncthreads();
    uint32_t amax_bits = 0;
#pragma unroll
    for (int w = 0; w < kRowWaves; ++w) amax_bits = max(amax_bits, red[w]);
    float s;
    if (amax_bits < 0x7f80u) s = scale_from_amax(bf16_bits_to_f32(amax_bits), scale_rule);
    else s = __uint_as_float(amax_bits == 0x7f80u ? 0x7f800000u : 0x7fc00000u);
    const float recip = recip_exact(s);
    if (threadIdx.x == 0) {
      if (scale) scale[r] = s;
      if (amax_out) amax_out[r] = (uint16_t)amax_bits;
    }
    if (q) {
      uint8_t *qrow = q + r * ldq;
      const bool finite = amax_bits < 0x7f80u;
      for (int c = threadIdx.x * 8; c < C; c += kRowBlock * 8) {
        const v4i v = *(const v4i *)(row + c);
        *(v2i *)(qrow + c) = finite ? cvt8(v, recip) : cvt8_slow(v, recip);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Column amax alone: each lane owns 8 columns and walks down a slab of rows.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void col_amax_kernel(const uint16_t *__restrict__ x, int64_t R, int C,
                                                       int64_t ldx, int rows_per_block,
                                                       uint32_t *__restrict__ col_amax) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r1 = (r0 + rows_per_block < R) ? r0 + rows_per_block : R;
  uint32_t m[4] = {0, 0, 0, 0};
  for (int64_t r = r0; r < r1; ++r) {
    const v4i v = __builtin_nontemporal_load((const v4i *)(x + r * ldx + c));
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = pk_absmax_u16(m[k], (uint32_t)v[k]);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (m[k] & 0xffffu) atomicMax(&col_amax[c + 2 * k], (m[k] & 0xffffu) << 16);
    if (m[k] >> 16) atomicMax(&col_amax[c + 2 * k + 1], m[k] & 0xffff0000u);
  }
}

// bf16 amax[n] -> bf16 amax_out[1]; one workgroup of 1024 threads.
__global__ __launch_bounds__(1024) void amax_reduce_kernel(const uint16_t *__restrict__ amax, int64_t n,
                                                           uint16_t *__restrict__ out) {
  __shared__ uint32_t red[16];
  uint32_t m = 0;
  for (int64_t i = threadIdx.x; i < n; i += 1024) m = max(m, (uint32_t)(amax[i] & 0x7fffu));
  m = wave_max_u32(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x < 64) {
    m = wave_max_u32(threadIdx.x < 16 ? red[threadIdx.x] : 0u);
    if (threadIdx.x == 0) out[0] = (uint16_t)m;
  }
}

// ---------------------------------------------------------------------------
// Tensor-wise, same layout out as in: pure streaming.
// ---------------------------------------------------------------------------
L8_DEV float scale_from_amax_bits16(uint32_t amax_bits, int scale_rule) {
  if (amax_bits < 0x7f80u) return scale_from_amax(bf16_bits_to_f32(amax_bits), scale_rule);
  return __uint_as_float(amax_bits == 0x7f80u ? 0x7f800000u : 0x7fc00000u);
}
L8_DEV float scale_from_amax_bits32(uint32_t amax_bits, int scale_rule) {  // fp32 bit pattern of a non-negative amax
  if (amax_bits < 0x7f800000u) return scale_from_amax(__uint_as_float(amax_bits), scale_rule);
  return __uint_as_float(amax_bits == 0x7f800000u ? 0x7f800000u : 0x7fc00000u);
}

// A device-resident amax scalar, bf16 or fp32 (sign ignored): its scale, and whether it is finite.
L8_DEV float scale_from_amax_scalar(const void *amax, int amax_f32, bool &finite, int scale_rule) {
  if (amax_f32) {
    const uint32_t bits = *(const uint32_t *)amax & 0x7fffffffu;
    finite = bits < 0x7f800000u;
    return scale_from_amax_bits32(bits, scale_rule);
  }
  const uint32_t bits = *(const uint16_t *)amax & 0x7fffu;
  finite = bits < 0x7f80u;
  return scale_from_amax_bits16(bits, scale_rule);
}

__global__ __launch_bounds__(256) void cast_tensorwise_kernel(const uint16_t *__restrict__ x, int64_t R, int C,
                                                              int64_t ldx, const void *__restrict__ amax, int amax_f32,
                                                              uint8_t *__restrict__ q, int64_t ldq,
                                                              float *__restrict__ scale, int scale_rule) {
  bool finite;
  const float s = scale_from_amax_scalar(amax, amax_f32, finite, scale_rule);
  const float recip = recip_exact(s);
  if (blockIdx.x == 0 && threadIdx.x == 0) scale[0] = s;
  const int cpr = C / 8;  // 16-byte chunks per row
  const int64_t total = R * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / cpr;
    const int c = (int)(i - r * cpr) * 8;
    const v4i v = __builtin_nontemporal_load((const v4i *)(x + r * ldx + c));
    // the amax is handed in and must bound |x|: then every product is within
    // the finite e4m3 range and the hardware converter agrees with the ATen cast
    *(v2i *)(q + r * ldq + c) = finite ? cvt8(v, recip) : cvt8_slow(v, recip);
  }
}

// Row-wise cast with the row amaxes handed in, as lingua/float8.py:43-47 is called: the amax is an
// argument there, not a by-product.  It need not be the true amax of the row (a repeated tensor amax, a
// stale amax of delayed scaling), so a product may leave the finite e4m3 range: chunks whose largest
// product exceeds 448 take the integer conversion, which reproduces the ATen cast there (<= 464 rounds
// to 448, above gives the NaN code).
__global__ __launch_bounds__(256) void cast_rowwise_given_amax_kernel(const uint16_t *__restrict__ x, int64_t R, int C,
                                                                      int64_t ldx, const void *__restrict__ amax, int amax_f32,
                                                                      uint8_t *__restrict__ q, int64_t ldq,
                                                                      float *__restrict__ scale, int scale_rule) {
  const int cpr = C / 8;  // 16-byte chunks per row
  const int64_t total = R * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / cpr;
    const int c = (int)(i - r * cpr) * 8;
    // clamp(min=EPS) also lifts a negative amax
    const float s = scale_from_amax(amax_f32 ? ((const float *)amax)[r] : bf16_bits_to_f32(((const uint16_t *)amax)[r]), scale_rule);
    const float recip = recip_exact(s);
    if (c == 0) scale[r] = s;
    const v4i v = __builtin_nontemporal_load((const v4i *)(x + r * ldx + c));
    uint32_t m = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) m = pk_absmax_u16(m, (uint32_t)v[k]);
    m = max(m & 0xffffu, m >> 16);
    // !(p <= 448) also catches a NaN product (NaN element, NaN or infinite scale)
    const float p = bf16_bits_to_f32(m) * recip;
    *(v2i *)(q + r * ldq + c) = (p <= kE4M3Max) ? cvt8(v, recip) : cvt8_slow(v, recip);
  }
}

// ---------------------------------------------------------------------------
// Transposed casts (tensor-wise for the dgrad weight, column-wise for wgrad):
// a [256 rows x 64 cols] tile of x becomes a [64 x 256] tile of q.
// Thread t loads 8 columns (one 16-byte load) from each of 4 consecutive rows,
// packs, for each of its 8 columns, the 4 row-consecutive e4m3 bytes into one
// dword and writes it to the transposed tile in LDS; the tile is then read
// back as 16-byte row segments and stored as 256-byte runs of the output rows.
// ---------------------------------------------------------------------------
// Tile shapes: TC columns x (256 / (TC / 8)) * 4 * TU rows.  128 x 128 (TC 128, TU 2) is the one used; 64 x 128 (TC 64,
// TU 1) for tensors with too few 128 x 128 tiles to fill the chip.  Inside the MLP step, against the 64 x 256 tile this
// kernel had before: [16384,4096] 39.1 -> 37.3 us, [16384,11008] 110.1 -> 107.9, weights 28.0 -> 28.0; Llama-1B shapes:
// [16384,8192] 80.1 -> 73.8, [16384,2048] 21.0 -> 21.1, [8192,2048] 12.4 -> 11.8, [2048,2048] 5.2 -> 4.9 (64 x 128).
// 128 x 256 was another 1-5 % ahead on the two widest activations and 4 % behind on every weight.
// Tensors of at least 16384 rows and 8192 columns take 128 x 256 (TU 4): over 26 activation shapes, each timed right
// behind the kernel that produces it, 128 x 128 and 128 x 256 are within 1-3 % of each other there except at 11008
// columns (the 7B ffn width), where 128 x 128 alone falls off -- [16384,11008] 100 against 90 us, [32768,11008] 206
// against 187 -- while 10880, 11136, 11264 and 11520 columns show nothing of the kind.
// The loads are non-temporal, the stores are not: a workgroup writes 128-byte pieces of 128 output rows, the pieces
// next to them come from other workgroups a little later, and ordinary stores leave it to the L2 to write neighbours
// back together.  Inside the MLP step, ordinary against non-temporal stores: [16384,11008] 99.4 against 108.4 us,
// [16384,4096] 35.5 against 37.2, weights 26.2 against 27.7; ordinary loads instead cost 2-4 %.
template <int TC, int TU>
struct TransposeTile {
  static constexpr int kTC = TC;                  // columns of x per tile
  static constexpr int kCCH = TC / 8;             // 8-column chunks per tile row
  static constexpr int kRG = 256 / kCCH;          // 4-row groups covered by the 256 threads in one pass
  static constexpr int kTU = TU;                  // passes (4-row units per thread)
  static constexpr int kTR = kRG * 4 * TU;        // rows of x per tile
  static constexpr int kTStride = kTR + 16;       // LDS row stride in bytes
};
constexpr int kMaxTileRows = 256;                 // no tile is taller (bounds the row stride the host accepts)

template <bool PER_COL, int TC, int TU>
__global__ __launch_bounds__(256) void cast_transposed_kernel(
    const uint16_t *__restrict__ x, int64_t R, int C, int64_t ldx, const void *__restrict__ amax_scalar, int amax_f32,
    const uint32_t *__restrict__ col_amax, uint8_t *__restrict__ q, int64_t ldq, float *__restrict__ scale,
    int vec_store, int scale_rule) {
#if defined(__HIP_DEVICE_COMPILE__)  // the buffer-resource type exists in the device pass only
  using T = TransposeTile<TC, TU>;
  constexpr int kTC = T::kTC, kCCH = T::kCCH, kRG = T::kRG, kTU = T::kTU, kTR = T::kTR, kTStride = T::kTStride;
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTC * kTStride];
  __shared__ float recips[kTC];
  const int t = threadIdx.x;
  // Workgroup w takes column block w % nct and row tile (w / nct + w % nct) % nrt:
  // a diagonal walk.  The workgroups resident at one time then touch addresses
  // that differ in their low bits on both sides, which keeps power-of-two row
  // strides (input stride C, output stride R) from piling onto a few memory
  // channels, while each column block still advances through consecutive row
  // tiles (long runs in the output rows) and each row tile through consecutive
  // column blocks (wide bands of the input rows).
  const int nct = (C + kTC - 1) / kTC;
  const int64_t nrt = (R + kTR - 1) / kTR;
  const int cb = (int)(blockIdx.x % nct);
  const int64_t rt = (blockIdx.x / nct + cb) % nrt;
  const int64_t r0 = rt * kTR;
  const int c0 = cb * kTC;
  const int cc = t % kCCH;  // which 8-column chunk of the tile
  const int rg = t / kCCH;  // which 4-row group of a pass
  const int c = c0 + cc * 8;

  // Loads without branches, through buffer descriptors whose range check returns zeros: the amax behind the
  // scale(s) first, the tile right behind it.  The counter of outstanding loads retires in order, so the wait for
  // the amax leaves the tile's loads in flight, and the division and the reciprocal run under them.  (With a branch
  // around each load the compiler waited for all of them after the fifth and again before the division.)
  uint32_t amax_lo, amax_hi = 0;
  if (PER_COL) {
    const __amdgpu_buffer_rsrc_t rsAmax = make_rsrc(col_amax, (uint32_t)C * 4u);
    amax_lo = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsAmax, (c0 + t % kTC) * 4, 0, 0);  // zero beyond column C
  } else {
    // two or four bytes (bf16 or fp32) as two halves: the upper half of a bf16 amax lies beyond the descriptor
    const __amdgpu_buffer_rsrc_t rsAmax = make_rsrc(amax_scalar, amax_f32 ? 4u : 2u);
    amax_lo = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsAmax, 0, 0, 0);
    amax_hi = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsAmax, 2, 0, 0);
  }
  // keep the amax's load(s) here, ahead of the tile's: neither sunk to their first use nor rescheduled
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  // kTU units of 4 rows x 8 columns per thread.  The descriptor covers the tile's rows that exist, up to the last
  // column of the last one: a row at or beyond R starts beyond it, and a chunk at or beyond column C (which would
  // otherwise read the next row) is sent there (the range check covers the sum of the lane's and the scalar offset, dword by
  // dword).  The host keeps kTR * ldx * 2 below 2^30.
  const int64_t rows_left = R - r0;
  const uint32_t row_bytes = (uint32_t)ldx * 2u;
  const uint32_t tile_bytes = (uint32_t)((rows_left < kTR ? (int)rows_left : kTR) - 1) * row_bytes + (uint32_t)C * 2u;
  const __amdgpu_buffer_rsrc_t rsX = make_rsrc(x + r0 * ldx, tile_bytes);
  const uint32_t voff = (c < C ? (uint32_t)c * 2u : tile_bytes) + (uint32_t)(rg * 4) * row_bytes;
  v4i in[kTU][4];
#pragma unroll
  for (int u = 0; u < kTU; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      in[u][i] = load16_nt(rsX, voff, (u * kRG * 4 + i) * row_bytes);

  if (PER_COL) {
    // every wave computes the 64 scales (a branch around the division would pull the amax's load into it, behind
    // the tile's loads); the first one keeps them
    const float s = scale_from_amax_bits32(amax_lo, scale_rule);
    float rc = recip_exact(s);
    if (amax_lo >= 0x7f800000u) rc = __uint_as_float(0x7fc00000u);  // flag: slow path for this column
    if (t < kTC) {
      if (rt == 0 && c0 + t < C) scale[c0 + t] = s;
      recips[t] = rc;
    }
    __syncthreads();
  }
  float rcp[8];
  bool finite = true;
  if (PER_COL) {
#pragma unroll
    for (int j = 0; j < 8; ++j) rcp[j] = recips[cc * 8 + j];
  } else {
    const uint32_t amax_bits = (amax_lo | (amax_hi << 16)) & (amax_f32 ? 0x7fffffffu : 0x7fffu);  // the sign is ignored
    finite = amax_bits < (amax_f32 ? 0x7f800000u : 0x7f80u);
    const float s = amax_f32 ? scale_from_amax_bits32(amax_bits, scale_rule) : scale_from_amax_bits16(amax_bits, scale_rule);
    const float rc = recip_exact(s);
#pragma unroll
    for (int j = 0; j < 8; ++j) rcp[j] = rc;
    if (blockIdx.x == 0 && t == 0) scale[0] = s;
  }

  // convert and transpose inside the thread: column j <- rows 0..3 of each unit
  bool all_fast = finite;
#pragma unroll
  for (int u = 0; u < kTU; ++u)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int w = j >> 1;
      const bool hi = j & 1;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t p = (uint32_t)in[u][i][w];
        v[i] = __uint_as_float(hi ? (p & 0xffff0000u) : (p << 16)) * rcp[j];
      }
      if (PER_COL && u == 0) all_fast &= rcp[j] == rcp[j];
      int packed = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], packed, true);
      *(int *)(tile + (cc * 8 + j) * kTStride + (u * kRG + rg) * 4) = packed;
    }
  if (!all_fast) {
    // A column whose amax is not finite: its bytes are redone from memory with the true reciprocal (0 for an
    // infinite amax, NaN for a NaN) and the integer conversion, and replace what the line above wrote.
#pragma unroll 1
    for (int uj = 0; uj < kTU * 8; ++uj) {
      const int u = uj >> 3, j = uj & 7;
      float rc;
      if (PER_COL) {
        if (recips[cc * 8 + j] == recips[cc * 8 + j]) continue;
        rc = recip_exact(scale_from_amax_bits32(col_amax[c + j < C ? c + j : 0], scale_rule));
      } else {
        rc = rcp[0];
      }
      uint32_t packed = 0;
      for (int i = 0; i < 4; ++i) {
        const int64_t r = r0 + (u * kRG + rg) * 4 + i;
        const uint32_t h = (r < R && c + j < C) ? x[r * ldx + c + j] : 0u;
        packed |= e4m3fn_from_f32_slow(bf16_bits_to_f32(h) * rc) << (8 * i);
      }
      *(uint32_t *)(tile + (cc * 8 + j) * kTStride + (u * kRG + rg) * 4) = packed;
    }
  }
  __syncthreads();
  // write out: 64 output rows (columns of x) x kTR bytes, 16 bytes per thread and step
  constexpr int SEGS = kTR / 16;  // 16-byte segments per output row
#pragma unroll
  for (int i = 0; i < kTC * SEGS / 256; ++i) {
    const int idx = i * 256 + t;
    const int oc = idx / SEGS;   // output row within the tile
    const int seg = idx % SEGS;
    const int col = c0 + oc;
    const int64_t r = r0 + seg * 16;
    if (col < C && r < R) {
      const v4i v = *(const v4i *)(tile + oc * kTStride + seg * 16);
      uint8_t *dst = q + (int64_t)col * ldq + r;
      if (vec_store && r + 16 <= R) {
        *(v4i *)dst = v;  // not a streaming store: see the note on the tile shapes
      } else {
        const uint8_t *src = tile + oc * kTStride + seg * 16;
        for (int b = 0; b < 16 && r + b < R; ++b) dst[b] = src[b];
      }
    }
  }
#endif
}

// ---------------------------------------------------------------------------
// host entry points
// ---------------------------------------------------------------------------
static bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

// Number of workgroups (= rows of the partial-maxima workspace) of the two
// register-resident row-wise kernels; 0 when the shape uses the two-pass kernel.
static int64_t rowwise_blocks(int64_t R, int64_t C, bool colmax) {
  const int64_t nch = (C + 511) / 512;
  const int64_t cus = num_cus();
  if (nch <= 8) {
    const int64_t blocks = (R + kRowWaves - 1) / kRowWaves, cap = cus * (colmax ? 2 : 8);
    return blocks < cap ? blocks : cap;
  }
  if ((nch + kRowWaves - 1) / kRowWaves <= 16) {
    const int64_t cap = cus * (colmax ? 2 : 8);
    return R < cap ? R : cap;
  }
  return 0;
}

int fold_colmax(const void *partials, int64_t slots, int64_t C, float *col_amax, hipStream_t st) {
  hipLaunchKernelGGL(colmax_fold_kernel, dim3((unsigned)((C + kFoldCols - 1) / kFoldCols)), dim3(kFoldThreads), 0, st,
                     (const uint16_t *)partials, (int)slots, (int)C, (uint32_t *)col_amax);
  L8_HIP(hipGetLastError());
  return L8_OK;
}

static int zero_u32(void *p, int64_t n, hipStream_t st) {
  hipLaunchKernelGGL(zero_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (uint32_t *)p, n);
  L8_HIP(hipGetLastError());
  return L8_OK;
}

template <int NCH>
static int launch_rowwise(const void *x, int64_t R, int64_t C, int64_t ldx, void *q, int64_t ldq, float *scale,
                          void *amax, float *col_amax, void *ws, hipStream_t st) {
  const int64_t blocks = rowwise_blocks(R, C, col_amax != nullptr);
  if (col_amax) {
    const size_t lds = (size_t)C * sizeof(uint16_t);
    hipLaunchKernelGGL((cast_rowwise_kernel<NCH, true>), dim3((unsigned)blocks), dim3(kRowBlock), lds, st,
                       (const uint16_t *)x, R, (int)C, ldx, (uint8_t *)q, ldq, scale, (uint16_t *)amax, (uint16_t *)ws, l8::scale_rule());
    L8_HIP(hipGetLastError());
    return fold_colmax(ws, blocks, C, col_amax, st);
  }
  hipLaunchKernelGGL((cast_rowwise_kernel<NCH, false>), dim3((unsigned)blocks), dim3(kRowBlock), 0, st,
                     (const uint16_t *)x, R, (int)C, ldx, (uint8_t *)q, ldq, scale, (uint16_t *)amax, (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

template <int NCHW>
static int launch_rowwise_wg(const void *x, int64_t R, int64_t C, int64_t ldx, void *q, int64_t ldq, float *scale,
                             void *amax, float *col_amax, void *ws, hipStream_t st) {
  const int64_t blocks = rowwise_blocks(R, C, col_amax != nullptr);
  if (col_amax) {
    hipLaunchKernelGGL((cast_rowwise_wg_kernel<NCHW, true>), dim3((unsigned)blocks), dim3(kRowBlock), 0, st,
                       (const uint16_t *)x, R, (int)C, ldx, (uint8_t *)q, ldq, scale, (uint16_t *)amax, (uint16_t *)ws, l8::scale_rule());
    L8_HIP(hipGetLastError());
    return fold_colmax(ws, blocks, C, col_amax, st);
  }
  hipLaunchKernelGGL((cast_rowwise_wg_kernel<NCHW, false>), dim3((unsigned)blocks), dim3(kRowBlock), 0, st,
                     (const uint16_t *)x, R, (int)C, ldx, (uint8_t *)q, ldq, scale, (uint16_t *)amax, (uint16_t *)nullptr, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

}  // namespace l8

using namespace l8;


extern "C" int64_t l8_cast_rowwise_workspace(int64_t R, int64_t C) {
  if (R <= 0 || C <= 0) return 0;
  return rowwise_blocks(R, C, true) * C * (int64_t)sizeof(uint16_t);
}

// Argument checks and dispatch shared by l8_cast_rowwise and l8_cast_rowwise_noalloc; `what` names the
// entry point in error messages.  `workspace` holds at least l8_cast_rowwise_workspace(R, C) bytes when
// col_amax is given (checked by the callers).
static int cast_rowwise_impl(const char *what, const void *x, int64_t R, int64_t C, int64_t ldx, void *q, int64_t ldq,
                             float *scale, void *amax, float *col_amax, void *workspace, hipStream_t st) {
  L8_REQUIRE(x != nullptr, "%s: x is null", what);
  L8_REQUIRE((q == nullptr) || (scale != nullptr), "%s: q given without scale", what);
  L8_REQUIRE(C % 8 == 0 && ldx % 8 == 0 && ldx >= C, "%s: C=%lld and ldx=%lld must be multiples of 8, ldx >= C", what,
             (long long)C, (long long)ldx);
  L8_REQUIRE(aligned(x, 16), "%s: x must be 16-byte aligned", what);
  if (q) L8_REQUIRE(ldq % 8 == 0 && ldq >= C && aligned(q, 8), "%s: q must be 8-byte aligned with ldq %% 8 == 0, ldq >= C", what);
  L8_REQUIRE(C < (1LL << 31), "%s: C too large", what);
  void *ws = workspace;
  const int64_t nch = (C + 511) / 512;
  if (nch <= 4) return launch_rowwise<4>(x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, st);
  if (nch <= 8) return launch_rowwise<8>(x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, st);
  // longer rows: one workgroup per row, nchw = chunks per lane
  const int64_t nchw = (nch + kRowWaves - 1) / kRowWaves;
  if (nchw <= 4) return launch_rowwise_wg<4>(x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, st);
  if (nchw <= 6) return launch_rowwise_wg<6>(x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, st);
  if (nchw <= 8) return launch_rowwise_wg<8>(x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, st);
  if (nchw <= 16) return launch_rowwise_wg<16>(x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, st);
  int64_t blocks = R < (int64_t)num_cus() * 8 ? R : (int64_t)num_cus() * 8;
  if (col_amax) {
    const int rc = zero_u32(col_amax, C, st);
    if (rc != L8_OK) return rc;
  }
  hipLaunchKernelGGL(cast_rowwise_long_kernel, dim3((unsigned)blocks), dim3(kRowBlock), 0, st, (const uint16_t *)x, R,
                     (int)C, ldx, (uint8_t *)q, ldq, scale, (uint16_t *)amax, (uint32_t *)col_amax, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

extern "C" int l8_cast_rowwise(const void *x, int64_t R, int64_t C, int64_t ldx, void *q, int64_t ldq, float *scale,
                               void *amax, float *col_amax, void *workspace, int64_t workspace_bytes, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_cast_rowwise: negative shape R=%lld C=%lld", (long long)R, (long long)C);
  if (R == 0 || C == 0) return L8_OK;
  if (col_amax) {
    const int64_t need = l8_cast_rowwise_workspace(R, C);
    L8_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need && aligned(workspace, 16)),
               "l8_cast_rowwise: col_amax needs a 16-byte aligned workspace of %lld bytes (l8_cast_rowwise_workspace)",
               (long long)need);
  }
  return cast_rowwise_impl("l8_cast_rowwise", x, R, C, ldx, q, ldq, scale, amax, col_amax, workspace, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------
// l8_cast_rowwise for callers that cannot allocate: the partial column maxima go to a static device
// array instead of a caller-supplied workspace.  Each GPU holds its own copy of the array at its own
// address; the address is looked up once per device (with that device current) and kept.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[L8_NOALLOC_SCRATCH_BYTES];
static std::atomic<void *> g_scratch_ptr[l8::kMaxDev];  // device address of `scratch`, per device
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up on first use).
static int scratch_of_current_device(void **out) {
  int dev = -1;
  L8_HIP(hipGetDevice(&dev));
  L8_REQUIRE(dev >= 0 && dev < kMaxDev, "device ordinal %d beyond the %d this library keeps state for", dev, kMaxDev);
  void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (!ptr) {
      L8_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
      L8_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null address for the scratch array");
      g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
  }
  *out = ptr;
  return L8_OK;
}

// Called by l8_device_check with `device` current, so that the look-up (which may load the code object)
// happens at set-up and not inside a caller's capture or serving loop.
int l8::noalloc_setup_current_device() {
  void *ptr = nullptr;
  return scratch_of_current_device(&ptr);
}

extern "C" int l8_cast_rowwise_noalloc(const void *x, int64_t R, int64_t C, int64_t ldx, void *q, int64_t ldq,
                                       float *scale, void *amax, float *col_amax, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_cast_rowwise_noalloc: negative shape R=%lld C=%lld", (long long)R, (long long)C);
  if (R == 0 || C == 0) return L8_OK;
  void *ws = nullptr;
  if (col_amax) {
    const int64_t need = l8_cast_rowwise_workspace(R, C);
    L8_REQUIRE(need <= (int64_t)L8_NOALLOC_SCRATCH_BYTES,
               "l8_cast_rowwise_noalloc: [%lld,%lld] with column amaxes needs %lld bytes of scratch, the static array "
               "holds %lld (use l8_cast_rowwise with a workspace)",
               (long long)R, (long long)C, (long long)need, (long long)L8_NOALLOC_SCRATCH_BYTES);
    const int rc = scratch_of_current_device(&ws);
    if (rc != L8_OK) return rc;
  }
  return cast_rowwise_impl("l8_cast_rowwise_noalloc", x, R, C, ldx, q, ldq, scale, amax, col_amax, ws, (hipStream_t)stream);
}

extern "C" int l8_cast_rowwise_given_amax(const void *x, int64_t R, int64_t C, int64_t ldx, const void *amax,
                                          int amax_dtype, void *q, int64_t ldq, float *scale, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_cast_rowwise_given_amax: negative shape");
  if (R == 0 || C == 0) return L8_OK;
  L8_REQUIRE(x && amax && q && scale, "l8_cast_rowwise_given_amax: null pointer");
  L8_REQUIRE(amax_dtype == L8_AMAX_BF16 || amax_dtype == L8_AMAX_F32, "l8_cast_rowwise_given_amax: bad amax_dtype %d", amax_dtype);
  L8_REQUIRE(aligned(amax, amax_dtype == L8_AMAX_F32 ? 4 : 2), "l8_cast_rowwise_given_amax: misaligned amax");
  L8_REQUIRE(C % 8 == 0 && ldx % 8 == 0 && ldx >= C && aligned(x, 16),
             "l8_cast_rowwise_given_amax: C, ldx multiples of 8 and x 16-byte aligned required");
  L8_REQUIRE(ldq >= C && ldq % 8 == 0 && aligned(q, 8),
             "l8_cast_rowwise_given_amax: q must be 8-byte aligned with ldq %% 8 == 0, ldq >= C");
  L8_REQUIRE(C < (1LL << 31), "l8_cast_rowwise_given_amax: C too large");
  const int64_t total = R * (C / 8);
  int64_t blocks = (total + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(cast_rowwise_given_amax_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t *)x, R, (int)C, ldx, amax, amax_dtype, (uint8_t *)q, ldq, scale, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

extern "C" int l8_col_amax(const void *x, int64_t R, int64_t C, int64_t ldx, float *col_amax, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_col_amax: negative shape");
  if (R == 0 || C == 0) return L8_OK;
  L8_REQUIRE(x && col_amax, "l8_col_amax: null pointer");
  L8_REQUIRE(C % 8 == 0 && ldx % 8 == 0 && ldx >= C && aligned(x, 16), "l8_col_amax: C, ldx multiples of 8 and x 16-byte aligned required");
  L8_REQUIRE(C < (1LL << 31), "l8_col_amax: C too large");
  const int gx = (int)((C / 8 + 255) / 256);
  // enough row slabs to fill the chip, at least 64 rows each
  int64_t slabs = (int64_t)num_cus() * 8 / gx;
  if (slabs < 1) slabs = 1;
  int64_t rows_per = (R + slabs - 1) / slabs;
  if (rows_per < 64) rows_per = 64;
  slabs = (R + rows_per - 1) / rows_per;
  L8_REQUIRE(slabs <= 65535, "l8_col_amax: too many row slabs");
  const int rc = zero_u32(col_amax, C, (hipStream_t)stream);
  if (rc != L8_OK) return rc;
  hipLaunchKernelGGL(col_amax_kernel, dim3(gx, (unsigned)slabs), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t *)x, R, (int)C, ldx, (int)rows_per, (uint32_t *)col_amax);
  L8_HIP(hipGetLastError());
  return L8_OK;
}

extern "C" int l8_amax_reduce(const void *amax, int64_t n, void *amax_out, void *stream) {
  L8_REQUIRE(n >= 1 && amax && amax_out, "l8_amax_reduce: need n >= 1 and non-null pointers");
  hipLaunchKernelGGL(amax_reduce_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const uint16_t *)amax, n,
                     (uint16_t *)amax_out);
  L8_HIP(hipGetLastError());
  return L8_OK;
}

template <int TC, int TU>
static int launch_transposed_tile(bool per_col, const void *x, int64_t R, int64_t C, int64_t ldx, const void *amax,
                                  int amax_f32, const float *col_amax, void *q, int64_t ldq, float *scale, hipStream_t st) {
  using T = TransposeTile<TC, TU>;
  static_assert(T::kTR <= kMaxTileRows, "the row-stride limit assumes no taller tile");
  const int64_t gx = ((C + T::kTC - 1) / T::kTC) * ((R + T::kTR - 1) / T::kTR);
  L8_REQUIRE(gx < (1LL << 31), "transposed cast: shape too large (%lld x %lld)", (long long)R, (long long)C);
  const int vec = (ldq % 16 == 0 && aligned(q, 16)) ? 1 : 0;
  if (per_col)
    hipLaunchKernelGGL((cast_transposed_kernel<true, TC, TU>), dim3((unsigned)gx), dim3(256), 0, st,
                       (const uint16_t *)x, R, (int)C, ldx, (const void *)nullptr, 0, (const uint32_t *)col_amax,
                       (uint8_t *)q, ldq, scale, vec, l8::scale_rule());
  else
    hipLaunchKernelGGL((cast_transposed_kernel<false, TC, TU>), dim3((unsigned)gx), dim3(256), 0, st,
                       (const uint16_t *)x, R, (int)C, ldx, amax, amax_f32, (const uint32_t *)nullptr,
                       (uint8_t *)q, ldq, scale, vec, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

static int launch_transposed(bool per_col, const void *x, int64_t R, int64_t C, int64_t ldx, const void *amax,
                             int amax_f32, const float *col_amax, void *q, int64_t ldq, float *scale, hipStream_t st) {
  // a tile's rows within 1 GiB: then no sum of a lane's offset (up to twice the tile) and a row's scalar offset wraps
  L8_REQUIRE((int64_t)kMaxTileRows * ldx * 2 < (1LL << 30), "transposed cast: row stride too large (%lld elements)", (long long)ldx);
  const int64_t tiles128 = ((C + 127) / 128) * ((R + 127) / 128);
  if (tiles128 < 4 * (int64_t)num_cus())  // too few 128 x 128 tiles for four workgroups per compute unit
    return launch_transposed_tile<64, 1>(per_col, x, R, C, ldx, amax, amax_f32, col_amax, q, ldq, scale, st);
  if (R >= 16384 && C >= 8192)  // the large activations: see the note on the tile shapes
    return launch_transposed_tile<128, 4>(per_col, x, R, C, ldx, amax, amax_f32, col_amax, q, ldq, scale, st);
  return launch_transposed_tile<128, 2>(per_col, x, R, C, ldx, amax, amax_f32, col_amax, q, ldq, scale, st);
}

extern "C" int l8_cast_tensorwise(const void *x, int64_t R, int64_t C, int64_t ldx, const void *amax, int amax_dtype,
                                  int transpose, void *q, int64_t ldq, float *scale, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_cast_tensorwise: negative shape");
  L8_REQUIRE(amax && scale, "l8_cast_tensorwise: amax and scale must be non-null");
  L8_REQUIRE(amax_dtype == L8_AMAX_BF16 || amax_dtype == L8_AMAX_F32, "l8_cast_tensorwise: bad amax_dtype %d", amax_dtype);
  L8_REQUIRE(aligned(amax, amax_dtype == L8_AMAX_F32 ? 4 : 2), "l8_cast_tensorwise: misaligned amax");
  if (R == 0 || C == 0) return L8_OK;
  L8_REQUIRE(x && q, "l8_cast_tensorwise: null pointer");
  L8_REQUIRE(C % 8 == 0 && ldx % 8 == 0 && ldx >= C && aligned(x, 16), "l8_cast_tensorwise: C, ldx multiples of 8 and x 16-byte aligned required");
  L8_REQUIRE(C < (1LL << 31), "l8_cast_tensorwise: C too large");
  hipStream_t st = (hipStream_t)stream;
  if (transpose) {
    L8_REQUIRE(ldq >= R, "l8_cast_tensorwise: transposed output needs ldq >= R");
    return launch_transposed(false, x, R, C, ldx, amax, amax_dtype, nullptr, q, ldq, scale, st);
  }
  L8_REQUIRE(ldq >= C && ldq % 8 == 0 && aligned(q, 8), "l8_cast_tensorwise: q must be 8-byte aligned with ldq %% 8 == 0, ldq >= C");
  const int64_t total = R * (C / 8);
  int64_t blocks = (total + 255) / 256;
  const int64_t cap = (int64_t)num_cus() * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(cast_tensorwise_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint16_t *)x, R, (int)C,
                     ldx, amax, amax_dtype, (uint8_t *)q, ldq, scale, l8::scale_rule());
  L8_HIP(hipGetLastError());
  return L8_OK;
}

extern "C" int l8_cast_colwise_transposed(const void *x, int64_t R, int64_t C, int64_t ldx, const float *col_amax,
                                          void *q, int64_t ldq, float *scale, void *stream) {
  L8_REQUIRE(R >= 0 && C >= 0, "l8_cast_colwise_transposed: negative shape");
  if (C == 0) return L8_OK;
  L8_REQUIRE(col_amax && scale, "l8_cast_colwise_transposed: col_amax and scale must be non-null");
  L8_REQUIRE(R > 0, "l8_cast_colwise_transposed: R must be positive when C > 0");
  L8_REQUIRE(x && q, "l8_cast_colwise_transposed: null pointer");
  L8_REQUIRE(C % 8 == 0 && ldx % 8 == 0 && ldx >= C && aligned(x, 16), "l8_cast_colwise_transposed: C, ldx multiples of 8 and x 16-byte aligned required");
  L8_REQUIRE(ldq >= R, "l8_cast_colwise_transposed: ldq >= R required");
  L8_REQUIRE(C < (1LL << 31), "l8_cast_colwise_transposed: C too large");
  return launch_transposed(true, x, R, C, ldx, nullptr, 0, col_amax, q, ldq, scale, (hipStream_t)stream);
}
