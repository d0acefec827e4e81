// Shared device helpers and host-side error plumbing for the gfx950 fp8 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lingua_fp8.h"

namespace l8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ---- host side ------------------------------------------------------------
int fail(int code, const char *fmt, ...);  // records the thread-local message, returns code
#define L8_HIP(expr)                                                                    \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess) return ::l8::fail(L8_EHIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)
#define L8_REQUIRE(cond, ...)                              \
  do {                                                     \
    if (!(cond)) return ::l8::fail(L8_EINVAL, __VA_ARGS__); \
  } while (0)

int num_cus();  // compute units of the current device (cached per device)

// How every cast evaluates clamp(amax, EPS) / 448 (l8_set_scale_rule); read once per launch and handed to the kernel.
int scale_rule();

// Per-device one-time set-up (function attributes are per device): index of the
// current device into tables of kMaxDev entries, or -1 (then nothing is cached).
constexpr int kMaxDev = 64;
int device_slot();

// Folds partial column maxima [slots, C] (bf16, one row per workgroup of a
// row-wise kernel) into col_amax[C] (fp32 bit patterns, overwritten).  Defined in cast_kernels.hip.
int fold_colmax(const void *partials, int64_t slots, int64_t C, float *col_amax, hipStream_t st);

// Looks up, for the current device, the address of the static scratch array of l8_cast_rowwise_noalloc.
// Defined in cast_kernels.hip; l8_device_check calls it so that the look-up happens at set-up.
int noalloc_setup_current_device();

// ---- device side ----------------------------------------------------------
#define L8_DEV __device__ __forceinline__

constexpr float kEps = 1e-12f;       // lingua/float8.py:11
constexpr float kE4M3Max = 448.0f;   // torch.finfo(float8_e4m3fn).max

L8_DEV float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// scale = clamp(f32(amax), min=EPS) / 448 (lingua/float8.py:44-45).  NaN passes through the clamp, as torch.clamp
// does.  Rule L8_SCALE_RULE_DIVIDE is the correctly rounded division, which is what the ATen CPU kernel computes;
// rule L8_SCALE_RULE_TIMES_INVERSE is what the ATen GPU kernel computes for a division by a Python scalar: the product
// with fp32(1/448), which differs from the quotient in the last bit for about half of all amaxes.
constexpr float kInvE4M3Max = 1.0f / 448.0f;
L8_DEV float scale_from_amax(float amax, int scale_rule) {
  float a = (amax < kEps) ? kEps : amax;
  return scale_rule == L8_SCALE_RULE_TIMES_INVERSE ? a * kInvE4M3Max : a / kE4M3Max;
}
L8_DEV float recip_exact(float s) { return 1.0f / s; }

// Integer restatement of the fp32 -> e4m3fn conversion of the ATen cast used at
// lingua/float8.py:46 (round to nearest even, |v| >= 480 and NaN/inf -> NaN
// code, sign kept).  Used where an operand is not finite or may exceed the
// finite range; the hardware converter handles every in-range value.
L8_DEV uint32_t e4m3fn_from_f32_slow(float v) {
  const uint32_t w = __float_as_uint(v);
  const uint32_t sign = (w >> 24) & 0x80u;
  const uint32_t mag = w & 0x7fffffffu;
  if (mag >= 0x43F00000u) return sign | 0x7Fu;
  const int e = (int)(mag >> 23);
  const uint32_t frac = mag & 0x7fffffu;
  if (e >= 121) {
    uint32_t t = ((uint32_t)(e - 120) << 23) | frac;
    t += 0x7ffffu + ((t >> 20) & 1u);
    return sign | (t >> 20);
  }
  if (e < 116) return sign;
  const uint32_t sig = frac | 0x800000u;
  const int sh = 141 - e;
  uint32_t q = sig >> sh;
  const uint32_t rem = sig & ((1u << sh) - 1u);
  const uint32_t half = 1u << (sh - 1);
  if (rem > half || (rem == half && (q & 1u))) q += 1;
  return sign | q;
}

// Two bf16 values packed in one dword (element 0 in the low half) times recip
// -> two e4m3 bytes in the low or high half of `old`.  The fp32 product is
// rounded to fp32 before the conversion, as the reference's `mul` then
// `_to_copy` do.
template <bool HI>
L8_DEV int cvt2(uint32_t packed, float recip, int old) {
  const float lo = __uint_as_float(packed << 16) * recip;
  const float hi = __uint_as_float(packed & 0xffff0000u) * recip;
  return __builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, old, HI);
}

L8_DEV int cvt2_slow(uint32_t packed, float recip) {
  const float lo = __uint_as_float(packed << 16) * recip;
  const float hi = __uint_as_float(packed & 0xffff0000u) * recip;
  return (int)(e4m3fn_from_f32_slow(lo) | (e4m3fn_from_f32_slow(hi) << 8));
}

// 8 bf16 (one 16-byte load) -> 8 e4m3 bytes (one 8-byte store)
L8_DEV v2i cvt8(v4i x, float recip) {
  v2i r;
  int a = cvt2<false>((uint32_t)x[0], recip, 0);
  r[0] = cvt2<true>((uint32_t)x[1], recip, a);
  int b = cvt2<false>((uint32_t)x[2], recip, 0);
  r[1] = cvt2<true>((uint32_t)x[3], recip, b);
  return r;
}
L8_DEV v2i cvt8_slow(v4i x, float recip) {
  v2i r;
  r[0] = cvt2_slow((uint32_t)x[0], recip) | (cvt2_slow((uint32_t)x[1], recip) << 16);
  r[1] = cvt2_slow((uint32_t)x[2], recip) | (cvt2_slow((uint32_t)x[3], recip) << 16);
  return r;
}

// max of |a| and |b| on two packed bf16 lanes at once: non-negative bf16 bit
// patterns order like unsigned 16-bit integers, and NaN patterns (> 0x7f80)
// sort above every number, so an integer max is a NaN-propagating amax.
L8_DEV uint32_t pk_absmax_u16(uint32_t acc, uint32_t x) {
  typedef unsigned short us2 __attribute__((ext_vector_type(2)));
  const uint32_t ax = x & 0x7fff7fffu;
  us2 a = __builtin_bit_cast(us2, acc), b = __builtin_bit_cast(us2, ax);
  us2 m = __builtin_elementwise_max(a, b);
  return __builtin_bit_cast(uint32_t, m);
}

// max over the 64 lanes of a wave, result uniform (DPP inside rows of 16,
// then four lane reads).
L8_DEV uint32_t wave_max_u32(uint32_t v) {
  int x = (int)v;
  auto step = [&](int moved) { x = (int)max((uint32_t)x, (uint32_t)moved); };
  step(__builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  step(__builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  step(__builtin_amdgcn_update_dpp(0, x, 0x124, 0xF, 0xF, true));  // row_ror:4
  step(__builtin_amdgcn_update_dpp(0, x, 0x128, 0xF, 0xF, true));  // row_ror:8
  uint32_t a = (uint32_t)__builtin_amdgcn_readlane(x, 0);
  uint32_t b = (uint32_t)__builtin_amdgcn_readlane(x, 16);
  uint32_t c = (uint32_t)__builtin_amdgcn_readlane(x, 32);
  uint32_t d = (uint32_t)__builtin_amdgcn_readlane(x, 48);
  return max(max(a, b), max(c, d));
}

// fp32 -> bf16 bits, round to nearest even (what a PyTorch op leaves when its fp32 result lands in a bf16 tensor)
L8_DEV uint32_t bf16_rne_bits(float v) {
  const __bf16 b = (__bf16)v;
  return (uint32_t) __builtin_bit_cast(unsigned short, b);
}
L8_DEV float bf16_round(float v) { return bf16_bits_to_f32(bf16_rne_bits(v)); }

// amax bits (uniform) -> scale, 1/scale, finite flag, as in the row-wise cast
struct RowScale {
  float s, recip;
  bool finite;
};
L8_DEV RowScale row_scale(uint32_t amax_bits, int scale_rule) {
  RowScale r;
  r.finite = amax_bits < 0x7f80u;
  r.s = r.finite ? scale_from_amax(bf16_bits_to_f32(amax_bits), scale_rule)
                 : __uint_as_float(amax_bits == 0x7f80u ? 0x7f800000u : 0x7fc00000u);
  r.recip = recip_exact(r.s);
  return r;
}

// Buffer descriptor over `bytes` bytes at p (raw: no stride, no swizzle).  A load through it whose byte offset --
// the lane's plus the scalar one -- reaches `bytes` returns zeros (dword by dword), a store there is dropped: kernels
// use that instead of a branch around the access, which keeps the compiler's count of outstanding loads exact.
// The type exists only in the device pass.
#if defined(__HIP_DEVICE_COMPILE__)
L8_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), (short)0, (int)bytes, 0x00020000);
}
// one 16-byte non-temporal load: lane offset voff, scalar offset soff (bytes)
L8_DEV v4i load16_nt(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
  return __builtin_amdgcn_raw_buffer_load_b128(rs, (int)voff, (int)soff, 2 /* cache policy: non-temporal */);
}
// One 8-byte store at lane offset voff (dropped beyond the descriptor's range).  An ordinary store, not a non-temporal
// one: inside the MLP step the row-wise casts ran 2-5 % faster with it (the output is the next GEMM's operand).
L8_DEV void store8(__amdgpu_buffer_rsrc_t rs, uint32_t voff, v2i data) {
  __builtin_amdgcn_raw_buffer_store_b64(data, rs, (int)voff, 0, 0);
}
#endif

// Workgroup-per-row kernels that produce their row on the fly (fused gate, fused
// norm) keep column maxima in registers (packed pairs, NCHW * 4 dwords per
// tensor) while that fits the 256-register budget of two workgroups per CU,
// else in a dynamic LDS array of one bf16 per column and tensor; either way
// every column belongs to exactly one thread, so no synchronisation is involved.
template <int NCHW, int TENSORS>
constexpr bool colmax_in_lds() { return NCHW * 4 * TENSORS > 32; }

}  // namespace l8
