// fp8 (e4m3fn) x fp8 -> bf16 "NT" GEMM on the gfx950 matrix cores.
//
//   C[m,n] = bf16( (sum_k A[m,k] * B[n,k]) * sa[m|0] * sb[n|0] + bias[n] )
//
// Stands in for torch._scaled_mm and the manual post-scaling around it at
// lingua/float8.py:65-77 (forward: row x row scales, bias fused; dgrad: row x
// scalar scales) and serves the fp8 wgrad (row x row scales, reduction over
// tokens).
//
// Structure
//   * workgroup tile BM x BN, K consumed in tiles of 64 bytes (one
//     v_mfma_f32_32x32x64_f8f6f4 deep), WM x WN wavefronts, each owning
//     TM x TN accumulator tiles of 32x32;
//   * global -> LDS by `buffer_load_dwordx4 ... lds` (no staging registers)
//     into a ring of NS stages.  Measured round-trip latency of a K tile under
//     load is well above the matrix-core time of one tile, so NS-1 tiles are
//     kept in flight; waits are partial (`s_waitcnt vmcnt(n)`), one barrier
//     per K tile;
//   * fragments are software-pipelined: right after the barrier that
//     publishes tile k+1, its fragments are read from LDS into a second
//     register set while the matrix cores work on tile k from the first;
//   * LDS rows are 64 bytes (4 chunks of 16 B); chunk c of row r lives at
//     position c ^ ((r >> 2) & 3): the 16-byte fragment reads of any 16
//     consecutive rows then cover all 64 banks once (no conflicts, checked
//     with SQ_LDS_BANK_CONFLICT).  The permutation is applied on the global
//     address side because the LDS side of a direct load is lane-linear;
//   * the matrix cores compute the tile transposed (D[n][m]) so that each lane
//     ends up with 4 consecutive n per accumulator quad; a v_permlane32_swap
//     pairs lanes l / l+32 into 16 consecutive n, scaled, rounded to bf16 and
//     stored as two 16-byte writes per 32x32 tile;
//   * workgroup -> tile mapping is XCD-aware: the 8 XCDs each get a contiguous
//     range of a grouped (GROUP_M tall) tile order so that the workgroups
//     resident on one XCD share A and B panels in that XCD's L2.
//
// L8_GEMM_DIAG (compile-time, never set in the shipped build) removes one side
// of the main loop to attribute stalls: 1 = no global loads after the prologue,
// 2 = no LDS reads / matrix-core work, 3 = no stores of C, 4 / 5 = as 2 with every workgroup (4) or every XCD (5)
// loading the same tile (all L2 hits).  Results are wrong by construction.
#include "l8_common.h"

namespace l8 {

struct GemmArgs {
  const uint8_t *A, *B;
  int M, N, K;
  int64_t lda, ldb, ldc;
  const float *sa, *sb;
  int sa_row, sb_row;
  const uint16_t *bias;
  uint16_t *C;
  int tiles_m, tiles_n;
};

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// The buffer-resource type and the matrix-core builtins exist only in the
// device pass; the host pass sees empty kernel bodies (it needs the symbols only).
#if defined(__HIP_DEVICE_COMPILE__)
L8_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), (short)0, (int)bytes, 0x00020000);
}
#endif

constexpr uint32_t kOOB = 0x80000000u;  // voffset that is out of range for every resource below

#ifndef L8_GEMM_DIAG
#define L8_GEMM_DIAG 0
#endif

// s_waitcnt for vmcnt <= n and lgkmcnt == 0 (expcnt untouched)
#define L8_WAIT_VM_LGKM0(n) \
  __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (0x7 << 4) | (0x0 << 8) | ((((n) >> 4) & 0x3) << 14))

#if defined(__HIP_DEVICE_COMPILE__)
// Scheduling recipe for one half trip: N_MMA groups of "one MFMA, then a share
// of the N_DSR LDS reads (spread over the first N_MMA-2 groups), then one of
// the N_VMEM global loads".  The group sizes must be literals, hence the recursion.
template <int N_MMA, int N_DSR, int N_VMEM, int I>
L8_DEV void interleave_step() {
  if constexpr (I < N_MMA) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    constexpr int slots = N_MMA > 2 ? N_MMA - 2 : 1;
    constexpr int r0 = (N_DSR * I) / slots, r1 = (N_DSR * (I + 1)) / slots;
    if constexpr (I < slots && r1 > r0) __builtin_amdgcn_sched_group_barrier(0x100, r1 - r0, 0);
    if constexpr (I < N_VMEM) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    interleave_step<N_MMA, N_DSR, N_VMEM, I + 1>();
  }
}
#endif

template <int WM, int WN, int TM, int TN, int NS, int GROUP_M>
__global__ __launch_bounds__(WM *WN * 64) void gemm_nt_kernel(const GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BK = 64;
  constexpr int NW = WM * WN;
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK, STAGE = A_BYTES + B_BYTES;
  static_assert((BM / 16) % NW == 0 && (BN / 16) % NW == 0, "tile rows must split evenly over waves");
  constexpr int NA = BM / 16 / NW, NB = BN / 16 / NW;  // 1 KiB wave loads (16 rows x 64 B) per stage per wave
  constexpr int LPT = NA + NB;                         // loads per K tile per wave
  static_assert(NS >= 2 && (NS - 1) * LPT <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;

  // ---- XCD-aware, grouped workgroup -> tile mapping ----
  int tile_m, tile_n;
  {
    const int nb = p.tiles_m * p.tiles_n;
    const int pid = blockIdx.x;
    const int q = nb >> 3, rem = nb & 7;
    const int xcd = pid & 7, loc = pid >> 3;
    const int lin = (xcd < rem) ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int per_group = GROUP_M * p.tiles_n;
    const int grp = lin / per_group;
    const int first_m = grp * GROUP_M;
    const int gsz = (p.tiles_m - first_m < GROUP_M) ? p.tiles_m - first_m : GROUP_M;
    const int in_grp = lin - grp * per_group;
    tile_m = first_m + in_grp % gsz;
    tile_n = in_grp / gsz;
  }
  if (L8_GEMM_DIAG == 4 || L8_GEMM_DIAG == 5) { tile_m = 0; tile_n = (L8_GEMM_DIAG == 5) ? (int)(blockIdx.x & 7) : 0; }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // ---- global -> LDS load plan ----
  // lane l of a wave load fills LDS row l/4, position l%4 of a 16-row group
  const int lrow = lane >> 2, lpos = lane & 3;
  const int lchunk = lpos ^ ((lrow >> 2) & 3);  // which 16-byte chunk of the row this lane fetches
  const uint8_t *Ablk = p.A + (int64_t)m0 * p.lda;
  const uint8_t *Bblk = p.B + (int64_t)n0 * p.ldb;
  const int64_t a_left = (int64_t)(p.M - m0 - 1) * p.lda + p.K;
  const int64_t b_left = (int64_t)(p.N - n0 - 1) * p.ldb + p.K;
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(Ablk, a_left < 0x7fffffff ? (uint32_t)a_left : 0x7fffffffu);
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(Bblk, b_left < 0x7fffffff ? (uint32_t)b_left : 0x7fffffffu);

  uint32_t a_voff[NA], b_voff[NB];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int row = (wave * NA + i) * 16 + lrow;
    a_voff[i] = (m0 + row < p.M) ? (uint32_t)(row * (int)p.lda + lchunk * 16) : kOOB;
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int row = (wave * NB + i) * 16 + lrow;
    b_voff[i] = (n0 + row < p.N) ? (uint32_t)(row * (int)p.ldb + lchunk * 16) : kOOB;
  }

  const int KT = (p.K + BK - 1) / BK;
  // Every call issues exactly LPT loads so that the vmcnt arithmetic below is
  // uniform; tiles at or beyond KT, rows beyond M / N and chunks beyond K use
  // an out-of-range offset, which the buffer unit turns into zeros in LDS.
  auto issue = [&](int kt) {
    const int stage = kt % NS;
    const int k0 = kt * BK;
    uint8_t *sA = smem + stage * STAGE + wave * (NA * 1024);
    uint8_t *sB = smem + stage * STAGE + A_BYTES + wave * (NB * 1024);
    // per-lane mask: chunks at or beyond K (partial last tile, tiles past the end) go out of range
    const uint32_t kmask = (k0 + lchunk * 16 < p.K) ? 0u : kOOB;
#pragma unroll
    for (int i = 0; i < NA; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (lds_ptr_t)(sA + i * 1024), 16, a_voff[i] | kmask, k0, 0, 0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, (lds_ptr_t)(sB + i * 1024), 16, b_voff[i] | kmask, k0, 0, 0);
  };

  // ---- LDS -> register fragment plan ----
  const int l31 = lane & 31, h = lane >> 5;
  const int fr = (l31 >> 2) & 3;
  const int foff0 = l31 * BK + (((h * 2 + 0) ^ fr) * 16);
  const int foff1 = l31 * BK + (((h * 2 + 1) ^ fr) * 16);
  const int a_base = wm * (TM * 32 * BK);
  const int b_base = A_BYTES + wn * (TN * 32 * BK);

  auto read_frags = [&](int kt, v8i (&af)[TM], v8i (&bf)[TN]) {
    const uint8_t *st = smem + (kt % NS) * STAGE;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const v4i lo = *(const v4i *)(st + a_base + tm * (32 * BK) + foff0);
      const v4i hi = *(const v4i *)(st + a_base + tm * (32 * BK) + foff1);
      af[tm] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const v4i lo = *(const v4i *)(st + b_base + tn * (32 * BK) + foff0);
      const v4i hi = *(const v4i *)(st + b_base + tn * (32 * BK) + foff1);
      bf[tn] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  v16f acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

  auto mma = [&](v8i (&af)[TM], v8i (&bf)[TN]) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        // D[i = n][j = m]: B rows feed the "A" port, A rows the "B" port
        acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[tn], af[tm], acc[tn][tm], 0, 0, 0, 0, 0, 0);
  };

  // Ring bookkeeping.  Tile t lives in stage t % NS; each wave issues LPT
  // loads per tile, in tile order.  At the top of iteration kt the loads of
  // tiles kt+1 .. kt+NS-1 may be outstanding; waiting until at most
  // (NS-2)*LPT remain means this wave's part of tile kt+1 has landed, and the
  // barrier extends that to every wave.  The same wait also drains this wave's
  // LDS reads of tile kt (lgkmcnt 0), so after the barrier every wave holds
  // tile kt in registers and stage kt % NS can be refilled with tile kt+NS.
  // The empty asm statements keep the compiler from moving LDS accesses across.
#define L8_PUBLISH_NEXT()                  \
  do {                                     \
    L8_WAIT_VM_LGKM0((NS - 2) * LPT);      \
    asm volatile("" ::: "memory");         \
    __builtin_amdgcn_s_barrier();          \
    asm volatile("" ::: "memory");         \
  } while (0)

  // prologue: all NS stages in flight, tile 0 published and read
#pragma unroll
  for (int t = 0; t < NS; ++t) issue(t);
  v8i af0[TM], bf0[TN], af1[TM], bf1[TN];
  L8_WAIT_VM_LGKM0((NS - 1) * LPT);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_frags(0, af0, bf0);

  // Issue order inside one half trip.  A wave issues in order, and right after
  // the barrier all waves push their LDS reads at once; if those came first,
  // each wave's matrix-core work would wait behind the whole backlog.  So the
  // reads (and the global loads) are spread between the MFMAs, which need
  // nothing but registers that are already valid.
  constexpr int N_MMA = TM * TN, N_DSR = 2 * (TM + TN);
  auto interleave = [&]() { interleave_step<N_MMA, N_DSR, (L8_GEMM_DIAG == 1 ? 0 : LPT), 0>(); };

  // Two tiles per trip so that the two fragment sets keep fixed registers.  An
  // odd tile count is rounded up: the extra tile was loaded out of range, i.e.
  // as zeros, and adds nothing.
  for (int kt = 0; kt < KT; kt += 2) {
    // matrix cores on tile kt (set 0) while tile kt+1 is read into set 1
    L8_PUBLISH_NEXT();
    if (L8_GEMM_DIAG != 1) issue(kt + NS);
    if (L8_GEMM_DIAG != 2 && L8_GEMM_DIAG != 4 && L8_GEMM_DIAG != 5) {
      read_frags(kt + 1, af1, bf1);
      mma(af0, bf0);
      interleave();
    }
    __builtin_amdgcn_sched_barrier(0);
    // matrix cores on tile kt+1 (set 1) while tile kt+2 is read into set 0
    L8_PUBLISH_NEXT();
    if (L8_GEMM_DIAG != 1) issue(kt + 1 + NS);
    if (L8_GEMM_DIAG != 2 && L8_GEMM_DIAG != 4 && L8_GEMM_DIAG != 5) {
      read_frags(kt + 2, af0, bf0);
      mma(af1, bf1);
      interleave();
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // drain the tail loads (out of range, zero-filling) before LDS is released
  L8_WAIT_VM_LGKM0(0);

  // ---- epilogue ----
  // lane (l31, h) of tile (tn, tm) holds m = l31 and, in accumulator quad qd,
  // n = 8*qd + 4*h + {0..3}.  After the half-wave swap, lanes with h == 0 hold
  // n = 0..15 and lanes with h == 1 hold n = 16..31 of row m.
  const float sa_s = p.sa[0], sb_s = p.sb[0];
  float sav[TM];
  bool m_okv[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int m = m0 + (wm * TM + tm) * 32 + l31;
    m_okv[tm] = m < p.M;
    sav[tm] = p.sa_row ? (m_okv[tm] ? p.sa[m] : 0.0f) : sa_s;
  }
  const bool c_vec = (p.ldc % 8 == 0) && (((uintptr_t)p.C & 15) == 0);
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int nt0 = n0 + (wn * TN + tn) * 32;
    // scales and bias of the 16 n this lane holds before the swap
    float sbv[4][4], biasv[4][4];
#pragma unroll
    for (int qd = 0; qd < 4; ++qd)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = nt0 + 8 * qd + 4 * h + e;
        const bool n_ok = n < p.N;
        sbv[qd][e] = p.sb_row ? (n_ok ? p.sb[n] : 0.0f) : sb_s;
        biasv[qd][e] = (p.bias && n_ok) ? bf16_bits_to_f32(p.bias[n]) : 0.0f;
      }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const int m = m0 + (wm * TM + tm) * 32 + l31;
      const float sa = sav[tm];
      uint32_t pk[8];  // quad qd -> pk[2qd], pk[2qd+1]
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[tn][tm][qd * 4 + e] * sa * sbv[qd][e] + biasv[qd][e];
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        bf2 lo = {(__bf16)v[0], (__bf16)v[1]}, hi = {(__bf16)v[2], (__bf16)v[3]};
        pk[2 * qd] = __builtin_bit_cast(uint32_t, lo);
        pk[2 * qd + 1] = __builtin_bit_cast(uint32_t, hi);
      }
      // swap: (quad0 of upper lanes) <-> (quad2 of lower lanes); (quad1 upper) <-> (quad3 lower)
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        auto r0 = __builtin_amdgcn_permlane32_swap(pk[0 + d], pk[4 + d], false, false);
        pk[0 + d] = r0[0];
        pk[4 + d] = r0[1];
        auto r1 = __builtin_amdgcn_permlane32_swap(pk[2 + d], pk[6 + d], false, false);
        pk[2 + d] = r1[0];
        pk[6 + d] = r1[1];
      }
      // lower lanes: pk[0,1]=n0..3 pk[4,5]=n4..7 pk[2,3]=n8..11 pk[6,7]=n12..15
      // upper lanes: pk[0,1]=n16..19 pk[4,5]=n20..23 pk[2,3]=n24..27 pk[6,7]=n28..31
      const int nbase = nt0 + 16 * h;
      if (m_okv[tm] && (L8_GEMM_DIAG != 3 || pk[0] == 0x12345678u)) {
        uint16_t *dst = p.C + (int64_t)m * p.ldc + nbase;
        if (c_vec && nbase + 16 <= p.N) {
          *(v4i *)dst = v4i{(int)pk[0], (int)pk[1], (int)pk[4], (int)pk[5]};
          *(v4i *)(dst + 8) = v4i{(int)pk[2], (int)pk[3], (int)pk[6], (int)pk[7]};
        } else {
          const uint32_t all[8] = {pk[0], pk[1], pk[4], pk[5], pk[2], pk[3], pk[6], pk[7]};
#pragma unroll
          for (int e = 0; e < 16; ++e)
            if (nbase + e < p.N) dst[e] = (uint16_t)(all[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
  }
#else
  (void)p;
#endif
}

// ---------------------------------------------------------------------------
// tile configurations ("algos")
// ---------------------------------------------------------------------------
typedef void (*gemm_fn)(const GemmArgs);
struct Algo {
  const char *name;
  gemm_fn fn;
  int bm, bn, threads, lds;
};

// X(WM, WN, TM, TN, NS, GROUP_M) -- 1-based position in this list is the `algo` number
#define L8_ALGO_LIST(X)                                                      \
  X(2, 4, 4, 2, 4, 8)  /* 1: 256x256, 8 waves (128x64 each), 4 stages     */ \
  X(2, 4, 4, 2, 5, 8)  /* 2: same, 5 stages (all 160 KiB of LDS)          */ \
  X(2, 2, 4, 4, 4, 8)  /* 3: 256x256, 4 waves (128x128 each), 4 stages    */ \
  X(2, 2, 4, 4, 5, 8)  /* 4: same, 5 stages                               */ \
  X(2, 2, 2, 2, 4, 8)  /* 5: 128x128, 4 waves (small problems)            */ \
  X(4, 2, 2, 4, 4, 8)  /* 6: 256x256, 8 waves (64x128 each), 4 stages     */ \
  X(2, 4, 4, 2, 3, 8)  /* 7: algo 1 with 3 stages                         */ \
  X(2, 4, 4, 2, 4, 4)  /* 8: algo 1 with shorter groups                   */ \
  X(2, 4, 4, 2, 4, 16) /* 9: algo 1 with taller groups                    */

#define L8_INSTANTIATE(WM, WN, TM, TN, NS, GM) \
  template __global__ void gemm_nt_kernel<WM, WN, TM, TN, NS, GM>(const GemmArgs);
L8_ALGO_LIST(L8_INSTANTIATE)

#define L8_ALGO_ROW(WM, WN, TM, TN, NS, GM)                                                        \
  {"mt" #WM "x" #WN "w_" #TM "x" #TN "t_ns" #NS "_g" #GM, gemm_nt_kernel<WM, WN, TM, TN, NS, GM>, \
   WM * TM * 32, WN * TN * 32, WM * WN * 64, NS * (WM * TM * 32 + WN * TN * 32) * 64},

static const Algo kAlgos[] = {L8_ALGO_LIST(L8_ALGO_ROW)};
constexpr int kNumAlgos = sizeof(kAlgos) / sizeof(kAlgos[0]);

}  // namespace l8

using namespace l8;

extern "C" int l8_gemm_algo_count(void) { return kNumAlgos; }
extern "C" const char *l8_gemm_algo_name(int algo) {
  return (algo >= 1 && algo <= kNumAlgos) ? kAlgos[algo - 1].name : nullptr;
}

static int pick_algo(int64_t M, int64_t N, int64_t K) {
  (void)K;
  // large problems: 256x256; problems that would leave most of the chip idle
  // with big tiles: 128x128
  const int64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (big_tiles >= num_cus()) return 1;
  return 5;
}

extern "C" int l8_gemm_nt(const void *A, const void *B, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                          const float *sa, int sa_mode, const float *sb, int sb_mode, const void *bias, void *C,
                          int64_t ldc, int algo, void *stream) {
  L8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "l8_gemm_nt: negative shape");
  if (M == 0 || N == 0) return L8_OK;
  L8_REQUIRE(A && B && C && sa && sb, "l8_gemm_nt: null pointer");
  L8_REQUIRE(K > 0, "l8_gemm_nt: K must be positive");
  L8_REQUIRE(K % 16 == 0, "l8_gemm_nt: K=%lld must be a multiple of 16", (long long)K);
  L8_REQUIRE(lda % 16 == 0 && ldb % 16 == 0 && lda >= K && ldb >= K, "l8_gemm_nt: lda=%lld, ldb=%lld must be multiples of 16 and >= K",
             (long long)lda, (long long)ldb);
  L8_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)B % 16) == 0, "l8_gemm_nt: A and B must be 16-byte aligned");
  L8_REQUIRE(ldc >= N, "l8_gemm_nt: ldc=%lld < N=%lld", (long long)ldc, (long long)N);
  L8_REQUIRE((sa_mode == L8_SCALE_SCALAR || sa_mode == L8_SCALE_ROW) && (sb_mode == L8_SCALE_SCALAR || sb_mode == L8_SCALE_ROW),
             "l8_gemm_nt: bad scale mode");
  L8_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31), "l8_gemm_nt: dimension too large");
  L8_REQUIRE(algo >= 0 && algo <= kNumAlgos, "l8_gemm_nt: algo %d out of range 0..%d", algo, kNumAlgos);
  if (algo == 0) algo = pick_algo(M, N, K);
  const Algo &al = kAlgos[algo - 1];
  // 32-bit in-tile byte offsets: (tile rows) * ld + K must stay below 2^31
  L8_REQUIRE((int64_t)al.bm * lda + K < (1LL << 31) && (int64_t)al.bn * ldb + K < (1LL << 31),
             "l8_gemm_nt: leading dimension too large for 32-bit tile offsets");
  GemmArgs p;
  p.A = (const uint8_t *)A;
  p.B = (const uint8_t *)B;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.lda = lda;
  p.ldb = ldb;
  p.ldc = ldc;
  p.sa = sa;
  p.sb = sb;
  p.sa_row = sa_mode == L8_SCALE_ROW;
  p.sb_row = sb_mode == L8_SCALE_ROW;
  p.bias = (const uint16_t *)bias;
  p.C = (uint16_t *)C;
  p.tiles_m = (int)((M + al.bm - 1) / al.bm);
  p.tiles_n = (int)((N + al.bn - 1) / al.bn);
  const int64_t nblocks = (int64_t)p.tiles_m * p.tiles_n;
  L8_REQUIRE(nblocks < (1LL << 31), "l8_gemm_nt: too many tiles");
  static bool attr_done[kNumAlgos] = {};
  if (!attr_done[algo - 1]) {  // idempotent; a race only repeats the call
    L8_HIP(hipFuncSetAttribute((const void *)al.fn, hipFuncAttributeMaxDynamicSharedMemorySize, al.lds));
    attr_done[algo - 1] = true;
  }
  hipLaunchKernelGGL(al.fn, dim3((unsigned)nblocks), dim3(al.threads), al.lds, (hipStream_t)stream, p);
  L8_HIP(hipGetLastError());
  return L8_OK;
}
