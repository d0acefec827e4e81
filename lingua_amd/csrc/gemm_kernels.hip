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
//   * workgroup tile BM x BN, K consumed in tiles of 128 bytes (two
//     v_mfma_f32_32x32x64_f8f6f4 steps), WM x WN wavefronts, each owning
//     TM x TN accumulator tiles of 32x32;
//   * global -> LDS by `buffer_load_dwordx4 ... lds` (no staging registers).
//     Each row segment is a full 128-byte line: 64-byte segments halve the
//     L2 request rate that can be sustained (measured).  LDS is a ring of R
//     slots, each holding the A or the B panel of one K tile; units are
//     issued in the order A(0), B(0), A(1), ...  With R = 5 the ring holds the
//     K tile being read, the K tile being published and one more unit, so
//     loads stay in flight across every barrier; waits are partial
//     (`s_waitcnt vmcnt(n)`), one barrier per K tile;
//   * fragments are software-pipelined through two register sets: each half
//     of a trip runs the MFMAs of one 64-byte step while the next step is
//     read from LDS.  A wave issues in order, so the instruction stream is
//     laid out by hand as groups of one MFMA + its share of the LDS reads +
//     its share of the panel loads, with scheduling fences between groups:
//     one unit is requested during each half of a trip.  (Requesting both
//     units in a burst after the barrier left the waves queueing at the
//     vector-memory port with idle matrix cores: 2830 -> 2310 shader clocks
//     per trip, the matrix cores alone need 2048.);
//   * LDS rows are 128 bytes (8 chunks of 16 B); chunk c of row r lives at
//     position c ^ f(r), f(r) = (r & 7) ^ ((r >> 3) & 1): the 16-byte
//     fragment reads of any 16 consecutive rows then cover all 64 banks once
//     (SQ_LDS_BANK_CONFLICT = 0; f(r) = r & 7 alone measured 50 % conflict
//     cycles).  The permutation is applied on the global address side because
//     the LDS side of a direct load is lane-linear;
//   * the matrix cores compute the tile transposed (D[n][m]) so that each lane
//     ends up with 4 consecutive n per accumulator quad; a v_permlane32_swap
//     pairs lanes l / l+32 into 16 consecutive n.  The scaled, bf16-rounded
//     C tile is staged through the (by then idle) LDS ring and leaves as
//     whole rows, 1 KiB of consecutive bytes per wave store;
//   * workgroup -> tile mapping is XCD-aware: the 8 XCDs each get a contiguous
//     range of a grouped (GROUP_M tall) tile order so that the workgroups
//     resident on one XCD share A and B panels in that XCD's L2.
//
// L8_GEMM_DIAG (compile-time, never set in the shipped build) removes one side
// of the main loop to attribute stalls: 1 = no global loads after the prologue,
// 2 = no LDS reads / matrix-core work, 3 = no stores of C, 4 = as 2 with every workgroup loading the same tile (all
// L2 hits).  Results are wrong by construction.
#include <atomic>
#include <type_traits>

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
  uint64_t *dbg;  // L8_GEMM_PROF builds only
  // persistent kernels, optional (null = every tile is computed by one workgroup): workspace for tiles whose
  // K range is shared out over several workgroups -- one flag and one fp32 tile of partial sums per workgroup
  uint32_t *sk_flags;
  float *sk_partials;
  uint32_t sk_epoch;  // value that marks a flag as set in THIS launch (never 0; flags are never cleared)
  int sk_wait_limit;  // polls of a flag before the waiting workgroup gives up and poisons its tile
};

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// The buffer-resource type and the matrix-core builtins exist only in the
// device pass; the host pass sees empty kernel bodies (it needs the symbols only).

// 16-byte-per-lane buffer store with a scalar-register offset, followed by two wait states.  A vector-ALU write to
// one of the store's data registers right behind it can reach the register before the store has read it: with two
// waves per SIMD the eight-wave kernel stored, now and then, the next row pair's values in 4 of 64 lanes (found by
// the exact-integer tests; two wait states cure it, which is what the compiler's hazard recognizer inserts behind
// stores of more than 8 bytes -- except behind buffer stores whose soffset is a register, like these, which an old
// rule exempts).  Every such store in this file goes through here.
#if defined(__HIP_DEVICE_COMPILE__)
template <int AUX>
L8_DEV void store16_aux(v4i data, __amdgpu_buffer_rsrc_t rs, uint32_t voff, int soff) {
  __builtin_amdgcn_raw_buffer_store_b128(data, rs, voff, soff, AUX);
  asm volatile("s_nop 1" : : "v"(data));  // the operand keeps every later write to these registers behind the wait
}
#endif
#define store16(data, rs, voff, soff, aux) store16_aux<aux>(data, rs, voff, soff)

[[maybe_unused]] constexpr uint32_t kOOB = 0x80000000u;
// cache policy of a buffer access that must be coherent over the whole device (sc0 | sc1)
[[maybe_unused]] constexpr int kCoherent = 1 | 16;
// Sharing out the K range of the last, partly filled round of tiles: what a partial tile costs its writer and its
// reader, in K tiles' time (256 KiB leave a compute unit at ~16 bytes per clock), and the least number of K tiles
// the split must take off the owners of the tail tiles to be used at all.
[[maybe_unused]] constexpr int kSkWriteCost = 8, kSkFixCost = 4, kSkMinSaved = 16;
// Workspace layout: kSkMaxGrid flag words (one per tail-tile slot), then 64 words of which the first counts the
// tiles whose owner gave up waiting for a helper (and stored NaNs), then the fp32 tiles of partial sums.
[[maybe_unused]] constexpr int kSkMaxGridWords = 1024, kSkGaveUpWord = kSkMaxGridWords;

#ifndef L8_GEMM_DIAG
#define L8_GEMM_DIAG 0
#endif
#ifndef L8_STRADDLE
#define L8_STRADDLE 2
#endif
// groups (of one MFMA each) of a half trip over which the persistent kernel issues the half's LDS reads
#ifndef L8_READ_GROUPS
#define L8_READ_GROUPS 13
#endif
// L8_GEMM_PROF (compile-time, never set in the shipped build): the persistent kernel takes the `bias` pointer for
// a buffer of 16 x uint64 per workgroup and records wall-clock ticks (100 MHz) at its start, after the prologue
// and at its end, and shader-clock cycles spent in the K loops and in the C-tile stores.
#ifndef L8_GEMM_PROF
#define L8_GEMM_PROF 0
#endif

// s_waitcnt for vmcnt <= n and lgkmcnt == 0 (expcnt untouched)
#define L8_WAIT_VM_LGKM0(n) \
  __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (0x7 << 4) | (0x0 << 8) | ((((n) >> 4) & 0x3) << 14))

template <int WM, int WN, int TM, int TN, int R, int GROUP_M, int PF>
__global__ __launch_bounds__(WM *WN * 64) void gemm_nt_kernel(const GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BK = 128;
  constexpr int NW = WM * WN;
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  constexpr int UNIT = A_BYTES > B_BYTES ? A_BYTES : B_BYTES;  // one ring slot holds an A or a B panel of one K tile
  static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "tile rows must split evenly over waves");
  constexpr int NA = BM / 8 / NW, NB = BN / 8 / NW;  // 1 KiB wave loads (8 rows x 128 B) per panel per wave
  // L2 touches (PF > 0): one lane per panel row, every wave covers 64 rows per instruction
  constexpr int PFA = PF > 0 ? (BM + NW * 64 - 1) / (NW * 64) : 0, PFB = PF > 0 ? (BN + NW * 64 - 1) / (NW * 64) : 0;
  constexpr int IA = NA + PFA, IB = NB + PFB;  // vector-memory instructions per unit per wave
  // loads of the units that may still be in flight when a K tile is published:
  // the ring holds the tile being read (2 slots), the tile being published (2
  // slots) and R-4 younger units, the first of which is an A panel
  constexpr int PEND = ((R - 4 + 1) / 2) * IA + ((R - 4) / 2) * IB;
  constexpr int PEND0 = ((R - 3 + 1) / 2) * IA + ((R - 3) / 2) * IB;  // same for the prologue (R-3 younger units)
  static_assert(R >= 4 && PEND0 <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;

  // ---- XCD-aware, grouped workgroup -> tile mapping ----
  int tile_m, tile_n, row_in_group;
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
    row_in_group = in_grp % gsz;
    tile_m = first_m + row_in_group;
    tile_n = in_grp / gsz;
  }
  if (L8_GEMM_DIAG == 4) { tile_m = 0; tile_n = 0; }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // ---- global -> LDS load plan ----
  // lane l of a wave load fills LDS row l/8, position l%8 of an 8-row group;
  // position p of row r holds chunk p ^ f(r), f(r) = (r & 7) ^ ((r >> 3) & 1)
  const int lrow = lane >> 3, lpos = lane & 7;
  const uint8_t *Ablk = p.A + (int64_t)m0 * p.lda;
  const uint8_t *Bblk = p.B + (int64_t)n0 * p.ldb;
  const int64_t a_left = (int64_t)(p.M - m0 - 1) * p.lda + p.K;
  const int64_t b_left = (int64_t)(p.N - n0 - 1) * p.ldb + p.K;
  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(Ablk, a_left < 0x7fffffff ? (uint32_t)a_left : 0x7fffffffu);
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(Bblk, b_left < 0x7fffffff ? (uint32_t)b_left : 0x7fffffffu);

  // Wave load j of a panel covers the 8 rows of group g = wave * N + j.  The
  // per-lane part of the address depends on the parity of g only (N is even, so
  // on the parity of j); the rest is scalar.  Rows beyond M / N need no test:
  // their offsets lie beyond the resource's range.
  static_assert(NA % 2 == 0 && NB % 2 == 0, "wave loads per panel must be even");
  const uint32_t a_voff[2] = {(uint32_t)(lrow * (int)p.lda + (lpos ^ lrow) * 16), (uint32_t)(lrow * (int)p.lda + (lpos ^ lrow ^ 1) * 16)};
  const uint32_t b_voff[2] = {(uint32_t)(lrow * (int)p.ldb + (lpos ^ lrow) * 16), (uint32_t)(lrow * (int)p.ldb + (lpos ^ lrow ^ 1) * 16)};
  const int a_lda8 = 8 * (int)p.lda, b_ldb8 = 8 * (int)p.ldb;
  const int a_srow = wave * NA * a_lda8, b_srow = wave * NB * b_ldb8;
  // L2 touches.  The 32 workgroups resident on an XCD form a GROUP_M x (32 / GROUP_M)
  // block of tiles: 32 / GROUP_M of them stream the same A panel and GROUP_M the
  // same B panel.  Each workgroup touches (one dword per 128-byte line) only its
  // share of the rows of the K tile PF trips ahead, so that the line is in the
  // XCD's L2 when the panel loads of all the sharers ask for it.
  uint32_t pfa_voff[PFA > 0 ? PFA : 1], pfb_voff[PFB > 0 ? PFB : 1];
  if constexpr (PF > 0) {
    constexpr int SA = 32 / GROUP_M >= 1 ? 32 / GROUP_M : 1, SB = GROUP_M;
    const int slice_a = tile_n % SA, slice_b = row_in_group % SB;
#pragma unroll
    for (int i = 0; i < PFA; ++i) {
      const int row = (i * NW + wave) * 64 + lane;
      pfa_voff[i] = (row < BM && row % SA == slice_a && m0 + row < p.M) ? (uint32_t)(row * (int)p.lda) : kOOB;
    }
#pragma unroll
    for (int i = 0; i < PFB; ++i) {
      const int row = (i * NW + wave) * 64 + lane;
      pfb_voff[i] = (row < BN && row % SB == slice_b && n0 + row < p.N) ? (uint32_t)(row * (int)p.ldb) : kOOB;
    }
  }
  const int chunk_even = (lpos ^ lrow) * 16, chunk_odd = (lpos ^ lrow ^ 1) * 16;  // byte offset in the row, by parity of g

  const int KT = (p.K + BK - 1) / BK;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  auto wrap = [](int slot) { return slot >= R ? slot - R : slot; };  // slot in [0, 2R)
  // Units are issued in the order A(0), B(0), A(1), B(1), ...; unit u lives in
  // ring slot u % R (the callers keep the slot numbers as running scalars).
  // Every unit issues its full count of loads so that the vmcnt arithmetic is
  // uniform; K tiles at or beyond the end, rows beyond M / N and chunks beyond
  // K use an out-of-range offset, which the buffer unit turns into zeros in LDS.
  // load_one: i-th vector-memory instruction (of IA or IB) of the unit of K
  // tile kt (A or B panel) into ring slot `slot`: first the L2 touches, then
  // the 1 KiB panel loads.
  auto load_one = [&](bool is_b, int kt, int slot, int i) {
    const int k0 = kt * BK;
    const uint32_t m_even = (k0 + chunk_even < p.K) ? 0u : kOOB, m_odd = (k0 + chunk_odd < p.K) ? 0u : kOOB;
    if (!is_b) {
      const uint32_t dst = lds0 + slot * UNIT + wave * (NA * 1024);
      // a touched dword lands in this wave's own part of the slot and is
      // overwritten by the panel loads that follow (a wave's loads return in order)
      if (i < PFA)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, reinterpret_cast<lds_ptr_t>(dst), 4,
                                                 pfa_voff[i < PFA ? i : 0] | ((k0 + PF * BK < p.K) ? 0u : kOOB), k0 + PF * BK, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, reinterpret_cast<lds_ptr_t>(dst + (i - PFA) * 1024), 16,
                                                 a_voff[(i - PFA) & 1] | (((i - PFA) & 1) ? m_odd : m_even),
                                                 k0 + a_srow + (i - PFA) * a_lda8, 0, 0);
    } else {
      const uint32_t dst = lds0 + slot * UNIT + wave * (NB * 1024);
      if (i < PFB)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, reinterpret_cast<lds_ptr_t>(dst), 4,
                                                 pfb_voff[i < PFB ? i : 0] | ((k0 + PF * BK < p.K) ? 0u : kOOB), k0 + PF * BK, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB, reinterpret_cast<lds_ptr_t>(dst + (i - PFB) * 1024), 16,
                                                 b_voff[(i - PFB) & 1] | (((i - PFB) & 1) ? m_odd : m_even),
                                                 k0 + b_srow + (i - PFB) * b_ldb8, 0, 0);
    }
  };

  // ---- LDS -> register fragment plan ----
  const int l31 = lane & 31, h = lane >> 5;
  const int fr = (l31 & 7) ^ ((l31 >> 3) & 1);
  uint32_t foff[2][2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < 2; ++j) foff[s][j] = l31 * BK + (((s * 4 + h * 2 + j) ^ fr) * 16);
  const int a_base = wm * (TM * 32 * BK);
  const int b_base = wn * (TN * 32 * BK);

  // LDS addresses of the two 16-byte pieces a lane reads of its row, for step s
  // of the K tile whose panels sit in slots slot_a / slot_b.  The additions are
  // opaque to the compiler on purpose: it would otherwise keep a register per
  // (slot, piece) combination alive across the loop.
  typedef const __attribute__((address_space(3))) v4i *lds_v4i_ptr;
  auto frag_addrs = [&](int slot_a, int slot_b, int s, uint32_t (&ad)[4]) {
    const uint32_t sa = lds0 + slot_a * UNIT + a_base, sb = lds0 + slot_b * UNIT + b_base;
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[0]) : "s"(sa), "v"(foff[s][0]));
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[1]) : "s"(sa), "v"(foff[s][1]));
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[2]) : "s"(sb), "v"(foff[s][0]));
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[3]) : "s"(sb), "v"(foff[s][1]));
  };
  // fragment f, in the order the MFMAs need them: B0, A0 .. A(TM-1), B1 ..
  auto read_one = [&](const uint32_t (&ad)[4], v8i (&af)[TM], v8i (&bf)[TN], int f) {
    const bool is_b = f == 0 || f > TM;
    const int t = f == 0 ? 0 : (f > TM ? f - TM : f - 1);
    const v4i lo = *reinterpret_cast<lds_v4i_ptr>(ad[is_b ? 2 : 0] + t * (32 * BK));
    const v4i hi = *reinterpret_cast<lds_v4i_ptr>(ad[is_b ? 3 : 1] + t * (32 * BK));
    const v8i v = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (is_b) bf[t] = v;
    else af[t] = v;
  };

  v16f acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[tn][tm][v] = 0.0f;

  // MFMA number idx (of TM*TN) of one 64-byte step
  auto mma_one = [&](v8i (&af)[TM], v8i (&bf)[TN], int idx) {
    const int tn = idx / TM, tm = idx % TM;
    // D[i = n][j = m]: B rows feed the "A" port, A rows the "B" port
    acc[tn][tm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[tn], af[tm], acc[tn][tm], 0, 0, 0, 0, 0, 0);
  };

  // The loads of one trip are two units.  The first is spread over the MFMAs of
  // the first half, the second over those of the second half: a burst of all
  // of them after the barrier would keep the waves queueing at the
  // vector-memory port instead of issuing MFMAs.
  //   prologue: units 0 .. R-2 in flight, K tile 0 published, its first half read
#pragma unroll
  for (int u = 0; u < R - 1; ++u) {
#pragma unroll
    for (int i = 0; i < ((u & 1) ? IB : IA); ++i) load_one(u & 1, u >> 1, u, i);
  }
  v8i af0[TM], bf0[TN], af1[TM], bf1[TN];
  uint32_t ad[4];
  L8_WAIT_VM_LGKM0(PEND0);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  frag_addrs(0, 1, 0, ad);
#pragma unroll
  for (int f = 0; f < TM + TN; ++f) read_one(ad, af0, bf0, f);

  // One trip = one K tile of 128 = two matrix-core steps of 64.
  //   first half : MFMAs on (kt, step 0) while (kt, step 1) is read from LDS and
  //                unit 2kt+R-1 is requested (its slot, of K tile kt-1, was
  //                released at the previous barrier);
  //   barrier    : every wave has now read all of K tile kt (lgkmcnt 0), and
  //                K tile kt+1 has landed for every wave (partial vmcnt wait);
  //   second half: MFMAs on (kt, step 1) while (kt+1, step 0) is read and unit
  //                2kt+R is requested into the slot K tile kt just released.
  // Each group below is one MFMA plus its share of the LDS reads and of the
  // loads; the scheduling fences keep the groups in this order.
  constexpr int N_MMA = TM * TN, NF = TM + TN;
  constexpr int STRADDLE = L8_STRADDLE < N_MMA - 2 ? L8_STRADDLE : 0;
  constexpr int S1 = N_MMA - STRADDLE;  // MFMA groups before the barrier
  constexpr int S2 = N_MMA + STRADDLE;  // and after it
  constexpr int SR = N_MMA > 2 ? N_MMA - 2 : N_MMA;  // the last two groups of a trip are left without reads
  constexpr bool U1_IS_B = ((R - 1) & 1) != 0, U2_IS_B = (R & 1) != 0;  // panel kind of units 2kt+R-1 and 2kt+R
  constexpr int I1 = U1_IS_B ? IB : IA, I2 = U2_IS_B ? IB : IA;
  int s0 = 0;  // ring slot of unit 2kt
  for (int kt = 0; kt < KT; ++kt) {
    const int slot_u1 = wrap(s0 + R - 1);  // unit 2kt+R-1 reuses the slot of unit 2kt-1
    frag_addrs(s0, wrap(s0 + 1), 1, ad);
#pragma unroll
    for (int i = 0; i < S1; ++i) {
      if (L8_GEMM_DIAG != 2 && L8_GEMM_DIAG != 4) {
        mma_one(af0, bf0, i);
#pragma unroll
        for (int f = (NF * i) / S1; f < (NF * (i + 1)) / S1; ++f) read_one(ad, af1, bf1, f);
      }
      if (L8_GEMM_DIAG != 1) {
#pragma unroll
        for (int j = (I1 * i) / S1; j < (I1 * (i + 1)) / S1; ++j) load_one(U1_IS_B, kt + (R - 1) / 2, slot_u1, j);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    L8_WAIT_VM_LGKM0(PEND);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // the last MFMAs of the first half are issued after the barrier: they need
    // registers only and keep the matrix cores busy while the waves regroup
    frag_addrs(wrap(s0 + 2), wrap(s0 + 3), 0, ad);
#pragma unroll
    for (int i = 0; i < S2; ++i) {
      if (L8_GEMM_DIAG != 2 && L8_GEMM_DIAG != 4) {
        if (i < STRADDLE) mma_one(af0, bf0, S1 + i);
        else mma_one(af1, bf1, i - STRADDLE);
        if (i >= STRADDLE) {  // (kt+1, step 0) replaces the fragments the straddling MFMAs have just consumed
#pragma unroll
          for (int f = (NF * (i - STRADDLE)) / SR; f < (NF * (i - STRADDLE + 1)) / SR && f < NF; ++f) read_one(ad, af0, bf0, f);
        }
      }
      if (L8_GEMM_DIAG != 1) {
#pragma unroll
        for (int j = (I2 * i) / S2; j < (I2 * (i + 1)) / S2; ++j) load_one(U2_IS_B, kt + R / 2, s0, j);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    s0 = wrap(s0 + 2);
  }
  // ---- epilogue ----
  // All scales of this wave's part of the tile are requested in one batch,
  // before the wait that drains the ring: one memory latency in total,
  // overlapped with that wait, instead of one per 32-column tile.
  const float sa_s = p.sa[0], sb_s = p.sb[0];
  float sav[TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int m = m0 + (wm * TM + tm) * 32 + l31;
    sav[tm] = p.sa_row ? (m < p.M ? p.sa[m] : 0.0f) : sa_s;
  }
  // scales of the 16 n per 32-column tile that this lane holds before the half-wave swap
  float sbv[TN][4][4];
  const bool sb_vec = p.sb_row && (((uintptr_t)p.sb & 15) == 0);
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int nq = n0 + (wn * TN + tn) * 32 + 8 * qd + 4 * h;  // four consecutive n
      if (sb_vec && nq + 4 <= p.N) {
        const v4f t = *(const v4f *)(p.sb + nq);
#pragma unroll
        for (int e = 0; e < 4; ++e) sbv[tn][qd][e] = t[e];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) sbv[tn][qd][e] = p.sb_row ? (nq + e < p.N ? p.sb[nq + e] : 0.0f) : sb_s;
      }
    }
  // every wave's tail loads (out of range, zero-filling) and LDS reads are done
  // before the ring is reused as the staging area of the C tile
  L8_WAIT_VM_LGKM0(0);
  __builtin_amdgcn_s_barrier();

  // lane (l31, h) of tile (tn, tm) holds m = l31 and, in accumulator quad qd,
  // n = 8*qd + 4*h + {0..3}.  After the half-wave swap, lanes with h == 0 hold
  // n = 0..15 and lanes with h == 1 hold n = 16..31 of row m: 32 bytes of bf16.
  // Stored from there, every store instruction would scatter 16-byte pieces
  // over 32 rows.  The tile goes through LDS instead (rows padded by 16 bytes
  // so that the 16 lanes of a write phase hit 16 different bank groups) and
  // leaves as whole rows: one store instruction covers 1 KiB of consecutive
  // bytes of C per row pair.
  constexpr int C_ROW = BN * 2 + 16;  // staged row pitch in bytes
  static_assert(BM * C_ROW <= R * UNIT, "the C tile must fit in the ring");
  typedef __attribute__((address_space(3))) v4i *lds_v4i_wptr;
  auto convert_and_stage = [&](auto has_bias) {
    constexpr bool HAS_BIAS = decltype(has_bias)::value;
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    // the bias (rare: the linears of the model have none) is fetched per 32-column tile
    float biasv[4][4];
    if constexpr (HAS_BIAS) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int n = n0 + (wn * TN + tn) * 32 + 8 * qd + 4 * h + e;
          biasv[qd][e] = n < p.N ? bf16_bits_to_f32(p.bias[n]) : 0.0f;
        }
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const float sa = sav[tm];
      uint32_t pk[8];  // quad qd -> pk[2qd], pk[2qd+1]
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = acc[tn][tm][qd * 4 + e] * sa * sbv[tn][qd][e];
          if constexpr (HAS_BIAS) v[e] += biasv[qd][e];
        }
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
      const uint32_t at = lds0 + ((wm * TM + tm) * 32 + l31) * C_ROW + ((wn * TN + tn) * 32 + 16 * h) * 2;
      *reinterpret_cast<lds_v4i_wptr>(at) = v4i{(int)pk[0], (int)pk[1], (int)pk[4], (int)pk[5]};
      *reinterpret_cast<lds_v4i_wptr>(at + 16) = v4i{(int)pk[2], (int)pk[3], (int)pk[6], (int)pk[7]};
    }
  }
  };
  if (p.bias) convert_and_stage(std::true_type{});
  else convert_and_stage(std::false_type{});
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's part of the tile is in LDS
  __builtin_amdgcn_s_barrier();
  // 16-byte chunk c of the tile: row c / CPR, columns 8 * (c % CPR) .. +7
  constexpr int CPR = BN / 8, CHUNKS = BM * CPR;
  static_assert(CHUNKS % (NW * 64) == 0, "whole wave stores");
  const bool c_vec = (p.ldc % 8 == 0) && (((uintptr_t)p.C & 15) == 0);
  constexpr int ITERS = CHUNKS / (NW * 64), ROWS_PER_IT = NW * 64 / CPR;
  static_assert((NW * 64) % CPR == 0, "a wave store covers whole rows");
  const int row0 = (wave * 64 + lane) / CPR, col = ((wave * 64 + lane) % CPR) * 8;
  if (c_vec && m0 + BM <= p.M && n0 + BN <= p.N && L8_GEMM_DIAG != 3) {
    // interior tile: no masks, one pointer and one LDS address stepped by constants; streaming stores, so
    // that the C tile on its way out does not push the operand panels out of the L2
    uint16_t *dst = p.C + (int64_t)(m0 + row0) * p.ldc + n0 + col;
    const uint32_t at = lds0 + row0 * C_ROW + col * 2;
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
      __builtin_nontemporal_store(*reinterpret_cast<lds_v4i_ptr>(at + it * (ROWS_PER_IT * C_ROW)),
                                  (v4i *)(dst + (int64_t)it * ROWS_PER_IT * p.ldc));
  } else if (L8_GEMM_DIAG != 3) {
#pragma unroll 4
    for (int it = 0; it < ITERS; ++it) {
      const int row = row0 + it * ROWS_PER_IT;
      const v4i v = *reinterpret_cast<lds_v4i_ptr>(lds0 + row * C_ROW + col * 2);
      const int m = m0 + row, n = n0 + col;
      if (m < p.M && n < p.N) {
        uint16_t *dst = p.C + (int64_t)m * p.ldc + n;
        if (c_vec && n + 8 <= p.N) {
          __builtin_nontemporal_store(v, (v4i *)dst);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < p.N) dst[e] = (uint16_t)((uint32_t)v[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
  }
#else
  (void)p;
#endif
}

// ---------------------------------------------------------------------------
// Persistent variant for large problems: one workgroup per compute unit walks a
// list of 256x256 tiles, and the panel stream (global -> LDS ring) runs on
// from the last K tile of one output tile into the first K tiles of the next,
// so that only the very first tile of a workgroup pays a prologue.
//
// The C tile leaves straight from the accumulators, with no staging in LDS
// (the ring stays in use by the panel stream) and no barrier:
//   * the matrix cores compute D[i = m][j = n'] (A rows on the first port);
//   * LDS row tn*32 + j of a wave's 128-row span of the B panel holds the
//     global B row 4*g(j) + tn of that span, g(j) = 2*(j & 15) + (j >> 4) (the
//     permutation is applied on the global-address side of the direct-to-LDS
//     loads, which is free), so that lane j owns, at the same accumulator
//     index of its four tn tiles, the four CONSECUTIVE output columns
//     4*g(j) .. 4*g(j)+3, and lanes j / j+16 own neighbouring groups;
//   * two v_permlane16_swap per pair of rows hand the lanes 0..15 of every 32
//     the first row (their own four columns and their partners' four) and the
//     lanes 16..31 the second: one 16-byte store per lane then covers 256
//     contiguous bytes of a C row per 16 lanes (four rows per wave instruction,
//     whole 128-byte lines).
// Work split: the tiles are dealt to the 8 XCDs in contiguous ranges of the
// grouped order (as in the kernel above); inside an XCD, workgroup `loc`
// takes tiles loc, loc + W, loc + 2W, ... of the range (W workgroups per XCD),
// so the workgroups resident on an XCD always work on W consecutive tiles of
// the grouped order and share their panels in that XCD's L2.
// ---------------------------------------------------------------------------
template <int GROUP_M, bool HAS_BIAS, bool SK = false, int NW = 4>
__global__ __launch_bounds__(NW * 64) void gemm_nt_stream_kernel(const GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  // NW = 4: one wave per SIMD, 128x128 per wave (the least LDS traffic per flop); NW = 8: two waves per SIMD,
  // 64x128 per wave (while one of them waits -- for the port of the vector memory unit, for LDS, at the barrier --
  // the other one's MFMAs keep the matrix core busy; half the stores per wave in the epilogue; 1.5 x the LDS reads)
  static_assert(NW == 4 || NW == 8, "four or eight waves");
  static_assert(!SK || NW == 4, "the shared-K exchange is written for four waves");
  constexpr int BM = 256, BN = 256, BK = 128, TM = 16 / NW, TN = 4, R = 5;
  constexpr int WROWS = TM * 32;  // rows of the tile per wave
  constexpr int UNIT = BM * BK;    // one ring slot: the A or the B panel of one K tile
  constexpr int NL = BM / 8 / NW;  // 1 KiB wave loads (8 rows x 128 B) per panel per wave
  constexpr int PEND = NL;         // in flight at the barrier of a trip: the unit requested in its first half
  constexpr int PEND0 = 2 * NL;    // prologue: K tile 1 may be in flight when K tile 0 is published
  constexpr int N_STORES = TM * 4 * 2;  // store instructions per wave and C tile
  static_assert(N_STORES + PEND <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // ---- this workgroup's tiles ----
  const int nb = p.tiles_m * p.tiles_n;
  const int xcd = blockIdx.x & 7, loc = blockIdx.x >> 3, W = gridDim.x >> 3;
  const int q = nb >> 3, rem = nb & 7;
  const int first = (xcd < rem) ? xcd * (q + 1) : rem * (q + 1) + (xcd - rem) * q;
  const int cnt = q + (xcd < rem ? 1 : 0);
  const int KT = (p.K + BK - 1) / BK;
  // SK instantiation -- tail of the XCD's range: the r = cnt % W tiles left after the full rounds would keep r
  // workgroups busy for a whole K loop and H = W - r idle.  When the idle ones can take enough off the others to
  // pay for an exchange of partial sums, each tail tile's K range is cut in two at the same place: the last r
  // workgroups take the first k_split K tiles of one tail tile each, in step with each other like a normal round
  // (workgroups that are at the same K tile at the same time share their panels in the XCD's L2; a split that
  // staggers them costs more in panel traffic than it saves), and own the tile; the first H workgroups (helpers)
  // multiply the remaining K tiles of tail tiles loc, loc + H, ... one after the other, again in step with each
  // other, and leave fp32 partial sums, which the owners add to their own before they store the tile.  Owners
  // wait only for workgroups with lower numbers (dispatched earlier), which never wait for anybody.
  // With m = ceil(r / H) pieces per helper, L K tiles per piece, a partial tile costing a helper about
  // kSkWriteCost K tiles' time to write and an owner kSkFixCost to add, both finish together when
  // m * (L + kSkWriteCost) = KT - L + kSkFixCost.
  const int n_rounds = cnt / W, r_tail = cnt - n_rounds * W, n_help = W - r_tail;
  const int m_help = (r_tail + n_help - 1) / n_help;
  const int l_help = (KT + kSkFixCost - m_help * kSkWriteCost) / (m_help + 1);
  const bool sk = SK && p.sk_partials != nullptr && n_rounds > 0 && r_tail > 0 && l_help >= kSkMinSaved;
  const int k_split = KT - l_help;
  const bool helper = loc < n_help;
  const int n_tail = !sk ? 0 : (helper ? (loc < r_tail ? (r_tail - loc + n_help - 1) / n_help : 0) : 1);  // pieces of this workgroup
  const int n_seg = sk ? n_rounds : (loc < cnt ? (cnt - loc + W - 1) / W : 0);                              // whole tiles
  if (n_seg + n_tail == 0) return;
  [[maybe_unused]] uint64_t prof[24] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  if (L8_GEMM_PROF) {
    prof[0] = __builtin_amdgcn_s_memrealtime();
    prof[5] = __builtin_readcyclecounter();
  }
  auto tile_at = [&](int lin, int &m0, int &n0) {
    const int per_group = GROUP_M * p.tiles_n;
    const int grp = lin / per_group;
    const int first_m = grp * GROUP_M;
    const int gsz = (p.tiles_m - first_m < GROUP_M) ? p.tiles_m - first_m : GROUP_M;
    const int in_grp = lin - grp * per_group;
    m0 = (first_m + in_grp % gsz) * BM;
    n0 = (in_grp / gsz) * BN;
  };
  // The whole tiles of a workgroup are first + loc, + W, + 2 W, ...: two cursors walk that sequence, one for the loader
  // (two K tiles ahead) and one for the multiply / store side, each holding (group, index in the group) so that a
  // tile's origin costs a shift and a mask.  (tile_at's divisions, a hundred dependent instructions each between the
  // scalar and the vector unit, took a thousand cycles per tile with idle matrix cores, on either side.)
  static_assert((GROUP_M & (GROUP_M - 1)) == 0, "GROUP_M is a power of two");
  struct TileCursor { int grp, in_grp; };
  const int per_group_c = GROUP_M * p.tiles_n;
  TileCursor cur_mul, cur_ld;
  {
    const int lin0 = first + loc;
    cur_mul.grp = lin0 / per_group_c;
    cur_mul.in_grp = lin0 - cur_mul.grp * per_group_c;
    cur_ld = cur_mul;
  }
  auto cursor_origin = [&](const TileCursor &c, int &m0, int &n0) {
    const int first_m = c.grp * GROUP_M;
    const int left = p.tiles_m - first_m;
    if (left >= GROUP_M) {
      m0 = (first_m + (c.in_grp & (GROUP_M - 1))) * BM;
      n0 = (c.in_grp / GROUP_M) * BN;
    } else {  // the last, shorter group of tile rows
      m0 = (first_m + c.in_grp % left) * BM;
      n0 = (c.in_grp / left) * BN;
    }
  };
  auto cursor_step = [&](TileCursor &c) {
    c.in_grp += W;
    while (c.in_grp >= per_group_c) {
      c.in_grp -= per_group_c;
      ++c.grp;
    }
  };
  // piece pc of the tail (highest tile first): tile origin, K-tile range [kb, ke); returns the tail tile's number
  // piece pc of this workgroup's tail: the tail tile's number (tile origin in m0, n0); every piece of a workgroup
  // covers the same K tiles [piece_kb, piece_ke)
  const int piece_kb = helper ? k_split : 0, piece_ke = helper ? KT : k_split;
  auto piece_of = [&](int pc, int &m0, int &n0) -> int {
    const int tt = helper ? loc + pc * n_help : loc - n_help;
    tile_at(first + n_rounds * W + tt, m0, n0);
    return tt;
  };

  // ---- global -> LDS load plan ----
  // lane l of a wave load fills LDS row l/8, position l%8 of an 8-row group; position p of LDS row r holds
  // chunk p ^ f(r), f(r) = (r & 7) ^ ((r >> 3) & 1).  Wave load i of a panel fills the LDS rows of group
  // g = wave * NL + i.  For the A panel LDS row = tile row.  For the B panel LDS row r = span*128 + tn*32 + j
  // holds tile row span*128 + 4*cg(j) + tn with cg(j) = 2*(j & 15) + (j >> 4): within a group (8 consecutive j)
  // the rows are 8 apart, and the group's first row is span*128 + 64*(g & 1) + 4*((g >> 1) & 1) + (g%16)/4.
  // The per-lane constants of the K loop (ten registers) are formed from an opaque copy of the lane number.  In the
  // instantiation that shares K ranges out they are formed afresh in front of every tile's K loop: there, values that
  // lived across the conversion of the C tile (the point of highest register pressure) were the ones the allocator
  // chose to spill, and it reloaded them inside the K loop.  The others have the registers to keep them (two hundred
  // cycles per tile with idle matrix cores otherwise).
  uint32_t a_voff[2], b_voff[2], foff[2][2];
  int chunk_even, chunk_odd;
  auto lane_consts = [&]() {
    int l = lane;
    asm volatile("" : "+v"(l));
    const int lrow = l >> 3, lpos = l & 7;
    chunk_even = (lpos ^ lrow) * 16;
    chunk_odd = (lpos ^ lrow ^ 1) * 16;
    a_voff[0] = (uint32_t)(lrow * (int)p.lda + chunk_even);
    a_voff[1] = (uint32_t)(lrow * (int)p.lda + chunk_odd);
    b_voff[0] = (uint32_t)(lrow * 8 * (int)p.ldb + chunk_even);
    b_voff[1] = (uint32_t)(lrow * 8 * (int)p.ldb + chunk_odd);
    const int l31 = l & 31, h = l >> 5;
    const int fr = (l31 & 7) ^ ((l31 >> 3) & 1);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int j = 0; j < 2; ++j) foff[s][j] = l31 * BK + (((s * 4 + h * 2 + j) ^ fr) * 16);
  };
  lane_consts();
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  auto wrap = [](int slot) { return slot >= R ? slot - R : slot; };

  // loader cursor: the K tile whose panels are requested next (two K tiles ahead of the one being multiplied)
  int ld_seg = 0, ld_kt = 0;
  [[maybe_unused]] int ld_ke = KT;  // SK: the loader's piece ends here
  __amdgpu_buffer_rsrc_t ld_rsA, ld_rsB;
  auto ld_open = [&](int seg) {
    if (seg < n_seg + n_tail) {
      int m0, n0;
      if (!SK || seg < n_seg) {
        cursor_origin(cur_ld, m0, n0);  // ld_open is called for seg = 0, 1, 2, ... in turn
        cursor_step(cur_ld);
        if (SK) ld_ke = KT;
      } else {
        piece_of(seg - n_seg, m0, n0);
        ld_kt = piece_kb;
        ld_ke = piece_ke;
      }
      const int64_t a_left = (int64_t)(p.M - m0 - 1) * p.lda + p.K;
      const int64_t b_left = (int64_t)(p.N - n0 - 1) * p.ldb + p.K;
      ld_rsA = make_rsrc(p.A + (int64_t)m0 * p.lda, a_left < 0x7fffffff ? (uint32_t)a_left : 0x7fffffffu);
      ld_rsB = make_rsrc(p.B + (int64_t)n0 * p.ldb, b_left < 0x7fffffff ? (uint32_t)b_left : 0x7fffffffu);
    } else {  // past the last tile: every load is out of range and fills its LDS bytes with zeros
      ld_rsA = make_rsrc(p.A, 0);
      ld_rsB = make_rsrc(p.B, 0);
      if (SK) ld_ke = 0x7fffffff;
    }
  };
  auto ld_advance = [&]() {
    if (++ld_kt == (SK ? ld_ke : KT)) {
      ld_kt = 0;
      ld_open(++ld_seg);
    }
  };
  // i-th wave load (of NL) of the A or B panel of the loader's K tile into ring slot `slot`
  auto load_one = [&](bool is_b, int slot, int i) {
    const int k0 = ld_kt * BK;
    const uint32_t m_even = (k0 + chunk_even < p.K) ? 0u : kOOB, m_odd = (k0 + chunk_odd < p.K) ? 0u : kOOB;
    const uint32_t dst = lds0 + slot * UNIT + (wave * NL + i) * 1024;
    if (!is_b) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rsA, reinterpret_cast<lds_ptr_t>(dst), 16, a_voff[i & 1] | ((i & 1) ? m_odd : m_even),
                                               k0 + (wave * NL + i) * 8 * (int)p.lda, 0, 0);
    } else {
      const int g = wave * NL + i;  // 8-row group of the panel's LDS image
      const int row = (g >> 4) * 128 + 64 * (g & 1) + 4 * ((g >> 1) & 1) + ((g & 15) >> 2);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ld_rsB, reinterpret_cast<lds_ptr_t>(dst), 16, b_voff[i & 1] | ((i & 1) ? m_odd : m_even),
                                               k0 + row * (int)p.ldb, 0, 0);
    }
  };

  // ---- LDS -> register fragment plan (as in the kernel above) ----
  const int a_base = wm * (TM * 32 * BK);
  const int b_base = wn * (TN * 32 * BK);
  typedef const __attribute__((address_space(3))) v4i *lds_v4i_ptr;
  auto frag_addrs = [&](int slot_a, int slot_b, int s, uint32_t (&ad)[4]) {
    const uint32_t sa = lds0 + slot_a * UNIT + a_base, sb = lds0 + slot_b * UNIT + b_base;
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[0]) : "s"(sa), "v"(foff[s][0]));
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[1]) : "s"(sa), "v"(foff[s][1]));
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[2]) : "s"(sb), "v"(foff[s][0]));
    asm volatile("v_add_u32 %0, %1, %2" : "=v"(ad[3]) : "s"(sb), "v"(foff[s][1]));
  };
  // fragment f, in the order the MFMAs need them: A0, B0 .. B(TN-1), A1 ..
  auto read_one = [&](const uint32_t (&ad)[4], v8i (&af)[TM], v8i (&bf)[TN], int f) {
    const bool is_a = f == 0 || f > TN;
    const int t = f == 0 ? 0 : (f > TN ? f - TN : f - 1);
    const v4i lo = *reinterpret_cast<lds_v4i_ptr>(ad[is_a ? 0 : 2] + t * (32 * BK));
    const v4i hi = *reinterpret_cast<lds_v4i_ptr>(ad[is_a ? 1 : 3] + t * (32 * BK));
    const v8i v = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (is_a) af[t] = v;
    else bf[t] = v;
  };

  v16f acc[TM][TN];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[tm][tn][v] = 0.0f;
  // MFMA number idx of one 64-byte step, tm-major
  auto mma_one = [&](v8i (&af)[TM], v8i (&bf)[TN], int idx) {
    const int tm = idx / TN, tn = idx % TN;
    acc[tm][tn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[tm], bf[tn], acc[tm][tn], 0, 0, 0, 0, 0, 0);
  };

  // One accumulator element, fetched where it is used.  Written as assembly with an accumulator-register operand:
  // given plain reads, the register allocator moves the whole accumulator set into ordinary vector registers in
  // front of the conversion of the C tile and pays for it with spills inside the K loop.
  auto acc_read = [&](int tm, int tn, int i) -> float {
    if constexpr (NW == 8) {
      return acc[tm][tn][i];  // 128 accumulators: the allocator may keep them in ordinary registers
    } else {
      float x;
      asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[tm][tn][i]));
      return x;
    }
  };
  // ---- C tile straight from the accumulators ----
  // acc[tm][tn][4*qd + e] of lane (l31, h) is C[m][n] with m = wm*WROWS + tm*32 + 8*qd + 4*h + e and
  // n = wn*128 + 4*cg(l31) + tn (tile coordinates).  The host launches this kernel only when every lane pair's
  // eight columns are in or out as a whole and its 16-byte store is aligned: N % 8 == 0, ldc % 8 == 0, C
  // 16-byte aligned, row scales 16-byte and bias 8-byte aligned.
  // The scales (and the bias) of a tile are requested before its K loop, a handful of registers per lane: lane l
  // holds the A scales of tile rows wm*WROWS + l and (four waves) + 64 + l (handed to the lanes that need them by lane
  // permutes at the end) and the B scales / bias of its own four columns.  Requested among the stores of the
  // tile they would make their consumer wait for every store ahead of them (the counter retires in order).
  int seg_sa[2] = {0, 0};
  v4i seg_sb = {0, 0, 0, 0};
  [[maybe_unused]] v2i seg_bias = {0, 0};
  // The descriptors cover the whole scale (bias) vectors and live as long as the kernel: a tile's requests then cost a
  // few address instructions (with a descriptor per tile, sixty scalar instructions at one per five cycles stood
  // between two tiles).  Rows past M and columns past N fall outside the range and read as zero; M, N < 2^29 here
  // (the host checks) so the byte offsets fit.
  const __amdgpu_buffer_rsrc_t rsSa = make_rsrc(p.sa, p.sa_row ? (uint32_t)p.M * 4u : 4u);
  const __amdgpu_buffer_rsrc_t rsSb = make_rsrc(p.sb, p.sb_row ? (uint32_t)p.N * 4u : 4u);
  [[maybe_unused]] const __amdgpu_buffer_rsrc_t rsBias = make_rsrc(HAS_BIAS ? (const void *)p.bias : (const void *)p.sb, (uint32_t)p.N * 2u);
  // a scale that is one number for the whole operand is read once (read per tile, between the stores of one tile
  // and the K loop of the next, it was a vector load whose result was copied at once: a wait for every store)
  const int sa_one = p.sa_row ? 0 : __builtin_amdgcn_readfirstlane(__float_as_int(p.sa[0]));
  const int sb_one = p.sb_row ? 0 : __builtin_amdgcn_readfirstlane(__float_as_int(p.sb[0]));
  auto load_scales = [&](int m0, int n0) {
    // lane-derived values are formed afresh from an opaque copy of the lane number wherever a tile's prologue or
    // epilogue needs them, so that none of them lives across a K loop
    int l = lane;
    asm volatile("" : "+v"(l));
    const int l31 = l & 31;
    const int cg = 2 * (l31 & 15) + (l31 >> 4);  // this lane's group of four output columns (of its wave's 32)
    if (p.sa_row) {
      seg_sa[0] = __builtin_amdgcn_raw_buffer_load_b32(rsSa, (wm * WROWS + l) * 4, m0 * 4, 0);
      if constexpr (TM == 4) seg_sa[1] = __builtin_amdgcn_raw_buffer_load_b32(rsSa, (wm * WROWS + 64 + l) * 4, m0 * 4, 0);
    } else {
      seg_sa[0] = seg_sa[1] = sa_one;
    }
    if (p.sb_row) {
      seg_sb = __builtin_amdgcn_raw_buffer_load_b128(rsSb, (wn * 128 + 4 * cg) * 4, n0 * 4, 0);
    } else {
      seg_sb = v4i{sb_one, sb_one, sb_one, sb_one};
    }
    if constexpr (HAS_BIAS) seg_bias = __builtin_amdgcn_raw_buffer_load_b64(rsBias, (wn * 128 + 4 * cg) * 2, n0 * 2, 0);
  };
  // (A compute unit drains its stores at about 16 bytes per clock: the 128 KiB of a C tile keep it busy for some
  // 8000 cycles, of which the conversion below hides about half.)
  // PARTS (a tile whose last K tiles were multiplied by another workgroup): rs_p is the partial sum over those K
  // tiles, added to the workgroup's own.
  // Byte offset of piece i (of 64) of this wave in a slot.  The slots are 256 KiB apart and the workgroups of a
  // launch write theirs in step: the pieces are rotated by the slot number so that stores issued at the same time
  // do not all fall on the same memory channels.
  [[maybe_unused]] auto piece_off = [&](int slot, int i) { return (wave * (TM * TN * 4) + ((i + slot * 5) & (TM * TN * 4 - 1))) * 1024; };
  [[maybe_unused]] __amdgpu_buffer_rsrc_t rs_p;
  [[maybe_unused]] int p_slot = 0;
  constexpr int P_AHEAD = 3;  // groups / pieces of the partial sum requested ahead of their use (their latency is long)
  auto store_tile_as = [&](int m0, int n0, auto parts_tag, auto sbrow_tag) {
    constexpr bool PARTS = decltype(parts_tag)::value;
    // SB_ROW false: one scale for all columns; it is folded into the row scales (two multiplications per lane and
    // tile instead of one per element)
    constexpr bool SB_ROW = decltype(sbrow_tag)::value;
    // Opaque copies: everything below would otherwise be hoisted out of the K loop as loop-invariant (row
    // offsets in scalar registers, per-lane addresses in vector registers) and held across it.
    int ldc2 = (int)p.ldc * 2;
    asm volatile("" : "+s"(ldc2));
    int l = lane;
    asm volatile("" : "+v"(l));
    const int l31 = l & 31, h = l >> 5;
    int lane_col = wn * 128 + 8 * (l31 & 15);  // first of the eight columns this lane stores
    asm volatile("" : "+v"(lane_col));
    const int64_t c_left = ((int64_t)(p.M - m0 - 1) * p.ldc + (p.N - n0)) * 2;
    const __amdgpu_buffer_rsrc_t rsC = make_rsrc(p.C + (int64_t)m0 * p.ldc + n0, c_left < 0x7fffffff ? (uint32_t)c_left : 0x7fffffffu);
    float sbv[4];
    [[maybe_unused]] float bv[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) sbv[e] = __int_as_float(seg_sb[e]);
    if constexpr (HAS_BIAS) {
      bv[0] = bf16_bits_to_f32((uint32_t)seg_bias[0] & 0xffffu);
      bv[1] = bf16_bits_to_f32((uint32_t)seg_bias[0] >> 16);
      bv[2] = bf16_bits_to_f32((uint32_t)seg_bias[1] & 0xffffu);
      bv[3] = bf16_bits_to_f32((uint32_t)seg_bias[1] >> 16);
    }
    // Row scale of tile row wm*WROWS + r: lane r % 64 of seg_sa[r / 64]; a lane needs r = tm*32 + 8*qd + 4*h + e.
    // The lane permutes of the next (tm, qd) group are in flight while the current group is converted.  They are
    // written as assembly for the immediate offset (as plain address arithmetic the 64 addresses were
    // precomputed into 64 registers and spilled) and are waited for by hand: LDS operations return in order, so
    // "at most 4 outstanding" means that everything but the group requested last has arrived.
    const int sa_addr = 16 * h;  // byte address of lane 4*h
    const int sa_regs[2] = {SB_ROW ? seg_sa[0] : __float_as_int(__int_as_float(seg_sa[0]) * sbv[0]),
                            SB_ROW ? seg_sa[1] : __float_as_int(__int_as_float(seg_sa[1]) * sbv[0])};
    float sa_grp[2][4];
    auto request_row_scales = [&](int g, float (&dst)[4]) {  // g = tm * 4 + qd
      const int tm = g >> 2, qd = g & 3;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        asm volatile("ds_bpermute_b32 %0, %1, %2 offset:%3"
                     : "=v"(dst[e])
                     : "v"(sa_addr), "v"(sa_regs[tm >> 1]), "n"(4 * ((tm & 1) * 32 + 8 * qd + e)));
    };
    request_row_scales(0, sa_grp[0]);
    // partial sums of the group (tm, qd): one 16-byte piece per lane and accumulator, laid out as write_partial
    // stores them; requested P_AHEAD groups ahead
    [[maybe_unused]] v4f pbuf[P_AHEAD + 1][TN];
    [[maybe_unused]] const int p_voff = lane * 16;
    [[maybe_unused]] auto request_parts = [&](int g, v4f (&dst)[TN]) {
      const int tm = g >> 2, qd = g & 3;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
        dst[tn] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
                                              rs_p, p_voff, piece_off(p_slot, (tm * TN + tn) * 4 + qd), kCoherent));
    };
    if constexpr (PARTS) {
#pragma unroll
      for (int g = 0; g < P_AHEAD; ++g) request_parts(g, pbuf[g]);
    }
    [[maybe_unused]] uint64_t tq0 = 0, tq1 = 0, tq2 = 0;
    if (L8_GEMM_PROF) {
      tq0 = __builtin_readcyclecounter();
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0), lgkmcnt(0): the panel loads in flight
      tq1 = __builtin_readcyclecounter();
      prof[8] += tq1 - tq0;
    }
    // A store instruction costs the same whatever it carries, so lanes j and j+16 pair up: of two consecutive
    // rows, lane j takes the first (its own four columns and its partner's four, 16 contiguous bytes) and lane
    // j+16 the second.  One instruction then writes four rows x 256 bytes.  Lanes whose columns lie beyond N
    // store nothing (N % 8 == 0 here: a lane pair is in or out as a whole).
    const int par = l31 >> 4;
    const uint32_t c_voff = (n0 + lane_col < p.N) ? (uint32_t)((4 * h + par) * ldc2 + lane_col * 2) : kOOB;
    if (L8_GEMM_PROF) {
      __builtin_amdgcn_s_waitcnt(0x0070);  // the scales
      tq2 = __builtin_readcyclecounter();
      prof[9] += tq2 - tq1;
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int row = wm * WROWS + tm * 32 + 8 * qd;  // + 4*h + e
        const int g = tm * 4 + qd;
        float(&sa_cur)[4] = sa_grp[g & 1];
        if constexpr (PARTS) {
          if (g + P_AHEAD < TM * 4) request_parts(g + P_AHEAD, pbuf[(g + P_AHEAD) % (P_AHEAD + 1)]);
        }
        if (g + 1 < TM * 4) {
          request_row_scales(g + 1, sa_grp[(g + 1) & 1]);
          asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(sa_cur[0]), "+v"(sa_cur[1]), "+v"(sa_cur[2]), "+v"(sa_cur[3]));
        } else {
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sa_cur[0]), "+v"(sa_cur[1]), "+v"(sa_cur[2]), "+v"(sa_cur[3]));
        }
#pragma unroll
        for (int e2 = 0; e2 < 4; e2 += 2) {
          int o[2][2];  // [row e2 / e2+1][low / high pair of columns]
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            const float sa = sa_cur[e2 + r];
            float v[4];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
              float a = acc_read(tm, tn, 4 * qd + e2 + r);
              if constexpr (PARTS) a = a + pbuf[g % (P_AHEAD + 1)][tn][e2 + r];  // ascending K
              v[tn] = SB_ROW ? a * sa * sbv[tn] : a * sa;
              if constexpr (HAS_BIAS) v[tn] += bv[tn];
            }
            typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
            const bf2 lo = {(__bf16)v[0], (__bf16)v[1]}, hi = {(__bf16)v[2], (__bf16)v[3]};
            o[r][0] = __builtin_bit_cast(int, lo);
            o[r][1] = __builtin_bit_cast(int, hi);
          }
          // lanes 0..15 of every 32 hand over their second row and get their partners' first, lanes 16..31 the
          // other way round: v_permlane16_swap exchanges the odd rows of 16 lanes of its first operand with the
          // even rows of its second
          const auto s0 = __builtin_amdgcn_permlane16_swap((unsigned)o[0][0], (unsigned)o[1][0], false, false);
          const auto s1 = __builtin_amdgcn_permlane16_swap((unsigned)o[0][1], (unsigned)o[1][1], false, false);
          const v4i out = {(int)s0[0], (int)s1[0], (int)s0[1], (int)s1[1]};
          if (L8_GEMM_DIAG != 3 && !(L8_GEMM_DIAG == 8 && (qd & 1)))  // experiments: no stores (3), half of them (8)
            store16(out, rsC, c_voff, (row + e2) * ldc2, 2 /* streaming */);
          // one row pair at a time: left free, the scheduler reads a hundred accumulator registers ahead and the
          // register pressure of this conversion makes the allocator spill values the K loop uses in every trip
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (L8_GEMM_PROF) {
      tq0 = __builtin_readcyclecounter();
      prof[10] += tq0 - tq2;
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tm][tn][v] = 0.0f;
  };

  auto store_tile = [&](int m0, int n0, auto parts_tag) {
    // The tile's scales (and bias) are used here, on every path, so that the compiler's bookkeeping of outstanding
    // loads knows them landed whichever conversion follows.  Without it the path "requested as a row of scales,
    // converted with a scalar scale" (which no launch takes) left their registers marked as awaited, and the first
    // write to one of them between two tiles got an s_waitcnt vmcnt(0) -- a wait for every store of the tile just
    // written, some 600 cycles with idle matrix cores.
    if constexpr (HAS_BIAS) asm volatile("" : : "v"(seg_sa[0]), "v"(seg_sa[1]), "v"(seg_sb), "v"(seg_bias));
    else asm volatile("" : : "v"(seg_sa[0]), "v"(seg_sa[1]), "v"(seg_sb));
    if (p.sb_row) store_tile_as(m0, n0, parts_tag, std::true_type{});
    else store_tile_as(m0, n0, parts_tag, std::false_type{});
  };

  // ---- SK: exchange of partial sums for tiles whose K range is shared out ----
  // Tail tile tt of XCD x has flag sk_flags[tt * 8 + x] and the fp32 tile sk_partials[(tt * 8 + x) * 65536 ...],
  // laid out the way the accumulators are held (one 16-byte piece per lane, wave, accumulator and quad: whole KiB per wave store).
  // Partial sums and flags are written and read with device-coherent accesses (they bypass the caches that are
  // not shared by all compute units), so no cache needs flushing or invalidating: a wave waits until its own
  // stores are acknowledged, the workgroup meets at a barrier, and one lane then raises the flag.
  [[maybe_unused]] auto partial_rsrc = [&](int slot) {
    return make_rsrc(p.sk_partials + (int64_t)slot * (BM * BN), BM * BN * 4);
  };
  [[maybe_unused]] auto write_partial = [&](int slot) {
    const __amdgpu_buffer_rsrc_t rs = partial_rsrc(slot);
    const int voff = lane * 16;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const v4f v = {acc_read(tm, tn, 4 * qd), acc_read(tm, tn, 4 * qd + 1), acc_read(tm, tn, 4 * qd + 2), acc_read(tm, tn, 4 * qd + 3)};
          store16(__builtin_bit_cast(v4i, v), rs, voff, piece_off(slot, (tm * TN + tn) * 4 + qd), kCoherent);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tm][tn][v] = 0.0f;
    L8_WAIT_VM_LGKM0(0);  // this wave's part of the tile has reached the point of coherence
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (threadIdx.x == 0) __hip_atomic_store(p.sk_flags + slot, p.sk_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // Wait until the partial sums in `slot` have been published in this launch.  Their maker has a lower number
  // than the caller (dispatched earlier) and never waits for anybody.  The wait is bounded all the same: a flag
  // that never comes poisons the tile with a NaN instead of hanging the GPU.
  [[maybe_unused]] auto wait_partial = [&](int slot) -> bool {
#pragma unroll 1
    for (int spin = 0; spin < p.sk_wait_limit; ++spin) {
      const uint32_t f = __hip_atomic_load(p.sk_flags + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((uint32_t)__builtin_amdgcn_readfirstlane((int)f) == p.sk_epoch) return true;
      __builtin_amdgcn_s_sleep(32);
    }
    return false;
  };

  if (L8_GEMM_DIAG == 5 || L8_GEMM_DIAG == 6) {  // experiments: XCD x starts x/8 of a tile's duration late (5); workgroup loc of an XCD starts loc/256 of it late (6)
    const uint64_t t_go = __builtin_amdgcn_s_memrealtime() + (L8_GEMM_DIAG == 5 ? (uint64_t)xcd * (uint64_t)KT * 17 : (uint64_t)loc * (uint64_t)KT * 17 / 32);  // ~1.36 us per K tile, 100 MHz ticks
    while (__builtin_amdgcn_s_memrealtime() < t_go) __builtin_amdgcn_s_sleep(8);
  }
  // ---- prologue: K tiles 0 and 1 of the workgroup's stream requested, K tile 0 published, its first step read ----
  ld_open(0);
#pragma unroll
  for (int u = 0; u < R - 1; ++u) {
#pragma unroll
    for (int i = 0; i < NL; ++i) load_one(u & 1, u, i);
    if (u & 1) ld_advance();
  }
  v8i af0[TM], bf0[TN], af1[TM], bf1[TN];
  uint32_t ad[4];
  L8_WAIT_VM_LGKM0(PEND0);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  frag_addrs(0, 1, 0, ad);
#pragma unroll
  for (int f = 0; f < TM + TN; ++f) read_one(ad, af0, bf0, f);

  // One trip = one K tile = two matrix-core steps of 64, laid out as in the kernel above: first half = MFMAs
  // of step 0 + LDS reads of step 1 + requests for the A panel two K tiles ahead; barrier; second half =
  // MFMAs of step 1 + LDS reads of the next K tile's step 0 + requests for the matching B panel.
  constexpr int N_MMA = TM * TN, NF = TM + TN;
  constexpr int STRADDLE = L8_STRADDLE < N_MMA - 2 ? L8_STRADDLE : 0;
  constexpr int S1 = N_MMA - STRADDLE, S2 = N_MMA + STRADDLE;
  int s0 = 0;  // ring slot of the A panel of the K tile being multiplied
  // WAIT = the count of the wait in front of the barrier: everything older than the WAIT youngest requests must
  // have landed.
  // A wave issues in order and the matrix cores want an MFMA every 64 cycles, about a dozen issue slots: a group
  // that carries more than that leaves them idle.  So nothing but its MFMA, LDS reads and panel loads goes into a
  // group: the fragment addresses of a half are formed in the middle of the half before (ad_a for the first half,
  // ad_b for the second), and the LDS reads of a half are all issued in its first RD groups, so that the wait for
  // them at the end of the half (barrier, loop top) finds them landed.
  constexpr int RD = L8_READ_GROUPS < S1 ? L8_READ_GROUPS : S1, G_ADDR = N_MMA / 2;
  static_assert(RD >= NF / 2 && RD <= S1 && RD <= S2 - STRADDLE && G_ADDR < S1, "group layout");
  uint32_t ad_a[4], ad_b[4];
  frag_addrs(0, 1, 1, ad_a);
  auto trip = [&](auto wait_tag) {
    constexpr int WAIT = decltype(wait_tag)::value;
    const int slot_u1 = wrap(s0 + R - 1);
#pragma unroll
    for (int i = 0; i < S1; ++i) {
      mma_one(af0, bf0, i);
      if (i < RD) {
#pragma unroll
        for (int f = (NF * i) / RD; f < (NF * (i + 1)) / RD; ++f) read_one(ad_a, af1, bf1, f);
      }
#pragma unroll
      for (int j = (NL * i) / S1; j < (NL * (i + 1)) / S1; ++j) load_one(false, slot_u1, j);
      if (i == G_ADDR) frag_addrs(wrap(s0 + 2), wrap(s0 + 3), 0, ad_b);
      __builtin_amdgcn_sched_barrier(0);
    }
    L8_WAIT_VM_LGKM0(WAIT);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < S2; ++i) {
      if (i < STRADDLE) mma_one(af0, bf0, S1 + i);
      else mma_one(af1, bf1, i - STRADDLE);
      if (i >= STRADDLE && i - STRADDLE < RD) {
#pragma unroll
        for (int f = (NF * (i - STRADDLE)) / RD; f < (NF * (i - STRADDLE + 1)) / RD; ++f) read_one(ad_b, af0, bf0, f);
      }
#pragma unroll
      for (int j = (NL * i) / S2; j < (NL * (i + 1)) / S2; ++j) load_one(true, s0, j);
      if (i == STRADDLE + G_ADDR) {
        const int s_next = wrap(s0 + 2);
        frag_addrs(s_next, wrap(s_next + 1), 1, ad_a);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    ld_advance();
    s0 = wrap(s0 + 2);
  };
  using std::integral_constant;
#pragma unroll 1
  for (int seg = 0; seg < n_seg; ++seg) {
    [[maybe_unused]] uint64_t t_loop = 0;
    if (L8_GEMM_PROF) {
      if (seg == 0) prof[1] = __builtin_amdgcn_s_memrealtime();
      t_loop = __builtin_readcyclecounter();
    }
    int m0, n0;
    cursor_origin(cur_mul, m0, n0);
    cursor_step(cur_mul);
    if (L8_GEMM_PROF && seg > 0) prof[17] += __builtin_readcyclecounter() - t_loop;
    if (SK && seg > 0) lane_consts();
    if (L8_GEMM_PROF && seg > 0) {
      asm volatile("" : "+v"(a_voff[0]), "+v"(b_voff[1]), "+v"(foff[1][1]));
      prof[18] += __builtin_readcyclecounter() - t_loop;
    }
    load_scales(m0, n0);
    int kt = 0;
    if (L8_GEMM_PROF && seg > 0) prof[16] += __builtin_readcyclecounter() - t_loop;  // tile origin, lane constants, scale requests
    if (seg > 0) {
      // The first barrier after the N_STORES stores of a C tile: they are younger than the panels waited for
      // and the counter retires in order, so the count allows for them (waiting for the stores themselves would
      // stall the start of every tile).
      trip(integral_constant<int, N_STORES + PEND>{});
      kt = 1;
      if (L8_GEMM_PROF && !SK && KT > 4) {  // the first trips after a stored tile, one by one
        const uint64_t ta = __builtin_readcyclecounter();
        prof[12] += ta - t_loop;
        trip(integral_constant<int, PEND>{});
        const uint64_t tb = __builtin_readcyclecounter();
        prof[13] += tb - ta;
        trip(integral_constant<int, PEND>{});
        const uint64_t tc = __builtin_readcyclecounter();
        prof[14] += tc - tb;
        trip(integral_constant<int, PEND>{});
        prof[15] += __builtin_readcyclecounter() - tc;
        kt = 4;
      }
    }
#pragma unroll 1
    for (; kt < KT; ++kt) trip(integral_constant<int, PEND>{});
    if (L8_GEMM_PROF) {
      const uint64_t t = __builtin_readcyclecounter();
      prof[3] += t - t_loop;
      t_loop = t;
    }
    store_tile(m0, n0, std::false_type{});
    if (L8_GEMM_PROF) prof[4] += __builtin_readcyclecounter() - t_loop;
  }
  if (L8_GEMM_PROF) prof[11] = __builtin_amdgcn_s_memrealtime();
  if constexpr (SK) {
    // ---- the workgroup's share of the tail ----
    bool after_store = true;  // the segment before ended with the N_STORES stores of a C tile (n_seg > 0 here)
#pragma unroll 1
    for (int pc = 0; pc < n_tail; ++pc) {
      int m0, n0;
      const int tt = piece_of(pc, m0, n0);
      const bool owns = !helper;  // the tile's first K tiles: this workgroup adds the helper's sums and stores the tile
      const int slot = tt * 8 + xcd;
      lane_consts();
      if (owns) load_scales(m0, n0);
      [[maybe_unused]] uint64_t t_a = 0, t_b = 0;
      if (L8_GEMM_PROF) t_a = __builtin_readcyclecounter();
      if (after_store) trip(integral_constant<int, N_STORES + PEND>{});
      else trip(integral_constant<int, PEND>{});  // write_partial waited for everything in flight
#pragma unroll 1
      for (int kt = piece_kb + 1; kt < piece_ke; ++kt) trip(integral_constant<int, PEND>{});
      if (L8_GEMM_PROF) {
        t_b = __builtin_readcyclecounter();
        prof[12] += t_b - t_a;
      }
      if (!owns) {
        write_partial(slot);
        after_store = false;
        if (L8_GEMM_PROF) prof[13] += __builtin_readcyclecounter() - t_b;
      } else {
        if (!wait_partial(slot)) {
          seg_sa[0] = seg_sa[1] = 0x7fc00000;  // every row scale a NaN
          // and the host can find out: one more tile poisoned, counted in the workspace (never reset by the library)
          if (threadIdx.x == 0) atomicAdd(p.sk_flags + kSkGaveUpWord, 1u);
        }
        if (L8_GEMM_PROF) {
          t_a = __builtin_readcyclecounter();
          prof[14] += t_a - t_b;
        }
        rs_p = partial_rsrc(slot);
        p_slot = slot;
        store_tile(m0, n0, std::true_type{});
        after_store = true;
        if (L8_GEMM_PROF) prof[15] += __builtin_readcyclecounter() - t_a;
      }
    }
  }
  // the tail requests (out of range, zero filling) must have landed before the workgroup's LDS is released
  L8_WAIT_VM_LGKM0(0);
  if (L8_GEMM_PROF) {
    prof[2] = __builtin_amdgcn_s_memrealtime();
    prof[5] = __builtin_readcyclecounter() - prof[5];
    prof[6] = n_seg;
    prof[7] = ((uint64_t)__builtin_amdgcn_s_getreg(63508) << 32) | (uint32_t)__builtin_amdgcn_s_getreg(63492);  // XCC_ID, HW_ID
    if (threadIdx.x == 0 && p.dbg) {
      uint64_t *d = p.dbg + (int64_t)blockIdx.x * 24;
      for (int i = 0; i < 24; ++i) d[i] = prof[i];
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
  bool persistent;   // one workgroup per compute unit walks a list of tiles
  gemm_fn fn_bias;   // persistent kernels: the instantiation that adds a bias (the plain kernels branch inside)
  gemm_fn fn_sk;     // persistent kernels: the instantiation that can share a tile's K range out (bias-free), or null
};

// X(WM, WN, TM, TN, R, GROUP_M, PF) -- 1-based position in this list is the `algo` number
#define L8_ALGO_LIST(X)                                                          \
  X(2, 2, 4, 4, 5, 4, 0)  /* 1: 256x256, 4 waves (128x128 each), ring of 5    */ \
  X(2, 2, 2, 2, 5, 4, 0)  /* 2: 128x128, 4 waves (small problems)             */ \
  X(2, 4, 4, 2, 5, 4, 0)  /* 3: 256x256, 8 waves (128x64 each)                */ \
  X(4, 2, 2, 4, 5, 4, 0)  /* 4: 256x256, 8 waves (64x128 each)                */ \
  X(2, 2, 4, 4, 5, 8, 0)  /* 5: algo 1 with taller groups                     */ \
  X(2, 2, 4, 4, 5, 2, 0)  /* 6: algo 1 with shorter groups                    */ \
  X(2, 2, 4, 4, 5, 4, 4)  /* 7: algo 1 with L2 touches 4 K tiles ahead        */ \
  X(2, 4, 4, 2, 5, 4, 4)  /* 8: algo 3 with L2 touches 4 K tiles ahead        */ \
  X(2, 2, 4, 4, 5, 16, 0) /* 9: algo 1 with groups of 16                      */ \
  X(2, 4, 4, 2, 5, 8, 0)  /* 10: algo 3 with taller groups                    */

#define L8_INSTANTIATE(WM, WN, TM, TN, R, GM, PF) \
  template __global__ void gemm_nt_kernel<WM, WN, TM, TN, R, GM, PF>(const GemmArgs);
L8_ALGO_LIST(L8_INSTANTIATE)

#define L8_MAX2(a, b) ((a) > (b) ? (a) : (b))
#define L8_ALGO_ROW(WM, WN, TM, TN, R, GM, PF)                                                                \
  {"mt" #WM "x" #WN "w_" #TM "x" #TN "t_r" #R "_g" #GM "_pf" #PF, gemm_nt_kernel<WM, WN, TM, TN, R, GM, PF>, \
   WM * TM * 32, WN * TN * 32, WM * WN * 64, R * L8_MAX2(WM * TM * 32, WN * TN * 32) * 128, false, nullptr, nullptr},

template __global__ void gemm_nt_stream_kernel<8, false>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<8, true>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<4, false>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<4, true>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<4, false, true>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<2, false>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<2, true>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<16, false>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<16, true>(const GemmArgs);
template __global__ void gemm_nt_stream_kernel<4, false, false, 8>(const GemmArgs);

static const Algo kAlgos[] = {
    L8_ALGO_LIST(L8_ALGO_ROW)
    /* 11, 12: persistent 256x256 tiles, 4 waves, one panel stream across tiles, C stored from the accumulators */
    {"stream_mt2x2w_4x4t_r5_g8", gemm_nt_stream_kernel<8, false>, 256, 256, 256, 5 * 256 * 128, true, gemm_nt_stream_kernel<8, true>, nullptr},
    {"stream_mt2x2w_4x4t_r5_g4", gemm_nt_stream_kernel<4, false>, 256, 256, 256, 5 * 256 * 128, true, gemm_nt_stream_kernel<4, true>, nullptr},
    /* 13, 14: other shapes of the block of tiles resident on an XCD (2 x 16 and 16 x 2 instead of 4 x 8: 18 panels
       shared by 32 tiles instead of 12), kept for the traffic comparison */
    {"stream_mt2x2w_4x4t_r5_g2", gemm_nt_stream_kernel<2, false>, 256, 256, 256, 5 * 256 * 128, true, gemm_nt_stream_kernel<2, true>, nullptr},
    {"stream_mt2x2w_4x4t_r5_g16", gemm_nt_stream_kernel<16, false>, 256, 256, 256, 5 * 256 * 128, true, gemm_nt_stream_kernel<16, true>, nullptr},
    /* 15: algo 12 that may share the K range of the last round's tiles out between workgroups (l8_gemm_nt_ws with
       a workspace; without one it is algo 12).  Measured neutral on the shapes it applies to: the part is
       power-limited, and the compute units that the plain split leaves idle in the last round let the busy ones
       clock higher, which recovers most of what the idle ones lose. */
    {"stream_mt2x2w_4x4t_r5_g4_sk", gemm_nt_stream_kernel<4, false>, 256, 256, 256, 5 * 256 * 128, true, gemm_nt_stream_kernel<4, true>,
     gemm_nt_stream_kernel<4, false, true>},
    /* 16: algo 12 with eight waves (two per SIMD, 64x128 each), kept for the comparison: measured 1-2 % ahead of
       algo 12 at K = 4096 and 2-4 % behind it at K >= 8192 (1.5 x the LDS reads); a product with a bias takes the
       plain kernel (the bias instantiation would not fit the 256 registers of a wave without spills) */
    {"stream_mt4x2w_2x4t_r5_g4", gemm_nt_stream_kernel<4, false, false, 8>, 256, 256, 512, 5 * 256 * 128, true, nullptr, nullptr},
};
constexpr int kNumAlgos = sizeof(kAlgos) / sizeof(kAlgos[0]);

}  // namespace l8

using namespace l8;

extern "C" int l8_gemm_algo_count(void) { return kNumAlgos; }
extern "C" const char *l8_gemm_algo_name(int algo) {
  return (algo >= 1 && algo <= kNumAlgos) ? kAlgos[algo - 1].name : nullptr;
}

// plain kernel for a problem with at least one 256x256 tile per compute unit: four waves with 128x128 wave
// tiles (least LDS traffic per flop) unless K is so short (measured: below 4096) that the conversion of the C
// tile, which eight waves share out over twice as many wave slots, weighs more than the K loop
static int pick_plain_big(int64_t K) { return K >= 4096 ? 5 : 3; }

static int pick_algo(int64_t M, int64_t N, int64_t K) {
  // large problems: the persistent kernel (measured 2-11 % ahead of the plain ones on every shape with at
  // least one 256x256 tile per compute unit; groups of 4 tile rows ahead of groups of 8 by 1-3 %), also when
  // the big tiles leave up to 7/16 of the compute units idle (measured with K = 2048 .. 16384: 144 to 240
  // tiles on 256 compute units run 10-25 % faster than with 128x128 tiles, 128 tiles and fewer 15-45 % slower);
  // problems that would leave more of the chip idle with big tiles: 128x128 tiles
  (void)K;
  const int64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (big_tiles * 16 >= (int64_t)num_cus() * 9) return 12;
  return 2;
}

// Host arithmetic only: the tile configuration `algo = 0` resolves to for this problem on the current device when
// the operands allow every kernel (aligned, N % 8 == 0): what a caller that reports per-kernel figures names.
extern "C" int l8_gemm_pick(int64_t M, int64_t N, int64_t K) {
  L8_REQUIRE(M > 0 && N > 0 && K > 0, "l8_gemm_pick: empty problem");
  return pick_algo(M, N, K);
}

// flags (one 4-byte word per workgroup, first 4 KiB) + one fp32 256x256 tile per workgroup of a persistent launch
constexpr int64_t kSkMaxGrid = kSkMaxGridWords, kSkFlagBytes = (kSkMaxGrid + 64) * 4, kSkTileBytes = 256 * 256 * 4;
static std::atomic<uint32_t> g_sk_epoch{0};
// polls (about a microsecond each) an owner spends on a helper's flag before it gives up: a third of a second
static std::atomic<int> g_sk_wait_limit{1 << 18};

extern "C" int l8_gemm_set_wait_limit(int polls) {
  L8_REQUIRE(polls >= 0, "l8_gemm_set_wait_limit: negative limit");
  g_sk_wait_limit = polls;
  return L8_OK;
}

extern "C" int64_t l8_gemm_workspace_gave_up_offset(void) { return (int64_t)kSkGaveUpWord * 4; }

extern "C" int64_t l8_gemm_workspace(void) {
  const int64_t cus8 = (num_cus() / 8) * 8;
  return kSkFlagBytes + (cus8 < 8 ? 8 : cus8) * kSkTileBytes;
}

// Does sharing out the K range of the last round's tiles pay for an XCD with `cnt` tiles, W workgroups and KT K
// tiles per tile?  (Same test as in the kernel.)
static bool sk_pays(int64_t cnt, int64_t W, int64_t KT) {
  const int64_t n_rounds = cnt / W, r = cnt % W, n_help = W - r;
  const int64_t m_help = (r + n_help - 1) / n_help;
  const int64_t l_help = (KT + kSkFixCost - m_help * kSkWriteCost) / (m_help + 1);
  return n_rounds > 0 && r > 0 && l_help >= kSkMinSaved;
}

// Host arithmetic only (no GPU needed): on a part with `compute_units` compute units, how many of the 8 XCDs would
// share out the K range of their last round's tiles under tile configuration 15 for this problem.
extern "C" int l8_gemm_shares_k(int64_t M, int64_t N, int64_t K, int compute_units) {
  L8_REQUIRE(M >= 0 && N >= 0 && K >= 0 && compute_units >= 8, "l8_gemm_shares_k: bad argument");
  const int64_t nblocks = ((M + 255) / 256) * ((N + 255) / 256), KT = (K + 127) / 128;
  const int64_t cus8 = (compute_units / 8) * 8, want = (nblocks + 7) / 8 * 8;
  int64_t grid = want < cus8 ? want : cus8;
  if (grid < 8) grid = 8;
  const int64_t W = grid / 8, q = nblocks / 8, rem = nblocks % 8;
  return (int)((sk_pays(q + 1, W, KT) ? rem : 0) + (sk_pays(q, W, KT) ? 8 - rem : 0));
}

static int gemm_nt_impl(const void *A, const void *B, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                        const float *sa, int sa_mode, const float *sb, int sb_mode, const void *bias, void *C,
                        int64_t ldc, int algo, void *workspace, int64_t workspace_bytes, void *stream) {
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
  if (kAlgos[algo - 1].persistent) {
    // the persistent kernel stores 16 aligned bytes (eight columns) per lane and reads the row scales 16 bytes
    // at a time; operands that do not allow that go to the plain kernel with the same tile shape
    // (and addresses its scale vectors with 32-bit byte offsets)
    const bool ok = N % 8 == 0 && ldc % 8 == 0 && ((uintptr_t)C % 16) == 0 && ldc < (1LL << 22) &&
                    M < (1LL << 29) && N < (1LL << 29) &&
                    (sa_mode != L8_SCALE_ROW || ((uintptr_t)sa % 16) == 0) &&
                    (sb_mode != L8_SCALE_ROW || ((uintptr_t)sb % 16) == 0) &&
                    (bias == nullptr || (((uintptr_t)bias % 8) == 0 && kAlgos[algo - 1].fn_bias != nullptr));
    if (!ok) algo = pick_plain_big(K);
  }
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
  p.sk_flags = nullptr;
  p.sk_partials = nullptr;
  p.sk_epoch = 0;
  p.sk_wait_limit = 0;
  p.dbg = nullptr;
  if (L8_GEMM_PROF && al.persistent) {
    p.dbg = (uint64_t *)bias;
    p.bias = nullptr;
  }
  p.C = (uint16_t *)C;
  p.tiles_m = (int)((M + al.bm - 1) / al.bm);
  p.tiles_n = (int)((N + al.bn - 1) / al.bn);
  const int64_t nblocks = (int64_t)p.tiles_m * p.tiles_n;
  L8_REQUIRE(nblocks < (1LL << 31), "l8_gemm_nt: too many tiles");
  static bool attr_done[kMaxDev][kNumAlgos] = {};  // idempotent; a race only repeats the call
  const int slot = device_slot();
  if (slot < 0 || !attr_done[slot][algo - 1]) {
    L8_HIP(hipFuncSetAttribute((const void *)al.fn, hipFuncAttributeMaxDynamicSharedMemorySize, al.lds));
    if (al.fn_bias) L8_HIP(hipFuncSetAttribute((const void *)al.fn_bias, hipFuncAttributeMaxDynamicSharedMemorySize, al.lds));
    if (al.fn_sk) L8_HIP(hipFuncSetAttribute((const void *)al.fn_sk, hipFuncAttributeMaxDynamicSharedMemorySize, al.lds));
    if (slot >= 0) attr_done[slot][algo - 1] = true;
  }
  int64_t grid = nblocks;
  if (al.persistent) {
    // one workgroup per compute unit, a multiple of 8 of them (the hardware deals workgroups to the 8 XCDs in turn)
    const int64_t cus8 = (num_cus() / 8) * 8;
    const int64_t want = (nblocks + 7) / 8 * 8;
    grid = want < cus8 ? want : cus8;
    if (grid < 8) grid = 8;
  }
  gemm_fn fn = (al.fn_bias && p.bias) ? al.fn_bias : al.fn;
  if (al.fn_sk && !p.bias && workspace != nullptr && grid <= kSkMaxGrid && workspace_bytes >= kSkFlagBytes + grid * kSkTileBytes) {
    // the kernel decides per XCD (their tile counts differ by at most one) with the same test
    const int64_t W = grid / 8, KT = (K + 127) / 128, q = nblocks / 8;
    bool use = sk_pays(q, W, KT) || (nblocks % 8 != 0 && sk_pays(q + 1, W, KT));
    if (use) {
      // Not inside a stream capture: the launch number is a kernel argument, and a replayed launch would find
      // the flags of the replay before already at its number.
      hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess) {
        (void)hipGetLastError();
        use = false;
      } else if (cs != hipStreamCaptureStatusNone) {
        use = false;
      }
    }
    if (use) {
      fn = al.fn_sk;
      p.sk_flags = (uint32_t *)workspace;
      p.sk_partials = (float *)((uint8_t *)workspace + kSkFlagBytes);
      uint32_t e = ++g_sk_epoch;
      if (e == 0) e = ++g_sk_epoch;  // 0 is what an untouched flag holds
      p.sk_epoch = e;
      p.sk_wait_limit = g_sk_wait_limit;
    }
  }
  hipLaunchKernelGGL(fn, dim3((unsigned)grid), dim3(al.threads), al.lds, (hipStream_t)stream, p);
  L8_HIP(hipGetLastError());
  return L8_OK;
}

extern "C" int l8_gemm_nt(const void *A, const void *B, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                          const float *sa, int sa_mode, const float *sb, int sb_mode, const void *bias, void *C,
                          int64_t ldc, int algo, void *stream) {
  return gemm_nt_impl(A, B, M, N, K, lda, ldb, sa, sa_mode, sb, sb_mode, bias, C, ldc, algo, nullptr, 0, stream);
}

extern "C" int l8_gemm_nt_ws(const void *A, const void *B, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                             const float *sa, int sa_mode, const float *sb, int sb_mode, const void *bias, void *C,
                             int64_t ldc, int algo, void *workspace, int64_t workspace_bytes, void *stream) {
  L8_REQUIRE(workspace == nullptr || ((uintptr_t)workspace % 16) == 0, "l8_gemm_nt_ws: workspace must be 16-byte aligned");
  return gemm_nt_impl(A, B, M, N, K, lda, ldb, sa, sa_mode, sb, sb_mode, bias, C, ldc, algo, workspace, workspace_bytes, stream);
}
