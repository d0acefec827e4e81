/*
 * lingua_fp8 -- C ABI of the MI355X (gfx950) float8 linear kernels.
 *
 * The reference (facebookresearch/lingua) has no native layer: its float8
 * path is Python issuing ATen ops.  Each entry point below replaces the ATen
 * call sequence at the cited lines of the reference's lingua/float8.py and is
 * what a Python binding (ctypes) of that file binds instead.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; the library
 *     allocates nothing, keeps no reference and never synchronises;
 *   - `stream` is a hipStream_t (NULL = the null stream); work is enqueued on
 *     it and the call returns at once;
 *   - bf16 / e4m3 data are passed as `void *` (2-byte / 1-byte elements);
 *     leading dimensions (`ld*`) are in ELEMENTS;
 *   - return value: 0 on success, a negative L8_E* code otherwise; the text
 *     of the last failure on the calling thread is l8_last_error();
 *   - entry points are re-entrant and thread-safe (forward and autograd
 *     threads may call concurrently).
 */
#ifndef LINGUA_FP8_H
#define LINGUA_FP8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define L8_OK 0
#define L8_EINVAL (-1)  /* bad shape, alignment or null pointer */
#define L8_EARCH (-2)   /* device is not gfx950 */
#define L8_EHIP (-3)    /* a HIP runtime call failed */

/* scale modes of l8_gemm_nt */
#define L8_SCALE_SCALAR 0 /* one fp32 value for the whole operand */
#define L8_SCALE_ROW 1    /* one fp32 value per row of the operand */

int l8_version(void);
const char *l8_last_error(void);

/* 0 when `device` (HIP ordinal) is a gfx950 part, L8_EARCH otherwise.  There
 * is no other code path: callers must fail when this fails. */
int l8_device_check(int device);

/* How every cast of this library evaluates `torch.clamp(amax_t.float(), min=EPS) / FP8_MAX` (lingua/float8.py:44):
 *   L8_SCALE_RULE_DIVIDE (default): the correctly rounded fp32 quotient amax / 448 -- what the ATen CPU kernel
 *     computes and what the benchmark's recipe states ("scale = amax/448, fp32").
 *   L8_SCALE_RULE_TIMES_INVERSE: amax * fp32(1/448) -- what ATen's GPU kernel computes for a division of a tensor
 *     by a Python scalar (it multiplies by the reciprocal), i.e. what the reference produces when it runs on a GPU.
 *     The product differs from the quotient in the last bit for about half of all amaxes; bf16 inputs land on
 *     exact rounding ties of e4m3 often enough that 0.03-0.1 % of the fp8 bytes then differ as well.
 * Process-wide; takes effect for calls made after it returns (quantised copies made before keep their rule). */
#define L8_SCALE_RULE_DIVIDE 0
#define L8_SCALE_RULE_TIMES_INVERSE 1
int l8_set_scale_rule(int rule);
int l8_get_scale_rule(void);

/* Row-wise amax -> scale -> cast.
 * Replaces lingua/float8.py:86-87 (abs/amax per row) + :43-47 (scale()).
 *   x        bf16 [R,C], row stride ldx
 *   q        e4m3fn [R,C], row stride ldq           (may be NULL: amax only)
 *   scale    fp32 [R] = max(f32(amax),1e-12)/448    (may be NULL with q)
 *   amax     bf16 [R] row amax, NaN propagating     (may be NULL)
 *   col_amax fp32 [C] (may be NULL): receives the column amaxes of x (as
 *            non-negative float bit patterns; overwritten, nothing to
 *            initialise), so that a later l8_cast_colwise_transposed() needs
 *            no pass of its own to find them.
 *   workspace  device scratch of at least l8_cast_rowwise_workspace(R, C)
 *            bytes, 16-byte aligned; needed only with col_amax (per-workgroup
 *            partial maxima, folded by a second launch on the same stream).
 * Requires C % 8 == 0, ldx % 8 == 0, ldq % 8 == 0 and 16-byte aligned x / 8-byte aligned q. */
int l8_cast_rowwise(const void *x, int64_t R, int64_t C, int64_t ldx,
                    void *q, int64_t ldq, float *scale, void *amax, float *col_amax,
                    void *workspace, int64_t workspace_bytes, void *stream);
int64_t l8_cast_rowwise_workspace(int64_t R, int64_t C);

/* l8_cast_rowwise for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose ATen ops
 * allocate freely.  Same arguments and results as l8_cast_rowwise without the workspace: the partial
 * column maxima go to a static device array of L8_NOALLOC_SCRATCH_BYTES that every GPU the library runs
 * on holds until the process ends.  Calls no allocator.
 *   - shapes whose l8_cast_rowwise_workspace(R, C) exceeds L8_NOALLOC_SCRATCH_BYTES are rejected
 *     (L8_EINVAL) when col_amax is given: with 256 compute units that is C > 16384 together with
 *     R >= 512; without col_amax no scratch is used and any shape goes;
 *   - all calls on one GPU share that GPU's array: two calls with col_amax that overlap in time on the
 *     same GPU (different streams or threads) race.  Nothing in it needs clearing between calls: every
 *     call writes the part it reads.
 *   - the array's address is looked up once per device, by l8_device_check(device) or else by the first
 *     call on that device; call l8_device_check before capturing. */
#define L8_NOALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
int l8_cast_rowwise_noalloc(const void *x, int64_t R, int64_t C, int64_t ldx,
                            void *q, int64_t ldq, float *scale, void *amax, float *col_amax, void *stream);

/* Row-wise scale -> cast with the row amaxes handed in, exactly as scale(t, amax_t) of
 * lingua/float8.py:43-47 takes them: scale[r] = max(f32(amax[r]),1e-12)/448, q = e4m3(x * (1/scale)).
 * The amax is used as given (a repeated tensor amax as at :116-118, an amax of an earlier step); where
 * it is smaller than the row's true amax the cast behaves like the ATen one: products up to 464 round
 * to +-448, larger ones give the NaN code.
 *   amax [R], bf16 (amax_dtype = L8_AMAX_BF16: what the reference's amax reductions of bf16 tensors return) or
 *   fp32 (L8_AMAX_F32: a caller's own fp32 amax, e.g. a history; the reference converts with .float(), so an
 *   fp32 amax must not be rounded to bf16 on the way);  q e4m3fn [R,C] (ldq);  scale fp32 [R]
 * Requires C % 8 == 0, ldx % 8 == 0, ldq % 8 == 0, 16-byte aligned x / 8-byte aligned q. */
#define L8_AMAX_BF16 0
#define L8_AMAX_F32 1
int l8_cast_rowwise_given_amax(const void *x, int64_t R, int64_t C, int64_t ldx, const void *amax, int amax_dtype,
                               void *q, int64_t ldq, float *scale, void *stream);

/* Column amax on its own: col_amax fp32 [C] is overwritten, as above. */
int l8_col_amax(const void *x, int64_t R, int64_t C, int64_t ldx, float *col_amax, void *stream);

/* bf16 amax[n] -> bf16 amax_out[1] = max, NaN propagating.
 * Replaces lingua/float8.py:115 (tensor amax of the weight from the row
 * amaxes saved by forward). */
int l8_amax_reduce(const void *amax, int64_t n, void *amax_out, void *stream);

/* Tensor-wise scale -> cast with a device-resident amax scalar (bf16 or fp32, amax_dtype as above).
 * Replaces lingua/float8.py:111 (b_t.t().contiguous()) + :116-118
 * (repeat_interleave of the scalar) + :43-47 (scale()) for the dgrad weight.
 *   transpose == 0 : q is [R,C] (ldq >= C);  != 0 : q is [C,R] (ldq >= R)
 *   scale    fp32 [1]
 * Requires C % 8 == 0, ldx % 8 == 0; with transpose != 0 also ldx < 2^21 elements. */
int l8_cast_tensorwise(const void *x, int64_t R, int64_t C, int64_t ldx,
                       const void *amax, int amax_dtype, int transpose,
                       void *q, int64_t ldq, float *scale, void *stream);

/* Column-wise (token-dimension) scale -> cast, written transposed:
 * equals scale(x.t().contiguous(), its row amax) (lingua/float8.py:43-47 applied to
 * the operand layout an fp8 wgrad needs; the reference computes wgrad in bf16 at :123).
 *   col_amax fp32 [C] column amaxes of x (from l8_cast_rowwise / l8_col_amax)
 *   q        e4m3fn [C,R], row stride ldq;  scale fp32 [C]
 * Requires C % 8 == 0, ldx % 8 == 0, ldx < 2^21 elements. */
int l8_cast_colwise_transposed(const void *x, int64_t R, int64_t C, int64_t ldx,
                               const float *col_amax,
                               void *q, int64_t ldq, float *scale, void *stream);

/* Scaled fp8 product, both operands reduction-contiguous ("NT"):
 *   C[m,n] = bf16( (sum_k A[m,k]*B[n,k]) * sa[m or 0] * sb[n or 0] + bias[n] )
 * fp32 accumulation on the fp8 matrix cores.  Replaces torch._scaled_mm and the
 * post-scaling around it at lingua/float8.py:65-77 (forward, dgrad) and serves
 * the fp8 wgrad.
 *   A e4m3fn [M,K] (lda), B e4m3fn [N,K] (ldb), C bf16 [M,N] (ldc)
 *   sa_mode / sb_mode: L8_SCALE_SCALAR or L8_SCALE_ROW;  bias bf16 [N] or NULL
 *   algo: 0 = library default; other values select a tile configuration (see l8_gemm_algo_count)
 * Requires K % 16 == 0, lda % 16 == 0, ldb % 16 == 0, 16-byte aligned A and B
 * (the same multiple-of-16 rule torch._scaled_mm enforces). */
int l8_gemm_nt(const void *A, const void *B, int64_t M, int64_t N, int64_t K,
               int64_t lda, int64_t ldb,
               const float *sa, int sa_mode, const float *sb, int sb_mode,
               const void *bias, void *C, int64_t ldc, int algo, void *stream);

/* l8_gemm_nt with a workspace.  Tile configuration 15 (opt-in, never the default) uses it to share the K
 * range of the last round's tiles out between workgroups when that round would leave part of the GPU idle
 * (long K, tile count a little above a multiple of the compute units): fp32 partial sums are exchanged
 * through the workspace and added in a fixed order, so results do not vary from call to call.  Every other
 * configuration ignores the workspace.  Same replacement as l8_gemm_nt (torch._scaled_mm at
 * lingua/float8.py:65-77 splits K internally as it sees fit).
 *   workspace: l8_gemm_workspace() bytes of device memory, 16-byte aligned, ZERO-FILLED ONCE before its
 *              first use and never written by anyone else afterwards (the library keeps launch numbers in
 *              it); calls that share a workspace must not overlap in time (one workspace per stream).
 *              NULL, too small, a bias, or a stream that is being captured: exactly l8_gemm_nt. */
int l8_gemm_nt_ws(const void *A, const void *B, int64_t M, int64_t N, int64_t K,
                  int64_t lda, int64_t ldb,
                  const float *sa, int sa_mode, const float *sb, int sb_mode,
                  const void *bias, void *C, int64_t ldc, int algo,
                  void *workspace, int64_t workspace_bytes, void *stream);
int64_t l8_gemm_workspace(void);
/* A workgroup that owns a shared tile waits for its helpers' partial sums for a bounded time (about a third of a
 * second; l8_gemm_set_wait_limit).  If the wait runs out -- helpers held up behind other work on the GPU -- the tile
 * is stored as NaNs (never as a wrong number) and the call still returns L8_OK: the kernel cannot report back.
 * Every such tile is counted in one 32-bit word of the workspace, at this byte offset; the library never resets it,
 * so a caller reads it (after synchronising the stream) and compares with what it read before.  No counterpart in
 * the reference. */
int64_t l8_gemm_workspace_gave_up_offset(void);
/* Host arithmetic only: the number of XCDs (0..8) that would share the K range of their last round's tiles out
 * under tile configuration 15, for this problem on a part with `compute_units` compute units (256 on MI355X).
 * 0 = configuration 15 behaves exactly like configuration 12.  No counterpart in the reference. */
int l8_gemm_shares_k(int64_t M, int64_t N, int64_t K, int compute_units);
/* Testing aid for the exchange above (no counterpart in the reference): how many times (about a microsecond
 * each) a workgroup polls for another's partial sums before it gives up and fills its tile with NaN instead
 * of waiting for ever.  Default 262144; 0 makes every shared tile give up at once, which is how the tests
 * reach that path without hanging anything.  Process-wide. */
int l8_gemm_set_wait_limit(int polls);

/* SwiGLU gate fused with the row-wise cast of the w2 input.
 * Replaces `F.silu(self.w1(x)) * self.w3(x)` of lingua/transformer.py:469-471 (two bf16
 * elementwise kernels) followed by the cast of that product in Fp8LinearFn.forward
 * (lingua/float8.py:86-87 + :43-47):
 *   h = bf16( bf16(silu(h1)) * h3 ),  silu(x) = x / (1 + exp(-x)) in fp32,
 *   then amax / scale / q of h as l8_cast_rowwise.
 *   h1, h3   bf16 [R,C] (ld1, ld3)
 *   h        bf16 [R,C] (ldh) or NULL when the caller does not need the product itself
 *   q, scale, amax, col_amax, workspace: as l8_cast_rowwise; the workspace needs
 *            l8_swiglu_workspace(R, C) / 2 bytes.
 * Requires C % 8 == 0, C <= 65536, every leading dimension % 8 == 0. */
int l8_swiglu_cast_rowwise(const void *h1, const void *h3, int64_t R, int64_t C, int64_t ld1, int64_t ld3,
                           void *h, int64_t ldh, void *q, int64_t ldq, float *scale, void *amax,
                           float *col_amax, void *workspace, int64_t workspace_bytes, void *stream);
int64_t l8_swiglu_workspace(int64_t R, int64_t C);

/* Backward of the SwiGLU gate fused with the row-wise casts of its two gradients.
 * Replaces autograd's mul / silu_backward kernels for lingua/transformer.py:469-471 and the
 * casts of grad_out in the backward of w1 and w3 (lingua/float8.py:112-114 + :43-47):
 *   g3 = bf16( dh * bf16(silu(h1)) )
 *   g1 = bf16( bf16(dh * h3) * sig * (1 + h1 * (1 - sig)) ),  sig = 1 / (1 + exp(-h1))
 *   then q1 / scale1 and q3 / scale3 as l8_cast_rowwise of g1 and g3.
 *   dh, h1, h3 bf16 [R,C];  g1, g3 bf16 [R,C] (ldg) are always written (wgrad needs them);
 *   col_amax1, col_amax3 fp32 [C]: both or neither; workspace of l8_swiglu_workspace(R, C) bytes with them.
 * Requires C % 8 == 0, C <= 32768, every leading dimension % 8 == 0. */
int l8_swiglu_bwd_cast_rowwise(const void *dh, const void *h1, const void *h3, int64_t R, int64_t C,
                               int64_t lddh, int64_t ld1, int64_t ld3, void *g1, void *g3, int64_t ldg,
                               void *q1, void *q3, int64_t ldq, float *scale1, float *scale3,
                               float *col_amax1, float *col_amax3,
                               void *workspace, int64_t workspace_bytes, void *stream);

/* RMSNorm fused with the row-wise cast of its output.
 * Replaces RMSNorm.forward of lingua/transformer.py:283-289 (x.float(), x*x, mean, rsqrt, two
 * multiplies, type_as: seven eager kernels) followed by the cast of that output in the forward of
 * the linears it feeds (wq/wk/wv, w1/w3; lingua/float8.py:86-87 + :43-47):
 *   r = rsqrt(mean(f32(x)^2) + eps);  y = bf16((f32(x) * r) * f32(w));  q, scale = row-wise cast of y.
 *   x     bf16 [R,C] (ldx);  w [C], bf16 (w_is_f32 == 0) or fp32
 *   y     bf16 [R,C] (ldy), always written
 *   q, scale: as l8_cast_rowwise, both or neither;  rstd fp32 [R] = r (may be NULL; what backward needs)
 *   col_amax, workspace: as l8_cast_rowwise, workspace of l8_rmsnorm_workspace(R, C) bytes
 * Requires C % 8 == 0, C <= 8192, every leading dimension % 8 == 0. */
int l8_rmsnorm_cast_rowwise(const void *x, const void *w, int w_is_f32, int64_t R, int64_t C, int64_t ldx,
                            float eps, void *y, int64_t ldy, void *q, int64_t ldq, float *scale, float *rstd,
                            float *col_amax, void *workspace, int64_t workspace_bytes, void *stream);
int64_t l8_rmsnorm_workspace(int64_t R, int64_t C);

/* Backward of that norm (what autograd derives from lingua/transformer.py:283-289), one pass over gy and x:
 *   xhat = f32(x) * rstd;  gh = f32(gy) * f32(w)
 *   gx = bf16( (gh - xhat * mean(gh * xhat)) * rstd )      [R,C] (ldgx)
 *   gw = sum over rows of f32(gy) * xhat                    fp32 [C], summed in a fixed order
 *   rstd fp32 [R] as written by l8_rmsnorm_cast_rowwise; workspace of l8_rmsnorm_bwd_workspace(R, C) bytes
 * Requires C % 8 == 0, C <= 8192, every leading dimension % 8 == 0. */
int l8_rmsnorm_bwd(const void *gy, const void *x, const void *w, int w_is_f32, const float *rstd,
                   int64_t R, int64_t C, int64_t ldg, int64_t ldx, void *gx, int64_t ldgx, float *gw,
                   void *workspace, int64_t workspace_bytes, void *stream);
int64_t l8_rmsnorm_bwd_workspace(int64_t R, int64_t C);

int l8_gemm_algo_count(void);
/* human-readable description of tile configuration `algo` (1-based), or NULL */
const char *l8_gemm_algo_name(int algo);
/* Host arithmetic only: the tile configuration that `algo = 0` resolves to for an M x N x K problem on the
 * current device when the operands allow every kernel (aligned, N % 8 == 0).  For callers that report
 * per-kernel figures and must name the kernel that ran.  No counterpart in the reference. */
int l8_gemm_pick(int64_t M, int64_t N, int64_t K);

#ifdef __cplusplus
}
#endif
#endif /* LINGUA_FP8_H */
