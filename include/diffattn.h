/*
 * libdiffattn -- C ABI of the MI355X (gfx950) differential-attention kernels.
 *
 * This is the device-call boundary of the path `layers.MultiheadDiffAttnKernel` ->
 * `kernel._diff_attention.forward/backward` -> kernel launch.  In the reference that boundary is
 * the pair of Triton launches `diff_attn_fwd[grid](...)` (src/kernel.py:476-503) and
 * `diff_attn_bwd[grid](...)` (src/kernel.py:531-570); the entry points below take the same
 * operands as plain device pointers and sizes.
 *
 * Conventions (all entry points):
 *   - every tensor is dense row-major fp16 ("half"; bfloat16 with DIFFATTN_BF16), [B,H,N,D] for q1,q2,k1,k2 and their
 *     gradients, [B,H,N,2D] for v, y, u2, dy, dv; row statistics are fp32 [B,H,N];
 *   - D is 32, 64 or 128; N is a multiple of 128;
 *   - lambda_scale is a DEVICE pointer to one fp16 value (the reference loads it in-kernel,
 *     src/kernel.py:138), or to H values with DIFFATTN_LAMBDA_PER_HEAD; fp32 values with DIFFATTN_LAMBDA_FP32;
 *   - `stream` is a hipStream_t passed as void*; work is only enqueued on it.  No entry point
 *     allocates, frees, synchronises or keeps global state; all are re-entrant;
 *   - return value: 0 on success, a negative DIFFATTN_E* code for rejected arguments, or a
 *     positive hipError_t value if a launch failed.
 */
#ifndef DIFFATTN_H_
#define DIFFATTN_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DIFFATTN_OK 0
#define DIFFATTN_EINVAL_NULL (-1)   /* a required pointer is null */
#define DIFFATTN_EINVAL_DIM (-2)    /* D not in {32,64,128} or B,H,N not positive */
#define DIFFATTN_EINVAL_SEQ (-3)    /* N not a multiple of 128, or n_valid outside 1..N */
#define DIFFATTN_EINVAL_WS (-4)     /* workspace too small */
#define DIFFATTN_EINVAL_ALIGN (-5)  /* a pointer is not 16-byte aligned */
#define DIFFATTN_EINVAL_FLAGS (-6)  /* unknown bits in `flags` */
#define DIFFATTN_EINVAL_SCRATCH (-7) /* problem too large for diffattn_backward_static */
#define DIFFATTN_EINVAL_LAYOUT (-8)  /* a stride in diffattn_layout is negative, not a multiple of 8, a row stride is below the row width, or y overlaps itself */
#define DIFFATTN_EINVAL_DROPOUT (-9) /* dropout probability outside [0, 255/256] */

/* `flags` of the forward and backward entry points.  DIFFATTN_RMS_NORM is the reference's boolean
 * `rms_norm` (src/kernel.py:464): a caller that passes a C boolean there keeps working.
 * DIFFATTN_CAUSAL has no counterpart in the reference, which lists masking as missing
 * (src/kernel.py:4): query i sees keys 0..i only, in both softmax streams.  Forward and backward of
 * one problem must be given the same flags. */
#define DIFFATTN_RMS_NORM 1
#define DIFFATTN_CAUSAL 2
/* Every 16-bit tensor (q1..v, y, u2, dy, the gradients, *lambda_scale, *dlambda) is bfloat16 instead of
 * fp16.  No counterpart in the reference, whose kernel hard-codes fp16 (src/kernel.py:175-176). */
#define DIFFATTN_BF16 4
/* lambda_scale points to H values, one per head (head h of every batch entry uses lambda_scale[h]), and
 * the backward writes H values to dlambda, each summed over the batch.  No counterpart in the
 * reference, which has one lambda per call (src/kernel.py:138). */
#define DIFFATTN_LAMBDA_PER_HEAD 8
/* *lambda_scale is read and *dlambda is written as fp32, whatever the type of the tensors.  The reference
 * returns the lambda gradient in the tensors' fp16 (`dtype=V.dtype`, src/kernel.py:573), where it
 * saturates at 65504: under a gradient scaler's loss scale the sum over all rows reaches that quickly.
 * With this flag the fixed-order fp32 sum leaves the library unrounded. */
#define DIFFATTN_LAMBDA_FP32 16
/* The caller's tensors (q1, q2, k1, k2, v, y, dy and the gradients) hold n_valid rows per (batch, head)
 * unit instead of N: a dense one is [B,H,n_valid,C].  See diffattn_forward_padded.  Without the flag a
 * dense tensor is [B,H,N,C] (the caller has padded it); either way no row past n_valid-1 of those
 * tensors is read or written. */
#define DIFFATTN_UNPADDED 32

/*
 * Element strides of the caller's tensors, for the entry points that take a `layout`.  The
 * reference passes the strides of Q1 (shared by Q2, K1, K2) and of V to its kernels
 * (src/kernel.py:487-494, :552-559) and assumes O and dO dense; here y and dy have strides of
 * their own.  Each tensor is logically [B,H,N,C] with the last dimension contiguous; `_b`, `_h`,
 * `_n` are the distances in elements between batch entries, heads and rows.  Every stride must be
 * a non-negative multiple of 8 (rows start 16-byte aligned) and a row stride at least C; a
 * [B,N,H,C] buffer viewed as [B,H,N,C] is `{N*H*C, C, H*C}`.  A zero batch or head stride broadcasts an
 * input; a tensor that is written (y, the gradients) must not overlap itself (non-zero batch and head
 * strides when B, H > 1).  The gradients have strides of their own, so that they can be written in the
 * layout of the tensors they belong to (dq1, dq2, dk1, dk2 share one set, like q1..k2); all three zero
 * means dense.  What the library writes for itself (u2, the row statistics, the workspace) is dense
 * [B,H,N,.].  A NULL `layout` means every tensor is dense.
 */
typedef struct diffattn_layout {
  long long qk_b, qk_h, qk_n;   /* q1, q2, k1, k2  (C = D)  */
  long long v_b, v_h, v_n;      /* v               (C = 2D) */
  long long y_b, y_h, y_n;      /* y               (C = 2D) */
  /* backward only; the forward neither reads nor checks these */
  long long dy_b, dy_h, dy_n;       /* dy                  (C = 2D) */
  long long dqk_b, dqk_h, dqk_n;    /* dq1, dq2, dk1, dk2  (C = D); all zero: dense  */
  long long dv_b, dv_h, dv_n;       /* dv                  (C = 2D); all zero: dense */
} diffattn_layout;

/*
 * Dropout on the two softmax maps.  No counterpart in the reference, which lists dropout as
 * missing (src/kernel.py:4, README.md:2).  Each (query, key) pair of each softmax stream is
 * dropped independently with probability p before the product with v, and the kept probabilities
 * are scaled by 1/(1-p), as torch's scaled_dot_product_attention does for its single map:
 *     x = (drop(softmax(s q1 k1^T)) - lambda drop'(softmax(s q2 k2^T))) v.
 * The decisions are a pure function of (seed, stream, batch*head unit, query, key, N): forward and
 * backward of one problem must be given the same struct, and diffattn_dropout_mask writes the same
 * decisions out.  p is used in steps of 1/256 (rounded to the nearest; the scale uses the rounded
 * value); p = 0 or a NULL pointer means no dropout.
 */
typedef struct diffattn_dropout {
  float p;                      /* drop probability, 0 <= p <= 255/256 */
  unsigned long long seed;
} diffattn_dropout;

/* ABI version of this header; bumped when a signature changes. */
int diffattn_abi_version(void);

/* Human-readable text for a return code of this library (static storage). */
const char* diffattn_strerror(int code);

/*
 * Forward.  Replaces the launch of diff_attn_fwd (src/kernel.py:476-503).
 *   y    [B,H,N,2D]  out: (softmax(s q1 k1^T) - lambda softmax(s q2 k2^T)) v, then, iff DIFFATTN_RMS_NORM,
 *                    (1 - lambda_init) * rmsnorm(.) with eps 1e-5 (src/kernel.py:188-198)
 *   u2   [B,H,N,2D]  out, optional (may be NULL when no backward follows): softmax(s q2 k2^T) v
 *   lse1, lse2 [B,H,N] fp32 out, optional: natural-log row logsumexp of the scaled scores
 *                    (the reference's M1/M2, src/kernel.py:188-189,203-204)
 *   rinv [B,H,N] fp32 out, optional, written only with DIFFATTN_RMS_NORM: rsqrt(mean(x^2) + 1e-5)
 * The reference additionally stores both per-stream outputs O1,O2 (src/kernel.py:205-206); here
 * the backward rebuilds the pre-norm row from y and rinv, so only u2 is kept.
 */
int diffattn_forward(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                     const void* lambda_scale, void* y, void* u2, float* lse1, float* lse2, float* rinv,
                     int B, int H, int N, int D, float sm_scale, float lambda_init, int flags,
                     void* stream);

/*
 * Forward for a sequence whose real length n_valid is not a multiple of 128.  No counterpart in the
 * reference, whose kernels require such a multiple and have no boundary checks (src/kernel.py:4,
 * :136-150, :527).  N is n_valid rounded up to a multiple of 128: the kernels work on N rows, u2, lse1,
 * lse2 and rinv have N rows per unit, and so has the backward's workspace.  Of q1, q2, k1, k2, v and y only
 * rows 0..n_valid-1 are touched: reads past them are redirected to the last real row inside the kernels,
 * keys n_valid..N-1 are ignored, and y gets no rows past n_valid-1.  So the caller's tensors need only
 * n_valid rows (say so with DIFFATTN_UNPADDED, or pass their strides in `layout`); tensors padded to N rows
 * by the caller work as well.  The matching backward is diffattn_backward_stages with the same N, n_valid
 * and flags.  diffattn_forward is this function with n_valid = N.  `layout` gives the strides of q1, q2,
 * k1, k2, v and y (NULL: all dense); `dropout` switches dropout on (NULL: none).
 */
int diffattn_forward_padded(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                            const void* lambda_scale, void* y, void* u2, float* lse1, float* lse2, float* rinv,
                            int B, int H, int N, int n_valid, int D, float sm_scale, float lambda_init, int flags,
                            const diffattn_layout* layout, const diffattn_dropout* dropout, void* stream);

/* Bytes of device workspace diffattn_backward needs for this problem size and these flags (0 on bad
 * sizes or unknown flag bits).  Counterpart of the scratch tensors the reference's backward
 * allocates itself (src/kernel.py:520-529). */
size_t diffattn_backward_workspace_bytes(int B, int H, int N, int D, int flags);

/*
 * Backward.  Replaces the launch of diff_attn_bwd (src/kernel.py:531-570) and the host-side
 * reduction of the lambda gradient (src/kernel.py:573).
 *   inputs : q1,q2,k1,k2,v,lambda_scale as in forward; y,u2,lse1,lse2,rinv as written by forward
 *            (rinv is ignored without DIFFATTN_RMS_NORM); dy [B,H,N,2D] upstream gradient, dense.
 *   outputs: dq1,dq2,dk1,dk2 [B,H,N,D], dv [B,H,N,2D] fp16; dlambda: one fp16 value (H values
 *            with DIFFATTN_LAMBDA_PER_HEAD; fp32 with DIFFATTN_LAMBDA_FP32), DEVICE memory, written
 *            (not accumulated), reduced in a fixed order: bit-reproducible.
 *   workspace: device memory of at least diffattn_backward_workspace_bytes(B,H,N,D,flags) bytes,
 *            256-byte aligned, contents undefined before and after.
 */
int diffattn_backward(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                      const void* lambda_scale, const void* y, const void* u2,
                      const float* lse1, const float* lse2, const float* rinv, const void* dy,
                      void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
                      void* workspace, size_t workspace_bytes,
                      int B, int H, int N, int D, float sm_scale, float lambda_init, int flags,
                      void* stream);

/*
 * Backward, restricted to some of its stream-ordered stages.  No counterpart in the reference
 * (whose backward is one fused launch); it exists so that a benchmark can time each kernel of
 * the backward with events on `stream`.  Stage bits, in execution order:
 *   DIFFATTN_STAGE_PREP    row preprocess: dX, row statistics, d(lambda) partials -> workspace
 *   DIFFATTN_STAGE_DLAMBDA fixed-order reduction of the partials -> dlambda
 *                          (a launch of its own only when neither DKDV nor DQ is asked for: otherwise it
 *                          rides in the first of their launches as one extra workgroup per lambda)
 *   DIFFATTN_STAGE_DKDV    dK1, dK2, dV   (reads the workspace written by PREP)
 *   DIFFATTN_STAGE_DQ      dQ1, dQ2       (reads the workspace written by PREP)
 * diffattn_backward(...) == diffattn_backward_stages(..., DIFFATTN_STAGE_ALL, stream).
 * The outputs of a stage that is not requested may be NULL: a caller that needs, say, only dQ1 and
 * dQ2 passes PREP | DQ and NULL for dk1, dk2, dv and dlambda.
 * n_valid (1..N) is the real sequence length of a problem that went through
 * diffattn_forward_padded (N when there is no padding): keys n_valid..N-1 are ignored, rows
 * n_valid..N-1 of q1, q2, k1, k2, v, y and dy are not read and those of the gradients not written.
 * `layout` gives the strides of q1, q2, k1, k2, v, y, dy and of the gradients (NULL: all dense).
 * `dropout` must be what the forward was given.
 */
#define DIFFATTN_STAGE_PREP 1u
#define DIFFATTN_STAGE_DLAMBDA 2u
#define DIFFATTN_STAGE_DKDV 4u
#define DIFFATTN_STAGE_DQ 8u
#define DIFFATTN_STAGE_ALL 15u
int diffattn_backward_stages(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                             const void* lambda_scale, const void* y, const void* u2,
                             const float* lse1, const float* lse2, const float* rinv, const void* dy,
                             void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
                             void* workspace, size_t workspace_bytes,
                             int B, int H, int N, int n_valid, int D, float sm_scale, float lambda_init, int flags,
                             unsigned stage_mask, const diffattn_layout* layout, const diffattn_dropout* dropout,
                             void* stream);

/*
 * Writes the keep decisions of `dropout` for softmax stream 0 or 1 of a [B,H,N,N] problem as bytes
 * (1 kept, 0 dropped) to `keep` (device memory, B*H*N*N bytes).  N is the padded length the
 * kernels are called with.  No counterpart in the reference; it lets a test hand the very masks
 * the kernels use to a reference implementation.
 */
int diffattn_dropout_mask(unsigned char* keep, int B, int H, int N, int softmax_stream, const diffattn_dropout* dropout,
                          void* stream);

/*
 * Backward without a workspace argument and without any allocation.  No counterpart in the
 * reference; it is for callers that cannot allocate device memory around the call: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same operands and results
 * as diffattn_backward (bit for bit); the workspace is a fixed array of
 * DIFFATTN_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process
 * ends.  Problems whose diffattn_backward_workspace_bytes exceed it are rejected with
 * DIFFATTN_EINVAL_SCRATCH (at D = 64 the limit is about 120 000 rows B*H*N).  The device the
 * stream belongs to must be current.  All calls on one GPU share the array: two calls that
 * overlap in time on the same GPU (different streams or threads) race; calls on one stream are
 * ordered and safe.
 */
#define DIFFATTN_STATIC_SCRATCH_BYTES (32u << 20)
int diffattn_backward_static(const void* q1, const void* q2, const void* k1, const void* k2, const void* v,
                             const void* lambda_scale, const void* y, const void* u2,
                             const float* lse1, const float* lse2, const float* rinv, const void* dy,
                             void* dq1, void* dq2, void* dk1, void* dk2, void* dv, void* dlambda,
                             int B, int H, int N, int D, float sm_scale, float lambda_init, int flags,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DIFFATTN_H_ */
