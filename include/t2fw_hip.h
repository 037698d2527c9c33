/*
 * t2fw_hip.h -- C ABI of libt2fw_hip.so: MI355X (gfx950) kernels for the
 * decaying-fast-weight ("LFW") and delta-rule ("DFW") recurrences.
 *
 * This is the boundary a binding of the reference's op layer would call instead of
 * its CUDA launchers.  Plain pointers and sizes only; no torch types.
 *
 *   reference interface replaced                         entry point here
 *   ---------------------------------------------------  -------------------------
 *   lfw_forward   (t2fw/csrc/lfw.cpp:28-48) =
 *     lfw_cuda_forward (t2fw/csrc/lfw_kernel.cu:124-171)
 *     + output einsum (lfw.cpp:45)                       t2fw_lfw_forward
 *   lfw_backward  (t2fw/csrc/lfw.cpp:50-96) =
 *     lfw_cuda_backward (lfw_kernel.cu:173-228)
 *     + six einsums (lfw.cpp:84-93)                      t2fw_lfw_backward
 *   the same with the caller's head-folding copies
 *     (layout required by lfw.cpp:24-26) absorbed        t2fw_lfw_forward_heads, t2fw_lfw_backward_heads
 *   T=1 use of lfw_forward in generation
 *     (tests/benchmark.py:86-88,104-105)                 t2fw_lfw_step
 *   dfw lfw_forward  (t2fw/csrc/dfw.cpp:27-39,
 *     dfw_kernel.cu:406-470)                             t2fw_dfw_forward
 *   dfw lfw_backward (t2fw/csrc/dfw.cpp:41-64,
 *     dfw_kernel.cu:472-558)                             t2fw_dfw_backward
 *
 * Conventions
 *   - All tensors are dense, row-major, device memory of ONE dtype (dtype code below):
 *       x, f, out, g_out, d_x, d_f           [B, T, D]
 *       q, k, f_key, d_q, d_k, d_f_key       [B, T, K]
 *       s0, next_state, g_state, d_s0        [B, D, K]
 *       ckpt                                 [B, NC, D, K],  NC = t2fw_lfw_num_ckpt(T, C)
 *   - ckpt[b, c] is the state at the START of chunk c (time steps [c*C, (c+1)*C)), so
 *     ckpt[b, 0] == s0[b].  It replaces the reference's [B, T, D, K] "ckpt_states"
 *     (lfw_kernel.cu:140-144), which stores every step.
 *   - The library owns no memory and keeps no state between calls.  Scratch space is
 *     passed by the caller (`workspace`, size from the *_workspace_bytes query, 16-byte
 *     aligned, no initialisation needed; may be NULL when the query returns 0).
 *   - `stream` is a hipStream_t (NULL = the null stream).  Launches are asynchronous;
 *     the current HIP device must be the one that owns the pointers.
 *   - Every function returns 0 on success, otherwise one of T2FW_ERR_* ; a message for
 *     the calling thread's last failure is available from t2fw_last_error().
 *   - Sizes are 64-bit; B or T may be 0 (no work, next_state = s0).
 */
#ifndef T2FW_HIP_H
#define T2FW_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define T2FW_ABI_VERSION 3

/* dtype codes (reference dispatch: AT_DISPATCH_FLOATING_TYPES_AND_HALF,
 * lfw_kernel.cu:157 -> fp64/fp32/fp16; bf16 is added here) */
#define T2FW_F32 0
#define T2FW_F16 1
#define T2FW_BF16 2
#define T2FW_F64 3

/* error codes */
#define T2FW_OK 0
#define T2FW_ERR_NULL_POINTER 1
#define T2FW_ERR_BAD_DTYPE 2
#define T2FW_ERR_BAD_SHAPE 3
#define T2FW_ERR_MISALIGNED 4
#define T2FW_ERR_UNSUPPORTED 5
#define T2FW_ERR_WORKSPACE 6
#define T2FW_ERR_HIP 7

/* kernel-path selection for the `flags` argument */
#define T2FW_FLAG_AUTO 0        /* fastest path that supports the shape/dtype      */
#define T2FW_FLAG_FORCE_SCAN 1  /* exact per-step scan kernels only (any shape)     */
#define T2FW_FLAG_FP16_OPERANDS 2 /* fp16 tensors: fp16 (not bf16) matrix-core operands;
                                     more mantissa, but rows whose 16-step gate products
                                     fall below 2^-8 take the exact scan path          */
#define T2FW_FLAG_NO_FIXUP 4      /* matrix-core path: do not redo what it flagged (the forward redoes it
                                     with the exact recurrence inside its kernel; the backward with one
                                     more launch of the block-wise kernel, which in turn redoes exactly
                                     what it cannot take); the caller reads the flags
                                     from the workspace (nonzero = that row's results are not
                                     valid; t2fw_lfw_flag_regions says where they are) and redoes
                                     those rows with T2FW_FLAG_FORCE_SCAN, or knows its gates are in
                                     range: a forward call whose hints (below) are all zero proves
                                     that for the backward call on the same gates.  Saves the
                                     backward's extra launch.                                     */

#define T2FW_FLAG_BLOCKWISE 8     /* matrix-core path, backward: the block-wise kernel (16-step blocks in one
                                     pass per batch row; takes 16-step gate products down to 2^-100)
                                     instead of the chunk-parallel ones (every chunk of every row at once;
                                     gate products over half a chunk down to 2^-80)                  */

#define T2FW_FLAG_BF16_OPERANDS 16 /* delta rule, matrix-core path: single bf16 operands (2^-9 per operand;
                                     results within 1e-2 of max|ref| like the LFW kernels') instead of
                                     operands split into bf16 head + remainder (fp32-level results before
                                     they are rounded to the tensors' type, three matrix-core products per
                                     product): for callers that train in reduced precision anyway.  With
                                     bf16 tensors it costs next to nothing in accuracy (what is stored is
                                     rounded to bf16 either way).  Off unless passed.                 */

int t2fw_abi_version(void);
const char *t2fw_last_error(void);

/* Number of checkpoints per batch row: ceil(T / C), at least 1. */
int64_t t2fw_lfw_num_ckpt(int64_t T, int32_t C);

/* Bytes of caller-provided scratch that serve both the forward and the backward call of a
 * shape (0 = none): row flags, and for the chunk-parallel backward kernels per chunk its flag,
 * six [64] fp32 gate-product vectors and the adjoint entering it, [B, NC, 64, 64] bf16. */
size_t t2fw_lfw_workspace_bytes(int64_t B, int64_t T, int64_t D, int64_t K,
                                int32_t C, int32_t dtype, int32_t flags);
/* The same for a caller that only runs the forward call. */
size_t t2fw_lfw_forward_workspace_bytes(int64_t B, int64_t T, int64_t D, int64_t K,
                                        int32_t C, int32_t dtype, int32_t flags);

/*
 * Where the calls of a shape leave their per-row flags in the workspace: three regions of int32,
 * written to regions[0..5] as (byte offset from the start of the workspace, number of entries):
 *   [0],[1]  forward verdicts: nonzero = the matrix-core form could not take the row (it has been redone
 *            exactly unless T2FW_FLAG_NO_FIXUP was given);
 *   [2],[3]  forward hints for the backward call on the same gates: all zero = the chunk-parallel
 *            backward will flag no row, so that call may be given T2FW_FLAG_NO_FIXUP; many nonzero =
 *            most rows would be declined and redone, and T2FW_FLAG_BLOCKWISE is the faster path
 *            (a gate outside [0, 1] or a 16-step gate product below 2^-40 sets a row's hint);
 *   [4],[5]  backward verdicts, as [0],[1].
 * A region a path does not write has zero entries (exact kernels: all three).  The workspace may be
 * any memory the GPU can write, pinned host memory included: a caller that wants to steer the
 * backward call from the host gives the forward call a pinned workspace and reads the hints once
 * the forward call has completed.  No counterpart in the reference, which has one path.
 */
int t2fw_lfw_flag_regions(int64_t B, int64_t T, int64_t D, int64_t K,
                          int32_t C, int32_t dtype, int32_t flags, int64_t *regions);

/* The address under which the current GPU sees a pinned host allocation (hipHostMalloc), for a caller
 * that keeps a workspace there; fails with T2FW_ERR_HIP for memory the GPU cannot reach. */
int t2fw_host_workspace_device_pointer(void *host_workspace, void **device_pointer);

/*
 * Forward scan.  S_t = S_{t-1} * (f_t (x) f_key_t) + x_t (x) k_t ;  out_t = S_t q_t ;
 * next_state = S_{T-1}.  Replaces lfw_forward (lfw.cpp:28-48).
 * ckpt may be NULL (inference: no checkpoints are written); otherwise C >= 1.
 */
int t2fw_lfw_forward(const void *x, const void *f, const void *q, const void *k,
                     const void *f_key, const void *s0,
                     void *out, void *next_state, void *ckpt,
                     int64_t B, int64_t T, int64_t D, int64_t K,
                     int32_t C, int32_t dtype, int32_t flags,
                     void *workspace, size_t workspace_bytes, void *stream);

/*
 * The forward scan for callers that cannot allocate device memory or pass a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose launcher allocates on every call, lfw_kernel.cu:140).
 * Same arguments and results as t2fw_lfw_forward, minus the workspace: the scratch lives in a
 * buffer of T2FW_STATIC_SCRATCH_BYTES bytes built into the library (one copy per GPU, held until
 * the process ends).  The call allocates and frees nothing.  A shape whose scratch
 * (t2fw_lfw_workspace_bytes) exceeds the buffer is rejected with T2FW_ERR_WORKSPACE.  All calls
 * on one GPU share the buffer: calls that overlap in time on one GPU (different streams or
 * threads) race on it; calls on one stream do not.
 * The first call on a GPU looks up the buffer's address, which may load the library's code onto that
 * GPU: make that call, or t2fw_static_init() with the GPU current, before a stream capture begins.
 */
#define T2FW_STATIC_SCRATCH_BYTES (1 << 20)
/* Looks up the built-in buffer of the current GPU (once per GPU; later calls return at once). */
int t2fw_static_init(void);
int t2fw_lfw_forward_static(const void *x, const void *f, const void *q, const void *k,
                            const void *f_key, const void *s0,
                            void *out, void *next_state, void *ckpt,
                            int64_t B, int64_t T, int64_t D, int64_t K,
                            int32_t C, int32_t dtype, int32_t flags, void *stream);

/*
 * Backward pass: recomputes the states inside each chunk from ckpt, runs the
 * reverse-time adjoint scan and writes all six gradients.  Replaces lfw_backward
 * (lfw.cpp:50-96); gradient order as returned there (lfw.cpp:95).
 */
int t2fw_lfw_backward(const void *g_out, const void *g_state,
                      const void *x, const void *f, const void *q, const void *k,
                      const void *f_key, const void *s0, const void *ckpt,
                      void *d_x, void *d_f, void *d_q, void *d_k, void *d_f_key,
                      void *d_s0,
                      int64_t B, int64_t T, int64_t D, int64_t K,
                      int32_t C, int32_t dtype, int32_t flags,
                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same two calls for tensors that keep the head axis next to the channels, as the
 * projections of an attention-shaped layer produce them:
 *       x, f, out, g_out, d_x, d_f           [B, T, H, D]
 *       q, k, f_key, d_q, d_k, d_f_key       [B, T, H, K]
 *       s0, next_state, g_state, d_s0        [B, H, D, K]
 *       ckpt                                 [B * H, ceil(T / C), D, K]
 * Every (batch, head) pair is one recurrence.  The reference takes only the folded,
 * contiguous [B * H, T, D] layout (checks in t2fw/csrc/lfw.cpp:24-26), which costs its
 * caller a transposing copy per input and per gradient; here the kernels step over the
 * head axis themselves.  H = 1 is the folded layout.  The workspace is that of B * H rows
 * (t2fw_lfw_workspace_bytes(B * H, ...)).  The matrix-core kernels need T * H < 2^24.
 */
int t2fw_lfw_forward_heads(const void *x, const void *f, const void *q, const void *k,
                           const void *f_key, const void *s0,
                           void *out, void *next_state, void *ckpt,
                           int64_t B, int64_t T, int64_t H, int64_t D, int64_t K,
                           int32_t C, int32_t dtype, int32_t flags,
                           void *workspace, size_t workspace_bytes, void *stream);

int t2fw_lfw_backward_heads(const void *g_out, const void *g_state,
                            const void *x, const void *f, const void *q, const void *k,
                            const void *f_key, const void *s0, const void *ckpt,
                            void *d_x, void *d_f, void *d_q, void *d_k, void *d_f_key,
                            void *d_s0,
                            int64_t B, int64_t T, int64_t H, int64_t D, int64_t K,
                            int32_t C, int32_t dtype, int32_t flags,
                            void *workspace, size_t workspace_bytes, void *stream);

/*
 * One generation step (T = 1) that may update the state in place
 * (next_state == s0 is allowed).  x,f,out [B,D]; q,k,f_key [B,K].
 */
int t2fw_lfw_step(const void *x, const void *f, const void *q, const void *k,
                  const void *f_key, const void *s0, void *out, void *next_state,
                  int64_t B, int64_t D, int64_t K, int32_t dtype, void *stream);

/*
 * Delta rule.  out_t = S_{t-1} q_t ; delta_t = v_t - S_{t-1} k_t ;
 * S_t = S_{t-1} + delta_t (x) k_t.   q,k,d_q,d_k [B,T,M]; v,out,delta,g_out,d_v [B,T,D];
 * s0,final_state,g_state,d_s0 [B,D,M].  Replaces dfw.cpp:27-39 / :41-64.
 * D = M = 64 with fp32, fp16 or bf16 tensors and 16-byte aligned pointers runs on the matrix cores in blocks of
 * 16 steps (flags: T2FW_FLAG_BF16_OPERANDS above); everything else, or T2FW_FLAG_FORCE_SCAN, the exact
 * per-step kernels.
 */
int t2fw_dfw_forward(const void *q, const void *k, const void *v, const void *s0,
                     void *out, void *final_state, void *delta,
                     int64_t B, int64_t T, int64_t D, int64_t M,
                     int32_t dtype, int32_t flags, void *stream);

int t2fw_dfw_backward(const void *g_out, const void *g_state,
                      const void *q, const void *k, const void *delta,
                      const void *final_state,
                      void *d_q, void *d_k, void *d_v, void *d_s0,
                      int64_t B, int64_t T, int64_t D, int64_t M,
                      int32_t dtype, int32_t flags, void *stream);

/*
 * Conversion of `count` (<= 8) arrays of n[i] elements each between float32 and float16 / bfloat16 in one
 * launch (src_dtype -> dst_dtype, one of them T2FW_F32); arrays 16-byte aligned, `src`, `dst`, `n` host arrays.
 * No counterpart in the reference (one kernel serves every dtype there, lfw_kernel.cu:157-168): it is what a
 * caller with float32 tensors uses to run the 16-bit matrix-core kernels (lfw_apply_16bit of the Python side).
 */
int t2fw_cast(const void *const *src, void *const *dst, const int64_t *n, int32_t count,
              int32_t src_dtype, int32_t dst_dtype, void *stream);

/*
 * Sigmoid gating of both forget gates in one launch: f = sigmoid(f_logit) [n_f elements],
 * f_key = sigmoid(fk_logit) [n_fk elements]; outputs may alias the inputs.  The reference leaves
 * the non-linearity to the caller (functional_lfw.py:25-30); dtype f32 / f16 / bf16.
 */
int t2fw_gate_forward(const void *f_logit, const void *fk_logit, void *f, void *f_key,
                      int64_t n_f, int64_t n_fk, int32_t dtype, void *stream);

/* d_logit = d_gate * gate * (1 - gate) for both gates; outputs may alias d_f / d_f_key. */
int t2fw_gate_backward(const void *d_f, const void *d_f_key, const void *f, const void *f_key,
                       void *d_f_logit, void *d_fk_logit,
                       int64_t n_f, int64_t n_fk, int32_t dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* T2FW_HIP_H */
