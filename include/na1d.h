/*
 * libna1d — 1-D neighbourhood attention (NA1D) for AMD MI355X (gfx950).
 *
 * C ABI of the shared library.  Every entry point takes raw device pointers,
 * 64-bit sizes, a dtype tag and the HIP stream to launch on; it allocates
 * nothing and returns an int status (NA1D_OK or a negative NA1D_ERR_* code)
 * instead of asserting.  The compute entry points are re-entrant and keep no
 * state between calls, with three stated exceptions at the end of this file:
 * the profiling hook (a per-thread pair of events), the kernel-family switch
 * (one process-wide flag) and na1d_fused_backward_noalloc (a per-GPU scratch
 * array).  All tensors are dense and contiguous:
 *
 *   q, k, v, out, d*  : [B, T, C]  16-bit (bf16 or fp16 by `dtype`), C fastest,
 *                       B = batch * heads (batch major, head minor)
 *   attn, dattn       : [B, T, W]  fp32, slot j of query t addresses key t-left+j
 *   keys outside [0,T) contribute exactly 0 (zero filled, never clamped/shifted)
 *
 * Limits: C % 8 == 0, 1 <= W <= 80, 0 <= left < W, B,T >= 1 (B == 0 or T == 0 is
 * a no-op that returns NA1D_OK).  Pointers must be 16-byte aligned.
 *
 * The six un-fused entry points replace, one for one, the pybind functions of
 * the reference extension (na1d_tensorcore/bf16_ana1d.cpp:8-104 and its fp16
 * twin; the same six appear as torch.ops.na_cuda.* in
 * pcf_nat_pytorch2.7.zip!/extension_na/na_cuda/csrc_tc240_or_bigger/main.cpp:27-41).
 */
#ifndef NA1D_H
#define NA1D_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NA1D_BF16 0
#define NA1D_FP16 1

#define NA1D_OK               0
#define NA1D_ERR_NULL        -1   /* a required pointer is NULL                      */
#define NA1D_ERR_DTYPE       -2   /* dtype is neither NA1D_BF16 nor NA1D_FP16         */
#define NA1D_ERR_HEAD_DIM    -3   /* C <= 0 or C % 8 != 0                             */
#define NA1D_ERR_WINDOW      -4   /* W < 1, W > 80, left < 0 or left >= W             */
#define NA1D_ERR_SHAPE       -5   /* negative B or T, B % H != 0, size overflow       */
#define NA1D_ERR_ALIGN       -6   /* a tensor pointer is not 16-byte aligned          */
#define NA1D_ERR_LAUNCH      -7   /* the HIP runtime rejected the launch              */
#define NA1D_ERR_UNSUPPORTED -8   /* valid arguments that no built kernel covers      */
#define NA1D_ERR_TOO_LARGE   -9   /* the problem needs more than the static scratch   */
#define NA1D_ERR_WORKSPACE   -10  /* a workspace was passed that is too small         */
#define NA1D_ERR_SCALE       -11  /* scale is not a finite number above zero          */

#define NA1D_MAX_WINDOW 80

/* Library version (major*10000 + minor*100 + patch) and message for a status. */
int         na1d_version(void);
const char *na1d_status_string(int status);

/* P1 — band QK^T:  attn[b,t,j] = sum_c q[b,t,c] * k~[b,t-left+j,c].
 * Replaces torch_ana_qk_forward (bf16_ana1d.cpp:8-27; kernels
 * bf16_ana1d_kernel.cu:42-282). */
int na1d_qk_forward(void *attn, const void *q, const void *k,
                    int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
                    int dtype, void *stream);

/* P2 — band times V:  out[b,t,c] = sum_j attn[b,t,j] * v~[b,t-left+j,c], fp32
 * accumulate, round-to-nearest-even store.  Replaces torch_ana_av_forward
 * (bf16_ana1d.cpp:57-69; kernel bf16_ana1d_kernel.cu:285-391). */
int na1d_av_forward(void *out, const void *attn, const void *v,
                    int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
                    int dtype, void *stream);

/* dQ = P2(dattn, k).  Replaces torch_ana_q_backward (bf16_ana1d.cpp:29-41); the
 * reference serves it with the same kernel as av_forward and so does this. */
int na1d_q_backward(void *dq, const void *dattn, const void *k,
                    int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
                    int dtype, void *stream);

/* P3 — inverse-neighbourhood gather, no atomics:
 *   dk[b,u,c] = sum_j dattn[b,u+left-j,j] * q[b,u+left-j,c]   (rows outside [0,T) dropped).
 * Replaces torch_ana_k_backward (bf16_ana1d.cpp:43-55; kernel
 * bf16_ana1d_kernel.cu:394-492). */
int na1d_k_backward(void *dk, const void *dattn, const void *q,
                    int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
                    int dtype, void *stream);

/* dattn = P1(dout, v).  Replaces torch_ana_a_backward (bf16_ana1d.cpp:71-90). */
int na1d_a_backward(void *dattn, const void *dout, const void *v,
                    int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
                    int dtype, void *stream);

/* dV = P3(attn, dout).  Replaces torch_ana_v_backward (bf16_ana1d.cpp:92-104). */
int na1d_v_backward(void *dv, const void *attn, const void *dout,
                    int64_t B, int64_t T, int64_t C, int64_t W, int64_t left,
                    int dtype, void *stream);

/*
 * Fused forward: QK^T -> (* scale) -> + rpb[h] -> + mask -> softmax -> . V, the
 * [B,T,W] tensor never touching memory.  Replaces the sequence
 * QK_Function -> +bias -> +mask -> softmax -> AV_Function of
 * models/PCF_NATransformer.py:141-150 (mask of :87-99).
 *
 *   rpb      : fp32 [H, W] or NULL (no bias); head of row b is b % H
 *   t_valid  : int32 [B / H] or NULL; valid length of each sample (T - padding).
 *              A slot gets the additive -100 of the reference when its query
 *              row t >= t_valid or its key lies outside [0, t_valid).
 *   scale    : multiplies the fp32 scores (pass 1.0f when q is pre-scaled, as
 *              the reference model does); finite and > 0 (the reference's is
 *              head_dim^-0.5), otherwise NA1D_ERR_SCALE
 *   lse      : fp32 [B, T] out, log-sum-exp of each row's logits (for backward);
 *              may be NULL for inference
 */
int na1d_fused_forward(void *out, float *lse,
                       const void *q, const void *k, const void *v,
                       const float *rpb, const int32_t *t_valid,
                       int64_t B, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                       float scale, int dtype, void *stream);

/*
 * Fused backward of the above.  Recomputes the probabilities from q, k, lse;
 * replaces AV_Function.backward -> softmax backward -> QK_Function.backward
 * (nattn.py:46-54,69-78).  dq is the gradient w.r.t. the q that was passed in
 * (it already includes `scale`).
 *
 *   drpb : fp32 [H, W], ACCUMULATED into (caller zeroes it), or NULL to skip
 *   workspace, workspace_bytes : optional device scratch for the d rpb reduction.
 *          With at least na1d_fused_backward_workspace_bytes(...) bytes the per-
 *          workgroup partial sums go there and a second small kernel folds them in a
 *          fixed order; with NULL they are added with float atomics (slower under
 *          contention, order not reproducible).  A non-NULL workspace of too few bytes
 *          is refused with NA1D_ERR_WORKSPACE rather than ignored.  Contents need no
 *          initialisation and are not meaningful afterwards.
 */
int na1d_fused_backward(void *dq, void *dk, void *dv, float *drpb,
                        const void *q, const void *k, const void *v,
                        const void *out, const void *dout, const float *lse,
                        const float *rpb, const int32_t *t_valid,
                        int64_t B, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                        float scale, int dtype, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * The same two operators on strided tensors.  They have no counterpart among the
 * reference's six native functions: they replace, together with the fused operator,
 * the head split / merge copies around it (models/PCF_NATransformer.py:126-139,
 * 151-152; models/MFA_NATransformer.py:127-138,150-151) by reading q, k, v straight
 * out of the qkv projection's output and writing `out` straight into the layout the
 * output projection reads.
 *
 *   N, H        : samples and heads (the packed entry points' B is N * H)
 *   qkv_strides : int64[3] = {sample, head, row} strides, in elements, shared by q, k, v
 *                 (and dq, dk, dv); element (n, h, t, c) of q is q[n*sample + h*head +
 *                 t*row + c].  E.g. for a projection output [N, T, 3, H, C]:
 *                 q = base, k = base + H*C, v = base + 2*H*C, strides {T*3*H*C, C, 3*H*C}.
 *   out_strides : the same for out (and dout); [N, T, H*C] is {T*H*C, C, H*C}.
 *   lse         : fp32 [N*H, T], packed
 * Strides must be multiples of 8 elements and row >= C; the caller guarantees that
 * distinct (n, h, t) rows do not overlap.  Returns NA1D_ERR_UNSUPPORTED when no
 * matrix-core kernel covers the shape (C > 128): the caller then packs the tensors
 * and uses the packed entry points.  The backward needs no `out`.
 */
int na1d_fused_forward_strided(void *out, float *lse,
                               const void *q, const void *k, const void *v,
                               const float *rpb, const int32_t *t_valid,
                               int64_t N, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                               float scale, int dtype,
                               const int64_t *qkv_strides, const int64_t *out_strides, void *stream);

int na1d_fused_backward_strided(void *dq, void *dk, void *dv, float *drpb,
                                const void *q, const void *k, const void *v,
                                const void *dout, const float *lse,
                                const float *rpb, const int32_t *t_valid,
                                int64_t N, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                                float scale, int dtype,
                                const int64_t *qkv_strides, const int64_t *out_strides,
                                void *workspace, int64_t workspace_bytes, void *stream);

/*
 * The fused operator with attention dropout: replaces nn.Dropout(attn_drop) between the softmax and the second
 * contraction (models/PCF_NATransformer.py:71,149; every configuration of the reference sets attn_drop = 0, which is
 * what na1d_fused_forward / na1d_fused_backward compute).  Probability (b, t, j) - packed sequence b, query row t,
 * window slot j - is kept iff
 *     mix32(key ^ (j * 0x9E3779B9)) >= floor(p_drop * 2^32),
 *     key = mix32(mix32(lo32(row) ^ lo32(seed)) + hi32(row) * 0x9E3779B9 + hi32(seed)),   row = b * T + t,
 *     mix32(x): x ^= x >> 16; x *= 0x7feb352d; x ^= x >> 15; x *= 0x846ca68b; x ^= x >> 16   (32-bit arithmetic)
 * and kept probabilities are scaled by 1 / (1 - p_drop); lse is that of the un-dropped softmax.  The mask is a pure
 * function of (seed, b, t, j): the backward recomputes it from the same p_drop and seed, nothing is stored, and the
 * stream differs from torch's (whose mask depends on its launch geometry).  0 <= p_drop < 1.  Every head_dim the
 * plain entry points take is covered (above 128 by the generic kernels).  Dilated windows:
 * na1d_fused_forward_strided_dropout.  All other arguments as in na1d_fused_forward / na1d_fused_backward.
 */
int na1d_fused_forward_dropout(void *out, float *lse, const void *q, const void *k, const void *v, const float *rpb,
                               const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                               int64_t left, float scale, int dtype, float p_drop, uint64_t seed, void *stream);
int na1d_fused_backward_dropout(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k, const void *v,
                                const void *out, const void *dout, const float *lse, const float *rpb,
                                const int32_t *t_valid, int64_t B, int64_t H, int64_t T, int64_t C, int64_t W,
                                int64_t left, float scale, int dtype, float p_drop, uint64_t seed, void *workspace,
                                int64_t workspace_bytes, void *stream);

/*
 * Attention dropout on strided tensors.  The strided entry points also serve dilated windows: slot j of row t meets
 * row t + (j - left) * d, so the rows of one residue class t mod d form an undilated problem on every d-th row
 * (row stride d times the tensor's).  For the dropout mask of such a launch to be the one of the whole operator,
 * its rows are named by their place in the whole sequence: row t of sequence (n, h) of the launch stands for
 *     row = (n * H + h) * seq_rows + row_offset + row_stride * t
 * in the keep rule stated at na1d_fused_forward_dropout (row_stride = d, row_offset = the residue class, seq_rows =
 * the whole sequence's length; 1, 0, T for an undilated launch).  Replaces nn.Dropout(attn_drop) of the reference's
 * CPU branch, the only one that runs dilated windows (models/PCF_NATransformer.py:158-170).  Requires
 * 0 <= row_offset < row_stride and seq_rows >= row_offset + row_stride * (T - 1) + 1.  All other arguments as in
 * na1d_fused_forward_strided / na1d_fused_backward_strided; NA1D_ERR_UNSUPPORTED when no matrix-core kernel covers the
 * shape (head_dim > 128): there is no dropout on the generic path.
 */
int na1d_fused_forward_strided_dropout(void *out, float *lse, const void *q, const void *k, const void *v,
                                       const float *rpb, const int32_t *t_valid, int64_t N, int64_t H, int64_t T,
                                       int64_t C, int64_t W, int64_t left, float scale, int dtype,
                                       const int64_t *qkv_strides, const int64_t *out_strides, float p_drop,
                                       uint64_t seed, int64_t row_stride, int64_t row_offset, int64_t seq_rows,
                                       void *stream);
int na1d_fused_backward_strided_dropout(void *dq, void *dk, void *dv, float *drpb, const void *q, const void *k,
                                        const void *v, const void *dout, const float *lse, const float *rpb,
                                        const int32_t *t_valid, int64_t N, int64_t H, int64_t T, int64_t C, int64_t W,
                                        int64_t left, float scale, int dtype, const int64_t *qkv_strides,
                                        const int64_t *out_strides, float p_drop, uint64_t seed, int64_t row_stride,
                                        int64_t row_offset, int64_t seq_rows, void *workspace, int64_t workspace_bytes,
                                        void *stream);

/*
 * Dense ("global") attention over whole sequences, forward and backward: replaces the body of the reference's
 * GlobalAttention.forward between the head split and the head merge (models/PCF_NATransformer.py:199-221),
 *     attn = softmax((q * scale) @ k^T + mask);  out = attn @ v
 * with the mask of get_attn_mask_global (models/PCF_NATransformer.py:406-414) built on the fly from t_valid:
 * -100 is added where the query row or the key column is >= t_valid[sample] (NULL: nothing is padded).
 * q, k, v, out and the gradients are packed [B, T, C] with B = samples * H, head fastest inside a sample;
 * lse [B, T] fp32 (natural log; may be NULL in the forward when no backward follows).  The probabilities are never
 * written to memory.  The backward needs a workspace of na1d_global_backward_workspace_bytes() bytes (one fp32 per
 * row: rowsum(dout * out); sequences of up to 128 rows keep it on chip and leave the workspace untouched) and writes
 * every gradient exactly once, so it is deterministic.
 * C % 8 == 0; C > 128 returns NA1D_ERR_UNSUPPORTED.  scale: finite and > 0 as in na1d_fused_forward.  p_drop, seed: attention dropout (attn_drop of
 * models/PCF_NATransformer.py:193,218; 0 in the reference's configurations) by the keep rule stated at
 * na1d_fused_forward_dropout with the key's row index as the slot j; 0 <= p_drop < 1, 0 switches it off.
 */
int na1d_global_forward(void *out, float *lse, const void *q, const void *k, const void *v, const int32_t *t_valid,
                        int64_t B, int64_t H, int64_t T, int64_t C, float scale, int dtype, float p_drop, uint64_t seed,
                        void *stream);
int na1d_global_backward(void *dq, void *dk, void *dv, const void *q, const void *k, const void *v, const void *out,
                         const void *dout, const float *lse, const int32_t *t_valid, int64_t B, int64_t H, int64_t T,
                         int64_t C, float scale, int dtype, float p_drop, uint64_t seed, void *workspace,
                         int64_t workspace_bytes, void *stream);
int64_t na1d_global_backward_workspace_bytes(int64_t B, int64_t H, int64_t T, int64_t C, int dtype);

/*
 * Profiling hook; no counterpart in the reference.  From this call on, the matrix-core fused kernels that the
 * CALLING THREAD launches record `start` just before and `stop` just after the kernel itself (hipEvent_t handles,
 * recorded by hipExtLaunchKernel: the dispatch's own begin and end, i.e. what a profiler's kernel trace reports,
 * without the gaps between launches that events recorded on the stream include).  Each launch re-records the same
 * pair, so read them (hipEventElapsedTime) or change them between launches.  NULL, NULL switches it off.  With the
 * workspace path of the backward the pair brackets the main kernel, not the small reduction that follows.  While a
 * pair is set, a launch on a stream that is being captured into a graph is refused with NA1D_ERR_LAUNCH (nothing is
 * recorded into the graph).
 */
int na1d_profile_events(void *start, void *stop);
/* Name of the last matrix-core kernel that the calling thread launched while a pair of events was set, spelt as a
 * kernel trace prints it without namespaces and arguments, e.g. "fused_bwd_kernel<FP16, 32, 2, false>"; "" before the
 * first such launch.  The string lives in thread-local storage and is overwritten by the next such launch. */
const char *na1d_profile_last_kernel(void);

/*
 * Test hook; no counterpart in the reference.  The library holds two independent implementations of every
 * operator: the matrix-core kernels and slower generic kernels that also serve the shapes the former do not cover.
 * na1d_force_generic(1) routes every later call, from any thread, to the generic ones, na1d_force_generic(0) back;
 * the previous setting is returned.  The initial setting is 1 if the environment holds NA1D_FORCE_GENERIC=1 when
 * the library is first called, else 0.  The strided entry points, which only the matrix-core kernels serve,
 * return NA1D_ERR_UNSUPPORTED while it is on.
 */
int na1d_force_generic(int on);

/* Bytes of workspace na1d_fused_backward can use for these arguments (0 if it has
 * no use for one, negative status on invalid arguments). */
int64_t na1d_fused_backward_workspace_bytes(int64_t B, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                                            int dtype);

/*
 * na1d_fused_backward with a deterministic d rpb and no workspace argument.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory and cannot bring a workspace either: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The per-workgroup partial sums
 * of d rpb, which na1d_fused_backward puts into the caller's workspace, go into a scratch array of
 * NA1D_NOALLOC_SCRATCH_BYTES that is part of the library's device code (each GPU the library runs on holds its own
 * copy until the process ends); the same second kernel folds them in a fixed order.  The call allocates nothing
 * (no hipMalloc / hipFree, no allocating library routine).  Results are bit-identical to na1d_fused_backward given
 * a workspace of na1d_fused_backward_workspace_bytes() bytes.
 *
 * Limits: the shape must be one the workspace path covers (head_dim <= 128; otherwise NA1D_ERR_UNSUPPORTED), and na1d_fused_backward_workspace_bytes() for it must not exceed
 * NA1D_NOALLOC_SCRATCH_BYTES (32768 workgroups; 13107 with windows the wide kernels serve), otherwise NA1D_ERR_TOO_LARGE.  All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (different streams or threads) race on it; calls on one
 * stream are ordered and safe.  The array needs no clearing between calls: a call writes every entry it reads.
 * The device that owns `stream` must be the current device.  The first call on a device looks the array's address
 * up (hipGetSymbolAddress): make that call outside stream capture; later ones record nothing but their two kernels.
 * While na1d_force_generic(1) is on the call returns NA1D_ERR_UNSUPPORTED like the strided entry points (the generic
 * kernels have no fixed-order reduction).
 */
#define NA1D_NOALLOC_SCRATCH_BYTES (4 * 1024 * 1024)
int na1d_fused_backward_noalloc(void *dq, void *dk, void *dv, float *drpb,
                                const void *q, const void *k, const void *v,
                                const void *out, const void *dout, const float *lse,
                                const float *rpb, const int32_t *t_valid,
                                int64_t B, int64_t H, int64_t T, int64_t C, int64_t W, int64_t left,
                                float scale, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* NA1D_H */
