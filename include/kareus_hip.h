/*
 * C ABI of libkareus_hip.so — hand-written gfx950 (MI355X) kernels for one GPU's shard of
 * a Llama-style decoder layer.  This is the boundary a drop-in replacement of the
 * reference's native calls binds to: every entry point below names the native call of the
 * reference it stands in for.
 *
 * Conventions (all entry points)
 *   - Pointers are raw device addresses; bf16 data is 2-byte brain-float, fp32 where stated.
 *   - Leading dimensions and strides are in ELEMENTS.  Rows must start 16-byte aligned.
 *   - The caller allocates every output and every workspace; the library never allocates
 *     or frees device memory, keeps no mutable global state and never synchronises the
 *     device.  Calls on different streams may be issued concurrently from different threads.
 *   - `stream` is a hipStream_t (NULL = the default stream).
 *   - Return value: KR_OK (0) or a negative KR_E* code.  Nothing is launched on error.
 */
#ifndef KAREUS_HIP_H
#define KAREUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KR_OK 0
#define KR_EINVAL (-1)       /* null pointer, non-positive size, misaligned pointer or stride */
#define KR_EUNSUPPORTED (-2) /* shape outside what the kernels are built for */
#define KR_ELAUNCH (-3)      /* the HIP runtime rejected the launch */

/* Library version, major*10000 + minor*100 + patch. */
int kr_version(void);
/* Static text for a return code. */
const char* kr_error_string(int code);
/* Rated shader clock of the current device in MHz (0 if it cannot be read): the label a profiling
 * sweep gives its rows when it leaves the clock alone.  The reference labels rows with the clock it
 * locks through NVML (tests/bayesian/common/hardware.py:52-59, :107-114). */
int kr_device_clock_mhz(void);

/* ---- GEMM ------------------------------------------------------------------------------
 * bf16 x bf16 -> fp32 accumulate -> bf16.  Replaces tex.generic_gemm (cuBLASLt) as called
 * by kareus/transformer_engine/pytorch/ops/basic/basic_linear.py:
 *   KR_GEMM_TN  :571-582  y  = x . W^T     A = x  [M,K] row-major, B = W  [N,K] row-major
 *   KR_GEMM_NN  :847-859  dx = dy . W      A = dy [M,K] row-major, B = W  [K,N] row-major
 *   KR_GEMM_NT  :898-909  dW = dy^T . x    A = dy [K,M] row-major, B = x  [K,N] row-major
 * C is [M,N] row-major.  M, N, K, lda, ldb, ldc must be multiples of 8.
 * accumulate != 0 adds the product to the existing contents of C (rounded once).
 * workspace may be NULL.  If it holds at least kr_gemm_workspace_bytes() bytes, shapes whose
 * output has too few tiles to occupy the GPU (weight gradients) are computed split-K through
 * fp32 partial tiles kept there; otherwise one workgroup walks the whole contraction.       */
#define KR_GEMM_TN 0
#define KR_GEMM_NN 1
#define KR_GEMM_NT 2
size_t kr_gemm_workspace_bytes(int layout, int M, int N, int K);
/* Workspace for a GEMM that shares the GPU with kernels of other streams.  The split count of
 * kr_gemm_workspace_bytes() minimises the GEMM's own latency; with latency_weight < 1 the choice
 * leans towards the smallest total CU-time instead, which never asks for more splits.  A launch
 * flagged KR_GEMM_BESIDE_OTHER_STREAMS is planned with weight 0.1: size its workspace with that
 * value, so that the cuts the dispatcher plans are the cuts the buffer holds.  kr_gemm_bf16 uses
 * as many splits as the workspace it is handed holds, at most the planned count.              */
size_t kr_gemm_workspace_bytes_shared(int layout, int M, int N, int K, float latency_weight);
int kr_gemm_bf16(int layout, int M, int N, int K,
                 const void* A, int64_t lda, const void* B, int64_t ldb,
                 void* C, int64_t ldc, int accumulate,
                 void* workspace, size_t workspace_bytes, void* stream);

/* The same GEMM with an operation fused into its epilogue and an optional compute-unit budget.
 * epilogue:
 *   KR_GEMM_EPI_NONE    plain kr_gemm_bf16.
 *   KR_GEMM_EPI_ADD     C = bf16(bf16(A.B) + aux), aux [M,N] bf16 with row stride ld_aux: the residual
 *                       add behind a row-parallel projection (fused_bias_dropout_add_forward with p = 0,
 *                       no bias, kareus/megatron/core/extensions/ops/bias_dropout_add.py:15-32) done where
 *                       the projection's output is produced (te_linear.py:188-206 writes that output
 *                       straight into its consumer's buffer); bit-identical to kr_gemm_bf16 + kr_add.
 *   KR_GEMM_EPI_SWIGLU  N = 2F, F a multiple of 80, 96, 112 or 128: C = x [M, 2F] as usual and
 *                       out2 [M, F] (row stride ld_out2) = silu(x[:, :F]) * x[:, F:] computed from the
 *                       bf16-rounded x (fused_swiglu_forward, bias_swiglu.py:14-20); bit-identical to
 *                       kr_gemm_bf16 + kr_swiglu_fwd.
 *   KR_GEMM_EPI_SWIGLU_BWD  layout NN (an input gradient, N = F): the product g = A.B [M, F] is the gradient
 *                       of the SwiGLU activation's output and is not stored; aux = x [M, 2F] (row stride ld_aux)
 *                       is the activation's input and C = dx [M, 2F] (ldc >= 2F) receives
 *                       fused_swiglu_backward(bf16(g), x) (bias_swiglu.py:34-44); bit-identical to
 *                       kr_gemm_bf16 + kr_swiglu_bwd.
 *   ADD and SWIGLU need layout TN, SWIGLU_BWD layout NN; all need accumulate == 0 and are never split-K.
 *   KR_GEMM_BESIDE_OTHER_STREAMS  a flag, or-ed to any of the above: kernels of other streams are
 *                       there to use the compute units this launch leaves idle, so an output with few
 *                       tiles keeps its wide tiles and is cut little or not at all (least compute-unit
 *                       time) instead of being spread over the device for the shortest latency; pass
 *                       the workspace kr_gemm_workspace_bytes_shared sizes.  Results do not depend on it
 *                       beyond the rounding of a cut's fp32 partial sums.
 * max_cus > 0 limits the launch to that many compute units (workgroups are persistent, one per
 * unit): the compute-unit share a schedule's resource_shape gives a partition
 * (kareus/megatron/core/partitions/partition_base.py:117-128); 0 = the whole device.             */
#define KR_GEMM_EPI_NONE 0
#define KR_GEMM_EPI_ADD 1
#define KR_GEMM_EPI_SWIGLU 2
#define KR_GEMM_EPI_SWIGLU_BWD 4
#define KR_GEMM_BESIDE_OTHER_STREAMS 0x100
int kr_gemm_bf16_fused(int layout, int M, int N, int K,
                       const void* A, int64_t lda, const void* B, int64_t ldb,
                       void* C, int64_t ldc, int accumulate,
                       int epilogue, const void* aux, int64_t ld_aux, void* out2, int64_t ld_out2,
                       int max_cus, void* workspace, size_t workspace_bytes, void* stream);

/* Row runs.  A nanobatch of r sequences cut out of a [seq, batch, hidden] tensor along the batch axis
 * (kareus/megatron/core/transformer/transformer_block.py:483-485) is not a matrix with one row
 * stride: its rows come in runs of r consecutive rows (stride hidden) whose starts are batch*hidden
 * elements apart.  The reference copies such a slice into a dense tensor in every linear layer
 * (kareus/transformer_engine/pytorch/ops/basic/basic_linear.py:565-569).  The *_runs entry points
 * address it in place: row i of an operand with `run_rows` rows per run and run starts `run_ld`
 * elements apart sits at (i / run_rows) * run_ld + (i % run_rows) * ld.  run_rows: a power of two that
 * divides the operand's row count, 1 for a plain matrix (run_ld is then ignored); run_ld: a multiple
 * of 8.
 * kr_gemm_bf16_runs = kr_gemm_bf16_fused with runs for A, C and aux, run_rows at most 16, for the
 * launches at the two ends of a layer stack: layout TN with the residual-add epilogue (aux and / or C
 * in runs: the block's input as residual, the block's output as destination), layout NN plain or with
 * the SwiGLU-backward epilogue and layout NT (A in runs: the block's incoming gradient; for NT the rows
 * of A are the contraction index).  An output in runs is never accumulated into or cut along K.
 * Anything else in runs returns KR_EUNSUPPORTED.                                                   */
int kr_gemm_bf16_runs(int layout, int M, int N, int K,
                      const void* A, int64_t lda, int a_run_rows, int64_t a_run_ld,
                      const void* B, int64_t ldb,
                      void* C, int64_t ldc, int c_run_rows, int64_t c_run_ld, int accumulate,
                      int epilogue, const void* aux, int64_t ld_aux, int aux_run_rows, int64_t aux_run_ld,
                      void* out2, int64_t ld_out2,
                      int max_cus, void* workspace, size_t workspace_bytes, void* stream);

/* The weight gradient of a linear layer over all nanobatches of a microbatch in one launch.  The
 * reference computes dW = dy^T . x once per nanobatch and sums the products in main_grad
 * (accumulate_into_grad_weight, kareus/transformer_engine/pytorch/ops/basic/basic_linear_bias.py:229-263,
 * GEMM call basic_linear.py:898-909): n launches whose contraction is a nanobatch's tokens, each with a
 * read-modify-write of the whole gradient.  The sum over nanobatches is the same contraction continued,
 * so this entry point takes the n operand pairs where they lie and runs one GEMM over all their tokens:
 *   C[M, N] (+)= sum_i A_i^T . B_i,  A_i [k_seg, M] (row stride lda), B_i [k_seg, N] (row stride ldb)
 * for i < nseg <= KR_GEMM_MAX_SEGMENTS; the pieces may be anywhere in memory (16-byte aligned), k_seg must
 * be a multiple of 64 (KR_EUNSUPPORTED otherwise: the caller then accumulates pair by pair).  Tiling,
 * cuts of the contraction, workspace and `max_cus` as for layout NT of kr_gemm_bf16_fused on
 * K = nseg * k_seg (size the workspace with that K); flags: 0 or KR_GEMM_BESIDE_OTHER_STREAMS.
 * The pieces of A may be in row runs, every piece alike (a_run_rows, a_run_ld as for kr_gemm_bf16_runs;
 * 1 = plain matrices): the incoming gradient of a layer stack, cut into nanobatches of several sequences.
 * The fp32 sum runs over the pieces in the order given and is rounded to bf16 once.                  */
#define KR_GEMM_MAX_SEGMENTS 8
int kr_gemm_bf16_nt_segments(int M, int N, int k_seg, int nseg,
                             const void* const* A, int64_t lda, int a_run_rows, int64_t a_run_ld,
                             const void* const* B, int64_t ldb,
                             void* C, int64_t ldc, int accumulate, int flags,
                             int max_cus, void* workspace, size_t workspace_bytes, void* stream);

/* ---- RMSNorm ---------------------------------------------------------------------------
 * Replaces transformer_engine_torch.rmsnorm_fwd / rmsnorm_bwd
 * (kareus/transformer_engine/pytorch/ops/basic/rmsnorm.py:210-219, 256-263).
 * x, dy: [rows, cols] bf16 with row strides x_ld, dy_ld (elements, multiples of 8, >= cols; a
 * nanobatch that is one sequence of a [seq, batch, hidden] tensor is such a matrix and needs no
 * copy); y, dx: [rows, cols] bf16 contiguous; gamma, dgamma: [cols] bf16; rstd: [rows] fp32.
 * cols must be a multiple of 8 and at most 8192.
 * fwd: rstd = rsqrt(mean(x^2) + eps), y = (x * rstd) * gamma.
 * bwd: dx = rstd * (g - xhat * mean(g * xhat)), g = gamma * dy, xhat = x * rstd;
 *      dgamma = sum over rows of dy * xhat.  workspace: kr_rmsnorm_bwd_workspace_bytes().  */
int kr_rmsnorm_fwd(const void* x, const void* gamma, void* y, float* rstd,
                   int rows, int cols, int64_t x_ld, float eps, void* stream);
/* kr_rmsnorm_fwd on an input whose rows come in runs (see "Row runs" above; same call of the
 * reference, rmsnorm.py:210-219, fed a nanobatch of several sequences without the copy).        */
int kr_rmsnorm_fwd_runs(const void* x, const void* gamma, void* y, float* rstd,
                        int rows, int cols, int64_t x_ld, int x_run_rows, int64_t x_run_ld,
                        float eps, void* stream);
size_t kr_rmsnorm_bwd_workspace_bytes(int rows, int cols);
int kr_rmsnorm_bwd(const void* dy, const void* x, const float* rstd, const void* gamma,
                   void* dx, void* dgamma, void* workspace, int rows, int cols,
                   int64_t dy_ld, int64_t x_ld, void* stream);
/* RMSNorm backward followed by the backward of the residual fork in front of the norm
 * (rmsnorm.py:256-263 then kareus/megatron/core/extensions/ops/residual_fork.py:104-106) in one
 * pass: dx = bf16(dx_norm) + dres, bit-identical to kr_rmsnorm_bwd followed by kr_add.  dres:
 * [rows, cols] bf16 with row stride dres_ld, or NULL for the plain backward; dx may be a slice of
 * a larger tensor (row stride dx_ld).  */
int kr_rmsnorm_bwd_add(const void* dy, const void* x, const float* rstd, const void* gamma,
                       const void* dres, void* dx, void* dgamma, void* workspace, int rows, int cols,
                       int64_t dy_ld, int64_t x_ld, int64_t dres_ld, int64_t dx_ld, void* stream);
/* kr_rmsnorm_bwd_add where the saved input x, the residual gradient dres and / or the result dx are
 * nanobatches of several sequences used in place (rows in runs, see "Row runs" above;
 * rmsnorm.py:256-263 and residual_fork.py:104-106 without the copies in and out).               */
int kr_rmsnorm_bwd_add_runs(const void* dy, const void* x, const float* rstd, const void* gamma,
                            const void* dres, void* dx, void* dgamma, void* workspace,
                            int rows, int cols, int64_t dy_ld,
                            int64_t x_ld, int x_run_rows, int64_t x_run_ld,
                            int64_t dres_ld, int dres_run_rows, int64_t dres_run_ld,
                            int64_t dx_ld, int dx_run_rows, int64_t dx_run_ld, void* stream);

/* Weight gradient of one RMSNorm over several nanobatches of a microbatch, summed in fp32 and
 * rounded once (the reference lets autograd add the per-nanobatch bf16 gradients,
 * kareus/megatron/core/partitions/autograd_function.py:346-372): call kr_rmsnorm_bwd_add with
 * dgamma == NULL for every nanobatch — it then only leaves its kr_rmsnorm_bwd_partial_rows(rows, cols)
 * fp32 partial rows of `cols` columns at `workspace` — with the nanobatches' workspaces back to back in
 * one buffer, then kr_rmsnorm_dgamma over all `nparts` rows of that buffer.                     */
int kr_rmsnorm_bwd_partial_rows(int rows, int cols);
int kr_rmsnorm_dgamma(const float* partial, int nparts, int cols, void* dgamma, void* stream);

/* kr_rmsnorm_bwd_add without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The fp32 partial rows of the weight gradient go to a 16 MiB array
 * that the library holds in device memory on every GPU it runs on until the process ends; the
 * call itself allocates and frees nothing (its first call on a device looks the array's address
 * up, so make one call per device before a region in which even that is unwelcome).
 * cols above 8192 return KR_EUNSUPPORTED; dgamma == NULL returns KR_EINVAL (the partial rows stay
 * in an array no caller can read, so the reduced gradient must have a destination).  Results are
 * bit-identical to kr_rmsnorm_bwd_add.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (different streams
 * or threads) race on it and must be ordered by the caller.                                     */
int kr_rmsnorm_bwd_add_noalloc(const void* dy, const void* x, const float* rstd, const void* gamma,
                               const void* dres, void* dx, void* dgamma, int rows, int cols,
                               int64_t dy_ld, int64_t x_ld, int64_t dres_ld, int64_t dx_ld,
                               void* stream);

/* ---- Query / key layernorm of the QKV split -----------------------------------------------
 * RMSNorm over the head dimension of every query head (weights gamma_q [hd]) and every key head
 * (gamma_k [hd]) of a fused QKV projection output: replaces the q_layernorm / k_layernorm calls of
 * QKVPostProcessOp (kareus/megatron/core/extensions/ops/qkv_postprocess.py:110-118 forward,
 * :147-160 backward; each is an RMSNorm as in kareus/transformer_engine/pytorch/ops/basic/
 * rmsnorm.py:165-273 with the head dimension as its width).
 * mixed, out, dmixed: [tokens, ng, per + 2, hd] bf16, dense: per query heads, one key head and one
 * value head per group.  rstd: [tokens, ng, per + 1] fp32, 1 / rms of every normalised head.
 * kr_qk_norm_fwd: out = the buffer with its query and key heads normalised (y = bf16(x * rstd *
 *   gamma)) and its value heads copied, so that out is again a fused buffer.  out must not alias
 *   mixed (the backward needs the input; out == mixed returns KR_EINVAL).
 * kr_qk_norm_bwd: rewrites the query and key heads of dmixed (the gradient w.r.t. out) in place
 *   with the gradient w.r.t. mixed, dx = rstd * (dy*gamma - xhat * mean(dy*gamma*xhat)), leaves the
 *   value heads alone, and writes dgamma_q, dgamma_k [hd] bf16 (sums of dy * xhat over all heads of
 *   the kind, in fp32, in a fixed order).  workspace: kr_qk_norm_bwd_workspace_bytes() bytes of
 *   device memory, 16-byte aligned.
 * hd must be 64, 128 or 256 (KR_EUNSUPPORTED otherwise; the workspace query then returns 0).     */
size_t kr_qk_norm_bwd_workspace_bytes(int64_t tokens, int ng, int per, int hd);
int kr_qk_norm_fwd(const void* mixed, const void* gamma_q, const void* gamma_k, void* out, float* rstd,
                   int64_t tokens, int ng, int per, int hd, float eps, void* stream);
int kr_qk_norm_bwd(void* dmixed, const void* mixed, const float* rstd, const void* gamma_q,
                   const void* gamma_k, void* dgamma_q, void* dgamma_k, void* workspace,
                   int64_t tokens, int ng, int per, int hd, void* stream);

/* ---- Rotary position embedding ---------------------------------------------------------
 * Replaces fused_rotary_positional_embedding.forward / backward (Apex), called from
 * kareus/apex/transformer/functional/fused_rope.py:27-35, 41-46.
 * t, out: [s, b, heads, hd] bf16 addressed as s*stride_s + b*stride_b + head*stride_h + d
 * (hd contiguous; strides multiples of 8).  freqs: [s, hd] fp32 angles; all hd channels are
 * rotated, halves layout: out = t*cos(f) + rotate_half(t)*sin(f), rotate_half([a,b]) = [-b,a].
 * backward != 0 rotates by -f (the gradient of the forward).  out may alias t.
 * Heads are taken in groups of group_size; only the first group_rotate heads of each group are
 * rotated, the others are copied (or left alone when out aliases t).  (1, 1) rotates every
 * head; (nq/nkv + 2, nq/nkv + 1) rotates the query and key heads of a fused QKV projection
 * output in place and leaves its value heads untouched.
 * hd must be a multiple of 16 and at most 256.                                             */
int kr_rope(const void* t, void* out, const float* freqs,
            int s, int b, int heads, int hd,
            int64_t t_stride_s, int64_t t_stride_b, int64_t t_stride_h,
            int64_t o_stride_s, int64_t o_stride_b, int64_t o_stride_h,
            int backward, int group_size, int group_rotate, void* stream);

/* ---- SwiGLU ----------------------------------------------------------------------------
 * Replaces the Inductor kernels of fused_swiglu_forward / fused_swiglu_backward
 * (kareus/megatron/core/extensions/ops/bias_swiglu.py:14-20, 34-44).
 * x, dx: [rows, 2*F] bf16; y, dy: [rows, F] bf16; all contiguous; F a multiple of 8.
 * y = silu(x[:, :F]) * x[:, F:].                                                           */
int kr_swiglu_fwd(const void* x, void* y, int64_t rows, int F, void* stream);
int kr_swiglu_bwd(const void* dy, const void* x, void* dx, int64_t rows, int F, void* stream);

/* ---- Residual add ----------------------------------------------------------------------
 * out = a + b over n bf16 elements (fp32 add, one rounding).  Replaces the Inductor kernel
 * of fused_bias_dropout_add_forward with p = 0 and no bias
 * (kareus/megatron/core/extensions/ops/bias_dropout_add.py:15-32) and the gradient sum of
 * ResidualForkOp (kareus/megatron/core/extensions/ops/residual_fork.py:104-106).
 * out may alias a or b.                                                                    */
int kr_add(const void* a, const void* b, void* out, int64_t n, void* stream);
/* The same sum over [rows, cols] matrices with row strides lda, ldb, ldo (elements, multiples of
 * 8, >= cols; cols a multiple of 8): lets the residual stream stay a strided nanobatch slice.   */
int kr_add_rows(const void* a, int64_t lda, const void* b, int64_t ldb, void* out, int64_t ldo,
                int64_t rows, int cols, void* stream);

/* ---- Hidden dropout in front of the residual add ---------------------------------------
 * out = residual + dropout(x) with probability p in [0, 1): replaces the Inductor kernels of
 * fused_bias_dropout_add_forward / _backward without bias
 * (kareus/megatron/core/extensions/ops/bias_dropout_add.py:15-45: native_dropout, then the add;
 * native_dropout_backward(grad, mask, 1 / (1 - p))).
 * kr_dropout_add: mask [rows, cols] bytes, dense (1 = kept), written for the backward;
 *   out = bf16(residual + bf16(x * mask / (1 - p))) — the product is rounded before the add, as the
 *   reference's is.  The mask comes from Philox-4x32-10 keyed by `seed`, counter `offset` + the
 *   index of the 8-element vector: the same (seed, offset) gives the same mask whatever the launch,
 *   and a caller that advances `offset` by rows * cols / 8 per call never reuses a counter.  It is
 *   not the mask PyTorch would draw from the same seed.
 * kr_dropout_bwd: dx = bf16(dy * mask * scale).
 * Matrices [rows, cols] with row strides in elements (multiples of 8, >= cols; cols a multiple of
 * 8), so that a strided nanobatch slice is used where it lies.  out may alias residual.        */
int kr_dropout_add(const void* x, int64_t ldx, const void* residual, int64_t ldr, void* out, int64_t ldo,
                   void* mask, int64_t rows, int cols, float p, uint64_t seed, uint64_t offset,
                   void* stream);
int kr_dropout_bwd(const void* dy, int64_t lddy, const void* mask, void* dx, int64_t lddx, int64_t rows,
                   int cols, float scale, void* stream);

/* ---- Causal grouped-query attention ----------------------------------------------------
 * Replaces flash_attn_2_cuda.fwd / bwd as called from
 * kareus/flash_attn/flash_attn_interface.py:66-80, 174-194.
 * bf16 tensors, head dimension contiguous.  Key-like tensors (k, v, dk, dv), nkv heads:
 *   element (si, bi, kvh, d) at si*stride_s + bi*stride_b + kvh*stride_h + d.
 * Query-like tensors (q, o, dout, dq), nq heads in nkv groups of per = nq/nkv:
 *   element (si, bi, h, d) at si*stride_s + bi*stride_b + (h/per)*stride_g + (h%per)*stride_h + d.
 * A dense [s, b, nq, hd] tensor has stride_g = per*stride_h; the grouped form lets the kernels
 * read q, k, v straight out of the fused QKV projection output, whose features are laid out
 * per KV group as (its query heads, its key head, its value head)
 * (kareus/megatron/core/extensions/ops/qkv_postprocess.py:84-109), and write dq, dk, dv
 * straight into a buffer of that layout.
 * lse: [b, nq, s] fp32 contiguous (natural log-sum-exp of the scaled, masked scores).
 * Query head h reads KV head h/per.  Causal, query i sees keys <= i.
 * hd: a multiple of 8, at most 128; any s.  Head dimension 128 with s a multiple of 128 (the
 * training workloads) runs on the MFMA kernels as it lies.  Every other shape is padded into them
 * through the workspace (zero channels up to 128, zero rows up to the next multiple of 128: the
 * causal mask keeps the added keys from every real query, and the added queries are given a
 * log-sum-exp that makes them inert in the backward pass): kr_attn_bwd always, the forward when it
 * is called as kr_attn_fwd_ws with a workspace.  Without one (kr_attn_fwd, kr_attn_fwd_flags), or
 * with KR_ATTN_GENERAL_KERNELS in the flags word, such a shape runs on general fp32 kernels that
 * are correct and slow.  All strides multiples of 8.
 * kr_attn_bwd needs a workspace of kr_attn_bwd_workspace_bytes() bytes (16-byte aligned).   */
int kr_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                int s, int b, int nq, int nkv, int hd, float scale,
                int64_t q_stride_s, int64_t q_stride_b, int64_t q_stride_g, int64_t q_stride_h,
                int64_t k_stride_s, int64_t k_stride_b, int64_t k_stride_h,
                int64_t v_stride_s, int64_t v_stride_b, int64_t v_stride_h,
                int64_t o_stride_s, int64_t o_stride_b, int64_t o_stride_g, int64_t o_stride_h,
                void* stream);
/* The same call with a flags word (0 = kr_attn_fwd).  KR_ATTN_BESIDE_OTHER_STREAMS: kernels of other
 * streams run beside this launch and use the compute units it leaves idle (the engine's nanobatch
 * streams), so the launch is shaped for the least compute-unit time rather than for its own latency:
 * whole rows / whole key tiles per workgroup whatever their number, no second pass and no merge.
 * The two shapes sum in different orders: results agree to rounding, and for a given flags word they
 * do not depend on the batch size.  No counterpart in the reference's call
 * (kareus/flash_attn/flash_attn_interface.py:66-80 runs one kernel at a time).                   */
#define KR_ATTN_BESIDE_OTHER_STREAMS 0x100
#define KR_ATTN_GENERAL_KERNELS 0x200
int kr_attn_fwd_flags(const void* q, const void* k, const void* v, void* o, float* lse,
                      int s, int b, int nq, int nkv, int hd, float scale,
                      int64_t q_stride_s, int64_t q_stride_b, int64_t q_stride_g, int64_t q_stride_h,
                      int64_t k_stride_s, int64_t k_stride_b, int64_t k_stride_h,
                      int64_t v_stride_s, int64_t v_stride_b, int64_t v_stride_h,
                      int64_t o_stride_s, int64_t o_stride_b, int64_t o_stride_g, int64_t o_stride_h,
                      int flags, void* stream);
/* kr_attn_fwd_flags with a workspace of kr_attn_fwd_workspace_bytes() bytes (0 for a shape the MFMA
 * kernels take as it lies; workspace may then be NULL; a workspace that is too small for a shape that
 * needs one is KR_EINVAL, none at all selects the general kernels): the call the reference's
 * flash_attn_gpu.fwd (kareus/flash_attn/flash_attn_interface.py:66-80) maps to for any head
 * dimension and sequence length it accepts.                                                      */
size_t kr_attn_fwd_workspace_bytes(int s, int b, int nq, int nkv, int hd);
int kr_attn_fwd_ws(const void* q, const void* k, const void* v, void* o, float* lse,
                   int s, int b, int nq, int nkv, int hd, float scale,
                   int64_t q_stride_s, int64_t q_stride_b, int64_t q_stride_g, int64_t q_stride_h,
                   int64_t k_stride_s, int64_t k_stride_b, int64_t k_stride_h,
                   int64_t v_stride_s, int64_t v_stride_b, int64_t v_stride_h,
                   int64_t o_stride_s, int64_t o_stride_b, int64_t o_stride_g, int64_t o_stride_h,
                   int flags, void* workspace, size_t workspace_bytes, void* stream);
size_t kr_attn_bwd_workspace_bytes(int s, int b, int nq, int nkv, int hd);
int kr_attn_bwd(const void* dout, const void* q, const void* k, const void* v,
                const void* o, const float* lse,
                void* dq, void* dk, void* dv, void* workspace,
                int s, int b, int nq, int nkv, int hd, float scale,
                int64_t q_stride_s, int64_t q_stride_b, int64_t q_stride_g, int64_t q_stride_h,
                int64_t k_stride_s, int64_t k_stride_b, int64_t k_stride_h,
                int64_t v_stride_s, int64_t v_stride_b, int64_t v_stride_h,
                int64_t o_stride_s, int64_t o_stride_b, int64_t o_stride_g, int64_t o_stride_h,
                int64_t do_stride_s, int64_t do_stride_b, int64_t do_stride_g, int64_t do_stride_h,
                int64_t dq_stride_s, int64_t dq_stride_b, int64_t dq_stride_g, int64_t dq_stride_h,
                int64_t dk_stride_s, int64_t dk_stride_b, int64_t dk_stride_h,
                int64_t dv_stride_s, int64_t dv_stride_b, int64_t dv_stride_h,
                void* stream);
/* kr_attn_bwd with the flags word of kr_attn_fwd_flags (same workspace size).
 * Replaces the same call, kareus/flash_attn/flash_attn_interface.py:174-194.                       */
int kr_attn_bwd_flags(const void* dout, const void* q, const void* k, const void* v,
                      const void* o, const float* lse,
                      void* dq, void* dk, void* dv, void* workspace,
                      int s, int b, int nq, int nkv, int hd, float scale,
                      int64_t q_stride_s, int64_t q_stride_b, int64_t q_stride_g, int64_t q_stride_h,
                      int64_t k_stride_s, int64_t k_stride_b, int64_t k_stride_h,
                      int64_t v_stride_s, int64_t v_stride_b, int64_t v_stride_h,
                      int64_t o_stride_s, int64_t o_stride_b, int64_t o_stride_g, int64_t o_stride_h,
                      int64_t do_stride_s, int64_t do_stride_b, int64_t do_stride_g, int64_t do_stride_h,
                      int64_t dq_stride_s, int64_t dq_stride_b, int64_t dq_stride_g, int64_t dq_stride_h,
                      int64_t dk_stride_s, int64_t dk_stride_b, int64_t dk_stride_h,
                      int64_t dv_stride_s, int64_t dv_stride_b, int64_t dv_stride_h,
                      int flags, void* stream);

/* ---- Ends of the layer stack: embedding and loss ------------------------------------------
 * Token embedding of one vocabulary shard.  Replaces F.embedding / weight[masked_input] and the
 * [b s h] -> [s b h] transpose of
 * 3rdparty/Megatron-LM/megatron/core/tensor_parallel/layers.py:245-263 and
 * 3rdparty/Megatron-LM/megatron/core/models/common/embeddings/language_model_embedding.py:106-116.
 * ids: [b, s] int64 token ids; weight, dweight: [vocab_rows, hidden] bf16, the shard holding ids
 * vocab_start .. vocab_start + vocab_rows - 1; out, dout: [s, b, hidden] bf16 contiguous.
 * fwd: out[si, bi, :] = weight[ids[bi, si] - vocab_start, :], zeros for ids of other shards.
 * bwd: dweight[r, :] = sum of dout over the tokens whose id is vocab_start + r, zeros for rows
 *      without a token; every row is written, sums are taken in one fixed order (no atomics on the result, the
 *      result is reproducible).  hidden: multiple of 8 (bwd: at most 8192, s*b below 2^26).                    */
int kr_embedding_fwd(const int64_t* ids, const void* weight, void* out, int s, int b, int hidden,
                     int64_t vocab_start, int64_t vocab_rows, void* stream);
int kr_embedding_bwd(const int64_t* ids, const void* dout, void* dweight, int s, int b, int hidden,
                     int64_t vocab_start, int64_t vocab_rows, void* stream);

/* Cross entropy over rows of logits.  Replaces vocab_parallel_cross_entropy /
 * te_parallel_cross_entropy as called from
 * 3rdparty/Megatron-LM/megatron/core/models/common/language_module/language_module.py:71-101 for
 * a vocabulary held by one shard.
 * logits: [rows, vocab] bf16 with row stride ld; labels: [rows] int64; loss, lse, dloss: [rows] fp32.
 * fwd: lse = log sum_j exp(logits[j]), loss = lse - logits[label]; a label outside [0, vocab)
 *      marks an ignored row (loss 0).
 * bwd: dlogits[j] = (exp(logits[j] - lse) - [j == label]) * dloss, zeros for ignored rows;
 *      dlogits ([rows, vocab] bf16, row stride ld_out) may be the logits buffer itself.
 * vocab, ld, ld_out: multiples of 8.                                                           */
int kr_cross_entropy_fwd(const void* logits, const int64_t* labels, float* loss, float* lse,
                         int64_t rows, int vocab, int64_t ld, void* stream);
int kr_cross_entropy_bwd(const void* logits, const int64_t* labels, const float* lse,
                         const float* dloss, void* dlogits, int64_t rows, int vocab, int64_t ld,
                         int64_t ld_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KAREUS_HIP_H */
