/*
 * librlk_hip -- C ABI of the MI355X (gfx950) fused linear-logprob path.
 *
 * Conventions shared by every entry point:
 *   - plain pointers and sizes only; every buffer is a caller-owned DEVICE pointer unless said
 *     otherwise; tensors are contiguous row-major;
 *   - work is enqueued on `stream` and the call returns without synchronising;
 *   - nothing is allocated or freed: scratch comes in through `workspace` (query its size with
 *     the matching *_workspace_bytes call);
 *   - return value 0 = enqueued, negative = RLK_ERR_* (nothing enqueued, message available from
 *     rlk_last_error());
 *   - results are deterministic: the grid and every reduction order are pure functions of the
 *     arguments, so repeated calls on the same input give the same bits.
 *
 * Each declaration cites the interface of the reference tree (RL-Align/RL-Kernel) it stands in
 * for; paths are relative to that tree.
 */
#ifndef RLK_HIP_H
#define RLK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* rlk_stream_t; /* == hipStream_t */

enum {
    RLK_DTYPE_BF16 = 0,
    RLK_DTYPE_F16 = 1,
    RLK_DTYPE_F32 = 2,
    RLK_DTYPE_F64 = 3
};

enum {
    RLK_OK = 0,
    RLK_ERR_ARG = -1,         /* bad pointer, size or scalar argument */
    RLK_ERR_UNSUPPORTED = -2, /* dtype / shape this entry point does not implement */
    RLK_ERR_LAUNCH = -3       /* HIP refused the launch */
};

/* ABI version of this header (major * 100 + minor): 101 (100 + rlk_device_info and
 * rlk_linear_logp_fwd_plan). */
int rlk_version(void);

/* Message of the last error returned on the calling thread ("" if none). Host pointer, valid
 * until the next failing call on the same thread. */
const char* rlk_last_error(void);

/* Compute units and maximum engine clock (kHz) of HIP device `device`, as the runtime reports
 * them: what a benchmark prices the matrix-core peak with (compute units x 4096 flop per clock x
 * clock for 16-bit inputs).  No counterpart in the reference.  Host pointers; launches nothing. */
int rlk_device_info(int32_t device, int32_t* compute_units, int32_t* max_clock_khz);

/* ------------------------------------------------------------------------------------------ *
 * Fused linear -> selected-token log-prob, forward.
 *
 * Stands in for `_C.fused_linear_logp_sm90(hidden, weight, target, bias) -> [logp, lse]`
 * (csrc/ops.cpp:84-85, csrc/cuda/fused_linear_logp_sm90.cu:305-381) and for the forward of
 * `NativeLinearLogpOp.apply` (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:476-520):
 *   z = (hidden W^T + bias) / temperature ; lse = logsumexp_v z ; logp = z[target] - lse.
 * The [N, V] logits are never stored.
 *
 *   hidden   [N, H] bf16/f16          weight [V, H] same dtype (a vocab shard starting at
 *   bias     [V] f32 or NULL                  global id `vocab_start`)
 *   targets  [N] int64 GLOBAL ids     logp, lse [N] f32 (lse in natural log)
 *   temperature > 0 (rl_engine/testing/reference_ops.py:15-47 semantics: divide before softmax)
 *   use_ignore != 0: rows whose target == ignore_index get logp = 0 exactly
 *            (rl_engine/testing/reference_ops.py:33-45; rl_engine/executors/deepspeed_trainer.py:559-569,639-641)
 *   strict_targets != 0: a non-ignored target outside [vocab_start, vocab_start + V) stores 1 to
 *            *err_flag (device int32, caller zeroes it; may be NULL when strict_targets == 0); the Python layer turns that into the
 *            reference's ValueError (rl_engine/kernels/ops/cuda/loss/linear_logp.py:352-358).
 *            With strict_targets == 0 such a row yields logp = -lse (z_t = 0), which is what a
 *            vocab-parallel shard must return (csrc/cuda/fused_linear_logp_sm90.cu:256-280).
 *   dtype: RLK_DTYPE_BF16 / RLK_DTYPE_F16 with H % 8 == 0 and 16-byte aligned matrices run on the
 *   16-bit MFMA tiles; RLK_DTYPE_F32, other H or misaligned matrices run on the fp32 matrix
 *   instruction (operands widened to fp32 on the way into LDS, same tiling, any N, H, V >= 1) --
 *   the counterpart of the reference's "unsupported dtype/shape falls back to the portable op"
 *   (rl_engine/kernels/ops/cuda/loss/linear_logp.py:45-55,350-351), except that here the
 *   portable op is a matrix-core HIP kernel too.  Every forward entry point below (static
 *   scratch, two heads, folded GRPO epilogue) and the backward take both kinds of input.
 * ------------------------------------------------------------------------------------------ */
int rlk_linear_logp_fwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                        size_t* bytes);

/* Schedule the forward will use for these sizes (the reference computes its own inside the host
 * function: 4 workgroups per SM divided by the token blocks, csrc/cuda/fused_linear_logp_sm90.cu:
 * 350-358,369, and does not expose it): out4 = { blocks of 256
 * tokens, vocab splits of the launch over the full vocab tiles, vocab splits of the launch over
 * the ragged last tile (all tiles for RLK_DTYPE_F32; 0 if there is no such launch), token blocks
 * per XCD patch }.  The contraction launches are blocks x splits workgroups.  Inputs whose rows
 * do not start on 16-byte boundaries run the RLK_DTYPE_F32 schedule.  Host only; touches no
 * device. */
int rlk_linear_logp_fwd_plan(int64_t N, int32_t H, int64_t V, int32_t dtype, int64_t* out4);

int rlk_linear_logp_fwd(const void* hidden, const void* weight, const float* bias,
                        const int64_t* targets, float* logp, float* lse, void* workspace,
                        size_t workspace_bytes, int64_t N, int32_t H, int64_t V,
                        int64_t vocab_start, int32_t dtype, float temperature,
                        int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                        int32_t* err_flag, rlk_stream_t stream);

/* Forward for callers that cannot allocate or pass a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, kernels and bits as rlk_linear_logp_fwd, but the per-split partial softmax
 * states live in a file-scope device array of RLK_STATIC_SCRATCH_BYTES inside the library (one
 * copy per GPU, held until the process ends) instead of `workspace`; the call allocates and frees
 * nothing.  Sizes whose partials (rlk_linear_logp_fwd_workspace_bytes) exceed that array are
 * rejected with RLK_ERR_ARG.  All calls on one GPU share the array: calls that overlap in time on
 * the same GPU (different streams or threads) race; serialise them.  Nothing in the array needs to
 * start at zero (every slot that is read was written by the same call). */
#define RLK_STATIC_SCRATCH_BYTES (8u << 20)

int rlk_linear_logp_fwd_static(const void* hidden, const void* weight, const float* bias,
                               const int64_t* targets, float* logp, float* lse, int64_t N,
                               int32_t H, int64_t V, int64_t vocab_start, int32_t dtype,
                               float temperature, int64_t ignore_index, int32_t use_ignore,
                               int32_t strict_targets, int32_t* err_flag, rlk_stream_t stream);

/* Policy head and frozen reference head over the same hidden states and targets in one launch:
 * logp / lse of `weight` and ref_logp / ref_lse of `ref_weight` ([V, H], same dtype), each equal
 * bit for bit to what rlk_linear_logp_fwd returns for that head alone.  A workgroup runs the vocab
 * tiles of the policy head and then the same tiles of the reference head through one pipeline
 * against its block of hidden states.  Stands in for the second lm_head pass that yields ref_logps
 * for the KL term (rl_engine/executors/deepspeed_trainer.py:146-167); the logits-fed counterpart
 * in the reference is the single program that scans both logit rows
 * (rl_engine/kernels/ops/triton/loss/ratio_kl.py:46-60).  Only the policy head is strict about
 * targets; both heads must have a bias or neither, and both weights must be 16-byte aligned or
 * neither (the two heads share one launch, hence one kind of kernel; a mixed pair is answered with
 * RLK_ERR_UNSUPPORTED rather than by moving the aligned head to the fp32 kernels).  Workspace:
 * twice the single-head size (rlk_linear_logp_fwd_pair_workspace_bytes). */
int rlk_linear_logp_fwd_pair_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                             size_t* bytes);

int rlk_linear_logp_fwd_pair(const void* hidden, const void* weight, const void* ref_weight,
                             const float* bias, const float* ref_bias, const int64_t* targets,
                             float* logp, float* lse, float* ref_logp, float* ref_lse,
                             void* workspace, size_t workspace_bytes, int64_t N, int32_t H,
                             int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                             int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                             int32_t* err_flag, rlk_stream_t stream);

/* ------------------------------------------------------------------------------------------ *
 * Fused linear -> log-prob, backward.
 *
 * Stands in for `chunked_linear_logp_backward`
 * (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:383-439) and, through `lse`, for the
 * vocab-parallel backward (same file :285-335):
 *   dZ = grad_logp / T * (onehot(target) - exp(z - lse)),  zero for ignored rows
 *   d_hidden = dZ W      (input dtype)
 *   d_weight = dZ^T H    (f32, overwritten)
 *   d_bias   = sum_n dZ  (f32, only when bias != NULL)
 * dZ only ever exists as one (token chunk) x (vocab piece) block of at most `dz_budget_bytes`
 * (0 = default 256 MiB; values are clamped to [128 KiB, 2 GiB], the upper limit keeping every
 * in-tile byte offset of the loaders within 32 bits) inside `workspace`, so extra memory does not
 * grow with N.
 * `lse` must be the natural-log logsumexp over the FULL vocabulary (for a shard: after the
 * cross-shard merge).  Any of d_hidden / d_weight / d_bias may be NULL to skip that gradient
 * (d_bias requires bias).
 * ------------------------------------------------------------------------------------------ */
int rlk_linear_logp_bwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                        size_t dz_budget_bytes, size_t* bytes);

/* Schedule the backward will use for these sizes (no counterpart in the reference, whose chunk is
 * fixed at 2^24 / V tokens, rl_engine/kernels/ops/pytorch/loss/linear_logp.py:398-400):
 * out5 = { tokens per chunk, vocab rows per piece, number of chunks, number of pieces, parts the
 * dH launch of a full block cuts the piece's vocab range into (1 unless there are few tokens; a
 * shorter last chunk or piece takes its own count by the same rule) }.  Host only; touches no
 * device. */
int rlk_linear_logp_bwd_plan(int64_t N, int32_t H, int64_t V, int32_t dtype,
                             size_t dz_budget_bytes, int64_t* out5);

int rlk_linear_logp_bwd(const float* grad_logp, const void* hidden, const void* weight,
                        const float* bias, const int64_t* targets, const float* lse,
                        void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                        size_t workspace_bytes, size_t dz_budget_bytes, int64_t N, int32_t H,
                        int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                        int64_t ignore_index, int32_t use_ignore, rlk_stream_t stream);

/* rlk_linear_logp_bwd into a running fp32 gradient: with accumulate != 0, d_weight and d_bias are
 * ADDED to what the buffers hold (d_weight += dZ^T H, d_bias += sum_n dZ) instead of overwritten;
 * accumulate == 0 is rlk_linear_logp_bwd.  d_hidden is always overwritten.  This is the reference's
 * own accumulation pattern moved to the caller's buffer: chunked_linear_logp_backward keeps one
 * fp32 grad_w over all token chunks and casts once at the end
 * (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:404,423-437).  A trainer that keeps fp32 main
 * gradients hands that buffer in and runs micro-batch after micro-batch into it: no [V, H]
 * temporary and no cast per call.  The sum over micro-batches is taken in call order (stream
 * order), so it is as repeatable as the calls. */
int rlk_linear_logp_bwd_accum(const float* grad_logp, const void* hidden, const void* weight,
                              const float* bias, const int64_t* targets, const float* lse,
                              void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                              size_t workspace_bytes, size_t dz_budget_bytes, int64_t N, int32_t H,
                              int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                              int64_t ignore_index, int32_t use_ignore, int32_t accumulate,
                              rlk_stream_t stream);

/* ------------------------------------------------------------------------------------------ *
 * Final RMSNorm in front of the head (the step before the path).
 *
 * rlk_rmsnorm_fwd stands in for NativeRMSNormOp.forward
 * (rl_engine/kernels/ops/pytorch/norm/rms_norm.py:28-70):
 *   out = cast_to_dtype( (x * rsqrt(mean(x^2, -1) + eps)) * gain ),  fp32 arithmetic,
 * x / out [N, H] of `dtype` (bf16 / f16 / f32), gain [H] ALWAYS f32 (the reference multiplies by
 * weight.float(), :66-70, so a gain kept in fp32 over 16-bit activations loses nothing), rstd [N]
 * f32 optional.  A row's
 * result does not depend on the other rows of the batch.  rlk_rmsnorm_bwd is its backward
 * (what autograd derives for that expression): d_x [N, H] of `dtype`, d_gain [H] f32
 * (overwritten; NULL to skip) from d_out [N, H] of `dtype`; the row statistics are recomputed.
 * ------------------------------------------------------------------------------------------ */
int rlk_rmsnorm_fwd(const void* x, const float* gain, float eps, void* out, float* rstd, int64_t N,
                    int32_t H, int32_t dtype, rlk_stream_t stream);

int rlk_rmsnorm_bwd_workspace_bytes(int64_t N, int32_t H, size_t* bytes);

int rlk_rmsnorm_bwd(const void* x, const float* gain, float eps, const void* d_out, void* d_x,
                    float* d_gain, void* workspace, size_t workspace_bytes, int64_t N, int32_t H,
                    int32_t dtype, rlk_stream_t stream);

/* Norm and head as one call each way (no counterpart as a single function in the reference, which
 * runs the model's final norm and `linear_logp` as separate modules): the entry points take the
 * UN-normalised hidden states x and the norm gain.
 *   forward : logp / lse of  linear_logp( rmsnorm(x, gain, eps), weight, bias, ... ),
 *             bit for bit what rlk_rmsnorm_fwd followed by rlk_linear_logp_fwd return on the same
 *             blocks of 8192 tokens (the whole input when N <= 8192);
 *   backward: d_x (gradient w.r.t. the un-normalised hidden states, `dtype`), d_gain [H] f32,
 *             d_weight [V, H] f32, d_bias [V] f32 -- rlk_linear_logp_bwd followed by rlk_rmsnorm_bwd.
 * The normalised rows are never saved: they exist as one block of at most 8192 tokens (64 MiB of
 * 16-bit rows at H = 4096) inside the workspace in either direction (the backward recomputes them),
 * so the caller keeps only x, and the extra memory stays independent of N.  In the backward the
 * head's gradient w.r.t. the normalised rows is written into the caller's d_x and the norm backward
 * runs on it in place.  Any gradient pointer may be NULL (without d_x the blocks are half as long
 * and the second half of the row region holds that gradient). */
int rlk_linear_logp_rmsnorm_fwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                                size_t* bytes);

int rlk_linear_logp_rmsnorm_fwd(const void* x, const float* gain, float eps, const void* weight,
                                const float* bias, const int64_t* targets, float* logp, float* lse,
                                void* workspace, size_t workspace_bytes, int64_t N, int32_t H,
                                int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                                int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                                int32_t* err_flag, rlk_stream_t stream);

int rlk_linear_logp_rmsnorm_bwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                                size_t dz_budget_bytes, size_t* bytes);

int rlk_linear_logp_rmsnorm_bwd(const float* grad_logp, const void* x, const float* gain, float eps,
                                const void* weight, const float* bias, const int64_t* targets,
                                const float* lse, void* d_x, float* d_gain, float* d_weight,
                                float* d_bias, void* workspace, size_t workspace_bytes,
                                size_t dz_budget_bytes, int64_t N, int32_t H, int64_t V,
                                int64_t vocab_start, int32_t dtype, float temperature,
                                int64_t ignore_index, int32_t use_ignore, rlk_stream_t stream);

/* ------------------------------------------------------------------------------------------ *
 * Selected-token log-prob from materialised logits (the `fused_logp` family).
 *
 * Stands in for the nine `_C.fused_logp*` symbols (csrc/ops.cpp:75-96, csrc/fused_logp_kernel.cu:
 * 452-588; signatures in rl_engine/_C.pyi:5-43): one single-pass online-softmax scan serves the
 * two-pass and the `online` variants alike (they compute the same value).
 *   logits [n_rows, vocab] bf16/f16/f32, ids [n_rows] int64, out [n_rows] of out_dtype
 *   (bf16/f16/f32/f64).  row_indices == NULL: every row is written (n_launch == n_rows).
 *   row_indices != NULL: only the n_launch listed rows are written, the others are left
 *   untouched; listed rows outside [0, n_rows) are skipped (csrc/fused_logp_kernel.cu:120-123).
 *   An id outside [0, vocab) yields 0, not an error (same file :147-155).
 *   lse_out (optional, f32 [n_rows]) receives logsumexp of each written row.
 * ------------------------------------------------------------------------------------------ */
int rlk_logp_from_logits(const void* logits, int32_t logits_dtype, const int64_t* ids, void* out,
                         int32_t out_dtype, float* lse_out, const int64_t* row_indices,
                         int64_t n_launch, int64_t n_rows, int64_t vocab, rlk_stream_t stream);

/* The same scan over two logits tensors of one shape and dtype (policy and reference) with shared
 * ids and row list in ONE launch, as the reference's ratio/KL program reads both rows
 * (rl_engine/kernels/ops/triton/loss/ratio_kl.py:46-60).  Each output equals the single call bit
 * for bit. */
int rlk_logp_from_logits_pair(const void* logits, const void* ref_logits, int32_t logits_dtype,
                              const int64_t* ids, void* out, void* ref_out, int32_t out_dtype,
                              float* lse_out, float* ref_lse_out, const int64_t* row_indices,
                              int64_t n_launch, int64_t n_rows, int64_t vocab, rlk_stream_t stream);

/* Backward of the above w.r.t. the logits:
 *   grad_logits[n][v] = coeff[n] * (onehot(ids[n])[v] - exp(logits[n][v] - lse[n]))
 * in the logits dtype; rows whose id is outside [0, vocab) get zeros.  Stands in for the
 * analytic backward of rl_engine/kernels/ops/triton/loss/ratio_kl.py:86-122 and for autograd
 * through rl_engine/kernels/ops/pytorch/loss/logp.py:16-32. */
int rlk_logp_from_logits_bwd(const void* logits, int32_t logits_dtype, const int64_t* ids,
                             const float* lse, const float* coeff, void* grad_logits,
                             int64_t n_rows, int64_t vocab, rlk_stream_t stream);

/* ------------------------------------------------------------------------------------------ *
 * Log-prob-fed GRPO / PPO loss epilogue.
 *
 * Stands in for the composition compute_policy_ratio / compute_reference_kl / masked_mean
 * (rl_engine/testing/reference_ops.py:50-106) as chained by
 * rl_engine/executors/deepspeed_trainer.py:160-167 and
 * rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:96-125:
 *   r = exp(cur - old) ; d = ref - cur ; M = max(sum(mask), 1e-8)
 *   policy = sum(mask * -min(r A, clip(r, 1-eps, 1+eps) A)) / M
 *   kl     = sum(mask * (e^d - d - 1)) / M               (0 when ref_logp == NULL)
 *   out3   = { policy + beta * kl, policy, kl }
 *   d_cur  = d out3[0] / d cur (optional; multiplied by *upstream when given)
 *   d_kl   = d out3[2] / d cur (optional, needs d_cur; so d out3[1]/d cur = d_cur - beta * d_kl)
 * advantages: per token [n_tokens] (adv_per_token != 0) or per sequence [n_tokens / seq_len].
 * mask: uint8 [n_tokens] or NULL (all active).  ratio / kl_terms (optional) receive the per-token
 * values with masked entries 0.  Sums use a fixed two-level tree.
 * ------------------------------------------------------------------------------------------ */
int rlk_grpo_loss_workspace_bytes(int64_t n_tokens, size_t* bytes);

int rlk_grpo_loss_from_logp(const float* cur_logp, const float* old_logp, const float* ref_logp,
                            const float* advantages, int32_t adv_per_token, const uint8_t* mask,
                            int64_t n_tokens, int64_t seq_len, float clip_eps, float beta,
                            float* out3, float* ratio, float* kl_terms, float* d_cur, float* d_kl,
                            const float* upstream, void* workspace, size_t workspace_bytes,
                            rlk_stream_t stream);

/* Forward of the fused linear log-prob with the loss epilogue above folded into its last launch
 * (the composition the trainer runs as two steps, rl_engine/executors/deepspeed_trainer.py:
 * 146-167): logp / lse exactly as rlk_linear_logp_fwd, and out3 / ratio / kl_terms / d_cur / d_kl
 * exactly as rlk_grpo_loss_from_logp(cur_logp = logp, upstream = NULL) -- same expressions, same
 * reduction tree, same bits -- without a second pass over the tokens: the active-token count is
 * taken from the mask before the contraction starts, the per-token terms and gradients leave the
 * launch that merges the vocab splits, and the workgroup of that launch that finishes last (an
 * integer ticket; the sums themselves use no atomics) adds up the block partials in block order.
 * Workspace: rlk_linear_logp_fwd_grpo_workspace_bytes (16-byte aligned).  Bit-equality of the
 * sums with the two-step route holds below 2^24 tokens. */
int rlk_linear_logp_fwd_grpo_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                             size_t* bytes);

int rlk_linear_logp_fwd_grpo(const void* hidden, const void* weight, const float* bias,
                             const int64_t* targets, float* logp, float* lse, void* workspace,
                             size_t workspace_bytes, int64_t N, int32_t H, int64_t V,
                             int64_t vocab_start, int32_t dtype, float temperature,
                             int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                             int32_t* err_flag, const float* old_logp, const float* ref_logp,
                             const float* advantages, int32_t adv_per_token, const uint8_t* mask,
                             int64_t seq_len, float clip_eps, float beta, float* out3, float* ratio,
                             float* kl_terms, float* d_cur, float* d_kl, rlk_stream_t stream);

/* Per-token policy ratio exp(cur - old) and k3 KL exp(ref - cur) - (ref - cur) - 1 of the
 * logits-fed ratio/KL op, the mask applied to the differences BEFORE the exponentials, so an
 * inactive position gives ratio 1 and kl 0: the tail of NativeRatioKLOp.forward
 * (rl_engine/kernels/ops/pytorch/loss/ratio_kl.py:53-58) and of _ratio_kl_fwd_kernel
 * (rl_engine/kernels/ops/triton/loss/ratio_kl.py:46-60) behind the log-prob scan.  All arrays
 * fp32 [N] on the device; mask uint8 [N] or NULL (all active).  The backward returns
 * d_cur = grad_ratio * ratio + grad_kl * (1 - exp(ref - cur)) on active positions, 0 elsewhere
 * (grad_ratio / grad_kl may be NULL = zero), the coefficient _ratio_kl_bwd_kernel feeds into
 * the logits gradient (same file :86-122). */
int rlk_ratio_kl_from_logp(const float* cur_logp, const float* ref_logp, const float* old_logp,
                           const uint8_t* mask, int64_t N, float* ratio, float* kl,
                           rlk_stream_t stream);
int rlk_ratio_kl_from_logp_bwd(const float* cur_logp, const float* ref_logp, const float* old_logp,
                               const uint8_t* mask, const float* grad_ratio, const float* grad_kl,
                               int64_t N, float* d_cur, rlk_stream_t stream);

/* Per-group reward normalisation (x - mean_g) / sqrt(max(E_g[x^2] - mean_g^2, eps^2)) over CSR
 * group boundaries (int64 [num_groups + 1], device).  Stands in for
 * NativeGRPOLossOp.group_advantages (rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:53-84) and
 * _group_norm_kernel (rl_engine/kernels/ops/triton/loss/grpo_loss.py:30-55). */
int rlk_group_advantages(const float* rewards, const int64_t* group_bounds, int64_t num_groups,
                         float eps, float* advantages, rlk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* RLK_HIP_H */
