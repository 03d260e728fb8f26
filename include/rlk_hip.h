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

/* ABI version of this header (major * 100 + minor). */
int rlk_version(void);

/* Message of the last error returned on the calling thread ("" if none). Host pointer, valid
 * until the next failing call on the same thread. */
const char* rlk_last_error(void);

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
 *            *err_flag (device int32, caller zeroes it); the Python layer turns that into the
 *            reference's ValueError (rl_engine/kernels/ops/cuda/loss/linear_logp.py:352-358).
 *            With strict_targets == 0 such a row yields logp = -lse (z_t = 0), which is what a
 *            vocab-parallel shard must return (csrc/cuda/fused_linear_logp_sm90.cu:256-280).
 *   H must be a multiple of 8 and the two matrices 16-byte aligned, else RLK_ERR_UNSUPPORTED /
 *   RLK_ERR_ARG.
 * ------------------------------------------------------------------------------------------ */
int rlk_linear_logp_fwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                        size_t* bytes);

int rlk_linear_logp_fwd(const void* hidden, const void* weight, const float* bias,
                        const int64_t* targets, float* logp, float* lse, void* workspace,
                        size_t workspace_bytes, int64_t N, int32_t H, int64_t V,
                        int64_t vocab_start, int32_t dtype, float temperature,
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
 * (0 = default 512 MiB) inside `workspace`, so extra memory does not grow with N.
 * `lse` must be the natural-log logsumexp over the FULL vocabulary (for a shard: after the
 * cross-shard merge).  Any of d_hidden / d_weight / d_bias may be NULL to skip that gradient
 * (d_bias requires bias).
 * ------------------------------------------------------------------------------------------ */
int rlk_linear_logp_bwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                        size_t dz_budget_bytes, size_t* bytes);

int rlk_linear_logp_bwd(const float* grad_logp, const void* hidden, const void* weight,
                        const float* bias, const int64_t* targets, const float* lse,
                        void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                        size_t workspace_bytes, size_t dz_budget_bytes, int64_t N, int32_t H,
                        int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                        int64_t ignore_index, int32_t use_ignore, rlk_stream_t stream);

/* ------------------------------------------------------------------------------------------ *
 * Hardware-contract self test (no counterpart in the reference): checks that the gfx950
 * transposing LDS read delivers the MFMA operand layout the backward contractions rely on.
 * out: device int32[512]; out[l*8 + e] must equal (8*(l/32) + e) * 256 + (l % 32).
 * ------------------------------------------------------------------------------------------ */
int rlk_selftest_transpose_read(int32_t* out, rlk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* RLK_HIP_H */
