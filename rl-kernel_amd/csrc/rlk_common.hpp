// Shared definitions of the librlk_hip C-ABI implementation (error codes, dtype ids).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/rlk_hip.h"

#ifndef RLK_BK
#define RLK_BK 64  // K elements staged through LDS per pipeline step
#endif

#ifndef RLK_DEFAULT_DZ_BUDGET
#define RLK_DEFAULT_DZ_BUDGET (static_cast<size_t>(256) << 20)  // bytes of one dZ block
#endif

#ifndef RLK_MAX_DZ_BUDGET
#define RLK_MAX_DZ_BUDGET (static_cast<size_t>(2) << 30)  // upper clamp of dz_budget_bytes
#endif

// Records `msg` as the calling thread's last error and returns `code` (always negative).
int rlk_fail(int code, const char* msg);

// fp32 matrix-core implementation of the same contractions for what the 16-bit MFMA tiles do not
// take: fp32 inputs, hidden sizes that are not a multiple of 8, misaligned matrices (rlk_wide.hip).
namespace rlk {
// Forward contraction only: per-split softmax states (max, sum, target logit; log2 domain) of the
// whole vocabulary cut into n_split <= ceil(V / 256) ranges, in the layout the split combine reads.
int wide_fwd_partials(const void* hidden, const void* weight, const float* bias, const int64_t* targets,
                      float* part_m, float* part_s, float* part_z, int n_split, int64_t N, int32_t H,
                      int64_t V, int64_t vocab_start, int32_t dtype, float temperature, hipStream_t stream);
size_t wide_bwd_workspace(int64_t N, int32_t H, int64_t V, size_t dz_budget_bytes);
int wide_bwd(const float* grad_logp, const void* hidden, const void* weight, const float* bias,
             const int64_t* targets, const float* lse, void* d_hidden, float* d_weight, float* d_bias,
             void* workspace, size_t dz_budget_bytes, int64_t N, int32_t H, int64_t V,
             int64_t vocab_start, int32_t dtype, float temperature, int64_t ignore_index,
             int32_t use_ignore, int32_t accumulate, hipStream_t stream);
// rlk_linear_logp_bwd with one more switch: accumulate != 0 adds d_weight / d_bias to what the
// buffers already hold (callers that feed the tokens in several blocks).
int linear_logp_bwd_accumulating(const float* grad_logp, const void* hidden, const void* weight,
                                 const float* bias, const int64_t* targets, const float* lse,
                                 void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                                 size_t workspace_bytes, size_t dz_budget_bytes, int64_t N, int32_t H,
                                 int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                                 int64_t ignore_index, int32_t use_ignore, int32_t accumulate,
                                 hipStream_t stream);
}  // namespace rlk
