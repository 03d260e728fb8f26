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

// Scalar-FMA implementation of the same two entry points for what the MFMA tiles do not take:
// fp32 inputs, hidden sizes that are not a multiple of 8, misaligned matrices (rlk_generic.hip).
namespace rlk {
int generic_fwd(const void* hidden, const void* weight, const float* bias, const int64_t* targets,
                float* logp, float* lse, int64_t N, int32_t H, int64_t V, int64_t vocab_start,
                int32_t dtype, float temperature, int64_t ignore_index, int32_t use_ignore,
                int32_t strict_targets, int32_t* err_flag, hipStream_t stream);
size_t generic_bwd_workspace(int64_t N, int32_t H, int64_t V);
int generic_bwd(const float* grad_logp, const void* hidden, const void* weight, const float* bias,
                const int64_t* targets, const float* lse, void* d_hidden, float* d_weight,
                float* d_bias, void* workspace, int64_t N, int32_t H, int64_t V,
                int64_t vocab_start, int32_t dtype, float temperature, int64_t ignore_index,
                int32_t use_ignore, hipStream_t stream);
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
