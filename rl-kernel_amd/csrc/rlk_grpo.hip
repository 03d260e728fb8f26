// Log-prob-fed GRPO / PPO loss epilogue: per-token policy ratio, clipped surrogate and k3 KL,
// masked token-mean with a fixed two-level reduction tree, and dloss/dlogp.  Also the per-group
// reward normalisation.  All sums run in a fixed order (no atomics): same input, same bits.
#include "rlk_grpo.hpp"

namespace rlk {

// Block b owns the contiguous element range [b*per, (b+1)*per); thread t walks it with stride
// 256 in ascending order.
__global__ __launch_bounds__(kRedThreads) void grpo_terms_kernel(GrpoArgs a)
{
    const int64_t per = (a.n + a.blocks - 1) / a.blocks;
    const int64_t lo = per * blockIdx.x;
    const int64_t hi = lo + per < a.n ? lo + per : a.n;
    Term t{0.f, 0.f, 0.f};
    for (int64_t i = lo + threadIdx.x; i < hi; i += kRedThreads) {
        const bool on = a.mask == nullptr || a.mask[i] != 0;
        float r = 0.f, k = 0.f;
        if (on) {
            float pol;
            token_terms(a, i, a.cur[i], r, pol, k);
            t.pol += pol;
            if (a.ref_lp != nullptr) t.kl += k;
            t.act += 1.f;
        }
        if (a.ratio) a.ratio[i] = r;
        if (a.kl_terms) a.kl_terms[i] = k;
    }
    const Term s = block_sum(t);
    if (threadIdx.x == 0) {
        a.partial[blockIdx.x * 3 + 0] = s.pol;
        a.partial[blockIdx.x * 3 + 1] = s.kl;
        a.partial[blockIdx.x * 3 + 2] = s.act;
    }
}

// d loss / d cur of every token (needs the denominator the finish kernel left).
__global__ void grpo_grad_kernel(GrpoArgs a)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    float g = 0.f, gk = 0.f;
    if (a.mask == nullptr || a.mask[i] != 0) token_grad(a, i, a.cur[i], a.denom[0], g, gk);
    a.dcur[i] = g;
    if (a.dkl != nullptr) a.dkl[i] = gk;
}

// Per-token policy ratio and k3 KL of the logits-fed ratio/KL op: the mask is applied to the
// log-prob differences before the exponentials, so inactive positions give ratio 1 and kl 0.
__global__ void ratio_kl_fwd_kernel(const float* cur, const float* ref, const float* old_lp,
                                    const uint8_t* mask, float* ratio, float* kl, int64_t n)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const bool on = mask == nullptr || mask[i] != 0;
    const float delta = on ? cur[i] - old_lp[i] : 0.f;
    const float diff = on ? ref[i] - cur[i] : 0.f;
    ratio[i] = expf(delta);
    kl[i] = expf(diff) - diff - 1.f;
}

// d/d cur of g_ratio * ratio + g_kl * kl: ratio' = ratio, kl' = 1 - exp(ref - cur); 0 when inactive.
__global__ void ratio_kl_bwd_kernel(const float* cur, const float* ref, const float* old_lp,
                                    const uint8_t* mask, const float* g_ratio, const float* g_kl,
                                    float* d_cur, int64_t n)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float g = 0.f;
    if (mask == nullptr || mask[i] != 0) {
        if (g_ratio != nullptr) g += g_ratio[i] * expf(cur[i] - old_lp[i]);
        if (g_kl != nullptr) g += g_kl[i] * (1.f - expf(ref[i] - cur[i]));
    }
    d_cur[i] = g;
}

// One wavefront per group: (x - mean) / sqrt(max(E[x^2] - mean^2, eps^2)).
__global__ __launch_bounds__(64) void group_advantages_kernel(const float* rewards,
                                                              const int64_t* bounds, float eps,
                                                              float* adv)
{
    const int64_t lo = bounds[blockIdx.x], hi = bounds[blockIdx.x + 1];
    float s1 = 0.f, s2 = 0.f;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 64) {
        const float x = rewards[i];
        s1 += x;
        s2 += x * x;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        s1 += __shfl_down(s1, o);
        s2 += __shfl_down(s2, o);
    }
    s1 = __shfl(s1, 0);
    s2 = __shfl(s2, 0);
    const float cnt = static_cast<float>(hi - lo);
    const float mean = s1 / cnt;
    const float var = fmaxf(s2 / cnt - mean * mean, eps * eps);
    const float sd = sqrtf(var);
    for (int64_t i = lo + threadIdx.x; i < hi; i += 64) adv[i] = (rewards[i] - mean) / sd;
}

}  // namespace rlk

using namespace rlk;

extern "C" {

int rlk_grpo_loss_workspace_bytes(int64_t n_tokens, size_t* bytes)
{
    if (!bytes || n_tokens < 0) return rlk_fail(RLK_ERR_ARG, "bad workspace query");
    *bytes = (static_cast<size_t>(kMaxBlocks) * 3 + kGrpoTailFloats) * sizeof(float);
    return 0;
}

int rlk_grpo_loss_from_logp(const float* cur_logp, const float* old_logp, const float* ref_logp,
                            const float* advantages, int32_t adv_per_token, const uint8_t* mask,
                            int64_t n_tokens, int64_t seq_len, float clip_eps, float beta,
                            float* out3, float* ratio, float* kl_terms, float* d_cur, float* d_kl,
                            const float* upstream, void* workspace, size_t workspace_bytes,
                            hipStream_t stream)
{
    if (!cur_logp || !old_logp || !advantages || !out3) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (n_tokens < 0 || seq_len <= 0) return rlk_fail(RLK_ERR_ARG, "bad sizes");
    if (!adv_per_token && n_tokens % seq_len != 0)
        return rlk_fail(RLK_ERR_ARG, "n_tokens must be a multiple of seq_len for per-sequence advantages");
    size_t need = 0;
    rlk_grpo_loss_workspace_bytes(n_tokens, &need);
    if (!workspace || workspace_bytes < need) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    GrpoArgs a;
    a.cur = cur_logp;
    a.old_lp = old_logp;
    a.ref_lp = ref_logp;
    a.adv = advantages;
    a.mask = mask;
    a.ratio = ratio;
    a.kl_terms = kl_terms;
    a.partial = static_cast<float*>(workspace);
    a.denom = a.partial + kMaxBlocks * 3;
    a.words = reinterpret_cast<int*>(a.denom + 4);
    a.out3 = out3;
    a.dcur = d_cur;
    a.dkl = d_kl;
    a.upstream = upstream;
    if (d_kl != nullptr && d_cur == nullptr) return rlk_fail(RLK_ERR_ARG, "d_kl requires d_cur");
    a.n = n_tokens;
    a.seq_len = seq_len;
    a.adv_per_token = adv_per_token;
    a.clip_lo = 1.f - clip_eps;
    a.clip_hi = 1.f + clip_eps;
    a.beta = beta;
    a.blocks = grpo_blocks(n_tokens);
    hipLaunchKernelGGL(grpo_terms_kernel, dim3(a.blocks), dim3(kRedThreads), 0, stream, a);
    hipLaunchKernelGGL(grpo_finish_kernel<0>, dim3(1), dim3(kRedThreads), 0, stream, a);
    if (d_cur != nullptr && n_tokens > 0)
        hipLaunchKernelGGL(grpo_grad_kernel, dim3(static_cast<unsigned>((n_tokens + 255) / 256)),
                           dim3(256), 0, stream, a);
    if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "grpo launch failed");
    return 0;
}

int rlk_ratio_kl_from_logp(const float* cur_logp, const float* ref_logp, const float* old_logp,
                           const uint8_t* mask, int64_t N, float* ratio, float* kl, hipStream_t stream)
{
    if (!cur_logp || !ref_logp || !old_logp || !ratio || !kl) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (N < 0) return rlk_fail(RLK_ERR_ARG, "bad sizes");
    if (N == 0) return 0;
    hipLaunchKernelGGL(ratio_kl_fwd_kernel, dim3(static_cast<unsigned>((N + 255) / 256)), dim3(256), 0, stream,
                       cur_logp, ref_logp, old_logp, mask, ratio, kl, N);
    if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "ratio / kl launch failed");
    return 0;
}

int rlk_ratio_kl_from_logp_bwd(const float* cur_logp, const float* ref_logp, const float* old_logp,
                               const uint8_t* mask, const float* grad_ratio, const float* grad_kl,
                               int64_t N, float* d_cur, hipStream_t stream)
{
    if (!cur_logp || !ref_logp || !old_logp || !d_cur) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (N < 0) return rlk_fail(RLK_ERR_ARG, "bad sizes");
    if (N == 0) return 0;
    hipLaunchKernelGGL(ratio_kl_bwd_kernel, dim3(static_cast<unsigned>((N + 255) / 256)), dim3(256), 0, stream,
                       cur_logp, ref_logp, old_logp, mask, grad_ratio, grad_kl, d_cur, N);
    if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "ratio / kl backward launch failed");
    return 0;
}

int rlk_group_advantages(const float* rewards, const int64_t* group_bounds, int64_t num_groups,
                         float eps, float* advantages, hipStream_t stream)
{
    if (!rewards || !group_bounds || !advantages) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (num_groups < 0 || num_groups > 0x7fffffffLL) return rlk_fail(RLK_ERR_ARG, "bad group count");
    if (num_groups == 0) return 0;
    hipLaunchKernelGGL(group_advantages_kernel, dim3(static_cast<unsigned>(num_groups)), dim3(64), 0,
                       stream, rewards, group_bounds, eps, advantages);
    if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "group advantages launch failed");
    return 0;
}

}  // extern "C"
