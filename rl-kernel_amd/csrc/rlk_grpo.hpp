// Per-token math and the fixed reduction tree of the log-prob-fed GRPO / PPO loss epilogue, shared
// by the stand-alone epilogue kernels and by the forward's combine launch that folds the epilogue
// in.  One definition of every expression, so both routes produce the same bits.
#pragma once
#include "rlk_common.hpp"

namespace rlk {

constexpr int kRedThreads = 256;
constexpr int kMaxBlocks = 1024;

struct GrpoArgs {
    const float* cur;
    const float* old_lp;
    const float* ref_lp;   // may be null: KL term is 0
    const float* adv;      // per token [n] or per sequence [n / seq_len]
    const uint8_t* mask;   // may be null: every token active
    float* ratio;          // optional per-token outputs (masked entries 0)
    float* kl_terms;
    float* partial;        // [blocks][3]: policy sum, kl sum, active count
    float* out3;           // loss, policy_loss, kl
    float* denom;          // max(count, 1e-8) kept for the gradient kernel
    int* words;            // integer words of the workspace tail (forward-folded route only)
    float* dcur;
    float* dkl;            // optional: d kl / d cur alone (not scaled by beta or upstream)
    const float* upstream; // optional device scalar multiplying dcur
    int64_t n;
    int64_t seq_len;
    int adv_per_token;
    float clip_lo, clip_hi, beta;
    int blocks;
};

struct Term {
    float pol, kl, act;
};

__device__ inline float adv_of(const GrpoArgs& a, int64_t i)
{
    return a.adv_per_token ? a.adv[i] : a.adv[i / a.seq_len];
}

// Fixed tree: lanes of a wavefront (shuffle), then wavefronts through LDS, left to right.
__device__ inline Term block_sum(Term t)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        t.pol += __shfl_down(t.pol, o);
        t.kl += __shfl_down(t.kl, o);
        t.act += __shfl_down(t.act, o);
    }
    __shared__ float sh[kRedThreads / 64][3];
    if ((threadIdx.x & 63) == 0) {
        sh[threadIdx.x >> 6][0] = t.pol;
        sh[threadIdx.x >> 6][1] = t.kl;
        sh[threadIdx.x >> 6][2] = t.act;
    }
    __syncthreads();
    Term r{0.f, 0.f, 0.f};
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 0; w < kRedThreads / 64; ++w) {
            r.pol += sh[w][0];
            r.kl += sh[w][1];
            r.act += sh[w][2];
        }
    }
    return r;
}

// Loss terms of one active token: probability ratio, its contribution to the clipped surrogate
// sum, and the k3 KL term (0 without a reference).
__device__ inline void token_terms(const GrpoArgs& a, int64_t i, float c, float& r, float& pol, float& k)
{
    r = expf(c - a.old_lp[i]);
    const float ad = adv_of(a, i);
    const float rc = fminf(fmaxf(r, a.clip_lo), a.clip_hi);
    pol = -fminf(r * ad, rc * ad);
    k = 0.f;
    if (a.ref_lp != nullptr) {
        const float d = a.ref_lp[i] - c;
        k = expf(d) - d - 1.f;
    }
}

// d loss / d cur and d kl / d cur of one active token.  torch semantics of the composition:
// `minimum` sends the gradient to the smaller branch and splits it on ties; `clamp` passes it on
// the closed interval.
__device__ inline void token_grad(const GrpoArgs& a, int64_t i, float c, float denom, float& g, float& gk)
{
    const float r = expf(c - a.old_lp[i]);
    const float ad = adv_of(a, i);
    const float rc = fminf(fmaxf(r, a.clip_lo), a.clip_hi);
    const float un = r * ad, cl = rc * ad;
    const float inside = (r >= a.clip_lo && r <= a.clip_hi) ? 1.f : 0.f;
    const float w_un = un < cl ? 1.f : (un == cl ? 0.5f : 0.f);
    g = -(w_un * ad * r + (1.f - w_un) * ad * r * inside);
    gk = 0.f;
    if (a.ref_lp != nullptr) gk = (1.f - expf(a.ref_lp[i] - c)) / denom;
    g = g / denom + a.beta * gk;
    if (a.upstream != nullptr) g *= a.upstream[0];
}

// Blocks of the two-level sum over n tokens: one token per thread up to kMaxBlocks blocks, several
// per thread beyond that.
inline int grpo_blocks(int64_t n)
{
    int64_t blocks = (n + kRedThreads - 1) / kRedThreads;
    if (blocks < 1) blocks = 1;
    if (blocks > kMaxBlocks) blocks = kMaxBlocks;
    return static_cast<int>(blocks);
}

// Tokens one workgroup of the active-token count covers, and the most such workgroups.
constexpr int64_t kCountSpan = 262144;
constexpr int kMaxCountParts = 64;
inline int grpo_count_parts(int64_t n)
{
    int64_t parts = (n + kCountSpan - 1) / kCountSpan;
    if (parts < 1) parts = 1;
    if (parts > kMaxCountParts) parts = kMaxCountParts;
    return static_cast<int>(parts);
}

// Floats of workspace behind the block partials: [0] denominator, [4 ..) the integer words
// (ticket of the last-block finish, number of count parts, the count parts).
constexpr int kGrpoTailFloats = 4 + 2 + kMaxCountParts + 2;

// Sum of the block partials and the three scalars: one workgroup.  (A template so that every
// translation unit that launches it holds its own instance.)
// (`coherent`: the partials were written by other workgroups of the same launch, read them past
// the L1.)
template <bool COHERENT>
__device__ inline void grpo_finish(const GrpoArgs& a)
{
    Term t{0.f, 0.f, 0.f};
    for (int b = threadIdx.x; b < a.blocks; b += kRedThreads) {
        if (COHERENT) {
            t.pol += __hip_atomic_load(a.partial + b * 3 + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            t.kl += __hip_atomic_load(a.partial + b * 3 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            t.act += __hip_atomic_load(a.partial + b * 3 + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            t.pol += a.partial[b * 3 + 0];
            t.kl += a.partial[b * 3 + 1];
            t.act += a.partial[b * 3 + 2];
        }
    }
    const Term s = block_sum(t);
    if (threadIdx.x == 0) {
        const float denom = fmaxf(s.act, 1e-8f);
        const float pol = s.pol / denom, kl = s.kl / denom;
        a.out3[0] = pol + a.beta * kl;
        a.out3[1] = pol;
        a.out3[2] = kl;
        a.denom[0] = denom;
    }
}

template <int kUnused = 0>
__global__ __launch_bounds__(kRedThreads) void grpo_finish_kernel(GrpoArgs a)
{
    grpo_finish<false>(a);
}

// Number of active tokens, known from the mask alone: lets a caller that fuses the per-token pass
// into an earlier kernel compute gradients before the sums exist.  Workgroup p counts the tokens
// [p * span, (p + 1) * span) with 16-byte loads and leaves an integer part; workgroup 0 also zeroes
// the ticket of the last-block finish.  (Integer count: equal to the fp32 sum of ones of
// grpo_finish_kernel below 2^24 tokens.)
template <int kUnused = 0>
__global__ __launch_bounds__(kRedThreads) void grpo_count_kernel(const uint8_t* mask, int64_t n,
                                                                 int parts, int* words)
{
    const int64_t span = (n + parts - 1) / parts;
    const int64_t lo = span * blockIdx.x;
    const int64_t hi = lo + span < n ? lo + span : n;
    int cnt = 0;
    if (mask != nullptr && lo < hi) {
        // head up to a 16-byte boundary, 16-byte body, tail
        const uintptr_t addr = reinterpret_cast<uintptr_t>(mask + lo);
        int64_t head = static_cast<int64_t>((16 - (addr & 15)) & 15);
        if (head > hi - lo) head = hi - lo;
        const int64_t body = (hi - lo - head) / 16;
        for (int64_t i = threadIdx.x; i < head; i += kRedThreads) cnt += mask[lo + i] != 0;
        const uint4* v = reinterpret_cast<const uint4*>(mask + lo + head);
#pragma unroll 8
        for (int64_t i = threadIdx.x; i < body; i += kRedThreads) {
            const uint4 w = v[i];
            const uint32_t q[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int k = 0; k < 4; ++k)  // a byte counts when it is non-zero
                cnt += ((q[k] & 0xffu) != 0) + ((q[k] & 0xff00u) != 0) + ((q[k] & 0xff0000u) != 0) +
                       ((q[k] & 0xff000000u) != 0);
        }
        for (int64_t i = lo + head + body * 16 + threadIdx.x; i < hi; i += kRedThreads) cnt += mask[i] != 0;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cnt += __shfl_down(cnt, o);
    __shared__ int sh[kRedThreads / 64];
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        for (int w = 0; w < kRedThreads / 64; ++w) total += sh[w];
        if (mask == nullptr) total = static_cast<int>(hi > lo ? hi - lo : 0);
        words[2 + blockIdx.x] = total;
        if (blockIdx.x == 0) {
            words[0] = 0;      // ticket
            words[1] = parts;
        }
    }
}

// max(active tokens, 1e-8) from the parts grpo_count_kernel left (uniform over the workgroup; all
// threads must call it).
__device__ inline float grpo_denominator(const int* words)
{
    __shared__ float denom_sh;
    if (threadIdx.x < 64) {
        const int parts = words[1];
        long long c = static_cast<int>(threadIdx.x) < parts ? words[2 + threadIdx.x] : 0;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) c += __shfl_down(c, o);
        if (threadIdx.x == 0) denom_sh = fmaxf(static_cast<float>(c), 1e-8f);
    }
    __syncthreads();
    return denom_sh;
}

}  // namespace rlk
