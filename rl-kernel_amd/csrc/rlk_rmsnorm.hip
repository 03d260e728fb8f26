// RMSNorm in front of the fused linear log-prob: out = x * rsqrt(mean(x^2) + eps) * gain, computed
// in fp32 and cast to the input dtype, its backward (d_x and d_gain), and the two entry points
// that take the UN-normalised hidden states and run norm + linear log-prob (forward) or linear
// log-prob backward + norm backward as one call.  The normalised rows only ever exist as one
// block of at most kNormBlockTokens tokens inside the workspace.  All sums run in a fixed order.
#include "rlk_common.hpp"

namespace rlk {

constexpr int kNormThreads = 256;
constexpr int kNormRowsPerGroup = 64;  // rows one workgroup of the backward walks (d_gain partial)

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4n;
typedef __attribute__((ext_vector_type(4))) float f32x4n;

template <int DT>
struct NormElem;
template <>
struct NormElem<RLK_DTYPE_BF16> {
    using type = uint16_t;
    __device__ static float get(uint16_t x) { return __builtin_bit_cast(float, static_cast<uint32_t>(x) << 16); }
    __device__ static uint16_t put(float x) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x)); }
};
template <>
struct NormElem<RLK_DTYPE_F16> {
    using type = uint16_t;
    __device__ static float get(uint16_t x) { return static_cast<float>(__builtin_bit_cast(_Float16, x)); }
    __device__ static uint16_t put(float x) { return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x)); }
};
template <>
struct NormElem<RLK_DTYPE_F32> {
    using type = float;
    __device__ static float get(float x) { return x; }
    __device__ static float put(float x) { return x; }
};

// Sum over the workgroup in a fixed tree (lanes by shuffle, wavefronts through LDS left to right);
// every thread receives the total.  All threads must call it.
__device__ inline float norm_block_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o);
    __shared__ float sh[kNormThreads / 64];
    __shared__ float total;
    __syncthreads();  // earlier readers of `total` are done
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < kNormThreads / 64; ++w) t += sh[w];
        total = t;
    }
    __syncthreads();
    return total;
}

// Thread t owns the elements h = (t + k * 256) * VEC + e, e < VEC, k = 0, 1, ...: VEC = 8 is one
// 16-byte load of 16-bit data (needs H % 8 == 0 and aligned rows), VEC = 1 the general case.
template <int DT, int VEC>
__device__ inline float row_sum_squares(const typename NormElem<DT>::type* x, int H)
{
    using E = typename NormElem<DT>::type;
    float ss = 0.f;
    for (int h = threadIdx.x * VEC; h < H; h += kNormThreads * VEC) {
        if constexpr (VEC == 8) {
            const u32x4n v = *reinterpret_cast<const u32x4n*>(x + h);
            const E* e = reinterpret_cast<const E*>(&v);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float f = NormElem<DT>::get(e[k]);
                ss += f * f;
            }
        } else {
            const float f = NormElem<DT>::get(x[h]);
            ss += f * f;
        }
    }
    return norm_block_sum(ss);
}

// One workgroup per row: rstd = rsqrt(mean(x^2) + eps); out = cast((x * rstd) * gain), gain in fp32.
template <int DT, int VEC>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_fwd_kernel(const void* x_v, const float* gain,
                                                                   float eps, void* out_v, float* rstd,
                                                                   int H)
{
    using E = typename NormElem<DT>::type;
    const int64_t row = blockIdx.x;
    const E* x = static_cast<const E*>(x_v) + row * H;
    E* out = static_cast<E*>(out_v) + row * H;
    const float r = rsqrtf(row_sum_squares<DT, VEC>(x, H) / static_cast<float>(H) + eps);
    if (rstd != nullptr && threadIdx.x == 0) rstd[row] = r;
    for (int h = threadIdx.x * VEC; h < H; h += kNormThreads * VEC) {
        if constexpr (VEC == 8) {
            const u32x4n xv = *reinterpret_cast<const u32x4n*>(x + h);
            const f32x4n g0 = *reinterpret_cast<const f32x4n*>(gain + h);
            const f32x4n g1 = *reinterpret_cast<const f32x4n*>(gain + h + 4);
            const float ge[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
            const E* xe = reinterpret_cast<const E*>(&xv);
            u32x4n ov;
            E* oe = reinterpret_cast<E*>(&ov);
#pragma unroll
            for (int k = 0; k < 8; ++k) oe[k] = NormElem<DT>::put((NormElem<DT>::get(xe[k]) * r) * ge[k]);
            *reinterpret_cast<u32x4n*>(out + h) = ov;
        } else {
            out[h] = NormElem<DT>::put((NormElem<DT>::get(x[h]) * r) * gain[h]);
        }
    }
}

// Backward of the norm for a group of rows.  With g = d_out * gain and r = rstd of the row:
//   d_x = r * g - x * (r^3 / H) * sum_h(g_h x_h)          d_gain_h += d_out_h * x_h * r
// d_gain of the group is accumulated per column in LDS (each thread owns its columns, rows in
// ascending order) and written as one partial row; rmsnorm_gain_finish_kernel adds the partials
// in group order.
template <int DT, int VEC>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_bwd_kernel(const void* x_v, const float* gain,
                                                                   float eps, const void* dout_v,
                                                                   void* dx_v, float* gain_part,
                                                                   int64_t n_rows, int H)
{
    using E = typename NormElem<DT>::type;
    extern __shared__ float dg[];  // [H]
    for (int h = threadIdx.x; h < H; h += kNormThreads) dg[h] = 0.f;  // (own columns only below)
    __syncthreads();
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kNormRowsPerGroup;
    const int64_t row1 = row0 + kNormRowsPerGroup < n_rows ? row0 + kNormRowsPerGroup : n_rows;
    for (int64_t row = row0; row < row1; ++row) {
        const E* x = static_cast<const E*>(x_v) + row * H;
        const E* dy = static_cast<const E*>(dout_v) + row * H;
        E* dx = static_cast<E*>(dx_v) + row * H;
        const float r = rsqrtf(row_sum_squares<DT, VEC>(x, H) / static_cast<float>(H) + eps);
        float dot = 0.f;
        for (int h = threadIdx.x * VEC; h < H; h += kNormThreads * VEC) {
#pragma unroll
            for (int k = 0; k < VEC; ++k)
                dot += (NormElem<DT>::get(dy[h + k]) * gain[h + k]) * NormElem<DT>::get(x[h + k]);
        }
        dot = norm_block_sum(dot);
        const float c = r * r * r * dot / static_cast<float>(H);
        for (int h = threadIdx.x * VEC; h < H; h += kNormThreads * VEC) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float xf = NormElem<DT>::get(x[h + k]);
                const float dyf = NormElem<DT>::get(dy[h + k]);
                const float g = dyf * gain[h + k];
                dx[h + k] = NormElem<DT>::put(r * g - xf * c);
                dg[h + k] += dyf * xf * r;
            }
        }
    }
    __syncthreads();
    float* part = gain_part + static_cast<int64_t>(blockIdx.x) * H;
    for (int h = threadIdx.x; h < H; h += kNormThreads) part[h] = dg[h];
}

// d_gain[h] (+)= sum over the groups' partial rows, in group order.  One thread per column.
__global__ void rmsnorm_gain_finish_kernel(const float* gain_part, int groups, int H, float* d_gain,
                                           int accumulate)
{
    const int h = blockIdx.x * blockDim.x + threadIdx.x;
    if (h >= H) return;
    float s = accumulate ? d_gain[h] : 0.f;
#pragma unroll 8
    for (int g = 0; g < groups; ++g) s += gain_part[static_cast<int64_t>(g) * H + h];
    d_gain[h] = s;
}

namespace {

bool vec_ok(const void* a, const void* b, const void* c, int H, int dtype)
{
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                           reinterpret_cast<uintptr_t>(c);
    return dtype != RLK_DTYPE_F32 && H % 8 == 0 && (bits & 15) == 0;
}

int check_norm(const void* x, const float* gain, int64_t N, int32_t H, int dtype)
{
    if (!x || !gain) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (N <= 0 || H <= 0) return rlk_fail(RLK_ERR_ARG, "N and H must be positive");
    if (N > 0x7fffffffLL) return rlk_fail(RLK_ERR_ARG, "N too large");
    if (dtype != RLK_DTYPE_BF16 && dtype != RLK_DTYPE_F16 && dtype != RLK_DTYPE_F32)
        return rlk_fail(RLK_ERR_UNSUPPORTED, "dtype must be RLK_DTYPE_BF16, RLK_DTYPE_F16 or RLK_DTYPE_F32");
    if (H > 36864) return rlk_fail(RLK_ERR_UNSUPPORTED, "RMSNorm rows above 36864 elements are not supported");
    return 0;
}

template <int DT>
int launch_fwd(const void* x, const float* gain, float eps, void* out, float* rstd, int64_t N, int H,
               bool vec, hipStream_t stream)
{
    const dim3 grid(static_cast<unsigned>(N)), block(kNormThreads);
    if (vec)
        hipLaunchKernelGGL((rmsnorm_fwd_kernel<DT, DT == RLK_DTYPE_F32 ? 1 : 8>), grid, block, 0, stream, x,
                           gain, eps, out, rstd, H);
    else
        hipLaunchKernelGGL((rmsnorm_fwd_kernel<DT, 1>), grid, block, 0, stream, x, gain, eps, out, rstd, H);
    return hipGetLastError() == hipSuccess ? 0 : rlk_fail(RLK_ERR_LAUNCH, "rmsnorm forward launch failed");
}

template <int DT>
int launch_bwd(const void* x, const float* gain, float eps, const void* dout, void* dx, float* part,
               int64_t N, int H, bool vec, hipStream_t stream)
{
    const unsigned groups = static_cast<unsigned>((N + kNormRowsPerGroup - 1) / kNormRowsPerGroup);
    const size_t lds = static_cast<size_t>(H) * sizeof(float);
    if (vec) {
        auto k = rmsnorm_bwd_kernel<DT, DT == RLK_DTYPE_F32 ? 1 : 8>;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds)) != hipSuccess)
            return rlk_fail(RLK_ERR_LAUNCH, "cannot size the rmsnorm backward LDS");
        hipLaunchKernelGGL(k, dim3(groups), dim3(kNormThreads), lds, stream, x, gain, eps, dout, dx, part,
                           N, H);
    } else {
        auto k = rmsnorm_bwd_kernel<DT, 1>;
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds)) != hipSuccess)
            return rlk_fail(RLK_ERR_LAUNCH, "cannot size the rmsnorm backward LDS");
        hipLaunchKernelGGL(k, dim3(groups), dim3(kNormThreads), lds, stream, x, gain, eps, dout, dx, part,
                           N, H);
    }
    return hipGetLastError() == hipSuccess ? 0 : rlk_fail(RLK_ERR_LAUNCH, "rmsnorm backward launch failed");
}

}  // namespace

int rmsnorm_fwd_enqueue(const void* x, const float* gain, float eps, void* out, float* rstd, int64_t N,
                        int32_t H, int32_t dtype, hipStream_t stream)
{
    const bool vec = vec_ok(x, gain, out, H, dtype);
    switch (dtype) {
        case RLK_DTYPE_BF16: return launch_fwd<RLK_DTYPE_BF16>(x, gain, eps, out, rstd, N, H, vec, stream);
        case RLK_DTYPE_F16: return launch_fwd<RLK_DTYPE_F16>(x, gain, eps, out, rstd, N, H, vec, stream);
        default: return launch_fwd<RLK_DTYPE_F32>(x, gain, eps, out, rstd, N, H, false, stream);
    }
}

size_t rmsnorm_bwd_workspace(int64_t N, int32_t H)
{
    const size_t groups = static_cast<size_t>((N + kNormRowsPerGroup - 1) / kNormRowsPerGroup);
    return groups * static_cast<size_t>(H) * sizeof(float);
}

int rmsnorm_bwd_enqueue(const void* x, const float* gain, float eps, const void* d_out, void* d_x,
                        float* d_gain, int accumulate_gain, void* workspace, int64_t N, int32_t H,
                        int32_t dtype, hipStream_t stream)
{
    float* part = static_cast<float*>(workspace);
    const bool vec = vec_ok(x, d_out, d_x, H, dtype) && (reinterpret_cast<uintptr_t>(gain) & 15) == 0;
    int rc;
    switch (dtype) {
        case RLK_DTYPE_BF16: rc = launch_bwd<RLK_DTYPE_BF16>(x, gain, eps, d_out, d_x, part, N, H, vec, stream); break;
        case RLK_DTYPE_F16: rc = launch_bwd<RLK_DTYPE_F16>(x, gain, eps, d_out, d_x, part, N, H, vec, stream); break;
        default: rc = launch_bwd<RLK_DTYPE_F32>(x, gain, eps, d_out, d_x, part, N, H, false, stream); break;
    }
    if (rc) return rc;
    if (d_gain != nullptr) {
        const int groups = static_cast<int>((N + kNormRowsPerGroup - 1) / kNormRowsPerGroup);
        hipLaunchKernelGGL(rmsnorm_gain_finish_kernel, dim3((H + 255) / 256), dim3(256), 0, stream, part,
                           groups, H, d_gain, accumulate_gain);
        if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "rmsnorm gain launch failed");
    }
    return 0;
}

}  // namespace rlk

using namespace rlk;

namespace {

// Tokens whose normalised rows are held at a time by the fused entry points (64 MiB of 16-bit rows
// at H = 4096; the head runs within 2 % of its large-batch rate on 8192 tokens).
constexpr int64_t kNormBlockTokens = 8192;

inline size_t up256(size_t x) { return (x + 255) / 256 * 256; }
inline size_t elt_bytes(int dtype) { return dtype == RLK_DTYPE_F32 ? 4 : 2; }
inline int64_t block_tokens(int64_t N) { return N < kNormBlockTokens ? N : kNormBlockTokens; }

}  // namespace

extern "C" {

int rlk_rmsnorm_fwd(const void* x, const float* gain, float eps, void* out, float* rstd, int64_t N,
                    int32_t H, int32_t dtype, hipStream_t stream)
{
    if (int rc = check_norm(x, gain, N, H, dtype)) return rc;
    if (!out) return rlk_fail(RLK_ERR_ARG, "null pointer");
    return rmsnorm_fwd_enqueue(x, gain, eps, out, rstd, N, H, dtype, stream);
}

int rlk_rmsnorm_bwd_workspace_bytes(int64_t N, int32_t H, size_t* bytes)
{
    if (!bytes || N <= 0 || H <= 0) return rlk_fail(RLK_ERR_ARG, "bad workspace query");
    *bytes = rmsnorm_bwd_workspace(N, H);
    return 0;
}

int rlk_rmsnorm_bwd(const void* x, const float* gain, float eps, const void* d_out, void* d_x,
                    float* d_gain, void* workspace, size_t workspace_bytes, int64_t N, int32_t H,
                    int32_t dtype, hipStream_t stream)
{
    if (int rc = check_norm(x, gain, N, H, dtype)) return rc;
    if (!d_out || !d_x) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (!workspace || workspace_bytes < rmsnorm_bwd_workspace(N, H))
        return rlk_fail(RLK_ERR_ARG, "workspace too small");
    return rmsnorm_bwd_enqueue(x, gain, eps, d_out, d_x, d_gain, 0, workspace, N, H, dtype, stream);
}

int rlk_linear_logp_rmsnorm_fwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                                size_t* bytes)
{
    if (!bytes || N <= 0 || H <= 0 || V <= 0) return rlk_fail(RLK_ERR_ARG, "bad workspace query");
    const int64_t nb = block_tokens(N);
    size_t fwd = 0;
    if (int rc = rlk_linear_logp_fwd_workspace_bytes(nb, H, V, dtype, &fwd)) return rc;
    *bytes = up256(static_cast<size_t>(nb) * H * elt_bytes(dtype)) + up256(fwd);
    return 0;
}

int rlk_linear_logp_rmsnorm_fwd(const void* x, const float* gain, float eps, const void* weight,
                                const float* bias, const int64_t* targets, float* logp, float* lse,
                                void* workspace, size_t workspace_bytes, int64_t N, int32_t H,
                                int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                                int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                                int32_t* err_flag, hipStream_t stream)
{
    if (int rc = check_norm(x, gain, N, H, dtype)) return rc;
    if (!weight || !targets || !logp || !lse) return rlk_fail(RLK_ERR_ARG, "null pointer");
    size_t need = 0;
    if (int rc = rlk_linear_logp_rmsnorm_fwd_workspace_bytes(N, H, V, dtype, &need)) return rc;
    if (!workspace || workspace_bytes < need) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 255)
        return rlk_fail(RLK_ERR_ARG, "workspace must be 256-byte aligned");
    const int64_t nb = block_tokens(N);
    const size_t es = elt_bytes(dtype);
    char* ws = static_cast<char*>(workspace);
    void* normed = ws;
    void* fwd_ws = ws + up256(static_cast<size_t>(nb) * H * es);
    const size_t fwd_bytes = need - up256(static_cast<size_t>(nb) * H * es);
    for (int64_t t0 = 0; t0 < N; t0 += nb) {
        const int64_t n = N - t0 < nb ? N - t0 : nb;
        const char* xb = static_cast<const char*>(x) + static_cast<size_t>(t0) * H * es;
        if (int rc = rmsnorm_fwd_enqueue(xb, gain, eps, normed, nullptr, n, H, dtype, stream)) return rc;
        if (int rc = rlk_linear_logp_fwd(normed, weight, bias, targets + t0, logp + t0, lse + t0, fwd_ws,
                                         fwd_bytes, n, H, V, vocab_start, dtype, temperature,
                                         ignore_index, use_ignore, strict_targets, err_flag, stream))
            return rc;
    }
    return 0;
}

int rlk_linear_logp_rmsnorm_bwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                                size_t dz_budget_bytes, size_t* bytes)
{
    if (!bytes || N <= 0 || H <= 0 || V <= 0) return rlk_fail(RLK_ERR_ARG, "bad workspace query");
    const int64_t nb = block_tokens(N);
    size_t bwd = 0;
    if (int rc = rlk_linear_logp_bwd_workspace_bytes(nb, H, V, dtype, dz_budget_bytes, &bwd)) return rc;
    // one block of normalised rows (+ 256 bytes so that it can be cut into two aligned halves, see
    // rlk_linear_logp_rmsnorm_bwd); the gradient w.r.t. the normalised rows goes straight into d_x
    const size_t rows = up256(static_cast<size_t>(nb) * H * elt_bytes(dtype)) + 256;
    *bytes = rows + up256(rmsnorm_bwd_workspace(nb, H)) + up256(bwd);
    return 0;
}

int rlk_linear_logp_rmsnorm_bwd(const float* grad_logp, const void* x, const float* gain, float eps,
                                const void* weight, const float* bias, const int64_t* targets,
                                const float* lse, void* d_x, float* d_gain, float* d_weight,
                                float* d_bias, void* workspace, size_t workspace_bytes,
                                size_t dz_budget_bytes, int64_t N, int32_t H, int64_t V,
                                int64_t vocab_start, int32_t dtype, float temperature,
                                int64_t ignore_index, int32_t use_ignore, hipStream_t stream)
{
    if (int rc = check_norm(x, gain, N, H, dtype)) return rc;
    if (!grad_logp || !weight || !targets || !lse) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (!d_x && !d_gain && !d_weight && !d_bias) return rlk_fail(RLK_ERR_ARG, "no gradient requested");
    size_t need = 0;
    if (int rc = rlk_linear_logp_rmsnorm_bwd_workspace_bytes(N, H, V, dtype, dz_budget_bytes, &need)) return rc;
    if (!workspace || workspace_bytes < need) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 255)
        return rlk_fail(RLK_ERR_ARG, "workspace must be 256-byte aligned");
    const size_t es = elt_bytes(dtype);
    const int64_t nb_full = block_tokens(N);
    const size_t rows = up256(static_cast<size_t>(nb_full) * H * es) + 256;
    char* ws = static_cast<char*>(workspace);
    void* gain_ws = ws + rows;
    void* bwd_ws = ws + rows + up256(rmsnorm_bwd_workspace(nb_full, H));
    const size_t bwd_bytes = need - (rows + up256(rmsnorm_bwd_workspace(nb_full, H)));
    const bool need_norm_bwd = d_x != nullptr || d_gain != nullptr;
    // The head's gradient w.r.t. the normalised rows is written into the caller's d_x block and the
    // norm backward then runs on it in place (a thread reads an element of d_out before it writes
    // the same element of d_x, and the row's dot product is complete before the first write).
    // Without d_x (only d_gain wanted) there is no such buffer: the block is halved and the second
    // half of the row region holds that gradient.
    const bool in_place = d_x != nullptr;
    const int64_t nb = (in_place || !need_norm_bwd) ? nb_full : (nb_full + 1) / 2;
    void* normed = ws;
    void* d_half = ws + up256(static_cast<size_t>(nb) * H * es);
    if (!in_place && need_norm_bwd) {
        size_t half_need = 0;
        if (int rc = rlk_linear_logp_bwd_workspace_bytes(nb, H, V, dtype, dz_budget_bytes, &half_need)) return rc;
        if (half_need > bwd_bytes) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    }
    for (int64_t t0 = 0; t0 < N; t0 += nb) {
        const int64_t n = N - t0 < nb ? N - t0 : nb;
        const char* xb = static_cast<const char*>(x) + static_cast<size_t>(t0) * H * es;
        void* dxb = d_x ? static_cast<char*>(d_x) + static_cast<size_t>(t0) * H * es : d_half;
        if (int rc = rmsnorm_fwd_enqueue(xb, gain, eps, normed, nullptr, n, H, dtype, stream)) return rc;
        // dW / db of the first block are written, those of later blocks added on top
        if (int rc = linear_logp_bwd_accumulating(grad_logp + t0, normed, weight, bias, targets + t0,
                                                  lse + t0, need_norm_bwd ? dxb : nullptr,
                                                  d_weight, d_bias, bwd_ws, bwd_bytes, dz_budget_bytes,
                                                  n, H, V, vocab_start, dtype, temperature,
                                                  ignore_index, use_ignore, t0 > 0 ? 1 : 0, stream))
            return rc;
        if (need_norm_bwd) {
            if (int rc = rmsnorm_bwd_enqueue(xb, gain, eps, dxb, dxb, d_gain, t0 > 0 ? 1 : 0, gain_ws,
                                             n, H, dtype, stream))
                return rc;
        }
    }
    return 0;
}

}  // extern "C"
