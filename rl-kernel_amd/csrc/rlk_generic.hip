// Scalar-FMA kernels of the fused linear-logprob path for inputs the MFMA tiles do not take
// (fp32 tensors, hidden sizes that are not a multiple of 8, misaligned matrices).  Same math,
// same fixed reduction order guarantees, fp32 arithmetic throughout; built for correctness on
// small and medium problems, not for roofline performance.
#include "rlk_common.hpp"

namespace rlk {

constexpr int kGT = 256;  // threads per workgroup

template <int DT>
__device__ inline float ld(const void* p, int64_t i)
{
    if (DT == RLK_DTYPE_F32) return static_cast<const float*>(p)[i];
    const uint16_t x = static_cast<const uint16_t*>(p)[i];
    if (DT == RLK_DTYPE_BF16) return __builtin_bit_cast(float, static_cast<uint32_t>(x) << 16);
    return static_cast<float>(__builtin_bit_cast(_Float16, x));
}

template <int DT>
__device__ inline void st(void* p, int64_t i, float v)
{
    if (DT == RLK_DTYPE_F32)
        static_cast<float*>(p)[i] = v;
    else if (DT == RLK_DTYPE_BF16)
        static_cast<uint16_t*>(p)[i] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
    else
        static_cast<uint16_t*>(p)[i] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
}

struct GenArgs {
    const void* hidden;
    const void* weight;
    const float* bias;
    const int64_t* targets;
    const float* lse_in;  // backward: saved natural-log lse
    const float* grad;    // backward: upstream d/dlogp
    float* logp;
    float* lse;
    float* dz;            // backward: [chunk][V] fp32
    int32_t* err_flag;
    int64_t N;            // tokens handled by this launch
    int64_t V;
    int H;
    int64_t vocab_start;
    int64_t ignore_index;
    int use_ignore;
    int strict;
    float inv_t;
};

// One workgroup = TB tokens whose hidden rows sit in LDS; thread t owns vocab rows t, t+256, ...
// MODE 0: forward (online logsumexp + target capture).  MODE 1: write dZ rows for the backward.
template <int DT, int TB, int MODE>
__global__ __launch_bounds__(kGT) void generic_rows_kernel(GenArgs a)
{
    extern __shared__ float hs[];  // [TB][H]
    const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * TB;
    const int t = threadIdx.x;
    for (int i = t; i < TB * a.H; i += kGT) {
        const int tb = i / a.H, k = i % a.H;
        const int64_t tok = tok0 + tb < a.N ? tok0 + tb : a.N - 1;
        hs[i] = ld<DT>(a.hidden, tok * a.H + k);
    }
    __syncthreads();

    float m[TB], s[TB], zt[TB], gs[TB], lsev[TB];
    int64_t tgt[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        m[tb] = -INFINITY;
        s[tb] = 0.f;
        zt[tb] = 0.f;
        const int64_t tok = tok0 + tb < a.N ? tok0 + tb : a.N - 1;
        tgt[tb] = a.targets[tok] - a.vocab_start;
        if (MODE == 1) {
            const bool live = tok0 + tb < a.N && !(a.use_ignore && a.targets[tok] == a.ignore_index);
            gs[tb] = live ? a.grad[tok] * a.inv_t : 0.f;
            lsev[tb] = a.lse_in[tok];
        }
    }

    for (int64_t v = t; v < a.V; v += kGT) {
        float acc[TB];
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) acc[tb] = 0.f;
        for (int k = 0; k < a.H; ++k) {
            const float w = ld<DT>(a.weight, v * a.H + k);
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) acc[tb] = fmaf(w, hs[tb * a.H + k], acc[tb]);
        }
        const float b = a.bias ? a.bias[v] : 0.f;
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            const float z = (acc[tb] + b) * a.inv_t;
            if (MODE == 0) {
                if (z > m[tb]) {
                    s[tb] = s[tb] * expf(m[tb] - z) + 1.f;
                    m[tb] = z;
                } else {
                    s[tb] += expf(z - m[tb]);
                }
                if (v == tgt[tb]) zt[tb] = z;
            } else if (tok0 + tb < a.N) {
                const float p = expf(z - lsev[tb]);
                a.dz[(tok0 + tb) * a.V + v] = gs[tb] * ((v == tgt[tb] ? 1.f : 0.f) - p);
            }
        }
    }
    if (MODE == 1) return;

    // merge the 256 per-thread states of each token in a fixed order
    __shared__ float red[kGT / 64][3];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        float mm = m[tb], ss = s[tb], zz = zt[tb];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float m2 = __shfl_down(mm, o), s2 = __shfl_down(ss, o), z2 = __shfl_down(zz, o);
            const float mx = fmaxf(mm, m2);
            const float mr = mx == -INFINITY ? 0.f : mx;
            ss = ss * expf(mm - mr) + s2 * expf(m2 - mr);
            mm = mx;
            zz += z2;
        }
        __syncthreads();
        if ((t & 63) == 0) {
            red[t >> 6][0] = mm;
            red[t >> 6][1] = ss;
            red[t >> 6][2] = zz;
        }
        __syncthreads();
        if (t == 0 && tok0 + tb < a.N) {
            float mx = -INFINITY;
            for (int w = 0; w < kGT / 64; ++w) mx = fmaxf(mx, red[w][0]);
            const float mr = mx == -INFINITY ? 0.f : mx;
            float sum = 0.f, zsum = 0.f;
            for (int w = 0; w < kGT / 64; ++w) {
                sum += red[w][1] * expf(red[w][0] - mr);
                zsum += red[w][2];
            }
            const float l = mx + logf(sum);
            const int64_t tok = tok0 + tb;
            const int64_t tg = a.targets[tok];
            const bool ignored = a.use_ignore && tg == a.ignore_index;
            const bool owned = tgt[tb] >= 0 && tgt[tb] < a.V;
            if (!ignored && !owned && a.strict) *a.err_flag = 1;
            a.lse[tok] = l;
            a.logp[tok] = ignored ? 0.f : zsum - l;
        }
    }
}

// d_hidden[tok][h] = sum_v dz[tok][v] W[v][h], v ascending.
template <int DT>
__global__ void generic_dh_kernel(const float* dz, const void* weight, void* dh, int64_t ntok, int H,
                                  int64_t V)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= ntok * H) return;
    const int64_t tok = i / H;
    const int h = static_cast<int>(i % H);
    float acc = 0.f;
    for (int64_t v = 0; v < V; ++v) acc = fmaf(dz[tok * V + v], ld<DT>(weight, v * H + h), acc);
    st<DT>(dh, i, acc);
}

// d_weight[v][h] (+)= sum_tok dz[tok][v] hidden[tok][h], tok ascending.
template <int DT>
__global__ void generic_dw_kernel(const float* dz, const void* hidden, float* dw, int64_t ntok, int H,
                                  int64_t V, int accumulate)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= V * H) return;
    const int64_t v = i / H;
    const int h = static_cast<int>(i % H);
    float acc = 0.f;
    for (int64_t tok = 0; tok < ntok; ++tok) acc = fmaf(dz[tok * V + v], ld<DT>(hidden, tok * H + h), acc);
    dw[i] = accumulate ? dw[i] + acc : acc;
}

__global__ void generic_db_kernel(const float* dz, float* db, int64_t ntok, int64_t V, int accumulate)
{
    const int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (v >= V) return;
    float acc = 0.f;
    for (int64_t tok = 0; tok < ntok; ++tok) acc += dz[tok * V + v];
    db[v] = accumulate ? db[v] + acc : acc;
}

namespace {

int pick_tb(int H)
{
    int tb = 8;
    while (tb > 1 && static_cast<int64_t>(tb) * H > 12288) tb >>= 1;
    return tb;
}

template <int DT, int MODE>
int launch_rows(const GenArgs& a, int tb, hipStream_t stream)
{
    const size_t smem = static_cast<size_t>(tb) * a.H * sizeof(float);
    const dim3 grid(static_cast<unsigned>((a.N + tb - 1) / tb)), block(kGT);
    switch (tb) {
        case 8: hipLaunchKernelGGL((generic_rows_kernel<DT, 8, MODE>), grid, block, smem, stream, a); break;
        case 4: hipLaunchKernelGGL((generic_rows_kernel<DT, 4, MODE>), grid, block, smem, stream, a); break;
        case 2: hipLaunchKernelGGL((generic_rows_kernel<DT, 2, MODE>), grid, block, smem, stream, a); break;
        default: hipLaunchKernelGGL((generic_rows_kernel<DT, 1, MODE>), grid, block, smem, stream, a); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : rlk_fail(RLK_ERR_LAUNCH, "generic kernel launch failed");
}

template <int MODE>
int launch_rows_dt(const GenArgs& a, int dtype, int tb, hipStream_t stream)
{
    if (dtype == RLK_DTYPE_F32) return launch_rows<RLK_DTYPE_F32, MODE>(a, tb, stream);
    if (dtype == RLK_DTYPE_BF16) return launch_rows<RLK_DTYPE_BF16, MODE>(a, tb, stream);
    return launch_rows<RLK_DTYPE_F16, MODE>(a, tb, stream);
}

int64_t bwd_chunk(int64_t N, int64_t V)
{
    int64_t c = (static_cast<int64_t>(1) << 24) / V;  // at most 64 MiB of fp32 dZ
    if (c < 1) c = 1;
    return c < N ? c : N;
}

}  // namespace

int generic_fwd(const void* hidden, const void* weight, const float* bias, const int64_t* targets,
                float* logp, float* lse, int64_t N, int32_t H, int64_t V, int64_t vocab_start,
                int32_t dtype, float temperature, int64_t ignore_index, int32_t use_ignore,
                int32_t strict_targets, int32_t* err_flag, hipStream_t stream)
{
    if (H > 12288) return rlk_fail(RLK_ERR_UNSUPPORTED, "scalar path supports H <= 12288");
    GenArgs a{};
    a.hidden = hidden;
    a.weight = weight;
    a.bias = bias;
    a.targets = targets;
    a.logp = logp;
    a.lse = lse;
    a.err_flag = err_flag;
    a.N = N;
    a.V = V;
    a.H = H;
    a.vocab_start = vocab_start;
    a.ignore_index = ignore_index;
    a.use_ignore = use_ignore;
    a.strict = strict_targets;
    a.inv_t = 1.f / temperature;
    return launch_rows_dt<0>(a, dtype, pick_tb(H), stream);
}

size_t generic_bwd_workspace(int64_t N, int32_t H, int64_t V)
{
    (void)H;
    return static_cast<size_t>(bwd_chunk(N, V)) * V * sizeof(float);
}

int generic_bwd(const float* grad_logp, const void* hidden, const void* weight, const float* bias,
                const int64_t* targets, const float* lse, void* d_hidden, float* d_weight,
                float* d_bias, void* workspace, int64_t N, int32_t H, int64_t V,
                int64_t vocab_start, int32_t dtype, float temperature, int64_t ignore_index,
                int32_t use_ignore, hipStream_t stream)
{
    if (H > 12288) return rlk_fail(RLK_ERR_UNSUPPORTED, "scalar path supports H <= 12288");
    const int64_t chunk = bwd_chunk(N, V);
    const size_t esz = dtype == RLK_DTYPE_F32 ? 4 : 2;
    float* dz = static_cast<float*>(workspace);
    for (int64_t t0 = 0; t0 < N; t0 += chunk) {
        const int64_t nt = (N - t0) < chunk ? (N - t0) : chunk;
        GenArgs a{};
        a.hidden = static_cast<const char*>(hidden) + t0 * H * esz;
        a.weight = weight;
        a.bias = bias;
        a.targets = targets + t0;
        a.lse_in = lse + t0;
        a.grad = grad_logp + t0;
        a.dz = dz;
        a.N = nt;
        a.V = V;
        a.H = H;
        a.vocab_start = vocab_start;
        a.ignore_index = ignore_index;
        a.use_ignore = use_ignore;
        a.inv_t = 1.f / temperature;
        if (int rc = launch_rows_dt<1>(a, dtype, pick_tb(H), stream)) return rc;
        const unsigned gh = static_cast<unsigned>((nt * H + 255) / 256);
        const unsigned gw = static_cast<unsigned>((V * H + 255) / 256);
        void* dh = d_hidden ? static_cast<char*>(d_hidden) + t0 * H * esz : nullptr;
        const int acc = t0 > 0;
        if (dtype == RLK_DTYPE_F32) {
            if (dh) hipLaunchKernelGGL(generic_dh_kernel<RLK_DTYPE_F32>, dim3(gh), dim3(256), 0, stream, dz, weight, dh, nt, H, V);
            if (d_weight) hipLaunchKernelGGL(generic_dw_kernel<RLK_DTYPE_F32>, dim3(gw), dim3(256), 0, stream, dz, a.hidden, d_weight, nt, H, V, acc);
        } else if (dtype == RLK_DTYPE_BF16) {
            if (dh) hipLaunchKernelGGL(generic_dh_kernel<RLK_DTYPE_BF16>, dim3(gh), dim3(256), 0, stream, dz, weight, dh, nt, H, V);
            if (d_weight) hipLaunchKernelGGL(generic_dw_kernel<RLK_DTYPE_BF16>, dim3(gw), dim3(256), 0, stream, dz, a.hidden, d_weight, nt, H, V, acc);
        } else {
            if (dh) hipLaunchKernelGGL(generic_dh_kernel<RLK_DTYPE_F16>, dim3(gh), dim3(256), 0, stream, dz, weight, dh, nt, H, V);
            if (d_weight) hipLaunchKernelGGL(generic_dw_kernel<RLK_DTYPE_F16>, dim3(gw), dim3(256), 0, stream, dz, a.hidden, d_weight, nt, H, V, acc);
        }
        if (d_bias)
            hipLaunchKernelGGL(generic_db_kernel, dim3(static_cast<unsigned>((V + 255) / 256)), dim3(256), 0, stream, dz, d_bias, nt, V, acc);
        if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "generic backward launch failed");
    }
    return 0;
}

}  // namespace rlk
