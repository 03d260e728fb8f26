// Selected-token log-prob from materialised logits (the `fused_logp` family): one workgroup
// scans one row once with 16-byte loads, keeping a per-thread running (max, sum) that is merged
// in a fixed tree order, then thread 0 gathers the target logit.  HBM-bound: N*V*elt bytes.
#include "rlk_common.hpp"

namespace rlk {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

struct LseState {
    float m;  // running max
    float s;  // running sum of exp(x - m)
};

__device__ inline void lse_push(LseState& st, float x)
{
    if (x == -INFINITY) return;  // a masked logit contributes nothing
    if (x <= st.m) {
        st.s += __expf(x - st.m);
    } else {
        st.s = st.s * __expf(st.m - x) + 1.f;
        st.m = x;
    }
}

__device__ inline LseState lse_merge(LseState a, LseState b)
{
    if (a.s == 0.f) return b;
    if (b.s == 0.f) return a;
    if (a.m >= b.m) return {a.m, a.s + b.s * __expf(b.m - a.m)};
    return {b.m, b.s + a.s * __expf(a.m - b.m)};
}

template <int DT>
struct Elem;
template <>
struct Elem<RLK_DTYPE_BF16> {
    using type = uint16_t;
    __device__ static float get(uint16_t x) { return __builtin_bit_cast(float, static_cast<uint32_t>(x) << 16); }
};
template <>
struct Elem<RLK_DTYPE_F16> {
    using type = uint16_t;
    __device__ static float get(uint16_t x) { return static_cast<float>(__builtin_bit_cast(_Float16, x)); }
};
template <>
struct Elem<RLK_DTYPE_F32> {
    using type = float;
    __device__ static float get(float x) { return x; }
};

__device__ inline void store_out(void* out, int dtype, int64_t i, float v)
{
    switch (dtype) {
        case RLK_DTYPE_F32: static_cast<float*>(out)[i] = v; break;
        case RLK_DTYPE_F64: static_cast<double*>(out)[i] = static_cast<double>(v); break;
        case RLK_DTYPE_BF16:
            static_cast<uint16_t*>(out)[i] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
            break;
        default:
            static_cast<uint16_t*>(out)[i] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
            break;
    }
}

constexpr int kScanThreads = 256;

// Second logits tensor of a pair launch (grid.y == 2): same ids and rows, own outputs.
struct ScanSecond {
    const void* logits;
    void* out;
    float* lse_out;
};

template <int DT>
__global__ __launch_bounds__(kScanThreads) void logp_scan_kernel(
    const void* __restrict__ logits_v, const int64_t* __restrict__ ids, void* __restrict__ out,
    int out_dtype, float* __restrict__ lse_out, const int64_t* __restrict__ row_indices,
    int64_t n_rows, int64_t vocab, ScanSecond second)
{
    if (blockIdx.y == 1) {  // uniform
        logits_v = second.logits;
        out = second.out;
        lse_out = second.lse_out;
    }
    using E = typename Elem<DT>::type;
    constexpr int kPer = 16 / sizeof(E);  // elements per 16-byte load
    const int64_t row = row_indices ? row_indices[blockIdx.x] : static_cast<int64_t>(blockIdx.x);
    if (row < 0 || row >= n_rows) return;  // uniform: rows outside the tensor are skipped
    const E* x = static_cast<const E*>(logits_v) + row * vocab;
    const int t = threadIdx.x;

    // [0, head) scalar until 16-byte aligned, [head, head + nvec*kPer) vector, rest scalar
    const uintptr_t addr = reinterpret_cast<uintptr_t>(x);
    int64_t head = ((16 - (addr & 15)) & 15) / sizeof(E);
    if (head > vocab) head = vocab;
    const int64_t nvec = (vocab - head) / kPer;
    const int64_t tail0 = head + nvec * kPer;

    LseState st{-INFINITY, 0.f};
    if (t < head) lse_push(st, Elem<DT>::get(x[t]));
    const u32x4* xv = reinterpret_cast<const u32x4*>(x + head);
    // Main scan in the log2 domain: (m2, s2) = running max of x*log2(e) and sum of 2^(x*log2e - m2).
    // kUnroll 16-byte loads are in flight per thread; a vector first raises the max (one rescale
    // per vector at most), then adds its terms without branches.  -inf logits add exactly 0.
    constexpr int kUnroll = 4;
    constexpr float kL2e = 1.4426950408889634f;
    float m2 = -INFINITY, s2 = 0.f;
    auto absorb = [&](const u32x4& v) {
        const E* e = reinterpret_cast<const E*>(&v);
        float f[kPer];
        float vmax = m2;
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            f[k] = Elem<DT>::get(e[k]) * kL2e;
            vmax = fmaxf(vmax, f[k]);
        }
        if (vmax > m2) {
            s2 *= __builtin_amdgcn_exp2f(m2 - vmax);  // m2 = -inf: s2 is 0 and stays 0
            m2 = vmax;
        }
        const float ref = m2 == -INFINITY ? 0.f : m2;
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int k = 0; k < kPer; k += 2) {
            acc0 += __builtin_amdgcn_exp2f(f[k] - ref);
            acc1 += __builtin_amdgcn_exp2f(f[k + 1] - ref);
        }
        s2 += acc0 + acc1;
    };
    int64_t i = t;
    for (; i + (kUnroll - 1) * kScanThreads < nvec; i += kUnroll * kScanThreads) {
        u32x4 v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(xv + i + u * kScanThreads);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) absorb(v[u]);
    }
    for (; i < nvec; i += kScanThreads) absorb(xv[i]);
    if (s2 > 0.f) st = lse_merge(st, LseState{m2 * 0.6931471805599453f, s2});
    if (tail0 + t < vocab) lse_push(st, Elem<DT>::get(x[tail0 + t]));

    // fixed-order tree: lanes inside the wavefront, then the wavefronts through LDS
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        LseState other{__shfl_down(st.m, o), __shfl_down(st.s, o)};
        st = lse_merge(st, other);
    }
    __shared__ float sm[kScanThreads / 64], ss[kScanThreads / 64];
    if ((t & 63) == 0) {
        sm[t >> 6] = st.m;
        ss[t >> 6] = st.s;
    }
    __syncthreads();
    if (t == 0) {
        LseState all{sm[0], ss[0]};
#pragma unroll
        for (int w = 1; w < kScanThreads / 64; ++w) all = lse_merge(all, LseState{sm[w], ss[w]});
        const int64_t id = ids[row];
        const float lse = all.m + logf(all.s);
        float r = 0.f;  // a target outside [0, V) yields 0, not an error
        if (id >= 0 && id < vocab) r = Elem<DT>::get(x[id]) - lse;
        store_out(out, out_dtype, row, r);
        if (lse_out) lse_out[row] = lse;
    }
}

// grad_logits[n][v] = coeff[n] * (onehot(ids[n])[v] - exp(logits[n][v] - lse[n])); rows whose id
// is outside [0, V) (the forward returned 0 for them) get a zero gradient.
template <int DT>
__global__ __launch_bounds__(kScanThreads) void logp_scan_bwd_kernel(
    const void* __restrict__ logits_v, const int64_t* __restrict__ ids,
    const float* __restrict__ lse, const float* __restrict__ coeff, void* __restrict__ grad_v,
    int64_t vocab)
{
    using E = typename Elem<DT>::type;
    const int64_t row = blockIdx.x;
    const E* x = static_cast<const E*>(logits_v) + row * vocab;
    E* g = static_cast<E*>(grad_v) + row * vocab;
    const int64_t id = ids[row];
    const bool live = id >= 0 && id < vocab;
    const float c = live ? coeff[row] : 0.f;
    const float l = lse[row];
    auto value = [&](int64_t v, E xe) -> E {
        const float p = __expf(Elem<DT>::get(xe) - l);
        float d = c * ((v == id ? 1.f : 0.f) - p);
        if (c == 0.f) d = 0.f;
        if constexpr (DT == RLK_DTYPE_F32)
            return d;
        else if constexpr (DT == RLK_DTYPE_BF16)
            return __builtin_bit_cast(uint16_t, static_cast<__bf16>(d));
        else
            return __builtin_bit_cast(uint16_t, static_cast<_Float16>(d));
    };
    // rows of logits and gradient share their alignment when both bases are 16-byte aligned (the
    // usual case): scalar head up to the first aligned element, 16-byte body, scalar tail
    constexpr int kPer = 16 / sizeof(E);
    const int t = threadIdx.x;
    const uintptr_t ax = reinterpret_cast<uintptr_t>(x), ag = reinterpret_cast<uintptr_t>(g);
    int64_t head = ((16 - (ax & 15)) & 15) / sizeof(E);
    if ((ax & 15) != (ag & 15) || head > vocab) head = vocab;  // misaligned pair: all scalar
    const int64_t nvec = (vocab - head) / kPer;
    const int64_t tail0 = head + nvec * kPer;
    for (int64_t v = t; v < head; v += kScanThreads) g[v] = value(v, x[v]);
    const u32x4* xv = reinterpret_cast<const u32x4*>(x + head);
    u32x4* gv = reinterpret_cast<u32x4*>(g + head);
    for (int64_t i = t; i < nvec; i += kScanThreads) {
        const u32x4 in = __builtin_nontemporal_load(xv + i);
        u32x4 o;
        const E* e = reinterpret_cast<const E*>(&in);
        E* r = reinterpret_cast<E*>(&o);
#pragma unroll
        for (int k = 0; k < kPer; ++k) r[k] = value(head + i * kPer + k, e[k]);
        gv[i] = o;
    }
    for (int64_t v = tail0 + t; v < vocab; v += kScanThreads) g[v] = value(v, x[v]);
}

}  // namespace rlk

using namespace rlk;

extern "C" int rlk_logp_from_logits_bwd(const void* logits, int32_t logits_dtype, const int64_t* ids,
                                        const float* lse, const float* coeff, void* grad_logits,
                                        int64_t n_rows, int64_t vocab, hipStream_t stream)
{
    if (!logits || !ids || !lse || !coeff || !grad_logits) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (n_rows < 0 || vocab <= 0 || n_rows > 0x7fffffffLL) return rlk_fail(RLK_ERR_ARG, "bad sizes");
    if (n_rows == 0) return 0;
    const dim3 grid(static_cast<unsigned>(n_rows)), block(kScanThreads);
    switch (logits_dtype) {
        case RLK_DTYPE_BF16:
            hipLaunchKernelGGL(logp_scan_bwd_kernel<RLK_DTYPE_BF16>, grid, block, 0, stream, logits,
                               ids, lse, coeff, grad_logits, vocab);
            break;
        case RLK_DTYPE_F16:
            hipLaunchKernelGGL(logp_scan_bwd_kernel<RLK_DTYPE_F16>, grid, block, 0, stream, logits,
                               ids, lse, coeff, grad_logits, vocab);
            break;
        case RLK_DTYPE_F32:
            hipLaunchKernelGGL(logp_scan_bwd_kernel<RLK_DTYPE_F32>, grid, block, 0, stream, logits,
                               ids, lse, coeff, grad_logits, vocab);
            break;
        default:
            return rlk_fail(RLK_ERR_UNSUPPORTED, "logits dtype must be bf16, f16 or f32");
    }
    if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "logp backward launch failed");
    return 0;
}


namespace {

int scan_enqueue(const void* logits, int32_t logits_dtype, const int64_t* ids, void* out,
                 int32_t out_dtype, float* lse_out, const int64_t* row_indices, int64_t n_launch,
                 int64_t n_rows, int64_t vocab, const rlk::ScanSecond* second, hipStream_t stream)
{
    using namespace rlk;
    if (!logits || !ids || !out) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (n_rows < 0 || vocab <= 0 || n_launch < 0) return rlk_fail(RLK_ERR_ARG, "bad sizes");
    if (n_launch > 0x7fffffffLL) return rlk_fail(RLK_ERR_ARG, "too many rows for one launch");
    if (out_dtype < RLK_DTYPE_BF16 || out_dtype > RLK_DTYPE_F64)
        return rlk_fail(RLK_ERR_UNSUPPORTED, "output dtype must be bf16, f16, f32 or f64");
    if (n_launch == 0 || n_rows == 0) return 0;
    const dim3 grid(static_cast<unsigned>(n_launch), second ? 2u : 1u), block(kScanThreads);
    const ScanSecond s2 = second ? *second : ScanSecond{nullptr, nullptr, nullptr};
    switch (logits_dtype) {
        case RLK_DTYPE_BF16:
            hipLaunchKernelGGL(logp_scan_kernel<RLK_DTYPE_BF16>, grid, block, 0, stream, logits, ids,
                               out, out_dtype, lse_out, row_indices, n_rows, vocab, s2);
            break;
        case RLK_DTYPE_F16:
            hipLaunchKernelGGL(logp_scan_kernel<RLK_DTYPE_F16>, grid, block, 0, stream, logits, ids,
                               out, out_dtype, lse_out, row_indices, n_rows, vocab, s2);
            break;
        case RLK_DTYPE_F32:
            hipLaunchKernelGGL(logp_scan_kernel<RLK_DTYPE_F32>, grid, block, 0, stream, logits, ids,
                               out, out_dtype, lse_out, row_indices, n_rows, vocab, s2);
            break;
        default:
            return rlk_fail(RLK_ERR_UNSUPPORTED, "logits dtype must be bf16, f16 or f32");
    }
    if (hipGetLastError() != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, "logp scan launch failed");
    return 0;
}

}  // namespace

extern "C" int rlk_logp_from_logits(const void* logits, int32_t logits_dtype, const int64_t* ids,
                                    void* out, int32_t out_dtype, float* lse_out,
                                    const int64_t* row_indices, int64_t n_launch, int64_t n_rows,
                                    int64_t vocab, hipStream_t stream)
{
    return scan_enqueue(logits, logits_dtype, ids, out, out_dtype, lse_out, row_indices, n_launch,
                        n_rows, vocab, nullptr, stream);
}

extern "C" int rlk_logp_from_logits_pair(const void* logits, const void* ref_logits,
                                         int32_t logits_dtype, const int64_t* ids, void* out,
                                         void* ref_out, int32_t out_dtype, float* lse_out,
                                         float* ref_lse_out, const int64_t* row_indices,
                                         int64_t n_launch, int64_t n_rows, int64_t vocab,
                                         hipStream_t stream)
{
    if (!ref_logits || !ref_out) return rlk_fail(RLK_ERR_ARG, "null pointer");
    const rlk::ScanSecond second{ref_logits, ref_out, ref_lse_out};
    return scan_enqueue(logits, logits_dtype, ids, out, out_dtype, lse_out, row_indices, n_launch,
                        n_rows, vocab, &second, stream);
}
