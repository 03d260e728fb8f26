// fp32 matrix-core kernels of the fused linear-logprob path for inputs the 16-bit MFMA tiles do
// not take: fp32 tensors, hidden sizes that are not a multiple of 8, matrices that do not start on
// a 16-byte boundary.  Every operand is widened to fp32 on its way into LDS (exact for bf16 and
// f16) and multiplied with v_mfma_f32_32x32x2_f32, so products and sums are plain fp32 and the
// results follow the reference's fp32 arithmetic.  Same workgroup tile (256 x 256, 2 x 4
// wavefronts), same accumulator layout and same split / combine structure as the 16-bit kernels;
// dZ stays fp32.  All loads are clamped or masked element by element, so any N, H, V >= 1 and any
// element alignment is accepted.  All reductions run in a fixed order: same input, same bits.
#include "rlk_common.hpp"

#include "rlk_gemm.hpp"
#include "rlk_tile_epilogue.hpp"

namespace rlk {

namespace {

constexpr int kWBK = 16;  // K elements per LDS stage

// Element access of the three input types, widened to fp32.
template <int DT>
struct WideElem;

template <>
struct WideElem<RLK_DTYPE_F32> {
    static constexpr int kBytes = 4;
    __device__ static inline float get(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
    __device__ static inline f32x4_t get4(const void* p, int64_t i)
    {
        return *reinterpret_cast<const f32x4_t*>(static_cast<const float*>(p) + i);
    }
    __device__ static inline void put(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
    __device__ static inline void put4(void* p, int64_t i, f32x4_t v)
    {
        *reinterpret_cast<f32x4_t*>(static_cast<float*>(p) + i) = v;
    }
};

template <>
struct WideElem<RLK_DTYPE_BF16> {
    static constexpr int kBytes = 2;
    __device__ static inline float get(const void* p, int64_t i)
    {
        return Bf16::to_float(static_cast<const uint16_t*>(p)[i]);
    }
    __device__ static inline f32x4_t get4(const void* p, int64_t i)
    {
        const u32x2_t w = *reinterpret_cast<const u32x2_t*>(static_cast<const uint16_t*>(p) + i);
        return f32x4_t{__builtin_bit_cast(float, w.x << 16), __builtin_bit_cast(float, w.x & 0xffff0000u),
                       __builtin_bit_cast(float, w.y << 16), __builtin_bit_cast(float, w.y & 0xffff0000u)};
    }
    __device__ static inline void put(void* p, int64_t i, float v)
    {
        static_cast<uint16_t*>(p)[i] = Bf16::from_float(v);
    }
    __device__ static inline void put4(void* p, int64_t i, f32x4_t v)
    {
        *reinterpret_cast<u32x2_t*>(static_cast<uint16_t*>(p) + i) =
            u32x2_t{Bf16::pack2(v.x, v.y), Bf16::pack2(v.z, v.w)};
    }
};

template <>
struct WideElem<RLK_DTYPE_F16> {
    static constexpr int kBytes = 2;
    __device__ static inline float get(const void* p, int64_t i)
    {
        return F16::to_float(static_cast<const uint16_t*>(p)[i]);
    }
    __device__ static inline f32x4_t get4(const void* p, int64_t i)
    {
        const u32x2_t w = *reinterpret_cast<const u32x2_t*>(static_cast<const uint16_t*>(p) + i);
        return f32x4_t{F16::to_float(static_cast<uint16_t>(w.x)), F16::to_float(static_cast<uint16_t>(w.x >> 16)),
                       F16::to_float(static_cast<uint16_t>(w.y)), F16::to_float(static_cast<uint16_t>(w.y >> 16))};
    }
    __device__ static inline void put(void* p, int64_t i, float v)
    {
        static_cast<uint16_t*>(p)[i] = F16::from_float(v);
    }
    __device__ static inline void put4(void* p, int64_t i, f32x4_t v)
    {
        *reinterpret_cast<u32x2_t*>(static_cast<uint16_t*>(p) + i) =
            u32x2_t{F16::pack2(v.x, v.y), F16::pack2(v.z, v.w)};
    }
};

// Operand of one workgroup tile.  `vec`: every group of four consecutive elements along the
// contiguous direction that starts at a multiple of four from `base` is 4-element aligned and may
// be fetched with one load (the leading dimension is a multiple of four and so is the origin).
struct WideOperand {
    const void* base;  // element (row 0, k 0) of the tile
    int64_t ld;        // elements between consecutive memory lines
    int rows;          // valid tile rows from the origin (>= 1)
    bool vec;
};

// One operand's way from global memory into an LDS stage and from there into MFMA fragments.
//   K-contiguous (memory [row][k]):  LDS [256 rows][16 k + 4 pad] floats
//   K-major      (memory [k][row]):  LDS [16 k][256 rows + 4 pad] floats
// The pads make the fragment reads below conflict-free.  A thread moves two groups of four
// consecutive elements per K step.  Rows past `rows` repeat the last valid row (finite values
// that no epilogue stores); elements at k >= K are zeros.
template <int DT, bool KMAJOR>
struct WideIO {
    static constexpr int kPitch = KMAJOR ? 260 : 20;  // floats
    static constexpr int kFloats = KMAJOR ? kWBK * 260 : 256 * 20;
    static constexpr int kBytes = kFloats * 4;
    using E = WideElem<DT>;

    const void* base;
    int64_t off[2];  // element offset of this thread's groups at K step 0 (clamped rows)
    int64_t step;    // element advance per K step
    int rows, K;
    bool vec;

    // FAST (see fast_ok): every group is one aligned 4-element load, no per-element checks.
    static __device__ inline bool fast_ok(const WideOperand& op, int K_)
    {
        return op.vec && K_ % kWBK == 0 && (!KMAJOR || (op.rows & 3) == 0);
    }

    __device__ inline void init(const WideOperand& op, int K_, bool fast)
    {
        base = op.base;
        rows = op.rows;
        K = K_;
        vec = op.vec;
        step = KMAJOR ? static_cast<int64_t>(kWBK) * op.ld : kWBK;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int idx = g * kThreads + static_cast<int>(threadIdx.x);
            if (KMAJOR) {
                const int line = idx >> 6, r = (idx & 63) * 4;
                // past the valid rows: the last valid element, or (FAST) the last valid group
                const int last = fast ? rows - 4 : rows - 1;
                off[g] = static_cast<int64_t>(line) * op.ld + (r < rows ? r : last);
            } else {
                const int row = idx >> 2, k = (idx & 3) * 4;
                off[g] = static_cast<int64_t>(row < rows ? row : rows - 1) * op.ld + k;
            }
        }
    }

    template <bool FAST>
    __device__ inline f32x4_t load(int kt, int g) const
    {
        if (FAST) return E::get4(base, off[g] + kt * step);
        const int idx = g * kThreads + static_cast<int>(threadIdx.x);
        f32x4_t v{0.f, 0.f, 0.f, 0.f};
        if (KMAJOR) {
            const int k = kt * kWBK + (idx >> 6);
            const int r = (idx & 63) * 4;
            if (k < K) {
                const int64_t o = off[g] + kt * step;  // points at min(r, rows - 1) of line k
                if (vec && r + 3 < rows) {
                    v = E::get4(base, o);
                } else {
                    const int64_t line0 = o - (r < rows ? r : rows - 1);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = E::get(base, line0 + (r + e < rows ? r + e : rows - 1));
                }
            }
        } else {
            const int k = kt * kWBK + (idx & 3) * 4;
            const int64_t o = off[g] + kt * step;
            if (vec && k + 3 < K) {
                v = E::get4(base, o);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (k + e < K) v[e] = E::get(base, o + e);
            }
        }
        return v;
    }

    __device__ static inline void store(float* lds, f32x4_t v, int g)
    {
        const int idx = g * kThreads + static_cast<int>(threadIdx.x);
        const int at = KMAJOR ? (idx >> 6) * kPitch + (idx & 63) * 4 : (idx >> 2) * kPitch + (idx & 3) * 4;
        *reinterpret_cast<f32x4_t*>(lds + at) = v;
    }

    // Half fragment (half = 0, 1) of the 32 tile rows from row0 on: lane l gets row (row0 + l % 32),
    // elements k = 8 * (l / 32) + 4 * half + 0..3 of the stage.  MFMA number j of the stage multiplies
    // element j of the A and B fragments: across the two half-waves that is k = j and k = 8 + j, the
    // same pairing on both operands, so the eight MFMAs together cover the 16 k of the stage once.
    __device__ static inline f32x4_t frag(const float* lds, int row0, int half)
    {
        const int l = threadIdx.x & 63;
        if (KMAJOR) {
            const float* p = lds + (8 * (l >> 5) + 4 * half) * kPitch + row0 + (l & 31);
            return f32x4_t{p[0], p[kPitch], p[2 * kPitch], p[3 * kPitch]};
        } else {
            return *reinterpret_cast<const f32x4_t*>(lds + (row0 + (l & 31)) * kPitch + 8 * (l >> 5) + 4 * half);
        }
    }
};

// Workgroup tile contraction on the fp32 matrix instruction: acc[i][j] += A rows x B rows over
// k in [0, K).  Two LDS stages and one barrier per stage, placed in the middle of the stage's
// MFMAs so that every memory latency has matrix work in front of it:
//   stage kt:  LDS stores of stage kt+1 (fetched one stage ago), global loads of stage kt+2,
//              fragment reads of the second half, 32 MFMAs of the first half,
//              barrier (stage kt+1 is now complete, nobody reads stage kt from LDS any more),
//              fragment reads of the first half of stage kt+1, 32 MFMAs of the second half.
// One MFMA of 32 x 32 x 2 takes 16 passes, so a stage is 4096 matrix cycles per wavefront against a
// dozen fragment reads and 4 global loads: the loop is bound by the matrix pipe.
// All 512 threads must call it (it barriers); on return LDS may be reused.
template <int DTA, int DTB, bool A_KMAJOR, bool B_KMAJOR>
struct WideGemm {
    using IOA = WideIO<DTA, A_KMAJOR>;
    using IOB = WideIO<DTB, B_KMAJOR>;
    static constexpr int kStageFloats = IOA::kFloats + IOB::kFloats;
    static constexpr int kSmemBytes = 2 * kStageFloats * 4;

    __device__ static inline void frags(const float* stage, int wm, int wn, int half, f32x4_t (&fa)[kTM],
                                        f32x4_t (&fb)[kTN])
    {
#pragma unroll
        for (int i = 0; i < kTM; ++i) fa[i] = IOA::frag(stage, wm * (kTM * 32) + i * 32, half);
#pragma unroll
        for (int j = 0; j < kTN; ++j) fb[j] = IOB::frag(stage + IOA::kFloats, wn * (kTN * 32) + j * 32, half);
    }

    __device__ static inline void multiply(const f32x4_t (&fa)[kTM], const f32x4_t (&fb)[kTN],
                                           f32x16_t (&acc)[kTM][kTN])
    {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int i = 0; i < kTM; ++i)
#pragma unroll
                for (int j = 0; j < kTN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][kk], fb[j][kk], acc[i][j], 0, 0, 0);
    }

    __device__ static inline void run(const WideOperand& A, const WideOperand& B, int K,
                                      f32x16_t (&acc)[kTM][kTN], char* smem_c)
    {
        if (IOA::fast_ok(A, K) && IOB::fast_ok(B, K))  // uniform
            run_impl<true>(A, B, K, acc, smem_c);
        else
            run_impl<false>(A, B, K, acc, smem_c);
    }

    template <bool FAST>
    __device__ static inline void run_impl(const WideOperand& A, const WideOperand& B, int K,
                                           f32x16_t (&acc)[kTM][kTN], char* smem_c)
    {
        float* smem = reinterpret_cast<float*>(smem_c);
        IOA la;
        IOB lb;
        la.init(A, K, FAST);
        lb.init(B, K, FAST);
        const int wave = threadIdx.x >> 6;
        const int wm = wave / kWN, wn = wave % kWN;
        const int nk = (K + kWBK - 1) / kWBK;
        f32x4_t ra[2], rb[2];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            ra[g] = la.template load<FAST>(0, g);
            rb[g] = lb.template load<FAST>(0, g);
        }
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            IOA::store(smem, ra[g], g);
            IOB::store(smem + IOA::kFloats, rb[g], g);
        }
        if (nk > 1) {  // uniform
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                ra[g] = la.template load<FAST>(1, g);
                rb[g] = lb.template load<FAST>(1, g);
            }
        }
        __syncthreads();
        f32x4_t fa0[kTM], fb0[kTN], fa1[kTM], fb1[kTN];
        frags(smem, wm, wn, 0, fa0, fb0);
        for (int kt = 0; kt < nk; ++kt) {
            const float* cur = smem + (kt & 1) * kStageFloats;
            float* nxt = smem + ((kt + 1) & 1) * kStageFloats;
            const bool more = kt + 1 < nk;  // uniform
            if (more) {
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    IOA::store(nxt, ra[g], g);
                    IOB::store(nxt + IOA::kFloats, rb[g], g);
                }
            }
            if (kt + 2 < nk) {
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    ra[g] = la.template load<FAST>(kt + 2, g);
                    rb[g] = lb.template load<FAST>(kt + 2, g);
                }
            }
            frags(cur, wm, wn, 1, fa1, fb1);
            multiply(fa0, fb0, acc);
            __syncthreads();
            if (more) frags(nxt, wm, wn, 0, fa0, fb0);
            multiply(fa1, fb1, acc);
        }
        __syncthreads();
    }
};

// ------------------------------------------------------------------------------------------- //
// Forward: partial softmax states of one (256-token block) x (range of vocab tiles)
// ------------------------------------------------------------------------------------------- //
struct WideFwdArgs {
    const void* hidden;  // [N][H]
    const void* weight;  // [V][H]
    const float* bias;   // [V] or null
    const int64_t* targets;
    float* part_m;       // [n_split][N]  running max (log2 domain)
    float* part_s;       // [n_split][N]  running sum of 2^(z - max)
    float* part_z;       // [n_split][N]  captured target logit (log2 domain), 0 if not owned
    int N;
    int H;
    int V;
    int64_t vocab_start;
    int n_split;
    int row_blocks;
    int vtiles;
    float scale2;  // log2(e) / temperature
    bool vec_h, vec_w;
};

template <int DT>
__global__ __launch_bounds__(kThreads) void wide_fwd_kernel(WideFwdArgs a)
{
    using Gemm = WideGemm<DT, DT, false, false>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    int tb, sp;
    xcd_tile(blockIdx.x, a.row_blocks * a.n_split, a.row_blocks, a.n_split, 8, tb, sp);
    const int base = a.vtiles / a.n_split, extra = a.vtiles % a.n_split;
    const int t0 = sp * base + (sp < extra ? sp : extra);
    const int t1 = t0 + base + (sp < extra ? 1 : 0);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int tok0 = tb * 256;
    const int tok_valid = min(256, a.N - tok0);

    float m[kTN], s[kTN], zt[kTN];
    int tgt[kTN];  // target id relative to the shard, -1 when not in [0, V)
#pragma unroll
    for (int j = 0; j < kTN; ++j) {
        const int t = wn * (kTN * 32) + j * 32 + (lane & 31);
        const int64_t g = a.targets[tok0 + (t < tok_valid ? t : tok_valid - 1)] - a.vocab_start;
        tgt[j] = (g >= 0 && g < a.V) ? static_cast<int>(g) : -1;
        m[j] = -INFINITY;
        s[j] = 0.f;
        zt[j] = 0.f;
    }
    const WideOperand B{static_cast<const char*>(a.hidden) +
                            static_cast<int64_t>(tok0) * a.H * WideElem<DT>::kBytes,
                        a.H, tok_valid, a.vec_h};
    for (int vt = t0; vt < t1; ++vt) {
        const int v0 = vt * 256;
        const WideOperand A{static_cast<const char*>(a.weight) +
                                static_cast<int64_t>(v0) * a.H * WideElem<DT>::kBytes,
                            a.H, min(256, a.V - v0), a.vec_w};
        f32x16_t acc[kTM][kTN];
        zero_acc(acc);
        Gemm::run(A, B, a.H, acc, smem);
        fwd_epilogue<true, Acc32>(acc, a, a.bias, v0 + wm * (kTM * 32), lane, tgt, m, s, zt);
    }

    // merge: the two half-wave row groups of a token, then the wavefronts along M (fixed order)
    float* red = reinterpret_cast<float*>(smem);  // [kWM][256 tokens][3]; the GEMM has left LDS
#pragma unroll
    for (int j = 0; j < kTN; ++j) {
        const float m2 = __shfl_xor(m[j], 32);
        const float s2 = __shfl_xor(s[j], 32);
        const float z2 = __shfl_xor(zt[j], 32);
        const float mm = fmaxf(m[j], m2);
        const float mref = mm == -INFINITY ? 0.f : mm;
        const float lo_m = lane < 32 ? m[j] : m2, hi_m = lane < 32 ? m2 : m[j];
        const float lo_s = lane < 32 ? s[j] : s2, hi_s = lane < 32 ? s2 : s[j];
        const float ss = lo_s * __builtin_amdgcn_exp2f(lo_m - mref) + hi_s * __builtin_amdgcn_exp2f(hi_m - mref);
        if (lane < 32) {
            float* dst = red + ((wm * 256) + wn * (kTN * 32) + j * 32 + lane) * 3;
            dst[0] = mm;
            dst[1] = ss;
            dst[2] = zt[j] + z2;
        }
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < tok_valid) {
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWM; ++w) mm = fmaxf(mm, red[(w * 256 + t) * 3]);
        const float mref = mm == -INFINITY ? 0.f : mm;
        float ss = 0.f, zz = 0.f;
#pragma unroll
        for (int w = 0; w < kWM; ++w) {
            const float* pw = red + (w * 256 + t) * 3;
            ss += pw[1] * __builtin_amdgcn_exp2f(pw[0] - mref);
            zz += pw[2];
        }
        const int64_t o = static_cast<int64_t>(sp) * a.N + tok0 + t;
        a.part_m[o] = mm;
        a.part_s[o] = ss;
        a.part_z[o] = zz;
    }
}

// ------------------------------------------------------------------------------------------- //
// Backward step 1: fp32 dZ[tok][v] = g/T * (onehot - softmax) for one token chunk, whole vocab
// ------------------------------------------------------------------------------------------- //
struct WideDzArgs {
    const void* hidden;      // chunk origin [tok][H]
    const void* weight;      // [V][H]
    const float* bias;       // [V] or null
    const int64_t* targets;  // chunk origin (global ids)
    const float* lse;        // chunk origin (natural log)
    const float* grad;       // chunk origin, upstream d/dlogp
    float* dz;               // [tok][ldz], ldz a multiple of 4, 16-byte aligned
    int64_t ldz;
    int tok_valid;
    int V;
    int H;
    int tok_tiles;
    int v_tiles;
    int64_t vocab_start;
    int64_t ignore_index;
    int use_ignore;
    float scale2;  // log2(e) / temperature
    float inv_t;
    bool vec_h, vec_w;
};

template <int DT>
__global__ __launch_bounds__(kThreads) void wide_dz_kernel(WideDzArgs a)
{
    using Gemm = WideGemm<DT, DT, false, false>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int hi = lane >> 5;
    for (TileWalk walk(a.tok_tiles * a.v_tiles, a.v_tiles, a.tok_tiles); walk.valid(); walk.advance()) {
        int vt, tt;
        walk.coords(false, vt, tt);
        const int tok0 = tt * 256, v0 = vt * 256;
        const int tok_rows = min(256, a.tok_valid - tok0);
        const WideOperand A{static_cast<const char*>(a.weight) +
                                static_cast<int64_t>(v0) * a.H * WideElem<DT>::kBytes,
                            a.H, min(256, a.V - v0), a.vec_w};
        const WideOperand B{static_cast<const char*>(a.hidden) +
                                static_cast<int64_t>(tok0) * a.H * WideElem<DT>::kBytes,
                            a.H, tok_rows, a.vec_h};
        f32x16_t acc[kTM][kTN];
        zero_acc(acc);
        Gemm::run(A, B, a.H, acc, smem);

        const int vw = v0 + wm * (kTM * 32);
#pragma unroll
        for (int j = 0; j < kTN; ++j) {
            const int tl = wn * (kTN * 32) + j * 32 + (lane & 31);
            const bool in = tl < tok_rows;
            const int tc = tok0 + (in ? tl : tok_rows - 1);
            const int64_t tg = a.targets[tc];
            const bool live = in && !(a.use_ignore && tg == a.ignore_index);
            const float gs = live ? a.grad[tc] * a.inv_t : 0.f;
            const float nlse2 = -a.lse[tc] * kLog2e;
            const int64_t trel = tg - a.vocab_start;  // row of the shard, any value when not owned
            float* row = a.dz + static_cast<int64_t>(tc) * a.ldz;
#pragma unroll
            for (int i = 0; i < kTM; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int v = vw + i * 32 + 8 * q + 4 * hi;  // first of four consecutive rows
                    f32x4_t d;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int vc = v + c;
                        float z = acc[i][j][q * 4 + c];
                        if (a.bias != nullptr) z += a.bias[vc < a.V ? vc : a.V - 1];
                        const float p = vc < a.V ? __builtin_amdgcn_exp2f(fmaf(z, a.scale2, nlse2)) : 0.f;
                        d[c] = gs * ((trel == vc ? 1.f : 0.f) - p);
                    }
                    // ldz is a multiple of 4 >= V: a quad that starts below V ends below ldz
                    if (in && v < a.V) *reinterpret_cast<f32x4_t*>(row + v) = d;
                }
        }
    }
}

// ------------------------------------------------------------------------------------------- //
// Backward step 2: dH[tok][h] = sum_v dZ[tok][v] W[v][h]   (M = h, N = token, K = vocab)
// The vocab range is cut into `ksplit` parts that run side by side into separate fp32 slots,
// added in slot order by wide_dh_reduce_kernel.
// ------------------------------------------------------------------------------------------- //
struct WideDhArgs {
    const float* dz;     // [tok][ldz]
    int64_t ldz;
    const void* weight;  // [V][H]
    float* part;         // [ksplit][tok_valid][H]
    int64_t slot_stride;
    int H;
    int V;
    int tok_valid;
    int h_tiles;
    int tok_tiles;
    int ksplit;
    int k_per;  // vocab rows per slot (multiple of 16)
    bool vec_w;
};

template <int DT>
__global__ __launch_bounds__(kThreads) void wide_dh_kernel(WideDhArgs a)
{
    using Gemm = WideGemm<DT, RLK_DTYPE_F32, true, false>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tiles = a.h_tiles * a.tok_tiles;
    const int slot = blockIdx.x / tiles;
    int ht, tt;
    xcd_tile(blockIdx.x % tiles, tiles, a.h_tiles, a.tok_tiles, 8, ht, tt);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int h0 = ht * 256, tok0 = tt * 256;
    const int k_lo = slot * a.k_per;
    const int k_n = min(a.k_per, a.V - k_lo);
    const int tok_rows = min(256, a.tok_valid - tok0);
    f32x16_t acc[kTM][kTN];
    zero_acc(acc);
    if (k_n > 0) {  // uniform
        const WideOperand A{static_cast<const char*>(a.weight) +
                                (static_cast<int64_t>(k_lo) * a.H + h0) * WideElem<DT>::kBytes,
                            a.H, min(256, a.H - h0), a.vec_w};
        const WideOperand B{a.dz + static_cast<int64_t>(tok0) * a.ldz + k_lo, a.ldz, tok_rows, true};
        Gemm::run(A, B, k_n, acc, smem);
    }
    float* out = a.part + static_cast<int64_t>(slot) * a.slot_stride;
    const bool vec = (a.H & 3) == 0;
#pragma unroll
    for (int j = 0; j < kTN; ++j) {
        const int tl = wn * (kTN * 32) + j * 32 + (lane & 31);
        if (tl >= tok_rows) continue;
        float* row = out + static_cast<int64_t>(tok0 + tl) * a.H;
#pragma unroll
        for (int i = 0; i < kTM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int h = h0 + wm * (kTM * 32) + i * 32 + 8 * q + 4 * (lane >> 5);
                const f32x4_t v{acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                                acc[i][j][q * 4 + 3]};
                if (vec) {
                    if (h < a.H) *reinterpret_cast<f32x4_t*>(row + h) = v;
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        if (h + c < a.H) row[h + c] = v[c];
                }
            }
    }
}

template <int DT>
__global__ void wide_dh_reduce_kernel(const float* part, int64_t slot_stride, int ksplit, void* out, int64_t n)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float acc = part[i];
    for (int sl = 1; sl < ksplit; ++sl) acc += part[sl * slot_stride + i];
    WideElem<DT>::put(out, i, acc);
}

// ------------------------------------------------------------------------------------------- //
// Backward step 3: dW[v][h] (+)= sum_tok dZ[tok][v] hidden[tok][h]   (M = h, N = vocab, K = token)
// ------------------------------------------------------------------------------------------- //
struct WideDwArgs {
    const float* dz;     // [tok][ldz]
    int64_t ldz;
    const void* hidden;  // chunk origin [tok][H]
    float* dw;           // [V][H] fp32
    int H;
    int V;
    int tok_valid;
    int v_tiles;
    int h_tiles;
    int accumulate;  // 1: dw += ..., 0: dw = ...
    bool vec_h;
};

template <int DT>
__global__ __launch_bounds__(kThreads) void wide_dw_kernel(WideDwArgs a)
{
    using Gemm = WideGemm<DT, RLK_DTYPE_F32, true, true>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const bool vec = (a.H & 3) == 0 && (reinterpret_cast<uintptr_t>(a.dw) & 15) == 0;
    for (TileWalk walk(a.v_tiles * a.h_tiles, a.v_tiles, a.h_tiles); walk.valid(); walk.advance()) {
        int vt, ht;
        walk.coords(false, vt, ht);
        const int v0 = vt * 256, h0 = ht * 256;
        const WideOperand A{static_cast<const char*>(a.hidden) + static_cast<int64_t>(h0) * WideElem<DT>::kBytes,
                            a.H, min(256, a.H - h0), a.vec_h};
        const WideOperand B{a.dz + v0, a.ldz, min(256, a.V - v0), true};
        f32x16_t acc[kTM][kTN];
        zero_acc(acc);
        Gemm::run(A, B, a.tok_valid, acc, smem);
#pragma unroll
        for (int j = 0; j < kTN; ++j) {
            const int v = v0 + wn * (kTN * 32) + j * 32 + (lane & 31);
            if (v >= a.V) continue;
            float* row = a.dw + static_cast<int64_t>(v) * a.H;
#pragma unroll
            for (int i = 0; i < kTM; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int h = h0 + wm * (kTM * 32) + i * 32 + 8 * q + 4 * (lane >> 5);
                    f32x4_t val{acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                                acc[i][j][q * 4 + 3]};
                    if (vec) {
                        if (h < a.H) {
                            if (a.accumulate) val += *reinterpret_cast<const f32x4_t*>(row + h);
                            *reinterpret_cast<f32x4_t*>(row + h) = val;
                        }
                    } else {
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            if (h + c < a.H) row[h + c] = a.accumulate ? row[h + c] + val[c] : val[c];
                    }
                }
        }
    }
}

// db[v] (+)= sum_tok dZ[tok][v], tokens in ascending order.
__global__ void wide_db_kernel(const float* dz, int64_t ldz, int tok_valid, int V, float* db, int accumulate)
{
    const int v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= V) return;
    float acc = 0.f;
    for (int t = 0; t < tok_valid; ++t) acc += dz[static_cast<int64_t>(t) * ldz + v];
    db[v] = accumulate ? db[v] + acc : acc;
}

// ------------------------------------------------------------------------------------------- //
// Host side
// ------------------------------------------------------------------------------------------- //
template <class K>
int wide_smem(K kernel, int bytes)
{
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess
               ? 0
               : rlk_fail(RLK_ERR_LAUNCH, "cannot raise the kernel's LDS limit");
}

int wide_check(const char* what)
{
    return hipGetLastError() == hipSuccess ? 0 : rlk_fail(RLK_ERR_LAUNCH, what);
}

// Four consecutive elements of a row may be fetched with one load when the matrix starts on a
// 4-element boundary and every row does (leading dimension a multiple of four).
bool quad_aligned(const void* p, int64_t ld, int dtype)
{
    const uintptr_t mask = dtype == RLK_DTYPE_F32 ? 15 : 7;
    return (reinterpret_cast<uintptr_t>(p) & mask) == 0 && (ld & 3) == 0;
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

struct WidePlan {
    int64_t chunk;  // tokens per dZ block (multiple of 256, or all N)
    int64_t ldz;
    int ksplit;
    int k_per;
    size_t dz_bytes, part_bytes, total;
};

WidePlan wide_plan(int64_t N, int32_t H, int64_t V, size_t budget)
{
    WidePlan p;
    p.ldz = (V + 3) / 4 * 4;
    const int64_t n_up = (N + 255) / 256 * 256;
    int64_t chunk = static_cast<int64_t>(budget / (static_cast<size_t>(p.ldz) * 4)) / 256 * 256;
    // the fp32 dH slots of a chunk (at least one, chunk x H) stay within half the budget
    const int64_t chunk_h = static_cast<int64_t>(budget / 2 / (static_cast<size_t>(H) * 4)) / 256 * 256;
    if (chunk > chunk_h) chunk = chunk_h;
    if (chunk < 256) chunk = 256;
    if (chunk > n_up) chunk = n_up;
    p.chunk = chunk;
    // dH launch: enough vocab parts to give every compute unit a tile, each at least 64 stages long
    const int64_t tiles = ((H + 255) / 256) * (chunk / 256);
    int64_t ks = (256 + tiles - 1) / tiles;
    const int64_t ks_max = (V + 1023) / 1024;
    if (ks > ks_max) ks = ks_max;
    if (ks > 32) ks = 32;
    if (ks < 1) ks = 1;
    int64_t k_per = ((V + ks - 1) / ks + 15) / 16 * 16;
    ks = (V + k_per - 1) / k_per;
    p.ksplit = static_cast<int>(ks);
    p.k_per = static_cast<int>(k_per);
    p.dz_bytes = align256(static_cast<size_t>(chunk) * p.ldz * 4);
    p.part_bytes = align256(static_cast<size_t>(p.ksplit) * chunk * H * 4);
    p.total = p.dz_bytes + p.part_bytes;
    return p;
}

template <int DT>
int wide_fwd_launch(const WideFwdArgs& a, hipStream_t stream)
{
    using G = WideGemm<DT, DT, false, false>;
    if (int rc = wide_smem(wide_fwd_kernel<DT>, G::kSmemBytes)) return rc;
    hipLaunchKernelGGL(wide_fwd_kernel<DT>, dim3(a.row_blocks * a.n_split), dim3(kThreads), G::kSmemBytes,
                       stream, a);
    return wide_check("wide_fwd_kernel launch failed");
}

template <int DT>
int wide_bwd_launch(const float* grad_logp, const void* hidden, const void* weight, const float* bias,
                    const int64_t* targets, const float* lse, void* d_hidden, float* d_weight,
                    float* d_bias, void* workspace, const WidePlan& p, int64_t N, int32_t H, int64_t V,
                    int64_t vocab_start, float temperature, int64_t ignore_index, int32_t use_ignore,
                    int32_t accumulate, hipStream_t stream)
{
    using GZ = WideGemm<DT, DT, false, false>;
    using GH = WideGemm<DT, RLK_DTYPE_F32, true, false>;
    using GW = WideGemm<DT, RLK_DTYPE_F32, true, true>;
    if (int rc = wide_smem(wide_dz_kernel<DT>, GZ::kSmemBytes)) return rc;
    if (int rc = wide_smem(wide_dh_kernel<DT>, GH::kSmemBytes)) return rc;
    if (int rc = wide_smem(wide_dw_kernel<DT>, GW::kSmemBytes)) return rc;
    constexpr int esz = WideElem<DT>::kBytes;
    float* dz = static_cast<float*>(workspace);
    float* part = reinterpret_cast<float*>(static_cast<char*>(workspace) + p.dz_bytes);
    const int v_tiles = static_cast<int>((V + 255) / 256);
    const int h_tiles = (H + 255) / 256;
    const bool vec_h = quad_aligned(hidden, H, DT), vec_w = quad_aligned(weight, H, DT);
    for (int64_t t0 = 0; t0 < N; t0 += p.chunk) {
        const int nt = static_cast<int>(N - t0 < p.chunk ? N - t0 : p.chunk);
        const int tok_tiles = (nt + 255) / 256;
        const void* hid = static_cast<const char*>(hidden) + t0 * H * esz;
        WideDzArgs z;
        z.hidden = hid;
        z.weight = weight;
        z.bias = bias;
        z.targets = targets + t0;
        z.lse = lse + t0;
        z.grad = grad_logp + t0;
        z.dz = dz;
        z.ldz = p.ldz;
        z.tok_valid = nt;
        z.V = static_cast<int>(V);
        z.H = H;
        z.tok_tiles = tok_tiles;
        z.v_tiles = v_tiles;
        z.vocab_start = vocab_start;
        z.ignore_index = ignore_index;
        z.use_ignore = use_ignore;
        z.scale2 = kLog2e / temperature;
        z.inv_t = 1.f / temperature;
        z.vec_h = vec_h;
        z.vec_w = vec_w;
        hipLaunchKernelGGL(wide_dz_kernel<DT>, dim3(tok_tiles * v_tiles), dim3(kThreads), GZ::kSmemBytes, stream, z);
        if (d_hidden) {
            WideDhArgs h;
            h.dz = dz;
            h.ldz = p.ldz;
            h.weight = weight;
            h.part = part;
            h.slot_stride = static_cast<int64_t>(nt) * H;
            h.H = H;
            h.V = static_cast<int>(V);
            h.tok_valid = nt;
            h.h_tiles = h_tiles;
            h.tok_tiles = tok_tiles;
            h.ksplit = p.ksplit;
            h.k_per = p.k_per;
            h.vec_w = vec_w;
            hipLaunchKernelGGL(wide_dh_kernel<DT>, dim3(h_tiles * tok_tiles * p.ksplit), dim3(kThreads),
                               GH::kSmemBytes, stream, h);
            const int64_t n = static_cast<int64_t>(nt) * H;
            hipLaunchKernelGGL(wide_dh_reduce_kernel<DT>, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256),
                               0, stream, part, h.slot_stride, p.ksplit,
                               static_cast<char*>(d_hidden) + t0 * H * esz, n);
        }
        const int acc = (t0 > 0 || accumulate) ? 1 : 0;
        if (d_weight) {
            WideDwArgs w;
            w.dz = dz;
            w.ldz = p.ldz;
            w.hidden = hid;
            w.dw = d_weight;
            w.H = H;
            w.V = static_cast<int>(V);
            w.tok_valid = nt;
            w.v_tiles = v_tiles;
            w.h_tiles = h_tiles;
            w.accumulate = acc;
            w.vec_h = vec_h;
            hipLaunchKernelGGL(wide_dw_kernel<DT>, dim3(v_tiles * h_tiles), dim3(kThreads), GW::kSmemBytes, stream, w);
        }
        if (d_bias)
            hipLaunchKernelGGL(wide_db_kernel, dim3(static_cast<unsigned>((V + 255) / 256)), dim3(256), 0, stream,
                               dz, p.ldz, nt, static_cast<int>(V), d_bias, acc);
        if (int rc = wide_check("wide backward launch failed")) return rc;
    }
    return 0;
}

}  // namespace

int wide_fwd_partials(const void* hidden, const void* weight, const float* bias, const int64_t* targets,
                      float* part_m, float* part_s, float* part_z, int n_split, int64_t N, int32_t H,
                      int64_t V, int64_t vocab_start, int32_t dtype, float temperature, hipStream_t stream)
{
    WideFwdArgs a;
    a.hidden = hidden;
    a.weight = weight;
    a.bias = bias;
    a.targets = targets;
    a.part_m = part_m;
    a.part_s = part_s;
    a.part_z = part_z;
    a.N = static_cast<int>(N);
    a.H = H;
    a.V = static_cast<int>(V);
    a.vocab_start = vocab_start;
    a.row_blocks = static_cast<int>((N + 255) / 256);
    a.vtiles = static_cast<int>((V + 255) / 256);
    a.n_split = n_split < a.vtiles ? n_split : a.vtiles;
    if (a.n_split != n_split) return rlk_fail(RLK_ERR_ARG, "more splits than vocab tiles");
    a.scale2 = kLog2e / temperature;
    a.vec_h = quad_aligned(hidden, H, dtype);
    a.vec_w = quad_aligned(weight, H, dtype);
    if (dtype == RLK_DTYPE_F32) return wide_fwd_launch<RLK_DTYPE_F32>(a, stream);
    if (dtype == RLK_DTYPE_BF16) return wide_fwd_launch<RLK_DTYPE_BF16>(a, stream);
    return wide_fwd_launch<RLK_DTYPE_F16>(a, stream);
}

size_t wide_bwd_workspace(int64_t N, int32_t H, int64_t V, size_t dz_budget_bytes)
{
    return wide_plan(N, H, V, dz_budget_bytes).total;
}

int wide_bwd(const float* grad_logp, const void* hidden, const void* weight, const float* bias,
             const int64_t* targets, const float* lse, void* d_hidden, float* d_weight, float* d_bias,
             void* workspace, size_t dz_budget_bytes, int64_t N, int32_t H, int64_t V,
             int64_t vocab_start, int32_t dtype, float temperature, int64_t ignore_index,
             int32_t use_ignore, int32_t accumulate, hipStream_t stream)
{
    const WidePlan p = wide_plan(N, H, V, dz_budget_bytes);
    if (dtype == RLK_DTYPE_F32)
        return wide_bwd_launch<RLK_DTYPE_F32>(grad_logp, hidden, weight, bias, targets, lse, d_hidden, d_weight,
                                              d_bias, workspace, p, N, H, V, vocab_start, temperature,
                                              ignore_index, use_ignore, accumulate, stream);
    if (dtype == RLK_DTYPE_BF16)
        return wide_bwd_launch<RLK_DTYPE_BF16>(grad_logp, hidden, weight, bias, targets, lse, d_hidden, d_weight,
                                               d_bias, workspace, p, N, H, V, vocab_start, temperature,
                                               ignore_index, use_ignore, accumulate, stream);
    return wide_bwd_launch<RLK_DTYPE_F16>(grad_logp, hidden, weight, bias, targets, lse, d_hidden, d_weight,
                                          d_bias, workspace, p, N, H, V, vocab_start, temperature,
                                          ignore_index, use_ignore, accumulate, stream);
}

}  // namespace rlk
