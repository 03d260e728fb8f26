// Fused linear -> selected-token log-prob for gfx950: forward (online logsumexp over vocab
// tiles, logits never stored), split combine, and the recompute-based backward (dZ block,
// dH and dW contractions).  All reductions run in a fixed order: same input, same bits.
//
// Orientation used by every kernel here: the MFMA "M" index lives in accumulator registers (the
// 4 registers of a 16 x 16 tile hold rows 4 (l / 16) + 0..3 of column l % 16), the "N" index is
// the lane.  In the forward and in the dZ recompute M = vocab and N = token, so the softmax
// reduction over vocab is an in-register loop per lane; the four lanes that share a token column
// (l, l + 16, l + 32, l + 48) merge their states by two shuffles once per split.
#include "rlk_common.hpp"
#include <algorithm>
#include <mutex>
#include <vector>

#include "rlk_gemm.hpp"
#include "rlk_grpo.hpp"
#include "rlk_tile_epilogue.hpp"

// Load windows (MFMA slots of a K step's second slice over which its 8 loads are spread, see
// TileGemmDtl), measured one kernel at a time at the Llama head (launch time with 16 / 24 / 32
// slots: dZ 791 / 801 / 819 us, dH 822 / 813 / 799 us, dW 866 / 852 / 846 us; forward 23.71 / 23.64 /
// 23.63 ms).
constexpr int kWinFwd = 32;
constexpr int kWinDz = 16;
constexpr int kWinDh = 32;
constexpr int kWinDw = 32;

namespace rlk {


// ------------------------------------------------------------------------------------------- //
// Forward
// ------------------------------------------------------------------------------------------- //
struct FwdArgs {
    const uint16_t* hidden;   // [N][H]
    const uint16_t* weight;   // [V][H]   (local vocab shard)
    const float* bias;        // [V] or null
    const int64_t* targets;   // [N] global ids
    float* part_m;            // [n_split][N] running max (log2 domain)
    float* part_s;            // [n_split][N] running sum of 2^(z - max)
    float* part_z;            // [n_split][N] captured target logit (log2 domain), 0 if not owned
    // optional second head over the same hidden states and targets (a frozen reference model):
    // its tiles follow the first head's in the same pipeline, its partials go to part2_*
    const uint16_t* weight2;  // [V][H] or null
    const float* bias2;       // [V] or null
    float* part2_m;
    float* part2_s;
    float* part2_z;
    int N;
    int H;
    int V;
    int64_t vocab_start;
    int n_split;     // splits handled by this launch
    int split_lo;    // first slot of the partial arrays this launch writes
    int row_blocks;
    int patch_rows;  // token blocks of the patch that the workgroups of one XCD cover per round
    int tile_lo;     // first vocab tile of this launch
    int vtiles;      // vocab tiles of this launch
    float scale2;    // log2(e) / temperature
};

// One workgroup = one block of 256 tokens x one contiguous range of vocab tiles.
// GENERAL = false covers only full vocab tiles [0, vtiles) split n_split ways (a bias is added to
// the finished tile before the softmax update); GENERAL = true handles masked rows over tiles
// [tile_lo, tile_lo+vtiles).
template <class T, int BK, bool GENERAL>
__global__ __launch_bounds__(kThreads) void linear_logp_fwd_kernel(FwdArgs a)
{
    using AT = Acc16;
    constexpr int TM = AT::TM, TN = AT::TN;
    using Gemm = TileGemm<T, false, false, BK>;
    using Dtl = TileGemmDtl<T, false, false, BK, kWinFwd>;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    int tb, sp;
    xcd_tile(blockIdx.x, a.row_blocks * a.n_split, a.row_blocks, a.n_split, a.patch_rows, tb, sp);
    // vocab tiles [t0, t1) of this split: the first (vtiles % n_split) splits take one extra.
    const int base = a.vtiles / a.n_split, extra = a.vtiles % a.n_split;
    const int t0 = a.tile_lo + sp * base + (sp < extra ? sp : extra);
    const int t1 = t0 + base + (sp < extra ? 1 : 0);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int tok0 = tb * 256;
    const int tok_valid = min(256, a.N - tok0);

    float m[TN], s[TN], zt[TN];
    int tgt[TN];  // target id relative to the shard, -1 when not in [0, V)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int t = wn * (TN * 16) + AT::col(j, lane);
        int64_t g = a.targets[tok0 + (t < tok_valid ? t : tok_valid - 1)] - a.vocab_start;
        tgt[j] = (g >= 0 && g < a.V) ? static_cast<int>(g) : -1;
    }
    auto reset_state = [&]() {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            m[j] = -INFINITY;
            s[j] = 0.f;
            zt[j] = 0.f;
        }
    };

    // Merge of one head's state: the four lane groups of a wavefront (same token, different vocab
    // rows; groups 16 apart first, then 32 apart), then the wavefronts along M through LDS, in a
    // fixed order; written to that head's partial arrays.  The LDS patch lies behind the pipeline
    // stages, so the merge of the first head can run while the second head's first K steps are
    // already on their way.
    float* red = reinterpret_cast<float*>(smem + Dtl::kSmemBytes);  // [kWM][256 tokens][3]
    static_assert(Dtl::kSmemBytes + kWM * 256 * 3 * 4 <= Gemm::kSmemBytes, "merge patch must fit the kernel's LDS");
    auto flush_state = [&](float* pm, float* ps, float* pz) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            float mj = m[j], sj = s[j], zj = zt[j];
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const float m2 = __shfl_xor(mj, off);
                const float s2 = __shfl_xor(sj, off);
                const float z2 = __shfl_xor(zj, off);
                const float mm = fmaxf(mj, m2);
                const float mref = mm == -INFINITY ? 0.f : mm;
                // both partners evaluate the same expression: the lower group's term first
                const bool low = (lane & off) == 0;
                const float lo_m = low ? mj : m2, hi_m = low ? m2 : mj;
                const float lo_s = low ? sj : s2, hi_s = low ? s2 : sj;
                sj = lo_s * __builtin_amdgcn_exp2f(lo_m - mref) + hi_s * __builtin_amdgcn_exp2f(hi_m - mref);
                mj = mm;
                zj = (low ? zj : z2) + (low ? z2 : zj);
            }
            if (lane < 16) {
                float* dst = red + ((wm * 256) + wn * (TN * 16) + j * 16 + lane) * 3;
                dst[0] = mj;
                dst[1] = sj;
                dst[2] = zj;
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
            const int64_t o = static_cast<int64_t>(a.split_lo + sp) * a.N + tok0 + t;
            pm[o] = mm;
            ps[o] = ss;
            pz[o] = zz;
        }
        __syncthreads();  // the patch may be written again
    };

    const int n_heads = a.weight2 != nullptr ? 2 : 1;
    Operand B{a.hidden + static_cast<int64_t>(tok0) * a.H, a.H, tok_valid};
    auto tile_origin = [&](int head, int vt) {
        return (head == 0 ? a.weight : a.weight2) + static_cast<int64_t>(vt) * 256 * a.H;
    };
    if (!GENERAL && a.H % BK == 0 && a.H >= 2 * BK && t0 < t1) {
        // every tile is full: one pipeline runs through all tiles of the range (and then through
        // the same range of the second head), the K loop of a tile already fetching the head of the
        // next one while the softmax update runs (the pipeline looks two K steps ahead, which stays
        // within the next tile from two steps up)
        typename Dtl::Stream st;
        Dtl::begin(st, Operand{tile_origin(0, t0), a.H, 256}, B, a.H, smem);
        for (int head = 0; head < n_heads; ++head) {
            reset_state();
            for (int vt = t0; vt < t1; ++vt) {
                f32x4_t acc[TM][TN];
                zero_acc(acc);
                const void* next = vt + 1 < t1 ? tile_origin(head, vt + 1)
                                               : (head + 1 < n_heads ? tile_origin(head + 1, t0)
                                                                     : tile_origin(head, vt));
                Dtl::template tile<true>(st, next, B.base, acc, smem);
                const float* bias = head == 0 ? a.bias : a.bias2;
                if (bias != nullptr) add_bias<AT>(acc, bias, vt * 256 + wm * (TM * 16), lane);  // uniform
                fwd_epilogue<GENERAL, AT>(acc, a, nullptr, vt * 256 + wm * (TM * 16), lane, tgt, m, s, zt);
            }
            if (head == 0)
                flush_state(a.part_m, a.part_s, a.part_z);
            else
                flush_state(a.part2_m, a.part2_s, a.part2_z);
        }
        Dtl::end(st);
    } else {
        for (int head = 0; head < n_heads; ++head) {
            reset_state();
            const float* bias = head == 0 ? a.bias : a.bias2;
            for (int vt = t0; vt < t1; ++vt) {
                const int v0 = vt * 256;
                Operand A{tile_origin(head, vt), a.H, min(256, a.V - v0)};
                f32x4_t acc[TM][TN];
                zero_acc(acc);
                Gemm::run(A, B, a.H, acc, smem);
                if (!GENERAL && bias != nullptr) add_bias<AT>(acc, bias, v0 + wm * (TM * 16), lane);  // uniform
                fwd_epilogue<GENERAL, AT>(acc, a, bias, v0 + wm * (TM * 16), lane, tgt, m, s, zt);
            }
            if (head == 0)
                flush_state(a.part_m, a.part_s, a.part_z);
            else
                flush_state(a.part2_m, a.part2_s, a.part2_z);
        }
    }
}

struct CombineArgs {
    const float* part_m;
    const float* part_s;
    const float* part_z;
    const int64_t* targets;
    float* logp;
    float* lse;
    int32_t* err_flag;
    int N;
    int V;
    int n_split;
    int64_t vocab_start;
    int64_t ignore_index;
    int use_ignore;
    int strict;  // 1: a non-ignored target outside [vocab_start, vocab_start+V) raises err_flag
};

// M = max_s m_s ; S = sum_s s_s 2^(m_s - M) ; z_t = sum_s z_t,s ; lse = ln2 (M + log2 S).
// Writes lse and logp of token n and returns the logp.
__device__ inline float combine_token(const CombineArgs& a, int64_t n)
{
    float mm = -INFINITY;
    for (int sp = 0; sp < a.n_split; ++sp) mm = fmaxf(mm, a.part_m[static_cast<int64_t>(sp) * a.N + n]);
    float ss = 0.f, zz = 0.f;
    for (int sp = 0; sp < a.n_split; ++sp) {
        const int64_t o = static_cast<int64_t>(sp) * a.N + n;
        ss += a.part_s[o] * exp2f(a.part_m[o] - mm);
        zz += a.part_z[o];
    }
    const float lse2 = mm + log2f(ss);
    const int64_t t = a.targets[n];
    const bool ignored = a.use_ignore && t == a.ignore_index;
    const int64_t tl = t - a.vocab_start;
    const bool owned = tl >= 0 && tl < a.V;
    if (!ignored && !owned && a.strict) *a.err_flag = 1;
    const float lp = ignored ? 0.f : (zz - lse2) * kLn2;
    a.lse[n] = lse2 * kLn2;
    a.logp[n] = lp;
    return lp;
}

__global__ void linear_logp_combine_kernel(CombineArgs a)
{
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= a.N) return;
    combine_token(a, n);
}

// Combine with the GRPO loss epilogue folded in: the launch has the block / thread partition of
// the stand-alone epilogue (block b owns a contiguous token range, thread t walks it with stride
// 256), merges the split partials of each of its tokens and feeds the fresh log-prob straight into
// the loss terms, the fixed-order partial sums and d loss / d logp.  The active-token count comes
// from grpo_count_kernel, which ran before the contraction.  The workgroup that finishes last
// (integer ticket) adds up the block partials in block order and writes the three scalars, so no
// further launch is needed.  Same expressions, same partition, same tree as combine +
// rlk_grpo_loss_from_logp: same bits.
__global__ __launch_bounds__(kRedThreads) void linear_logp_combine_grpo_kernel(CombineArgs c, GrpoArgs g)
{
    const int64_t per = (g.n + g.blocks - 1) / g.blocks;
    const int64_t lo = per * blockIdx.x;
    const int64_t hi = lo + per < g.n ? lo + per : g.n;
    const float denom = grpo_denominator(g.words);
    Term t{0.f, 0.f, 0.f};
    for (int64_t i = lo + threadIdx.x; i < hi; i += kRedThreads) {
        const float lp = combine_token(c, i);
        const bool on = g.mask == nullptr || g.mask[i] != 0;
        float r = 0.f, k = 0.f, gr = 0.f, gk = 0.f;
        if (on) {
            float pol;
            token_terms(g, i, lp, r, pol, k);
            t.pol += pol;
            if (g.ref_lp != nullptr) t.kl += k;
            t.act += 1.f;
            if (g.dcur != nullptr) token_grad(g, i, lp, denom, gr, gk);
        }
        if (g.ratio) g.ratio[i] = r;
        if (g.kl_terms) g.kl_terms[i] = k;
        if (g.dcur) g.dcur[i] = gr;
        if (g.dkl) g.dkl[i] = gk;
    }
    const Term s = block_sum(t);
    __shared__ int last_block;
    if (threadIdx.x == 0) {
        g.partial[blockIdx.x * 3 + 0] = s.pol;
        g.partial[blockIdx.x * 3 + 1] = s.kl;
        g.partial[blockIdx.x * 3 + 2] = s.act;
        __threadfence();  // the partials are visible before the ticket is taken
        last_block = atomicAdd(&g.words[0], 1) == g.blocks - 1;
    }
    __syncthreads();
    if (last_block) {  // uniform: every other workgroup has published its partials
        __threadfence();
        grpo_finish<true>(g);
    }
}

// ------------------------------------------------------------------------------------------- //
// Backward step 1: dZ block = g/T * (onehot - softmax) for a (token chunk) x (vocab piece)
// ------------------------------------------------------------------------------------------- //
struct DzArgs {
    const uint16_t* hidden;  // chunk origin [tok][H]
    const uint16_t* weight;  // piece origin [v][H]
    const float* bias;       // piece origin or null
    const int64_t* targets;  // chunk origin (global ids)
    const float* lse;        // chunk origin (natural log)
    const float* grad;       // chunk origin, upstream d/dlogp
    const float* scales;     // [0] = loss_scale / temperature (device resident)
    uint16_t* dz;            // [tok_tiles*256][ldz]
    int64_t ldz;
    int tok_valid;
    int v_valid;
    int H;
    int tok_tiles;
    int v_tiles;        // vocab tiles of this launch
    int v_tile_lo;      // first vocab tile of this launch
    int64_t v_global0;  // global id of the piece's first vocab row
    int64_t ignore_index;
    int use_ignore;
    float scale2;
};

// LDS each wavefront needs to turn its part of a dZ tile into full rows: 64 tokens x 32 vocab
// columns of 16-bit values, 64 bytes per token row, no padding.
constexpr int kDzStageBytes = 64 * 64;

// dZ epilogue of one 256 x 256 tile.  A wavefront owns 128 vocab rows x 64 tokens of the tile; for
// each of its four 32-row groups (two 16-row MFMA tiles) it writes the rounded values into its
// private LDS patch as [token][vocab] rows and reads them back row-wise, so that the tile leaves
// in runs of 64 contiguous bytes per token.  Only the wavefront itself touches its patch: no
// workgroup barrier.  The 8-byte units of a row are XOR-swizzled with 2 * ((token / 4) & 3), which
// makes both the writes (16 tokens x 2 lane groups per pass) and the reads (4 rows x 8 units)
// conflict-free.
template <class T, bool GENERAL>
__device__ inline void dz_epilogue(const f32x4_t (&acc)[Acc16::TM][Acc16::TN], const DzArgs& a, int vt, int tt,
                                   char* stage)
{
    using AT = Acc16;
    constexpr int TM = AT::TM, TN = AT::TN;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int tok0 = tt * 256, v0 = vt * 256;
    const int tok_rows = min(256, a.tok_valid - tok0);
    const float gscale = a.scales[0];
    const int vw = v0 + wm * (TM * 16);
    const int grp = lane >> 4;  // this lane holds rows 4 * grp + 0..3 of every 16-row tile

    float gs[TN], nlse2[TN];
    int etgt[TN];  // register index (i*4 + r) of the target row in this lane, or -1
    bool any_target = false;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int tl = wn * (TN * 16) + AT::col(j, lane);
        const int tc = tok0 + (tl < tok_rows ? tl : tok_rows - 1);
        const int64_t tg = a.targets[tc];
        const bool live = tl < tok_rows && !(a.use_ignore && tg == a.ignore_index);
        gs[j] = live ? a.grad[tc] * gscale : 0.f;
        nlse2[j] = -a.lse[tc] * kLog2e;
        const int64_t trel = tg - a.v_global0 - vw;
        etgt[j] = (trel >= 0 && trel < TM * 16) ? AT::reg_of_row(static_cast<int>(trel), lane) : -1;
        any_target = any_target || etgt[j] >= 0;
    }
    // the one-hot term is added only when some lane of the wavefront owns its target row here
    const bool hot = __builtin_amdgcn_ballot_w64(any_target) != 0;  // uniform

    uint16_t* dtile = a.dz + static_cast<int64_t>(tok0 + wn * (TN * 16)) * a.ldz + vw;
    auto stage_rows = [&](auto ipc, auto hot_c) {
        constexpr int ip = decltype(ipc)::value;  // 32-row group = MFMA tiles 2 ip and 2 ip + 1
        constexpr bool HOT = decltype(hot_c)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int t = j * 16 + (lane & 15);  // token row inside the wavefront's patch
            char* srow = stage + t * 64;
            const int sw = ((t >> 2) & 3) << 1;
#pragma unroll
            for (int ii = 0; ii < 2; ++ii) {
                constexpr int i0 = 2 * ip;
                const int i = i0 + ii;
                float d[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float z = acc[i][j][c];
                    float pr;
                    if (GENERAL) {
                        const int v = vw + i * 16 + 4 * grp + c;
                        if (a.bias != nullptr) z += a.bias[v < a.v_valid ? v : a.v_valid - 1];
                        pr = v < a.v_valid ? __builtin_amdgcn_exp2f(fmaf(z, a.scale2, nlse2[j])) : 0.f;
                    } else {
                        pr = __builtin_amdgcn_exp2f(fmaf(z, a.scale2, nlse2[j]));
                    }
                    if constexpr (HOT) {
                        const float hit = (etgt[j] == i * 4 + c) ? gs[j] : 0.f;
                        d[c] = fmaf(-gs[j], pr, hit);
                    } else {
                        d[c] = -gs[j] * pr;
                    }
                }
                // rows 16 ii + 4 grp + 0..3 of this 32-row group: unit 4 ii + grp of the token's row
                *reinterpret_cast<u32x2_t*>(srow + (((4 * ii + grp) ^ sw) * 8)) =
                    u32x2_t{T::pack2(d[0], d[1]), T::pack2(d[2], d[3])};
            }
        }
    };
    static_for<0, TM / 2>([&](auto ipc) {
        constexpr int ip = decltype(ipc)::value;
        if (hot)
            stage_rows(ipc, std::true_type{});
        else
            stage_rows(ipc, std::false_type{});
        __builtin_amdgcn_wave_barrier();
        // copy-out: 8 lanes move one token row (64 bytes), 8 rows per instruction
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int row = it * 8 + (lane >> 3);
            const int u = lane & 7;
            const u32x2_t v =
                *reinterpret_cast<const u32x2_t*>(stage + row * 64 + ((u ^ (((row >> 2) & 3) << 1)) * 8));
            *reinterpret_cast<u32x2_t*>(dtile + static_cast<int64_t>(row) * a.ldz + ip * 32 + u * 4) = v;
        }
        __builtin_amdgcn_wave_barrier();
    });
}

// GENERAL = false: every vocab tile of the launch is full (a bias is added to the finished tile).
// CHAIN (needs !GENERAL, full token tiles, H a multiple of BK and >= 2 BK): the workgroup walks
// its tiles through one pipeline; while a tile's epilogue runs, the first K steps of the next
// tile are already on their way into LDS.
template <class T, int BK, bool GENERAL, bool CHAIN>
__global__ __launch_bounds__(kThreads) void linear_logp_dz_kernel(DzArgs a)
{
    static_assert(!(GENERAL && CHAIN), "the chained variant covers full tiles only");
    using AT = Acc16;
    using Gemm = TileGemm<T, false, false, BK>;
    using Dtl = TileGemmDtl<T, false, false, BK, kWinDz>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int wave = threadIdx.x >> 6;
    TileWalk walk(a.tok_tiles * a.v_tiles, a.v_tiles, a.tok_tiles);
    if (!walk.valid()) return;
    int vt, tt;
    walk.coords(false, vt, tt);
    auto w_origin = [&](int v) { return a.weight + static_cast<int64_t>(v + a.v_tile_lo) * 256 * a.H; };
    auto h_origin = [&](int t) { return a.hidden + static_cast<int64_t>(t) * 256 * a.H; };
    f32x4_t acc[AT::TM][AT::TN];
    if constexpr (CHAIN) {
        char* stage = smem + Dtl::kSmemBytes + wave * kDzStageBytes;
        typename Dtl::Stream st;
        Dtl::begin(st, Operand{w_origin(vt), a.H, 256}, Operand{h_origin(tt), a.H, 256}, a.H, smem);
        for (;;) {
            const bool more = walk.has_next();
            int nvt = vt, ntt = tt;
            if (more) walk.coords(true, nvt, ntt);
            zero_acc(acc);
            Dtl::template tile<true>(st, w_origin(nvt), h_origin(ntt), acc, smem);
            if (a.bias != nullptr)  // uniform
                add_bias<AT>(acc, a.bias, (vt + a.v_tile_lo) * 256 + (wave / kWN) * (AT::TM * 16), threadIdx.x & 63);
            dz_epilogue<T, GENERAL>(acc, a, vt + a.v_tile_lo, tt, stage);
            if (!more) break;
            walk.advance();
            vt = nvt;
            tt = ntt;
        }
        Dtl::end(st);
    } else {
        static_assert(kDzStageBytes * (kThreads / 64) <= Gemm::kSmemBytes, "staging must fit the GEMM's LDS");
        for (;;) {
            const int tok0 = tt * 256, v0 = (vt + a.v_tile_lo) * 256;
            Operand A{w_origin(vt), a.H, min(256, a.v_valid - v0)};
            Operand B{h_origin(tt), a.H, min(256, a.tok_valid - tok0)};
            zero_acc(acc);
            Gemm::run(A, B, a.H, acc, smem);  // ends with a barrier: LDS is free
            if (!GENERAL && a.bias != nullptr)  // uniform
                add_bias<AT>(acc, a.bias, v0 + (wave / kWN) * (AT::TM * 16), threadIdx.x & 63);
            dz_epilogue<T, GENERAL>(acc, a, vt + a.v_tile_lo, tt, smem + wave * kDzStageBytes);
            if (!walk.has_next()) break;
            walk.advance();
            walk.coords(false, vt, tt);
            __syncthreads();  // every wavefront has left its staging patch
        }
    }
}

// ------------------------------------------------------------------------------------------- //
// Backward step 2: dH[tok][h] (+)= sum_v dZ[tok][v] W[v][h]      (M = h, N = token, K = vocab)
// ------------------------------------------------------------------------------------------- //
struct DhArgs {
    const uint16_t* dz;      // [tok_tiles*256][ldz]
    const uint16_t* weight;  // piece origin [v][H]
    const float* scales;     // [1] = 1 / loss_scale
    float* acc;              // fp32 partial dH of the chunk [tok_tiles*256][H] (may be null if single)
    uint16_t* out;           // dH chunk origin [tok][H], written when `last`
    int64_t ldz;
    int H;
    int v_valid;
    int tok_valid;
    int tok_tiles;
    int h_tiles;
    int first;  // 1: do not read acc
    int last;   // 1: write the 16-bit output instead of acc
    int ksplit;           // > 1: the vocab range is cut into ksplit parts computed by separate
    float* part;          //      workgroups, each writing its own fp32 slot [ksplit][rows][H]
    int64_t part_stride;  //      (elements per slot); linear_logp_dh_reduce_kernel adds them up
};

// Epilogue of one dH tile.  The read-modify-write of the running fp32 partial is latency-bound, so
// it runs in two batches (one per pair of 16-token column groups): the 16 reads of a batch are all
// issued before the first use, then added and stored.  FULL (the tile lies inside the chunk and
// inside H): addresses are a uniform tile origin plus a 32-bit lane offset and no predicates are
// needed; otherwise rows and columns are clamped for the reads and predicated for the stores.
// The tile covers hidden columns [h0, h0 + 256) and owns those from h_min on (h_min > h0 for the
// last tile of a persistent walk when H is not a multiple of 256: it is shifted back to end at H
// and must leave the columns of its left neighbour alone).
template <class T, bool FULL>
__device__ inline void dh_epilogue_impl(const f32x4_t (&acc)[Acc16::TM][Acc16::TN], const DhArgs& a, int tt,
                                        int h0, int h_min, float* acc_dst, bool first, bool last)
{
    using AT = Acc16;
    constexpr int TM = AT::TM, TN = AT::TN;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int tok0 = tt * 256;
    const float oscale = a.scales[1];
    const int hbase = h0 + wm * (TM * 16) + 4 * (lane >> 4);  // + i * 16
    const uint32_t ldh = static_cast<uint32_t>(a.H);
    // FULL: byte offsets inside the tile stay below 256 * H * 4 (32 bits)
    const int64_t origin = static_cast<int64_t>(tok0) * a.H + h0;
    char* acc_tile = reinterpret_cast<char*>(acc_dst + origin);
    char* out_tile = reinterpret_cast<char*>(a.out + origin);
    const uint32_t lane_el = static_cast<uint32_t>(wn * (TN * 16) + (lane & 15)) * ldh +
                             static_cast<uint32_t>(wm * (TM * 16) + 4 * (lane >> 4));
#pragma unroll
    for (int jb = 0; jb < TN; jb += 2) {
        f32x4_t old[2][TM];
        bool tok_ok[2];
        int64_t trow[2];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = jb + jj;
            const int tl = tok0 + wn * (TN * 16) + AT::col(j, lane);
            tok_ok[jj] = FULL || tl < a.tok_valid;
            trow[jj] = static_cast<int64_t>(tok_ok[jj] ? tl : a.tok_valid - 1) * a.H;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                old[jj][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                if (!first) {  // uniform
                    if (FULL) {
                        const char* rowp = acc_tile + (static_cast<size_t>(j * 16) * ldh + i * 16) * 4u;
                        old[jj][i] = *reinterpret_cast<const f32x4_t*>(rowp + lane_el * 4u);
                    } else {
                        const int h = hbase + i * 16;
                        old[jj][i] = *reinterpret_cast<const f32x4_t*>(acc_dst + trow[jj] + (h < a.H ? h : 0));
                    }
                }
            }
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = jb + jj;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int h = hbase + i * 16;
                const f32x4_t v = acc[i][j] + old[jj][i];
                const size_t uni = static_cast<size_t>(j * 16) * ldh + i * 16;  // uniform
                if (FULL || (tok_ok[jj] && h >= h_min && h < a.H)) {  // H % 8 == 0: a quad is all-in or all-out
                    if (last) {
                        u32x2_t pk{T::pack2(v.x * oscale, v.y * oscale), T::pack2(v.z * oscale, v.w * oscale)};
                        if (FULL)
                            *reinterpret_cast<u32x2_t*>(out_tile + uni * 2u + lane_el * 2u) = pk;
                        else
                            *reinterpret_cast<u32x2_t*>(a.out + trow[jj] + h) = pk;
                    } else {
                        if (FULL)
                            *reinterpret_cast<f32x4_t*>(acc_tile + uni * 4u + lane_el * 4u) = v;
                        else
                            *reinterpret_cast<f32x4_t*>(acc_dst + trow[jj] + h) = v;
                    }
                }
            }
        }
    }
}

// Returns whether the tile was full (then every wavefront issued all its stores unconditionally).
template <class T>
__device__ inline bool dh_epilogue(const f32x4_t (&acc)[Acc16::TM][Acc16::TN], const DhArgs& a, int tt, int h0,
                                   int h_min, float* acc_dst, bool first, bool last)
{
    const bool full = tt * 256 + 256 <= a.tok_valid && h0 + 256 <= a.H && h_min == h0;  // uniform
    if (full)
        dh_epilogue_impl<T, true>(acc, a, tt, h0, h_min, acc_dst, first, last);
    else
        dh_epilogue_impl<T, false>(acc, a, tt, h0, h_min, acc_dst, first, last);
    return full;
}

// CHAIN (needs ksplit == 1, H >= 256, v_valid a multiple of BK and >= 2 BK): the workgroup walks
// its tiles through one pipeline.
template <class T, int BK, bool CHAIN>
__global__ __launch_bounds__(kThreads) void linear_logp_dh_kernel(DhArgs a)
{
    using Gemm = TileGemm<T, true, false, BK>;
    using Dtl = TileGemmDtl<T, true, false, BK, kWinDh>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    f32x4_t acc[Acc16::TM][Acc16::TN];
    if constexpr (CHAIN) {
        TileWalk walk(a.tok_tiles * a.h_tiles, a.tok_tiles, a.h_tiles);
        if (!walk.valid()) return;
        int tt, ht;
        walk.coords(false, tt, ht);
        // first hidden column of h tile `h`: the last tile is shifted back so that it ends at H
        auto h_col = [&](int h) { return min(h * 256, a.H - 256); };
        auto w_origin = [&](int h) { return a.weight + h_col(h); };
        auto z_origin = [&](int t) { return a.dz + static_cast<int64_t>(t) * 256 * a.ldz; };
        typename Dtl::Stream st;
        bool counted = false;
        Dtl::begin(st, Operand{w_origin(ht), a.H, 256}, Operand{z_origin(tt), a.ldz, 256}, a.v_valid, smem);
        for (;;) {
            const bool more = walk.has_next();
            int ntt = tt, nht = ht;
            if (more) walk.coords(true, ntt, nht);
            zero_acc(acc);
            // a full tile's epilogue issues TM * TN unconditional stores per wavefront
            Dtl::template tile<true, Acc16::TM * Acc16::TN / 2>(st, w_origin(nht), z_origin(ntt), acc, smem, counted);
            counted = dh_epilogue<T>(acc, a, tt, h_col(ht), ht * 256, a.acc, a.first != 0, a.last != 0);
            if (!more) break;
            walk.advance();
            tt = ntt;
            ht = nht;
        }
        Dtl::end(st);
    } else {
        int tt, ht, ks = 0;
        xcd_tile(blockIdx.x, a.tok_tiles * a.h_tiles * a.ksplit, a.tok_tiles, a.h_tiles * a.ksplit, 8,
                 tt, ht);
        // K range of this workgroup: whole BK-row steps, the first (steps % ksplit) parts take one more
        int k0 = 0, kn = a.v_valid;
        float* acc_dst = a.acc;
        bool first = a.first != 0, last = a.last != 0, empty_part = false;
        if (a.ksplit > 1) {  // uniform
            ks = ht % a.ksplit;
            ht /= a.ksplit;
            const int steps = (a.v_valid + BK - 1) / BK;
            const int base = steps / a.ksplit, extra = steps % a.ksplit;
            const int s0 = ks * base + (ks < extra ? ks : extra);
            const int s1 = s0 + base + (ks < extra ? 1 : 0);
            k0 = s0 * BK;
            kn = min(a.v_valid, s1 * BK) - k0;
            if (kn <= 0) {  // a short last piece can leave a part without K steps: it computes one
                empty_part = true;  // step of the piece's head and discards it
                k0 = 0;
                kn = min(a.v_valid, BK);
            }
            acc_dst = a.part + static_cast<int64_t>(ks) * a.part_stride;
            first = true;
            last = false;
        }
        const int tok0 = tt * 256, h0 = ht * 256;
        Operand A{a.weight + static_cast<int64_t>(k0) * a.H + h0, a.H, min(256, a.H - h0)};
        Operand B{a.dz + static_cast<int64_t>(tok0) * a.ldz + k0, a.ldz, 256};
        zero_acc(acc);
        Gemm::run(A, B, kn, acc, smem);
        if (empty_part) zero_acc(acc);  // uniform: this part's slot must hold zeros
        dh_epilogue<T>(acc, a, tt, h0, h0, acc_dst, first, last);
    }
}

// Sum of the ksplit partial dH slots of one chunk in slot order (plus the running fp32 partial of
// earlier vocab pieces unless `first`), written back as the running partial or, for the last
// piece, as the 16-bit gradient.  One thread per 4 consecutive elements of a row.
template <class T>
__global__ void linear_logp_dh_reduce_kernel(const float* part, int ksplit, int64_t part_stride,
                                             float* acc, uint16_t* out, const float* scales,
                                             int64_t n4, int first, int last)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    f32x4_t v{0.f, 0.f, 0.f, 0.f};
    if (!first) v = reinterpret_cast<const f32x4_t*>(acc)[i];
    for (int k = 0; k < ksplit; ++k) v += reinterpret_cast<const f32x4_t*>(part + k * part_stride)[i];
    if (last) {
        const float oscale = scales[1];
        u32x2_t pk{T::pack2(v.x * oscale, v.y * oscale), T::pack2(v.z * oscale, v.w * oscale)};
        reinterpret_cast<u32x2_t*>(out)[i] = pk;
    } else {
        reinterpret_cast<f32x4_t*>(acc)[i] = v;
    }
}

// ------------------------------------------------------------------------------------------- //
// Backward step 3: dW[v][h] (+)= sum_tok dZ[tok][v] hidden[tok][h]   (M = h, N = vocab, K = token)
// ------------------------------------------------------------------------------------------- //
struct DwArgs {
    const uint16_t* dz;      // [tok_tiles*256][ldz]
    const uint16_t* hidden;  // chunk origin [tok][H]
    const float* scales;     // [1] = 1 / loss_scale
    float* dw;               // piece origin [v][H] fp32
    int64_t ldz;
    int H;
    int v_valid;
    int tok_valid;
    int v_tiles;
    int h_tiles;
    int accumulate;  // 1: dw += ..., 0: dw = ...
};

// Epilogue of one dW tile.  Orientation: M (accumulator registers) = hidden column, N (lane) =
// vocab row, so a lane holds 4 consecutive columns of one dW row and the read-modify-write of the
// fp32 tile moves 16 bytes per lane (the four lane groups of a 16 x 16 tile make 64 contiguous
// bytes per row).  It is latency-bound and therefore runs in two batches (one per pair of 16-row
// groups): the 16 reads of a batch are issued before the first use.  FULL (the tile lies inside the
// piece and inside H): a uniform tile origin plus a 32-bit lane offset, no predicates; otherwise
// clamped reads and predicated stores.
// The tile covers hidden columns [h0, h0 + 256) and owns those from h_min on (see dh_epilogue_impl).
template <bool FULL>
__device__ inline void dw_epilogue_impl(const f32x4_t (&acc)[Acc16::TM][Acc16::TN], const DwArgs& a, int vt,
                                        int h0, int h_min)
{
    using AT = Acc16;
    constexpr int TM = AT::TM, TN = AT::TN;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / kWN, wn = wave % kWN;
    const int v0 = vt * 256;
    const float oscale = a.scales[1];
    const int hbase = h0 + wm * (TM * 16) + 4 * (lane >> 4);  // + i * 16
    const uint32_t ldw = static_cast<uint32_t>(a.H);
    // FULL: byte offsets inside the tile stay below 256 * H * 4 (32 bits)
    char* tile = reinterpret_cast<char*>(a.dw + static_cast<int64_t>(v0) * a.H + h0);
    const uint32_t lane_el = static_cast<uint32_t>(wn * (TN * 16) + (lane & 15)) * ldw +
                             static_cast<uint32_t>(wm * (TM * 16) + 4 * (lane >> 4));
#pragma unroll
    for (int jb = 0; jb < TN; jb += 2) {
        f32x4_t old[2][TM];
        bool v_ok[2];
        int64_t vrow[2];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = jb + jj;
            const int v = v0 + wn * (TN * 16) + AT::col(j, lane);
            v_ok[jj] = FULL || v < a.v_valid;
            vrow[jj] = static_cast<int64_t>(v_ok[jj] ? v : a.v_valid - 1) * a.H;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                old[jj][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                if (a.accumulate) {  // uniform
                    if (FULL) {
                        const char* rowp = tile + (static_cast<size_t>(j * 16) * ldw + i * 16) * 4u;
                        old[jj][i] = *reinterpret_cast<const f32x4_t*>(rowp + lane_el * 4u);
                    } else {
                        const int h = hbase + i * 16;
                        old[jj][i] = *reinterpret_cast<const f32x4_t*>(a.dw + vrow[jj] + (h < a.H ? h : 0));
                    }
                }
            }
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = jb + jj;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int h = hbase + i * 16;
                const f32x4_t val = acc[i][j] * oscale + old[jj][i];
                if (FULL) {
                    char* rowp = tile + (static_cast<size_t>(j * 16) * ldw + i * 16) * 4u;
                    *reinterpret_cast<f32x4_t*>(rowp + lane_el * 4u) = val;
                } else if (v_ok[jj] && h >= h_min && h < a.H) {  // H % 8 == 0: a quad is all-in or all-out
                    *reinterpret_cast<f32x4_t*>(a.dw + vrow[jj] + h) = val;
                }
            }
        }
    }
}

// Returns whether the tile was full (then every wavefront issued all its stores unconditionally).
__device__ inline bool dw_epilogue(const f32x4_t (&acc)[Acc16::TM][Acc16::TN], const DwArgs& a, int vt, int h0,
                                   int h_min)
{
    const bool full = vt * 256 + 256 <= a.v_valid && h0 + 256 <= a.H && h_min == h0;  // uniform
    if (full)
        dw_epilogue_impl<true>(acc, a, vt, h0, h_min);
    else
        dw_epilogue_impl<false>(acc, a, vt, h0, h_min);
    return full;
}

// CHAIN (needs H >= 256, tok_valid a multiple of BK and >= 2 BK): the workgroup walks its tiles
// through one pipeline.
template <class T, int BK, bool CHAIN>
__global__ __launch_bounds__(kThreads) void linear_logp_dw_kernel(DwArgs a)
{
    using Gemm = TileGemm<T, true, true, BK>;
    using Dtl = TileGemmDtl<T, true, true, BK, kWinDw>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    TileWalk walk(a.v_tiles * a.h_tiles, a.v_tiles, a.h_tiles);
    if (!walk.valid()) return;
    int vt, ht;
    walk.coords(false, vt, ht);
    f32x4_t acc[Acc16::TM][Acc16::TN];
    auto z_origin = [&](int v) { return a.dz + static_cast<int64_t>(v) * 256; };      // N rows
    if constexpr (CHAIN) {
        // first hidden column of h tile `h`: the last tile is shifted back so that it ends at H
        auto h_col = [&](int h) { return min(h * 256, a.H - 256); };
        auto h_origin = [&](int h) { return a.hidden + h_col(h); };  // M rows
        typename Dtl::Stream st;
        bool counted = false;
        Dtl::begin(st, Operand{h_origin(ht), a.H, 256}, Operand{z_origin(vt), a.ldz, 256}, a.tok_valid, smem);
        for (;;) {
            const bool more = walk.has_next();
            int nvt = vt, nht = ht;
            if (more) walk.coords(true, nvt, nht);
            zero_acc(acc);
            // a full tile's epilogue issues TM * TN unconditional stores per wavefront
            Dtl::template tile<true, Acc16::TM * Acc16::TN / 2>(st, h_origin(nht), z_origin(nvt), acc, smem, counted);
            counted = dw_epilogue(acc, a, vt, h_col(ht), ht * 256);
            if (!more) break;
            walk.advance();
            vt = nvt;
            ht = nht;
        }
        Dtl::end(st);
    } else {
        for (;;) {
            Operand A{a.hidden + static_cast<int64_t>(ht) * 256, a.H, min(256, a.H - ht * 256)};
            Operand B{z_origin(vt), a.ldz, 256};
            zero_acc(acc);
            Gemm::run(A, B, a.tok_valid, acc, smem);
            dw_epilogue(acc, a, vt, ht * 256, ht * 256);
            if (!walk.has_next()) break;
            walk.advance();
            walk.coords(false, vt, ht);
        }
    }
}

// db[v] (+)= sum_tok dZ[tok][v] in two fixed-order levels.  Level 1: one workgroup per (256
// columns) x (256-token tile); a thread owns 8 columns (one 16-byte load per row) of every eighth
// row, the eight row groups are added in order through LDS: part[tile][v].  The dZ block is written
// in whole tiles (padding rows and columns hold zeros), so no row or column check is needed here.
template <class T>
__global__ __launch_bounds__(256) void linear_logp_db_partial_kernel(const uint16_t* dz, int64_t ldz, float* part,
                                                                     int64_t part_ld)
{
    __shared__ float red[8][256];
    const int cg = threadIdx.x & 31, rg = threadIdx.x >> 5;
    const int v0 = blockIdx.x * 256 + cg * 8;
    const uint16_t* p = dz + (static_cast<int64_t>(blockIdx.y) * 256 + rg) * ldz + v0;
    float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int k = 0; k < 32; ++k) {
        const u32x4_t w = *reinterpret_cast<const u32x4_t*>(p + static_cast<int64_t>(k) * 8 * ldz);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sum[2 * e] += T::to_float(static_cast<uint16_t>(w[e] & 0xffffu));
            sum[2 * e + 1] += T::to_float(static_cast<uint16_t>(w[e] >> 16));
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) red[rg][cg * 8 + e] = sum[e];
    __syncthreads();
    float acc = red[0][threadIdx.x];
#pragma unroll
    for (int r = 1; r < 8; ++r) acc += red[r][threadIdx.x];
    part[static_cast<int64_t>(blockIdx.y) * part_ld + blockIdx.x * 256 + threadIdx.x] = acc;
}

// Level 2: the token tiles of the block in ascending order, times 1 / loss_scale.
__global__ void linear_logp_db_finish_kernel(const float* part, int64_t part_ld, int tok_tiles, int v_valid,
                                             const float* scales, float* db, int accumulate)
{
    const int v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= v_valid) return;
    float sum = part[v];
    for (int t = 1; t < tok_tiles; ++t) sum += part[static_cast<int64_t>(t) * part_ld + v];
    sum *= scales[1];
    db[v] = accumulate ? db[v] + sum : sum;
}

// scales[0] = loss_scale / T, scales[1] = 1 / loss_scale.  For f16 the loss scale is the power of
// two that brings max|g|/T to about 2^12 so that tiny probabilities survive the f16 dZ; bf16 uses 1.
__global__ void linear_logp_scales_kernel(const float* grad, int n, float inv_temperature,
                                          int dtype, float* scales)
{
    __shared__ float red[1024];
    float mx = 0.f;
    if (dtype == 1) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const float g = fabsf(grad[i]);
            if (g == g && g != INFINITY) mx = fmaxf(mx, g);
        }
    }
    red[threadIdx.x] = mx;
    __syncthreads();
    for (unsigned o = blockDim.x / 2; o > 0; o >>= 1) {
        if (threadIdx.x < o) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + o]);
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        float ls = 1.f;
        if (dtype == 1) {
            const float top = red[0] * inv_temperature;
            if (top > 0.f) {
                int e;
                frexpf(top, &e);  // top = f * 2^e, f in [0.5, 1)
                int shift = 12 - e;
                shift = shift < -24 ? -24 : (shift > 60 ? 60 : shift);
                ls = ldexpf(1.f, shift);
            }
        }
        scales[0] = ls * inv_temperature;
        scales[1] = 1.f / ls;
    }
}

}  // namespace rlk

// ------------------------------------------------------------------------------------------- //
// C ABI
// ------------------------------------------------------------------------------------------- //
using namespace rlk;

namespace {

constexpr int kBK = RLK_BK;

// Forward launch plan: a pure function of (N, H, V, which kernels run).
//   fast launch   : full vocab tiles [0, full_tiles) split n_fast ways
//   general launch: the ragged last tile (all tiles for the fp32 kernels) split n_gen ways
struct FwdPlan {
    int row_blocks;
    int patch_rows;
    int fast_tiles, n_fast;
    int gen_tiles, n_gen;
    int total_splits;
};

// Token blocks per XCD patch.  The 32 workgroups resident on one XCD cover patch_rows token blocks
// x 32 / patch_rows vocab splits; the hidden blocks of all eight patches in flight (8 x patch_rows
// x 256 x H x 2 bytes) are re-read for every vocab tile and should stay inside the 256 MB
// memory-side cache next to the weight tiles: 8 blocks up to H = 4096, 4 up to 8192, 2 beyond
// (measured at H = 8192 with 16384 tokens and more: 8 blocks 1268 TFLOP/s).
int patch_rows_for(int H)
{
    return H <= 4096 ? 8 : (H <= 8192 ? 4 : 2);
}

// Vocab splits of one forward launch.  The launch is row_blocks x splits workgroups, one per CU at
// a time, each walking ceil(tiles / splits) vocab tiles: it takes ceil(workgroups / 256) rounds of
// the 256 CUs, so a count that lands just above a multiple of 256 wastes most of a round (88 token
// blocks x 6 splits = 528 workgroups ran three rounds for the work of two: 976 instead of 1370
// TFLOP/s).  The count with the lowest rounds x (run + half a tile of start-up and state flush)
// wins, a smaller one when it is within 1.5 %, among the counts that leave every workgroup a run of
// at least 8 tiles and keep the split partials (12 bytes per token and split) within the 8 MiB the
// allocation-free entry point has; measured over 4 - 32 splits at 48 - 243 token blocks, this
// choice is within 1.5 % of the best count tried.
int split_count(int row_blocks, int tiles, int patch_rows)
{
    if (tiles <= 0) return 0;
    // At least 32 / patch_rows splits when each still gets a long run of tiles: the 32 workgroups
    // resident on one XCD then form a compact (token blocks x splits) patch that fetches 12 distinct
    // operand streams into its L2 (8 x 4 or 4 x 8) instead of 18 (16 x 2) or 33 (32 x 1); with 243
    // token blocks, 2 or 3 splits ran at 1160 - 1190 TFLOP/s where 4 ran at 1383.
    const int want = 32 / patch_rows;
    const int lo = tiles >= want * 16 ? want : 1;
    int hi = tiles < 64 ? tiles : 64;
    const int64_t fit = static_cast<int64_t>(RLK_STATIC_SCRATCH_BYTES) / (3072LL * row_blocks);
    if (hi > fit) hi = fit > lo ? static_cast<int>(fit) : lo;
    int best = lo;
    int64_t best_cost = -1;
    for (int s = lo; s <= hi; ++s) {
        const int64_t run = (tiles + s - 1) / s;
        if (s > lo && run < 8) break;
        const int64_t rounds = (static_cast<int64_t>(row_blocks) * s + 255) / 256;
        const int64_t cost = rounds * (2 * run + 1);
        // a larger count has to be 1.5 % better than the best smaller one to replace it
        if (best_cost < 0 || cost * 1000 < best_cost * 985) {
            best = s;
            best_cost = cost;
        }
    }
    return best;
}

FwdPlan fwd_plan(int64_t N, int H, int64_t V, bool all_general)
{
    FwdPlan p;
    p.row_blocks = static_cast<int>((N + 255) / 256);
    p.patch_rows = patch_rows_for(H);
    const int all = static_cast<int>((V + 255) / 256);
    const int full = static_cast<int>(V / 256);
    p.fast_tiles = all_general ? 0 : full;
    p.gen_tiles = all - p.fast_tiles;
    p.n_fast = split_count(p.row_blocks, p.fast_tiles, p.patch_rows);
    p.n_gen = split_count(p.row_blocks, p.gen_tiles, p.patch_rows);
    p.total_splits = p.n_fast + p.n_gen;
    return p;
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// One dZ block is at least one 256 x 256 tile and at most RLK_MAX_DZ_BUDGET bytes: the tile
// loaders address rows inside a tile with 32-bit byte offsets (256 rows x leading dimension), so
// the leading dimension of the block must stay below 2^23 elements.
inline size_t clamp_dz_budget(size_t budget)
{
    if (budget == 0) budget = RLK_DEFAULT_DZ_BUDGET;
    if (budget < 131072) budget = 131072;
    if (budget > RLK_MAX_DZ_BUDGET) budget = RLK_MAX_DZ_BUDGET;
    return budget;
}

struct BwdPlan {
    int tok_chunk;   // tokens per chunk (multiple of 256)
    int v_piece;     // vocab rows per piece (multiple of 256)
    int n_chunks;
    int n_pieces;
    int ksplit;      // dH launch of a full block: parts of the piece's vocab range computed side by
                     // side; a shorter last chunk / last piece takes its own count (dh_parts)
    int64_t ldz;     // elements between consecutive token rows of the dZ block
    size_t dz_bytes;
    size_t acc_bytes;
    size_t part_bytes;
    size_t db_bytes;
    size_t scales_off, dz_off, acc_off, part_off, db_off, total;
};

// Cost of the three launches of one dZ block of ct x pt tiles, in K steps of one CU: a launch of
// t tiles occupies ceil(t / 256) rounds of the 256 CUs, a tile costs its K steps plus an epilogue.
// Measured on MI355X with wall-clock stamps inside the kernels, one K step (256 x 256 x 64) takes
// about 1.56 us in all three kernels; the dZ epilogue (exp + 16-bit store) 4.4 us = 3 steps, the
// fp32 read-modify-write of a dH or dW tile 13 - 14 us = 9 steps.
// Few tokens or a narrow hidden dimension: a dH launch of at most 128 tiles over a long vocab range
// is cut into parts that run side by side (fp32 slots, added up in slot order afterwards).
inline int dh_parts(int64_t ct, int64_t pt, int64_t ht)
{
    const int64_t tiles = ct * ht;
    int parts = 1;
    if (tiles <= 128 && pt >= 32) {
        int64_t lim = 256 / tiles;
        if (lim > pt / 16) lim = pt / 16;
        if (lim > 8) lim = 8;
        while (parts * 2 <= lim) parts *= 2;
    }
    return parts;
}

inline int64_t block_cost(int64_t ct, int64_t pt, int64_t ht, int64_t hk)
{
    const int64_t dz = (ct * pt + 255) / 256 * (hk + 3);
    const int parts = dh_parts(ct, pt, ht);
    // split launch: every part is a workgroup of its own; the slot reduction costs about 10 steps
    const int64_t dh = parts > 1 ? (ct * ht * parts + 255) / 256 * (4 * pt / parts + 9) + 10
                                 : (ct * ht + 255) / 256 * (4 * pt + 9);
    const int64_t dw = (pt * ht + 255) / 256 * (4 * ct + 9);
    return dz + dh + dw;
}

// Token chunks x vocab pieces such that one dZ block stays within `budget` bytes and block plus
// fp32 dH accumulator within 1.5 x budget.  Among the shapes that fit, the one with the lowest
// modelled time wins: tile counts just above a multiple of 256 waste most of a round, and small
// blocks pay the read-modify-write epilogues more often.
BwdPlan bwd_plan(int64_t N, int H, int64_t V, size_t budget)
{
    struct Key {
        int64_t N, V;
        int H;
        size_t budget;
        BwdPlan plan;
    };
    static thread_local Key memo{0, 0, 0, 0, {}};
    if (memo.N == N && memo.V == V && memo.H == H && memo.budget == budget) return memo.plan;

    const int64_t n_t = (N + 255) / 256, v_t = (V + 255) / 256;
    const int64_t ht = (H + 255) / 256, hk = (H + kBK - 1) / kBK;
    const int64_t tile_bytes = 131072;                          // 256 x 256 16-bit
    const int64_t max_tiles = static_cast<int64_t>(budget) / tile_bytes;
    const int64_t cap = static_cast<int64_t>(budget) + static_cast<int64_t>(budget) / 2;

    // candidate sizes: balanced splits ceil(x / k) and multiples of 8 tiles
    auto candidates = [](int64_t x, std::vector<int64_t>& out) {
        for (int64_t k = 1; k <= x; ++k) {
            const int64_t c = (x + k - 1) / k;
            if (out.empty() || out.back() != c) out.push_back(c);
        }
        for (int64_t c = 8; c <= x; c += 8) out.push_back(c);
    };
    std::vector<int64_t> cts, pts;
    candidates(n_t, cts);
    candidates(v_t, pts);

    int64_t best_ct = 1, best_pt = 1, best_cost = -1, best_bytes = 0;
    for (int64_t ct : cts) {
        if (ct > max_tiles) continue;
        const int64_t nc = (n_t + ct - 1) / ct, ct_last = n_t - (nc - 1) * ct;
        for (int64_t pt : pts) {
            if (ct * pt > max_tiles) continue;
            const int64_t np = (v_t + pt - 1) / pt, pt_last = v_t - (np - 1) * pt;
            const int64_t bytes = ct * pt * tile_bytes + (np > 1 ? ct * 256 * H * 4 : 0);
            if (bytes > cap && ct * pt > 1) continue;
            const int64_t cost = (nc - 1) * (np - 1) * block_cost(ct, pt, ht, hk) +
                                 (np - 1) * block_cost(ct_last, pt, ht, hk) +
                                 (nc - 1) * block_cost(ct, pt_last, ht, hk) +
                                 block_cost(ct_last, pt_last, ht, hk);
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && bytes < best_bytes)) {
                best_cost = cost;
                best_ct = ct;
                best_pt = pt;
                best_bytes = bytes;
            }
        }
    }

    BwdPlan p;
    p.tok_chunk = static_cast<int>(best_ct) * 256;
    p.v_piece = static_cast<int>(best_pt) * 256;
    p.n_chunks = static_cast<int>((n_t + best_ct - 1) / best_ct);
    p.n_pieces = static_cast<int>((v_t + best_pt - 1) / best_pt);
    p.ldz = p.v_piece;
    p.dz_bytes = static_cast<size_t>(p.tok_chunk) * p.ldz * 2;
    p.acc_bytes = p.n_pieces > 1 ? static_cast<size_t>(p.tok_chunk) * H * 4 : 0;
    p.scales_off = 0;
    p.dz_off = 256;
    p.acc_off = p.dz_off + align_up(p.dz_bytes, 256);
    // Few tokens: the dH launch has fewer tiles than the chip has CUs but a long vocab range, so
    // the range is cut into parts that run side by side and are added up in a fixed order.
    p.ksplit = dh_parts(best_ct, best_pt, ht);
    // fp32 slots of the split dH launches: every (chunk, piece) kind picks its own part count, so
    // a short last chunk does not run its few tiles on a quarter of the chip
    const int64_t ct_last = n_t - (p.n_chunks - 1) * best_ct, pt_last = v_t - (p.n_pieces - 1) * best_pt;
    p.part_bytes = 0;
    for (int64_t ct : {best_ct, ct_last})
        for (int64_t pt : {best_pt, pt_last}) {
            const int parts = dh_parts(ct, pt, ht);
            if (parts > 1)
                p.part_bytes = std::max(p.part_bytes, static_cast<size_t>(parts) * ct * 256 * H * 4);
        }
    p.part_off = p.acc_off + align_up(p.acc_bytes, 256);
    // per-token-tile column sums of the dZ block (d_bias): 1 KiB per dZ tile
    p.db_bytes = static_cast<size_t>(best_ct) * p.v_piece * 4;
    p.db_off = p.part_off + align_up(p.part_bytes, 256);
    p.total = p.db_off + align_up(p.db_bytes, 256);
    memo = Key{N, V, H, budget, p};
    return p;
}

// Raises the dynamic-LDS limit of `kernel` to `bytes` on the current device.  The attribute is
// per device and sticks, so each (kernel instance, device) pair pays the runtime call once.
template <class K>
int set_smem(K kernel, int bytes)
{
    constexpr int kMaxDev = 64;
    static std::mutex mu;
    static int done[kMaxDev] = {};  // one table per template instance = per kernel
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, hipGetErrorString(e));
    const bool tracked = dev >= 0 && dev < kMaxDev;
    if (tracked) {
        std::lock_guard<std::mutex> lock(mu);
        if (done[dev] >= bytes) return 0;
    }
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, hipGetErrorString(e));
    if (tracked) {
        std::lock_guard<std::mutex> lock(mu);
        if (done[dev] < bytes) done[dev] = bytes;
    }
    return 0;
}

int check_launch(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, what);
    return 0;
}

int check_common(int64_t N, int32_t H, int64_t V, int dtype)
{
    if (dtype != RLK_DTYPE_BF16 && dtype != RLK_DTYPE_F16 && dtype != RLK_DTYPE_F32)
        return rlk_fail(RLK_ERR_UNSUPPORTED, "dtype must be RLK_DTYPE_BF16, RLK_DTYPE_F16 or RLK_DTYPE_F32");
    if (N <= 0 || H <= 0 || V <= 0) return rlk_fail(RLK_ERR_ARG, "N, H and V must be positive");
    if (N > 0x7fff0000LL || V > 0x7fff0000LL) return rlk_fail(RLK_ERR_ARG, "N or V too large");
    if (H > (1 << 20)) return rlk_fail(RLK_ERR_UNSUPPORTED, "hidden size above 2^20");
    return 0;
}

// The 16-bit MFMA tiles take bf16 / f16 inputs whose rows start on 16-byte boundaries; everything
// else runs on the fp32 matrix-core kernels (rlk_wide.hip).
bool use_mfma(const void* hidden, const void* weight, int32_t H, int dtype)
{
    return (dtype == RLK_DTYPE_BF16 || dtype == RLK_DTYPE_F16) && H % 8 == 0 &&
           (reinterpret_cast<uintptr_t>(hidden) & 15) == 0 && (reinterpret_cast<uintptr_t>(weight) & 15) == 0;
}

// Compute units of the current device (looked up once per device): the chained kernels launch
// one workgroup per compute unit.  Which workgroup computes a tile never changes the tile's bits.
int compute_units(int* out)
{
    constexpr int kMaxDev = 64;
    static std::mutex mu;
    static int cached[kMaxDev] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDev) return rlk_fail(RLK_ERR_UNSUPPORTED, "device index too large");
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == 0) {
        int n = 0;
        e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess || n <= 0) return rlk_fail(RLK_ERR_LAUNCH, "cannot read the compute-unit count");
        cached[dev] = n;
    }
    *out = cached[dev];
    return 0;
}

struct BwdCall {
    const float* grad_logp;
    const void* hidden;
    const void* weight;
    const float* bias;
    const int64_t* targets;
    const float* lse;
    void* d_hidden;
    float* d_weight;
    float* d_bias;
    void* workspace;
    int64_t N;
    int32_t H;
    int64_t V;
    int64_t vocab_start;
    int32_t dtype;
    float temperature;
    int64_t ignore_index;
    int32_t use_ignore;
    hipStream_t stream;
    int accumulate;  // 1: d_weight / d_bias already hold the sums of earlier tokens, add to them
};

// Grid of a chained launch: one workgroup per compute unit, rounded down to a multiple of 8 so
// that a workgroup stays on one XCD from round to round; never more workgroups than tiles.
inline int chain_grid(int tiles, int n_cu)
{
    int g = n_cu >= 8 ? n_cu / 8 * 8 : n_cu;
    return tiles < g ? tiles : g;
}

// Enqueues the backward schedule: for every (token chunk, vocab piece) block
//   dZ recompute -> dH (+)= dZ W -> dW (+)= dZ^T hidden (-> db).
template <class T>
int bwd_enqueue(const BwdCall& c, const BwdPlan& p, int n_cu)
{
    using GZ = TileGemm<T, false, false, kBK>;
    using GH = TileGemm<T, true, false, kBK>;
    using GW = TileGemm<T, true, true, kBK>;
    constexpr int kChainSmem = TileGemmDtl<T, false, false, kBK, 32>::kSmemBytes;
    constexpr int kDzChainSmem = kChainSmem + kDzStageBytes * (kThreads / 64);
    const int H = c.H;
    const int64_t N = c.N, V = c.V;
    hipStream_t stream = c.stream;

    char* ws = static_cast<char*>(c.workspace);
    float* scales = reinterpret_cast<float*>(ws + p.scales_off);
    uint16_t* dz = reinterpret_cast<uint16_t*>(ws + p.dz_off);
    float* hacc = p.acc_bytes ? reinterpret_cast<float*>(ws + p.acc_off) : nullptr;
    const uint16_t* hid = static_cast<const uint16_t*>(c.hidden);
    const uint16_t* w = static_cast<const uint16_t*>(c.weight);
    uint16_t* dh = static_cast<uint16_t*>(c.d_hidden);
    const int h_tiles = (H + 255) / 256;

    hipLaunchKernelGGL(linear_logp_scales_kernel, dim3(1), dim3(1024), 0, stream, c.grad_logp,
                       static_cast<int>(N), 1.f / c.temperature, c.dtype, scales);
    if (int rc = check_launch("scales kernel launch failed")) return rc;

    if (int rc = set_smem(linear_logp_dz_kernel<T, kBK, false, true>, kDzChainSmem)) return rc;
    if (int rc = set_smem(linear_logp_dz_kernel<T, kBK, false, false>, GZ::kSmemBytes)) return rc;
    if (int rc = set_smem(linear_logp_dz_kernel<T, kBK, true, false>, GZ::kSmemBytes)) return rc;
    if (int rc = set_smem(linear_logp_dh_kernel<T, kBK, true>, kChainSmem)) return rc;
    if (int rc = set_smem(linear_logp_dh_kernel<T, kBK, false>, GH::kSmemBytes)) return rc;
    if (int rc = set_smem(linear_logp_dw_kernel<T, kBK, true>, kChainSmem)) return rc;
    if (int rc = set_smem(linear_logp_dw_kernel<T, kBK, false>, GW::kSmemBytes)) return rc;

    for (int ci = 0; ci < p.n_chunks; ++ci) {
        const int64_t tok_lo = static_cast<int64_t>(ci) * p.tok_chunk;
        const int tok_valid = static_cast<int>((N - tok_lo) < p.tok_chunk ? (N - tok_lo) : p.tok_chunk);
        if (tok_valid <= 0) break;
        const int tok_tiles = (tok_valid + 255) / 256;
        for (int pi = 0; pi < p.n_pieces; ++pi) {
            const int64_t v_lo = static_cast<int64_t>(pi) * p.v_piece;
            const int v_valid = static_cast<int>((V - v_lo) < p.v_piece ? (V - v_lo) : p.v_piece);
            if (v_valid <= 0) break;
            const int v_tiles = (v_valid + 255) / 256;
            const bool last_piece = (v_lo + p.v_piece >= V);

            DzArgs z;
            z.hidden = hid + tok_lo * H;
            z.weight = w + v_lo * H;
            z.bias = c.bias ? c.bias + v_lo : nullptr;
            z.targets = c.targets + tok_lo;
            z.lse = c.lse + tok_lo;
            z.grad = c.grad_logp + tok_lo;
            z.scales = scales;
            z.dz = dz;
            z.ldz = p.ldz;
            z.tok_valid = tok_valid;
            z.v_valid = v_valid;
            z.H = H;
            z.tok_tiles = tok_tiles;
            z.v_global0 = c.vocab_start + v_lo;
            z.ignore_index = c.ignore_index;
            z.use_ignore = c.use_ignore;
            z.scale2 = kLog2e / c.temperature;

            DhArgs h;
            h.dz = dz;
            h.weight = w + v_lo * H;
            h.scales = scales;
            h.acc = hacc;
            h.out = dh ? dh + tok_lo * H : nullptr;
            h.ldz = p.ldz;
            h.H = H;
            h.v_valid = v_valid;
            h.tok_valid = tok_valid;
            h.tok_tiles = tok_tiles;
            h.h_tiles = h_tiles;
            h.first = pi == 0;
            h.last = last_piece;
            // same rule as the plan's cost model: per (chunk, piece) kind
            const int ksplit = dh_parts(tok_tiles, v_tiles, h_tiles);
            h.ksplit = ksplit;
            h.part = ksplit > 1 ? reinterpret_cast<float*>(ws + p.part_off) : nullptr;
            h.part_stride = static_cast<int64_t>(tok_tiles) * 256 * H;

            DwArgs d;
            d.dz = dz;
            d.hidden = hid + tok_lo * H;
            d.scales = scales;
            d.dw = c.d_weight ? c.d_weight + v_lo * H : nullptr;
            d.ldz = p.ldz;
            d.H = H;
            d.v_valid = v_valid;
            d.tok_valid = tok_valid;
            d.v_tiles = v_tiles;
            d.h_tiles = h_tiles;
            d.accumulate = ci > 0 || c.accumulate != 0;

            // dZ block: full vocab tiles through the fast variant (chained through one pipeline
            // when the token tiles are full too), the ragged last one through the general one
            const int fast_tiles = v_valid / 256;
            const int gen_tiles = v_tiles - fast_tiles;
            const bool k_ok = H % kBK == 0 && H >= 2 * kBK;
            if (fast_tiles > 0) {
                z.v_tiles = fast_tiles;
                z.v_tile_lo = 0;
                const int tiles = tok_tiles * fast_tiles;
                if (k_ok && tok_valid % 256 == 0)
                    hipLaunchKernelGGL((linear_logp_dz_kernel<T, kBK, false, true>),
                                       dim3(chain_grid(tiles, n_cu)), dim3(kThreads), kDzChainSmem,
                                       stream, z);
                else
                    hipLaunchKernelGGL((linear_logp_dz_kernel<T, kBK, false, false>), dim3(tiles),
                                       dim3(kThreads), GZ::kSmemBytes, stream, z);
            }
            if (gen_tiles > 0) {
                z.v_tiles = gen_tiles;
                z.v_tile_lo = fast_tiles;
                hipLaunchKernelGGL((linear_logp_dz_kernel<T, kBK, true, false>),
                                   dim3(tok_tiles * gen_tiles), dim3(kThreads), GZ::kSmemBytes,
                                   stream, z);
            }
            if (dh) {
                const int tiles = tok_tiles * h_tiles;
                if (ksplit == 1 && H >= 256 && v_valid % kBK == 0 && v_valid >= 2 * kBK) {
                    hipLaunchKernelGGL((linear_logp_dh_kernel<T, kBK, true>),
                                       dim3(chain_grid(tiles, n_cu)), dim3(kThreads), kChainSmem,
                                       stream, h);
                } else {
                    hipLaunchKernelGGL((linear_logp_dh_kernel<T, kBK, false>),
                                       dim3(tiles * ksplit), dim3(kThreads), GH::kSmemBytes, stream, h);
                    if (ksplit > 1) {
                        const int64_t n4 = static_cast<int64_t>(tok_valid) * H / 4;
                        hipLaunchKernelGGL((linear_logp_dh_reduce_kernel<T>),
                                           dim3(static_cast<unsigned>((n4 + 255) / 256)), dim3(256), 0,
                                           stream, h.part, ksplit, h.part_stride, h.acc, h.out,
                                           scales, n4, h.first, h.last);
                    }
                }
            }
            if (c.d_weight) {
                const int tiles = v_tiles * h_tiles;
                if (H >= 256 && tok_valid % kBK == 0 && tok_valid >= 2 * kBK)
                    hipLaunchKernelGGL((linear_logp_dw_kernel<T, kBK, true>),
                                       dim3(chain_grid(tiles, n_cu)), dim3(kThreads), kChainSmem,
                                       stream, d);
                else
                    hipLaunchKernelGGL((linear_logp_dw_kernel<T, kBK, false>), dim3(tiles),
                                       dim3(kThreads), GW::kSmemBytes, stream, d);
            }
            if (c.d_bias != nullptr) {
                float* db_part = reinterpret_cast<float*>(ws + p.db_off);
                hipLaunchKernelGGL(linear_logp_db_partial_kernel<T>, dim3(v_tiles, tok_tiles), dim3(256), 0,
                                   stream, dz, p.ldz, db_part, static_cast<int64_t>(p.v_piece));
                hipLaunchKernelGGL(linear_logp_db_finish_kernel, dim3((v_valid + 255) / 256), dim3(256), 0,
                                   stream, db_part, static_cast<int64_t>(p.v_piece), tok_tiles, v_valid,
                                   scales, c.d_bias + v_lo, (ci > 0 || c.accumulate != 0) ? 1 : 0);
            }
            if (int rc = check_launch("linear_logp backward launch failed")) return rc;
        }
    }
    return 0;
}

// One forward contraction launch: a.row_blocks x a.n_split workgroups of the given variant.
template <class T, bool GENERAL>
int launch_fwd_as(const FwdArgs& a, hipStream_t stream)
{
    using G = TileGemm<T, false, false, kBK>;
    if (int rc = set_smem(linear_logp_fwd_kernel<T, kBK, GENERAL>, G::kSmemBytes)) return rc;
    hipLaunchKernelGGL((linear_logp_fwd_kernel<T, kBK, GENERAL>), dim3(a.row_blocks * a.n_split),
                       dim3(kThreads), G::kSmemBytes, stream, a);
    return 0;
}

template <bool GENERAL>
int launch_fwd(const FwdArgs& a, int32_t dtype, hipStream_t stream)
{
    return dtype == RLK_DTYPE_BF16 ? launch_fwd_as<Bf16, GENERAL>(a, stream)
                                   : launch_fwd_as<F16, GENERAL>(a, stream);
}

// A second head over the same hidden states and targets (a frozen reference model).
struct SecondHead {
    const void* weight;
    const float* bias;
    float* logp;
    float* lse;
};

int fwd_enqueue(const void* hidden, const void* weight, const float* bias, const int64_t* targets,
                float* logp, float* lse, void* workspace, size_t workspace_bytes, int64_t N,
                int32_t H, int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                int32_t* err_flag, hipStream_t stream, const GrpoArgs* epilogue = nullptr,
                const SecondHead* second = nullptr);

}  // namespace

// Scratch of rlk_linear_logp_fwd_static: the forward's per-split partial softmax states live in
// this file-scope device array instead of a caller workspace, so that entry point allocates
// nothing.  Every GPU the library runs on holds its own copy until the process ends.  In host code
// the array's name is only a handle; the device address is looked up once per device below and
// that pointer is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[RLK_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (resolved on the first call per device).
int static_scratch_ptr(void** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return rlk_fail(RLK_ERR_LAUNCH, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return rlk_fail(RLK_ERR_UNSUPPORTED, "device index too large");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return rlk_fail(RLK_ERR_LAUNCH, e != hipSuccess ? hipGetErrorString(e)
                                                            : "static scratch has no device address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace

extern "C" {

int rlk_linear_logp_fwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                        size_t* bytes)
{
    (void)dtype;
    if (!bytes || N <= 0 || V <= 0 || H <= 0) return rlk_fail(RLK_ERR_ARG, "bad workspace query");
    // sized for the larger of the two plans so that one query serves both kinds of kernels
    const int a = fwd_plan(N, H, V, false).total_splits, b = fwd_plan(N, H, V, true).total_splits;
    *bytes = static_cast<size_t>(3) * (a > b ? a : b) * N * sizeof(float);
    return 0;
}

int rlk_linear_logp_fwd(const void* hidden, const void* weight, const float* bias,
                        const int64_t* targets, float* logp, float* lse, void* workspace,
                        size_t workspace_bytes, int64_t N, int32_t H, int64_t V,
                        int64_t vocab_start, int32_t dtype, float temperature,
                        int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                        int32_t* err_flag, hipStream_t stream)
{
    return fwd_enqueue(hidden, weight, bias, targets, logp, lse, workspace, workspace_bytes, N, H, V,
                       vocab_start, dtype, temperature, ignore_index, use_ignore, strict_targets,
                       err_flag, stream);
}

int rlk_linear_logp_fwd_static(const void* hidden, const void* weight, const float* bias,
                               const int64_t* targets, float* logp, float* lse, int64_t N,
                               int32_t H, int64_t V, int64_t vocab_start, int32_t dtype,
                               float temperature, int64_t ignore_index, int32_t use_ignore,
                               int32_t strict_targets, int32_t* err_flag, hipStream_t stream)
{
    if (int rc = check_common(N, H, V, dtype)) return rc;
    size_t need = 0;
    if (int rc = rlk_linear_logp_fwd_workspace_bytes(N, H, V, dtype, &need)) return rc;
    if (need > static_cast<size_t>(RLK_STATIC_SCRATCH_BYTES))
        return rlk_fail(RLK_ERR_ARG,
                        "rlk_linear_logp_fwd_static: the split partials of this N exceed the "
                        "library's static scratch (RLK_STATIC_SCRATCH_BYTES); use "
                        "rlk_linear_logp_fwd with a caller workspace");
    void* ws = nullptr;
    if (int rc = static_scratch_ptr(&ws)) return rc;
    return fwd_enqueue(hidden, weight, bias, targets, logp, lse, ws, RLK_STATIC_SCRATCH_BYTES, N, H,
                       V, vocab_start, dtype, temperature, ignore_index, use_ignore,
                       strict_targets, err_flag, stream);
}

int rlk_linear_logp_fwd_pair_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                             size_t* bytes)
{
    if (int rc = rlk_linear_logp_fwd_workspace_bytes(N, H, V, dtype, bytes)) return rc;
    *bytes *= 2;
    return 0;
}

int rlk_linear_logp_fwd_pair(const void* hidden, const void* weight, const void* ref_weight,
                             const float* bias, const float* ref_bias, const int64_t* targets,
                             float* logp, float* lse, float* ref_logp, float* ref_lse,
                             void* workspace, size_t workspace_bytes, int64_t N, int32_t H,
                             int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                             int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                             int32_t* err_flag, hipStream_t stream)
{
    if (!ref_weight || !ref_logp || !ref_lse) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if ((bias == nullptr) != (ref_bias == nullptr))
        return rlk_fail(RLK_ERR_UNSUPPORTED, "both heads must have a bias or neither");
    const SecondHead second{ref_weight, ref_bias, ref_logp, ref_lse};
    return fwd_enqueue(hidden, weight, bias, targets, logp, lse, workspace, workspace_bytes, N, H, V,
                       vocab_start, dtype, temperature, ignore_index, use_ignore, strict_targets,
                       err_flag, stream, nullptr, &second);
}

int rlk_linear_logp_fwd_grpo_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                             size_t* bytes)
{
    size_t fwd = 0, epi = 0;
    if (int rc = rlk_linear_logp_fwd_workspace_bytes(N, H, V, dtype, &fwd)) return rc;
    if (int rc = rlk_grpo_loss_workspace_bytes(N, &epi)) return rc;
    *bytes = (fwd + 255) / 256 * 256 + epi;
    return 0;
}

int rlk_linear_logp_fwd_grpo(const void* hidden, const void* weight, const float* bias,
                             const int64_t* targets, float* logp, float* lse, void* workspace,
                             size_t workspace_bytes, int64_t N, int32_t H, int64_t V,
                             int64_t vocab_start, int32_t dtype, float temperature,
                             int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                             int32_t* err_flag, const float* old_logp, const float* ref_logp,
                             const float* advantages, int32_t adv_per_token, const uint8_t* mask,
                             int64_t seq_len, float clip_eps, float beta, float* out3, float* ratio,
                             float* kl_terms, float* d_cur, float* d_kl, hipStream_t stream)
{
    if (int rc = check_common(N, H, V, dtype)) return rc;
    if (!old_logp || !advantages || !out3 || !logp) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (seq_len <= 0) return rlk_fail(RLK_ERR_ARG, "bad sizes");
    if (!adv_per_token && N % seq_len != 0)
        return rlk_fail(RLK_ERR_ARG, "N must be a multiple of seq_len for per-sequence advantages");
    if (d_kl != nullptr && d_cur == nullptr) return rlk_fail(RLK_ERR_ARG, "d_kl requires d_cur");
    size_t need = 0, fwd = 0;
    if (int rc = rlk_linear_logp_fwd_grpo_workspace_bytes(N, H, V, dtype, &need)) return rc;
    rlk_linear_logp_fwd_workspace_bytes(N, H, V, dtype, &fwd);
    if (!workspace || workspace_bytes < need) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 15) return rlk_fail(RLK_ERR_ARG, "workspace must be 16-byte aligned");
    GrpoArgs g;
    g.cur = logp;
    g.old_lp = old_logp;
    g.ref_lp = ref_logp;
    g.adv = advantages;
    g.mask = mask;
    g.ratio = ratio;
    g.kl_terms = kl_terms;
    g.partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + (fwd + 255) / 256 * 256);
    g.denom = g.partial + kMaxBlocks * 3;
    g.words = reinterpret_cast<int*>(g.denom + 4);
    g.out3 = out3;
    g.dcur = d_cur;
    g.dkl = d_kl;
    g.upstream = nullptr;
    g.n = N;
    g.seq_len = seq_len;
    g.adv_per_token = adv_per_token;
    g.clip_lo = 1.f - clip_eps;
    g.clip_hi = 1.f + clip_eps;
    g.beta = beta;
    g.blocks = grpo_blocks(N);
    return fwd_enqueue(hidden, weight, bias, targets, logp, lse, workspace, fwd, N, H, V, vocab_start,
                       dtype, temperature, ignore_index, use_ignore, strict_targets, err_flag, stream,
                       &g);
}

}  // extern "C"

namespace {

// `epilogue` (optional): GRPO loss arguments whose `cur` is the logp this call produces; the
// per-token loss pass then runs inside the combine launch.
int fwd_enqueue(const void* hidden, const void* weight, const float* bias, const int64_t* targets,
                float* logp, float* lse, void* workspace, size_t workspace_bytes, int64_t N,
                int32_t H, int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                int64_t ignore_index, int32_t use_ignore, int32_t strict_targets,
                int32_t* err_flag, hipStream_t stream, const GrpoArgs* epilogue,
                const SecondHead* second)
{
    if (int rc = check_common(N, H, V, dtype)) return rc;
    if (!(temperature > 0.f)) return rlk_fail(RLK_ERR_ARG, "temperature must be greater than zero");
    if (!hidden || !weight || !targets || !logp || !lse) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (strict_targets && !err_flag)
        return rlk_fail(RLK_ERR_ARG, "strict_targets needs an err_flag to report through");
    const bool mfma = use_mfma(hidden, weight, H, dtype);
    // Both heads of a pair run through one launch, so they must take the same kind of kernel:
    // otherwise the policy head's results would depend on the reference head's alignment and no
    // longer equal the single-head call bit for bit.
    if (second != nullptr && use_mfma(hidden, second->weight, H, dtype) != mfma)
        return rlk_fail(RLK_ERR_UNSUPPORTED,
                        "rlk_linear_logp_fwd_pair: weight and ref_weight must both start on a 16-byte "
                        "boundary or neither (one would run on the 16-bit MFMA tiles, the other on the "
                        "fp32 matrix-core kernels); call rlk_linear_logp_fwd once per head instead");
    size_t need = 0;
    rlk_linear_logp_fwd_workspace_bytes(N, H, V, dtype, &need);
    if (second != nullptr) need *= 2;
    if (!workspace || workspace_bytes < need) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    if (epilogue != nullptr) {
        // the active-token count only needs the mask: it is ready long before the contraction ends
        const int parts = grpo_count_parts(epilogue->n);
        hipLaunchKernelGGL(grpo_count_kernel<0>, dim3(parts), dim3(kRedThreads), 0, stream,
                           epilogue->mask, epilogue->n, parts, epilogue->words);
        if (int rc = check_launch("grpo_count_kernel launch failed")) return rc;
    }

    FwdArgs a;
    a.hidden = static_cast<const uint16_t*>(hidden);
    a.weight = static_cast<const uint16_t*>(weight);
    a.bias = bias;
    a.weight2 = second ? static_cast<const uint16_t*>(second->weight) : nullptr;
    a.bias2 = second ? second->bias : nullptr;
    a.targets = targets;
    a.N = static_cast<int>(N);
    a.H = H;
    a.V = static_cast<int>(V);
    a.vocab_start = vocab_start;
    // the fp32 matrix-core kernels treat every tile as general
    const FwdPlan plan = fwd_plan(N, H, V, !mfma);
    a.row_blocks = plan.row_blocks;
    a.patch_rows = plan.patch_rows;
    a.part_m = static_cast<float*>(workspace);
    a.part_s = a.part_m + static_cast<size_t>(plan.total_splits) * N;
    a.part_z = a.part_s + static_cast<size_t>(plan.total_splits) * N;
    a.part2_m = a.part_z + static_cast<size_t>(plan.total_splits) * N;
    a.part2_s = a.part2_m + static_cast<size_t>(plan.total_splits) * N;
    a.part2_z = a.part2_s + static_cast<size_t>(plan.total_splits) * N;
    a.scale2 = kLog2e / temperature;

    if (!mfma) {
        if (int rc = wide_fwd_partials(hidden, weight, bias, targets, a.part_m, a.part_s, a.part_z,
                                       plan.total_splits, N, H, V, vocab_start, dtype, temperature, stream))
            return rc;
        if (second != nullptr)
            if (int rc = wide_fwd_partials(hidden, second->weight, second->bias, targets, a.part2_m,
                                           a.part2_s, a.part2_z, plan.total_splits, N, H, V, vocab_start,
                                           dtype, temperature, stream))
                return rc;
    }
    if (mfma && plan.n_fast > 0) {
        a.n_split = plan.n_fast;
        a.split_lo = 0;
        a.tile_lo = 0;
        a.vtiles = plan.fast_tiles;
        if (int rc = launch_fwd<false>(a, dtype, stream)) return rc;
    }
    if (mfma && plan.n_gen > 0) {
        a.n_split = plan.n_gen;
        a.split_lo = plan.n_fast;
        a.tile_lo = plan.fast_tiles;
        a.vtiles = plan.gen_tiles;
        if (int rc = launch_fwd<true>(a, dtype, stream)) return rc;
    }
    if (int rc = check_launch("linear_logp_fwd_kernel launch failed")) return rc;

    CombineArgs c;
    c.part_m = a.part_m;
    c.part_s = a.part_s;
    c.part_z = a.part_z;
    c.targets = targets;
    c.logp = logp;
    c.lse = lse;
    c.err_flag = err_flag;
    c.N = a.N;
    c.V = a.V;
    c.n_split = plan.total_splits;
    c.vocab_start = vocab_start;
    c.ignore_index = ignore_index;
    c.use_ignore = use_ignore;
    c.strict = strict_targets;
    if (second != nullptr) {  // the reference head: same merge, never strict
        CombineArgs c2 = c;
        c2.part_m = a.part2_m;
        c2.part_s = a.part2_s;
        c2.part_z = a.part2_z;
        c2.logp = second->logp;
        c2.lse = second->lse;
        c2.strict = 0;
        hipLaunchKernelGGL(linear_logp_combine_kernel, dim3((a.N + 255) / 256), dim3(256), 0, stream, c2);
    }
    if (epilogue == nullptr) {
        hipLaunchKernelGGL(linear_logp_combine_kernel, dim3((a.N + 255) / 256), dim3(256), 0, stream, c);
        return check_launch("linear_logp_combine_kernel launch failed");
    }
    hipLaunchKernelGGL(linear_logp_combine_grpo_kernel, dim3(epilogue->blocks), dim3(kRedThreads), 0,
                       stream, c, *epilogue);
    return check_launch("combine + GRPO epilogue launch failed");
}

}  // namespace

extern "C" {

int rlk_linear_logp_bwd_workspace_bytes(int64_t N, int32_t H, int64_t V, int32_t dtype,
                                        size_t dz_budget_bytes, size_t* bytes)
{
    (void)dtype;
    if (!bytes || N <= 0 || V <= 0 || H <= 0) return rlk_fail(RLK_ERR_ARG, "bad workspace query");
    dz_budget_bytes = clamp_dz_budget(dz_budget_bytes);
    // large enough for either implementation (the choice also depends on pointer alignment)
    const size_t a = bwd_plan(N, H, V, dz_budget_bytes).total, b = wide_bwd_workspace(N, H, V, dz_budget_bytes);
    *bytes = a > b ? a : b;
    return 0;
}

int rlk_linear_logp_fwd_plan(int64_t N, int32_t H, int64_t V, int32_t dtype, int64_t* out4)
{
    if (!out4 || N <= 0 || V <= 0 || H <= 0) return rlk_fail(RLK_ERR_ARG, "bad plan query");
    const FwdPlan p = fwd_plan(N, H, V, dtype == RLK_DTYPE_F32);
    out4[0] = p.row_blocks;
    out4[1] = p.n_fast;
    out4[2] = p.n_gen;
    out4[3] = p.patch_rows;
    return 0;
}

int rlk_linear_logp_bwd_plan(int64_t N, int32_t H, int64_t V, int32_t dtype, size_t dz_budget_bytes,
                             int64_t* out5)
{
    (void)dtype;
    if (!out5 || N <= 0 || V <= 0 || H <= 0) return rlk_fail(RLK_ERR_ARG, "bad plan query");
    dz_budget_bytes = clamp_dz_budget(dz_budget_bytes);
    const BwdPlan p = bwd_plan(N, H, V, dz_budget_bytes);
    out5[0] = p.tok_chunk;
    out5[1] = p.v_piece;
    out5[2] = p.n_chunks;
    out5[3] = p.n_pieces;
    out5[4] = p.ksplit;
    return 0;
}

int rlk_linear_logp_bwd(const float* grad_logp, const void* hidden, const void* weight,
                        const float* bias, const int64_t* targets, const float* lse,
                        void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                        size_t workspace_bytes, size_t dz_budget_bytes, int64_t N, int32_t H,
                        int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                        int64_t ignore_index, int32_t use_ignore, hipStream_t stream)
{
    return rlk::linear_logp_bwd_accumulating(grad_logp, hidden, weight, bias, targets, lse, d_hidden,
                                             d_weight, d_bias, workspace, workspace_bytes,
                                             dz_budget_bytes, N, H, V, vocab_start, dtype, temperature,
                                             ignore_index, use_ignore, 0, stream);
}

int rlk_linear_logp_bwd_accum(const float* grad_logp, const void* hidden, const void* weight,
                              const float* bias, const int64_t* targets, const float* lse,
                              void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                              size_t workspace_bytes, size_t dz_budget_bytes, int64_t N, int32_t H,
                              int64_t V, int64_t vocab_start, int32_t dtype, float temperature,
                              int64_t ignore_index, int32_t use_ignore, int32_t accumulate,
                              hipStream_t stream)
{
    return rlk::linear_logp_bwd_accumulating(grad_logp, hidden, weight, bias, targets, lse, d_hidden,
                                             d_weight, d_bias, workspace, workspace_bytes,
                                             dz_budget_bytes, N, H, V, vocab_start, dtype, temperature,
                                             ignore_index, use_ignore, accumulate != 0 ? 1 : 0, stream);
}

}  // extern "C"

int rlk::linear_logp_bwd_accumulating(const float* grad_logp, const void* hidden, const void* weight,
                                      const float* bias, const int64_t* targets, const float* lse,
                                      void* d_hidden, float* d_weight, float* d_bias, void* workspace,
                                      size_t workspace_bytes, size_t dz_budget_bytes, int64_t N,
                                      int32_t H, int64_t V, int64_t vocab_start, int32_t dtype,
                                      float temperature, int64_t ignore_index, int32_t use_ignore,
                                      int32_t accumulate, hipStream_t stream)
{
    if (int rc = check_common(N, H, V, dtype)) return rc;
    if (!(temperature > 0.f)) return rlk_fail(RLK_ERR_ARG, "temperature must be greater than zero");
    if (!grad_logp || !hidden || !weight || !targets || !lse) return rlk_fail(RLK_ERR_ARG, "null pointer");
    if (!d_hidden && !d_weight && !d_bias) return rlk_fail(RLK_ERR_ARG, "no gradient requested");
    if (bias == nullptr && d_bias != nullptr) return rlk_fail(RLK_ERR_ARG, "d_bias given without bias");
    dz_budget_bytes = clamp_dz_budget(dz_budget_bytes);
    size_t need = 0;
    rlk_linear_logp_bwd_workspace_bytes(N, H, V, dtype, dz_budget_bytes, &need);
    if (!workspace || workspace_bytes < need) return rlk_fail(RLK_ERR_ARG, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 255)
        return rlk_fail(RLK_ERR_ARG, "workspace must be 256-byte aligned");
    if (!use_mfma(hidden, weight, H, dtype))
        return wide_bwd(grad_logp, hidden, weight, bias, targets, lse, d_hidden, d_weight, d_bias,
                        workspace, dz_budget_bytes, N, H, V, vocab_start, dtype, temperature,
                        ignore_index, use_ignore, accumulate, stream);
    const BwdPlan p = bwd_plan(N, H, V, dz_budget_bytes);
    int n_cu = 0;
    if (int rc = compute_units(&n_cu)) return rc;
    BwdCall c{grad_logp, hidden, weight, bias, targets, lse, d_hidden, d_weight, d_bias, workspace,
              N, H, V, vocab_start, dtype, temperature, ignore_index, use_ignore, stream, accumulate};
    return dtype == RLK_DTYPE_BF16 ? bwd_enqueue<Bf16>(c, p, n_cu) : bwd_enqueue<F16>(c, p, n_cu);
}
