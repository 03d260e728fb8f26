// Pieces shared by the 16-bit MFMA kernels and the fp32 MFMA kernels of the fused linear-logprob
// path: both work on the same 256 x 256 workgroup tile with the same wavefront grid, and their
// accumulator layouts (16 x 16 and 32 x 32 MFMA tiles) differ only in the constants of AccTile, so
// the code that consumes a finished tile is written once.
#pragma once
#include "rlk_gemm.hpp"

namespace rlk {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Online-softmax update of one wavefront slab (128 vocab rows x 64 tokens) held in `acc`, for
// either accumulator geometry AT (see AccTile).  `a` supplies V (vocab rows of the shard) and scale2
// (log2(e) / temperature).
// GENERAL = false: no bias and no masked vocab rows (every tile full), the common case.
// The target logit is picked up in the same pass that feeds the sum, so the captured value is
// the very fp32 number that entered the softmax.
template <bool GENERAL, class AT, class Args>
__device__ inline void fwd_epilogue(const typename AT::vec (&acc)[AT::TM][AT::TN], const Args& a,
                                    const float* bias, int vw, int lane, const int (&tgt)[AT::TN],
                                    float (&m)[AT::TN], float (&s)[AT::TN], float (&zt)[AT::TN])
{
    constexpr int TM = AT::TM, TN = AT::TN, R = AT::kRegs;
    auto logit = [&](int i, int j, int r) -> float {
        float z = acc[i][j][r];
        if (GENERAL) {
            const int v = vw + AT::quad_row(i, r >> 2, lane) + (r & 3);
            if (bias != nullptr) z += bias[v < a.V ? v : a.V - 1];
            if (v >= a.V) z = -INFINITY;
        }
        return z;
    };
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < R; ++r) tmax = fmaxf(tmax, logit(i, j, r));
        __builtin_amdgcn_sched_barrier(0);
        tmax *= a.scale2;
        const float mnew = fmaxf(m[j], tmax);
        const float mref = mnew == -INFINITY ? 0.f : mnew;
        // register index (i * R + r) of the target row in this lane, or -1
        const int etgt = AT::reg_of_row(tgt[j] - vw, lane);
        // four partial sums (fixed association) keep the exp results off a single add chain; the
        // target capture runs only when some lane of the wavefront owns a target row in this slab
        float ps[4] = {0.f, 0.f, 0.f, 0.f};
        float zraw = 0.f;
        if (__builtin_amdgcn_ballot_w64(etgt >= 0) != 0) {  // uniform
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float z = logit(i, j, r);
                    ps[r & 3] += __builtin_amdgcn_exp2f(fmaf(z, a.scale2, -mref));
                    zraw = (etgt == i * R + r) ? z : zraw;
                }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < R; ++r)
                    ps[r & 3] += __builtin_amdgcn_exp2f(fmaf(logit(i, j, r), a.scale2, -mref));
        }
        const float sum = (ps[0] + ps[1]) + (ps[2] + ps[3]);
        __builtin_amdgcn_sched_barrier(0);
        s[j] = s[j] * __builtin_amdgcn_exp2f(m[j] - mref) + sum;
        m[j] = mnew;
        if (etgt >= 0) zt[j] = zraw * a.scale2;
    }
}

// acc += bias of a full tile: `vw` is the first vocab row of this wavefront's slab, relative to
// bias[0].  A lane holds quads of four consecutive vocab rows, so the bias arrives in 16-byte
// loads that are the same for every lane of a lane group (one broadcast request each).
template <class AT>
__device__ inline void add_bias(typename AT::vec (&acc)[AT::TM][AT::TN], const float* bias, int vw, int lane)
{
#pragma unroll
    for (int i = 0; i < AT::TM; ++i)
#pragma unroll
        for (int q = 0; q < AT::kQuads; ++q) {
            const float* p = bias + vw + AT::quad_row(i, q, lane);
            const float b0 = p[0], b1 = p[1], b2 = p[2], b3 = p[3];
#pragma unroll
            for (int j = 0; j < AT::TN; ++j) {
                acc[i][j][q * 4 + 0] += b0;
                acc[i][j][q * 4 + 1] += b1;
                acc[i][j][q * 4 + 2] += b2;
                acc[i][j][q * 4 + 3] += b3;
            }
        }
}

// Tiles of a launch are handed out round by round: workgroup b computes the tiles with linear ids
// b, b + gridDim.x, b + 2 gridDim.x, ...  With a grid that is a multiple of 8, a workgroup keeps
// its XCD from round to round, so every round forms the same L2-sharing patches as a launch with
// one workgroup per tile would.
constexpr int kWalkPatch = 8;  // tile rows of the patch the 32 workgroups of one XCD cover per round
struct TileWalk {
    int lin, total, gm, gn;
    __device__ inline TileWalk(int total_, int gm_, int gn_)
        : lin(blockIdx.x), total(total_), gm(gm_), gn(gn_) {}
    __device__ inline bool valid() const { return lin < total; }
    __device__ inline bool has_next() const { return lin + static_cast<int>(gridDim.x) < total; }
    __device__ inline void coords(bool next, int& tm, int& tn) const
    {
        xcd_tile(next ? lin + static_cast<int>(gridDim.x) : lin, total, gm, gn, kWalkPatch, tm, tn);
    }
    __device__ inline void advance() { lin += static_cast<int>(gridDim.x); }
};

template <class V, int TM, int TN>
__device__ inline void zero_acc(V (&acc)[TM][TN])
{
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < static_cast<int>(sizeof(V) / sizeof(float)); ++r) acc[i][j][r] = 0.f;
}

}  // namespace rlk
