// MFMA tile GEMM mainloop for gfx950 (CDNA4), shared by the four contraction kernels of the
// fused linear-logprob path (forward logits tile, dZ recompute, dH, dW).
//
// One workgroup = kWM x kWN wavefronts (2 x 4 by default).  The workgroup computes a
// 256 x 256 tile D = A * B^T-like contraction over K with v_mfma_f32_32x32x16
// (bf16 or f16 inputs, fp32 accumulate); each wavefront owns TM x TN MFMA tiles of 32x32.
//
// Operands are described by (base pointer at the tile origin, leading dimension, valid rows):
//   * "K-contiguous" operand: memory is [row][k] with k fastest (W and hidden in the forward).
//   * "K-major" operand:      memory is [k][row] with row fastest (W in dH, dZ and hidden in dW).
//     Its fragments are fetched from LDS with the gfx950 transposing read
//     ds_read_b64_tr_b16, so no transposed copy of any tensor is ever written to HBM.
//
// Pipeline: global -> registers -> LDS (double buffered, one barrier per K step) -> MFMA.
// Loads never leave the valid part of the tensor: row indices are clamped, and K chunks beyond
// the valid K range are replaced by zeros, so no out-of-bounds address is ever formed.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace rlk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;

#define RLK_LDS __attribute__((address_space(3)))

// 1: the forward runs all vocab tiles of a workgroup through one pipeline (the K loop of a tile
// fetches the head of the next); 0: every tile fills and drains its own pipeline.
#ifndef RLK_STREAM
#define RLK_STREAM 1
#endif
// Main-loop variant: 1 = global memory is copied straight into LDS (no staging registers),
// 0 = global -> registers -> LDS.  K steps that are not a whole BK always take the second.
#ifndef RLK_DTL
#define RLK_DTL 1
#endif
#ifndef RLK_LW
#define RLK_LW 2  // direct-to-LDS: slices over which the loads of one K step are spread
#endif
// The persistent dZ and dH kernels stall more on operand loads than the forward: for them all loads
// of a K step go out in the first slice of the window, a full K step ahead of their barrier (the
// forward loses up to 1.4 % with that window).
#ifndef RLK_LW_BWD
#define RLK_LW_BWD 1
#endif
#ifndef RLK_RD
#define RLK_RD 8  // direct-to-LDS: fragment reads issued per 8 MFMA slots (8 = one per slot)
#endif

// Workgroup shape: kWM x kWN wavefronts tile the 256 x 256 block; each wavefront owns
// kTM x kTN MFMA tiles of 32 x 32.
#ifndef RLK_WM
#define RLK_WM 2
#endif
#ifndef RLK_WN
#define RLK_WN 4
#endif
constexpr int kWM = RLK_WM;
constexpr int kWN = RLK_WN;
constexpr int kThreads = 64 * kWM * kWN;
constexpr int kTM = 256 / (32 * kWM);
constexpr int kTN = 256 / (32 * kWN);
static_assert(kTM * kWM * 32 == 256 && kTN * kWN * 32 == 256, "wave grid must tile 256 x 256");

struct Bf16 {
    static constexpr int kId = 0;
    using scalar = __bf16;
    __device__ static inline f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    __device__ static inline uint16_t from_float(float x)
    {
        return __builtin_bit_cast(uint16_t, static_cast<__bf16>(x));
    }
    __device__ static inline float to_float(uint16_t x)
    {
        return __builtin_bit_cast(float, static_cast<uint32_t>(x) << 16);
    }
    // two values rounded and packed by one conversion instruction (lo in bits 0..15)
    __device__ static inline uint32_t pack2(float lo, float hi)
    {
        typedef __attribute__((ext_vector_type(2))) float f32x2_t;
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
    }
};

struct F16 {
    static constexpr int kId = 1;
    using scalar = _Float16;
    __device__ static inline f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    __device__ static inline uint16_t from_float(float x)
    {
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x));
    }
    __device__ static inline float to_float(uint16_t x)
    {
        return static_cast<float>(__builtin_bit_cast(_Float16, x));
    }
    __device__ static inline uint32_t pack2(float lo, float hi)
    {
        typedef __attribute__((ext_vector_type(2))) float f32x2_t;
        typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, f16x2_t));
    }
};

// 16-bit matrix operand of one workgroup tile.
struct Operand {
    const uint16_t* base;  // element (row 0, k 0) of the tile
    int64_t ld;            // elements between consecutive memory lines
    int rows;              // valid tile rows from the origin (>= 1)
};

// LDS geometry of one operand tile.
template <bool KMAJOR, int ROWS, int BK>
struct TileGeom {
    // K-contiguous: one line per tile row, BK elements + 16 B pad (conflict-free b128 fragment reads).
    // K-major:      one line per k, ROWS elements + 64 B pad (conflict-free transposing reads).
    static constexpr int kPitch = KMAJOR ? (ROWS * 2 + 64) : (BK * 2 + 16);
    static constexpr int kLines = KMAJOR ? BK : ROWS;
    static constexpr int kBytes = kPitch * kLines;
    static constexpr int kChunksPerLine = KMAJOR ? (ROWS / 8) : (BK / 8);
    static constexpr int kLinesPerPass = kThreads / kChunksPerLine;
    static constexpr int kPasses = kLines / kLinesPerPass;
    static_assert(kLines % kLinesPerPass == 0, "tile does not divide over 256 threads");
};

template <bool KMAJOR, int ROWS, int BK>
struct TileIO {
    using G = TileGeom<KMAJOR, ROWS, BK>;

    // Per-thread addressing of one operand: a uniform base pointer plus 32-bit byte offsets of
    // this thread's chunks at K step 0 (already clamped into the valid part of the tensor).
    const char* base;
    uint32_t off[G::kPasses];
    uint32_t step;  // byte advance per K step

    __device__ inline void init(const Operand& op, int K)
    {
        const int t = threadIdx.x;
        const int chunk = t % G::kChunksPerLine;
        const int line0 = t / G::kChunksPerLine;
        base = reinterpret_cast<const char*>(op.base);
        const uint32_t ld = static_cast<uint32_t>(op.ld);
        step = KMAJOR ? static_cast<uint32_t>(BK) * ld * 2u : static_cast<uint32_t>(BK) * 2u;
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int line = p * G::kLinesPerPass + line0;
            if (KMAJOR) {
                const int k = line < K ? line : K - 1;
                const int r = chunk * 8 < op.rows ? chunk * 8 : 0;
                off[p] = (static_cast<uint32_t>(k) * ld + static_cast<uint32_t>(r)) * 2u;
            } else {
                const int r = line < op.rows ? line : op.rows - 1;
                const int k = chunk * 8 < K ? chunk * 8 : 0;
                off[p] = (static_cast<uint32_t>(r) * ld + static_cast<uint32_t>(k)) * 2u;
            }
        }
    }

    // Fetch this thread's 16-byte chunks of K step kt.  CHECKED: chunks at k >= K come back as
    // zeros (only needed for the last, partial K step).
    template <bool CHECKED>
    __device__ inline void load(int kt, int K, u32x4_t (&reg)[G::kPasses]) const
    {
        const int t = threadIdx.x;
        const int chunk = t % G::kChunksPerLine;
        const int line0 = t / G::kChunksPerLine;
        const size_t adv = static_cast<size_t>(kt) * step;  // 64-bit: K * ld can pass 4 GiB
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            if (CHECKED) {
                const int k = kt * BK + (KMAJOR ? p * G::kLinesPerPass + line0 : chunk * 8);
                const bool live = k < K;
                const size_t o = live ? off[p] + adv : off[p];
                u32x4_t v = *reinterpret_cast<const u32x4_t*>(base + o);
                if (!live) v = u32x4_t{0u, 0u, 0u, 0u};
                reg[p] = v;
            } else {
                reg[p] = *reinterpret_cast<const u32x4_t*>(base + (off[p] + adv));
            }
        }
    }

    // Single-pass forms used by the software-pipelined main loop.  CHECKED: a chunk at k >= K is
    // fetched from a clamped (valid) address and replaced by zeros when it is stored to LDS.
    __device__ inline bool live(int kt, int K, int p) const
    {
        const int t = threadIdx.x;
        const int k = kt * BK + (KMAJOR ? p * G::kLinesPerPass + t / G::kChunksPerLine
                                        : (t % G::kChunksPerLine) * 8);
        return k < K;
    }

    template <bool CHECKED>
    __device__ inline void load_one(int kt, int K, u32x4_t (&reg)[G::kPasses], int p) const
    {
        const size_t adv = static_cast<size_t>(kt) * step;  // 64-bit: K * ld can pass 4 GiB
        size_t o = off[p] + adv;
        if (CHECKED) o = live(kt, K, p) ? o : off[p];
        reg[p] = *reinterpret_cast<const u32x4_t*>(base + o);
    }

    template <bool CHECKED>
    __device__ inline void store_one(char* lds, const u32x4_t (&reg)[G::kPasses], int p, int kt,
                                     int K) const
    {
        const int t = threadIdx.x;
        const int chunk = t % G::kChunksPerLine;
        const int line = p * G::kLinesPerPass + t / G::kChunksPerLine;
        u32x4_t v = reg[p];
        if (CHECKED) v = live(kt, K, p) ? v : u32x4_t{0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4_t*>(lds + line * G::kPitch + chunk * 16) = v;
    }

    __device__ static inline void store(char* lds, const u32x4_t (&reg)[G::kPasses])
    {
        const int t = threadIdx.x;
        const int chunk = t % G::kChunksPerLine;
        const int line0 = t / G::kChunksPerLine;
#pragma unroll
        for (int p = 0; p < G::kPasses; ++p) {
            const int line = p * G::kLinesPerPass + line0;
            *reinterpret_cast<u32x4_t*>(lds + line * G::kPitch + chunk * 16) = reg[p];
        }
    }

    // MFMA 32x32x16 operand fragment: lane l holds row (row0 + l%32), k = kk*16 + 8*(l/32) + 0..7.
    __device__ static inline u32x4_t frag(const char* lds, int row0, int kk)
    {
        const int l = threadIdx.x & 63;
        if (KMAJOR) {
            // ds_read_b64_tr_b16: inside each group of 16 lanes, lane 4a+b supplies the address of
            // 4 consecutive rows (4b..4b+3) of k-line a; lane i receives row i of k-lines 0..3.
            const int a = (l & 15) >> 2;
            const int b = l & 3;
            const int kline = kk * 16 + 8 * (l >> 5) + a;
            const int col = row0 + 16 * ((l >> 4) & 1) + 4 * b;
            const char* p0 = lds + kline * G::kPitch + col * 2;
            const char* p1 = p0 + 4 * G::kPitch;
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p0));
            s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p1));
            u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
            u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
            return u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y};
        } else {
            const char* p = lds + (row0 + (l & 31)) * G::kPitch + (kk * 16 + 8 * (l >> 5)) * 2;
            return *reinterpret_cast<const u32x4_t*>(p);
        }
    }
};

// Compile-time loop: f(std::integral_constant<int, I>) for I in [B, E).
template <int B, int E, class F>
__device__ inline void static_for(F&& f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

template <class T, bool A_KMAJOR, bool B_KMAJOR, int BK, int LWIN = RLK_LW>
struct TileGemmDtl;

// Workgroup tile contraction.  acc[i][j] (+)= A rows x B rows over k in [0, K).
// smem must hold 2 * (A tile + B tile) bytes.  All 256 threads must call it (it barriers).
//
// The K loop is software pipelined by hand and the issue order is pinned with scheduling
// barriers: every MFMA is followed by at most a couple of memory instructions, so LDS
// fragment reads (for the next 16-wide k slice), LDS stores (next K step) and global loads
// (the K step after that) all travel under the shadow of the matrix pipe.
//   K step kt:  slices 0..KK-2: MFMAs | fragment reads for the next slice
//                               | every few MFMAs: one LDS store of K step kt+1, then the global
//                                 load of K step kt+2 into the registers that store just freed
//               barrier
//               last slice    : MFMAs | fragment reads for slice 0 of K step kt+1
template <class T, bool A_KMAJOR, bool B_KMAJOR, int BK>
struct TileGemm {
    static constexpr int TM = kTM;
    static constexpr int TN = kTN;
    static constexpr int BM = kWM * TM * 32;
    static constexpr int BN = kWN * TN * 32;
    static constexpr int KK = BK / 16;
    static_assert(KK >= 2 && KK % 2 == 0, "BK must be 32 or 64");
    using IOA = TileIO<A_KMAJOR, BM, BK>;
    using IOB = TileIO<B_KMAJOR, BN, BK>;
    static constexpr int PA = IOA::G::kPasses;
    static constexpr int PB = IOB::G::kPasses;
    static constexpr int kStageBytes = IOA::G::kBytes + IOB::G::kBytes;
    static constexpr int kSmemBytes = 2 * kStageBytes;

    // One 16-wide k slice of K step kt: TM*TN MFMAs from fragment set (KKI & 1), with this
    // slice's share of memory instructions spread between them.  The loop body is identical for
    // every K step (the K steps past the end re-fetch the last one into buffers nobody reads),
    // which keeps the accumulator in one fixed set of registers.
    template <int KKI, bool CHECKED>
    __device__ static inline void slice(const IOA& la, const IOB& lb, u32x4_t (&ra)[PA],
                                        u32x4_t (&rb)[PB], u32x4_t (&fa)[2][TM],
                                        u32x4_t (&fb)[2][TN], int wm, int wn, int kstore, int kload,
                                        int K,
                                        const char* cur, char* nxt, f32x16_t (&acc)[TM][TN])
    {
        constexpr bool last = KKI == KK - 1;
        constexpr int setc = KKI & 1, setn = setc ^ 1;
        constexpr int NR = TM + TN;
        constexpr int NM = TM * TN;
        constexpr int NW = PA + PB;                  // LDS stores == global loads per K step
        constexpr int SP = (NM * (KK - 1)) / NW;     // MFMA slots between consecutive stores
        static_assert(SP >= 2, "not enough MFMA slots before the barrier");
        const char* rsrc = last ? nxt : cur;
        constexpr int kkn = last ? 0 : KKI + 1;
        static_for<0, NM>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int i = q / TN, j = q % TN;
            constexpr int slot = KKI * NM + q;       // MFMA index inside the K step
            acc[i][j] = T::mfma(fa[setc][i], fb[setc][j], acc[i][j]);
            // fragment reads for the next slice, spread evenly over this slice and issued in the
            // order the next slice's MFMAs (i-major) first need them: A0, B0..B(TN-1), A1..A(TM-1)
            static_for<q * NR / NM, (q + 1) * NR / NM>([&](auto oc) {
                constexpr int o = decltype(oc)::value;
                if constexpr (o == 0 || o > TN) {
                    constexpr int fi = o == 0 ? 0 : o - TN;
                    fa[setn][fi] = IOA::frag(rsrc, wm * (TM * 32) + fi * 32, kkn);
                } else {
                    constexpr int fj = o - 1;
                    fb[setn][fj] =
                        IOB::frag(rsrc + IOA::G::kBytes, wn * (TN * 32) + fj * 32, kkn);
                }
            });
            // pass w: LDS store at slot w*SP, the global load that refills the same registers
            // right after it, so loads are spaced evenly and get a full K step of latency
            if constexpr (slot % SP == 0 && slot / SP < NW) {
                constexpr int w = slot / SP;
                if constexpr (w < PA)
                    la.template store_one<CHECKED>(nxt, ra, w, kstore, K);
                else
                    lb.template store_one<CHECKED>(nxt + IOA::G::kBytes, rb, w - PA, kstore, K);
            }
            if constexpr (slot % SP == 1 && slot / SP < NW) {
                constexpr int g = slot / SP;
                if constexpr (g < PA)
                    la.template load_one<CHECKED>(kload, K, ra, g);
                else
                    lb.template load_one<CHECKED>(kload, K, rb, g - PA);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    template <bool CHECKED>
    __device__ static inline void run_impl(const Operand& A, const Operand& B, int K,
                                           f32x16_t (&acc)[TM][TN], char* smem)
    {
        IOA la;
        IOB lb;
        u32x4_t ra[PA];
        u32x4_t rb[PB];
        u32x4_t fa[2][TM];
        u32x4_t fb[2][TN];
        const int wave = threadIdx.x >> 6;
        const int wm = wave / kWN;
        const int wn = wave % kWN;
        la.init(A, K);
        lb.init(B, K);
        const int nk = (K + BK - 1) / BK;

        la.template load<CHECKED>(0, K, ra);
        lb.template load<CHECKED>(0, K, rb);
        IOA::store(smem, ra);
        IOB::store(smem + IOA::G::kBytes, rb);
        {
            const int k1 = nk > 1 ? 1 : 0;
            la.template load<CHECKED>(k1, K, ra);
            lb.template load<CHECKED>(k1, K, rb);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[0][i] = IOA::frag(smem, wm * (TM * 32) + i * 32, 0);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[0][j] = IOB::frag(smem + IOA::G::kBytes, wn * (TN * 32) + j * 32, 0);

        for (int kt = 0; kt < nk; ++kt) {
            const char* cur = smem + (kt & 1) * kStageBytes;
            char* nxt = smem + ((kt + 1) & 1) * kStageBytes;
            const int kstore = kt + 1 < nk ? kt + 1 : nk - 1;  // K step held in ra/rb
            const int kload = kt + 2 < nk ? kt + 2 : nk - 1;
            static_for<0, KK - 1>([&](auto kc) {
                slice<decltype(kc)::value, CHECKED>(la, lb, ra, rb, fa, fb, wm, wn, kstore, kload, K,
                                                    cur, nxt, acc);
            });
            __syncthreads();
            slice<KK - 1, CHECKED>(la, lb, ra, rb, fa, fb, wm, wn, kstore, kload, K, cur, nxt, acc);
        }
        __syncthreads();  // LDS may be reused by the caller
    }

    __device__ static inline void run(const Operand& A, const Operand& B, int K,
                                      f32x16_t (&acc)[TM][TN], char* smem)
    {
        if (K % BK == 0) {
#if RLK_DTL
            TileGemmDtl<T, A_KMAJOR, B_KMAJOR, BK>::run(A, B, K, acc, smem);
#else
            run_impl<false>(A, B, K, acc, smem);
#endif
        } else {
            run_impl<true>(A, B, K, acc, smem);
        }
    }
};

// ------------------------------------------------------------------------------------------- //
// Direct-to-LDS variant of the main loop (used when K is a multiple of BK).
//
// Global memory is copied straight into LDS by `global_load_lds_dwordx4` (each lane's 16 bytes land
// at M0 + lane * 16, so one wavefront instruction fills 1 KiB of consecutive LDS): no staging
// registers, no LDS store instructions.  Because the destination is dense, bank conflicts are
// avoided by an XOR swizzle applied on the GLOBAL side (which 16-byte chunk a lane fetches):
//   K-contiguous tile, row r (128 B), chunk c      -> LDS  r*128 + ((c ^ ((r >> 1) & 7)) * 16)
//   K-major tile,      k-line k (512 B), chunk c   -> LDS  k*512 + ((c ^ ((k & 3) << 2)) * 16)
// which makes both the b128 fragment reads and the transposing b64 reads conflict-free.
// Two LDS stages of BK = 64; the loads of K step kt+1 are issued during the last slice of step
// kt-1 (right after the barrier that frees their buffer) and the first slices of step kt.
// ------------------------------------------------------------------------------------------- //
// s_waitcnt immediate that waits only for vmcnt <= n (expcnt and lgkmcnt left at "no wait").
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

template <bool KMAJOR, int ROWS, int BK>
struct DtlIO {
    static_assert(BK == 64 && ROWS == 256, "direct-to-LDS layout is written for 256 x 64 tiles");
    static constexpr int kBytes = ROWS * BK * 2;            // 32 KiB, dense
    static constexpr int kInstr = kBytes / 1024;            // wavefront loads per tile (32)
    static constexpr int kWaves = kThreads / 64;
    static constexpr int kPasses = kInstr / kWaves;         // loads per wavefront per K step
    static_assert(kInstr % kWaves == 0, "loads must divide over the wavefronts");

    const char* base;        // uniform: origin of the current tile
    const char* next;        // uniform: origin of the tile whose first K steps follow this one's
    uint32_t off[kPasses];   // per-lane byte offset of this lane's chunk for load p at K step 0
    uint32_t step;           // uniform byte advance per K step
    int nk;                  // K steps per tile
    int wave;                // uniform wavefront index

    __device__ inline void init(const Operand& op, int K)
    {
        const int lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        base = reinterpret_cast<const char*>(op.base);
        next = base;
        nk = K / BK;
        const uint32_t ld = static_cast<uint32_t>(op.ld);
        step = KMAJOR ? static_cast<uint32_t>(BK) * ld * 2u : static_cast<uint32_t>(BK) * 2u;
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int q = wave + kWaves * p;  // which 1 KiB block of the tile
            if (KMAJOR) {
                const int k = 2 * q + (lane >> 5);
                const int c = (lane & 31) ^ ((k & 3) << 2);
                const int kc = k < K ? k : K - 1;
                const int r = c * 8 < op.rows ? c * 8 : 0;
                off[p] = (static_cast<uint32_t>(kc) * ld + static_cast<uint32_t>(r)) * 2u;
            } else {
                const int r = 8 * q + (lane >> 3);
                const int c = (lane & 7) ^ ((r >> 1) & 7);
                const int rc = r < op.rows ? r : op.rows - 1;
                off[p] = (static_cast<uint32_t>(rc) * ld + static_cast<uint32_t>(c * 8)) * 2u;
            }
        }
    }

    // Issue load p of K step kt into the tile at `lds` (uniform pointer).  Written as inline
    // assembly (M0 = LDS destination, then the load with a scalar base and a 32-bit lane offset):
    // the compiler then neither tracks the LDS write nor guards later LDS reads with vmcnt(0);
    // the main loop waits explicitly (s_waitcnt vmcnt) before the barrier that publishes a stage.
    __device__ inline void load_one(int kt, char* lds, int p) const
    {
        // K steps past the end of this tile are the first steps of the next one (all uniform)
        const bool over = kt >= nk;
        const int rel = over ? (kt - nk < nk ? kt - nk : nk - 1) : kt;
        const char* src = (over ? next : base) + static_cast<size_t>(rel) * step;
        const uint32_t dst = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                                 (RLK_LDS char*)(lds))) + static_cast<uint32_t>((wave + kWaves * p) * 1024);
        asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(off[p]), "s"(src), "s"(dst)
                     : "memory", "m0");
    }

    // MFMA 32x32x16 operand fragment: lane l holds row (row0 + l%32), k = kk*16 + 8*(l/32) + 0..7.
    __device__ static inline u32x4_t frag(const char* lds, int row0, int kk)
    {
        const int l = threadIdx.x & 63;
        if (KMAJOR) {
            const int a = (l & 15) >> 2;
            const int b = l & 3;
            const int kline = kk * 16 + 8 * (l >> 5) + a;           // kline & 3 == a
            const int c = (row0 >> 3) + 2 * ((l >> 4) & 1) + (b >> 1);
            const char* p0 = lds + kline * 512 + ((c ^ (a << 2)) * 16) + (b & 1) * 8;
            const char* p1 = p0 + 4 * 512;                           // k-line + 4: same swizzle
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p0));
            s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p1));
            u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
            u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
            return u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y};
        } else {
            const int r = row0 + (l & 31);
            const int c = (2 * kk + (l >> 5)) ^ (((l & 31) >> 1) & 7);  // row0 is a multiple of 32
            return *reinterpret_cast<const u32x4_t*>(lds + r * 128 + c * 16);
        }
    }
};

template <class T, bool A_KMAJOR, bool B_KMAJOR, int BK, int LWIN>
struct TileGemmDtl {
    static constexpr int TM = kTM;
    static constexpr int TN = kTN;
    static constexpr int KK = BK / 16;
    using IOA = DtlIO<A_KMAJOR, 256, BK>;
    using IOB = DtlIO<B_KMAJOR, 256, BK>;
    static constexpr int PA = IOA::kPasses;
    static constexpr int PB = IOB::kPasses;
    static constexpr int NL = PA + PB;                 // loads per wavefront per K step
    static constexpr int NM = TM * TN;                 // MFMAs per slice
    static constexpr int LW = LWIN;                    // load window in slices
    static_assert(LW >= 1 && LW <= KK - 1, "load window must end before the barrier slice");
    static constexpr int kStageBytes = IOA::kBytes + IOB::kBytes;
    static constexpr int kSmemBytes = 2 * kStageBytes;

    // Load j of a K step is issued after MFMA slot j * (LW*NM) / NL of the window that starts at
    // the last slice of the previous step.
    // SKIP: the non-last slices issue no loads (the K step they would fetch is already on its way).
    template <int KKI, bool SKIP = false>
    __device__ static inline void slice(const IOA& la, const IOB& lb, u32x4_t (&fa)[2][TM],
                                        u32x4_t (&fb)[2][TN], int wm, int wn, int kt,
                                        char* cur, char* nxt, f32x16_t (&acc)[TM][TN])
    {
        constexpr bool last = KKI == KK - 1;
        constexpr int setc = KKI & 1, setn = setc ^ 1;
        constexpr int NR = TM + TN;
        const char* rsrc = last ? nxt : cur;
        constexpr int kkn = last ? 0 : KKI + 1;
        // window slice index of this slice: the last slice opens the window of step kt+2
        constexpr int wslice = last ? 0 : KKI + 1;
        static_for<0, NM>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int i = q / TN, j = q % TN;
            acc[i][j] = T::mfma(fa[setc][i], fb[setc][j], acc[i][j]);
            // fragment reads for the next slice: one per MFMA slot from the start of the slice, so
            // that all of them have returned when the next slice begins
            static_for<q * RLK_RD / 8, (q + 1) * RLK_RD / 8>([&](auto oc) {
                constexpr int o = decltype(oc)::value;
                if constexpr (o >= NR) {
                } else if constexpr (o == 0 || o > TN) {
                    constexpr int fi = o == 0 ? 0 : o - TN;
                    fa[setn][fi] = IOA::frag(rsrc, wm * (TM * 32) + fi * 32, kkn);
                } else {
                    constexpr int fj = o - 1;
                    fb[setn][fj] = IOB::frag(rsrc + IOA::kBytes, wn * (TN * 32) + fj * 32, kkn);
                }
            });
            if constexpr (wslice < LW && !(SKIP && !last)) {
                constexpr int wslot = wslice * NM + q;
                constexpr int lo = (wslot * NL + LW * NM - 1) / (LW * NM);        // ceil
                constexpr int hi = ((wslot + 1) * NL + LW * NM - 1) / (LW * NM);  // ceil
                static_for<lo, hi>([&](auto lc) {
                    constexpr int g = decltype(lc)::value;
                    // last slice: first loads of step kt+2 into the buffer this step just freed;
                    // other slices: remaining loads of step kt+1 into the other buffer
                    const int ks = last ? kt + 2 : kt + 1;  // past the end = next tile (load_one)
                    char* dst = last ? cur : nxt;
                    if constexpr (g < PA)
                        la.load_one(ks, dst, g);
                    else
                        lb.load_one(ks, dst + IOA::kBytes, g - PA);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // Pipeline state that lives across the tiles one workgroup computes back to back: the K loop
    // of a tile fetches the first K steps of the next tile where it would otherwise run dry, so
    // only the first tile of a workgroup pays the fill latency.
    struct Stream {
        IOA la;
        IOB lb;
        u32x4_t fa[2][TM];
        u32x4_t fb[2][TN];
        int wm, wn, nk, phase;
        bool ahead;  // every load of the current tile's K step 1 was issued by fetch_ahead()
    };

    // Fill the pipeline for the first tile: K step 0 in LDS and published, the fragments of its
    // first slice in registers, the head of K step 1 in flight.
    __device__ static inline void begin(Stream& st, const Operand& A, const Operand& B, int K,
                                        char* smem)
    {
        const int wave = threadIdx.x >> 6;
        st.wm = wave / kWN;
        st.wn = wave % kWN;
        st.la.init(A, K);
        st.lb.init(B, K);
        st.nk = K / BK;
        st.phase = 0;
        st.ahead = false;
        static_for<0, PA>([&](auto pc) { st.la.load_one(0, smem, decltype(pc)::value); });
        static_for<0, PB>(
            [&](auto pc) { st.lb.load_one(0, smem + IOA::kBytes, decltype(pc)::value); });
        constexpr int first = (NM * NL + LW * NM - 1) / (LW * NM);  // loads of window slice 0
        static_for<0, first>([&](auto lc) {
            constexpr int g = decltype(lc)::value;
            if constexpr (g < PA)
                st.la.load_one(1, smem + kStageBytes, g);
            else
                st.lb.load_one(1, smem + kStageBytes + IOA::kBytes, g - PA);
        });
        constexpr int wait_first = vmcnt_imm(first);
        __builtin_amdgcn_s_waitcnt(wait_first);  // K step 0 has landed
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TM; ++i) st.fa[0][i] = IOA::frag(smem, st.wm * (TM * 32) + i * 32, 0);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            st.fb[0][j] = IOB::frag(smem + IOA::kBytes, st.wn * (TN * 32) + j * 32, 0);
    }

    // All K steps of the current tile into `acc` (callers that chain tiles need K >= 2 * BK: the
    // loop looks two K steps ahead and knows one following tile).  `next_a` / `next_b` are the operand origins of
    // the tile that follows (same leading dimensions and row counts; pass the current origins
    // after the last tile: the extra fetches then stay inside the same tile).  On return the
    // stream stands at the start of that tile exactly as begin() leaves it.
    // REFETCH: the fragments of the first slice are read again from LDS here instead of being
    // carried in registers from the previous tile's last slice; callers with a register-hungry
    // epilogue between tiles use it (the K step they come from is already published).
    // YOUNGER: after fetch_ahead() the caller's epilogue issued at least this many vector-memory
    // instructions per wavefront (stores that may still be in flight).  The counter retires in
    // issue order, so the first K step only has to wait until at most YOUNGER operations are
    // outstanding to know that its own loads, which are older, have landed; the stores drain
    // under the MFMAs instead of in front of the barrier.  A value below the true count is safe.
    // `counted` (uniform) says whether that promise holds for the epilogue that just ran.
    template <bool REFETCH = false, int YOUNGER = 0>
    __device__ static inline void tile(Stream& st, const void* next_a, const void* next_b,
                                       f32x16_t (&acc)[TM][TN], char* smem, bool counted = false)
    {
        st.la.next = reinterpret_cast<const char*>(next_a);
        st.lb.next = reinterpret_cast<const char*>(next_b);
        const int nk = st.nk;
        if constexpr (REFETCH) {
            const char* cur0 = smem + (st.phase & 1) * kStageBytes;
#pragma unroll
            for (int i = 0; i < TM; ++i) st.fa[0][i] = IOA::frag(cur0, st.wm * (TM * 32) + i * 32, 0);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                st.fb[0][j] = IOB::frag(cur0 + IOA::kBytes, st.wn * (TN * 32) + j * 32, 0);
        }
        int kt = 0;
        if (st.ahead) {  // uniform: K step 1 is already on its way, issue nothing for it
            char* cur = smem + (st.phase & 1) * kStageBytes;
            char* nxt = smem + ((st.phase + 1) & 1) * kStageBytes;
            static_for<0, KK - 1>([&](auto kc) {
                slice<decltype(kc)::value, true>(st.la, st.lb, st.fa, st.fb, st.wm, st.wn, 0, cur,
                                                 nxt, acc);
            });
            constexpr int wait_older = vmcnt_imm(YOUNGER < 63 ? YOUNGER : 63);
            constexpr int wait_every = vmcnt_imm(0);
            if (YOUNGER > 0 && counted)
                __builtin_amdgcn_s_waitcnt(wait_older);
            else
                __builtin_amdgcn_s_waitcnt(wait_every);
            __syncthreads();
            slice<KK - 1>(st.la, st.lb, st.fa, st.fb, st.wm, st.wn, 0, cur, nxt, acc);
            st.ahead = false;
            kt = 1;
        }
        for (; kt < nk; ++kt) {
            char* cur = smem + ((kt + st.phase) & 1) * kStageBytes;
            char* nxt = smem + ((kt + st.phase + 1) & 1) * kStageBytes;
            static_for<0, KK - 1>([&](auto kc) {
                slice<decltype(kc)::value>(st.la, st.lb, st.fa, st.fb, st.wm, st.wn, kt, cur, nxt,
                                           acc);
            });
            constexpr int wait_all = vmcnt_imm(0);
            __builtin_amdgcn_s_waitcnt(wait_all);  // my loads of K step kt+1 have landed
            __syncthreads();
            slice<KK - 1>(st.la, st.lb, st.fa, st.fb, st.wm, st.wn, kt, cur, nxt, acc);
        }
        st.phase = (st.phase + nk) & 1;
        st.la.base = st.la.next;
        st.lb.base = st.lb.next;
    }

    // Call right after tile() when an epilogue with stores follows and another tile comes after
    // it: issues now the loads of that tile's K step 1 which its first K step would otherwise
    // issue behind the epilogue's stores (the head of the step is already in flight, the LDS stage
    // is free since the last barrier).  The next tile() then waits with a counted vmcnt.
    __device__ static inline void fetch_ahead(Stream& st, char* smem)
    {
        constexpr int first = (NM * NL + LW * NM - 1) / (LW * NM);  // loads of window slice 0
        char* dst = smem + ((st.phase + 1) & 1) * kStageBytes;
        static_for<first, NL>([&](auto lc) {
            constexpr int g = decltype(lc)::value;
            if constexpr (g < PA)
                st.la.load_one(1, dst, g);
            else
                st.lb.load_one(1, dst + IOA::kBytes, g - PA);
        });
        st.ahead = true;
    }

    // Drain the fetches issued for a tile that will not be computed; LDS is free afterwards.
    __device__ static inline void end(Stream&)
    {
        constexpr int wait_drain = vmcnt_imm(0);
        __builtin_amdgcn_s_waitcnt(wait_drain);
        __syncthreads();
    }

    __device__ static inline void run(const Operand& A, const Operand& B, int K,
                                      f32x16_t (&acc)[TM][TN], char* smem)
    {
        Stream st;
        begin(st, A, B, K, smem);
        tile(st, A.base, B.base, acc, smem);
        end(st);
    }
};

// Row of the 32x32 accumulator held in register r of lane l: D[8*(r/4) + 4*(l/32) + r%4][l%32].
__device__ inline int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// Map a linear workgroup id to a tile so that the 32 workgroups resident on one XCD (ids equal
// modulo 8 run on the same XCD and share its L2) cover a compact patch of `group` tile rows.
__device__ inline void xcd_tile(int lin, int total, int gm, int gn, int group, int& tm, int& tn)
{
    const int per = total >> 3;
    const int rem = total & 7;
    const int xcd = lin & 7;
    const int idx = lin >> 3;
    const int seq = xcd * per + (xcd < rem ? xcd : rem) + idx;
    const int gsz = group * gn;
    const int gid = seq / gsz;
    const int first = gid * group;
    const int rows = (gm - first) < group ? (gm - first) : group;
    const int in = seq - gid * gsz;
    tm = first + in % rows;
    tn = in / rows;
}

}  // namespace rlk
