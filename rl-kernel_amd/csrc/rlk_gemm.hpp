// MFMA tile GEMM mainloop for gfx950 (CDNA4), shared by the four contraction kernels of the
// fused linear-logprob path (forward logits tile, dZ recompute, dH, dW).
//
// One workgroup = 2 x 4 wavefronts.  The workgroup computes a 256 x 256 tile D = A * B^T-like
// contraction over K with v_mfma_f32_16x16x32 (bf16 or f16 inputs, fp32 accumulate); each
// wavefront owns a 128 x 64 slab = 8 x 4 MFMA tiles of 16 x 16.  The 16 x 16 x 32 instruction does
// the same multiply-adds per cycle as the 32 x 32 x 16 one but sums 8 products before each fp32
// accumulate instead of 2; under the board's power limit the chip clocks about 10 % higher with it
// (measured with the same tile loop, same LDS traffic, both shapes).
//
// Operands are described by (base pointer at the tile origin, leading dimension, valid rows):
//   * "K-contiguous" operand: memory is [row][k] with k fastest (W and hidden in the forward).
//   * "K-major" operand:      memory is [k][row] with row fastest (W in dH, dZ and hidden in dW).
//     Its fragments are fetched from LDS with the gfx950 transposing read
//     ds_read_b64_tr_b16, so no transposed copy of any tensor is ever written to HBM.
//
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

// Workgroup shape: kWM x kWN wavefronts tile the 256 x 256 block.
constexpr int kWM = 2;
constexpr int kWN = 4;
constexpr int kThreads = 64 * kWM * kWN;

// Accumulator geometry of a wavefront slab built from MI x MI MFMA tiles (MI = 16: the 16-bit
// kernels; MI = 32: the fp32 matrix-core kernels).  In both, the M index lives in accumulator
// registers and the N index is the lane: lane l of tile (i, j) holds column j * MI + l % MI and,
// in register quad q, the four consecutive rows from quad_row(i, q, l) on.
template <int MI>
struct AccTile {
    static constexpr int kMI = MI;
    static constexpr int kRegs = MI * MI / 64;   // accumulator registers per tile: 4 or 16
    static constexpr int kQuads = kRegs / 4;     // quads of four consecutive rows per lane: 1 or 4
    static constexpr int kGroups = 64 / MI;      // lane groups that hold different rows: 4 or 2
    static constexpr int TM = 256 / (MI * kWM);  // tiles per wavefront along M: 8 or 4
    static constexpr int TN = 256 / (MI * kWN);  // tiles per wavefront along N: 4 or 2
    typedef __attribute__((ext_vector_type(kRegs))) float vec;
    __device__ static inline int quad_row(int i, int q, int lane)
    {
        return i * MI + 4 * kGroups * q + 4 * (lane / MI);
    }
    __device__ static inline int col(int j, int lane) { return j * MI + lane % MI; }
    // Register index (i * kRegs + r) that holds slab row `row` in lane `lane`, or -1 when the
    // row is outside [0, TM * MI) or lives in another lane group.
    __device__ static inline int reg_of_row(int row, int lane)
    {
        if (static_cast<unsigned>(row) >= static_cast<unsigned>(TM * MI)) return -1;
        const int x = row % MI;
        if ((x >> 2) % kGroups != lane / MI) return -1;
        return (row / MI) * kRegs + (x / (4 * kGroups)) * 4 + (x & 3);
    }
};

using Acc16 = AccTile<16>;  // 16-bit kernels
using Acc32 = AccTile<32>;  // fp32 matrix-core kernels
constexpr int kTM = Acc32::TM;  // slab of the fp32 kernels in 32 x 32 tiles
constexpr int kTN = Acc32::TN;

struct Bf16 {
    static constexpr int kId = 0;
    using scalar = __bf16;
    __device__ static inline f32x4_t mfma(u32x4_t a, u32x4_t b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
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
    __device__ static inline f32x4_t mfma(u32x4_t a, u32x4_t b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
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

// Compile-time loop: f(std::integral_constant<int, I>) for I in [B, E).
template <int B, int E, class F>
__device__ inline void static_for(F&& f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Issue plan of the fragment reads of one 32-wide k slice (TM * TN = 32 MFMA slots, row-major over
// the slab: slot = i * TN + j).  While a slice multiplies, the fragments of the next slice are
// fetched: the TN fragments of B first (each stays live through the whole next slice), then
// fragment i of A as soon as row i of the current slice has been issued, so that the old and
// the new A fragment of a row overlap for a few slots only.  That keeps about TM + 1 + 2 TN
// fragments live instead of two full sets.
// One slot carries at most one read instruction group (a K-major fragment is two transposing reads).
template <int TM, int TN>
struct FragPlan {
    // fragment o of the next slice: o < TN is B fragment o, otherwise A fragment o - TN
    static constexpr int kReads = TM + TN;
    // slot after whose MFMA read o is issued
    static constexpr int slot_of(int o)
    {
        if (o < TN) return o;                              // B'0 .. B'(TN-1) in slots 0 .. TN-1
        const int i = o - TN;
        const int s = (i + 1) * TN;                        // first slot after row i
        return s < TM * TN ? s : TM * TN - 1;              // the last row's fragment goes last
    }
};

// LDS geometry of one operand tile of the register-staged loop.
template <bool KMAJOR, int ROWS, int BK>
struct TileGeom {
    // K-contiguous: one line per tile row, BK elements + 16 B pad (conflict-free b128 fragment reads).
    // K-major:      one line per k, ROWS elements + 64 B pad.
    static constexpr int kPitch = KMAJOR ? (ROWS * 2 + 64) : (BK * 2 + 16);
    static constexpr int kLines = KMAJOR ? BK : ROWS;
    static constexpr int kBytes = kPitch * kLines;
    static constexpr int kChunksPerLine = KMAJOR ? (ROWS / 8) : (BK / 8);
    static constexpr int kLinesPerPass = kThreads / kChunksPerLine;
    static constexpr int kPasses = kLines / kLinesPerPass;
    static_assert(kLines % kLinesPerPass == 0, "tile does not divide over the workgroup's threads");
};

// Register-staged operand path (global -> VGPR -> padded LDS rows) of K steps that are not whole:
// every 16-byte chunk at k >= K is replaced by zeros when it is stored to LDS.
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

    // Whether this thread's chunk p of K step kt lies inside [0, K).
    __device__ inline bool live(int kt, int K, int p) const
    {
        const int t = threadIdx.x;
        const int k = kt * BK + (KMAJOR ? p * G::kLinesPerPass + t / G::kChunksPerLine
                                        : (t % G::kChunksPerLine) * 8);
        return k < K;
    }

    // A chunk at k >= K is fetched from a clamped (valid) address.
    __device__ inline void load_one(int kt, int K, u32x4_t (&reg)[G::kPasses], int p) const
    {
        const size_t adv = static_cast<size_t>(kt) * step;  // 64-bit: K * ld can pass 4 GiB
        const size_t o = live(kt, K, p) ? off[p] + adv : off[p];
        reg[p] = *reinterpret_cast<const u32x4_t*>(base + o);
    }

    __device__ inline void store_one(char* lds, const u32x4_t (&reg)[G::kPasses], int p, int kt,
                                     int K) const
    {
        const int t = threadIdx.x;
        const int chunk = t % G::kChunksPerLine;
        const int line = p * G::kLinesPerPass + t / G::kChunksPerLine;
        const u32x4_t v = live(kt, K, p) ? reg[p] : u32x4_t{0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4_t*>(lds + line * G::kPitch + chunk * 16) = v;
    }

    // MFMA 16x16x32 operand fragment: lane l holds row (row0 + l%16), k = kk*32 + 8*(l/16) + 0..7.
    __device__ static inline u32x4_t frag(const char* lds, int row0, int kk)
    {
        const int l = threadIdx.x & 63;
        if (KMAJOR) {
            // ds_read_b64_tr_b16: inside each group of 16 lanes, lane 4a+b supplies the address of
            // 4 consecutive rows (4b..4b+3) of k-line a; lane i receives row i of k-lines 0..3.
            const int a = (l & 15) >> 2;
            const int b = l & 3;
            const int kline = kk * 32 + 8 * (l >> 4) + a;
            const char* p0 = lds + kline * G::kPitch + (row0 + 4 * b) * 2;
            const char* p1 = p0 + 4 * G::kPitch;
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p0));
            s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p1));
            u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
            u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
            return u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y};
        } else {
            const char* p = lds + (row0 + (l & 15)) * G::kPitch + (kk * 32 + 8 * (l >> 4)) * 2;
            return *reinterpret_cast<const u32x4_t*>(p);
        }
    }
};

template <class T, bool A_KMAJOR, bool B_KMAJOR, int BK, int WIN>
struct TileGemmDtl;

// Workgroup tile contraction for any K.  acc[i][j] (+)= A rows x B rows over k in [0, K).
// smem must hold kSmemBytes.  All threads of the workgroup must call run() (it barriers).
//
// K a multiple of BK: the direct-to-LDS loop below (TileGemmDtl).  Otherwise the register-staged
// loop of this class, software pipelined by hand with the issue order pinned by scheduling barriers:
//   K step kt:  first slice : MFMAs | fragment reads for the second slice
//                             | every fourth MFMA: one LDS store of K step kt+1, then the global
//                               load of K step kt+2 into the registers that store just freed
//               barrier
//               second slice: MFMAs | fragment reads for the first slice of K step kt+1
template <class T, bool A_KMAJOR, bool B_KMAJOR, int BK>
struct TileGemm {
    using AT = Acc16;
    static constexpr int TM = AT::TM;
    static constexpr int TN = AT::TN;
    static constexpr int KK = BK / 32;
    static_assert(KK == 2, "the loop is written for two 32-wide slices per K step");
    using IOA = TileIO<A_KMAJOR, 256, BK>;
    using IOB = TileIO<B_KMAJOR, 256, BK>;
    using Plan = FragPlan<TM, TN>;
    static constexpr int PA = IOA::G::kPasses;
    static constexpr int PB = IOB::G::kPasses;
    static constexpr int NM = TM * TN;
    static constexpr int kStageBytes = IOA::G::kBytes + IOB::G::kBytes;
    static constexpr int kSmemBytes = 2 * kStageBytes;

    template <int KKI>
    __device__ static inline void slice(const IOA& la, const IOB& lb, u32x4_t (&ra)[PA],
                                        u32x4_t (&rb)[PB], u32x4_t (&fa)[2][TM],
                                        u32x4_t (&fb)[2][TN], int wm, int wn, int kstore, int kload,
                                        int K, const char* cur, char* nxt, f32x4_t (&acc)[TM][TN])
    {
        constexpr bool last = KKI == KK - 1;
        constexpr int setc = KKI & 1, setn = setc ^ 1;
        constexpr int NW = PA + PB;   // LDS stores == global loads per K step
        constexpr int SP = NM / NW;   // MFMA slots between consecutive stores
        static_assert(SP >= 2, "not enough MFMA slots before the barrier");
        const char* rsrc = last ? nxt : cur;
        constexpr int kkn = last ? 0 : KKI + 1;
        static_for<0, NM>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int i = q / TN, j = q % TN;
            acc[i][j] = T::mfma(fa[setc][i], fb[setc][j], acc[i][j]);
            static_for<0, Plan::kReads>([&](auto oc) {
                constexpr int o = decltype(oc)::value;
                if constexpr (Plan::slot_of(o) == q) {
                    if constexpr (o < TN)
                        fb[setn][o] = IOB::frag(rsrc + IOA::G::kBytes, wn * (TN * 16) + o * 16, kkn);
                    else
                        fa[setn][o - TN] = IOA::frag(rsrc, wm * (TM * 16) + (o - TN) * 16, kkn);
                }
            });
            if constexpr (!last) {
                // pass w: LDS store at slot w*SP, the global load that refills the same registers
                // right after it, so loads are spaced evenly and get a full K step of latency
                if constexpr (q % SP == 0 && q / SP < NW) {
                    constexpr int w = q / SP;
                    if constexpr (w < PA)
                        la.store_one(nxt, ra, w, kstore, K);
                    else
                        lb.store_one(nxt + IOA::G::kBytes, rb, w - PA, kstore, K);
                }
                if constexpr (q % SP == 1 && q / SP < NW) {
                    constexpr int g = q / SP;
                    if constexpr (g < PA)
                        la.load_one(kload, K, ra, g);
                    else
                        lb.load_one(kload, K, rb, g - PA);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    __device__ static inline void run_staged(const Operand& A, const Operand& B, int K,
                                             f32x4_t (&acc)[TM][TN], char* smem)
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

        static_for<0, PA>([&](auto pc) { la.load_one(0, K, ra, decltype(pc)::value); });
        static_for<0, PB>([&](auto pc) { lb.load_one(0, K, rb, decltype(pc)::value); });
        static_for<0, PA>([&](auto pc) { la.store_one(smem, ra, decltype(pc)::value, 0, K); });
        static_for<0, PB>(
            [&](auto pc) { lb.store_one(smem + IOA::G::kBytes, rb, decltype(pc)::value, 0, K); });
        {
            const int k1 = nk > 1 ? 1 : 0;
            static_for<0, PA>([&](auto pc) { la.load_one(k1, K, ra, decltype(pc)::value); });
            static_for<0, PB>([&](auto pc) { lb.load_one(k1, K, rb, decltype(pc)::value); });
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[0][i] = IOA::frag(smem, wm * (TM * 16) + i * 16, 0);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[0][j] = IOB::frag(smem + IOA::G::kBytes, wn * (TN * 16) + j * 16, 0);

        for (int kt = 0; kt < nk; ++kt) {
            const char* cur = smem + (kt & 1) * kStageBytes;
            char* nxt = smem + ((kt + 1) & 1) * kStageBytes;
            const int kstore = kt + 1 < nk ? kt + 1 : nk - 1;  // K step held in ra/rb
            const int kload = kt + 2 < nk ? kt + 2 : nk - 1;
            slice<0>(la, lb, ra, rb, fa, fb, wm, wn, kstore, kload, K, cur, nxt, acc);
            __syncthreads();
            slice<1>(la, lb, ra, rb, fa, fb, wm, wn, kstore, kload, K, cur, nxt, acc);
        }
        __syncthreads();  // LDS may be reused by the caller
    }

    __device__ static inline void run(const Operand& A, const Operand& B, int K,
                                      f32x4_t (&acc)[TM][TN], char* smem)
    {
        if (K % BK == 0)
            TileGemmDtl<T, A_KMAJOR, B_KMAJOR, BK, 32>::run(A, B, K, acc, smem);
        else
            run_staged(A, B, K, acc, smem);
    }
};

// ------------------------------------------------------------------------------------------- //
// Direct-to-LDS main loop (K a multiple of BK).
//
// Global memory is copied straight into LDS by `global_load_lds_dwordx4` (each lane's 16 bytes land
// at M0 + lane * 16, so one wavefront instruction fills 1 KiB of consecutive LDS): no staging
// registers, no LDS store instructions.  Because the destination is dense, bank conflicts are
// avoided by an XOR swizzle applied on the GLOBAL side (which 16-byte chunk a lane fetches):
//   K-contiguous tile, row r (128 B), chunk c      -> LDS  r*128 + ((c ^ ((r >> 1) & 7)) * 16)
//   K-major tile,      k-line k (512 B), chunk c   -> LDS  k*512 + ((c ^ kmajor_swizzle(k)) * 16)
// which makes both the b128 fragment reads and the transposing b64 reads conflict-free.
// Two LDS stages of BK = 64.  All loads of K step kt+2 are issued during the second slice of step
// kt (right after the barrier that frees their buffer), a full K step ahead of the barrier that
// publishes them.
// ------------------------------------------------------------------------------------------- //
// s_waitcnt immediate that waits only for vmcnt <= n (expcnt and lgkmcnt left at "no wait").
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// Chunk swizzle of k-line k of a K-major tile: the four k-lines one transposing read touches
// (k & 3) move by 4 chunks each, the two 8-line blocks that the lower 32 lanes of a fragment read
// cover ((k >> 3) & 1) by 2 chunks, so those 32 lanes hit 32 different 8-byte bank pairs.
__device__ inline int kmajor_swizzle(int k) { return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1); }

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
                const int c = (lane & 31) ^ kmajor_swizzle(k);
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

    // MFMA 16x16x32 operand fragment: lane l holds row (row0 + l%16), k = kk*32 + 8*(l/16) + 0..7
    // (row0 a multiple of 16).
    __device__ static inline u32x4_t frag(const char* lds, int row0, int kk)
    {
        const int l = threadIdx.x & 63;
        if (KMAJOR) {
            const int g = l >> 4;
            const int a = (l & 15) >> 2;
            const int b = l & 3;
            const int kline = kk * 32 + 8 * g + a;                  // kline & 3 == a, bit 3 == g & 1
            const int c = (row0 >> 3) + (b >> 1);
            const char* p0 = lds + kline * 512 + ((c ^ ((a << 2) ^ ((g & 1) << 1))) * 16) + (b & 1) * 8;
            const char* p1 = p0 + 4 * 512;                           // k-line + 4: same swizzle
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p0));
            s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RLK_LDS s16x4_t*)(p1));
            u32x2_t lo2 = __builtin_bit_cast(u32x2_t, lo);
            u32x2_t hi2 = __builtin_bit_cast(u32x2_t, hi);
            return u32x4_t{lo2.x, lo2.y, hi2.x, hi2.y};
        } else {
            const int r = row0 + (l & 15);
            const int c = (4 * kk + (l >> 4)) ^ (((l & 15) >> 1) & 7);
            return *reinterpret_cast<const u32x4_t*>(lds + r * 128 + c * 16);
        }
    }
};

// WIN: MFMA slots (of the 32 of the second slice) over which the 8 loads of a K step are spread.
// 32 spaces them evenly over the slice; 16 sends them all out in its first half, which the
// persistent dZ and dH kernels prefer (they stall more on operand loads than the forward).
template <class T, bool A_KMAJOR, bool B_KMAJOR, int BK, int WIN>
struct TileGemmDtl {
    using AT = Acc16;
    static constexpr int TM = AT::TM;
    static constexpr int TN = AT::TN;
    static constexpr int KK = BK / 32;
    static_assert(KK == 2, "the loop is written for two 32-wide slices per K step");
    using IOA = DtlIO<A_KMAJOR, 256, BK>;
    using IOB = DtlIO<B_KMAJOR, 256, BK>;
    using Plan = FragPlan<TM, TN>;
    static constexpr int PA = IOA::kPasses;
    static constexpr int PB = IOB::kPasses;
    static constexpr int NL = PA + PB;                 // loads per wavefront per K step
    static constexpr int NM = TM * TN;                 // MFMAs per slice
    static_assert(WIN >= NL && WIN <= NM, "load window must lie inside the second slice");
    static constexpr int kStageBytes = IOA::kBytes + IOB::kBytes;
    static constexpr int kSmemBytes = 2 * kStageBytes;

    // Slice KKI of K step kt.  The second slice also issues the loads of step kt+2 into the stage
    // this step has just finished reading (`cur`).
    template <int KKI>
    __device__ static inline void slice(const IOA& la, const IOB& lb, u32x4_t (&fa)[2][TM],
                                        u32x4_t (&fb)[2][TN], int wm, int wn, int kt,
                                        char* cur, char* nxt, f32x4_t (&acc)[TM][TN])
    {
        constexpr bool last = KKI == KK - 1;
        constexpr int setc = KKI & 1, setn = setc ^ 1;
        const char* rsrc = last ? nxt : cur;
        constexpr int kkn = last ? 0 : KKI + 1;
        static_for<0, NM>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int i = q / TN, j = q % TN;
            acc[i][j] = T::mfma(fa[setc][i], fb[setc][j], acc[i][j]);
            static_for<0, Plan::kReads>([&](auto oc) {
                constexpr int o = decltype(oc)::value;
                if constexpr (Plan::slot_of(o) == q) {
                    if constexpr (o < TN)
                        fb[setn][o] = IOB::frag(rsrc + IOA::kBytes, wn * (TN * 16) + o * 16, kkn);
                    else
                        fa[setn][o - TN] = IOA::frag(rsrc, wm * (TM * 16) + (o - TN) * 16, kkn);
                }
            });
            if constexpr (last) {
                constexpr int lo = (q * NL + WIN - 1) / WIN;        // ceil
                constexpr int hi = ((q + 1) * NL + WIN - 1) / WIN;  // ceil
                static_for<(lo < NL ? lo : NL), (hi < NL ? hi : NL)>([&](auto lc) {
                    constexpr int g = decltype(lc)::value;
                    if constexpr (g < PA)
                        la.load_one(kt + 2, cur, g);  // past the end = next tile (load_one)
                    else
                        lb.load_one(kt + 2, cur + IOA::kBytes, g - PA);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    }

    // Pipeline state that lives across the tiles one workgroup computes back to back: the K loop
    // of a tile fetches the first two K steps of the next tile where it would otherwise run dry,
    // so only the first tile of a workgroup pays the fill latency.
    struct Stream {
        IOA la;
        IOB lb;
        u32x4_t fa[2][TM];
        u32x4_t fb[2][TN];
        int wm, wn, nk, phase;
    };

    __device__ static inline void first_frags(Stream& st, const char* stage)
    {
#pragma unroll
        for (int j = 0; j < TN; ++j)
            st.fb[0][j] = IOB::frag(stage + IOA::kBytes, st.wn * (TN * 16) + j * 16, 0);
#pragma unroll
        for (int i = 0; i < TM; ++i) st.fa[0][i] = IOA::frag(stage, st.wm * (TM * 16) + i * 16, 0);
    }

    // Fill the pipeline for the first tile: K step 0 in LDS and published, the fragments of its
    // first slice in registers, K step 1 in flight.
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
        static_for<0, PA>([&](auto pc) { st.la.load_one(0, smem, decltype(pc)::value); });
        static_for<0, PB>(
            [&](auto pc) { st.lb.load_one(0, smem + IOA::kBytes, decltype(pc)::value); });
        // K step 1 (with a single K step: the same step again, into the stage nobody reads)
        static_for<0, PA>([&](auto pc) { st.la.load_one(1, smem + kStageBytes, decltype(pc)::value); });
        static_for<0, PB>([&](auto pc) {
            st.lb.load_one(1, smem + kStageBytes + IOA::kBytes, decltype(pc)::value);
        });
        constexpr int wait_first = vmcnt_imm(NL);
        __builtin_amdgcn_s_waitcnt(wait_first);  // K step 0 has landed
        __syncthreads();
        first_frags(st, smem);
    }

    // All K steps of the current tile into `acc`.  `next_a` / `next_b` are the operand origins of
    // the tile that follows (same leading dimensions and row counts; pass the current origins
    // after the last tile: the extra fetches then stay inside the same tile).  Callers that chain
    // tiles need K >= 2 * BK (the loop looks two K steps ahead and knows one following tile).  On
    // return the stream stands at the start of that tile exactly as begin() leaves it: its K step
    // 0 published, its K step 1 in flight.
    // REFETCH: the fragments of the first slice are read again from LDS here instead of being
    // carried in registers from the previous tile's last slice; callers with a register-hungry
    // epilogue between tiles use it (the K step they come from is already published).
    // YOUNGER: since the previous tile() returned, the caller's epilogue issued at least this many
    // vector-memory instructions per wavefront (stores that may still be in flight).  The counter
    // retires in issue order, so the first K step only has to wait until at most YOUNGER
    // operations are outstanding to know that its own loads, which are older, have landed; the
    // stores drain under the MFMAs instead of in front of the barrier.  A value below the true
    // count is safe.  `counted` (uniform) says whether that promise holds for the epilogue that
    // just ran.
    template <bool REFETCH = false, int YOUNGER = 0>
    __device__ static inline void tile(Stream& st, const void* next_a, const void* next_b,
                                       f32x4_t (&acc)[TM][TN], char* smem, bool counted = false)
    {
        st.la.next = reinterpret_cast<const char*>(next_a);
        st.lb.next = reinterpret_cast<const char*>(next_b);
        const int nk = st.nk;
        if constexpr (REFETCH) first_frags(st, smem + (st.phase & 1) * kStageBytes);
        for (int kt = 0; kt < nk; ++kt) {
            char* cur = smem + ((kt + st.phase) & 1) * kStageBytes;
            char* nxt = smem + ((kt + st.phase + 1) & 1) * kStageBytes;
            slice<0>(st.la, st.lb, st.fa, st.fb, st.wm, st.wn, kt, cur, nxt, acc);
            constexpr int wait_older = vmcnt_imm(YOUNGER < 63 ? YOUNGER : 63);
            constexpr int wait_all = vmcnt_imm(0);
            if (YOUNGER > 0 && kt == 0 && counted)   // uniform
                __builtin_amdgcn_s_waitcnt(wait_older);
            else
                __builtin_amdgcn_s_waitcnt(wait_all);  // my loads of K step kt+1 have landed
            __syncthreads();
            slice<1>(st.la, st.lb, st.fa, st.fb, st.wm, st.wn, kt, cur, nxt, acc);
        }
        st.phase = (st.phase + nk) & 1;
        st.la.base = st.la.next;
        st.lb.base = st.lb.next;
    }

    // Drain the fetches issued for a tile that will not be computed; LDS is free afterwards.
    __device__ static inline void end(Stream&)
    {
        constexpr int wait_drain = vmcnt_imm(0);
        __builtin_amdgcn_s_waitcnt(wait_drain);
        __syncthreads();
    }

    __device__ static inline void run(const Operand& A, const Operand& B, int K,
                                      f32x4_t (&acc)[TM][TN], char* smem)
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
