// gemm.hip - FP32 GEMM family on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32):
//   C[M,N] (+)= op(A) * op(B)      NN = dgrad, TN(+=) = wgrad, NT = forward, TT for completeness.
//
// Shape of the kernel
//   * 256 lanes = 4 wavefronts in a 2x2 grid; each wave owns TM x TN MFMA blocks of 32x32,
//     so the workgroup tile is (64 TM) x (64 TN): 128x128 for the large backward GEMMs and
//     64x64 when a 128x128 grid would leave most of the 256 CUs idle.
//   * K advances 32 at a time through a double-buffered LDS stage; the next stage's global
//     loads are issued into registers before the current stage's MFMAs and written to the
//     other LDS buffer afterwards, so one barrier per stage is enough.
//   * An operand keeps the orientation it has in memory.  "k-contiguous" operands
//     (A in NN/NT, B in NT) sit in LDS as [mn][32+4]; a lane fetches four consecutive k
//     with one 16-byte LDS read and feeds them to four successive MFMA steps.
//     "mn-contiguous" operands (A in TN, B in NN/TN) sit as [k][tile+4] and are fetched
//     four bytes at a time, 32 consecutive lanes on 32 consecutive addresses.  Within a
//     step the two half-waves supply k = 4h+s and both operands use that same mapping,
//     so no transpose is ever materialised.
//   * Workgroup ids are first regrouped per XCD (ids are dealt round-robin to the 8 XCDs,
//     each with a private L2), then walked in bands 8 tiles tall so the tiles an XCD holds
//     at one time share operand panels in its L2.
// Accumulator layout of the 32x32x2 instruction: lane l, register v holds
//   row 8*(v/4) + 4*(l/32) + v%4, column l%32.
#include "common.hpp"
#include <type_traits>

namespace seraph {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kBK = 32;                 // K extent of one LDS stage
constexpr int kPadK = 4;                // [mn][kBK + kPadK]: 16-byte reads of 8 lanes fall on distinct banks
constexpr int kPadM = 4;                // [k][tile + kPadM]
constexpr int kGemmThreads = 256;
constexpr int kGroupM = 8;

__device__ __forceinline__ int xcd_regroup(int bid, int total) {
    // Contiguous range of logical ids per XCD; a bijection on [0,total) for any total.
    const int per = (total + kNumXcd - 1) / kNumXcd;
    int tall = total % kNumXcd;
    if (tall == 0) tall = kNumXcd;
    const int xcd = bid % kNumXcd, local = bid / kNumXcd;
    return xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
}

// One operand tile (TILE rows of mn, kBK of k) from global memory into registers.
// KC: the operand is stored [mn_total, K] (k contiguous); otherwise [K, mn_total].
template <int TILE, bool KC, bool VEC>
struct TileLoader {
    static constexpr int kSlots = TILE * kBK / 4 / kGemmThreads;      // float4 slots per lane
    float4 r[kSlots];

    __device__ __forceinline__ void load(const float* __restrict__ P, int64_t ld, int64_t mn0, int64_t mn_total,
                                         int64_t k0, int64_t K) {
#pragma unroll
        for (int u = 0; u < kSlots; u++) {
            const int f = threadIdx.x + kGemmThreads * u;
            int64_t mn, k;
            if (KC) { mn = mn0 + f / (kBK / 4); k = k0 + 4 * (f % (kBK / 4)); }
            else    { k = k0 + f / (TILE / 4);  mn = mn0 + 4 * (f % (TILE / 4)); }
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (VEC) {
                // ld % 4 == 0 and both origins are multiples of 4: a slot is wholly inside or wholly outside
                if (mn < mn_total && k < K)
                    v = *reinterpret_cast<const float4*>(P + (KC ? mn * ld + k : k * ld + mn));
            } else {
                float* e = &v.x;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int64_t mq = KC ? mn : mn + q, kq = KC ? k + q : k;
                    if (mq < mn_total && kq < K) e[q] = P[KC ? mq * ld + kq : kq * ld + mq];
                }
            }
            r[u] = v;
        }
    }

    __device__ __forceinline__ void store(float* __restrict__ lds) const {
#pragma unroll
        for (int u = 0; u < kSlots; u++) {
            const int f = threadIdx.x + kGemmThreads * u;
            int off;
            if (KC) off = (f / (kBK / 4)) * (kBK + kPadK) + 4 * (f % (kBK / 4));
            else    off = (f / (TILE / 4)) * (TILE + kPadM) + 4 * (f % (TILE / 4));
            *reinterpret_cast<float4*>(lds + off) = r[u];
        }
    }
};

template <int TILE, bool KC>
constexpr int lds_floats() { return KC ? TILE * (kBK + kPadK) : kBK * (TILE + kPadM); }

template <int TM, int TN, bool A_KC, bool B_KC, bool VEC>
__global__ __launch_bounds__(kGemmThreads) void gemm_f32_mfma_kernel(const float* __restrict__ A,
                                                                     const float* __restrict__ B,
                                                                     float* __restrict__ C,
                                                                     int64_t M, int64_t N, int64_t K,
                                                                     int accumulate, int nbm, int nbn) {
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int A_FLOATS = lds_floats<BM, A_KC>(), B_FLOATS = lds_floats<BN, B_KC>();
    __shared__ __attribute__((aligned(16))) float lds_a[2][A_FLOATS];
    __shared__ __attribute__((aligned(16))) float lds_b[2][B_FLOATS];

    // ---- tile assignment
    const int total = nbm * nbn;
    const int pid = xcd_regroup(blockIdx.x, total);
    const int width = kGroupM * nbn;
    const int group = pid / width;
    const int first_m = group * kGroupM;
    const int gsize = (nbm - first_m) < kGroupM ? (nbm - first_m) : kGroupM;
    const int pm = first_m + (pid % width) % gsize;
    const int pn = (pid % width) / gsize;
    const int64_t m0 = (int64_t)pm * BM, n0 = (int64_t)pn * BN;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int wm0 = (wave >> 1) * (32 * TM), wn0 = (wave & 1) * (32 * TN);

    const int64_t lda = A_KC ? K : M, ldb = B_KC ? K : N;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    TileLoader<BM, A_KC, VEC> la;
    TileLoader<BN, B_KC, VEC> lb;
    const int nk = (int)((K + kBK - 1) / kBK);

    la.load(A, lda, m0, M, 0, K);
    lb.load(B, ldb, n0, N, 0, K);
    la.store(lds_a[0]);
    lb.store(lds_b[0]);
    __syncthreads();

    for (int kt = 0; kt < nk; kt++) {
        const int cur = kt & 1;
        if (kt + 1 < nk) {
            la.load(A, lda, m0, M, (int64_t)(kt + 1) * kBK, K);
            lb.load(B, ldb, n0, N, (int64_t)(kt + 1) * kBK, K);
        }
        const float* sa = lds_a[cur];
        const float* sb = lds_b[cur];
        // Operand fragments are read from LDS one 8-deep slab ahead of the MFMAs that use them.
        float fa[2][TM][4], fb[2][TN][4];
        auto read_slab = [&](int slab, int buf) {
#pragma unroll
            for (int i = 0; i < TM; i++) {
                if (A_KC) {
                    const float4 t = *reinterpret_cast<const float4*>(sa + (wm0 + 32 * i + r) * (kBK + kPadK) + slab * 8 + 4 * h);
                    fa[buf][i][0] = t.x; fa[buf][i][1] = t.y; fa[buf][i][2] = t.z; fa[buf][i][3] = t.w;
                } else {
#pragma unroll
                    for (int q = 0; q < 4; q++) fa[buf][i][q] = sa[(slab * 8 + 4 * h + q) * (BM + kPadM) + wm0 + 32 * i + r];
                }
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (B_KC) {
                    const float4 t = *reinterpret_cast<const float4*>(sb + (wn0 + 32 * j + r) * (kBK + kPadK) + slab * 8 + 4 * h);
                    fb[buf][j][0] = t.x; fb[buf][j][1] = t.y; fb[buf][j][2] = t.z; fb[buf][j][3] = t.w;
                } else {
#pragma unroll
                    for (int q = 0; q < 4; q++) fb[buf][j][q] = sb[(slab * 8 + 4 * h + q) * (BN + kPadM) + wn0 + 32 * j + r];
                }
            }
        };
        read_slab(0, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
#pragma unroll
        for (int slab = 0; slab < kBK / 8; slab++) {
            if (slab + 1 < kBK / 8) read_slab(slab + 1, (slab + 1) & 1);
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[slab & 1][i][q], fb[slab & 1][j][q], acc[i][j], 0, 0, 0);
            if (slab + 1 < kBK / 8) __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 4 * TM * TN, 0);
        }
        if (kt + 1 < nk) {
            la.store(lds_a[cur ^ 1]);
            lb.store(lds_b[cur ^ 1]);
        }
        __syncthreads();
    }

    // ---- epilogue
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int64_t col = n0 + wn0 + 32 * j + r;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t row = m0 + wm0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
                if (row < M && col < N) {
                    float* dst = C + row * N + col;
                    *dst = accumulate ? *dst + acc[i][j][v] : acc[i][j][v];
                }
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Pipelined kernel for the aligned case (K a multiple of 32, 16-byte aligned rows): the same
// tiling, LDS layout and fragment mapping as above, with everything that is not a matrix
// instruction, an LDS access or a global load moved out of the K loop.
//   * Global addresses are a uniform tile pointer (scalar registers, advanced once per stage)
//     plus a per-lane 32-bit offset fixed before the loop.  Rows past the edge of the operand
//     are clamped to the last valid row: they feed only output rows/columns that are never
//     stored, so no per-element predicate is needed.
//   * A stage is four 8-deep slabs.  The fragments of slab s+1 are read from LDS while the 16
//     matrix instructions of slab s issue; the next stage's tile is written to the other LDS
//     buffer after slab 2, and the barrier plus the first fragment read of the next stage sit
//     in front of slab 3's matrix instructions, which do not depend on them.
// A wave-uniform pointer moved into scalar registers, so that loads through it take the
// scalar-base + 32-bit lane offset form and need no per-lane address arithmetic.
template <typename T>
__device__ __forceinline__ T* scalar_ptr(T* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
}

template <int TILE, bool KC, int NSET = 2>
struct FastLoader {
    static constexpr int kSlots = TILE * kBK / 4 / kGemmThreads;
    uint32_t off[kSlots];                                  // byte offsets
    float4 r[NSET][kSlots];                                // NSET tiles in flight

    // offsets relative to the tile origin (KC: P + mn0*ld + k0, else P + k0*ld + mn0)
    __device__ __forceinline__ void init(int64_t ld, int64_t mn0, int64_t mn_total) {
#pragma unroll
        for (int u = 0; u < kSlots; u++) {
            const int f = threadIdx.x + kGemmThreads * u;
            if (KC) {
                int64_t row = mn0 + f / (kBK / 4);
                if (row > mn_total - 1) row = mn_total - 1;
                off[u] = (uint32_t)(4 * ((row - mn0) * ld + 4 * (f % (kBK / 4))));
            } else {
                int64_t mn = mn0 + 4 * (f % (TILE / 4));
                if (mn > mn_total - 4) mn = mn_total - 4;
                off[u] = (uint32_t)(4 * ((int64_t)(f / (TILE / 4)) * ld + (mn - mn0)));
            }
        }
    }
    template <int SET>
    __device__ __forceinline__ void load(const float* __restrict__ tile) {
        // buffer load: scalar descriptor (base = tile origin) + 32-bit lane offset, no address arithmetic
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(tile), 0, 0x7fffffff, 0x00020000);
#pragma unroll
        for (int u = 0; u < kSlots; u++)
            r[SET][u] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off[u], 0, 0));
    }
    template <int SET>
    __device__ __forceinline__ void store(float* __restrict__ lds) const {
#pragma unroll
        for (int u = 0; u < kSlots; u++) {
            const int f = threadIdx.x + kGemmThreads * u;
            int o;
            if (KC) o = (f / (kBK / 4)) * (kBK + kPadK) + 4 * (f % (kBK / 4));
            else    o = (f / (TILE / 4)) * (TILE + kPadM) + 4 * (f % (TILE / 4));
            *reinterpret_cast<float4*>(lds + o) = r[SET][u];
        }
    }
};

// pid: the workgroup's tile number within this product (0 .. nbm * nbn - 1), already regrouped per XCD
// With CHAIN the tile is the sum of several products that share M and N (terms of one input gradient: gate and up, or
// q, k and v): the accumulators stay in registers from one term to the next and C is written once.
constexpr int kMaxChain = 3;
struct GemmChain {
    const float* A[kMaxChain]; const float* B[kMaxChain];
    int64_t K[kMaxChain];
    int count;
};

template <int TM, int TN, bool A_KC, bool B_KC, bool CHAIN = false>
__device__ __forceinline__ void pipelined_body(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                               int64_t M, int64_t N, int64_t K, int accumulate, int nbm, int nbn, int pid,
                                               const GemmChain* chain = nullptr) {
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int A_FLOATS = lds_floats<BM, A_KC>(), B_FLOATS = lds_floats<BN, B_KC>();
    __shared__ __attribute__((aligned(16))) float lds_a[2][A_FLOATS];
    __shared__ __attribute__((aligned(16))) float lds_b[2][B_FLOATS];

    const int width = kGroupM * nbn;
    const int group = pid / width;
    const int first_m = group * kGroupM;
    const int gsize = (nbm - first_m) < kGroupM ? (nbm - first_m) : kGroupM;
    const int pm = first_m + (pid % width) % gsize;
    const int pn = (pid % width) / gsize;
    const int64_t m0 = (int64_t)pm * BM, n0 = (int64_t)pn * BN;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int wm0 = (wave >> 1) * (32 * TM), wn0 = (wave & 1) * (32 * TN);

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int terms = CHAIN ? chain->count : 1;
    for (int term = 0; term < terms; term++) {
    if (CHAIN) {
        A = chain->A[term]; B = chain->B[term]; K = chain->K[term];
        if (term > 0) __syncthreads();                       // the previous term's last fragment reads precede this term's first LDS writes
    }
    const int64_t lda = A_KC ? K : M, ldb = B_KC ? K : N;
    FastLoader<BM, A_KC> la;
    FastLoader<BN, B_KC> lb;
    la.init(lda, m0, M);
    lb.init(ldb, n0, N);
    const float* ta = A_KC ? A + m0 * lda : A + m0;          // tile origin at k = 0 (uniform)
    const float* tb = B_KC ? B + n0 * ldb : B + n0;
    const int64_t step_a = A_KC ? kBK : kBK * lda, step_b = B_KC ? kBK : kBK * ldb;
    const int nk = (int)(K / kBK);

    // per-lane LDS fragment addresses (floats) inside one buffer
    const int fa_off = A_KC ? (wm0 + r) * (kBK + kPadK) + 4 * h : (4 * h) * (BM + kPadM) + wm0 + r;
    const int fb_off = B_KC ? (wn0 + r) * (kBK + kPadK) + 4 * h : (4 * h) * (BN + kPadM) + wn0 + r;

    float fa[2][TM][4], fb[2][TN][4];
    auto read_slab = [&](const float* sa, const float* sb, int slab, int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
            if (A_KC) {
                const float4 t = *reinterpret_cast<const float4*>(sa + fa_off + 32 * i * (kBK + kPadK) + slab * 8);
                fa[buf][i][0] = t.x; fa[buf][i][1] = t.y; fa[buf][i][2] = t.z; fa[buf][i][3] = t.w;
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) fa[buf][i][q] = sa[fa_off + (slab * 8 + q) * (BM + kPadM) + 32 * i];
            }
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if (B_KC) {
                const float4 t = *reinterpret_cast<const float4*>(sb + fb_off + 32 * j * (kBK + kPadK) + slab * 8);
                fb[buf][j][0] = t.x; fb[buf][j][1] = t.y; fb[buf][j][2] = t.z; fb[buf][j][3] = t.w;
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) fb[buf][j][q] = sb[fb_off + (slab * 8 + q) * (BN + kPadM) + 32 * j];
            }
        }
    };
    auto mfma_slab = [&](int buf) {
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[buf][i][q], fb[buf][j][q], acc[i][j], 0, 0, 0);
    };
    constexpr int kMfmaPerSlab = 4 * TM * TN;

    // Tile t travels global -> register set (t & 1) -> LDS buffer (t & 1).  Stage kt issues the
    // loads of tile kt+2 and, after slab 2, moves tile kt+1 (loaded during stage kt-1) into LDS,
    // so a load has more than a whole stage of matrix work to complete.  The loop body has no
    // branches: past the end of K the last tile is simply loaded and staged again (never used),
    // which keeps the compiler's wait counts exact (a conditional load would force every wait to
    // assume the load had not been issued).
    la.template load<0>(ta);
    lb.template load<0>(tb);
    if (nk > 1) { ta += step_a; tb += step_b; }
    la.template load<1>(ta);
    lb.template load<1>(tb);
    if (nk > 2) { ta += step_a; tb += step_b; }
    la.template store<0>(lds_a[0]);
    lb.template store<0>(lds_b[0]);
    __syncthreads();
    read_slab(lds_a[0], lds_b[0], 0, 0);

    auto stage = [&](auto parity, int kt) {
        constexpr int CUR = decltype(parity)::value;
        const float* sa = lds_a[CUR];
        const float* sb = lds_b[CUR];
        la.template load<CUR>(ta);
        lb.template load<CUR>(tb);
        const bool adv = kt + 3 < nk;
        ta += adv ? step_a : 0;
        tb += adv ? step_b : 0;
        // Source order: everything a slab needs is requested before its matrix instructions.  The
        // group barriers then deal the memory instructions out one at a time between consecutive
        // matrix instructions (a 32x32x2 takes 64 cycles and lets other instruction types issue
        // meanwhile), so no burst of loads, LDS writes or the barrier leaves the matrix pipe idle.
        constexpr int kPairs = kMfmaPerSlab < 8 ? kMfmaPerSlab : 8;
        constexpr int kRest = kMfmaPerSlab - kPairs;
        auto deal = [&](auto mask) {                       // kPairs x { 1 MFMA, 1 instruction of `mask` }
#pragma unroll
            for (int g = 0; g < kPairs; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(decltype(mask)::value, 1, 0);
            }
        };
        constexpr std::integral_constant<int, 0x020> kVmem{};
        constexpr std::integral_constant<int, 0x100> kDsRead{};
        read_slab(sa, sb, 1, 1);
        mfma_slab(0);
        if (kRest > 0) {
            deal(kVmem);                                   // global loads of tile kt+2
#pragma unroll
            for (int g = 0; g < kRest; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);     // fragment reads of slab 1
            }
        } else {
            __builtin_amdgcn_sched_group_barrier(0x020, 2 * FastLoader<BM, A_KC>::kSlots, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmaPerSlab, 0);
        }
        read_slab(sa, sb, 2, 0);
        mfma_slab(1);
        deal(kDsRead);
        __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, kRest, 0);
        read_slab(sa, sb, 3, 1);
        la.template store<CUR ^ 1>(lds_a[CUR ^ 1]);
        lb.template store<CUR ^ 1>(lds_b[CUR ^ 1]);
        mfma_slab(0);
        deal(kDsRead);
        __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
        if (kRest > 0) {
#pragma unroll
            for (int g = 0; g < kRest; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);     // LDS writes of tile kt+1
            }
        }
        __builtin_amdgcn_sched_group_barrier(0x200, 32, 0);
        __syncthreads();
        read_slab(lds_a[CUR ^ 1], lds_b[CUR ^ 1], 0, 0);
        mfma_slab(1);
        deal(kDsRead);
        __builtin_amdgcn_sched_group_barrier(0x100, 32, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, kRest, 0);
    };
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
        stage(std::integral_constant<int, 0>{}, kt);
        stage(std::integral_constant<int, 1>{}, kt + 1);
    }
    if (kt < nk) stage(std::integral_constant<int, 0>{}, kt);
    }   // term

    // ---- epilogue: uniform tile pointer + 32-bit lane offsets; predicates only on edge tiles
    float* ct = scalar_ptr(C + m0 * N + n0);
    const bool full = (m0 + BM <= M) && (n0 + BN <= N);
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = wn0 + 32 * j + r;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = wm0 + 32 * i + 8 * (v >> 2) + 4 * h + (v & 3);
                const uint32_t o = 4u * ((uint32_t)row * (uint32_t)N + (uint32_t)col);
                if (full || (m0 + row < M && n0 + col < N)) {
                    float* dst = reinterpret_cast<float*>(reinterpret_cast<char*>(ct) + o);
                    *dst = accumulate ? *dst + acc[i][j][v] : acc[i][j][v];
                }
            }
        }
}

template <int TM, int TN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_f32_mfma_pipelined_kernel(const float* __restrict__ A,
                                                                               const float* __restrict__ B,
                                                                               float* __restrict__ C,
                                                                               int64_t M, int64_t N, int64_t K,
                                                                               int accumulate, int nbm, int nbn) {
    pipelined_body<TM, TN, A_KC, B_KC>(A, B, C, M, N, K, accumulate, nbm, nbn, xcd_regroup(blockIdx.x, nbm * nbn));
}

template <int TM, int TN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_f32_mfma_pipelined_chain_kernel(const GemmChain chain, float* __restrict__ C,
                                                                                     int64_t M, int64_t N, int accumulate, int nbm, int nbn) {
    pipelined_body<TM, TN, A_KC, B_KC, true>(nullptr, nullptr, C, M, N, 0, accumulate, nbm, nbn, xcd_regroup(blockIdx.x, nbm * nbn), &chain);
}

// Several products with the same K, operand orientations and accumulate flag in one launch (the q / k / v and the
// gate / up projections of a layer and their weight gradients): the tiles of all of them form one grid, so a product
// too small to fill the chip shares it with its siblings, and operands that siblings have in common (the layer input
// forward, the activations in the weight gradients) are fetched into each L2 once.  Every tile is computed exactly as
// the single-product kernel computes it.
constexpr int kMaxGroup = 4;
struct GemmGroup {
    const float* A[kMaxGroup]; const float* B[kMaxGroup]; float* C[kMaxGroup];
    int64_t M[kMaxGroup], N[kMaxGroup];
    int nbm[kMaxGroup], nbn[kMaxGroup], first[kMaxGroup + 1];      // first[i]: the product's first tile in the launch
    int count;
};

template <int TM, int TN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_f32_mfma_pipelined_grouped_kernel(const GemmGroup g, int64_t K, int accumulate) {
    const int pid = xcd_regroup(blockIdx.x, g.first[g.count]);
    int i = 0;
    while (i + 1 < g.count && pid >= g.first[i + 1]) i++;          // uniform
    pipelined_body<TM, TN, A_KC, B_KC>(g.A[i], g.B[i], g.C[i], g.M[i], g.N[i], K, accumulate, g.nbm[i], g.nbn[i], pid - g.first[i]);
}

// ---------------------------------------------------------------------------------------------
// Small outputs with a long K (weight gradients of narrow layers, the rank-sized LoRA products):
// too few 64x64 tiles to occupy the chip.  Here a workgroup owns a 32x32 tile of C and its four
// waves split every 32-deep K stage between them (wave w takes the 8-deep slab w); the four
// partial accumulators are added in a fixed order through LDS, so the result does not depend on
// timing.  Same loaders and staging as the pipelined kernel.
// With `slices` > 1 the grid's y index also cuts K into that many equal runs of stages; a workgroup then
// stores its tile of run y, unscaled, into part[y] (M x N each) and gemm_slices_sum_kernel adds the runs.
// With CHAIN the tile is the sum of several products (one run of K each): the four partial accumulators go on from one
// term to the next and meet in LDS once.
template <bool A_KC, bool B_KC, bool CHAIN = false>
__device__ __forceinline__ void splitk_body(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                            int64_t M, int64_t N, int64_t K, int accumulate, int nbn, int tile,
                                            int slices, int slice, float* __restrict__ part, const GemmChain* chain = nullptr) {
    constexpr int BT = 32;
    constexpr int A_FLOATS = lds_floats<BT, A_KC>(), B_FLOATS = lds_floats<BT, B_KC>();
    __shared__ __attribute__((aligned(16))) float lds_a[2][A_FLOATS];
    __shared__ __attribute__((aligned(16))) float lds_b[2][B_FLOATS];
    __shared__ __attribute__((aligned(16))) float red[4][BT * BT];
    const int pm = tile / nbn, pn = tile % nbn;
    const int64_t m0 = (int64_t)pm * BT, n0 = (int64_t)pn * BT;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;

    v16f acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;

    const int terms = CHAIN ? chain->count : 1;
    for (int term = 0; term < terms; term++) {                 // (a term's last stage ends with a barrier: its LDS reads are over)
    if (CHAIN) { A = chain->A[term]; B = chain->B[term]; K = chain->K[term]; }
    const int64_t lda = A_KC ? K : M, ldb = B_KC ? K : N;

    // Four stages of both operands in flight (two float4 per lane and stage): with one or two workgroups per
    // CU nothing else hides the memory latency, and two stages ahead is less than one round trip.
    constexpr int R = 4;
    FastLoader<BT, A_KC, R> la;
    FastLoader<BT, B_KC, R> lb;
    la.init(lda, m0, M);
    lb.init(ldb, n0, N);
    const int64_t k_run = K / slices, k0 = (int64_t)slice * k_run;               // whole stages: the launcher sees to it
    const float* ta = A_KC ? A + m0 * lda + k0 : A + m0 + k0 * lda;
    const float* tb = B_KC ? B + n0 * ldb + k0 : B + n0 + k0 * ldb;
    const int64_t step_a = A_KC ? kBK : kBK * lda, step_b = B_KC ? kBK : kBK * ldb;
    const int nk = (int)(k_run / kBK);
    // this wave's slab of a stage: k = 8*wave + 4h + q
    const int fa_off = A_KC ? r * (kBK + kPadK) + 8 * wave + 4 * h : (8 * wave + 4 * h) * (BT + kPadM) + r;
    const int fb_off = B_KC ? r * (kBK + kPadK) + 8 * wave + 4 * h : (8 * wave + 4 * h) * (BT + kPadM) + r;

    // stage i of the run sits in register set i % R; past the last stage the last one is simply requested again
    la.template load<0>(ta); lb.template load<0>(tb);
    if (nk > 1) { ta += step_a; tb += step_b; }
    la.template load<1>(ta); lb.template load<1>(tb);
    if (nk > 2) { ta += step_a; tb += step_b; }
    la.template load<2>(ta); lb.template load<2>(tb);
    if (nk > 3) { ta += step_a; tb += step_b; }
    la.template load<3>(ta); lb.template load<3>(tb);
    if (nk > 4) { ta += step_a; tb += step_b; }
    la.template store<0>(lds_a[0]);
    lb.template store<0>(lds_b[0]);
    __syncthreads();

    auto stage = [&](auto set, int kt) {
        constexpr int SET = decltype(set)::value, CUR = SET & 1;       // R is even: the LDS buffer follows the set's parity
        la.template load<SET>(ta);                                     // stage kt + R; set SET went to LDS a stage ago
        lb.template load<SET>(tb);
        const bool adv = kt + R + 1 < nk;
        ta += adv ? step_a : 0;
        tb += adv ? step_b : 0;
        float fa[4], fb[4];
        if (A_KC) {
            const float4 t = *reinterpret_cast<const float4*>(lds_a[CUR] + fa_off);
            fa[0] = t.x; fa[1] = t.y; fa[2] = t.z; fa[3] = t.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fa[q] = lds_a[CUR][fa_off + q * (BT + kPadM)];
        }
        if (B_KC) {
            const float4 t = *reinterpret_cast<const float4*>(lds_b[CUR] + fb_off);
            fb[0] = t.x; fb[1] = t.y; fb[2] = t.z; fb[3] = t.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fb[q] = lds_b[CUR][fb_off + q * (BT + kPadM)];
        }
#pragma unroll
        for (int q = 0; q < 4; q++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[q], fb[q], acc, 0, 0, 0);
        la.template store<(SET + 1) % R>(lds_a[CUR ^ 1]);
        lb.template store<(SET + 1) % R>(lds_b[CUR ^ 1]);
        __syncthreads();
    };
    int kt = 0;
    for (; kt + 3 < nk; kt += 4) {
        stage(std::integral_constant<int, 0>{}, kt);
        stage(std::integral_constant<int, 1>{}, kt + 1);
        stage(std::integral_constant<int, 2>{}, kt + 2);
        stage(std::integral_constant<int, 3>{}, kt + 3);
    }
    if (kt < nk) stage(std::integral_constant<int, 0>{}, kt);
    if (kt + 1 < nk) stage(std::integral_constant<int, 1>{}, kt + 1);
    if (kt + 2 < nk) stage(std::integral_constant<int, 2>{}, kt + 2);
    }   // term

    // fixed-order sum of the four partial tiles
#pragma unroll
    for (int v = 0; v < 16; v++) red[wave][(8 * (v >> 2) + 4 * h + (v & 3)) * BT + r] = acc[v];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < BT * BT / kGemmThreads; i++) {
        const int e = threadIdx.x + kGemmThreads * i;
        const int64_t row = m0 + e / BT, col = n0 + e % BT;
        if (row < M && col < N) {
            const float v = ((red[0][e] + red[1][e]) + red[2][e]) + red[3][e];
            if (slices > 1) {
                part[(int64_t)slice * M * N + row * N + col] = v;
            } else {
                float* dst = C + row * N + col;
                *dst = accumulate ? *dst + v : v;
            }
        }
    }
}

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 4) void gemm_f32_mfma_splitk_kernel(const float* __restrict__ A,
                                                                               const float* __restrict__ B,
                                                                               float* __restrict__ C,
                                                                               int64_t M, int64_t N, int64_t K,
                                                                               int accumulate, int nbm, int nbn,
                                                                               int slices, float* __restrict__ part) {
    (void)nbm;
    splitk_body<A_KC, B_KC>(A, B, C, M, N, K, accumulate, nbn, (int)blockIdx.x, slices, (int)blockIdx.y, part);
}

// the sum of up to three products into one C (one run of K each, no slices)
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 4) void gemm_f32_mfma_splitk_chain_kernel(const GemmChain chain, float* __restrict__ C,
                                                                                     int64_t M, int64_t N, int accumulate, int nbn) {
    splitk_body<A_KC, B_KC, true>(nullptr, nullptr, C, M, N, 0, accumulate, nbn, (int)blockIdx.x, 1, 0, nullptr, &chain);
}

// the grouped form of the above (one run of K, no slices); nbm / nbn / first count 32 x 32 tiles here
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 4) void gemm_f32_mfma_splitk_grouped_kernel(const GemmGroup g, int64_t K, int accumulate) {
    const int tile = (int)blockIdx.x;
    int i = 0;
    while (i + 1 < g.count && tile >= g.first[i + 1]) i++;
    splitk_body<A_KC, B_KC>(g.A[i], g.B[i], g.C[i], g.M[i], g.N[i], K, accumulate, g.nbn[i], tile - g.first[i], 1, 0, nullptr);
}

// ---------------------------------------------------------------------------------------------
// C[M,N] (+)= A[M,K] B[N,K]^T with K <= 32 (a rank-sized inner dimension): bound by the traffic of C, so no
// matrix instructions.  A lane keeps its four columns' rows of B in registers, a wave walks down rows of A,
// whose K values are the same for all lanes (scalar loads), and adds in ascending k.
template <int K4>
__device__ __forceinline__ void smallk_body(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                            int64_t M, int64_t N, int accumulate, int rows_per_wave, int block_x, int block_y);

template <int K4>
__global__ __launch_bounds__(256) void gemm_smallk_kernel(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                                          int64_t M, int64_t N, int accumulate, int rows_per_wave) {
    smallk_body<K4>(A, B, C, M, N, accumulate, rows_per_wave, (int)blockIdx.x, (int)blockIdx.y);
}

// C (+)= alpha * (part[0] + part[1] + ... ), the runs added in index order
__global__ __launch_bounds__(256) void gemm_slices_sum_kernel(const float* __restrict__ part, float* __restrict__ C, int64_t n,
                                                              int slices, float alpha, int accumulate) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = part[i];
    for (int p = 1; p < slices; p++) v += part[(int64_t)p * n + i];
    v *= alpha;
    C[i] = accumulate ? C[i] + v : v;
}

// ---------------------------------------------------------------------------------------------
// The rank-sized products of several LoRA adapters of one layer in one launch each.  Every product keeps its own K and
// its own number of runs, a workgroup is one (product, run, tile) and does what the single-product kernels above do
// for it: the results are the single calls' bits.
struct GemmRuns {
    const float* A[kMaxGroup]; const float* B[kMaxGroup]; float* C[kMaxGroup]; float* part[kMaxGroup];
    int64_t M[kMaxGroup], N[kMaxGroup], K[kMaxGroup];
    int nbn[kMaxGroup], tiles[kMaxGroup], slices[kMaxGroup];
    int first[kMaxGroup + 1];                                      // first workgroup of product i (runs kernel) / first block (sum kernel)
    int count;
};

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(kGemmThreads, 4) void gemm_f32_mfma_splitk_runs_grouped_kernel(const GemmRuns g) {
    const int wg = (int)blockIdx.x;
    int i = 0;
    while (i + 1 < g.count && wg >= g.first[i + 1]) i++;           // uniform
    const int local = wg - g.first[i];
    splitk_body<A_KC, B_KC>(g.A[i], g.B[i], g.C[i], g.M[i], g.N[i], g.K[i], 0, g.nbn[i], local % g.tiles[i], g.slices[i],
                            local / g.tiles[i], g.part[i]);
}

__global__ __launch_bounds__(256) void gemm_slices_sum_grouped_kernel(const GemmRuns g, float alpha, int accumulate) {
    const int b = (int)blockIdx.x;
    int i = 0;
    while (i + 1 < g.count && b >= g.first[i + 1]) i++;
    const int64_t n = g.M[i] * g.N[i];
    const int64_t e = (int64_t)(b - g.first[i]) * 256 + threadIdx.x;
    if (e >= n) return;
    const float* part = g.part[i];
    float v = part[e];
    for (int p = 1; p < g.slices[i]; p++) v += part[(int64_t)p * n + e];
    v *= alpha;
    float* C = g.C[i];
    C[e] = accumulate ? C[e] + v : v;
}

template <int K4>
__device__ __forceinline__ void smallk_body(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                            int64_t M, int64_t N, int accumulate, int rows_per_wave, int block_x, int block_y) {
    constexpr int K = 4 * K4;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t n = ((int64_t)block_x * 64 + lane) * 4;
    const bool col_ok = n < N;                                  // N is a multiple of 4
    float4 b[4][K4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int q = 0; q < K4; q++)
            b[j][q] = col_ok ? *reinterpret_cast<const float4*>(B + (n + j) * K + 4 * q) : make_float4(0.f, 0.f, 0.f, 0.f);
    const int64_t m0 = ((int64_t)block_y * 4 + wave) * rows_per_wave;
    for (int r = 0; r < rows_per_wave && m0 + r < M; r++) {
        const float* a = A + (m0 + r) * K;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < K4; q++) {
            const float4 av = *reinterpret_cast<const float4*>(a + 4 * q);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc[j] = fmaf(av.x, b[j][q].x, acc[j]);
                acc[j] = fmaf(av.y, b[j][q].y, acc[j]);
                acc[j] = fmaf(av.z, b[j][q].z, acc[j]);
                acc[j] = fmaf(av.w, b[j][q].w, acc[j]);
            }
        }
        if (col_ok) {
            float4* dst = reinterpret_cast<float4*>(C + (m0 + r) * N + n);
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
            if (accumulate) o = *dst;
            o.x += acc[0]; o.y += acc[1]; o.z += acc[2]; o.w += acc[3];
            *dst = o;
        }
    }
}

// grid x: the column blocks of all products one after the other; grid y: row blocks (of the tallest product)
template <int K4>
__global__ __launch_bounds__(256) void gemm_smallk_grouped_kernel(const GemmRuns g, int accumulate, int rows_per_wave) {
    const int b = (int)blockIdx.x;
    int i = 0;
    while (i + 1 < g.count && b >= g.first[i + 1]) i++;
    smallk_body<K4>(g.A[i], g.B[i], g.C[i], g.M[i], g.N[i], accumulate, rows_per_wave, b - g.first[i], (int)blockIdx.y);
}

// The pipelined kernel needs whole K stages, and every per-lane offset inside a tile panel
// (up to 128 rows of a k-contiguous operand, 32 rows of the other kind, 128 rows of C) in 32 bits.
static bool pipelined_ok(int64_t M, int64_t N, int64_t K, int tA, int tB) {
    const int64_t lda = tA ? M : K, ldb = tB ? K : N;
    const int64_t lim = (int64_t)1 << 31;
    return K >= kBK && K % kBK == 0 && M >= 4 && N >= 4 && 4 * 129 * lda < lim && 4 * 129 * ldb < lim && 4 * 129 * N < lim;
}

template <int TM, int TN>
static int launch_gemm(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                       int tA, int tB, int accumulate, bool vec, hipStream_t st) {
    const int64_t nbm = ceil_div(M, 64 * TM), nbn = ceil_div(N, 64 * TN);
    SERAPH_REQUIRE(nbm * nbn <= 0x7fffffff, "gemm: too many tiles");
    const dim3 grid((unsigned)(nbm * nbn)), block(kGemmThreads);
#define GO(AKC, BKC, V) \
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, TN, AKC, BKC, V>), grid, block, 0, st, A, B, C, M, N, K, accumulate, (int)nbm, (int)nbn)
#define GOFAST(AKC, BKC) \
    hipLaunchKernelGGL((gemm_f32_mfma_pipelined_kernel<TM, TN, AKC, BKC>), grid, block, 0, st, A, B, C, M, N, K, accumulate, (int)nbm, (int)nbn)
    // A is k-contiguous unless transposed; B is k-contiguous when transposed.
    if (vec && pipelined_ok(M, N, K, tA, tB)) {
        if (!tA && !tB) GOFAST(true, false);
        else if (!tA && tB) GOFAST(true, true);
        else if (tA && !tB) GOFAST(false, false);
        else GOFAST(false, true);
    } else if (vec) {
        if (!tA && !tB) GO(true, false, true);
        else if (!tA && tB) GO(true, true, true);
        else if (tA && !tB) GO(false, false, true);
        else GO(false, true, true);
    } else {
        if (!tA && !tB) GO(true, false, false);
        else if (!tA && tB) GO(true, true, false);
        else if (tA && !tB) GO(false, false, false);
        else GO(false, true, false);
    }
#undef GO
#undef GOFAST
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

}  // namespace seraph

using namespace seraph;

// 128x128 or 64x64 tiles, by the rounds the chip needs for them.  A CU works through ceil(tiles / CUs) big tiles, or
// through its small tiles two at a time (half a round is the step there); a small tile costs a quarter of a big one
// and runs at about 0.88 of its rate (measured: 2048 x 2816, K 512 with 352 big tiles 67 us, with 1408 small ones
// 57 us; 2048 x 8192, K 512 with 1024 / 4096 tiles 151 / 167 us; 2048 x 2048 x 2048 with 256 / 1024 tiles 135 / 140 us).
static bool big_tiles_pay(int64_t t128, int64_t t64) {
    const int64_t cus = num_compute_units();
    if (10 * t128 < 9 * cus) return false;                       // big tiles would leave more than a tenth of the chip idle
    const double cost128 = 4.0 * (double)ceil_div(t128, cus);
    const double cost64 = 0.5 * (double)ceil_div(2 * t64, cus) / 0.88;
    return cost128 <= cost64;
}
static bool use_big_tiles(int64_t M, int64_t N) {
    return big_tiles_pay(ceil_div(M, 128) * ceil_div(N, 128), ceil_div(M, 64) * ceil_div(N, 64));
}

// A k-contiguous pair of operands with at most 32 values of k and a C of whole 16-byte groups.
static bool use_smallk(const float* A, const float* B, const float* C, int64_t M, int64_t N, int64_t K, int tA, int tB) {
    return !tA && tB && K >= 4 && K <= 32 && K % 4 == 0 && N % 4 == 0 && M * N >= 65536 &&
           (!A || (aligned16(A) && aligned16(B) && aligned16(C)));
}

// 32x32 tiles whose four waves share out every K stage, instead of 64x64 tiles.  Always when there are fewer 64x64
// tiles than compute units.  Beyond that the small-tile kernel (four workgroups per CU, so a CU's last tiles still
// overlap each other's ramps) keeps winning while a CU would see only a few 64x64 tiles: measured on 2048 x 512 ...
// 2816 x 1024 outputs in all orientations, 352 tiles 55 against 75 us at K 2048 and 19 against 21 us at K 512, 512
// tiles 74 against 81 us (K 2048) but 24 against 22 us (K 512), 704 tiles 100 against 107 us (K 2048) and 31 against
// 30 us (K 512); from 1024 tiles on the 128x128 kernel is ahead of both.
static bool small_tiles_pay(int64_t t64, int64_t K) {
    const int64_t cus = num_compute_units();
    if (t64 < cus) return true;
    if (K >= 1024) return t64 < 4 * cus;
    return t64 > cus && 4 * t64 < 7 * cus;
}
static bool use_splitk(int64_t M, int64_t N, int64_t K, int tA, int tB) {
    return !use_big_tiles(M, N) && K >= 256 && small_tiles_pay(ceil_div(M, 64) * ceil_div(N, 64), K) && pipelined_ok(M, N, K, tA, tB);
}

extern "C" const char* seraph_gemm_kernel_name(int64_t M, int64_t N, int64_t K, int transpose_A, int transpose_B) {
    // names for 16-byte aligned operands (the case the training step always has)
    static const char* generic[2][4] = {
        {"seraph::gemm_f32_mfma_kernel<1, 1, true, false, true>", "seraph::gemm_f32_mfma_kernel<1, 1, true, true, true>",
         "seraph::gemm_f32_mfma_kernel<1, 1, false, false, true>", "seraph::gemm_f32_mfma_kernel<1, 1, false, true, true>"},
        {"seraph::gemm_f32_mfma_kernel<2, 2, true, false, true>", "seraph::gemm_f32_mfma_kernel<2, 2, true, true, true>",
         "seraph::gemm_f32_mfma_kernel<2, 2, false, false, true>", "seraph::gemm_f32_mfma_kernel<2, 2, false, true, true>"}};
    static const char* pipelined[2][4] = {
        {"seraph::gemm_f32_mfma_pipelined_kernel<1, 1, true, false>", "seraph::gemm_f32_mfma_pipelined_kernel<1, 1, true, true>",
         "seraph::gemm_f32_mfma_pipelined_kernel<1, 1, false, false>", "seraph::gemm_f32_mfma_pipelined_kernel<1, 1, false, true>"},
        {"seraph::gemm_f32_mfma_pipelined_kernel<2, 2, true, false>", "seraph::gemm_f32_mfma_pipelined_kernel<2, 2, true, true>",
         "seraph::gemm_f32_mfma_pipelined_kernel<2, 2, false, false>", "seraph::gemm_f32_mfma_pipelined_kernel<2, 2, false, true>"}};
    static const char* smallk[8] = {"seraph::gemm_smallk_kernel<1>", "seraph::gemm_smallk_kernel<2>", "seraph::gemm_smallk_kernel<3>",
                                    "seraph::gemm_smallk_kernel<4>", "seraph::gemm_smallk_kernel<5>", "seraph::gemm_smallk_kernel<6>",
                                    "seraph::gemm_smallk_kernel<7>", "seraph::gemm_smallk_kernel<8>"};
    if (use_smallk(nullptr, nullptr, nullptr, M, N, K, transpose_A, transpose_B)) return smallk[K / 4 - 1];
    const int64_t lda = transpose_A ? M : K, ldb = transpose_B ? K : N;
    const bool fast = lda % 4 == 0 && ldb % 4 == 0 && pipelined_ok(M, N, K, transpose_A, transpose_B);
    static const char* splitk[4] = {"seraph::gemm_f32_mfma_splitk_kernel<true, false>", "seraph::gemm_f32_mfma_splitk_kernel<true, true>",
                                    "seraph::gemm_f32_mfma_splitk_kernel<false, false>", "seraph::gemm_f32_mfma_splitk_kernel<false, true>"};
    if (fast && use_splitk(M, N, K, transpose_A, transpose_B)) return splitk[(transpose_A ? 2 : 0) + (transpose_B ? 1 : 0)];
    return (fast ? pipelined : generic)[use_big_tiles(M, N) ? 1 : 0][(transpose_A ? 2 : 0) + (transpose_B ? 1 : 0)];
}

extern "C" int seraph_gemm(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                           int transpose_A, int transpose_B, int accumulate, seraph_stream_t s) {
    if (M == 0 || N == 0) return SERAPH_OK;
    SERAPH_REQUIRE(A && B && C, "gemm: NULL pointer");
    SERAPH_REQUIRE(M > 0 && N > 0 && K >= 0, "gemm: bad shape %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
    const int64_t lda = transpose_A ? M : K, ldb = transpose_B ? K : N;
    const bool vec = (lda % 4 == 0) && (ldb % 4 == 0) && aligned16(A) && aligned16(B);
    hipStream_t st = as_stream(s);
    if (use_smallk(A, B, C, M, N, K, transpose_A, transpose_B)) {
        const int rows_per_wave = 8;
        const dim3 grid((unsigned)ceil_div(N, 256), (unsigned)ceil_div(M, 4 * rows_per_wave));
        SERAPH_REQUIRE(grid.y <= 65535u * 1024u, "gemm: too many rows");
        switch (K / 4) {
#define GOK(K4) case K4: hipLaunchKernelGGL(gemm_smallk_kernel<K4>, grid, dim3(256), 0, st, A, B, C, M, N, accumulate, rows_per_wave); break;
            GOK(1) GOK(2) GOK(3) GOK(4) GOK(5) GOK(6) GOK(7) GOK(8)
#undef GOK
        }
        SERAPH_LAUNCH_CHECK();
        return SERAPH_OK;
    }
    if (use_big_tiles(M, N))
        return launch_gemm<2, 2>(A, B, C, M, N, K, transpose_A, transpose_B, accumulate, vec, st);
    if (vec && use_splitk(M, N, K, transpose_A, transpose_B)) {
        const int64_t nbm = ceil_div(M, 32), nbn = ceil_div(N, 32);
        const dim3 grid((unsigned)(nbm * nbn)), block(kGemmThreads);
#define GOSK(AKC, BKC) \
    hipLaunchKernelGGL((gemm_f32_mfma_splitk_kernel<AKC, BKC>), grid, block, 0, st, A, B, C, M, N, K, accumulate, (int)nbm, (int)nbn, 1, \
                       (float*)nullptr)
        if (!transpose_A && !transpose_B) GOSK(true, false);
        else if (!transpose_A && transpose_B) GOSK(true, true);
        else if (transpose_A && !transpose_B) GOSK(false, false);
        else GOSK(false, true);
#undef GOSK
        SERAPH_LAUNCH_CHECK();
        return SERAPH_OK;
    }
    return launch_gemm<1, 1>(A, B, C, M, N, K, transpose_A, transpose_B, accumulate, vec, st);
}

// ---------------------------------------------------------------------------------------------
// Several products in one launch.  0: not groupable (a product that needs the general kernel), else the tile edge
// the group runs with: 128 or 64 (pipelined kernel) or 32 (the kernel whose waves split K).
static int group_tile(const seraph_gemm_problem_t* p, int count, int64_t K, int tA, int tB) {
    if (count < 2 || count > kMaxGroup) return 0;
    int64_t t128 = 0, t64 = 0, t32 = 0;
    for (int i = 0; i < count; i++) {
        const int64_t M = p[i].M, N = p[i].N, lda = tA ? M : K, ldb = tB ? K : N;
        if (M <= 0 || N <= 0 || !p[i].A || !p[i].B || !p[i].C) return 0;
        if (lda % 4 || ldb % 4 || !aligned16(p[i].A) || !aligned16(p[i].B) || !pipelined_ok(M, N, K, tA, tB)) return 0;
        if (use_smallk(p[i].A, p[i].B, p[i].C, M, N, K, tA, tB)) return 0;
        t128 += ceil_div(M, 128) * ceil_div(N, 128);
        t64 += ceil_div(M, 64) * ceil_div(N, 64);
        t32 += ceil_div(M, 32) * ceil_div(N, 32);
    }
    if (t32 > 0x7fffffff) return 0;
    if (big_tiles_pay(t128, t64)) return 128;
    return (K >= 256 && small_tiles_pay(t64, K)) ? 32 : 64;
}

extern "C" const char* seraph_gemm_grouped_kernel_name(const seraph_gemm_problem_t* problems, int count, int64_t K,
                                                       int transpose_A, int transpose_B) {
    static const char* names[3][4] = {
        {"seraph::gemm_f32_mfma_pipelined_grouped_kernel<2, 2, true, false>", "seraph::gemm_f32_mfma_pipelined_grouped_kernel<2, 2, true, true>",
         "seraph::gemm_f32_mfma_pipelined_grouped_kernel<2, 2, false, false>", "seraph::gemm_f32_mfma_pipelined_grouped_kernel<2, 2, false, true>"},
        {"seraph::gemm_f32_mfma_pipelined_grouped_kernel<1, 1, true, false>", "seraph::gemm_f32_mfma_pipelined_grouped_kernel<1, 1, true, true>",
         "seraph::gemm_f32_mfma_pipelined_grouped_kernel<1, 1, false, false>", "seraph::gemm_f32_mfma_pipelined_grouped_kernel<1, 1, false, true>"},
        {"seraph::gemm_f32_mfma_splitk_grouped_kernel<true, false>", "seraph::gemm_f32_mfma_splitk_grouped_kernel<true, true>",
         "seraph::gemm_f32_mfma_splitk_grouped_kernel<false, false>", "seraph::gemm_f32_mfma_splitk_grouped_kernel<false, true>"}};
    const int tile = problems ? group_tile(problems, count, K, transpose_A, transpose_B) : 0;
    if (!tile) return "gemm (group run as single products)";
    return names[tile == 128 ? 0 : tile == 64 ? 1 : 2][(transpose_A ? 2 : 0) + (transpose_B ? 1 : 0)];
}

extern "C" int seraph_gemm_grouped(const seraph_gemm_problem_t* problems, int count, int64_t K,
                                   int transpose_A, int transpose_B, int accumulate, seraph_stream_t s) {
    if (count <= 0) return SERAPH_OK;
    SERAPH_REQUIRE(problems, "gemm_grouped: NULL problem list");
    const int tile = group_tile(problems, count, K, transpose_A, transpose_B);
    if (!tile) {                                            // one launch each, exactly as seraph_gemm
        for (int i = 0; i < count; i++) {
            int rc = seraph_gemm(problems[i].A, problems[i].B, problems[i].C, problems[i].M, problems[i].N, K, transpose_A, transpose_B, accumulate, s);
            if (rc != SERAPH_OK) return rc;
        }
        return SERAPH_OK;
    }
    GemmGroup g;
    g.count = count;
    int total = 0;
    for (int i = 0; i < count; i++) {
        g.A[i] = problems[i].A; g.B[i] = problems[i].B; g.C[i] = problems[i].C; g.M[i] = problems[i].M; g.N[i] = problems[i].N;
        g.nbm[i] = (int)ceil_div(problems[i].M, tile); g.nbn[i] = (int)ceil_div(problems[i].N, tile);
        g.first[i] = total;
        total += g.nbm[i] * g.nbn[i];
    }
    for (int i = count; i <= kMaxGroup; i++) g.first[i] = total;
    hipStream_t st = as_stream(s);
    const dim3 grid((unsigned)total), block(kGemmThreads);
    const int form = (transpose_A ? 2 : 0) + (transpose_B ? 1 : 0);
#define GOG(KERNEL, ...) \
    switch (form) { \
        case 0: hipLaunchKernelGGL((KERNEL<__VA_ARGS__ true, false>), grid, block, 0, st, g, K, accumulate); break; \
        case 1: hipLaunchKernelGGL((KERNEL<__VA_ARGS__ true, true>), grid, block, 0, st, g, K, accumulate); break; \
        case 2: hipLaunchKernelGGL((KERNEL<__VA_ARGS__ false, false>), grid, block, 0, st, g, K, accumulate); break; \
        default: hipLaunchKernelGGL((KERNEL<__VA_ARGS__ false, true>), grid, block, 0, st, g, K, accumulate); break; \
    }
    if (tile == 128) { GOG(gemm_f32_mfma_pipelined_grouped_kernel, 2, 2,) }
    else if (tile == 64) { GOG(gemm_f32_mfma_pipelined_grouped_kernel, 1, 1,) }
    else { GOG(gemm_f32_mfma_splitk_grouped_kernel,) }
#undef GOG
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

// ---------------------------------------------------------------------------------------------
// C (+)= sum of products that share M and N: one launch when every term suits the pipelined loaders (whole K stages,
// 16-byte aligned operands), else one product after the other.
static bool chain_ok(const seraph_gemm_term_t* t, int count, const float* C, int64_t M, int64_t N, int tA, int tB) {
    if (count < 2 || count > kMaxChain || M <= 0 || N <= 0 || !C) return false;
    for (int i = 0; i < count; i++) {
        const int64_t K = t[i].K, lda = tA ? M : K, ldb = tB ? K : N;
        if (!t[i].A || !t[i].B || lda % 4 || ldb % 4 || !aligned16(t[i].A) || !aligned16(t[i].B)) return false;
        if (!pipelined_ok(M, N, K, tA, tB)) return false;
    }
    return ceil_div(M, 32) * ceil_div(N, 32) <= 0x7fffffff;
}
// The sum on 32x32 tiles whose waves share out K: with fewer 64x64 tiles than compute units.  From there up to the
// single product's limit (small_tiles_pay) the 32x32 form is 3 % ahead alone (2048 x 512 with K 1408 + 1408: 57 against
// 59 us) but 2.4 % behind inside the 33M step, where its 1024 workgroups crowd the weight gradients on the second
// stream (4.46 against 4.36 ms, alternating builds on one GPU): there the 64x64 form stays.
static bool chain_splitk(const seraph_gemm_term_t* t, int count, int64_t M, int64_t N) {
    int64_t ksum = 0;
    for (int i = 0; i < count; i++) ksum += t[i].K;
    return !use_big_tiles(M, N) && ksum >= 256 && ceil_div(M, 64) * ceil_div(N, 64) < num_compute_units();
}

extern "C" const char* seraph_gemm_chain_kernel_name(const seraph_gemm_term_t* terms, int count, const float* C, int64_t M, int64_t N,
                                                     int transpose_A, int transpose_B) {
    static const char* names[2][4] = {
        {"seraph::gemm_f32_mfma_pipelined_chain_kernel<1, 1, true, false>", "seraph::gemm_f32_mfma_pipelined_chain_kernel<1, 1, true, true>",
         "seraph::gemm_f32_mfma_pipelined_chain_kernel<1, 1, false, false>", "seraph::gemm_f32_mfma_pipelined_chain_kernel<1, 1, false, true>"},
        {"seraph::gemm_f32_mfma_pipelined_chain_kernel<2, 2, true, false>", "seraph::gemm_f32_mfma_pipelined_chain_kernel<2, 2, true, true>",
         "seraph::gemm_f32_mfma_pipelined_chain_kernel<2, 2, false, false>", "seraph::gemm_f32_mfma_pipelined_chain_kernel<2, 2, false, true>"}};
    if (!terms || !chain_ok(terms, count, C, M, N, transpose_A, transpose_B)) return "gemm (chain run as single products)";
    static const char* split[4] = {"seraph::gemm_f32_mfma_splitk_chain_kernel<true, false>", "seraph::gemm_f32_mfma_splitk_chain_kernel<true, true>",
                                   "seraph::gemm_f32_mfma_splitk_chain_kernel<false, false>", "seraph::gemm_f32_mfma_splitk_chain_kernel<false, true>"};
    if (chain_splitk(terms, count, M, N)) return split[(transpose_A ? 2 : 0) + (transpose_B ? 1 : 0)];
    return names[use_big_tiles(M, N) ? 1 : 0][(transpose_A ? 2 : 0) + (transpose_B ? 1 : 0)];
}

extern "C" int seraph_gemm_chain(const seraph_gemm_term_t* terms, int count, float* C, int64_t M, int64_t N,
                                 int transpose_A, int transpose_B, int accumulate, seraph_stream_t s) {
    if (count <= 0 || M == 0 || N == 0) return SERAPH_OK;
    SERAPH_REQUIRE(terms && C, "gemm_chain: NULL pointer");
    if (!chain_ok(terms, count, C, M, N, transpose_A, transpose_B)) {
        for (int i = 0; i < count; i++) {
            int rc = seraph_gemm(terms[i].A, terms[i].B, C, M, N, terms[i].K, transpose_A, transpose_B, (accumulate || i > 0) ? 1 : 0, s);
            if (rc != SERAPH_OK) return rc;
        }
        return SERAPH_OK;
    }
    GemmChain ch;
    ch.count = count;
    for (int i = 0; i < kMaxChain; i++) {
        const int j = i < count ? i : count - 1;
        ch.A[i] = terms[j].A; ch.B[i] = terms[j].B; ch.K[i] = terms[j].K;
    }
    hipStream_t st = as_stream(s);
    const int form = (transpose_A ? 2 : 0) + (transpose_B ? 1 : 0);
    if (chain_splitk(terms, count, M, N)) {
        const int64_t nbn = ceil_div(N, 32);
        const dim3 grid((unsigned)(ceil_div(M, 32) * nbn)), block(kGemmThreads);
        switch (form) {
            case 0: hipLaunchKernelGGL((gemm_f32_mfma_splitk_chain_kernel<true, false>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbn); break;
            case 1: hipLaunchKernelGGL((gemm_f32_mfma_splitk_chain_kernel<true, true>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbn); break;
            case 2: hipLaunchKernelGGL((gemm_f32_mfma_splitk_chain_kernel<false, false>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbn); break;
            default: hipLaunchKernelGGL((gemm_f32_mfma_splitk_chain_kernel<false, true>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbn); break;
        }
        SERAPH_LAUNCH_CHECK();
        return SERAPH_OK;
    }
    const bool big = use_big_tiles(M, N);
    const int tile = big ? 128 : 64;
    const int64_t nbm = ceil_div(M, tile), nbn = ceil_div(N, tile);
    const dim3 grid((unsigned)(nbm * nbn)), block(kGemmThreads);
#define GOC(TMN) \
    switch (form) { \
        case 0: hipLaunchKernelGGL((gemm_f32_mfma_pipelined_chain_kernel<TMN, TMN, true, false>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbm, (int)nbn); break; \
        case 1: hipLaunchKernelGGL((gemm_f32_mfma_pipelined_chain_kernel<TMN, TMN, true, true>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbm, (int)nbn); break; \
        case 2: hipLaunchKernelGGL((gemm_f32_mfma_pipelined_chain_kernel<TMN, TMN, false, false>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbm, (int)nbn); break; \
        default: hipLaunchKernelGGL((gemm_f32_mfma_pipelined_chain_kernel<TMN, TMN, false, true>), grid, block, 0, st, ch, C, M, N, accumulate, (int)nbm, (int)nbn); break; \
    }
    if (big) { GOC(2) } else { GOC(1) }
#undef GOC
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

// ---------------------------------------------------------------------------------------------
// C (+)= alpha * op(A) op(B) for products with a small output and a long K (the rank-sized LoRA products):
// K is cut into runs that separate workgroups take, the runs are added in a fixed order.
constexpr int kMaxSlices = 8;

// runs of at least four stages, about two workgroups per compute unit in all
static int slice_count(int64_t M, int64_t N, int64_t K, int tA, int tB) {
    if (!use_splitk(M, N, K, tA, tB)) return 1;
    const int64_t tiles = ceil_div(M, 32) * ceil_div(N, 32);
    int64_t s = 2 * (int64_t)num_compute_units() / tiles;
    if (s > kMaxSlices) s = kMaxSlices;
    while (s > 1 && (K % (s * kBK) != 0 || K / s < 4 * kBK)) s--;
    return (int)(s < 1 ? 1 : s);
}

extern "C" size_t seraph_gemm_scaled_ws_bytes(int64_t M, int64_t N, int64_t K, int transpose_A, int transpose_B) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const int s = slice_count(M, N, K, transpose_A, transpose_B);
    return s > 1 ? (size_t)s * (size_t)M * (size_t)N * 4 : 0;
}

extern "C" int seraph_gemm_scaled(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                                  int transpose_A, int transpose_B, int accumulate, float alpha,
                                  void* ws, size_t ws_bytes, seraph_stream_t s) {
    if (M == 0 || N == 0) return SERAPH_OK;
    SERAPH_REQUIRE(A && B && C, "gemm_scaled: NULL pointer");
    SERAPH_REQUIRE(M > 0 && N > 0 && K >= 0, "gemm_scaled: bad shape %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
    const int64_t lda = transpose_A ? M : K, ldb = transpose_B ? K : N;
    const bool vec = (lda % 4 == 0) && (ldb % 4 == 0) && aligned16(A) && aligned16(B);
    const int slices = vec ? slice_count(M, N, K, transpose_A, transpose_B) : 1;
    hipStream_t st = as_stream(s);
    if (slices > 1 && ws && aligned16(ws) && ws_bytes >= (size_t)slices * (size_t)M * (size_t)N * 4) {
        const int64_t nbm = ceil_div(M, 32), nbn = ceil_div(N, 32);
        const dim3 grid((unsigned)(nbm * nbn), (unsigned)slices), block(kGemmThreads);
        float* part = (float*)ws;
#define GOSK(AKC, BKC) \
    hipLaunchKernelGGL((gemm_f32_mfma_splitk_kernel<AKC, BKC>), grid, block, 0, st, A, B, C, M, N, K, 0, (int)nbm, (int)nbn, slices, part)
        if (!transpose_A && !transpose_B) GOSK(true, false);
        else if (!transpose_A && transpose_B) GOSK(true, true);
        else if (transpose_A && !transpose_B) GOSK(false, false);
        else GOSK(false, true);
#undef GOSK
        SERAPH_LAUNCH_CHECK();
        const int64_t n = M * N;
        hipLaunchKernelGGL(gemm_slices_sum_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, st, part, C, n, slices, alpha, accumulate);
        SERAPH_LAUNCH_CHECK();
        return SERAPH_OK;
    }
    // one pass; a scale that cannot be folded in follows as its own sweep
    SERAPH_REQUIRE(!accumulate || alpha == 1.0f, "gemm_scaled: scratch of %zu bytes needed to accumulate a scaled product of this shape",
                   seraph_gemm_scaled_ws_bytes(M, N, K, transpose_A, transpose_B));
    int rc = seraph_gemm(A, B, C, M, N, K, transpose_A, transpose_B, accumulate, s);
    if (rc != SERAPH_OK || alpha == 1.0f) return rc;
    return seraph_scale(C, (size_t)(M * N), alpha, s);
}

// ---------------------------------------------------------------------------------------------
// Several seraph_gemm_scaled products that share the orientations, alpha and the accumulate flag: one pair of launches
// when every product is cut into runs of K, one launch when every product has the same rank-sized K, else one call each.
static int scaled_group_kind(const seraph_gemm_scaled_problem_t* p, int count, int tA, int tB, float alpha, int* slices, size_t* need) {
    if (count < 2 || count > kMaxGroup) return 0;
    bool runs = true, small = alpha == 1.0f;
    size_t bytes = 0;
    for (int i = 0; i < count; i++) {
        const int64_t M = p[i].M, N = p[i].N, K = p[i].K, lda = tA ? M : K, ldb = tB ? K : N;
        if (M <= 0 || N <= 0 || K <= 0 || !p[i].A || !p[i].B || !p[i].C) return 0;
        const bool vec = lda % 4 == 0 && ldb % 4 == 0 && aligned16(p[i].A) && aligned16(p[i].B);
        slices[i] = vec ? slice_count(M, N, K, tA, tB) : 1;
        runs = runs && slices[i] > 1 && ceil_div(M, 32) * ceil_div(N, 32) * slices[i] < (1 << 24);
        small = small && use_smallk(p[i].A, p[i].B, p[i].C, M, N, K, tA, tB) && K == p[0].K && ceil_div(N, 256) < (1 << 24);
        bytes += (((size_t)slices[i] * (size_t)M * (size_t)N + 3) & ~(size_t)3) * 4;     // every product's runs start on a 16-byte boundary
    }
    *need = runs ? bytes : 0;
    return runs ? 1 : small ? 2 : 0;
}

extern "C" size_t seraph_gemm_scaled_grouped_ws_bytes(const seraph_gemm_scaled_problem_t* problems, int count,
                                                      int transpose_A, int transpose_B) {
    if (!problems || count <= 0) return 0;
    int slices[kMaxGroup];
    size_t need = 0;
    if (scaled_group_kind(problems, count, transpose_A, transpose_B, 0.5f, slices, &need) == 1) return need;
    for (int i = 0; i < count; i++) {                      // run one by one: the largest single requirement
        const size_t one = seraph_gemm_scaled_ws_bytes(problems[i].M, problems[i].N, problems[i].K, transpose_A, transpose_B);
        if (one > need) need = one;
    }
    return need;
}

extern "C" int seraph_gemm_scaled_grouped(const seraph_gemm_scaled_problem_t* problems, int count, int transpose_A, int transpose_B,
                                          int accumulate, float alpha, void* ws, size_t ws_bytes, seraph_stream_t s) {
    if (count <= 0) return SERAPH_OK;
    SERAPH_REQUIRE(problems, "gemm_scaled_grouped: NULL problem list");
    int slices[kMaxGroup];
    size_t need = 0;
    int kind = scaled_group_kind(problems, count, transpose_A, transpose_B, alpha, slices, &need);
    if (kind == 1 && (!ws || !aligned16(ws) || ws_bytes < need)) kind = 0;
    hipStream_t st = as_stream(s);
    if (kind == 0) {                                       // exactly as the single calls
        for (int i = 0; i < count; i++) {
            int rc = seraph_gemm_scaled(problems[i].A, problems[i].B, problems[i].C, problems[i].M, problems[i].N, problems[i].K,
                                        transpose_A, transpose_B, accumulate, alpha, ws, ws_bytes, s);
            if (rc != SERAPH_OK) return rc;
        }
        return SERAPH_OK;
    }
    GemmRuns g;
    g.count = count;
    if (kind == 1) {
        float* part = (float*)ws;
        int total = 0;
        for (int i = 0; i < kMaxGroup; i++) {
            const int j = i < count ? i : count - 1;
            g.A[i] = problems[j].A; g.B[i] = problems[j].B; g.C[i] = problems[j].C;
            g.M[i] = problems[j].M; g.N[i] = problems[j].N; g.K[i] = problems[j].K;
            g.nbn[i] = (int)ceil_div(g.N[i], 32); g.tiles[i] = (int)(ceil_div(g.M[i], 32) * ceil_div(g.N[i], 32)); g.slices[i] = slices[j];
            g.first[i] = total;
            if (i < count) {
                g.part[i] = part;
                part += ((size_t)slices[i] * (size_t)g.M[i] * (size_t)g.N[i] + 3) & ~(size_t)3;
                total += g.tiles[i] * g.slices[i];
            } else {
                g.part[i] = g.part[count - 1];
            }
        }
        g.first[kMaxGroup] = total;
        for (int i = count; i <= kMaxGroup; i++) g.first[i] = total;
        const dim3 grid((unsigned)total), block(kGemmThreads);
        const int form = (transpose_A ? 2 : 0) + (transpose_B ? 1 : 0);
        switch (form) {
            case 0: hipLaunchKernelGGL((gemm_f32_mfma_splitk_runs_grouped_kernel<true, false>), grid, block, 0, st, g); break;
            case 1: hipLaunchKernelGGL((gemm_f32_mfma_splitk_runs_grouped_kernel<true, true>), grid, block, 0, st, g); break;
            case 2: hipLaunchKernelGGL((gemm_f32_mfma_splitk_runs_grouped_kernel<false, false>), grid, block, 0, st, g); break;
            default: hipLaunchKernelGGL((gemm_f32_mfma_splitk_runs_grouped_kernel<false, true>), grid, block, 0, st, g); break;
        }
        SERAPH_LAUNCH_CHECK();
        int blocks = 0;
        for (int i = 0; i < count; i++) { g.first[i] = blocks; blocks += (int)ceil_div(g.M[i] * g.N[i], 256); }
        for (int i = count; i <= kMaxGroup; i++) g.first[i] = blocks;
        hipLaunchKernelGGL(gemm_slices_sum_grouped_kernel, dim3((unsigned)blocks), dim3(256), 0, st, g, alpha, accumulate);
        SERAPH_LAUNCH_CHECK();
        return SERAPH_OK;
    }
    // rank-sized K: the column blocks of all products side by side
    const int rows_per_wave = 8;
    int blocks = 0;
    int64_t max_m = 0;
    for (int i = 0; i < kMaxGroup; i++) {
        const int j = i < count ? i : count - 1;
        g.A[i] = problems[j].A; g.B[i] = problems[j].B; g.C[i] = problems[j].C; g.part[i] = nullptr;
        g.M[i] = problems[j].M; g.N[i] = problems[j].N; g.K[i] = problems[j].K;
        g.nbn[i] = 0; g.tiles[i] = 0; g.slices[i] = 1;
        g.first[i] = blocks;
        if (i < count) { blocks += (int)ceil_div(g.N[i], 256); if (g.M[i] > max_m) max_m = g.M[i]; }
    }
    for (int i = count; i <= kMaxGroup; i++) g.first[i] = blocks;
    const dim3 grid((unsigned)blocks, (unsigned)ceil_div(max_m, 4 * rows_per_wave));
    SERAPH_REQUIRE(grid.y <= 65535u * 1024u, "gemm_scaled_grouped: too many rows");
    switch (problems[0].K / 4) {
#define GOK(K4) case K4: hipLaunchKernelGGL(gemm_smallk_grouped_kernel<K4>, grid, dim3(256), 0, st, g, accumulate, rows_per_wave); break;
        GOK(1) GOK(2) GOK(3) GOK(4) GOK(5) GOK(6) GOK(7) GOK(8)
#undef GOK
    }
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}
