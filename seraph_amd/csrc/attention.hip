// attention.hip - causal, grouped-query, packed-sequence attention on the FP32 matrix
// cores: forward (with log-sum-exp) and a deterministic backward.
//
// Mathematics (shaders/batch_attention_backward.comp:50-196, ..._stream.comp:34-202):
//   S = scale Q K^T (causal, block-diagonal over packed sequences), P = softmax(S),
//   dV = P^T dO, dP = dO V^T, dS = P (dP - rowsum(P dP)), dQ = scale dS K, dK = scale dS^T Q.
// rowsum(P dP) equals rowsum(dO O), so the backward takes the forward's O and LSE (saved
// by the caller, or recomputed here) and never rebuilds the softmax statistics.
//
// All matrix products run on v_mfma_f32_32x32x2_f32.  Tiles sit in LDS as [row][D+4] in
// their memory orientation and nothing is ever transposed through LDS: the accumulator
// layout of the instruction (lane = column, registers = rows 8(v/4)+4(l/32)+v%4) is
// exactly the operand layout of the next product when that product contracts over the
// accumulator's row index, because both half-waves may supply any k as long as the two
// operands agree.  Hence
//   forward :  S^T = K Q^T  (lane = query)  ->  O^T += V^T P^T   (P straight from registers)
//   dK/dV   :  S = Q K^T    (lane = key)    ->  dV += P^T dO, dK += dS^T Q
//   dQ      :  S^T = K Q^T  (lane = query)  ->  dQ += dS K
// The softmax statistics of a query are therefore per-lane scalars in the forward and dQ
// kernels, and per-register values (read from LDS) in the dK/dV kernel.
//
// No atomics: one workgroup owns a key/value tile (for all query heads of its group) or a
// query tile, so every output element is written by exactly one lane in a fixed order.
// The price is that S and dP are formed twice (7 products instead of 5).
//
// Packed sequences: each lane looks up the start of its token's sequence once (binary
// search over the batch+1 offsets); a score (i, j) is kept when start[i] <= j <= i.  Tiles are anchored on the global token
// axis at multiples of 32/128, so ragged sequence lengths need no padding.
#include <limits.h>
#include <type_traits>
#include <algorithm>
#include <atomic>
#include <mutex>

#include "common.hpp"

namespace seraph {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kAttnThreads = 256;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ v16f mfma(float a, float b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
// row index inside a 32x32 accumulator block held by register v of a lane in half-wave h
__device__ __forceinline__ int acc_row(int v, int h) { return 8 * (v >> 2) + 4 * h + (v & 3); }

// The products that contract over the accumulator's row index take their other operand from a
// tile row in LDS, one value per (lane, 32-wide block of head_dim).  Lane r of block db is given
// feature d = DB*r + db (DB = head_dim/32) instead of db*32 + r, so the DB values a lane needs sit
// next to each other and arrive with one 4/8/16-byte LDS read that feeds DB MFMAs; results are
// written back with the same mapping, which also makes the final global accesses DB floats wide.
template <int DB> struct DVec { float v[DB]; };
template <int DB>
__device__ __forceinline__ DVec<DB> lds_dvec(const float* row, int r) {
    DVec<DB> o;
    if (DB == 4) { const float4 t = *reinterpret_cast<const float4*>(row + 4 * r); o.v[0] = t.x; o.v[1] = t.y; o.v[2 % DB] = t.z; o.v[3 % DB] = t.w; }
    else if (DB == 2) { const float2 t = *reinterpret_cast<const float2*>(row + 2 * r); o.v[0] = t.x; o.v[1 % DB] = t.y; }
    else { o.v[0] = row[r]; }
    return o;
}

// ---------------------------------------------------------------- packed-sequence offsets
// Every workgroup copies the batch+1 prefix offsets into LDS once (up to kMaxSeqLds of
// them; larger batches are searched in global memory) and binary-searches them there:
// a lookup costs a few LDS round trips instead of a chain of dependent global loads.
constexpr int kMaxSeqLds = 1024;

struct SeqTable {
    const uint32_t* g;     // global offsets (NULL = one sequence of T tokens)
    const uint32_t* s;     // LDS copy or NULL
    int batch;
    int T;
    __device__ __forceinline__ int find(int t) const {
        const uint32_t* p = s ? s : g;
        int lo = 0, hi = batch;
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if ((int)p[mid + 1] <= t) lo = mid + 1; else hi = mid;
        }
        return lo;
    }
    __device__ __forceinline__ int start_of(int t) const { return g ? (int)(s ? s : g)[find(t)] : 0; }
    __device__ __forceinline__ int end_of(int t) const {
        if (!g) return T;
        int e = (int)(s ? s : g)[find(t) + 1];
        return e < T ? e : T;
    }
};

// Call from all lanes of the workgroup, before any lookup; contains a barrier.
__device__ __forceinline__ SeqTable load_seq_table(const uint32_t* __restrict__ seq_starts, int batch, int T,
                                                   uint32_t* __restrict__ lds) {
    SeqTable st;
    st.g = seq_starts; st.s = nullptr; st.batch = batch; st.T = T;
    if (seq_starts && batch + 1 <= kMaxSeqLds) {
        for (int i = threadIdx.x; i <= batch; i += (int)blockDim.x) lds[i] = seq_starts[i];
        st.s = lds;
    }
    __syncthreads();
    return st;
}

// ---------------------------------------------------------------- dynamic tile queue
// Causal attention tiles differ in cost by up to two orders of magnitude, and the hardware
// deals workgroups to CUs in a fixed rotation, so a one-tile-per-workgroup launch leaves half of
// the machine idle behind the CUs that drew the long tiles.  The kernels are therefore
// persistent: a resident set of workgroups pulls tile indices, longest first, from a device
// counter until it runs dry.  Every workgroup makes exactly one failing pull and then leaves, so
// the grid always drains; the last one out rewinds the counter pair for the next launch.
// Counters come from a fixed pool in device memory (zero at module load), one pair per launch in
// rotation, so launches on different streams do not share a pair.
constexpr int kQueueSlots = 1024;
static __device__ unsigned int g_tile_queues[2 * kQueueSlots];

struct TileQueue {
    unsigned int* q;        // q[0] next item, q[1] workgroups finished
    int* slot;              // one int of LDS
    int total;
    int extra = 0;          // workgroups at the end of the grid that do other work and never draw
    int drawn = 0;
    // A launch with no more workgroups than items' worth of residency gets exactly one workgroup per item
    // (persistent_grid): the item is then the workgroup's index and the counters stay untouched, which
    // saves the two round trips of the atomics, the whole cost of the queue for a short item.
    __device__ __forceinline__ bool one_each() const { return total <= (int)gridDim.x - extra; }
    __device__ __forceinline__ int next() {
        if (one_each()) {
            const int item = drawn ? -1 : (int)blockIdx.x;
            drawn = 1;
            return item < total ? item : -1;
        }
        if (threadIdx.x == 0) *slot = (int)atomicAdd(&q[0], 1u);
        __syncthreads();
        const int item = __builtin_amdgcn_readfirstlane(*slot);    // the same for every lane: keep it, and what follows from it, scalar
        __syncthreads();
        return item < total ? item : -1;
    }
    __device__ __forceinline__ void leave() const {
        if (one_each()) return;
        if (threadIdx.x == 0 && atomicAdd(&q[1], 1u) == gridDim.x - (unsigned)extra - 1) {
            q[0] = 0u;
            q[1] = 0u;
            __threadfence();
        }
    }
};

// Longest tiles first.  Within one sequence the tile index already orders the work, but a packed batch
// repeats the long-to-short ramp once per sequence, and the long tiles of the last sequence would
// start late and finish alone.  Every workgroup therefore ranks the tiles by their length (number of
// 32-wide tiles on the other axis) once, in LDS, and maps queue position -> tile through that ranking.
// All workgroups compute the same permutation.  Very many tiles (more than kMaxOrder) or very few (where
// the ranking costs more than it saves) keep the natural order of one sequence: ascending for key tiles,
// descending for query tiles.
constexpr int kMaxOrder = 1024;
constexpr int kMinOrder = 32;
struct TileOrder {
    const int* order;      // LDS, or NULL = natural order
    int n;
    bool descending;
    __device__ __forceinline__ int operator()(int rank) const {   // rank is uniform, and so is the answer
        return order ? __builtin_amdgcn_readfirstlane(order[rank]) : (descending ? n - 1 - rank : rank);
    }
};
template <typename LenFn>
__device__ __forceinline__ TileOrder rank_tiles_by_length(int* lens, int* order, int n, bool descending, bool all_at_once, LenFn len) {
    TileOrder t{nullptr, n, descending};
    if (n > kMaxOrder || n < kMinOrder || all_at_once) return t;       // every item starts at once: any order will do
    for (int i = threadIdx.x; i < n; i += (int)blockDim.x) lens[i] = len(i);
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += (int)blockDim.x) {
        const int me = lens[i];
        int rank = 0;
        for (int j = 0; j < n; j++) {
            const int o = lens[j];
            rank += (o > me) || (o == me && j < i);
        }
        order[rank] = i;
    }
    __syncthreads();
    t.order = order;
    return t;
}

// ---------------------------------------------------------------- tile staging (32 rows x D)
template <int D>
struct Tile32 {
    static constexpr int LD = D + 4;
    static constexpr int kSlots = 32 * D / 4 / kAttnThreads;
    float4 r[kSlots];
    // rows row0..row0+31 of a token-major matrix with `stride` floats per token, columns col0..col0+D-1.
    // One buffer descriptor per tile (scalar registers): origin at the tile's first element, extent up to
    // the end of token T-1, so rows past the end read as zeros without a per-lane predicate, and the
    // per-lane part of the address is a 32-bit offset that needs no 64-bit arithmetic.
    __device__ __forceinline__ void gload(const float* __restrict__ base, int64_t row0, int64_t T, int64_t stride, int col0) {
        const float* origin = base + row0 * stride + col0;
        const int64_t left = T - row0;
        int64_t bytes = left > 0 ? left * stride * 4 - (int64_t)col0 * 4 : 0;
        if (bytes > 0xffffffffLL) bytes = 0xffffffffLL;
        const uint64_t o = reinterpret_cast<uint64_t>(origin);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)o), hi = __builtin_amdgcn_readfirstlane((uint32_t)(o >> 32));
        const uint32_t nb = __builtin_amdgcn_readfirstlane((uint32_t)bytes);
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0, (int)nb, 0x00020000);
        const int st4 = (int)stride * 4;
#pragma unroll
        for (int u = 0; u < kSlots; u++) {
            const int f = threadIdx.x + kAttnThreads * u;
            const int off = (f / (D / 4)) * st4 + 16 * (f % (D / 4));
            r[u] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0));
        }
    }
    __device__ __forceinline__ void sstore(float* __restrict__ lds) const {
#pragma unroll
        for (int u = 0; u < kSlots; u++) {
            const int f = threadIdx.x + kAttnThreads * u;
            *reinterpret_cast<float4*>(lds + (f / (D / 4)) * LD + 4 * (f % (D / 4))) = r[u];
        }
    }
};

// ---------------------------------------------------------------- forward
// grid (query tiles of 128, heads); wave w owns queries i0+32w .. +31; key/value tiles of 32.
// KSPLIT (a short batch: fewer 128-query tiles than the chip has room for, and the longest one alone sets the
// time): a work item is 64 queries; waves 0,1 take them against the even key tiles, waves 2,3 the same queries
// against the odd ones - two key tiles are staged per iteration - and the two softmax states (m, l, O) of a
// query are merged through LDS at the end, in a fixed order.
template <int D, bool KSPLIT>
__global__ __launch_bounds__(kAttnThreads, (KSPLIT ? 1 : 2)) void attn_fwd_kernel(const float* __restrict__ Q, const float* __restrict__ K,
                                                                const float* __restrict__ V, float* __restrict__ O,
                                                                float* __restrict__ LSE, const uint32_t* __restrict__ seq_starts, int batch,
                                                                int64_t T, int H, int KVH, float scale_log2e,
                                                                unsigned int* __restrict__ queue) {
    constexpr int LD = D + 4, DB = D / 32;
    constexpr int KT = KSPLIT ? 2 : 1, QROWS = KSPLIT ? 64 : 128;     // key tiles staged per iteration, queries per item
    __shared__ __attribute__((aligned(16))) float sK[2][KT * 32 * LD];
    __shared__ __attribute__((aligned(16))) float sV[2][KT * 32 * LD];
    __shared__ uint32_t sSeq[kMaxSeqLds];
    __shared__ int sItem;
    const SeqTable seqs = load_seq_table(seq_starts, batch, (int)T, sSeq);
    const int nqt = (int)((T + QROWS - 1) / QROWS);
    TileQueue tq_{queue, &sItem, nqt * H};
    __shared__ int sLen[kMaxOrder], sOrd[kMaxOrder];
    // key tiles a query tile runs over: from the start of its first query's sequence to its last query
    const TileOrder by_len = rank_tiles_by_length(sLen, sOrd, nqt, true, tq_.one_each(), [&](int q) {
        const int64_t a = (int64_t)q * QROWS, z = (a + QROWS - 1 < T - 1) ? a + QROWS - 1 : T - 1;
        return (int)((z + 1 - (seqs.start_of((int)a) / 32) * 32 + 31) / 32);
    });
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
    const int wq = KSPLIT ? (w & 1) : w, kp = KSPLIT ? (w >> 1) : 0;  // the wave's 32 queries within the item; its key-tile parity
    for (int item = tq_.next(); item >= 0; item = tq_.next()) {
    const int head = item % H, kvh = head / (H / KVH);
    const int qt = by_len(item / H);                           // long rows first
    const int64_t i0 = (int64_t)qt * QROWS;
    const int64_t iw0 = i0 + 32 * wq, i_lane = iw0 + r;
    const bool row_ok = i_lane < T;
    const int ss_lane = row_ok ? seqs.start_of((int)i_lane) : INT_MAX;
    const int64_t qw = (int64_t)H * D, kw = (int64_t)KVH * D;

    float4 qf[D / 8];
#pragma unroll
    for (int s8 = 0; s8 < D / 8; s8++)
        qf[s8] = row_ok ? *reinterpret_cast<const float4*>(Q + i_lane * qw + head * D + s8 * 8 + 4 * h) : make_float4(0.f, 0.f, 0.f, 0.f);

    const int64_t i_last = (i0 + QROWS - 1 < T - 1) ? i0 + QROWS - 1 : T - 1;
    const int64_t jbeg = (seqs.start_of((int)i0) / 32) * 32;
    const int ntiles = (int)((i_last + 1 - jbeg + 31) / 32);

    float m = -INFINITY, l = 0.0f;
    v16f o[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[db][v] = 0.0f;

    Tile32<D> tk[KT], tv[KT];
    auto kv_load = [&](int t0) {                               // tiles t0 .. t0+KT-1; rows past the last token read as zeros
#pragma unroll
        for (int u = 0; u < KT; u++) {
            tk[u].gload(K, jbeg + 32 * (int64_t)(t0 + u), T, kw, kvh * D);
            tv[u].gload(V, jbeg + 32 * (int64_t)(t0 + u), T, kw, kvh * D);
        }
    };
    auto kv_store = [&](int buf) {
#pragma unroll
        for (int u = 0; u < KT; u++) { tk[u].sstore(sK[buf] + u * 32 * LD); tv[u].sstore(sV[buf] + u * 32 * LD); }
    };
    kv_load(0);
    kv_store(0);
    __syncthreads();

    for (int tp = 0; tp < ntiles; tp += KT) {
        const int cur = (tp / KT) & 1;
        const int t = tp + kp;                                   // this wave's tile of the staged ones
        const int64_t j0 = jbeg + 32 * (int64_t)t;
        const float* sKt = sK[cur] + kp * 32 * LD;
        const float* sVt = sV[cur] + kp * 32 * LD;
        if (tp + KT < ntiles) kv_load(tp + KT);
        if (t < ntiles && j0 <= iw0 + 31 && iw0 < T) {          // some query of this wave can see this tile
            v16f s;
#pragma unroll
            for (int v = 0; v < 16; v++) s[v] = 0.0f;
            // LDS operands are fetched one step ahead of the MFMAs that consume them
            float4 kb[2];
            kb[0] = *reinterpret_cast<const float4*>(&sKt[r * LD + 4 * h]);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
            for (int s8 = 0; s8 < D / 8; s8++) {
                if (s8 + 1 < D / 8) kb[(s8 + 1) & 1] = *reinterpret_cast<const float4*>(&sKt[r * LD + (s8 + 1) * 8 + 4 * h]);
                const float4 a = kb[s8 & 1];
                s = mfma(a.x, qf[s8].x, s); s = mfma(a.y, qf[s8].y, s);
                s = mfma(a.z, qf[s8].z, s); s = mfma(a.w, qf[s8].w, s);
                if (s8 + 1 < D / 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
            }
            // The softmax between the two runs of matrix instructions is this wave's only stretch of plain vector
            // work; beside a wave of the co-resident workgroup that always has a matrix instruction ready it is
            // served slowly.  Raised priority for just this stretch lets it through (the neighbour's matrix
            // instructions have 64 cycles of slack each): forward 207 -> 200 us at 8 x 1024 tokens, 16 heads of 64.
            __builtin_amdgcn_s_setprio(3);
            float mloc = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int j = (int)j0 + acc_row(v, h);
                const bool valid = (j >= ss_lane) && (j <= (int)i_lane);
                s[v] = valid ? s[v] * scale_log2e : -INFINITY;
                mloc = fmaxf(mloc, s[v]);
            }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
            // Lazy rescaling: the running maximum is only advanced (and O, l rescaled) when some
            // query of the wave has outgrown it by more than 2^8; until then probabilities are formed
            // against the slightly stale maximum, which is exact after the final division by l.
            const float mnew = fmaxf(m, mloc);
            if (__any(mnew > m + 8.0f)) {
                const float alpha = fast_exp2(m - (mnew == -INFINITY ? 0.0f : mnew));
                l *= alpha;
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int v = 0; v < 16; v++) o[db][v] *= alpha;
                m = mnew;
            }
            const float msafe = m == -INFINITY ? 0.0f : m;
            float lsum = 0.0f;
#pragma unroll
            for (int v = 0; v < 16; v++) { s[v] = fast_exp2(s[v] - msafe); lsum += s[v]; }
            lsum += __shfl_xor(lsum, 32, 64);
            l += lsum;
            __builtin_amdgcn_s_setprio(0);
            DVec<DB> vb[2];
            vb[0] = lds_dvec<DB>(&sVt[acc_row(0, h) * LD], r);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                if (v + 1 < 16) vb[(v + 1) & 1] = lds_dvec<DB>(&sVt[acc_row(v + 1, h) * LD], r);
#pragma unroll
                for (int db = 0; db < DB; db++) o[db] = mfma(vb[v & 1].v[db], s[v], o[db]);
                if (v + 1 < 16) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, DB, 0);
            }
        }
        if (tp + KT < ntiles) kv_store(cur ^ 1);
        __syncthreads();
    }

    if (KSPLIT) {
        // Waves 2,3 hand their state to waves 0,1 (same queries, same register layout) through the tile buffers,
        // which nobody reads any more; the next item restages them only behind the queue's barriers.
        float* xo = &sK[0][0];                                  // [wave pair][DB * 16 + 2][64 lanes]
        static_assert(!KSPLIT || 2 * KT * 32 * LD >= 2 * (DB * 16 + 2) * 64, "tile buffers too small for the exchange");
        float* mine = xo + (size_t)wq * (DB * 16 + 2) * 64;
        if (kp == 1) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) mine[(db * 16 + v) * 64 + lane] = o[db][v];
            mine[(DB * 16) * 64 + lane] = m;
            mine[(DB * 16 + 1) * 64 + lane] = l;
        }
        __syncthreads();
        if (kp == 0) {
            const float m2 = mine[(DB * 16) * 64 + lane], l2 = mine[(DB * 16 + 1) * 64 + lane];
            const float mm = fmaxf(m, m2);
            const float ref = mm == -INFINITY ? 0.0f : mm;       // both empty: every factor below is exp2(-inf) = 0
            const float f1 = fast_exp2(m - ref), f2 = fast_exp2(m2 - ref);
            l = l * f1 + l2 * f2;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) o[db][v] = o[db][v] * f1 + mine[(db * 16 + v) * 64 + lane] * f2;
            m = mm;
        }
    }

    if (row_ok && kp == 0) {
        const float inv = 1.0f / l;
        // accumulator row a of block db is feature DB*a + db: registers 4g..4g+3 of all blocks are
        // 4*DB consecutive features starting at DB*(8g + 4h)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            float* dst = O + i_lane * qw + head * D + DB * (8 * g + 4 * h);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (DB == 4) *reinterpret_cast<float4*>(dst + 4 * e) = make_float4(o[0][4 * g + e] * inv, o[1 % DB][4 * g + e] * inv, o[2 % DB][4 * g + e] * inv, o[3 % DB][4 * g + e] * inv);
                else if (DB == 2) *reinterpret_cast<float2*>(dst + 2 * e) = make_float2(o[0][4 * g + e] * inv, o[1 % DB][4 * g + e] * inv);
                else dst[e] = o[0][4 * g + e] * inv;
            }
        }
        if (LSE && h == 0) LSE[i_lane * H + head] = (m + __log2f(l)) * kLn2;
    }
    }   // tile queue
    tq_.leave();
}

// ---------------------------------------------------------------- delta = rowsum(dO * O)
// one wave per token; a head's D values are spread over D/4 consecutive lanes.  The wave also looks up the first
// token of its token's sequence once, so the dK/dV kernel reads it like any other row statistic instead of
// walking the offsets table for every (key tile, head) it visits the row for.
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const float* __restrict__ dO, const float* __restrict__ O,
                                                         float* __restrict__ delta, int64_t T, int H,
                                                         const uint32_t* __restrict__ seq_starts, int batch, int* __restrict__ row_start,
                                                         int ds_slots, int epoch, int* __restrict__ band_overflow,
                                                         unsigned int* __restrict__ queue_a, unsigned int* __restrict__ queue_b) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    // The two persistent kernels that follow on this stream start from counter pairs this launch has zeroed:
    // a pair left non-zero by a launch that never finished cannot make them skip tiles.
    if (blockIdx.x == 0 && threadIdx.x < 4) (threadIdx.x < 2 ? queue_a : queue_b)[threadIdx.x & 1] = 0u;
    if (t >= T) return;
    if (lane == 0) {
        int start = 0;
        if (seq_starts) {
            int lo = 0, hi = batch;                            // last sequence whose start is <= t
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if ((int64_t)seq_starts[mid + 1] <= t) lo = mid + 1; else hi = mid;
            }
            start = (int)seq_starts[lo];
        }
        row_start[t] = start;
        // A query whose sequence starts more key tiles back than the dS band holds (the caller's bound on the
        // sequence length was too small): the launch is marked, the banded dQ kernel stands down and the
        // recomputing one runs instead.  Every marking lane stores the same value.
        if (ds_slots > 0 && (int)(t >> 5) - (start >> 5) >= ds_slots) *band_overflow = epoch;
    }
    const int64_t qw = (int64_t)H * D;
    constexpr int LPH = D / 4;                                  // lanes per head
    for (int64_t c = lane * 4; c < qw; c += 256) {
        const float4 a = *reinterpret_cast<const float4*>(dO + t * qw + c);
        const float4 b = *reinterpret_cast<const float4*>(O + t * qw + c);
        float s = a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
#pragma unroll
        for (int o = LPH / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if ((lane % LPH) == 0) delta[t * H + c / D] = s;
    }
}

// ---------------------------------------------------------------- backward: dK, dV
// grid (key tiles of 128, kv heads); wave w owns keys j0+32w .. +31 for every query head of the group.
template <int D, bool WRITE_DS>
__global__ __launch_bounds__(kAttnThreads, 1) void attn_bwd_dkv_kernel(const float* __restrict__ Q, const float* __restrict__ K,
                                                                    const float* __restrict__ V, const float* __restrict__ dO,
                                                                    const float* __restrict__ LSE, const float* __restrict__ DELTA,
                                                                    const int* __restrict__ ROWSTART,
                                                                    float* __restrict__ dK, float* __restrict__ dV,
                                                                    const uint32_t* __restrict__ seq_starts, int batch,
                                                                    int64_t T, int H, int KVH, float scale, float scale_log2e,
                                                                    unsigned int* __restrict__ queue,
                                                                    float* __restrict__ DS, int ds_slots,
                                                                    int split, float* __restrict__ partK, float* __restrict__ partV,
                                                                    int assign) {
    constexpr int LD = D + 4, DB = D / 32;
    // Query rows per iteration: two 32-row sub-tiles up to head_dim 64, so that one staging phase and
    // one barrier serve 256 matrix instructions per wave, as one 32-row tile does at head_dim 128.
    constexpr int QB = D <= 64 ? 2 : 1, QR = 32 * QB;
    __shared__ __attribute__((aligned(16))) float sQ[2][QR * LD];
    __shared__ __attribute__((aligned(16))) float sG[2][QR * LD];     // dO
    // Row statistics of the staged queries.  Every lane of the workgroup stores (lanes past the QR rows into a
    // dummy tail), which keeps the pipelined iterations free of branches: one scheduling region.
    constexpr int SR = kAttnThreads;
    __shared__ __attribute__((aligned(16))) float sLse[2][SR];
    __shared__ __attribute__((aligned(16))) float sDel[2][SR];
    __shared__ __attribute__((aligned(16))) int sSS[2][SR];
    __shared__ uint32_t sSeq[kMaxSeqLds];
    __shared__ int sItem;
    const SeqTable seqs = load_seq_table(seq_starts, batch, (int)T, sSeq);
    const int G = H / KVH;
    // With few key tiles (short batches) the longest item, the first key tile of a sequence looping over
    // every query tile of every head of its group, is the critical path.  `split` > 1 deals the
    // iterations of each (key tile, kv head) round-robin to that many work items; each writes its partial
    // dK/dV to its own slice of partK/partV and a second kernel adds the slices in a fixed order.
    const int nkt = (int)((T + 127) / 128);
    TileQueue tq_{queue, &sItem, nkt * KVH * split};
    __shared__ int sLen[kMaxOrder], sOrd[kMaxOrder];
    // query tiles a 128-key tile is visible to: up to the end of its last key's sequence
    const TileOrder by_len = rank_tiles_by_length(sLen, sOrd, nkt, false, tq_.one_each(), [&](int k) {
        const int64_t a = (int64_t)k * 128, z = (a + 127 < T - 1) ? a + 127 : T - 1;
        return (int)((seqs.end_of((int)z) - a + 31) / 32);
    });
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
    for (int item = tq_.next(); item >= 0; item = tq_.next()) {
    const int sub = item % split;
    const int kvh = (item / split) % KVH;
    const int64_t j0 = (int64_t)by_len(item / split / KVH) * 128;    // long key tiles (early keys of a sequence) first
    const int64_t jw0 = j0 + 32 * w, j_lane = jw0 + r;
    const bool col_ok = j_lane < T;
    const int64_t qw = (int64_t)H * D, kw = (int64_t)KVH * D;

    // This wave's 32 keys as B operands (lane = key, k = d).  K always lives in registers; V
    // does too for head_dim <= 64, but at 128 the two fragments plus the dK/dV accumulators
    // exceed the register file, so V for the workgroup's 128 keys is parked in LDS instead.
    constexpr bool kVinLds = D >= 64;
    __shared__ __attribute__((aligned(16))) float sVt[kVinLds ? 128 * LD : 4];
    float4 kf[D / 8], vf[kVinLds ? 1 : D / 8];
#pragma unroll
    for (int s8 = 0; s8 < D / 8; s8++) {
        kf[s8] = col_ok ? *reinterpret_cast<const float4*>(K + j_lane * kw + kvh * D + s8 * 8 + 4 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
        if (!kVinLds)
            vf[s8] = col_ok ? *reinterpret_cast<const float4*>(V + j_lane * kw + kvh * D + s8 * 8 + 4 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    // Every global load of the item's set-up (K, V, the first query tile and its row statistics) is requested
    // before the first result is used, so the set-up costs one memory round trip.
    Tile32<D> tvv[kVinLds ? 4 : 1];
    if (kVinLds) {
#pragma unroll
        for (int q = 0; q < 4; q++) tvv[q].gload(V, j0 + 32 * q, T, kw, kvh * D);
    }
    v16f dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) { dk[db][v] = 0.0f; dv[db][v] = 0.0f; }

    const int64_t j_last = (j0 + 127 < T - 1) ? j0 + 127 : T - 1;
    const int64_t i_end = seqs.end_of((int)j_last);                         // queries of the last key's sequence
    const int nq = (int)((i_end - j0 + QR - 1) / QR);             // iterations per query head
    const int iters = nq * G;

    Tile32<D> tq[QB], tg[QB];
    float st_lse = 0.f, st_del = 0.f;
    int st_ss = INT_MAX;
    // Row statistics (log-sum-exp, delta, first token of the row's sequence) of the staged queries; lanes past the
    // QR rows repeat them.  Iterations are named by (hg, n): query head hg of the kv head's group and the n-th run
    // of QR queries.  Rows past the end are read from the last token and replaced when they are stored.
    bool st_ok = false;
    auto stats_load = [&](int hg, int n) {
        const int head = kvh * G + hg;
        const int64_t i = j0 + QR * (int64_t)n + (threadIdx.x & (QR - 1));
        st_ok = i < T;
        const int64_t ic = st_ok ? i : T - 1;
        if (SR == kAttnThreads || threadIdx.x < QR) {
            st_lse = LSE[ic * H + head];
            st_del = DELTA[ic * H + head];
            st_ss = ROWSTART[ic];
        }
    };
    auto stats_store = [&](int buf) {
        if (SR == kAttnThreads || threadIdx.x < QR) {
            sLse[buf][threadIdx.x] = st_ok ? st_lse * kLog2e : 0.f;
            sDel[buf][threadIdx.x] = st_ok ? st_del : 0.f;
            sSS[buf][threadIdx.x] = st_ok ? st_ss : INT_MAX;
        }
    };
    auto tiles_load = [&](int hg, int n) {
        const int head = kvh * G + hg;
        const int64_t i0 = j0 + QR * (int64_t)n;
#pragma unroll
        for (int qb = 0; qb < QB; qb++) {
            tq[qb].gload(Q, i0 + 32 * qb, T, qw, head * D);
            tg[qb].gload(dO, i0 + 32 * qb, T, qw, head * D);
        }
    };
    auto tiles_store = [&](int buf) {
#pragma unroll
        for (int qb = 0; qb < QB; qb++) { tq[qb].sstore(sQ[buf] + 32 * qb * LD); tg[qb].sstore(sG[buf] + 32 * qb * LD); }
    };

    {
        const int first = sub < iters ? sub : iters - 1;      // an item without iterations still stages a valid tile
        stats_load(first / nq, first % nq); tiles_load(first / nq, first % nq);
    }
#pragma unroll
    for (int s8 = 0; s8 < D / 8; s8++) {   // S comes out in base-2 units
        kf[s8].x *= scale_log2e; kf[s8].y *= scale_log2e; kf[s8].z *= scale_log2e; kf[s8].w *= scale_log2e;
    }
    if (kVinLds) {
#pragma unroll
        for (int q = 0; q < 4; q++) tvv[q].sstore(sVt + q * 32 * LD);
    }
    tiles_store(0); stats_store(0);
    __syncthreads();

    // One iteration = QB 32-query tiles of one query head against the workgroup's 128 keys.  Only the
    // first query tiles of a head (the diagonal) leave some wave without a visible key, so the loop is
    // written twice: with the per-wave test for those, and as straight-line code for the rest, where
    // every wave works.  (A conditional around the accumulating matrix instructions in the main
    // loop makes the compiler shuttle the 128 dK/dV accumulator registers in and out of the
    // accumulation register file on every iteration.)  `iteration` below is the copy with the test; the
    // straight-line iterations run `iteration1` (one sub-tile) or `iteration2` (two), which are pipelined.
    const bool wave_has_keys = jw0 < T;
    auto iteration = [&](int hg, int n, int li, int hg2, int n2) {
        const int cur = li & 1;
        // No branch around the loads and the LDS staging: past the last tile the same tile is simply
        // fetched and staged again.  (Loads and stores share one in-order counter; behind a branch the
        // compiler must wait for everything, including the dS stores, before it may touch the tile.)
        stats_load(hg2, n2);
        tiles_load(hg2, n2);
#pragma unroll
        for (int qb = 0; qb < QB; qb++) {
        const int64_t i0 = j0 + QR * (int64_t)n + 32 * qb;
        const int ro = 32 * qb;                                              // this sub-tile's first row in the staged tiles
        if (i0 + 31 >= jw0 && wave_has_keys) {                               // some query of the tile can see this wave's keys
            v16f s, dp;
#pragma unroll
            for (int v = 0; v < 16; v++) { s[v] = 0.0f; dp[v] = 0.0f; }
            {
                // operands of step s8+1 are requested from LDS before the 8 matrix instructions of step s8
                float4 fa[2], fb[2], fv[2];
                auto fetch = [&](int s8, int buf) {
                    fa[buf] = *reinterpret_cast<const float4*>(&sQ[cur][(ro + r) * LD + s8 * 8 + 4 * h]);
                    fb[buf] = *reinterpret_cast<const float4*>(&sG[cur][(ro + r) * LD + s8 * 8 + 4 * h]);
                    if (kVinLds) fv[buf] = *reinterpret_cast<const float4*>(&sVt[(32 * w + r) * LD + s8 * 8 + 4 * h]);
                };
                fetch(0, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
#pragma unroll
                for (int s8 = 0; s8 < D / 8; s8++) {
                    if (s8 + 1 < D / 8) fetch(s8 + 1, (s8 + 1) & 1);
                    const float4 a = fa[s8 & 1], b = fb[s8 & 1];
                    const float4 vv = kVinLds ? fv[s8 & 1] : vf[kVinLds ? 0 : s8];
                    s = mfma(a.x, kf[s8].x, s); dp = mfma(b.x, vv.x, dp);
                    s = mfma(a.y, kf[s8].y, s); dp = mfma(b.y, vv.y, dp);
                    s = mfma(a.z, kf[s8].z, s); dp = mfma(b.z, vv.z, dp);
                    s = mfma(a.w, kf[s8].w, s); dp = mfma(b.w, vv.w, dp);
                    if (s8 + 1 < D / 8) {
#pragma unroll
                        for (int g = 0; g < 3; g++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 5, 0);
                    } else {
                        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
                    }
                }
            }
            // K was scaled by scale*log2(e) when it was loaded, so s is already the base-2 logit.  A tile whose
            // keys all precede its queries and all lie inside the sequence of its last (hence every) query
            // needs no mask: p = 2^(s - lse) for every element.
            const int ss_last = __builtin_amdgcn_readfirstlane(sSS[cur][ro + 31]);   // INT_MAX if the tile runs past T
            const bool interior = (jw0 + 31 <= i0) && ((int)jw0 >= ss_last);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 lse4 = *reinterpret_cast<const float4*>(&sLse[cur][ro + 8 * g + 4 * h]);
                const float4 del4 = *reinterpret_cast<const float4*>(&sDel[cur][ro + 8 * g + 4 * h]);
                const float* lse_p = &lse4.x; const float* del_p = &del4.x;
                if (interior) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int v = 4 * g + e;
                        const float p = fast_exp2(s[v] - lse_p[e]);
                        s[v] = p;
                        dp[v] = p * (dp[v] - del_p[e]);
                    }
                } else {
                    const int4 ss4 = *reinterpret_cast<const int4*>(&sSS[cur][ro + 8 * g + 4 * h]);
                    const int* ss_p = &ss4.x;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int v = 4 * g + e;
                        const int i = (int)i0 + 8 * g + 4 * h + e;
                        const bool valid = ((int)j_lane <= i) && ((int)j_lane >= ss_p[e]);     // ss = INT_MAX for i >= T
                        const float p = valid ? fast_exp2(s[v] - lse_p[e]) : 0.0f;
                        s[v] = p;
                        dp[v] = p * (dp[v] - del_p[e]);
                    }
                }
            }
            if (WRITE_DS) {
                // dS tile (32 queries x 32 keys, row-major) for the dQ pass: band slot = query tile - key tile.
                // A tile outside the band (it is all zeros: another sequence) goes to a spare tile behind the band.
                const int qt = (int)(i0 >> 5), slot = qt - (int)(jw0 >> 5);
                const int head = kvh * G + hg;
                const int64_t ntile = (int64_t)H * ((T + 31) >> 5) * ds_slots;
                int64_t tidx = (((int64_t)head * ((T + 31) >> 5) + qt) * ds_slots + slot);
                tidx = (slot >= 0 && slot < ds_slots && qt < (int)((T + 31) >> 5)) ? tidx : ntile;
                const uint64_t ta = reinterpret_cast<uint64_t>(DS + (tidx << 10));
                const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)ta), hi = __builtin_amdgcn_readfirstlane((uint32_t)(ta >> 32));
                const __amdgpu_buffer_rsrc_t rs =
                    __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0, 4096, 0x00020000);
                const int lane_off = (4 * h * 32 + r) * 4;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const float val = dp[v];
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), rs, lane_off + (8 * (v >> 2) + (v & 3)) * 128, 0, 0);
                }
            }
            {
                DVec<DB> go[2], qq[2];
                auto fetch = [&](int v, int buf) {
                    go[buf] = lds_dvec<DB>(&sG[cur][(ro + acc_row(v, h)) * LD], r);
                    qq[buf] = lds_dvec<DB>(&sQ[cur][(ro + acc_row(v, h)) * LD], r);
                };
                fetch(0, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    if (v + 1 < 16) fetch(v + 1, (v + 1) & 1);
#pragma unroll
                    for (int db = 0; db < DB; db++) {
                        dv[db] = mfma(s[v], go[v & 1].v[db], dv[db]);
                        dk[db] = mfma(dp[v], qq[v & 1].v[db], dk[db]);
                    }
                    if (v + 1 < 16) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        if (2 * DB - 2 > 0) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);     // one LDS write of the next tile
                            __builtin_amdgcn_sched_group_barrier(0x008, 2 * DB - 3, 0);
                        }
                    } else {
                        __builtin_amdgcn_sched_group_barrier(0x008, 2 * DB, 0);
                    }
                }
            }
        }
        }   // sub-tiles
        tiles_store(cur ^ 1); stats_store(cur ^ 1);
        __syncthreads();
    };
    // The straight-line iteration for one sub-tile (head_dim 128), in four runs of matrix instructions that carry
    // the other work between them (a SIMD runs one wave here, and while a wave's next instruction is a matrix
    // instruction waiting for the pipe nothing else issues): S with the first half of dP, and the next tile's
    // requests; the second half of dP with p = 2^(s - lse); dV = P^T dO with dS = p (dP - delta) and the LDS
    // writes of the next tile; dK = dS^T Q with the dS stores.
    auto iteration1 = [&](int hg, int n, int li, int hg2, int n2) {
        constexpr int NS = D / 8, NH = NS / 2, EPS = 16 / NH;  // S steps, steps per half, exponentials per step
        static_assert(QB == 2 || (NH >= 4 && 16 % NH == 0 && EPS <= 4), "one-sub-tile pipeline: head_dim 64 or 128");
        const int cur = li & 1;
        const int64_t i0 = j0 + QR * (int64_t)n;
        v16f s, dp;
#pragma unroll
        for (int v = 0; v < 16; v++) { s[v] = 0.0f; dp[v] = 0.0f; }
        float4 fa[2], fah[2], fb[2], fv[2];
        auto qfetch = [&](int s8, int buf) {
            fa[buf] = *reinterpret_cast<const float4*>(&sQ[cur][r * LD + s8 * 8 + 4 * h]);
            fah[buf] = *reinterpret_cast<const float4*>(&sQ[cur][r * LD + (s8 + NH) * 8 + 4 * h]);
        };
        auto gfetch = [&](int s8, int buf) {
            fb[buf] = *reinterpret_cast<const float4*>(&sG[cur][r * LD + s8 * 8 + 4 * h]);
            if (kVinLds) fv[buf] = *reinterpret_cast<const float4*>(&sVt[(32 * w + r) * LD + s8 * 8 + 4 * h]);
        };
        auto dpmma = [&](int s8) {
            const float4 b = fb[s8 & 1];
            const float4 vv = kVinLds ? fv[s8 & 1] : vf[kVinLds ? 0 : s8];
            dp = mfma(b.x, vv.x, dp); dp = mfma(b.y, vv.y, dp); dp = mfma(b.z, vv.z, dp); dp = mfma(b.w, vv.w, dp);
        };
        float4 lse4[2], del4[2];
        int4 ss4[2];
        __amdgpu_buffer_rsrc_t ds_rs;
        const int ds_lane_off = (4 * h * 32 + r) * 4;
        auto ds_open = [&]() {
            if (WRITE_DS) {
                const int qt = (int)(i0 >> 5), slot = qt - (int)(jw0 >> 5);
                const int head = kvh * G + hg;
                const int64_t ntile = (int64_t)H * ((T + 31) >> 5) * ds_slots;
                int64_t tidx = (((int64_t)head * ((T + 31) >> 5) + qt) * ds_slots + slot);
                tidx = (slot >= 0 && slot < ds_slots && qt < (int)((T + 31) >> 5)) ? tidx : ntile;
                const uint64_t ta = reinterpret_cast<uint64_t>(DS + (tidx << 10));
                const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)ta), hi = __builtin_amdgcn_readfirstlane((uint32_t)(ta >> 32));
                ds_rs = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0, 4096, 0x00020000);
            }
        };
        DVec<DB> go[2], qq[2];

        // run 1: S over the whole head and dP over its first half
        qfetch(0, 0); gfetch(0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s8 = 0; s8 < NH; s8++) {
            if (s8 + 1 < NH) { qfetch(s8 + 1, (s8 + 1) & 1); gfetch(s8 + 1, (s8 + 1) & 1); } else gfetch(NH, NH & 1);
            if (s8 == 0) tiles_load(hg2, n2);                  // address arithmetic and requests in the shadow of the matrix pipe
            if (s8 == 1) stats_load(hg2, n2);
            if (s8 == 2) ds_open();
            if (s8 == NH - 1) {
                lse4[0] = *reinterpret_cast<const float4*>(&sLse[cur][4 * h]);
                ss4[0] = *reinterpret_cast<const int4*>(&sSS[cur][4 * h]);
            }
            const float4 a = fa[s8 & 1], ah = fah[s8 & 1], b = fb[s8 & 1];
            const float4 vv = kVinLds ? fv[s8 & 1] : vf[kVinLds ? 0 : s8];
            s = mfma(a.x, kf[s8].x, s); dp = mfma(b.x, vv.x, dp); s = mfma(ah.x, kf[s8 + NH].x, s);
            s = mfma(a.y, kf[s8].y, s); dp = mfma(b.y, vv.y, dp); s = mfma(ah.y, kf[s8 + NH].y, s);
            s = mfma(a.z, kf[s8].z, s); dp = mfma(b.z, vv.z, dp); s = mfma(ah.z, kf[s8 + NH].z, s);
            s = mfma(a.w, kf[s8].w, s); dp = mfma(b.w, vv.w, dp); s = mfma(ah.w, kf[s8 + NH].w, s);
            __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // run 2: the second half of dP; every key of the workgroup precedes every query of a straight-line iteration,
        // so the mask only drops queries of a later sequence and rows past the end (their start is INT_MAX).  The
        // compiler moves most of the exponentials to the head of run 3; pinning them between the matrix instructions
        // here measured slower (19.2k against 18.8k cycles per iteration).
#pragma unroll
        for (int s8 = NH; s8 < NS; s8++) {
            if (s8 + 1 < NS) gfetch(s8 + 1, (s8 + 1) & 1);
            else { go[0] = lds_dvec<DB>(&sG[cur][acc_row(0, h) * LD], r); del4[0] = *reinterpret_cast<const float4*>(&sDel[cur][4 * h]); }
            const int v0 = (s8 - NH) * EPS;
            if ((v0 & 3) == 0 && (v0 >> 2) + 1 < 4) {
                lse4[((v0 >> 2) + 1) & 1] = *reinterpret_cast<const float4*>(&sLse[cur][8 * ((v0 >> 2) + 1) + 4 * h]);
                ss4[((v0 >> 2) + 1) & 1] = *reinterpret_cast<const int4*>(&sSS[cur][8 * ((v0 >> 2) + 1) + 4 * h]);
            }
            dpmma(s8);
#pragma unroll
            for (int k = 0; k < EPS; k++) {
                const int v = v0 + k, g = v >> 2, e = v & 3;
                s[v] = (int)j_lane >= (&ss4[g & 1].x)[e] ? fast_exp2(s[v] - (&lse4[g & 1].x)[e]) : 0.0f;
            }
#pragma unroll
            for (int m = 0; m < 4; m++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 2 * EPS, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // run 3: dV, with dS = p (dP - delta) one step ahead of its use in run 4 and the next tile's LDS writes
        // (ahead of the dS stores: loads and stores share one completion counter)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            if (v + 1 < 16) go[(v + 1) & 1] = lds_dvec<DB>(&sG[cur][acc_row(v + 1, h) * LD], r);
            else qq[0] = lds_dvec<DB>(&sQ[cur][acc_row(0, h) * LD], r);
            if ((v & 3) == 0 && (v >> 2) + 1 < 4) del4[((v >> 2) + 1) & 1] = *reinterpret_cast<const float4*>(&sDel[cur][8 * ((v >> 2) + 1) + 4 * h]);
#pragma unroll
            for (int db = 0; db < DB; db++) dv[db] = mfma(s[v], go[v & 1].v[db], dv[db]);
            dp[v] = s[v] * (dp[v] - (&del4[(v >> 2) & 1].x)[v & 3]);
            if (v == 0) tq[0].sstore(sQ[cur ^ 1]);
            if (v == 1) tg[0].sstore(sG[cur ^ 1]);
            if (v == 2) stats_store(cur ^ 1);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
            for (int m = 0; m < DB; m++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // run 4: dK, the dS values leaving one per step
#pragma unroll
        for (int v = 0; v < 16; v++) {
            if (v + 1 < 16) qq[(v + 1) & 1] = lds_dvec<DB>(&sQ[cur][acc_row(v + 1, h) * LD], r);
#pragma unroll
            for (int db = 0; db < DB; db++) dk[db] = mfma(dp[v], qq[v & 1].v[db], dk[db]);
            if (WRITE_DS)
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(dp[v]), ds_rs, ds_lane_off + (8 * (v >> 2) + (v & 3)) * 128, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };
    // The straight-line iteration for two sub-tiles, software-pipelined.  A SIMD runs one wave here (a second wave
    // brought nothing: while a wave's next instruction is a matrix instruction waiting for the pipe, the other wave's
    // arithmetic crawls), so everything that is not a matrix instruction is written into the runs of matrix
    // instructions of the same wave: S/dP of sub-tile 1 carries the softmax of sub-tile 0, dV/dK of sub-tile 0 the
    // softmax of sub-tile 1, the LDS writes of the next tile and the dS stores.  The memory and LDS instructions stay
    // where they are written (every step is one scheduling region); the optimiser still gathers most of the
    // exponentials at the head of the following phase, which measured faster than pinning them to their steps.
    auto iteration2 = [&](int hg, int n, int li, int hg2, int n2) {
        constexpr int NS = D / 8, EPS = 16 / NS;               // S-phase steps, softmax elements per step
        const int cur = li & 1;
        const int64_t i00 = j0 + QR * (int64_t)n;
        v16f s[2], dp[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) { s[t][v] = 0.0f; dp[t][v] = 0.0f; }
        float4 fa[2], fb[2], fv[2];
        auto sfetch = [&](int ro, int s8, int buf) {
            fa[buf] = *reinterpret_cast<const float4*>(&sQ[cur][(ro + r) * LD + s8 * 8 + 4 * h]);
            fb[buf] = *reinterpret_cast<const float4*>(&sG[cur][(ro + r) * LD + s8 * 8 + 4 * h]);
            if (kVinLds) fv[buf] = *reinterpret_cast<const float4*>(&sVt[(32 * w + r) * LD + s8 * 8 + 4 * h]);
        };
        auto smma = [&](int t, int s8) {
            const float4 a = fa[s8 & 1], b = fb[s8 & 1];
            const float4 vv = kVinLds ? fv[s8 & 1] : vf[kVinLds ? 0 : s8];
            s[t] = mfma(a.x, kf[s8].x, s[t]); dp[t] = mfma(b.x, vv.x, dp[t]);
            s[t] = mfma(a.y, kf[s8].y, s[t]); dp[t] = mfma(b.y, vv.y, dp[t]);
            s[t] = mfma(a.z, kf[s8].z, s[t]); dp[t] = mfma(b.z, vv.z, dp[t]);
            s[t] = mfma(a.w, kf[s8].w, s[t]); dp[t] = mfma(b.w, vv.w, dp[t]);
        };
        // row statistics of four rows (accumulator rows 8g+4h .. +3 of sub-tile t), double-buffered like the operands
        float4 lse4[2], del4[2];
        int4 ss4[2];
        auto stats_fetch = [&](int t, int g) {
            lse4[g & 1] = *reinterpret_cast<const float4*>(&sLse[cur][32 * t + 8 * g + 4 * h]);
            del4[g & 1] = *reinterpret_cast<const float4*>(&sDel[cur][32 * t + 8 * g + 4 * h]);
            ss4[g & 1] = *reinterpret_cast<const int4*>(&sSS[cur][32 * t + 8 * g + 4 * h]);
        };
        // Element v of sub-tile t.  Every key of the workgroup precedes every query of a straight-line iteration, so
        // the mask only has to drop queries of a later sequence and rows past the end (their start is INT_MAX).
        auto soft = [&](int t, int v) {
            const int g = v >> 2, e = v & 3;
            const float lse = (&lse4[g & 1].x)[e], del = (&del4[g & 1].x)[e];
            const int ssv = (&ss4[g & 1].x)[e];
            const float p = (int)j_lane >= ssv ? fast_exp2(s[t][v] - lse) : 0.0f;
            s[t][v] = p;
            dp[t][v] = p * (dp[t][v] - del);
        };
        __amdgpu_buffer_rsrc_t ds_rs[2];
        const int ds_lane_off = (4 * h * 32 + r) * 4;
        auto ds_open = [&](int t) {
            if (WRITE_DS) {
                const int64_t i0 = i00 + 32 * t;
                const int qt = (int)(i0 >> 5), slot = qt - (int)(jw0 >> 5);
                const int head = kvh * G + hg;
                const int64_t ntile = (int64_t)H * ((T + 31) >> 5) * ds_slots;
                int64_t tidx = (((int64_t)head * ((T + 31) >> 5) + qt) * ds_slots + slot);
                tidx = (slot >= 0 && slot < ds_slots && qt < (int)((T + 31) >> 5)) ? tidx : ntile;
                const uint64_t ta = reinterpret_cast<uint64_t>(DS + (tidx << 10));
                const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)ta), hi = __builtin_amdgcn_readfirstlane((uint32_t)(ta >> 32));
                ds_rs[t] = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0, 4096, 0x00020000);
            }
        };
        auto ds_put = [&](int t, int v) {
            if (WRITE_DS)
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(dp[t][v]), ds_rs[t], ds_lane_off + (8 * (v >> 2) + (v & 3)) * 128, 0, 0);
        };
        DVec<DB> go[2], qq[2];
        auto dfetch = [&](int t, int v, int buf) {
            go[buf] = lds_dvec<DB>(&sG[cur][(32 * t + acc_row(v, h)) * LD], r);
            qq[buf] = lds_dvec<DB>(&sQ[cur][(32 * t + acc_row(v, h)) * LD], r);
        };
        auto dmma = [&](int t, int v) {
#pragma unroll
            for (int db = 0; db < DB; db++) {
                dv[db] = mfma(s[t][v], go[v & 1].v[db], dv[db]);
                dk[db] = mfma(dp[t][v], qq[v & 1].v[db], dk[db]);
            }
        };

        // Every step below is one scheduling region (nothing crosses the barrier that ends it), so the order of
        // the steps is the order written here and the group barriers only arrange the inside of a step.
        // phase 1: S/dP of sub-tile 0
        sfetch(0, 0, 0);
        stats_fetch(0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s8 = 0; s8 < NS; s8++) {
            if (s8 + 1 < NS) sfetch(0, s8 + 1, (s8 + 1) & 1); else sfetch(32, 0, 0);
            if (s8 == 0) tiles_load(hg2, n2);                  // address arithmetic and requests in the shadow of the matrix pipe
            if (s8 == 1) stats_load(hg2, n2);
            smma(0, s8);
            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // phase 2: S/dP of sub-tile 1, softmax of sub-tile 0 between its matrix instructions
#pragma unroll
        for (int s8 = 0; s8 < NS; s8++) {
            if (s8 + 1 < NS) sfetch(32, s8 + 1, (s8 + 1) & 1);
            const int g = (s8 * EPS) >> 2;
            const bool new_g = ((s8 * EPS) & 3) == 0;
            if (new_g) { if (g + 1 < 4) stats_fetch(0, g + 1); else stats_fetch(1, 0); }
            smma(1, s8);
            if (s8 < 2) ds_open(s8);
#pragma unroll
            for (int k = 0; k < EPS; k++) soft(0, s8 * EPS + k);
            if (s8 + 1 < NS && new_g) __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
            else if (s8 + 1 < NS || new_g) __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
#pragma unroll
            for (int m = 0; m < 8; m++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, EPS, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // phase 3: dV/dK of sub-tile 0 with the softmax of sub-tile 1 between its matrix instructions.  The first
        // four steps also move the next tile to LDS (ahead of the dS stores: loads and stores share one completion
        // counter), the others send out the dS values of sub-tile 0.
        dfetch(0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int v = 0; v < 16; v++) {
            if (v + 1 < 16) dfetch(0, v + 1, (v + 1) & 1); else dfetch(1, 0, 0);
            const bool new_g = (v & 3) == 0 && (v >> 2) + 1 < 4;
            if (new_g) stats_fetch(1, (v >> 2) + 1);
            dmma(0, v);
            soft(1, v);
            if (v == 0) tq[0].sstore(sQ[cur ^ 1]);
            if (v == 1) tg[0].sstore(sG[cur ^ 1]);
            if (v == 2) tq[1].sstore(sQ[cur ^ 1] + 32 * LD);
            if (v == 3) { tg[1].sstore(sG[cur ^ 1] + 32 * LD); stats_store(cur ^ 1); }
            if (v >= 4 && v < 8) { ds_put(0, 2 * (v - 4)); ds_put(0, 2 * (v - 4) + 1); }
            if (v >= 8) ds_put(0, v);
            if (new_g) __builtin_amdgcn_sched_group_barrier(0x100, 5, 0);
            else __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
            for (int m = 0; m < 2 * DB; m++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, (8 + 2 * DB - 1) / (2 * DB), 0);
                if (v < 4) __builtin_amdgcn_sched_group_barrier(0x200, (Tile32<D>::kSlots + 3 + 2 * DB - 1) / (2 * DB), 0);
                else if (m < (v < 8 ? 2 : 1)) __builtin_amdgcn_sched_group_barrier(0x040, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // phase 4: dV/dK of sub-tile 1, its dS values leaving one per step
#pragma unroll
        for (int v = 0; v < 16; v++) {
            if (v + 1 < 16) dfetch(1, v + 1, (v + 1) & 1);
            dmma(1, v);
            ds_put(1, v);
            if (v + 1 < 16) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x040, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * DB - 1, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    };
    {
        // waves without keys (ragged end of the token axis) never take the straight-line copy
        constexpr int kDiag = (4 + QB - 1) / QB;               // iterations that reach into the 128-key diagonal block
        const int ndiag = j0 + 127 < T ? (nq < kDiag ? nq : kDiag) : nq;
        int li = 0;
        // the item's next iteration in (head, run) order, `split` places on; the last one names itself
        auto successor = [&](int g, int n, int& g2, int& n2) {
            g2 = g; n2 = n + split;
            while (n2 >= nq && g2 + 1 < G) { n2 -= nq; g2++; }
            if (n2 >= nq) { g2 = g; n2 = n; }
        };
        for (int g = 0; g < G; g++) {
            int n = ((sub - g * nq) % split + split) % split;      // this item's first query tile of head g
            int g2, n2;
            for (; n < ndiag; n += split, li++) { successor(g, n, g2, n2); iteration(g, n, li, g2, n2); }
            for (; n < nq; n += split, li++) {
                successor(g, n, g2, n2);
                if constexpr (QB == 2) iteration2(g, n, li, g2, n2); else iteration1(g, n, li, g2, n2);
            }
        }
    }
    const bool rmw = split <= 1;                               // else: plain store into this item's slice
    const bool add_old = rmw && !assign;                       // assign: dK/dV are this call's result alone
    float* outK = rmw ? dK : partK + (int64_t)sub * T * kw;
    float* outV = rmw ? dV : partV + (int64_t)sub * T * kw;

    {
        // lane r owns features DB*r .. DB*r+DB-1 of key row jw0 + acc_row(v, h).  When accumulating in place all
        // 32 old values are requested before the first is used: one memory round trip instead of sixteen.
        DVec<DB> oldk[16], oldv[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int64_t j = jw0 + acc_row(v, h);
#pragma unroll
            for (int db = 0; db < DB; db++) { oldk[v].v[db] = 0.f; oldv[v].v[db] = 0.f; }
            if (add_old && j < T) {
                oldk[v] = lds_dvec<DB>(outK + j * kw + kvh * D, r);
                oldv[v] = lds_dvec<DB>(outV + j * kw + kvh * D, r);
            }
        }
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int64_t j = jw0 + acc_row(v, h);
            if (j < T) {
                float* pk = outK + j * kw + kvh * D + DB * r;
                float* pv = outV + j * kw + kvh * D + DB * r;
                float a[DB], b[DB];
#pragma unroll
                for (int db = 0; db < DB; db++) { a[db] = oldk[v].v[db] + dk[db][v] * scale; b[db] = oldv[v].v[db] + dv[db][v]; }
                if (DB == 4) {
                    *reinterpret_cast<float4*>(pk) = make_float4(a[0], a[1 % DB], a[2 % DB], a[3 % DB]);
                    *reinterpret_cast<float4*>(pv) = make_float4(b[0], b[1 % DB], b[2 % DB], b[3 % DB]);
                } else if (DB == 2) {
                    *reinterpret_cast<float2*>(pk) = make_float2(a[0], a[1 % DB]);
                    *reinterpret_cast<float2*>(pv) = make_float2(b[0], b[1 % DB]);
                } else {
                    pk[0] = a[0]; pv[0] = b[0];
                }
            }
        }
    }
    }   // tile queue
    tq_.leave();
}

// dK += sum of the split items' slices, in slice order (likewise dV); with `assign` the sum starts from zero
__device__ __forceinline__ void split_reduce(float* __restrict__ dK, float* __restrict__ dV,
                                             const float* __restrict__ partK, const float* __restrict__ partV,
                                             int64_t n4, int split, int assign, int block, int blocks) {
    for (int64_t i = (int64_t)block * blockDim.x + threadIdx.x; i < n4; i += (int64_t)blocks * blockDim.x) {
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
        if (!assign) { a = reinterpret_cast<float4*>(dK)[i]; b = reinterpret_cast<float4*>(dV)[i]; }
        for (int p = 0; p < split; p++) {
            const float4 x = reinterpret_cast<const float4*>(partK)[p * n4 + i], y = reinterpret_cast<const float4*>(partV)[p * n4 + i];
            a.x += x.x; a.y += x.y; a.z += x.z; a.w += x.w;
            b.x += y.x; b.y += y.y; b.z += y.z; b.w += y.w;
        }
        reinterpret_cast<float4*>(dK)[i] = a;
        reinterpret_cast<float4*>(dV)[i] = b;
    }
}
__global__ __launch_bounds__(256) void attn_split_reduce_kernel(float* __restrict__ dK, float* __restrict__ dV,
                                                                const float* __restrict__ partK, const float* __restrict__ partV,
                                                                int64_t n4, int split, int assign) {
    split_reduce(dK, dV, partK, partV, n4, split, assign, (int)blockIdx.x, (int)gridDim.x);
}
// The same reduction as the last `blocks` workgroups of the dQ-from-dS launch: both only wait for the dK/dV kernel,
// and a short step saves the launch.
struct SplitReduce {
    float* dK; float* dV; const float* partK; const float* partV;
    int64_t n4;
    int split, assign, blocks;          // blocks == 0: nothing to do
};

// ---------------------------------------------------------------- backward: dQ
// grid (query tiles of 128, heads); wave w owns queries i0+32w .. +31; key/value tiles of 32.
template <int D>
__global__ __launch_bounds__(kAttnThreads, (D <= 64 ? 2 : 1)) void attn_bwd_dq_kernel(const float* __restrict__ Q, const float* __restrict__ K,
                                                                   const float* __restrict__ V, const float* __restrict__ dO,
                                                                   const float* __restrict__ LSE, const float* __restrict__ DELTA,
                                                                   float* __restrict__ dQ, const uint32_t* __restrict__ seq_starts, int batch,
                                                                   int64_t T, int H, int KVH, float scale, float scale_log2e,
                                                                   unsigned int* __restrict__ queue,
                                                                   const int* __restrict__ band_overflow, int epoch) {
    constexpr int LD = D + 4, DB = D / 32;
    // As the stand-in of the banded kernel this launch only works when the delta kernel marked the launch.
    if (band_overflow && *band_overflow != epoch) return;
    __shared__ __attribute__((aligned(16))) float sK[2][32 * LD];
    __shared__ __attribute__((aligned(16))) float sV[2][32 * LD];
    __shared__ uint32_t sSeq[kMaxSeqLds];
    __shared__ int sItem;
    const SeqTable seqs = load_seq_table(seq_starts, batch, (int)T, sSeq);
    const int nqt = (int)((T + 127) / 128);
    TileQueue tq_{queue, &sItem, nqt * H};
    __shared__ int sLen[kMaxOrder], sOrd[kMaxOrder];
    const TileOrder by_len = rank_tiles_by_length(sLen, sOrd, nqt, true, tq_.one_each(), [&](int q) {
        const int64_t a = (int64_t)q * 128, z = (a + 127 < T - 1) ? a + 127 : T - 1;
        return (int)((z + 1 - (seqs.start_of((int)a) / 32) * 32 + 31) / 32);
    });
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
    for (int item = tq_.next(); item >= 0; item = tq_.next()) {
    const int head = item % H, kvh = head / (H / KVH);
    const int qt = by_len(item / H);
    const int64_t i0 = (int64_t)qt * 128;
    const int64_t iw0 = i0 + 32 * w, i_lane = iw0 + r;
    const bool row_ok = i_lane < T;
    const int ss_lane = row_ok ? seqs.start_of((int)i_lane) : INT_MAX;
    const float lse_i = row_ok ? LSE[i_lane * H + head] * kLog2e : 0.0f;
    const float del_i = row_ok ? DELTA[i_lane * H + head] : 0.0f;
    const int64_t qw = (int64_t)H * D, kw = (int64_t)KVH * D;

    float4 qf[D / 8], gf[D / 8];
#pragma unroll
    for (int s8 = 0; s8 < D / 8; s8++) {
        qf[s8] = row_ok ? *reinterpret_cast<const float4*>(Q + i_lane * qw + head * D + s8 * 8 + 4 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
        gf[s8] = row_ok ? *reinterpret_cast<const float4*>(dO + i_lane * qw + head * D + s8 * 8 + 4 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    v16f dq[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) dq[db][v] = 0.0f;

    const int64_t i_last = (i0 + 127 < T - 1) ? i0 + 127 : T - 1;
    const int64_t jbeg = (seqs.start_of((int)i0) / 32) * 32;
    const int ntiles = (int)((i_last + 1 - jbeg + 31) / 32);

    Tile32<D> tk, tv;
    tk.gload(K, jbeg, T, kw, kvh * D);
    tv.gload(V, jbeg, T, kw, kvh * D);
    tk.sstore(sK[0]);
    tv.sstore(sV[0]);
    __syncthreads();

    for (int t = 0; t < ntiles; t++) {
        const int cur = t & 1;
        const int64_t j0 = jbeg + 32 * (int64_t)t;
        if (t + 1 < ntiles) {
            tk.gload(K, j0 + 32, T, kw, kvh * D);
            tv.gload(V, j0 + 32, T, kw, kvh * D);
        }
        if (j0 <= iw0 + 31 && iw0 < T) {
            v16f s, dp;
#pragma unroll
            for (int v = 0; v < 16; v++) { s[v] = 0.0f; dp[v] = 0.0f; }
#pragma unroll
            for (int s8 = 0; s8 < D / 8; s8++) {
                const float4 a = *reinterpret_cast<const float4*>(&sK[cur][r * LD + s8 * 8 + 4 * h]);
                const float4 b = *reinterpret_cast<const float4*>(&sV[cur][r * LD + s8 * 8 + 4 * h]);
                s = mfma(a.x, qf[s8].x, s); dp = mfma(b.x, gf[s8].x, dp);
                s = mfma(a.y, qf[s8].y, s); dp = mfma(b.y, gf[s8].y, dp);
                s = mfma(a.z, qf[s8].z, s); dp = mfma(b.z, gf[s8].z, dp);
                s = mfma(a.w, qf[s8].w, s); dp = mfma(b.w, gf[s8].w, dp);
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int j = (int)j0 + acc_row(v, h);
                const bool valid = (j >= ss_lane) && (j <= (int)i_lane);
                const float p = valid ? fast_exp2(s[v] * scale_log2e - lse_i) : 0.0f;
                dp[v] = p * (dp[v] - del_i);
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const DVec<DB> kk = lds_dvec<DB>(&sK[cur][acc_row(v, h) * LD], r);
#pragma unroll
                for (int db = 0; db < DB; db++) dq[db] = mfma(dp[v], kk.v[db], dq[db]);
            }
        }
        if (t + 1 < ntiles) {
            tk.sstore(sK[cur ^ 1]);
            tv.sstore(sV[cur ^ 1]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int64_t i = iw0 + acc_row(v, h);
        if (i < T) {
            float* pq = dQ + i * qw + head * D + DB * r;
            if (DB == 4) *reinterpret_cast<float4*>(pq) = make_float4(dq[0][v] * scale, dq[1 % DB][v] * scale, dq[2 % DB][v] * scale, dq[3 % DB][v] * scale);
            else if (DB == 2) *reinterpret_cast<float2*>(pq) = make_float2(dq[0][v] * scale, dq[1 % DB][v] * scale);
            else pq[0] = dq[0][v] * scale;
        }
    }
    }   // tile queue
    tq_.leave();
}

// ---------------------------------------------------------------- backward: dQ from stored dS
// The dK/dV kernel can leave dS = P (dP - delta) behind, one 32x32 row-major tile per (head,
// query tile, key tile) in a band of ds_slots key tiles below the diagonal.  dQ = scale dS K is
// then a single product per tile and the backward executes 5 products instead of 7.
// grid: persistent over (128-query tiles, heads); wave w owns queries i0+32w .. +31.
// KSPLIT (short batches, as in the forward kernel): 64-query items; waves 0,1 take the even key tiles, waves 2,3 the
// odd ones of the same queries, two key tiles are staged per iteration and the two partial dQ meet in LDS.
template <int D, bool KSPLIT>
__global__ __launch_bounds__(kAttnThreads, 2) void attn_bwd_dq_ds_kernel(const float* __restrict__ K, const float* __restrict__ DS,
                                                                         float* __restrict__ dQ, const uint32_t* __restrict__ seq_starts,
                                                                         int batch, int64_t T, int H, int KVH, float scale, int ds_slots,
                                                                         unsigned int* __restrict__ queue,
                                                                         const int* __restrict__ band_overflow, int epoch,
                                                                         const SplitReduce red) {
    constexpr int LD = D + 4, DB = D / 32;
    constexpr int KT = KSPLIT ? 2 : 1, QROWS = KSPLIT ? 64 : 128;
    if (red.blocks > 0 && blockIdx.x >= gridDim.x - (unsigned)red.blocks) {          // uniform over the workgroup
        split_reduce(red.dK, red.dV, red.partK, red.partV, red.n4, red.split, red.assign,
                     (int)(blockIdx.x - (gridDim.x - (unsigned)red.blocks)), red.blocks);
        return;
    }
    // Some sequence is longer than the band was sized for: dQ comes from the recomputing kernel launched next.
    if (*band_overflow == epoch) return;
    __shared__ __attribute__((aligned(16))) float sK[2][KT * 32 * LD];
    __shared__ uint32_t sSeq[kMaxSeqLds];
    __shared__ int sItem;
    const SeqTable seqs = load_seq_table(seq_starts, batch, (int)T, sSeq);
    const int nqt = (int)((T + QROWS - 1) / QROWS);
    const int64_t nqt32 = (T + 31) >> 5;
    TileQueue tq_{queue, &sItem, nqt * H, red.blocks};
    __shared__ int sLen[kMaxOrder], sOrd[kMaxOrder];
    const TileOrder by_len = rank_tiles_by_length(sLen, sOrd, nqt, true, tq_.one_each(), [&](int q) {
        const int64_t a = (int64_t)q * QROWS, z = (a + QROWS - 1 < T - 1) ? a + QROWS - 1 : T - 1;
        return (int)((z + 1 - (seqs.start_of((int)a) / 32) * 32 + 31) / 32);
    });
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
    const int wq = KSPLIT ? (w & 1) : w, kp = KSPLIT ? (w >> 1) : 0;  // the wave's 32 queries within the item; its key-tile parity
    for (int item = tq_.next(); item >= 0; item = tq_.next()) {
    const int head = item % H, kvh = head / (H / KVH);
    const int qtile = by_len(item / H);
    const int64_t i0 = (int64_t)qtile * QROWS;
    const int64_t iw0 = i0 + 32 * wq;
    const int64_t qw = (int64_t)H * D, kw = (int64_t)KVH * D;
    const int64_t i_last = (i0 + QROWS - 1 < T - 1) ? i0 + QROWS - 1 : T - 1;
    const int64_t jbeg = (seqs.start_of((int)i0) / 32) * 32;
    const int ntiles = (int)((i_last + 1 - jbeg + 31) / 32);
    // this wave's own range of key tiles (relative to jbeg): from the tile holding the start of its
    // first query's sequence up to its diagonal tile; empty when the wave lies past the end
    const bool wave_ok = iw0 < T;
    const int qt = (int)(iw0 >> 5);
    int tb = 0, te = -1;
    if (wave_ok) {
        tb = (int)(((int64_t)(seqs.start_of((int)iw0) / 32) * 32 - jbeg) / 32);
        te = (int)((iw0 - jbeg) / 32);
        // never read a slot the band does not have (only possible in a launch that is marked as overflowing,
        // which returns above; the clamp keeps every address inside the scratch regardless)
        const int tmin = qt - (int)(jbeg >> 5) - (ds_slots - 1);
        tb = tb < tmin ? tmin : tb;
    }
    const float* band = DS + ((((int64_t)head * nqt32 + (wave_ok ? qt : 0)) * ds_slots) << 10);   // slot 0 = diagonal tile
    const int kt0 = (int)(jbeg >> 5);

    v16f dq[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) dq[db][v] = 0.0f;

    float4 dsf[2][4];
    auto ds_load = [&](int t, int buf) {                       // buf is a literal at every call site
        // a tile outside the wave's range is replaced by one inside it (loaded, never used)
        int tc = t < tb ? tb : t;
        tc = tc > te ? te : tc;
        const int slot = wave_ok ? qt - (kt0 + tc) : 0;
        const float* tile = band + ((int64_t)slot << 10) + r * 32 + 4 * h;
#pragma unroll
        for (int s8 = 0; s8 < 4; s8++) dsf[buf][s8] = *reinterpret_cast<const float4*>(tile + 8 * s8);
    };

    Tile32<D> tk[KT];
    auto k_load = [&](int t0) {                                // tiles t0 .. t0+KT-1; rows past the last token read as zeros
#pragma unroll
        for (int u = 0; u < KT; u++) tk[u].gload(K, jbeg + 32 * (int64_t)(t0 + u), T, kw, kvh * D);
    };
    auto k_store = [&](int buf) {
#pragma unroll
        for (int u = 0; u < KT; u++) tk[u].sstore(sK[buf] + u * 32 * LD);
    };
    k_load(0);
    ds_load(kp, 0);
    k_store(0);
    __syncthreads();

    // tp = first of the KT staged tiles; this wave's tile is tp + kp
    auto body = [&](auto parity, int tp) {
        constexpr int CUR = decltype(parity)::value;          // register and LDS buffers by compile-time parity
        const int t = tp + kp;
        const float* sKt = sK[CUR] + kp * 32 * LD;
        if (tp + KT < ntiles) k_load(tp + KT);
        ds_load(t + KT, CUR ^ 1);                               // clamped into the wave's range inside
        if (t >= tb && t <= te) {
#pragma unroll
            for (int s8 = 0; s8 < 4; s8++) {
                const float e[4] = {dsf[CUR][s8].x, dsf[CUR][s8].y, dsf[CUR][s8].z, dsf[CUR][s8].w};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const DVec<DB> kk = lds_dvec<DB>(&sKt[(8 * s8 + 4 * h + q) * LD], r);
#pragma unroll
                    for (int db = 0; db < DB; db++) dq[db] = mfma(e[q], kk.v[db], dq[db]);
                }
            }
        }
        if (tp + KT < ntiles) k_store(CUR ^ 1);
        __syncthreads();
    };
    int tp = 0;
    for (; tp + KT < ntiles; tp += 2 * KT) {
        body(std::integral_constant<int, 0>{}, tp);
        body(std::integral_constant<int, 1>{}, tp + KT);
    }
    if (tp < ntiles) body(std::integral_constant<int, 0>{}, tp);

    if (KSPLIT) {
        // waves 2,3 hand their partial dQ to waves 0,1 through the tile buffers (nobody reads them any more; the
        // next item restages them only behind the queue's barriers)
        float* xo = &sK[0][0] + (size_t)wq * DB * 16 * 64;
        static_assert(!KSPLIT || 2 * KT * 32 * LD >= 2 * DB * 16 * 64, "tile buffers too small for the exchange");
        if (kp == 1) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) xo[(db * 16 + v) * 64 + lane] = dq[db][v];
        }
        __syncthreads();
        if (kp == 0) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) dq[db][v] += xo[(db * 16 + v) * 64 + lane];
        }
    }

    if (kp == 0)
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int64_t i = iw0 + acc_row(v, h);
        if (i < T) {
            float* pq = dQ + i * qw + head * D + DB * r;
            if (DB == 4) *reinterpret_cast<float4*>(pq) = make_float4(dq[0][v] * scale, dq[1 % DB][v] * scale, dq[2 % DB][v] * scale, dq[3 % DB][v] * scale);
            else if (DB == 2) *reinterpret_cast<float2*>(pq) = make_float2(dq[0][v] * scale, dq[1 % DB][v] * scale);
            else pq[0] = dq[0][v] * scale;
        }
    }
    }   // tile queue
    tq_.leave();
}

// ---------------------------------------------------------------- host side
struct AttnWs { float* lse; float* delta; float* out; float* partK; float* partV; int* row_start; int* overflow; float* ds; };
constexpr int kMaxSplit = 4;

// Band of dS tiles: for every head and 32-query tile, the key tiles from the diagonal down to the
// tile that holds the start of the longest sequence allowed.
static int ds_slot_count(int64_t max_seq_len) { return (int)((max_seq_len + 31) / 32) + 1; }
static size_t ds_band_bytes(int64_t T, int H, int64_t max_seq_len) {
    return ((size_t)H * (size_t)((T + 31) / 32) * (size_t)ds_slot_count(max_seq_len) + 1) * 4096;     // + one spare tile
}

static size_t a256(size_t x) { return (x + 255) & ~(size_t)255; }

static size_t attn_ws_layout(int64_t T, int H, int KVH, int D, char* base, AttnWs* w) {
    size_t o = 0;
    auto take = [&](size_t bytes) { char* p = base ? base + o : nullptr; o += a256(bytes); return p; };
    char* c = take((size_t)T * H * 4); char* d = take((size_t)T * H * 4);
    char* e = take((size_t)T * H * D * 4);
    char* pk = take((size_t)kMaxSplit * T * KVH * D * 4); char* pv = take((size_t)kMaxSplit * T * KVH * D * 4);
    char* rs = take((size_t)T * 4);
    char* ov = take(4);
    if (w) {
        w->overflow = (int*)ov;
        w->lse = (float*)c; w->delta = (float*)d; w->out = (float*)e; w->partK = (float*)pk; w->partV = (float*)pv;
        w->row_start = (int*)rs;
        w->ds = base ? (float*)(base + o) : nullptr;
    }
    return o;
}

static int check_attn_shape(const char* who, int64_t T, int H, int KVH, int D) {
    SERAPH_REQUIRE(T > 0 && T < 0x7fffff00LL, "%s: bad token count %lld", who, (long long)T);
    SERAPH_REQUIRE(H > 0 && KVH > 0 && H % KVH == 0, "%s: heads (%d) must be a multiple of kv_heads (%d)", who, H, KVH);
    SERAPH_REQUIRE(D == 32 || D == 64 || D == 128, "%s: head_dim %d not supported (32, 64, 128)", who, D);
    return SERAPH_OK;
}

// One counter pair per launch, in rotation over the pool.
static int acquire_tile_queue(unsigned int** out) {
    static std::mutex mu;
    static unsigned int* base[64] = {nullptr};
    static unsigned next_slot = 0;
    int dev = 0;
    SERAPH_HIP_CHECK(hipGetDevice(&dev));
    SERAPH_REQUIRE(dev >= 0 && dev < 64, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lk(mu);
    if (!base[dev]) SERAPH_HIP_CHECK(hipGetSymbolAddress((void**)&base[dev], HIP_SYMBOL(g_tile_queues)));
    *out = base[dev] + 2 * (next_slot++ % kQueueSlots);
    return SERAPH_OK;
}

// Resident workgroups for a persistent launch: as many as fit per CU, never more than there are tiles.
static unsigned persistent_grid(int64_t items, int per_cu) {
    int64_t cap = (int64_t)num_compute_units() * per_cu;
    return (unsigned)(items < cap ? items : cap);
}

template <int D>
static int run_forward(const float* Q, const float* K, const float* V, float* O, float* lse, const uint32_t* seq_starts, int batch,
                       int64_t T, int H, int KVH, float scale, hipStream_t st) {
    unsigned int* queue = nullptr;
    int rc = acquire_tile_queue(&queue);
    if (rc != SERAPH_OK) return rc;
    // A short batch leaves CUs without a 128-query tile while the longest tile alone sets the time: 64-query
    // items whose keys two wave pairs share out (one workgroup per CU: twice the LDS tiles).
    // (measured at 16 heads of 128: 4096 tokens in one sequence 1.08 -> 0.71 ms, 2048 tokens 0.30 -> 0.20 ms; from
    // four tiles per CU on the plain kernel is faster: 8192 tokens 1.16 against 1.39 ms)
    if (ceil_div(T, 128) * H <= 2 * (int64_t)num_compute_units()) {
        dim3 grid(persistent_grid(ceil_div(T, 64) * H, 1));
        hipLaunchKernelGGL((attn_fwd_kernel<D, true>), grid, dim3(kAttnThreads), 0, st, Q, K, V, O, lse, seq_starts, batch, T, H, KVH, scale * kLog2e, queue);
    } else {
        dim3 grid(persistent_grid(ceil_div(T, 128) * H, 2));
        hipLaunchKernelGGL((attn_fwd_kernel<D, false>), grid, dim3(kAttnThreads), 0, st, Q, K, V, O, lse, seq_starts, batch, T, H, KVH, scale * kLog2e, queue);
    }
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

template <int D>
static int run_backward(const float* Q, const float* K, const float* V, const float* dO, const float* O, const float* lse,
                        float* delta, int* row_start, int* overflow, float* dQ, float* dK, float* dV, const uint32_t* seq_starts, int batch,
                        int64_t T, int H, int KVH, float scale, int64_t longest_seq, float* ds, int ds_slots, float* partK, float* partV,
                        bool assign, bool bound_verified, hipStream_t st) {
    unsigned int *qkv = nullptr, *qq = nullptr;
    int rc = acquire_tile_queue(&qkv);
    if (rc == SERAPH_OK) rc = acquire_tile_queue(&qq);
    if (rc != SERAPH_OK) return rc;
    // The bound on the sequence length is the caller's word; the device checks it against the real offsets.  A
    // launch number that the scratch cannot hold by accident marks "this launch overflowed its band".
    static std::atomic<int> launch_counter{0};
    const int epoch = (launch_counter.fetch_add(1) & 0x3fffffff) + 1;
    const bool bound_can_fail = ds && !bound_verified && (int64_t)ds_slots < ceil_div(T, 32) + 1;
    hipLaunchKernelGGL(attn_delta_kernel<D>, dim3((unsigned)ceil_div(T, 4)), dim3(256), 0, st, dO, O, delta, T, H, seq_starts, batch, row_start,
                       ds ? ds_slots : 0, epoch, overflow, qkv, qq);
    SERAPH_LAUNCH_CHECK();
    const int per_cu = D <= 64 ? 2 : 1;
    constexpr int kv_per_cu = 1;                               // the dK/dV kernel's registers and LDS tiles leave room for one workgroup
    const int64_t kv_items = ceil_div(T, 128) * KVH;
    // Few (key tile, kv head) items: split each between several workgroups.  The longest item (a sequence's first
    // key tile) is about twice the average, so the aim is two items per CU; an item keeps at least four 32-query
    // tiles, below which its set-up costs more than the split saves.  Measured at 2048 tokens in one sequence,
    // 16/8 heads of 128: 1.21 / 0.71 / 0.49 / 0.52 ms for 1 / 2 / 4 / 8 ways; at 8 x 256 tokens, 8 heads of 64:
    // 0.069 / 0.061 / 0.070 / 0.090 ms.
    int split = (int)(2 * (int64_t)num_compute_units() / kv_items);
    const int64_t by_length = longest_seq * (H / KVH) / 128;
    split = split > by_length ? (int)by_length : split;
    split = split < 1 ? 1 : (split > kMaxSplit ? kMaxSplit : split);
    dim3 gkv(persistent_grid(kv_items * split, kv_per_cu)), gq(persistent_grid(ceil_div(T, 128) * H, per_cu));
    if (ds)
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<D, true>), gkv, dim3(kAttnThreads), 0, st, Q, K, V, dO, lse, delta, row_start, dK, dV, seq_starts, batch,
                           T, H, KVH, scale, scale * kLog2e, qkv, ds, ds_slots, split, partK, partV, assign ? 1 : 0);
    else
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<D, false>), gkv, dim3(kAttnThreads), 0, st, Q, K, V, dO, lse, delta, row_start, dK, dV, seq_starts, batch,
                           T, H, KVH, scale, scale * kLog2e, qkv, ds, ds_slots, split, partK, partV, assign ? 1 : 0);
    const int64_t n4 = T * KVH * D / 4;
    SplitReduce red{dK, dV, partK, partV, n4, split, assign ? 1 : 0, 0};
    if (split > 1 && !ds) {
        SERAPH_LAUNCH_CHECK();
        hipLaunchKernelGGL(attn_split_reduce_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(n4, 256), 4096)), dim3(256), 0, st,
                           dK, dV, partK, partV, n4, split, assign ? 1 : 0);
    }
    SERAPH_LAUNCH_CHECK();
    if (ds) {
        // the slices of a split dK/dV are added by workgroups at the end of the dQ launch (nothing else is between the
        // dK/dV kernel and either of them)
        if (split > 1) red.blocks = (int)std::min<int64_t>(ceil_div(n4, 256), 2 * (int64_t)num_compute_units());
        if (ceil_div(T, 128) * H <= 2 * (int64_t)num_compute_units()) {        // short batch: see run_forward
            dim3 gds((unsigned)std::min<int64_t>(ceil_div(T, 64) * H, (int64_t)num_compute_units() * 2) + (unsigned)red.blocks);
            hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<D, true>), gds, dim3(kAttnThreads), 0, st, K, ds, dQ, seq_starts, batch, T, H, KVH, scale, ds_slots, qq, overflow, epoch, red);
        } else {
            dim3 gds((unsigned)std::min<int64_t>(ceil_div(T, 128) * H, (int64_t)num_compute_units() * 2) + (unsigned)red.blocks);
            hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<D, false>), gds, dim3(kAttnThreads), 0, st, K, ds, dQ, seq_starts, batch, T, H, KVH, scale, ds_slots, qq, overflow, epoch, red);
        }
        if (bound_can_fail) {                                   // stands down at once unless the delta kernel marked the launch
            SERAPH_LAUNCH_CHECK();
            hipLaunchKernelGGL(attn_bwd_dq_kernel<D>, gq, dim3(kAttnThreads), 0, st, Q, K, V, dO, lse, delta, dQ, seq_starts, batch,
                               T, H, KVH, scale, scale * kLog2e, qq, (const int*)overflow, epoch);
        }
    } else {
        hipLaunchKernelGGL(attn_bwd_dq_kernel<D>, gq, dim3(kAttnThreads), 0, st, Q, K, V, dO, lse, delta, dQ, seq_starts, batch,
                           T, H, KVH, scale, scale * kLog2e, qq, (const int*)nullptr, 0);
    }
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

}  // namespace seraph

using namespace seraph;

extern "C" {

size_t seraph_attention_backward_ws_bytes(int64_t T, int heads, int kv_heads, int head_dim) {
    (void)kv_heads;
    if (T <= 0 || heads <= 0 || head_dim <= 0) return 0;
    return attn_ws_layout(T, heads, kv_heads, head_dim, nullptr, nullptr);
}

int seraph_attention_forward(const float* Q, const float* K, const float* V, float* out, float* lse,
                             const uint32_t* seq_starts, int batch, int64_t T,
                             int heads, int kv_heads, int head_dim, float scale, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(Q && K && V && out, "attention_forward: NULL pointer");
    int rc = check_attn_shape("attention_forward", T, heads, kv_heads, head_dim);
    if (rc != SERAPH_OK) return rc;
    SERAPH_REQUIRE(aligned16(Q) && aligned16(K) && aligned16(V) && aligned16(out), "attention_forward: buffers must be 16-byte aligned");
    SERAPH_REQUIRE(!seq_starts || batch >= 1, "attention_forward: packed call needs batch >= 1");
    hipStream_t st = as_stream(s);
    switch (head_dim) {
        case 32: rc = run_forward<32>(Q, K, V, out, lse, seq_starts, batch, T, heads, kv_heads, scale, st); break;
        case 64: rc = run_forward<64>(Q, K, V, out, lse, seq_starts, batch, T, heads, kv_heads, scale, st); break;
        default: rc = run_forward<128>(Q, K, V, out, lse, seq_starts, batch, T, heads, kv_heads, scale, st); break;
    }
    return rc;
}

size_t seraph_attention_backward_ws_bytes_banded(int64_t T, int heads, int kv_heads, int head_dim, int64_t max_seq_len) {
    (void)kv_heads;
    if (T <= 0 || heads <= 0 || head_dim <= 0) return 0;
    if (max_seq_len <= 0 || max_seq_len > T) max_seq_len = T;
    return attn_ws_layout(T, heads, kv_heads, head_dim, nullptr, nullptr) + ds_band_bytes(T, heads, max_seq_len);
}

int seraph_attention_backward(const float* Q, const float* K, const float* V, const float* dO,
                              const float* attn_out, const float* lse,
                              float* dQ, float* dK, float* dV,
                              const uint32_t* seq_starts, int batch, int64_t T,
                              int heads, int kv_heads, int head_dim, float scale,
                              void* ws, size_t ws_bytes, seraph_stream_t s) {
    return seraph_attention_backward_banded(Q, K, V, dO, attn_out, lse, dQ, dK, dV, seq_starts, batch, T, heads, kv_heads,
                                            head_dim, scale, T, ws, ws_bytes, s);
}

static int attention_backward_any(const float* Q, const float* K, const float* V, const float* dO,
                                  const float* attn_out, const float* lse,
                                  float* dQ, float* dK, float* dV,
                                  const uint32_t* seq_starts, int batch, int64_t T,
                                  int heads, int kv_heads, int head_dim, float scale, int64_t max_seq_len,
                                  bool assign, bool bound_verified,
                                  void* ws, size_t ws_bytes, seraph_stream_t s);

int seraph_attention_backward_banded(const float* Q, const float* K, const float* V, const float* dO,
                                     const float* attn_out, const float* lse,
                                     float* dQ, float* dK, float* dV,
                                     const uint32_t* seq_starts, int batch, int64_t T,
                                     int heads, int kv_heads, int head_dim, float scale, int64_t max_seq_len,
                                     void* ws, size_t ws_bytes, seraph_stream_t s) {
    return attention_backward_any(Q, K, V, dO, attn_out, lse, dQ, dK, dV, seq_starts, batch, T, heads, kv_heads, head_dim, scale,
                                  max_seq_len, false, false, ws, ws_bytes, s);
}

int seraph_attention_backward_assign(const float* Q, const float* K, const float* V, const float* dO,
                                     const float* attn_out, const float* lse,
                                     float* dQ, float* dK, float* dV,
                                     const uint32_t* seq_starts, const uint32_t* host_seq_starts, int batch, int64_t T,
                                     int heads, int kv_heads, int head_dim, float scale,
                                     void* ws, size_t ws_bytes, seraph_stream_t s) {
    // The host's copy of the offsets gives the exact longest sequence, so the dS band is sized by a bound that
    // cannot fail and the launch that stands by for a failed bound is left out.
    int64_t longest = T;
    if (seq_starts) {
        SERAPH_REQUIRE(host_seq_starts && batch >= 1, "attention_backward_assign: packed call needs the host copy of seq_starts");
        SERAPH_REQUIRE(host_seq_starts[0] == 0 && (int64_t)host_seq_starts[batch] == T, "attention_backward_assign: seq_starts must run from 0 to T");
        longest = 1;
        for (int b = 0; b < batch; b++) {
            SERAPH_REQUIRE(host_seq_starts[b + 1] >= host_seq_starts[b], "attention_backward_assign: seq_starts must not decrease");
            const int64_t len = (int64_t)host_seq_starts[b + 1] - host_seq_starts[b];
            longest = len > longest ? len : longest;
        }
    }
    return attention_backward_any(Q, K, V, dO, attn_out, lse, dQ, dK, dV, seq_starts, batch, T, heads, kv_heads, head_dim, scale,
                                  longest, true, true, ws, ws_bytes, s);
}

static int attention_backward_any(const float* Q, const float* K, const float* V, const float* dO,
                                  const float* attn_out, const float* lse,
                                  float* dQ, float* dK, float* dV,
                                  const uint32_t* seq_starts, int batch, int64_t T,
                                  int heads, int kv_heads, int head_dim, float scale, int64_t max_seq_len,
                                  bool assign, bool bound_verified,
                                  void* ws, size_t ws_bytes, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(Q && K && V && dO && dQ && dK && dV, "attention_backward: NULL pointer");
    int rc = check_attn_shape("attention_backward", T, heads, kv_heads, head_dim);
    if (rc != SERAPH_OK) return rc;
    SERAPH_REQUIRE(aligned16(Q) && aligned16(K) && aligned16(V) && aligned16(dO) && (!attn_out || aligned16(attn_out)),
                   "attention_backward: buffers must be 16-byte aligned");
    SERAPH_REQUIRE(!seq_starts || batch >= 1, "attention_backward: packed call needs batch >= 1");
    if (!ws || !aligned16(ws) || ws_bytes < seraph_attention_backward_ws_bytes(T, heads, kv_heads, head_dim)) {
        set_error("attention_backward: 16-byte aligned scratch of %zu bytes required",
                  seraph_attention_backward_ws_bytes(T, heads, kv_heads, head_dim));
        return SERAPH_ERR_WORKSPACE;
    }
    AttnWs w;
    attn_ws_layout(T, heads, kv_heads, head_dim, (char*)ws, &w);
    // the 5-product path needs the dS band behind the fixed part of the scratch
    if (max_seq_len <= 0 || max_seq_len > T) max_seq_len = T;
    const bool banded = ws_bytes >= seraph_attention_backward_ws_bytes_banded(T, heads, kv_heads, head_dim, max_seq_len);
    float* ds = banded ? w.ds : nullptr;
    const int ds_slots = banded ? ds_slot_count(max_seq_len) : 0;
    hipStream_t st = as_stream(s);
    const float* O = attn_out;
    const float* L = lse;
    if (!O || !L) {                                              // recompute the forward results
        switch (head_dim) {
            case 32: rc = run_forward<32>(Q, K, V, w.out, w.lse, seq_starts, batch, T, heads, kv_heads, scale, st); break;
            case 64: rc = run_forward<64>(Q, K, V, w.out, w.lse, seq_starts, batch, T, heads, kv_heads, scale, st); break;
            default: rc = run_forward<128>(Q, K, V, w.out, w.lse, seq_starts, batch, T, heads, kv_heads, scale, st); break;
        }
        if (rc != SERAPH_OK) return rc;
        O = w.out; L = w.lse;
    }
    switch (head_dim) {
        case 32: return run_backward<32>(Q, K, V, dO, O, L, w.delta, w.row_start, w.overflow, dQ, dK, dV, seq_starts, batch, T, heads, kv_heads, scale, max_seq_len, ds, ds_slots, w.partK, w.partV, assign, bound_verified, st);
        case 64: return run_backward<64>(Q, K, V, dO, O, L, w.delta, w.row_start, w.overflow, dQ, dK, dV, seq_starts, batch, T, heads, kv_heads, scale, max_seq_len, ds, ds_slots, w.partK, w.partV, assign, bound_verified, st);
        default: return run_backward<128>(Q, K, V, dO, O, L, w.delta, w.row_start, w.overflow, dQ, dK, dV, seq_starts, batch, T, heads, kv_heads, scale, max_seq_len, ds, ds_slots, w.partK, w.partV, assign, bound_verified, st);
    }
}

}  // extern "C"
