// cross_entropy.hip - fused softmax cross-entropy loss + gradient.
//
// Three shapes of the same arithmetic (shaders/cross_entropy_grad.comp:44-98):
//   * rows that fit one workgroup's registers (cols <= 32768) are owned by one workgroup and read from HBM once;
//   * longer rows (a 151936-entry vocabulary is 608 KB) are shared out between P workgroups that each keep their
//     part in registers and exchange one (max, sum of exponentials) pair per row through device memory: every
//     logit crosses HBM once in each direction (16384 x 151936: 3.44 ms, 5.8 TB/s; the earlier form that kept a
//     row in one workgroup's registers and LDS and re-read a quarter of it took 4.05 ms);
//   * unaligned or odd-length rows take an online max / sum-of-exponentials sweep and a second
//     sweep in the opposite direction.
// Rows without supervision (target >= cols, or the last token of a packed sequence)
// are written as zeros without being read.  All offsets are 64-bit: rows*cols exceeds
// 2^31 at the shapes this runs on.
#include <atomic>
#include <mutex>

#include "common.hpp"

namespace seraph {

constexpr float kNegBig = -3.4e38f;      // the shader's initial maximum
constexpr size_t kLastLevelCacheBytes = 256u << 20;   // MI355X Infinity Cache

struct MaxSum { float m, s; };

__device__ __forceinline__ MaxSum combine(MaxSum a, MaxSum b) {
    float m = fmaxf(a.m, b.m);
    MaxSum r;
    r.m = m;
    r.s = a.s * __expf(a.m - m) + b.s * __expf(b.m - m);
    return r;
}

template <int BLOCK>
__device__ __forceinline__ MaxSum block_combine(MaxSum v, MaxSum* lds) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        MaxSum other;
        other.m = __shfl_xor(v.m, o, 64);
        other.s = __shfl_xor(v.s, o, 64);
        v = combine(v, other);
    }
    if (lane == 0) lds[wv] = v;
    __syncthreads();
    MaxSum r = lds[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; w++) r = combine(r, lds[w]);
    return r;
}

// Is row `row` supervised?  Packed batches: every token but the last of its sequence.
__device__ __forceinline__ bool row_live(const uint32_t* seq_starts, int batch, int64_t row) {
    if (!seq_starts) return true;
    int sq = find_seq(seq_starts, batch, row);
    return row < (int64_t)seq_starts[sq + 1] - 1;
}

__device__ __forceinline__ float grad_of(float x, float mx, float inv_sum, float scale, bool is_target) {
    float p = __expf(x - mx) * inv_sum;
    return (is_target ? p - 1.0f : p) * scale;
}

// ---------------------------------------------------------------- register-resident rows
template <int BLOCK, int VPT>
__global__ __launch_bounds__(BLOCK) void ce_small_kernel(const float* __restrict__ logits,
                                                         const uint32_t* __restrict__ targets,
                                                         float* __restrict__ grad, float* __restrict__ loss_rows,
                                                         const uint32_t* __restrict__ seq_starts, int batch,
                                                         int cols, float scale) {
    __shared__ MaxSum lds[BLOCK / 64];
    const int64_t row = blockIdx.x;
    const int n4 = cols >> 2;
    const uint32_t target = targets[row];
    float4* gr = reinterpret_cast<float4*>(grad + row * cols);
    if (target >= (uint32_t)cols || !row_live(seq_starts, batch, row)) {
        for (int i4 = threadIdx.x; i4 < n4; i4 += BLOCK) gr[i4] = make_float4(0, 0, 0, 0);
        if (threadIdx.x == 0) loss_rows[row] = 0.0f;
        return;
    }
    const float4* xr = reinterpret_cast<const float4*>(logits + row * cols);
    float4 v[VPT];
    float mx = kNegBig;
#pragma unroll
    for (int k = 0; k < VPT; k++) {
        int i4 = threadIdx.x + BLOCK * k;
        v[k] = i4 < n4 ? xr[i4] : make_float4(kNegBig, kNegBig, kNegBig, kNegBig);
        mx = fmaxf(mx, fmaxf(fmaxf(v[k].x, v[k].y), fmaxf(v[k].z, v[k].w)));
    }
    MaxSum ms;
    ms.m = mx;
    ms.s = 0.0f;
#pragma unroll
    for (int k = 0; k < VPT; k++)
        ms.s += __expf(v[k].x - mx) + __expf(v[k].y - mx) + __expf(v[k].z - mx) + __expf(v[k].w - mx);
    ms = block_combine<BLOCK>(ms, lds);
    const float inv_sum = 1.0f / ms.s;
#pragma unroll
    for (int k = 0; k < VPT; k++) {
        int i4 = threadIdx.x + BLOCK * k;
        if (i4 < n4) {
            uint32_t c = (uint32_t)i4 * 4;
            if ((target >> 2) == (uint32_t)i4) {     // the lane that holds the target logit writes the loss
                uint32_t e = target & 3u;            // (grad may alias logits: nothing is re-read from memory)
                float xt = e == 0 ? v[k].x : e == 1 ? v[k].y : e == 2 ? v[k].z : v[k].w;
                loss_rows[row] = -((xt - ms.m) - __logf(ms.s));
            }
            gr[i4] = make_float4(grad_of(v[k].x, ms.m, inv_sum, scale, c == target),
                                 grad_of(v[k].y, ms.m, inv_sum, scale, c + 1 == target),
                                 grad_of(v[k].z, ms.m, inv_sum, scale, c + 2 == target),
                                 grad_of(v[k].w, ms.m, inv_sum, scale, c + 3 == target));
        }
    }
}

// ---------------------------------------------------------------- helpers of the long-row kernel
typedef float f4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ld_stream4(const float4* p) {
    const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st_stream4(float4* p, float4 v) {
    const f4v r = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(r, reinterpret_cast<f4v*>(p));
}
__device__ __forceinline__ float max4(float4 a) { return fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)); }
__device__ __forceinline__ float sumexp4(float4 a, float m) {
    return (__expf(a.x - m) + __expf(a.y - m)) + (__expf(a.z - m) + __expf(a.w - m));
}
__device__ __forceinline__ float4 grad4(float4 a, float m, float inv_sum, float scale, uint32_t c, uint32_t target) {
    return make_float4(grad_of(a.x, m, inv_sum, scale, c == target), grad_of(a.y, m, inv_sum, scale, c + 1 == target),
                       grad_of(a.z, m, inv_sum, scale, c + 2 == target), grad_of(a.w, m, inv_sum, scale, c + 3 == target));
}

constexpr int kStreamAux = 2;            // buffer access cache policy: nontemporal

// One row as a buffer: a scalar descriptor plus one 32-bit byte offset per lane, so the register
// slots need no address registers of their own; reads past the end of the row return zeros and
// stores past it are dropped by the hardware.
struct RowBuf {
    __amdgpu_buffer_rsrc_t rsrc;
    __device__ __forceinline__ RowBuf(const float* row, int64_t cols) {
        const uint64_t o = reinterpret_cast<uint64_t>(row);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)o), hi = __builtin_amdgcn_readfirstlane((uint32_t)(o >> 32));
        const uint32_t nb = __builtin_amdgcn_readfirstlane((uint32_t)(cols * 4));
        rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uint64_t)hi << 32) | lo), 0, (int)nb, 0x00020000);
    }
    template <int AUX>
    __device__ __forceinline__ float4 load(int lane_off, int slot_off) const {
        return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off, slot_off, AUX));
    }
    __device__ __forceinline__ void store(float4 v, int lane_off, int slot_off) const {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, v),
                                               rsrc, lane_off, slot_off, kStreamAux);
    }
};

constexpr float kLog2e = 1.4426950408889634f;

// exp(x - m) as one fused multiply-add and one exp2: mc = m * log2(e)
__device__ __forceinline__ float4 exp4(float4 a, float mc) {
    return make_float4(__builtin_amdgcn_exp2f(fmaf(a.x, kLog2e, -mc)), __builtin_amdgcn_exp2f(fmaf(a.y, kLog2e, -mc)),
                       __builtin_amdgcn_exp2f(fmaf(a.z, kLog2e, -mc)), __builtin_amdgcn_exp2f(fmaf(a.w, kLog2e, -mc)));
}
__device__ __forceinline__ float sum4(float4 a) { return (a.x + a.y) + (a.z + a.w); }
// e * k, with `scale` taken off the target's component when this is its slot
__device__ __forceinline__ float4 finish4(float4 e, float k, float scale, int i4, uint32_t target) {
    float4 r = make_float4(e.x * k, e.y * k, e.z * k, e.w * k);
    if ((uint32_t)i4 == (target >> 2)) {
        const uint32_t c = target & 3u;
        if (c == 0) r.x -= scale; else if (c == 1) r.y -= scale; else if (c == 2) r.z -= scale; else r.w -= scale;
    }
    return r;
}

template <int BLOCK, bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* lds) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float other = __shfl_xor(v, o, 64);
        v = IS_MAX ? fmaxf(v, other) : v + other;
    }
    if (lane == 0) lds[wv] = v;
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; w++) r = IS_MAX ? fmaxf(r, lds[w]) : r + lds[w];
    return r;
}

// ---------------------------------------------------------------- rows shared out between workgroups
// A row is cut into chunks of 4 KB (one float4 per lane of a 256-lane workgroup); chunk c belongs to part c % P, and P
// workgroups with consecutive indices hold one part each entirely in registers (kCoopVpt float4 per lane), so every
// logit crosses HBM once in each direction and the partners sweep the row side by side.  Four workgroups share a CU
// (while one reduces or waits for its partners the others stream; two of twice the size measured 3.65 ms against
// 3.44).  A part's (max, sum of exponentials against that max) is published through a small record in device memory;
// each workgroup combines its row's P records itself, in part order, so all of them derive the same maximum and total.
//
// The grid is persistent (a multiple of P workgroups, at most four per CU); workgroup g takes units g, g + G, ...
// where unit u = (row u / P, part u % P): the P partners of a row work on it in the same round.  Every unit of a
// launch has a record of its own, written once and never overwritten while the launch runs, tagged (launch, round):
// a tag from another launch never matches.  The wait for a partner is bounded: past the limit (a partner that has
// not been scheduled yet) the workgroup forms that part's statistics itself from the logits, with the owner's own
// slots per lane, order of additions and reductions, so it arrives at the owner's bits; and it takes the published
// pair instead if that has appeared meanwhile (in place the partner may by then be overwriting its logits with the
// gradient: it publishes before it stores, and what it published stays readable however far ahead it runs).
// Whichever way a workgroup learns a part's statistics, it learns the same two floats.
constexpr int kCoopBlock = 256;
constexpr int kCoopVpt = 19;                         // float4 per lane: 76 of the 128 registers a lane has at four workgroups per CU
constexpr int kCoopWgsPerCu = 4;
constexpr int kCoopMaxParts = 64;                     // one lane of the first wave per partner
constexpr int kCoopMaxGrid = 2048;
constexpr int kCoopLaunchSlots = 4;                   // launches that may be in flight on one device at a time
constexpr int kCoopMaxUnits = 1 << 18;                // (row, part) units per launch; longer inputs go in several launches

// Each word of a record validates itself: (statistic, half of a 64-bit hash of (launch, round)).  No ordering between
// the two stores or the two loads is needed, hence no release/acquire fence (at device scope those write back and
// invalidate whole caches on this part); the accesses are relaxed device-scope atomics, which go past the per-XCD L2s.
struct CoopRec { unsigned long long max_word; unsigned long long sum_word; };
static __device__ CoopRec g_ce_records[kCoopLaunchSlots][kCoopMaxUnits];

__device__ __forceinline__ unsigned long long coop_tag(unsigned launch, unsigned round) {
    unsigned long long z = (((unsigned long long)launch << 32) | round) + 0x9e3779b97f4a7c15ull;      // splitmix64
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
__device__ __forceinline__ void coop_publish(CoopRec* rec, float m, float sum, unsigned long long tag) {
    __hip_atomic_store(&rec->max_word, (tag << 32) | __float_as_uint(m), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&rec->sum_word, (tag & 0xffffffff00000000ull) | __float_as_uint(sum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool coop_try_read(const CoopRec* rec, unsigned long long tag, MaxSum* out) {
    const unsigned long long a = __hip_atomic_load(&rec->max_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long b = __hip_atomic_load(&rec->sum_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((a >> 32) != (tag & 0xffffffffull) || (b >> 32) != (tag >> 32)) return false;
    out->m = __uint_as_float((unsigned)a);
    out->s = __uint_as_float((unsigned)b);
    return true;
}

__global__ __launch_bounds__(kCoopBlock, kCoopWgsPerCu) void ce_coop_kernel(const float* __restrict__ logits,
                                                               const uint32_t* __restrict__ targets,
                                                               float* __restrict__ grad, float* __restrict__ loss_rows,
                                                               const uint32_t* __restrict__ seq_starts, int batch,
                                                               int64_t row_begin, int64_t row_end, int64_t cols, float scale, int P,
                                                               CoopRec* __restrict__ recs, unsigned launch, int spin_limit,
                                                               int in_place) {
    __shared__ float red[2][kCoopBlock / 64];
    __shared__ MaxSum parts[kCoopMaxParts];
    __shared__ unsigned long long missing;
    __shared__ float bcast[2];
    constexpr int kChunkBytes = kCoopBlock * 16;                   // one slot of every lane: 4 KB of the row
    const int G = gridDim.x;
    const int n4 = (int)(cols >> 2);
    const int part = (int)(blockIdx.x % P);
    // Chunk c of the row belongs to part c % P: the P partners sweep the row side by side, and slot k of this
    // workgroup is chunk k P + part.  A slot whose chunk lies past the end of the row reads zeros and its store is
    // dropped (the row is addressed as a buffer), so no slot needs a test of its own.
    const int lane_off = threadIdx.x * 16;
    const int step_bytes = P * kChunkBytes, first_bytes = part * kChunkBytes;
    const float4 pad = make_float4(kNegBig, kNegBig, kNegBig, kNegBig);
    const int64_t unit0 = row_begin * P, units = row_end * P;     // this launch's units: records are indexed by u - unit0
    auto is_live = [&](int64_t r) { return r < row_end && (int64_t)targets[r] < cols && row_live(seq_starts, batch, r); };

    float4 v[kCoopVpt];
    bool loaded = false;
    unsigned round = 0;
    for (int64_t u = unit0 + blockIdx.x; u < units; u += G, round++) {
        const int64_t row = u / P;
        const RowBuf x(logits + row * cols, cols), g(grad + row * cols, cols);
        if (!is_live(row)) {
            for (int k = 0; k < kCoopVpt; k++) g.store(make_float4(0, 0, 0, 0), lane_off, first_bytes + k * step_bytes);
            if (part == 0 && threadIdx.x == 0) loss_rows[row] = 0.0f;
            loaded = false;
            continue;
        }
        const uint32_t target = targets[row];
        if (!loaded) {
            int off = first_bytes;                                // a running scalar offset, kept opaque so that the
#pragma unroll                                                    // compiler does not hold one scalar register per slot
            for (int k = 0; k < kCoopVpt; k++) {
                v[k] = x.load<kStreamAux>(lane_off, off);
                off += step_bytes;
                asm volatile("" : "+s"(off));
            }
        }
        // the target's logit, read by the part that owns it before any of this workgroup's stores (grad may alias logits)
        const bool owns_target = ((int)(target >> 2) / kCoopBlock) % P == part;
        float xt = 0.0f;
        if (owns_target && threadIdx.x == 0) xt = logits[row * cols + target];
        float mx = kNegBig;
        {
            int room = n4 - part * kCoopBlock;                    // float4 slots from this chunk's start to the end of the row
#pragma unroll
            for (int k = 0; k < kCoopVpt; k++) {
                if ((int)threadIdx.x >= room) v[k] = pad;         // past the end (read as zeros): out of the maximum and the sum
                mx = fmaxf(mx, max4(v[k]));
                room -= P * kCoopBlock;
                asm volatile("" : "+s"(room));
            }
        }
        MaxSum mine;
        mine.m = block_reduce<kCoopBlock, true>(mx, red[0]);
        const float mc = mine.m * kLog2e;
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < kCoopVpt; k++) { v[k] = exp4(v[k], mc); sum += sum4(v[k]); }    // padding: exp(-huge) = 0
        mine.s = block_reduce<kCoopBlock, false>(sum, red[1]);

        float m = mine.m, total = mine.s;
        if (P > 1) {
            const unsigned long long tag = coop_tag(launch, round);
            CoopRec* row_recs = recs + (row - row_begin) * P;     // the row's P records, one per part
            if (threadIdx.x == 0) {
                missing = 0ull;
                coop_publish(row_recs + part, mine.m, mine.s, tag);
                // In place the gradient will overwrite this part's logits: the record has to be out before that, for a
                // partner that gave up waiting and is reading these logits (it looks at the record again afterwards).
                if (in_place) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __syncthreads();
            if (threadIdx.x < (unsigned)P) {                      // one lane per partner (its own part included)
                const CoopRec* rec = row_recs + threadIdx.x;
                MaxSum got;
                bool ok = coop_try_read(rec, tag, &got);
                for (int spin = 0; !ok && spin < spin_limit; spin++) {
                    __builtin_amdgcn_s_sleep(4);
                    ok = coop_try_read(rec, tag, &got);
                }
                if (ok) parts[threadIdx.x] = got;
                else atomicOr(&missing, 1ull << threadIdx.x);
            }
            __syncthreads();
            unsigned long long todo = missing;
            while (todo) {                                        // uniform across the workgroup
                const int p = __builtin_ctzll(todo);
                todo &= todo - 1;
                // That part's statistics from its logits, formed as its owner forms them: lane t takes the same
                // slots (chunks p, p + P, ...) in the same order, and the two reductions are the owner's.  Two sweeps
                // over memory: the registers hold this workgroup's own part.
                const float4* src = reinterpret_cast<const float4*>(logits + row * cols);
                float pm = kNegBig;
#pragma unroll 1
                for (int k = 0; k < kCoopVpt; k++) {
                    const int i4 = (p + k * P) * kCoopBlock + (int)threadIdx.x;
                    if (i4 < n4) pm = fmaxf(pm, max4(src[i4]));
                }
                MaxSum ms;
                ms.m = block_reduce<kCoopBlock, true>(pm, red[0]);
                const float pmc = ms.m * kLog2e;
                float ps = 0.0f;
#pragma unroll 1
                for (int k = 0; k < kCoopVpt; k++) {
                    const int i4 = (p + k * P) * kCoopBlock + (int)threadIdx.x;
                    ps += sum4(exp4(i4 < n4 ? src[i4] : pad, pmc));
                }
                ms.s = block_reduce<kCoopBlock, false>(ps, red[1]);
                if (threadIdx.x == 0) {                           // (after the reductions' barriers: every lane's loads have returned)
                    MaxSum got;
                    parts[p] = coop_try_read(row_recs + p, tag, &got) ? got : ms;
                }
                __syncthreads();
            }
            if (threadIdx.x < 64) {                               // first wave: combine in part order
                MaxSum r = parts[0];
                for (int p = 1; p < P; p++) r = combine(r, parts[p]);
                if (threadIdx.x == 0) { bcast[0] = r.m; bcast[1] = r.s; }
            }
            __syncthreads();
            m = bcast[0]; total = bcast[1];
        }
        const float k_out = (scale / total) * __expf(mine.m - m);
        if (owns_target && threadIdx.x == 0) loss_rows[row] = -((xt - m) - __logf(total));

        const int64_t next = u + G;
        const bool refill = next < units && is_live(next / P);
        const RowBuf xn(logits + (refill ? next / P : row) * cols, cols);
        int off = first_bytes, i4 = part * kCoopBlock + (int)threadIdx.x;
#pragma unroll
        for (int k = 0; k < kCoopVpt; k++) {
            g.store(finish4(v[k], k_out, scale, i4, target), lane_off, off);   // dropped past the row's end
            if (refill) v[k] = xn.load<kStreamAux>(lane_off, off);
            off += step_bytes; i4 += P * kCoopBlock;
            asm volatile("" : "+s"(off));
        }
        loaded = refill;
    }
}

// ---------------------------------------------------------------- streamed rows
template <int BLOCK, bool VEC>
__global__ __launch_bounds__(BLOCK) void ce_stream_kernel(const float* __restrict__ logits,
                                                          const uint32_t* __restrict__ targets,
                                                          float* __restrict__ grad, float* __restrict__ loss_rows,
                                                          const uint32_t* __restrict__ seq_starts, int batch,
                                                          int64_t cols, float scale) {
    extern __shared__ char dyn_lds[];        // optional padding that caps workgroups per CU
    __shared__ MaxSum lds[BLOCK / 64];
    const int64_t row = blockIdx.x;
    const uint32_t target = targets[row];
    const float* xrow = logits + row * cols;
    float* grow = grad + row * cols;
    const int64_t n4 = VEC ? cols >> 2 : 0;
    const bool live = (int64_t)target < cols && row_live(seq_starts, batch, row);
    if (!live) {
        if (VEC) for (int64_t i4 = threadIdx.x; i4 < n4; i4 += BLOCK) reinterpret_cast<float4*>(grow)[i4] = make_float4(0, 0, 0, 0);
        for (int64_t c = n4 * 4 + threadIdx.x; c < cols; c += BLOCK) grow[c] = 0.0f;
        if (threadIdx.x == 0) loss_rows[row] = 0.0f;
        return;
    }

    // sweep 1: online (max, sum exp) per lane, four float4 in flight
    MaxSum ms;
    ms.m = kNegBig;
    ms.s = 0.0f;
    if (VEC) {
        const float4* xr = reinterpret_cast<const float4*>(xrow);
        int64_t i4 = threadIdx.x;
        for (; i4 + 3 * BLOCK < n4; i4 += 4 * BLOCK) {
            float4 a = xr[i4], b = xr[i4 + BLOCK], c = xr[i4 + 2 * BLOCK], d = xr[i4 + 3 * BLOCK];
            float cm = fmaxf(fmaxf(fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)), fmaxf(fmaxf(b.x, b.y), fmaxf(b.z, b.w))),
                             fmaxf(fmaxf(fmaxf(c.x, c.y), fmaxf(c.z, c.w)), fmaxf(fmaxf(d.x, d.y), fmaxf(d.z, d.w))));
            if (cm > ms.m) { ms.s *= __expf(ms.m - cm); ms.m = cm; }
            float m = ms.m;
            ms.s += (__expf(a.x - m) + __expf(a.y - m) + __expf(a.z - m) + __expf(a.w - m))
                  + (__expf(b.x - m) + __expf(b.y - m) + __expf(b.z - m) + __expf(b.w - m))
                  + (__expf(c.x - m) + __expf(c.y - m) + __expf(c.z - m) + __expf(c.w - m))
                  + (__expf(d.x - m) + __expf(d.y - m) + __expf(d.z - m) + __expf(d.w - m));
        }
        for (; i4 < n4; i4 += BLOCK) {
            float4 a = xr[i4];
            float cm = fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w));
            if (cm > ms.m) { ms.s *= __expf(ms.m - cm); ms.m = cm; }
            float m = ms.m;
            ms.s += __expf(a.x - m) + __expf(a.y - m) + __expf(a.z - m) + __expf(a.w - m);
        }
    }
    for (int64_t c = n4 * 4 + threadIdx.x; c < cols; c += BLOCK) {
        float a = xrow[c];
        if (a > ms.m) { ms.s *= __expf(ms.m - a); ms.m = a; }
        ms.s += __expf(a - ms.m);
    }
    ms = block_combine<BLOCK>(ms, lds);      // contains the barrier that orders sweep 1 before sweep 2's stores
    const float inv_sum = 1.0f / ms.s;
    if (threadIdx.x == 0) loss_rows[row] = -((xrow[target] - ms.m) - __logf(ms.s));
    __syncthreads();                         // grad may alias logits: the target logit is read before any store

    // sweep 2: gradient, walking back from the end of the row
    for (int64_t c = cols - 1 - threadIdx.x; c >= n4 * 4; c -= BLOCK)
        grow[c] = grad_of(xrow[c], ms.m, inv_sum, scale, (uint32_t)c == target);
    if (VEC) {
        const float4* xr = reinterpret_cast<const float4*>(xrow);
        float4* gr = reinterpret_cast<float4*>(grow);
        int64_t i4 = n4 - 1 - threadIdx.x;
        for (; i4 - 3 * BLOCK >= 0; i4 -= 4 * BLOCK) {
            float4 q[4];
#pragma unroll
            for (int u = 0; u < 4; u++) q[u] = xr[i4 - u * BLOCK];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                uint32_t c = (uint32_t)((i4 - u * BLOCK) * 4);
                gr[i4 - u * BLOCK] = make_float4(grad_of(q[u].x, ms.m, inv_sum, scale, c == target),
                                                 grad_of(q[u].y, ms.m, inv_sum, scale, c + 1 == target),
                                                 grad_of(q[u].z, ms.m, inv_sum, scale, c + 2 == target),
                                                 grad_of(q[u].w, ms.m, inv_sum, scale, c + 3 == target));
            }
        }
        for (; i4 >= 0; i4 -= BLOCK) {
            float4 a = xr[i4];
            uint32_t c = (uint32_t)(i4 * 4);
            gr[i4] = make_float4(grad_of(a.x, ms.m, inv_sum, scale, c == target),
                                 grad_of(a.y, ms.m, inv_sum, scale, c + 1 == target),
                                 grad_of(a.z, ms.m, inv_sum, scale, c + 2 == target),
                                 grad_of(a.w, ms.m, inv_sum, scale, c + 3 == target));
        }
    }
}

// device address of the exchange records on the current device
static int coop_records(CoopRec** out) {
    static std::mutex mu;
    static CoopRec* base[64] = {nullptr};
    int dev = 0;
    SERAPH_HIP_CHECK(hipGetDevice(&dev));
    SERAPH_REQUIRE(dev >= 0 && dev < 64, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lk(mu);
    if (!base[dev]) SERAPH_HIP_CHECK(hipGetSymbolAddress((void**)&base[dev], HIP_SYMBOL(g_ce_records)));
    *out = base[dev];
    return SERAPH_OK;
}

static int g_ce_spin_limit = 1 << 16;     // waits of ~0.3 us each: several milliseconds before a partner is given up on

}  // namespace seraph

using namespace seraph;

extern "C" void seraph_cross_entropy_exchange_spins(int spins) {
    if (spins >= 0) g_ce_spin_limit = spins;
}

extern "C" int seraph_cross_entropy_grad(const float* logits, const uint32_t* targets, float* grad, float* loss_rows,
                                         const uint32_t* seq_starts, int batch,
                                         int64_t rows, int64_t cols, int64_t valid_rows, seraph_stream_t s) {
    if (rows == 0 || cols == 0) return SERAPH_OK;
    SERAPH_REQUIRE(logits && targets && grad && loss_rows, "cross_entropy_grad: NULL pointer");
    SERAPH_REQUIRE(rows > 0 && cols > 0 && rows <= 0x7fffffff && cols <= 0x7fffffff,
                   "cross_entropy_grad: bad shape %lld x %lld", (long long)rows, (long long)cols);
    SERAPH_REQUIRE(!seq_starts || batch >= 1, "cross_entropy_grad: packed call needs batch >= 1");
    const float scale = valid_rows > 0 ? 1.0f / (float)valid_rows : 0.0f;      // cross_entropy_grad.comp:85
    hipStream_t st = as_stream(s);
    const bool vec = (cols % 4 == 0) && aligned16(logits) && aligned16(grad);
    const dim3 grid((unsigned)rows);
    if (vec && cols <= 32768) {
        int64_t n4 = cols / 4;
#define SMALL(V) hipLaunchKernelGGL((ce_small_kernel<256, V>), grid, dim3(256), 0, st, logits, targets, grad, loss_rows, seq_starts, batch, (int)cols, scale)
        if (n4 <= 256) SMALL(1);
        else if (n4 <= 512) SMALL(2);
        else if (n4 <= 1024) SMALL(4);
        else if (n4 <= 2048) SMALL(8);
        else if (n4 <= 4096) SMALL(16);
        else SMALL(32);
#undef SMALL
    } else if (vec && ceil_div(ceil_div(cols / 4, kCoopBlock), kCoopVpt) <= kCoopMaxParts) {
        // rows cut into P register-resident parts: one pass over HBM
        const int P = (int)ceil_div(ceil_div(cols / 4, kCoopBlock), kCoopVpt);
        int64_t G = (int64_t)num_compute_units() * kCoopWgsPerCu;
        if (G > kCoopMaxGrid) G = kCoopMaxGrid;
        G = (G / P) * P;
        static std::atomic<unsigned> launches{0};
        CoopRec* all_recs = nullptr;
        int rc = coop_records(&all_recs);
        if (rc != SERAPH_OK) return rc;
        const int64_t rows_per_launch = kCoopMaxUnits / P;        // every unit of a launch keeps a record of its own
        for (int64_t r0 = 0; r0 < rows; r0 += rows_per_launch) {
            const int64_t r1 = r0 + rows_per_launch < rows ? r0 + rows_per_launch : rows;
            const int64_t g = G > (r1 - r0) * P ? (r1 - r0) * P : G;
            unsigned launch = launches.fetch_add(1) + 1;
            if (launch == 0) launch = launches.fetch_add(1) + 1;  // a zeroed record must never look published
            CoopRec* recs = all_recs + (size_t)(launch % kCoopLaunchSlots) * kCoopMaxUnits;
            hipLaunchKernelGGL(ce_coop_kernel, dim3((unsigned)g), dim3(kCoopBlock), 0, st, logits, targets, grad, loss_rows,
                               seq_starts, batch, r0, r1, cols, scale, P, recs, launch, g_ce_spin_limit, grad == logits ? 1 : 0);
        }
    } else if (vec) {
        // Rows in flight are re-read by the second sweep: keep their total under the last-level cache.
        // Two 1024-lane workgroups fit a CU; when that many long rows would overflow the cache, an
        // LDS reservation of more than half a CU's LDS holds residency to one workgroup per CU.
        const size_t in_flight = (size_t)num_compute_units() * 2 * (size_t)cols * sizeof(float);
        const size_t lds_pad = in_flight > kLastLevelCacheBytes * 3 / 4 ? 84 * 1024 : 0;
        if (lds_pad) {
            static bool attr_set = false;
            if (!attr_set) {
                SERAPH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&ce_stream_kernel<1024, true>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_pad));
                attr_set = true;
            }
        }
        hipLaunchKernelGGL((ce_stream_kernel<1024, true>), grid, dim3(1024), lds_pad, st, logits, targets, grad, loss_rows,
                           seq_starts, batch, cols, scale);
    } else {
        hipLaunchKernelGGL((ce_stream_kernel<256, false>), grid, dim3(256), 0, st, logits, targets, grad, loss_rows,
                           seq_starts, batch, cols, scale);
    }
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}
