// cross_entropy.hip - fused softmax cross-entropy loss + gradient, one workgroup per row.
//
// Two shapes of the same arithmetic (shaders/cross_entropy_grad.comp:44-98):
//   * rows that fit the workgroup's registers (cols <= 32768) are read from HBM once;
//   * longer rows (a 151936-entry vocabulary is 608 KB) are owned by one 512-lane workgroup that
//     has a CU to itself: the first 77824 columns stay in its registers (38 float4 per lane), the
//     next 32768 in its LDS (128 KB), and only what is left (27 % of that vocabulary) is read a
//     second time, last-fetched-first while it is still cache resident.  HBM sees 2.27 passes
//     instead of 3 (4.5 -> 4.06 ms at 16384 x 151936; a CU still idles while its one row is
//     reduced, which is what separates this from the 3.5 ms the traffic alone would take);
//   * unaligned or odd-length rows take an online max / sum-of-exponentials sweep and a second
//     sweep in the opposite direction.
// Rows without supervision (target >= cols, or the last token of a packed sequence)
// are written as zeros without being read.  All offsets are 64-bit: rows*cols exceeds
// 2^31 at the shapes this runs on.
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

// ---------------------------------------------------------------- rows resident in registers + LDS
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

constexpr int kResBlock = 512;           // 8 waves: two per SIMD, 256 registers each
constexpr int kResVpt = 38;              // float4 per lane held in registers (152 of the 256 a lane has; 40 would spill)
constexpr int kResLds4 = 8192;           // float4 held in LDS (128 KB)
constexpr int kBatch = 8;                // independent loads in flight per lane outside the register part
constexpr int kStreamAux = 2;            // buffer access cache policy: nontemporal

// One row as a buffer: a scalar descriptor plus one 32-bit byte offset per lane, so the 40 register
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

// cols % 4 == 0, 16-byte aligned rows of at most 2^29 columns.  Slot i4 of the row lives in registers
// when i4 < BLOCK*VPT, in LDS when it is one of the next kResLds4, and is read twice otherwise.
// The row maximum is found first; every resident logit is then turned into exp(x - max) once, in
// place, and only scaled when it is stored (the overflow keeps the online form and pays a second
// exponential).  A workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ...; while it stores the
// gradient of one row out of its registers it refills each register, and its LDS slots, with the same
// slots of its next row, so a CU's loads and stores overlap although it holds one row at a time.
__global__ __launch_bounds__(kResBlock) void ce_resident_kernel(const float* __restrict__ logits,
                                                                const uint32_t* __restrict__ targets,
                                                                float* __restrict__ grad, float* __restrict__ loss_rows,
                                                                const uint32_t* __restrict__ seq_starts, int batch,
                                                                int64_t rows, int64_t cols, float scale) {
    __shared__ float4 stash[kResLds4];
    __shared__ float red[2][kResBlock / 64];
    constexpr int kReg4 = kResBlock * kResVpt;
    constexpr int kSlotBytes = kResBlock * 16;               // distance between a lane's consecutive slots
    const int n4 = (int)(cols >> 2);
    const int lds_end = n4 < kReg4 + kResLds4 ? n4 : kReg4 + kResLds4;
    const int lane_off = threadIdx.x * 16;
    const float4 pad = make_float4(kNegBig, kNegBig, kNegBig, kNegBig);
    auto is_live = [&](int64_t r) { return r < rows && (int64_t)targets[r] < cols && row_live(seq_starts, batch, r); };

    // The LDS part travels memory -> LDS without passing through registers: lane l of a wave lands at
    // the wave's base + 16 l, so a lane finds its own slots at stash[u * BLOCK + threadIdx.x].
    typedef __attribute__((address_space(3))) void* lds_ptr;
    auto fetch_stash = [&](const RowBuf& xb) {
#pragma unroll
        for (int u = 0; u < kResLds4 / kResBlock; u++) {
            const int s4 = kReg4 + u * kResBlock;
            if (s4 < lds_end)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xb.rsrc, (lds_ptr)&stash[u * kResBlock + (threadIdx.x & ~63u)], 16, lane_off,
                                                         s4 * 16, 0, kStreamAux);
        }
    };

    float4 v[kResVpt];
    bool loaded = false;                     // v and stash already hold (or are receiving) this row's resident part
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const RowBuf x(logits + row * cols, cols), g(grad + row * cols, cols);
        if (!is_live(row)) {
            for (int b = 0; b * kResBlock < n4; b++) g.store(make_float4(0, 0, 0, 0), lane_off, b * kSlotBytes);
            if (threadIdx.x == 0) loss_rows[row] = 0.0f;
            loaded = false;
            continue;
        }
        const uint32_t target = targets[row];
        if (!loaded) {
#pragma unroll
            for (int k = 0; k < kResVpt; k++) v[k] = x.load<kStreamAux>(lane_off, k * kSlotBytes);
            fetch_stash(x);
        }
        // sweep 1, overflow: online (max, sum of exponentials), kBatch independent loads in flight per lane;
        // read again in sweep 2, so kept cacheable
        MaxSum ms;
        ms.m = kNegBig;
        ms.s = 0.0f;
        for (int b4 = lds_end; b4 < n4; b4 += kBatch * kResBlock) {
            float4 a[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; u++) a[u] = x.load<0>(lane_off, (b4 + u * kResBlock) * 16);
            float cm = ms.m;
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                if (b4 + u * kResBlock + (int)threadIdx.x >= n4) a[u] = pad;
                cm = fmaxf(cm, max4(a[u]));
            }
            if (cm > ms.m) { ms.s *= __expf(ms.m - cm); ms.m = cm; }
            const float mc = ms.m * kLog2e;
            float acc = 0.0f;
#pragma unroll
            for (int u = 0; u < kBatch; u++) acc += sum4(exp4(a[u], mc));       // padding adds exp(-huge) = 0
            ms.s += acc;
        }
        // Everything requested has landed: the register part and, written straight into LDS, this lane's
        // own stash slots.  (Explicit: the wait count the compiler derives for v[] does not include the
        // LDS-bound loads issued after them.)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        float mx = kNegBig;
#pragma unroll
        for (int k = 0; k < kResVpt; k++) {
            if ((int)threadIdx.x + kResBlock * k >= n4) v[k] = pad;
            mx = fmaxf(mx, max4(v[k]));
        }
        for (int i4 = kReg4 + threadIdx.x; i4 < lds_end; i4 += kResBlock) mx = fmaxf(mx, max4(stash[i4 - kReg4]));
        const float m = block_reduce<kResBlock, true>(fmaxf(mx, ms.m), red[0]);
        const float mc = m * kLog2e;
        // every resident logit becomes exp(x - m), once
        float sum = ms.s * __expf(ms.m - m);
#pragma unroll
        for (int k = 0; k < kResVpt; k++) { v[k] = exp4(v[k], mc); sum += sum4(v[k]); }
        for (int i4 = kReg4 + threadIdx.x; i4 < lds_end; i4 += kResBlock) {
            const float4 e = exp4(stash[i4 - kReg4], mc);
            stash[i4 - kReg4] = e;
            sum += sum4(e);
        }
        const float total = block_reduce<kResBlock, false>(sum, red[1]);
        const float k_out = scale / total;
        if (threadIdx.x == 0) loss_rows[row] = -((logits[row * cols + target] - m) - __logf(total));
        __syncthreads();                     // grad may alias logits: the target logit is read before any store

        // sweep 2: the overflow first (most recently fetched first), then LDS, then registers
        for (int e4 = n4; e4 > lds_end; e4 -= kBatch * kResBlock) {
            float4 a[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                const int s4 = e4 - (u + 1) * kResBlock;                      // may reach below lds_end: masked below
                a[u] = x.load<0>(lane_off, (s4 < 0 ? 0 : s4) * 16);
            }
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                const int s4 = e4 - (u + 1) * kResBlock;
                const int i4 = s4 + (int)threadIdx.x;
                if (i4 >= lds_end && i4 < n4) g.store(finish4(exp4(a[u], mc), k_out, scale, i4, target), lane_off, s4 * 16);
            }
        }
        for (int i4 = kReg4 + threadIdx.x; i4 < lds_end; i4 += kResBlock)
            g.store(finish4(stash[i4 - kReg4], k_out, scale, i4, target), lane_off, (i4 - (int)threadIdx.x) * 16);
        const int64_t next = row + gridDim.x;
        const bool refill = is_live(next);
        const RowBuf xn(logits + (refill ? next : row) * cols, cols);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this row's LDS slots have been read: they may be overwritten
        if (refill) fetch_stash(xn);
#pragma unroll
        for (int k = 0; k < kResVpt; k++) {
            const int i4 = threadIdx.x + kResBlock * k;
            g.store(finish4(v[k], k_out, scale, i4, target), lane_off, k * kSlotBytes);   // dropped past the row's end
            if (refill) v[k] = xn.load<kStreamAux>(lane_off, k * kSlotBytes);
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

}  // namespace seraph

using namespace seraph;

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
    } else if (vec && cols <= ((int64_t)1 << 29)) {
        const int64_t cus = num_compute_units();          // one workgroup fills a CU's registers and LDS
        hipLaunchKernelGGL(ce_resident_kernel, dim3((unsigned)(rows < cus ? rows : cus)), dim3(kResBlock), 0, st, logits, targets,
                           grad, loss_rows, seq_starts, batch, rows, cols, scale);
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
