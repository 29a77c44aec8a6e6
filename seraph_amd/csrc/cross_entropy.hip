// cross_entropy.hip - fused softmax cross-entropy loss + gradient, one workgroup per row.
//
// Two shapes of the same arithmetic (shaders/cross_entropy_grad.comp:44-98):
//   * rows that fit the workgroup's registers (cols <= 32768) are read from HBM once;
//   * longer rows (a 151936-entry vocabulary is 608 KB, more than LDS holds) take an
//     online max / sum-of-exponentials sweep and then a second sweep in the opposite
//     direction, so the part of the row that was fetched last is revisited first while
//     it is still cache resident; the row's statistics are combined through LDS.
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
