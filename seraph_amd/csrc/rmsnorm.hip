// rmsnorm.hip - RMSNorm forward, batched RMSNorm backward with FP64 intermediates,
// and the gain-less all-heads qk_norm with its derivative.
//
// A row (and, going backward, dy) lives in registers as float4 slots while its two sums are
// reduced, so each byte of x / dy / dx crosses HBM exactly once.  Short rows (<= 512) are
// owned by one wavefront (wave reductions only, no LDS, no barrier); longer rows by one
// workgroup, two float4 per lane at 2048 columns, which keeps the register footprint small
// enough for four or more waves per SIMD to overlap the FP64 arithmetic with the loads.
// The column reduction for grad_scale is deterministic: a lane keeps per-column partial sums
// over the rows it visits, each workgroup writes one partial row to scratch, and a second
// small kernel adds the partial rows in a fixed order.
#include <mutex>

#include "common.hpp"

namespace seraph {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

// ---------------------------------------------------------------- forward
template <int VPL>
__global__ __launch_bounds__(kBlock) void rmsnorm_fwd_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ addend,   // NULL, or added to x first
                                                             float* __restrict__ sum,            // where x + addend goes
                                                             const float* __restrict__ scale,
                                                             float* __restrict__ y,
                                                             int64_t rows, int cols, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    const int n4 = cols >> 2;
    float4 sc[VPL];
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        int i4 = lane + 64 * k;
        sc[k] = i4 < n4 ? reinterpret_cast<const float4*>(scale)[i4] : make_float4(0, 0, 0, 0);
    }
    for (int64_t row = wave; row < rows; row += nwaves) {
        const float4* xr = reinterpret_cast<const float4*>(x + row * cols);
        float4 v[VPL];
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            int i4 = lane + 64 * k;
            v[k] = i4 < n4 ? xr[i4] : make_float4(0, 0, 0, 0);
            if (addend && i4 < n4) {
                const float4 b = reinterpret_cast<const float4*>(addend + row * cols)[i4];
                v[k] = make_float4(v[k].x + b.x, v[k].y + b.y, v[k].z + b.z, v[k].w + b.w);
                reinterpret_cast<float4*>(sum + row * cols)[i4] = v[k];
            }
            ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        }
        ss = wave_sum(ss);
        float inv = rsqrtf(ss / (float)cols + eps);       // shaders/rmsnorm.comp: inversesqrt(mean_sq + eps)
        float4* yr = reinterpret_cast<float4*>(y + row * cols);
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            int i4 = lane + 64 * k;
            if (i4 < n4)
                yr[i4] = make_float4(v[k].x * inv * sc[k].x, v[k].y * inv * sc[k].y,
                                     v[k].z * inv * sc[k].z, v[k].w * inv * sc[k].w);
        }
    }
}

// Any cols / alignment: the row is read twice (the second read is served by cache).
__global__ __launch_bounds__(kBlock) void rmsnorm_fwd_generic_kernel(const float* __restrict__ x,
                                                                     const float* __restrict__ addend,
                                                                     float* __restrict__ sum,
                                                                     const float* __restrict__ scale,
                                                                     float* __restrict__ y,
                                                                     int64_t rows, int64_t cols, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t row = wave; row < rows; row += nwaves) {
        const float* xr = x + row * cols;
        if (addend) {                                     // the sum is stored first and then normalised like any input
            for (int64_t c = lane; c < cols; c += 64) sum[row * cols + c] = xr[c] + addend[row * cols + c];
            xr = sum + row * cols;                        // each lane rereads only what it wrote
        }
        float ss = 0.0f;
        for (int64_t c = lane; c < cols; c += 64) ss += xr[c] * xr[c];
        ss = wave_sum(ss);
        float inv = rsqrtf(ss / (float)cols + eps);
        for (int64_t c = lane; c < cols; c += 64) y[row * cols + c] = xr[c] * inv * scale[c];
    }
}

// ---------------------------------------------------------------- backward
// Row statistics of shaders/rmsnorm_backward_batch.comp:44-79 in double.
struct RowStats { double inv, k; };     // 1/rms and coupled/rms^3
__device__ __forceinline__ RowStats row_stats(double ssq, double cp, int64_t cols, float eps) {
    double denom = cols > 1 ? (double)cols : 1.0;         // max(1.0, cols)
    double rms = sqrt(ssq / denom + (double)eps);
    rms = fmax(rms, 0.01);                                // floor, :59
    double inv = 1.0 / rms;
    RowStats r;
    r.inv = inv;
    r.k = (cp / denom) * (inv * inv * inv);               // coupled * inv_rms3, :79,:98
    return r;
}

template <int VPL>
__global__ __launch_bounds__(kBlock) void rmsnorm_bwd_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ scale,
                                                             const float* __restrict__ dy,
                                                             const float* res,              // NULL, or added to dx (may be dx itself)
                                                             float* dx,
                                                             float* __restrict__ partial,   // [gridDim.x, cols]
                                                             int64_t rows, int cols, float eps) {
    extern __shared__ float lds[];                        // [kWavesPerBlock, cols]
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + wv;
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    const int n4 = cols >> 2;

    float4 sc[VPL], gs[VPL];
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        int i4 = lane + 64 * k;
        sc[k] = i4 < n4 ? reinterpret_cast<const float4*>(scale)[i4] : make_float4(0, 0, 0, 0);
        gs[k] = make_float4(0, 0, 0, 0);
    }

    // The next row is requested before the current one is reduced: a wave has few rows (two at 2048 x 512), and
    // without this each pays the full memory latency in turn.
    float4 xv[VPL], gv[VPL], rv[VPL];
    auto request = [&](int64_t row, float4* xo, float4* go, float4* ro) {
        const bool live = row < rows;
        const int64_t at = live ? row * cols : 0;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            const int i4 = lane + 64 * k;
            const bool in = live && i4 < n4;
            xo[k] = in ? reinterpret_cast<const float4*>(x + at)[i4] : make_float4(0, 0, 0, 0);
            go[k] = in ? reinterpret_cast<const float4*>(dy + at)[i4] : make_float4(0, 0, 0, 0);
            ro[k] = (res && in) ? reinterpret_cast<const float4*>(res + at)[i4] : make_float4(0, 0, 0, 0);
        }
    };
    request(wave, xv, gv, rv);
    for (int64_t row = wave; row < rows; row += nwaves) {
        float4 xn[VPL], gn[VPL], rn[VPL];
        request(row + nwaves, xn, gn, rn);
        double ssq = 0.0, cp = 0.0;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            const float* xs = &xv[k].x; const float* g = &gv[k].x; const float* s = &sc[k].x;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                double xd = (double)xs[e];
                ssq += xd * xd;
                cp += (double)g[e] * (double)s[e] * xd;
            }
        }
        ssq = wave_sum(ssq);
        cp = wave_sum(cp);
        RowStats st = row_stats(ssq, cp, cols, eps);
        float4* dr = reinterpret_cast<float4*>(dx + row * cols);
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            int i4 = lane + 64 * k;
            const float* xs = &xv[k].x; const float* g = &gv[k].x; const float* s = &sc[k].x;
            float o[4]; float* acc = &gs[k].x;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                double xd = (double)xs[e], gd = (double)g[e];
                acc[e] += (float)(gd * xd * st.inv);                                 // :90
                o[e] = (float)(gd * (double)s[e] * st.inv - xd * st.k);              // :98
            }
            if (i4 < n4) dr[i4] = make_float4(rv[k].x + o[0], rv[k].y + o[1], rv[k].z + o[2], rv[k].w + o[3]);
        }
#pragma unroll
        for (int k = 0; k < VPL; k++) { xv[k] = xn[k]; gv[k] = gn[k]; rv[k] = rn[k]; }
    }

    // combine the block's waves, then one partial row per block
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        int i4 = lane + 64 * k;
        if (i4 < n4) reinterpret_cast<float4*>(lds + (size_t)wv * cols)[i4] = gs[k];
    }
    __syncthreads();
    for (int i4 = threadIdx.x; i4 < n4; i4 += kBlock) {
        float4 a = reinterpret_cast<float4*>(lds)[i4];
#pragma unroll
        for (int w = 1; w < kWavesPerBlock; w++) {
            float4 b = reinterpret_cast<float4*>(lds + (size_t)w * cols)[i4];
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        reinterpret_cast<float4*>(partial + (size_t)blockIdx.x * cols)[i4] = a;
    }
}

// Rows of up to 8192 columns: one workgroup per row, VPL float4 per lane.  The four waves
// exchange their two partial sums through a double-buffered LDS slot, one barrier per row.
// x, dy and dx are streamed (nontemporal): each is touched exactly once (5.1 -> 5.8 TB/s on cold
// 16384 x 2048 operands).  PREFETCH requests the next row before the current one is reduced; it
// measured no better (the four workgroups per CU already overlap each other's phases) and is off.
typedef float f4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ldnt4(const float4* p) {
    const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stnt4(float4* p, float4 v) {
    const f4v r = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(r, reinterpret_cast<f4v*>(p));
}

template <int VPL, int AHEAD>
__global__ __launch_bounds__(kBlock) void rmsnorm_bwd_block_kernel(const float* __restrict__ x,
                                                                   const float* __restrict__ scale,
                                                                   const float* __restrict__ dy,
                                                                   const float* res,              // NULL, or added to dx (may be dx itself)
                                                                   float* dx,
                                                                   float* __restrict__ partial,   // [gridDim.x, cols]
                                                                   int64_t rows, int cols, float eps) {
    __shared__ double red[2][kWavesPerBlock][2];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n4 = cols >> 2;
    float4 gs[VPL];
    double sd[VPL][4];                                            // the gains, widened once
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        int i4 = threadIdx.x + kBlock * k;
        const float4 sc = i4 < n4 ? reinterpret_cast<const float4*>(scale)[i4] : make_float4(0, 0, 0, 0);
        sd[k][0] = (double)sc.x; sd[k][1] = (double)sc.y; sd[k][2] = (double)sc.z; sd[k][3] = (double)sc.w;
        gs[k] = make_float4(0, 0, 0, 0);
    }
    struct Row { float4 x[VPL], g[VPL], r[VPL]; };
    auto fetch = [&](Row& b, int64_t row) {
        const float4* xr = reinterpret_cast<const float4*>(x + row * cols);
        const float4* gr = reinterpret_cast<const float4*>(dy + row * cols);
        const float4* rr = reinterpret_cast<const float4*>(res + row * cols);
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            int i4 = threadIdx.x + kBlock * k;
            b.x[k] = i4 < n4 ? ldnt4(xr + i4) : make_float4(0, 0, 0, 0);
            b.g[k] = i4 < n4 ? ldnt4(gr + i4) : make_float4(0, 0, 0, 0);
            b.r[k] = (res && i4 < n4) ? ldnt4(rr + i4) : make_float4(0, 0, 0, 0);
        }
    };
    // a row's residual is read with the row, and a workgroup's rows are fetched in the order it stores them, so dx may be
    // the residual itself
    auto process = [&](const Row& b, int64_t row, int it) {
        // Every value is widened once and kept: x, dy and dy * scale are needed on both sides of the barrier.
        double xd[VPL][4], gd[VPL][4], td[VPL][4];
        double ssq = 0.0, cp = 0.0;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            const float* xs = &b.x[k].x; const float* g = &b.g[k].x;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                xd[k][e] = (double)xs[e];
                gd[k][e] = (double)g[e];
                td[k][e] = gd[k][e] * sd[k][e];
                ssq += xd[k][e] * xd[k][e];
                cp += td[k][e] * xd[k][e];                                           // dy * scale * x, :70
            }
        }
        ssq = wave_sum(ssq);
        cp = wave_sum(cp);
        if (lane == 0) { red[it][wv][0] = ssq; red[it][wv][1] = cp; }
        __syncthreads();
        ssq = (red[it][0][0] + red[it][1][0]) + (red[it][2][0] + red[it][3][0]);
        cp = (red[it][0][1] + red[it][1][1]) + (red[it][2][1] + red[it][3][1]);
        RowStats st = row_stats(ssq, cp, cols, eps);
        float4* dr = reinterpret_cast<float4*>(dx + row * cols);
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            int i4 = threadIdx.x + kBlock * k;
            float o[4]; float* acc = &gs[k].x;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                acc[e] += (float)(gd[k][e] * xd[k][e] * st.inv);                     // :90
                o[e] = (float)(td[k][e] * st.inv - xd[k][e] * st.k);                 // :98
            }
            const float4 ov = make_float4(b.r[k].x + o[0], b.r[k].y + o[1], b.r[k].z + o[2], b.r[k].w + o[3]);
            if (i4 < n4) stnt4(dr + i4, ov);
        }
    };
    const int64_t G = gridDim.x;
    int64_t row = blockIdx.x;
    if (AHEAD == 1) {
        // the next row's loads are issued before the current row's arithmetic (FP64: a third of the kernel's time if
        // nothing else ran beside it); two register sets take turns, so no row is ever copied
        Row a, b;
        if (row < rows) fetch(a, row);
        while (row < rows) {
            if (row + G < rows) fetch(b, row + G);
            process(a, row, 0);
            row += G;
            if (row >= rows) break;
            if (row + G < rows) fetch(a, row + G);
            process(b, row, 1);
            row += G;
        }
    } else {
        Row a;
        int it = 0;
        if (row < rows) fetch(a, row);
        for (; row < rows; row += G, it ^= 1) {
            process(a, row, it);
            if (row + G < rows) fetch(a, row + G);
        }
    }
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        int i4 = threadIdx.x + kBlock * k;
        if (i4 < n4) reinterpret_cast<float4*>(partial + (size_t)blockIdx.x * cols)[i4] = gs[k];
    }
}

// Generic shape: one wave per row, scalar accesses, per-wave partial rows in scratch.
__global__ __launch_bounds__(kBlock) void rmsnorm_bwd_generic_kernel(const float* __restrict__ x,
                                                                     const float* __restrict__ scale,
                                                                     const float* __restrict__ dy,
                                                                     const float* res,              // NULL, or added to dx (may be dx itself)
                                                                     float* dx,
                                                                     float* __restrict__ partial,   // [nwaves, cols], zeroed
                                                                     int64_t rows, int64_t cols, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    float* mine = partial + wave * cols;
    for (int64_t row = wave; row < rows; row += nwaves) {
        const float* xr = x + row * cols;
        const float* gr = dy + row * cols;
        double ssq = 0.0, cp = 0.0;
        for (int64_t c = lane; c < cols; c += 64) {
            double xd = (double)xr[c];
            ssq += xd * xd;
            cp += (double)gr[c] * (double)scale[c] * xd;
        }
        ssq = wave_sum(ssq);
        cp = wave_sum(cp);
        RowStats st = row_stats(ssq, cp, cols, eps);
        for (int64_t c = lane; c < cols; c += 64) {
            double xd = (double)xr[c], gd = (double)gr[c];
            mine[c] += (float)(gd * xd * st.inv);          // same lane revisits the same column: no race
            const float o = (float)(gd * (double)scale[c] * st.inv - xd * st.k);
            dx[row * cols + c] = res ? res[row * cols + c] + o : o;
        }
    }
}

// grad_scale[c] += sum over partial rows in a fixed order.  64 columns x 64 row groups per workgroup when the width
// allows 16-byte loads (a lane takes four columns of rows g, g + 64, ..., all loads in flight, added in double in row
// order; the 64 group sums are then combined in group order), else 64 columns x 16 row groups with scalar loads.
template <bool VEC>
__device__ __forceinline__ void colsum_add_body(const float* __restrict__ partial, int nparts,
                                                int64_t cols, float* __restrict__ grad_scale) {
    constexpr int GROUPS = VEC ? 64 : 16;
    __shared__ double part[GROUPS][64];
    double t4[4] = {0.0, 0.0, 0.0, 0.0};
    int g, cx;
    if (VEC) {
        cx = (threadIdx.x & 15) * 4; g = threadIdx.x >> 4;
        const int64_t c = (int64_t)blockIdx.x * 64 + cx;
        if (c < cols) {
            int p = g;
            for (; p + 7 * GROUPS < nparts; p += 8 * GROUPS) {
                float4 a[8];
#pragma unroll
                for (int u = 0; u < 8; u++) a[u] = *reinterpret_cast<const float4*>(partial + (size_t)(p + GROUPS * u) * cols + c);
#pragma unroll
                for (int u = 0; u < 8; u++) { t4[0] += (double)a[u].x; t4[1] += (double)a[u].y; t4[2] += (double)a[u].z; t4[3] += (double)a[u].w; }
            }
            for (; p < nparts; p += GROUPS) {
                const float4 a = *reinterpret_cast<const float4*>(partial + (size_t)p * cols + c);
                t4[0] += (double)a.x; t4[1] += (double)a.y; t4[2] += (double)a.z; t4[3] += (double)a.w;
            }
        }
#pragma unroll
        for (int e = 0; e < 4; e++) part[g][cx + e] = t4[e];
    } else {
        cx = threadIdx.x & 63; g = threadIdx.x >> 6;
        const int64_t c = (int64_t)blockIdx.x * 64 + cx;
        double s = 0.0;
        if (c < cols) {
            int p = g;
            for (; p + 15 * 16 < nparts; p += 16 * 16) {          // sixteen loads in flight, added in row order
                float a[16];
#pragma unroll
                for (int u = 0; u < 16; u++) a[u] = partial[(size_t)(p + 16 * u) * cols + c];
#pragma unroll
                for (int u = 0; u < 16; u++) s += (double)a[u];
            }
            for (; p < nparts; p += 16) s += (double)partial[(size_t)p * cols + c];
        }
        part[g][cx] = s;
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        const int64_t c = (int64_t)blockIdx.x * 64 + threadIdx.x;
        if (c < cols) {
            double t = 0.0;
#pragma unroll
            for (int k = 0; k < GROUPS; k++) t += part[k][threadIdx.x];
            grad_scale[c] = (float)((double)grad_scale[c] + t);
        }
    }
}

template <bool VEC>
__global__ __launch_bounds__(1024) void colsum_add_kernel(const float* __restrict__ partial, int nparts,
                                                           int64_t cols, float* __restrict__ grad_scale) {
    colsum_add_body<VEC>(partial, nparts, cols, grad_scale);
}

// The column sums of several backward passes of one width in one launch (grid y = the pass): a step driver whose
// norms are small lets their partial rows lie until the end of its backward and folds them all here, which takes
// one launch per norm off its chain of dependent kernels.  Each pass is summed exactly as colsum_add_kernel does it.
constexpr int kMaxColsumJobs = 64;
struct ColsumJobs {
    const float* partial[kMaxColsumJobs];
    float* grad_scale[kMaxColsumJobs];
    int nparts[kMaxColsumJobs];
};
template <bool VEC>
__global__ __launch_bounds__(1024) void colsum_add_multi_kernel(ColsumJobs jobs, int64_t cols) {
    colsum_add_body<VEC>(jobs.partial[blockIdx.y], jobs.nparts[blockIdx.y], cols, jobs.grad_scale[blockIdx.y]);
}

// ---------------------------------------------------------------- qk_norm
// shaders/qk_norm.comp:38-75: y = x / max(sqrt(mean(x^2)), eps) over all heads of a token, in place.  One wavefront
// per token holds the token's n = heads * head_dim values in registers (16-byte streamed accesses, no LDS); rms_out,
// when given, receives the unclamped root mean square for the backward.
template <int VPL>
__global__ __launch_bounds__(kBlock) void qk_norm_vec_kernel(float* __restrict__ qk, float* __restrict__ rms_out,
                                                             int64_t T, int n, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (t >= T) return;
    const int n4 = n >> 2;
    float4* row = reinterpret_cast<float4*>(qk + t * n);
    float4 v[VPL];
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        const int i4 = lane + 64 * k;
        v[k] = i4 < n4 ? ldnt4(row + i4) : make_float4(0, 0, 0, 0);
        ss += (v[k].x * v[k].x + v[k].y * v[k].y) + (v[k].z * v[k].z + v[k].w * v[k].w);
    }
    ss = wave_sum(ss);
    const float rms = sqrtf(ss / (float)n);
    const float inv = 1.0f / fmaxf(rms, eps);
    if (rms_out && lane == 0) rms_out[t] = rms;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        const int i4 = lane + 64 * k;
        if (i4 < n4) stnt4(row + i4, make_float4(v[k].x * inv, v[k].y * inv, v[k].z * inv, v[k].w * inv));
    }
}

__global__ __launch_bounds__(kBlock) void qk_norm_kernel(float* __restrict__ qk, float* __restrict__ rms_out, int64_t T, int64_t n, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t t = wave; t < T; t += nwaves) {
        float* xr = qk + t * n;
        float ss = 0.0f;
        for (int64_t c = lane; c < n; c += 64) ss += xr[c] * xr[c];
        ss = wave_sum(ss);
        const float rms = sqrtf(ss / (float)n);
        if (rms_out && lane == 0) rms_out[t] = rms;
        float inv = 1.0f / fmaxf(rms, eps);
        for (int64_t c = lane; c < n; c += 64) xr[c] *= inv;
    }
}

// d/dx of the above from the input: dx = dy/r - x (dy.x)/(n r^3) while r = rms > eps; dx = dy/eps when clamped.
__global__ __launch_bounds__(kBlock) void qk_norm_bwd_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                             float* __restrict__ dx, int64_t T, int64_t n, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t t = wave; t < T; t += nwaves) {
        const float* xr = x + t * n;
        const float* gr = dy + t * n;
        float ss = 0.0f, gx = 0.0f;
        for (int64_t c = lane; c < n; c += 64) { ss += xr[c] * xr[c]; gx += gr[c] * xr[c]; }
        ss = wave_sum(ss);
        gx = wave_sum(gx);
        float rms = sqrtf(ss / (float)n);
        if (rms < eps) {
            float inv = 1.0f / eps;
            for (int64_t c = lane; c < n; c += 64) dx[t * n + c] = gr[c] * inv;
        } else {
            float inv = 1.0f / rms;
            float k = gx / ((float)n * rms * rms * rms);
            for (int64_t c = lane; c < n; c += 64) dx[t * n + c] = gr[c] * inv - xr[c] * k;
        }
    }
}

// The same derivative from what the training step has at hand: the normalised output y (which the attention reads
// and the step keeps) and the saved rms.  With x = r y:  dx = (dy - y (dy.y)/n) / r  while r = rms >= eps, and
// dx = dy/eps when the forward clamped.  dx may be dy.
template <int VPL>
__global__ __launch_bounds__(kBlock) void qk_norm_bwd_saved_vec_kernel(const float* __restrict__ y, const float* __restrict__ rms,
                                                                       const float* dy, float* dx, int64_t T, int n, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (t >= T) return;
    const int n4 = n >> 2;
    const float4* yr = reinterpret_cast<const float4*>(y + t * n);
    const float4* gr = reinterpret_cast<const float4*>(dy + t * n);
    float4 yv[VPL], gv[VPL];
    float gy = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        const int i4 = lane + 64 * k;
        yv[k] = i4 < n4 ? ldnt4(yr + i4) : make_float4(0, 0, 0, 0);
        gv[k] = i4 < n4 ? ldnt4(gr + i4) : make_float4(0, 0, 0, 0);
        gy += (gv[k].x * yv[k].x + gv[k].y * yv[k].y) + (gv[k].z * yv[k].z + gv[k].w * yv[k].w);
    }
    gy = wave_sum(gy);
    const float r = rms[t];
    const bool clamped = r < eps;
    const float inv = 1.0f / (clamped ? eps : r);
    const float c = clamped ? 0.0f : gy / (float)n;
    float4* dr = reinterpret_cast<float4*>(dx + t * n);
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        const int i4 = lane + 64 * k;
        if (i4 < n4) stnt4(dr + i4, make_float4((gv[k].x - yv[k].x * c) * inv, (gv[k].y - yv[k].y * c) * inv,
                                                (gv[k].z - yv[k].z * c) * inv, (gv[k].w - yv[k].w * c) * inv));
    }
}

__global__ __launch_bounds__(kBlock) void qk_norm_bwd_saved_kernel(const float* __restrict__ y, const float* __restrict__ rms,
                                                                   const float* dy, float* dx, int64_t T, int64_t n, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t t = wave; t < T; t += nwaves) {
        const float* yr = y + t * n;
        const float* gr = dy + t * n;
        float gy = 0.0f;
        for (int64_t c = lane; c < n; c += 64) gy += gr[c] * yr[c];
        gy = wave_sum(gy);                                     // every lane has read its dy before any lane writes dx
        const float r = rms[t];
        const bool clamped = r < eps;
        const float inv = 1.0f / (clamped ? eps : r);
        const float k = clamped ? 0.0f : gy / (float)n;
        for (int64_t c = lane; c < n; c += 64) dx[t * n + c] = (gr[c] - yr[c] * k) * inv;
    }
}

// ---------------------------------------------------------------- static scratch
// Partial rows for callers that can neither allocate nor bring a workspace (code under graph capture,
// serving loops).  One array per GPU, held until the process ends.  `scratch` is a host-side stand-in
// in host code: only the address hipGetSymbolAddress returns for the current device may reach a kernel.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];
constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices];              // device address of `scratch` on each GPU
static std::mutex g_scratch_mutex;

// Address of this file's scratch array on the current device (looked up once per device).
static int static_scratch(float** out) {
    int dev = -1;
    SERAPH_HIP_CHECK(hipGetDevice(&dev));
    SERAPH_REQUIRE(dev >= 0 && dev < kMaxDevices, "rmsnorm_backward_static: device index %d not supported", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        SERAPH_HIP_CHECK(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
        SERAPH_REQUIRE(ptr != nullptr, "rmsnorm_backward_static: no device address for the scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return SERAPH_OK;
}

int rmsnorm_static_scratch_setup() {
    float* p = nullptr;
    return static_scratch(&p);
}

// ---------------------------------------------------------------- host side
static int pick_vpl(int64_t cols) {
    if (cols % 4 != 0) return 0;
    int64_t n4 = cols / 4;
    for (int v = 1; v <= 16; v *= 2) if (n4 <= 64 * v) return v;
    return 0;
}

// wave-per-row kernels (short or odd rows): workgroups in the grid
static int bwd_grid(int64_t rows) {
    int64_t want = ceil_div(rows, kWavesPerBlock * 2);          // at least two rows per wave
    int64_t cap = (int64_t)num_compute_units() * 4;
    if (want < 1) want = 1;
    return (int)(want < cap ? want : cap);
}

// block-per-row kernel: float4 slots per lane, or 0 when the shape does not qualify
static int pick_block_vpl(int64_t cols) {
    if (cols % 4 != 0 || cols <= 512) return 0;
    int64_t n4 = cols / 4;
    for (int v = 1; v <= 8; v *= 2) if (n4 <= kBlock * v) return v;
    return 0;
}

static int bwd_block_grid(int64_t rows) {
    // two workgroups per CU: 6.05 TB/s on 16384 x 2048 against 5.8 with four and 5.4 with five, and
    // half as many partial rows for the column reduction
    int64_t cap = (int64_t)num_compute_units() * 2;
    return (int)(rows < cap ? rows : cap);
}

}  // namespace seraph

using namespace seraph;

extern "C" {

int seraph_rmsnorm(const float* x, const float* scale, float* y, int64_t rows, int64_t cols, float eps,
                   seraph_stream_t s) {
    return seraph_add_rmsnorm(x, nullptr, nullptr, scale, y, rows, cols, eps, s);
}

int seraph_add_rmsnorm(const float* x, const float* addend, float* sum, const float* scale, float* y,
                       int64_t rows, int64_t cols, float eps, seraph_stream_t s) {
    if (rows == 0 || cols == 0) return SERAPH_OK;
    SERAPH_REQUIRE(x && scale && y, "rmsnorm: NULL pointer");
    SERAPH_REQUIRE(!addend == !sum, "add_rmsnorm: the addend and the place for the sum come together");
    SERAPH_REQUIRE(!sum || (sum != x && sum != addend && sum != y), "add_rmsnorm: the sum needs a buffer of its own");
    SERAPH_REQUIRE(rows > 0 && cols > 0, "rmsnorm: bad shape %lld x %lld", (long long)rows, (long long)cols);
    int64_t want = ceil_div(rows, kWavesPerBlock);
    int64_t cap = (int64_t)num_compute_units() * 8;
    int grid = (int)(want < cap ? want : cap);
    int vpl = (aligned16(x) && aligned16(scale) && aligned16(y) && (!addend || (aligned16(addend) && aligned16(sum)))) ? pick_vpl(cols) : 0;
    hipStream_t st = as_stream(s);
#define FWD(V) hipLaunchKernelGGL(rmsnorm_fwd_kernel<V>, dim3(grid), dim3(kBlock), 0, st, x, addend, sum, scale, y, rows, (int)cols, eps)
    switch (vpl) {
        case 1: FWD(1); break;
        case 2: FWD(2); break;
        case 4: FWD(4); break;
        case 8: FWD(8); break;
        case 16: FWD(16); break;
        default:
            hipLaunchKernelGGL(rmsnorm_fwd_generic_kernel, dim3(grid), dim3(kBlock), 0, st, x, addend, sum, scale, y, rows, cols, eps);
    }
#undef FWD
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

// Partial rows that rmsnorm_backward_launch writes for a shape, by the kernel it will pick (`aligned`: every
// operand on a 16-byte boundary).
static size_t bwd_partial_rows(int64_t rows, int64_t cols, bool aligned) {
    if (aligned && pick_block_vpl(cols)) return (size_t)bwd_block_grid(rows);                  // one per workgroup
    if (aligned && cols <= 512 && pick_vpl(cols)) return (size_t)bwd_grid(rows);               // one per workgroup
    return (size_t)bwd_grid(rows) * kWavesPerBlock;                                            // one per wave
}

size_t seraph_rmsnorm_backward_ws_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    // the generic path needs one partial row per wave, the register path one per block
    size_t parts = (size_t)bwd_grid(rows) * kWavesPerBlock;
    if ((size_t)bwd_block_grid(rows) > parts) parts = (size_t)bwd_block_grid(rows);
    return parts * (size_t)cols * sizeof(float);
}

int seraph_rmsnorm_backward(const float* x, const float* scale, const float* dy, float* dx, float* grad_scale,
                            int64_t rows, int64_t cols, float eps, void* ws, size_t ws_bytes, seraph_stream_t s) {
    return seraph_rmsnorm_backward_residual(x, scale, dy, nullptr, dx, grad_scale, rows, cols, eps, ws, ws_bytes, s);
}

// Launches of the backward on checked arguments; `partial` holds seraph_rmsnorm_backward_ws_bytes(rows, cols).
// With nparts_out the column sum is left out: the partial rows stay in `partial` and their number is reported.
static int rmsnorm_backward_launch(const float* x, const float* scale, const float* dy, const float* res, float* dx,
                                   float* grad_scale, int64_t rows, int64_t cols, float eps, float* partial,
                                   seraph_stream_t s, int* nparts_out = nullptr) {
    hipStream_t st = as_stream(s);
    const hipEvent_t done = take_armed_event();                 // belongs to the last launch: the column sum, or the row pass alone
    const bool aligned = aligned16(x) && aligned16(scale) && aligned16(dy) && aligned16(dx) && aligned16(partial) && (!res || aligned16(res));
    const int bvpl = aligned ? pick_block_vpl(cols) : 0;
    const int wvpl = (aligned && !bvpl && cols <= 512) ? pick_vpl(cols) : 0;
    int nparts;
    if (bvpl) {
        const int grid = bwd_block_grid(rows);
        nparts = grid;
        if (nparts_out) arm_event(done);
#define BBWD(V) SERAPH_LAUNCH_LAST((rmsnorm_bwd_block_kernel<V, 0>), dim3(grid), dim3(kBlock), 0, st, x, scale, dy, res, dx, partial, rows, (int)cols, eps)
        switch (bvpl) {
            case 1: BBWD(1); break;
            case 2: BBWD(2); break;
            case 4: BBWD(4); break;
            default: BBWD(8); break;
        }
#undef BBWD
    } else if (wvpl) {
        const int grid = bwd_grid(rows);
        nparts = grid;
        const size_t lds = (size_t)kWavesPerBlock * cols * sizeof(float);
        if (nparts_out) arm_event(done);
#define BWD(V) SERAPH_LAUNCH_LAST(rmsnorm_bwd_kernel<V>, dim3(grid), dim3(kBlock), lds, st, x, scale, dy, res, dx, partial, rows, (int)cols, eps)
        if (wvpl == 1) BWD(1); else BWD(2);
#undef BWD
    } else {
        const int grid = bwd_grid(rows);
        nparts = grid * kWavesPerBlock;
        int rc = seraph_fill_u32(partial, 0u, (size_t)nparts * cols, s);
        if (rc != SERAPH_OK) return rc;
        if (nparts_out) arm_event(done);
        SERAPH_LAUNCH_LAST(rmsnorm_bwd_generic_kernel, dim3(grid), dim3(kBlock), 0, st, x, scale, dy, res, dx, partial, rows, cols, eps);
    }
    SERAPH_LAUNCH_CHECK();
    if (nparts_out) { *nparts_out = nparts; return SERAPH_OK; }
    arm_event(done);
    if (cols % 4 == 0 && aligned16(partial))
        SERAPH_LAUNCH_LAST(colsum_add_kernel<true>, dim3((unsigned)ceil_div(cols, 64)), dim3(1024), 0, st, partial, nparts, cols, grad_scale);
    else
        SERAPH_LAUNCH_LAST(colsum_add_kernel<false>, dim3((unsigned)ceil_div(cols, 64)), dim3(1024), 0, st, partial, nparts, cols, grad_scale);
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

int seraph_rmsnorm_backward_residual(const float* x, const float* scale, const float* dy, const float* residual, float* dx,
                                     float* grad_scale, int64_t rows, int64_t cols, float eps, void* ws, size_t ws_bytes,
                                     seraph_stream_t s) {
    if (rows == 0 || cols == 0) return SERAPH_OK;
    SERAPH_REQUIRE(x && scale && dy && dx && grad_scale, "rmsnorm_backward: NULL pointer");
    SERAPH_REQUIRE(rows > 0 && cols > 0, "rmsnorm_backward: bad shape");
    if (!ws || ws_bytes < seraph_rmsnorm_backward_ws_bytes(rows, cols)) {
        set_error("rmsnorm_backward: scratch of %zu bytes required", seraph_rmsnorm_backward_ws_bytes(rows, cols));
        return SERAPH_ERR_WORKSPACE;
    }
    return rmsnorm_backward_launch(x, scale, dy, residual, dx, grad_scale, rows, cols, eps, (float*)ws, s);
}

int seraph_rmsnorm_backward_rows(const float* x, const float* scale, const float* dy, const float* residual, float* dx,
                                 int64_t rows, int64_t cols, float eps, void* ws, size_t ws_bytes, int* nparts,
                                 seraph_stream_t s) {
    SERAPH_REQUIRE(nparts, "rmsnorm_backward_rows: NULL pointer");
    *nparts = 0;
    if (rows == 0 || cols == 0) return SERAPH_OK;
    SERAPH_REQUIRE(x && scale && dy && dx, "rmsnorm_backward_rows: NULL pointer");
    SERAPH_REQUIRE(rows > 0 && cols > 0, "rmsnorm_backward_rows: bad shape");
    if (!ws || ws_bytes < seraph_rmsnorm_backward_ws_bytes(rows, cols)) {
        set_error("rmsnorm_backward_rows: scratch of %zu bytes required", seraph_rmsnorm_backward_ws_bytes(rows, cols));
        return SERAPH_ERR_WORKSPACE;
    }
    return rmsnorm_backward_launch(x, scale, dy, residual, dx, nullptr, rows, cols, eps, (float*)ws, s, nparts);
}

int seraph_rmsnorm_colsum_multi(const seraph_colsum_job_t* jobs, int count, int64_t cols, seraph_stream_t s) {
    if (count == 0 || cols == 0) return SERAPH_OK;
    SERAPH_REQUIRE(jobs && count > 0 && cols > 0, "rmsnorm_colsum_multi: bad arguments");
    bool vec = cols % 4 == 0;
    for (int i = 0; i < count; i++) {
        SERAPH_REQUIRE(jobs[i].partial && jobs[i].grad_scale && jobs[i].nparts >= 0, "rmsnorm_colsum_multi: job %d is incomplete", i);
        vec = vec && aligned16(jobs[i].partial);
    }
    hipStream_t st = as_stream(s);
    for (int at = 0; at < count; at += kMaxColsumJobs) {
        const int n = count - at < kMaxColsumJobs ? count - at : kMaxColsumJobs;
        ColsumJobs j;
        for (int i = 0; i < n; i++) { j.partial[i] = jobs[at + i].partial; j.grad_scale[i] = jobs[at + i].grad_scale; j.nparts[i] = jobs[at + i].nparts; }
        for (int i = n; i < kMaxColsumJobs; i++) { j.partial[i] = nullptr; j.grad_scale[i] = nullptr; j.nparts[i] = 0; }
        const dim3 grid((unsigned)ceil_div(cols, 64), (unsigned)n);
        if (at + n < count) {
            if (vec) hipLaunchKernelGGL(colsum_add_multi_kernel<true>, grid, dim3(1024), 0, st, j, cols);
            else hipLaunchKernelGGL(colsum_add_multi_kernel<false>, grid, dim3(1024), 0, st, j, cols);
        } else {
            if (vec) SERAPH_LAUNCH_LAST(colsum_add_multi_kernel<true>, grid, dim3(1024), 0, st, j, cols);
            else SERAPH_LAUNCH_LAST(colsum_add_multi_kernel<false>, grid, dim3(1024), 0, st, j, cols);
        }
        SERAPH_LAUNCH_CHECK();
    }
    return SERAPH_OK;
}

size_t seraph_rmsnorm_backward_static_max_bytes(void) { return kStaticScratchBytes; }

int seraph_rmsnorm_backward_static(const float* x, const float* scale, const float* dy, const float* residual, float* dx,
                                   float* grad_scale, int64_t rows, int64_t cols, float eps, seraph_stream_t s) {
    if (rows == 0 || cols == 0) return SERAPH_OK;
    SERAPH_REQUIRE(x && scale && dy && dx && grad_scale, "rmsnorm_backward_static: NULL pointer");
    SERAPH_REQUIRE(rows > 0 && cols > 0, "rmsnorm_backward_static: bad shape");
    float* partial = nullptr;
    int rc = static_scratch(&partial);
    if (rc != SERAPH_OK) return rc;
    // what the kernel that these operands select will write (the workspace query answers for any alignment)
    const bool aligned = aligned16(x) && aligned16(scale) && aligned16(dy) && aligned16(dx) && aligned16(partial) &&
                         (!residual || aligned16(residual));
    const size_t need = bwd_partial_rows(rows, cols, aligned) * (size_t)cols * sizeof(float);
    if (need > kStaticScratchBytes) {
        set_error("rmsnorm_backward_static: %lld x %lld needs %zu bytes of scratch, the built-in array holds %zu; "
                  "use seraph_rmsnorm_backward_residual with a workspace", (long long)rows, (long long)cols, need,
                  kStaticScratchBytes);
        return SERAPH_ERR_WORKSPACE;
    }
    return rmsnorm_backward_launch(x, scale, dy, residual, dx, grad_scale, rows, cols, eps, partial, s);
}

int seraph_qk_norm(float* qk, int64_t T, int heads, int head_dim, int use_qk_norm, float eps, seraph_stream_t s) {
    if (!use_qk_norm) return SERAPH_OK;                           // shaders/qk_norm.comp:32
    return seraph_qk_norm_saved(qk, nullptr, T, heads, head_dim, eps, s);
}

int seraph_qk_norm_saved(float* qk, float* rms_out, int64_t T, int heads, int head_dim, float eps, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(qk && heads > 0 && head_dim > 0 && T > 0, "qk_norm: bad argument");
    const int64_t n = (int64_t)heads * head_dim;
    const int vpl = aligned16(qk) ? pick_vpl(n) : 0;
    hipStream_t st = as_stream(s);
    const dim3 grid((unsigned)ceil_div(T, kWavesPerBlock));
#define QKN(V) hipLaunchKernelGGL(qk_norm_vec_kernel<V>, grid, dim3(kBlock), 0, st, qk, rms_out, T, (int)n, eps)
    switch (vpl) {
        case 1: QKN(1); break;
        case 2: QKN(2); break;
        case 4: QKN(4); break;
        case 8: QKN(8); break;
        case 16: QKN(16); break;
        default: {
            int64_t want = ceil_div(T, kWavesPerBlock), cap = (int64_t)num_compute_units() * 8;
            hipLaunchKernelGGL(qk_norm_kernel, dim3((unsigned)(want < cap ? want : cap)), dim3(kBlock), 0, st, qk, rms_out, T, n, eps);
        }
    }
#undef QKN
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

int seraph_qk_norm_backward_saved(const float* y, const float* rms, const float* dy, float* dx, int64_t T, int heads, int head_dim,
                                  float eps, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(y && rms && dy && dx && heads > 0 && head_dim > 0 && T > 0, "qk_norm_backward_saved: bad argument");
    const int64_t n = (int64_t)heads * head_dim;
    const int vpl = (aligned16(y) && aligned16(dy) && aligned16(dx)) ? pick_vpl(n) : 0;
    hipStream_t st = as_stream(s);
    const dim3 grid((unsigned)ceil_div(T, kWavesPerBlock));
#define QKB(V) hipLaunchKernelGGL(qk_norm_bwd_saved_vec_kernel<V>, grid, dim3(kBlock), 0, st, y, rms, dy, dx, T, (int)n, eps)
    switch (vpl) {
        case 1: QKB(1); break;
        case 2: QKB(2); break;
        case 4: QKB(4); break;
        case 8: QKB(8); break;
        case 16: QKB(16); break;
        default: {
            int64_t want = ceil_div(T, kWavesPerBlock), cap = (int64_t)num_compute_units() * 8;
            hipLaunchKernelGGL(qk_norm_bwd_saved_kernel, dim3((unsigned)(want < cap ? want : cap)), dim3(kBlock), 0, st, y, rms, dy, dx, T, n, eps);
        }
    }
#undef QKB
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

int seraph_qk_norm_backward(const float* x_pre, const float* dy, float* dx, int64_t T, int heads, int head_dim,
                            float eps, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(x_pre && dy && dx && heads > 0 && head_dim > 0, "qk_norm_backward: bad argument");
    int64_t want = ceil_div(T, kWavesPerBlock), cap = (int64_t)num_compute_units() * 8;
    hipLaunchKernelGGL(qk_norm_bwd_kernel, dim3((unsigned)(want < cap ? want : cap)), dim3(kBlock), 0, as_stream(s),
                       x_pre, dy, dx, T, (int64_t)heads * head_dim, eps);
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

}  // extern "C"
