// rope.hip - rotary position embedding, forward and inverse (backward), in place or not.
//
// The rotation angle depends on (position, pair) only, so one lane owns two neighbouring pairs
// of one token and applies their sines/cosines to every head: two accurate sincosf per `heads`
// 16-byte loads and stores instead of the per-element pow/sin/cos of
// shaders/rope_backward.comp:40-45.  Lanes of a wave cover consecutive pairs, so each head's
// accesses are contiguous; heads are taken eight at a time with all eight loads issued before
// the first store, and the data is streamed (nontemporal) - it is touched once.  Head sizes
// that are not a multiple of 4, or 8-byte aligned buffers, take the one-pair-per-lane kernel.
//
// angle = float(pos) * inv_freq[i] is an FP32 product of an FP32 table entry, as the
// shader forms it; the table 1/powf(theta, 2i/D) is evaluated once per (D, theta) on
// the host and cached on the device, which keeps the angle independent of the device
// pow implementation at large positions.
#include <math.h>
#include <mutex>
#include <string.h>
#include <vector>

#include "common.hpp"

namespace seraph {

struct FreqTable { int D; uint32_t theta_bits; int device; float* dev; };
static std::mutex g_freq_mu;
static std::vector<FreqTable> g_freq;

static int get_inv_freq(int D, float theta, const float** out) {
    uint32_t bits;
    memcpy(&bits, &theta, 4);
    int device = 0;
    SERAPH_HIP_CHECK(hipGetDevice(&device));
    std::lock_guard<std::mutex> lk(g_freq_mu);
    for (const FreqTable& t : g_freq)
        if (t.D == D && t.theta_bits == bits && t.device == device) { *out = t.dev; return SERAPH_OK; }
    std::vector<float> host((size_t)D / 2);
    for (int i = 0; i < D / 2; i++) {
        float exponent = (float)(2 * i) / (float)D;          // rope.comp: float(2*pair_idx)/float(head_dim)
        host[i] = 1.0f / powf(theta, exponent);
    }
    float* dev = nullptr;
    SERAPH_HIP_CHECK(hipMalloc((void**)&dev, host.size() * sizeof(float)));
    SERAPH_HIP_CHECK(hipMemcpy(dev, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
    g_freq.push_back(FreqTable{D, bits, device, dev});
    *out = dev;
    return SERAPH_OK;
}

typedef float f4v __attribute__((ext_vector_type(4)));

constexpr int kRope4Block = 64;

template <bool BACKWARD>
__device__ __forceinline__ void rotate_heads(const float* __restrict__ in, float* __restrict__ out, int64_t base, int heads, int D,
                                             float s0, float c0, float s1, float c1);

// One or two tensors (query and key heads of the same tokens) per launch.
template <bool BACKWARD>
__global__ __launch_bounds__(kRope4Block) void rope4_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                    const float* __restrict__ in2, float* __restrict__ out2,
                                                    const float* __restrict__ inv_freq,
                                                    const uint32_t* __restrict__ seq_starts, int batch,
                                                    int64_t T, int heads, int heads2, int D) {
    const int quarter = D >> 2;
    const int64_t idx = (int64_t)blockIdx.x * kRope4Block + threadIdx.x;
    if (idx >= T * quarter) return;
    const int64_t t = idx / quarter;
    const int j = (int)(idx - t * quarter);                  // pairs 2j and 2j+1
    int64_t pos = t;
    if (seq_starts) pos = t - (int64_t)seq_starts[find_seq(seq_starts, batch, t)];
    float s0, c0, s1, c1;
    sincosf((float)pos * inv_freq[2 * j], &s0, &c0);
    sincosf((float)pos * inv_freq[2 * j + 1], &s1, &c1);
    if (BACKWARD) { s0 = -s0; s1 = -s1; }                    // R^T: rope_backward.comp:53-54
    rotate_heads<BACKWARD>(in, out, t * (int64_t)heads * D + 4 * j, heads, D, s0, c0, s1, c1);
    if (in2) rotate_heads<BACKWARD>(in2, out2, t * (int64_t)heads2 * D + 4 * j, heads2, D, s0, c0, s1, c1);
}

template <bool BACKWARD>
__device__ __forceinline__ void rotate_heads(const float* __restrict__ in, float* __restrict__ out, int64_t base, int heads, int D,
                                             float s0, float c0, float s1, float c1) {
    constexpr int G = 8;
    for (int h0 = 0; h0 < heads; h0 += G) {
        f4v v[G];
#pragma unroll
        for (int g = 0; g < G; g++)
            if (h0 + g < heads) v[g] = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(in + base + (int64_t)(h0 + g) * D));
#pragma unroll
        for (int g = 0; g < G; g++)
            if (h0 + g < heads) {
                f4v r;
                r.x = v[g].x * c0 - v[g].y * s0;
                r.y = v[g].x * s0 + v[g].y * c0;
                r.z = v[g].z * c1 - v[g].w * s1;
                r.w = v[g].z * s1 + v[g].w * c1;
                __builtin_nontemporal_store(r, reinterpret_cast<f4v*>(out + base + (int64_t)(h0 + g) * D));
            }
    }
}

template <bool BACKWARD>
__global__ __launch_bounds__(256) void rope_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                   const float* __restrict__ inv_freq,
                                                   const uint32_t* __restrict__ seq_starts, int batch,
                                                   int64_t T, int heads, int D) {
    const int half = D >> 1;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= T * half) return;
    const int64_t t = idx / half;
    const int i = (int)(idx - t * half);
    int64_t pos = t;
    if (seq_starts) pos = t - (int64_t)seq_starts[find_seq(seq_starts, batch, t)];
    const float angle = (float)pos * inv_freq[i];
    float sn, cs;
    sincosf(angle, &sn, &cs);
    if (BACKWARD) sn = -sn;                                  // R^T: rope_backward.comp:53-54
    const int64_t base = t * (int64_t)heads * D + 2 * i;
    for (int h = 0; h < heads; h++) {
        const float2 v = *reinterpret_cast<const float2*>(in + base + (int64_t)h * D);
        float2 r;
        r.x = v.x * cs - v.y * sn;
        r.y = v.x * sn + v.y * cs;
        *reinterpret_cast<float2*>(out + base + (int64_t)h * D) = r;
    }
}

}  // namespace seraph

using namespace seraph;

static int rope_launch(const float* in, float* out, int heads, const float* in2, float* out2, int heads2,
                       const uint32_t* seq_starts, int batch, int64_t T, int head_dim, float theta, int backward, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(in && out && (!in2 || out2), "rope: NULL pointer");
    SERAPH_REQUIRE(heads > 0 && (!in2 || heads2 > 0) && head_dim >= 2 && head_dim % 2 == 0, "rope: bad heads/head_dim %d/%d", heads, head_dim);
    SERAPH_REQUIRE(((uintptr_t)in & 7u) == 0 && ((uintptr_t)out & 7u) == 0 && ((uintptr_t)in2 & 7u) == 0 && ((uintptr_t)out2 & 7u) == 0,
                   "rope: buffers must be 8-byte aligned");
    SERAPH_REQUIRE(!seq_starts || batch >= 1, "rope: packed call needs batch >= 1");
    const float* table = nullptr;
    int rc = get_inv_freq(head_dim, theta, &table);
    if (rc != SERAPH_OK) return rc;
    hipStream_t st = as_stream(s);
    const bool wide = head_dim % 4 == 0 && (((uintptr_t)in | (uintptr_t)out | (uintptr_t)in2 | (uintptr_t)out2) & 15u) == 0;
    if (wide) {
        dim3 grid4((unsigned)ceil_div(T * (head_dim / 4), (int64_t)kRope4Block));
        if (backward)
            SERAPH_LAUNCH_LAST(rope4_kernel<true>, grid4, dim3(kRope4Block), 0, st, in, out, in2, out2, table, seq_starts, batch, T, heads, heads2, head_dim);
        else
            SERAPH_LAUNCH_LAST(rope4_kernel<false>, grid4, dim3(kRope4Block), 0, st, in, out, in2, out2, table, seq_starts, batch, T, heads, heads2, head_dim);
        SERAPH_LAUNCH_CHECK();
        return SERAPH_OK;
    }
    const int64_t total = T * (head_dim / 2);
    dim3 grid((unsigned)ceil_div(total, 256));
    for (int pass = 0; pass < (in2 ? 2 : 1); pass++) {
        const float* a = pass ? in2 : in;
        float* b = pass ? out2 : out;
        const int h = pass ? heads2 : heads;
        if (backward)
            hipLaunchKernelGGL(rope_kernel<true>, grid, dim3(256), 0, st, a, b, table, seq_starts, batch, T, h, head_dim);
        else
            hipLaunchKernelGGL(rope_kernel<false>, grid, dim3(256), 0, st, a, b, table, seq_starts, batch, T, h, head_dim);
        SERAPH_LAUNCH_CHECK();
    }
    return SERAPH_OK;
}

extern "C" int seraph_rope(const float* in, float* out, const uint32_t* seq_starts, int batch, int64_t T,
                           int heads, int head_dim, float theta, int backward, seraph_stream_t s) {
    return rope_launch(in, out, heads, nullptr, nullptr, 0, seq_starts, batch, T, head_dim, theta, backward, s);
}

extern "C" int seraph_rope_qk(const float* q_in, float* q_out, int q_heads, const float* k_in, float* k_out, int k_heads,
                              const uint32_t* seq_starts, int batch, int64_t T, int head_dim, float theta, int backward,
                              seraph_stream_t s) {
    SERAPH_REQUIRE(k_in && k_out, "rope_qk: NULL pointer");
    return rope_launch(q_in, q_out, q_heads, k_in, k_out, k_heads, seq_starts, batch, T, head_dim, theta, backward, s);
}
