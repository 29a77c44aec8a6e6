// rope.hip - rotary position embedding, forward and inverse (backward), in place or not.
//
// The rotation angle depends on (position, pair) only, so one lane owns one (token, pair)
// and applies the same sine/cosine to every head: one accurate sincosf per `heads`
// float2 loads and stores instead of the per-element pow/sin/cos of
// shaders/rope_backward.comp:40-45.  Lanes of a wave cover consecutive pairs, so each
// head's accesses are contiguous 8-byte elements.
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

extern "C" int seraph_rope(const float* in, float* out, const uint32_t* seq_starts, int batch, int64_t T,
                           int heads, int head_dim, float theta, int backward, seraph_stream_t s) {
    if (T == 0) return SERAPH_OK;
    SERAPH_REQUIRE(in && out, "rope: NULL pointer");
    SERAPH_REQUIRE(heads > 0 && head_dim >= 2 && head_dim % 2 == 0, "rope: bad heads/head_dim %d/%d", heads, head_dim);
    SERAPH_REQUIRE(((uintptr_t)in & 7u) == 0 && ((uintptr_t)out & 7u) == 0, "rope: buffers must be 8-byte aligned");
    SERAPH_REQUIRE(!seq_starts || batch >= 1, "rope: packed call needs batch >= 1");
    const float* table = nullptr;
    int rc = get_inv_freq(head_dim, theta, &table);
    if (rc != SERAPH_OK) return rc;
    int64_t total = T * (head_dim / 2);
    dim3 grid((unsigned)ceil_div(total, 256));
    if (backward)
        hipLaunchKernelGGL(rope_kernel<true>, grid, dim3(256), 0, as_stream(s), in, out, table, seq_starts, batch, T, heads, head_dim);
    else
        hipLaunchKernelGGL(rope_kernel<false>, grid, dim3(256), 0, as_stream(s), in, out, table, seq_starts, batch, T, heads, head_dim);
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}
