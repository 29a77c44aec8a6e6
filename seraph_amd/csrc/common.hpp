// common.hpp - shared device/host helpers for the gfx950 kernel library.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>

#include "seraph_hip.h"

namespace seraph {

constexpr int kWave = 64;          // CDNA wavefront
constexpr int kNumXcd = 8;         // MI355X: 8 XCDs, workgroups are dealt to them round-robin

void set_error(const char* fmt, ...);

#define SERAPH_REQUIRE(cond, ...)                                \
    do {                                                         \
        if (!(cond)) {                                           \
            ::seraph::set_error(__VA_ARGS__);                    \
            return SERAPH_ERR_INVALID;                           \
        }                                                        \
    } while (0)

#define SERAPH_HIP_CHECK(expr)                                                         \
    do {                                                                               \
        hipError_t e_ = (expr);                                                        \
        if (e_ != hipSuccess) {                                                        \
            ::seraph::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                                __FILE__, __LINE__);                                   \
            return SERAPH_ERR_HIP;                                                     \
        }                                                                              \
    } while (0)

#define SERAPH_LAUNCH_CHECK() SERAPH_HIP_CHECK(hipGetLastError())

// Launch of the kernel that ends an op.  When the caller has armed an event for this thread
// (seraph_hip_event_on_next_op) the event completes with this very dispatch, so a second stream can wait for
// the op without a marker packet between this kernel and the next one on its own stream.
hipEvent_t take_armed_event();
void arm_event(hipEvent_t ev);      // an op with several launches takes the event at entry and arms it again before its last one
#define SERAPH_LAUNCH_LAST(kernel, grid, block, shmem, st, ...)                                          \
    do {                                                                                                 \
        hipEvent_t ev_ = ::seraph::take_armed_event();                                                   \
        if (ev_) hipExtLaunchKernelGGL(kernel, grid, block, shmem, st, nullptr, ev_, 0, __VA_ARGS__);    \
        else hipLaunchKernelGGL(kernel, grid, block, shmem, st, __VA_ARGS__);                            \
    } while (0)

static inline hipStream_t as_stream(seraph_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

int num_compute_units();           // cached after seraph_hip_init / first use
int rmsnorm_static_scratch_setup(); // rmsnorm.hip: looks up its built-in scratch array on the current device

// ---------------------------------------------------------------- device helpers
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Index of the packed sequence that holds token `pos` (starts has batch+1 entries).
__device__ __forceinline__ int find_seq(const uint32_t* __restrict__ starts, int batch, int64_t pos) {
    int lo = 0, hi = batch;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if ((int64_t)starts[mid + 1] <= pos) lo = mid + 1; else hi = mid;
    }
    return lo;
}

}  // namespace seraph
