// runtime.hip - device runtime half of the C ABI: init, memory, streams, events.
#include <stdarg.h>
#include <string.h>

#include "common.hpp"

namespace seraph {

static thread_local char g_err[512] = "";
static thread_local hipEvent_t g_armed_event = nullptr;

void arm_event(hipEvent_t ev) { g_armed_event = ev; }

hipEvent_t take_armed_event() {
    hipEvent_t ev = g_armed_event;
    g_armed_event = nullptr;
    return ev;
}
static int g_cu_count = 0;

// Every error path of the library goes through here: an op that fails before its last launch must not leave its
// caller's event armed for whatever op the thread calls next.
void set_error(const char* fmt, ...) {
    g_armed_event = nullptr;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int num_compute_units() {
    if (g_cu_count == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_cu_count = n;
        else
            g_cu_count = 256;
    }
    return g_cu_count;
}

}  // namespace seraph

using namespace seraph;

extern "C" {

const char* seraph_hip_last_error(void) { return g_err; }

int seraph_hip_init(int device_index) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        set_error("no HIP device visible");
        return SERAPH_ERR_NODEVICE;
    }
    int dev = device_index < 0 ? 0 : device_index;
    SERAPH_REQUIRE(dev < count, "device index %d out of range (%d devices)", dev, count);
    SERAPH_HIP_CHECK(hipSetDevice(dev));
    hipDeviceProp_t prop;
    SERAPH_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
        return SERAPH_ERR_NODEVICE;
    }
    g_cu_count = prop.multiProcessorCount;
    return rmsnorm_static_scratch_setup();     // per-device address of the built-in scratch array
}

int seraph_hip_device_info(seraph_device_info_t* out) {
    SERAPH_REQUIRE(out, "device_info: NULL out");
    int dev = 0;
    SERAPH_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    SERAPH_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", prop.name);
    snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
    out->hbm_bytes = prop.totalGlobalMem;
    out->compute_units = (uint32_t)prop.multiProcessorCount;
    out->wavefront_size = (uint32_t)prop.warpSize;
    out->lds_bytes_per_block = (uint32_t)prop.sharedMemPerBlock;
    out->clock_khz = (uint32_t)prop.clockRate;
    return SERAPH_OK;
}

int seraph_hip_malloc(void** out, size_t bytes) {
    SERAPH_REQUIRE(out, "malloc: NULL out");
    *out = nullptr;
    SERAPH_HIP_CHECK(hipMalloc(out, bytes ? bytes : 4));
    return SERAPH_OK;
}

int seraph_hip_free(void* p) {
    if (p) SERAPH_HIP_CHECK(hipFree(p));
    return SERAPH_OK;
}

int seraph_hip_host_alloc(void** out, size_t bytes) {
    SERAPH_REQUIRE(out, "host_alloc: NULL out");
    *out = nullptr;
    SERAPH_HIP_CHECK(hipHostMalloc(out, bytes ? bytes : 4, hipHostMallocDefault));
    return SERAPH_OK;
}

int seraph_hip_host_free(void* p) {
    if (p) SERAPH_HIP_CHECK(hipHostFree(p));
    return SERAPH_OK;
}

// Copies from/to pageable host memory complete before returning (the reference's
// uploads are immediate memcpys into mapped memory, src/vulkan_backend.c:1109-1182).
int seraph_hip_h2d(void* dst, const void* src, size_t bytes, seraph_stream_t s) {
    if (bytes == 0) return SERAPH_OK;
    SERAPH_REQUIRE(dst && src, "h2d: NULL pointer");
    SERAPH_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(s)));
    SERAPH_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return SERAPH_OK;
}

int seraph_hip_d2h(void* dst, const void* src, size_t bytes, seraph_stream_t s) {
    if (bytes == 0) return SERAPH_OK;
    SERAPH_REQUIRE(dst && src, "d2h: NULL pointer");
    SERAPH_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(s)));
    SERAPH_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return SERAPH_OK;
}

int seraph_hip_d2d(void* dst, const void* src, size_t bytes, seraph_stream_t s) {
    if (bytes == 0) return SERAPH_OK;
    SERAPH_REQUIRE(dst && src, "d2d: NULL pointer");
    SERAPH_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(s)));
    return SERAPH_OK;
}

int seraph_hip_stream_create(seraph_stream_t* out) {
    SERAPH_REQUIRE(out, "stream_create: NULL out");
    hipStream_t st;
    SERAPH_HIP_CHECK(hipStreamCreate(&st));      // default priority
    *out = reinterpret_cast<seraph_stream_t>(st);
    return SERAPH_OK;
}

int seraph_hip_stream_destroy(seraph_stream_t s) {
    if (s) SERAPH_HIP_CHECK(hipStreamDestroy(as_stream(s)));
    return SERAPH_OK;
}

int seraph_hip_stream_sync(seraph_stream_t s) {
    SERAPH_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return SERAPH_OK;
}

int seraph_hip_device_sync(void) {
    SERAPH_HIP_CHECK(hipDeviceSynchronize());
    return SERAPH_OK;
}

int seraph_hip_event_create(void** out) {
    SERAPH_REQUIRE(out, "event_create: NULL out");
    hipEvent_t ev;
    SERAPH_HIP_CHECK(hipEventCreate(&ev));
    *out = reinterpret_cast<void*>(ev);
    return SERAPH_OK;
}

int seraph_hip_event_create_sync(void** out) {
    SERAPH_REQUIRE(out, "event_create_sync: NULL out");
    hipEvent_t ev;
    // no timestamps, and no system-scope fence when the event completes: it orders streams of this device, whose
    // kernels release their writes at device scope anyway; the host never inspects it
    SERAPH_HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming | hipEventDisableSystemFence));
    *out = reinterpret_cast<void*>(ev);
    return SERAPH_OK;
}

int seraph_hip_event_on_next_op(void* ev) {
    g_armed_event = reinterpret_cast<hipEvent_t>(ev);
    return SERAPH_OK;
}

int seraph_hip_event_armed(void) { return g_armed_event != nullptr; }

int seraph_hip_event_destroy(void* ev) {
    if (ev) SERAPH_HIP_CHECK(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)));
    return SERAPH_OK;
}

int seraph_hip_event_record(void* ev, seraph_stream_t s) {
    SERAPH_REQUIRE(ev, "event_record: NULL event");
    SERAPH_HIP_CHECK(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), as_stream(s)));
    return SERAPH_OK;
}

int seraph_hip_stream_wait_event(seraph_stream_t s, void* ev) {
    SERAPH_REQUIRE(ev, "stream_wait_event: NULL event");
    SERAPH_HIP_CHECK(hipStreamWaitEvent(as_stream(s), reinterpret_cast<hipEvent_t>(ev), 0));
    return SERAPH_OK;
}

int seraph_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
    SERAPH_REQUIRE(start && stop && ms, "event_elapsed: NULL argument");
    SERAPH_HIP_CHECK(hipEventSynchronize(reinterpret_cast<hipEvent_t>(stop)));
    SERAPH_HIP_CHECK(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
    return SERAPH_OK;
}

}  // extern "C"
