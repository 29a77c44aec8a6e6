/* hip_backend_internal.h - private state shared by hip_backend.c and hip_backend_backward.c */
#ifndef HIP_BACKEND_INTERNAL_H
#define HIP_BACKEND_INTERNAL_H

#include <stdio.h>

#include "hip_backend.h"
#include "seraph_hip.h"

#define HIP_PROF_MAX_OPS 8192

typedef struct {
    char name[128];              /* as the reference names the op (src/vulkan_backend.c:31-43): its report sorts ops by substrings */
    void* ev_start;
    void* ev_stop;
} hip_prof_op_t;

typedef struct {
    seraph_stream_t stream;
    int recording;               /* between vulkan_cmd_begin and vulkan_cmd_end_submit */
    void* ws;                    /* device scratch shared by the ops that need one */
    size_t ws_bytes;
    int errors;
    /* profiler: one event pair per op of the current step */
    hip_prof_op_t* prof_ops;
    int prof_count;
    int prof_events_made;
} hip_state_t;

static inline hip_state_t* hip_state(vulkan_context_t* ctx) { return ctx ? (hip_state_t*)ctx->device : NULL; }

/* Grows the shared scratch to at least `bytes`; returns NULL on failure. */
void* hip_backend_scratch(vulkan_context_t* ctx, size_t bytes);
void hip_backend_report(vulkan_context_t* ctx, const char* op, int rc);
void hip_prof_begin(vulkan_context_t* ctx, const char* name);
void hip_prof_end(vulkan_context_t* ctx);

/* 1 when each of the `pairs` (buffer, number of 4-byte values) arguments that follow fits its buffer.  Otherwise the op
 * is reported as refused and counted as an error, and the caller returns without launching anything: a shape that
 * reaches past the end of a buffer is a memory fault on this device, which can take more than the process with it. */
int hip_backend_fits(vulkan_context_t* ctx, const char* op, int pairs, ...);
#define FIT(buf, n) (const vulkan_buffer_t*)(buf), (size_t)(n)

/* Runs one kernel-library call for op `name`: timing when profiling, error report when it fails. */
#define HIP_OP(ctx, name, call)                       \
    do {                                              \
        hip_prof_begin((ctx), (name));                \
        int rc_ = (call);                             \
        hip_prof_end((ctx));                          \
        if (rc_ != SERAPH_OK) hip_backend_report((ctx), (name), rc_); \
    } while (0)

/* The same with a formatted name, e.g. HIP_OPF(ctx, call, "matmul [%dx%d K=%d]", M, N, K). */
#define HIP_OPF(ctx, call, ...)                       \
    do {                                              \
        char pn_[128];                                \
        snprintf(pn_, sizeof(pn_), __VA_ARGS__);      \
        HIP_OP((ctx), pn_, (call));                   \
    } while (0)

#define DPTR(buf) ((buf)->buffer)
#define FPTR(buf) ((float*)(buf)->buffer)
#define UPTR(buf) ((uint32_t*)(buf)->buffer)

#endif
