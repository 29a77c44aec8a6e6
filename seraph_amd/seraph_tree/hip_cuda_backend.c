/*
 * hip_cuda_backend.c - Seraph's CUDA training backend API over the MI355X kernel library.
 *
 * Seraph's packed-batch trainer (src/train_cuda.c: cuda_train_step_gpu_full_batch,
 * cuda_train_step_gpu_lora_batch and their single-sequence forms; front end
 * tools/seraph_train_cuda.c) is plain C.  It reaches the GPU only through the functions declared
 * in include/cuda_train_context.h:239-325 and include/cuda_profiler.h:54-84, which the reference
 * implements in src/cuda_train_context.cu and src/cuda_profiler.cu.  This file implements the
 * same functions over include/seraph_hip.h, so those two C files link and run unmodified on an
 * MI355X.  It is compiled inside a Seraph tree (it needs Seraph's own headers for
 * cuda_train_context_t and lora_model_t):
 *
 *   cc -I<seraph>/include -I<this repo>/include tools/seraph_train_cuda.c src/train_cuda.c src/train.c ... \
 *      <this repo>/seraph_amd/seraph_tree/hip_cuda_backend.c <this repo>/seraph_amd/src/hip_backend*.c \
 *      -L<this repo>/seraph_amd/lib -lseraph_hip -lm
 *
 * Semantics kept from the reference's implementation (src/cuda_train_context.cu):
 *   - every op is asynchronous on the context's one stream; downloads wait (:2605-2619)
 *   - fill_buffer takes a BYTE value, as cudaMemsetAsync does (:2621-2631)
 *   - reduce_sum leaves the total in out[0] (:2966-2976); it also leaves the partial sums of
 *     every gpu_max_threads_per_block inputs in out[0..], which is what the caller's pass loop
 *     (src/train_cuda.c:2239-2250) needs to get the right total for more than one pass
 *   - attention backward ADDS into dK/dV, the caller clears them (src/train_cuda.c:2231-2234);
 *     rmsnorm backward and embedding backward add into their gradient outputs
 *   - use_flash_attn only changes the operation names: one streaming kernel pair serves both
 *     modes, saves the log-sum-exp whenever the caller passes a buffer for it and recomputes the
 *     statistics in the backward when it has none
 *   - AdamW: bias corrections from powf(beta, step) (:2187-2207)
 * What differs: use_bf16 is ignored (FP32 matrix cores; the device reports compute capability
 * 0.0 so that the front end's own --bf16 check falls back to FP32), launch geometry fields of
 * the profiler stay 0, and rmsnorm backward floors the rms at 0.01 as the Vulkan shader does.
 *
 * ctx->stream holds this file's private state, not a raw stream; cuda_profiler_* take that same
 * handle as their `stream` argument, which is what the reference's callers pass.
 */
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "hip_cuda_backend.h"       /* Seraph's cuda_train_context.h and cuda_profiler.h */
#include "lora.h"
#include "seraph_hip.h"

/* ------------------------------------------------------------------ private state */
typedef struct live_buf { cuda_buffer_t* buf; struct live_buf* next; } live_buf_t;

typedef struct {
    seraph_stream_t stream;
    live_buf_t* live;             /* buffers handed out and not yet freed */
    void* ws;                     /* grow-only kernel scratch */
    size_t ws_bytes;
    cuda_profiler_t* prof;
    int errors;
} hc_state_t;

static hc_state_t* state_of(cuda_train_context_t* ctx) { return ctx ? (hc_state_t*)ctx->stream : NULL; }

static void op_failed(hc_state_t* st, const char* what) {
    if (st->errors++ < 20) fprintf(stderr, "HIP: %s failed: %s\n", what, seraph_hip_last_error());
}

/* 1 when each of the `pairs` (buffer, number of 4-byte values) arguments fits its buffer (a NULL buffer is an optional
 * operand the op goes without).  Otherwise the op is refused with a message and nothing is launched: a shape that
 * reaches past the end of a buffer is a memory fault on this device, not the silent garbage it is elsewhere. */
#define FIT(buf, n) (const cuda_buffer_t*)(buf), (size_t)(n)
static int fits(hc_state_t* st, const char* op, int pairs, ...) {
    va_list ap;
    va_start(ap, pairs);
    int ok = 1;
    for (int i = 0; i < pairs; i++) {
        const cuda_buffer_t* buf = va_arg(ap, const cuda_buffer_t*);
        const size_t n = va_arg(ap, size_t);
        if (!buf || n <= buf->size / 4) continue;
        if (ok && st->errors++ < 20)
            fprintf(stderr, "HIP: %s skipped: operand %d has %zu bytes, the shape needs %zu\n", op, i, buf->size, n * 4);
        ok = 0;
    }
    va_end(ap);
    return ok;
}

static void* scratch(hc_state_t* st, size_t bytes) {
    if (bytes <= st->ws_bytes) return st->ws;
    seraph_hip_stream_sync(st->stream);
    if (st->ws) seraph_hip_free(st->ws);
    st->ws = NULL; st->ws_bytes = 0;
    if (seraph_hip_malloc(&st->ws, bytes) != SERAPH_OK) { op_failed(st, "scratch allocation"); return NULL; }
    st->ws_bytes = bytes;
    return st->ws;
}

/* ------------------------------------------------------------------ profiler (include/cuda_profiler.h) */
cuda_profiler_t* cuda_profiler_create(void) { return (cuda_profiler_t*)calloc(1, sizeof(cuda_profiler_t)); }

void cuda_profiler_destroy(cuda_profiler_t* p) {
    if (!p) return;
    for (int i = 0; i < PROFILER_MAX_OPS; i++) {
        if (p->ops[i].event_start) seraph_hip_event_destroy(p->ops[i].event_start);
        if (p->ops[i].event_end) seraph_hip_event_destroy(p->ops[i].event_end);
    }
    free(p);
}

static void prof_clear_totals(cuda_profiler_t* p) {
    p->total_step_ms = p->total_matmul_ms = p->total_attention_ms = p->total_attention_bwd_ms = 0.0f;
    p->total_rmsnorm_ms = p->total_rmsnorm_bwd_ms = p->total_cross_entropy_ms = p->total_adamw_ms = 0.0f;
    p->total_copy_ms = p->total_other_ms = 0.0f;
}

void cuda_profiler_enable(cuda_profiler_t* p) { if (p) { p->enabled = 1; p->num_ops = 0; } }
void cuda_profiler_disable(cuda_profiler_t* p) { if (p) p->enabled = 0; }
void cuda_profiler_reset(cuda_profiler_t* p) { if (p) { p->num_ops = 0; prof_clear_totals(p); } }
void cuda_profiler_set_log(cuda_profiler_t* p, void* file) { if (p) p->log_file = file; }

int cuda_profiler_begin_op(cuda_profiler_t* p, const char* name, void* stream) {
    hc_state_t* st = (hc_state_t*)stream;
    if (!p || !p->enabled || !st || p->num_ops >= PROFILER_MAX_OPS) return -1;
    profiler_op_t* op = &p->ops[p->num_ops];
    if (!op->event_start && (seraph_hip_event_create(&op->event_start) != SERAPH_OK ||
                             seraph_hip_event_create(&op->event_end) != SERAPH_OK)) return -1;
    void *e0 = op->event_start, *e1 = op->event_end;
    memset(op, 0, sizeof(*op));
    op->event_start = e0; op->event_end = e1;
    snprintf(op->name, sizeof(op->name), "%s", name ? name : "");
    seraph_hip_event_record(op->event_start, st->stream);
    return p->num_ops++;
}

void cuda_profiler_end_op(cuda_profiler_t* p, int idx, void* stream) {
    hc_state_t* st = (hc_state_t*)stream;
    if (!p || !p->enabled || !st || idx < 0 || idx >= p->num_ops) return;
    seraph_hip_event_record(p->ops[idx].event_end, st->stream);
}

void cuda_profiler_set_launch(cuda_profiler_t* p, int idx, int gx, int gy, int gz, int bx, int by, int bz, size_t smem) {
    if (!p || idx < 0 || idx >= p->num_ops) return;
    profiler_op_t* op = &p->ops[idx];
    op->grid_x = gx; op->grid_y = gy; op->grid_z = gz;
    op->block_x = bx; op->block_y = by; op->block_z = bz;
    op->shared_mem = smem;
}
void cuda_profiler_set_flops(cuda_profiler_t* p, int idx, size_t flops) { if (p && idx >= 0 && idx < p->num_ops) p->ops[idx].flops = flops; }
void cuda_profiler_set_bytes(cuda_profiler_t* p, int idx, size_t bytes) { if (p && idx >= 0 && idx < p->num_ops) p->ops[idx].bytes = bytes; }

/* the category an operation's time is booked under, chosen by name as src/cuda_profiler.cu:152-172 does */
static float* prof_bucket(cuda_profiler_t* p, const char* name) {
    static const struct { const char* needle; int which; } rules[] = {
        {"matmul", 0}, {"Matmul", 0}, {"attn_bwd", 1}, {"attention_bwd", 1}, {"attn", 2}, {"attention", 2},
        {"rmsnorm_bwd", 3}, {"rmsnorm", 4}, {"cross_entropy", 5}, {"adamw", 6}, {"copy", 7}, {"memset", 7}, {"memcpy", 7}};
    float* slots[8] = {&p->total_matmul_ms, &p->total_attention_bwd_ms, &p->total_attention_ms, &p->total_rmsnorm_bwd_ms,
                       &p->total_rmsnorm_ms, &p->total_cross_entropy_ms, &p->total_adamw_ms, &p->total_copy_ms};
    for (size_t i = 0; i < sizeof(rules) / sizeof(rules[0]); i++)
        if (strstr(name, rules[i].needle)) return slots[rules[i].which];
    return &p->total_other_ms;
}

/* An entry whose time is known already (the fused step reports a kernel class of a step as one entry): marked by a
 * shared-memory size no launch can have, so that the analysis keeps the time instead of asking the events. */
#define PROF_TIME_GIVEN ((size_t)-1)

cuda_profiler_t* hip_cuda_active_profiler(cuda_train_context_t* ctx) {
    hc_state_t* st = state_of(ctx);
    return (st && st->prof && st->prof->enabled) ? st->prof : NULL;
}

void hip_cuda_profiler_add(cuda_profiler_t* p, const char* name, float elapsed_ms, size_t flops, size_t bytes) {
    if (!p || !p->enabled || p->num_ops >= PROFILER_MAX_OPS) return;
    profiler_op_t* op = &p->ops[p->num_ops++];
    void *e0 = op->event_start, *e1 = op->event_end;          /* events made for this slot by an earlier step stay */
    memset(op, 0, sizeof(*op));
    op->event_start = e0; op->event_end = e1;
    snprintf(op->name, sizeof(op->name), "%s", name ? name : "");
    op->elapsed_ms = elapsed_ms;
    op->flops = flops; op->bytes = bytes;
    op->shared_mem = PROF_TIME_GIVEN;
}

void cuda_profiler_sync_and_analyze(cuda_profiler_t* p, void* stream) {
    hc_state_t* st = (hc_state_t*)stream;
    if (!p || p->num_ops == 0 || !st) return;
    seraph_hip_stream_sync(st->stream);
    prof_clear_totals(p);
    for (int i = 0; i < p->num_ops; i++) {
        profiler_op_t* op = &p->ops[i];
        if (op->shared_mem == PROF_TIME_GIVEN) {
            p->total_step_ms += op->elapsed_ms;
            *prof_bucket(p, op->name) += op->elapsed_ms;
            continue;
        }
        op->elapsed_ms = 0.0f;
        seraph_hip_event_elapsed_ms(op->event_start, op->event_end, &op->elapsed_ms);
        p->total_step_ms += op->elapsed_ms;
        *prof_bucket(p, op->name) += op->elapsed_ms;
    }
}

static void prof_out(cuda_profiler_t* p, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
#include <stdarg.h>
static void prof_out(cuda_profiler_t* p, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vprintf(fmt, ap);
    va_end(ap);
    if (p->log_file) {
        va_start(ap, fmt);
        vfprintf((FILE*)p->log_file, fmt, ap);
        va_end(ap);
    }
}

/* Same sections, column layouts and markers as src/cuda_profiler.cu:186-283, which tools that read
 * profile.log rely on. */
void cuda_profiler_print(cuda_profiler_t* p) {
    if (!p || p->num_ops == 0) { if (p) prof_out(p, "  [profiler] No operations recorded\n"); return; }
    const float total = p->total_step_ms > 0 ? p->total_step_ms : 1e-6f;
    static const char* const rule = "══════════════════════════════════════════════════════════════════";
    prof_out(p, "\n  %s\n  SERAPH STEP PROFILER (%d operations, %.2f ms total)\n  %s\n", rule, p->num_ops, p->total_step_ms, rule);
    prof_out(p, "\n  ── CATEGORY BREAKDOWN ──\n\n");
    prof_out(p, "  %-24s %10s  %6s  %s\n", "Category", "Time (ms)", "%", "Bar");
    prof_out(p, "  %-24s %10s  %6s  %s\n", "────────────────────────", "──────────", "──────", "────────────────────────────────────────");
    const char* names[9] = {"matmul (all)", "attention fwd", "attention bwd", "rmsnorm fwd", "rmsnorm bwd", "cross_entropy",
                            "adamw", "copy/memset", "other"};
    const float ms[9] = {p->total_matmul_ms, p->total_attention_ms, p->total_attention_bwd_ms, p->total_rmsnorm_ms,
                         p->total_rmsnorm_bwd_ms, p->total_cross_entropy_ms, p->total_adamw_ms, p->total_copy_ms, p->total_other_ms};
    for (int i = 0; i < 9; i++) {
        const float pct = 100.0f * ms[i] / total;
        char bar[41];
        int n = (int)(pct * 0.4f);
        if (n > 40) n = 40;
        if (n < 0) n = 0;
        memset(bar, '#', (size_t)n);
        bar[n] = '\0';
        prof_out(p, "  %-24s %10.3f  %5.1f%%  %s\n", names[i], ms[i], pct, bar);
    }
    prof_out(p, "\n  ── PER-OPERATION DETAIL ──\n\n");
    prof_out(p, "  %4s  %-60s %10s  %5s", "#", "Operation", "Time (ms)", "%");
    prof_out(p, "  %s\n", "Grid / Block");
    prof_out(p, "  %4s  %-60s %10s  %5s  %s\n", "────", "────────────────────────────────────────────────────────────",
             "──────────", "─────", "──────────────────");
    int with_perf = 0;
    for (int i = 0; i < p->num_ops; i++) {
        const profiler_op_t* op = &p->ops[i];
        const float pct = 100.0f * op->elapsed_ms / total;
        char launch[40] = "";
        if (op->block_x > 0) snprintf(launch, sizeof(launch), "%d/%d", op->grid_x, op->block_x);
        prof_out(p, "  %4d  %-60s %10.3f  %4.1f%%  %-20s%s\n", i, op->name, op->elapsed_ms, pct, launch,
                 pct > 5.0f ? " <<<" : pct > 1.0f ? " <<" : "");
        if (op->flops || op->bytes) with_perf = 1;
    }
    if (with_perf) {
        prof_out(p, "\n  ── PERFORMANCE METRICS ──\n\n");
        prof_out(p, "  %4s  %-40s %10s  %10s  %10s\n", "#", "Operation", "GFLOPS", "GB/s", "Time (ms)");
        prof_out(p, "  %4s  %-40s %10s  %10s  %10s\n", "────", "────────────────────────────────────────", "──────────", "──────────", "──────────");
        for (int i = 0; i < p->num_ops; i++) {
            const profiler_op_t* op = &p->ops[i];
            if (!op->flops && !op->bytes) continue;
            const float denom = op->elapsed_ms > 0 ? op->elapsed_ms * 1e6f : 0.0f;
            prof_out(p, "  %4d  %-40.40s %10.2f  %10.2f  %10.3f\n", i, op->name, denom > 0 ? (float)op->flops / denom : 0.0f,
                     denom > 0 ? (float)op->bytes / denom : 0.0f, op->elapsed_ms);
        }
    }
    prof_out(p, "\n");
}

static const cuda_profiler_t* g_sort_prof;
static int by_time_desc(const void* a, const void* b) {
    const float x = g_sort_prof->ops[*(const int*)a].elapsed_ms, y = g_sort_prof->ops[*(const int*)b].elapsed_ms;
    return x < y ? 1 : x > y ? -1 : (*(const int*)a - *(const int*)b);
}

void cuda_profiler_print_top(cuda_profiler_t* p, int top_n) {
    if (!p || p->num_ops == 0) return;
    int* order = (int*)malloc((size_t)p->num_ops * sizeof(int));
    if (!order) return;
    for (int i = 0; i < p->num_ops; i++) order[i] = i;
    g_sort_prof = p;
    qsort(order, (size_t)p->num_ops, sizeof(int), by_time_desc);
    const float total = p->total_step_ms > 0 ? p->total_step_ms : 1e-6f;
    prof_out(p, "\n  ── TOP %d SLOWEST OPERATIONS ──\n\n", top_n);
    prof_out(p, "  %4s  %-55s %10s  %5s\n", "Rank", "Operation", "Time (ms)", "%");
    prof_out(p, "  %4s  %-55s %10s  %5s\n", "────", "───────────────────────────────────────────────────────", "──────────", "─────");
    for (int i = 0; i < top_n && i < p->num_ops; i++) {
        const profiler_op_t* op = &p->ops[order[i]];
        prof_out(p, "  %4d  %-55.55s %10.3f  %4.1f%%\n", i + 1, op->name, op->elapsed_ms, 100.0f * op->elapsed_ms / total);
    }
    free(order);
}

void cuda_train_set_profiler(cuda_train_context_t* ctx, cuda_profiler_t* prof) {
    hc_state_t* st = state_of(ctx);
    if (st) st->prof = prof;
}

/* One kernel-library call, timed when a profiler is attached and enabled. */
#define RUN(ST, NAME, FLOPS, BYTES, CALL)                                               \
    do {                                                                                \
        hc_state_t* st_ = (ST);                                                         \
        const int pi_ = st_->prof ? cuda_profiler_begin_op(st_->prof, (NAME), st_) : -1; \
        const int rc_ = (CALL);                                                         \
        if (pi_ >= 0) {                                                                 \
            cuda_profiler_end_op(st_->prof, pi_, st_);                                  \
            st_->prof->ops[pi_].flops = (size_t)(FLOPS);                                \
            st_->prof->ops[pi_].bytes = (size_t)(BYTES);                                \
        }                                                                               \
        if (rc_ != SERAPH_OK) op_failed(st_, (NAME));                                   \
    } while (0)

/* ------------------------------------------------------------------ context (include/cuda_train_context.h:239-242) */
cuda_train_context_t* cuda_train_init(int device_id) {
    if (seraph_hip_init(device_id < 0 ? 0 : device_id) != SERAPH_OK) {
        fprintf(stderr, "HIP: Failed to set device %d: %s\n", device_id, seraph_hip_last_error());
        return NULL;
    }
    cuda_train_context_t* ctx = (cuda_train_context_t*)calloc(1, sizeof(*ctx));
    hc_state_t* st = (hc_state_t*)calloc(1, sizeof(*st));
    if (!ctx || !st || seraph_hip_stream_create(&st->stream) != SERAPH_OK) {
        fprintf(stderr, "HIP: Failed to create stream: %s\n", seraph_hip_last_error());
        free(ctx); free(st);
        return NULL;
    }
    seraph_device_info_t info;
    memset(&info, 0, sizeof(info));
    seraph_hip_device_info(&info);
    ctx->device_id = device_id < 0 ? 0 : device_id;
    ctx->stream = st;
    ctx->initialized = 1;
    ctx->gpu_sm_count = (int)info.compute_units;
    ctx->gpu_warp_size = (int)info.wavefront_size;
    /* the trainer sizes its loss-reduction passes by this number (src/train_cuda.c:2239-2250):
     * it is the fan-in of reduce_sum below, not the hardware's launch limit */
    ctx->gpu_max_threads_per_block = 512;
    ctx->gpu_shared_mem_per_block = (int)info.lds_bytes_per_block;
    ctx->gpu_shared_mem_per_sm = 160 * 1024;
    ctx->gpu_max_shared_per_block_optin = (int)info.lds_bytes_per_block;
    ctx->gpu_max_threads_per_sm = 2048;
    ctx->gpu_regs_per_sm = 4 * 512 * 64;
    ctx->gpu_l2_cache_bytes = 4 * 1024 * 1024;
    ctx->gpu_compute_major = 0;                    /* not a CUDA device: --bf16 falls back to FP32 in the front end */
    ctx->gpu_compute_minor = 0;
    ctx->matmul_tile_dim = 128;
    ctx->matmul_block_k = 32;
    ctx->parallel_block_size = 256;
    ctx->attention_block_size = 256;
    ctx->attention_num_warps = 4;
    printf("  HIP device: %s (%s), %u CUs, %.0f GB\n", info.name, info.arch, info.compute_units, (double)info.hbm_bytes / 1e9);
    return ctx;
}

void cuda_train_get_gpu_info(cuda_train_context_t* ctx, char* name, int name_len, float* memory_gb) {
    (void)ctx;
    seraph_device_info_t info;
    memset(&info, 0, sizeof(info));
    seraph_hip_device_info(&info);
    if (name && name_len > 0) snprintf(name, (size_t)name_len, "%s", info.name);
    if (memory_gb) *memory_gb = (float)((double)info.hbm_bytes / (1024.0 * 1024.0 * 1024.0));
}

void cuda_train_sync(cuda_train_context_t* ctx) {
    hc_state_t* st = state_of(ctx);
    if (st) seraph_hip_stream_sync(st->stream);
}

/* ------------------------------------------------------------------ buffers (:248-256) */
cuda_buffer_t* cuda_train_buffer_create(cuda_train_context_t* ctx, size_t size) {
    hc_state_t* st = state_of(ctx);
    cuda_buffer_t* buf = (cuda_buffer_t*)malloc(sizeof(*buf));
    live_buf_t* node = st ? (live_buf_t*)malloc(sizeof(*node)) : NULL;
    void* dev = NULL;
    if (!buf || (st && !node) || seraph_hip_malloc(&dev, size ? size : 4) != SERAPH_OK) {
        fprintf(stderr, "HIP: Failed to allocate %zu bytes: %s\n", size, seraph_hip_last_error());
        free(buf); free(node);
        return NULL;
    }
    buf->data = (float*)dev;
    buf->size = size;
    if (node) { node->buf = buf; node->next = st->live; st->live = node; }
    return buf;
}

void cuda_train_buffer_free(cuda_train_context_t* ctx, cuda_buffer_t* buf) {
    if (!buf) return;
    hc_state_t* st = state_of(ctx);
    if (st) {
        seraph_hip_stream_sync(st->stream);             /* work queued on the buffer finishes first */
        for (live_buf_t** p = &st->live; *p; p = &(*p)->next)
            if ((*p)->buf == buf) { live_buf_t* dead = *p; *p = dead->next; free(dead); break; }
    }
    if (buf->data) seraph_hip_free(buf->data);
    free(buf);
}

void cuda_train_buffer_upload(cuda_train_context_t* ctx, cuda_buffer_t* buf, const float* data, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (!st || !buf || !data) return;
    if (seraph_hip_h2d(buf->data, data, count * sizeof(float), st->stream) != SERAPH_OK) op_failed(st, "buffer_upload");
}
void cuda_train_buffer_upload_u32(cuda_train_context_t* ctx, cuda_buffer_t* buf, const uint32_t* data, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (!st || !buf || !data) return;
    if (seraph_hip_h2d(buf->data, data, count * sizeof(uint32_t), st->stream) != SERAPH_OK) op_failed(st, "buffer_upload_u32");
}
void cuda_train_buffer_download(cuda_train_context_t* ctx, cuda_buffer_t* buf, float* data, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (!st || !buf || !data) return;
    if (seraph_hip_d2h(data, buf->data, count * sizeof(float), st->stream) != SERAPH_OK) op_failed(st, "buffer_download");
}
void cuda_train_buffer_download_bytes(cuda_train_context_t* ctx, cuda_buffer_t* buf, void* data, size_t bytes) {
    hc_state_t* st = state_of(ctx);
    if (!st || !buf || !data) return;
    if (seraph_hip_d2h(data, buf->data, bytes, st->stream) != SERAPH_OK) op_failed(st, "buffer_download_bytes");
}

void cuda_train_fill_buffer_range(cuda_train_context_t* ctx, cuda_buffer_t* buf, size_t offset, uint32_t value, size_t bytes) {
    hc_state_t* st = state_of(ctx);
    if (!st || !buf || bytes < 4) return;
    const uint32_t pattern = (value & 0xFFu) * 0x01010101u;                  /* memset semantics: one byte repeated */
    RUN(st, "memset", 0, bytes, seraph_fill_u32((char*)buf->data + (offset & ~(size_t)3), pattern, bytes / 4, st->stream));
}
void cuda_train_fill_buffer(cuda_train_context_t* ctx, cuda_buffer_t* buf, uint32_t value, size_t bytes) {
    cuda_train_fill_buffer_range(ctx, buf, 0, value, bytes);
}
void cuda_train_copy_buffer(cuda_train_context_t* ctx, cuda_buffer_t* src, cuda_buffer_t* dst, size_t bytes) {
    hc_state_t* st = state_of(ctx);
    if (!st || !src || !dst) return;
    RUN(st, "memcpy d2d", 0, 2 * bytes, seraph_hip_d2d(dst->data, src->data, bytes, st->stream));
}

/* ------------------------------------------------------------------ forward ops (:263-275) */
static void gemm_op(cuda_train_context_t* ctx, const char* label, const float* A, const float* B, float* C,
                    int M, int N, int K, int tA, int tB, int acc) {
    hc_state_t* st = state_of(ctx);
    if (!st) return;
    char name[80];
    snprintf(name, sizeof(name), "%s [%dx%d K=%d]%s", label, M, N, K, acc ? " +=" : "");
    /* a small output with a long K runs in slices of K through the scratch; other shapes are the plain product */
    const size_t need = seraph_gemm_scaled_ws_bytes(M, N, K, tA, tB);
    void* ws = need ? scratch(st, need) : NULL;
    RUN(st, name, (size_t)2 * (size_t)M * (size_t)N * (size_t)K, 0,
        seraph_gemm_scaled(A, B, C, M, N, K, tA, tB, acc, 1.0f, ws, ws ? need : 0, st->stream));
}

/* (The reference's batched LoRA step hands every adapter the final hidden gradient as its output gradient,
 * src/train_cuda.c:2596-2644, which is smaller than tokens x out_dim for any adapter whose out_dim exceeds hidden_size:
 * the products check their operands like every other op here.) */
static int gemm_fits(cuda_train_context_t* ctx, const char* label, const cuda_buffer_t* A, const cuda_buffer_t* B, const cuda_buffer_t* C,
                     int M, int N, int K) {
    hc_state_t* st = state_of(ctx);
    if (!st || M < 0 || N < 0 || K < 0) return 0;
    char name[80];
    snprintf(name, sizeof(name), "%s [%dx%d K=%d]", label, M, N, K);
    return fits(st, name, 3, FIT(A, (size_t)M * K), FIT(B, (size_t)N * K), FIT(C, (size_t)M * N));
}
static void gemm_bufs(cuda_train_context_t* ctx, const char* label, cuda_buffer_t* A, cuda_buffer_t* B, cuda_buffer_t* C,
                      int M, int N, int K, int tA, int tB, int acc) {
    if (A && B && C && gemm_fits(ctx, label, A, B, C, M, N, K)) gemm_op(ctx, label, A->data, B->data, C->data, M, N, K, tA, tB, acc);
}

void cuda_train_matmul(cuda_train_context_t* ctx, cuda_buffer_t* A, cuda_buffer_t* B, cuda_buffer_t* C, int M, int N, int K) {
    gemm_bufs(ctx, "matmul", A, B, C, M, N, K, 0, 0, 0);
}
void cuda_train_matmul_transpose(cuda_train_context_t* ctx, cuda_buffer_t* A, cuda_buffer_t* B, cuda_buffer_t* C, int M, int N, int K,
                                 int transpose_A, int transpose_B, int accumulate) {
    const char* label = (transpose_A && !transpose_B) ? "matmul_At" : (!transpose_A && transpose_B) ? "matmul_Bt" : "matmul";
    gemm_bufs(ctx, label, A, B, C, M, N, K, transpose_A, transpose_B, accumulate);
}

void cuda_train_silu(cuda_train_context_t* ctx, cuda_buffer_t* input, cuda_buffer_t* output, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (st && input && output && fits(st, "silu", 2, FIT(input, count), FIT(output, count))) RUN(st, "silu", 0, 8 * count, seraph_silu(input->data, output->data, count, st->stream));
}
void cuda_train_rmsnorm(cuda_train_context_t* ctx, cuda_buffer_t* input, cuda_buffer_t* scale, cuda_buffer_t* output, int rows, int cols, float eps) {
    hc_state_t* st = state_of(ctx);
    if (!st || !input || !scale || !output || rows < 0 || cols < 0) return;
    char name[80];
    snprintf(name, sizeof(name), "rmsnorm [%dx%d]", rows, cols);
    if (!fits(st, name, 3, FIT(input, (size_t)rows * cols), FIT(scale, cols), FIT(output, (size_t)rows * cols))) return;
    RUN(st, name, 0, (size_t)8 * rows * cols, seraph_rmsnorm(input->data, scale->data, output->data, rows, cols, eps, st->stream));
}
void cuda_train_rope(cuda_train_context_t* ctx, cuda_buffer_t* x_in, cuda_buffer_t* x_out, int seq_len, int num_heads, int head_dim, float rope_theta) {
    hc_state_t* st = state_of(ctx);
    if (st && x_in && x_out && seq_len >= 0 && num_heads >= 0 && head_dim >= 0 &&
        fits(st, "rope_fwd", 2, FIT(x_in, (size_t)seq_len * num_heads * head_dim), FIT(x_out, (size_t)seq_len * num_heads * head_dim)))
        RUN(st, "rope_fwd", 0, (size_t)8 * seq_len * num_heads * head_dim,
                                 seraph_rope(x_in->data, x_out->data, NULL, 1, seq_len, num_heads, head_dim, rope_theta, 0, st->stream));
}
void cuda_train_rope_packed(cuda_train_context_t* ctx, cuda_buffer_t* x_in, cuda_buffer_t* x_out, cuda_buffer_t* seq_starts,
                            int total_tokens, int batch_size, int num_heads, int head_dim, float rope_theta) {
    hc_state_t* st = state_of(ctx);
    if (st && x_in && x_out && seq_starts && total_tokens >= 0 && batch_size >= 0 && num_heads >= 0 && head_dim >= 0 &&
        fits(st, "rope_fwd_packed", 3, FIT(x_in, (size_t)total_tokens * num_heads * head_dim), FIT(x_out, (size_t)total_tokens * num_heads * head_dim),
             FIT(seq_starts, (size_t)batch_size + 1)))
        RUN(st, "rope_fwd_packed", 0, (size_t)8 * total_tokens * num_heads * head_dim,
            seraph_rope(x_in->data, x_out->data, (const uint32_t*)seq_starts->data, batch_size, total_tokens, num_heads, head_dim, rope_theta, 0, st->stream));
}
void cuda_train_add(cuda_train_context_t* ctx, cuda_buffer_t* A, cuda_buffer_t* B, cuda_buffer_t* C, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (st && A && B && C && fits(st, "add", 3, FIT(A, count), FIT(B, count), FIT(C, count))) RUN(st, "add", 0, 12 * count, seraph_add(A->data, B->data, C->data, count, st->stream));
}
void cuda_train_mul(cuda_train_context_t* ctx, cuda_buffer_t* A, cuda_buffer_t* B, cuda_buffer_t* C, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (st && A && B && C && fits(st, "mul", 3, FIT(A, count), FIT(B, count), FIT(C, count))) RUN(st, "mul", 0, 12 * count, seraph_mul(A->data, B->data, C->data, count, st->stream));
}
void cuda_train_scale(cuda_train_context_t* ctx, cuda_buffer_t* A, size_t count, float alpha) {
    hc_state_t* st = state_of(ctx);
    if (st && A && fits(st, "scale", 1, FIT(A, count))) RUN(st, "scale", 0, 8 * count, seraph_scale(A->data, count, alpha, st->stream));
}

static void attention_fwd(cuda_train_context_t* ctx, const char* name, cuda_buffer_t* Q, cuda_buffer_t* K, cuda_buffer_t* V,
                          cuda_buffer_t* out, cuda_buffer_t* lse_out, const uint32_t* starts, int batch, int T, int H, int KVH, int D) {
    hc_state_t* st = state_of(ctx);
    if (!st || !Q || !K || !V || !out || batch < 0 || T < 0 || H < 0 || KVH < 0 || D < 0) return;
    if (!fits(st, name, 5, FIT(Q, (size_t)T * H * D), FIT(K, (size_t)T * KVH * D), FIT(V, (size_t)T * KVH * D), FIT(out, (size_t)T * H * D),
              FIT(lse_out, (size_t)T * H)))
        return;
    /* the reference's standard kernel ignores lse_out (:2855); writing it costs nothing here and lets the
     * backward skip its recomputation in both modes - same numbers either way */
    float* lse = lse_out ? lse_out->data : NULL;
    RUN(st, name, 0, 0, seraph_attention_forward(Q->data, K->data, V->data, out->data, lse, starts, batch, T, H, KVH, D,
                                                 1.0f / sqrtf((float)D), st->stream));
}
void cuda_train_batch_attention(cuda_train_context_t* ctx, cuda_buffer_t* Q, cuda_buffer_t* K, cuda_buffer_t* V, cuda_buffer_t* out,
                                cuda_buffer_t* lse_out, int seq_len, int num_heads, int kv_heads, int head_dim) {
    char name[80];
    snprintf(name, sizeof(name), "%s [seq=%d h=%d hd=%d]", ctx && ctx->use_flash_attn ? "flash_attn_fwd" : "attn_fwd", seq_len, num_heads, head_dim);
    attention_fwd(ctx, name, Q, K, V, out, lse_out, NULL, 1, seq_len, num_heads, kv_heads, head_dim);
}
void cuda_train_batch_attention_packed(cuda_train_context_t* ctx, cuda_buffer_t* Q, cuda_buffer_t* K, cuda_buffer_t* V, cuda_buffer_t* out,
                                       cuda_buffer_t* lse_out, cuda_buffer_t* seq_starts, int total_tokens, int batch_size,
                                       int num_heads, int kv_heads, int head_dim, int max_seq_in_batch) {
    (void)max_seq_in_batch;
    hc_state_t* st = state_of(ctx);
    if (!st || !seq_starts || batch_size < 0 || !fits(st, "attn_fwd_packed", 1, FIT(seq_starts, (size_t)batch_size + 1))) return;
    attention_fwd(ctx, ctx && ctx->use_flash_attn ? "flash_attn_fwd_packed" : "attn_fwd_packed", Q, K, V, out, lse_out,
                  (const uint32_t*)seq_starts->data, batch_size, total_tokens, num_heads, kv_heads, head_dim);
}

void cuda_train_embed_lookup(cuda_train_context_t* ctx, cuda_buffer_t* tokens_u32, cuda_buffer_t* embed_weight, cuda_buffer_t* out_hidden,
                             int seq_len, int hidden_size, int vocab_size) {
    hc_state_t* st = state_of(ctx);
    if (st && tokens_u32 && embed_weight && out_hidden && seq_len >= 0 && hidden_size >= 0 && vocab_size >= 0 &&
        fits(st, "embed_lookup", 3, FIT(tokens_u32, seq_len), FIT(embed_weight, (size_t)vocab_size * hidden_size), FIT(out_hidden, (size_t)seq_len * hidden_size)))
        RUN(st, "embed_lookup", 0, (size_t)8 * seq_len * hidden_size,
            seraph_embed_lookup((const uint32_t*)tokens_u32->data, embed_weight->data, out_hidden->data, seq_len, hidden_size, vocab_size, st->stream));
}

/* ------------------------------------------------------------------ loss and backward ops (:278-294) */
void cuda_train_cross_entropy_grad(cuda_train_context_t* ctx, cuda_buffer_t* logits, cuda_buffer_t* targets_u32, cuda_buffer_t* grad_logits,
                                   cuda_buffer_t* loss_rows, int rows, int cols) {
    hc_state_t* st = state_of(ctx);
    if (!st || !logits || !targets_u32 || !grad_logits || !loss_rows || rows < 0 || cols < 0) return;
    char name[80];
    snprintf(name, sizeof(name), "cross_entropy [%dx%d]", rows, cols);
    if (!fits(st, name, 4, FIT(logits, (size_t)rows * cols), FIT(targets_u32, rows), FIT(grad_logits, (size_t)rows * cols), FIT(loss_rows, rows))) return;
    RUN(st, name, 0, (size_t)rows * cols * 4 * 3,
        seraph_cross_entropy_grad(logits->data, (const uint32_t*)targets_u32->data, grad_logits->data, loss_rows->data, NULL, 1, rows, cols, rows, st->stream));
}
void cuda_train_cross_entropy_grad_packed(cuda_train_context_t* ctx, cuda_buffer_t* logits, cuda_buffer_t* targets_u32, cuda_buffer_t* grad_logits,
                                          cuda_buffer_t* loss_rows, cuda_buffer_t* seq_starts, int total_tokens, int batch_size, int vocab_size,
                                          int num_valid_predictions) {
    hc_state_t* st = state_of(ctx);
    if (!st || !logits || !targets_u32 || !grad_logits || !loss_rows || !seq_starts || total_tokens < 0 || batch_size < 0 || vocab_size < 0) return;
    if (!fits(st, "cross_entropy_packed", 5, FIT(logits, (size_t)total_tokens * vocab_size), FIT(targets_u32, total_tokens),
              FIT(grad_logits, (size_t)total_tokens * vocab_size), FIT(loss_rows, total_tokens), FIT(seq_starts, (size_t)batch_size + 1)))
        return;
    RUN(st, "cross_entropy_packed", 0, (size_t)total_tokens * vocab_size * 8,
        seraph_cross_entropy_grad(logits->data, (const uint32_t*)targets_u32->data, grad_logits->data, loss_rows->data,
                                  (const uint32_t*)seq_starts->data, batch_size, total_tokens, vocab_size, num_valid_predictions, st->stream));
}
void cuda_train_reduce_sum(cuda_train_context_t* ctx, cuda_buffer_t* in_buf, cuda_buffer_t* out_buf, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (st && in_buf && out_buf && count && fits(st, "reduce_sum", 2, FIT(in_buf, count), FIT(out_buf, (count + 511) / 512))) RUN(st, "reduce_sum", 0, 4 * count, seraph_reduce_sum(in_buf->data, out_buf->data, count, st->stream));
}
void cuda_train_silu_backward(cuda_train_context_t* ctx, cuda_buffer_t* input, cuda_buffer_t* grad_output, cuda_buffer_t* grad_input, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (st && input && grad_output && grad_input && fits(st, "silu_bwd", 3, FIT(input, count), FIT(grad_output, count), FIT(grad_input, count)))
        RUN(st, "silu_bwd", 0, 12 * count, seraph_silu_backward(input->data, grad_output->data, grad_input->data, count, st->stream));
}
void cuda_train_elementwise_mul_backward(cuda_train_context_t* ctx, cuda_buffer_t* A, cuda_buffer_t* B, cuda_buffer_t* grad_C,
                                         cuda_buffer_t* grad_A, cuda_buffer_t* grad_B, size_t count) {
    hc_state_t* st = state_of(ctx);
    if (st && A && B && grad_C && grad_A && grad_B &&
        fits(st, "mul_bwd", 5, FIT(A, count), FIT(B, count), FIT(grad_C, count), FIT(grad_A, count), FIT(grad_B, count)))
        RUN(st, "mul_bwd", 0, 20 * count, seraph_mul_backward(A->data, B->data, grad_C->data, grad_A->data, grad_B->data, count, st->stream));
}
void cuda_train_rmsnorm_backward_batch(cuda_train_context_t* ctx, cuda_buffer_t* input, cuda_buffer_t* scale, cuda_buffer_t* grad_output,
                                       cuda_buffer_t* grad_input, cuda_buffer_t* grad_scale, int rows, int cols, float eps) {
    hc_state_t* st = state_of(ctx);
    if (!st || !input || !scale || !grad_output || !grad_input || !grad_scale || rows < 0 || cols < 0) return;
    if (!fits(st, "rmsnorm_bwd", 5, FIT(input, (size_t)rows * cols), FIT(scale, cols), FIT(grad_output, (size_t)rows * cols),
              FIT(grad_input, (size_t)rows * cols), FIT(grad_scale, cols)))
        return;
    void* ws = scratch(st, seraph_rmsnorm_backward_ws_bytes(rows, cols));
    if (!ws) return;
    char name[80];
    snprintf(name, sizeof(name), "rmsnorm_bwd [%dx%d]", rows, cols);
    RUN(st, name, 0, (size_t)12 * rows * cols,
        seraph_rmsnorm_backward(input->data, scale->data, grad_output->data, grad_input->data, grad_scale->data, rows, cols, eps, ws, st->ws_bytes, st->stream));
}
void cuda_train_rope_backward(cuda_train_context_t* ctx, cuda_buffer_t* x_in, cuda_buffer_t* x_out, int seq_len, int num_heads, int head_dim, float rope_theta) {
    hc_state_t* st = state_of(ctx);
    if (st && x_in && x_out && seq_len >= 0 && num_heads >= 0 && head_dim >= 0 &&
        fits(st, "rope_bwd", 2, FIT(x_in, (size_t)seq_len * num_heads * head_dim), FIT(x_out, (size_t)seq_len * num_heads * head_dim)))
        RUN(st, "rope_bwd", 0, (size_t)8 * seq_len * num_heads * head_dim,
                                 seraph_rope(x_in->data, x_out->data, NULL, 1, seq_len, num_heads, head_dim, rope_theta, 1, st->stream));
}
void cuda_train_rope_backward_packed(cuda_train_context_t* ctx, cuda_buffer_t* x_in, cuda_buffer_t* x_out, cuda_buffer_t* seq_starts,
                                     int total_tokens, int batch_size, int num_heads, int head_dim, float rope_theta) {
    hc_state_t* st = state_of(ctx);
    if (st && x_in && x_out && seq_starts && total_tokens >= 0 && batch_size >= 0 && num_heads >= 0 && head_dim >= 0 &&
        fits(st, "rope_bwd_packed", 3, FIT(x_in, (size_t)total_tokens * num_heads * head_dim), FIT(x_out, (size_t)total_tokens * num_heads * head_dim),
             FIT(seq_starts, (size_t)batch_size + 1)))
        RUN(st, "rope_bwd_packed", 0, (size_t)8 * total_tokens * num_heads * head_dim,
            seraph_rope(x_in->data, x_out->data, (const uint32_t*)seq_starts->data, batch_size, total_tokens, num_heads, head_dim, rope_theta, 1, st->stream));
}

static void attention_bwd(cuda_train_context_t* ctx, const char* name, cuda_buffer_t* Q, cuda_buffer_t* K, cuda_buffer_t* V,
                          cuda_buffer_t* attn_out, cuda_buffer_t* lse, cuda_buffer_t* grad_out, cuda_buffer_t* gQ, cuda_buffer_t* gK,
                          cuda_buffer_t* gV, const uint32_t* starts, int batch, int T, int H, int KVH, int D, int max_seq) {
    hc_state_t* st = state_of(ctx);
    if (!st || !Q || !K || !V || !grad_out || !gQ || !gK || !gV || batch < 0 || T < 0 || H < 0 || KVH < 0 || D < 0) return;
    const size_t nq = (size_t)T * H * D, nkv = (size_t)T * KVH * D;
    if (!fits(st, name, 9, FIT(Q, nq), FIT(K, nkv), FIT(V, nkv), FIT(attn_out, nq), FIT(lse, (size_t)T * H), FIT(grad_out, nq), FIT(gQ, nq),
              FIT(gK, nkv), FIT(gV, nkv)))
        return;
    const int saved = attn_out && lse;             /* both come from attention_fwd above; else recomputed */
    size_t need = seraph_attention_backward_ws_bytes_banded(T, H, KVH, D, max_seq);
    if (need > ((size_t)8 << 30)) need = seraph_attention_backward_ws_bytes(T, H, KVH, D);
    void* ws = scratch(st, need);
    if (!ws) return;
    RUN(st, name, 0, 0, seraph_attention_backward_banded(Q->data, K->data, V->data, grad_out->data, saved ? attn_out->data : NULL,
                                                         saved ? lse->data : NULL, gQ->data, gK->data, gV->data, starts, batch, T, H, KVH, D,
                                                         1.0f / sqrtf((float)D), max_seq, ws, st->ws_bytes, st->stream));
}
void cuda_train_batch_attention_backward(cuda_train_context_t* ctx, cuda_buffer_t* Q, cuda_buffer_t* K, cuda_buffer_t* V, cuda_buffer_t* attn_out,
                                         cuda_buffer_t* lse, cuda_buffer_t* grad_out, cuda_buffer_t* grad_Q, cuda_buffer_t* grad_K,
                                         cuda_buffer_t* grad_V, int seq_len, int num_heads, int kv_heads, int head_dim) {
    char name[80];
    snprintf(name, sizeof(name), "%s [seq=%d h=%d hd=%d]", ctx && ctx->use_flash_attn ? "flash_attn_bwd" : "attn_bwd", seq_len, num_heads, head_dim);
    attention_bwd(ctx, name, Q, K, V, attn_out, lse, grad_out, grad_Q, grad_K, grad_V, NULL, 1, seq_len, num_heads, kv_heads, head_dim, seq_len);
}
void cuda_train_batch_attention_backward_packed(cuda_train_context_t* ctx, cuda_buffer_t* Q, cuda_buffer_t* K, cuda_buffer_t* V,
                                                cuda_buffer_t* attn_out, cuda_buffer_t* lse, cuda_buffer_t* grad_out, cuda_buffer_t* grad_Q,
                                                cuda_buffer_t* grad_K, cuda_buffer_t* grad_V, cuda_buffer_t* seq_starts, int total_tokens,
                                                int batch_size, int num_heads, int kv_heads, int head_dim, int max_seq_in_batch) {
    hc_state_t* st = state_of(ctx);
    if (!st || !seq_starts || batch_size < 0 || !fits(st, "attn_bwd_packed", 1, FIT(seq_starts, (size_t)batch_size + 1))) return;
    attention_bwd(ctx, ctx && ctx->use_flash_attn ? "flash_attn_bwd_packed" : "attn_bwd_packed", Q, K, V, attn_out, lse, grad_out, grad_Q,
                  grad_K, grad_V, (const uint32_t*)seq_starts->data, batch_size, total_tokens, num_heads, kv_heads, head_dim,
                  max_seq_in_batch > 0 ? max_seq_in_batch : total_tokens);
}

void cuda_train_embedding_backward(cuda_train_context_t* ctx, cuda_buffer_t* tokens_u32, cuda_buffer_t* grad_hidden, cuda_buffer_t* grad_embed,
                                   int seq_len, int hidden_size, int vocab_size) {
    hc_state_t* st = state_of(ctx);
    if (!st || !tokens_u32 || !grad_hidden || !grad_embed || seq_len < 0 || hidden_size < 0 || vocab_size < 0) return;
    if (!fits(st, "embed_bwd", 3, FIT(tokens_u32, seq_len), FIT(grad_hidden, (size_t)seq_len * hidden_size), FIT(grad_embed, (size_t)vocab_size * hidden_size)))
        return;
    void* ws = scratch(st, seraph_embedding_backward_ws_bytes(seq_len, vocab_size));
    if (!ws) return;
    RUN(st, "embed_bwd", 0, (size_t)12 * seq_len * hidden_size,
        seraph_embedding_backward((const uint32_t*)tokens_u32->data, grad_hidden->data, grad_embed->data, seq_len, hidden_size, vocab_size,
                                  ws, st->ws_bytes, st->stream));
}

void cuda_train_adamw_update(cuda_train_context_t* ctx, cuda_buffer_t* weight, cuda_buffer_t* grad, cuda_buffer_t* m, cuda_buffer_t* v,
                             float lr, float beta1, float beta2, float weight_decay, float eps, int step, size_t size,
                             const char* tensor_name, int rows, int cols) {
    hc_state_t* st = state_of(ctx);
    if (!st || !weight || !grad || !m || !v) return;
    char name[80];
    if (cols > 0) snprintf(name, sizeof(name), "adamw %s [%dx%d]", tensor_name ? tensor_name : "", rows, cols);
    else snprintf(name, sizeof(name), "adamw %s [%d]", tensor_name ? tensor_name : "", rows);
    if (!fits(st, name, 4, FIT(weight, size), FIT(grad, size), FIT(m, size), FIT(v, size))) return;
    RUN(st, name, 0, size * 4 * 4, seraph_adamw(weight->data, grad->data, m->data, v->data, size, lr, beta1, beta2, weight_decay, eps, step, 0.0f, st->stream));
}

void cuda_train_nan_check(cuda_train_context_t* ctx, cuda_buffer_t* input, size_t count_floats, cuda_buffer_t* flags_u32, uint32_t flag_index) {
    hc_state_t* st = state_of(ctx);
    if (st && input && flags_u32 && fits(st, "nan_check", 2, FIT(input, count_floats), FIT(flags_u32, (size_t)flag_index + 1))) RUN(st, "nan_check", 0, 4 * count_floats,
                                      seraph_nan_check(input->data, count_floats, (uint32_t*)flags_u32->data, flag_index, st->stream));
}

/* ------------------------------------------------------------------ LoRA (:309-325) */
/* gB += (dY^T (x A^T s)),  gA += ((dY B s)^T x): the four products of src/cuda_train_context.cu:3240-3279 */
void cuda_train_lora_backward(cuda_train_context_t* ctx, cuda_buffer_t* grad_output, cuda_buffer_t* input, cuda_buffer_t* A, cuda_buffer_t* B,
                              cuda_buffer_t* gA, cuda_buffer_t* gB, cuda_buffer_t* hidden_tmp, int seq_len, int in_dim, int out_dim, int rank,
                              float scale) {
    if (!grad_output || !input || !A || !B || !gA || !gB || !hidden_tmp) return;
    const size_t n = (size_t)seq_len * (size_t)rank;
    /* all four products or none: a half-updated adapter would be worse than an untouched one */
    if (!gemm_fits(ctx, "lora_recompute", input, A, hidden_tmp, seq_len, rank, in_dim) ||
        !gemm_fits(ctx, "lora_gB", grad_output, hidden_tmp, gB, out_dim, rank, seq_len) ||
        !gemm_fits(ctx, "lora_grad_hidden", grad_output, B, hidden_tmp, seq_len, rank, out_dim) ||
        !gemm_fits(ctx, "lora_gA", hidden_tmp, input, gA, rank, in_dim, seq_len))
        return;
    gemm_op(ctx, "lora_recompute", input->data, A->data, hidden_tmp->data, seq_len, rank, in_dim, 0, 1, 0);
    cuda_train_scale(ctx, hidden_tmp, n, scale);
    gemm_op(ctx, "lora_gB", grad_output->data, hidden_tmp->data, gB->data, out_dim, rank, seq_len, 1, 0, 1);
    gemm_op(ctx, "lora_grad_hidden", grad_output->data, B->data, hidden_tmp->data, seq_len, rank, out_dim, 0, 0, 0);
    cuda_train_scale(ctx, hidden_tmp, n, scale);
    gemm_op(ctx, "lora_gA", hidden_tmp->data, input->data, gA->data, rank, in_dim, seq_len, 1, 0, 1);
}

static cuda_lora_gpu_adapter_t* lora_kinds(cuda_lora_gpu_state_t* lg, int i) {
    cuda_lora_gpu_adapter_t* all[7] = {&lg->q, &lg->k, &lg->v, &lg->o, &lg->gate, &lg->up, &lg->down};
    return all[i];
}

void cuda_train_zero_lora_grads(cuda_train_context_t* ctx) {
    if (!ctx || !ctx->lora_gpu) return;
    cuda_lora_gpu_state_t* lg = (cuda_lora_gpu_state_t*)ctx->lora_gpu;
    for (int k = 0; k < 7; k++) {
        cuda_lora_gpu_adapter_t* a = lora_kinds(lg, k);
        if (!a->active) continue;
        for (int l = 0; l < lg->num_layers; l++) {
            if (a->gA && a->gA[l]) cuda_train_fill_buffer(ctx, a->gA[l], 0, a->gA[l]->size);
            if (a->gB && a->gB[l]) cuda_train_fill_buffer(ctx, a->gB[l], 0, a->gB[l]->size);
        }
    }
}

void cuda_download_lora_weights(cuda_train_context_t* ctx, void* lora_ptr) {
    if (!ctx || !ctx->lora_gpu || !lora_ptr) return;
    lora_model_t* lora = (lora_model_t*)lora_ptr;
    cuda_lora_gpu_state_t* lg = (cuda_lora_gpu_state_t*)ctx->lora_gpu;
    lora_adapter_t** host[7] = {lora->q_adapters, lora->k_adapters, lora->v_adapters, lora->o_adapters,
                                lora->gate_adapters, lora->up_adapters, lora->down_adapters};
    for (int k = 0; k < 7; k++) {
        cuda_lora_gpu_adapter_t* g = lora_kinds(lg, k);
        if (!g->active || !host[k]) continue;
        for (int l = 0; l < lg->num_layers; l++) {
            lora_adapter_t* a = host[k][l];
            if (!a) continue;
            const size_t na = (size_t)a->rank * (size_t)a->in_dim, nb = (size_t)a->out_dim * (size_t)a->rank;
            if (g->A && g->A[l]) cuda_train_buffer_download(ctx, g->A[l], a->A, na);
            if (g->B && g->B[l]) cuda_train_buffer_download(ctx, g->B[l], a->B, nb);
            if (g->mA && g->mA[l]) cuda_train_buffer_download(ctx, g->mA[l], a->m_A, na);      /* moments too, for resume */
            if (g->vA && g->vA[l]) cuda_train_buffer_download(ctx, g->vA[l], a->v_A, na);
            if (g->mB && g->mB[l]) cuda_train_buffer_download(ctx, g->mB[l], a->m_B, nb);
            if (g->vB && g->vB[l]) cuda_train_buffer_download(ctx, g->vB[l], a->v_B, nb);
        }
    }
    cuda_train_sync(ctx);
}

/* ------------------------------------------------------------------ teardown (:240) */
/* Every device buffer the trainer created through cuda_train_buffer_create is on the live list:
 * releasing the list releases the context's weights, moments, caches and LoRA state whatever
 * fields they hang from.  The small host arrays of pointers are released through the list below. */
/* hip_fused_step.c, when it is part of the link: the fused trainer that serves this context goes first */
__attribute__((weak)) void hip_fused_step_release(cuda_train_context_t* ctx);

void cuda_train_free(cuda_train_context_t* ctx) {
    if (!ctx) return;
    if (hip_fused_step_release) hip_fused_step_release(ctx);
    hc_state_t* st = state_of(ctx);
    if (st) {
        seraph_hip_stream_sync(st->stream);
        while (st->live) {
            live_buf_t* n = st->live;
            st->live = n->next;
            if (n->buf->data) seraph_hip_free(n->buf->data);
            free(n->buf);
            free(n);
        }
        if (st->ws) seraph_hip_free(st->ws);
        seraph_hip_stream_destroy(st->stream);
    }
    cuda_buffer_t*** arrays[] = {
        &ctx->fwd_cache_x_norm_attn, &ctx->fwd_cache_x_norm_ffn, &ctx->fwd_cache_attn_out, &ctx->fwd_cache_ffn_gate_out,
        &ctx->fwd_cache_ffn_up_out, &ctx->fwd_cache_ffn_hidden, &ctx->fwd_cache_layer_input, &ctx->fwd_cache_post_attn_in,
        &ctx->fwd_cache_silu_out, &ctx->fwd_cache_q, &ctx->fwd_cache_k, &ctx->fwd_cache_v, &ctx->fwd_cache_attn_lse,
        &ctx->gpu_w_q, &ctx->gpu_g_q, &ctx->gpu_m_q, &ctx->gpu_v_q, &ctx->gpu_w_k, &ctx->gpu_g_k, &ctx->gpu_m_k, &ctx->gpu_v_k,
        &ctx->gpu_w_v, &ctx->gpu_g_v, &ctx->gpu_m_v, &ctx->gpu_v_v, &ctx->gpu_w_o, &ctx->gpu_g_o, &ctx->gpu_m_o, &ctx->gpu_v_o,
        &ctx->gpu_w_gate, &ctx->gpu_g_gate, &ctx->gpu_m_gate, &ctx->gpu_v_gate, &ctx->gpu_w_up, &ctx->gpu_g_up, &ctx->gpu_m_up, &ctx->gpu_v_up,
        &ctx->gpu_w_down, &ctx->gpu_g_down, &ctx->gpu_m_down, &ctx->gpu_v_down, &ctx->gpu_w_in_norm, &ctx->gpu_g_in_norm,
        &ctx->gpu_m_in_norm, &ctx->gpu_v_in_norm, &ctx->gpu_w_post_norm, &ctx->gpu_g_post_norm, &ctx->gpu_m_post_norm, &ctx->gpu_v_post_norm};
    for (size_t i = 0; i < sizeof(arrays) / sizeof(arrays[0]); i++) { free(*arrays[i]); *arrays[i] = NULL; }
    if (ctx->lora_gpu) {
        cuda_lora_gpu_state_t* lg = (cuda_lora_gpu_state_t*)ctx->lora_gpu;
        for (int k = 0; k < 7; k++) {
            cuda_lora_gpu_adapter_t* a = lora_kinds(lg, k);
            free(a->A); free(a->B); free(a->gA); free(a->gB); free(a->mA); free(a->vA); free(a->mB); free(a->vB);
        }
        free(lg);
    }
    free(st);
    free(ctx);
}
