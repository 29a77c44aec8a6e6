/*
 * hip_backend.c - runtime, buffers, forward ops and the optimizer op of the backend API
 * (the counterpart of Seraph's src/vulkan_backend.c), over the MI355X kernel library.
 * Plain C, no HIP headers: everything device-side goes through include/seraph_hip.h.
 *
 * One in-order HIP stream replaces the command buffer: ops are enqueued as they are
 * called, vulkan_cmd_end_submit waits for the stream, and transfers from or to host
 * memory wait for the work queued before them - which is the ordering the reference
 * gets from its barrier after every recorded op (src/vulkan_backend_backward.c:124-142).
 */
#include <math.h>
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include "hip_backend_internal.h"

/* ------------------------------------------------------------------ helpers */
void hip_backend_report(vulkan_context_t* ctx, const char* op, int rc) {
    hip_state_t* st = hip_state(ctx);
    if (st) st->errors++;
    fprintf(stderr, "ERROR: %s failed (%d): %s\n", op, rc, seraph_hip_last_error());
}

int hip_backend_error_count(vulkan_context_t* ctx) {
    hip_state_t* st = hip_state(ctx);
    return st ? st->errors : -1;
}

int hip_backend_fits(vulkan_context_t* ctx, const char* op, int pairs, ...) {
    va_list ap;
    va_start(ap, pairs);
    int ok = 1;
    for (int i = 0; i < pairs; i++) {
        const vulkan_buffer_t* buf = va_arg(ap, const vulkan_buffer_t*);
        const size_t n = va_arg(ap, size_t);
        if (!buf || n <= buf->size / 4) continue;              /* NULL: an optional operand the op goes without */
        if (ok) {
            hip_state_t* st = hip_state(ctx);
            if (st && st->errors++ < 20)
                fprintf(stderr, "ERROR: %s refused: operand %d has %zu bytes, the shape needs %zu\n", op, i, buf->size, n * 4);
        }
        ok = 0;
    }
    va_end(ap);
    return ok;
}

void* hip_backend_scratch(vulkan_context_t* ctx, size_t bytes) {
    hip_state_t* st = hip_state(ctx);
    if (!st) return NULL;
    if (bytes <= st->ws_bytes && st->ws) return st->ws;
    /* queued kernels may still read the old block */
    if (seraph_hip_stream_sync(st->stream) != SERAPH_OK) return NULL;
    seraph_hip_free(st->ws);
    st->ws = NULL;
    st->ws_bytes = 0;
    size_t want = bytes + bytes / 4 + (1u << 20);
    void* p = NULL;
    if (seraph_hip_malloc(&p, want) != SERAPH_OK) {
        hip_backend_report(ctx, "scratch allocation", SERAPH_ERR_HIP);
        return NULL;
    }
    st->ws = p;
    st->ws_bytes = want;
    return p;
}

/* ------------------------------------------------------------------ profiler
 * hipEvent pairs per op, named as the reference names its ops; vulkan_profiler_end_step prints the
 * reference's report (src/vulkan_backend.c:105-207). */
void hip_prof_begin(vulkan_context_t* ctx, const char* name) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !ctx->profiling || st->prof_count >= HIP_PROF_MAX_OPS) return;
    if (!st->prof_ops) st->prof_ops = (hip_prof_op_t*)calloc(HIP_PROF_MAX_OPS, sizeof(hip_prof_op_t));
    if (!st->prof_ops) return;
    hip_prof_op_t* op = &st->prof_ops[st->prof_count];
    if (st->prof_count >= st->prof_events_made) {
        if (seraph_hip_event_create(&op->ev_start) != SERAPH_OK || seraph_hip_event_create(&op->ev_stop) != SERAPH_OK) return;
        st->prof_events_made = st->prof_count + 1;
    }
    strncpy(op->name, name, sizeof(op->name) - 1);
    op->name[sizeof(op->name) - 1] = '\0';
    seraph_hip_event_record(op->ev_start, st->stream);
}

void hip_prof_end(vulkan_context_t* ctx) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !ctx->profiling || !st->prof_ops || st->prof_count >= st->prof_events_made) return;
    seraph_hip_event_record(st->prof_ops[st->prof_count].ev_stop, st->stream);
    st->prof_count++;
    ctx->prof_num_ops = st->prof_count;
}

void vulkan_profiler_enable(vulkan_context_t* ctx) { if (ctx) ctx->profiling = 1; }
void vulkan_profiler_disable(vulkan_context_t* ctx) { if (ctx) ctx->profiling = 0; }
void vulkan_profiler_set_log(vulkan_context_t* ctx, void* file_ptr) { if (ctx) ctx->prof_log = file_ptr; }

void vulkan_profiler_begin_step(vulkan_context_t* ctx) {
    hip_state_t* st = hip_state(ctx);
    if (!st) return;
    st->prof_count = 0;
    ctx->prof_num_ops = 0;
}

/* Both to stdout and to the log file, as the reference's PROF_LOG (src/vulkan_backend.c:25-28). */
static void prof_log(vulkan_context_t* ctx, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vprintf(fmt, ap);
    va_end(ap);
    if (ctx->prof_log) {
        va_start(ap, fmt);
        vfprintf((FILE*)ctx->prof_log, fmt, ap);
        va_end(ap);
        fflush((FILE*)ctx->prof_log);
    }
}

/* The report of src/vulkan_backend.c:105-207: header, nine categories found by substrings of the op names, one line
 * per op.  The Grid / Block column stays empty (as it does in the reference for an op that records no launch shape):
 * the kernel library chooses its launches itself and an op may be several of them. */
void vulkan_profiler_end_step(vulkan_context_t* ctx, int step, int seq_len, float loss) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !ctx->profiling || !st->prof_ops || st->prof_count == 0) return;
    const int nops = st->prof_count;
    seraph_hip_stream_sync(st->stream);
    float* ms_of = (float*)calloc((size_t)nops, sizeof(float));
    if (!ms_of) return;
    double total_ms = 0;
    double cat_matmul = 0, cat_attn = 0, cat_attn_bwd = 0, cat_rmsnorm = 0, cat_rmsnorm_bwd = 0;
    double cat_cross_entropy = 0, cat_adamw = 0, cat_copy = 0, cat_other = 0;
    for (int i = 0; i < nops; i++) {
        float ms = 0.f;
        seraph_hip_event_elapsed_ms(st->prof_ops[i].ev_start, st->prof_ops[i].ev_stop, &ms);
        ms_of[i] = ms;
        total_ms += ms;
        const char* n = st->prof_ops[i].name;
        if (strstr(n, "matmul"))           cat_matmul += ms;
        else if (strstr(n, "attn_bwd"))    cat_attn_bwd += ms;
        else if (strstr(n, "attn"))        cat_attn += ms;
        else if (strstr(n, "rmsnorm_bwd")) cat_rmsnorm_bwd += ms;
        else if (strstr(n, "rmsnorm"))     cat_rmsnorm += ms;
        else if (strstr(n, "cross_ent"))   cat_cross_entropy += ms;
        else if (strstr(n, "adamw"))       cat_adamw += ms;
        else if (strstr(n, "copy") || strstr(n, "fill") || strstr(n, "barrier")) cat_copy += ms;
        else                               cat_other += ms;
    }
    if (total_ms <= 0) total_ms = 1e-6;

    prof_log(ctx, "\n");
    prof_log(ctx, "  ══════════════════════════════════════════════════════════════════\n");
    prof_log(ctx, "  SERAPH VULKAN STEP PROFILER (step %d, seq=%d, loss=%.4f)\n", step, seq_len, loss);
    prof_log(ctx, "  %d operations, %.2f ms total\n", nops, total_ms);
    prof_log(ctx, "  ══════════════════════════════════════════════════════════════════\n");
    prof_log(ctx, "\n  ── CATEGORY BREAKDOWN ──\n\n");
    prof_log(ctx, "  %-24s %10s  %6s  %s\n", "Category", "Time (ms)", "%", "Bar");
    prof_log(ctx, "  %-24s %10s  %6s  %s\n", "------------------------", "----------", "------",
             "----------------------------------------");
    const struct { const char* name; double ms; } cats[] = {
        {"matmul (all)", cat_matmul}, {"attention fwd", cat_attn}, {"attention bwd", cat_attn_bwd},
        {"rmsnorm fwd", cat_rmsnorm}, {"rmsnorm bwd", cat_rmsnorm_bwd}, {"cross_entropy", cat_cross_entropy},
        {"adamw", cat_adamw}, {"copy/fill", cat_copy}, {"other", cat_other},
    };
    for (size_t i = 0; i < sizeof(cats) / sizeof(cats[0]); i++) {
        const double pct = 100.0 * cats[i].ms / total_ms;
        int bar_len = (int)(pct * 0.4);
        if (bar_len > 40) bar_len = 40;
        char bar[41];
        memset(bar, '#', (size_t)bar_len);
        bar[bar_len] = '\0';
        prof_log(ctx, "  %-24s %10.3f  %5.1f%%  %s\n", cats[i].name, cats[i].ms, pct, bar);
    }
    prof_log(ctx, "\n  ── PER-OPERATION DETAIL ──\n\n");
    prof_log(ctx, "  %4s  %-60s %10s  %5s  %s\n", "#", "Operation", "Time (ms)", "%", "Grid / Block");
    prof_log(ctx, "  %4s  %-60s %10s  %5s  %s\n", "----", "------------------------------------------------------------",
             "----------", "-----", "------------------");
    for (int i = 0; i < nops; i++) {
        const double pct = 100.0 * ms_of[i] / total_ms;
        const char* marker = (pct > 5.0) ? " <<<" : (pct > 1.0) ? " <<" : "";
        prof_log(ctx, "  %4d  %-60s %10.3f  %4.1f%%  %-20s%s\n", i, st->prof_ops[i].name, ms_of[i], pct, "", marker);
    }
    prof_log(ctx, "\n");
    fflush(stdout);
    free(ms_of);
}

/* ------------------------------------------------------------------ init / free */
vulkan_context_t* vulkan_init_ex(int pool_size_hint, int device_index) {
    (void)pool_size_hint;
    if (seraph_hip_init(device_index) != SERAPH_OK) {
        fprintf(stderr, "ERROR: HIP backend init failed: %s\n", seraph_hip_last_error());
        return NULL;
    }
    vulkan_context_t* ctx = (vulkan_context_t*)calloc(1, sizeof(vulkan_context_t));
    hip_state_t* st = (hip_state_t*)calloc(1, sizeof(hip_state_t));
    if (!ctx || !st) { free(ctx); free(st); return NULL; }
    if (seraph_hip_stream_create(&st->stream) != SERAPH_OK) {
        fprintf(stderr, "ERROR: HIP stream creation failed: %s\n", seraph_hip_last_error());
        free(ctx); free(st);
        return NULL;
    }
    seraph_device_info_t info;
    if (seraph_hip_device_info(&info) == SERAPH_OK) {
        snprintf(ctx->gpu_name, sizeof(ctx->gpu_name), "%.180s (%.60s)", info.name, info.arch);
        ctx->vram_bytes = info.hbm_bytes;
        ctx->max_compute_units = info.compute_units;
        ctx->subgroup_size = ctx->min_subgroup_size = ctx->max_subgroup_size = info.wavefront_size;
        ctx->max_shared_memory = info.lds_bytes_per_block;
    }
    ctx->device_type = 2;                         /* discrete */
    ctx->vendor_id = 0x1002;
    ctx->max_workgroup_invocations = 1024;
    ctx->max_workgroup_size[0] = 1024; ctx->max_workgroup_size[1] = 1024; ctx->max_workgroup_size[2] = 1024;
    ctx->max_workgroup_count[0] = 0x7fffffffu; ctx->max_workgroup_count[1] = 65535; ctx->max_workgroup_count[2] = 65535;
    ctx->max_storage_buffer_range = 0xffffffffu;
    ctx->has_shader_atomic_float = 1;
    ctx->wg_size_1d = 256;                        /* vulkan_reduce_sum's caller assumes 512 inputs per output */
    ctx->wg_size_attn = 64;
    ctx->wg_size_matmul = 128; ctx->matmul_reg = 32; ctx->matmul_bk = 32;
    ctx->device = st;
    ctx->queue = st->stream;
    ctx->initialized = 1;
    return ctx;
}

vulkan_context_t* vulkan_init(int pool_size_hint) { return vulkan_init_ex(pool_size_hint, -1); }

void vulkan_free(vulkan_context_t* ctx) {
    if (!ctx) return;
    hip_state_t* st = hip_state(ctx);
    if (st) {
        seraph_hip_stream_sync(st->stream);
        seraph_hip_free(st->ws);
        if (st->prof_ops) {
            for (int i = 0; i < st->prof_events_made; i++) {
                seraph_hip_event_destroy(st->prof_ops[i].ev_start);
                seraph_hip_event_destroy(st->prof_ops[i].ev_stop);
            }
            free(st->prof_ops);
        }
        seraph_hip_stream_destroy(st->stream);
        free(st);
    }
    /* Buffers parked in the context's slot table belong to the caller (train.c frees them). */
    free(ctx);
}

int vulkan_cmd_begin(vulkan_context_t* ctx) {
    hip_state_t* st = hip_state(ctx);
    if (!st || st->recording) return 0;
    st->recording = 1;
    return 1;
}

int vulkan_cmd_end_submit(vulkan_context_t* ctx) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !st->recording) return 0;
    st->recording = 0;
    int rc = seraph_hip_stream_sync(st->stream);
    if (rc != SERAPH_OK) { hip_backend_report(ctx, "vulkan_cmd_end_submit", rc); return 0; }
    return 1;
}

/* ------------------------------------------------------------------ buffers */
vulkan_buffer_t* vulkan_buffer_create(vulkan_context_t* ctx, size_t size) {
    if (!hip_state(ctx)) return NULL;
    vulkan_buffer_t* buf = (vulkan_buffer_t*)calloc(1, sizeof(vulkan_buffer_t));
    if (!buf) return NULL;
    if (seraph_hip_malloc(&buf->buffer, size) != SERAPH_OK) {
        hip_backend_report(ctx, "vulkan_buffer_create", SERAPH_ERR_HIP);
        free(buf);
        return NULL;
    }
    buf->memory = buf->buffer;
    buf->size = size;
    buf->mapped = NULL;
    return buf;
}

void vulkan_buffer_free(vulkan_context_t* ctx, vulkan_buffer_t* buf) {
    hip_state_t* st = hip_state(ctx);
    if (!buf) return;
    if (st) seraph_hip_stream_sync(st->stream);           /* queued ops may still use it */
    seraph_hip_free(buf->buffer);
    free(buf);
}

void vulkan_buffer_upload_bytes(vulkan_context_t* ctx, vulkan_buffer_t* buf, const void* data, size_t bytes) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !buf || !data) return;
    if (bytes > buf->size) bytes = buf->size;
    int rc = seraph_hip_h2d(DPTR(buf), data, bytes, st->stream);
    if (rc != SERAPH_OK) hip_backend_report(ctx, "vulkan_buffer_upload", rc);
}

void vulkan_buffer_upload(vulkan_context_t* ctx, vulkan_buffer_t* buf, const float* data, size_t count) {
    vulkan_buffer_upload_bytes(ctx, buf, data, count * sizeof(float));
}

void vulkan_buffer_upload_u32(vulkan_context_t* ctx, vulkan_buffer_t* buf, const uint32_t* data, size_t count) {
    vulkan_buffer_upload_bytes(ctx, buf, data, count * sizeof(uint32_t));
}

void vulkan_buffer_download_bytes(vulkan_context_t* ctx, vulkan_buffer_t* buf, void* data, size_t bytes) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !buf || !data) return;
    if (bytes > buf->size) bytes = buf->size;
    int rc = seraph_hip_d2h(data, DPTR(buf), bytes, st->stream);
    if (rc != SERAPH_OK) hip_backend_report(ctx, "vulkan_buffer_download", rc);
}

void vulkan_buffer_download(vulkan_context_t* ctx, vulkan_buffer_t* buf, float* data, size_t count) {
    vulkan_buffer_download_bytes(ctx, buf, data, count * sizeof(float));
}

void vulkan_fill_buffer_range(vulkan_context_t* ctx, vulkan_buffer_t* buf, size_t offset_bytes, uint32_t value, size_t bytes) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !buf || bytes == 0) return;
    if (offset_bytes >= buf->size) return;
    if (bytes > buf->size - offset_bytes) bytes = buf->size - offset_bytes;
    offset_bytes &= ~(size_t)3;                           /* as src/vulkan_backend.c:1216-1223 */
    bytes &= ~(size_t)3;
    if (bytes == 0) return;
    HIP_OP(ctx, "fill_buffer", seraph_fill_u32((char*)DPTR(buf) + offset_bytes, value, bytes / 4, st->stream));
}

void vulkan_fill_buffer(vulkan_context_t* ctx, vulkan_buffer_t* buf, uint32_t value, size_t bytes) {
    vulkan_fill_buffer_range(ctx, buf, 0, value, bytes);
}

void vulkan_copy_buffer(vulkan_context_t* ctx, vulkan_buffer_t* src, vulkan_buffer_t* dst, size_t bytes) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !src || !dst || bytes == 0) return;
    if (bytes > src->size) bytes = src->size;
    if (bytes > dst->size) bytes = dst->size;
    HIP_OP(ctx, "copy_buffer", seraph_hip_d2d(DPTR(dst), DPTR(src), bytes, st->stream));
}

void vulkan_copy_buffer_cache(vulkan_context_t* ctx, vulkan_buffer_t* src, vulkan_buffer_t* dst, size_t bytes) {
    vulkan_copy_buffer(ctx, src, dst, bytes);             /* the stream already orders it */
}

void vulkan_barrier_transfer_to_compute(vulkan_context_t* ctx) { (void)ctx; }

void vulkan_nan_check(vulkan_context_t* ctx, vulkan_buffer_t* input, size_t count_floats, vulkan_buffer_t* flags_u32, uint32_t flag_index) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !flags_u32 || count_floats == 0) return;
    if ((size_t)(flag_index + 1) * 4 > flags_u32->size) return;
    if (!hip_backend_fits(ctx, "nan_check", 1, FIT(input, count_floats))) return;
    HIP_OP(ctx, "nan_check", seraph_nan_check(FPTR(input), count_floats, UPTR(flags_u32), flag_index, st->stream));
}

/* ------------------------------------------------------------------ forward ops */
/* A small output with a long K (narrow weight gradients, rank-sized LoRA products) is computed in runs of K
 * through the context's scratch; every other shape is the plain product. */
static void backend_gemm(vulkan_context_t* ctx, hip_state_t* st, const char* what, const float* A, const float* B, float* C,
                         int M, int N, int K, int tA, int tB, int accumulate) {
    const size_t need = seraph_gemm_scaled_ws_bytes(M, N, K, tA, tB);
    void* ws = need ? hip_backend_scratch(ctx, need) : NULL;
    HIP_OPF(ctx, seraph_gemm_scaled(A, B, C, M, N, K, tA, tB, accumulate, 1.0f, ws, ws ? need : 0, st->stream),
            "%s [%dx%d K=%d]", what, M, N, K);                        /* src/vulkan_backend.c:1674, :1848 */
}

void hip_matmul_scaled(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C,
                       int M, int N, int K, int transpose_A, int transpose_B, int accumulate, float alpha) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !B || !C || M < 0 || N < 0 || K < 0) return;
    if (!hip_backend_fits(ctx, "matmul_scaled", 3, FIT(A, (size_t)M * K), FIT(B, (size_t)K * N), FIT(C, (size_t)M * N))) return;
    const size_t need = seraph_gemm_scaled_ws_bytes(M, N, K, transpose_A, transpose_B);
    void* ws = need ? hip_backend_scratch(ctx, need) : NULL;
    HIP_OPF(ctx, seraph_gemm_scaled(FPTR(A), FPTR(B), FPTR(C), M, N, K, transpose_A, transpose_B, accumulate, alpha,
                                    ws, ws ? need : 0, st->stream), "matmul_scaled [%dx%d K=%d]", M, N, K);
}

void vulkan_matmul(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C, int M, int N, int K) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !B || !C || M < 0 || N < 0 || K < 0) return;
    if (!hip_backend_fits(ctx, "matmul", 3, FIT(A, (size_t)M * K), FIT(B, (size_t)K * N), FIT(C, (size_t)M * N))) return;
    backend_gemm(ctx, st, "matmul", FPTR(A), FPTR(B), FPTR(C), M, N, K, 0, 0, 0);
}

void vulkan_matmul_transpose(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C,
                             int M, int N, int K, int transpose_A, int transpose_B, int accumulate) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !B || !C || M < 0 || N < 0 || K < 0) return;
    if (!hip_backend_fits(ctx, "matmul_t", 3, FIT(A, (size_t)M * K), FIT(B, (size_t)K * N), FIT(C, (size_t)M * N))) return;
    backend_gemm(ctx, st, "matmul_t", FPTR(A), FPTR(B), FPTR(C), M, N, K, transpose_A, transpose_B, accumulate);
}

void vulkan_add(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !B || !C || !hip_backend_fits(ctx, "add", 3, FIT(A, count), FIT(B, count), FIT(C, count))) return;
    HIP_OP(ctx, "add", seraph_add(FPTR(A), FPTR(B), FPTR(C), count, st->stream));
}

void vulkan_mul(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !B || !C || !hip_backend_fits(ctx, "mul", 3, FIT(A, count), FIT(B, count), FIT(C, count))) return;
    HIP_OP(ctx, "mul", seraph_mul(FPTR(A), FPTR(B), FPTR(C), count, st->stream));
}

void vulkan_scale(vulkan_context_t* ctx, vulkan_buffer_t* A, size_t count, float alpha) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !hip_backend_fits(ctx, "scale", 1, FIT(A, count))) return;
    HIP_OP(ctx, "scale", seraph_scale(FPTR(A), count, alpha, st->stream));
}

void vulkan_silu(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* output, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !output || !hip_backend_fits(ctx, "silu", 2, FIT(input, count), FIT(output, count))) return;
    HIP_OP(ctx, "silu", seraph_silu(FPTR(input), FPTR(output), count, st->stream));
}

void hip_swiglu(vulkan_context_t* ctx, vulkan_buffer_t* gate, vulkan_buffer_t* up, vulkan_buffer_t* out, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !gate || !up || !out || !hip_backend_fits(ctx, "silu_mul", 3, FIT(gate, count), FIT(up, count), FIT(out, count))) return;
    HIP_OP(ctx, "silu_mul", seraph_swiglu(FPTR(gate), FPTR(up), FPTR(out), count, st->stream));
}

void vulkan_rmsnorm(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale, vulkan_buffer_t* output,
                    int rows, int cols, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !scale || !output || rows < 0 || cols < 0) return;
    if (!hip_backend_fits(ctx, "rmsnorm", 3, FIT(input, (size_t)rows * cols), FIT(scale, cols), FIT(output, (size_t)rows * cols))) return;
    HIP_OPF(ctx, seraph_rmsnorm(FPTR(input), FPTR(scale), FPTR(output), rows, cols, eps, st->stream), "rmsnorm [%dx%d] %u-thr", rows, cols, ctx->wg_size_1d);
}

/* vulkan_add of a residual branch and the vulkan_rmsnorm that reads the sum (src/train.c:4705-4711): sum = input + addend,
 * output = rmsnorm(sum); sum is a buffer of its own. */
void hip_add_rmsnorm(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* addend, vulkan_buffer_t* sum,
                     vulkan_buffer_t* scale, vulkan_buffer_t* output, int rows, int cols, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !addend || !sum || !scale || !output || rows < 0 || cols < 0) return;
    const size_t rc = (size_t)rows * cols;
    if (!hip_backend_fits(ctx, "add+rmsnorm", 5, FIT(input, rc), FIT(addend, rc), FIT(sum, rc), FIT(scale, cols), FIT(output, rc))) return;
    HIP_OPF(ctx, seraph_add_rmsnorm(FPTR(input), FPTR(addend), FPTR(sum), FPTR(scale), FPTR(output), rows, cols, eps, st->stream), "add+rmsnorm [%dx%d] %u-thr", rows, cols, ctx->wg_size_1d);
}

void vulkan_rope(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out,
                 int seq_len, int num_heads, int head_dim, float rope_theta) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !x_in || !x_out || seq_len < 0 || num_heads < 0 || head_dim < 0) return;
    const size_t n = (size_t)seq_len * num_heads * head_dim;
    if (!hip_backend_fits(ctx, "rope_fwd", 2, FIT(x_in, n), FIT(x_out, n))) return;
    HIP_OP(ctx, "rope_fwd", seraph_rope(FPTR(x_in), FPTR(x_out), NULL, 1, seq_len, num_heads, head_dim, rope_theta, 0, st->stream));
}

void hip_rope_packed(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out, vulkan_buffer_t* seq_starts,
                     int total_tokens, int batch_size, int num_heads, int head_dim, float rope_theta) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !x_in || !x_out || !seq_starts || total_tokens < 0 || batch_size < 0 || num_heads < 0 || head_dim < 0) return;
    const size_t n = (size_t)total_tokens * num_heads * head_dim;
    if (!hip_backend_fits(ctx, "rope_fwd_packed", 3, FIT(x_in, n), FIT(x_out, n), FIT(seq_starts, (size_t)batch_size + 1))) return;
    HIP_OP(ctx, "rope_fwd_packed", seraph_rope(FPTR(x_in), FPTR(x_out), UPTR(seq_starts), batch_size, total_tokens, num_heads, head_dim, rope_theta, 0, st->stream));
}

void vulkan_batch_attention(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                            vulkan_buffer_t* out, int seq_len, int num_heads, int kv_heads, int head_dim) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !Q || !K || !V || !out || seq_len < 0 || num_heads < 0 || kv_heads < 0 || head_dim < 0) return;
    const size_t nq = (size_t)seq_len * num_heads * head_dim, nkv = (size_t)seq_len * kv_heads * head_dim;
    if (!hip_backend_fits(ctx, "attn_fwd", 4, FIT(Q, nq), FIT(K, nkv), FIT(V, nkv), FIT(out, nq))) return;
    float scale = 1.0f / sqrtf((float)head_dim);          /* src/vulkan_backend.c:2980-2984 */
    HIP_OPF(ctx, seraph_attention_forward(FPTR(Q), FPTR(K), FPTR(V), FPTR(out), NULL, NULL, 1, seq_len,
                                                            num_heads, kv_heads, head_dim, scale, st->stream), "attn_fwd [seq=%d h=%d hd=%d]", seq_len, num_heads, head_dim);
}

void hip_batch_attention_packed(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                                vulkan_buffer_t* out, vulkan_buffer_t* lse_out, vulkan_buffer_t* seq_starts,
                                int total_tokens, int batch_size, int num_heads, int kv_heads, int head_dim) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !Q || !K || !V || !out || !seq_starts || total_tokens < 0 || batch_size < 0 || num_heads < 0 || kv_heads < 0 || head_dim < 0) return;
    const size_t nq = (size_t)total_tokens * num_heads * head_dim, nkv = (size_t)total_tokens * kv_heads * head_dim;
    if (!hip_backend_fits(ctx, "attn_fwd_packed", 6, FIT(Q, nq), FIT(K, nkv), FIT(V, nkv), FIT(out, nq),
                          FIT(lse_out, (size_t)total_tokens * num_heads), FIT(seq_starts, (size_t)batch_size + 1))) return;
    float scale = 1.0f / sqrtf((float)head_dim);
    HIP_OPF(ctx, seraph_attention_forward(FPTR(Q), FPTR(K), FPTR(V), FPTR(out), lse_out ? FPTR(lse_out) : NULL,
                                                                   UPTR(seq_starts), batch_size, total_tokens,
                                                                   num_heads, kv_heads, head_dim, scale, st->stream), "attn_fwd_packed [tok=%d seqs=%d h=%d hd=%d]", total_tokens, batch_size, num_heads, head_dim);
}

void vulkan_embed_lookup(vulkan_context_t* ctx, vulkan_buffer_t* tokens_u32, vulkan_buffer_t* embed_weight,
                         vulkan_buffer_t* out_hidden, int seq_len, int hidden_size, int vocab_size) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !tokens_u32 || !embed_weight || !out_hidden || seq_len < 0 || hidden_size < 0 || vocab_size < 0) return;
    if (!hip_backend_fits(ctx, "embed_lookup", 3, FIT(tokens_u32, seq_len), FIT(embed_weight, (size_t)vocab_size * hidden_size),
                          FIT(out_hidden, (size_t)seq_len * hidden_size))) return;
    HIP_OP(ctx, "embed_lookup", seraph_embed_lookup(UPTR(tokens_u32), FPTR(embed_weight), FPTR(out_hidden), seq_len, hidden_size, vocab_size, st->stream));
}

void vulkan_qk_norm(vulkan_context_t* ctx, vulkan_buffer_t* qk, int seq_len, int num_heads, int head_dim, int use_qk_norm, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !qk || !use_qk_norm) return;               /* src/vulkan_backend.c:3481 */
    if (seq_len < 0 || num_heads < 0 || head_dim < 0 || !hip_backend_fits(ctx, "qk_norm", 1, FIT(qk, (size_t)seq_len * num_heads * head_dim))) return;
    HIP_OP(ctx, "qk_norm", seraph_qk_norm(FPTR(qk), seq_len, num_heads, head_dim, use_qk_norm, eps, st->stream));
}

/* ------------------------------------------------------------------ optimizer */
void hip_adamw_update_clipped(vulkan_context_t* ctx, vulkan_buffer_t* weight, vulkan_buffer_t* grad, vulkan_buffer_t* m,
                              vulkan_buffer_t* v, float lr, float beta1, float beta2, float weight_decay, float eps,
                              int step, size_t size, float clip) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !weight || !grad || !m || !v || size == 0) return;
    if (!hip_backend_fits(ctx, "adamw", 4, FIT(weight, size), FIT(grad, size), FIT(m, size), FIT(v, size))) return;
    HIP_OPF(ctx, seraph_adamw(FPTR(weight), FPTR(grad), FPTR(m), FPTR(v), size, lr, beta1, beta2, weight_decay, eps, step, clip, st->stream), "adamw [%zu] %u-thr", (size_t)size, ctx->wg_size_1d);
}

void hip_adamw_update_multi(vulkan_context_t* ctx, int count, vulkan_buffer_t* const* weights, vulkan_buffer_t* const* grads,
                            vulkan_buffer_t* const* m, vulkan_buffer_t* const* v, const size_t* sizes,
                            float lr, float beta1, float beta2, float weight_decay, float eps, int step, float clip) {
    hip_state_t* st = hip_state(ctx);
    if (!st || count <= 0 || !weights || !grads || !m || !v || !sizes) return;
    seraph_adamw_tensor_t* list = (seraph_adamw_tensor_t*)malloc((size_t)count * sizeof(*list));
    if (!list) { hip_backend_report(ctx, "adamw", SERAPH_ERR_INVALID); return; }
    int k = 0;
    for (int i = 0; i < count; i++) {
        if (!weights[i] || !grads[i] || !m[i] || !v[i] || sizes[i] == 0) continue;      /* as vulkan_adamw_update: silently */
        if (!hip_backend_fits(ctx, "adamw", 4, FIT(weights[i], sizes[i]), FIT(grads[i], sizes[i]), FIT(m[i], sizes[i]), FIT(v[i], sizes[i]))) continue;
        list[k].w = FPTR(weights[i]); list[k].g = FPTR(grads[i]); list[k].m = FPTR(m[i]); list[k].v = FPTR(v[i]);
        list[k].n = sizes[i];
        k++;
    }
    HIP_OPF(ctx, seraph_adamw_multi(list, k, lr, beta1, beta2, weight_decay, eps, step, clip, st->stream), "adamw [%d tensors] %u-thr", k, ctx->wg_size_1d);
    free(list);
}

void vulkan_adamw_update(vulkan_context_t* ctx, vulkan_buffer_t* weight, vulkan_buffer_t* grad, vulkan_buffer_t* m,
                         vulkan_buffer_t* v, float lr, float beta1, float beta2, float weight_decay, float eps,
                         int step, size_t size) {
    hip_adamw_update_clipped(ctx, weight, grad, m, v, lr, beta1, beta2, weight_decay, eps, step, size, 0.0f);
}

/* ------------------------------------------------------------------ video-mode ops
 * Not on the LLM training path (reached only when num_queries > 0). */
static void video_op_unsupported(vulkan_context_t* ctx, const char* name) {
    static int warned = 0;
    if (!warned) fprintf(stderr, "ERROR: %s: video-mode ops are not provided by the HIP backend\n", name);
    warned = 1;
    hip_state_t* st = hip_state(ctx);
    if (st) st->errors++;
}

void vulkan_patch_extract(vulkan_context_t* ctx, vulkan_buffer_t* frame, vulkan_buffer_t* patches,
                          int frame_h, int frame_w, int channels, int patch_t, int patch_h, int patch_w) {
    (void)frame; (void)patches; (void)frame_h; (void)frame_w; (void)channels; (void)patch_t; (void)patch_h; (void)patch_w;
    video_op_unsupported(ctx, "vulkan_patch_extract");
}
void vulkan_add_bias(vulkan_context_t* ctx, vulkan_buffer_t* data, vulkan_buffer_t* bias, int rows, int cols) {
    (void)data; (void)bias; (void)rows; (void)cols;
    video_op_unsupported(ctx, "vulkan_add_bias");
}
void vulkan_bce_loss_grad(vulkan_context_t* ctx, vulkan_buffer_t* logits, vulkan_buffer_t* targets,
                          vulkan_buffer_t* grad_logits, vulkan_buffer_t* loss_out, size_t count) {
    (void)logits; (void)targets; (void)grad_logits; (void)loss_out; (void)count;
    video_op_unsupported(ctx, "vulkan_bce_loss_grad");
}
void vulkan_sum_cols(vulkan_context_t* ctx, vulkan_buffer_t* data, vulkan_buffer_t* out, int rows, int cols) {
    (void)data; (void)out; (void)rows; (void)cols;
    video_op_unsupported(ctx, "vulkan_sum_cols");
}
