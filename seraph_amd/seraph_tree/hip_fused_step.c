/*
 * hip_fused_step.c - gives Seraph's batched front end (tools/seraph_train_cuda.c) the fused
 * MI355X training step behind the step functions it already calls.
 *
 * Compiled inside a Seraph tree next to hip_cuda_backend.c.  The tree's own src/train_cuda.c is
 * compiled unmodified, with its full-weight entry points renamed on the compiler's command line
 *     -Dcuda_train_step_gpu_full_batch=cuda_train_step_gpu_full_batch_opbyop   (and the five below)
 * so the op-by-op steps stay in the binary under the _opbyop names, and this file provides the names
 * that the front end and src/train.c call (include/train_cuda.h:22-66):
 *
 *   cuda_train_step_gpu_full_batch   src/train_cuda.c:1966-2326   -> hip_train_step_full_batch
 *   cuda_train_step_gpu_full         src/train_cuda.c:597-1242    -> the same with one sequence
 *   cuda_download_full_weights       src/train_cuda.c:1244-1315   -> weights and Adam moments out of the flat arenas
 *   cuda_download_gpu_gradients      src/train_cuda.c:1317-1380   -> gradients out of the flat arena
 *   cuda_eval_forward, cuda_evaluate src/train_cuda.c:2677-2847   -> hip_eval_forward_batch, hip_evaluate
 *
 * The weights of the trainer's train_state_t are mirrored into the flat parameter arena once, at the first
 * step (what ensure_cuda_gpu_weights does for the per-tensor buffers, src/train_cuda.c:395-470); the
 * state's bookkeeping - accumulation_counter, optimizer_step, the warm-up schedule of
 * src/train_cuda.c:2287-2303 - is handed to the fused step before every call and read back after it, so
 * checkpoints, logs and resume see the numbers the reference's step would have left.
 *
 * LoRA steps are not forwarded: the reference's CUDA LoRA step keeps running op by op over cuda_train_*.
 * Video models (num_queries > 0) and SERAPH_HIP_FUSED_STEP=0 in the environment take the op-by-op step too.
 * SERAPH_HIP_FUSED_TOKENS=n sets the room the fused trainer starts with (default: batch size x longest sequence of the
 * training configuration).
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "train_cuda.h"
#include "hip_train.h"

float cuda_train_step_gpu_full_batch_opbyop(train_state_t* state, int* tokens_packed, int total_tokens, int* seq_starts,
                                            int batch_size, cuda_train_context_t* ctx);
float cuda_train_step_gpu_full_opbyop(train_state_t* state, int* tokens, int num_tokens, cuda_train_context_t* ctx);
void cuda_download_full_weights_opbyop(cuda_train_context_t* ctx, train_state_t* state);
void cuda_download_gpu_gradients_opbyop(cuda_train_context_t* ctx, train_state_t* state);
float cuda_eval_forward_opbyop(train_state_t* state, int* tokens, int num_tokens, cuda_train_context_t* ctx);
float cuda_evaluate_opbyop(train_state_t* state, int* val_tokens, int num_val_tokens, int* offsets, int num_samples,
                           int max_seq_len, int max_eval_samples, cuda_train_context_t* ctx, float* out_perplexity);

/* hip_cuda_backend.c: the front end's profiler when it is attached and recording this step, and an entry with a known time */
cuda_profiler_t* hip_cuda_active_profiler(cuda_train_context_t* ctx);
void hip_cuda_profiler_add(cuda_profiler_t* p, const char* name, float elapsed_ms, size_t flops, size_t bytes);

/* one fused trainer per process: the front end drives one model */
static struct {
    cuda_train_context_t* ctx;
    train_state_t* state;
    hip_trainer_t* t;
    int max_tokens, max_batch;
    int opbyop;                     /* this state has taken an op-by-op step: its weights live in the per-tensor buffers */
    int nan_check;                  /* the trainer's NaN checks are on */
} g;

static double now_ms(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return 1e3 * (double)ts.tv_sec + 1e-6 * (double)ts.tv_nsec;
}

static int fused_wanted(const train_state_t* state) {
    const char* e = getenv("SERAPH_HIP_FUSED_STEP");
    if (e && e[0] == '0') return 0;
    if (!state || !state->config || !state->full_weights) return 0;
    if (state->config->num_queries > 0) return 0;                  /* video mode: ops this path does not have */
    return !g.opbyop;
}

/* The tensors of trainable_weights_t in the order of the flat arenas. */
typedef struct { weight_tensor_t* t; int64_t off; } slot_t;

static slot_t* arena_slots(const train_state_t* state, const hip_model_config_t* c, int* count) {
    hip_param_layout_t L;
    hip_param_layout(c, &L);
    trainable_weights_t* w = state->full_weights;
    const int n = 2 + 9 * c->layers;
    slot_t* s = (slot_t*)calloc((size_t)n, sizeof(slot_t));
    if (!s) return NULL;
    int k = 0;
    s[k].t = &w->embed_tokens; s[k++].off = L.embed;
    s[k].t = &w->final_norm;   s[k++].off = L.final_norm;
    for (int l = 0; l < c->layers; l++) {
        layer_weights_t* lw = &w->layers[l];
        const int64_t base = L.layer0 + (int64_t)l * L.layer_stride;
        weight_tensor_t* ts[9] = {&lw->input_norm, &lw->q_proj, &lw->k_proj, &lw->v_proj, &lw->o_proj, &lw->post_norm,
                                  &lw->gate_proj, &lw->up_proj, &lw->down_proj};
        const int64_t offs[9] = {L.in_norm, L.q, L.k, L.v, L.o, L.post_norm, L.gate, L.up, L.down};
        for (int i = 0; i < 9; i++) { s[k].t = ts[i]; s[k++].off = base + offs[i]; }
    }
    *count = n;
    return s;
}

static void model_config_of(const train_state_t* state, hip_model_config_t* c) {
    const model_config_t* m = state->config;
    memset(c, 0, sizeof(*c));
    c->hidden = m->hidden_size; c->layers = m->num_hidden_layers; c->heads = m->num_attention_heads;
    c->kv_heads = m->num_key_value_heads; c->head_dim = m->head_dim; c->ffn = m->intermediate_size; c->vocab = m->vocab_size;
    c->rms_eps = 1e-5f;                                             /* src/train_cuda.c:1984: the step's own constant */
    c->rope_theta = m->rope_theta > 0 ? m->rope_theta : 10000.0f;   /* :1985 */
}

/* The fused trainer for this state, with room for the batch; NULL when the op-by-op step has to run. */
static hip_trainer_t* fused_trainer(train_state_t* state, cuda_train_context_t* ctx, int total_tokens, int batch_size) {
    if (!fused_wanted(state)) return NULL;
    if (g.t && (g.state != state || g.ctx != ctx)) return NULL;    /* a second model in one process: not this path */
    if (g.t && total_tokens <= g.max_tokens && batch_size <= g.max_batch) return g.t;

    hip_model_config_t c;
    model_config_of(state, &c);
    hip_optim_config_t o = {state->learning_rate, 0.9f, 0.999f, 0.01f, 1e-8f, 0.0f, 100,
                            state->gradient_accumulation_steps < 1 ? 1 : state->gradient_accumulation_steps};
    int want_tokens = total_tokens, want_batch = batch_size;
    /* Room for the largest batch the training configuration allows, so that the trainer is created once.
     * SERAPH_HIP_FUSED_TOKENS=n in the environment starts with room for n tokens instead (activation memory for the
     * batches that actually arrive); a batch that does not fit makes a larger trainer and carries the arenas over. */
    const char* room = getenv("SERAPH_HIP_FUSED_TOKENS");
    if (room && atol(room) > 0 && atol(room) < (1L << 30)) {
        if (atol(room) > want_tokens) want_tokens = (int)atol(room);
    } else if (state->train_cfg && state->train_cfg->batch_size > 0 && state->train_cfg->max_seq_len > 0) {
        const long cap = (long)state->train_cfg->batch_size * (long)state->train_cfg->max_seq_len;
        if (cap > want_tokens && cap < (1L << 30)) want_tokens = (int)cap;
        if (state->train_cfg->batch_size > want_batch) want_batch = state->train_cfg->batch_size;
    }
    if (g.max_tokens > want_tokens) want_tokens = g.max_tokens;
    if (g.max_batch > want_batch) want_batch = g.max_batch;

    /* a trainer that has become too small: carry its arenas over through the host */
    const int64_t n = hip_param_count(&c);
    float* keep[4] = {NULL, NULL, NULL, NULL};
    if (g.t) {
        for (int a = 0; a < 4; a++) {
            keep[a] = (float*)malloc((size_t)n * sizeof(float));
            if (!keep[a] || hip_trainer_download(g.t, a, keep[a], n) != 0) {
                for (int b = 0; b <= a; b++) free(keep[b]);
                fprintf(stderr, "ERROR: fused step: could not carry the arenas over to a larger trainer\n");
                return NULL;
            }
        }
        hip_trainer_free(g.t);
        g.t = NULL;
    }
    hip_trainer_t* t = hip_trainer_create(&c, &o, want_tokens, want_batch, ctx->device_id, NULL, NULL, NULL, NULL);
    if (!t) {
        for (int a = 0; a < 4; a++) free(keep[a]);
        if (keep[0]) { fprintf(stderr, "ERROR: fused step: the larger trainer could not be created\n"); exit(1); }
        fprintf(stderr, "WARNING: fused step unavailable, running the op-by-op step\n");
        g.opbyop = 1;
        return NULL;
    }
    if (keep[0]) {
        for (int a = 0; a < 4; a++) { hip_trainer_upload(t, a, keep[a], n); free(keep[a]); }
        fprintf(stderr, "[HIP] fused training step: room grown to %d tokens in %d sequences\n", want_tokens, want_batch);
    } else {
        /* weights (and moments, zero in a fresh state) of every tensor into its place in the arenas */
        int ns = 0;
        slot_t* s = arena_slots(state, &c, &ns);
        if (!s) { hip_trainer_free(t); return NULL; }
        for (int i = 0; i < ns; i++) {
            hip_trainer_upload_at(t, 0, s[i].off, s[i].t->weight, (int64_t)s[i].t->size);
            if (s[i].t->m) hip_trainer_upload_at(t, 2, s[i].off, s[i].t->m, (int64_t)s[i].t->size);
            if (s[i].t->v) hip_trainer_upload_at(t, 3, s[i].off, s[i].t->v, (int64_t)s[i].t->size);
        }
        free(s);
        fprintf(stderr, "[HIP] fused training step: %lld parameters in flat arenas, room for %d tokens in %d sequences\n",
                (long long)n, want_tokens, want_batch);
    }
    g.t = t; g.ctx = ctx; g.state = state; g.max_tokens = want_tokens; g.max_batch = want_batch;
    g.nan_check = 0;                                                /* a new trainer starts without them */
    return t;
}

/* An op-by-op step updates the per-tensor buffers, so from then on the fused step's arenas would be stale - unless the
 * step belongs to another model than the one the fused trainer serves, whose arenas it does not touch. */
static void took_opbyop_step(const train_state_t* state) {
    if (!g.t || g.state == state) g.opbyop = 1;
}

/* hip_cuda_backend.c calls this from cuda_train_free when it is linked in */
void hip_fused_step_release(cuda_train_context_t* ctx) {
    if (g.t && g.ctx == ctx) { hip_trainer_free(g.t); memset(&g, 0, sizeof(g)); }
}

float cuda_train_step_gpu_full_batch(train_state_t* state, int* tokens_packed, int total_tokens, int* seq_starts, int batch_size,
                                     cuda_train_context_t* ctx) {
    if (!state || !state->full_weights || !state->config || !ctx) return -1.0f;      /* src/train_cuda.c:1970 */
    hip_trainer_t* t = fused_trainer(state, ctx, total_tokens, batch_size);
    if (!t) {
        took_opbyop_step(state);
        return cuda_train_step_gpu_full_batch_opbyop(state, tokens_packed, total_tokens, seq_starts, batch_size, ctx);
    }
    const double t0 = now_ms();
    if (total_tokens - batch_size <= 0) return 0.0f;                                 /* :1990-1991 */
    /* the state's counters and learning rate are the truth (a resume sets them): src/train_cuda.c:2287-2303 */
    hip_trainer_set_schedule(t, state->learning_rate, state->optimizer_step, state->accumulation_counter);
    /* --debug-nan-check: the flag lattice, the held-back optimizer and the dump files of the reference's single-sequence
     * step (src/train_cuda.c:633-661, :1080-1187), for packed batches as well (the reference's packed step has no checks) */
    const int want_nan = state->debug_nan_check ? 1 : 0;
    if (want_nan != g.nan_check && hip_trainer_enable_nan_check(t, want_nan) == 0) g.nan_check = want_nan;
    if (g.nan_check) hip_trainer_set_step_counter(t, state->current_step);
    /* --profile: the fused step has no per-call ops to bracket; its kernels are timed per class (event pairs around
     * every kernel-library call of this one step) and each class goes to the front end's profiler as one entry, named so
     * that the profiler's substring categories (src/cuda_profiler.cu:152-172) file it where the op-by-op step's ops go */
    cuda_profiler_t* prof = hip_cuda_active_profiler(ctx);
    if (prof) { hip_trainer_enable_op_timing(t, 1); hip_trainer_reset_op_stats(t); }
    const float loss = hip_train_step_full_batch(t, tokens_packed, total_tokens, seq_starts, batch_size, 1);
    if (prof) {
        static hip_op_stat_t stats[64];
        const int n = hip_trainer_op_stats(t, stats, 64);
        for (int i = 0; i < n; i++) {
            const char* nm = stats[i].name ? stats[i].name : "";
            const char* cat = strstr(nm, "gemm") ? "matmul " : !strcmp(nm, "attention_backward") ? "attn_bwd " :
                              !strcmp(nm, "attention_forward") ? "attn_fwd " : !strcmp(nm, "rmsnorm_backward") ? "rmsnorm_bwd " :
                              !strcmp(nm, "fill") ? "memset " : "";
            const char* shortn = strncmp(nm, "seraph::", 8) == 0 ? nm + 8 : nm;
            char label[80];
            snprintf(label, sizeof(label), "%s%.*s x%lld", cat, 58 - (int)strlen(cat), shortn, (long long)stats[i].launches);
            hip_cuda_profiler_add(prof, label, (float)stats[i].ms, (size_t)stats[i].flops, (size_t)stats[i].bytes);
        }
        hip_trainer_enable_op_timing(t, 0);
    }
    if (g.nan_check && hip_trainer_nan_detected(t)) {                                /* src/train_cuda.c:1097-1183 */
        fprintf(stderr, "[NAN] detected at step=%d seq=%d (optimizer skipped)\n", state->current_step + 1, total_tokens);
        fprintf(stderr, "  - lr(base)=%g opt_step=%d accum=%d/%d\n", (double)state->learning_rate, state->optimizer_step,
                state->accumulation_counter, state->gradient_accumulation_steps);
        hip_trainer_nan_report(t, stderr);
        fprintf(stderr, "[NAN-DUMP] wrote buffers with prefix /tmp/seraph_nan_step_%d_*\n", state->current_step + 1);
        state->nan_detected = 1;
        return NAN;
    }
    state->optimizer_step = hip_trainer_optimizer_step(t);
    state->accumulation_counter = hip_trainer_accumulation_counter(t);
    if ((state->current_step % 20) == 0) {                                           /* :2311-2320 */
        if (batch_size > 1)
            fprintf(stderr, "[TIMING] step=%d batch=%dx%d cuda_step=%.2fms (gpu=on)\n", state->current_step, batch_size, total_tokens, now_ms() - t0);
        else
            fprintf(stderr, "[TIMING] step=%d seq=%d cuda_step=%.2fms (gpu=on)\n", state->current_step, total_tokens, now_ms() - t0);
    }
    return loss;
}

float cuda_train_step_gpu_full(train_state_t* state, int* tokens, int num_tokens, cuda_train_context_t* ctx) {
    if (!state || !state->full_weights || !state->config || !ctx) return -1.0f;
    if (!fused_trainer(state, ctx, num_tokens, 1)) {
        took_opbyop_step(state);
        return cuda_train_step_gpu_full_opbyop(state, tokens, num_tokens, ctx);
    }
    int starts[2] = {0, num_tokens};
    return cuda_train_step_gpu_full_batch(state, tokens, num_tokens, starts, 1, ctx);
}

static void download_arena(train_state_t* state, int which, int field) {
    hip_model_config_t c;
    model_config_of(state, &c);
    int ns = 0;
    slot_t* s = arena_slots(state, &c, &ns);
    if (!s) return;
    for (int i = 0; i < ns; i++) {
        float* dst = field == 0 ? s[i].t->weight : field == 1 ? s[i].t->grad : field == 2 ? s[i].t->m : s[i].t->v;
        if (dst) hip_trainer_download_at(g.t, which, s[i].off, dst, (int64_t)s[i].t->size);
    }
    free(s);
}

void cuda_download_full_weights(cuda_train_context_t* ctx, train_state_t* state) {
    if (!ctx || !state || !state->full_weights || !state->config) return;
    if (!g.t || g.state != state) { cuda_download_full_weights_opbyop(ctx, state); return; }
    download_arena(state, 0, 0);                                    /* weights, then both moments: src/train_cuda.c:1256-1314 */
    download_arena(state, 2, 2);
    download_arena(state, 3, 3);
}

void cuda_download_gpu_gradients(cuda_train_context_t* ctx, train_state_t* state) {
    if (!ctx || !state || !state->full_weights || !state->config) return;
    if (!g.t || g.state != state) { cuda_download_gpu_gradients_opbyop(ctx, state); return; }
    download_arena(state, 1, 1);
}

float cuda_eval_forward(train_state_t* state, int* tokens, int num_tokens, cuda_train_context_t* ctx) {
    if (!state || !state->config || !ctx || num_tokens < 2) return -1.0f;            /* src/train_cuda.c:2679 */
    hip_trainer_t* t = state->full_weights ? fused_trainer(state, ctx, num_tokens, 1) : NULL;
    if (!t) return cuda_eval_forward_opbyop(state, tokens, num_tokens, ctx);
    int starts[2] = {0, num_tokens};
    return hip_eval_forward_batch(t, tokens, num_tokens, starts, 1);
}

float cuda_evaluate(train_state_t* state, int* val_tokens, int num_val_tokens, int* offsets, int num_samples, int max_seq_len,
                    int max_eval_samples, cuda_train_context_t* ctx, float* out_perplexity) {
    if (!state || !val_tokens || num_samples <= 0 || !ctx) {                         /* src/train_cuda.c:2816-2819 */
        if (out_perplexity) *out_perplexity = 0.0f;
        return -1.0f;
    }
    hip_trainer_t* t = state->full_weights ? fused_trainer(state, ctx, max_seq_len > 2 ? max_seq_len : 2, 1) : NULL;
    if (!t) return cuda_evaluate_opbyop(state, val_tokens, num_val_tokens, offsets, num_samples, max_seq_len, max_eval_samples, ctx, out_perplexity);
    return hip_evaluate(t, val_tokens, num_val_tokens, offsets, num_samples, max_seq_len, max_eval_samples, out_perplexity);
}
