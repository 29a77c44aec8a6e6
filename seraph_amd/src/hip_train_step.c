/*
 * hip_train_step.c - packed-batch full-weight and LoRA training steps (see hip_train.h).
 * Plain C over the kernel library's C ABI; one in-order stream, no host round trips
 * between the token upload and the 4-byte loss download.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "hip_train.h"
#include "seraph_hip.h"

#define CK(call)                                                                         \
    do {                                                                                 \
        int rc_ = (call);                                                                \
        if (rc_ != SERAPH_OK) {                                                          \
            fprintf(stderr, "ERROR: %s failed (%d): %s\n", #call, rc_, seraph_hip_last_error()); \
            return -1;                                                                   \
        }                                                                                \
    } while (0)

#define OPT_MAX_CLASSES 48
#define OPT_MAX_EVENTS  32768

typedef struct { int64_t in_norm, q, k, v, o, post_norm, gate, up, down, stride; } layer_layout_t;
typedef struct { int64_t A[7], B[7], in[7], out[7], stride; } lora_layout_t;   /* q k v o gate up down */

typedef struct {
    float *layer_in, *xn_attn, *q, *k, *v, *attn_out, *lse, *post_in, *xn_ffn, *gate, *up, *ffn_h;
    float *rms_q, *rms_k;        /* per token, with use_qk_norm */
    float* xa[7];                /* LoRA: scale * x A^T of each adapter present, kept for the backward */
} layer_act_t;

struct hip_trainer {
    hip_model_config_t cfg;
    hip_optim_config_t opt;
    int max_tokens, max_batch, lora;
    int64_t nparams, nlora;
    int64_t off_embed, off_final_norm, off_layer0;
    layer_layout_t L;
    lora_layout_t LL;
    seraph_stream_t stream;
    /* full-weight mode: the weight gradients run on a second stream beside the chain of input gradients, which
     * alone decides how soon the next kernel of the chain can start; events order the two streams around every
     * buffer they share */
    seraph_stream_t stream2;
    void* side_ev[6];            /* fork | down | gate-up | o | q-k-v | end */
    void* ws2;                   /* scratch of the products on stream2 */
    size_t ws2_bytes;
    char* norm_parts;            /* small steps: one region of partial rows per norm, folded by one launch after the backward */
    size_t norm_part_bytes;      /* size of one region; 0 = each norm's column sum follows its row pass */
    seraph_colsum_job_t* norm_jobs; /* host: the regions filled so far in this backward */
    int norm_job_count;
    int overlap;
    /* arenas */
    float *P, *G, *M, *V;
    int own_P, own_G, own_M, own_V;
    float *LP, *LG, *LM, *LV;
    /* activations */
    char* act_arena;
    size_t act_bytes;
    layer_act_t* act;
    float *final_in, *xn_final, *logits, *loss_rows, *red_a, *red_b, *tmp_h, *lora_tmp, *lora_tmp2;
    float *g_hidden, *g_tmp, *g_xn, *g_ffn, *g_gate, *g_up, *g_attn, *g_q, *g_k, *g_v;
    uint32_t *d_tokens, *d_targets, *d_starts;
    uint32_t* h_stage;           /* pinned: tokens | targets | starts */
    void* ws;
    size_t ws_bytes;
    void* attn_ws;               /* attention-backward scratch incl. the dS band; grown to the longest sequence seen */
    size_t attn_ws_bytes;
    int64_t max_seq_len;         /* of the current batch */
    size_t device_bytes;
    /* bookkeeping of src/train.c:5439-5463 */
    int accumulation_counter, optimizer_step;
    float last_lr;
    /* NaN/Inf flag lattice of src/train.c:4499-4546 (off unless enabled) */
    int nan_check, nan_detected;
    int step_counter;            /* training steps run (state->current_step of the reference) */
    char nan_dump_prefix[256];   /* "" = no buffer dumps on detection */
    uint32_t* d_nan_flags;
    uint32_t* h_nan_flags;
    uint32_t nan_flag_count;
    double attn_pairs;           /* sum over sequences of S(S+1)/2 for the current batch */
    void* ev[4];
    float phase_ms[3];
    /* optional per-op timing: one event pair per kernel-library call, folded per kernel class */
    int op_timing;
    hip_op_stat_t op_stats[OPT_MAX_CLASSES];
    int op_classes;
    void** op_ev;                /* [2 * OPT_MAX_EVENTS], created on demand */
    int op_ev_made, op_ev_used;
    int op_ev_class[OPT_MAX_EVENTS];
};

static int op_class(hip_trainer_t* t, const char* name) {
    for (int i = 0; i < t->op_classes; i++)
        if (t->op_stats[i].name == name || strcmp(t->op_stats[i].name, name) == 0) return i;
    if (t->op_classes >= OPT_MAX_CLASSES) return -1;
    memset(&t->op_stats[t->op_classes], 0, sizeof(hip_op_stat_t));
    t->op_stats[t->op_classes].name = name;
    return t->op_classes++;
}

/* Brackets one kernel-library call with events when op timing is on. */
static int op_begin(hip_trainer_t* t, const char* name, double flops, double bytes) {
    if (!t->op_timing || t->op_ev_used >= OPT_MAX_EVENTS) return -1;
    int c = op_class(t, name);
    if (c < 0) return -1;
    if (!t->op_ev) t->op_ev = (void**)calloc(2 * OPT_MAX_EVENTS, sizeof(void*));
    if (!t->op_ev) return -1;
    int i = t->op_ev_used;
    if (i >= t->op_ev_made) {
        if (seraph_hip_event_create(&t->op_ev[2 * i]) != SERAPH_OK || seraph_hip_event_create(&t->op_ev[2 * i + 1]) != SERAPH_OK) return -1;
        t->op_ev_made = i + 1;
    }
    t->op_stats[c].launches++;
    t->op_stats[c].flops += flops;
    t->op_stats[c].bytes += bytes;
    t->op_ev_class[i] = c;
    seraph_hip_event_record(t->op_ev[2 * i], t->stream);
    return i;
}

static void op_end(hip_trainer_t* t, int i) {
    if (i < 0) return;
    seraph_hip_event_record(t->op_ev[2 * i + 1], t->stream);
    t->op_ev_used = i + 1;
}

static void op_fold(hip_trainer_t* t) {
    for (int i = 0; i < t->op_ev_used; i++) {
        float ms = 0.f;
        if (seraph_hip_event_elapsed_ms(t->op_ev[2 * i], t->op_ev[2 * i + 1], &ms) == SERAPH_OK)
            t->op_stats[t->op_ev_class[i]].ms += ms;
    }
    t->op_ev_used = 0;
}

#define OP(name, flops, bytes, call)                     \
    do {                                                 \
        int oi_ = op_begin(t, (name), (flops), (bytes)); \
        int rc_ = (call);                                \
        op_end(t, oi_);                                  \
        if (rc_ != SERAPH_OK) {                          \
            fprintf(stderr, "ERROR: %s failed (%d): %s\n", #call, rc_, seraph_hip_last_error()); \
            return -1;                                   \
        }                                                \
    } while (0)

/* GEMM through the kernel library, classed by the kernel instantiation that will run */
#define GEMM(A_, B_, C_, M_, N_, K_, tA_, tB_, acc_)                                                   \
    OP(seraph_gemm_kernel_name((M_), (N_), (K_), (tA_), (tB_)), 2.0 * (double)(M_) * (double)(N_) * (double)(K_), 0.0, \
       seraph_gemm_scaled((A_), (B_), (C_), (M_), (N_), (K_), (tA_), (tB_), (acc_), 1.0f, t->ws, t->ws_bytes, t->stream))

/* a weight gradient: on the second stream with its own scratch when the step overlaps them (sw / w2 / w2b of run_step) */
#define WGEMM(A_, B_, C_, M_, N_, K_)                                                                  \
    OP(seraph_gemm_kernel_name((M_), (N_), (K_), 1, 0), 2.0 * (double)(M_) * (double)(N_) * (double)(K_), 0.0, \
       seraph_gemm_scaled((A_), (B_), (C_), (M_), (N_), (K_), 1, 0, 1, 1.0f, w2, w2b, sw))

/* several products sharing K, orientations and the accumulate flag in one launch (q / k / v, gate / up) */
#define GEMM_GROUP(probs_, count_, K_, tA_, tB_, acc_)                                                 \
    do {                                                                                               \
        double fl_ = 0.0;                                                                              \
        for (int gi_ = 0; gi_ < (count_); gi_++) fl_ += 2.0 * (double)(probs_)[gi_].M * (double)(probs_)[gi_].N * (double)(K_); \
        OP(seraph_gemm_grouped_kernel_name((probs_), (count_), (K_), (tA_), (tB_)), fl_, 0.0,          \
           seraph_gemm_grouped((probs_), (count_), (K_), (tA_), (tB_), (acc_), t->stream));            \
    } while (0)

/* an input gradient that is the sum of several products (gate + up, q + k + v) in one launch */
#define GEMM_CHAIN(terms_, count_, C_, M_, N_)                                                         \
    do {                                                                                               \
        double fl_ = 0.0;                                                                              \
        for (int gi_ = 0; gi_ < (count_); gi_++) fl_ += 2.0 * (double)(M_) * (double)(N_) * (double)(terms_)[gi_].K; \
        OP(seraph_gemm_chain_kernel_name((terms_), (count_), (C_), (M_), (N_), 0, 0), fl_, 0.0,        \
           seraph_gemm_chain((terms_), (count_), (C_), (M_), (N_), 0, 0, 0, t->stream));               \
    } while (0)

#define WGEMM_GROUP(probs_, count_, K_)                                                                \
    do {                                                                                               \
        double fl_ = 0.0;                                                                              \
        for (int gi_ = 0; gi_ < (count_); gi_++) fl_ += 2.0 * (double)(probs_)[gi_].M * (double)(probs_)[gi_].N * (double)(K_); \
        OP(seraph_gemm_grouped_kernel_name((probs_), (count_), (K_), 1, 0), fl_, 0.0,                  \
           seraph_gemm_grouped((probs_), (count_), (K_), 1, 0, 1, sw));                                \
    } while (0)

/* vulkan_rmsnorm_backward_batch of a norm (src/train.c:5071-5077, :5180-5193, :5342-5355).  A small full-weight step
 * runs the row pass alone and books the column sum for the one launch after the backward; a LoRA step has no use
 * for the norms' weight gradients (the reference sums them into a scratch that nothing reads, src/train.c:6381-6390)
 * and runs the row pass alone; otherwise the column sum follows its row pass. */
#define NORM_BWD(x_, w_, dy_, res_, dx_, gs_, bytes_)                                                  \
    do {                                                                                               \
        if (lora) {                                                                                    \
            int np_ = 0;                                                                               \
            OP("rmsnorm_backward", 0.0, (bytes_), seraph_rmsnorm_backward_rows((x_), (w_), (dy_), (res_), (dx_), T, h, eps, \
                                                                               t->ws, t->ws_bytes, &np_, s)); \
        } else if (t->norm_part_bytes) {                                                               \
            seraph_colsum_job_t* j_ = &t->norm_jobs[t->norm_job_count];                                \
            float* part_ = (float*)(t->norm_parts + (size_t)t->norm_job_count * t->norm_part_bytes);   \
            OP("rmsnorm_backward", 0.0, (bytes_), seraph_rmsnorm_backward_rows((x_), (w_), (dy_), (res_), (dx_), T, h, eps, \
                                                                               part_, t->norm_part_bytes, &j_->nparts, s)); \
            j_->partial = part_; j_->grad_scale = (gs_);                                               \
            t->norm_job_count++;                                                                       \
        } else {                                                                                       \
            OP("rmsnorm_backward", 0.0, (bytes_), seraph_rmsnorm_backward_residual((x_), (w_), (dy_), (res_), (dx_), (gs_), T, h, eps, \
                                                                                   t->ws, t->ws_bytes, s)); \
        }                                                                                              \
    } while (0)

/* the second stream picks up from this point of the first | marks a point of the second | the first waits for a mark */
#define SIDE_FORK()  do { if (ov) { if (!fork_armed || seraph_hip_event_armed()) { seraph_hip_event_on_next_op(NULL); CK(seraph_hip_event_record(t->side_ev[0], s)); } \
                                    fork_armed = 0; CK(seraph_hip_stream_wait_event(sw, t->side_ev[0])); } } while (0)
/* before the op that ends at a fork point: its last kernel completes the fork's event itself */
#define SIDE_ARM()   do { if (ov) { CK(seraph_hip_event_on_next_op(t->side_ev[0])); fork_armed = 1; } } while (0)
#define SIDE_MARK(i) do { if (ov) CK(seraph_hip_event_record(t->side_ev[(i)], sw)); } while (0)
#define SIDE_JOIN(i) do { if (ov) CK(seraph_hip_stream_wait_event(s, t->side_ev[(i)])); } while (0)

/* C (+)= alpha * product; K cut into runs through the trainer's scratch when the shape gains from it */
#define GEMM_SCALED(A_, B_, C_, M_, N_, K_, tA_, tB_, acc_, alpha_)                                    \
    OP("gemm_scaled", 2.0 * (double)(M_) * (double)(N_) * (double)(K_), 0.0,                           \
       seraph_gemm_scaled((A_), (B_), (C_), (M_), (N_), (K_), (tA_), (tB_), (acc_), (alpha_), t->ws, t->ws_bytes, t->stream))


/* ------------------------------------------------------------------ layouts */
static void make_layouts(hip_trainer_t* t) {
    const hip_model_config_t* c = &t->cfg;
    int64_t h = c->hidden, qd = (int64_t)c->heads * c->head_dim, kv = (int64_t)c->kv_heads * c->head_dim, f = c->ffn;
    t->off_embed = 0;
    t->off_final_norm = (int64_t)c->vocab * h;
    t->off_layer0 = t->off_final_norm + h;
    int64_t o = 0;
    t->L.in_norm = o; o += h;
    t->L.q = o; o += qd * h;
    t->L.k = o; o += kv * h;
    t->L.v = o; o += kv * h;
    t->L.o = o; o += h * qd;
    t->L.post_norm = o; o += h;
    t->L.gate = o; o += f * h;
    t->L.up = o; o += f * h;
    t->L.down = o; o += h * f;
    t->L.stride = o;
    t->nparams = t->off_layer0 + o * c->layers;
    int64_t ins[7] = {h, h, h, qd, h, h, f}, outs[7] = {qd, kv, kv, h, f, f, h};   /* src/lora.c:372-396 */
    o = 0;
    for (int p = 0; p < 7; p++) {
        t->LL.in[p] = ins[p]; t->LL.out[p] = outs[p];
        t->LL.A[p] = t->LL.B[p] = -1;
        if (c->lora_rank > 0 && ((c->lora_mask >> p) & 1)) {
            t->LL.A[p] = o; o += (int64_t)c->lora_rank * ins[p];
            t->LL.B[p] = o; o += outs[p] * (int64_t)c->lora_rank;
        }
    }
    t->LL.stride = o;
    t->nlora = o * c->layers;
}

void hip_param_layout(const hip_model_config_t* cfg, hip_param_layout_t* out) {
    hip_trainer_t tmp;
    memset(&tmp, 0, sizeof(tmp));
    tmp.cfg = *cfg;
    make_layouts(&tmp);
    out->embed = tmp.off_embed; out->final_norm = tmp.off_final_norm; out->layer0 = tmp.off_layer0;
    out->layer_stride = tmp.L.stride;
    out->in_norm = tmp.L.in_norm; out->q = tmp.L.q; out->k = tmp.L.k; out->v = tmp.L.v; out->o = tmp.L.o;
    out->post_norm = tmp.L.post_norm; out->gate = tmp.L.gate; out->up = tmp.L.up; out->down = tmp.L.down;
    out->count = tmp.nparams;
}

void hip_lora_layout(const hip_model_config_t* cfg, hip_lora_layout_t* out) {
    hip_trainer_t tmp;
    memset(&tmp, 0, sizeof(tmp));
    tmp.cfg = *cfg;
    make_layouts(&tmp);
    for (int p = 0; p < 7; p++) {
        out->A[p] = tmp.LL.A[p]; out->B[p] = tmp.LL.B[p];
        out->in_dim[p] = tmp.LL.in[p]; out->out_dim[p] = tmp.LL.out[p];
    }
    out->layer_stride = tmp.LL.stride;
    out->count = tmp.nlora;
}

int64_t hip_param_count(const hip_model_config_t* cfg) {
    hip_trainer_t tmp;
    memset(&tmp, 0, sizeof(tmp));
    tmp.cfg = *cfg;
    make_layouts(&tmp);
    return tmp.nparams;
}

int64_t hip_lora_param_count(const hip_model_config_t* cfg) {
    hip_trainer_t tmp;
    memset(&tmp, 0, sizeof(tmp));
    tmp.cfg = *cfg;
    make_layouts(&tmp);
    return tmp.nlora;
}

/* ------------------------------------------------------------------ create / free */
static const size_t kAttnBandLimit = (size_t)24 << 30;

static size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

static int dev_alloc(hip_trainer_t* t, void** p, size_t bytes) {
    if (seraph_hip_malloc(p, bytes) != SERAPH_OK) {
        fprintf(stderr, "ERROR: device allocation of %zu bytes failed: %s\n", bytes, seraph_hip_last_error());
        return -1;
    }
    t->device_bytes += bytes;
    return 0;
}

static size_t max_sz(size_t a, size_t b) { return a > b ? a : b; }

hip_trainer_t* hip_trainer_create(const hip_model_config_t* cfg, const hip_optim_config_t* opt,
                                  int max_tokens, int max_batch, int device_index,
                                  float* ext_params, float* ext_grads, float* ext_m, float* ext_v) {
    if (!cfg || !opt || max_tokens < 2 || max_batch < 1) return NULL;
    if (cfg->heads % cfg->kv_heads != 0 || cfg->hidden % 4 != 0 || cfg->ffn % 4 != 0 ||
        !(cfg->head_dim == 32 || cfg->head_dim == 64 || cfg->head_dim == 128)) {
        fprintf(stderr, "ERROR: unsupported model shape (heads %% kv_heads, hidden/ffn %% 4, head_dim in {32,64,128})\n");
        return NULL;
    }
    if (seraph_hip_init(device_index) != SERAPH_OK) {
        fprintf(stderr, "ERROR: %s\n", seraph_hip_last_error());
        return NULL;
    }
    hip_trainer_t* t = (hip_trainer_t*)calloc(1, sizeof(*t));
    if (!t) return NULL;
    t->cfg = *cfg; t->opt = *opt;
    t->max_tokens = max_tokens; t->max_batch = max_batch;
    t->lora = cfg->lora_rank > 0;
    snprintf(t->nan_dump_prefix, sizeof(t->nan_dump_prefix), "/tmp/seraph_nan_step");   /* src/train.c:5566 */
    make_layouts(t);
    if (seraph_hip_stream_create(&t->stream) != SERAPH_OK) goto fail;
    for (int i = 0; i < 4; i++) if (seraph_hip_event_create(&t->ev[i]) != SERAPH_OK) goto fail;
    if (seraph_hip_stream_create(&t->stream2) != SERAPH_OK) goto fail;
    for (int i = 0; i < 6; i++)
        if (seraph_hip_event_create_sync(&t->side_ev[i]) != SERAPH_OK) goto fail;
    /* Beside a chain of small products the second stream fills CUs that the chain's ramps and tails leave idle
     * (+3 % at 2048 tokens x 512); beside products that fill the chip by themselves it only interleaves two tile
     * orders in every L2 (-7 % at 16384 tokens x 2048).  The adapter gradients of a LoRA step (rank-sized products,
     * eight short launches per adapter that nothing on the chain waits for) can leave the chain the same way, but
     * beside the frozen model's large products that costs more than the launches it hides (1 x 2048 tokens of the
     * 1.7B shape: 128.9 against 126.5 ms), so a LoRA step stays on one stream unless told otherwise.
     * hip_trainer_enable_wgrad_overlap overrides the choice. */
    t->overlap = t->lora ? 0 : (int64_t)max_tokens * cfg->hidden <= ((int64_t)1 << 22);

    const size_t pbytes = (size_t)t->nparams * sizeof(float);
    t->P = ext_params;
    if (!t->P) { if (dev_alloc(t, (void**)&t->P, pbytes)) goto fail; t->own_P = 1; }
    if (!t->lora) {
        t->G = ext_grads; t->M = ext_m; t->V = ext_v;
        if (!t->G) { if (dev_alloc(t, (void**)&t->G, pbytes)) goto fail; t->own_G = 1; }
        if (!t->M) { if (dev_alloc(t, (void**)&t->M, pbytes)) goto fail; t->own_M = 1; }
        if (!t->V) { if (dev_alloc(t, (void**)&t->V, pbytes)) goto fail; t->own_V = 1; }
        if (t->own_G && seraph_fill_u32(t->G, 0, (size_t)t->nparams, t->stream) != SERAPH_OK) goto fail;
        if (t->own_M && seraph_fill_u32(t->M, 0, (size_t)t->nparams, t->stream) != SERAPH_OK) goto fail;
        if (t->own_V && seraph_fill_u32(t->V, 0, (size_t)t->nparams, t->stream) != SERAPH_OK) goto fail;
    } else {
        const size_t lbytes = (size_t)t->nlora * sizeof(float);
        if (dev_alloc(t, (void**)&t->LP, lbytes) || dev_alloc(t, (void**)&t->LG, lbytes) ||
            dev_alloc(t, (void**)&t->LM, lbytes) || dev_alloc(t, (void**)&t->LV, lbytes)) goto fail;
        float* all[4] = {t->LP, t->LG, t->LM, t->LV};
        for (int i = 0; i < 4; i++) if (seraph_fill_u32(all[i], 0, (size_t)t->nlora, t->stream) != SERAPH_OK) goto fail;
    }

    /* activation arena */
    {
        const size_t T = (size_t)max_tokens, h = (size_t)cfg->hidden, f = (size_t)cfg->ffn, Vv = (size_t)cfg->vocab;
        const size_t qd = (size_t)cfg->heads * cfg->head_dim, kv = (size_t)cfg->kv_heads * cfg->head_dim;
        const size_t r = cfg->lora_rank > 0 ? (size_t)cfg->lora_rank : 1;
        size_t adapters = 0;
        for (int q = 0; q < 7; q++) adapters += t->LL.A[q] >= 0 ? 1 : 0;
        const size_t per_layer = 4 * up256(T * h * 4) + 2 * up256(T * qd * 4) + 2 * up256(T * kv * 4) +
                                 up256(T * cfg->heads * 4) + 3 * up256(T * f * 4) + (cfg->use_qk_norm ? 2 * up256(T * 4) : 0) +
                                 adapters * up256(T * r * 4);
        const size_t rest = 2 * up256(T * h * 4) + up256(T * Vv * 4) + 3 * up256(T * 4) + up256(T * h * 4) + up256(4 * T * r * 4) + up256(T * r * 4) +
                            3 * up256(T * h * 4) + 3 * up256(T * f * 4) + 2 * up256(T * qd * 4) + 2 * up256(T * kv * 4) +
                            2 * up256(T * 4) + up256(((size_t)max_batch + 1) * 4);
        t->act_bytes = per_layer * (size_t)cfg->layers + rest;
        if (dev_alloc(t, (void**)&t->act_arena, t->act_bytes)) goto fail;
        t->act = (layer_act_t*)calloc((size_t)cfg->layers, sizeof(layer_act_t));
        if (!t->act) goto fail;
        char* p = t->act_arena;
#define TAKE(dst, bytes) do { (dst) = (void*)p; p += up256(bytes); } while (0)
        for (int l = 0; l < cfg->layers; l++) {
            layer_act_t* a = &t->act[l];
            TAKE(a->layer_in, T * h * 4); TAKE(a->xn_attn, T * h * 4); TAKE(a->post_in, T * h * 4); TAKE(a->xn_ffn, T * h * 4);
            TAKE(a->q, T * qd * 4); TAKE(a->attn_out, T * qd * 4); TAKE(a->k, T * kv * 4); TAKE(a->v, T * kv * 4);
            TAKE(a->lse, T * cfg->heads * 4);
            if (cfg->use_qk_norm) { TAKE(a->rms_q, T * 4); TAKE(a->rms_k, T * 4); }
            TAKE(a->gate, T * f * 4); TAKE(a->up, T * f * 4); TAKE(a->ffn_h, T * f * 4);
            for (int q = 0; q < 7; q++) if (t->LL.A[q] >= 0) TAKE(a->xa[q], T * r * 4);
        }
        TAKE(t->final_in, T * h * 4); TAKE(t->xn_final, T * h * 4); TAKE(t->logits, T * Vv * 4);
        TAKE(t->loss_rows, T * 4); TAKE(t->red_a, T * 4); TAKE(t->red_b, T * 4);
        TAKE(t->tmp_h, T * h * 4); TAKE(t->lora_tmp, 4 * T * r * 4); TAKE(t->lora_tmp2, T * r * 4);
        TAKE(t->g_hidden, T * h * 4); TAKE(t->g_tmp, T * h * 4); TAKE(t->g_xn, T * h * 4);
        TAKE(t->g_ffn, T * f * 4); TAKE(t->g_gate, T * f * 4); TAKE(t->g_up, T * f * 4);
        TAKE(t->g_attn, T * qd * 4); TAKE(t->g_q, T * qd * 4); TAKE(t->g_k, T * kv * 4); TAKE(t->g_v, T * kv * 4);
        TAKE(t->d_tokens, T * 4); TAKE(t->d_targets, T * 4); TAKE(t->d_starts, ((size_t)max_batch + 1) * 4);
#undef TAKE
        if ((size_t)(p - t->act_arena) > t->act_bytes) { fprintf(stderr, "ERROR: activation arena layout overflow\n"); goto fail; }
    }
    t->ws_bytes = max_sz(seraph_rmsnorm_backward_ws_bytes(max_tokens, cfg->hidden),
                         seraph_embedding_backward_ws_bytes(max_tokens, cfg->vocab));
    {
        /* products with a small output and K = tokens (narrow weight gradients, the rank-sized LoRA products) run
         * with K cut into runs through the same scratch; a call whose scratch is too small falls back by itself */
        const int64_t Tm = max_tokens, r = cfg->lora_rank, wide = (int64_t)cfg->heads * cfg->head_dim;
        const int64_t kvw = (int64_t)cfg->kv_heads * cfg->head_dim;
        const int64_t dims[4] = {cfg->hidden, wide, cfg->ffn, kvw};
        for (int i = 0; i < 4; i++) {
            if (r > 0) {
                t->ws_bytes = max_sz(t->ws_bytes, seraph_gemm_scaled_ws_bytes(Tm, r, dims[i], 0, 1));
                t->ws_bytes = max_sz(t->ws_bytes, seraph_gemm_scaled_ws_bytes(Tm, r, dims[i], 0, 0));
                t->ws_bytes = max_sz(t->ws_bytes, seraph_gemm_scaled_ws_bytes(dims[i], r, Tm, 1, 0));
                t->ws_bytes = max_sz(t->ws_bytes, seraph_gemm_scaled_ws_bytes(r, dims[i], Tm, 1, 0));
                t->ws2_bytes = t->ws_bytes;
                if (i == 3) t->ws_bytes = 4 * t->ws_bytes + 64;    /* the adapters of a layer share launches: all their runs at once */
            } else {
                for (int j = 0; j < 4; j++) {
                    t->ws_bytes = max_sz(t->ws_bytes, seraph_gemm_scaled_ws_bytes(dims[i], dims[j], Tm, 1, 0));
                    t->ws2_bytes = max_sz(t->ws2_bytes, seraph_gemm_scaled_ws_bytes(dims[i], dims[j], Tm, 1, 0));
                }
            }
        }
        if (r <= 0) t->ws2_bytes = max_sz(t->ws2_bytes, seraph_gemm_scaled_ws_bytes(cfg->vocab, cfg->hidden, Tm, 1, 0));
    }
    if (dev_alloc(t, &t->ws, t->ws_bytes)) goto fail;
    if (t->stream2 && t->ws2_bytes && dev_alloc(t, &t->ws2, t->ws2_bytes)) goto fail;
    /* The 2 L + 1 column sums of the norms' weight gradients are 4-5 us launches on the chain of dependent kernels
     * and nothing waits for them before the optimizer: a step small enough for that to show (the same bound as for
     * the second stream) keeps every norm's partial rows and folds them all with one launch after the backward. */
    if (!t->lora && (int64_t)max_tokens * cfg->hidden <= ((int64_t)1 << 22)) {
        const size_t regions = 2 * (size_t)cfg->layers + 1;
        t->norm_part_bytes = (seraph_rmsnorm_backward_ws_bytes(max_tokens, cfg->hidden) + 255) & ~(size_t)255;
        if (dev_alloc(t, (void**)&t->norm_parts, regions * t->norm_part_bytes)) goto fail;
        t->norm_jobs = (seraph_colsum_job_t*)calloc(regions, sizeof(*t->norm_jobs));
        if (!t->norm_jobs) goto fail;
    }
    if (seraph_hip_host_alloc((void**)&t->h_stage, ((size_t)2 * max_tokens + max_batch + 1) * 4) != SERAPH_OK) goto fail;
    if (seraph_hip_stream_sync(t->stream) != SERAPH_OK) goto fail;
    return t;
fail:
    fprintf(stderr, "ERROR: hip_trainer_create failed: %s\n", seraph_hip_last_error());
    hip_trainer_free(t);
    return NULL;
}

void hip_trainer_free(hip_trainer_t* t) {
    if (!t) return;
    if (t->stream2) seraph_hip_stream_sync(t->stream2);
    if (t->stream) seraph_hip_stream_sync(t->stream);
    if (t->own_P) seraph_hip_free(t->P);
    if (t->own_G) seraph_hip_free(t->G);
    if (t->own_M) seraph_hip_free(t->M);
    if (t->own_V) seraph_hip_free(t->V);
    seraph_hip_free(t->LP); seraph_hip_free(t->LG); seraph_hip_free(t->LM); seraph_hip_free(t->LV);
    seraph_hip_free(t->act_arena);
    seraph_hip_free(t->ws);
    seraph_hip_free(t->ws2);
    seraph_hip_free(t->norm_parts);
    free(t->norm_jobs);
    seraph_hip_free(t->attn_ws);
    seraph_hip_free(t->d_nan_flags);
    free(t->h_nan_flags);
    seraph_hip_host_free(t->h_stage);
    for (int i = 0; i < 4; i++) seraph_hip_event_destroy(t->ev[i]);
    if (t->op_ev) {
        for (int i = 0; i < 2 * t->op_ev_made; i++) seraph_hip_event_destroy(t->op_ev[i]);
        free(t->op_ev);
    }
    for (int i = 0; i < 6; i++) if (t->side_ev[i]) seraph_hip_event_destroy(t->side_ev[i]);
    if (t->stream2) seraph_hip_stream_destroy(t->stream2);
    seraph_hip_stream_destroy(t->stream);
    free(t->act);
    free(t);
}

static float* arena_of(hip_trainer_t* t, int which, int64_t* count) {
    float* all[8] = {t->P, t->G, t->M, t->V, t->LP, t->LG, t->LM, t->LV};
    if (which < 0 || which > 7) return NULL;
    *count = which < 4 ? t->nparams : t->nlora;
    return all[which];
}

int hip_trainer_upload(hip_trainer_t* t, int which, const float* host, int64_t count) {
    int64_t n = 0;
    float* d = t ? arena_of(t, which, &n) : NULL;
    if (!d || !host || count != n) return -1;
    return seraph_hip_h2d(d, host, (size_t)n * 4, t->stream) == SERAPH_OK ? 0 : -1;
}

int hip_trainer_download(hip_trainer_t* t, int which, float* host, int64_t count) {
    int64_t n = 0;
    float* d = t ? arena_of(t, which, &n) : NULL;
    if (!d || !host || count != n) return -1;
    return seraph_hip_d2h(host, d, (size_t)n * 4, t->stream) == SERAPH_OK ? 0 : -1;
}

int hip_trainer_upload_at(hip_trainer_t* t, int which, int64_t offset, const float* host, int64_t count) {
    int64_t n = 0;
    float* d = t ? arena_of(t, which, &n) : NULL;
    if (!d || !host || offset < 0 || count < 0 || offset + count > n) return -1;
    if (count == 0) return 0;
    return seraph_hip_h2d(d + offset, host, (size_t)count * 4, t->stream) == SERAPH_OK ? 0 : -1;
}

int hip_trainer_download_at(hip_trainer_t* t, int which, int64_t offset, float* host, int64_t count) {
    int64_t n = 0;
    float* d = t ? arena_of(t, which, &n) : NULL;
    if (!d || !host || offset < 0 || count < 0 || offset + count > n) return -1;
    if (count == 0) return 0;
    return seraph_hip_d2h(host, d + offset, (size_t)count * 4, t->stream) == SERAPH_OK ? 0 : -1;
}

void hip_trainer_set_schedule(hip_trainer_t* t, float learning_rate, int optimizer_step, int accumulation_counter) {
    if (!t) return;
    t->opt.learning_rate = learning_rate;
    if (optimizer_step >= 0) t->optimizer_step = optimizer_step;
    if (accumulation_counter >= 0) t->accumulation_counter = accumulation_counter;
}

void hip_trainer_set_step_counter(hip_trainer_t* t, int steps_run) {
    if (t && steps_run >= 0) t->step_counter = steps_run;
}

int hip_trainer_accumulation_counter(const hip_trainer_t* t) { return t ? t->accumulation_counter : -1; }

int64_t hip_trainer_arena_count(hip_trainer_t* t, int which) {
    int64_t n = 0;
    return (t && arena_of(t, which, &n)) ? n : 0;
}

void* hip_trainer_device_ptr(hip_trainer_t* t, int which) {
    int64_t n;
    return t ? (void*)arena_of(t, which, &n) : NULL;
}

int hip_trainer_optimizer_step(const hip_trainer_t* t) { return t ? t->optimizer_step : -1; }
float hip_trainer_last_lr(const hip_trainer_t* t) { return t ? t->last_lr : 0.0f; }
size_t hip_trainer_device_bytes(const hip_trainer_t* t) { return t ? t->device_bytes : 0; }
void hip_trainer_last_timing(const hip_trainer_t* t, float ms[3]) {
    for (int i = 0; i < 3; i++) ms[i] = t ? t->phase_ms[i] : 0.0f;
}

void hip_trainer_enable_op_timing(hip_trainer_t* t, int on) { if (t) t->op_timing = on ? 1 : 0; }

void hip_trainer_enable_wgrad_overlap(hip_trainer_t* t, int on) { if (t) t->overlap = (on && t->stream2) ? 1 : 0; }
void hip_trainer_reset_op_stats(hip_trainer_t* t) { if (t) { t->op_classes = 0; t->op_ev_used = 0; } }
int hip_trainer_op_stats(const hip_trainer_t* t, hip_op_stat_t* out, int max) {
    if (!t || !out) return 0;
    int n = t->op_classes < max ? t->op_classes : max;
    memcpy(out, t->op_stats, (size_t)n * sizeof(hip_op_stat_t));
    return n;
}

/* ------------------------------------------------------------------ the step */
/* out (+)= ((x A^T) s) B^T, src/train.c:5778-5796 */
/* xa receives (x A^T) s and stays: the backward's first product (src/train.c:5815-5822) is this same one */
static int lora_forward_add(hip_trainer_t* t, const float* x, float* out, const float* A, const float* B,
                            int64_t T, int64_t in, int64_t outd, float* xa) {
    const int r = t->cfg.lora_rank;
    const float s = t->cfg.lora_alpha / (float)r;
    GEMM_SCALED(x, A, xa, T, r, in, 0, 1, 0, s);
    GEMM(xa, B, out, T, outd, r, 0, 1, 1);
    return 0;
}

/* src/train.c:5803-5845 with grad_input == NULL, as every call site passes it; (x A^T) s comes from the forward (xa)
 * instead of being formed again */
/* The four products are rank-sized and nothing on the chain of input gradients reads their results, so the step may
 * run them on its second stream (side != 0: that stream's scratch and its own tmp). */
static int lora_backward(hip_trainer_t* t, const float* dY, const float* x, const float* xa, const float* B,
                         float* gA, float* gB, int64_t T, int64_t in, int64_t outd, int side) {
    const int r = t->cfg.lora_rank;
    const float s = t->cfg.lora_alpha / (float)r;
    float* tmp = side ? t->lora_tmp2 : t->lora_tmp;
    void* ws = side ? t->ws2 : t->ws;
    const size_t wsb = side ? t->ws2_bytes : t->ws_bytes;
    seraph_stream_t st = side ? t->stream2 : t->stream;
#define LGEMM(A_, B_, C_, M_, N_, K_, tA_, tB_, acc_, alpha_)                                          \
    OP("gemm_scaled", 2.0 * (double)(M_) * (double)(N_) * (double)(K_), 0.0,                           \
       seraph_gemm_scaled((A_), (B_), (C_), (M_), (N_), (K_), (tA_), (tB_), (acc_), (alpha_), ws, wsb, st))
    LGEMM(dY, xa, gB, outd, r, T, 1, 0, 1, 1.0f);
    LGEMM(dY, B, tmp, T, r, outd, 0, 0, 0, s);
    LGEMM(tmp, x, gA, r, in, T, 1, 0, 1, 1.0f);
#undef LGEMM
    return 0;
}

/* The same for the adapters of one layer that are due at the same point of the step (q, k, v; gate, up; in the backward
 * also o with q, k, v and down with gate, up, whose operands are still in place then): each kind of product is one
 * launch for all of them (seraph_gemm_scaled_grouped), every product computed exactly as the single call computes it. */
typedef struct { const float* x; float* out; const float* A; const float* B; int64_t in, outd; float* xa; } lora_fwd_item_t;
typedef struct { const float* dY; const float* x; const float* xa; const float* B; float* gA; float* gB; int64_t in, outd; } lora_bwd_item_t;

static int lora_forward_group(hip_trainer_t* t, const lora_fwd_item_t* it, int n, int64_t T) {
    if (n <= 0) return 0;
    const int r = t->cfg.lora_rank;
    const float s = t->cfg.lora_alpha / (float)r;
    seraph_gemm_scaled_problem_t p1[4], p2[4];
    double fl = 0.0;
    for (int i = 0; i < n; i++) {
        p1[i] = (seraph_gemm_scaled_problem_t){it[i].x, it[i].A, it[i].xa, T, r, it[i].in};
        p2[i] = (seraph_gemm_scaled_problem_t){it[i].xa, it[i].B, it[i].out, T, it[i].outd, r};
        fl += 2.0 * (double)T * r * (double)it[i].in;
    }
    OP("gemm_scaled", fl, 0.0, seraph_gemm_scaled_grouped(p1, n, 0, 1, 0, s, t->ws, t->ws_bytes, t->stream));
    fl = 0.0;
    for (int i = 0; i < n; i++) fl += 2.0 * (double)T * r * (double)it[i].outd;
    OP("gemm_scaled", fl, 0.0, seraph_gemm_scaled_grouped(p2, n, 0, 1, 1, 1.0f, t->ws, t->ws_bytes, t->stream));
    return 0;
}

static int lora_backward_group(hip_trainer_t* t, const lora_bwd_item_t* it, int n, int64_t T) {
    if (n <= 0) return 0;
    const int r = t->cfg.lora_rank;
    const float s = t->cfg.lora_alpha / (float)r;
    seraph_gemm_scaled_problem_t pb[4], pt[4], pa[4];
    double fb = 0.0, fa = 0.0;
    for (int i = 0; i < n; i++) {
        float* tmp = t->lora_tmp + (size_t)i * (size_t)T * (size_t)r;
        pb[i] = (seraph_gemm_scaled_problem_t){it[i].dY, it[i].xa, it[i].gB, it[i].outd, r, T};     /* src/train.c:5823-5829 */
        pt[i] = (seraph_gemm_scaled_problem_t){it[i].dY, it[i].B, tmp, T, r, it[i].outd};           /* :5831-5836 */
        pa[i] = (seraph_gemm_scaled_problem_t){tmp, it[i].x, it[i].gA, r, it[i].in, T};             /* :5837-5841 */
        fb += 2.0 * (double)T * r * (double)it[i].outd;
        fa += 2.0 * (double)T * r * (double)it[i].in;
    }
    OP("gemm_scaled", fb, 0.0, seraph_gemm_scaled_grouped(pb, n, 1, 0, 1, 1.0f, t->ws, t->ws_bytes, t->stream));
    OP("gemm_scaled", fb, 0.0, seraph_gemm_scaled_grouped(pt, n, 0, 0, 0, s, t->ws, t->ws_bytes, t->stream));
    OP("gemm_scaled", fa, 0.0, seraph_gemm_scaled_grouped(pa, n, 1, 0, 1, 1.0f, t->ws, t->ws_bytes, t->stream));
    return 0;
}

static int upload_batch(hip_trainer_t* t, const int* tokens, int T, const int* seq_starts, int batch) {
    uint32_t* tok = t->h_stage;
    uint32_t* tgt = tok + T;
    uint32_t* st = tgt + T;
    for (int b = 0; b <= batch; b++) st[b] = seq_starts ? (uint32_t)seq_starts[b] : (b == 0 ? 0u : (uint32_t)T);
    if (st[0] != 0 || st[batch] != (uint32_t)T) { fprintf(stderr, "ERROR: seq_starts must run from 0 to total_tokens\n"); return -1; }
    t->attn_pairs = 0.0;
    t->max_seq_len = 1;
    for (int b = 0; b < batch; b++) {
        if (st[b + 1] > st[b] && (int64_t)(st[b + 1] - st[b]) > t->max_seq_len) t->max_seq_len = st[b + 1] - st[b];
        if (st[b + 1] > st[b]) t->attn_pairs += 0.5 * (double)(st[b + 1] - st[b]) * (double)(st[b + 1] - st[b] + 1);
        if (st[b + 1] <= st[b]) { fprintf(stderr, "ERROR: empty or decreasing sequence %d in seq_starts\n", b); return -1; }
        for (uint32_t i = st[b]; i < st[b + 1]; i++) {                     /* src/train_cuda.c:2029-2043 */
            tok[i] = tokens[i] < 0 ? 0u : (uint32_t)tokens[i];
            tgt[i] = (i + 1 < st[b + 1]) ? (tokens[i + 1] < 0 ? 0u : (uint32_t)tokens[i + 1]) : 0u;
        }
    }
    /* attention-backward scratch: the dS band for this batch's longest sequence when it stays under
     * kAttnBandLimit bytes (5 matrix products), else the fixed part only (7 products) */
    {
        const hip_model_config_t* c = &t->cfg;
        size_t need = seraph_attention_backward_ws_bytes_banded(T, c->heads, c->kv_heads, c->head_dim, t->max_seq_len);
        if (need > kAttnBandLimit) need = seraph_attention_backward_ws_bytes(T, c->heads, c->kv_heads, c->head_dim);
        if (need > t->attn_ws_bytes) {
            CK(seraph_hip_stream_sync(t->stream));
            if (t->attn_ws) { seraph_hip_free(t->attn_ws); t->device_bytes -= t->attn_ws_bytes; t->attn_ws = NULL; t->attn_ws_bytes = 0; }
            if (dev_alloc(t, &t->attn_ws, need)) return -1;
            t->attn_ws_bytes = need;
        }
    }
    CK(seraph_hip_h2d(t->d_tokens, tok, (size_t)T * 4, t->stream));
    CK(seraph_hip_h2d(t->d_targets, tgt, (size_t)T * 4, t->stream));
    CK(seraph_hip_h2d(t->d_starts, st, ((size_t)batch + 1) * 4, t->stream));
    return 0;
}

/* One flag of the lattice: flags[idx] |= 1 when the buffer holds a NaN or Inf. */
#define NANCHK(ptr, n, idx)                                                                              \
    do {                                                                                                 \
        if (t->nan_check)                                                                                \
            OP("nan_check", 0.0, 4.0 * (double)(n), seraph_nan_check((ptr), (size_t)(n), t->d_nan_flags, (idx), s)); \
    } while (0)

static int nan_flags_any(hip_trainer_t* t) {
    if (seraph_hip_d2h(t->h_nan_flags, t->d_nan_flags, (size_t)t->nan_flag_count * 4, t->stream) != SERAPH_OK) return -1;
    for (uint32_t i = 0; i < t->nan_flag_count; i++) if (t->h_nan_flags[i]) return 1;
    return 0;
}

/* One-shot dump of the step's buffers when the flag lattice reports a NaN/Inf, in the files and layouts of
 * src/train.c:5562-5653 (raw little-endian FP32 / uint32, "<prefix>_<step>_<name>"), which the reference's
 * tools/nan_dump_inspect.c reads.  Differences that the layout cannot hide: the cross entropy writes its gradient
 * over the logits, so logits.f32 is recomputed from hidden_norm and the embedding after grad_logits has been
 * written; silu(gate) is not cached by this step and is recomputed too; with packed batches targets and
 * grad_logits hold the first T - 1 rows (rows of sequence-final tokens are zero). */
static int dump_dev(hip_trainer_t* t, const char* prefix, const char* name, const void* dev, size_t count) {
    char path[512];
    snprintf(path, sizeof(path), "%s_%s", prefix, name);
    FILE* f = fopen(path, "wb");
    if (!f) return -1;
    const size_t chunk = (size_t)16 << 20;                     /* elements per round trip */
    uint32_t* host = (uint32_t*)malloc((count < chunk ? count : chunk) * 4);
    int rc = host ? 0 : -1;
    for (size_t o = 0; o < count && rc == 0; o += chunk) {
        const size_t n = count - o < chunk ? count - o : chunk;
        if (seraph_hip_d2h(host, (const uint32_t*)dev + o, n * 4, t->stream) != SERAPH_OK || fwrite(host, 4, n, f) != n) rc = -1;
    }
    free(host);
    fclose(f);
    return rc;
}

static void nan_dump(hip_trainer_t* t, int total_tokens) {
    if (!t->nan_dump_prefix[0]) return;
    const hip_model_config_t* c = &t->cfg;
    const size_t T = (size_t)total_tokens, h = (size_t)c->hidden, f = (size_t)c->ffn, V = (size_t)c->vocab;
    const size_t qd = (size_t)c->heads * c->head_dim, kv = (size_t)c->kv_heads * c->head_dim, np = T - 1;
    char prefix[320], path[400];
    snprintf(prefix, sizeof(prefix), "%s_%d", t->nan_dump_prefix, t->step_counter + 1);
    snprintf(path, sizeof(path), "%s_meta.txt", prefix);
    FILE* meta = fopen(path, "wb");
    if (meta) {
        fprintf(meta, "step=%d\nseq=%d\nnum_predictions=%d\nhidden_size=%d\nq_dim=%d\nkv_dim=%d\nvocab_size=%d\n"
                "num_layers=%d\nnum_heads=%d\nkv_heads=%d\nhead_dim=%d\nlr=%g\n", t->step_counter + 1, total_tokens, (int)np,
                c->hidden, (int)qd, (int)kv, c->vocab, c->layers, c->heads, c->kv_heads, c->head_dim, (double)t->opt.learning_rate);
        fclose(meta);
    }
    dump_dev(t, prefix, "tokens.u32", t->d_tokens, T);
    dump_dev(t, prefix, "targets.u32", t->d_targets, np);
    dump_dev(t, prefix, "hidden.f32", t->final_in, T * h);
    dump_dev(t, prefix, "hidden_norm.f32", t->xn_final, T * h);
    dump_dev(t, prefix, "grad_logits.f32", t->logits, np * V);
    if (seraph_gemm(t->xn_final, t->P + t->off_embed, t->logits, (int64_t)T, (int64_t)V, (int64_t)h, 0, 1, 0, t->stream) == SERAPH_OK)
        dump_dev(t, prefix, "logits.f32", t->logits, T * V);
    dump_dev(t, prefix, "grad_hidden.f32", t->g_hidden, T * h);
    dump_dev(t, prefix, "grad_tmp_hidden.f32", t->g_tmp, T * h);
    dump_dev(t, prefix, "grad_x_norm.f32", t->g_xn, T * h);
    dump_dev(t, prefix, "grad_hidden_start.f32", t->g_hidden, T * h);
    dump_dev(t, prefix, "grad_ffn.f32", t->g_ffn, T * f);
    dump_dev(t, prefix, "grad_gate.f32", t->g_gate, T * f);
    dump_dev(t, prefix, "grad_up.f32", t->g_up, T * f);
    if (c->layers > 0) {
        const layer_act_t* a = &t->act[0];
        dump_dev(t, prefix, "L0_layer_in.f32", a->layer_in, T * h);
        dump_dev(t, prefix, "L0_x_norm_attn.f32", a->xn_attn, T * h);
        dump_dev(t, prefix, "L0_post_attn_in.f32", a->post_in, T * h);
        dump_dev(t, prefix, "L0_x_norm_ffn.f32", a->xn_ffn, T * h);
        dump_dev(t, prefix, "L0_ffn_gate.f32", a->gate, T * f);
        dump_dev(t, prefix, "L0_ffn_up.f32", a->up, T * f);
        if (seraph_silu(a->gate, t->g_ffn, T * f, t->stream) == SERAPH_OK)     /* grad_ffn is on disk already */
            dump_dev(t, prefix, "L0_silu.f32", t->g_ffn, T * f);
        dump_dev(t, prefix, "L0_ffn_hidden.f32", a->ffn_h, T * f);
        dump_dev(t, prefix, "L0_q.f32", a->q, T * qd);
        dump_dev(t, prefix, "L0_k.f32", a->k, T * kv);
        dump_dev(t, prefix, "L0_v.f32", a->v, T * kv);
        dump_dev(t, prefix, "L0_attn_out.f32", a->attn_out, T * qd);
        dump_dev(t, prefix, "grad_attn.f32", t->g_attn, T * qd);
        dump_dev(t, prefix, "grad_q.f32", t->g_q, T * qd);
        dump_dev(t, prefix, "grad_k.f32", t->g_k, T * kv);
        dump_dev(t, prefix, "grad_v.f32", t->g_v, T * kv);
    }
    fprintf(stderr, "[NAN-DUMP] wrote buffers with prefix %s_*\n", prefix);
}

enum { STEP_TRAIN = 0, STEP_EVAL = 1 };

static float run_step(hip_trainer_t* t, const int* tokens, int total_tokens, const int* seq_starts, int batch,
                      int run_optimizer, int mode) {
    if (!t || !tokens || total_tokens < 2 || batch < 1) return -1.0f;
    if (total_tokens > t->max_tokens || batch > t->max_batch) {
        fprintf(stderr, "ERROR: batch of %d tokens / %d sequences exceeds the trainer's capacity (%d / %d)\n",
                total_tokens, batch, t->max_tokens, t->max_batch);
        return -1.0f;
    }
    if (!seq_starts && batch != 1) return -1.0f;
    const hip_model_config_t* c = &t->cfg;
    const int lora = t->lora;
    const int64_t T = total_tokens, h = c->hidden, f = c->ffn, V = c->vocab;
    const int H = c->heads, KVH = c->kv_heads, D = c->head_dim, NL = c->layers;
    const int64_t qd = (int64_t)H * D, kv = (int64_t)KVH * D;
    const float scale = 1.0f / sqrtf((float)D);
    const float eps = c->rms_eps, theta = c->rope_theta > 0 ? c->rope_theta : 10000.0f;
    const int num_valid = total_tokens - batch;                         /* src/train_cuda.c:1989-1991 */
    if (num_valid <= 0) return 0.0f;
    seraph_stream_t s = t->stream;
    const float* P = t->P;

    seraph_hip_event_on_next_op(NULL);      /* an event this thread armed before the step belongs to none of its ops */
    if (upload_batch(t, tokens, total_tokens, seq_starts, batch)) return -1.0f;
    const uint32_t* starts = t->d_starts;

    /* flag indices, src/train.c:4499-4537 */
    const uint32_t nan_fwd = 10u, nan_bwd = nan_fwd + (uint32_t)NL, nan_gh = nan_bwd + 5u * (uint32_t)NL,
                   nan_opt = nan_gh + (uint32_t)NL;
    if (t->nan_check) {
        CK(seraph_fill_u32(t->d_nan_flags, 0, t->nan_flag_count, s));
        t->nan_detected = 0;
        NANCHK(P + t->off_embed, V * h, nan_opt + 0u);                       /* src/train.c:4548-4554 */
    }

    if (mode == STEP_TRAIN && t->accumulation_counter == 0) {            /* src/train.c:4399-4400 */
        if (lora) OP("fill", 0.0, 4.0 * (double)t->nlora, seraph_fill_u32(t->LG, 0, (size_t)t->nlora, s));
        else OP("fill", 0.0, 4.0 * (double)t->nparams, seraph_fill_u32(t->G, 0, (size_t)t->nparams, s));
    }
    CK(seraph_hip_event_record(t->ev[0], s));

    /* ---------------- forward */
    OP("embed_lookup", 0.0, 8.0 * (double)(T * h), seraph_embed_lookup(t->d_tokens, P + t->off_embed, t->act[0].layer_in, T, h, V, s));
    NANCHK(t->act[0].layer_in, T * h, 7u);
    for (int l = 0; l < NL; l++) {
        const float* W = P + t->off_layer0 + t->L.stride * l;
        const float* LW = lora ? t->LP + t->LL.stride * l : NULL;
        layer_act_t* a = &t->act[l];
        float* next = (l + 1 < NL) ? t->act[l + 1].layer_in : t->final_in;
        /* the input norm of every layer but the first comes out of the add that ended the previous layer */
        if (l == 0) OP("rmsnorm", 0.0, 8.0 * (double)(T * h), seraph_rmsnorm(a->layer_in, W + t->L.in_norm, a->xn_attn, T, h, eps, s));
        {   /* the three projections of the same input (src/train.c:4676-4681) as one launch */
            const seraph_gemm_problem_t qkv[3] = {{a->xn_attn, W + t->L.q, a->q, T, qd}, {a->xn_attn, W + t->L.k, a->k, T, kv},
                                                  {a->xn_attn, W + t->L.v, a->v, T, kv}};
            GEMM_GROUP(qkv, 3, h, 0, 1, 0);
        }
        if (lora) {                                                        /* the q, k and v adapters in one launch per product */
            float* outs[3] = {a->q, a->k, a->v};
            const int64_t od[3] = {qd, kv, kv};
            lora_fwd_item_t it[3];
            int n = 0;
            for (int p = 0; p < 3; p++)
                if (t->LL.A[p] >= 0) it[n++] = (lora_fwd_item_t){a->xn_attn, outs[p], LW + t->LL.A[p], LW + t->LL.B[p], h, od[p], a->xa[p]};
            if (lora_forward_group(t, it, n, T)) return -1.0f;
        }
        OP("rope", 0.0, 8.0 * (double)(T * (qd + kv)), seraph_rope_qk(a->q, a->q, H, a->k, a->k, KVH, starts, batch, T, D, theta, 0, s));
        if (c->use_qk_norm) {                                              /* after RoPE, before the attention: src/train.c:4687-4689 */
            OP("qk_norm", 0.0, 8.0 * (double)(T * qd), seraph_qk_norm_saved(a->q, a->rms_q, T, H, D, eps, s));
            OP("qk_norm", 0.0, 8.0 * (double)(T * kv), seraph_qk_norm_saved(a->k, a->rms_k, T, KVH, D, eps, s));
        }
        OP("attention_forward", 4.0 * D * t->attn_pairs * H, 0.0, seraph_attention_forward(a->q, a->k, a->v, a->attn_out, a->lse, starts, batch, T, H, KVH, D, scale, s));
        GEMM(a->attn_out, W + t->L.o, t->tmp_h, T, h, qd, 0, 1, 0);
        if (lora && t->LL.A[3] >= 0 && lora_forward_add(t, a->attn_out, t->tmp_h, LW + t->LL.A[3], LW + t->LL.B[3], T, qd, h, a->xa[3])) return -1.0f;
        OP("add_rmsnorm", 0.0, 16.0 * (double)(T * h), seraph_add_rmsnorm(a->layer_in, t->tmp_h, a->post_in, W + t->L.post_norm, a->xn_ffn, T, h, eps, s));
        {   /* gate and up projections (src/train.c:4718-4725) as one launch */
            const seraph_gemm_problem_t gu[2] = {{a->xn_ffn, W + t->L.gate, a->gate, T, f}, {a->xn_ffn, W + t->L.up, a->up, T, f}};
            GEMM_GROUP(gu, 2, h, 0, 1, 0);
        }
        if (lora) {
            float* outs[2] = {a->gate, a->up};
            lora_fwd_item_t it[2];
            int n = 0;
            for (int p = 4; p < 6; p++)
                if (t->LL.A[p] >= 0) it[n++] = (lora_fwd_item_t){a->xn_ffn, outs[p - 4], LW + t->LL.A[p], LW + t->LL.B[p], h, f, a->xa[p]};
            if (lora_forward_group(t, it, n, T)) return -1.0f;
        }
        OP("swiglu", 0.0, 12.0 * (double)(T * f), seraph_swiglu(a->gate, a->up, a->ffn_h, (size_t)(T * f), s));
        GEMM(a->ffn_h, W + t->L.down, t->tmp_h, T, h, f, 0, 1, 0);
        if (lora && t->LL.A[6] >= 0 && lora_forward_add(t, a->ffn_h, t->tmp_h, LW + t->LL.A[6], LW + t->LL.B[6], T, f, h, a->xa[6])) return -1.0f;
        /* residual add and the norm that reads its result: the next layer's input norm, or the final norm */
        const float* next_gain = (l + 1 < NL) ? P + t->off_layer0 + t->L.stride * (l + 1) + t->L.in_norm : P + t->off_final_norm;
        float* next_xn = (l + 1 < NL) ? t->act[l + 1].xn_attn : t->xn_final;
        OP("add_rmsnorm", 0.0, 16.0 * (double)(T * h), seraph_add_rmsnorm(a->post_in, t->tmp_h, next, next_gain, next_xn, T, h, eps, s));
        NANCHK(next, T * h, nan_fwd + (uint32_t)l);
    }
    if (NL == 0) OP("rmsnorm", 0.0, 8.0 * (double)(T * h), seraph_rmsnorm(t->final_in, P + t->off_final_norm, t->xn_final, T, h, eps, s));
    NANCHK(t->xn_final, T * h, 2u);
    NANCHK(t->final_in, T * h, 6u);
    GEMM(t->xn_final, P + t->off_embed, t->logits, T, V, h, 0, 1, 0);      /* tied head, src/train.c:4869-4872 */
    NANCHK(t->logits, T * V, 1u);

    /* ---------------- loss: gradient written over the logits */
    OP("cross_entropy_grad", 0.0, 8.0 * (double)T * (double)V + 8.0 * (double)T, seraph_cross_entropy_grad(t->logits, t->d_targets, t->logits, t->loss_rows, starts, batch, T, V, num_valid, s));
    float* red_in = t->loss_rows;
    float* red_out = t->red_a;
    for (size_t n = (size_t)T; n > 1; n = (n + 511) / 512) {                              /* src/train.c:4902-4913 */
        CK(seraph_reduce_sum(red_in, red_out, n, s));
        red_in = red_out;
        red_out = (red_out == t->red_a) ? t->red_b : t->red_a;
    }
    CK(seraph_hip_event_record(t->ev[1], s));
    if (mode == STEP_EVAL) {                                               /* src/train_cuda.c:2792-2809 */
        float eval_sum = 0.0f;
        CK(seraph_hip_d2h(&eval_sum, red_in, sizeof(float), s));
        op_fold(t);
        return eval_sum / (float)num_valid;
    }

    /* ---------------- backward */
    float* glog = t->logits;
    NANCHK(glog, T * V, 3u);
    /* Weight gradients leave the chain: each one starts on the second stream once its two operands are complete
     * (fork), and the first stream waits for it (join) only where it is about to overwrite one of them: g_hidden at
     * the next norm backward, g_gate / g_up and g_q / g_k / g_v in the next layer down. With per-op timing or the NaN
     * lattice on, everything stays on one stream. */
    const int ov = t->overlap && t->stream2 && !t->op_timing && !t->nan_check;
    seraph_stream_t sw = ov ? t->stream2 : s;
    void* w2 = ov ? t->ws2 : t->ws;
    const size_t w2b = ov ? t->ws2_bytes : t->ws_bytes;
    enum { MK_DOWN = 1, MK_GU = 2, MK_O = 3, MK_QKV = 4, MK_END = 5 };
    int fork_armed = 0;
    SIDE_FORK();
    if (!lora) WGEMM(glog, t->xn_final, t->G + t->off_embed, V, h, T);      /* LM head wgrad */
    GEMM(glog, P + t->off_embed, t->g_hidden, T, h, V, 0, 0, 0);            /* LM head dgrad */
    NANCHK(t->g_hidden, T * h, 4u);
    SIDE_ARM();
    t->norm_job_count = 0;
    NORM_BWD(t->final_in, P + t->off_final_norm, t->g_hidden, NULL, t->g_tmp, t->G + t->off_final_norm, 12.0 * (double)(T * h));
    NANCHK(t->g_tmp, T * h, 5u);
    { float* sw = t->g_hidden; t->g_hidden = t->g_tmp; t->g_tmp = sw; }                   /* grad_hidden = grad_tmp (copy, src/train.c:5089) */
    NANCHK(t->g_hidden, T * h, 0u);

    for (int l = NL - 1; l >= 0; l--) {
        const float* W = P + t->off_layer0 + t->L.stride * l;
        float* GW = lora ? NULL : t->G + t->off_layer0 + t->L.stride * l;
        const float* LW = lora ? t->LP + t->LL.stride * l : NULL;
        float* LGW = lora ? t->LG + t->LL.stride * l : NULL;
        layer_act_t* a = &t->act[l];

        /* FFN */
        /* what leaves the chain at each fork: the weight gradient of the projection, or (LoRA) its adapter's gradients */
        SIDE_FORK();
        if (!lora) WGEMM(t->g_hidden, a->ffn_h, GW + t->L.down, h, f, T);
        else if (ov && t->LL.A[6] >= 0 &&                                    /* src/train.c:6422-6429 */
                 lora_backward(t, t->g_hidden, a->ffn_h, a->xa[6], LW + t->LL.B[6], LGW + t->LL.A[6], LGW + t->LL.B[6], T, f, h, ov)) return -1.0f;
        SIDE_MARK(MK_DOWN);
        GEMM(t->g_hidden, W + t->L.down, t->g_ffn, T, f, h, 0, 0, 0);
        SIDE_JOIN(MK_GU);                                                    /* the layer above still reads g_gate / g_up */
        SIDE_ARM();
        OP("swiglu_backward", 0.0, 20.0 * (double)(T * f), seraph_swiglu_backward(a->gate, a->up, t->g_ffn, t->g_gate, t->g_up, (size_t)(T * f), s));
        SIDE_FORK();
        if (!lora) {
            const seraph_gemm_problem_t gu[2] = {{t->g_gate, a->xn_ffn, GW + t->L.gate, f, h}, {t->g_up, a->xn_ffn, GW + t->L.up, f, h}};
            WGEMM_GROUP(gu, 2, T);
        } else if (ov) {                                                     /* src/train.c:6446-6461 */
            if (t->LL.A[4] >= 0 &&
                lora_backward(t, t->g_gate, a->xn_ffn, a->xa[4], LW + t->LL.B[4], LGW + t->LL.A[4], LGW + t->LL.B[4], T, h, f, ov)) return -1.0f;
            if (t->LL.A[5] >= 0 &&
                lora_backward(t, t->g_up, a->xn_ffn, a->xa[5], LW + t->LL.B[5], LGW + t->LL.A[5], LGW + t->LL.B[5], T, h, f, ov)) return -1.0f;
        } else {
            /* gate, up and the down adapter left over from above (g_hidden is not rewritten before the norm backward
             * below, ffn_h stays): one launch per kind of product */
            const float* dYs[3] = {t->g_gate, t->g_up, t->g_hidden};
            const float* xs[3] = {a->xn_ffn, a->xn_ffn, a->ffn_h};
            const int64_t ind[3] = {h, h, f}, od[3] = {f, f, h};
            lora_bwd_item_t it[3];
            int n = 0;
            for (int p = 4; p < 7; p++)
                if (t->LL.A[p] >= 0)
                    it[n++] = (lora_bwd_item_t){dYs[p - 4], xs[p - 4], a->xa[p], LW + t->LL.B[p], LGW + t->LL.A[p], LGW + t->LL.B[p], ind[p - 4], od[p - 4]};
            if (lora_backward_group(t, it, n, T)) return -1.0f;
        }
        SIDE_MARK(MK_GU);
        {   /* grad_x_norm_ffn = grad_gate Wgate + grad_up Wup (src/train.c:5162-5179) */
            const seraph_gemm_term_t gu[2] = {{t->g_gate, W + t->L.gate, f}, {t->g_up, W + t->L.up, f}};
            GEMM_CHAIN(gu, 2, t->g_xn, T, h);
        }
        SIDE_JOIN(MK_DOWN);                                                  /* g_hidden is rewritten next */
        /* the input gradient is added to the residual stream's gradient as it is stored (src/train.c:5180-5193) */
        SIDE_ARM();
        NORM_BWD(a->post_in, W + t->L.post_norm, t->g_xn, t->g_hidden, t->g_hidden, GW + t->L.post_norm, 16.0 * (double)(T * h));

        /* attention */
        SIDE_FORK();
        if (!lora) WGEMM(t->g_hidden, a->attn_out, GW + t->L.o, h, qd, T);
        else if (ov && t->LL.A[3] >= 0 &&
                 lora_backward(t, t->g_hidden, a->attn_out, a->xa[3], LW + t->LL.B[3], LGW + t->LL.A[3], LGW + t->LL.B[3], T, qd, h, ov)) return -1.0f;
        SIDE_MARK(MK_O);
        GEMM(t->g_hidden, W + t->L.o, t->g_attn, T, qd, h, 0, 0, 0);
        NANCHK(t->g_attn, T * qd, nan_bwd + 5u * (uint32_t)l + 0u);
        SIDE_JOIN(MK_QKV);                                                   /* the layer above still reads g_q / g_k / g_v */
        /* dK / dV are assigned, so the zero fills of src/train.c:5221-5222 have nothing left to do; the host's copy
         * of the offsets sizes the dS band */
        OP("attention_backward", 10.0 * D * t->attn_pairs * H, 0.0, seraph_attention_backward_assign(a->q, a->k, a->v, t->g_attn, a->attn_out, a->lse, t->g_q, t->g_k, t->g_v,
                                     starts, t->h_stage + 2 * (size_t)T, batch, T, H, KVH, D, scale, t->attn_ws, t->attn_ws_bytes, s));
        NANCHK(t->g_q, T * qd, nan_bwd + 5u * (uint32_t)l + 1u);
        NANCHK(t->g_k, T * kv, nan_bwd + 5u * (uint32_t)l + 2u);
        NANCHK(t->g_v, T * kv, nan_bwd + 5u * (uint32_t)l + 3u);
        if (c->use_qk_norm) {                                              /* from the kept outputs and the saved rms, in place */
            OP("qk_norm_backward", 0.0, 12.0 * (double)(T * qd), seraph_qk_norm_backward_saved(a->q, a->rms_q, t->g_q, t->g_q, T, H, D, eps, s));
            OP("qk_norm_backward", 0.0, 12.0 * (double)(T * kv), seraph_qk_norm_backward_saved(a->k, a->rms_k, t->g_k, t->g_k, T, KVH, D, eps, s));
        }
        SIDE_ARM();
        OP("rope", 0.0, 8.0 * (double)(T * (qd + kv)), seraph_rope_qk(t->g_q, t->g_q, H, t->g_k, t->g_k, KVH, starts, batch, T, D, theta, 1, s));
        NANCHK(t->g_q, T * qd, nan_bwd + 5u * (uint32_t)l + 4u);
        SIDE_FORK();
        if (!lora) {
            const seraph_gemm_problem_t qkv[3] = {{t->g_q, a->xn_attn, GW + t->L.q, qd, h}, {t->g_k, a->xn_attn, GW + t->L.k, kv, h},
                                                  {t->g_v, a->xn_attn, GW + t->L.v, kv, h}};
            WGEMM_GROUP(qkv, 3, T);
        } else if (ov) {
            float* gs[3] = {t->g_q, t->g_k, t->g_v};
            int64_t outs[3] = {qd, kv, kv};
            for (int p = 0; p < 3; p++)
                if (t->LL.A[p] >= 0 &&
                    lora_backward(t, gs[p], a->xn_attn, a->xa[p], LW + t->LL.B[p], LGW + t->LL.A[p], LGW + t->LL.B[p], T, h, outs[p], ov)) return -1.0f;
        } else {
            /* q, k, v and the o adapter left over from above (g_hidden and attn_out are still what they were there) */
            const float* dYs[4] = {t->g_q, t->g_k, t->g_v, t->g_hidden};
            const float* xs[4] = {a->xn_attn, a->xn_attn, a->xn_attn, a->attn_out};
            const int64_t ind[4] = {h, h, h, qd}, od[4] = {qd, kv, kv, h};
            lora_bwd_item_t it[4];
            int n = 0;
            for (int p = 0; p < 4; p++)
                if (t->LL.A[p] >= 0)
                    it[n++] = (lora_bwd_item_t){dYs[p], xs[p], a->xa[p], LW + t->LL.B[p], LGW + t->LL.A[p], LGW + t->LL.B[p], ind[p], od[p]};
            if (lora_backward_group(t, it, n, T)) return -1.0f;
        }
        SIDE_MARK(MK_QKV);
        {   /* grad_x_norm = grad_q Wq + grad_k Wk + grad_v Wv (src/train.c:5294-5339) */
            const seraph_gemm_term_t qkv[3] = {{t->g_q, W + t->L.q, qd}, {t->g_k, W + t->L.k, kv}, {t->g_v, W + t->L.v, kv}};
            GEMM_CHAIN(qkv, 3, t->g_xn, T, h);
        }
        SIDE_JOIN(MK_O);                                                     /* g_hidden is rewritten next */
        if (l > 0) SIDE_ARM();
        NORM_BWD(a->layer_in, W + t->L.in_norm, t->g_xn, t->g_hidden, t->g_hidden, GW + t->L.in_norm, 16.0 * (double)(T * h));   /* src/train.c:5342-5355 */
        NANCHK(t->g_hidden, T * h, nan_gh + (uint32_t)l);
    }
    NANCHK(t->g_hidden, T * h, 8u);
    if (t->norm_job_count > 0) {
        OP("rmsnorm_colsum", 0.0, 0.0, seraph_rmsnorm_colsum_multi(t->norm_jobs, t->norm_job_count, h, s));
        t->norm_job_count = 0;
    }
    SIDE_MARK(MK_END);
    SIDE_JOIN(MK_END);                                                       /* every weight gradient is complete from here on */
    if (!lora) OP("embedding_backward", 0.0, 12.0 * (double)(T * h), seraph_embedding_backward(t->d_tokens, t->g_hidden, t->G + t->off_embed, T, h, V, t->ws, t->ws_bytes, s));
    if (!lora) NANCHK(t->G + t->off_embed, V * h, 9u);
    CK(seraph_hip_event_record(t->ev[2], s));

    /* ---------------- optimizer (src/train.c:5439-5463, LoRA :6617-6640) */
    t->accumulation_counter++;
    int accum = t->opt.gradient_accumulation_steps < 1 ? 1 : t->opt.gradient_accumulation_steps;
    if (t->accumulation_counter >= accum) {
        if (run_optimizer) {
            t->optimizer_step++;
            float lr = t->opt.learning_rate;
            float warm = (float)t->opt.warmup_steps;
            if ((float)t->optimizer_step < warm) lr = t->opt.learning_rate * ((float)t->optimizer_step / warm);
            lr = lr / (float)accum;
            t->last_lr = lr;
            if (t->nan_check) {
                /* the optimizer waits for the flags so that a NaN cannot reach the weights
                 * (src/train.c:5446-5448, :5472-5660); then grad/m/v of the embedding are checked
                 * before AdamW and the embedding after it (:5662-5720) */
                int any = nan_flags_any(t);
                if (any) {
                    t->nan_detected = 1;
                    if (any > 0) nan_dump(t, total_tokens);
                    t->step_counter++;
                    op_fold(t);
                    return any < 0 ? -1.0f : NAN;
                }
                if (!lora) {
                    NANCHK(t->G + t->off_embed, V * h, nan_opt + 1u);
                    NANCHK(t->M + t->off_embed, V * h, nan_opt + 2u);
                    NANCHK(t->V + t->off_embed, V * h, nan_opt + 3u);
                }
            }
            if (lora) OP("adamw", 0.0, 28.0 * (double)t->nlora, seraph_adamw(t->LP, t->LG, t->LM, t->LV, (size_t)t->nlora, lr, t->opt.beta1, t->opt.beta2,
                                      t->opt.weight_decay, t->opt.eps, t->optimizer_step, t->opt.clip, s));
            else OP("adamw", 0.0, 28.0 * (double)t->nparams, seraph_adamw(t->P, t->G, t->M, t->V, (size_t)t->nparams, lr, t->opt.beta1, t->opt.beta2,
                                 t->opt.weight_decay, t->opt.eps, t->optimizer_step, t->opt.clip, s));
            if (t->nan_check && !lora) NANCHK(t->P + t->off_embed, V * h, nan_opt + 4u);
        }
        t->accumulation_counter = 0;
    }
    CK(seraph_hip_event_record(t->ev[3], s));
    if (t->nan_check) {
        int any = nan_flags_any(t);
        if (any) {
            t->nan_detected = 1;
            if (any > 0) nan_dump(t, total_tokens);
            t->step_counter++;
            op_fold(t);
            return any < 0 ? -1.0f : NAN;
        }
    }
    t->step_counter++;

    float loss_sum = 0.0f;
    CK(seraph_hip_d2h(&loss_sum, red_in, sizeof(float), s));               /* waits for the whole step */
    for (int i = 0; i < 3; i++) seraph_hip_event_elapsed_ms(t->ev[i], t->ev[i + 1], &t->phase_ms[i]);
    op_fold(t);
    return loss_sum / (float)num_valid;
}

float hip_train_step_full_batch(hip_trainer_t* t, const int* tokens_packed, int total_tokens,
                                const int* seq_starts, int batch_size, int run_optimizer) {
    if (!t || t->lora) { fprintf(stderr, "ERROR: trainer is not in full-weight mode\n"); return -1.0f; }
    return run_step(t, tokens_packed, total_tokens, seq_starts, batch_size, run_optimizer, STEP_TRAIN);
}

float hip_train_step_lora_batch(hip_trainer_t* t, const int* tokens_packed, int total_tokens,
                                const int* seq_starts, int batch_size, int run_optimizer) {
    if (!t || !t->lora) { fprintf(stderr, "ERROR: trainer is not in LoRA mode\n"); return -1.0f; }
    return run_step(t, tokens_packed, total_tokens, seq_starts, batch_size, run_optimizer, STEP_TRAIN);
}

float hip_eval_forward_batch(hip_trainer_t* t, const int* tokens_packed, int total_tokens,
                             const int* seq_starts, int batch_size) {
    if (!t) return -1.0f;
    return run_step(t, tokens_packed, total_tokens, seq_starts, batch_size, 0, STEP_EVAL);
}

/* src/train_cuda.c:2812-2847 */
float hip_evaluate(hip_trainer_t* t, const int* val_tokens, int num_val_tokens, const int* offsets, int num_samples,
                   int max_seq_len, int max_eval_samples, float* out_perplexity) {
    if (out_perplexity) *out_perplexity = 0.0f;
    if (!t || !val_tokens || !offsets || num_samples <= 0) return -1.0f;
    const int max_eval = max_eval_samples > 0 ? max_eval_samples : num_samples;
    const int stride = num_samples > max_eval ? num_samples / max_eval : 1;
    double total = 0.0;
    int valid = 0;
    for (int i = 0; i < num_samples; i += stride) {
        const int start = offsets[i];
        const int end = (i + 1 < num_samples) ? offsets[i + 1] : num_val_tokens;
        int len = end - start;
        if (len > max_seq_len) len = max_seq_len;
        if (len > t->max_tokens) len = t->max_tokens;
        if (len < 2) continue;
        const float loss = hip_eval_forward_batch(t, val_tokens + start, len, NULL, 1);
        if (loss >= 0.0f && !isnan(loss)) { total += loss; valid++; }
    }
    const float avg = valid > 0 ? (float)(total / valid) : -1.0f;
    if (out_perplexity) *out_perplexity = avg > 0.0f ? expf(avg) : 0.0f;
    return avg;
}

int hip_trainer_enable_nan_check(hip_trainer_t* t, int on) {
    if (!t) return -1;
    if (on && !t->d_nan_flags) {
        t->nan_flag_count = 10u + 7u * (uint32_t)t->cfg.layers + 5u;       /* src/train.c:4525-4537 */
        if (dev_alloc(t, (void**)&t->d_nan_flags, (size_t)t->nan_flag_count * 4)) return -1;
        t->h_nan_flags = (uint32_t*)calloc(t->nan_flag_count, sizeof(uint32_t));
        if (!t->h_nan_flags) return -1;
    }
    t->nan_check = on ? 1 : 0;
    return 0;
}

int hip_trainer_nan_detected(const hip_trainer_t* t) { return t ? t->nan_detected : 0; }

void hip_trainer_set_nan_dump_prefix(hip_trainer_t* t, const char* prefix) {
    if (!t) return;
    snprintf(t->nan_dump_prefix, sizeof(t->nan_dump_prefix), "%s", prefix ? prefix : "");
}

int hip_trainer_nan_flags(const hip_trainer_t* t, uint32_t* out, int max) {
    if (!t || !t->h_nan_flags) return 0;
    int n = (int)t->nan_flag_count < max ? (int)t->nan_flag_count : max;
    if (out) memcpy(out, t->h_nan_flags, (size_t)n * 4);
    return (int)t->nan_flag_count;
}

/* names the first poisoned buffers the way src/train.c:5500-5560 does */
void hip_trainer_nan_report(const hip_trainer_t* t, FILE* out) {
    if (!t || !t->h_nan_flags || !out) return;
    static const char* const global_names[10] = {
        "grad_hidden (after final rmsnorm backward)", "logits", "hidden_norm (input to LM head)", "grad_logits",
        "grad_hidden (after LM head backward)", "grad_tmp_hidden (final rmsnorm backward output)",
        "final_input (input to final rmsnorm)", "hidden (after embedding lookup)",
        "grad_hidden (before embedding_backward)", "g_embed (after embedding_backward)"};
    const uint32_t* fl = t->h_nan_flags;
    const int NL = t->cfg.layers;
    const uint32_t fwd = 10u, bwd = fwd + (uint32_t)NL, gh = bwd + 5u * (uint32_t)NL, opt = gh + (uint32_t)NL;
    for (int i = 0; i < 10; i++) if (fl[i]) fprintf(out, "  - buffer: %s\n", global_names[i]);
    for (int l = 0; l < NL; l++) if (fl[fwd + l]) { fprintf(out, "  - buffer: hidden after layer=%d (first)\n", l); break; }
    if (fl[opt + 0]) fprintf(out, "  - buffer: w_embed (weights already poisoned)\n");
    for (int l = NL - 1; l >= 0; l--) if (fl[gh + l]) { fprintf(out, "  - buffer: grad_hidden after backward of layer=%d (first)\n", l); break; }
    static const char* const bwd_names[5] = {"grad_attn (input to attn backward)", "grad_q (pre rope_backward)",
        "grad_k (post attn backward)", "grad_v (post attn backward)", "grad_q (post rope_backward)"};
    for (int l = NL - 1; l >= 0; l--) {
        int hit = 0;
        for (int k = 0; k < 5 && !hit; k++) if (fl[bwd + 5u * l + k]) { fprintf(out, "  - buffer: %s layer=%d\n", bwd_names[k], l); hit = 1; }
        if (hit) break;
    }
    if (fl[opt + 1]) fprintf(out, "  - buffer: g_embed (pre AdamW)\n");
    if (fl[opt + 2]) fprintf(out, "  - buffer: m_embed (pre AdamW)\n");
    if (fl[opt + 3]) fprintf(out, "  - buffer: v_embed (pre AdamW)\n");
    if (fl[opt + 4]) fprintf(out, "  - buffer: w_embed (post AdamW)\n");
}
