/*
 * ref_step_harness.c - drives Seraph's own, unmodified training step
 * (train_step -> train_step_gpu_full, src/train.c:6808 / :4365) over this
 * repository's HIP backend, and dumps what it produced.
 *
 * TEST INFRASTRUCTURE.  Built only where the Seraph tree is present, by
 * `make -C oracle ref` (sources compiled where they lie, output in oracle/_ref/).
 * It is the integration check of the drop-in boundary: the reference's step driver,
 * its buffer management and its optimizer schedule run as they are; only the 40
 * vulkan_* symbols come from src/hip_backend*.c.  It is NOT an independent oracle
 * for the ops (those are this build's kernels); it cross-checks the op ORDER of the
 * oracle's step against the reference's own driver.
 *
 * usage: ref_step_hip [--cpu] [--time] [--profile] <in.bin> <out.bin>
 *   --profile : the backend's vulkan_profiler_* is switched on around every step (nothing in the reference calls it;
 *            it is the interface of include/vulkan_backend.h:638-642) and prints its report to stdout
 *   --cpu  : no backend is created, so train_step takes the reference's CPU path (src/train.c:6842-6983:
 *            train_forward_fp32, the scalar loss loops, train_backward, the CPU AdamW); full-weight mode only.
 *            This is the timed "reference" CPU baseline; its gradients are NOT those of the GPU path
 *            (the CPU backward is an approximation) and nothing is compared with them.
 *   --time : prints "seconds_per_step <mean over all steps but the first>" (all steps when there is only one)
 *   in : int32 hidden, layers, heads, kv_heads, head_dim, ffn, vocab, steps, T, lora_rank, lora_mask
 *        float32 lr, rope_theta, lora_alpha
 *        float32 params[...] in this build's arena order
 *        float32 lora[...]   (lora_rank > 0) per layer, per selected adapter q k v o gate up down: A[r,in], B[out,r]
 *        int32 tokens[steps * T]
 *   out (full): float32 loss[steps], grads[...] (last step), weights[...] (after last step)
 *   out (LoRA): float32 loss[steps], lora weights[...], adam m[...], adam v[...]  (after last step; pulled
 *               back through the reference's own save_checkpoint -> lora_gpu_download_to_cpu, src/train.c:7760-7767)
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "model_config.h"
#include "lora.h"
#include "train.h"
#include "vulkan_backend.h"

static int rd(void* p, size_t n, FILE* f) { return fread(p, 1, n, f) == n ? 0 : -1; }

typedef struct { weight_tensor_t* t; vulkan_buffer_t* w; vulkan_buffer_t* g; } slot_t;

static double now_s(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

int main(int argc, char** argv) {
    int cpu_only = 0, timed = 0, profile = 0;
    while (argc > 1 && argv[1][0] == '-' && argv[1][1] == '-') {
        if (!strcmp(argv[1], "--cpu")) cpu_only = 1;
        else if (!strcmp(argv[1], "--time")) timed = 1;
        else if (!strcmp(argv[1], "--profile")) profile = 1;
        else { fprintf(stderr, "unknown option %s\n", argv[1]); return 2; }
        argv++; argc--;
    }
    if (argc != 3) { fprintf(stderr, "usage: %s [--cpu] [--time] in.bin out.bin\n", argv[0]); return 2; }
    FILE* f = fopen(argv[1], "rb");
    if (!f) { perror("in.bin"); return 2; }
    int hdr[11]; float fl[3];
    if (rd(hdr, sizeof(hdr), f) || rd(fl, sizeof(fl), f)) return 2;
    const int hidden = hdr[0], layers = hdr[1], heads = hdr[2], kvh = hdr[3], hd = hdr[4], ffn = hdr[5], vocab = hdr[6];
    const int steps = hdr[7], T = hdr[8], rank = hdr[9], mask = hdr[10];

    model_config_t cfg;
    memset(&cfg, 0, sizeof(cfg));
    cfg.vocab_size = vocab; cfg.hidden_size = hidden; cfg.num_hidden_layers = layers; cfg.intermediate_size = ffn;
    cfg.num_attention_heads = heads; cfg.num_key_value_heads = kvh; cfg.head_dim = hd; cfg.kv_dim = kvh * hd;
    cfg.rms_norm_eps = 1e-6f; cfg.rope_theta = fl[1]; cfg.max_position_embeddings = 4096; cfg.tie_word_embeddings = 1;

    train_state_t st;
    memset(&st, 0, sizeof(st));
    st.config = &cfg;
    st.use_full_training = rank == 0;
    trainable_weights_t* w = trainable_weights_alloc(&cfg);   /* in LoRA mode only a host staging area */
    if (rank == 0) st.full_weights = w;
    st.learning_rate = fl[0];
    st.gradient_accumulation_steps = 1;
    if (!w) return 3;

    /* this build's arena order: embed, final_norm, per layer in_norm q k v o post_norm gate up down */
    int nslots = 2 + 9 * layers, k = 0;
    slot_t* slots = calloc((size_t)nslots, sizeof(slot_t));
    slots[k++].t = &w->embed_tokens; slots[k++].t = &w->final_norm;
    for (int l = 0; l < layers; l++) {
        layer_weights_t* L = &w->layers[l];
        weight_tensor_t* order[9] = {&L->input_norm, &L->q_proj, &L->k_proj, &L->v_proj, &L->o_proj,
                                     &L->post_norm, &L->gate_proj, &L->up_proj, &L->down_proj};
        for (int i = 0; i < 9; i++) slots[k++].t = order[i];
    }
    size_t total = 0;
    for (int i = 0; i < nslots; i++) {
        if (rd(slots[i].t->weight, slots[i].t->size * sizeof(float), f)) { fprintf(stderr, "short params\n"); return 2; }
        total += slots[i].t->size;
    }
    /* LoRA adapters (src/lora.c:342-397 creates q and v; the others are added the same way) */
    lora_adapter_t*** kinds[7];
    size_t nlora = 0;
    if (rank > 0) {
        lora_model_t* lm = lora_model_create_from_config(&cfg, rank, fl[2]);
        const int qd = heads * hd, kvd = kvh * hd;
        const int ins[7] = {hidden, hidden, hidden, qd, hidden, hidden, ffn};
        const int outs[7] = {qd, kvd, kvd, hidden, ffn, ffn, hidden};
        kinds[0] = &lm->q_adapters; kinds[1] = &lm->k_adapters; kinds[2] = &lm->v_adapters; kinds[3] = &lm->o_adapters;
        kinds[4] = &lm->gate_adapters; kinds[5] = &lm->up_adapters; kinds[6] = &lm->down_adapters;
        lm->apply_to_q = mask & 1; lm->apply_to_k = (mask >> 1) & 1; lm->apply_to_v = (mask >> 2) & 1;
        lm->apply_to_o = (mask >> 3) & 1; lm->apply_to_ffn = (mask >> 4) != 0;
        for (int l = 0; l < layers; l++)
            for (int p = 0; p < 7; p++) {
                lora_adapter_t** slot = &(*kinds[p])[l];
                if (!((mask >> p) & 1)) { if (*slot) { lora_adapter_free(*slot); *slot = NULL; } continue; }
                if (!*slot) *slot = lora_adapter_create(ins[p], outs[p], rank, fl[2]);
                size_t na = (size_t)rank * ins[p], nb = (size_t)outs[p] * rank;
                if (rd((*slot)->A, na * sizeof(float), f) || rd((*slot)->B, nb * sizeof(float), f)) { fprintf(stderr, "short lora\n"); return 2; }
                nlora += na + nb;
            }
        st.lora = lm;
    }
    int* tokens = malloc((size_t)steps * T * sizeof(int));
    if (rd(tokens, (size_t)steps * T * sizeof(int), f)) { fprintf(stderr, "short tokens\n"); return 2; }
    fclose(f);

    if (cpu_only) {
        if (rank > 0) { fprintf(stderr, "--cpu: full-weight mode only\n"); return 2; }
        /* what train_init leaves behind for the CPU path (src/train.c:7927-7934); vulkan_ctx stays NULL */
        st.act_cache = activation_cache_alloc(layers, hidden, ffn, heads * hd, kvh * hd, T);
        float* closs = malloc((size_t)steps * sizeof(float));
        double t_first = 0.0, t_rest = 0.0;
        for (int s = 0; s < steps; s++) {
            const double t0 = now_s();
            closs[s] = train_step(&st, tokens + (size_t)s * T, T);
            const double dt = now_s() - t0;
            if (s == 0) t_first = dt; else t_rest += dt;
        }
        printf("ref_step_hip: CPU path, %d steps of %d tokens, %zu parameters, optimizer_step=%d, last loss %.6f\n",
               steps, T, total, st.optimizer_step, closs[steps - 1]);
        if (timed) printf("seconds_per_step %.6f\n", steps > 1 ? t_rest / (steps - 1) : t_first);
        FILE* o = fopen(argv[2], "wb");
        if (o) { fwrite(closs, sizeof(float), (size_t)steps, o); fclose(o); }
        return 0;
    }
    vulkan_context_t* ctx = vulkan_init_ex(0, -1);
    if (!ctx) { fprintf(stderr, "backend init failed\n"); return 4; }
    st.vulkan_ctx = ctx;
    /* what train_init does after vulkan_init_ex (src/train.c:7996-8019, :8073-8076) */
    size_t max_size = 0;
    for (int i = 0; i < nslots; i++) if (slots[i].t->size > max_size) max_size = slots[i].t->size;
    st.max_tensor_size = max_size * sizeof(float);
    ctx->max_buffer_size = st.max_tensor_size;
    ctx->max_fwd_buffer_size = st.max_tensor_size;

    if (rank > 0) {
        /* frozen base weights: what ensure_lora_gpu_base_weights (src/train.c:2039-2151) leaves in the context,
         * minus the BF16 checkpoint it reads them from -- FP32 values go up as they are */
        ctx->gpu_weights_num_layers = layers; ctx->gpu_weights_hidden_size = hidden;
        ctx->gpu_weights_intermediate_size = ffn; ctx->gpu_weights_vocab_size = vocab;
        ctx->gpu_weights_q_dim = heads * hd; ctx->gpu_weights_kv_dim = kvh * hd;
        void*** arrs[9] = {(void***)&ctx->gpu_w_in_norm, (void***)&ctx->gpu_w_q, (void***)&ctx->gpu_w_k, (void***)&ctx->gpu_w_v,
                           (void***)&ctx->gpu_w_o, (void***)&ctx->gpu_w_post_norm, (void***)&ctx->gpu_w_gate,
                           (void***)&ctx->gpu_w_up, (void***)&ctx->gpu_w_down};
        for (int i = 0; i < 9; i++) *arrs[i] = calloc((size_t)layers, sizeof(void*));
        for (int i = 0; i < nslots; i++) {
            vulkan_buffer_t* b = vulkan_buffer_create(ctx, slots[i].t->size * sizeof(float));
            vulkan_buffer_upload(ctx, b, slots[i].t->weight, slots[i].t->size);
            if (i == 0) ctx->gpu_w_embed = b;
            else if (i == 1) ctx->gpu_w_final_norm = b;
            else (*arrs[(i - 2) % 9])[(i - 2) / 9] = b;
        }
    }

    float* loss = malloc((size_t)steps * sizeof(float));
    double t_first = 0.0, t_rest = 0.0;
    if (profile) vulkan_profiler_enable(ctx);
    for (int s = 0; s < steps; s++) {                    /* train_step returns after its submit-and-wait and loss download */
        if (profile) vulkan_profiler_begin_step(ctx);
        const double t0 = now_s();
        loss[s] = train_step(&st, tokens + (size_t)s * T, T);
        const double dt = now_s() - t0;
        if (s == 0) t_first = dt; else t_rest += dt;
        if (profile) vulkan_profiler_end_step(ctx, s + 1, T, loss[s]);
    }
    if (timed) printf("seconds_per_step %.6f\n", steps > 1 ? t_rest / (steps - 1) : t_first);

    if (rank > 0) {
        if (save_checkpoint(&st, argv[2]) != 0) return 5;      /* pulls A, B, m, v back into st.lora */
        FILE* o = fopen(argv[2], "wb");
        if (!o) { perror("out.bin"); return 2; }
        fwrite(loss, sizeof(float), (size_t)steps, o);
        for (int pass = 0; pass < 3; pass++)
            for (int l = 0; l < layers; l++)
                for (int p = 0; p < 7; p++) {
                    lora_adapter_t* a = (*kinds[p])[l];
                    if (!a) continue;
                    size_t na = (size_t)a->rank * a->in_dim, nb = (size_t)a->out_dim * a->rank;
                    fwrite(pass == 0 ? a->A : pass == 1 ? a->m_A : a->v_A, sizeof(float), na, o);
                    fwrite(pass == 0 ? a->B : pass == 1 ? a->m_B : a->v_B, sizeof(float), nb, o);
                }
        fclose(o);
        printf("ref_step_hip: LoRA %d steps of %d tokens, %zu adapter parameters, optimizer_step=%d, last loss %.6f\n",
               steps, T, nlora, st.optimizer_step, loss[steps - 1]);
        return 0;
    }

    /* device buffers the reference step keeps in its context (include/vulkan_backend.h:258-311) */
    k = 0;
    slots[k].w = ctx->gpu_w_embed; slots[k++].g = ctx->gpu_g_embed;
    slots[k].w = ctx->gpu_w_final_norm; slots[k++].g = ctx->gpu_g_final_norm;
    for (int l = 0; l < layers; l++) {
        void* ws[9] = {ctx->gpu_w_in_norm, ctx->gpu_w_q, ctx->gpu_w_k, ctx->gpu_w_v, ctx->gpu_w_o, ctx->gpu_w_post_norm,
                       ctx->gpu_w_gate, ctx->gpu_w_up, ctx->gpu_w_down};
        void* gs[9] = {ctx->gpu_g_in_norm, ctx->gpu_g_q, ctx->gpu_g_k, ctx->gpu_g_v, ctx->gpu_g_o, ctx->gpu_g_post_norm,
                       ctx->gpu_g_gate, ctx->gpu_g_up, ctx->gpu_g_down};
        for (int i = 0; i < 9; i++) { slots[k].w = ((vulkan_buffer_t**)ws[i])[l]; slots[k++].g = ((vulkan_buffer_t**)gs[i])[l]; }
    }
    FILE* o = fopen(argv[2], "wb");
    if (!o) { perror("out.bin"); return 2; }
    fwrite(loss, sizeof(float), (size_t)steps, o);
    float* tmp = malloc(total * sizeof(float));
    for (int pass = 0; pass < 2; pass++) {
        size_t off = 0;
        for (int i = 0; i < nslots; i++) {
            vulkan_buffer_download(ctx, pass == 0 ? slots[i].g : slots[i].w, tmp + off, slots[i].t->size);
            off += slots[i].t->size;
        }
        fwrite(tmp, sizeof(float), total, o);
    }
    fclose(o);
    printf("ref_step_hip: %d steps of %d tokens, %zu parameters, optimizer_step=%d, last loss %.6f\n",
           steps, T, total, st.optimizer_step, loss[steps - 1]);
    return 0;
}
