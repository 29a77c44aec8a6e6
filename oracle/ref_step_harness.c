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
 * usage: ref_step_hip <in.bin> <out.bin>
 *   in : int32 hidden, layers, heads, kv_heads, head_dim, ffn, vocab, steps, T
 *        float32 lr, rope_theta
 *        float32 params[...] in this build's arena order
 *        int32 tokens[steps * T]
 *   out: float32 loss[steps], float32 grads[...] (last step), float32 weights[...] (after last step)
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "model_config.h"
#include "train.h"
#include "vulkan_backend.h"

static int rd(void* p, size_t n, FILE* f) { return fread(p, 1, n, f) == n ? 0 : -1; }

typedef struct { weight_tensor_t* t; vulkan_buffer_t* w; vulkan_buffer_t* g; } slot_t;

int main(int argc, char** argv) {
    if (argc != 3) { fprintf(stderr, "usage: %s in.bin out.bin\n", argv[0]); return 2; }
    FILE* f = fopen(argv[1], "rb");
    if (!f) { perror("in.bin"); return 2; }
    int hdr[9]; float fl[2];
    if (rd(hdr, sizeof(hdr), f) || rd(fl, sizeof(fl), f)) return 2;
    const int hidden = hdr[0], layers = hdr[1], heads = hdr[2], kvh = hdr[3], hd = hdr[4], ffn = hdr[5], vocab = hdr[6];
    const int steps = hdr[7], T = hdr[8];

    model_config_t cfg;
    memset(&cfg, 0, sizeof(cfg));
    cfg.vocab_size = vocab; cfg.hidden_size = hidden; cfg.num_hidden_layers = layers; cfg.intermediate_size = ffn;
    cfg.num_attention_heads = heads; cfg.num_key_value_heads = kvh; cfg.head_dim = hd; cfg.kv_dim = kvh * hd;
    cfg.rms_norm_eps = 1e-6f; cfg.rope_theta = fl[1]; cfg.max_position_embeddings = 4096; cfg.tie_word_embeddings = 1;

    train_state_t st;
    memset(&st, 0, sizeof(st));
    st.config = &cfg;
    st.use_full_training = 1;
    st.full_weights = trainable_weights_alloc(&cfg);
    st.learning_rate = fl[0];
    st.gradient_accumulation_steps = 1;
    if (!st.full_weights) return 3;

    /* this build's arena order: embed, final_norm, per layer in_norm q k v o post_norm gate up down */
    trainable_weights_t* w = st.full_weights;
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
    int* tokens = malloc((size_t)steps * T * sizeof(int));
    if (rd(tokens, (size_t)steps * T * sizeof(int), f)) { fprintf(stderr, "short tokens\n"); return 2; }
    fclose(f);

    vulkan_context_t* ctx = vulkan_init_ex(0, -1);
    if (!ctx) { fprintf(stderr, "backend init failed\n"); return 4; }
    st.vulkan_ctx = ctx;
    /* what train_init does after vulkan_init_ex (src/train.c:7996-8019, :8073-8076) */
    size_t max_size = 0;
    for (int i = 0; i < nslots; i++) if (slots[i].t->size > max_size) max_size = slots[i].t->size;
    st.max_tensor_size = max_size * sizeof(float);
    ctx->max_buffer_size = st.max_tensor_size;
    ctx->max_fwd_buffer_size = st.max_tensor_size;

    float* loss = malloc((size_t)steps * sizeof(float));
    for (int s = 0; s < steps; s++) loss[s] = train_step(&st, tokens + (size_t)s * T, T);

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
