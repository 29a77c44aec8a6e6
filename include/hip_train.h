/*
 * hip_train.h - packed-batch training steps for Seraph-shaped decoder models on one
 * MI355X: forward, loss, backward and AdamW, all device resident.
 *
 * Stands in for cuda_train_step_gpu_full_batch / cuda_train_step_gpu_lora_batch
 * (include/train_cuda.h:41-49): same arguments (a packed token stream plus seq_starts
 * prefix offsets), same return value (mean loss over total_tokens - batch_size
 * predictions), same accumulation / warm-up / optimizer-step bookkeeping as
 * src/train.c:5439-5463.  The mathematics of every op is the Vulkan path's
 * (shaders/ *.comp in the op order of src/train.c:4365-5763 and :5847-6719); the LoRA step
 * follows train_step_gpu_lora, not the approximate CUDA variant.
 *
 * What differs from the reference is layout and fusion only: parameters, gradients and
 * the two Adam moments are four flat arenas (one AdamW launch covers the model),
 * activations are written once where the backward reads them (no cache copies),
 * silu*mul and its backward are single passes, the attention backward reuses the
 * forward's output and log-sum-exp, and sums of weight-side gradients use GEMM
 * accumulation instead of a temporary and an add.
 *
 * Arena layout (floats): embed[V,h], final_norm[h], then per layer
 *   in_norm[h], q[q,h], k[kv,h], v[kv,h], o[h,q], post_norm[h], gate[f,h], up[f,h], down[h,f].
 * LoRA arena: per layer, for each of q,k,v,o,gate,up,down selected by lora_mask (bit 0..6): A[r,in], B[out,r].
 */
#ifndef HIP_TRAIN_H
#define HIP_TRAIN_H

#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int32_t hidden, layers, heads, kv_heads, head_dim, ffn, vocab;
    float   rms_eps;        /* the reference's step hard-codes 1e-5 (src/train.c:4378) */
    float   rope_theta;
    int32_t lora_rank;      /* 0 = full-weight training */
    float   lora_alpha;
    int32_t lora_mask;      /* bit0 q, 1 k, 2 v, 3 o, 4 gate, 5 up, 6 down (src/lora.c:372-396) */
    int32_t use_qk_norm;    /* 0 (the reference's language-model mode, src/model_config.c:282): off.  1: q and k are divided by
                               their root mean square over all heads of a token after RoPE (shaders/qk_norm.comp, called at
                               src/train.c:4688-4689 with the step's eps) and, unlike the reference, whose backward treats the
                               op as the identity, the backward applies its derivative before the RoPE backward */
} hip_model_config_t;

typedef struct {
    float   learning_rate;
    float   beta1, beta2, weight_decay, eps;     /* reference: 0.9, 0.999, 0.01, 1e-8 (src/train.c:5449-5452) */
    float   clip;                                /* per-element gradient clamp; <= 0 = off (the reference) */
    int32_t warmup_steps;                        /* reference: 100 (src/train.c:5456) */
    int32_t gradient_accumulation_steps;
} hip_optim_config_t;

typedef struct hip_trainer hip_trainer_t;

int64_t hip_param_count(const hip_model_config_t* cfg);
int64_t hip_lora_param_count(const hip_model_config_t* cfg);

/* Float offsets of every tensor inside the parameter arena (gradients and moments share them):
 * tensor X of layer l starts at layer0 + l * layer_stride + X. */
typedef struct {
    int64_t embed, final_norm, layer0, layer_stride;
    int64_t in_norm, q, k, v, o, post_norm, gate, up, down;
    int64_t count;
} hip_param_layout_t;
void hip_param_layout(const hip_model_config_t* cfg, hip_param_layout_t* out);

/* Same for the adapter arena; index 0..6 = q k v o gate up down, offset -1 = adapter not selected.
 * A is [rank, in_dim], B is [out_dim, rank] (src/lora.c:54-81). */
typedef struct {
    int64_t A[7], B[7], in_dim[7], out_dim[7];
    int64_t layer_stride, count;
} hip_lora_layout_t;
void hip_lora_layout(const hip_model_config_t* cfg, hip_lora_layout_t* out);

/* ext_* are optional caller-owned DEVICE arenas of hip_param_count floats (NULL: allocated
 * here).  In LoRA mode (cfg->lora_rank > 0) only ext_params is used: the base model is frozen
 * and the adapter arenas are always owned by the trainer.  Returns NULL on failure with the
 * reason on stderr. */
hip_trainer_t* hip_trainer_create(const hip_model_config_t* cfg, const hip_optim_config_t* opt,
                                  int max_tokens, int max_batch, int device_index,
                                  float* ext_params, float* ext_grads, float* ext_m, float* ext_v);
void hip_trainer_free(hip_trainer_t* t);

/* host <-> device transfers of whole arenas; `which`: 0 params, 1 grads, 2 m, 3 v,
 * 4 lora params, 5 lora grads, 6 lora m, 7 lora v.  Return 0 on success. */
int hip_trainer_upload(hip_trainer_t* t, int which, const float* host, int64_t count);
int hip_trainer_download(hip_trainer_t* t, int which, float* host, int64_t count);
/* the same for `count` floats starting `offset` floats into the arena (tensor-by-tensor loading) */
int hip_trainer_upload_at(hip_trainer_t* t, int which, int64_t offset, const float* host, int64_t count);
int hip_trainer_download_at(hip_trainer_t* t, int which, int64_t offset, float* host, int64_t count);
void* hip_trainer_device_ptr(hip_trainer_t* t, int which);
int64_t hip_trainer_arena_count(hip_trainer_t* t, int which);     /* floats in that arena; 0 if the mode has none */

/* One packed step.  tokens_packed[total_tokens]; seq_starts[batch_size + 1] (NULL with
 * batch_size 1 = one sequence).  Negative ids are treated as 0 (src/train.c:4473).
 * run_optimizer = 0 leaves the weights untouched (gradients only).  Returns the mean loss,
 * or -1 on error. */
float hip_train_step_full_batch(hip_trainer_t* t, const int* tokens_packed, int total_tokens,
                                const int* seq_starts, int batch_size, int run_optimizer);
float hip_train_step_lora_batch(hip_trainer_t* t, const int* tokens_packed, int total_tokens,
                                const int* seq_starts, int batch_size, int run_optimizer);

/* Forward and loss only, as cuda_eval_forward (src/train_cuda.c:2672-2810): no gradient, no
 * bookkeeping change.  hip_evaluate walks a validation set the way cuda_evaluate does
 * (src/train_cuda.c:2812-2847): one sequence per sample, truncated to max_seq_len, at most
 * max_eval_samples evenly spaced samples (0 = all); returns the mean loss (-1 if none), perplexity
 * in *out_perplexity. */
float hip_eval_forward_batch(hip_trainer_t* t, const int* tokens_packed, int total_tokens,
                             const int* seq_starts, int batch_size);
float hip_evaluate(hip_trainer_t* t, const int* val_tokens, int num_val_tokens, const int* offsets, int num_samples,
                   int max_seq_len, int max_eval_samples, float* out_perplexity);

/* Resume support: the learning rate and the two counters of src/train.c:5439-5463
 * (state->optimizer_step, state->accumulation_counter); a negative counter is left unchanged. */
void  hip_trainer_set_schedule(hip_trainer_t* t, float learning_rate, int optimizer_step, int accumulation_counter);
/* The number of training steps run so far (state->current_step of the reference): the step number in the names of
 * the NaN dump files and in their metadata is this plus one. */
void  hip_trainer_set_step_counter(hip_trainer_t* t, int steps_run);
int   hip_trainer_accumulation_counter(const hip_trainer_t* t);

/* NaN/Inf flag lattice of the reference's --debug-nan-check (src/train.c:4499-4546): with it on,
 * a step checks the same buffers at the same points into the same flag indices
 *   [0..9] global checkpoints, [10 + l] hidden after layer l, [10 + L + 5l + k] attention-backward
 *   checkpoints of layer l, [10 + 6L + l] grad_hidden after layer l's backward, [10 + 7L + 0..4]
 *   embedding weight / gradient / m / v before AdamW and weight after it,
 * holds AdamW back until the flags have been read, skips it when any is set and returns NAN
 * (src/train.c:5446-5448, :5486-5660).  hip_trainer_nan_flags copies the last step's flags and
 * returns their count; hip_trainer_nan_report prints the "- buffer: ..." lines.
 * When a step detects a NaN/Inf it also writes the step's buffers for offline inspection, in the files and layouts
 * of src/train.c:5562-5653 that tools/nan_dump_inspect.c reads: "<prefix>_<step>_meta.txt", "_tokens.u32",
 * "_hidden.f32", "_logits.f32", "_grad_logits.f32", ..., "_L0_q.f32", "_grad_v.f32".  The prefix defaults to the
 * reference's "/tmp/seraph_nan_step"; hip_trainer_set_nan_dump_prefix changes it (NULL or "": no dumps). */
int   hip_trainer_enable_nan_check(hip_trainer_t* t, int on);
void  hip_trainer_set_nan_dump_prefix(hip_trainer_t* t, const char* prefix);
int   hip_trainer_nan_detected(const hip_trainer_t* t);
int   hip_trainer_nan_flags(const hip_trainer_t* t, uint32_t* out, int max);
void  hip_trainer_nan_report(const hip_trainer_t* t, FILE* out);

int   hip_trainer_optimizer_step(const hip_trainer_t* t);
float hip_trainer_last_lr(const hip_trainer_t* t);
/* device time of the phases of the last step, in ms: [0] forward+loss, [1] backward, [2] optimizer */
void  hip_trainer_last_timing(const hip_trainer_t* t, float ms[3]);
size_t hip_trainer_device_bytes(const hip_trainer_t* t);

/* Optional per-kernel accounting (the counterpart of the reference's per-op profilers,
 * src/vulkan_backend.c:105-210, include/cuda_profiler.h:18-28): with timing on, every
 * kernel-library call of a step is bracketed by an event pair on the step's stream and
 * folded per kernel class with its algorithmic work (flops for the matrix-core kernels,
 * compulsory HBM bytes for the streaming ones). */
typedef struct {
    const char* name;      /* GEMMs: the kernel instantiation, as a profiler names it */
    int64_t     launches;
    double      ms;        /* summed device time */
    double      flops;     /* summed algorithmic flops (0 for bandwidth-bound classes) */
    double      bytes;     /* summed algorithmic bytes (0 for matrix-core classes)     */
} hip_op_stat_t;
void hip_trainer_enable_op_timing(hip_trainer_t* t, int on);
/* Full-weight steps run the weight-gradient products on a second stream beside the chain of input gradients (on by
 * default where max_tokens * hidden <= 2^22, off above, where each product fills the chip by itself; results are the
 * same either way, each product being one kernel whichever stream carries it). Per-op timing
 * and the NaN lattice keep the step on one stream. No counterpart in the reference, whose steps are one stream. */
void hip_trainer_enable_wgrad_overlap(hip_trainer_t* t, int on);
void hip_trainer_reset_op_stats(hip_trainer_t* t);
int  hip_trainer_op_stats(const hip_trainer_t* t, hip_op_stat_t* out, int max);

#ifdef __cplusplus
}
#endif
#endif
