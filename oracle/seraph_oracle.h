/*
 * seraph_oracle.h - CPU restatement of Seraph's training backward / optimizer
 * path.  TEST INFRASTRUCTURE ONLY: this code is the parity checker and the
 * timed CPU baseline.  Nothing in the shipped library links, loads or calls it.
 *
 * Every function restates the arithmetic of one reference compute shader
 * (shaders/<name>.comp) or one host routine, cited at each prototype.  Unless a
 * note says otherwise, reductions are carried in double so that the oracle sits
 * well inside the 1e-4 relative / 1e-5 absolute band in which an FP32 device
 * kernel with any summation order must agree.
 *
 * Layout conventions (all row-major FP32):
 *   activations  [T, width]  token-major, heads interleaved per token
 *   projections  [out, in]   (forward is X * W^T)
 *   seq_starts   [B+1]       prefix offsets of the packed sequences, or NULL
 *                            with batch = 1 meaning one sequence of T tokens.
 *
 * Pinning status (what fixes each function besides its own formula) is listed
 * in tests/test_oracle_pins.py; functions with no independent reference-side
 * vector are marked there.  The reference ships no golden vectors for any of
 * these ops (its only test of the path is a 64^3 integer matmul).
 */
#ifndef SERAPH_ORACLE_H
#define SERAPH_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- loss ------------------------------------------------------------- */

/* shaders/cross_entropy_grad.comp:33-99 (host: src/vulkan_backend_backward.c:571-689).
 * rows with target >= cols give loss 0 and a zero gradient row; scale is
 * 1/valid_rows, or 0 when valid_rows == 0. */
void orc_cross_entropy_grad(const float* logits, const uint32_t* targets,
                            float* grad, float* loss_rows,
                            int64_t rows, int64_t cols, int64_t valid_rows);

/* Packed structure of src/cuda_train_context.cu:1657-1741 with the numerics
 * of the shader above: the last token of every sequence yields a zero row and
 * loss 0; scale is 1/num_valid_predictions. */
void orc_cross_entropy_grad_packed(const float* logits, const uint32_t* targets,
                                   float* grad, float* loss_rows,
                                   const uint32_t* seq_starts, int64_t total_tokens,
                                   int batch, int64_t cols, int64_t num_valid);

/* shaders/reduce_sum.comp:20-43 with the 512-per-group contract the caller
 * assumes (src/train.c:4906-4913). out has ceil(count/512) entries. */
void orc_reduce_sum(const float* in, float* out, int64_t count);

/* ---- GEMM family ------------------------------------------------------ */

/* shaders/matmul.comp and shaders/matmul_transpose.comp:35-169.
 * C[M,N] (+)= op(A) * op(B); op(A) is A[M,K] or, transposed, A stored [K,M];
 * op(B) is B[K,N] or, transposed, B stored [N,K]. */
void orc_matmul(const float* A, const float* B, float* C,
                int64_t M, int64_t N, int64_t K, int tA, int tB, int accumulate);
/* The same product as a plain loop nest with every term accumulated in double.  orc_matmul
 * uses it for small shapes and a cache-blocked form (FP32 fused multiply-adds over runs of
 * 256 terms, runs added in double) for large ones; the tests compare the two. */
void orc_matmul_exact(const float* A, const float* B, float* C,
                      int64_t M, int64_t N, int64_t K, int tA, int tB, int accumulate);

/* ---- attention -------------------------------------------------------- */

/* shaders/batch_attention_stream.comp (forward, causal, GQA map
 * kv_head = head*kv_heads/num_heads, scale = 1/sqrt(head_dim) from
 * src/vulkan_backend.c:2980-2984); packed block-diagonal mask as
 * src/cuda_train_context.cu:1289-1440.  lse (optional) is
 * rowmax + log(rowsum) of the scaled scores, src/cuda_train_context.cu:1279. */
void orc_attention_forward(const float* Q, const float* K, const float* V,
                           float* out, float* lse,
                           const uint32_t* seq_starts, int batch, int64_t T,
                           int H, int KVH, int D, float scale);

/* shaders/batch_attention_backward.comp:50-196 and
 * shaders/batch_attention_backward_stream.comp:34-202 (same mathematics);
 * packed mask as src/cuda_train_context.cu:1013-1138.
 * dQ is overwritten, dK and dV are ACCUMULATED into (caller zeroes them,
 * src/train.c:5221-5222). */
void orc_attention_backward(const float* Q, const float* K, const float* V,
                            const float* dO, float* dQ, float* dK, float* dV,
                            const uint32_t* seq_starts, int batch, int64_t T,
                            int H, int KVH, int D, float scale);

/* ---- normalisation / position ---------------------------------------- */

/* shaders/rmsnorm.comp (FP32: y = x * rsqrt(mean(x^2)+eps) * scale). */
void orc_rmsnorm(const float* x, const float* scale, float* y,
                 int64_t rows, int64_t cols, float eps);

/* shaders/rmsnorm_backward_batch.comp:34-100: FP64 intermediates,
 * rms = max(sqrt(ms+eps), 0.01); grad_scale is accumulated (+=). */
void orc_rmsnorm_backward_batch(const float* x, const float* scale, const float* dy,
                                float* dx, float* grad_scale,
                                int64_t rows, int64_t cols, float eps);

/* inv_freq[i] = 1/powf(theta, (2i)/D) evaluated in FP32 exactly as
 * shaders/rope.comp / rope_backward.comp:40-41 write it. */
void orc_rope_inv_freq(float* inv_freq, int D, float theta);

/* shaders/rope.comp and shaders/rope_backward.comp:26-59; interleaved pairs
 * (2i, 2i+1); position is the index inside the packed sequence
 * (src/cuda_train_context.cu:652-704). in/out may alias. */
void orc_rope(const float* in, float* out, const uint32_t* seq_starts, int batch,
              int64_t T, int heads, int D, float theta, int backward);

/* shaders/qk_norm.comp:30-76 forward (gain-less RMS over all heads of a
 * token, rms = max(rms, eps)), and its exact derivative.  The reference has
 * no backward for this op: the derivative is this build's own mathematics. */
void orc_qk_norm(float* qk, int64_t T, int heads, int D, float eps);
void orc_qk_norm_backward(const float* x_pre, const float* dy, float* dx,
                          int64_t T, int heads, int D, float eps);

/* ---- element-wise ----------------------------------------------------- */

void orc_silu(const float* x, float* y, int64_t n);                    /* shaders/silu.comp */
void orc_silu_backward(const float* x, const float* dy, float* dx, int64_t n); /* shaders/silu_backward.comp:26-41 */
void orc_mul_backward(const float* A, const float* B, const float* dC,
                      float* dA, float* dB, int64_t n);                /* shaders/elementwise_mul_backward.comp:24-35 */
/* The two ops above composed as src/train.c:5131-5140 composes them:
 * dUp = dH*silu(gate), dGate = dH*up*silu'(gate). */
void orc_swiglu_backward(const float* gate, const float* up, const float* dH,
                         float* dGate, float* dUp, int64_t n);

/* ---- embedding -------------------------------------------------------- */

void orc_embed_lookup(const uint32_t* tokens, const float* embed, float* out,
                      int64_t T, int64_t hidden, int64_t vocab);        /* shaders/embed_lookup.comp */
/* shaders/embedding_backward.comp:22-44: grad_embed[tok] += dH[p]; tokens
 * >= vocab are skipped.  Rows are summed in position order in double and the
 * total is added to the existing row once. */
void orc_embedding_backward(const uint32_t* tokens, const float* dH, float* grad_embed,
                            int64_t T, int64_t hidden, int64_t vocab);

/* ---- optimizer -------------------------------------------------------- */

/* shaders/adamw.comp:36-61 evaluated in FP32 in the shader's own expression
 * order; bias corrections 1-powf(beta,step) in FP32 as
 * src/vulkan_backend.c:2151-2152.  clip <= 0 disables clipping (the
 * reference formula); clip > 0 clamps each gradient element to [-clip, clip]
 * first (this build's extension, absent from the reference). */
void orc_adamw(float* w, const float* g, float* m, float* v, int64_t n,
               float lr, float beta1, float beta2, float weight_decay, float eps,
               int step, float clip);

/* shaders/nan_check.comp: returns 1 if any element is NaN or Inf. */
int orc_nan_check(const float* x, int64_t n);

/* ---- whole training step --------------------------------------------- */

typedef struct {
    int32_t hidden, layers, heads, kv_heads, head_dim, ffn, vocab;
    float   rms_eps;      /* the reference hard-codes 1e-5 (src/train.c:4378) */
    float   rope_theta;
    /* LoRA (rank 0 = full-weight training) */
    int32_t lora_rank;
    float   lora_alpha;
    int32_t lora_mask;    /* bit0 q, 1 k, 2 v, 3 o, 4 gate, 5 up, 6 down */
    /* 1: shaders/qk_norm.comp on q and k after RoPE, as src/train.c:4688-4689 calls it (eps = the step's rms eps),
     * and its exact derivative in the backward.  The reference's backward has no counterpart (it treats the op as
     * the identity, src/train.c:5224-5266) and its language-model mode never enables it (src/model_config.c:282):
     * PARITY UNPINNED by the reference; pinned by float64 autograd of the forward definition only. */
    int32_t use_qk_norm;
} orc_config_t;

/* Element offsets of every tensor inside one flat parameter vector:
 *   embed[V,h], final_norm[h], then per layer
 *   in_norm[h], q[q,h], k[kv,h], v[kv,h], o[h,q], post_norm[h],
 *   gate[f,h], up[f,h], down[h,f].                                       */
int64_t orc_param_count(const orc_config_t* c);
/* LoRA vector: per layer, for each of q,k,v,o,gate,up,down selected by lora_mask in that
 * order: A[r,in] then B[out,r]. */
int64_t orc_lora_param_count(const orc_config_t* c);

/* One packed full-weight step: forward, loss, backward into `grads`
 * (accumulated: caller zeroes), no optimizer.  Operation order follows
 * src/train.c:4365-5470 with the packed structure of
 * src/train_cuda.c:1966-2326.  Returns the mean loss over T-B predictions. */
float orc_step_full(const orc_config_t* c, const float* params, float* grads,
                    const int32_t* tokens, const int32_t* seq_starts, int batch,
                    int64_t T);

/* One packed LoRA step per src/train.c:5847-6719: base weights frozen, adapter
 * gradients accumulated into lora_grads; the adapter's own contribution to
 * the input gradient is dropped as the reference drops it
 * (grad_input = NULL at every call site, src/train.c:6423-6556). */
float orc_step_lora(const orc_config_t* c, const float* params, const float* lora,
                    float* lora_grads, const int32_t* tokens,
                    const int32_t* seq_starts, int batch, int64_t T);

/* Learning-rate schedule baked into the step: linear warm-up over 100
 * optimizer steps, divided by the accumulation count (src/train.c:5451-5461). */
float orc_lr_schedule(float base_lr, int optimizer_step, int accum_steps);

int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
