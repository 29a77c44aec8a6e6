/*
 * hip_backend_backward.c - loss, backward and scatter ops of the backend API (the
 * counterpart of Seraph's src/vulkan_backend_backward.c) over the MI355X kernel library.
 * Each function keeps the reference's signature and conventions: void return, NULL
 * arguments ignored, outputs that the reference accumulates into are accumulated into.
 */
#include <math.h>
#include <stdlib.h>

#include "hip_backend_internal.h"

/* src/vulkan_backend_backward.c:571-689 */
void vulkan_cross_entropy_grad(vulkan_context_t* ctx, vulkan_buffer_t* logits, vulkan_buffer_t* targets_u32,
                               vulkan_buffer_t* grad_logits, vulkan_buffer_t* loss_rows, int rows, int cols, int valid_rows) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !logits || !targets_u32 || !grad_logits || !loss_rows || rows < 0 || cols < 0) return;
    if (!hip_backend_fits(ctx, "cross_entropy_grad", 4, FIT(logits, (size_t)rows * cols), FIT(targets_u32, rows),
                          FIT(grad_logits, (size_t)rows * cols), FIT(loss_rows, rows))) return;
    HIP_OPF(ctx, seraph_cross_entropy_grad(FPTR(logits), UPTR(targets_u32), FPTR(grad_logits), FPTR(loss_rows),
                                                               NULL, 1, rows, cols, valid_rows, st->stream), "cross_entropy_grad [%dx%d] %u-thr", rows, cols, ctx->wg_size_1d);
}

void hip_cross_entropy_grad_packed(vulkan_context_t* ctx, vulkan_buffer_t* logits, vulkan_buffer_t* targets_u32,
                                   vulkan_buffer_t* grad_logits, vulkan_buffer_t* loss_rows, vulkan_buffer_t* seq_starts,
                                   int total_tokens, int batch_size, int vocab_size, int num_valid_predictions) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !logits || !targets_u32 || !grad_logits || !loss_rows || !seq_starts || total_tokens < 0 || vocab_size < 0 || batch_size < 0) return;
    if (!hip_backend_fits(ctx, "cross_entropy_grad_packed", 5, FIT(logits, (size_t)total_tokens * vocab_size), FIT(targets_u32, total_tokens),
                          FIT(grad_logits, (size_t)total_tokens * vocab_size), FIT(loss_rows, total_tokens),
                          FIT(seq_starts, (size_t)batch_size + 1))) return;
    HIP_OPF(ctx, seraph_cross_entropy_grad(FPTR(logits), UPTR(targets_u32), FPTR(grad_logits), FPTR(loss_rows),
                                                                      UPTR(seq_starts), batch_size, total_tokens, vocab_size,
                                                                      num_valid_predictions, st->stream), "cross_entropy_grad_packed [%dx%d] %u-thr", total_tokens, vocab_size, ctx->wg_size_1d);
}

/* src/vulkan_backend_backward.c:691-800: 512 inputs per output (src/train.c:4906-4913) */
void vulkan_reduce_sum(vulkan_context_t* ctx, vulkan_buffer_t* in_buf, vulkan_buffer_t* out_buf, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !in_buf || !out_buf || count == 0) return;
    if (!hip_backend_fits(ctx, "reduce_sum", 2, FIT(in_buf, count), FIT(out_buf, (count + 511) / 512))) return;
    HIP_OP(ctx, "reduce_sum", seraph_reduce_sum(FPTR(in_buf), FPTR(out_buf), count, st->stream));
}

/* src/vulkan_backend_backward.c:802-929 */
void vulkan_rmsnorm_backward_batch(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale,
                                   vulkan_buffer_t* grad_output, vulkan_buffer_t* grad_input, vulkan_buffer_t* grad_scale,
                                   int rows, int cols, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !scale || !grad_output || !grad_input || !grad_scale || rows < 0 || cols < 0) return;
    const size_t rc = (size_t)rows * cols;
    if (!hip_backend_fits(ctx, "rmsnorm_bwd", 5, FIT(input, rc), FIT(scale, cols), FIT(grad_output, rc), FIT(grad_input, rc), FIT(grad_scale, cols))) return;
    size_t need = seraph_rmsnorm_backward_ws_bytes(rows, cols);
    void* ws = hip_backend_scratch(ctx, need);
    if (!ws) return;
    HIP_OPF(ctx, seraph_rmsnorm_backward(FPTR(input), FPTR(scale), FPTR(grad_output), FPTR(grad_input),
                                                                  FPTR(grad_scale), rows, cols, eps, ws, st->ws_bytes, st->stream), "rmsnorm_bwd [%dx%d] %u-thr", rows, cols, ctx->wg_size_1d);
}

/* vulkan_rmsnorm_backward_batch and the vulkan_add of the residual gradient that follows it (src/train.c:5180-5193):
 * grad_input = residual + input gradient; residual may be grad_input itself. */
void hip_rmsnorm_backward_residual(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale,
                                   vulkan_buffer_t* grad_output, vulkan_buffer_t* residual, vulkan_buffer_t* grad_input,
                                   vulkan_buffer_t* grad_scale, int rows, int cols, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !scale || !grad_output || !residual || !grad_input || !grad_scale || rows < 0 || cols < 0) return;
    const size_t rc = (size_t)rows * cols;
    if (!hip_backend_fits(ctx, "rmsnorm_bwd+add", 6, FIT(input, rc), FIT(scale, cols), FIT(grad_output, rc), FIT(residual, rc),
                          FIT(grad_input, rc), FIT(grad_scale, cols))) return;
    size_t need = seraph_rmsnorm_backward_ws_bytes(rows, cols);
    void* ws = hip_backend_scratch(ctx, need);
    if (!ws) return;
    HIP_OPF(ctx, seraph_rmsnorm_backward_residual(FPTR(input), FPTR(scale), FPTR(grad_output), FPTR(residual),
                                                                              FPTR(grad_input), FPTR(grad_scale), rows, cols, eps, ws,
                                                                              st->ws_bytes, st->stream), "rmsnorm_bwd+add [%dx%d] %u-thr", rows, cols, ctx->wg_size_1d);
}

/* The row pass of vulkan_rmsnorm_backward_batch alone (residual may be NULL): grad_input is complete, and the column
 * sums behind grad_scale stay in `partial`, a buffer of hip_rmsnorm_backward_partial_bytes(rows, cols) bytes that the
 * caller keeps for this norm until hip_rmsnorm_colsum_multi has run.  Returns the number of partial rows, 0 on error. */
size_t hip_rmsnorm_backward_partial_bytes(int rows, int cols) { return seraph_rmsnorm_backward_ws_bytes(rows, cols); }

int hip_rmsnorm_backward_rows(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale, vulkan_buffer_t* grad_output,
                              vulkan_buffer_t* residual, vulkan_buffer_t* grad_input, vulkan_buffer_t* partial,
                              int rows, int cols, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !scale || !grad_output || !grad_input || !partial || rows < 0 || cols < 0) return 0;
    const size_t rc = (size_t)rows * cols;
    if (!hip_backend_fits(ctx, "rmsnorm_bwd_rows", 5, FIT(input, rc), FIT(scale, cols), FIT(grad_output, rc), FIT(residual, rc), FIT(grad_input, rc))) return 0;
    int nparts = 0;
    HIP_OPF(ctx, seraph_rmsnorm_backward_rows(FPTR(input), FPTR(scale), FPTR(grad_output),
                                                                      residual ? FPTR(residual) : NULL, FPTR(grad_input), rows, cols, eps,
                                                                      DPTR(partial), partial->size, &nparts, st->stream), "rmsnorm_bwd_rows [%dx%d] %u-thr", rows, cols, ctx->wg_size_1d);
    return nparts;
}

/* grad_scale[i] += column sums of partial[i] (nparts[i] rows as hip_rmsnorm_backward_rows returned them), for `count`
 * norms of one width in one recorded op: the 2 L + 1 norms of a step (src/train.c:5071-5355) folded after the last
 * layer.  Bit-identical to vulkan_rmsnorm_backward_batch's grad_scale. */
void hip_rmsnorm_colsum_multi(vulkan_context_t* ctx, int count, vulkan_buffer_t* const* partial, const int* nparts,
                              vulkan_buffer_t* const* grad_scale, int cols) {
    hip_state_t* st = hip_state(ctx);
    if (!st || count <= 0 || !partial || !nparts || !grad_scale) return;
    seraph_colsum_job_t* jobs = (seraph_colsum_job_t*)malloc((size_t)count * sizeof(*jobs));
    if (!jobs) { hip_backend_report(ctx, "rmsnorm_colsum_multi", SERAPH_ERR_INVALID); return; }
    int k = 0;
    for (int i = 0; i < count; i++) {
        if (!partial[i] || !grad_scale[i] || nparts[i] <= 0) continue;                 /* skipped silently, like a NULL op argument */
        if (!hip_backend_fits(ctx, "rmsnorm_bwd_colsum", 2, FIT(partial[i], (size_t)nparts[i] * cols), FIT(grad_scale[i], cols))) continue;
        jobs[k].partial = FPTR(partial[i]); jobs[k].nparts = nparts[i]; jobs[k].grad_scale = FPTR(grad_scale[i]);
        k++;
    }
    HIP_OP(ctx, "rmsnorm_bwd_colsum", seraph_rmsnorm_colsum_multi(jobs, k, cols, st->stream));
    free(jobs);
}

/* src/vulkan_backend_backward.c:931-1045 */
void vulkan_rope_backward(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out,
                          int seq_len, int num_heads, int head_dim, float rope_theta) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !x_in || !x_out || seq_len < 0 || num_heads < 0 || head_dim < 0) return;
    const size_t n = (size_t)seq_len * num_heads * head_dim;
    if (!hip_backend_fits(ctx, "rope_bwd", 2, FIT(x_in, n), FIT(x_out, n))) return;
    HIP_OP(ctx, "rope_bwd", seraph_rope(FPTR(x_in), FPTR(x_out), NULL, 1, seq_len, num_heads, head_dim, rope_theta, 1, st->stream));
}

void hip_rope_backward_packed(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out, vulkan_buffer_t* seq_starts,
                              int total_tokens, int batch_size, int num_heads, int head_dim, float rope_theta) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !x_in || !x_out || !seq_starts || total_tokens < 0 || batch_size < 0 || num_heads < 0 || head_dim < 0) return;
    const size_t n = (size_t)total_tokens * num_heads * head_dim;
    if (!hip_backend_fits(ctx, "rope_bwd_packed", 3, FIT(x_in, n), FIT(x_out, n), FIT(seq_starts, (size_t)batch_size + 1))) return;
    HIP_OP(ctx, "rope_bwd_packed", seraph_rope(FPTR(x_in), FPTR(x_out), UPTR(seq_starts), batch_size, total_tokens, num_heads,
                                                    head_dim, rope_theta, 1, st->stream));
}

/* src/vulkan_backend_backward.c:1047-1183.  The reference saves neither the attention output
 * nor the log-sum-exp, so this entry point recomputes both; no sequence-length cap. */
void vulkan_batch_attention_backward(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                                     vulkan_buffer_t* grad_out, vulkan_buffer_t* grad_Q, vulkan_buffer_t* grad_K,
                                     vulkan_buffer_t* grad_V, int seq_len, int num_heads, int kv_heads, int head_dim) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !Q || !K || !V || !grad_out || !grad_Q || !grad_K || !grad_V || seq_len < 0 || num_heads < 0 || kv_heads < 0 || head_dim < 0) return;
    const size_t nq = (size_t)seq_len * num_heads * head_dim, nkv = (size_t)seq_len * kv_heads * head_dim;
    if (!hip_backend_fits(ctx, "attn_bwd", 7, FIT(Q, nq), FIT(K, nkv), FIT(V, nkv), FIT(grad_out, nq), FIT(grad_Q, nq), FIT(grad_K, nkv), FIT(grad_V, nkv))) return;
    /* one sequence of known length: scratch for the dS band (5 matrix products) unless that is huge */
    size_t need = seraph_attention_backward_ws_bytes_banded(seq_len, num_heads, kv_heads, head_dim, seq_len);
    if (need > ((size_t)8 << 30)) need = seraph_attention_backward_ws_bytes(seq_len, num_heads, kv_heads, head_dim);
    void* ws = hip_backend_scratch(ctx, need);
    if (!ws) return;
    float scale = 1.0f / sqrtf((float)head_dim);          /* :1168 */
    HIP_OPF(ctx, seraph_attention_backward_banded(FPTR(Q), FPTR(K), FPTR(V), FPTR(grad_out), NULL, NULL,
                                                                     FPTR(grad_Q), FPTR(grad_K), FPTR(grad_V), NULL, 1, seq_len,
                                                                     num_heads, kv_heads, head_dim, scale, seq_len, ws, need, st->stream), "attn_bwd [seq=%d h=%d hd=%d]", seq_len, num_heads, head_dim);
}

void hip_batch_attention_backward_packed(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                                         vulkan_buffer_t* attn_out, vulkan_buffer_t* lse, vulkan_buffer_t* grad_out,
                                         vulkan_buffer_t* grad_Q, vulkan_buffer_t* grad_K, vulkan_buffer_t* grad_V,
                                         vulkan_buffer_t* seq_starts, int total_tokens, int batch_size,
                                         int num_heads, int kv_heads, int head_dim) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !Q || !K || !V || !grad_out || !grad_Q || !grad_K || !grad_V || !seq_starts || total_tokens < 0 || batch_size < 0 ||
        num_heads < 0 || kv_heads < 0 || head_dim < 0) return;
    const size_t nq = (size_t)total_tokens * num_heads * head_dim, nkv = (size_t)total_tokens * kv_heads * head_dim;
    if (!hip_backend_fits(ctx, "attn_bwd_packed", 10, FIT(Q, nq), FIT(K, nkv), FIT(V, nkv), FIT(attn_out, nq), FIT(lse, (size_t)total_tokens * num_heads),
                          FIT(grad_out, nq), FIT(grad_Q, nq), FIT(grad_K, nkv), FIT(grad_V, nkv), FIT(seq_starts, (size_t)batch_size + 1))) return;
    size_t need = seraph_attention_backward_ws_bytes(total_tokens, num_heads, kv_heads, head_dim);
    void* ws = hip_backend_scratch(ctx, need);
    if (!ws) return;
    float scale = 1.0f / sqrtf((float)head_dim);
    HIP_OPF(ctx, seraph_attention_backward(FPTR(Q), FPTR(K), FPTR(V), FPTR(grad_out), attn_out ? FPTR(attn_out) : NULL, lse ? FPTR(lse) : NULL,
                                     FPTR(grad_Q), FPTR(grad_K), FPTR(grad_V), UPTR(seq_starts), batch_size, total_tokens,
                                     num_heads, kv_heads, head_dim, scale, ws, st->ws_bytes, st->stream), "attn_bwd_packed [tok=%d seqs=%d h=%d hd=%d]", total_tokens, batch_size, num_heads, head_dim);
}

/* src/vulkan_backend_backward.c:1185-1300 */
void vulkan_embedding_backward(vulkan_context_t* ctx, vulkan_buffer_t* tokens_u32, vulkan_buffer_t* grad_hidden,
                               vulkan_buffer_t* grad_embed, int seq_len, int hidden_size, int vocab_size) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !tokens_u32 || !grad_hidden || !grad_embed || seq_len < 0 || hidden_size < 0 || vocab_size < 0) return;
    if (!hip_backend_fits(ctx, "embed_bwd", 3, FIT(tokens_u32, seq_len), FIT(grad_hidden, (size_t)seq_len * hidden_size),
                          FIT(grad_embed, (size_t)vocab_size * hidden_size))) return;
    size_t need = seraph_embedding_backward_ws_bytes(seq_len, vocab_size);
    void* ws = hip_backend_scratch(ctx, need);
    if (!ws) return;
    HIP_OP(ctx, "embed_bwd", seraph_embedding_backward(UPTR(tokens_u32), FPTR(grad_hidden), FPTR(grad_embed), seq_len,
                                                                hidden_size, vocab_size, ws, st->ws_bytes, st->stream));
}

/* src/vulkan_backend_backward.c:159-297 */
void vulkan_silu_backward(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* grad_output,
                          vulkan_buffer_t* grad_input, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !input || !grad_output || !grad_input) return;
    if (!hip_backend_fits(ctx, "silu_bwd", 3, FIT(input, count), FIT(grad_output, count), FIT(grad_input, count))) return;
    HIP_OP(ctx, "silu_bwd", seraph_silu_backward(FPTR(input), FPTR(grad_output), FPTR(grad_input), count, st->stream));
}

/* src/vulkan_backend_backward.c:300-452 */
void vulkan_elementwise_mul_backward(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* grad_C,
                                     vulkan_buffer_t* grad_A, vulkan_buffer_t* grad_B, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !A || !B || !grad_C || !grad_A || !grad_B) return;
    if (!hip_backend_fits(ctx, "mul_bwd", 5, FIT(A, count), FIT(B, count), FIT(grad_C, count), FIT(grad_A, count), FIT(grad_B, count))) return;
    HIP_OP(ctx, "mul_bwd", seraph_mul_backward(FPTR(A), FPTR(B), FPTR(grad_C), FPTR(grad_A), FPTR(grad_B), count, st->stream));
}

void hip_swiglu_backward(vulkan_context_t* ctx, vulkan_buffer_t* gate, vulkan_buffer_t* up, vulkan_buffer_t* grad_hidden,
                         vulkan_buffer_t* grad_gate, vulkan_buffer_t* grad_up, size_t count) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !gate || !up || !grad_hidden || !grad_gate || !grad_up) return;
    if (!hip_backend_fits(ctx, "silu_mul_bwd", 5, FIT(gate, count), FIT(up, count), FIT(grad_hidden, count), FIT(grad_gate, count), FIT(grad_up, count))) return;
    HIP_OP(ctx, "silu_mul_bwd", seraph_swiglu_backward(FPTR(gate), FPTR(up), FPTR(grad_hidden), FPTR(grad_gate), FPTR(grad_up), count, st->stream));
}

void hip_qk_norm_backward(vulkan_context_t* ctx, vulkan_buffer_t* qk_pre, vulkan_buffer_t* grad_out, vulkan_buffer_t* grad_in,
                          int seq_len, int num_heads, int head_dim, float eps) {
    hip_state_t* st = hip_state(ctx);
    if (!st || !qk_pre || !grad_out || !grad_in || seq_len < 0 || num_heads < 0 || head_dim < 0) return;
    const size_t n = (size_t)seq_len * num_heads * head_dim;
    if (!hip_backend_fits(ctx, "qk_norm_bwd", 3, FIT(qk_pre, n), FIT(grad_out, n), FIT(grad_in, n))) return;
    HIP_OP(ctx, "qk_norm_bwd", seraph_qk_norm_backward(FPTR(qk_pre), FPTR(grad_out), FPTR(grad_in), seq_len, num_heads, head_dim, eps, st->stream));
}
