/*
 * hip_backend.h - the backend op API that Seraph's training code links against
 * (include/vulkan_backend.h:357-642 of the Seraph tree), served by the MI355X
 * kernel library instead of Vulkan.
 *
 * Two ways to build src/hip_backend.c and src/hip_backend_backward.c:
 *
 *   inside the Seraph tree (`make hip`, -DSERAPH_TREE): Seraph's own
 *   vulkan_backend.h supplies vulkan_context_t / vulkan_buffer_t and the
 *   prototypes, so the struct layout train.c reads is Seraph's by construction;
 *
 *   stand-alone (this repository's tests and drivers): the declarations below are
 *   used.  The context then only carries the fields this backend itself fills;
 *   the rest of Seraph's context is a table of buffer slots that train.c owns and
 *   the backend never touches (src/train.c:2606-3218 fills them).
 *
 * Semantics kept from the reference: ops return void and ignore NULL arguments
 * (src/vulkan_backend_backward.c:577); vulkan_cmd_begin / vulkan_cmd_end_submit
 * return 1 on success; ops issued between them run in issue order with full memory
 * visibility and end_submit blocks until they are done (src/vulkan_backend.c:1282-1353);
 * uploads and downloads are synchronous; buffer->mapped is NULL (device memory), which
 * sends train.c down its malloc + upload path (src/train.c:4466-4474).
 */
#ifndef HIP_BACKEND_H
#define HIP_BACKEND_H

#include <stddef.h>
#include <stdint.h>

#if defined(SERAPH_TREE)
#include "vulkan_backend.h"
#else

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    void*    device;               /* this backend: private state */
    void*    physical_device;
    void*    instance;
    void*    command_pool;
    void*    queue;                /* this backend: the HIP stream */
    uint32_t queue_family;
    int      initialized;
    char     gpu_name[256];
    uint32_t api_version, driver_version, vendor_id, device_id, device_type;
    uint32_t max_workgroup_size[3];
    uint32_t max_workgroup_invocations;
    uint32_t max_workgroup_count[3];
    uint32_t subgroup_size;
    uint32_t max_subgroups_per_workgroup;
    uint32_t max_shared_memory;
    uint32_t max_push_constant_size;
    uint32_t max_bound_descriptor_sets;
    uint32_t max_storage_buffer_range;
    uint64_t vram_bytes;
    uint64_t shared_system_bytes;
    uint32_t min_storage_buffer_offset, min_uniform_buffer_offset;
    uint32_t max_storage_buffers_per_stage;
    uint32_t max_compute_units;
    uint32_t warps_per_compute_unit;
    uint32_t min_subgroup_size, max_subgroup_size;
    int      has_sm_builtins, has_shader_atomic_float, has_cooperative_matrix, has_shader_clock;
    uint32_t subgroup_supported_stages, subgroup_supported_ops, subgroup_quad_ops;
    float    timestamp_period;
    uint32_t timestamp_valid_bits;
    uint32_t wg_size_1d, wg_size_attn, wg_size_matmul, matmul_reg, matmul_bk;
    int      profiling;
    int      prof_num_ops;
    void*    prof_ops;
    void*    prof_query_pool;
    void*    prof_log;
    void*    caller_slots[512];    /* stands for the caller-owned buffer table of the reference context */
} vulkan_context_t;

typedef struct {
    void*  buffer;                 /* device pointer */
    void*  memory;                 /* unused */
    size_t size;                   /* bytes */
    void*  mapped;                 /* always NULL: device memory is not host visible */
} vulkan_buffer_t;

/* runtime */
vulkan_context_t* vulkan_init(int pool_size_hint);
vulkan_context_t* vulkan_init_ex(int pool_size_hint, int device_index);
void vulkan_free(vulkan_context_t* ctx);
int  vulkan_cmd_begin(vulkan_context_t* ctx);
int  vulkan_cmd_end_submit(vulkan_context_t* ctx);

/* buffers; counts are in elements, *_bytes in bytes, all clamped to the buffer size */
vulkan_buffer_t* vulkan_buffer_create(vulkan_context_t* ctx, size_t size);
void vulkan_buffer_free(vulkan_context_t* ctx, vulkan_buffer_t* buf);
void vulkan_buffer_upload(vulkan_context_t* ctx, vulkan_buffer_t* buf, const float* data, size_t count);
void vulkan_buffer_upload_bytes(vulkan_context_t* ctx, vulkan_buffer_t* buf, const void* data, size_t bytes);
void vulkan_buffer_upload_u32(vulkan_context_t* ctx, vulkan_buffer_t* buf, const uint32_t* data, size_t count);
void vulkan_buffer_download(vulkan_context_t* ctx, vulkan_buffer_t* buf, float* data, size_t count);
void vulkan_buffer_download_bytes(vulkan_context_t* ctx, vulkan_buffer_t* buf, void* data, size_t bytes);
void vulkan_fill_buffer(vulkan_context_t* ctx, vulkan_buffer_t* buf, uint32_t value, size_t bytes);
void vulkan_fill_buffer_range(vulkan_context_t* ctx, vulkan_buffer_t* buf, size_t offset_bytes, uint32_t value, size_t bytes);
void vulkan_copy_buffer(vulkan_context_t* ctx, vulkan_buffer_t* src, vulkan_buffer_t* dst, size_t bytes);
void vulkan_copy_buffer_cache(vulkan_context_t* ctx, vulkan_buffer_t* src, vulkan_buffer_t* dst, size_t bytes);
void vulkan_barrier_transfer_to_compute(vulkan_context_t* ctx);
void vulkan_nan_check(vulkan_context_t* ctx, vulkan_buffer_t* input, size_t count_floats, vulkan_buffer_t* flags_u32, uint32_t flag_index);

/* forward ops */
void vulkan_matmul(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C, int M, int N, int K);
void vulkan_matmul_transpose(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C,
                             int M, int N, int K, int transpose_A, int transpose_B, int accumulate);
void vulkan_add(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C, size_t count);
void vulkan_mul(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C, size_t count);
void vulkan_scale(vulkan_context_t* ctx, vulkan_buffer_t* A, size_t count, float alpha);
void vulkan_silu(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* output, size_t count);
void vulkan_rmsnorm(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale, vulkan_buffer_t* output,
                    int rows, int cols, float eps);
void vulkan_rope(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out,
                 int seq_len, int num_heads, int head_dim, float rope_theta);
void vulkan_batch_attention(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                            vulkan_buffer_t* out, int seq_len, int num_heads, int kv_heads, int head_dim);
void vulkan_embed_lookup(vulkan_context_t* ctx, vulkan_buffer_t* tokens_u32, vulkan_buffer_t* embed_weight,
                         vulkan_buffer_t* out_hidden, int seq_len, int hidden_size, int vocab_size);
void vulkan_qk_norm(vulkan_context_t* ctx, vulkan_buffer_t* qk, int seq_len, int num_heads, int head_dim,
                    int use_qk_norm, float eps);

/* loss, backward, optimizer */
void vulkan_cross_entropy_grad(vulkan_context_t* ctx, vulkan_buffer_t* logits, vulkan_buffer_t* targets_u32,
                               vulkan_buffer_t* grad_logits, vulkan_buffer_t* loss_rows, int rows, int cols, int valid_rows);
void vulkan_reduce_sum(vulkan_context_t* ctx, vulkan_buffer_t* in_buf, vulkan_buffer_t* out_buf, size_t count);
void vulkan_rmsnorm_backward_batch(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale,
                                   vulkan_buffer_t* grad_output, vulkan_buffer_t* grad_input, vulkan_buffer_t* grad_scale,
                                   int rows, int cols, float eps);
void vulkan_rope_backward(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out,
                          int seq_len, int num_heads, int head_dim, float rope_theta);
void vulkan_batch_attention_backward(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                                     vulkan_buffer_t* grad_out, vulkan_buffer_t* grad_Q, vulkan_buffer_t* grad_K,
                                     vulkan_buffer_t* grad_V, int seq_len, int num_heads, int kv_heads, int head_dim);
void vulkan_embedding_backward(vulkan_context_t* ctx, vulkan_buffer_t* tokens_u32, vulkan_buffer_t* grad_hidden,
                               vulkan_buffer_t* grad_embed, int seq_len, int hidden_size, int vocab_size);
void vulkan_silu_backward(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* grad_output,
                          vulkan_buffer_t* grad_input, size_t count);
void vulkan_elementwise_mul_backward(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* grad_C,
                                     vulkan_buffer_t* grad_A, vulkan_buffer_t* grad_B, size_t count);
void vulkan_adamw_update(vulkan_context_t* ctx, vulkan_buffer_t* weight, vulkan_buffer_t* grad, vulkan_buffer_t* m,
                         vulkan_buffer_t* v, float lr, float beta1, float beta2, float weight_decay, float eps,
                         int step, size_t size);

/* video-mode ops: present so the training object links; not part of the LLM path */
void vulkan_patch_extract(vulkan_context_t* ctx, vulkan_buffer_t* frame, vulkan_buffer_t* patches,
                          int frame_h, int frame_w, int channels, int patch_t, int patch_h, int patch_w);
void vulkan_add_bias(vulkan_context_t* ctx, vulkan_buffer_t* data, vulkan_buffer_t* bias, int rows, int cols);
void vulkan_bce_loss_grad(vulkan_context_t* ctx, vulkan_buffer_t* logits, vulkan_buffer_t* targets,
                          vulkan_buffer_t* grad_logits, vulkan_buffer_t* loss_out, size_t count);
void vulkan_sum_cols(vulkan_context_t* ctx, vulkan_buffer_t* data, vulkan_buffer_t* out, int rows, int cols);

/* per-op timing */
void vulkan_profiler_enable(vulkan_context_t* ctx);
void vulkan_profiler_disable(vulkan_context_t* ctx);
void vulkan_profiler_set_log(vulkan_context_t* ctx, void* file_ptr);
void vulkan_profiler_begin_step(vulkan_context_t* ctx);
void vulkan_profiler_end_step(vulkan_context_t* ctx, int step, int seq_len, float loss);

#ifdef __cplusplus
}
#endif
#endif /* !SERAPH_TREE */

/* ---------------------------------------------------------------------------
 * Additions of this backend (both build modes).  The packed-batch forms carry the
 * arguments of include/cuda_train_context.h:273-288; the fused forms have no reference
 * counterpart and replace op pairs of src/train.c:4726-4732 and :5131-5140.
 * ------------------------------------------------------------------------- */
#ifdef __cplusplus
extern "C" {
#endif

void hip_rope_packed(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out, vulkan_buffer_t* seq_starts,
                     int total_tokens, int batch_size, int num_heads, int head_dim, float rope_theta);
void hip_rope_backward_packed(vulkan_context_t* ctx, vulkan_buffer_t* x_in, vulkan_buffer_t* x_out, vulkan_buffer_t* seq_starts,
                              int total_tokens, int batch_size, int num_heads, int head_dim, float rope_theta);
void hip_batch_attention_packed(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                                vulkan_buffer_t* out, vulkan_buffer_t* lse_out, vulkan_buffer_t* seq_starts,
                                int total_tokens, int batch_size, int num_heads, int kv_heads, int head_dim);
void hip_batch_attention_backward_packed(vulkan_context_t* ctx, vulkan_buffer_t* Q, vulkan_buffer_t* K, vulkan_buffer_t* V,
                                         vulkan_buffer_t* attn_out, vulkan_buffer_t* lse, vulkan_buffer_t* grad_out,
                                         vulkan_buffer_t* grad_Q, vulkan_buffer_t* grad_K, vulkan_buffer_t* grad_V,
                                         vulkan_buffer_t* seq_starts, int total_tokens, int batch_size,
                                         int num_heads, int kv_heads, int head_dim);
void hip_cross_entropy_grad_packed(vulkan_context_t* ctx, vulkan_buffer_t* logits, vulkan_buffer_t* targets_u32,
                                   vulkan_buffer_t* grad_logits, vulkan_buffer_t* loss_rows, vulkan_buffer_t* seq_starts,
                                   int total_tokens, int batch_size, int vocab_size, int num_valid_predictions);
void hip_swiglu(vulkan_context_t* ctx, vulkan_buffer_t* gate, vulkan_buffer_t* up, vulkan_buffer_t* out, size_t count);
void hip_swiglu_backward(vulkan_context_t* ctx, vulkan_buffer_t* gate, vulkan_buffer_t* up, vulkan_buffer_t* grad_hidden,
                         vulkan_buffer_t* grad_gate, vulkan_buffer_t* grad_up, size_t count);
void hip_qk_norm_backward(vulkan_context_t* ctx, vulkan_buffer_t* qk_pre, vulkan_buffer_t* grad_out, vulkan_buffer_t* grad_in,
                          int seq_len, int num_heads, int head_dim, float eps);
/* AdamW with the per-element gradient clamp (clip <= 0: identical to vulkan_adamw_update) */
void hip_adamw_update_clipped(vulkan_context_t* ctx, vulkan_buffer_t* weight, vulkan_buffer_t* grad, vulkan_buffer_t* m,
                              vulkan_buffer_t* v, float lr, float beta1, float beta2, float weight_decay, float eps,
                              int step, size_t size, float clip);
/* vulkan_adamw_update over `count` tensors as one recorded op: a maintainer replaces the body of
 * full_weights_optimizer_step_gpu_resident_record (src/train.c:4225-4284: one vulkan_adamw_update and one barrier per
 * tensor, 2 + 9 L of them) by filling the four arrays and calling this once.  sizes are element counts; NULL entries
 * or zero sizes are skipped like the single-tensor op skips them.  Bit-identical to the per-tensor calls. */
void hip_adamw_update_multi(vulkan_context_t* ctx, int count, vulkan_buffer_t* const* weights, vulkan_buffer_t* const* grads,
                            vulkan_buffer_t* const* m, vulkan_buffer_t* const* v, const size_t* sizes,
                            float lr, float beta1, float beta2, float weight_decay, float eps, int step, float clip);
/* sum = input + addend, output = rmsnorm(sum): the vulkan_add that closes a residual branch and the vulkan_rmsnorm
 * that reads its result (src/train.c:4705-4711) in one pass; sum is a buffer of its own */
void hip_add_rmsnorm(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* addend, vulkan_buffer_t* sum,
                     vulkan_buffer_t* scale, vulkan_buffer_t* output, int rows, int cols, float eps);
/* vulkan_rmsnorm_backward_batch with the vulkan_add that follows it (src/train.c:5180-5193) folded in:
 * grad_input = residual + input gradient; residual may be grad_input itself */
void hip_rmsnorm_backward_residual(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale,
                                   vulkan_buffer_t* grad_output, vulkan_buffer_t* residual, vulkan_buffer_t* grad_input,
                                   vulkan_buffer_t* grad_scale, int rows, int cols, float eps);
/* vulkan_rmsnorm_backward_batch in two halves, for a step whose norms are small enough that each column-sum launch
 * counts: hip_rmsnorm_backward_rows is the row pass (grad_input complete; residual may be NULL; the column sums behind
 * grad_scale stay in `partial`, a buffer of hip_rmsnorm_backward_partial_bytes(rows, cols) bytes kept per norm) and
 * returns the number of partial rows (0 on error); one hip_rmsnorm_colsum_multi after the last layer then adds every
 * norm's column sums into its grad_scale (src/train.c:5071-5355: 2 L + 1 norms), bit-identically to the one-call op. */
size_t hip_rmsnorm_backward_partial_bytes(int rows, int cols);
int hip_rmsnorm_backward_rows(vulkan_context_t* ctx, vulkan_buffer_t* input, vulkan_buffer_t* scale, vulkan_buffer_t* grad_output,
                              vulkan_buffer_t* residual, vulkan_buffer_t* grad_input, vulkan_buffer_t* partial,
                              int rows, int cols, float eps);
void hip_rmsnorm_colsum_multi(vulkan_context_t* ctx, int count, vulkan_buffer_t* const* partial, const int* nparts,
                              vulkan_buffer_t* const* grad_scale, int cols);
/* C (+)= alpha * op(A) op(B): vulkan_matmul_transpose followed by vulkan_scale of the product, the pair the
 * LoRA path issues (src/train.c:5785-5792, :5815-5841), as one op.  accumulate with alpha != 1 is only possible
 * for the shapes the library computes through its scratch (small output, long K); otherwise the op reports an
 * error and leaves C untouched. */
void hip_matmul_scaled(vulkan_context_t* ctx, vulkan_buffer_t* A, vulkan_buffer_t* B, vulkan_buffer_t* C,
                       int M, int N, int K, int transpose_A, int transpose_B, int accumulate, float alpha);
/* number of ops whose kernel library call failed since init (errors are also printed to stderr) */
int hip_backend_error_count(vulkan_context_t* ctx);

#ifdef __cplusplus
}
#endif
#endif
