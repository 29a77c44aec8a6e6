/*
 * seraph_hip.h - C ABI of libseraph_hip.so: hand-written gfx950 (MI355X)
 * kernels for the backward pass and optimizer of Seraph's training engine,
 * plus the forward ops and the small device runtime a training step needs.
 *
 * Plain C: raw device pointers, sizes, and a stream handle (a hipStream_t
 * passed as void*; NULL = the default stream).  No HIP types appear here, so
 * the host side (src/hip_backend*.c, or the reference's own C code) compiles
 * with any C compiler and without ROCm headers.
 *
 * Every entry point returns SERAPH_OK (0) or a negative error code and never
 * aborts; seraph_hip_last_error() describes the most recent failure on the
 * calling thread.  All launches are asynchronous on `stream`; ordering is the
 * stream's in-order guarantee, which is the guarantee the reference gives
 * between recorded ops (src/vulkan_backend_backward.c:124-142).
 *
 * Layouts (row-major FP32): activations [T, width] token-major with heads
 * interleaved per token; projections [out, in]; seq_starts is a DEVICE array
 * of batch+1 prefix offsets of the packed sequences, or NULL for one sequence.
 * "ws"/"ws_bytes" is caller-owned device scratch; the matching *_ws_bytes()
 * query gives the size an op needs (0 = none).  Scratch contents need not be
 * preserved or initialised between calls.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the Seraph source tree).
 */
#ifndef SERAPH_HIP_H
#define SERAPH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SERAPH_OK             0
#define SERAPH_ERR_INVALID   -1   /* NULL pointer, bad shape, misaligned buffer */
#define SERAPH_ERR_HIP       -2   /* a HIP runtime call or launch failed        */
#define SERAPH_ERR_WORKSPACE -3   /* ws missing or smaller than *_ws_bytes()    */
#define SERAPH_ERR_NODEVICE  -4   /* no gfx950 device visible                   */

typedef void* seraph_stream_t;

/* ---------------------------------------------------------------- runtime
 * Stands in for the device half of vulkan_init_ex / vulkan_buffer_* /
 * vulkan_cmd_end_submit (include/vulkan_backend.h:357-420). */
typedef struct {
    char     name[256];
    char     arch[64];            /* "gfx950..."                          */
    uint64_t hbm_bytes;
    uint32_t compute_units;
    uint32_t wavefront_size;
    uint32_t lds_bytes_per_block;
    uint32_t clock_khz;
} seraph_device_info_t;

const char* seraph_hip_last_error(void);
int  seraph_hip_init(int device_index);                 /* -1 = device 0 */
int  seraph_hip_device_info(seraph_device_info_t* out);
int  seraph_hip_malloc(void** out, size_t bytes);
int  seraph_hip_free(void* p);
int  seraph_hip_host_alloc(void** out, size_t bytes);   /* pinned host memory */
int  seraph_hip_host_free(void* p);
int  seraph_hip_h2d(void* dst, const void* src, size_t bytes, seraph_stream_t s);
int  seraph_hip_d2h(void* dst, const void* src, size_t bytes, seraph_stream_t s);
int  seraph_hip_d2d(void* dst, const void* src, size_t bytes, seraph_stream_t s);
int  seraph_hip_stream_create(seraph_stream_t* out);
int  seraph_hip_stream_destroy(seraph_stream_t s);
int  seraph_hip_stream_sync(seraph_stream_t s);
int  seraph_hip_device_sync(void);
/* event pair timing on a stream (vulkan_profiler_* stand-in, include/vulkan_backend.h:638-642) */
int  seraph_hip_event_create(void** out);
int  seraph_hip_event_create_sync(void** out);                         /* orders streams of one device only: no timestamps, not for the host to wait on */
int  seraph_hip_event_destroy(void* ev);
/* Arms `ev` for the calling thread: the next op of this library that supports it completes the event with its last
 * kernel, which is what hipEventRecord after the op would give, minus the marker packet that a record puts between that
 * kernel and the next.  The ops that take the event: every one-pass element-wise op (fill, add, mul, scale, silu, SwiGLU,
 * their backward forms, AdamW), RoPE, RMSNorm backward and the column sums, reduce_sum - so arm it directly before the op
 * it is meant for.  An op that returns an error disarms it.  seraph_hip_event_armed() tells afterwards whether the event
 * is still waiting for such an op (then record it the ordinary way; seraph_hip_event_on_next_op(NULL) disarms). */
int  seraph_hip_event_on_next_op(void* ev);
int  seraph_hip_event_armed(void);
int  seraph_hip_event_record(void* ev, seraph_stream_t s);
int  seraph_hip_event_elapsed_ms(void* start, void* stop, float* ms);  /* waits for stop */
/* work submitted to `s` after this call starts only when everything recorded into `ev` has completed (two streams of
 * one step: weight gradients beside the chain of input gradients) */
int  seraph_hip_stream_wait_event(seraph_stream_t s, void* ev);

/* ---------------------------------------------------------------- utility ops */
/* vulkan_fill_buffer / vulkan_fill_buffer_range, include/vulkan_backend.h:411-415,525-528 */
int seraph_fill_u32(void* dst, uint32_t value, size_t count, seraph_stream_t s);
/* vulkan_add / vulkan_mul / vulkan_scale, include/vulkan_backend.h:461-473 (shaders/add.comp, mul.comp, scale.comp) */
int seraph_add(const float* a, const float* b, float* c, size_t n, seraph_stream_t s);
int seraph_mul(const float* a, const float* b, float* c, size_t n, seraph_stream_t s);
int seraph_scale(float* a, size_t n, float alpha, seraph_stream_t s);
/* vulkan_nan_check, include/vulkan_backend.h:419-423 (shaders/nan_check.comp): flags[flag_index] |= 1 */
int seraph_nan_check(const float* x, size_t n, uint32_t* flags, uint32_t flag_index, seraph_stream_t s);
/* vulkan_reduce_sum, include/vulkan_backend.h:546-549 (shaders/reduce_sum.comp): out[g] = sum of 512 inputs */
int seraph_reduce_sum(const float* in, float* out, size_t count, seraph_stream_t s);

/* ---------------------------------------------------------------- loss */
/* vulkan_cross_entropy_grad, include/vulkan_backend.h:538-543 (shaders/cross_entropy_grad.comp:33-99).
 * seq_starts != NULL selects the packed form of cuda_train_cross_entropy_grad_packed
 * (include/cuda_train_context.h:288): the last token of every sequence gives a zero row.
 * valid_rows is the divisor (0 -> all gradients 0).  grad may alias logits. */
int seraph_cross_entropy_grad(const float* logits, const uint32_t* targets, float* grad, float* loss_rows,
                              const uint32_t* seq_starts, int batch,
                              int64_t rows, int64_t cols, int64_t valid_rows, seraph_stream_t s);

/* Rows beyond 32768 columns are shared out between workgroups that exchange their partial (max, sum) through
 * device memory.  This bounds the wait for a partner, in polls of about 0.3 us (default 65536).  With 0 every
 * workgroup computes its partners' statistics itself, which is the path a workgroup takes when a partner has not
 * been scheduled: tests use it to run that path.  A negative value changes nothing.  No reference counterpart. */
void seraph_cross_entropy_exchange_spins(int spins);

/* ---------------------------------------------------------------- GEMM family */
/* vulkan_matmul (include/vulkan_backend.h:431-433, shaders/matmul.comp) and
 * vulkan_matmul_transpose (include/vulkan_backend.h:439-442, shaders/matmul_transpose.comp:35-169):
 * C[M,N] (+)= op(A) op(B); transposed A is stored [K,M], transposed B is stored [N,K]. */
int seraph_gemm(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                int transpose_A, int transpose_B, int accumulate, seraph_stream_t s);
/* Name of the kernel instantiation seraph_gemm launches for this shape with 16-byte aligned
 * operands, as a profiler prints it (no reference counterpart; used to label timings). */
const char* seraph_gemm_kernel_name(int64_t M, int64_t N, int64_t K, int transpose_A, int transpose_B);
/* Several products with the same K, orientations and accumulate flag in ONE launch: the q / k / v (or gate / up)
 * projections of a layer, which the reference issues back to back (src/train.c:4676-4681, :4718-4725), and their weight
 * gradients (:5143-5160, :5276-5300).  The tiles of all products form one grid, so products that are too small to
 * fill the chip share it.  At most 4 products; each is computed as seraph_gemm would (same tile kernel, chosen
 * for the group as a whole; a group that cannot share a launch is run as single seraph_gemm calls).  `problems`
 * is a HOST array.  The outputs must not overlap. */
typedef struct { const float* A; const float* B; float* C; int64_t M, N; } seraph_gemm_problem_t;
int seraph_gemm_grouped(const seraph_gemm_problem_t* problems, int count, int64_t K,
                        int transpose_A, int transpose_B, int accumulate, seraph_stream_t s);
const char* seraph_gemm_grouped_kernel_name(const seraph_gemm_problem_t* problems, int count, int64_t K,
                                            int transpose_A, int transpose_B);

/* C (+)= op(A_0) op(B_0) + op(A_1) op(B_1) (+ op(A_2) op(B_2)): products that share M, N and the orientations but not K,
 * as the input gradient of a layer's gate and up projections (src/train.c:5162-5179) or of q, k and v (:5294-5339), which
 * the reference forms as separate vulkan_matmul products joined by vulkan_add.  One launch (the sum forms in the accumulators and C is
 * written once) when every term suits the pipelined kernel, else one seraph_gemm per term.  count 1..3. */
typedef struct { const float* A; const float* B; int64_t K; } seraph_gemm_term_t;
int seraph_gemm_chain(const seraph_gemm_term_t* terms, int count, float* C, int64_t M, int64_t N,
                      int transpose_A, int transpose_B, int accumulate, seraph_stream_t s);
const char* seraph_gemm_chain_kernel_name(const seraph_gemm_term_t* terms, int count, const float* C, int64_t M, int64_t N,
                                          int transpose_A, int transpose_B);
/* C (+)= alpha * op(A) op(B): the step "product, then vulkan_scale of the product" of the LoRA path
 * (src/train.c:5778-5796, :5803-5845) as one call.  With the scratch of seraph_gemm_scaled_ws_bytes a small
 * output with a long K is cut into runs of K that separate workgroups take and a second kernel adds in run
 * order (deterministic); without it, or for other shapes, it is seraph_gemm followed by seraph_scale.
 * accumulate with alpha != 1 needs the scratch path.  No reference counterpart as a single op. */
size_t seraph_gemm_scaled_ws_bytes(int64_t M, int64_t N, int64_t K, int transpose_A, int transpose_B);
int seraph_gemm_scaled(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                       int transpose_A, int transpose_B, int accumulate, float alpha,
                       void* ws, size_t ws_bytes, seraph_stream_t s);

/* Several such products in one launch each: the rank-sized products of the LoRA adapters of a layer (four adapters
 * times x A^T, then B^T onto the output, and three gradient products each: src/train.c:5778-5845 runs them one by one).
 * The products share the orientations, alpha and the accumulate flag, not their shapes.  Every product is computed
 * exactly as seraph_gemm_scaled computes it alone (same runs of K, same order of additions); a list that cannot share
 * launches is run as single calls.  `problems` is a HOST array of at most 4; the outputs must not overlap; the scratch
 * holds the runs of all products at once. */
typedef struct { const float* A; const float* B; float* C; int64_t M, N, K; } seraph_gemm_scaled_problem_t;
size_t seraph_gemm_scaled_grouped_ws_bytes(const seraph_gemm_scaled_problem_t* problems, int count, int transpose_A, int transpose_B);
int seraph_gemm_scaled_grouped(const seraph_gemm_scaled_problem_t* problems, int count, int transpose_A, int transpose_B,
                               int accumulate, float alpha, void* ws, size_t ws_bytes, seraph_stream_t s);

/* ---------------------------------------------------------------- attention */
/* vulkan_batch_attention (include/vulkan_backend.h:485-488, shaders/batch_attention_stream.comp)
 * and cuda_train_batch_attention_packed (include/cuda_train_context.h:273): causal, GQA,
 * block-diagonal over packed sequences; lse (optional, [T,H]) = logsumexp of the scaled scores. */
int seraph_attention_forward(const float* Q, const float* K, const float* V, float* out, float* lse,
                             const uint32_t* seq_starts, int batch, int64_t T,
                             int heads, int kv_heads, int head_dim, float scale, seraph_stream_t s);
/* vulkan_batch_attention_backward (include/vulkan_backend.h:566-572;
 * shaders/batch_attention_backward.comp:50-196 and ..._stream.comp:34-202, no sequence cap) and
 * cuda_train_batch_attention_backward_packed (include/cuda_train_context.h:285).
 * attn_out and lse are optional saved forward results; when either is NULL both are
 * recomputed from Q, K, V.  dQ is overwritten; dK/dV are ADDED into (the caller zeroes
 * them first, src/train.c:5221-5222).  Deterministic: no atomics. */
size_t seraph_attention_backward_ws_bytes(int64_t T, int heads, int kv_heads, int head_dim);
int seraph_attention_backward(const float* Q, const float* K, const float* V, const float* dO,
                              const float* attn_out, const float* lse,
                              float* dQ, float* dK, float* dV,
                              const uint32_t* seq_starts, int batch, int64_t T,
                              int heads, int kv_heads, int head_dim, float scale,
                              void* ws, size_t ws_bytes, seraph_stream_t s);

/* The same backward with a bound on the length of any packed sequence.  When the scratch holds
 * seraph_attention_backward_ws_bytes_banded(...) bytes, the dK/dV pass leaves dS behind in a band of
 * 32x32 tiles (heads x ceil(T/32) x (ceil(max_seq_len/32)+1) x 4 KiB) and dQ is one product over it:
 * 5 matrix products instead of 7.  With the smaller scratch of seraph_attention_backward_ws_bytes the
 * call is identical to seraph_attention_backward.  max_seq_len <= 0 means T.  The bound is checked on the
 * device against seq_starts: when some sequence is longer than max_seq_len the band is left unread and dQ
 * comes from the recomputing kernel, so the results stay correct and only the saving is lost.
 * Same reference ops as seraph_attention_backward. */
size_t seraph_attention_backward_ws_bytes_banded(int64_t T, int heads, int kv_heads, int head_dim, int64_t max_seq_len);
int seraph_attention_backward_banded(const float* Q, const float* K, const float* V, const float* dO,
                                     const float* attn_out, const float* lse,
                                     float* dQ, float* dK, float* dV,
                                     const uint32_t* seq_starts, int batch, int64_t T,
                                     int heads, int kv_heads, int head_dim, float scale, int64_t max_seq_len,
                                     void* ws, size_t ws_bytes, seraph_stream_t s);

/* The form a step driver wants: dK and dV are ASSIGNED (no zero fill before the call; their old contents are not read),
 * and the longest sequence comes from host_seq_starts, the host's copy of the batch + 1 offsets that seq_starts holds on
 * the device (NULL with seq_starts NULL: one sequence of T).  The dS band is then sized by a bound that cannot fail:
 * scratch of seraph_attention_backward_ws_bytes_banded(T, ..., longest sequence) bytes selects the 5-product path, with no
 * stand-by launch.  Offsets that do not run from 0 to T without decreasing are an error.  Otherwise as
 * seraph_attention_backward_banded; results are bit-identical to it on zeroed dK / dV. */
int seraph_attention_backward_assign(const float* Q, const float* K, const float* V, const float* dO,
                                     const float* attn_out, const float* lse,
                                     float* dQ, float* dK, float* dV,
                                     const uint32_t* seq_starts, const uint32_t* host_seq_starts, int batch, int64_t T,
                                     int heads, int kv_heads, int head_dim, float scale,
                                     void* ws, size_t ws_bytes, seraph_stream_t s);

/* ---------------------------------------------------------------- norm / position */
/* vulkan_rmsnorm, include/vulkan_backend.h:499-503 (shaders/rmsnorm.comp) */
int seraph_rmsnorm(const float* x, const float* scale, float* y, int64_t rows, int64_t cols, float eps,
                   seraph_stream_t s);
/* sum = x + addend, y = rmsnorm(sum): the vulkan_add that closes a residual branch and the vulkan_rmsnorm
 * that opens the next one (src/train.c:4705-4711; :4737 with the next layer's :4668) in one pass.  sum is a
 * buffer of its own.  addend == NULL and sum == NULL: seraph_rmsnorm. */
int seraph_add_rmsnorm(const float* x, const float* addend, float* sum, const float* scale, float* y,
                       int64_t rows, int64_t cols, float eps, seraph_stream_t s);
/* vulkan_rmsnorm_backward_batch, include/vulkan_backend.h:552-558
 * (shaders/rmsnorm_backward_batch.comp:34-100): FP64 intermediates, rms floor 0.01,
 * grad_scale accumulated (+=) with a deterministic two-stage column reduction. */
size_t seraph_rmsnorm_backward_ws_bytes(int64_t rows, int64_t cols);
int seraph_rmsnorm_backward(const float* x, const float* scale, const float* dy, float* dx, float* grad_scale,
                            int64_t rows, int64_t cols, float eps, void* ws, size_t ws_bytes, seraph_stream_t s);
/* The same with dx = residual + (the RMSNorm input gradient): the vulkan_add that follows every
 * vulkan_rmsnorm_backward_batch of a layer (src/train.c:5180-5193, :5342-5355) folded into the store.
 * residual may be dx itself (in place) or NULL (then it is seraph_rmsnorm_backward). */
int seraph_rmsnorm_backward_residual(const float* x, const float* scale, const float* dy, const float* residual, float* dx,
                                     float* grad_scale, int64_t rows, int64_t cols, float eps, void* ws, size_t ws_bytes,
                                     seraph_stream_t s);
/* seraph_rmsnorm_backward_residual in two halves, for a step driver whose norms are small enough that the launch of
 * each column sum counts (the 2 L + 1 vulkan_rmsnorm_backward_batch calls of src/train.c:5071-5355): the row pass
 * completes dx and leaves *nparts partial rows of cols floats at the start of ws; seraph_rmsnorm_colsum_multi later
 * adds the column sums of any number of such passes of one width into their grad_scale in one launch, each summed in
 * the order seraph_rmsnorm_backward_residual uses, so the results are the same bits.  ws must stay untouched between
 * the two calls; `jobs` is a HOST array.  A caller that has no use for grad_scale (frozen norms) calls the row pass
 * alone. */
int seraph_rmsnorm_backward_rows(const float* x, const float* scale, const float* dy, const float* residual, float* dx,
                                 int64_t rows, int64_t cols, float eps, void* ws, size_t ws_bytes, int* nparts,
                                 seraph_stream_t s);
typedef struct { const float* partial; int nparts; float* grad_scale; } seraph_colsum_job_t;
int seraph_rmsnorm_colsum_multi(const seraph_colsum_job_t* jobs, int count, int64_t cols, seraph_stream_t s);
/* seraph_rmsnorm_backward_residual for callers that cannot allocate device memory or bring a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The partial rows of the column reduction live in an array built into the
 * library (seraph_rmsnorm_backward_static_max_bytes() = 16 MiB on every GPU the library runs on, held until
 * the process ends); the call allocates nothing.  The requirement is that of the kernel the operands
 * select: 16-byte aligned rows of 516 to 8192 columns write one partial row per workgroup (two workgroups
 * per compute unit: 16384 x 2048 needs 4 MiB, and such rows fit at any row count), aligned rows of up to
 * 512 columns likewise, anything else one partial row per wavefront.  A call that needs more is refused
 * with SERAPH_ERR_WORKSPACE before anything is touched.  Results are bit-identical to the workspace form.  Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race. */
size_t seraph_rmsnorm_backward_static_max_bytes(void);
int seraph_rmsnorm_backward_static(const float* x, const float* scale, const float* dy, const float* residual, float* dx,
                                   float* grad_scale, int64_t rows, int64_t cols, float eps, seraph_stream_t s);
/* vulkan_rope / vulkan_rope_backward, include/vulkan_backend.h:493-495,561-563
 * (shaders/rope.comp, rope_backward.comp:26-59) and the packed forms
 * (include/cuda_train_context.h:275,286).  in and out may alias.  backward != 0 applies
 * the inverse rotation. */
int seraph_rope(const float* in, float* out, const uint32_t* seq_starts, int batch, int64_t T,
                int heads, int head_dim, float theta, int backward, seraph_stream_t s);
/* The query and the key heads of the same tokens in one launch (the trainer rotates both back to
 * back, src/train.c:4700-4704, :5252-5262): identical results to two seraph_rope calls. */
int seraph_rope_qk(const float* q_in, float* q_out, int q_heads, const float* k_in, float* k_out, int k_heads,
                   const uint32_t* seq_starts, int batch, int64_t T, int head_dim, float theta, int backward,
                   seraph_stream_t s);
/* vulkan_qk_norm, include/vulkan_backend.h:600-603 (shaders/qk_norm.comp:30-76): in place,
 * no-op when use_qk_norm == 0.  The backward has no reference counterpart. */
int seraph_qk_norm(float* qk, int64_t T, int heads, int head_dim, int use_qk_norm, float eps, seraph_stream_t s);
int seraph_qk_norm_backward(const float* x_pre, const float* dy, float* dx, int64_t T, int heads, int head_dim,
                            float eps, seraph_stream_t s);
/* The pair a training step uses: the forward (always applied) also leaves each token's unclamped root mean square in
 * rms_out [T] (NULL: not wanted), and the backward works from the normalised output y, which the step keeps for the
 * attention anyway, and that rms: dx = (dy - y (dy.y)/n) / rms, or dy/eps where the forward clamped.  dx may be dy.
 * Same derivative as seraph_qk_norm_backward; no reference counterpart (the reference treats qk_norm as the identity
 * in its backward, src/train.c:5224-5266). */
int seraph_qk_norm_saved(float* qk, float* rms_out, int64_t T, int heads, int head_dim, float eps, seraph_stream_t s);
int seraph_qk_norm_backward_saved(const float* y, const float* rms, const float* dy, float* dx, int64_t T, int heads,
                                  int head_dim, float eps, seraph_stream_t s);

/* ---------------------------------------------------------------- element-wise */
/* vulkan_silu, include/vulkan_backend.h:476-478 (shaders/silu.comp) */
int seraph_silu(const float* x, float* y, size_t n, seraph_stream_t s);
/* vulkan_silu_backward, include/vulkan_backend.h:582-586 (shaders/silu_backward.comp:26-41); dx may alias dy */
int seraph_silu_backward(const float* x, const float* dy, float* dx, size_t n, seraph_stream_t s);
/* vulkan_elementwise_mul_backward, include/vulkan_backend.h:591-597 (shaders/elementwise_mul_backward.comp:24-35) */
int seraph_mul_backward(const float* A, const float* B, const float* dC, float* dA, float* dB, size_t n,
                        seraph_stream_t s);
/* The pair above fused as src/train.c:5131-5140 composes it, in one pass and without the
 * cached silu(gate): dUp = dH*silu(gate), dGate = dH*up*silu'(gate). */
int seraph_swiglu_backward(const float* gate, const float* up, const float* dH, float* dGate, float* dUp,
                           size_t n, seraph_stream_t s);
/* silu.comp then mul.comp in one pass (src/train.c:4726-4732): out = silu(gate)*up */
int seraph_swiglu(const float* gate, const float* up, float* out, size_t n, seraph_stream_t s);

/* ---------------------------------------------------------------- embedding */
/* vulkan_embed_lookup, include/vulkan_backend.h:531-535 (shaders/embed_lookup.comp) */
int seraph_embed_lookup(const uint32_t* tokens, const float* embed, float* out,
                        int64_t T, int64_t hidden, int64_t vocab, seraph_stream_t s);
/* vulkan_embedding_backward, include/vulkan_backend.h:575-579 (shaders/embedding_backward.comp:22-44):
 * grad_embed[tok[p]] += dH[p], ids >= vocab skipped.  Deterministic: positions are grouped
 * by token and each touched row is summed in position order by one workgroup. */
size_t seraph_embedding_backward_ws_bytes(int64_t T, int64_t vocab);
int seraph_embedding_backward(const uint32_t* tokens, const float* dH, float* grad_embed,
                              int64_t T, int64_t hidden, int64_t vocab,
                              void* ws, size_t ws_bytes, seraph_stream_t s);

/* ---------------------------------------------------------------- optimizer */
/* vulkan_adamw_update, include/vulkan_backend.h:445-452 (shaders/adamw.comp:36-61); bias
 * corrections 1-powf(beta,step) on the host as src/vulkan_backend.c:2151-2152.
 * clip <= 0: the reference formula.  clip > 0: each gradient element is first clamped to
 * [-clip, clip] (an extension; the reference never clips). */
int seraph_adamw(float* w, const float* g, float* m, float* v, size_t n,
                 float lr, float beta1, float beta2, float weight_decay, float eps, int step, float clip,
                 seraph_stream_t s);

/* The same update for a list of tensors in one launch (48 per launch for longer lists): the reference records one
 * vulkan_adamw_update and one barrier per tensor, 2 + 9 L of them per optimizer step (src/train.c:4225-4284).
 * `tensors` is a HOST array; the descriptors travel as kernel arguments.  Every element receives exactly the
 * arithmetic of seraph_adamw, so the results are bit-identical to per-tensor calls.  Tensors must not overlap. */
typedef struct { float* w; const float* g; float* m; float* v; size_t n; } seraph_adamw_tensor_t;
int seraph_adamw_multi(const seraph_adamw_tensor_t* tensors, int count,
                       float lr, float beta1, float beta2, float weight_decay, float eps, int step, float clip,
                       seraph_stream_t s);

#ifdef __cplusplus
}
#endif
#endif
