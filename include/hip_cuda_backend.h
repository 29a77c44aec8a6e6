/*
 * hip_cuda_backend.h - entry points of seraph_amd/seraph_tree/hip_cuda_backend.c.
 *
 * That file defines, over include/seraph_hip.h, the functions Seraph declares for its CUDA
 * training backend.  Their prototypes are Seraph's own (this header includes them, so it is usable
 * only with a Seraph tree on the include path); the reference file:line each one replaces:
 *
 *   context      cuda_train_init, _free, _sync, _get_gpu_info       include/cuda_train_context.h:239-242
 *                                                                     (src/cuda_train_context.cu:2246-2566)
 *   buffers      cuda_train_buffer_create, _free, _upload, _upload_u32, _download, _download_bytes,
 *                cuda_train_fill_buffer, _fill_buffer_range, cuda_train_copy_buffer
 *                                                                     :248-256 (.cu:2568-2638)
 *   forward      cuda_train_matmul, _matmul_transpose, _silu, _rmsnorm, _rope, _rope_packed, _add, _mul,
 *                _scale, _batch_attention, _batch_attention_packed, _embed_lookup
 *                                                                     :263-275 (.cu:2697-2941)
 *   loss/bwd     cuda_train_cross_entropy_grad, _cross_entropy_grad_packed, _reduce_sum, _silu_backward,
 *                _elementwise_mul_backward, _rmsnorm_backward_batch, _rope_backward, _rope_backward_packed,
 *                _batch_attention_backward, _batch_attention_backward_packed, _embedding_backward
 *                                                                     :278-288 (.cu:2943-3201)
 *   optimizer    cuda_train_adamw_update                              :291 (.cu:3203-3226)
 *   debug        cuda_train_nan_check, cuda_train_set_profiler        :294-299 (.cu:20, :3228-3234)
 *   LoRA         cuda_train_lora_backward, cuda_train_zero_lora_grads, cuda_download_lora_weights
 *                                                                     :309-325 (.cu:3240-3361)
 *   profiler     cuda_profiler_create, _destroy, _enable, _disable, _reset, _begin_op, _end_op, _set_launch,
 *                _set_flops, _set_bytes, _sync_and_analyze, _print, _print_top, _set_log
 *                                                                     include/cuda_profiler.h:53-84
 *                                                                     (src/cuda_profiler.cu:26-325)
 *
 * cuda_train_softmax (include/cuda_train_context.h:267) is declared by Seraph but called by none of
 * its sources; it is not provided.
 */
#ifndef HIP_CUDA_BACKEND_H
#define HIP_CUDA_BACKEND_H

#include "cuda_train_context.h"
#include "cuda_profiler.h"

#endif
