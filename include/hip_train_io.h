/*
 * hip_train_io.h - the data formats either side of the training step: token files, model
 * directories, checkpoints.  Host C, no GPU call in this file's functions except through
 * the hip_trainer_* transfers they are handed.
 *
 * Every reader accepts exactly what the reference's reader accepts and every writer produces
 * files the reference's readers load:
 *   .ttok token files        src/train.c:812-863 (reader), tools/tokenize_dataset.c:113 (writer)
 *   packed batches           tools/seraph_train_cuda.c:370-402
 *   fixed windows            src/train.c:7242-7264
 *   config.json              src/model_config.c:200-330
 *   model weights            src/train.c:282-432 (BF16 safetensors -> FP32), names src/train.c:340-422,
 *                            prefix stripping src/transformer.c:353-389
 *   full-weight checkpoints  src/train.c:433-560 (writer), :562-625 (reader), sidecar :7791-7802
 *   LoRA adapter files       src/lora.c:441-494 (writer), :496-566 (reader)
 */
#ifndef HIP_TRAIN_IO_H
#define HIP_TRAIN_IO_H

#include <stddef.h>
#include <stdint.h>

#include "hip_train.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------- token files */
#define HIP_TTOK_MAGIC 0x544F4B54u   /* "TTOK", src/train.c:20 */

typedef struct {
    int32_t* tokens;        /* all samples back to back */
    int32_t* offsets;       /* [num_samples + 1] */
    int32_t  num_samples;
    int32_t  num_tokens;
    uint32_t version;       /* header[1] */
    uint32_t vocab_size;    /* header[3], informational (tools/tokenize_dataset.c:113) */
} hip_ttok_t;

/* header u32[4] = {magic, version, num_samples, vocab}; then per sample u32 n and n int32 ids.
 * Returns 0, or -1 with the reason on stderr (missing file, bad magic, truncated data). */
int  hip_ttok_load(const char* path, hip_ttok_t* out);
void hip_ttok_free(hip_ttok_t* d);
int  hip_ttok_write(const char* path, const int32_t* tokens, const int32_t* offsets, int32_t num_samples,
                    uint32_t vocab_size);

/* Training units: each sample truncated to max_seq_len (fixed_windows = 0), or every full
 * max_seq_len window of every sample with remainders dropped (fixed_windows = 1).  Allocates
 * *starts and *lengths (free() them); returns the unit count or -1. */
int hip_ttok_units(const hip_ttok_t* d, int max_seq_len, int fixed_windows, int32_t** starts, int32_t** lengths);

/* Gathers up to batch_size units from *unit_idx on into one contiguous stream: units shorter
 * than 2 tokens are skipped, longer than max_seq_len truncated; seq_starts[0..count] is the
 * prefix sum.  Advances *unit_idx past everything consumed; returns the number of sequences
 * packed (0 = nothing left). */
int hip_pack_batch(const int32_t* tokens, const int32_t* unit_starts, const int32_t* unit_lengths, int num_units,
                   int* unit_idx, int batch_size, int max_seq_len,
                   int32_t* packed, int32_t* seq_starts, int* total_tokens);

/* ---------------------------------------------------------------- model directory */
/* Reads <model_dir>/config.json with the reference's keys, nesting ("text_config",
 * "rope_parameters") and defaults.  rms_eps is set to the file's rms_norm_eps; the reference's
 * training step ignores it and uses 1e-5 (src/train.c:4378), which is the caller's choice here.
 * lora_* fields are left 0. */
int hip_model_config_load(const char* model_dir, hip_model_config_t* cfg);

/* A sink receives `count` converted floats for arena offset `offset`; a source fills them. */
typedef int (*hip_arena_put_fn)(void* user, int64_t offset, const float* data, int64_t count);
typedef int (*hip_arena_get_fn)(void* user, int64_t offset, float* data, int64_t count);

/* Loads every tensor of the model from <path>: a directory holding model.safetensors or
 * model-0000i-of-0000N.safetensors shards, or one .safetensors file.  Tensors are found by name
 * after stripping any prefix in front of the last "model." component; BF16, F16 and F32 are
 * widened to FP32.  An embedding with fewer rows than cfg->vocab gets the remaining rows from the
 * reference's seeded He initialisation (src/train.c:318-332).  Tensors absent from the files stay
 * untouched (the reference leaves them zero) and are counted in *missing.  Returns 0 or -1. */
int hip_weights_load(const char* path, const hip_model_config_t* cfg, hip_arena_put_fn put, void* user, int* missing);
int hip_weights_load_host(const char* path, const hip_model_config_t* cfg, float* arena, int* missing);
int hip_trainer_load_weights(hip_trainer_t* t, const hip_model_config_t* cfg, const char* path, int* missing);

/* ---------------------------------------------------------------- checkpoints */
/* The reference's full-weight checkpoint: a safetensors file of BF16 tensors (FP32 truncated to
 * its upper 16 bits) in the order embed, per layer q k v o gate up down input_norm post_norm,
 * final norm, with the reference's metadata block.  The header carries the true shapes. */
int hip_checkpoint_save(const char* path, const hip_model_config_t* cfg, hip_arena_get_fn get, void* user);
int hip_checkpoint_save_host(const char* path, const hip_model_config_t* cfg, const float* arena);
int hip_trainer_save_checkpoint(hip_trainer_t* t, const hip_model_config_t* cfg, const char* path);
/* Reads such a file the way the reference does: header skipped, tensors taken in file order. */
int hip_checkpoint_load(const char* path, const hip_model_config_t* cfg, hip_arena_put_fn put, void* user);
int hip_checkpoint_load_host(const char* path, const hip_model_config_t* cfg, float* arena);
int hip_trainer_load_checkpoint(hip_trainer_t* t, const hip_model_config_t* cfg, const char* path);

/* "<checkpoint>.state": int epoch, int step, float loss, int optimizer_step (src/train.c:7791-7802). */
typedef struct { int32_t epoch, step; float loss; int32_t optimizer_step; } hip_train_state_file_t;
int hip_train_state_save(const char* checkpoint_path, const hip_train_state_file_t* st);
int hip_train_state_load(const char* checkpoint_path, hip_train_state_file_t* st);

/* Exact resume, which the reference cannot do (it keeps neither FP32 weights nor Adam moments):
 * "<checkpoint>.optim" holds the FP32 parameter arena and both moments (full-weight mode) or the
 * adapter arena and its moments (LoRA mode) as three F32 safetensors tensors "params", "adam.m",
 * "adam.v".  Load returns 1 when the file does not exist, 0 on success, -1 on error. */
int hip_trainer_save_optimizer_state(hip_trainer_t* t, const char* checkpoint_path);
int hip_trainer_load_optimizer_state(hip_trainer_t* t, const char* checkpoint_path);

/* ---------------------------------------------------------------- LoRA adapters */
/* Kaiming-normal A (std sqrt(2/in_dim), Marsaglia polar method over rand() after srand(seed)),
 * B = 0, adapters created per layer in the order q k v o gate up down - the draw sequence of
 * lora_model_create_from_config (src/lora.c:20-81, :372-396). */
int hip_lora_init(const hip_model_config_t* cfg, unsigned seed, float* lora_arena);

/* The reference's adapter file (version 2): header, then per layer the q and the v adapter
 * (A then B) when selected - the only two it persists.  Adapters on k, o, gate, up, down follow
 * in an appended block the reference's reader never reaches.  Load checks layers, rank and
 * dimensions against cfg and leaves adapters absent from the file untouched. */
int hip_lora_save(const char* path, const hip_model_config_t* cfg, const float* lora_arena);
int hip_lora_load(const char* path, const hip_model_config_t* cfg, float* lora_arena);

#ifdef __cplusplus
}
#endif
#endif
