/*
 * seraph-train-hip - batched training front end for one MI355X.
 *
 *   seraph-train-hip <model_dir> <train.ttok> [options]
 *
 * The counterpart of the reference's CUDA front end (tools/seraph_train_cuda.c): same
 * positional arguments, same options, same packing of samples into one contiguous token stream
 * per step (:370-402), the same log, validation and checkpoint lines and files
 * (train.log, checkpoint_N.safetensors / .bin with their .state sidecars, profile.log), so that
 * scripts and monitors written around that tool keep working.  What it drives is the packed
 * step of hip_train.h; what it reads and writes goes through hip_train_io.h.
 *
 * Not here: --bf16 and --flash (the step is FP32 and its attention is always the tiled
 * streaming kernel), gradient snapshots, video data.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <time.h>

#include "hip_train.h"
#include "hip_train_io.h"

typedef struct {
    const char* model_dir;
    const char* train_path;
    const char* val_path;
    const char* resume_path;
    const char* checkpoint_dir;
    int epochs, batch, max_seq, fixed_seq, accum;
    float lr;
    int full_training, lora_rank, lora_mask;
    float lora_alpha;
    int save_every, log_every, eval_every, eval_max_samples;
    float eval_split;
    int device, debug_nan_check, profile_steps, random_init, max_steps;
    unsigned seed;
    int seed_given;
} options_t;

static void usage(const char* prog) {
    printf("\nUsage: %s <model_dir> <train.ttok> [options]\n\n", prog);
    printf("Training Mode:\n");
    printf("  --full-training   Train all weights (FP32)\n");
    printf("  (default)         LoRA mode - train adapter weights only\n\n");
    printf("Options:\n");
    printf("  --resume PATH     Resume from checkpoint (e.g., checkpoints/checkpoint_5000.safetensors)\n");
    printf("  --epochs N        Number of epochs (default: 1)\n");
    printf("  --lr RATE         Learning rate (default: 1e-4)\n");
    printf("  --accum N         Gradient accumulation steps (default: 1)\n");
    printf("  --lora-rank N     LoRA rank (default: 8, LoRA mode only)\n");
    printf("  --lora-alpha F    LoRA alpha (default: 16.0, LoRA mode only)\n");
    printf("  --lora-targets S  Comma list of q,k,v,o,gate,up,down or ffn (default: q,v)\n");
    printf("  --max-seq N       Max sequence length (default: 512)\n");
    printf("  --fixed-seq       Fixed-length windows only\n");
    printf("  --save-every N    Save checkpoint every N steps (default: 1000)\n");
    printf("  --log-every N     Log every N steps (default: 100)\n");
    printf("  --checkpoint DIR  Checkpoint directory (default: ./checkpoints)\n");
    printf("  --gpu-device N    GPU index (default: 0)\n");
    printf("  --batch N         Sequences packed per step (default: 1)\n");
    printf("  --val PATH        Validation .ttok file\n");
    printf("  --eval-every N [M] [S]  Evaluate every N steps, max M samples, S = val split ratio\n");
    printf("  --debug-nan-check Check buffers for NaN/Inf and stop before the weights are poisoned\n");
    printf("  --profile N       Profile N training steps (per-kernel GPU timing), then exit\n");
    printf("  --random-init     Do not read model weights: N(0, 0.02) projections, unit norms (with --seed)\n");
    printf("  --seed N          Seed for adapter / random initialisation (default: time)\n");
    printf("  --max-steps N     Stop after N steps\n\n");
}

static double now_ms(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec * 1000.0 + (double)ts.tv_nsec / 1e6;
}

static int parse_targets(const char* s) {
    static const char* const names[7] = {"q", "k", "v", "o", "gate", "up", "down"};
    int mask = 0;
    char buf[128];
    snprintf(buf, sizeof(buf), "%s", s);
    for (char* tok = strtok(buf, ","); tok; tok = strtok(NULL, ",")) {
        int hit = 0;
        if (!strcmp(tok, "ffn")) { mask |= 0x70; hit = 1; }
        for (int i = 0; i < 7; i++) if (!strcmp(tok, names[i])) { mask |= 1 << i; hit = 1; }
        if (!hit) return -1;
    }
    return mask;
}

static int is_number(const char* s) { return s && s[0] >= '0' && s[0] <= '9'; }

static int parse_options(int argc, char** argv, options_t* o) {
    memset(o, 0, sizeof(*o));
    o->model_dir = argv[1];
    o->train_path = argv[2];
    o->checkpoint_dir = "./checkpoints";
    o->epochs = 1; o->batch = 1; o->max_seq = 512; o->accum = 1;
    o->lr = 1e-4f;
    o->lora_rank = 8; o->lora_alpha = 16.0f; o->lora_mask = 0x5;         /* q and v, src/lora.c:355-360 */
    o->save_every = 1000; o->log_every = 100; o->eval_max_samples = 32;
    for (int i = 3; i < argc; i++) {
        const char* a = argv[i];
        const int has = i + 1 < argc;
        if (!strcmp(a, "--epochs") && has) o->epochs = atoi(argv[++i]);
        else if (!strcmp(a, "--lr") && has) o->lr = (float)atof(argv[++i]);
        else if (!strcmp(a, "--accum") && has) o->accum = atoi(argv[++i]);
        else if (!strcmp(a, "--max-seq") && has) o->max_seq = atoi(argv[++i]);
        else if (!strcmp(a, "--fixed-seq")) o->fixed_seq = 1;
        else if (!strcmp(a, "--save-every") && has) o->save_every = atoi(argv[++i]);
        else if (!strcmp(a, "--log-every") && has) o->log_every = atoi(argv[++i]);
        else if (!strcmp(a, "--checkpoint") && has) o->checkpoint_dir = argv[++i];
        else if (!strcmp(a, "--full-training")) o->full_training = 1;
        else if (!strcmp(a, "--lora-rank") && has) o->lora_rank = atoi(argv[++i]);
        else if (!strcmp(a, "--lora-alpha") && has) o->lora_alpha = (float)atof(argv[++i]);
        else if (!strcmp(a, "--lora-targets") && has) {
            o->lora_mask = parse_targets(argv[++i]);
            if (o->lora_mask <= 0) { fprintf(stderr, "ERROR: --lora-targets takes q,k,v,o,gate,up,down,ffn\n"); return -1; }
        }
        else if (!strcmp(a, "--gpu-device") && has) o->device = atoi(argv[++i]);
        else if (!strcmp(a, "--batch") && has) {
            o->batch = atoi(argv[++i]);
            if (o->batch < 1) { fprintf(stderr, "ERROR: --batch must be >= 1\n"); return -1; }
        }
        else if (!strcmp(a, "--debug") || !strcmp(a, "--debug-nan-check")) o->debug_nan_check = 1;
        else if (!strcmp(a, "--debug-weight-delta") || !strcmp(a, "--flash")) { /* accepted, nothing to switch */ }
        else if (!strcmp(a, "--bf16")) fprintf(stderr, "WARNING: --bf16 is not available; training runs in FP32\n");
        else if (!strcmp(a, "--snapshot-every") && has) { i++; fprintf(stderr, "WARNING: gradient snapshots are not written by this tool\n"); }
        else if (!strcmp(a, "--resume") && has) o->resume_path = argv[++i];
        else if (!strcmp(a, "--val") && has) o->val_path = argv[++i];
        else if (!strcmp(a, "--eval-every") && has) {                     /* <steps> [max_samples] [split] */
            o->eval_every = atoi(argv[++i]);
            if (i + 1 < argc && is_number(argv[i + 1])) o->eval_max_samples = atoi(argv[++i]);
            if (i + 1 < argc && is_number(argv[i + 1])) o->eval_split = (float)atof(argv[++i]);
        }
        else if (!strcmp(a, "--profile") && has) o->profile_steps = atoi(argv[++i]);
        else if (!strcmp(a, "--random-init")) o->random_init = 1;
        else if (!strcmp(a, "--seed") && has) { o->seed = (unsigned)strtoul(argv[++i], NULL, 10); o->seed_given = 1; }
        else if (!strcmp(a, "--max-steps") && has) o->max_steps = atoi(argv[++i]);
        else { fprintf(stderr, "ERROR: unknown or incomplete option %s\n", a); return -1; }
    }
    if (o->epochs < 1 || o->max_seq < 2 || o->accum < 1) { fprintf(stderr, "ERROR: --epochs, --max-seq (>= 2) and --accum must be positive\n"); return -1; }
    if (!o->seed_given) o->seed = (unsigned)time(NULL);
    return 0;
}

/* both stdout and the run's log file */
static void log_line(FILE* log, const char* line) {
    fputs(line, stdout);
    if (log) { fputs(line, log); fflush(log); }
}

/* N(0, 0.02) projections and embedding, unit norm scales, drawn over rand() */
static int random_weights(hip_trainer_t* t, const hip_model_config_t* cfg, unsigned seed) {
    hip_param_layout_t L;
    hip_param_layout(cfg, &L);
    const int64_t chunk = (int64_t)1 << 20;
    float* buf = (float*)malloc((size_t)chunk * sizeof(float));
    if (!buf) return -1;
    srand(seed);
    int rc = 0;
    for (int64_t at = 0; at < L.count && !rc; at += chunk) {
        const int64_t n = L.count - at < chunk ? L.count - at : chunk;
        for (int64_t i = 0; i < n; i += 2) {
            const float u1 = ((float)rand() + 1.0f) / ((float)RAND_MAX + 2.0f), u2 = (float)rand() / (float)RAND_MAX;
            const float r = sqrtf(-2.0f * logf(u1)) * 0.02f;
            buf[i] = r * cosf(6.2831853f * u2);
            if (i + 1 < n) buf[i + 1] = r * sinf(6.2831853f * u2);
        }
        rc = hip_trainer_upload_at(t, 0, at, buf, n);
    }
    for (int64_t i = 0; i < cfg->hidden; i++) buf[i] = 1.0f;
    if (!rc) rc = hip_trainer_upload_at(t, 0, L.final_norm, buf, cfg->hidden);
    for (int l = 0; l < cfg->layers && !rc; l++) {
        const int64_t b = L.layer0 + L.layer_stride * l;
        rc = hip_trainer_upload_at(t, 0, b + L.in_norm, buf, cfg->hidden) || hip_trainer_upload_at(t, 0, b + L.post_norm, buf, cfg->hidden);
    }
    free(buf);
    return rc;
}

static int save_all(hip_trainer_t* t, const hip_model_config_t* cfg, const options_t* o, const char* stem,
                    const hip_train_state_file_t* st, FILE* log) {
    char path[1024], line[1200];
    if (o->full_training) {
        snprintf(path, sizeof(path), "%s/%s.safetensors", o->checkpoint_dir, stem);
        printf("    Converting FP32 -> BF16 and saving to %s\n", path);
        if (hip_trainer_save_checkpoint(t, cfg, path)) return -1;
    } else {
        snprintf(path, sizeof(path), "%s/%s.bin", o->checkpoint_dir, stem);
        const int64_t n = hip_lora_param_count(cfg);
        float* host = (float*)malloc((size_t)n * sizeof(float));
        if (!host || hip_trainer_download(t, 4, host, n) || hip_lora_save(path, cfg, host)) { free(host); return -1; }
        free(host);
        printf("  Saved LoRA weights: %s\n", path);
    }
    if (hip_train_state_save(path, st) == 0) printf("  Saved training state: %s.state\n", path);
    if (hip_trainer_save_optimizer_state(t, path) == 0) printf("  Saved optimizer state: %s.optim\n", path);
    snprintf(line, sizeof(line), "  Saved checkpoint: %s\n", path);
    log_line(log, line);
    return 0;
}

static void print_profile(hip_trainer_t* t, FILE* plog, int step, int batch, int tokens, float loss, double step_ms) {
    hip_op_stat_t st[64];
    const int n = hip_trainer_op_stats(t, st, 64);
    double total = 0.0;
    for (int i = 0; i < n; i++) total += st[i].ms;
    FILE* outs[2] = {stdout, plog};
    for (int k = 0; k < 2; k++) {
        FILE* f = outs[k];
        if (!f) continue;
        if (batch > 1) fprintf(f, "\n  -- PROFILE STEP %d (batch=%d, packed_tokens=%d, loss=%.4f) --\n", step, batch, tokens, loss);
        else fprintf(f, "\n  -- PROFILE STEP %d (seq_len=%d, loss=%.4f) --\n", step, tokens, loss);
        fprintf(f, "  SERAPH STEP PROFILER (%d kernel classes, %.2f ms on the device, %.2f ms wall)\n\n", n, total, step_ms);
        fprintf(f, "  %-62s %8s %10s  %6s  %10s  %10s\n", "Kernel", "Launches", "Time (ms)", "%", "GFLOPS", "GB/s");
        for (int i = 0; i < n; i++) {
            const double ms = st[i].ms > 0 ? st[i].ms : 1e-9;
            fprintf(f, "  %-62.62s %8lld %10.3f  %5.1f%%  %10.1f  %10.1f\n", st[i].name, (long long)st[i].launches, st[i].ms,
                    total > 0 ? 100.0 * st[i].ms / total : 0.0, st[i].flops / ms * 1e-6, st[i].bytes / ms * 1e-6);
        }
        fflush(f);
    }
}

int main(int argc, char** argv) {
    if (argc < 3) { usage(argv[0]); return 1; }
    options_t o;
    if (parse_options(argc, argv, &o)) { usage(argv[0]); return 1; }
    setvbuf(stdout, NULL, _IOLBF, 0);

    printf("\n  SERAPH HIP TRAINING (MI355X)\n\n");
    printf("[1/5] Loading model configuration...\n");
    hip_model_config_t cfg;
    if (hip_model_config_load(o.model_dir, &cfg)) return 1;
    cfg.rms_eps = 1e-5f;                                                   /* the training step's constant, src/train.c:4378 */
    if (!o.full_training) { cfg.lora_rank = o.lora_rank; cfg.lora_alpha = o.lora_alpha; cfg.lora_mask = o.lora_mask; }
    printf("  Vocab %d, hidden %d, layers %d, ffn %d, heads %d/%d x %d, rope theta %.1f\n", cfg.vocab, cfg.hidden, cfg.layers,
           cfg.ffn, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.rope_theta);

    printf("[2/5] Loading training data...\n");
    hip_ttok_t data, val;
    memset(&val, 0, sizeof(val));
    if (hip_ttok_load(o.train_path, &data)) return 1;
    printf("  Loaded %d tokens across %d samples\n", data.num_tokens, data.num_samples);
    int num_samples = data.num_samples;
    const int32_t* val_tokens = NULL;
    const int32_t* val_offsets = NULL;
    int num_val_samples = 0, num_val_tokens = 0;
    if (o.val_path) {
        if (hip_ttok_load(o.val_path, &val) == 0) {
            val_tokens = val.tokens; val_offsets = val.offsets; num_val_samples = val.num_samples; num_val_tokens = val.num_tokens;
            printf("  Validation:     %d samples, %d tokens (%s)\n", num_val_samples, num_val_tokens, o.val_path);
        } else {
            fprintf(stderr, "WARNING: Could not load validation data: %s\n", o.val_path);
        }
    } else if (o.eval_split > 0.0f && o.eval_split < 1.0f && num_samples > 1) {   /* tools/seraph_train_cuda.c:289-306 */
        int split = (int)((float)num_samples * (1.0f - o.eval_split));
        if (split < 1) split = 1;
        if (split >= num_samples) split = num_samples - 1;
        num_val_samples = num_samples - split;
        val_offsets = data.offsets + split;
        val_tokens = data.tokens;
        num_val_tokens = data.num_tokens;
        num_samples = split;
        printf("  Val split:      %.0f%% -> %d train / %d val samples\n", o.eval_split * 100.0f, num_samples, num_val_samples);
    }
    hip_ttok_t train_view = data;
    train_view.num_samples = num_samples;
    int32_t *unit_starts = NULL, *unit_lengths = NULL;
    const int num_units = hip_ttok_units(&train_view, o.max_seq, o.fixed_seq, &unit_starts, &unit_lengths);
    if (num_units < 0) return 1;
    if (o.fixed_seq) printf("  Fixed-seq mode: %d windows of %d tokens\n", num_units, o.max_seq);

    printf("[3/5] Creating the trainer on GPU %d...\n", o.device);
    hip_optim_config_t opt = {o.lr, 0.9f, 0.999f, 0.01f, 1e-8f, 0.0f, 100, o.accum};   /* src/train.c:5449-5456 */
    hip_trainer_t* t = hip_trainer_create(&cfg, &opt, o.batch * o.max_seq, o.batch, o.device, NULL, NULL, NULL, NULL);
    if (!t) return 1;
    printf("  Device memory:  %.2f GB\n", (double)hip_trainer_device_bytes(t) / 1e9);

    printf("[4/5] Loading model weights...\n");
    if (o.random_init) {
        if (random_weights(t, &cfg, o.seed)) { fprintf(stderr, "ERROR: random initialisation failed\n"); return 1; }
        printf("  Random initialisation (seed %u)\n", o.seed);
    } else {
        int missing = 0;
        if (hip_trainer_load_weights(t, &cfg, o.model_dir, &missing)) return 1;
        if (missing) fprintf(stderr, "WARNING: %d model tensors were not found in %s and stay zero\n", missing, o.model_dir);
        printf("  Loaded %.2fM FP32 parameters\n", (double)hip_param_count(&cfg) / 1e6);
    }
    if (!o.full_training) {
        const int64_t n = hip_lora_param_count(&cfg);
        float* host = (float*)malloc((size_t)n * sizeof(float));
        if (!host || hip_lora_init(&cfg, o.seed, host) || hip_trainer_upload(t, 4, host, n)) { fprintf(stderr, "ERROR: adapter initialisation failed\n"); return 1; }
        free(host);
        printf("  LoRA adapters:  rank %d, alpha %.1f, mask 0x%x, %.2fM trainable parameters\n", cfg.lora_rank, cfg.lora_alpha,
               cfg.lora_mask, (double)n / 1e6);
    }
    if (o.debug_nan_check && hip_trainer_enable_nan_check(t, 1)) return 1;

    hip_train_state_file_t st = {0, 0, 0.0f, 0};
    if (o.resume_path) {                                                   /* src/train.c:7808-7846 */
        printf("\nResuming from checkpoint: %s\n", o.resume_path);
        int rc;
        if (o.full_training) rc = hip_trainer_load_checkpoint(t, &cfg, o.resume_path);
        else {
            const int64_t n = hip_lora_param_count(&cfg);
            float* host = (float*)malloc((size_t)n * sizeof(float));
            rc = (!host || hip_trainer_download(t, 4, host, n) || hip_lora_load(o.resume_path, &cfg, host) || hip_trainer_upload(t, 4, host, n)) ? -1 : 0;
            free(host);
        }
        if (rc) fprintf(stderr, "WARNING: Could not load checkpoint, starting fresh\n");
        else {
            if (hip_train_state_load(o.resume_path, &st) == 0) printf("  Loaded training state: %s.state\n", o.resume_path);
            else printf("  No training state found at %s.state (starting fresh)\n", o.resume_path);
            const int exact = hip_trainer_load_optimizer_state(t, o.resume_path);
            if (exact == 0) printf("  Loaded FP32 weights and Adam moments: %s.optim\n", o.resume_path);
            else if (exact < 0) fprintf(stderr, "WARNING: %s.optim could not be read; moments restart at zero\n", o.resume_path);
            hip_trainer_set_schedule(t, o.lr, st.optimizer_step, 0);
            printf("  Resuming from epoch %d, step %d, loss %.4f\n", st.epoch, st.step, st.loss);
        }
    }

    mkdir(o.checkpoint_dir, 0755);
    char path[1024], line[1024];
    snprintf(path, sizeof(path), "%s/train.log", o.checkpoint_dir);
    FILE* log = fopen(path, "a");
    FILE* plog = NULL;
    if (o.profile_steps > 0) {
        snprintf(path, sizeof(path), "%s/profile.log", o.checkpoint_dir);
        plog = fopen(path, "w");
        if (plog) fprintf(plog, "# HARDWARE gfx950 compute_units=256 wave_size=64 lds_per_cu=163840\n");
        hip_trainer_enable_op_timing(t, 1);
        printf("  Profiling:      %d steps -> %s\n", o.profile_steps, plog ? path : "stdout");
    }

    printf("[5/5] Training\n\n");
    printf("  Samples:        %d\n", num_samples);
    printf("  Total tokens:   %d\n", data.num_tokens);
    printf("  Epochs:         %d\n", o.epochs);
    printf("  Learning rate:  %.6f\n", o.lr);
    if (!o.full_training) { printf("  LoRA rank:      %d\n  LoRA alpha:     %.1f\n", cfg.lora_rank, cfg.lora_alpha); }
    else printf("  Training:       Full weights\n");
    if (o.batch > 1) printf("  Batch size:     %d\n", o.batch);
    printf("  Precision:      FP32\n");
    if (num_val_samples > 0) {
        printf("  Validation:     %d samples", num_val_samples);
        if (o.eval_every > 0) printf(" (every %d steps)", o.eval_every);
        printf("\n");
    }
    printf("\n");

    /* rolling loss over the logging window, tools/seraph_train_cuda.c:353-358, :483-491 */
    const int window = o.log_every > 0 ? o.log_every : 100;
    float* ring = (float*)calloc((size_t)window, sizeof(float));
    int32_t* packed = (int32_t*)malloc((size_t)o.batch * (size_t)o.max_seq * sizeof(int32_t));
    int32_t* seq_starts = (int32_t*)malloc(((size_t)o.batch + 1) * sizeof(int32_t));
    if (!ring || !packed || !seq_starts) { fprintf(stderr, "ERROR: out of memory\n"); return 1; }
    float ring_sum = 0.0f;
    int ring_pos = 0, ring_filled = 0, total_steps = 0, stop = 0, exit_code = 0;
    int current_step = st.step;
    float current_loss = st.loss, best_val = 0.0f;
    const int steps_per_epoch = (num_units + o.batch - 1) / o.batch;

    for (int epoch = st.epoch; epoch < o.epochs && !stop; epoch++) {
        float epoch_sum = 0.0f;
        int epoch_count = 0, unit = 0;
        printf("Epoch %d/%d\n", epoch + 1, o.epochs);
        for (;;) {
            int tokens = 0;
            const int count = hip_pack_batch(data.tokens, unit_starts, unit_lengths, num_units, &unit, o.batch, o.max_seq,
                                             packed, seq_starts, &tokens);
            if (count <= 0) break;
            const double t0 = now_ms();
            const int profiled = o.profile_steps > 0 && total_steps < o.profile_steps;
            if (profiled) hip_trainer_reset_op_stats(t);
            const float loss = o.full_training ? hip_train_step_full_batch(t, packed, tokens, seq_starts, count, 1)
                                               : hip_train_step_lora_batch(t, packed, tokens, seq_starts, count, 1);
            const double step_ms = now_ms() - t0;
            if (profiled) print_profile(t, plog, total_steps + 1, count, tokens, loss, step_ms);
            if (hip_trainer_nan_detected(t)) {                              /* tools/seraph_train_cuda.c:457-470 */
                fprintf(stderr, "\n[NAN] detected at step=%d tokens=%d (optimizer skipped)\n", current_step + 1, tokens);
                hip_trainer_nan_report(t, stderr);
                fprintf(stderr, "[FATAL] NaN detected at step %d - stopping training\n", current_step + 1);
                if (log) { fprintf(log, "[FATAL] NaN detected at step %d - stopping training\n", current_step + 1); fflush(log); }
                stop = 1; exit_code = 2;
                break;
            }
            if (loss < 0.0f) { fprintf(stderr, "ERROR: training step failed\n"); stop = 1; exit_code = 1; break; }
            const float tok_per_sec = (float)tokens / (float)(step_ms / 1000.0);
            epoch_sum += loss; epoch_count++;
            current_loss = loss; current_step++; total_steps++;
            ring_sum -= ring[ring_pos]; ring[ring_pos] = loss; ring_sum += loss;
            ring_pos = (ring_pos + 1) % window;
            if (!ring_filled && ring_pos == 0) ring_filled = 1;
            const int ring_count = ring_filled ? window : ring_pos;
            const float rolling = ring_count > 0 ? ring_sum / (float)ring_count : loss;

            if (o.log_every > 0 && total_steps % o.log_every == 0) {
                const float avg = epoch_sum / (float)epoch_count;
                if (count > 1)
                    printf("  Step %d/%d | Loss: %.4f | Avg: %.4f | PPL: %.1f | %.0f tok/s | batch=%d\n", total_steps,
                           steps_per_epoch * o.epochs, rolling, avg, expf(rolling), tok_per_sec, count);
                else
                    printf("  Step %d/%d | Loss: %.4f | Avg: %.4f | PPL: %.1f | %.0f tok/s\n", total_steps,
                           steps_per_epoch * o.epochs, rolling, avg, expf(rolling), tok_per_sec);
                if (log) {
                    fprintf(log, "  Step %d/%d | Loss: %.4f | Avg: %.4f | PPL: %.1f | %.0f tok/s\n", total_steps,
                            steps_per_epoch * o.epochs, rolling, avg, expf(rolling), tok_per_sec);
                    fflush(log);
                }
            }
            if (o.eval_every > 0 && num_val_samples > 0 && total_steps % o.eval_every == 0) {
                float ppl = 0.0f;
                const float vl = hip_evaluate(t, val_tokens, num_val_tokens, val_offsets, num_val_samples, o.max_seq,
                                              o.eval_max_samples, &ppl);
                snprintf(line, sizeof(line), "  [VAL] Step %d | Val Loss: %.4f | Val PPL: %.1f\n", total_steps, vl, ppl);
                log_line(log, line);
                if (vl > 0.0f && (best_val <= 0.0f || vl < best_val)) best_val = vl;
            }
            if (o.save_every > 0 && current_step % o.save_every == 0) {
                char stem[64];
                snprintf(stem, sizeof(stem), "checkpoint_%d", current_step);
                hip_train_state_file_t now = {epoch, current_step, current_loss, hip_trainer_optimizer_step(t)};
                if (save_all(t, &cfg, &o, stem, &now, log)) fprintf(stderr, "ERROR: could not save %s\n", stem);
            }
            if (o.profile_steps > 0 && total_steps >= o.profile_steps) {
                printf("\n  Profiling complete (%d steps). Exiting.\n\n", o.profile_steps);
                if (plog) fprintf(plog, "\n  Profiling complete (%d steps).\n\n", o.profile_steps);
                stop = 1;
                break;
            }
            if (o.max_steps > 0 && total_steps >= o.max_steps) { stop = 1; break; }
        }
        if (!stop || epoch_count > 0)
            printf("  Epoch %d complete | Avg Loss: %.4f\n\n", epoch + 1, epoch_count > 0 ? epoch_sum / (float)epoch_count : 0.0f);
        st.epoch = epoch;
    }

    if (exit_code == 0 && o.profile_steps == 0) {
        hip_train_state_file_t fin = {st.epoch, current_step, current_loss, hip_trainer_optimizer_step(t)};
        if (save_all(t, &cfg, &o, "checkpoint_final", &fin, log)) exit_code = 1;
        printf("  Final loss: %.4f\n", current_loss);
        if (best_val > 0.0f) printf("  Best val loss: %.4f\n", best_val);
    }
    if (plog) fclose(plog);
    if (log) fclose(log);
    free(ring); free(packed); free(seq_starts); free(unit_starts); free(unit_lengths);
    hip_ttok_free(&data);
    hip_ttok_free(&val);
    hip_trainer_free(t);
    printf("\n  SERAPH HIP TRAINING COMPLETE\n\n");
    return exit_code;
}
