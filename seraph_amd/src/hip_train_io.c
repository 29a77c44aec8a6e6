/*
 * hip_train_io.c - token files, model directories and checkpoints in the reference's formats
 * (see hip_train_io.h for the file:line of each format).  Plain host C.
 */
#define _FILE_OFFSET_BITS 64
#include <errno.h>
#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "hip_train_io.h"

#define IO_ERR(...) do { fprintf(stderr, "ERROR: " __VA_ARGS__); fputc('\n', stderr); } while (0)

/* ================================================================= a small JSON reader
 * Enough for config.json and safetensors headers: objects, arrays, strings (with escapes),
 * numbers, true/false/null.  Nodes form a first-child / next-sibling tree. */
typedef enum { J_NULL, J_BOOL, J_NUM, J_STR, J_ARR, J_OBJ } jtype_t;
typedef struct jnode {
    jtype_t type;
    double num;
    char* str;              /* J_STR value */
    char* key;              /* member name when the parent is an object */
    struct jnode* child;
    struct jnode* next;
} jnode_t;

typedef struct { const char* p; const char* end; int depth; int failed; } jparse_t;

static void json_free(jnode_t* n) {
    while (n) {
        jnode_t* nx = n->next;
        json_free(n->child);
        free(n->str);
        free(n->key);
        free(n);
        n = nx;
    }
}

static void j_ws(jparse_t* s) {
    while (s->p < s->end && (*s->p == ' ' || *s->p == '\t' || *s->p == '\n' || *s->p == '\r')) s->p++;
}

static char* j_string(jparse_t* s) {
    if (s->p >= s->end || *s->p != '"') { s->failed = 1; return NULL; }
    s->p++;
    size_t cap = 32, len = 0;
    char* out = (char*)malloc(cap);
    if (!out) { s->failed = 1; return NULL; }
    while (s->p < s->end && *s->p != '"') {
        unsigned cp = (unsigned char)*s->p++;
        if (cp == '\\') {
            if (s->p >= s->end) break;
            char e = *s->p++;
            switch (e) {
                case 'n': cp = '\n'; break;
                case 't': cp = '\t'; break;
                case 'r': cp = '\r'; break;
                case 'b': cp = '\b'; break;
                case 'f': cp = '\f'; break;
                case 'u': {
                    cp = 0;
                    for (int i = 0; i < 4 && s->p < s->end; i++) {
                        char c = *s->p++;
                        cp = cp * 16 + (unsigned)(c >= '0' && c <= '9' ? c - '0' : (c | 32) >= 'a' && (c | 32) <= 'f' ? (c | 32) - 'a' + 10 : 0);
                    }
                    break;
                }
                default: cp = (unsigned char)e; break;       /* \" \\ \/ */
            }
        }
        if (len + 5 > cap) {
            cap *= 2;
            char* grown = (char*)realloc(out, cap);
            if (!grown) { free(out); s->failed = 1; return NULL; }
            out = grown;
        }
        if (cp < 0x80) out[len++] = (char)cp;
        else if (cp < 0x800) { out[len++] = (char)(0xC0 | (cp >> 6)); out[len++] = (char)(0x80 | (cp & 0x3F)); }
        else { out[len++] = (char)(0xE0 | (cp >> 12)); out[len++] = (char)(0x80 | ((cp >> 6) & 0x3F)); out[len++] = (char)(0x80 | (cp & 0x3F)); }
    }
    if (s->p >= s->end) { free(out); s->failed = 1; return NULL; }
    s->p++;                                                   /* closing quote */
    out[len] = '\0';
    return out;
}

static jnode_t* j_value(jparse_t* s);

static jnode_t* j_container(jparse_t* s, int is_obj) {
    jnode_t* n = (jnode_t*)calloc(1, sizeof(*n));
    if (!n) { s->failed = 1; return NULL; }
    n->type = is_obj ? J_OBJ : J_ARR;
    const char close = is_obj ? '}' : ']';
    s->p++;
    jnode_t** tail = &n->child;
    j_ws(s);
    if (s->p < s->end && *s->p == close) { s->p++; return n; }
    while (!s->failed) {
        char* key = NULL;
        j_ws(s);
        if (is_obj) {
            key = j_string(s);
            j_ws(s);
            if (s->failed || s->p >= s->end || *s->p != ':') { free(key); s->failed = 1; break; }
            s->p++;
        }
        jnode_t* v = j_value(s);
        if (!v) { free(key); s->failed = 1; break; }
        v->key = key;
        *tail = v;
        tail = &v->next;
        j_ws(s);
        if (s->p < s->end && *s->p == ',') { s->p++; continue; }
        if (s->p < s->end && *s->p == close) { s->p++; return n; }
        s->failed = 1;
    }
    json_free(n);
    return NULL;
}

static jnode_t* j_value(jparse_t* s) {
    j_ws(s);
    if (s->p >= s->end || s->depth > 64) { s->failed = 1; return NULL; }
    const char c = *s->p;
    if (c == '{' || c == '[') {
        s->depth++;
        jnode_t* n = j_container(s, c == '{');
        s->depth--;
        return n;
    }
    jnode_t* n = (jnode_t*)calloc(1, sizeof(*n));
    if (!n) { s->failed = 1; return NULL; }
    if (c == '"') {
        n->type = J_STR;
        n->str = j_string(s);
        if (!n->str) { free(n); return NULL; }
        return n;
    }
    const size_t left = (size_t)(s->end - s->p);
    if (left >= 4 && !strncmp(s->p, "true", 4)) { n->type = J_BOOL; n->num = 1; s->p += 4; return n; }
    if (left >= 5 && !strncmp(s->p, "false", 5)) { n->type = J_BOOL; n->num = 0; s->p += 5; return n; }
    if (left >= 4 && !strncmp(s->p, "null", 4)) { n->type = J_NULL; s->p += 4; return n; }
    char buf[64];
    size_t k = 0;
    while (s->p + k < s->end && k + 1 < sizeof(buf) && strchr("+-0123456789.eE", s->p[k])) { buf[k] = s->p[k]; k++; }
    buf[k] = '\0';
    char* endp = NULL;
    n->num = strtod(buf, &endp);
    if (k == 0 || endp == buf) { free(n); s->failed = 1; return NULL; }
    n->type = J_NUM;
    s->p += (size_t)(endp - buf);
    return n;
}

static jnode_t* json_parse(const char* text, size_t len) {
    jparse_t s = {text, text + len, 0, 0};
    jnode_t* n = j_value(&s);
    if (s.failed) { json_free(n); return NULL; }
    return n;
}

static const jnode_t* j_get(const jnode_t* obj, const char* key) {
    if (!obj || obj->type != J_OBJ) return NULL;
    for (const jnode_t* c = obj->child; c; c = c->next) if (c->key && !strcmp(c->key, key)) return c;
    return NULL;
}
static int j_int(const jnode_t* obj, const char* key, int dflt) {
    const jnode_t* v = j_get(obj, key);
    return (v && v->type == J_NUM) ? (int)v->num : dflt;
}
static float j_float(const jnode_t* obj, const char* key, float dflt) {
    const jnode_t* v = j_get(obj, key);
    return (v && v->type == J_NUM) ? (float)v->num : dflt;
}

static char* read_text_file(const char* path, size_t* len) {
    FILE* f = fopen(path, "rb");
    if (!f) return NULL;
    fseeko(f, 0, SEEK_END);
    off_t n = ftello(f);
    fseeko(f, 0, SEEK_SET);
    char* buf = (n >= 0) ? (char*)malloc((size_t)n + 1) : NULL;
    if (buf && fread(buf, 1, (size_t)n, f) != (size_t)n) { free(buf); buf = NULL; }
    fclose(f);
    if (buf) { buf[n] = '\0'; *len = (size_t)n; }
    return buf;
}

/* ================================================================= token files */
int hip_ttok_load(const char* path, hip_ttok_t* out) {
    if (!path || !out) return -1;
    memset(out, 0, sizeof(*out));
    FILE* f = fopen(path, "rb");
    if (!f) { IO_ERR("Cannot open %s", path); return -1; }
    uint32_t header[4];
    if (fread(header, sizeof(uint32_t), 4, f) != 4) { IO_ERR("%s: short header", path); fclose(f); return -1; }
    if (header[0] != HIP_TTOK_MAGIC) { IO_ERR("Invalid .ttok file (bad magic)"); fclose(f); return -1; }
    const uint32_t declared = header[2];
    if (declared > 0x7FFFFFFEu) { IO_ERR("%s: sample count %u out of range", path, declared); fclose(f); return -1; }
    const off_t data_start = ftello(f);
    fseeko(f, 0, SEEK_END);
    const off_t file_end = ftello(f);
    fseeko(f, data_start, SEEK_SET);

    /* pass 1: sizes (src/train.c:833-840), checked against the file length */
    int64_t total = 0;
    off_t pos = data_start;
    for (uint32_t i = 0; i < declared; i++) {
        uint32_t n;
        if (fread(&n, sizeof(uint32_t), 1, f) != 1) { IO_ERR("%s: truncated at sample %u of %u", path, i, declared); fclose(f); return -1; }
        pos += 4 + (off_t)n * 4;
        if (pos > file_end) { IO_ERR("%s: sample %u (%u tokens) runs past the end of the file", path, i, n); fclose(f); return -1; }
        total += n;
        if (total > 0x7FFFFFFF) { IO_ERR("%s: more than 2^31-1 tokens", path); fclose(f); return -1; }
        fseeko(f, (off_t)n * 4, SEEK_CUR);
    }
    out->tokens = (int32_t*)malloc(((size_t)total + 1) * sizeof(int32_t));
    out->offsets = (int32_t*)malloc(((size_t)declared + 1) * sizeof(int32_t));
    if (!out->tokens || !out->offsets) { IO_ERR("out of memory for %lld tokens", (long long)total); fclose(f); hip_ttok_free(out); return -1; }

    /* pass 2: tokens (src/train.c:849-857) */
    fseeko(f, data_start, SEEK_SET);
    int32_t off = 0;
    for (uint32_t i = 0; i < declared; i++) {
        uint32_t n = 0;
        out->offsets[i] = off;
        if (fread(&n, sizeof(uint32_t), 1, f) != 1 || fread(out->tokens + off, sizeof(int32_t), n, f) != n) {
            IO_ERR("%s: read failed at sample %u", path, i);
            fclose(f); hip_ttok_free(out); return -1;
        }
        off += (int32_t)n;
    }
    out->offsets[declared] = off;
    out->num_samples = (int32_t)declared;
    out->num_tokens = off;
    out->version = header[1];
    out->vocab_size = header[3];
    fclose(f);
    return 0;
}

void hip_ttok_free(hip_ttok_t* d) {
    if (!d) return;
    free(d->tokens);
    free(d->offsets);
    memset(d, 0, sizeof(*d));
}

int hip_ttok_write(const char* path, const int32_t* tokens, const int32_t* offsets, int32_t num_samples, uint32_t vocab_size) {
    if (!path || !tokens || !offsets || num_samples < 0) return -1;
    FILE* f = fopen(path, "wb");
    if (!f) { IO_ERR("Cannot create %s", path); return -1; }
    uint32_t header[4] = {HIP_TTOK_MAGIC, 1u, (uint32_t)num_samples, vocab_size};     /* tools/tokenize_dataset.c:113 */
    int ok = fwrite(header, sizeof(uint32_t), 4, f) == 4;
    for (int32_t i = 0; ok && i < num_samples; i++) {
        const uint32_t n = (uint32_t)(offsets[i + 1] - offsets[i]);
        ok = fwrite(&n, sizeof(uint32_t), 1, f) == 1 && fwrite(tokens + offsets[i], sizeof(int32_t), n, f) == n;
    }
    if (fclose(f) != 0) ok = 0;
    return ok ? 0 : -1;
}

int hip_ttok_units(const hip_ttok_t* d, int max_seq_len, int fixed_windows, int32_t** starts, int32_t** lengths) {
    if (!d || !starts || !lengths || max_seq_len < 1) return -1;
    size_t cap = 0;
    if (fixed_windows) {
        for (int i = 0; i < d->num_samples; i++) cap += (size_t)((d->offsets[i + 1] - d->offsets[i]) / max_seq_len);
    } else {
        cap = (size_t)d->num_samples;
    }
    *starts = (int32_t*)malloc((cap + 1) * sizeof(int32_t));
    *lengths = (int32_t*)malloc((cap + 1) * sizeof(int32_t));
    if (!*starts || !*lengths) { free(*starts); free(*lengths); *starts = *lengths = NULL; return -1; }
    int n = 0;
    for (int i = 0; i < d->num_samples; i++) {
        const int32_t start = d->offsets[i], len = d->offsets[i + 1] - start;
        if (fixed_windows) {
            for (int w = 0; w < len / max_seq_len; w++) { (*starts)[n] = start + w * max_seq_len; (*lengths)[n] = max_seq_len; n++; }
        } else {
            (*starts)[n] = start;
            (*lengths)[n] = len > max_seq_len ? max_seq_len : len;
            n++;
        }
    }
    return n;
}

int hip_pack_batch(const int32_t* tokens, const int32_t* unit_starts, const int32_t* unit_lengths, int num_units,
                   int* unit_idx, int batch_size, int max_seq_len,
                   int32_t* packed, int32_t* seq_starts, int* total_tokens) {
    if (!tokens || !unit_starts || !unit_lengths || !unit_idx || !packed || !seq_starts || batch_size < 1) return -1;
    int count = 0, total = 0, i = *unit_idx;
    seq_starts[0] = 0;
    while (count < batch_size && i < num_units) {
        int len = unit_lengths[i];
        if (len > max_seq_len) len = max_seq_len;
        if (len < 2) { i++; continue; }                                  /* nothing to predict */
        memcpy(packed + total, tokens + unit_starts[i], (size_t)len * sizeof(int32_t));
        total += len;
        seq_starts[++count] = total;
        i++;
    }
    *unit_idx = i;
    if (total_tokens) *total_tokens = total;
    return count;
}

/* ================================================================= config.json */
int hip_model_config_load(const char* model_dir, hip_model_config_t* cfg) {
    if (!model_dir || !cfg) return -1;
    char path[1024];
    snprintf(path, sizeof(path), "%s/config.json", model_dir);
    size_t len = 0;
    char* text = read_text_file(path, &len);
    if (!text) { IO_ERR("Cannot read %s", path); return -1; }
    jnode_t* root = json_parse(text, len);
    free(text);
    if (!root || root->type != J_OBJ) { IO_ERR("Failed to parse config.json"); json_free(root); return -1; }
    const jnode_t* text_cfg = j_get(root, "text_config");                  /* src/model_config.c:232-233 */
    const jnode_t* src = (text_cfg && text_cfg->type == J_OBJ) ? text_cfg : root;
    memset(cfg, 0, sizeof(*cfg));
    cfg->vocab = j_int(src, "vocab_size", 32000);
    cfg->hidden = j_int(src, "hidden_size", 4096);
    cfg->layers = j_int(src, "num_hidden_layers", 32);
    cfg->ffn = j_int(src, "intermediate_size", 11008);
    cfg->heads = j_int(src, "num_attention_heads", 32);
    cfg->kv_heads = j_int(src, "num_key_value_heads", cfg->heads);
    const int explicit_hd = j_int(src, "head_dim", 0);
    cfg->head_dim = explicit_hd > 0 ? explicit_hd : (cfg->heads > 0 ? cfg->hidden / cfg->heads : 0);
    cfg->rms_eps = j_float(src, "rms_norm_eps", 1e-6f);
    cfg->rope_theta = j_float(src, "rope_theta", 0.0f);
    if (cfg->rope_theta == 0.0f) {                                         /* src/model_config.c:270-279 */
        const jnode_t* rp = j_get(src, "rope_parameters");
        cfg->rope_theta = rp ? j_float(rp, "rope_theta", 10000.0f) : 10000.0f;
    }
    cfg->use_qk_norm = j_int(src, "use_qk_norm", 0) ? 1 : 0;              /* src/model_config.c:282 */
    json_free(root);
    if (cfg->vocab < 1 || cfg->hidden < 1 || cfg->layers < 1 || cfg->ffn < 1 || cfg->heads < 1 || cfg->kv_heads < 1 || cfg->head_dim < 1) {
        IO_ERR("config.json holds a non-positive model dimension");
        return -1;
    }
    return 0;
}

/* ================================================================= safetensors files */
enum { ST_F32 = 0, ST_F16 = 1, ST_BF16 = 2, ST_OTHER = 3 };
typedef struct {
    char* name;             /* as in the file */
    const char* norm;       /* points into name: after the wrapper prefix */
    int dtype;
    int64_t count;
    size_t begin, end;      /* byte range inside the data section */
} st_entry_t;
typedef struct {
    void* map;
    size_t size, data_base;
    int n;
    st_entry_t* e;
} st_file_t;

static void st_close(st_file_t* f) {
    if (!f) return;
    for (int i = 0; i < f->n; i++) free(f->e[i].name);
    free(f->e);
    if (f->map && f->map != MAP_FAILED) munmap(f->map, f->size);
    memset(f, 0, sizeof(*f));
}

/* "language_model.model.layers.0..." -> "model.layers.0...": the last "model." that starts the
 * name or follows a dot (src/transformer.c:369-386) */
static const char* normalized_name(const char* name) {
    const char* best = NULL;
    const char* s = name;
    while ((s = strstr(s, "model.")) != NULL) {
        if (s == name || s[-1] == '.') best = s;
        s += 6;
    }
    return best ? best : name;
}

static int st_open(const char* path, st_file_t* f) {
    memset(f, 0, sizeof(*f));
    int fd = open(path, O_RDONLY);
    if (fd < 0) { IO_ERR("Cannot open %s", path); return -1; }
    struct stat sb;
    if (fstat(fd, &sb) != 0 || sb.st_size < 8) { IO_ERR("%s: not a safetensors file", path); close(fd); return -1; }
    f->size = (size_t)sb.st_size;
    f->map = mmap(NULL, f->size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (f->map == MAP_FAILED) { IO_ERR("%s: mmap failed: %s", path, strerror(errno)); f->map = NULL; return -1; }
    uint64_t hlen;
    memcpy(&hlen, f->map, 8);
    if (hlen > f->size - 8) { IO_ERR("%s: header length %llu exceeds the file", path, (unsigned long long)hlen); st_close(f); return -1; }
    f->data_base = 8 + (size_t)hlen;
    jnode_t* root = json_parse((const char*)f->map + 8, (size_t)hlen);
    if (!root || root->type != J_OBJ) { IO_ERR("%s: header is not a JSON object", path); json_free(root); st_close(f); return -1; }
    int n = 0;
    for (const jnode_t* c = root->child; c; c = c->next) n++;
    f->e = (st_entry_t*)calloc((size_t)n + 1, sizeof(st_entry_t));
    if (!f->e) { json_free(root); st_close(f); return -1; }
    for (const jnode_t* c = root->child; c; c = c->next) {
        if (!c->key || !strcmp(c->key, "__metadata__") || c->type != J_OBJ) continue;
        const jnode_t* dt = j_get(c, "dtype");
        const jnode_t* shape = j_get(c, "shape");
        const jnode_t* offs = j_get(c, "data_offsets");
        if (!dt || dt->type != J_STR || !offs || offs->type != J_ARR || !offs->child || !offs->child->next) continue;
        st_entry_t* e = &f->e[f->n];
        e->dtype = !strcmp(dt->str, "F32") ? ST_F32 : !strcmp(dt->str, "F16") ? ST_F16 : !strcmp(dt->str, "BF16") ? ST_BF16 : ST_OTHER;
        e->begin = (size_t)offs->child->num;
        e->end = (size_t)offs->child->next->num;
        if (e->end < e->begin || e->end > f->size - f->data_base) {
            IO_ERR("%s: tensor %s lies outside the file", path, c->key);
            json_free(root); st_close(f); return -1;
        }
        const size_t width = e->dtype == ST_F32 ? 4 : (e->dtype == ST_OTHER ? 1 : 2);
        e->count = (int64_t)((e->end - e->begin) / width);
        if (shape && shape->type == J_ARR) {                         /* the shape must agree with the byte range */
            int64_t prod = 1;
            for (const jnode_t* d = shape->child; d; d = d->next) prod *= (int64_t)d->num;
            if (e->dtype != ST_OTHER && prod != e->count) {
                IO_ERR("%s: tensor %s: shape (%lld elements) disagrees with its %zu bytes", path, c->key, (long long)prod, e->end - e->begin);
                json_free(root); st_close(f); return -1;
            }
        }
        e->name = strdup(c->key);
        if (!e->name) { json_free(root); st_close(f); return -1; }
        e->norm = normalized_name(e->name);
        f->n++;
    }
    json_free(root);
    return 0;
}

static const st_entry_t* st_find(const st_file_t* files, int nfiles, const char* name, const st_file_t** where) {
    for (int i = 0; i < nfiles; i++)
        for (int k = 0; k < files[i].n; k++)
            if (!strcmp(files[i].e[k].norm, name)) { *where = &files[i]; return &files[i].e[k]; }
    return NULL;
}

static inline float bf16_to_f32(uint16_t v) {
    uint32_t bits = (uint32_t)v << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
static inline uint16_t f32_to_bf16_trunc(float f) {                         /* src/train.c:262-266: truncation */
    uint32_t bits;
    memcpy(&bits, &f, 4);
    return (uint16_t)(bits >> 16);
}
static inline float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int shift = 0;
            while (!(man & 0x400u)) { man <<= 1; shift++; }
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
    else bits = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static void st_convert(const st_file_t* f, const st_entry_t* e, int64_t first, int64_t count, float* dst) {
    const char* base = (const char*)f->map + f->data_base + e->begin;
    if (e->dtype == ST_F32) memcpy(dst, base + first * 4, (size_t)count * 4);
    else {
        /* a safetensors header of odd length leaves 16-bit data at odd addresses: read through memcpy */
        const char* s = base + first * 2;
        for (int64_t i = 0; i < count; i++) {
            uint16_t h;
            memcpy(&h, s + 2 * i, 2);
            dst[i] = e->dtype == ST_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
        }
    }
}

/* ------------------------------------------------------------------ the model's tensor list */
typedef struct { char name[128]; int64_t offset, count, rows, cols; } tensor_slot_t;

/* In the reference's checkpoint order (src/train.c:470-506): embed, per layer q k v o gate up
 * down input_norm post_norm, final norm. */
static int tensor_slots(const hip_model_config_t* c, tensor_slot_t** out) {
    hip_param_layout_t L;
    hip_param_layout(c, &L);
    const int n = 2 + 9 * c->layers;
    tensor_slot_t* s = (tensor_slot_t*)calloc((size_t)n, sizeof(*s));
    if (!s) return -1;
    const int64_t h = c->hidden, qd = (int64_t)c->heads * c->head_dim, kv = (int64_t)c->kv_heads * c->head_dim, f = c->ffn;
    int k = 0;
#define SLOT(off, r, cc, ...) do { snprintf(s[k].name, sizeof(s[k].name), __VA_ARGS__); s[k].offset = (off); s[k].rows = (r); s[k].cols = (cc); \
                                   s[k].count = (int64_t)(r) * ((cc) > 0 ? (cc) : 1); k++; } while (0)
    SLOT(L.embed, c->vocab, h, "model.embed_tokens.weight");
    for (int l = 0; l < c->layers; l++) {
        const int64_t b = L.layer0 + L.layer_stride * l;
        SLOT(b + L.q, qd, h, "model.layers.%d.self_attn.q_proj.weight", l);
        SLOT(b + L.k, kv, h, "model.layers.%d.self_attn.k_proj.weight", l);
        SLOT(b + L.v, kv, h, "model.layers.%d.self_attn.v_proj.weight", l);
        SLOT(b + L.o, h, qd, "model.layers.%d.self_attn.o_proj.weight", l);
        SLOT(b + L.gate, f, h, "model.layers.%d.mlp.gate_proj.weight", l);
        SLOT(b + L.up, f, h, "model.layers.%d.mlp.up_proj.weight", l);
        SLOT(b + L.down, h, f, "model.layers.%d.mlp.down_proj.weight", l);
        SLOT(b + L.in_norm, h, 0, "model.layers.%d.input_layernorm.weight", l);
        SLOT(b + L.post_norm, h, 0, "model.layers.%d.post_attention_layernorm.weight", l);
    }
    SLOT(L.final_norm, h, 0, "model.norm.weight");
#undef SLOT
    *out = s;
    return n;
}

#define STAGE_FLOATS ((int64_t)1 << 22)            /* 16 MiB of FP32 per conversion chunk */

static int is_dir(const char* path) {
    struct stat sb;
    return stat(path, &sb) == 0 && S_ISDIR(sb.st_mode);
}
static int file_exists(const char* path) {
    struct stat sb;
    return stat(path, &sb) == 0 && S_ISREG(sb.st_mode);
}

int hip_weights_load(const char* path, const hip_model_config_t* cfg, hip_arena_put_fn put, void* user, int* missing) {
    if (!path || !cfg || !put) return -1;
    if (missing) *missing = 0;
    st_file_t* files = NULL;
    int nfiles = 0, rc = -1;
    float* stage = NULL;
    tensor_slot_t* slots = NULL;

    if (is_dir(path)) {                                                     /* src/model_config.c:343-371 */
        char p[1200];
        snprintf(p, sizeof(p), "%s/model.safetensors", path);
        if (file_exists(p)) {
            files = (st_file_t*)calloc(1, sizeof(st_file_t));
            if (!files || st_open(p, &files[0])) goto done;
            nfiles = 1;
        } else {
            int total = 0;
            for (int t = 2; t <= 999 && !total; t++) {
                snprintf(p, sizeof(p), "%s/model-00001-of-%05d.safetensors", path, t);
                if (file_exists(p)) total = t;
            }
            if (!total) { IO_ERR("no model.safetensors or model-00001-of-N.safetensors in %s", path); goto done; }
            files = (st_file_t*)calloc((size_t)total, sizeof(st_file_t));
            if (!files) goto done;
            for (int i = 1; i <= total; i++) {
                snprintf(p, sizeof(p), "%s/model-%05d-of-%05d.safetensors", path, i, total);
                if (!file_exists(p)) continue;
                if (st_open(p, &files[nfiles])) goto done;
                nfiles++;
            }
        }
    } else {
        files = (st_file_t*)calloc(1, sizeof(st_file_t));
        if (!files || st_open(path, &files[0])) goto done;
        nfiles = 1;
    }

    const int nslots = tensor_slots(cfg, &slots);
    stage = (float*)malloc((size_t)STAGE_FLOATS * sizeof(float));
    if (nslots < 0 || !stage) goto done;
    for (int k = 0; k < nslots; k++) {
        const st_file_t* where = NULL;
        const st_entry_t* e = st_find(files, nfiles, slots[k].name, &where);
        if (!e) { if (missing) (*missing)++; continue; }
        if (e->dtype == ST_OTHER) { IO_ERR("tensor %s has a dtype that cannot be widened to FP32", e->name); goto done; }
        int64_t have = e->count;
        const int is_embed = (k == 0);
        if (have != slots[k].count && !(is_embed && have < slots[k].count && have % cfg->hidden == 0)) {
            IO_ERR("tensor %s holds %lld elements, the model needs %lld", e->name, (long long)have, (long long)slots[k].count);
            goto done;
        }
        for (int64_t at = 0; at < have; at += STAGE_FLOATS) {
            const int64_t n = have - at < STAGE_FLOATS ? have - at : STAGE_FLOATS;
            st_convert(where, e, at, n, stage);
            if (put(user, slots[k].offset + at, stage, n)) goto done;
        }
        if (is_embed && have < slots[k].count) {                             /* src/train.c:318-332 */
            const float scale = sqrtf(2.0f / (float)cfg->hidden);
            srand(42);
            for (int64_t at = have; at < slots[k].count; at += STAGE_FLOATS) {
                const int64_t n = slots[k].count - at < STAGE_FLOATS ? slots[k].count - at : STAGE_FLOATS;
                for (int64_t i = 0; i < n; i++) {
                    const float u1 = ((float)rand() / (float)RAND_MAX) + 1e-7f;
                    const float u2 = ((float)rand() / (float)RAND_MAX);
                    stage[i] = sqrtf(-2.0f * logf(u1)) * cosf(2.0f * 3.14159265f * u2) * scale;
                }
                if (put(user, slots[k].offset + at, stage, n)) goto done;
            }
        }
    }
    rc = 0;
done:
    free(stage);
    free(slots);
    for (int i = 0; i < nfiles; i++) st_close(&files[i]);
    free(files);
    return rc;
}

static int put_host(void* user, int64_t offset, const float* data, int64_t count) {
    memcpy((float*)user + offset, data, (size_t)count * 4);
    return 0;
}
static int get_host(void* user, int64_t offset, float* data, int64_t count) {
    memcpy(data, (const float*)user + offset, (size_t)count * 4);
    return 0;
}
typedef struct { hip_trainer_t* t; int which; } trainer_arena_t;
static int put_trainer(void* user, int64_t offset, const float* data, int64_t count) {
    trainer_arena_t* a = (trainer_arena_t*)user;
    return hip_trainer_upload_at(a->t, a->which, offset, data, count);
}
static int get_trainer(void* user, int64_t offset, float* data, int64_t count) {
    trainer_arena_t* a = (trainer_arena_t*)user;
    return hip_trainer_download_at(a->t, a->which, offset, data, count);
}

int hip_weights_load_host(const char* path, const hip_model_config_t* cfg, float* arena, int* missing) {
    return arena ? hip_weights_load(path, cfg, put_host, arena, missing) : -1;
}
int hip_trainer_load_weights(hip_trainer_t* t, const hip_model_config_t* cfg, const char* path, int* missing) {
    trainer_arena_t a = {t, 0};
    return t ? hip_weights_load(path, cfg, put_trainer, &a, missing) : -1;
}

/* ================================================================= checkpoints */
int hip_checkpoint_save(const char* path, const hip_model_config_t* cfg, hip_arena_get_fn get, void* user) {
    if (!path || !cfg || !get) return -1;
    tensor_slot_t* slots = NULL;
    const int nslots = tensor_slots(cfg, &slots);
    if (nslots < 0) return -1;
    int rc = -1;
    float* stage = (float*)malloc((size_t)STAGE_FLOATS * sizeof(float));
    uint16_t* half = (uint16_t*)malloc((size_t)STAGE_FLOATS * sizeof(uint16_t));
    size_t cap = 512 + (size_t)nslots * 256, len = 0;
    char* header = (char*)malloc(cap);
    FILE* out = NULL;
    if (!stage || !half || !header) goto done;
    len += (size_t)snprintf(header + len, cap - len,
                            "{\"__metadata__\":{\"format\":\"pt\",\"framework\":\"tetyah\",\"trained\":\"full_weight_fp32_adamw\"}");
    size_t data_off = 0;
    for (int k = 0; k < nslots; k++) {
        const size_t bytes = (size_t)slots[k].count * 2;
        if (slots[k].cols > 0)
            len += (size_t)snprintf(header + len, cap - len, ",\"%s\":{\"dtype\":\"BF16\",\"shape\":[%lld,%lld],\"data_offsets\":[%zu,%zu]}",
                                    slots[k].name, (long long)slots[k].rows, (long long)slots[k].cols, data_off, data_off + bytes);
        else
            len += (size_t)snprintf(header + len, cap - len, ",\"%s\":{\"dtype\":\"BF16\",\"shape\":[%lld],\"data_offsets\":[%zu,%zu]}",
                                    slots[k].name, (long long)slots[k].rows, data_off, data_off + bytes);
        data_off += bytes;
    }
    len += (size_t)snprintf(header + len, cap - len, "}");
    out = fopen(path, "wb");
    if (!out) { IO_ERR("Cannot create %s", path); goto done; }
    const uint64_t hlen = (uint64_t)len;
    if (fwrite(&hlen, 8, 1, out) != 1 || fwrite(header, 1, len, out) != len) goto done;
    for (int k = 0; k < nslots; k++) {
        for (int64_t at = 0; at < slots[k].count; at += STAGE_FLOATS) {
            const int64_t n = slots[k].count - at < STAGE_FLOATS ? slots[k].count - at : STAGE_FLOATS;
            if (get(user, slots[k].offset + at, stage, n)) goto done;
            for (int64_t i = 0; i < n; i++) half[i] = f32_to_bf16_trunc(stage[i]);
            if (fwrite(half, 2, (size_t)n, out) != (size_t)n) { IO_ERR("write to %s failed", path); goto done; }
        }
    }
    rc = 0;
done:
    if (out && fclose(out) != 0) rc = -1;
    free(stage); free(half); free(header); free(slots);
    return rc;
}

int hip_checkpoint_load(const char* path, const hip_model_config_t* cfg, hip_arena_put_fn put, void* user) {
    if (!path || !cfg || !put) return -1;
    FILE* f = fopen(path, "rb");
    if (!f) { IO_ERR("Cannot open %s", path); return -1; }
    tensor_slot_t* slots = NULL;
    const int nslots = tensor_slots(cfg, &slots);
    float* stage = (float*)malloc((size_t)STAGE_FLOATS * sizeof(float));
    uint16_t* half = (uint16_t*)malloc((size_t)STAGE_FLOATS * sizeof(uint16_t));
    int rc = -1;
    uint64_t hlen = 0;
    if (nslots < 0 || !stage || !half) goto done;
    if (fread(&hlen, 8, 1, f) != 1) { IO_ERR("Failed to read header size"); goto done; }
    if (fseeko(f, (off_t)hlen, SEEK_CUR) != 0) goto done;                    /* header skipped, src/train.c:579-580 */
    for (int k = 0; k < nslots; k++) {
        for (int64_t at = 0; at < slots[k].count; at += STAGE_FLOATS) {
            const int64_t n = slots[k].count - at < STAGE_FLOATS ? slots[k].count - at : STAGE_FLOATS;
            if (fread(half, 2, (size_t)n, f) != (size_t)n) { IO_ERR("Failed to read tensor data (%s)", slots[k].name); goto done; }
            for (int64_t i = 0; i < n; i++) stage[i] = bf16_to_f32(half[i]);
            if (put(user, slots[k].offset + at, stage, n)) goto done;
        }
    }
    rc = 0;
done:
    fclose(f);
    free(stage); free(half); free(slots);
    return rc;
}

int hip_checkpoint_save_host(const char* path, const hip_model_config_t* cfg, const float* arena) {
    return arena ? hip_checkpoint_save(path, cfg, get_host, (void*)arena) : -1;
}
int hip_checkpoint_load_host(const char* path, const hip_model_config_t* cfg, float* arena) {
    return arena ? hip_checkpoint_load(path, cfg, put_host, arena) : -1;
}
int hip_trainer_save_checkpoint(hip_trainer_t* t, const hip_model_config_t* cfg, const char* path) {
    trainer_arena_t a = {t, 0};
    return t ? hip_checkpoint_save(path, cfg, get_trainer, &a) : -1;
}
int hip_trainer_load_checkpoint(hip_trainer_t* t, const hip_model_config_t* cfg, const char* path) {
    trainer_arena_t a = {t, 0};
    return t ? hip_checkpoint_load(path, cfg, put_trainer, &a) : -1;
}

int hip_train_state_save(const char* checkpoint_path, const hip_train_state_file_t* st) {
    if (!checkpoint_path || !st) return -1;
    char p[1200];
    snprintf(p, sizeof(p), "%s.state", checkpoint_path);
    FILE* f = fopen(p, "wb");
    if (!f) return -1;
    int ok = fwrite(&st->epoch, sizeof(int32_t), 1, f) == 1 && fwrite(&st->step, sizeof(int32_t), 1, f) == 1 &&
             fwrite(&st->loss, sizeof(float), 1, f) == 1 && fwrite(&st->optimizer_step, sizeof(int32_t), 1, f) == 1;
    if (fclose(f) != 0) ok = 0;
    return ok ? 0 : -1;
}

int hip_train_state_load(const char* checkpoint_path, hip_train_state_file_t* st) {
    if (!checkpoint_path || !st) return -1;
    char p[1200];
    snprintf(p, sizeof(p), "%s.state", checkpoint_path);
    FILE* f = fopen(p, "rb");
    if (!f) return -1;
    int ok = fread(&st->epoch, sizeof(int32_t), 1, f) == 1 && fread(&st->step, sizeof(int32_t), 1, f) == 1 &&
             fread(&st->loss, sizeof(float), 1, f) == 1 && fread(&st->optimizer_step, sizeof(int32_t), 1, f) == 1;
    fclose(f);
    return ok ? 0 : -1;
}

/* ------------------------------------------------------------------ exact resume */
int hip_trainer_save_optimizer_state(hip_trainer_t* t, const char* checkpoint_path) {
    if (!t || !checkpoint_path) return -1;
    const int lora = hip_trainer_device_ptr(t, 4) != NULL;
    const int base = lora ? 4 : 0;
    int64_t n = hip_trainer_arena_count(t, base);
    if (n <= 0) return -1;
    char p[1200];
    snprintf(p, sizeof(p), "%s.optim", checkpoint_path);
    FILE* f = fopen(p, "wb");
    if (!f) { IO_ERR("Cannot create %s", p); return -1; }
    const size_t bytes = (size_t)n * 4;
    char header[512];
    const int hl = snprintf(header, sizeof(header),
                            "{\"__metadata__\":{\"format\":\"seraph-hip-optim\",\"mode\":\"%s\"},"
                            "\"params\":{\"dtype\":\"F32\",\"shape\":[%lld],\"data_offsets\":[%zu,%zu]},"
                            "\"adam.m\":{\"dtype\":\"F32\",\"shape\":[%lld],\"data_offsets\":[%zu,%zu]},"
                            "\"adam.v\":{\"dtype\":\"F32\",\"shape\":[%lld],\"data_offsets\":[%zu,%zu]}}",
                            lora ? "lora" : "full", (long long)n, (size_t)0, bytes, (long long)n, bytes, 2 * bytes, (long long)n, 2 * bytes, 3 * bytes);
    const uint64_t hlen = (uint64_t)hl;
    int rc = -1;
    float* stage = (float*)malloc((size_t)STAGE_FLOATS * sizeof(float));
    if (!stage || fwrite(&hlen, 8, 1, f) != 1 || fwrite(header, 1, (size_t)hl, f) != (size_t)hl) goto done;
    const int which[3] = {base + 0, base + 2, base + 3};
    for (int a = 0; a < 3; a++)
        for (int64_t at = 0; at < n; at += STAGE_FLOATS) {
            const int64_t c = n - at < STAGE_FLOATS ? n - at : STAGE_FLOATS;
            if (hip_trainer_download_at(t, which[a], at, stage, c) || fwrite(stage, 4, (size_t)c, f) != (size_t)c) goto done;
        }
    rc = 0;
done:
    if (fclose(f) != 0) rc = -1;
    free(stage);
    return rc;
}

int hip_trainer_load_optimizer_state(hip_trainer_t* t, const char* checkpoint_path) {
    if (!t || !checkpoint_path) return -1;
    char p[1200];
    snprintf(p, sizeof(p), "%s.optim", checkpoint_path);
    if (!file_exists(p)) return 1;
    st_file_t f;
    if (st_open(p, &f)) return -1;
    const int lora = hip_trainer_device_ptr(t, 4) != NULL;
    const int base = lora ? 4 : 0;
    const int64_t n = hip_trainer_arena_count(t, base);
    const char* names[3] = {"params", "adam.m", "adam.v"};
    const int which[3] = {base + 0, base + 2, base + 3};
    int rc = -1;
    float* stage = (float*)malloc((size_t)STAGE_FLOATS * sizeof(float));
    if (!stage) goto done;
    for (int a = 0; a < 3; a++) {
        const st_file_t* where = NULL;
        const st_entry_t* e = st_find(&f, 1, names[a], &where);
        if (!e || e->dtype != ST_F32 || e->count != n) { IO_ERR("%s: tensor %s missing or of the wrong size", p, names[a]); goto done; }
        for (int64_t at = 0; at < n; at += STAGE_FLOATS) {
            const int64_t c = n - at < STAGE_FLOATS ? n - at : STAGE_FLOATS;
            st_convert(where, e, at, c, stage);
            if (hip_trainer_upload_at(t, which[a], at, stage, c)) goto done;
        }
    }
    rc = 0;
done:
    free(stage);
    st_close(&f);
    return rc;
}

/* ================================================================= LoRA adapters */
typedef struct { int have_spare; float spare; } gauss_t;

static float gauss_next(gauss_t* g) {                                       /* src/lora.c:20-40 */
    if (g->have_spare) { g->have_spare = 0; return g->spare; }
    float u, v, s;
    do {
        u = (float)rand() / (float)RAND_MAX * 2.0f - 1.0f;
        v = (float)rand() / (float)RAND_MAX * 2.0f - 1.0f;
        s = u * u + v * v;
    } while (s >= 1.0f || s == 0.0f);
    s = sqrtf(-2.0f * logf(s) / s);
    g->spare = v * s;
    g->have_spare = 1;
    return u * s;
}

int hip_lora_init(const hip_model_config_t* cfg, unsigned seed, float* lora_arena) {
    if (!cfg || !lora_arena || cfg->lora_rank < 1) return -1;
    hip_lora_layout_t L;
    hip_lora_layout(cfg, &L);
    memset(lora_arena, 0, (size_t)L.count * sizeof(float));
    srand(seed);
    gauss_t g = {0, 0.0f};
    for (int l = 0; l < cfg->layers; l++)
        for (int p = 0; p < 7; p++) {
            if (L.A[p] < 0) continue;
            float* A = lora_arena + L.layer_stride * l + L.A[p];
            const float std = sqrtf(2.0f / (float)L.in_dim[p]);
            const int64_t n = (int64_t)cfg->lora_rank * L.in_dim[p];
            for (int64_t i = 0; i < n; i++) A[i] = gauss_next(&g) * std;
        }
    return 0;
}

#define LORA_MAGIC 0x4C4F5241u           /* "LORA", src/lora.c:446 */
#define LORA_EXT_MAGIC 0x3158524Cu       /* "LRX1": adapters the version-2 body does not carry */

static uint32_t lora_file_mask(int mask7) {                                 /* src/lora.c:468-474 */
    uint32_t m = 0;
    if (mask7 & 1) m |= 1;
    if (mask7 & 2) m |= 2;
    if (mask7 & 4) m |= 4;
    if (mask7 & 8) m |= 8;
    if (mask7 & 0x70) m |= 16;
    return m;
}

int hip_lora_save(const char* path, const hip_model_config_t* cfg, const float* lora_arena) {
    if (!path || !cfg || !lora_arena || cfg->lora_rank < 1) return -1;
    hip_lora_layout_t L;
    hip_lora_layout(cfg, &L);
    FILE* f = fopen(path, "wb");
    if (!f) return -1;
    const uint32_t magic = LORA_MAGIC, version = 2, mask = lora_file_mask(cfg->lora_mask);
    const int32_t layers = cfg->layers, rank = cfg->lora_rank;
    const int32_t hidden = (cfg->lora_mask & 1) ? cfg->hidden : 0;           /* taken from the q adapter, src/lora.c:455-459 */
    const int32_t q_out = (cfg->lora_mask & 1) ? cfg->heads * cfg->head_dim : 0;
    const int32_t kv_out = (cfg->lora_mask & 4) ? cfg->kv_heads * cfg->head_dim : 0;
    const float alpha = cfg->lora_alpha;
    int ok = fwrite(&magic, 4, 1, f) == 1 && fwrite(&version, 4, 1, f) == 1 && fwrite(&layers, 4, 1, f) == 1 &&
             fwrite(&rank, 4, 1, f) == 1 && fwrite(&alpha, 4, 1, f) == 1 && fwrite(&hidden, 4, 1, f) == 1 &&
             fwrite(&q_out, 4, 1, f) == 1 && fwrite(&kv_out, 4, 1, f) == 1 && fwrite(&mask, 4, 1, f) == 1;
    static const int body[2] = {0, 2};                                       /* q then v, src/lora.c:478-489 */
    for (int l = 0; ok && l < layers; l++)
        for (int b = 0; ok && b < 2; b++) {
            const int p = body[b];
            if (L.A[p] < 0) continue;
            const float* base = lora_arena + L.layer_stride * l;
            const size_t na = (size_t)rank * (size_t)L.in_dim[p], nb = (size_t)L.out_dim[p] * (size_t)rank;
            ok = fwrite(base + L.A[p], 4, na, f) == na && fwrite(base + L.B[p], 4, nb, f) == nb;
        }
    static const int ext[5] = {1, 3, 4, 5, 6};
    if (ok && (cfg->lora_mask & 0x7A)) {
        const uint32_t em = LORA_EXT_MAGIC, m7 = (uint32_t)cfg->lora_mask;
        ok = fwrite(&em, 4, 1, f) == 1 && fwrite(&m7, 4, 1, f) == 1;
        for (int l = 0; ok && l < layers; l++)
            for (int b = 0; ok && b < 5; b++) {
                const int p = ext[b];
                if (L.A[p] < 0) continue;
                const float* base = lora_arena + L.layer_stride * l;
                const size_t na = (size_t)rank * (size_t)L.in_dim[p], nb = (size_t)L.out_dim[p] * (size_t)rank;
                ok = fwrite(base + L.A[p], 4, na, f) == na && fwrite(base + L.B[p], 4, nb, f) == nb;
            }
    }
    if (fclose(f) != 0) ok = 0;
    return ok ? 0 : -1;
}

int hip_lora_load(const char* path, const hip_model_config_t* cfg, float* lora_arena) {
    if (!path || !cfg || !lora_arena || cfg->lora_rank < 1) return -1;
    hip_lora_layout_t L;
    hip_lora_layout(cfg, &L);
    FILE* f = fopen(path, "rb");
    if (!f) { fprintf(stderr, "Failed to open LoRA file: %s\n", path); return -1; }
    uint32_t magic = 0, version = 0, mask = 0;
    int32_t layers = 0, rank = 0, hidden = 0, q_out = 0, kv_out = 0;
    float alpha = 0.0f;
    int rc = -1;
    if (fread(&magic, 4, 1, f) != 1 || magic != LORA_MAGIC) { fprintf(stderr, "Invalid LoRA file magic\n"); goto done; }
    if (fread(&version, 4, 1, f) != 1 || version != 2) { fprintf(stderr, "Unsupported LoRA format version: %u \n", version); goto done; }
    if (fread(&layers, 4, 1, f) != 1 || fread(&rank, 4, 1, f) != 1 || fread(&alpha, 4, 1, f) != 1 || fread(&hidden, 4, 1, f) != 1 ||
        fread(&q_out, 4, 1, f) != 1 || fread(&kv_out, 4, 1, f) != 1 || fread(&mask, 4, 1, f) != 1) goto done;
    if (layers != cfg->layers || rank != cfg->lora_rank) {
        IO_ERR("%s: %d layers of rank %d, the trainer has %d of rank %d", path, layers, rank, cfg->layers, cfg->lora_rank);
        goto done;
    }
    const int file_has[2] = {(mask & 1) != 0, (mask & 4) != 0};
    const int64_t file_in[2] = {hidden, hidden}, file_out[2] = {q_out, kv_out};
    static const int body[2] = {0, 2};
    for (int l = 0; l < layers; l++)
        for (int b = 0; b < 2; b++) {
            if (!file_has[b]) continue;
            const int p = body[b];
            const size_t na = (size_t)rank * (size_t)file_in[b], nb = (size_t)file_out[b] * (size_t)rank;
            if (L.A[p] >= 0) {
                if (file_in[b] != L.in_dim[p] || file_out[b] != L.out_dim[p]) { IO_ERR("%s: adapter dimensions do not match the model", path); goto done; }
                float* base = lora_arena + L.layer_stride * l;
                if (fread(base + L.A[p], 4, na, f) != na || fread(base + L.B[p], 4, nb, f) != nb) goto done;
            } else if (fseeko(f, (off_t)((na + nb) * 4), SEEK_CUR) != 0) goto done;
        }
    uint32_t em = 0, m7 = 0;
    if (fread(&em, 4, 1, f) == 1 && em == LORA_EXT_MAGIC && fread(&m7, 4, 1, f) == 1) {
        static const int ext[5] = {1, 3, 4, 5, 6};
        for (int l = 0; l < layers; l++)
            for (int b = 0; b < 5; b++) {
                const int p = ext[b];
                if (!((m7 >> p) & 1)) continue;
                const size_t na = (size_t)rank * (size_t)L.in_dim[p], nb = (size_t)L.out_dim[p] * (size_t)rank;
                if (L.A[p] >= 0) {
                    float* base = lora_arena + L.layer_stride * l;
                    if (fread(base + L.A[p], 4, na, f) != na || fread(base + L.B[p], 4, nb, f) != nb) goto done;
                } else if (fseeko(f, (off_t)((na + nb) * 4), SEEK_CUR) != 0) goto done;
            }
    }
    rc = 0;
done:
    fclose(f);
    return rc;
}
