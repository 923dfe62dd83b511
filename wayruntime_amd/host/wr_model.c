/*
 * wr_model.c — engine lifecycle, logging, counters, and the GGUF model loader
 * of the host engine.
 *
 * Engine: one per process; creating it brings up the device attention library
 * (reference attach points: src/core/engine.c:119-178 create, :180 destroy).
 * Loader: the F16 / F32 subset of GGUF v2/v3 for the "llama" and "qwen3"
 * architectures.  Hyperparameter rules follow the reference loader
 * (reference: src/core/loader.c:522-668), tensor names, required shapes and
 * the orientation check follow src/core/loader.c:200-231, 283-401.  The file
 * is mapped read-only and weights are used in place (F16 weights are widened
 * row by row inside the matmul), so nothing is copied at load.
 */
#define _GNU_SOURCE
#include "wr_host.h"

#include <fcntl.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

wr_engine *wrh_engine = NULL;

/* ------------------------------------------------------------------ misc -- */

const char *wr_version(void) { return "0.1.0"; }

const char *wr_status_str(wr_status s)
{
    switch (s) {
    case WR_OK: return "WR_OK";
    case WR_ERR_IO: return "WR_ERR_IO";
    case WR_ERR_FORMAT: return "WR_ERR_FORMAT";
    case WR_ERR_UNSUPPORTED: return "WR_ERR_UNSUPPORTED";
    case WR_ERR_INVAL: return "WR_ERR_INVAL";
    case WR_ERR_NOMEM: return "WR_ERR_NOMEM";
    case WR_ERR_CTX_FULL: return "WR_ERR_CTX_FULL";
    case WR_ERR_STATE: return "WR_ERR_STATE";
    case WR_ERR_LIMIT: return "WR_ERR_LIMIT";
    case WR_ERR_BUSY: return "WR_ERR_BUSY";
    case WR_ERR_INTERNAL: return "WR_ERR_INTERNAL";
    }
    return "WR_ERR_UNKNOWN";
}

void wr_free(void *ptr) { free(ptr); }

void wrh_logf(wr_engine *e, int level, const char *fmt, ...)
{
    char line[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(line, sizeof line, fmt, ap);
    va_end(ap);
    if (!e) e = wrh_engine;
    if (e && e->cfg.log_fn) {
        e->cfg.log_fn(level, line, e->cfg.log_user);
        return;
    }
    static const char *tag[] = {"error", "warn", "info", "debug"};
    fprintf(stderr, "wayruntime %s: %s\n", tag[level < 0 ? 0 : (level > 3 ? 3 : level)], line);
}

static void device_log(int level, const char *msg, void *user)
{
    (void)user;
    wrh_logf(NULL, level, "%s", msg);
}

/* ---------------------------------------------------------------- engine -- */

wr_status wr_engine_create(const wr_engine_config *cfg, wr_engine **out)
{
    if (!out) return WR_ERR_INVAL;
    *out = NULL;
    if (wrh_engine) {
        wrh_logf(NULL, 0, "engine_create: an engine already exists (one per process)");
        return WR_ERR_STATE;
    }
    wr_engine *e = calloc(1, sizeof *e);
    if (!e) return WR_ERR_NOMEM;
    if (cfg) e->cfg = *cfg;
    long n = e->cfg.n_threads ? (long)e->cfg.n_threads : sysconf(_SC_NPROCESSORS_ONLN);
    if (n < 1) n = 1;
    if (n > 64) n = 64;
    e->n_threads = (int)n;
    e->cfg.n_threads = (uint32_t)n;

    wrh_engine = e;
    wr_hip_attn_set_log(device_log, NULL);
    int dev = 0;
    const char *env = getenv("WR_HIP_DEVICE");
    if (env && *env) dev = atoi(env);
    int rc = wr_hip_attn_init(dev);
    if (rc != WR_HIP_OK) {
        wrh_logf(e, 0, "engine_create: device attention library failed to start (rc=%d); "
                      "there is no CPU attention path", rc);
        wrh_engine = NULL;
        free(e);
        return (wr_status)rc;
    }
    /* Keys per decode workgroup (0 / unset = the library's batch-oriented
     * rule).  A deployment that serves one session at a time wants smaller
     * splits: 256-512 keys halve the attention latency of a single long
     * session.  The rule stays a function of the session alone either way, so
     * batched steps still equal serial ones bit for bit. */
    const char *kpw = getenv("WAYRT_DECODE_KEYS_PER_WG");
    if (kpw && *kpw && atoi(kpw) > 0) {
        wr_hip_attn_set_tuning((uint32_t)atoi(kpw), 0);
        wrh_logf(e, 2, "engine: %d keys per decode workgroup (WAYRT_DECODE_KEYS_PER_WG)", atoi(kpw));
    }
    wrh_logf(e, 2, "engine ready: version %s, %d host thread(s), device %s", wr_version(),
            e->n_threads, wr_hip_attn_device_name());
    *out = e;
    return WR_OK;
}

void wr_engine_destroy(wr_engine *e)
{
    if (!e) return;
    if (e->models_live) {
        wrh_logf(e, 0, "engine_destroy: %u model(s) still alive; refused", e->models_live);
        return;
    }
    wr_hip_attn_shutdown();
    if (wrh_engine == e) wrh_engine = NULL;
    free(e);
}

int wr_engine_simd_variant(const wr_engine *e)
{
    (void)e;
#if defined(__AVX2__)
    return WR_SIMD_AVX2;
#else
    return WR_SIMD_SCALAR;
#endif
}

int wr_engine_thread_count(const wr_engine *e)
{
    if (!e) return WR_ERR_INVAL;
    if (e != wrh_engine) return WR_ERR_STATE;
    return e->n_threads;
}

wr_status wr_engine_counters(const wr_engine *e, uint64_t out[WR_COUNTER_COUNT])
{
    if (!e || !out) return WR_ERR_INVAL;
    for (int i = 0; i < WR_COUNTER_COUNT; i++)
        out[i] = __atomic_load_n(&e->ctr[i], __ATOMIC_RELAXED);
    out[WR_CTR_ATTENTION_CALLS] = wr_hip_attn_calls();
    out[WR_CTR_MATMUL_VARIANT] = (uint64_t)wr_engine_simd_variant(e);
    out[WR_CTR_MATMUL_GGML_VARIANT] = (uint64_t)wr_engine_simd_variant(e);
    return WR_OK;
}

/* ------------------------------------------------------------------ gguf -- */

enum { GT_U8, GT_I8, GT_U16, GT_I16, GT_U32, GT_I32, GT_F32, GT_BOOL, GT_STR, GT_ARR, GT_U64,
       GT_I64, GT_F64 };
enum { GGML_F32 = 0, GGML_F16 = 1 };

typedef struct rd {
    const uint8_t *p, *end;
    int bad;
} rd;

static uint64_t rd_int(rd *r, int bytes)
{
    if (r->bad || (size_t)(r->end - r->p) < (size_t)bytes) {
        r->bad = 1;
        return 0;
    }
    uint64_t v = 0;
    memcpy(&v, r->p, (size_t)bytes);       /* little-endian host */
    r->p += bytes;
    return v;
}

static const char *rd_str(rd *r, uint64_t *len)
{
    *len = rd_int(r, 8);
    if (r->bad || *len > (uint64_t)(r->end - r->p)) {
        r->bad = 1;
        return NULL;
    }
    const char *s = (const char *)r->p;
    r->p += *len;
    return s;
}

static int scalar_bytes(uint32_t t)
{
    switch (t) {
    case GT_U8: case GT_I8: case GT_BOOL: return 1;
    case GT_U16: case GT_I16: return 2;
    case GT_U32: case GT_I32: case GT_F32: return 4;
    case GT_U64: case GT_I64: case GT_F64: return 8;
    }
    return 0;
}

/* Skip one value of type t (strings and arrays included). */
static void rd_skip(rd *r, uint32_t t, int depth)
{
    uint64_t n;
    if (t == GT_STR) {
        (void)rd_str(r, &n);
    } else if (t == GT_ARR) {
        if (depth > 2) {
            r->bad = 1;
            return;
        }
        const uint32_t et = (uint32_t)rd_int(r, 4);
        n = rd_int(r, 8);
        const int sb = scalar_bytes(et);
        if (sb) {
            if (n > (uint64_t)(r->end - r->p) / (uint64_t)sb) r->bad = 1;
            else r->p += n * (uint64_t)sb;
        } else {
            for (uint64_t i = 0; i < n && !r->bad; i++) rd_skip(r, et, depth + 1);
        }
    } else {
        const int sb = scalar_bytes(t);
        if (!sb) r->bad = 1;
        else (void)rd_int(r, sb);
    }
}

/* Read a numeric value of type t as u32 / f32 (any integer or float width). */
static int rd_num(rd *r, uint32_t t, uint32_t *u, float *f)
{
    const int sb = scalar_bytes(t);
    if (!sb || t == GT_BOOL) {
        rd_skip(r, t, 0);
        return 0;
    }
    const uint64_t raw = rd_int(r, sb);
    double d;
    if (t == GT_F32) {
        float x;
        memcpy(&x, &raw, 4);
        d = x;
    } else if (t == GT_F64) {
        memcpy(&d, &raw, 8);
    } else if (t == GT_I8) d = (int8_t)raw;
    else if (t == GT_I16) d = (int16_t)raw;
    else if (t == GT_I32) d = (int32_t)raw;
    else if (t == GT_I64) d = (double)(int64_t)raw;
    else d = (double)raw;
    if (u) *u = (d < 0) ? 0 : (d > 4294967295.0 ? 0xFFFFFFFFu : (uint32_t)d);
    if (f) *f = (float)d;
    return 1;
}

typedef struct tinfo {
    const char *name;
    uint64_t    name_len;
    uint32_t    n_dims, type;
    uint64_t    dims[4];
    uint64_t    offset;
} tinfo;

typedef struct gguf_file {
    const uint8_t *base;
    size_t         bytes;
    uint64_t       n_tensors;
    tinfo         *t;
    const uint8_t *data;              /* start of the aligned data section */
    char           arch[32];
    uint32_t block_count, context_length, embedding_length, feed_forward_length;
    uint32_t head_count, head_count_kv, key_length, rope_dim_count, vocab_from_tokens;
    float    rms_eps, rope_base;
    uint32_t alignment;
    /* Gemma family keys (reference: src/core/gguf.c:920-938) */
    uint32_t key_length_swa, sliding_window, shared_kv_layers, has_swa_pattern, pl_emb_dim;
    float    rope_base_swa, softcap;
    uint8_t  swa_pattern[WRH_MAX_LAYERS];
} gguf_file;

static int key_is(const char *k, uint64_t klen, const char *lit)
{
    return klen == strlen(lit) && memcmp(k, lit, klen) == 0;
}

/* Per-layer sliding-window flags: an array of any scalar type, non-zero = local
 * layer (reference: src/core/gguf.c:850-881). */
static void rd_swa_pattern(rd *r, gguf_file *g)
{
    const uint32_t et = (uint32_t)rd_int(r, 4);
    const uint64_t n = rd_int(r, 8);
    const int sb = scalar_bytes(et);
    if (!sb) {
        for (uint64_t i = 0; i < n && !r->bad; i++) rd_skip(r, et, 1);
        return;
    }
    if (n > (uint64_t)(r->end - r->p) / (uint64_t)sb) {
        r->bad = 1;
        return;
    }
    for (uint64_t k = 0; k < n; k++) {
        uint32_t u = 0;
        float f = 0.0f;
        if (et == GT_BOOL) {
            u = (uint32_t)rd_int(r, 1);
        } else {
            rd_num(r, et, &u, &f);
            if (f != 0.0f) u = 1;
        }
        if (k < WRH_MAX_LAYERS) g->swa_pattern[k] = (uint8_t)(u != 0);
    }
    g->has_swa_pattern = 1;
}

static int parse_gguf(wr_engine *e, gguf_file *g)
{
    rd r = {g->base, g->base + g->bytes, 0};
    if (g->bytes < 24 || memcmp(r.p, "GGUF", 4) != 0) {
        wrh_logf(e, 0, "gguf: bad magic");
        return WR_ERR_FORMAT;
    }
    r.p += 4;
    const uint32_t version = (uint32_t)rd_int(&r, 4);
    if (version != 2 && version != 3) {
        wrh_logf(e, 0, "gguf: unsupported container version %u", version);
        return WR_ERR_FORMAT;
    }
    g->n_tensors = rd_int(&r, 8);
    const uint64_t n_kv = rd_int(&r, 8);
    if (r.bad || g->n_tensors > 65536 || n_kv > 65536) return WR_ERR_FORMAT;
    g->alignment = 32;

    /* pass 1 over the key/values: architecture first (its keys are prefixed by it) */
    const uint8_t *kv_start = r.p;
    for (int pass = 0; pass < 2; pass++) {
        r.p = kv_start;
        for (uint64_t i = 0; i < n_kv && !r.bad; i++) {
            uint64_t klen;
            const char *k = rd_str(&r, &klen);
            const uint32_t t = (uint32_t)rd_int(&r, 4);
            if (r.bad) break;
            if (pass == 0) {
                if (key_is(k, klen, "general.architecture") && t == GT_STR) {
                    uint64_t vlen;
                    const char *v = rd_str(&r, &vlen);
                    if (v && vlen < sizeof g->arch) {
                        memcpy(g->arch, v, vlen);
                        g->arch[vlen] = 0;
                    }
                } else if (key_is(k, klen, "general.alignment")) {
                    uint32_t a = 0;
                    if (!rd_num(&r, t, &a, NULL) || a < 8 || a > 4096 || (a & (a - 1))) {
                        wrh_logf(e, 0, "gguf: general.alignment is not a power of two in [8,4096]");
                        return WR_ERR_FORMAT;
                    }
                    g->alignment = a;
                } else if (key_is(k, klen, "tokenizer.ggml.tokens") && t == GT_ARR) {
                    const uint8_t *save = r.p;
                    (void)rd_int(&r, 4);
                    g->vocab_from_tokens = (uint32_t)rd_int(&r, 8);
                    r.p = save;
                    rd_skip(&r, t, 0);
                } else {
                    rd_skip(&r, t, 0);
                }
                continue;
            }
            const size_t alen = strlen(g->arch);
            if (alen && klen > alen + 1 && memcmp(k, g->arch, alen) == 0 && k[alen] == '.') {
                const char *sfx = k + alen + 1;
                const uint64_t sl = klen - alen - 1;
                if (key_is(sfx, sl, "block_count")) rd_num(&r, t, &g->block_count, NULL);
                else if (key_is(sfx, sl, "context_length")) rd_num(&r, t, &g->context_length, NULL);
                else if (key_is(sfx, sl, "embedding_length")) rd_num(&r, t, &g->embedding_length, NULL);
                else if (key_is(sfx, sl, "feed_forward_length")) rd_num(&r, t, &g->feed_forward_length, NULL);
                else if (key_is(sfx, sl, "attention.head_count")) rd_num(&r, t, &g->head_count, NULL);
                else if (key_is(sfx, sl, "attention.head_count_kv")) rd_num(&r, t, &g->head_count_kv, NULL);
                else if (key_is(sfx, sl, "attention.key_length")) rd_num(&r, t, &g->key_length, NULL);
                else if (key_is(sfx, sl, "attention.layer_norm_rms_epsilon")) rd_num(&r, t, NULL, &g->rms_eps);
                else if (key_is(sfx, sl, "rope.freq_base")) rd_num(&r, t, NULL, &g->rope_base);
                else if (key_is(sfx, sl, "rope.dimension_count")) rd_num(&r, t, &g->rope_dim_count, NULL);
                else if (key_is(sfx, sl, "rope.freq_base_swa")) rd_num(&r, t, NULL, &g->rope_base_swa);
                else if (key_is(sfx, sl, "attention.key_length_swa")) rd_num(&r, t, &g->key_length_swa, NULL);
                else if (key_is(sfx, sl, "attention.sliding_window")) rd_num(&r, t, &g->sliding_window, NULL);
                else if (key_is(sfx, sl, "attention.shared_kv_layers")) rd_num(&r, t, &g->shared_kv_layers, NULL);
                else if (key_is(sfx, sl, "final_logit_softcapping")) rd_num(&r, t, NULL, &g->softcap);
                else if (key_is(sfx, sl, "embedding_length_per_layer_input")) rd_num(&r, t, &g->pl_emb_dim, NULL);
                else if (key_is(sfx, sl, "attention.sliding_window_pattern") && t == GT_ARR) rd_swa_pattern(&r, g);
                else rd_skip(&r, t, 0);
            } else {
                rd_skip(&r, t, 0);
            }
        }
        if (r.bad) {
            wrh_logf(e, 0, "gguf: truncated or malformed key/value section");
            return WR_ERR_FORMAT;
        }
    }

    g->t = calloc(g->n_tensors ? g->n_tensors : 1, sizeof *g->t);
    if (!g->t) return WR_ERR_NOMEM;
    for (uint64_t i = 0; i < g->n_tensors; i++) {
        tinfo *t = &g->t[i];
        t->name = rd_str(&r, &t->name_len);
        t->n_dims = (uint32_t)rd_int(&r, 4);
        if (r.bad || t->n_dims == 0 || t->n_dims > 4) return WR_ERR_FORMAT;
        for (uint32_t d = 0; d < t->n_dims; d++) t->dims[d] = rd_int(&r, 8);
        t->type = (uint32_t)rd_int(&r, 4);
        t->offset = rd_int(&r, 8);
        if (r.bad) return WR_ERR_FORMAT;
    }
    const size_t used = (size_t)(r.p - g->base);
    const size_t data_off = (used + g->alignment - 1) / g->alignment * g->alignment;
    if (data_off > g->bytes) return WR_ERR_FORMAT;
    g->data = g->base + data_off;
    return WR_OK;
}

static const tinfo *find_tensor(const gguf_file *g, const char *name)
{
    const size_t n = strlen(name);
    for (uint64_t i = 0; i < g->n_tensors; i++)
        if (g->t[i].name_len == n && memcmp(g->t[i].name, name, n) == 0) return &g->t[i];
    return NULL;
}

/* Bind one weight matrix [rows][cols] (cols = the file's innermost dim). */
static int bind_matrix(wr_engine *e, const gguf_file *g, const char *name, uint32_t rows,
                       uint32_t cols, int required, wrh_weight *out)
{
    const tinfo *t = find_tensor(g, name);
    if (!t) {
        if (!required) return 1;
        wrh_logf(e, 0, "loader: required tensor %s is missing", name);
        return WR_ERR_FORMAT;
    }
    uint64_t elems = 1;
    for (uint32_t d = 0; d < t->n_dims; d++) elems *= t->dims[d];
    if (elems != (uint64_t)rows * cols || elems == 0) {
        wrh_logf(e, 0, "loader: tensor %s has %llu elements, expected %llu", name,
                (unsigned long long)elems, (unsigned long long)rows * cols);
        return WR_ERR_FORMAT;
    }
    if (t->n_dims < 2 || t->dims[0] != cols) {
        wrh_logf(e, 0, "loader: tensor %s is not laid out with innermost dim %u", name, cols);
        return WR_ERR_FORMAT;
    }
    if (t->type != GGML_F16 && t->type != GGML_F32) {
        wrh_logf(e, 0, "loader: tensor %s is stored as ggml type %u; only F16 and F32 have a "
                      "compute path here (WR_ERR_UNSUPPORTED)", name, t->type);
        return WR_ERR_UNSUPPORTED;
    }
    const uint64_t bytes = elems * (t->type == GGML_F16 ? 2u : 4u);
    const uint64_t avail = (uint64_t)(g->base + g->bytes - g->data);
    if (t->offset % g->alignment || t->offset > avail || bytes > avail - t->offset) {
        wrh_logf(e, 0, "loader: tensor %s lies outside the file", name);
        return WR_ERR_FORMAT;
    }
    out->data = g->data + t->offset;
    out->rows = rows;
    out->cols = cols;
    out->is_f16 = (t->type == GGML_F16);
    return WR_OK;
}

static int bind_vector(wr_engine *e, const gguf_file *g, const char *name, uint32_t n, wrh_vec *out)
{
    const tinfo *t = find_tensor(g, name);
    if (!t) {
        wrh_logf(e, 0, "loader: required tensor %s is missing", name);
        return WR_ERR_FORMAT;
    }
    uint64_t elems = 1;
    for (uint32_t d = 0; d < t->n_dims; d++) elems *= t->dims[d];
    if (elems != n) {
        wrh_logf(e, 0, "loader: tensor %s has %llu elements, expected %u", name,
                (unsigned long long)elems, n);
        return WR_ERR_FORMAT;
    }
    if (t->type != GGML_F32) {
        wrh_logf(e, 0, "loader: norm vector %s must be F32 (ggml type %u found)", name, t->type);
        return WR_ERR_UNSUPPORTED;
    }
    const uint64_t avail = (uint64_t)(g->base + g->bytes - g->data);
    if (t->offset % g->alignment || t->offset > avail || (uint64_t)n * 4 > avail - t->offset)
        return WR_ERR_FORMAT;
    out->data = (const float *)(g->data + t->offset);
    out->n = n;
    return WR_OK;
}

/* ----------------------------------------------------------------- model -- */

wr_status wr_model_load(wr_engine *e, const char *path, const wr_model_params *params,
                        wr_model **out)
{
    if (!out) return WR_ERR_INVAL;
    *out = NULL;
    if (!e || !path) return WR_ERR_INVAL;
    if (e != wrh_engine) return WR_ERR_STATE;
    wr_model_params p = {0, 0, 0, 0};
    if (params) p = *params;
    if (p.keep_quantized < 0 || p.keep_quantized > WR_QUANT_F32 || p.swa_mode < 0 ||
        p.swa_mode > WR_SWA_DISABLED || p.use_mmap < -1)
        return WR_ERR_INVAL;
    if (p.max_context > WR_HIP_ATTN_MAX_SEQ) {
        wrh_logf(e, 0, "loader: max_context %u exceeds the attention sequence cap %u "
                      "(WR_ERR_LIMIT; never clamped)", p.max_context, WR_HIP_ATTN_MAX_SEQ);
        return WR_ERR_LIMIT;
    }

    const int fd = open(path, O_RDONLY);
    if (fd < 0) {
        wrh_logf(e, 0, "loader: cannot open %s", path);
        return WR_ERR_IO;
    }
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        close(fd);
        return WR_ERR_IO;
    }
    void *map = mmap(NULL, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return WR_ERR_IO;

    gguf_file g;
    memset(&g, 0, sizeof g);
    g.base = map;
    g.bytes = (size_t)st.st_size;
    wr_model *m = NULL;
    int rc = parse_gguf(e, &g);
    if (rc != WR_OK) goto fail;

    int is_qwen3 = strcmp(g.arch, "qwen3") == 0;
    const int is_gemma = strcmp(g.arch, "gemma4") == 0;
    if (!is_qwen3 && !is_gemma && strcmp(g.arch, "llama") != 0) {
        wrh_logf(e, 0, "loader: architecture '%s' is not served by this engine "
                      "(llama, qwen3 and gemma4 are)", g.arch);
        rc = WR_ERR_UNSUPPORTED;
        goto fail;
    }
    m = calloc(1, sizeof *m);
    if (!m) {
        rc = WR_ERR_NOMEM;
        goto fail;
    }
    m->engine = e;
    snprintf(m->arch, sizeof m->arch, "%s", g.arch);
    m->n_layers = g.block_count;
    if (m->n_layers == 0) {
        wrh_logf(e, 0, "loader: %s.block_count missing or 0", g.arch);
        rc = WR_ERR_FORMAT;
        goto fail;
    }
    if (m->n_layers > WRH_MAX_LAYERS) {
        wrh_logf(e, 0, "loader: model has %u layers; the compiled cap is %u (WR_ERR_LIMIT)",
                m->n_layers, WRH_MAX_LAYERS);
        rc = WR_ERR_LIMIT;
        goto fail;
    }
    m->hidden = g.embedding_length;
    m->vocab = g.vocab_from_tokens;
    if (m->vocab == 0) {
        const tinfo *te = find_tensor(&g, "token_embd.weight");
        if (te && te->n_dims >= 2) m->vocab = (uint32_t)te->dims[1];
    }
    if (m->hidden == 0 || m->vocab == 0) {
        wrh_logf(e, 0, "loader: missing core metadata (hidden=%u vocab=%u)", m->hidden, m->vocab);
        rc = WR_ERR_FORMAT;
        goto fail;
    }
    m->n_q = g.head_count ? g.head_count : 1;
    m->n_kv = g.head_count_kv ? g.head_count_kv : m->n_q;
    if (m->n_q % m->n_kv) {
        wrh_logf(e, 0, "loader: head_count %u not a multiple of head_count_kv %u", m->n_q, m->n_kv);
        rc = WR_ERR_FORMAT;
        goto fail;
    }
    m->train_context = g.context_length;
    m->ffn = g.feed_forward_length;
    m->rope_base = (g.rope_base > 0.0f) ? g.rope_base : 10000.0f;
    m->has_qk_norm = (uint8_t)(is_qwen3 || is_gemma);
    m->rms_eps = (g.rms_eps > 0.0f) ? g.rms_eps : (is_gemma ? 1e-6f : 1e-5f);
    m->head_dim = g.key_length ? g.key_length : (is_gemma ? 0 : m->hidden / m->n_q);
    if (is_gemma && m->head_dim == 0) {
        wrh_logf(e, 0, "loader: gemma4 requires %s.attention.key_length", g.arch);
        rc = WR_ERR_FORMAT;
        goto fail;
    }
    if (m->head_dim == 0) m->head_dim = 64;
    m->attn_scale = 0.0f;                       /* 0 = 1/sqrt(head_dim) */
    for (uint32_t l = 0; l < m->n_layers; l++) {
        m->hd_layer[l] = m->head_dim;
        m->kv_src[l] = l;
    }
    if (is_gemma) {
        /* reference: src/core/loader.c:576-628 */
        if (g.pl_emb_dim) {
            wrh_logf(e, 0, "loader: per-layer input tables (embedding_length_per_layer_input=%u) are "
                          "not served by this engine (WR_ERR_UNSUPPORTED)", g.pl_emb_dim);
            rc = WR_ERR_UNSUPPORTED;
            goto fail;
        }
        m->is_gemma = 1;
        m->swa_mode = (uint8_t)p.swa_mode;
        m->head_dim_swa = g.key_length_swa;
        m->rope_base_swa = (g.rope_base_swa >= 1.0f) ? g.rope_base_swa : 10000.0f;
        m->sliding_window = g.sliding_window;
        m->kv_shared_layers = g.shared_kv_layers;
        if (m->kv_shared_layers >= m->n_layers) {
            wrh_logf(e, 0, "loader: shared_kv_layers %u >= block_count %u", m->kv_shared_layers,
                    m->n_layers);
            rc = WR_ERR_FORMAT;
            goto fail;
        }
        m->has_swa = (uint8_t)(g.has_swa_pattern ? 1 : 0);
        for (uint32_t l = 0; l < m->n_layers; l++) {
            m->swa[l] = (uint8_t)(m->has_swa && g.swa_pattern[l]);
            if (m->swa[l] && m->head_dim_swa) m->hd_layer[l] = m->head_dim_swa;
        }
        /* a shared layer reads the last earlier layer of its own kind that owns a
         * cache (reference: src/core/session.c:115-134) */
        if (m->kv_shared_layers) {
            const uint32_t first_shared = m->n_layers - m->kv_shared_layers;
            for (uint32_t l = first_shared; l < m->n_layers; l++)
                for (int c = (int)first_shared - 1; c >= 0; c--)
                    if (m->swa[c] == m->swa[l]) {
                        m->kv_src[l] = (uint32_t)c;
                        break;
                    }
        }
        /* sqrt(hidden) by 24 Newton steps from the value itself, as the reference
         * computes it (loader.c:46-54) */
        float gs = (float)m->hidden;
        for (int i = 0; i < 24; i++) gs = 0.5f * (gs + (float)m->hidden / gs);
        m->embed_scale = gs;
        m->attn_scale = 1.0f;                    /* the Q/K norms set the magnitude */
        m->logit_softcap = g.softcap;
        m->n_rot_pairs = m->head_dim / 8;        /* partial rotary on global layers */
        if (m->head_dim_swa & 1) {
            rc = WR_ERR_FORMAT;
            goto fail;
        }
    }
    if (m->head_dim & 1) {
        rc = WR_ERR_FORMAT;
        goto fail;
    }
    if (!is_gemma && g.rope_dim_count && g.rope_dim_count < m->head_dim)
        m->n_rot_pairs = g.rope_dim_count / 2;
    if (p.max_context) {
        m->max_context = p.max_context;
    } else {
        uint32_t eff = m->train_context ? m->train_context : WRH_DEFAULT_CTX;
        if (eff > WRH_DEFAULT_CTX) eff = WRH_DEFAULT_CTX;
        m->max_context = eff;
    }

    char nb[96];
    if ((rc = bind_matrix(e, &g, "token_embd.weight", m->vocab, m->hidden, 1, &m->embed)) < 0) goto fail;
    if ((rc = bind_vector(e, &g, "output_norm.weight", m->hidden, &m->final_norm)) < 0) goto fail;
    rc = bind_matrix(e, &g, "output.weight", m->vocab, m->hidden, 0, &m->lm_head);
    if (rc < 0) goto fail;
    if (rc == 1) {
        m->lm_head = m->embed;
        m->tied_head = 1;
    }
    m->all_f16 = m->embed.is_f16;
    for (uint32_t l = 0; l < m->n_layers; l++) {
#define NAME(sfx) (snprintf(nb, sizeof nb, "blk.%u." sfx, l), nb)
        uint32_t ffn_l = m->ffn;
        const tinfo *tg = find_tensor(&g, NAME("ffn_gate.weight"));
        if (tg && tg->n_dims >= 2) ffn_l = (uint32_t)tg->dims[1];
        if (ffn_l == 0) {
            wrh_logf(e, 0, "loader: layer %u has no FFN dim", l);
            rc = WR_ERR_FORMAT;
            goto fail;
        }
        if (m->ffn == 0) m->ffn = ffn_l;
        if (ffn_l != m->ffn) {
            wrh_logf(e, 0, "loader: per-layer FFN widths are not served by this engine");
            rc = WR_ERR_UNSUPPORTED;
            goto fail;
        }
        const uint32_t hd_l = m->hd_layer[l];
        const uint32_t qd = m->n_q * hd_l, kd = m->n_kv * hd_l;
        if ((rc = bind_vector(e, &g, NAME("attn_norm.weight"), m->hidden, &m->attn_norm[l])) < 0) goto fail;
        if ((rc = bind_matrix(e, &g, NAME("attn_q.weight"), qd, m->hidden, 1, &m->wq[l])) < 0) goto fail;
        if ((rc = bind_matrix(e, &g, NAME("attn_k.weight"), kd, m->hidden, 1, &m->wk[l])) < 0) goto fail;
        if ((rc = bind_matrix(e, &g, NAME("attn_v.weight"), kd, m->hidden, 1, &m->wv[l])) < 0) goto fail;
        if (m->has_qk_norm) {
            if ((rc = bind_vector(e, &g, NAME("attn_q_norm.weight"), hd_l, &m->q_norm[l])) < 0) goto fail;
            if ((rc = bind_vector(e, &g, NAME("attn_k_norm.weight"), hd_l, &m->k_norm[l])) < 0) goto fail;
        }
        if ((rc = bind_matrix(e, &g, NAME("attn_output.weight"), m->hidden, qd, 1, &m->wo[l])) < 0) goto fail;
        if (m->is_gemma) {
            if ((rc = bind_vector(e, &g, NAME("post_attention_norm.weight"), m->hidden, &m->post_attn_norm[l])) < 0) goto fail;
            if ((rc = bind_vector(e, &g, NAME("post_ffw_norm.weight"), m->hidden, &m->post_ffw_norm[l])) < 0) goto fail;
        }
        if ((rc = bind_vector(e, &g, NAME("ffn_norm.weight"), m->hidden, &m->ffn_norm[l])) < 0) goto fail;
        if ((rc = bind_matrix(e, &g, NAME("ffn_gate.weight"), m->ffn, m->hidden, 1, &m->w_gate[l])) < 0) goto fail;
        if ((rc = bind_matrix(e, &g, NAME("ffn_up.weight"), m->ffn, m->hidden, 1, &m->w_up[l])) < 0) goto fail;
        if ((rc = bind_matrix(e, &g, NAME("ffn_down.weight"), m->hidden, m->ffn, 1, &m->w_down[l])) < 0) goto fail;
        m->all_f16 = (uint8_t)(m->all_f16 && m->wq[l].is_f16);
#undef NAME
    }
    /* every matrix F16, not only the first one looked at */
    for (uint32_t l = 0; l < m->n_layers; l++)
        m->all_f16 = (uint8_t)(m->all_f16 && m->wk[l].is_f16 && m->wv[l].is_f16 && m->wo[l].is_f16 &&
                               m->w_gate[l].is_f16 && m->w_up[l].is_f16 && m->w_down[l].is_f16);
    m->all_f16 = (uint8_t)(m->all_f16 && m->lm_head.is_f16);
    /* weights and layer walk on the device where the library and the model allow it */
    if ((rc = wrh_device_model_init(m)) != WR_OK) goto fail;
    free(g.t);
    m->map = map;
    m->map_bytes = (size_t)st.st_size;
    pthread_mutex_init(&m->lock, NULL);
    e->models_live++;
    wrh_logf(e, 2, "loader: %s: arch=%s layers=%u hidden=%u heads=%u/%u head_dim=%u vocab=%u "
                  "ffn=%u ctx=%u%s", path, m->arch, m->n_layers, m->hidden, m->n_q, m->n_kv,
            m->head_dim, m->vocab, m->ffn, m->max_context, m->tied_head ? " tied-lm-head" : "");
    *out = m;
    return WR_OK;

fail:
    free(g.t);
    free(m);
    munmap(map, (size_t)st.st_size);
    return (wr_status)rc;
}

void wr_model_free(wr_model *m)
{
    if (!m) return;
    pthread_mutex_lock(&m->lock);
    const uint32_t refs = m->session_refs;
    pthread_mutex_unlock(&m->lock);
    if (refs) {
        wrh_logf(m->engine, 0, "model_free: %u session(s) still alive; refused", refs);
        return;
    }
    if (m->engine && m->engine->models_live) m->engine->models_live--;
    wrh_scratch_free_all(m);
    wrh_device_model_free(m);
    munmap(m->map, m->map_bytes);
    pthread_mutex_destroy(&m->lock);
    free(m);
}

wr_status wr_model_get_info(const wr_model *m, wr_model_info *out)
{
    if (!m || !out) return WR_ERR_INVAL;
    memset(out, 0, sizeof *out);
    snprintf(out->arch, sizeof out->arch, "%s", m->arch);
    snprintf(out->quant, sizeof out->quant, "%s", m->all_f16 ? "F16" : "F32");
    out->n_layers = m->n_layers;
    out->n_q_heads = m->n_q;
    out->n_kv_heads = m->n_kv;
    out->head_dim = m->head_dim;
    out->hidden_dim = m->hidden;
    out->ffn_dim = m->ffn;
    out->vocab_size = m->vocab;
    out->train_context = m->train_context;
    out->max_context = m->max_context;
    out->rope_freq_base = m->rope_base;
    out->rms_eps = m->rms_eps;
    out->has_qk_norm = m->has_qk_norm;
    out->is_gemma = m->is_gemma;
    out->has_swa = m->has_swa;
    out->head_dim_swa = m->head_dim_swa;
    out->sliding_window = m->sliding_window;
    out->logit_softcap = m->logit_softcap;
    out->tied_lm_head = m->tied_head;
    return WR_OK;
}
