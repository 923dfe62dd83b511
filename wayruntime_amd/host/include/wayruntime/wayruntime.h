/*
 * wayruntime.h — the engine / model / session surface of the reference's public
 * C API, as served by the MI355X host engine in this directory.
 *
 * Names, argument order, struct layouts and enum values follow the reference's
 * public header (reference: include/wayruntime/wayruntime.h) so a harness
 * written against it (for example its test/sdk_gen.c batch and context tests)
 * compiles unchanged.  Only the part of the API that reaches the attention
 * path is implemented here: engine, model load / info, session, prefill, step,
 * batched step.  Tokenizer, sampler and the generate facade are outside that
 * path and are not provided.
 *
 * What differs from the CPU reference is behind the API: the per-session KV
 * cache lives in device memory and attention runs through wr_hip_attn_*.
 */
#ifndef WAYRUNTIME_H
#define WAYRUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WR_VERSION_MAJOR 0
#define WR_VERSION_MINOR 1
#define WR_VERSION_PATCH 0
const char *wr_version(void);

/* reference: wayruntime.h:82-107 */
typedef enum wr_status {
    WR_OK              = 0,
    WR_ERR_IO          = -1,
    WR_ERR_FORMAT      = -2,
    WR_ERR_UNSUPPORTED = -3,
    WR_ERR_INVAL       = -4,
    WR_ERR_NOMEM       = -5,
    WR_ERR_CTX_FULL    = -6,
    WR_ERR_STATE       = -7,
    WR_ERR_LIMIT       = -8,
    WR_ERR_BUSY        = -9,
    WR_ERR_INTERNAL    = -10
} wr_status;
const char *wr_status_str(wr_status s);

typedef struct wr_engine  wr_engine;
typedef struct wr_model   wr_model;
typedef struct wr_session wr_session;

/* level 0 error, 1 warn, 2 info, 3 debug (reference: wayruntime.h:126-130) */
typedef void (*wr_log_fn)(int level, const char *msg, void *user);

/* ---- engine (reference: wayruntime.h:156-226) ---- */
enum { WR_SIMD_SCALAR = 0, WR_SIMD_AVX2 = 1, WR_SIMD_AVX512 = 2, WR_SIMD_NEON = 3 };

typedef struct wr_engine_config {
    uint32_t  n_threads;     /* host worker threads for the CPU ops; 0 = all */
    int32_t   force_scalar;  /* accepted for layout compatibility */
    int32_t   prefer_avx2;   /* accepted for layout compatibility */
    uint32_t  arena_mb;      /* accepted for layout compatibility */
    wr_log_fn log_fn;        /* NULL = stderr */
    void     *log_user;
} wr_engine_config;

/* One engine per process; creating it also initialises device 0 (override
 * with the environment variable WR_HIP_DEVICE).  No device: WR_ERR_UNSUPPORTED. */
wr_status wr_engine_create(const wr_engine_config *cfg, wr_engine **out);
void      wr_engine_destroy(wr_engine *e);
int       wr_engine_simd_variant(const wr_engine *e);
int       wr_engine_thread_count(const wr_engine *e);

enum {
    WR_CTR_MATMUL_CALLS = 0, WR_CTR_MATMUL_ELEMS = 1, WR_CTR_SOFTMAX_CALLS = 2,
    WR_CTR_ATTENTION_CALLS = 3, WR_CTR_FUSED_CALLS = 4, WR_CTR_MATMUL_VARIANT = 5,
    WR_CTR_SOFTMAX_VARIANT = 6, WR_CTR_MATMUL_GGML_SIMD = 7, WR_CTR_MATMUL_GGML_VARIANT = 8,
    WR_CTR_MATMUL_GGML_QUANT = 9, WR_CTR_MATMUL_PERELEM = 10, WR_CTR_MATMUL_PAR_N = 11,
    WR_COUNTER_COUNT = 12
};
/* WR_CTR_ATTENTION_CALLS counts one per session-layer attention, as the
 * reference does (src/core/kernels.c:1423). */
wr_status wr_engine_counters(const wr_engine *e, uint64_t out[WR_COUNTER_COUNT]);

/* ---- model (reference: wayruntime.h:232-318) ---- */
enum { WR_QUANT_AUTO = 0, WR_QUANT_KEEP = 1, WR_QUANT_F32 = 2 };
enum { WR_SWA_ENABLED = 0, WR_SWA_DISABLED = 1 };
enum { WR_MMAP_DISABLED = -1, WR_MMAP_AUTO = 0, WR_MMAP_ENABLED = 1 };

typedef struct wr_model_params {
    uint32_t max_context;     /* 0 = min(trained context, 4096) */
    int32_t  keep_quantized;
    int32_t  swa_mode;
    int32_t  use_mmap;
} wr_model_params;

/* GGUF v2/v3, architectures "llama" and "qwen3", F16 / F32 tensors. */
wr_status wr_model_load(wr_engine *e, const char *gguf_path,
                        const wr_model_params *params, wr_model **out);
void      wr_model_free(wr_model *m);

typedef struct wr_model_info {
    char     arch[32];
    char     quant[16];
    uint32_t n_layers, n_q_heads, n_kv_heads, head_dim, head_dim_swa;
    uint32_t hidden_dim, ffn_dim, vocab_size, train_context, max_context;
    float    rope_freq_base, rms_eps, logit_softcap;
    uint32_t sliding_window;
    uint8_t  is_gemma, has_qk_norm, tied_lm_head, has_swa;
} wr_model_info;
wr_status wr_model_get_info(const wr_model *m, wr_model_info *out);

/* ---- session (reference: wayruntime.h:381-444) ---- */
typedef struct wr_session_params {
    uint32_t max_context;     /* 0 = the model's bound */
} wr_session_params;

wr_status wr_session_create(wr_model *m, const wr_session_params *params, wr_session **out);
void      wr_session_destroy(wr_session *s);

/* Prefill n tokens without logits; all-or-nothing; returns n or a negative
 * status.  Runs layer-major over chunks of the prompt: per layer one append of
 * the chunk's K/V rows and one causal prefill attention. */
int wr_prefill(wr_session *s, const uint32_t *ids, uint32_t n);

/* One decode step; borrowed logits pointer (vocab floats) or NULL on error. */
const float *wr_step(wr_session *s, uint32_t token);

#define WR_BATCH_MAX 16
/* Up to WR_BATCH_MAX distinct sessions of one model in one step, layer-major:
 * per layer one batched attention launch.  Returns n, or a negative status
 * with no session advanced. */
int wr_batch_step(wr_session *const *sessions, const uint32_t *tokens, uint32_t n,
                  const float **logits_out);

uint32_t  wr_session_pos(const wr_session *s);
uint32_t  wr_session_max_context(const wr_session *s);
wr_status wr_session_status(const wr_session *s);

void wr_free(void *ptr);

#ifdef __cplusplus
}
#endif
#endif /* WAYRUNTIME_H */
