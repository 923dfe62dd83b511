/*
 * wr_hip_attn_cpu_shim.c — TEST DOUBLE of the device attention library.
 * TEST INFRASTRUCTURE, never shipped: it exists so the C11 host engine's own
 * logic (locking, all-or-nothing rollback, context limits, layer-major batch
 * and prefill drivers, the GGUF loader) can be exercised on a machine without
 * a GPU.  It implements the wr_hip_attn_* entry points the host engine calls
 * on top of the CPU oracle (wr_oracle.c) and is linked ONLY into
 * oracle/libwayruntime_cpuattn.so, which only the tests load.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../include/wr_hip_attn.h"
#include "wr_oracle.h"

struct wr_hip_kv {
    uint32_t n_layers, nkv, max_ctx;
    uint32_t hd[WR_HIP_MAX_LAYERS];
    uint16_t *k[WR_HIP_MAX_LAYERS], *v[WR_HIP_MAX_LAYERS];   /* position-major [max_ctx][nkv][hd] */
    uint64_t bytes;
};

static int g_inited;
static uint64_t g_calls;
/* Test hook: the k-th attention call from now (1 = the next one) does its work
 * and then reports WR_HIP_ERR_INTERNAL, the way the device library reports a
 * kernel that gave up a bounded wait: found at the wait that ends the call,
 * after the outputs have been written with data that cannot be trusted. */
static int g_late_error_in;

void wr_hip_attn_debug_late_error_in(int k) { g_late_error_in = k; }

static int late_error(void)
{
    if (g_late_error_in > 0 && --g_late_error_in == 0) return WR_HIP_ERR_INTERNAL;
    return WR_HIP_OK;
}

int wr_hip_attn_init(int device)
{
    (void)device;
    if (g_inited) return WR_HIP_ERR_STATE;
    g_inited = 1;
    g_calls = 0;
    wro_set_attn_max_seq(WR_HIP_ATTN_MAX_SEQ);
    return WR_HIP_OK;
}

void wr_hip_attn_shutdown(void) { g_inited = 0; }
void wr_hip_attn_set_log(wr_hip_log_fn fn, void *user) { (void)fn; (void)user; }
uint64_t wr_hip_attn_calls(void) { return g_calls; }
const char *wr_hip_attn_device_name(void) { return "cpu test double (oracle)"; }

int wr_hip_attn_kv_create(uint32_t n_layers, const uint32_t *hd, uint32_t nkv, uint32_t max_ctx,
                          wr_hip_kv **out)
{
    if (!out) return WR_HIP_ERR_INVAL;
    *out = NULL;
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!hd || !n_layers || !nkv || !max_ctx) return WR_HIP_ERR_INVAL;
    if (n_layers > WR_HIP_MAX_LAYERS || max_ctx > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    wr_hip_kv *kv = calloc(1, sizeof *kv);
    if (!kv) return WR_HIP_ERR_NOMEM;
    kv->n_layers = n_layers;
    kv->nkv = nkv;
    kv->max_ctx = max_ctx;
    for (uint32_t L = 0; L < n_layers; L++) {
        kv->hd[L] = hd[L];
        if (!hd[L]) continue;
        const size_t n = (size_t)max_ctx * nkv * hd[L];
        kv->k[L] = calloc(n, 2);
        kv->v[L] = calloc(n, 2);
        kv->bytes += 4 * n;
        if (!kv->k[L] || !kv->v[L]) {
            wr_hip_attn_kv_destroy(kv);
            return WR_HIP_ERR_NOMEM;
        }
    }
    *out = kv;
    return WR_HIP_OK;
}

void wr_hip_attn_kv_destroy(wr_hip_kv *kv)
{
    if (!kv) return;
    for (uint32_t L = 0; L < kv->n_layers; L++) {
        free(kv->k[L]);
        free(kv->v[L]);
    }
    free(kv);
}

uint64_t wr_hip_attn_kv_bytes(const wr_hip_kv *kv) { return kv ? kv->bytes : 0; }

static int layer_ok(const wr_hip_kv *kv, uint32_t layer)
{
    return kv && layer < kv->n_layers && kv->hd[layer] != 0;
}

int wr_hip_attn_append(wr_hip_kv *kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                       const float *k, const float *v)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!layer_ok(kv, layer)) return WR_HIP_ERR_INVAL;
    if (n_rows == 0) return WR_HIP_OK;
    if (!k || !v) return WR_HIP_ERR_INVAL;
    if ((uint64_t)pos + n_rows > kv->max_ctx) return WR_HIP_ERR_CTX_FULL;
    const size_t row = (size_t)kv->nkv * kv->hd[layer];
    for (size_t i = 0; i < (size_t)n_rows * row; i++) {
        kv->k[layer][(size_t)pos * row + i] = wro_f32_to_f16(k[i]);
        kv->v[layer][(size_t)pos * row + i] = wro_f32_to_f16(v[i]);
    }
    return WR_HIP_OK;
}

int wr_hip_attn_append_rope(wr_hip_kv *kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                            const float *k, const float *v, const float *cos_sin, uint32_t n_rot)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!layer_ok(kv, layer)) return WR_HIP_ERR_INVAL;
    if (n_rows == 0) return WR_HIP_OK;
    if (!k || !v || (!cos_sin && n_rot > 0)) return WR_HIP_ERR_INVAL;
    if ((uint64_t)pos + n_rows > kv->max_ctx) return WR_HIP_ERR_CTX_FULL;
    const uint32_t hd = kv->hd[layer], half = hd / 2;
    if (n_rot > half) return WR_HIP_ERR_INVAL;
    const size_t row = (size_t)kv->nkv * hd;
    for (uint32_t r = 0; r < n_rows; r++)
        for (uint32_t h = 0; h < kv->nkv; h++) {
            const float *x = k + (size_t)r * row + (size_t)h * hd;
            uint16_t *dst = kv->k[layer] + ((size_t)pos + r) * row + (size_t)h * hd;
            for (uint32_t j = 0; j < hd; j++) dst[j] = wro_f32_to_f16(x[j]);
            for (uint32_t j = 0; j < n_rot; j++) {
                const float c = cos_sin[((size_t)r * n_rot + j) * 2];
                const float sn = cos_sin[((size_t)r * n_rot + j) * 2 + 1];
                const float x0 = x[j], x1 = x[j + half];
                dst[j] = wro_f32_to_f16(x0 * c - x1 * sn);
                dst[j + half] = wro_f32_to_f16(x0 * sn + x1 * c);
            }
        }
    for (size_t i = 0; i < (size_t)n_rows * row; i++)
        kv->v[layer][(size_t)pos * row + i] = wro_f32_to_f16(v[i]);
    return WR_HIP_OK;
}

int wr_hip_attn_kv_read(wr_hip_kv *kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                        uint16_t *k, uint16_t *v)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!layer_ok(kv, layer) || !k || !v || (uint64_t)pos + n_rows > kv->max_ctx)
        return WR_HIP_ERR_INVAL;
    const size_t row = (size_t)kv->nkv * kv->hd[layer];
    memcpy(k, kv->k[layer] + (size_t)pos * row, (size_t)n_rows * row * 2);
    memcpy(v, kv->v[layer] + (size_t)pos * row, (size_t)n_rows * row * 2);
    return WR_HIP_OK;
}

int wr_hip_attn_kv_write(wr_hip_kv *kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                         const uint16_t *k, const uint16_t *v)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!layer_ok(kv, layer) || !k || !v) return WR_HIP_ERR_INVAL;
    if ((uint64_t)pos + n_rows > kv->max_ctx) return WR_HIP_ERR_CTX_FULL;
    const size_t row = (size_t)kv->nkv * kv->hd[layer];
    memcpy(kv->k[layer] + (size_t)pos * row, k, (size_t)n_rows * row * 2);
    memcpy(kv->v[layer] + (size_t)pos * row, v, (size_t)n_rows * row * 2);
    return WR_HIP_OK;
}

static int check_decode(const wr_hip_kv *kv, uint32_t layer, uint32_t seq_k, uint32_t nq)
{
    if (!layer_ok(kv, layer)) return WR_HIP_ERR_INVAL;
    if (nq == 0 || nq % kv->nkv) return WR_HIP_ERR_INVAL;
    if (seq_k == 0) return WR_HIP_ERR_INVAL;
    if (seq_k > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    if (seq_k > kv->max_ctx) return WR_HIP_ERR_INVAL;
    return WR_HIP_OK;
}

int wr_hip_attn_decode(wr_hip_kv *kv, uint32_t layer, uint32_t seq_k, const float *q, float *out,
                       uint32_t nq, float scale_override, uint32_t window)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!kv || !q || !out) return WR_HIP_ERR_INVAL;
    g_calls++;                 /* counted before the shape checks (src/core/kernels.c:1423) */
    int rc = check_decode(kv, layer, seq_k, nq);
    if (rc) return rc;
    wro_attention_f16kv(q, kv->k[layer], kv->v[layer], out, 1, nq, kv->nkv, kv->hd[layer], seq_k,
                        scale_override, window);
    return late_error();
}

int wr_hip_attn_decode_batched(uint32_t n, wr_hip_kv *const *kv, uint32_t layer,
                               const uint32_t *seq_k, const float *const *q, float *const *out,
                               uint32_t nq, float scale_override, uint32_t window)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!kv || !seq_k || !q || !out) return WR_HIP_ERR_INVAL;
    if (n == 0 || n > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    for (uint32_t i = 0; i < n; i++)
        if (!kv[i]) return WR_HIP_ERR_INVAL;
    g_calls += n;
    for (uint32_t i = 0; i < n; i++) {
        int rc = check_decode(kv[i], layer, seq_k[i], nq);
        if (rc) return rc;
        for (uint32_t j = 0; j < i; j++)
            if (kv[i] == kv[j]) return WR_HIP_ERR_INVAL;
    }
    for (uint32_t i = 0; i < n; i++)
        wro_attention_f16kv(q[i], kv[i]->k[layer], kv[i]->v[layer], out[i], 1, nq, kv[i]->nkv,
                            kv[i]->hd[layer], seq_k[i], scale_override, window);
    return late_error();
}

int wr_hip_attn_append_decode_batched(uint32_t n, wr_hip_kv *const *kv, uint32_t layer,
                                      const uint32_t *pos, const float *const *k,
                                      const float *const *v, const float *const *q,
                                      float *const *out, uint32_t nq, float scale_override,
                                      uint32_t window)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!kv || !pos || !k || !v || !q || !out) return WR_HIP_ERR_INVAL;
    if (n == 0 || n > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    uint32_t seq_k[WR_HIP_BATCH_MAX];
    for (uint32_t i = 0; i < n; i++) {
        if (!k[i] || !v[i] || !q[i] || !out[i] || !layer_ok(kv[i], layer)) return WR_HIP_ERR_INVAL;
        if (pos[i] >= kv[i]->max_ctx) return WR_HIP_ERR_CTX_FULL;
        seq_k[i] = pos[i] + 1;
    }
    g_calls += n;
    for (uint32_t i = 0; i < n; i++) {
        int rc = check_decode(kv[i], layer, seq_k[i], nq);
        if (rc) return rc;
        for (uint32_t j = 0; j < i; j++)
            if (kv[i] == kv[j]) return WR_HIP_ERR_INVAL;
    }
    for (uint32_t i = 0; i < n; i++) {
        int rc = wr_hip_attn_append(kv[i], layer, pos[i], 1, k[i], v[i]);
        if (rc) return rc;
        wro_attention_f16kv(q[i], kv[i]->k[layer], kv[i]->v[layer], out[i], 1, nq, kv[i]->nkv,
                            kv[i]->hd[layer], seq_k[i], scale_override, window);
    }
    return late_error();
}

int wr_hip_attn_append_decode(wr_hip_kv *kv, uint32_t layer, uint32_t pos, const float *k,
                              const float *v, const float *q, float *out, uint32_t nq,
                              float scale_override, uint32_t window)
{
    return wr_hip_attn_append_decode_batched(1, &kv, layer, &pos, &k, &v, &q, &out, nq, scale_override,
                                             window);
}

int wr_hip_attn_prefill(wr_hip_kv *kv, uint32_t layer, uint32_t p0, uint32_t T, const float *q,
                        float *out, uint32_t nq, float scale_override, uint32_t window)
{
    if (!g_inited) return WR_HIP_ERR_STATE;
    if (!kv || !q || !out) return WR_HIP_ERR_INVAL;
    g_calls += T;
    if (!layer_ok(kv, layer) || T == 0) return WR_HIP_ERR_INVAL;
    if (nq == 0 || nq % kv->nkv) return WR_HIP_ERR_INVAL;
    if ((uint64_t)p0 + T > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    if ((uint64_t)p0 + T > kv->max_ctx) return WR_HIP_ERR_INVAL;
    wro_causal_prefill(q, kv->k[layer], kv->v[layer], out, p0, T, nq, kv->nkv, kv->hd[layer],
                       scale_override, window);
    return late_error();
}

/* ---- not offered by the test double -----------------------------------------
 * The host engine asks wr_hip_attn_caps() before it uses any of these and keeps
 * its own CPU walk when the answer is 0; they exist so the engine links. */
uint32_t wr_hip_attn_caps(void) { return 0; }
void wr_hip_attn_set_tuning(uint32_t keys_per_wg, int force_generic) { (void)keys_per_wg; (void)force_generic; }
void wr_hip_attn_set_prefill_one_wave(int on) { (void)on; }
void *wr_hip_attn_dev_alloc(size_t bytes) { (void)bytes; return NULL; }
void wr_hip_attn_dev_free(void *p) { (void)p; }
int wr_hip_attn_h2d(void *d, const void *s, size_t n) { (void)d; (void)s; (void)n; return WR_HIP_ERR_STATE; }
int wr_hip_attn_d2h(void *d, const void *s, size_t n) { (void)d; (void)s; (void)n; return WR_HIP_ERR_STATE; }
int wr_hip_attn_sync(void) { return WR_HIP_ERR_STATE; }
int wr_hip_attn_append_dev(wr_hip_kv *kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                           const float *k, const float *v)
{
    (void)kv; (void)layer; (void)pos; (void)n_rows; (void)k; (void)v;
    return WR_HIP_ERR_STATE;
}
int wr_hip_attn_append_batched_dev(uint32_t n, wr_hip_kv *const *kv, uint32_t layer,
                                   const uint32_t *pos, const float *k, const float *v)
{
    (void)n; (void)kv; (void)layer; (void)pos; (void)k; (void)v;
    return WR_HIP_ERR_STATE;
}
int wr_hip_attn_decode_batched_dev(uint32_t n, wr_hip_kv *const *kv, uint32_t layer,
                                   const uint32_t *seq_k, const float *q, float *out, uint32_t nq,
                                   float scale_override, uint32_t window)
{
    (void)n; (void)kv; (void)layer; (void)seq_k; (void)q; (void)out; (void)nq; (void)scale_override;
    (void)window;
    return WR_HIP_ERR_STATE;
}
int wr_hip_attn_append_decode_batched_dev(uint32_t n, wr_hip_kv *const *kv, uint32_t layer,
                                          const uint32_t *pos, const float *qkv, uint32_t ld, uint32_t nq,
                                          const float *q_norm, const float *k_norm, float eps,
                                          const float *cos_sin, uint32_t n_rot, float *out,
                                          float scale_override, uint32_t window)
{
    (void)n; (void)kv; (void)layer; (void)pos; (void)qkv; (void)ld; (void)nq; (void)q_norm; (void)k_norm;
    (void)eps; (void)cos_sin; (void)n_rot; (void)out; (void)scale_override; (void)window;
    return WR_HIP_ERR_STATE;
}
int wr_hip_attn_rope_table_dev(float *cos_sin, uint32_t rows, uint32_t pos0, const uint32_t *pos,
                               uint32_t hd, float theta_base, uint32_t n_rot_pairs)
{
    (void)cos_sin; (void)rows; (void)pos0; (void)pos; (void)hd; (void)theta_base; (void)n_rot_pairs;
    return WR_HIP_ERR_STATE;
}
int wr_hip_attn_prefill_dev(wr_hip_kv *kv, uint32_t layer, uint32_t p0, uint32_t T, const float *q,
                            float *out, uint32_t nq, float scale_override, uint32_t window)
{
    (void)kv; (void)layer; (void)p0; (void)T; (void)q; (void)out; (void)nq; (void)scale_override;
    (void)window;
    return WR_HIP_ERR_STATE;
}
int wr_hip_proj_weight_create(uint32_t n_parts, const uint16_t *const *parts, const uint32_t *rows,
                              uint32_t n_in, wr_hip_weight **out)
{
    (void)n_parts; (void)parts; (void)rows; (void)n_in;
    if (out) *out = NULL;
    return WR_HIP_ERR_STATE;
}
void wr_hip_proj_weight_destroy(wr_hip_weight *w) { (void)w; }
int wr_hip_proj_rows_dev(const wr_hip_weight *w, uint32_t rows, const float *x, uint32_t ldx,
                         const float *add, float *y, uint32_t ldy)
{
    (void)w; (void)rows; (void)x; (void)ldx; (void)add; (void)y; (void)ldy;
    return WR_HIP_ERR_STATE;
}
int wr_hip_proj_rows_norm_dev(const wr_hip_weight *w, uint32_t rows, const float *x, uint32_t ldx,
                              const float *nw, float eps, const float *add, float *y, uint32_t ldy)
{
    (void)w; (void)rows; (void)x; (void)ldx; (void)nw; (void)eps; (void)add; (void)y; (void)ldy;
    return WR_HIP_ERR_STATE;
}
int wr_hip_proj_rows_swiglu_dev(const wr_hip_weight *w, uint32_t rows, const float *gu, uint32_t ld,
                                const float *add, float *y, uint32_t ldy)
{
    (void)w; (void)rows; (void)gu; (void)ld; (void)add; (void)y; (void)ldy;
    return WR_HIP_ERR_STATE;
}
int wr_hip_rows_rmsnorm_dev(const float *x, uint32_t ldx, const float *w, uint32_t wn, float *out,
                            uint32_t ldo, uint32_t rows, uint32_t dim, float eps)
{
    (void)x; (void)ldx; (void)w; (void)wn; (void)out; (void)ldo; (void)rows; (void)dim; (void)eps;
    return WR_HIP_ERR_STATE;
}
int wr_hip_rows_qkv_prep_dev(const float *qkv, uint32_t ld, uint32_t rows, uint32_t nq, uint32_t nkv,
                             uint32_t hd, const float *qn, const float *kn, float eps,
                             const float *cs, uint32_t n_rot, float *q, float *k, float *v)
{
    (void)qkv; (void)ld; (void)rows; (void)nq; (void)nkv; (void)hd; (void)qn; (void)kn; (void)eps;
    (void)cs; (void)n_rot; (void)q; (void)k; (void)v;
    return WR_HIP_ERR_STATE;
}
void *wr_hip_attn_host_alloc(size_t bytes) { return malloc(bytes); }
void wr_hip_attn_host_free(void *p) { free(p); }
int wr_hip_rows_qkv_append_dev(const float *qkv, uint32_t ld, uint32_t rows, uint32_t nq,
                               const float *qn, const float *kn, float eps, const float *cs,
                               uint32_t n_rot, uint32_t n_kv, wr_hip_kv *const *kv, uint32_t layer,
                               const uint32_t *pos, float *q, uint32_t flags)
{
    (void)qkv; (void)ld; (void)rows; (void)nq; (void)qn; (void)kn; (void)eps; (void)cs; (void)n_rot;
    (void)n_kv; (void)kv; (void)layer; (void)pos; (void)q; (void)flags;
    return WR_HIP_ERR_STATE;
}
int wr_hip_rows_qkv_append_q16_dev(const float *qkv, uint32_t ld, uint32_t rows, uint32_t nq,
                                   const float *qn, const float *kn, float eps, const float *cs,
                                   uint32_t n_rot, uint32_t n_kv, wr_hip_kv *const *kv, uint32_t layer,
                                   const uint32_t *pos, uint16_t *q16, float scale_override, uint32_t flags)
{
    (void)qkv; (void)ld; (void)rows; (void)nq; (void)qn; (void)kn; (void)eps; (void)cs; (void)n_rot;
    (void)n_kv; (void)kv; (void)layer; (void)pos; (void)q16; (void)scale_override; (void)flags;
    return WR_HIP_ERR_STATE;
}
int wr_hip_attn_prefill_q16_dev(wr_hip_kv *kv, uint32_t layer, uint32_t p0, uint32_t T, const uint16_t *q16,
                                float *out, uint32_t nq, float scale_override, uint32_t window)
{
    (void)kv; (void)layer; (void)p0; (void)T; (void)q16; (void)out; (void)nq; (void)scale_override;
    (void)window;
    return WR_HIP_ERR_STATE;
}
int wr_hip_rows_rmsnorm_add_dev(const float *x, uint32_t ldx, const float *w, uint32_t wn, float *acc,
                                uint32_t lda, uint32_t rows, uint32_t dim, float eps)
{
    (void)x; (void)ldx; (void)w; (void)wn; (void)acc; (void)lda; (void)rows; (void)dim; (void)eps;
    return WR_HIP_ERR_STATE;
}
int wr_hip_proj_rows_geglu_dev(const wr_hip_weight *w, uint32_t rows, const float *gu, uint32_t ld,
                               const float *add, float *y, uint32_t ldy)
{
    (void)w; (void)rows; (void)gu; (void)ld; (void)add; (void)y; (void)ldy;
    return WR_HIP_ERR_STATE;
}
int wr_hip_rows_swiglu_dev(const float *gu, uint32_t ld, float *act, uint32_t ldo, uint32_t rows,
                           uint32_t ffn)
{
    (void)gu; (void)ld; (void)act; (void)ldo; (void)rows; (void)ffn;
    return WR_HIP_ERR_STATE;
}
