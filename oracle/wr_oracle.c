/*
 * wr_oracle.c — CPU oracle for the GQA attention path.  TEST INFRASTRUCTURE;
 * see wr_oracle.h for the rules on who may use it and how it is pinned.
 *
 * Reference ranges followed (relative to the reference tree):
 *   attention        src/core/kernels.c:1414-1527
 *   F16 codecs       src/core/quant.c:86-136
 *   exp/log/sqrt     src/core/mathx.c:37-110
 *   sin/cos          src/core/mathx.c:121-147
 *   append + cursor  src/core/session.c:139-154, src/core/tensor.c:124-134
 *   prefill loop     src/core/session.c:615-625
 *   batch loop       src/core/batch.c:156-164
 *   RoPE             src/core/kernels.c:1356-1412
 */
#include "wr_oracle.h"

#include <stdlib.h>
#include <string.h>

static uint32_t g_attn_max_seq = 4096;   /* internal.h:187 default */

void wro_set_attn_max_seq(uint32_t cap) { g_attn_max_seq = cap; }
uint32_t wro_get_attn_max_seq(void) { return g_attn_max_seq; }

/* ------------------------------------------------------------------ math -- */

static uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}

static float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* mathx.c:37-57.  Range clamp, nearest-integer split against ln2 with the
 * sign-dependent half, degree-5 polynomial summed left to right in the
 * written association, exponent-field add. */
float wro_exp(float x)
{
    if (x < -88.0f) return 0.0f;
    if (x > 88.0f) return 1e38f;

    const float ln2 = 0.6931471805599453f;
    const float half = (x >= 0) ? 0.5f : -0.5f;
    const int k = (int)(x / ln2 + half);
    const float r = x - (float)k * ln2;

    const float r2 = r * r;
    float e = 1.0f + r;
    e = e + r2 * 0.5f;
    e = e + r2 * r * (1.0f / 6.0f);
    e = e + r2 * r2 * (1.0f / 24.0f);
    e = e + r2 * r2 * r * (1.0f / 120.0f);

    if (k >= -126 && k <= 127)
        e = bits_f32(f32_bits(e) + ((uint32_t)k << 23));
    return e;
}

/* mathx.c:72-86 */
float wro_log(float x)
{
    if (x <= 0.0f) return -1e38f;
    uint32_t u = f32_bits(x);
    const int e = (int)((u >> 23) & 0xFF) - 127;
    const float m = bits_f32((u & 0x007FFFFFu) | 0x3F800000u);
    const float t = (m - 1.0f) / (m + 1.0f);
    const float t2 = t * t;
    const float lnm = 2.0f * t *
        (1.0f + t2 * (1.0f / 3.0f + t2 * (1.0f / 5.0f + t2 * (1.0f / 7.0f))));
    return lnm + (float)e * 0.6931471805599453f;
}

/* mathx.c:98-110: halve-the-bit-pattern seed, four Newton steps. */
float wro_sqrt(float x)
{
    if (x <= 0) return 0;
    float g = bits_f32((f32_bits(x) + 0x3f800000u) >> 1);
    for (int it = 0; it < 4; it++)
        g = 0.5f * (g + x / g);
    return g;
}

static const float ORACLE_PI    = 3.14159265358979f;   /* mathx.c:121 */
static const float ORACLE_TWOPI = 6.28318530717958f;   /* mathx.c:122 */

static float reduce_angle(float x)
{
    while (x >  ORACLE_PI) x -= ORACLE_TWOPI;
    while (x < -ORACLE_PI) x += ORACLE_TWOPI;
    return x;
}

/* mathx.c:124-135 */
float wro_sin(float x)
{
    x = reduce_angle(x);
    const float x2 = x * x;
    const float x3 = x2 * x;
    const float x5 = x3 * x2;
    const float x7 = x5 * x2;
    return x - x3 * (1.0f / 6.0f) + x5 * (1.0f / 120.0f)
             - x7 * (1.0f / 5040.0f);
}

/* mathx.c:137-147 */
float wro_cos(float x)
{
    x = reduce_angle(x);
    const float x2 = x * x;
    const float x4 = x2 * x2;
    const float x6 = x4 * x2;
    return 1.0f - x2 * 0.5f + x4 * (1.0f / 24.0f) - x6 * (1.0f / 720.0f);
}

/* ---------------------------------------------------------------- codecs -- */

/* quant.c:86-114 */
float wro_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    uint32_t e = (h >> 10) & 0x1F;
    uint32_t mant = h & 0x3FF;

    if (e == 0x1F)
        return bits_f32(sign | 0x7F800000u | (mant << 13));
    if (e == 0) {
        if (mant == 0)
            return bits_f32(sign);
        /* subnormal: shift the leading one up to the implicit-bit slot */
        e = 1;
        while ((mant & 0x400) == 0) {
            mant <<= 1;
            e--;                       /* may wrap; the sum below is mod 2^32 */
        }
        mant &= 0x3FF;
    }
    return bits_f32(sign | ((e + 112u) << 23) | (mant << 13));
}

/* quant.c:121-136: truncate the mantissa, flush e<=0 to signed zero,
 * saturate e>=31 (NaN included) to signed infinity. */
uint16_t wro_f32_to_f16(float f)
{
    const uint32_t bits = f32_bits(f);
    const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000);
    const int32_t e = (int32_t)((bits >> 23) & 0xFF) - 112;
    const uint32_t mant = (bits >> 13) & 0x3FF;

    if (e <= 0) return sign;
    if (e >= 31) return (uint16_t)(sign | 0x7C00);
    return (uint16_t)(sign | ((uint32_t)e << 10) | mant);
}

/* ---------------------------------------------------------------- tensor -- */

void wro_tensor_wrap(wro_tensor *t, void *data, uint8_t dtype, uint8_t ndim,
                     const uint32_t *shape, uint16_t flags)
{
    memset(t, 0, sizeof *t);
    uint64_t n = 1;
    for (uint8_t i = 0; i < ndim; i++) {
        t->shape[i] = shape[i];
        n *= shape[i];
    }
    t->data = data;
    t->dtype = dtype;
    t->ndim = ndim;
    t->flags = flags;
    t->size_bytes = n * (dtype == WRO_DTYPE_F32 ? 4u : 2u);
}

/* tensor.c:124-134 */
int wro_tensor_set_valid_rows(wro_tensor *t, uint32_t new_rows)
{
    if (!t) return WRO_ERR_INVAL;
    if (!(t->flags & WRO_TENSOR_GROWABLE)) return WRO_ERR_INVAL;
    if (new_rows > t->shape[0]) return WRO_ERR_INVAL;
    t->valid_rows = new_rows;
    return WRO_OK;
}

/* quant.c:516-523 restricted to the two dtypes on this path. */
static uint64_t elem_capacity(const wro_tensor *t)
{
    if (t->dtype == WRO_DTYPE_F32) return t->size_bytes / 4;
    if (t->dtype == WRO_DTYPE_F16) return t->size_bytes / 2;
    return 0;
}

static uint64_t shape_elems(const wro_tensor *t)
{
    uint64_t n = 1;
    for (uint32_t i = 0; i < t->ndim; i++) n *= t->shape[i];
    return n;
}

/* quant.c:539-552: the accessor decodes F16 through the software codec. */
static inline float load_elem(const void *base, int is_f16, uint64_t i)
{
    if (is_f16)
        return wro_f16_to_f32(((const uint16_t *)base)[i]);
    return ((const float *)base)[i];
}

/* ------------------------------------------------------------- attention -- */

/*
 * One (query row, query head) pass of kernels.c:1480-1521.
 *   qv      hd F32 query values
 *   kbase   first element of this KV head in row 0; row stride `kv_stride`
 * State (m, l, acc[hd]) follows the reference exactly: m starts at the
 * finite sentinel -1e30f; a tile whose running max is still the sentinel
 * forces the rescale factor to 0; masked keys keep score -1e30f and still
 * pass through exp (which clamps to 0 below -88, or yields 1 when the whole
 * tile is masked — wiped by the next live tile).
 */
static void attend_one_head(const float *qv, const void *kdata,
                            const void *vdata, int k_f16, int v_f16,
                            uint64_t head_off, uint64_t kv_stride,
                            uint64_t hd, uint64_t seq_k, uint64_t key_lo,
                            float scale, float *acc, float *dst)
{
    float m = -1e30f;
    float l = 0;
    for (uint64_t d = 0; d < hd; d++) acc[d] = 0.0f;

    for (uint64_t t0 = 0; t0 < seq_k; t0 += WRO_FLASH_BLOCK) {
        uint64_t bn = seq_k - t0;
        if (bn > WRO_FLASH_BLOCK) bn = WRO_FLASH_BLOCK;

        float s[WRO_FLASH_BLOCK];
        float tile_max = -1e30f;
        for (uint64_t b = 0; b < bn; b++) {
            if (t0 + b < key_lo) {
                s[b] = -1e30f;
                continue;
            }
            const uint64_t kr = (t0 + b) * kv_stride + head_off;
            float dot = 0;
            for (uint64_t d = 0; d < hd; d++)
                dot += qv[d] * load_elem(kdata, k_f16, kr + d);
            s[b] = dot * scale;
            if (s[b] > tile_max) tile_max = s[b];
        }

        const float m_new = (m > tile_max) ? m : tile_max;
        const float a = (m == -1e30f) ? 0.0f : wro_exp(m - m_new);
        for (uint64_t d = 0; d < hd; d++) acc[d] *= a;
        l *= a;

        for (uint64_t b = 0; b < bn; b++) {
            const float pw = wro_exp(s[b] - m_new);
            l += pw;
            const uint64_t vr = (t0 + b) * kv_stride + head_off;
            for (uint64_t d = 0; d < hd; d++)
                acc[d] += pw * load_elem(vdata, v_f16, vr + d);
        }
        m = m_new;
    }

    const float inv = (l > 0) ? 1.0f / l : 0.0f;
    for (uint64_t d = 0; d < hd; d++) dst[d] = acc[d] * inv;
}

static float resolve_scale(float scale_override, uint64_t hd)
{
    /* kernels.c:1457-1459 */
    return (scale_override > 0.0f) ? scale_override
                                   : 1.0f / wro_sqrt((float)hd);
}

static uint64_t resolve_key_lo(uint32_t window, uint64_t seq_k)
{
    /* kernels.c:1463-1464 */
    return (window > 0 && seq_k > (uint64_t)window) ? seq_k - window : 0;
}

/* Loop nest kernels.c:1475-1523 over raw buffers. */
static int attention_core(const void *q, int q_f16, const void *k, int k_f16,
                          const void *v, int v_f16, void *out, int out_f16,
                          uint64_t seq_q, uint64_t nq, uint64_t nkv,
                          uint64_t hd, uint64_t seq_k, float scale_override,
                          uint32_t window)
{
    const uint64_t group = nq / nkv;
    const float scale = resolve_scale(scale_override, hd);
    const uint64_t key_lo = resolve_key_lo(window, seq_k);

    float *acc = (float *)malloc((size_t)hd * sizeof(float) * 3);
    if (!acc) return WRO_ERR_NOMEM;
    float *qv = acc + hd;
    float *res = qv + hd;

    for (uint64_t qs = 0; qs < seq_q; qs++) {
        for (uint64_t qh = 0; qh < nq; qh++) {
            const uint64_t kvh = qh / group;
            const uint64_t row = (qs * nq + qh) * hd;
            for (uint64_t d = 0; d < hd; d++)
                qv[d] = load_elem(q, q_f16, row + d);
            attend_one_head(qv, k, v, k_f16, v_f16, kvh * hd, nkv * hd, hd,
                            seq_k, key_lo, scale, acc, res);
            if (out_f16) {
                for (uint64_t d = 0; d < hd; d++)
                    ((uint16_t *)out)[row + d] = wro_f32_to_f16(res[d]);
            } else {
                memcpy((float *)out + row, res, (size_t)hd * sizeof(float));
            }
        }
    }
    free(acc);
    return WRO_OK;
}

int wro_op_gqa_attention(const wro_tensor *Q, const wro_tensor *K,
                         const wro_tensor *V, wro_tensor *C,
                         float scale_override, uint32_t window,
                         uint64_t *calls_counter)
{
    /* kernels.c:1418-1421 */
    if (!Q || !K || !V || !C || !Q->data || !K->data || !V->data || !C->data)
        return WRO_ERR_INVAL;
    if (Q->ndim < 3 || K->ndim < 3 || V->ndim < 3)
        return WRO_ERR_INVAL;

    /* kernels.c:1423 */
    if (calls_counter)
        __atomic_fetch_add(calls_counter, 1, __ATOMIC_RELAXED);

    /* kernels.c:1425-1434 */
    const uint64_t seq_q = Q->shape[0];
    const uint64_t nq = Q->shape[1];
    const uint64_t hd = Q->shape[2];
    const uint64_t nkv = K->shape[1];
    if (nq == 0 || nkv == 0 || hd == 0 || seq_q == 0) return WRO_ERR_INVAL;
    if (nq % nkv != 0) return WRO_ERR_INVAL;
    if (K->shape[2] != hd || V->shape[2] != hd || V->shape[1] != nkv)
        return WRO_ERR_INVAL;

    /* kernels.c:1437-1440: a GROWABLE cache exposes valid_rows, except that
     * a zero cursor falls back to the allocated row count. */
    const uint64_t seq_k =
        ((K->flags & WRO_TENSOR_GROWABLE) && K->valid_rows > 0)
            ? K->valid_rows : K->shape[0];
    if (seq_k == 0) return WRO_ERR_INVAL;

    /* kernels.c:1444-1447 */
    if (seq_k > g_attn_max_seq) return WRO_ERR_LIMIT;
    if (hd > WRO_FLASH_D_MAX) return WRO_ERR_LIMIT;

    /* kernels.c:1449-1454 */
    if (elem_capacity(Q) < seq_q * nq * hd ||
        elem_capacity(K) < seq_k * nkv * hd ||
        elem_capacity(V) < seq_k * nkv * hd ||
        elem_capacity(C) < seq_q * nq * hd ||
        shape_elems(C) < seq_q * nq * hd)
        return WRO_ERR_INVAL;

    return attention_core(Q->data, Q->dtype == WRO_DTYPE_F16,
                          K->data, K->dtype == WRO_DTYPE_F16,
                          V->data, V->dtype == WRO_DTYPE_F16,
                          C->data, C->dtype == WRO_DTYPE_F16,
                          seq_q, nq, nkv, hd, seq_k, scale_override, window);
}

void wro_attention_f16kv(const float *q, const uint16_t *k, const uint16_t *v,
                         float *out, uint32_t seq_q, uint32_t nq, uint32_t nkv,
                         uint32_t hd, uint32_t seq_k, float scale_override,
                         uint32_t window)
{
    (void)attention_core(q, 0, k, 1, v, 1, out, 0, seq_q, nq, nkv, hd, seq_k,
                         scale_override, window);
}

/* ---------------------------------------------------------------- append -- */

/* session.c:139-154 */
int wro_kv_append_row(wro_tensor *kv, const float *row, uint32_t nkv,
                      uint32_t hd)
{
    if (!kv->data || !row) return WRO_ERR_INTERNAL;
    const uint32_t at = kv->valid_rows;
    if (at >= kv->shape[0]) return WRO_ERR_CTX_FULL;
    const uint64_t n = (uint64_t)nkv * hd;
    if (((uint64_t)at + 1u) * n * 2u > kv->size_bytes) return WRO_ERR_INTERNAL;
    uint16_t *dst = (uint16_t *)kv->data + (uint64_t)at * n;
    for (uint64_t i = 0; i < n; i++) dst[i] = wro_f32_to_f16(row[i]);
    return wro_tensor_set_valid_rows(kv, at + 1) == WRO_OK ? WRO_OK
                                                            : WRO_ERR_INTERNAL;
}

/* -------------------------------------------------- prefill / batch loops -- */

void wro_causal_prefill_rows(const float *q, const uint16_t *k,
                             const uint16_t *v, float *out, uint32_t p0,
                             uint32_t row_lo, uint32_t row_hi, uint32_t nq,
                             uint32_t nkv, uint32_t hd, float scale_override,
                             uint32_t window)
{
    /* session.c:615-625: token i runs a seq_q = 1 body whose cache cursor is
     * p0 + i + 1 (its own row was appended before attention). */
    const uint64_t row_elems = (uint64_t)nq * hd;
    for (uint32_t i = row_lo; i < row_hi; i++)
        (void)attention_core(q + i * row_elems, 0, k, 1, v, 1,
                             out + i * row_elems, 0, 1, nq, nkv, hd,
                             (uint64_t)p0 + i + 1, scale_override, window);
}

void wro_causal_prefill(const float *q, const uint16_t *k, const uint16_t *v,
                        float *out, uint32_t p0, uint32_t T, uint32_t nq,
                        uint32_t nkv, uint32_t hd, float scale_override,
                        uint32_t window)
{
    wro_causal_prefill_rows(q, k, v, out, p0, 0, T, nq, nkv, hd,
                            scale_override, window);
}

void wro_batched_decode(uint32_t n, const float *const *q,
                        const uint16_t *const *k, const uint16_t *const *v,
                        float *const *out, const uint32_t *seq_k, uint32_t nq,
                        uint32_t nkv, uint32_t hd, float scale_override,
                        uint32_t window)
{
    /* batch.c:156-164: sessions in caller order, one body each. */
    for (uint32_t i = 0; i < n; i++)
        (void)attention_core(q[i], 0, k[i], 1, v[i], 1, out[i], 0, 1, nq, nkv,
                             hd, seq_k[i], scale_override, window);
}

/* ------------------------------------------------------------------ RoPE -- */

/* The (cos, sin) pairs wro_rope uses for `seq` rows starting at `pos`
 * (kernels.c:1384-1404, the angle arithmetic lifted out of the rotation):
 * out[s][j] = {cos, sin} for j < n_rot, n_rot as resolved by wro_rope.  Returns
 * n_rot, or a negative status. */
int wro_rope_table(float *out, uint32_t seq, uint32_t hd, uint32_t pos,
                   float theta_base, uint32_t n_rot_pairs)
{
    if (!out || seq == 0) return WRO_ERR_INVAL;
    if (hd < 2 || (hd & 1)) return WRO_ERR_INVAL;
    const uint64_t half = hd / 2;
    if (theta_base < 1.0f) theta_base = 10000.0f;
    const float lnb = wro_log(theta_base);
    uint64_t n_rot = half;
    if (n_rot_pairs >= 1 && (uint64_t)n_rot_pairs < half) n_rot = n_rot_pairs;
    for (uint64_t s = 0; s < seq; s++) {
        const uint64_t p = (uint64_t)pos + s;
        for (uint64_t j = 0; j < n_rot; j++) {
            const float exponent = (float)(2 * j) / (float)hd;
            const float powv = wro_exp(exponent * lnb);
            const float angle = (float)p / powv;
            out[(s * n_rot + j) * 2] = wro_cos(angle);
            out[(s * n_rot + j) * 2 + 1] = wro_sin(angle);
        }
    }
    return (int)n_rot;
}

/* kernels.c:1356-1412 */
int wro_rope(float *x, uint32_t seq, uint32_t heads, uint32_t hd,
             uint32_t pos, float theta_base, uint32_t n_rot_pairs)
{
    if (!x || seq == 0 || heads == 0) return WRO_ERR_INVAL;
    if (hd < 2 || (hd & 1)) return WRO_ERR_INVAL;
    const uint64_t half = hd / 2;

    if (theta_base < 1.0f) theta_base = 10000.0f;
    const float lnb = wro_log(theta_base);

    uint64_t n_rot = half;
    if (n_rot_pairs >= 1 && (uint64_t)n_rot_pairs < half) n_rot = n_rot_pairs;

    for (uint64_t s = 0; s < seq; s++) {
        const uint64_t p = (uint64_t)pos + s;
        for (uint64_t h = 0; h < heads; h++) {
            float *r = x + (s * heads + h) * hd;
            for (uint64_t j = 0; j < n_rot; j++) {
                const float x0 = r[j];
                const float x1 = r[j + half];
                const float exponent = (float)(2 * j) / (float)hd;
                const float powv = wro_exp(exponent * lnb);
                const float angle = (float)p / powv;
                const float cs = wro_cos(angle);
                const float sn = wro_sin(angle);
                r[j] = x0 * cs - x1 * sn;
                r[j + half] = x0 * sn + x1 * cs;
            }
        }
    }
    return WRO_OK;
}

/* ------------------------------------------------------------------------
 * Projections.  The reference widens F16 weights to F32 when it loads them
 * (src/core/loader.c:164-190) and multiplies activation rows with the
 * GGML-layout weight W[out][in] in F32 (wri_op_matmul, src/core/kernels.c,
 * GGML branch).  Its inner loop is chosen at run time from a scalar, an AVX2
 * and an AVX-512 variant that sum in different orders (kernels.c:124-137,
 * 273-340), so its own results differ in the last bits from host to host; the
 * restatement follows the scalar variant (kernels.c:124-137): one running F32
 * sum per output, inputs in ascending order, product and sum rounded
 * separately.
 * ---------------------------------------------------------------------- */
int wro_matmul_w16(const float *a, const uint16_t *w_f16, float *c, uint32_t M,
                   uint32_t K, uint32_t N)
{
    if (!a || !w_f16 || !c || M == 0 || K == 0 || N == 0) return WRO_ERR_INVAL;
    for (uint32_t i = 0; i < M; i++) {
        const float *arow = a + (size_t)i * K;
        for (uint32_t j = 0; j < N; j++) {
            const uint16_t *wrow = w_f16 + (size_t)j * K;
            float sum = 0;
            for (uint32_t k = 0; k < K; k++)
                sum += arow[k] * wro_f16_to_f32(wrow[k]);
            c[(size_t)i * N + j] = sum;
        }
    }
    return WRO_OK;
}

/* Weighted RMS normalisation of `rows` rows of `dim` values, w indexed modulo
 * wn (wn == 0: no weight).  src/core/kernels.c:1276-1316. */
int wro_rmsnorm(const float *x, const float *w, uint32_t wn, float *out,
                uint32_t rows, uint32_t dim, float eps)
{
    if (!x || !out || dim == 0) return WRO_ERR_INVAL;
    if (wn > 0 && !w) return WRO_ERR_INVAL;
    for (uint32_t r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * dim;
        float sumsq = 0;
        for (uint32_t j = 0; j < dim; j++) {
            const float v = xr[j];
            sumsq += v * v;
        }
        const float inv_rms = 1.0f / wro_sqrt(sumsq / (float)dim + eps);
        for (uint32_t j = 0; j < dim; j++) {
            const float v = xr[j];
            const float ww = (wn > 0) ? w[j % wn] : 1.0f;
            out[(size_t)r * dim + j] = v * inv_rms * ww;
        }
    }
    return WRO_OK;
}

/* Gated activation, src/core/kernels.c:1243-1258 with silu at :963-967:
 * out[i] = (g[i] * (1 / (1 + exp(-g[i])))) * u[i], exp being the polynomial. */
int wro_silu_mul(const float *g, const float *u, float *out, uint64_t n)
{
    if (!g || !u || !out) return WRO_ERR_INVAL;
    for (uint64_t i = 0; i < n; i++) {
        const float a = g[i];
        const float sig = 1.0f / (1.0f + wro_exp(-a));
        out[i] = (a * sig) * u[i];
    }
    return WRO_OK;
}
