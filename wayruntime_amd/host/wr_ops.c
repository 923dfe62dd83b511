/*
 * wr_ops.c — the CPU ops around the attention path (host glue): embedding
 * fetch, RMSNorm, weight matmul, RoPE, SwiGLU, residual add.
 *
 * Formulas follow the reference ops (reference: src/core/kernels.c:1276-1313
 * RMSNorm, :1356-1412 RoPE, :963-967 and :1243-1258 SwiGLU, :1529-1574 embed,
 * :124-137 weight matmul W[out][in]).  Everything is row-wise; matmul reduces
 * each output column whole inside one thread, so a row's result does not
 * depend on how many rows travel together or on the thread count — the
 * property the reference's N-split gives it (src/core/internal.h:269-281).
 * The reduction ORDER inside a column is this file's own (8-lane AVX2 FMA),
 * not the reference's, so logits agree to rounding, not bit for bit.
 */
#include "wr_host.h"

#include <stdlib.h>
#include <string.h>

#if defined(__AVX2__) && defined(__FMA__) && defined(__F16C__)
#include <immintrin.h>
#define WRH_AVX2 1
#else
#define WRH_AVX2 0
#endif

/* binary16 -> binary32, exact (subnormals included). */
static inline float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FF, bits;
    if (e == 0x1F) {
        bits = sign | 0x7F800000u | (m << 13);
    } else if (e != 0) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0) {
        bits = sign;
    } else {
        e = 113;
        while (!(m & 0x400)) {
            m <<= 1;
            e--;
        }
        bits = sign | (e << 23) | ((m & 0x3FF) << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static void widen_row(const wrh_weight *w, uint32_t row, float *dst)
{
    const uint32_t n = w->cols;
    if (!w->is_f16) {
        memcpy(dst, (const float *)w->data + (size_t)row * n, (size_t)n * 4);
        return;
    }
    const uint16_t *src = (const uint16_t *)w->data + (size_t)row * n;
    uint32_t i = 0;
#if WRH_AVX2
    for (; i + 8 <= n; i += 8)
        _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(src + i))));
#endif
    for (; i < n; i++) dst[i] = half_to_float(src[i]);
}

int wrh_embed(const wrh_weight *table, uint32_t token, float *out_row)
{
    if (!table->data || !out_row) return WR_ERR_INVAL;
    if (token >= table->rows) return WR_ERR_INVAL;        /* never clamped */
    widen_row(table, token, out_row);
    return WR_OK;
}

void wrh_rmsnorm(const float *x, const float *w, uint32_t wn, float *out, uint32_t rows,
                 uint32_t dim, float eps)
{
    for (uint32_t r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * dim;
        float *orow = out + (size_t)r * dim;
        float sumsq = 0;
        for (uint32_t j = 0; j < dim; j++) sumsq += xr[j] * xr[j];
        const float inv_rms = 1.0f / wrh_sqrt(sumsq / (float)dim + eps);
        for (uint32_t j = 0; j < dim; j++) {
            const float wj = (wn > 0) ? w[j % wn] : 1.0f;
            orow[j] = xr[j] * inv_rms * wj;
        }
    }
}

/* Fixed-order dot product: four 8-lane FMA accumulators over strides of 32,
 * an 8-lane tail, then a scalar tail; lanes are summed in one fixed tree. */
static inline float dot_f32(const float *a, const float *b, uint32_t n)
{
#if WRH_AVX2
    __m256 s0 = _mm256_setzero_ps(), s1 = s0, s2 = s0, s3 = s0;
    uint32_t k = 0;
    for (; k + 32 <= n; k += 32) {
        s0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + k), _mm256_loadu_ps(b + k), s0);
        s1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + k + 8), _mm256_loadu_ps(b + k + 8), s1);
        s2 = _mm256_fmadd_ps(_mm256_loadu_ps(a + k + 16), _mm256_loadu_ps(b + k + 16), s2);
        s3 = _mm256_fmadd_ps(_mm256_loadu_ps(a + k + 24), _mm256_loadu_ps(b + k + 24), s3);
    }
    for (; k + 8 <= n; k += 8)
        s0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + k), _mm256_loadu_ps(b + k), s0);
    const __m256 s = _mm256_add_ps(_mm256_add_ps(s0, s1), _mm256_add_ps(s2, s3));
    float lanes[8];
    _mm256_storeu_ps(lanes, s);
    float sum = ((lanes[0] + lanes[4]) + (lanes[1] + lanes[5])) +
                ((lanes[2] + lanes[6]) + (lanes[3] + lanes[7]));
    for (; k < n; k++) sum += a[k] * b[k];
    return sum;
#else
    float sum = 0;
    for (uint32_t k = 0; k < n; k++) sum += a[k] * b[k];
    return sum;
#endif
}

void wrh_matmul(wr_engine *e, const float *A, uint32_t R, uint32_t lda, const wrh_weight *W,
                float *C, uint32_t ldc)
{
    const uint32_t N = W->rows, K = W->cols;
    const int threads = (e && e->n_threads > 0) ? e->n_threads : 1;
    if (e) {
        __atomic_fetch_add(&e->ctr[WR_CTR_MATMUL_CALLS], 1, __ATOMIC_RELAXED);
        __atomic_fetch_add(&e->ctr[WR_CTR_MATMUL_ELEMS], (uint64_t)R * N, __ATOMIC_RELAXED);
        __atomic_fetch_add(&e->ctr[WR_CTR_MATMUL_PAR_N], 1, __ATOMIC_RELAXED);
    }
#pragma omp parallel num_threads(threads)
    {
        float *wrow = (float *)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (uint32_t j = 0; j < N; j++) {
            const float *wr;
            if (!W->is_f16) {
                wr = (const float *)W->data + (size_t)j * K;
            } else if (wrow) {
                widen_row(W, j, wrow);
                wr = wrow;
            } else {
                /* no scratch: widen element by element (same values, same order) */
                const uint16_t *hw = (const uint16_t *)W->data + (size_t)j * K;
                for (uint32_t r = 0; r < R; r++) {
                    float sum = 0;
                    for (uint32_t k = 0; k < K; k++)
                        sum += A[(size_t)r * lda + k] * half_to_float(hw[k]);
                    C[(size_t)r * ldc + j] = sum;
                }
                continue;
            }
            for (uint32_t r = 0; r < R; r++)
                C[(size_t)r * ldc + j] = dot_f32(A + (size_t)r * lda, wr, K);
        }
        free(wrow);
    }
}

/* One row [heads][hd] rotated in place at absolute position pos: pair
 * (j, j + hd/2), angle pos / theta^(2j/hd) through the polynomial exp / sin /
 * cos; pairs at or above n_rot pass through. */
void wrh_rope(float *x, uint32_t heads, uint32_t hd, uint32_t pos, float theta,
              uint32_t n_rot_pairs)
{
    const uint32_t half = hd / 2;
    if (theta < 1.0f) theta = 10000.0f;
    const float lnb = wrh_log(theta);
    uint32_t n_rot = half;
    if (n_rot_pairs >= 1 && n_rot_pairs < half) n_rot = n_rot_pairs;
    for (uint32_t j = 0; j < n_rot; j++) {
        const float exponent = (float)(2 * j) / (float)hd;
        const float powv = wrh_exp(exponent * lnb);
        const float angle = (float)pos / powv;
        const float cs = wrh_cos(angle), sn = wrh_sin(angle);
        for (uint32_t h = 0; h < heads; h++) {
            float *r = x + (size_t)h * hd;
            const float x0 = r[j], x1 = r[j + half];
            r[j] = x0 * cs - x1 * sn;
            r[j + half] = x0 * sn + x1 * cs;
        }
    }
}

/* The (cos, sin) pairs wrh_rope uses at position pos: cos_sin[j] = {cos, sin}
 * for j < n_rot (returned; n_rot <= hd/2). */
uint32_t wrh_rope_table(float *cos_sin, uint32_t hd, uint32_t pos, float theta,
                        uint32_t n_rot_pairs)
{
    const uint32_t half = hd / 2;
    if (theta < 1.0f) theta = 10000.0f;
    const float lnb = wrh_log(theta);
    uint32_t n_rot = half;
    if (n_rot_pairs >= 1 && n_rot_pairs < half) n_rot = n_rot_pairs;
    for (uint32_t j = 0; j < n_rot; j++) {
        const float exponent = (float)(2 * j) / (float)hd;
        const float powv = wrh_exp(exponent * lnb);
        const float angle = (float)pos / powv;
        cos_sin[2 * j] = wrh_cos(angle);
        cos_sin[2 * j + 1] = wrh_sin(angle);
    }
    return n_rot;
}

void wrh_rope_apply(float *x, uint32_t heads, uint32_t hd, const float *cos_sin, uint32_t n_rot)
{
    const uint32_t half = hd / 2;
    for (uint32_t j = 0; j < n_rot; j++) {
        const float cs = cos_sin[2 * j], sn = cos_sin[2 * j + 1];
        for (uint32_t h = 0; h < heads; h++) {
            float *r = x + (size_t)h * hd;
            const float x0 = r[j], x1 = r[j + half];
            r[j] = x0 * cs - x1 * sn;
            r[j + half] = x0 * sn + x1 * cs;
        }
    }
}

void wrh_swiglu(wr_engine *e, float *gate, const float *up, uint64_t n)
{
    if (e) __atomic_fetch_add(&e->ctr[WR_CTR_FUSED_CALLS], 1, __ATOMIC_RELAXED);
    for (uint64_t i = 0; i < n; i++) {
        const float a = gate[i];
        const float sig = 1.0f / (1.0f + wrh_exp(-a));
        gate[i] = (a * sig) * up[i];
    }
}

/* GeGLU, gelu_pytorch_tanh(gate) * up (reference: src/core/kernels.c:969-976 and
 * wri_op_fused_gelu_mul). */
void wrh_geglu(wr_engine *e, float *gate, const float *up, uint64_t n)
{
    if (e) __atomic_fetch_add(&e->ctr[WR_CTR_FUSED_CALLS], 1, __ATOMIC_RELAXED);
    for (uint64_t i = 0; i < n; i++) {
        const float x = gate[i];
        const float x3 = x * x * x;
        const float z = 0.7978845608f * (x + 0.044715f * x3);
        gate[i] = 0.5f * x * (1.0f + wrh_tanh(z)) * up[i];
    }
}

/* x = cap * tanh(x / cap): divides, as the reference does (src/core/kernels.c:1576-1584) */
void wrh_softcap(float *x, uint64_t n, float cap)
{
    if (!x || cap <= 0.0f) return;
    for (uint64_t i = 0; i < n; i++) x[i] = cap * wrh_tanh(x[i] / cap);
}

void wrh_scale(float *x, uint64_t n, float s)
{
    for (uint64_t i = 0; i < n; i++) x[i] *= s;
}

void wrh_add(float *acc, const float *x, uint64_t n)
{
    for (uint64_t i = 0; i < n; i++) acc[i] = acc[i] + x[i];
}
