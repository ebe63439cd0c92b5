/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.  See llama2j_oracle.h.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp (see Makefile).
 * Java float arithmetic is strict IEEE binary32 per operation with no fused
 * multiply-add, so every intermediate below that is a Java `float` is a C
 * `float`, contraction is off, and no sum is reassociated.
 */
#include "llama2j_oracle.h"

#include <float.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ */
/* Java semantics helpers                                              */
/* ------------------------------------------------------------------ */

/* K/Kernel.java:221-227, J/Quant.java:110-116: big-endian bytes -> float */
static inline float be_float(const uint8_t *b)
{
    uint32_t u = ((uint32_t)b[0] << 24) | ((uint32_t)b[1] << 16) | ((uint32_t)b[2] << 8) | (uint32_t)b[3];
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline void put_be_float(uint8_t *b, float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    b[0] = (uint8_t)(u >> 24);
    b[1] = (uint8_t)(u >> 16);
    b[2] = (uint8_t)(u >> 8);
    b[3] = (uint8_t)u;
}

/* java.lang.Math.round(float): floor(x + 1/2) without double rounding, NaN -> 0,
 * saturating at the int range.  The sum is exact in double for every float. */
static inline int32_t java_round_float(float x)
{
    if (x != x) return 0;
    double r = floor((double)x + 0.5);
    if (r >= 2147483647.0) return 2147483647;
    if (r <= -2147483648.0) return (int32_t)(-2147483647 - 1);
    return (int32_t)r;
}

/* java.lang.Math.max(float,float): NaN wins, +0 > -0 */
static inline float java_maxf(float a, float b)
{
    if (a != a) return a;
    if (a == 0.0f && b == 0.0f) return signbit(a) ? b : a;
    return (a >= b) ? a : b;
}

/* ------------------------------------------------------------------ */
/* codec: J/Quant.java                                                  */
/* ------------------------------------------------------------------ */

int64_t orc_quant_nbytes(int64_t n_floats)
{
    /* J/Quant.java:39-48 */
    int64_t groups = (n_floats + ORC_GROUP_SIZE - 1) / ORC_GROUP_SIZE;
    return groups * ORC_GROUP_BYTES;
}

void orc_quant_encode(const float *in, int64_t n, uint8_t *out)
{
    /* J/Quant.java:156-193 */
    int64_t chunks = (n + ORC_GROUP_SIZE - 1) / ORC_GROUP_SIZE;
#pragma omp parallel for schedule(static) if (chunks > 64)
    for (int64_t chunk = 0; chunk < chunks; chunk++) {
        int64_t i = chunk * ORC_GROUP_SIZE;
        uint8_t *o = out + chunk * ORC_GROUP_BYTES;
        float mn = in[i];
        float mx = mn;
        for (int j = 1; j < ORC_GROUP_SIZE; j++) {
            if (i + j < n) {
                if (in[i + j] < mn) mn = in[i + j];
                if (in[i + j] > mx) mx = in[i + j];
            }
        }
        float range = mx - mn;
        put_be_float(o, mn);
        put_be_float(o + 4, mx);
        for (int j = 0; j < ORC_GROUP_SIZE; j++) {
            if (i + j < n) {
                float t = in[i + j] - mn;
                t = t / range;
                t = t * 255.0f;
                o[8 + j] = (uint8_t)java_round_float(t);
            } else {
                o[8 + j] = 0;
            }
        }
    }
}

void orc_quant_decode(const uint8_t *enc, int64_t float_index, int64_t size, float *out)
{
    /* J/Quant.java:79-108 */
    if (size <= 0) return;
    int64_t g0 = float_index / ORC_GROUP_SIZE;
    int64_t g1 = (float_index + size - 1) / ORC_GROUP_SIZE;
    int64_t o = 0;
    for (int64_t g = g0; g <= g1; g++) {
        const uint8_t *base = enc + g * ORC_GROUP_BYTES;
        float mn = be_float(base);
        float mx = be_float(base + 4);
        float range = mx - mn;
        int64_t start = g * ORC_GROUP_SIZE;
        for (int j = 0; j < ORC_GROUP_SIZE; j++) {
            int64_t jj = start + j;
            if (jj >= float_index && jj < float_index + size) {
                int bv = base[8 + j];
                float value = (float)bv / 255.0f * range + mn;
                out[o++] = value;
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* ops                                                                  */
/* ------------------------------------------------------------------ */

void orc_rms(float *sum, const float *x, int size)
{
    /* K/RootMeanSquare.java:25-35 */
    float ss = 0.0f;
    for (int j = 0; j < size; j++) ss += x[j] * x[j];
    ss /= (float)size;
    ss += 1e-5f;
    ss = 1.0f / (float)sqrt((double)ss);
    sum[0] = ss;
}

void orc_wns_i8(float *out, const float *x, const uint8_t *enc, int64_t weight_index,
                const float *sum_of_squares, int size)
{
    /* K/WeightNormalizeAndScale.java:32-77 */
    float ss = sum_of_squares[0];
    int64_t g0 = weight_index / ORC_GROUP_SIZE;
    int64_t g1 = (weight_index + size - 1) / ORC_GROUP_SIZE;
    for (int64_t g = g0; g <= g1; g++) {
        const uint8_t *base = enc + g * ORC_GROUP_BYTES;
        float mn = be_float(base);
        float mx = be_float(base + 4);
        float range = mx - mn;
        int64_t start = g * ORC_GROUP_SIZE;
        for (int j = 0; j < ORC_GROUP_SIZE; j++) {
            int64_t index = start + j;
            if (index >= weight_index + size) break;
            if (index >= weight_index) {
                int64_t off = index - weight_index;
                int bv = base[8 + j];
                float value = (float)bv / 255.0f * range + mn;
                out[off] = value * (ss * x[off]);
            }
        }
    }
}

void orc_matmul_i8_unaligned(float *xout, const float *x, const uint8_t *enc,
                             int64_t weight_index, int n, int d)
{
    /* K/MatMul.java:153-212 : literal per-element walk, any (weight_index, n) */
#pragma omp parallel for schedule(static)
    for (int i = 0; i < d; i++) {
        int64_t wpos = weight_index + (int64_t)i * n;
        int index = 0;
        float val = 0.0f;
        int64_t g0 = wpos / ORC_GROUP_SIZE;
        int64_t g1 = (wpos + n - 1) / ORC_GROUP_SIZE;
        for (int64_t g = g0; g <= g1; g++) {
            const uint8_t *base = enc + g * ORC_GROUP_BYTES;
            float mn = be_float(base);
            float mx = be_float(base + 4);
            float rm = (mx - mn) / 255.0f;
            int64_t start = g * ORC_GROUP_SIZE;
            for (int j = 0; j < ORC_GROUP_SIZE; j++) {
                int64_t jj = start + j;
                if (jj >= wpos && jj < wpos + n) {
                    float w = (float)base[8 + j] * rm + mn;
                    val += w * x[index++];
                }
            }
        }
        xout[i] = val;
    }
}

/* One row of K/MatMul.java:124-149. */
static inline float row_aligned(const float *x, const uint8_t *enc, int64_t wpos, int n)
{
    float val = 0.0f;
    int index = 0;
    int64_t g0 = wpos / ORC_GROUP_SIZE;
    int64_t g1 = (wpos + n - 1) / ORC_GROUP_SIZE;
    for (int64_t g = g0; g <= g1; g++) {
        const uint8_t *base = enc + g * ORC_GROUP_BYTES;
        float mn = be_float(base);
        float mx = be_float(base + 4);
        float rm = (mx - mn) / 255.0f;
        int64_t lim64 = wpos + n - g * ORC_GROUP_SIZE;
        int limit = lim64 < ORC_GROUP_SIZE ? (int)lim64 : ORC_GROUP_SIZE;
        for (int j = 0; j < limit; j++) {
            float w = (float)base[8 + j] * rm + mn;
            val += w * x[index++];
        }
    }
    return val;
}

void orc_matmul_i8_aligned(float *xout, const float *x, const uint8_t *enc,
                           int64_t weight_index, int n, int d)
{
    /* K/MatMul.java:97-151.  Rows are independent, so four of them are walked side by
     * side to hide the latency of the sequential adds; each row still sees exactly the
     * reference's operation order (tests check bit-equality with the literal walk). */
    int ngroups = n / ORC_GROUP_SIZE;
    int d4 = (n % ORC_GROUP_SIZE == 0 && weight_index % ORC_GROUP_SIZE == 0) ? (d / 4) * 4 : 0;
#pragma omp parallel for schedule(static)
    for (int i0 = 0; i0 < d4; i0 += 4) {
        const uint8_t *b0 = enc + ((weight_index + (int64_t)(i0 + 0) * n) / ORC_GROUP_SIZE) * ORC_GROUP_BYTES;
        const uint8_t *b1 = enc + ((weight_index + (int64_t)(i0 + 1) * n) / ORC_GROUP_SIZE) * ORC_GROUP_BYTES;
        const uint8_t *b2 = enc + ((weight_index + (int64_t)(i0 + 2) * n) / ORC_GROUP_SIZE) * ORC_GROUP_BYTES;
        const uint8_t *b3 = enc + ((weight_index + (int64_t)(i0 + 3) * n) / ORC_GROUP_SIZE) * ORC_GROUP_BYTES;
        float v0 = 0.0f, v1 = 0.0f, v2 = 0.0f, v3 = 0.0f;
        const float *xp = x;
        for (int g = 0; g < ngroups; g++) {
            float m0 = be_float(b0), r0 = (be_float(b0 + 4) - m0) / 255.0f;
            float m1 = be_float(b1), r1 = (be_float(b1 + 4) - m1) / 255.0f;
            float m2 = be_float(b2), r2 = (be_float(b2 + 4) - m2) / 255.0f;
            float m3 = be_float(b3), r3 = (be_float(b3 + 4) - m3) / 255.0f;
            for (int j = 0; j < ORC_GROUP_SIZE; j++) {
                float xv = xp[j];
                float w0 = (float)b0[8 + j] * r0 + m0;
                float w1 = (float)b1[8 + j] * r1 + m1;
                float w2 = (float)b2[8 + j] * r2 + m2;
                float w3 = (float)b3[8 + j] * r3 + m3;
                v0 += w0 * xv;
                v1 += w1 * xv;
                v2 += w2 * xv;
                v3 += w3 * xv;
            }
            xp += ORC_GROUP_SIZE;
            b0 += ORC_GROUP_BYTES; b1 += ORC_GROUP_BYTES; b2 += ORC_GROUP_BYTES; b3 += ORC_GROUP_BYTES;
        }
        xout[i0] = v0; xout[i0 + 1] = v1; xout[i0 + 2] = v2; xout[i0 + 3] = v3;
    }
    for (int i = d4; i < d; i++)
        xout[i] = row_aligned(x, enc, weight_index + (int64_t)i * n, n);
}

void orc_matmul_i8(float *xout, const float *x, const uint8_t *enc, int64_t weight_index,
                   int n, int d)
{
    /* K/MatMul.java:77-85 */
    if (weight_index % ORC_GROUP_SIZE == 0 && n % ORC_GROUP_SIZE == 0)
        orc_matmul_i8_aligned(xout, x, enc, weight_index, n, d);
    else
        orc_matmul_i8_unaligned(xout, x, enc, weight_index, n, d);
}

void orc_matmul_f32(float *xout, const float *x, const float *w, int64_t weight_index, int n, int d)
{
    /* K/MatMul.java:29-60 : contiguous row blocks over threads; each row sequential in j.
     * Two rows side by side for latency, same per-row order. */
    int d2 = (d / 2) * 2;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < d2; i += 2) {
        const float *w0 = w + weight_index + (int64_t)i * n;
        const float *w1 = w0 + n;
        float v0 = 0.0f, v1 = 0.0f;
        for (int j = 0; j < n; j++) {
            v0 += w0[j] * x[j];
            v1 += w1[j] * x[j];
        }
        xout[i] = v0;
        xout[i + 1] = v1;
    }
    for (int i = d2; i < d; i++) {
        const float *w0 = w + weight_index + (int64_t)i * n;
        float v = 0.0f;
        for (int j = 0; j < n; j++) v += w0[j] * x[j];
        xout[i] = v;
    }
}

void orc_rope_table(float *cos_t, float *sin_t, int dim, int head_size, int seq_len)
{
    /* K/ApplyRope.java:34-59 */
    for (int i = 0; i < dim; i += 2) {
        int head_dim = i % head_size;
        float e = (float)head_dim / (float)head_size;
        float freq = (float)(1.0 / pow((double)10000.0f, (double)e)); /* 1.0f widened: double divide */
        for (int pos = 0; pos < seq_len; pos++) {
            float val = (float)pos * freq;
            int64_t index = ((int64_t)pos * dim / 2) + i / 2;
            cos_t[index] = (float)cos((double)val);
            sin_t[index] = (float)sin((double)val);
        }
    }
}

void orc_rope(float *q, float *k, const float *cos_t, const float *sin_t, int pos, int dim, int kv_dim)
{
    /* K/ApplyRope.java:61-92 */
    for (int i = 0; i < dim; i += 2) {
        int64_t index = ((int64_t)pos * dim / 2) + i / 2;
        float fcr = cos_t[index], fci = sin_t[index];
        float v0 = q[i], v1 = q[i + 1];
        q[i] = v0 * fcr - v1 * fci;
        q[i + 1] = v0 * fci + v1 * fcr;
    }
    for (int i = 0; i < kv_dim; i += 2) {
        int64_t index = ((int64_t)pos * dim / 2) + i / 2;
        float fcr = cos_t[index], fci = sin_t[index];
        float v0 = k[i], v1 = k[i + 1];
        k[i] = v0 * fcr - v1 * fci;
        k[i + 1] = v0 * fci + v1 * fcr;
    }
}

void orc_attention_loop(const float *q, const float *key_cache, float *att, float *max,
                        int max_index, int64_t att_index, int64_t keybase, int kv_dim,
                        int query_index, int pos, int head_size)
{
    /* K/AttentionLoop.java:29-54.  The "max" is over element-wise products, is folded
     * into max[max_index] without a reset, and the score is divided (not multiplied). */
    float head_max = -FLT_MAX;
    float root = (float)sqrt((double)head_size);
    for (int t = 0; t <= pos; t++) {
        int64_t key_index = keybase + (int64_t)t * kv_dim;
        float score = 0.0f;
        for (int i = 0; i < head_size; i++) {
            float value = q[query_index + i] * key_cache[key_index + i];
            score += value;
            head_max = java_maxf(head_max, value);
        }
        att[att_index + t] = score / root;
        if (max != NULL) max[max_index] = java_maxf(max[max_index], head_max);
    }
}

void orc_exp_sum_normalize(float *x, const float *max_value, int max_index, int64_t index, int size)
{
    /* K/ExpSumNormalize.java:25-38 */
    float sum = 0.0f;
    float max_val = max_value[max_index];
    for (int i = 0; i < size; i++) {
        float a = x[index + i] - max_val;
        x[index + i] = (float)exp((double)a);
        sum += x[index + i];
    }
    if (sum != 0.0f) {
        for (int i = 0; i < size; i++) x[index + i] /= sum;
    }
}

void orc_accum_weighted_value(float *xb, const float *att, const float *value_cache, int pos,
                              int xb_index, int64_t value_base, int head_size, int kv_dim,
                              int64_t att_index)
{
    /* K/AccumWeightedValue.java:31-88 : the unrolled and plain variants perform the same
     * per-element sequence (t outer, one multiply then one add). */
    int64_t v_index = value_base;
    for (int i = 0; i < head_size; i++) xb[xb_index + i] = 0.0f;
    for (int t = 0; t <= pos; t++) {
        float a = att[att_index + t];
        for (int i = 0; i < head_size; i++) xb[xb_index + i] += a * value_cache[v_index + i];
        v_index += kv_dim;
    }
}

void orc_accum(float *a, const float *b, int size)
{
    /* K/Accum.java:26-30 */
    for (int i = 0; i < size; i++) a[i] += b[i];
}

#define SILU_TABLE_SIZE 8192
#define SILU_MAX_ABS 5
#define SILU_MULT (SILU_TABLE_SIZE / (2 * SILU_MAX_ABS)) /* integer 819, K/Silu.java:43 */

void orc_silu_table(float *table)
{
    /* K/Silu.java:47-57 */
    for (int i = 0; i < SILU_TABLE_SIZE; i++) {
        double val = ((double)i / (double)SILU_TABLE_SIZE) * (2.0 * SILU_MAX_ABS) - SILU_MAX_ABS;
        table[i] = (float)(1.0 / (1.0 + exp(-val)));
    }
}

float orc_silu_lookup(const float *table, float val)
{
    /* K/Silu.java:59-70 */
    float position = (val + (float)SILU_MAX_ABS) * (float)SILU_MULT;
    if (position > 0 && position < (float)(SILU_TABLE_SIZE - 1)) {
        int index = (int)position;
        float lower = table[index];
        return lower + (position - (float)index) * (table[index + 1] - lower);
    }
    return (float)(1.0 / (1.0 + exp(-(double)val)));
}

void orc_silu(float *hb, const float *hb2, const float *table, int hidden_dim)
{
    /* K/Silu.java:72-78 : hb[i] = hb[i] * (sigma * hb2[i]) */
    for (int i = 0; i < hidden_dim; i++) {
        float s = orc_silu_lookup(table, hb[i]);
        hb[i] = hb[i] * (s * hb2[i]);
    }
}

int orc_argmax(const float *logits, int n)
{
    /* J/Sampler.java:46-57 : first index of the strict maximum */
    int max_i = 0;
    float max_p = logits[0];
    for (int i = 1; i < n; i++) {
        if (logits[i] > max_p) {
            max_i = i;
            max_p = logits[i];
        }
    }
    return max_i;
}

/* ------------------------------------------------------------------ */
/* model                                                                */
/* ------------------------------------------------------------------ */

struct orc_model {
    orc_config cfg;
    int kv_dim, kv_mul, head_size;
    uint8_t *quant[ORC_T_COUNT];
    int64_t quant_bytes[ORC_T_COUNT];
    float *emb;
    float *wcls; /* == emb when shared */
    /* J/RunState.java:20-34 */
    float *x, *xb, *xb2, *hb, *hb2, *q, *k, *v, *att, *logits, *tmp1;
    float *key_cache, *value_cache;
    int64_t tmp1_len;
    float *rope_cos, *rope_sin;
    float silu_table[SILU_TABLE_SIZE];
    float *taps[ORC_TAP_COUNT]; /* per-layer copies, NULL unless enabled */
};

static const char *const TENSOR_NAMES[ORC_T_COUNT] = {
    "l_rms_att_weight", "l_wq", "l_wk", "l_wv", "l_wo",
    "l_rms_ffn_weight", "l_w1", "l_w2", "l_w3", "rms_final_weight"};

const char *orc_tensor_name(int tensor)
{
    return (tensor >= 0 && tensor < ORC_T_COUNT) ? TENSOR_NAMES[tensor] : NULL;
}

int64_t orc_tensor_floats(const orc_config *c, int tensor)
{
    /* J/TransformerWeights.java:54-111 */
    int64_t L = c->n_layers, dim = c->dim, hid = c->hidden_dim;
    int64_t hs = c->dim / c->n_heads;
    switch (tensor) {
    case ORC_T_RMS_ATT: return L * dim;
    case ORC_T_WQ: return L * dim * (c->n_heads * hs);
    case ORC_T_WK: return L * dim * (c->n_kv_heads * hs);
    case ORC_T_WV: return L * dim * (c->n_kv_heads * hs);
    case ORC_T_WO: return L * (c->n_heads * hs) * dim;
    case ORC_T_RMS_FFN: return L * dim;
    case ORC_T_W1: return L * dim * hid;
    case ORC_T_W2: return L * hid * dim;
    case ORC_T_W3: return L * dim * hid;
    case ORC_T_RMS_FINAL: return dim;
    default: return -1;
    }
}

static float *zalloc_f(int64_t n)
{
    return (float *)calloc((size_t)(n > 0 ? n : 1), sizeof(float));
}

orc_model *orc_model_new(const orc_config *cfg)
{
    orc_model *m = (orc_model *)calloc(1, sizeof(orc_model));
    if (!m) return NULL;
    m->cfg = *cfg;
    m->head_size = cfg->dim / cfg->n_heads;
    m->kv_dim = (cfg->dim * cfg->n_kv_heads) / cfg->n_heads;
    m->kv_mul = cfg->n_heads / cfg->n_kv_heads;
    for (int t = 0; t < ORC_T_COUNT; t++) {
        m->quant_bytes[t] = orc_quant_nbytes(orc_tensor_floats(cfg, t));
        m->quant[t] = (uint8_t *)malloc((size_t)m->quant_bytes[t]);
        if (!m->quant[t]) { orc_model_free(m); return NULL; }
    }
    int64_t vd = (int64_t)cfg->vocab_size * cfg->dim;
    m->emb = (float *)malloc((size_t)vd * sizeof(float));
    m->wcls = cfg->shared_weights ? m->emb : (float *)malloc((size_t)vd * sizeof(float));
    /* J/RunState.java:77-102 */
    m->tmp1_len = (int64_t)(cfg->dim > cfg->vocab_size ? cfg->dim : cfg->vocab_size) * 4;
    m->tmp1 = zalloc_f(m->tmp1_len);
    m->x = zalloc_f(cfg->dim);
    m->xb = zalloc_f(cfg->dim);
    m->xb2 = zalloc_f(cfg->dim);
    m->hb = zalloc_f(cfg->hidden_dim);
    m->hb2 = zalloc_f(cfg->hidden_dim);
    m->q = zalloc_f(cfg->dim);
    m->k = zalloc_f(m->kv_dim);
    m->v = zalloc_f(m->kv_dim);
    m->att = zalloc_f((int64_t)cfg->n_heads * cfg->seq_len);
    m->logits = zalloc_f(cfg->vocab_size);
    int64_t kvn = (int64_t)cfg->n_layers * cfg->seq_len * m->kv_dim;
    m->key_cache = zalloc_f(kvn);
    m->value_cache = zalloc_f(kvn);
    int64_t rn = (int64_t)(cfg->dim / 2) * cfg->seq_len;
    m->rope_cos = zalloc_f(rn);
    m->rope_sin = zalloc_f(rn);
    if (!m->emb || !m->wcls || !m->tmp1 || !m->x || !m->xb || !m->xb2 || !m->hb || !m->hb2 || !m->q ||
        !m->k || !m->v || !m->att || !m->logits || !m->key_cache || !m->value_cache || !m->rope_cos ||
        !m->rope_sin) {
        orc_model_free(m);
        return NULL;
    }
    orc_rope_table(m->rope_cos, m->rope_sin, cfg->dim, m->head_size, cfg->seq_len);
    orc_silu_table(m->silu_table);
    return m;
}

void orc_model_free(orc_model *m)
{
    if (!m) return;
    for (int t = 0; t < ORC_TAP_COUNT; t++) free(m->taps[t]);
    for (int t = 0; t < ORC_T_COUNT; t++) free(m->quant[t]);
    if (m->wcls != m->emb) free(m->wcls);
    free(m->emb);
    free(m->tmp1); free(m->x); free(m->xb); free(m->xb2); free(m->hb); free(m->hb2);
    free(m->q); free(m->k); free(m->v); free(m->att); free(m->logits);
    free(m->key_cache); free(m->value_cache); free(m->rope_cos); free(m->rope_sin);
    free(m);
}

int orc_model_set_quant(orc_model *m, int tensor, const uint8_t *bytes, int64_t nbytes)
{
    if (tensor < 0 || tensor >= ORC_T_COUNT) return -1;
    if (nbytes != m->quant_bytes[tensor]) return -2; /* J/TransformerWeights.java:228-232 */
    memcpy(m->quant[tensor], bytes, (size_t)nbytes);
    return 0;
}

int orc_model_set_emb(orc_model *m, const float *emb, int64_t nfloats)
{
    if (nfloats != (int64_t)m->cfg.vocab_size * m->cfg.dim) return -2;
    memcpy(m->emb, emb, (size_t)nfloats * sizeof(float));
    return 0;
}

int orc_model_set_wcls(orc_model *m, const float *wcls, int64_t nfloats)
{
    if (nfloats != (int64_t)m->cfg.vocab_size * m->cfg.dim) return -2;
    if (m->wcls == m->emb) return 0;
    memcpy(m->wcls, wcls, (size_t)nfloats * sizeof(float));
    return 0;
}

uint8_t *orc_model_quant_ptr(orc_model *m, int tensor)
{
    return (tensor >= 0 && tensor < ORC_T_COUNT) ? m->quant[tensor] : NULL;
}
float *orc_model_emb_ptr(orc_model *m) { return m->emb; }
float *orc_model_wcls_ptr(orc_model *m) { return m->wcls; }

float *orc_model_buffer(orc_model *m, int which)
{
    switch (which) {
    case ORC_B_X: return m->x;
    case ORC_B_XB: return m->xb;
    case ORC_B_XB2: return m->xb2;
    case ORC_B_HB: return m->hb;
    case ORC_B_HB2: return m->hb2;
    case ORC_B_Q: return m->q;
    case ORC_B_K: return m->k;
    case ORC_B_V: return m->v;
    case ORC_B_ATT: return m->att;
    case ORC_B_LOGITS: return m->logits;
    case ORC_B_KCACHE: return m->key_cache;
    case ORC_B_VCACHE: return m->value_cache;
    case ORC_B_TMP1: return m->tmp1;
    default: return NULL;
    }
}

void orc_model_reset(orc_model *m)
{
    int64_t kvn = (int64_t)m->cfg.n_layers * m->cfg.seq_len * m->kv_dim;
    memset(m->key_cache, 0, (size_t)kvn * sizeof(float));
    memset(m->value_cache, 0, (size_t)kvn * sizeof(float));
    memset(m->tmp1, 0, (size_t)m->tmp1_len * sizeof(float));
    memset(m->att, 0, (size_t)m->cfg.n_heads * m->cfg.seq_len * sizeof(float));
}

static int64_t tap_len(const orc_model *m, int which)
{
    switch (which) {
    case ORC_TAP_HB: return m->cfg.hidden_dim;
    case ORC_TAP_K: case ORC_TAP_V: return m->kv_dim;
    default: return m->cfg.dim;
    }
}

int orc_model_enable_taps(orc_model *m)
{
    for (int t = 0; t < ORC_TAP_COUNT; t++) {
        if (m->taps[t]) continue;
        m->taps[t] = zalloc_f((int64_t)m->cfg.n_layers * tap_len(m, t));
        if (!m->taps[t]) return -1;
    }
    return 0;
}

float *orc_model_tap(orc_model *m, int which, int layer)
{
    if (which < 0 || which >= ORC_TAP_COUNT || !m->taps[which]) return NULL;
    return m->taps[which] + (int64_t)layer * tap_len(m, which);
}

static void tap(orc_model *m, int which, int layer, const float *src)
{
    if (m->taps[which]) memcpy(orc_model_tap(m, which, layer), src, (size_t)tap_len(m, which) * sizeof(float));
}

static void forward_impl(orc_model *m, int token, int pos, int n_layers_run, int run_head)
{
    /* J/Run.java:62-169 */
    const orc_config *p = &m->cfg;
    const int dim = p->dim;
    const int kv_dim = m->kv_dim;
    const int kv_mul = m->kv_mul;
    const int hidden_dim = p->hidden_dim;
    const int head_size = m->head_size;

    memcpy(m->x, m->emb + (int64_t)token * dim, (size_t)dim * sizeof(float)); /* :72 */

    for (int l = 0; l < n_layers_run; l++) {
        orc_rms(m->tmp1, m->x, dim);                                                          /* :78 */
        orc_wns_i8(m->xb, m->x, m->quant[ORC_T_RMS_ATT], (int64_t)l * dim, m->tmp1, dim);     /* :80 */

        orc_matmul_i8(m->q, m->xb, m->quant[ORC_T_WQ], (int64_t)l * dim * dim, dim, dim);       /* :83 */
        orc_matmul_i8(m->k, m->xb, m->quant[ORC_T_WK], (int64_t)l * dim * kv_dim, dim, kv_dim); /* :84 */
        orc_matmul_i8(m->v, m->xb, m->quant[ORC_T_WV], (int64_t)l * dim * kv_dim, dim, kv_dim); /* :85 */

        orc_rope(m->q, m->k, m->rope_cos, m->rope_sin, pos, dim, kv_dim);                     /* :88 */

        int64_t loff = (int64_t)l * p->seq_len * kv_dim;                                      /* :91 */
        memcpy(m->key_cache + loff + (int64_t)pos * kv_dim, m->k, (size_t)kv_dim * sizeof(float));   /* :95 */
        memcpy(m->value_cache + loff + (int64_t)pos * kv_dim, m->v, (size_t)kv_dim * sizeof(float)); /* :99 */
        tap(m, ORC_TAP_Q, l, m->q);
        tap(m, ORC_TAP_K, l, m->k);
        tap(m, ORC_TAP_V, l, m->v);

#pragma omp parallel for schedule(static)
        for (int h = 0; h < p->n_heads; h++) {                                                /* :102-131 */
            int query_index = h * head_size;
            int64_t att_index = (int64_t)h * p->seq_len;
            int64_t key_base = loff + (int64_t)(h / kv_mul) * head_size;
            int max_index = h;
            orc_attention_loop(m->q, m->key_cache, m->att, m->tmp1, max_index, att_index, key_base,
                               kv_dim, query_index, pos, head_size);
            orc_exp_sum_normalize(m->att, m->tmp1, max_index, att_index, pos + 1);
            int xb_index = h * head_size;
            int64_t value_base = loff + (int64_t)(h / kv_mul) * head_size;
            orc_accum_weighted_value(m->xb, m->att, m->value_cache, pos, xb_index, value_base,
                                     head_size, kv_dim, att_index);
        }

        tap(m, ORC_TAP_ATT_OUT, l, m->xb);
        orc_matmul_i8(m->xb2, m->xb, m->quant[ORC_T_WO], (int64_t)l * dim * dim, dim, dim);    /* :134 */
        orc_accum(m->x, m->xb2, dim);                                                         /* :136 */
        tap(m, ORC_TAP_X_ATT, l, m->x);

        orc_rms(m->tmp1, m->x, dim);                                                          /* :142 */
        orc_wns_i8(m->xb, m->x, m->quant[ORC_T_RMS_FFN], (int64_t)l * dim, m->tmp1, dim);     /* :143 */

        orc_matmul_i8(m->hb, m->xb, m->quant[ORC_T_W1], (int64_t)l * dim * hidden_dim, dim, hidden_dim);  /* :147 */
        orc_matmul_i8(m->hb2, m->xb, m->quant[ORC_T_W3], (int64_t)l * dim * hidden_dim, dim, hidden_dim); /* :148 */

        orc_silu(m->hb, m->hb2, m->silu_table, hidden_dim);                                   /* :152 */
        tap(m, ORC_TAP_HB, l, m->hb);

        orc_matmul_i8(m->xb, m->hb, m->quant[ORC_T_W2], (int64_t)l * dim * hidden_dim, hidden_dim, dim); /* :155 */
        orc_accum(m->x, m->xb, dim);                                                          /* :158 */
        tap(m, ORC_TAP_X_FFN, l, m->x);
    }
    if (!run_head) return;

    orc_rms(m->tmp1, m->x, dim);                                                              /* :164 */
    orc_wns_i8(m->x, m->x, m->quant[ORC_T_RMS_FINAL], 0, m->tmp1, dim);                       /* :165 in place */
    orc_matmul_f32(m->logits, m->x, m->wcls, 0, dim, p->vocab_size);                          /* :168 */
}

void orc_forward(orc_model *m, int token, int pos)
{
    forward_impl(m, token, pos, m->cfg.n_layers, 1);
}

void orc_forward_layers(orc_model *m, int token, int pos, int n_layers_run)
{
    forward_impl(m, token, pos, n_layers_run, 0);
}

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

int orc_generate_greedy(orc_model *m, const int32_t *prompt, int n_prompt, int steps,
                        int32_t *out_tokens, float *logits_out, double *seconds)
{
    /* J/Run.java:599-603, 611-685 (temperature 0) */
    if (steps <= 0 || steps > m->cfg.seq_len) steps = m->cfg.seq_len;
    double start = 0.0;
    int started = 0;
    int token = 1;
    int pos = 0;
    while (pos < steps) {
        orc_forward(m, token, pos);
        if (logits_out)
            memcpy(logits_out + (int64_t)pos * m->cfg.vocab_size, m->logits,
                   (size_t)m->cfg.vocab_size * sizeof(float));
        int next;
        if (pos < n_prompt) next = prompt[pos];
        else next = orc_argmax(m->logits, m->cfg.vocab_size);
        out_tokens[pos] = next;
        pos++;
        if (next == 1) break;
        token = next;
        if (!started) { start = now_s(); started = 1; }
    }
    if (seconds) *seconds = started ? now_s() - start : 0.0;
    return pos;
}

/* ------------------------------------------------------------------ */
/* sampling                                                             */
/* ------------------------------------------------------------------ */

void orc_find_max(float *max, int max_index, const float *x, int64_t index, int size)
{
    /* K/FindMax.java:40-48 */
    float max_val = x[index];
    for (int i = 1; i < size; i++) {
        if (x[index + i] > max_val) max_val = x[index + i];
    }
    max[max_index] = max_val;
}

struct orc_sampler {
    uint64_t rng;     /* java.util.Random's 48-bit state */
    int n;
    float *prob;      /* J/Sampler.java:18,60-62 : the ProbIndex array, kept between calls */
    int32_t *index;
    float *tprob;     /* merge buffers */
    int32_t *tindex;
};

#define JRAND_MULT 0x5DEECE66DULL
#define JRAND_MASK ((1ULL << 48) - 1)

orc_sampler *orc_sampler_new(int64_t rng_seed, int vocab_size)
{
    /* J/Sampler.java:24-31; new Random(seed): state = (seed ^ 0x5DEECE66D) mod 2^48 */
    orc_sampler *s = (orc_sampler *)calloc(1, sizeof(*s));
    if (!s) return NULL;
    s->rng = ((uint64_t)rng_seed ^ JRAND_MULT) & JRAND_MASK;
    s->n = vocab_size;
    s->prob = (float *)calloc((size_t)vocab_size, sizeof(float));      /* new ProbIndex(): prob 0, index 0 */
    s->index = (int32_t *)calloc((size_t)vocab_size, sizeof(int32_t));
    s->tprob = (float *)calloc((size_t)vocab_size, sizeof(float));
    s->tindex = (int32_t *)calloc((size_t)vocab_size, sizeof(int32_t));
    if (!s->prob || !s->index || !s->tprob || !s->tindex) { orc_sampler_free(s); return NULL; }
    return s;
}

void orc_sampler_free(orc_sampler *s)
{
    if (!s) return;
    free(s->prob); free(s->index); free(s->tprob); free(s->tindex);
    free(s);
}

int32_t orc_sampler_next_bits(orc_sampler *s, int bits)
{
    /* java.util.Random.next(bits) */
    s->rng = (s->rng * JRAND_MULT + 0xBULL) & JRAND_MASK;
    return (int32_t)(uint32_t)(s->rng >> (48 - bits));
}

float orc_sampler_next_float(orc_sampler *s)
{
    /* J/Sampler.java:20-22 -> java.util.Random.nextFloat() = next(24) / (float)(1 << 24) */
    return (float)orc_sampler_next_bits(s, 24) / (float)(1 << 24);
}

int orc_sample_coin(const float *probs, int n, float r)
{
    /* J/Sampler.java:33-44 */
    float cdf = 0.0f;
    for (int i = 0; i < n; i++) {
        cdf += probs[i];
        if (r < cdf) return i;
    }
    return n - 1;
}

int orc_sample(orc_sampler *s, const float *probs, int n)
{
    return orc_sample_coin(probs, n, orc_sampler_next_float(s));
}

/* Stable descending merge sort of the whole ProbIndex array: Arrays.sort(Object[]) is a stable
 * merge sort and ProbIndex.compareTo (J/Sampler.java:64-73) orders by prob, larger first. */
static void sort_prob_index(orc_sampler *s)
{
    float *a = s->prob, *b = s->tprob;
    int32_t *ai = s->index, *bi = s->tindex;
    const int n = s->n;
    for (int width = 1; width < n; width *= 2) {
        for (int lo = 0; lo < n; lo += 2 * width) {
            int mid = lo + width < n ? lo + width : n;
            int hi = lo + 2 * width < n ? lo + 2 * width : n;
            int i = lo, j = mid, k = lo;
            while (i < mid && j < hi) {
                if (a[j] > a[i]) { b[k] = a[j]; bi[k] = ai[j]; j++; }   /* strictly larger moves ahead */
                else { b[k] = a[i]; bi[k] = ai[i]; i++; }
                k++;
            }
            while (i < mid) { b[k] = a[i]; bi[k] = ai[i]; i++; k++; }
            while (j < hi) { b[k] = a[j]; bi[k] = ai[j]; j++; k++; }
        }
        float *t = a; a = b; b = t;
        int32_t *ti = ai; ai = bi; bi = ti;
    }
    if (a != s->prob) {
        memcpy(s->prob, a, (size_t)n * sizeof(float));
        memcpy(s->index, ai, (size_t)n * sizeof(int32_t));
    }
}

static int topp_pick(orc_sampler *s, const float *probs, int n, float topp, int draw, float coin)
{
    /* J/Sampler.java:76-120 */
    int n0 = 0;
    float cutoff = (1.0f - topp) / (float)(n - 1);
    for (int i = 0; i < n; i++) {
        if (probs[i] != probs[i]) return -1;        /* :88-90 */
        if (probs[i] >= cutoff) {
            s->index[n0] = i;
            s->prob[n0] = probs[i];
            n0++;
        }
    }
    sort_prob_index(s);                             /* :97 : the whole array */
    if (n0 == 0) return -2;                         /* :101,119 : probIndex[-1], ArrayIndexOutOfBoundsException */
    float cumulative_prob = 0.0f;
    int last_idx = n0 - 1;
    for (int i = 0; i < n0; i++) {
        cumulative_prob += s->prob[i];
        if (cumulative_prob > topp) { last_idx = i; break; }
    }
    if (draw) coin = orc_sampler_next_float(s);
    float r = coin * cumulative_prob;
    float cdf = 0.0f;
    for (int i = 0; i <= last_idx; i++) {
        cdf += s->prob[i];
        if (r < cdf) return s->index[i];
    }
    return s->index[last_idx];
}

int orc_sample_topp(orc_sampler *s, const float *probs, int n, float topp)
{
    return topp_pick(s, probs, n, topp, 1, 0.0f);
}

int orc_sample_topp_coin(orc_sampler *s, const float *probs, int n, float topp, float coin)
{
    return topp_pick(s, probs, n, topp, 0, coin);
}

int orc_sample_step(orc_sampler *s, float *logits, int n, float temperature, float topp)
{
    /* J/Run.java:643-665 */
    if (temperature == 0.0f) return orc_argmax(logits, n);
    for (int q = 0; q < n; q++) logits[q] /= temperature;
    float max[1] = {0.0f};
    orc_find_max(max, 0, logits, 0, n);
    orc_exp_sum_normalize(logits, max, 0, 0, n);
    if ((double)topp > 0.999) return orc_sample(s, logits, n);
    return orc_sample_topp(s, logits, n, topp);
}

int orc_generate(orc_model *m, const int32_t *prompt, int n_prompt, int steps, float temperature,
                 float topp, int64_t rng_seed, int32_t *out_tokens, double *seconds)
{
    /* J/Run.java:599-603, 611-685 */
    if (steps <= 0 || steps > m->cfg.seq_len) steps = m->cfg.seq_len;
    orc_sampler *s = orc_sampler_new(rng_seed, m->cfg.vocab_size);
    if (!s) return -1;
    double start = 0.0;
    int started = 0;
    int token = 1;
    int pos = 0;
    while (pos < steps) {
        orc_forward(m, token, pos);
        int next;
        if (pos < n_prompt) next = prompt[pos];
        else next = orc_sample_step(s, m->logits, m->cfg.vocab_size, temperature, topp);
        out_tokens[pos] = next;
        pos++;
        if (next == 1) break;
        token = next;
        if (!started) { start = now_s(); started = 1; }
    }
    if (seconds) *seconds = started ? now_s() - start : 0.0;
    orc_sampler_free(s);
    return pos;
}

/* ------------------------------------------------------------------ */
/* files                                                                */
/* ------------------------------------------------------------------ */

int orc_write_quant_file(const char *path, const uint8_t *bytes, int64_t nbytes)
{
    /* J/BinFileWriter.java:20-34 : little-endian int32 length, then the bytes */
    FILE *f = fopen(path, "wb");
    if (!f) return -1;
    uint32_t n = (uint32_t)nbytes;
    uint8_t hdr[4] = {(uint8_t)n, (uint8_t)(n >> 8), (uint8_t)(n >> 16), (uint8_t)(n >> 24)};
    int ok = fwrite(hdr, 1, 4, f) == 4 && fwrite(bytes, 1, (size_t)nbytes, f) == (size_t)nbytes;
    fclose(f);
    return ok ? 0 : -1;
}

int64_t orc_read_quant_file(const char *path, uint8_t *dst, int64_t cap)
{
    /* J/TransformerWeights.java:219-221 */
    FILE *f = fopen(path, "rb");
    if (!f) return -1;
    uint8_t hdr[4];
    if (fread(hdr, 1, 4, f) != 4) { fclose(f); return -1; }
    int64_t n = (int64_t)((uint32_t)hdr[0] | ((uint32_t)hdr[1] << 8) | ((uint32_t)hdr[2] << 16) | ((uint32_t)hdr[3] << 24));
    if (n > cap) { fclose(f); return -2; }
    int64_t got = (int64_t)fread(dst, 1, (size_t)n, f);
    fclose(f);
    return got == n ? n : -1;
}

static int file_exists(const char *p)
{
    struct stat st;
    return stat(p, &st) == 0;
}

orc_model *orc_load_checkpoint(const char *bin_path, int write_caches, char *err, int errlen)
{
    /* J/Run.java:561-573, J/TransformerWeights.java:43-122,191-232 */
#define FAIL(...)                                          \
    do {                                                   \
        if (err) snprintf(err, (size_t)errlen, __VA_ARGS__); \
        if (f) fclose(f);                                  \
        if (m) orc_model_free(m);                          \
        free(tmp);                                         \
        return NULL;                                       \
    } while (0)
    orc_model *m = NULL;
    float *tmp = NULL;
    FILE *f = fopen(bin_path, "rb");
    if (!f) FAIL("cannot open %s", bin_path);
    int32_t h[7];
    if (fread(h, 4, 7, f) != 7) FAIL("short header");
    orc_config c;
    c.dim = h[0]; c.hidden_dim = h[1]; c.n_layers = h[2]; c.n_heads = h[3]; c.n_kv_heads = h[4];
    c.shared_weights = h[5] > 0;
    c.vocab_size = h[5] < 0 ? -h[5] : h[5];
    c.seq_len = h[6];
    m = orc_model_new(&c);
    if (!m) FAIL("out of memory");
    int64_t vd = (int64_t)c.vocab_size * c.dim;
    if ((int64_t)fread(m->emb, 4, (size_t)vd, f) != vd) FAIL("short embedding");

    /* directory and base name: J/BinFileReader.java:35-49 */
    char dir[1024], base[512];
    const char *slash = strrchr(bin_path, '/');
    if (slash) { snprintf(dir, sizeof dir, "%.*s", (int)(slash - bin_path), bin_path); snprintf(base, sizeof base, "%s", slash + 1); }
    else { snprintf(dir, sizeof dir, "."); snprintf(base, sizeof base, "%s", bin_path); }
    char *dot = strrchr(base, '.');
    if (dot && dot != base) *dot = 0;

    for (int t = 0; t < ORC_T_COUNT; t++) {
        int64_t nf = orc_tensor_floats(&c, t);
        char qpath[2048];
        snprintf(qpath, sizeof qpath, "%s/%s_%s_%d_%d.quant", dir, base, TENSOR_NAMES[t], ORC_GROUP_SIZE, 8);
        if (file_exists(qpath)) {
            if (fseek(f, (long)(nf * 4), SEEK_CUR) != 0) FAIL("seek");
            int64_t got = orc_read_quant_file(qpath, m->quant[t], m->quant_bytes[t]);
            if (got != m->quant_bytes[t]) FAIL("totalByteSize != quant.numberOfBytesByFloatSize(floatSize): %s", qpath);
        } else {
            tmp = (float *)malloc((size_t)nf * 4);
            if (!tmp) FAIL("out of memory");
            if ((int64_t)fread(tmp, 4, (size_t)nf, f) != nf) FAIL("short tensor %s", TENSOR_NAMES[t]);
            orc_quant_encode(tmp, nf, m->quant[t]);
            free(tmp);
            tmp = NULL;
            if (write_caches && orc_write_quant_file(qpath, m->quant[t], m->quant_bytes[t]) != 0)
                FAIL("cannot write %s", qpath);
        }
    }
    int64_t skip = 2 * ((int64_t)c.seq_len * (c.dim / c.n_heads) / 2); /* :119-120 */
    if (fseek(f, (long)(skip * 4), SEEK_CUR) != 0) FAIL("seek");
    if (!c.shared_weights) {
        if ((int64_t)fread(m->wcls, 4, (size_t)vd, f) != vd) FAIL("short classifier");
    }
    fclose(f);
    return m;
#undef FAIL
}

/* ------------------------------------------------------------------ */
/* seeded synthetic tensors                                             */
/* ------------------------------------------------------------------ */

static inline uint64_t splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

static inline float synth_value(uint64_t base, int64_t i, float scale)
{
    uint64_t r = splitmix64(base + (uint64_t)i);
    int32_t s = (int32_t)(r & 0xFFFF) + (int32_t)((r >> 16) & 0xFFFF) + (int32_t)((r >> 32) & 0xFFFF) +
                (int32_t)(r >> 48) - 131070;
    return (float)s * scale;
}

static inline uint64_t synth_base(uint64_t seed, uint32_t stream)
{
    return seed * 0x9E3779B97F4A7C15ULL + (uint64_t)stream * 0xD1B54A32D192ED03ULL;
}

void orc_synth_fill(uint64_t seed, uint32_t stream, int64_t first, int64_t n, float sigma, float *out)
{
    float scale = sigma / 37837.2265625f;
    uint64_t base = synth_base(seed, stream);
#pragma omp parallel for schedule(static) if (n > 65536)
    for (int64_t i = 0; i < n; i++) out[i] = synth_value(base, first + i, scale);
}

void orc_model_fill_synth(orc_model *m, uint64_t seed, float sigma)
{
    int64_t vd = (int64_t)m->cfg.vocab_size * m->cfg.dim;
    orc_synth_fill(seed, 0, 0, vd, sigma, m->emb);
    if (m->wcls != m->emb) orc_synth_fill(seed, 11, 0, vd, sigma, m->wcls);
    float scale = sigma / 37837.2265625f;
    for (int t = 0; t < ORC_T_COUNT; t++) {
        int64_t nf = orc_tensor_floats(&m->cfg, t);
        int64_t groups = (nf + ORC_GROUP_SIZE - 1) / ORC_GROUP_SIZE;
        uint64_t base = synth_base(seed, (uint32_t)(t + 1));
        uint8_t *dst = m->quant[t];
#pragma omp parallel for schedule(static)
        for (int64_t g = 0; g < groups; g++) {
            float buf[ORC_GROUP_SIZE];
            int64_t i0 = g * ORC_GROUP_SIZE;
            int64_t cnt = nf - i0 < ORC_GROUP_SIZE ? nf - i0 : ORC_GROUP_SIZE;
            for (int64_t j = 0; j < cnt; j++) buf[j] = synth_value(base, i0 + j, scale);
            orc_quant_encode(buf, cnt, dst + g * ORC_GROUP_BYTES);
        }
    }
}

void orc_synth_prompt(uint64_t seed, int n, int vocab, int32_t *out)
{
    uint64_t base = synth_base(seed, 0xFFFFu);
    for (int i = 0; i < n; i++) {
        uint64_t r = splitmix64(base + (uint64_t)i);
        out[i] = 3 + (int32_t)((r >> 33) % (uint64_t)(vocab - 3));
    }
}

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
