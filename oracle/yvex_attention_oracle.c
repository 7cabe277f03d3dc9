/*
 * CPU restatement of the YVEX attention hot path.  TEST INFRASTRUCTURE ONLY:
 * see yvex_attention_oracle.h for the pin status of every function and for who
 * may call this library (tests, the smoke check, the benchmark's CPU leg).
 *
 * Plain C11 + OpenMP.  Arithmetic follows the reference CPU operator exactly:
 * double dot products, the score stored as float and re-read, the reference's
 * own 18-term exp, probabilities rounded to float twice, double PV accumulate.
 */
#include "yvex_attention_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int yvo_hardware_threads(void)
{
#ifdef _OPENMP
    return omp_get_num_procs();
#else
    return 1;
#endif
}

static int clamp_threads(int threads)
{
    int limit = yvo_hardware_threads();
    if (threads < 1) return 1;
    return threads > limit ? limit : threads;
}

/* ------------------------------------------------------------------ exp ---- */

/* src/backend/cpu.c:217-255: clamp to [-60, 60] (below -60 is exactly 0), peel
 * multiples of ln2 until |x| <= 0.5, 18-term Taylor series, rescale by 2^n with
 * repeated doubling/halving. */
double yvo_exp(double x)
{
    static const double LN2 = 0.69314718055994530942;
    double term = 1.0, sum = 1.0;
    int n = 0;
    unsigned i;
    if (x < -60.0) return 0.0;
    if (x > 60.0) x = 60.0;
    for (; x > 0.5; ++n) x -= LN2;
    for (; x < -0.5; --n) x += LN2;
    for (i = 1u; i <= 18u; ++i) {
        term *= x / (double)i;
        sum += term;
    }
    for (; n > 0; --n) sum *= 2.0;
    for (; n < 0; ++n) sum *= 0.5;
    return sum;
}

/* ------------------------------------------------------- scalar codecs ---- */

static uint32_t f32_bits(float v)
{
    uint32_t b;
    memcpy(&b, &v, sizeof b);
    return b;
}

static float bits_f32(uint32_t b)
{
    float v;
    memcpy(&v, &b, sizeof v);
    return v;
}

/* src/gguf/quant_scalar.c:125-143: widen by shifting; RNE narrowing; a NaN keeps
 * its upper half with the quiet bit forced. */
float yvo_bf16_decode(uint16_t bits) { return bits_f32((uint32_t)bits << 16); }

uint16_t yvo_bf16_encode(float value)
{
    uint32_t b = f32_bits(value);
    uint32_t hi = b >> 16, lo = b & 0xffffu;
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(hi | 0x40u);
    if (lo > 0x8000u || (lo == 0x8000u && (hi & 1u))) ++hi;
    return (uint16_t)hi;
}

void yvo_bf16_decode_n(const uint16_t *src, float *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; ++i) dst[i] = yvo_bf16_decode(src[i]);
}

void yvo_bf16_encode_n(const float *src, uint16_t *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; ++i) dst[i] = yvo_bf16_encode(src[i]);
}

/* src/gguf/quant_scalar.c:40-67: subnormals are renormalised, inf/NaN keep their
 * payload with the quiet bit set for NaN. */
float yvo_f16_decode(uint16_t bits)
{
    uint32_t sign = ((uint32_t)bits & 0x8000u) << 16;
    uint32_t e = ((uint32_t)bits >> 10) & 0x1fu;
    uint32_t m = (uint32_t)bits & 0x3ffu;
    if (e == 0x1fu)
        return bits_f32(sign | 0x7f800000u | (m << 13) | (m ? 0x00400000u : 0u));
    if (e != 0u) return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
    if (m == 0u) return bits_f32(sign);
    {
        uint32_t exponent = 113u;
        while (!(m & 0x400u)) {
            m <<= 1;
            --exponent;
        }
        return bits_f32(sign | (exponent << 23) | ((m & 0x3ffu) << 13));
    }
}

/* src/gguf/quant_scalar.c:74-123: RNE; overflow to inf; values below half the
 * smallest subnormal flush to signed zero; NaN -> quiet NaN keeping 9 payload bits. */
uint16_t yvo_f16_encode(float value)
{
    uint32_t b = f32_bits(value);
    uint32_t sign = (b >> 16) & 0x8000u;
    uint32_t e = (b >> 23) & 0xffu;
    uint32_t m = b & 0x7fffffu;
    uint32_t q, rem, half;
    if (e == 0xffu)
        return (uint16_t)(m ? (sign | 0x7e00u | ((m >> 13) & 0x1ffu)) : (sign | 0x7c00u));
    if (e > 142u) return (uint16_t)(sign | 0x7c00u);
    if (e >= 113u) {
        q = ((e - 112u) << 10) | (m >> 13);
        rem = m & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;
        if ((q & 0x7c00u) == 0x7c00u) q &= 0x7c00u;
        return (uint16_t)(sign | q);
    }
    if (e < 102u) return (uint16_t)sign;
    {
        uint32_t shift = 126u - e;
        uint32_t sig = m | 0x800000u;
        q = sig >> shift;
        rem = sig & ((1u << shift) - 1u);
        half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
}

/* ----------------------------------------------------------------- Q8_0 ---- */

/* src/gguf/quant_block.c:160-186: scale = f16(absmax/127) re-decoded; inverse of
 * the decoded scale; roundf (half away from zero); clamp to [-127,127]; layout
 * [f16 little endian][32 x int8]. */
int yvo_q8_0_encode_block(const float *source, unsigned char *encoded)
{
    float amax = 0.0f, scale, inv;
    uint16_t hbits;
    int i;
    for (i = 0; i < YVO_Q8_0_ELEMENTS; ++i) {
        float a = fabsf(source[i]);
        if (a > amax) amax = a;
    }
    hbits = yvo_f16_encode(amax / 127.0f);
    encoded[0] = (unsigned char)(hbits & 0xffu);
    encoded[1] = (unsigned char)(hbits >> 8);
    scale = yvo_f16_decode(hbits);
    if (!isfinite(scale) || scale < 0.0f || (amax > 0.0f && scale == 0.0f)) return 0;
    inv = scale != 0.0f ? 1.0f / scale : 0.0f;
    for (i = 0; i < YVO_Q8_0_ELEMENTS; ++i) {
        int code = (int)roundf(source[i] * inv);
        if (code < -127) code = -127;
        if (code > 127) code = 127;
        encoded[2 + i] = (unsigned char)(code & 0xff);
    }
    return 1;
}

/* src/gguf/quant_block.c:819-833: refuse a negative or non-finite scale; x = scale * (float)q. */
int yvo_q8_0_decode_block(const unsigned char *encoded, float *out)
{
    float scale = yvo_f16_decode((uint16_t)(encoded[0] | ((uint16_t)encoded[1] << 8)));
    int i;
    if (!isfinite(scale) || scale < 0.0f) return 0;
    for (i = 0; i < YVO_Q8_0_ELEMENTS; ++i)
        out[i] = scale * (float)(int)(signed char)encoded[2 + i];
    return 1;
}

int yvo_q8_0_encode_row(const float *source, size_t n, unsigned char *encoded)
{
    size_t b;
    if (n % YVO_Q8_0_ELEMENTS) return YVO_ERR_FORMAT;
    for (b = 0; b < n / YVO_Q8_0_ELEMENTS; ++b)
        if (!yvo_q8_0_encode_block(source + b * YVO_Q8_0_ELEMENTS,
                                   encoded + b * YVO_Q8_0_BYTES))
            return YVO_ERR_BOUNDS;
    return YVO_OK;
}

int yvo_q8_0_decode_row(const unsigned char *encoded, size_t n, float *out)
{
    size_t b;
    if (n % YVO_Q8_0_ELEMENTS) return YVO_ERR_FORMAT;
    for (b = 0; b < n / YVO_Q8_0_ELEMENTS; ++b)
        if (!yvo_q8_0_decode_block(encoded + b * YVO_Q8_0_BYTES,
                                   out + b * YVO_Q8_0_ELEMENTS))
            return YVO_ERR_FORMAT;
    return YVO_OK;
}

/* ------------------------------------------------- single-head attention ---- */

/* src/backend/cpu.c:307-399, with src/backend/core.c:1095-1141 for the argument
 * checks that precede it (seq_len 0 -> INVALID_ARG, position >= seq_len -> BOUNDS,
 * non-finite or non-positive scale -> INVALID_ARG). */
int yvo_attention_head(const float *q, const float *k, size_t k_stride,
                       const float *v, size_t v_stride, uint64_t seq_len,
                       uint64_t position, uint64_t head_dim, float scale,
                       int causal, float *score, float *prob, float *out,
                       double *lse)
{
    float *own = NULL;
    double max_score = 0.0, sum_exp = 0.0;
    uint64_t visible, i, d;
    if (!q || !k || !v || !out || !head_dim) return YVO_ERR_INVALID_ARG;
    if (seq_len == 0) return YVO_ERR_INVALID_ARG;
    if (position >= seq_len) return YVO_ERR_BOUNDS;
    if (!isfinite(scale) || scale <= 0.0f) return YVO_ERR_INVALID_ARG;
    if (!score || !prob) {
        own = (float *)malloc((size_t)seq_len * 2u * sizeof(float));
        if (!own) return YVO_ERR_STATE;
        if (!score) score = own;
        if (!prob) prob = own + seq_len;
    }
    visible = causal ? position + 1u : seq_len;
    for (i = 0; i < seq_len; ++i) {
        const float *row = k + i * k_stride;
        double s = 0.0;
        if (causal && i > position) {
            score[i] = 0.0f;
            prob[i] = 0.0f;
            continue;
        }
        for (d = 0; d < head_dim; ++d) s += (double)q[d] * (double)row[d];
        s *= (double)scale;
        score[i] = (float)s;
        /* the running maximum is taken over the double score ... */
        if (i == 0 || s > max_score) max_score = s;
    }
    for (i = 0; i < visible; ++i) {
        /* ... but the exponent uses the score as re-read from float storage */
        double e = yvo_exp((double)score[i] - max_score);
        prob[i] = (float)e;
        sum_exp += e;
    }
    if (sum_exp <= 0.0) {
        free(own);
        return YVO_ERR_STATE;
    }
    for (i = 0; i < visible; ++i) prob[i] = (float)((double)prob[i] / sum_exp);
    /* The reference sums over rows for one output lane at a time; summing all lanes
     * row by row performs the identical additions per lane in the identical order. */
    {
        double *acc = (double *)calloc((size_t)head_dim, sizeof(double));
        if (!acc) {
            free(own);
            return YVO_ERR_STATE;
        }
        for (i = 0; i < visible; ++i) {
            const float *row = v + i * v_stride;
            double p = (double)prob[i];
            for (d = 0; d < head_dim; ++d) acc[d] += p * (double)row[d];
        }
        for (d = 0; d < head_dim; ++d) out[d] = (float)acc[d];
        free(acc);
    }
    if (lse) *lse = max_score + log(sum_exp);
    free(own);
    return YVO_OK;
}

/* ---------------------------------------------------- multi-token GQA ---- */

static int u64_mul(uint64_t a, uint64_t b, uint64_t *out)
{
    if (a && b > UINT64_MAX / a) return 0;
    *out = a * b;
    return 1;
}

/* Admission follows src/backend/cuda/exact_attention.c:8-34. */
int yvo_gqa_attention(const float *q, const float *k, const float *v, float *out,
                      double *lse, uint64_t query_tokens, uint64_t kv_tokens,
                      uint64_t query_start, uint64_t query_heads,
                      uint64_t kv_heads, uint64_t head_dim, uint64_t q_stride,
                      uint64_t k_stride, uint64_t v_stride, int causal,
                      int threads)
{
    uint64_t q_width, kv_width, units, group;
    float scale;
    int status = YVO_OK;
    long long unit;
    if (!q || !k || !v || !out || !query_tokens || !kv_tokens ||
        query_start > UINT64_MAX - query_tokens ||
        query_start + query_tokens > kv_tokens || !query_heads || !kv_heads ||
        query_heads % kv_heads || !head_dim ||
        !u64_mul(query_heads, head_dim, &q_width) ||
        !u64_mul(kv_heads, head_dim, &kv_width) ||
        (q_stride && q_stride < q_width) || (k_stride && k_stride < kv_width) ||
        (v_stride && v_stride < kv_width) ||
        !u64_mul(query_tokens, query_heads, &units))
        return YVO_ERR_INVALID_ARG;
    if (!q_stride) q_stride = q_width;
    if (!k_stride) k_stride = kv_width;
    if (!v_stride) v_stride = kv_width;
    group = query_heads / kv_heads;
    scale = 1.0f / sqrtf((float)head_dim);
    threads = clamp_threads(threads);
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (unit = 0; unit < (long long)units; ++unit) {
        uint64_t token = (uint64_t)unit / query_heads;
        uint64_t head = (uint64_t)unit % query_heads;
        /* src/backend/cuda/transformer_kernels.cu:151: kv head = q head / group */
        uint64_t kv_head = head / group;
        /* visibility: source <= query_start + token; evaluate over that prefix with a
         * causal position at its last row (or over all rows when the mask is FULL) */
        uint64_t position = causal ? query_start + token : kv_tokens - 1u;
        double unit_lse = 0.0;
        int rc = yvo_attention_head(
            q + token * q_stride + head * head_dim, k + kv_head * head_dim, k_stride,
            v + kv_head * head_dim, v_stride, kv_tokens, position, head_dim, scale,
            causal, NULL, NULL, out + (token * query_heads + head) * head_dim,
            &unit_lse);
        if (lse) lse[token * query_heads + head] = unit_lse;
        if (rc != YVO_OK) {
#pragma omp critical
            status = rc;
        }
    }
    return status;
}

int yvo_gqa_attention_bf16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                           float *out_f32, uint16_t *out_bf16, double *lse,
                           uint64_t query_tokens, uint64_t kv_tokens,
                           uint64_t query_start, uint64_t query_heads,
                           uint64_t kv_heads, uint64_t head_dim, int causal,
                           int threads)
{
    size_t qn = (size_t)(query_tokens * query_heads * head_dim);
    size_t kn = (size_t)(kv_tokens * kv_heads * head_dim);
    float *qf = (float *)malloc(qn * sizeof(float));
    float *kf = (float *)malloc(kn * sizeof(float));
    float *vf = (float *)malloc(kn * sizeof(float));
    float *own_out = NULL;
    int rc = YVO_ERR_STATE;
    if (!out_f32) out_f32 = own_out = (float *)malloc(qn * sizeof(float));
    if (qf && kf && vf && out_f32) {
        yvo_bf16_decode_n(q, qf, qn);
        yvo_bf16_decode_n(k, kf, kn);
        yvo_bf16_decode_n(v, vf, kn);
        rc = yvo_gqa_attention(qf, kf, vf, out_f32, lse, query_tokens, kv_tokens,
                               query_start, query_heads, kv_heads, head_dim, 0, 0, 0,
                               causal, threads);
        if (rc == YVO_OK && out_bf16) yvo_bf16_encode_n(out_f32, out_bf16, qn);
    }
    free(qf);
    free(kf);
    free(vf);
    free(own_out);
    return rc;
}

/* ------------------------------------------------------- paged decode ---- */

typedef void (*row_widen_fn)(const void *pool, uint64_t row_index, uint64_t head_dim,
                             float *dst, int *ok);

static void widen_bf16(const void *pool, uint64_t row_index, uint64_t head_dim,
                       float *dst, int *ok)
{
    (void)ok;
    yvo_bf16_decode_n((const uint16_t *)pool + row_index * head_dim, dst, (size_t)head_dim);
}

static void widen_q8_0(const void *pool, uint64_t row_index, uint64_t head_dim,
                       float *dst, int *ok)
{
    const unsigned char *row = (const unsigned char *)pool +
                               row_index * (head_dim / YVO_Q8_0_ELEMENTS) * YVO_Q8_0_BYTES;
    if (yvo_q8_0_decode_row(row, (size_t)head_dim, dst) != YVO_OK) *ok = 0;
}

/* Gathers one session's K and V rows for one kv head through the page table into
 * contiguous F32 [context][head_dim], then applies the single-head operator for
 * each query head of the group.  The gathered copy is what makes "paged ==
 * contiguous" hold bit for bit. */
static int paged_decode(const uint16_t *q, const void *k_pool, const void *v_pool,
                        row_widen_fn widen, const int32_t *page_table,
                        const int32_t *context, float *out_f32, uint16_t *out_bf16,
                        double *lse, uint64_t sessions, uint64_t query_heads,
                        uint64_t kv_heads, uint64_t head_dim, uint64_t page_tokens,
                        uint64_t pool_pages, uint64_t table_stride, int threads)
{
    uint64_t group, units, s;
    float scale;
    int status = YVO_OK;
    long long unit;
    if (!q || !k_pool || !v_pool || !page_table || !context || !sessions ||
        !query_heads || !kv_heads || query_heads % kv_heads || !head_dim ||
        !page_tokens || !pool_pages || !table_stride)
        return YVO_ERR_INVALID_ARG;
    for (s = 0; s < sessions; ++s) {
        uint64_t pages, p;
        if (context[s] <= 0) return YVO_ERR_INVALID_ARG;
        pages = ((uint64_t)context[s] + page_tokens - 1u) / page_tokens;
        if (pages > table_stride) return YVO_ERR_BOUNDS;
        for (p = 0; p < pages; ++p) {
            int32_t id = page_table[s * table_stride + p];
            if (id < 0 || (uint64_t)id >= pool_pages) return YVO_ERR_BOUNDS;
        }
    }
    group = query_heads / kv_heads;
    units = sessions * kv_heads;
    scale = 1.0f / sqrtf((float)head_dim);
    threads = clamp_threads(threads);
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (unit = 0; unit < (long long)units; ++unit) {
        uint64_t session = (uint64_t)unit / kv_heads, kv_head = (uint64_t)unit % kv_heads;
        uint64_t n = (uint64_t)context[session], t, g;
        float *kf = (float *)malloc((size_t)(n * head_dim) * sizeof(float));
        float *vf = (float *)malloc((size_t)(n * head_dim) * sizeof(float));
        float *qf = (float *)malloc((size_t)head_dim * sizeof(float));
        float *of = (float *)malloc((size_t)head_dim * sizeof(float));
        int ok = kf && vf && qf && of, rc = YVO_OK;
        for (t = 0; ok && t < n; ++t) {
            uint64_t page = (uint64_t)page_table[session * table_stride + t / page_tokens];
            uint64_t row = (page * page_tokens + t % page_tokens) * kv_heads + kv_head;
            widen(k_pool, row, head_dim, kf + t * head_dim, &ok);
            widen(v_pool, row, head_dim, vf + t * head_dim, &ok);
        }
        if (!ok) rc = YVO_ERR_FORMAT;
        for (g = 0; rc == YVO_OK && g < group; ++g) {
            uint64_t head = kv_head * group + g;
            uint64_t o = (session * query_heads + head) * head_dim;
            double unit_lse = 0.0;
            yvo_bf16_decode_n(q + o, qf, (size_t)head_dim);
            rc = yvo_attention_head(qf, kf, (size_t)head_dim, vf, (size_t)head_dim, n,
                                    n - 1u, head_dim, scale, 1, NULL, NULL, of, &unit_lse);
            if (rc != YVO_OK) break;
            if (out_f32) memcpy(out_f32 + o, of, (size_t)head_dim * sizeof(float));
            if (out_bf16) yvo_bf16_encode_n(of, out_bf16 + o, (size_t)head_dim);
            if (lse) lse[session * query_heads + head] = unit_lse;
        }
        if (rc != YVO_OK) {
#pragma omp critical
            status = rc;
        }
        free(kf);
        free(vf);
        free(qf);
        free(of);
    }
    return status;
}

int yvo_paged_decode_bf16(const uint16_t *q, const uint16_t *k_pool,
                          const uint16_t *v_pool, const int32_t *page_table,
                          const int32_t *context, float *out_f32,
                          uint16_t *out_bf16, double *lse, uint64_t sessions,
                          uint64_t query_heads, uint64_t kv_heads,
                          uint64_t head_dim, uint64_t page_tokens,
                          uint64_t pool_pages, uint64_t table_stride, int threads)
{
    return paged_decode(q, k_pool, v_pool, widen_bf16, page_table, context, out_f32,
                        out_bf16, lse, sessions, query_heads, kv_heads, head_dim,
                        page_tokens, pool_pages, table_stride, threads);
}

int yvo_paged_decode_q8_0(const uint16_t *q, const unsigned char *k_pool,
                          const unsigned char *v_pool, const int32_t *page_table,
                          const int32_t *context, float *out_f32,
                          uint16_t *out_bf16, double *lse, uint64_t sessions,
                          uint64_t query_heads, uint64_t kv_heads,
                          uint64_t head_dim, uint64_t page_tokens,
                          uint64_t pool_pages, uint64_t table_stride, int threads)
{
    if (head_dim % YVO_Q8_0_ELEMENTS) return YVO_ERR_FORMAT;
    return paged_decode(q, k_pool, v_pool, widen_q8_0, page_table, context, out_f32,
                        out_bf16, lse, sessions, query_heads, kv_heads, head_dim,
                        page_tokens, pool_pages, table_stride, threads);
}

/* ------------------------------------------------ rotary positions ---- */

/* src/graph/numeric.c:877-917 */
double yvo_yarn_frequency(const yvo_position_policy *policy, uint64_t pair, uint64_t rope_dims)
{
    static const double pi = 3.14159265358979323846264338327950288;
    double frequency;
    if (!policy || rope_dims < 2u || policy->theta <= 1u) return 0.0;
    frequency = 1.0 / pow((double)policy->theta, (double)(pair * 2u) / (double)rope_dims);
    if (policy->original_context && policy->scaling_factor) {
        const double denominator = 2.0 * log((double)policy->theta);
        double low = floor((double)rope_dims *
                           log((double)policy->original_context /
                               ((double)policy->beta_fast * 2.0 * pi)) / denominator);
        double high = ceil((double)rope_dims *
                           log((double)policy->original_context /
                               ((double)policy->beta_slow * 2.0 * pi)) / denominator);
        double ramp, smooth;
        if (low < 0.0) low = 0.0;
        if (high > (double)rope_dims - 1.0) high = (double)rope_dims - 1.0;
        if (low == high) high += 0.001;
        ramp = ((double)pair - low) / (high - low);
        if (ramp < 0.0) ramp = 0.0;
        if (ramp > 1.0) ramp = 1.0;
        smooth = 1.0 - ramp;
        frequency = frequency / (double)policy->scaling_factor * (1.0 - smooth) + frequency * smooth;
    }
    return frequency;
}

/* src/graph/numeric.c:919-949 */
int yvo_rope_apply(float *values, uint64_t count, uint64_t rope_dims, uint64_t position,
                   const yvo_position_policy *policy, int inverse)
{
    uint64_t start, i;
    if (!values || !count || rope_dims < 2u || rope_dims > count || !policy || policy->theta <= 1u)
        return YVO_ERR_INVALID_ARG;
    if (rope_dims & 1u) rope_dims--;
    start = count - rope_dims;
    for (i = 0; i < rope_dims; i += 2u) {
        const double angle = (double)position * yvo_yarn_frequency(policy, i / 2u, rope_dims);
        const double c = cos(angle), s = inverse ? -sin(angle) : sin(angle);
        const double x = values[start + i], y = values[start + i + 1u];
        if (!isfinite(x) || !isfinite(y) || !isfinite(c) || !isfinite(s)) return YVO_ERR_FORMAT;
        values[start + i] = (float)(x * c - y * s);
        values[start + i + 1u] = (float)(x * s + y * c);
    }
    return YVO_OK;
}

/* src/graph/core.c:499-507 */
int yvo_reduce_output_finish(float *rows, uint64_t heads, uint64_t dim, uint64_t position,
                             const yvo_position_policy *policy)
{
    uint64_t head, lane;
    if (!rows || !heads || !dim || !policy) return YVO_ERR_INVALID_ARG;
    for (head = 0; head < heads; ++head) {
        float *row = rows + head * dim;
        int rc;
        for (lane = 0; lane < dim; ++lane) row[lane] = yvo_bf16_decode(yvo_bf16_encode(row[lane]));
        rc = yvo_rope_apply(row, dim, policy->rope_dimensions, position, policy, 1);
        if (rc != YVO_OK) return rc;
        for (lane = 0; lane < dim; ++lane) {
            if (!isfinite(row[lane])) return YVO_ERR_FORMAT;
            row[lane] = yvo_bf16_decode(yvo_bf16_encode(row[lane]));
        }
    }
    return YVO_OK;
}

/* ------------------------------------------------ shared-KV (MLA) head ---- */

/* src/graph/core.c:361-388 (row visit) and :471-508 (head): the sink logit seeds
 * the maximum and the denominator; pass 1 finds the maximum, pass 2 accumulates
 * exp(score - max) into the denominator (double) and into the float destination. */
int yvo_shared_kv_head(const float *q, const float *rows, size_t row_stride,
                       uint64_t row_count, uint64_t key_dim, uint64_t value_dim,
                       double scale, const float *sink, float *out, double *lse)
{
    double maximum = sink ? (double)*sink : -INFINITY, denominator;
    uint64_t i, lane;
    if (!q || !rows || !out || !key_dim || !value_dim || value_dim > key_dim ||
        row_stride < key_dim)
        return YVO_ERR_INVALID_ARG;
    if (sink && !isfinite(*sink)) return YVO_ERR_FORMAT;
    if (!sink && !row_count) return YVO_ERR_INVALID_ARG;
    for (i = 0; i < row_count; ++i) {
        const float *row = rows + i * row_stride;
        double s = 0.0;
        for (lane = 0; lane < key_dim; ++lane) {
            if (!isfinite(q[lane]) || !isfinite(row[lane])) return YVO_ERR_FORMAT;
            s += (double)q[lane] * (double)row[lane];
        }
        s *= scale;
        if (!isfinite(s)) return YVO_ERR_FORMAT;
        if (s > maximum) maximum = s;
    }
    denominator = sink ? exp((double)*sink - maximum) : 0.0;
    memset(out, 0, (size_t)value_dim * sizeof(float));
    for (i = 0; i < row_count; ++i) {
        const float *row = rows + i * row_stride;
        double s = 0.0, w;
        for (lane = 0; lane < key_dim; ++lane) s += (double)q[lane] * (double)row[lane];
        w = exp(s * scale - maximum);
        if (!isfinite(w)) return YVO_ERR_FORMAT;
        denominator += w;
        for (lane = 0; lane < value_dim; ++lane) out[lane] += (float)(w * row[lane]);
    }
    if (!isfinite(denominator) || denominator <= 0.0) return YVO_ERR_FORMAT;
    for (lane = 0; lane < value_dim; ++lane)
        out[lane] = (float)((double)out[lane] / denominator);
    if (lse) *lse = maximum + log(denominator);
    return YVO_OK;
}

int yvo_mla_decode_bf16(const uint16_t *q, const uint16_t *pool,
                        const int32_t *page_table, const int32_t *context,
                        float *out_f32, uint16_t *out_bf16, double *lse,
                        uint64_t batch, uint64_t heads, uint64_t key_dim,
                        uint64_t value_dim, uint64_t page_tokens,
                        uint64_t pool_pages, uint64_t table_stride,
                        const float *sinks, uint64_t sliding_window,
                        const uint16_t *compressed_pool, const int32_t *compressed_table,
                        const int32_t *compressed_count, uint64_t compressed_pool_pages,
                        uint64_t compressed_table_stride, const int32_t *selected,
                        uint64_t selected_stride, int threads)
{
    uint64_t b;
    double scale;
    int status = YVO_OK;
    long long unit;
    if (!q || !pool || !page_table || !context || !batch || !heads || !key_dim ||
        !value_dim || value_dim > key_dim || !page_tokens || !pool_pages || !table_stride)
        return YVO_ERR_INVALID_ARG;
    for (b = 0; b < batch; ++b) {
        uint64_t pages, p;
        if (context[b] <= 0) return YVO_ERR_INVALID_ARG;
        pages = ((uint64_t)context[b] + page_tokens - 1u) / page_tokens;
        if (pages > table_stride) return YVO_ERR_BOUNDS;
        for (p = 0; p < pages; ++p) {
            int32_t id = page_table[b * table_stride + p];
            if (id < 0 || (uint64_t)id >= pool_pages) return YVO_ERR_BOUNDS;
        }
        if (compressed_pool) {
            if (!compressed_table || !compressed_count || compressed_count[b] < 0)
                return YVO_ERR_INVALID_ARG;
            if (selected) {
                /* src/graph/core.c:443-452: the list names the rows, in list order */
                if ((uint64_t)compressed_count[b] > selected_stride) return YVO_ERR_BOUNDS;
                for (p = 0; p < (uint64_t)compressed_count[b]; ++p) {
                    int32_t index = selected[b * selected_stride + p], id;
                    if (index < 0 || (uint64_t)index / page_tokens >= compressed_table_stride)
                        return YVO_ERR_BOUNDS;
                    id = compressed_table[b * compressed_table_stride + (uint64_t)index / page_tokens];
                    if (id < 0 || (uint64_t)id >= compressed_pool_pages) return YVO_ERR_BOUNDS;
                }
                continue;
            }
            pages = ((uint64_t)compressed_count[b] + page_tokens - 1u) / page_tokens;
            if (pages > compressed_table_stride) return YVO_ERR_BOUNDS;
            for (p = 0; p < pages; ++p) {
                int32_t id = compressed_table[b * compressed_table_stride + p];
                if (id < 0 || (uint64_t)id >= compressed_pool_pages) return YVO_ERR_BOUNDS;
            }
        }
    }
    /* src/graph/core.c:604 */
    scale = 1.0 / sqrt((double)key_dim);
    threads = clamp_threads(threads);
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (unit = 0; unit < (long long)batch; ++unit) {
        /* src/backend/cuda/attention_kernels.cu:79-84: the token at position context - 1
         * sees positions first .. context - 1, first = context - window (or 0) */
        const uint64_t total = (uint64_t)context[unit];
        const uint64_t first = sliding_window && total > sliding_window ? total - sliding_window : 0u;
        /* src/graph/core.c:437-468: the compressed rows follow the local ones in the same
         * two passes (one maximum, one denominator) */
        const uint64_t extra = compressed_pool ? (uint64_t)compressed_count[unit] : 0u;
        const uint64_t local = total - first;
        uint64_t n = local + extra, t, h;
        float *rows = (float *)malloc((size_t)(n * key_dim) * sizeof(float));
        float *qf = (float *)malloc((size_t)key_dim * sizeof(float));
        float *of = (float *)malloc((size_t)value_dim * sizeof(float));
        int rc = rows && qf && of ? YVO_OK : YVO_ERR_STATE;
        for (t = 0; rc == YVO_OK && t < extra; ++t) {
            const uint64_t at = selected ? (uint64_t)selected[(uint64_t)unit * selected_stride + t] : t;
            uint64_t page = (uint64_t)compressed_table[(uint64_t)unit * compressed_table_stride +
                                                       at / page_tokens];
            yvo_bf16_decode_n(compressed_pool + (page * page_tokens + at % page_tokens) * key_dim,
                              rows + (local + t) * key_dim, (size_t)key_dim);
        }
        for (t = 0; rc == YVO_OK && t < local; ++t) {
            const uint64_t at = first + t;
            uint64_t page = (uint64_t)page_table[(uint64_t)unit * table_stride + at / page_tokens];
            yvo_bf16_decode_n(pool + (page * page_tokens + at % page_tokens) * key_dim,
                              rows + t * key_dim, (size_t)key_dim);
        }
        for (h = 0; rc == YVO_OK && h < heads; ++h) {
            uint64_t qo = ((uint64_t)unit * heads + h) * key_dim;
            uint64_t oo = ((uint64_t)unit * heads + h) * value_dim;
            double unit_lse = 0.0;
            yvo_bf16_decode_n(q + qo, qf, (size_t)key_dim);
            rc = yvo_shared_kv_head(qf, rows, (size_t)key_dim, n, key_dim, value_dim,
                                    scale, sinks ? sinks + h : NULL, of, &unit_lse);
            if (rc != YVO_OK) break;
            if (out_f32) memcpy(out_f32 + oo, of, (size_t)value_dim * sizeof(float));
            if (out_bf16) yvo_bf16_encode_n(of, out_bf16 + oo, (size_t)value_dim);
            if (lse) lse[(uint64_t)unit * heads + h] = unit_lse;
        }
        if (rc != YVO_OK) {
#pragma omp critical
            status = rc;
        }
        free(rows);
        free(qf);
        free(of);
    }
    return status;
}

/* ---------------------------------------------------------- LSE merge ---- */

int yvo_lse_merge(const float *part_out, const double *part_lse, uint64_t parts,
                  uint64_t dim, float *out, double *lse)
{
    double top = -INFINITY, total = 0.0;
    uint64_t p, d;
    if (!part_out || !part_lse || !out || !parts || !dim) return YVO_ERR_INVALID_ARG;
    for (p = 0; p < parts; ++p)
        if (part_lse[p] > top) top = part_lse[p];
    if (!isfinite(top)) return YVO_ERR_STATE;
    for (p = 0; p < parts; ++p) total += exp(part_lse[p] - top);
    for (d = 0; d < dim; ++d) {
        double acc = 0.0;
        for (p = 0; p < parts; ++p)
            if (part_lse[p] > -INFINITY)
                acc += exp(part_lse[p] - top) * (double)part_out[p * dim + d];
        out[d] = (float)(acc / total);
    }
    if (lse) *lse = top + log(total);
    return YVO_OK;
}

/* src/backend/cuda/transformer_kernels.cu:79-108 */
int yvo_rotary_half_bf16(uint16_t *values, const float *cosines, const float *sines,
                         uint64_t tokens, uint64_t heads, uint64_t head_dim,
                         uint64_t rotary_dim)
{
    const uint64_t half = rotary_dim / 2u;
    uint64_t vector, lane;
    if (!values || !cosines || !sines || !tokens || !heads || !half || rotary_dim > head_dim)
        return -1;
    for (vector = 0; vector < tokens * heads; ++vector) {
        const uint64_t token = vector / heads;
        uint16_t *base = values + vector * head_dim;
        for (lane = 0; lane < half; ++lane) {
            const float cosine = cosines[token * rotary_dim + lane];
            const float sine = sines[token * rotary_dim + lane];
            const float first = yvo_bf16_decode(base[lane]);
            const float second = yvo_bf16_decode(base[half + lane]);
            float first_product = yvo_bf16_decode(yvo_bf16_encode(first * cosine));
            float second_product = yvo_bf16_decode(yvo_bf16_encode(second * sine));
            base[lane] = yvo_bf16_encode(first_product - second_product);
            first_product = yvo_bf16_decode(yvo_bf16_encode(second * cosine));
            second_product = yvo_bf16_decode(yvo_bf16_encode(first * sine));
            base[half + lane] = yvo_bf16_encode(first_product + second_product);
        }
    }
    return 0;
}

/* src/backend/cuda/transformer_kernels.cu:79-108 on the F32 values the kernel itself takes:
 * the inputs enter the products unrounded, every product and sum is rounded to bf16. */
int yvo_rotary_half_f32(float *values, const float *cosines, const float *sines,
                        uint64_t tokens, uint64_t heads, uint64_t head_dim,
                        uint64_t rotary_dim)
{
    const uint64_t half = rotary_dim / 2u;
    uint64_t vector, lane;
    if (!values || !cosines || !sines || !tokens || !heads || !half || rotary_dim > head_dim)
        return -1;
    for (vector = 0; vector < tokens * heads; ++vector) {
        const uint64_t token = vector / heads;
        float *base = values + vector * head_dim;
        for (lane = 0; lane < half; ++lane) {
            const float cosine = cosines[token * rotary_dim + lane];
            const float sine = sines[token * rotary_dim + lane];
            const float first = base[lane], second = base[half + lane];
            float first_product = yvo_bf16_decode(yvo_bf16_encode(first * cosine));
            float second_product = yvo_bf16_decode(yvo_bf16_encode(second * sine));
            base[lane] = yvo_bf16_decode(yvo_bf16_encode(first_product - second_product));
            first_product = yvo_bf16_decode(yvo_bf16_encode(second * cosine));
            second_product = yvo_bf16_decode(yvo_bf16_encode(first * sine));
            base[half + lane] = yvo_bf16_decode(yvo_bf16_encode(first_product + second_product));
        }
    }
    return 0;
}

/* The decoder's own order (src/runtime/decoder.c:1112-1131): the plain F32 rotation
 * (yvex_rotary_half_plain_f32, src/backend/cuda/transformer_kernels.cu:110-134) followed by
 * the bf16 rounding of the whole tensor (decoder_round -> yvex_attention_bf16_round,
 * src/backend/cuda/kernels.cu:40-58), suffix lanes included.  The two float expressions
 * first * cosine - second * sine and second * cosine + first * sine are evaluated with the
 * contraction LLVM's combiner applies on both GPU targets at default flags: the first
 * product fused into the sum, the second rounded to float on its own. */
int yvo_rotary_half_f32_rounded(float *values, const float *cosines, const float *sines,
                                uint64_t tokens, uint64_t heads, uint64_t head_dim,
                                uint64_t rotary_dim)
{
    uint64_t index;
    const int rc = yvo_rotary_half_plain_f32(values, cosines, sines, tokens, heads, head_dim, rotary_dim);
    if (rc != 0) return rc;
    for (index = 0; index < tokens * heads * head_dim; ++index)
        values[index] = yvo_bf16_decode(yvo_bf16_encode(values[index]));
    return 0;
}

/* The rotation alone (the kernel behind the rotary_half_f32 operator slot,
 * src/backend/cuda/capability.c:35, src/backend/cuda/transformer_kernels.cu:110-134), nothing
 * rounded to bf16, with the contraction described above. */
int yvo_rotary_half_plain_f32(float *values, const float *cosines, const float *sines,
                              uint64_t tokens, uint64_t heads, uint64_t head_dim,
                              uint64_t rotary_dim)
{
    const uint64_t half = rotary_dim / 2u;
    uint64_t vector, lane;
    if (!values || !cosines || !sines || !tokens || !heads || !half || rotary_dim > head_dim)
        return -1;
    for (vector = 0; vector < tokens * heads; ++vector) {
        const uint64_t token = vector / heads;
        float *base = values + vector * head_dim;
        for (lane = 0; lane < half; ++lane) {
            const float cosine = cosines[token * rotary_dim + lane];
            const float sine = sines[token * rotary_dim + lane];
            const float first = base[lane], second = base[half + lane];
            const float second_sine = second * sine, first_sine = first * sine;
            base[lane] = fmaf(first, cosine, -second_sine);
            base[half + lane] = fmaf(second, cosine, first_sine);
        }
    }
    return 0;
}

/* src/backend/cuda/transformer_kernels.cu:353-364 */
int yvo_sigmoid_gate_bf16(const float *values, const float *gate, uint64_t count, float *out)
{
    uint64_t index;
    if (!values || !gate || !out) return YVO_ERR_INVALID_ARG;
    for (index = 0; index < count; ++index) {
        const float scale = 1.0f / (1.0f + expf(-gate[index]));
        out[index] = yvo_bf16_decode(yvo_bf16_encode(values[index] * scale));
    }
    return YVO_OK;
}
