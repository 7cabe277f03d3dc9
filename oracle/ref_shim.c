/*
 * Thin exporter around the reference's own CPU attention operator and scalar /
 * block codecs.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is compiled together with the reference sources where they lie
 * (see oracle/Makefile, target "ref"); nothing from the reference tree is copied
 * here.  It exposes flat C entry points so a test can feed plain arrays to
 * yvex_backend_op_attention (src/backend/core.c:1095, CPU arm
 * src/backend/cpu.c:307-399) and to the public codec functions
 * (src/gguf/quant_scalar.c:40-143, src/gguf/quant_block.c yvex_quant_encode_block /
 * yvex_quant_decode_block).  The result validates the restatement in
 * yvex_attention_oracle.c; it is also usable as the "reference" CPU baseline.
 */
#include <string.h>

#include <yvex/backend.h>
#include <yvex/internal/backend.h>
#include <yvex/internal/quant_numeric.h>
#include <yvex/qtype.h>

#define YVREF_EXPORT __attribute__((visibility("default")))

static int ref_tensor(yvex_backend *backend, const char *name, unsigned int rank,
                      unsigned long long d0, unsigned long long d1, const float *data,
                      yvex_device_tensor **out, yvex_error *err)
{
    yvex_backend_tensor_desc desc;
    int rc;
    memset(&desc, 0, sizeof(desc));
    desc.name = name;
    desc.dtype = YVEX_DTYPE_F32;
    desc.rank = rank;
    desc.dims[0] = d0;
    desc.dims[1] = rank > 1u ? d1 : 0ull;
    desc.bytes = d0 * (rank > 1u ? d1 : 1ull) * sizeof(float);
    rc = yvex_backend_tensor_alloc(backend, &desc, out, err);
    if (rc == YVEX_OK && data)
        rc = yvex_backend_tensor_write(backend, *out, data, desc.bytes, err);
    return rc;
}

/* Runs the reference CPU operator on packed F32 arrays.  Returns its status. */
YVREF_EXPORT int yvref_op_attention(const float *q, const float *k, const float *v,
                                    unsigned long long seq_len,
                                    unsigned long long position,
                                    unsigned long long head_dim, float scale, int causal,
                                    float *score, float *prob, float *out)
{
    yvex_backend *backend = NULL;
    yvex_device_tensor *tq = NULL, *tk = NULL, *tv = NULL, *ts = NULL, *tp = NULL, *to = NULL;
    yvex_error err;
    int rc;
    yvex_error_clear(&err);
    rc = yvex_backend_open_cpu(&backend, &err);
    if (rc != YVEX_OK) return rc;
    if (seq_len && head_dim) {
        rc = ref_tensor(backend, "q", 1u, head_dim, 0ull, q, &tq, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "k", 2u, seq_len, head_dim, k, &tk, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "v", 2u, seq_len, head_dim, v, &tv, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "s", 1u, seq_len, 0ull, NULL, &ts, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "p", 1u, seq_len, 0ull, NULL, &tp, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "o", 1u, head_dim, 0ull, NULL, &to, &err);
    } else {
        /* the dispatch refuses seq_len 0 before looking at the tensors: give it
         * well-formed placeholders */
        rc = ref_tensor(backend, "q", 1u, 1ull, 0ull, NULL, &tq, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "k", 2u, 1ull, 1ull, NULL, &tk, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "v", 2u, 1ull, 1ull, NULL, &tv, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "s", 1u, 1ull, 0ull, NULL, &ts, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "p", 1u, 1ull, 0ull, NULL, &tp, &err);
        if (rc == YVEX_OK) rc = ref_tensor(backend, "o", 1u, 1ull, 0ull, NULL, &to, &err);
    }
    if (rc == YVEX_OK)
        rc = yvex_backend_op_attention(backend, tq, tk, tv, seq_len, position, scale, causal,
                                       ts, tp, to, &err);
    if (rc == YVEX_OK && score)
        rc = yvex_backend_tensor_read(backend, ts, score, seq_len * sizeof(float), &err);
    if (rc == YVEX_OK && prob)
        rc = yvex_backend_tensor_read(backend, tp, prob, seq_len * sizeof(float), &err);
    if (rc == YVEX_OK && out)
        rc = yvex_backend_tensor_read(backend, to, out, head_dim * sizeof(float), &err);
    yvex_backend_tensor_free(backend, to);
    yvex_backend_tensor_free(backend, tp);
    yvex_backend_tensor_free(backend, ts);
    yvex_backend_tensor_free(backend, tv);
    yvex_backend_tensor_free(backend, tk);
    yvex_backend_tensor_free(backend, tq);
    yvex_backend_close(backend);
    return rc;
}

YVREF_EXPORT float yvref_f16_decode(unsigned short bits) { return yvex_quant_f16_decode(bits); }
YVREF_EXPORT unsigned short yvref_f16_encode(float v) { return yvex_quant_f16_encode(v); }
YVREF_EXPORT float yvref_bf16_decode(unsigned short bits) { return yvex_quant_bf16_decode(bits); }
YVREF_EXPORT unsigned short yvref_bf16_encode(float v) { return yvex_quant_bf16_encode(v); }

/* Bulk forms so an exhaustive sweep does not pay one foreign call per value. */
YVREF_EXPORT void yvref_bf16_encode_n(const float *src, unsigned short *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; ++i) dst[i] = yvex_quant_bf16_encode(src[i]);
}

YVREF_EXPORT void yvref_f16_encode_n(const float *src, unsigned short *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; ++i) dst[i] = yvex_quant_f16_encode(src[i]);
}

YVREF_EXPORT void yvref_f16_decode_n(const unsigned short *src, float *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; ++i) dst[i] = yvex_quant_f16_decode(src[i]);
}

#ifdef YVREF_WITH_QUANT_BLOCK
YVREF_EXPORT int yvref_q8_0_encode_block(const float *source, unsigned char *encoded)
{
    yvex_quant_failure failure;
    yvex_error err;
    size_t bytes = 0u;
    yvex_error_clear(&err);
    return yvex_quant_encode_block(YVEX_GGUF_QTYPE_Q8_0, source, 32ull, encoded, 34u, &bytes,
                                   &failure, &err);
}

YVREF_EXPORT int yvref_q8_0_decode_block(const unsigned char *encoded, float *out)
{
    yvex_quant_failure failure;
    yvex_error err;
    yvex_error_clear(&err);
    return yvex_quant_decode_block(YVEX_GGUF_QTYPE_Q8_0, encoded, 34u, out, 32ull, &failure,
                                   &err);
}
#endif
