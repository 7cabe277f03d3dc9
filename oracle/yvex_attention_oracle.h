/*
 * CPU restatement of the YVEX attention hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is the parity checker for the gfx950 attention backend.  It is
 * linked or loaded only by tests, by the smoke check and by the benchmark's
 * CPU-baseline leg; no product code path may call into it.
 *
 * Every function names the reference source (relative to the yailabs/clori
 * tree) whose arithmetic it restates.  Pin status of each function:
 *
 *   yvo_exp, yvo_attention_head      pinned: reference literals
 *       (tests/unit/backend_ops.c:455-510), position-0 / uniform / dominant-key
 *       closed forms, libm brute force, and the compiled reference operator
 *       (oracle/_ref) on seeded inputs
 *   yvo_gqa_attention                pinned: reference KAT
 *       (tests/unit/cuda/quant_qtype.c:2117-2136) and the reference tests'
 *       integer-pattern inputs against an independent float two-pass softmax
 *   yvo_bf16_*, yvo_f16_*            pinned: reference literals
 *       (tests/reference/deepseek_attention.c:2696-2698), exhaustive 2^16
 *       round trips, compiled reference codecs (oracle/_ref)
 *   yvo_q8_0_*                       pinned: golden block
 *       (tests/unit/quant_numeric.c:514-526), zero block, refusal cases, the
 *       compiled reference block encoder and decoder (oracle/_ref, through
 *       yvex_quant_encode_block / yvex_quant_decode_block) on seeded blocks,
 *       and the invariants decode(encode(x)) error <= scale/2, idempotence
 *   yvo_shared_kv_head, and through it yvo_mla_decode_bf16 with sink logits, the
 *   sliding window and the dense compressed rows
 *       pinned: sink KAT (tests/reference/deepseek_attention.c:2722-2725); the
 *       reference's own reduce (yvex_attention_reduce_chunk, src/graph/core.c)
 *       compiled into oracle/_ref/libyvex_ref_reduce.so, bit for bit on every
 *       lane it does not rotate and on the other two after the same rotation;
 *       committed outputs of that reduce (tests/golden); the sink-free path
 *       equals a sink that underflows, bit for bit
 *   yvo_yarn_frequency, yvo_rope_apply, yvo_reduce_output_finish
       pinned: the reference's own reduce (oracle/_ref/libyvex_ref_reduce.so) run with
       64 rope lanes, with and without the YaRN ramp, bit for bit on every lane of the
       published row; committed outputs of that reduce (tests/golden); forward then
       inverse rotation returns the row within float rounding; position 0 is the
       identity; pair 0 has frequency 1
   yvo_rotary_half_bf16             pinned: known-answer case
 *       (tests/unit/cuda/quant_qtype.c:1988-2061), identity, quarter turn,
 *       float64 rotation within bf16 rounding
 *   yvo_rotary_half_f32              pinned: the same known-answer case on its F32
 *       literals, bit equality with yvo_rotary_half_bf16 on representable inputs,
 *       identity and quarter turn on inputs that are not
 *   yvo_rotary_half_f32_rounded      pinned: known-answer case of the plain rotation
 *       (tests/unit/cuda/quant_qtype.c:3050-3105), identity, quarter turn, float64
 *       rotation within one bf16 rounding; the choice of fused product is
 *       parity unpinned (results within a float rounding of a bf16 tie)
 *   yvo_rotary_half_plain_f32        pinned: the same known-answer case (exact in float),
 *       identity, quarter turn, float64 rotation within two float roundings; the
 *       choice of fused product is parity unpinned (the last bit of a result)
 *   yvo_sigmoid_gate_bf16            pinned: known-answer case
 *       (tests/unit/cuda/quant_qtype.c:2979-2981,3019-3033), closed forms
 *   yvo_paged_*, the page tables and LSE output of yvo_mla_*, the selected
 *   compressed class, yvo_lse_merge
 *       parity unpinned by the reference (it has no page table, no LSE, no
 *       split-K, no Q8_0 KV cache; its selected class needs the indexer that
 *       is outside this path).  Pinned here only by construction invariants:
 *       paged == contiguous on the gathered copy (bit-exact), page-placement
 *       permutation invariance, LSE closed forms, merge associativity,
 *       selected list == the listed rows concatenated (bit-exact).
 */
#ifndef YVEX_ATTENTION_ORACLE_H
#define YVEX_ATTENTION_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status values mirror include/yvex/core.h:13-26 of the reference. */
enum {
    YVO_OK = 0,
    YVO_ERR_FORMAT = -4,
    YVO_ERR_UNSUPPORTED = -5,
    YVO_ERR_BOUNDS = -7,
    YVO_ERR_STATE = -8,
    YVO_ERR_INVALID_ARG = -10
};

enum { YVO_Q8_0_ELEMENTS = 32, YVO_Q8_0_BYTES = 34 };

/* src/backend/cpu.c:217-255 */
double yvo_exp(double x);

/* src/gguf/quant_scalar.c:40-143 */
float yvo_f16_decode(uint16_t bits);
uint16_t yvo_f16_encode(float value);
float yvo_bf16_decode(uint16_t bits);
uint16_t yvo_bf16_encode(float value);
void yvo_bf16_decode_n(const uint16_t *src, float *dst, size_t n);
void yvo_bf16_encode_n(const float *src, uint16_t *dst, size_t n);

/* src/gguf/quant_block.c:160-186 (encode), :819-833 (decode).  encode returns 1 on
 * success and 0 when the scale is not representable, like the reference. */
int yvo_q8_0_encode_block(const float *source, unsigned char *encoded);
int yvo_q8_0_decode_block(const unsigned char *encoded, float *out);
/* Row helpers: n must be a multiple of 32. Return YVO_OK or YVO_ERR_FORMAT/BOUNDS. */
int yvo_q8_0_encode_row(const float *source, size_t n, unsigned char *encoded);
int yvo_q8_0_decode_row(const unsigned char *encoded, size_t n, float *out);

/*
 * One head, one query (src/backend/cpu.c:307-399).  K and V rows are addressed
 * as base + i*stride (elements); the reference operator is the stride == head_dim
 * case.  score/prob may be NULL (then internal scratch is used); lse may be NULL.
 * LSE is max + ln(sum_exp) formed from the same doubles the reference computes.
 */
int yvo_attention_head(const float *q, const float *k, size_t k_stride,
                       const float *v, size_t v_stride, uint64_t seq_len,
                       uint64_t position, uint64_t head_dim, float scale,
                       int causal, float *score, float *prob, float *out,
                       double *lse);

/*
 * Multi-token grouped-query attention, token/head/dim layout, strides in
 * elements per token (0 = packed), visibility source <= query_start + t for the
 * causal mask (include/yvex/internal/transformer.h:258-275,
 * src/backend/cuda/exact_attention.c:8-53,
 * src/backend/cuda/transformer_kernels.cu:146-166).  Each (token, head) unit is
 * evaluated with yvo_attention_head; scale is 1/sqrt(head_dim) as float.
 * out is packed [Tq, Hq, d] F32; lse (optional) is [Tq, Hq] doubles.
 * threads <= 1 runs serially.
 */
int yvo_gqa_attention(const float *q, const float *k, const float *v, float *out,
                      double *lse, uint64_t query_tokens, uint64_t kv_tokens,
                      uint64_t query_start, uint64_t query_heads,
                      uint64_t kv_heads, uint64_t head_dim, uint64_t q_stride,
                      uint64_t k_stride, uint64_t v_stride, int causal,
                      int threads);

/* bf16 in / bf16 out wrapper used for benchmark configurations 1 and 2: widens exactly to
 * F32, runs yvo_gqa_attention, returns the F32 result and its RNE bf16 rounding. */
int yvo_gqa_attention_bf16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                           float *out_f32, uint16_t *out_bf16, double *lse,
                           uint64_t query_tokens, uint64_t kv_tokens,
                           uint64_t query_start, uint64_t query_heads,
                           uint64_t kv_heads, uint64_t head_dim, int causal,
                           int threads);

/*
 * Paged decode.  Canonical pool layout (token-major rows, the reference's
 * [token, kv_head, dim] history rows cut into pages):
 *   bf16:  K and V pools are uint16 [pool_pages][page_tokens][kv_heads][head_dim]
 *   q8_0:  K and V pools are bytes  [pool_pages][page_tokens][kv_heads][head_dim/32][34]
 * page_table is int32 [sessions][table_stride]; context[s] tokens are visible
 * (non-causal over the first context[s] tokens; the single query sits at the
 * last position).  Refuses (YVO_ERR_BOUNDS) a page id outside [0,pool_pages) or
 * a context needing more than table_stride pages; context 0 is YVO_ERR_INVALID_ARG.
 * q is bf16 [sessions][query_heads][head_dim].
 */
int yvo_paged_decode_bf16(const uint16_t *q, const uint16_t *k_pool,
                          const uint16_t *v_pool, const int32_t *page_table,
                          const int32_t *context, float *out_f32,
                          uint16_t *out_bf16, double *lse, uint64_t sessions,
                          uint64_t query_heads, uint64_t kv_heads,
                          uint64_t head_dim, uint64_t page_tokens,
                          uint64_t pool_pages, uint64_t table_stride, int threads);

int yvo_paged_decode_q8_0(const uint16_t *q, const unsigned char *k_pool,
                          const unsigned char *v_pool, const int32_t *page_table,
                          const int32_t *context, float *out_f32,
                          uint16_t *out_bf16, double *lse, uint64_t sessions,
                          uint64_t query_heads, uint64_t kv_heads,
                          uint64_t head_dim, uint64_t page_tokens,
                          uint64_t pool_pages, uint64_t table_stride, int threads);

/*
 * Shared-KV head with optional sink logit (src/graph/core.c:361-388,471-508):
 * every row is both key (first key_dim lanes) and value (first value_dim lanes);
 * two passes, double score and denominator, libm exp, float accumulator updated
 * as dest += (float)(w * row), divide in double.  sink may be NULL (no sink).
 * rows are addressed as base + i*row_stride.  The reference has key_dim ==
 * value_dim == head_dimension; the absorbed-MLA form uses key_dim 576, value_dim 512.
 */
int yvo_shared_kv_head(const float *q, const float *rows, size_t row_stride,
                       uint64_t row_count, uint64_t key_dim, uint64_t value_dim,
                       double scale, const float *sink, float *out, double *lse);

/*
 * Absorbed-latent MLA decode over a paged latent cache (benchmark configuration 5).
 * q bf16 [batch][heads][key_dim]; pool bf16 [pool_pages][page_tokens][key_dim];
 * value = first value_dim lanes of each row; scale = 1/sqrt(key_dim) in double
 * (src/graph/core.c:604).  Output is F32 plus RNE bf16 [batch][heads][value_dim].
 * sinks: optional F32 [heads] sink logits handed to yvo_shared_kv_head; sliding_window:
 * 0 for the whole context, else only positions >= context - sliding_window are rows
 * (the position filter of src/backend/cuda/attention_kernels.cu:79-84 for the token at
 * position context - 1).  compressed_pool (optional): a second paged row set of the same
 * format; its first compressed_count[b] rows join the same softmax after the local rows
 * (src/graph/core.c:437-468, the class whose visible compressed rows are a prefix).
 * selected (optional, int32 [batch][selected_stride]): the compressed rows are instead the
 * listed positions of the session's compressed sequence, in list order, compressed_count[b]
 * of them (the selected class, src/graph/core.c:443-452).
 */
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
                        uint64_t selected_stride, int threads);

/*
 * Log-sum-exp merge of split partials for one head: part p holds a normalised
 * output o_p[dim] and lse_p; result = sum_p exp(lse_p - L) o_p with
 * L = log sum_p exp(lse_p).  Parts with lse = -inf are empty.
 */
int yvo_lse_merge(const float *part_out, const double *part_lse, uint64_t parts,
                  uint64_t dim, float *out, double *lse);

/*
 * Rotary position policy (include/yvex/internal/backend.h:51-54, the fields the rotation
 * reads) and the rotation itself (src/graph/numeric.c:877-949): the LAST rope_dims lanes of
 * a row of `count` lanes, adjacent pairs (2i, 2i+1), angle = position * frequency(i) with
 * the YaRN ramp when original_context and scaling_factor are set; all in double, each
 * result rounded to float.  inverse rotates by the negative angle.
 */
typedef struct {
    uint64_t theta, scaling_factor, original_context, beta_fast, beta_slow, rope_dimensions;
} yvo_position_policy;
double yvo_yarn_frequency(const yvo_position_policy *policy, uint64_t pair, uint64_t rope_dims);
int yvo_rope_apply(float *values, uint64_t count, uint64_t rope_dims, uint64_t position,
                   const yvo_position_policy *policy, int inverse);
/* What the shared-KV reduce does to each head's row after the softmax
 * (src/graph/core.c:499-507): round to bf16, rotate the rope lanes back by the token's
 * position, round again.  rows is [heads][dim] float, in place. */
int yvo_reduce_output_finish(float *rows, uint64_t heads, uint64_t dim, uint64_t position,
                             const yvo_position_policy *policy);

/*
 * Rotate-half position encoding on packed bf16 [tokens][heads][head_dim] vectors in
 * place, with explicit F32 cos/sin tables [tokens][rotary_dim] (only the first
 * rotary_dim / 2 entries of a row are used) and every product and sum rounded to bf16:
 * restates src/backend/cuda/transformer_kernels.cu:79-108 (yvex_rotary_half_f32), whose
 * F32 values are bf16-representable.  Pinned by the known-answer case the reference's own
 * GPU test holds (tests/unit/cuda/quant_qtype.c:1988-2061: one 4-wide vector, rotary
 * dimension 2, untouched suffix), by the identity rotation (cos 1, sin 0), the quarter
 * turn (cos 0, sin 1: halves swap with one sign flip), norm preservation up to bf16
 * rounding and a float64 rotation within that rounding.
 */
int yvo_rotary_half_bf16(uint16_t *values, const float *cosines, const float *sines,
                         uint64_t tokens, uint64_t heads, uint64_t head_dim,
                         uint64_t rotary_dim);
/* The same kernel on the F32 values it takes in the reference (in place): the inputs enter
 * the products as they are, products and sums are rounded to bf16 and stored as F32.
 * Pinned by the reference's known-answer case on its own F32 literals
 * (tests/unit/cuda/quant_qtype.c:1988-2061), by bit equality with yvo_rotary_half_bf16 on
 * bf16-representable inputs, and on other inputs by the identity rotation (the result is
 * the input rounded to bf16) and the quarter turn. */
int yvo_rotary_half_f32(float *values, const float *cosines, const float *sines,
                        uint64_t tokens, uint64_t heads, uint64_t head_dim,
                        uint64_t rotary_dim);
/* The order the reference's decoder runs in front of attention
 * (src/runtime/decoder.c:1112-1131, 1236-1242): the plain F32 rotation
 * (src/backend/cuda/transformer_kernels.cu:110-134) and then one bf16 rounding of every lane
 * of the tensor (src/backend/cuda/kernels.cu:40-58).  Pinned by the reference's
 * known-answer case for the plain rotation (tests/unit/cuda/quant_qtype.c:3050-3105, exact
 * in float), the identity and the quarter turn, a float64 rotation within one bf16
 * rounding, and agreement with the staged form within one bf16 step.  Which of the two
 * products of each sum the reference's compiler fuses is not visible in its sources: the
 * last bit of a result that lies within a float rounding of a bf16 tie is parity unpinned. */
int yvo_rotary_half_f32_rounded(float *values, const float *cosines, const float *sines,
                                uint64_t tokens, uint64_t heads, uint64_t head_dim,
                                uint64_t rotary_dim);
/* The rotation alone, nothing rounded to bf16: what the rotary_half_f32 operator slot runs
 * (src/backend/cuda/capability.c:35 binds it to yvex_rotary_half_plain_f32).  Same pins; with
 * no bf16 rounding behind it the unpinned choice of fused product is the last bit of every
 * result that is not exact. */
int yvo_rotary_half_plain_f32(float *values, const float *cosines, const float *sines,
                              uint64_t tokens, uint64_t heads, uint64_t head_dim,
                              uint64_t rotary_dim);

/*
 * Sigmoid output gate on attention rows: out = bf16(values * (1 / (1 + expf(-gate)))), all
 * F32 carriers; restates src/backend/cuda/transformer_kernels.cu:353-364
 * (yvex_sigmoid_product_bf16_f32), which the decoder applies to the published attention
 * rows (src/runtime/decoder.c:1266-1269).  Pinned by the reference's known-answer case
 * (tests/unit/cuda/quant_qtype.c:2979-2981,3019-3033: values {1,-2,0.5,4}, gates
 * {0, ln 3, -ln 3, 1}), gate 0 halves, large gates saturate to identity and zero.
 */
int yvo_sigmoid_gate_bf16(const float *values, const float *gate, uint64_t count, float *out);

/* Number of worker threads the *_threads arguments are clamped to. */
int yvo_hardware_threads(void);

#ifdef __cplusplus
}
#endif

#endif /* YVEX_ATTENTION_ORACLE_H */
