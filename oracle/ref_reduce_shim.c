/*
 * Thin exporter around the reference's own shared-KV attention reduce
 * (yvex_attention_reduce_chunk, src/graph/core.c:609-700, declared in
 * src/graph/private.h:438).  TEST INFRASTRUCTURE ONLY.
 *
 * Compiled together with the reference sources where they lie (oracle/Makefile, target
 * "ref"); nothing from the reference tree is copied here.  It fills the reference's plan
 * and history structures from flat arrays for ONE query token and calls the reduce, so a
 * test can hold the restatement in yvex_attention_oracle.c (sink logits, sliding-window
 * filter, compressed candidate rows) against the reference's own arithmetic.
 *
 * What the reference does after the softmax belongs to its model family and is kept as it
 * is: the rows are rounded to bf16, the last rope_dims lanes are rotated back by the
 * token's position, and the row is rounded again (src/graph/core.c:499-507).  A caller
 * that asks for rope_dims = 2 gets bf16(softmax row) on every lane but the last two; the
 * rotation's own policy fields (theta and the YaRN scaling) are passed through.
 */
#include <string.h>

#include <yvex/backend.h>
#include <yvex/internal/backend.h>
#include <yvex/internal/graph.h>

#include "src/graph/private.h"

#define YVREF_EXPORT __attribute__((visibility("default")))

/*
 * query [heads][dim]; local [local_count][dim] with local_positions (the last row is the
 * query token's own row at `position`); compressed [compressed_count][dim] with
 * compressed_positions; sinks [heads]; attention_class 0 (local window only) or 2 (dense
 * compressed class, compression_ratio given); out [heads][dim].
 */
YVREF_EXPORT int yvref_attention_reduce(const float *query, const float *local,
                                        const unsigned long long *local_positions,
                                        unsigned long long local_count, const float *compressed,
                                        const unsigned long long *compressed_positions,
                                        unsigned long long compressed_count, const float *sinks,
                                        unsigned long long heads, unsigned long long dim,
                                        unsigned long long sliding_window,
                                        unsigned long long compression_ratio,
                                        unsigned int attention_class, unsigned long long position,
                                        unsigned long long rope_dims, unsigned long long theta,
                                        unsigned long long scaling_factor,
                                        unsigned long long original_context,
                                        unsigned long long beta_fast, unsigned long long beta_slow,
                                        float *out)
{
    yvex_attention_layer_plan layer;
    yvex_attention_history_view history;
    yvex_attention_failure failure;
    yvex_error err;
    if (!local_count) return YVEX_ERR_INVALID_ARG;
    memset(&layer, 0, sizeof(layer));
    memset(&history, 0, sizeof(history));
    memset(&failure, 0, sizeof(failure));
    yvex_error_clear(&err);
    layer.attention_class = (yvex_attention_class)attention_class;
    layer.compute_contract = YVEX_ATTENTION_COMPUTE_BF16_F32_RNE_V1;
    layer.compression_ratio = compression_ratio;
    layer.sliding_window = sliding_window;
    layer.query_heads = heads;
    layer.kv_heads = 1ull;
    layer.head_dimension = dim;
    layer.rope_head_dimension = rope_dims;
    layer.position.rope_dimension = rope_dims;
    layer.position.theta = theta;
    layer.position.scaling_factor = scaling_factor;
    layer.position.original_context = original_context;
    layer.position.beta_fast = beta_fast;
    layer.position.beta_slow = beta_slow;
    history.token_count = local_count - 1ull;
    history.local_tail_count = local_count - 1ull;
    history.local_kv = local;
    history.local_kv_stride = dim;
    history.local_positions = local_positions;
    history.compressed_entry_count = compressed_count;
    history.compressed_kv = compressed;
    history.compressed_kv_stride = dim;
    history.compressed_positions = compressed_positions;
    history.immutable = 1;
    return yvex_attention_reduce_chunk(
        &layer, query, &history, local + (local_count - 1ull) * dim, dim, NULL, 0ull, 0ull, NULL,
        NULL, 0ull, 0ull, NULL, NULL, 0ull, NULL, 0ull, sinks, 1ull, position, out, 0, NULL, NULL,
        0ull, NULL, NULL, &failure, &err);
}
