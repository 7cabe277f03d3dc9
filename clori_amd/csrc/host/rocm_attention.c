/* Attention operations of the ROCm arm: admission, workspace, launch geometry and
 * physical facts.  No arithmetic happens on the host.
 *
 *   yvex_rocm_op_attention            src/backend/cuda/ops.c:1717-1807 (bounded primitive)
 *   attention_workspace_required /
 *   attention_execute                 src/backend/cuda/exact_attention.c:8-107,
 *                                     src/backend/cuda/transformer.c:725-807
 *   paged / MLA decode                new surface (the reference has no paged KV)
 */
#include "rocm_state.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "../kernel_params.h"
#include "rocm_scratch.h"

_Static_assert(YVEX_ROCM_STATIC_SCRATCH_BYTES == YVEX_ROCM_STATIC_WORKSPACE_BYTES,
               "the public limit and the device array must have the same size");

enum {
    ROCM_EXACT_HEAD_MAX = 256,   /* src/backend/cuda/exact_attention.c:6 */
    ROCM_MFMA_HEAD_DIM = 128,
    ROCM_PAGE_TOKENS = 16,
    ROCM_GROUP_MAX = 16,
    ROCM_DECODE_WAVES = 2048,
    ROCM_DECODE_MIN_TILES = 8, /* 8 and 16 measure alike on a 4096-token context; 4 and 32 are a third slower */
    ROCM_TEAM_WAVES = 8,       /* waves of a decode team (one workgroup) */
    /* tiles a wave of a team is given when the history is short enough (context 4096: 10.3 us;
     * 1: 11.6, 4: 11.9, 8: 15.9) */
    ROCM_TEAM_TILES = 2,
    /* the same at head dimension 256, teams of four waves (24/4 heads, context 4096: 16.0 us;
     * 2: 18.3, 8: 19.7) */
    ROCM_TEAM_TILES_WIDE = 4,
    ROCM_TEAMS_MAX = 32,       /* teams per (session, kv head): two load trips of the last team's merge */
    ROCM_TEAM_GROUP_MAX = 8,   /* query heads per kv head a team's LDS holds */
    ROCM_PREFILL_ROWS = YVEX_ROCM_PREFILL_ROWS, /* query rows per prefill workgroup */
    ROCM_WORK_ALIGNMENT = 256    /* src/backend/cuda/transformer.c:17 */
};

static int refuse(yvex_error *err, yvex_status status, const char *where, const char *reason)
{
    yvex_error_set(err, status, where, reason);
    return status;
}

static unsigned long long align_up(unsigned long long value, unsigned long long alignment)
{
    return (value + alignment - 1ull) / alignment * alignment;
}

/* ------------------------------------------------- bounded primitive ---- */

int yvex_rocm_op_attention(yvex_backend *backend, const yvex_device_tensor *query,
                           const yvex_device_tensor *keys, const yvex_device_tensor *values,
                           unsigned long long seq_len, unsigned long long position, float scale,
                           int causal, yvex_device_tensor *score_scratch,
                           yvex_device_tensor *probability_scratch, yvex_device_tensor *out,
                           yvex_error *err)
{
    static const char where[] = "yvex_backend_op_attention";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_backend_operation_variant variant = causal
                                                 ? YVEX_BACKEND_VARIANT_ATTENTION_CAUSAL_F32
                                                 : YVEX_BACKEND_VARIANT_ATTENTION_NONCAUSAL_F32;
    yvex_rocm_attention_f32_params params;
    unsigned long long head_dim = 0ull, kv_elements = 0ull;
    int rc;
    if (!isfinite(scale) || scale <= 0.0f)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "scale must be finite and positive");
    rc = yvex_backend_validate_attention(backend, query, keys, values, seq_len, position,
                                         score_scratch, probability_scratch, out, &head_dim,
                                         &kv_elements, where, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_tensor_backed(query) || !yvex_rocm_tensor_backed(keys) ||
        !yvex_rocm_tensor_backed(values) || !yvex_rocm_tensor_backed(score_scratch) ||
        !yvex_rocm_tensor_backed(probability_scratch) || !yvex_rocm_tensor_backed(out))
        return refuse(err, YVEX_ERR_STATE, where,
                      "a tensor over a reserved address range reaches pages that are not committed");
    rc = yvex_rocm_require_capability(backend, variant, where, err);
    if (rc != YVEX_OK) return rc;
    memset(&params, 0, sizeof(params));
    params.q = (const float *)query->data;
    params.k = (const float *)keys->data;
    params.v = (const float *)values->data;
    params.score = (float *)score_scratch->data;
    params.prob = (float *)probability_scratch->data;
    params.out = (float *)out->data;
    params.status = state->device_status;
    params.seq_len = seq_len;
    params.position = position;
    params.head_dim = head_dim;
    params.scale = scale;
    params.causal = causal ? 1 : 0;
    rc = yvex_rocm_launch(backend, YVEX_ROCM_FN_ATTENTION_F32, variant, 1u, 1u, 1u, 256u, 0u,
                          &params, where, err);
    if (rc == YVEX_OK) rc = yvex_rocm_complete(backend, variant, where, NULL, err);
    if (rc != YVEX_OK) return rc;
    score_scratch->is_written = 1;
    probability_scratch->is_written = 1;
    out->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ------------------------------------------------ split-K decode core ---- */

/* Wave count and workspace of the balanced split-K decode are pure functions of the
 * request geometry (never of the device) so the planner's workspace_required and the
 * execution always agree: 2048 waves = 2 per SIMD of a 256-CU part, fewer when the
 * worst-case work cannot give each wave ROCM_DECODE_MIN_TILES tiles. */
static unsigned int decode_wave_count(unsigned long long sessions, unsigned long long kv_heads,
                                      unsigned long long max_context)
{
    unsigned long long tiles = sessions * kv_heads *
                               ((max_context + ROCM_PAGE_TOKENS - 1ull) / ROCM_PAGE_TOKENS);
    unsigned long long waves = (tiles + ROCM_DECODE_MIN_TILES - 1ull) / ROCM_DECODE_MIN_TILES;
    if (waves > ROCM_DECODE_WAVES) waves = ROCM_DECODE_WAVES;
    return (unsigned int)(waves ? waves : 1ull);
}

static int decode_workspace_bytes(unsigned long long slots, unsigned long long heads,
                                  unsigned long long head_dim, unsigned long long element_bytes,
                                  unsigned long long *acc_bytes, unsigned long long *total)
{
    unsigned long long rows, acc, ml;
    if (!yvex_core_u64_mul(slots, heads, &rows) ||
        !yvex_core_u64_mul(rows, head_dim * element_bytes, &acc) ||
        !yvex_core_u64_mul(rows, 2ull * sizeof(float), &ml))
        return 0;
    acc = align_up(acc, ROCM_WORK_ALIGNMENT);
    ml = align_up(ml, ROCM_WORK_ALIGNMENT);
    if (!yvex_core_u64_add(acc, ml, total)) return 0;
    *acc_bytes = acc;
    return 1;
}

/* A launch that fills the device merges its split segments with a second kernel; a smaller
 * one is bound by launch latency and merges inside the decode kernel (arrival counters). */
static int decode_merges_in_kernel(unsigned int waves) { return waves < ROCM_DECODE_WAVES; }

/* Waves of a team: eight, two per SIMD; four at head dimension 256, whose tiles and
 * accumulators take twice the registers. */
static unsigned int decode_team_waves(unsigned long long head_dim)
{
    return head_dim > ROCM_MFMA_HEAD_DIM ? ROCM_TEAM_WAVES / 2u : ROCM_TEAM_WAVES;
}

/* Teams per (session, kv head) of the token-major decode, 0 when that form does not apply
 * (paged pools, wide groups).  A pure function of the request geometry. */
static unsigned int decode_team_count(int paged, unsigned long long group, unsigned long long head_dim,
                                      unsigned long long max_context)
{
    const unsigned long long tiles = (max_context + ROCM_PAGE_TOKENS - 1ull) / ROCM_PAGE_TOKENS;
    const unsigned long long per_team = (unsigned long long)decode_team_waves(head_dim) *
                                        (head_dim > ROCM_MFMA_HEAD_DIM ? ROCM_TEAM_TILES_WIDE : ROCM_TEAM_TILES);
    unsigned long long teams = (tiles + per_team - 1ull) / per_team;
    if (paged || group > ROCM_TEAM_GROUP_MAX) return 0u;
    if (teams > ROCM_TEAMS_MAX) teams = ROCM_TEAMS_MAX;
    return (unsigned int)(teams ? teams : 1ull);
}

/* A single query token over a token-major bf16 history takes the split decode kernels at
 * head dimension 128, and the team form of them at 64 and 256 (groups of at most eight query
 * heads); other single tokens run as a one-row tile of the prefill kernel. */
static int decode_rows_geometry(const yvex_transformer_attention_requirement *r)
{
    return r->query_tokens == 1ull &&
           (r->head_dimension == ROCM_MFMA_HEAD_DIM ||
            r->query_heads / r->key_value_heads <= ROCM_TEAM_GROUP_MAX);
}

/* Balanced decode: two partial slots per wave, then (two-kernel form) the per-session offset
 * table. */
static int balanced_workspace_bytes(unsigned long long waves, unsigned long long group,
                                    unsigned long long head_dim, unsigned long long sessions,
                                    unsigned long long *acc_bytes, unsigned long long *ml_bytes,
                                    unsigned long long *total)
{
    unsigned long long parts = 0ull, offsets;
    if (!decode_workspace_bytes(2ull * waves, group, head_dim, sizeof(float), acc_bytes, &parts)) return 0;
    offsets = decode_merges_in_kernel((unsigned int)waves)
                  ? 0ull : align_up((sessions + 1ull) * sizeof(uint32_t), ROCM_WORK_ALIGNMENT);
    *ml_bytes = parts - *acc_bytes;
    return yvex_core_u64_add(parts, offsets, total);
}

typedef struct {
    yvex_rocm_function_id function, merged_function; /* two-launch form, one-launch form */
    yvex_backend_operation_variant variant;
    const void *q, *k, *v;
    const int32_t *page_table, *context;
    void *out, *lse;
    const void *gate;
    unsigned long long sessions, query_heads, kv_heads, head_dim;
    unsigned long long pool_pages, table_stride, max_context, fixed_context;
    unsigned int page_shift; /* paged pools: a page is 16 << page_shift tokens */
    unsigned long long k_token_stride, v_token_stride;
    float scale;
    /* when set, the partials live here (nothing is acquired or released) */
    void *fixed_work;
    unsigned long long fixed_work_bytes;
    int two_launches; /* the function has no build that merges in the kernel */
} decode_job;

/* Launches the decode kernel, the finish (merge) kernel when the launch fills the device, and
 * completes the operation. */
static int decode_run(yvex_backend *backend, const decode_job *job, const char *where,
                      yvex_backend_operation_facts *facts, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_decode_params dp;
    unsigned long long acc_bytes = 0ull, ml_bytes = 0ull, total = 0ull, items;
    const unsigned long long group = job->query_heads / job->kv_heads;
    const unsigned int waves = decode_wave_count(job->sessions, job->kv_heads, job->max_context);
    const unsigned int teams = decode_team_count(job->page_table != NULL, group, job->head_dim,
                                                 job->max_context);
    const int in_kernel = !job->two_launches && (teams || decode_merges_in_kernel(waves));
    void *work = NULL;
    yvex_error cleanup;
    int owned = 0, rc, cleanup_rc;
    if (!yvex_core_u64_mul(job->sessions * job->kv_heads,
                           (job->max_context + ROCM_PAGE_TOKENS - 1ull) / ROCM_PAGE_TOKENS, &items) ||
        items > 0x7fffffffull || job->sessions > 65535ull || job->query_heads > 65535ull ||
        (in_kernel && job->sessions * job->kv_heads > YVEX_ROCM_DECODE_SEGMENTS_MAX) ||
        !(teams ? decode_workspace_bytes(job->sessions * job->kv_heads * teams, group, job->head_dim,
                                         sizeof(float), &acc_bytes, &total)
                : balanced_workspace_bytes(waves, group, job->head_dim, job->sessions, &acc_bytes,
                                           &ml_bytes, &total)))
        return refuse(err, YVEX_ERR_BOUNDS, where, "decode geometry exceeds admitted integer range");
    backend_workspace_reset(backend);
    if (job->fixed_work) {
        if (total > job->fixed_work_bytes)
            return refuse(err, YVEX_ERR_BOUNDS, where,
                          "decode partials exceed the fixed device scratch "
                          "(YVEX_ROCM_STATIC_WORKSPACE_BYTES)");
        work = job->fixed_work;
    } else {
        rc = yvex_rocm_temporary_acquire(backend, total, &work, &owned, where, err);
        if (rc != YVEX_OK) return rc;
    }
    memset(&dp, 0, sizeof(dp));
    dp.q = (const uint16_t *)job->q;
    dp.k_pool = job->k;
    dp.v_pool = job->v;
    dp.page_table = job->page_table;
    dp.context = job->context;
    dp.out = (uint16_t *)job->out;
    dp.lse = (float *)job->lse;
    dp.gate = (const uint16_t *)job->gate;
    dp.part_acc = (float *)work;
    dp.part_ml = (float *)((unsigned char *)work + acc_bytes);
    dp.arrivals = in_kernel ? state->decode_arrivals : NULL;
    dp.offsets = in_kernel ? NULL : (uint32_t *)((unsigned char *)work + acc_bytes + ml_bytes);
    dp.status = state->device_status;
    dp.k_token_stride = job->k_token_stride;
    dp.v_token_stride = job->v_token_stride;
    dp.sessions = (uint32_t)job->sessions;
    dp.query_heads = (uint32_t)job->query_heads;
    dp.kv_heads = (uint32_t)job->kv_heads;
    dp.head_dim = (uint32_t)job->head_dim;
    dp.pool_pages = (uint32_t)job->pool_pages;
    dp.page_shift = job->page_shift;
    dp.table_stride = (uint32_t)job->table_stride;
    dp.min_tiles = ROCM_DECODE_MIN_TILES;
    dp.fixed_context = (uint32_t)job->fixed_context;
    dp.waves = waves;
    dp.scale_log2 = job->scale * 1.4426950408889634f;
    if (teams) /* teams of waves, merged through LDS and then between the teams */
        rc = yvex_rocm_launch(backend,
                              job->head_dim == 64ull    ? YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM_64
                              : job->head_dim == 256ull ? YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM_256
                                                        : YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM,
                              job->variant, teams, (unsigned int)job->kv_heads, (unsigned int)job->sessions,
                              64u * decode_team_waves(job->head_dim), 0u, &dp, where, err);
    else
        rc = yvex_rocm_launch(backend, in_kernel ? job->merged_function : job->function, job->variant,
                              waves, 1u, 1u, 64u, 0u, &dp, where, err);
    if (rc == YVEX_OK && !in_kernel)
        rc = yvex_rocm_launch(backend,
                              job->head_dim > 128ull ? YVEX_ROCM_FN_DECODE_FINISH_256
                                                     : YVEX_ROCM_FN_DECODE_FINISH,
                              job->variant, (unsigned int)job->query_heads, (unsigned int)job->sessions, 1u,
                              (unsigned int)job->head_dim, 0u, &dp, where, err);
    if (rc == YVEX_OK) {
        facts->kernel_launches = in_kernel ? 1ull : 2ull;
        facts->accelerated_matrix_launches = 1ull;
        facts->temporary_bytes = total;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, job->variant, where, facts, err);
    }
    /* a launch that did not run to a clean end may leave arrival counts behind */
    if (rc != YVEX_OK && in_kernel && !state->recording &&
        backend->status != YVEX_BACKEND_STATUS_FAILED)
        (void)state->driver.hipMemsetAsync(state->decode_arrivals, 0,
                                           YVEX_ROCM_DECODE_SEGMENTS_MAX * sizeof(uint32_t),
                                           yvex_rocm_stream(state));
    yvex_error_clear(&cleanup);
    cleanup_rc = yvex_rocm_temporary_release(backend, work, total, owned, &cleanup);
    backend_workspace_reset(backend);
    if (rc == YVEX_OK && cleanup_rc != YVEX_OK) {
        rc = cleanup_rc;
        if (err) *err = cleanup;
    }
    return rc;
}

/* ------------------------------------------- multi-token GQA contract ---- */

static int attention_validate(const yvex_transformer_attention_requirement *r, const char *stage,
                              yvex_error *err)
{
    unsigned long long query_end, query_width, kv_width;
    if (!r || !r->query_tokens || !r->key_value_tokens ||
        !yvex_core_u64_add(r->query_start, r->query_tokens, &query_end) ||
        query_end > r->key_value_tokens || !r->query_heads || !r->key_value_heads ||
        r->query_heads % r->key_value_heads || !r->head_dimension ||
        !yvex_core_u64_mul(r->query_heads, r->head_dimension, &query_width) ||
        !yvex_core_u64_mul(r->key_value_heads, r->head_dimension, &kv_width) ||
        (r->query_token_stride && r->query_token_stride < query_width) ||
        (r->key_token_stride && r->key_token_stride < kv_width) ||
        (r->value_token_stride && r->value_token_stride < kv_width))
        return refuse(err, YVEX_ERR_INVALID_ARG, stage,
                      "complete exact-attention geometry is required");
    if (r->layout != YVEX_TRANSFORMER_ATTENTION_LAYOUT_TOKEN_HEAD_DIM ||
        r->mask < YVEX_TRANSFORMER_ATTENTION_MASK_FULL ||
        r->mask > YVEX_TRANSFORMER_ATTENTION_MASK_CAUSAL || !r->deterministic)
        return refuse(err, YVEX_ERR_UNSUPPORTED, stage,
                      "ROCm requires deterministic token/head/dimension attention");
    if (r->numeric_contract == YVEX_TRANSFORMER_ATTENTION_NUMERIC_EXACT_F32) {
        if (r->head_dimension > ROCM_EXACT_HEAD_MAX || r->query_dtype != YVEX_DTYPE_F32 ||
            r->key_dtype != YVEX_DTYPE_F32 || r->value_dtype != YVEX_DTYPE_F32 ||
            r->output_dtype != YVEX_DTYPE_F32)
            return refuse(err, YVEX_ERR_UNSUPPORTED, stage,
                          "ROCm requires deterministic token/head/dimension exact F32 attention");
    } else if (r->numeric_contract == YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE) {
        if ((r->head_dimension != 64ull && r->head_dimension != ROCM_MFMA_HEAD_DIM &&
             r->head_dimension != 256ull) ||
            r->query_dtype != YVEX_DTYPE_BF16 ||
            r->key_dtype != YVEX_DTYPE_BF16 || r->value_dtype != YVEX_DTYPE_BF16 ||
            r->output_dtype != YVEX_DTYPE_BF16 ||
            r->query_heads / r->key_value_heads > ROCM_GROUP_MAX ||
            r->key_value_tokens > 0x7fffffffull || (r->query_token_stride % 8ull) ||
            (r->key_token_stride % 8ull) || (r->value_token_stride % 8ull))
            return refuse(err, YVEX_ERR_UNSUPPORTED, stage,
                          "ROCm bf16 attention requires BF16 tensors, head dimension 64, 128 or 256, "
                          "a query group of at most 16 and 16-byte aligned token strides");
    } else {
        return refuse(err, YVEX_ERR_UNSUPPORTED, stage,
                      "ROCm admits the exact F32 and the bf16/fp32-accumulate contracts only");
    }
    yvex_error_clear(err);
    return YVEX_OK;
}

static unsigned long long visible_tokens(const yvex_transformer_attention_requirement *r)
{
    return r->mask == YVEX_TRANSFORMER_ATTENTION_MASK_CAUSAL ? r->query_start + r->query_tokens
                                                             : r->key_value_tokens;
}

/* The EXACT_F32 request has three kernels; the choice is a function of the request geometry
 * (and of the 16-byte alignment of the views) only.
 *   - Prefill-shaped requests (at least 32 query tokens, head dimension 64, 128 or 256) run in
 *     32 x 32 tiles on the fp32 matrix cores with float statistics, the arithmetic of the
 *     reference's own device kernel (src/backend/cuda/transformer_kernels.cu:136-208).
 *   - Other requests over 512 or more keys (the decode step of the session layer,
 *     src/runtime/stateful_attention.c:326-352) are cut into runs of keys, one wave per
 *     (token, head, run) with double-precision statistics, eight runs per workgroup; the
 *     workgroups of a (token, head) merge in the kernel (arrival counters), one launch.
 *   - Everything else runs one wave per (token, head), double-precision statistics. */
enum { ROCM_EXACT_TILE_QUERIES = 128, ROCM_EXACT_TILE_MIN_TOKENS = 32, ROCM_EXACT_SPLIT_MIN_KEYS = 512,
       ROCM_EXACT_SPLIT_WAVES = 2048, ROCM_EXACT_SPLIT_RUN_MIN = 64, ROCM_EXACT_SPLIT_TEAM = 8 };

static int exact_strides_aligned(const yvex_transformer_attention_requirement *r)
{
    const unsigned long long q_stride = r->query_token_stride ? r->query_token_stride
                                                              : r->query_heads * r->head_dimension;
    const unsigned long long kv_width = r->key_value_heads * r->head_dimension;
    const unsigned long long k_stride = r->key_token_stride ? r->key_token_stride : kv_width;
    const unsigned long long v_stride = r->value_token_stride ? r->value_token_stride : kv_width;
    return ((q_stride | k_stride | v_stride) & 3ull) == 0ull;
}

static int exact_tile_geometry(const yvex_transformer_attention_requirement *r)
{
    return r->query_tokens >= ROCM_EXACT_TILE_MIN_TOKENS &&
           (r->head_dimension == 64ull || r->head_dimension == 128ull || r->head_dimension == 256ull) &&
           exact_strides_aligned(r);
}

/* Runs of the split form: 0 when the request does not take it.  keys_per_run is a multiple of
 * 64 (the kernel's step); there are about ROCM_EXACT_SPLIT_WAVES waves in all and no run is
 * shorter than ROCM_EXACT_SPLIT_RUN_MIN keys. */
static unsigned long long exact_split_runs(const yvex_transformer_attention_requirement *r,
                                           unsigned long long *keys_per_run)
{
    unsigned long long units, runs, per_run;
    *keys_per_run = 0ull;
    if (exact_tile_geometry(r) || r->key_value_tokens < ROCM_EXACT_SPLIT_MIN_KEYS ||
        (r->head_dimension & 7ull) || r->head_dimension > 256ull || !exact_strides_aligned(r) ||
        !yvex_core_u64_mul(r->query_tokens, r->query_heads, &units) ||
        units > YVEX_ROCM_DECODE_SEGMENTS_MAX /* one arrival counter per (token, head) */)
        return 0ull;
    runs = ROCM_EXACT_SPLIT_WAVES / units ? ROCM_EXACT_SPLIT_WAVES / units : 1ull;
    if (runs > r->key_value_tokens / ROCM_EXACT_SPLIT_RUN_MIN)
        runs = r->key_value_tokens / ROCM_EXACT_SPLIT_RUN_MIN;
    if (runs < 2ull) return 0ull;
    per_run = align_up((r->key_value_tokens + runs - 1ull) / runs, 64ull);
    runs = (r->key_value_tokens + per_run - 1ull) / per_run;
    if (runs < 2ull || runs > 65535ull) return 0ull;
    *keys_per_run = per_run;
    return runs;
}

static int exact_split_workspace(const yvex_transformer_attention_requirement *r,
                                 unsigned long long runs, unsigned long long *acc_bytes,
                                 unsigned long long *total)
{
    unsigned long long slots, acc, ml;
    /* one partial per team of ROCM_EXACT_SPLIT_TEAM runs */
    if (!yvex_core_u64_mul(r->query_tokens * r->query_heads,
                           (runs + ROCM_EXACT_SPLIT_TEAM - 1ull) / ROCM_EXACT_SPLIT_TEAM, &slots) ||
        !yvex_core_u64_mul(slots, r->head_dimension * sizeof(double), &acc) ||
        !yvex_core_u64_mul(slots, 2ull * sizeof(double), &ml))
        return 0;
    acc = align_up(acc, ROCM_WORK_ALIGNMENT);
    ml = align_up(ml, ROCM_WORK_ALIGNMENT);
    *acc_bytes = acc;
    return yvex_core_u64_add(acc, ml, total);
}

static int rocm_attention_workspace_required(const yvex_transformer_attention_requirement *r,
                                             unsigned long long *bytes, yvex_error *err)
{
    static const char where[] = "rocm.transformer.attention.workspace";
    unsigned long long acc = 0ull, ml = 0ull, total = 0ull;
    int rc;
    if (bytes) *bytes = 0ull;
    rc = attention_validate(r, where, err);
    if (rc != YVEX_OK) return rc;
    if (!bytes) return refuse(err, YVEX_ERR_INVALID_ARG, where, "workspace byte output is required");
    if (r->numeric_contract == YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE &&
        decode_rows_geometry(r)) {
        /* split-K decode partials; geometry must match decode_run */
        const unsigned int waves = decode_wave_count(1ull, r->key_value_heads, visible_tokens(r));
        const unsigned long long group = r->query_heads / r->key_value_heads;
        const unsigned int teams = decode_team_count(0, group, r->head_dimension, visible_tokens(r));
        if (!(teams ? decode_workspace_bytes(r->key_value_heads * teams, group, r->head_dimension,
                                             sizeof(float), &acc, &total)
                    : balanced_workspace_bytes(waves, group, r->head_dimension, 1ull, &acc, &ml, &total)))
            return refuse(err, YVEX_ERR_BOUNDS, where, "decode workspace geometry overflowed");
        *bytes = total;
    } else if (r->numeric_contract == YVEX_TRANSFORMER_ATTENTION_NUMERIC_EXACT_F32) {
        unsigned long long per_run;
        const unsigned long long runs = exact_split_runs(r, &per_run);
        if (runs) {
            if (!exact_split_workspace(r, runs, &acc, &total))
                return refuse(err, YVEX_ERR_BOUNDS, where, "attention workspace geometry overflowed");
            *bytes = total;
        }
    }
    yvex_error_clear(err);
    return YVEX_OK;
}

static int view_ok(const yvex_backend *backend, const yvex_device_tensor *tensor, yvex_dtype dtype,
                   unsigned long long elements, int require_written)
{
    unsigned long long bytes;
    if (!backend_tensor_owner_is(backend, tensor) || (require_written && !tensor->is_written) ||
        tensor->dtype != dtype || !tensor->data ||
        !yvex_core_u64_mul(elements, yvex_rocm_dtype_bytes(dtype), &bytes) ||
        tensor->bytes != bytes)
        return 0;
    if (!yvex_rocm_tensor_backed(tensor)) {
        yvex_rocm_state(backend)->unbacked_view = 1;
        return 0;
    }
    return 1;
}

/* The refusal after a view_ok that said no: a view over a reserved address range that
 * reaches pages nobody committed is a state error of the caller, anything else a
 * malformed request. */
static int view_refusal(const yvex_backend *backend, yvex_error *err, const char *where,
                        const char *reason)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    if (state && state->unbacked_view) {
        state->unbacked_view = 0;
        return refuse(err, YVEX_ERR_STATE, where,
                      "a tensor over a reserved address range reaches pages that are not committed");
    }
    return refuse(err, YVEX_ERR_FORMAT, where, reason);
}

static int exact_tile_function(const yvex_transformer_attention_requirement *r,
                               unsigned long long q_stride, unsigned long long k_stride,
                               unsigned long long v_stride,
                               const yvex_transformer_attention_request *request,
                               yvex_rocm_function_id *function)
{
    if (!exact_tile_geometry(r) || ((q_stride | k_stride | v_stride) & 3ull) ||
        (((uintptr_t)request->query->data | (uintptr_t)request->key->data |
          (uintptr_t)request->value->data | (uintptr_t)request->output->data) & 15u))
        return 0;
    *function = r->head_dimension == 64ull    ? YVEX_ROCM_FN_GQA_F32_TILE_64
                : r->head_dimension == 128ull ? YVEX_ROCM_FN_GQA_F32_TILE_128
                                              : YVEX_ROCM_FN_GQA_F32_TILE_256;
    return 1;
}

/* What attention_execute_common has worked out of a request before it picks a kernel. */
typedef struct attention_geometry {
    unsigned long long q_stride, k_stride, v_stride; /* elements between tokens */
    unsigned long long rows;                         /* query tokens x query heads */
    int causal;
} attention_geometry;

/* The EXACT_F32 contract: the tile kernel on the fp32 matrix cores for prefill-shaped requests,
 * runs of keys for single rows over long histories, the row kernel for the rest. */
static int attention_execute_exact(yvex_backend *backend, const yvex_transformer_attention_request *request,
                                   yvex_device_tensor *lse, const attention_geometry *g,
                                   yvex_backend_operation_facts *facts, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const yvex_transformer_attention_requirement *r = &request->requirement;
    int rc;
    yvex_rocm_gqa_f32_params params;
    yvex_rocm_function_id tile_function = YVEX_ROCM_FN_GQA_F32;
    unsigned long long split_runs = 0ull, split_keys = 0ull, split_bytes = 0ull;
    void *split_work = NULL;
    int tiled = 0, split_owned = 0;
    memset(&params, 0, sizeof(params));
    params.q = (const float *)request->query->data;
    params.k = (const float *)request->key->data;
    params.v = (const float *)request->value->data;
    params.out = (float *)request->output->data;
    params.lse = lse ? (float *)lse->data : NULL;
    params.status = state->device_status;
    params.query_tokens = r->query_tokens;
    params.kv_tokens = r->key_value_tokens;
    params.query_start = r->query_start;
    params.query_heads = r->query_heads;
    params.kv_heads = r->key_value_heads;
    params.head_dim = r->head_dimension;
    params.q_stride = g->q_stride;
    params.k_stride = g->k_stride;
    params.v_stride = g->v_stride;
    params.scale = 1.0f / sqrtf((float)r->head_dimension);
    params.causal = g->causal;
    backend_workspace_reset(backend);
    if (exact_tile_function(r, g->q_stride, g->k_stride, g->v_stride, request, &tile_function)) {
        /* 128 query tokens of one head per workgroup, on the fp32 matrix cores */
        const unsigned long long groups =
            r->query_heads * ((r->query_tokens + ROCM_EXACT_TILE_QUERIES - 1ull) / ROCM_EXACT_TILE_QUERIES);
        if (groups > 0x7fffffffull)
            return refuse(err, YVEX_ERR_BOUNDS, "rocm.transformer.gqa",
                          "attention geometry exceeds the launch range");
        /* two workgroups per unit at head dimension 64 and 128 (registers and LDS), one (of eight
         * waves) at 256 */
        const unsigned int per_unit = r->head_dimension == 256ull ? 1u : 2u;
        unsigned int workgroups = 0u;
        if (g->causal) {
            /* a geometry that repeats gets item lists with equal work per unit; until then,
             * and when no lists can be made, the pairs of workgroups of a unit at least sum
             * to the same */
            yvex_rocm_schedule_key key;
            memset(&key, 0, sizeof(key));
            key.query_tokens = r->query_tokens;
            key.kv_tokens = r->key_value_tokens;
            key.query_start = r->query_start;
            key.query_heads = (uint32_t)r->query_heads;
            key.item_rows = (uint32_t)ROCM_EXACT_TILE_QUERIES;
            key.step_keys = 32u;
            key.per_unit = per_unit;
            key.kind = (uint32_t)tile_function;
            if (r->query_heads <= 0xffffull)
                workgroups = yvex_rocm_schedule_lists(backend, &key, &params.lists);
            if (!workgroups && per_unit == 2u && state->compute_units > 0 &&
                groups >= 2ull * (unsigned long long)state->compute_units)
                params.pair_units = (uint32_t)state->compute_units;
        }
        rc = yvex_rocm_launch(backend, tile_function, YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
                              workgroups ? workgroups : (unsigned int)groups, 1u, 1u,
                              /* at 256 pairs of waves split the head dimension: eight waves */
                              r->head_dimension == 256ull ? 512u : 256u, 0u,
                              &params, "rocm.transformer.gqa", err);
        tiled = 1;
    } else if ((split_runs = exact_split_runs(r, &split_keys)) != 0ull &&
               !(((uintptr_t)request->query->data | (uintptr_t)request->key->data |
                  (uintptr_t)request->value->data) & 15u)) {
        /* runs of keys, one wave per (token, head, run), eight runs per workgroup */
        unsigned long long acc_bytes = 0ull;
        if (!exact_split_workspace(r, split_runs, &acc_bytes, &split_bytes))
            return refuse(err, YVEX_ERR_BOUNDS, "rocm.transformer.gqa",
                          "attention workspace geometry overflowed");
        rc = yvex_rocm_temporary_acquire(backend, split_bytes, &split_work, &split_owned,
                                         "rocm.transformer.gqa", err);
        if (rc != YVEX_OK) return rc;
        params.part_acc = (double *)split_work;
        params.part_ml = (double *)((unsigned char *)split_work + acc_bytes);
        params.splits = (uint32_t)split_runs;
        params.keys_per_split = (uint32_t)split_keys;
        params.arrivals = state->decode_arrivals;
        rc = yvex_rocm_launch(backend,
                              r->head_dimension > 128ull ? YVEX_ROCM_FN_GQA_F32_SPLIT_WIDE
                                                         : YVEX_ROCM_FN_GQA_F32_SPLIT,
                              YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, (unsigned int)g->rows,
                              (unsigned int)((split_runs + ROCM_EXACT_SPLIT_TEAM - 1ull) /
                                             ROCM_EXACT_SPLIT_TEAM),
                              1u, 64u * ROCM_EXACT_SPLIT_TEAM, 0u, &params, "rocm.transformer.gqa", err);
        /* a launch that did not run to a clean end may leave arrival counts behind */
        if (rc != YVEX_OK && !state->recording && backend->status != YVEX_BACKEND_STATUS_FAILED)
            (void)state->driver.hipMemsetAsync(state->decode_arrivals, 0,
                                               YVEX_ROCM_DECODE_SEGMENTS_MAX * sizeof(uint32_t),
                                               yvex_rocm_stream(state));
    } else {
        split_runs = 0ull;
        rc = yvex_rocm_launch(backend, YVEX_ROCM_FN_GQA_F32,
                              YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, (unsigned int)g->rows, 1u,
                              1u, 64u, 0u, &params, "rocm.transformer.gqa", err);
    }
    if (rc == YVEX_OK) {
        facts->kernel_launches = 1ull;
        facts->accelerated_matrix_launches = tiled ? 1ull : 0ull;
        facts->temporary_bytes = split_bytes;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
                                "rocm.transformer.gqa", facts, err);
    }
    if (split_work) {
        yvex_error cleanup;
        int cleanup_rc;
        yvex_error_clear(&cleanup);
        cleanup_rc = yvex_rocm_temporary_release(backend, split_work, split_bytes, split_owned, &cleanup);
        backend_workspace_reset(backend);
        if (rc == YVEX_OK && cleanup_rc != YVEX_OK) {
            rc = cleanup_rc;
            if (err) *err = cleanup;
        }
    }
    return rc;
}

/* The BF16 contract over more than one query row (or a geometry the decode teams do not take):
 * the MFMA prefill kernel, 128 query rows of one head per workgroup. */
static int attention_execute_prefill(yvex_backend *backend, const yvex_transformer_attention_request *request,
                                     yvex_device_tensor *lse, const yvex_device_tensor *gate,
                                     const attention_geometry *g, yvex_backend_operation_facts *facts,
                                     yvex_error *err)
{
    static const char where[] = "rocm.transformer.attention";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const yvex_transformer_attention_requirement *r = &request->requirement;
    int rc;
    yvex_rocm_prefill_params params;
    const unsigned long long q_tiles = (r->query_tokens + ROCM_PREFILL_ROWS - 1ull) /
                                       ROCM_PREFILL_ROWS;
    memset(&params, 0, sizeof(params));
    params.q = (const uint16_t *)request->query->data;
    params.k = (const uint16_t *)request->key->data;
    params.v = (const uint16_t *)request->value->data;
    params.out = (uint16_t *)request->output->data;
    params.lse = lse ? (float *)lse->data : NULL;
    params.gate = gate ? (const uint16_t *)gate->data : NULL;
    params.status = state->device_status;
    params.q_stride = g->q_stride;
    params.k_stride = g->k_stride;
    params.v_stride = g->v_stride;
    params.query_tokens = (uint32_t)r->query_tokens;
    params.kv_tokens = (uint32_t)r->key_value_tokens;
    params.query_start = (uint32_t)r->query_start;
    params.query_heads = (uint32_t)r->query_heads;
    params.kv_heads = (uint32_t)r->key_value_heads;
    params.head_dim = (uint32_t)r->head_dimension;
    params.causal = (uint32_t)g->causal;
    params.scale_log2 = (1.0f / sqrtf((float)r->head_dimension)) * 1.4426950408889634f;
    backend_workspace_reset(backend);
    /* the kernel addresses K and V through 32-bit buffer offsets */
    if (r->query_heads > 65535ull || q_tiles > 65535ull ||
        r->query_heads * q_tiles > 0x7fffffffull ||
        r->key_value_tokens * g->k_stride * 2ull >= 0xffffffffull ||
        r->key_value_tokens * g->v_stride * 2ull >= 0xffffffffull)
        return refuse(err, YVEX_ERR_BOUNDS, where,
                      "prefill geometry exceeds admitted launch range");
    rc = yvex_rocm_launch(backend,
                          r->head_dimension == 64ull    ? YVEX_ROCM_FN_PREFILL_BF16_64
                          : r->head_dimension == 256ull ? YVEX_ROCM_FN_PREFILL_BF16_256
                                                        : YVEX_ROCM_FN_PREFILL_BF16,
                          YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
                          (unsigned int)(r->query_heads * q_tiles), 1u, 1u, 256u, 0u,
                          &params, "rocm.transformer.gqa.prefill", err);
    if (rc == YVEX_OK) {
        facts->kernel_launches = 1ull;
        facts->accelerated_matrix_launches = 1ull;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
                                "rocm.transformer.gqa.prefill", facts, err);
    }
    return rc;
}

static int attention_execute_common(yvex_backend *backend,
                                    const yvex_transformer_attention_request *request,
                                    yvex_device_tensor *lse, const yvex_device_tensor *gate,
                                    yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.transformer.attention";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const yvex_transformer_attention_requirement *r;
    unsigned long long q_width, kv_width, q_stride, k_stride, v_stride;
    unsigned long long q_elements, k_elements, v_elements, o_elements, rows;
    attention_geometry geometry;
    int exact, rc, causal;
    if (!request || !request->query || !request->key || !request->value || !request->output ||
        !facts)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "complete exact-attention tensors and result facts are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    r = &request->requirement;
    rc = attention_validate(r, where, err);
    if (rc != YVEX_OK) return rc;
    memset(facts, 0, sizeof(*facts));
    exact = r->numeric_contract == YVEX_TRANSFORMER_ATTENTION_NUMERIC_EXACT_F32;
    causal = r->mask == YVEX_TRANSFORMER_ATTENTION_MASK_CAUSAL;
    if (gate && exact)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "the fused output gate requires the BF16 numeric contract");
    q_width = r->query_heads * r->head_dimension;
    kv_width = r->key_value_heads * r->head_dimension;
    q_stride = r->query_token_stride ? r->query_token_stride : q_width;
    k_stride = r->key_token_stride ? r->key_token_stride : kv_width;
    v_stride = r->value_token_stride ? r->value_token_stride : kv_width;
    /* src/backend/cuda/transformer.c:746-770: every view is exactly as large as its
     * strides imply, inputs are written, everything belongs to this backend */
    if (!state || !yvex_core_u64_mul(r->query_tokens, r->query_heads, &rows) ||
        rows > 0xffffffffull ||
        !yvex_core_u64_mul(r->query_tokens - 1ull, q_stride, &q_elements) ||
        !yvex_core_u64_add(q_elements, q_width, &q_elements) ||
        !yvex_core_u64_mul(r->query_tokens, q_width, &o_elements) ||
        !yvex_core_u64_mul(r->key_value_tokens - 1ull, k_stride, &k_elements) ||
        !yvex_core_u64_add(k_elements, kv_width, &k_elements) ||
        !yvex_core_u64_mul(r->key_value_tokens - 1ull, v_stride, &v_elements) ||
        !yvex_core_u64_add(v_elements, kv_width, &v_elements) ||
        !view_ok(backend, request->query, r->query_dtype, q_elements, 1) ||
        !view_ok(backend, request->key, r->key_dtype, k_elements, 1) ||
        !view_ok(backend, request->value, r->value_dtype, v_elements, 1) ||
        !view_ok(backend, request->output, r->output_dtype, o_elements, 0) ||
        (lse && !view_ok(backend, lse, YVEX_DTYPE_F32, rows, 0)) ||
        (gate && (!view_ok(backend, gate, YVEX_DTYPE_BF16, o_elements, 1) ||
                  gate->data == request->output->data)))
        return view_refusal(backend, err, "rocm.transformer.gqa",
                      "bounded Q/K/V views matching the declared token strides are required");
    geometry.q_stride = q_stride;
    geometry.k_stride = k_stride;
    geometry.v_stride = v_stride;
    geometry.rows = rows;
    geometry.causal = causal;
    if (exact) {
        rc = attention_execute_exact(backend, request, lse, &geometry, facts, err);
    } else if (decode_rows_geometry(r)) {
        decode_job job;
        memset(&job, 0, sizeof(job));
        job.function = YVEX_ROCM_FN_DECODE_ROWS_BF16;
        job.merged_function = YVEX_ROCM_FN_DECODE_ROWS_BF16_MERGED;
        job.variant = YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16;
        job.q = request->query->data;
        job.k = request->key->data;
        job.v = request->value->data;
        job.out = request->output->data;
        job.lse = lse ? lse->data : NULL;
        job.gate = gate ? gate->data : NULL;
        job.sessions = 1ull;
        job.query_heads = r->query_heads;
        job.kv_heads = r->key_value_heads;
        job.head_dim = r->head_dimension;
        job.max_context = job.fixed_context = visible_tokens(r);
        job.k_token_stride = k_stride;
        job.v_token_stride = v_stride;
        job.scale = 1.0f / sqrtf((float)r->head_dimension);
        rc = decode_run(backend, &job, "rocm.transformer.gqa.decode", facts, err);
    } else {
        rc = attention_execute_prefill(backend, request, lse, gate, &geometry, facts, err);
    }
    if (rc != YVEX_OK) return rc;
    request->output->is_written = 1;
    if (lse) lse->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_attention_execute(yvex_backend *backend,
                                  const yvex_transformer_attention_request *request,
                                  yvex_backend_operation_facts *facts, yvex_error *err)
{
    return attention_execute_common(backend, request, NULL, NULL, facts, err);
}

static int rocm_attention_execute_lse(yvex_backend *backend,
                                      const yvex_transformer_attention_request *request,
                                      yvex_device_tensor *lse, yvex_backend_operation_facts *facts,
                                      yvex_error *err)
{
    if (!lse)
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.transformer.attention",
                      "an LSE output tensor is required");
    return attention_execute_common(backend, request, lse, NULL, facts, err);
}

static int rocm_attention_execute_fused(yvex_backend *backend,
                                        const yvex_transformer_attention_request *request,
                                        const yvex_rocm_attention_epilogue *epilogue,
                                        yvex_device_tensor *lse,
                                        yvex_backend_operation_facts *facts, yvex_error *err)
{
    if (!epilogue || !epilogue->output_gate)
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.transformer.attention",
                      "an epilogue with an output gate tensor is required");
    return attention_execute_common(backend, request, lse, epilogue->output_gate, facts, err);
}

/* ------------------------------------------------------- paged decode ---- */

static int paged_validate(const yvex_rocm_paged_decode_requirement *r, const char *where,
                          yvex_error *err)
{
    unsigned long long capacity;
    if (!r || !r->sessions || !r->query_heads || !r->key_value_heads ||
        r->query_heads % r->key_value_heads || !r->head_dimension || !r->page_tokens ||
        !r->pool_pages || !r->page_table_stride || !r->max_context_tokens ||
        !yvex_core_u64_mul(r->page_table_stride, r->page_tokens, &capacity) ||
        r->max_context_tokens > capacity)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "complete paged-decode geometry is required");
    /* bf16 pages at head dimension 64, 128 or 256; Q8_0 pages at 128 */
    if ((r->head_dimension != ROCM_MFMA_HEAD_DIM &&
         !(r->kv_storage == YVEX_ROCM_KV_BF16 &&
           (r->head_dimension == 64ull || r->head_dimension == 256ull))) ||
        (r->page_tokens != ROCM_PAGE_TOKENS && r->page_tokens != 4ull * ROCM_PAGE_TOKENS) ||
        r->query_heads / r->key_value_heads > ROCM_GROUP_MAX ||
        (r->kv_storage != YVEX_ROCM_KV_BF16 && r->kv_storage != YVEX_ROCM_KV_Q8_0) ||
        r->numeric_contract != YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE ||
        !r->deterministic || r->pool_pages > 0x7fffffffull || capacity > 0x7fffffffull)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm paged decode requires head dimension 128 (bf16 pages: 64, 128 or 256), pages "
                      "of 16 or 64 tokens, a query group of at most 16 and the deterministic "
                      "bf16/fp32-accumulate contract");
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_paged_decode_workspace_required(const yvex_rocm_paged_decode_requirement *r,
                                                unsigned long long *bytes, yvex_error *err)
{
    static const char where[] = "rocm.attention.paged.workspace";
    unsigned long long acc = 0ull, ml = 0ull, total = 0ull;
    unsigned int waves;
    int rc;
    if (bytes) *bytes = 0ull;
    rc = paged_validate(r, where, err);
    if (rc != YVEX_OK) return rc;
    if (!bytes) return refuse(err, YVEX_ERR_INVALID_ARG, where, "workspace byte output is required");
    waves = decode_wave_count(r->sessions, r->key_value_heads, r->max_context_tokens);
    if (!balanced_workspace_bytes(waves, r->query_heads / r->key_value_heads, r->head_dimension,
                                  r->sessions, &acc, &ml, &total))
        return refuse(err, YVEX_ERR_BOUNDS, where, "decode workspace geometry overflowed");
    *bytes = total;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int paged_decode_execute_common(yvex_backend *backend,
                                       const yvex_rocm_paged_decode_request *request,
                                       const yvex_device_tensor *gate, void *fixed_work,
                                       unsigned long long fixed_work_bytes,
                                       yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.attention.paged";
    const yvex_rocm_paged_decode_requirement *r;
    unsigned long long q_elements, pool_bytes, block_bytes, table_elements;
    yvex_dtype pool_dtype;
    decode_job job;
    int rc;
    if (!request || !request->query || !request->key_pages || !request->value_pages ||
        !request->page_table || !request->context_tokens || !request->output || !facts)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "complete paged-decode tensors and result facts are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    r = &request->requirement;
    rc = paged_validate(r, where, err);
    if (rc != YVEX_OK) return rc;
    memset(facts, 0, sizeof(*facts));
    pool_dtype = r->kv_storage == YVEX_ROCM_KV_BF16 ? YVEX_DTYPE_BF16 : YVEX_DTYPE_I8;
    block_bytes = yvex_rocm_kv_page_block_bytes(r->kv_storage, r->head_dimension, r->page_tokens);
    q_elements = r->sessions * r->query_heads * r->head_dimension;
    table_elements = r->sessions * r->page_table_stride;
    if (!yvex_core_u64_mul(r->pool_pages * r->key_value_heads, block_bytes, &pool_bytes) ||
        !view_ok(backend, request->query, YVEX_DTYPE_BF16, q_elements, 1) ||
        !view_ok(backend, request->key_pages, pool_dtype,
                 pool_bytes / yvex_rocm_dtype_bytes(pool_dtype), 1) ||
        !view_ok(backend, request->value_pages, pool_dtype,
                 pool_bytes / yvex_rocm_dtype_bytes(pool_dtype), 1) ||
        !view_ok(backend, request->page_table, YVEX_DTYPE_I32, table_elements, 1) ||
        !view_ok(backend, request->context_tokens, YVEX_DTYPE_I32, r->sessions, 1) ||
        !view_ok(backend, request->output, YVEX_DTYPE_BF16, q_elements, 0) ||
        (request->lse &&
         !view_ok(backend, request->lse, YVEX_DTYPE_F32, r->sessions * r->query_heads, 0)) ||
        (gate && (!view_ok(backend, gate, YVEX_DTYPE_BF16, q_elements, 1) ||
                  gate->data == request->output->data)))
        return view_refusal(backend, err, where,
                      "query, page pools, page table, context lengths and outputs must be written "
                      "tensors of this backend with the declared geometry");
    memset(&job, 0, sizeof(job));
    if (r->kv_storage == YVEX_ROCM_KV_BF16 && r->head_dimension != ROCM_MFMA_HEAD_DIM) {
        /* the other head dimensions have the two-launch form only */
        job.function = r->head_dimension == 64ull ? YVEX_ROCM_FN_DECODE_PAGED_BF16_64
                                                  : YVEX_ROCM_FN_DECODE_PAGED_BF16_256;
        job.two_launches = 1;
        job.variant = YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16;
    } else if (r->kv_storage == YVEX_ROCM_KV_BF16) {
        job.function = YVEX_ROCM_FN_DECODE_PAGED_BF16;
        job.merged_function = YVEX_ROCM_FN_DECODE_PAGED_BF16_MERGED;
        job.variant = YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16;
    } else {
        job.function = YVEX_ROCM_FN_DECODE_PAGED_Q8_0;
        job.merged_function = YVEX_ROCM_FN_DECODE_PAGED_Q8_0_MERGED;
        job.variant = YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0;
    }
    job.q = request->query->data;
    job.k = request->key_pages->data;
    job.v = request->value_pages->data;
    job.page_table = (const int32_t *)request->page_table->data;
    job.context = (const int32_t *)request->context_tokens->data;
    job.out = request->output->data;
    job.lse = request->lse ? request->lse->data : NULL;
    job.gate = gate ? gate->data : NULL;
    job.sessions = r->sessions;
    job.query_heads = r->query_heads;
    job.kv_heads = r->key_value_heads;
    job.head_dim = r->head_dimension;
    job.pool_pages = r->pool_pages;
    job.page_shift = r->page_tokens == ROCM_PAGE_TOKENS ? 0u : 2u;
    job.table_stride = r->page_table_stride;
    job.max_context = r->max_context_tokens;
    job.scale = 1.0f / sqrtf((float)r->head_dimension);
    job.fixed_work = fixed_work;
    job.fixed_work_bytes = fixed_work_bytes;
    rc = decode_run(backend, &job, where, facts, err);
    if (rc != YVEX_OK) return rc;
    request->output->is_written = 1;
    if (request->lse) request->lse->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_paged_decode_execute(yvex_backend *backend,
                                     const yvex_rocm_paged_decode_request *request,
                                     yvex_backend_operation_facts *facts, yvex_error *err)
{
    return paged_decode_execute_common(backend, request, NULL, NULL, 0ull, facts, err);
}

/* paged_decode_execute for callers that cannot allocate: the split-K partials go to the
 * fixed device array of rocm_scratch.hip, whose address was taken when the backend was
 * opened.  No allocation or release call is made on this path, whether or not a workspace
 * is attached. */
int yvex_backend_rocm_paged_decode_execute_static(yvex_backend *backend,
                                                  const yvex_rocm_paged_decode_request *request,
                                                  yvex_backend_operation_facts *facts,
                                                  yvex_error *err)
{
    static const char where[] = "rocm.attention.paged.static";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    if (!state)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "a ROCm backend is required");
    if (state->kernel_bundle_state != YVEX_ROCM_KERNEL_BUNDLE_ADMITTED)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where, "no kernel bundle is admitted");
    if (!state->static_scratch) {
        yvex_error_setf(err, YVEX_ERR_UNSUPPORTED, where,
                        "the fixed device scratch is unavailable on this device (HIP error %d)",
                        state->static_scratch_error);
        return YVEX_ERR_UNSUPPORTED;
    }
    return paged_decode_execute_common(backend, request, NULL, state->static_scratch,
                                       YVEX_ROCM_STATIC_SCRATCH_BYTES, facts, err);
}

static int rocm_paged_decode_execute_fused(yvex_backend *backend,
                                           const yvex_rocm_paged_decode_request *request,
                                           const yvex_rocm_attention_epilogue *epilogue,
                                           yvex_backend_operation_facts *facts, yvex_error *err)
{
    if (!epilogue || !epilogue->output_gate)
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.attention.paged",
                      "an epilogue with an output gate tensor is required");
    return paged_decode_execute_common(backend, request, epilogue->output_gate, NULL, 0ull, facts,
                                       err);
}

/* --------------------------------------------------------- MLA decode ---- */

enum { ROCM_MLA_HEADS = 128, ROCM_MLA_REDUCE_HEADS = 64, ROCM_MLA_KEY_DIM = 576, ROCM_MLA_VALUE_DIM = 512,
       ROCM_MLA_PAGE_TOKENS = 64, ROCM_MLA_TILE_TOKENS = 32 };

static int mla_validate(const yvex_rocm_mla_decode_requirement *r, const char *where,
                        yvex_error *err)
{
    unsigned long long capacity;
    if (!r || !r->batch || !r->heads || !r->key_dimension || !r->value_dimension ||
        r->value_dimension > r->key_dimension || !r->page_tokens || !r->pool_pages ||
        !r->page_table_stride || !r->max_context_tokens ||
        !yvex_core_u64_mul(r->page_table_stride, r->page_tokens, &capacity) ||
        r->max_context_tokens > capacity ||
        (r->max_compressed_tokens &&
         (!r->compressed_pool_pages || !r->compressed_page_table_stride ||
          r->compressed_page_table_stride > 0xffffffffull ||
          r->max_compressed_tokens > r->compressed_page_table_stride * r->page_tokens)) ||
        (r->compressed_selected_stride && !r->max_compressed_tokens))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "complete MLA decode geometry is required");
    /* two geometries: the absorbed form (128 heads, 512 latent + 64 rope lanes scored, 512
     * lanes returned) and the reference's own reduce (64 heads, key and value the same 512-lane
     * row with the rope lanes inside, tests/unit/deepseek_arch_ir.c:110-125) */
    if (!((r->heads == ROCM_MLA_HEADS && r->key_dimension == ROCM_MLA_KEY_DIM) ||
          (r->heads == ROCM_MLA_REDUCE_HEADS && r->key_dimension == ROCM_MLA_VALUE_DIM)) ||
        r->value_dimension != ROCM_MLA_VALUE_DIM || r->page_tokens != ROCM_MLA_PAGE_TOKENS ||
        r->numeric_contract != YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE ||
        !r->deterministic || r->pool_pages > 0x7fffffffull || capacity > 0x7fffffffull ||
        r->batch > 65535ull || r->sliding_window > 0x7fffffffull ||
        r->compressed_pool_pages > 0x7fffffffull || r->compressed_selected_stride > 0x7fffffull ||
        r->compressed_page_table_stride * r->page_tokens > 0x7fffffffull)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm MLA decode requires 128 heads with a 512+64 latent row or 64 heads with a "
                      "512-lane row, 64-token pages and the deterministic bf16/fp32-accumulate "
                      "contract");
    if (r->output_inverse_rope.rope_dimensions) {
        const yvex_backend_attention_position *position = &r->output_inverse_rope;
        /* src/backend/cuda/kernels.cu:1006-1012: the same refusals as the reference's rotation */
        if (position->theta <= 1ull ||
            (position->original_context &&
             (!position->scaling_factor || !position->beta_slow ||
              position->beta_fast <= position->beta_slow)))
            return refuse(err, YVEX_ERR_INVALID_ARG, where, "output rotation policy is invalid");
        if ((position->rope_dimensions & 7ull) || position->rope_dimensions > r->value_dimension ||
            position->rope_dimensions > 2ull * YVEX_ROCM_ROPE_PAIRS_MAX)
            return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                          "ROCm MLA decode rotates at most 128 output lanes, in multiples of 8");
    }
    if (!(r->scale >= 0.0f) || !isfinite(r->scale))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "softmax scale must be finite and not negative");
    yvex_error_clear(err);
    return YVEX_OK;
}

/* Frequency of rotary pair `pair` (src/graph/numeric.c:877-917): theta^(-2 pair / dims), and
 * with a YaRN policy the blend between that and the same divided by the scaling factor, by a
 * linear ramp between the two corner pairs that beta_fast and beta_slow set. */
static double mla_rope_frequency(const yvex_backend_attention_position *position,
                                 unsigned long long pair)
{
    static const double pi = 3.14159265358979323846264338327950288;
    const double dims = (double)position->rope_dimensions;
    double frequency = 1.0 / pow((double)position->theta, (double)(pair * 2ull) / dims);
    if (position->original_context && position->scaling_factor) {
        const double denominator = 2.0 * log((double)position->theta);
        double low = floor(dims * log((double)position->original_context /
                                      ((double)position->beta_fast * 2.0 * pi)) / denominator);
        double high = ceil(dims * log((double)position->original_context /
                                      ((double)position->beta_slow * 2.0 * pi)) / denominator);
        double ramp, smooth;
        if (low < 0.0) low = 0.0;
        if (high > dims - 1.0) high = dims - 1.0;
        if (low == high) high += 0.001;
        ramp = ((double)pair - low) / (high - low);
        if (ramp < 0.0) ramp = 0.0;
        if (ramp > 1.0) ramp = 1.0;
        smooth = 1.0 - ramp;
        frequency = frequency / (double)position->scaling_factor * (1.0 - smooth) + frequency * smooth;
    }
    return frequency;
}

/* Chunks are a function of the request geometry only: about one workgroup per compute
 * unit of a 256-CU part, in whole pages. */
/* Tokens a session can have live: the context, or with a sliding window the window plus the
 * part of a 32-token tile in front of it. */
static unsigned long long mla_live_tokens(const yvex_rocm_mla_decode_requirement *r)
{
    if (r->sliding_window && r->sliding_window + ROCM_MLA_TILE_TOKENS - 1ull < r->max_context_tokens)
        return r->sliding_window + ROCM_MLA_TILE_TOKENS - 1ull;
    return r->max_context_tokens;
}

static unsigned int mla_chunk_for(const yvex_rocm_mla_decode_requirement *r,
                                  unsigned long long tokens, int windowed);

static unsigned int mla_chunk_tokens(const yvex_rocm_mla_decode_requirement *r)
{
    return mla_chunk_for(r, mla_live_tokens(r), r->sliding_window != 0ull);
}

static unsigned int mla_chunk_for(const yvex_rocm_mla_decode_requirement *r,
                                  unsigned long long tokens, int windowed)
{
    unsigned long long per_batch = 256ull / r->batch ? 256ull / r->batch : 1ull;
    unsigned long long chunk = (tokens + per_batch - 1ull) / per_batch;
    chunk = align_up(chunk, ROCM_MLA_PAGE_TOKENS);
    /* a windowed chunk may start in the middle of a page and so touch one page more */
    if (chunk > (unsigned long long)(YVEX_ROCM_MLA_MAX_CHUNK_PAGES - (windowed ? 1 : 0)) *
                    ROCM_MLA_PAGE_TOKENS)
        chunk = (unsigned long long)(YVEX_ROCM_MLA_MAX_CHUNK_PAGES - (windowed ? 1 : 0)) *
                ROCM_MLA_PAGE_TOKENS;
    return (unsigned int)chunk;
}

/* Chunk sizes and partial slots per batch element: the local set, then the compressed one. */
static void mla_partition(const yvex_rocm_mla_decode_requirement *r, unsigned long long *chunk,
                          unsigned long long *max_chunks, unsigned long long *extra_chunk,
                          unsigned long long *extra_max_chunks)
{
    *chunk = mla_chunk_tokens(r);
    *max_chunks = (mla_live_tokens(r) + *chunk - 1ull) / *chunk;
    *extra_chunk = *extra_max_chunks = 0ull;
    if (r->max_compressed_tokens) {
        const unsigned long long rows = r->compressed_selected_stride ? r->compressed_selected_stride
                                                                      : r->max_compressed_tokens;
        *extra_chunk = mla_chunk_for(r, rows, 0);
        *extra_max_chunks = (rows + *extra_chunk - 1ull) / *extra_chunk;
    }
}

/* Bytes behind the partials for the gathered rows of the selected class and their identity
 * page table; 0 without a selection. */
static int mla_gather_bytes(const yvex_rocm_mla_decode_requirement *r, unsigned long long *pages_each,
                            unsigned long long *rows_bytes, unsigned long long *table_bytes)
{
    *pages_each = *rows_bytes = *table_bytes = 0ull;
    if (!r->compressed_selected_stride) return 1;
    *pages_each = (r->compressed_selected_stride + r->page_tokens - 1ull) / r->page_tokens;
    if (!yvex_core_u64_mul(r->batch * *pages_each, r->page_tokens * r->key_dimension * sizeof(uint16_t),
                           rows_bytes) ||
        r->batch * *pages_each > 0x7fffffffull)
        return 0;
    *rows_bytes = align_up(*rows_bytes, ROCM_WORK_ALIGNMENT);
    *table_bytes = align_up(r->batch * *pages_each * sizeof(int32_t), ROCM_WORK_ALIGNMENT);
    return 1;
}

static int rocm_mla_decode_workspace_required(const yvex_rocm_mla_decode_requirement *r,
                                              unsigned long long *bytes, yvex_error *err)
{
    static const char where[] = "rocm.attention.mla.workspace";
    unsigned long long acc = 0ull, total = 0ull, chunk, max_chunks, extra_chunk, extra_max_chunks;
    unsigned long long gather_pages, gather_rows, gather_table;
    int rc;
    if (bytes) *bytes = 0ull;
    rc = mla_validate(r, where, err);
    if (rc != YVEX_OK) return rc;
    if (!bytes) return refuse(err, YVEX_ERR_INVALID_ARG, where, "workspace byte output is required");
    mla_partition(r, &chunk, &max_chunks, &extra_chunk, &extra_max_chunks);
    if (!decode_workspace_bytes(r->batch * (max_chunks + extra_max_chunks), r->heads, r->value_dimension,
                                sizeof(uint16_t), &acc, &total) ||
        !mla_gather_bytes(r, &gather_pages, &gather_rows, &gather_table) ||
        !yvex_core_u64_add(total, gather_rows + gather_table, &total))
        return refuse(err, YVEX_ERR_BOUNDS, where, "MLA workspace geometry overflowed");
    *bytes = total;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_mla_decode_execute(yvex_backend *backend,
                                   const yvex_rocm_mla_decode_request *request,
                                   yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.attention.mla";
    const yvex_backend_operation_variant variant = YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16;
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const yvex_rocm_mla_decode_requirement *r;
    yvex_rocm_mla_params kp;
    yvex_rocm_decode_merge_params mp;
    yvex_rocm_function_id decode_function;
    unsigned long long acc_bytes = 0ull, total = 0ull, max_chunks, chunk, extra_chunk, extra_max_chunks;
    unsigned long long gather_pages, gather_rows, gather_table, partial_bytes;
    void *work = NULL;
    yvex_error cleanup;
    int owned = 0, rc, cleanup_rc, gathered = 0;
    if (!request || !request->query || !request->latent_pages || !request->page_table ||
        !request->context_tokens || !request->output || !facts)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "complete MLA decode tensors and result facts are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    r = &request->requirement;
    rc = mla_validate(r, where, err);
    if (rc != YVEX_OK) return rc;
    memset(facts, 0, sizeof(*facts));
    if (!state ||
        !view_ok(backend, request->query, YVEX_DTYPE_BF16, r->batch * r->heads * r->key_dimension, 1) ||
        !view_ok(backend, request->latent_pages, YVEX_DTYPE_BF16,
                 r->pool_pages * r->page_tokens * r->key_dimension, 1) ||
        !view_ok(backend, request->page_table, YVEX_DTYPE_I32, r->batch * r->page_table_stride, 1) ||
        !view_ok(backend, request->context_tokens, YVEX_DTYPE_I32, r->batch, 1) ||
        !view_ok(backend, request->output, YVEX_DTYPE_BF16,
                 r->batch * r->heads * r->value_dimension, 0) ||
        (request->lse && !view_ok(backend, request->lse, YVEX_DTYPE_F32, r->batch * r->heads, 0)) ||
        (request->sinks && !view_ok(backend, request->sinks, YVEX_DTYPE_F32, r->heads, 1)) ||
        (request->output_positions &&
         (!r->output_inverse_rope.rope_dimensions ||
          !view_ok(backend, request->output_positions, YVEX_DTYPE_I64, r->batch, 1))) ||
        (r->max_compressed_tokens &&
         (!request->compressed_pages || !request->compressed_page_table ||
          !request->compressed_tokens ||
          !view_ok(backend, request->compressed_pages, YVEX_DTYPE_BF16,
                   r->compressed_pool_pages * r->page_tokens * r->key_dimension, 1) ||
          !view_ok(backend, request->compressed_page_table, YVEX_DTYPE_I32,
                   r->batch * r->compressed_page_table_stride, 1) ||
          !view_ok(backend, request->compressed_tokens, YVEX_DTYPE_I32, r->batch, 1) ||
          (r->compressed_selected_stride &&
           (!request->compressed_selected ||
            !view_ok(backend, request->compressed_selected, YVEX_DTYPE_I32,
                     r->batch * r->compressed_selected_stride, 1))))))
        return view_refusal(backend, err, where,
                      "query, latent pages, page table, context lengths and outputs must be "
                      "written tensors of this backend with the declared geometry");
    mla_partition(r, &chunk, &max_chunks, &extra_chunk, &extra_max_chunks);
    if (max_chunks + extra_max_chunks > 0x7fffffffull ||
        !decode_workspace_bytes(r->batch * (max_chunks + extra_max_chunks), r->heads, r->value_dimension,
                                sizeof(uint16_t), &acc_bytes, &total) ||
        !mla_gather_bytes(r, &gather_pages, &gather_rows, &gather_table))
        return refuse(err, YVEX_ERR_BOUNDS, where, "MLA decode geometry exceeds admitted range");
    /* partials first, then the gathered rows and their page table */
    partial_bytes = total;
    if (!yvex_core_u64_add(partial_bytes, gather_rows + gather_table, &total))
        return refuse(err, YVEX_ERR_BOUNDS, where, "MLA decode geometry exceeds admitted range");
    backend_workspace_reset(backend);
    rc = yvex_rocm_temporary_acquire(backend, total, &work, &owned, where, err);
    if (rc != YVEX_OK) return rc;
    memset(&kp, 0, sizeof(kp));
    kp.q = (const uint16_t *)request->query->data;
    kp.pool = (const uint16_t *)request->latent_pages->data;
    kp.page_table = (const int32_t *)request->page_table->data;
    kp.context = (const int32_t *)request->context_tokens->data;
    kp.part_acc = (uint16_t *)work;
    kp.part_ml = (float *)((unsigned char *)work + acc_bytes);
    kp.status = state->device_status;
    kp.batch = (uint32_t)r->batch;
    kp.heads = (uint32_t)r->heads;
    kp.key_dim = (uint32_t)r->key_dimension;
    kp.value_dim = (uint32_t)r->value_dimension;
    kp.page_tokens = (uint32_t)r->page_tokens;
    kp.pool_pages = (uint32_t)r->pool_pages;
    kp.table_stride = (uint32_t)r->page_table_stride;
    kp.chunk_tokens = (uint32_t)chunk;
    kp.max_chunks = (uint32_t)max_chunks;
    kp.window = (uint32_t)r->sliding_window;
    kp.slot_stride = (uint32_t)(max_chunks + extra_max_chunks);
    /* src/graph/core.c:604: scale = 1/sqrt(head_dimension), here over the 576-lane key */
    kp.scale_log2 = (float)(1.4426950408889634 *
                            (r->scale > 0.0f ? (double)r->scale : 1.0 / sqrt((double)r->key_dimension)));
    decode_function = r->key_dimension == ROCM_MLA_KEY_DIM ? YVEX_ROCM_FN_MLA_DECODE_BF16
                                                           : YVEX_ROCM_FN_MLA_DECODE_512_BF16;
    rc = yvex_rocm_launch(backend, decode_function, variant, (unsigned int)max_chunks,
                          (unsigned int)r->batch, 1u, 256u, 0u, &kp, where, err);
    if (rc == YVEX_OK && extra_max_chunks) {
        /* the compressed rows: same kernel over the second pool, partials after the local ones */
        yvex_rocm_mla_params cp = kp;
        cp.pool = (const uint16_t *)request->compressed_pages->data;
        cp.page_table = (const int32_t *)request->compressed_page_table->data;
        cp.context = (const int32_t *)request->compressed_tokens->data;
        cp.pool_pages = (uint32_t)r->compressed_pool_pages;
        cp.table_stride = (uint32_t)r->compressed_page_table_stride;
        cp.chunk_tokens = (uint32_t)extra_chunk;
        cp.max_chunks = (uint32_t)extra_max_chunks;
        cp.window = 0u;
        cp.first_slot = (uint32_t)max_chunks;
        cp.empty_ok = 1u;
        if (r->compressed_selected_stride) {
            /* the selected class: copy the listed rows next to each other, then walk them */
            yvex_rocm_gather_rows_params gp;
            memset(&gp, 0, sizeof(gp));
            gp.pool = cp.pool;
            gp.page_table = cp.page_table;
            gp.selected = (const int32_t *)request->compressed_selected->data;
            gp.count = cp.context;
            gp.rows = (uint16_t *)((unsigned char *)work + partial_bytes);
            gp.table = (int32_t *)((unsigned char *)work + partial_bytes + gather_rows);
            gp.status = state->device_status;
            gp.batch = kp.batch;
            gp.page_tokens = kp.page_tokens;
            gp.pool_pages = cp.pool_pages;
            gp.table_stride = cp.table_stride;
            gp.selected_stride = (uint32_t)r->compressed_selected_stride;
            gp.pages_each = (uint32_t)gather_pages;
            gp.row_elements = kp.key_dim;
            gp.max_rows = (uint32_t)r->max_compressed_tokens;
            rc = yvex_rocm_launch(backend, YVEX_ROCM_FN_GATHER_ROWS, variant,
                                  (unsigned int)r->compressed_selected_stride, (unsigned int)r->batch,
                                  1u, 128u, 0u, &gp, where, err);
            cp.pool = gp.rows;
            cp.page_table = gp.table;
            cp.pool_pages = (uint32_t)(r->batch * gather_pages);
            cp.table_stride = (uint32_t)gather_pages;
            if (rc == YVEX_OK) gathered = 1;
        }
        if (rc == YVEX_OK)
            rc = yvex_rocm_launch(backend, decode_function, variant,
                              (unsigned int)extra_max_chunks, (unsigned int)r->batch, 1u, 256u, 0u,
                              &cp, where, err);
    }
    if (rc == YVEX_OK) {
        memset(&mp, 0, sizeof(mp));
        mp.part_acc = kp.part_acc;
        mp.part_ml = kp.part_ml;
        mp.context = kp.context;
        mp.out = (uint16_t *)request->output->data;
        mp.lse = request->lse ? (float *)request->lse->data : NULL;
        mp.status = state->device_status;
        mp.sessions = kp.batch;
        mp.query_heads = kp.heads;
        mp.head_dim = kp.value_dim;
        mp.chunk_tokens = kp.chunk_tokens;
        mp.max_chunks = kp.max_chunks;
        mp.sinks = request->sinks ? (const float *)request->sinks->data : NULL;
        mp.window = kp.window;
        mp.window_align = ROCM_MLA_TILE_TOKENS;
        if (r->output_inverse_rope.rope_dimensions) {
            unsigned long long pair;
            mp.rope_dims = (uint32_t)r->output_inverse_rope.rope_dimensions;
            mp.positions = request->output_positions
                               ? (const int64_t *)request->output_positions->data : NULL;
            for (pair = 0ull; pair < r->output_inverse_rope.rope_dimensions / 2ull; ++pair)
                mp.rope_frequency[pair] = mla_rope_frequency(&r->output_inverse_rope, pair);
        }
        if (extra_max_chunks) {
            mp.extra_context = (const int32_t *)request->compressed_tokens->data;
            mp.extra_chunk_tokens = (uint32_t)extra_chunk;
            mp.extra_max_chunks = (uint32_t)extra_max_chunks;
        }
        rc = yvex_rocm_launch(backend,
                              mp.rope_dims ? YVEX_ROCM_FN_DECODE_MERGE_ROPE : YVEX_ROCM_FN_DECODE_MERGE,
                              variant,
                              (unsigned int)((r->heads + 3ull) / 4ull), (unsigned int)r->batch, 1u,
                              256u, 0u, &mp, where, err);
    }
    if (rc == YVEX_OK) {
        facts->kernel_launches = (extra_max_chunks ? 3ull : 2ull) + (gathered ? 1ull : 0ull);
        facts->accelerated_matrix_launches = extra_max_chunks ? 2ull : 1ull;
        facts->temporary_bytes = total;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, variant, where, facts, err);
    }
    yvex_error_clear(&cleanup);
    cleanup_rc = yvex_rocm_temporary_release(backend, work, total, owned, &cleanup);
    backend_workspace_reset(backend);
    if (rc == YVEX_OK && cleanup_rc != YVEX_OK) {
        rc = cleanup_rc;
        if (err) *err = cleanup;
    }
    if (rc != YVEX_OK) return rc;
    request->output->is_written = 1;
    if (request->lse) request->lse->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ------------------------------------------------------------ KV append ---- */

/* Writes new key/value rows into the paged pools (rotary on the keys, Q8_0 quantise on
 * write).  One launch; the pools stay written tensors. */
static int rocm_kv_append_execute(yvex_backend *backend, const yvex_rocm_kv_append_request *request,
                                  yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.attention.kv_append";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const yvex_rocm_kv_append_requirement *r;
    yvex_rocm_kv_append_params kp;
    yvex_backend_operation_variant variant;
    yvex_dtype pool_dtype;
    unsigned long long block_bytes, pool_bytes, row_elements, capacity, page_slots;
    int rc;
    if (!request || !request->key || !request->value || !request->row_start ||
        !request->position_start || !request->token_count || !request->page_table ||
        !request->k_pool || !request->v_pool || !facts)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "complete KV-append tensors and result facts are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    r = &request->requirement;
    if (!r->sessions || !r->total_tokens || !r->max_tokens_per_session || !r->key_value_heads ||
        !r->head_dimension || !r->page_tokens || !r->pool_pages || !r->page_table_stride ||
        r->max_tokens_per_session > r->total_tokens ||
        !yvex_core_u64_mul(r->page_table_stride, r->page_tokens, &capacity) ||
        (r->rotary_dimension && (!request->cosine || !request->sine)))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "complete KV-append geometry is required");
    block_bytes = yvex_rocm_kv_page_block_bytes(r->storage, r->head_dimension, r->page_tokens);
    if (!block_bytes || r->rotary_dimension > r->head_dimension || r->rotary_dimension % 16ull ||
        (r->rotary_mode != YVEX_ROCM_ROTARY_BF16_STAGED && r->rotary_mode != YVEX_ROCM_ROTARY_F32_ROUNDED) ||
        r->sessions > 65535ull || r->key_value_heads > 65535ull || r->pool_pages > 0x7fffffffull ||
        capacity > 0x7fffffffull || r->total_tokens > 0x7fffffffull)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm KV append requires head dimension 128 (bf16 pages: 64, 128 or 256), pages of 16 "
                      "or 64 tokens, BF16 or Q8_0 storage and a rotary dimension that is a multiple of 16");
    memset(facts, 0, sizeof(*facts));
    pool_dtype = r->storage == YVEX_ROCM_KV_BF16 ? YVEX_DTYPE_BF16 : YVEX_DTYPE_I8;
    row_elements = r->total_tokens * r->key_value_heads * r->head_dimension;
    /* the pools may be fresh (all zero) or hold earlier tokens: written state is not required */
    if (!state || !yvex_core_u64_mul(r->pool_pages * r->key_value_heads, block_bytes, &pool_bytes) ||
        !view_ok(backend, request->key, YVEX_DTYPE_BF16, row_elements, 1) ||
        !view_ok(backend, request->value, YVEX_DTYPE_BF16, row_elements, 1) ||
        (r->rotary_dimension &&
         (!view_ok(backend, request->cosine, YVEX_DTYPE_F32, r->total_tokens * r->rotary_dimension, 1) ||
          !view_ok(backend, request->sine, YVEX_DTYPE_F32, r->total_tokens * r->rotary_dimension, 1))) ||
        !view_ok(backend, request->row_start, YVEX_DTYPE_I32, r->sessions, 1) ||
        !view_ok(backend, request->position_start, YVEX_DTYPE_I32, r->sessions, 1) ||
        !view_ok(backend, request->token_count, YVEX_DTYPE_I32, r->sessions, 1) ||
        !view_ok(backend, request->page_table, YVEX_DTYPE_I32, r->sessions * r->page_table_stride, 1) ||
        !view_ok(backend, request->k_pool, pool_dtype,
                 pool_bytes / yvex_rocm_dtype_bytes(pool_dtype), 0) ||
        !view_ok(backend, request->v_pool, pool_dtype,
                 pool_bytes / yvex_rocm_dtype_bytes(pool_dtype), 0))
        return view_refusal(backend, err, where,
                      "rows, tables, descriptors and pools must be tensors of this backend with "
                      "the declared geometry");
    memset(&kp, 0, sizeof(kp));
    kp.key = (const uint16_t *)request->key->data;
    kp.value = (const uint16_t *)request->value->data;
    kp.cosine = r->rotary_dimension ? (const float *)request->cosine->data : NULL;
    kp.sine = r->rotary_dimension ? (const float *)request->sine->data : NULL;
    kp.row_start = (const int32_t *)request->row_start->data;
    kp.position_start = (const int32_t *)request->position_start->data;
    kp.token_count = (const int32_t *)request->token_count->data;
    kp.page_table = (const int32_t *)request->page_table->data;
    kp.k_pool = request->k_pool->data;
    kp.v_pool = request->v_pool->data;
    kp.status = state->device_status;
    kp.total_tokens = r->total_tokens;
    kp.sessions = (uint32_t)r->sessions;
    kp.kv_heads = (uint32_t)r->key_value_heads;
    kp.head_dim = (uint32_t)r->head_dimension;
    kp.rotary_dim = (uint32_t)r->rotary_dimension;
    kp.rotary_mode = (uint32_t)r->rotary_mode;
    kp.page_shift = r->page_tokens == ROCM_PAGE_TOKENS ? 0u : 2u;
    kp.pool_pages = (uint32_t)r->pool_pages;
    kp.table_stride = (uint32_t)r->page_table_stride;
    /* one workgroup row per 16-token block: a run of n tokens touches at most
     * (n + 16 - 2) / 16 + 1 of them, whatever the page size */
    page_slots = (r->max_tokens_per_session + ROCM_PAGE_TOKENS - 2ull) / ROCM_PAGE_TOKENS + 1ull;
    if (page_slots > 0x7fffffffull)
        return refuse(err, YVEX_ERR_BOUNDS, where, "KV-append geometry exceeds admitted range");
    variant = r->storage == YVEX_ROCM_KV_BF16 ? YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16
                                               : YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0;
    backend_workspace_reset(backend);
    rc = yvex_rocm_launch(backend,
                          r->storage != YVEX_ROCM_KV_BF16   ? YVEX_ROCM_FN_KV_APPEND_Q8_0
                          : r->head_dimension == 64ull  ? YVEX_ROCM_FN_KV_APPEND_BF16_64
                          : r->head_dimension == 256ull ? YVEX_ROCM_FN_KV_APPEND_BF16_256
                                                        : YVEX_ROCM_FN_KV_APPEND_BF16,
                          variant, (unsigned int)page_slots,
                          (unsigned int)((r->key_value_heads + YVEX_ROCM_KV_APPEND_HEADS - 1ull) /
                                         YVEX_ROCM_KV_APPEND_HEADS),
                          (unsigned int)r->sessions, 64u * YVEX_ROCM_KV_APPEND_HEADS, 0u, &kp, where,
                          err);
    if (rc == YVEX_OK) {
        facts->kernel_launches = 1ull;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, variant, where, facts, err);
    }
    if (rc != YVEX_OK) return rc;
    request->k_pool->is_written = 1;
    request->v_pool->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ------------------------------------------- token-major history writer ---- */

static int rocm_history_append_execute(yvex_backend *backend,
                                       const yvex_rocm_history_append_request *request,
                                       yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.history_append";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const yvex_rocm_history_append_requirement *r;
    yvex_backend_operation_variant variant;
    yvex_rocm_history_append_params hp;
    yvex_dtype dtype;
    unsigned long long width, k_stride, v_stride, rows, new_elements, k_elements, v_elements, pieces;
    unsigned long long query_elements = 0ull;
    unsigned long long piece; /* elements in 16 bytes */
    int rc;
    if (!request || !request->key || !request->value || !request->key_history ||
        !request->value_history || !facts)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "complete history-append tensors and result facts are required");
    if ((request->requirement.query_heads != 0ull) != (request->query != NULL))
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "a query tensor and its head count are given together or not at all");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    r = &request->requirement;
    if (!r->tokens || !r->key_value_heads || !r->head_dimension ||
        !yvex_core_u64_mul(r->key_value_heads, r->head_dimension, &width) ||
        !yvex_core_u64_add(r->first_row, r->tokens, &rows) ||
        (r->rotary_dimension && (!request->cosine || !request->sine)))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "complete history-append geometry is required");
    k_stride = r->key_token_stride ? r->key_token_stride : width;
    v_stride = r->value_token_stride ? r->value_token_stride : width;
    if (k_stride < width || v_stride < width)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "a history token stride is narrower than one row of key/value heads");
    dtype = request->key->dtype;
    if (dtype != YVEX_DTYPE_BF16 && dtype != YVEX_DTYPE_F32)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm history append takes BF16 or F32 rows and histories of the same type");
    piece = 16ull / yvex_rocm_dtype_bytes(dtype);
    if (r->head_dimension % piece || r->head_dimension > 256ull || (k_stride | v_stride) % piece ||
        (r->rotary_mode != YVEX_ROCM_ROTARY_BF16_STAGED && r->rotary_mode != YVEX_ROCM_ROTARY_F32_ROUNDED) ||
        r->rotary_dimension > r->head_dimension || r->rotary_dimension % (2ull * piece) ||
        r->tokens > 0x7fffffffull || r->key_value_heads > 65535ull || r->query_heads > 65535ull)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm history append requires a head dimension (at most 256) and token strides "
                      "that are multiples of 16 bytes and rotary halves that are too");
    memset(facts, 0, sizeof(*facts));
    if (!state || !yvex_core_u64_mul(r->tokens, width, &new_elements) ||
        !yvex_core_u64_mul(rows - 1ull, k_stride, &k_elements) ||
        !yvex_core_u64_add(k_elements, width, &k_elements) ||
        !yvex_core_u64_mul(rows - 1ull, v_stride, &v_elements) ||
        !yvex_core_u64_add(v_elements, width, &v_elements) ||
        !yvex_core_u64_mul(r->tokens * r->query_heads, r->head_dimension, &query_elements) ||
        !yvex_core_u64_mul(r->tokens * (r->key_value_heads + r->query_heads),
                           r->head_dimension / piece, &pieces) ||
        (pieces + 255ull) / 256ull > 0x7fffffffull)
        return refuse(err, YVEX_ERR_BOUNDS, where, "history-append geometry exceeds admitted range");
    /* a history may be fresh or hold earlier tokens: written state is not required of it */
    if (!view_ok(backend, request->key, dtype, new_elements, 1) ||
        !view_ok(backend, request->value, dtype, new_elements, 1) ||
        (request->query && !view_ok(backend, request->query, dtype, query_elements, 1)) ||
        (r->rotary_dimension &&
         (!view_ok(backend, request->cosine, YVEX_DTYPE_F32, r->tokens * r->rotary_dimension, 1) ||
          !view_ok(backend, request->sine, YVEX_DTYPE_F32, r->tokens * r->rotary_dimension, 1))) ||
        !view_ok(backend, request->key_history, dtype, k_elements, 0) ||
        !view_ok(backend, request->value_history, dtype, v_elements, 0))
        return view_refusal(backend, err, where,
                            "new rows, tables and history views must be tensors of this backend "
                            "with the declared geometry and one element type");
    if (((uintptr_t)request->key->data | (uintptr_t)request->value->data |
         (uintptr_t)request->key_history->data | (uintptr_t)request->value_history->data |
         (uintptr_t)(request->query ? request->query->data : NULL)) & 15u)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm history append requires 16-byte aligned rows");
    if (request->query) {
        /* rotated where it lies by threads of the launch that reads and writes the others */
        const yvex_device_tensor *others[4] = {request->key, request->value, request->key_history,
                                               request->value_history};
        uintptr_t lo = (uintptr_t)request->query->data, hi = lo + request->query->bytes;
        size_t i;
        for (i = 0u; i < 4u; ++i) {
            uintptr_t at = (uintptr_t)others[i]->data;
            if (at < hi && lo < at + others[i]->bytes)
                return refuse(err, YVEX_ERR_INVALID_ARG, where,
                              "the query tensor overlaps another tensor of the request");
        }
    }
    memset(&hp, 0, sizeof(hp));
    hp.key = request->key->data;
    hp.value = request->value->data;
    hp.cosine = r->rotary_dimension ? (const float *)request->cosine->data : NULL;
    hp.sine = r->rotary_dimension ? (const float *)request->sine->data : NULL;
    hp.key_history = request->key_history->data;
    hp.value_history = request->value_history->data;
    hp.status = state->device_status;
    hp.first_row = r->first_row;
    hp.key_token_stride = k_stride;
    hp.value_token_stride = v_stride;
    hp.tokens = (uint32_t)r->tokens;
    hp.kv_heads = (uint32_t)r->key_value_heads;
    hp.head_dim = (uint32_t)r->head_dimension;
    hp.rotary_dim = (uint32_t)r->rotary_dimension;
    hp.rotary_mode = (uint32_t)r->rotary_mode;
    hp.query_heads = (uint32_t)r->query_heads;
    hp.query = request->query ? request->query->data : NULL;
    variant = dtype == YVEX_DTYPE_BF16 ? YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16
                                       : YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32;
    backend_workspace_reset(backend);
    rc = yvex_rocm_launch(backend,
                          dtype == YVEX_DTYPE_BF16 ? YVEX_ROCM_FN_HISTORY_APPEND_BF16
                                                   : YVEX_ROCM_FN_HISTORY_APPEND_F32,
                          variant, (unsigned int)((pieces + 255ull) / 256ull), 1u, 1u, 256u, 0u, &hp,
                          where, err);
    if (rc == YVEX_OK) {
        facts->kernel_launches = 1ull;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, variant, where, facts, err);
    }
    if (rc != YVEX_OK) return rc;
    request->key_history->is_written = 1;
    request->value_history->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ---------------------------------------------------------- op tables ---- */

/* The attention slots and the four element-wise slots the reference's decoder calls around
 * them; every other slot stays NULL ("not published"). */
static const yvex_backend_transformer_operations rocm_transformer_ops = {
    .attention_workspace_required = rocm_attention_workspace_required,
    .attention_execute = rocm_attention_execute,
    .rotary_half_f32 = yvex_rocm_rotary_half_f32,
    .split_interleaved_two_f32 = yvex_rocm_split_interleaved_two_f32,
    .sigmoid_product_bf16 = yvex_rocm_sigmoid_product_bf16,
    .bf16_round = yvex_rocm_bf16_round,
};

static const yvex_backend_rocm_attention_operations rocm_attention_ops = {
    .attention_execute_lse = rocm_attention_execute_lse,
    .paged_decode_workspace_required = rocm_paged_decode_workspace_required,
    .paged_decode_execute = rocm_paged_decode_execute,
    .mla_decode_workspace_required = rocm_mla_decode_workspace_required,
    .mla_decode_execute = rocm_mla_decode_execute,
    .kv_append_execute = rocm_kv_append_execute,
    .attention_execute_fused = rocm_attention_execute_fused,
    .paged_decode_execute_fused = rocm_paged_decode_execute_fused,
    .history_append_execute = rocm_history_append_execute,
};

/* A table is published only once the kernel bundle is admitted
 * (tests/unit/backend_cpu.c:44-48 asserts the same rule for a backend without kernels). */
const yvex_backend_transformer_operations *yvex_rocm_transformer_operations(
    const yvex_backend *backend)
{
    const yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    return state && state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_ADMITTED
               ? &rocm_transformer_ops
               : NULL;
}

/* The operations without a reference counterpart.  Not a vtable slot (the reference's table
 * has none for them): a function of the ROCm arm that answers for ROCm backends with an
 * admitted bundle and NULL ("not published") for everything else. */
const yvex_backend_rocm_attention_operations *yvex_backend_rocm_attention_operations_get(
    const yvex_backend *backend)
{
    const yvex_rocm_backend_state *state;
    if (!backend || backend->kind != YVEX_BACKEND_KIND_ROCM) return NULL;
    state = yvex_rocm_state(backend);
    return state && state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_ADMITTED
               ? &rocm_attention_ops
               : NULL;
}
