/*
 * C ABI of the MI355X (gfx950) attention backend for YVEX, second part: the operations the
 * reference has no counterpart for (NEW SURFACE: paged GQA decode over bf16 or Q8_0 pages, the
 * absorbed MLA decode, the page and history writers, the fused epilogues, recorded launch
 * sequences, the entry point that allocates nothing), the benchmark record, and the host-side
 * codecs and page packers.  Builds on yvex_rocm.h (statuses, tensors, the attention contract);
 * the two modes of compiling described there apply here too.
 */
#ifndef YVEX_ROCM_OPERATIONS_H
#define YVEX_ROCM_OPERATIONS_H

#include "yvex_rocm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ======================= NEW SURFACE (no reference counterpart) ============ */

/* KV cache storage kinds for paged decode. */
typedef enum {
    YVEX_ROCM_KV_BF16 = 1,
    YVEX_ROCM_KV_Q8_0 = 2
} yvex_rocm_kv_storage;

/*
 * Paged GQA decode: one query token per session against a paged KV pool.
 * Device page layouts (head_dimension 128; bf16 pages also 64 and 256, with d/8 chunks of K
 * and d rows of V in the same order), per (page, kv_head) and block of 16 tokens; a
 * page of 16 tokens (page_tokens 16) is one block, a page of 64 tokens (page_tokens 64) four
 * blocks one behind the other, tokens 16 s .. 16 s + 15 of the page in block s:
 *   BF16  K block: uint16 [d/8][16 tokens][8]           (4096 B)
 *         V block: uint16 [d][16 tokens]                (4096 B)
 *   Q8_0  K block: 2048 int8 codes + f16 scale [16 tokens][4 blocks]; V block likewise (2176 B each).
 *         The codes are ordered for the reading wave: lane L takes 32 of them ([4 blocks][8] of one
 *         token for K, [8 dim blocks][4 tokens] of one dim for V), 16 at byte 16 L and 16 at byte
 *         1024 + 16 L of the block.  Build and read pages with yvex_rocm_kv_pack_pages /
 *         yvex_rocm_kv_unpack_pages, or write them with kv_append_execute.
 * Pool = [pool_pages][key_value_heads][page_tokens / 16][block].  yvex_rocm_kv_pack_* build these from
 * token-major rows.  page_table is I32 [sessions][page_table_stride]; context_tokens is
 * I32 [sessions] (both device tensors).  Output is BF16 [sessions][query_heads][d], lse is
 * F32 [sessions][query_heads] (natural-log log-sum-exp of the scaled scores; optional).
 */
typedef struct yvex_rocm_paged_decode_requirement {
    unsigned long long sessions, query_heads, key_value_heads, head_dimension;
    unsigned long long page_tokens, pool_pages, page_table_stride;
    /* upper bound on any session's context, used only to size the launch and workspace */
    unsigned long long max_context_tokens;
    yvex_rocm_kv_storage kv_storage;
    yvex_transformer_attention_numeric_contract numeric_contract;
    int deterministic;
} yvex_rocm_paged_decode_requirement;

typedef struct yvex_rocm_paged_decode_request {
    yvex_rocm_paged_decode_requirement requirement;
    const yvex_device_tensor *query, *key_pages, *value_pages, *page_table, *context_tokens;
    yvex_device_tensor *output, *lse;
} yvex_rocm_paged_decode_request;

/*
 * Shared-KV (MLA) decode: `heads` query heads share one row per token; score over
 * key_dimension lanes, value = the first value_dimension lanes of the same row.
 * Pool: BF16 [pool_pages][page_tokens][key_dimension] (token-major, page_tokens 64).
 * query BF16 [batch][heads][key_dimension]; output BF16 [batch][heads][value_dimension].
 * Admitted geometries: the absorbed form, 128 heads, key_dimension 576 (512 latent + 64 rope),
 * value_dimension 512; and the reference's own reduce (src/graph/core.c:361-508,
 * tests/unit/deepseek_arch_ir.c:110-125), 64 heads, key_dimension == value_dimension == 512
 * with the rope lanes inside the row.
 */
/* Rotary position policy of an attention layer: the fields the rotation reads
 * (include/yvex/internal/backend.h:51-54, same names and order). */
#ifndef YVEX_ROCM_IN_TREE
typedef struct {
    unsigned long long theta, scaling_factor, original_context;
    unsigned long long beta_fast, beta_slow, rope_dimensions;
} yvex_backend_attention_position;
#endif /* !YVEX_ROCM_IN_TREE */

typedef struct yvex_rocm_mla_decode_requirement {
    unsigned long long batch, heads, key_dimension, value_dimension;
    unsigned long long page_tokens, pool_pages, page_table_stride, max_context_tokens;
    yvex_transformer_attention_numeric_contract numeric_contract;
    int deterministic;
    /* Sliding-window position filter of the shared-KV reduce
     * (src/backend/cuda/attention_kernels.cu:79-84): the query at position context - 1 sees
     * positions >= context - sliding_window.  0: the whole context. */
    unsigned long long sliding_window;
    /* Second candidate set of the shared-KV reduce: compressed rows visited after the local
     * ones inside the same softmax (src/graph/core.c:437-468, the dense class whose visible
     * rows are a prefix; attention_kernels.cu:85-97).  Same row format and page size as the
     * latent pool.  max_compressed_tokens = 0: no such set. */
    unsigned long long compressed_pool_pages, compressed_page_table_stride, max_compressed_tokens;
    /* The selected class (src/graph/core.c:443-452, attention_kernels.cu:88-90): the visible
     * compressed rows are the entries of a per-session index list, in list order, instead of
     * a prefix.  compressed_selected_stride is the list capacity; 0: the prefix class. */
    unsigned long long compressed_selected_stride;
    /* Inverse rotation of the published rows (src/graph/core.c:499-507,
     * src/backend/cuda/attention.c:1424-1429): each head's row is rounded to bf16, its LAST
     * rope_dimensions lanes are rotated back by the query token's position, adjacent pairs
     * (2i, 2i+1), angle = position * frequency(i) with the YaRN ramp of
     * src/graph/numeric.c:877-917 when original_context and scaling_factor are set, and the
     * row is rounded again.  rope_dimensions = 0: rows are published as they are.  Admitted:
     * rope_dimensions a multiple of 8, at most 128 and at most value_dimension; theta > 1;
     * with original_context set, scaling_factor >= 1 and beta_fast > beta_slow >= 1. */
    yvex_backend_attention_position output_inverse_rope;
    /* Softmax scale; 0 selects 1 / sqrt(key_dimension) (src/graph/core.c:604). */
    float scale;
} yvex_rocm_mla_decode_requirement;

typedef struct yvex_rocm_mla_decode_request {
    yvex_rocm_mla_decode_requirement requirement;
    const yvex_device_tensor *query, *latent_pages, *page_table, *context_tokens;
    yvex_device_tensor *output, *lse;
    /* Optional F32 [heads] sink logits (src/graph/core.c:471-508, attention_kernels.cu:164-166):
     * each seeds the head's maximum and adds exp(sink - max) to its denominator with a zero
     * value row; the LSE output includes it.  NULL: no sink. */
    const yvex_device_tensor *sinks;
    /* With max_compressed_tokens > 0: BF16 [compressed_pool_pages][page_tokens][key_dimension],
     * I32 [batch][compressed_page_table_stride], and I32 [batch] visible compressed rows per
     * session (0 allowed: position + ratio - 1 <= token position holds for a prefix of
     * floor(context / ratio) rows, which the caller passes). */
    const yvex_device_tensor *compressed_pages, *compressed_page_table, *compressed_tokens;
    /* With compressed_selected_stride > 0: I32 [batch][compressed_selected_stride] indices of
     * compressed rows (positions in the session's compressed sequence, below
     * max_compressed_tokens); compressed_tokens then holds the number of list entries. */
    const yvex_device_tensor *compressed_selected;
    /* With output_inverse_rope: optional I64 [batch] absolute position of each query token
     * (token_position + token of src/graph/core.c:475); NULL: context_tokens[b] - 1, the
     * position of the newest row of a history that starts at 0. */
    const yvex_device_tensor *output_positions;
} yvex_rocm_mla_decode_request;

/* KV page writer (no reference counterpart as one operation: it is the rotary step of
 * src/runtime/decoder.c:1236-1242 fused with the history append of
 * src/runtime/stateful_attention.c:183-243, writing the paged device layouts).  Session s
 * contributes token_count[s] consecutive rows of `key` / `value` starting at row_start[s];
 * they become positions position_start[s] .. of that session.  rotary_dimension = 0 writes
 * the keys as given; otherwise cosine / sine are F32 [total_tokens][rotary_dimension] tables
 * indexed by input row and the keys are rotated in the order rotary_mode names (below).
 * page_tokens is 16 or 64 (the layouts of the paged decode).
 * Caller contract: within one call no page id appears in the rows of two sessions, and the
 * token ranges of one session do not overlap.  A V page block is filled by a read-modify-
 * write of whole 16-byte groups, one workgroup per (session, page): two sessions writing the
 * same page in one launch race on it and the result is undefined (nothing is flagged).  Pages
 * shared between sessions (a common prefix) are fine as long as no session of the call
 * writes to them. */
/* How the keys are rotated on their way into a pool or a history.  The reference has both
 * orders: BF16_STAGED is its bf16 rotary kernel, every product and sum rounded to bf16
 * (yvex_rotary_half_f32, src/backend/cuda/transformer_kernels.cu:79-108; the joint transformer
 * and the text encoder, src/backend/cuda/joint_transformer.c:606-618, text_encoder.c:600-609);
 * F32_ROUNDED is what its decoder runs in front of attention (decoder_rotary,
 * src/runtime/decoder.c:1112-1131,1236-1242): the plain F32 rotation
 * (yvex_rotary_half_plain_f32, transformer_kernels.cu:110-134) and then one bf16 rounding of
 * every lane of the tensor (decoder_round, src/backend/cuda/kernels.cu:40-58). */
typedef enum {
    YVEX_ROCM_ROTARY_BF16_STAGED = 0,
    YVEX_ROCM_ROTARY_F32_ROUNDED = 1
} yvex_rocm_rotary_mode;

typedef struct yvex_rocm_kv_append_requirement {
    unsigned long long sessions, total_tokens, max_tokens_per_session;
    unsigned long long key_value_heads, head_dimension, page_tokens, pool_pages, page_table_stride;
    unsigned long long rotary_dimension;
    yvex_rocm_kv_storage storage;
    yvex_rocm_rotary_mode rotary_mode;
} yvex_rocm_kv_append_requirement;

typedef struct yvex_rocm_kv_append_request {
    yvex_rocm_kv_append_requirement requirement;
    const yvex_device_tensor *key, *value;                /* BF16 [total_tokens][kv_heads][d] */
    const yvex_device_tensor *cosine, *sine;              /* F32, or NULL without rotary */
    const yvex_device_tensor *row_start, *position_start, *token_count; /* I32 [sessions] */
    const yvex_device_tensor *page_table;                 /* I32 [sessions][stride] */
    yvex_device_tensor *k_pool, *v_pool;
} yvex_rocm_kv_append_request;

/*
 * Token-major history writer: the step in front of attention for the reference's own
 * history layout.  The reference rotates the new keys in a pass of their own
 * (src/runtime/decoder.c:1236-1242) and then appends every token with two device copies,
 * key then value, into row history_tokens + t of the layer's [K | V] history
 * (src/runtime/stateful_attention.c:183-222).  This does both in one launch: rows
 * first_row .. first_row + tokens - 1 of key_history and value_history receive the new rows
 * (keys rotated: rotate-half over the first rotary_dimension lanes of every head,
 * src/backend/cuda/transformer_kernels.cu:79-108, every product and sum rounded to BF16),
 * nothing else is touched.  key_history / value_history are the views attention_execute is
 * handed afterwards for key_value_tokens = first_row + tokens:
 * (first_row + tokens - 1) * stride + key_value_heads * head_dimension elements, strides in
 * elements (0 = packed); for the reference's interleaved rows both views lie in one tensor,
 * the value view key_value_heads * head_dimension elements behind the key view, stride twice
 * that.  New rows and histories are all BF16 (the bf16 kernels' histories) or all F32 (the
 * reference's own histories and the EXACT_F32 kernels'; the F32 inputs enter the rotary
 * products as they are, as in yvex_rotary_half_f32, and the results are bf16 values stored
 * as F32).  Over a reserved address range the rows must be committed first.  Rows, strides
 * and rotary halves must be multiples of 16 bytes; non-finite inputs, table entries or
 * results are YVEX_ERR_FORMAT.  With query_heads and a query tensor the same launch also
 * rotates the new tokens' queries where they lie, with the arithmetic and mode of the keys
 * (the decoder's pass over the queries, src/runtime/decoder.c:1235-1238), so that attention
 * is the next call; the query tensor must not overlap any other tensor of the request.
 */
typedef struct yvex_rocm_history_append_requirement {
    unsigned long long tokens, first_row;
    unsigned long long key_value_heads, head_dimension, rotary_dimension;
    unsigned long long key_token_stride, value_token_stride;
    yvex_rocm_rotary_mode rotary_mode; /* F32_ROUNDED also rounds the key lanes behind the rotary ones */
    unsigned long long query_heads;    /* 0 without a query tensor */
} yvex_rocm_history_append_requirement;

typedef struct yvex_rocm_history_append_request {
    yvex_rocm_history_append_requirement requirement;
    const yvex_device_tensor *key, *value;   /* BF16 or F32 [tokens][kv_heads][d] */
    const yvex_device_tensor *cosine, *sine; /* F32 [tokens][rotary_dimension], or NULL without rotary */
    yvex_device_tensor *key_history, *value_history; /* the element type of key and value */
    yvex_device_tensor *query; /* [tokens][query_heads][d] of that type, or NULL */
} yvex_rocm_history_append_request;

/*
 * Epilogue fused into the attention kernels.  The arithmetic is the reference's sigmoid
 * output gate (yvex_sigmoid_product_bf16_f32, src/backend/cuda/transformer_kernels.cu:353-364),
 * which the decoder runs as a separate pass right after attention
 * (src/runtime/decoder.c:1266-1269): output = bf16(bf16(attention) * 1 / (1 + exp(-gate))).
 * output_gate is a written BF16 tensor with the geometry of the output
 * ([rows][query_heads][head_dimension], packed).  Only the BF16 contract takes an epilogue.
 */
typedef struct yvex_rocm_attention_epilogue {
    const yvex_device_tensor *output_gate;
} yvex_rocm_attention_epilogue;

typedef struct yvex_backend_rocm_attention_operations {
    /* attention_execute with an additional F32 [query_tokens][query_heads] LSE output */
    int (*attention_execute_lse)(yvex_backend *, const yvex_transformer_attention_request *,
                                 yvex_device_tensor *lse, yvex_backend_operation_facts *,
                                 yvex_error *);
    int (*paged_decode_workspace_required)(const yvex_rocm_paged_decode_requirement *,
                                           unsigned long long *, yvex_error *);
    int (*paged_decode_execute)(yvex_backend *, const yvex_rocm_paged_decode_request *,
                                yvex_backend_operation_facts *, yvex_error *);
    int (*mla_decode_workspace_required)(const yvex_rocm_mla_decode_requirement *,
                                         unsigned long long *, yvex_error *);
    int (*mla_decode_execute)(yvex_backend *, const yvex_rocm_mla_decode_request *,
                              yvex_backend_operation_facts *, yvex_error *);
    int (*kv_append_execute)(yvex_backend *, const yvex_rocm_kv_append_request *,
                             yvex_backend_operation_facts *, yvex_error *);
    /* attention_execute / paged_decode_execute with the epilogue applied before the rows are
     * published; lse may be NULL */
    int (*attention_execute_fused)(yvex_backend *, const yvex_transformer_attention_request *,
                                   const yvex_rocm_attention_epilogue *, yvex_device_tensor *lse,
                                   yvex_backend_operation_facts *, yvex_error *);
    int (*paged_decode_execute_fused)(yvex_backend *, const yvex_rocm_paged_decode_request *,
                                      const yvex_rocm_attention_epilogue *,
                                      yvex_backend_operation_facts *, yvex_error *);
    int (*history_append_execute)(yvex_backend *, const yvex_rocm_history_append_request *,
                                  yvex_backend_operation_facts *, yvex_error *);
} yvex_backend_rocm_attention_operations;
const yvex_backend_rocm_attention_operations *yvex_backend_rocm_attention_operations_get(
    const yvex_backend *backend);

/*
 * paged_decode_execute for callers that cannot allocate.  It has no counterpart in the
 * reference; it is for code that runs where hipMalloc is not allowed: under stream capture,
 * in tight serving loops, in harnesses that forbid allocation.  Same request, same kernels
 * and bit-identical results as paged_decode_execute, but the split-K partials go to a fixed
 * device array of YVEX_ROCM_STATIC_WORKSPACE_BYTES that each GPU holds from the moment the
 * library is loaded until the process ends; an attached workspace is ignored and no
 * allocation or release call is made.  A request whose partials need more
 * (paged_decode_workspace_required tells) is refused with YVEX_ERR_BOUNDS.  Every call on a
 * GPU shares that GPU's array: calls that overlap on one GPU race (one backend stream
 * serialises its own calls; two backends on one device must not use it at the same time).
 */
#define YVEX_ROCM_STATIC_WORKSPACE_BYTES (16ull << 20)
int yvex_backend_rocm_paged_decode_execute_static(yvex_backend *backend,
                                                  const yvex_rocm_paged_decode_request *request,
                                                  yvex_backend_operation_facts *facts,
                                                  yvex_error *err);

/*
 * Completion mode.  IMMEDIATE (default) is the reference's behaviour: every operation
 * synchronises once and reads the device status word before returning
 * (src/backend/cuda/transformer.c:655-673).  DEFERRED enqueues only; the status word is
 * checked by the next yvex_backend_sync, which reports the first recorded failure.
 */
typedef enum {
    YVEX_ROCM_COMPLETION_IMMEDIATE = 0,
    YVEX_ROCM_COMPLETION_DEFERRED = 1
} yvex_rocm_completion_mode;
int yvex_backend_rocm_completion_mode_set(yvex_backend *backend, yvex_rocm_completion_mode mode,
                                          yvex_error *err);

/*
 * Measured device bandwidth (include/yvex/internal/backend.h:180-192,261;
 * src/backend/core.c:483-502 dispatch, src/backend/cuda/backend.c:1356-1500 the CUDA probe).
 * Same record, same rule: five samples of `iterations` passes over a working set, the
 * sustainable rate is bytes over the median sample.  stream_* times a pure streaming read of
 * the working set (HBM read rate), copy_* a device-to-device copy (counted as read plus
 * write).  The coherent-host fields are for unified-memory parts and stay zero here; the
 * identity strings are left empty.  The first successful probe is kept and returned again.
 */
#ifndef YVEX_ROCM_IN_TREE
#define YVEX_BACKEND_BANDWIDTH_SCHEMA_V1 1u
#define YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT 5u
#define YVEX_SHA256_HEX_BYTES 65u
typedef struct {
    unsigned int schema_version;
    unsigned long long working_set_bytes, iterations, sample_count;
    unsigned long long stream_elapsed_ns[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned long long copy_elapsed_ns[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned long long coherent_host_elapsed_ns[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned long long sustainable_read_bytes_per_second, sustainable_copy_bytes_per_second;
    unsigned long long sustainable_coherent_host_bytes_per_second;
    char kernel_bundle_identity[YVEX_SHA256_HEX_BYTES], identity[YVEX_SHA256_HEX_BYTES];
} yvex_backend_bandwidth_evidence;
#endif /* !YVEX_ROCM_IN_TREE */
int yvex_backend_bandwidth_probe(yvex_backend *backend, yvex_backend_bandwidth_evidence *out,
                                 yvex_error *err);

/*
 * Recorded launch sequences (no reference counterpart; for launch-bound steps such as a
 * single-session decode, where two kernel launches cost more host time than device time).
 * Between begin and end the attention operations of this backend are recorded on its stream
 * instead of being run: they validate and launch as usual but nothing executes, no status is
 * read, and results are undefined until the sequence is replayed.  Everything that would
 * allocate, free, copy, clear or wait is refused with YVEX_ERR_STATE while recording: attach
 * a workspace large enough for the recorded operations first.  launch() enqueues the whole
 * sequence with one call and then completes like any operation (status check in the
 * immediate mode, at the next sync in the deferred mode).  The tensors the recorded
 * operations named must stay allocated, at the same geometry, until the sequence is
 * released; their contents may change between replays.  The library holds the caller to it
 * where it can: freeing a tensor that existed when an unreleased sequence was recorded is
 * refused with YVEX_ERR_STATE (tensors allocated afterwards are free to go), and a replay is
 * refused with YVEX_ERR_STATE unless the workspace that was attached during the recording is
 * still the attached one.
 */
typedef struct yvex_rocm_graph yvex_rocm_graph;
int yvex_backend_rocm_graph_begin(yvex_backend *backend, yvex_error *err);
int yvex_backend_rocm_graph_end(yvex_backend *backend, yvex_rocm_graph **out, yvex_error *err);
int yvex_backend_rocm_graph_launch(yvex_backend *backend, yvex_rocm_graph *graph,
                                   yvex_backend_operation_facts *facts, yvex_error *err);
int yvex_backend_rocm_graph_release(yvex_backend *backend, yvex_rocm_graph **graph,
                                    yvex_error *err);

/* Device-event timing on the backend's stream (cf. yvex_cuda_timing,
 * src/backend/cuda/private.h:421-428).  end() synchronises and returns milliseconds. */
int yvex_backend_rocm_timing_begin(yvex_backend *backend, yvex_error *err);
int yvex_backend_rocm_timing_end(yvex_backend *backend, double *milliseconds, yvex_error *err);

/* Per-kernel device time: while a probe is open, every launch of the named kernel on the
 * backend's stream is bracketed by its own event pair (at most 256 launches; later ones
 * are not measured).  end() synchronises and returns the measured launch count and the
 * sum of their durations.  The name is the kernel symbol in the bundle. */
int yvex_backend_rocm_kernel_probe_begin(yvex_backend *backend, const char *kernel,
                                         yvex_error *err);
int yvex_backend_rocm_kernel_probe_end(yvex_backend *backend, unsigned int *launches,
                                       double *milliseconds, yvex_error *err);

/* Kernel-bundle facts (cf. `inspect backend cuda`, src/backend/core.c:1824-1916). */
typedef struct {
    int driver_loaded, device_ready, bundle_built, bundle_admitted;
    unsigned int image_count, function_count;
    char architecture[32];
    char device_name[128];
    char driver_library[256];
    char rejection[YVEX_ERROR_MESSAGE_CAP];
} yvex_backend_rocm_report;
int yvex_backend_rocm_report_get(const yvex_backend *backend, yvex_backend_rocm_report *out,
                                 yvex_error *err);

/*
 * Immutable backend reports and the inspection commands over them
 * (include/yvex/internal/backend.h:501-533, src/backend/core.c:1824-1916,
 * src/cli/render/backend.c:51-160, src/cli/commands/backend.c:11-52).  The first three report
 * kinds keep the reference's values; the ROCM kinds are the `inspect rocm [bandwidth]`
 * counterparts of the CUDA ones.  A backend that cannot be opened here is reported, not
 * failed: available = 0, the reason text, exit_code 5.  `variants` holds the reference's
 * variants in order, then this backend's attention variants.
 */
#ifndef YVEX_ROCM_IN_TREE
typedef enum {
    YVEX_BACKEND_REPORT_CAPABILITIES = 0,
    YVEX_BACKEND_REPORT_CUDA_INFO,
    YVEX_BACKEND_REPORT_CUDA_BANDWIDTH,
    YVEX_BACKEND_REPORT_ROCM_INFO,
    YVEX_BACKEND_REPORT_ROCM_BANDWIDTH
} yvex_backend_report_kind;
typedef enum {
    YVEX_BACKEND_BUNDLE_NOT_APPLICABLE = 0,
    YVEX_BACKEND_BUNDLE_ABSENT,
    YVEX_BACKEND_BUNDLE_ADMITTED,
    YVEX_BACKEND_BUNDLE_REJECTED
} yvex_backend_bundle_admission;
typedef struct {
    yvex_backend_report_kind kind;
    yvex_backend_kind backend_kind;
} yvex_backend_report_request;
#define YVEX_BACKEND_REPORT_VARIANT_CAP \
    (YVEX_BACKEND_VARIANT_COUNT + (YVEX_BACKEND_VARIANT_ROCM_END - YVEX_BACKEND_VARIANT_ROCM_FIRST))
typedef struct {
    yvex_backend_report_kind kind;
    yvex_backend_kind backend_kind;
    yvex_backend_status backend_status;
    int exit_code, available, has_device_info, kernel_bundle_native;
    yvex_backend_device_info device_info;
    char device_name[128], reason[256], kernel_bundle_architecture[16];
    char kernel_bundle_identity[YVEX_SHA256_HEX_BYTES];
    yvex_backend_memory_stats memory;
    int capabilities[YVEX_BACKEND_CAP_OP_ATTENTION + 1];
    yvex_backend_capability_result variants[YVEX_BACKEND_REPORT_VARIANT_CAP];
    unsigned int variant_count, context_available;
    yvex_backend_bundle_admission bundle_admission;
    yvex_backend_capability_reason bundle_reason;
    yvex_backend_bandwidth_evidence bandwidth;
    unsigned int kernel_image_count, kernel_function_count;
    char driver_library[256];
} yvex_backend_report;
#endif /* !YVEX_ROCM_IN_TREE */
int yvex_backend_report_build(const yvex_backend_report_request *request,
                              yvex_backend_report *report, yvex_error *err);
const char *yvex_backend_bundle_admission_name(yvex_backend_bundle_admission admission);
/* `fp` is a FILE *; declared void * so that this header needs no <stdio.h>. */
int yvex_backend_render(void *fp, const yvex_backend_report *report);
/* Command entry points with the adapter's argv: {program, "backend", "rocm"} and
 * {program, "rocm-info"[, "bandwidth"]}.  They print to stdout (errors to stderr) and return
 * the process exit code: 0, 5 when the backend is unsupported here, 2 for a grammar error
 * (src/cli/io/out.c:1277-1292). */
int yvex_backend_command(int argc, char **argv);
int yvex_rocm_info_command(int argc, char **argv);

/*
 * Sample summary of a component benchmark (include/yvex/internal/benchmark.h:82-97,
 * src/runtime/benchmark.c:388-447,559-573): sorts `seconds` in place, takes nearest-rank
 * percentiles sample[(count * p + 99) / 100 - 1], the mean and the population standard
 * deviation, and stores them as whole nanoseconds.  Samples must be finite and positive.
 */
#ifndef YVEX_ROCM_IN_TREE /* in the tree: include/yvex/internal/benchmark.h */
typedef enum {
    YVEX_RUNTIME_BENCHMARK_MINIMUM = 0,
    YVEX_RUNTIME_BENCHMARK_P50,
    YVEX_RUNTIME_BENCHMARK_P90,
    YVEX_RUNTIME_BENCHMARK_P95,
    YVEX_RUNTIME_BENCHMARK_P99,
    YVEX_RUNTIME_BENCHMARK_MAXIMUM,
    YVEX_RUNTIME_BENCHMARK_MEAN,
    YVEX_RUNTIME_BENCHMARK_STANDARD_DEVIATION,
    YVEX_RUNTIME_BENCHMARK_STATISTIC_COUNT
} yvex_runtime_benchmark_statistic;
typedef struct {
    int available;
    unsigned long long values[YVEX_RUNTIME_BENCHMARK_STATISTIC_COUNT];
} yvex_runtime_benchmark_timing_distribution;
int yvex_runtime_benchmark_samples_summarize(double *seconds, unsigned long long count,
                                             yvex_runtime_benchmark_timing_distribution *out,
                                             yvex_error *err);
/* Field name of a statistic in a benchmark record ("minimum_ns", "p50_ns", ...;
 * src/runtime/benchmark.c:127-140); device timing prefixes it with "device_". */
const char *yvex_runtime_benchmark_statistic_name(yvex_runtime_benchmark_statistic statistic);
#endif

/* ---- scalar and block codecs (host): src/gguf/quant_scalar.c:40-143,
 *      src/gguf/quant_block.c:160-186,819-833 ------------------------------- */
float yvex_quant_f16_decode(unsigned short bits);
unsigned short yvex_quant_f16_encode(float value);
float yvex_quant_bf16_decode(unsigned short bits);
unsigned short yvex_quant_bf16_encode(float value);
#ifndef YVEX_QUANT_Q8_0_ELEMENTS
#define YVEX_QUANT_Q8_0_ELEMENTS 32u
#define YVEX_QUANT_Q8_0_BYTES 34u
#endif
/* Row forms (elements % 32 == 0).  encode refuses an unrepresentable scale with
 * YVEX_ERR_BOUNDS; decode refuses a negative or non-finite scale with YVEX_ERR_FORMAT. */
int yvex_rocm_q8_0_encode_row(const float *source, unsigned long long elements,
                              unsigned char *encoded, yvex_error *err);
int yvex_rocm_q8_0_decode_row(const unsigned char *encoded, unsigned long long elements,
                              float *out, yvex_error *err);

/* ---- host-side page packers (layout only, bytes are moved, never recomputed) ---- */
unsigned long long yvex_rocm_kv_page_block_bytes(yvex_rocm_kv_storage storage,
                                                 unsigned long long head_dimension,
                                                 unsigned long long page_tokens);
/* rows: token-major [pool_pages][page_tokens][kv_heads][row] where row is d bf16 values
 * (BF16) or d/32 canonical 34-byte blocks (Q8_0).  is_value selects the V block layout. */
int yvex_rocm_kv_pack_pages(yvex_rocm_kv_storage storage, int is_value, const void *rows,
                            unsigned long long pool_pages, unsigned long long page_tokens,
                            unsigned long long kv_heads, unsigned long long head_dimension,
                            void *packed, yvex_error *err);
int yvex_rocm_kv_unpack_pages(yvex_rocm_kv_storage storage, int is_value, const void *packed,
                              unsigned long long pool_pages, unsigned long long page_tokens,
                              unsigned long long kv_heads, unsigned long long head_dimension,
                              void *rows, yvex_error *err);

#ifdef __cplusplus
}
#endif

#endif /* YVEX_ROCM_OPERATIONS_H */
