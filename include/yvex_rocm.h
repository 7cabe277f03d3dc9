/*
 * C ABI of the MI355X (gfx950) attention backend for YVEX.
 *
 * Every type and function below either mirrors one interface of the reference
 * tree (cited as path:line, relative to yailabs/clori) with the same name,
 * argument meaning and error behaviour; what the reference has no counterpart for
 * (paged KV, Q8_0 KV, LSE output, absorbed MLA) is declared in
 * yvex_rocm_operations.h and marked NEW SURFACE there.
 * Only plain C types cross this boundary: opaque handles, integers, pointers.
 *
 * The library talks to the HIP runtime through a dlopen'ed function table and
 * loads its gfx950 code objects from an embedded bundle; it never computes
 * attention on the host and has no CPU fallback: when the device, the bundle or
 * an exact implementation is unavailable every operation refuses.
 */
#ifndef YVEX_ROCM_H
#define YVEX_ROCM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Two ways to compile against this header.  By default it is self-contained: the reference's
 * own types are re-declared below with the reference's names, members and values.  With
 * YVEX_ROCM_IN_TREE defined (the ROCm arm built inside the reference tree) those
 * declarations come from the reference's headers instead and this header adds only what the
 * reference lacks; the values the integration adds to the reference's enumerations (the
 * ROCm operation variants, the bf16 numeric contract, the two ROCm report kinds) are given
 * as constants of the enumeration's type until the enumerations themselves carry them.
 * Function declarations are not hidden in either mode: where the reference declares the
 * same function, the compiler holds the two declarations against each other.
 */
#ifdef YVEX_ROCM_IN_TREE
#include <yvex/backend.h>
#include <yvex/internal/backend.h>
#include <yvex/internal/core.h>
#include <yvex/internal/transformer.h>
#ifndef YVEX_BACKEND_VARIANT_ROCM_FIRST
#define YVEX_BACKEND_VARIANT_ROCM_FIRST ((yvex_backend_operation_variant)64)
#define YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32 ((yvex_backend_operation_variant)64)
#define YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16 ((yvex_backend_operation_variant)65)
#define YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16 ((yvex_backend_operation_variant)66)
#define YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0 ((yvex_backend_operation_variant)67)
#define YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16 ((yvex_backend_operation_variant)68)
#define YVEX_BACKEND_VARIANT_ROCM_END ((yvex_backend_operation_variant)69)
#endif
#ifndef YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE
#define YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE \
    ((yvex_transformer_attention_numeric_contract)2)
#endif
#ifndef YVEX_BACKEND_REPORT_ROCM_INFO
#define YVEX_BACKEND_REPORT_ROCM_INFO ((yvex_backend_report_kind)3)
#define YVEX_BACKEND_REPORT_ROCM_BANDWIDTH ((yvex_backend_report_kind)4)
#endif
#endif /* YVEX_ROCM_IN_TREE */

#ifndef YVEX_ROCM_IN_TREE
/* ---- status and error: include/yvex/core.h:13-48 ------------------------ */
typedef enum {
    YVEX_OK = 0,
    YVEX_ERR = -1,
    YVEX_ERR_NOMEM = -2,
    YVEX_ERR_IO = -3,
    YVEX_ERR_FORMAT = -4,
    YVEX_ERR_UNSUPPORTED = -5,
    YVEX_ERR_BACKEND = -6,
    YVEX_ERR_BOUNDS = -7,
    YVEX_ERR_STATE = -8,
    YVEX_ERR_CANCELLED = -9,
    YVEX_ERR_INVALID_ARG = -10,
    YVEX_ERR_TIMEOUT = -11
} yvex_status;

#define YVEX_ERROR_WHERE_CAP 96
#define YVEX_ERROR_MESSAGE_CAP 256

typedef struct {
    yvex_status code;
    char where[YVEX_ERROR_WHERE_CAP];
    char message[YVEX_ERROR_MESSAGE_CAP];
} yvex_error;

const char *yvex_status_name(yvex_status status);
void yvex_error_clear(yvex_error *err);
void yvex_error_set(yvex_error *err, yvex_status code, const char *where, const char *message);

/* ---- dtypes: include/yvex/model.h:19-59 (values are part of the ABI) ----- */
typedef enum {
    YVEX_DTYPE_UNKNOWN = 0,
    YVEX_DTYPE_F32 = 1,
    YVEX_DTYPE_F16 = 2,
    YVEX_DTYPE_BF16 = 3,
    YVEX_DTYPE_F64 = 4,
    YVEX_DTYPE_I8 = 5,
    YVEX_DTYPE_I16 = 6,
    YVEX_DTYPE_I32 = 7,
    YVEX_DTYPE_I64 = 8,
    YVEX_DTYPE_Q8_0 = 13
} yvex_dtype;

#define YVEX_TENSOR_MAX_DIMS 4u

/* ---- backend objects: include/yvex/backend.h:13-140 ---------------------- */
typedef struct yvex_backend yvex_backend;
typedef struct yvex_device_tensor yvex_device_tensor;

typedef enum {
    YVEX_BACKEND_KIND_CPU = 0,
    YVEX_BACKEND_KIND_CUDA,
    YVEX_BACKEND_KIND_METAL,
    YVEX_BACKEND_KIND_ROCM
} yvex_backend_kind;

typedef enum {
    YVEX_BACKEND_STATUS_READY = 0,
    YVEX_BACKEND_STATUS_CONTEXT_READY,
    YVEX_BACKEND_STATUS_UNSUPPORTED,
    YVEX_BACKEND_STATUS_FAILED
} yvex_backend_status;

typedef struct {
    yvex_backend_kind kind;
    const char *device;
    unsigned long long memory_limit_bytes;
} yvex_backend_options;

typedef struct {
    unsigned long long allocated_bytes;
    unsigned long long allocation_count, allocation_events, release_events;
    unsigned long long h2d_bytes, d2h_bytes;
    unsigned long long peak_allocated_bytes;
    unsigned long long memory_limit_bytes;
} yvex_backend_memory_stats;

typedef struct {
    const char *name;
    yvex_dtype dtype;
    unsigned int rank;
    unsigned long long dims[YVEX_TENSOR_MAX_DIMS];
    unsigned long long bytes;
} yvex_backend_tensor_desc;

typedef struct {
    yvex_backend_kind kind;
    const char *name;
    int device_index;
    int compute_capability_major;
    int compute_capability_minor;
    unsigned long long global_memory_bytes;
    unsigned long long free_memory_bytes;
    unsigned long long total_memory_bytes;
    int unified_addressing;
    int managed_memory;
} yvex_backend_device_info;

typedef enum {
    YVEX_BACKEND_CAP_TENSOR_ALLOC = 0,
    YVEX_BACKEND_CAP_TENSOR_READ_WRITE,
    YVEX_BACKEND_CAP_OP_EMBED,
    YVEX_BACKEND_CAP_OP_MATMUL,
    YVEX_BACKEND_CAP_OP_MLP,
    YVEX_BACKEND_CAP_OP_RMS_NORM,
    YVEX_BACKEND_CAP_OP_ROPE,
    YVEX_BACKEND_CAP_OP_ATTENTION
} yvex_backend_capability;

/* Values 0..16 are the reference's (include/yvex/backend.h:72-91).  Values from 64
 * are NEW SURFACE: one variant per attention kernel family of this backend so that a
 * capability query names exactly what is admitted. */
typedef enum {
    YVEX_BACKEND_VARIANT_TENSOR_ALLOC = 0,
    YVEX_BACKEND_VARIANT_TENSOR_ZERO,
    YVEX_BACKEND_VARIANT_TENSOR_WRITE,
    YVEX_BACKEND_VARIANT_TENSOR_READ,
    YVEX_BACKEND_VARIANT_TENSOR_COPY,
    YVEX_BACKEND_VARIANT_EMBED_F32_TO_F32,
    YVEX_BACKEND_VARIANT_EMBED_F16_TO_F32,
    YVEX_BACKEND_VARIANT_RMS_NORM_F32_WEIGHT_F32,
    YVEX_BACKEND_VARIANT_RMS_NORM_F32_WEIGHT_F16,
    YVEX_BACKEND_VARIANT_ROPE_F32,
    YVEX_BACKEND_VARIANT_MATMUL_F32,
    YVEX_BACKEND_VARIANT_MLP_DENSE_F32,
    YVEX_BACKEND_VARIANT_MLP_ROUTED_F32,
    YVEX_BACKEND_VARIANT_ATTENTION_CAUSAL_F32,
    YVEX_BACKEND_VARIANT_ATTENTION_NONCAUSAL_F32,
    YVEX_BACKEND_VARIANT_QTYPE_ROW_DOT,
    YVEX_BACKEND_VARIANT_ATTENTION_ENCODED,
    YVEX_BACKEND_VARIANT_COUNT,
    YVEX_BACKEND_VARIANT_ROCM_FIRST = 64,
    YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32 = 64,
    YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
    YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
    YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0,
    YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16,
    YVEX_BACKEND_VARIANT_ROCM_END
} yvex_backend_operation_variant;

typedef enum {
    YVEX_BACKEND_CAPABILITY_UNSUPPORTED = 0,
    YVEX_BACKEND_CAPABILITY_SUPPORTED,
    YVEX_BACKEND_CAPABILITY_FAILED
} yvex_backend_capability_state;

typedef enum {
    YVEX_BACKEND_CAPABILITY_REASON_NONE = 0,
    YVEX_BACKEND_CAPABILITY_REASON_DRIVER_UNAVAILABLE,
    YVEX_BACKEND_CAPABILITY_REASON_DEVICE_UNAVAILABLE,
    YVEX_BACKEND_CAPABILITY_REASON_CONTEXT_UNAVAILABLE,
    YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT,
    YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_REJECTED,
    YVEX_BACKEND_CAPABILITY_REASON_FUNCTION_MISSING,
    YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED,
    YVEX_BACKEND_CAPABILITY_REASON_LAUNCH_FAILED,
    YVEX_BACKEND_CAPABILITY_REASON_SYNCHRONIZATION_FAILED,
    YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED
} yvex_backend_capability_reason;

typedef struct {
    yvex_backend_kind backend_kind;
    yvex_backend_operation_variant variant;
    yvex_backend_capability_state state;
    yvex_backend_capability_reason reason;
    yvex_dtype input_dtype;
    yvex_dtype weight_dtype;
    yvex_dtype output_dtype;
    int context_available;
    int kernel_bundle_available;
    int function_available;
} yvex_backend_capability_result;

/* include/yvex/internal/backend.h:284-290 */
typedef struct yvex_backend_operation_facts {
    unsigned long long h2d_bytes, d2h_bytes, d2d_bytes, kernel_launches, upload_count;
    unsigned long long download_count, queue_synchronizations, device_synchronizations;
    unsigned long long active_weight_bytes, state_bytes;
    unsigned long long activation_bytes, temporary_bytes, accelerated_matrix_launches;
    int compulsory_memory_facts_available;
} yvex_backend_operation_facts;

/* include/yvex/internal/backend.h:215-228.  Callers may copy a tensor struct and
 * offset `data` to form a sub-view (src/backend/core.c:1763-1778). */
struct yvex_device_tensor {
    yvex_backend *owner;
    unsigned long long owner_id;
    char *name;
    yvex_dtype dtype;
    unsigned int rank;
    unsigned long long dims[YVEX_TENSOR_MAX_DIMS];
    unsigned long long bytes;
    unsigned char *data, *host_data;
    void *backend_allocation;
    unsigned long long resident_bytes;
    int virtual_reserved;
    int is_written, host_accessible, borrowed_host;
};

#endif /* !YVEX_ROCM_IN_TREE */

/* ---- lifecycle: include/yvex/backend.h:143-160, src/backend/core.c:255-416 --- */
/* Opens kind ROCM only; any other kind is YVEX_ERR_UNSUPPORTED ("backend %s is not
 * implemented", src/backend/core.c:280-283).  `device` is NULL / "" / "0".."N". */
int yvex_backend_open(yvex_backend **out, const yvex_backend_options *options, yvex_error *err);
/* The opener the reference's yvex_backend_open would call from its ROCM arm, next to
 * yvex_backend_open_cuda_impl (src/backend/core.c:276-279). */
int yvex_backend_open_rocm_impl(yvex_backend **out, const char *device,
                                unsigned long long memory_limit_bytes, yvex_error *err);
int yvex_backend_rocm_context_available(void);
int yvex_backend_rocm_available(void);
int yvex_backend_close_checked(yvex_backend **backend, yvex_error *err);
void yvex_backend_close(yvex_backend *backend);

yvex_backend_kind yvex_backend_kind_of(const yvex_backend *backend);
const char *yvex_backend_kind_name(yvex_backend_kind kind);
/* src/backend/core.c:204-216, widened to accept "rocm". */
int yvex_backend_kind_parse(const char *name, yvex_backend_kind *out, yvex_error *err);
yvex_backend_status yvex_backend_status_of(const yvex_backend *backend);
const char *yvex_backend_status_name(yvex_backend_status status);
int yvex_backend_get_memory_stats(const yvex_backend *backend, yvex_backend_memory_stats *out,
                                  yvex_error *err);
int yvex_backend_get_device_info(const yvex_backend *backend, yvex_backend_device_info *out,
                                 yvex_error *err);

/* ---- tensors: include/yvex/backend.h:169-199, src/backend/core.c:1143-1290 ---- */
int yvex_backend_tensor_alloc(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                              yvex_device_tensor **out, yvex_error *err);
void yvex_backend_tensor_free(yvex_backend *backend, yvex_device_tensor *tensor);
int yvex_backend_tensor_release(yvex_backend *backend, yvex_device_tensor **tensor,
                                yvex_error *err);
/* Virtual-range tensors (include/yvex/internal/backend.h:479-483, dispatch
 * src/backend/core.c:613-680, device side src/backend/cuda/backend.c:500-834): the tensor
 * owns a stable device address range of desc->bytes and no memory; commit_range backs the
 * granules (of *granularity bytes) that intersect [offset, offset+bytes) and are not backed
 * yet, zero-filled, and reports their bytes; it is idempotent and all-or-nothing, and only
 * committed bytes count against the memory limit.  decommit returns every page and keeps
 * the range; release returns both.  This is how the reference holds a layer's attention
 * history that grows with the sequence (src/runtime/state_residency.c:258-287,441-446).
 * A tensor or view handed to any operation of this backend must lie on committed pages,
 * else YVEX_ERR_STATE.  Refusals: INVALID_ARG (missing argument, empty or out-of-range
 * span, foreign or non-virtual tensor), STATE (backend failed / closing / recording),
 * UNSUPPORTED (runtime or device without virtual memory management), NOMEM (limit). */
/* include/yvex/internal/backend.h:257, src/backend/residency.c:12-17: what the caller asks
 * before it plans a paged history (src/runtime/state_residency.c:593). */
int yvex_backend_virtual_tensor_supported(const yvex_backend *backend);
int yvex_backend_tensor_reserve(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                                yvex_device_tensor **out, unsigned long long *granularity,
                                yvex_error *err);
int yvex_backend_tensor_commit_range(yvex_backend *backend, yvex_device_tensor *tensor,
                                     unsigned long long offset, unsigned long long bytes,
                                     unsigned long long *resident_delta, yvex_error *err);
int yvex_backend_tensor_decommit(yvex_backend *backend, yvex_device_tensor *tensor,
                                 unsigned long long *released_bytes, yvex_error *err);
const char *yvex_device_tensor_name(const yvex_device_tensor *tensor);
unsigned long long yvex_device_tensor_bytes(const yvex_device_tensor *tensor);
int yvex_device_tensor_is_written(const yvex_device_tensor *tensor);
int yvex_backend_tensor_write(yvex_backend *backend, yvex_device_tensor *tensor, const void *src,
                              unsigned long long len, yvex_error *err);
int yvex_backend_tensor_read(yvex_backend *backend, const yvex_device_tensor *tensor, void *dst,
                             unsigned long long len, yvex_error *err);
int yvex_backend_tensor_zero(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err);
int yvex_backend_tensor_copy(yvex_backend *backend, yvex_device_tensor *dst,
                             const yvex_device_tensor *src, yvex_error *err);
/* include/yvex/internal/backend.h (dispatch src/backend/core.c:822-840, vtable slot
 * src/backend/private.h:45-46, CUDA arm src/backend/cuda/backend.c:1159-1191): the copy is
 * put on the backend's launch stream and not waited for, so the kernels enqueued after it see
 * the rows without a synchronisation in between.  This is the call the session layer makes
 * twice per token when it appends a step's keys and values to the history
 * (src/runtime/stateful_attention.c:206,215).  Refusals in the reference's order: lifecycle
 * (YVEX_ERR_STATE), ownership (YVEX_ERR_STATE), descriptors that differ (YVEX_ERR_BOUNDS). */
int yvex_backend_tensor_copy_async(yvex_backend *backend, yvex_device_tensor *destination,
                                   const yvex_device_tensor *source, yvex_error *err);
/* src/backend/core.c:842-874, src/backend/private.h:47-48, CUDA arm
 * src/backend/cuda/backend.c:1194-1265: copy between two backends that share one physical
 * owner (a primary backend and the session backends opened on it), ordered by events: the
 * executor's stream waits for the source's stream before the copy, the source's stream waits
 * for the copy before it goes on. */
int yvex_backend_tensor_copy_shared_async(yvex_backend *executor, yvex_device_tensor *destination,
                                          const yvex_device_tensor *source, yvex_error *err);
/* include/yvex/internal/backend.h:205-206 (src/backend/cuda/backend.c:1795-1879): a session
 * backend on the device of a primary one: its own launch stream, timing events, workspace,
 * kernel functions, arrival counters and status word, memory accounted against its own limit.
 * The primary holds a lease per session backend and cannot be closed while one is open
 * (YVEX_ERR_STATE from the close, the handle is retained).  The only thing backends of one
 * device share is the fixed scratch of yvex_backend_rocm_paged_decode_execute_static. */
int yvex_backend_open_shared_rocm(yvex_backend **out, yvex_backend *context_owner,
                                  unsigned long long memory_limit_bytes, yvex_error *err);
int yvex_backend_tensor_owned_by(const yvex_backend *backend, const yvex_device_tensor *tensor);
/* src/backend/core.c:1763-1778: rank-1 F32 view of `count` elements at `offset`. */
int yvex_backend_tensor_f32_subview(const yvex_device_tensor *source, unsigned long long offset,
                                    unsigned long long count, yvex_device_tensor *view);
int yvex_backend_sync(yvex_backend *backend, yvex_error *err);

/* ---- capability: include/yvex/backend.h:201-213, src/backend/cuda/capability.c:622-760 */
int yvex_backend_supports(const yvex_backend *backend, yvex_backend_capability capability);
const char *yvex_backend_capability_name(yvex_backend_capability capability);
int yvex_backend_query_capability(const yvex_backend *backend,
                                  yvex_backend_operation_variant variant,
                                  yvex_backend_capability_result *out, yvex_error *err);
const char *yvex_backend_operation_variant_name(yvex_backend_operation_variant variant);
const char *yvex_backend_capability_state_name(yvex_backend_capability_state state);
const char *yvex_backend_capability_reason_name(yvex_backend_capability_reason reason);

/* ---- reusable device workspace: src/backend/residency.c:207-283 ----------- */
#ifndef YVEX_ROCM_IN_TREE
typedef enum {
    YVEX_BACKEND_RESIDENT_INVALID = -1,
    YVEX_BACKEND_RESIDENT_MISS = 0,
    YVEX_BACKEND_RESIDENT_HIT = 1
} yvex_backend_resident_result;
#endif /* !YVEX_ROCM_IN_TREE */
int yvex_backend_workspace_attach(yvex_backend *backend, const yvex_device_tensor *device_tensor,
                                  unsigned long long generation, yvex_error *err);
void yvex_backend_workspace_detach(yvex_backend *backend);
int yvex_backend_workspace_acquire(yvex_backend *backend, unsigned long long bytes,
                                   unsigned long long alignment,
                                   unsigned long long *device_address);

/* ---- bounded single-head primitive: include/yvex/backend.h:244-255,
 *      src/backend/core.c:1095-1141,1547-1616, src/backend/cuda/ops.c:1717-1807 ---- */
int yvex_backend_op_attention(yvex_backend *backend, const yvex_device_tensor *query,
                              const yvex_device_tensor *keys, const yvex_device_tensor *values,
                              unsigned long long seq_len, unsigned long long position,
                              float scale, int causal, yvex_device_tensor *score_scratch,
                              yvex_device_tensor *probability_scratch, yvex_device_tensor *out,
                              yvex_error *err);

/* ---- multi-token attention contract: include/yvex/internal/transformer.h:245-275 ---- */
#ifndef YVEX_ROCM_IN_TREE
typedef enum {
    YVEX_TRANSFORMER_ATTENTION_LAYOUT_UNKNOWN = 0,
    YVEX_TRANSFORMER_ATTENTION_LAYOUT_TOKEN_HEAD_DIM
} yvex_transformer_attention_layout;
typedef enum {
    YVEX_TRANSFORMER_ATTENTION_MASK_UNKNOWN = 0,
    YVEX_TRANSFORMER_ATTENTION_MASK_FULL,
    YVEX_TRANSFORMER_ATTENTION_MASK_CAUSAL
} yvex_transformer_attention_mask;
/* EXACT_F32 is the reference's only contract.  BF16_F32_ACCUMULATE is NEW SURFACE:
 * bf16 Q/K/V/output, fp32 scores, fp32 online softmax, fp32 accumulation, MFMA
 * products; it is never substituted for EXACT_F32 (a request states its contract and
 * is refused when that contract is not admitted). */
typedef enum {
    YVEX_TRANSFORMER_ATTENTION_NUMERIC_UNKNOWN = 0,
    YVEX_TRANSFORMER_ATTENTION_NUMERIC_EXACT_F32,
    YVEX_TRANSFORMER_ATTENTION_NUMERIC_BF16_F32_ACCUMULATE
} yvex_transformer_attention_numeric_contract;

typedef struct yvex_transformer_attention_requirement {
    unsigned long long query_tokens, key_value_tokens, query_start;
    unsigned long long query_heads, key_value_heads, head_dimension;
    /* 0 = packed; otherwise elements (of the tensor's dtype) per token */
    unsigned long long query_token_stride, key_token_stride, value_token_stride;
    yvex_dtype query_dtype, key_dtype, value_dtype, output_dtype;
    yvex_transformer_attention_layout layout;
    yvex_transformer_attention_mask mask;
    yvex_transformer_attention_numeric_contract numeric_contract;
    int deterministic;
} yvex_transformer_attention_requirement;

typedef struct yvex_transformer_attention_request {
    yvex_transformer_attention_requirement requirement;
    const yvex_device_tensor *query, *key, *value;
    yvex_device_tensor *output;
} yvex_transformer_attention_request;

/* struct yvex_backend_transformer_operations, include/yvex/internal/transformer.h:276-339:
 * every member of the reference table, in the reference's order and with the reference's
 * signatures, so that a caller compiled against the reference header finds
 * attention_workspace_required and attention_execute at the same offsets in the table
 * this backend returns.  Published by this backend: the two attention slots and the four
 * element-wise slots the reference's decoder calls around them on F32 activations
 * (src/runtime/decoder.c:989-997,1112-1131,1225-1270): rotary_half_f32 (the plain F32
 * rotate-half, src/backend/cuda/transformer.c:460-470), split_interleaved_two_f32
 * (src/backend/cuda/decoder.c:11-73), sigmoid_product_bf16 (src/backend/cuda/decoder.c:75-130)
 * and bf16_round (src/backend/cuda/transformer.c:1356-1392), each with the reference's
 * validation (YVEX_ERR_FORMAT for anything but packed, written F32 tensors of this backend
 * with the declared counts; bf16_round also for a value that is not finite).  The request/plan
 * types of the slots this backend does not publish are opaque here (only pointers to them
 * cross the boundary); those slots are NULL in the ROCm table, which the reference's callers
 * treat as "not published" and refuse with YVEX_ERR_UNSUPPORTED
 * (src/runtime/stateful_attention.c:294-298). */
typedef struct yvex_gated_delta_plan yvex_gated_delta_plan;
typedef struct yvex_gated_delta_device_request yvex_gated_delta_device_request;
typedef struct yvex_gated_delta_device_result yvex_gated_delta_device_result;
typedef struct yvex_transformer_linear_compile_request yvex_transformer_linear_compile_request;
typedef struct yvex_transformer_linear_executable yvex_transformer_linear_executable;
typedef struct yvex_transformer_linear_executable_summary yvex_transformer_linear_executable_summary;
typedef struct yvex_transformer_linear_execution_request yvex_transformer_linear_execution_request;
typedef struct yvex_transformer_dense_decoder_request yvex_transformer_dense_decoder_request;
typedef struct yvex_transformer_dense_decoder_result yvex_transformer_dense_decoder_result;
typedef struct yvex_backend_transformer_operations {
    int (*initial)(yvex_backend *, const yvex_device_tensor *, unsigned int, unsigned long long,
                   unsigned long long, unsigned long long, yvex_device_tensor *,
                   yvex_device_tensor *, yvex_backend_operation_facts *, yvex_error *);
    int (*feature_mean)(yvex_backend *, const yvex_device_tensor *, unsigned long long,
                        unsigned long long, unsigned long long, yvex_device_tensor *,
                        yvex_device_tensor *, unsigned long long, unsigned long long,
                        unsigned long long, float *, yvex_backend_operation_facts *, yvex_error *);
    int (*final)(yvex_backend *, const yvex_device_tensor *, const yvex_device_tensor *,
                 const yvex_device_tensor *, const yvex_device_tensor *, const yvex_device_tensor *,
                 unsigned long long, unsigned long long, unsigned long long, double, double,
                 yvex_device_tensor *, yvex_device_tensor *, yvex_backend_operation_facts *,
                 yvex_error *);
    int (*attention_workspace_required)(const yvex_transformer_attention_requirement *,
                                        unsigned long long *, yvex_error *);
    int (*attention_execute)(yvex_backend *, const yvex_transformer_attention_request *,
                             yvex_backend_operation_facts *, yvex_error *);
    int (*gated_delta_workspace_required)(const yvex_gated_delta_plan *, unsigned long long,
                                          unsigned long long *, yvex_error *);
    int (*gated_delta_execute)(yvex_backend *, const yvex_gated_delta_plan *,
                               const yvex_gated_delta_device_request *,
                               yvex_gated_delta_device_result *, yvex_backend_operation_facts *,
                               yvex_error *);
    int (*linear_workspace_required)(const yvex_transformer_linear_compile_request *,
                                     unsigned long long *, yvex_error *);
    int (*linear_compile)(yvex_backend *, const yvex_transformer_linear_compile_request *,
                          yvex_transformer_linear_executable **,
                          yvex_transformer_linear_executable_summary *, yvex_error *);
    int (*linear_execute)(yvex_backend *, const yvex_transformer_linear_execution_request *,
                          yvex_backend_operation_facts *, yvex_error *);
    int (*linear_summary)(const yvex_transformer_linear_executable *,
                          yvex_transformer_linear_executable_summary *, yvex_error *);
    int (*linear_release)(yvex_backend *, yvex_transformer_linear_executable **, yvex_error *);
    int (*rotary_half_f32)(yvex_backend *, yvex_device_tensor *, const yvex_device_tensor *,
                           const yvex_device_tensor *, unsigned long long, unsigned long long,
                           unsigned long long, unsigned long long, yvex_backend_operation_facts *,
                           yvex_error *);
    int (*split_interleaved_two_f32)(yvex_backend *, const yvex_device_tensor *,
                                     yvex_device_tensor *, yvex_device_tensor *, unsigned long long,
                                     unsigned long long, unsigned long long,
                                     yvex_backend_operation_facts *, yvex_error *);
    int (*silu_product_bf16)(yvex_backend *, const yvex_device_tensor *, const yvex_device_tensor *,
                             yvex_device_tensor *, unsigned long long,
                             yvex_backend_operation_facts *, yvex_error *);
    int (*sigmoid_product_bf16)(yvex_backend *, const yvex_device_tensor *,
                                const yvex_device_tensor *, yvex_device_tensor *, unsigned long long,
                                yvex_backend_operation_facts *, yvex_error *);
    int (*add_bf16)(yvex_backend *, const yvex_device_tensor *, const yvex_device_tensor *,
                    yvex_device_tensor *, unsigned long long, unsigned long long,
                    yvex_backend_operation_facts *, yvex_error *);
    int (*bf16_round)(yvex_backend *, yvex_device_tensor *, unsigned long long,
                      yvex_backend_operation_facts *, yvex_error *);
    int (*dense_decoder_execute)(yvex_backend *, const yvex_transformer_dense_decoder_request *,
                                 yvex_transformer_dense_decoder_result *, yvex_error *);
} yvex_backend_transformer_operations;
#endif /* !YVEX_ROCM_IN_TREE */
/* include/yvex/internal/backend.h:211-212; NULL when the kernel bundle is not admitted. */
const yvex_backend_transformer_operations *yvex_backend_transformer_operations_get(
    const yvex_backend *backend);

/* ---- encoded attention transaction: include/yvex/internal/backend.h:143-198,
 *      src/backend/cuda/attention.c:1915-1990, attention_completion.c:110-160 ----
 * The reference's whole-layer DeepSeek attention job (projections, compressor, indexer,
 * reduce, output) behind one symbol.  This backend owns only the reduce stage
 * (mla_decode_execute below), so the symbol is exported and fails closed: the failure
 * record says CAPABILITY at stage "rocm.attention.encoded" and the status is
 * YVEX_ERR_UNSUPPORTED, the same answer query_capability gives for
 * YVEX_BACKEND_VARIANT_ATTENTION_ENCODED.  Nothing of the job is read and `output` is left
 * untouched, so the job and output records stay opaque here. */
#ifndef YVEX_ROCM_IN_TREE
typedef struct yvex_backend_attention_job yvex_backend_attention_job;
typedef struct yvex_backend_attention_output yvex_backend_attention_output;
typedef struct yvex_backend_attention_completion yvex_backend_attention_completion;
typedef enum {
    YVEX_BACKEND_ATTENTION_FAILURE_NONE = 0,
    YVEX_BACKEND_ATTENTION_FAILURE_INVALID_ARGUMENT,
    YVEX_BACKEND_ATTENTION_FAILURE_CAPABILITY,
    YVEX_BACKEND_ATTENTION_FAILURE_BUDGET,
    YVEX_BACKEND_ATTENTION_FAILURE_ALLOCATION,
    YVEX_BACKEND_ATTENTION_FAILURE_COPY,
    YVEX_BACKEND_ATTENTION_FAILURE_LAUNCH,
    YVEX_BACKEND_ATTENTION_FAILURE_SYNCHRONIZE,
    YVEX_BACKEND_ATTENTION_FAILURE_NUMERIC,
    YVEX_BACKEND_ATTENTION_FAILURE_CANCELLED,
    YVEX_BACKEND_ATTENTION_FAILURE_CLEANUP
} yvex_backend_attention_failure_code;
typedef struct {
    yvex_backend_attention_failure_code code;
    const char *stage;
    unsigned long long expected, actual;
} yvex_backend_attention_failure;
#endif /* !YVEX_ROCM_IN_TREE */
int yvex_backend_attention_execute(yvex_backend *backend, const yvex_backend_attention_job *job,
                                   yvex_backend_attention_output *output,
                                   yvex_backend_attention_failure *failure, yvex_error *err);
int yvex_backend_attention_complete(yvex_backend *backend,
                                    yvex_backend_attention_completion *completion,
                                    int barrier_observed, yvex_error *err);

/* The operations the reference has no counterpart for (paged KV, Q8_0 KV, LSE output, absorbed MLA,
 * the fused writers), the benchmark record and the host-side codecs and page packers are declared
 * in yvex_rocm_operations.h, which builds on this header. */

#ifdef __cplusplus
}
#endif

#endif /* YVEX_ROCM_H */
