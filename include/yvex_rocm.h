/*
 * C ABI of the MI355X (gfx950) attention backend for YVEX.
 *
 * Every type and function below either mirrors one interface of the reference
 * tree (cited as path:line, relative to yailabs/clori) with the same name,
 * argument meaning and error behaviour, or is marked NEW SURFACE where the
 * reference has no counterpart (paged KV, Q8_0 KV, LSE output, absorbed MLA).
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

#endif /* YVEX_ROCM_H */
