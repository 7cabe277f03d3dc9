/* State of one ROCm backend instance, shared by the arm's translation units. */
#ifndef YVEX_ROCM_STATE_H
#define YVEX_ROCM_STATE_H

#include "private.h"
#include "rocm_driver.h"
#include "../kernel_params.h"

#define YVEX_ROCM_MODULE_MAX 8u

/* Every device function of the bundle.  The order indexes yvex_rocm_backend_state.functions
 * and the binding table in rocm_capability.c. */
typedef enum {
    YVEX_ROCM_FN_ATTENTION_F32 = 0,
    YVEX_ROCM_FN_GQA_F32,
    YVEX_ROCM_FN_GQA_F32_SPLIT,
    YVEX_ROCM_FN_GQA_F32_SPLIT_WIDE,
    YVEX_ROCM_FN_GQA_F32_TILE_64,
    YVEX_ROCM_FN_GQA_F32_TILE_128,
    YVEX_ROCM_FN_GQA_F32_TILE_256,
    YVEX_ROCM_FN_FILL_U32,
    YVEX_ROCM_FN_DECODE_PAGED_BF16,
    YVEX_ROCM_FN_DECODE_PAGED_BF16_64,
    YVEX_ROCM_FN_DECODE_PAGED_BF16_256,
    YVEX_ROCM_FN_DECODE_ROWS_BF16,
    YVEX_ROCM_FN_DECODE_MERGE,
    YVEX_ROCM_FN_DECODE_MERGE_ROPE,
    YVEX_ROCM_FN_DECODE_FINISH,
    YVEX_ROCM_FN_DECODE_FINISH_256,
    YVEX_ROCM_FN_DECODE_PAGED_Q8_0,
    YVEX_ROCM_FN_DECODE_PAGED_BF16_MERGED,
    YVEX_ROCM_FN_DECODE_PAGED_Q8_0_MERGED,
    YVEX_ROCM_FN_DECODE_ROWS_BF16_MERGED,
    YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM,
    YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM_64,
    YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM_256,
    YVEX_ROCM_FN_PREFILL_BF16,
    YVEX_ROCM_FN_PREFILL_BF16_64,
    YVEX_ROCM_FN_PREFILL_BF16_256,
    YVEX_ROCM_FN_MLA_DECODE_BF16,
    YVEX_ROCM_FN_MLA_DECODE_512_BF16,
    YVEX_ROCM_FN_KV_APPEND_BF16,
    YVEX_ROCM_FN_KV_APPEND_BF16_64,
    YVEX_ROCM_FN_KV_APPEND_BF16_256,
    YVEX_ROCM_FN_KV_APPEND_Q8_0,
    YVEX_ROCM_FN_HISTORY_APPEND_BF16,
    YVEX_ROCM_FN_HISTORY_APPEND_F32,
    YVEX_ROCM_FN_STREAM_READ,
    YVEX_ROCM_FN_ROTARY_HALF_PLAIN_F32,
    YVEX_ROCM_FN_BF16_ROUND_F32,
    YVEX_ROCM_FN_SIGMOID_PRODUCT_BF16_F32,
    YVEX_ROCM_FN_SPLIT_INTERLEAVED_TWO_F32,
    YVEX_ROCM_FN_STATUS_FORWARD,
    YVEX_ROCM_FN_COPY_BATCH,
    YVEX_ROCM_FN_SMALL_WRITE,
    YVEX_ROCM_FN_SMALL_READ,
    YVEX_ROCM_FN_GATHER_ROWS,
    YVEX_ROCM_FN_COUNT
} yvex_rocm_function_id;

#define YVEX_ROCM_PROBE_MAX 256u
/* (session, kv head) segments one split-K decode launch may have: one arrival counter each */
#define YVEX_ROCM_DECODE_SEGMENTS_MAX (1u << 18)

typedef enum {
    YVEX_ROCM_KERNEL_BUNDLE_ABSENT = 0,
    YVEX_ROCM_KERNEL_BUNDLE_ADMITTED,
    YVEX_ROCM_KERNEL_BUNDLE_REJECTED
} yvex_rocm_kernel_bundle_state;

/* What decides the item lists of a causal launch (rocm_schedule.c); zero the padding, the key
 * is compared as bytes. */
#define YVEX_ROCM_LISTS_MAX 512u
#define YVEX_ROCM_LIST_STRIDE 8u
#define YVEX_ROCM_LIST_ITEMS_MAX 2048u
typedef struct {
    unsigned long long query_tokens, kv_tokens, query_start;
    uint32_t query_heads;
    uint32_t item_rows;  /* query rows of an item */
    uint32_t step_keys;  /* keys of one step of an item's walk */
    uint32_t per_unit;   /* workgroups of the kernel that fit a compute unit */
    uint32_t kind, reserved; /* kernel family the lists are for */
} yvex_rocm_schedule_key;

typedef struct yvex_rocm_backend_state {
    yvex_rocm_driver driver;
    int device_index;
    int compute_units;
    hipStream_t stream_handle; /* work goes through yvex_rocm_stream(), which orders it behind queued copies */
    /* small asynchronous device-to-device copies wait here to leave as one launch: the
     * kernel's parameter block, how many entries it holds and the largest of them */
    struct {
        yvex_rocm_copy_batch_params params;
        uint32_t count, largest;
        int failed; /* a queued copy could not be issued: reported by the next wait */
    } copy_queue;
    hipEvent_t timing_start, timing_stop;
    int timing_active;
    /* per-kernel probe: event pairs around launches of one function */
    hipEvent_t probe_events[2 * YVEX_ROCM_PROBE_MAX];
    unsigned int probe_count;
    int probe_function; /* -1: closed */
    hipModule_t modules[YVEX_ROCM_MODULE_MAX];
    unsigned int module_count;
    hipFunction_t functions[YVEX_ROCM_FN_COUNT];
    yvex_rocm_kernel_bundle_state kernel_bundle_state;
    yvex_backend_capability_reason kernel_bundle_reason;
    yvex_backend_operation_variant kernel_bundle_failure_variant;
    char kernel_bundle_rejection[YVEX_ERROR_MESSAGE_CAP];
    /* per-variant and whole-backend failure reasons (src/backend/cuda/capability.c:447-461) */
    yvex_backend_capability_reason variant_failures[YVEX_BACKEND_VARIANT_ROCM_END];
    yvex_backend_capability_reason backend_failure_reason;
    int32_t *device_status; /* one status word, zero between operations */
    /* the status word's way to the host without a copy: a word of host memory the device can
     * write, its device address, and the sequence number of the last forward asked for */
    volatile uint64_t *status_mailbox;
    uint64_t *status_mailbox_device;
    uint32_t status_sequence;
    /* behind the mailbox in the same allocation: where small tensor reads arrive */
    unsigned char *read_staging, *read_staging_device;
    uint32_t *decode_arrivals; /* YVEX_ROCM_DECODE_SEGMENTS_MAX counters, zero between operations */
    int status_dirty;       /* deferred mode: launches since the last check */
    yvex_rocm_completion_mode completion_mode;
    unsigned long long live_tensors;
    struct yvex_rocm_virtual_range *virtual_ranges; /* every reserved range that is alive */
    int unbacked_view;  /* the last view check failed on uncommitted pages, not on geometry */
    int virtual_memory; /* the runtime and the device can reserve, map and unmap address ranges */
    int recording;                  /* a launch sequence is being recorded on the stream */
    unsigned long long live_graphs; /* recorded sequences not yet released */
    struct yvex_rocm_graph *graphs; /* ... and the list of them */
    unsigned long long recorded_launches; /* kernel launches of the sequence being recorded */
    void *static_scratch;     /* device address of the fixed scratch array on this device, or NULL */
    int static_scratch_error; /* the runtime's code when it could not be resolved */
    /* the item lists of the last scheduled causal launch (rocm_schedule.c): the geometry, how
     * often it came in a row, the rows on the host and on the device */
    struct {
        yvex_rocm_schedule_key key;
        uint32_t lists, seen;
        uint16_t rows[YVEX_ROCM_LISTS_MAX * YVEX_ROCM_LIST_STRIDE];
    } schedule;
    uint16_t *schedule_device;
    int bandwidth_ready; /* the probe ran: later calls return the kept evidence */
    yvex_backend_bandwidth_evidence bandwidth_evidence;
} yvex_rocm_backend_state;

/* A recorded launch sequence (rocm_backend.c). */
struct yvex_rocm_graph {
    hipGraph_t graph;
    hipGraphExec_t executable;
    unsigned long long kernel_launches;
    /* the workspace the recorded launches write their temporaries to */
    unsigned long long workspace_address, workspace_bytes;
    /* tensors with an id below this one existed when the recording ended: the sequence may
     * name any of them */
    unsigned long long tensor_id_mark;
    struct yvex_rocm_graph *next; /* the backend's list of unreleased sequences */
};

/* Bytes of one element of the dtypes a device tensor of this backend can have; 0 for any other. */
static inline unsigned long long yvex_rocm_dtype_bytes(yvex_dtype dtype)
{
    switch (dtype) {
    case YVEX_DTYPE_F32: case YVEX_DTYPE_I32: return 4ull;
    case YVEX_DTYPE_F16: case YVEX_DTYPE_BF16: case YVEX_DTYPE_I16: return 2ull;
    case YVEX_DTYPE_F64: case YVEX_DTYPE_I64: return 8ull;
    case YVEX_DTYPE_I8: return 1ull;
    default: return 0ull;
    }
}

static inline yvex_rocm_backend_state *yvex_rocm_state(const yvex_backend *backend)
{
    return backend && backend->kind == YVEX_BACKEND_KIND_ROCM
               ? (yvex_rocm_backend_state *)backend->impl
               : NULL;
}

/* Launches what the copy queue holds (rocm_backend.c). */
void yvex_rocm_copy_queue_flush(yvex_rocm_backend_state *state);

/* The backend's stream, for work that is ordered behind everything asked for so far: copies
 * that are still queued are launched first.  Every submission and every wait takes the stream
 * from here. */
static inline hipStream_t yvex_rocm_stream(yvex_rocm_backend_state *state)
{
    if (state->copy_queue.count) yvex_rocm_copy_queue_flush(state);
    return state->stream_handle;
}

/* rocm_capability.c */
/* Small transfers by kernel (see kernel_params.h): YVEX_ERR_UNSUPPORTED, with nothing done,
 * when the transfer is not one of them or the backend lacks what they need. */
int yvex_rocm_small_write(yvex_backend *backend, void *dst, const void *src, unsigned long long bytes,
                          const char *where, yvex_error *err);
int yvex_rocm_small_read(yvex_backend *backend, void *dst, const void *src, unsigned long long bytes,
                         const char *where, yvex_error *err);
int yvex_rocm_kernel_bundle_admit(yvex_backend *backend, yvex_error *err);
int yvex_rocm_kernel_bundle_close(yvex_backend *backend, yvex_error *err);
int yvex_rocm_query_capability(const yvex_backend *backend, yvex_backend_operation_variant variant,
                               yvex_backend_capability_result *out, yvex_error *err);
int yvex_rocm_require_capability(yvex_backend *backend, yvex_backend_operation_variant variant,
                                 const char *where, yvex_error *err);
unsigned int yvex_rocm_bundle_image_count(void);
/* One kernel launch on the backend stream; params is the kernel's single argument block. */
int yvex_rocm_function_find(const char *symbol);
int yvex_rocm_launch(yvex_backend *backend, yvex_rocm_function_id function,
                     yvex_backend_operation_variant variant, unsigned int grid_x,
                     unsigned int grid_y, unsigned int grid_z, unsigned int block,
                     unsigned int lds_bytes, void *params, const char *where, yvex_error *err);
/* Stream synchronise; a failure moves the whole backend to FAILED. */
int yvex_rocm_synchronize(yvex_backend *backend, yvex_backend_operation_variant variant,
                          const char *where, yvex_error *err);
/* Ends an operation: IMMEDIATE mode synchronises, reads the device status word and
 * maps it to a status; DEFERRED mode only marks the word as pending. */
int yvex_rocm_complete(yvex_backend *backend, yvex_backend_operation_variant variant,
                       const char *where, yvex_backend_operation_facts *facts, yvex_error *err);
int yvex_rocm_status_check(yvex_backend *backend, const char *where,
                           yvex_backend_operation_facts *facts, yvex_error *err);

/* rocm_backend.c */
int yvex_rocm_temporary_acquire(yvex_backend *backend, unsigned long long bytes, void **address,
                                int *owned, const char *where, yvex_error *err);
int yvex_rocm_temporary_release(yvex_backend *backend, void *address, unsigned long long bytes,
                                int owned, yvex_error *err);

/* rocm_virtual.c: tensors over a reserved address range, backed where committed */
int yvex_rocm_tensor_reserve(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                             yvex_device_tensor **out, unsigned long long *granularity,
                             yvex_error *err);
int yvex_rocm_tensor_commit(yvex_backend *backend, yvex_device_tensor *tensor,
                            unsigned long long offset, unsigned long long bytes,
                            unsigned long long *resident_delta, yvex_error *err);
int yvex_rocm_tensor_decommit(yvex_backend *backend, yvex_device_tensor *tensor,
                              unsigned long long *released_bytes, yvex_error *err);
int yvex_rocm_virtual_release(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err);
/* 1 for an ordinary tensor; for a tensor or view over a reserved range, 1 only when every
 * byte of it lies on committed pages.  Anything handed to the device is checked with it: a
 * read or write of an address without memory behind it is a device fault, not an error code. */
int yvex_rocm_tensor_backed(const yvex_device_tensor *tensor);

/* rocm_attention.c */
int yvex_rocm_op_attention(yvex_backend *backend, const yvex_device_tensor *query,
                           const yvex_device_tensor *keys, const yvex_device_tensor *values,
                           unsigned long long seq_len, unsigned long long position, float scale,
                           int causal, yvex_device_tensor *score_scratch,
                           yvex_device_tensor *probability_scratch, yvex_device_tensor *out,
                           yvex_error *err);
/* rocm_elementwise.c: the element-wise slots of the transformer operations table */
int yvex_rocm_rotary_half_f32(yvex_backend *backend, yvex_device_tensor *values,
                              const yvex_device_tensor *cosines, const yvex_device_tensor *sines,
                              unsigned long long tokens, unsigned long long heads,
                              unsigned long long head_dim, unsigned long long rotary_dim,
                              yvex_backend_operation_facts *facts, yvex_error *err);
int yvex_rocm_bf16_round(yvex_backend *backend, yvex_device_tensor *values, unsigned long long count,
                         yvex_backend_operation_facts *facts, yvex_error *err);
int yvex_rocm_sigmoid_product_bf16(yvex_backend *backend, const yvex_device_tensor *values,
                                   const yvex_device_tensor *gate, yvex_device_tensor *output,
                                   unsigned long long count, yvex_backend_operation_facts *facts,
                                   yvex_error *err);
int yvex_rocm_split_interleaved_two_f32(yvex_backend *backend, const yvex_device_tensor *input,
                                        yvex_device_tensor *first, yvex_device_tensor *second,
                                        unsigned long long rows, unsigned long long heads,
                                        unsigned long long head_dimension,
                                        yvex_backend_operation_facts *facts, yvex_error *err);

/* rocm_schedule.c */
unsigned int yvex_rocm_schedule_lists(yvex_backend *backend, const yvex_rocm_schedule_key *key,
                                      const uint16_t **device_rows);

const yvex_backend_transformer_operations *yvex_rocm_transformer_operations(
    const yvex_backend *backend);
#endif /* YVEX_ROCM_STATE_H */
