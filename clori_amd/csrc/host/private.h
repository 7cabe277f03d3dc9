/* Source-local ABI shared by the dispatch layer and the ROCm backend arm.
 * Field names of struct yvex_backend follow src/backend/private.h:83-110 of the
 * reference for every field this path touches, so the ROCm arm reads the same
 * members it would read inside the reference tree. */
#ifndef YVEX_ROCM_HOST_PRIVATE_H
#define YVEX_ROCM_HOST_PRIVATE_H

#include <limits.h>
#include <stdatomic.h>
#include <stdint.h>

#ifdef YVEX_ROCM_IN_TREE
/* Inside the reference tree (the root of the tree on the include path, as for the CUDA arm)
 * the backend object, the vtable and the helpers below are the tree's own; what remains is
 * the one function of the dispatch layer the arm calls that the tree keeps private to its
 * CUDA arm (src/backend/cuda/backend.c:1598-1623). */
#include "src/backend/private.h"
#include <yvex/internal/core.h>
#include "yvex_rocm.h"
#include "yvex_rocm_operations.h"
int yvex_backend_shared_owner_acquire(yvex_backend *owner, yvex_error *err);
#else

#include "yvex_rocm.h"
#include "yvex_rocm_operations.h"

/* The slots of the reference vtable (src/backend/private.h:16-81) that lie on the
 * attention path, under the reference's names.  Everything else (embed, matmul, MoE,
 * sampling, ...) is not published by this backend: its dispatchers answer
 * YVEX_ERR_UNSUPPORTED.  There is no slot the reference's table lacks: the operations that
 * have no reference counterpart are reached through
 * yvex_backend_rocm_attention_operations_get, which belongs to the ROCm arm and tests the
 * backend's kind itself. */
typedef struct yvex_backend_vtable {
    int (*close)(yvex_backend *, yvex_error *);
    int (*memory_stats)(const yvex_backend *, yvex_backend_memory_stats *, yvex_error *);
    int (*device_info)(const yvex_backend *, yvex_backend_device_info *, yvex_error *);
    int (*tensor_alloc)(yvex_backend *, const yvex_backend_tensor_desc *, yvex_device_tensor **,
                        yvex_error *);
    int (*tensor_reserve)(yvex_backend *, const yvex_backend_tensor_desc *, yvex_device_tensor **,
                          unsigned long long *, yvex_error *);
    int (*tensor_commit)(yvex_backend *, yvex_device_tensor *, unsigned long long,
                         unsigned long long, unsigned long long *, yvex_error *);
    int (*tensor_decommit)(yvex_backend *, yvex_device_tensor *, unsigned long long *,
                           yvex_error *);
    int (*tensor_free)(yvex_backend *, yvex_device_tensor *, yvex_error *);
    int (*tensor_write)(yvex_backend *, yvex_device_tensor *, const void *, unsigned long long,
                        yvex_error *);
    int (*tensor_read)(yvex_backend *, const yvex_device_tensor *, void *, unsigned long long,
                       yvex_error *);
    int (*tensor_zero)(yvex_backend *, yvex_device_tensor *, yvex_error *);
    int (*tensor_copy)(yvex_backend *, yvex_device_tensor *, const yvex_device_tensor *,
                       yvex_error *);
    int (*tensor_copy_async)(yvex_backend *, yvex_device_tensor *, const yvex_device_tensor *,
                             yvex_error *);
    int (*tensor_copy_shared_async)(yvex_backend *, yvex_device_tensor *,
                                    const yvex_device_tensor *, yvex_error *);
    int (*sync)(yvex_backend *, yvex_error *);
    int (*bandwidth_probe)(yvex_backend *, yvex_backend_bandwidth_evidence *, yvex_error *);
    int (*query_capability)(const yvex_backend *, yvex_backend_operation_variant,
                            yvex_backend_capability_result *, yvex_error *);
    int (*op_attention)(yvex_backend *, const yvex_device_tensor *, const yvex_device_tensor *,
                        const yvex_device_tensor *, unsigned long long, unsigned long long, float,
                        int, yvex_device_tensor *, yvex_device_tensor *, yvex_device_tensor *,
                        yvex_error *);
    const yvex_backend_transformer_operations *(*transformer_operations)(const yvex_backend *);
} yvex_backend_vtable;

struct yvex_backend {
    yvex_backend_kind kind;
    _Atomic(yvex_backend_status) status;
    const yvex_backend_vtable *vtable;
    yvex_backend_memory_stats stats;
    yvex_backend_device_info device_info;
    char device_name_storage[128];
    void *impl;
    struct yvex_backend *resource_owner; /* itself for a primary backend, the primary for a session backend */
    _Atomic unsigned long long lifecycle; /* CLOSING bit, below it the count of open session backends */
    unsigned long long tensor_id_next;
    const yvex_device_tensor *workspace_device_tensor;
    unsigned long long workspace_device_address, workspace_bytes, workspace_cursor;
    unsigned long long workspace_peak, workspace_generation;
    int shared_owner_registered; /* this session backend holds a lease on resource_owner */
    int virtual_tensor_ready; /* src/backend/private.h:109 */
};

#define YVEX_BACKEND_LIFECYCLE_CLOSING (1ull << 63)
#define YVEX_BACKEND_LIFECYCLE_CHILD_MASK (YVEX_BACKEND_LIFECYCLE_CLOSING - 1ull)

static inline int backend_cleanup_only(const yvex_backend *backend)
{
    return backend && (atomic_load_explicit(&backend->lifecycle, memory_order_acquire) &
                       YVEX_BACKEND_LIFECYCLE_CLOSING) != 0ull;
}

/* src/backend/private.h:122-132 */
static inline int backend_dispatch_admit(const yvex_backend *backend, const char *where,
                                         yvex_error *err)
{
    if (!backend || backend_cleanup_only(backend) ||
        backend->status == YVEX_BACKEND_STATUS_FAILED) {
        yvex_error_set(err, YVEX_ERR_STATE, where, "backend is retained for cleanup only");
        return YVEX_ERR_STATE;
    }
    return YVEX_OK;
}

static inline int backend_tensor_owner_is(const yvex_backend *backend,
                                          const yvex_device_tensor *tensor)
{
    return backend && tensor && tensor->owner == backend && tensor->owner_id != 0ull;
}

static inline void backend_memory_acquire(yvex_backend *backend, unsigned long long bytes)
{
    backend->stats.allocated_bytes += bytes;
    backend->stats.allocation_count += 1ull;
    backend->stats.allocation_events += 1ull;
    if (backend->stats.allocated_bytes > backend->stats.peak_allocated_bytes)
        backend->stats.peak_allocated_bytes = backend->stats.allocated_bytes;
}

static inline void backend_memory_release(yvex_backend *backend, unsigned long long bytes)
{
    backend->stats.allocated_bytes =
        backend->stats.allocated_bytes >= bytes ? backend->stats.allocated_bytes - bytes : 0ull;
    if (backend->stats.allocation_count > 0ull) {
        backend->stats.allocation_count -= 1ull;
        backend->stats.release_events += 1ull;
    }
}

static inline void backend_workspace_reset(yvex_backend *backend)
{
    if (backend) backend->workspace_cursor = 0ull;
}

/* status.c */
int yvex_core_u64_add(unsigned long long left, unsigned long long right,
                      unsigned long long *out);
int yvex_core_u64_mul(unsigned long long left, unsigned long long right,
                      unsigned long long *out);
void yvex_core_text_copy(char *destination, size_t capacity, const char *source);
void yvex_error_setf(yvex_error *err, yvex_status code, const char *where, const char *fmt, ...);

/* core.c: lease of a session backend on its primary (src/backend/cuda/backend.c:1598-1623) */
int yvex_backend_shared_owner_acquire(yvex_backend *owner, yvex_error *err);

/* core.c: shared validators (src/backend/core.c:1143-1171,1224-1290,1547-1616) */
int yvex_backend_memory_can_add(const yvex_backend *backend, unsigned long long bytes,
                                const char *backend_name, const char *where, yvex_error *err);
int yvex_backend_tensor_rw_validate(const char *where, const yvex_backend *backend,
                                    const yvex_device_tensor *tensor, unsigned long long len,
                                    yvex_error *err);
int yvex_backend_tensor_copy_validate(const yvex_backend *backend, const yvex_device_tensor *dst,
                                      const yvex_device_tensor *src, const char *where,
                                      yvex_error *err);
int yvex_backend_validate_attention(const yvex_backend *backend, const yvex_device_tensor *query,
                                    const yvex_device_tensor *keys,
                                    const yvex_device_tensor *values, unsigned long long seq_len,
                                    unsigned long long position,
                                    yvex_device_tensor *score_scratch,
                                    yvex_device_tensor *probability_scratch,
                                    yvex_device_tensor *out, unsigned long long *head_dim_out,
                                    unsigned long long *kv_elements_out, const char *where,
                                    yvex_error *err);

#endif /* !YVEX_ROCM_IN_TREE */

#endif /* YVEX_ROCM_HOST_PRIVATE_H */
