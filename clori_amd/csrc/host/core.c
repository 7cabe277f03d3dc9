/* Backend-neutral dispatch for the attention path: argument checks, lifecycle
 * admission and vtable forwarding with the same refusal order and status codes as
 * src/backend/core.c of the reference.  Inside the reference tree this layer is the
 * reference's own core.c; it exists here so the ROCm arm can be used stand-alone. */
#include "private.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define ARRAY_COUNT(a) (sizeof(a) / sizeof((a)[0]))

static const char *const kind_names[] = {"cpu", "cuda", "metal", "rocm"};
static const char *const status_names[] = {"ready", "context-ready", "unsupported", "failed"};
static const char *const variant_names[YVEX_BACKEND_VARIANT_COUNT] = {
    "tensor-alloc", "tensor-zero", "tensor-write", "tensor-read", "tensor-copy",
    "embed-f32-to-f32", "embed-f16-to-f32", "rms-norm-f32-weight-f32",
    "rms-norm-f32-weight-f16", "rope-f32", "matmul-f32", "mlp-dense-f32", "mlp-routed-f32",
    "attention-causal-f32", "attention-noncausal-f32", "qtype-row-dot", "encoded-attention"};
static const char *const rocm_variant_names[] = {
    "rocm-attention-gqa-f32", "rocm-attention-gqa-bf16", "rocm-attention-paged-bf16",
    "rocm-attention-paged-q8-0", "rocm-attention-mla-bf16"};
static const char *const capability_state_names[] = {"unsupported", "supported", "failed"};
static const char *const capability_reason_names[] = {
    "none", "driver-unavailable", "device-unavailable", "context-unavailable",
    "kernel-bundle-absent", "kernel-bundle-rejected", "required-function-missing",
    "variant-unsupported", "launch-failed", "synchronization-failed", "cleanup-failed"};
static const char *const capability_names[] = {
    "tensor_alloc", "tensor_read_write", "op_embed", "op_matmul",
    "op_mlp", "op_rms_norm", "op_rope", "op_attention"};

static const char *name_at(const char *const *names, size_t count, unsigned int index)
{
    return index < count ? names[index] : "unknown";
}

static int refuse(yvex_error *err, yvex_status status, const char *where, const char *reason)
{
    yvex_error_set(err, status, where, reason);
    return status;
}

const char *yvex_backend_kind_name(yvex_backend_kind kind)
{
    return name_at(kind_names, ARRAY_COUNT(kind_names), (unsigned int)kind);
}

const char *yvex_backend_status_name(yvex_backend_status status)
{
    return name_at(status_names, ARRAY_COUNT(status_names), (unsigned int)status);
}

const char *yvex_backend_operation_variant_name(yvex_backend_operation_variant variant)
{
    if ((int)variant >= YVEX_BACKEND_VARIANT_ROCM_FIRST && variant < YVEX_BACKEND_VARIANT_ROCM_END)
        return rocm_variant_names[variant - YVEX_BACKEND_VARIANT_ROCM_FIRST];
    return name_at(variant_names, YVEX_BACKEND_VARIANT_COUNT, (unsigned int)variant);
}

const char *yvex_backend_capability_state_name(yvex_backend_capability_state state)
{
    return name_at(capability_state_names, ARRAY_COUNT(capability_state_names),
                   (unsigned int)state);
}

const char *yvex_backend_capability_reason_name(yvex_backend_capability_reason reason)
{
    return name_at(capability_reason_names, ARRAY_COUNT(capability_reason_names),
                   (unsigned int)reason);
}

const char *yvex_backend_capability_name(yvex_backend_capability capability)
{
    return name_at(capability_names, ARRAY_COUNT(capability_names), (unsigned int)capability);
}

/* src/backend/core.c:195-216, with "rocm" admitted. */
int yvex_backend_kind_parse(const char *name, yvex_backend_kind *out, yvex_error *err)
{
    if (!out)
        return refuse(err, YVEX_ERR_INVALID_ARG, "backend_kind", "output backend kind is required");
    if (!name || strcmp(name, "cpu") == 0) {
        *out = YVEX_BACKEND_KIND_CPU;
    } else if (strcmp(name, "cuda") == 0) {
        *out = YVEX_BACKEND_KIND_CUDA;
    } else if (strcmp(name, "rocm") == 0) {
        *out = YVEX_BACKEND_KIND_ROCM;
    } else {
        yvex_error_setf(err, YVEX_ERR_INVALID_ARG, "backend_kind", "unknown backend kind: %s",
                        name);
        return YVEX_ERR_INVALID_ARG;
    }
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/core.c:255-284: this library builds the ROCM arm only. */
int yvex_backend_open(yvex_backend **out, const yvex_backend_options *options, yvex_error *err)
{
    yvex_backend_kind kind = YVEX_BACKEND_KIND_CPU;
    if (!out) return refuse(err, YVEX_ERR_INVALID_ARG, "yvex_backend_open", "out is required");
    *out = NULL;
    if (options) kind = options->kind;
    if (kind == YVEX_BACKEND_KIND_ROCM)
        return yvex_backend_open_rocm_impl(out, options->device, options->memory_limit_bytes,
                                           err);
    yvex_error_setf(err, YVEX_ERR_UNSUPPORTED, "yvex_backend_open",
                    "backend %s is not implemented", yvex_backend_kind_name(kind));
    return YVEX_ERR_UNSUPPORTED;
}

int yvex_backend_rocm_context_available(void)
{
    yvex_backend *backend = NULL;
    yvex_backend_options options;
    yvex_error err;
    int rc, close_rc;
    memset(&options, 0, sizeof(options));
    options.kind = YVEX_BACKEND_KIND_ROCM;
    yvex_error_clear(&err);
    rc = yvex_backend_open(&backend, &options, &err);
    close_rc = yvex_backend_close_checked(&backend, &err);
    return rc == YVEX_OK && close_rc == YVEX_OK;
}

int yvex_backend_rocm_available(void) { return yvex_backend_rocm_context_available(); }

/* A primary backend counts the session backends opened on it in the low bits of its lifecycle
 * word (src/backend/core.c:305-356, src/backend/cuda/backend.c:1598-1623). */
int yvex_backend_shared_owner_acquire(yvex_backend *owner, yvex_error *err)
{
    static const char where[] = "backend.shared.acquire";
    unsigned long long seen;
    if (!owner || owner->resource_owner != owner || owner->status == YVEX_BACKEND_STATUS_FAILED)
        return refuse(err, YVEX_ERR_STATE, where, "one live primary backend resource owner is required");
    seen = atomic_load_explicit(&owner->lifecycle, memory_order_acquire);
    do {
        if ((seen & YVEX_BACKEND_LIFECYCLE_CLOSING) != 0ull ||
            (seen & YVEX_BACKEND_LIFECYCLE_CHILD_MASK) == YVEX_BACKEND_LIFECYCLE_CHILD_MASK)
            return refuse(err, YVEX_ERR_STATE, where, "backend resource owner is closing or saturated");
    } while (!atomic_compare_exchange_weak_explicit(&owner->lifecycle, &seen, seen + 1ull,
                                                    memory_order_acq_rel, memory_order_acquire));
    yvex_error_clear(err);
    return YVEX_OK;
}

static int shared_owner_release(yvex_backend *owner, yvex_error *err)
{
    static const char where[] = "backend.shared.release";
    unsigned long long seen;
    if (!owner) return refuse(err, YVEX_ERR_STATE, where, "backend resource owner is required");
    seen = atomic_load_explicit(&owner->lifecycle, memory_order_acquire);
    do {
        if ((seen & YVEX_BACKEND_LIFECYCLE_CHILD_MASK) == 0ull)
            return refuse(err, YVEX_ERR_STATE, where, "backend shared-resource lease is not registered");
    } while (!atomic_compare_exchange_weak_explicit(&owner->lifecycle, &seen, seen - 1ull,
                                                    memory_order_acq_rel, memory_order_acquire));
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/core.c:330-356: CLOSING is sticky and the backend FAILED from here on, so nothing
 * dispatches; a primary backend with open session backends is not discharged yet. */
static int close_admit(yvex_backend *backend, yvex_error *err)
{
    const unsigned long long before = atomic_fetch_or_explicit(
        &backend->lifecycle, YVEX_BACKEND_LIFECYCLE_CLOSING, memory_order_acq_rel);
    backend->status = YVEX_BACKEND_STATUS_FAILED;
    if ((before & YVEX_BACKEND_LIFECYCLE_CHILD_MASK) != 0ull)
        return refuse(err, YVEX_ERR_STATE, "backend.close.admit",
                      "backend context still has live shared children");
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/core.c:362-416: the owner pointer is nulled only after the arm
 * discharged its resources; a failed discharge keeps the handle for a retry.  A session
 * backend gives its lease back last. */
int yvex_backend_close_checked(yvex_backend **backend_ptr, yvex_error *err)
{
    yvex_backend *backend, *owner;
    int rc;
    if (!backend_ptr || !*backend_ptr) {
        yvex_error_clear(err);
        return YVEX_OK;
    }
    backend = *backend_ptr;
    owner = backend->resource_owner;
    if (backend->shared_owner_registered &&
        (!owner || owner == backend ||
         (atomic_load_explicit(&owner->lifecycle, memory_order_acquire) &
          YVEX_BACKEND_LIFECYCLE_CHILD_MASK) == 0ull))
        return refuse(err, YVEX_ERR_STATE, "backend.close",
                      "shared backend owner registration is inconsistent");
    rc = close_admit(backend, err);
    if (rc != YVEX_OK) return rc;
    if (backend->vtable && backend->vtable->close) {
        yvex_error cleanup;
        yvex_error_clear(&cleanup);
        rc = backend->vtable->close(backend, &cleanup);
        if (rc != YVEX_OK) {
            if (err) *err = cleanup;
            if (backend->impl) return rc;
        }
    }
    if (backend->shared_owner_registered) {
        yvex_error cleanup;
        int lease_rc;
        yvex_error_clear(&cleanup);
        lease_rc = shared_owner_release(owner, &cleanup);
        if (lease_rc != YVEX_OK) {
            if (err) *err = cleanup;
            return lease_rc;
        }
        backend->shared_owner_registered = 0;
        backend->resource_owner = NULL;
    }
    free(backend);
    *backend_ptr = NULL;
    if (rc == YVEX_OK) yvex_error_clear(err);
    return rc;
}

void yvex_backend_close(yvex_backend *backend)
{
    yvex_error ignored;
    yvex_error_clear(&ignored);
    (void)yvex_backend_close_checked(&backend, &ignored);
}

yvex_backend_kind yvex_backend_kind_of(const yvex_backend *backend)
{
    return backend ? backend->kind : YVEX_BACKEND_KIND_CPU;
}

yvex_backend_status yvex_backend_status_of(const yvex_backend *backend)
{
    return backend ? atomic_load_explicit(&backend->status, memory_order_acquire)
                   : YVEX_BACKEND_STATUS_FAILED;
}

int yvex_backend_tensor_owned_by(const yvex_backend *backend, const yvex_device_tensor *tensor)
{
    return backend_tensor_owner_is(backend, tensor);
}

int yvex_backend_get_memory_stats(const yvex_backend *backend, yvex_backend_memory_stats *out,
                                  yvex_error *err)
{
    if (!backend || !out)
        return refuse(err, YVEX_ERR_INVALID_ARG, "yvex_backend_get_memory_stats",
                      "backend and out are required");
    if (!backend->vtable || !backend->vtable->memory_stats)
        return refuse(err, YVEX_ERR_UNSUPPORTED, "yvex_backend_get_memory_stats",
                      "backend does not provide memory stats");
    return backend->vtable->memory_stats(backend, out, err);
}

int yvex_backend_get_device_info(const yvex_backend *backend, yvex_backend_device_info *out,
                                 yvex_error *err)
{
    if (!backend || !out)
        return refuse(err, YVEX_ERR_INVALID_ARG, "yvex_backend_get_device_info",
                      "backend and out are required");
    if (!backend->vtable || !backend->vtable->device_info)
        return refuse(err, YVEX_ERR_UNSUPPORTED, "yvex_backend_get_device_info",
                      "backend does not provide device info");
    return backend->vtable->device_info(backend, out, err);
}

/* src/backend/core.c:483-502 */
int yvex_backend_bandwidth_probe(yvex_backend *backend, yvex_backend_bandwidth_evidence *out,
                                 yvex_error *err)
{
    int rc;
    if (out) memset(out, 0, sizeof(*out));
    if (!backend || !out)
        return refuse(err, YVEX_ERR_INVALID_ARG, "backend.bandwidth",
                      "backend and bandwidth output are required");
    rc = backend_dispatch_admit(backend, "backend.bandwidth", err);
    if (rc != YVEX_OK) return rc;
    if (!backend->vtable || !backend->vtable->bandwidth_probe)
        return refuse(err, YVEX_ERR_UNSUPPORTED, "backend.bandwidth",
                      "backend does not provide measured bandwidth evidence");
    return backend->vtable->bandwidth_probe(backend, out, err);
}

/* ------------------------------------------------------------- tensors ---- */

/* src/backend/core.c:1143-1171 */
static int desc_valid(const yvex_backend_tensor_desc *desc, yvex_error *err)
{
    static const char where[] = "yvex_backend_tensor_alloc";
    unsigned int i;
    if (!desc) return refuse(err, YVEX_ERR_INVALID_ARG, where, "descriptor is required");
    if (desc->rank == 0 || desc->rank > YVEX_TENSOR_MAX_DIMS)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "rank is out of range");
    if (desc->bytes == 0) return refuse(err, YVEX_ERR_INVALID_ARG, where, "bytes must be non-zero");
    if (desc->bytes > (unsigned long long)SIZE_MAX)
        return refuse(err, YVEX_ERR_BOUNDS, where, "bytes exceed host allocation size");
    for (i = 0; i < desc->rank; ++i)
        if (desc->dims[i] == 0)
            return refuse(err, YVEX_ERR_INVALID_ARG, where, "dimensions must be non-zero");
    yvex_error_clear(err);
    return YVEX_OK;
}

int yvex_backend_memory_can_add(const yvex_backend *backend, unsigned long long bytes,
                                const char *backend_name, const char *where, yvex_error *err)
{
    if (backend->stats.allocated_bytes > ULLONG_MAX - bytes ||
        backend->stats.allocation_count == ULLONG_MAX ||
        backend->stats.allocation_events == ULLONG_MAX)
        return refuse(err, YVEX_ERR_NOMEM, where, "allocated byte counter overflow");
    if (backend->stats.memory_limit_bytes != 0ull &&
        backend->stats.allocated_bytes + bytes > backend->stats.memory_limit_bytes) {
        yvex_error_setf(err, YVEX_ERR_NOMEM, where,
                        "allocation exceeds %s backend memory limit %llu", backend_name,
                        backend->stats.memory_limit_bytes);
        return YVEX_ERR_NOMEM;
    }
    return YVEX_OK;
}

int yvex_backend_tensor_rw_validate(const char *where, const yvex_backend *backend,
                                    const yvex_device_tensor *tensor, unsigned long long len,
                                    yvex_error *err)
{
    if (!backend_tensor_owner_is(backend, tensor))
        return refuse(err, YVEX_ERR_STATE, where, "tensor does not belong to this backend");
    if (len != tensor->bytes) {
        yvex_error_setf(err, YVEX_ERR_BOUNDS, where,
                        "length %llu does not match tensor bytes %llu", len, tensor->bytes);
        return YVEX_ERR_BOUNDS;
    }
    return YVEX_OK;
}

static int same_shape(const yvex_device_tensor *a, const yvex_device_tensor *b)
{
    unsigned int i;
    if (a->dtype != b->dtype || a->rank != b->rank || a->bytes != b->bytes) return 0;
    for (i = 0; i < a->rank; ++i)
        if (a->dims[i] != b->dims[i]) return 0;
    return 1;
}

int yvex_backend_tensor_copy_validate(const yvex_backend *backend, const yvex_device_tensor *dst,
                                      const yvex_device_tensor *src, const char *where,
                                      yvex_error *err)
{
    if (!backend_tensor_owner_is(backend, dst) || !backend_tensor_owner_is(backend, src))
        return refuse(err, YVEX_ERR_STATE, where,
                      "source and destination must belong to this backend");
    if (!same_shape(dst, src))
        return refuse(err, YVEX_ERR_BOUNDS, where,
                      "source and destination tensor descriptors differ");
    return YVEX_OK;
}

int yvex_backend_tensor_alloc(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                              yvex_device_tensor **out, yvex_error *err)
{
    static const char where[] = "yvex_backend_tensor_alloc";
    int rc;
    if (!out) return refuse(err, YVEX_ERR_INVALID_ARG, where, "out is required");
    *out = NULL;
    if (!backend) return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend is required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    rc = desc_valid(desc, err);
    if (rc != YVEX_OK) return rc;
    if (!backend->vtable || !backend->vtable->tensor_alloc)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "backend does not support tensor allocation");
    return backend->vtable->tensor_alloc(backend, desc, out, err);
}

/* src/backend/residency.c:12-17 */
int yvex_backend_virtual_tensor_supported(const yvex_backend *backend)
{
    return backend && !backend_cleanup_only(backend) &&
           backend->status != YVEX_BACKEND_STATUS_FAILED && backend->virtual_tensor_ready;
}

/* src/backend/core.c:613-634 */
int yvex_backend_tensor_reserve(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                                yvex_device_tensor **out, unsigned long long *granularity,
                                yvex_error *err)
{
    static const char where[] = "backend.tensor.reserve";
    int rc;
    if (out) *out = NULL;
    if (granularity) *granularity = 0ull;
    if (!backend || !out || !granularity)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "backend, tensor output, and granularity output are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc == YVEX_OK) rc = desc_valid(desc, err);
    if (rc != YVEX_OK) return rc;
    if (!backend->vtable || !backend->vtable->tensor_reserve)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "backend does not support virtual tensor reservation");
    return backend->vtable->tensor_reserve(backend, desc, out, granularity, err);
}

/* src/backend/core.c:636-659 */
int yvex_backend_tensor_commit_range(yvex_backend *backend, yvex_device_tensor *tensor,
                                     unsigned long long offset, unsigned long long bytes,
                                     unsigned long long *resident_delta, yvex_error *err)
{
    static const char where[] = "backend.tensor.commit";
    int rc;
    if (resident_delta) *resident_delta = 0ull;
    if (!backend || !tensor || !resident_delta || !bytes || offset > tensor->bytes ||
        bytes > tensor->bytes - offset)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "one owned virtual tensor range is required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!backend->vtable || !backend->vtable->tensor_commit)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "backend does not support physical page commitment");
    return backend->vtable->tensor_commit(backend, tensor, offset, bytes, resident_delta, err);
}

/* src/backend/core.c:661-680 */
int yvex_backend_tensor_decommit(yvex_backend *backend, yvex_device_tensor *tensor,
                                 unsigned long long *released_bytes, yvex_error *err)
{
    static const char where[] = "backend.tensor.decommit";
    int rc;
    if (released_bytes) *released_bytes = 0ull;
    if (!backend || !tensor || !released_bytes)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "backend, virtual tensor, and release output are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!backend->vtable || !backend->vtable->tensor_decommit)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "backend does not support physical page decommitment");
    return backend->vtable->tensor_decommit(backend, tensor, released_bytes, err);
}

/* src/backend/core.c:689-715: release is allowed on a cleanup-only backend. */
int yvex_backend_tensor_release(yvex_backend *backend, yvex_device_tensor **tensor,
                                yvex_error *err)
{
    static const char where[] = "yvex_backend_tensor_release";
    int rc;
    if (!backend || !tensor || !*tensor)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and tensor are required");
    if (!backend->vtable || !backend->vtable->tensor_free)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where, "backend does not support tensor release");
    rc = backend->vtable->tensor_free(backend, *tensor, err);
    if (rc == YVEX_OK) *tensor = NULL;
    return rc;
}

void yvex_backend_tensor_free(yvex_backend *backend, yvex_device_tensor *tensor)
{
    yvex_device_tensor *owned = tensor;
    yvex_error err;
    yvex_error_clear(&err);
    (void)yvex_backend_tensor_release(backend, &owned, &err);
}

const char *yvex_device_tensor_name(const yvex_device_tensor *tensor)
{
    return tensor && tensor->name ? tensor->name : "";
}

unsigned long long yvex_device_tensor_bytes(const yvex_device_tensor *tensor)
{
    return tensor ? tensor->bytes : 0ull;
}

int yvex_device_tensor_is_written(const yvex_device_tensor *tensor)
{
    return tensor ? tensor->is_written : 0;
}

#define TENSOR_DISPATCH(where_text, required, slot, call)                                      \
    do {                                                                                       \
        static const char where[] = where_text;                                                \
        int rc_;                                                                               \
        if (!(required)) return refuse(err, YVEX_ERR_INVALID_ARG, where, "arguments are required"); \
        rc_ = backend_dispatch_admit(backend, where, err);                                     \
        if (rc_ != YVEX_OK) return rc_;                                                        \
        if (!backend->vtable || !backend->vtable->slot)                                        \
            return refuse(err, YVEX_ERR_UNSUPPORTED, where, "backend does not support this tensor operation"); \
        return call;                                                                           \
    } while (0)

int yvex_backend_tensor_write(yvex_backend *backend, yvex_device_tensor *tensor, const void *src,
                              unsigned long long len, yvex_error *err)
{
    TENSOR_DISPATCH("yvex_backend_tensor_write", backend && tensor && src, tensor_write,
                    backend->vtable->tensor_write(backend, tensor, src, len, err));
}

int yvex_backend_tensor_read(yvex_backend *backend, const yvex_device_tensor *tensor, void *dst,
                             unsigned long long len, yvex_error *err)
{
    TENSOR_DISPATCH("yvex_backend_tensor_read", backend && tensor && dst, tensor_read,
                    backend->vtable->tensor_read(backend, tensor, dst, len, err));
}

int yvex_backend_tensor_zero(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err)
{
    TENSOR_DISPATCH("yvex_backend_tensor_zero", backend && tensor, tensor_zero,
                    backend->vtable->tensor_zero(backend, tensor, err));
}

int yvex_backend_tensor_copy(yvex_backend *backend, yvex_device_tensor *dst,
                             const yvex_device_tensor *src, yvex_error *err)
{
    TENSOR_DISPATCH("yvex_backend_tensor_copy", backend && dst && src, tensor_copy,
                    backend->vtable->tensor_copy(backend, dst, src, err));
}

/* src/backend/core.c:822-840: lifecycle, then ownership and descriptors, then the slot. */
int yvex_backend_tensor_copy_async(yvex_backend *backend, yvex_device_tensor *destination,
                                   const yvex_device_tensor *source, yvex_error *err)
{
    static const char where[] = "backend.tensor.copy-async";
    int rc = backend_dispatch_admit(backend, where, err);
    if (rc == YVEX_OK) rc = yvex_backend_tensor_copy_validate(backend, destination, source, where, err);
    if (rc != YVEX_OK) return rc;
    if (!backend->vtable || !backend->vtable->tensor_copy_async)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "backend does not support asynchronous tensor copy");
    return backend->vtable->tensor_copy_async(backend, destination, source, err);
}

static yvex_backend *physical_owner(yvex_backend *backend)
{
    return backend->resource_owner ? backend->resource_owner : backend;
}

/* src/backend/core.c:842-874: the executor owns the destination, the source belongs to a
 * backend with the same physical owner, same descriptors, source written. */
int yvex_backend_tensor_copy_shared_async(yvex_backend *executor, yvex_device_tensor *destination,
                                          const yvex_device_tensor *source, yvex_error *err)
{
    static const char where[] = "backend.tensor.copy-shared";
    int rc;
    if (!executor || !destination || !source || !destination->owner || !source->owner)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "executor and two owned tensors are required");
    rc = backend_dispatch_admit(executor, where, err);
    if (rc == YVEX_OK) rc = backend_dispatch_admit(source->owner, where, err);
    if (rc != YVEX_OK) return rc;
    if (destination->owner != executor ||
        physical_owner(source->owner) != physical_owner(executor) ||
        !same_shape(destination, source) || !source->is_written)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "same-physical-owner initialized tensor shapes are required");
    if (!executor->vtable || !executor->vtable->tensor_copy_shared_async)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "backend does not support cross-stream tensor copy");
    return executor->vtable->tensor_copy_shared_async(executor, destination, source, err);
}

int yvex_backend_sync(yvex_backend *backend, yvex_error *err)
{
    TENSOR_DISPATCH("yvex_backend_sync", backend, sync, backend->vtable->sync(backend, err));
}

/* src/backend/core.c:1763-1778 */
int yvex_backend_tensor_f32_subview(const yvex_device_tensor *source, unsigned long long offset,
                                    unsigned long long count, yvex_device_tensor *view)
{
    unsigned long long elements;
    if (!source || !view || !count || source->dtype != YVEX_DTYPE_F32 || !source->data ||
        source->bytes % sizeof(float))
        return 0;
    elements = source->bytes / sizeof(float);
    if (offset > elements || count > elements - offset) return 0;
    *view = *source;
    view->rank = 1u;
    memset(view->dims, 0, sizeof(view->dims));
    view->dims[0] = count;
    view->bytes = count * sizeof(float);
    view->data = source->data + offset * sizeof(float);
    return 1;
}

/* ---------------------------------------------------------- capability ---- */

typedef struct {
    yvex_dtype input, weight, output;
} dtype_projection;

static void variant_dtypes(yvex_backend_capability_result *out)
{
    dtype_projection p = {YVEX_DTYPE_UNKNOWN, YVEX_DTYPE_UNKNOWN, YVEX_DTYPE_UNKNOWN};
    switch (out->variant) {
    case YVEX_BACKEND_VARIANT_ATTENTION_CAUSAL_F32:
    case YVEX_BACKEND_VARIANT_ATTENTION_NONCAUSAL_F32:
    case YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32:
        p = (dtype_projection){YVEX_DTYPE_F32, YVEX_DTYPE_F32, YVEX_DTYPE_F32};
        break;
    case YVEX_BACKEND_VARIANT_ATTENTION_ENCODED:
        p.output = YVEX_DTYPE_F32;
        break;
    case YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16:
    case YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16:
    case YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16:
        p = (dtype_projection){YVEX_DTYPE_BF16, YVEX_DTYPE_BF16, YVEX_DTYPE_BF16};
        break;
    case YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0:
        p = (dtype_projection){YVEX_DTYPE_BF16, YVEX_DTYPE_Q8_0, YVEX_DTYPE_BF16};
        break;
    default:
        break;
    }
    out->input_dtype = p.input;
    out->weight_dtype = p.weight;
    out->output_dtype = p.output;
}

/* src/backend/core.c:905-945 */
int yvex_backend_query_capability(const yvex_backend *backend,
                                  yvex_backend_operation_variant variant,
                                  yvex_backend_capability_result *out, yvex_error *err)
{
    static const char where[] = "yvex_backend_query_capability";
    int rc;
    if (!backend || !out) return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and out are required");
    if ((int)variant < 0 ||
        ((int)variant >= YVEX_BACKEND_VARIANT_COUNT &&
         ((int)variant < YVEX_BACKEND_VARIANT_ROCM_FIRST || variant >= YVEX_BACKEND_VARIANT_ROCM_END)))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "operation variant is out of range");
    memset(out, 0, sizeof(*out));
    out->backend_kind = backend->kind;
    out->variant = variant;
    variant_dtypes(out);
    if (backend_cleanup_only(backend)) {
        out->state = YVEX_BACKEND_CAPABILITY_FAILED;
        out->reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
        yvex_error_clear(err);
        return YVEX_OK;
    }
    out->state = YVEX_BACKEND_CAPABILITY_UNSUPPORTED;
    out->reason = YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED;
    if (!backend->vtable || !backend->vtable->query_capability) {
        yvex_error_clear(err);
        return YVEX_OK;
    }
    rc = backend->vtable->query_capability(backend, variant, out, err);
    if (rc == YVEX_OK) {
        out->backend_kind = backend->kind;
        out->variant = variant;
        variant_dtypes(out);
    }
    return rc;
}

static int variant_supported(const yvex_backend *backend, yvex_backend_operation_variant variant)
{
    yvex_backend_capability_result result;
    yvex_error err;
    yvex_error_clear(&err);
    return yvex_backend_query_capability(backend, variant, &result, &err) == YVEX_OK &&
           result.state == YVEX_BACKEND_CAPABILITY_SUPPORTED;
}

/* src/backend/core.c:75-100,947-963: a capability is a rule over variants. */
int yvex_backend_supports(const yvex_backend *backend, yvex_backend_capability capability)
{
    if (!backend) return 0;
    switch (capability) {
    case YVEX_BACKEND_CAP_TENSOR_ALLOC:
        return variant_supported(backend, YVEX_BACKEND_VARIANT_TENSOR_ALLOC) &&
               variant_supported(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO);
    case YVEX_BACKEND_CAP_TENSOR_READ_WRITE:
        return variant_supported(backend, YVEX_BACKEND_VARIANT_TENSOR_WRITE) &&
               variant_supported(backend, YVEX_BACKEND_VARIANT_TENSOR_READ) &&
               variant_supported(backend, YVEX_BACKEND_VARIANT_TENSOR_COPY);
    case YVEX_BACKEND_CAP_OP_ATTENTION:
        return variant_supported(backend, YVEX_BACKEND_VARIANT_ATTENTION_CAUSAL_F32) ||
               variant_supported(backend, YVEX_BACKEND_VARIANT_ATTENTION_NONCAUSAL_F32);
    default:
        return 0;
    }
}

const yvex_backend_transformer_operations *yvex_backend_transformer_operations_get(
    const yvex_backend *backend)
{
    return backend && backend->vtable && backend->vtable->transformer_operations
               ? backend->vtable->transformer_operations(backend)
               : NULL;
}


/* The encoded-attention transaction (include/yvex/internal/backend.h:193-198).  The
 * reference's only implementation is the CUDA one (src/backend/cuda/attention.c:1924);
 * this backend owns none of the job's projection, compressor or indexer stages, so the
 * symbol answers the way an unadmitted capability does: argument errors first, then the
 * lifecycle gate, then a CAPABILITY failure with YVEX_ERR_UNSUPPORTED.  The job is not read
 * and the output record is not written. */
int yvex_backend_attention_execute(yvex_backend *backend, const yvex_backend_attention_job *job,
                                   yvex_backend_attention_output *output,
                                   yvex_backend_attention_failure *failure, yvex_error *err)
{
    static const char where[] = "rocm.attention.encoded";
    int rc;
    if (failure) memset(failure, 0, sizeof(*failure));
    yvex_error_clear(err);
    if (!backend || !job || !output) {
        if (failure) {
            failure->code = YVEX_BACKEND_ATTENTION_FAILURE_INVALID_ARGUMENT;
            failure->stage = where;
            failure->expected = 1ull;
        }
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "backend, attention job and output record are required");
    }
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (failure) {
        failure->code = YVEX_BACKEND_ATTENTION_FAILURE_CAPABILITY;
        failure->stage = where;
        failure->expected = 1ull;
    }
    return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                  "the encoded attention transaction is not admitted by the ROCm backend");
}

/* src/backend/cuda/attention_completion.c:110-120: a completion this backend never made
 * pending has no valid owner. */
int yvex_backend_attention_complete(yvex_backend *backend,
                                    yvex_backend_attention_completion *completion,
                                    int barrier_observed, yvex_error *err)
{
    (void)backend;
    (void)completion;
    (void)barrier_observed;
    return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.attention.complete",
                  "ROCm attention completion owner is invalid");
}

/* ----------------------------------------------------------- workspace ---- */

/* The attached workspace is one tensor of the backend used as a bump arena: operations carve
 * aligned pieces off its front for the length of one dispatch and the dispatch rewinds it.  The
 * arena never grows and never allocates.  Behaviour follows the contract of
 * src/backend/residency.c:207-283 (and tests/test_host_backend.py holds it to that):
 *   attach   INVALID_ARG unless a live backend of this kind, a written-to-able tensor it owns
 *            (not a reserved address range) and a non-zero generation; STATE when one is attached
 *   detach   forgets the arena and its statistics; harmless without one
 *   acquire  MISS without a usable arena or without room, INVALID for a zero size or an
 *            alignment that is not a power of two, HIT with the address otherwise */
static int workspace_backend_live(const yvex_backend *backend)
{
    return backend && !backend_cleanup_only(backend) && backend->status != YVEX_BACKEND_STATUS_FAILED;
}

static int workspace_tensor_usable(const yvex_backend *backend, const yvex_device_tensor *tensor)
{
    return tensor && tensor->data && tensor->bytes != 0ull && !tensor->virtual_reserved &&
           backend_tensor_owner_is(backend, tensor);
}

static void workspace_bind(yvex_backend *backend, const yvex_device_tensor *tensor,
                           unsigned long long generation)
{
    backend->workspace_device_tensor = tensor;
    backend->workspace_device_address = tensor ? (unsigned long long)(uintptr_t)tensor->data : 0ull;
    backend->workspace_bytes = tensor ? tensor->bytes : 0ull;
    backend->workspace_generation = generation;
    backend->workspace_cursor = 0ull;
    backend->workspace_peak = 0ull;
}

int yvex_backend_workspace_attach(yvex_backend *backend, const yvex_device_tensor *device_tensor,
                                  unsigned long long generation, yvex_error *err)
{
    static const char where[] = "backend.workspace.attach";
    if (!workspace_backend_live(backend) || backend->kind != YVEX_BACKEND_KIND_ROCM ||
        generation == 0ull || !workspace_tensor_usable(backend, device_tensor))
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "same-owner ROCm workspace tensor and generation are required");
    if (backend->workspace_device_tensor != NULL)
        return refuse(err, YVEX_ERR_STATE, where, "backend workspace is already attached");
    workspace_bind(backend, device_tensor, generation);
    yvex_error_clear(err);
    return YVEX_OK;
}

void yvex_backend_workspace_detach(yvex_backend *backend)
{
    if (backend) workspace_bind(backend, NULL, 0ull);
}

int yvex_backend_workspace_acquire(yvex_backend *backend, unsigned long long bytes,
                                   unsigned long long alignment,
                                   unsigned long long *device_address)
{
    unsigned long long begin, end, address;
    if (device_address) *device_address = 0ull;
    if (!device_address || !workspace_backend_live(backend) || !backend->workspace_device_tensor)
        return YVEX_BACKEND_RESIDENT_MISS;
    if (bytes == 0ull || alignment == 0ull || (alignment & (alignment - 1ull)) != 0ull)
        return YVEX_BACKEND_RESIDENT_INVALID;
    /* first multiple of the alignment at or behind the cursor */
    if (!yvex_core_u64_add(backend->workspace_cursor, alignment - 1ull, &begin))
        return YVEX_BACKEND_RESIDENT_INVALID;
    begin -= begin % alignment;
    if (!yvex_core_u64_add(begin, bytes, &end) || end > backend->workspace_bytes ||
        !yvex_core_u64_add(backend->workspace_device_address, begin, &address))
        return YVEX_BACKEND_RESIDENT_MISS;
    backend->workspace_cursor = end;
    if (end > backend->workspace_peak) backend->workspace_peak = end;
    *device_address = address;
    return YVEX_BACKEND_RESIDENT_HIT;
}

/* --------------------------------------------------- op_attention path ---- */

/* src/backend/core.c:1095-1141: refusal order NULL -> lifecycle -> seq_len ->
 * position -> scale -> missing slot. */
int yvex_backend_op_attention(yvex_backend *backend, const yvex_device_tensor *query,
                              const yvex_device_tensor *keys, const yvex_device_tensor *values,
                              unsigned long long seq_len, unsigned long long position,
                              float scale, int causal, yvex_device_tensor *score_scratch,
                              yvex_device_tensor *probability_scratch, yvex_device_tensor *out,
                              yvex_error *err)
{
    static const char where[] = "yvex_backend_op_attention";
    int rc;
    if (!backend || !query || !keys || !values || !score_scratch || !probability_scratch || !out)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "backend, Q/K/V, scratches, and output are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (seq_len == 0) return refuse(err, YVEX_ERR_INVALID_ARG, where, "seq_len must be positive");
    if (position >= seq_len) return refuse(err, YVEX_ERR_BOUNDS, where, "position-out-of-range");
    if (!isfinite(scale) || scale <= 0.0f)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "scale must be finite and positive");
    if (!backend->vtable || !backend->vtable->op_attention)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where, "backend does not support attention op");
    return backend->vtable->op_attention(backend, query, keys, values, seq_len, position, scale,
                                         causal, score_scratch, probability_scratch, out, err);
}

static int f32_elements(const yvex_device_tensor *tensor, unsigned long long elements)
{
    return tensor && elements <= ULLONG_MAX / sizeof(float) &&
           tensor->bytes == elements * (unsigned long long)sizeof(float);
}

/* src/backend/core.c:1547-1616: ownership -> dtype -> rank/shape -> byte accounting. */
int yvex_backend_validate_attention(const yvex_backend *backend, const yvex_device_tensor *query,
                                    const yvex_device_tensor *keys,
                                    const yvex_device_tensor *values, unsigned long long seq_len,
                                    unsigned long long position,
                                    yvex_device_tensor *score_scratch,
                                    yvex_device_tensor *probability_scratch,
                                    yvex_device_tensor *out, unsigned long long *head_dim_out,
                                    unsigned long long *kv_elements_out, const char *where,
                                    yvex_error *err)
{
    const yvex_device_tensor *set[6] = {query, keys, values, score_scratch, probability_scratch,
                                        out};
    unsigned long long head_dim, kv_elements;
    size_t i;
    for (i = 0; i < 6u; ++i)
        if (!backend_tensor_owner_is(backend, set[i]))
            return refuse(err, YVEX_ERR_STATE, where,
                          "Q/K/V, scratches, and output tensors must belong to this backend");
    for (i = 0; i < 6u; ++i)
        if (set[i]->dtype != YVEX_DTYPE_F32)
            return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                          "attention primitive supports F32 Q/K/V, scratches, and output");
    if (!head_dim_out || !kv_elements_out || seq_len == 0ull || query->rank != 1 ||
        query->dims[0] == 0ull)
        return refuse(err, YVEX_ERR_FORMAT, where,
                      seq_len == 0ull ? "attention-seq-len-zero"
                                      : "attention query must be rank 1 with non-zero head_dim");
    if (position >= seq_len) return refuse(err, YVEX_ERR_BOUNDS, where, "position-out-of-range");
    head_dim = query->dims[0];
    if (seq_len > ULLONG_MAX / head_dim)
        return refuse(err, YVEX_ERR_BOUNDS, where, "attention-element-count-overflow");
    kv_elements = seq_len * head_dim;
    if (keys->rank != 2 || keys->dims[0] != seq_len || keys->dims[1] != head_dim ||
        values->rank != 2 || values->dims[0] != seq_len || values->dims[1] != head_dim)
        return refuse(err, YVEX_ERR_FORMAT, where,
                      "attention keys and values must have dims [seq_len, head_dim]");
    if (out->rank != 1 || out->dims[0] != head_dim)
        return refuse(err, YVEX_ERR_FORMAT, where, "attention output must have dims [head_dim]");
    if (score_scratch->rank != 1 || score_scratch->dims[0] != seq_len ||
        probability_scratch->rank != 1 || probability_scratch->dims[0] != seq_len)
        return refuse(err, YVEX_ERR_FORMAT, where,
                      "attention score/probability scratches must have dims [seq_len]");
    if (!f32_elements(query, head_dim) || !f32_elements(keys, kv_elements) ||
        !f32_elements(values, kv_elements) || !f32_elements(score_scratch, seq_len) ||
        !f32_elements(probability_scratch, seq_len) || !f32_elements(out, head_dim))
        return refuse(err, YVEX_ERR_BOUNDS, where,
                      "attention tensor bytes must match F32 shape accounting");
    *head_dim_out = head_dim;
    *kv_elements_out = kv_elements;
    return YVEX_OK;
}
