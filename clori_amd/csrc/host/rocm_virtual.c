/* Virtual-range tensors: one stable device address range per tensor, backed by physical
 * memory only where the caller has committed it.  The reference keeps each layer's
 * attention history this way, committing as the sequence grows
 * (src/runtime/state_residency.c:258-287,441-446), through its backend's reserve /
 * commit / decommit slots (src/backend/private.h:31-36, src/backend/cuda/backend.c:500-834,
 * 944-980).  Contract kept from there: reservation costs no physical memory and is not
 * counted against the memory limit; a commit backs exactly the granules that intersect the
 * range and are not backed yet, one physical allocation each, reports their bytes,
 * zero-fills them, and is idempotent; a failed commit leaves what was committed before it
 * untouched; decommit returns every granule and keeps the address range; release does both.
 *
 * What is this arm's own: the granule is 2 MiB (or the runtime's recommended granularity
 * where that is larger), the size this part's page tables map in one entry, although the
 * runtime reports 4 KiB; every mapping has that one size, because on this part
 * hipMemSetAccess refuses (invalid argument) a mapping placed directly above a mapping of
 * another size in the same range, while equal-sized neighbours, gaps and mappings placed
 * below are accepted; the granules of one commit are cleared on the stream and waited for
 * once; and a granule whose access could not be set is never touched: it is unmapped and
 * released.  Every tensor or view that reaches the device is first checked to lie on
 * committed granules (yvex_rocm_tensor_backed), since an access to a reserved address
 * without memory behind it is a device fault, not an error code. */
#include "rocm_state.h"

#include <limits.h>
#include <stdlib.h>
#include <string.h>

#define ROCM_VIRTUAL_GRANULE_MIN ((size_t)2u << 20)

typedef struct yvex_rocm_virtual_range {
    unsigned char *address;
    size_t logical_bytes, reserved_bytes, granularity, granule_count;
    hipMemGenericAllocationHandle_t *handles; /* per granule */
    unsigned char *state;                     /* per granule: GRANULE_* bits */
    /* the backend keeps every live range in a list: a view is a struct copy that carries the
     * range pointer and the owner's id, and may outlive the tensor it was taken from */
    struct yvex_rocm_virtual_range *next;
    yvex_device_tensor *owner_tensor; /* the tensor that owns the range: residency is counted there */
    unsigned long long owner_id;
} yvex_rocm_virtual_range;

enum { GRANULE_CREATED = 1, GRANULE_MAPPED = 2 };

static int refuse(yvex_error *err, yvex_status status, const char *where, const char *reason)
{
    yvex_error_set(err, status, where, reason);
    return status;
}

static void range_properties(const yvex_rocm_backend_state *state, hipMemAllocationProp *properties,
                             hipMemAccessDesc *access)
{
    memset(properties, 0, sizeof(*properties));
    properties->type = hipMemAllocationTypePinned;
    properties->location.type = hipMemLocationTypeDevice;
    properties->location.id = state->device_index;
    if (access) {
        memset(access, 0, sizeof(*access));
        access->location = properties->location;
        access->flags = hipMemAccessFlagsProtReadWrite;
    }
}

/* The live range a tensor or a view of it lies in.  The pointer a view carries is only
 * compared, never followed, until it is found among the backend's live ranges with the id the
 * view was copied with: a view kept past the release of its tensor finds nothing (and an
 * address that a later range happens to reuse has another id). */
static yvex_rocm_virtual_range *range_of(const yvex_device_tensor *tensor)
{
    const yvex_rocm_backend_state *state;
    yvex_rocm_virtual_range *range;
    if (!tensor || !tensor->virtual_reserved || !tensor->owner || !tensor->owner_id) return NULL;
    state = yvex_rocm_state(tensor->owner);
    for (range = state ? state->virtual_ranges : NULL; range; range = range->next)
        if ((void *)range == tensor->backend_allocation && range->owner_id == tensor->owner_id)
            return range;
    return NULL;
}

/* The granules under [tensor->data + offset, + bytes), or 0 when that is not inside the range. */
static int granule_span(const yvex_device_tensor *tensor, const yvex_rocm_virtual_range *range,
                        unsigned long long offset, unsigned long long bytes, size_t *first,
                        size_t *last)
{
    unsigned long long base, end;
    if (!range || !bytes || tensor->data < range->address) return 0;
    base = (unsigned long long)(tensor->data - range->address);
    if (!yvex_core_u64_add(base, offset, &base) || !yvex_core_u64_add(base, bytes, &end) ||
        end > range->logical_bytes)
        return 0;
    *first = (size_t)(base / range->granularity);
    *last = (size_t)((end - 1ull) / range->granularity);
    return 1;
}

int yvex_rocm_tensor_backed(const yvex_device_tensor *tensor)
{
    const yvex_rocm_virtual_range *range = range_of(tensor);
    size_t first, last, granule;
    if (!tensor || !tensor->virtual_reserved) return 1;
    if (!granule_span(tensor, range, 0ull, tensor->bytes, &first, &last)) return 0;
    for (granule = first; granule <= last; ++granule)
        if (range->state[granule] != (GRANULE_CREATED | GRANULE_MAPPED)) return 0;
    return 1;
}

static int named_by_recorded_sequence(const yvex_backend *backend,
                                      const yvex_rocm_backend_state *state,
                                      const yvex_device_tensor *tensor)
{
    const yvex_rocm_graph *graph;
    if (backend_cleanup_only(backend)) return 0;
    for (graph = state->graphs; graph; graph = graph->next)
        if (tensor->owner_id < graph->tensor_id_mark) return 1;
    return 0;
}

/* src/backend/cuda/backend.c:559-648 */
int yvex_rocm_tensor_reserve(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                             yvex_device_tensor **out, unsigned long long *granularity_out,
                             yvex_error *err)
{
    static const char where[] = "rocm.tensor.reserve";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_virtual_range *range = NULL;
    yvex_device_tensor *tensor = NULL;
    hipMemAllocationProp properties;
    size_t granularity = 0u, reserved, name_bytes;
    void *address = NULL;
    unsigned int i;
    int rc;
    if (!state || !desc || !out || !granularity_out || !state->virtual_memory)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where,
                      "ROCm virtual-memory reservation is unavailable");
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where,
                      "not available while a launch sequence is being recorded");
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_ALLOC, where, err);
    if (rc != YVEX_OK) return rc;
    range_properties(state, &properties, NULL);
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipMemGetAllocationGranularity(
                              &granularity, &properties, hipMemAllocationGranularityRecommended),
                          "rocm.tensor.reserve.granularity", err);
    if (rc != YVEX_OK) return rc;
    if (granularity && granularity < ROCM_VIRTUAL_GRANULE_MIN)
        granularity = (ROCM_VIRTUAL_GRANULE_MIN + granularity - 1u) / granularity * granularity;
    if (!granularity || desc->bytes > (unsigned long long)SIZE_MAX - (granularity - 1u))
        return refuse(err, YVEX_ERR_BOUNDS, where, "virtual tensor reservation geometry overflowed");
    reserved = ((size_t)desc->bytes + granularity - 1u) / granularity * granularity;
    range = (yvex_rocm_virtual_range *)calloc(1u, sizeof(*range));
    tensor = (yvex_device_tensor *)calloc(1u, sizeof(*tensor));
    if (range) {
        range->logical_bytes = (size_t)desc->bytes;
        range->reserved_bytes = reserved;
        range->granularity = granularity;
        range->granule_count = reserved / granularity;
        range->handles = (hipMemGenericAllocationHandle_t *)calloc(range->granule_count,
                                                                   sizeof(*range->handles));
        range->state = (unsigned char *)calloc(range->granule_count, sizeof(*range->state));
    }
    name_bytes = strlen(desc->name ? desc->name : "") + 1u;
    if (tensor) tensor->name = (char *)malloc(name_bytes);
    if (!range || !range->handles || !range->state || !tensor || !tensor->name) {
        rc = refuse(err, YVEX_ERR_NOMEM, where, "virtual tensor page directory allocation failed");
    } else {
        memcpy(tensor->name, desc->name ? desc->name : "", name_bytes);
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemAddressReserve(&address, reserved, granularity,
                                                                 NULL, 0ull),
                              where, err);
    }
    if (rc != YVEX_OK) {
        if (range) {
            free(range->handles);
            free(range->state);
        }
        free(range);
        if (tensor) free(tensor->name);
        free(tensor);
        return rc;
    }
    range->address = (unsigned char *)address;
    tensor->owner = backend;
    tensor->owner_id = backend->tensor_id_next++;
    tensor->dtype = desc->dtype;
    tensor->rank = desc->rank;
    for (i = 0; i < desc->rank; ++i) tensor->dims[i] = desc->dims[i];
    tensor->bytes = desc->bytes;
    tensor->data = range->address;
    tensor->backend_allocation = range;
    tensor->virtual_reserved = 1;
    range->owner_tensor = tensor;
    range->owner_id = tensor->owner_id;
    range->next = state->virtual_ranges;
    state->virtual_ranges = range;
    state->live_tensors += 1ull;
    *out = tensor;
    *granularity_out = (unsigned long long)granularity;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* Gives one granule back: unmap, release, accounting.  What succeeded stays recorded, so a
 * second attempt repeats only the part that failed (src/backend/cuda/backend.c:650-675). */
static int granule_release(yvex_backend *backend, yvex_rocm_virtual_range *range, size_t granule,
                           yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc = YVEX_OK;
    if (range->state[granule] & GRANULE_MAPPED) {
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemUnmap(range->address + granule * range->granularity,
                                                        range->granularity),
                              "rocm.tensor.decommit.unmap", err);
        if (rc == YVEX_OK) range->state[granule] &= (unsigned char)~GRANULE_MAPPED;
    }
    if (rc == YVEX_OK && (range->state[granule] & GRANULE_CREATED)) {
        rc = yvex_rocm_status(&state->driver, state->driver.hipMemRelease(range->handles[granule]),
                              "rocm.tensor.decommit.release", err);
        if (rc == YVEX_OK) {
            range->state[granule] = 0u;
            backend_memory_release(backend, range->granularity);
        }
    }
    return rc;
}

/* src/backend/cuda/backend.c:679-794 */
int yvex_rocm_tensor_commit(yvex_backend *backend, yvex_device_tensor *tensor,
                            unsigned long long offset, unsigned long long bytes,
                            unsigned long long *resident_delta, yvex_error *err)
{
    static const char where[] = "rocm.tensor.commit";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_virtual_range *range = range_of(tensor);
    hipMemAllocationProp properties;
    hipMemAccessDesc access;
    size_t first, last, granule, missing = 0u, added = 0u, *fresh;
    unsigned long long required;
    int rc;
    if (!state || !range || !resident_delta || !backend_tensor_owner_is(backend, tensor) ||
        !bytes || offset > tensor->bytes || bytes > tensor->bytes - offset ||
        !granule_span(tensor, range, offset, bytes, &first, &last))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "one owned virtual tensor range is required");
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where,
                      "not available while a launch sequence is being recorded");
    /* A granule that an earlier release left half done (unmapped, its memory not given back
     * yet) is neither backed nor missing: finish that release first, or say why it cannot be
     * finished; it then counts as missing like any other. */
    for (granule = first; granule <= last; ++granule)
        if (range->state[granule] && range->state[granule] != (GRANULE_CREATED | GRANULE_MAPPED)) {
            rc = granule_release(backend, range, granule, err);
            if (rc != YVEX_OK) {
                state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
                backend->status = YVEX_BACKEND_STATUS_FAILED;
                return rc;
            }
            range->owner_tensor->resident_bytes =
                range->owner_tensor->resident_bytes >= range->granularity
                    ? range->owner_tensor->resident_bytes - range->granularity : 0ull;
        }
    for (granule = first; granule <= last; ++granule)
        if (!range->state[granule]) ++missing;
    if (!missing) {
        *resident_delta = 0ull;
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (!yvex_core_u64_mul(missing, range->granularity, &required) ||
        range->owner_tensor->resident_bytes > ULLONG_MAX - required)
        return refuse(err, YVEX_ERR_BOUNDS, where, "physical page commitment extent overflowed");
    rc = yvex_backend_memory_can_add(backend, required, "ROCm state pages", where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO, where, err);
    if (rc != YVEX_OK) return rc;
    fresh = (size_t *)calloc(missing, sizeof(*fresh));
    if (!fresh) return refuse(err, YVEX_ERR_NOMEM, where, "physical page transaction allocation failed");
    range_properties(state, &properties, &access);
    for (granule = first; rc == YVEX_OK && granule <= last; ++granule) {
        unsigned char *address = range->address + granule * range->granularity;
        if (range->state[granule]) continue; /* backed already */
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemCreate(&range->handles[granule], range->granularity,
                                                         &properties, 0ull),
                              "rocm.tensor.commit.create", err);
        if (rc != YVEX_OK) break;
        range->state[granule] = GRANULE_CREATED;
        backend_memory_acquire(backend, range->granularity);
        fresh[added++] = granule;
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemMap(address, range->granularity, 0u,
                                                      range->handles[granule], 0ull),
                              "rocm.tensor.commit.map", err);
        if (rc == YVEX_OK) {
            range->state[granule] |= GRANULE_MAPPED;
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipMemSetAccess(address, range->granularity, &access,
                                                                1u),
                                  "rocm.tensor.commit.access", err);
        }
        if (rc == YVEX_OK)
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipMemsetAsync(address, 0, range->granularity,
                                                               yvex_rocm_stream(state)),
                                  "rocm.tensor.commit.zero", err);
    }
    if (rc == YVEX_OK)
        rc = yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO,
                                   "rocm.tensor.commit.zero_sync", err);
    if (rc != YVEX_OK) {
        yvex_error primary, cleanup;
        int undone = YVEX_OK;
        yvex_error_clear(&primary);
        if (err) primary = *err;
        /* the clears of this call may still be in flight */
        (void)state->driver.hipStreamSynchronize(yvex_rocm_stream(state));
        while (added && undone == YVEX_OK) {
            yvex_error_clear(&cleanup);
            undone = granule_release(backend, range, fresh[--added], &cleanup);
        }
        free(fresh);
        if (undone != YVEX_OK) {
            state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
            backend->status = YVEX_BACKEND_STATUS_FAILED;
            if (err) *err = cleanup;
            return undone;
        }
        if (err) *err = primary;
        return rc;
    }
    free(fresh);
    /* residency is a property of the range: counted on the tensor that owns it, also when the
     * commit came through a view */
    range->owner_tensor->resident_bytes += required;
    *resident_delta = required;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/cuda/backend.c:796-834 */
int yvex_rocm_tensor_decommit(yvex_backend *backend, yvex_device_tensor *tensor,
                              unsigned long long *released_bytes, yvex_error *err)
{
    static const char where[] = "rocm.tensor.decommit";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_virtual_range *range = range_of(tensor);
    unsigned long long released = 0ull;
    size_t granule;
    int rc;
    if (!state || !range || !released_bytes || !backend_tensor_owner_is(backend, tensor))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "one owned virtual tensor is required");
    if (tensor->data != range->address)
        return refuse(err, YVEX_ERR_INVALID_ARG, where,
                      "the tensor that owns the range is required, not a view into it");
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where,
                      "not available while a launch sequence is being recorded");
    if (named_by_recorded_sequence(backend, state, tensor))
        return refuse(err, YVEX_ERR_STATE, where,
                      "a recorded launch sequence may still name this tensor: release the "
                      "sequence first");
    /* nothing may still read the pages: drain the stream first */
    rc = yvex_rocm_status(&state->driver, state->driver.hipStreamSynchronize(yvex_rocm_stream(state)), where,
                          err);
    for (granule = 0u; rc == YVEX_OK && granule < range->granule_count; ++granule)
        if (range->state[granule]) {
            rc = granule_release(backend, range, granule, err);
            if (rc == YVEX_OK) released += range->granularity;
        }
    tensor->resident_bytes =
        tensor->resident_bytes >= released ? tensor->resident_bytes - released : 0ull;
    if (rc != YVEX_OK) {
        /* pages that could not be given back: as for a tensor that cannot be freed, the
         * backend is retained for cleanup only and a later release tries again */
        state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return rc;
    }
    *released_bytes = released;
    tensor->is_written = 0;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* The virtual half of tensor_free (src/backend/cuda/backend.c:964-980): every page back,
 * then the address range.  On failure the tensor keeps its range and can be released again. */
int yvex_rocm_virtual_release(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_virtual_range *range = range_of(tensor);
    unsigned long long released = 0ull;
    int rc;
    if (!state || !range)
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.tensor_free", "one owned virtual tensor is required");
    rc = yvex_rocm_tensor_decommit(backend, tensor, &released, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemAddressFree(range->address, range->reserved_bytes),
                              "rocm.tensor.free.address", err);
    if (rc != YVEX_OK) return rc;
    {
        yvex_rocm_virtual_range **link = &state->virtual_ranges;
        while (*link && *link != range) link = &(*link)->next;
        if (*link) *link = range->next;
    }
    free(range->handles);
    free(range->state);
    free(range);
    tensor->backend_allocation = NULL;
    tensor->data = NULL;
    return YVEX_OK;
}
