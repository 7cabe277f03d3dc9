/* ROCm backend arm: runtime binding, device and stream ownership, tensor traffic,
 * synchronisation, timing and the vtable.  Structure follows the reference's CUDA arm
 * (src/backend/cuda/backend.c:836-1100,1561-1789): the opener binds the runtime, takes
 * the device, creates the launch stream, admits the kernel bundle and publishes READY;
 * without a bundle it publishes CONTEXT_READY and every operation variant refuses. */
#define _GNU_SOURCE /* dladdr */
#include "rocm_state.h"

#include <dlfcn.h>
#include <stdlib.h>
#include <string.h>

#include "../kernel_params.h"
#include "rocm_scratch.h"

static void probe_release(yvex_rocm_backend_state *state);

static int refuse(yvex_error *err, yvex_status status, const char *where, const char *reason)
{
    yvex_error_set(err, status, where, reason);
    return status;
}

static char *text_dup(const char *text)
{
    size_t n = strlen(text ? text : "") + 1u;
    char *copy = (char *)malloc(n);
    if (copy) memcpy(copy, text ? text : "", n);
    return copy;
}

/* ------------------------------------------------------------- tensors ---- */

static const char kUnbacked[] =
    "a tensor over a reserved address range reaches pages that are not committed";

/* src/backend/cuda/backend.c:836-905: capability, limit, allocate, zero, publish. */
static int rocm_tensor_alloc(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                             yvex_device_tensor **out, yvex_error *err)
{
    static const char where[] = "rocm.tensor_alloc";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_device_tensor *tensor;
    void *ptr = NULL;
    unsigned int i;
    int rc;
    if (!backend || !state || !out)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and out are required");
    *out = NULL;
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_ALLOC, where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO, where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_backend_memory_can_add(backend, desc->bytes, "ROCm", where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_status(&state->driver, state->driver.hipMalloc(&ptr, (size_t)desc->bytes),
                          where, err);
    if (rc != YVEX_OK) {
        if (err) err->code = YVEX_ERR_NOMEM;
        return YVEX_ERR_NOMEM;
    }
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipMemsetAsync(ptr, 0, (size_t)desc->bytes, yvex_rocm_stream(state)),
                          where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO,
                                   "rocm.tensor_alloc.zero_sync", err);
    tensor = rc == YVEX_OK ? (yvex_device_tensor *)calloc(1, sizeof(*tensor)) : NULL;
    if (rc == YVEX_OK && !tensor) rc = refuse(err, YVEX_ERR_NOMEM, where, "failed to allocate ROCm tensor object");
    if (rc == YVEX_OK && !(tensor->name = text_dup(desc->name))) {
        free(tensor);
        rc = refuse(err, YVEX_ERR_NOMEM, where, "failed to copy ROCm tensor name");
    }
    if (rc != YVEX_OK) {
        (void)state->driver.hipFree(ptr);
        return rc;
    }
    tensor->owner = backend;
    tensor->owner_id = backend->tensor_id_next++;
    tensor->dtype = desc->dtype;
    tensor->rank = desc->rank;
    for (i = 0; i < desc->rank; ++i) tensor->dims[i] = desc->dims[i];
    tensor->bytes = desc->bytes;
    tensor->data = (unsigned char *)ptr;
    tensor->backend_allocation = ptr;
    backend_memory_acquire(backend, desc->bytes);
    state->live_tensors += 1ull;
    *out = tensor;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_tensor_free(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err)
{
    static const char where[] = "rocm.tensor_free";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!backend || !state || !tensor)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and tensor are required");
    if (!backend_tensor_owner_is(backend, tensor))
        return refuse(err, YVEX_ERR_STATE, where, "tensor does not belong to this backend");
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where,
                      "not available while a launch sequence is being recorded");
    /* a recorded sequence holds the device addresses of the tensors its operations named and
     * of the workspace: none of them may go away before the sequence does */
    if (!backend_cleanup_only(backend)) {
        const yvex_rocm_graph *graph;
        for (graph = state->graphs; graph; graph = graph->next)
            if (tensor->owner_id < graph->tensor_id_mark)
                return refuse(err, YVEX_ERR_STATE, where,
                              "a recorded launch sequence may still name this tensor: release the "
                              "sequence first");
    }
    if (backend->workspace_device_tensor == tensor) yvex_backend_workspace_detach(backend);
    /* nothing may still read the allocation: drain the stream first */
    rc = yvex_rocm_status(&state->driver, state->driver.hipStreamSynchronize(yvex_rocm_stream(state)), where,
                          err);
    if (rc == YVEX_OK && getenv("YVEX_TEST_ROCM_CLEANUP_FAILURE"))
        rc = refuse(err, YVEX_ERR_BACKEND, where, "injected ROCm tensor cleanup failure");
    if (rc == YVEX_OK && tensor->virtual_reserved)
        rc = yvex_rocm_virtual_release(backend, tensor, err);
    else if (rc == YVEX_OK && tensor->backend_allocation)
        rc = yvex_rocm_status(&state->driver, state->driver.hipFree(tensor->backend_allocation),
                              where, err);
    if (rc != YVEX_OK) {
        state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return rc;
    }
    /* the pages of a virtual range were counted, and given back, extent by extent */
    if (!tensor->virtual_reserved) backend_memory_release(backend, tensor->bytes);
    if (state->live_tensors) state->live_tensors -= 1ull;
    tensor->owner = NULL;
    tensor->owner_id = 0ull;
    free(tensor->name);
    free(tensor);
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_copy(yvex_backend *backend, void *dst, const void *src, unsigned long long bytes,
                     hipMemcpyKind kind, yvex_backend_operation_variant variant, const char *where,
                     yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc = yvex_rocm_require_capability(backend, variant, where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipMemcpyAsync(dst, src, (size_t)bytes, kind, yvex_rocm_stream(state)),
                          where, err);
    if (rc == YVEX_OK) rc = yvex_rocm_synchronize(backend, variant, where, err);
    return rc;
}

static int rocm_tensor_write(yvex_backend *backend, yvex_device_tensor *tensor, const void *src,
                             unsigned long long len, yvex_error *err)
{
    static const char where[] = "rocm.tensor_write";
    int rc = yvex_backend_tensor_rw_validate(where, backend, tensor, len, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_tensor_backed(tensor)) return refuse(err, YVEX_ERR_STATE, where, kUnbacked);
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_WRITE, where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_small_write(backend, tensor->data, src, len, where, err);
    if (rc == YVEX_ERR_UNSUPPORTED)
        rc = rocm_copy(backend, tensor->data, src, len, hipMemcpyHostToDevice,
                       YVEX_BACKEND_VARIANT_TENSOR_WRITE, where, err);
    if (rc != YVEX_OK) return rc;
    backend->stats.h2d_bytes += len;
    tensor->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_tensor_read(yvex_backend *backend, const yvex_device_tensor *tensor, void *dst,
                            unsigned long long len, yvex_error *err)
{
    static const char where[] = "rocm.tensor_read";
    int rc = yvex_backend_tensor_rw_validate(where, backend, tensor, len, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_tensor_backed(tensor)) return refuse(err, YVEX_ERR_STATE, where, kUnbacked);
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_READ, where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_small_read(backend, dst, tensor->data, len, where, err);
    if (rc == YVEX_ERR_UNSUPPORTED)
        rc = rocm_copy(backend, dst, tensor->data, len, hipMemcpyDeviceToHost,
                       YVEX_BACKEND_VARIANT_TENSOR_READ, where, err);
    if (rc != YVEX_OK) return rc;
    backend->stats.d2h_bytes += len;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_tensor_zero(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err)
{
    static const char where[] = "rocm.tensor_zero";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!backend_tensor_owner_is(backend, tensor))
        return refuse(err, YVEX_ERR_STATE, where, "tensor does not belong to this backend");
    if (!yvex_rocm_tensor_backed(tensor)) return refuse(err, YVEX_ERR_STATE, where, kUnbacked);
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO, where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipMemsetAsync(tensor->data, 0, (size_t)tensor->bytes,
                                                       yvex_rocm_stream(state)),
                          where, err);
    if (rc == YVEX_OK) rc = yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_ZERO, where, err);
    if (rc != YVEX_OK) return rc;
    tensor->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_tensor_copy(yvex_backend *backend, yvex_device_tensor *dst,
                            const yvex_device_tensor *src, yvex_error *err)
{
    static const char where[] = "rocm.tensor_copy";
    int rc = yvex_backend_tensor_copy_validate(backend, dst, src, where, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_tensor_backed(dst) || !yvex_rocm_tensor_backed(src))
        return refuse(err, YVEX_ERR_STATE, where, kUnbacked);
    rc = rocm_copy(backend, dst->data, src->data, src->bytes, hipMemcpyDeviceToDevice,
                   YVEX_BACKEND_VARIANT_TENSOR_COPY, where, err);
    if (rc != YVEX_OK) return rc;
    dst->is_written = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/cuda/backend.c:1159-1191: the copy goes on the launch stream and is not waited
 * for; whatever is enqueued behind it sees the bytes. */
/* ---- queued copies ----------------------------------------------------------------------
 * The reference's session layer appends every new token to a layer's history with two
 * asynchronous copies of one row each (src/runtime/stateful_attention.c:183-222): 4096 calls
 * for a prompt of 2048 tokens, each a launch of its own if handed to the runtime one by one.
 * Small copies wait in a queue instead and leave together, one launch per
 * YVEX_ROCM_COPY_BATCH_MAX of them, as soon as anything else is asked of the stream
 * (yvex_rocm_stream): the order the caller sees is the stream's order.  The copies of one
 * launch run side by side, so one that touches what a queued one writes, or writes what a
 * queued one reads, sends the queue off first. */
enum { ROCM_COPY_QUEUE_BYTES_MAX = 256 * 1024, ROCM_COPY_PIECE_BYTES = 256 * 16 };

void yvex_rocm_copy_queue_flush(yvex_rocm_backend_state *state)
{
    const uint32_t count = state->copy_queue.count;
    void *arguments[1] = {&state->copy_queue.params};
    unsigned int columns = (state->copy_queue.largest + ROCM_COPY_PIECE_BYTES - 1u) / ROCM_COPY_PIECE_BYTES;
    uint32_t i;
    if (!count) return;
    state->copy_queue.count = 0u; /* first: the stream is taken below without another flush */
    state->copy_queue.largest = 0u;
    if (columns > 16u) columns = 16u;
    if (state->functions[YVEX_ROCM_FN_COPY_BATCH] &&
        state->driver.hipModuleLaunchKernel(state->functions[YVEX_ROCM_FN_COPY_BATCH], columns, count, 1u,
                                            256u, 1u, 1u, 0u, state->stream_handle, arguments,
                                            NULL) == hipSuccess)
        return;
    /* the launch was refused: the copies one by one; what still fails is reported by the next wait */
    for (i = 0u; i < count; ++i)
        if (state->driver.hipMemcpyAsync((void *)(uintptr_t)state->copy_queue.params.dst[i],
                                         (const void *)(uintptr_t)state->copy_queue.params.src[i],
                                         state->copy_queue.params.bytes[i], hipMemcpyDeviceToDevice,
                                         state->stream_handle) != hipSuccess)
            state->copy_queue.failed = 1;
}

static int ranges_meet(uint64_t a, uint64_t a_bytes, uint64_t b, uint64_t b_bytes)
{
    return a < b + b_bytes && b < a + a_bytes;
}

/* 1 when the copy was queued, 0 when it is for the runtime (large, not in 16-byte pieces, or
 * no kernel to carry it). */
static int copy_queue_take(yvex_rocm_backend_state *state, const void *dst, const void *src,
                           unsigned long long bytes)
{
    yvex_rocm_copy_batch_params *q = &state->copy_queue.params;
    const uint64_t to = (uint64_t)(uintptr_t)dst, from = (uint64_t)(uintptr_t)src;
    uint32_t i;
    if (!state->functions[YVEX_ROCM_FN_COPY_BATCH] || !bytes || bytes > ROCM_COPY_QUEUE_BYTES_MAX ||
        ((to | from | bytes) & 15ull))
        return 0;
    for (i = 0u; i < state->copy_queue.count; ++i)
        if (ranges_meet(to, bytes, q->dst[i], q->bytes[i]) || ranges_meet(to, bytes, q->src[i], q->bytes[i]) ||
            ranges_meet(from, bytes, q->dst[i], q->bytes[i])) {
            yvex_rocm_copy_queue_flush(state);
            break;
        }
    if (state->copy_queue.count == YVEX_ROCM_COPY_BATCH_MAX) yvex_rocm_copy_queue_flush(state);
    i = state->copy_queue.count++;
    q->dst[i] = to;
    q->src[i] = from;
    q->bytes[i] = (uint32_t)bytes;
    if ((uint32_t)bytes > state->copy_queue.largest) state->copy_queue.largest = (uint32_t)bytes;
    return 1;
}

static int rocm_tensor_copy_async(yvex_backend *backend, yvex_device_tensor *dst,
                                  const yvex_device_tensor *src, yvex_error *err)
{
    static const char where[] = "runtime.state.residency.copy";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc = yvex_backend_tensor_copy_validate(backend, dst, src, where, err);
    if (rc != YVEX_OK) return rc;
    if (!state || backend->kind != YVEX_BACKEND_KIND_ROCM)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "ROCm state residency requires a ROCm backend");
    if (!yvex_rocm_tensor_backed(dst) || !yvex_rocm_tensor_backed(src))
        return refuse(err, YVEX_ERR_STATE, where, kUnbacked);
    rc = yvex_rocm_require_capability(backend, YVEX_BACKEND_VARIANT_TENSOR_COPY, where, err);
    if (rc != YVEX_OK) return rc;
    if (!copy_queue_take(state, dst->data, src->data, src->bytes))
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemcpyAsync(dst->data, src->data, (size_t)src->bytes,
                                                           hipMemcpyDeviceToDevice, yvex_rocm_stream(state)),
                              where, err);
    if (rc != YVEX_OK) return rc;
    dst->is_written = src->is_written;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/cuda/backend.c:1194-1265: the source belongs to another backend of the same
 * device.  An event recorded on the source's stream makes the copy wait for whatever produces
 * the source; an event recorded behind the copy makes the source's stream wait before it
 * overwrites it.  Both events are released at once: the runtime keeps what a recorded event
 * needs until the waits that name it have passed. */
static int rocm_tensor_copy_shared_async(yvex_backend *backend, yvex_device_tensor *dst,
                                         const yvex_device_tensor *src, yvex_error *err)
{
    static const char where[] = "backend.tensor.copy-shared";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_backend_state *source_state = src && src->owner ? yvex_rocm_state(src->owner) : NULL;
    hipEvent_t ready = NULL, consumed = NULL;
    int rc = YVEX_OK, cleanup;
    if (!state || !source_state || !dst || !state->stream_handle || !source_state->stream_handle)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where, "ROCm cross-stream event ordering is unavailable");
    if (!yvex_rocm_tensor_backed(dst) || !yvex_rocm_tensor_backed(src))
        return refuse(err, YVEX_ERR_STATE, where, kUnbacked);
    if (source_state->stream_handle != state->stream_handle) {
        rc = yvex_rocm_status(&state->driver, state->driver.hipEventCreate(&ready), where, err);
        if (rc == YVEX_OK)
            rc = yvex_rocm_status(&state->driver, state->driver.hipEventCreate(&consumed), where, err);
        if (rc == YVEX_OK)
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipEventRecord(ready, yvex_rocm_stream(source_state)), where, err);
        if (rc == YVEX_OK)
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipStreamWaitEvent(yvex_rocm_stream(state), ready, 0u), where, err);
    }
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemcpyAsync(dst->data, src->data, (size_t)src->bytes,
                                                           hipMemcpyDeviceToDevice, yvex_rocm_stream(state)),
                              where, err);
    if (rc == YVEX_OK && consumed) {
        rc = yvex_rocm_status(&state->driver, state->driver.hipEventRecord(consumed, yvex_rocm_stream(state)),
                              where, err);
        if (rc == YVEX_OK)
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipStreamWaitEvent(yvex_rocm_stream(source_state), consumed, 0u),
                                  where, err);
    }
    if (consumed) {
        cleanup = yvex_rocm_status(&state->driver, state->driver.hipEventDestroy(consumed), where,
                                   rc == YVEX_OK ? err : NULL);
        if (rc == YVEX_OK) rc = cleanup;
    }
    if (ready) {
        cleanup = yvex_rocm_status(&state->driver, state->driver.hipEventDestroy(ready), where,
                                   rc == YVEX_OK ? err : NULL);
        if (rc == YVEX_OK) rc = cleanup;
    }
    if (rc != YVEX_OK) return rc;
    dst->is_written = src->is_written;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* Synchronise; in DEFERRED completion mode this is also where the device status word of
 * the operations enqueued since the last check is read and reported. */
static int rocm_sync(yvex_backend *backend, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    if (state && state->recording)
        return refuse(err, YVEX_ERR_STATE, "rocm.sync",
                      "cannot wait for the stream while a launch sequence is being recorded");
    if (state && state->status_dirty)
        return yvex_rocm_status_check(backend, "rocm.sync.status", NULL, err);
    return yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_READ, "rocm.sync", err);
}

/* ---------------------------------------------------------- bandwidth ---- */

static unsigned long long median_of(const unsigned long long *samples, unsigned int count)
{
    unsigned long long sorted[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned int i, j;
    for (i = 0; i < count; ++i) {
        unsigned long long value = samples[i];
        for (j = i; j > 0 && sorted[j - 1] > value; --j) sorted[j] = sorted[j - 1];
        sorted[j] = value;
    }
    return sorted[count / 2u];
}

/* One timed sample: `iterations` passes of the streaming read, or of the copy. */
static int bandwidth_sample(yvex_backend *backend, yvex_device_tensor *source,
                            yvex_device_tensor *copy, yvex_device_tensor *sink, int copying,
                            unsigned long long iterations, unsigned long long *elapsed_ns,
                            yvex_error *err)
{
    static const char where[] = "rocm.bandwidth";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_stream_params params;
    unsigned long long i;
    double milliseconds = 0.0;
    int rc;
    memset(&params, 0, sizeof(params));
    params.data = source->data;
    params.sink = (uint32_t *)sink->data;
    params.words = source->bytes / 16ull;
    params.never = 0x5ca1ab1eu; /* the working set is all zero */
    rc = yvex_backend_rocm_timing_begin(backend, err);
    for (i = 0; rc == YVEX_OK && i < iterations; ++i) {
        if (copying)
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipMemcpyAsync(copy->data, source->data,
                                                               (size_t)source->bytes,
                                                               hipMemcpyDeviceToDevice,
                                                               yvex_rocm_stream(state)),
                                  where, err);
        else
            rc = yvex_rocm_launch(backend, YVEX_ROCM_FN_STREAM_READ,
                                  YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
                                  (unsigned int)(state->compute_units > 0 ? state->compute_units * 8 : 2048),
                                  1u, 1u, 256u, 0u, &params, where, err);
    }
    if (rc == YVEX_OK) rc = yvex_backend_rocm_timing_end(backend, &milliseconds, err);
    else state->timing_active = 0;
    if (rc != YVEX_OK) return rc;
    *elapsed_ns = (unsigned long long)(milliseconds * 1.0e6);
    if (!*elapsed_ns) *elapsed_ns = 1ull;
    return YVEX_OK;
}

/* src/backend/cuda/backend.c:1428-1530: allocate the working set, warm up, take the samples,
 * publish medians; the evidence of the first successful run is kept. */
static int rocm_bandwidth_probe(yvex_backend *backend, yvex_backend_bandwidth_evidence *out,
                                yvex_error *err)
{
    static const char where[] = "rocm.bandwidth";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_backend_bandwidth_evidence evidence;
    yvex_backend_tensor_desc descriptor;
    yvex_device_tensor *source = NULL, *copy = NULL, *sink = NULL;
    const char *forced = getenv("YVEX_TEST_ROCM_BANDWIDTH_BYTES");
    unsigned long long scratch;
    yvex_error cleanup;
    unsigned int sample;
    int rc;
    if (!state || !out) return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and out are required");
    if (state->bandwidth_ready) {
        *out = state->bandwidth_evidence;
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (state->kernel_bundle_state != YVEX_ROCM_KERNEL_BUNDLE_ADMITTED)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where, "no kernel bundle is admitted");
    if (state->recording || state->timing_active)
        return refuse(err, YVEX_ERR_STATE, where, "close the recording or timing section first");
    memset(&evidence, 0, sizeof(evidence));
    evidence.schema_version = YVEX_BACKEND_BANDWIDTH_SCHEMA_V1;
    /* well beyond the 256 MB last-level cache of the part */
    evidence.working_set_bytes = forced && atoll(forced) >= 8192 ? (unsigned long long)atoll(forced) & ~8191ull
                                                                 : 1ull << 30;
    evidence.iterations = 8ull;
    evidence.sample_count = YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT;
    memset(&descriptor, 0, sizeof(descriptor));
    descriptor.dtype = YVEX_DTYPE_I8;
    descriptor.rank = 1u;
    descriptor.dims[0] = descriptor.bytes = evidence.working_set_bytes;
    descriptor.name = "bandwidth-source";
    rc = yvex_backend_tensor_alloc(backend, &descriptor, &source, err);
    descriptor.name = "bandwidth-copy";
    if (rc == YVEX_OK) rc = yvex_backend_tensor_alloc(backend, &descriptor, &copy, err);
    descriptor.name = "bandwidth-sink";
    descriptor.dims[0] = descriptor.bytes = 256ull;
    if (rc == YVEX_OK) rc = yvex_backend_tensor_alloc(backend, &descriptor, &sink, err);
    /* warm-up pass of each kind, not timed */
    if (rc == YVEX_OK) rc = bandwidth_sample(backend, source, copy, sink, 0, 1ull, &scratch, err);
    if (rc == YVEX_OK) rc = bandwidth_sample(backend, source, copy, sink, 1, 1ull, &scratch, err);
    for (sample = 0u; rc == YVEX_OK && sample < evidence.sample_count; ++sample)
        rc = bandwidth_sample(backend, source, copy, sink, 0, evidence.iterations,
                              &evidence.stream_elapsed_ns[sample], err);
    for (sample = 0u; rc == YVEX_OK && sample < evidence.sample_count; ++sample)
        rc = bandwidth_sample(backend, source, copy, sink, 1, evidence.iterations,
                              &evidence.copy_elapsed_ns[sample], err);
    if (rc == YVEX_OK) {
        const double read_ns = (double)median_of(evidence.stream_elapsed_ns, evidence.sample_count);
        const double copy_ns = (double)median_of(evidence.copy_elapsed_ns, evidence.sample_count);
        const double bytes = (double)evidence.working_set_bytes * (double)evidence.iterations;
        evidence.sustainable_read_bytes_per_second = (unsigned long long)(bytes / read_ns * 1.0e9);
        evidence.sustainable_copy_bytes_per_second = (unsigned long long)(2.0 * bytes / copy_ns * 1.0e9);
    }
    yvex_error_clear(&cleanup);
    if (sink) (void)yvex_backend_tensor_release(backend, &sink, &cleanup);
    if (copy) (void)yvex_backend_tensor_release(backend, &copy, &cleanup);
    if (source) (void)yvex_backend_tensor_release(backend, &source, &cleanup);
    if (rc != YVEX_OK) return rc;
    state->bandwidth_evidence = evidence;
    state->bandwidth_ready = 1;
    *out = evidence;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_memory_stats(const yvex_backend *backend, yvex_backend_memory_stats *out,
                             yvex_error *err)
{
    *out = backend->stats;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int rocm_device_info(const yvex_backend *backend, yvex_backend_device_info *out,
                            yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    size_t free_bytes = 0u, total_bytes = 0u;
    *out = backend->device_info;
    if (state && state->stream_handle &&
        state->driver.hipMemGetInfo(&free_bytes, &total_bytes) == hipSuccess) {
        out->free_memory_bytes = free_bytes;
        out->total_memory_bytes = total_bytes;
    }
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ---------------------------------------------------------- temporaries ---- */

/* Operation temporaries come from the attached workspace when it has room
 * (src/backend/residency.c:251-283), otherwise from a counted allocation that the
 * operation releases before it returns. */
int yvex_rocm_temporary_acquire(yvex_backend *backend, unsigned long long bytes, void **address,
                                int *owned, const char *where, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    unsigned long long device_address = 0ull;
    int hit = yvex_backend_workspace_acquire(backend, bytes, 256ull, &device_address);
    *address = NULL;
    *owned = 0;
    if (hit == YVEX_BACKEND_RESIDENT_HIT) {
        *address = (void *)(uintptr_t)device_address;
        return YVEX_OK;
    }
    if (hit == YVEX_BACKEND_RESIDENT_INVALID)
        return refuse(err, YVEX_ERR_BOUNDS, where, "temporary workspace geometry is invalid");
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where,
                      "a recorded operation needs an attached workspace that holds its temporaries");
    if (getenv("YVEX_TEST_ROCM_ATTENTION_FAILURE") &&
        strcmp(getenv("YVEX_TEST_ROCM_ATTENTION_FAILURE"), "allocation") == 0)
        return refuse(err, YVEX_ERR_NOMEM, where, "injected ROCm temporary allocation failure");
    if (yvex_backend_memory_can_add(backend, bytes, "ROCm", where, err) != YVEX_OK)
        return YVEX_ERR_NOMEM;
    if (yvex_rocm_status(&state->driver, state->driver.hipMalloc(address, (size_t)bytes), where,
                         err) != YVEX_OK) {
        if (err) err->code = YVEX_ERR_NOMEM;
        return YVEX_ERR_NOMEM;
    }
    backend_memory_acquire(backend, bytes);
    *owned = 1;
    return YVEX_OK;
}

int yvex_rocm_temporary_release(yvex_backend *backend, void *address, unsigned long long bytes,
                                int owned, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!owned || !address) return YVEX_OK;
    rc = yvex_rocm_status(&state->driver, state->driver.hipStreamSynchronize(yvex_rocm_stream(state)),
                          "rocm.temporary.release", err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipFree(address),
                              "rocm.temporary.release", err);
    if (rc != YVEX_OK) {
        state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return rc;
    }
    backend_memory_release(backend, bytes);
    return YVEX_OK;
}

/* ------------------------------------------------------- open and close ---- */

static int rocm_close(yvex_backend *backend, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!state) {
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (state->recording) { /* an abandoned recording: end it and drop what it held */
        hipGraph_t dropped = NULL;
        (void)state->driver.hipStreamEndCapture(yvex_rocm_stream(state), &dropped);
        if (dropped) (void)state->driver.hipGraphDestroy(dropped);
        state->recording = 0;
    }
    if (state->stream_handle) (void)state->driver.hipStreamSynchronize(yvex_rocm_stream(state));
    rc = yvex_rocm_kernel_bundle_close(backend, err);
    if (rc != YVEX_OK) return rc; /* impl retained: checked close can be retried */
    if (state->device_status) (void)state->driver.hipFree(state->device_status);
    if (state->status_mailbox) (void)state->driver.hipHostFree((void *)state->status_mailbox);
    if (state->decode_arrivals) (void)state->driver.hipFree(state->decode_arrivals);
    if (state->schedule_device) (void)state->driver.hipFree(state->schedule_device);
    probe_release(state);
    if (state->timing_start) (void)state->driver.hipEventDestroy(state->timing_start);
    if (state->timing_stop) (void)state->driver.hipEventDestroy(state->timing_stop);
    if (state->stream_handle) (void)state->driver.hipStreamDestroy(state->stream_handle);
    yvex_rocm_driver_unload(&state->driver);
    free(state);
    backend->impl = NULL;
    yvex_error_clear(err);
    return YVEX_OK;
}

static const yvex_backend_vtable rocm_vtable = {
    .close = rocm_close,
    .memory_stats = rocm_memory_stats,
    .device_info = rocm_device_info,
    .tensor_alloc = rocm_tensor_alloc,
    .tensor_reserve = yvex_rocm_tensor_reserve,
    .tensor_commit = yvex_rocm_tensor_commit,
    .tensor_decommit = yvex_rocm_tensor_decommit,
    .tensor_free = rocm_tensor_free,
    .tensor_write = rocm_tensor_write,
    .tensor_read = rocm_tensor_read,
    .tensor_zero = rocm_tensor_zero,
    .tensor_copy = rocm_tensor_copy,
    .tensor_copy_async = rocm_tensor_copy_async,
    .tensor_copy_shared_async = rocm_tensor_copy_shared_async,
    .sync = rocm_sync,
    .bandwidth_probe = rocm_bandwidth_probe,
    .query_capability = yvex_rocm_query_capability,
    .op_attention = yvex_rocm_op_attention,
    .transformer_operations = yvex_rocm_transformer_operations,
};

static int parse_device(const char *device, int *index)
{
    char *end = NULL;
    long value;
    *index = 0;
    if (!device || !*device) return 1;
    value = strtol(device, &end, 10);
    if (!end || *end != '\0' || value < 0 || value > 1023) return 0;
    *index = (int)value;
    return 1;
}

/* The fixed device array of the entry point that allocates nothing lives in a companion
 * object that is linked against the HIP runtime; this library is not, so that it loads (and
 * answers "unsupported") on a machine without the runtime.  The companion is looked up beside
 * this library and only when the runtime in use is the real one: under a substituted runtime
 * (YVEX_TEST_ROCM_DRIVER_LIBRARY) no second runtime is brought into the process.  Its absence
 * only disables that entry point. */
static void scratch_companion_resolve(yvex_rocm_backend_state *state)
{
    static void *companion;
    const char *override = getenv("YVEX_TEST_ROCM_DRIVER_LIBRARY");
    yvex_rocm_static_scratch_resolve_fn resolve;
    Dl_info self;
    char path[4096];
    const char *slash;
    size_t directory;
    state->static_scratch = NULL;
    state->static_scratch_error = 0;
    if (override && *override) return;
    if (!companion) {
        if (!dladdr((void *)&scratch_companion_resolve, &self) || !self.dli_fname) return;
        slash = strrchr(self.dli_fname, '/');
        directory = slash ? (size_t)(slash - self.dli_fname) + 1u : 0u;
        if (directory + sizeof(YVEX_ROCM_SCRATCH_LIBRARY) > sizeof(path)) return;
        memcpy(path, self.dli_fname, directory);
        memcpy(path + directory, YVEX_ROCM_SCRATCH_LIBRARY, sizeof(YVEX_ROCM_SCRATCH_LIBRARY));
        /* stays mapped for the life of the process, like the runtime itself */
        companion = dlopen(path, RTLD_NOW | RTLD_LOCAL);
        if (!companion) return;
    }
    resolve = (yvex_rocm_static_scratch_resolve_fn)dlsym(companion, YVEX_ROCM_SCRATCH_RESOLVE_SYMBOL);
    if (resolve)
        (void)resolve(state->device_index, &state->static_scratch, &state->static_scratch_error);
}

/* `owner` NULL: a primary backend on the device named by `device`.  Otherwise a session
 * backend on the owner's device; the caller holds the lease on the owner. */
static int rocm_open(yvex_backend **out, const char *device, unsigned long long memory_limit_bytes,
                     yvex_backend *owner, yvex_error *err)
{
    static const char where[] = "yvex_backend_open_rocm";
    yvex_backend *backend;
    yvex_rocm_backend_state *state;
    yvex_error admit;
    int count = 0, value = 0, rc;
    size_t total = 0u;
    if (!out) return refuse(err, YVEX_ERR_INVALID_ARG, where, "out is required");
    *out = NULL;
    backend = (yvex_backend *)calloc(1, sizeof(*backend));
    state = (yvex_rocm_backend_state *)calloc(1, sizeof(*state));
    if (state) state->probe_function = -1;
    if (!backend || !state) {
        free(backend);
        free(state);
        return refuse(err, YVEX_ERR_NOMEM, where, "failed to allocate ROCm backend");
    }
    backend->kind = YVEX_BACKEND_KIND_ROCM;
    backend->status = YVEX_BACKEND_STATUS_UNSUPPORTED;
    backend->vtable = &rocm_vtable;
    backend->impl = state;
    backend->tensor_id_next = 1ull;
    backend->stats.memory_limit_bytes = memory_limit_bytes;
    state->kernel_bundle_reason = YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT;
    state->kernel_bundle_failure_variant = YVEX_BACKEND_VARIANT_COUNT;

    backend->resource_owner = owner ? owner : backend;
    if (owner) {
        state->device_index = yvex_rocm_state(owner)->device_index;
        rc = YVEX_OK;
    } else {
        rc = parse_device(device, &state->device_index)
                 ? YVEX_OK
                 : refuse(err, YVEX_ERR_INVALID_ARG, where, "device must be a non-negative index");
    }
    if (rc == YVEX_OK) rc = yvex_rocm_driver_load(&state->driver, err);
    if (rc == YVEX_OK && state->driver.hipInit(0u) != hipSuccess)
        rc = refuse(err, YVEX_ERR_UNSUPPORTED, where, "HIP runtime initialisation failed");
    if (rc == YVEX_OK &&
        (state->driver.hipGetDeviceCount(&count) != hipSuccess || count <= state->device_index))
        rc = refuse(err, YVEX_ERR_UNSUPPORTED, where, "no usable ROCm device");
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipSetDevice(state->device_index),
                              where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipStreamCreate(&state->stream_handle), where,
                              err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipEventCreate(&state->timing_start),
                              where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipEventCreate(&state->timing_stop),
                              where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMalloc((void **)&state->device_status, 256u), where,
                              err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemsetAsync(state->device_status, 0, 256u,
                                                           yvex_rocm_stream(state)),
                              where, err);
    if (rc == YVEX_OK && state->driver.pinned_memory) {
        /* the status mailbox is an economy, not a requirement: without it the word is copied */
        void *host = NULL, *mapped = NULL;
        if (state->driver.hipHostMalloc(&host, 256u + YVEX_ROCM_SMALL_READ_MAX, hipHostMallocMapped) ==
                hipSuccess && host) {
            if (state->driver.hipHostGetDevicePointer(&mapped, host, 0u) == hipSuccess && mapped) {
                memset(host, 0, 256u + YVEX_ROCM_SMALL_READ_MAX);
                state->status_mailbox = (volatile uint64_t *)host;
                state->status_mailbox_device = (uint64_t *)mapped;
                state->read_staging = (unsigned char *)host + 256u;
                state->read_staging_device = (unsigned char *)mapped + 256u;
            } else {
                (void)state->driver.hipHostFree(host);
            }
        }
    }
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMalloc((void **)&state->decode_arrivals,
                                                      YVEX_ROCM_DECODE_SEGMENTS_MAX * sizeof(uint32_t)),
                              where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemsetAsync(state->decode_arrivals, 0,
                                                           YVEX_ROCM_DECODE_SEGMENTS_MAX * sizeof(uint32_t),
                                                           yvex_rocm_stream(state)),
                              where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMalloc((void **)&state->schedule_device,
                                                      sizeof(state->schedule.rows)),
                              where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipStreamSynchronize(yvex_rocm_stream(state)),
                              where, err);
    if (rc != YVEX_OK) {
        yvex_error keep = err ? *err : (yvex_error){0};
        yvex_error scratch;
        if (state->device_status) (void)state->driver.hipFree(state->device_status);
        if (state->status_mailbox) (void)state->driver.hipHostFree((void *)state->status_mailbox);
        if (state->decode_arrivals) (void)state->driver.hipFree(state->decode_arrivals);
        if (state->schedule_device) (void)state->driver.hipFree(state->schedule_device);
        if (state->timing_start) (void)state->driver.hipEventDestroy(state->timing_start);
        if (state->timing_stop) (void)state->driver.hipEventDestroy(state->timing_stop);
        if (state->stream_handle) (void)state->driver.hipStreamDestroy(state->stream_handle);
        (void)scratch;
        free(state);
        free(backend);
        if (err) *err = keep;
        return rc;
    }

    /* the fixed scratch of the entry point that allocates nothing: resolved here, once per
     * device, with the device current; its absence only disables that entry point */
    scratch_companion_resolve(state);

    backend->device_info.kind = YVEX_BACKEND_KIND_ROCM;
    backend->device_info.device_index = state->device_index;
    if (state->driver.hipDeviceGetName(backend->device_name_storage,
                                       (int)sizeof(backend->device_name_storage),
                                       state->device_index) != hipSuccess ||
        backend->device_name_storage[0] == '\0') /* some drivers publish an empty marketing name */
        yvex_core_text_copy(backend->device_name_storage, sizeof(backend->device_name_storage),
                            "rocm");
    backend->device_info.name = backend->device_name_storage;
    if (state->driver.hipDeviceGetAttribute(&value, hipDeviceAttributeComputeCapabilityMajor,
                                            state->device_index) == hipSuccess)
        backend->device_info.compute_capability_major = value;
    if (state->driver.hipDeviceGetAttribute(&value, hipDeviceAttributeComputeCapabilityMinor,
                                            state->device_index) == hipSuccess)
        backend->device_info.compute_capability_minor = value;
    if (state->driver.hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount,
                                            state->device_index) == hipSuccess)
        state->compute_units = value;
    state->virtual_memory =
        state->driver.virtual_memory &&
        state->driver.hipDeviceGetAttribute(&value,
                                            hipDeviceAttributeVirtualMemoryManagementSupported,
                                            state->device_index) == hipSuccess &&
        value != 0;
    backend->virtual_tensor_ready = state->virtual_memory;
    if (state->driver.hipDeviceTotalMem(&total, state->device_index) == hipSuccess) {
        backend->device_info.global_memory_bytes = total;
        backend->device_info.total_memory_bytes = total;
    }
    backend->device_info.unified_addressing = 1;

    backend->status = YVEX_BACKEND_STATUS_CONTEXT_READY;
    yvex_error_clear(&admit);
    if (yvex_rocm_kernel_bundle_admit(backend, &admit) == YVEX_OK)
        backend->status = YVEX_BACKEND_STATUS_READY;
    else if (!state->kernel_bundle_rejection[0])
        yvex_core_text_copy(state->kernel_bundle_rejection,
                            sizeof(state->kernel_bundle_rejection), admit.message);
    *out = backend;
    yvex_error_clear(err);
    return YVEX_OK;
}

int yvex_backend_open_rocm_impl(yvex_backend **out, const char *device,
                                unsigned long long memory_limit_bytes, yvex_error *err)
{
    return rocm_open(out, device, memory_limit_bytes, NULL, err);
}

/* src/backend/cuda/backend.c:1795-1879.  HIP has no context object to lend: what a session
 * backend takes from its primary is the device, and the lease that keeps the primary open. */
int yvex_backend_open_shared_rocm(yvex_backend **out, yvex_backend *context_owner,
                                  unsigned long long memory_limit_bytes, yvex_error *err)
{
    static const char where[] = "rocm.shared.open";
    int rc;
    if (out) *out = NULL;
    if (!out || !context_owner || context_owner->kind != YVEX_BACKEND_KIND_ROCM ||
        context_owner->resource_owner != context_owner || !yvex_rocm_state(context_owner))
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "one owning ROCm backend is required");
    rc = yvex_backend_shared_owner_acquire(context_owner, err);
    if (rc != YVEX_OK) return rc;
    /* from here on the primary waits for its small writes (yvex_rocm_small_write); the ones it
     * made while it was alone are waited for now, before another stream can read them */
    rc = yvex_rocm_synchronize(context_owner, YVEX_BACKEND_VARIANT_TENSOR_WRITE, where, err);
    if (rc == YVEX_OK) rc = rocm_open(out, NULL, memory_limit_bytes, context_owner, err);
    if (rc != YVEX_OK) {
        /* nothing was published: give the lease back */
        atomic_fetch_sub_explicit(&context_owner->lifecycle, 1ull, memory_order_acq_rel);
        return rc;
    }
    (*out)->shared_owner_registered = 1;
    return YVEX_OK;
}

/* ------------------------------------------------------ NEW SURFACE bits ---- */

int yvex_backend_rocm_completion_mode_set(yvex_backend *backend, yvex_rocm_completion_mode mode,
                                          yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!state || (mode != YVEX_ROCM_COMPLETION_IMMEDIATE && mode != YVEX_ROCM_COMPLETION_DEFERRED))
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.completion_mode",
                      "ROCm backend and a known completion mode are required");
    rc = backend_dispatch_admit(backend, "rocm.completion_mode", err);
    if (rc != YVEX_OK) return rc;
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, "rocm.completion_mode",
                      "not available while a launch sequence is being recorded");
    if (state->status_dirty) {
        rc = yvex_rocm_status_check(backend, "rocm.completion_mode", NULL, err);
        if (rc != YVEX_OK) return rc;
    }
    state->completion_mode = mode;
    yvex_error_clear(err);
    return YVEX_OK;
}

static void probe_release(yvex_rocm_backend_state *state)
{
    unsigned int i;
    for (i = 0; i < 2u * YVEX_ROCM_PROBE_MAX; ++i)
        if (state->probe_events[i]) {
            (void)state->driver.hipEventDestroy(state->probe_events[i]);
            state->probe_events[i] = NULL;
        }
    state->probe_count = 0u;
    state->probe_function = -1;
}

int yvex_backend_rocm_kernel_probe_begin(yvex_backend *backend, const char *kernel,
                                         yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    unsigned int i;
    int function, rc;
    if (!state || !kernel)
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.probe", "ROCm backend and kernel name are required");
    rc = backend_dispatch_admit(backend, "rocm.probe", err);
    if (rc != YVEX_OK) return rc;
    function = yvex_rocm_function_find(kernel);
    if (function < 0 || !state->functions[function])
        return refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.probe", "no such kernel in the admitted bundle");
    if (state->probe_function >= 0)
        return refuse(err, YVEX_ERR_STATE, "rocm.probe", "a kernel probe is already open");
    for (i = 0; i < 2u * YVEX_ROCM_PROBE_MAX; ++i) {
        if (state->probe_events[i]) continue;
        rc = yvex_rocm_status(&state->driver, state->driver.hipEventCreate(&state->probe_events[i]),
                              "rocm.probe.begin", err);
        if (rc != YVEX_OK) {
            probe_release(state);
            return rc;
        }
    }
    state->probe_count = 0u;
    state->probe_function = function;
    yvex_error_clear(err);
    return YVEX_OK;
}

int yvex_backend_rocm_kernel_probe_end(yvex_backend *backend, unsigned int *launches,
                                       double *milliseconds, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    double total = 0.0;
    unsigned int i;
    int rc = YVEX_OK;
    if (!state || !launches || !milliseconds || state->probe_function < 0)
        return refuse(err, YVEX_ERR_STATE, "rocm.probe.end", "no kernel probe is open");
    state->probe_function = -1;
    if (state->probe_count)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipEventSynchronize(
                                  state->probe_events[2u * state->probe_count - 1u]),
                              "rocm.probe.end", err);
    for (i = 0; rc == YVEX_OK && i < state->probe_count; ++i) {
        float elapsed = 0.0f;
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipEventElapsedTime(&elapsed, state->probe_events[2u * i],
                                                                state->probe_events[2u * i + 1u]),
                              "rocm.probe.end", err);
        total += (double)elapsed;
    }
    *launches = rc == YVEX_OK ? state->probe_count : 0u;
    *milliseconds = rc == YVEX_OK ? total : 0.0;
    state->probe_count = 0u;
    if (rc == YVEX_OK) yvex_error_clear(err);
    return rc;
}

int yvex_backend_rocm_timing_begin(yvex_backend *backend, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!state) return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.timing", "ROCm backend is required");
    rc = backend_dispatch_admit(backend, "rocm.timing", err);
    if (rc != YVEX_OK) return rc;
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, "rocm.timing",
                      "not available while a launch sequence is being recorded");
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipEventRecord(state->timing_start, yvex_rocm_stream(state)),
                          "rocm.timing.begin", err);
    if (rc == YVEX_OK) state->timing_active = 1;
    return rc;
}

int yvex_backend_rocm_timing_end(yvex_backend *backend, double *milliseconds, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    float elapsed = 0.0f;
    int rc;
    if (!state || !milliseconds || !state->timing_active || state->recording)
        return refuse(err, YVEX_ERR_STATE, "rocm.timing.end",
                      "timing was not started, or a launch sequence is being recorded");
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipEventRecord(state->timing_stop, yvex_rocm_stream(state)),
                          "rocm.timing.end", err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver, state->driver.hipEventSynchronize(state->timing_stop),
                              "rocm.timing.end", err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipEventElapsedTime(&elapsed, state->timing_start,
                                                                state->timing_stop),
                              "rocm.timing.end", err);
    state->timing_active = 0;
    if (rc != YVEX_OK) return rc;
    *milliseconds = (double)elapsed;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ---------------------------------------------- recorded launch sequences ---- */

int yvex_backend_rocm_graph_begin(yvex_backend *backend, yvex_error *err)
{
    static const char where[] = "rocm.graph.begin";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!state) return refuse(err, YVEX_ERR_INVALID_ARG, where, "ROCm backend is required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where, "a launch sequence is already being recorded");
    if (state->kernel_bundle_state != YVEX_ROCM_KERNEL_BUNDLE_ADMITTED)
        return refuse(err, YVEX_ERR_UNSUPPORTED, where, "no kernel bundle is admitted");
    if (state->timing_active || state->probe_function >= 0)
        return refuse(err, YVEX_ERR_STATE, where, "close the timing or probe section first");
    /* earlier deferred work is checked before the stream stops executing */
    if (state->status_dirty) {
        rc = yvex_rocm_status_check(backend, where, NULL, err);
        if (rc != YVEX_OK) return rc;
    }
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipStreamBeginCapture(yvex_rocm_stream(state),
                                                              hipStreamCaptureModeThreadLocal),
                          where, err);
    if (rc != YVEX_OK) return rc;
    state->recording = 1;
    state->recorded_launches = 0ull;
    yvex_error_clear(err);
    return YVEX_OK;
}

int yvex_backend_rocm_graph_end(yvex_backend *backend, yvex_rocm_graph **out, yvex_error *err)
{
    static const char where[] = "rocm.graph.end";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_graph *graph;
    hipGraph_t captured = NULL;
    int rc;
    if (out) *out = NULL;
    if (!state || !out) return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and out are required");
    if (!state->recording) return refuse(err, YVEX_ERR_STATE, where, "no launch sequence is being recorded");
    rc = yvex_rocm_status(&state->driver, state->driver.hipStreamEndCapture(yvex_rocm_stream(state), &captured),
                          where, err);
    state->recording = 0;
    if (rc != YVEX_OK) {
        if (captured) (void)state->driver.hipGraphDestroy(captured);
        return rc;
    }
    graph = (yvex_rocm_graph *)calloc(1u, sizeof(*graph));
    if (!graph) {
        (void)state->driver.hipGraphDestroy(captured);
        return refuse(err, YVEX_ERR_NOMEM, where, "out of host memory");
    }
    graph->graph = captured;
    graph->kernel_launches = state->recorded_launches;
    graph->workspace_address = backend->workspace_device_address;
    graph->workspace_bytes = backend->workspace_bytes;
    graph->tensor_id_mark = backend->tensor_id_next;
    rc = yvex_rocm_status(&state->driver,
                          state->driver.hipGraphInstantiate(&graph->executable, captured, NULL, NULL, 0u),
                          where, err);
    if (rc != YVEX_OK) {
        (void)state->driver.hipGraphDestroy(captured);
        free(graph);
        return rc;
    }
    state->live_graphs++;
    graph->next = state->graphs;
    state->graphs = graph;
    *out = graph;
    yvex_error_clear(err);
    return YVEX_OK;
}

int yvex_backend_rocm_graph_launch(yvex_backend *backend, yvex_rocm_graph *graph,
                                   yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.graph.launch";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!state || !graph || !graph->executable)
        return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and a recorded sequence are required");
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where, "a launch sequence is being recorded");
    /* the recorded launches write to the workspace that was attached then: a replay after it
     * was detached or replaced would write to memory the caller has taken back */
    if (graph->kernel_launches && (graph->workspace_address != backend->workspace_device_address ||
                                   graph->workspace_bytes != backend->workspace_bytes))
        return refuse(err, YVEX_ERR_STATE, where,
                      "the workspace attached when the sequence was recorded is no longer attached");
    if (facts) memset(facts, 0, sizeof(*facts));
    rc = yvex_rocm_status(&state->driver, state->driver.hipGraphLaunch(graph->executable, yvex_rocm_stream(state)),
                          where, err);
    if (rc != YVEX_OK) {
        state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_LAUNCH_FAILED;
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return rc;
    }
    if (facts) {
        facts->kernel_launches = graph->kernel_launches;
        facts->compulsory_memory_facts_available = 1;
    }
    return yvex_rocm_complete(backend, YVEX_BACKEND_VARIANT_TENSOR_READ, where, facts, err);
}

int yvex_backend_rocm_graph_release(yvex_backend *backend, yvex_rocm_graph **graph, yvex_error *err)
{
    static const char where[] = "rocm.graph.release";
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc;
    if (!state || !graph) return refuse(err, YVEX_ERR_INVALID_ARG, where, "backend and graph are required");
    if (!*graph) {
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (state->recording)
        return refuse(err, YVEX_ERR_STATE, where, "a launch sequence is being recorded");
    /* a replay may still be running */
    rc = yvex_rocm_status(&state->driver, state->driver.hipStreamSynchronize(yvex_rocm_stream(state)), where, err);
    if (rc != YVEX_OK) return rc;
    {
        yvex_rocm_graph **link = &state->graphs;
        while (*link && *link != *graph) link = &(*link)->next;
        if (*link) *link = (*graph)->next;
    }
    if ((*graph)->executable) (void)state->driver.hipGraphExecDestroy((*graph)->executable);
    if ((*graph)->graph) (void)state->driver.hipGraphDestroy((*graph)->graph);
    free(*graph);
    *graph = NULL;
    if (state->live_graphs) state->live_graphs--;
    yvex_error_clear(err);
    return YVEX_OK;
}

extern const char yvex_rocm_bundle_architecture[];

int yvex_backend_rocm_report_get(const yvex_backend *backend, yvex_backend_rocm_report *out,
                                 yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    unsigned int f;
    if (!state || !out)
        return refuse(err, YVEX_ERR_INVALID_ARG, "rocm.report", "ROCm backend and out are required");
    memset(out, 0, sizeof(*out));
    out->driver_loaded = state->driver.library != NULL;
    out->device_ready = state->stream_handle != NULL;
    out->bundle_built = yvex_rocm_bundle_image_count() != 0u;
    out->bundle_admitted = state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_ADMITTED;
    out->image_count = yvex_rocm_bundle_image_count();
    for (f = 0u; f < YVEX_ROCM_FN_COUNT; ++f) out->function_count += state->functions[f] != NULL;
    yvex_core_text_copy(out->architecture, sizeof(out->architecture), yvex_rocm_bundle_architecture);
    yvex_core_text_copy(out->device_name, sizeof(out->device_name), backend->device_name_storage);
    yvex_core_text_copy(out->driver_library, sizeof(out->driver_library),
                        state->driver.library_name);
    yvex_core_text_copy(out->rejection, sizeof(out->rejection), state->kernel_bundle_rejection);
    yvex_error_clear(err);
    return YVEX_OK;
}
