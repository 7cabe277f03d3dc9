/* A stand-in HIP runtime for host-logic tests on machines without a GPU.
 *
 * It implements exactly the entry points the backend binds (rocm_driver.h) with host
 * memory and no computation: kernel launches are counted and otherwise do nothing (but for
 * the one-thread kernel that hands the status word to the host and the batch of queued
 * copies), so nothing numerical can be tested (or accidentally served) through it.  It is loaded
 * only when a test sets YVEX_TEST_ROCM_DRIVER_LIBRARY; it exists so admission,
 * bookkeeping, failure transitions and cleanup of the C host can run on the CPU, the
 * way the reference swaps entries of its driver table in tests/unit/cuda/graph.c:265-289.
 */
#define _GNU_SOURCE
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>

static unsigned long long launches, allocations, frees, loads, unloads, forwards, copy_batches, async_copies,
    small_transfers;
static int capturing;                       /* a stream capture is open */
static unsigned long long captured_launches;

static unsigned int last_grid_x;
static unsigned char last_params[512];
unsigned long long fake_hip_launches(void) { return launches; }
/* launches that carried a batch of queued copies, and copies handed to the runtime one by one */
unsigned long long fake_hip_copy_batches(void) { return copy_batches; }
unsigned long long fake_hip_device_copies(void) { return async_copies; }
/* tensor reads and writes of a few bytes carried by a kernel */
unsigned long long fake_hip_small_transfers(void) { return small_transfers; }
/* status words handed to the host through its mailbox */
unsigned long long fake_hip_status_forwards(void) { return forwards; }
unsigned int fake_hip_last_grid_x(void) { return last_grid_x; }
/* the bytes kept of the last launch's parameter struct */
const unsigned char *fake_hip_last_params(void) { return last_params; }
unsigned long long fake_hip_live_allocations(void) { return allocations - frees; }
unsigned long long fake_hip_live_modules(void) { return loads - unloads; }

static int env_is(const char *name, const char *value)
{
    const char *v = getenv(name);
    return v && strcmp(v, value) == 0;
}

hipError_t hipInit(unsigned int flags)
{
    (void)flags;
    return env_is("FAKE_HIP_INIT", "fail") ? hipErrorNoDevice : hipSuccess;
}

hipError_t hipGetDeviceCount(int *count)
{
    const char *v = getenv("FAKE_HIP_DEVICES");
    *count = v ? atoi(v) : 1;
    return hipSuccess;
}

hipError_t hipSetDevice(int device) { (void)device; return hipSuccess; }

hipError_t hipDeviceGetName(char *name, int len, hipDevice_t device)
{
    (void)device;
    strncpy(name, "fake-gfx950", (size_t)len - 1u);
    name[len - 1] = '\0';
    return hipSuccess;
}

hipError_t hipDeviceGetAttribute(int *value, hipDeviceAttribute_t attribute, int device)
{
    (void)device;
    if (attribute == hipDeviceAttributeVirtualMemoryManagementSupported)
        *value = env_is("FAKE_HIP_VIRTUAL_MEMORY", "absent") ? 0 : 1;
    else
        *value = attribute == hipDeviceAttributeMultiprocessorCount ? 256 : 9;
    return hipSuccess;
}

hipError_t hipDeviceTotalMem(size_t *bytes, hipDevice_t device)
{
    (void)device;
    *bytes = (size_t)288 << 30;
    return hipSuccess;
}

hipError_t hipMemGetInfo(size_t *free_bytes, size_t *total)
{
    *free_bytes = (size_t)200 << 30;
    *total = (size_t)288 << 30;
    return hipSuccess;
}

const char *hipGetErrorString(hipError_t error) { (void)error; return "fake hip error"; }

hipError_t hipStreamCreate(hipStream_t *stream)
{
    *stream = (hipStream_t)malloc(8);
    return *stream ? hipSuccess : hipErrorOutOfMemory;
}

hipError_t hipStreamDestroy(hipStream_t stream) { free(stream); return hipSuccess; }

hipError_t hipStreamSynchronize(hipStream_t stream)
{
    (void)stream;
    return env_is("FAKE_HIP_SYNC", "fail") ? hipErrorUnknown : hipSuccess;
}

hipError_t hipMalloc(void **ptr, size_t size)
{
    if (env_is("FAKE_HIP_MALLOC", "fail")) return hipErrorOutOfMemory;
    *ptr = calloc(1, size ? size : 1u);
    if (!*ptr) return hipErrorOutOfMemory;
    ++allocations;
    return hipSuccess;
}

hipError_t hipFree(void *ptr)
{
    if (ptr) ++frees;
    free(ptr);
    return hipSuccess;
}

/* host memory the device can write: the stand-in's device is the host */
hipError_t hipHostMalloc(void **ptr, size_t size, unsigned int flags)
{
    (void)flags;
    if (env_is("FAKE_HIP_HOST_MALLOC", "fail")) return hipErrorOutOfMemory;
    return hipMalloc(ptr, size);
}

hipError_t hipHostFree(void *ptr) { return hipFree(ptr); }

hipError_t hipHostGetDevicePointer(void **device, void *host, unsigned int flags)
{
    (void)flags;
    *device = host;
    return hipSuccess;
}

hipError_t hipMemcpyAsync(void *dst, const void *src, size_t size, hipMemcpyKind kind,
                          hipStream_t stream)
{
    (void)stream;
    if (kind == hipMemcpyDeviceToDevice) ++async_copies;
    memcpy(dst, src, size);
    return hipSuccess;
}

hipError_t hipMemsetAsync(void *dst, int value, size_t size, hipStream_t stream)
{
    (void)stream;
    memset(dst, value, size);
    return hipSuccess;
}

hipError_t hipModuleLoadData(hipModule_t *module, const void *image)
{
    static const unsigned char elf[4] = {0x7f, 'E', 'L', 'F'};
    if (!image || memcmp(image, elf, 4u) != 0) return hipErrorInvalidImage;
    *module = (hipModule_t)malloc(8);
    ++loads;
    return hipSuccess;
}

hipError_t hipModuleUnload(hipModule_t module)
{
    free(module);
    ++unloads;
    return hipSuccess;
}

hipError_t hipModuleGetFunction(hipFunction_t *function, hipModule_t module, const char *name)
{
    const char *missing = getenv("FAKE_HIP_MISSING_FUNCTION");
    (void)module;
    if (missing && strcmp(missing, name) == 0) return hipErrorNotFound;
    /* every symbol "exists" in the first module asked; the handle is never called */
    *function = (hipFunction_t)(void *)name;
    return hipSuccess;
}

hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned int gx, unsigned int gy, unsigned int gz,
                                 unsigned int bx, unsigned int by, unsigned int bz,
                                 unsigned int shared, hipStream_t stream, void **params,
                                 void **extra)
{
    (void)gz; (void)bx; (void)by; (void)bz;
    (void)shared; (void)stream; (void)extra;
    if (f && strcmp((const char *)f, "yvex_rocm_small_write") == 0 && params && params[0]) {
        /* small transfers by kernel are carried out as well */
        struct { void *dst; uint32_t bytes, reserved; unsigned char data[2048]; } *p = params[0];
        memcpy(p->dst, p->data, p->bytes);
        ++small_transfers;
        return hipSuccess;
    }
    if (f && strcmp((const char *)f, "yvex_rocm_small_read") == 0 && params && params[0]) {
        struct { const void *src; void *staging; uint64_t *mailbox; uint32_t bytes, sequence; } *p = params[0];
        memcpy(p->staging, p->src, p->bytes);
        /* a device that does not answer: the host's watch runs out and it asks the runtime */
        if (!env_is("FAKE_HIP_SYNC", "fail")) *p->mailbox = (uint64_t)p->sequence << 32;
        ++small_transfers;
        return hipSuccess;
    }
    if (f && strcmp((const char *)f, "yvex_rocm_copy_batch") == 0 && params && params[0]) {
        /* the batch of small copies is carried out too: gy copies, as the host queued them */
        struct { uint64_t dst[128], src[128]; uint32_t bytes[128]; } *p = params[0];
        unsigned int i;
        if (env_is("FAKE_HIP_COPY_BATCH", "fail")) return hipErrorLaunchFailure;
        for (i = 0u; i < gy && i < 128u; ++i)
            memcpy((void *)(uintptr_t)p->dst[i], (const void *)(uintptr_t)p->src[i], p->bytes[i]);
        ++copy_batches;
        return hipSuccess;
    }
    if (env_is("FAKE_HIP_LAUNCH", "fail")) return hipErrorLaunchFailure;
    if (f && strcmp((const char *)f, "yvex_rocm_status_forward") == 0 && params && params[0]) {
        /* the one kernel the stand-in carries out: (sequence, status) into the host's mailbox,
         * the status word cleared.  Not counted as a launch of the operation. */
        struct { int32_t *status; uint64_t *mailbox; uint32_t sequence; } *p = params[0];
        const int32_t status = *p->status;
        *p->status = 0;
        if (!env_is("FAKE_HIP_SYNC", "fail")) *p->mailbox = ((uint64_t)p->sequence << 32) | (uint32_t)status;
        ++forwards;
        return hipSuccess;
    }
    /* the last launch's grid width and the head of its one by-value parameter, for tests that
     * look at what the host handed to a kernel */
    last_grid_x = gx;
    {
        /* FAKE_HIP_PARAM_BYTES: how many bytes of the parameter struct the test wants kept (it
         * knows the struct it expects; nothing is read unless it asks) */
        const char *want = getenv("FAKE_HIP_PARAM_BYTES");
        size_t bytes = want ? (size_t)strtoul(want, NULL, 10) : 0u;
        if (bytes > sizeof(last_params)) bytes = sizeof(last_params);
        if (bytes && params && params[0]) memcpy(last_params, params[0], bytes);
    }
    if (capturing) ++captured_launches;
    else ++launches;
    return hipSuccess;
}

hipError_t hipEventCreate(hipEvent_t *event)
{
    *event = (hipEvent_t)malloc(8);
    return *event ? hipSuccess : hipErrorOutOfMemory;
}

hipError_t hipEventDestroy(hipEvent_t event) { free(event); return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) { (void)event; (void)stream; return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t event) { (void)event; return hipSuccess; }
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned int flags)
{
    (void)stream; (void)event; (void)flags; /* every stream of the stand-in runs its work at once */
    return hipSuccess;
}

hipError_t hipEventElapsedTime(float *ms, hipEvent_t start, hipEvent_t stop)
{
    (void)start;
    (void)stop;
    *ms = 1.0f;
    return hipSuccess;
}

/* Stream capture: while a capture is open launches are counted into the graph instead of
 * the launch counter; a replay adds them. */
struct fake_graph { unsigned long long launches; };

hipError_t hipStreamBeginCapture(hipStream_t stream, hipStreamCaptureMode mode)
{
    (void)stream; (void)mode;
    if (capturing) return hipErrorIllegalState;
    capturing = 1;
    captured_launches = 0;
    return hipSuccess;
}

hipError_t hipStreamEndCapture(hipStream_t stream, hipGraph_t *graph)
{
    struct fake_graph *g;
    (void)stream;
    if (!capturing) return hipErrorIllegalState;
    capturing = 0;
    g = (struct fake_graph *)calloc(1, sizeof(*g));
    g->launches = captured_launches;
    *graph = (hipGraph_t)g;
    return hipSuccess;
}

hipError_t hipGraphInstantiate(hipGraphExec_t *exec, hipGraph_t graph, hipGraphNode_t *error_node,
                               char *log, size_t log_size)
{
    struct fake_graph *g = (struct fake_graph *)calloc(1, sizeof(*g));
    (void)error_node; (void)log; (void)log_size;
    g->launches = ((struct fake_graph *)graph)->launches;
    *exec = (hipGraphExec_t)g;
    return hipSuccess;
}

hipError_t hipGraphLaunch(hipGraphExec_t exec, hipStream_t stream)
{
    (void)stream;
    launches += ((struct fake_graph *)exec)->launches;
    return hipSuccess;
}

hipError_t hipGraphExecDestroy(hipGraphExec_t exec) { free(exec); return hipSuccess; }
hipError_t hipGraphDestroy(hipGraph_t graph) { free(graph); return hipSuccess; }

/* Virtual memory management on host pages: a reservation is an inaccessible mapping, mapping
 * a physical handle makes its pages readable and writable, unmapping takes that away and
 * drops their contents.  Touching a reserved but unmapped address is a segmentation fault,
 * as it is a fault on the device. */
#define FAKE_GRANULARITY ((size_t)1u << 16)
struct fake_physical { size_t size; };
static unsigned long long physical_created, physical_released, ranges_reserved, ranges_freed;
static unsigned long long mapped_bytes;

unsigned long long fake_hip_live_physical(void) { return physical_created - physical_released; }
unsigned long long fake_hip_live_ranges(void) { return ranges_reserved - ranges_freed; }
unsigned long long fake_hip_mapped_bytes(void) { return mapped_bytes; }

hipError_t hipMemGetAllocationGranularity(size_t *granularity, const hipMemAllocationProp *prop,
                                          hipMemAllocationGranularity_flags option)
{
    (void)prop; (void)option;
    *granularity = FAKE_GRANULARITY;
    return hipSuccess;
}

hipError_t hipMemAddressReserve(void **ptr, size_t size, size_t alignment, void *addr,
                                unsigned long long flags)
{
    void *base;
    (void)alignment; (void)addr; (void)flags;
    if (env_is("FAKE_HIP_RESERVE", "fail") || size % FAKE_GRANULARITY) return hipErrorOutOfMemory;
    base = mmap(NULL, size, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (base == MAP_FAILED) return hipErrorOutOfMemory;
    *ptr = base;
    ++ranges_reserved;
    return hipSuccess;
}

hipError_t hipMemAddressFree(void *ptr, size_t size)
{
    if (env_is("FAKE_HIP_ADDRESS_FREE", "fail")) return hipErrorUnknown;
    if (munmap(ptr, size) != 0) return hipErrorInvalidValue;
    ++ranges_freed;
    return hipSuccess;
}

hipError_t hipMemCreate(hipMemGenericAllocationHandle_t *handle, size_t size,
                        const hipMemAllocationProp *prop, unsigned long long flags)
{
    const char *limit = getenv("FAKE_HIP_PHYSICAL_LIMIT"); /* handles that may be live at once */
    struct fake_physical *physical;
    (void)prop; (void)flags;
    if (size == 0u || size % FAKE_GRANULARITY) return hipErrorInvalidValue;
    if (limit && fake_hip_live_physical() >= strtoull(limit, NULL, 10)) return hipErrorOutOfMemory;
    physical = (struct fake_physical *)calloc(1, sizeof(*physical));
    if (!physical) return hipErrorOutOfMemory;
    physical->size = size;
    *handle = (hipMemGenericAllocationHandle_t)physical;
    ++physical_created;
    return hipSuccess;
}

hipError_t hipMemRelease(hipMemGenericAllocationHandle_t handle)
{
    if (env_is("FAKE_HIP_RELEASE", "fail")) return hipErrorUnknown;
    free((struct fake_physical *)handle);
    ++physical_released;
    return hipSuccess;
}

hipError_t hipMemMap(void *ptr, size_t size, size_t offset, hipMemGenericAllocationHandle_t handle,
                     unsigned long long flags)
{
    (void)flags;
    if (env_is("FAKE_HIP_MAP", "fail")) return hipErrorOutOfMemory;
    if (offset != 0u || size != ((struct fake_physical *)handle)->size) return hipErrorInvalidValue;
    if (mprotect(ptr, size, PROT_READ | PROT_WRITE) != 0) return hipErrorInvalidValue;
    memset(ptr, 0xa5, size); /* fresh device memory is not zero */
    mapped_bytes += size;
    return hipSuccess;
}

hipError_t hipMemUnmap(void *ptr, size_t size)
{
    if (env_is("FAKE_HIP_UNMAP", "fail")) return hipErrorUnknown;
    if (madvise(ptr, size, MADV_DONTNEED) != 0 || mprotect(ptr, size, PROT_NONE) != 0)
        return hipErrorInvalidValue;
    mapped_bytes -= size;
    return hipSuccess;
}

hipError_t hipMemSetAccess(void *ptr, size_t size, const hipMemAccessDesc *desc, size_t count)
{
    (void)ptr; (void)size;
    if (env_is("FAKE_HIP_ACCESS", "fail")) return hipErrorInvalidValue;
    return desc && count == 1u && desc->flags == hipMemAccessFlagsProtReadWrite ? hipSuccess
                                                                               : hipErrorInvalidValue;
}
