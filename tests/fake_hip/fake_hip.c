/* A stand-in HIP runtime for host-logic tests on machines without a GPU.
 *
 * It implements exactly the entry points the backend binds (rocm_driver.h) with host
 * memory and no computation: kernel launches are counted and otherwise do nothing, so
 * nothing numerical can be tested (or accidentally served) through it.  It is loaded
 * only when a test sets YVEX_TEST_ROCM_DRIVER_LIBRARY; it exists so admission,
 * bookkeeping, failure transitions and cleanup of the C host can run on the CPU, the
 * way the reference swaps entries of its driver table in tests/unit/cuda/graph.c:265-289.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <stdlib.h>
#include <string.h>

static unsigned long long launches, allocations, frees, loads, unloads;
static int capturing;                       /* a stream capture is open */
static unsigned long long captured_launches;

unsigned long long fake_hip_launches(void) { return launches; }
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

hipError_t hipMemcpyAsync(void *dst, const void *src, size_t size, hipMemcpyKind kind,
                          hipStream_t stream)
{
    (void)kind;
    (void)stream;
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
    (void)f; (void)gx; (void)gy; (void)gz; (void)bx; (void)by; (void)bz;
    (void)shared; (void)stream; (void)params; (void)extra;
    if (env_is("FAKE_HIP_LAUNCH", "fail")) return hipErrorLaunchFailure;
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
