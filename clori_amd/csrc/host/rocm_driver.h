/* The thin C-ABI layer between the C11 host and HIP: a table of runtime entry points
 * resolved with dlopen/dlsym, the way the reference binds the CUDA driver
 * (src/backend/cuda/private.h:102-206, src/backend/cuda/info.c:47-49).  Because the
 * runtime is a struct of function pointers a test can substitute another library
 * (YVEX_TEST_ROCM_DRIVER_LIBRARY) and exercise admission, bookkeeping and failure
 * transitions of the host code on a machine with no GPU. */
#ifndef YVEX_ROCM_DRIVER_H
#define YVEX_ROCM_DRIVER_H

#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>

#include "yvex_rocm.h"

#define YVEX_ROCM_DRIVER_ENTRIES(X)                                                      \
    X(hipInit) X(hipGetDeviceCount) X(hipSetDevice) X(hipDeviceGetName)                  \
    X(hipDeviceGetAttribute) X(hipDeviceTotalMem) X(hipMemGetInfo) X(hipGetErrorString)  \
    X(hipStreamCreate) X(hipStreamDestroy) X(hipStreamSynchronize) X(hipMalloc) X(hipFree) \
    X(hipMemcpyAsync) X(hipMemsetAsync) X(hipModuleLoadData) X(hipModuleUnload)          \
    X(hipModuleGetFunction) X(hipModuleLaunchKernel) X(hipEventCreate) X(hipEventDestroy) \
    X(hipEventRecord) X(hipEventSynchronize) X(hipEventElapsedTime) X(hipStreamWaitEvent) \
    X(hipStreamBeginCapture) X(hipStreamEndCapture) X(hipGraphInstantiate) X(hipGraphLaunch) \
    X(hipGraphExecDestroy) X(hipGraphDestroy)

/* Virtual memory management: an address range reserved once and backed by physical memory
 * piece by piece.  Bound all or none; a runtime without them still opens and only the
 * virtual-range tensor calls refuse. */
#define YVEX_ROCM_DRIVER_VIRTUAL_ENTRIES(X)                                              \
    X(hipMemGetAllocationGranularity) X(hipMemAddressReserve) X(hipMemAddressFree)       \
    X(hipMemCreate) X(hipMemRelease) X(hipMemMap) X(hipMemUnmap) X(hipMemSetAccess)

/* Host memory the device can write: the mailbox through which an operation's status word
 * reaches the host without a copy.  Bound all or none; without them the status is copied. */
#define YVEX_ROCM_DRIVER_PINNED_ENTRIES(X) X(hipHostMalloc) X(hipHostFree) X(hipHostGetDevicePointer)

/* hipExtModuleLaunchKernel (hip/hip_ext.h, a C++ header): a launch whose two events take the
 * kernel's own begin and end timestamps.  Work sizes are in threads, not workgroups. */
typedef hipError_t (*yvex_rocm_timed_launch_fn)(hipFunction_t, uint32_t, uint32_t, uint32_t, uint32_t,
                                                uint32_t, uint32_t, size_t, hipStream_t, void **,
                                                void **, hipEvent_t, hipEvent_t, uint32_t);

typedef struct yvex_rocm_driver {
    void *library;
    char library_name[256];
#define X(name) __typeof__(&name) name;
    YVEX_ROCM_DRIVER_ENTRIES(X)
    YVEX_ROCM_DRIVER_VIRTUAL_ENTRIES(X) /* optional: all NULL when any is missing */
    YVEX_ROCM_DRIVER_PINNED_ENTRIES(X)  /* optional, likewise */
#undef X
    int virtual_memory;                 /* the virtual memory entries are bound */
    int pinned_memory;                  /* the pinned host memory entries are bound */
    yvex_rocm_timed_launch_fn timed_launch; /* optional: NULL when the runtime lacks it */
} yvex_rocm_driver;

/* Loads the runtime library and resolves every entry or none (YVEX_ERR_UNSUPPORTED). */
int yvex_rocm_driver_load(yvex_rocm_driver *driver, yvex_error *err);
void yvex_rocm_driver_unload(yvex_rocm_driver *driver);
/* Maps a hipError_t to YVEX_OK / YVEX_ERR_BACKEND with the runtime's message. */
int yvex_rocm_status(const yvex_rocm_driver *driver, hipError_t code, const char *where,
                     yvex_error *err);

#endif /* YVEX_ROCM_DRIVER_H */
