// Device-resident scratch that exists without any allocation call.
//
// Callers that may not allocate (code under stream capture, tight serving loops, harnesses
// that forbid hipMalloc) still need somewhere to put the split-K partials of the paged
// decode.  This translation unit owns one fixed array in device memory, `scratch`: it is
// part of the code object the HIP runtime loads with the library, so every GPU the library
// runs on holds its own copy, at its own address, until the process ends.
//
// In host code the array's name is only a stand-in for the symbol: it is never passed to a
// kernel or a memory routine.  The device address is obtained once per device, with that
// device current, by hipGetSymbolAddress, kept in `scratch_pointer`, and handed out from
// there; kernels receive it as an ordinary pointer argument.
//
// The array is shared by every call on one GPU and keeps the contents of the last call.
// The paged decode writes each partial slot and the offsets table before it reads them, so
// nothing needs clearing between calls; calls that overlap on one GPU race on it.
#include <hip/hip_runtime.h>
#include <pthread.h>

#include "rocm_scratch.h"

static __device__ __align__(256) unsigned char scratch[YVEX_ROCM_STATIC_SCRATCH_BYTES];

// Keeps a device-side reference to the array so it is emitted into the code object whatever
// the host side does with the symbol; also the fill kernel a caller can use to clear it.
extern "C" __global__ void yvex_rocm_static_scratch_fill(unsigned int value, unsigned long long words)
{
    unsigned int *data = reinterpret_cast<unsigned int *>(scratch);
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < words;
         i += stride)
        data[i] = value;
}

enum { kMaxDevices = 64 };
static void *scratch_pointer[kMaxDevices];
static int scratch_resolved[kMaxDevices];
static pthread_mutex_t scratch_lock = PTHREAD_MUTEX_INITIALIZER;

extern "C" int yvex_rocm_static_scratch_resolve(int device, void **address, int *hip_error)
{
    int previous = -1;
    hipError_t code = hipSuccess;
    void *pointer = nullptr;
    if (address) *address = nullptr;
    if (hip_error) *hip_error = 0;
    if (!address || device < 0 || device >= kMaxDevices) return YVEX_ROCM_SCRATCH_BAD_DEVICE;
    pthread_mutex_lock(&scratch_lock);
    if (!scratch_resolved[device]) {
        // once per device, with that device current
        code = hipGetDevice(&previous);
        if (code == hipSuccess && previous != device) code = hipSetDevice(device);
        if (code == hipSuccess) code = hipGetSymbolAddress(&pointer, HIP_SYMBOL(scratch));
        if (code == hipSuccess && previous != device && previous >= 0) code = hipSetDevice(previous);
        if (code == hipSuccess && pointer) {
            scratch_pointer[device] = pointer;
            scratch_resolved[device] = 1;
        }
    }
    pointer = scratch_resolved[device] ? scratch_pointer[device] : nullptr;
    pthread_mutex_unlock(&scratch_lock);
    if (!pointer) {
        if (hip_error) *hip_error = (int)code;
        (void)hipGetLastError();  // the failure is reported here, not by a later call
        return YVEX_ROCM_SCRATCH_UNAVAILABLE;
    }
    *address = pointer;
    return YVEX_ROCM_SCRATCH_OK;
}
