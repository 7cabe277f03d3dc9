/* dlopen binding of the HIP runtime (see rocm_driver.h). */
#define _GNU_SOURCE
#include "rocm_driver.h"

#include <dlfcn.h>
#include <stdlib.h>
#include <string.h>

#include "private.h"

static const char *const default_libraries[] = {
    "libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6", "/opt/rocm/lib/libamdhip64.so"};

int yvex_rocm_driver_load(yvex_rocm_driver *driver, yvex_error *err)
{
    const char *override = getenv("YVEX_TEST_ROCM_DRIVER_LIBRARY");
    size_t i;
    memset(driver, 0, sizeof(*driver));
    if (override && *override) {
        driver->library = dlopen(override, RTLD_NOW | RTLD_LOCAL);
        yvex_core_text_copy(driver->library_name, sizeof(driver->library_name), override);
    } else {
        for (i = 0; !driver->library && i < sizeof(default_libraries) / sizeof(default_libraries[0]);
             ++i) {
            driver->library = dlopen(default_libraries[i], RTLD_NOW | RTLD_LOCAL);
            if (driver->library)
                yvex_core_text_copy(driver->library_name, sizeof(driver->library_name),
                                    default_libraries[i]);
        }
    }
    if (!driver->library) {
        yvex_error_set(err, YVEX_ERR_UNSUPPORTED, "rocm.driver.load",
                       "HIP runtime library is unavailable");
        return YVEX_ERR_UNSUPPORTED;
    }
#define X(name)                                                                          \
    driver->name = (__typeof__(driver->name))dlsym(driver->library, #name);              \
    if (!driver->name) {                                                                 \
        yvex_error_setf(err, YVEX_ERR_UNSUPPORTED, "rocm.driver.load",                   \
                        "HIP runtime entry point is missing: %s", #name);                \
        yvex_rocm_driver_unload(driver);                                                 \
        return YVEX_ERR_UNSUPPORTED;                                                     \
    }
    YVEX_ROCM_DRIVER_ENTRIES(X)
#undef X
    driver->virtual_memory = 1;
#define X(name)                                                                          \
    driver->name = (__typeof__(driver->name))dlsym(driver->library, #name);              \
    if (!driver->name) driver->virtual_memory = 0;
    YVEX_ROCM_DRIVER_VIRTUAL_ENTRIES(X)
#undef X
#define X(name) driver->name = NULL;
    if (!driver->virtual_memory) { YVEX_ROCM_DRIVER_VIRTUAL_ENTRIES(X) }
#undef X
    driver->pinned_memory = 1;
#define X(name)                                                                          \
    driver->name = (__typeof__(driver->name))dlsym(driver->library, #name);              \
    if (!driver->name) driver->pinned_memory = 0;
    YVEX_ROCM_DRIVER_PINNED_ENTRIES(X)
#undef X
#define X(name) driver->name = NULL;
    if (!driver->pinned_memory) { YVEX_ROCM_DRIVER_PINNED_ENTRIES(X) }
#undef X
    driver->timed_launch =
        (yvex_rocm_timed_launch_fn)dlsym(driver->library, "hipExtModuleLaunchKernel");
    yvex_error_clear(err);
    return YVEX_OK;
}

void yvex_rocm_driver_unload(yvex_rocm_driver *driver)
{
    /* The runtime library stays mapped for the life of the process: unloading a GPU
     * runtime that still owns device state is not safe, and a later open reuses it. */
    if (driver) memset(driver, 0, sizeof(*driver));
}

int yvex_rocm_status(const yvex_rocm_driver *driver, hipError_t code, const char *where,
                     yvex_error *err)
{
    const char *text = NULL;
    if (code == hipSuccess) return YVEX_OK;
    if (driver && driver->hipGetErrorString) text = driver->hipGetErrorString(code);
    yvex_error_setf(err, YVEX_ERR_BACKEND, where, "HIP error %d: %s", (int)code,
                    text ? text : "unknown");
    return YVEX_ERR_BACKEND;
}
