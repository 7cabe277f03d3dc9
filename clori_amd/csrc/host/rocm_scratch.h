/* Fixed device scratch for the entry point that allocates nothing (rocm_scratch.hip). */
#ifndef YVEX_ROCM_SCRATCH_H
#define YVEX_ROCM_SCRATCH_H

/* Size of the array each GPU holds for the life of the process: room for the split-K
 * partials of a paged decode with up to 2048 waves and a query group of 7 (the admitted
 * configurations use a group of 4: 8.5 MB). */
#define YVEX_ROCM_STATIC_SCRATCH_BYTES (16ull << 20)

enum {
    YVEX_ROCM_SCRATCH_OK = 0,
    YVEX_ROCM_SCRATCH_BAD_DEVICE = 1,
    YVEX_ROCM_SCRATCH_UNAVAILABLE = 2
};

#define YVEX_ROCM_SCRATCH_LIBRARY "libyvex_rocm_scratch.so"
#define YVEX_ROCM_SCRATCH_RESOLVE_SYMBOL "yvex_rocm_static_scratch_resolve"

#ifdef __cplusplus
extern "C" {
#endif
/* Exported by the companion object (rocm_scratch.hip), the only object of this library that is
 * linked against the HIP runtime: device address of the scratch array on `device` (resolved on
 * the first call for that device, cached afterwards).  hip_error receives the runtime's code
 * when unavailable. */
typedef int (*yvex_rocm_static_scratch_resolve_fn)(int device, void **address, int *hip_error);
int yvex_rocm_static_scratch_resolve(int device, void **address, int *hip_error);
#ifdef __cplusplus
}
#endif

#endif /* YVEX_ROCM_SCRATCH_H */
