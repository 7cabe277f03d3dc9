/* Kernel-bundle admission, capability projection and fail-closed launch/synchronise
 * for the ROCm arm.  The rules are those of src/backend/cuda/capability.c in the
 * reference: nothing is published before every image loaded and every required symbol
 * resolved (all or nothing); an absent bundle leaves the backend CONTEXT_READY with
 * tensor traffic only; a launch failure fails that variant; a synchronise or cleanup
 * failure fails the whole backend.  Test-only fault injection uses
 * YVEX_TEST_ROCM_BUNDLE_FAILURE (module | symbol | <function name>),
 * YVEX_TEST_ROCM_LAUNCH_FAILURE, YVEX_TEST_ROCM_SYNC_FAILURE (all | <variant name>) and
 * YVEX_TEST_ROCM_CLEANUP_FAILURE, mirroring the YVEX_TEST_CUDA_* switches. */
#ifndef _POSIX_C_SOURCE
#define _POSIX_C_SOURCE 200809L /* clock_gettime */
#endif
#include "rocm_state.h"
#include "../kernel_params.h"

#include <stdlib.h>
#include <string.h>
#include <time.h>

typedef struct {
    const char *name;
    const unsigned char *begin, *end;
} yvex_rocm_bundle_image;

/* Generated next to the code objects by the build (bundle_table.c). */
extern const yvex_rocm_bundle_image yvex_rocm_bundle_images[];
extern const unsigned int yvex_rocm_bundle_image_total;
extern const char yvex_rocm_bundle_architecture[];

typedef struct {
    const char *symbol;
    yvex_backend_operation_variant variant;
    yvex_rocm_function_id slot;
} rocm_kernel_binding;

static const rocm_kernel_binding rocm_kernel_bindings[] = {
    {"yvex_rocm_attention_f32", YVEX_BACKEND_VARIANT_ATTENTION_CAUSAL_F32,
     YVEX_ROCM_FN_ATTENTION_F32},
    {"yvex_rocm_gqa_f32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_GQA_F32},
    {"yvex_rocm_gqa_f32_split", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_GQA_F32_SPLIT},
    {"yvex_rocm_gqa_f32_split_wide", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_GQA_F32_SPLIT_WIDE},
    {"yvex_rocm_gqa_f32_tile_64", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_GQA_F32_TILE_64},
    {"yvex_rocm_gqa_f32_tile_128", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_GQA_F32_TILE_128},
    {"yvex_rocm_gqa_f32_tile_256", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_GQA_F32_TILE_256},
    {"yvex_rocm_fill_u32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_FILL_U32},
    {"yvex_rocm_stream_read", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_STREAM_READ},
    {"yvex_rocm_rotary_half_plain_f32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_ROTARY_HALF_PLAIN_F32},
    {"yvex_rocm_bf16_round_f32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_BF16_ROUND_F32},
    {"yvex_rocm_sigmoid_product_bf16_f32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_SIGMOID_PRODUCT_BF16_F32},
    {"yvex_rocm_split_interleaved_two_f32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_SPLIT_INTERLEAVED_TWO_F32},
    {"yvex_rocm_decode_paged_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_PAGED_BF16},
    {"yvex_rocm_decode_paged_bf16_64", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_PAGED_BF16_64},
    {"yvex_rocm_decode_paged_bf16_256", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_PAGED_BF16_256},
    {"yvex_rocm_decode_finish_256", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_FINISH_256},
    {"yvex_rocm_decode_merge", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_MERGE},
    {"yvex_rocm_decode_merge_rope", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16,
     YVEX_ROCM_FN_DECODE_MERGE_ROPE},
    {"yvex_rocm_decode_finish", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_FINISH},
    {"yvex_rocm_decode_rows_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_DECODE_ROWS_BF16},
    {"yvex_rocm_prefill_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_PREFILL_BF16},
    {"yvex_rocm_prefill_bf16_64", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_PREFILL_BF16_64},
    {"yvex_rocm_prefill_bf16_256", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_PREFILL_BF16_256},
    {"yvex_rocm_mla_decode_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16,
     YVEX_ROCM_FN_MLA_DECODE_BF16},
    {"yvex_rocm_mla_decode_512_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16,
     YVEX_ROCM_FN_MLA_DECODE_512_BF16},
    {"yvex_rocm_decode_paged_q8_0", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0,
     YVEX_ROCM_FN_DECODE_PAGED_Q8_0},
    {"yvex_rocm_decode_paged_bf16_merged", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_DECODE_PAGED_BF16_MERGED},
    {"yvex_rocm_decode_paged_q8_0_merged", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0,
     YVEX_ROCM_FN_DECODE_PAGED_Q8_0_MERGED},
    {"yvex_rocm_decode_rows_bf16_merged", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_DECODE_ROWS_BF16_MERGED},
    {"yvex_rocm_decode_rows_bf16_team", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM},
    {"yvex_rocm_decode_rows_bf16_team_64", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM_64},
    {"yvex_rocm_decode_rows_bf16_team_256", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_DECODE_ROWS_BF16_TEAM_256},
    {"yvex_rocm_status_forward", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_STATUS_FORWARD},
    {"yvex_rocm_copy_batch", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_COPY_BATCH},
    {"yvex_rocm_small_write", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_SMALL_WRITE},
    {"yvex_rocm_small_read", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32, YVEX_ROCM_FN_SMALL_READ},
    {"yvex_rocm_gather_rows", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16, YVEX_ROCM_FN_GATHER_ROWS},
    {"yvex_rocm_kv_append_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_KV_APPEND_BF16},
    {"yvex_rocm_kv_append_bf16_64", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_KV_APPEND_BF16_64},
    {"yvex_rocm_kv_append_bf16_256", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16,
     YVEX_ROCM_FN_KV_APPEND_BF16_256},
    {"yvex_rocm_kv_append_q8_0", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0,
     YVEX_ROCM_FN_KV_APPEND_Q8_0},
    {"yvex_rocm_history_append_bf16", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
     YVEX_ROCM_FN_HISTORY_APPEND_BF16},
    {"yvex_rocm_history_append_f32", YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,
     YVEX_ROCM_FN_HISTORY_APPEND_F32},
};
#define ROCM_KERNEL_BINDING_COUNT (sizeof(rocm_kernel_bindings) / sizeof(rocm_kernel_bindings[0]))

unsigned int yvex_rocm_bundle_image_count(void) { return yvex_rocm_bundle_image_total; }

/* Failure injection for the host tests, named and read the way the reference's CUDA arm does
 * it (getenv("YVEX_TEST_CUDA_ATTENTION_FAILURE"), src/backend/cuda/ops.c:88-200;
 * YVEX_TEST_CUDA_*_FAILURE, src/backend/cuda/residency.c:57-240): only variables with the
 * YVEX_TEST_ROCM_ prefix are ever read, and none of them changes launch geometry. */
static int test_failure_matches(const char *name, yvex_backend_operation_variant variant)
{
    const char *value = getenv(name);
    return value && value[0] != '\0' &&
           (strcmp(value, "all") == 0 ||
            strcmp(value, yvex_backend_operation_variant_name(variant)) == 0);
}

static void capability_fail(yvex_backend *backend, yvex_backend_operation_variant variant,
                            yvex_backend_capability_reason reason)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    if (!state || (int)variant < 0 || variant >= YVEX_BACKEND_VARIANT_ROCM_END) return;
    state->variant_failures[variant] = reason;
    if (reason == YVEX_BACKEND_CAPABILITY_REASON_SYNCHRONIZATION_FAILED ||
        reason == YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED) {
        state->backend_failure_reason = reason;
        backend->status = YVEX_BACKEND_STATUS_FAILED;
    }
}

static void bundle_reject(yvex_rocm_backend_state *state, yvex_backend_capability_reason reason,
                          yvex_backend_operation_variant variant, const yvex_error *err)
{
    state->kernel_bundle_state = YVEX_ROCM_KERNEL_BUNDLE_REJECTED;
    state->kernel_bundle_reason = reason;
    state->kernel_bundle_failure_variant = variant;
    yvex_core_text_copy(state->kernel_bundle_rejection, sizeof(state->kernel_bundle_rejection),
                        err ? err->message : "");
}

/* src/backend/cuda/capability.c:511-620: handles are committed only after every image
 * loaded and every symbol resolved; otherwise everything loaded so far is unloaded. */
int yvex_rocm_kernel_bundle_admit(yvex_backend *backend, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    hipModule_t modules[YVEX_ROCM_MODULE_MAX] = {0};
    hipFunction_t functions[YVEX_ROCM_FN_COUNT] = {0};
    const char *injected = getenv("YVEX_TEST_ROCM_BUNDLE_FAILURE");
    unsigned int loaded = 0u, index;
    size_t b;
    int rc = YVEX_OK;
    if (!backend || !state || !state->stream_handle) {
        yvex_error_set(err, YVEX_ERR_STATE, "rocm.kernels.admit",
                       "ROCm context is required for kernel admission");
        return YVEX_ERR_STATE;
    }
    rc = backend_dispatch_admit(backend, "rocm.kernels.admit", err);
    if (rc != YVEX_OK) return rc;
    if (state->module_count) {
        if (state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_ADMITTED) {
            yvex_error_clear(err);
            return YVEX_OK;
        }
        yvex_error_set(err, YVEX_ERR_STATE, "rocm.kernels.admit",
                       "retained ROCm module ownership requires checked cleanup");
        return YVEX_ERR_STATE;
    }
    memset(state->functions, 0, sizeof(state->functions));
    state->kernel_bundle_state = YVEX_ROCM_KERNEL_BUNDLE_ABSENT;
    state->kernel_bundle_reason = YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT;
    state->kernel_bundle_failure_variant = YVEX_BACKEND_VARIANT_COUNT;
    state->kernel_bundle_rejection[0] = '\0';
    if (!yvex_rocm_bundle_image_total) {
        yvex_error_set(err, YVEX_ERR_UNSUPPORTED, "rocm.kernels.admit",
                       "gfx950 kernel bundle was not built");
        return YVEX_ERR_UNSUPPORTED;
    }
    if (yvex_rocm_bundle_image_total > YVEX_ROCM_MODULE_MAX) {
        yvex_error_set(err, YVEX_ERR_BOUNDS, "rocm.kernels.admit",
                       "kernel bundle holds more images than the module table");
        bundle_reject(state, YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_REJECTED,
                      YVEX_BACKEND_VARIANT_COUNT, err);
        return YVEX_ERR_BOUNDS;
    }
    for (loaded = 0u; loaded < yvex_rocm_bundle_image_total; ++loaded) {
        const yvex_rocm_bundle_image *image = &yvex_rocm_bundle_images[loaded];
        if (injected && strcmp(injected, "module") == 0) {
            yvex_error_set(err, YVEX_ERR_BACKEND, "rocm.kernels.load",
                           "injected ROCm module admission failure");
            rc = YVEX_ERR_BACKEND;
        } else if (image->end <= image->begin) {
            yvex_error_setf(err, YVEX_ERR_FORMAT, "rocm.kernels.load", "empty code object: %s",
                            image->name);
            rc = YVEX_ERR_FORMAT;
        } else {
            rc = yvex_rocm_status(&state->driver,
                                  state->driver.hipModuleLoadData(&modules[loaded], image->begin),
                                  "rocm.kernels.load", err);
        }
        if (rc != YVEX_OK) {
            bundle_reject(state, YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_REJECTED,
                          YVEX_BACKEND_VARIANT_COUNT, err);
            goto reject;
        }
    }
    for (b = 0; b < ROCM_KERNEL_BINDING_COUNT; ++b) {
        const rocm_kernel_binding *binding = &rocm_kernel_bindings[b];
        hipFunction_t function = NULL;
        if (!(injected && (strcmp(injected, "symbol") == 0 ||
                           strcmp(injected, binding->symbol) == 0))) {
            for (index = 0u; index < loaded && !function; ++index)
                if (state->driver.hipModuleGetFunction(&function, modules[index],
                                                       binding->symbol) != hipSuccess)
                    function = NULL;
        }
        if (!function) {
            yvex_error_setf(err, YVEX_ERR_BACKEND, "rocm.kernels.resolve",
                            "required ROCm function unavailable: %s", binding->symbol);
            rc = YVEX_ERR_BACKEND;
            bundle_reject(state, YVEX_BACKEND_CAPABILITY_REASON_FUNCTION_MISSING,
                          binding->variant, err);
            goto reject;
        }
        functions[binding->slot] = function;
    }
    memcpy(state->modules, modules, loaded * sizeof(modules[0]));
    state->module_count = loaded;
    memcpy(state->functions, functions, sizeof(functions));
    state->kernel_bundle_state = YVEX_ROCM_KERNEL_BUNDLE_ADMITTED;
    state->kernel_bundle_reason = YVEX_BACKEND_CAPABILITY_REASON_NONE;
    yvex_error_clear(err);
    return YVEX_OK;
reject:
    for (index = 0u; index < loaded; ++index)
        if (modules[index]) (void)state->driver.hipModuleUnload(modules[index]);
    return rc;
}

/* src/backend/cuda/capability.c:622-657 */
int yvex_rocm_kernel_bundle_close(yvex_backend *backend, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    unsigned int index;
    int rc = YVEX_OK;
    if (!state) {
        yvex_error_clear(err);
        return YVEX_OK;
    }
    for (index = 0u; index < state->module_count; ++index) {
        int unload_rc;
        if (!state->modules[index]) continue;
        if (getenv("YVEX_TEST_ROCM_CLEANUP_FAILURE")) {
            yvex_error_set(err, YVEX_ERR_BACKEND, "rocm.kernels.unload",
                           "injected ROCm module cleanup failure");
            unload_rc = YVEX_ERR_BACKEND;
        } else {
            unload_rc = yvex_rocm_status(&state->driver,
                                         state->driver.hipModuleUnload(state->modules[index]),
                                         "rocm.kernels.unload", err);
        }
        if (unload_rc == YVEX_OK)
            state->modules[index] = NULL;
        else
            rc = unload_rc;
    }
    if (rc != YVEX_OK) {
        state->kernel_bundle_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
        state->backend_failure_reason = YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED;
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return rc;
    }
    state->module_count = 0u;
    memset(state->functions, 0, sizeof(state->functions));
    state->kernel_bundle_state = YVEX_ROCM_KERNEL_BUNDLE_ABSENT;
    state->kernel_bundle_reason = YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT;
    yvex_error_clear(err);
    return YVEX_OK;
}

static int variant_functions_present(const yvex_rocm_backend_state *state,
                                     yvex_backend_operation_variant variant, int *bound)
{
    size_t b;
    *bound = 0;
    if (variant == YVEX_BACKEND_VARIANT_ATTENTION_NONCAUSAL_F32)
        variant = YVEX_BACKEND_VARIANT_ATTENTION_CAUSAL_F32;
    for (b = 0; b < ROCM_KERNEL_BINDING_COUNT; ++b) {
        if (rocm_kernel_bindings[b].variant != variant) continue;
        *bound = 1;
        if (!state->functions[rocm_kernel_bindings[b].slot]) return 0;
    }
    return *bound;
}

static int publish(yvex_backend_capability_result *out, yvex_backend_capability_state state,
                   yvex_backend_capability_reason reason, int function_available,
                   yvex_error *err)
{
    out->state = state;
    out->reason = reason;
    out->function_available = function_available;
    yvex_error_clear(err);
    return YVEX_OK;
}

/* src/backend/cuda/capability.c:659-722 */
int yvex_rocm_query_capability(const yvex_backend *backend, yvex_backend_operation_variant variant,
                               yvex_backend_capability_result *out, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int bound, present;
    if (!backend || !state || !out) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "rocm.query_capability",
                       "backend, ROCm state, and out are required");
        return YVEX_ERR_INVALID_ARG;
    }
    out->context_available = state->stream_handle != NULL;
    out->kernel_bundle_available = state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_ADMITTED;
    if (!state->stream_handle)
        return publish(out, YVEX_BACKEND_CAPABILITY_UNSUPPORTED,
                       YVEX_BACKEND_CAPABILITY_REASON_CONTEXT_UNAVAILABLE, 0, err);
    if (backend->status == YVEX_BACKEND_STATUS_FAILED &&
        state->backend_failure_reason != YVEX_BACKEND_CAPABILITY_REASON_NONE)
        return publish(out, YVEX_BACKEND_CAPABILITY_FAILED, state->backend_failure_reason, 0, err);
    if (state->variant_failures[variant] != YVEX_BACKEND_CAPABILITY_REASON_NONE)
        return publish(out, YVEX_BACKEND_CAPABILITY_FAILED, state->variant_failures[variant], 0,
                       err);
    if (variant >= YVEX_BACKEND_VARIANT_TENSOR_ALLOC && variant <= YVEX_BACKEND_VARIANT_TENSOR_COPY)
        return publish(out, YVEX_BACKEND_CAPABILITY_SUPPORTED, YVEX_BACKEND_CAPABILITY_REASON_NONE,
                       1, err);
    if (state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_ABSENT)
        return publish(out, YVEX_BACKEND_CAPABILITY_UNSUPPORTED,
                       YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT, 0, err);
    if (state->kernel_bundle_state == YVEX_ROCM_KERNEL_BUNDLE_REJECTED) {
        yvex_backend_capability_reason reason = state->kernel_bundle_reason;
        if (reason == YVEX_BACKEND_CAPABILITY_REASON_FUNCTION_MISSING &&
            state->kernel_bundle_failure_variant != variant)
            reason = YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_REJECTED;
        return publish(out, YVEX_BACKEND_CAPABILITY_FAILED, reason, 0, err);
    }
    present = variant_functions_present(state, variant, &bound);
    if (!bound)
        /* a variant this backend has no kernel for (embed, matmul, MoE, ...) */
        return publish(out, YVEX_BACKEND_CAPABILITY_UNSUPPORTED,
                       YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED, 0, err);
    return publish(out,
                   present ? YVEX_BACKEND_CAPABILITY_SUPPORTED : YVEX_BACKEND_CAPABILITY_FAILED,
                   present ? YVEX_BACKEND_CAPABILITY_REASON_NONE
                           : YVEX_BACKEND_CAPABILITY_REASON_FUNCTION_MISSING,
                   present, err);
}

/* src/backend/cuda/capability.c:724-748 */
int yvex_rocm_require_capability(yvex_backend *backend, yvex_backend_operation_variant variant,
                                 const char *where, yvex_error *err)
{
    yvex_backend_capability_result result;
    const yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc = yvex_backend_query_capability(backend, variant, &result, err);
    if (rc != YVEX_OK) return rc;
    /* tensor traffic allocates, copies, clears or waits: none of it can be recorded */
    if (state && state->recording && variant <= YVEX_BACKEND_VARIANT_TENSOR_COPY) {
        yvex_error_set(err, YVEX_ERR_STATE, where ? where : "rocm.require_capability",
                       "not available while a launch sequence is being recorded");
        return YVEX_ERR_STATE;
    }
    if (result.state == YVEX_BACKEND_CAPABILITY_SUPPORTED) return YVEX_OK;
    rc = result.state == YVEX_BACKEND_CAPABILITY_FAILED ? YVEX_ERR_BACKEND : YVEX_ERR_UNSUPPORTED;
    yvex_error_setf(err, rc, where ? where : "rocm.require_capability", "%s refused: %s",
                    yvex_backend_operation_variant_name(variant),
                    yvex_backend_capability_reason_name(result.reason));
    return rc;
}

/* Function id of a bundle symbol, -1 when the bundle has no such kernel. */
int yvex_rocm_function_find(const char *symbol)
{
    size_t i;
    if (!symbol) return -1;
    for (i = 0; i < sizeof(rocm_kernel_bindings) / sizeof(rocm_kernel_bindings[0]); ++i)
        if (strcmp(rocm_kernel_bindings[i].symbol, symbol) == 0)
            return (int)rocm_kernel_bindings[i].slot;
    return -1;
}

/* src/backend/cuda/capability.c:750-791 */
int yvex_rocm_launch(yvex_backend *backend, yvex_rocm_function_id function,
                     yvex_backend_operation_variant variant, unsigned int grid_x,
                     unsigned int grid_y, unsigned int grid_z, unsigned int block,
                     unsigned int lds_bytes, void *params, const char *where, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    void *arguments[1];
    int probe;
    int rc = yvex_rocm_require_capability(backend, variant, where, err);
    if (rc != YVEX_OK) return rc;
    if (!state || function >= YVEX_ROCM_FN_COUNT || !state->functions[function]) {
        capability_fail(backend, variant, YVEX_BACKEND_CAPABILITY_REASON_FUNCTION_MISSING);
        yvex_error_set(err, YVEX_ERR_BACKEND, where, "admitted ROCm function handle is missing");
        return YVEX_ERR_BACKEND;
    }
    if (!grid_x || !grid_y || !grid_z || !block || block > 1024u) {
        yvex_error_set(err, YVEX_ERR_BOUNDS, where, "launch geometry is out of range");
        return YVEX_ERR_BOUNDS;
    }
    if (test_failure_matches("YVEX_TEST_ROCM_LAUNCH_FAILURE", variant)) {
        capability_fail(backend, variant, YVEX_BACKEND_CAPABILITY_REASON_LAUNCH_FAILED);
        yvex_error_set(err, YVEX_ERR_BACKEND, where, "injected ROCm launch failure");
        return YVEX_ERR_BACKEND;
    }
    arguments[0] = params;
    probe = !state->recording && state->probe_function == (int)function &&
            state->probe_count < YVEX_ROCM_PROBE_MAX;
    if (probe && state->driver.timed_launch && (unsigned long long)grid_x * block <= 0xffffffffull) {
        /* the two events take the kernel's own begin and end timestamps */
        rc = yvex_rocm_status(&state->driver,
                              state->driver.timed_launch(state->functions[function], grid_x * block,
                                                         grid_y, grid_z, block, 1u, 1u, lds_bytes,
                                                         yvex_rocm_stream(state), arguments, NULL,
                                                         state->probe_events[2u * state->probe_count],
                                                         state->probe_events[2u * state->probe_count + 1u],
                                                         0u),
                              where, err);
        if (rc == YVEX_OK) state->probe_count++;
    } else {
        if (probe)
            probe = state->driver.hipEventRecord(state->probe_events[2u * state->probe_count],
                                                 yvex_rocm_stream(state)) == hipSuccess;
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipModuleLaunchKernel(state->functions[function], grid_x,
                                                                  grid_y, grid_z, block, 1u, 1u,
                                                                  lds_bytes, yvex_rocm_stream(state), arguments,
                                                                  NULL),
                              where, err);
        if (probe && rc == YVEX_OK &&
            state->driver.hipEventRecord(state->probe_events[2u * state->probe_count + 1u],
                                         yvex_rocm_stream(state)) == hipSuccess)
            state->probe_count++;
    }
    if (rc != YVEX_OK) capability_fail(backend, variant, YVEX_BACKEND_CAPABILITY_REASON_LAUNCH_FAILED);
    else if (state->recording) state->recorded_launches++;
    return rc;
}

/* A queued copy that neither the batch launch nor the runtime took: the stream's contents are
 * not what the caller asked for, which fails the backend like a wait that failed. */
static int refuse_copy_queue(yvex_backend *backend, const char *where, yvex_error *err)
{
    capability_fail(backend, YVEX_BACKEND_VARIANT_TENSOR_COPY,
                    YVEX_BACKEND_CAPABILITY_REASON_SYNCHRONIZATION_FAILED);
    yvex_error_set(err, YVEX_ERR_BACKEND, where, "a queued device-to-device copy could not be issued");
    return YVEX_ERR_BACKEND;
}

/* src/backend/cuda/capability.c:793-830 */
int yvex_rocm_synchronize(yvex_backend *backend, yvex_backend_operation_variant variant,
                          const char *where, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!state) {
        yvex_error_set(err, YVEX_ERR_STATE, where, "ROCm backend state is missing");
        return YVEX_ERR_STATE;
    }
    if (state->recording) {
        yvex_error_set(err, YVEX_ERR_STATE, where,
                       "cannot wait for the stream while a launch sequence is being recorded");
        return YVEX_ERR_STATE;
    }
    if (test_failure_matches("YVEX_TEST_ROCM_SYNC_FAILURE", variant)) {
        capability_fail(backend, variant, YVEX_BACKEND_CAPABILITY_REASON_SYNCHRONIZATION_FAILED);
        yvex_error_set(err, YVEX_ERR_BACKEND, where, "injected ROCm synchronization failure");
        return YVEX_ERR_BACKEND;
    }
    rc = yvex_rocm_status(&state->driver, state->driver.hipStreamSynchronize(yvex_rocm_stream(state)), where,
                          err);
    if (rc == YVEX_OK && state->copy_queue.failed) return refuse_copy_queue(backend, where, err);
    if (rc != YVEX_OK)
        capability_fail(backend, variant, YVEX_BACKEND_CAPABILITY_REASON_SYNCHRONIZATION_FAILED);
    return rc;
}

/* How long the host watches the mailbox before it leaves the wait to the runtime. */
#define ROCM_MAILBOX_SPIN_NS 200000ll

static long long monotonic_ns(void)
{
    struct timespec now;
    clock_gettime(CLOCK_MONOTONIC, &now);
    return (long long)now.tv_sec * 1000000000ll + (long long)now.tv_nsec;
}

/* Watches the mailbox for `sequence`.  A device that does not answer within
 * ROCM_MAILBOX_SPIN_NS is waited for through the runtime, which also reports a device that
 * has failed. */
static int mailbox_wait(yvex_backend *backend, uint32_t sequence, const char *where, uint64_t *seen,
                        yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const long long deadline = monotonic_ns() + ROCM_MAILBOX_SPIN_NS;
    unsigned int turn = 0u;
    int rc;
    for (;;) {
        *seen = __atomic_load_n(state->status_mailbox, __ATOMIC_ACQUIRE);
        if ((uint32_t)(*seen >> 32) == sequence) return YVEX_OK;
        if ((++turn & 63u) == 0u && monotonic_ns() > deadline) break;
    }
    rc = yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_READ, where, err);
    if (rc != YVEX_OK) return rc;
    *seen = __atomic_load_n(state->status_mailbox, __ATOMIC_ACQUIRE);
    if ((uint32_t)(*seen >> 32) == sequence) return YVEX_OK;
    yvex_error_set(err, YVEX_ERR_BACKEND, where,
                   "the stream ended without the operation's answer reaching the host");
    return YVEX_ERR_BACKEND;
}

static int mailbox_launch(yvex_rocm_backend_state *state, yvex_rocm_function_id function,
                          unsigned int block, void *params, const char *where, yvex_error *err)
{
    void *arguments[1] = {params};
    return yvex_rocm_status(&state->driver,
                            state->driver.hipModuleLaunchKernel(state->functions[function], 1u, 1u, 1u,
                                                                block, 1u, 1u, 0u, yvex_rocm_stream(state),
                                                                arguments, NULL),
                            where, err);
}

/* The status word by way of the mailbox: a one-thread kernel behind the operation's kernels
 * stores (sequence, status) into host memory and the host watches for the sequence number,
 * about 8 us for an operation of one small kernel where a copy of the word and a wait for the
 * stream take 22.  Returns YVEX_ERR_UNSUPPORTED (and has done nothing) when this backend has
 * no mailbox. */
static int status_by_mailbox(yvex_backend *backend, const char *where, int32_t *host_status,
                             yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_status_forward_params fp;
    uint64_t seen = 0ull;
    int rc;
    if (!state->status_mailbox || !state->functions[YVEX_ROCM_FN_STATUS_FORWARD])
        return YVEX_ERR_UNSUPPORTED;
    fp.status = state->device_status;
    fp.mailbox = state->status_mailbox_device;
    fp.sequence = ++state->status_sequence;
    rc = mailbox_launch(state, YVEX_ROCM_FN_STATUS_FORWARD, 64u, &fp, where, err);
    if (rc == YVEX_OK) rc = mailbox_wait(backend, fp.sequence, where, &seen, err);
    if (rc != YVEX_OK) return rc;
    *host_status = (int32_t)(uint32_t)seen;
    return YVEX_OK;
}

/* Transfers of a few bytes cost the runtime's copy path 13 us (to the device) and 21 us (from
 * it) each, and the session layer makes three per layer and step
 * (src/runtime/stateful_attention.c:222-272).  A write of up to YVEX_ROCM_SMALL_WRITE_MAX
 * bytes travels in the arguments of a kernel instead (3 us, nothing waited for: the host's
 * buffer is free when the launch returns and later work is behind it on the stream); a read of
 * up to YVEX_ROCM_SMALL_READ_MAX bytes is copied by a kernel into host memory the device can
 * write while the host watches the mailbox (8 us).  Not while a launch sequence is recorded,
 * and not under an injected synchronisation failure, which belongs to the runtime's wait. */
static int small_transfer_admitted(const yvex_rocm_backend_state *state, yvex_rocm_function_id function,
                                   yvex_backend_operation_variant variant)
{
    return state && !state->recording && state->functions[function] &&
           !test_failure_matches("YVEX_TEST_ROCM_SYNC_FAILURE", variant);
}

/* Returns when everything asked of the stream so far has ended: an empty small read posts the
 * number the host watches for; without a mailbox, the runtime's wait. */
static int stream_reached(yvex_backend *backend, const char *where, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_small_read_params rp;
    uint64_t seen = 0ull;
    int rc;
    if (!state->status_mailbox || !state->functions[YVEX_ROCM_FN_SMALL_READ])
        return yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_WRITE, where, err);
    rp.src = NULL;
    rp.staging = state->read_staging_device;
    rp.mailbox = state->status_mailbox_device;
    rp.bytes = 0u;
    rp.sequence = ++state->status_sequence;
    rc = mailbox_launch(state, YVEX_ROCM_FN_SMALL_READ, 256u, &rp, where, err);
    if (rc == YVEX_OK) rc = mailbox_wait(backend, rp.sequence, where, &seen, err);
    return rc;
}

int yvex_rocm_small_write(yvex_backend *backend, void *dst, const void *src, unsigned long long bytes,
                          const char *where, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_small_write_params wp;
    int rc;
    if (!bytes || bytes > YVEX_ROCM_SMALL_WRITE_MAX ||
        !small_transfer_admitted(state, YVEX_ROCM_FN_SMALL_WRITE, YVEX_BACKEND_VARIANT_TENSOR_WRITE))
        return YVEX_ERR_UNSUPPORTED;
    wp.dst = dst;
    wp.bytes = (uint32_t)bytes;
    wp.reserved = 0u;
    memcpy(wp.data, src, (size_t)bytes);
    rc = mailbox_launch(state, YVEX_ROCM_FN_SMALL_WRITE, 256u, &wp, where, err);
    /* Alone on its device, everything that can read the tensor is behind the write on this
     * stream.  With session backends about (each has a stream of its own, and a written
     * tensor may be read from any of them with no event in between) the write is waited for,
     * as the runtime's copy was; opening a session backend waits for the primary's stream. */
    if (rc == YVEX_OK &&
        (backend->resource_owner != backend ||
         (atomic_load_explicit(&backend->lifecycle, memory_order_acquire) & YVEX_BACKEND_LIFECYCLE_CHILD_MASK)))
        rc = stream_reached(backend, where, err);
    return rc;
}

int yvex_rocm_small_read(yvex_backend *backend, void *dst, const void *src, unsigned long long bytes,
                         const char *where, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    yvex_rocm_small_read_params rp;
    uint64_t seen = 0ull;
    int rc;
    if (!bytes || bytes > YVEX_ROCM_SMALL_READ_MAX ||
        !small_transfer_admitted(state, YVEX_ROCM_FN_SMALL_READ, YVEX_BACKEND_VARIANT_TENSOR_READ) ||
        !state->status_mailbox || !state->read_staging)
        return YVEX_ERR_UNSUPPORTED;
    rp.src = src;
    rp.staging = state->read_staging_device;
    rp.mailbox = state->status_mailbox_device;
    rp.bytes = (uint32_t)bytes;
    rp.sequence = ++state->status_sequence;
    rc = mailbox_launch(state, YVEX_ROCM_FN_SMALL_READ, 256u, &rp, where, err);
    if (rc == YVEX_OK) rc = mailbox_wait(backend, rp.sequence, where, &seen, err);
    if (rc == YVEX_OK && state->copy_queue.failed) rc = refuse_copy_queue(backend, where, err);
    if (rc != YVEX_OK) return rc;
    memcpy(dst, state->read_staging, (size_t)bytes);
    return YVEX_OK;
}

/* Reads the device status word once the stream's work has ended (through the mailbox, or
 * with a copy whose wait synchronises the stream), clears it when set, and maps it like
 * src/backend/cuda/transformer.c:648-660. */
int yvex_rocm_status_check(yvex_backend *backend, const char *where,
                           yvex_backend_operation_facts *facts, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    int32_t host_status = 0;
    int rc, cleared = 0;
    if (state->recording) {
        yvex_error_set(err, YVEX_ERR_STATE, where,
                       "cannot read the device status while a launch sequence is being recorded");
        return YVEX_ERR_STATE;
    }
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    rc = test_failure_matches("YVEX_TEST_ROCM_SYNC_FAILURE", YVEX_BACKEND_VARIANT_TENSOR_READ)
             ? YVEX_ERR_UNSUPPORTED /* the injected failure belongs to the runtime's wait */
             : status_by_mailbox(backend, where, &host_status, err);
    if (rc == YVEX_OK) {
        cleared = 1; /* the forwarding kernel cleared a word that was set */
    } else if (rc == YVEX_ERR_UNSUPPORTED) {
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemcpyAsync(&host_status, state->device_status,
                                                           sizeof(host_status), hipMemcpyDeviceToHost,
                                                           yvex_rocm_stream(state)),
                              where, err);
        if (rc == YVEX_OK)
            rc = yvex_rocm_synchronize(backend, YVEX_BACKEND_VARIANT_TENSOR_READ, where, err);
    }
    if (rc == YVEX_OK && state->copy_queue.failed)
        rc = refuse_copy_queue(backend, where, err);
    if (rc != YVEX_OK) return rc;
    state->status_dirty = 0;
    backend->stats.d2h_bytes += sizeof(host_status);
    if (facts) {
        facts->download_count += 1ull;
        facts->d2h_bytes += sizeof(host_status);
        facts->device_synchronizations += 1ull;
    }
    if (!host_status) {
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (!cleared) {
        rc = yvex_rocm_status(&state->driver,
                              state->driver.hipMemsetAsync(state->device_status, 0,
                                                           sizeof(host_status), yvex_rocm_stream(state)),
                              where, err);
        if (rc != YVEX_OK) return rc;
    }
    switch (host_status) {
    case 2:
        yvex_error_set(err, YVEX_ERR_BOUNDS, where,
                       "attention kernel refused a page id or context length out of range");
        return YVEX_ERR_BOUNDS;
    case 3:
        yvex_error_set(err, YVEX_ERR_STATE, where, "attention softmax sum is zero");
        return YVEX_ERR_STATE;
    default:
        yvex_error_set(err, YVEX_ERR_FORMAT, where, "attention produced invalid numerics");
        return YVEX_ERR_FORMAT;
    }
}

int yvex_rocm_complete(yvex_backend *backend, yvex_backend_operation_variant variant,
                       const char *where, yvex_backend_operation_facts *facts, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    (void)variant;
    if (state->recording) { /* nothing ran: the replay completes the operation */
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (state->completion_mode == YVEX_ROCM_COMPLETION_DEFERRED) {
        state->status_dirty = 1;
        yvex_error_clear(err);
        return YVEX_OK;
    }
    return yvex_rocm_status_check(backend, where, facts, err);
}
