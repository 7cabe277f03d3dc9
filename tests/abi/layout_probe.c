/* Prints the byte layout of the structures that cross the backend boundary, either as
 * this repository's header declares them or (with -DPROBE_REFERENCE_HEADERS and the
 * reference's include directory on the path) as the reference tree declares them.  The
 * test compiles it both ways and requires identical output. */
#include <stddef.h>
#include <stdio.h>
#ifdef PROBE_REFERENCE_HEADERS
#include <yvex/internal/transformer.h>
#else
#include "yvex_rocm.h"
#include "yvex_rocm_operations.h"
#endif

#define SIZE(type) printf("sizeof %s %zu\n", #type, sizeof(type))
#define OFFSET(type, member) printf("offsetof %s.%s %zu\n", #type, #member, offsetof(type, member))

int main(void)
{
    SIZE(yvex_error);
    SIZE(yvex_backend_options);
    SIZE(yvex_backend_memory_stats);
    SIZE(yvex_backend_tensor_desc);
    SIZE(yvex_backend_device_info);
    SIZE(yvex_backend_capability_result);
    SIZE(yvex_backend_operation_facts);
    SIZE(yvex_backend_bandwidth_evidence);
    SIZE(yvex_backend_attention_failure);
    SIZE(struct yvex_device_tensor);
    OFFSET(struct yvex_device_tensor, dtype);
    OFFSET(struct yvex_device_tensor, dims);
    OFFSET(struct yvex_device_tensor, bytes);
    OFFSET(struct yvex_device_tensor, data);
    OFFSET(struct yvex_device_tensor, backend_allocation);
    OFFSET(struct yvex_device_tensor, is_written);
    SIZE(yvex_transformer_attention_requirement);
    OFFSET(yvex_transformer_attention_requirement, query_token_stride);
    OFFSET(yvex_transformer_attention_requirement, query_dtype);
    OFFSET(yvex_transformer_attention_requirement, numeric_contract);
    OFFSET(yvex_transformer_attention_requirement, deterministic);
    SIZE(yvex_transformer_attention_request);
    OFFSET(yvex_transformer_attention_request, query);
    OFFSET(yvex_transformer_attention_request, output);
    SIZE(struct yvex_backend_transformer_operations);
    OFFSET(struct yvex_backend_transformer_operations, initial);
    OFFSET(struct yvex_backend_transformer_operations, attention_workspace_required);
    OFFSET(struct yvex_backend_transformer_operations, attention_execute);
    OFFSET(struct yvex_backend_transformer_operations, gated_delta_workspace_required);
    OFFSET(struct yvex_backend_transformer_operations, sigmoid_product_bf16);
    OFFSET(struct yvex_backend_transformer_operations, dense_decoder_execute);
    printf("value YVEX_BACKEND_KIND_ROCM %d\n", (int)YVEX_BACKEND_KIND_ROCM);
    printf("value YVEX_ERR_UNSUPPORTED %d\n", (int)YVEX_ERR_UNSUPPORTED);
    printf("value YVEX_DTYPE_BF16 %d\n", (int)YVEX_DTYPE_BF16);
    printf("value YVEX_BACKEND_VARIANT_ATTENTION_ENCODED %d\n", (int)YVEX_BACKEND_VARIANT_ATTENTION_ENCODED);
    printf("value YVEX_BACKEND_VARIANT_COUNT %d\n", (int)YVEX_BACKEND_VARIANT_COUNT);
    printf("value YVEX_TRANSFORMER_ATTENTION_NUMERIC_EXACT_F32 %d\n", (int)YVEX_TRANSFORMER_ATTENTION_NUMERIC_EXACT_F32);
    printf("value YVEX_TRANSFORMER_ATTENTION_MASK_CAUSAL %d\n", (int)YVEX_TRANSFORMER_ATTENTION_MASK_CAUSAL);
    printf("value YVEX_BACKEND_ATTENTION_FAILURE_CAPABILITY %d\n", (int)YVEX_BACKEND_ATTENTION_FAILURE_CAPABILITY);
    printf("value YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED %d\n", (int)YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED);
    return 0;
}
