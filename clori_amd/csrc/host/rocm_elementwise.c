/* The element-wise operator slots of the transformer operations table that the reference's
 * decoder calls around attention (include/yvex/internal/transformer.h:276-339; callers
 * src/runtime/decoder.c:989-997 bf16_round, :1030-1046 and :1266-1269 sigmoid_product_bf16,
 * :1112-1131 rotary_half_f32, the query/gate split of the attention projections):
 * validation and refusal as in src/backend/cuda/transformer.c:409-470,1356-1392 and
 * src/backend/cuda/decoder.c:11-130 (YVEX_ERR_FORMAT for anything but packed, written F32
 * tensors of this backend with the declared element counts), one launch each, completed like
 * every operation of this backend. */
#include "rocm_state.h"
#include "../kernel_params.h"

#include <limits.h>
#include <string.h>

enum { ELEMENTWISE_VARIANT = YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32 };

static int refuse_format(yvex_error *err, const char *where, const char *message)
{
    yvex_error_set(err, YVEX_ERR_FORMAT, where, message);
    return YVEX_ERR_FORMAT;
}

/* A packed F32 tensor of this backend with exactly `elements` values (and written, when it is
 * an input). */
static int f32_tensor(const yvex_backend *backend, const yvex_device_tensor *tensor,
                      unsigned long long elements, int require_written)
{
    unsigned long long bytes;
    return backend_tensor_owner_is(backend, tensor) && (!require_written || tensor->is_written) &&
           tensor->dtype == YVEX_DTYPE_F32 && tensor->data &&
           yvex_core_u64_mul(elements, sizeof(float), &bytes) && tensor->bytes == bytes;
}

static int elementwise_run(yvex_backend *backend, yvex_rocm_function_id function,
                           yvex_rocm_elementwise_params *params, unsigned long long threads,
                           const char *where, yvex_backend_operation_facts *facts, yvex_error *err)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const unsigned long long grid = (threads + YVEX_ROCM_ELEMENTWISE_BLOCK - 1ull) /
                                    YVEX_ROCM_ELEMENTWISE_BLOCK;
    int rc;
    params->status = state->device_status;
    backend_workspace_reset(backend);
    rc = yvex_rocm_launch(backend, function, (yvex_backend_operation_variant)ELEMENTWISE_VARIANT,
                          (unsigned int)grid, 1u, 1u, YVEX_ROCM_ELEMENTWISE_BLOCK, 0u, params, where, err);
    if (rc == YVEX_OK) {
        facts->kernel_launches = 1ull;
        facts->compulsory_memory_facts_available = 1;
        rc = yvex_rocm_complete(backend, (yvex_backend_operation_variant)ELEMENTWISE_VARIANT, where,
                                facts, err);
    }
    return rc;
}

/* Every tensor handed to a kernel lies on committed memory (reserved ranges). */
static int backed(const yvex_device_tensor *a, const yvex_device_tensor *b,
                  const yvex_device_tensor *c, const yvex_device_tensor *d)
{
    return yvex_rocm_tensor_backed(a) && (!b || yvex_rocm_tensor_backed(b)) &&
           (!c || yvex_rocm_tensor_backed(c)) && (!d || yvex_rocm_tensor_backed(d));
}

static int unbacked(yvex_error *err, const char *where)
{
    yvex_error_set(err, YVEX_ERR_STATE, where, "a tensor reaches into a reserved range that is not committed");
    return YVEX_ERR_STATE;
}

/* src/backend/cuda/transformer.c:409-470 */
int yvex_rocm_rotary_half_f32(yvex_backend *backend, yvex_device_tensor *values,
                              const yvex_device_tensor *cosines, const yvex_device_tensor *sines,
                              unsigned long long tokens, unsigned long long heads,
                              unsigned long long head_dim, unsigned long long rotary_dim,
                              yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.transformer.rotary-f32";
    unsigned long long vectors, elements, table_elements, tasks;
    yvex_rocm_elementwise_params params;
    int rc;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (!backend || !facts) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, where, "backend and result facts are required");
        return YVEX_ERR_INVALID_ARG;
    }
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_state(backend) || !tokens || !heads || !head_dim || !rotary_dim ||
        rotary_dim > head_dim || (rotary_dim & 1ull) || !yvex_core_u64_mul(tokens, heads, &vectors) ||
        !yvex_core_u64_mul(vectors, head_dim, &elements) ||
        !yvex_core_u64_mul(tokens, rotary_dim, &table_elements) ||
        !yvex_core_u64_mul(vectors, rotary_dim / 2ull, &tasks) ||
        !f32_tensor(backend, values, elements, 1) || !f32_tensor(backend, cosines, table_elements, 1) ||
        !f32_tensor(backend, sines, table_elements, 1) ||
        tasks > (unsigned long long)UINT_MAX * YVEX_ROCM_ELEMENTWISE_BLOCK)
        return refuse_format(err, where, "packed F32 vectors and explicit rotary tables are required");
    if (!backed(values, cosines, sines, NULL)) return unbacked(err, where);
    memset(&params, 0, sizeof(params));
    params.values = (float *)values->data;
    params.left = (const float *)cosines->data;
    params.right = (const float *)sines->data;
    params.count = tasks;
    params.heads = heads;
    params.head_dim = head_dim;
    params.rotary_dim = rotary_dim;
    rc = elementwise_run(backend, YVEX_ROCM_FN_ROTARY_HALF_PLAIN_F32, &params, tasks, where, facts, err);
    if (rc == YVEX_OK) yvex_error_clear(err);
    return rc;
}

/* src/backend/cuda/transformer.c:1356-1392 */
int yvex_rocm_bf16_round(yvex_backend *backend, yvex_device_tensor *values, unsigned long long count,
                         yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.transformer.bf16-round";
    unsigned long long tasks;
    yvex_rocm_elementwise_params params;
    int rc;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (!backend || !facts) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, where, "backend and result facts are required");
        return YVEX_ERR_INVALID_ARG;
    }
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_state(backend) || !count || !f32_tensor(backend, values, count, 1) ||
        !yvex_core_u64_add(count, YVEX_ROCM_ELEMENTWISE_BLOCK - 1ull, &tasks) ||
        tasks / YVEX_ROCM_ELEMENTWISE_BLOCK > UINT_MAX)
        return refuse_format(err, where, "one finite bounded F32 activation is required");
    if (!backed(values, NULL, NULL, NULL)) return unbacked(err, where);
    memset(&params, 0, sizeof(params));
    params.values = (float *)values->data;
    params.count = count;
    rc = elementwise_run(backend, YVEX_ROCM_FN_BF16_ROUND_F32, &params, count, where, facts, err);
    if (rc == YVEX_OK) yvex_error_clear(err);
    return rc;
}

/* src/backend/cuda/decoder.c:75-130 */
int yvex_rocm_sigmoid_product_bf16(yvex_backend *backend, const yvex_device_tensor *values,
                                   const yvex_device_tensor *gate, yvex_device_tensor *output,
                                   unsigned long long count, yvex_backend_operation_facts *facts,
                                   yvex_error *err)
{
    static const char where[] = "rocm.decoder.sigmoid-product";
    unsigned long long bytes, tasks;
    yvex_rocm_elementwise_params params;
    int rc;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (!backend || !facts) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, where, "backend and result facts are required");
        return YVEX_ERR_INVALID_ARG;
    }
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_state(backend) || !count || !yvex_core_u64_mul(count, sizeof(float), &bytes) ||
        !yvex_core_u64_add(count, YVEX_ROCM_ELEMENTWISE_BLOCK - 1ull, &tasks) ||
        tasks / YVEX_ROCM_ELEMENTWISE_BLOCK > UINT_MAX || !f32_tensor(backend, values, count, 1) ||
        !f32_tensor(backend, gate, count, 1) || !f32_tensor(backend, output, count, 0))
        return refuse_format(err, where, "equal bounded F32 decoder activations are required");
    if (!backed(values, gate, output, NULL)) return unbacked(err, where);
    memset(&params, 0, sizeof(params));
    params.values = (float *)output->data;
    params.left = (const float *)values->data;
    params.right = (const float *)gate->data;
    params.count = count;
    rc = elementwise_run(backend, YVEX_ROCM_FN_SIGMOID_PRODUCT_BF16_F32, &params, count, where, facts, err);
    if (rc == YVEX_OK) {
        output->is_written = 1;
        facts->activation_bytes = 3ull * bytes;
        yvex_error_clear(err);
    }
    return rc;
}

/* src/backend/cuda/decoder.c:11-73 */
int yvex_rocm_split_interleaved_two_f32(yvex_backend *backend, const yvex_device_tensor *input,
                                        yvex_device_tensor *first, yvex_device_tensor *second,
                                        unsigned long long rows, unsigned long long heads,
                                        unsigned long long head_dimension,
                                        yvex_backend_operation_facts *facts, yvex_error *err)
{
    static const char where[] = "rocm.decoder.split-interleaved-two";
    unsigned long long width, output_values, input_values, tasks;
    yvex_rocm_elementwise_params params;
    int rc;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (!backend || !facts) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, where, "backend and result facts are required");
        return YVEX_ERR_INVALID_ARG;
    }
    rc = backend_dispatch_admit(backend, where, err);
    if (rc != YVEX_OK) return rc;
    if (!yvex_rocm_state(backend) || !rows || !heads || !head_dimension ||
        !yvex_core_u64_mul(heads, head_dimension, &width) ||
        !yvex_core_u64_mul(rows, width, &output_values) ||
        !yvex_core_u64_mul(output_values, 2ull, &input_values) ||
        !yvex_core_u64_add(output_values, YVEX_ROCM_ELEMENTWISE_BLOCK - 1ull, &tasks) ||
        tasks / YVEX_ROCM_ELEMENTWISE_BLOCK > UINT_MAX || !f32_tensor(backend, input, input_values, 1) ||
        !f32_tensor(backend, first, output_values, 0) || !f32_tensor(backend, second, output_values, 0) ||
        input == first || input == second || first == second || first->data == second->data ||
        input->data == first->data || input->data == second->data)
        return refuse_format(err, where,
                             "one per-head interleaved F32 pair and independent outputs are required");
    if (!backed(input, first, second, NULL)) return unbacked(err, where);
    memset(&params, 0, sizeof(params));
    params.values = (float *)first->data;
    params.second = (float *)second->data;
    params.left = (const float *)input->data;
    params.count = output_values;
    params.heads = heads;
    params.head_dim = head_dimension;
    rc = elementwise_run(backend, YVEX_ROCM_FN_SPLIT_INTERLEAVED_TWO_F32, &params, output_values, where,
                         facts, err);
    if (rc == YVEX_OK) {
        first->is_written = second->is_written = 1;
        facts->activation_bytes = 4ull * output_values * sizeof(float);
        yvex_error_clear(err);
    }
    return rc;
}
