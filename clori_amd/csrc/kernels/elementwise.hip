// The element-wise operators the reference's decoder runs around attention, on F32
// activations whose values are bf16-representable between the operators
// (src/runtime/decoder.c:1112-1131 rotary then rounding, :1266-1269 output gate, the split of
// the interleaved query/gate projection in front of them).  Memory-bound, one thread per
// element; they exist so that the reference's attention block runs on this backend through
// the reference's own operator slots, call for call.  The fused forms (page writer, history
// writer, gate in the attention epilogue) are what a caller that can change its calls uses.
#include "mfma.h"

#include "../kernel_params.h"

namespace {

__device__ inline uint64_t element_index()
{
    return (uint64_t)blockIdx.x * (uint64_t)YVEX_ROCM_ELEMENTWISE_BLOCK + (uint64_t)threadIdx.x;
}

// Round to nearest even onto the bf16 grid, as a float (the hardware convert rounds exactly
// as the reference's float_to_bf16_rne for every finite value and for overflow).
__device__ inline float bf16_rounded(float value)
{
    return __builtin_bit_cast(float, pack_bf16x2(value, 0.f) << 16);
}

}  // namespace

// src/backend/cuda/transformer_kernels.cu:110-134 (the kernel behind the rotary_half_f32 slot,
// src/backend/cuda/capability.c:35): plain F32 rotate-half, nothing rounded.  The two float
// expressions are evaluated as fma(first, cosine, -(second * sine)) and
// fma(second, cosine, first * sine): one legal contraction of the reference's source, the one
// LLVM picks for both GPU targets; which one the reference's compiler picks is not visible in
// its sources, so the last bit of a result is not pinned by the reference.
extern "C" __global__ void __launch_bounds__(YVEX_ROCM_ELEMENTWISE_BLOCK)
yvex_rocm_rotary_half_plain_f32(const yvex_rocm_elementwise_params p)
{
#pragma clang fp contract(off)
    const uint64_t pair = element_index(), half = p.rotary_dim / 2u;
    if (pair >= p.count) return;
    const uint64_t vector = pair / half, lane = pair % half;
    const uint64_t token = vector / p.heads, base = vector * p.head_dim;
    const float cosine = p.left[token * p.rotary_dim + lane], sine = p.right[token * p.rotary_dim + lane];
    const float first = p.values[base + lane], second = p.values[base + half + lane];
    const float second_sine = second * sine, first_sine = first * sine;
    p.values[base + lane] = __builtin_fmaf(first, cosine, -second_sine);
    p.values[base + half + lane] = __builtin_fmaf(second, cosine, first_sine);
}

// src/backend/cuda/kernels.cu:40-58: every value onto the bf16 grid in place; a value that is
// not finite is left as it is and reported.
extern "C" __global__ void __launch_bounds__(YVEX_ROCM_ELEMENTWISE_BLOCK)
yvex_rocm_bf16_round_f32(const yvex_rocm_elementwise_params p)
{
    const uint64_t index = element_index();
    if (index >= p.count) return;
    const float value = p.values[index];
    if (!isfinite(value)) {
        atomicCAS(p.status, 0, YVEX_ROCM_DEVICE_NUMERIC);
        return;
    }
    p.values[index] = bf16_rounded(value);
}

// src/backend/cuda/transformer_kernels.cu:353-364: values * 1 / (1 + exp(-gate)), rounded to
// bf16; the same sigmoid as the gate fused into the attention epilogues.
extern "C" __global__ void __launch_bounds__(YVEX_ROCM_ELEMENTWISE_BLOCK)
yvex_rocm_sigmoid_product_bf16_f32(const yvex_rocm_elementwise_params p)
{
    const uint64_t index = element_index();
    if (index >= p.count) return;
    p.values[index] = bf16_rounded(p.left[index] * sigmoid(p.right[index]));
}

// src/backend/cuda/transformer_kernels.cu:455-473: rows of [heads][2][head_dim] into two rows
// of [heads][head_dim] (the query and the gate halves of one projection).
extern "C" __global__ void __launch_bounds__(YVEX_ROCM_ELEMENTWISE_BLOCK)
yvex_rocm_split_interleaved_two_f32(const yvex_rocm_elementwise_params p)
{
    const uint64_t index = element_index(), width = p.heads * p.head_dim;
    if (index >= p.count) return;
    const uint64_t row = index / width, within = index % width;
    const uint64_t head = within / p.head_dim, lane = within % p.head_dim;
    const uint64_t at = row * 2u * width + head * 2u * p.head_dim + lane;
    p.values[index] = p.left[at];
    p.second[index] = p.left[at + p.head_dim];
}

// Completion of an operation without a copy: the status word as the operation's kernels left
// it (cleared here when set) goes, with the sequence number the host is waiting for, into a
// word of host memory in one 8-byte store.  It runs behind those kernels on their stream, so
// the host that sees the number knows they have ended.
extern "C" __global__ void __launch_bounds__(64)
yvex_rocm_status_forward(const yvex_rocm_status_forward_params p)
{
    if (threadIdx.x != 0u) return;
    const int32_t status = __hip_atomic_load(p.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (status != 0) __hip_atomic_store(p.status, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(p.mailbox, ((uint64_t)p.sequence << 32) | (uint32_t)status, __ATOMIC_RELEASE,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}

// Small device-to-device copies queued by the host, one workgroup column per copy.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_copy_batch(const yvex_rocm_copy_batch_params p)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const uint32_t copy = blockIdx.y, pieces = p.bytes[copy] / 16u;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(p.src[copy]);
    u32x4 *dst = reinterpret_cast<u32x4 *>(p.dst[copy]);
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < pieces; i += gridDim.x * 256u) dst[i] = src[i];
}

// A tensor write of a few bytes (the session layer writes a layer's token positions, eight
// bytes per token, at every step: src/runtime/stateful_attention.c:222-243): the bytes arrive
// in the kernel's arguments, so the host's buffer is free when the launch returns and nothing
// waits.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_small_write(const yvex_rocm_small_write_params p)
{
    unsigned char *dst = static_cast<unsigned char *>(p.dst);
    if (((reinterpret_cast<uintptr_t>(p.dst) | p.bytes) & 3u) == 0u) {
        const uint32_t *words = reinterpret_cast<const uint32_t *>(p.data);
        for (uint32_t i = threadIdx.x; i < p.bytes / 4u; i += 256u) reinterpret_cast<uint32_t *>(dst)[i] = words[i];
    } else {
        for (uint32_t i = threadIdx.x; i < p.bytes; i += 256u) dst[i] = p.data[i];
    }
}

// A tensor read of a few KB (the session layer reads the new key and value rows back at every
// step, src/runtime/stateful_attention.c:245-272): the bytes go into host memory the device
// can write, then the sequence number the host is watching for.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_small_read(const yvex_rocm_small_read_params p)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const unsigned char *src = static_cast<const unsigned char *>(p.src);
    unsigned char *staging = static_cast<unsigned char *>(p.staging);
    if (((reinterpret_cast<uintptr_t>(p.src) | p.bytes) & 15u) == 0u) {
        for (uint32_t i = threadIdx.x; i < p.bytes / 16u; i += 256u)
            reinterpret_cast<u32x4 *>(staging)[i] = reinterpret_cast<const u32x4 *>(src)[i];
    } else {
        for (uint32_t i = threadIdx.x; i < p.bytes; i += 256u) staging[i] = src[i];
    }
    __threadfence_system();  // this thread's bytes are in host memory before the number is
    __syncthreads();
    if (threadIdx.x == 0u)
        __hip_atomic_store(p.mailbox, (uint64_t)p.sequence << 32, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
