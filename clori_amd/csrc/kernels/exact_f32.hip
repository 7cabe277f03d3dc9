// Exact F32 attention kernels for gfx950 (wave64).
//
// These serve the reference's only numeric contract, EXACT_F32: F32 tensors in, F32
// out, no reduced-precision products.  They follow the CPU operator's arithmetic
// (src/backend/cpu.c:307-399 of the reference): double-precision dot products,
// softmax statistics and PV accumulation, the score stored as float and re-read.
// They are the correctness path for the reference's own test vectors; the bf16 MFMA
// kernels are the throughput path and are never substituted for these.
#include <hip/hip_runtime.h>

#include "../kernel_params.h"

namespace {

constexpr int kWave = 64;

__device__ inline double wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ inline double wave_max(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmax(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ inline void flag(int32_t *status, int code)
{
    atomicCAS(status, 0, code);
}

}  // namespace

// Single head, single query, with the score and probability scratches the reference
// primitive publishes.  grid 1, block 256.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_attention_f32(const yvex_rocm_attention_f32_params p)
{
    __shared__ double red[4];
    __shared__ double stat[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t d = p.head_dim;
    const uint64_t visible = p.causal ? p.position + 1 : p.seq_len;

    // pass 1: scores (one wave per row, lanes over the head dimension)
    double local_max = -INFINITY;
    for (uint64_t i = wave; i < p.seq_len; i += 4) {
        if (i >= visible) {
            if (lane == 0) {
                p.score[i] = 0.0f;
                p.prob[i] = 0.0f;
            }
            continue;
        }
        double acc = 0.0;
        for (uint64_t c = lane; c < d; c += kWave)
            acc += (double)p.q[c] * (double)p.k[i * d + c];
        acc = wave_sum(acc) * (double)p.scale;
        if (lane == 0) p.score[i] = (float)acc;
        local_max = fmax(local_max, acc);
    }
    if (lane == 0) red[wave] = local_max;
    __syncthreads();
    if (tid == 0) stat[0] = fmax(fmax(red[0], red[1]), fmax(red[2], red[3]));
    __syncthreads();
    const double max_score = stat[0];

    // pass 2: exponentials of the float-stored score, summed in a fixed order
    double part = 0.0;
    for (uint64_t i = tid; i < visible; i += 256) {
        double x = (double)p.score[i] - max_score;
        double e = x < -60.0 ? 0.0 : exp(x);
        p.prob[i] = (float)e;
        part += e;
    }
    part = wave_sum(part);
    __syncthreads();
    if (lane == 0) red[wave] = part;
    __syncthreads();
    if (tid == 0) stat[1] = (red[0] + red[1]) + (red[2] + red[3]);
    __syncthreads();
    const double sum_exp = stat[1];
    if (!(sum_exp > 0.0) || !isfinite(sum_exp)) {
        if (tid == 0) flag(p.status, sum_exp <= 0.0 ? YVEX_ROCM_DEVICE_SOFTMAX_ZERO
                                                   : YVEX_ROCM_DEVICE_NUMERIC);
        return;
    }
    for (uint64_t i = tid; i < visible; i += 256)
        p.prob[i] = (float)((double)p.prob[i] / sum_exp);
    __syncthreads();

    // pass 3: one thread per output lane, rows in ascending order like the reference
    for (uint64_t c = tid; c < d; c += 256) {
        double acc = 0.0;
        for (uint64_t i = 0; i < visible; ++i)
            acc += (double)p.prob[i] * (double)p.v[i * d + c];
        float o = (float)acc;
        if (!isfinite(o)) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        p.out[c] = o;
    }
}

// Multi-token grouped-query attention, one wave per (query token, query head).
// Lanes own head_dim/64 lanes of the row (head_dim <= 256); scores are reduced across
// the wave; online softmax and the PV accumulation run in double.
// grid = query_tokens * query_heads, block 64.
extern "C" __global__ void __launch_bounds__(64)
yvex_rocm_gqa_f32(const yvex_rocm_gqa_f32_params p)
{
    const int lane = threadIdx.x;
    const uint64_t unit = blockIdx.x;
    const uint64_t token = unit / p.query_heads, head = unit % p.query_heads;
    const uint64_t kv_head = head / (p.query_heads / p.kv_heads);
    const uint64_t visible = p.causal ? p.query_start + token + 1 : p.kv_tokens;
    const uint64_t d = p.head_dim;
    const float *q = p.q + token * p.q_stride + head * d;
    const float *k = p.k + kv_head * d;
    const float *v = p.v + kv_head * d;

    double qr[4], acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint64_t c = (uint64_t)lane + 64u * j;
        qr[j] = c < d ? (double)q[c] : 0.0;
        acc[j] = 0.0;
    }
    double m = -INFINITY, l = 0.0;
    for (uint64_t i = 0; i < visible; ++i) {
        const float *krow = k + i * p.k_stride;
        const float *vrow = v + i * p.v_stride;
        double s = 0.0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint64_t c = (uint64_t)lane + 64u * j;
            if (c < d) s += qr[j] * (double)krow[c];
        }
        s = (double)(float)(wave_sum(s) * (double)p.scale);
        double m_new = fmax(m, s);
        double alpha = exp(m - m_new), w = exp(s - m_new);
        l = l * alpha + w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint64_t c = (uint64_t)lane + 64u * j;
            if (c < d) acc[j] = acc[j] * alpha + w * (double)vrow[c];
        }
        m = m_new;
    }
    if (!(l > 0.0) || !isfinite(l) || !isfinite(m)) {
        if (lane == 0) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        return;
    }
    float *out = p.out + (token * p.query_heads + head) * d;
    bool bad = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint64_t c = (uint64_t)lane + 64u * j;
        if (c < d) {
            float o = (float)(acc[j] / l);
            bad |= !isfinite(o);
            out[c] = o;
        }
    }
    if (bad) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    if (p.lse && lane == 0) p.lse[token * p.query_heads + head] = (float)(m + log(l));
}

// Word fill, used instead of a memset node so the clear can be recorded in a graph.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_fill_u32(const yvex_rocm_fill_params p)
{
    uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * 256u;
    for (; i < p.words; i += stride) p.data[i] = p.value;
}

// Streaming read for the bandwidth probe (the counterpart of the in-place pass the reference
// times in src/backend/cuda/backend.c:1356-1399): each wave takes whole 8 KB blocks, eight
// independent 1 KB wave-loads in flight, blocks dealt round-robin to the waves; nothing is
// written.  The working set is a whole number of blocks.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_stream_read(const yvex_rocm_stream_params p)
{
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 *words = reinterpret_cast<const u32x4 *>(p.data);
    const uint64_t lane = threadIdx.x & 63u;
    const uint64_t wave = ((uint64_t)blockIdx.x * 256u + threadIdx.x) >> 6;
    const uint64_t waves = (uint64_t)gridDim.x * 4u, blocks = p.words / 512u;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (uint64_t b = wave; b < blocks; b += waves) {
        const u32x4 *base = words + b * 512u + lane;
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = base[j * 64];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc ^= v[j];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == p.never) p.sink[0] = 1u;
}
