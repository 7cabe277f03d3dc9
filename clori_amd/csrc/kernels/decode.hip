// Split-K flash-decoding for gfx950 (wave64): one query token per session against a
// bf16 KV cache, grouped-query heads sharing each K/V read.
//
// One wave owns one (context chunk, kv head, session).  The query heads of the group
// are the N dimension of the MFMA tiles (padded to 16), so K and V are read from HBM
// once per group.  Per 16-token tile:
//     S^T[token][head]  = K[token][:] . Q[head][:]      4 x v_mfma_f32_16x16x32_bf16
//     online softmax over tokens in fp32 (exp2, scale*log2e folded into the score)
//     O^T[dim][head]   += V^T[dim][token] . P[token][head]   8 x v_mfma_f32_16x16x16_bf16
// The S^T accumulator layout (lane = head, 4 consecutive tokens per lane) is exactly
// the B-operand layout of the second product, so P never leaves registers.  K and V
// tiles go from global memory straight into MFMA operand registers: the paged layouts
// below make every wave-level load one contiguous run (no LDS, no barriers).
//
// Paged layout, per (page, kv head), 16 tokens x 128 lanes:
//     K block  uint16 [16 lane-chunks of 8][16 tokens][8]      elem(t,c) = ((c/8)*16+t)*8 + c%8
//     V block  uint16 [128 lanes][16 tokens]                   elem(t,c) = c*16 + t
// Token-major layout (the reference's [token][kv head][dim] history rows, with a
// per-token stride so the interleaved [K|V] rows of
// src/runtime/stateful_attention.c:326-352 are addressable): K rows are read in 16-byte
// pieces, V is gathered transposed.
//
// Partials (running max in log2 units, sum, unnormalised accumulator) go to the
// workspace; yvex_rocm_decode_merge combines them with a log-sum-exp merge.
#include "mfma.h"

#include "../kernel_params.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kPageTokens = 16;

struct Tile {
    u32x4 k[4];  // K[token = lane%16][32*j + 8*(lane/16) .. +7]
    u32x2 v[8];  // V[tokens 4*(lane/16)..+3][dim 16*b + lane%16]
};

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

__device__ inline void load_tile_paged(Tile &t, const uint16_t *kblock, const uint16_t *vblock,
                                       int lane)
{
    const int n = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) t.k[j] = load_b128(kblock + (j * 64 + lane) * 8);
#pragma unroll
    for (int b = 0; b < 8; ++b) t.v[b] = load_b64(vblock + (b * 16 + n) * 16 + g * 4);
}

// rows_left: tokens available from `first` on (rows beyond are clamped to the last
// valid row so no out-of-range address is formed; they are masked later).
__device__ inline void load_tile_rows(Tile &t, const uint16_t *k, const uint16_t *v,
                                      uint64_t k_stride, uint64_t v_stride, uint32_t first,
                                      uint32_t rows_left, int lane)
{
    const int n = lane & 15, g = lane >> 4;
    const uint32_t last = rows_left - 1u;
    const uint16_t *krow = k + (uint64_t)(first + min((uint32_t)n, last)) * k_stride;
#pragma unroll
    for (int j = 0; j < 4; ++j) t.k[j] = load_b128(krow + j * 32 + g * 8);
    const uint16_t *v0 = v + (uint64_t)(first + min((uint32_t)(g * 4 + 0), last)) * v_stride;
    const uint16_t *v1 = v + (uint64_t)(first + min((uint32_t)(g * 4 + 1), last)) * v_stride;
    const uint16_t *v2 = v + (uint64_t)(first + min((uint32_t)(g * 4 + 2), last)) * v_stride;
    const uint16_t *v3 = v + (uint64_t)(first + min((uint32_t)(g * 4 + 3), last)) * v_stride;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const int c = b * 16 + n;
        t.v[b].x = (uint32_t)v0[c] | ((uint32_t)v1[c] << 16);
        t.v[b].y = (uint32_t)v2[c] | ((uint32_t)v3[c] << 16);
    }
}

struct State {
    floatx4 o[8];  // O^T[dim 16*b + 4*(lane/16) + i][head lane%16]
    float m, l;    // running max (log2 units) and per-lane partial sum
};

// valid: number of real tokens in this 16-token tile (1..16).
__device__ inline void consume(State &st, const Tile &t, const bf16x8 (&q)[4], float scale_log2,
                               uint32_t valid, int lane)
{
    const int g = lane >> 4;
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) s = mfma_16x16x32(as_bf16x8(t.k[j]), q[j], s);
    float x[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        x[i] = (uint32_t)(g * 4 + i) < valid ? s[i] * scale_log2 : -INFINITY;
    float mloc = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
    mloc = fmaxf(mloc, xor_lanes(mloc, 16));
    mloc = fmaxf(mloc, xor_lanes(mloc, 32));
    const float m_new = fmaxf(st.m, mloc);
    // The running maximum rarely moves after the first tiles: rescale the accumulators
    // only when some lane of the wave saw a larger score.
    if (__builtin_amdgcn_ballot_w64(m_new > st.m) != 0ull) {
        const float alpha = fast_exp2(st.m - m_new);
        st.l *= alpha;
#pragma unroll
        for (int b = 0; b < 8; ++b) st.o[b] *= alpha;
        st.m = m_new;
    }
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = fast_exp2(x[i] - st.m);
    st.l += (p[0] + p[1]) + (p[2] + p[3]);
    u32x2 pb;
    pb.x = pack_bf16x2(p[0], p[1]);
    pb.y = pack_bf16x2(p[2], p[3]);
    const short4v pv = as_short4(pb);
    if (valid < (uint32_t)kPageTokens) {
        // rows past the context may hold anything (even NaN): a zero weight does not
        // neutralise them inside the MFMA, so clear them in the V operand
        uint32_t keep_lo = ((uint32_t)(g * 4 + 0) < valid ? 0x0000ffffu : 0u) |
                           ((uint32_t)(g * 4 + 1) < valid ? 0xffff0000u : 0u);
        uint32_t keep_hi = ((uint32_t)(g * 4 + 2) < valid ? 0x0000ffffu : 0u) |
                           ((uint32_t)(g * 4 + 3) < valid ? 0xffff0000u : 0u);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            u32x2 v = t.v[b];
            v.x &= keep_lo;
            v.y &= keep_hi;
            st.o[b] = mfma_16x16x16(as_short4(v), pv, st.o[b]);
        }
    } else {
#pragma unroll
        for (int b = 0; b < 8; ++b) st.o[b] = mfma_16x16x16(as_short4(t.v[b]), pv, st.o[b]);
    }
}

template <bool PAGED, int kDepth>
__device__ inline void decode_body(const yvex_rocm_decode_params &p)
{
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
    const uint32_t chunk = blockIdx.x, kv_head = blockIdx.y, session = blockIdx.z;
    const uint32_t limit = PAGED ? p.table_stride * (uint32_t)kPageTokens : p.fixed_context;
    const uint32_t ctx = p.context ? (uint32_t)p.context[session] : p.fixed_context;
    if (ctx == 0u || ctx > limit) {
        if (chunk == 0u && kv_head == 0u && lane == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return;
    }
    const uint32_t t0 = chunk * p.chunk_tokens;
    if (t0 >= ctx) return;
    const uint32_t t1 = min(ctx, t0 + p.chunk_tokens);
    const uint32_t group = p.query_heads / p.kv_heads;
    const uint32_t tiles = (t1 - t0 + kPageTokens - 1) / kPageTokens;

    bf16x8 q[4];
    {
        const uint16_t *qrow =
            p.q + ((uint64_t)session * p.query_heads + kv_head * group + min((uint32_t)n, group - 1u)) *
                      kHeadDim;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x4 raw = load_b128(qrow + j * 32 + g * 8);
            if ((uint32_t)n >= group) raw = (u32x4){0u, 0u, 0u, 0u};
            q[j] = as_bf16x8(raw);
        }
    }

    int32_t my_page = 0;
    const uint16_t *kbase = (const uint16_t *)p.k_pool, *vbase = (const uint16_t *)p.v_pool;
    if (PAGED) {
        // one coalesced read brings the chunk's page ids into the wave (chunk <= 64 pages)
        const int32_t *table =
            p.page_table + (uint64_t)session * p.table_stride + t0 / kPageTokens;
        if ((uint32_t)lane < tiles) {
            my_page = table[lane];
            if (my_page < 0 || (uint32_t)my_page >= p.pool_pages) {
                flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
                my_page = 0;
            }
        }
    } else {
        kbase += (uint64_t)kv_head * kHeadDim;
        vbase += (uint64_t)kv_head * kHeadDim;
    }
    const uint64_t block_elems = (uint64_t)kPageTokens * kHeadDim;

    auto fetch = [&](Tile &t, uint32_t i) {
        if (PAGED) {
            const uint32_t page = (uint32_t)__builtin_amdgcn_readlane(my_page, (int)i);
            const uint64_t off = ((uint64_t)page * p.kv_heads + kv_head) * block_elems;
            load_tile_paged(t, kbase + off, vbase + off, lane);
        } else {
            const uint32_t first = t0 + i * kPageTokens;
            load_tile_rows(t, kbase, vbase, p.k_token_stride, p.v_token_stride, first,
                           t1 - first, lane);
        }
    };

    State st;
#pragma unroll
    for (int b = 0; b < 8; ++b) st.o[b] = (floatx4){0.f, 0.f, 0.f, 0.f};
    st.m = -INFINITY;
    st.l = 0.f;

    // Ring of kDepth tile buffers: kDepth-1 tiles (8 KB each) stay in flight per wave
    // while one is consumed.  Every refill in the steady-state loop is unconditional (the
    // index is clamped to the last tile, a cache hit) so the number of outstanding loads
    // is the same on every trip and the waits the compiler places are partial
    // (vmcnt > 0) instead of draining the whole queue.
    Tile ring[kDepth];
    const uint32_t last_tile = tiles - 1u;
#pragma unroll
    for (int r = 0; r < kDepth; ++r) fetch(ring[r], min((uint32_t)r, last_tile));
    uint32_t i = 0u;
    for (; i + kDepth <= tiles; i += kDepth) {
#pragma unroll
        for (int r = 0; r < kDepth; ++r) {
            const uint32_t tile = i + (uint32_t)r;
            consume(st, ring[r], q, p.scale_log2,
                    min((uint32_t)kPageTokens, t1 - (t0 + tile * kPageTokens)), lane);
            fetch(ring[r], min(tile + kDepth, last_tile));
        }
    }
#pragma unroll
    for (int r = 0; r < kDepth - 1; ++r) {
        const uint32_t tile = i + (uint32_t)r;
        if (tile < tiles)
            consume(st, ring[r], q, p.scale_log2,
                    min((uint32_t)kPageTokens, t1 - (t0 + tile * kPageTokens)), lane);
    }

    float l = st.l;
    l += xor_lanes(l, 16);
    l += xor_lanes(l, 32);
    if ((uint32_t)n < group) {
        const uint64_t slot =
            ((uint64_t)session * p.max_chunks + chunk) * p.query_heads + kv_head * group + n;
        float *acc = p.part_acc + slot * kHeadDim + g * 4;
#pragma unroll
        for (int bb = 0; bb < 8; ++bb) *reinterpret_cast<floatx4 *>(acc + bb * 16) = st.o[bb];
        if (g == 0) {
            p.part_ml[slot * 2 + 0] = st.m;
            p.part_ml[slot * 2 + 1] = l;
        }
    }
}

}  // namespace

extern "C" __global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2)))
yvex_rocm_decode_paged_bf16(const yvex_rocm_decode_params p)
{
    decode_body<true, 3>(p);
}

extern "C" __global__ void __launch_bounds__(64)
yvex_rocm_decode_rows_bf16(const yvex_rocm_decode_params p)
{
    decode_body<false, 2>(p);
}

// Log-sum-exp merge of the chunk partials of one (session, query head); one thread per
// output lane.  grid = (query_heads, sessions), block = head_dim.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_decode_merge(const yvex_rocm_decode_merge_params p)
{
    const uint32_t head = blockIdx.x, session = blockIdx.y, d = threadIdx.x;
    const uint32_t ctx = p.context ? (uint32_t)p.context[session] : p.fixed_context;
    if (ctx == 0u || d >= p.head_dim) return;
    const uint32_t chunks = min(p.max_chunks, (ctx + p.chunk_tokens - 1u) / p.chunk_tokens);
    const uint64_t base = ((uint64_t)session * p.max_chunks) * p.query_heads + head;
    // The chunk loops carry no dependent loads: unrolled, eight partial rows are in
    // flight per thread, which is what keeps this pass in the microsecond range.
    float top = -INFINITY;
#pragma unroll 8
    for (uint32_t c = 0; c < chunks; ++c)
        top = fmaxf(top, p.part_ml[(base + (uint64_t)c * p.query_heads) * 2]);
    float total = 0.f, acc = 0.f;
#pragma unroll 8
    for (uint32_t c = 0; c < chunks; ++c) {
        const uint64_t slot = base + (uint64_t)c * p.query_heads;
        const float w = fast_exp2(p.part_ml[slot * 2] - top);
        total += w * p.part_ml[slot * 2 + 1];
        acc += w * p.part_acc[slot * p.head_dim + d];
    }
    const float o = acc / total;
    if (!isfinite(o)) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    p.out[((uint64_t)session * p.query_heads + head) * p.head_dim + d] = bf16_bits(o);
    if (p.lse && d == 0u)
        p.lse[(uint64_t)session * p.query_heads + head] = (top + fast_log2(total)) * YVEX_LN2;
}
