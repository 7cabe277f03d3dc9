// EXACT_F32 grouped-query attention on the fp32 matrix cores of gfx950 (wave64).
//
// F32 tensors in, F32 out, every product an F32 product: the numeric contract of the
// reference's only attention request (src/backend/cuda/exact_attention.c:35-49) and the
// arithmetic of its own device kernel (float dot products, float online softmax,
// src/backend/cuda/transformer_kernels.cu:136-208), here in 32x32 tiles on
// v_mfma_f32_32x32x2_f32 instead of one row at a time.
//
// One workgroup = 128 consecutive query tokens of one query head, four waves of 32 queries.
// Key and value rows of the head's KV group go through LDS in tiles of 32 tokens, shared by
// the four waves, double buffered: the rows of tile t+1 are fetched into registers before
// the matrix work of tile t and written to the other buffer after it.
//
// Per tile a wave computes S^T = K Q^T (keys x queries), so that a lane owns one query
// column and 16 of the 32 key rows: the softmax statistics are in-lane but for one exchange
// with the lane 32 apart, and the exponentials are already in the operand layout of
// O^T += V^T P^T (head dims x queries), whose 32x32 blocks stay in registers for the whole
// row of tiles.  The contraction index of an MFMA is split between the two lane halves
// (lane / 32); both products are sums over it, so each half takes the part that is
// contiguous for it: half the head dimension for S^T, its own 16 key rows for O^T.
//
// grid = query_heads * ceil(query_tokens / 128), the longest (last) query tiles first;
// block = 256.
#include <hip/hip_runtime.h>

#include "../kernel_params.h"
#include "mfma.h"

namespace {

__device__ inline void flag_status(int32_t *status, int code)
{
    atomicCAS(status, 0, code);
}

__device__ inline floatx16 mfma_32x32x2(float a, float b, floatx16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// kBlocks: head_dim / 32.
template <int kBlocks>
struct GqaTile {
    static constexpr int kDim = 32 * kBlocks, kHalf = kDim / 2;
    static constexpr int kKeys = 32, kQueries = 128;
    // row strides in floats: the K operand is read 16 bytes per lane with the key in the lane
    // index (stride = 4 mod 64 banks), the V operand 4 bytes per lane with rows 4 apart in the
    // two lane halves (4 * stride = 32 mod 64 banks)
    static constexpr int kKStride = kDim + 4, kVStride = kDim + 8;
    static constexpr int kStageFloats = kKeys * (kKStride + kVStride);
    static constexpr int kChunks = kDim / 32;  // 16-byte pieces of a K (or V) tile per thread

    const yvex_rocm_gqa_f32_params &p;
    float *lds;
    const int tid, lane, wave, column, half;

    __device__ GqaTile(const yvex_rocm_gqa_f32_params &params, float *shared)
        : p(params), lds(shared), tid(threadIdx.x), lane(threadIdx.x & 63), wave(threadIdx.x >> 6),
          column(threadIdx.x & 31), half((threadIdx.x >> 5) & 1)
    {
    }

    // This thread's 16-byte pieces of one K or V tile on their way from global memory to LDS.
    struct Staged {
        floatx4 piece[kChunks];
    };

    // rows of tile `tile` of `rows` (K or V, `stride` elements per token); rows past the end
    // read as zero
    __device__ void fetch(const float *rows, uint64_t stride, uint64_t tile, uint64_t kv_head, Staged &s) const
    {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int c = tid + 256 * j, row = c / (kDim / 4), piece = c % (kDim / 4);
            const uint64_t key = tile * kKeys + (uint64_t)row;
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            s.piece[j] = zero;
            if (key < p.kv_tokens)
                s.piece[j] = *reinterpret_cast<const floatx4 *>(rows + key * stride + kv_head * kDim + 4 * piece);
        }
    }

    __device__ void stage(float *tile, int row_stride, const Staged &s) const
    {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int c = tid + 256 * j, row = c / (kDim / 4), piece = c % (kDim / 4);
            *reinterpret_cast<floatx4 *>(tile + row * row_stride + 4 * piece) = s.piece[j];
        }
    }

    // Items (one head, one tile of queries) are numbered heaviest first.  A scheduled launch
    // hands every workgroup a row of items (the count, then the items, 16 bytes: one scalar
    // load); otherwise the workgroup runs the one item its number stands for.
    __device__ void run() const
    {
        uint32_t count = 1u;
        u32x4 row = {0u, 0u, 0u, 0u};
        if (p.lists != nullptr) {
            typedef __attribute__((address_space(4))) const u32x4 constant_u32x4;
            row = *(constant_u32x4 *)(uintptr_t)(p.lists + (uint64_t)blockIdx.x * 8u);
            count = min(row.x & 0xffffu, 7u);
        }
        for (uint32_t j = 1u; j <= count; ++j) {
            const uint32_t word = j >> 1 == 0u ? row.x : j >> 1 == 1u ? row.y : j >> 1 == 2u ? row.z : row.w;
            item(p.lists != nullptr ? (word >> ((j & 1u) * 16u)) & 0xffffu : paired_item());
            // every wave is done with the tiles in LDS before the next item stages its own
            if (j < count) __syncthreads();
        }
    }

    __device__ uint32_t paired_item() const
    {
        // Without lists: the hardware gives workgroup b of the first 2 * pair_units to compute
        // unit b % pair_units, and the kernel is bound by the matrix cores, so a unit's time
        // follows the key tiles it walks: the second workgroup of a unit takes the second tier of
        // items in reverse, and the unit that got the heaviest item gets the lightest of them
        // (equal sums for causal walks; 433 against 459 us for 40 heads x 16 tiles of 2048 tokens).
        return blockIdx.x >= p.pair_units && blockIdx.x < 2u * p.pair_units
                   ? 3u * p.pair_units - 1u - blockIdx.x
                   : blockIdx.x;
    }

    __device__ void item(const uint64_t id) const
    {
        const uint64_t tiles_q = (p.query_tokens + kQueries - 1) / kQueries;
        const uint64_t head = id % p.query_heads;
        const uint64_t q_tile = tiles_q - 1 - id / p.query_heads;
        const uint64_t kv_head = head / (p.query_heads / p.kv_heads);
        const uint64_t q0 = q_tile * kQueries + (uint64_t)wave * 32u;
        // rows past the last query repeat it: they compute, they are not stored
        const uint64_t token = min(q0 + (uint64_t)column, p.query_tokens - 1);
        const uint64_t own = p.query_start + token;  // absolute position of this lane's query
        // last key any query of the workgroup, and of this wave, may see
        const uint64_t group_last = p.causal
            ? min(p.kv_tokens, p.query_start + min((q_tile + 1) * kQueries, p.query_tokens))
            : p.kv_tokens;
        const uint64_t wave_last = p.causal
            ? min(p.kv_tokens, p.query_start + min(q0 + 32u, p.query_tokens))
            : p.kv_tokens;
        const uint64_t tiles = (group_last + kKeys - 1) / kKeys;
        const uint64_t wave_tiles = q0 < p.query_tokens ? (wave_last + kKeys - 1) / kKeys : 0;

        // this lane's half of its query row: Q[token][half * kHalf + s], s = 0 .. kHalf-1
        float q[kHalf];
        {
            const float *row = p.q + token * p.q_stride + head * kDim + half * kHalf;
#pragma unroll
            for (int s = 0; s < kHalf; s += 4) {
                const floatx4 piece = *reinterpret_cast<const floatx4 *>(row + s);
                q[s] = piece[0];
                q[s + 1] = piece[1];
                q[s + 2] = piece[2];
                q[s + 3] = piece[3];
            }
        }

        floatx16 out[kBlocks];
#pragma unroll
        for (int b = 0; b < kBlocks; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) out[b][i] = 0.f;
        float top = -INFINITY, sum = 0.f;  // running maximum (natural units), this half's share of the denominator

        // The rows of tile t+1 travel in two halves so that only one tile's worth of registers
        // is tied up: K is fetched before the first product of tile t and written to the other
        // buffer after it, V likewise around the second product.  Every wave left both halves
        // of that buffer at the barrier that ended tile t-1.
        Staged next;
        fetch(p.k, p.k_stride, 0, kv_head, next);
        stage(lds, kKStride, next);
        fetch(p.v, p.v_stride, 0, kv_head, next);
        stage(lds + kKeys * kKStride, kVStride, next);
        __syncthreads();
        for (uint64_t t = 0; t < tiles; ++t) {
            const bool more = t + 1 < tiles;
            float *other = lds + (int)((t + 1) & 1) * kStageFloats;
            if (more) fetch(p.k, p.k_stride, t + 1, kv_head, next);
            const bool active = t < wave_tiles;
            floatx16 s;
            if (active) {
                const float *kt = lds + (int)(t & 1) * kStageFloats;
                // S^T (32 keys x 32 queries): the key row is the lane's column index
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = 0.f;
                const float *krow = kt + column * kKStride + half * kHalf;
#pragma unroll
                for (int step = 0; step < kHalf; step += 4) {
                    const floatx4 piece = *reinterpret_cast<const floatx4 *>(krow + step);
                    s = mfma_32x32x2(piece[0], q[step], s);
                    s = mfma_32x32x2(piece[1], q[step + 1], s);
                    s = mfma_32x32x2(piece[2], q[step + 2], s);
                    s = mfma_32x32x2(piece[3], q[step + 3], s);
                }
            }
            if (more) {
                stage(other, kKStride, next);
                fetch(p.v, p.v_stride, t + 1, kv_head, next);
            }
            if (active) {
                const float *vt = lds + (int)(t & 1) * kStageFloats + kKeys * kKStride;
                // lane holds keys 8 * (i / 4) + 4 * half + i % 4 of the tile for its query
                float peak = -INFINITY;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint64_t key = t * kKeys + (uint64_t)(8 * (i / 4) + 4 * half + i % 4);
                    const bool visible = key < p.kv_tokens && (!p.causal || key <= own);
                    s[i] = visible ? s[i] * p.scale : -INFINITY;
                    peak = fmaxf(peak, s[i]);
                }
                peak = max_xor32(peak);
                const float top_new = fmaxf(top, peak);
                // key 0 is visible to every query, so top_new is finite from the first tile on
                const float keep = fast_exp2((top - top_new) * YVEX_LOG2E);
                sum *= keep;
#pragma unroll
                for (int b = 0; b < kBlocks; ++b)
#pragma unroll
                    for (int i = 0; i < 16; ++i) out[b][i] *= keep;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = fast_exp2((s[i] - top_new) * YVEX_LOG2E);
                    sum += s[i];
                }
                top = top_new;
                // O^T (head dims x queries) += V^T P^T over this lane half's 16 keys
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float *vrow = vt + (8 * (i / 4) + 4 * half + i % 4) * kVStride + column;
#pragma unroll
                    for (int b = 0; b < kBlocks; ++b) out[b] = mfma_32x32x2(vrow[32 * b], s[i], out[b]);
                }
            }
            if (more) stage(other + kKeys * kKStride, kVStride, next);
            __syncthreads();
        }

        // (no early exit above this point: every wave of the workgroup keeps the barriers)
        if (q0 + (uint64_t)column >= p.query_tokens) return;
        sum = sum_xor32(sum);
        if (!(sum > 0.f) || !isfinite(sum) || !isfinite(top)) {
            flag_status(p.status, YVEX_ROCM_DEVICE_NUMERIC);
            return;
        }
        float *row = p.out + (token * p.query_heads + head) * kDim;
        bool bad = false;
#pragma unroll
        for (int b = 0; b < kBlocks; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                floatx4 piece;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    piece[r] = out[b][4 * g + r] / sum;
                    bad |= !isfinite(piece[r]);
                }
                *reinterpret_cast<floatx4 *>(row + 32 * b + 8 * g + 4 * half) = piece;
            }
        if (bad) flag_status(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        if (p.lse && half == 0) p.lse[token * p.query_heads + head] = top + logf(sum);
    }
};

// Head dimension 256.  With 128 query and 128 accumulator registers per lane the form above
// leaves room for one wave per SIMD, and whatever a wave issues between its matrix
// instructions is then not hidden by another.  Here a workgroup has eight waves: waves w and
// w + 4 share 32 queries and split the head dimension in two.  Each computes the part of S^T
// that its 128 dims contribute (64 matrix instructions instead of 128), leaves it in LDS, and
// after a barrier adds the partner's part, lower dims first in both, so both hold the same
// scores and the same statistics; each then accumulates its own 128 dims of O^T (64 matrix
// instructions).  64 query and 64 accumulator registers per lane: two waves per SIMD.
// The exchange area is the V half of the buffer that tile t+1 will use: V(t+1) is fetched
// into registers during tile t and written there at the start of tile t+1, after the barrier
// that ended tile t and before the one that follows the exchange.  LDS as before, 131 KB.
struct GqaTilePair {
    static constexpr int kDim = 256, kPart = kDim / 2, kLane = kPart / 2, kBlocks = kPart / 32;
    static constexpr int kKeys = 32, kQueries = 128, kThreads = 512;
    static constexpr int kKStride = kDim + 4, kVStride = kDim + 8;  // as in GqaTile
    static constexpr int kStageFloats = kKeys * (kKStride + kVStride);
    static constexpr int kChunks = kKeys * (kDim / 4) / kThreads;  // 16-byte pieces of a tile per thread
    static constexpr int kExchangeFloats = 64 * 16;                 // one wave's part of S^T
    static_assert(8 * kExchangeFloats <= kKeys * kVStride, "the exchange fits the V half of a buffer");

    const yvex_rocm_gqa_f32_params &p;
    float *lds;
    const int tid, lane, wave, column, half, quarter, part;

    __device__ GqaTilePair(const yvex_rocm_gqa_f32_params &params, float *shared)
        : p(params), lds(shared), tid(threadIdx.x), lane(threadIdx.x & 63), wave(threadIdx.x >> 6),
          column(threadIdx.x & 31), half((threadIdx.x >> 5) & 1), quarter((threadIdx.x >> 6) & 3),
          part(threadIdx.x >> 8)
    {
    }

    struct Staged {
        floatx4 piece[kChunks];
    };

    __device__ void fetch(const float *rows, uint64_t stride, uint64_t tile, uint64_t kv_head, Staged &s) const
    {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int c = tid + kThreads * j, row = c / (kDim / 4), piece = c % (kDim / 4);
            const uint64_t key = tile * kKeys + (uint64_t)row;
            const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
            s.piece[j] = zero;
            if (key < p.kv_tokens)
                s.piece[j] = *reinterpret_cast<const floatx4 *>(rows + key * stride + kv_head * kDim + 4 * piece);
        }
    }

    __device__ void stage(float *tile, int row_stride, const Staged &s) const
    {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int c = tid + kThreads * j, row = c / (kDim / 4), piece = c % (kDim / 4);
            *reinterpret_cast<floatx4 *>(tile + row * row_stride + 4 * piece) = s.piece[j];
        }
    }

    // item lists as in GqaTile::run
    __device__ void run() const
    {
        uint32_t count = 1u;
        u32x4 row = {0u, 0u, 0u, 0u};
        if (p.lists != nullptr) {
            typedef __attribute__((address_space(4))) const u32x4 constant_u32x4;
            row = *(constant_u32x4 *)(uintptr_t)(p.lists + (uint64_t)blockIdx.x * 8u);
            count = min(row.x & 0xffffu, 7u);
        }
        for (uint32_t j = 1u; j <= count; ++j) {
            const uint32_t word = j >> 1 == 0u ? row.x : j >> 1 == 1u ? row.y : j >> 1 == 2u ? row.z : row.w;
            item(p.lists != nullptr ? (word >> ((j & 1u) * 16u)) & 0xffffu : blockIdx.x);
            if (j < count) __syncthreads();
        }
    }

    __device__ void item(const uint64_t id) const
    {
        const uint64_t tiles_q = (p.query_tokens + kQueries - 1) / kQueries;
        const uint64_t head = id % p.query_heads;
        const uint64_t q_tile = tiles_q - 1 - id / p.query_heads;
        const uint64_t kv_head = head / (p.query_heads / p.kv_heads);
        const uint64_t q0 = q_tile * kQueries + (uint64_t)quarter * 32u;
        const uint64_t token = min(q0 + (uint64_t)column, p.query_tokens - 1);
        const uint64_t own = p.query_start + token;
        const uint64_t group_last = p.causal
            ? min(p.kv_tokens, p.query_start + min((q_tile + 1) * kQueries, p.query_tokens))
            : p.kv_tokens;
        const uint64_t wave_last = p.causal
            ? min(p.kv_tokens, p.query_start + min(q0 + 32u, p.query_tokens))
            : p.kv_tokens;
        const uint64_t tiles = (group_last + kKeys - 1) / kKeys;
        const uint64_t wave_tiles = q0 < p.query_tokens ? (wave_last + kKeys - 1) / kKeys : 0;
        const int dim0 = part * kPart;  // first head dim of this wave's half

        // this lane's share of its query row: Q[token][dim0 + half * kLane + s], s = 0 .. kLane-1
        float q[kLane];
        {
            const float *row = p.q + token * p.q_stride + head * kDim + dim0 + half * kLane;
#pragma unroll
            for (int s = 0; s < kLane; s += 4) {
                const floatx4 piece = *reinterpret_cast<const floatx4 *>(row + s);
                q[s] = piece[0];
                q[s + 1] = piece[1];
                q[s + 2] = piece[2];
                q[s + 3] = piece[3];
            }
        }

        floatx16 out[kBlocks];
#pragma unroll
        for (int b = 0; b < kBlocks; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) out[b][i] = 0.f;
        float top = -INFINITY, sum = 0.f;

        Staged next;
        fetch(p.k, p.k_stride, 0, kv_head, next);
        stage(lds, kKStride, next);
        fetch(p.v, p.v_stride, 0, kv_head, next);  // written at the head of the first trip
        for (uint64_t t = 0; t < tiles; ++t) {
            const bool more = t + 1 < tiles;
            float *here = lds + (int)(t & 1) * kStageFloats;
            float *other = lds + (int)((t + 1) & 1) * kStageFloats;
            float *exchange = other + kKeys * kKStride;
            // V(t) into its place: the area held the parts of S^T of tile t-1, read before the
            // barrier that ended it
            stage(here + kKeys * kKStride, kVStride, next);
            if (t == 0) __syncthreads();  // K(0), written by every thread of the workgroup
            if (more) fetch(p.k, p.k_stride, t + 1, kv_head, next);
            const bool active = t < wave_tiles;  // the two waves of a pair alike
            floatx16 s;
            if (active) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = 0.f;
                const float *krow = here + column * kKStride + dim0 + half * kLane;
#pragma unroll
                for (int step = 0; step < kLane; step += 4) {
                    const floatx4 piece = *reinterpret_cast<const floatx4 *>(krow + step);
                    s = mfma_32x32x2(piece[0], q[step], s);
                    s = mfma_32x32x2(piece[1], q[step + 1], s);
                    s = mfma_32x32x2(piece[2], q[step + 2], s);
                    s = mfma_32x32x2(piece[3], q[step + 3], s);
                }
                // 16 bytes per lane and store, lanes side by side: no bank is met twice
                float *mine = exchange + wave * kExchangeFloats + lane * 4;
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    *reinterpret_cast<floatx4 *>(mine + g * 256) =
                        (floatx4){s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
            }
            __syncthreads();  // the parts of S^T, and V(t)
            if (active) {
                const float *theirs = exchange + (wave ^ 4) * kExchangeFloats + lane * 4;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const floatx4 piece = *reinterpret_cast<const floatx4 *>(theirs + g * 256);
#pragma unroll
                    for (int r = 0; r < 4; ++r)  // lower dims + upper dims, in both waves
                        s[4 * g + r] = part == 0 ? s[4 * g + r] + piece[r] : piece[r] + s[4 * g + r];
                }
            }
            if (more) {
                stage(other, kKStride, next);
                fetch(p.v, p.v_stride, t + 1, kv_head, next);
            }
            if (active) {
                const float *vt = here + kKeys * kKStride + dim0;
                float peak = -INFINITY;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint64_t key = t * kKeys + (uint64_t)(8 * (i / 4) + 4 * half + i % 4);
                    const bool visible = key < p.kv_tokens && (!p.causal || key <= own);
                    s[i] = visible ? s[i] * p.scale : -INFINITY;
                    peak = fmaxf(peak, s[i]);
                }
                peak = max_xor32(peak);
                const float top_new = fmaxf(top, peak);
                const float keep = fast_exp2((top - top_new) * YVEX_LOG2E);
                sum *= keep;
#pragma unroll
                for (int b = 0; b < kBlocks; ++b)
#pragma unroll
                    for (int i = 0; i < 16; ++i) out[b][i] *= keep;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = fast_exp2((s[i] - top_new) * YVEX_LOG2E);
                    sum += s[i];
                }
                top = top_new;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float *vrow = vt + (8 * (i / 4) + 4 * half + i % 4) * kVStride + column;
#pragma unroll
                    for (int b = 0; b < kBlocks; ++b) out[b] = mfma_32x32x2(vrow[32 * b], s[i], out[b]);
                }
            }
            __syncthreads();  // every wave is done with tile t and with the exchange
        }

        if (q0 + (uint64_t)column >= p.query_tokens) return;
        sum = sum_xor32(sum);
        if (!(sum > 0.f) || !isfinite(sum) || !isfinite(top)) {
            flag_status(p.status, YVEX_ROCM_DEVICE_NUMERIC);
            return;
        }
        float *row = p.out + (token * p.query_heads + head) * kDim + dim0;
        bool bad = false;
#pragma unroll
        for (int b = 0; b < kBlocks; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                floatx4 piece;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    piece[r] = out[b][4 * g + r] / sum;
                    bad |= !isfinite(piece[r]);
                }
                *reinterpret_cast<floatx4 *>(row + 32 * b + 8 * g + 4 * half) = piece;
            }
        if (bad) flag_status(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        if (p.lse && half == 0 && part == 0) p.lse[token * p.query_heads + head] = top + logf(sum);
    }
};

}  // namespace

// `waves`: waves per SIMD the register budget is sized for.
#define YVEX_GQA_F32_TILE_KERNEL(name, blocks, waves)                                                   \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(waves, waves))) \
    name(const yvex_rocm_gqa_f32_params p)                                                                \
    {                                                                                                     \
        __shared__ __attribute__((aligned(16))) float lds[2 * GqaTile<blocks>::kStageFloats];             \
        GqaTile<blocks>(p, lds).run();                                                                    \
    }

YVEX_GQA_F32_TILE_KERNEL(yvex_rocm_gqa_f32_tile_64, 2, 2)
YVEX_GQA_F32_TILE_KERNEL(yvex_rocm_gqa_f32_tile_128, 4, 2)

// head dimension 256: pairs of waves, see GqaTilePair
extern "C" __global__ void __launch_bounds__(GqaTilePair::kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
yvex_rocm_gqa_f32_tile_256(const yvex_rocm_gqa_f32_params p)
{
    __shared__ __attribute__((aligned(16))) float lds[2 * GqaTilePair::kStageFloats];
    GqaTilePair(p, lds).run();
}
