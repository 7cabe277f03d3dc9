// Exact F32 attention kernels for gfx950 (wave64).
//
// These serve the reference's only numeric contract, EXACT_F32: F32 tensors in, F32
// out, no reduced-precision products.  They follow the CPU operator's arithmetic
// (src/backend/cpu.c:307-399 of the reference): double-precision dot products,
// softmax statistics and PV accumulation, the score stored as float and re-read.
// They are the correctness path for the reference's own test vectors; the bf16 MFMA
// kernels are the throughput path and are never substituted for these.
#include <hip/hip_runtime.h>

#include "device_scope.h"

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

__device__ inline float wave_max_f32(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Sum of a double over the 16 lanes of a DPP row, left in all 16: lane exchanges on the vector
// ALU (quad permutes, then the half-row and row mirrors), no trip through the LDS permute
// network.  The order of the additions differs from lane to lane only by commutation, so all
// 16 lanes hold the same bits.
template <int kControl>
__device__ inline double dpp_exchange(double v)
{
    const uint64_t bits = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)bits, kControl, 0xf, 0xf, true);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(bits >> 32), kControl, 0xf, 0xf, true);
    return __builtin_bit_cast(double, (uint64_t)lo | ((uint64_t)hi << 32));
}

__device__ inline double row_sum(double v)
{
    v += dpp_exchange<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_exchange<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_exchange<0x141>(v);  // row_half_mirror: the other quad of the half row
    v += dpp_exchange<0x140>(v);  // row_mirror: the other half of the row
    return v;
}

// Decode-shaped EXACT_F32 requests over long contexts: the same arithmetic as
// yvex_rocm_gqa_f32 (double dot products, the score rounded to float, double exponentials,
// denominator and accumulators), but the keys a query sees are cut into `splits` runs, one wave
// per (query token, query head, run).  A workgroup is a team of kSplitTeam waves on consecutive
// runs: they merge through LDS in wave order, the team leaves one partial (write-through
// stores), counts itself in on the arrival counter of its (token, head), and the team that
// completes the count merges the teams' partials in team order and publishes.  One launch;
// the result does not depend on who was last.
// Inside a run a wave takes 64 keys at a time, four keys per step: the 16 lanes of a group
// hold 8 head dims each (kPieces = 2 such pieces above 128 dims), so a key or value row is one
// contiguous read of the group.  The dot product is reduced over the group, lane `piece` of
// the group keeps the score of the group's key of step `piece` (all 64 keys of the tile, one
// per lane, for the statistics), and the value sum runs over the same steps with the weight
// fetched from that lane; the four groups' sums are added once at the end.
// The rows of several steps are fetched before the first is used, with no branch in between:
// a key past the run reads the run's last key (its score is masked, its weight is zero), a
// lane past the head dimension reads the row's last 8 dims against a zero query and its
// sums are never stored.
// grid = (query_tokens * query_heads, ceil(splits / kSplitTeam)), block 64 * kSplitTeam;
// head_dim % 8 == 0, <= 128 * kPieces; LDS: kSplitTeam rows of 256 doubles, then (max, sum) pairs.
constexpr int kSplitTeam = 8;

// 8 bytes to and from global memory at device scope: write-through stores that are visible to
// the other XCDs once they have completed, loads that see them without an L2 invalidate.
__device__ inline void store_f64_device(double *p, double v)
{
    __hip_atomic_store(reinterpret_cast<uint64_t *>(p), __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline double load_f64_device(const double *p)
{
    return __builtin_bit_cast(double, __hip_atomic_load(reinterpret_cast<const uint64_t *>(p), __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT));
}

// Which (token, head) workgroup `unit` of a launch row works on.  Consecutive workgroup ids go
// to consecutive XCDs, each with its own L2; when the head count is a multiple of eight the
// heads are dealt so that an XCD gets a contiguous eighth of them, i.e. the query heads that
// share a KV head read its rows through one L2 (dealt in order, the four heads of a group sat
// on four XCDs and the history was fetched from memory four times).
__device__ __forceinline__ void split_unit(const yvex_rocm_gqa_f32_params &p, uint64_t unit, uint64_t &token,
                                           uint64_t &head)
{
    token = unit / p.query_heads;
    head = unit % p.query_heads;
    if ((p.query_heads & 7u) == 0u) head = (head & 7u) * (p.query_heads >> 3) + (head >> 3);
}

// The partials of a unit's teams (maximum, sum and one value per thread), merged in team order:
// what the last team of a unit to arrive does.  Eight teams per trip of independent loads.
__device__ __forceinline__ void merge_team_partials(const yvex_rocm_gqa_f32_params &p, uint64_t unit,
                                                    uint32_t teams, uint32_t t, uint64_t d, double &top,
                                                    double &total, double &o)
{
    top = -INFINITY;
    total = 0.0;
    o = 0.0;
    // eight teams per trip of independent loads (teams past the end alias the last one
    // with weight zero)
    for (uint32_t t0 = 0u; t0 < teams; t0 += 8u) {
        double mt[8], lt[8], vt[8];
#pragma unroll
        for (uint32_t i = 0u; i < 8u; ++i) {
            const uint64_t from = unit * teams + min(t0 + i, teams - 1u);
            mt[i] = load_f64_device(p.part_ml + from * 2u);
            lt[i] = load_f64_device(p.part_ml + from * 2u + 1u);
            vt[i] = t < d ? load_f64_device(p.part_acc + from * d + t) : 0.0;
        }
        double trip = -INFINITY;
#pragma unroll
        for (uint32_t i = 0u; i < 8u; ++i) {
            if (t0 + i >= teams) mt[i] = -INFINITY;
            trip = fmax(trip, mt[i]);
        }
        const double top_new = fmax(top, trip);
        const double keep = top == -INFINITY ? 0.0 : exp(top - top_new);
        total *= keep;
        o *= keep;
#pragma unroll
        for (uint32_t i = 0u; i < 8u; ++i) {
            const double weight = mt[i] == -INFINITY ? 0.0 : exp(mt[i] - top_new);
            total += weight * lt[i];
            o += weight * vt[i];
        }
        top = top_new;
    }
}

template <int kPieces>
__device__ __forceinline__ void gqa_f32_split(const yvex_rocm_gqa_f32_params &p, double *team_lds)
{
    typedef float floatx4 __attribute__((ext_vector_type(4)));
    constexpr int kBatch = 8 / kPieces;  // steps whose rows are in flight together
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int group = lane >> 4, piece = lane & 15;
    // a run past `splits` (the last team's padding) starts past the visible keys: it has none
    const uint64_t unit = blockIdx.x, split = (uint64_t)blockIdx.y * kSplitTeam + (uint64_t)wave;
    uint64_t token, head;
    split_unit(p, unit, token, head);
    const uint64_t kv_head = head / (p.query_heads / p.kv_heads);
    const uint64_t visible = p.causal ? min(p.kv_tokens, p.query_start + token + 1) : p.kv_tokens;
    const uint64_t d = p.head_dim;
    const uint64_t k0 = split * p.keys_per_split, k1 = min(visible, k0 + (uint64_t)p.keys_per_split);
    uint64_t dim[kPieces];   // first of this lane's 8 dims in piece j, clamped into the row
    bool live[kPieces];
#pragma unroll
    for (int j = 0; j < kPieces; ++j) {
        const uint64_t want = (uint64_t)piece * 8u + 128u * (uint64_t)j;
        live[j] = want < d;
        dim[j] = live[j] ? want : d - 8u;
    }

    double q[kPieces][8];
    {
        const float *row = p.q + token * p.q_stride + head * d;
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            const floatx4 a = *reinterpret_cast<const floatx4 *>(row + dim[j]);
            const floatx4 b = *reinterpret_cast<const floatx4 *>(row + dim[j] + 4u);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                q[j][e] = live[j] ? (double)a[e] : 0.0;
                q[j][4 + e] = live[j] ? (double)b[e] : 0.0;
            }
        }
    }
    double acc[kPieces][8];
#pragma unroll
    for (int j = 0; j < kPieces; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] = 0.0;
    double m = -INFINITY, l = 0.0;
    if (k0 < k1) {
        const float *kbase = p.k + kv_head * d, *vbase = p.v + kv_head * d;
        for (uint64_t tile = k0; tile < k1; tile += 64u) {
            // scores: step `it` handles keys tile + 4 * it + group
            float mine = -INFINITY;
#pragma unroll
            for (int it0 = 0; it0 < 16; it0 += kBatch) {
                floatx4 ra[kBatch][kPieces], rb[kBatch][kPieces];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const uint64_t key = min(tile + (uint64_t)(4 * (it0 + u) + group), k1 - 1u);
#pragma unroll
                    for (int j = 0; j < kPieces; ++j) {
                        const float *at = kbase + key * p.k_stride + dim[j];
                        ra[u][j] = *reinterpret_cast<const floatx4 *>(at);
                        rb[u][j] = *reinterpret_cast<const floatx4 *>(at + 4u);
                    }
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    double part = 0.0;
#pragma unroll
                    for (int j = 0; j < kPieces; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            part += q[j][e] * (double)ra[u][j][e];
                            part += q[j][4 + e] * (double)rb[u][j][e];
                        }
                    part = row_sum(part);
                    const bool seen = tile + (uint64_t)(4 * (it0 + u) + group) < k1;
                    const float s = seen ? (float)(part * (double)p.scale) : -INFINITY;
                    if (piece == it0 + u) mine = s;
                }
            }
            // lane (group, piece) now holds the score of key tile + 4 * piece + group
            const double m_new = fmax(m, (double)wave_max_f32(mine));
            const double alpha = exp(m - m_new);
            const double w = mine == -INFINITY ? 0.0 : exp((double)mine - m_new);
            l = l * alpha + wave_sum(w);
#pragma unroll
            for (int j = 0; j < kPieces; ++j)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[j][e] *= alpha;
            m = m_new;
#pragma unroll
            for (int it0 = 0; it0 < 16; it0 += kBatch) {
                floatx4 ra[kBatch][kPieces], rb[kBatch][kPieces];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const uint64_t key = min(tile + (uint64_t)(4 * (it0 + u) + group), k1 - 1u);
#pragma unroll
                    for (int j = 0; j < kPieces; ++j) {
                        const float *at = vbase + key * p.v_stride + dim[j];
                        ra[u][j] = *reinterpret_cast<const floatx4 *>(at);
                        rb[u][j] = *reinterpret_cast<const floatx4 *>(at + 4u);
                    }
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const double wi = __shfl(w, (lane & 48) + it0 + u, kWave);  // 0 past the run
#pragma unroll
                    for (int j = 0; j < kPieces; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            acc[j][e] += wi * (double)ra[u][j][e];
                            acc[j][4 + e] += wi * (double)rb[u][j][e];
                        }
                }
            }
        }
    }
    // the four key groups hold partial sums of the same dims
#pragma unroll
    for (int j = 0; j < kPieces; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[j][e] += __shfl_xor(acc[j][e], 16, kWave);
            acc[j][e] += __shfl_xor(acc[j][e], 32, kWave);
        }
    // ---- the team: the waves' parts through LDS, merged in wave order ---------------------
    double *rows = team_lds, *stats = team_lds + kSplitTeam * 256;
    if (group == 0) {
#pragma unroll
        for (int j = 0; j < kPieces; ++j)
            if (live[j])
#pragma unroll
                for (int e = 0; e < 8; ++e) rows[wave * 256 + (int)dim[j] + e] = acc[j][e];
    }
    if (lane == 0) {
        stats[wave * 2] = m;  // -inf for a run without visible keys
        stats[wave * 2 + 1] = l;
    }
    __syncthreads();
    const uint32_t t = threadIdx.x, teams = gridDim.y, team = blockIdx.y;
    double top = -INFINITY, total = 0.0, o = 0.0;
#pragma unroll
    for (int w = 0; w < kSplitTeam; ++w) top = fmax(top, stats[w * 2]);
#pragma unroll
    for (int w = 0; w < kSplitTeam; ++w) {
        const double mw = stats[w * 2];
        const double weight = mw == -INFINITY ? 0.0 : exp(mw - top);
        total += weight * stats[w * 2 + 1];
        if (t < d) o += weight * rows[w * 256 + (int)t];
    }
    if (teams > 1u) {
        // ---- the teams: one partial each, merged in team order by the last to arrive --------
        const uint64_t slot = unit * teams + team;
        if (t < d) store_f64_device(p.part_acc + slot * d + t, o);
        if (t == 0u) {
            store_f64_device(p.part_ml + slot * 2u, top);
            store_f64_device(p.part_ml + slot * 2u + 1u, total);
        }
        stores_completed();  // this thread's stores have completed, and nothing moves across
        __syncthreads();
        uint32_t *last = reinterpret_cast<uint32_t *>(team_lds);  // the LDS parts are done with
        if (t == 0u) {
            const uint32_t before =
                __hip_atomic_fetch_add(p.arrivals + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before == teams - 1u)
                __hip_atomic_store(p.arrivals + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *last = before == teams - 1u ? 1u : 0u;
        }
        __syncthreads();
        if (*last == 0u) return;
        loads_ordered();
        merge_team_partials(p, unit, teams, t, d, top, total, o);
    }
    if (!(total > 0.0) || !isfinite(total) || !isfinite(top)) {
        if (t == 0u) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        return;
    }
    if (t < d) {
        const float value = (float)(o / total);
        if (!isfinite(value)) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        p.out[(token * p.query_heads + head) * d + t] = value;
    }
    if (p.lse && t == 0u) p.lse[token * p.query_heads + head] = (float)(top + log(total));
}

extern "C" __global__ void __launch_bounds__(64 * kSplitTeam)
yvex_rocm_gqa_f32_split(const yvex_rocm_gqa_f32_params p)
{
    __shared__ double team_lds[kSplitTeam * 256 + kSplitTeam * 2];
    gqa_f32_split<1>(p, team_lds);
}

extern "C" __global__ void __launch_bounds__(64 * kSplitTeam)
yvex_rocm_gqa_f32_split_wide(const yvex_rocm_gqa_f32_params p)
{
    __shared__ double team_lds[kSplitTeam * 256 + kSplitTeam * 2];
    gqa_f32_split<2>(p, team_lds);
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
        // read once, as the page blocks are
        for (int j = 0; j < 8; ++j) v[j] = __builtin_nontemporal_load(base + j * 64);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc ^= v[j];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == p.never) p.sink[0] = 1u;
}
