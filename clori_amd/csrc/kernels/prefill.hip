// Causal / full grouped-query attention prefill for gfx950 (wave64), bf16 in and out,
// fp32 scores, online softmax and accumulation.  head_dim 128, token-major tensors
// ([token][head][dim], per-token strides in elements).
//
// A workgroup of 4 waves owns one (query head, 128-row query tile): each wave owns
// 32 query rows and walks the key/value tokens in tiles of 64 that the workgroup
// stages in LDS once and all four waves share.  Two workgroups are resident per CU, so
// the softmax VALU work of one overlaps the MFMAs of the other.  Both products are computed transposed
// so the probabilities never leave registers:
//     S^T[key][query] = K[key][:] . Q[query][:]        v_mfma_f32_32x32x16_bf16, A = K (LDS)
//     O^T[dim][query] += V^T[dim][key] . P^T[key][query]                A = V^T (LDS)
// The accumulator layout of S^T (lane = query row, 16 key rows per lane) is the B-operand
// layout of the second product once the 16-key K-slices are taken as accumulator
// registers 8u..8u+7; V^T is fetched from LDS in the matching key order.  Softmax
// statistics are per lane (= per query row) plus one exchange with lane^32.
//
// LDS layout: K and V tiles are both [64 keys][128 dims] bf16 in row-major order with
// 256-byte rows and no padding; the 16-byte chunk c of row r sits at chunk position
// c ^ x(r), x(r) = ((r & 3) << 2) | ((r >> 2) & 3).  That makes both operand fetches
// bank-conflict free: the K operand is one ds_read_b128 per lane (16 rows x one chunk
// column hit 16 distinct chunk positions), the V^T operand is two ds_read_b64_tr_b16
// (each 16-lane group transposes 4 keys x 16 dims; 4 consecutive rows place one 64-byte
// column segment in 4 distinct bank groups).
// The tiles are filled by buffer loads that write LDS directly (no staging registers,
// no LDS store instructions): lane L of a 1 KB load owns chunk position L % 16 of row
// L / 16 and fetches the global chunk that belongs there.  Rows past the end of the
// tensor read as zero through the buffer range check.  Two buffers; the loads of tile
// t+1 are issued one by one behind the first MFMAs of tile t (issuing one costs the wave
// about 50 cycles), one barrier per tile.
//
// The running maximum is only raised when a tile exceeds it by more than kLazyLog2 (in
// log2 units), so the accumulator rescale is rare; probabilities are then at most
// 2^kLazyLog2, harmless in fp32 sums and in the bf16 operand of the second product.
// Workgroups are numbered so that heavier (later) query tiles start first and, when the
// kv head count is a multiple of the 8 XCDs, all users of one kv head share an L2.
#include "mfma.h"

#include "../kernel_params.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kKeyTile = 64;
constexpr int kRowBytes = kHeadDim * 2;            // 256
constexpr int kTileBytes = kKeyTile * kRowBytes;   // 16384 per K or V tile
constexpr int kBufBytes = 2 * kTileBytes;          // K then V
constexpr int kThreads = 256;
constexpr float kLazyLog2 = 8.0f;

typedef __attribute__((address_space(3))) short4v lds_short4;

// chunk swizzle of tile row r
__device__ inline int swizzle(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

template <int NB>
__device__ inline void prefill_body(const yvex_rocm_prefill_params &p, unsigned char *lds)
{
    constexpr int kRowsPerWave = 32 * NB;
    constexpr int kRowsPerBlock = 4 * kRowsPerWave;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, g = lane >> 5;
    // heavier (later) query tiles are dispatched first; id % kv_heads picks the kv head
    const uint32_t q_tiles = (p.query_tokens + kRowsPerBlock - 1) / kRowsPerBlock;
    const uint32_t q_tile = q_tiles - 1u - blockIdx.x / p.query_heads;
    const uint32_t in_tile = blockIdx.x % p.query_heads;
    const uint32_t kv_head = in_tile % p.kv_heads;
    const uint32_t head = kv_head * (p.query_heads / p.kv_heads) + in_tile / p.kv_heads;
    const uint32_t row0 = q_tile * kRowsPerBlock + wave * kRowsPerWave;  // first row of this wave

    // keys visible to the last row of the workgroup bound the walk
    const uint32_t block_last_row = min(p.query_tokens, (q_tile + 1u) * kRowsPerBlock) - 1u;
    const uint32_t kv_end = p.causal ? min(p.kv_tokens, p.query_start + block_last_row + 1u)
                                     : p.kv_tokens;
    const uint32_t tiles = (kv_end + kKeyTile - 1) / kKeyTile;

    // ---- Q fragments: B operand, lane (n, g) holds Q[row n][16*kk + 8g .. +7] ----
    bf16x8 q[NB][8];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const uint32_t row = min(row0 + nb * 32 + n, p.query_tokens - 1u);
        const uint16_t *src = p.q + (uint64_t)row * p.q_stride + (uint64_t)head * kHeadDim + g * 8;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) q[nb][kk] = as_bf16x8(load_b128(src + kk * 16));
    }

    // ---- tile staging: buffer loads that write LDS directly -----------------------
    // 1 KB load j of wave w fills rows 16w + 4j .. +3 of the tile; lane L owns chunk
    // position L % 16 of row 16w + 4j + L / 16 and fetches chunk (L % 16) ^ x(row).
    const uint32_t k_row_bytes = (uint32_t)p.k_stride * 2u, v_row_bytes = (uint32_t)p.v_stride * 2u;
    const i32x4 k_rsrc = raw_buffer(p.k + (uint64_t)kv_head * kHeadDim,
                                    p.kv_tokens * k_row_bytes - kv_head * kRowBytes);
    const i32x4 v_rsrc = raw_buffer(p.v + (uint64_t)kv_head * kHeadDim,
                                    p.kv_tokens * v_row_bytes - kv_head * kRowBytes);
    const uint32_t lds_base = lds_address_of(lds);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    uint32_t k_off[4], v_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = 16 * wave + 4 * j + (lane >> 4);
        const uint32_t chunk = (uint32_t)((lane & 15) ^ swizzle(r));
        k_off[j] = (uint32_t)r * k_row_bytes + chunk * 16u;
        v_off[j] = (uint32_t)r * v_row_bytes + chunk * 16u;
    }
    // load j (0..7) of a tile: 0..3 fill this wave's K rows, 4..7 its V rows
    auto stage_one = [&](uint32_t tile, int buf, int j) {
        const uint32_t dst = lds_base + buf * kBufBytes + wave_u * 4096;
        if (j < 4)
            lds_dma_b128(dst + j * 1024, k_rsrc, k_off[j], tile * kKeyTile * k_row_bytes);
        else
            lds_dma_b128(dst + kTileBytes + (j - 4) * 1024, v_rsrc, v_off[j - 4],
                         tile * kKeyTile * v_row_bytes);
    };
    auto stage_tile = [&](uint32_t tile, int buf) {
#pragma unroll
        for (int j = 0; j < 8; ++j) stage_one(tile, buf, j);
    };

    // ---- operand addresses inside a tile ------------------------------------------
    // K operand (mb, kk): row mb*32 + n, chunk (2kk + g) ^ x(n); one address per kk
    uint32_t k_addr[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk)
        k_addr[kk] = (uint32_t)(n * kRowBytes + (((2 * kk + g) ^ swizzle(n)) << 4));
    // V^T operand (db, mb, u, h): 16-lane group b = lane / 16 (dims 16 * (b & 1), key half
    // g = b / 2), lane a = lane % 16 addresses key row mb*32 + 16u + 8h + 4g + a/4 and
    // dims db*32 + 16*(b&1) + 4*(a%4) .. +3; one address per (db, h)
    uint32_t v_addr[4][2];
    {
        const int a = lane & 15, b1 = (lane >> 4) & 1;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int r = 8 * h + 4 * g + (a >> 2);
                const int chunk = (db * 4 + 2 * b1 + ((a >> 1) & 1)) ^ swizzle(r);
                v_addr[db][h] = (uint32_t)(kTileBytes + r * kRowBytes + (chunk << 4) + 8 * (a & 1));
            }
    }

    floatx16 o[4][NB];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[db][nb][i] = 0.f;
    float m_run[NB], l_run[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        m_run[nb] = -INFINITY;
        l_run[nb] = 0.f;
    }

    // rows of this wave at or past query_tokens do no work but still help staging
    const bool wave_active = row0 < p.query_tokens;
    // last key visible to the wave's first / last row (causal)
    const uint32_t wave_first_vis = p.causal ? p.query_start + row0 : p.kv_tokens - 1u;
    const uint32_t wave_last_vis =
        p.causal ? p.query_start + min(row0 + kRowsPerWave, p.query_tokens) - 1u : p.kv_tokens - 1u;

    stage_tile(0u, 0);
    for (uint32_t t = 0; t < tiles; ++t) {
        const int buf = (int)(t & 1u);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of tile t is in LDS
        __syncthreads();
        const uint32_t key0 = t * kKeyTile;
        const bool more = t + 1u < tiles;
        // a wave whose every row sees nothing of this tile skips the products
        if (!wave_active || key0 > wave_last_vis) {
            if (more) stage_tile(t + 1u, buf ^ 1);
            continue;
        }
        const unsigned char *tile = lds + buf * kBufBytes;

        // ---- S^T = K . Q^T -------------------------------------------------
        floatx16 s[2][NB];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[mb][nb][i] = 0.f;
        {
            // operand fetches run kDepth steps ahead of the MFMAs, the eight loads of the
            // next tile ride behind the first eight steps; the order is pinned
            constexpr int kDepth = 4;
            auto fetch = [&](int i) {  // i = kk * 2 + mb
                return *reinterpret_cast<const u32x4 *>(tile + k_addr[i >> 1] +
                                                        (i & 1) * 32 * kRowBytes);
            };
            u32x4 frag[kDepth];
#pragma unroll
            for (int i = 0; i < kDepth; ++i) frag[i] = fetch(i);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const bf16x8 a = as_bf16x8(frag[i % kDepth]);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    s[i & 1][nb] = mfma_32x32x16(a, q[nb][i >> 1], s[i & 1][nb]);
                if (i + kDepth < 16) frag[i % kDepth] = fetch(i + kDepth);
                if (i < 8 && more) stage_one(t + 1u, buf ^ 1, i);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- mask, online softmax (per lane = per query row) ----------------------
        // scores stay raw; the softmax scale is folded into the exponent's multiply-add
        const bool need_mask = (key0 + kKeyTile - 1u > wave_first_vis) ||
                               (key0 + kKeyTile > p.kv_tokens);
        uint32_t pk[2][NB][8];  // bf16 pairs: [mb][nb][u*4 + pair]
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            if (need_mask) {
                const uint32_t row = row0 + nb * 32 + n;
                const uint32_t vis = p.causal ? min(p.query_start + row, p.kv_tokens - 1u)
                                              : p.kv_tokens - 1u;
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const uint32_t key = key0 + mb * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
                        if (key > vis) s[mb][nb][i] = -INFINITY;
                    }
            }
            float mloc = -INFINITY;
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[mb][nb][i]);
            mloc = fmaxf(mloc, xor_lanes(mloc, 32)) * p.scale_log2;
            if (__builtin_amdgcn_ballot_w64(mloc > m_run[nb] + kLazyLog2) != 0ull) {
                const float m_new = fmaxf(m_run[nb], mloc);
                // a row that has seen nothing yet keeps m = -inf: guard the subtraction
                const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2(m_run[nb] - m_new);
                l_run[nb] *= alpha;
#pragma unroll
                for (int db = 0; db < 4; ++db) o[db][nb] *= alpha;
                m_run[nb] = m_new;
            }
            const float neg_m = m_run[nb] == -INFINITY ? 0.f : -m_run[nb];
            float lsum = 0.f;
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int i = 0; i < 16; i += 2) {
                    const float p0 = fast_exp2(__builtin_fmaf(s[mb][nb][i], p.scale_log2, neg_m));
                    const float p1 =
                        fast_exp2(__builtin_fmaf(s[mb][nb][i + 1], p.scale_log2, neg_m));
                    lsum += p0 + p1;
                    pk[mb][nb][i >> 1] = pack_bf16x2(p0, p1);
                }
            l_run[nb] += lsum;
        }

        // ---- O^T += V^T . P^T -------------------------------------------------
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                bf16x8 pb[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    u32x4 w = {pk[mb][nb][u * 4 + 0], pk[mb][nb][u * 4 + 1], pk[mb][nb][u * 4 + 2],
                               pk[mb][nb][u * 4 + 3]};
                    pb[nb] = as_bf16x8(w);
                }
#pragma unroll
                for (int db = 0; db < 4; ++db) {
                    const int base = (mb * 32 + u * 16) * kRowBytes;
                    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (lds_short4 *)(tile + v_addr[db][0] + base));
                    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (lds_short4 *)(tile + v_addr[db][1] + base));
                    typedef short short8v __attribute__((ext_vector_type(8)));
                    const short8v av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    const bf16x8 a = __builtin_bit_cast(bf16x8, av);
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) o[db][nb] = mfma_32x32x16(a, pb[nb], o[db][nb]);
                }
            }
    }

    // ---- epilogue: normalise, publish bf16 rows and LSE -------------------------
    if (!wave_active) return;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const uint32_t row = row0 + nb * 32 + n;
        float l = l_run[nb];
        l += xor_lanes(l, 32);
        const bool live = row < p.query_tokens;
        const float inv = 1.0f / l;
        bool bad = false;
        uint16_t *dst = p.out + ((uint64_t)row * p.query_heads + head) * kHeadDim;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                const float a0 = o[db][nb][grp * 4 + 0] * inv, a1 = o[db][nb][grp * 4 + 1] * inv;
                const float a2 = o[db][nb][grp * 4 + 2] * inv, a3 = o[db][nb][grp * 4 + 3] * inv;
                bad |= !(isfinite(a0) && isfinite(a1) && isfinite(a2) && isfinite(a3));
                u32x2 w;
                w.x = pack_bf16x2(a0, a1);
                w.y = pack_bf16x2(a2, a3);
                if (p.gate && live) {
                    w = gate_four(w, p.gate + (dst - p.out) + db * 32 + grp * 8 + g * 4);
                    bad |= pair_not_finite(w.x) || pair_not_finite(w.y);
                }
                if (live) *reinterpret_cast<u32x2 *>(dst + db * 32 + grp * 8 + g * 4) = w;
            }
        if (live && bad) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        if (live && p.lse && g == 0)
            p.lse[(uint64_t)row * p.query_heads + head] = (m_run[nb] + fast_log2(l)) * YVEX_LN2;
    }
}

}  // namespace

// grid = query heads x query tiles of YVEX_ROCM_PREFILL_ROWS rows, block 256,
// LDS 2 x (K + V^T) tiles; two workgroups per CU.
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
yvex_rocm_prefill_bf16(const yvex_rocm_prefill_params p)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufBytes];
    prefill_body<YVEX_ROCM_PREFILL_ROWS / 128>(p, lds);
}
