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
// LDS layout (chosen so every MFMA operand fetch is bank-conflict free on 64 banks):
//     K tile    [64 keys][128 dims] bf16, row pitch 272 B   ds_read_b128 per A operand
//     V^T tile  [128 dims][64 keys] bf16, row pitch 136 B   2 x ds_read_b64 per A operand
// Two buffers of each; the global loads of tile t+1 are issued before the products of
// tile t and land in registers while the MFMAs run, one barrier per tile.
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
constexpr int kKPitch = 272;   // bytes per K row in LDS
constexpr int kVPitch = 136;   // bytes per V^T row in LDS
constexpr int kKBytes = kKeyTile * kKPitch;   // 17408
constexpr int kVBytes = kHeadDim * kVPitch;   // 17408
constexpr int kBufBytes = kKBytes + kVBytes;
constexpr int kThreads = 256;
constexpr float kLazyLog2 = 8.0f;

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

    const uint16_t *kbase = p.k + (uint64_t)kv_head * kHeadDim;
    const uint16_t *vbase = p.v + (uint64_t)kv_head * kHeadDim;

    // global -> registers for one tile.  K: thread covers rows tid/16 + 16r, chunk tid%16.
    // V: thread covers keys 4*(tid%16) .. +3 and dims 8*(tid/16) .. +7 (transposed on store).
    u32x4 kreg[4], vreg[4];
    auto load_tile = [&](uint32_t tile) {
        const uint32_t first = tile * kKeyTile;
        const uint32_t last = p.kv_tokens - 1u;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t key = min(first + (uint32_t)(tid >> 4) + 16u * r, last);
            kreg[r] = load_b128(kbase + (uint64_t)key * p.k_stride + (tid & 15) * 8);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t key = min(first + 4u * (tid & 15) + r, last);
            vreg[r] = load_b128(vbase + (uint64_t)key * p.v_stride + (tid >> 4) * 8);
        }
    };
    auto store_tile = [&](int buf) {
        unsigned char *kl = lds + buf * kBufBytes;
        unsigned char *vl = kl + kKBytes;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            *reinterpret_cast<u32x4 *>(kl + ((tid >> 4) + 16 * r) * kKPitch + (tid & 15) * 16) =
                kreg[r];
        // transpose 4 keys x 8 dims: dim e of the chunk gets the four keys' values
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int w = e >> 1;
            const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
            u32x2 out;
            out.x = __builtin_amdgcn_perm(vreg[1][w], vreg[0][w], sel);
            out.y = __builtin_amdgcn_perm(vreg[3][w], vreg[2][w], sel);
            *reinterpret_cast<u32x2 *>(vl + ((tid >> 4) * 8 + e) * kVPitch + (tid & 15) * 8) = out;
        }
    };

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

    load_tile(0u);
    for (uint32_t t = 0; t < tiles; ++t) {
        const int buf = (int)(t & 1u);
        store_tile(buf);
        __syncthreads();
        if (t + 1u < tiles) load_tile(t + 1u);
        const uint32_t key0 = t * kKeyTile;
        // a wave whose every row sees nothing of this tile skips the products
        const uint32_t wave_last_vis = p.causal
                                           ? p.query_start + min(row0 + kRowsPerWave, p.query_tokens) - 1u
                                           : p.kv_tokens - 1u;
        if (!wave_active || key0 > wave_last_vis) continue;
        const unsigned char *kl = lds + buf * kBufBytes;
        const unsigned char *vl = kl + kKBytes;

        // ---- S^T = K . Q^T -------------------------------------------------
        floatx16 s[2][NB];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[mb][nb][i] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                const bf16x8 a = as_bf16x8(*reinterpret_cast<const u32x4 *>(
                    kl + (mb * 32 + n) * kKPitch + kk * 32 + g * 16));
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) s[mb][nb] = mfma_32x32x16(a, q[nb][kk], s[mb][nb]);
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
                    const unsigned char *row = vl + (db * 32 + n) * kVPitch + (mb * 32 + u * 16 + g * 4) * 2;
                    u32x4 a;
                    const u32x2 lo = *reinterpret_cast<const u32x2 *>(row);
                    const u32x2 hi = *reinterpret_cast<const u32x2 *>(row + 16);
                    a.x = lo.x;
                    a.y = lo.y;
                    a.z = hi.x;
                    a.w = hi.y;
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        o[db][nb] = mfma_32x32x16(as_bf16x8(a), pb[nb], o[db][nb]);
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
