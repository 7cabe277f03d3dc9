// Absorbed-latent MLA decode for gfx950 (wave64): `heads` query heads of one batch
// element attend one shared latent row per token.  The score runs over key_dim = 576
// lanes (512 latent + 64 decoupled rope), the value is the first 512 lanes of the same
// row, so every latent row is read from HBM once and used for both products.
//
// The context of a batch element is split into chunks; one workgroup of 4 waves owns one
// (chunk, batch element) and all 128 heads: wave w owns heads 32w..32w+31 as the N
// dimension of 32x32x16 MFMA tiles.  Per 32-token tile staged in LDS:
//     S^T[token][head] = C[token][:576] . Q[head][:576]      36 MFMAs, A = rows (LDS)
//     online softmax per lane (= per head), exp2 with scale*log2e folded in
//     O^T[dim][head]  += C^T[dim][token] . P^T[token][head]  32 MFMAs, A = transposed copy
// The latent tile is kept twice in LDS: row-major for the score product and transposed
// ([dim][token]) for the value product; both pitches are bank-conflict free.
// Unnormalised partials (max in log2 units, sum, accumulator) go to the workspace and
// yvex_rocm_decode_merge performs the log-sum-exp merge.
#include "mfma.h"

#include "../kernel_params.h"

namespace {

constexpr int kKeyDim = 576;
constexpr int kValueDim = 512;
constexpr int kTile = 32;                       // tokens per LDS tile
constexpr int kRowPitch = kKeyDim * 2 + 16;     // 1168 B: ds_read_b128 rows hit distinct banks
constexpr int kTPitch = kTile * 2 + 8;          // 72 B: ds_read_b64 rows hit distinct banks
constexpr int kRowBytes = kTile * kRowPitch;    // 37376
constexpr int kTBytes = kValueDim * kTPitch;    // 36864
constexpr int kBufBytes = kRowBytes + kTBytes;  // 74240
constexpr int kHeadsPerWave = 32;

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

}  // namespace

// grid = (chunks, batch), block 256 (heads must be 128), LDS 2 * kBufBytes = 145 KB.
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
yvex_rocm_mla_decode_bf16(const yvex_rocm_mla_params p)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kBufBytes];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, g = lane >> 5;
    const uint32_t chunk = blockIdx.x, batch = blockIdx.y;
    const uint32_t ctx = (uint32_t)p.context[batch];
    if (ctx == 0u || ctx > p.table_stride * p.page_tokens) {
        if (chunk == 0u && tid == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return;
    }
    const uint32_t t0 = chunk * p.chunk_tokens;
    if (t0 >= ctx) return;
    const uint32_t t1 = min(ctx, t0 + p.chunk_tokens);
    const uint32_t tiles = (t1 - t0 + kTile - 1) / kTile;
    const uint32_t head = wave * kHeadsPerWave + n;

    // Q fragments: B operand, lane (n, g) holds Q[head n][16*kk + 8g .. +7], kk = 0..35
    bf16x8 q[36];
    {
        const uint16_t *src = p.q + ((uint64_t)batch * p.heads + head) * kKeyDim + g * 8;
#pragma unroll
        for (int kk = 0; kk < 36; ++kk) q[kk] = as_bf16x8(load_b128(src + kk * 16));
    }

    const int32_t *table = p.page_table + (uint64_t)batch * p.table_stride;
    // staging registers: 8 x 16 B of the latent part (2 groups of 4 tokens x 8 dims, to be
    // transposed) + 1 x 16 B of the rope part
    u32x4 lat[2][4], rope;
    auto row_ptr = [&](uint32_t token) -> const uint16_t * {
        token = min(token, t1 - 1u);
        int32_t page = table[token / p.page_tokens];
        if (page < 0 || (uint32_t)page >= p.pool_pages) {
            flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
            page = 0;
        }
        return p.pool + ((uint64_t)page * p.page_tokens + token % p.page_tokens) * kKeyDim;
    };
    // item = tid + 256*s covers (token group tg = item % 8, dim chunk dc = item / 8)
    auto load_tile = [&](uint32_t tile) {
        const uint32_t first = t0 + tile * kTile;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int item = tid + 256 * s, tg = item & 7, dc = item >> 3;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                lat[s][r] = load_b128(row_ptr(first + tg * 4 + r) + dc * 8);
        }
        rope = load_b128(row_ptr(first + (tid >> 3)) + kValueDim + (tid & 7) * 8);
    };
    auto store_tile = [&](int buf) {
        unsigned char *rows = lds + buf * kBufBytes;
        unsigned char *tr = rows + kRowBytes;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int item = tid + 256 * s, tg = item & 7, dc = item >> 3;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                *reinterpret_cast<u32x4 *>(rows + (tg * 4 + r) * kRowPitch + dc * 16) = lat[s][r];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int w = e >> 1;
                const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
                u32x2 out;
                out.x = __builtin_amdgcn_perm(lat[s][1][w], lat[s][0][w], sel);
                out.y = __builtin_amdgcn_perm(lat[s][3][w], lat[s][2][w], sel);
                *reinterpret_cast<u32x2 *>(tr + (dc * 8 + e) * kTPitch + tg * 8) = out;
            }
        }
        *reinterpret_cast<u32x4 *>(rows + (tid >> 3) * kRowPitch + kValueDim * 2 + (tid & 7) * 16) =
            rope;
    };

    floatx16 o[16];
#pragma unroll
    for (int db = 0; db < 16; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    load_tile(0u);
    for (uint32_t t = 0; t < tiles; ++t) {
        const int buf = (int)(t & 1u);
        store_tile(buf);
        __syncthreads();
        if (t + 1u < tiles) load_tile(t + 1u);
        const unsigned char *rows = lds + buf * kBufBytes;
        const unsigned char *tr = rows + kRowBytes;
        const uint32_t key0 = t0 + t * kTile;

        floatx16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 36; ++kk) {
            const bf16x8 a = as_bf16x8(
                *reinterpret_cast<const u32x4 *>(rows + n * kRowPitch + kk * 32 + g * 16));
            s = mfma_32x32x16(a, q[kk], s);
        }
        const bool tail = key0 + kTile > t1;
        float mloc = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float x = s[i] * p.scale_log2;
            if (tail && key0 + (i >> 2) * 8 + g * 4 + (i & 3) >= t1) x = -INFINITY;
            s[i] = x;
            mloc = fmaxf(mloc, x);
        }
        mloc = fmaxf(mloc, xor_lanes(mloc, 32));
        const float m_new = fmaxf(m_run, mloc);
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0ull) {
            const float alpha = fast_exp2(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < 16; ++db) o[db] *= alpha;
            m_run = m_new;
        }
        uint32_t pk[8];
        float lsum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float p0 = fast_exp2(s[i] - m_run), p1 = fast_exp2(s[i + 1] - m_run);
            lsum += p0 + p1;
            pk[i >> 1] = pack_bf16x2(p0, p1);
        }
        l_run += lsum;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const u32x4 w = {pk[u * 4 + 0], pk[u * 4 + 1], pk[u * 4 + 2], pk[u * 4 + 3]};
            const bf16x8 pb = as_bf16x8(w);
#pragma unroll
            for (int db = 0; db < 16; ++db) {
                const unsigned char *src = tr + (db * 32 + n) * kTPitch + (u * 16 + g * 4) * 2;
                const u32x2 lo = *reinterpret_cast<const u32x2 *>(src);
                const u32x2 hi = *reinterpret_cast<const u32x2 *>(src + 16);
                u32x4 a;
                a.x = lo.x;
                a.y = lo.y;
                a.z = hi.x;
                a.w = hi.y;
                if (tail) {
                    // tokens past the context alias the last valid row (finite unless the
                    // data itself is not), their weights are exact zeros
                }
                o[db] = mfma_32x32x16(as_bf16x8(a), pb, o[db]);
            }
        }
    }

    float l = l_run;
    l += xor_lanes(l, 32);
    const uint64_t slot = ((uint64_t)batch * p.max_chunks + chunk) * p.heads + head;
    float *acc = p.part_acc + slot * kValueDim;
#pragma unroll
    for (int db = 0; db < 16; ++db)
#pragma unroll
        for (int grp = 0; grp < 4; ++grp) {
            floatx4 v = {o[db][grp * 4 + 0], o[db][grp * 4 + 1], o[db][grp * 4 + 2],
                         o[db][grp * 4 + 3]};
            *reinterpret_cast<floatx4 *>(acc + db * 32 + grp * 8 + g * 4) = v;
        }
    if (g == 0) {
        p.part_ml[slot * 2 + 0] = m_run;
        p.part_ml[slot * 2 + 1] = l;
    }
}
