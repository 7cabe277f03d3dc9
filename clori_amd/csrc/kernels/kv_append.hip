// KV page writer for gfx950 (wave64): takes the new key/value rows of a batch of sessions
// (bf16, token-major [row][kv head][128]) and writes them into the paged device layouts the
// decode kernels read, applying the rotate-half position encoding to the keys on the way
// and, for Q8_0 pools, quantising on write.  This is the step in front of attention
// (src/runtime/decoder.c:1236-1242 rotary, src/runtime/stateful_attention.c:183-243 append).
//
// One wave owns one (session, touched page, kv head): it reads up to 16 rows of 256 bytes,
// and writes one 4096-byte (bf16) or 2176-byte (Q8_0) block per pool.  A page that is only
// partly covered by the new tokens keeps its other tokens (read-modify-write inside the
// wave; sessions never share a page).
//
// Rotary (src/backend/cuda/transformer_kernels.cu:79-108): with half = rotary_dim / 2 and
// c < half, first = k[c], second = k[c + half], cosine/sine = table[row][c]:
//     k[c]        = bf16(bf16(first * cosine)  - bf16(second * sine))
//     k[c + half] = bf16(bf16(second * cosine) + bf16(first * sine))
// every product and sum rounded to bf16 (round to nearest even), dims >= rotary_dim unchanged.
//
// Q8_0 (src/gguf/quant_block.c:160-186): per 32 values scale = f16(max|x| / 127), codes =
// clamp(roundf(x * (1 / f32(scale))), -127, 127), roundf half away from zero.
//
// Page layouts, per (page, kv head), 16 tokens t, 128 dims c:
//   BF16  K  [c/8][t][8]                     V  [c][t]
//   Q8_0  K  codes [g][t][j][8], c = 32j+8g+e    V  codes [t/4][c%16][c/16][t%4]
//         then f16 scales [t][j] in both
#include "mfma.h"

#include "../kernel_params.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kPageTokens = 16;

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

// bf16 bits of a float with the reference's rounding; inputs here are finite or flagged
__device__ inline float round_bf16(float v) { return bf16_to_f32(bf16_bits(v)); }

struct Span {
    uint32_t page_id;   // pool page
    uint32_t lo, hi;    // token slots [lo, hi) of the page that are new
    uint32_t row;       // input row of slot lo
    bool valid;
};

// Which page this workgroup writes and which input rows land in it.
__device__ inline Span locate(const yvex_rocm_kv_append_params &p)
{
    Span s;
    s.valid = false;
    const uint32_t session = blockIdx.z, slot = blockIdx.x;
    const int32_t count = p.token_count[session], start = p.position_start[session];
    const int32_t row0 = p.row_start[session];
    if (count <= 0) return s;
    if (start < 0 || row0 < 0 || (uint64_t)row0 + (uint32_t)count > p.total_tokens ||
        (uint64_t)start + (uint32_t)count > (uint64_t)p.table_stride * kPageTokens) {
        if (slot == 0u && blockIdx.y == 0u && threadIdx.x == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return s;
    }
    const uint32_t first_page = (uint32_t)start / kPageTokens;
    const uint32_t last_page = ((uint32_t)start + (uint32_t)count - 1u) / kPageTokens;
    const uint32_t page = first_page + slot;
    if (page > last_page) return s;
    const int32_t id = p.page_table[(uint64_t)session * p.table_stride + page];
    if (id < 0 || (uint32_t)id >= p.pool_pages) {
        if (threadIdx.x == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return s;
    }
    const uint32_t begin = max((uint32_t)start, page * kPageTokens);
    const uint32_t end = min((uint32_t)start + (uint32_t)count, (page + 1u) * kPageTokens);
    s.page_id = (uint32_t)id;
    s.lo = begin - page * kPageTokens;
    s.hi = end - page * kPageTokens;
    s.row = (uint32_t)row0 + (begin - (uint32_t)start);
    s.valid = true;
    return s;
}

// Eight consecutive dims [c0, c0+8) of input row `row`, kv head `head`, as floats; keys get
// the rotary applied.  Returns false when a value is not finite.
__device__ inline bool load_eight(const yvex_rocm_kv_append_params &p, const uint16_t *src,
                                  uint32_t row, uint32_t head, uint32_t c0, bool rotate,
                                  float (&out)[8])
{
    const uint16_t *base = src + ((uint64_t)row * p.kv_heads + head) * kHeadDim;
    const u32x4 own = load_b128(base + c0);
    bool ok = true;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i + 0] = bf16_to_f32((uint16_t)(own[i] & 0xffffu));
        out[2 * i + 1] = bf16_to_f32((uint16_t)(own[i] >> 16));
    }
    if (rotate && c0 < p.rotary_dim) {
        const uint32_t half = p.rotary_dim / 2u;
        const bool upper = c0 >= half;
        const uint32_t partner_c = upper ? c0 - half : c0 + half, table_c = upper ? c0 - half : c0;
        const u32x4 other = load_b128(base + partner_c);
        const float *cs = p.cosine + (uint64_t)row * p.rotary_dim + table_c;
        const float *sn = p.sine + (uint64_t)row * p.rotary_dim + table_c;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t word = other[i >> 1];
            const float partner = bf16_to_f32((uint16_t)((i & 1) ? word >> 16 : word & 0xffffu));
            const float cosine = cs[i], sine = sn[i];
            ok &= isfinite(cosine) && isfinite(sine);
            // lower half: first = own, second = partner; upper half: first = partner, second = own
            const float a = round_bf16(out[i] * cosine);
            const float b = round_bf16(partner * sine);
            out[i] = round_bf16(upper ? a + b : a - b);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) ok &= isfinite(out[i]);
    return ok;
}

}  // namespace

// grid = (pages a session can touch, kv heads, sessions), block 64.
extern "C" __global__ void __launch_bounds__(64)
yvex_rocm_kv_append_bf16(const yvex_rocm_kv_append_params p)
{
    __shared__ uint16_t v_rows[kPageTokens][kHeadDim + 8];
    const Span s = locate(p);
    if (!s.valid) return;
    const uint32_t lane = threadIdx.x, head = blockIdx.y;
    const uint64_t block = ((uint64_t)s.page_id * p.kv_heads + head) * (kPageTokens * kHeadDim);
    uint16_t *kdst = (uint16_t *)p.k_pool + block, *vdst = (uint16_t *)p.v_pool + block;
    bool ok = true;
    // keys: 256 chunks of 8 dims, chunk id = c8 * 16 + t is also its place in the block
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t id = lane + 64u * i, t = id & 15u, c8 = id >> 4;
        if (t < s.lo || t >= s.hi) continue;
        float k[8];
        ok &= load_eight(p, p.key, s.row + (t - s.lo), head, c8 * 8u, p.rotary_dim != 0u, k);
        u32x4 w;
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = (uint32_t)bf16_bits(k[2 * j]) | ((uint32_t)bf16_bits(k[2 * j + 1]) << 16);
        *reinterpret_cast<u32x4 *>(kdst + id * 8u) = w;
    }
    // values: through LDS, then 8 tokens of one dim per 16-byte piece
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t id = lane + 64u * i, t = id >> 4, c8 = id & 15u;
        if (t < s.lo || t >= s.hi) continue;
        float v[8];
        ok &= load_eight(p, p.value, s.row + (t - s.lo), head, c8 * 8u, false, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) v_rows[t][c8 * 8u + j] = bf16_bits(v[j]);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t id = lane + 64u * i, c = id >> 1, t8 = (id & 1u) * 8u;
        if (t8 + 8u <= s.lo || t8 >= s.hi) continue;
        u32x4 w = *reinterpret_cast<const u32x4 *>(vdst + c * 16u + t8);  // tokens that stay
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t t = t8 + j;
            if (t < s.lo || t >= s.hi) continue;
            const uint32_t bits = v_rows[t][c];
            w[j >> 1] = (j & 1) ? (w[j >> 1] & 0x0000ffffu) | (bits << 16)
                                : (w[j >> 1] & 0xffff0000u) | bits;
        }
        *reinterpret_cast<u32x4 *>(vdst + c * 16u + t8) = w;
    }
    if (!ok) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
}

// grid as above.  Lane (t = lane / 4, j = lane % 4) owns the 32 dims of Q8_0 block j of token t.
extern "C" __global__ void __launch_bounds__(64)
yvex_rocm_kv_append_q8_0(const yvex_rocm_kv_append_params p)
{
    __shared__ unsigned char v_codes[kPageTokens][kHeadDim + 16];
    const Span s = locate(p);
    if (!s.valid) return;
    const uint32_t lane = threadIdx.x, head = blockIdx.y;
    const uint32_t t = lane >> 2, j = lane & 3u;
    constexpr uint32_t kBlockBytes = kPageTokens * kHeadDim + kPageTokens * 4 * 2;
    const uint64_t block = ((uint64_t)s.page_id * p.kv_heads + head) * kBlockBytes;
    unsigned char *kdst = (unsigned char *)p.k_pool + block, *vdst = (unsigned char *)p.v_pool + block;
    const bool mine = t >= s.lo && t < s.hi;
    bool ok = true, representable = true;
#pragma unroll
    for (int pool = 0; pool < 2; ++pool) {
        if (!mine) continue;
        const uint16_t *src = pool == 0 ? p.key : p.value;
        float x[32];
        float maximum = 0.f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float part[8];
            ok &= load_eight(p, src, s.row + (t - s.lo), head, 32u * j + 8u * g,
                             pool == 0 && p.rotary_dim != 0u, part);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[8 * g + e] = part[e];
                maximum = fmaxf(maximum, fabsf(part[e]));
            }
        }
        const _Float16 half = (_Float16)(maximum / 127.0f);
        const float scale = (float)half;
        representable &= isfinite(scale) && !(maximum > 0.f && scale == 0.f);
        const float inverse = scale != 0.f ? 1.0f / scale : 0.f;
        unsigned char *dst = pool == 0 ? kdst : vdst;
        *reinterpret_cast<uint16_t *>(dst + kPageTokens * kHeadDim + (t * 4u + j) * 2u) =
            __builtin_bit_cast(uint16_t, half);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            uint32_t packed[2] = {0u, 0u};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float scaled = roundf(x[8 * g + e] * inverse);
                const int code = scaled < -127.f ? -127 : scaled > 127.f ? 127 : (int)scaled;
                packed[e >> 2] |= ((uint32_t)code & 0xffu) << (8 * (e & 3));
                if (pool == 1) v_codes[t][32u * j + 8u * g + e] = (unsigned char)code;
            }
            if (pool == 0) {
                u32x2 w = {packed[0], packed[1]};
                *reinterpret_cast<u32x2 *>(kdst + (((g * 16u + t) * 4u + j) * 8u)) = w;
            }
        }
    }
    __syncthreads();
    // value codes: 4-byte groups (4 tokens of one dim) at ((tg*16 + m)*8 + b)*4, c = 16b + m
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t id = lane + 64u * i;  // 512 groups = tg (4) x m (16) x b (8)
        const uint32_t b = id & 7u, m = (id >> 3) & 15u, tg = id >> 7, c = 16u * b + m;
        if (4u * tg + 4u <= s.lo || 4u * tg >= s.hi) continue;
        uint32_t w = *reinterpret_cast<const uint32_t *>(vdst + id * 4u);  // tokens that stay
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t tt = 4u * tg + q;
            if (tt < s.lo || tt >= s.hi) continue;
            w = (w & ~(0xffu << (8 * q))) | ((uint32_t)v_codes[tt][c] << (8 * q));
        }
        *reinterpret_cast<uint32_t *>(vdst + id * 4u) = w;
    }
    if (!ok) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    if (!representable) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
}
