// KV page writer for gfx950 (wave64): takes the new key/value rows of a batch of sessions
// (bf16, token-major [row][kv head][128]) and writes them into the paged device layouts the
// decode kernels read, applying the rotate-half position encoding to the keys on the way
// and, for Q8_0 pools, quantising on write.  This is the step in front of attention
// (src/runtime/decoder.c:1236-1242 rotary, src/runtime/stateful_attention.c:183-243 append).
//
// One wave owns one (session, touched page, kv head): it reads up to 16 rows of 256 bytes,
// and writes one 4096-byte (bf16) or 2176-byte (Q8_0) block per pool; a workgroup is four
// such waves (four kv heads of one page).  Every global load of a wave is issued before the
// first result is used.  A page that is only partly covered by the new tokens keeps its
// other tokens (read-modify-write inside the wave; sessions never share a page).
//
// Keys are handled as 16-byte chunks (token t, dims 8*c8 .. 8*c8+7).  With rotary dimension
// R the chunks c8 < R/16 are the lower half, R/16 <= c8 < R/8 the upper half, the rest are
// copied.  The lane of a lower chunk loads its partner chunk and one cos and one sin piece
// and produces both rotated chunks; the lanes of upper chunks load and compute nothing.
//
// Rotary, mode 0 (src/backend/cuda/transformer_kernels.cu:79-108): with half = rotary_dim / 2
// and c < half, first = k[c], second = k[c + half], cosine/sine = table[row][c]:
//     k[c]        = bf16(bf16(first * cosine)  - bf16(second * sine))
//     k[c + half] = bf16(bf16(second * cosine) + bf16(first * sine))
// every product and sum rounded to bf16 (round to nearest even), dims >= rotary_dim unchanged.
// Mode 1 is the order of the reference's decoder (src/runtime/decoder.c:1112-1131): the plain
// F32 rotation (transformer_kernels.cu:110-134) and then one bf16 rounding,
//     k[c]        = bf16(fma(first, cosine, -(second * sine)))
//     k[c + half] = bf16(fma(second, cosine, first * sine))
// with the first product of each sum fused, as the compilers of both GPU targets contract
// these expressions at their default flags.
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
constexpr int kWaves = YVEX_ROCM_KV_APPEND_HEADS;
constexpr int kRowPitch = kHeadDim + 8;       // bf16 elements per LDS row (272 bytes)
constexpr int kCodePitch = kHeadDim + 16;     // bytes per LDS row of value codes

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

__device__ inline float bf16_of(const u32x4 &w, int i)
{
    const uint32_t word = w[i >> 1];
    return __builtin_bit_cast(float, (i & 1) ? word & 0xffff0000u : word << 16);
}

// the two bf16 values of a packed word as floats
__device__ inline float low_half(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ inline float high_half(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// true when none of the eight bf16 values is an infinity or a NaN
__device__ inline bool finite_bits(const u32x4 &w)
{
    bool ok = true;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        ok &= (w[j] & 0x7f80u) != 0x7f80u && (w[j] & 0x7f800000u) != 0x7f800000u;
    return ok;
}

struct Span {
    uint32_t page_id;   // pool page
    uint32_t sub;       // 16-token block of the page
    uint32_t lo, hi;    // token slots [lo, hi) of the page that are new
    uint32_t row;       // input row of slot lo
    bool valid;
};

// Which page this workgroup writes and which input rows land in it.
__device__ inline Span locate(const yvex_rocm_kv_append_params &p)
{
    Span s;
    s.valid = false;
    s.page_id = 0u;
    s.sub = 0u;
    s.lo = 0u;
    s.hi = 1u;
    s.row = 0u;
    const uint32_t session = blockIdx.z, slot = blockIdx.x;
    const int32_t count = p.token_count[session], start = p.position_start[session];
    const int32_t row0 = p.row_start[session];
    if (count <= 0) return s;
    if (start < 0 || row0 < 0 || (uint64_t)row0 + (uint32_t)count > p.total_tokens ||
        (uint64_t)start + (uint32_t)count > ((uint64_t)p.table_stride * kPageTokens) << p.page_shift) {
        if (slot == 0u && blockIdx.y == 0u && threadIdx.x == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return s;
    }
    const uint32_t first_page = (uint32_t)start / kPageTokens;
    const uint32_t last_page = ((uint32_t)start + (uint32_t)count - 1u) / kPageTokens;
    if (last_page - first_page >= gridDim.x) {
        // more tokens than the launch was sized for (max_tokens_per_session): refuse rather
        // than drop the pages no workgroup covers
        if (slot == 0u && blockIdx.y == 0u && threadIdx.x == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return s;
    }
    const uint32_t page = first_page + slot;
    if (page > last_page) return s;
    // `page` counts 16-token blocks; a pool page holds 1 << page_shift of them
    const int32_t id = p.page_table[(uint64_t)session * p.table_stride + (page >> p.page_shift)];
    if (id < 0 || (uint32_t)id >= p.pool_pages) {
        if (threadIdx.x == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return s;
    }
    const uint32_t begin = max((uint32_t)start, page * kPageTokens);
    const uint32_t end = min((uint32_t)start + (uint32_t)count, (page + 1u) * kPageTokens);
    s.page_id = (uint32_t)id;
    s.sub = page & ((1u << p.page_shift) - 1u);
    s.lo = begin - page * kPageTokens;
    s.hi = end - page * kPageTokens;
    s.row = (uint32_t)row0 + (begin - (uint32_t)start);
    s.valid = true;
    return s;
}

// Input row that lands in token slot t; slots outside [lo, hi) read a neighbouring row of the
// span (the value is loaded and dropped) so that loads need no branches.
__device__ inline uint32_t row_of(const Span &s, uint32_t t)
{
    return s.row + (min(max(t, s.lo), s.hi - 1u) - s.lo);
}

enum Role { kLower, kUpper, kPlain };

// One key chunk in flight: raw loads first, arithmetic later.
struct KeyChunk {
    u32x4 own, other, cs[2], sn[2];
    uint32_t t, c8;
    int role;
};

template <int kDim = kHeadDim>
__device__ inline void key_issue(const yvex_rocm_kv_append_params &p, const Span &s, uint32_t head,
                                 uint32_t id, KeyChunk &k)
{
    const uint32_t pairs = p.rotary_dim / 16u;   // chunks in each rotary half
    k.t = id & 15u;
    k.c8 = id >> 4;
    k.role = k.c8 < pairs ? kLower : k.c8 < 2u * pairs ? kUpper : kPlain;
    const uint32_t row = row_of(s, k.t);
    const uint16_t *base = p.key + ((uint64_t)row * p.kv_heads + head) * kDim + k.c8 * 8u;
    if (k.role != kUpper) k.own = load_b128(base);
    if (k.role == kLower) {
        const uint64_t at = (uint64_t)row * p.rotary_dim + k.c8 * 8u;
        k.other = load_b128(base + p.rotary_dim / 2u);
        k.cs[0] = load_b128(p.cosine + at);
        k.cs[1] = load_b128(p.cosine + at + 4);
        k.sn[0] = load_b128(p.sine + at);
        k.sn[1] = load_b128(p.sine + at + 4);
    }
}

// Rotated (or copied) chunk(s) as packed bf16; `upper` is produced by lower-half lanes only.
// Returns false when a table entry, an input or a result is not finite.
__device__ inline bool key_finish(const KeyChunk &k, u32x4 &lower, u32x4 &upper, bool plain)
{
    if (k.role == kUpper) return true;
    if (k.role == kPlain) {
        lower = k.own;
        return finite_bits(k.own);
    }
    // Two dims at a time; v_cvt_pk_bf16_f32 rounds to nearest even exactly as the reference
    // codec does for every finite value and for overflow.  A non-finite table entry or input
    // always leaves a non-finite result (inf * 0 and inf - inf are NaN), so checking the
    // results covers all of them.
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float first0 = bf16_of(k.own, 2 * j), first1 = bf16_of(k.own, 2 * j + 1);
        const float second0 = bf16_of(k.other, 2 * j), second1 = bf16_of(k.other, 2 * j + 1);
        const uint32_t c0 = k.cs[j >> 1][(2 * j) & 3], c1 = k.cs[j >> 1][(2 * j + 1) & 3];
        const uint32_t s0 = k.sn[j >> 1][(2 * j) & 3], s1 = k.sn[j >> 1][(2 * j + 1) & 3];
        const float cosine0 = __builtin_bit_cast(float, c0), cosine1 = __builtin_bit_cast(float, c1);
        const float sine0 = __builtin_bit_cast(float, s0), sine1 = __builtin_bit_cast(float, s1);
        if (plain) {
            // first * cosine - second * sine and second * cosine + first * sine with the second
            // product rounded and the first fused into the sum: one of the legal contractions of
            // the reference's plain F32 kernel (src/backend/cuda/transformer_kernels.cu:110-134),
            // the one LLVM picks for these expressions.  Which one the reference's compiler picks
            // is not visible in its sources: the last bit of a result next to a bf16 tie is not
            // pinned by the reference (the unfused evaluation differs there, by one bf16 step).
            lower[j] = pack_bf16x2(__builtin_fmaf(first0, cosine0, -(second0 * sine0)),
                                   __builtin_fmaf(first1, cosine1, -(second1 * sine1)));
            upper[j] = pack_bf16x2(__builtin_fmaf(second0, cosine0, first0 * sine0),
                                   __builtin_fmaf(second1, cosine1, first1 * sine1));
            continue;
        }
        const uint32_t fc = pack_bf16x2(first0 * cosine0, first1 * cosine1);
        const uint32_t ss = pack_bf16x2(second0 * sine0, second1 * sine1);
        const uint32_t sc = pack_bf16x2(second0 * cosine0, second1 * cosine1);
        const uint32_t fs = pack_bf16x2(first0 * sine0, first1 * sine1);
        lower[j] = pack_bf16x2(low_half(fc) - low_half(ss), high_half(fc) - high_half(ss));
        upper[j] = pack_bf16x2(low_half(sc) + low_half(fs), high_half(sc) + high_half(fs));
    }
    return finite_bits(lower) && finite_bits(upper);
}

}  // namespace

namespace {

// The bf16 writer for one head dimension: a wave moves the 16 x kDim / 8 key chunks and as many
// value chunks of its block, kDim / 32 of each per lane (128 is the tuned build; 64 and 256 are
// the same code with other counts).
template <int kDim>
__device__ __forceinline__ void kv_append_bf16(const yvex_rocm_kv_append_params &p,
                                               uint16_t (*v_rows_all)[kPageTokens][kDim + 8])
{
    constexpr int kPerLane = kDim / 32;          // 16-byte chunks of K (and of V) per lane
    constexpr uint32_t kRowChunks = kDim / 8;    // 16-byte chunks of a row
    constexpr int kRowPitch = kDim + 8;
    const Span s = locate(p);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t head = blockIdx.y * kWaves + wave;
    const bool active = s.valid && head < p.kv_heads;
    uint16_t (*v_rows)[kRowPitch] = v_rows_all[wave];
    const uint64_t block = ((((uint64_t)s.page_id * p.kv_heads + head) << p.page_shift) + s.sub) *
                           (kPageTokens * kDim);
    uint16_t *kdst = (uint16_t *)p.k_pool + block, *vdst = (uint16_t *)p.v_pool + block;
    const bool partial = s.lo != 0u || s.hi != (uint32_t)kPageTokens;
    const uint32_t pairs = p.rotary_dim / 16u;
    bool ok = true;
    KeyChunk k[kPerLane];
    u32x4 v[kPerLane], old[kPerLane] = {};
    if (active) {
        // every load of the wave, then the arithmetic
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) key_issue<kDim>(p, s, head, lane + 64u * i, k[i]);
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const uint32_t id = lane + 64u * i, t = id / kRowChunks, c8 = id % kRowChunks;
            v[i] = load_b128(p.value + ((uint64_t)row_of(s, t) * p.kv_heads + head) * kDim + c8 * 8u);
        }
        if (partial) {
#pragma unroll
            for (int i = 0; i < kPerLane; ++i) old[i] = load_b128(vdst + (lane + 64u * i) * 8u);
        }
        // keys: chunk (c8, t) sits at 16-byte slot c8 * 16 + t of the block
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            u32x4 lower, upper;
            ok &= key_finish(k[i], lower, upper, p.rotary_mode != 0u);
            if (k[i].t < s.lo || k[i].t >= s.hi) continue;
            if (k[i].role != kUpper)
                *reinterpret_cast<u32x4 *>(kdst + (k[i].c8 * 16u + k[i].t) * 8u) = lower;
            if (k[i].role == kLower)
                *reinterpret_cast<u32x4 *>(kdst + ((k[i].c8 + pairs) * 16u + k[i].t) * 8u) = upper;
        }
        // values: rows into LDS, then 8 tokens of one dim per 16-byte piece
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const uint32_t id = lane + 64u * i, t = id / kRowChunks, c8 = id % kRowChunks;
            if (t >= s.lo && t < s.hi) ok &= finite_bits(v[i]);
            *reinterpret_cast<u32x4 *>(&v_rows[t][c8 * 8u]) = v[i];
        }
    }
    __syncthreads();
    if (active) {
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            const uint32_t id = lane + 64u * i, c = id >> 1, t8 = (id & 1u) * 8u;
            if (t8 + 8u <= s.lo || t8 >= s.hi) continue;
            u32x4 w;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = (uint32_t)v_rows[t8 + 2 * j][c] | ((uint32_t)v_rows[t8 + 2 * j + 1][c] << 16);
            if (partial) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t t = t8 + j, mask = (j & 1) ? 0xffff0000u : 0x0000ffffu;
                    if (t < s.lo || t >= s.hi) w[j >> 1] = (w[j >> 1] & ~mask) | (old[i][j >> 1] & mask);
                }
            }
            *reinterpret_cast<u32x4 *>(vdst + id * 8u) = w;
        }
        if (!ok) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    }
}

}  // namespace

// grid = (pages a session can touch, kv heads / 4, sessions), block 256: wave w writes kv head
// 4 * blockIdx.y + w.
#define YVEX_KV_APPEND_BF16_KERNEL(name, head_dim)                                                   \
    extern "C" __global__ void __launch_bounds__(64 * kWaves) name(const yvex_rocm_kv_append_params p) \
    {                                                                                                \
        __shared__ __attribute__((aligned(16))) uint16_t v_rows_all[kWaves][kPageTokens][head_dim + 8]; \
        kv_append_bf16<head_dim>(p, v_rows_all);                                                      \
    }

YVEX_KV_APPEND_BF16_KERNEL(yvex_rocm_kv_append_bf16, 128)
YVEX_KV_APPEND_BF16_KERNEL(yvex_rocm_kv_append_bf16_64, 64)
YVEX_KV_APPEND_BF16_KERNEL(yvex_rocm_kv_append_bf16_256, 256)

namespace {

// Q8_0 block of 32 values: f16 scale bits and 32 codes packed four to a word.
__device__ inline bool quantise(const float (&x)[32], uint16_t &scale_bits, uint32_t (&codes)[8])
{
#pragma clang fp contract(off)   // the product is rounded before the rounding add, as in the reference
    float maximum = 0.f;
#pragma unroll
    for (int e = 0; e < 32; ++e) maximum = fmaxf(maximum, fabsf(x[e]));
    const _Float16 half = (_Float16)(maximum / 127.0f);
    const float scale = (float)half;
    const float inverse = scale != 0.f ? 1.0f / scale : 0.f;
    scale_bits = __builtin_bit_cast(uint16_t, half);
    // roundf (half away from zero) as a truncating convert of x + copysign(0.5 - 2^-25, x):
    // exact for |x| < 2^23 (ties land on or above the next integer, the value just below a
    // tie stays below it), then the clamp on the integer
    const float nudge = __builtin_bit_cast(float, 0x3effffffu);
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        uint32_t word = 0u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float scaled = x[4 * w + e] * inverse;
            const int code = min(max((int)(scaled + copysignf(nudge, scaled)), -127), 127);
            word |= ((uint32_t)code & 0xffu) << (8 * e);
        }
        codes[w] = word;
    }
    return isfinite(scale) && !(maximum > 0.f && scale == 0.f);
}

}  // namespace

// grid and waves as above.  After the rotary, lane (t = lane / 4, j = lane % 4) owns the 32
// dims of Q8_0 block j of token t.
extern "C" __global__ void __launch_bounds__(64 * kWaves)
yvex_rocm_kv_append_q8_0(const yvex_rocm_kv_append_params p)
{
    __shared__ __attribute__((aligned(16))) uint16_t k_rows_all[kWaves][kPageTokens][kRowPitch];
    __shared__ __attribute__((aligned(16))) unsigned char v_codes_all[kWaves][kPageTokens][kCodePitch];
    const Span s = locate(p);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t head = blockIdx.y * kWaves + wave;
    const bool active = s.valid && head < p.kv_heads;
    uint16_t (*k_rows)[kRowPitch] = k_rows_all[wave];
    unsigned char (*v_codes)[kCodePitch] = v_codes_all[wave];
    const uint32_t t = lane >> 2, j = lane & 3u;
    constexpr uint32_t kCodeBytes = kPageTokens * kHeadDim;
    constexpr uint32_t kBlockBytes = kCodeBytes + kPageTokens * 4 * 2;
    const uint64_t block = ((((uint64_t)s.page_id * p.kv_heads + head) << p.page_shift) + s.sub) *
                           kBlockBytes;
    unsigned char *kdst = (unsigned char *)p.k_pool + block, *vdst = (unsigned char *)p.v_pool + block;
    const bool partial = s.lo != 0u || s.hi != (uint32_t)kPageTokens;
    const bool mine = t >= s.lo && t < s.hi;
    const uint32_t pairs = p.rotary_dim / 16u;
    bool ok = true, representable = true;
    KeyChunk k[4];
    u32x4 v[4];
    uint32_t old[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    if (active) {
#pragma unroll
        for (int i = 0; i < 4; ++i) key_issue(p, s, head, lane + 64u * i, k[i]);
        {
            const uint16_t *src = p.value + ((uint64_t)row_of(s, t) * p.kv_heads + head) * kHeadDim + 32u * j;
#pragma unroll
            for (int g = 0; g < 4; ++g) v[g] = load_b128(src + 8 * g);
        }
        if (partial) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                old[i] = *reinterpret_cast<const uint32_t *>(vdst + YVEX_ROCM_Q8_CODE_OFFSET((lane + 64u * i) * 4u));
        }
        // rotated key rows into LDS
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4 lower, upper;
            ok &= key_finish(k[i], lower, upper, p.rotary_mode != 0u) || k[i].t < s.lo || k[i].t >= s.hi;
            if (k[i].role != kUpper)
                *reinterpret_cast<u32x4 *>(&k_rows[k[i].t][k[i].c8 * 8u]) = lower;
            if (k[i].role == kLower)
                *reinterpret_cast<u32x4 *>(&k_rows[k[i].t][(k[i].c8 + pairs) * 8u]) = upper;
        }
        // values: quantise this lane's block, codes into LDS, scale straight to the pool
        if (mine) {
            float x[32];
            uint32_t codes[8];
            uint16_t scale_bits;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                ok &= finite_bits(v[g]);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[8 * g + e] = bf16_of(v[g], e);
            }
            representable &= quantise(x, scale_bits, codes);
            *reinterpret_cast<uint16_t *>(vdst + kCodeBytes + (t * 4u + j) * 2u) = scale_bits;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x2 w = {codes[2 * g], codes[2 * g + 1]};
                *reinterpret_cast<u32x2 *>(&v_codes[t][32u * j + 8u * g]) = w;
            }
        }
    }
    __syncthreads();
    if (active) {
        if (mine) {
            float x[32];
            uint32_t codes[8];
            uint16_t scale_bits;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(&k_rows[t][32u * j + 8u * g]);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[8 * g + e] = bf16_of(w, e);
            }
            representable &= quantise(x, scale_bits, codes);
            *reinterpret_cast<uint16_t *>(kdst + kCodeBytes + (t * 4u + j) * 2u) = scale_bits;
            // key codes: 8-byte groups, bytes 8j .. 8j+7 of the 32 that lane 16g + t of a reading
            // wave consumes (dims 32j + 8g + e)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x2 w = {codes[2 * g], codes[2 * g + 1]};
                *reinterpret_cast<u32x2 *>(kdst + YVEX_ROCM_Q8_CODE_OFFSET(((g * 16u + t) * 4u + j) * 8u)) = w;
            }
        }
        // value codes: 4-byte groups (4 tokens of one dim), bytes 4b .. 4b+3 of the 32 that lane
        // 16 tg + m of a reading wave consumes, c = 16b + m
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t id = lane + 64u * i;  // 512 groups = tg (4) x m (16) x b (8)
            const uint32_t b = id & 7u, m = (id >> 3) & 15u, tg = id >> 7, c = 16u * b + m;
            if (4u * tg + 4u <= s.lo || 4u * tg >= s.hi) continue;
            uint32_t w = 0u;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t tt = 4u * tg + q;
                const bool fresh = tt >= s.lo && tt < s.hi;
                const uint32_t byte = fresh ? (uint32_t)v_codes[tt][c] : (old[i] >> (8 * q)) & 0xffu;
                w |= byte << (8 * q);
            }
            *reinterpret_cast<uint32_t *>(vdst + YVEX_ROCM_Q8_CODE_OFFSET(id * 4u)) = w;
        }
        // a block whose scale f16 cannot hold is refused like a non-finite value, as the
        // reference encoder refuses it (src/gguf/quant_block.c:172-174)
        if (!ok || !representable) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    }
}

// Token-major history writer: the reference appends the new tokens to a layer's history with
// two device copies per token, key then value, into rows of [K | V]
// (src/runtime/stateful_attention.c:183-222) after a separate rotary pass over the keys
// (src/runtime/decoder.c:1236-1242).  Here one launch does both: thread i owns the 16-byte
// piece (token, kv head, dims 8 * c8 .. 8 * c8 + 7) of the value row and of the key row, with
// the rotary roles and modes of the page writer (a lower-half piece produces its upper-half
// partner).  With a query tensor, threads behind the key/value pieces own the 16-byte pieces
// (token, query head) of it and rotate them where they lie, as the decoder rotates the
// queries in a pass of their own before attention (src/runtime/decoder.c:1235-1238): every
// location of the tensor is read and written by one thread only.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_history_append_bf16(const yvex_rocm_history_append_params p)
{
    const uint32_t pieces = p.head_dim / 8u, pairs = p.rotary_dim / 16u;
    const uint64_t id = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t total = (uint64_t)p.tokens * p.kv_heads * pieces;
    if (id >= total + (uint64_t)p.tokens * p.query_heads * pieces) return;
    const bool is_query = id >= total;
    const uint64_t local = is_query ? id - total : id;
    const uint32_t heads = is_query ? p.query_heads : p.kv_heads;
    const uint32_t c8 = (uint32_t)(local % pieces), head = (uint32_t)(local / pieces % heads);
    const uint32_t token = (uint32_t)(local / pieces / heads);
    const uint64_t in = ((uint64_t)token * heads + head) * p.head_dim + c8 * 8u;
    const uint64_t row = p.first_row + token;
    const uint16_t *key = is_query ? (const uint16_t *)p.query : (const uint16_t *)p.key;
    uint16_t *kdst = is_query ? (uint16_t *)p.query + in
                              : (uint16_t *)p.key_history + row * p.key_token_stride +
                                    (uint64_t)head * p.head_dim + c8 * 8u;
    KeyChunk k;
    k.t = 0u;
    k.c8 = c8;
    k.role = c8 < pairs ? kLower : c8 < 2u * pairs ? kUpper : kPlain;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (!is_query) v = load_b128((const uint16_t *)p.value + in);
    if (k.role != kUpper) k.own = load_b128(key + in);
    if (k.role == kLower) {
        const uint64_t at = (uint64_t)token * p.rotary_dim + c8 * 8u;
        k.other = load_b128(key + in + p.rotary_dim / 2u);
        k.cs[0] = load_b128(p.cosine + at);
        k.cs[1] = load_b128(p.cosine + at + 4);
        k.sn[0] = load_b128(p.sine + at);
        k.sn[1] = load_b128(p.sine + at + 4);
    }
    u32x4 lower, upper;
    bool ok = key_finish(k, lower, upper, p.rotary_mode != 0u) && finite_bits(v);
    if (!is_query)
        *reinterpret_cast<u32x4 *>((uint16_t *)p.value_history + row * p.value_token_stride +
                                   (uint64_t)head * p.head_dim + c8 * 8u) = v;
    if (k.role != kUpper) *reinterpret_cast<u32x4 *>(kdst) = lower;
    if (k.role == kLower) *reinterpret_cast<u32x4 *>(kdst + p.rotary_dim / 2u) = upper;
    if (!ok) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
}

namespace {

// a * b and c * d rounded to bf16, as floats
__device__ inline void rounded_products(float a, float b, float c, float d, float &ab, float &cd)
{
    const uint32_t w = pack_bf16x2(a * b, c * d);
    ab = low_half(w);
    cd = high_half(w);
}

__device__ inline bool finite_floats(const u32x4 &w)
{
    bool ok = true;
#pragma unroll
    for (int j = 0; j < 4; ++j) ok &= (w[j] & 0x7f800000u) != 0x7f800000u;
    return ok;
}

}  // namespace

// The F32 form of the history writer, for the histories the reference itself keeps (F32 rows,
// src/runtime/stateful_attention.c:183-222) and the EXACT_F32 kernels read.  Thread i owns the
// 16-byte piece (token, kv head, lanes 4 * c4 .. 4 * c4 + 3).  The rotary arithmetic is
// yvex_rotary_half_f32 (src/backend/cuda/transformer_kernels.cu:79-108): the F32 inputs enter
// the products as they are, every product and sum is rounded to bf16 and stored as F32.  In
// mode 1 (the decoder's order) the rotation is plain F32 and every key lane, the ones behind
// the rotary lanes included, is rounded to bf16 once; values are copied in both modes.
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_history_append_f32(const yvex_rocm_history_append_params p)
{
    const uint32_t pieces = p.head_dim / 4u, pairs = p.rotary_dim / 8u;
    const uint64_t id = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint64_t total = (uint64_t)p.tokens * p.kv_heads * pieces;
    if (id >= total + (uint64_t)p.tokens * p.query_heads * pieces) return;
    // pieces behind the key/value ones belong to the query tensor, rotated where it lies
    const bool is_query = id >= total;
    const uint64_t local = is_query ? id - total : id;
    const uint32_t heads = is_query ? p.query_heads : p.kv_heads;
    const uint32_t c4 = (uint32_t)(local % pieces), head = (uint32_t)(local / pieces % heads);
    const uint32_t token = (uint32_t)(local / pieces / heads);
    const uint64_t in = ((uint64_t)token * heads + head) * p.head_dim + c4 * 4u;
    const uint64_t row = p.first_row + token;
    const float *key = is_query ? (const float *)p.query : (const float *)p.key;
    float *kdst = is_query ? (float *)p.query + in
                           : (float *)p.key_history + row * p.key_token_stride +
                                 (uint64_t)head * p.head_dim + c4 * 4u;
    const int role = c4 < pairs ? kLower : c4 < 2u * pairs ? kUpper : kPlain;
    u32x4 own = {0u, 0u, 0u, 0u}, other = own, cs = own, sn = own, v = own;
    if (!is_query) v = load_b128((const float *)p.value + in);
    if (role != kUpper) own = load_b128(key + in);
    if (role == kLower) {
        const uint64_t at = (uint64_t)token * p.rotary_dim + c4 * 4u;
        other = load_b128(key + in + p.rotary_dim / 2u);
        cs = load_b128(p.cosine + at);
        sn = load_b128(p.sine + at);
    }
    bool ok = finite_floats(v);
    if (!is_query)
        *reinterpret_cast<u32x4 *>((float *)p.value_history + row * p.value_token_stride +
                                   (uint64_t)head * p.head_dim + c4 * 4u) = v;
    if (role == kPlain) {
        ok &= finite_floats(own);
        if (p.rotary_mode != 0u) {
            // the rounding pass of the decoder's order covers the lanes behind the rotary ones too
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const uint32_t a = own[j], b = own[j + 1];
                const uint32_t w = pack_bf16x2(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
                own[j] = w << 16;
                own[j + 1] = w & 0xffff0000u;
            }
        }
        *reinterpret_cast<u32x4 *>(kdst) = own;
    } else if (role == kLower) {
        u32x4 lower, upper;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // the elements go through scalars first: a bit cast applied directly to a vector
            // element reads element 0 whatever the index with this compiler
            const uint32_t own_j = own[j], other_j = other[j], cs_j = cs[j], sn_j = sn[j];
            const float first = __builtin_bit_cast(float, own_j), second = __builtin_bit_cast(float, other_j);
            const float cosine = __builtin_bit_cast(float, cs_j), sine = __builtin_bit_cast(float, sn_j);
            float fc, ss, sc, fs, lo, hi;
            if (p.rotary_mode != 0u) {
                rounded_products(__builtin_fmaf(first, cosine, -(second * sine)), 1.0f,
                                 __builtin_fmaf(second, cosine, first * sine), 1.0f, lo, hi);
            } else {
                rounded_products(first, cosine, second, sine, fc, ss);
                rounded_products(second, cosine, first, sine, sc, fs);
                rounded_products(fc - ss, 1.0f, sc + fs, 1.0f, lo, hi);
            }
            lower[j] = __builtin_bit_cast(uint32_t, lo);
            upper[j] = __builtin_bit_cast(uint32_t, hi);
        }
        // a non-finite input or table entry always leaves a non-finite result
        ok &= finite_floats(lower) && finite_floats(upper);
        *reinterpret_cast<u32x4 *>(kdst) = lower;
        *reinterpret_cast<u32x4 *>(kdst + p.rotary_dim / 2u) = upper;
    }
    if (!ok) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
}
