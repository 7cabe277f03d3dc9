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
// src/runtime/stateful_attention.c:326-352 are addressable): K and V rows are both read in
// 16-byte pieces; the V tile (16 tokens x 128 dims) is turned into the V^T operand through
// 4 KB of LDS private to the wave (ds_write_b128 of swizzled rows, ds_read_b64_tr_b16 back).
//
// Q8_0 paged layout, per (page, kv head): the canonical GGUF blocks (32 int8 codes and
// one f16 scale along the head dimension) are kept byte for byte but stored as
//     K codes  int8 [4 lane groups g][16 tokens][4 blocks j][8]     code(t, 32j+8g+e)
//     V codes  int8 [4 token groups][16 dims m][8 dim blocks b][4]  code(4tg+i, 16b+m)
//     scales   f16  [16 tokens][4 blocks]  after each 2048-byte code area
// so that every lane reads 32 contiguous bytes of codes.  Codes are widened to bf16 in
// registers (exact: |code| <= 127); a 32-wide MFMA covers exactly one quantisation
// block, so the K scale is applied to the fp32 partial dot per block, and the V scale
// is folded into the probabilities per 32-lane block before the second product.
//
// Work distribution: the (session, kv head, tile) items of the whole batch form one
// sequence that is cut into gridDim.x equal ranges, so every wave streams the same
// number of tiles whatever the mix of context lengths.  A wave that covers a whole
// (session, kv head) segment publishes its rows directly.  The waves of a split segment
// leave partials (running max in log2 units, sum, unnormalised accumulator) in the
// workspace.  Two ways to merge them, chosen by the host from the launch size:
//   * launches that do not fill the device are bound by launch latency, so the merge
//     happens in this kernel: each wave counts itself in on a per-segment arrival counter
//     and the wave that arrives last merges all partials of the segment in wave order (the
//     result does not depend on who was last) and publishes.  One launch.
//   * full-size launches use yvex_rocm_decode_finish as a second launch: with every SIMD
//     streaming, the device-scope stores, the counter and the merge's load trips at the end
//     of each wave cost more (measured +6..11 us on 190..275 us) than one more launch.
//   Visibility across the eight XCDs without a cache write-back per wave: the partials are
// written with device-scope write-through stores (sc1), the wave waits for them to complete
// (s_waitcnt vmcnt(0)) and only then adds to the counter with a device-scope atomic; the
// merging wave, after seeing the full count, reads them with device-scope loads (sc1), not
// through an L2 invalidate, which stalls the waves of the XCD that are still streaming.  The
// counters live in backend-owned memory that is zero between launches: the last arriver
// puts its counter back to zero.
// yvex_rocm_decode_merge is the stand-alone merge used by the per-chunk MLA path.
#include "mfma.h"
#include "device_scope.h"
#include "merge_rows.h"

#include "../kernel_params.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kPageTokens = 16;


__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

typedef __attribute__((address_space(3))) short4v lds_short4;
// LDS staging of a token-major V tile: row r (256 bytes at head dimension 128) keeps its
// 16-byte chunk c at position c ^ (r & 14), which spreads the 16 rows a transposed read
// touches over all banks (each 32-byte column segment is hit by exactly two rows).  A row of
// 64 lanes has eight chunks and swizzles over them (r & 6); one of 256 lanes swizzles within
// each half.
template <int kDim>
__device__ inline uint32_t vt_offset(int row, int chunk)
{
    return (uint32_t)(row * (kDim * 2) + ((chunk ^ (row & (kDim >= 128 ? 14 : 6))) << 4));
}

template <int kDim>
struct State {
    floatx4 o[kDim / 16];  // O^T[dim 16*b + 4*(lane/16) + i][head lane%16]
    float m, l;            // running max (log2 units) and per-lane partial sum
};

// Online-softmax step shared by every KV format: takes the scaled scores of the lane's
// four tokens (masked ones at -inf), updates (m, l), rescales the accumulators only when
// some lane of the wave saw a larger score (after the first tiles the running maximum
// rarely moves), and returns the four probabilities.
template <int kDim>
__device__ inline void softmax_step(State<kDim> &st, const float (&x)[4], float (&p)[4])
{
    float mloc = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
    mloc = max_xor32(max_xor16(mloc));
    const float m_new = fmaxf(st.m, mloc);
    if (__builtin_amdgcn_ballot_w64(m_new > st.m) != 0ull) {
        const float alpha = fast_exp2(st.m - m_new);
        st.l *= alpha;
#pragma unroll
        for (int b = 0; b < kDim / 16; ++b) st.o[b] *= alpha;
        st.m = m_new;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = fast_exp2(x[i] - st.m);
    st.l += (p[0] + p[1]) + (p[2] + p[3]);
}

// ---- bf16 KV --------------------------------------------------------------------
template <int kDim>
struct Bf16Tile {
    u32x4 k[kDim / 32];  // K[token = lane%16][32*j + 8*(lane/16) .. +7]
    u32x2 v[kDim / 16];  // paged: V[tokens 4*(lane/16)..+3][dim 16*b + lane%16]
                 // token-major: raw row chunks, (v[2j], v[2j+1]) = chunk e = 64 * j + lane of the tile,
                 // V[token e / (kDim / 8)][8 * (e % (kDim / 8)) .. +7]
};

// kHeadDimension: 128 is the tuned build (paged and token-major); 64 and 256 are the same
// paged code with other counts.
template <int kHeadDimension>
struct Bf16Kv {
    static constexpr int kDim = kHeadDimension;
    typedef Bf16Tile<kDim> Tile;
    static constexpr uint32_t kBlockBytes = kPageTokens * kDim * 2;

    __device__ static inline void load_paged(Tile &t, const unsigned char *kblock,
                                             const unsigned char *vblock, int lane)
    {
        const int n = lane & 15, g = lane >> 4;
        const uint16_t *k = (const uint16_t *)kblock, *v = (const uint16_t *)vblock;
#pragma unroll
        // Pages are read once per step and a batch's pages are far more than the caches hold:
        // non-temporal loads (config 3: 182 -> 165 us; head dimension 256: 237 -> 222 us).  At
        // head dimension 64 the 2 KB blocks came no faster that way (49.1 -> 50.3 us).
        for (int j = 0; j < kDim / 32; ++j)
            t.k[j] = kDim >= 128 ? stream_b128(k + (j * 64 + lane) * 8) : load_b128(k + (j * 64 + lane) * 8);
#pragma unroll
        for (int b = 0; b < kDim / 16; ++b)
            t.v[b] = kDim >= 128 ? stream_b64(v + (b * 16 + n) * 16 + g * 4) : load_b64(v + (b * 16 + n) * 16 + g * 4);
    }

    // rows_left: tokens available from `first` on (rows beyond are clamped to the last
    // valid row so no out-of-range address is formed; they are masked later).
    __device__ static inline void load_rows(Tile &t, const unsigned char *kbytes,
                                            const unsigned char *vbytes,
                                            const yvex_rocm_decode_params &p, uint32_t first,
                                            uint32_t rows_left, int lane)
    {
        constexpr int kChunks = kDim / 8;  // 16-byte chunks of a row
        const int n = lane & 15, g = lane >> 4;
        const uint16_t *k = (const uint16_t *)kbytes, *v = (const uint16_t *)vbytes;
        const uint32_t last = rows_left - 1u;
        const uint16_t *krow = k + (uint64_t)(first + min((uint32_t)n, last)) * p.k_token_stride;
#pragma unroll
        for (int j = 0; j < kDim / 32; ++j) t.k[j] = load_b128(krow + j * 32 + g * 8);
#pragma unroll
        for (int j = 0; j < kDim / 32; ++j) {
            const int e = 64 * j + lane;
            const uint16_t *vrow = v + (uint64_t)(first + min((uint32_t)(e / kChunks), last)) * p.v_token_stride;
            const u32x4 chunk = load_b128(vrow + (e % kChunks) * 8);
            t.v[2 * j] = (u32x2){chunk.x, chunk.y};
            t.v[2 * j + 1] = (u32x2){chunk.z, chunk.w};
        }
    }

    // Token-major tiles: the raw V rows go through the wave's LDS area and come back as the
    // V^T operand (lane (a, g) gets V[tokens 4g..4g+3][dim 16b + a]).  LDS operations of one
    // wave execute in order, so the area can be reused tile after tile without a barrier.
    __device__ static inline void transpose_rows(Tile &t, unsigned char *vt, int lane)
    {
        constexpr int kChunks = kDim / 8;
        const int a = lane & 15, g = lane >> 4;
#pragma unroll
        for (int j = 0; j < kDim / 32; ++j) {
            const int e = 64 * j + lane;
            const u32x4 chunk = {t.v[2 * j].x, t.v[2 * j].y, t.v[2 * j + 1].x, t.v[2 * j + 1].y};
            *reinterpret_cast<u32x4 *>(vt + vt_offset<kDim>(e / kChunks, e % kChunks)) = chunk;
        }
        const int row = 4 * g + (a >> 2);
#pragma unroll
        for (int b = 0; b < kDim / 16; ++b) {
            const short4v w = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (lds_short4 *)(vt + vt_offset<kDim>(row, 2 * b + ((a >> 1) & 1)) + 8 * (a & 1)));
            t.v[b] = __builtin_bit_cast(u32x2, w);
        }
    }

    // valid: number of real tokens in this 16-token tile (1..16).
    __device__ static inline void consume(State<kDim> &st, const Tile &t, const bf16x8 (&q)[kDim / 32],
                                          float scale_log2, uint32_t valid, int lane)
    {
        const int g = lane >> 4;
        floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < kDim / 32; ++j) s = mfma_16x16x32(as_bf16x8(t.k[j]), q[j], s);
        float x[4], p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            x[i] = (uint32_t)(g * 4 + i) < valid ? s[i] * scale_log2 : -INFINITY;
        softmax_step(st, x, p);
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
            for (int b = 0; b < kDim / 16; ++b) {
                u32x2 v = t.v[b];
                v.x &= keep_lo;
                v.y &= keep_hi;
                st.o[b] = mfma_16x16x16(as_short4(v), pv, st.o[b]);
            }
        } else {
#pragma unroll
            for (int b = 0; b < kDim / 16; ++b)
                st.o[b] = mfma_16x16x16(as_short4(t.v[b]), pv, st.o[b]);
        }
    }
};

// ---- Q8_0 KV ----------------------------------------------------------------------
struct Q8Tile {
    u32x4 kc[2];  // 32 K codes: token lane%16, dims 32j + 8*(lane/16) + e at byte 8j + e
    u32x4 ks[2];  // 16 f16 K scales: tokens 4*(lane/16)+i, block j at half index 4i + j
    u32x4 vc[2];  // 32 V codes: dim 16b + lane%16, tokens 4*(lane/16)+i at byte 4b + i
    u32x4 vs[2];  // 16 f16 V scales, same indexing as ks
};

// Sign-extends byte `k` of a word and widens it: exact for every int8 code.
__device__ inline float code_f32(uint32_t word, int k)
{
    return (float)((int32_t)(word << (24 - 8 * k)) >> 24);
}

__device__ inline float half_f32(uint32_t word, int hi)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(hi ? word >> 16 : word & 0xffffu));
}

struct Q8Kv {
    static constexpr int kDim = kHeadDim;
    typedef Q8Tile Tile;
    static constexpr uint32_t kCodeBytes = kPageTokens * kHeadDim;
    static constexpr uint32_t kBlockBytes = kCodeBytes + kPageTokens * (kHeadDim / 32) * 2;

    __device__ static inline void load_paged(Tile &t, const unsigned char *kblock,
                                             const unsigned char *vblock, int lane)
    {
        const int g = lane >> 4;
        // the two halves of a lane's 32 code bytes are 1 KB apart: each load is one contiguous KB
        t.kc[0] = stream_b128(kblock + lane * 16);
        t.kc[1] = stream_b128(kblock + lane * 16 + 1024);
        t.ks[0] = stream_b128(kblock + kCodeBytes + g * 32);
        t.ks[1] = stream_b128(kblock + kCodeBytes + g * 32 + 16);
        t.vc[0] = stream_b128(vblock + lane * 16);
        t.vc[1] = stream_b128(vblock + lane * 16 + 1024);
        t.vs[0] = stream_b128(vblock + kCodeBytes + g * 32);
        t.vs[1] = stream_b128(vblock + kCodeBytes + g * 32 + 16);
    }

    __device__ static inline void load_rows(Tile &, const unsigned char *, const unsigned char *,
                                            const yvex_rocm_decode_params &, uint32_t, uint32_t, int)
    {
    }
    __device__ static inline void transpose_rows(Tile &, unsigned char *, int) {}

    __device__ static inline void consume(State<kDim> &st, const Tile &t, const bf16x8 (&q)[4],
                                          float scale_log2, uint32_t valid, int lane)
    {
        const int g = lane >> 4;
        float x[4] = {0.f, 0.f, 0.f, 0.f}, p[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // block j: bytes 8j..8j+7 of the lane's 32 code bytes
            const uint32_t w0 = t.kc[j >> 1][(j & 1) * 2], w1 = t.kc[j >> 1][(j & 1) * 2 + 1];
            u32x4 a;
            a.x = pack_bf16x2_exact(code_f32(w0, 0), code_f32(w0, 1));
            a.y = pack_bf16x2_exact(code_f32(w0, 2), code_f32(w0, 3));
            a.z = pack_bf16x2_exact(code_f32(w1, 0), code_f32(w1, 1));
            a.w = pack_bf16x2_exact(code_f32(w1, 2), code_f32(w1, 3));
            const floatx4 s = mfma_16x16x32(as_bf16x8(a), q[j], (floatx4){0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int h = 4 * i + j;  // scale of (token 4g+i, block j)
                x[i] += half_f32(t.ks[h >> 3][(h >> 1) & 3], h & 1) * s[i];
            }
        }
        // only a context's last tile has tokens to mask: the full tile takes a path of its own
        // (wave-uniform), without the 20 selects per tile of the masked one
        const bool tail = valid < (uint32_t)kPageTokens;
        short4v pv[4];
        if (!tail) {
#pragma unroll
            for (int i = 0; i < 4; ++i) x[i] *= scale_log2;
            softmax_step(st, x, p);
            // fold the V scale of each 32-lane block into the probabilities
#pragma unroll
            for (int jb = 0; jb < 4; ++jb) {
                float w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int h = 4 * i + jb;
                    w[i] = p[i] * half_f32(t.vs[h >> 3][(h >> 1) & 3], h & 1);
                }
                u32x2 pb;
                pb.x = pack_bf16x2(w[0], w[1]);
                pb.y = pack_bf16x2(w[2], w[3]);
                pv[jb] = as_short4(pb);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                x[i] = (uint32_t)(g * 4 + i) < valid ? x[i] * scale_log2 : -INFINITY;
            softmax_step(st, x, p);
            // masked tokens get an exact zero whatever their (possibly garbage) scale bits are
#pragma unroll
            for (int jb = 0; jb < 4; ++jb) {
                float w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int h = 4 * i + jb;
                    w[i] = (uint32_t)(g * 4 + i) < valid ? p[i] * half_f32(t.vs[h >> 3][(h >> 1) & 3], h & 1) : 0.f;
                }
                u32x2 pb;
                pb.x = pack_bf16x2(w[0], w[1]);
                pb.y = pack_bf16x2(w[2], w[3]);
                pv[jb] = as_short4(pb);
            }
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const uint32_t w = t.vc[b >> 2][b & 3];
            u32x2 a;
            a.x = pack_bf16x2_exact(code_f32(w, 0), code_f32(w, 1));
            a.y = pack_bf16x2_exact(code_f32(w, 2), code_f32(w, 3));
            st.o[b] = mfma_16x16x16(as_short4(a), pv[b >> 1], st.o[b]);
        }
    }
};

__device__ inline uint32_t wave_inclusive_scan(uint32_t v, int lane)
{
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(v, off, 64);
        if (lane >= off) v += up;
    }
    return v;
}

// MERGE: split segments are merged in this kernel (arrival counters) instead of by
// yvex_rocm_decode_finish; a compile-time choice so that the full-size kernels carry none of
// the merge or gate code: with either present the compiler moves the tile bookkeeping of the
// streaming loop from scalar to vector registers and the paged bf16 kernel loses 4 %.
template <class Kv, bool PAGED, int kDepth, bool MERGE>
struct Decoder {
    static constexpr int kDim = Kv::kDim;
    typedef typename Kv::Tile Tile;
    typedef ::State<kDim> State;
    const yvex_rocm_decode_params &p;
    unsigned char *const vt;  // token-major layout: 4 KB of LDS for the V transposition
    const int lane, n, g;
    const uint32_t group, limit;

    __device__ Decoder(const yvex_rocm_decode_params &params, unsigned char *transpose_area)
        : p(params), vt(transpose_area), lane(threadIdx.x & 63), n(threadIdx.x & 15), g((threadIdx.x & 63) >> 4),
          group(params.query_heads / params.kv_heads),
          limit(PAGED ? params.table_stride * ((uint32_t)kPageTokens << params.page_shift)
                      : params.fixed_context)
    {
    }

    // context of a session, 0 when it is out of contract (flagged once, by wave 0)
    __device__ inline uint32_t context_of(uint32_t session) const
    {
        const uint32_t ctx = p.context ? (uint32_t)p.context[session] : p.fixed_context;
        if (ctx == 0u || ctx > limit) {
            if (blockIdx.x == 0u) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
            return 0u;
        }
        return ctx;
    }

    // Finds the session whose block of (tiles * kv_heads) work items contains `target`.
    // Returns false when target is at or past the end; `total` then holds the item count.
    __device__ inline bool locate(uint32_t target, uint32_t &session, uint32_t &offset,
                                  uint32_t &tiles, uint32_t &total) const
    {
        uint32_t carry = 0u;
        for (uint32_t base = 0u; base < p.sessions; base += 64u) {
            const uint32_t s = base + (uint32_t)lane;
            const uint32_t t = s < p.sessions ? (context_of(s) + kPageTokens - 1u) / kPageTokens : 0u;
            const uint32_t items = t * p.kv_heads;
            const uint32_t incl = wave_inclusive_scan(items, lane);
            const uint32_t excl = carry + incl - items;
            const uint64_t hit = __builtin_amdgcn_ballot_w64(items != 0u && target >= excl &&
                                                             target < excl + items);
            if (hit != 0ull) {
                const int src = __builtin_ctzll(hit);
                session = base + (uint32_t)src;
                offset = (uint32_t)__builtin_amdgcn_readlane((int)excl, src);
                tiles = (uint32_t)__builtin_amdgcn_readlane((int)t, src);
                return true;
            }
            carry += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        }
        total = carry;
        return false;
    }

    // Streams `count` (<= 128) tiles of (session, kv_head) starting at tile `first`.
    __device__ inline void stream(State &st, const bf16x8 (&q)[kDim / 32], uint32_t session,
                                  uint32_t kv_head, uint32_t ctx, uint32_t first,
                                  uint32_t count) const
    {
        const uint32_t t0 = first * kPageTokens;
        const uint32_t t1 = min(ctx, t0 + count * kPageTokens);
        int32_t my_page = 0, my_page_hi = 0;
        const unsigned char *kbase = (const unsigned char *)p.k_pool;
        const unsigned char *vbase = (const unsigned char *)p.v_pool;
        // a page holds 1 << shift tiles; tile i of this call is block (sub0 + i) of the pages
        // from the one that holds tile `first` on
        const uint32_t shift = PAGED ? p.page_shift : 0u, sub0 = first & ((1u << shift) - 1u);
        if (PAGED) {
            // two coalesced reads bring the page ids of these tiles into the wave
            const uint32_t pages = (sub0 + count + (1u << shift) - 1u) >> shift;
            const int32_t *table = p.page_table + (uint64_t)session * p.table_stride + (first >> shift);
            if ((uint32_t)lane < pages) my_page = table[lane];
            if ((uint32_t)lane + 64u < pages) my_page_hi = table[lane + 64];
            if (my_page < 0 || (uint32_t)my_page >= p.pool_pages || my_page_hi < 0 ||
                (uint32_t)my_page_hi >= p.pool_pages) {
                flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
                my_page = 0;
                my_page_hi = 0;
            }
        } else {
            kbase += (uint64_t)kv_head * kDim * 2u;
            vbase += (uint64_t)kv_head * kDim * 2u;
        }
        auto fetch = [&](Tile &t, uint32_t i) {
            if constexpr (PAGED) {
                const uint32_t at = sub0 + i, slot = at >> shift;
                const uint32_t page = (uint32_t)(slot < 64u
                                                     ? __builtin_amdgcn_readlane(my_page, (int)slot)
                                                     : __builtin_amdgcn_readlane(my_page_hi, (int)(slot - 64u)));
                const uint64_t off = ((((uint64_t)page * p.kv_heads + kv_head) << shift) +
                                      (at & ((1u << shift) - 1u))) * Kv::kBlockBytes;
                Kv::load_paged(t, kbase + off, vbase + off, lane);
            } else {
                const uint32_t row = t0 + i * kPageTokens;
                Kv::load_rows(t, kbase, vbase, p, row, t1 - row, lane);
            }
        };
        // Ring of kDepth tile buffers: kDepth-1 tiles stay in flight per wave while one is
        // consumed.  Every refill in the steady-state loop is unconditional (the index is
        // clamped to the last tile, a cache hit) so the number of outstanding loads is
        // the same on every trip and the waits the compiler places are partial
        // (vmcnt > 0) instead of draining the whole queue.
        Tile ring[kDepth];
        const uint32_t last_tile = count - 1u;
#pragma unroll
        for (int r = 0; r < kDepth; ++r) fetch(ring[r], min((uint32_t)r, last_tile));
        uint32_t i = 0u;
        for (; i + kDepth <= count; i += kDepth) {
#pragma unroll
            for (int r = 0; r < kDepth; ++r) {
                const uint32_t tile = i + (uint32_t)r;
                if constexpr (!PAGED) Kv::transpose_rows(ring[r], vt, lane);
                Kv::consume(st, ring[r], q, p.scale_log2,
                            min((uint32_t)kPageTokens, t1 - (t0 + tile * kPageTokens)), lane);
                fetch(ring[r], min(tile + kDepth, last_tile));
            }
        }
#pragma unroll
        for (int r = 0; r < kDepth - 1; ++r) {
            const uint32_t tile = i + (uint32_t)r;
            if (tile < count) {
                if constexpr (!PAGED) Kv::transpose_rows(ring[r], vt, lane);
                Kv::consume(st, ring[r], q, p.scale_log2,
                            min((uint32_t)kPageTokens, t1 - (t0 + tile * kPageTokens)), lane);
            }
        }
    }

    // Publishes normalised rows for the lane's head from a final (m, l, O^T) state.
    __device__ inline void publish(const State &st, float l, uint32_t session,
                                   uint32_t kv_head) const
    {
        if ((uint32_t)n >= group) return;
        const uint32_t head = kv_head * group + (uint32_t)n;
        const float inv = 1.0f / l;
        uint16_t *dst = p.out + ((uint64_t)session * p.query_heads + head) * kDim + g * 4;
        bool bad = false;
#pragma unroll
        for (int b = 0; b < kDim / 16; ++b) {
            const float a0 = st.o[b][0] * inv, a1 = st.o[b][1] * inv;
            const float a2 = st.o[b][2] * inv, a3 = st.o[b][3] * inv;
            bad |= !(isfinite(a0) && isfinite(a1) && isfinite(a2) && isfinite(a3));
            u32x2 w;
            w.x = pack_bf16x2(a0, a1);
            w.y = pack_bf16x2(a2, a3);
            if (MERGE && p.gate) {  // two-launch form: the finish kernel applies the gate
                w = gate_four(w, p.gate + (dst - p.out) + b * 16);
                bad |= pair_not_finite(w.x) || pair_not_finite(w.y);
            }
            *reinterpret_cast<u32x2 *>(dst + b * 16) = w;
        }
        if (bad) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        if (p.lse && g == 0)
            p.lse[(uint64_t)session * p.query_heads + head] = (st.m + fast_log2(l)) * YVEX_LN2;
    }

    // Leaves the wave's part of a split segment in its workspace slot.  With arrival counters
    // the stores are written through to device scope and the wave waits until they have
    // completed; without, the finish kernel reads them after this kernel has ended.
    __device__ inline void leave_partial(const State &st, float l, uint32_t wave, bool starts_here) const
    {
        if ((uint32_t)n < group) {
            // slot 1 when the segment starts inside this wave's range, else slot 0
            const uint64_t slot = ((uint64_t)wave * 2u + (starts_here ? 1u : 0u)) * group + n;
            float *acc = p.part_acc + slot * kDim + g * 4;
            if (MERGE) {
#pragma unroll
                for (int b = 0; b < kDim / 16; ++b) store_b128_device(acc + b * 16, st.o[b]);
                if (g == 0) store_b64_device(p.part_ml + slot * 2, st.m, l);
            } else {
#pragma unroll
                for (int b = 0; b < kDim / 16; ++b) *reinterpret_cast<floatx4 *>(acc + b * 16) = st.o[b];
                if (g == 0) {
                    p.part_ml[slot * 2 + 0] = st.m;
                    p.part_ml[slot * 2 + 1] = l;
                }
            }
        }
        if (MERGE) stores_completed();
    }

    // Log-sum-exp merge of the partials that waves w_first..w_last left for one segment, in
    // wave order, and publication of the rows.  Lane = (head hl of a block of four, dims
    // 8c..8c+7); kMergeWidth partials are in flight per trip (indices past the end alias the
    // last one with weight zero).
    __device__ inline void merge_segment(uint32_t session, uint32_t kv_head, uint32_t seg_begin,
                                         uint32_t per_wave, uint32_t w_first, uint32_t w_last) const
    {
        // the token-major kernel keeps a two-deep ring and has the registers for twice as many
        // partials in flight: a 4096-token context (32 partials per head) merges in two trips
        constexpr int kMergeWidth = PAGED ? 8 : 16;
        const uint32_t hl = (uint32_t)lane >> 4, c = (uint32_t)lane & 15u;
        for (uint32_t h0 = 0u; h0 < group; h0 += 4u) {
            const bool live = h0 + hl < group;
            const uint32_t hh = min(h0 + hl, group - 1u);
            float top = -INFINITY, sum = 0.f, acc[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = 0.f;
            for (uint32_t j0 = w_first; j0 <= w_last; j0 += (uint32_t)kMergeWidth) {
                // device-scope loads (sc1): they see the write-through stores of the other
                // XCDs without an L2 invalidate, which would stall the waves still streaming
                uint64_t ml[kMergeWidth], part[kMergeWidth][4];
#pragma unroll
                for (int i = 0; i < kMergeWidth; ++i) {
                    const uint32_t j = min(j0 + (uint32_t)i, w_last);
                    const uint64_t slot = ((uint64_t)j * 2u + (seg_begin >= j * per_wave ? 1u : 0u)) * group + hh;
                    const uint64_t *row = reinterpret_cast<const uint64_t *>(p.part_acc + slot * kHeadDim + c * 8u);
                    ml[i] = __hip_atomic_load(reinterpret_cast<const uint64_t *>(p.part_ml + slot * 2u),
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        part[i][e] = __hip_atomic_load(row + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                typedef float floatx2 __attribute__((ext_vector_type(2)));
                float m[kMergeWidth], l[kMergeWidth];
                float trip = -INFINITY;
#pragma unroll
                for (int i = 0; i < kMergeWidth; ++i) {
                    const floatx2 pair = __builtin_bit_cast(floatx2, ml[i]);  // (max, sum)
                    m[i] = j0 + (uint32_t)i > w_last ? -INFINITY : pair.x;  // past the end: weight zero
                    l[i] = pair.y;
                    trip = fmaxf(trip, m[i]);
                }
                const float m_new = fmaxf(top, trip);
                const float keep = fast_exp2(top - m_new);  // 0 on the first trip
                sum *= keep;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] *= keep;
#pragma unroll
                for (int i = 0; i < kMergeWidth; ++i) {
                    const float w = fast_exp2(m[i] - m_new);
                    sum += w * l[i];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const floatx2 two = __builtin_bit_cast(floatx2, part[i][e]);
                        acc[2 * e] += w * two.x;
                        acc[2 * e + 1] += w * two.y;
                    }
                }
                top = m_new;
            }
            if (!live) continue;
            const uint32_t head = kv_head * group + hh;
            const uint64_t at = ((uint64_t)session * p.query_heads + head) * kHeadDim + c * 8u;
            const float inv = 1.0f / sum;
            bool bad = false;
            u32x2 w0, w1;
            {
                const float a0 = acc[0] * inv, a1 = acc[1] * inv, a2 = acc[2] * inv, a3 = acc[3] * inv;
                const float a4 = acc[4] * inv, a5 = acc[5] * inv, a6 = acc[6] * inv, a7 = acc[7] * inv;
                bad |= !(isfinite(a0) && isfinite(a1) && isfinite(a2) && isfinite(a3) &&
                         isfinite(a4) && isfinite(a5) && isfinite(a6) && isfinite(a7));
                w0.x = pack_bf16x2(a0, a1);
                w0.y = pack_bf16x2(a2, a3);
                w1.x = pack_bf16x2(a4, a5);
                w1.y = pack_bf16x2(a6, a7);
            }
            if (p.gate) {
                w0 = gate_four(w0, p.gate + at);
                w1 = gate_four(w1, p.gate + at + 4);
                bad |= pair_not_finite(w0.x) || pair_not_finite(w0.y) || pair_not_finite(w1.x) ||
                       pair_not_finite(w1.y);
            }
            *reinterpret_cast<u32x4 *>(p.out + at) = (u32x4){w0.x, w0.y, w1.x, w1.y};
            if (bad) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
            if (p.lse && c == 0u)
                p.lse[(uint64_t)session * p.query_heads + head] = (top + fast_log2(sum)) * YVEX_LN2;
        }
    }

    // Wave 0 leaves the exclusive prefix of per-session work items (and the total at index
    // `sessions`) for the finish kernel.
    __device__ inline void publish_offsets(uint32_t total) const
    {
        uint32_t carry = 0u;
        for (uint32_t base = 0u; base < p.sessions; base += 64u) {
            const uint32_t s = base + (uint32_t)lane;
            const uint32_t t = s < p.sessions ? (context_of(s) + kPageTokens - 1u) / kPageTokens : 0u;
            const uint32_t items = t * p.kv_heads;
            const uint32_t incl = wave_inclusive_scan(items, lane);
            if (s < p.sessions) p.offsets[s] = carry + incl - items;
            carry += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        }
        if (lane == 0) p.offsets[p.sessions] = total;
    }

    __device__ inline void run() const
    {
        static_assert(kDim == 128 || (PAGED && !MERGE),
                      "other head dimensions: the two-launch paged form, or teams over token-major rows");
        const uint32_t wave = blockIdx.x, waves = gridDim.x;
        uint32_t session = 0u, offset = 0u, tiles = 0u, total = 0u;
        (void)locate(0xffffffffu, session, offset, tiles, total);
        if (wave == 0u && !MERGE) publish_offsets(total);
        if (total == 0u) return;
        const uint32_t per_wave = max((total + waves - 1u) / waves, p.min_tiles);
        uint32_t cur = wave * per_wave;
        if (cur >= total) return;
        const uint32_t end = min(total, cur + per_wave);
        while (cur < end) {
            if (!locate(cur, session, offset, tiles, total)) return;
            const uint32_t rel = cur - offset;
            const uint32_t kv_head = rel / tiles, first = rel % tiles;
            const uint32_t seg_begin = offset + kv_head * tiles, seg_end = seg_begin + tiles;
            const uint32_t stop = min(seg_end, end), count = stop - cur;
            const uint32_t ctx = context_of(session);

            bf16x8 q[kDim / 32];
            {
                const uint16_t *qrow = p.q + ((uint64_t)session * p.query_heads + kv_head * group +
                                              min((uint32_t)n, group - 1u)) * kDim;
#pragma unroll
                for (int j = 0; j < kDim / 32; ++j) {
                    u32x4 raw = load_b128(qrow + j * 32 + g * 8);
                    if ((uint32_t)n >= group) raw = (u32x4){0u, 0u, 0u, 0u};
                    q[j] = as_bf16x8(raw);
                }
            }
            State st;
#pragma unroll
            for (int b = 0; b < kDim / 16; ++b) st.o[b] = (floatx4){0.f, 0.f, 0.f, 0.f};
            st.m = -INFINITY;
            st.l = 0.f;
            for (uint32_t done = 0u; done < count; done += 128u)
                stream(st, q, session, kv_head, ctx, first + done, min(128u, count - done));

            float l = st.l;
            l = sum_xor32(sum_xor16(l));
            if (first == 0u && stop == seg_end) {
                publish(st, l, session, kv_head);  // the whole segment was ours
            } else {
                leave_partial(st, l, wave, first == 0u);
                if constexpr (!MERGE) {
                    cur = stop;
                    continue;  // the finish kernel merges
                } else {
                // count this wave in; whoever completes the count merges the segment
                const uint32_t w_first = seg_begin / per_wave, w_last = (seg_end - 1u) / per_wave;
                uint32_t *arrivals = p.arrivals + (uint64_t)session * p.kv_heads + kv_head;
                uint32_t before = 0u;
                if (lane == 0)
                    before = __hip_atomic_fetch_add(arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                before = (uint32_t)__builtin_amdgcn_readfirstlane((int)before);
                if (before == w_last - w_first) {
                    if (lane == 0)
                        __hip_atomic_store(arrivals, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    // no cache invalidate: the merge reads with device-scope loads; this only
                    // keeps the compiler from moving them above the count
                    loads_ordered();
                    merge_segment(session, kv_head, seg_begin, per_wave, w_first, w_last);
                }
                }
            }
            cur = stop;
        }
    }

    // ---- teams --------------------------------------------------------------------------
    // The form for a launch that is all latency (one query token per session over a
    // token-major history): a workgroup is a team of kTeam waves that share one stretch of
    // one (session, kv head) segment, kTeam times shorter chains of dependent loads per wave
    // than one wave per stretch would have, and merge their partials through LDS before the
    // team leaves ONE partial for the segment; the teams of a segment then merge as above
    // (arrival counter, last team merges in team order).  The exchange between workgroups --
    // write-through stores, the counter's round trip, the merge's load trip -- costs about
    // as much as the streaming itself, so it pays to have few, short parts on both levels.
    // grid = (teams per segment, kv_heads, sessions), block = 64 * kTeam; group <= 8.
    // team_lds: kTeam areas of 4 KB, a wave's V transposition first and its accumulators
    // ([group][128] F32) once it has streamed its tiles, then [kTeam][8][2] (max, sum).
    // At head dimension 256 a wave's tiles and accumulators take twice the registers: teams
    // of four waves, one per SIMD.
    static constexpr int kTeam = kDim > 128 ? 4 : 8;
    static constexpr uint32_t kTeamArea = kPageTokens * kDim * 2u / sizeof(float);  // floats
    static constexpr uint32_t kTeamLdsBytes = kTeam * (kPageTokens * kDim * 2u + 8u * 2u * sizeof(float));

    __device__ inline void run_team(float *parts) const
    {
        const uint32_t wave = threadIdx.x >> 6;
        const uint32_t team = blockIdx.x, teams = gridDim.x, kv_head = blockIdx.y, session = blockIdx.z;
        const uint32_t ctx = context_of(session);
        if (ctx == 0u) return;  // out of contract (flagged), for the whole workgroup alike
        const uint32_t tiles = (ctx + kPageTokens - 1u) / kPageTokens;
        const uint32_t per_wave = (tiles + teams * kTeam - 1u) / (teams * kTeam);
        const uint32_t first = min(tiles, (team * kTeam + wave) * per_wave);
        const uint32_t count = min(per_wave, tiles - first);

        bf16x8 q[kDim / 32];
        {
            const uint16_t *qrow = p.q + ((uint64_t)session * p.query_heads + kv_head * group +
                                          min((uint32_t)n, group - 1u)) * kDim;
#pragma unroll
            for (int j = 0; j < kDim / 32; ++j) {
                u32x4 raw = load_b128(qrow + j * 32 + g * 8);
                if ((uint32_t)n >= group) raw = (u32x4){0u, 0u, 0u, 0u};
                q[j] = as_bf16x8(raw);
            }
        }
        State st;
#pragma unroll
        for (int b = 0; b < kDim / 16; ++b) st.o[b] = (floatx4){0.f, 0.f, 0.f, 0.f};
        st.m = -INFINITY;
        st.l = 0.f;
        for (uint32_t done = 0u; done < count; done += 128u)
            stream(st, q, session, kv_head, ctx, first + done, min(128u, count - done));
        float l = st.l;
        l = sum_xor32(sum_xor16(l));

        // the wave's part into LDS (a wave without tiles leaves max -inf, sum 0, zeros)
        float *acc = parts, *ml = parts + kTeam * kTeamArea;
        if ((uint32_t)n < group) {
            float *row = acc + wave * kTeamArea + (uint32_t)n * kDim + g * 4;
#pragma unroll
            for (int b = 0; b < kDim / 16; ++b) *reinterpret_cast<floatx4 *>(row + b * 16) = st.o[b];
            if (g == 0) {
                ml[(wave * 8u + (uint32_t)n) * 2u] = st.m;
                ml[(wave * 8u + (uint32_t)n) * 2u + 1u] = l;
            }
        }
        __syncthreads();

        // the team's part: thread t merges (head, dim) pairs t, t + 64 * kTeam, ... over the waves,
        // in wave order
        const uint32_t values = group * kDim;
        const uint64_t segment = (uint64_t)session * p.kv_heads + kv_head;
        const uint64_t slot0 = (segment * teams + team) * group;
        const bool whole = teams == 1u;
        for (uint32_t at = threadIdx.x; at < values; at += 64u * kTeam) {
            const uint32_t hh = at / kDim, d = at % kDim;
            float top = -INFINITY;
#pragma unroll
            for (int w = 0; w < kTeam; ++w) top = fmaxf(top, ml[(w * 8u + hh) * 2u]);
            float sum = 0.f, o = 0.f;
#pragma unroll
            for (int w = 0; w < kTeam; ++w) {
                const float m = ml[(w * 8u + hh) * 2u];
                const float weight = m == -INFINITY ? 0.f : fast_exp2(m - top);
                sum += weight * ml[(w * 8u + hh) * 2u + 1u];
                o += weight * acc[w * kTeamArea + hh * kDim + d];
            }
            if (whole) {
                publish_value(session, kv_head * group + hh, d, o, sum, top);
            } else {
                __hip_atomic_store(p.part_acc + (slot0 + hh) * kDim + d, o, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                if (d == 0u) store_b64_device(p.part_ml + (slot0 + hh) * 2u, top, sum);
            }
        }
        if (whole) return;
        // every thread's stores have completed before the team is counted in
        stores_completed();
        __syncthreads();
        uint32_t *last = reinterpret_cast<uint32_t *>(parts);  // the LDS parts are done with
        if (threadIdx.x == 0u) {
            uint32_t *arrivals = p.arrivals + segment;
            const uint32_t before =
                __hip_atomic_fetch_add(arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before == teams - 1u)
                __hip_atomic_store(arrivals, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *last = before == teams - 1u ? 1u : 0u;
        }
        __syncthreads();
        if (*last == 0u) return;
        // the last team merges the segment's parts in team order; every load of a thread is
        // independent of the others (teams past the end alias the last one with weight
        // zero): one memory round trip per kTeamsPerTrip teams
        loads_ordered();
        constexpr uint32_t kTeamsPerTrip = 16u;
        // a thread takes kLanes neighbouring lanes of a head at a time: one at head dimension
        // 64 and 128, where a thread has one value or two in all; eight at 256, whose team of
        // four waves would otherwise walk up to eight values per thread, two dependent trips each
        constexpr uint32_t kLanes = kDim > 128 ? 8u : 1u;
        for (uint32_t at = threadIdx.x * kLanes; at < values; at += 64u * kTeam * kLanes) {
            const uint32_t hh = at / kDim, d = at % kDim;
            float top = -INFINITY, sum = 0.f, o[kLanes];
#pragma unroll
            for (uint32_t e = 0u; e < kLanes; ++e) o[e] = 0.f;
            for (uint32_t t0 = 0u; t0 < teams; t0 += kTeamsPerTrip) {
                float m[kTeamsPerTrip], part_l[kTeamsPerTrip], v[kTeamsPerTrip][kLanes];
#pragma unroll
                for (uint32_t i = 0u; i < kTeamsPerTrip; ++i) {
                    const uint64_t slot = (segment * teams + min(t0 + i, teams - 1u)) * group + hh;
                    load_b64_device(p.part_ml + slot * 2u, m[i], part_l[i]);
                    if constexpr (kLanes == 1u) {
                        v[i][0] = __hip_atomic_load(p.part_acc + slot * kDim + d, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
                    } else {
#pragma unroll
                        for (uint32_t e = 0u; e < kLanes; e += 2u)
                            load_b64_device(p.part_acc + slot * kDim + d + e, v[i][e], v[i][e + 1u]);
                    }
                }
                float trip = -INFINITY;
#pragma unroll
                for (uint32_t i = 0u; i < kTeamsPerTrip; ++i) {
                    if (t0 + i >= teams) m[i] = -INFINITY;
                    trip = fmaxf(trip, m[i]);
                }
                const float m_new = fmaxf(top, trip);
                const float keep = top == -INFINITY ? 0.f : fast_exp2(top - m_new);
                sum *= keep;
#pragma unroll
                for (uint32_t e = 0u; e < kLanes; ++e) o[e] *= keep;
#pragma unroll
                for (uint32_t i = 0u; i < kTeamsPerTrip; ++i) {
                    const float weight = m[i] == -INFINITY ? 0.f : fast_exp2(m[i] - m_new);
                    sum += weight * part_l[i];
#pragma unroll
                    for (uint32_t e = 0u; e < kLanes; ++e) o[e] += weight * v[i][e];
                }
                top = m_new;
            }
#pragma unroll
            for (uint32_t e = 0u; e < kLanes; ++e)
                publish_value(session, kv_head * group + hh, d + e, o[e], sum, top);
        }
    }

    // One normalised output value (and, from the thread of dim 0, the row's LSE).
    __device__ inline void publish_value(uint32_t session, uint32_t head, uint32_t d, float o, float sum,
                                         float top) const
    {
        const uint64_t at = ((uint64_t)session * p.query_heads + head) * kDim + d;
        float value = o / sum;
        if (p.gate) value = bf16_to_f32(bf16_bits(value)) * sigmoid(bf16_to_f32(p.gate[at]));
        if (!isfinite(value)) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
        p.out[at] = bf16_bits(value);
        if (p.lse && d == 0u)
            p.lse[(uint64_t)session * p.query_heads + head] = (top + fast_log2(sum)) * YVEX_LN2;
    }
};

}  // namespace

#define YVEX_DECODE_KERNEL(name, Kv, PAGED, DEPTH, MERGE) YVEX_DECODE_KERNEL_WAVES(name, Kv, PAGED, DEPTH, MERGE, 2)
#define YVEX_DECODE_KERNEL_WAVES(name, Kv, PAGED, DEPTH, MERGE, WAVES)                              \
    extern "C" __global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) \
    name(const yvex_rocm_decode_params p)                                                      \
    {                                                                                          \
        __shared__ __attribute__((aligned(16))) unsigned char vt[PAGED ? 16 : kPageTokens * kHeadDim * 2]; \
        Decoder<Kv, PAGED, DEPTH, MERGE>(p, vt).run();                                         \
    }

// full-size launches: partials for yvex_rocm_decode_finish
YVEX_DECODE_KERNEL(yvex_rocm_decode_paged_bf16, Bf16Kv<128>, true, 3, false)
YVEX_DECODE_KERNEL(yvex_rocm_decode_paged_q8_0, Q8Kv, true, 3, false)
YVEX_DECODE_KERNEL(yvex_rocm_decode_rows_bf16, Bf16Kv<128>, false, 2, false)
// head dimensions 64 and 256: paged bf16 pages only, always with the second launch (one wave
// per SIMD at 256, whose tiles and accumulators take twice the registers)
YVEX_DECODE_KERNEL(yvex_rocm_decode_paged_bf16_64, Bf16Kv<64>, true, 3, false)
YVEX_DECODE_KERNEL_WAVES(yvex_rocm_decode_paged_bf16_256, Bf16Kv<256>, true, 2, false, 1)
// launches that do not fill the device: merge in the kernel, one launch
YVEX_DECODE_KERNEL(yvex_rocm_decode_paged_bf16_merged, Bf16Kv<128>, true, 3, true)
YVEX_DECODE_KERNEL(yvex_rocm_decode_paged_q8_0_merged, Q8Kv, true, 3, true)
YVEX_DECODE_KERNEL(yvex_rocm_decode_rows_bf16_merged, Bf16Kv<128>, false, 2, true)

// teams of waves over a token-major history (see Decoder::run_team): eight waves, two per
// SIMD; four, one per SIMD, at head dimension 256
#define YVEX_DECODE_TEAM_KERNEL(name, head_dim, THREADS, WAVES)                                      \
    extern "C" __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) \
    name(const yvex_rocm_decode_params p)                                                      \
    {                                                                                          \
        typedef Decoder<Bf16Kv<head_dim>, false, 2, true> Team;                                \
        static_assert(THREADS == 64 * Team::kTeam, "one workgroup is one team");               \
        __shared__ __attribute__((aligned(16))) unsigned char team_lds[Team::kTeamLdsBytes];   \
        const uint32_t wave = threadIdx.x >> 6;                                                \
        Team(p, team_lds + wave * (kPageTokens * head_dim * 2)).run_team(reinterpret_cast<float *>(team_lds)); \
    }

YVEX_DECODE_TEAM_KERNEL(yvex_rocm_decode_rows_bf16_team, 128, 512, 2)
YVEX_DECODE_TEAM_KERNEL(yvex_rocm_decode_rows_bf16_team_64, 64, 512, 2)
YVEX_DECODE_TEAM_KERNEL(yvex_rocm_decode_rows_bf16_team_256, 256, 256, 1)

// Merge of the split segments of the balanced decode when the decode kernel was launched
// without arrival counters (large launches).  grid = (query_heads, sessions), block =
// head_dim threads (one per output lane).  A segment that one wave covered was already
// published by that wave and is skipped.
__device__ __forceinline__ void decode_finish(const yvex_rocm_decode_params &p)
{
    const uint32_t head = blockIdx.x, session = blockIdx.y, d = threadIdx.x;
    const uint32_t group = p.query_heads / p.kv_heads;
    const uint32_t offset = p.offsets[session], next = p.offsets[session + 1u];
    const uint32_t total = p.offsets[p.sessions];
    const uint32_t tiles = (next - offset) / p.kv_heads;
    if (tiles == 0u || d >= p.head_dim) return;
    const uint32_t per_wave = max((total + p.waves - 1u) / p.waves, p.min_tiles);
    const uint32_t kv_head = head / group, hh = head % group;
    const uint32_t seg_begin = offset + kv_head * tiles, seg_end = seg_begin + tiles;
    const uint32_t w_first = seg_begin / per_wave, w_last = (seg_end - 1u) / per_wave;
    if (w_first == w_last) {
        // published by the decode kernel itself; only the output gate is left to apply
        if (p.gate) {
            const uint64_t at = ((uint64_t)session * p.query_heads + head) * p.head_dim + d;
            const float o = bf16_to_f32(p.out[at]) * sigmoid(bf16_to_f32(p.gate[at]));
            if (!isfinite(o)) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
            p.out[at] = bf16_bits(o);
        }
        return;
    }
    auto slot_of = [&](uint32_t j) -> uint64_t {
        return ((uint64_t)j * 2u + (seg_begin >= j * per_wave ? 1u : 0u)) * group + hh;
    };
    // kWidth parts at a time: all loads of a trip are independent and in flight together
    // (indices past the end alias the last part with weight zero).  A 16384-token context is
    // cut into at most 17 parts when 2048 waves share the work of 32 such sessions, so one
    // trip, one memory round trip, covers every segment of the full-size launches (widths 8
    // and 16 take three and two trips there and measure 1.4 and 4 us slower per step).
    constexpr int kWidth = 24;
    float top = -INFINITY, sum = 0.f, acc = 0.f;
    for (uint32_t j0 = w_first; j0 <= w_last; j0 += (uint32_t)kWidth) {
        float m[kWidth], l[kWidth], v[kWidth];
#pragma unroll
        for (int i = 0; i < kWidth; ++i) {
            const uint64_t slot = slot_of(min(j0 + (uint32_t)i, w_last));
            m[i] = p.part_ml[slot * 2u];
            l[i] = p.part_ml[slot * 2u + 1u];
            v[i] = p.part_acc[slot * p.head_dim + d];
        }
        float trip = -INFINITY;
#pragma unroll
        for (int i = 0; i < kWidth; ++i) {
            if (j0 + (uint32_t)i > w_last) m[i] = -INFINITY;
            trip = fmaxf(trip, m[i]);
        }
        const float m_new = fmaxf(top, trip);
        const float keep = fast_exp2(top - m_new);
        sum *= keep;
        acc *= keep;
#pragma unroll
        for (int i = 0; i < kWidth; ++i) {
            const float w = fast_exp2(m[i] - m_new);
            sum += w * l[i];
            acc += w * v[i];
        }
        top = m_new;
    }
    float o = acc / sum;
    const uint64_t at = ((uint64_t)session * p.query_heads + head) * p.head_dim + d;
    if (p.gate) o = bf16_to_f32(bf16_bits(o)) * sigmoid(bf16_to_f32(p.gate[at]));
    if (!isfinite(o)) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    p.out[at] = bf16_bits(o);
    if (p.lse && d == 0u)
        p.lse[(uint64_t)session * p.query_heads + head] = (top + fast_log2(sum)) * YVEX_LN2;
}

extern "C" __global__ void __launch_bounds__(128)
yvex_rocm_decode_finish(const yvex_rocm_decode_params p)
{
    decode_finish(p);
}

// head dimension 256: a block of 256 threads
extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_decode_finish_256(const yvex_rocm_decode_params p)
{
    decode_finish(p);
}

// Log-sum-exp merge of the chunk partials of one (session, query head): one wave per head,
// eight output dims per lane (one 16-byte load of bf16 partials per chunk), four heads per
// workgroup.  grid = (ceil(query_heads / 4), sessions), block = 256; head_dim = 512.
// kRope: the build that also turns the rope lanes of the published row back (its double
// precision sine and cosine double the register use, so rows without a rotation keep their
// own build).
template <bool kRope>
__device__ __forceinline__ void decode_merge_rows(const yvex_rocm_decode_merge_params &p)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t head = blockIdx.x * 4u + (threadIdx.x >> 6), session = blockIdx.y;
    const uint32_t ctx = p.context ? (uint32_t)p.context[session] : p.fixed_context;
    if (ctx == 0u || head >= p.query_heads || lane * 8u >= p.head_dim) return;
    const uint32_t first_visible = p.window != 0u && ctx > p.window ? ctx - p.window : 0u;
    const uint32_t live = ctx - (first_visible & ~(p.window_align - 1u));
    const uint32_t own = min(p.max_chunks, (live + p.chunk_tokens - 1u) / p.chunk_tokens);
    // the chunks of a second candidate set follow the max_chunks slots of the first
    const uint32_t extra_ctx = p.extra_context ? (uint32_t)p.extra_context[session] : 0u;
    const uint32_t extra = p.extra_context
        ? min(p.extra_max_chunks, (extra_ctx + p.extra_chunk_tokens - 1u) / p.extra_chunk_tokens) : 0u;
    const uint32_t chunks = own + extra, skip = p.max_chunks - own;
    const uint64_t base =
        ((uint64_t)session * (p.max_chunks + (p.extra_context ? p.extra_max_chunks : 0u))) * p.query_heads + head;
    float top, total, acc[8];
    merge_chunk_rows(
        chunks,
        [&](uint32_t c, float &m, float &l) {
            const uint64_t slot = base + (uint64_t)(c < own ? c : c + skip) * p.query_heads;
            m = p.part_ml[slot * 2];
            l = p.part_ml[slot * 2 + 1];
        },
        [&](uint32_t c) {
            const uint64_t slot = base + (uint64_t)(c < own ? c : c + skip) * p.query_heads;
            return load_b128(p.part_acc + slot * p.head_dim + lane * 8u);
        },
        top, total, acc);
    bool bad = false;
    if (p.sinks) bad |= !merge_sink(p.sinks[head], top, total, acc);
    const float inv = 1.0f / total;
    // Inverse rotation of the rope lanes (src/graph/core.c:499-507): the row is rounded to
    // bf16, its last rope_dims lanes are turned back by the token position in adjacent pairs,
    // in double as the reference does it (src/graph/numeric.c:935-947), and rounded again.  A
    // lane's eight dims hold four whole pairs; rope_dims and head_dim are multiples of 8.
    const uint32_t rope_start = p.head_dim - p.rope_dims;
    const bool turn = kRope && p.rope_dims != 0u && lane * 8u >= rope_start;
    const double position =
        turn ? (p.positions ? (double)(uint64_t)p.positions[session] : (double)(ctx - 1u)) : 0.0;
    u32x4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float a = acc[2 * i] * inv, b = acc[2 * i + 1] * inv;
        bad |= !(isfinite(a) && isfinite(b));
        if (kRope && turn) {
            // products and sums rounded one by one, as the C reference computes them
            // (src/graph/numeric.c:935-947 is built without contraction)
#pragma clang fp contract(off)
            const double angle = position * p.rope_frequency[(lane * 8u - rope_start) / 2u + (uint32_t)i];
            const double c = cos(angle), s = -sin(angle);
            const double x = (double)bf16_to_f32(bf16_bits(a)), y = (double)bf16_to_f32(bf16_bits(b));
            a = (float)(x * c - y * s);
            b = (float)(x * s + y * c);
            bad |= !(isfinite(a) && isfinite(b));
        }
        out[i] = (uint32_t)bf16_bits(a) | ((uint32_t)bf16_bits(b) << 16);
    }
    if (bad) flag(p.status, YVEX_ROCM_DEVICE_NUMERIC);
    *reinterpret_cast<u32x4 *>(p.out + ((uint64_t)session * p.query_heads + head) * p.head_dim +
                               lane * 8u) = out;
    if (p.lse && lane == 0u)
        p.lse[(uint64_t)session * p.query_heads + head] = (top + fast_log2(total)) * YVEX_LN2;
}

extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_decode_merge(const yvex_rocm_decode_merge_params p)
{
    decode_merge_rows<false>(p);
}

extern "C" __global__ void __launch_bounds__(256)
yvex_rocm_decode_merge_rope(const yvex_rocm_decode_merge_params p)
{
    decode_merge_rows<true>(p);
}
