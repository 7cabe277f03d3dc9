// Causal / full grouped-query attention prefill for gfx950 (wave64), bf16 in and out,
// fp32 scores, online softmax and accumulation.  Token-major tensors ([token][head][dim],
// per-token strides in elements); head_dim 128 is the tuned build, 64 and 256 are the same
// code with other counts (the numbers in this comment are those of 128).
//
// A workgroup of 4 waves owns one (query head, 128-row query tile): each wave owns
// 32 query rows and walks the key/value tokens in tiles of 64 that the workgroup
// stages in LDS once and all four waves share.  Two workgroups are resident per CU; they
// are not synchronised with each other, so the serial part of one trip (barrier, maximum
// bookkeeping) of one overlaps the matrix work of the other.
// Both products are computed transposed so the probabilities never leave registers:
//     S^T[key][query] = K[key][:] . Q[query][:]        v_mfma_f32_32x32x16_bf16, A = K (LDS)
//     O^T[dim][query] += V^T[dim][key] . P^T[key][query]                A = V^T (LDS)
// The accumulator layout of S^T (lane = query row, 16 key rows per lane) is the B-operand
// layout of the second product once the 16-key K-slices are taken as accumulator
// registers 8u..8u+7; V^T is fetched from LDS in the matching key order.  Softmax
// statistics are per lane (= per query row) plus one exchange with lane^32.
//
// Software pipeline.  The matrix pipe and the vector ALU of a SIMD only overlap when their
// instructions alternate finely in one wave's stream (measured: up to seven 4-cycle vector
// instructions ride behind one 32-cycle MFMA almost for free; phases of MFMAs followed by
// phases of vector work simply add up, also across the two waves of a SIMD).  So one trip
// of the main loop issues 32 MFMAs -- the 16 of S^T for tile t+1, then the 16 of the O^T
// update with tile t -- and behind each of them a slice of the softmax of tile t (scale,
// exp2, bf16 pack, row sums: the scores of tile t were produced one trip earlier), the
// running maximum of tile t+1 once its scores are complete, one LDS operand fetch four
// MFMAs ahead of its use, and in the first eight slots one of the eight LDS-DMA loads of a
// later tile.  The order is pinned slot by slot with scheduling barriers.
//
// LDS layout: two buffers, each a K tile and a V tile of [64 keys][128 dims] bf16 in
// row-major order with 256-byte rows and no padding; the 16-byte chunk c of row r sits at
// chunk position c ^ x(r), x(r) = ((r & 3) << 2) | ((r >> 2) & 3).  That makes both operand
// fetches bank-conflict free: the K operand is one ds_read_b128 per lane (16 rows x one
// chunk column hit 16 distinct chunk positions), the V^T operand is two ds_read_b64_tr_b16
// (each 16-lane group transposes 4 keys x 16 dims; 4 consecutive rows place one 64-byte
// column segment in 4 distinct bank groups).  Tile t uses buffer t % 2 for both;
// while trip t reads K(t+1) and V(t), K(t+2) and V(t+1) are in flight into the halves that
// trip t-1 finished with, so one workgroup barrier per trip is enough.
// The tiles are filled by buffer loads that write LDS directly (no staging registers,
// no LDS store instructions): lane L of a 1 KB load owns chunk position L % 16 of row
// L / 16 and fetches the global chunk that belongs there.  Rows past the end of the
// tensor read as zero through the buffer range check.
//
// The running maximum is only raised when a tile exceeds it by more than kLazyLog2 (in
// log2 units), so the accumulator rescale is rare; probabilities are then at most
// 2^kLazyLog2, harmless in fp32 sums and in the bf16 operand of the second product.
// Row sums are taken over the unrounded fp32 probabilities: with a handful of visible keys
// the rounding of single bf16 terms would show in the log-sum-exp output.
// Workgroups are numbered so that heavier (later) query tiles start first and, when the
// kv head count is a multiple of the 8 XCDs, all users of one kv head share an L2.
//
#include "mfma.h"

#include "../kernel_params.h"

namespace {

constexpr int kKeyTile = 64;
constexpr float kLazyLog2 = 8.0f;
constexpr int kRowsPerWave = 32;
constexpr int kRowsPerBlock = 4 * kRowsPerWave;
constexpr int kDepth = 4;  // operand fetches in flight ahead of the MFMA that consumes them

typedef __attribute__((address_space(3))) short4v lds_short4;

// Chunk swizzle of tile row r: the 16-byte chunk c of the row sits at chunk position c ^ x(r).
// Rows of 256 and of 512 bytes all start in the same bank, x(r) permutes the 16 chunk
// positions of a 256-byte bank span by the row's low four bits (rows r..r+3 go four chunks
// apart, which is what the transposed read needs; 16 consecutive rows take 16 different
// positions, which is what the row read needs).  Rows of 128 bytes (head_dim 64) alternate
// between the two halves of a bank span, so the row's bit 0 already separates them and x(r)
// permutes the eight chunk positions of a half by bits 1..3: bit 1 moves a row by four
// chunks (two 32-byte column segments, so that the segments the two dim halves of a
// transposed read touch stay apart), bits 2 and 3 by two and one.
template <int D>
__device__ inline int swizzle(int r)
{
    return D == 64 ? ((((r >> 1) & 1) << 2) | (((r >> 2) & 1) << 1) | ((r >> 3) & 1))
                   : (((r & 3) << 2) | ((r >> 2) & 3));
}

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

// The value the lane 32 away holds (the two key halves of a query row): v_permlane32_swap
// on the vector ALU instead of a round trip through the LDS permute network.
__device__ inline float other_half(float v)
{
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const u32x2 r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    // r.x holds the lower half's value in every lane, r.y the upper half's
    return __builtin_bit_cast(float, (threadIdx.x & 32u) ? r.x : r.y);
}

template <int kHeadDim>
struct Prefill {
    static constexpr int kRowBytes = kHeadDim * 2;            // 256
    static constexpr int kRowChunks = kRowBytes / 16;         // 16-byte chunks of a row
    static constexpr int kTileBytes = kKeyTile * kRowBytes;   // 16384 per K or V tile
    static constexpr int kBufBytes = 2 * kTileBytes;          // K then V
    static constexpr int kSteps = kHeadDim / 16;              // k-steps of S^T per 32-key half
    static constexpr int kDimBlocks = kHeadDim / 32;          // 32-dim blocks of O^T
    static constexpr int kHalfSlots = 2 * kSteps;             // MFMAs of S^T (= of the O^T update) per trip
    static constexpr int kSlots = 2 * kHalfSlots;
    static constexpr int kLoads = kTileBytes / 1024 / 4;      // 1 KB loads per wave and K or V tile
    static constexpr int kLoadRows = 64 / kRowChunks;         // tile rows one 1 KB load covers
    static constexpr int kSoftmaxSlots = 3 * kSlots / 4;      // the exponentials ride behind these slots
    static constexpr int kMaxPerSlot = 32 / (kSlots - kSoftmaxSlots);
    static_assert(kHeadDim == 64 || kHeadDim == 128 || kHeadDim == 256, "head_dim 64, 128 or 256");

    const yvex_rocm_prefill_params &p;
    unsigned char *const lds;
    const int lane, wave, n, g;
    uint32_t head, kv_head, row0;
    // staging
    i32x4 k_rsrc, v_rsrc;
    uint32_t k_row_bytes, v_row_bytes, lds_base, k_off[kLoads], v_off[kLoads];
    // operand addresses inside a buffer
    uint32_t k_addr[kSteps], v_addr[kDimBlocks][2];
    bf16x8 q[kSteps];
    floatx16 o[kDimBlocks];
    float m_run, neg_m, l_run;

    __device__ Prefill(const yvex_rocm_prefill_params &params, unsigned char *shared)
        : p(params), lds(shared), lane(threadIdx.x & 63),
          wave(__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)), n(threadIdx.x & 31),
          g((threadIdx.x & 63) >> 5)
    {
    }

    // 1 KB load j (0..kLoads-1) of this wave for the K or V tile `tile` into buffer `buf`.  A tile
    // that is not wanted is still "loaded", from an offset past the range of the descriptor:
    // the range check returns zeros without touching memory, and the trip stays branch-free
    // with the same number of loads in flight.
    __device__ inline void stage_k(uint32_t tile, bool wanted, int buf, int j) const
    {
        lds_dma_b128(lds_base + buf * kBufBytes + wave * (16 * kRowBytes) + j * 1024, k_rsrc, k_off[j],
                     (uint32_t)__builtin_amdgcn_readfirstlane(
                         (int)(wanted ? tile * kKeyTile * k_row_bytes : 0xfffffff0u)));
    }
    __device__ inline void stage_v(uint32_t tile, bool wanted, int buf, int j) const
    {
        lds_dma_b128(lds_base + buf * kBufBytes + kTileBytes + wave * (16 * kRowBytes) + j * 1024, v_rsrc,
                     v_off[j],
                     (uint32_t)__builtin_amdgcn_readfirstlane(
                         (int)(wanted ? tile * kKeyTile * v_row_bytes : 0xfffffff0u)));
    }

    // K operand of S^T MFMA i (i = kk * 2 + mb): rows mb*32 + n, dims 16kk + 8g .. +7
    __device__ inline u32x4 fetch_k(const unsigned char *buf, int i) const
    {
        return *reinterpret_cast<const u32x4 *>(buf + k_addr[i >> 1] + (i & 1) * 32 * kRowBytes);
    }
    // V^T operand of O^T MFMA i (i = (mb * 2 + u) * kDimBlocks + db): dims db*32 .., keys mb*32 + 16u ..
    __device__ inline u32x4 fetch_v(const unsigned char *buf, int i) const
    {
        const int db = i % kDimBlocks, grp = i / kDimBlocks;
        const int base = ((grp >> 1) * 32 + (grp & 1) * 16) * kRowBytes;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4 *)(buf + v_addr[db][0] + base));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4 *)(buf + v_addr[db][1] + base));
        return __builtin_bit_cast(u32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }

    // Masks the keys of tile `tile` that the lane's row does not see (causal diagonal, end of
    // the tensor).
    __device__ inline void mask_tile(floatx16 (&s)[2], uint32_t tile) const
    {
        const uint32_t key0 = tile * kKeyTile, row = row0 + n;
        const uint32_t vis = p.causal ? min(p.query_start + row, p.kv_tokens - 1u) : p.kv_tokens - 1u;
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t key = key0 + mb * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
                if (key > vis) s[mb][i] = -INFINITY;
            }
    }

    // Raises the running maximum when the tile whose per-lane maximum is `mloc` (raw score
    // units) needs it, rescaling what has been accumulated so far.
    __device__ inline void settle(float mloc)
    {
        mloc = fmaxf(mloc, other_half(mloc)) * p.scale_log2;
        if (__builtin_amdgcn_ballot_w64(mloc > m_run + kLazyLog2) != 0ull) {
            const float m_new = fmaxf(m_run, mloc);
            // a row that has seen nothing yet keeps m = -inf: guard the subtraction
            const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db) o[db] *= alpha;
            m_run = m_new;
            neg_m = m_new == -INFINITY ? 0.f : -m_new;
        }
    }

    __device__ inline float tile_max(const floatx16 (&s)[2]) const
    {
        float m = -INFINITY;
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int i = 0; i < 16; i += 2) m = fmaxf(m, fmaxf(s[mb][i], s[mb][i + 1]));
        return m;
    }

    __device__ inline void run()
    {
        // heavier (later) query tiles are dispatched first; id % kv_heads picks the kv head
        const uint32_t q_tiles = (p.query_tokens + kRowsPerBlock - 1) / kRowsPerBlock;
        const uint32_t q_tile = q_tiles - 1u - blockIdx.x / p.query_heads;
        const uint32_t in_tile = blockIdx.x % p.query_heads;
        kv_head = in_tile % p.kv_heads;
        head = kv_head * (p.query_heads / p.kv_heads) + in_tile / p.kv_heads;
        row0 = q_tile * kRowsPerBlock + wave * kRowsPerWave;  // first row of this wave

        // keys visible to the last row of the workgroup bound the walk
        const uint32_t block_last_row = min(p.query_tokens, (q_tile + 1u) * kRowsPerBlock) - 1u;
        const uint32_t kv_end = p.causal ? min(p.kv_tokens, p.query_start + block_last_row + 1u)
                                         : p.kv_tokens;
        const uint32_t all_tiles = (kv_end + kKeyTile - 1) / kKeyTile;
        const uint32_t tiles = all_tiles;

        // ---- Q fragments: B operand, lane (n, g) holds Q[row n][16*kk + 8g .. +7] ----
        {
            const uint32_t row = min(row0 + n, p.query_tokens - 1u);
            const uint16_t *src = p.q + (uint64_t)row * p.q_stride + (uint64_t)head * kHeadDim + g * 8;
#pragma unroll
            for (int kk = 0; kk < kSteps; ++kk) q[kk] = as_bf16x8(load_b128(src + kk * 16));
        }

        // ---- tile staging: buffer loads that write LDS directly -----------------------
        // 1 KB load j of wave w fills rows 16w + 4j .. +3 of the tile; lane L owns chunk
        // position L % 16 of row 16w + 4j + L / 16 and fetches chunk (L % 16) ^ x(row)
        // (rows of 128 bytes: eight rows per load, of 512 bytes: two).
        k_row_bytes = (uint32_t)p.k_stride * 2u;
        v_row_bytes = (uint32_t)p.v_stride * 2u;
        k_rsrc = raw_buffer(p.k + (uint64_t)kv_head * kHeadDim,
                            p.kv_tokens * k_row_bytes - kv_head * kRowBytes);
        v_rsrc = raw_buffer(p.v + (uint64_t)kv_head * kHeadDim,
                            p.kv_tokens * v_row_bytes - kv_head * kRowBytes);
        lds_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_address_of(lds));
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            const int r = 16 * wave + kLoadRows * j + lane / kRowChunks;
            const uint32_t chunk = (uint32_t)((lane % kRowChunks) ^ swizzle<kHeadDim>(r));
            k_off[j] = (uint32_t)r * k_row_bytes + chunk * 16u;
            v_off[j] = (uint32_t)r * v_row_bytes + chunk * 16u;
        }

        // ---- operand addresses inside a buffer ----------------------------------------
        // K operand (mb, kk): row mb*32 + n, chunk (2kk + g) ^ x(n); one address per kk
#pragma unroll
        for (int kk = 0; kk < kSteps; ++kk)
            k_addr[kk] = (uint32_t)(n * kRowBytes + (((2 * kk + g) ^ swizzle<kHeadDim>(n)) << 4));
        // V^T operand (db, mb, u, h): 16-lane group b = lane / 16 (dims 16 * (b & 1), key half
        // g = b / 2), lane a = lane % 16 addresses key row mb*32 + 16u + 8h + 4g + a/4 and
        // dims db*32 + 16*(b&1) + 4*(a%4) .. +3; one address per (db, h)
        {
            const int a = lane & 15, b1 = (lane >> 4) & 1;
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int r = 8 * h + 4 * g + (a >> 2);
                    const int chunk = (db * 4 + 2 * b1 + ((a >> 1) & 1)) ^ swizzle<kHeadDim>(r);
                    v_addr[db][h] = (uint32_t)(kTileBytes + r * kRowBytes + (chunk << 4) + 8 * (a & 1));
                }
        }

#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
        m_run = -INFINITY;
        neg_m = 0.f;
        l_run = 0.f;

        // rows of this wave at or past query_tokens do no work but still help staging
        const bool wave_active = row0 < p.query_tokens;
        // last key visible to the wave's first / last row (causal)
        const uint32_t wave_first_vis = p.causal ? p.query_start + row0 : p.kv_tokens - 1u;
        const uint32_t wave_last_vis =
            p.causal ? p.query_start + min(row0 + kRowsPerWave, p.query_tokens) - 1u : p.kv_tokens - 1u;
        // tiles this wave computes with: those that hold a key one of its rows sees
        const uint32_t my_tiles = wave_active ? min(tiles, wave_last_vis / kKeyTile + 1u) : 0u;
        auto needs_mask = [&](uint32_t tile) {
            return tile * kKeyTile + kKeyTile - 1u > wave_first_vis || (tile + 1u) * kKeyTile > p.kv_tokens;
        };

        // ---- prologue: K(0) and V(0) land, K(1) starts, S^T of tile 0 --------------------
#pragma unroll
        for (int j = 0; j < kLoads; ++j) stage_k(0u, tiles > 0u, 0, j);
#pragma unroll
        for (int j = 0; j < kLoads; ++j) stage_v(0u, tiles > 0u, 0, j);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kLoads; ++j) stage_k(1u, tiles > 1u, 1, j);
        floatx16 s_cur[2];
        if (my_tiles != 0u) {
            const unsigned char *buf = lds;
            u32x4 frag[kDepth];
#pragma unroll
            for (int i = 0; i < kDepth; ++i) frag[i] = fetch_k(buf, i);
#pragma unroll
            for (int i = 0; i < kHalfSlots; ++i) {
                const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                s_cur[i & 1] = mfma_32x32x16(as_bf16x8(frag[i % kDepth]), q[i >> 1], i < 2 ? zero : s_cur[i & 1]);
                if (i + kDepth < kHalfSlots) frag[i % kDepth] = fetch_k(buf, i + kDepth);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (needs_mask(0u)) mask_tile(s_cur, 0u);
            settle(tile_max(s_cur));
        }

        // ---- main loop --------------------------------------------------------------------
        // One trip; the caller alternates the two score sets so that "next" becomes "current"
        // without a register copy.
        auto trip = [&](uint32_t t, floatx16 (&s_cur)[2], floatx16 (&s_next)[2]) {
            const int cur = (int)(t & 1u), nxt = cur ^ 1;
            // K(t+1) and V(t) have landed (this wave's loads, then everybody's); every wave is
            // done with K(t) and V(t-1)
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
            __syncthreads();
            const bool stage_next_k = t + 2u < tiles, stage_next_v = t + 1u < tiles;
            if (t >= my_tiles) {
                // nothing of this tile is visible to the wave: it only keeps staging
#pragma unroll
                for (int j = 0; j < kLoads; ++j) stage_k(t + 2u, stage_next_k, cur, j);
#pragma unroll
                for (int j = 0; j < kLoads; ++j) stage_v(t + 1u, stage_next_v, nxt, j);
                return;
            }
            // S^T of tile t+1 is computed in every trip; on the wave's last tile the product
            // reads whatever the other buffer holds and is simply not used
            const bool have_next = t + 1u < my_tiles;
            const unsigned char *kbuf = lds + nxt * kBufBytes, *vbuf = lds + cur * kBufBytes;

            uint32_t pk[16];  // bf16 pairs of tile t: [mb * 8 + u * 4 + pair]
            float lsum = 0.f, mloc = -INFINITY;
            u32x4 frag[kDepth];
            // operand of slot i: K fragments for the first half of the slots, V^T fragments for the second
            auto fetch = [&](int i) -> u32x4 {
                return i < kHalfSlots ? fetch_k(kbuf, i) : fetch_v(vbuf, i - kHalfSlots);
            };
#pragma unroll
            for (int i = 0; i < kDepth; ++i) frag[i] = fetch(i);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kSlots; ++i) {
                // ---- the MFMA of this slot ----
                if (i < kHalfSlots) {
                    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f,
                                           0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    s_next[i & 1] = mfma_32x32x16(as_bf16x8(frag[i % kDepth]), q[i >> 1],
                                                  i < 2 ? zero : s_next[i & 1]);
                } else {
                    const int j = i - kHalfSlots, grp = j / kDimBlocks;  // grp = mb * 2 + u
                    const u32x4 w = {pk[grp * 4 + 0], pk[grp * 4 + 1], pk[grp * 4 + 2], pk[grp * 4 + 3]};
                    o[j % kDimBlocks] = mfma_32x32x16(as_bf16x8(frag[i % kDepth]), as_bf16x8(w), o[j % kDimBlocks]);
                }
                if (i + kDepth < kSlots) frag[i % kDepth] = fetch(i + kDepth);
                // ---- one LDS-DMA load of a later tile ----
                if (i < kLoads) stage_k(t + 2u, stage_next_k, cur, i);
                else if (i < 2 * kLoads) stage_v(t + 1u, stage_next_v, nxt, i - kLoads);
                // ---- a slice of the softmax of tile t: the 32 elements spread evenly over
                //      the first three quarters of the slots (3e/4 == i), each before the
                //      O^T MFMA that takes its probability ----
#pragma unroll
                for (int e = (i * 32 + kSoftmaxSlots - 1) / kSoftmaxSlots;
                     e < ((i + 1) * 32 + kSoftmaxSlots - 1) / kSoftmaxSlots && e < 32; ++e) {
                    const int mb = e >> 4, r = e & 15;
                    const float pe = fast_exp2(__builtin_fmaf(s_cur[mb][r], p.scale_log2, neg_m));
                    s_cur[mb][r] = pe;
                    lsum += pe;
                    if (r & 1) pk[mb * 8 + (r >> 1)] = pack_bf16x2(s_cur[mb][r - 1], pe);
                }
                // ---- the per-lane maximum of tile t+1, once its scores are complete ----
                if (i >= kSoftmaxSlots) {
                    const int first = (i - kSoftmaxSlots) * kMaxPerSlot;  // four of the 32 scores per slot
#pragma unroll
                    for (int k4 = first; k4 < first + kMaxPerSlot; k4 += 4) {
                        const int mb = k4 >> 4, r = k4 & 15;
                        if (kMaxPerSlot >= 4)
                            mloc = fmaxf(fmaxf(mloc, s_next[mb][r]),
                                         fmaxf(fmaxf(s_next[mb][r + 1], s_next[mb][r + 2]), s_next[mb][r + 3]));
                        else
                            mloc = fmaxf(mloc, fmaxf(s_next[mb][r], s_next[mb][r + 1]));
                    }
                    asm volatile("" : "+v"(mloc));  // keeps this slice in its slot
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            l_run += lsum;
            if (have_next) {
                if (needs_mask(t + 1u)) {
                    mask_tile(s_next, t + 1u);
                    mloc = tile_max(s_next);
                }
                settle(mloc);
            }
        };
        floatx16 s_alt[2];
        uint32_t t = 0u;
        for (; t + 1u < tiles; t += 2u) {
            trip(t, s_cur, s_alt);
            trip(t + 1u, s_alt, s_cur);
        }
        if (t < tiles) trip(t, s_cur, s_alt);
        // nothing may still be in flight into LDS when the workgroup ends
        __builtin_amdgcn_s_waitcnt(0x0f70);

        // ---- epilogue: normalise, publish bf16 rows and LSE -------------------------
        if (!wave_active) return;
        const uint32_t row = row0 + n;
        float l = l_run;
        l += other_half(l);
        const bool live = row < p.query_tokens;
        const float inv = 1.0f / l;
        bool bad = false;
        uint16_t *dst = p.out + ((uint64_t)row * p.query_heads + head) * kHeadDim;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                const float a0 = o[db][grp * 4 + 0] * inv, a1 = o[db][grp * 4 + 1] * inv;
                const float a2 = o[db][grp * 4 + 2] * inv, a3 = o[db][grp * 4 + 3] * inv;
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
            p.lse[(uint64_t)row * p.query_heads + head] = (m_run + fast_log2(l)) * YVEX_LN2;
    }
};

}  // namespace

// grid = query heads x query tiles of YVEX_ROCM_PREFILL_ROWS rows, block 256,
// LDS 2 x (K + V) tiles.  `waves`: waves per SIMD the register budget is sized for: two
// workgroups per CU for head_dim 64 and 128; head_dim 256 keeps 128 accumulator, 64 query and
// 64 score registers per lane and its tiles fill 128 KB of LDS: one workgroup per CU.
#define YVEX_PREFILL_KERNEL(name, head_dim, waves)                                                        \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(waves, waves)))  \
    name(const yvex_rocm_prefill_params p)                                                                \
    {                                                                                                     \
        static_assert(YVEX_ROCM_PREFILL_ROWS == kRowsPerBlock, "host and kernel agree on the query tile"); \
        __shared__ __attribute__((aligned(16))) unsigned char lds[2 * Prefill<head_dim>::kBufBytes];      \
        Prefill<head_dim>(p, lds).run();                                                                  \
    }

YVEX_PREFILL_KERNEL(yvex_rocm_prefill_bf16, 128, 2)
YVEX_PREFILL_KERNEL(yvex_rocm_prefill_bf16_64, 64, 2)
YVEX_PREFILL_KERNEL(yvex_rocm_prefill_bf16_256, 256, 1)
