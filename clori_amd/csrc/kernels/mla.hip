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
//     O^T[dim][head]  += C^T[dim][token] . P^T[token][head]  32 MFMAs, A = transposed read
// The latent tile is kept once in LDS, row-major with 1152-byte rows and no padding; the
// 16-byte chunk c of row r sits at chunk position c ^ x(r) with
// x(r) = (((r >> 1) & 1) << 2) | ((r >> 2) & 3), which only permutes chunks inside
// aligned groups of 8.  Rows are 128 bytes apart modulo the 256-byte bank span, so
// this makes the row fetch of the first product (ds_read_b128, lane = token) and the
// transposed fetch of the second (ds_read_b64_tr_b16, 4 tokens x 16 dims per 16 lanes)
// both bank-conflict free.
// Tiles are filled by buffer loads that write LDS directly (lds_dma_b128): lane L of 1 KB load j of
// wave w owns linear chunk (9w + j) * 64 + L of the tile and fetches the global chunk that
// belongs there.  A tile never straddles a page (pages are multiples of 32 tokens), so
// the page id is wave-uniform and the buffer descriptor is rebuilt per tile from the page
// base; rows past the context read as zero through the descriptor's range check.
// Four LDS buffers form a ring: two tiles being read, two in flight.  The page ids of the chunk are
// copied to LDS first, so staging never waits on a dependent global load.
// Unnormalised partials (max in log2 units, sum, bf16 accumulator) go to the workspace and
// yvex_rocm_decode_merge performs the log-sum-exp merge.
#include "mfma.h"

#include <type_traits>

#include "../kernel_params.h"

namespace {

constexpr int kValueDim = 512;
constexpr int kTile = 32;                          // tokens per LDS tile
constexpr int kRowBytes = 1152;                    // LDS row pitch, for both geometries
constexpr int kRowChunks = kRowBytes / 16;         // 72
constexpr int kTileBytes = kTile * kRowBytes;      // 36864
constexpr int kBuffers = 4;
constexpr int kHeadsPerWave = 32;
constexpr float kLazyLog2 = 8.0f;
constexpr int kQkDepth = 4;  // operand fetches in flight ahead of the first product
constexpr uint32_t kPageShift = 6;  // pages of 64 tokens (the host admits no other size)

typedef __attribute__((address_space(3))) short4v lds_short4;
typedef short short8v __attribute__((ext_vector_type(8)));
// The page table is read through the constant address space: the address is wave-uniform and
// nothing writes the table while the kernel runs, so every read is a scalar load that counts
// on lgkmcnt and leaves the hand-counted vmcnt of the tile ring alone.
typedef __attribute__((address_space(4))) const int32_t constant_i32;

__device__ inline void flag(int32_t *status, int code) { atomicCAS(status, 0, code); }

__device__ inline int swizzle(int r) { return (((r >> 1) & 1) << 2) | ((r >> 2) & 3); }

// Two geometries share the code.  <576, 128>: the absorbed form, rows of 512 latent + 64 rope
// lanes, 128 heads on four waves; a tile is 36 KB of contiguous rows and every wave stages
// nine linear 1 KB pieces of it.  <512, 64>: the reference's own reduce geometry
// (tests/unit/deepseek_arch_ir.c:110-125: 64 heads, one 512-lane row per token with the rope
// lanes inside, key and value the same row); rows are 1024 bytes in memory and keep the
// 1152-byte pitch in LDS (so the bank analysis above holds unchanged), every wave stages
// eight whole rows, one per load, and waves 2 and 3 only stage: they own no heads.
template <int kKeyDim, int kHeads>
__device__ __forceinline__ void mla_decode(const yvex_rocm_mla_params &p, unsigned char *lds)
{
    constexpr int kSteps = kKeyDim / 16;                     // k-steps of the first product
    constexpr int kSourceRowBytes = kKeyDim * 2;             // row size in global memory
    constexpr bool kRowPerLoad = kSourceRowBytes == 1024;    // one 1 KB load is one row
    constexpr int kLoadsPerWave = kRowPerLoad ? kTile / 4 : kTileBytes / 1024 / 4;  // 8 or 9
    constexpr int kLoadPitch = kRowPerLoad ? kRowBytes : 1024;  // LDS distance between a wave's loads
    constexpr int kActiveWaves = kHeads / kHeadsPerWave;
    constexpr int kQueryRounds = kActiveWaves / 2;           // two head groups per round
    static_assert(kSteps % 4 == 0 && kSteps / 4 == kLoadsPerWave,
                  "the loads of a tile ride behind k-steps 1, 5, 9, ...");
    static_assert(kRowPerLoad || kSourceRowBytes == kRowBytes, "rows are 1024 or 1152 bytes");
    static_assert(kActiveWaves == 2 || kActiveWaves == 4, "head groups come in pairs");
    // at most one younger tile outstanding: vmcnt(kLoadsPerWave), lgkmcnt and expcnt untouched
    constexpr int kWaitTile = 0x0f70 | kLoadsPerWave;
    // at most two younger tiles outstanding
    constexpr int kWaitTwoTiles = 0x0f70 | ((2 * kLoadsPerWave) & 15) | (((2 * kLoadsPerWave) >> 4) << 14);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, g = lane >> 5;
    // Workgroups go to the eight XCDs round robin by their linear id.  They are renumbered so
    // that the chunks of a batch element sit on one XCD: its queries (read by every chunk) and
    // its page table then come from HBM once instead of once per XCD.
    uint32_t chunk = blockIdx.x, batch = blockIdx.y;
    {
        const uint32_t total = gridDim.x * gridDim.y;
        if ((total & 7u) == 0u) {
            const uint32_t linear = blockIdx.x + gridDim.x * blockIdx.y;
            const uint32_t renumbered = (linear & 7u) * (total >> 3) + (linear >> 3);
            batch = renumbered / gridDim.x;
            chunk = renumbered % gridDim.x;
        }
    }
    const uint32_t lds_base = lds_address_of(lds);
    // source offset of this lane's 16 bytes in load j: the chunk that belongs at the lane's
    // (linear) LDS position
    uint32_t stage_off[kLoadsPerWave];
#pragma unroll
    for (int j = 0; j < kLoadsPerWave; ++j) {
        if (kRowPerLoad) {
            const int r = wave * kLoadsPerWave + j;
            stage_off[j] = (uint32_t)(r * kSourceRowBytes + ((lane ^ swizzle(r)) << 4));
        } else {
            const int linear = (wave * kLoadsPerWave + j) * 64 + lane;
            const int r = linear / kRowChunks, pos = linear % kRowChunks;
            stage_off[j] = (uint32_t)(r * kRowBytes + ((pos ^ swizzle(r)) << 4));
        }
    }
    // The queries of the batch element go through the tile buffers too (coalesced 1 KB loads,
    // same swizzle, 32 heads = one "tile"), two head groups per round into buffers 2 and 3,
    // while tiles 0 and 1 are already on their way into buffers 0 and 1: the first tiles'
    // trip to memory runs under the query rounds instead of after them.  A lane's fragments
    // sit 1152 bytes apart in global memory; fetched directly they cost 36 loads of 32
    // separate lines each.
    auto stage_queries = [&](int round) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const i32x4 rsrc = raw_buffer(
                p.q + ((uint64_t)batch * p.heads + (2 * round + j) * kHeadsPerWave) * kKeyDim,
                kHeadsPerWave * kSourceRowBytes);
            const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + (2 + j) * kTileBytes +
                                                                wave * (kLoadsPerWave * kLoadPitch));
#pragma unroll
            for (int i = 0; i < kLoadsPerWave; ++i) lds_dma_b128(dst + i * kLoadPitch, rsrc, stage_off[i], 0u);
        }
    };
    // The first query round is on its way before the context length is known: its address
    // needs only the batch element.  A workgroup that turns out to have nothing to do waits for
    // these loads before it ends (they write its LDS).
    stage_queries(0);
    const uint32_t ctx = (uint32_t)p.context[batch];
    if (ctx == 0u && p.empty_ok != 0u) {
        __builtin_amdgcn_s_waitcnt(0x0f70);
        return;
    }
    if (ctx == 0u || ctx > p.table_stride * p.page_tokens || p.page_tokens != (1u << kPageShift)) {
        if (chunk == 0u && tid == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        return;
    }
    // sliding window (src/backend/cuda/attention_kernels.cu:79-84): positions below
    // ctx - window are not visible; chunks start at the tile that holds the first visible one
    const uint32_t w0 = p.window != 0u && ctx > p.window ? ctx - p.window : 0u;
    const uint32_t t0 = (w0 & ~(uint32_t)(kTile - 1)) + chunk * p.chunk_tokens;
    if (t0 >= ctx) {
        __builtin_amdgcn_s_waitcnt(0x0f70);
        return;
    }
    const uint32_t t1 = min(ctx, t0 + p.chunk_tokens);
    const uint32_t tiles = (t1 - t0 + kTile - 1) / kTile;
    const uint32_t head = wave * kHeadsPerWave + n;

    // ---- tile staging --------------------------------------------------------------
    // Page ids come by scalar loads, one tile ahead of the staging that needs them; an id
    // outside the pool is a contract violation (page 0 is read instead, the status says so).
    constant_i32 *table = (constant_i32 *)(p.page_table + (uint64_t)batch * p.table_stride);
    const uint32_t last_page_index = (t1 - 1u) >> kPageShift;
    auto page_fetch = [&](uint32_t tile) -> int32_t {
        return table[min((t0 + tile * kTile) >> kPageShift, last_page_index)];
    };
    auto page_checked = [&](int32_t id) -> uint32_t {
        const bool outside = id < 0 || (uint32_t)id >= p.pool_pages;
        if (outside && lane == 0) flag(p.status, YVEX_ROCM_DEVICE_CONTRACT);
        return (uint32_t)__builtin_amdgcn_readfirstlane(outside ? 0 : id);
    };
    // A tile's destination and descriptor.  Loads are always issued (with an empty range
    // past the last tile) so that the outstanding-load count at the top of every step is
    // the same.
    auto stage_target = [&](uint32_t tile, uint32_t page, uint32_t &dst, i32x4 &rsrc) {
        const uint32_t first = t0 + tile * kTile;
        uint32_t valid = 0u;
        const uint16_t *base = p.pool;
        if (tile < tiles) {
            valid = min((uint32_t)kTile, t1 - first);
            base = p.pool + (((uint64_t)page << kPageShift) + (first & ((1u << kPageShift) - 1u))) * kKeyDim;
        }
        rsrc = raw_buffer(base, valid * kSourceRowBytes);
        dst = __builtin_amdgcn_readfirstlane(lds_base + (tile % kBuffers) * kTileBytes +
                                             wave * (kLoadsPerWave * kLoadPitch));
    };
    auto stage_tile = [&](uint32_t tile, uint32_t page) {
        uint32_t dst;
        i32x4 rsrc;
        stage_target(tile, page, dst, rsrc);
#pragma unroll
        for (int j = 0; j < kLoadsPerWave; ++j) lds_dma_b128(dst + j * kLoadPitch, rsrc, stage_off[j], 0u);
    };
    const int32_t id0 = page_fetch(0u), id1 = page_fetch(1u);
    int32_t id_ahead = page_fetch(2u);  // fetched a step before the staging that uses it
    stage_tile(0u, page_checked(id0));
    stage_tile(1u, page_checked(id1));

    // ---- operand addresses inside a tile ----------------------------------------------
    // first product, k-step kk: row n, chunk 2kk + g; one address per kk % 4, the rest is
    // an immediate (kk / 4) * 128
    uint32_t k_addr[4];
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4)
        k_addr[k4] = (uint32_t)(n * kRowBytes + (((2 * k4 + g) ^ swizzle(n)) << 4));
    // second product, (db, u, h): 16-lane group b = lane / 16 covers dims 16 * (b & 1) of
    // the 32-dim block and token half g = b / 2; lane a = lane % 16 addresses token row
    // 16u + 8h + 4g + a / 4 and dims db*32 + 16*(b&1) + 4*(a%4) .. +3.  The swizzle flips
    // the chunk's bit 2 by (a >> 3) & 1: one address per (db parity, h), the rest is an
    // immediate (db - parity) * 64 + u * 16 rows.
    uint32_t v_addr[2][2];
    {
        const int a = lane & 15, b1 = (lane >> 4) & 1;
#pragma unroll
        for (int par = 0; par < 2; ++par)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int r = 8 * h + 4 * g + (a >> 2);
                const int chunk16 = (par * 4 + 2 * b1 + ((a >> 1) & 1)) ^ swizzle(r);
                v_addr[par][h] = (uint32_t)(r * kRowBytes + (chunk16 << 4) + 8 * (a & 1));
            }
    }

    // Q fragments: B operand, lane (n, g) holds Q[head n][16*kk + 8g .. +7], kk = 0..35.  The
    // head group of wave w arrives in round w / 2, in buffer 2 + w % 2.
    bf16x8 q[kSteps];
    auto take_queries = [&]() {
        const unsigned char *rows = lds + (2 + (wave & 1)) * kTileBytes;
#pragma unroll
        for (int kk = 0; kk < kSteps; ++kk)
            q[kk] = as_bf16x8(*reinterpret_cast<const u32x4 *>(rows + k_addr[kk & 3] + (kk >> 2) * 128));
    };
    // round 0 has landed when only the two tiles behind it are outstanding
    __builtin_amdgcn_s_waitcnt(kWaitTwoTiles);
    __syncthreads();
    if (wave < 2) take_queries();
    if (kQueryRounds == 2) {
        __syncthreads();  // buffers 2 and 3 are free again
        stage_queries(1);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): round 1, and tiles 0 and 1 with it
        __syncthreads();
        if (wave >= 2) take_queries();
    }
    __syncthreads();  // buffers 2 and 3 are free for tiles once every wave holds its fragments
    if (kActiveWaves < 4 && wave >= kActiveWaves) {
        // a wave without heads: it stages its quarter of every tile and keeps the barriers of
        // the computing waves (one per tile, one before their epilogue)
        for (uint32_t t = 0; t < tiles; ++t) {
            __builtin_amdgcn_s_waitcnt(kWaitTile);
            __syncthreads();
            stage_tile(t + 2u, page_checked(id_ahead));
            id_ahead = page_fetch(t + 3u);
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        return;
    }

    floatx16 o[16];
#pragma unroll
    for (int db = 0; db < 16; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m_run = -INFINITY, neg_m = 0.f, l_run = 0.f;

    // S^T of one tile; `extra(kk)` is work placed behind MFMA kk (operand fetches run
    // kQkDepth k-steps ahead; the order is pinned with scheduling barriers because the
    // register budget leaves the scheduler no room to do it on its own)
    // The score accumulator lives in vector registers (all 256 accumulation registers hold
    // O^T), which the compiler's own MFMA selection does not offer in a kernel that uses
    // accumulation registers at all: these 36 MFMAs are written as assembly.  The compiler
    // still sees their operands (it waits for the LDS fetches), but not their latency: the
    // wait states a vector instruction needs before it reads an 8-pass MFMA's result are
    // spent by hand after the last one.
    auto score = [&](const unsigned char *tile, floatx16 &s, auto extra) {
        u32x4 frag[kQkDepth];
#pragma unroll
        for (int kk = 0; kk < kQkDepth; ++kk)
            frag[kk] = *reinterpret_cast<const u32x4 *>(tile + k_addr[kk & 3] + (kk >> 2) * 128);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < kSteps; ++kk) {
            if (kk == 0)
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(frag[0]), "v"(q[0]));
            else
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"
                             : "+v"(s) : "v"(frag[kk % kQkDepth]), "v"(q[kk]));
            if (kk + kQkDepth < kSteps)
                frag[kk % kQkDepth] = *reinterpret_cast<const u32x4 *>(
                    tile + k_addr[(kk + kQkDepth) & 3] + ((kk + kQkDepth) >> 2) * 128);
            extra(kk);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // masks the tail (and the keys in front of a sliding window), then raises the running maximum if this
    // tile needs it (both token halves of a head must agree on the reference maximum)
    // `first`: the chunk's first tile, nothing accumulated yet: the maximum is taken as it is
    // and there is nothing to rescale (the general path would multiply 256 zeros)
    auto settle = [&](uint32_t key0, floatx16 &s, uint32_t (&pending)[8], auto first) {
        if (key0 + kTile > t1 || key0 < w0) {
            // visible keys are w0 <= key < t1: one unsigned compare
#pragma unroll
            for (int i = 0; i < 16; ++i)
                if (key0 + (i >> 2) * 8 + g * 4 + (i & 3) - w0 >= t1 - w0) s[i] = -INFINITY;
        }
        float mloc = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[i]);
        mloc *= p.scale_log2;
        if (decltype(first)::value) {
            m_run = max_xor32(mloc);
            neg_m = m_run == -INFINITY ? 0.f : -m_run;
        } else if (__builtin_amdgcn_ballot_w64(mloc > m_run + kLazyLog2) != 0ull) {
            const float m_new = fmaxf(m_run, max_xor32(mloc));
            const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2(m_run - m_new);
            l_run *= alpha;
            // one block at a time through the VALU; the accumulators live in AGPRs
#pragma unroll
            for (int db = 0; db < 16; ++db) {
                asm volatile("" : "+a"(o[db]));
                o[db] *= alpha;
                asm volatile("" : "+a"(o[db]));
            }
            // probabilities computed under the old maximum that are not in O yet
#pragma unroll
            for (int j = 0; j < 8; ++j)
                pending[j] = pack_bf16x2(bf16_to_f32((uint16_t)(pending[j] & 0xffffu)) * alpha,
                                         bf16_to_f32((uint16_t)(pending[j] >> 16)) * alpha);
            m_run = m_new;
            neg_m = m_new == -INFINITY ? 0.f : -m_new;
        }
    };

    // Software pipeline over tiles: step t computes the scores of tile t (with the loads
    // of tile t+2 spread behind its MFMAs), settles the maximum, then issues the O^T update
    // with tile t-1 and, behind its MFMAs, the exponentials of tile t.  Tiles t-1 and t
    // are being read during a step, tiles t+1 and t+2 are in flight.
    uint32_t pk_prev[8], pk_cur[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) pk_prev[j] = 0u;
    // O^T += C^T . P^T with the tile at `tile`, MFMAs [first, last) of the 32 (token half u =
    // index / 16, dim block db = index % 16)
    auto value_operand = [&](const unsigned char *tile, int index) -> bf16x8 {
        const int u = index >> 4, db = index & 15;
        const int imm = (db & ~1) * 64 + u * 16 * kRowBytes;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4 *)(tile + v_addr[db & 1][0] + imm));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4 *)(tile + v_addr[db & 1][1] + imm));
        const short8v av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, av);
    };
    auto accumulate = [&](const unsigned char *tile, const uint32_t (&pk)[8], int first, int last) {
#pragma unroll
        for (int index = first; index < last; ++index) {
            const int u = index >> 4, db = index & 15;
            const u32x4 w = {pk[u * 4 + 0], pk[u * 4 + 1], pk[u * 4 + 2], pk[u * 4 + 3]};
            o[db] = mfma_32x32x16(value_operand(tile, index), as_bf16x8(w), o[db]);
        }
    };
    constexpr int kEarly = 4;  // update MFMAs issued under the settling of the next tile's maximum
    auto step = [&](uint32_t t, auto with_update) {
        // tile t has landed when at most one younger tile is outstanding: vmcnt(9)
        __builtin_amdgcn_s_waitcnt(kWaitTile);
        __syncthreads();
        uint32_t stage_dst;
        i32x4 stage_rsrc;
        stage_target(t + 2u, page_checked(id_ahead), stage_dst, stage_rsrc);
        id_ahead = page_fetch(t + 3u);
        const unsigned char *tile = lds + (t % kBuffers) * kTileBytes;
        const unsigned char *prev_tile = lds + ((t + kBuffers - 1u) % kBuffers) * kTileBytes;

        // ---- S^T of tile t, the loads of tile t+2 behind its MFMAs ------------------------
        floatx16 s;
        bf16x8 early[kEarly];
        score(tile, s, [&](int kk) {
            if ((kk & 3) == 1) lds_dma_b128(stage_dst + (kk >> 2) * kLoadPitch, stage_rsrc, stage_off[kk >> 2], 0u);
            // the last k-steps fetch no further score operand: the first operands of the update
            // take their place
            if (decltype(with_update)::value && kk >= kSteps - kEarly)
                early[kk - (kSteps - kEarly)] = value_operand(prev_tile, kk - (kSteps - kEarly));
        });
        // The first MFMAs of the update with tile t-1 go out at once: they need nothing of tile t,
        // and the wait for the last score MFMA, the row maximum and the decision about a new
        // reference maximum run under them.  Should the maximum move, O (with what these MFMAs
        // added) and the probabilities still waiting are rescaled together.
        if (decltype(with_update)::value) {
            const u32x4 w = {pk_prev[0], pk_prev[1], pk_prev[2], pk_prev[3]};
#pragma unroll
            for (int index = 0; index < kEarly; ++index)
                o[index] = mfma_32x32x16(early[index], as_bf16x8(w), o[index]);
        }
        // wait states between the last score MFMA (8 passes) and the first vector read of its result
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(s));
        settle(t0 + t * kTile, s, pk_prev, std::integral_constant<bool, !decltype(with_update)::value>());

        // ---- the rest of the O^T update with tile t-1 (none in the first step) and the
        //      exponentials of tile t behind its MFMAs ---------------------------------------
        float lsum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float p0 = fast_exp2(__builtin_fmaf(s[i], p.scale_log2, neg_m));
            const float p1 = fast_exp2(__builtin_fmaf(s[i + 1], p.scale_log2, neg_m));
            lsum += p0 + p1;
            pk_cur[i >> 1] = pack_bf16x2(p0, p1);
        }
        l_run += lsum;
        if (decltype(with_update)::value) {
            accumulate(prev_tile, pk_prev, kEarly, 32);
            // three transposed operand pairs in flight ahead of the MFMAs that consume them,
            // one exponential behind every second MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
            for (int i = 0; i < (32 - kEarly - 4) / 2; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) pk_prev[j] = pk_cur[j];
    };
    step(0u, std::integral_constant<bool, false>());
    for (uint32_t t = 1; t < tiles; ++t)
        step(t, std::integral_constant<bool, true>());
    // the update with the last tile
    __builtin_amdgcn_sched_barrier(0);
    accumulate(lds + ((tiles - 1u) % kBuffers) * kTileBytes, pk_prev, 0, 32);
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
    for (int i = 0; i < 29; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
    // drain the loads that were issued past the last tile before the workgroup ends
    __builtin_amdgcn_s_waitcnt(0x0f70);

    float l = l_run;
    l = sum_xor32(l);
    const uint64_t slot = ((uint64_t)batch * p.slot_stride + p.first_slot + chunk) * p.heads + head;
    // The accumulators are lane = head, registers = dims; through LDS they become one
    // contiguous 1 KB bf16 row per head, written by one 16-byte store per lane.
    constexpr int kOutPitch = kValueDim * 2 + 16;  // 1040 B, keeps 16-byte alignment
    static_assert(4 * kHeadsPerWave * kOutPitch <= kBuffers * kTileBytes, "epilogue fits the tiles");
    __syncthreads();  // every wave is done with the tile buffers
    unsigned char *rows = lds + wave * (kHeadsPerWave * kOutPitch);
#pragma unroll
    for (int db = 0; db < 16; ++db)
#pragma unroll
        for (int grp = 0; grp < 4; ++grp) {
            u32x2 v;
            v.x = pack_bf16x2(o[db][grp * 4 + 0], o[db][grp * 4 + 1]);
            v.y = pack_bf16x2(o[db][grp * 4 + 2], o[db][grp * 4 + 3]);
            *reinterpret_cast<u32x2 *>(rows + n * kOutPitch + (db * 32 + grp * 8 + g * 4) * 2) = v;
        }
    // only this wave reads what it wrote: no workgroup barrier needed
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    {
        const uint64_t slot0 =
            ((uint64_t)batch * p.slot_stride + p.first_slot + chunk) * p.heads + wave * kHeadsPerWave;
        uint16_t *dst = p.part_acc + slot0 * kValueDim + lane * 8;
        // every workgroup starts its 32 rows at another one: the rows of all workgroups are
        // 1 KB apart at the same offsets of 128 KB regions, and written in step they would all
        // be in the same memory channels at the same time
        const int skew = (int)((chunk * 5u + batch * 3u) & 31u);
#pragma unroll 8
        for (int i = 0; i < kHeadsPerWave; ++i) {
            const int hh = (i + skew) & (kHeadsPerWave - 1);
            const u32x4 v = *reinterpret_cast<const u32x4 *>(rows + hh * kOutPitch + lane * 16);
            *reinterpret_cast<u32x4 *>(dst + (uint64_t)hh * kValueDim) = v;
        }
    }
    if (g == 0) {
        p.part_ml[slot * 2 + 0] = m_run;
        p.part_ml[slot * 2 + 1] = l;
    }
}

}  // namespace

// grid = (chunks, batch), block 256 (pages a multiple of 32 tokens), LDS 4 x 36 KB.
#define YVEX_MLA_KERNEL(name, key_dim, heads)                                                       \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))     \
    name(const yvex_rocm_mla_params p)                                                               \
    {                                                                                                \
        __shared__ __attribute__((aligned(16))) unsigned char lds[kBuffers * kTileBytes];            \
        mla_decode<key_dim, heads>(p, lds);                                                          \
    }

YVEX_MLA_KERNEL(yvex_rocm_mla_decode_bf16, 576, 128)
YVEX_MLA_KERNEL(yvex_rocm_mla_decode_512_bf16, 512, 64)

// Row gather for the selected class of compressed candidates (src/graph/core.c:443-452): list
// entry i of batch element b names a compressed row; it is copied to row i of that element's
// slice of a contiguous pool, so that the decode kernel above walks the list as an ordinary
// paged context.  One workgroup per list entry, 16 bytes per lane.
extern "C" __global__ void __launch_bounds__(128)
yvex_rocm_gather_rows(const yvex_rocm_gather_rows_params p)
{
    const uint32_t entry = blockIdx.x, batch = blockIdx.y, lane = threadIdx.x;
    const int32_t count = p.count[batch];
    if (count < 0 || (uint32_t)count > p.selected_stride) {
        if (entry == 0u && lane == 0u) atomicCAS(p.status, 0, YVEX_ROCM_DEVICE_CONTRACT);
        return;
    }
    if (entry % p.page_tokens == 0u && lane == 0u)
        p.table[(uint64_t)batch * p.pages_each + entry / p.page_tokens] =
            (int32_t)(batch * p.pages_each + entry / p.page_tokens);
    if (entry >= (uint32_t)count) return;
    const int32_t index = p.selected[(uint64_t)batch * p.selected_stride + entry];
    if (index < 0 || (uint32_t)index >= p.max_rows) {
        if (lane == 0u) atomicCAS(p.status, 0, YVEX_ROCM_DEVICE_CONTRACT);
        return;
    }
    const int32_t page = p.page_table[(uint64_t)batch * p.table_stride + (uint32_t)index / p.page_tokens];
    if (page < 0 || (uint32_t)page >= p.pool_pages) {
        if (lane == 0u) atomicCAS(p.status, 0, YVEX_ROCM_DEVICE_CONTRACT);
        return;
    }
    const uint16_t *src = p.pool + ((uint64_t)page * p.page_tokens + (uint32_t)index % p.page_tokens) * p.row_elements;
    uint16_t *dst = p.rows + ((uint64_t)batch * p.pages_each * p.page_tokens + entry) * p.row_elements;
    if (lane * 8u < p.row_elements)
        *reinterpret_cast<u32x4 *>(dst + lane * 8u) = load_b128(src + lane * 8u);
}
