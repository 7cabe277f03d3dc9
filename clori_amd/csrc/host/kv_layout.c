/* Host-side packers between token-major KV rows and the device page layouts the decode
 * kernels read.  Bytes are moved, never recomputed: a Q8_0 block keeps its f16 scale
 * and its 32 codes exactly as src/gguf/quant_block.c:160-186 produced them.
 *
 * Token-major input (what a cache writer holds before paging; the reference's
 * [token][kv head][dim] history rows cut into pages):
 *     rows[pool_pages][page_tokens][kv_heads][row]
 * with row = d bf16 values, or d/32 canonical 34-byte Q8_0 blocks.
 *
 * A page of 64 tokens is four consecutive blocks of 16 tokens in the layout below, tokens
 * 16 s .. 16 s + 15 in block s: what a wave reads at once is a 16-token block either way, a
 * larger page only makes four of them contiguous.
 *
 * Device layouts, per (page, kv head) and block of 16 tokens; d = 128, and for BF16 pages
 * also 64 and 256 (the same formulas with fewer or more chunks):
 *   BF16  K  uint16 [d/8][16][8]        elem(t,c) at ((c/8)*16 + t)*8 + c%8
 *         V  uint16 [d][16]             elem(t,c) at c*16 + t
 *   Q8_0  K  codes int8: lane L = 16 g + t of a wave consumes the 32 bytes (j, e) of
 *            code(t, c = 32j + 8g + e), byte r = 8j + e of them; it lies at
 *            (r / 16) * 1024 + 16 L + r % 16 (YVEX_ROCM_Q8_CODE_OFFSET of 32 L + r): the halves of
 *            all lanes side by side, one KB each.  Then f16 scale [16 t][4 j]
 *         V  codes int8: lane L = 16 tg + m consumes the bytes (b, i) of code(t = 4tg + i,
 *            c = 16b + m), byte r = 4b + i, placed the same way; then f16 scale [16 t][4 j]  (j = c/32)
 */
#include "private.h"
#include "../kernel_params.h"

#include <string.h>

enum { PAGE_TOKENS = 16, HEAD_DIM = 128, Q8_BLOCKS = HEAD_DIM / 32 };

/* bytes of one 16-token block; 0 for a storage and head dimension that have no layout */
static unsigned long long block16_bytes(yvex_rocm_kv_storage storage, unsigned long long head_dimension)
{
    if (storage == YVEX_ROCM_KV_BF16 &&
        (head_dimension == 64ull || head_dimension == HEAD_DIM || head_dimension == 256ull))
        return (unsigned long long)PAGE_TOKENS * head_dimension * 2ull;
    if (storage == YVEX_ROCM_KV_Q8_0 && head_dimension == HEAD_DIM)
        return (unsigned long long)PAGE_TOKENS * HEAD_DIM + PAGE_TOKENS * Q8_BLOCKS * 2ull;
    return 0ull;
}

unsigned long long yvex_rocm_kv_page_block_bytes(yvex_rocm_kv_storage storage,
                                                 unsigned long long head_dimension,
                                                 unsigned long long page_tokens)
{
    if (page_tokens != 16ull && page_tokens != 64ull) return 0ull;
    return block16_bytes(storage, head_dimension) * (page_tokens / PAGE_TOKENS);
}

static size_t bf16_index(int is_value, unsigned int t, unsigned int c)
{
    return is_value ? (size_t)c * PAGE_TOKENS + t
                    : ((size_t)(c / 8u) * PAGE_TOKENS + t) * 8u + c % 8u;
}

static size_t q8_code_index(int is_value, unsigned int t, unsigned int c)
{
    unsigned int lane_byte; /* 32 * lane + byte of the lane's 32 */
    if (is_value) {
        unsigned int tg = t / 4u, i = t % 4u, b = c / 16u, m = c % 16u;
        lane_byte = ((tg * 16u + m) * 8u + b) * 4u + i;
    } else {
        unsigned int j = c / 32u, g = (c % 32u) / 8u, e = c % 8u;
        lane_byte = ((g * PAGE_TOKENS + t) * 4u + j) * 8u + e;
    }
    return (size_t)YVEX_ROCM_Q8_CODE_OFFSET(lane_byte);
}

static int layout_move(yvex_rocm_kv_storage storage, int is_value, int pack,
                       unsigned char *rows, unsigned char *packed,
                       unsigned long long pool_pages, unsigned long long page_tokens,
                       unsigned long long kv_heads, unsigned long long head_dimension,
                       yvex_error *err)
{
    const unsigned long long block = yvex_rocm_kv_page_block_bytes(storage, head_dimension,
                                                                   page_tokens);
    const size_t row_bytes = storage == YVEX_ROCM_KV_BF16 ? (size_t)head_dimension * 2u : Q8_BLOCKS * 34u;
    const unsigned long long sub_blocks = page_tokens / PAGE_TOKENS;
    const unsigned long long sub_bytes = block16_bytes(storage, head_dimension);
    unsigned long long page, head, sub;
    unsigned int t, c;
    if (!rows || !packed || !pool_pages || !kv_heads || !block) {
        yvex_error_set(err, block ? YVEX_ERR_INVALID_ARG : YVEX_ERR_UNSUPPORTED, "rocm.kv.layout",
                       block ? "rows, packed buffer and a non-empty pool are required"
                             : "page layout requires head dimension 128 (bf16 pages: 64, 128 or 256) "
                               "and pages of 16 or 64 tokens");
        return block ? YVEX_ERR_INVALID_ARG : YVEX_ERR_UNSUPPORTED;
    }
    for (page = 0ull; page < pool_pages; ++page)
        for (head = 0ull; head < kv_heads; ++head)
          for (sub = 0ull; sub < sub_blocks; ++sub) {
            unsigned char *dst = packed + (page * kv_heads + head) * block + sub * sub_bytes;
            for (t = 0u; t < PAGE_TOKENS; ++t) {
                unsigned char *row =
                    rows + ((page * page_tokens + sub * PAGE_TOKENS + t) * kv_heads + head) * row_bytes;
                if (storage == YVEX_ROCM_KV_BF16) {
                    for (c = 0u; c < (unsigned int)head_dimension; ++c) {
                        unsigned char *p = dst + bf16_index(is_value, t, c) * 2u;
                        unsigned char *r = row + (size_t)c * 2u;
                        if (pack) memcpy(p, r, 2u); else memcpy(r, p, 2u);
                    }
                } else {
                    unsigned char *scales = dst + (size_t)PAGE_TOKENS * HEAD_DIM;
                    for (c = 0u; c < HEAD_DIM; ++c) {
                        unsigned char *p = dst + q8_code_index(is_value, t, c);
                        unsigned char *r = row + (size_t)(c / 32u) * 34u + 2u + c % 32u;
                        if (pack) *p = *r; else *r = *p;
                    }
                    for (c = 0u; c < Q8_BLOCKS; ++c) {
                        unsigned char *p = scales + ((size_t)t * Q8_BLOCKS + c) * 2u;
                        unsigned char *r = row + (size_t)c * 34u;
                        if (pack) memcpy(p, r, 2u); else memcpy(r, p, 2u);
                    }
                }
            }
        }
    yvex_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_kv_pack_pages(yvex_rocm_kv_storage storage, int is_value, const void *rows,
                            unsigned long long pool_pages, unsigned long long page_tokens,
                            unsigned long long kv_heads, unsigned long long head_dimension,
                            void *packed, yvex_error *err)
{
    return layout_move(storage, is_value, 1, (unsigned char *)(uintptr_t)rows,
                       (unsigned char *)packed, pool_pages, page_tokens, kv_heads, head_dimension,
                       err);
}

int yvex_rocm_kv_unpack_pages(yvex_rocm_kv_storage storage, int is_value, const void *packed,
                              unsigned long long pool_pages, unsigned long long page_tokens,
                              unsigned long long kv_heads, unsigned long long head_dimension,
                              void *rows, yvex_error *err)
{
    return layout_move(storage, is_value, 0, (unsigned char *)rows,
                       (unsigned char *)(uintptr_t)packed, pool_pages, page_tokens, kv_heads,
                       head_dimension, err);
}
