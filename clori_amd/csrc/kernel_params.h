/* Kernel argument blocks shared by the C11 host and the gfx950 device code.  Each
 * kernel takes exactly one of these structs by value.  Only fixed-width scalars and
 * pointers, ordered so that no implicit padding exists on either compiler. */
#ifndef YVEX_ROCM_KERNEL_PARAMS_H
#define YVEX_ROCM_KERNEL_PARAMS_H

#include <stdint.h>

/* Device status word values, as in the reference kernels (atomicCAS(status,0,1) for a
 * numeric failure, atomicCAS(status,0,2) for a contract violation). */
enum {
    YVEX_ROCM_DEVICE_OK = 0,
    YVEX_ROCM_DEVICE_NUMERIC = 1,
    YVEX_ROCM_DEVICE_CONTRACT = 2,
    YVEX_ROCM_DEVICE_SOFTMAX_ZERO = 3
};

typedef struct {
    const float *q, *k, *v;
    float *score, *prob, *out;
    int32_t *status;
    uint64_t seq_len, position, head_dim;
    float scale;
    int32_t causal;
} yvex_rocm_attention_f32_params;

typedef struct {
    const float *q, *k, *v;
    float *out;
    float *lse; /* optional [Tq][Hq] */
    int32_t *status;
    uint64_t query_tokens, kv_tokens, query_start, query_heads, kv_heads, head_dim;
    uint64_t q_stride, k_stride, v_stride;
    float scale;
    int32_t causal;
    /* split form (yvex_rocm_gqa_f32_split[_wide]): the keys a query sees are cut into `splits`
     * runs of keys_per_split, eight consecutive runs per workgroup (a team); part_acc is F64
     * [Tq*Hq][teams][head_dim], part_ml F64 [Tq*Hq][teams][2] = (running maximum,
     * denominator), teams = ceil(splits / 8); arrivals holds one counter per (token, head),
     * zero before the launch and after it */
    double *part_acc, *part_ml;
    uint32_t splits, keys_per_split;
    uint32_t *arrivals;
    /* tile form (yvex_rocm_gqa_f32_tile_*): compute units when workgroups b and b + units share
     * a unit and are to carry equal work (causal launches of at least two tiers of items), else 0 */
    uint32_t pair_units, reserved_tile;
    /* tile form, scheduled launches: workgroup b runs the items of row b of `lists`, one after
     * the other; a row is 8 uint16, the count of items, then the items.  NULL: one item per
     * workgroup */
    const uint16_t *lists;
} yvex_rocm_gqa_f32_params;

typedef struct {
    uint32_t *data;
    uint64_t words;
    uint32_t value;
    uint32_t reserved;
} yvex_rocm_fill_params;

/* Streaming read of `words` 16-byte words; the sink is written only if the XOR of
 * everything read equals `never` (it does not: the loads cannot be dropped). */
typedef struct {
    const void *data;
    uint32_t *sink;
    uint64_t words;
    uint32_t never;
    uint32_t reserved;
} yvex_rocm_stream_params;

/* Split-K decode over a balanced partition.  The (session, kv head, 16-token tile) work
 * of the whole batch is laid out as one sequence and cut into gridDim.x equal ranges,
 * one wave each.  A wave that covers a whole (session, kv head) segment publishes the
 * final rows itself; otherwise it leaves a partial in one of its two slots, adds one to the
 * segment's arrival counter, and the wave that completes the count merges the parts in
 * wave order and publishes.
 * part_acc is [2*waves][group][head_dim] F32 (unnormalised), part_ml is
 * [2*waves][group][2] F32 = (running max in log2 units, sum); arrivals is
 * [sessions][kv_heads] U32, zero before the launch and zero again after it, or NULL: then
 * wave 0 writes offsets ([sessions + 1] U32: exclusive prefix of work items per session, then
 * the total) and yvex_rocm_decode_finish merges in a second launch. */
typedef struct {
    const uint16_t *q;
    const void *k_pool, *v_pool;
    const int32_t *page_table; /* NULL for the token-major layout */
    const int32_t *context;    /* NULL: every session uses fixed_context */
    uint16_t *out;             /* bf16 [sessions][query_heads][head_dim] */
    float *lse;                /* optional F32 [sessions][query_heads] */
    float *part_acc, *part_ml;
    uint32_t *arrivals;
    uint32_t *offsets;
    int32_t *status;
    uint64_t k_token_stride, v_token_stride; /* token-major layout: elements per token */
    uint32_t sessions, query_heads, kv_heads, head_dim;
    uint32_t pool_pages, table_stride, min_tiles, fixed_context;
    uint32_t waves;
    uint32_t page_shift; /* a page is 16 << page_shift tokens: that many consecutive 16-token blocks */
    float scale_log2; /* softmax scale * log2(e) */
    float reserved_f;
    const uint16_t *gate; /* optional bf16 [sessions][query_heads][head_dim] sigmoid output gate */
} yvex_rocm_decode_params;

#define YVEX_ROCM_ROPE_PAIRS_MAX 64

/* Log-sum-exp merge of per-chunk partials (used by the MLA path).  With a sliding window the
 * chunks start at the first visible token rounded down to window_align, as in the producer.  The accumulators are
 * unnormalised and stored as bf16: they are 44 % of that path's HBM traffic in fp32. */
typedef struct {
    const uint16_t *part_acc;
    const float *part_ml;
    const int32_t *context;
    uint16_t *out; /* bf16 [sessions][query_heads][head_dim] */
    float *lse;    /* optional F32 [sessions][query_heads] */
    int32_t *status;
    uint32_t sessions, query_heads, head_dim, chunk_tokens, max_chunks, fixed_context;
    const float *sinks; /* optional F32 [query_heads]: one extra logit per head with value 0 */
    uint32_t window;    /* sliding window of the producing kernel (sets its first chunk) */
    uint32_t window_align; /* the producer starts its chunks at first_visible rounded down to this */
    /* second candidate set: its chunks sit in slots max_chunks .. max_chunks + extra_max_chunks - 1
     * of each batch element; extra_context NULL: none */
    const int32_t *extra_context;
    uint32_t extra_chunk_tokens, extra_max_chunks;
    /* inverse rotation of the last rope_dims lanes of each published row (0: none): angle of
     * pair i = position * rope_frequency[i]; positions NULL: context - 1 */
    const int64_t *positions;
    uint32_t rope_dims, reserved;
    double rope_frequency[YVEX_ROCM_ROPE_PAIRS_MAX];
} yvex_rocm_decode_merge_params;

/* Q8_0 pages: where byte r (0..31) of the 32 code bytes that lane L (0..63) of a wave consumes
 * lies in the 2048 code bytes of a 16-token block, written for the offset o = 32 L + r.  The two
 * 16-byte halves of a lane's bytes are 1 KB apart, so that each of a wave's two 16-byte loads
 * reads one contiguous KB (lanes side by side): 230 us against 264 us for config 4's 1.5 GB
 * when the lanes' loads were 32 bytes apart. */
#define YVEX_ROCM_Q8_CODE_OFFSET(o) ((((o) & 16u) << 6) + (((o) >> 5) << 4) + ((o) & 15u))

/* A batch of small device-to-device copies in one launch: the reference's session layer
 * appends every new token to a layer's history with two asynchronous copies
 * (src/runtime/stateful_attention.c:183-222), 4096 of them for a prompt of 2048 tokens.
 * grid = (pieces, count): workgroup (x, y) copies 16-byte pieces x * 256 + thread,
 * + gridDim.x * 256, ... of copy y; addresses and sizes are multiples of 16 bytes. */
#define YVEX_ROCM_COPY_BATCH_MAX 128
typedef struct {
    uint64_t dst[YVEX_ROCM_COPY_BATCH_MAX], src[YVEX_ROCM_COPY_BATCH_MAX];
    uint32_t bytes[YVEX_ROCM_COPY_BATCH_MAX];
} yvex_rocm_copy_batch_params;

/* Small transfers between the host and a tensor without the runtime's copy path.
 * write: up to YVEX_ROCM_SMALL_WRITE_MAX bytes travel in the kernel's arguments and one
 * workgroup of 256 threads stores them at dst; the host does not wait.
 * read: one workgroup copies `bytes` from src into host memory the device can write
 * (staging) and then leaves sequence << 32 in the mailbox the host is watching. */
#define YVEX_ROCM_SMALL_WRITE_MAX 2048
#define YVEX_ROCM_SMALL_READ_MAX 16384
typedef struct {
    void *dst;
    uint32_t bytes, reserved;
    unsigned char data[YVEX_ROCM_SMALL_WRITE_MAX];
} yvex_rocm_small_write_params;

typedef struct {
    const void *src;
    void *staging;
    uint64_t *mailbox;
    uint32_t bytes, sequence;
} yvex_rocm_small_read_params;

/* Completion: one workgroup of 64 threads behind an operation's kernels.  Takes the status
 * word (and clears it when set) and leaves (sequence << 32 | status) in a word of host memory,
 * which the host is watching. */
typedef struct {
    int32_t *status;
    uint64_t *mailbox;
    uint32_t sequence;
} yvex_rocm_status_forward_params;

/* The element-wise operators the reference's decoder runs around attention on F32 activations
 * (src/runtime/decoder.c:989-997,1030-1046,1112-1131,1266-1269): one thread per element (per
 * rotated pair for the rotation), blocks of YVEX_ROCM_ELEMENTWISE_BLOCK threads.
 *   rotary:  values in place, left = cosines, right = sines [tokens][rotary_dim]; count pairs
 *   round:   values in place; a value that is not finite sets the status word
 *   sigmoid: values = output, left = values, right = gate
 *   split:   left = input [rows][heads][2][head_dim], values = first, second = second */
#define YVEX_ROCM_ELEMENTWISE_BLOCK 256
typedef struct {
    float *values, *second;
    const float *left, *right;
    int32_t *status;
    uint64_t count, heads, head_dim, rotary_dim;
} yvex_rocm_elementwise_params;

/* Causal / full GQA prefill on bf16 token-major tensors.  The grid is one-dimensional:
 * query_heads * ceil(query_tokens / YVEX_ROCM_PREFILL_ROWS) workgroups of 256 threads. */
#define YVEX_ROCM_PREFILL_ROWS 128
typedef struct {
    const uint16_t *q, *k, *v;
    uint16_t *out;
    float *lse; /* optional F32 [Tq][Hq] */
    int32_t *status;
    uint64_t q_stride, k_stride, v_stride; /* elements per token */
    uint32_t query_tokens, kv_tokens, query_start, query_heads, kv_heads, head_dim;
    uint32_t causal, reserved;
    float scale_log2;
    float reserved_f;
    const uint16_t *gate; /* optional bf16 [Tq][Hq][head_dim] sigmoid output gate */
} yvex_rocm_prefill_params;

/* Absorbed-latent MLA decode, split over the context.  A chunk spans at most
 * YVEX_ROCM_MLA_MAX_CHUNK_PAGES pages (a bound of the host's partition; the kernel reads the
 * page ids as it goes). */
#define YVEX_ROCM_MLA_MAX_CHUNK_PAGES 256
typedef struct {
    const uint16_t *q;      /* [batch][heads][key_dim] */
    const uint16_t *pool;   /* [pool_pages][page_tokens][key_dim] */
    const int32_t *page_table, *context;
    uint16_t *part_acc; /* bf16 [batch][max_chunks][heads][value_dim] */
    float *part_ml;     /* [batch][max_chunks][heads][2] */
    int32_t *status;
    uint32_t batch, heads, key_dim, value_dim;
    uint32_t page_tokens, pool_pages, table_stride, chunk_tokens, max_chunks;
    uint32_t window; /* sliding window in tokens, 0: the whole context */
    float scale_log2;
    float reserved_f;
    uint32_t first_slot;  /* partial slot of chunk 0 (a second candidate set writes after the first) */
    uint32_t slot_stride; /* partial slots per batch element, all sets together */
    uint32_t empty_ok;    /* a context of 0 rows is an empty set, not a contract violation */
    uint32_t reserved;
} yvex_rocm_mla_params;

/* Gathers the selected compressed rows of every batch element into a contiguous paged pool
 * (batch * pages_each pages of page_tokens rows) and writes the identity page table for it.
 * grid = (selected_stride, batch), block = 128. */
typedef struct {
    const uint16_t *pool;         /* [pool_pages][page_tokens][row_elements] */
    const int32_t *page_table;    /* [batch][table_stride] */
    const int32_t *selected;      /* [batch][selected_stride] logical row indices */
    const int32_t *count;         /* [batch] list entries */
    uint16_t *rows;               /* [batch * pages_each][page_tokens][row_elements] */
    int32_t *table;               /* [batch][pages_each] */
    int32_t *status;
    uint32_t batch, page_tokens, pool_pages, table_stride;
    uint32_t selected_stride, pages_each, row_elements, max_rows;
} yvex_rocm_gather_rows_params;

/* KV page writer: new key/value rows -> paged pools (bf16 or Q8_0), rotary on the keys.
 * A workgroup is YVEX_ROCM_KV_APPEND_HEADS waves, one kv head each. */
#define YVEX_ROCM_KV_APPEND_HEADS 4
typedef struct {
    const uint16_t *key, *value;      /* bf16 [total_tokens][kv_heads][head_dim] */
    const float *cosine, *sine;       /* F32 [total_tokens][rotary_dim]; unused when rotary_dim = 0 */
    const int32_t *row_start;         /* [sessions] first input row of the session's new tokens */
    const int32_t *position_start;    /* [sessions] position of its first new token */
    const int32_t *token_count;       /* [sessions] new tokens (0: nothing to do) */
    const int32_t *page_table;        /* [sessions][table_stride] */
    void *k_pool, *v_pool;
    int32_t *status;
    uint64_t total_tokens;
    uint32_t sessions, kv_heads, head_dim, rotary_dim;
    uint32_t pool_pages, table_stride;
    uint32_t rotary_mode;             /* 0: products staged through bf16; 1: F32 rotation, one rounding */
    uint32_t page_shift;              /* a page is 16 << page_shift tokens: consecutive 16-token blocks */
} yvex_rocm_kv_append_params;

/* Token-major history writer: new key/value rows -> rows [first_row, first_row + tokens) of
 * the strided K and V histories the GQA kernels read, rotary on the keys.  One thread per
 * 16-byte piece of a row (8 bf16 or 4 F32 lanes), the pieces of the optional query tensor
 * behind those of the keys and values; grid = ceil(pieces / 256), block = 256.
 * The bf16 and the F32 kernel take the same block; pointers are to the element type. */
typedef struct {
    const void *key, *value;          /* [tokens][kv_heads][head_dim] */
    const float *cosine, *sine;       /* F32 [tokens][rotary_dim]; unused when rotary_dim = 0 */
    void *key_history, *value_history; /* row r of a history at r * its token stride */
    int32_t *status;
    uint64_t first_row, key_token_stride, value_token_stride; /* strides in elements */
    uint32_t tokens, kv_heads, head_dim, rotary_dim;
    uint32_t rotary_mode;             /* as in yvex_rocm_kv_append_params */
    uint32_t query_heads;             /* 0 without a query tensor */
    void *query;                      /* [tokens][query_heads][head_dim], rotated where it lies */
} yvex_rocm_history_append_params;

#endif /* YVEX_ROCM_KERNEL_PARAMS_H */
