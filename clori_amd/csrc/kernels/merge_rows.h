// Log-sum-exp merge of the chunk partials of one (batch element, head) by one wave: eight
// output dims per lane, one 16-byte piece of each chunk's bf16 accumulator row.
#ifndef YVEX_ROCM_KERNELS_MERGE_ROWS_H
#define YVEX_ROCM_KERNELS_MERGE_ROWS_H

#include "mfma.h"

// Sixteen chunks per trip, every load of a trip independent of the others (indices past the
// end alias the last chunk with weight zero): one memory round trip per trip.
//   stats(c, m, l): running maximum (log2 units) and denominator of chunk c
//   piece(c):       the lane's 16 bytes of chunk c's row
template <class Stats, class Piece>
__device__ inline void merge_chunk_rows(uint32_t chunks, Stats stats, Piece piece, float &top,
                                        float &total, float (&acc)[8])
{
    top = -INFINITY;
    total = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    for (uint32_t c0 = 0; c0 < chunks; c0 += 16u) {
        float m[16], l[16];
        u32x4 row[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const uint32_t c = min(c0 + (uint32_t)j, chunks - 1u);
            stats(c, m[j], l[j]);
            row[j] = piece(c);
        }
        float trip = -INFINITY;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if (c0 + (uint32_t)j >= chunks) m[j] = -INFINITY;
            trip = fmaxf(trip, m[j]);
        }
        const float m_new = fmaxf(top, trip);
        const float keep = fast_exp2(top - m_new);  // 0 on the first trip (top = -inf)
        total *= keep;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= keep;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float w = fast_exp2(m[j] - m_new);
            total += w * l[j];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i + 0] += w * bf16_to_f32((uint16_t)(row[j][i] & 0xffffu));
                acc[2 * i + 1] += w * bf16_to_f32((uint16_t)(row[j][i] >> 16));
            }
        }
        top = m_new;
    }
}

// The head's sink logit joins the softmax with a zero value row
// (src/graph/core.c:471-508): it only enlarges the denominator.  Returns false for a sink
// that is not finite.
__device__ inline bool merge_sink(float sink_logit, float &top, float &total, float (&acc)[8])
{
    const float sink = sink_logit * 1.4426950408889634f;  // log2 units, as the maxima
    const float m_new = fmaxf(top, sink);
    const float keep = fast_exp2(top - m_new);
    total = total * keep + fast_exp2(sink - m_new);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= keep;
    top = m_new;
    return isfinite(sink);
}

#endif  // YVEX_ROCM_KERNELS_MERGE_ROWS_H
