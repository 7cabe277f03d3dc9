/* Deals the items of a causal multi-token launch to workgroups so that every compute unit
 * carries the same number of key tiles.
 *
 * An item is one (query head, tile of query rows); items are numbered heaviest first
 * (item / query_heads counts the query tiles down from the last) and walk the keys their
 * last row sees, so the items of one launch differ many-fold in length.  The hardware gives
 * workgroup b of the first per_unit * units workgroups to compute unit b % units and hands
 * out later ones as slots come free; a kernel that is bound by the matrix cores takes as long
 * as the unit with the most tiles.  Here every unit gets `per_unit` lists and workgroup b runs
 * list b, one item after the other.  The items are dealt heaviest first to the unit with the
 * least work, then exchanged between random pairs of units (moves and swaps that bring both
 * closer to the mean, ties at random) until every unit is within one step of the mean or the
 * bounded number of tries is spent; within a unit each item goes to the shorter list.
 *
 * The lists are built when a geometry comes for the second time in a row (a caller that never
 * repeats a geometry pays nothing) and kept, on the host and on the device, while it repeats:
 * rows of YVEX_ROCM_LIST_STRIDE uint16, the count of items, then the items. */
#include "rocm_state.h"

#include <stdlib.h>
#include <string.h>

#define SCHEDULE_UNIT_ITEMS 6u
#define SCHEDULE_ITEM_STEPS 1u /* what the start and the end of an item cost, in steps */

static uint32_t item_steps(const yvex_rocm_schedule_key *key, unsigned int q_tiles, unsigned int item)
{
    const unsigned int q_tile = q_tiles - 1u - item / key->query_heads;
    unsigned long long last_row = ((unsigned long long)q_tile + 1ull) * key->item_rows;
    unsigned long long keys;
    if (last_row > key->query_tokens) last_row = key->query_tokens;
    keys = key->query_start + last_row;
    if (keys > key->kv_tokens) keys = key->kv_tokens;
    return (uint32_t)((keys + key->step_keys - 1ull) / key->step_keys);
}

static int lists_build(yvex_rocm_backend_state *state, const yvex_rocm_schedule_key *key,
                       unsigned int q_tiles, unsigned int units)
{
    const unsigned int items = q_tiles * key->query_heads, per_unit = key->per_unit;
    const unsigned int lists = units * per_unit;
    /* no unit holds more items than the fullest must */
    const unsigned int unit_cap = (items + units - 1u) / units;
    uint16_t(*held)[SCHEDULE_UNIT_ITEMS];
    uint16_t *steps, *rows = state->schedule.rows;
    uint32_t *load;
    uint8_t *count;
    unsigned long long total = 0ull;
    uint32_t low, high, random = 0x2545f491u;
    unsigned int i, u, k, outside, tries;
    void *block;
    if (unit_cap > SCHEDULE_UNIT_ITEMS) return 0;
    block = calloc(1u, (size_t)units * sizeof(*held) + (size_t)items * sizeof(*steps) +
                           (size_t)units * sizeof(*load) + (size_t)units);
    if (!block) return 0;
    load = (uint32_t *)block;
    held = (uint16_t(*)[SCHEDULE_UNIT_ITEMS])(load + units);
    steps = (uint16_t *)(held + units);
    count = (uint8_t *)(steps + items);
    for (i = 0u; i < items; ++i) {
        unsigned int best = 0u;
        steps[i] = (uint16_t)(item_steps(key, q_tiles, i) + SCHEDULE_ITEM_STEPS);
        total += steps[i];
        while (best < units && count[best] >= unit_cap) ++best;
        for (u = best + 1u; u < units; ++u)
            if (count[u] < unit_cap && load[u] < load[best]) best = u;
        if (best >= units) {
            free(block);
            return 0;
        }
        held[best][count[best]++] = (uint16_t)i;
        load[best] += steps[i];
    }
    /* every unit within one step of the mean */
    low = (uint32_t)(total / units);
    low -= low > 0u;
    high = low + 2u;
    outside = 0u;
    for (u = 0u; u < units; ++u) outside += load[u] < low || load[u] > high;
    for (tries = 0u; outside && tries < 8u * items; ++tries) {
        unsigned int a, b, ia, ib, best_ia = 0u, best_ib = 0u, ties = 0u;
        long long best_cost, now;
        const long long middle = (long long)low + (long long)high; /* twice the middle */
        random = random * 1664525u + 1013904223u;
        a = (random >> 8) % units;
        /* walk on to the next unit outside the band */
        for (k = 0u; k < units && load[a] >= low && load[a] <= high; ++k) a = (a + 1u) % units;
        random = random * 1664525u + 1013904223u;
        b = (random >> 8) % units;
        if (a == b) continue;
#define SCHEDULE_COST(la, lb) \
    ((2ll * (la) - middle) * (2ll * (la) - middle) + (2ll * (lb) - middle) * (2ll * (lb) - middle))
        now = SCHEDULE_COST((long long)load[a], (long long)load[b]);
        best_cost = now + 1ll;
        /* ia / ib == count: nothing leaves that side */
        for (ia = 0u; ia <= count[a]; ++ia)
            for (ib = 0u; ib <= count[b]; ++ib) {
                const long long give = ia < count[a] ? steps[held[a][ia]] : 0;
                const long long take = ib < count[b] ? steps[held[b][ib]] : 0;
                long long cost;
                if (give == take) continue;
                if (ia < count[a] && ib == count[b] && count[b] >= unit_cap) continue;
                if (ib < count[b] && ia == count[a] && count[a] >= unit_cap) continue;
                cost = SCHEDULE_COST((long long)load[a] - give + take, (long long)load[b] + give - take);
                if (cost > now || cost > best_cost) continue;
                if (cost < best_cost) ties = 0u;
                random = random * 1664525u + 1013904223u;
                if (cost < best_cost || (random >> 8) % (++ties) == 0u) {
                    best_cost = cost;
                    best_ia = ia;
                    best_ib = ib;
                }
                if (!ties) ties = 1u;
            }
#undef SCHEDULE_COST
        if (best_cost > now) continue;
        outside -= (load[a] < low || load[a] > high) + (load[b] < low || load[b] > high);
        {
            const int gives = best_ia < count[a], takes = best_ib < count[b];
            const uint16_t given = gives ? held[a][best_ia] : 0u, taken = takes ? held[b][best_ib] : 0u;
            if (gives) {
                load[a] -= steps[given];
                held[a][best_ia] = held[a][--count[a]];
            }
            if (takes) {
                /* the slot of `taken` did not move: best_ib indexes b's array */
                load[b] -= steps[taken];
                held[b][best_ib] = held[b][--count[b]];
            }
            if (gives) {
                held[b][count[b]++] = given;
                load[b] += steps[given];
            }
            if (takes) {
                held[a][count[a]++] = taken;
                load[a] += steps[taken];
            }
        }
        outside += (load[a] < low || load[a] > high) + (load[b] < low || load[b] > high);
    }
    /* within a unit: heaviest item first, each to the shorter of the unit's lists */
    memset(rows, 0, sizeof(state->schedule.rows));
    for (u = 0u; u < units; ++u) {
        uint32_t list_load[8] = {0u};
        for (i = 0u; i < count[u]; ++i) {
            unsigned int heaviest = i, list = 0u, j;
            uint16_t *row, item;
            for (j = i + 1u; j < count[u]; ++j)
                if (held[u][j] < held[u][heaviest]) heaviest = j; /* lower number: heavier or equal */
            item = held[u][heaviest];
            held[u][heaviest] = held[u][i];
            held[u][i] = item;
            for (k = 1u; k < per_unit; ++k)
                if (list_load[k] < list_load[list]) list = k;
            list_load[list] += steps[item];
            row = rows + (size_t)(u + list * units) * YVEX_ROCM_LIST_STRIDE;
            if (row[0] + 1u >= YVEX_ROCM_LIST_STRIDE) {
                free(block);
                return 0;
            }
            row[1u + row[0]++] = item;
        }
    }
    free(block);
    (void)lists;
    return 1;
}

/* Returns the number of workgroups of the scheduled launch and the device rows, or 0 when the
 * launch keeps one item per workgroup. */
unsigned int yvex_rocm_schedule_lists(yvex_backend *backend, const yvex_rocm_schedule_key *key,
                                      const uint16_t **device_rows)
{
    yvex_rocm_backend_state *state = yvex_rocm_state(backend);
    const unsigned int units = state && state->compute_units > 0 ? (unsigned int)state->compute_units : 0u;
    unsigned long long q_tiles, items;
    unsigned int lists;
    if (!state || !key || !device_rows || !units || !key->per_unit || key->per_unit > 8u ||
        !key->item_rows || !key->step_keys || !key->query_heads || !state->schedule_device)
        return 0u;
    q_tiles = (key->query_tokens + key->item_rows - 1ull) / key->item_rows;
    items = q_tiles * key->query_heads;
    lists = units * key->per_unit;
    if (lists > YVEX_ROCM_LISTS_MAX || items > YVEX_ROCM_LIST_ITEMS_MAX || items <= units) return 0u;
    if (memcmp(&state->schedule.key, key, sizeof(*key)) != 0) {
        /* a new geometry: remembered, and scheduled when it comes again */
        state->schedule.key = *key;
        state->schedule.lists = 0u;
        state->schedule.seen = 1u;
        return 0u;
    }
    if (!state->schedule.lists) {
        /* the copy below reads the host rows and an earlier launch may still read the device
         * rows: a recorded sequence keeps neither alive, and the stream must be idle.  A
         * geometry that could not be scheduled is not tried again */
        if (state->schedule.seen != 1u || state->recording) return 0u;
        state->schedule.seen = 2u;
        if (!lists_build(state, key, (unsigned int)q_tiles, units) ||
            state->driver.hipStreamSynchronize(yvex_rocm_stream(state)) != hipSuccess ||
            state->driver.hipMemcpyAsync(state->schedule_device, state->schedule.rows,
                                         (size_t)lists * YVEX_ROCM_LIST_STRIDE * sizeof(uint16_t),
                                         hipMemcpyHostToDevice, yvex_rocm_stream(state)) != hipSuccess ||
            state->driver.hipStreamSynchronize(yvex_rocm_stream(state)) != hipSuccess)
            return 0u;
        backend->stats.h2d_bytes += (unsigned long long)lists * YVEX_ROCM_LIST_STRIDE * sizeof(uint16_t);
        state->schedule.lists = lists;
    }
    *device_rows = state->schedule_device;
    return lists;
}
