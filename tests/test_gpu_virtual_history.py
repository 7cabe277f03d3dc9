"""GPU: tensors over a reserved address range (reserve / commit_range / decommit), the way
the reference holds an attention history that grows with the sequence
(src/runtime/state_residency.c:258-287,441-446), and decode over such a history.  The
range's bytes are exactly those of an ordinary tensor, so the decode over it must equal the
decode over an ordinary tensor bit for bit, and the CPU oracle within the bf16 bar."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError, lib
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu


def test_virtual_tensor_sequence_of_the_reference_unit_test(backend):
    """The steps of tests/unit/cuda/tensor.c:30-89 on the device."""
    assert lib().yvex_backend_virtual_tensor_supported(backend.handle) == 1
    before = backend.memory_stats().allocated_bytes
    t = backend.reserve("rocm_virtual_pages", B.DTYPE_I8, (64 << 20,))
    g = t.granularity
    assert g and (g & (g - 1)) == 0 and 8 * g <= 64 << 20, g
    assert t.handle.contents.virtual_reserved and t.resident_bytes == 0
    assert backend.memory_stats().allocated_bytes == before
    assert t.commit(g + 1, 1) == g and t.resident_bytes == g
    assert t.commit(g + 2, 1) == 0 and t.resident_bytes == g
    assert t.commit(3 * g, 1) == g and t.resident_bytes == 2 * g
    view = t.view(g + 1, B.DTYPE_I8, (1,))
    view.write(np.array([0x5a], np.int8))
    assert view.read()[0] == 0x5a
    assert np.all(t.view(3 * g, B.DTYPE_I8, (g,)).read() == 0)       # committed pages read as zero
    assert backend.memory_stats().allocated_bytes == before + 2 * g
    with pytest.raises(YvexError) as e:                              # a hole is never touched
        t.view(g, B.DTYPE_I8, (2 * g + 1,)).read()
    assert e.value.code == B.YVEX_ERR_STATE
    assert t.decommit() == 2 * g and t.resident_bytes == 0
    assert backend.memory_stats().allocated_bytes == before
    assert t.commit(g + 1, 1) == g                                   # the range is still owned,
    assert t.view(g + 1, B.DTYPE_I8, (1,)).read()[0] == 0            # and the old byte is gone
    t.release()
    assert backend.memory_stats().allocated_bytes == before


def test_decode_over_a_history_that_is_committed_as_it_grows(backend):
    """One layer's interleaved [K|V] history rows (src/runtime/stateful_attention.c:326-352) in
    a reserved range of 32768 rows; the context grows in three steps, each committing only the
    rows it adds, and every step decodes one token over the rows so far."""
    hq, hkv, d, capacity = 32, 8, 128, 32768
    width = hkv * d
    row_bytes = 2 * width * 2
    rng = np.random.default_rng(2718)
    k = bf16_normal(rng, (capacity, hkv, d))
    v = bf16_normal(rng, (capacity, hkv, d))
    rows = np.empty((capacity, 2 * width), np.uint16)
    rows[:, :width] = k.reshape(capacity, width)
    rows[:, width:] = v.reshape(capacity, width)
    base = backend.memory_stats().allocated_bytes
    history = backend.reserve("history", B.DTYPE_BF16, (capacity, 2 * width))
    g = history.granularity
    have = 0
    for tokens in (100, 4096, 21000):
        delta = history.commit(have * row_bytes, (tokens - have) * row_bytes)
        assert delta % g == 0 and history.resident_bytes == -(-tokens * row_bytes // g) * g
        assert backend.memory_stats().allocated_bytes == base + history.resident_bytes
        history.view(have * row_bytes, B.DTYPE_BF16, (tokens - have, 2 * width)).write(rows[have:tokens])
        have = tokens
        q = bf16_normal(rng, (1, hq, d))
        req = backend.attention_requirement(1, tokens, hq, hkv, d, causal=True,
                                            query_start=tokens - 1, dtype=B.DTYPE_BF16,
                                            contract=B.NUMERIC_BF16_F32_ACCUMULATE,
                                            k_stride=2 * width, v_stride=2 * width)
        count = (tokens - 1) * 2 * width + width
        tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
        out = backend.tensor("o", B.DTYPE_BF16, q.shape)
        lse = backend.tensor("lse", B.DTYPE_F32, (1, hq))
        # the views carry is_written from the struct they copy: mark the range written first
        history.handle.contents.is_written = 1
        backend.attention_execute(req, tq, history.view(0, B.DTYPE_BF16, (count,)),
                                  history.view(width * 2, B.DTYPE_BF16, (count,)), out, lse=lse)
        got, got_lse = out.read(), lse.read()
        plain = backend.tensor("plain", B.DTYPE_BF16, (tokens, 2 * width), rows[:tokens])
        out2 = backend.tensor("o2", B.DTYPE_BF16, q.shape)
        lse2 = backend.tensor("lse2", B.DTYPE_F32, (1, hq))
        backend.attention_execute(req, tq, plain.view(0, B.DTYPE_BF16, (count,)),
                                  plain.view(width * 2, B.DTYPE_BF16, (count,)), out2, lse=lse2)
        assert np.array_equal(got, out2.read()) and np.array_equal(got_lse, lse2.read())
        rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k[:tokens], v[:tokens], query_start=tokens - 1,
                                              causal=True)
        assert rc == 0
        assert_close_bf16(got, ref, "history %d" % tokens)
        assert_lse(got_lse, ref_lse, "history %d" % tokens)
        # one row past the committed rows may or may not share the last granule; a request
        # that reaches past the last committed granule is refused before anything is launched
        beyond = history.resident_bytes // row_bytes + 1
        if beyond <= capacity:
            far = backend.attention_requirement(1, beyond, hq, hkv, d, causal=True,
                                                query_start=beyond - 1, dtype=B.DTYPE_BF16,
                                                contract=B.NUMERIC_BF16_F32_ACCUMULATE,
                                                k_stride=2 * width, v_stride=2 * width)
            far_count = (beyond - 1) * 2 * width + width
            with pytest.raises(YvexError) as e:
                backend.attention_execute(far, tq, history.view(0, B.DTYPE_BF16, (far_count,)),
                                          history.view(width * 2, B.DTYPE_BF16, (far_count,)), out)
            assert e.value.code == B.YVEX_ERR_STATE and "not committed" in e.value.message
        for tensor in (tq, out, lse, plain, out2, lse2):
            tensor.release()
    assert history.decommit() == -(-have * row_bytes // g) * g
    assert backend.memory_stats().allocated_bytes == base
    history.release()


def test_paged_decode_over_page_pools_committed_up_to_the_pages_in_use(backend):
    """K and V page pools reserved for 4096 pages each, committed only up to the pages handed
    out so far; the request names the committed prefix as its pool."""
    from clori_amd.backend import kv_pack_pages
    from test_gpu_decode import make_paged_case
    hq, hkv, d = 32, 8, 128
    rng = np.random.default_rng(31415)
    contexts = [700, 16, 3000, 1025]
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, hq, hkv)
    kp = kv_pack_pages(k_rows, B.KV_BF16, False, hkv).view(np.uint16)
    vp = kv_pack_pages(v_rows, B.KV_BF16, True, hkv).view(np.uint16)
    page_elems = kp.size // pool_pages
    capacity = 4096
    pools = [backend.reserve(name, B.DTYPE_BF16, (capacity * page_elems,)) for name in ("k", "v")]
    views = []
    for pool, packed in zip(pools, (kp, vp)):
        assert pool.commit(0, packed.nbytes) == -(-packed.nbytes // pool.granularity) * pool.granularity
        pool.view(0, B.DTYPE_BF16, (packed.size,)).write(packed)
        pool.handle.contents.is_written = 1
        views.append(pool.view(0, B.DTYPE_BF16, (packed.size,)))
    plain = [backend.tensor(name, B.DTYPE_BF16, (packed.size,), packed)
             for name, packed in (("kp", kp), ("vp", vp))]
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tt = backend.tensor("table", B.DTYPE_I32, table.shape, table)
    tc = backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)
    req = backend.paged_requirement(len(contexts), hq, hkv, d, 16, pool_pages, table.shape[1],
                                    int(table.shape[1] * 16))
    results = []
    for key_pages, value_pages in (views, plain):
        out = backend.tensor("o", B.DTYPE_BF16, q.shape)
        lse = backend.tensor("lse", B.DTYPE_F32, (len(contexts), hq))
        backend.paged_decode_execute(req, tq, key_pages, value_pages, tt, tc, out, lse)
        results.append((out.read(), lse.read()))
        out.release()
        lse.release()
    assert np.array_equal(results[0][0], results[1][0]) and np.array_equal(results[0][1], results[1][1])
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, hkv, 16)
    assert rc == 0
    assert_close_bf16(results[0][0], ref, "paged over a reserved range")
    assert_lse(results[0][1], ref_lse, "paged over a reserved range")
    # a pool that claims pages beyond the committed granules is refused, nothing is launched
    wide = pools[0].resident_bytes // (page_elems * 2) + 1
    far = backend.paged_requirement(len(contexts), hq, hkv, d, 16, wide, table.shape[1],
                                    int(table.shape[1] * 16))
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    with pytest.raises(YvexError) as e:
        backend.paged_decode_execute(far, tq, pools[0].view(0, B.DTYPE_BF16, (wide * page_elems,)),
                                     pools[1].view(0, B.DTYPE_BF16, (wide * page_elems,)), tt, tc, out)
    assert e.value.code == B.YVEX_ERR_STATE
    for tensor in pools + plain + [tq, tt, tc, out]:
        tensor.release()
