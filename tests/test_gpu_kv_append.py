"""GPU parity: the KV page writer (rotary on the keys, bf16 and Q8_0 pages) against the CPU
restatement, bit for bit, through the C ABI; then decode over the pages it wrote."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError, kv_pack_pages, kv_unpack_pages, q8_0_encode_rows
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu

HKV, D, PAGE = 8, 128, 16


def expected_rows(canonical, k_new, v_new, table, starts, counts, row_starts, q8):
    """Applies the append on the canonical [page][token][head][row] host copy."""
    k_rows, v_rows = canonical
    for s in range(len(starts)):
        for i in range(counts[s]):
            pos = starts[s] + i
            page, slot = table[s, pos // PAGE], pos % PAGE
            for pool, new in ((k_rows, k_new), (v_rows, v_new)):
                row = new[row_starts[s] + i]
                pool[page, slot] = q8_0_encode_rows(ORACLE.bf16_decode(row)).reshape(HKV, -1) \
                    if q8 else row
    return k_rows, v_rows


def run_case(backend, rng, starts, counts, storage, rotary_dim, pool_state="zero",
             rotary_mode=B.ROTARY_BF16_STAGED, d=D):
    sessions = len(starts)
    q8 = storage == B.KV_Q8_0
    stride = max((s + c + PAGE - 1) // PAGE for s, c in zip(starts, counts)) + 1
    pool_pages = sessions * stride + 3
    table = rng.permutation(pool_pages)[:sessions * stride].astype(np.int32).reshape(sessions, stride)
    total = int(sum(counts))
    row_starts = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    k_new = bf16_normal(rng, (total, HKV, d))
    v_new = bf16_normal(rng, (total, HKV, d))
    angles = rng.uniform(-3.0, 3.0, size=(total, max(rotary_dim, 16))).astype(np.float32)
    cosine, sine = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    # pools start either zeroed or holding earlier tokens everywhere
    row_width = (d // 32) * 34 if q8 else d
    row_dtype = np.uint8 if q8 else np.uint16
    if pool_state == "zero":
        k_rows = np.zeros((pool_pages, PAGE, HKV, row_width), row_dtype)
        v_rows = np.zeros((pool_pages, PAGE, HKV, row_width), row_dtype)
    else:
        old_k, old_v = bf16_normal(rng, (pool_pages, PAGE, HKV, d)), bf16_normal(rng, (pool_pages, PAGE, HKV, d))
        k_rows = q8_0_encode_rows(ORACLE.bf16_decode(old_k)).reshape(pool_pages, PAGE, HKV, -1) if q8 else old_k
        v_rows = q8_0_encode_rows(ORACLE.bf16_decode(old_v)).reshape(pool_pages, PAGE, HKV, -1) if q8 else old_v
    pool_dtype = B.DTYPE_I8 if q8 else B.DTYPE_BF16
    kp = kv_pack_pages(k_rows, storage, False, HKV, head_dim=d)
    vp = kv_pack_pages(v_rows, storage, True, HKV, head_dim=d)
    elems = kp.size // B.DTYPE_BYTES[pool_dtype]
    t = dict(
        key=backend.tensor("k-new", B.DTYPE_BF16, k_new.shape, k_new),
        value=backend.tensor("v-new", B.DTYPE_BF16, v_new.shape, v_new),
        cosine=backend.tensor("cos", B.DTYPE_F32, cosine.shape, cosine),
        sine=backend.tensor("sin", B.DTYPE_F32, sine.shape, sine),
        row_start=backend.tensor("rows", B.DTYPE_I32, (sessions,), row_starts),
        position_start=backend.tensor("starts", B.DTYPE_I32, (sessions,), np.array(starts, np.int32)),
        token_count=backend.tensor("counts", B.DTYPE_I32, (sessions,), np.array(counts, np.int32)),
        page_table=backend.tensor("table", B.DTYPE_I32, table.shape, table),
        k_pool=backend.tensor("kpool", pool_dtype, (elems,), kp),
        v_pool=backend.tensor("vpool", pool_dtype, (elems,), vp))
    use_rotary = rotary_dim > 0
    facts = backend.kv_append_execute(
        t["key"], t["value"], t["row_start"], t["position_start"], t["token_count"],
        t["page_table"], t["k_pool"], t["v_pool"], HKV, pool_pages, max(max(counts), 1),
        storage=storage, cosine=t["cosine"] if use_rotary else None,
        sine=t["sine"] if use_rotary else None, rotary_dimension=rotary_dim,
        rotary_mode=rotary_mode, head_dimension=d)
    assert facts.kernel_launches == 1
    got_k = kv_unpack_pages(t["k_pool"].read(np.uint8, (-1,)), storage, False, pool_pages, HKV, head_dim=d)
    got_v = kv_unpack_pages(t["v_pool"].read(np.uint8, (-1,)), storage, True, pool_pages, HKV, head_dim=d)
    if use_rotary and rotary_mode == B.ROTARY_F32_ROUNDED:
        k_rot = ORACLE.bf16_encode(ORACLE.rotary_half_f32_rounded(
            ORACLE.bf16_decode(k_new), cosine[:, :rotary_dim], sine[:, :rotary_dim], rotary_dim))
    elif use_rotary:
        k_rot = ORACLE.rotary_half_bf16(k_new, cosine[:, :rotary_dim], sine[:, :rotary_dim], rotary_dim)
    else:
        k_rot = k_new
    want_k, want_v = expected_rows((k_rows.copy(), v_rows.copy()), k_rot, v_new, table, starts,
                                   counts, row_starts, q8)
    return t, (got_k, got_v), (want_k, want_v), table, pool_pages


@pytest.mark.parametrize("storage", [B.KV_BF16, B.KV_Q8_0], ids=["bf16", "q8_0"])
@pytest.mark.parametrize("rotary_dim", [0, 64, 128])
def test_append_writes_exactly_the_host_layout(backend, storage, rotary_dim):
    """Decode-style (one token) and prefill-style (many tokens, unaligned starts) appends into
    pools that already hold other tokens: every byte of both pools equals the host-side
    restatement (rotary, Q8_0 encoder, page packer), untouched tokens included."""
    rng = np.random.default_rng(11 + rotary_dim)
    starts, counts = [0, 5, 16, 31, 47, 100], [1, 1, 40, 0, 17, 33]
    t, got, want, _, _ = run_case(backend, rng, starts, counts, storage, rotary_dim, "filled")
    assert np.array_equal(got[0].reshape(want[0].shape), want[0])
    assert np.array_equal(got[1].reshape(want[1].shape), want[1])
    for x in t.values():
        x.release()


@pytest.mark.parametrize("storage", [B.KV_BF16, B.KV_Q8_0], ids=["bf16", "q8_0"])
@pytest.mark.parametrize("rotary_dim", [32, 128])
def test_append_in_the_decoder_order_of_rotary(backend, storage, rotary_dim):
    """The same appends with the rotation the reference's decoder runs in front of attention
    (src/runtime/decoder.c:1112-1131): plain F32 rotation, one bf16 rounding.  Byte-exact
    against that restatement, and different from the staged order somewhere."""
    rng = np.random.default_rng(31 + rotary_dim)
    starts, counts = [3, 0, 50, 16], [44, 1, 0, 130]
    t, got, want, _, _ = run_case(backend, rng, starts, counts, storage, rotary_dim, "filled",
                                  rotary_mode=B.ROTARY_F32_ROUNDED)
    assert np.array_equal(got[0].reshape(want[0].shape), want[0])
    assert np.array_equal(got[1].reshape(want[1].shape), want[1])
    for x in t.values():
        x.release()
    if storage == B.KV_BF16:
        rng = np.random.default_rng(31 + rotary_dim)
        t2, staged, _, _, _ = run_case(backend, rng, starts, counts, storage, rotary_dim, "filled")
        differing = np.count_nonzero(staged[0].reshape(want[0].shape) != want[0])
        # the orders differ by roundings only, but in a good part of the rotated values
        assert 0 < differing < want[0].size // 2
        apart = np.abs(ORACLE.bf16_decode(staged[0].reshape(want[0].shape)).astype(np.float64) -
                       ORACLE.bf16_decode(want[0]).astype(np.float64))
        assert apart.max() <= 2.0 ** -5
        for x in t2.values():
            x.release()
    with pytest.raises(YvexError) as e:
        run_case(backend, np.random.default_rng(1), [0], [1], storage, rotary_dim, rotary_mode=2)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED


def test_decode_over_appended_pages_matches_cpu_operator(backend):
    """Prefill-style append of whole contexts, then paged decode on those pages."""
    rng = np.random.default_rng(21)
    contexts = [700, 129, 2049]
    t, got, want, table, pool_pages = run_case(backend, rng, [0, 0, 0], contexts, B.KV_BF16, 128)
    assert np.array_equal(got[0].reshape(want[0].shape), want[0])
    q = bf16_normal(rng, (len(contexts), 32, D))
    ctx = np.array(contexts, np.int32)
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tc = backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    lse = backend.tensor("lse", B.DTYPE_F32, (len(contexts), 32))
    req = backend.paged_requirement(len(contexts), 32, HKV, D, PAGE, pool_pages, table.shape[1],
                                    int(table.shape[1] * PAGE), storage=B.KV_BF16)
    backend.paged_decode_execute(req, tq, t["k_pool"], t["v_pool"], t["page_table"], tc, out, lse)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, want[0], want[1], table, ctx, HKV, PAGE)
    assert rc == 0
    assert_close_bf16(out.read(), ref, "decode after append")
    assert_lse(lse.read(), ref_lse, "decode after append")


def small_append(backend, k_new, start, count, pool_pages=4):
    table = np.array([[0, 1]], np.int32)
    tensors = [
        backend.tensor("k", B.DTYPE_BF16, k_new.shape, k_new),
        backend.tensor("v", B.DTYPE_BF16, k_new.shape, k_new),
        backend.tensor("r", B.DTYPE_I32, (1,), np.array([0], np.int32)),
        backend.tensor("s", B.DTYPE_I32, (1,), np.array([start], np.int32)),
        backend.tensor("c", B.DTYPE_I32, (1,), np.array([count], np.int32)),
        backend.tensor("t", B.DTYPE_I32, table.shape, table),
        backend.tensor("kp", B.DTYPE_BF16, (pool_pages * HKV * PAGE * D,)),
        backend.tensor("vp", B.DTYPE_BF16, (pool_pages * HKV * PAGE * D,))]
    try:
        return backend.kv_append_execute(*tensors, HKV, pool_pages, count)
    finally:
        for x in tensors:
            x.release()


def test_q8_0_ties_round_half_away_from_zero(backend):
    """Blocks whose scale is exactly 1 and whose values sit on k + 0.5: the reference encoder
    rounds them away from zero (roundf); also the largest magnitudes and signed zeros."""
    ladder = np.array([127.0] + [k + 0.5 for k in range(0, 31)], np.float32)
    rows = np.zeros((3, HKV, D), np.float32)
    for h in range(HKV):
        rows[0, h] = np.tile(ladder, 4) * np.where(np.arange(D) % 3 == h % 3, -1.0, 1.0)
        rows[1, h] = np.tile(np.array([127.0, 126.5, -126.5, 125.5, -0.0, 0.0, 63.5, -64.5] * 4,
                                      np.float32), 4)
        rows[2, h] = np.tile(ladder[::-1], 4) * 2.0 ** (h - 4)      # other exact scales
    new = ORACLE.bf16_encode(rows)
    assert np.array_equal(ORACLE.bf16_decode(new), rows)            # all bf16-representable
    table = np.array([[1, 0]], np.int32)
    pool_bytes = 2 * HKV * 2176
    tensors = [backend.tensor("k", B.DTYPE_BF16, new.shape, new),
               backend.tensor("v", B.DTYPE_BF16, new.shape, new[::-1].copy()),
               backend.tensor("r", B.DTYPE_I32, (1,), np.array([0], np.int32)),
               backend.tensor("s", B.DTYPE_I32, (1,), np.array([14], np.int32)),
               backend.tensor("c", B.DTYPE_I32, (1,), np.array([3], np.int32)),
               backend.tensor("t", B.DTYPE_I32, table.shape, table),
               backend.tensor("kp", B.DTYPE_I8, (pool_bytes,)),
               backend.tensor("vp", B.DTYPE_I8, (pool_bytes,))]
    tensors[6].zero()
    tensors[7].zero()
    backend.kv_append_execute(*tensors, HKV, 2, 3, storage=B.KV_Q8_0)
    want = q8_0_encode_rows(rows).reshape(3, HKV, -1)
    for pool, rows_in in ((tensors[6], want), (tensors[7], want[::-1])):
        got = kv_unpack_pages(pool.read(np.uint8, (-1,)), B.KV_Q8_0, False if pool is tensors[6] else True,
                              2, HKV).reshape(2, PAGE, HKV, -1)
        # positions 14, 15 -> page id 1 slots 14, 15; position 16 -> page id 0 slot 0
        assert np.array_equal(got[1, 14], rows_in[0])
        assert np.array_equal(got[1, 15], rows_in[1])
        assert np.array_equal(got[0, 0], rows_in[2])
    for x in tensors:
        x.release()


def test_append_refusals(backend):
    rng = np.random.default_rng(31)
    # the same call inside the table succeeds
    small_append(backend, bf16_normal(rng, (4, HKV, D)), 20, 4)
    # a run that leaves the two-page table: device contract -> BOUNDS
    with pytest.raises(YvexError) as e:
        small_append(backend, bf16_normal(rng, (4, HKV, D)), 30, 4)
    assert e.value.code == B.YVEX_ERR_BOUNDS
    # more tokens in a session than the request declared -> BOUNDS, nothing dropped silently
    with pytest.raises(YvexError) as e:
        k_new = bf16_normal(rng, (32, HKV, D))
        tensors = [backend.tensor("k", B.DTYPE_BF16, k_new.shape, k_new),
                   backend.tensor("v", B.DTYPE_BF16, k_new.shape, k_new),
                   backend.tensor("r", B.DTYPE_I32, (1,), np.array([0], np.int32)),
                   backend.tensor("s", B.DTYPE_I32, (1,), np.array([0], np.int32)),
                   backend.tensor("c", B.DTYPE_I32, (1,), np.array([32], np.int32)),
                   backend.tensor("t", B.DTYPE_I32, (1, 2), np.array([[0, 1]], np.int32)),
                   backend.tensor("kp", B.DTYPE_BF16, (4 * HKV * PAGE * D,)),
                   backend.tensor("vp", B.DTYPE_BF16, (4 * HKV * PAGE * D,))]
        backend.kv_append_execute(*tensors, HKV, 4, 1)        # declared: one token per session
    assert e.value.code == B.YVEX_ERR_BOUNDS
    # a NaN key -> FORMAT
    k_bad = bf16_normal(rng, (2, HKV, D))
    k_bad[1, 3, 7] = 0x7FC0
    with pytest.raises(YvexError) as e:
        small_append(backend, k_bad, 0, 2)
    assert e.value.code == B.YVEX_ERR_FORMAT
    # a Q8_0 block whose scale overflows f16 (max / 127 > 65504) -> FORMAT, as the encoder refuses it
    huge = bf16_normal(rng, (1, HKV, D))
    huge[0, 2, 40] = ORACLE.bf16_encode(np.array([1.0e7], np.float32))[0]
    tensors = [backend.tensor("k", B.DTYPE_BF16, huge.shape, huge),
               backend.tensor("v", B.DTYPE_BF16, huge.shape, huge),
               backend.tensor("r", B.DTYPE_I32, (1,), np.array([0], np.int32)),
               backend.tensor("s", B.DTYPE_I32, (1,), np.array([0], np.int32)),
               backend.tensor("c", B.DTYPE_I32, (1,), np.array([1], np.int32)),
               backend.tensor("t", B.DTYPE_I32, (1, 2), np.array([[0, 1]], np.int32)),
               backend.tensor("kp", B.DTYPE_I8, (4 * HKV * 2176,)),
               backend.tensor("vp", B.DTYPE_I8, (4 * HKV * 2176,))]
    with pytest.raises(YvexError) as e:
        backend.kv_append_execute(*tensors, HKV, 4, 1, storage=B.KV_Q8_0)
    assert e.value.code == B.YVEX_ERR_FORMAT
    # rotary dimension that is not a multiple of 16 -> UNSUPPORTED (refused on the host)
    with pytest.raises(YvexError) as e:
        run_case(backend, rng, [0], [1], B.KV_BF16, 24)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED


@pytest.mark.parametrize("storage", [B.KV_BF16, B.KV_Q8_0], ids=["bf16", "q8_0"])
def test_append_into_pages_of_64_tokens(backend, storage):
    """The page writer with pages of 64 tokens (four 16-token blocks per page and kv head):
    every byte of both pools against the host-side restatement, then decode over them."""
    rng = np.random.default_rng(640 + storage)
    q8 = storage == B.KV_Q8_0
    page, rotary_dim = 64, 64
    starts, counts = [0, 61, 130, 64, 200], [1, 10, 300, 0, 77]
    sessions = len(starts)
    stride = max((s + c + page - 1) // page for s, c in zip(starts, counts)) + 1
    pool_pages = sessions * stride + 2
    table = rng.permutation(pool_pages)[:sessions * stride].astype(np.int32).reshape(sessions, stride)
    total = int(sum(counts))
    row_starts = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    k_new, v_new = bf16_normal(rng, (total, HKV, D)), bf16_normal(rng, (total, HKV, D))
    angles = rng.uniform(-3.0, 3.0, size=(total, rotary_dim)).astype(np.float32)
    cosine, sine = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
    old_k, old_v = bf16_normal(rng, (pool_pages, page, HKV, D)), bf16_normal(rng, (pool_pages, page, HKV, D))

    def stored(rows):
        return q8_0_encode_rows(ORACLE.bf16_decode(rows)).reshape(rows.shape[:-1] + (-1,)) if q8 else rows
    k_rows, v_rows = stored(old_k), stored(old_v)
    pool_dtype = B.DTYPE_I8 if q8 else B.DTYPE_BF16
    kp = kv_pack_pages(k_rows, storage, False, HKV, page_tokens=page)
    vp = kv_pack_pages(v_rows, storage, True, HKV, page_tokens=page)
    elems = kp.size // B.DTYPE_BYTES[pool_dtype]
    t = [backend.tensor("k-new", B.DTYPE_BF16, k_new.shape, k_new),
         backend.tensor("v-new", B.DTYPE_BF16, v_new.shape, v_new),
         backend.tensor("rows", B.DTYPE_I32, (sessions,), row_starts),
         backend.tensor("starts", B.DTYPE_I32, (sessions,), np.array(starts, np.int32)),
         backend.tensor("counts", B.DTYPE_I32, (sessions,), np.array(counts, np.int32)),
         backend.tensor("table", B.DTYPE_I32, table.shape, table),
         backend.tensor("kpool", pool_dtype, (elems,), kp),
         backend.tensor("vpool", pool_dtype, (elems,), vp)]
    tc = backend.tensor("cos", B.DTYPE_F32, cosine.shape, cosine)
    ts = backend.tensor("sin", B.DTYPE_F32, sine.shape, sine)
    facts = backend.kv_append_execute(*t, HKV, pool_pages, max(counts), storage=storage, cosine=tc, sine=ts,
                                      rotary_dimension=rotary_dim, page_tokens=page)
    assert facts.kernel_launches == 1
    k_rot = ORACLE.rotary_half_bf16(k_new, cosine, sine, rotary_dim)
    want_k, want_v = k_rows.copy(), v_rows.copy()
    for s in range(sessions):
        for i in range(counts[s]):
            position = starts[s] + i
            want_k[table[s, position // page], position % page] = stored(k_rot[row_starts[s] + i][None])[0]
            want_v[table[s, position // page], position % page] = stored(v_new[row_starts[s] + i][None])[0]
    got_k = kv_unpack_pages(t[6].read(np.uint8, (-1,)), storage, False, pool_pages, HKV, page_tokens=page)
    got_v = kv_unpack_pages(t[7].read(np.uint8, (-1,)), storage, True, pool_pages, HKV, page_tokens=page)
    assert np.array_equal(got_k.reshape(want_k.shape), want_k)
    assert np.array_equal(got_v.reshape(want_v.shape), want_v)
    # decode over what was written
    ctx = np.array([s + c for s, c in zip(starts, counts)], np.int32)
    q = bf16_normal(rng, (sessions, 32, D))
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tctx = backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    req = backend.paged_requirement(sessions, 32, HKV, D, page, pool_pages, stride, stride * page,
                                    storage=storage)
    backend.paged_decode_execute(req, tq, t[6], t[7], t[5], tctx, out)
    rc, ref, _, _ = ORACLE.paged_decode(q, want_k, want_v, table, ctx, HKV, page, q8=q8)
    assert rc == 0
    assert_close_bf16(out.read(), ref, "decode over 64-token pages")
    for x in t + [tc, ts, tq, tctx, out]:
        x.release()


@pytest.mark.parametrize("d,rotary_dim", [(64, 0), (64, 32), (64, 64), (256, 0), (256, 64), (256, 256)])
@pytest.mark.parametrize("rotary_mode", [B.ROTARY_BF16_STAGED, B.ROTARY_F32_ROUNDED], ids=["staged", "decoder"])
def test_append_bf16_pages_at_other_head_dimensions(backend, d, rotary_dim, rotary_mode):
    """bf16 pages at head dimension 64 and 256: every byte of both pools against the host-side
    restatement, pools that already hold other tokens, both rotary orders, then a decode over
    the written pages against the oracle."""
    rng = np.random.default_rng(500 + d + rotary_dim)
    starts, counts = [0, 5, 16, 31, 47, 100], [1, 1, 40, 0, 17, 33]
    t, got, want, table, pool_pages = run_case(backend, rng, starts, counts, B.KV_BF16, rotary_dim,
                                               "filled", rotary_mode=rotary_mode, d=d)
    assert np.array_equal(got[0].reshape(want[0].shape), want[0])
    assert np.array_equal(got[1].reshape(want[1].shape), want[1])
    hq = 2 * HKV
    contexts = np.array([s + c for s, c in zip(starts, counts)], np.int32)
    q = bf16_normal(rng, (len(starts), hq, d))
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tc = backend.tensor("ctx", B.DTYPE_I32, contexts.shape, contexts)
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    lse = backend.tensor("lse", B.DTYPE_F32, (len(starts), hq))
    req = backend.paged_requirement(len(starts), hq, HKV, d, PAGE, pool_pages, table.shape[1],
                                    int(table.shape[1] * PAGE))
    backend.paged_decode_execute(req, tq, t["k_pool"], t["v_pool"], t["page_table"], tc, out, lse)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, want[0], want[1], table, contexts, HKV, PAGE)
    assert rc == 0
    assert_close_bf16(out.read(), ref, "decode over appended pages d=%d" % d)
    assert_lse(lse.read(), ref_lse, "decode over appended pages d=%d" % d)
    for x in list(t.values()) + [tq, tc, out, lse]:
        x.release()
