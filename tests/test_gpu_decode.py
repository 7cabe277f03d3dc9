"""GPU parity: split-K decode (token-major and paged bf16) against the CPU oracle,
called through the C ABI."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError, kv_pack_pages
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu


def run_rows_decode(backend, q, k, v, query_start, causal=True, k_stride=0, v_stride=0,
                    kv_storage=None):
    """q uint16 [1,Hq,d]; k/v uint16 [Tk,Hkv,d] (or interleaved storage with strides)."""
    _, hq, d = q.shape
    tk, hkv = k.shape[0], k.shape[1]
    req = backend.attention_requirement(1, tk, hq, hkv, d, causal=causal, query_start=query_start,
                                        dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE,
                                        k_stride=k_stride, v_stride=v_stride)
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    if kv_storage is None:
        tk_ = backend.tensor("k", B.DTYPE_BF16, k.shape, k)
        tv_ = backend.tensor("v", B.DTYPE_BF16, v.shape, v)
    else:
        store = backend.tensor("kv", B.DTYPE_BF16, kv_storage.shape, kv_storage)
        width = hkv * d
        count = (tk - 1) * k_stride + width
        tk_ = store.view(0, B.DTYPE_BF16, (count,))
        tv_ = store.view(width * 2, B.DTYPE_BF16, (count,))
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    lse = backend.tensor("lse", B.DTYPE_F32, (1, hq))
    facts = backend.attention_execute(req, tq, tk_, tv_, out, lse=lse)
    result = out.read(), lse.read(), facts
    return result


def test_config1_contiguous_decode_matches_cpu_operator(backend):
    """Benchmark configuration 1: B=1, 32/8 heads, d=128, ctx 4096, contiguous KV, seed 1."""
    rng = np.random.default_rng(1)
    q = bf16_normal(rng, (1, 32, 128))
    k = bf16_normal(rng, (4096, 8, 128))
    v = bf16_normal(rng, (4096, 8, 128))
    got, lse, facts = run_rows_decode(backend, q, k, v, query_start=4095)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=4095, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, "config1")
    assert_lse(lse, ref_lse, "config1")
    assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
    assert facts.temporary_bytes > 0


@pytest.mark.parametrize("ctx", [1, 2, 15, 16, 17, 63, 64, 65, 1000, 1025])
def test_rows_decode_ragged_lengths(backend, ctx):
    rng = np.random.default_rng(100 + ctx)
    q = bf16_normal(rng, (1, 8, 128))
    k = bf16_normal(rng, (ctx + 3, 2, 128))
    v = bf16_normal(rng, (ctx + 3, 2, 128))
    got, lse, _ = run_rows_decode(backend, q, k, v, query_start=ctx - 1)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, "ctx=%d" % ctx)
    assert_lse(lse, ref_lse, "ctx=%d" % ctx)
    # FULL mask sees the rows past the query position too
    got, lse, _ = run_rows_decode(backend, q, k, v, query_start=ctx - 1, causal=False)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=False)
    assert_close_bf16(got, ref, "full ctx=%d" % ctx)
    assert_lse(lse, ref_lse, "full ctx=%d" % ctx)


@pytest.mark.parametrize("hq,hkv,ctx", [(1, 1, 700), (4, 2, 5000), (10, 2, 300), (64, 8, 9000),
                                        (8, 1, 20000), (32, 2, 2100), (16, 1, 33)])
def test_rows_decode_group_sizes_and_team_counts(backend, hq, hkv, ctx):
    """One query token over a token-major history: groups of 1 to 8 query heads per kv head go
    through teams of eight waves (1, few, 16 and the maximum of 32 teams per kv head: one and
    two load trips of the last team's merge), wider groups through one wave per stretch."""
    rng = np.random.default_rng(hq * 100000 + ctx)
    q = bf16_normal(rng, (1, hq, 128))
    k = bf16_normal(rng, (ctx, hkv, 128))
    v = bf16_normal(rng, (ctx, hkv, 128))
    got, lse, facts = run_rows_decode(backend, q, k, v, query_start=ctx - 1)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=True)
    assert rc == 0
    label = "hq=%d hkv=%d ctx=%d" % (hq, hkv, ctx)
    assert_close_bf16(got, ref, label)
    assert_lse(lse, ref_lse, label)
    assert facts.kernel_launches == 1
    again, lse_again, _ = run_rows_decode(backend, q, k, v, query_start=ctx - 1)
    assert np.array_equal(got, again) and np.array_equal(lse, lse_again)


def test_rows_decode_interleaved_kv_history_rows(backend):
    """The reference caller passes K at offset 0 and V at offset kv_width of one interleaved
    [K|V] history row with stride 2*kv_width (src/runtime/stateful_attention.c:326-352)."""
    rng = np.random.default_rng(7)
    tk, hq, hkv, d = 300, 16, 4, 128
    q = bf16_normal(rng, (1, hq, d))
    k = bf16_normal(rng, (tk, hkv, d))
    v = bf16_normal(rng, (tk, hkv, d))
    width = hkv * d
    store = np.zeros((tk, 2 * width), dtype=np.uint16)
    store[:, :width] = k.reshape(tk, width)
    store[:, width:] = v.reshape(tk, width)
    got, lse, _ = run_rows_decode(backend, q, k, v, query_start=tk - 1, k_stride=2 * width,
                                  v_stride=2 * width, kv_storage=store)
    packed, lse2, _ = run_rows_decode(backend, q, k, v, query_start=tk - 1)
    assert np.array_equal(got, packed) and np.array_equal(lse, lse2)   # strided == packed, bit for bit
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=tk - 1, causal=True)
    assert_close_bf16(got, ref, "interleaved")


@pytest.mark.parametrize("d", [64, 256])
@pytest.mark.parametrize("hq,hkv,ctx", [(24, 4, 4096), (1, 1, 1), (8, 1, 17), (6, 2, 1000), (16, 2, 9000),
                                        (4, 4, 40000), (32, 2, 700)])
def test_rows_decode_other_head_dimensions(backend, d, hq, hkv, ctx):
    """One query token over a token-major history at head dimension 64 and 256 (the reference's
    own Qwen pattern is 24/4/256, tests/unit/cuda/quant_qtype.c:2413-2418): teams of waves as at
    128 for groups of at most eight query heads (partials in the workspace once there is more
    than one team), a one-row tile of the prefill kernel for wider groups.  Packed and
    interleaved [K|V] rows give the same bits; the FULL mask sees the rows behind the query."""
    rng = np.random.default_rng(d * 1000003 + hq * 1009 + ctx)
    q = bf16_normal(rng, (1, hq, d))
    k = bf16_normal(rng, (ctx + 2, hkv, d))
    v = bf16_normal(rng, (ctx + 2, hkv, d))
    label = "d=%d hq=%d hkv=%d ctx=%d" % (d, hq, hkv, ctx)
    got, lse, facts = run_rows_decode(backend, q, k, v, query_start=ctx - 1)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, label)
    assert_lse(lse, ref_lse, label)
    assert facts.kernel_launches == 1
    assert (facts.temporary_bytes > 0) == (hq // hkv <= 8), label   # teams leave partials, the tile none
    again, lse_again, _ = run_rows_decode(backend, q, k, v, query_start=ctx - 1)
    assert np.array_equal(got, again) and np.array_equal(lse, lse_again)
    width, tk = hkv * d, ctx + 2
    store = np.zeros((tk, 2 * width), dtype=np.uint16)
    store[:, :width] = k.reshape(tk, width)
    store[:, width:] = v.reshape(tk, width)
    strided, lse_strided, _ = run_rows_decode(backend, q, k, v, query_start=ctx - 1, k_stride=2 * width,
                                              v_stride=2 * width, kv_storage=store)
    assert np.array_equal(got, strided) and np.array_equal(lse, lse_strided)
    if ctx <= 9000:
        full, lse_full, _ = run_rows_decode(backend, q, k, v, query_start=ctx - 1, causal=False)
        rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=False)
        assert_close_bf16(full, ref, "full " + label)
        assert_lse(lse_full, ref_lse, "full " + label)


def make_paged_case(rng, contexts, hq, hkv, d=128, page_tokens=16, spare=5, q8=False):
    sessions = len(contexts)
    need = [(c + page_tokens - 1) // page_tokens for c in contexts]
    pool_pages = sum(need) + spare
    perm = rng.permutation(pool_pages).astype(np.int32)
    stride = max(need) + 2
    table = np.full((sessions, stride), 0, dtype=np.int32)
    at = 0
    for s, n in enumerate(need):
        table[s, :n] = perm[at:at + n]
        at += n
    k_rows = bf16_normal(rng, (pool_pages, page_tokens, hkv, d))
    v_rows = bf16_normal(rng, (pool_pages, page_tokens, hkv, d))
    q = bf16_normal(rng, (sessions, hq, d))
    return q, k_rows, v_rows, table, np.array(contexts, dtype=np.int32), pool_pages


def run_paged(backend, q, k_rows, v_rows, table, ctx, hkv, pool_pages, storage=B.KV_BF16,
              max_context=None, page_tokens=16):
    sessions, hq, d = q.shape
    kp = kv_pack_pages(k_rows, storage, False, hkv, head_dim=d, page_tokens=page_tokens)
    vp = kv_pack_pages(v_rows, storage, True, hkv, head_dim=d, page_tokens=page_tokens)
    pool_dtype = B.DTYPE_BF16 if storage == B.KV_BF16 else B.DTYPE_I8
    elems = kp.size // B.DTYPE_BYTES[pool_dtype]
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tkp = backend.tensor("kpool", pool_dtype, (elems,), kp)
    tvp = backend.tensor("vpool", pool_dtype, (elems,), vp)
    tt = backend.tensor("table", B.DTYPE_I32, table.shape, table)
    tc = backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    lse = backend.tensor("lse", B.DTYPE_F32, (sessions, hq))
    req = backend.paged_requirement(sessions, hq, hkv, d, page_tokens, pool_pages, table.shape[1],
                                    max_context or int(table.shape[1] * page_tokens), storage=storage)
    facts = backend.paged_decode_execute(req, tq, tkp, tvp, tt, tc, out, lse)
    return out.read(), lse.read(), facts


def test_paged_decode_matches_oracle_ragged(backend):
    rng = np.random.default_rng(3)
    contexts = [1, 15, 16, 17, 100, 333, 1024, 1025, 2500]
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, 32, 8)
    got, lse, facts = run_paged(backend, q, k_rows, v_rows, table, ctx, 8, pool_pages)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, 8, 16)
    assert rc == 0
    assert_close_bf16(got, ref, "paged")
    assert_lse(lse, ref_lse, "paged")
    assert facts.kernel_launches in (1, 2) and facts.device_synchronizations == 1


def test_paged_decode_page_placement_is_bit_invariant(backend):
    """Moving every page to another pool slot and rewriting the table must not change a
    single output bit (index handling is exact)."""
    rng = np.random.default_rng(4)
    contexts = [40, 700, 129]
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, 8, 2)
    got, lse, _ = run_paged(backend, q, k_rows, v_rows, table, ctx, 2, pool_pages)
    perm = rng.permutation(pool_pages)
    k2, v2 = np.empty_like(k_rows), np.empty_like(v_rows)
    k2[perm], v2[perm] = k_rows, v_rows
    table2 = perm[table].astype(np.int32)
    got2, lse2, _ = run_paged(backend, q, k2, v2, table2, ctx, 2, pool_pages)
    assert np.array_equal(got, got2) and np.array_equal(lse, lse2)
    # garbage (NaN bit patterns) in rows past each context must not leak into the result
    k3, v3 = k_rows.copy(), v_rows.copy()
    for s, c in enumerate(contexts):
        last = table[s, (c - 1) // 16]
        k3[last, c % 16 or 16:] = 0x7FC0
        v3[last, c % 16 or 16:] = 0x7FC0
    got3, lse3, _ = run_paged(backend, q, k3, v3, table, ctx, 2, pool_pages)
    assert np.array_equal(got, got3) and np.array_equal(lse, lse3)


def test_paged_decode_refuses_bad_page_ids_and_lengths(backend):
    rng = np.random.default_rng(5)
    contexts = [50, 90]
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, 8, 2)
    bad = table.copy()
    bad[1, 3] = pool_pages
    with pytest.raises(YvexError) as e:
        run_paged(backend, q, k_rows, v_rows, bad, ctx, 2, pool_pages)
    assert e.value.code == B.YVEX_ERR_BOUNDS
    bad[1, 3] = -1
    with pytest.raises(YvexError) as e:
        run_paged(backend, q, k_rows, v_rows, bad, ctx, 2, pool_pages)
    assert e.value.code == B.YVEX_ERR_BOUNDS
    with pytest.raises(YvexError) as e:
        run_paged(backend, q, k_rows, v_rows, table, np.array([50, 0], np.int32), 2, pool_pages)
    assert e.value.code == B.YVEX_ERR_BOUNDS
    too_long = np.array([50, table.shape[1] * 16 + 1], np.int32)
    with pytest.raises(YvexError) as e:
        run_paged(backend, q, k_rows, v_rows, table, too_long, 2, pool_pages)
    assert e.value.code == B.YVEX_ERR_BOUNDS
    # the backend stays usable after a refusal and the next call is clean
    got, _, _ = run_paged(backend, q, k_rows, v_rows, table, ctx, 2, pool_pages)
    rc, ref, _, _ = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, 2, 16)
    assert_close_bf16(got, ref, "after refusal")


def test_config3_shape_sample(backend):
    """Benchmark configuration 3 at reduced session count (the oracle finishes in seconds): 32/8
    heads, d=128, contexts uniform in [512,16384], seeded permutation page tables."""
    rng = np.random.default_rng(3)
    contexts = [int(c) for c in rng.integers(512, 16385, size=6)]
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, 32, 8)
    got, lse, _ = run_paged(backend, q, k_rows, v_rows, table, ctx, 8, pool_pages,
                            max_context=16384 if table.shape[1] * 16 >= 16384 else None)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, 8, 16)
    assert rc == 0
    assert_close_bf16(got, ref, "config3")
    assert_lse(lse, ref_lse, "config3")


# ------------------------------------------------------------- Q8_0 paged KV ----

def make_q8_case(rng, contexts, hq, hkv, d=128, page_tokens=16):
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, hq, hkv, d, page_tokens)
    # quantise on the host with the product's own encoder (round-to-nearest absmax/127)
    from clori_amd.backend import q8_0_encode_rows
    k_blocks = q8_0_encode_rows(ORACLE.bf16_decode(k_rows))
    v_blocks = q8_0_encode_rows(ORACLE.bf16_decode(v_rows))
    return q, k_blocks, v_blocks, table, ctx, pool_pages


def test_q8_0_paged_decode_matches_cpu_on_same_bytes(backend):
    rng = np.random.default_rng(4)
    contexts = [1, 15, 16, 17, 100, 333, 1024, 1025, 4097]
    q, k_blocks, v_blocks, table, ctx, pool_pages = make_q8_case(rng, contexts, 32, 8)
    got, lse, facts = run_paged(backend, q, k_blocks, v_blocks, table, ctx, 8, pool_pages,
                                storage=B.KV_Q8_0)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_blocks, v_blocks, table, ctx, 8, 16, q8=True)
    assert rc == 0
    assert_close_bf16(got, ref, "q8_0 paged")
    assert_lse(lse, ref_lse, "q8_0 paged")
    assert facts.kernel_launches in (1, 2)


def test_q8_0_paged_placement_invariance_and_garbage_tail(backend):
    rng = np.random.default_rng(44)
    contexts = [40, 700, 129]
    q, k_blocks, v_blocks, table, ctx, pool_pages = make_q8_case(rng, contexts, 8, 2)
    got, lse, _ = run_paged(backend, q, k_blocks, v_blocks, table, ctx, 2, pool_pages,
                            storage=B.KV_Q8_0)
    perm = rng.permutation(pool_pages)
    k2, v2 = np.empty_like(k_blocks), np.empty_like(v_blocks)
    k2[perm], v2[perm] = k_blocks, v_blocks
    got2, lse2, _ = run_paged(backend, q, k2, v2, perm[table].astype(np.int32), ctx, 2,
                              pool_pages, storage=B.KV_Q8_0)
    assert np.array_equal(got, got2) and np.array_equal(lse, lse2)
    # rows past each context filled with 0xFF bytes (NaN scales, -1 codes) must not matter
    k3, v3 = k_blocks.copy(), v_blocks.copy()
    for s, c in enumerate(contexts):
        last = table[s, (c - 1) // 16]
        k3[last, c % 16 or 16:] = 0xFF
        v3[last, c % 16 or 16:] = 0xFF
    got3, lse3, _ = run_paged(backend, q, k3, v3, table, ctx, 2, pool_pages, storage=B.KV_Q8_0)
    assert np.array_equal(got, got3) and np.array_equal(lse, lse3)


def test_config4_shape_sample(backend):
    """Benchmark configuration 4 at reduced session count: contexts uniform in [4096,32768], K/V as
    GGUF Q8_0 blocks quantised on the host from N(0,1) bf16 values, seed 4."""
    rng = np.random.default_rng(4)
    contexts = [int(c) for c in rng.integers(4096, 32769, size=3)]
    q, k_blocks, v_blocks, table, ctx, pool_pages = make_q8_case(rng, contexts, 32, 8)
    got, lse, _ = run_paged(backend, q, k_blocks, v_blocks, table, ctx, 8, pool_pages,
                            storage=B.KV_Q8_0)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_blocks, v_blocks, table, ctx, 8, 16, q8=True)
    assert rc == 0
    assert_close_bf16(got, ref, "config4")
    assert_lse(lse, ref_lse, "config4")


# ------------------------------------------------------------ long contexts ----

@pytest.mark.parametrize("contexts,q8", [([150000], False), ([90000, 3, 40000], False),
                                          ([120000], True)])
def test_paged_decode_long_contexts(backend, contexts, q8):
    """Contexts far beyond the benchmark's: one (session, kv head) segment is split over
    hundreds of waves, so the second kernel merges its partials over many load trips, and a
    three-token session sits between two long ones."""
    rng = np.random.default_rng(len(contexts) * 1000 + int(q8))
    make = make_q8_case if q8 else make_paged_case
    q, k_rows, v_rows, table, ctx, pool_pages = make(rng, contexts, 32, 8)
    storage = B.KV_Q8_0 if q8 else B.KV_BF16
    got, lse, facts = run_paged(backend, q, k_rows, v_rows, table, ctx, 8, pool_pages, storage=storage)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, 8, 16, q8=q8)
    assert rc == 0
    assert_close_bf16(got, ref, "long paged %s" % contexts)
    assert_lse(lse, ref_lse, "long paged %s" % contexts)
    assert facts.kernel_launches == 2
    again, lse_again, _ = run_paged(backend, q, k_rows, v_rows, table, ctx, 8, pool_pages, storage=storage)
    assert np.array_equal(got, again) and np.array_equal(lse, lse_again)


def test_rows_decode_long_context(backend):
    rng = np.random.default_rng(150)
    ctx = 150000
    q = bf16_normal(rng, (1, 32, 128))
    k = bf16_normal(rng, (ctx, 8, 128))
    v = bf16_normal(rng, (ctx, 8, 128))
    got, lse, facts = run_rows_decode(backend, q, k, v, query_start=ctx - 1)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, "long rows")
    assert_lse(lse, ref_lse, "long rows")
    assert facts.kernel_launches == 1


@pytest.mark.parametrize("q8", [False, True], ids=["bf16", "q8_0"])
def test_paged_decode_many_short_sessions(backend, q8):
    """Three thousand sessions of 1 to 100 tokens: more (session, kv head) segments than waves,
    several whole segments per wave."""
    rng = np.random.default_rng(3000 + int(q8))
    contexts = [int(c) for c in rng.integers(1, 101, size=3000)]
    make = make_q8_case if q8 else make_paged_case
    q, k_rows, v_rows, table, ctx, pool_pages = make(rng, contexts, 8, 2)
    got, lse, _ = run_paged(backend, q, k_rows, v_rows, table, ctx, 2, pool_pages,
                            storage=B.KV_Q8_0 if q8 else B.KV_BF16)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, 2, 16, q8=q8)
    assert rc == 0
    assert_close_bf16(got, ref, "many sessions")
    assert_lse(lse, ref_lse, "many sessions")


# ------------------------------------------------------- pages of 64 tokens ----

@pytest.mark.parametrize("q8", [False, True], ids=["bf16", "q8_0"])
def test_paged_decode_with_pages_of_64_tokens(backend, q8):
    """Pages of 64 tokens (four 16-token blocks each): ragged contexts around block and page
    edges against the oracle on 64-token pages, and bit for bit against the same rows cut
    into 16-token pages."""
    rng = np.random.default_rng(64 + int(q8))
    contexts = [1, 15, 16, 17, 63, 64, 65, 127, 129, 1000, 4097, 20000]
    make = make_q8_case if q8 else make_paged_case
    storage = B.KV_Q8_0 if q8 else B.KV_BF16
    q, k_rows, v_rows, table, ctx, pool_pages = make(rng, contexts, 32, 8, page_tokens=64)
    got, lse, facts = run_paged(backend, q, k_rows, v_rows, table, ctx, 8, pool_pages,
                                storage=storage, page_tokens=64)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, 8, 64, q8=q8)
    assert rc == 0
    assert_close_bf16(got, ref, "64-token pages")
    assert_lse(lse, ref_lse, "64-token pages")
    # the same rows as pages of 16: page p of 64 becomes pages 4p .. 4p+3
    narrow_rows = [rows.reshape((pool_pages * 4, 16) + rows.shape[2:]) for rows in (k_rows, v_rows)]
    narrow_table = (table[:, :, None] * 4 + np.arange(4, dtype=np.int32)).reshape(len(contexts), -1)
    got16, lse16, _ = run_paged(backend, q, narrow_rows[0], narrow_rows[1],
                                np.ascontiguousarray(narrow_table, np.int32), ctx, 8, pool_pages * 4,
                                storage=storage)
    assert np.array_equal(got, got16) and np.array_equal(lse, lse16)
    # a page id out of range is still caught
    bad = table.copy()
    bad[11, 5] = pool_pages
    with pytest.raises(YvexError) as e:
        run_paged(backend, q, k_rows, v_rows, bad, ctx, 8, pool_pages, storage=storage, page_tokens=64)
    assert e.value.code == B.YVEX_ERR_BOUNDS


@pytest.mark.parametrize("d,hq,hkv", [(64, 16, 4), (256, 24, 4), (256, 8, 8)])
@pytest.mark.parametrize("page_tokens", [16, 64])
def test_paged_decode_other_head_dimensions(backend, d, hq, hkv, page_tokens):
    """bf16 pages at head dimension 64 and 256 (the reference admits up to 256 and its own
    Qwen pattern is 24/4/256, tests/unit/cuda/quant_qtype.c:2413-2418): ragged contexts around
    block and page edges against the oracle, placement invariance bit for bit, garbage past the
    context; these head dimensions always take the second launch."""
    rng = np.random.default_rng(1000 + d + page_tokens)
    contexts = [1, 15, 16, 17, 63, 64, 65, 333, 1024, 1025, 2500, 9000]
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, hq, hkv, d=d,
                                                                 page_tokens=page_tokens)
    got, lse, facts = run_paged(backend, q, k_rows, v_rows, table, ctx, hkv, pool_pages,
                                page_tokens=page_tokens)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, hkv, page_tokens)
    assert rc == 0
    assert_close_bf16(got, ref, "paged d=%d" % d)
    assert_lse(lse, ref_lse, "paged d=%d" % d)
    assert facts.kernel_launches == 2
    perm = rng.permutation(pool_pages)
    k2, v2 = np.empty_like(k_rows), np.empty_like(v_rows)
    k2[perm], v2[perm] = k_rows, v_rows
    for s, c in enumerate(contexts):  # rows past each context: NaN bit patterns
        last = perm[table[s, (c - 1) // page_tokens]]
        k2[last, c % page_tokens or page_tokens:] = 0x7FC0
        v2[last, c % page_tokens or page_tokens:] = 0x7FC0
    got2, lse2, _ = run_paged(backend, q, k2, v2, perm[table].astype(np.int32), ctx, hkv, pool_pages,
                              page_tokens=page_tokens)
    assert np.array_equal(got, got2) and np.array_equal(lse, lse2)


def test_paged_decode_other_head_dimensions_refusals(backend):
    """Q8_0 pages exist at head dimension 128 only; 96 has no kernel at all."""
    for d, storage in ((64, B.KV_Q8_0), (256, B.KV_Q8_0), (96, B.KV_BF16)):
        req = backend.paged_requirement(1, 8, 2, d, 16, 4, 4, 64, storage=storage)
        with pytest.raises(YvexError) as e:
            backend.paged_decode_workspace_required(req)
        assert e.value.code == B.YVEX_ERR_UNSUPPORTED
