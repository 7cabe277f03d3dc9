"""GPU parity: absorbed-latent MLA decode against the shared-KV CPU restatement
(src/graph/core.c:361-508 semantics), through the C ABI."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu

HEADS, KEY_DIM, VALUE_DIM, PAGE = 128, 576, 512, 64


def make_case(rng, contexts, spare=2, heads=HEADS, key_dim=KEY_DIM):
    batch = len(contexts)
    need = [(c + PAGE - 1) // PAGE for c in contexts]
    pool_pages = sum(need) + spare
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((batch, max(need) + 1), dtype=np.int32)
    at = 0
    for b, n in enumerate(need):
        table[b, :n] = perm[at:at + n]
        at += n
    pool = bf16_normal(rng, (pool_pages, PAGE, key_dim))
    q = bf16_normal(rng, (batch, heads, key_dim))
    return q, pool, table, np.array(contexts, dtype=np.int32)


def run_mla(backend, q, pool, table, ctx, max_context=None, sinks=None, window=0, compressed=None,
            selected=None, rope=None, positions=None, scale=0.0):
    batch, heads, key_dim = q.shape
    extra = {}
    if compressed is not None:
        extra = dict(compressed_pool_pages=compressed[0].shape[0],
                     compressed_table_stride=compressed[1].shape[1],
                     max_compressed_tokens=int(compressed[1].shape[1] * PAGE),
                     compressed_selected_stride=selected.shape[1] if selected is not None else 0)
    req = backend.mla_requirement(batch, heads, key_dim, VALUE_DIM, PAGE, pool.shape[0],
                                  table.shape[1], max_context or int(table.shape[1] * PAGE),
                                  sliding_window=window, output_inverse_rope=rope, scale=scale,
                                  **extra)
    out = backend.tensor("o", B.DTYPE_BF16, (batch, heads, VALUE_DIM))
    lse = backend.tensor("lse", B.DTYPE_F32, (batch, heads))
    tensors = [backend.tensor("q", B.DTYPE_BF16, q.shape, q),
               backend.tensor("pool", B.DTYPE_BF16, pool.shape, pool),
               backend.tensor("table", B.DTYPE_I32, table.shape, table),
               backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)]
    ts = backend.tensor("sinks", B.DTYPE_F32, (heads,), sinks) if sinks is not None else None
    tc = None
    if compressed is not None:
        tc = [backend.tensor("cpool", B.DTYPE_BF16, compressed[0].shape, compressed[0]),
              backend.tensor("ctable", B.DTYPE_I32, compressed[1].shape, compressed[1]),
              backend.tensor("ccount", B.DTYPE_I32, compressed[2].shape, compressed[2])]
        if selected is not None:
            tc.append(backend.tensor("selected", B.DTYPE_I32, selected.shape, selected))
    tp = backend.tensor("positions", B.DTYPE_I64, (batch,), np.asarray(positions, np.int64)) \
        if positions is not None else None
    facts = backend.mla_decode_execute(req, *tensors, out, lse, sinks=ts, compressed=tc,
                                       output_positions=tp)
    result = out.read(), lse.read(), facts
    for t in tensors + [out, lse] + ([ts] if ts else []) + (tc or []) + ([tp] if tp else []):
        t.release()
    return result


def test_mla_decode_matches_shared_kv_oracle_ragged(backend):
    rng = np.random.default_rng(5)
    contexts = [1, 31, 32, 33, 64, 65, 500, 1300]
    q, pool, table, ctx = make_case(rng, contexts)
    got, lse, facts = run_mla(backend, q, pool, table, ctx)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE)
    assert rc == 0
    assert_close_bf16(got, ref, "mla ragged")
    assert_lse(lse, ref_lse, "mla ragged")
    assert facts.kernel_launches == 2 and facts.device_synchronizations == 1


def test_config5_shape_sample(backend):
    """Benchmark configuration 5 at reduced batch: 128 heads, 512+64 latent, context 8192 in 64-token
    pages, scale 1/sqrt(576), seed 5."""
    rng = np.random.default_rng(5)
    q, pool, table, ctx = make_case(rng, [8192, 8192])
    got, lse, _ = run_mla(backend, q, pool, table, ctx, max_context=8192)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE)
    assert rc == 0
    assert_close_bf16(got, ref, "config5")
    assert_lse(lse, ref_lse, "config5")


def test_mla_page_placement_invariance_and_refusals(backend):
    rng = np.random.default_rng(55)
    q, pool, table, ctx = make_case(rng, [200, 77])
    got, lse, _ = run_mla(backend, q, pool, table, ctx)
    perm = rng.permutation(pool.shape[0])
    pool2 = np.empty_like(pool)
    pool2[perm] = pool
    got2, lse2, _ = run_mla(backend, q, pool2, perm[table].astype(np.int32), ctx)
    assert np.array_equal(got, got2) and np.array_equal(lse, lse2)
    bad = table.copy()
    bad[0, 1] = pool.shape[0]
    with pytest.raises(YvexError) as e:
        run_mla(backend, q, pool, bad, ctx)
    assert e.value.code == B.YVEX_ERR_BOUNDS
    with pytest.raises(YvexError) as e:
        run_mla(backend, q, pool, table, np.array([200, 0], np.int32))
    assert e.value.code == B.YVEX_ERR_BOUNDS
    req = backend.mla_requirement(2, 64, KEY_DIM, VALUE_DIM, PAGE, 8, 4, 256)
    with pytest.raises(YvexError) as e:
        backend.mla_decode_workspace_required(req)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED


@pytest.mark.parametrize("window", [0, 1, 31, 32, 33, 100, 1024, 100000])
def test_mla_sink_logits_and_sliding_window(backend, window):
    """Per-head sink logits in the softmax denominator and the sliding-window position filter
    (src/backend/cuda/attention_kernels.cu:79-84,164-166), ragged contexts around the 32-token
    tile and 64-token page edges."""
    rng = np.random.default_rng(500 + window)
    contexts = [1, 31, 32, 33, 63, 64, 65, 100, 129, 500, 1300, 4097]
    q, pool, table, ctx = make_case(rng, contexts)
    sinks = (rng.standard_normal(HEADS) * 3.0).astype(np.float32)
    got, lse, facts = run_mla(backend, q, pool, table, ctx, sinks=sinks, window=window)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE, sinks=sinks,
                                            sliding_window=window)
    assert rc == 0
    assert_close_bf16(got, ref, "mla sink window=%d" % window)
    assert_lse(lse, ref_lse, "mla sink window=%d" % window)
    assert facts.kernel_launches == 2
    # without sinks the window alone
    got, lse, _ = run_mla(backend, q, pool, table, ctx, window=window)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE,
                                            sliding_window=window)
    assert rc == 0
    assert_close_bf16(got, ref, "mla window=%d" % window)
    assert_lse(lse, ref_lse, "mla window=%d" % window)


def test_mla_window_at_config5_context(backend):
    """Context 8192 with a 4096-token window: only the last 4096 positions count, and the
    workspace shrinks with the window."""
    rng = np.random.default_rng(58)
    q, pool, table, ctx = make_case(rng, [8192, 8000, 4096, 5000])
    full = backend.mla_requirement(4, HEADS, KEY_DIM, VALUE_DIM, PAGE, pool.shape[0], table.shape[1], 8192)
    windowed = backend.mla_requirement(4, HEADS, KEY_DIM, VALUE_DIM, PAGE, pool.shape[0], table.shape[1],
                                       8192, sliding_window=4096)
    assert backend.mla_decode_workspace_required(windowed) < backend.mla_decode_workspace_required(full)
    got, lse, _ = run_mla(backend, q, pool, table, ctx, max_context=8192, window=4096)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE, sliding_window=4096)
    assert rc == 0
    assert_close_bf16(got, ref, "mla window 4096")
    assert_lse(lse, ref_lse, "mla window 4096")


def test_mla_non_finite_sink_is_a_numeric_failure(backend):
    rng = np.random.default_rng(59)
    q, pool, table, ctx = make_case(rng, [70])
    sinks = np.zeros(HEADS, np.float32)
    sinks[17] = np.inf
    with pytest.raises(YvexError) as e:
        run_mla(backend, q, pool, table, ctx, sinks=sinks)
    assert e.value.code == B.YVEX_ERR_FORMAT


@pytest.mark.parametrize("window", [0, 128])
def test_mla_compressed_candidate_rows(backend, window):
    """A second paged row set (compressed rows, src/graph/core.c:437-468) in the same softmax:
    counts of 0, below one tile, across pages and chunks; with sinks and a local window."""
    rng = np.random.default_rng(600 + window)
    contexts = [1, 70, 128, 129, 1000, 4097, 8192, 300]
    counts = [0, 1, 31, 64, 65, 32, 64, 700]
    q, pool, table, ctx = make_case(rng, contexts)
    _, cpool, ctable, _ = make_case(rng, [max(c, 1) for c in counts])
    ccount = np.array(counts, np.int32)
    sinks = (rng.standard_normal(HEADS) * 2.0).astype(np.float32)
    got, lse, facts = run_mla(backend, q, pool, table, ctx, sinks=sinks, window=window,
                              compressed=(cpool, ctable, ccount))
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE, sinks=sinks,
                                            sliding_window=window, compressed=(cpool, ctable, ccount))
    assert rc == 0
    assert_close_bf16(got, ref, "mla compressed window=%d" % window)
    assert_lse(lse, ref_lse, "mla compressed window=%d" % window)
    assert facts.kernel_launches == 3 and facts.accelerated_matrix_launches == 2


def test_mla_selected_compressed_rows(backend):
    """The selected class (src/graph/core.c:443-452): per-session index lists into the compressed
    sequence, gathered in list order (repeats allowed), list lengths from 0 to the capacity."""
    rng = np.random.default_rng(700)
    contexts = [1, 70, 129, 1000, 4097, 300]
    stored = [64, 10, 200, 700, 2048, 65]
    capacity = 512
    counts = np.array([0, 1, 31, 512, 300, 65], np.int32)
    q, pool, table, ctx = make_case(rng, contexts)
    _, cpool, ctable, _ = make_case(rng, stored)
    lists = np.stack([rng.integers(0, stored[i], capacity) for i in range(len(stored))]).astype(np.int32)
    sinks = (rng.standard_normal(HEADS) * 2.0).astype(np.float32)
    got, lse, facts = run_mla(backend, q, pool, table, ctx, sinks=sinks, window=128,
                              compressed=(cpool, ctable, counts), selected=lists)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE, sinks=sinks,
                                            sliding_window=128, compressed=(cpool, ctable, counts),
                                            selected=lists)
    assert rc == 0
    assert_close_bf16(got, ref, "mla selected")
    assert_lse(lse, ref_lse, "mla selected")
    assert facts.kernel_launches == 4
    bad = lists.copy()
    bad[3, 100] = int(ctable.shape[1] * PAGE)          # one past what the table can address
    with pytest.raises(YvexError) as e:
        run_mla(backend, q, pool, table, ctx, compressed=(cpool, ctable, counts), selected=bad)
    assert e.value.code == B.YVEX_ERR_BOUNDS


ROPE_POLICIES = [
    dict(rope_dimensions=64, theta=10000),
    dict(rope_dimensions=64, theta=10000, scaling_factor=40, original_context=4096, beta_fast=32,
         beta_slow=1),
    dict(rope_dimensions=128, theta=500000, scaling_factor=8, original_context=8192, beta_fast=32,
         beta_slow=1),
    dict(rope_dimensions=8, theta=10000),
]


def oracle_policy(rope):
    return ORACLE.position_policy(rope["rope_dimensions"], **{k: v for k, v in rope.items()
                                                             if k != "rope_dimensions"})


@pytest.mark.parametrize("rope", ROPE_POLICIES, ids=["plain64", "yarn64", "yarn128", "plain8"])
def test_mla_output_inverse_rotation(backend, rope):
    """The rotation the shared-KV reduce applies to its published rows (src/graph/core.c:499-507:
    bf16 round, the last rope lanes turned back by the token position with the frequencies of
    src/graph/numeric.c:877-917, bf16 round).  Checked twice: against the oracle end to end
    within the bf16 tolerance of the attention itself, and bit for bit against the oracle's
    rotation applied to the rows the same kernels publish without it."""
    rng = np.random.default_rng(600 + rope["rope_dimensions"])
    contexts = [1, 33, 64, 500, 1300, 4097]
    q, pool, table, ctx = make_case(rng, contexts)
    sinks = (rng.standard_normal(HEADS) * 3.0).astype(np.float32)
    plain, lse0, _ = run_mla(backend, q, pool, table, ctx, sinks=sinks)
    got, lse, facts = run_mla(backend, q, pool, table, ctx, sinks=sinks, rope=rope)
    assert facts.kernel_launches == 2 and np.array_equal(lse, lse0)
    rc, ref, _, _ = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE, sinks=sinks)
    assert rc == 0
    policy = oracle_policy(rope)
    keep = VALUE_DIM - rope["rope_dimensions"]
    for b, n in enumerate(contexts):
        rc, want = ORACLE.reduce_output_finish(ref[b], n - 1, policy)
        assert rc == 0
        assert_close_bf16(got[b:b + 1], want[None], "mla rotation b=%d" % b)
        rc, exact = ORACLE.reduce_output_finish(ORACLE.bf16_decode(plain[b]), n - 1, policy)
        assert rc == 0
        assert np.array_equal(got[b], ORACLE.bf16_encode(exact)), (rope, n)
        assert np.array_equal(got[b][:, :keep], plain[b][:, :keep])
        if n > 1:
            assert not np.array_equal(got[b][:, keep:], plain[b][:, keep:])
    # explicit positions: long-context angles on the same rows
    where = [20000 + 7 * b for b in range(len(contexts))]
    got, _, _ = run_mla(backend, q, pool, table, ctx, sinks=sinks, rope=rope, positions=where)
    for b in range(len(contexts)):
        rc, exact = ORACLE.reduce_output_finish(ORACLE.bf16_decode(plain[b]), where[b], policy)
        assert rc == 0
        assert np.array_equal(got[b], ORACLE.bf16_encode(exact)), (rope, where[b])


def test_mla_rotation_and_scale_refusals_and_explicit_scale(backend):
    rng = np.random.default_rng(601)
    q, pool, table, ctx = make_case(rng, [200, 77])
    for bad, code in ((dict(rope_dimensions=64, theta=1), B.YVEX_ERR_INVALID_ARG),
                      (dict(rope_dimensions=64, theta=10000, original_context=4096, scaling_factor=40,
                            beta_fast=1, beta_slow=1), B.YVEX_ERR_INVALID_ARG),
                      (dict(rope_dimensions=64, theta=10000, original_context=4096), B.YVEX_ERR_INVALID_ARG),
                      (dict(rope_dimensions=12, theta=10000), B.YVEX_ERR_UNSUPPORTED),
                      (dict(rope_dimensions=256, theta=10000), B.YVEX_ERR_UNSUPPORTED)):
        with pytest.raises(YvexError) as e:
            run_mla(backend, q, pool, table, ctx, rope=bad)
        assert e.value.code == code, bad
    with pytest.raises(YvexError) as e:                 # positions without a rotation to use them
        run_mla(backend, q, pool, table, ctx, positions=[1, 2])
    assert e.value.code == B.YVEX_ERR_FORMAT
    with pytest.raises(YvexError) as e:
        run_mla(backend, q, pool, table, ctx, scale=float("nan"))
    assert e.value.code == B.YVEX_ERR_INVALID_ARG
    # an explicit scale: twice the default on a query halved (exact in bf16) gives the same scores
    base, lse0, _ = run_mla(backend, q, pool, table, ctx)
    half = ORACLE.bf16_encode(ORACLE.bf16_decode(q) * 0.5)
    got, lse, _ = run_mla(backend, half, pool, table, ctx, scale=2.0 / np.sqrt(KEY_DIM))
    assert np.array_equal(got, base)
    assert np.allclose(lse, lse0, rtol=0, atol=2e-6)


# ------------------------------------- the reference's own reduce geometry (64 heads, 512) ----

R_HEADS, R_DIM = 64, 512
YARN = dict(rope_dimensions=64, theta=10000, scaling_factor=40, original_context=4096, beta_fast=32,
            beta_slow=1)


@pytest.mark.parametrize("window", [0, 128])
def test_reduce_geometry_matches_shared_kv_oracle(backend, window):
    """64 heads over one 512-lane row per token, key and value the same row with the rope lanes
    inside (tests/unit/deepseek_arch_ir.c:110-125), sink logits, the model's 128-token window,
    dense compressed rows and the output rotation: the whole reduce of src/graph/core.c:471-508."""
    rng = np.random.default_rng(700 + window)
    contexts = [1, 31, 33, 64, 65, 129, 500, 1300, 4097]
    q, pool, table, ctx = make_case(rng, contexts, heads=R_HEADS, key_dim=R_DIM)
    ratio = 128
    stored = [n // ratio + 1 for n in contexts]
    _, cpool, ctable, _ = make_case(rng, stored, heads=R_HEADS, key_dim=R_DIM)
    visible = np.array([n // ratio for n in contexts], np.int32)
    sinks = (rng.standard_normal(R_HEADS) * 3.0).astype(np.float32)
    got, lse, facts = run_mla(backend, q, pool, table, ctx, sinks=sinks, window=window,
                              compressed=(cpool, ctable, visible), rope=YARN)
    assert facts.kernel_launches == 3
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, R_DIM, PAGE, sinks=sinks,
                                            sliding_window=window, compressed=(cpool, ctable, visible))
    assert rc == 0
    policy = oracle_policy(YARN)
    for b, n in enumerate(contexts):
        rc, want = ORACLE.reduce_output_finish(ref[b], n - 1, policy)
        assert rc == 0
        assert_close_bf16(got[b:b + 1], want[None], "reduce geometry b=%d window=%d" % (b, window))
    assert_lse(lse, ref_lse, "reduce geometry window=%d" % window)
    # the plain decode of the same geometry, and placement invariance
    plain, lse0, facts = run_mla(backend, q, pool, table, ctx)
    assert facts.kernel_launches == 2
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, R_DIM, PAGE)
    assert_close_bf16(plain, ref, "reduce geometry plain")
    assert_lse(lse0, ref_lse, "reduce geometry plain")
    perm = rng.permutation(pool.shape[0])
    pool2 = np.empty_like(pool)
    pool2[perm] = pool
    again, lse2, _ = run_mla(backend, q, pool2, perm[table].astype(np.int32), ctx)
    assert np.array_equal(plain, again) and np.array_equal(lse0, lse2)


def test_reduce_geometry_against_the_reference_reduce(backend):
    """The device result at the reference's geometry against the reference's own
    yvex_attention_reduce_chunk: the compiled one where it was built, and its committed output
    (tests/golden, case reduce-model-geometry) everywhere."""
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(here, "golden", "make_golden.py"))
    golden_inputs = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(golden_inputs)
    golden = np.load(os.path.join(here, "golden", "reference_attention.npz"), allow_pickle=False)
    name, attention_class, window, context, stored, heads, dim, policy = golden_inputs.MODEL_GEOMETRY_CASE
    assert (heads, dim) == (R_HEADS, R_DIM)
    qf, local, compressed, sinks = golden_inputs.reduce_inputs(heads, dim, context, stored)

    def paged(rows):
        pages = max((len(rows) + PAGE - 1) // PAGE, 1)
        pool = np.zeros((pages, PAGE, dim), np.uint16)
        pool.reshape(-1, dim)[:len(rows)] = ORACLE.bf16_encode(rows)
        return pool, np.arange(pages, dtype=np.int32)[None, :]

    pool, table = paged(local)
    cpool, ctable = paged(compressed)
    visible = np.array([context // golden_inputs.REDUCE_RATIO], np.int32)
    rope = dict(rope_dimensions=policy["rope_dims"], **{k: v for k, v in policy.items() if k != "rope_dims"})
    got, _, _ = run_mla(backend, ORACLE.bf16_encode(qf)[None], pool, table, np.array([context], np.int32),
                        sinks=sinks, window=window, compressed=(cpool, ctable, visible), rope=rope)
    want = golden[name + "/out"]
    assert_close_bf16(got, want[None], "reference reduce, committed output")


def test_mla_decode_long_context(backend):
    """A context twelve times the benchmark's next to a seven-token one: hundreds of chunks
    for one batch element in the merge, one for the other."""
    rng = np.random.default_rng(55)
    q, pool, table, ctx = make_case(rng, [100000, 7])
    got, lse, _ = run_mla(backend, q, pool, table, ctx)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE)
    assert rc == 0
    assert_close_bf16(got, ref, "mla long")
    assert_lse(lse, ref_lse, "mla long")


def test_mla_decode_many_short_contexts(backend):
    rng = np.random.default_rng(56)
    contexts = [int(c) for c in rng.integers(1, 200, size=150)]
    q, pool, table, ctx = make_case(rng, contexts)
    got, lse, _ = run_mla(backend, q, pool, table, ctx)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, VALUE_DIM, PAGE)
    assert rc == 0
    assert_close_bf16(got, ref, "mla many")
    assert_lse(lse, ref_lse, "mla many")
