"""GPU parity for the exact F32 contract: the reference's own test vectors and refusal
behaviour (tests/unit/backend_ops.c:444-532, tests/unit/cuda/ops.c:567-623,
tests/unit/cuda/quant_qtype.c:2100-2970), run through the C ABI."""
import math

import numpy as np
import pytest

import reference_vectors as rv
from clori_amd import binding as B
from clori_amd.backend import YvexError
from gpu_common import ORACLE, backend  # noqa: F401

pytestmark = pytest.mark.gpu


def f32(backend, name, array=None, shape=None):
    if array is not None:
        array = np.ascontiguousarray(array, dtype=np.float32)
        return backend.tensor(name, B.DTYPE_F32, array.shape, array)
    return backend.tensor(name, B.DTYPE_F32, shape)


def test_bounded_primitive_reference_literals(backend):
    q = f32(backend, "attention_query", rv.CPU_OP_QUERY)
    k = f32(backend, "attention_keys", rv.CPU_OP_KEYS)
    v = f32(backend, "attention_values", rv.CPU_OP_VALUES)
    s = f32(backend, "attention_scores", shape=(3,))
    p = f32(backend, "attention_probabilities", shape=(3,))
    o = f32(backend, "attention_out", shape=(4,))
    assert not o.is_written
    backend.op_attention(q, k, v, 3, 0, 0.5, True, s, p, o)
    assert np.allclose(o.read(), rv.CPU_OP_VALUES[0], atol=1e-6) and o.is_written
    backend.op_attention(q, k, v, 3, 2, 0.5, True, s, p, o)
    rc, ref, ref_s, ref_p, _ = ORACLE.attention_head(rv.CPU_OP_QUERY, rv.CPU_OP_KEYS,
                                                     rv.CPU_OP_VALUES, 2, 0.5)
    assert np.allclose(o.read(), ref, atol=1e-6)
    assert np.allclose(s.read(), ref_s, atol=1e-7) and np.allclose(p.read(), ref_p, atol=1e-7)
    backend.op_attention(q, k, v, 3, 0, 0.5, False, s, p, o)      # non-causal sees all rows
    assert np.allclose(o.read(), ref, atol=1e-6)
    with pytest.raises(YvexError) as e:
        backend.op_attention(q, k, v, 3, 3, 0.5, True, s, p, o)
    assert e.value.code == B.YVEX_ERR_BOUNDS and "position-out-of-range" in e.value.message
    with pytest.raises(YvexError) as e:
        backend.op_attention(q, k, v, 0, 0, 0.5, True, s, p, o)
    assert e.value.code == B.YVEX_ERR_INVALID_ARG
    for scale in (float("nan"), 0.0, -1.0, float("inf")):
        with pytest.raises(YvexError) as e:
            backend.op_attention(q, k, v, 3, 0, scale, True, s, p, o)
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
    wrong = f32(backend, "wrong", shape=(5,))
    with pytest.raises(YvexError) as e:
        backend.op_attention(q, k, v, 3, 0, 0.5, True, s, p, wrong)
    assert e.value.code == B.YVEX_ERR_FORMAT
    half = backend.tensor("half", B.DTYPE_BF16, (4,))
    with pytest.raises(YvexError) as e:
        backend.op_attention(q, k, v, 3, 0, 0.5, True, s, p, half)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED


def test_bounded_primitive_long_row_matches_cpu_operator(backend):
    rng = np.random.default_rng(12)
    n, d = 4096, 128
    qv = rng.standard_normal(d).astype(np.float32)
    kv = rng.standard_normal((n, d)).astype(np.float32)
    vv = rng.standard_normal((n, d)).astype(np.float32)
    q, k, v = f32(backend, "q", qv), f32(backend, "k", kv), f32(backend, "v", vv)
    s, p, o = f32(backend, "s", shape=(n,)), f32(backend, "p", shape=(n,)), f32(backend, "o", shape=(d,))
    scale = 1.0 / math.sqrt(d)
    backend.op_attention(q, k, v, n, n - 1, scale, True, s, p, o)
    rc, ref, ref_s, ref_p, _ = ORACLE.attention_head(qv, kv, vv, n - 1, scale)
    assert np.allclose(o.read(), ref, atol=1e-6)
    assert np.allclose(s.read(), ref_s, atol=1e-6) and abs(p.read().sum() - 1.0) < 1e-5


def execute(backend, q, k, v, query_start=0, causal=True, **kw):
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    req = backend.attention_requirement(tq, tk, hq, hkv, d, causal=causal, query_start=query_start,
                                        **kw)
    out = f32(backend, "out", shape=(tq, hq, d))
    facts = backend.attention_execute(req, f32(backend, "q", q), f32(backend, "k", k),
                                      f32(backend, "v", v), out)
    return out.read(), facts


def test_gqa_known_answer(backend):
    q, k, v, mixed = rv.gqa_kat()
    out, facts = execute(backend, q, k, v, causal=True)
    assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
    assert np.array_equal(out[0], np.array([[2.0, 4.0], [2.0, 4.0]], np.float32))
    assert np.allclose(out[1], mixed, atol=1e-6)
    out, _ = execute(backend, q, k, v, causal=False)
    assert np.allclose(out, np.broadcast_to(mixed, (2, 2, 2)), atol=1e-6)
    req = backend.attention_requirement(2, 2, 2, 1, 2)
    assert backend.attention_workspace_required(req) == 0


@pytest.mark.parametrize("maker,tol_abs,tol_rel", [
    (rv.small_5x128, 2e-5, 0.0), (rv.qwen_24_4_256, 2e-4, 2e-4), (rv.tiled_257x128, 0.0, 2e-3)])
def test_gqa_reference_patterns(backend, maker, tol_abs, tol_rel):
    q, k, v = maker()
    for causal in (True, False):
        out, _ = execute(backend, q, k, v, causal=causal)
        rc, ref, _ = ORACLE.gqa(q, k, v, causal=causal)
        assert rc == 0
        assert np.all(np.abs(out - ref) <= tol_abs + tol_rel * (1.0 + np.abs(ref)) + 1e-7)
        # and far tighter against the CPU operator: double statistics on the row kernel, float
        # ones (as in the reference's device kernel) on the matrix-core kernel
        assert np.abs(out - ref).max() < (2e-5 if q.shape[0] >= 32 else 2e-6)
        again, _ = execute(backend, q, k, v, causal=causal)
        assert np.array_equal(out, again)               # deterministic: byte-identical repeat


def test_gqa_cached_decode_strided_and_refusals(backend):
    q, k, v = rv.cached_decode_qwen()
    out, _ = execute(backend, q, k, v, query_start=2)
    rc, ref, _ = ORACLE.gqa(q, k, v, query_start=2)
    assert np.abs(out - ref).max() < 2e-6
    with pytest.raises(YvexError) as e:
        execute(backend, q, k, v, query_start=3)                    # query range beyond KV
    assert e.value.code == B.YVEX_ERR_INVALID_ARG
    # strided [Q|gate] and [K|V] views
    q, k, v = rv.strided_qwen()
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    qi = np.full((tq, 2 * hq * d), 55.0, np.float32)
    qi[:, :hq * d] = q.reshape(tq, -1)
    kvi = np.zeros((tk, 2 * hkv * d), np.float32)
    kvi[:, :hkv * d] = k.reshape(tk, -1)
    kvi[:, hkv * d:] = v.reshape(tk, -1)
    qs = f32(backend, "q-storage", qi)
    kvs = f32(backend, "kv-storage", kvi)
    q_view = qs.view(0, B.DTYPE_F32, ((tq - 1) * 2 * hq * d + hq * d,))
    k_view = kvs.view(0, B.DTYPE_F32, ((tk - 1) * 2 * hkv * d + hkv * d,))
    v_view = kvs.view(hkv * d * 4, B.DTYPE_F32, ((tk - 1) * 2 * hkv * d + hkv * d,))
    out_t = f32(backend, "out", shape=(tq, hq, d))
    req = backend.attention_requirement(tq, tk, hq, hkv, d, query_start=2, q_stride=2 * hq * d,
                                        k_stride=2 * hkv * d, v_stride=2 * hkv * d)
    backend.attention_execute(req, q_view, k_view, v_view, out_t)
    packed, _ = execute(backend, q, k, v, query_start=2)
    assert np.array_equal(out_t.read(), packed)                     # strided == packed, bit for bit
    req.query_token_stride = hq * d - 1
    with pytest.raises(YvexError) as e:
        backend.attention_execute(req, q_view, k_view, v_view, out_t)
    assert e.value.code == B.YVEX_ERR_INVALID_ARG                   # stride below the row width


def test_gqa_admission_is_fail_closed(backend):
    q, k, v = rv.small_5x128()
    # head dimension beyond the admitted bound
    req = backend.attention_requirement(3, 3, 24, 4, 257)
    with pytest.raises(YvexError) as e:
        backend.attention_workspace_required(req)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    # a bf16 output under the exact contract is a silent precision change: refused
    req = backend.attention_requirement(5, 5, 1, 1, 128)
    req.output_dtype = B.DTYPE_BF16
    with pytest.raises(YvexError) as e:
        backend.attention_workspace_required(req)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    # F32 tensors under the bf16 contract are refused as well
    req = backend.attention_requirement(5, 5, 1, 1, 128, contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    with pytest.raises(YvexError) as e:
        backend.attention_workspace_required(req)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    req = backend.attention_requirement(5, 5, 1, 1, 128, deterministic=0)
    with pytest.raises(YvexError) as e:
        backend.attention_workspace_required(req)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    # NaN input -> YVEX_ERR_FORMAT through the device status word; output stays unwritten
    qn = q.copy()
    qn[2, 0, 5] = np.nan
    req = backend.attention_requirement(5, 5, 1, 1, 128)
    out = f32(backend, "out", shape=(5, 1, 128))
    with pytest.raises(YvexError) as e:
        backend.attention_execute(req, f32(backend, "q", qn), f32(backend, "k", k),
                                  f32(backend, "v", v), out)
    assert e.value.code == B.YVEX_ERR_FORMAT and not out.is_written
    # inputs that were never written are refused
    with pytest.raises(YvexError) as e:
        backend.attention_execute(req, f32(backend, "q", shape=(5, 1, 128)), f32(backend, "k", k),
                                  f32(backend, "v", v), out)
    assert e.value.code == B.YVEX_ERR_FORMAT
    good, _ = execute(backend, q, k, v)                            # backend still healthy
    assert np.all(np.isfinite(good))


def test_gqa_uniform_analytic_large(backend):
    for tokens in (65, 5757):
        q, k, v = rv.uniform_large(tokens, 2)
        out, _ = execute(backend, q, k, v, causal=False)
        assert np.abs(out - v).max() <= 2e-3 and np.abs(out - v).max() < 1e-5


def test_lse_output_exact_contract(backend):
    rng = np.random.default_rng(8)
    q = rng.standard_normal((3, 4, 64)).astype(np.float32)
    k = rng.standard_normal((9, 2, 64)).astype(np.float32)
    v = rng.standard_normal((9, 2, 64)).astype(np.float32)
    req = backend.attention_requirement(3, 9, 4, 2, 64, query_start=6)
    out = f32(backend, "out", shape=(3, 4, 64))
    lse = f32(backend, "lse", shape=(3, 4))
    backend.attention_execute(req, f32(backend, "q", q), f32(backend, "k", k), f32(backend, "v", v),
                              out, lse=lse)
    rc, ref, ref_lse = ORACLE.gqa(q, k, v, query_start=6)
    assert np.abs(out.read() - ref).max() < 2e-6
    assert np.abs(lse.read() - ref_lse).max() < 1e-5


# ------------------------------------------------ the fp32 matrix-core kernel ----

def run_exact(backend, q, k, v, **kw):
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    req = backend.attention_requirement(tq, tk, hq, hkv, d, **kw)
    tensors = [f32(backend, "q", q), f32(backend, "k", k), f32(backend, "v", v)]
    out, lse = f32(backend, "out", shape=(tq, hq, d)), f32(backend, "lse", shape=(tq, hq))
    facts = backend.attention_execute(req, *tensors, out, lse=lse)
    result = out.read(), lse.read(), facts
    for t in tensors + [out, lse]:
        t.release()
    return result


@pytest.mark.parametrize("tq,tk,hq,hkv,d,start,causal", [
    (32, 32, 4, 2, 64, 0, True), (33, 33, 4, 1, 128, 0, True), (128, 128, 2, 2, 128, 0, True),
    (129, 129, 5, 1, 64, 0, True), (257, 257, 8, 2, 128, 0, True), (257, 257, 8, 2, 128, 0, False),
    (100, 371, 4, 4, 64, 271, True), (40, 1000, 10, 2, 128, 960, True), (64, 95, 3, 3, 128, 0, False),
    (32, 32, 6, 1, 256, 0, True), (161, 161, 6, 2, 256, 0, True), (70, 333, 24, 4, 256, 263, True),
    (96, 200, 4, 4, 256, 0, False),
])
def test_gqa_matrix_core_kernel_matches_cpu_operator(backend, tq, tk, hq, hkv, d, start, causal):
    """Prefill-shaped EXACT_F32 requests run in tiles on the fp32 matrix cores.  Tolerance is
    the reference's own for its float device kernel against the CPU operator
    (tests/unit/cuda/quant_qtype.c:2293-2333: 2e-5 absolute on N(0,1)-scale rows); ragged
    query and key tails, GQA groups of 1 to 5, cached prefixes and both masks."""
    rng = np.random.default_rng(tq * 131 + tk + d)
    q = rng.standard_normal((tq, hq, d)).astype(np.float32)
    k = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    v = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    out, lse, facts = run_exact(backend, q, k, v, query_start=start, causal=causal)
    assert facts.kernel_launches == 1 and facts.accelerated_matrix_launches == 1
    rc, ref, ref_lse = ORACLE.gqa(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    assert np.abs(out - ref).max() < 2e-5, np.abs(out - ref).max()
    assert np.abs(lse - ref_lse).max() < 2e-5
    again, _, _ = run_exact(backend, q, k, v, query_start=start, causal=causal)
    assert np.array_equal(out, again)                   # deterministic: byte-identical repeat


def test_gqa_kernel_choice_is_a_function_of_geometry(backend):
    """Decode-shaped and odd-sized requests keep the row kernel (double statistics); the two
    kernels agree within the float kernel's tolerance where both could run."""
    rng = np.random.default_rng(77)
    k = rng.standard_normal((300, 2, 128)).astype(np.float32)
    v = rng.standard_normal((300, 2, 128)).astype(np.float32)
    q = rng.standard_normal((32, 4, 128)).astype(np.float32)
    tiled, _, facts = run_exact(backend, q, k, v, query_start=268)
    assert facts.accelerated_matrix_launches == 1
    rows, _, facts = run_exact(backend, q[:31], k[:299], v[:299], query_start=268)   # 31 tokens
    assert facts.accelerated_matrix_launches == 0
    assert np.abs(rows - tiled[:31]).max() < 2e-5
    _, _, facts = run_exact(backend, rng.standard_normal((40, 2, 96)).astype(np.float32),
                            rng.standard_normal((40, 1, 96)).astype(np.float32),
                            rng.standard_normal((40, 1, 96)).astype(np.float32))     # d = 96
    assert facts.accelerated_matrix_launches == 0
    # interleaved [K|V] rows: strided == packed, bit for bit, on the matrix-core kernel too
    tq, hq, d, tk, hkv = 64, 4, 64, 200, 2
    q = rng.standard_normal((tq, hq, d)).astype(np.float32)
    k = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    v = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    kvi = np.zeros((tk, 2 * hkv * d), np.float32)
    kvi[:, :hkv * d] = k.reshape(tk, -1)
    kvi[:, hkv * d:] = v.reshape(tk, -1)
    kvs = f32(backend, "kv-storage", kvi)
    k_view = kvs.view(0, B.DTYPE_F32, ((tk - 1) * 2 * hkv * d + hkv * d,))
    v_view = kvs.view(hkv * d * 4, B.DTYPE_F32, ((tk - 1) * 2 * hkv * d + hkv * d,))
    out_t = f32(backend, "out", shape=(tq, hq, d))
    req = backend.attention_requirement(tq, tk, hq, hkv, d, query_start=tk - tq,
                                        k_stride=2 * hkv * d, v_stride=2 * hkv * d)
    facts = backend.attention_execute(req, f32(backend, "q", q), k_view, v_view, out_t)
    assert facts.accelerated_matrix_launches == 1
    packed, _, _ = run_exact(backend, q, k, v, query_start=tk - tq)
    assert np.array_equal(out_t.read(), packed)


def test_gqa_matrix_core_kernel_flags_non_finite_input(backend):
    rng = np.random.default_rng(78)
    q = rng.standard_normal((64, 2, 64)).astype(np.float32)
    k = rng.standard_normal((64, 1, 64)).astype(np.float32)
    v = rng.standard_normal((64, 1, 64)).astype(np.float32)
    k[17, 0, 3] = np.nan
    with pytest.raises(YvexError) as e:
        run_exact(backend, q, k, v)
    assert e.value.code == B.YVEX_ERR_FORMAT
    good, _, _ = run_exact(backend, q, np.nan_to_num(k), v)       # backend still healthy
    assert np.all(np.isfinite(good))


def test_gqa_matrix_core_kernel_config2_shape(backend):
    """The prefill configuration (2048 tokens, 40/8 heads, d=128) under the exact contract:
    a uniform-key input has the running mean of V as its closed form, and sampled heads are
    held against the CPU operator."""
    rng = np.random.default_rng(79)
    t, hq, hkv, d = 2048, 40, 8, 128
    q = rng.standard_normal((t, hq, d)).astype(np.float32)
    k = rng.standard_normal((t, hkv, d)).astype(np.float32)
    v = rng.standard_normal((t, hkv, d)).astype(np.float32)
    out, lse, facts = run_exact(backend, q, k, v)
    assert facts.accelerated_matrix_launches == 1
    for head in (0, 17, 39):
        group = head // (hq // hkv)
        rc, ref, ref_lse = ORACLE.gqa(q[:, head:head + 1], k[:, group:group + 1], v[:, group:group + 1])
        assert rc == 0
        assert np.abs(out[:, head] - ref[:, 0]).max() < 2e-5
        assert np.abs(lse[:, head] - ref_lse[:, 0]).max() < 2e-5
    # zero queries: every visible key weighs the same, the output is the causal running mean
    out, lse, _ = run_exact(backend, np.zeros_like(q), k, v)
    mean = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, t + 1)[:, None, None]
    want = np.repeat(mean, hq // hkv, axis=1)
    assert np.abs(out - want).max() < 1e-5
    assert np.abs(lse - np.log(np.arange(1, t + 1))[:, None]).max() < 1e-5


@pytest.mark.parametrize("tq,start,hq,hkv,d", [(1000, 0, 40, 8, 128), (777, 300, 48, 8, 64),
                                               (2048, 0, 24, 4, 256)])
def test_gqa_matrix_core_kernel_scheduled_launch_equals_the_first(backend, tq, start, hq, hkv, d):
    """A causal geometry that repeats is launched from item lists (equal work per compute unit)
    from its second call on: the same items, so every output bit and every LSE bit equals the
    first call's, ragged last tiles and a query offset included; sampled heads against the CPU
    operator."""
    rng = np.random.default_rng(tq + d)
    tk = start + tq
    q = rng.standard_normal((tq, hq, d)).astype(np.float32)
    k = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    v = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    req = backend.attention_requirement(tq, tk, hq, hkv, d, query_start=start)
    tensors = [f32(backend, "q", q), f32(backend, "k", k), f32(backend, "v", v)]
    results = []
    for _ in range(3):
        out, lse = f32(backend, "out", shape=(tq, hq, d)), f32(backend, "lse", shape=(tq, hq))
        facts = backend.attention_execute(req, *tensors, out, lse=lse)
        assert facts.accelerated_matrix_launches == 1
        results.append((out.read(), lse.read()))
        out.release()
        lse.release()
    for out, lse in results[1:]:
        assert np.array_equal(out.view(np.uint32), results[0][0].view(np.uint32))
        assert np.array_equal(lse.view(np.uint32), results[0][1].view(np.uint32))
    for head in (0, hq // 2 + 1, hq - 1):
        group = head // (hq // hkv)
        rc, ref, ref_lse = ORACLE.gqa(q[:, head:head + 1], k[:, group:group + 1], v[:, group:group + 1],
                                      query_start=start)
        assert rc == 0
        assert np.abs(results[2][0][:, head] - ref[:, 0]).max() < 2e-5
        assert np.abs(results[2][1][:, head] - ref_lse[:, 0]).max() < 2e-5
    for t in tensors:
        t.release()


# ------------------------------------------------ decode-shaped requests over long contexts ----

@pytest.mark.parametrize("tq,tk,hq,hkv,d,causal", [
    (1, 4096, 32, 8, 128, True), (1, 600, 4, 4, 64, True), (4, 5000, 6, 2, 96, True),
    (2, 1024, 3, 1, 256, True), (1, 513, 2, 2, 8, True), (3, 2000, 4, 2, 128, False),
    (31, 700, 2, 1, 40, True), (1, 16384, 8, 8, 128, True), (1, 70000, 1, 1, 64, True),
])
def test_gqa_split_runs_match_cpu_operator(backend, tq, tk, hq, hkv, d, causal):
    """The decode step of the session layer under the exact contract (one or a few query tokens
    over the whole cached history, src/runtime/stateful_attention.c:326-352): the keys are cut
    into runs, one wave per (token, head, run), double statistics, eight runs per workgroup,
    the workgroups of a (token, head) merged in the kernel by the one that arrives last.
    Same tight bound against the CPU operator as the row kernel."""
    rng = np.random.default_rng(tq * 7 + tk + d)
    q = rng.standard_normal((tq, hq, d)).astype(np.float32)
    k = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    v = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    start = tk - tq if causal else 0
    out, lse, facts = run_exact(backend, q, k, v, query_start=start, causal=causal)
    assert facts.kernel_launches == 1 and facts.accelerated_matrix_launches == 0
    assert facts.temporary_bytes > 0
    rc, ref, ref_lse = ORACLE.gqa(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    assert np.abs(out - ref).max() < 2e-6, np.abs(out - ref).max()
    assert np.abs(lse - ref_lse).max() < 1e-5
    again, _, _ = run_exact(backend, q, k, v, query_start=start, causal=causal)
    assert np.array_equal(out, again)
    # with an attached workspace of the advertised size: no temporary, same bits
    req = backend.attention_requirement(tq, tk, hq, hkv, d, query_start=start, causal=causal)
    need = backend.attention_workspace_required(req)
    assert need == facts.temporary_bytes
    work = backend.tensor("work", B.DTYPE_I8, (need,))
    backend.workspace_attach(work)
    before = backend.memory_stats().allocation_events
    attached, _, facts2 = run_exact(backend, q, k, v, query_start=start, causal=causal)
    assert backend.memory_stats().allocation_events == before + 5      # the five tensors of run_exact
    backend.workspace_detach()
    work.release()
    assert np.array_equal(out, attached) and facts2.kernel_launches == 1


def test_gqa_split_threshold_and_failures(backend):
    rng = np.random.default_rng(80)
    q = rng.standard_normal((1, 4, 64)).astype(np.float32)
    k = rng.standard_normal((511, 2, 64)).astype(np.float32)
    v = rng.standard_normal((511, 2, 64)).astype(np.float32)
    out, _, facts = run_exact(backend, q, k, v, query_start=510)
    assert facts.kernel_launches == 1 and facts.temporary_bytes == 0     # short history: the row kernel
    rc, ref, _ = ORACLE.gqa(q, k, v, query_start=510)
    assert np.abs(out - ref).max() < 2e-6
    k = rng.standard_normal((2048, 2, 64)).astype(np.float32)
    v = rng.standard_normal((2048, 2, 64)).astype(np.float32)
    bad = k.copy()
    bad[1500, 1, 7] = np.inf
    with pytest.raises(YvexError) as e:
        run_exact(backend, q, bad, v, query_start=2047)
    assert e.value.code == B.YVEX_ERR_FORMAT
    bad = v.copy()
    bad[3, 0, 63] = np.nan
    with pytest.raises(YvexError) as e:
        run_exact(backend, q, k, bad, query_start=2047)
    assert e.value.code == B.YVEX_ERR_FORMAT
    good, _, facts = run_exact(backend, q, k, v, query_start=2047)
    assert facts.kernel_launches == 1 and facts.temporary_bytes > 0 and np.all(np.isfinite(good))
    # a query in the middle of the history: runs past its visible keys contribute nothing
    mid, _, _ = run_exact(backend, q, k, v, query_start=700)
    rc, ref, _ = ORACLE.gqa(q, k[:701], v[:701], query_start=700)
    assert np.abs(mid - ref).max() < 2e-6
