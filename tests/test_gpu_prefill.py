"""GPU parity: bf16 MFMA prefill (multi-token GQA, causal and full) against the CPU
operator, through the reference's attention_execute contract."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu


def run_prefill(backend, q, k, v, query_start=0, causal=True, want_lse=True):
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    req = backend.attention_requirement(tq, tk, hq, hkv, d, causal=causal, query_start=query_start,
                                        dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    lse = backend.tensor("lse", B.DTYPE_F32, (tq, hq)) if want_lse else None
    facts = backend.attention_execute(req, backend.tensor("q", B.DTYPE_BF16, q.shape, q),
                                      backend.tensor("k", B.DTYPE_BF16, k.shape, k),
                                      backend.tensor("v", B.DTYPE_BF16, v.shape, v), out, lse=lse)
    return out.read(), (lse.read() if lse else None), facts


@pytest.mark.parametrize("tq,tk,start,hq,hkv,causal", [
    (2, 2, 0, 2, 1, True), (5, 5, 0, 1, 1, True), (64, 64, 0, 4, 2, True),
    (65, 65, 0, 5, 1, True), (257, 257, 0, 2, 2, True), (300, 300, 0, 10, 2, False),
    (3, 131, 128, 8, 2, True), (200, 1000, 800, 5, 1, True), (129, 640, 100, 4, 4, False),
    (512, 512, 0, 40, 8, True),
])
def test_prefill_matches_cpu_operator(backend, tq, tk, start, hq, hkv, causal):
    rng = np.random.default_rng(tq * 1000 + tk)
    q = bf16_normal(rng, (tq, hq, 128))
    k = bf16_normal(rng, (tk, hkv, 128))
    v = bf16_normal(rng, (tk, hkv, 128))
    got, lse, facts = run_prefill(backend, q, k, v, query_start=start, causal=causal)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    label = "tq=%d tk=%d start=%d %s" % (tq, tk, start, "causal" if causal else "full")
    assert_close_bf16(got, ref, label)
    assert_lse(lse, ref_lse, label)
    assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
    if causal and start == 0:
        # the first causal row sees only key 0: the output is exactly V[0] of its kv head
        for h in range(hq):
            assert np.array_equal(got[0, h], v[0, h // (hq // hkv)])


def test_config2_prefill_qwen_shape(backend):
    """Benchmark configuration 2: T=2048, 40/8 heads, d=128, causal, N(0,1) values with a per-head
    scale drawn U[0.5,1.5], seed 2."""
    rng = np.random.default_rng(2)
    t, hq, hkv, d = 2048, 40, 8, 128
    q = bf16_normal(rng, (t, hq, d)) if False else None
    sq = rng.uniform(0.5, 1.5, size=(1, hq, 1)).astype(np.float32)
    skv = rng.uniform(0.5, 1.5, size=(1, hkv, 1)).astype(np.float32)
    q = ORACLE.bf16_encode(rng.standard_normal((t, hq, d)).astype(np.float32) * sq)
    k = ORACLE.bf16_encode(rng.standard_normal((t, hkv, d)).astype(np.float32) * skv)
    v = ORACLE.bf16_encode(rng.standard_normal((t, hkv, d)).astype(np.float32) * skv)
    got, lse, _ = run_prefill(backend, q, k, v)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=0, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, "config2")
    assert_lse(lse, ref_lse, "config2")
    again, lse2, _ = run_prefill(backend, q, k, v)
    assert np.array_equal(got, again) and np.array_equal(lse, lse2)   # deterministic


def test_prefill_strided_views_equal_packed(backend):
    rng = np.random.default_rng(9)
    tq, tk, hq, hkv, d = 70, 200, 8, 2, 128
    q = bf16_normal(rng, (tq, hq, d))
    k = bf16_normal(rng, (tk, hkv, d))
    v = bf16_normal(rng, (tk, hkv, d))
    qw, kw = hq * d, hkv * d
    qi = np.full((tq, 2 * qw), 0x7FC0, dtype=np.uint16)      # [Q | gate], gate = NaN pattern
    qi[:, :qw] = q.reshape(tq, qw)
    kvi = np.zeros((tk, 2 * kw), dtype=np.uint16)           # [K | V]
    kvi[:, :kw] = k.reshape(tk, kw)
    kvi[:, kw:] = v.reshape(tk, kw)
    qs = backend.tensor("q-storage", B.DTYPE_BF16, qi.shape, qi)
    kvs = backend.tensor("kv-storage", B.DTYPE_BF16, kvi.shape, kvi)
    q_view = qs.view(0, B.DTYPE_BF16, ((tq - 1) * 2 * qw + qw,))
    k_view = kvs.view(0, B.DTYPE_BF16, ((tk - 1) * 2 * kw + kw,))
    v_view = kvs.view(kw * 2, B.DTYPE_BF16, ((tk - 1) * 2 * kw + kw,))
    out = backend.tensor("o", B.DTYPE_BF16, (tq, hq, d))
    req = backend.attention_requirement(tq, tk, hq, hkv, d, query_start=tk - tq,
                                        dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE,
                                        q_stride=2 * qw, k_stride=2 * kw, v_stride=2 * kw)
    backend.attention_execute(req, q_view, k_view, v_view, out)
    packed, _, _ = run_prefill(backend, q, k, v, query_start=tk - tq, want_lse=False)
    assert np.array_equal(out.read(), packed)


def test_prefill_refusals(backend):
    rng = np.random.default_rng(10)
    q = bf16_normal(rng, (4, 2, 128))
    k = bf16_normal(rng, (4, 1, 128))
    with pytest.raises(YvexError) as e:                      # query range beyond KV history
        run_prefill(backend, q, k, k, query_start=1)
    assert e.value.code == B.YVEX_ERR_INVALID_ARG
    req = backend.attention_requirement(4, 4, 2, 1, 96, dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    with pytest.raises(YvexError) as e:                      # head dimension the MFMA path lacks
        backend.attention_workspace_required(req)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    qn = q.copy()
    qn[1, 0, 3] = 0x7FC0                                     # NaN query -> FORMAT, output unwritten
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    req = backend.attention_requirement(4, 4, 2, 1, 128, dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    with pytest.raises(YvexError) as e:
        backend.attention_execute(req, backend.tensor("q", B.DTYPE_BF16, q.shape, qn),
                                  backend.tensor("k", B.DTYPE_BF16, k.shape, k),
                                  backend.tensor("v", B.DTYPE_BF16, k.shape, k), out)
    assert e.value.code == B.YVEX_ERR_FORMAT and not out.is_written


@pytest.mark.parametrize("tq,tk,start,hq,hkv", [(4100, 4100, 0, 4, 1), (700, 9000, 8300, 4, 2)])
def test_prefill_long_sequences(backend, tq, tk, start, hq, hkv):
    """Twice the benchmark's sequence length, and a prompt chunk behind a long history."""
    rng = np.random.default_rng(tq + tk)
    q = bf16_normal(rng, (tq, hq, 128))
    k = bf16_normal(rng, (tk, hkv, 128))
    v = bf16_normal(rng, (tk, hkv, 128))
    got, lse, _ = run_prefill(backend, q, k, v, query_start=start, causal=True)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=start, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, "long prefill %d/%d" % (tq, tk))
    assert_lse(lse, ref_lse, "long prefill %d/%d" % (tq, tk))


@pytest.mark.parametrize("d", [64, 256])
@pytest.mark.parametrize("tq,tk,start,hq,hkv,causal", [
    (2, 2, 0, 2, 1, True), (65, 65, 0, 5, 1, True), (257, 257, 0, 4, 2, True),
    (300, 300, 0, 6, 2, False), (3, 131, 128, 8, 2, True), (200, 1000, 800, 4, 1, True),
    (1, 700, 699, 8, 2, True),          # one query token: a one-row tile of the same kernel
])
def test_prefill_other_head_dimensions(backend, d, tq, tk, start, hq, hkv, causal):
    """Head dimensions 64 and 256 are the same kernel with other counts (k-steps, dim blocks,
    loads per tile, LDS swizzle for 128-byte rows)."""
    rng = np.random.default_rng(d * 100000 + tq * 1000 + tk)
    q = bf16_normal(rng, (tq, hq, d))
    k = bf16_normal(rng, (tk, hkv, d))
    v = bf16_normal(rng, (tk, hkv, d))
    got, lse, facts = run_prefill(backend, q, k, v, query_start=start, causal=causal)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    label = "d=%d tq=%d tk=%d start=%d %s" % (d, tq, tk, start, "causal" if causal else "full")
    assert_close_bf16(got, ref, label)
    assert_lse(lse, ref_lse, label)
    assert facts.kernel_launches == 1 and facts.accelerated_matrix_launches == 1
    if causal and start == 0:
        for h in range(hq):
            assert np.array_equal(got[0, h], v[0, h // (hq // hkv)])


@pytest.mark.parametrize("t,hq,hkv,d", [(1024, 24, 4, 256), (1024, 16, 4, 64)])
def test_prefill_reference_qwen_patterns(backend, t, hq, hkv, d):
    """The geometry of the reference's own Qwen attention test (24 query heads, 4 KV heads,
    head dimension 256: tests/unit/cuda/quant_qtype.c:2413-2454) and its narrow sibling, as
    causal prefill under the bf16 contract, with per-head scales as in configuration 2."""
    rng = np.random.default_rng(t + d)
    sq = rng.uniform(0.5, 1.5, size=(1, hq, 1)).astype(np.float32)
    skv = rng.uniform(0.5, 1.5, size=(1, hkv, 1)).astype(np.float32)
    q = ORACLE.bf16_encode(rng.standard_normal((t, hq, d)).astype(np.float32) * sq)
    k = ORACLE.bf16_encode(rng.standard_normal((t, hkv, d)).astype(np.float32) * skv)
    v = ORACLE.bf16_encode(rng.standard_normal((t, hkv, d)).astype(np.float32) * skv)
    got, lse, _ = run_prefill(backend, q, k, v)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=0, causal=True)
    assert rc == 0
    assert_close_bf16(got, ref, "qwen pattern d=%d" % d)
    assert_lse(lse, ref_lse, "qwen pattern d=%d" % d)
    again, lse2, _ = run_prefill(backend, q, k, v)
    assert np.array_equal(got, again) and np.array_equal(lse, lse2)
