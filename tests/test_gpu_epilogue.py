"""GPU parity: the sigmoid output gate fused into the attention epilogue (prefill, row decode,
paged decode), against the CPU operator followed by the CPU gate, through the C ABI."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError, kv_pack_pages, q8_0_encode_rows
from gpu_common import ORACLE, assert_close_bf16, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu


def gated_reference(attention_f32, gate_bits):
    """The reference order of operations: publish the attention rows as bf16, then
    bf16(row * sigmoid(gate)) (src/runtime/decoder.c:1266-1269)."""
    published = ORACLE.bf16_decode(ORACLE.bf16_encode(attention_f32))
    return ORACLE.sigmoid_gate_bf16(published, ORACLE.bf16_decode(gate_bits)).reshape(attention_f32.shape)


def assert_gate_of(fused_bits, plain_bits, gate_bits, label):
    """The fused rows against the CPU gate applied to the device's own ungated rows: only the
    device exp/reciprocal differ from libm, so at most one bf16 step, and rarely."""
    want = ORACLE.bf16_encode(ORACLE.sigmoid_gate_bf16(ORACLE.bf16_decode(plain_bits),
                                                       ORACLE.bf16_decode(gate_bits)))
    want = want.reshape(fused_bits.shape)
    step = np.abs(fused_bits.astype(np.int32) - want.astype(np.int32))
    assert step.max() <= 1, "%s: %d bf16 steps" % (label, step.max())
    assert np.count_nonzero(step) <= max(4, fused_bits.size // 200), label


@pytest.mark.parametrize("tq,tk,start,hq,hkv,causal", [
    (5, 5, 0, 2, 1, True), (130, 130, 0, 4, 2, True), (257, 700, 443, 8, 2, True),
    (200, 333, 0, 5, 5, False), (512, 512, 0, 40, 8, True),
])
def test_prefill_with_fused_gate(backend, tq, tk, start, hq, hkv, causal):
    rng = np.random.default_rng(7000 + tq + tk)
    q, k, v = (bf16_normal(rng, (n, h, 128)) for n, h in ((tq, hq), (tk, hkv), (tk, hkv)))
    gate = bf16_normal(rng, (tq, hq, 128), scale=2.5)
    req = backend.attention_requirement(tq, tk, hq, hkv, 128, causal=causal, query_start=start,
                                        dtype=B.DTYPE_BF16, contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    t = [backend.tensor("q", B.DTYPE_BF16, q.shape, q), backend.tensor("k", B.DTYPE_BF16, k.shape, k),
         backend.tensor("v", B.DTYPE_BF16, v.shape, v)]
    tg = backend.tensor("gate", B.DTYPE_BF16, gate.shape, gate)
    plain, fused = backend.tensor("o", B.DTYPE_BF16, q.shape), backend.tensor("og", B.DTYPE_BF16, q.shape)
    lse = backend.tensor("lse", B.DTYPE_F32, (tq, hq))
    backend.attention_execute(req, *t, plain)
    facts = backend.attention_execute(req, *t, fused, lse=lse, gate=tg)
    assert facts.kernel_launches == 1
    rc, ref, _, _ = ORACLE.gqa_bf16(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    label = "prefill gate tq=%d tk=%d" % (tq, tk)
    assert_close_bf16(fused.read(), gated_reference(ref, gate), label)
    assert_gate_of(fused.read(), plain.read(), gate, label)
    assert np.all(np.isfinite(lse.read()))
    for x in t + [tg, plain, fused, lse]:
        x.release()


@pytest.mark.parametrize("d", [128, 64, 256])
@pytest.mark.parametrize("ctx", [1, 17, 300, 4096])
def test_row_decode_with_fused_gate(backend, ctx, d):
    rng = np.random.default_rng(7100 + ctx + d)
    q = bf16_normal(rng, (1, 32, d))
    k, v = bf16_normal(rng, (ctx, 8, d)), bf16_normal(rng, (ctx, 8, d))
    gate = bf16_normal(rng, (1, 32, d), scale=2.5)
    req = backend.attention_requirement(1, ctx, 32, 8, d, causal=True, query_start=ctx - 1,
                                        dtype=B.DTYPE_BF16, contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    t = [backend.tensor("q", B.DTYPE_BF16, q.shape, q), backend.tensor("k", B.DTYPE_BF16, k.shape, k),
         backend.tensor("v", B.DTYPE_BF16, v.shape, v)]
    tg = backend.tensor("gate", B.DTYPE_BF16, gate.shape, gate)
    plain, fused = backend.tensor("o", B.DTYPE_BF16, q.shape), backend.tensor("og", B.DTYPE_BF16, q.shape)
    backend.attention_execute(req, *t, plain)
    facts = backend.attention_execute(req, *t, fused, gate=tg)
    assert facts.kernel_launches == 1
    rc, ref, _, _ = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=True)
    assert rc == 0
    assert_close_bf16(fused.read(), gated_reference(ref, gate), "row decode gate ctx=%d" % ctx)
    assert_gate_of(fused.read(), plain.read(), gate, "row decode gate ctx=%d" % ctx)
    for x in t + [tg, plain, fused]:
        x.release()


@pytest.mark.parametrize("q8", [False, True], ids=["bf16", "q8_0"])
def test_paged_decode_with_fused_gate(backend, q8):
    """Short contexts (rows published by the decode kernel itself) and long ones (merged by
    the merging wave) in one batch: the gate reaches both."""
    rng = np.random.default_rng(7200 + q8)
    sessions, hq, hkv, d, page = 6, 32, 8, 128, 16
    contexts = np.array([1, 16, 33, 900, 5000, 12000], np.int32)
    need = (contexts + page - 1) // page
    pool_pages, stride = int(need.sum()) + 2, int(need.max())
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((sessions, stride), np.int32)
    at = 0
    for s in range(sessions):
        table[s, :need[s]] = perm[at:at + need[s]]
        at += int(need[s])
    k_rows, v_rows = bf16_normal(rng, (pool_pages, page, hkv, d)), bf16_normal(rng, (pool_pages, page, hkv, d))
    storage, dtype = (B.KV_Q8_0, B.DTYPE_I8) if q8 else (B.KV_BF16, B.DTYPE_BF16)
    if q8:
        k_rows = q8_0_encode_rows(ORACLE.bf16_decode(k_rows))
        v_rows = q8_0_encode_rows(ORACLE.bf16_decode(v_rows))
    q = bf16_normal(rng, (sessions, hq, d))
    gate = bf16_normal(rng, (sessions, hq, d), scale=2.5)
    kp, vp = kv_pack_pages(k_rows, storage, False, hkv), kv_pack_pages(v_rows, storage, True, hkv)
    t = [backend.tensor("q", B.DTYPE_BF16, q.shape, q),
         backend.tensor("kp", dtype, (kp.size // B.DTYPE_BYTES[dtype],), kp),
         backend.tensor("vp", dtype, (vp.size // B.DTYPE_BYTES[dtype],), vp),
         backend.tensor("t", B.DTYPE_I32, table.shape, table),
         backend.tensor("c", B.DTYPE_I32, contexts.shape, contexts)]
    tg = backend.tensor("gate", B.DTYPE_BF16, gate.shape, gate)
    plain, fused = backend.tensor("o", B.DTYPE_BF16, q.shape), backend.tensor("og", B.DTYPE_BF16, q.shape)
    req = backend.paged_requirement(sessions, hq, hkv, d, page, pool_pages, stride,
                                    int(stride * page), storage=storage)
    backend.paged_decode_execute(req, *t, plain)
    facts = backend.paged_decode_execute(req, *t, fused, gate=tg)
    assert facts.kernel_launches in (1, 2)
    rc, ref, _, _ = ORACLE.paged_decode(q, k_rows, v_rows, table, contexts, hkv, page, q8=q8)
    assert rc == 0
    assert_close_bf16(fused.read(), gated_reference(ref, gate), "paged gate")
    assert_gate_of(fused.read(), plain.read(), gate, "paged gate")
    for x in t + [tg, plain, fused]:
        x.release()


def test_fused_gate_refusals(backend):
    rng = np.random.default_rng(7300)
    tq, hq, hkv = 4, 2, 1
    q, k, v = (bf16_normal(rng, (tq, h, 128)) for h in (hq, hkv, hkv))
    req = backend.attention_requirement(tq, tq, hq, hkv, 128, causal=True, dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    t = [backend.tensor("q", B.DTYPE_BF16, q.shape, q), backend.tensor("k", B.DTYPE_BF16, k.shape, k),
         backend.tensor("v", B.DTYPE_BF16, v.shape, v)]
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    short = backend.tensor("g", B.DTYPE_BF16, (tq, hq, 64), bf16_normal(rng, (tq, hq, 64)))
    with pytest.raises(YvexError) as e:                       # gate geometry
        backend.attention_execute(req, *t, out, gate=short)
    assert e.value.code == B.YVEX_ERR_FORMAT
    unwritten = backend.tensor("g2", B.DTYPE_BF16, q.shape)
    with pytest.raises(YvexError) as e:                       # gate never written
        backend.attention_execute(req, *t, out, gate=unwritten)
    assert e.value.code == B.YVEX_ERR_FORMAT
    nan_gate = bf16_normal(rng, q.shape)
    nan_gate[2, 1, 5] = 0x7FC0
    with pytest.raises(YvexError) as e:                       # NaN gate -> numeric flag
        backend.attention_execute(req, *t, out, gate=backend.tensor("g3", B.DTYPE_BF16, q.shape, nan_gate))
    assert e.value.code == B.YVEX_ERR_FORMAT
    # the exact F32 contract takes no epilogue
    qf, kf, vf = (ORACLE.bf16_decode(x) for x in (q, k, v))
    exact = backend.attention_requirement(tq, tq, hq, hkv, 128, causal=True)
    tf = [backend.tensor("qf", B.DTYPE_F32, qf.shape, qf), backend.tensor("kf", B.DTYPE_F32, kf.shape, kf),
          backend.tensor("vf", B.DTYPE_F32, vf.shape, vf)]
    outf = backend.tensor("of", B.DTYPE_F32, qf.shape)
    good = backend.tensor("g4", B.DTYPE_BF16, q.shape, bf16_normal(rng, q.shape))
    with pytest.raises(YvexError) as e:
        backend.attention_execute(exact, *tf, outf, gate=good)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
