"""Pins the CPU oracle: reference-held vectors, the compiled reference operator
(oracle/_ref, when built), closed forms and brute force.  CPU only."""
import ctypes as C
import math

import numpy as np
import pytest

import reference_vectors as rv
from oracle_binding import (Oracle, load_reference, load_reference_reduce, reference_reduce, _ptr,
                            f32p, u16p, u8p)

ORACLE = Oracle()
REF = load_reference()
needs_ref = pytest.mark.skipif(REF is None, reason="oracle/_ref not built (reference tree absent)")
REF_REDUCE = load_reference_reduce()
needs_ref_reduce = pytest.mark.skipif(REF_REDUCE is None,
                                      reason="oracle/_ref not built (reference tree absent)")


# ---------------------------------------------------------------- exp -------

def test_exp_matches_libm_and_clamps():
    xs = np.concatenate([np.linspace(-60, 0, 4001), np.linspace(0, 60, 401)])
    for x in xs:
        got = ORACLE.lib.yvo_exp(float(x))
        assert abs(got - math.exp(x)) <= 1e-13 * math.exp(x)   # range reduction by repeated ln2 steps
    assert ORACLE.lib.yvo_exp(-60.0000001) == 0.0          # below -60 is exactly zero
    assert ORACLE.lib.yvo_exp(100.0) == ORACLE.lib.yvo_exp(60.0)   # clamp above 60
    assert ORACLE.lib.yvo_exp(0.0) == 1.0


# ------------------------------------------------------------- codecs -------

def test_bf16_reference_literals():
    for value, bits in rv.BF16_LITERALS:
        assert ORACLE.lib.yvo_bf16_encode(value) == bits


def test_bf16_exhaustive_round_trip_and_ties():
    bits = np.arange(1 << 16, dtype=np.uint16)
    vals = ORACLE.bf16_decode(bits)
    back = ORACLE.bf16_encode(vals)
    nan = np.isnan(vals)
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.all((back[nan] & 0x0040) != 0)        # NaNs come back quiet
    # ties go to even: 1 + 2^-8 is halfway between 0x3f80 and 0x3f81 -> even (0x3f80);
    # 1 + 3*2^-8 is halfway between 0x3f81 and 0x3f82 -> even (0x3f82)
    assert ORACLE.lib.yvo_bf16_encode(1.0 + 2.0 ** -8) == 0x3F80
    assert ORACLE.lib.yvo_bf16_encode(1.0 + 3 * 2.0 ** -8) == 0x3F82
    # independent check against numpy integer arithmetic on random floats
    rng = np.random.default_rng(7)
    x = rng.standard_normal(200000).astype(np.float32) * np.float32(37.0)
    u = x.view(np.uint32)
    expect = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(ORACLE.bf16_encode(x), expect)


def test_f16_exhaustive_round_trip_against_numpy():
    bits = np.arange(1 << 16, dtype=np.uint16)
    expect = bits.view(np.float16).astype(np.float32)
    got = np.array([ORACLE.lib.yvo_f16_decode(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(expect)
    assert np.array_equal(got[~nan].view(np.uint32), expect[~nan].view(np.uint32))
    assert np.all(np.isnan(got[nan]))
    back = np.array([ORACLE.lib.yvo_f16_encode(float(v)) for v in got[~nan]], dtype=np.uint16)
    assert np.array_equal(back, bits[~nan])
    # RNE against numpy for random floats incl. subnormal and overflow ranges
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(20000) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 3e4, 1e6)])
    x = x.astype(np.float32)
    mine = np.array([ORACLE.lib.yvo_f16_encode(float(v)) for v in x], dtype=np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(mine, x.astype(np.float16).view(np.uint16))


@needs_ref
def test_codecs_match_compiled_reference():
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(300000) * s for s in (1e-8, 1e-4, 1.0, 1e5)])
    x = np.concatenate([x, [0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65520.0, 6e-8, 3e-8]])
    x = x.astype(np.float32)
    ref_b = np.empty(x.size, dtype=np.uint16)
    ref_h = np.empty(x.size, dtype=np.uint16)
    REF.yvref_bf16_encode_n(_ptr(x, f32p), _ptr(ref_b, u16p), x.size)
    REF.yvref_f16_encode_n(_ptr(x, f32p), _ptr(ref_h, u16p), x.size)
    assert np.array_equal(ORACLE.bf16_encode(x), ref_b)
    mine_h = np.array([ORACLE.lib.yvo_f16_encode(float(v)) for v in x], dtype=np.uint16)
    # python float() of a float32 NaN loses nothing that matters here: compare non-NaN exactly
    ok = ~np.isnan(x)
    assert np.array_equal(mine_h[ok], ref_h[ok])
    bits = np.arange(1 << 16, dtype=np.uint16)
    ref_d = np.empty(bits.size, dtype=np.float32)
    REF.yvref_f16_decode_n(_ptr(bits, u16p), _ptr(ref_d, f32p), bits.size)
    mine_d = np.array([ORACLE.lib.yvo_f16_decode(int(b)) for b in bits], dtype=np.float32)
    assert np.array_equal(mine_d.view(np.uint32), ref_d.view(np.uint32))


def test_q8_0_golden_zero_and_refusals():
    enc = ORACLE.q8_0_encode_rows(rv.Q8_0_GOLDEN_SOURCE)
    assert bytes(enc[:6]) == rv.Q8_0_GOLDEN_PREFIX            # halfway codes round away from zero
    assert not enc[6:].any()
    zero = ORACLE.q8_0_encode_rows(np.zeros(32, dtype=np.float32))
    assert not zero.any()                                        # canonical zero block
    assert np.array_equal(ORACLE.q8_0_decode_rows(zero, 32).view(np.uint32),
                          np.zeros(32, dtype=np.uint32))
    out = np.empty(34, dtype=np.uint8)
    huge = np.full(32, np.finfo(np.float32).max, dtype=np.float32)
    assert ORACLE.lib.yvo_q8_0_encode_block(_ptr(huge, f32p), _ptr(out, u8p)) == 0
    bad = np.zeros(34, dtype=np.uint8)
    bad[1] = 0x7C                                                 # +inf scale
    dec = np.empty(32, dtype=np.float32)
    assert ORACLE.lib.yvo_q8_0_decode_block(_ptr(bad, u8p), _ptr(dec, f32p)) == 0
    bad[1] = 0xBC                                                 # negative scale
    assert ORACLE.lib.yvo_q8_0_decode_block(_ptr(bad, u8p), _ptr(dec, f32p)) == 0


def test_q8_0_invariants():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((512, 128)).astype(np.float32)
    enc = ORACLE.q8_0_encode_rows(x)
    dec = ORACLE.q8_0_decode_rows(enc, 128)
    scales = enc.reshape(512, 4, 34)[:, :, :2].copy().view(np.float16).astype(np.float32)
    err = np.abs(dec - x).reshape(512, 4, 32)
    # half a step, plus the clamp slack when the f16 scale rounded below absmax/127
    amax = np.abs(x).reshape(512, 4, 32).max(axis=2, keepdims=True)
    slack = np.maximum(amax - 127.0 * scales, 0.0)
    assert np.all(err <= scales / 2 + slack + 1e-7)
    # idempotent on decoded values
    assert np.array_equal(ORACLE.q8_0_encode_rows(dec), enc)
    codes = enc.reshape(512, 4, 34)[:, :, 2:].view(np.int8)
    assert codes.min() >= -127


@needs_ref
def test_q8_0_matches_compiled_reference():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((4000, 32)) * rng.uniform(1e-6, 50.0, (4000, 1))).astype(np.float32)
    x[0] = 0.0
    x[1, 3] = 0.5 * 127 / 127   # exact-half code cases
    mine = ORACLE.q8_0_encode_rows(x)
    for row in range(x.shape[0]):
        out = np.zeros(34, dtype=np.uint8)
        src = np.ascontiguousarray(x[row])
        assert REF.yvref_q8_0_encode_block(_ptr(src, f32p), _ptr(out, u8p)) == 0
        assert np.array_equal(out, mine[row]), row
        dec = np.zeros(32, dtype=np.float32)
        assert REF.yvref_q8_0_decode_block(_ptr(out, u8p), _ptr(dec, f32p)) == 0
        assert np.array_equal(dec.view(np.uint32),
                              ORACLE.q8_0_decode_rows(mine[row], 32).view(np.uint32))


# --------------------------------------------------- single-head operator ----

def test_single_head_reference_literals():
    rc, out, _, _, _ = ORACLE.attention_head(rv.CPU_OP_QUERY, rv.CPU_OP_KEYS, rv.CPU_OP_VALUES,
                                             0, rv.CPU_OP_SCALE)
    assert rc == 0 and np.allclose(out, rv.CPU_OP_VALUES[0], atol=1e-6)
    rc, out, score, prob, lse = ORACLE.attention_head(rv.CPU_OP_QUERY, rv.CPU_OP_KEYS,
                                                      rv.CPU_OP_VALUES, 2, rv.CPU_OP_SCALE)
    assert rc == 0 and abs(out[0] - rv.CPU_OP_VALUES[0, 0]) > 1e-4
    s = (rv.CPU_OP_KEYS.astype(np.float64) @ rv.CPU_OP_QUERY.astype(np.float64)) * 0.5
    p = np.exp(s - s.max())
    p /= p.sum()
    assert np.allclose(out, p @ rv.CPU_OP_VALUES.astype(np.float64), atol=1e-5)
    assert abs(lse - (s.max() + math.log(np.exp(s - s.max()).sum()))) < 1e-7
    assert abs(prob.sum() - 1.0) < 1e-6
    rc, *_ = ORACLE.attention_head(rv.CPU_OP_QUERY, rv.CPU_OP_KEYS, rv.CPU_OP_VALUES, 3,
                                   rv.CPU_OP_SCALE)
    assert rc == -7                                               # YVEX_ERR_BOUNDS
    for bad in (0.0, -1.0, float("nan"), float("inf")):
        rc, *_ = ORACLE.attention_head(rv.CPU_OP_QUERY, rv.CPU_OP_KEYS, rv.CPU_OP_VALUES, 0, bad)
        assert rc == -10                                          # YVEX_ERR_INVALID_ARG


def test_single_head_closed_forms():
    rng = np.random.default_rng(1)
    n, d = 300, 64
    k = rng.standard_normal((n, d)).astype(np.float32)
    v = rng.standard_normal((n, d)).astype(np.float32)
    # Q = 0  =>  uniform mean of the visible values, LSE = ln(visible)
    rc, out, _, prob, lse = ORACLE.attention_head(np.zeros(d, np.float32), k, v, 99, 0.125)
    assert rc == 0 and np.allclose(out, v[:100].astype(np.float64).mean(axis=0), atol=1e-6)
    assert abs(lse - math.log(100)) < 1e-12 and not prob[100:].any()
    # one dominant key => that value row; masked future rows are never read
    q = rng.standard_normal(d).astype(np.float32)
    k2 = k * np.float32(0.01)
    k2[17] = q * np.float32(40.0)
    k2[250] = q * np.float32(400.0)          # beyond the causal position: must not matter
    rc, out, *_ = ORACLE.attention_head(q, k2, v, 200, 1.0)
    assert rc == 0 and np.allclose(out, v[17], atol=1e-6)
    # non-causal sees every row
    rc, out, *_ = ORACLE.attention_head(q, k2, v, 0, 1.0, causal=False)
    assert rc == 0 and np.allclose(out, v[250], atol=1e-6)


def test_single_head_brute_force_libm():
    rng = np.random.default_rng(2)
    for n, d, scale in ((1, 8, 1.0), (7, 16, 0.25), (513, 128, 0.088388346)):
        q = rng.standard_normal(d).astype(np.float32)
        k = rng.standard_normal((n, d)).astype(np.float32)
        v = rng.standard_normal((n, d)).astype(np.float32)
        pos = n - 1
        rc, out, score, prob, lse = ORACLE.attention_head(q, k, v, pos, scale)
        s = (k.astype(np.float64) @ q.astype(np.float64)) * np.float64(np.float32(scale))
        e = np.exp(s - s.max())
        expect = (e / e.sum()) @ v.astype(np.float64)
        assert rc == 0 and np.allclose(out, expect, atol=3e-6)
        assert abs(lse - (s.max() + math.log(e.sum()))) < 1e-6


@needs_ref
def test_single_head_bit_exact_against_compiled_reference():
    """The restatement must reproduce the reference operator bit for bit, including the
    float score store and both probability roundings."""
    rng = np.random.default_rng(4)
    cases = [(3, 4, 0, 0.5, 1), (64, 128, 63, 0.0883883461356163, 1),
             (777, 128, 500, 0.0883883461356163, 1), (777, 96, 3, 0.3, 0),
             (4096, 128, 4095, 0.0883883461356163, 1), (2000, 256, 1999, 0.0625, 1)]
    for n, d, pos, scale, causal in cases:
        q = (rng.standard_normal(d) * 1.5).astype(np.float32)
        k = rng.standard_normal((n, d)).astype(np.float32)
        v = rng.standard_normal((n, d)).astype(np.float32)
        rs = np.zeros(n, np.float32)
        rp = np.zeros(n, np.float32)
        ro = np.zeros(d, np.float32)
        rc_ref = REF.yvref_op_attention(_ptr(q, f32p), _ptr(k, f32p), _ptr(v, f32p), n, pos, d,
                                        scale, causal, _ptr(rs, f32p), _ptr(rp, f32p),
                                        _ptr(ro, f32p))
        rc, out, score, prob, _ = ORACLE.attention_head(q, k, v, pos, scale, bool(causal))
        assert rc == rc_ref == 0
        assert np.array_equal(score.view(np.uint32), rs.view(np.uint32))
        assert np.array_equal(prob.view(np.uint32), rp.view(np.uint32))
        assert np.array_equal(out.view(np.uint32), ro.view(np.uint32))
    # refusal statuses agree too
    q = np.ones(4, np.float32)
    k = np.ones((3, 4), np.float32)
    for n, pos, scale in ((3, 3, 0.5), (3, 0, 0.0), (3, 0, float("nan")), (0, 0, 0.5)):
        rc_ref = REF.yvref_op_attention(_ptr(q, f32p), _ptr(k, f32p), _ptr(k, f32p), n, pos, 4,
                                        scale, 1, None, None, None)
        rc = ORACLE.lib.yvo_attention_head(_ptr(q, f32p), _ptr(k, f32p), 4, _ptr(k, f32p), 4, n,
                                           pos, 4, scale, 1, None, None, _ptr(q.copy(), f32p),
                                           None)
        assert rc == rc_ref and rc != 0


# ------------------------------------------------------- multi-token GQA ----

def test_gqa_reference_known_answer():
    q, k, v, mixed = rv.gqa_kat()
    rc, out, _ = ORACLE.gqa(q, k, v, causal=True)
    assert rc == 0
    assert np.array_equal(out[0], np.array([[2.0, 4.0], [2.0, 4.0]], dtype=np.float32))
    assert np.allclose(out[1], mixed, atol=1e-6)
    rc, out, _ = ORACLE.gqa(q, k, v, causal=False)
    assert rc == 0 and np.allclose(out, np.broadcast_to(mixed, (2, 2, 2)), atol=1e-6)


@pytest.mark.parametrize("maker,start,tol_abs,tol_rel", [
    (rv.small_5x128, 0, 2e-5, 0.0),
    (rv.qwen_24_4_256, 0, 2e-4, 2e-4),
    (rv.tiled_257x128, 0, 0.0, 2e-3),
])
def test_gqa_reference_patterns_against_float_checker(maker, start, tol_abs, tol_rel):
    q, k, v = maker()
    for causal in (True, False):
        rc, out, _ = ORACLE.gqa(q, k, v, query_start=start, causal=causal)
        ref = rv.float_two_pass_gqa(q, k, v, start, causal)
        assert rc == 0
        assert np.all(np.abs(out - ref) <= tol_abs + tol_rel * (1.0 + np.abs(ref)) + 1e-7)


def test_gqa_cached_decode_and_query_range():
    q, k, v = rv.cached_decode_qwen()
    rc, out, _ = ORACLE.gqa(q, k, v, query_start=2, causal=True)
    ref = rv.float_two_pass_gqa(q, k, v, 2, True)
    assert rc == 0 and np.all(np.abs(out - ref) <= 2e-4 * (1.0 + np.abs(ref)))
    rc, *_ = ORACLE.gqa(q, k, v, query_start=3, causal=True)      # query range beyond KV
    assert rc == -10


def test_gqa_strided_views_equal_packed():
    q, k, v = rv.strided_qwen()
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    qi = np.zeros((tq, 2 * hq * d), np.float32)          # [Q | gate]
    qi[:, :hq * d] = q.reshape(tq, -1)
    qi[:, hq * d:] = 123.0
    kv = np.zeros((tk, 2 * hkv * d), np.float32)         # [K | V]
    kv[:, :hkv * d] = k.reshape(tk, -1)
    kv[:, hkv * d:] = v.reshape(tk, -1)
    rc, packed, _ = ORACLE.gqa(q, k, v, query_start=2, causal=True)
    v_view = kv.reshape(-1)[hkv * d:]
    rc2, strided, _ = ORACLE.gqa(qi, kv, np.ascontiguousarray(v_view), query_start=2, causal=True,
                                 q_stride=2 * hq * d, k_stride=2 * hkv * d,
                                 v_stride=2 * hkv * d, query_tokens=tq, kv_tokens=tk,
                                 query_heads=hq, kv_heads=hkv, head_dim=d)
    assert rc == rc2 == 0 and np.array_equal(packed, strided)
    rc3, *_ = ORACLE.gqa(qi, kv, kv, q_stride=hq * d - 1, query_tokens=tq, kv_tokens=tk,
                         query_heads=hq, kv_heads=hkv, head_dim=d)
    assert rc3 == -10                                             # stride below row width


def test_gqa_uniform_analytic():
    q, k, v = rv.uniform_large(65, 2)
    rc, out, lse = ORACLE.gqa(q, k, v, causal=False)
    assert rc == 0 and np.array_equal(out, v)
    assert np.allclose(lse, math.log(65), atol=1e-12)


def test_gqa_rows_equal_single_head_operator():
    rng = np.random.default_rng(6)
    q = rng.standard_normal((4, 8, 32)).astype(np.float32)
    k = rng.standard_normal((9, 2, 32)).astype(np.float32)
    v = rng.standard_normal((9, 2, 32)).astype(np.float32)
    rc, out, lse = ORACLE.gqa(q, k, v, query_start=5, causal=True)
    assert rc == 0
    scale = float(np.float32(1.0) / np.sqrt(np.float32(32)))
    for t in range(4):
        for h in range(8):
            rc1, o1, _, _, l1 = ORACLE.attention_head(q[t, h], k[:, h // 4], v[:, h // 4], 5 + t,
                                                     scale)
            assert rc1 == 0 and np.array_equal(o1, out[t, h]) and l1 == lse[t, h]


# ------------------------------------------------ paged decode (new surface) --

def _paged_case(rng, sessions, hq, hkv, d, page_tokens, contexts, q8=False, spare=3):
    need = [(c + page_tokens - 1) // page_tokens for c in contexts]
    pool_pages = sum(need) + spare
    perm = rng.permutation(pool_pages)
    table = np.full((sessions, max(need) + 1), -1, dtype=np.int32)
    at = 0
    for s, n in enumerate(need):
        table[s, :n] = perm[at:at + n]
        at += n
    kf = ORACLE.bf16_decode(ORACLE.bf16_encode(
        rng.standard_normal((pool_pages, page_tokens, hkv, d)).astype(np.float32)))
    vf = ORACLE.bf16_decode(ORACLE.bf16_encode(
        rng.standard_normal((pool_pages, page_tokens, hkv, d)).astype(np.float32)))
    q = ORACLE.bf16_encode(rng.standard_normal((sessions, hq, d)).astype(np.float32))
    if q8:
        kp, vp = ORACLE.q8_0_encode_rows(kf), ORACLE.q8_0_encode_rows(vf)
        kf, vf = ORACLE.q8_0_decode_rows(kp, d), ORACLE.q8_0_decode_rows(vp, d)
    else:
        kp, vp = ORACLE.bf16_encode(kf), ORACLE.bf16_encode(vf)
    return q, kp, vp, kf, vf, table, np.array(contexts, dtype=np.int32)


@pytest.mark.parametrize("q8", [False, True])
def test_paged_equals_contiguous_on_gathered_copy(q8):
    rng = np.random.default_rng(21)
    contexts = [1, 15, 16, 17, 100, 333]
    q, kp, vp, kf, vf, table, ctx = _paged_case(rng, 6, 8, 2, 64, 16, contexts, q8=q8)
    rc, out, outb, lse = ORACLE.paged_decode(q, kp, vp, table, ctx, 2, 16, q8=q8)
    assert rc == 0
    qf = ORACLE.bf16_decode(q)
    for s, n in enumerate(contexts):
        pages = table[s, :(n + 15) // 16]
        kc = kf[pages].reshape(-1, 2, 64)[:n]
        vc = vf[pages].reshape(-1, 2, 64)[:n]
        rc2, ref, lse2 = ORACLE.gqa(qf[s:s + 1], kc, vc, query_start=n - 1, causal=True)
        assert rc2 == 0
        assert np.array_equal(out[s], ref[0]) and np.array_equal(lse[s], lse2[0])
        assert np.array_equal(outb[s], ORACLE.bf16_encode(ref[0]))


def test_paged_placement_invariance_and_refusals():
    rng = np.random.default_rng(22)
    contexts = [40, 70]
    q, kp, vp, _, _, table, ctx = _paged_case(rng, 2, 4, 1, 32, 16, contexts)
    rc, out, _, lse = ORACLE.paged_decode(q, kp, vp, table, ctx, 1, 16)
    # move every page to a new slot and rewrite the table: same answer, bit for bit
    pool_pages = kp.shape[0]
    perm = rng.permutation(pool_pages)
    kp2, vp2 = np.empty_like(kp), np.empty_like(vp)
    kp2[perm], vp2[perm] = kp, vp
    table2 = np.where(table >= 0, perm[np.maximum(table, 0)], -1).astype(np.int32)
    rc2, out2, _, lse2 = ORACLE.paged_decode(q, kp2, vp2, table2, ctx, 1, 16)
    assert rc == rc2 == 0 and np.array_equal(out, out2) and np.array_equal(lse, lse2)
    # stale entries beyond the used pages are ignored
    table3 = table.copy()
    table3[0, 3:] = 10 ** 6
    rc3, out3, *_ = ORACLE.paged_decode(q, kp, vp, table3, ctx, 1, 16)
    assert rc3 == 0 and np.array_equal(out3, out)
    bad = table.copy()
    bad[1, 2] = pool_pages                                           # out of range
    assert ORACLE.paged_decode(q, kp, vp, bad, ctx, 1, 16)[0] == -7
    bad[1, 2] = -1
    assert ORACLE.paged_decode(q, kp, vp, bad, ctx, 1, 16)[0] == -7
    assert ORACLE.paged_decode(q, kp, vp, table, np.array([40, 0], np.int32), 1, 16)[0] == -10
    too_long = np.array([40, table.shape[1] * 16 + 1], np.int32)
    assert ORACLE.paged_decode(q, kp, vp, table, too_long, 1, 16)[0] == -7


# --------------------------------------------------- shared-KV / MLA / merge --

def test_shared_kv_sink_known_answer():
    kat = rv.SINK_KAT
    # logits are produced as q.row*scale with q = [1,0,...]: put the logit in a key-only lane
    rows = np.array([[kat["values"][0][0], kat["values"][0][1], kat["logits"][0]],
                     [kat["values"][1][0], kat["values"][1][1], kat["logits"][1]]], np.float32)
    q = np.array([0.0, 0.0, 1.0], np.float32)
    rc, out, lse = ORACLE.shared_kv_head(q, rows, 3, 2, 1.0, sink=kat["sink"])
    assert rc == 0 and np.allclose(out, kat["expected"], atol=1e-7)
    assert abs(lse - math.log(4.0)) < 1e-7                 # e^0 + e^0 + e^{ln 2}
    # a very negative sink is the reference's "no sink" (tests/unit/deepseek_attention.c:589-628)
    rc, out_lo, _ = ORACLE.shared_kv_head(q, rows, 3, 2, 1.0, sink=-100.0)
    rc2, out_no, _ = ORACLE.shared_kv_head(q, rows, 3, 2, 1.0, sink=None)
    assert rc == rc2 == 0 and np.allclose(out_lo, out_no, atol=1e-7)
    assert np.allclose(out_no, [(1 + 2 * 3) / 3, (2 + 2 * 4) / 3], atol=1e-6)


def test_shared_kv_without_sink_equals_plain_operator():
    rng = np.random.default_rng(31)
    n, kd, vd = 200, 48, 32
    rows = rng.standard_normal((n, kd)).astype(np.float32)
    q = rng.standard_normal(kd).astype(np.float32)
    scale = 1.0 / math.sqrt(kd)
    rc, out, lse = ORACLE.shared_kv_head(q, rows, kd, vd, scale)
    # plain operator on K = rows, V = first vd lanes (zero-pad V to kd lanes for the shape rule)
    rc2, ref, _, _, lse2 = ORACLE.attention_head(q, rows, rows, n - 1, np.float32(scale))
    assert rc == rc2 == 0
    assert np.allclose(out, ref[:vd], atol=2e-6) and abs(lse - lse2) < 1e-6
    # output is a convex combination of the latent rows
    assert np.all(out <= rows[:, :vd].max(axis=0) + 1e-6)
    assert np.all(out >= rows[:, :vd].min(axis=0) - 1e-6)


def test_mla_paged_equals_per_head_shared_kv():
    rng = np.random.default_rng(32)
    batch, heads, kd, vd, pt = 3, 5, 96, 64, 8
    contexts = [5, 8, 29]
    need = [(c + pt - 1) // pt for c in contexts]
    pool_pages = sum(need) + 2
    perm = rng.permutation(pool_pages)
    table = np.zeros((batch, max(need)), np.int32)
    at = 0
    for b, n in enumerate(need):
        table[b, :n] = perm[at:at + n]
        at += n
    pool = ORACLE.bf16_encode(rng.standard_normal((pool_pages, pt, kd)).astype(np.float32))
    q = ORACLE.bf16_encode(rng.standard_normal((batch, heads, kd)).astype(np.float32))
    rc, out, outb, lse = ORACLE.mla_decode(q, pool, table, np.array(contexts, np.int32), vd, pt)
    assert rc == 0
    pf, qf = ORACLE.bf16_decode(pool), ORACLE.bf16_decode(q)
    for b, n in enumerate(contexts):
        rows = pf[table[b, :need[b]]].reshape(-1, kd)[:n]
        for h in range(heads):
            rc1, o1, l1 = ORACLE.shared_kv_head(qf[b, h], rows, kd, vd, 1.0 / math.sqrt(kd))
            assert rc1 == 0 and np.array_equal(o1, out[b, h]) and l1 == lse[b, h]
    assert np.array_equal(outb, ORACLE.bf16_encode(out))


def test_lse_merge_is_associative_with_single_pass():
    rng = np.random.default_rng(33)
    n, d = 1000, 32
    q = rng.standard_normal(d).astype(np.float32)
    k = rng.standard_normal((n, d)).astype(np.float32)
    v = rng.standard_normal((n, d)).astype(np.float32)
    scale = 0.2
    rc, full, _, _, full_lse = ORACLE.attention_head(q, k, v, n - 1, scale)
    for cuts in ([0, 1000], [0, 1, 1000], [0, 137, 512, 999, 1000], list(range(0, 1001, 50))):
        outs, lses = [], []
        for a, b in zip(cuts[:-1], cuts[1:]):
            rc1, o, _, _, l = ORACLE.attention_head(q, k[a:b], v[a:b], b - a - 1, scale)
            assert rc1 == 0
            outs.append(o)
            lses.append(l)
        rc2, merged, merged_lse = ORACLE.lse_merge(np.array(outs), np.array(lses))
        assert rc2 == 0 and np.allclose(merged, full, atol=1e-6)
        assert abs(merged_lse - full_lse) < 1e-6
    # uniform scores: LSE = s + ln n
    rc, _, _, _, lse = ORACLE.attention_head(np.zeros(d, np.float32), k, v, n - 1, scale)
    assert abs(lse - math.log(n)) < 1e-12
    # an empty part (lse = -inf) does not contribute
    rc, merged, merged_lse = ORACLE.lse_merge(np.array([full, np.zeros(d, np.float32)]),
                                              np.array([full_lse, -np.inf]))
    assert rc == 0 and np.allclose(merged, full, atol=1e-7) and abs(merged_lse - full_lse) < 1e-12


# ------------------------------------------------------------- rotary -------

def test_rotary_reference_known_answer():
    """tests/unit/cuda/quant_qtype.c:1988-2061: products staged through bf16, the sum
    rounded again, the non-rotary suffix untouched.  The literals are those products worked
    by hand: -1.34375*0.63671875 -> -0.85546875, -2.0625*0.546875 -> -1.125, and so on."""
    values = ORACLE.bf16_encode(np.array([[[-1.34375, -2.0625, 3.0, 4.0]]], np.float32))
    cosines = np.full((1, 2), 0.63671875, np.float32)
    sines = np.full((1, 2), 0.546875, np.float32)
    got = ORACLE.bf16_decode(ORACLE.rotary_half_bf16(values, cosines, sines, 2))
    assert got.tolist() == [[[0.26953125, -2.046875, 3.0, 4.0]]]


def test_rotary_closed_forms():
    rng = np.random.default_rng(44)
    tokens, heads, d = 5, 3, 128
    x = ORACLE.bf16_encode(rng.standard_normal((tokens, heads, d)).astype(np.float32))
    xf = ORACLE.bf16_decode(x)
    for rotary in (32, 64, 128):
        half = rotary // 2
        one, zero = np.ones((tokens, rotary), np.float32), np.zeros((tokens, rotary), np.float32)
        assert np.array_equal(ORACLE.rotary_half_bf16(x, one, zero, rotary), x)
        quarter = ORACLE.bf16_decode(ORACLE.rotary_half_bf16(x, zero, one, rotary))
        assert np.array_equal(quarter[..., :half], -xf[..., half:rotary])
        assert np.array_equal(quarter[..., half:rotary], xf[..., :half])
        assert np.array_equal(quarter[..., rotary:], xf[..., rotary:])
        # per-token angles: float64 rotation within bf16 rounding, norms kept; the second
        # half of each table row is never read
        angles = rng.uniform(-3.0, 3.0, (tokens, rotary))
        angles[:, half:] = np.nan
        cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
        got = ORACLE.bf16_decode(ORACLE.rotary_half_bf16(x, cosines, sines, rotary)).astype(np.float64)
        c, s = np.cos(angles[:, None, :half]), np.sin(angles[:, None, :half])
        a, b = xf[..., :half].astype(np.float64), xf[..., half:rotary].astype(np.float64)
        want = np.concatenate([a * c - b * s, b * c + a * s, xf[..., rotary:]], axis=-1)
        assert np.all(np.isfinite(got))
        assert np.max(np.abs(got - want)) < 3 * 2.0 ** -8 * np.max(np.abs(xf))
        assert np.allclose(np.linalg.norm(got, axis=-1), np.linalg.norm(xf, axis=-1), rtol=5e-3)


def test_rotary_f32_pins():
    """The F32 form: the reference's known-answer case on its own literals
    (tests/unit/cuda/quant_qtype.c:1988-2061), bit equality with the bf16 form where the
    inputs are representable, and closed forms where they are not."""
    values = np.array([[[-1.34375, -2.0625, 3.0, 4.0]]], np.float32)
    cosines, sines = np.full((1, 2), 0.63671875, np.float32), np.full((1, 2), 0.546875, np.float32)
    assert ORACLE.rotary_half_f32(values, cosines, sines, 2).tolist() == [[[0.26953125, -2.046875, 3.0, 4.0]]]
    rng = np.random.default_rng(45)
    tokens, heads, d = 4, 3, 64
    x = rng.standard_normal((tokens, heads, d)).astype(np.float32)
    xb = ORACLE.bf16_encode(x)
    for rotary in (16, 32, 64):
        half = rotary // 2
        angles = rng.uniform(-3.0, 3.0, (tokens, rotary))
        cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
        representable = ORACLE.bf16_decode(xb)
        assert np.array_equal(ORACLE.rotary_half_f32(representable, cosines, sines, rotary),
                              ORACLE.bf16_decode(ORACLE.rotary_half_bf16(xb, cosines, sines, rotary)))
        one, zero = np.ones((tokens, rotary), np.float32), np.zeros((tokens, rotary), np.float32)
        same = ORACLE.rotary_half_f32(x, one, zero, rotary)
        assert np.array_equal(same[..., :rotary], representable[..., :rotary])   # rounded once
        assert np.array_equal(same[..., rotary:], x[..., rotary:])               # suffix untouched
        quarter = ORACLE.rotary_half_f32(x, zero, one, rotary)
        assert np.array_equal(quarter[..., :half], -representable[..., half:rotary])
        assert np.array_equal(quarter[..., half:rotary], representable[..., :half])


def test_rotary_rounded_pins():
    """The decoder's order: plain F32 rotation, then one bf16 rounding of every lane.  The
    reference's known-answer case (tests/unit/cuda/quant_qtype.c:3050-3105: two heads of
    width 2, cos 0.75, sin 0.5) is exact in float and in bf16."""
    values = np.array([[[1.0, 2.0], [7.0, 8.0]]], np.float32)
    cosines, sines = np.full((1, 2), 0.75, np.float32), np.full((1, 2), 0.5, np.float32)
    assert ORACLE.rotary_half_f32_rounded(values, cosines, sines, 2).tolist() == \
        [[[-0.25, 2.0], [1.25, 9.5]]]
    rng = np.random.default_rng(46)
    tokens, heads, d = 6, 2, 64
    x = rng.standard_normal((tokens, heads, d)).astype(np.float32)
    rounded = ORACLE.bf16_decode(ORACLE.bf16_encode(x))
    for rotary in (16, 32, 64):
        half = rotary // 2
        one, zero = np.ones((tokens, rotary), np.float32), np.zeros((tokens, rotary), np.float32)
        assert np.array_equal(ORACLE.rotary_half_f32_rounded(x, one, zero, rotary), rounded)
        quarter = ORACLE.rotary_half_f32_rounded(x, zero, one, rotary)
        assert np.array_equal(quarter[..., :half], -rounded[..., half:rotary])
        assert np.array_equal(quarter[..., half:rotary], rounded[..., :half])
        assert np.array_equal(quarter[..., rotary:], rounded[..., rotary:])       # suffix rounded too
        angles = rng.uniform(-3.0, 3.0, (tokens, rotary))
        cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
        got = ORACLE.rotary_half_f32_rounded(x, cosines, sines, rotary)
        c = cosines[:, None, :half].astype(np.float64)
        s = sines[:, None, :half].astype(np.float64)
        a, b = x[..., :half].astype(np.float64), x[..., half:rotary].astype(np.float64)
        exact = np.concatenate([a * c - b * s, b * c + a * s, x[..., rotary:]], axis=-1)
        # one rounding to bf16 of a value that carries at most a float rounding or two
        step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 1e-30))) - 7)
        assert np.all(np.abs(got - exact) <= 0.5 * step * (1 + 2.0 ** -14) + 1e-12)
        assert np.array_equal(ORACLE.bf16_decode(ORACLE.bf16_encode(got)), got)
        # Against the expression as the reference's source writes it, every product and sum
        # rounded to float on its own (src/backend/cuda/transformer_kernels.cu:110-134): which
        # product the reference's compiler fuses is not visible in its sources, so this is the
        # part of the function whose last bit is "parity unpinned".  A fused and an unfused
        # evaluation differ by a float rounding before the bf16 rounding: equal bf16 results
        # but for values next to a bf16 tie, and then one bf16 step apart.
        cf, sf = cosines[:, None, :half], sines[:, None, :half]
        af, bf = x[..., :half], x[..., half:rotary]
        plain = np.concatenate([(af * cf).astype(np.float32) - (bf * sf).astype(np.float32),
                                (bf * cf).astype(np.float32) + (af * sf).astype(np.float32),
                                x[..., rotary:]], axis=-1).astype(np.float32)
        plain = ORACLE.bf16_decode(ORACLE.bf16_encode(plain))
        differing = plain != got
        assert np.count_nonzero(differing) <= got.size // 100
        assert np.all(np.abs(plain - got)[differing] <= step[differing] * (1 + 2.0 ** -14))
        # the staged form rounds three times: the two agree within a few bf16 steps of the inputs
        staged = ORACLE.rotary_half_f32(x, cosines, sines, rotary)
        assert np.max(np.abs(staged - got)[..., :rotary]) <= 3 * 2.0 ** -8 * np.max(np.abs(x))


def test_rotary_plain_pins():
    """The rotation alone (what the rotary_half_f32 operator slot runs): the reference's
    known-answer case (tests/unit/cuda/quant_qtype.c:3050-3105), identity, quarter turn, a
    float64 rotation within two float roundings, the unfused expression within one float
    rounding, and the rounded form as this one followed by the bf16 rounding."""
    values = np.array([[[1.0, 2.0], [7.0, 8.0]]], np.float32)
    cosines, sines = np.full((1, 2), 0.75, np.float32), np.full((1, 2), 0.5, np.float32)
    assert ORACLE.rotary_half_plain_f32(values, cosines, sines, 2).tolist() == \
        [[[-0.25, 2.0], [1.25, 9.5]]]
    rng = np.random.default_rng(47)
    tokens, heads, d = 5, 3, 64
    x = rng.standard_normal((tokens, heads, d)).astype(np.float32)
    for rotary in (2, 16, 64):
        half = rotary // 2
        one, zero = np.ones((tokens, rotary), np.float32), np.zeros((tokens, rotary), np.float32)
        assert np.array_equal(ORACLE.rotary_half_plain_f32(x, one, zero, rotary), x)
        quarter = ORACLE.rotary_half_plain_f32(x, zero, one, rotary)
        assert np.array_equal(quarter[..., :half], -x[..., half:rotary])
        assert np.array_equal(quarter[..., half:rotary], x[..., :half])
        assert np.array_equal(quarter[..., rotary:], x[..., rotary:])
        angles = rng.uniform(-3.0, 3.0, (tokens, rotary))
        cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
        got = ORACLE.rotary_half_plain_f32(x, cosines, sines, rotary)
        c, s = cosines[:, None, :half].astype(np.float64), sines[:, None, :half].astype(np.float64)
        a, b = x[..., :half].astype(np.float64), x[..., half:rotary].astype(np.float64)
        exact = np.concatenate([a * c - b * s, b * c + a * s, x[..., rotary:]], axis=-1)
        scale = np.concatenate([np.abs(a * c) + np.abs(b * s), np.abs(b * c) + np.abs(a * s),
                                np.zeros_like(x[..., rotary:], np.float64)], axis=-1)
        assert np.all(np.abs(got - exact) <= 2.0 ** -23 * scale)
        cf, sf = cosines[:, None, :half], sines[:, None, :half]
        af, bf = x[..., :half], x[..., half:rotary]
        unfused = np.concatenate([(af * cf).astype(np.float32) - (bf * sf).astype(np.float32),
                                  (bf * cf).astype(np.float32) + (af * sf).astype(np.float32),
                                  x[..., rotary:]], axis=-1).astype(np.float32)
        assert np.all(np.abs(unfused.astype(np.float64) - got) <= 2.0 ** -23 * scale)
        assert np.array_equal(ORACLE.bf16_decode(ORACLE.bf16_encode(got)),
                              ORACLE.rotary_half_f32_rounded(x, cosines, sines, rotary))


# -------------------------------------------------------- output gate -------

def test_sigmoid_gate_reference_known_answer():
    """tests/unit/cuda/quant_qtype.c:2979-2981,3019-3033.  sigmoid(0) = 1/2, sigmoid(+-ln 3)
    = 3/4 and 1/4, sigmoid(1) = 0.7310586: 4 * 0.7310586 = 2.9242 rounds to 2.921875 in bf16."""
    values = np.array([1.0, -2.0, 0.5, 4.0], np.float32)
    gates = np.array([0.0, 1.0986122886681098, -1.0986122886681098, 1.0], np.float32)
    assert ORACLE.sigmoid_gate_bf16(values, gates).tolist() == [0.5, -1.5, 0.125, 2.921875]


def test_sigmoid_gate_closed_forms():
    rng = np.random.default_rng(55)
    values = ORACLE.bf16_decode(ORACLE.bf16_encode(rng.standard_normal(4096).astype(np.float32)))
    assert np.array_equal(ORACLE.sigmoid_gate_bf16(values, np.full(4096, 40.0)), values)
    assert np.all(ORACLE.sigmoid_gate_bf16(values, np.full(4096, -200.0)) == 0.0)
    half = ORACLE.sigmoid_gate_bf16(values, np.zeros(4096))
    assert np.array_equal(half, values * 0.5)              # exact: a power-of-two scale
    gates = rng.uniform(-8.0, 8.0, 4096).astype(np.float32)
    want = values.astype(np.float64) / (1.0 + np.exp(-gates.astype(np.float64)))
    got = ORACLE.sigmoid_gate_bf16(values, gates)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) <= 2.0 ** -8
    # symmetry sigmoid(g) + sigmoid(-g) = 1 on a value whose products are exact in bf16
    plus, minus = ORACLE.sigmoid_gate_bf16(np.ones(4096), gates), ORACLE.sigmoid_gate_bf16(np.ones(4096), -gates)
    assert np.max(np.abs(plus + minus - 1.0)) <= 2.0 ** -8


# ------------------------------------------- MLA sink and sliding window ----

def _mla_case(rng, contexts, heads=4, kd=64, vd=48, pt=16):
    need = [(c + pt - 1) // pt for c in contexts]
    pool_pages = sum(need) + 1
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((len(contexts), max(need)), np.int32)
    at = 0
    for b, n in enumerate(need):
        table[b, :n] = perm[at:at + n]
        at += n
    pool = ORACLE.bf16_encode(rng.standard_normal((pool_pages, pt, kd)).astype(np.float32))
    q = ORACLE.bf16_encode(rng.standard_normal((len(contexts), heads, kd)).astype(np.float32))
    return q, pool, table, np.array(contexts, np.int32), vd, pt


def test_mla_sink_is_one_more_logit_with_a_zero_row():
    """With a sink s: out = out0 * e^lse0 / (e^lse0 + e^s) and lse = log(e^lse0 + e^s), where
    (out0, lse0) is the result without it (softmax over one more logit whose value is 0)."""
    rng = np.random.default_rng(66)
    q, pool, table, ctx, vd, pt = _mla_case(rng, [1, 5, 40, 333])
    sinks = np.array([-3.0, 0.0, 1.5, 9.0], np.float32)
    rc0, out0, _, lse0 = ORACLE.mla_decode(q, pool, table, ctx, vd, pt)
    rc1, out1, _, lse1 = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, sinks=sinks)
    assert rc0 == 0 and rc1 == 0
    keep = 1.0 / (1.0 + np.exp(sinks[None, :].astype(np.float64) - lse0))
    assert np.allclose(out1, out0 * keep[..., None], rtol=1e-5, atol=1e-7)
    assert np.allclose(lse1, np.logaddexp(lse0, sinks[None, :]), atol=1e-9)
    rc, _, _, _ = ORACLE.mla_decode(q, pool, table, ctx, vd, pt,
                                    sinks=np.array([0, np.inf, 0, 0], np.float32))
    assert rc != 0                                         # a non-finite sink is refused


@pytest.mark.parametrize("window", [1, 7, 16, 100, 10 ** 6])
def test_mla_sliding_window_equals_decode_on_the_trimmed_context(window):
    rng = np.random.default_rng(67)
    contexts = [1, 16, 17, 90, 257]
    q, pool, table, ctx, vd, pt = _mla_case(rng, contexts)
    rc, out, outb, lse = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, sliding_window=window)
    assert rc == 0
    for b, n in enumerate(contexts):
        first = max(0, n - window)
        rows = pool[table[b, :(n + pt - 1) // pt]].reshape(-1, pool.shape[-1])[first:n]
        live = n - first
        pages = (live + pt - 1) // pt
        trimmed = np.zeros((pages, pt, pool.shape[-1]), np.uint16)
        trimmed.reshape(-1, pool.shape[-1])[:live] = rows
        rc1, out1, outb1, lse1 = ORACLE.mla_decode(
            q[b:b + 1], trimmed, np.arange(pages, dtype=np.int32)[None, :],
            np.array([live], np.int32), vd, pt)
        assert rc1 == 0
        assert np.array_equal(out1[0], out[b]) and np.array_equal(lse1[0], lse[b])


def test_mla_compressed_rows_join_the_same_softmax_after_the_local_rows():
    """Local window rows then the visible compressed prefix == one context holding those rows in
    that order, bit for bit; an empty compressed set changes nothing."""
    rng = np.random.default_rng(68)
    contexts, counts, window = [3, 40, 130], [0, 5, 33], 32
    q, pool, table, ctx, vd, pt = _mla_case(rng, contexts)
    _, cpool, ctable, ccount, _, _ = _mla_case(rng, [max(c, 1) for c in counts])
    ccount = np.array(counts, np.int32)
    sinks = np.array([0.5, -1.0, 2.0, 0.0], np.float32)
    rc, out, _, lse = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, sinks=sinks,
                                        sliding_window=window, compressed=(cpool, ctable, ccount))
    assert rc == 0
    kd = pool.shape[-1]
    for b, n in enumerate(contexts):
        first = max(0, n - window)
        rows = np.concatenate([
            pool[table[b, :(n + pt - 1) // pt]].reshape(-1, kd)[first:n],
            cpool[ctable[b, :(counts[b] + pt - 1) // pt]].reshape(-1, kd)[:counts[b]]])
        pages = (len(rows) + pt - 1) // pt
        joined = np.zeros((pages, pt, kd), np.uint16)
        joined.reshape(-1, kd)[:len(rows)] = rows
        rc1, out1, _, lse1 = ORACLE.mla_decode(q[b:b + 1], joined, np.arange(pages, dtype=np.int32)[None, :],
                                               np.array([len(rows)], np.int32), vd, pt, sinks=sinks)
        assert rc1 == 0 and np.array_equal(out1[0], out[b]) and np.array_equal(lse1[0], lse[b])
    rc2, out2, _, lse2 = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, sinks=sinks, sliding_window=window,
                                           compressed=(cpool, ctable, np.zeros(3, np.int32)))
    rc3, out3, _, lse3 = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, sinks=sinks, sliding_window=window)
    assert rc2 == 0 and rc3 == 0 and np.array_equal(out2, out3) and np.array_equal(lse2, lse3)


def test_mla_selected_rows_are_the_listed_rows_in_list_order():
    """The identity list equals the prefix class bit for bit; an arbitrary list (repeats
    allowed) equals one context holding the local rows then the listed rows."""
    rng = np.random.default_rng(69)
    contexts, stored = [20, 130], [40, 90]
    q, pool, table, ctx, vd, pt = _mla_case(rng, contexts)
    _, cpool, ctable, _, _, _ = _mla_case(rng, stored)
    kd = pool.shape[-1]
    counts = np.array([7, 33], np.int32)
    identity = np.tile(np.arange(40, dtype=np.int32), (2, 1))
    a = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, compressed=(cpool, ctable, counts))
    b = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, compressed=(cpool, ctable, counts), selected=identity)
    assert a[0] == 0 and b[0] == 0 and np.array_equal(a[1], b[1]) and np.array_equal(a[3], b[3])
    lists = np.stack([rng.integers(0, stored[i], 40) for i in range(2)]).astype(np.int32)
    rc, out, _, lse = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, compressed=(cpool, ctable, counts),
                                        selected=lists)
    assert rc == 0
    for i, n in enumerate(contexts):
        local = pool[table[i, :(n + pt - 1) // pt]].reshape(-1, kd)[:n]
        stored_rows = cpool[ctable[i, :(stored[i] + pt - 1) // pt]].reshape(-1, kd)
        rows = np.concatenate([local, stored_rows[lists[i, :counts[i]]]])
        pages = (len(rows) + pt - 1) // pt
        joined = np.zeros((pages, pt, kd), np.uint16)
        joined.reshape(-1, kd)[:len(rows)] = rows
        rc1, out1, _, lse1 = ORACLE.mla_decode(q[i:i + 1], joined, np.arange(pages, dtype=np.int32)[None, :],
                                               np.array([len(rows)], np.int32), vd, pt)
        assert rc1 == 0 and np.array_equal(out1[0], out[i]) and np.array_equal(lse1[0], lse[i])
    bad = lists.copy()
    bad[1, 3] = 10 ** 6
    assert ORACLE.mla_decode(q, pool, table, ctx, vd, pt, compressed=(cpool, ctable, counts),
                             selected=bad)[0] != 0


# ------------------------- the shared-KV oracle against the compiled reference reduce ----

def _reference_tail(row_bf16, position, theta=10000):
    """What the reference does to a published row after the softmax (src/graph/core.c:499-507)
    when it is run with two rope lanes: the last two lanes rotated back by the token position,
    then rounded to bf16 again."""
    rc, out = ORACLE.reduce_output_finish(row_bf16[None, :], position,
                                          ORACLE.position_policy(2, theta=theta))
    assert rc == 0
    return out[0]


@needs_ref_reduce
@pytest.mark.parametrize("attention_class,window,contexts", [
    (0, 10 ** 6, [1, 2, 17, 300]), (0, 16, [1, 16, 17, 90]), (0, 1, [5]),
    (2, 64, [1, 127, 128, 129, 700]), (2, 10 ** 6, [255, 256, 1000]),
])
def test_mla_oracle_matches_compiled_reference_reduce(attention_class, window, contexts):
    """Sink logits, the sliding-window filter and the dense compressed class of
    yvo_mla_decode_bf16 (paged rows, key_dim == value_dim as in the reference) against
    yvex_attention_reduce_chunk compiled from the reference sources: every lane the reference
    does not rotate is bit-identical, and so are the two it rotates once the same rotation
    is applied."""
    rng = np.random.default_rng(71 + attention_class + window % 97)
    heads, d, pt, ratio = 4, 64, 16, 128
    q, pool, table, ctx, _, _ = _mla_case(rng, contexts, heads=heads, kd=d, vd=d, pt=pt)
    stored = [n // ratio + 2 for n in contexts]                      # two not yet visible
    _, cpool, ctable, _, _, _ = _mla_case(rng, stored, heads=heads, kd=d, vd=d, pt=pt)
    visible = np.array([n // ratio for n in contexts], np.int32) if attention_class == 2 \
        else np.zeros(len(contexts), np.int32)
    sinks = (rng.standard_normal(heads) * 2.0).astype(np.float32)
    rc, out, _, _ = ORACLE.mla_decode(q, pool, table, ctx, d, pt, sinks=sinks, sliding_window=window,
                                      compressed=(cpool, ctable, visible) if attention_class == 2 else None)
    assert rc == 0
    for b, n in enumerate(contexts):
        local = ORACLE.bf16_decode(pool[table[b, :(n + pt - 1) // pt]].reshape(-1, d)[:n])
        comp = ORACLE.bf16_decode(cpool[ctable[b, :(stored[b] + pt - 1) // pt]].reshape(-1, d)[:stored[b]])
        rc1, ref = reference_reduce(
            REF_REDUCE, ORACLE.bf16_decode(q[b]), local, np.arange(n), comp if attention_class == 2 else
            np.zeros((0, d), np.float32), np.arange(stored[b]) * ratio if attention_class == 2 else [],
            sinks, window, ratio if attention_class == 2 else 0, attention_class, n - 1)
        assert rc1 == 0
        mine = ORACLE.bf16_decode(ORACLE.bf16_encode(out[b]))
        assert np.array_equal(mine[:, :-2], ref[:, :-2]), (attention_class, window, n)
        for h in range(heads):
            assert np.array_equal(_reference_tail(mine[h], n - 1)[-2:], ref[h, -2:])


@needs_ref_reduce
def test_no_sink_equals_a_sink_that_underflows():
    """The reference always has a sink; the oracle's sink-free path equals a sink so negative
    that exp() of it is zero, which is how the sink-free configurations are tied to it."""
    rng = np.random.default_rng(72)
    q, pool, table, ctx, vd, pt = _mla_case(rng, [1, 40, 333])
    a = ORACLE.mla_decode(q, pool, table, ctx, vd, pt)
    b = ORACLE.mla_decode(q, pool, table, ctx, vd, pt, sinks=np.full(4, -1e30, np.float32))
    assert a[0] == 0 and b[0] == 0 and np.array_equal(a[1], b[1]) and np.array_equal(a[3], b[3])


# ------------------------------------------ the output rotation of the shared-KV reduce ----

ROPE_POLICIES = [
    dict(rope_dims=64, theta=10000),
    dict(rope_dims=64, theta=10000, scaling_factor=40, original_context=4096, beta_fast=32, beta_slow=1),
    dict(rope_dims=32, theta=500000, scaling_factor=8, original_context=8192, beta_fast=32, beta_slow=1),
    dict(rope_dims=2, theta=10000),
]


@needs_ref_reduce
@pytest.mark.parametrize("policy", ROPE_POLICIES, ids=["plain64", "yarn64", "yarn32", "plain2"])
@pytest.mark.parametrize("dim", [64, 128])
def test_reduce_output_finish_matches_compiled_reference_reduce(policy, dim):
    """yvo_reduce_output_finish (bf16 round, inverse rotation of the rope lanes with the
    reference's frequency rule, bf16 round) after yvo_mla_decode_bf16 against the published
    rows of yvex_attention_reduce_chunk compiled from the reference sources, every lane, bit
    for bit; positions up to 20000 so that the angle reduction matters."""
    rng = np.random.default_rng(91 + dim + policy["rope_dims"])
    heads, pt = 4, 16
    contexts = [1, 2, 77, 300, 1500]
    q, pool, table, ctx, _, _ = _mla_case(rng, contexts, heads=heads, kd=dim, vd=dim, pt=pt)
    sinks = (rng.standard_normal(heads) * 2.0).astype(np.float32)
    rc, out, _, _ = ORACLE.mla_decode(q, pool, table, ctx, dim, pt, sinks=sinks)
    assert rc == 0
    for b, n in enumerate(contexts):
        local = ORACLE.bf16_decode(pool[table[b, :(n + pt - 1) // pt]].reshape(-1, dim)[:n])
        # the reference takes the token position separately from the rows' positions: a large
        # offset exercises the rotation at long-context angles with a short history
        offset = [0, 20000][b % 2]
        rc1, ref = reference_reduce(REF_REDUCE, ORACLE.bf16_decode(q[b]), local,
                                    np.arange(n) + offset, np.zeros((0, dim), np.float32), [],
                                    sinks, 10 ** 6, 0, 0, n - 1 + offset, **policy)
        assert rc1 == 0
        rc2, mine = ORACLE.reduce_output_finish(out[b], n - 1 + offset,
                                                ORACLE.position_policy(**policy))
        assert rc2 == 0
        assert np.array_equal(mine.view(np.uint32), ref.view(np.uint32)), (policy, dim, n)


def test_yarn_frequency_closed_forms():
    """Without scaling the frequency of pair i is theta^(-2i/dims) (pair 0: exactly 1).  With
    the YaRN ramp the pairs below the low corner keep that frequency and the pairs above the
    high corner have it divided by the factor (src/graph/numeric.c:888-915)."""
    plain = ORACLE.position_policy(64, theta=10000)
    f = [ORACLE.lib.yvo_yarn_frequency(C.byref(plain), i, 64) for i in range(32)]
    assert f[0] == 1.0
    assert np.allclose(f, 10000.0 ** (-np.arange(32) * 2 / 64), rtol=1e-15)
    yarn = ORACLE.position_policy(64, theta=10000, scaling_factor=40, original_context=4096,
                                  beta_fast=32, beta_slow=1)
    g = [ORACLE.lib.yvo_yarn_frequency(C.byref(yarn), i, 64) for i in range(32)]
    low = math.floor(64 * math.log(4096 / (32 * 2 * math.pi)) / (2 * math.log(10000)))
    high = math.ceil(64 * math.log(4096 / (1 * 2 * math.pi)) / (2 * math.log(10000)))
    assert 0 < low < high < 31
    for i in range(32):
        if i <= low:
            assert g[i] == f[i]
        elif i >= high:
            assert math.isclose(g[i], f[i] / 40, rel_tol=1e-15)
        else:
            assert f[i] / 40 < g[i] < f[i]
    assert all(a > b for a, b in zip(g, g[1:]))          # still strictly decreasing


def test_rope_apply_properties():
    rng = np.random.default_rng(92)
    policy = ORACLE.position_policy(64, theta=10000, scaling_factor=40, original_context=4096,
                                    beta_fast=32, beta_slow=1)
    row = rng.standard_normal(128).astype(np.float32)
    rc, same = ORACLE.rope_apply(row, 0, policy)                      # position 0: identity
    assert rc == 0 and np.array_equal(same, row)
    rc, turned = ORACLE.rope_apply(row, 4321, policy)
    assert rc == 0 and np.array_equal(turned[:64], row[:64])          # only the last 64 lanes move
    assert not np.array_equal(turned[64:], row[64:])
    pairs = turned[64:].reshape(-1, 2).astype(np.float64)
    assert np.allclose((pairs ** 2).sum(1), (row[64:].reshape(-1, 2).astype(np.float64) ** 2).sum(1),
                       rtol=1e-6)                                      # a rotation keeps pair norms
    rc, back = ORACLE.rope_apply(turned, 4321, policy, inverse=True)
    assert rc == 0 and np.allclose(back, row, atol=1e-6)
    # pair 0 turns by exactly `position` radians (frequency 1)
    rc, unit = ORACLE.rope_apply(np.array([1.0, 0.0], np.float32), 3, ORACLE.position_policy(2))
    assert rc == 0 and np.allclose(unit, [math.cos(3.0), math.sin(3.0)], atol=1e-7)
    # refusals of the reference (numeric.c:930-932): theta <= 1, more rope lanes than lanes
    assert ORACLE.rope_apply(row, 1, ORACLE.position_policy(64, theta=1))[0] != 0
    assert ORACLE.rope_apply(row[:32], 1, ORACLE.position_policy(64))[0] != 0
