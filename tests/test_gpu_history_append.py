"""GPU parity: the token-major history writer (new K/V rows into the reference's [K | V]
history layout, rotary on the keys) against the CPU restatement, bit for bit, through the C
ABI; then a history in a reserved address range that is committed, appended to and decoded
over step by step, the way the reference's caller grows it
(src/runtime/stateful_attention.c:183-222, src/runtime/state_residency.c:258-287)."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu


def tables(rng, tokens, rotary_dim):
    angles = rng.uniform(-3.0, 3.0, size=(tokens, max(rotary_dim, 16))).astype(np.float32)
    return np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)


@pytest.mark.parametrize("tokens,first,hkv,d,rotary,interleaved", [
    (1, 0, 8, 128, 128, True),        # the first token of a sequence
    (1, 4095, 8, 128, 64, True),      # one decode step behind a long history
    (37, 100, 8, 128, 64, True),      # a prompt chunk, partial rotary
    (300, 7, 2, 128, 0, True),        # no rotary: plain rows
    (19, 5, 4, 64, 32, True),         # other head widths
    (6, 9, 2, 256, 256, False),       # separate packed K and V histories
    (23, 0, 1, 128, 16, False),
])
def test_history_append_matches_oracle_bit_for_bit(backend, tokens, first, hkv, d, rotary, interleaved):
    rng = np.random.default_rng(tokens * 1000 + first + d)
    width = hkv * d
    rows = first + tokens + 3                                   # three rows behind stay untouched
    k_new, v_new = bf16_normal(rng, (tokens, hkv, d)), bf16_normal(rng, (tokens, hkv, d))
    cosine, sine = tables(rng, tokens, rotary)
    tk = backend.tensor("k-new", B.DTYPE_BF16, k_new.shape, k_new)
    tv = backend.tensor("v-new", B.DTYPE_BF16, v_new.shape, v_new)
    tc = backend.tensor("cos", B.DTYPE_F32, (tokens, max(rotary, 1)), cosine[:, :max(rotary, 1)])
    ts = backend.tensor("sin", B.DTYPE_F32, (tokens, max(rotary, 1)), sine[:, :max(rotary, 1)])
    want_k = ORACLE.rotary_half_bf16(k_new, cosine[:, :rotary], sine[:, :rotary], rotary) \
        if rotary else k_new
    used = first + tokens
    if interleaved:
        before = bf16_normal(rng, (rows, 2 * width))
        store = backend.tensor("history", B.DTYPE_BF16, before.shape, before)
        count = (used - 1) * 2 * width + width
        kh, vh = store.view(0, B.DTYPE_BF16, (count,)), store.view(2 * width, B.DTYPE_BF16, (count,))
        facts = backend.history_append_execute(
            tk, tv, kh, vh, first, hkv, head_dimension=d, cosine=tc if rotary else None,
            sine=ts if rotary else None, rotary_dimension=rotary, key_token_stride=2 * width,
            value_token_stride=2 * width)
        want = before.copy()
        want[first:used, :width] = want_k.reshape(tokens, width)
        want[first:used, width:] = v_new.reshape(tokens, width)
        assert np.array_equal(store.read(), want)
        stores = [store]
    else:
        before_k, before_v = bf16_normal(rng, (rows, width)), bf16_normal(rng, (rows, width))
        sk = backend.tensor("k-history", B.DTYPE_BF16, before_k.shape, before_k)
        sv = backend.tensor("v-history", B.DTYPE_BF16, before_v.shape, before_v)
        kh, vh = sk.view(0, B.DTYPE_BF16, (used * width,)), sv.view(0, B.DTYPE_BF16, (used * width,))
        facts = backend.history_append_execute(
            tk, tv, kh, vh, first, hkv, head_dimension=d, cosine=tc if rotary else None,
            sine=ts if rotary else None, rotary_dimension=rotary)
        want_kh, want_vh = before_k.copy(), before_v.copy()
        want_kh[first:used] = want_k.reshape(tokens, width)
        want_vh[first:used] = v_new.reshape(tokens, width)
        assert np.array_equal(sk.read(), want_kh) and np.array_equal(sv.read(), want_vh)
        stores = [sk, sv]
    assert facts.kernel_launches == 1 and facts.device_synchronizations == 1
    for tensor in stores + [tk, tv, tc, ts]:
        tensor.release()


def test_history_append_refuses_values_that_are_not_finite(backend):
    rng = np.random.default_rng(5)
    hkv, d, tokens = 2, 128, 4
    width = hkv * d
    k_new, v_new = bf16_normal(rng, (tokens, hkv, d)), bf16_normal(rng, (tokens, hkv, d))
    store = backend.tensor("history", B.DTYPE_BF16, (tokens, 2 * width))
    count = (tokens - 1) * 2 * width + width
    kh, vh = store.view(0, B.DTYPE_BF16, (count,)), store.view(2 * width, B.DTYPE_BF16, (count,))
    for which in ("key", "value"):
        bad_k, bad_v = k_new.copy(), v_new.copy()
        (bad_k if which == "key" else bad_v)[2, 1, 77] = 0x7FC0
        tk = backend.tensor("k", B.DTYPE_BF16, bad_k.shape, bad_k)
        tv = backend.tensor("v", B.DTYPE_BF16, bad_v.shape, bad_v)
        with pytest.raises(YvexError) as e:
            backend.history_append_execute(tk, tv, kh, vh, 0, hkv, key_token_stride=2 * width,
                                           value_token_stride=2 * width)
        assert e.value.code == B.YVEX_ERR_FORMAT, which
        tk.release()
        tv.release()
    store.release()


def test_history_grows_in_a_reserved_range_append_then_decode(backend):
    """Prompt, then single tokens: each step commits the rows it adds (usually nothing new:
    a 2 MiB granule holds 512 rows here), appends them with the keys rotated, and decodes
    the step's last token over everything so far.  Every decode must equal the oracle on the
    rows the oracle rotated itself."""
    hq, hkv, d, rotary, capacity = 32, 8, 128, 64, 16384
    width = hkv * d
    row_bytes = 2 * width * 2
    rng = np.random.default_rng(99)
    history = backend.reserve("history", B.DTYPE_BF16, (capacity, 2 * width))
    k_all = np.empty((0, hkv, d), np.uint16)
    v_all = np.empty((0, hkv, d), np.uint16)
    have = 0
    for step_tokens in (700, 1, 1, 330, 1, 2100, 1):
        k_new, v_new = bf16_normal(rng, (step_tokens, hkv, d)), bf16_normal(rng, (step_tokens, hkv, d))
        cosine, sine = tables(rng, step_tokens, rotary)
        used = have + step_tokens
        delta = history.commit(have * row_bytes, step_tokens * row_bytes)
        assert delta % history.granularity == 0
        assert history.resident_bytes == -(-used * row_bytes // history.granularity) * history.granularity
        count = (used - 1) * 2 * width + width
        kh = history.view(0, B.DTYPE_BF16, (count,))
        vh = history.view(2 * width, B.DTYPE_BF16, (count,))
        tk = backend.tensor("k-new", B.DTYPE_BF16, k_new.shape, k_new)
        tv = backend.tensor("v-new", B.DTYPE_BF16, v_new.shape, v_new)
        tc = backend.tensor("cos", B.DTYPE_F32, cosine[:, :rotary].shape, cosine[:, :rotary])
        ts = backend.tensor("sin", B.DTYPE_F32, sine[:, :rotary].shape, sine[:, :rotary])
        backend.history_append_execute(tk, tv, kh, vh, have, hkv, cosine=tc, sine=ts,
                                       rotary_dimension=rotary, key_token_stride=2 * width,
                                       value_token_stride=2 * width)
        assert kh.is_written and vh.is_written                    # the views it wrote are usable as they are
        k_all = np.concatenate([k_all, ORACLE.rotary_half_bf16(k_new, cosine[:, :rotary],
                                                               sine[:, :rotary], rotary)])
        v_all = np.concatenate([v_all, v_new])
        have = used
        q = bf16_normal(rng, (1, hq, d))
        req = backend.attention_requirement(1, have, hq, hkv, d, causal=True, query_start=have - 1,
                                            dtype=B.DTYPE_BF16,
                                            contract=B.NUMERIC_BF16_F32_ACCUMULATE,
                                            k_stride=2 * width, v_stride=2 * width)
        tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
        out = backend.tensor("o", B.DTYPE_BF16, q.shape)
        lse = backend.tensor("lse", B.DTYPE_F32, (1, hq))
        backend.attention_execute(req, tq, kh, vh, out, lse=lse)
        rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k_all, v_all, query_start=have - 1, causal=True)
        assert rc == 0
        assert_close_bf16(out.read(), ref, "history of %d rows" % have)
        assert_lse(lse.read(), ref_lse, "history of %d rows" % have)
        for tensor in (tk, tv, tc, ts, tq, out, lse):
            tensor.release()
    got = history.view(0, B.DTYPE_BF16, (have, 2 * width)).read()
    assert np.array_equal(got[:, :width], k_all.reshape(have, width))
    assert np.array_equal(got[:, width:], v_all.reshape(have, width))
    history.release()


@pytest.mark.parametrize("seed", [21, 22])
def test_history_append_random_sweep(backend, seed):
    """Random geometry: head widths 64 to 256, partial and full rotary, packed, interleaved and
    padded strides, ordinary tensors and reserved ranges committed for exactly the rows in
    use.  Byte-exact, and nothing outside the new rows changes."""
    rng = np.random.default_rng(seed)
    for _ in range(40):
        d = int(rng.choice([64, 128, 256]))
        hkv = int(rng.choice([1, 2, 3, 8]))
        rotary = int(rng.choice([0, 16, 32, d // 2, d]))
        tokens = int(rng.choice([1, 1, rng.integers(2, 50), rng.integers(50, 700)]))
        first = int(rng.choice([0, rng.integers(1, 40), rng.integers(40, 3000)]))
        width = hkv * d
        pad = int(rng.choice([0, 8, 64]))
        interleaved = bool(rng.integers(0, 2))
        stride = (2 * width if interleaved else width) + pad
        used = first + tokens
        rows = used + int(rng.integers(0, 3))
        reserved = bool(rng.integers(0, 2))
        k_new, v_new = bf16_normal(rng, (tokens, hkv, d)), bf16_normal(rng, (tokens, hkv, d))
        cosine, sine = tables(rng, tokens, rotary)
        want_k = ORACLE.rotary_half_bf16(k_new, cosine[:, :rotary], sine[:, :rotary], rotary) \
            if rotary else k_new
        held = []

        def device(*args):
            held.append(backend.tensor(*args))
            return held[-1]

        def history(name, before):
            if not reserved:
                return device(name, B.DTYPE_BF16, before.shape, before)
            t = backend.reserve(name, B.DTYPE_BF16, (rows + 5000, stride))
            held.append(t)
            t.commit(0, before.nbytes)
            t.view(0, B.DTYPE_BF16, before.shape).write(before)
            return t
        count = (used - 1) * stride + width
        if interleaved:
            before = bf16_normal(rng, (rows, stride))
            store = history("history", before)
            kh, vh = store.view(0, B.DTYPE_BF16, (count,)), store.view(2 * width, B.DTYPE_BF16, (count,))
            want = before.copy()
            want[first:used, :width] = want_k.reshape(tokens, width)
            want[first:used, width:2 * width] = v_new.reshape(tokens, width)
            checks = [(store, want)]
        else:
            before_k, before_v = bf16_normal(rng, (rows, stride)), bf16_normal(rng, (rows, stride))
            sk, sv = history("k-history", before_k), history("v-history", before_v)
            kh, vh = sk.view(0, B.DTYPE_BF16, (count,)), sv.view(0, B.DTYPE_BF16, (count,))
            want_kh, want_vh = before_k.copy(), before_v.copy()
            want_kh[first:used, :width] = want_k.reshape(tokens, width)
            want_vh[first:used, :width] = v_new.reshape(tokens, width)
            checks = [(sk, want_kh), (sv, want_vh)]
        label = (seed, d, hkv, rotary, tokens, first, pad, interleaved, reserved)
        backend.history_append_execute(
            device("k-new", B.DTYPE_BF16, k_new.shape, k_new), device("v-new", B.DTYPE_BF16, v_new.shape, v_new),
            kh, vh, first, hkv, head_dimension=d,
            cosine=device("cos", B.DTYPE_F32, (tokens, rotary), cosine[:, :rotary]) if rotary else None,
            sine=device("sin", B.DTYPE_F32, (tokens, rotary), sine[:, :rotary]) if rotary else None,
            rotary_dimension=rotary, key_token_stride=stride, value_token_stride=stride)
        for store, want in checks:
            got = store.view(0, B.DTYPE_BF16, want.shape).read()
            assert np.array_equal(got, want), label
        for t in held:
            t.release()


@pytest.mark.parametrize("tokens,first,hkv,d,rotary,interleaved", [
    (1, 0, 8, 128, 128, True), (1, 1000, 2, 128, 64, True), (45, 3, 4, 64, 32, True),
    (200, 17, 2, 128, 0, True), (9, 2, 1, 256, 8, False), (33, 0, 3, 96, 48, False),
])
def test_history_append_f32_matches_oracle_bit_for_bit(backend, tokens, first, hkv, d, rotary, interleaved):
    """The F32 form (the reference's own history element type).  The inputs are arbitrary
    floats, not bf16-representable ones: they enter the products unrounded."""
    rng = np.random.default_rng(tokens * 77 + first + d)
    width = hkv * d
    rows = first + tokens + 2
    k_new = rng.standard_normal((tokens, hkv, d)).astype(np.float32)
    v_new = rng.standard_normal((tokens, hkv, d)).astype(np.float32)
    cosine, sine = tables(rng, tokens, rotary)
    want_k = ORACLE.rotary_half_f32(k_new, cosine[:, :rotary], sine[:, :rotary], rotary) if rotary else k_new
    held = [backend.tensor("k-new", B.DTYPE_F32, k_new.shape, k_new),
            backend.tensor("v-new", B.DTYPE_F32, v_new.shape, v_new)]
    tc = ts = None
    if rotary:
        tc = backend.tensor("cos", B.DTYPE_F32, (tokens, rotary), cosine[:, :rotary])
        ts = backend.tensor("sin", B.DTYPE_F32, (tokens, rotary), sine[:, :rotary])
        held += [tc, ts]
    used = first + tokens
    if interleaved:
        before = rng.standard_normal((rows, 2 * width)).astype(np.float32)
        store = backend.tensor("history", B.DTYPE_F32, before.shape, before)
        count = (used - 1) * 2 * width + width
        kh, vh = store.view(0, B.DTYPE_F32, (count,)), store.view(4 * width, B.DTYPE_F32, (count,))
        strides = dict(key_token_stride=2 * width, value_token_stride=2 * width)
        want = before.copy()
        want[first:used, :width] = want_k.reshape(tokens, width)
        want[first:used, width:] = v_new.reshape(tokens, width)
        checks = [(store, want)]
    else:
        before_k = rng.standard_normal((rows, width)).astype(np.float32)
        before_v = rng.standard_normal((rows, width)).astype(np.float32)
        sk = backend.tensor("k-history", B.DTYPE_F32, before_k.shape, before_k)
        sv = backend.tensor("v-history", B.DTYPE_F32, before_v.shape, before_v)
        kh, vh = sk.view(0, B.DTYPE_F32, (used * width,)), sv.view(0, B.DTYPE_F32, (used * width,))
        strides = {}
        want_kh, want_vh = before_k.copy(), before_v.copy()
        want_kh[first:used] = want_k.reshape(tokens, width)
        want_vh[first:used] = v_new.reshape(tokens, width)
        checks = [(sk, want_kh), (sv, want_vh)]
    facts = backend.history_append_execute(held[0], held[1], kh, vh, first, hkv, head_dimension=d,
                                           cosine=tc, sine=ts, rotary_dimension=rotary, **strides)
    assert facts.kernel_launches == 1
    for store, want in checks:
        assert np.array_equal(store.read().view(np.uint32), want.view(np.uint32))
        store.release()
    for t in held:
        t.release()
    # a bf16 history does not take F32 rows
    mixed = backend.tensor("bf16-history", B.DTYPE_BF16, (used, width))
    k2 = backend.tensor("k-new", B.DTYPE_F32, k_new.shape, k_new)
    with pytest.raises(YvexError) as e:
        backend.history_append_execute(k2, k2, mixed.view(0, B.DTYPE_BF16, (used * width,)),
                                       mixed.view(0, B.DTYPE_BF16, (used * width,)), first, hkv,
                                       head_dimension=d)
    assert e.value.code == B.YVEX_ERR_FORMAT
    mixed.release()
    k2.release()


def test_f32_history_in_a_reserved_range_append_then_exact_decode(backend):
    """The reference's own chain under its own contract: F32 [K | V] rows, rotary products
    rounded to bf16, EXACT_F32 attention over the strided views."""
    hq, hkv, d, rotary = 8, 2, 128, 128
    width = hkv * d
    row_bytes = 2 * width * 4
    rng = np.random.default_rng(123)
    history = backend.reserve("history", B.DTYPE_F32, (8192, 2 * width))
    k_all = np.empty((0, hkv, d), np.float32)
    v_all = np.empty((0, hkv, d), np.float32)
    have = 0
    for step_tokens in (300, 1, 1500, 1):
        k_new = ORACLE.bf16_decode(bf16_normal(rng, (step_tokens, hkv, d)))
        v_new = ORACLE.bf16_decode(bf16_normal(rng, (step_tokens, hkv, d)))
        cosine, sine = tables(rng, step_tokens, rotary)
        used = have + step_tokens
        history.commit(have * row_bytes, step_tokens * row_bytes)
        count = (used - 1) * 2 * width + width
        kh = history.view(0, B.DTYPE_F32, (count,))
        vh = history.view(4 * width, B.DTYPE_F32, (count,))
        held = [backend.tensor("k-new", B.DTYPE_F32, k_new.shape, k_new),
                backend.tensor("v-new", B.DTYPE_F32, v_new.shape, v_new),
                backend.tensor("cos", B.DTYPE_F32, cosine.shape, cosine),
                backend.tensor("sin", B.DTYPE_F32, sine.shape, sine)]
        backend.history_append_execute(held[0], held[1], kh, vh, have, hkv, cosine=held[2], sine=held[3],
                                       rotary_dimension=rotary, key_token_stride=2 * width,
                                       value_token_stride=2 * width)
        k_all = np.concatenate([k_all, ORACLE.rotary_half_f32(k_new, cosine, sine, rotary)])
        v_all = np.concatenate([v_all, v_new])
        have = used
        q = ORACLE.bf16_decode(bf16_normal(rng, (1, hq, d)))
        req = backend.attention_requirement(1, have, hq, hkv, d, causal=True, query_start=have - 1,
                                            k_stride=2 * width, v_stride=2 * width)
        tq = backend.tensor("q", B.DTYPE_F32, q.shape, q)
        out = backend.tensor("o", B.DTYPE_F32, q.shape)
        backend.attention_execute(req, tq, kh, vh, out)
        rc, ref = ORACLE.gqa(q, k_all, v_all, query_start=have - 1)[:2]
        assert rc == 0
        err = np.abs(out.read() - ref).max()
        assert err < 2e-6, (have, err)
        for t in held + [tq, out]:
            t.release()
    history.release()



@pytest.mark.parametrize("f32", [False, True], ids=["bf16", "f32"])
@pytest.mark.parametrize("d,rotary", [(128, 64), (64, 64), (256, 32)])
def test_history_append_in_the_decoder_order_of_rotary(backend, f32, d, rotary):
    """Mode F32_ROUNDED: plain F32 rotation then one bf16 rounding (the decoder's order,
    src/runtime/decoder.c:1112-1131).  In F32 the key lanes behind the rotary ones are rounded
    too, as decoder_round rounds the whole tensor; values are copied as they are."""
    rng = np.random.default_rng(d + rotary + int(f32))
    tokens, first, hkv = 29, 6, 3
    width = hkv * d
    used = first + tokens
    cosine, sine = tables(rng, tokens, rotary)
    if f32:
        k_new = rng.standard_normal((tokens, hkv, d)).astype(np.float32)
        v_new = rng.standard_normal((tokens, hkv, d)).astype(np.float32)
        want_k = ORACLE.rotary_half_f32_rounded(k_new, cosine[:, :rotary], sine[:, :rotary], rotary)
        dtype, before = B.DTYPE_F32, rng.standard_normal((used, 2 * width)).astype(np.float32)
        offset = 4 * width
    else:
        k_new, v_new = bf16_normal(rng, (tokens, hkv, d)), bf16_normal(rng, (tokens, hkv, d))
        want_k = ORACLE.bf16_encode(ORACLE.rotary_half_f32_rounded(
            ORACLE.bf16_decode(k_new), cosine[:, :rotary], sine[:, :rotary], rotary))
        dtype, before = B.DTYPE_BF16, bf16_normal(rng, (used, 2 * width))
        offset = 2 * width
    held = [backend.tensor("k-new", dtype, k_new.shape, k_new), backend.tensor("v-new", dtype, v_new.shape, v_new),
            backend.tensor("cos", B.DTYPE_F32, (tokens, rotary), cosine[:, :rotary]),
            backend.tensor("sin", B.DTYPE_F32, (tokens, rotary), sine[:, :rotary]),
            backend.tensor("history", dtype, before.shape, before)]
    count = (used - 1) * 2 * width + width
    kh, vh = held[4].view(0, dtype, (count,)), held[4].view(offset, dtype, (count,))
    backend.history_append_execute(held[0], held[1], kh, vh, first, hkv, head_dimension=d, cosine=held[2],
                                   sine=held[3], rotary_dimension=rotary, key_token_stride=2 * width,
                                   value_token_stride=2 * width, rotary_mode=B.ROTARY_F32_ROUNDED)
    want = before.copy()
    want[first:, :width] = want_k.reshape(tokens, width)
    want[first:, width:] = v_new.reshape(tokens, width)
    got = held[4].read()
    assert np.array_equal(got.view(np.uint32 if f32 else np.uint16), want.view(np.uint32 if f32 else np.uint16))
    with pytest.raises(YvexError) as e:
        backend.history_append_execute(held[0], held[1], kh, vh, first, hkv, head_dimension=d,
                                       key_token_stride=2 * width, value_token_stride=2 * width,
                                       rotary_mode=7)
    assert e.value.code == B.YVEX_ERR_UNSUPPORTED
    for t in held:
        t.release()


@pytest.mark.parametrize("tokens", [5, 700])
def test_session_layer_copy_loop_equals_the_history_writer(backend, tokens):
    """The unchanged caller (src/runtime/stateful_attention.c:183-222): per token, one
    asynchronous copy of the key row and one of the value row into the [K | V] history row,
    F32 as the session layer keeps it, nothing waited for; then attention over the views.  The
    history must equal, byte for byte, what the one-launch writer leaves (no rotary: the
    session layer's rows arrive rotated), and the attention enqueued right behind the copies,
    with no synchronisation in between, must equal the attention over the writer's history.
    The copies are small: they wait in the backend's queue and leave in batches, the last of
    them when the attention asks for the stream."""
    rng = np.random.default_rng(314 + tokens)
    hq, hkv, d, have = 8, 2, 64, 37   # 700 tokens: 1400 small copies, eleven launches of the copy queue
    width = hkv * d
    rows = have + tokens
    before = rng.standard_normal((rows, 2 * width)).astype(np.float32)
    k_new = rng.standard_normal((tokens, hkv, d)).astype(np.float32)
    v_new = rng.standard_normal((tokens, hkv, d)).astype(np.float32)
    q = rng.standard_normal((tokens, hq, d)).astype(np.float32)
    tk = backend.tensor("k-new", B.DTYPE_F32, k_new.shape, k_new)
    tv = backend.tensor("v-new", B.DTYPE_F32, v_new.shape, v_new)
    tq = backend.tensor("q", B.DTYPE_F32, q.shape, q)
    looped = backend.tensor("history-loop", B.DTYPE_F32, before.shape, before)
    written = backend.tensor("history-writer", B.DTYPE_F32, before.shape, before)
    out_loop = backend.tensor("out-loop", B.DTYPE_F32, q.shape)
    out_writer = backend.tensor("out-writer", B.DTYPE_F32, q.shape)
    count = (rows - 1) * 2 * width + width
    req = backend.attention_requirement(tokens, rows, hq, hkv, d, causal=True, query_start=have,
                                        k_stride=2 * width, v_stride=2 * width)

    def views(store):
        return (store.view(0, B.DTYPE_F32, (count,)), store.view(width * 4, B.DTYPE_F32, (count,)))

    backend.set_completion_mode(B.COMPLETION_DEFERRED)
    try:
        row_bytes = 2 * width * 4
        for token in range(tokens):
            target = (have + token) * row_bytes
            looped.view(target, B.DTYPE_F32, (width,)).copy_from_async(
                tk.view(token * width * 4, B.DTYPE_F32, (width,)))
            looped.view(target + width * 4, B.DTYPE_F32, (width,)).copy_from_async(
                tv.view(token * width * 4, B.DTYPE_F32, (width,)))
        kh, vh = views(looped)
        backend.attention_execute(req, tq, kh, vh, out_loop)      # no wait since the copies
        backend.sync()
    finally:
        backend.set_completion_mode(B.COMPLETION_IMMEDIATE)
    kh2, vh2 = views(written)
    backend.history_append_execute(tk, tv, kh2, vh2, have, hkv, head_dimension=d,
                                   key_token_stride=2 * width, value_token_stride=2 * width)
    backend.attention_execute(req, tq, kh2, vh2, out_writer)
    want = before.copy()
    want[have:, :width] = k_new.reshape(tokens, width)
    want[have:, width:] = v_new.reshape(tokens, width)
    assert np.array_equal(looped.read(), want)
    assert np.array_equal(written.read(), want)
    assert np.array_equal(out_loop.read(), out_writer.read())
    rc, ref = ORACLE.gqa(q, want[:, :width].reshape(rows, hkv, d).copy(),
                         want[:, width:].reshape(rows, hkv, d).copy(), query_start=have)[:2]
    assert rc == 0
    assert np.allclose(out_loop.read(), ref, rtol=2e-5, atol=2e-6)
    for tensor in (tk, tv, tq, looped, written, out_loop, out_writer):
        tensor.release()


def test_session_backend_on_the_device_copies_between_streams(backend):
    """A session backend opened on the device of the primary one
    (yvex_backend_open_shared_rocm) runs its own kernels on its own stream; a tensor written by
    a kernel of one is copied into the other with yvex_backend_tensor_copy_shared_async, ordered
    by events, with no host wait between the producing kernel and the copy."""
    from clori_amd.backend import Backend
    rng = np.random.default_rng(271)
    hq, hkv, d, ctx = 8, 2, 128, 900
    q = bf16_normal(rng, (1, hq, d))
    k, v = bf16_normal(rng, (ctx, hkv, d)), bf16_normal(rng, (ctx, hkv, d))
    session = Backend(shared_with=backend)
    try:
        assert session.status == B.STATUS_READY
        tq = session.tensor("q", B.DTYPE_BF16, q.shape, q)
        tk = session.tensor("k", B.DTYPE_BF16, k.shape, k)
        tv = session.tensor("v", B.DTYPE_BF16, v.shape, v)
        produced = session.tensor("out", B.DTYPE_BF16, q.shape)
        received = backend.tensor("received", B.DTYPE_BF16, q.shape)
        req = session.attention_requirement(1, ctx, hq, hkv, d, causal=True, query_start=ctx - 1,
                                            dtype=B.DTYPE_BF16, contract=B.NUMERIC_BF16_F32_ACCUMULATE)
        session.set_completion_mode(B.COMPLETION_DEFERRED)
        session.attention_execute(req, tq, tk, tv, produced)       # enqueued on the session's stream
        received.copy_from_shared_async(produced)                  # primary's stream waits for it
        got = received.read()
        session.sync()
        assert np.array_equal(got, produced.read())
        rc, ref = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1)[:2]
        assert rc == 0
        assert_close_bf16(got, ref, "session backend")
        received.release()
    finally:
        session.close()


@pytest.mark.parametrize("f32", [False, True], ids=["bf16", "f32"])
@pytest.mark.parametrize("mode", [B.ROTARY_BF16_STAGED, B.ROTARY_F32_ROUNDED], ids=["staged", "decoder-order"])
@pytest.mark.parametrize("tokens,hq,hkv,d,rotary", [
    (1, 40, 8, 128, 64), (1, 16, 2, 256, 64), (37, 5, 1, 64, 64), (300, 6, 2, 128, 0), (9, 3, 3, 96, 32)])
def test_history_append_rotates_the_queries_in_the_same_launch(backend, f32, mode, tokens, hq, hkv, d, rotary):
    """With a query tensor the launch also does the decoder's rotary pass over the queries
    (src/runtime/decoder.c:1235-1238) where they lie: the queries equal the restatement's
    rotation for the element type and mode, the histories equal those of a call without."""
    rng = np.random.default_rng(tokens * 31 + hq * 7 + d + rotary + int(f32) + 2 * mode)
    if d % (8 if not f32 else 4) or (not f32 and rotary % 16):
        pytest.skip("not a geometry of this element type")
    first, width = 11, hkv * d
    used = first + tokens
    cosine, sine = tables(rng, tokens, rotary)
    cs, sn = cosine[:, :rotary], sine[:, :rotary]
    if f32:
        dtype, elem = B.DTYPE_F32, 4
        q, k_new, v_new = (rng.standard_normal((tokens, h, d)).astype(np.float32) for h in (hq, hkv, hkv))
        before = rng.standard_normal((used, 2 * width)).astype(np.float32)
        rotate = ORACLE.rotary_half_f32 if mode == B.ROTARY_BF16_STAGED else ORACLE.rotary_half_f32_rounded
        if rotary:
            want_q = rotate(q, cs, sn, rotary)
        else:  # the decoder's order still rounds every lane once
            want_q = ORACLE.bf16_decode(ORACLE.bf16_encode(q)) if mode == B.ROTARY_F32_ROUNDED else q
    else:
        dtype, elem = B.DTYPE_BF16, 2
        q, k_new, v_new = (bf16_normal(rng, (tokens, h, d)) for h in (hq, hkv, hkv))
        before = bf16_normal(rng, (used, 2 * width))
        if not rotary:
            want_q = q
        elif mode == B.ROTARY_BF16_STAGED:
            want_q = ORACLE.rotary_half_bf16(q, cs, sn, rotary)
        else:
            want_q = ORACLE.bf16_encode(ORACLE.rotary_half_f32_rounded(ORACLE.bf16_decode(q), cs, sn, rotary))
    bits = np.uint32 if f32 else np.uint16
    held = [backend.tensor("k-new", dtype, k_new.shape, k_new), backend.tensor("v-new", dtype, v_new.shape, v_new),
            backend.tensor("q", dtype, q.shape, q), backend.tensor("with", dtype, before.shape, before),
            backend.tensor("without", dtype, before.shape, before)]
    tc = ts = None
    if rotary:
        tc, ts = backend.tensor("cos", B.DTYPE_F32, cs.shape, cs), backend.tensor("sin", B.DTYPE_F32, sn.shape, sn)
        held += [tc, ts]
    count = (used - 1) * 2 * width + width
    common = dict(head_dimension=d, cosine=tc, sine=ts, rotary_dimension=rotary, key_token_stride=2 * width,
                  value_token_stride=2 * width, rotary_mode=mode)
    views = [(s.view(0, dtype, (count,)), s.view(elem * width, dtype, (count,))) for s in (held[3], held[4])]
    facts = backend.history_append_execute(held[0], held[1], *views[0], first, hkv, query=held[2],
                                           query_heads=hq, **common)
    assert facts.kernel_launches == 1
    backend.history_append_execute(held[0], held[1], *views[1], first, hkv, **common)
    assert np.array_equal(held[2].read().view(bits), np.ascontiguousarray(want_q).view(bits))
    assert np.array_equal(held[3].read().view(bits), held[4].read().view(bits))
    assert not np.array_equal(held[3].read().view(bits), before.view(bits))
    # the new rows are untouched, and a query that overlaps them or comes without a head count is refused
    assert np.array_equal(held[0].read().view(bits), k_new.view(bits))
    for bad in (dict(query=held[2], query_heads=0), dict(query=None, query_heads=hq),
                dict(query=held[0], query_heads=hkv)):
        with pytest.raises(YvexError) as e:
            backend.history_append_execute(held[0], held[1], *views[0], first, hkv, **bad, **common)
        assert e.value.code == B.YVEX_ERR_INVALID_ARG
    for t in held:
        t.release()
