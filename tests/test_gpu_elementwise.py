"""GPU parity: the element-wise operator slots the reference's decoder calls around attention
(rotary_half_f32, bf16_round, split_interleaved_two_f32, sigmoid_product_bf16) through the
transformer operations table, against the oracle; then the decoder's attention block call
for call (src/runtime/decoder.c:1225-1270, src/runtime/stateful_attention.c:183-222,326-352)
on F32 activations under the reference's EXACT_F32 contract."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError
from gpu_common import ORACLE, backend  # noqa: F401

pytestmark = pytest.mark.gpu


def f32(backend, name, array):
    array = np.ascontiguousarray(array, np.float32)
    return backend.tensor(name, B.DTYPE_F32, array.shape, array)


def bf16_grid(x):
    return ORACLE.bf16_decode(ORACLE.bf16_encode(np.asarray(x, np.float32)))


def test_rotary_slot_matches_the_reference_case_and_the_oracle(backend):
    # tests/unit/cuda/quant_qtype.c:3050-3105
    values = f32(backend, "v", [[[1.0, 2.0], [7.0, 8.0]]])
    cos, sin = f32(backend, "c", [[0.75, 0.75]]), f32(backend, "s", [[0.5, 0.5]])
    facts = backend.rotary_half_f32(values, cos, sin, 1, 2, 2, 2)
    assert facts.kernel_launches == 1
    assert values.read(np.float32, (4,)).tolist() == [-0.25, 2.0, 1.25, 9.5]
    rng = np.random.default_rng(61)
    for tokens, heads, d, rotary in ((37, 5, 128, 64), (3, 24, 256, 256), (129, 2, 64, 16), (1, 1, 8, 2)):
        x = rng.standard_normal((tokens, heads, d)).astype(np.float32)
        angles = rng.uniform(-3.0, 3.0, (tokens, rotary))
        cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)
        t = f32(backend, "x", x)
        backend.rotary_half_f32(t, f32(backend, "c", cosines), f32(backend, "s", sines), tokens, heads, d,
                                rotary)
        got = t.read(np.float32, x.shape)
        want = ORACLE.rotary_half_plain_f32(x, cosines, sines, rotary)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (tokens, heads, d, rotary)


def test_round_slot_rounds_in_place_and_reports_what_is_not_finite(backend):
    rng = np.random.default_rng(62)
    x = (rng.standard_normal(100003) * np.exp(rng.uniform(-20, 20, 100003))).astype(np.float32)
    x[:7] = [0.0, -0.0, 1.0, 3.3895314e38, -3.3895314e38, 1.0000001, 1.00390625]   # overflow to inf, ties
    t = f32(backend, "x", x)
    facts = backend.bf16_round(t, x.size)
    assert facts.kernel_launches == 1
    got = t.read(np.float32, x.shape)
    assert np.array_equal(got.view(np.uint32), bf16_grid(x).view(np.uint32))
    for bad in (np.nan, np.inf, -np.inf):
        y = x.copy()
        y[50000] = bad
        t = f32(backend, "y", y)
        with pytest.raises(YvexError) as e:
            backend.bf16_round(t, y.size)
        assert e.value.code == B.YVEX_ERR_FORMAT


def test_split_slot_separates_the_two_halves_of_every_head(backend):
    # tests/unit/cuda/quant_qtype.c:2977-3008
    source = f32(backend, "in", np.arange(1, 9))
    first, second = backend.tensor("a", B.DTYPE_F32, (4,)), backend.tensor("b", B.DTYPE_F32, (4,))
    facts = backend.split_interleaved_two_f32(source, first, second, 1, 2, 2)
    assert facts.kernel_launches == 1
    assert first.read(np.float32, (4,)).tolist() == [1.0, 2.0, 5.0, 6.0]
    assert second.read(np.float32, (4,)).tolist() == [3.0, 4.0, 7.0, 8.0]
    rng = np.random.default_rng(63)
    rows, heads, d = 77, 24, 256
    x = rng.standard_normal((rows, heads, 2, d)).astype(np.float32)
    first = backend.tensor("a", B.DTYPE_F32, (rows, heads * d))
    second = backend.tensor("b", B.DTYPE_F32, (rows, heads * d))
    backend.split_interleaved_two_f32(f32(backend, "in", x), first, second, rows, heads, d)
    assert np.array_equal(first.read(np.float32, (rows, heads, d)), x[:, :, 0])
    assert np.array_equal(second.read(np.float32, (rows, heads, d)), x[:, :, 1])
    with pytest.raises(YvexError) as e:   # the outputs may not alias
        backend.split_interleaved_two_f32(f32(backend, "in", x), first, first, rows, heads, d)
    assert e.value.code == B.YVEX_ERR_FORMAT


def test_sigmoid_product_slot(backend):
    # tests/unit/cuda/quant_qtype.c:2979-2981,3019-3033: exact on the reference's four values
    values = np.array([1.0, -2.0, 0.5, 4.0], np.float32)
    gates = np.array([0.0, 1.0986122886681098, -1.0986122886681098, 1.0], np.float32)
    out = backend.tensor("o", B.DTYPE_F32, (4,))
    facts = backend.sigmoid_product_bf16(f32(backend, "v", values), f32(backend, "g", gates), out, 4)
    assert facts.kernel_launches == 1
    want = bf16_grid(values / (1.0 + np.exp(-gates.astype(np.float64))))
    assert np.array_equal(out.read(np.float32, (4,)), want)
    # the device's exponential and reciprocal are not libm's: equal but for the rare value next
    # to a bf16 tie, and then one bf16 step apart (the same bar as the fused gate)
    rng = np.random.default_rng(64)
    n = 200000
    values = bf16_grid(rng.standard_normal(n) * 2)
    gates = bf16_grid(rng.standard_normal(n) * 3)
    out = backend.tensor("o", B.DTYPE_F32, (n,))
    backend.sigmoid_product_bf16(f32(backend, "v", values), f32(backend, "g", gates), out, n)
    got = ORACLE.bf16_encode(out.read(np.float32, (n,))).astype(np.int32)
    assert np.array_equal(bf16_grid(out.read(np.float32, (n,))), out.read(np.float32, (n,)))
    want = ORACLE.bf16_encode(ORACLE.sigmoid_gate_bf16(values, gates)).astype(np.int32)
    step = np.abs(got - want)
    assert step.max() <= 1 and np.count_nonzero(step) <= n // 200


def test_refusals_are_the_reference_s(backend):
    x = f32(backend, "x", np.zeros(64))
    half = backend.tensor("h", B.DTYPE_BF16, (64,), np.zeros(64, np.uint16))
    fresh = backend.tensor("n", B.DTYPE_F32, (64,))       # never written
    table = f32(backend, "t", np.zeros(16))
    for call in (lambda: backend.rotary_half_f32(x, table, table, 1, 4, 16, 15),    # odd rotary width
                 lambda: backend.rotary_half_f32(x, table, table, 1, 4, 16, 32),    # wider than the head
                 lambda: backend.rotary_half_f32(x, table, table, 2, 4, 16, 16),    # counts do not match
                 lambda: backend.rotary_half_f32(half, table, table, 1, 4, 16, 16),
                 lambda: backend.rotary_half_f32(fresh, table, table, 1, 4, 16, 16),
                 lambda: backend.bf16_round(x, 63),
                 lambda: backend.bf16_round(x, 0),
                 lambda: backend.bf16_round(half, 64),
                 lambda: backend.sigmoid_product_bf16(x, fresh, fresh, 64),
                 lambda: backend.sigmoid_product_bf16(x, x, half, 64),
                 lambda: backend.split_interleaved_two_f32(x, table, table, 1, 2, 16)):
        with pytest.raises(YvexError) as e:
            call()
        assert e.value.code == B.YVEX_ERR_FORMAT


def test_the_decoder_s_attention_block_call_for_call(backend):
    """What src/runtime/decoder.c:1225-1270 does between the projections and the output
    projection, with the reference's own calls: split the query/gate projection, rotate and
    round Q and K, append K and V to the [K | V] history with two asynchronous copies per token
    (src/runtime/stateful_attention.c:183-222), attention under EXACT_F32 over the strided
    views, round, gate.  Against the same composition of the oracle's functions."""
    rng = np.random.default_rng(65)
    tokens, past, hq, hkv, d, rotary = 9, 70, 8, 2, 128, 64
    kv_width, total = hkv * d, past + tokens
    qg = bf16_grid(rng.standard_normal((tokens, hq, 2, d)))
    k_new, v_new = bf16_grid(rng.standard_normal((tokens, hkv, d))), bf16_grid(rng.standard_normal((tokens, hkv, d)))
    history = np.zeros((total, 2 * kv_width), np.float32)
    history[:past] = bf16_grid(rng.standard_normal((past, 2 * kv_width)))
    angles = rng.uniform(-3.0, 3.0, (tokens, rotary))
    cosines, sines = np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)

    # ---- device, call for call ----
    t_q, t_gate = backend.tensor("q", B.DTYPE_F32, (tokens, hq * d)), backend.tensor("g", B.DTYPE_F32, (tokens, hq * d))
    backend.split_interleaved_two_f32(f32(backend, "qg", qg), t_q, t_gate, tokens, hq, d)
    t_cos, t_sin = f32(backend, "c", cosines), f32(backend, "s", sines)
    t_k, t_v = f32(backend, "k", k_new), f32(backend, "v", v_new)
    backend.rotary_half_f32(t_q, t_cos, t_sin, tokens, hq, d, rotary)
    backend.bf16_round(t_q, tokens * hq * d)
    backend.rotary_half_f32(t_k, t_cos, t_sin, tokens, hkv, d, rotary)
    backend.bf16_round(t_k, tokens * hkv * d)
    t_hist = f32(backend, "history", history)
    for i in range(tokens):
        row = (past + i) * 2 * kv_width * 4
        t_hist.view(row, B.DTYPE_F32, (kv_width,)).copy_from_async(
            t_k.view(i * kv_width * 4, B.DTYPE_F32, (kv_width,)))
        t_hist.view(row + kv_width * 4, B.DTYPE_F32, (kv_width,)).copy_from_async(
            t_v.view(i * kv_width * 4, B.DTYPE_F32, (kv_width,)))
    span = (total - 1) * 2 * kv_width + kv_width
    k_view = t_hist.view(0, B.DTYPE_F32, (span,))
    v_view = t_hist.view(kv_width * 4, B.DTYPE_F32, (span,))
    mixer = backend.tensor("mixer", B.DTYPE_F32, (tokens, hq * d))
    req = backend.attention_requirement(tokens, total, hq, hkv, d, causal=True, query_start=past,
                                        k_stride=2 * kv_width, v_stride=2 * kv_width)
    backend.attention_execute(req, t_q, k_view, v_view, mixer)
    backend.bf16_round(mixer, tokens * hq * d)
    gated = backend.tensor("gated", B.DTYPE_F32, (tokens, hq * d))
    backend.sigmoid_product_bf16(mixer, t_gate, gated, tokens * hq * d)
    got = gated.read(np.float32, (tokens, hq, d))

    # ---- the oracle's composition ----
    q_ref = ORACLE.rotary_half_f32_rounded(qg[:, :, 0], cosines, sines, rotary)
    k_ref = ORACLE.rotary_half_f32_rounded(k_new, cosines, sines, rotary)
    hist_ref = history.copy().reshape(total, 2, hkv, d)
    hist_ref[past:, 0], hist_ref[past:, 1] = k_ref, v_new
    assert np.array_equal(t_hist.read(np.float32, history.shape).reshape(hist_ref.shape), hist_ref)
    rc, attention, _ = ORACLE.gqa(q_ref, np.ascontiguousarray(hist_ref[:, 0]), np.ascontiguousarray(hist_ref[:, 1]),
                                  query_start=past)
    assert rc == 0
    want = ORACLE.sigmoid_gate_bf16(bf16_grid(attention), qg[:, :, 1]).reshape(tokens, hq, d)
    step = np.abs(ORACLE.bf16_encode(got).astype(np.int32) - ORACLE.bf16_encode(want).astype(np.int32))
    # the attention rows agree to F32 tolerance before the rounding, so a rounded row may sit one
    # bf16 step off where the unrounded value lies next to a tie; the gate adds the same
    assert step.max() <= 1 and np.count_nonzero(step) <= got.size // 50, (step.max(), np.count_nonzero(step))


@pytest.mark.parametrize("offset", [0, 1, 2, 3, 16])
def test_small_tensor_transfers_by_kernel_equal_the_runtime_copies(backend, offset):
    """Writes of up to 2048 bytes travel in a kernel's arguments and reads of up to 16384 bytes
    come back through host memory the device writes (the session layer's three small transfers
    per layer and step, src/runtime/stateful_attention.c:222-272); longer ones take the runtime's
    copies.  Every size either side of the limits, at every byte alignment, reads back what was
    written, and a write that is not waited for is seen by the copy and the read behind it."""
    rng = np.random.default_rng(900 + offset)
    store = backend.tensor("bytes", B.DTYPE_I8, (1 << 17,))
    store.zero()
    for size in (1, 3, 4, 8, 15, 16, 17, 255, 2047, 2048, 2049, 4096, 16383, 16384, 16385, 65536):
        data = rng.integers(-128, 128, size, dtype=np.int8)
        view = store.view(offset, B.DTYPE_I8, (size,))
        view.write(data)
        assert np.array_equal(view.read(), data), size
        guard = store.view(offset + size, B.DTYPE_I8, (16,)).read()
        assert not guard.any(), size                                   # nothing behind the view was touched
        view.write(np.zeros(size, np.int8))
    # a small write, an asynchronous copy of it, a small read of the copy: stream order, no wait
    a, b2 = backend.tensor("a", B.DTYPE_F32, (64,)), backend.tensor("b", B.DTYPE_F32, (64,))
    for turn in range(20):
        values = rng.standard_normal(64).astype(np.float32)
        a.write(values)
        b2.copy_from_async(a)
        assert np.array_equal(b2.read(), values), turn
    for t in (store, a, b2):
        t.release()
