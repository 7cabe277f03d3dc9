"""GPU parity: a seeded random sweep over the kernel families (prefill with and without
the fused gate, paged decode bf16 / Q8_0, MLA decode with sinks, window and compressed rows,
page writer with rotary, single-token decode over token-major rows, EXACT_F32 requests) at shapes the fixed cases do not list: odd head groups, ragged
contexts around tile and page edges, empty sessions, unaligned spans.  Same bar as the fixed
cases; the page writer is byte-exact."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import kv_pack_pages, kv_unpack_pages, q8_0_encode_rows
from gpu_common import ORACLE, MAX_ABS, REL_L2, LSE_ABS, backend  # noqa: F401

pytestmark = pytest.mark.gpu
CONTRACT = B.NUMERIC_BF16_F32_ACCUMULATE


def close(got_bits, ref, label):
    got = ORACLE.bf16_decode(got_bits).astype(np.float64)
    ref = ref.astype(np.float64)
    err = np.abs(got - ref).max()
    rel = np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30)
    assert np.all(np.isfinite(got)) and err <= MAX_ABS and rel <= REL_L2, (label, err, rel)


def gated(ref, gate):
    """The reference order: publish bf16 rows, then bf16(row * sigmoid(gate))."""
    published = ORACLE.bf16_decode(ORACLE.bf16_encode(ref))
    return ORACLE.sigmoid_gate_bf16(published, ORACLE.bf16_decode(gate)).reshape(ref.shape)


class Case:
    """Device tensors of one case, released together."""

    def __init__(self, backend, rng):
        self.backend, self.rng, self.tensors = backend, rng, []

    def tensor(self, *args):
        t = self.backend.tensor(*args)
        self.tensors.append(t)
        return t

    def bf16(self, shape, scale=1.0):
        return ORACLE.bf16_encode((self.rng.standard_normal(shape) * scale).astype(np.float32))

    def release(self):
        for t in self.tensors:
            t.release()


def prefill_case(c):
    b, rng = c.backend, c.rng
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 4, 5, 8]))
    tq = int(rng.integers(2, 400))
    start = int(rng.choice([0, 0, rng.integers(0, 500)]))
    causal = bool(rng.integers(0, 2))
    tk = start + tq if causal else tq + int(rng.integers(0, 400))
    if not causal:
        start = 0
    d = int(rng.choice([128, 128, 64, 256]))
    q, k, v = c.bf16((tq, hq, d)), c.bf16((tk, hkv, d)), c.bf16((tk, hkv, d))
    gate = c.bf16((tq, hq, d), 2.0) if rng.integers(0, 2) else None
    req = b.attention_requirement(tq, tk, hq, hkv, d, causal=causal, query_start=start,
                                  dtype=B.DTYPE_BF16, contract=CONTRACT)
    out, lse = c.tensor("o", B.DTYPE_BF16, q.shape), c.tensor("l", B.DTYPE_F32, (tq, hq))
    b.attention_execute(req, c.tensor("q", B.DTYPE_BF16, q.shape, q),
                        c.tensor("k", B.DTYPE_BF16, k.shape, k),
                        c.tensor("v", B.DTYPE_BF16, v.shape, v), out, lse=lse,
                        gate=c.tensor("g", B.DTYPE_BF16, gate.shape, gate) if gate is not None else None)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    label = ("prefill", tq, tk, start, hq, hkv, d, causal, gate is not None)
    close(out.read(), gated(ref, gate) if gate is not None else ref, label)
    assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label


def paged_case(c):
    b, rng = c.backend, c.rng
    hkv = int(rng.choice([1, 2, 8]))
    hq = hkv * int(rng.choice([1, 2, 4, 8, 16]))
    sessions = int(rng.integers(1, 12))
    q8 = bool(rng.integers(0, 2))
    ctx = rng.integers(1, int(rng.choice([40, 600, 6000])), size=sessions).astype(np.int32)
    need = (ctx + 15) // 16
    pool_pages = int(need.sum()) + 3
    stride = int(need.max()) + int(rng.integers(0, 3))
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((sessions, stride), np.int32)
    at = 0
    for s in range(sessions):
        table[s, :need[s]] = perm[at:at + need[s]]
        at += int(need[s])
    d = 128 if q8 else int(rng.choice([128, 128, 64, 256]))   # Q8_0 pages exist at 128 only
    kr, vr = c.bf16((pool_pages, 16, hkv, d)), c.bf16((pool_pages, 16, hkv, d))
    storage, dtype = (B.KV_Q8_0, B.DTYPE_I8) if q8 else (B.KV_BF16, B.DTYPE_BF16)
    if q8:
        kr = q8_0_encode_rows(ORACLE.bf16_decode(kr))
        vr = q8_0_encode_rows(ORACLE.bf16_decode(vr))
    kp = kv_pack_pages(kr, storage, False, hkv, head_dim=d)
    vp = kv_pack_pages(vr, storage, True, hkv, head_dim=d)
    q = c.bf16((sessions, hq, d))
    gate = c.bf16(q.shape, 2.0) if rng.integers(0, 2) else None
    out, lse = c.tensor("o", B.DTYPE_BF16, q.shape), c.tensor("l", B.DTYPE_F32, (sessions, hq))
    req = b.paged_requirement(sessions, hq, hkv, d, 16, pool_pages, stride, stride * 16,
                              storage=storage)
    elements = kp.size // B.DTYPE_BYTES[dtype]
    b.paged_decode_execute(req, c.tensor("q", B.DTYPE_BF16, q.shape, q),
                           c.tensor("kp", dtype, (elements,), kp), c.tensor("vp", dtype, (elements,), vp),
                           c.tensor("t", B.DTYPE_I32, table.shape, table),
                           c.tensor("c", B.DTYPE_I32, ctx.shape, ctx), out, lse,
                           gate=c.tensor("g", B.DTYPE_BF16, gate.shape, gate) if gate is not None else None)
    rc, ref, _, ref_lse = ORACLE.paged_decode(q, kr, vr, table, ctx, hkv, 16, q8=q8)
    assert rc == 0
    label = ("paged", sessions, hq, hkv, d, q8, ctx.tolist(), gate is not None)
    close(out.read(), gated(ref, gate) if gate is not None else ref, label)
    assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label


def mla_case(c):
    b, rng = c.backend, c.rng
    batch = int(rng.integers(1, 5))
    ctx = rng.integers(1, int(rng.choice([100, 700, 3000])), size=batch).astype(np.int32)
    need = (ctx + 63) // 64
    pool_pages = int(need.sum()) + 2
    stride = int(need.max()) + 1
    perm = rng.permutation(pool_pages).astype(np.int32)
    table = np.zeros((batch, stride), np.int32)
    at = 0
    for s in range(batch):
        table[s, :need[s]] = perm[at:at + need[s]]
        at += int(need[s])
    pool, q = c.bf16((pool_pages, 64, 576)), c.bf16((batch, 128, 576))
    window = int(rng.choice([0, 0, rng.integers(1, 2000)]))
    sinks = (rng.standard_normal(128) * 2).astype(np.float32) if rng.integers(0, 2) else None
    compressed, selected, extra = None, None, {}
    if rng.integers(0, 2):
        stored = rng.integers(1, 300, size=batch)
        cneed = (stored + 63) // 64
        cpages = int(cneed.sum()) + 1
        cstride = int(cneed.max())
        cperm = rng.permutation(cpages).astype(np.int32)
        ctable = np.zeros((batch, cstride), np.int32)
        at = 0
        for s in range(batch):
            ctable[s, :cneed[s]] = cperm[at:at + cneed[s]]
            at += int(cneed[s])
        cpool = c.bf16((cpages, 64, 576))
        if rng.integers(0, 2):
            capacity = int(rng.integers(1, 200))
            selected = np.stack([rng.integers(0, stored[s], capacity)
                                 for s in range(batch)]).astype(np.int32)
            ccount = rng.integers(0, capacity + 1, size=batch).astype(np.int32)
        else:
            ccount = np.array([rng.integers(0, stored[s] + 1) for s in range(batch)], np.int32)
        compressed = (cpool, ctable, ccount)
        extra = dict(compressed_pool_pages=cpages, compressed_table_stride=cstride,
                     max_compressed_tokens=cstride * 64,
                     compressed_selected_stride=selected.shape[1] if selected is not None else 0)
    req = b.mla_requirement(batch, 128, 576, 512, 64, pool_pages, stride, stride * 64,
                            sliding_window=window, **extra)
    out, lse = c.tensor("o", B.DTYPE_BF16, (batch, 128, 512)), c.tensor("l", B.DTYPE_F32, (batch, 128))
    device_compressed = None
    if compressed is not None:
        device_compressed = [c.tensor("cp", B.DTYPE_BF16, compressed[0].shape, compressed[0]),
                             c.tensor("ct", B.DTYPE_I32, compressed[1].shape, compressed[1]),
                             c.tensor("cc", B.DTYPE_I32, compressed[2].shape, compressed[2])]
        if selected is not None:
            device_compressed.append(c.tensor("sel", B.DTYPE_I32, selected.shape, selected))
    b.mla_decode_execute(req, c.tensor("q", B.DTYPE_BF16, q.shape, q),
                         c.tensor("p", B.DTYPE_BF16, pool.shape, pool),
                         c.tensor("t", B.DTYPE_I32, table.shape, table),
                         c.tensor("c", B.DTYPE_I32, ctx.shape, ctx), out, lse,
                         sinks=c.tensor("s", B.DTYPE_F32, (128,), sinks) if sinks is not None else None,
                         compressed=device_compressed)
    rc, ref, _, ref_lse = ORACLE.mla_decode(q, pool, table, ctx, 512, 64, sinks=sinks,
                                            sliding_window=window, compressed=compressed,
                                            selected=selected)
    assert rc == 0
    label = ("mla", batch, ctx.tolist(), window, sinks is not None, compressed is not None,
             selected is not None)
    close(out.read(), ref, label)
    assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label


def append_case(c):
    b, rng = c.backend, c.rng
    hkv = int(rng.choice([1, 3, 4, 8]))
    sessions = int(rng.integers(1, 6))
    q8 = bool(rng.integers(0, 2))
    rotary = int(rng.choice([0, 16, 32, 64, 96, 128]))
    starts = rng.integers(0, 200, size=sessions).astype(np.int32)
    counts = rng.integers(0, int(rng.choice([2, 40, 150])), size=sessions).astype(np.int32)
    if counts.sum() == 0:
        counts[0] = 1
    stride = int(((starts + counts + 15) // 16).max()) + 1
    pool_pages = sessions * stride + 2
    table = rng.permutation(pool_pages)[:sessions * stride].astype(np.int32).reshape(sessions, stride)
    total = int(counts.sum())
    first_rows = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    k_new, v_new = c.bf16((total, hkv, 128)), c.bf16((total, hkv, 128))
    angles = rng.uniform(-3, 3, (total, max(rotary, 16))).astype(np.float32)
    cosine, sine = np.cos(angles), np.sin(angles)
    old_k, old_v = c.bf16((pool_pages, 16, hkv, 128)), c.bf16((pool_pages, 16, hkv, 128))
    storage, dtype = (B.KV_Q8_0, B.DTYPE_I8) if q8 else (B.KV_BF16, B.DTYPE_BF16)

    def stored(rows):
        return q8_0_encode_rows(ORACLE.bf16_decode(rows)) if q8 else rows

    k_rows, v_rows = stored(old_k), stored(old_v)
    kp, vp = kv_pack_pages(k_rows, storage, False, hkv), kv_pack_pages(v_rows, storage, True, hkv)
    elements = kp.size // B.DTYPE_BYTES[dtype]
    k_pool, v_pool = c.tensor("kp", dtype, (elements,), kp), c.tensor("vp", dtype, (elements,), vp)
    b.kv_append_execute(
        c.tensor("k", B.DTYPE_BF16, k_new.shape, k_new), c.tensor("v", B.DTYPE_BF16, v_new.shape, v_new),
        c.tensor("r", B.DTYPE_I32, (sessions,), first_rows), c.tensor("s", B.DTYPE_I32, (sessions,), starts),
        c.tensor("c", B.DTYPE_I32, (sessions,), counts), c.tensor("t", B.DTYPE_I32, table.shape, table),
        k_pool, v_pool, hkv, pool_pages, int(max(counts.max(), 1)), storage=storage,
        cosine=c.tensor("cos", B.DTYPE_F32, cosine.shape, cosine) if rotary else None,
        sine=c.tensor("sin", B.DTYPE_F32, sine.shape, sine) if rotary else None,
        rotary_dimension=rotary)
    k_rotated = ORACLE.rotary_half_bf16(k_new, cosine[:, :rotary], sine[:, :rotary], rotary) \
        if rotary else k_new
    want_k, want_v = k_rows.copy(), v_rows.copy()
    for s in range(sessions):
        for i in range(counts[s]):
            position = starts[s] + i
            page, slot = table[s, position // 16], position % 16
            want_k[page, slot] = stored(k_rotated[first_rows[s] + i][None])[0]
            want_v[page, slot] = stored(v_new[first_rows[s] + i][None])[0]
    got_k = kv_unpack_pages(k_pool.read(np.uint8, (-1,)), storage, False, pool_pages, hkv)
    got_v = kv_unpack_pages(v_pool.read(np.uint8, (-1,)), storage, True, pool_pages, hkv)
    label = ("append", sessions, hkv, q8, rotary, starts.tolist(), counts.tolist())
    assert np.array_equal(got_k.reshape(want_k.shape), want_k), label
    assert np.array_equal(got_v.reshape(want_v.shape), want_v), label


def rows_case(c):
    """One query token over a token-major bf16 history: head dimension 64, 128 or 256, groups of
    1 to 16, packed or interleaved [K | V] rows, with and without the gate."""
    b, rng = c.backend, c.rng
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 3, 4, 8, 16]))
    d = int(rng.choice([128, 64, 256]))
    ctx = int(rng.integers(1, int(rng.choice([40, 700, 9000]))))
    causal = bool(rng.integers(0, 2))
    tk = ctx if causal else ctx + int(rng.integers(0, 50))
    width = hkv * d
    q, k, v = c.bf16((1, hq, d)), c.bf16((tk, hkv, d)), c.bf16((tk, hkv, d))
    gate = c.bf16(q.shape, 2.0) if rng.integers(0, 2) else None
    interleaved = bool(rng.integers(0, 2))
    req = b.attention_requirement(1, tk, hq, hkv, d, causal=causal, query_start=ctx - 1, dtype=B.DTYPE_BF16,
                                  contract=CONTRACT, k_stride=2 * width if interleaved else 0,
                                  v_stride=2 * width if interleaved else 0)
    if interleaved:
        rows = np.zeros((tk, 2 * width), np.uint16)
        rows[:, :width], rows[:, width:] = k.reshape(tk, width), v.reshape(tk, width)
        store = c.tensor("kv", B.DTYPE_BF16, rows.shape, rows)
        count = (tk - 1) * 2 * width + width
        tk_, tv_ = store.view(0, B.DTYPE_BF16, (count,)), store.view(2 * width, B.DTYPE_BF16, (count,))
    else:
        tk_, tv_ = c.tensor("k", B.DTYPE_BF16, k.shape, k), c.tensor("v", B.DTYPE_BF16, v.shape, v)
    out, lse = c.tensor("o", B.DTYPE_BF16, q.shape), c.tensor("l", B.DTYPE_F32, (1, hq))
    b.attention_execute(req, c.tensor("q", B.DTYPE_BF16, q.shape, q), tk_, tv_, out, lse=lse,
                        gate=c.tensor("g", B.DTYPE_BF16, gate.shape, gate) if gate is not None else None)
    rc, ref, _, ref_lse = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=causal)
    assert rc == 0
    label = ("rows", ctx, tk, hq, hkv, d, causal, interleaved, gate is not None)
    close(out.read(), gated(ref, gate) if gate is not None else ref, label)
    assert np.abs(lse.read() - ref_lse).max() <= LSE_ABS, label


def exact_case(c):
    """EXACT_F32 requests of every shape: the matrix-core tiles (head dimension 64, 128, 256 with
    at least 32 query tokens), the runs of keys (long histories) and the row kernel (the rest),
    at the reference's tolerance for its float device kernel against the CPU operator
    (tests/unit/cuda/quant_qtype.c:2293-2333: 2e-5 on N(0,1)-scale rows)."""
    b, rng = c.backend, c.rng
    hkv = int(rng.choice([1, 2, 4]))
    hq = hkv * int(rng.choice([1, 2, 5, 6]))
    d = int(rng.choice([128, 64, 256, 256, 96, 8]))
    tq = int(rng.choice([1, 1, rng.integers(2, 32), rng.integers(32, 300)]))
    start = int(rng.choice([0, rng.integers(0, 40), rng.integers(500, 3000)])) if tq < 32 else int(rng.integers(0, 300))
    causal = bool(rng.integers(0, 4))
    tk = start + tq if causal else start + tq + int(rng.integers(0, 100))
    q = rng.standard_normal((tq, hq, d)).astype(np.float32)
    k = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    v = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    req = b.attention_requirement(tq, tk, hq, hkv, d, causal=causal, query_start=start)
    work = c.tensor("w", B.DTYPE_I8, (max(b.attention_workspace_required(req), 16),))
    b.workspace_attach(work)
    try:
        out, lse = c.tensor("o", B.DTYPE_F32, q.shape), c.tensor("l", B.DTYPE_F32, (tq, hq))
        b.attention_execute(req, c.tensor("q", B.DTYPE_F32, q.shape, q), c.tensor("k", B.DTYPE_F32, k.shape, k),
                            c.tensor("v", B.DTYPE_F32, v.shape, v), out, lse=lse)
        got, got_lse = out.read(), lse.read()
    finally:
        b.workspace_detach()
    rc, ref, ref_lse = ORACLE.gqa(q, k, v, query_start=start, causal=causal)
    assert rc == 0
    label = ("exact", tq, tk, start, hq, hkv, d, causal)
    assert np.abs(got - ref).max() < 2e-5 and np.abs(got_lse - ref_lse).max() < 2e-5, label


FAMILIES = {"prefill": prefill_case, "paged": paged_case, "mla": mla_case, "append": append_case,
            "rows": rows_case, "exact": exact_case}


@pytest.mark.parametrize("seed", [11, 12])
def test_random_sweep(backend, seed):
    rng = np.random.default_rng(seed)
    counts = dict.fromkeys(FAMILIES, 0)
    for _ in range(120):
        kind = str(rng.choice(sorted(FAMILIES)))
        case = Case(backend, rng)
        FAMILIES[kind](case)
        case.release()
        counts[kind] += 1
    assert min(counts.values()) > 5, counts
