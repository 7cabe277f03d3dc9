"""GPU: recorded launch sequences.  Every replay is checked against the same operations run
eagerly on the same inputs (bit for bit: the kernels are deterministic), with unrelated eager
work and synchronisations between the replays."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import kv_pack_pages
from gpu_common import ORACLE, assert_close_bf16, backend, bf16_normal  # noqa: F401

pytestmark = pytest.mark.gpu


def unrelated_eager_work(backend, rng):
    """A prefill of another shape through the same backend, stream and workspace."""
    q, k = bf16_normal(rng, (70, 4, 128)), bf16_normal(rng, (70, 2, 128))
    req = backend.attention_requirement(70, 70, 4, 2, 128, dtype=B.DTYPE_BF16,
                                        contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    t = [backend.tensor("q", B.DTYPE_BF16, q.shape, q), backend.tensor("k", B.DTYPE_BF16, k.shape, k),
         backend.tensor("v", B.DTYPE_BF16, k.shape, k), backend.tensor("o", B.DTYPE_BF16, q.shape)]
    backend.attention_execute(req, *t)
    backend.sync()
    for x in t:
        x.release()


def test_recorded_row_decode_replays_equal_eager(backend):
    """Benchmark configuration 1 (B=1, 32/8 heads, ctx 4096) as a recorded two-launch sequence."""
    rng = np.random.default_rng(801)
    ctx = 4096
    k, v = bf16_normal(rng, (ctx, 8, 128)), bf16_normal(rng, (ctx, 8, 128))
    req = backend.attention_requirement(1, ctx, 32, 8, 128, causal=True, query_start=ctx - 1,
                                        dtype=B.DTYPE_BF16, contract=B.NUMERIC_BF16_F32_ACCUMULATE)
    tq = backend.tensor("q", B.DTYPE_BF16, (1, 32, 128), bf16_normal(rng, (1, 32, 128)))
    tk, tv = backend.tensor("k", B.DTYPE_BF16, k.shape, k), backend.tensor("v", B.DTYPE_BF16, v.shape, v)
    out, eager = backend.tensor("o", B.DTYPE_BF16, (1, 32, 128)), backend.tensor("e", B.DTYPE_BF16, (1, 32, 128))
    work = backend.tensor("work", B.DTYPE_I8, (backend.attention_workspace_required(req),))
    backend.workspace_attach(work)
    backend.graph_begin()
    backend.attention_execute(req, tq, tk, tv, out)
    graph = backend.graph_end()
    for replay in range(4):
        q = bf16_normal(rng, (1, 32, 128))
        tq.write(q)
        out.zero()
        facts = backend.graph_launch(graph)
        assert facts.kernel_launches == 1
        got = out.read()
        unrelated_eager_work(backend, rng)
        backend.attention_execute(req, tq, tk, tv, eager)
        assert np.array_equal(got, eager.read()), "replay %d" % replay
        rc, ref, _, _ = ORACLE.gqa_bf16(q, k, v, query_start=ctx - 1, causal=True)
        assert rc == 0
        assert_close_bf16(got, ref, "recorded decode replay %d" % replay)
    backend.graph_release(graph)
    backend.workspace_detach()
    for x in (tq, tk, tv, out, eager, work):
        x.release()


def test_recorded_decode_step_appends_then_attends(backend):
    """One serving step as one sequence: write the new token of every session into its pages
    (rotary on the key), then paged decode with the fused gate.  Positions, page tables and
    contexts are device tensors, so the same sequence serves step after step."""
    rng = np.random.default_rng(802)
    sessions, hq, hkv, d, page = 4, 32, 8, 128, 16
    start = np.array([0, 15, 100, 2047], np.int32)
    steps = 5
    stride = int((start.max() + steps + page - 1) // page) + 1
    pool_pages = sessions * stride
    table = rng.permutation(pool_pages).astype(np.int32).reshape(sessions, stride)
    history_k = bf16_normal(rng, (pool_pages, page, hkv, d))
    history_v = bf16_normal(rng, (pool_pages, page, hkv, d))
    kp, vp = (kv_pack_pages(x, B.KV_BF16, is_v, hkv) for x, is_v in ((history_k, False), (history_v, True)))

    def pools():
        return (backend.tensor("kp", B.DTYPE_BF16, (kp.size // 2,), kp),
                backend.tensor("vp", B.DTYPE_BF16, (vp.size // 2,), vp))

    tensors = dict(
        k_new=backend.tensor("kn", B.DTYPE_BF16, (sessions, hkv, d)),
        v_new=backend.tensor("vn", B.DTYPE_BF16, (sessions, hkv, d)),
        cos=backend.tensor("cos", B.DTYPE_F32, (sessions, d)), sin=backend.tensor("sin", B.DTYPE_F32, (sessions, d)),
        rows=backend.tensor("rows", B.DTYPE_I32, (sessions,), np.arange(sessions, dtype=np.int32)),
        pos=backend.tensor("pos", B.DTYPE_I32, (sessions,)),
        one=backend.tensor("one", B.DTYPE_I32, (sessions,), np.ones(sessions, np.int32)),
        table=backend.tensor("table", B.DTYPE_I32, table.shape, table),
        ctx=backend.tensor("ctx", B.DTYPE_I32, (sessions,)),
        q=backend.tensor("q", B.DTYPE_BF16, (sessions, hq, d)),
        gate=backend.tensor("gate", B.DTYPE_BF16, (sessions, hq, d)))
    req = backend.paged_requirement(sessions, hq, hkv, d, page, pool_pages, stride, stride * page)
    work = backend.tensor("work", B.DTYPE_I8, (backend.paged_decode_workspace_required(req),))

    def step_operations(k_pool, v_pool, out):
        t = tensors
        backend.kv_append_execute(t["k_new"], t["v_new"], t["rows"], t["pos"], t["one"], t["table"],
                                  k_pool, v_pool, hkv, pool_pages, 1, cosine=t["cos"], sine=t["sin"],
                                  rotary_dimension=d)
        backend.paged_decode_execute(req, t["q"], k_pool, v_pool, t["table"], t["ctx"], out, gate=t["gate"])

    rec_k, rec_v = pools()
    eag_k, eag_v = pools()
    rec_out = backend.tensor("ro", B.DTYPE_BF16, (sessions, hq, d))
    eag_out = backend.tensor("eo", B.DTYPE_BF16, (sessions, hq, d))
    for name in ("k_new", "v_new", "cos", "sin", "pos", "ctx", "q", "gate"):
        tensors[name].zero()
    backend.workspace_attach(work)
    backend.graph_begin()
    step_operations(rec_k, rec_v, rec_out)
    graph = backend.graph_end()
    for step in range(steps):
        angles = rng.uniform(-3, 3, (sessions, d)).astype(np.float32)
        tensors["k_new"].write(bf16_normal(rng, (sessions, hkv, d)))
        tensors["v_new"].write(bf16_normal(rng, (sessions, hkv, d)))
        tensors["cos"].write(np.cos(angles))
        tensors["sin"].write(np.sin(angles))
        tensors["pos"].write(start + step)
        tensors["ctx"].write(start + step + 1)
        tensors["q"].write(bf16_normal(rng, (sessions, hq, d)))
        tensors["gate"].write(bf16_normal(rng, (sessions, hq, d)))
        facts = backend.graph_launch(graph)
        assert facts.kernel_launches == 2
        got = rec_out.read()
        unrelated_eager_work(backend, rng)
        step_operations(eag_k, eag_v, eag_out)
        assert np.array_equal(got, eag_out.read()), "step %d" % step
        assert np.array_equal(rec_k.read(np.uint8, (-1,)), eag_k.read(np.uint8, (-1,))), "step %d" % step
        assert np.array_equal(rec_v.read(np.uint8, (-1,)), eag_v.read(np.uint8, (-1,))), "step %d" % step
    backend.graph_release(graph)
    backend.workspace_detach()


def test_bandwidth_probe_on_the_device(backend):
    """The probe's record on a real part: a streaming read of 1 GiB sustains terabytes per
    second, below the published peak; the copy moves read plus write."""
    e = backend.bandwidth_probe()
    assert e.working_set_bytes == 1 << 30 and e.sample_count == 5
    assert 1.0e12 < e.sustainable_read_bytes_per_second < 8.5e12
    assert 1.0e12 < e.sustainable_copy_bytes_per_second < 8.5e12
    assert max(e.stream_elapsed_ns) < 2 * min(e.stream_elapsed_ns)
