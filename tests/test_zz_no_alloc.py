"""GPU: the paged-decode entry point that allocates nothing
(yvex_backend_rocm_paged_decode_execute_static) against paged_decode_execute, through the
C ABI: same kernels and geometry, so every output bit and every LSE bit must be equal.  Two
calls in a row, the second smaller, so stale partials of the first call in the fixed scratch
would show; then a request too large for the scratch, which must be refused."""
import numpy as np
import pytest

from clori_amd import binding as B
from clori_amd.backend import YvexError, kv_pack_pages
from gpu_common import ORACLE, assert_close_bf16, assert_lse, backend, bf16_normal  # noqa: F401
from test_gpu_decode import make_paged_case

pytestmark = pytest.mark.gpu


def run_both(backend, contexts, hq, hkv, storage, seed, d=128):
    rng = np.random.default_rng(seed)
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, hq, hkv, d=d)
    if storage == B.KV_Q8_0:
        from clori_amd.backend import q8_0_encode_rows
        k_rows = q8_0_encode_rows(ORACLE.bf16_decode(k_rows))
        v_rows = q8_0_encode_rows(ORACLE.bf16_decode(v_rows))
    kp = kv_pack_pages(k_rows, storage, False, hkv, head_dim=d)
    vp = kv_pack_pages(v_rows, storage, True, hkv, head_dim=d)
    pool_dtype = B.DTYPE_BF16 if storage == B.KV_BF16 else B.DTYPE_I8
    elems = kp.size // B.DTYPE_BYTES[pool_dtype]
    sessions = len(contexts)
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tkp = backend.tensor("kpool", pool_dtype, (elems,), kp)
    tvp = backend.tensor("vpool", pool_dtype, (elems,), vp)
    tt = backend.tensor("table", B.DTYPE_I32, table.shape, table)
    tc = backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)
    req = backend.paged_requirement(sessions, hq, hkv, d, 16, pool_pages, table.shape[1],
                                    int(table.shape[1] * 16), storage=storage)
    results = []
    for static in (False, True):
        out = backend.tensor("o", B.DTYPE_BF16, q.shape)
        lse = backend.tensor("lse", B.DTYPE_F32, (sessions, hq))
        before = backend.memory_stats().allocation_events
        if static:
            facts = backend.paged_decode_execute_static(req, tq, tkp, tvp, tt, tc, out, lse)
            assert backend.memory_stats().allocation_events == before   # nothing was acquired
        else:
            facts = backend.paged_decode_execute(req, tq, tkp, tvp, tt, tc, out, lse)
        assert facts.kernel_launches in (1, 2)
        results.append((out.read(), lse.read()))
    (ref_out, ref_lse), (got_out, got_lse) = results
    assert np.array_equal(got_out, ref_out), "output bits differ from paged_decode_execute"
    assert np.array_equal(got_lse.view(np.uint32), ref_lse.view(np.uint32)), "LSE bits differ"
    rc, oracle_out, _, oracle_lse = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, hkv, 16,
                                                        q8=storage == B.KV_Q8_0)
    assert rc == 0
    assert_close_bf16(got_out, oracle_out, "static paged")
    assert_lse(got_lse, oracle_lse, "static paged")


@pytest.mark.parametrize("storage", [B.KV_BF16, B.KV_Q8_0])
def test_static_entry_matches_paged_decode_twice_in_a_row(backend, storage):
    # large first (every wave slot of the scratch is written), then a smaller request
    run_both(backend, [3000, 17, 1024, 2049, 555, 4096, 1, 800], 32, 8, storage, seed=11)
    run_both(backend, [40, 700, 129], 8, 2, storage, seed=12)


@pytest.mark.parametrize("d,hq,hkv", [(64, 16, 4), (256, 24, 4)])
def test_static_entry_at_other_head_dimensions(backend, d, hq, hkv):
    run_both(backend, [3000, 17, 1024, 2049, 555, 4096, 1, 800], hq, hkv, B.KV_BF16, seed=14, d=d)
    run_both(backend, [40, 700, 129], hq, hkv, B.KV_BF16, seed=15, d=d)


def test_static_entry_refuses_what_does_not_fit(backend):
    # a query group of 16 at the full wave count needs 2*2048*16*(128+2)*4 B > 16 MiB
    rng = np.random.default_rng(13)
    contexts = [16384] * 4
    hq, hkv = 32, 2
    q, k_rows, v_rows, table, ctx, pool_pages = make_paged_case(rng, contexts, hq, hkv)
    kp = kv_pack_pages(k_rows, B.KV_BF16, False, hkv)
    vp = kv_pack_pages(v_rows, B.KV_BF16, True, hkv)
    tq = backend.tensor("q", B.DTYPE_BF16, q.shape, q)
    tkp = backend.tensor("kpool", B.DTYPE_BF16, (kp.size // 2,), kp)
    tvp = backend.tensor("vpool", B.DTYPE_BF16, (vp.size // 2,), vp)
    tt = backend.tensor("table", B.DTYPE_I32, table.shape, table)
    tc = backend.tensor("ctx", B.DTYPE_I32, ctx.shape, ctx)
    out = backend.tensor("o", B.DTYPE_BF16, q.shape)
    req = backend.paged_requirement(4, hq, hkv, 128, 16, pool_pages, table.shape[1],
                                    int(table.shape[1] * 16))
    assert backend.paged_decode_workspace_required(req) > (16 << 20)
    with pytest.raises(YvexError) as e:
        backend.paged_decode_execute_static(req, tq, tkp, tvp, tt, tc, out)
    assert e.value.code == B.YVEX_ERR_BOUNDS and "fixed device scratch" in e.value.message
    assert not out.is_written
    backend.paged_decode_execute(req, tq, tkp, tvp, tt, tc, out)   # the allocating entry still serves it
    rc, ref, _, _ = ORACLE.paged_decode(q, k_rows, v_rows, table, ctx, hkv, 16)
    assert_close_bf16(out.read(), ref, "group 16")
